// Attention of a few query rows against a long key/value cache (the decode step of
// run_flash_attn_kvcache, reference: flash_api.cu:434-567 -> compute_attn_1rowblock_splitkv,
// flash_fwd_kernel.h:480-970).  HBM-bound: the job is to read K and V once, at full rate.
//
// All query heads that share a key/value head (h / h_k of them) times all query rows are the
// up to 32 columns of one S^T tile, so a cache row is fetched once for the whole group.  The
// key axis is cut three ways: into `n_splits` chunks over workgroups (so that a small batch
// still fills the chip), inside a workgroup round-robin over its four waves in units of 32
// keys, and a wave walks its units with the next one in flight.  There is no barrier in the
// loop: a wave streams its K and V rows with coalesced non-temporal 16-byte loads (16 lanes per
// 256-byte row) into registers and from there into private LDS tiles, from which the MFMA
// operands are read (K plainly, V through the transposing read); the tiles are single-buffered,
// the stores of unit u+1 follow the reads of unit u in the wave's in-order LDS queue.  (Loading
// the K fragments directly in operand layout, 32 bytes per row and instruction, measured 10 %
// slower with the math removed, and 30 % slower with non-temporal loads: every cache line is
// then touched by four consecutive instructions.)  The waves'
// partial (max, sum, O) are merged through LDS at the end; with more than one chunk the
// workgroups write unnormalised fp32 partials and a second kernel merges them
// (the reference's flash_fwd_splitkv_combine_kernel plays that role; its entry point fixes
// num_splits = 1 for want of a workspace, flash_api.cu:548-563 -- here the workspace is a
// stream-ordered allocation).
// Arithmetic as in the forward kernel: fp32 scores, exp2 with scale*log2(e) folded in, P rounded
// to the storage type before P V, O divided by the row sum at the very end, LSE = max*scale +
// ln(sum), a row without keys gives O = 0 and LSE = +inf.
#include "flash_common.h"

namespace fa {
namespace {

constexpr int kDecWaves = 4;
constexpr int kUnit = 32;  // keys per unit

struct DecodeArgs {
  float *o_part;   // [n_splits][b][h][sq][D] unnormalised O relative to the partial max; null: one chunk
  float *ml_part;  // [n_splits][b][h][sq][2] partial max (score units) and row sum
  int n_splits;
  int chunk;       // keys per chunk, a multiple of kUnit
};

template <typename T, int D>
__global__ void __launch_bounds__(kDecWaves * 64, D <= 128 ? 2 : 1) decode_kernel(const Params p, const DecodeArgs a) {
  using vec8 = typename Traits<T>::vec8;
  constexpr int KS = Pad<D>::kPlain, VS = Pad<D>::kTr;
  constexpr int CPR = D / 8;         // 16-byte chunks per row
  constexpr int RPP = 64 / CPR;      // rows per pass of a wave
  constexpr int NPV = kUnit / RPP;   // passes per unit
  constexpr int kWaveLds = kUnit * (KS + VS) * (int)sizeof(T);  // a wave's K and V tile, reused for the merge
  static_assert(kWaveLds >= (D * 32 + 64) * 4, "merge buffers must fit the tiles");
  __shared__ __attribute__((aligned(16))) unsigned char lds[kDecWaves][kWaveLds];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, g = lane >> 5;
  const int split = blockIdx.x % a.n_splits;
  const int bhk = blockIdx.x / a.n_splits;
  const int bi = bhk / p.h_k, hk = bhk % p.h_k;
  const int group = p.h / p.h_k;
  int sk = p.sk;
  if (p.seqlens_k) sk = min(p.sk, p.seqlens_k[bi] + p.seqlen_knew);

  // column n of the S^T tile: query head hk*group + n / sq, query row n % sq
  const bool col_ok = r32 < group * p.sq;
  const int qi = col_ok ? r32 % p.sq : 0, hq = hk * group + (col_ok ? r32 / p.sq : 0);
  int lo_lim = 0, hi_lim = 0;
  if (col_ok) row_limits_sk(p, sk, qi, lo_lim, hi_lim);
  // keys of this chunk that some row can see
  int lo_all, hi_all, t0, t1;
  row_limits_sk(p, sk, 0, lo_all, t0);
  row_limits_sk(p, sk, p.sq - 1, t1, hi_all);
  const int c0 = max(split * a.chunk, lo_all / kUnit * kUnit);
  const int c1 = min((split + 1) * a.chunk, hi_all);
  const int n_units = c1 > c0 ? (c1 - c0 + kUnit - 1) / kUnit : 0;

  const T *kg = static_cast<const T *>(p.k) + bi * p.k_bs + hk * p.k_hs;
  const T *vg = static_cast<const T *>(p.v) + bi * p.v_bs + hk * p.v_hs;
  vec8 qf[D / 16];
  {
    const T *qg = static_cast<const T *>(p.q) + bi * p.q_bs + (int64_t)qi * p.q_rs + hq * p.q_hs;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks)
      qf[ks] = (col_ok && ks * 16 + g * 8 < p.d) ? *reinterpret_cast<const vec8 *>(qg + ks * 16 + g * 8) : vec8{0};
  }

  T *Kt = reinterpret_cast<T *>(lds[wave]), *Vt = Kt + kUnit * KS;
  uint4 kn[NPV], vn[NPV];
  const int v_c = lane % CPR, v_r = lane / CPR;
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  // Appending (p.fuse_append): rows [new0, new0 + seqlen_knew) of this batch come from k_new /
  // v_new instead of the cache and are written to the cache by the one lane that loads them
  // (reference: the Append_KV branch of compute_attn_1rowblock_splitkv, flash_fwd_kernel.h:660-740).
  const int new0 = p.fuse_append ? p.seqlens_k[bi] : 0x7fffffff;
  const T *kng = p.fuse_append ? static_cast<const T *>(p.k_new) + bi * p.knew_bs + hk * p.knew_hs : nullptr;
  const T *vng = p.fuse_append ? static_cast<const T *>(p.v_new) + bi * p.vnew_bs + hk * p.vnew_hs : nullptr;
  auto load_unit = [&](int j) {  // unit j of the chunk into the staging registers
#pragma unroll
    for (int s = 0; s < NPV; ++s) {
      const int key = c0 + j * kUnit + s * RPP + v_r;
      if (key < c1 && v_c * 8 < p.d) {  // columns from head_dim up to D stay zero
        const bool fresh = key >= new0;
        T *kc_row = const_cast<T *>(kg) + (int64_t)key * p.k_rs + v_c * 8;
        T *vc_row = const_cast<T *>(vg) + (int64_t)key * p.v_rs + v_c * 8;
        const T *ks_row = fresh ? kng + (int64_t)(key - new0) * p.knew_rs + v_c * 8 : kc_row;
        const T *vs_row = fresh ? vng + (int64_t)(key - new0) * p.vnew_rs + v_c * 8 : vc_row;
        const u32x4 a = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(ks_row));
        const u32x4 b = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(vs_row));
        kn[s] = uint4{a.x, a.y, a.z, a.w};
        vn[s] = uint4{b.x, b.y, b.z, b.w};
        if (fresh) {
          *reinterpret_cast<uint4 *>(kc_row) = kn[s];
          *reinterpret_cast<uint4 *>(vc_row) = vn[s];
        }
      } else {  // zero rows: 0 * finite stays finite in P V
        kn[s] = uint4{0, 0, 0, 0};
        vn[s] = uint4{0, 0, 0, 0};
      }
    }
  };
  auto store_unit = [&]() {
#pragma unroll
    for (int s = 0; s < NPV; ++s) {
      *reinterpret_cast<uint4 *>(&Kt[(s * RPP + v_r) * KS + v_c * 8]) = kn[s];
      *reinterpret_cast<uint4 *>(&Vt[(s * RPP + v_r) * VS + v_c * 8]) = vn[s];
    }
    FA_WAVE_SYNC();  // the wave's own tile: written by all its lanes, read across lanes, no workgroup barrier
  };

  float16v o_acc[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) o_acc[i] = float16v{0};
  float m_run = -INFINITY, l_run = 0.f;
  const float c = p.scale_log2;

  if (wave < n_units) {
    load_unit(wave);
    store_unit();
  }
  for (int j = wave; j < n_units; j += kDecWaves) {
    const bool has_next = j + kDecWaves < n_units;
    if (has_next) load_unit(j + kDecWaves);
    float16v s = float16v{0};
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks)
      s = Traits<T>::mfma(lds_read8<T>(&Kt[r32 * KS + ks * 16 + g * 8]), qf[ks], s);
    const int kv0 = c0 + j * kUnit;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int kv = kv0 + (i >> 2) * 8 + g * 4 + (i & 3);
      if (kv >= hi_lim || kv < lo_lim) s[i] = -INFINITY;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[i]);
    mx = fmaxf(mx, partner32(mx));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = exp2_fast((m_run - m_use) * c);
    const float m_scaled = m_use * c;
    float rs = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float e = exp2_fast(fmaf(s[i], c, -m_scaled));
      s[i] = e;
      rs += e;
    }
    l_run = l_run * alpha + rs;
    m_run = m_new;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o_acc[db][i] *= alpha;
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      float pf[8];
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) pf[jj] = s[w * 8 + jj];
      const vec8 pb = pack8<T>(pf);
#pragma unroll
      for (int db = 0; db < D / 32; ++db) {
        const vec8 av = lds_read_operand_tr<T>(Vt, VS, w * 16, db * 32);
        o_acc[db] = Traits<T>::mfma(av, pb, o_acc[db]);
      }
    }
    if (has_next) store_unit();  // after every read of unit j in program order
  }

  // ---- merge the four waves' partials through LDS (each wave writes into its own region) ----
  const float l_wave = l_run + partner32(l_run);
  float *Ow = reinterpret_cast<float *>(lds[wave]);  // [D][32]
  float *MLw = Ow + D * 32;                          // [2][32]
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) Ow[(db * 32 + (i >> 2) * 8 + g * 4 + (i & 3)) * 32 + r32] = o_acc[db][i];
  if (g == 0) { MLw[r32] = m_run; MLw[32 + r32] = l_wave; }
  __syncthreads();

  const int n = tid & 31, slice = tid >> 5;  // eight slices of D / 8 output elements per column
  float mw[kDecWaves], wgt[kDecWaves], m_all = -INFINITY, l_all = 0.f;
#pragma unroll
  for (int w = 0; w < kDecWaves; ++w) {
    mw[w] = reinterpret_cast<const float *>(lds[w])[D * 32 + n];
    m_all = fmaxf(m_all, mw[w]);
  }
  const float m_ref = m_all == -INFINITY ? 0.f : m_all;
#pragma unroll
  for (int w = 0; w < kDecWaves; ++w) {
    wgt[w] = exp2_fast((mw[w] - m_ref) * c);  // 0 for a wave that saw no key
    l_all += wgt[w] * reinterpret_cast<const float *>(lds[w])[D * 32 + 32 + n];
  }
  const bool out_ok = n < group * p.sq;
  const int oi = out_ok ? n % p.sq : 0, oh = hk * group + (out_ok ? n / p.sq : 0);
  const bool final_pass = a.o_part == nullptr;
  const bool empty = l_all == 0.f || l_all != l_all;
  const float inv = final_pass ? (empty ? 1.f : 1.f / l_all) : 1.f;
  T *og = static_cast<T *>(p.o_w) + bi * p.o_bs + (int64_t)oi * p.o_rs + oh * p.o_hs;
  const int64_t prow = (((int64_t)split * p.b + bi) * p.h + oh) * p.sq + oi;
#pragma unroll
  for (int x = 0; x < D / 8; ++x) {
    const int dcol = slice * (D / 8) + x;
    float acc = 0.f;
#pragma unroll
    for (int w = 0; w < kDecWaves; ++w) acc += wgt[w] * reinterpret_cast<const float *>(lds[w])[dcol * 32 + n];
    if (out_ok) {
      if (!final_pass) a.o_part[prow * D + dcol] = acc;
      else if (dcol < p.d) og[dcol] = (T)(acc * inv);
    }
  }
  if (out_ok && slice == 0) {
    if (final_pass) p.lse[((int64_t)bi * p.h + oh) * p.sq + oi] = empty ? INFINITY : m_all * p.scale + log2_fast(l_all) * kLn2;
    else { a.ml_part[prow * 2] = m_all; a.ml_part[prow * 2 + 1] = l_all; }
  }
}

// merges the chunks' partials of one (batch, head, query row) per workgroup, one thread per
// output element; n_splits <= 64, so lane s of every wave takes chunk s for the statistics
template <typename T, int D>
__global__ void __launch_bounds__(D < 64 ? 64 : D) decode_merge_kernel(const Params p, const DecodeArgs a) {
  __shared__ float wgt[64];
  const int64_t row = blockIdx.x;  // (batch * h + head) * sq + query row
  const int64_t rows = (int64_t)p.b * p.h * p.sq;
  const int dcol = threadIdx.x < D ? threadIdx.x : D - 1, lane = threadIdx.x & 63;  // whole waves only
  const bool has = lane < a.n_splits;
  const float m_s = has ? a.ml_part[(lane * rows + row) * 2] : -INFINITY;
  const float l_s = has ? a.ml_part[(lane * rows + row) * 2 + 1] : 0.f;
  float m_all = m_s;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m_all = fmaxf(m_all, __shfl_xor(m_all, off, 64));
  const float m_ref = m_all == -INFINITY ? 0.f : m_all;
  const float w_s = exp2_fast((m_s - m_ref) * p.scale_log2);  // 0 for a chunk that saw no key
  float l_all = w_s * l_s;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) l_all += __shfl_xor(l_all, off, 64);
  if (threadIdx.x < 64) wgt[threadIdx.x] = w_s;
  __syncthreads();
  float acc = 0.f;
  const float *op = a.o_part + row * D + dcol;
#pragma unroll 8
  for (int s = 0; s < a.n_splits; ++s) acc += wgt[s] * op[s * rows * D];
  const bool empty = l_all == 0.f || l_all != l_all;
  const int qi = (int)(row % p.sq), hq = (int)((row / p.sq) % p.h), bi = (int)(row / ((int64_t)p.sq * p.h));
  T *og = static_cast<T *>(p.o_w) + bi * p.o_bs + (int64_t)qi * p.o_rs + hq * p.o_hs;
  if (threadIdx.x < p.d) og[dcol] = (T)(empty ? 0.f : acc / l_all);
  if (threadIdx.x == 0) p.lse[row] = empty ? INFINITY : m_all * p.scale + log2_fast(l_all) * kLn2;
}

template <typename T, int D>
hipError_t decode_td(const Params &p, hipStream_t stream) {
  const int base = p.b * p.h_k;
  // enough workgroups for two per CU, but at least 512 keys per chunk
  int n_splits = (2 * 256 + base - 1) / base;
  n_splits = max(1, min(n_splits, min(64, p.sk / 512)));
  DecodeArgs a{};
  a.n_splits = n_splits;
  a.chunk = ((p.sk + n_splits - 1) / n_splits + kUnit * kDecWaves - 1) / (kUnit * kDecWaves) * (kUnit * kDecWaves);
  void *ws = nullptr;
  bool owned = false;
  const size_t rows = (size_t)p.b * p.h * p.sq;
  const size_t need = n_splits > 1 ? (size_t)n_splits * rows * (D + 2) * sizeof(float) : 0;
  if (p.ws_query) { *p.ws_query = need; return hipSuccess; }
  if (need) {
    if (p.ws && (reinterpret_cast<uintptr_t>(p.ws) & 15) == 0 && p.ws_bytes >= need) ws = p.ws;
    else if (hipMallocAsync(&ws, need, stream) == hipSuccess) owned = true;
    else { (void)hipGetLastError(); ws = nullptr; }
    if (!ws) {  // no scratch: one chunk per (batch, key/value head)
      a.n_splits = 1;
      a.chunk = (p.sk + kUnit - 1) / kUnit * kUnit;
    } else {
      a.o_part = static_cast<float *>(ws);
      a.ml_part = a.o_part + (size_t)n_splits * rows * D;
    }
  }
  FA_LAUNCH((decode_kernel<T, D>), dim3((unsigned)(base * a.n_splits)), dim3(kDecWaves * 64), stream, p, a);
  hipError_t e = hipGetLastError();
  if (ws) {
    if (e == hipSuccess) {
      FA_LAUNCH((decode_merge_kernel<T, D>), dim3((unsigned)rows), dim3(D < 64 ? 64 : D), stream, p, a);
      e = hipGetLastError();
    }
    if (owned) {
      const hipError_t f = hipFreeAsync(ws, stream);
      if (e == hipSuccess) e = f;
    }
  }
  return e;
}

template <typename T>
hipError_t split_merge_t(const Params &p, hipStream_t stream) {
  DecodeArgs a{};
  a.o_part = p.o_part; a.ml_part = p.ml_part; a.n_splits = p.n_splits;
  const dim3 grid((unsigned)((size_t)p.b * p.h * p.sq));
  switch (p.d) {
  case 32: FA_LAUNCH((decode_merge_kernel<T, 32>), grid, dim3(64), stream, p, a); break;
  case 64: FA_LAUNCH((decode_merge_kernel<T, 64>), grid, dim3(64), stream, p, a); break;
  case 128: FA_LAUNCH((decode_merge_kernel<T, 128>), grid, dim3(128), stream, p, a); break;
  default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_split_merge(const Params &p, int dtype, hipStream_t stream) {
  if (p.n_splits > 64) return hipErrorInvalidValue;
  return dtype == 1 ? split_merge_t<_Float16>(p, stream) : split_merge_t<__bf16>(p, stream);
}

bool decode_eligible(const Params &p) {
  return p.d <= 256 && p.sq > 0 && (p.h / p.h_k) * p.sq <= 32 && p.sk >= 1 && !p.drop;
}

// The decode kernel can do the append itself when every appended row is certain to be loaded by
// it: no left window (rows below the window are never fetched).
bool decode_can_append(const Params &p) {
  return decode_eligible(p) && p.k_new && p.v_new && p.seqlens_k && p.seqlen_knew > 0 && p.wl < 0;
}

hipError_t launch_decode(Params &p, int dtype, hipStream_t stream) {
  if (p.b * p.h == 0 || p.sq == 0) return hipSuccess;
  // D is the tile width: the smallest of 32, 64, 128, 256 that holds head_dim (a multiple of 8);
  // the columns between head_dim and D are zero in the tiles and never loaded or stored
  if (p.d <= 32) return dtype == 1 ? decode_td<_Float16, 32>(p, stream) : decode_td<__bf16, 32>(p, stream);
  if (p.d <= 64) return dtype == 1 ? decode_td<_Float16, 64>(p, stream) : decode_td<__bf16, 64>(p, stream);
  if (p.d <= 128) return dtype == 1 ? decode_td<_Float16, 128>(p, stream) : decode_td<__bf16, 128>(p, stream);
  return dtype == 1 ? decode_td<_Float16, 256>(p, stream) : decode_td<__bf16, 256>(p, stream);
}

}  // namespace fa
