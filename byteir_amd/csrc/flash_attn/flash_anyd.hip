// Flash-attention forward and backward for every head dimension the reference accepts
// (a multiple of 8 up to 256; external_libs/runtime/flash_attn/lib/flash_api.cu:163-225
// dispatches on head_dim <= 32, 64, ... 256) other than the three that have tuned kernels
// (32, 64, 128).
//
// The head dimension d is rounded up to DR (32, 64, 96, 128, 192 or 256): tiles and operand
// fragments are DR wide, columns d..DR-1 are filled with zeros on the way in (they add nothing
// to Q K^T or dO V^T and give zero output columns) and are not written on the way out.  The
// structure is the plain one: one workgroup of four waves owns 128 rows (queries in forward
// and dQ, keys in dK/dV), each wave 32 of them; the other operand streams through one LDS tile
// of 64 rows, prefetched into registers during the math of the previous tile when DR <= 128
// and loaded between the two barriers otherwise (the wide kernels have no registers to spare).
// The arithmetic, the masks and the operand orientation are those of flash_fwd.hip and
// flash_bwd.hip: S^T = K Q^T with one query per lane, P rounded to the storage type before
// P V, exp2 with scale*log2(e) folded in, LSE = max*scale + ln(sum); backward recomputes P
// from the forward's LSE, dS = P * (dP - D), no atomics, one launch each for D, dK/dV and dQ.
//
// These kernels also carry dropout for every head dimension (the tuned kernels do not): the
// keep-mask is the reference's function of (seed, offset, batch, head, row, column)
// (lib/dropout.h, lib/philox.cuh), evaluated here for the elements a lane holds in the MFMA
// accumulator layout; the scalings follow the reference (forward: row sums of the undropped P,
// O / p_keep; backward: D * p_keep, dS = P * (keep ? dP - D : -D), dQ and dK / p_keep, dV / p_keep).
#include "flash_common.h"

namespace fa {
namespace {

constexpr int kRows = 128;  // rows per workgroup, 32 per wave
constexpr int kTile = 64;   // rows per LDS tile

// Copies a [ROWS x DR] tile (rows row0.. of a strided [n_rows, d] matrix) through registers
// into LDS; rows >= n_rows and columns >= d arrive as zeros.  DR / 8 chunks of 16 bytes per
// row need not divide the workgroup: the threads left over after the last whole row idle.
template <typename T, int DR, int ROWS>
struct AnyTileLoader {
  static constexpr int CPR = DR / 8;
  static constexpr int RPP = 256 / CPR;
  static constexpr int NP = (ROWS + RPP - 1) / RPP;
  uint4 reg[NP];
  __device__ __forceinline__ void gload(const T *base, int64_t row_stride, int row0, int n_rows, int d) {
    const int c = threadIdx.x % CPR, r = threadIdx.x / CPR;
#pragma unroll
    for (int s = 0; s < NP; ++s) {
      const int row = row0 + s * RPP + r;
      if (r < RPP && s * RPP + r < ROWS && row < n_rows && c * 8 < d)
        reg[s] = *reinterpret_cast<const uint4 *>(base + (int64_t)row * row_stride + c * 8);
      else
        reg[s] = uint4{0, 0, 0, 0};
    }
  }
  __device__ __forceinline__ void lstore(T *tile, int stride) const {
    const int c = threadIdx.x % CPR, r = threadIdx.x / CPR;
#pragma unroll
    for (int s = 0; s < NP; ++s)
      if (r < RPP && s * RPP + r < ROWS)
        *reinterpret_cast<uint4 *>(&tile[(s * RPP + r) * stride + c * 8]) = reg[s];
  }
};

// the 8 elements at column ks*16 + g*8 of a global row, zero beyond d or for a row that does not exist
template <typename T>
__device__ __forceinline__ typename Traits<T>::vec8 load_frag(const T *row, bool row_ok, int col, int d) {
  using vec8 = typename Traits<T>::vec8;
  if (row_ok && col < d) return *reinterpret_cast<const vec8 *>(row + col);
  return vec8{0};
}

// 16 accumulator values of a lane -> 4 stores of 4 elements at columns db*32 + i4*8 + g*4
template <typename T>
__device__ __forceinline__ void store_acc(T *row, const float16v &acc, int db, int g, float mul, int d) {
  typedef T vec4 __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int i4 = 0; i4 < 4; ++i4) {
    const int col = db * 32 + i4 * 8 + g * 4;
    if (col < d) {
      vec4 v;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = (T)(acc[i4 * 4 + j] * mul);
      *reinterpret_cast<vec4 *>(row + col) = v;
    }
  }
}

// Philox4x32 with 7 rounds (lib/philox.cuh:22-52): key = seed, counter = (offset, subsequence).
__device__ __forceinline__ uint4 philox7(uint32_t k0, uint32_t k1, uint64_t offset, uint32_t sub_lo, uint32_t sub_hi) {
  uint32_t c0 = (uint32_t)offset, c1 = (uint32_t)(offset >> 32), c2 = sub_lo, c3 = sub_hi;
#pragma unroll
  for (int r = 0; r < 7; ++r) {
    if (r > 0) { k0 += 0x9E3779B9u; k1 += 0xBB67AE85u; }
    // one 32 x 32 -> 64-bit multiply per product (v_mad_u64_u32) instead of a high and a low one
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0, hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
    c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
  }
  return uint4{c0, c1, c2, c3};
}

// The reference draws one Philox value per (16-row x 32-column block of the attention matrix,
// lane of a 32-lane warp): 16 bytes, one per element that lane holds in the m16n8 accumulator
// layout: row = lane/4 (+8), column = 8*tile + 2*(lane%4) (+1) for four 8-column tiles, byte =
// 4*tile + 2*(row half) + (column & 1); subsequence = (row block, column block), offset =
// rng_state[1] + (batch*heads + head)*32 + lane; an element is kept iff its byte <= threshold
// (lib/dropout.h:19-23,38-84; call sites flash_fwd_kernel.h:321-334, flash_bwd_kernel.h:524-533).
struct DropCtx {
  uint32_t k0, k1;
  uint64_t off;   // rng_state[1] + (batch*heads + head)*32
  uint32_t thr;
  __device__ __forceinline__ void init(const Params &p, int bh) {
    const uint64_t seed = p.rng_state[0];
    k0 = (uint32_t)seed; k1 = (uint32_t)(seed >> 32);
    off = p.rng_state[1] + (uint64_t)(bh * 32);
    thr = p.keep_thr;
  }
  // One Philox value per lane covers a whole 32 x 32 block of the attention matrix (rows q32..,
  // columns kv32.., both multiples of 32): lane L draws the value of warp lane L % 32 in row
  // block q32/16 + L/32.  Bit 4*tile + 2*(row half) + (column & 1) of the result is set when
  // that byte is kept.  Every lane of the wave must take part (the callers below exchange the
  // words across lanes).
  __device__ __forceinline__ uint32_t draw(int q32, int kv32) const {
    const int L = threadIdx.x & 63;
    const uint4 r = philox7(k0, k1, off + (uint32_t)(L & 31), (uint32_t)((q32 >> 4) + (L >> 5)), (uint32_t)(kv32 >> 5));
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
    uint32_t m = 0;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int b = 0; b < 4; ++b)
        if (((w[t] >> (8 * b)) & 0xffu) <= thr) m |= 1u << (4 * t + b);
    return m;
  }
  // Scores held with the query on the lane (column of S^T): bit i of the result is set when
  // key kv32 + 8*(i/4) + 4*g + i%4 is kept for query q = q32 + lane % 32.  The 16 elements lie
  // in the values of warp lanes (q%8)*4 + 2*g + {0, 1} of row block q/16.
  __device__ __forceinline__ uint32_t keep_q_on_lane(int q, int kv32, int g) const {
    const uint32_t own = draw(q & ~31, kv32);
    const int src = ((q >> 4) & 1) * 32 + (q & 7) * 4 + g * 2, sh = ((q >> 3) & 1) * 2;
    uint32_t m = 0;
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2) {
      const uint32_t w = (uint32_t)__builtin_amdgcn_ds_bpermute((src + c2) * 4, (int)own);
      m |= ((w >> sh) & 0x3333u) << (2 * c2);
    }
    return m;
  }
  // Scores held with the key on the lane (column of S): bit i is set when query
  // q32 + 8*(i/4) + 4*g + i%4 is kept for key kv = kv32 + lane % 32.  The 16 elements lie in the
  // values of warp lanes (4*g + j)*4 + (kv%8)/2, j = 0..3, of both row blocks.
  __device__ __forceinline__ uint32_t keep_k_on_lane(int q32, int kv, int g) const {
    const uint32_t own = draw(q32, kv & ~31);
    const uint32_t other = (uint32_t)__builtin_amdgcn_ds_bpermute(((threadIdx.x & 63) ^ 32) * 4, (int)own);
    const uint32_t both = (threadIdx.x & 32) ? (other | own << 16) : (own | other << 16);  // row block 0 low
    const int sh = ((kv & 31) >> 3) * 4 + (kv & 1);
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t x = (uint32_t)__builtin_amdgcn_ds_bpermute(((g * 4 + j) * 4 + ((kv & 7) >> 1)) * 4, (int)both) >> sh;
      // bits 0, 2 (row halves of row block 0) and 16, 18 (row block 1) -> rows 8*a + 4*g + j, a = 0..3
      m |= ((x & 1u) | ((x & 4u) << 2) | ((x >> 8) & 0x100u) | ((x >> 6) & 0x1000u)) << j;
    }
    return m;
  }
};

__device__ __forceinline__ void block_of(const Params &p, int n_blocks, bool reversed, int &blk, int &bh,
                                         int n_bh = -1) {  // n_bh: (batch, head) pairs, b * h by default
  if (n_bh < 0) n_bh = p.b * p.h;
  const int L = blockIdx.x;
  if (p.xcd_remap == 2) {  // unequal blocks: the longest block of every (batch, head) first
    const int xcd = L & 7, slot = L >> 3, per_xcd = n_bh >> 3;
    bh = (slot % per_xcd) * 8 + xcd;
    blk = slot / per_xcd;
  } else if (p.xcd_remap == 3) {  // the same order when b*h is not a multiple of the XCD count
    bh = L % n_bh;
    blk = L / n_bh;
  } else if (p.xcd_remap) {  // consecutive workgroup ids go round-robin over the 8 XCDs
    const int xcd = L & 7, slot = L >> 3;
    bh = (slot / n_blocks) * 8 + xcd;
    blk = slot % n_blocks;
  } else {
    bh = L / n_blocks;
    blk = L % n_blocks;
  }
  if (reversed) blk = n_blocks - 1 - blk;  // longest (causal) blocks first
}

// ---- forward ----------------------------------------------------------------------------------
template <typename T, int DR, bool Drop>
__global__ void __launch_bounds__(256, DR <= 128 ? 2 : 1) fwd_anyd_kernel(const Params p) {
  using vec8 = typename Traits<T>::vec8;
  constexpr int KS = Pad<DR>::kPlain, VS = Pad<DR>::kTr;
  constexpr bool kPrefetch = DR <= 128;
  __shared__ __attribute__((aligned(16))) T Ks[kTile * KS];
  __shared__ __attribute__((aligned(16))) T Vs[kTile * VS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, g = lane >> 5;
  int m_block, bh;
  block_of(p, p.n_mblocks, true, m_block, bh);
  const int bi = bh / p.h, hi = bh % p.h, hk = hi / (p.h / p.h_k);
  int sk = p.sk;
  if (p.seqlens_k) sk = min(p.sk, p.seqlens_k[bi] + p.seqlen_knew);
  const int m0 = m_block * kRows, wq0 = m0 + wave * 32, qrow = wq0 + r32;

  int lo_lim, hi_lim, w_lo_first, w_hi_first, w_lo_last, w_hi_last, b_lo, b_hi, t0, t1;
  row_limits_sk(p, sk, qrow, lo_lim, hi_lim);
  row_limits_sk(p, sk, wq0, w_lo_first, w_hi_first);
  row_limits_sk(p, sk, wq0 + 31, w_lo_last, w_hi_last);
  row_limits_sk(p, sk, m0, b_lo, t0);
  row_limits_sk(p, sk, m0 + kRows - 1, t1, b_hi);
  const int n_min = b_lo / kTile;
  const int n_max = b_hi > 0 ? (b_hi + kTile - 1) / kTile : 0;

  const T *qg = static_cast<const T *>(p.q) + bi * p.q_bs + (int64_t)qrow * p.q_rs + hi * p.q_hs;
  const T *kg = static_cast<const T *>(p.k) + bi * p.k_bs + hk * p.k_hs;
  const T *vg = static_cast<const T *>(p.v) + bi * p.v_bs + hk * p.v_hs;

  vec8 qf[DR / 16];
#pragma unroll
  for (int ks = 0; ks < DR / 16; ++ks) qf[ks] = load_frag<T>(qg, qrow < p.sq, ks * 16 + g * 8, p.d);

  AnyTileLoader<T, DR, kTile> lk, lv;
  auto gload = [&](int t) {
    lk.gload(kg, p.k_rs, t * kTile, sk, p.d);
    lv.gload(vg, p.v_rs, t * kTile, sk, p.d);  // zero rows: 0 * finite stays finite in P V
  };
  auto lstore = [&]() { lk.lstore(Ks, KS); lv.lstore(Vs, VS); };

  float16v o_acc[DR / 32];
#pragma unroll
  for (int i = 0; i < DR / 32; ++i) o_acc[i] = float16v{0};
  float m_run = -INFINITY, l_run = 0.f;
  const float c = p.scale_log2;
  DropCtx drop;
  if constexpr (Drop) drop.init(p, bh);

  if (kPrefetch && n_min < n_max) {
    gload(n_min);
    lstore();
    __syncthreads();
  }
  for (int t = n_min; t < n_max; ++t) {
    const int kv0 = t * kTile;
    if constexpr (kPrefetch) {
      if (t + 1 < n_max) gload(t + 1);
    } else {
      gload(t);
      lstore();
      __syncthreads();
    }
    // the wave sees nothing of this tile when it lies wholly outside the widest row window
    const bool skip = kv0 >= w_hi_last || kv0 + kTile <= w_lo_first;
    if (!skip) {
      float16v s[2];
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb) {
        s[kvb] = float16v{0};
#pragma unroll
        for (int ks = 0; ks < DR / 16; ++ks) {
          const vec8 a = lds_read8<T>(&Ks[(kvb * 32 + r32) * KS + ks * 16 + g * 8]);
          s[kvb] = Traits<T>::mfma(a, qf[ks], s[kvb]);
        }
      }
      if (kv0 + kTile > w_hi_first || kv0 < w_lo_last) {  // a tile on the edge of the window
#pragma unroll
        for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int kv = kv0 + kvb * 32 + (i >> 2) * 8 + g * 4 + (i & 3);
            if (kv >= hi_lim || kv < lo_lim) s[kvb][i] = -INFINITY;
          }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kvb][i]);
      mx = fmaxf(mx, partner32(mx));
      const float m_new = fmaxf(m_run, mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = exp2_fast((m_run - m_use) * c);
      const float m_scaled = m_use * c;
      float rs = 0.f;
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float e = exp2_fast(fmaf(s[kvb][i], c, -m_scaled));
          s[kvb][i] = e;
          rs += e;
        }
      l_run = l_run * alpha + rs;
      m_run = m_new;
      if constexpr (Drop) {  // the row sum above is that of the undropped P
#pragma unroll
        for (int kvb = 0; kvb < 2; ++kvb) {
          const uint32_t keep = drop.keep_q_on_lane(qrow, kv0 + kvb * 32, g);
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if (!((keep >> i) & 1u)) s[kvb][i] = 0.f;
        }
      }
#pragma unroll
      for (int db = 0; db < DR / 32; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[db][i] *= alpha;
      // O^T += V^T P^T, 16 keys per step
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float pf[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) pf[j] = s[w >> 1][(w & 1) * 8 + j];
        const vec8 pb = pack8<T>(pf);
#pragma unroll
        for (int db = 0; db < DR / 32; ++db) {
          const vec8 a = lds_read_operand_tr<T>(Vs, VS, w * 16, db * 32);
          o_acc[db] = Traits<T>::mfma(a, pb, o_acc[db]);
        }
      }
    }
    __syncthreads();  // every wave is done with the tile in LDS
    if constexpr (kPrefetch) {
      if (t + 1 < n_max) lstore();
      __syncthreads();
    }
  }

  // epilogue: normalise, write O and LSE
  const float l_tot = l_run + partner32(l_run);
  const bool empty = l_tot == 0.f || l_tot != l_tot;
  float inv = empty ? 1.f : 1.f / l_tot;
  if constexpr (Drop) inv *= p.rp_keep;
  if (qrow < p.sq) {
    T *og = static_cast<T *>(p.o_w) + bi * p.o_bs + (int64_t)qrow * p.o_rs + hi * p.o_hs;
#pragma unroll
    for (int db = 0; db < DR / 32; ++db) store_acc<T>(og, o_acc[db], db, g, inv, p.d);
    if (g == 0)
      p.lse[((int64_t)bi * p.h + hi) * p.sq + qrow] =
          empty ? INFINITY : m_run * p.scale + log2_fast(l_tot) * kLn2;
  }
}

// ---- backward 1: D = rowsum(dO * O), half a wave per row ------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) dot_do_o_anyd_kernel(const Params p) {
  const int sub = threadIdx.x & 31;
  const int64_t row = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);  // over b * h * sq
  const int64_t total = (int64_t)p.b * p.h * p.sq;
  const bool ok = row < total;
  const int64_t rr = ok ? row : total - 1;
  const int i = (int)(rr % p.sq);
  const int hi = (int)((rr / p.sq) % p.h);
  const int bi = (int)(rr / ((int64_t)p.sq * p.h));
  const int64_t off = bi * p.o_bs + (int64_t)i * p.o_rs + hi * p.o_hs + sub * 8;
  typedef T vec8 __attribute__((ext_vector_type(8)));
  float s = 0.f;
  if (sub * 8 < p.d) {
    const vec8 a = *reinterpret_cast<const vec8 *>(static_cast<const T *>(p.dout) + off);
    const vec8 o = *reinterpret_cast<const vec8 *>(static_cast<const T *>(p.o) + off);
#pragma unroll
    for (int j = 0; j < 8; ++j) s += (float)a[j] * (float)o[j];
  }
#pragma unroll
  for (int m = 16; m > 0; m >>= 1) s += __shfl_xor(s, m, 64);
  if (p.drop) s *= p.p_keep;  // flash_bwd_preprocess_kernel.h:124-128
  if (ok && sub == 0) p.dsoftmax[((int64_t)bi * p.h + hi) * p.sq_rounded + i] = s;
}

// ---- backward 2: dK, dV -----------------------------------------------------------------------------
template <typename T, int DR, bool Drop>
__global__ void __launch_bounds__(256, DR <= 64 ? 2 : 1) dkdv_anyd_kernel(const Params p) {
  using vec8 = typename Traits<T>::vec8;
  constexpr int QS = Pad<DR>::kPlain;  // tiles are read both plainly and transposed
  constexpr bool kPrefetch = DR <= 128;
  __shared__ __attribute__((aligned(16))) T Qs[kTile * QS];
  __shared__ __attribute__((aligned(16))) T dOs[kTile * QS];
  __shared__ float lse_s[kTile];
  __shared__ float dsm_s[kTile];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, g = lane >> 5;
  int n_block, bh;
  block_of(p, p.n_nblocks, false, n_block, bh, p.b * p.h_k);
  // a workgroup belongs to a key/value head; its dK, dV sum over the query heads of the group
  // (with shares: bh runs over virtual heads; hk = key/value head * gsplit + group share)
  const int bi = bh / p.h_k, vh = bh % p.h_k, hk = vh / p.qsplit, q_share = vh % p.qsplit;
  const int group = p.h / (p.h_k / p.qsplit);
  const int kvb0 = n_block * kRows;
  const int kvcol = kvb0 + wave * 32 + r32;  // the key this lane owns
  const int off = p.sk - p.sq;

  const T *qg = nullptr, *dog = nullptr;  // of the query head being streamed (set per head below)
  const float *lse_g = nullptr, *dsm_g = nullptr;
  const int hkv = hk / p.gsplit;  // the key/value head whose query heads this workgroup takes a share of
  const T *kg = static_cast<const T *>(p.k) + bi * p.k_bs + (int64_t)kvcol * p.k_rs + hkv * p.k_hs;
  const T *vg = static_cast<const T *>(p.v) + bi * p.v_bs + (int64_t)kvcol * p.v_rs + hkv * p.v_hs;

  vec8 kf[DR / 16], vf[DR / 16];
#pragma unroll
  for (int ks = 0; ks < DR / 16; ++ks) {
    kf[ks] = load_frag<T>(kg, kvcol < p.sk, ks * 16 + g * 8, p.d);
    vf[ks] = load_frag<T>(vg, kvcol < p.sk, ks * 16 + g * 8, p.d);
  }
  float16v dk_acc[DR / 32], dv_acc[DR / 32];
#pragma unroll
  for (int i = 0; i < DR / 32; ++i) { dk_acc[i] = float16v{0}; dv_acc[i] = float16v{0}; }

  // query tiles that can see keys [kvb0, kvb0 + 128)
  int q_lo = 0, q_hi = p.sq;
  if (p.wr >= 0) q_lo = max(0, kvb0 - off - p.wr);              // hi(q) = q+1+off+wr > kvb0
  if (p.wl >= 0) q_hi = min(p.sq, kvb0 + kRows - off + p.wl);   // lo(q) = q+off-wl < kvb0+128
  int m_min = q_lo / kTile;
  int m_max = q_hi > 0 ? (q_hi + kTile - 1) / kTile : 0;
  if (p.qsplit > 1) {  // this workgroup's share of the visible query tiles
    const int per = (max(m_max - m_min, 0) + p.qsplit - 1) / p.qsplit;
    m_min += q_share * per;
    m_max = min(m_max, m_min + per);
  }
  const float c = p.scale_log2;
  DropCtx drop;

  AnyTileLoader<T, DR, kTile> lq, ldo;
  float lse_r = 0.f, dsm_r = 0.f;
  auto gload = [&](int m) {
    lq.gload(qg, p.q_rs, m * kTile, p.sq, p.d);
    ldo.gload(dog, p.o_rs, m * kTile, p.sq, p.d);
    if (tid < kTile) {
      const int q = m * kTile + tid;
      lse_r = q < p.sq ? lse_g[q] : INFINITY;  // +inf: the row contributes P = 0
      dsm_r = q < p.sq ? dsm_g[q] : 0.f;
    }
  };
  auto lstore = [&]() {
    lq.lstore(Qs, QS);
    ldo.lstore(dOs, QS);
    if (tid < kTile) { lse_s[tid] = lse_r * kLog2e; dsm_s[tid] = dsm_r; }
  };

  int drop_bh = 0;  // batch * heads + query head: the dropout stream of the head being processed
  for (int gq = 0; gq < group; ++gq) {  // the query heads that share this key/value head
  const int hi = hk * group + gq;
  qg = static_cast<const T *>(p.q) + bi * p.q_bs + hi * p.q_hs;
  dog = static_cast<const T *>(p.dout) + bi * p.o_bs + hi * p.o_hs;
  lse_g = p.lse + ((int64_t)bi * p.h + hi) * p.sq;
  dsm_g = p.dsoftmax + ((int64_t)bi * p.h + hi) * p.sq_rounded;
  drop_bh = bi * p.h + hi;
  if constexpr (Drop) drop.init(p, drop_bh);
  if (kPrefetch && m_min < m_max) {
    gload(m_min);
    lstore();
    __syncthreads();
  }
  for (int m = m_min; m < m_max; ++m) {
    if constexpr (kPrefetch) {
      if (m + 1 < m_max) gload(m + 1);
    } else {
      gload(m);
      lstore();
      __syncthreads();
    }
#pragma unroll
    for (int qs = 0; qs < kTile / 32; ++qs) {
      const int q0 = m * kTile + qs * 32;  // first query row of this 32-row sub-tile
      // wave-uniform visibility of the sub-tile against the wave's 32 keys
      const int wkv0 = kvb0 + wave * 32;
      int lo_first, hi_first, lo_last, hi_last;
      row_limits(p, q0, lo_first, hi_first);
      row_limits(p, q0 + 31, lo_last, hi_last);
      if (wkv0 >= hi_last || wkv0 + 32 <= lo_first) continue;  // nothing kept
      const bool need_mask = wkv0 + 32 > hi_first || wkv0 < lo_last || q0 + 32 > p.sq;

      float16v s = float16v{0}, dp = float16v{0};
#pragma unroll
      for (int ks = 0; ks < DR / 16; ++ks) {
        const vec8 aq = lds_read8<T>(&Qs[(qs * 32 + r32) * QS + ks * 16 + g * 8]);
        s = Traits<T>::mfma(aq, kf[ks], s);
        const vec8 ad = lds_read8<T>(&dOs[(qs * 32 + r32) * QS + ks * 16 + g * 8]);
        dp = Traits<T>::mfma(ad, vf[ks], dp);
      }
      float pv[16], dsv[16];
      uint32_t keep = 0xffffu;
      if constexpr (Drop) keep = drop.keep_k_on_lane(q0, kvcol, g);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int ql = qs * 32 + (i >> 2) * 8 + g * 4 + (i & 3);  // row inside the LDS tile
        float pe = exp2_fast(fmaf(s[i], c, -lse_s[ql]));
        if (need_mask) {
          int lo, hi_;
          row_limits(p, m * kTile + ql, lo, hi_);
          if (kvcol >= hi_ || kvcol < lo) pe = 0.f;
        }
        const bool kept = !Drop || ((keep >> i) & 1u);
        pv[i] = kept ? pe : 0.f;
        dsv[i] = pe * ((kept ? dp[i] : 0.f) - dsm_s[ql]);
      }
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const vec8 pb = pack8<T>(&pv[w * 8]);
        const vec8 dsb = pack8<T>(&dsv[w * 8]);
#pragma unroll
        for (int db = 0; db < DR / 32; ++db) {
          const vec8 a_do = lds_read_operand_tr<T>(dOs, QS, qs * 32 + w * 16, db * 32);
          dv_acc[db] = Traits<T>::mfma(a_do, pb, dv_acc[db]);
          const vec8 a_q = lds_read_operand_tr<T>(Qs, QS, qs * 32 + w * 16, db * 32);
          dk_acc[db] = Traits<T>::mfma(a_q, dsb, dk_acc[db]);
        }
      }
    }
    __syncthreads();
    if constexpr (kPrefetch) {
      if (m + 1 < m_max) lstore();
      __syncthreads();
    }
  }

  }
  if (kvcol < p.sk) {
    const float mk = Drop ? p.scale * p.rp_keep : p.scale, mv = Drop ? p.rp_keep : 1.f;
    if (p.gsplit * p.qsplit > 1) {  // a share of the work of a key/value head: float partials [b, sk, virtual heads, d]
      float *dkp = static_cast<float *>(p.dk) + bi * p.dk_bs + (int64_t)kvcol * p.dk_rs + vh * p.dk_hs;
      float *dvp = static_cast<float *>(p.dv) + bi * p.dv_bs + (int64_t)kvcol * p.dv_rs + vh * p.dv_hs;
#pragma unroll
      for (int db = 0; db < DR / 32; ++db) {
        store_acc<float>(dkp, dk_acc[db], db, g, mk, p.d);
        store_acc<float>(dvp, dv_acc[db], db, g, mv, p.d);
      }
    } else {
      T *dkg = static_cast<T *>(p.dk) + bi * p.dk_bs + (int64_t)kvcol * p.dk_rs + hk * p.dk_hs;
      T *dvg = static_cast<T *>(p.dv) + bi * p.dv_bs + (int64_t)kvcol * p.dv_rs + hk * p.dv_hs;
#pragma unroll
      for (int db = 0; db < DR / 32; ++db) {
        store_acc<T>(dkg, dk_acc[db], db, g, mk, p.d);
        store_acc<T>(dvg, dv_acc[db], db, g, mv, p.d);
      }
    }
  }
}

// ---- backward 3: dQ ---------------------------------------------------------------------------------
template <typename T, int DR, bool Drop>
__global__ void __launch_bounds__(256, (DR <= 96 || (DR == 128 && !Drop)) ? 2 : 1) dq_anyd_kernel(const Params p) {
  using vec8 = typename Traits<T>::vec8;
  constexpr int KS = Pad<DR>::kPlain;  // K tile: plain and transposed reads
  constexpr int VS = Pad<DR>::kPlain;  // V tile: plain reads only
  constexpr bool kPrefetch = DR <= 128;
  __shared__ __attribute__((aligned(16))) T Ks[kTile * KS];
  __shared__ __attribute__((aligned(16))) T Vs[kTile * VS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, g = lane >> 5;
  int m_block, bh;
  block_of(p, p.n_mblocks, true, m_block, bh);
  const int bi = bh / p.h, hi = bh % p.h;
  const int m0 = m_block * kRows, wq0 = m0 + wave * 32, qrow = wq0 + r32;

  int lo_lim, hi_lim, w_lo_first, w_hi_first, w_lo_last, w_hi_last, b_lo, b_hi, t0, t1;
  row_limits(p, qrow, lo_lim, hi_lim);
  row_limits(p, wq0, w_lo_first, w_hi_first);
  row_limits(p, wq0 + 31, w_lo_last, w_hi_last);
  row_limits(p, m0, b_lo, t0);
  row_limits(p, m0 + kRows - 1, t1, b_hi);
  const int n_min = b_lo / kTile;
  const int n_max = b_hi > 0 ? (b_hi + kTile - 1) / kTile : 0;

  const T *qg = static_cast<const T *>(p.q) + bi * p.q_bs + (int64_t)qrow * p.q_rs + hi * p.q_hs;
  const T *dog = static_cast<const T *>(p.dout) + bi * p.o_bs + (int64_t)qrow * p.o_rs + hi * p.o_hs;
  const int hk = hi / (p.h / p.h_k);
  const T *kg = static_cast<const T *>(p.k) + bi * p.k_bs + hk * p.k_hs;
  const T *vg = static_cast<const T *>(p.v) + bi * p.v_bs + hk * p.v_hs;

  vec8 qf[DR / 16], dof[DR / 16];
#pragma unroll
  for (int ks = 0; ks < DR / 16; ++ks) {
    qf[ks] = load_frag<T>(qg, qrow < p.sq, ks * 16 + g * 8, p.d);
    dof[ks] = load_frag<T>(dog, qrow < p.sq, ks * 16 + g * 8, p.d);
  }
  float lse_l = INFINITY, dsm_l = 0.f;
  if (qrow < p.sq) {
    lse_l = p.lse[((int64_t)bi * p.h + hi) * p.sq + qrow] * kLog2e;
    dsm_l = p.dsoftmax[((int64_t)bi * p.h + hi) * p.sq_rounded + qrow];
  }
  float16v dq_acc[DR / 32];
#pragma unroll
  for (int i = 0; i < DR / 32; ++i) dq_acc[i] = float16v{0};
  const float c = p.scale_log2;
  DropCtx drop;
  if constexpr (Drop) drop.init(p, bh);

  AnyTileLoader<T, DR, kTile> lk, lv;
  auto gload = [&](int t) {
    lk.gload(kg, p.k_rs, t * kTile, p.sk, p.d);
    lv.gload(vg, p.v_rs, t * kTile, p.sk, p.d);
  };
  auto lstore = [&]() { lk.lstore(Ks, KS); lv.lstore(Vs, VS); };

  if (kPrefetch && n_min < n_max) {
    gload(n_min);
    lstore();
    __syncthreads();
  }
  for (int t = n_min; t < n_max; ++t) {
    const int kv0 = t * kTile;
    if constexpr (kPrefetch) {
      if (t + 1 < n_max) gload(t + 1);
    } else {
      gload(t);
      lstore();
      __syncthreads();
    }
    const bool skip = kv0 >= w_hi_last || kv0 + kTile <= w_lo_first;
    if (!skip) {
      const bool need_mask = kv0 + kTile > w_hi_first || kv0 < w_lo_last;
      float16v s[2], dp[2];
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb) {
        s[kvb] = float16v{0};
        dp[kvb] = float16v{0};
#pragma unroll
        for (int ks = 0; ks < DR / 16; ++ks) {
          const vec8 ak = lds_read8<T>(&Ks[(kvb * 32 + r32) * KS + ks * 16 + g * 8]);
          s[kvb] = Traits<T>::mfma(ak, qf[ks], s[kvb]);
          const vec8 av = lds_read8<T>(&Vs[(kvb * 32 + r32) * VS + ks * 16 + g * 8]);
          dp[kvb] = Traits<T>::mfma(av, dof[ks], dp[kvb]);
        }
      }
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb) {
        uint32_t keep = 0xffffu;
        if constexpr (Drop) keep = drop.keep_q_on_lane(qrow, kv0 + kvb * 32, g);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float pe = exp2_fast(fmaf(s[kvb][i], c, -lse_l));
          if (need_mask) {
            const int kv = kv0 + kvb * 32 + (i >> 2) * 8 + g * 4 + (i & 3);
            if (kv >= hi_lim || kv < lo_lim) pe = 0.f;
          }
          const bool kept = !Drop || ((keep >> i) & 1u);
          s[kvb][i] = pe * ((kept ? dp[kvb][i] : 0.f) - dsm_l);  // dS^T
        }
      }
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float f[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] = s[w >> 1][(w & 1) * 8 + j];
        const vec8 dsb = pack8<T>(f);
#pragma unroll
        for (int db = 0; db < DR / 32; ++db) {
          const vec8 a = lds_read_operand_tr<T>(Ks, KS, w * 16, db * 32);
          dq_acc[db] = Traits<T>::mfma(a, dsb, dq_acc[db]);
        }
      }
    }
    __syncthreads();
    if constexpr (kPrefetch) {
      if (t + 1 < n_max) lstore();
      __syncthreads();
    }
  }

  if (qrow < p.sq) {
    T *dqg = static_cast<T *>(p.dq) + bi * p.q_bs + (int64_t)qrow * p.q_rs + hi * p.q_hs;
#pragma unroll
    for (int db = 0; db < DR / 32; ++db)
      store_acc<T>(dqg, dq_acc[db], db, g, Drop ? p.scale * p.rp_keep : p.scale, p.d);
  }
}

template <typename T, int DR>
hipError_t fwd_anyd_d(const Params &p, hipStream_t stream) {
  const dim3 grid((unsigned)(p.n_mblocks * p.b * p.h)), block(256);
  if (p.drop) FA_LAUNCH((fwd_anyd_kernel<T, DR, true>), grid, block, stream, p);
  else FA_LAUNCH((fwd_anyd_kernel<T, DR, false>), grid, block, stream, p);
  return hipGetLastError();
}

template <typename T, int DR>
hipError_t bwd_anyd_d(const Params &p, hipStream_t stream) {
  const dim3 gk((unsigned)(p.n_nblocks * p.b * p.h_k)), gq((unsigned)(p.n_mblocks * p.b * p.h)), block(256);
  if (p.n_nblocks > 0) {
    Params pk = p;  // the dK/dV grid runs over key/value heads (or shares of their groups)
    pk.dk_bs = p.k_bs; pk.dk_rs = p.k_rs; pk.dk_hs = p.k_hs;
    pk.dv_bs = p.v_bs; pk.dv_rs = p.v_rs; pk.dv_hs = p.v_hs;
    pk.gsplit = pk.qsplit = 1;
    const GroupSplit split = plan_group_split(p, (int64_t)p.n_nblocks * p.b * p.h_k, 256 * (DR <= 64 ? 2 : 1), p.d, kTile, stream);
    if (p.ws_query) return hipSuccess;  // planning only
    apply_group_split(pk, p, split, p.d);
    pk.xcd_remap = ((p.b * pk.h_k) % 8 == 0) ? (p.wr >= 0 ? 2 : 1) : (p.wr >= 0 ? 3 : 0);
    const dim3 gks((unsigned)(p.n_nblocks * p.b * pk.h_k));
    if (p.drop) FA_LAUNCH((dkdv_anyd_kernel<T, DR, true>), gks, block, stream, pk);
    else FA_LAUNCH((dkdv_anyd_kernel<T, DR, false>), gks, block, stream, pk);
    if (split.gs * split.qs > 1) {
      const hipError_t e = launch_group_sum(p, split, p.d, std::is_same<T, _Float16>::value ? 1 : 2, stream);
      if (e != hipSuccess) return e;
    }
  }
  if (p.n_mblocks > 0 && !p.ws_query) {
    if (p.drop) FA_LAUNCH((dq_anyd_kernel<T, DR, true>), gq, block, stream, p);
    else FA_LAUNCH((dq_anyd_kernel<T, DR, false>), gq, block, stream, p);
  }
  return hipGetLastError();
}

template <typename T>
hipError_t fwd_anyd_t(const Params &p, hipStream_t stream) {
  if (p.d <= 32) return fwd_anyd_d<T, 32>(p, stream);
  if (p.d <= 64) return fwd_anyd_d<T, 64>(p, stream);
  if (p.d <= 96) return fwd_anyd_d<T, 96>(p, stream);
  if (p.d <= 128) return fwd_anyd_d<T, 128>(p, stream);
  if (p.d <= 192) return fwd_anyd_d<T, 192>(p, stream);
  return fwd_anyd_d<T, 256>(p, stream);
}

template <typename T>
hipError_t bwd_anyd_t(const Params &p, hipStream_t stream) {
  const int64_t rows = (int64_t)p.b * p.h * p.sq;
  if (rows > 0 && !p.ws_query) FA_LAUNCH((dot_do_o_anyd_kernel<T>), dim3((unsigned)((rows + 7) / 8)), dim3(256), stream, p);
  if (p.d <= 32) return bwd_anyd_d<T, 32>(p, stream);
  if (p.d <= 64) return bwd_anyd_d<T, 64>(p, stream);
  if (p.d <= 96) return bwd_anyd_d<T, 96>(p, stream);
  if (p.d <= 128) return bwd_anyd_d<T, 128>(p, stream);
  if (p.d <= 192) return bwd_anyd_d<T, 192>(p, stream);
  return bwd_anyd_d<T, 256>(p, stream);
}

}  // namespace

hipError_t launch_fwd_anyd(Params &p, int dtype, hipStream_t stream) {
  if (p.d <= 0 || p.d > 256 || p.d % 8 != 0) return hipErrorInvalidValue;
  p.n_mblocks = (p.sq + kRows - 1) / kRows;
  if (p.n_mblocks == 0 || p.ws_query) return hipSuccess;  // this path takes no scratch
  return dtype == 1 ? fwd_anyd_t<_Float16>(p, stream) : fwd_anyd_t<__bf16>(p, stream);
}

// dQ alone, head_dim 128 without dropout, for the tuned backward: at two waves per SIMD (two
// workgroups per CU, which overlap each other's start and end) this kernel is 3-8 % faster than
// a kernel tuned for one wave per SIMD once the grid has two workgroups for every CU (512...2048
// heads x 1024...4096 keys, causal and full); the caller keeps the tuned kernel for smaller grids.
hipError_t launch_dq_anyd128(const Params &p, int dtype, hipStream_t stream) {
  Params pq = p;
  pq.n_mblocks = (p.sq + kRows - 1) / kRows;
  if (pq.n_mblocks == 0) return hipSuccess;
  const dim3 grid((unsigned)(pq.n_mblocks * p.b * p.h)), block(256);
  if (dtype == 1) FA_LAUNCH((dq_anyd_kernel<_Float16, 128, false>), grid, block, stream, pq);
  else FA_LAUNCH((dq_anyd_kernel<__bf16, 128, false>), grid, block, stream, pq);
  return hipGetLastError();
}

hipError_t launch_bwd_anyd(Params &p, int dtype, hipStream_t stream) {
  if (p.d <= 0 || p.d > 256 || p.d % 8 != 0) return hipErrorInvalidValue;
  p.n_mblocks = (p.sq + kRows - 1) / kRows;
  p.n_nblocks = (p.sk + kRows - 1) / kRows;
  return dtype == 1 ? bwd_anyd_t<_Float16>(p, stream) : bwd_anyd_t<__bf16>(p, stream);
}

}  // namespace fa
