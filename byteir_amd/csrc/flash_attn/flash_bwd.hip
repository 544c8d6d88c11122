// Flash-attention backward for gfx950.  Three launches, no atomics, deterministic:
//   1. dot_do_o_kernel : D[b,h,i] = sum_d dO[i,d] * O[i,d]                      (fp32)
//   2. dkdv_kernel     : one workgroup per 128 keys, loops over query tiles;
//                        dV = P^T dO, dK = scale * dS^T Q accumulate in registers
//   3. dq_kernel       : one workgroup per 128 queries, loops over key tiles;
//                        dQ = scale * dS K accumulates in registers
// P = exp2(scale*log2e * S - log2e * LSE) is recomputed from the forward's LSE in both main
// kernels; dS = P * (dO V^T - D).  P and dS are rounded to the storage type before they
// enter a GEMM, as in the reference (external_libs/runtime/flash_attn/lib/
// flash_bwd_kernel.h:455-718, flash_bwd_preprocess_kernel.h:23-136,180-262).  The reference
// accumulates dQ across key blocks with float atomics into dq_accum and converts it in a
// third kernel; here the dQ pass owns its rows instead, which removes the atomics (and the
// run-to-run variation they cause) at the price of recomputing S and dP.
//
// Operand orientation (see flash_common.h for the register layouts):
//   dkdv: S = Q K^T and dP = dO V^T have queries on rows, keys on columns, so a lane owns one
//         key; P and dS then feed dV^T += dO^T P and dK^T += Q^T dS as B operands while dO^T
//         and Q^T come out of the row-major LDS tiles through the transposing read.
//   dq:   S^T = K Q^T and dP^T = V dO^T have queries on columns (LSE and D are lane-local);
//         dS^T feeds dQ^T += K^T dS^T as the B operand, K^T through the transposing read.
#include <algorithm>
#include "flash_common.h"

namespace fa {

// ---- 1. D = rowsum(dO * O) ----------------------------------------------------------------
template <typename T, int D>
__global__ void __launch_bounds__(256) dot_do_o_kernel(const Params p) {
  constexpr int LPR = D / 8;       // lanes per row, 16 bytes each
  constexpr int RPB = 256 / LPR;   // rows per workgroup
  const int sub = threadIdx.x % LPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;  // over b * h * sq
  const int64_t total = (int64_t)p.b * p.h * p.sq;
  const bool ok = row < total;
  const int64_t rr = ok ? row : total - 1;
  const int i = (int)(rr % p.sq);
  const int hi = (int)((rr / p.sq) % p.h);
  const int bi = (int)(rr / ((int64_t)p.sq * p.h));
  const int64_t off = bi * p.o_bs + (int64_t)i * p.o_rs + hi * p.o_hs + sub * 8;
  typedef T vec8 __attribute__((ext_vector_type(8)));
  const vec8 a = *reinterpret_cast<const vec8 *>(static_cast<const T *>(p.dout) + off);
  const vec8 o = *reinterpret_cast<const vec8 *>(static_cast<const T *>(p.o) + off);
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) s += (float)a[j] * (float)o[j];
#pragma unroll
  for (int m = LPR / 2; m > 0; m >>= 1) s += __shfl_xor(s, m, 64);
  if (ok && sub == 0) p.dsoftmax[((int64_t)bi * p.h + hi) * p.sq_rounded + i] = s;
}

constexpr int kKvBlock = 128;  // keys per workgroup in dkdv (32 per wave)
constexpr int kQTile = 64;     // query rows per LDS tile in dkdv
constexpr int kQBlock = 128;   // queries per workgroup in dq (32 per wave)
constexpr int kKvTile = 64;    // key rows per LDS tile in dq

// Streams consecutive [ROWS x D] tiles of a [n_rows, D] strided matrix through registers: a
// running 32-bit offset to this thread's chunks of the next tile, advanced by one tile per
// gload, into a buffer descriptor over the matrix.
template <typename T, int D, int ROWS>
struct TileLoader {
  static constexpr int CPR = D / 8;
  static constexpr int RPP = 256 / CPR;
  static constexpr int NP = ROWS / RPP;
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  uint4 reg[NP];
  __amdgpu_buffer_rsrc_t rsrc;  // covers rows [0, n_rows): rows beyond read as zeros
  unsigned vo[NP];              // byte offset of this thread's chunk in the next tile, per pass
  unsigned tile_b;              // bytes from one tile to the next
  // The first gload fetches the tile that starts at row0.  Raw buffer loads: no bounds branch
  // and no 64-bit address arithmetic per load (measured 3 % on the bf16 head_dim-64
  // backward).  The running offsets travel in the vector offset, which is what the hardware
  // checks against the descriptor's size; the launcher keeps a (batch, head) slice below
  // 2 GiB so they cannot wrap.
  __device__ __forceinline__ void start(const T *base, int64_t row_stride, int row0, int n_rows) {
    const int c = threadIdx.x % CPR, r = threadIdx.x / CPR;
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(base), 0, idx::rsrc_bytes(n_rows, row_stride, D), 0x00020000);
#pragma unroll
    for (int s = 0; s < NP; ++s) vo[s] = idx::chunk_offset(row0 + r + s * RPP, c, row_stride);
    tile_b = idx::tile_bytes(ROWS, row_stride);
  }
  // the next tile into a register set of the caller's (two tiles in flight at a workgroup's start)
  __device__ __forceinline__ void gload_into(uint4 (&r)[NP]) {
#pragma unroll
    for (int s = 0; s < NP; ++s) {
      const u32x4 a = __builtin_amdgcn_raw_buffer_load_b128(rsrc, vo[s], 0, 0);
      r[s] = uint4{a.x, a.y, a.z, a.w};
      vo[s] += tile_b;
    }
  }
  __device__ __forceinline__ void gload() { gload_into(reg); }
  __device__ __forceinline__ void lstore_swz_from(T *tile, const uint4 (&rr)[NP]) const {
    const int c = threadIdx.x % CPR, r = threadIdx.x / CPR;
#pragma unroll
    for (int s = 0; s < NP; ++s)
      *reinterpret_cast<uint4 *>(&tile[Swz<D>::off(s * RPP + r, c)]) = rr[s];
  }
  __device__ __forceinline__ void lstore(T *tile, int stride) const {
    const int c = threadIdx.x % CPR, r = threadIdx.x / CPR;
#pragma unroll
    for (int s = 0; s < NP; ++s)
      *reinterpret_cast<uint4 *>(&tile[(s * RPP + r) * stride + c * 8]) = reg[s];
  }
  // the same into a tile laid out with Swz<D> (no padding, chunks permuted per row)
  __device__ __forceinline__ void lstore_swz(T *tile) const {
    const int c = threadIdx.x % CPR, r = threadIdx.x / CPR;
#pragma unroll
    for (int s = 0; s < NP; ++s)
      *reinterpret_cast<uint4 *>(&tile[Swz<D>::off(s * RPP + r, c)]) = reg[s];
  }
};

// ---- 2. dK, dV ------------------------------------------------------------------------------
// One workgroup (4 waves) per 128 keys; a wave keeps the K and V fragments of its 32 keys in
// registers and walks the query axis in units of 32 rows, two units per 64-row LDS tile of Q,
// dO, LSE and D.  The tiles go through a three-deep LDS ring with one barrier per tile.
//
// Per unit a wave does A: S = Q K^T, dP = dO V^T (MFMA); B: P = exp2(..), dS = P (dP - D),
// rounded to the storage type and packed (vector ALU); C: dV^T += dO^T P, dK^T += Q^T dS
// (MFMA).  The loop is software pipelined with C one unit behind: a step holds A and B of the
// current unit and C of the previous one, whose MFMAs do not depend on the vector work of B
// and run under it (delaying C costs 16 registers for a second set of packed P / dS;
// producing S and dP one unit ahead would cost 32 and does not fit two waves per SIMD).
// The step has a single instance: window edges are applied as -inf scores between A and B, a
// unit that the wave's keys do not see at all is treated like an edge unit (it adds zeros),
// and the first step accumulates a zero P / dS.
// KB: 32-key blocks per wave; the workgroup covers 128*KB keys and every Q / dO fragment read
// from LDS feeds KB MFMAs.
template <typename T, int D, int KB>
__global__ void __launch_bounds__(256, (D <= 64 && KB == 1) ? 2 : 1) dkdv_kernel(const Params p) {
  using vec8 = typename Traits<T>::vec8;
  // Tiles are read both plainly and transposed.  A stride of 4*odd banks keeps the plain reads
  // free of bank conflicts; the transposed ones then conflict in about a fifth of the LDS
  // cycles (a third with D + 16, nearly half with D + 32) -- with < 3 % effect on the time.
  constexpr int QS = D;  // unpadded, chunks permuted per row (Swz<D>): read plainly and transposed
  constexpr int kRing = 3;
  __shared__ __attribute__((aligned(16))) T Qs[kRing][kQTile * QS];
  __shared__ __attribute__((aligned(16))) T dOs[kRing][kQTile * QS];
  __shared__ __attribute__((aligned(16))) float lse_s[kRing][kQTile];
  __shared__ __attribute__((aligned(16))) float dsm_s[kRing][kQTile];

  const int tid = threadIdx.x, lane = tid & 63;
  // the wave index in a scalar register: everything derived from it (row windows, edge
  // decisions) then stays scalar and branches on it are real branches
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r32 = lane & 31, g = lane >> 5;
  // unequal blocks (a window): the longest (first) key block of every head first
  const idx::BlockId blk = idx::decode_block((int)blockIdx.x, p.xcd_remap, p.b * p.h_k, p.n_nblocks);
  const int bh = blk.bh, n_block = blk.blk;
  // a workgroup belongs to a key/value head; its dK, dV sum over the query heads of the group
  // (with shares: bh runs over virtual heads; hk = key/value head * gsplit + group share)
  const int bi = bh / p.h_k, vh = bh % p.h_k, hk = vh / p.qsplit, q_share = vh % p.qsplit;
  const int group = p.h / (p.h_k / p.qsplit);
  constexpr int kKeys = kKvBlock * KB;
  const int kvb0 = n_block * kKeys;
  const int wkv0 = kvb0 + wave * 32 * KB;  // first key of the wave
  const int off = p.sk - p.sq;

  // pointers of the query head being streamed (set per head below)
  const T *qg = nullptr, *dog = nullptr;
  const float *lse_g = nullptr, *dsm_g = nullptr;

  int kvcol[KB];  // the keys this lane owns
  vec8 kf[KB][D / 16], vf[KB][D / 16];
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    kvcol[kb] = wkv0 + kb * 32 + r32;
    const int hkv = hk / p.gsplit;  // the key/value head whose query heads this workgroup takes a share of
    const T *kg = static_cast<const T *>(p.k) + bi * p.k_bs + (int64_t)kvcol[kb] * p.k_rs + hkv * p.k_hs;
    const T *vg = static_cast<const T *>(p.v) + bi * p.v_bs + (int64_t)kvcol[kb] * p.v_rs + hkv * p.v_hs;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      if (kvcol[kb] < p.sk) {
        kf[kb][ks] = *reinterpret_cast<const vec8 *>(kg + ks * 16 + g * 8);
        vf[kb][ks] = *reinterpret_cast<const vec8 *>(vg + ks * 16 + g * 8);
      } else {
        kf[kb][ks] = vec8{0};
        vf[kb][ks] = vec8{0};
      }
    }
  }
  // head_dim 128 leaves room for one wave per SIMD, i.e. one workgroup per CU, so nothing covers
  // a workgroup's start and end: the first two Q / dO tiles then travel together with the K / V
  // fragments (a second register set, free at this occupancy), and dK / dV leave through LDS
  // as whole rows.  A round of 256 workgroups costs 13.7 us + 2.26 us per tile without this.
  constexpr bool kLean = D == 128;
  // consume the fragments once so that the wait for their loads sits here, not inside the loop
  auto consume_kv = [&]() {
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) FA_PIN2(kf[kb][ks], vf[kb][ks]);
  };
  if constexpr (!kLean) consume_kv();
  float16v dk_acc[KB][D / 32], dv_acc[KB][D / 32];
#pragma unroll
  for (int kb = 0; kb < KB; ++kb)
#pragma unroll
    for (int i = 0; i < D / 32; ++i) { dk_acc[kb][i] = float16v{0}; dv_acc[kb][i] = float16v{0}; }

  // query tiles that can see keys [kvb0, kvb0 + kKeys); with shares, this workgroup's part of them
  int m_min, m_max;
  idx::query_tile_range(p.sq, p.sk, p.wl, p.wr, kvb0, kKeys, kQTile, p.qsplit, q_share, m_min, m_max);
  // the same for the wave's own keys [wkv0, wkv0 + 32*KB)
  int qw_lo = 0, qw_hi = p.sq;
  if (p.wr >= 0) qw_lo = max(0, wkv0 - off - p.wr);
  if (p.wl >= 0) qw_hi = min(p.sq, wkv0 + 32 * KB - off + p.wl);
  const int m_w_min = min(m_max, max(m_min, qw_lo / kQTile));
  const int m_w_max = max(m_w_min, min(m_max, qw_hi > 0 ? (qw_hi + kQTile - 1) / kQTile : 0));
  const float c = p.scale_log2;
  // a key is kept for a query when key - (query + sk - sq) lies in [win_lo, win_lo + win_span]
  // (mask.h:160-200 of the reference; an unbounded side becomes +-2^30)
  const int win_lo = p.wl >= 0 ? -p.wl : -(1 << 30);
  const unsigned win_span = (unsigned)((p.wr >= 0 ? p.wr : (1 << 30)) - win_lo);

  TileLoader<T, D, kQTile> lq, ldo;  // tiles are fetched in order, m_min first
  float lse_r = 0.f, dsm_r = 0.f;
  int q_next = 0;  // the row whose LSE and D this thread stages next
  auto gload = [&]() {
    lq.gload();
    ldo.gload();
    if (tid < kQTile) {
      lse_r = q_next < p.sq ? lse_g[q_next] : INFINITY;  // +inf: the row contributes P = 0
      dsm_r = q_next < p.sq ? dsm_g[q_next] : 0.f;
    }
    q_next += kQTile;
  };
  auto lstore = [&](int buf) {
    lq.lstore_swz(Qs[buf]);
    ldo.lstore_swz(dOs[buf]);
    if (tid < kQTile) { lse_s[buf][tid] = lse_r * kLog2e; dsm_s[buf][tid] = -dsm_r; }
  };

  struct Unit { float16v s[KB], dp[KB]; };
  int frag_rd[D / 16];  // this lane's plain fragments inside a 32-row unit
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) frag_rd[ks] = Swz<D>::off(r32, ks * 2 + g);

  // A: S = Q K^T, dP - D = dO V^T - D for the 32 query rows of unit `qs` of a tile.  The
  // accumulator of dP starts from -D (staged negated in LDS, four consecutive rows per read in
  // the C layout), which takes the subtraction of dS = P (dP - D) off the vector ALU.
  auto part_a = [&](const T *Qt, const T *dOt, const float *negD, int qs, Unit &u) {
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const float4 d4 = *reinterpret_cast<const float4 *>(&negD[qs * 32 + i4 * 8 + g * 4]);
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        u.dp[kb][i4 * 4 + 0] = d4.x; u.dp[kb][i4 * 4 + 1] = d4.y;
        u.dp[kb][i4 * 4 + 2] = d4.z; u.dp[kb][i4 * 4 + 3] = d4.w;
      }
    }
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) u.s[kb] = float16v{0};
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      const vec8 aq = lds_read8<T>(&Qt[qs * 32 * QS + frag_rd[ks]]);
      const vec8 ad = lds_read8<T>(&dOt[qs * 32 * QS + frag_rd[ks]]);
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        u.s[kb] = Traits<T>::mfma(aq, kf[kb][ks], u.s[kb]);
        u.dp[kb] = Traits<T>::mfma(ad, vf[kb][ks], u.dp[kb]);
      }
    }
  };
  // scores outside the window become -inf (P = 0): key - (query + sk - sq) must lie in
  // [-wl, wr], one unsigned compare per element
  auto mask = [&](Unit &u, int q0) {
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const unsigned rel = (unsigned)(kvcol[kb] - off - q0 - g * 4 - ((i >> 2) * 8 + (i & 3)) - win_lo);
        if (rel > win_span) u.s[kb][i] = -INFINITY;
      }
  };
  // B: P and dS of the unit, rounded and packed as B operands [16-query window]
  auto part_b = [&](Unit &u, int buf, int qs, vec8 (&pb)[KB][2], vec8 (&dsb)[KB][2]) {
    float pv[KB][16], dsv[KB][16];
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const int ql = qs * 32 + i4 * 8 + g * 4;  // 4 consecutive rows of the LDS tile
      const float4 l4 = *reinterpret_cast<const float4 *>(&lse_s[buf][ql]);
      const float lq4[4] = {l4.x, l4.y, l4.z, l4.w};
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int i = i4 * 4 + j;
          const float pe = exp2_fast(fmaf(u.s[kb][i], c, -lq4[j]));
          pv[kb][i] = pe;
          dsv[kb][i] = pe * u.dp[kb][i];  // dp already holds dP - D
        }
    }
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        pb[kb][w] = pack8<T>(&pv[kb][w * 8]);
        dsb[kb][w] = pack8<T>(&dsv[kb][w * 8]);
      }
  };
  // C: dV^T += dO^T P, dK^T += Q^T dS
  auto part_c = [&](const T *Qt, const T *dOt, int qs, const vec8 (&pb)[KB][2], const vec8 (&dsb)[KB][2]) {
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int db = 0; db < D / 32; ++db) {
        const vec8 a_do = lds_read_operand_tr_swz<T, D>(dOt, qs * 32 + w * 16, db);
        const vec8 a_q = lds_read_operand_tr_swz<T, D>(Qt, qs * 32 + w * 16, db);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          dv_acc[kb][db] = Traits<T>::mfma(a_do, pb[kb][w], dv_acc[kb][db]);
          dk_acc[kb][db] = Traits<T>::mfma(a_q, dsb[kb][w], dk_acc[kb][db]);
        }
      }
  };
  // does the window keep every (query, key) pair of the 32 rows from q0 and the wave's keys?
  auto all_kept = [&](int q0) {
    int lo_first, hi_first, lo_last, hi_last;
    row_limits(p, q0, lo_first, hi_first);
    row_limits(p, q0 + 31, lo_last, hi_last);
    return wkv0 + 32 * KB <= hi_first && wkv0 >= lo_last;
  };
  vec8 pb[KB][2], dsb[KB][2];  // packed P and dS of the previous unit, still to be accumulated
#pragma unroll
  for (int kb = 0; kb < KB; ++kb)
#pragma unroll
    for (int w = 0; w < 2; ++w) { pb[kb][w] = vec8{0}; dsb[kb][w] = vec8{0}; }
  auto step = [&](int buf, int qs, int q0, int pbuf, int pqs) {
    Unit u;
    part_a(Qs[buf], dOs[buf], dsm_s[buf], qs, u);
    if (!all_kept(q0)) mask(u, q0);
    vec8 pb_new[KB][2], dsb_new[KB][2];
    part_c(Qs[pbuf], dOs[pbuf], pqs, pb, dsb);
    part_b(u, buf, qs, pb_new, dsb_new);
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int w = 0; w < 2; ++w) { pb[kb][w] = pb_new[kb][w]; dsb[kb][w] = dsb_new[kb][w]; }
  };

  const int n_tiles = m_max > m_min ? m_max - m_min : 0;
  for (int gq = 0; gq < group; ++gq) {  // the query heads that share this key/value head
  const int hi = hk * group + gq;
  qg = static_cast<const T *>(p.q) + bi * p.q_bs + hi * p.q_hs;
  dog = static_cast<const T *>(p.dout) + bi * p.o_bs + hi * p.o_hs;
  lse_g = p.lse + ((int64_t)bi * p.h + hi) * p.sq;
  dsm_g = p.dsoftmax + ((int64_t)bi * p.h + hi) * p.sq_rounded;
  lq.start(qg, p.q_rs, m_min * kQTile, p.sq);
  ldo.start(dog, p.o_rs, m_min * kQTile, p.sq);
  q_next = m_min * kQTile + tid;
  if (gq > 0) {
    __syncthreads();  // every wave has left the previous head's last tile
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int w = 0; w < 2; ++w) { pb[kb][w] = vec8{0}; dsb[kb][w] = vec8{0}; }
  }
  // prologue: tiles m_min and m_min+1 into the ring, tile m_min+2 into registers
  if constexpr (kLean) {
    uint4 q1[TileLoader<T, D, kQTile>::NP], do1[TileLoader<T, D, kQTile>::NP];
    float lse1 = 0.f, dsm1 = 0.f;
    if (n_tiles > 0) gload();
    if (n_tiles > 1) {  // tile m_min+1 in flight together with tile m_min
      lq.gload_into(q1);
      ldo.gload_into(do1);
      if (tid < kQTile) {
        lse1 = q_next < p.sq ? lse_g[q_next] : INFINITY;
        dsm1 = q_next < p.sq ? dsm_g[q_next] : 0.f;
      }
      q_next += kQTile;
    }
    if (gq == 0) consume_kv();
    if (n_tiles > 0) {
      lstore(0);
      if (n_tiles > 1) {
        lq.lstore_swz_from(Qs[1], q1);
        ldo.lstore_swz_from(dOs[1], do1);
        if (tid < kQTile) { lse_s[1][tid] = lse1 * kLog2e; dsm_s[1][tid] = -dsm1; }
      }
      if (n_tiles > 2) gload();
      __syncthreads();
    }
  } else if (n_tiles > 0) {
    gload();
    lstore(0);
    if (n_tiles > 1) { gload(); lstore(1); }
    if (n_tiles > 2) gload();
    __syncthreads();
  }
  int buf = 0, pbuf = 0;  // ring slots of tile m and of the tile of the pending unit
  int m = m_min;
  // query tiles that the wave's own 32*KB keys cannot see (the first ones under a right window,
  // the last ones under a left window): keep loading and meeting the barriers, compute nothing
  auto idle_tile = [&]() {
    const int buf1 = buf + 1 == kRing ? 0 : buf + 1;
    const int buf2 = buf1 + 1 == kRing ? 0 : buf1 + 1;
    __syncthreads();
    if (m + 2 < m_max) lstore(buf2);
    if (m + 3 < m_max) gload();
    buf = buf1;
  };
  for (; m < m_w_min; ++m) idle_tile();
  for (; m < m_w_max; ++m) {
    const int buf1 = buf + 1 == kRing ? 0 : buf + 1;
    const int buf2 = buf1 + 1 == kRing ? 0 : buf1 + 1;
    const int q0 = m * kQTile;
    // unit 0 of tile m; C of unit 1 of tile m-1 (still in its ring slot) rides along
    step(buf, 0, q0, pbuf, 1);
    __syncthreads();  // tile m+1 is visible; every wave has left tile m-1
    // tile m+2: registers -> the ring slot tile m-1 occupied; tile m+3 in flight
    if (m + 2 < m_max) lstore(buf2);
    if (m + 3 < m_max) gload();
    // unit 1 of tile m; C of unit 0 rides along
    step(buf, 1, q0 + 32, buf, 0);
    pbuf = buf;
    buf = buf1;
  }
  if (m_w_max > m_w_min) part_c(Qs[pbuf], dOs[pbuf], 1, pb, dsb);  // the last unit's C, before its slot is reused
  for (; m < m_max; ++m) idle_tile();
  }

  if (p.gsplit * p.qsplit > 1) {  // a share of the work of a key/value head: float partials [b, sk, virtual heads, D]
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      if (kvcol[kb] < p.sk) {
        float *dkp = static_cast<float *>(p.dk) + bi * p.dk_bs + (int64_t)kvcol[kb] * p.dk_rs + vh * p.dk_hs;
        float *dvp = static_cast<float *>(p.dv) + bi * p.dv_bs + (int64_t)kvcol[kb] * p.dv_rs + vh * p.dv_hs;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            const float16v &a = dk_acc[kb][db], &b = dv_acc[kb][db];
            *reinterpret_cast<float4 *>(dkp + db * 32 + i4 * 8 + g * 4) =
                float4{a[i4 * 4] * p.scale, a[i4 * 4 + 1] * p.scale, a[i4 * 4 + 2] * p.scale, a[i4 * 4 + 3] * p.scale};
            *reinterpret_cast<float4 *>(dvp + db * 32 + i4 * 8 + g * 4) = float4{b[i4 * 4], b[i4 * 4 + 1], b[i4 * 4 + 2], b[i4 * 4 + 3]};
          }
      }
    }
    return;
  }
  if constexpr (kLean) {
    // the wave's dK and dV rows -> its own [32][D] tiles in the idle Q and dO rings -> whole rows
    static_assert(KB == 1, "one key block per wave");
    // unpadded tiles; the 16-byte chunks of row r are permuted by r >> 1 and odd rows swap the
    // two 8-byte halves of a chunk: no bank conflicts for the 8-byte writes (a lane per row)
    // nor for the 16-byte reads (16 lanes per row)
    constexpr int OS = D, CPRO = D / 8, RPI = 64 / CPRO;
    static_assert(!kLean || (D == 128 && 4 * 32 * OS <= kRing * kQTile * QS), "staging must fit the ring; 16 chunks per row");
    __syncthreads();  // every wave has left the last Q / dO tile
    T *Kt = &Qs[0][0] + wave * 32 * OS, *Vt = &dOs[0][0] + wave * 32 * OS;
    typedef T vec4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        vec4 a, b;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          a[j] = (T)(dk_acc[0][db][i4 * 4 + j] * p.scale);
          b[j] = (T)(dv_acc[0][db][i4 * 4 + j]);
        }
        const int so = idx::ostage_write_offset(r32, g, db, i4);
        *reinterpret_cast<vec4 *>(&Kt[so]) = a;
        *reinterpret_cast<vec4 *>(&Vt[so]) = b;
      }
    FA_WAVE_SYNC();  // the wave's two tiles are complete; they are read back across lanes
    const int oc = lane % CPRO, orow = lane / CPRO;
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
      const int r = it * RPI + orow, kv = wkv0 + r;
      uint4 a = *reinterpret_cast<const uint4 *>(&Kt[idx::ostage_read_offset(r, oc)]);
      uint4 b = *reinterpret_cast<const uint4 *>(&Vt[idx::ostage_read_offset(r, oc)]);
      if (r & 1) { a = uint4{a.z, a.w, a.x, a.y}; b = uint4{b.z, b.w, b.x, b.y}; }
      if (kv < p.sk) {
        *reinterpret_cast<uint4 *>(static_cast<T *>(p.dk) + bi * p.dk_bs + (int64_t)kv * p.dk_rs + hk * p.dk_hs + oc * 8) = a;
        *reinterpret_cast<uint4 *>(static_cast<T *>(p.dv) + bi * p.dv_bs + (int64_t)kv * p.dv_rs + hk * p.dv_hs + oc * 8) = b;
      }
    }
    return;
  }
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    if (kvcol[kb] < p.sk) {
      T *dkg = static_cast<T *>(p.dk) + bi * p.dk_bs + (int64_t)kvcol[kb] * p.dk_rs + hk * p.dk_hs;
      T *dvg = static_cast<T *>(p.dv) + bi * p.dv_bs + (int64_t)kvcol[kb] * p.dv_rs + hk * p.dv_hs;
      typedef T vec4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          vec4 a, b;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            a[j] = (T)(dk_acc[kb][db][i4 * 4 + j] * p.scale);
            b[j] = (T)(dv_acc[kb][db][i4 * 4 + j]);
          }
          *reinterpret_cast<vec4 *>(dkg + db * 32 + i4 * 8 + g * 4) = a;
          *reinterpret_cast<vec4 *>(dvg + db * 32 + i4 * 8 + g * 4) = b;
        }
    }
  }
}

// ---- 3. dQ ----------------------------------------------------------------------------------
// One workgroup (4 waves x 32 query rows) per 128 queries; Q and dO fragments, LSE and D of a
// wave's rows stay in registers.  K and V go through a three-deep LDS ring in 64-row tiles with
// one barrier per tile, and are consumed in units of 32 keys.  Per unit: A: S^T = K Q^T and
// dP^T = V dO^T (MFMA); B: dS^T = P^T o (dP^T - D) in place of S^T, rounded and packed (vector
// ALU); C: dQ^T += K^T dS^T (MFMA, K^T through the transposing LDS read).  The loop is
// software pipelined like the forward kernel: one step holds A of the next unit together
// with B and C of the current one in a single basic block, so that matrix instructions run
// under the exponentials, and the K / V fragments of a unit are fetched from LDS a step before
// that.  Window edges are applied beforehand, by setting the masked scores
// of an edge unit to -inf in a block of their own, which keeps B free of branches.
template <typename T, int D>
__global__ void __launch_bounds__(256, D <= 64 ? 2 : 1) dq_kernel(const Params p) {
  using vec8 = typename Traits<T>::vec8;
  constexpr int KS = D;               // K tile: plain and transposed reads, laid out with Swz<D>
  constexpr int VS = Pad<D>::kPlain;  // V tile: plain reads only
  constexpr int kRing = 3;
  __shared__ __attribute__((aligned(16))) T Ks[kRing][kKvTile * KS];
  __shared__ __attribute__((aligned(16))) T Vs[kRing][kKvTile * VS];

  const int tid = threadIdx.x, lane = tid & 63;
  // the wave index in a scalar register: the skip and edge decisions derived from it are
  // scalar and every combination is its own straight-line instance of the step
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r32 = lane & 31, g = lane >> 5;
  // unequal blocks (a window): the longest (last) query block of every head first
  const idx::BlockId blk = idx::decode_block((int)blockIdx.x, p.xcd_remap, p.b * p.h, p.n_mblocks);
  const int bh = blk.bh, m_block = p.n_mblocks - 1 - blk.blk;
  const int bi = bh / p.h, hi = bh % p.h;
  const int m0 = m_block * kQBlock;
  const int wq0 = m0 + wave * 32;
  const int qrow = wq0 + r32;

  int lo_lim, hi_lim, w_lo_first, w_hi_first, w_lo_last, w_hi_last;
  row_limits(p, qrow, lo_lim, hi_lim);
  row_limits(p, wq0, w_lo_first, w_hi_first);
  row_limits(p, wq0 + 31, w_lo_last, w_hi_last);
  int n_min, n_max;
  idx::key_tile_range(p.sq, p.sk, p.wl, p.wr, m0, kQBlock, kKvTile, n_min, n_max);

  const int hk = hi / (p.h / p.h_k);
  const T *kg = static_cast<const T *>(p.k) + bi * p.k_bs + hk * p.k_hs;
  const T *vg = static_cast<const T *>(p.v) + bi * p.v_bs + hk * p.v_hs;

  vec8 qf[D / 16], dof[D / 16];
  float lse_l = INFINITY, dsm_l = 0.f;  // +inf: a row beyond seqlen_q contributes P = 0
  if (qrow < p.sq) {
    const T *qg = static_cast<const T *>(p.q) + bi * p.q_bs + (int64_t)qrow * p.q_rs + hi * p.q_hs;
    const T *dog = static_cast<const T *>(p.dout) + bi * p.o_bs + (int64_t)qrow * p.o_rs + hi * p.o_hs;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      qf[ks] = *reinterpret_cast<const vec8 *>(qg + ks * 16 + g * 8);
      dof[ks] = *reinterpret_cast<const vec8 *>(dog + ks * 16 + g * 8);
    }
    lse_l = p.lse[((int64_t)bi * p.h + hi) * p.sq + qrow] * kLog2e;
    dsm_l = p.dsoftmax[((int64_t)bi * p.h + hi) * p.sq_rounded + qrow];
  } else {
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) { qf[ks] = vec8{0}; dof[ks] = vec8{0}; }
  }
  // consume the fragments once so that the wait for their loads sits here, not inside the loop
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) FA_PIN2(qf[ks], dof[ks]);
  FA_PIN2(lse_l, dsm_l);
  // -D of the lane's row in all 16 accumulator slots: dP^T starts from it (the MFMA's C
  // operand), which takes the subtraction of dS = P (dP - D) off the vector ALU
  float16v neg_d;
#pragma unroll
  for (int i = 0; i < 16; ++i) neg_d[i] = -dsm_l;
  float16v dq_acc[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) dq_acc[i] = float16v{0};
  const float c = p.scale_log2;

  TileLoader<T, D, kKvTile> lk, lv;  // tiles are fetched in order, n_min first
  lk.start(kg, p.k_rs, n_min * kKvTile, p.sk);
  lv.start(vg, p.v_rs, n_min * kKvTile, p.sk);
  auto gload = [&]() { lk.gload(); lv.gload(); };
  auto lstore = [&](int buf) { lk.lstore_swz(Ks[buf]); lv.lstore(Vs[buf], VS); };

  struct Unit { float16v s, dp; };
  const int frag_v = r32 * VS + g * 8;
  int frag_k[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) frag_k[ks] = Swz<D>::off(r32, ks * 2 + g);

  // what the wave's 32 rows see of the 32 keys from kv0: 0 nothing, 1 all, 2 an edge crosses
  auto visibility = [&](int kv0) {
    if (kv0 >= w_hi_last || kv0 + 32 <= w_lo_first) return 0;
    return (kv0 + 32 > w_hi_first || kv0 < w_lo_last) ? 2 : 1;
  };
  // K and V fragments of one 32-key unit, fetched from LDS one step before the MFMAs that
  // use them, so that the LDS latency is not on the path of the step that consumes them
  vec8 fk[D / 16], fv[D / 16];
  auto fetch = [&](const T *Kt, const T *Vt, int kvb) {
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      fk[ks] = lds_read8<T>(&Kt[kvb * 32 * KS + frag_k[ks]]);
      fv[ks] = lds_read8<T>(&Vt[kvb * 32 * VS + frag_v + ks * 16]);
    }
  };
  // A: S^T = K Q^T, dP^T = V dO^T for the unit whose fragments are in fk / fv
  auto part_a = [&](Unit &u) {
    u.s = float16v{0};
    u.dp = neg_d;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      u.s = Traits<T>::mfma(fk[ks], qf[ks], u.s);
      u.dp = Traits<T>::mfma(fv[ks], dof[ks], u.dp);
    }
  };
  // the scores of an edge unit that fall outside the row's window become -inf (P = 0)
  auto mask = [&](Unit &u, int kv0) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int kv = kv0 + (i >> 2) * 8 + g * 4 + (i & 3);
      if (kv >= hi_lim || kv < lo_lim) u.s[i] = -INFINITY;
    }
  };
  // B: dS^T in place of S^T, packed as B operands [16-key window]
  auto part_b = [&](Unit &u, vec8 (&dsb)[2]) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float pe = exp2_fast(fmaf(u.s[i], c, -lse_l));
      u.s[i] = pe * u.dp[i];  // dp already holds dP - D
    }
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      float f[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = u.s[w * 8 + j];
      dsb[w] = pack8<T>(f);
    }
  };
  // C: dQ^T += K^T dS^T
  auto part_c = [&](const T *Kt, int kvb, const vec8 (&dsb)[2]) {
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int db = 0; db < D / 32; ++db) {
        const vec8 a = lds_read_operand_tr_swz<T, D>(Kt, kvb * 32 + w * 16, db);
        dq_acc[db] = Traits<T>::mfma(a, dsb[w], dq_acc[db]);
      }
  };
  // One pipeline step: finish unit `cur` (B, C) and, in the same basic block, start `nxt` (A).
  // The step has a single instance: a unit that a wave does not see at all is masked like an
  // edge unit (P = 0, it adds nothing) instead of being skipped, and the look-ahead past the
  // last tile reads a stale ring slot whose result is never used.  Variants of the step would
  // each accumulate into dQ, and the register allocator then reconciles their assignments
  // with 16 moves (and a drain of the matrix pipe) at the end of every step.
  auto step = [&](int vis, Unit &cur, int kv0, int buf, int kvb, Unit &nxt, int fbuf, int fkvb) {
    if (vis != 1) mask(cur, kv0);
    vec8 dsb[2];
    part_a(nxt);                        // the next unit, from the fragments fetched a step ago
    fetch(Ks[fbuf], Vs[fbuf], fkvb);    // fragments of the unit after next
    part_b(cur, dsb);
    part_c(Ks[buf], kvb, dsb);
  };

  // prologue: tiles n_min and n_min+1 into the ring, tile n_min+2 into registers
  const int n_tiles = n_max > n_min ? n_max - n_min : 0;
  Unit ua, ub;
  if (n_tiles > 0) {
    gload();
    lstore(0);
    if (n_tiles > 1) { gload(); lstore(1); }
    if (n_tiles > 2) gload();
    __syncthreads();
    fetch(Ks[0], Vs[0], 0);
    part_a(ua);
    fetch(Ks[0], Vs[0], 1);
  }
  // Under a right window (causal) the wave's rows see no key from w_hi_last on: it computes up
  // to the tile that holds that key and only keeps loading and meeting the barriers afterwards.
  const int n_w_max = min(n_max, max(n_min, (w_hi_last + kKvTile - 1) / kKvTile));
  int buf = 0;  // ring slot of tile t
  for (int t = n_min; t < n_max; ++t) {
    const int buf1 = buf + 1 == kRing ? 0 : buf + 1;
    const int buf2 = buf1 + 1 == kRing ? 0 : buf1 + 1;
    const int kv0 = t * kKvTile;
    if (t > n_min) __syncthreads();  // tile t+1 is visible; every wave has left tile t-1
    // tile t+2: registers -> the ring slot tile t-1 occupied; tile t+3 in flight
    if (t + 2 < n_max) lstore(buf2);
    if (t + 3 < n_max) gload();
    if (t < n_w_max) {
      // unit 0 of tile t (in ua); unit 1 is produced into ub; fragments of unit 0 of tile t+1
      step(visibility(kv0), ua, kv0, buf, 0, ub, buf1, 0);
      // unit 1 of tile t (in ub); unit 0 of tile t+1 into ua; fragments of its unit 1
      step(visibility(kv0 + 32), ub, kv0 + 32, buf, 1, ua, buf1, 1);
    }
    buf = buf1;
  }

  if (qrow < p.sq) {
    T *dqg = static_cast<T *>(p.dq) + bi * p.q_bs + (int64_t)qrow * p.q_rs + hi * p.q_hs;
    typedef T vec4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        vec4 a;
#pragma unroll
        for (int j = 0; j < 4; ++j) a[j] = (T)(dq_acc[db][i4 * 4 + j] * p.scale);
        *reinterpret_cast<vec4 *>(dqg + db * 32 + i4 * 8 + g * 4) = a;
      }
  }
}

// dk, dv = sums over the `gs` partial heads per key/value head; partials are float
// [b, sk, h_k*gs, row] (row = head_dim), one thread per 16 bytes of output, one rounding.
template <typename T>
__global__ void __launch_bounds__(256) group_sum_kernel(const Params p, const void *dk_part, const void *dv_part, int gs, int row) {
  const int cpr = row / 8;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t chunks = (int64_t)p.b * p.sk * p.h_k * cpr;
  if (idx >= chunks) return;
  const int c = (int)(idx % cpr);
  const int hk = (int)((idx / cpr) % p.h_k);
  const int64_t r = idx / ((int64_t)cpr * p.h_k);  // batch * sk + key
  const int kv = (int)(r % p.sk), bi = (int)(r / p.sk);
  const int64_t src = ((r * p.h_k + hk) * gs) * row + c * 8;
  float ak[8], av[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) { ak[j] = 0.f; av[j] = 0.f; }
  for (int s = 0; s < gs; ++s) {
    const float4 *rk = reinterpret_cast<const float4 *>(static_cast<const float *>(dk_part) + src + (int64_t)s * row);
    const float4 *rv = reinterpret_cast<const float4 *>(static_cast<const float *>(dv_part) + src + (int64_t)s * row);
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const float4 k4 = rk[half], v4 = rv[half];
      ak[half * 4] += k4.x; ak[half * 4 + 1] += k4.y; ak[half * 4 + 2] += k4.z; ak[half * 4 + 3] += k4.w;
      av[half * 4] += v4.x; av[half * 4 + 1] += v4.y; av[half * 4 + 2] += v4.z; av[half * 4 + 3] += v4.w;
    }
  }
  uint4 ok, ov;
  T *pk_ = reinterpret_cast<T *>(&ok), *pv_ = reinterpret_cast<T *>(&ov);
#pragma unroll
  for (int j = 0; j < 8; ++j) { pk_[j] = (T)ak[j]; pv_[j] = (T)av[j]; }
  *reinterpret_cast<uint4 *>(static_cast<T *>(p.dk) + bi * p.k_bs + (int64_t)kv * p.k_rs + hk * p.k_hs + c * 8) = ok;
  *reinterpret_cast<uint4 *>(static_cast<T *>(p.dv) + bi * p.v_bs + (int64_t)kv * p.v_rs + hk * p.v_hs + c * 8) = ov;
}

template <typename T, int D>
hipError_t launch_bwd_td(const Params &p, hipStream_t stream) {
  const int64_t rows = (int64_t)p.b * p.h * p.sq;
  if (rows > 0 && !p.ws_query) {
    constexpr int RPB = 256 / (D / 8);
    FA_LAUNCH((dot_do_o_kernel<T, D>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), stream, p);
  }
  // One 32-key block per wave.  Two blocks halve the LDS reads per MFMA (LDS bandwidth is
  // what bounds this kernel) but need about 450 registers: one wave per SIMD and accumulators
  // in AccVGPRs, whose results reach the vector ALU through a v_accvgpr_read per value;
  // measured 1.43 ms against 1.31 ms on the bf16 head_dim-64 benchmark.
  constexpr int KB = 1;
  Params pk = p;
  pk.n_nblocks = (p.sk + kKvBlock * KB - 1) / (kKvBlock * KB);
  pk.dk_bs = p.k_bs; pk.dk_rs = p.k_rs; pk.dk_hs = p.k_hs;
  pk.dv_bs = p.v_bs; pk.dv_rs = p.v_rs; pk.dv_hs = p.v_hs;
  pk.gsplit = pk.qsplit = 1;
  // chip slots for this kernel: 256 CUs, two workgroups each up to head_dim 64
  const GroupSplit split = plan_group_split(p, (int64_t)pk.n_nblocks * p.b * p.h_k, 256 * (D <= 64 ? 2 : 1), D, kQTile, stream);
  if (p.ws_query) return hipSuccess;  // planning only
  apply_group_split(pk, p, split, D);
  pk.xcd_remap = idx::block_order_mode(p.b * pk.h_k, p.wr);
  if (pk.n_nblocks > 0)
    FA_LAUNCH((dkdv_kernel<T, D, KB>), dim3((unsigned)(pk.n_nblocks * p.b * pk.h_k)), dim3(256), stream, pk);
  if (split.gs * split.qs > 1) {
    const hipError_t e = launch_group_sum(p, split, D, std::is_same<T, _Float16>::value ? 1 : 2, stream);
    if (e != hipSuccess) return e;
  }
  Params pq = p;
  pq.n_mblocks = (p.sq + kQBlock - 1) / kQBlock;
  if constexpr (D == 128) {
    // dq_kernel needs a whole SIMD per wave at this head dimension; the generic dQ kernel fits
    // two, and once there are two workgroups for every CU they overlap each other and it is
    // the faster one (3-8 %); on a smaller grid the one-wave kernel's deeper pipeline wins
    // (b1 h16 s1024 causal backward: 87 against 106 us)
    if ((int64_t)pq.n_mblocks * p.b * p.h >= 512) {
      const hipError_t e = hipGetLastError();
      return e != hipSuccess ? e : launch_dq_anyd128(p, std::is_same<T, _Float16>::value ? 1 : 2, stream);
    }
  }
  if (pq.n_mblocks > 0)
    FA_LAUNCH((dq_kernel<T, D>), dim3((unsigned)(pq.n_mblocks * p.b * p.h)), dim3(256), stream, pq);
  return hipGetLastError();
}

template <typename T>
hipError_t launch_bwd_t(const Params &p, hipStream_t stream) {
  switch (p.d) {
  case 32: return launch_bwd_td<T, 32>(p, stream);
  case 64: return launch_bwd_td<T, 64>(p, stream);
  case 128: return launch_bwd_td<T, 128>(p, stream);
  default: return hipErrorInvalidValue;
  }
}

hipError_t launch_group_sum(const Params &p, const GroupSplit &s, int row, int dtype, hipStream_t stream) {
  const int64_t chunks = (int64_t)p.b * p.sk * p.h_k * (row / 8);
  hipError_t e = hipSuccess;
  if (chunks > 0) {
    const dim3 grid((unsigned)((chunks + 255) / 256)), block(256);
    if (dtype == 1) FA_LAUNCH((group_sum_kernel<_Float16>), grid, block, stream, p, s.dk, s.dv, s.gs * s.qs, row);
    else FA_LAUNCH((group_sum_kernel<__bf16>), grid, block, stream, p, s.dk, s.dv, s.gs * s.qs, row);
    e = hipGetLastError();
  }
  if (s.owned) {
    const hipError_t f = hipFreeAsync(s.owned, stream);
    if (e == hipSuccess) e = f;
  }
  return e;
}

hipError_t launch_bwd(Params &p, int dtype, hipStream_t stream) {
  p.n_mblocks = (p.sq + kQBlock - 1) / kQBlock;
  p.n_nblocks = (p.sk + kKvBlock - 1) / kKvBlock;
  p.xcd_remap = idx::block_order_mode(p.b * p.h, p.wr);
  if (p.b * p.h == 0) return hipSuccess;
  // The tuned kernels address Q / dO / K / V tiles with 32-bit offsets inside a (batch, head)
  // slice (buffer loads), including a few tiles of look-ahead past the end: larger slices
  // take the generic kernels.
  const int64_t max_rs = std::max(std::max(p.q_rs, p.o_rs), std::max(p.k_rs, p.v_rs));
  const int64_t span = idx::bwd_stream_span_bytes(std::max(p.sq, p.sk), max_rs);
  if (p.drop || (p.d != 32 && p.d != 64 && p.d != 128) || span >= (int64_t(1) << 31)) return launch_bwd_anyd(p, dtype, stream);
  return dtype == 1 ? launch_bwd_t<_Float16>(p, stream) : launch_bwd_t<__bf16>(p, stream);
}

}  // namespace fa
