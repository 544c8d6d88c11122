// Flash-attention forward for gfx950: O = softmax(scale * Q K^T + mask) V, LSE = ln sum exp.
//
// One workgroup (8 waves, one per CU, two waves per SIMD) owns 256 query rows of one (batch,
// head); each wave owns 32 of them for the whole kernel.  K/V are streamed in 64-row tiles
// through a three-deep LDS ring with one barrier per tile.  Per unit of 32 keys a wave computes
// S^T = K Q^T (keys on rows, queries on columns, so every softmax statistic is lane-local),
// does the online-softmax update in registers, rounds P^T to the storage type and feeds it
// straight back as the B operand of O^T += V^T P^T; V^T comes out of the row-major LDS tile
// through the transposing LDS read.  Measured limiter: LDS read bandwidth (every wave reads the
// whole K and V unit, 16 KiB per 16 MFMAs), not the exponentials and not LDS latency.
//
// The key dimension is consumed in units of 32 keys and the loop is software pipelined inside
// each wave: S^T of unit u+1 is produced (MFMA) in the same basic block in which unit u goes
// through exp/max/convert (VALU) and O^T += V^T P^T, so the vector work of the softmax runs in
// the shadow of matrix instructions.  The ring is three deep: tile t is read by everyone,
// K of tile t+1 is read by the look-ahead, and tile t+2 is being written.
//
// Arithmetic follows the reference kernel (external_libs/runtime/flash_attn/lib/
// flash_fwd_kernel.h:276-469, softmax.h:128-178): fp32 accumulation, exp2 with
// scale*log2(e) folded in, unrounded row sums, P rounded to the storage type before P V,
// O divided by the row sum at the end, LSE = max*scale + ln(sum); a row that keeps no key
// gives O = 0 and LSE = +inf.  One deviation: the running maximum is only raised when it
// would grow by more than kRescaleSlack (in log2 units), or from -inf; exp2 then stays below
// 2^kRescaleSlack, the identities O = acc / sum and LSE = max*scale + ln(sum) hold for any
// reference maximum, and the accumulator rescale (D/2 multiplies per lane per tile) rarely runs.
#include <algorithm>
#include <cmath>

#include "flash_common.h"

namespace fa {

constexpr int kBN = 64;        // key rows per tile
constexpr int kStages = 3;     // LDS ring depth
constexpr float kRescaleSlack = 8.0f;

// QB: 32-row halves per wave (1 or 2); NW: waves per workgroup; the workgroup owns 32*QB*NW rows
// VarK: the number of keys is read per batch (key/value cache calls): seqlens_k[b] + seqlen_knew
template <typename T, int D, int QB, int NW, bool VarK>
__global__ void __launch_bounds__(NW * 64, NW * QB >= 16 ? 2 : (QB == 2 ? 1 : 2)) flash_fwd_kernel(const Params p) {
  constexpr int kThreads = NW * 64;
  constexpr int kBM = 32 * QB * NW;
  using vec8 = typename Traits<T>::vec8;
  constexpr int KS = Pad<D>::kPlain;  // K tile row stride
  constexpr int VS = Pad<D>::kTr;     // V tile row stride
  __shared__ __attribute__((aligned(16))) T Ks[kStages][kBN * KS];
  __shared__ __attribute__((aligned(16))) T Vs[kStages][kBN * VS];

  // The wave index is deliberately left in a vector register: with a scalar one the compiler
  // turns the per-wave skip tests of the pipelined loop into real branches, which splits the
  // block in which MFMA and softmax instructions interleave (measured 20-40 % slower).
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, g = lane >> 5;

  // Block order (idx::decode_block): consecutive workgroup ids go round-robin over the 8 XCDs and
  // the blocks of a (batch, head) share one, so that its K/V are fetched into a single L2; with
  // blocks of unequal length (a right window) the longest block of every (batch, head) comes
  // first within an XCD, then the second longest of every one, ...: longest-first list
  // scheduling, which fills the CUs evenly over the causal triangle (measured 216 -> 178 us on
  // fp16 causal b4 h32 s2048 d128) at the price of more (batch, head) pairs in flight per L2.
  const idx::BlockId blk = idx::decode_block((int)blockIdx.x, p.xcd_remap, p.b * p.h, p.n_mblocks);
  const int bh = blk.bh, m_block = p.n_mblocks - 1 - blk.blk;  // longest (causal) blocks first
  const int bi = bh / p.h, hi = bh % p.h, hk = hi / (p.h / p.h_k);
  int sk = p.sk;
  if constexpr (VarK) sk = min(p.sk, p.seqlens_k[bi] + p.seqlen_knew);
  const int m0 = m_block * kBM;
  const int wq0 = m0 + wave * 32 * QB;

  int qrow[QB], lo_lim[QB], hi_lim[QB];
  // limits of each half's first and last row bound what the half can see
  int h_lo_first[QB], h_hi_first[QB], h_lo_last[QB], h_hi_last[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    qrow[qb] = wq0 + qb * 32 + r32;
    row_limits_sk(p, sk, qrow[qb], lo_lim[qb], hi_lim[qb]);
    row_limits_sk(p, sk, wq0 + qb * 32, h_lo_first[qb], h_hi_first[qb]);
    row_limits_sk(p, sk, wq0 + qb * 32 + 31, h_lo_last[qb], h_hi_last[qb]);
  }
  const int w_lo_first = h_lo_first[0], w_hi_last = h_hi_last[QB - 1];  // the wave's widest window
  // tile range of the workgroup
  int n_min, n_max;
  idx::key_tile_range(p.sq, sk, p.wl, p.wr, m0, kBM, kBN, n_min, n_max);
  const int split = blockIdx.y;  // key axis split over workgroups: this one's share of the tiles
  if (p.n_splits > 1) {
    n_min = max(n_min, split * p.split_tiles);
    n_max = min(n_max, (split + 1) * p.split_tiles);
  }

  const T *kg = static_cast<const T *>(p.k) + bi * p.k_bs + hk * p.k_hs;
  const T *vg = static_cast<const T *>(p.v) + bi * p.v_bs + hk * p.v_hs;

  vec8 qf[QB][D / 16];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const T *qg = static_cast<const T *>(p.q) + bi * p.q_bs + (int64_t)qrow[qb] * p.q_rs + hi * p.q_hs;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      if (qrow[qb] < p.sq) qf[qb][ks] = *reinterpret_cast<const vec8 *>(qg + ks * 16 + g * 8);
      else qf[qb][ks] = vec8{0};
    }
  }
  // Consume the Q fragments once here: the wait for their global loads is then placed before
  // the loop instead of in front of the first MFMA of every iteration, where it would also
  // drain the K/V prefetch that has just been issued.
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) FA_PIN(qf[qb][ks]);

  constexpr int CPR = D / 8;                       // 16-byte chunks per tile row
  constexpr int RPP = kThreads / CPR;              // rows covered by one pass of the workgroup
  constexpr int NP = RPP >= kBN ? 1 : kBN / RPP;   // passes per tile
  const int ld_c = tid % CPR, ld_r = tid / CPR;
  const bool ld_on = RPP <= kBN || ld_r < kBN;     // narrow heads: surplus threads stay idle
  uint4 kreg[NP], vreg[NP];
  // Buffer loads: the descriptors cover this head's rows [0, sk), so rows beyond the last key
  // read as zeros without an address check (0 * finite stays finite in P V).  The tile offset
  // is added to the per-thread offset (the vector offset is what the hardware checks against
  // the descriptor's size); launch_fwd keeps head slices below 2 GiB so the sum cannot wrap.
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  constexpr unsigned kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format
  const unsigned k_bytes = idx::rsrc_bytes(sk, p.k_rs, D), v_bytes = idx::rsrc_bytes(sk, p.v_rs, D);
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(kg), 0, k_bytes, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(vg), 0, v_bytes, kRsrcFlags);
  unsigned k_vo[NP], v_vo[NP];
#pragma unroll
  for (int s = 0; s < NP; ++s) {  // surplus threads of a narrow head point beyond the buffer
    k_vo[s] = ld_on ? idx::chunk_offset(ld_r + s * RPP, ld_c, p.k_rs) : 0xffffffffu;
    v_vo[s] = ld_on ? idx::chunk_offset(ld_r + s * RPP, ld_c, p.v_rs) : 0xffffffffu;
  }
  const unsigned k_tile_b = idx::tile_bytes(kBN, p.k_rs), v_tile_b = idx::tile_bytes(kBN, p.v_rs);
  unsigned k_so = (unsigned)n_min * k_tile_b, v_so = (unsigned)n_min * v_tile_b;  // byte offset of the next tile to fetch
  auto gload = [&]() {
#pragma unroll
    for (int s = 0; s < NP; ++s) {
      const u32x4 a = __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, ld_on ? k_vo[s] + k_so : 0xffffffffu, 0, 0);
      const u32x4 b = __builtin_amdgcn_raw_buffer_load_b128(v_rsrc, ld_on ? v_vo[s] + v_so : 0xffffffffu, 0, 0);
      kreg[s] = uint4{a.x, a.y, a.z, a.w};
      vreg[s] = uint4{b.x, b.y, b.z, b.w};
    }
    k_so += k_tile_b; v_so += v_tile_b;
  };
  const int st_off_k = ld_r * KS + ld_c * 8, st_off_v = ld_r * VS + ld_c * 8;
  auto lstore = [&](int buf) {
#pragma unroll
    for (int s = 0; s < NP; ++s) {
      if (ld_on) {
        *reinterpret_cast<uint4 *>(&Ks[buf][st_off_k + s * RPP * KS]) = kreg[s];
        *reinterpret_cast<uint4 *>(&Vs[buf][st_off_v + s * RPP * VS]) = vreg[s];
      }
    }
  };

  float16v o_acc[QB][D / 32];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int i = 0; i < D / 32; ++i) o_acc[qb][i] = float16v{0};
  float m_run[QB], ms_run[QB], l_run[QB];  // reference maximum, the same times scale*log2e (0 for -inf), row sum
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) { m_run[qb] = -INFINITY; ms_run[qb] = 0.f; l_run[qb] = 0.f; }
  const float c = p.scale_log2;
  const int k_rd = r32 * KS + g * 8;  // this lane's K fragment offset inside a 32-row block

  // The key dimension is consumed in units of 32 keys (half an LDS tile).  The loop is software
  // pipelined inside each wave: the MFMAs of S^T for unit u+1 are independent of the softmax of
  // unit u, so they share a basic block and the exp/max/convert work runs in the MFMA shadow.
  // a wave sees nothing of a unit that lies wholly outside its widest row window
  auto skipped = [&](int kv0) { return kv0 >= w_hi_last || kv0 + 32 <= w_lo_first; };

  struct Unit { float16v s[QB]; };  // S^T of one unit: [half]

  auto qk = [&](const T *Kt, int kvb, Unit &out) {  // S^T (32 keys x 64 queries) = K Q^T
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) out.s[qb] = float16v{0};
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      const vec8 a = lds_read8<T>(&Kt[k_rd + kvb * 32 * KS + ks * 16]);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) out.s[qb] = Traits<T>::mfma(a, qf[qb][ks], out.s[qb]);
    }
  };

  // online softmax of one unit, first part: mask, running maximum, rare accumulator rescale
  auto sm_head = [&](Unit &u, int kv0) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float16v &sc = u.s[qb];
      if (kv0 + 32 > h_hi_first[qb] || kv0 < h_lo_last[qb]) {  // a unit on the edge of the window
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int kv = kv0 + (i >> 2) * 8 + g * 4 + (i & 3);
          if (kv >= hi_lim[qb] || kv < lo_lim[qb]) sc[i] = -INFINITY;
        }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, sc[i]);
      // Raise the reference maximum only when it would grow by more than the slack.  The test
      // is made on this lane's half of the keys first: +inf for the first finite score of a
      // row (m_run = -inf), NaN (false) for -inf - -inf; only when some lane of the wave
      // fires do the two lanes of a row exchange their maxima.
      if (__builtin_amdgcn_ballot_w64((mx - m_run[qb]) * c > kRescaleSlack) != 0) {
        mx = fmaxf(mx, partner32(mx));
        const bool grow = (mx - m_run[qb]) * c > kRescaleSlack;
        const float m_new = grow ? mx : m_run[qb];
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = exp2_fast((m_run[qb] - m_use) * c);
        l_run[qb] *= alpha;
        m_run[qb] = m_new;
        ms_run[qb] = m_use * c;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) o_acc[qb][db][i] *= alpha;
      }
    }
  };

  // exponentials, row sums and P^T of one unit (branch free).  At head_dim 128 the row sum is
  // taken over the rounded P that the P V product uses, two elements per v_dot2c (fp32
  // accumulation), which halves the additions; at head_dim 64 that measured no faster and the
  // sum stays on the unrounded exponentials.
  constexpr bool kDotSum = D >= 128;
  auto sm_exp = [&](Unit &u, vec8 (&pb)[QB][2]) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float16v &sc = u.s[qb];
      const float m_scaled = ms_run[qb];
      float rs = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float e = exp2_fast(fmaf(sc[i], c, -m_scaled));
        sc[i] = e;
        if constexpr (!kDotSum) rs += e;
      }
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        float pf[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) pf[j] = sc[w * 8 + j];
        pb[qb][w] = pack8<T>(pf);
        if constexpr (kDotSum) rs = sum8_acc<T>(pb[qb][w], rs);
      }
      l_run[qb] += rs;
    }
  };

  // O^T += V^T P^T for the unit's two 16-key windows; each V^T fragment serves both halves
  auto pv = [&](const T *Vt, int kvb, const vec8 (&pb)[QB][2]) {
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int db = 0; db < D / 32; ++db) {
        const vec8 a = lds_read_operand_tr<T>(Vt, VS, kvb * 32 + w * 16, db * 32);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) o_acc[qb][db] = Traits<T>::mfma(a, pb[qb][w], o_acc[qb][db]);
      }
  };

  // one pipeline step: finish unit `cur` (softmax, P V) and, in the same basic block, start
  // unit `nxt` (S^T) so that matrix and vector instructions interleave
  auto step = [&](bool do_cur, Unit &cur, int kv0, const T *Vt, int kvb, bool do_nxt, Unit &nxt,
                  const T *Knext, int kvb_next) {
    if (do_cur) sm_head(cur, kv0);
    vec8 pb[QB][2];
    if (do_cur && do_nxt) {
      qk(Knext, kvb_next, nxt);
      sm_exp(cur, pb);
      pv(Vt, kvb, pb);
    } else if (do_cur) {
      sm_exp(cur, pb);
      pv(Vt, kvb, pb);
    } else if (do_nxt) {
      qk(Knext, kvb_next, nxt);
    }
  };

  // prologue: tiles n_min and n_min+1 into the ring, tile n_min+2 into registers
  const int n_tiles = n_max > n_min ? n_max - n_min : 0;
  Unit ua, ub;  // S^T of the unit being consumed / being produced
  if (n_tiles > 0) {
    // All three tiles are requested before the first is stored: one memory latency, not
    // three.  (Tiles beyond the last one read rows that are in bounds or zeros, and stay unused.)
    uint4 k1[NP], v1[NP], k2[NP], v2[NP];
    gload();
#pragma unroll
    for (int s = 0; s < NP; ++s) { k1[s] = kreg[s]; v1[s] = vreg[s]; }
    gload();
#pragma unroll
    for (int s = 0; s < NP; ++s) { k2[s] = kreg[s]; v2[s] = vreg[s]; }
    gload();
#pragma unroll
    for (int s = 0; s < NP; ++s) {  // kreg / vreg: tile n_min + 2, as the loop expects; k1: n_min, k2: n_min + 1
      const uint4 a = kreg[s], b = vreg[s];
      kreg[s] = k1[s]; vreg[s] = v1[s];
      k1[s] = a; v1[s] = b;
    }
    lstore(0);
#pragma unroll
    for (int s = 0; s < NP; ++s) { kreg[s] = k2[s]; vreg[s] = v2[s]; }
    lstore(1);
#pragma unroll
    for (int s = 0; s < NP; ++s) { kreg[s] = k1[s]; vreg[s] = v1[s]; }
    __syncthreads();
    if (!skipped(n_min * kBN)) qk(Ks[0], 0, ua);
  }
  int buf = 0;  // ring slot of tile t
  for (int t = n_min; t < n_max; ++t) {
    const int buf1 = buf + 1 == kStages ? 0 : buf + 1;
    const int buf2 = buf1 + 1 == kStages ? 0 : buf1 + 1;
    const int kv0 = t * kBN;
    // unit 0 of tile t (S in ua) while S of unit 1 is produced into ub
    step(!skipped(kv0), ua, kv0, Vs[buf], 0, !skipped(kv0 + 32), ub, Ks[buf], 1);
    __syncthreads();  // tile t+1 is visible; every wave has left tile t-1
    // tile t+2: registers -> the ring slot tile t-1 occupied; tile t+3 in flight
    if (t + 2 < n_max) lstore(buf2);
    if (t + 3 < n_max) gload();
    // unit 1 of tile t (S in ub) while S of unit 0 of tile t+1 is produced into ua
    step(!skipped(kv0 + 32), ub, kv0 + 32, Vs[buf], 1, t + 1 < n_max && !skipped(kv0 + kBN), ua, Ks[buf1], 0);
    buf = buf1;
  }

  // epilogue: normalise, write O and LSE
  // D = 128, one workgroup per CU: nothing else hides the store latency, so O goes through LDS
  // and leaves as whole rows (measured 3 % on causal b4 h32 s2048); with two workgroups
  // per CU (D <= 64) the direct 8-byte stores are faster (8 % on b2 h16 s8192 d64).
  constexpr bool kStageO = D == 128;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float l_tot = l_run[qb] + partner32(l_run[qb]);
    const bool empty = l_tot == 0.f || l_tot != l_tot;
    const float inv = empty ? 1.f : 1.f / l_tot;
    if (p.n_splits > 1) {  // unnormalised partial, relative to this split's reference maximum
      if (qrow[qb] < p.sq) {
        const int64_t prow = (((int64_t)split * p.b + bi) * p.h + hi) * p.sq + qrow[qb];
        float *og = p.o_part + prow * D;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4)
            *reinterpret_cast<float4 *>(og + db * 32 + i4 * 8 + g * 4) =
                float4{o_acc[qb][db][i4 * 4], o_acc[qb][db][i4 * 4 + 1], o_acc[qb][db][i4 * 4 + 2], o_acc[qb][db][i4 * 4 + 3]};
        if (g == 0) { p.ml_part[prow * 2] = m_run[qb]; p.ml_part[prow * 2 + 1] = l_tot; }
      }
      continue;
    }
    if constexpr (kStageO) {
      // O^T in the accumulators -> the wave's own [32][D] tile in the (now idle) K/V ring ->
      // whole 2*D-byte rows to global memory, 16 bytes per lane
      // The tile is unpadded; the 16-byte chunks of row r are permuted by r >> 1 and odd rows
      // swap the two 8-byte halves of a chunk, which keeps both the 8-byte writes (a lane per
      // row) and the 16-byte reads (16 lanes per row) free of bank conflicts (counter-checked
      // in isolation: a padded tile costs 96 conflict cycles per wave, permuting by r & 15
      // with the halves of rows 16..31 swapped 64, this layout none).
      constexpr int OS = D;
      static_assert(D == 128, "the chunk permutation assumes 16 chunks per row");
      static_assert(!kStageO || (NW / 2 * 32 * OS <= kStages * kBN * KS && NW / 2 * 32 * OS <= kStages * kBN * VS), "O staging must fit the ring");
      if (qb == 0) __syncthreads();  // every wave has left the last K/V tile
      else FA_WAVE_SYNC();           // every lane has read the previous half back
      T *Ot = (wave < NW / 2 ? &Ks[0][0] : &Vs[0][0]) + (wave % (NW / 2)) * 32 * OS;
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          typedef T vec4 __attribute__((ext_vector_type(4)));
          vec4 v;
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = (T)(o_acc[qb][db][i4 * 4 + j] * inv);
          *reinterpret_cast<vec4 *>(&Ot[idx::ostage_write_offset(r32, g, db, i4)]) = v;
        }
      FA_WAVE_SYNC();  // the wave's tile is complete; it is read back across lanes
      constexpr int CPRO = D / 8, RPI = 64 / CPRO;  // 16-byte chunks per row, rows per store instruction
      const int oc = lane % CPRO, orow = lane / CPRO;
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int r = it * RPI + orow, q = wq0 + qb * 32 + r;
        uint4 v = *reinterpret_cast<const uint4 *>(&Ot[idx::ostage_read_offset(r, oc)]);
        if (r & 1) v = uint4{v.z, v.w, v.x, v.y};
        if (q < p.sq)
          *reinterpret_cast<uint4 *>(static_cast<T *>(p.o_w) + bi * p.o_bs + (int64_t)q * p.o_rs + hi * p.o_hs + oc * 8) = v;
      }
    } else if (qrow[qb] < p.sq) {
      T *og = static_cast<T *>(p.o_w) + bi * p.o_bs + (int64_t)qrow[qb] * p.o_rs + hi * p.o_hs;
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          typedef T vec4 __attribute__((ext_vector_type(4)));
          vec4 v;
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = (T)(o_acc[qb][db][i4 * 4 + j] * inv);
          *reinterpret_cast<vec4 *>(og + db * 32 + i4 * 8 + g * 4) = v;
        }
    }
    if (qrow[qb] < p.sq) {
      if (g == 0)
        p.lse[((int64_t)bi * p.h + hi) * p.sq + qrow[qb]] =
            empty ? INFINITY : m_run[qb] * p.scale + log2_fast(l_tot) * kLn2;
    }
  }
}

// Number of key-axis splits for `n_wg` workgroups over `n_tiles` key tiles on 256 CUs: as the
// reference's num_splits_heuristic (flash_api.cu:118-160) -- one split when the chip is already
// 80 % full; otherwise the smallest count whose last round of workgroups is at least 85 % as
// full as the best count's -- with at most 32 splits of at least eight tiles.
inline int pick_splits(int n_wg, int n_tiles) {
  constexpr int kCUs = 256;
  if (n_wg >= 0.8f * kCUs) return 1;
  const int max_splits = std::min(32, n_tiles / 8);
  auto tiles_per = [&](int s) { return (n_tiles + s - 1) / s; };
  auto eligible = [&](int s) { return s == 1 || tiles_per(s) != tiles_per(s - 1); };
  auto eff = [&](int s) {
    const float waves = float(n_wg * s) / kCUs;
    return waves / std::ceil(waves);
  };
  float best = 0.f;
  for (int s = 1; s <= max_splits; ++s)
    if (eligible(s)) best = std::max(best, eff(s));
  for (int s = 1; s <= max_splits; ++s)
    if (eligible(s) && eff(s) >= 0.85f * best) return s;
  return 1;
}

// Geometry: 8 waves of 32 rows, two waves per SIMD.  The kernel is written for 32*QB rows per
// wave; QB = 2 halves the LDS traffic per MFMA, but either needs a whole SIMD per wave
// (head_dim 128: slower, the compiler's schedule leaves the single wave stalled) or brought no
// gain when it fits (head_dim 64), so QB = 1 is what is instantiated.
template <int D> struct FwdGeom { static constexpr int QB = 1, NW = 8; };

template <typename T, int D>
hipError_t launch_fwd_d(Params &p, hipStream_t stream) {
  constexpr int QB = FwdGeom<D>::QB, NW = FwdGeom<D>::NW;
  constexpr int BM = 32 * QB * NW;
  p.n_mblocks = (p.sq + BM - 1) / BM;
  if (p.n_mblocks == 0) return hipSuccess;
  // Few query blocks and many keys (a long prompt chunk of one sequence): split the key axis over
  // workgroups until the chip is full, at least eight tiles per split (the reference's
  // num_splits_heuristic has the same aim, flash_api.cu:118-160, but its entry points never
  // enable it).  The partials live in the caller's workspace or, without one, in a
  // stream-ordered allocation; with neither: one split.
  const int n_wg = p.n_mblocks * p.b * p.h, n_tiles = (p.sk + kBN - 1) / kBN;
  const int n_splits = pick_splits(n_wg, n_tiles);
  void *ws = nullptr;
  bool owned = false;
  const size_t rows = (size_t)p.b * p.h * p.sq;
  const size_t need = n_splits > 1 ? (size_t)n_splits * rows * (D + 2) * sizeof(float) : 0;
  if (p.ws_query) { *p.ws_query = need; return hipSuccess; }
  p.n_splits = 1;
  if (need) {
    if (p.ws && (reinterpret_cast<uintptr_t>(p.ws) & 15) == 0 && p.ws_bytes >= need) ws = p.ws;
    else if (hipMallocAsync(&ws, need, stream) == hipSuccess) owned = true;
    else { (void)hipGetLastError(); ws = nullptr; }  // no scratch: one split
  }
  if (ws) {
    p.n_splits = n_splits;
    p.split_tiles = (n_tiles + n_splits - 1) / n_splits;
    p.o_part = static_cast<float *>(ws);
    p.ml_part = p.o_part + (size_t)n_splits * rows * D;
  }
  const dim3 grid((unsigned)n_wg, (unsigned)p.n_splits), block(NW * 64);
  if (p.seqlens_k) FA_LAUNCH((flash_fwd_kernel<T, D, QB, NW, true>), grid, block, stream, p);
  else FA_LAUNCH((flash_fwd_kernel<T, D, QB, NW, false>), grid, block, stream, p);
  hipError_t e = hipGetLastError();
  if (ws) {
    if (e == hipSuccess) e = launch_split_merge(p, std::is_same<T, _Float16>::value ? 1 : 2, stream);
    if (owned) {
      const hipError_t fr = hipFreeAsync(ws, stream);
      if (e == hipSuccess) e = fr;
    }
  }
  return e;
}

template <typename T>
hipError_t launch_fwd_t(Params &p, hipStream_t stream) {
  switch (p.d) {
  case 32: return launch_fwd_d<T, 32>(p, stream);
  case 64: return launch_fwd_d<T, 64>(p, stream);
  case 128: return launch_fwd_d<T, 128>(p, stream);
  default: return hipErrorInvalidValue;
  }
}

// Appends k_new / v_new [b, seqlen_knew, h_k, d] to the caches at row seqlens_k[b] of each
// batch (reference: the Append_KV branch of compute_attn_1rowblock_splitkv,
// flash_fwd_kernel.h:660-740, without rotary embedding).  One lane copies 16 bytes; rows that
// would fall beyond the cache's p.sk rows are dropped.
template <typename T>
__global__ void __launch_bounds__(256) append_kv_kernel(const Params p) {
  const int cpr = p.d / 8;  // 16-byte chunks per row
  const int64_t total = (int64_t)p.b * p.seqlen_knew * p.h_k * cpr;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int c = (int)(idx % cpr);
  const int hk = (int)((idx / cpr) % p.h_k);
  const int i = (int)((idx / ((int64_t)cpr * p.h_k)) % p.seqlen_knew);
  const int bi = (int)(idx / ((int64_t)cpr * p.h_k * p.seqlen_knew));
  const int row = p.seqlens_k[bi] + i;
  if (row < 0 || row >= p.sk) return;
  const T *ks = static_cast<const T *>(p.k_new) + bi * p.knew_bs + (int64_t)i * p.knew_rs + hk * p.knew_hs + c * 8;
  const T *vs = static_cast<const T *>(p.v_new) + bi * p.vnew_bs + (int64_t)i * p.vnew_rs + hk * p.vnew_hs + c * 8;
  T *kd = const_cast<T *>(static_cast<const T *>(p.k)) + bi * p.k_bs + (int64_t)row * p.k_rs + hk * p.k_hs + c * 8;
  T *vd = const_cast<T *>(static_cast<const T *>(p.v)) + bi * p.v_bs + (int64_t)row * p.v_rs + hk * p.v_hs + c * 8;
  *reinterpret_cast<uint4 *>(kd) = *reinterpret_cast<const uint4 *>(ks);
  *reinterpret_cast<uint4 *>(vd) = *reinterpret_cast<const uint4 *>(vs);
}

hipError_t launch_append_kv(const Params &p, int dtype, hipStream_t stream) {
  const int64_t total = (int64_t)p.b * p.seqlen_knew * p.h_k * (p.d / 8);
  if (total == 0) return hipSuccess;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (dtype == 1) FA_LAUNCH((append_kv_kernel<_Float16>), grid, block, stream, p);
  else FA_LAUNCH((append_kv_kernel<__bf16>), grid, block, stream, p);
  return hipGetLastError();
}

hipError_t launch_fwd(Params &p, int dtype, hipStream_t stream) {
  p.xcd_remap = idx::block_order_mode(p.b * p.h, p.wr);
  if (p.b * p.h == 0 || p.sq == 0) return hipSuccess;
  if (decode_eligible(p)) return launch_decode(p, dtype, stream);
  // the tuned kernel addresses a head's K and V rows through 32-bit buffer offsets
  // (the padded rows of the last tile and the tiles of look-ahead that the prologue always
  // requests are part of the span: their offsets must not wrap either)
  const int64_t kv_span = idx::fwd_stream_span_bytes(p.sk, std::max(p.k_rs, p.v_rs));
  if (p.drop || (p.d != 32 && p.d != 64 && p.d != 128) || kv_span >= (int64_t(1) << 31)) return launch_fwd_anyd(p, dtype, stream);
  return dtype == 1 ? launch_fwd_t<_Float16>(p, stream) : launch_fwd_t<__bf16>(p, stream);
}

}  // namespace fa
