// Flash-attention forward for gfx950: O = softmax(scale * Q K^T + mask) V, LSE = ln sum exp.
//
// One workgroup (4 waves) owns 128 query rows of one (batch, head); each wave owns 32 of
// them for the whole kernel.  K/V are streamed in 64-row tiles through LDS.  Per tile a wave
// computes S^T = K Q^T (keys on rows, queries on columns, so every softmax statistic is
// lane-local), does the online-softmax update in registers, rounds P^T to the storage type
// and feeds it straight back as the B operand of O^T += V^T P^T; V^T comes out of the
// row-major LDS tile through the transposing LDS read.  The next tile's global loads are
// issued before the math of the current one.
//
// Arithmetic follows the reference kernel (external_libs/runtime/flash_attn/lib/
// flash_fwd_kernel.h:276-469, softmax.h:128-178): fp32 accumulation, exp2 with
// scale*log2(e) folded in, unrounded row sums, P rounded to the storage type before P V,
// O divided by the row sum at the end, LSE = max*scale + ln(sum); a row that keeps no key
// gives O = 0 and LSE = +inf.
#include "flash_common.h"

namespace fa {

constexpr int kBM = 128;  // query rows per workgroup
constexpr int kBN = 64;   // key rows per tile

template <typename T, int D>
__global__ void __launch_bounds__(256, 2) flash_fwd_kernel(const Params p) {
  using vec8 = typename Traits<T>::vec8;
  constexpr int KS = Pad<D>::kPlain;  // K tile row stride
  constexpr int VS = Pad<D>::kTr;     // V tile row stride
  __shared__ __attribute__((aligned(16))) T Ks[kBN * KS];
  __shared__ __attribute__((aligned(16))) T Vs[kBN * VS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, g = lane >> 5;

  int m_block, bh;
  {
    const int L = blockIdx.x;
    if (p.xcd_remap) {  // consecutive workgroup ids go round-robin over the 8 XCDs
      const int xcd = L & 7, slot = L >> 3;
      bh = (slot / p.n_mblocks) * 8 + xcd;
      m_block = slot % p.n_mblocks;
    } else {
      bh = L / p.n_mblocks;
      m_block = L % p.n_mblocks;
    }
    m_block = p.n_mblocks - 1 - m_block;  // longest (causal) blocks first
  }
  const int bi = bh / p.h, hi = bh % p.h, hk = hi / (p.h / p.h_k);
  const int m0 = m_block * kBM;
  const int wq0 = m0 + wave * 32;
  const int qrow = wq0 + r32;

  int lo_lim, hi_lim;
  row_limits(p, qrow, lo_lim, hi_lim);
  // limits of the wave's first and last row bound what the wave can see
  int w_lo_first, w_hi_first, w_lo_last, w_hi_last;
  row_limits(p, wq0, w_lo_first, w_hi_first);
  row_limits(p, wq0 + 31, w_lo_last, w_hi_last);
  // tile range of the workgroup
  int b_lo, b_hi, t0, t1;
  row_limits(p, m0, b_lo, t0);
  row_limits(p, m0 + kBM - 1, t1, b_hi);
  const int n_min = b_lo / kBN;
  const int n_max = b_hi > 0 ? (b_hi + kBN - 1) / kBN : 0;

  const T *qg = static_cast<const T *>(p.q) + bi * p.q_bs + (int64_t)qrow * p.q_rs + hi * p.q_hs;
  const T *kg = static_cast<const T *>(p.k) + bi * p.k_bs + hk * p.k_hs;
  const T *vg = static_cast<const T *>(p.v) + bi * p.v_bs + hk * p.v_hs;

  vec8 qf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    if (qrow < p.sq) qf[ks] = *reinterpret_cast<const vec8 *>(qg + ks * 16 + g * 8);
    else qf[ks] = vec8{0};
  }

  constexpr int CPR = D / 8;       // 16-byte chunks per tile row
  constexpr int RPP = 256 / CPR;   // rows covered by one pass of the workgroup
  constexpr int NP = kBN / RPP;    // passes per tile
  const int ld_c = tid % CPR, ld_r = tid / CPR;
  uint4 kreg[NP], vreg[NP];
  auto gload = [&](int t) {
#pragma unroll
    for (int s = 0; s < NP; ++s) {
      const int kv = t * kBN + s * RPP + ld_r;
      if (kv < p.sk) {
        kreg[s] = *reinterpret_cast<const uint4 *>(kg + (int64_t)kv * p.k_rs + ld_c * 8);
        vreg[s] = *reinterpret_cast<const uint4 *>(vg + (int64_t)kv * p.v_rs + ld_c * 8);
      } else {  // zero rows: 0 * finite stays finite in P V
        kreg[s] = uint4{0, 0, 0, 0};
        vreg[s] = uint4{0, 0, 0, 0};
      }
    }
  };
  auto lstore = [&]() {
#pragma unroll
    for (int s = 0; s < NP; ++s) {
      const int row = s * RPP + ld_r;
      *reinterpret_cast<uint4 *>(&Ks[row * KS + ld_c * 8]) = kreg[s];
      *reinterpret_cast<uint4 *>(&Vs[row * VS + ld_c * 8]) = vreg[s];
    }
  };

  float16v o_acc[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) o_acc[i] = float16v{0};
  float m_run = -INFINITY, l_run = 0.f;
  const float c = p.scale_log2;

  if (n_min < n_max) {
    gload(n_min);
    lstore();
    __syncthreads();
  }
  for (int t = n_min; t < n_max; ++t) {
    const int kv0 = t * kBN;
    if (t + 1 < n_max) gload(t + 1);
    // the wave sees nothing of this tile when it lies wholly outside the widest row window
    const bool skip = kv0 >= w_hi_last || kv0 + kBN <= w_lo_first;
    if (!skip) {
      float16v s[2];
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb) {
        s[kvb] = float16v{0};
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) {
          const vec8 a = lds_read8<T>(&Ks[(kvb * 32 + r32) * KS + ks * 16 + g * 8]);
          s[kvb] = Traits<T>::mfma(a, qf[ks], s[kvb]);
        }
      }
      const bool need_mask = kv0 + kBN > w_hi_first || kv0 < w_lo_last;
      if (need_mask) {
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
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
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
        for (int db = 0; db < D / 32; ++db) {
          const vec8 a = lds_read_operand_tr<T>(Vs, VS, w * 16, db * 32);
          o_acc[db] = Traits<T>::mfma(a, pb, o_acc[db]);
        }
      }
    }
    __syncthreads();  // every wave is done with the tile in LDS
    if (t + 1 < n_max) lstore();
    __syncthreads();
  }

  // epilogue: normalise, write O and LSE
  const float l_tot = l_run + partner32(l_run);
  const bool empty = l_tot == 0.f || l_tot != l_tot;
  const float inv = empty ? 1.f : 1.f / l_tot;
  if (qrow < p.sq) {
    T *og = static_cast<T *>(p.o_w) + bi * p.o_bs + (int64_t)qrow * p.o_rs + hi * p.o_hs;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        typedef T vec4 __attribute__((ext_vector_type(4)));
        vec4 v;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = (T)(o_acc[db][i4 * 4 + j] * inv);
        *reinterpret_cast<vec4 *>(og + db * 32 + i4 * 8 + g * 4) = v;
      }
    if (g == 0)
      p.lse[((int64_t)bi * p.h + hi) * p.sq + qrow] =
          empty ? INFINITY : m_run * p.scale + log2_fast(l_tot) * kLn2;
  }
}

template <typename T>
hipError_t launch_fwd_t(const Params &p, hipStream_t stream) {
  const dim3 grid((unsigned)(p.n_mblocks * p.b * p.h)), block(256);
  switch (p.d) {
  case 32: flash_fwd_kernel<T, 32><<<grid, block, 0, stream>>>(p); break;
  case 64: flash_fwd_kernel<T, 64><<<grid, block, 0, stream>>>(p); break;
  case 128: flash_fwd_kernel<T, 128><<<grid, block, 0, stream>>>(p); break;
  default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_fwd(Params &p, int dtype, hipStream_t stream) {
  p.n_mblocks = (p.sq + kBM - 1) / kBM;
  p.xcd_remap = ((p.b * p.h) % 8 == 0) ? 1 : 0;
  if (p.n_mblocks == 0 || p.b * p.h == 0) return hipSuccess;
  return dtype == 1 ? launch_fwd_t<_Float16>(p, stream) : launch_fwd_t<__bf16>(p, stream);
}

}  // namespace fa
