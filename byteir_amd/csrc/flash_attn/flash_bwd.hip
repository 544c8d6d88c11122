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

// copies a [ROWS x D] tile (rows row0.. of a [n_rows, D] strided matrix) into registers
template <typename T, int D, int ROWS>
struct TileLoader {
  static constexpr int CPR = D / 8;
  static constexpr int RPP = 256 / CPR;
  static constexpr int NP = ROWS / RPP;
  uint4 reg[NP];
  __device__ __forceinline__ void gload(const T *base, int64_t row_stride, int row0, int n_rows) {
    const int c = threadIdx.x % CPR, r = threadIdx.x / CPR;
#pragma unroll
    for (int s = 0; s < NP; ++s) {
      const int row = row0 + s * RPP + r;
      if (row < n_rows) reg[s] = *reinterpret_cast<const uint4 *>(base + (int64_t)row * row_stride + c * 8);
      else reg[s] = uint4{0, 0, 0, 0};
    }
  }
  __device__ __forceinline__ void lstore(T *tile, int stride) const {
    const int c = threadIdx.x % CPR, r = threadIdx.x / CPR;
#pragma unroll
    for (int s = 0; s < NP; ++s)
      *reinterpret_cast<uint4 *>(&tile[(s * RPP + r) * stride + c * 8]) = reg[s];
  }
};

// ---- 2. dK, dV ------------------------------------------------------------------------------
template <typename T, int D>
__global__ void __launch_bounds__(256) dkdv_kernel(const Params p) {
  using vec8 = typename Traits<T>::vec8;
  constexpr int QS = D + 16;  // tiles are read both plainly and transposed
  __shared__ __attribute__((aligned(16))) T Qs[kQTile * QS];
  __shared__ __attribute__((aligned(16))) T dOs[kQTile * QS];
  __shared__ float lse_s[kQTile];
  __shared__ float dsm_s[kQTile];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, g = lane >> 5;
  int n_block, bh;
  {
    const int L = blockIdx.x;
    if (p.xcd_remap) {
      const int xcd = L & 7, slot = L >> 3;
      bh = (slot / p.n_nblocks) * 8 + xcd;
      n_block = slot % p.n_nblocks;
    } else {
      bh = L / p.n_nblocks;
      n_block = L % p.n_nblocks;
    }
  }
  const int bi = bh / p.h, hi = bh % p.h;
  const int kvb0 = n_block * kKvBlock;
  const int kvcol = kvb0 + wave * 32 + r32;  // the key this lane owns
  const int off = p.sk - p.sq;

  const T *qg = static_cast<const T *>(p.q) + bi * p.q_bs + hi * p.q_hs;
  const T *dog = static_cast<const T *>(p.dout) + bi * p.o_bs + hi * p.o_hs;
  const T *kg = static_cast<const T *>(p.k) + bi * p.k_bs + (int64_t)kvcol * p.k_rs + hi * p.k_hs;
  const T *vg = static_cast<const T *>(p.v) + bi * p.v_bs + (int64_t)kvcol * p.v_rs + hi * p.v_hs;
  const float *lse_g = p.lse + ((int64_t)bi * p.h + hi) * p.sq;
  const float *dsm_g = p.dsoftmax + ((int64_t)bi * p.h + hi) * p.sq_rounded;

  vec8 kf[D / 16], vf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    if (kvcol < p.sk) {
      kf[ks] = *reinterpret_cast<const vec8 *>(kg + ks * 16 + g * 8);
      vf[ks] = *reinterpret_cast<const vec8 *>(vg + ks * 16 + g * 8);
    } else {
      kf[ks] = vec8{0};
      vf[ks] = vec8{0};
    }
  }
  float16v dk_acc[D / 32], dv_acc[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) { dk_acc[i] = float16v{0}; dv_acc[i] = float16v{0}; }

  // query tiles that can see keys [kvb0, kvb0 + 128)
  int q_lo = 0, q_hi = p.sq;
  if (p.wr >= 0) q_lo = max(0, kvb0 - off - p.wr);                 // hi(q) = q+1+off+wr > kvb0
  if (p.wl >= 0) q_hi = min(p.sq, kvb0 + kKvBlock - off + p.wl);   // lo(q) = q+off-wl < kvb0+128
  const int m_min = q_lo / kQTile;
  const int m_max = q_hi > 0 ? (q_hi + kQTile - 1) / kQTile : 0;
  const float c = p.scale_log2;

  TileLoader<T, D, kQTile> lq, ldo;
  float lse_r = 0.f, dsm_r = 0.f;
  auto gload = [&](int m) {
    lq.gload(qg, p.q_rs, m * kQTile, p.sq);
    ldo.gload(dog, p.o_rs, m * kQTile, p.sq);
    if (tid < kQTile) {
      const int q = m * kQTile + tid;
      lse_r = q < p.sq ? lse_g[q] : INFINITY;  // +inf: the row contributes P = 0
      dsm_r = q < p.sq ? dsm_g[q] : 0.f;
    }
  };
  auto lstore = [&]() {
    lq.lstore(Qs, QS);
    ldo.lstore(dOs, QS);
    if (tid < kQTile) { lse_s[tid] = lse_r * kLog2e; dsm_s[tid] = dsm_r; }
  };

  if (m_min < m_max) {
    gload(m_min);
    lstore();
    __syncthreads();
  }
  for (int m = m_min; m < m_max; ++m) {
    if (m + 1 < m_max) gload(m + 1);
#pragma unroll
    for (int qs = 0; qs < kQTile / 32; ++qs) {
      const int q0 = m * kQTile + qs * 32;  // first query row of this 32-row sub-tile
      // wave-uniform visibility of the sub-tile against the wave's 32 keys
      const int wkv0 = kvb0 + wave * 32;
      int lo_first, hi_first, lo_last, hi_last;
      row_limits(p, q0, lo_first, hi_first);
      row_limits(p, q0 + 31, lo_last, hi_last);
      if (wkv0 >= hi_last || wkv0 + 32 <= lo_first) continue;  // nothing kept
      const bool need_mask = wkv0 + 32 > hi_first || wkv0 < lo_last || q0 + 32 > p.sq;

      float16v s = float16v{0}, dp = float16v{0};
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks) {
        const vec8 aq = lds_read8<T>(&Qs[(qs * 32 + r32) * QS + ks * 16 + g * 8]);
        s = Traits<T>::mfma(aq, kf[ks], s);
        const vec8 ad = lds_read8<T>(&dOs[(qs * 32 + r32) * QS + ks * 16 + g * 8]);
        dp = Traits<T>::mfma(ad, vf[ks], dp);
      }
      float pv[16], dsv[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int ql = qs * 32 + (i >> 2) * 8 + g * 4 + (i & 3);  // row inside the LDS tile
        float pe = exp2_fast(fmaf(s[i], c, -lse_s[ql]));
        if (need_mask) {
          int lo, hi_;
          row_limits(p, m * kQTile + ql, lo, hi_);
          if (kvcol >= hi_ || kvcol < lo) pe = 0.f;
        }
        pv[i] = pe;
        dsv[i] = pe * (dp[i] - dsm_s[ql]);
      }
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const vec8 pb = pack8<T>(&pv[w * 8]);
        const vec8 dsb = pack8<T>(&dsv[w * 8]);
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          const vec8 a_do = lds_read_operand_tr<T>(dOs, QS, qs * 32 + w * 16, db * 32);
          dv_acc[db] = Traits<T>::mfma(a_do, pb, dv_acc[db]);
          const vec8 a_q = lds_read_operand_tr<T>(Qs, QS, qs * 32 + w * 16, db * 32);
          dk_acc[db] = Traits<T>::mfma(a_q, dsb, dk_acc[db]);
        }
      }
    }
    __syncthreads();
    if (m + 1 < m_max) lstore();
    __syncthreads();
  }

  if (kvcol < p.sk) {
    T *dkg = static_cast<T *>(p.dk) + bi * p.k_bs + (int64_t)kvcol * p.k_rs + hi * p.k_hs;
    T *dvg = static_cast<T *>(p.dv) + bi * p.v_bs + (int64_t)kvcol * p.v_rs + hi * p.v_hs;
    typedef T vec4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        vec4 a, b;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          a[j] = (T)(dk_acc[db][i4 * 4 + j] * p.scale);
          b[j] = (T)(dv_acc[db][i4 * 4 + j]);
        }
        *reinterpret_cast<vec4 *>(dkg + db * 32 + i4 * 8 + g * 4) = a;
        *reinterpret_cast<vec4 *>(dvg + db * 32 + i4 * 8 + g * 4) = b;
      }
  }
}

// ---- 3. dQ ----------------------------------------------------------------------------------
template <typename T, int D>
__global__ void __launch_bounds__(256) dq_kernel(const Params p) {
  using vec8 = typename Traits<T>::vec8;
  constexpr int KS = D + 16;          // K tile: plain and transposed reads
  constexpr int VS = Pad<D>::kPlain;  // V tile: plain reads only
  __shared__ __attribute__((aligned(16))) T Ks[kKvTile * KS];
  __shared__ __attribute__((aligned(16))) T Vs[kKvTile * VS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, g = lane >> 5;
  int m_block, bh;
  {
    const int L = blockIdx.x;
    if (p.xcd_remap) {
      const int xcd = L & 7, slot = L >> 3;
      bh = (slot / p.n_mblocks) * 8 + xcd;
      m_block = slot % p.n_mblocks;
    } else {
      bh = L / p.n_mblocks;
      m_block = L % p.n_mblocks;
    }
    m_block = p.n_mblocks - 1 - m_block;
  }
  const int bi = bh / p.h, hi = bh % p.h;
  const int m0 = m_block * kQBlock;
  const int wq0 = m0 + wave * 32;
  const int qrow = wq0 + r32;

  int lo_lim, hi_lim, w_lo_first, w_hi_first, w_lo_last, w_hi_last, b_lo, b_hi, t0, t1;
  row_limits(p, qrow, lo_lim, hi_lim);
  row_limits(p, wq0, w_lo_first, w_hi_first);
  row_limits(p, wq0 + 31, w_lo_last, w_hi_last);
  row_limits(p, m0, b_lo, t0);
  row_limits(p, m0 + kQBlock - 1, t1, b_hi);
  const int n_min = b_lo / kKvTile;
  const int n_max = b_hi > 0 ? (b_hi + kKvTile - 1) / kKvTile : 0;

  const T *qg = static_cast<const T *>(p.q) + bi * p.q_bs + (int64_t)qrow * p.q_rs + hi * p.q_hs;
  const T *dog = static_cast<const T *>(p.dout) + bi * p.o_bs + (int64_t)qrow * p.o_rs + hi * p.o_hs;
  const T *kg = static_cast<const T *>(p.k) + bi * p.k_bs + hi * p.k_hs;
  const T *vg = static_cast<const T *>(p.v) + bi * p.v_bs + hi * p.v_hs;

  vec8 qf[D / 16], dof[D / 16];
  float lse_l = INFINITY, dsm_l = 0.f;
  if (qrow < p.sq) {
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
  float16v dq_acc[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i) dq_acc[i] = float16v{0};
  const float c = p.scale_log2;

  TileLoader<T, D, kKvTile> lk, lv;
  if (n_min < n_max) {
    lk.gload(kg, p.k_rs, n_min * kKvTile, p.sk);
    lv.gload(vg, p.v_rs, n_min * kKvTile, p.sk);
    lk.lstore(Ks, KS);
    lv.lstore(Vs, VS);
    __syncthreads();
  }
  for (int t = n_min; t < n_max; ++t) {
    const int kv0 = t * kKvTile;
    if (t + 1 < n_max) {
      lk.gload(kg, p.k_rs, (t + 1) * kKvTile, p.sk);
      lv.gload(vg, p.v_rs, (t + 1) * kKvTile, p.sk);
    }
    const bool skip = kv0 >= w_hi_last || kv0 + kKvTile <= w_lo_first;
    if (!skip) {
      const bool need_mask = kv0 + kKvTile > w_hi_first || kv0 < w_lo_last;
      float16v s[2], dp[2];
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb) {
        s[kvb] = float16v{0};
        dp[kvb] = float16v{0};
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) {
          const vec8 ak = lds_read8<T>(&Ks[(kvb * 32 + r32) * KS + ks * 16 + g * 8]);
          s[kvb] = Traits<T>::mfma(ak, qf[ks], s[kvb]);
          const vec8 av = lds_read8<T>(&Vs[(kvb * 32 + r32) * VS + ks * 16 + g * 8]);
          dp[kvb] = Traits<T>::mfma(av, dof[ks], dp[kvb]);
        }
      }
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float pe = exp2_fast(fmaf(s[kvb][i], c, -lse_l));
          if (need_mask) {
            const int kv = kv0 + kvb * 32 + (i >> 2) * 8 + g * 4 + (i & 3);
            if (kv >= hi_lim || kv < lo_lim) pe = 0.f;
          }
          s[kvb][i] = pe * (dp[kvb][i] - dsm_l);  // dS^T
        }
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float f[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] = s[w >> 1][(w & 1) * 8 + j];
        const vec8 dsb = pack8<T>(f);
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          const vec8 a = lds_read_operand_tr<T>(Ks, KS, w * 16, db * 32);
          dq_acc[db] = Traits<T>::mfma(a, dsb, dq_acc[db]);
        }
      }
    }
    __syncthreads();
    if (t + 1 < n_max) { lk.lstore(Ks, KS); lv.lstore(Vs, VS); }
    __syncthreads();
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

template <typename T, int D>
hipError_t launch_bwd_td(const Params &p, hipStream_t stream) {
  const int64_t rows = (int64_t)p.b * p.h * p.sq;
  if (rows > 0) {
    constexpr int RPB = 256 / (D / 8);
    dot_do_o_kernel<T, D><<<dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, stream>>>(p);
  }
  if (p.n_nblocks > 0)
    dkdv_kernel<T, D><<<dim3((unsigned)(p.n_nblocks * p.b * p.h)), dim3(256), 0, stream>>>(p);
  if (p.n_mblocks > 0)
    dq_kernel<T, D><<<dim3((unsigned)(p.n_mblocks * p.b * p.h)), dim3(256), 0, stream>>>(p);
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

hipError_t launch_bwd(Params &p, int dtype, hipStream_t stream) {
  p.n_mblocks = (p.sq + kQBlock - 1) / kQBlock;
  p.n_nblocks = (p.sk + kKvBlock - 1) / kKvBlock;
  p.xcd_remap = ((p.b * p.h) % 8 == 0) ? 1 : 0;
  if (p.b * p.h == 0) return hipSuccess;
  return dtype == 1 ? launch_bwd_t<_Float16>(p, stream) : launch_bwd_t<__bf16>(p, stream);
}

}  // namespace fa
