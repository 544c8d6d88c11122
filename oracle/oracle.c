/*
 * oracle.c -- CPU restatement of the reference's arithmetic for the op-kernel hot path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is the checker that the parity
 * tests, the smoke test and the benchmark's "cpu_baseline" leg compare the HIP kernels
 * against.  Nothing in the shipped package may link, import or call it.
 *
 * Every function cites the reference file it follows (paths relative to the reference
 * checkout).  Plain C99, no dependencies beyond libm (OpenMP is used only when the caller
 * raises the thread count with oracle_set_threads; the default is one thread, which is what
 * the reference's CPU path -- single-threaded LLVM-JIT'ed loop nests,
 * runtime/lib/backends/cpu/providers/default/llvm/jit.cc:79-128 -- uses).
 *
 * What pins each function (see tests/test_oracle_*.py):
 *   shape canonicalisation / workspace rule : the reference test's shape list
 *       (runtime/test/backends/cuda/providers/default/kernel/reduction_test.cc:171-180),
 *       brute force by index decode, closed forms for the workspace of the benchmark shapes.
 *   reduce sum / max                         : numpy (pairwise / exact), fp64, NaN cases.
 *   softmax                                  : scipy.special.softmax in fp64, shift
 *       invariance, rows summing to one, one-hot limit.
 *   attention forward O                      : the reference's golden vectors
 *       (runtime/test/test_files/flash_attn_{inputs_*,fwd_outputs}.data) and torch's CPU
 *       scaled_dot_product_attention.
 *   attention forward LSE                    : no reference fixture holds LSE; pinned by
 *       scipy.special.logsumexp and by reconstructing O from LSE.
 *   attention backward dQ,dK,dV              : the reference's golden vectors
 *       (flash_attn_bwd_outputs_{dq,dk,dv}.data), torch autograd through CPU SDPA and a
 *       finite-difference check.
 *   Philox4x32                               : the published known-answer vectors of the
 *       10-round generator (the library's 7-round call differs in the round count only).
 *   attention dropout                        : the arithmetic around the mask by its closed form
 *       on an explicit mask (tests build it element by element with oracle_dropout_keep) and by
 *       finite differences; the keep rate against the 8-bit threshold.  The element-to-random-byte
 *       mapping of oracle_dropout_keep (no reference fixture exercises dropout) is pinned by a
 *       thread-by-thread emulation of the reference's own loop nest, lib/dropout.h:26-84 on the
 *       register fragment of every thread of a block, with the register-to-element map taken
 *       from the reference's mask code (tests/test_oracle_dropout_layout.py, forward and
 *       backward tilings, with negative controls).
 *   extra_args blob                          : byte-level known answer from the reference's
 *       fixture module runtime/test/test_files/flash_attn_fwd.mlir:9.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;
void oracle_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int oracle_get_threads(void) { return g_threads; }

/* ------------------------------------------------------------------------------------ */
/* Counter-based synthetic data, the host side of brt_rocm_fill (include/brt_rocm_kernels.h): */
/* element i = f(seed, i) through splitmix64 (Steele, Lea, Flood 2014; the mixer of           */
/* java.util.SplittableRandom), integer sums and exact float operations.  Pinned by the        */
/* published splitmix64 outputs for seed 1234567 and by moments of the two distributions.      */
/* ------------------------------------------------------------------------------------ */
uint64_t oracle_splitmix64_at(uint64_t seed, uint64_t i) {
  uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
float oracle_h2f(uint16_t h);
uint16_t oracle_f2h(float f);
uint16_t oracle_f2bf(float f);
/* dist 0: uniform [a, b); 1: normal, mean 0, sigma b.  dtype 0 f32, 1 f16, 2 bf16 (RNE).
 * Fills out[0 .. count) with the elements first .. first + count - 1 of the sequence. */
void oracle_fill(int dtype, int dist, uint64_t seed, uint64_t first, uint64_t count, float a, float b, void *out) {
  for (uint64_t k = 0; k < count; ++k) {
    const uint64_t i = first + k;
    volatile float x;  /* every operation rounds to float, no contraction */
    if (dist == 0) {
      const float u = (float)(uint32_t)(oracle_splitmix64_at(seed, i) >> 40) * 0x1p-24f;
      volatile float w = b - a;
      x = fmaf(u, w, a);  /* one rounding, as the device's fused multiply-add */
    } else {
      uint32_t sum = 0;
      for (int j = 0; j < 3; ++j) {
        const uint64_t z = oracle_splitmix64_at(seed, 3 * i + j);
        sum += (uint32_t)(z & 0xffff) + (uint32_t)((z >> 16) & 0xffff) + (uint32_t)((z >> 32) & 0xffff) + (uint32_t)(z >> 48);
      }
      volatile float t = (float)((int32_t)sum - 393210) * 0x1p-16f;
      x = t * b;
    }
    if (dtype == 0) ((float *)out)[k] = x;
    else if (dtype == 1) ((uint16_t *)out)[k] = oracle_f2h(x);
    else ((uint16_t *)out)[k] = oracle_f2bf(x);
  }
}

/* ------------------------------------------------------------------------------------ */
/* 16-bit float storage types (round-to-nearest-even), bit-exact with IEEE binary16 and  */
/* bfloat16.  dtype codes: 0 = f32, 1 = f16, 2 = bf16.                                   */
/* ------------------------------------------------------------------------------------ */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float oracle_h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return u2f(sign);
    /* subnormal: value = man * 2^-24 */
    float v = (float)man * 5.9604644775390625e-08f;
    return sign ? -v : v;
  }
  if (exp == 31) return u2f(sign | 0x7f800000u | (man << 13));
  return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t oracle_f2h(float f) {
  uint32_t x = f2u(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0u));
  }
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* rounds to >= 65520 -> inf */
  if (ax < 0x38800000u) {                                   /* result is subnormal or zero */
    if (ax < 0x33000000u) return (uint16_t)sign;            /* < 2^-25 -> 0 */
    /* value * 2^24 rounded to nearest even integer */
    float v = u2f(ax) * 16777216.0f;
    uint32_t r = (uint32_t)lrintf(v); /* default rounding mode is RNE */
    return (uint16_t)(sign | r);
  }
  uint32_t mant = ax & 0x7fffffu;
  uint32_t e = (ax >> 23) - 112u;
  uint32_t h = (e << 10) | (mant >> 13);
  uint32_t rem = mant & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
  return (uint16_t)(sign | h);
}

float oracle_bf2f(uint16_t b) { return u2f((uint32_t)b << 16); }

uint16_t oracle_f2bf(float f) {
  uint32_t x = f2u(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u); /* quiet nan */
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

static inline float load_elem(const void *p, size_t i, int dtype) {
  switch (dtype) {
  case 0: return ((const float *)p)[i];
  case 1: return oracle_h2f(((const uint16_t *)p)[i]);
  default: return oracle_bf2f(((const uint16_t *)p)[i]);
  }
}
static inline void store_elem(void *p, size_t i, int dtype, float v) {
  switch (dtype) {
  case 0: ((float *)p)[i] = v; break;
  case 1: ((uint16_t *)p)[i] = oracle_f2h(v); break;
  default: ((uint16_t *)p)[i] = oracle_f2bf(v); break;
  }
}
/* round a float to the storage type and back */
static inline float round_storage(float v, int dtype) {
  if (dtype == 1) return oracle_h2f(oracle_f2h(v));
  if (dtype == 2) return oracle_bf2f(oracle_f2bf(v));
  return v;
}

void oracle_convert_from_f32(const float *src, void *dst, size_t n, int dtype) {
  for (size_t i = 0; i < n; ++i) store_elem(dst, i, dtype, src[i]);
}
void oracle_convert_to_f32(const void *src, float *dst, size_t n, int dtype) {
  for (size_t i = 0; i < n; ++i) dst[i] = load_elem(src, i, dtype);
}

/* ------------------------------------------------------------------------------------ */
/* Reductions                                                                            */
/* ------------------------------------------------------------------------------------ */

/* reduction::DeduceOutputShape, runtime/lib/core/common/utils/math_helper.cc:145-159.
 * Returns the output rank, or -1 when a dimension is out of range. */
int oracle_deduce_output_shape(const int64_t *shape, int rank, const int64_t *dims, int ndims,
                               int64_t *out_shape) {
  int mask[64] = {0};
  if (rank > 64) return -1;
  for (int i = 0; i < ndims; ++i) {
    if (dims[i] < 0 || dims[i] >= rank) return -1;
    mask[dims[i]] = 1;
  }
  int r = 0;
  for (int i = 0; i < rank; ++i)
    if (!mask[i]) out_shape[r++] = shape[i];
  return r;
}

/* ReduceImpl constructor, runtime/lib/backends/cuda/providers/default/reduction/reduce_impl.h:30-59.
 * Returns 0 and fills A,B,C; 1 when the IR output shape differs from the deduced one (:35);
 * 2 when the (size-1-stripped, sorted) dimensions are not consecutive (:41-42);
 * 3 when a dimension is out of range.  "Nothing left to reduce" yields A=B=0, C=numel (:55-58). */
int oracle_reduce_canonicalize(const int64_t *in_shape, int rank, const int64_t *out_shape,
                               int out_rank, const int64_t *dims_in, int ndims, uint64_t *A,
                               uint64_t *B, uint64_t *C) {
  int64_t deduced[64];
  int r = oracle_deduce_output_shape(in_shape, rank, dims_in, ndims, deduced);
  if (r < 0) return 3;
  if (r != out_rank) return 1;
  for (int i = 0; i < r; ++i)
    if (deduced[i] != out_shape[i]) return 1;
  int64_t dims[64];
  int n = 0;
  for (int i = 0; i < ndims; ++i) /* remove_one, :82-91 */
    if (in_shape[dims_in[i]] != 1) dims[n++] = dims_in[i];
  if (n == 0) {
    uint64_t numel = 1;
    for (int i = 0; i < rank; ++i) numel *= (uint64_t)in_shape[i];
    *A = 0; *B = 0; *C = numel;
    return 0;
  }
  for (int i = 1; i < n; ++i) { /* insertion sort */
    int64_t v = dims[i]; int j = i - 1;
    while (j >= 0 && dims[j] > v) { dims[j + 1] = dims[j]; --j; }
    dims[j + 1] = v;
  }
  for (int i = 0; i + 1 < n; ++i)
    if (dims[i + 1] - dims[i] != 1) return 2;
  uint64_t a = 1, b = 1, c = 1;
  for (int64_t i = 0; i < dims[0]; ++i) a *= (uint64_t)in_shape[i];
  for (int i = 0; i < n; ++i) b *= (uint64_t)in_shape[dims[i]];
  for (int64_t i = dims[n - 1] + 1; i < rank; ++i) c *= (uint64_t)in_shape[i];
  *A = a; *B = b; *C = c;
  return 0;
}

/* use_reduce_column, .../reduction/kernels/reduction.cu:411-413 */
int oracle_use_reduce_column(uint64_t A, uint64_t B, uint64_t C) {
  return C == 1 && (B <= A * 4 || B <= 32);
}

/* get_reduce_workspace_in_bytes<T>, .../reduction/kernels/reduction.cu:393-409,428-434 with
 * ExecPolicy (:152-181).  elem_size is sizeof(T) of the tensor type the reference sizes by. */
uint64_t oracle_reference_workspace_bytes(uint64_t A, uint64_t B, uint64_t C, uint64_t elem_size) {
  if (oracle_use_reduce_column(A, B, C)) return 0;
  uint64_t BX = 1;
  while (BX < 32 && BX < C) BX *= 2;
  uint64_t BY = 512 / BX, factor = BY * 4;
  uint64_t nr = 0, tmp = B;
  while (tmp > 1) { tmp = (tmp + factor - 1) / factor; ++nr; }
  if (nr == 0) nr = 1;
  if (nr == 1) return 0;
  uint64_t B2 = (B + factor - 1) / factor;
  if (nr == 2) return elem_size * A * B2 * C;
  uint64_t B3 = (B2 + factor - 1) / factor;
  return elem_size * A * B2 * C + elem_size * A * B3 * C;
}

/* SumOp::apply / MaxOp<...,float>::apply, .../reduction/kernels/reduction_helper.h:18-36,158-179 */
static inline float op_sum(float l, float r) { return l + r; }
static inline float op_max(float l, float r) { return (isnan(l) || l > r) ? l : r; }
/* The operators the reference defines without registering an op kernel for them: MeanOp
 * :37-56 (sum; the store divides by float(B)), SumSqrOp :58-77 (read squares in float), ProdOp
 * :80-95 (init 1), MinOp<...,float> :116-137 (init +inf, NaN from either side wins). */
static inline float fold_init(int op) {
  return op == 1 ? -INFINITY : op == 2 ? INFINITY : op == 3 ? 1.f : 0.f;
}
static inline float fold_map(int op, float x) { return op == 5 ? x * x : x; }
static inline float fold_apply(int op, float l, float r) {
  switch (op) {
  case 1: return op_max(l, r);
  case 2: return (isnan(l) || l < r) ? l : r;
  case 3: return l * r;
  default: return l + r;
  }
}
static inline float fold_finish(int op, float r, uint64_t B) { return op == 4 ? r / (float)B : r; }

/* out[a,c] = fold_b in[a,b,c] as one left-to-right chain per output in the working type
 * float, the order of the reference's own test oracle GoldenReduction
 * (runtime/test/backends/cuda/providers/default/kernel/reduction_test.cc:66-92) and of the
 * linalg loop nest the CPU path executes.  op: 0 = sum (init 0), 1 = max (init -inf),
 * 2 = min, 3 = prod, 4 = mean, 5 = sum of squares.
 * dtype 0 = f32, 1 = f16 (accumulated in float, reduce_impl.h:64-69).
 * A == 0 and B == 0 means "plain copy of C elements" (reduce_impl.h:55-58,71-74). */
void oracle_reduce(int op, int dtype, const void *in, void *out, uint64_t A, uint64_t B,
                   uint64_t C) {
  if (A == 0 && B == 0) {
    size_t es = dtype == 0 ? 4 : 2;
    memcpy(out, in, C * es);
    return;
  }
  /* an empty tensor: no output, or (B == 0) an empty fold per output, which the loops below
   * turn into the operator's identity; the reference's copy branch would read past an input
   * without elements here (reduce_impl.h:61-75) */
  if (dtype == 0 && C == 1 && op <= 1) { /* tight loop for the timed baseline */
    const float *x = (const float *)in;
    float *y = (float *)out;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t a = 0; a < (int64_t)A; ++a) {
      const float *row = x + (size_t)a * B;
      if (op == 0) { float acc = 0.f; for (uint64_t b = 0; b < B; ++b) acc += row[b]; y[a] = acc; }
      else { float acc = -INFINITY; for (uint64_t b = 0; b < B; ++b) acc = op_max(acc, row[b]); y[a] = acc; }
    }
    return;
  }
  if (dtype == 0 && op <= 1) {
    const float *x = (const float *)in;
    float *y = (float *)out;
    for (uint64_t a = 0; a < A; ++a) {
      float *o = y + a * C;
      const float init = op == 0 ? 0.f : -INFINITY;
      for (uint64_t c = 0; c < C; ++c) o[c] = init;
      /* for b, for c: keeps each output's chain in b order and walks memory linearly; with
       * several threads every thread owns a contiguous stripe of columns and does the same */
      const int nt = (C >= 4096 && g_threads > 1) ? g_threads : 1;
#pragma omp parallel for num_threads(nt) schedule(static)
      for (int t = 0; t < nt; ++t) {
        const uint64_t c0 = C * (uint64_t)t / (uint64_t)nt, c1 = C * (uint64_t)(t + 1) / (uint64_t)nt;
        for (uint64_t b = 0; b < B; ++b) {
          const float *row = x + (a * B + b) * C;
          if (op == 0) { for (uint64_t c = c0; c < c1; ++c) o[c] = o[c] + row[c]; }
          else { for (uint64_t c = c0; c < c1; ++c) o[c] = op_max(o[c], row[c]); }
        }
      }
    }
    return;
  }
  for (uint64_t a = 0; a < A; ++a)
    for (uint64_t c = 0; c < C; ++c) {
      float acc = fold_init(op);
      for (uint64_t b = 0; b < B; ++b) {
        float v = fold_map(op, load_elem(in, (a * B + b) * C + c, dtype));
        acc = fold_apply(op, acc, v);
      }
      store_elem(out, a * C + c, dtype, fold_finish(op, acc, B));
    }
}

/* The same fold accumulated in double: the yardstick the 1e-5 tolerance is measured
 * against.  Also returns sum |x| per output, the scale for near-zero sums. */
void oracle_reduce_sum_f64(int dtype, const void *in, double *out, double *out_abs, uint64_t A,
                           uint64_t B, uint64_t C) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t ac = 0; ac < (int64_t)(A * C); ++ac) {
    uint64_t a = (uint64_t)ac / C, c = (uint64_t)ac % C;
    double acc = 0.0, aabs = 0.0;
    for (uint64_t b = 0; b < B; ++b) {
      double v = (double)load_elem(in, (a * B + b) * C + c, dtype);
      acc += v; aabs += fabs(v);
    }
    out[ac] = acc;
    if (out_abs) out_abs[ac] = aabs;
  }
}

/* ------------------------------------------------------------------------------------ */
/* Softmax over the last axis of a [rows, cols] tensor.                                  */
/* linalg_ext.softmax lowering, compiler/lib/Conversion/ToLinalg/LinalgExtToLinalg.cpp:286-410:
 * m = max (init -inf, maxnumf), e = exp(x - m), s = sum e (init 0), y = e / s.
 * Internals are float for every storage type; one rounding at the store.               */
/* ------------------------------------------------------------------------------------ */
void oracle_softmax(int dtype, const void *in, void *out, uint64_t rows, uint64_t cols) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t r = 0; r < (int64_t)rows; ++r) {
    size_t base = (size_t)r * cols;
    float m = -INFINITY;
    for (uint64_t j = 0; j < cols; ++j) m = fmaxf(m, load_elem(in, base + j, dtype)); /* maxnumf */
    float s = 0.f;
    for (uint64_t j = 0; j < cols; ++j) s += expf(load_elem(in, base + j, dtype) - m);
    for (uint64_t j = 0; j < cols; ++j)
      store_elem(out, base + j, dtype, expf(load_elem(in, base + j, dtype) - m) / s);
  }
}

/* ------------------------------------------------------------------------------------ */
/* Flash attention                                                                       */
/* ------------------------------------------------------------------------------------ */

/* The 25 fields of the custom op's extra_args blob, in the order the compiler emits them
 * (compiler/lib/Conversion/HloToByreTensor/HloToByreCustom.cpp:149-176) and the library
 * parses them (external_libs/runtime/flash_attn/lib/flash_api.cu:586-624). */
typedef struct {
  int64_t q_batch_stride, k_batch_stride, v_batch_stride, o_batch_stride;
  int64_t q_row_stride, k_row_stride, v_row_stride, o_row_stride;
  int64_t q_head_stride, k_head_stride, v_head_stride, o_head_stride;
  int64_t b, h, h_k, d, d_rounded;
  float softmax_scale;
  int64_t seqlen_q, seqlen_k, seqlen_q_rounded, seqlen_k_rounded;
  float p_dropout;
  int64_t window_size_left, window_size_right;
} oracle_fa_args;

/* OpAccessor::GetAttrAsVoidPtr packing, runtime/lib/core/framework/op_accessor.cc:212-242:
 * i64 -> 8 bytes, f32 -> 4 bytes, no padding.  Writes 192 bytes, returns the size. */
size_t oracle_fa_pack_args(const oracle_fa_args *a, unsigned char *blob) {
  size_t pos = 0;
#define PUT_I(v) do { int64_t t = (v); memcpy(blob + pos, &t, 8); pos += 8; } while (0)
#define PUT_F(v) do { float t = (v); memcpy(blob + pos, &t, 4); pos += 4; } while (0)
  PUT_I(a->q_batch_stride); PUT_I(a->k_batch_stride); PUT_I(a->v_batch_stride); PUT_I(a->o_batch_stride);
  PUT_I(a->q_row_stride); PUT_I(a->k_row_stride); PUT_I(a->v_row_stride); PUT_I(a->o_row_stride);
  PUT_I(a->q_head_stride); PUT_I(a->k_head_stride); PUT_I(a->v_head_stride); PUT_I(a->o_head_stride);
  PUT_I(a->b); PUT_I(a->h); PUT_I(a->h_k); PUT_I(a->d); PUT_I(a->d_rounded);
  PUT_F(a->softmax_scale);
  PUT_I(a->seqlen_q); PUT_I(a->seqlen_k); PUT_I(a->seqlen_q_rounded); PUT_I(a->seqlen_k_rounded);
  PUT_F(a->p_dropout);
  PUT_I(a->window_size_left); PUT_I(a->window_size_right);
#undef PUT_I
#undef PUT_F
  return pos;
}

size_t oracle_fa_unpack_args(const unsigned char *blob, oracle_fa_args *a) {
  size_t pos = 0;
#define GET_I(f) do { int64_t t; memcpy(&t, blob + pos, 8); a->f = t; pos += 8; } while (0)
#define GET_F(f) do { float t; memcpy(&t, blob + pos, 4); a->f = t; pos += 4; } while (0)
  GET_I(q_batch_stride); GET_I(k_batch_stride); GET_I(v_batch_stride); GET_I(o_batch_stride);
  GET_I(q_row_stride); GET_I(k_row_stride); GET_I(v_row_stride); GET_I(o_row_stride);
  GET_I(q_head_stride); GET_I(k_head_stride); GET_I(v_head_stride); GET_I(o_head_stride);
  GET_I(b); GET_I(h); GET_I(h_k); GET_I(d); GET_I(d_rounded);
  GET_F(softmax_scale);
  GET_I(seqlen_q); GET_I(seqlen_k); GET_I(seqlen_q_rounded); GET_I(seqlen_k_rounded);
  GET_F(p_dropout);
  GET_I(window_size_left); GET_I(window_size_right);
#undef GET_I
#undef GET_F
  return pos;
}

/* Window normalisation of run_mha (flash_api.cu:300-309) and the mask of
 * flash::Mask::apply_mask (lib/mask.h:160-200): key column j is kept for query row i iff
 *   j < sk, j < i + 1 + sk - sq + wr (when a right window exists) and
 *   j >= i + sk - sq - wl (when a left window exists).
 * causal is (wl < 0 && wr == 0); full attention is (wl < 0 && wr < 0). */
static inline void window_bounds(int64_t i, int64_t sq, int64_t sk, int64_t wl, int64_t wr,
                                 int64_t *lo, int64_t *hi) {
  if (wl < 0 && wr >= 0) wl = sk;
  if (wl >= 0 && wr < 0) wr = sk;
  int64_t l = 0, h = sk;
  if (wl >= 0 || wr >= 0) { /* local or causal */
    int64_t right = i + 1 + sk - sq + wr;
    int64_t left = i + sk - sq - wl;
    if (right < h) h = right;
    if (left > l) l = left;
  }
  if (h < 0) h = 0;
  *lo = l; *hi = h;
}

/* Philox4x32 with `rounds` rounds: key = seed, counter = (offset, subsequence)
 * (lib/philox.cuh:22-52; the library runs 7 rounds: six with a key bump and a last one). */
void oracle_philox4x32(uint64_t seed, uint64_t subsequence, uint64_t offset, int rounds, uint32_t out[4]) {
  uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
  uint32_t c[4] = {(uint32_t)offset, (uint32_t)(offset >> 32), (uint32_t)subsequence, (uint32_t)(subsequence >> 32)};
  for (int r = 0; r < rounds; ++r) {
    if (r > 0) { k0 += 0x9E3779B9u; k1 += 0xBB67AE85u; }
    uint64_t p0 = (uint64_t)0xD2511F53u * c[0], p1 = (uint64_t)0xCD9E8D57u * c[2];
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0, n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1, n3 = (uint32_t)p0;
    c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
  }
  memcpy(out, c, 16);
}

/* Dropout keep-mask of the attention matrix (lib/dropout.h:19-23,26-44,76-84 with the call sites
 * flash_fwd_kernel.h:321-334 and flash_bwd_kernel.h:524-533).  The matrix is cut into blocks of
 * 16 rows x 32 columns; one Philox call per (block, lane of a 32-lane warp) yields 16 bytes, one
 * per element the lane holds in the m16n8 accumulator layout (row = lane/4 [+8], column =
 * 8*tile + 2*(lane%4) [+1], four 8-column tiles): byte = 4*tile + 2*(row half) + (column & 1).
 * subsequence = (row block, column block) as (low, high) words, offset = rng_state[1] +
 * (batch*heads + head)*32 + lane, seed = rng_state[0]; kept iff byte <= floor(p_keep*255).
 * Pinned by tests/test_oracle_dropout_layout.py: every thread of a block is walked through the
 * loop nest of apply_dropout over its own register fragment, for the forward and the backward
 * warp tilings; the closed form above must reproduce that bit for bit. */
int oracle_dropout_keep(const uint64_t *rng_state, int64_t bh, int64_t row, int64_t col, uint8_t threshold) {
  const uint32_t lane = (uint32_t)((row % 8) * 4 + (col % 8) / 2);
  const uint64_t subseq = (uint64_t)(uint32_t)(row / 16) | ((uint64_t)(uint32_t)(col / 32) << 32);
  uint32_t r[4];
  oracle_philox4x32(rng_state[0], subseq, rng_state[1] + (uint64_t)((int)bh * 32) + lane, 7, r);
  const int tile = (int)((col % 32) / 8);
  const int byte = 4 * tile + 2 * (int)((row % 16) / 8) + (int)(col & 1);
  return (uint8_t)(r[byte >> 2] >> (8 * (byte & 3))) <= threshold;
}

/* p_keep, its 8-bit threshold and reciprocal as run_mha_fwd derives them (flash_api.cu:291-294) */
static inline void dropout_consts(float p_dropout, float *p_keep, uint8_t *thr, float *rp) {
  *p_keep = 1.f - p_dropout;
  *thr = (uint8_t)floor(*p_keep * 255.0);
  *rp = 1.f / *p_keep;
}

/* Forward, per (batch, head, query row): flash_fwd_kernel.h:276-469 with softmax.h:128-178.
 *   s_j = q_i . k_j in float; m = max_j s_j; p_j = exp2((s_j - m) * scale*log2e);
 *   l = sum_j p_j (float, unrounded p); o = (sum_j round16(p_j) v_j) / l, rounded to storage;
 *   lse = m*scale + ln(l); a row with nothing kept gives o = 0, lse = +inf (softmax.h:171-172).
 * round_p = 0 skips the rounding of P (plain float attention, the "fp32 reference").
 * dtype: 1 = f16, 2 = bf16, 0 = f32 storage.  lse layout [b, h, sq] float.
 * o_f32, when non-null, additionally receives the unrounded output [b, sq, h, d] dense.
 * With a->p_dropout > 0 (rng_state = {seed, offset} required): the row sum and LSE are those of
 * the undropped P; dropped entries of the rounded P are zeroed before P V and O is multiplied
 * by 1/p_keep (flash_fwd_kernel.h:333-335, softmax.h:173). */
void oracle_flash_fwd_rng(const oracle_fa_args *a, int dtype, int round_p, const void *q,
                          const void *k, const void *v, const uint64_t *rng_state, void *o,
                          float *lse, float *o_f32) {
  const int64_t b = a->b, h = a->h, hk = a->h_k, d = a->d, sq = a->seqlen_q, sk = a->seqlen_k;
  const float scale = a->softmax_scale;
  const int drop = a->p_dropout > 0.f && rng_state;
  float p_keep, rp_keep; uint8_t thr;
  dropout_consts(drop ? a->p_dropout : 0.f, &p_keep, &thr, &rp_keep);
  const float scale_log2 = (float)(scale * M_LOG2E); /* flash_api.cu:289 */
  const int64_t ratio = h / hk;
#pragma omp parallel for num_threads(g_threads) schedule(dynamic, 8) collapse(3)
  for (int64_t bi = 0; bi < b; ++bi)
    for (int64_t hi = 0; hi < h; ++hi)
      for (int64_t i = 0; i < sq; ++i) {
        float *s = (float *)malloc(sizeof(float) * (size_t)(sk > 0 ? sk : 1));
        float *acc = (float *)calloc((size_t)d, sizeof(float));
        float *qf = (float *)malloc(sizeof(float) * (size_t)d);
        int64_t lo, hi_;
        window_bounds(i, sq, sk, a->window_size_left, a->window_size_right, &lo, &hi_);
        size_t qoff = (size_t)(bi * a->q_batch_stride + i * a->q_row_stride + hi * a->q_head_stride);
        size_t ooff = (size_t)(bi * a->o_batch_stride + i * a->o_row_stride + hi * a->o_head_stride);
        for (int64_t x = 0; x < d; ++x) qf[x] = load_elem(q, qoff + x, dtype);
        float m = -INFINITY;
        for (int64_t j = lo; j < hi_; ++j) {
          size_t koff = (size_t)(bi * a->k_batch_stride + j * a->k_row_stride + (hi / ratio) * a->k_head_stride);
          float dot = 0.f;
          for (int64_t x = 0; x < d; ++x) dot += qf[x] * load_elem(k, koff + x, dtype);
          s[j] = dot;
          if (dot > m) m = dot;
        }
        float l = 0.f;
        for (int64_t j = lo; j < hi_; ++j) {
          float p = exp2f((s[j] - m) * scale_log2);
          l += p;
          float pr = round_p ? round_storage(p, dtype) : p;
          if (drop && !oracle_dropout_keep(rng_state, bi * h + hi, i, j, thr)) continue;
          size_t voff = (size_t)(bi * a->v_batch_stride + j * a->v_row_stride + (hi / ratio) * a->v_head_stride);
          for (int64_t x = 0; x < d; ++x) acc[x] += pr * load_elem(v, voff + x, dtype);
        }
        int empty = (l == 0.f || l != l);
        float inv = empty ? 1.f : 1.f / l;
        if (drop) inv *= rp_keep;
        for (int64_t x = 0; x < d; ++x) {
          float val = acc[x] * inv;
          store_elem(o, ooff + x, dtype, val);
          if (o_f32) o_f32[((size_t)(bi * sq + i) * h + hi) * d + x] = val;
        }
        lse[(size_t)(bi * h + hi) * sq + i] = empty ? INFINITY : m * scale + logf(l);
        free(s); free(acc); free(qf);
      }
}

void oracle_flash_fwd(const oracle_fa_args *a, int dtype, int round_p, const void *q,
                      const void *k, const void *v, void *o, float *lse, float *o_f32) {
  oracle_flash_fwd_rng(a, dtype, round_p, q, k, v, NULL, o, lse, o_f32);
}

/* Backward: flash_bwd_preprocess_kernel.h:23-50 (D = rowsum(dO*O)) and
 * flash_bwd_kernel.h:455-718:
 *   p_ij = exp2(s_ij*scale*log2e - lse_i*log2e) (0 where masked); dp_ij = dO_i . v_j;
 *   ds_ij = p_ij (dp_ij - D_i); dV_j = sum_i round16(p_ij) dO_i;
 *   dK_j = scale sum_i round16(ds_ij) q_i; dQ_i = scale sum_j round16(ds_ij) k_j.
 * Accumulation in float; outputs rounded to storage.  round_p = 0 keeps p and ds unrounded.
 * dq/dk/dv use the strides of q/k/v (flash_api.cu:377-389).  With grouped heads (h_k < h) dK and
 * dV of a key/value head are the sums over its h / h_k query heads -- the mathematical gradient;
 * the reference's own dK/dV addressing is only right for h == h_k, where this reduces to it.  d_softmax [b, h, sq] float,
 * when non-null, receives D.
 * With a->p_dropout > 0 (rng_state = {seed, offset} required), as the reference arranges it
 * (flash_bwd_preprocess_kernel.h:124-128, flash_bwd_kernel.h:524-536,571-573,667,713-718):
 * D is scaled by p_keep; a dropped entry contributes p = 0 to dV and ds = p * (-D); dQ and dK
 * are scaled by scale/p_keep, dV by 1/p_keep. */
void oracle_flash_bwd_rng(const oracle_fa_args *a, int dtype, int round_p, const void *dout,
                          const void *q, const void *k, const void *v, const void *o,
                          const float *lse, const uint64_t *rng_state, void *dq, void *dk, void *dv,
                          float *d_softmax) {
  const int64_t b = a->b, h = a->h, hk = a->h_k, d = a->d, sq = a->seqlen_q, sk = a->seqlen_k;
  const int64_t ratio = h / hk; /* query heads per key/value head: their dK, dV contributions add up */
  const int drop = a->p_dropout > 0.f && rng_state;
  float p_keep, rp_keep; uint8_t thr;
  dropout_consts(drop ? a->p_dropout : 0.f, &p_keep, &thr, &rp_keep);
  const float scale = drop ? a->softmax_scale * rp_keep : a->softmax_scale;
  const float scale_log2 = (float)(a->softmax_scale * M_LOG2E);
#pragma omp parallel for num_threads(g_threads) schedule(dynamic, 1) collapse(2)
  for (int64_t bi = 0; bi < b; ++bi)
    for (int64_t hki = 0; hki < hk; ++hki) {
      float *dkacc = (float *)calloc((size_t)(sk * d), sizeof(float));
      float *dvacc = (float *)calloc((size_t)(sk * d), sizeof(float));
      float *dqacc = (float *)malloc(sizeof(float) * (size_t)d);
      float *qf = (float *)malloc(sizeof(float) * (size_t)d);
      float *dof = (float *)malloc(sizeof(float) * (size_t)d);
      for (int64_t hi = hki * ratio; hi < (hki + 1) * ratio; ++hi)
      for (int64_t i = 0; i < sq; ++i) {
        size_t qoff = (size_t)(bi * a->q_batch_stride + i * a->q_row_stride + hi * a->q_head_stride);
        size_t ooff = (size_t)(bi * a->o_batch_stride + i * a->o_row_stride + hi * a->o_head_stride);
        float D = 0.f;
        for (int64_t x = 0; x < d; ++x) {
          qf[x] = load_elem(q, qoff + x, dtype);
          dof[x] = load_elem(dout, ooff + x, dtype);
          D += dof[x] * load_elem(o, ooff + x, dtype);
          dqacc[x] = 0.f;
        }
        if (drop) D *= p_keep;
        if (d_softmax) d_softmax[(size_t)(bi * h + hi) * sq + i] = D;
        float lse_i = lse[(size_t)(bi * h + hi) * sq + i];
        int64_t lo, hi_;
        window_bounds(i, sq, sk, a->window_size_left, a->window_size_right, &lo, &hi_);
        for (int64_t j = lo; j < hi_; ++j) {
          size_t koff = (size_t)(bi * a->k_batch_stride + j * a->k_row_stride + hki * a->k_head_stride);
          size_t voff = (size_t)(bi * a->v_batch_stride + j * a->v_row_stride + hki * a->v_head_stride);
          float dot = 0.f, dp = 0.f;
          for (int64_t x = 0; x < d; ++x) {
            dot += qf[x] * load_elem(k, koff + x, dtype);
            dp += dof[x] * load_elem(v, voff + x, dtype);
          }
          float p = exp2f(dot * scale_log2 - lse_i * (float)M_LOG2E);
          float ds = p * (dp - D);
          if (drop && !oracle_dropout_keep(rng_state, bi * h + hi, i, j, thr)) { ds = p * -D; p = 0.f; }
          float pr = round_p ? round_storage(p, dtype) : p;
          float dsr = round_p ? round_storage(ds, dtype) : ds;
          for (int64_t x = 0; x < d; ++x) {
            dvacc[j * d + x] += pr * dof[x];
            dkacc[j * d + x] += dsr * qf[x];
            dqacc[x] += dsr * load_elem(k, koff + x, dtype);
          }
        }
        for (int64_t x = 0; x < d; ++x) store_elem(dq, qoff + x, dtype, dqacc[x] * scale);
      }
      for (int64_t j = 0; j < sk; ++j) {
        size_t koff = (size_t)(bi * a->k_batch_stride + j * a->k_row_stride + hki * a->k_head_stride);
        size_t voff = (size_t)(bi * a->v_batch_stride + j * a->v_row_stride + hki * a->v_head_stride);
        for (int64_t x = 0; x < d; ++x) {
          store_elem(dk, koff + x, dtype, dkacc[j * d + x] * scale);
          store_elem(dv, voff + x, dtype, drop ? dvacc[j * d + x] * rp_keep : dvacc[j * d + x]);
        }
      }
      free(dkacc); free(dvacc); free(dqacc); free(qf); free(dof);
    }
}

void oracle_flash_bwd(const oracle_fa_args *a, int dtype, int round_p, const void *dout,
                      const void *q, const void *k, const void *v, const void *o,
                      const float *lse, void *dq, void *dk, void *dv, float *d_softmax) {
  oracle_flash_bwd_rng(a, dtype, round_p, dout, q, k, v, o, lse, NULL, dq, dk, dv, d_softmax);
}
