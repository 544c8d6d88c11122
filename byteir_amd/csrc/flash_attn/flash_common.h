// Shared building blocks of the gfx950 flash-attention kernels: element traits, MFMA
// wrappers, LDS helpers and the kernel parameter block.
//
// Register layouts used throughout (wave64, lane l, r = l % 32, g = l / 32):
//   v_mfma_f32_32x32x16_{f16,bf16}:  A[32 x 16]: lane holds A[r][8g .. 8g+7]
//                                     B[16 x 32]: lane holds B[8g .. 8g+7][r]
//                                     C[32 x 32]: lane holds C[8*(i/4) + 4g + i%4][r], i = 0..15
// so a C tile keeps one matrix *column* per lane.  All score tiles are therefore computed
// with the query index on the column axis where per-query statistics (running max, sum, LSE,
// D) must be lane-local, and a C tile feeds the next MFMA as its B operand without moving
// between lanes: B slot (g, j) of 16-row window w is C register 8w + j, i.e. matrix row
// 16w + 8*(j/4) + 4g + j%4.  The other operand is fetched with the same row permutation.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "flash_index.h"

// A kernel launch on `stream` without dynamic LDS.  The kernel name goes in parentheses (its
// template arguments hold commas).  A host build of these sources for tests defines its own
// FA_LAUNCH (and FA_PIN) before this header and runs the workgroups on the CPU.
#ifndef FA_LAUNCH
#define FA_LAUNCH(kernel, grid, block, stream, ...) kernel<<<(grid), (block), 0, (stream)>>>(__VA_ARGS__)
#endif
// Consumes a value in a vector register at this point of the program: the wait for the loads
// that produce it is placed here instead of in front of its first use.
// Marks a point where the lanes of one wave exchange data through LDS without a workgroup
// barrier: what all lanes wrote before it is read by other lanes of the same wave after it.
// On the GPU a wave executes its LDS instructions in program order for all lanes at once, so
// nothing is needed; a lane-by-lane host execution joins the wave's lanes here.
#ifndef FA_WAVE_SYNC
#define FA_WAVE_SYNC() ((void)0)
#endif
#ifndef FA_PIN
#define FA_PIN(x) asm volatile("" : "+v"(x))
#define FA_PIN2(x, y) asm volatile("" : "+v"(x), "+v"(y))
#endif

namespace fa {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

template <typename T> struct Traits;
template <> struct Traits<_Float16> {
  using vec8 = half8;
  static __device__ __forceinline__ float16v mfma(vec8 a, vec8 b, float16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Traits<__bf16> {
  using vec8 = bf16x8;
  static __device__ __forceinline__ float16v mfma(vec8 a, vec8 b, float16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

// 8 floats -> 8 storage elements, round to nearest even
template <typename T>
__device__ __forceinline__ typename Traits<T>::vec8 pack8(const float *f) {
  typename Traits<T>::vec8 v;
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = (T)f[j];
  return v;
}

// acc + the sum of the 8 storage elements of v (exact products with 1, fp32 accumulation):
// four v_dot2c instructions instead of eight adds
template <typename T> __device__ __forceinline__ float sum8_acc(typename Traits<T>::vec8 v, float acc);
template <> __device__ __forceinline__ float sum8_acc<_Float16>(half8 v, float acc) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  const h2 one{(_Float16)1, (_Float16)1};
#pragma unroll
  for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_fdot2(h2{v[2 * j], v[2 * j + 1]}, one, acc, false);
  return acc;
}
template <> __device__ __forceinline__ float sum8_acc<__bf16>(bf16x8 v, float acc) {
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  const b2 one{(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
  for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_fdot2_f32_bf16(b2{v[2 * j], v[2 * j + 1]}, one, acc, false);
  return acc;
}

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float log2_fast(float x) { return __builtin_amdgcn_logf(x); }

// value of the partner lane (l ^ 32)
__device__ __forceinline__ float partner32(float v) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  // lanes < 32 receive (own, partner); lanes >= 32 receive (partner, own)
  const unsigned other = (threadIdx.x & 32) ? r[0] : r[1];
  return __builtin_bit_cast(float, other);
}

// 128-bit LDS read of 8 consecutive elements
template <typename T>
__device__ __forceinline__ typename Traits<T>::vec8 lds_read8(const T *p) {
  return *reinterpret_cast<const typename Traits<T>::vec8 *>(p);
}

// Transposing LDS read (ds_read_b64_tr_b16).  Within each group of 16 lanes, lane i passes
// the address of 4 consecutive elements: lanes 4r..4r+3 together name row r (16 elements) of
// a 4 x 16 block; lane i receives column i of that block (4 elements, rows 0..3).
template <typename T> __device__ __forceinline__ short4v lds_read_tr4(const T *p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) short4v *)(p));
}

// An MFMA A (or B) operand taken "down the rows" of a row-major LDS tile: the lane ends up
// with tile[row0 + perm(g, j)][col0 + r], j = 0..7, where perm(g, j) = 8*(j/4) + 4g + j%4 is
// the row order a C tile presents to the next MFMA.  `stride` in elements.
template <typename T>
__device__ __forceinline__ typename Traits<T>::vec8 lds_read_operand_tr(const T *tile, int stride,
                                                                         int row0, int col0) {
  const T *p = tile + idx::tr_operand_offset(threadIdx.x & 63, stride, row0, col0);
  const short4v lo = lds_read_tr4(p);
  const short4v hi = lds_read_tr4(p + 8 * stride);
  short8v v;
  v.s0 = lo.s0; v.s1 = lo.s1; v.s2 = lo.s2; v.s3 = lo.s3;
  v.s4 = hi.s0; v.s5 = hi.s1; v.s6 = hi.s2; v.s7 = hi.s3;
  return __builtin_bit_cast(typename Traits<T>::vec8, v);
}

// LDS row strides (elements).  Rows read with plain 128-bit loads (32 rows x 16 B at a time)
// want a stride of 4*odd banks; rows read with the transposing load (4 rows x 64 B per
// half-wave) want a stride of 16 (mod 32) banks.
template <int D> struct Pad {
  static constexpr int kPlain = idx::pad_plain(D);
  static constexpr int kTr = idx::pad_tr(D);
};

// Unpadded tiles that are read both ways (backward: Q, dO and K) cannot satisfy both stride
// rules, so their 16-byte chunks are permuted inside each row instead: chunk c of row r lives
// at chunk c ^ key(r).  key() is chosen so that (a) 16 consecutive rows put one logical chunk
// into 16 different 16-byte bank groups (plain reads), and (b) the 4 rows x 4 chunks that one
// half-wave fetches in a transposing read fall into four different 64-byte bank windows.
// A row is D/8 chunks = D/2 banks, so four rows (D = 32), two (D = 64) or one (D = 128) span
// the 64 banks.  key(r) = key(r + 32), so a lane's offsets inside a 32-row unit do not depend
// on the unit.
template <int D> struct Swz {
  static __device__ __forceinline__ int key(int row) { return idx::swz_key<D>(row); }
  // element offset of logical chunk `chunk` of row `row`
  static __device__ __forceinline__ int off(int row, int chunk) { return idx::swz_off<D>(row, chunk); }
};

// lds_read_operand_tr for a tile laid out with Swz<D>: rows row0.., columns db*32..
template <typename T, int D>
__device__ __forceinline__ typename Traits<T>::vec8 lds_read_operand_tr_swz(const T *tile, int row0, int db) {
  const int lane = threadIdx.x & 63;
  const short4v lo = lds_read_tr4(tile + idx::swz_tr_operand_offset<D>(lane, row0, db, false));
  const short4v hi = lds_read_tr4(tile + idx::swz_tr_operand_offset<D>(lane, row0, db, true));
  short8v v;
  v.s0 = lo.s0; v.s1 = lo.s1; v.s2 = lo.s2; v.s3 = lo.s3;
  v.s4 = hi.s0; v.s5 = hi.s1; v.s6 = hi.s2; v.s7 = hi.s3;
  return __builtin_bit_cast(typename Traits<T>::vec8, v);
}

struct Params {
  const void *q, *k, *v, *o, *dout;  // o is written by forward, read by backward
  void *o_w;                          // forward output
  float *lse;                         // [b, h, sq]
  void *dq, *dk, *dv;
  float *dsoftmax;                    // [b, h, sq_rounded]
  void *dq_accum;                     // the caller's [b, sq_rounded, h, d_rounded] float scratch (may be null)
  size_t dq_accum_bytes;
  // dK/dV only: where a workgroup writes its rows (dk / dv with the strides of k / v, or partial
  // buffers), and, when the query heads of a key/value head are shared out over `gsplit`
  // workgroups, the factor by which h_k has been multiplied (K and V of virtual head hk are
  // those of head hk / gsplit)
  int64_t dk_bs, dk_rs, dk_hs, dv_bs, dv_rs, dv_hs;
  int gsplit;
  // ... and the number of shares the visible query tiles of a key block are cut into on top of
  // that (virtual head = (key/value head * gsplit + group share) * qsplit + query share)
  int qsplit;
  int64_t q_bs, k_bs, v_bs, o_bs;     // batch strides (elements)
  int64_t q_rs, k_rs, v_rs, o_rs;     // row strides
  int64_t q_hs, k_hs, v_hs, o_hs;     // head strides
  int b, h, h_k, d;
  int sq, sk, sq_rounded;
  float scale, scale_log2;
  int wl, wr;                         // window sizes after normalisation; < 0 = unbounded
  int n_mblocks, n_nblocks;
  int xcd_remap;                      // 0: by (batch, head); 1: blocks of a (batch, head) share an XCD; 2: 1 + longest blocks of all heads first; 3: longest first without XCD grouping
  // key/value cache calls only: per-batch number of keys already in the cache (the cache
  // holds p.sk rows), rows appended from k_new / v_new before attending
  const int *seqlens_k;
  int seqlen_knew;
  const void *k_new, *v_new;
  int64_t knew_bs, vnew_bs, knew_rs, vnew_rs, knew_hs, vnew_hs;
  int fuse_append;                    // 1: the decode kernel appends k_new / v_new itself
  // forward with the key axis split over workgroups (few query blocks, many keys): grid.y =
  // n_splits, split s takes key tiles [s * split_tiles, (s + 1) * split_tiles) and writes
  // unnormalised fp32 partials, merged by launch_split_merge
  float *o_part;                      // [n_splits][b][h][sq][d]
  float *ml_part;                     // [n_splits][b][h][sq][2]: reference maximum, row sum
  int n_splits, split_tiles;
  // Scratch for the partial results above and for the backward's partial dK / dV: the caller's
  // workspace when the call came through a flash_attn_*_ws entry point and it is large enough,
  // else a stream-ordered allocation of the library's own.  ws_query != nullptr is the
  // planning mode behind flash_attn_*_workspace_bytes: the launch code runs up to the point
  // where it would take scratch, writes the size there and returns without launching anything.
  void *ws;
  size_t ws_bytes;
  size_t *ws_query;
  // dropout (forward and backward calls): rng_state = {seed, offset} in device memory,
  // keep probability, its reciprocal and its 8-bit threshold floor(p_keep * 255)
  const uint64_t *rng_state;
  float p_keep, rp_keep;
  unsigned keep_thr;
  int drop;                           // 1: p_dropout > 0
};

// Kept key range [lo, hi) for query row `q` when the sequence has `sk` keys
// (reference: lib/mask.h:160-200).
__device__ __forceinline__ void row_limits_sk(const Params &p, int sk, int q, int &lo, int &hi) {
  idx::row_limits(p.sq, sk, p.wl, p.wr, q, lo, hi);
}
__device__ __forceinline__ void row_limits(const Params &p, int q, int &lo, int &hi) {
  row_limits_sk(p, p.sk, q, lo, hi);
}

// Kernels for the head dimensions without a tuned instantiation (flash_anyd.hip); the callers
// have set everything in `p` but the block counts.
hipError_t launch_fwd_anyd(Params &p, int dtype, hipStream_t stream);
hipError_t launch_bwd_anyd(Params &p, int dtype, hipStream_t stream);
hipError_t launch_dq_anyd128(const Params &p, int dtype, hipStream_t stream);

// Grouped heads with few key blocks (one or two sequences per GPU): a dK/dV workgroup per
// key/value head and key block leaves most CUs idle, so the query heads of a group are shared
// out over `gs` workgroups that write float partials [b, sk, h_k * gs, row] of dK / dV, which
// launch_group_sum adds (and rounds once).  The partials take the caller's dq_accum scratch as
// far as it reaches; the rest goes to the caller's workspace (flash_attn_bwd_ws) or, without
// one, to a stream-ordered allocation.
struct GroupSplit {
  int gs = 1;             // shares of a group's query heads; 1: no split
  int qs = 1;             // shares of a key block's query tiles on top of that
  void *dk = nullptr, *dv = nullptr;
  void *owned = nullptr;  // to be released with hipFreeAsync after the sum
};
// Rounds of dK/dV workgroups wanted when a window makes them unequal.  Measured (bf16, causal,
// 32 query heads on 8; one / two / four rounds): D = 64 b1 s8192 1235 / 1083 / 1050 us,
// b4 s4096 h16/4 637 / 571 / 570, b8 s2048 615 / 604 / 652; D = 128 b1 s4096 h32/4
// 838 / 626 / 626, b4 s2048 626 / 628 / 681.
using idx::kGroupRounds;
inline GroupSplit plan_group_split(const Params &p, int64_t base_wg, int slots, int row, int q_tile, hipStream_t stream) {
  GroupSplit r;
  // wanted: one round of workgroups over the chip's slots; more when a window makes them
  // unequal, so that the longest-first order can even them out.  First the query heads of a
  // group are shared out; when that is still short, the query axis is cut too, at least sixteen
  // tiles per share, at most eight shares (bf16 backward, with / without: b1 h8 s4096 D=128
  // causal 242 / 270 us, b1 h4 s2048 D=64 causal 71 / 88, b2 h8 on 2 s2048 D=128 causal
  // 147 / 164; with eight tiles per share b1 h16 s1024 D=128 causal lost 6 %)
  int gs, qs;
  idx::group_split_counts(p.h, p.h_k, p.sq, p.wl, p.wr, base_wg, slots, q_tile, gs, qs);
  if (gs * qs == 1) return r;
  const size_t one = (size_t)idx::partial_bytes(p.b, p.sk, p.h_k, gs, qs, row);
  const bool usable = p.dq_accum && (reinterpret_cast<uintptr_t>(p.dq_accum) & 15) == 0;
  const size_t in_accum = !usable ? 0 : p.dq_accum_bytes >= 2 * one ? 2 * one : p.dq_accum_bytes >= one ? one : 0;
  const size_t need = 2 * one - in_accum;  // beyond what dq_accum holds
  if (p.ws_query) { *p.ws_query = need; return r; }
  char *extra = nullptr;
  if (need) {
    if (p.ws && (reinterpret_cast<uintptr_t>(p.ws) & 15) == 0 && p.ws_bytes >= need) extra = static_cast<char *>(p.ws);
    else if (hipMallocAsync(&r.owned, need, stream) == hipSuccess) extra = static_cast<char *>(r.owned);
    else { (void)hipGetLastError(); r.owned = nullptr; return r; }  // no scratch: no split
  }
  char *accum = static_cast<char *>(p.dq_accum);
  if (in_accum == 2 * one) { r.dk = accum; r.dv = accum + one; }
  else if (in_accum == one) { r.dk = accum; r.dv = extra; }
  else { r.dk = extra; r.dv = extra + one; }
  r.gs = gs;
  r.qs = qs;
  return r;
}
// the Params of the dK/dV launch for a split: virtual key/value heads, partial outputs
inline void apply_group_split(Params &pk, const Params &p, const GroupSplit &s, int row) {
  pk.gsplit = s.gs;
  pk.qsplit = s.qs;
  if (s.gs * s.qs == 1) return;
  pk.h_k = p.h_k * s.gs * s.qs;
  pk.dk = s.dk;
  pk.dv = s.dv;
  pk.dk_hs = pk.dv_hs = row;
  pk.dk_rs = pk.dv_rs = (int64_t)pk.h_k * row;
  pk.dk_bs = pk.dv_bs = (int64_t)p.sk * pk.h_k * row;
}
hipError_t launch_group_sum(const Params &p, const GroupSplit &s, int row, int dtype, hipStream_t stream);

// A few query rows against a long key sequence (flash_decode.hip): all query heads of a
// key/value head times all query rows must fit the 32 columns of one score tile.
// merges p.n_splits partials (p.o_part, p.ml_part) into p.o_w and p.lse
hipError_t launch_split_merge(const Params &p, int dtype, hipStream_t stream);
bool decode_eligible(const Params &p);
bool decode_can_append(const Params &p);  // then set p.fuse_append and skip launch_append_kv
hipError_t launch_decode(Params &p, int dtype, hipStream_t stream);

}  // namespace fa
