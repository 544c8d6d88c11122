// C entry points of libflash_attn.so (see include/flash_api.h): blob parsing, validation,
// kernel dispatch.  Counterpart of the reference's run_flash_attn_fwd / run_flash_attn_bwd
// (external_libs/runtime/flash_attn/lib/flash_api.cu:586-725) and run_mha / run_mha_bwd
// (:228-432) for the ROCm provider.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "flash_api.h"
#include "flash_common.h"

namespace fa {
hipError_t launch_fwd(Params &p, int dtype, hipStream_t stream);
hipError_t launch_bwd(Params &p, int dtype, hipStream_t stream);
hipError_t launch_append_kv(const Params &p, int dtype, hipStream_t stream);
}  // namespace fa

namespace {

thread_local char g_err[256] = "";

int fail(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return -1;
}

struct Blob {
  int64_t q_bs, k_bs, v_bs, o_bs, q_rs, k_rs, v_rs, o_rs, q_hs, k_hs, v_hs, o_hs;
  int64_t b, h, h_k, d, d_rounded;
  float softmax_scale;
  int64_t seqlen_q, seqlen_k, seqlen_q_rounded, seqlen_k_rounded;
  float p_dropout;
  int64_t window_size_left, window_size_right;
};

// The blob is unpadded: every i64 after the first float is 4-byte misaligned.
Blob parse(const void *extra_args) {
  const unsigned char *s = static_cast<const unsigned char *>(extra_args);
  size_t pos = 0;
  auto i64 = [&]() { int64_t v; memcpy(&v, s + pos, 8); pos += 8; return v; };
  auto f32 = [&]() { float v; memcpy(&v, s + pos, 4); pos += 4; return v; };
  Blob a;
  a.q_bs = i64(); a.k_bs = i64(); a.v_bs = i64(); a.o_bs = i64();
  a.q_rs = i64(); a.k_rs = i64(); a.v_rs = i64(); a.o_rs = i64();
  a.q_hs = i64(); a.k_hs = i64(); a.v_hs = i64(); a.o_hs = i64();
  a.b = i64(); a.h = i64(); a.h_k = i64(); a.d = i64(); a.d_rounded = i64();
  a.softmax_scale = f32();
  a.seqlen_q = i64(); a.seqlen_k = i64(); a.seqlen_q_rounded = i64(); a.seqlen_k_rounded = i64();
  a.p_dropout = f32();
  // the reference reads the windows through uint32_t and passes them on as int
  // (flash_api.cu:621-624,652-653); -1 survives the round trip
  a.window_size_left = (int32_t)(uint32_t)i64();
  a.window_size_right = (int32_t)(uint32_t)i64();
  return a;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int fill(const Blob &a, fa::Params &p) {
  if (a.b < 0 || a.h <= 0 || a.h_k <= 0 || a.seqlen_q < 0 || a.seqlen_k < 0)
    return fail("negative or zero dimension (b=%ld h=%ld h_k=%ld sq=%ld sk=%ld)", (long)a.b,
                (long)a.h, (long)a.h_k, (long)a.seqlen_q, (long)a.seqlen_k);
  if (a.d <= 0 || a.d > 256 || a.d % 8 != 0)
    return fail("head_dim %ld is not supported (a multiple of 8 up to 256)", (long)a.d);
  if (a.h % a.h_k != 0) return fail("h (%ld) must be a multiple of h_k (%ld)", (long)a.h, (long)a.h_k);
  if (!(a.p_dropout >= 0.f && a.p_dropout < 1.f)) return fail("p_dropout %g is outside [0, 1)", a.p_dropout);
  const int64_t strides[] = {a.q_bs, a.k_bs, a.v_bs, a.o_bs, a.q_rs, a.k_rs,
                             a.v_rs, a.o_rs, a.q_hs, a.k_hs, a.v_hs, a.o_hs};
  for (int64_t s : strides)
    if (s % 8 != 0) return fail("stride %ld is not a multiple of 8 elements (16-byte rows needed)", (long)s);
  if (a.seqlen_q > (1 << 30) || a.seqlen_k > (1 << 30) || a.b * a.h > (1 << 24))
    return fail("problem too large for 32-bit tile indices");
  p.q_bs = a.q_bs; p.k_bs = a.k_bs; p.v_bs = a.v_bs; p.o_bs = a.o_bs;
  p.q_rs = a.q_rs; p.k_rs = a.k_rs; p.v_rs = a.v_rs; p.o_rs = a.o_rs;
  p.q_hs = a.q_hs; p.k_hs = a.k_hs; p.v_hs = a.v_hs; p.o_hs = a.o_hs;
  p.b = (int)a.b; p.h = (int)a.h; p.h_k = (int)a.h_k; p.d = (int)a.d;
  p.sq = (int)a.seqlen_q; p.sk = (int)a.seqlen_k;
  p.sq_rounded = (int)a.seqlen_q_rounded;
  p.scale = a.softmax_scale;
  p.scale_log2 = (float)(a.softmax_scale * M_LOG2E);  // flash_api.cu:289
  // run_mha turns a one-sided window into seqlen_k on the open side (flash_api.cu:300-309);
  // "unbounded" (< 0) is the same thing
  p.wl = a.window_size_left < 0 ? -1 : (int)a.window_size_left;
  p.wr = a.window_size_right < 0 ? -1 : (int)a.window_size_right;
  // flash_api.cu:291-294
  p.p_keep = 1.f - a.p_dropout;
  p.keep_thr = (unsigned)(uint8_t)std::floor(p.p_keep * 255.0);
  p.rp_keep = 1.f / p.p_keep;
  p.drop = a.p_dropout > 0.f ? 1 : 0;
  return 0;
}

// extra_args of run_flash_attn_kvcache (flash_api.cu:727-773): 18 strides, 6 sizes, the scale,
// 4 sequence lengths, 2 window sizes; 31 fields, 244 bytes, unpadded.
struct KvBlob {
  int64_t q_bs, k_bs, v_bs, knew_bs, vnew_bs, o_bs;
  int64_t q_rs, k_rs, v_rs, knew_rs, vnew_rs, o_rs;
  int64_t q_hs, k_hs, v_hs, knew_hs, vnew_hs, o_hs;
  int64_t b, h, h_k, d, d_rounded, seqlen_knew;
  float softmax_scale;
  int64_t seqlen_q, seqlen_k, seqlen_q_rounded, seqlen_k_rounded;
  int64_t window_size_left, window_size_right;
};

KvBlob parse_kv(const void *extra_args) {
  const unsigned char *s = static_cast<const unsigned char *>(extra_args);
  size_t pos = 0;
  auto i64 = [&]() { int64_t v; memcpy(&v, s + pos, 8); pos += 8; return v; };
  auto f32 = [&]() { float v; memcpy(&v, s + pos, 4); pos += 4; return v; };
  KvBlob a;
  a.q_bs = i64(); a.k_bs = i64(); a.v_bs = i64(); a.knew_bs = i64(); a.vnew_bs = i64(); a.o_bs = i64();
  a.q_rs = i64(); a.k_rs = i64(); a.v_rs = i64(); a.knew_rs = i64(); a.vnew_rs = i64(); a.o_rs = i64();
  a.q_hs = i64(); a.k_hs = i64(); a.v_hs = i64(); a.knew_hs = i64(); a.vnew_hs = i64(); a.o_hs = i64();
  a.b = i64(); a.h = i64(); a.h_k = i64(); a.d = i64(); a.d_rounded = i64(); a.seqlen_knew = i64();
  a.softmax_scale = f32();
  a.seqlen_q = i64(); a.seqlen_k = i64(); a.seqlen_q_rounded = i64(); a.seqlen_k_rounded = i64();
  a.window_size_left = (int32_t)i64();  // read as int (flash_api.cu:771-772)
  a.window_size_right = (int32_t)i64();
  return a;
}

}  // namespace

extern "C" {

const char *VERSION = "2.5.3";

const char *flash_attn_last_error(void) { return g_err; }

}  // extern "C"

namespace {
// What every entry point funnels into.  query != nullptr: planning only (tensors may be null),
// *query receives the scratch the same call would take.
struct Scratch { void *ws; size_t ws_bytes; size_t *query; };

int fwd_impl(void **tensors, const void *extra_args, int dtype, const Scratch &sc, void *stream) {
  if ((!tensors && !sc.query) || !extra_args) return fail("null argument");
  if (dtype != 1 && dtype != 2) return fail("dtype %d is not supported (1 = fp16, 2 = bf16)", dtype);
  const Blob a = parse(extra_args);
  fa::Params p{};
  if (int r = fill(a, p)) return r;
  p.ws = sc.ws; p.ws_bytes = sc.ws_bytes; p.ws_query = sc.query;
  if (sc.query) {
    *sc.query = 0;
    return p.b == 0 || p.sq == 0 ? 0 : fa::launch_fwd(p, dtype, nullptr);
  }
  // tensors: q, k, v, rng_state, o, softmax_lse, softmax_P
  p.q = tensors[0]; p.k = tensors[1]; p.v = tensors[2];
  p.rng_state = static_cast<const uint64_t *>(tensors[3]);
  p.o_w = tensors[4];
  p.lse = static_cast<float *>(tensors[5]);
  if (p.b == 0 || p.sq == 0) return 0;
  if (p.drop && !p.rng_state) return fail("p_dropout > 0 needs the rng_state tensor {seed, offset}");
  if (!p.q || !p.o_w || !p.lse || (p.sk > 0 && (!p.k || !p.v))) return fail("null tensor pointer");
  if (!aligned16(p.q) || !aligned16(p.k) || !aligned16(p.v) || !aligned16(p.o_w))
    return fail("q, k, v and o must be 16-byte aligned");
  return fa::launch_fwd(p, dtype, static_cast<hipStream_t>(stream));
}

// dq_accum_bytes: only read when planning (the size of the dq_accum tensor the call will get)
int bwd_impl(void **tensors, const void *extra_args, int dtype, const Scratch &sc, size_t dq_accum_bytes, void *stream) {
  if ((!tensors && !sc.query) || !extra_args) return fail("null argument");
  if (dtype != 1 && dtype != 2) return fail("dtype %d is not supported (1 = fp16, 2 = bf16)", dtype);
  const Blob a = parse(extra_args);
  fa::Params p{};
  if (int r = fill(a, p)) return r;
  if (a.seqlen_q_rounded < a.seqlen_q) return fail("seqlen_q_rounded < seqlen_q");
  p.ws = sc.ws; p.ws_bytes = sc.ws_bytes; p.ws_query = sc.query;
  if (sc.query) {
    *sc.query = 0;
    p.dq_accum = dq_accum_bytes ? reinterpret_cast<void *>(uintptr_t(256)) : nullptr;  // never dereferenced when planning
    p.dq_accum_bytes = dq_accum_bytes;
    return p.b == 0 ? 0 : fa::launch_bwd(p, dtype, nullptr);
  }
  // tensors: dout, q, k, v, out, softmax_lse, rng_state, dq, dk, dv, d_softmax, dq_accum
  p.dout = tensors[0]; p.q = tensors[1]; p.k = tensors[2]; p.v = tensors[3]; p.o = tensors[4];
  p.lse = static_cast<float *>(tensors[5]);
  p.rng_state = static_cast<const uint64_t *>(tensors[6]);
  p.dq = tensors[7]; p.dk = tensors[8]; p.dv = tensors[9];
  p.dsoftmax = static_cast<float *>(tensors[10]);
  p.dq_accum = tensors[11];
  p.dq_accum_bytes = p.dq_accum ? (size_t)a.b * (size_t)a.seqlen_q_rounded * (size_t)a.h * (size_t)a.d_rounded * sizeof(float) : 0;
  if (p.b == 0) return 0;
  if (p.drop && !p.rng_state) return fail("p_dropout > 0 needs the rng_state tensor {seed, offset}");
  // a side without rows (seqlen_q == 0 or seqlen_k == 0) may come as null pointers
  const void *q_side[] = {p.dout, p.q, p.o, p.dq}, *k_side[] = {p.k, p.v, p.dk, p.dv};
  if (p.sq > 0 && (!p.lse || !p.dsoftmax)) return fail("null tensor pointer");
  for (const void *t : q_side) {
    if (!t && p.sq > 0) return fail("null tensor pointer");
    if (!aligned16(t)) return fail("tensors must be 16-byte aligned");
  }
  for (const void *t : k_side) {
    if (!t && p.sk > 0) return fail("null tensor pointer");
    if (!aligned16(t)) return fail("tensors must be 16-byte aligned");
  }
  return fa::launch_bwd(p, dtype, static_cast<hipStream_t>(stream));
}

int kvcache_impl(void **tensors, const void *extra_args, int dtype, const Scratch &sc, void *stream_) {
  if ((!tensors && !sc.query) || !extra_args) return fail("null argument");
  if (dtype != 1 && dtype != 2) return fail("dtype %d is not supported (1 = fp16, 2 = bf16)", dtype);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const KvBlob k = parse_kv(extra_args);
  Blob a{};
  a.q_bs = k.q_bs; a.k_bs = k.k_bs; a.v_bs = k.v_bs; a.o_bs = k.o_bs;
  a.q_rs = k.q_rs; a.k_rs = k.k_rs; a.v_rs = k.v_rs; a.o_rs = k.o_rs;
  a.q_hs = k.q_hs; a.k_hs = k.k_hs; a.v_hs = k.v_hs; a.o_hs = k.o_hs;
  a.b = k.b; a.h = k.h; a.h_k = k.h_k; a.d = k.d; a.d_rounded = k.d_rounded;
  a.softmax_scale = k.softmax_scale;
  a.seqlen_q = k.seqlen_q; a.seqlen_k = k.seqlen_k;
  a.seqlen_q_rounded = k.seqlen_q_rounded; a.seqlen_k_rounded = k.seqlen_k_rounded;
  a.p_dropout = 0.f;
  a.window_size_left = k.window_size_left; a.window_size_right = k.window_size_right;
  fa::Params p{};
  if (int r = fill(a, p)) return r;
  p.ws = sc.ws; p.ws_bytes = sc.ws_bytes; p.ws_query = sc.query;
  if (sc.query) {  // the split depends on the cache capacity, not on seqlens_k
    *sc.query = 0;
    return p.b == 0 || p.sq == 0 ? 0 : fa::launch_fwd(p, dtype, nullptr);
  }
  // tensors: q, k cache, v cache, k new, v new, seqlens_k, o, softmax_lse (flash_api.cu:775-777)
  p.q = tensors[0]; p.k = tensors[1]; p.v = tensors[2];
  p.k_new = tensors[3]; p.v_new = tensors[4];
  p.seqlens_k = static_cast<const int *>(tensors[5]);
  p.o_w = tensors[6];
  p.lse = static_cast<float *>(tensors[7]);
  if (p.b == 0 || p.sq == 0) return 0;
  if (!p.q || !p.o_w || !p.lse || (p.sk > 0 && (!p.k || !p.v))) return fail("null tensor pointer");
  if (!aligned16(p.q) || !aligned16(p.k) || !aligned16(p.v) || !aligned16(p.o_w))
    return fail("q, k, v and o must be 16-byte aligned");
  if ((p.k_new == nullptr) != (p.v_new == nullptr)) return fail("k_new and v_new must be given together");
  if (p.k_new) {
    if (k.seqlen_knew < 0 || k.seqlen_knew > (1 << 30)) return fail("bad seqlen_knew %ld", (long)k.seqlen_knew);
    if (!p.seqlens_k) return fail("appending to the cache needs seqlens_k");
    if (!aligned16(p.k_new) || !aligned16(p.v_new)) return fail("k_new and v_new must be 16-byte aligned");
    const int64_t strides[] = {k.knew_bs, k.vnew_bs, k.knew_rs, k.vnew_rs, k.knew_hs, k.vnew_hs};
    for (int64_t st : strides)
      if (st % 8 != 0) return fail("stride %ld is not a multiple of 8 elements (16-byte rows needed)", (long)st);
    p.seqlen_knew = (int)k.seqlen_knew;
    p.knew_bs = k.knew_bs; p.vnew_bs = k.vnew_bs; p.knew_rs = k.knew_rs; p.vnew_rs = k.vnew_rs;
    p.knew_hs = k.knew_hs; p.vnew_hs = k.vnew_hs;
    if (fa::decode_can_append(p)) p.fuse_append = 1;
    else if (hipError_t e = fa::launch_append_kv(p, dtype, stream)) return e;
  }
  // without seqlens_k every batch attends to all seqlen_k cache rows (BlockInfo, block_info.h:27-37)
  return fa::launch_fwd(p, dtype, stream);
}

}  // namespace

extern "C" {

int flash_attn_fwd_checked(void **tensors, const void *extra_args, int dtype, void *stream) {
  return fwd_impl(tensors, extra_args, dtype, Scratch{nullptr, 0, nullptr}, stream);
}
int flash_attn_bwd_checked(void **tensors, const void *extra_args, int dtype, void *stream) {
  return bwd_impl(tensors, extra_args, dtype, Scratch{nullptr, 0, nullptr}, 0, stream);
}
int flash_attn_kvcache_checked(void **tensors, const void *extra_args, int dtype, void *stream) {
  return kvcache_impl(tensors, extra_args, dtype, Scratch{nullptr, 0, nullptr}, stream);
}
int flash_attn_fwd_ws(void **tensors, const void *extra_args, int dtype, void *workspace, size_t workspace_bytes, void *stream) {
  return fwd_impl(tensors, extra_args, dtype, Scratch{workspace, workspace_bytes, nullptr}, stream);
}
int flash_attn_bwd_ws(void **tensors, const void *extra_args, int dtype, void *workspace, size_t workspace_bytes, void *stream) {
  return bwd_impl(tensors, extra_args, dtype, Scratch{workspace, workspace_bytes, nullptr}, 0, stream);
}
int flash_attn_kvcache_ws(void **tensors, const void *extra_args, int dtype, void *workspace, size_t workspace_bytes, void *stream) {
  return kvcache_impl(tensors, extra_args, dtype, Scratch{workspace, workspace_bytes, nullptr}, stream);
}
size_t flash_attn_fwd_workspace_bytes(const void *extra_args, int dtype) {
  size_t n = 0;
  return fwd_impl(nullptr, extra_args, dtype, Scratch{nullptr, 0, &n}, nullptr) == 0 ? n : 0;
}
size_t flash_attn_bwd_workspace_bytes(const void *extra_args, int dtype, size_t dq_accum_bytes) {
  size_t n = 0;
  return bwd_impl(nullptr, extra_args, dtype, Scratch{nullptr, 0, &n}, dq_accum_bytes, nullptr) == 0 ? n : 0;
}
size_t flash_attn_kvcache_workspace_bytes(const void *extra_args, int dtype) {
  size_t n = 0;
  return kvcache_impl(nullptr, extra_args, dtype, Scratch{nullptr, 0, &n}, nullptr) == 0 ? n : 0;
}

static void die(const char *who, int r) {
  if (r < 0) fprintf(stderr, "libflash_attn: %s: unsupported arguments: %s\n", who, g_err);
  else fprintf(stderr, "libflash_attn: %s: %s\n", who, hipGetErrorString(static_cast<hipError_t>(r)));
  abort();
}

void run_flash_attn_fwd(void **tensors, void *extra_args, void *stream) {
  if (int r = flash_attn_fwd_checked(tensors, extra_args, 1, stream)) die("run_flash_attn_fwd", r);
}
void run_flash_attn_bwd(void **tensors, void *extra_args, void *stream) {
  if (int r = flash_attn_bwd_checked(tensors, extra_args, 1, stream)) die("run_flash_attn_bwd", r);
}
void run_flash_attn_fwd_bf16(void **tensors, void *extra_args, void *stream) {
  if (int r = flash_attn_fwd_checked(tensors, extra_args, 2, stream)) die("run_flash_attn_fwd_bf16", r);
}
void run_flash_attn_kvcache(void **tensors, void *extra_args, void *stream) {
  if (int r = flash_attn_kvcache_checked(tensors, extra_args, 1, stream)) die("run_flash_attn_kvcache", r);
}
void run_flash_attn_kvcache_bf16(void **tensors, void *extra_args, void *stream) {
  if (int r = flash_attn_kvcache_checked(tensors, extra_args, 2, stream)) die("run_flash_attn_kvcache_bf16", r);
}
void run_flash_attn_bwd_bf16(void **tensors, void *extra_args, void *stream) {
  if (int r = flash_attn_bwd_checked(tensors, extra_args, 2, stream)) die("run_flash_attn_bwd_bf16", r);
}

}  // extern "C"
