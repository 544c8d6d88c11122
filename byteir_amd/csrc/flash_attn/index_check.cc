// Host-side bounds check of the tuned flash-attention kernels' index arithmetic (g++, no GPU).
// For one problem shape it walks every workgroup, wave, lane and tile of the forward, dK/dV, dQ,
// D and group-sum launches, forms every global and LDS address with the functions of
// flash_index.h -- the same functions the kernels call -- and verifies:
//   * every decoded (batch, head, block) index lies inside its extent, under each block order;
//   * every tile range lies inside the tile count of its axis;
//   * no 32-bit buffer offset wraps, and an offset the hardware range check lets through
//     (offset + 16 <= descriptor size) addresses bytes inside the tensor;
//   * every guarded global access (Q, O, LSE, D, dQ, dK, dV, partial buffers) lies inside its tensor;
//   * every LDS index lies inside its array (and inside the wave's own region where it has one).
// Tensors are taken as dense [batch, seq, heads, head_dim] (the layout the op kernels pass);
// extents are in elements.  The loop structure of the kernels (which tiles are requested, which
// accesses are guarded by a row test) is restated here; the arithmetic is shared.
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "flash_index.h"

namespace {

using namespace fa::idx;

struct Shape {
  int b, h, h_k, sq, sk, d, wl, wr;
  int qb;            // forward: 32-row halves per wave (1 or 2)
  int64_t dq_accum_bytes;
  int rs_scale;      // row strides are this many times the dense ones (a view into a wider tensor)
};

struct Check {
  long long n_checked = 0, n_failed = 0;
  char first[512] = "";
  void fail(const char *fmt, ...) {
    if (n_failed++ == 0) {
      va_list ap;
      va_start(ap, fmt);
      vsnprintf(first, sizeof(first), fmt, ap);
      va_end(ap);
    }
  }
  // [off, off + n) inside [0, extent)
  void inside(int64_t off, int64_t n, int64_t extent, const char *what, int L, int tid, int extra) {
    ++n_checked;
    if (off < 0 || off + n > extent) fail("%s: [%lld, %lld) outside [0, %lld) (workgroup %d, thread %d, step %d)", what, (long long)off, (long long)(off + n), (long long)extent, L, tid, extra);
  }
  void lt(int64_t v, int64_t bound, const char *what, int L) {
    ++n_checked;
    if (v < 0 || v >= bound) fail("%s: %lld outside [0, %lld) (workgroup %d)", what, (long long)v, (long long)bound, L);
  }
};

int ceil_div(int a, int b) { return (a + b - 1) / b; }

// A tile stream through a buffer descriptor: chunk (row, c) of tiles first .. last-1 (`rows` rows
// each) of the matrix at element offset `base` with n_rows rows of stride rs, inside a tensor
// of `extent` elements.
void check_stream(Check &ck, const char *what, int64_t base, int n_rows, int64_t rs, int d, int row_in_tile, int c,
                  int tile_rows, int first, int last, int64_t extent, int L, int tid) {
  const uint32_t bytes = rsrc_bytes(n_rows, rs, d);
  ck.inside(base * 2, bytes, extent * 2, what, L, tid, -1);  // the descriptor itself covers tensor bytes only
  for (int t = first; t < last; ++t) {
    const int64_t off64 = chunk_offset64((int64_t)t * tile_rows + row_in_tile, c, rs);
    const uint32_t off32 = chunk_offset(row_in_tile, c, rs) + (uint32_t)t * tile_bytes(tile_rows, rs);
    ++ck.n_checked;
    if (off64 >= (int64_t(1) << 32) || (int64_t)off32 != off64)
      ck.fail("%s: 32-bit offset wraps: %lld (workgroup %d, thread %d, tile %d)", what, (long long)off64, L, tid, t);
    if (off64 + 16 <= (int64_t)bytes) ck.inside(base * 2 + off64, 16, extent * 2, what, L, tid, t);
  }
}

template <int D>
void check_forward(Check &ck, const Shape &s) {
  const int QB = s.qb, NW = 8, kThreads = NW * 64, kBM = 32 * QB * NW, kBN = 64, kStages = 3;
  const int KS = pad_plain(D), VS = pad_tr(D);
  const int64_t q_rs = (int64_t)s.h * D * s.rs_scale, q_hs = D, q_bs = (int64_t)s.sq * q_rs;
  const int64_t k_rs = (int64_t)s.h_k * D * s.rs_scale, k_hs = D, k_bs = (int64_t)s.sk * k_rs;
  const int64_t q_ext = (int64_t)s.b * q_bs, k_ext = (int64_t)s.b * k_bs, lse_ext = (int64_t)s.b * s.h * s.sq;
  const int n_mblocks = ceil_div(s.sq, kBM);
  const int grid = n_mblocks * s.b * s.h, mode = block_order_mode(s.b * s.h, s.wr);
  const int CPR = D / 8, RPP = kThreads / CPR, NP = RPP >= kBN ? 1 : kBN / RPP;
  const int lds_k = kBN * KS, lds_v = kBN * VS;
  for (int L = 0; L < grid; ++L) {
    const BlockId blk = decode_block(L, mode, s.b * s.h, n_mblocks);
    ck.lt(blk.bh, s.b * s.h, "forward: batch*head index", L);
    ck.lt(blk.blk, n_mblocks, "forward: query block index", L);
    const int m_block = n_mblocks - 1 - blk.blk, bi = blk.bh / s.h, hi = blk.bh % s.h, hk = hi / (s.h / s.h_k);
    const int m0 = m_block * kBM;
    int n_min, n_max;
    key_tile_range(s.sq, s.sk, s.wl, s.wr, m0, kBM, kBN, n_min, n_max);
    ck.lt(n_min, ceil_div(s.sk, kBN) + 1, "forward: first key tile", L);
    ck.lt(n_max, ceil_div(s.sk, kBN) + 1, "forward: end of key tiles", L);
    const int n_tiles = n_max > n_min ? n_max - n_min : 0;
    // tiles requested: the prologue always asks for three, the loop for the rest
    const int last_req = n_tiles > 0 ? (n_min + 3 > n_max ? n_min + 3 : n_max) : n_min;
    const int64_t kbase = bi * k_bs + hk * k_hs;
    for (int tid = 0; tid < kThreads; ++tid) {
      const int ld_c = tid % CPR, ld_r = tid / CPR;
      const bool ld_on = RPP <= kBN || ld_r < kBN;
      if (ld_on)
        for (int p = 0; p < NP; ++p) {
          check_stream(ck, "forward: K/V tile load", kbase, s.sk, k_rs, D, ld_r + p * RPP, ld_c, kBN, n_min, last_req, k_ext, L, tid);
          ck.inside(ld_r * KS + ld_c * 8 + p * RPP * KS, 8, lds_k, "forward: K tile LDS store", L, tid, p);
          ck.inside(ld_r * VS + ld_c * 8 + p * RPP * VS, 8, lds_v, "forward: V tile LDS store", L, tid, p);
        }
      const int lane = tid & 63, wave = tid >> 6, r32 = lane & 31, g = lane >> 5;
      const int wq0 = m0 + wave * 32 * QB;
      for (int qb = 0; qb < QB; ++qb) {
        const int qrow = wq0 + qb * 32 + r32;
        if (qrow < s.sq) {
          for (int ks = 0; ks < D / 16; ++ks)
            ck.inside(bi * q_bs + (int64_t)qrow * q_rs + hi * q_hs + ks * 16 + g * 8, 8, q_ext, "forward: Q fragment load", L, tid, ks);
          if (D != 128)
            for (int db = 0; db < D / 32; ++db)
              for (int i4 = 0; i4 < 4; ++i4)
                ck.inside(bi * q_bs + (int64_t)qrow * q_rs + hi * q_hs + db * 32 + i4 * 8 + g * 4, 4, q_ext, "forward: O store", L, tid, db);
          ck.inside(((int64_t)bi * s.h + hi) * s.sq + qrow, 1, lse_ext, "forward: LSE store", L, tid, qb);
        }
        if (D == 128) {  // O through the wave's own [32][D] region of the idle ring
          const int region = (wave % (NW / 2)) * 32 * D, ring = kStages * (wave < NW / 2 ? lds_k : lds_v);
          for (int db = 0; db < D / 32; ++db)
            for (int i4 = 0; i4 < 4; ++i4) {
              ck.inside(ostage_write_offset(r32, g, db, i4), 4, 32 * D, "forward: O staging write (own region)", L, tid, db);
              ck.inside(region + ostage_write_offset(r32, g, db, i4), 4, ring, "forward: O staging write (ring)", L, tid, db);
            }
          const int CPRO = D / 8, RPI = 64 / CPRO, oc = lane % CPRO, orow = lane / CPRO;
          for (int it = 0; it < 32 / RPI; ++it) {
            const int r = it * RPI + orow, q = wq0 + qb * 32 + r;
            ck.inside(ostage_read_offset(r, oc), 8, 32 * D, "forward: O staging read", L, tid, it);
            if (q < s.sq) ck.inside(bi * q_bs + (int64_t)q * q_rs + hi * q_hs + oc * 8, 8, q_ext, "forward: O row store", L, tid, it);
          }
        }
      }
      // LDS operand reads of one tile (independent of the tile)
      if (L == 0) {
        const int k_rd = r32 * KS + g * 8;
        for (int kvb = 0; kvb < 2; ++kvb) {
          for (int ks = 0; ks < D / 16; ++ks) ck.inside(k_rd + kvb * 32 * KS + ks * 16, 8, lds_k, "forward: K fragment LDS read", L, tid, ks);
          for (int w = 0; w < 2; ++w)
            for (int db = 0; db < D / 32; ++db) {
              const int o = tr_operand_offset(lane, VS, kvb * 32 + w * 16, db * 32);
              ck.inside(o, 4, lds_v, "forward: V^T LDS read", L, tid, db);
              ck.inside(o + 8 * VS, 4, lds_v, "forward: V^T LDS read (second)", L, tid, db);
            }
        }
      }
    }
  }
}

template <int D>
void check_backward(Check &ck, const Shape &s) {
  const int kKvBlock = 128, kQTile = 64, kQBlock = 128, kKvTile = 64;
  const int64_t q_rs = (int64_t)s.h * D * s.rs_scale, q_hs = D, q_bs = (int64_t)s.sq * q_rs;
  const int64_t k_rs = (int64_t)s.h_k * D * s.rs_scale, k_hs = D, k_bs = (int64_t)s.sk * k_rs;
  const int64_t q_ext = (int64_t)s.b * q_bs, k_ext = (int64_t)s.b * k_bs;
  const int sq_rounded = ceil_div(s.sq, 128) * 128;
  const int64_t lse_ext = (int64_t)s.b * s.h * s.sq, dsm_ext = (int64_t)s.b * s.h * sq_rounded;
  const int CPR = D / 8, RPP = 256 / CPR;

  // ---- D = rowsum(dO o O): one row per D/8 lanes
  {
    const int RPB = 256 / CPR;
    const int64_t total = (int64_t)s.b * s.h * s.sq;
    const int64_t grid = (total + RPB - 1) / RPB;
    for (int64_t blk = 0; blk < grid; blk += (grid > 64 ? grid / 64 : 1))  // the arithmetic is the same for every block: sample them, plus the last
      for (int tid = 0; tid < 256; ++tid) {
        const int64_t row = blk * RPB + tid / CPR, rr = row < total ? row : total - 1;
        const int i = (int)(rr % s.sq), hi = (int)((rr / s.sq) % s.h), bi = (int)(rr / ((int64_t)s.sq * s.h));
        ck.inside(bi * q_bs + (int64_t)i * q_rs + hi * q_hs + (tid % CPR) * 8, 8, q_ext, "D kernel: dO / O load", (int)blk, tid, 0);
        if (row < total) ck.inside(((int64_t)bi * s.h + hi) * sq_rounded + i, 1, dsm_ext, "D kernel: store", (int)blk, tid, 0);
      }
    if (grid > 0)
      for (int tid = 0; tid < 256; ++tid) {
        const int64_t row = (grid - 1) * RPB + tid / CPR, rr = row < total ? row : total - 1;
        const int i = (int)(rr % s.sq), hi = (int)((rr / s.sq) % s.h), bi = (int)(rr / ((int64_t)s.sq * s.h));
        ck.inside(bi * q_bs + (int64_t)i * q_rs + hi * q_hs + (tid % CPR) * 8, 8, q_ext, "D kernel: dO / O load (last block)", (int)(grid - 1), tid, 0);
      }
  }

  // ---- dK / dV
  const int n_nblocks = ceil_div(s.sk, kKvBlock);
  int gs, qs;
  group_split_counts(s.h, s.h_k, s.sq, s.wl, s.wr, (int64_t)n_nblocks * s.b * s.h_k, 256 * (D <= 64 ? 2 : 1), kQTile, gs, qs);
  const int64_t one = partial_bytes(s.b, s.sk, s.h_k, gs, qs, D);
  if (gs * qs > 1 && s.dq_accum_bytes >= 2 * one) ck.inside(0, 2 * one, s.dq_accum_bytes, "dK/dV partials in dq_accum", 0, 0, 0);
  const int vh_k = s.h_k * gs * qs;  // virtual key/value heads
  const int64_t p_hs = D, p_rs = (int64_t)vh_k * D, p_bs = (int64_t)s.sk * p_rs;
  {
    const int grid = n_nblocks * s.b * vh_k, mode = block_order_mode(s.b * vh_k, s.wr);
    const int NP = kQTile / RPP, lds_t = kQTile * D;
    for (int L = 0; L < grid; ++L) {
      const BlockId blk = decode_block(L, mode, s.b * vh_k, n_nblocks);
      ck.lt(blk.bh, s.b * vh_k, "dK/dV: batch*head index", L);
      ck.lt(blk.blk, n_nblocks, "dK/dV: key block index", L);
      const int bi = blk.bh / vh_k, vh = blk.bh % vh_k, hk = vh / qs, q_share = vh % qs;
      const int group = s.h / (vh_k / qs), hkv = hk / gs;
      ck.lt(hkv, s.h_k, "dK/dV: key/value head", L);
      const int kvb0 = blk.blk * kKvBlock;
      int m_min, m_max;
      query_tile_range(s.sq, s.sk, s.wl, s.wr, kvb0, kKvBlock, kQTile, qs, q_share, m_min, m_max);
      if (m_max > m_min) ck.lt(m_max, ceil_div(s.sq, kQTile) + 1, "dK/dV: end of query tiles", L);
      for (int tid = 0; tid < 256; ++tid) {
        const int lane = tid & 63, wave = tid >> 6, r32 = lane & 31, g = lane >> 5;
        const int kv = kvb0 + wave * 32 + r32;
        if (kv < s.sk) {
          for (int ks = 0; ks < D / 16; ++ks)
            ck.inside(bi * k_bs + (int64_t)kv * k_rs + hkv * k_hs + ks * 16 + g * 8, 8, k_ext, "dK/dV: K / V fragment load", L, tid, ks);
          for (int db = 0; db < D / 32; ++db)
            for (int i4 = 0; i4 < 4; ++i4) {
              if (gs * qs > 1) ck.inside((bi * p_bs + (int64_t)kv * p_rs + vh * p_hs + db * 32 + i4 * 8 + g * 4) * 4, 16, one, "dK/dV: partial store", L, tid, db);
              else if (D != 128) ck.inside(bi * k_bs + (int64_t)kv * k_rs + hk * k_hs + db * 32 + i4 * 8 + g * 4, 4, k_ext, "dK/dV: dK / dV store", L, tid, db);
            }
        }
        if (D == 128 && gs * qs == 1) {  // rows through the wave's own region of the idle Q / dO ring
          for (int db = 0; db < D / 32; ++db)
            for (int i4 = 0; i4 < 4; ++i4)
              ck.inside(wave * 32 * D + ostage_write_offset(r32, g, db, i4), 4, 3 * lds_t, "dK/dV: staging write", L, tid, db);
          const int CPRO = D / 8, RPI = 64 / CPRO, oc = lane % CPRO, orow = lane / CPRO;
          for (int it = 0; it < 32 / RPI; ++it) {
            const int r = it * RPI + orow, kvr = kvb0 + wave * 32 + r;
            ck.inside(ostage_read_offset(r, oc), 8, 32 * D, "dK/dV: staging read", L, tid, it);
            if (kvr < s.sk) ck.inside(bi * k_bs + (int64_t)kvr * k_rs + hk * k_hs + oc * 8, 8, k_ext, "dK/dV: row store", L, tid, it);
          }
        }
        for (int gq = 0; gq < group; ++gq) {
          const int hi = hk * group + gq;
          ck.lt(hi, s.h, "dK/dV: query head", L);
          const int c = tid % CPR, r = tid / CPR;
          for (int p = 0; p < NP; ++p)
            check_stream(ck, "dK/dV: Q / dO tile load", bi * q_bs + hi * q_hs, s.sq, q_rs, D, r + p * RPP, c, kQTile, m_min, m_max, q_ext, L, tid);
          if (tid < kQTile)
            for (int m = m_min; m < m_max; ++m) {
              const int q = m * kQTile + tid;
              if (q < s.sq) {
                ck.inside(((int64_t)bi * s.h + hi) * s.sq + q, 1, lse_ext, "dK/dV: LSE load", L, tid, m);
                ck.inside(((int64_t)bi * s.h + hi) * sq_rounded + q, 1, dsm_ext, "dK/dV: D load", L, tid, m);
              }
            }
        }
        if (L == 0) {
          const int c = tid % CPR, r = tid / CPR;
          for (int p = 0; p < NP; ++p) ck.inside(swz_off<D>(p * RPP + r, c), 8, lds_t, "dK/dV: Q / dO tile LDS store", L, tid, p);
          for (int qsu = 0; qsu < 2; ++qsu) {
            for (int ks = 0; ks < D / 16; ++ks) ck.inside(qsu * 32 * D + swz_off<D>(r32, ks * 2 + g), 8, lds_t, "dK/dV: Q / dO fragment LDS read", L, tid, ks);
            for (int w = 0; w < 2; ++w)
              for (int db = 0; db < D / 32; ++db)
                for (int second = 0; second < 2; ++second)
                  ck.inside(swz_tr_operand_offset<D>(lane, qsu * 32 + w * 16, db, second != 0), 4, lds_t, "dK/dV: transposed LDS read", L, tid, db);
            for (int i4 = 0; i4 < 4; ++i4) ck.inside(qsu * 32 + i4 * 8 + g * 4, 4, kQTile, "dK/dV: LSE / D LDS read", L, tid, i4);
          }
        }
      }
    }
    // ---- sum of the partials
    if (gs * qs > 1) {
      const int cpr = D / 8;
      const int64_t chunks = (int64_t)s.b * s.sk * s.h_k * cpr;
      for (int64_t idx = 0; idx < chunks; idx += (chunks > 4096 ? chunks / 4096 : 1)) {
        const int c = (int)(idx % cpr), hk = (int)((idx / cpr) % s.h_k);
        const int64_t r = idx / ((int64_t)cpr * s.h_k);
        const int kv = (int)(r % s.sk), bi = (int)(r / s.sk);
        const int64_t src = ((r * s.h_k + hk) * (gs * qs)) * D + c * 8;
        for (int sh = 0; sh < gs * qs; ++sh) ck.inside((src + (int64_t)sh * D) * 4, 32, one, "group sum: partial load", (int)(idx / 256), (int)(idx % 256), sh);
        ck.inside(bi * k_bs + (int64_t)kv * k_rs + hk * k_hs + c * 8, 8, k_ext, "group sum: dK / dV store", (int)(idx / 256), (int)(idx % 256), 0);
      }
    }
  }

  // ---- dQ
  {
    const int n_mblocks = ceil_div(s.sq, kQBlock), grid = n_mblocks * s.b * s.h, mode = block_order_mode(s.b * s.h, s.wr);
    const int VS = pad_plain(D), NP = kKvTile / RPP, lds_k = kKvTile * D, lds_v = kKvTile * VS;
    for (int L = 0; L < grid; ++L) {
      const BlockId blk = decode_block(L, mode, s.b * s.h, n_mblocks);
      ck.lt(blk.bh, s.b * s.h, "dQ: batch*head index", L);
      ck.lt(blk.blk, n_mblocks, "dQ: query block index", L);
      const int m_block = n_mblocks - 1 - blk.blk, bi = blk.bh / s.h, hi = blk.bh % s.h, hk = hi / (s.h / s.h_k);
      const int m0 = m_block * kQBlock;
      int n_min, n_max;
      key_tile_range(s.sq, s.sk, s.wl, s.wr, m0, kQBlock, kKvTile, n_min, n_max);
      ck.lt(n_max, ceil_div(s.sk, kKvTile) + 1, "dQ: end of key tiles", L);
      for (int tid = 0; tid < 256; ++tid) {
        const int lane = tid & 63, wave = tid >> 6, r32 = lane & 31, g = lane >> 5;
        const int qrow = m0 + wave * 32 + r32;
        if (qrow < s.sq) {
          for (int ks = 0; ks < D / 16; ++ks)
            ck.inside(bi * q_bs + (int64_t)qrow * q_rs + hi * q_hs + ks * 16 + g * 8, 8, q_ext, "dQ: Q / dO fragment load", L, tid, ks);
          ck.inside(((int64_t)bi * s.h + hi) * s.sq + qrow, 1, lse_ext, "dQ: LSE load", L, tid, 0);
          ck.inside(((int64_t)bi * s.h + hi) * sq_rounded + qrow, 1, dsm_ext, "dQ: D load", L, tid, 0);
          for (int db = 0; db < D / 32; ++db)
            for (int i4 = 0; i4 < 4; ++i4)
              ck.inside(bi * q_bs + (int64_t)qrow * q_rs + hi * q_hs + db * 32 + i4 * 8 + g * 4, 4, q_ext, "dQ: store", L, tid, db);
        }
        const int c = tid % CPR, r = tid / CPR;
        for (int p = 0; p < NP; ++p)
          check_stream(ck, "dQ: K / V tile load", bi * k_bs + hk * k_hs, s.sk, k_rs, D, r + p * RPP, c, kKvTile, n_min, n_max, k_ext, L, tid);
        if (L == 0) {
          for (int p = 0; p < NP; ++p) {
            ck.inside(swz_off<D>(p * RPP + r, c), 8, lds_k, "dQ: K tile LDS store", L, tid, p);
            ck.inside((p * RPP + r) * VS + c * 8, 8, lds_v, "dQ: V tile LDS store", L, tid, p);
          }
          for (int kvb = 0; kvb < 2; ++kvb) {
            for (int ks = 0; ks < D / 16; ++ks) {
              ck.inside(kvb * 32 * D + swz_off<D>(r32, ks * 2 + g), 8, lds_k, "dQ: K fragment LDS read", L, tid, ks);
              ck.inside(kvb * 32 * VS + r32 * VS + g * 8 + ks * 16, 8, lds_v, "dQ: V fragment LDS read", L, tid, ks);
            }
            for (int w = 0; w < 2; ++w)
              for (int db = 0; db < D / 32; ++db)
                for (int second = 0; second < 2; ++second)
                  ck.inside(swz_tr_operand_offset<D>(lane, kvb * 32 + w * 16, db, second != 0), 4, lds_k, "dQ: K^T LDS read", L, tid, db);
          }
        }
      }
    }
  }
}

}  // namespace

// shape: b, h, h_k, sq, sk, d, wl, wr, qb, which (1 forward, 2 backward, 3 both), rs_scale.  Returns the
// number of failed checks (the first one described in msg), -1 for an unsupported head_dim;
// *n_checked receives the number of checks made.
extern "C" long long fa_index_check(const long long *shape, long long dq_accum_bytes, long long *n_checked, char *msg, int msg_len) {
  Shape s{(int)shape[0], (int)shape[1], (int)shape[2], (int)shape[3], (int)shape[4], (int)shape[5], (int)shape[6], (int)shape[7], (int)shape[8], dq_accum_bytes, shape[10] > 0 ? (int)shape[10] : 1};
  const int which = (int)shape[9];
  Check ck;
  switch (s.d) {
  case 32: if (which & 1) check_forward<32>(ck, s); if (which & 2) check_backward<32>(ck, s); break;
  case 64: if (which & 1) check_forward<64>(ck, s); if (which & 2) check_backward<64>(ck, s); break;
  case 128: if (which & 1) check_forward<128>(ck, s); if (which & 2) check_backward<128>(ck, s); break;
  default: return -1;
  }
  if (n_checked) *n_checked = ck.n_checked;
  if (msg && msg_len > 0) { strncpy(msg, ck.first, msg_len - 1); msg[msg_len - 1] = 0; }
  return ck.n_failed;
}

// The launchers' 2 GiB guards (what routes a call to the generic kernels instead).
extern "C" long long fa_fwd_stream_span_bytes(long long sk, long long rs) { return fa::idx::fwd_stream_span_bytes(sk, rs); }
extern "C" long long fa_bwd_stream_span_bytes(long long n_rows, long long rs) { return fa::idx::bwd_stream_span_bytes(n_rows, rs); }
