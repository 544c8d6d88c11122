// Index arithmetic of the tuned flash-attention kernels (flash_fwd.hip, flash_bwd.hip): which
// (batch, head, block) a workgroup takes, which tiles it visits, where a thread's 16-byte chunk
// of a tile lies in global memory and in LDS.  Plain integer functions without any GPU header,
// so that the kernels and a host-side bounds check (index_check.cc, compiled with g++) run the
// very same code: the check enumerates every (workgroup, thread, tile) of a launch and verifies
// that each address formed here stays inside its tensor, its buffer descriptor or its LDS array.
#pragma once
#include <cstdint>

#if defined(__HIPCC__)
#define FA_HD __host__ __device__ __forceinline__
#else
#define FA_HD inline
#endif

namespace fa {
namespace idx {

// Kept key range [lo, hi) of query row q (reference: lib/mask.h:160-200); wl / wr < 0: unbounded.
FA_HD void row_limits(int sq, int sk, int wl, int wr, int q, int &lo, int &hi) {
  lo = 0; hi = sk;
  const int off = sk - sq;
  if (wr >= 0) { const int h = q + 1 + off + wr; hi = sk < h ? sk : h; }
  if (wl >= 0) { const int l = q + off - wl; lo = l > 0 ? l : 0; }
}

// Workgroup id -> (batch * heads index, block index in launch order).  mode 0: by (batch, head);
// 1: consecutive ids go round-robin over the 8 XCDs and the blocks of a (batch, head) share one;
// 2: as 1, and within an XCD the first block of every (batch, head) comes first, then the second
// of every one, ...; 3: the order of 2 without the XCD grouping (n_bh no multiple of 8).
struct BlockId { int bh, blk; };
FA_HD BlockId decode_block(int L, int mode, int n_bh, int n_blocks) {
  BlockId r;
  if (mode == 2) {
    const int xcd = L & 7, slot = L >> 3, per_xcd = n_bh >> 3;
    r.bh = (slot % per_xcd) * 8 + xcd;
    r.blk = slot / per_xcd;
  } else if (mode == 3) {
    r.bh = L % n_bh;
    r.blk = L / n_bh;
  } else if (mode) {
    const int xcd = L & 7, slot = L >> 3;
    r.bh = (slot / n_blocks) * 8 + xcd;
    r.blk = slot % n_blocks;
  } else {
    r.bh = L / n_blocks;
    r.blk = L % n_blocks;
  }
  return r;
}
FA_HD int block_order_mode(int n_bh, int wr) { return (n_bh % 8 == 0) ? (wr >= 0 ? 2 : 1) : (wr >= 0 ? 3 : 0); }

// Key tiles [n_min, n_max) of `bn` rows that the query rows [m0, m0 + bm) can see.
FA_HD void key_tile_range(int sq, int sk, int wl, int wr, int m0, int bm, int bn, int &n_min, int &n_max) {
  int b_lo, b_hi, t0, t1;
  row_limits(sq, sk, wl, wr, m0, b_lo, t0);
  row_limits(sq, sk, wl, wr, m0 + bm - 1, t1, b_hi);
  n_min = b_lo / bn;
  n_max = b_hi > 0 ? (b_hi + bn - 1) / bn : 0;
}

// Query tiles [m_min, m_max) of `qt` rows that can see the keys [kv0, kv0 + keys); with
// qsplit > 1 the share `q_share` of them.
FA_HD void query_tile_range(int sq, int sk, int wl, int wr, int kv0, int keys, int qt, int qsplit, int q_share,
                            int &m_min, int &m_max) {
  const int off = sk - sq;
  int q_lo = 0, q_hi = sq;
  if (wr >= 0) { const int v = kv0 - off - wr; q_lo = v > 0 ? v : 0; }                    // hi(q) = q+1+off+wr > kv0
  if (wl >= 0) { const int v = kv0 + keys - off + wl; q_hi = sq < v ? sq : v; }            // lo(q) = q+off-wl < kv0+keys
  m_min = q_lo / qt;
  m_max = q_hi > 0 ? (q_hi + qt - 1) / qt : 0;
  if (qsplit > 1) {
    const int n = m_max - m_min > 0 ? m_max - m_min : 0;
    const int per = (n + qsplit - 1) / qsplit;
    m_min += q_share * per;
    m_max = m_max < m_min + per ? m_max : m_min + per;
  }
}

// ---- raw buffer addressing of a [n_rows, D] matrix with `rs` elements between rows ----------
// size of the descriptor: rows beyond n_rows read as zeros
FA_HD uint32_t rsrc_bytes(int n_rows, int64_t rs, int d) {
  return n_rows > 0 ? (uint32_t)((((int64_t)n_rows - 1) * rs + d) * 2) : 0u;
}
// byte offset of the 16-byte chunk c of row `row`
FA_HD uint32_t chunk_offset(int row, int c, int64_t rs) { return (uint32_t)(((int64_t)row * rs + c * 8) * 2); }
// bytes from one tile of `rows` rows to the next
FA_HD uint32_t tile_bytes(int rows, int64_t rs) { return (uint32_t)(rows * rs * 2); }
// the same quantities without the truncation to 32 bits (what the check compares against)
FA_HD int64_t chunk_offset64(int64_t row, int c, int64_t rs) { return (row * rs + c * 8) * 2; }

// ---- LDS layouts (element offsets) -------------------------------------------------------------
// Row strides: rows read with plain 128-bit loads (32 rows x 16 B at a time) want a stride of
// 4*odd banks; rows read with the transposing load (4 rows x 64 B per half-wave) want a stride of
// 16 (mod 32) banks.
FA_HD constexpr int pad_plain(int d) { return d + 8; }
FA_HD constexpr int pad_tr(int d) { return d % 64 == 32 ? d : d + 32; }

// Transposing operand read (two ds_read_b64_tr_b16 per lane) "down the rows" of a row-major tile
// with `stride` elements per row: offset of the first read; the second lies 8 rows below.
FA_HD int tr_operand_offset(int lane, int stride, int row0, int col0) {
  const int i16 = lane & 15, b16 = lane >> 4, gg = b16 >> 1;
  return (row0 + gg * 4 + (i16 >> 2)) * stride + col0 + (b16 & 1) * 16 + (i16 & 3) * 4;
}

// Unpadded tiles read both plainly and transposed: chunk c of row r lives at chunk c ^ key(r).
template <int D> FA_HD int swz_key(int row) {
  if (D == 64) {
    const int x = (row >> 1) & 7;  // rows 2x, 2x+1 share a key and differ in bank parity
    return ((x & 1) << 2) | (x >> 1);
  } else if (D == 128) {
    return ((row & 3) << 2) | ((row >> 2) & 3);
  } else {
    return (row >> 2) & 3;  // D == 32: four rows span the banks
  }
}
template <int D> FA_HD int swz_off(int row, int chunk) { return row * D + ((chunk ^ swz_key<D>(row)) << 3); }
// transposing operand read from such a tile: rows row0.., columns db*32..; `second`: the read 8 rows below
template <int D> FA_HD int swz_tr_operand_offset(int lane, int row0, int db, bool second) {
  const int i16 = lane & 15, b16 = lane >> 4;
  const int row = row0 + (b16 >> 1) * 4 + (i16 >> 2) + (second ? 8 : 0);
  const int chunk = db * 4 + (b16 & 1) * 2 + ((i16 & 3) >> 1), in_chunk = (i16 & 1) * 4;
  return swz_off<D>(row, chunk) + in_chunk;
}

// One wave's [32][128] output tile staged through LDS (head_dim 128): the 16-byte chunks of row
// r are permuted by r >> 1 and odd rows swap the two 8-byte halves of a chunk.
FA_HD int ostage_write_offset(int r32, int g, int db, int i4) {  // 4 elements of row r32, columns db*32 + i4*8 + g*4 ..
  return r32 * 128 + (((db * 4 + i4) ^ (r32 >> 1)) * 8) + ((g ^ (r32 & 1)) * 4);
}
FA_HD int ostage_read_offset(int r, int oc) { return r * 128 + ((oc ^ (r >> 1)) * 8); }  // chunk oc of row r (halves swapped when r is odd)

// ---- backward: sharing the work of a key/value head out over several dK/dV workgroups -------
// base_wg workgroups (one per key/value head and key block) against `slots` workgroup slots on the
// chip: gs = shares of a group's query heads, qs = shares of a key block's query tiles on top.
constexpr int kGroupRounds = 2;  // rounds of workgroups wanted when a window makes them unequal
FA_HD void group_split_counts(int h, int h_k, int sq, int wl, int wr, int64_t base_wg, int slots, int q_tile,
                              int &gs, int &qs) {
  gs = 1; qs = 1;
  const int group = h / h_k;
  const int64_t want_wg = (int64_t)slots * ((wr >= 0 || wl >= 0) ? kGroupRounds : 1);
  if (base_wg <= 0 || base_wg >= want_wg) return;
  if (group > 1) {
    gs = group;
    for (int c = 2; c <= group; ++c)
      if (group % c == 0 && base_wg * c >= want_wg) { gs = c; break; }
  }
  // still short: cut the query axis too, at least sixteen tiles per share, at most eight shares
  if (base_wg * gs < want_wg) {
    const int64_t n_q_tiles = (sq + q_tile - 1) / q_tile;
    qs = (int)((want_wg + base_wg * gs - 1) / (base_wg * gs));
    if (qs > n_q_tiles / 16) qs = (int)(n_q_tiles / 16);
    if (qs > 8) qs = 8;
    if (qs < 1) qs = 1;
  }
}
// float partials [b, sk, virtual heads, row]: bytes of one of the two buffers, and the strides
FA_HD int64_t partial_bytes(int b, int sk, int h_k, int gs, int qs, int row) { return (int64_t)b * sk * h_k * gs * qs * row * 4; }

// ---- the launchers' 2 GiB guards ---------------------------------------------------------------
// Upper bound of the byte offsets a tile stream of the tuned kernels forms inside a (batch, head)
// slice with n_rows rows of stride rs elements: the padded rows of the last tile, the tiles of
// look-ahead that are requested unconditionally and the rows one pass of the workgroup spans.
// Slices for which this reaches 2^31 take the generic kernels (64-bit addressing).
FA_HD int64_t fwd_stream_span_bytes(int64_t sk, int64_t rs) { return 2 * ((sk + 4 * 64 + 128) * rs + 256); }
FA_HD int64_t bwd_stream_span_bytes(int64_t n_rows, int64_t rs) { return 2 * ((n_rows + 256) * rs + 256); }

}  // namespace idx
}  // namespace fa
