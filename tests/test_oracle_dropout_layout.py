"""Pins oracle_dropout_keep (the element -> random byte mapping of attention dropout) by an
independent emulation of the reference's own loop nest, thread by thread.

The closed form in oracle/oracle.c says: byte = 4*tile + 2*(row half) + (column parity) of the
Philox value drawn for (row/16, col/32) by lane (row%8)*4 + (col%8)/2.  Nothing in this file uses
that formula.  Instead every thread of a CUDA thread block is walked through
`flash::Dropout::apply_dropout` (lib/dropout.h:26-84) as written there: its accumulator registers
are a flat array addressed through the layout `(4, MMA_M, MMA_N)`, re-viewed as
`((4, 2), MMA_M, MMA_N / 2)` (lib/utils.h:215-223), the loops over m, n, j, i run in the
reference's order, and byte `j * 8 + i` of the Philox value decides register `(i, m, 2n + j)`.
Which matrix element a register holds comes from the reference's own mask code, which spells
the m16n8 accumulator layout out in index arithmetic: forward rows/columns from
flash_fwd_kernel.h:378-380 with mask.h:45-66, backward from flash_bwd_kernel.h:505-516 and
:524-531 (warps tiled AtomLayoutMS x kNWarps/AtomLayoutMS over the score tile).  Philox is
re-implemented here from lib/philox.cuh:22-52 in Python integers.

A swapped row half / column parity, a wrong tile index, a wrong lane formula or a transposed
(row block, column block) subsequence makes the emulation and the closed form disagree; the
negative controls at the end show that they do."""
import numpy as np
import pytest

import oracle

M32 = 0xFFFFFFFF


def philox_7(seed, subsequence, offset):
    """flash::philox (lib/philox.cuh:32-52): six rounds with a key bump after each, then a last one."""
    key = [seed & M32, (seed >> 32) & M32]
    ctr = [offset & M32, (offset >> 32) & M32, subsequence & M32, (subsequence >> 32) & M32]

    def single_round(c, k):  # philox_single_round (:22-30)
        res0 = 0xD2511F53 * c[0]
        res1 = 0xCD9E8D57 * c[2]
        return [((res1 >> 32) ^ c[1] ^ k[0]) & M32, res1 & M32, ((res0 >> 32) ^ c[3] ^ k[1]) & M32, res0 & M32]

    for _ in range(6):
        ctr = single_round(ctr, key)
        key = [(key[0] + 0x9E3779B9) & M32, (key[1] + 0xBB67AE85) & M32]
    out = single_round(ctr, key)
    return b"".join(int(w).to_bytes(4, "little") for w in out)  # reinterpret uint4 as uint8[16]


def apply_dropout(regs_keep, mma_m, mma_n, seed, offset, threshold, block_row_start, block_col_start,
                  block_row_stride):
    """lib/dropout.h:26-84 on one thread.  regs_keep is the thread's flat accumulator array (one
    bool per register); register (v, m, nj) of the `(4, MMA_M, MMA_N)` fragment lives at
    v + 4*m + 4*MMA_M*nj (compact column-major fragment, as partition_fragment_C makes it)."""
    def converted(i, m, n2):
        # convert_layout_acc_dropout: logical_divide of mode 2 by 2 -> (2, MMA_N/2); mode 0 becomes
        # (4, 2) = (atom value, which of two adjacent 8-column tiles): coordinate i = v + 4*t.
        v, t = i % 4, i // 4
        return v + 4 * m + 4 * mma_m * (t + 2 * n2)

    assert mma_n % 4 == 0  # static_assert(size<2>(tensor) % 2 == 0) on the converted tensor
    size2 = mma_n // 2
    for m in range(mma_m):
        row, col = block_row_start, block_col_start
        for n in range(size2 // 2):
            rnd_8 = philox_7(seed, row | (col << 32), offset)  # reinterpret_cast<ull&>(uint2{row, col})
            for j in range(2):
                for i in range(8):
                    regs_keep[converted(i, m, n * 2 + j)] = rnd_8[j * 8 + i] <= threshold
            col += 1
        block_row_start += block_row_stride


def forward_mask(sq, sk, seed, offset0, bid, hid, nheads, threshold, kBlockM, kBlockN, kNWarps):
    """The forward kernel's use (flash_fwd_kernel.h:321-334): all warps along the rows."""
    keep = np.full((sq, sk), -1, dtype=np.int8)
    mma_m, mma_n = kBlockM // (16 * kNWarps), kBlockN // 8
    for m_block in range(sq // kBlockM):
        for n_block in range(sk // kBlockN):
            for tidx in range(kNWarps * 32):
                warp, lane = tidx // 32, tidx % 32
                offset = offset0 + (bid * nheads + hid) * 32 + tidx % 32  # dropout.h:19-23
                regs = [None] * (4 * mma_m * mma_n)
                apply_dropout(regs, mma_m, mma_n, seed, offset, threshold,
                              m_block * (kBlockM // 16) + tidx // 32, n_block * (kBlockN // 32), kNWarps)
                # where each register sits in the matrix: mask.h:45-66 called from
                # flash_fwd_kernel.h:378-380 (row offset, warp_row_stride = kNWarps * 16)
                row_off = m_block * kBlockM + warp * 16 + lane // 4
                col_off = n_block * kBlockN + (lane % 4) * 2
                for mi in range(mma_m):
                    for i in range(2):
                        for nj in range(mma_n):
                            for j in range(2):
                                r = row_off + mi * kNWarps * 16 + i * 8
                                c = col_off + nj * 8 + j
                                v = j + 2 * i  # convert_layout_acc_rowcol: value index (j, i)
                                assert keep[r, c] == -1
                                keep[r, c] = regs[v + 4 * mi + 4 * mma_m * nj]
    assert (keep >= 0).all()
    return keep.astype(bool)


def backward_mask(sq, sk, seed, offset0, bid, hid, nheads, threshold, kBlockM, kBlockN, kNWarps, AtomLayoutMS):
    """The backward kernel's use (flash_bwd_kernel.h:524-531): warps tiled over rows and columns."""
    keep = np.full((sq, sk), -1, dtype=np.int8)
    warps_n = kNWarps // AtomLayoutMS
    mma_m = kBlockM // (16 * AtomLayoutMS)
    mma_n_sdp = kBlockN // (16 * warps_n)
    mma_n = 2 * mma_n_sdp
    for m_block in range(sq // kBlockM):
        for n_block in range(sk // kBlockN):
            for tidx in range(kNWarps * 32):
                warp_id, lane = tidx // 32, tidx % 32
                offset = offset0 + (bid * nheads + hid) * 32 + tidx % 32
                regs = [None] * (4 * mma_m * mma_n)
                apply_dropout(regs, mma_m, mma_n, seed, offset, threshold,
                              m_block * (kBlockM // 16) + warp_id % AtomLayoutMS,
                              n_block * (kBlockN // 32) + (warp_id // AtomLayoutMS) * (mma_n_sdp // 2),
                              AtomLayoutMS)
                # flash_bwd_kernel.h:505-508: column offset of the warp, row offset and row stride
                row_off = m_block * kBlockM + (warp_id % AtomLayoutMS) * 16 + lane // 4
                col_off = n_block * kBlockN + (warp_id // AtomLayoutMS) * mma_n_sdp * 16 + (lane % 4) * 2
                for mi in range(mma_m):
                    for i in range(2):
                        for nj in range(mma_n):
                            for j in range(2):
                                r = row_off + mi * AtomLayoutMS * 16 + i * 8
                                c = col_off + nj * 8 + j
                                assert keep[r, c] == -1
                                keep[r, c] = regs[(j + 2 * i) + 4 * mi + 4 * mma_m * nj]
    assert (keep >= 0).all()
    return keep.astype(bool)


SEED, OFFSET = 0x1234_5678_9ABC_DEF0, 0xFFFF_FFF0  # offset + lane carries into the high word
P_DROPOUT = 0.37


def _oracle_mask(b, h, bid, hid, sq, sk):
    return oracle.dropout_keep_mask(np.array([SEED, OFFSET], dtype=np.uint64), b, h, sq, sk, P_DROPOUT)[bid, hid]


# forward tile shapes the reference launches with dropout (flash_fwd_launch_template.h: head_dim
# 32 -> 128x128, 64 -> 128x64, 128 -> 128x32, all 4 warps) and an 8-warp one
@pytest.mark.parametrize("kBlockM,kBlockN,kNWarps", [(128, 128, 4), (128, 64, 4), (128, 32, 4), (128, 64, 8)])
def test_forward_loop_nest_equals_closed_form(kBlockM, kBlockN, kNWarps):
    b, h, bid, hid, sq, sk = 2, 3, 1, 2, 256, 256
    thr = oracle.dropout_threshold(P_DROPOUT)
    got = forward_mask(sq, sk, SEED, OFFSET, bid, hid, h, thr, kBlockM, kBlockN, kNWarps)
    want = _oracle_mask(b, h, bid, hid, sq, sk)
    assert 0.55 < got.mean() < 0.70
    assert np.array_equal(got, want)


# backward traits of flash_bwd_launch_template.h: head_dim 32/64 -> <128,128,8,AtomLayoutMSdP=4>,
# head_dim 128 -> <64,128,8,2>, and the small-shared-memory variants <64,128,8,4> / <64,64,8,4>
@pytest.mark.parametrize("kBlockM,kBlockN,kNWarps,AtomLayoutMS", [(128, 128, 8, 4), (64, 128, 8, 2), (64, 128, 8, 4), (64, 64, 4, 2)])
def test_backward_loop_nest_equals_closed_form(kBlockM, kBlockN, kNWarps, AtomLayoutMS):
    b, h, bid, hid, sq, sk = 2, 3, 0, 1, 128, 256
    thr = oracle.dropout_threshold(P_DROPOUT)
    got = backward_mask(sq, sk, SEED, OFFSET, bid, hid, h, thr, kBlockM, kBlockN, kNWarps, AtomLayoutMS)
    assert np.array_equal(got, _oracle_mask(b, h, bid, hid, sq, sk))


def test_philox_reimplementation_matches_the_oracle_and_known_answers():
    words = np.frombuffer(philox_7(0, 0, 0), dtype="<u4")
    assert [int(w) for w in words] == [0x5F6FB709, 0x0D893F64, 0x4F121F81, 0x4F730A48]  # Random123 philox4x32_7 KAT
    for seed, sub, off in ((SEED, 5 | (7 << 32), OFFSET + 31), (1, 2, 3)):
        assert [int(w) for w in np.frombuffer(philox_7(seed, sub, off), dtype="<u4")] == \
            [int(w) for w in oracle.philox4x32(seed, sub, off, 7)]


def test_plausible_mistakes_do_not_survive():
    """Negative controls: each wrong closed form differs from the emulated loop nest."""
    sq, sk, h, bid, hid = 32, 64, 3, 1, 2
    thr = oracle.dropout_threshold(P_DROPOUT)
    got = forward_mask(128, 128, SEED, OFFSET, bid, hid, h, thr, 128, 128, 4)[:sq, :sk]

    def closed(lane_f, byte_f, sub_f):
        m = np.zeros((sq, sk), dtype=bool)
        for r in range(sq):
            for c in range(sk):
                rnd = philox_7(SEED, sub_f(r, c), OFFSET + (bid * h + hid) * 32 + lane_f(r, c))
                m[r, c] = rnd[byte_f(r, c)] <= thr
        return m

    lane = lambda r, c: (r % 8) * 4 + (c % 8) // 2
    byte = lambda r, c: 4 * ((c % 32) // 8) + 2 * ((r % 16) // 8) + (c & 1)
    sub = lambda r, c: (r // 16) | ((c // 32) << 32)
    assert np.array_equal(closed(lane, byte, sub), got)  # the right one, written out once more
    wrong = {
        "row half and column parity swapped": (lane, lambda r, c: 4 * ((c % 32) // 8) + 2 * (c & 1) + ((r % 16) // 8), sub),
        "tile index taken as the low bits": (lane, lambda r, c: ((c % 32) // 8) + 4 * (2 * ((r % 16) // 8) + (c & 1)), sub),
        "lane = column group major": (lambda r, c: ((c % 8) // 2) * 8 + r % 8, byte, sub),
        "subsequence words transposed": (lane, byte, lambda r, c: (c // 32) | ((r // 16) << 32)),
        "32-row blocks": (lane, byte, lambda r, c: (r // 32) | ((c // 32) << 32)),
    }
    for what, (lf, bf, sf) in wrong.items():
        assert not np.array_equal(closed(lf, bf, sf), got), what
