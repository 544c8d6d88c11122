#!/usr/bin/env python3
"""Re-encode the reference's flash-attention golden vectors as compact fp16 .npy fixtures.

The reference keeps the inputs and expected outputs of its one flash-attention
forward/backward test case (b=1, seqlen=128, heads=3, head_dim=32, causal,
softmax_scale=0.5, dout = 1/32) as whitespace-separated decimal text, one value per
element, under runtime/test/test_files/flash_attn_*.data.  The reference test parses each
value as a double and casts it to __half (runtime/test/include/brt/test/common/cuda/util.h:76-94),
so every value is exactly representable in fp16; this script performs the same parse and
cast and stores the 12288 values of each file as a little-endian fp16 array of shape
[1, 128, 3, 32]; the files of the key/value-cache case (flash_attn_kvcache_*.data) likewise, with
their own shapes, and the two cache lengths as int32.  Only data is carried over: no reference
source is read.

Run in a container that mounts the reference:
    python tests/golden/make_flash_attn_golden.py [/root/reference]
"""
import os
import sys

import numpy as np

FILES = {
    "flash_attn_inputs_q.data": "fa_q.npy",
    "flash_attn_inputs_k.data": "fa_k.npy",
    "flash_attn_inputs_v.data": "fa_v.npy",
    "flash_attn_inputs_dout.data": "fa_dout.npy",
    "flash_attn_fwd_outputs.data": "fa_out.npy",
    "flash_attn_bwd_outputs_dq.data": "fa_dq.npy",
    "flash_attn_bwd_outputs_dk.data": "fa_dk.npy",
    "flash_attn_bwd_outputs_dv.data": "fa_dv.npy",
}
SHAPE = (1, 128, 3, 32)  # [batch, seqlen, heads, head_dim]

# the key/value-cache case (b=2, one query row, cache of 128 rows with 64 valid, 3 heads,
# head_dim 32; runtime/test/backends/cuda/providers/default/kernel/flash_attn_fwd_test.cc:183-330)
KV_FILES = {
    "flash_attn_kvcache_inputs_q.data": ("fa_kv_q.npy", (2, 1, 3, 32)),
    "flash_attn_kvcache_inputs_k.data": ("fa_kv_knew.npy", (2, 1, 3, 32)),
    "flash_attn_kvcache_inputs_v.data": ("fa_kv_vnew.npy", (2, 1, 3, 32)),
    "flash_attn_kvcache_inputs_kcache.data": ("fa_kv_kcache.npy", (2, 128, 3, 32)),
    "flash_attn_kvcache_inputs_vcache.data": ("fa_kv_vcache.npy", (2, 128, 3, 32)),
    "flash_attn_kvcache_outputs.data": ("fa_kv_out.npy", (2, 1, 3, 32)),
    "flash_attn_kvcache_outputs_kcache.data": ("fa_kv_kcache_out.npy", (2, 128, 3, 32)),
    "flash_attn_kvcache_outputs_vcache.data": ("fa_kv_vcache_out.npy", (2, 128, 3, 32)),
}


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    src_dir = os.path.join(ref_root, "runtime", "test", "test_files")
    dst_dir = os.path.dirname(os.path.abspath(__file__))
    for src, dst in FILES.items():
        with open(os.path.join(src_dir, src)) as f:
            vals = np.array(f.read().split(), dtype=np.float64)
        assert vals.size == int(np.prod(SHAPE)), (src, vals.size)
        h = vals.astype(np.float16)
        # the text must round-trip: every decimal is an exact fp16 value
        assert np.array_equal(h.astype(np.float64), vals), src
        np.save(os.path.join(dst_dir, dst), h.reshape(SHAPE))
        print(f"{src} -> {dst}  min={h.min()} max={h.max()}")
    for src, (dst, shape) in KV_FILES.items():
        with open(os.path.join(src_dir, src)) as f:
            vals = np.array(f.read().split(), dtype=np.float64)
        assert vals.size == int(np.prod(shape)), (src, vals.size)
        h = vals.astype(np.float16)
        assert np.array_equal(h.astype(np.float64), vals), src
        np.save(os.path.join(dst_dir, dst), h.reshape(shape))
        print(f"{src} -> {dst}  min={h.min()} max={h.max()}")
    with open(os.path.join(src_dir, "flash_attn_kvcache_inputs_cache_seqlens.data")) as f:
        seqlens = np.array(f.read().split(), dtype=np.int32)
    assert seqlens.shape == (2,)
    np.save(os.path.join(dst_dir, "fa_kv_seqlens.npy"), seqlens)
    print("cache_seqlens ->", seqlens)


if __name__ == "__main__":
    main()
