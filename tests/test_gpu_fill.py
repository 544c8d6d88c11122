"""brt_rocm_fill on the GPU against oracle.fill on the host: the same bits, every storage type,
both distributions, lengths off the block grid."""
import numpy as np
import pytest
import torch

import oracle
from byteir_amd import _lib, ops

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [1, 255, 4097, 1 << 20])
@pytest.mark.parametrize("dist,a,b", [(_lib.FILL_UNIFORM, -1.0, 1.0), (_lib.FILL_UNIFORM, 0.25, 3.0), (_lib.FILL_NORMAL, 0.0, 1.0), (_lib.FILL_NORMAL, 0.0, 2.0)])
@pytest.mark.parametrize("dtype,code", [(torch.float32, 0), (torch.float16, 1), (torch.bfloat16, 2)])
def test_gpu_fill_equals_host_fill(dtype, code, dist, a, b, n):
    seed = 0xC2 + (3 << 32)
    t = ops.fill(torch.empty(n, dtype=dtype, device="cuda"), dist, seed, a, b)
    want = oracle.fill(code, dist, seed, n, a, b)
    got = t.cpu().numpy() if code == 0 else t.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got, want)
