"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def dev(a):
    """numpy array (f32/f16, or uint16 bf16 bits) -> device tensor with the same bits."""
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16).copy()).cuda().view(torch.bfloat16)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    """device tensor -> numpy (bf16 comes back as uint16 bits)."""
    t = t.detach()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()
