"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def to_np(t):
    """Device tensor -> numpy; bfloat16 comes back as uint16 bit patterns."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def to_dev(a, dtype=None):
    """numpy -> cuda tensor; uint16 arrays are bf16 bit patterns."""
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16).copy()).cuda().view(torch.bfloat16)
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


def make_grad(oracle, n, density, dtype, seed, sigma=1e-3):
    """Sparse random gradient as a numpy array in the oracle's representation."""
    rng = np.random.default_rng(seed)
    g = np.where(rng.random(n) < density, rng.standard_normal(n) * sigma, 0).astype(np.float32)
    return oracle.f32_to_bf16_bits(g) if dtype == "bf16" else g
