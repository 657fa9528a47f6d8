"""zen_topk_threshold_static, the entry point that allocates nothing (its
radix-select counters live in a static device array inside the library),
against zen_topk_threshold and the CPU oracle: bit-exact, on two calls in a row,
the second on a smaller input, so that anything the first call leaves in the
shared array would show."""
import numpy as np
import pytest
import torch

from gpu_util import to_dev

pytestmark = pytest.mark.gpu


def _both(L, _lib, grad, k):
    """(static entry point's answer, workspace entry point's answer) as numpy uint32[2]."""
    dev = grad.device
    thr_static = torch.full((2,), -1, dtype=torch.int32, device=dev)
    thr_ws = torch.full((2,), -2, dtype=torch.int32, device=dev)
    ws = torch.empty(L.zen_topk_threshold_workspace(), dtype=torch.uint8, device=dev)
    stream = _lib.stream_of(dev)
    rc = L.zen_topk_threshold_static(_lib.ptr(grad), _lib.dtype_code(grad), grad.numel(), k, _lib.ptr(thr_static),
                                     stream)
    assert rc == 0, L.zen_last_error()
    rc = L.zen_topk_threshold(_lib.ptr(grad), _lib.dtype_code(grad), grad.numel(), k, _lib.ptr(thr_ws), _lib.ptr(ws),
                              ws.numel(), stream)
    assert rc == 0, L.zen_last_error()
    torch.cuda.synchronize()
    return thr_static.cpu().numpy().view(np.uint32), thr_ws.cpu().numpy().view(np.uint32)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_static_scratch_topk_matches_the_workspace_entry_point(oracle, dtype):
    from zen_repro_amd import _lib

    L = _lib.lib()
    rng = np.random.default_rng(77)
    # a large call first, then a smaller one with other data and another k
    for n, k in ((3_000_001, 30_000), (70_001, 69)):
        g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        g[rng.integers(0, n, n // 50)] = 0.0
        g_np = oracle.f32_to_bf16_bits(g) if dtype == "bf16" else g
        grad = to_dev(g_np)
        got, want = _both(L, _lib, grad, k)
        assert np.array_equal(got, want), (n, k, got, want)
        key = oracle.kth_key(g_np, k)
        assert int(got[0]) == key
        keys = (g_np.view(np.uint16) & 0x7FFF) if dtype == "bf16" else (g_np.view(np.uint32) & 0x7FFFFFFF)
        assert int(got[1]) == int((keys >= key).sum())


def test_static_scratch_topk_rejects_bad_sizes():
    from zen_repro_amd import _lib

    L = _lib.lib()
    grad = torch.ones(1024, dtype=torch.float32, device="cuda")
    thr = torch.zeros(2, dtype=torch.int32, device="cuda")
    stream = _lib.stream_of(grad.device)
    too_many = 1 << 31  # beyond ZEN_TOPK_STATIC_MAX_N; rejected on the host, nothing is launched
    assert L.zen_topk_threshold_static(_lib.ptr(grad), _lib.F32, too_many, 1, _lib.ptr(thr), stream) == _lib.EINVAL
    assert b"ZEN_TOPK_STATIC_MAX_N" in L.zen_last_error()
    assert L.zen_topk_threshold_static(_lib.ptr(grad), _lib.F32, 1024, 0, _lib.ptr(thr), stream) == _lib.EINVAL
    assert L.zen_topk_threshold_static(_lib.ptr(grad), _lib.F32, 1024, 1025, _lib.ptr(thr), stream) == _lib.EINVAL
    assert L.zen_topk_threshold_static(None, _lib.F32, 1024, 1, _lib.ptr(thr), stream) == _lib.EINVAL
    torch.cuda.synchronize()
