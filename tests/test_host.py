"""CPU-only checks: the C-ABI library loads and exports what include/zen_hip.h
declares, argument validation happens on the host, the host-side helpers and
the synthetic workloads behave, and the CPU baseline restatement agrees with
the oracle.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    from zen_repro_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    return _lib.lib()


def test_every_declared_symbol_is_exported(L):
    header = open(os.path.join(ROOT, "include", "zen_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    names = set(re.findall(r"\b(zen_[a-z0-9_]+)\s*\(", header))
    assert len(names) >= 20
    raw = ctypes.CDLL(os.path.join(ROOT, "zen_repro_amd", "csrc", "libzen_hip.so"))
    for n in sorted(names):
        assert hasattr(raw, n), f"{n} declared in zen_hip.h but not exported"
    from zen_repro_amd import _lib

    declared = int(re.search(r"#define\s+ZEN_ABI_VERSION\s+(\d+)", header).group(1))
    assert L.zen_abi_version() == declared == _lib.ABI_VERSION


def test_workspace_queries_are_host_only(L):
    assert L.zen_topk_threshold_workspace() >= 2048 * 4
    a, b = L.zen_sort_pairs_workspace(1000), L.zen_sort_pairs_workspace(1 << 20)
    assert 0 < a < b
    assert L.zen_merge_workspace(1 << 20, 1 << 30) >= 4 * 4 * (1 << 20)
    assert L.zen_load_balance_workspace(1 << 24, 1 << 24, 1, 1 << 18, 16) >= 6 * 4 * (1 << 18)
    assert L.zen_select_workspace(1 << 24, 1) >= (1 << 24) // 8192 * 8
    assert L.zen_mapping_workspace(1 << 20, 8) >= 16 * (1 << 20)
    assert L.zen_decode_dense_workspace(1000, 5000) > L.zen_merge_workspace(1000, 5000)


def test_path_selection_is_host_only(L):
    """Which implementation a call takes depends on sizes alone."""
    # c3: 743 M bf16 elements, top 0.5 %, 16 partitions -> bucket slabs; the same as fp32 too
    from zen_repro_amd import _lib

    slabs = _lib.MODE_SLABS  # without it the answer depends on the device: 3 (wide buckets) on a chip of 256 compute units
    assert L.zen_load_balance_path(743440384, 743440384, 1, 4650000, 16, 3717201, slabs) == 2
    assert L.zen_load_balance_path(743440384, 743440384, 0, 4650000, 16, 3717201, slabs) == 2
    assert L.zen_load_balance_path(743440384, 743440384, 0, 4650000, 16, 0, slabs) == 2
    assert L.zen_load_balance_path(743440384, 743440384, 1, 4650000, 16, 3717201, 0) in (2, 3)
    assert L.zen_load_balance_path(743440384, 743440384, 1, 4650000, 16, 3717201, 1) == 0   # general mode
    assert L.zen_load_balance_path(1 << 20, 1 << 20, 1, 1 << 14, 4, 0, 0) == 1             # small table
    assert L.zen_load_balance_path(1 << 24, 1 << 24, 1, 1 << 24, 16, 0, 0) == 1            # capacity = everything
    assert L.zen_merge_path(3717200, 743440384, slabs) == 2
    assert L.zen_merge_path(3717200, 743440384, 0) in (2, 3)
    assert L.zen_merge_path(3717200, 743440384, 1) == 0
    assert L.zen_merge_path(1000, 1 << 20, 0) == 0


def test_bad_arguments_are_rejected_on_the_host(L):
    from zen_repro_amd import _lib

    one = ctypes.c_void_p(256)  # never dereferenced: validation comes first
    assert L.zen_hash_index(None, 16, 4, None) == _lib.EINVAL
    assert L.zen_hash_index(one, 3, 4, None) == _lib.EINVAL          # n < P
    assert L.zen_hash_index(one, 1 << 31, 4, None) == _lib.EINVAL    # n >= 2^31
    assert L.zen_hash_index(one, 16, 0, None) == _lib.EINVAL
    assert b"partitions" in L.zen_last_error()
    # table not a multiple of P, bad dtype, oversize
    assert L.zen_sparse_balance(one, 1, 64, one, 62, one, 4, one, 4, 3, one, None) == _lib.EINVAL
    assert L.zen_sparse_balance(one, 7, 64, one, 64, one, 4, one, 4, 3, one, None) == _lib.EINVAL
    assert L.zen_sparse_balance(one, 1, 1 << 31, one, 64, one, 4, one, 4, 3, one, None) == _lib.EINVAL
    assert L.zen_topk_threshold(one, 0, 100, 0, one, one, 1 << 20, None) == _lib.EINVAL    # k < 1
    assert L.zen_topk_threshold(one, 0, 100, 101, one, one, 1 << 20, None) == _lib.EINVAL  # k > n
    assert L.zen_topk_threshold(one, 0, 100, 5, one, one, 16, None) == _lib.EWORKSPACE
    assert L.zen_load_balance(one, 1, 1024, 1022, 4, 3, None, 0, None, one, one, 64, one, one, 0, one, 1 << 30, one, None) == _lib.EINVAL
    assert L.zen_load_balance(one, 1, 1024, 1024, 4, 3, one, 5, None, one, one, 64, one, one, 0, one, 1 << 30, one, None) == _lib.EINVAL  # thr and k
    assert L.zen_load_balance(one, 1, 1024, 1024, 4, 3, None, 0, None, one, one, 64, one, one, 0, one, 16, one, None) == _lib.EWORKSPACE
    assert L.zen_merge(one, 0, one, 0, 10, 0, one, 0, one, 10, one, 0, one, 1 << 20, one, None) == _lib.EINVAL  # dense_n
    assert L.zen_merge(one, 0, one, 0, 10, 100, one, 0, one, 10, one, 7, one, 1 << 20, one, None) == _lib.EINVAL  # mode
    assert L.zen_merge(one, 0, one, 0, 10, 100, one, 0, one, 10, one, 0, one, 16, one, None) == _lib.EWORKSPACE
    assert L.zen_sort_pairs(one, one, 100, None, 33, one, 1 << 20, one, None) == _lib.EINVAL
    # zen_encode_merge: a next call of its own size must take a path that keeps a sample in its table
    n = 1 << 24
    a = _lib.EncodeMergeArgs(
        256, 1, n, n, 16, 3, None, n // 200, None, 256, 256, n // 100, 256, 256, _lib.MODE_FAST | _lib.MODE_SLABS, 256,
        1 << 40, 256, 256, 0, 256, 1000, n, 256, 0, 256, 1000, 256, _lib.MODE_FAST, 256, 1 << 40, 256, None, None,
        256, 20, 4096, 4096, 64, 256)
    assert L.zen_encode_merge(ctypes.byref(a)) == _lib.EINVAL and b"next call" in L.zen_last_error()
    assert L.zen_encode_merge(None) == _lib.EINVAL
    with pytest.raises(ValueError):
        _lib.check(_lib.EINVAL, "x")
    with pytest.raises(RuntimeError):
        _lib.check(_lib.EHIP, "x")


def test_wrappers_assert_like_the_reference():
    import zen_repro_amd as zen

    g = torch.zeros(64, dtype=torch.bfloat16)
    mem = torch.zeros(64, dtype=torch.int32)
    with pytest.raises(AssertionError):  # extensions/cuda/functions.py:5: CPU tensors are refused
        zen.sparse_balance(g, mem, mem[:4], 4, 3)
    with pytest.raises(AssertionError):
        zen.hash_index(mem, 4)


def test_missing_library_fails_loudly(monkeypatch):
    from zen_repro_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libzen_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.lib()


def test_table_sizes_follow_the_reference(oracle):
    from zen_repro_amd.tensor_load_balance import TensorPartition

    tp = TensorPartition.__new__(TensorPartition)
    for n, P, scale in [(1 << 20, 4, 1), (1003, 4, 1), (5000, 4, 1.5), (743440384, 16, 1), (100, 64, 2)]:
        tp.partitions, tp.memory_scale = P, scale
        assert tp.table_sizes(n) == oracle.table_sizes(n, P, scale)
        m, s = tp.table_sizes(n)
        assert m % P == 0 and s % P == 0 and s == n // P // 10 * P


def test_consecutive_views_are_recognised():
    from zen_repro_amd.comm import _as_one_buffer

    buf = torch.arange(50, dtype=torch.int32)
    whole = _as_one_buffer([buf[:10], buf[10:30], buf[30:]])
    assert whole is not None and whole.data_ptr() == buf.data_ptr() and whole.numel() == 50
    assert _as_one_buffer([buf[:10], buf[11:30]]) is None
    assert _as_one_buffer([buf[:10], torch.arange(5, dtype=torch.int32)]) is None
    assert _as_one_buffer([buf[:10], buf[10:20].long()]) is None


def test_workload_hash_matches_oracle(oracle):
    from zen_repro_amd import workloads

    rng = np.random.default_rng(0)
    for m in (1 << 20, 743440384, 1003, (1 << 31) - 1):
        t = rng.integers(0, m, 3000)
        got = workloads.hash_slot(torch.from_numpy(t), m).numpy()
        want = np.array([oracle.hash32(int(x)) % m for x in t])
        assert np.array_equal(got, want)


def test_peer_payloads_have_the_stated_shape(oracle):
    from zen_repro_amd import workloads

    cfg, g = workloads.make("c1", device="cpu", seed=0)
    assert g.numel() == 1 << 20 and g.dtype == torch.float32 and cfg.k == 10485
    per = 2600
    idx_l, val_l, flat_idx, flat_val = workloads.peer_payloads(cfg, per, device="cpu")
    assert len(idx_l) == 4 and flat_idx.numel() == 4 * per and flat_idx.dtype == torch.int32
    part = oracle.hash_index(cfg.n, cfg.partitions)
    sets = [set(i.tolist()) for i in idx_l]
    for i, s in zip(idx_l, sets):
        assert len(s) == per and (part[i.numpy()] == 0).all()
        slots = workloads.hash_slot(i.long(), cfg.n)
        assert (slots[1:] >= slots[:-1]).all()  # slot order, as an encoder emits
    common = set.intersection(*sets)
    assert len(common) == int(per * cfg.overlap)  # the shared pool, and nothing else
    assert idx_l[1].data_ptr() == flat_idx.data_ptr() + per * 4


@pytest.mark.parametrize("name,shrink", [("c2", 64), ("c3", 256), ("c4", 1024), ("c5", 64)])
def test_workloads_small(name, shrink):
    from zen_repro_amd import workloads

    cfg, g = workloads.make(name, device="cpu", seed=0, shrink=shrink)
    assert g.numel() == cfg.n and cfg.n % cfg.partitions == 0 and g.dtype == cfg.dtype
    nz = int(torch.count_nonzero(g))
    if name == "c3":
        assert nz > 0.99 * cfg.n and cfg.k == int(cfg.n * 0.005)
    elif name == "c2":
        # two gradient buckets: the embedding (row-sparse, taken as it is) and the dense rest (top 1 % by the path)
        emb, rest = workloads.buckets(cfg)
        assert emb.offset == 0 and rest.offset == emb.n and emb.n + rest.n == cfg.n
        assert emb.k == 0 and rest.k == rest.n // 100
        assert emb.n % cfg.partitions == 0 and rest.n % cfg.partitions == 0
        assert 0 < int(torch.count_nonzero(g[:emb.n])) < 0.05 * emb.n
        assert int(torch.count_nonzero(g[emb.n:])) > 0.99 * rest.n
    else:
        assert 0 < nz < 0.05 * cfg.n
        assert workloads.buckets(cfg) == [cfg]
    if name == "c4":
        idx = torch.nonzero(g, as_tuple=True)[0]
        h, r = workloads.bucket_imbalance(idx, cfg.n, cfg.partitions)
        assert h < 1.2 < r  # the hash flattens what range partitioning piles up


def test_cpu_baseline_restatement_agrees_with_oracle(oracle):
    from oracle import torch_path
    from zen_repro_amd import workloads

    cfg, g = workloads.make("c3", device="cpu", seed=0, shrink=1024)
    per = cfg.k // cfg.partitions
    idx_l, val_l, flat_idx, flat_val = workloads.peer_payloads(cfg, per, device="cpu")
    times, (indices, values, splits, status, m_idx, m_val) = torch_path.timed_pass(g, cfg.k, cfg.partitions, idx_l, val_l)
    bits = g.view(torch.int16).numpy().view(np.uint16)
    key = oracle.kth_key(bits, cfg.k)
    masked, _ = oracle.mask_dense(bits, key)
    idx_o, val_o, splits_o, st = oracle.load_balance(masked, cfg.partitions)
    assert status == st == 0
    assert np.array_equal(torch.cat(indices).numpy(), idx_o)
    assert np.array_equal(torch.cat(values).view(torch.int16).numpy().view(np.uint16), val_o)
    assert np.array_equal(splits.numpy(), splits_o)
    # merge: torch's CPU kernel sums bf16 in fp32 and rounds once
    f32 = oracle.decode(flat_idx.numpy(), flat_val.view(torch.int16).numpy().view(np.uint16), cfg.n, "f32acc")
    mi, mv = oracle.encode(oracle.f32_to_bf16_bits(f32))
    assert np.array_equal(m_idx.numpy(), mi)
    assert np.array_equal(m_val.view(torch.int16).numpy().view(np.uint16), mv)
    assert set(times) == {"select", "partition", "merge"}


def test_ranges_are_off_by_default_and_cost_nothing():
    """The named ranges (the reference's nvtx names) are plain null contexts unless switched on."""
    import contextlib

    from zen_repro_amd import _lib

    was = _lib._ranges_on
    try:
        _lib.ranges_enable(False)
        assert isinstance(_lib.annotate("load_balance"), contextlib.nullcontext)
        with _lib.annotate("load_balance"), _lib.annotate("decode_sparse_tensors"):
            pass
        _lib.ranges_enable(True)
        assert not isinstance(_lib.annotate("load_balance"), contextlib.nullcontext)
    finally:
        _lib.ranges_enable(was)
