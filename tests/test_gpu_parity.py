"""Parity of the HIP library against the CPU oracle on seeded inputs.  Every
test goes through libzen_hip.so's C ABI (directly or via the package's thin
wrappers).  Bar: bit-exact for indices, slots, order and bit-copied values;
merged sums bit-exact against the fp32 sequential oracle (same order of adds)
and within 1e-6 relative of the fp64 truth."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import make_grad, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def zen():
    import zen_repro_amd
    from zen_repro_amd import _lib

    _lib.lib()
    assert torch.cuda.is_available()
    return zen_repro_amd


# ------------------------------------------------------------------ sort


@pytest.mark.parametrize("count", [1, 63, 64, 65, 1000, 4095, 4096, 4097, 70001, 1 << 20])
@pytest.mark.parametrize("bits", [1, 8, 9, 17, 30, 32])
def test_sort_pairs_is_stable_sort(zen, count, bits):
    from zen_repro_amd import _lib

    rng = np.random.default_rng(count * 131 + bits)
    hi = (1 << bits) - 1
    # few distinct keys on purpose: stability must show
    keys = rng.integers(0, min(hi, 500) + 1, count, dtype=np.uint64).astype(np.uint32)
    if bits >= 9:
        keys = (keys * np.uint32(max(1, hi // 501))).astype(np.uint32)
    vals = np.arange(count, dtype=np.uint32)
    dk = to_dev(keys.view(np.int32))
    dv = to_dev(vals.view(np.int32))
    L = _lib.lib()
    ws = torch.empty(L.zen_sort_pairs_workspace(count), dtype=torch.uint8, device="cuda")
    st = torch.zeros(1, dtype=torch.int32, device="cuda")
    rc = L.zen_sort_pairs(_lib.ptr(dk), _lib.ptr(dv), count, None, bits, _lib.ptr(ws), ws.numel(),
                          _lib.ptr(st), _lib.stream_of(dk.device))
    assert rc == 0 and st.item() == 0
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(to_np(dk).view(np.uint32), keys[order])
    assert np.array_equal(to_np(dv).view(np.uint32), vals[order])


def test_sort_pairs_device_count(zen):
    from zen_repro_amd import _lib

    cap, live = 50000, 12345
    rng = np.random.default_rng(9)
    keys = rng.integers(0, 1 << 20, cap, dtype=np.uint64).astype(np.uint32)
    vals = np.arange(cap, dtype=np.uint32)
    dk, dv = to_dev(keys.view(np.int32)), to_dev(vals.view(np.int32))
    cnt = torch.tensor([live], dtype=torch.int32, device="cuda")
    L = _lib.lib()
    ws = torch.empty(L.zen_sort_pairs_workspace(cap), dtype=torch.uint8, device="cuda")
    st = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert L.zen_sort_pairs(_lib.ptr(dk), _lib.ptr(dv), cap, _lib.ptr(cnt), 20, _lib.ptr(ws), ws.numel(),
                            _lib.ptr(st), _lib.stream_of(dk.device)) == 0
    order = np.argsort(keys[:live], kind="stable")
    assert np.array_equal(to_np(dk).view(np.uint32)[:live], keys[:live][order])
    assert np.array_equal(to_np(dv).view(np.uint32)[:live], vals[:live][order])
    assert np.array_equal(to_np(dk).view(np.uint32)[live:], keys[live:])  # tail untouched


@pytest.mark.parametrize("count,sentinel,live,distinct", [
    (1 << 16, 1 << 20, None, None), (70001, 743440384, None, None), (1 << 20, (1 << 30) + 7, None, None),
    (3800000, 743440384, None, None), (1 << 20, 5000011, 300000, None), (1 << 18, 1 << 24, None, 700),
])
def test_bucket_sort_pairs_is_stable_sort(zen, count, sentinel, live, distinct):
    """Evenly spread keys below the sentinel, some at or above it; duplicates keep their arrival order."""
    from zen_repro_amd import _lib

    rng = np.random.default_rng(count + sentinel % 1000)
    keys = rng.integers(0, sentinel, count, dtype=np.uint64).astype(np.uint32)
    if distinct:  # many equal keys
        keys = (keys // np.uint32(sentinel // distinct) * np.uint32(sentinel // distinct)).astype(np.uint32)
    tail = rng.random(count) < 0.05
    keys[tail] = sentinel + (rng.integers(0, 2, int(tail.sum())).astype(np.uint32))
    vals = np.arange(count, dtype=np.uint32)
    dk, dv = to_dev(keys.view(np.int32)), to_dev(vals.view(np.int32))
    n = count if live is None else live
    cnt = None if live is None else torch.tensor([live], dtype=torch.int32, device="cuda")
    L = _lib.lib()
    assert L.zen_bucket_sort_fits(count, sentinel)
    ws = torch.empty(L.zen_sort_pairs_workspace(count), dtype=torch.uint8, device="cuda")
    st = torch.zeros(1, dtype=torch.int32, device="cuda")
    rc = L.zen_bucket_sort_pairs(_lib.ptr(dk), _lib.ptr(dv), count, _lib.ptr(cnt), sentinel, _lib.ptr(ws),
                                 ws.numel(), _lib.ptr(st), _lib.stream_of(dk.device))
    assert rc == 0 and st.item() == 0
    below = np.flatnonzero(keys[:n] < sentinel)
    order = below[np.argsort(keys[below], kind="stable")]
    got_k, got_v = to_np(dk).view(np.uint32), to_np(dv).view(np.uint32)
    assert np.array_equal(got_k[:len(order)], keys[order])
    assert np.array_equal(got_v[:len(order)], vals[order])
    rest = np.flatnonzero(keys[:n] >= sentinel)  # behind, as a set, each still with its own value
    assert np.array_equal(np.sort(got_v[len(order):n]), rest)
    assert np.array_equal(got_k[len(order):n], keys[got_v[len(order):n]])
    assert np.array_equal(got_k[n:], keys[n:])


def test_bucket_sort_pairs_crowded_range_asks_for_retry(zen):
    from zen_repro_amd import _lib

    count, sentinel = 1 << 17, 1 << 24
    keys = np.random.default_rng(5).integers(0, 20000, count, dtype=np.uint64).astype(np.uint32)  # one key range
    dk, dv = to_dev(keys.view(np.int32)), to_dev(np.arange(count, dtype=np.int32))
    L = _lib.lib()
    ws = torch.empty(L.zen_sort_pairs_workspace(count), dtype=torch.uint8, device="cuda")
    st = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert L.zen_bucket_sort_pairs(_lib.ptr(dk), _lib.ptr(dv), count, None, sentinel, _lib.ptr(ws), ws.numel(),
                                   _lib.ptr(st), _lib.stream_of(dk.device)) == 0
    assert st.item() == _lib.STAT_RETRY
    assert not L.zen_bucket_sort_fits(1000, sentinel) and not L.zen_bucket_sort_fits(count, 1000)
    assert L.zen_bucket_sort_pairs(_lib.ptr(dk), _lib.ptr(dv), 1000, None, sentinel, _lib.ptr(ws), ws.numel(),
                                   _lib.ptr(st), _lib.stream_of(dk.device)) == _lib.EINVAL


# ------------------------------------------------------------------ hash


@pytest.mark.parametrize("n,P", [(1 << 20, 4), (1003, 4), (38597376 // 16, 16), (999983, 7), (64, 64)])
def test_hash_index(zen, oracle, n, P):
    idx = torch.full((n,), -7, dtype=torch.int32, device="cuda")
    zen.hash_index(idx, P)
    assert np.array_equal(to_np(idx), oracle.hash_index(n, P))


def test_hash_index_rejects(zen):
    with pytest.raises(ValueError):
        zen.hash_index(torch.zeros(3, dtype=torch.int32, device="cuda"), 4)
    with pytest.raises(AssertionError):
        zen.hash_index(torch.zeros(8, dtype=torch.int64, device="cuda"), 4)


@pytest.mark.parametrize("n,P", [(1 << 16, 8), (1003, 4), (300000, 16)])
def test_calculate_mapping(zen, oracle, n, P):
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P), None, None)
    got = lba.calculate_mapping(n)
    want = oracle.mapping(n, P)
    assert len(got) == P
    for g, w in zip(got, want):
        assert g.dtype == torch.int64 and np.array_equal(to_np(g), w)


# ---------------------------------------------------------------- insert

INSERT_CASES = [
    (4096, 4, 0.01, 1), (4096, 4, 0.3, 1), (1 << 16, 16, 0.05, 1), (1 << 16, 8, 0.5, 1),
    (100000, 5, 0.2, 1), (1 << 18, 32, 0.01, 1), (60000, 6, 0.35, 2), (50000, 4, 0.25, 1.5),
    (1000000, 4, 0.4, 1),  # rehash 1: > 8192 serial entries per partition (sorted in global memory)
]


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("rehash", [1, 2, 3])
@pytest.mark.parametrize("n,P,density,scale", INSERT_CASES)
def test_sparse_balance_tables_byte_identical(zen, oracle, n, P, density, scale, rehash, dtype):
    g = make_grad(oracle, n, density, dtype, seed=n + P)
    g[0] = g[g != 0][0] if (g != 0).any() else 1  # index 0 nonzero: must never be stored
    m, sn = oracle.table_sizes(n, P, scale)
    mem_o, ser_o, off_o, st_o = oracle.sparse_balance(g, m, sn, P, rehash)
    d = to_dev(g)
    mem = torch.zeros(m, dtype=torch.int32, device="cuda")
    ser = torch.zeros(sn, dtype=torch.int32, device="cuda")
    assert zen.sparse_balance(d, mem, ser, P, rehash) is None  # like the reference's
    pending = zen.last_status()
    assert np.array_equal(to_np(pending.offsets), off_o)
    assert int(pending.status.item()) == st_o
    assert np.array_equal(to_np(mem), mem_o)
    if st_o == 0:
        assert np.array_equal(to_np(ser), ser_o)


def test_sparse_balance_overflow_is_flagged_not_oob(zen, oracle):
    n, P = 40000, 4
    g = np.ones(n, np.float32)
    m, sn = oracle.table_sizes(n, P)
    mem_o, _, off_o, st_o = oracle.sparse_balance(g, m, sn, P, 1)
    assert st_o == oracle.SERIAL_OVERFLOW
    mem = torch.zeros(m, dtype=torch.int32, device="cuda")
    ser = torch.zeros(sn + 64, dtype=torch.int32, device="cuda")  # guard zone behind the table
    assert zen.sparse_balance(to_dev(g), mem, ser[:sn], P, 1) is None  # like the reference's
    pending = zen.last_status()
    assert int(pending.status.item()) & 1
    with pytest.raises(RuntimeError):
        pending.check()
    assert np.array_equal(to_np(mem), mem_o)
    assert np.array_equal(to_np(pending.offsets), off_o)
    assert not to_np(ser)[sn:].any()


def test_sparse_balance_argument_errors(zen):
    g = torch.zeros(64, dtype=torch.bfloat16, device="cuda")
    mem = torch.zeros(64, dtype=torch.int32, device="cuda")
    ser = torch.zeros(4, dtype=torch.int32, device="cuda")
    with pytest.raises(AssertionError):
        zen.sparse_balance(g.cpu(), mem, ser, 4, 3)
    with pytest.raises(AssertionError):
        zen.sparse_balance(g.half(), mem, ser, 4, 3)
    with pytest.raises(AssertionError):
        zen.sparse_balance(g, mem.long(), ser, 4, 3)
    with pytest.raises(RuntimeError):
        zen.sparse_balance(g[::2], mem, ser, 4, 3)
    with pytest.raises(ValueError):
        zen.sparse_balance(g, mem[:62], ser, 4, 3)  # table not a multiple of P


def test_reference_style_compaction_over_tables(zen, oracle):
    # balance_sparse_tensor + get_sub_sparse_tensors, the reference's two-step route
    n, P = 100000, 5
    g = make_grad(oracle, n, 0.2, "bf16", seed=77)
    tp = zen.TensorPartition(P, 1, 3)
    d = to_dev(g)
    mem, ser = tp.balance_sparse_tensor(d)
    i1, v1, s1 = tp.get_sub_sparse_tensors(d, mem)
    i2, v2, s2 = tp.get_sub_sparse_tensors(d, ser)
    idx_o, val_o, splits_o, st = oracle.load_balance(g, P, 1, 3)
    assert st == 0 and s2.sum().item() > 0  # the serial region is in use at this density
    got_i = np.concatenate([np.concatenate([to_np(a), to_np(b)]) for a, b in zip(i1, i2)])
    got_v = np.concatenate([np.concatenate([to_np(a), to_np(b)]) for a, b in zip(v1, v2)])
    assert np.array_equal(got_i, idx_o) and np.array_equal(got_v, val_o)
    assert np.array_equal(to_np(s1 + s2), splits_o)


# ---------------------------------------------------------------- select


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("n", [5000, 1 << 16, 1 << 20, 3 * (1 << 20) + 17])
def test_topk_threshold(zen, oracle, n, dtype):
    g = make_grad(oracle, n, 1.0, dtype, seed=n)
    d = to_dev(g)
    for k in (1, 2, n // 200, n // 100, n // 3, n):
        thr = zen.topk_threshold(d, k)
        key, count = (int(x) & 0xFFFFFFFF for x in to_np(thr))
        assert key == oracle.kth_key(g, k), (n, dtype, k)
        keys = (g & 0x7FFF) if dtype == "bf16" else (g.view(np.uint32) & 0x7FFFFFFF)
        assert count == int((keys >= key).sum())


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("n,s", [(5000, 50), (1 << 20, 10486), (3 * (1 << 20) + 17, 1 << 20), (1 << 16, 1 << 18)])
def test_sample_threshold(zen, oracle, n, s, dtype):
    """The threshold over tensor[sample_index] (train.py:78-82) in one call: positions drawn with replacement
    (more positions than elements in the last case), against the k-th largest key of the gathered sample."""
    import importlib

    C = importlib.import_module("zen_repro_amd.compress")
    from zen_repro_amd import _lib

    g = make_grad(oracle, n, 1.0, dtype, seed=n + s)
    d = to_dev(g)
    rng = np.random.default_rng(s)
    at = rng.integers(0, n, s)
    at[0], at[-1] = 0, n - 1
    at_dev = torch.from_numpy(at).cuda()
    keys = (g & 0x7FFF) if dtype == "bf16" else (g.view(np.uint32) & 0x7FFFFFFF)
    for k in (1, max(1, s // 100), s // 2 + 1, s):
        thr, status = C.sample_threshold(d, at_dev, k)
        key, count = (int(x) & 0xFFFFFFFF for x in to_np(thr))
        assert int(status) == 0
        assert key == oracle.kth_key(g[at], k), (n, s, dtype, k)
        assert count == int((keys[at] >= key).sum())
    # an unaligned view of the tensor, and a position outside it: flagged, counted as a zero
    thr, status = C.sample_threshold(d[1:], at_dev[: s // 2].clamp(max=n - 2), max(1, s // 200))
    assert int(status) == 0
    assert int(to_np(thr)[0]) & 0xFFFFFFFF == oracle.kth_key(g[1:][np.minimum(at[: s // 2], n - 2)], max(1, s // 200))
    bad = at.copy()
    bad[s // 3] = n
    bad[s // 2] = -1
    thr, status = C.sample_threshold(d, torch.from_numpy(bad).cuda(), max(1, s // 100))
    assert int(status) == _lib.STAT_BAD_INDEX
    sample = g[np.clip(bad, 0, n - 1)].copy()
    sample[[s // 3, s // 2]] = 0
    assert int(to_np(thr)[0]) & 0xFFFFFFFF == oracle.kth_key(sample, max(1, s // 100))


def test_topk_threshold_heavy_ties_and_zeros(zen, oracle):
    n = 1 << 18
    g = np.zeros(n, np.float32)
    g[::7] = 0.5
    g[::11] = -0.5
    g[5::13] = 2.0
    d = to_dev(g)
    for k in (1, 1000, int((g != 0).sum()), n):
        thr = zen.topk_threshold(d, k)
        assert int(to_np(thr)[0]) == oracle.kth_key(g, k)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_compress_masked_copy(zen, oracle, dtype):
    import importlib

    C = importlib.import_module("zen_repro_amd.compress")

    n = (1 << 18) + 5
    g = make_grad(oracle, n, 1.0, dtype, seed=5)
    d = to_dev(g)
    k = n // 100
    thr = C.topk_threshold(d, k)
    want, kept = oracle.mask_dense(g, oracle.kth_key(g, k))
    assert np.array_equal(to_np(C.mask_below(d, thr)), want)
    # unaligned views take the scalar path
    got = C.mask_below(d[1:], C.topk_threshold(d[1:], k))
    want1, _ = oracle.mask_dense(g[1:], oracle.kth_key(g[1:], k))
    assert np.array_equal(to_np(got), want1)
    # the reference-shaped entry: caller-supplied sample positions
    rng = np.random.default_rng(1)
    sample = rng.integers(0, n, -(-n // 100))
    out = zen.compress(5, d, torch.from_numpy(sample).cuda())
    ks = len(sample) * 5 // 100
    want2, _ = oracle.mask_dense(g, oracle.kth_key(g[sample], ks))
    assert np.array_equal(to_np(out), want2)
    small = d[:4096]
    assert zen.compress(1, small) is small  # train.py:77-78
    # threshold over the samples of several ranks (train.py:56-73); the exchange is the caller's
    others = [make_grad(oracle, n, 1.0, dtype, seed=6 + r) for r in range(3)]
    everyone = np.concatenate([g[sample]] + [o[sample] for o in others])
    gather = lambda mine: torch.cat([mine] + [to_dev(o)[torch.from_numpy(sample).cuda()] for o in others])  # noqa: E731
    out = zen.compress_with_allgather(5, d, zen.LocalGroup(4), torch.from_numpy(sample).cuda(), gather)
    want3, _ = oracle.mask_dense(g, oracle.kth_key(everyone, len(everyone) * 5 // 100))
    assert np.array_equal(to_np(out), want3)
    assert np.array_equal(to_np(zen.compress_with_allgather(5, d, zen.LocalGroup(1), torch.from_numpy(sample).cuda())),
                          want2)
    with pytest.raises(RuntimeError):
        zen.compress_with_allgather(5, d, zen.LocalGroup(4))


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("n,density", [(1, 1.0), (100, 0.5), (8192, 0.0), (8193, 1.0), (1 << 20, 0.01),
                                       (5 * (1 << 20) + 3, 0.3), (40 * 1000 * 1000 + 3, 0.5),
                                       (70 * 1000 * 1000, 0.004)])
def test_encode_sparse_tensor(zen, oracle, n, density, dtype):
    g = make_grad(oracle, n, density, dtype, seed=n * 3 + 1)
    if n > 4:
        g[3] = 0x8000 if dtype == "bf16" else -0.0  # negative zero is a zero
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(4), None, None)
    idx, val = lba.encode_sparse_tensor(to_dev(g))
    idx_o, val_o = oracle.encode(g)
    assert idx.dtype == torch.int64
    assert np.array_equal(to_np(idx), idx_o) and np.array_equal(to_np(val), val_o)
    if n > 64:
        off = to_dev(g)[3:]
        i2, v2 = lba.encode_sparse_tensor(off)
        io, vo = oracle.encode(g[3:])
        assert np.array_equal(to_np(i2), io) and np.array_equal(to_np(v2), vo)


def test_select_capacity_flag(zen, oracle):
    from zen_repro_amd import _lib

    n = 100000
    g = make_grad(oracle, n, 0.5, "f32", seed=2)
    d = to_dev(g)
    L = _lib.lib()
    cap = 1000
    oi = torch.full((cap + 16,), -1, dtype=torch.int32, device="cuda")
    ov = torch.zeros(cap + 16, dtype=torch.float32, device="cuda")
    cnt = torch.zeros(1, dtype=torch.int64, device="cuda")
    st = torch.zeros(1, dtype=torch.int32, device="cuda")
    ws = torch.empty(L.zen_select_workspace(n, 0), dtype=torch.uint8, device="cuda")
    assert L.zen_select(_lib.ptr(d), 0, n, None, _lib.ptr(oi), 0, _lib.ptr(ov), cap, _lib.ptr(cnt),
                        _lib.ptr(ws), ws.numel(), _lib.ptr(st), _lib.stream_of(d.device)) == 0
    io, _ = oracle.encode(g)
    assert cnt.item() == len(io) and st.item() == _lib.STAT_CAPACITY
    assert np.array_equal(to_np(oi)[:cap], io[:cap].astype(np.int32))
    assert (to_np(oi)[cap:] == -1).all()


# ---------------------------------------------------------- load balance

LB_CASES = [
    (8192, 4, 0.01, 1, 3), (1 << 16, 16, 0.005, 1, 3), (1 << 16, 8, 0.3, 1, 3), (1 << 18, 32, 0.05, 1, 2),
    (100000, 5, 0.4, 1, 1), (1 << 20, 16, 0.01, 1, 3), (60000, 6, 0.2, 2, 3), (50000, 4, 0.25, 1.5, 3),
    (1 << 20, 64, 0.001, 1, 3),
]


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("n,P,density,scale,rehash", LB_CASES)
def test_load_balance_bit_exact(zen, oracle, n, P, density, scale, rehash, dtype, mode):
    """mode 0: sort-based owner resolution; mode 1: owner table like the reference."""
    g = make_grad(oracle, n, density, dtype, seed=n ^ P)
    g[0] = 0x3F80 if dtype == "bf16" else 1.0
    idx_o, val_o, splits_o, st_o = oracle.load_balance(g, P, scale, rehash)
    tp = zen.TensorPartition(P, scale, rehash)
    d = to_dev(g)
    for rep in range(2):  # the second call reuses the (re-zeroed) owner table
        if st_o:
            with pytest.raises(RuntimeError):
                tp.load_balance(d, mode=mode)
            continue
        indices, values, splits = tp.load_balance(d, mode=mode)
        assert np.array_equal(to_np(splits), splits_o)
        assert np.array_equal(np.concatenate([to_np(i) for i in indices]), idx_o)
        assert np.array_equal(np.concatenate([to_np(v) for v in values]), val_o)
        assert indices[0].dtype == torch.int32 and values[0].dtype == d.dtype
    m, _ = oracle.table_sizes(n, P, scale)
    assert not tp._table(d.device, m).any()  # left empty for the next call


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_topk_then_load_balance(zen, oracle, dtype):
    n, P = 1 << 20, 16
    g = make_grad(oracle, n, 1.0, dtype, seed=123)
    k = n // 200
    key = oracle.kth_key(g, k)
    masked, kept = oracle.mask_dense(g, key)
    idx_o, val_o, splits_o, st_o = oracle.load_balance(masked, P, 1, 3)
    d = to_dev(g)
    thr = zen.topk_threshold(d, k)
    tp = zen.TensorPartition(P, 1, 3)
    indices, values, splits = tp.load_balance(d, thr=thr, capacity=2 * k + 1024)
    assert st_o == 0
    assert np.array_equal(to_np(splits), splits_o)
    assert np.array_equal(np.concatenate([to_np(i) for i in indices]), idx_o)
    assert np.array_equal(np.concatenate([to_np(v) for v in values]), val_o)
    part = oracle.hash_index(n, P)
    for p, i in enumerate(indices):
        assert (part[to_np(i)] == p).all()


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("dtype,shape", [("bf16", "flat"), ("f32", "flat"), ("bf16", "columns")])
def test_load_balance_fused_topk(zen, oracle, dtype, shape, mode):
    """k-largest selection inside the call: the one-pass sampled route (mode 0,
    tensors of 2^24 elements and more) and the exact full-histogram route must
    both equal oracle top-k followed by oracle load balance."""
    from zen_repro_amd import _lib

    n, P = (1 << 25) + 4096, 16
    rng = np.random.default_rng(11)
    x = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    if shape == "columns":  # a few hot columns of a 4096-wide matrix: a stride-aligned sample would be fooled
        x.reshape(-1, 4096)[:, ::509] *= 50.0
    g = oracle.f32_to_bf16_bits(x) if dtype == "bf16" else x
    k = n // 200
    key = oracle.kth_key(g, k)
    masked, kept = oracle.mask_dense(g, key)
    idx_o, val_o, splits_o, st_o = oracle.load_balance(masked, P, 1, 3)
    assert st_o == 0
    tp = zen.TensorPartition(P, 1, 3)
    d = to_dev(g)
    thr_out = torch.zeros(2, dtype=torch.int32, device="cuda")
    oi, ov, splits, status = tp.load_balance_flat(d, capacity=int(1.3 * k) + 4096, k=k, mode=mode, thr_out=thr_out)
    assert status.item() == 0
    assert to_np(thr_out).tolist() == [key, kept]
    assert np.array_equal(to_np(splits), splits_o)
    total = int(splits_o.sum())
    assert np.array_equal(to_np(oi)[:total], idx_o)
    assert np.array_equal(to_np(ov)[:total], val_o)
    if mode == 0:  # the reference-shaped call picks the mode by itself
        indices, values, _ = tp.load_balance(d, capacity=int(1.3 * k) + 4096, k=k)
        assert np.array_equal(np.concatenate([to_np(i) for i in indices]), idx_o)


def test_load_balance_sampled_floor_too_high_asks_for_retry(zen, oracle):
    """k larger than the number of nonzeros the floor lets through cannot
    happen with a fair sample; force it with a tensor whose large values all
    hide from the 1-in-256 sample's expectation: nearly all zeros."""
    from zen_repro_amd import _lib

    n, P = 1 << 25, 8
    g = np.zeros(n, np.float32)
    rng = np.random.default_rng(5)
    hot = rng.choice(n, 3000, replace=False)
    g[hot] = rng.standard_normal(3000).astype(np.float32)
    k = 2000
    tp = zen.TensorPartition(P, 1, 3)
    d = to_dev(g)
    indices, values, splits = tp.load_balance(d, capacity=8192, k=k)  # retries in general mode if it must
    key = oracle.kth_key(g, k)
    masked, _ = oracle.mask_dense(g, key)
    idx_o, val_o, splits_o, _ = oracle.load_balance(masked, P, 1, 3)
    assert np.array_equal(to_np(splits), splits_o)
    assert np.array_equal(np.concatenate([to_np(i) for i in indices]), idx_o)


def test_load_balance_capacity_flag(zen, oracle):
    n, P = 1 << 16, 4
    g = make_grad(oracle, n, 0.5, "f32", seed=4)
    tp = zen.TensorPartition(P, 1, 3)
    with pytest.raises(RuntimeError, match="capacity"):
        tp.load_balance(to_dev(g), capacity=100)


# ----------------------------------------------------------------- merge


def make_payloads(oracle, rng, n, peers, per_peer, overlap, dtype):
    pool = rng.choice(n, max(1, int(per_peer * overlap)), replace=False)
    idx, val = [], []
    for _ in range(peers):
        shared = rng.choice(pool, int(per_peer * overlap), replace=False) if overlap > 0 else np.empty(0, np.int64)
        own = rng.integers(0, n, per_peer - len(shared))
        i = np.concatenate([shared, own]).astype(np.int32)
        rng.shuffle(i)
        v = (rng.standard_normal(len(i)) * 1e-3).astype(np.float32)
        idx.append(i)
        val.append(oracle.f32_to_bf16_bits(v) if dtype == "bf16" else v)
    return idx, val


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("n,peers,per_peer,overlap", [(1000, 4, 50, 0.2), (1 << 20, 16, 5000, 0.3),
                                                      (1 << 22, 64, 3000, 0.4), (4096, 8, 4096, 0.9),
                                                      (1 << 16, 1, 1, 0.0)])
def test_merge_sparse(zen, oracle, n, peers, per_peer, overlap, dtype):
    rng = np.random.default_rng(n + peers)
    idx, val = make_payloads(oracle, rng, n, peers, per_peer, overlap, dtype)
    ci, cv = np.concatenate(idx), np.concatenate(val)
    want_i, want_v = oracle.merge_sparse(ci, cv, n)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(peers), None, None)
    gi, gv = lba.merge_sparse([to_dev(i) for i in idx], [to_dev(v) for v in val], n)
    assert gi.dtype == torch.int64 and gv.dtype == torch.float32
    assert np.array_equal(to_np(gi), want_i)
    # same adds in the same order: bit-exact against the sequential fp32 oracle
    assert np.array_equal(to_np(gv).view(np.uint32), want_v.view(np.uint32))
    # and within 1e-6 (relative to the summed magnitudes) of the fp64 truth
    truth = oracle.decode(ci, cv, n, "f64")[want_i]
    vf = oracle.bf16_bits_to_f32(cv) if dtype == "bf16" else cv
    scale = np.zeros(n)
    np.add.at(scale, ci, np.abs(vf.astype(np.float64)))
    assert (np.abs(to_np(gv) - truth) <= 1e-6 * scale[want_i] + 1e-30).all()


@pytest.mark.parametrize("mode", [0, 1])
def test_merge_modes_agree_with_oracle(zen, oracle, mode):
    rng = np.random.default_rng(77 + mode)
    n = 3000017
    idx, val = make_payloads(oracle, rng, n, 16, 20000, 0.3, "bf16")
    ci, cv = np.concatenate(idx), np.concatenate(val)
    want_i, want_v = oracle.merge_sparse(ci, cv, n)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(16), None, None)
    gi, gv, cnt, st = lba.merge_sparse_flat(to_dev(ci), to_dev(cv), n, mode=mode)
    assert st.item() == 0 and cnt.item() == len(want_i)
    assert np.array_equal(to_np(gi)[:len(want_i)], want_i.astype(np.int32))
    assert np.array_equal(to_np(gv)[:len(want_i)].view(np.uint32), want_v.view(np.uint32))


def test_merge_piled_up_keys_fall_back_to_general_mode(zen, oracle):
    from zen_repro_amd import _lib

    n = 1 << 20
    rng = np.random.default_rng(3)
    idx = np.concatenate([np.full(100000, 12345), rng.integers(0, n, 50000)]).astype(np.int32)
    val = (rng.standard_normal(len(idx)) * 1e-3).astype(np.float32)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(4), None, None)
    _, _, cnt, st = lba.merge_sparse_flat(to_dev(idx), to_dev(val), n, mode=_lib.MODE_FAST)
    assert st.item() == _lib.STAT_RETRY  # one key range holds more than a workgroup sorts in LDS
    gi, gv = lba.merge_sparse(to_dev(idx), to_dev(val), n)  # retries by itself
    wi, wv = oracle.merge_sparse(idx, val, n)
    assert np.array_equal(to_np(gi), wi) and np.array_equal(to_np(gv).view(np.uint32), wv.view(np.uint32))
    dense = lba.decode_sparse_tensors(to_dev(idx), to_dev(val), n)
    assert np.array_equal(to_np(dense), oracle.decode(idx, val, n, "f32acc"))


def test_merge_cancellation_nan_and_bad_index(zen, oracle):
    from zen_repro_amd import _lib

    n = 64
    idx = np.array([5, 9, 5, 63, 9, 0, 0, 17], np.int32)
    val = np.array([1.0, 2.0, -1.0, 4.0, np.nan, 3.0, -3.0, -0.0], np.float32)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(2), None, None)
    gi, gv = lba.merge_sparse(to_dev(idx), to_dev(val), n)
    wi, wv = oracle.merge_sparse(idx, val, n)
    assert to_np(gi).tolist() == wi.tolist() == [9, 63]
    assert np.array_equal(to_np(gv).view(np.uint32) & 0x7FC00000, wv.view(np.uint32) & 0x7FC00000)
    bad = np.array([5, 64, -1, 7], np.int64)
    for mode in (0, 1):
        i2, v2, cnt, st = lba.merge_sparse_flat(to_dev(bad), to_dev(np.ones(4, np.float32)), n, idx64=True, mode=mode)
        assert cnt.item() == 2 and st.item() == _lib.STAT_BAD_INDEX
        assert to_np(i2)[:2].tolist() == [5, 7]


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_decode_sparse_tensors_dense(zen, oracle, dtype):
    rng = np.random.default_rng(8)
    n, peers = 1 << 18, 8
    idx, val = make_payloads(oracle, rng, n, peers, 4000, 0.3, dtype)
    ci, cv = np.concatenate(idx), np.concatenate(val)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(peers), None, None)
    dense = lba.decode_sparse_tensors([to_dev(i) for i in idx], [to_dev(v) for v in val], n)
    f32 = oracle.decode(ci, cv, n, "f32acc")
    want = oracle.f32_to_bf16_bits(f32) if dtype == "bf16" else f32
    got = to_np(dense)
    assert dense.dtype == (torch.bfloat16 if dtype == "bf16" else torch.float32)
    assert np.array_equal(got, want)
    # single-tensor form with int64 indices (comm.py:40-44)
    d2 = lba.decode_sparse_tensors(to_dev(ci.astype(np.int64)), to_dev(cv), n)
    assert np.array_equal(to_np(d2), want)
    if dtype == "bf16":
        # against the reference's own accumulation dtype: 1e-3 relative
        native = oracle.bf16_bits_to_f32(oracle.decode(ci, cv, n, "native"))
        scale = np.zeros(n)
        np.add.at(scale, ci, np.abs(oracle.bf16_bits_to_f32(cv).astype(np.float64)))
        assert (np.abs(oracle.bf16_bits_to_f32(got) - native) <= 2e-2 * scale + 1e-30).all()


def ascending_lists(oracle, rng, n, nlists, per_list, shared, dtype, idx_dtype):
    """nlists strictly ascending index lists over [0, n); a fraction `shared` of every list comes from one pool
    (lists meet on those indices), the rest lies in the list's own residue class (disjoint)."""
    pool = rng.choice(n // nlists, max(1, int(per_list * shared) * 2), replace=False) * nlists
    idx, val = [], []
    for l in range(nlists):
        common = rng.choice(pool, int(per_list * shared), replace=False) if shared > 0 else np.empty(0, np.int64)
        own = rng.choice(n // nlists, per_list - len(common), replace=False) * nlists + (l if l else 0)
        i = np.unique(np.concatenate([common, own])).astype(idx_dtype)
        v = (rng.standard_normal(len(i)) * 1e-3).astype(np.float32)
        v[::97] = -0.0  # +0 + -0 = +0: the dense element stays a plain zero
        idx.append(i)
        val.append(oracle.f32_to_bf16_bits(v) if dtype == "bf16" else v)
    return idx, val


@pytest.mark.parametrize("idx_dtype", [np.int64, np.int32])
@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("n,nlists,per_list,shared", [
    ((1 << 22) + 4099, 16, 20000, 0.0),   # the second exchange: disjoint shards; size not a multiple of the tile
    (1 << 22, 16, 20000, 0.4),            # method 1: every rank's own selection, lists meet on many indices
    (1 << 20, 1, 5000, 0.0),
    (3000, 5, 40, 0.5),                   # less than one tile
    (1 << 21, 64, 3000, 0.1),
])
def test_decode_ascending_lists_without_a_sort(zen, oracle, n, nlists, per_list, shared, dtype, idx_dtype):
    """zen_decode_dense_sorted through decode_sparse_tensors(ascending=True): bit-identical to the oracle's
    sequential fp32 scatter_add (and therefore to zen_decode_dense), straight through the C-ABI too."""
    from zen_repro_amd import _lib

    rng = np.random.default_rng(n % 977 + nlists)
    idx, val = ascending_lists(oracle, rng, n, nlists, per_list, shared, dtype, idx_dtype)
    ci, cv = np.concatenate(idx), np.concatenate(val)
    f32 = oracle.decode(ci.astype(np.int64), cv, n, "f32acc")
    want = oracle.f32_to_bf16_bits(f32) if dtype == "bf16" else f32
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(max(nlists, 2)), None, None)
    d_idx, d_val = [to_dev(i) for i in idx], [to_dev(v) for v in val]
    got = lba.decode_sparse_tensors(d_idx, d_val, n, ascending=True)
    assert np.array_equal(to_np(got).view(want.dtype), want)
    assert np.array_equal(to_np(lba.decode_sparse_tensors(d_idx, d_val, n)).view(want.dtype), want)
    # the entry point itself: it must have taken the lists as they are (status 0), into a buffer full of ones
    L = _lib.lib()
    flat_i, flat_v = to_dev(ci), to_dev(cv)
    dense = torch.full((n,), 1.0, dtype=flat_v.dtype, device="cuda")
    starts = (ctypes.c_int64 * (nlists + 1))(0, *np.cumsum([len(i) for i in idx]).tolist())
    ws = torch.empty(L.zen_decode_dense_sorted_workspace(n, nlists), dtype=torch.uint8, device="cuda")
    status = _lib.status_word("cuda")
    rc = L.zen_decode_dense_sorted(_lib.ptr(flat_i), int(idx_dtype == np.int64), _lib.ptr(flat_v), _lib.dtype_code(flat_v),
                                   starts, nlists, _lib.ptr(dense), n, _lib.ptr(ws), ws.numel(), _lib.ptr(status),
                                   _lib.stream_of("cuda"))
    assert rc == 0 and status.item() == 0
    assert np.array_equal(to_np(dense).view(want.dtype), want)


def test_decode_ascending_declines_what_is_not_ascending(zen, oracle):
    """A list with a descent, a repeated index inside one list or an index outside the dense tensor raise
    ZEN_STAT_RETRY; decode_sparse_tensors then answers through the general entry point (or raises, for the
    bad index, as the reference's scatter_add_ does)."""
    from zen_repro_amd import _lib

    n = 1 << 20
    rng = np.random.default_rng(3)
    idx, val = ascending_lists(oracle, rng, n, 4, 3000, 0.2, "f32", np.int64)
    L = _lib.lib()

    def status_of(lists):
        flat_i, flat_v = to_dev(np.concatenate(lists)), to_dev(np.concatenate(val))
        dense = torch.empty(n, dtype=torch.float32, device="cuda")
        starts = (ctypes.c_int64 * 5)(0, *np.cumsum([len(i) for i in lists]).tolist())
        ws = torch.empty(L.zen_decode_dense_sorted_workspace(n, 4), dtype=torch.uint8, device="cuda")
        status = _lib.status_word("cuda")
        rc = L.zen_decode_dense_sorted(_lib.ptr(flat_i), 1, _lib.ptr(flat_v), _lib.F32, starts, 4, _lib.ptr(dense), n,
                                       _lib.ptr(ws), ws.numel(), _lib.ptr(status), _lib.stream_of("cuda"))
        assert rc == 0
        return int(status.item())

    assert status_of(idx) == 0
    swapped = [i.copy() for i in idx]
    swapped[2][[100, 101]] = swapped[2][[101, 100]]          # one descent
    assert status_of(swapped) == _lib.STAT_RETRY
    twice = [i.copy() for i in idx]
    twice[1][500] = twice[1][499]                             # the same index twice in one list
    assert status_of(twice) == _lib.STAT_RETRY
    beyond = [i.copy() for i in idx]
    beyond[3][-1] = n + 5                                     # ascending, but outside the tensor
    assert status_of(beyond) == _lib.STAT_RETRY
    below = [i.copy() for i in idx]
    below[0][0] = -3
    assert status_of(below) == _lib.STAT_RETRY
    # through the wrapper the result is right all the same
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(4), None, None)
    for lists in (swapped, twice):
        got = lba.decode_sparse_tensors([to_dev(i) for i in lists], [to_dev(v) for v in val], n, ascending=True)
        assert np.array_equal(to_np(got), oracle.decode(np.concatenate(lists), np.concatenate(val), n, "f32acc"))
    with pytest.raises(RuntimeError):
        lba.decode_sparse_tensors([to_dev(i) for i in beyond], [to_dev(v) for v in val], n, ascending=True)
    # bad arguments are the host's business
    ws = torch.empty(1024, dtype=torch.uint8, device="cuda")
    status = _lib.status_word("cuda")
    bad = (ctypes.c_int64 * 3)(0, 10, 5)
    assert L.zen_decode_dense_sorted(_lib.ptr(ws), 1, _lib.ptr(ws), _lib.F32, bad, 2, _lib.ptr(ws), 100, _lib.ptr(ws),
                                     ws.numel(), _lib.ptr(status), None) == _lib.EINVAL
    ok = (ctypes.c_int64 * 2)(0, 10)
    assert L.zen_decode_dense_sorted(_lib.ptr(ws), 1, _lib.ptr(ws), _lib.F32, ok, 1, _lib.ptr(ws), 1 << 30,
                                     _lib.ptr(ws), ws.numel(), _lib.ptr(status), None) == _lib.EWORKSPACE


def test_stack_tensors_views_are_not_copied(zen):
    buf = torch.arange(100, device="cuda", dtype=torch.int32)
    parts = [buf[0:10], buf[10:45], buf[45:100]]
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(3), None, None)
    assert lba.stack_tensors(parts).data_ptr() == buf.data_ptr()
    other = [buf[0:10], buf[20:30]]
    assert lba.stack_tensors(other).tolist() == list(range(10)) + list(range(20, 30))


def test_zero_pool_pieces_are_zero_apart_and_per_stream(zen):
    """Status words, counts and split sizes are cut from pooled zeroed blocks: every piece is zero, aligned,
    handed out once, and belongs to the stream that was current when its block was made."""
    from zen_repro_amd import _lib

    pool = _lib.ZeroPool()
    a = pool.take("cuda", 1, torch.int32)
    b = pool.take("cuda", 16, torch.int64)
    c = pool.take("cuda", 3, torch.int32)
    for t, n, dt in ((a, 1, torch.int32), (b, 16, torch.int64), (c, 3, torch.int32)):
        assert t.dtype == dt and t.numel() == n and t.data_ptr() % 16 == 0 and int(t.abs().sum()) == 0
    spans = sorted((t.data_ptr(), t.data_ptr() + t.numel() * t.element_size()) for t in (a, b, c))
    assert all(spans[i][1] <= spans[i + 1][0] for i in range(2))
    a.fill_(7)  # a holder may write: the neighbours stay zero
    assert int(b.abs().sum()) == 0 and int(c.abs().sum()) == 0
    base = a.data_ptr()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        d = pool.take("cuda", 1, torch.int32)
        assert int(d.item()) == 0
    assert not (base <= d.data_ptr() < base + pool.BLOCK)  # another stream, another block
    # a block that is used up is replaced, not reused
    seen = set()
    for _ in range(2 * pool.BLOCK // 16 + 3):
        t = pool.take("cuda", 1, torch.int32)
        assert t.data_ptr() not in seen
        seen.add(t.data_ptr())
    assert int(t.item()) == 0
    big = pool.take("cuda", pool.BLOCK, torch.uint8)  # too large for a block: a tensor of its own
    assert big.numel() == pool.BLOCK and int(big.sum()) == 0


def test_profile_every_nth_launch(zen, oracle):
    """zen_profile_every(n): of a tag's launches since recording began, the first and every n-th after it
    carry events."""
    from zen_repro_amd import _lib

    vals = to_dev(make_grad(oracle, 1 << 16, 0.05, "f32", seed=5))
    try:
        _lib.profile_enable(True, only="k_compress", every=3)
        for _ in range(7):
            zen.compress(10, vals)
        torch.cuda.synchronize()
        got = _lib.profile_read()
        assert set(got) == {"k_compress"} and got["k_compress"][1] == 3 and got["k_compress"][0] > 0
        _lib.profile_enable(True, every=1)
        for _ in range(2):
            zen.compress(10, vals)
        assert _lib.profile_read()["k_compress"][1] == 2
        with pytest.raises(ValueError):
            _lib.profile_enable(True, every=0)
    finally:
        _lib.profile_enable(False)
        _lib.check(_lib.lib().zen_profile_every(1), "profile_every")


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("idx64", [False, True])
@pytest.mark.parametrize("count", [0, 1, 2047, 2049, 300000])
def test_round_merged_sums(zen, oracle, dtype, idx64, count):
    """zen_round_compact: what comm.py:125-127 makes of the merged sums (a dense tensor of the gradient's type,
    then its nonzeros): every fp32 sum rounded once to the type, entries that round to zero dropped, order
    kept; only the first `count` entries (a device value) are looked at.  Sums that are tiny, negative zeros,
    NaN and infinities included."""
    cap = count + 100
    rng = np.random.default_rng(count + 7)
    sums = (rng.standard_normal(cap) * 1e-3).astype(np.float32)
    sums[rng.integers(0, cap, cap // 5)] = 0.0
    sums[rng.integers(0, cap, cap // 7)] = -0.0
    sums[rng.integers(0, cap, cap // 9)] = 1e-41 if dtype == "bf16" else 1e-45  # bf16: rounds to zero
    sums[rng.integers(0, cap, 3)] = np.nan
    sums[rng.integers(0, cap, 3)] = -np.inf
    idx = np.sort(rng.choice(1 << 30, cap, replace=False)).astype(np.int64 if idx64 else np.int32)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(4), None, None)
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float32
    cnt = torch.tensor([count], dtype=torch.int64, device="cuda")
    o_idx, o_val, kept, status = lba.round_merged_flat(to_dev(idx), to_dev(sums), cnt, tdt)
    assert int(status) == 0
    rounded = torch.from_numpy(sums[:count]).to(tdt)
    keep = (rounded != 0).numpy()  # NaN != 0 is true, -0.0 != 0 false: what torch.nonzero keeps
    u = int(kept)
    assert u == int(keep.sum())
    assert np.array_equal(to_np(o_idx)[:u], idx[:count][keep])
    bits = torch.int16 if dtype == "bf16" else torch.int32
    got, want = o_val[:u].cpu(), rounded[torch.from_numpy(keep)]
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan)  # a NaN stays a NaN (which of the NaN patterns is the converter's business)
    assert torch.equal(got[~nan].view(bits), want[~nan].view(bits))
