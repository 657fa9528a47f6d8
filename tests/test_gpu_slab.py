"""Parity of the bucket-slab fast paths (large inputs) against the CPU oracle:
load balance with many collisions (levels 2 and 3, serial entries, declined
calls that fall back to the general mode), merge with heavy duplication, bad
indices and 64-bit indices, and calls in flight on two streams with their own
slots.  Every test first checks through zen_*_path that the sizes really take
the slab path.  Bar: bit-exact, as in test_gpu_parity.py."""
import numpy as np
import pytest
import torch

from gpu_util import make_grad, to_dev, to_np

pytestmark = pytest.mark.gpu

SLAB = 2
WIDE = 3
FLAGS = 0  # OR-ed into the fast mode of every call and path query of this module (set per run, below)


@pytest.fixture(scope="module", autouse=True, params=["wide", "slabs"])
def fast_path(request):
    """Every test of this module runs twice: on the wide buckets (where the sizes suit them) and with
    MODE_SLABS, which keeps the calls on the bucket slabs."""
    global FLAGS
    import zen_repro_amd
    from zen_repro_amd import _lib

    FLAGS = _lib.MODE_SLABS if request.param == "slabs" else 0
    zen_repro_amd.TensorPartition.fast_flags = FLAGS
    zen_repro_amd.LoadBalanceAllreduce.fast_flags = FLAGS
    yield request.param
    FLAGS = 0
    zen_repro_amd.TensorPartition.fast_flags = 0
    zen_repro_amd.LoadBalanceAllreduce.fast_flags = 0


def on_fast_path(code):
    """Whether a zen_*_path answer is the path this run is about: the bucket slabs with MODE_SLABS, else the
    wide buckets (sizes that take the bucket slabs either way are covered by the other run)."""
    if FLAGS:
        return code == SLAB
    if code == SLAB:
        pytest.skip("these sizes take the bucket slabs with or without MODE_SLABS: covered by the other run")
    return code == WIDE


@pytest.fixture(scope="module")
def zen():
    import zen_repro_amd
    from zen_repro_amd import _lib

    _lib.lib()
    assert torch.cuda.is_available()
    return zen_repro_amd


def lb_path(zen, n, P, dtype, capacity, k=0, mode=0, scale=1):
    from zen_repro_amd import _lib

    m = int(n * scale // P * P)
    return _lib.lib().zen_load_balance_path(n, m, 1 if dtype == "bf16" else 0, capacity, P, k, mode | FLAGS)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("n,P,density,rehash", [
    ((1 << 23), 16, 0.15, 3),        # 15 % of the slots taken: thousands of level-2/3 moves per partition
    ((1 << 23), 16, 0.15, 2),        # two levels: serial entries in every partition
    ((1 << 23) + 4096, 8, 0.05, 3),  # table size not a power of two
    ((1 << 24), 64, 0.01, 3),
    (6000000, 3, 0.02, 3),           # partitions not a power of two, odd bucket widths
])
def test_slab_load_balance_bit_exact(zen, oracle, n, P, density, rehash, dtype):
    from zen_repro_amd import _lib

    n = n // P * P
    g = make_grad(oracle, n, density, dtype, seed=n ^ (P * 131) ^ rehash)
    g[0] = 0x3F80 if dtype == "bf16" else 1.0  # index 0 holds a value and is never transmitted
    idx_o, val_o, splits_o, st_o = oracle.load_balance(g, P, 1, rehash)
    assert st_o == 0
    capacity = int(len(idx_o) * 1.1) + 1024
    assert on_fast_path(lb_path(zen, n, P, dtype, capacity))
    tp = zen.TensorPartition(P, 1, rehash)
    d = to_dev(g)
    for rep in range(2):  # the second call finds the borrowed table zero again
        oi, ov, splits, status = tp.load_balance_flat(d, capacity=capacity, mode=_lib.MODE_FAST)
        assert status.item() == 0
        assert np.array_equal(to_np(splits), splits_o)
        total = int(splits_o.sum())
        assert np.array_equal(to_np(oi)[:total], idx_o)
        assert np.array_equal(to_np(ov)[:total], val_o)
    m, _ = oracle.table_sizes(n, P, 1)
    assert not tp._table(d.device, m).any()


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_slab_load_balance_odd_length_unaligned_and_empty(zen, oracle, dtype):
    """A tensor whose length is no multiple of anything and whose first element is not 16-byte aligned (the
    streaming kernel's element-wise loads and its ragged last tile), and a tensor of zeros."""
    from zen_repro_amd import _lib

    n, P = (1 << 23) + 1237, 16
    g = make_grad(oracle, n, 0.03, dtype, seed=4242)
    g[-1] = 0x3F80 if dtype == "bf16" else 1.0  # the very last element is selected
    idx_o, val_o, splits_o, st_o = oracle.load_balance(g, P, 1, 3)
    assert st_o == 0
    capacity = len(idx_o) + 2048
    assert on_fast_path(lb_path(zen, n, P, dtype, capacity))
    buf = to_dev(np.concatenate([g[:3], g]))
    d = buf[3:]
    assert d.data_ptr() % 16 != 0
    tp = zen.TensorPartition(P, 1, 3)
    oi, ov, splits, status = tp.load_balance_flat(d, capacity=capacity)
    total = int(splits_o.sum())
    assert status.item() == 0 and np.array_equal(to_np(splits), splits_o)
    assert np.array_equal(to_np(oi)[:total], idx_o) and np.array_equal(to_np(ov)[:total], val_o)
    # the same tensor 16-byte aligned: whole vectors stream, the few elements behind the last one (the
    # selected last element among them) go through a stage of their own
    a = to_dev(g)
    assert a.data_ptr() % 16 == 0 and n % 8 != 0
    oi, ov, splits, status = tp.load_balance_flat(a, capacity=capacity)
    assert status.item() == 0 and np.array_equal(to_np(splits), splits_o)
    assert np.array_equal(to_np(oi)[:total], idx_o) and np.array_equal(to_np(ov)[:total], val_o)
    zeros = torch.zeros(n, dtype=d.dtype, device="cuda")
    oi, ov, splits, status = tp.load_balance_flat(zeros, capacity=capacity)
    assert status.item() == 0 and int(splits.sum()) == 0


def test_slab_load_balance_declines_and_general_mode_takes_over(zen, oracle):
    """One rehash level at 15 % load sends every level-1 loser to the serial
    lists: far more than the slab path carries per partition.  It must say so
    (RETRY), and the reference-shaped call must come back with the right
    answer from the general mode."""
    from zen_repro_amd import _lib

    n, P = (1 << 23) + 16000, 16  # not a power of two: about 8000 level-1 losers per partition
    g = make_grad(oracle, n, 0.15, "bf16", seed=99)
    idx_o, val_o, splits_o, st_o = oracle.load_balance(g, P, 1, 1)
    assert st_o == 0
    capacity = int(len(idx_o) * 1.1) + 1024
    assert on_fast_path(lb_path(zen, n, P, "bf16", capacity))
    tp = zen.TensorPartition(P, 1, 1)
    d = to_dev(g)
    _, _, _, status = tp.load_balance_flat(d, capacity=capacity, mode=_lib.MODE_FAST)
    assert status.item() & _lib.STAT_RETRY
    tp._table(d.device, n).zero_()
    indices, values, splits = tp.load_balance(d, capacity=capacity)
    assert np.array_equal(to_np(splits), splits_o)
    assert np.array_equal(np.concatenate([to_np(i) for i in indices]), idx_o)
    assert np.array_equal(np.concatenate([to_np(v) for v in values]), val_o)


def test_slab_load_balance_too_many_candidates_declines(zen, oracle):
    """A capacity far below what is selected: the candidate list overflows, the
    call declines instead of writing out of bounds."""
    from zen_repro_amd import _lib

    n, P = 1 << 23, 8
    g = make_grad(oracle, n, 0.05, "f32", seed=5)
    capacity = 1 << 16  # about a sixth of the nonzeros
    assert on_fast_path(lb_path(zen, n, P, "f32", capacity))
    tp = zen.TensorPartition(P, 1, 3)
    _, _, _, status = tp.load_balance_flat(to_dev(g), capacity=capacity, mode=_lib.MODE_FAST)
    assert status.item() & (_lib.STAT_RETRY | _lib.STAT_CAPACITY)


def test_slab_load_balance_fused_topk_fp32(zen, oracle):
    """fp32 top-k inside the call on the slab path: the candidates' histogram resolves 15 key bits, the last
    16 come from a second histogram over the candidates of the threshold's bin.  The k-th value is shared
    by many elements (ties are kept), element 0 lies in the threshold's bin above the threshold (it counts
    towards k and is never transmitted), and the very last element holds the largest value."""
    n, P = (1 << 24) + 24, 16
    rng = np.random.default_rng(77)
    x = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    k = n // 100
    key0 = int(oracle.kth_key(x, k))
    tie = np.array([key0], dtype=np.uint32).view(np.float32)[0]
    x[rng.integers(1, n - 1, 300)] = -tie                                    # 300 more elements at the k-th magnitude
    x[0] = np.array([key0 + 5], dtype=np.uint32).view(np.float32)[0]         # same bin of 65536 keys, above it
    x[-1] = 1.0
    key = int(oracle.kth_key(x, k))
    assert key >> 16 == key0 >> 16
    masked, kept = oracle.mask_dense(x, key)
    assert kept > k and masked[0] != 0
    idx_o, val_o, splits_o, st_o = oracle.load_balance(masked, P, 1, 3)
    assert st_o == 0 and 0 not in idx_o
    capacity = int(1.25 * k) + 4096
    assert on_fast_path(lb_path(zen, n, P, "f32", capacity, k=k))
    tp = zen.TensorPartition(P, 1, 3)
    d = to_dev(x)
    thr_out = torch.zeros(2, dtype=torch.int32, device="cuda")
    for rep in range(2):  # the second call finds its counters cleared again
        oi, ov, splits, status = tp.load_balance_flat(d, capacity=capacity, k=k, thr_out=thr_out)
        assert status.item() == 0
        assert to_np(thr_out).tolist() == [key, kept]
        assert np.array_equal(to_np(splits), splits_o)
        total = int(splits_o.sum())
        assert np.array_equal(to_np(oi)[:total], idx_o)
        assert np.array_equal(to_np(ov)[:total], val_o)


def test_fused_topk_fp32_wherever_the_kth_key_lies_in_its_bin(zen, oracle, fast_path):
    """The fp32 threshold's last 16 bits for a k-th key at the top, the bottom and the middle of the threshold's
    bin of 65536 keys, at even and odd keys and either side of a multiple of 128 (the refinement's last
    workgroup gives a thread 128 keys and a lane of its first wave two of them)."""
    n, P = (1 << 20) if fast_path == "wide" else (1 << 24), 4
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(n) * 0.2).astype(np.float32)
    base = 0x3F000000  # 0.5: the bin is [0.5, 0.50390625)
    keys = x.view(np.uint32) & 0x7FFFFFFF
    x[(keys >> 16) == (base >> 16)] = 0.3  # nobody else in that bin
    x[0] = 0.25
    lows = [65535, 65534, 65409, 65408, 65407, 32769, 32768, 129, 128, 127, 1, 0]
    at = rng.choice(np.arange(1, n), 3 * len(lows), replace=False)
    sign = np.where(rng.random(len(at)) < 0.5, 0x80000000, 0).astype(np.uint32)
    x.view(np.uint32)[at] = (np.repeat(np.array(lows, np.uint32), 3) + np.uint32(base)) | sign  # three of each
    ordered = np.sort(x.view(np.uint32) & 0x7FFFFFFF)
    above = n - int(np.searchsorted(ordered, base + 65536, "left"))
    assert int(oracle.kth_key(x, above + 4)) == base + lows[1]
    capacity = int(1.5 * above) + 4096
    tp = zen.TensorPartition(P, 1, 3)
    d = to_dev(x)
    thr_out = torch.zeros(2, dtype=torch.int32, device="cuda")
    for j in range(1, 3 * len(lows) + 1):
        k = above + j
        key = base + lows[(j - 1) // 3]  # the k-th largest key: the ((j - 1) // 3)-th of the planted ones
        kept = n - int(np.searchsorted(ordered, key, "left"))
        assert on_fast_path(lb_path(zen, n, P, "f32", capacity, k=k))
        _, _, splits, status = tp.load_balance_flat(d, capacity=capacity, k=k, thr_out=thr_out)
        assert status.item() == 0, (j, status.item())
        assert to_np(thr_out).tolist() == [key, kept], j
        assert int(to_np(splits).sum()) == kept - int((x.view(np.uint32)[0] & 0x7FFFFFFF) >= key)  # index 0 is never handed on


def test_slab_load_balance_threshold_given(zen, oracle):
    """Selection by a threshold the caller computed (topk_threshold) instead of k."""
    from zen_repro_amd import _lib

    n, P = 1 << 24, 16
    rng = np.random.default_rng(8)
    g = oracle.f32_to_bf16_bits((rng.standard_normal(n) * 1e-3).astype(np.float32))
    k = n // 100
    key = oracle.kth_key(g, k)
    masked, kept = oracle.mask_dense(g, key)
    idx_o, val_o, splits_o, _ = oracle.load_balance(masked, P, 1, 3)
    d = to_dev(g)
    thr = zen.topk_threshold(d, k)
    capacity = kept + 4096
    assert on_fast_path(lb_path(zen, n, P, "bf16", capacity))
    tp = zen.TensorPartition(P, 1, 3)
    oi, ov, splits, status = tp.load_balance_flat(d, thr=thr, capacity=capacity)
    assert status.item() == 0 and np.array_equal(to_np(splits), splits_o)
    assert np.array_equal(to_np(oi)[:kept], idx_o) and np.array_equal(to_np(ov)[:kept], val_o)


def test_two_slots_in_flight_give_the_same_answer(zen, oracle):
    """Two encodes and two merges enqueued on four streams, each pair with its
    own slot (workspace and table): same bytes as one call alone."""
    n, P = 1 << 24, 16
    rng = np.random.default_rng(21)
    g = oracle.f32_to_bf16_bits((rng.standard_normal(n) * 1e-3).astype(np.float32))
    d = to_dev(g)
    k = n // 200
    capacity = int(1.3 * k) + 4096
    assert on_fast_path(lb_path(zen, n, P, "bf16", capacity, k=k))
    tp = zen.TensorPartition(P, 1, 3)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P), None, None)
    mi = to_dev(rng.integers(1, n, 400000).astype(np.int32))
    mv = to_dev((rng.standard_normal(400000) * 1e-3).astype(np.float32))
    ref = tp.load_balance_flat(d, capacity=capacity, k=k)
    ref_m = lba.merge_sparse_flat(mi, mv, n)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(4)]
    outs = []
    for rep in range(3):
        for slot in range(2):
            with torch.cuda.stream(streams[slot]):
                outs.append(("e", tp.load_balance_flat(d, capacity=capacity, k=k, slot=slot)))
            with torch.cuda.stream(streams[2 + slot]):
                outs.append(("m", lba.merge_sparse_flat(mi, mv, n, slot=slot)))
    torch.cuda.synchronize()
    total = int(ref[2].sum())
    for kind, o in outs:
        if kind == "e":
            assert o[3].item() == 0 and torch.equal(o[2], ref[2])
            assert torch.equal(o[0][:total], ref[0][:total]) and torch.equal(o[1][:total], ref[1][:total])
        else:
            cnt = int(ref_m[2])
            assert o[3].item() == 0 and int(o[2]) == cnt
            assert torch.equal(o[0][:cnt], ref_m[0][:cnt]) and torch.equal(o[1][:cnt], ref_m[1][:cnt])


# ------------------------------------------------------------------ merge


def payloads(oracle, rng, n, peers, per_peer, overlap, dtype):
    pool = rng.choice(n, max(1, int(per_peer * overlap) * 2), replace=False)
    idx, val = [], []
    for _ in range(peers):
        shared = rng.choice(pool, int(per_peer * overlap), replace=False) if overlap > 0 else np.empty(0, np.int64)
        own = rng.integers(0, n, per_peer - len(shared))
        i = np.concatenate([shared, own])
        rng.shuffle(i)
        v = (rng.standard_normal(len(i)) * 1e-3).astype(np.float32)
        idx.append(i)
        val.append(oracle.f32_to_bf16_bits(v) if dtype == "bf16" else v)
    return np.concatenate(idx), np.concatenate(val)


@pytest.mark.parametrize("idx64", [False, True])
@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("n,peers,per_peer,overlap", [
    (1 << 24, 16, 20000, 0.3),
    (50000000, 64, 4000, 0.5),   # every shared index arrives 64 times
    (1 << 24, 16, 20000, 0.9),   # nine records in ten share their index with fifteen others: more than a
                                 # workgroup sets aside for ranking in a second round
    ((1 << 23) + 12345, 4, 30000, 0.0),
])
def test_slab_merge_bit_exact(zen, oracle, n, peers, per_peer, overlap, dtype, idx64):
    from zen_repro_amd import _lib

    rng = np.random.default_rng(n % 1000 + peers)
    ci, cv = payloads(oracle, rng, n, peers, per_peer, overlap, dtype)
    ci = ci.astype(np.int64 if idx64 else np.int32)
    assert on_fast_path(_lib.lib().zen_merge_path(len(ci), n, _lib.MODE_FAST | FLAGS))
    want_i, want_v = oracle.merge_sparse(ci, cv, n)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(peers), None, None)
    gi, gv, cnt, st = lba.merge_sparse_flat(to_dev(ci), to_dev(cv), n, idx64=idx64, mode=_lib.MODE_FAST)
    assert st.item() == 0 and cnt.item() == len(want_i)
    assert np.array_equal(to_np(gi)[:len(want_i)], want_i.astype(np.int64 if idx64 else np.int32))
    # same adds in the same order as a sequential scatter_add_: bit-exact
    assert np.array_equal(to_np(gv)[:len(want_i)].view(np.uint32), want_v.view(np.uint32))
    # and the dense form of the same merge
    dense = lba.decode_sparse_tensors(to_dev(ci), to_dev(cv), n)
    f32 = oracle.decode(ci, cv, n, "f32acc")
    assert np.array_equal(to_np(dense), oracle.f32_to_bf16_bits(f32) if dtype == "bf16" else f32)


def test_slab_merge_bad_indices_cancellation_and_pile_up(zen, oracle):
    from zen_repro_amd import _lib

    n = 1 << 24
    rng = np.random.default_rng(17)
    idx = rng.integers(0, n, 200000).astype(np.int64)
    val = (rng.standard_normal(len(idx)) * 1e-3).astype(np.float32)
    idx[1000:1100] = idx[0:100]          # pairs that cancel exactly
    val[1000:1100] = -val[0:100]
    idx[5000] = -7                        # out of range on both sides
    idx[5001] = n
    assert on_fast_path(_lib.lib().zen_merge_path(len(idx), n, _lib.MODE_FAST | FLAGS))
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(4), None, None)
    gi, gv, cnt, st = lba.merge_sparse_flat(to_dev(idx), to_dev(val), n, idx64=True, mode=_lib.MODE_FAST)
    assert st.item() == _lib.STAT_BAD_INDEX
    good = (idx >= 0) & (idx < n)
    wi, wv = oracle.merge_sparse(idx[good], val[good], n)
    assert cnt.item() == len(wi)
    assert np.array_equal(to_np(gi)[:len(wi)], wi) and np.array_equal(to_np(gv)[:len(wi)].view(np.uint32), wv.view(np.uint32))
    # one index received 50000 times: the slab path declines, the general mode answers
    idx2 = np.concatenate([np.full(50000, 4242), rng.integers(0, n, 100000)]).astype(np.int32)
    val2 = (rng.standard_normal(len(idx2)) * 1e-3).astype(np.float32)
    _, _, _, st2 = lba.merge_sparse_flat(to_dev(idx2), to_dev(val2), n, mode=_lib.MODE_FAST)
    assert st2.item() & _lib.STAT_RETRY
    gi2, gv2 = lba.merge_sparse(to_dev(idx2), to_dev(val2), n)
    wi2, wv2 = oracle.merge_sparse(idx2, val2, n)
    assert np.array_equal(to_np(gi2), wi2) and np.array_equal(to_np(gv2).view(np.uint32), wv2.view(np.uint32))


# ------------------------------------------------ counters are left at zero

def test_table_and_merge_workspace_are_zero_again_after_every_call(zen, oracle):
    """The slab paths clear no counters up front: they rely on the table (encode) and the head of the merge
    workspace being zero, and put them back to zero themselves.  Calls of different sizes and selections in a
    row, on one table and one workspace, must each give the oracle's answer and leave both all zero."""
    from zen_repro_amd import _lib

    L = _lib.lib()
    P = 8
    n = 1 << 23
    tp = zen.TensorPartition(P, 1, 3)
    rng = np.random.default_rng(5)
    g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    cases = [("f32", 0.004, 0), ("bf16", 0.01, 0), ("f32", 1.0, n // 200), ("bf16", 1.0, n // 100), ("f32", 0.002, 0)]
    for dtype, density, k in cases:
        x = np.where(rng.random(n) < density, g, 0).astype(np.float32)
        x_np = oracle.f32_to_bf16_bits(x) if dtype == "bf16" else x
        grad = to_dev(x_np)
        if k:
            key = oracle.kth_key(x_np, k)
            masked, kept = oracle.mask_dense(x_np, key)
            cap = kept + 1024
        else:
            masked, cap = x_np, int(np.count_nonzero(x)) + 1024
        m, _ = tp.table_sizes(n)
        assert on_fast_path(L.zen_load_balance_path(n, m, _lib.dtype_code(grad), cap, P, k, _lib.MODE_FAST | FLAGS))
        idx, val, splits, st = tp.load_balance_flat(grad, None, cap, k=k)
        idx_o, val_o, splits_o, st_o = oracle.load_balance(masked, P, 1, 3)
        assert int(st.item()) == 0 and st_o == 0
        total = int(splits.sum())
        assert np.array_equal(splits.cpu().numpy(), splits_o)
        assert np.array_equal(idx[:total].cpu().numpy(), idx_o)
        assert np.array_equal(to_np(val[:total]), val_o)
        assert int(tp._table(grad.device, m).count_nonzero()) == 0, (dtype, density, k)

    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P), None, None)
    dense_n = 1 << 26
    for r in (400_000, 3_000_000, 70_000):
        idx = rng.integers(1, dense_n, r).astype(np.int32)
        idx[rng.integers(0, r, r // 3)] = idx[rng.integers(0, r, r // 3)]  # duplicates
        val = (rng.standard_normal(r) * 1e-3).astype(np.float32)
        assert on_fast_path(L.zen_merge_path(r, dense_n, _lib.MODE_FAST | FLAGS))
        m_idx, m_val, count, st = lba.merge_sparse_flat(to_dev(idx), to_dev(val), dense_n)
        assert int(st.item()) == 0
        mi_o, mv_o = oracle.merge_sparse(idx, val, dense_n)
        c = int(count.item())
        assert np.array_equal(m_idx[:c].cpu().numpy(), mi_o)
        assert np.array_equal(m_val[:c].cpu().numpy().view(np.uint32), mv_o.view(np.uint32))
        ws = _lib.scratch.get(m_idx.device, "merge/0", 256, zero=True)
        assert int(ws[:L.zen_merge_zero_bytes()].count_nonzero()) == 0, r


def test_load_balance_without_a_capacity_takes_the_slab_path(zen, oracle):
    """TensorPartition.load_balance(tensor) as the reference calls it (tensor_load_balance.py:43): the capacity
    it works out for itself keeps a bucket-sized, sparse tensor on the bucket-slab path, and the result is the
    oracle's."""
    from zen_repro_amd import _lib

    L = _lib.lib()
    n, P = 1 << 26, 16  # a 128 MB bf16 bucket (run_all.sh:22)
    g_np = make_grad(oracle, n, 0.005, "bf16", seed=21)
    grad = to_dev(g_np)
    tp = zen.TensorPartition(P, 1, 3)
    cap = tp._honest_capacity(grad, None, 0)
    m, _ = tp.table_sizes(n)
    assert cap < n // 100
    assert on_fast_path(L.zen_load_balance_path(n, m, _lib.BF16, cap, P, 0, _lib.MODE_FAST | FLAGS))
    assert L.zen_load_balance_workspace(n, m, _lib.BF16, cap, P) < 1 << 28
    indices, values, splits = tp.load_balance(grad)
    idx_o, val_o, splits_o, st_o = oracle.load_balance(g_np, P, 1, 3)
    assert st_o == 0
    assert np.array_equal(splits.cpu().numpy(), splits_o)
    assert np.array_equal(torch.cat(indices).cpu().numpy(), idx_o)
    assert np.array_equal(to_np(torch.cat(values)), val_o)
    # with a threshold: the count that came with it sizes the call
    thr = zen.topk_threshold(grad, 200_000)
    assert tp._honest_capacity(grad, thr, 0) == int(thr[1].item()) + 1024
    indices, values, splits = tp.load_balance(grad, thr=thr)
    masked, kept = oracle.mask_dense(g_np, int(thr[0].item()))
    idx_o, val_o, splits_o, st_o = oracle.load_balance(masked, P, 1, 3)
    assert int(splits.sum()) == kept and np.array_equal(torch.cat(indices).cpu().numpy(), idx_o)


def test_sample_taken_ahead_gives_the_same_result(zen, oracle):
    """TensorPartition.prepare takes a top-k call's sample on another stream before the call: same bytes out
    as without, over several calls in a row with the two sets of sampling memory in turn, also when a sample
    is taken for a call that never comes (it is dropped), and the table is all zero afterwards."""
    from zen_repro_amd import _lib

    n, P = 1 << 25, 16
    rng = np.random.default_rng(31)
    side = torch.cuda.Stream()
    tp = zen.TensorPartition(P, 1, 3)
    grads, wants = [], []
    for i in range(3):
        g_np = oracle.f32_to_bf16_bits((rng.standard_normal(n) * 1e-3).astype(np.float32))
        k = n // 200 + 1000 * i
        key = oracle.kth_key(g_np, k)
        masked, kept = oracle.mask_dense(g_np, key)
        grads.append((to_dev(g_np), k, int(k * 1.25) + 4096))
        wants.append(oracle.load_balance(masked, P, 1, 3))
    torch.cuda.synchronize()
    m, _ = tp.table_sizes(n)
    assert on_fast_path(_lib.lib().zen_load_balance_path(n, m, _lib.BF16, grads[0][2], P, grads[0][1], _lib.MODE_FAST | FLAGS))

    def check(out, want):
        idx, val, splits, st = out
        idx_o, val_o, splits_o, st_o = want
        assert int(st.item()) == 0 and st_o == 0
        total = int(splits.sum())
        assert np.array_equal(splits.cpu().numpy(), splits_o)
        assert np.array_equal(idx[:total].cpu().numpy(), idx_o) and np.array_equal(to_np(val[:total]), val_o)

    # call i's sample is taken while call i - 1 is still being enqueued / running
    with torch.cuda.stream(side):
        tp.prepare(*grads[0])
    outs = []
    for i in range(6):
        g, k, cap = grads[i % 3]
        outs.append(tp.load_balance_flat(g, None, cap, k=k))
        if i + 1 < 6:
            with torch.cuda.stream(side):
                tp.prepare(*grads[(i + 1) % 3])
    for i, out in enumerate(outs):
        check(out, wants[i % 3])
    # a sample whose call comes later: the calls in between (other buckets on the same slot) leave it alone and
    # sample for themselves, in the other set of sampling memory
    with torch.cuda.stream(side):
        tp.prepare(*grads[1])
    g, k, cap = grads[2]
    check(tp.load_balance_flat(g, None, cap, k=k), wants[2])
    check(tp.load_balance_flat(grads[0][0], None, grads[0][2], k=grads[0][1]), wants[0])
    state = tp._ahead_state(g.device, 0)
    assert len(state["pending"]) == 1
    check(tp.load_balance_flat(grads[1][0], None, grads[1][2], k=grads[1][1]), wants[1])
    assert not state["pending"]
    # both sets hold samples of calls still to come and a third bucket turns up: the older sample gives way
    with torch.cuda.stream(side):
        tp.prepare(*grads[1])
        tp.prepare(*grads[2])
    assert len(state["pending"]) == 2
    check(tp.load_balance_flat(grads[0][0], None, grads[0][2], k=grads[0][1]), wants[0])
    assert len(state["pending"]) == 1
    check(tp.load_balance_flat(grads[1][0], None, grads[1][2], k=grads[1][1]), wants[1])  # samples again
    check(tp.load_balance_flat(g, None, cap, k=k), wants[2])                                # picks its sample up
    assert not state["pending"]
    torch.cuda.synchronize()
    assert int(tp._table(g.device, m).count_nonzero()) == 0


def test_step_replayed_from_a_captured_graph(zen, oracle):
    """An encode (fused top-k) and a merge captured into a HIP graph, the merge forked onto a second stream:
    every replay, with eager calls on the same workspaces and a synchronisation in between, leaves the bytes
    the eager call leaves (the calls record kernels only: nothing a replay would skip or do twice)."""
    from zen_repro_amd import _lib

    n, P = 1 << 25, 16
    rng = np.random.default_rng(41)
    g_np = oracle.f32_to_bf16_bits((rng.standard_normal(n) * 1e-3).astype(np.float32))
    k = n // 200
    cap = int(k * 1.25) + 4096
    key = oracle.kth_key(g_np, k)
    masked, _ = oracle.mask_dense(g_np, key)
    idx_o, val_o, splits_o, st_o = oracle.load_balance(masked, P, 1, 3)
    per_peer = k // P
    peers_i = [rng.choice(n - 1, per_peer, replace=False).astype(np.int32) + 1 for _ in range(P)]
    flat_i = np.concatenate(peers_i)
    flat_v = oracle.f32_to_bf16_bits((rng.standard_normal(flat_i.size) * 1e-3).astype(np.float32))
    want_i, want_v = oracle.merge_sparse(flat_i, flat_v, n)
    grad, fi, fv = to_dev(g_np), to_dev(flat_i), to_dev(flat_v)
    tp = zen.TensorPartition(P, 1, 3)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P), None, None)
    m, _ = tp.table_sizes(n)
    assert on_fast_path(_lib.lib().zen_load_balance_path(n, m, _lib.BF16, cap, P, k, _lib.MODE_FAST | FLAGS))
    assert on_fast_path(_lib.lib().zen_merge_path(flat_i.size, n, _lib.MODE_FAST | FLAGS))

    def check(enc, mrg):
        idx, val, splits, st = enc
        m_idx, m_val, m_count, m_st = mrg
        assert int(st.item()) == 0 and int(m_st.item()) == 0
        total = int(splits.sum())
        assert np.array_equal(splits.cpu().numpy(), splits_o)
        assert np.array_equal(idx[:total].cpu().numpy(), idx_o) and np.array_equal(to_np(val[:total]), val_o)
        u = int(m_count.item())
        assert u == len(want_i) and np.array_equal(m_idx[:u].cpu().numpy(), want_i.astype(np.int32))
        assert np.array_equal(m_val[:u].cpu().numpy().view(np.uint32), want_v.view(np.uint32))

    def eager():
        return (tp.load_balance_flat(grad, None, cap, k=k),
                lba.merge_sparse_flat(fi, fv, n, capacity=flat_i.size))

    check(*eager())  # also makes the workspaces, outside the capture
    torch.cuda.synchronize()
    side, cap_stream = torch.cuda.Stream(), torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=cap_stream):
        cur = torch.cuda.current_stream()
        _lib.zeros.fresh(grad.device)
        side.wait_stream(cur)
        enc = tp.load_balance_flat(grad, None, cap, k=k)
        with torch.cuda.stream(side):
            _lib.zeros.fresh(grad.device)
            mrg = lba.merge_sparse_flat(fi, fv, n, capacity=flat_i.size)
        cur.wait_stream(side)
    _lib.zeros.fresh(grad.device)
    for s_ in (side, cap_stream):
        with torch.cuda.stream(s_):
            _lib.zeros.fresh(grad.device)
    for _ in range(3):
        enc[0].fill_(-1)
        mrg[0].fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        check(enc, mrg)
        check(*eager())  # the same tables and workspaces, between two replays
        torch.cuda.synchronize()
    assert int(tp._table(grad.device, m).count_nonzero()) == 0


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_threshold_of_an_earlier_call_replaces_the_sample(zen, oracle, dtype):
    """load_balance_flat(..., k, near=thr_out of an earlier call): no sample kernel, same bytes out, on the
    same gradient and on gradients a few per cent larger and smaller; a key that is far off (the gradient
    halved or doubled) makes the call decline (STAT_RETRY) or still gives the exact answer, never a wrong one."""
    from zen_repro_amd import _lib

    n, P = 1 << 24, 16
    rng = np.random.default_rng(53)
    base = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    k = n // 200
    cap = int(k * 1.25) + 4096
    tp = zen.TensorPartition(P, 1, 3)
    m, _ = tp.table_sizes(n)
    code = _lib.BF16 if dtype == "bf16" else _lib.F32
    assert on_fast_path(_lib.lib().zen_load_balance_path(n, m, code, cap, P, k, _lib.MODE_FAST | FLAGS))

    def bits(x):
        return oracle.f32_to_bf16_bits(x) if dtype == "bf16" else x

    def want(g_np):
        key = oracle.kth_key(g_np, k)
        masked, _ = oracle.mask_dense(g_np, key)
        return key, oracle.load_balance(masked, P, 1, 3)

    g0 = bits(base)
    thr_out = torch.zeros(2, dtype=torch.int32, device="cuda")
    g0_dev = to_dev(g0)
    dev = g0_dev.device
    first = tp.load_balance_flat(g0_dev, None, cap, k=k, thr_out=thr_out)
    key0, w0 = want(g0)
    assert int(first[3].item()) == 0 and int(thr_out[0].item()) == key0
    near = thr_out.clone()
    exact = 0
    for scale in (1.0, 1.02, 0.98, 0.5, 2.0):
        g_np = bits((base * np.float32(scale)).astype(np.float32))
        key, (idx_o, val_o, splits_o, st_o) = want(g_np)
        thr_now = torch.zeros(2, dtype=torch.int32, device="cuda")
        idx, val, splits, st = tp.load_balance_flat(to_dev(g_np), None, cap, k=k, thr_out=thr_now, near=near)
        status = int(st.item())
        if status & (_lib.STAT_RETRY | _lib.STAT_INTERNAL):
            assert scale in (0.5, 2.0), f"declined at scale {scale}"
            tp._table(dev, m).zero_()  # a declined call leaves the table for its caller to clear
            continue
        assert status == 0 and st_o == 0
        total = int(splits.sum())
        assert int(thr_now[0].item()) == key
        assert np.array_equal(splits.cpu().numpy(), splits_o)
        assert np.array_equal(idx[:total].cpu().numpy(), idx_o) and np.array_equal(to_np(val[:total]), val_o)
        exact += 1
    assert exact >= 3
    torch.cuda.synchronize()
    assert int(tp._table(dev, m).count_nonzero()) == 0


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_encode_and_merge_in_one_call(zen, oracle, dtype):
    """encode_merge_flat (zen_encode_merge) against the two calls it stands for, bit for bit: a top-k bucket and
    the entries received for it, twice in a row (the second call finds every counter where the first left it),
    then with a sample taken ahead, and with the merge on a stream of its own."""
    from zen_repro_amd import _lib

    n, P, k = 1 << 25, 16, (1 << 25) // 100
    g = make_grad(oracle, n, 1.0, dtype, seed=31)
    rng = np.random.default_rng(5)
    ci, cv = payloads(oracle, rng, n, P, 20000, 0.25, dtype)
    ci = ci.astype(np.int32)
    cap = int(k * 1.25) + 4096
    d, di, dv = to_dev(g), to_dev(ci), to_dev(cv)
    tp = zen.TensorPartition(P, 1, 3)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P), None, None)
    e0 = tp.load_balance_flat(d, None, cap, k=k, slot=1)
    m0 = lba.merge_sparse_flat(di, dv, n, slot=1)
    torch.cuda.synchronize()
    assert e0[3].item() == 0 and m0[3].item() == 0
    total, cnt = int(e0[2].sum()), int(m0[2])
    side = torch.cuda.Stream()

    def same(e, m):
        torch.cuda.synchronize()
        assert e[3].item() == 0 and m[3].item() == 0
        assert torch.equal(e[2], e0[2]) and int(m[2]) == cnt
        assert torch.equal(e[0][:total], e0[0][:total]) and torch.equal(to_dev(to_np(e[1][:total])), to_dev(to_np(e0[1][:total])))
        assert torch.equal(m[0][:cnt], m0[0][:cnt]) and torch.equal(m[1][:cnt].view(torch.int32), m0[1][:cnt].view(torch.int32))

    for rep in range(2):
        same(*lba.encode_merge_flat(tp, d, cap, k, di, dv, n))
    tp.prepare(d, k, cap)
    same(*lba.encode_merge_flat(tp, d, cap, k, di, dv, n))
    side.wait_stream(torch.cuda.current_stream())
    same(*lba.encode_merge_flat(tp, d, cap, k, di, dv, n, merge_stream=side))
    torch.cuda.current_stream().wait_stream(side)
    m, _ = oracle.table_sizes(n, P, 1)
    assert not tp._table(d.device, m).any()


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_sample_taken_along_by_the_call_before(zen, oracle, dtype):
    """encode_merge_flat(..., next_tensor=): the pass over one bucket takes the next bucket's sample along.  Four
    different gradients in a row on one slot, the third of another size (with its own k, capacity and table),
    each call handed its successor; every result equals the oracle's (so the floor the call before left behind
    selected nothing wrong), and every call after the first picks its sample up (no sample kernel of its own is
    launched: counted)."""
    from zen_repro_amd import _lib

    n, P = 1 << 24, 16
    sizes = [n, n, n // 4 * 3, n]
    ks = [s // 200 for s in sizes]
    caps = [int(k * 1.25) + 4096 for k in ks]
    grads = [make_grad(oracle, s, 1.0, dtype, seed=41 + i) for i, s in enumerate(sizes)]
    rng = np.random.default_rng(9)
    ci, cv = payloads(oracle, rng, n, P, 9000, 0.25, dtype)
    ci = ci.astype(np.int32)
    ds = [to_dev(g) for g in grads]
    di, dv = to_dev(ci), to_dev(cv)
    tp = zen.TensorPartition(P, 1, 3)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P), None, None)
    for s_, k_, c_ in zip(sizes, ks, caps):
        m, _ = oracle.table_sizes(s_, P, 1)
        assert on_fast_path(_lib.lib().zen_load_balance_path(s_, m, _lib.dtype_code(ds[0]), c_, P, k_, _lib.MODE_FAST | FLAGS))
    want_m = oracle.merge_sparse(ci, cv, n)
    _lib.profile_enable(True)
    outs = []
    for i in range(4):
        more = i + 1 < 4
        outs.append(lba.encode_merge_flat(tp, ds[i], caps[i], ks[i], di, dv, n, next_tensor=ds[i + 1] if more else None,
                                          next_k=ks[i + 1] if more else None,
                                          next_capacity=caps[i + 1] if more else None))
    torch.cuda.synchronize()
    launched = _lib.profile_read()
    _lib.profile_enable(False)
    assert launched["k_sample_hist"][1] == 1 and launched["k_select_stage"][1] == 4  # only the first call sampled for itself
    state = tp._ahead_state(ds[0].device, 0)
    assert state is not None and not state["pending"]
    for i, (e, mg) in enumerate(outs):
        assert e[3].item() == 0 and mg[3].item() == 0
        key = oracle.kth_key(grads[i], ks[i])
        sel, _ = oracle.mask_dense(grads[i], key)
        idx_o, val_o, splits_o, st_o = oracle.load_balance(sel, P, 1, 3)
        total = int(splits_o.sum())
        assert st_o == 0 and np.array_equal(to_np(e[2]), splits_o)
        assert np.array_equal(to_np(e[0])[:total], idx_o) and np.array_equal(to_np(e[1])[:total], val_o)
        cnt = int(mg[2])
        assert cnt == len(want_m[0]) and np.array_equal(to_np(mg[0])[:cnt], want_m[0].astype(np.int32))
        assert np.array_equal(to_np(mg[1])[:cnt].view(np.uint32), want_m[1].view(np.uint32))
    for s_ in set(sizes):
        assert not tp._table(ds[0].device, oracle.table_sizes(s_, P, 1)[0]).any()
    # a successor whose sizes take no path that keeps a sample is refused by the library, and not offered by the wrapper
    small = ds[0][: 1 << 12]
    e, _ = lba.encode_merge_flat(tp, ds[0], caps[0], ks[0], di, dv, n, next_tensor=small, next_k=20, next_capacity=64)
    assert e[3].item() == 0 and not tp._ahead_state(ds[0].device, 0)["pending"]
