"""Parity of the bitmap index codec (comm.py:59-99) against the CPU oracle
(itself pinned by numpy.packbits), its edge cases, a full-size round trip, and
the whole sparse all-reduce (comm.py:101-150, methods 1-3) with four ranks
played by four host threads on the one GPU.  Bar: bit-exact bitmaps and
indices; summed values within 1e-6 of the summed magnitudes (fp32) or one
bf16 rounding of the fp32 sum."""
import threading

import numpy as np
import pytest
import torch

from gpu_util import to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def zen():
    import zen_repro_amd
    from zen_repro_amd import _lib

    _lib.lib()
    assert torch.cuda.is_available()
    return zen_repro_amd


def lba_with_mapping(zen, n, P, rank):
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P, rank), None, None)
    lba.mapping[n] = lba.calculate_mapping(n)
    return lba


@pytest.mark.parametrize("idx_dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("n,P,rank,frac", [
    (1 << 12, 8, 3, 0.05),
    (1 << 20, 4, 0, 0.01),
    (1 << 20, 4, 3, 0.5),          # every second member
    (6000000, 3, 1, 0.001),        # partitions not a power of two
    ((1 << 22) + 40, 8, 7, 1.0),   # all members; list length not a multiple of 8
])
def test_bitmap_matches_oracle(zen, oracle, n, P, rank, frac, idx_dtype):
    n = n // P * P
    lba = lba_with_mapping(zen, n, P, rank)
    mp = oracle.mapping(n, P)
    for p in range(P):  # the lists themselves are the oracle's
        assert np.array_equal(to_np(lba.mapping[n][p]), mp[p])
    members = mp[rank]
    rng = np.random.default_rng(n ^ P ^ rank)
    pick = np.sort(rng.choice(members, max(1, int(len(members) * frac)), replace=False))
    want = oracle.bitmap_encode(members, pick)
    got = lba.encode_bitmap(to_dev(pick).to(idx_dtype), n)
    assert got.dtype == torch.uint8 and got.numel() == (len(members) + 7) // 8
    assert np.array_equal(to_np(got), want)
    # order of the indices does not matter, nor do repeats
    shuffled = np.concatenate([rng.permutation(pick), pick[:7]])
    assert np.array_equal(to_np(lba.encode_bitmap(to_dev(shuffled).to(idx_dtype), n)), want)
    # the same through the C-ABI without the rank table (search from an interpolated position)
    from zen_repro_amd import _lib

    L = _lib.lib()
    d_idx = to_dev(shuffled).to(idx_dtype)
    d_map = lba.mapping[n][rank]
    words = torch.full((L.zen_bitmap_words(len(members)),), -1, dtype=torch.int32, device="cuda")
    status = _lib.status_word("cuda")
    rc = L.zen_bitmap_encode(_lib.ptr(d_map), len(members), _lib.ptr(d_idx), int(idx_dtype == torch.int64),
                             d_idx.numel(), None, None, 0, _lib.ptr(words), _lib.ptr(status), _lib.stream_of("cuda"))
    assert rc == 0 and status.item() == 0
    assert np.array_equal(to_np(words.view(torch.uint8))[:len(want)], want)
    assert int(words.view(torch.uint8)[len(want):].sum()) == 0  # the padding up to a whole word is zero
    # decode: one bitmap per rank, each against that rank's list
    lba0 = lba_with_mapping(zen, n, P, 0)
    bitmaps, wants = [], []
    for p in range(P):
        sel = np.sort(rng.choice(mp[p], max(1, len(mp[p]) // 50), replace=False))
        bm = oracle.bitmap_encode(mp[p], sel)
        # what allgather_padding hands back may be a view at any byte offset
        holder = torch.zeros(len(bm) + 3, dtype=torch.uint8, device="cuda")
        holder[1 + (p % 3):1 + (p % 3) + len(bm)] = to_dev(bm)
        bitmaps.append(holder[1 + (p % 3):1 + (p % 3) + len(bm)])
        wants.append(sel)
        assert np.array_equal(oracle.bitmap_decode(mp[p], bm), sel)
    outs = lba0.decode_bitmap(bitmaps, n)
    assert len(outs) == P
    for p in range(P):
        assert outs[p].dtype == torch.int64
        assert np.array_equal(to_np(outs[p]), wants[p])


def test_bitmap_edge_cases(zen, oracle):
    n, P, rank = 1 << 16, 4, 2
    lba = lba_with_mapping(zen, n, P, rank)
    members = oracle.mapping(n, P)[rank]
    nbytes = (len(members) + 7) // 8
    solo = zen.LoadBalanceAllreduce(zen.LocalGroup(P, 0), None, None)  # decodes against this one list
    solo.mapping[n] = [lba.mapping[n][rank]]
    # nothing selected
    empty = lba.encode_bitmap(torch.empty(0, dtype=torch.int64, device="cuda"), n)
    assert empty.numel() == nbytes and int(empty.sum()) == 0
    assert solo.decode_bitmap([empty], n)[0].numel() == 0
    # an index that is no member marks the next member (searchsorted, left side)
    gap = np.setdiff1d(np.arange(members[5] + 1, members[-1]), members)[:9]
    want = oracle.bitmap_encode(members, gap)
    assert np.array_equal(to_np(lba.encode_bitmap(to_dev(gap), n)), want)
    assert want.sum() > 0
    # first and last member, and the values around them
    ends = np.array([0, members[0], members[-1]], dtype=np.int64)
    assert np.array_equal(to_np(lba.encode_bitmap(to_dev(ends), n)), oracle.bitmap_encode(members, ends))
    # beyond the last member: the reference indexes one past the end of its mask
    with pytest.raises(IndexError):
        lba.encode_bitmap(to_dev(np.array([members[-1] + 1], dtype=np.int64)), n)
    # a device-side count limits what is read
    pick = members[::3].copy()
    count = torch.tensor([100], dtype=torch.int64, device="cuda")
    bm, status = lba.encode_bitmap_flat(to_dev(pick), n, count=count)
    assert status.item() == 0
    assert np.array_equal(to_np(bm), oracle.bitmap_encode(members, pick[:100]))
    # padding after the last byte is ignored, bits past the last member too; a short bitmap is refused
    full = oracle.bitmap_encode(members, members)
    padded = np.concatenate([full, np.full(5, 0xFF, dtype=np.uint8)])
    padded[nbytes - 1] = 0xFF
    assert np.array_equal(to_np(solo.decode_bitmap([to_dev(padded)], n)[0]), members)
    with pytest.raises(IndexError):
        solo.decode_bitmap([to_dev(full[:-1])], n)


def test_bitmap_full_size_round_trip(zen):
    """c3's index space (743 M, 16 partitions): the merged indices of rank 0's
    received payloads -> bitmap -> indices, and the bitmap against the
    reference's own recipe (searchsorted, mask, weights 1..128) in torch ops."""
    from zen_repro_amd import workloads

    cfg, grad = workloads.make("c3", device="cuda", seed=0, shrink=1)
    del grad
    n, P = cfg.n, cfg.partitions
    lba = lba_with_mapping(zen, n, P, 0)
    members = lba.mapping[n][0]
    assert sum(m.numel() for m in lba.mapping[n]) == n
    _, _, flat_idx, flat_val = workloads.peer_payloads(cfg, cfg.k // P, device="cuda", seed=1)
    m_idx, _ = lba.merge_sparse(flat_idx, flat_val, n)
    bitmap = lba.encode_bitmap(m_idx, n)
    pos = torch.searchsorted(members, m_idx)
    mask = torch.zeros(members.numel() + 7, dtype=torch.uint8, device="cuda")
    mask[pos] = 1
    weights = 2 ** torch.arange(8, dtype=torch.uint8, device="cuda")
    want = (mask[:(members.numel() + 7) // 8 * 8].view(-1, 8) * weights).sum(dim=1).to(torch.uint8)
    assert torch.equal(bitmap, want)
    back = lba.decode_bitmap([bitmap], n)[0]
    assert torch.equal(back, m_idx)


class ThreadExchange:
    """The reference backend's calls (DDPbackend.py:13-41, 71-81) between host
    threads that each play one rank on the same GPU."""

    def __init__(self, size):
        self.size = size
        self.barrier = threading.Barrier(size)
        self.slots = [None] * size

    def view(self, rank):
        return _RankView(self, rank)

    def exchange(self, rank, item):
        torch.cuda.current_stream().synchronize()
        self.slots[rank] = item
        self.barrier.wait()
        got = list(self.slots)
        self.barrier.wait()
        return got


class _RankView:
    def __init__(self, ex, rank):
        self.ex, self.rank = ex, rank

    def allgather(self, tensor, async_op=True):
        return [t.clone() for t in self.ex.exchange(self.rank, tensor)]

    def allgather_padding(self, tensor, async_op=True):
        return [t.clone() for t in self.ex.exchange(self.rank, tensor)]

    def alltoallv(self, tensors, gather_splits):
        everyone = self.ex.exchange(self.rank, tensors)
        got = [everyone[src][self.rank].clone() for src in range(self.ex.size)]
        for src in range(self.ex.size):
            assert got[src].numel() == int(gather_splits[src][self.rank])
        return got


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("method", [1, 2, 3])
def test_sparse_allreduce_between_four_ranks(zen, method, dtype):
    """Every rank ends with the sum of all ranks' sparse tensors."""
    P, n = 4, 1 << 20
    gen = torch.Generator(device="cuda").manual_seed(7 + method)
    tensors = []
    for r in range(P):
        g = torch.randn(n, device="cuda", generator=gen) * 1e-3
        keep = torch.rand(n, device="cuda", generator=gen) < 0.01
        shared = torch.rand(n, device="cuda", generator=gen) < 0.002  # positions several ranks hold
        if r == 0:
            common = shared
        tensors.append(torch.where(keep | common, g, torch.zeros_like(g)).to(dtype))
    ex = ThreadExchange(P)
    results, errors = [None] * P, []

    def run(rank):
        try:
            torch.cuda.set_device(0)
            lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P, rank), None, None)
            lba.ddp = ex.view(rank)
            results[rank] = lba.zen_sparse_comm(tensors[rank], method)
            torch.cuda.current_stream().synchronize()
        except BaseException as e:  # noqa: BLE001 - reported below, and the others must not wait for ever
            errors.append((rank, repr(e)))
            ex.barrier.abort()

    threads = [threading.Thread(target=run, args=(r,)) for r in range(P)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    total = torch.stack([t.double() for t in tensors]).sum(dim=0)
    scale = torch.stack([t.double().abs() for t in tensors]).sum(dim=0)
    for r in range(P):
        out = results[r]
        assert out.dtype == dtype and out.numel() == n
        assert torch.equal(out != 0, total != 0)
        err = (out.double() - total).abs()
        tol = scale * (1e-6 if dtype == torch.float32 else 2.0 ** -7)
        assert bool((err <= tol).all())
        assert torch.equal(out, results[0])


# ---------------------------------------------- bitmaps + values -> dense in one pass


def _shards(oracle, n, P, frac, dtype, seed):
    """Per rank: (members of its partition that are present, their values), as the merge of the first
    exchange would leave them: ascending indices of partition p, nonzero values."""
    rng = np.random.default_rng(seed)
    mp = oracle.mapping(n, P)
    idx, val = [], []
    for p in range(P):
        take = max(1, int(len(mp[p]) * frac))
        pick = np.sort(rng.choice(mp[p], take, replace=False))
        v = (rng.standard_normal(take) * 1e-3).astype(np.float32)
        v[v == 0] = 1e-3
        idx.append(pick)
        val.append(oracle.f32_to_bf16_bits(v) if dtype == "bf16" else v)
    return mp, idx, val


def _dense_truth(oracle, n, idx, val):
    """oracle.decode of all lists (fp32 accumulation, rounded once to the values' type)."""
    flat_i, flat_v = np.concatenate(idx), np.concatenate(val)
    f32 = oracle.decode(flat_i, flat_v, n, "f32acc")
    return oracle.f32_to_bf16_bits(f32) if flat_v.dtype == np.uint16 else f32


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("n,P,frac", [
    (1 << 16, 4, 0.05),
    ((1 << 20) + 48, 16, 0.06),      # a last tile that is not full
    (3000000, 3, 0.3),               # partitions not a power of two, n % 8192 != 0
    (1 << 20, 64, 0.02),             # the most lists the kernel takes
    (1 << 19, 2, 0.9),               # nearly every member present
    (1003 * 7, 7, 0.5),              # below one tile per ... and n % P == 0 with odd sizes
])
def test_bitmaps_to_dense_in_one_pass_matches_oracle(zen, oracle, n, P, frac, dtype):
    n = n // P * P
    mp, idx, val = _shards(oracle, n, P, frac, dtype, seed=n + P)
    bitmaps = [oracle.bitmap_encode(mp[p], idx[p]) for p in range(P)]
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P, 0), None, None)
    got = lba.decode_bitmaps_dense([to_dev(b) for b in bitmaps], [to_dev(v) for v in val], n)
    want = _dense_truth(oracle, n, idx, val)
    assert got.numel() == n and np.array_equal(to_np(got), want)
    # the two-step path of the reference (decode_bitmap, then decode_sparse_tensors) gives the same bytes
    lba.mapping[n] = lba.calculate_mapping(n)
    idx_lists = lba.decode_bitmap([to_dev(b) for b in bitmaps], n)
    for p in range(P):
        assert np.array_equal(to_np(idx_lists[p]), idx[p])
    two_step = lba.decode_sparse_tensors(idx_lists, [to_dev(v) for v in val], n, ascending=True)
    assert torch.equal(two_step.view(torch.int16 if dtype == "bf16" else torch.int32),
                       got.view(torch.int16 if dtype == "bf16" else torch.int32))
    # a second call on the cached dictionary, other data
    mp, idx, val = _shards(oracle, n, P, frac / 2, dtype, seed=n + P + 1)
    bitmaps = [oracle.bitmap_encode(mp[p], idx[p]) for p in range(P)]
    got = lba.decode_bitmaps_dense([to_dev(b) for b in bitmaps], [to_dev(v) for v in val], n)
    assert np.array_equal(to_np(got), _dense_truth(oracle, n, idx, val))


def test_bitmaps_to_dense_edge_cases(zen, oracle):
    n, P = 1 << 18, 8
    mp, idx, val = _shards(oracle, n, P, 0.1, "f32", seed=3)
    bitmaps = [oracle.bitmap_encode(mp[p], idx[p]) for p in range(P)]
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P, 0), None, None)
    want = _dense_truth(oracle, n, idx, val)
    # padding behind a bitmap (allgather_padding pads to the longest, DDPbackend.py:26-41; garbage bits past the
    # list's length are ignored, comm.py:97) and lists that do not sit in one buffer
    padded = [np.concatenate([b, np.full(5 + p, 0xFF, np.uint8)]) for p, b in enumerate(bitmaps)]
    last_bits = [len(mp[p]) % 8 for p in range(P)]
    for p in range(P):  # garbage in the unused bits of the last byte too
        if last_bits[p]:
            padded[p][len(bitmaps[p]) - 1] |= np.uint8((0xFF << last_bits[p]) & 0xFF)
    got = lba.decode_bitmaps_dense([to_dev(b) for b in padded], [to_dev(v) for v in val], n)
    assert np.array_equal(to_np(got), want)
    # -0.0 among the values becomes +0.0, as 0 + (-0) does in scatter_add_; NaN stays
    val2 = [v.copy() for v in val]
    val2[0][0] = -0.0
    val2[1][0] = np.nan
    got = to_np(lba.decode_bitmaps_dense([to_dev(b) for b in bitmaps], [to_dev(v) for v in val2], n))
    assert got.view(np.uint32)[idx[0][0]] == 0 and np.isnan(got[idx[1][0]])
    # an empty list (no bit set, no values)
    empty = [b.copy() for b in bitmaps]
    empty[2][:] = 0
    vals3 = [v if p != 2 else v[:0] for p, v in enumerate(val)]
    got = to_np(lba.decode_bitmaps_dense([to_dev(b) for b in empty], [to_dev(v) for v in vals3], n))
    want3 = want.copy()
    want3[idx[2]] = 0
    assert np.array_equal(got, want3)
    # a bitmap shorter than its list, and fewer values than set bits: the reference raises an index error
    short = [b if p != 1 else b[:-2] for p, b in enumerate(bitmaps)]
    with pytest.raises(IndexError):
        lba.decode_bitmaps_dense([to_dev(b) for b in short], [to_dev(v) for v in val], n)
    fewer = [v if p != 3 else v[:-1] for p, v in enumerate(val)]
    with pytest.raises(IndexError):
        lba.decode_bitmaps_dense([to_dev(b) for b in bitmaps], [to_dev(v) for v in fewer], n)
    # n % P != 0: some indices belong to no list (hash_index gives P for them, functions_cuda_kernel.cu:172-175)
    n2, P2 = 100003, 4
    part = oracle.hash_index(n2, P2)
    mp2 = oracle.mapping(n2, P2)
    rng = np.random.default_rng(8)
    idx2 = [np.sort(rng.choice(m, len(m) // 3, replace=False)) for m in mp2]
    val2 = [(rng.standard_normal(len(i)) * 1e-3).astype(np.float32) + 1.0 for i in idx2]
    bm2 = [oracle.bitmap_encode(mp2[p], idx2[p]) for p in range(P2)]
    lba2 = zen.LoadBalanceAllreduce(zen.LocalGroup(P2, 0), None, None)
    got = to_np(lba2.decode_bitmaps_dense([to_dev(b) for b in bm2], [to_dev(v) for v in val2], n2))
    assert np.array_equal(got, _dense_truth(oracle, n2, idx2, val2)) and (got[part == P2] == 0).all()


# ---------------------------------------------------------- the DDP hook


class _StubBucket:
    """What the hook asks of a dist.GradBucket: its flat buffer (train.py:168)."""

    def __init__(self, tensor):
        self._t = tensor

    def buffer(self):
        return self._t


def test_comm_hook_on_one_rank(zen, oracle):
    """custom_comm_hook (train.py:167-183) with a stub bucket: the first call passes the bucket through, later
    ones return a completed future holding the compressed bucket (one rank: no exchange, train.py:178); the
    compression is the reference's sampled threshold with the sample positions given."""
    n = 1 << 20
    gen = torch.Generator(device="cuda").manual_seed(11)
    grad = (torch.randn(n, device="cuda", generator=gen) * 1e-3).to(torch.bfloat16)
    sample = torch.randint(0, n, ((n + 99) // 100,), device="cuda", generator=gen)
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(1, 0), None, None)
    hook = zen.SparseCommHook(lba, top_k=5, method=3, tp_group=zen.LocalGroup(1, 0), sample_index=lambda numel: sample)
    first = hook(None, _StubBucket(grad))
    assert first.done() and first.value() is grad  # train.py:170-174
    fut = hook(None, _StubBucket(grad))
    assert isinstance(fut, torch.futures.Future) and fut.done()
    out = fut.value()
    hook.stream.synchronize()
    # the reference's rule on the CPU: threshold = smallest of the top 5 % of the sampled magnitudes
    g = grad.float().cpu()
    s = g.abs()[sample.cpu()]
    thr = torch.topk(s, s.numel() * 5 // 100, largest=True, sorted=False)[0].min()
    want = torch.where(g.abs() >= thr, g, torch.zeros(())).to(torch.bfloat16)
    assert out.dtype == grad.dtype and torch.equal(out.cpu().view(torch.int16), want.view(torch.int16))
    # buckets of at most 4096 elements pass through (train.py:58-59)
    small = grad[:4096].clone()
    assert hook(None, _StubBucket(small)).value() is small


@pytest.mark.parametrize("method,fused", [(3, True), (3, False), (2, True), (1, True)])
def test_comm_hook_between_four_ranks(zen, method, fused):
    """The hook end to end with four ranks played by host threads: every rank's future holds the sum of all
    ranks' compressed buckets (method 3: buckets exchanged, merged, sent round as bitmaps and decoded in one
    pass), whether the threshold is handed to the all-reduce (fused) or applied to a copy of the bucket first
    as in the reference."""
    P, n = 4, 1 << 20
    gen = torch.Generator(device="cuda").manual_seed(5)
    grads = [(torch.randn(n, device="cuda", generator=gen) * 1e-3) for _ in range(P)]
    samples = [torch.randint(0, n, ((n + 99) // 100,), device="cuda", generator=gen) for _ in range(P)]
    ex = ThreadExchange(P)
    results, compressed, errors = [None] * P, [None] * P, []

    def run(rank):
        try:
            torch.cuda.set_device(0)
            lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P, rank), None, None)
            lba.ddp = ex.view(rank)
            hook = zen.SparseCommHook(lba, top_k=2, method=method, tp_group=zen.LocalGroup(1, 0),
                                      sample_index=lambda numel, r=rank: samples[r], fused=fused)
            hook(None, _StubBucket(grads[rank]))  # the first call is passed through
            compressed[rank] = zen.compress_with_allgather(2, grads[rank], zen.LocalGroup(1, 0), sample_index=samples[rank])
            results[rank] = hook(None, _StubBucket(grads[rank])).value()
            hook.stream.synchronize()
            torch.cuda.current_stream().synchronize()
        except BaseException as e:  # noqa: BLE001
            errors.append((rank, repr(e)))
            ex.barrier.abort()

    threads = [threading.Thread(target=run, args=(r,)) for r in range(P)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    total = torch.stack([c.double() for c in compressed]).sum(dim=0)
    scale = torch.stack([c.double().abs() for c in compressed]).sum(dim=0)
    for r in range(P):
        out = results[r]
        assert out.numel() == n and torch.equal(out != 0, total != 0)
        assert bool(((out.double() - total).abs() <= scale * 1e-6).all())
        assert torch.equal(out, results[0])


@pytest.mark.parametrize("fused,headroom", [(True, 1.5), (True, 0.05), (False, 1.5)])
def test_comm_hook_on_a_bucket_of_training_size(zen, fused, headroom):
    """The hook between two ranks on a bucket of 64 Mi bf16 elements, the size at which the load balance takes
    its fast paths (asserted), with the threshold handed to the all-reduce (fused), with far too little room
    for the selection (the call is declined, falls back, learns the size and starts again), and the reference's
    way (masked copy first): all three give every rank the same tensor, the sum of the ranks' compressed
    buckets."""
    from zen_repro_amd import _lib

    P, n, top_k = 2, 64 << 20, 1
    gen = torch.Generator(device="cuda").manual_seed(21)
    grads = [(torch.randn(n, device="cuda", generator=gen) * 1e-3).to(torch.bfloat16) for _ in range(P)]
    samples = [torch.randint(0, n, ((n + 99) // 100,), device="cuda", generator=gen) for _ in range(P)]
    L = _lib.lib()
    m = zen.TensorPartition(P, 1, 3).table_sizes(n)[0]
    room = int(n * top_k / 100 * 1.5) + 4096
    assert L.zen_load_balance_path(n, m, _lib.BF16, room, P, 0, _lib.MODE_FAST) >= 2
    ex = ThreadExchange(P)
    results, compressed, errors = [None] * P, [None] * P, []

    def run(rank):
        try:
            torch.cuda.set_device(0)
            lba = zen.LoadBalanceAllreduce(zen.LocalGroup(P, rank), None, None)
            lba.ddp = ex.view(rank)
            hook = zen.SparseCommHook(lba, top_k=top_k, method=3, tp_group=zen.LocalGroup(1, 0),
                                      sample_index=lambda numel, r=rank: samples[r], fused=fused, headroom=headroom)
            hook(None, _StubBucket(grads[rank]))  # the first call is passed through
            compressed[rank] = zen.compress_with_allgather(top_k, grads[rank], zen.LocalGroup(1, 0),
                                                           sample_index=samples[rank])
            results[rank] = hook(None, _StubBucket(grads[rank])).value()
            torch.cuda.current_stream().synchronize()  # the hook made this stream wait for its own
        except BaseException as e:  # noqa: BLE001
            errors.append((rank, repr(e)))
            ex.barrier.abort()

    threads = [threading.Thread(target=run, args=(r,)) for r in range(P)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=150)
    assert not errors, errors
    # two bf16 values per index at most: their fp32 sum rounded once to bf16
    want = (compressed[0].float() + compressed[1].float()).to(torch.bfloat16)
    want = torch.where(want == 0, torch.zeros((), dtype=torch.bfloat16, device="cuda"), want)  # no negative zeros
    for r in range(P):
        assert results[r].dtype == torch.bfloat16 and results[r].numel() == n
        assert torch.equal(results[r].view(torch.int16), want.view(torch.int16))


def test_comm_hook_needs_a_backend_for_more_than_one_rank(zen):
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(2, 0), None, None)
    hook = zen.SparseCommHook(lba, top_k=1, method=3, tp_group=zen.LocalGroup(1, 0))
    grad = torch.zeros(8192, device="cuda")
    hook(None, _StubBucket(grad))
    with pytest.raises(RuntimeError):
        hook(None, _StubBucket(grad))
