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
