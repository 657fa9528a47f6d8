"""Synthetic inputs for the five benchmark configurations: the rank's own flat
gradient and the payloads P peers would send to one destination.  Everything
is drawn from a seeded torch generator on the requested device, so CPU tests
and GPU runs use the same code.  This is data synthesis only; nothing here is
on the encode/merge path."""
import math
from dataclasses import dataclass

import torch

_M32 = 0xFFFFFFFF
_D, _A, _B, _SEED1 = 573729859, 0xCC9E2D51, 0x1B873593, 10001861


def hash_slot(t, m):
    """Level-1 slot (h1(t) % m) of int64 indices t < 2^31, in int64 arithmetic:
    every product stays below 2^63 (functions_cuda_kernel.cu:80-88, :101)."""
    h = (_D * t) & _M32
    h = (((h + _A) & _M32) * t) & _M32
    h = (((h + _B) & _M32) * t) & _M32
    return ((h + _SEED1) & _M32) % m


@dataclass
class Config:
    name: str
    n: int
    dtype: torch.dtype
    partitions: int
    peers: int
    overlap: float
    k: int = 0            # > 0: exact top-k selection inside the timed path
    note: str = ""
    offset: int = 0       # where this bucket starts in the flat gradient make() returns
    parts: tuple = ()     # (name, offset, length, k) of the gradient buckets the tensor is handed over in
                          # (empty: one bucket, the whole tensor)


def buckets(cfg):
    """The gradient buckets of a configuration, each as a Config of its own
    (the reference's hook is called once per bucket, train.py:167-185, and
    hashes each with the bucket's own length)."""
    if not cfg.parts:
        return [cfg]
    return [Config(f"{cfg.name}/{name}", length, cfg.dtype, cfg.partitions, cfg.peers, cfg.overlap, k=k,
                   note=cfg.note, offset=offset) for name, offset, length, k in cfg.parts]


def _gen(seed, device):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def _normal(n, gen, device, sigma=1e-3, chunk=1 << 27):
    out = torch.empty(n, dtype=torch.float32, device=device)
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        out[lo:hi] = torch.randn(hi - lo, generator=gen, device=device) * sigma
    return out


def _zipf_distinct(universe, count, s, seed):
    """`count` distinct ids drawn with P(rank r) ~ r^-s: sampling without
    replacement is the distinct set of a with-replacement stream."""
    w = torch.arange(1, universe + 1, dtype=torch.float64).pow(-s)
    g = torch.Generator().manual_seed(seed)
    return torch.multinomial(w, count, replacement=False, generator=g)


def _row_sparse(rows, cols, active, s, gen, device, seed):
    flat = torch.zeros(rows * cols, dtype=torch.float32, device=device)
    ids = _zipf_distinct(rows, active, s, seed).to(device)
    vals = torch.randn(active, cols, generator=gen, device=device) * 1e-3
    flat.view(rows, cols)[ids] = vals
    return flat


def make(name, device="cuda", seed=0, shrink=1):
    """(Config, flat gradient tensor) for configuration c1..c5.  `shrink`
    divides the sizes (rows / elements) to get small parity-test cases."""
    gen = _gen(seed, device)
    if name == "c1":
        n = (1 << 20) // shrink
        cfg = Config("c1", n, torch.float32, 4, 4, 0.2, k=n // 100, note="flat fp32 N(0,1e-3), top 1%")
        return cfg, _normal(n, gen, device)
    if name == "c2":
        # two gradient buckets, as the hook would see them: the embedding (row-sparse, taken as it is) and the
        # dense rest, whose top 1 % the path itself has to find
        rows, cols = 50257 // shrink, 768
        rest = 85842432 // shrink // 16 * 16
        emb = _row_sparse(rows, cols, max(1, 2048 // shrink), 1.1, gen, device, seed + 1)
        g = torch.cat([emb, _normal(rest, gen, device)])
        del emb
        cfg = Config("c2", g.numel(), torch.float32, 16, 16, 0.3,
                     note="GPT-2-small: row-sparse embedding (nonzeros) + dense rest (top 1%)",
                     parts=(("embedding", 0, rows * cols, 0), ("rest", rows * cols, rest, max(1, rest // 100))))
        return cfg, g
    if name == "c3":
        n = 743440384 // shrink // 16 * 16
        cfg = Config("c3", n, torch.bfloat16, 16, 16, 0.25, k=int(n * 0.005),
                     note="Llama-3-8B embedding + one decoder layer, bf16, top 0.5%")
        g = torch.empty(n, dtype=torch.bfloat16, device=device)
        step = 1 << 27
        for lo in range(0, n, step):
            hi = min(n, lo + step)
            g[lo:hi] = (torch.randn(hi - lo, generator=gen, device=device) * 1e-3).to(torch.bfloat16)
        return cfg, g
    if name == "c4":
        n = (1 << 30) // shrink
        block = 4096
        nblocks = n // block
        w = torch.arange(1, nblocks + 1, dtype=torch.float64).pow(-1.3)
        want = (w / w.sum() * (0.01 * n)).clamp_(max=block)
        # mass that saturated blocks cannot hold spills to the next ranks
        spill = 0.01 * n - want.sum().item()
        room = block - want
        fill = torch.cumsum(room, 0)
        want = want + torch.where(fill <= spill, room, torch.zeros_like(room))
        prob = (want / block).to(torch.float32).to(device)
        g = torch.empty(n, dtype=torch.float32, device=device)
        per = max(1, (1 << 26) // block)
        for b0 in range(0, nblocks, per):
            b1 = min(nblocks, b0 + per)
            cnt = (b1 - b0) * block
            hit = torch.rand(cnt, generator=gen, device=device) < prob[b0:b1].repeat_interleave(block)
            vals = torch.randn(cnt, generator=gen, device=device) * 1e-3
            g[b0 * block:b1 * block] = torch.where(hit, vals, torch.zeros((), device=device))
        cfg = Config("c4", n, torch.float32, 32, 32, 0.0, note="Zipf(1.3) hot 4096-blocks, 1% nonzeros")
        return cfg, g
    if name == "c5":
        rows, cols = 256000 // shrink, 3072
        g = _row_sparse(rows, cols, max(1, 256 // shrink), 1.2, gen, device, seed + 1).to(torch.bfloat16)
        cfg = Config("c5", g.numel(), torch.bfloat16, 64, 64, 0.4, note="Gemma-7B embedding rows, 0.1%")
        return cfg, g
    raise ValueError(name)


def per_peer_entries(cfg, nnz):
    """Entries each of cfg.peers ranks sends to one destination when every rank selected about `nnz`: nnz / P,
    but never more than the destination's index range can supply (the payloads hold distinct indices of one
    partition, all but the shared fraction different from peer to peer)."""
    distinct_per_entry = cfg.overlap + cfg.peers * (1.0 - cfg.overlap)
    room = int((cfg.n // cfg.partitions) * 0.5 / distinct_per_entry)
    return max(1, min(nnz // cfg.partitions, room))


def peer_payloads(cfg, per_peer, dest=0, device="cuda", seed=1):
    """What `cfg.peers` ranks send to rank `dest`: per peer an (int32 indices,
    values) pair of `per_peer` entries whose partition is `dest`, a fraction
    `cfg.overlap` of them common to every peer, each payload in the slot order
    an encoder emits.  Returned as lists of views into two flat buffers (the
    layout a variable all-to-all into one buffer leaves, DDPbackend.py:76-81),
    plus those flat buffers."""
    n, parts = cfg.n, cfg.partitions
    assert n % parts == 0
    npp = n // parts
    gen = _gen(seed, device)
    n_pool = int(per_peer * cfg.overlap)
    n_own = per_peer - n_pool
    need = n_pool + cfg.peers * n_own
    if need > 0.9 * npp:
        raise ValueError(f"peer_payloads: {need} distinct indices wanted of a partition that has {npp}")
    have = torch.empty(0, dtype=torch.int64, device=device)
    while have.numel() < need:
        draw = torch.randint(1, n, (int((need - have.numel()) * parts * 1.25) + 4096,), generator=gen, device=device)
        draw = draw[hash_slot(draw, n) // npp == dest]
        have = torch.unique(torch.cat([have, draw]))
    have = have[torch.randperm(have.numel(), generator=gen, device=device)][:need]
    pool, own = have[:n_pool], have[n_pool:].view(cfg.peers, n_own)
    flat_idx = torch.empty(cfg.peers * per_peer, dtype=torch.int32, device=device)
    for q in range(cfg.peers):
        idx = torch.cat([pool, own[q]])
        order = torch.argsort(hash_slot(idx, n) * n + idx)  # slot order, ties by index
        flat_idx[q * per_peer:(q + 1) * per_peer] = idx[order].to(torch.int32)
    flat_val = (torch.randn(cfg.peers * per_peer, generator=gen, device=device) * 1e-3).to(cfg.dtype)
    idx_list = [flat_idx[q * per_peer:(q + 1) * per_peer] for q in range(cfg.peers)]
    val_list = [flat_val[q * per_peer:(q + 1) * per_peer] for q in range(cfg.peers)]
    return idx_list, val_list, flat_idx, flat_val


def algorithmic_bytes(n, elem_size, nnz, received, merged):
    """Bytes the path must move: one read of the gradient, the compacted
    (index, value) buffers out, the received entries in, the merged sparse
    result (int32 index + fp32 sum) out."""
    return n * elem_size + nnz * (4 + elem_size) + received * (4 + elem_size) + merged * 8


def bucket_imbalance(idx, n, parts):
    """(hash max/mean, range max/mean) of per-bucket loads for a set of
    nonzero indices: the skew measure of utils.py:66-88 applied to both
    partitioners."""
    idx = idx.to(torch.int64)
    by_hash = torch.bincount(hash_slot(idx, n) // (n // parts), minlength=parts).double()
    by_range = torch.bincount(idx // math.ceil(n / parts), minlength=parts).double()
    return (by_hash.max() / by_hash.mean()).item(), (by_range.max() / by_range.mean()).item()
