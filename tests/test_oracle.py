"""Pins the CPU oracle: closed forms, known answers, brute force on tiny
inputs, library routines (numpy / torch CPU) and schedule-free invariants.
The reference ships no tests or golden vectors for this path."""
import numpy as np
import pytest
import torch

MASK = (1 << 32) - 1
D, A, B = 573729859, 0xCC9E2D51, 0x1B873593
S1, S2, S3 = 10001861, 100703, 5002639


def big_hash(k, c):
    """functions_cuda_kernel.cu:80-88 in unbounded integers, reduced at the end."""
    return (D * k**3 + A * k**2 + B * k + c) & MASK


# ------------------------------------------------------------------ hash


def test_hash_known_answers(oracle):
    kat = {
        1: 183528684,
        2: 2075336775,
        3: 537870696,
        4096: 3304181189,
        65535: 2939627840,
        (1 << 20) - 1: 2333944128,
        (1 << 30) - 1: 259860800,
    }
    assert oracle.hash32(0, S1) == S1
    for k, v in kat.items():
        assert oracle.hash32(k, S1) == v
        assert big_hash(k, S1) == v
    assert oracle.hash32(1, S2) == 173627526
    assert oracle.hash32(1, S3) == 178529462


def test_hash_matches_bigint_and_horner(oracle):
    rng = np.random.default_rng(1)
    keys = np.concatenate([np.arange(0, 1 << 12), rng.integers(0, (1 << 31) - 1, 4000)])
    for k in keys.tolist():
        for c in (S1, S2, S3, 0, MASK):
            h = oracle.hash32(k, c)
            assert h == big_hash(k, c)
            horner = ((((D * k) & MASK) + A) * k & MASK) + B
            horner = ((horner & MASK) * k + c) & MASK
            assert h == horner


def test_hash_seed_is_additive(oracle):
    for k in (1, 7, 12345, (1 << 29) + 3):
        h1 = oracle.hash32(k, S1)
        assert (h1 - 9901158) & MASK == oracle.hash32(k, S2)
        assert (h1 - 4999222) & MASK == oracle.hash32(k, S3)


def test_hash_index_known_and_invariants(oracle):
    n, P = 1 << 20, 4
    part = oracle.hash_index(n, P)
    assert part[1:9].tolist() == [0, 0, 3, 0, 3, 3, 0, 1]
    assert part.min() >= 0 and part.max() < P
    counts = np.bincount(part, minlength=P)
    assert counts.max() / counts.mean() == 1.0  # power-of-two n: perfectly equal
    # definition, vectorised in uint64
    t = np.arange(n, dtype=np.uint64)
    h = (((D * t % (1 << 32) + A) % (1 << 32) * t % (1 << 32) + B) % (1 << 32) * t + S1) % (1 << 32)
    assert np.array_equal(part, ((h % n) // (n // P)).astype(np.int32))


def test_hash_index_non_divisible_can_emit_P(oracle):
    # n % P != 0: slot / (n // P) can reach P (functions_cuda_kernel.cu:172-175)
    n, P = 1003, 4
    part = oracle.hash_index(n, P)
    want = [(big_hash(t, S1) % n) // (n // P) for t in range(n)]
    assert part.tolist() == want
    assert part.max() == P


def test_hash_index_rejects_bad_args(oracle):
    with pytest.raises(ValueError):
        oracle.hash_index(3, 4)
    with pytest.raises(ValueError):
        oracle.hash_index(16, 0)


# ---------------------------------------------------------------- insert


def py_sequential(nz, m, P, spp, levels):
    """functions_cuda_kernel.cu:97-167 for tid ascending, in plain python."""
    mem = [0] * m
    ser = [0] * (spp * P)
    off = [p * spp for p in range(P)]
    npp = m // P
    for t in nz:
        s = big_hash(t, S1) % m
        part = s // npp
        cands = [s]
        if levels >= 2:
            cands.append(part * npp + big_hash(t, S2) % npp)
        if levels >= 3:
            cands.append(part * npp + big_hash(t, S3) % npp)
        for c in cands:
            if mem[c] == 0:
                mem[c] = t
                break
        else:
            i = off[part]
            off[part] += 1
            if i < len(ser):
                ser[i] = t
    return mem, ser, off


def py_min_owner(nz, m, P, levels):
    """Fixed point: a slot belongs to the smallest tid that ever attempts it;
    a tid attempts level l+1 only if a smaller tid owns its level-l slot."""
    npp = m // P
    probes = {}
    for t in nz:
        s = big_hash(t, S1) % m
        part = s // npp
        c = [s]
        if levels >= 2:
            c.append(part * npp + big_hash(t, S2) % npp)
        if levels >= 3:
            c.append(part * npp + big_hash(t, S3) % npp)
        probes[t] = (part, c)
    owner = {}
    changed = True
    while changed:
        changed = False
        for t in nz:
            if t == 0:
                continue
            for c in probes[t][1]:
                cur = owner.get(c)
                if cur is None or cur > t:
                    owner[c] = t
                    changed = True
                    break
                if cur == t:
                    break
    placed = set(owner.values())
    serial = {p: [] for p in range(P)}
    for t in sorted(nz):
        if t != 0 and t not in placed:
            serial[probes[t][0]].append(t)
    return owner, serial


@pytest.mark.parametrize("levels", [1, 2, 3])
@pytest.mark.parametrize("n,P,density", [(64, 4, 0.5), (480, 4, 0.9), (1000, 5, 0.3), (4096, 16, 0.1), (2000, 8, 0.97)])
def test_insert_matches_python_models(oracle, levels, n, P, density):
    rng = np.random.default_rng(n * 7 + levels)
    g = np.where(rng.random(n) < density, rng.standard_normal(n), 0).astype(np.float32)
    g[0] = 1.0  # index 0 is nonzero but can never be stored
    m, sn = oracle.table_sizes(n, P)
    mem, ser, off, st = oracle.sparse_balance(g, m, sn, P, levels)
    nz = np.flatnonzero(g).tolist()
    pm, ps, po = py_sequential(nz, m, P, sn // P, levels)
    overflow = any(po[p] > (p + 1) * (sn // P) for p in range(P))
    assert off.tolist() == po
    assert st == (1 if overflow else 0)
    assert mem.tolist() == pm
    assert ser.tolist() == ps
    # min-tid-owner fixed point == sequential execution
    owner, serial = py_min_owner(nz, m, P, levels)
    want = [0] * m
    for s, t in owner.items():
        want[s] = t
    assert mem.tolist() == want
    if not overflow:
        spp = sn // P
        for p in range(P):
            got = [x for x in ser[p * spp:(p + 1) * spp].tolist() if x]
            assert got == serial[p]


def test_insert_invariants_and_special_cases(oracle):
    n, P = 1 << 14, 8
    rng = np.random.default_rng(3)
    g = np.zeros(n, np.float32)
    nz = rng.choice(np.arange(1, n), 600, replace=False)
    g[nz] = 1.0
    m, sn = oracle.table_sizes(n, P)
    mem, ser, off, st = oracle.sparse_balance(g, m, sn, P, 3)
    stored = np.concatenate([mem[mem != 0], ser[ser != 0]])
    assert st == 0 and len(stored) == len(set(stored.tolist())) == 600
    assert set(stored.tolist()) == set(nz.tolist())
    npp = m // P
    for s in np.flatnonzero(mem):
        t = int(mem[s])
        s1 = big_hash(t, S1) % m
        base = (s1 // npp) * npp
        assert s in (s1, base + big_hash(t, S2) % npp, base + big_hash(t, S3) % npp)
    # a single nonzero lands at h1 % m
    g1 = np.zeros(n, np.float32)
    g1[777] = -2.0
    mem1, ser1, _, _ = oracle.sparse_balance(g1, m, sn, P, 3)
    assert mem1[big_hash(777, S1) % m] == 777 and np.count_nonzero(mem1) == 1 and not ser1.any()


def test_insert_predicate_negzero_nan_bf16(oracle):
    # float(x) != 0.0f: -0.0 is skipped, NaN is inserted (functions_cuda_kernel.cu:100)
    n, P = 256, 4
    g = np.zeros(n, np.float32)
    g[5] = -0.0
    g[9] = np.nan
    g[11] = 1e-45  # denormal: nonzero
    m, sn = oracle.table_sizes(n, P)
    mem, _, _, _ = oracle.sparse_balance(g, m, sn, P, 3)
    assert sorted(mem[mem != 0].tolist()) == [9, 11]
    b = np.zeros(n, np.uint16)
    b[5] = 0x8000
    b[9] = 0x7FC0
    b[11] = 0x0001
    mem, _, _, _ = oracle.sparse_balance(b, m, sn, P, 3)
    assert sorted(mem[mem != 0].tolist()) == [9, 11]


def test_insert_serial_overflow_flag(oracle):
    n, P = 400, 4
    g = np.ones(n, np.float32)
    m, sn = oracle.table_sizes(n, P)
    mem, ser, off, st = oracle.sparse_balance(g, m, sn, P, 1)
    assert st == oracle.SERIAL_OVERFLOW
    # every ticket is counted even when it cannot be stored
    assert (off - np.arange(P) * (sn // P)).sum() + np.count_nonzero(mem) == n - 1


def test_rehash_other_values_mean_one_level(oracle):
    n, P = 2048, 4
    rng = np.random.default_rng(5)
    g = (rng.random(n) < 0.4).astype(np.float32)
    m, sn = oracle.table_sizes(n, P)
    a = oracle.sparse_balance(g, m, sn, P, 1)
    for r in (0, 4, 7):
        b = oracle.sparse_balance(g, m, sn, P, r)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


# ---------------------------------------------------------- load balance


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("n,P,density,scale", [(4096, 4, 0.2, 1), (6000, 6, 0.6, 1), (4096, 8, 0.05, 2), (5000, 4, 0.3, 1.5)])
def test_load_balance_is_slot_order_compaction(oracle, dtype, n, P, density, scale):
    rng = np.random.default_rng(11)
    g = np.where(rng.random(n) < density, rng.standard_normal(n), 0).astype(np.float32)
    if dtype == "bf16":
        g = oracle.f32_to_bf16_bits(g)
    m, sn = oracle.table_sizes(n, P, scale)
    mem, ser, _, st = oracle.sparse_balance(g, m, sn, P, 3)
    idx, val, splits, st2 = oracle.load_balance(g, P, scale, 3)
    assert st == st2
    npp, spp = m // P, sn // P
    want = []
    for p in range(P):
        tab = mem[p * npp:(p + 1) * npp]
        sr = ser[p * spp:(p + 1) * spp]
        part = np.concatenate([tab[np.flatnonzero(tab)], sr[np.flatnonzero(sr)]])
        assert splits[p] == len(part)
        want.append(part)
    want = np.concatenate(want)
    assert np.array_equal(idx, want)
    assert np.array_equal(val, g[idx])
    if st == 0:
        nzcount = np.count_nonzero(g if dtype == "f32" else g & 0x7FFF) - (1 if (g[0] if dtype == "f32" else g[0] & 0x7FFF) != 0 else 0)
        assert splits.sum() == nzcount
        part_of = oracle.hash_index(m, P) if m == n else None
        if part_of is not None:
            ends = np.cumsum(splits)
            for p in range(P):
                assert (part_of[idx[ends[p] - splits[p]:ends[p]]] == p).all()


# ---------------------------------------------------------------- select


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_kth_key_matches_numpy_and_torch(oracle, dtype):
    rng = np.random.default_rng(21)
    n = 50000
    x = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    if dtype == "bf16":
        bits = oracle.f32_to_bf16_bits(x)
        mag = np.abs(oracle.bf16_bits_to_f32(bits))
        g = bits
    else:
        mag = np.abs(x)
        g = x
    for k in (1, 7, 500, n // 100, n):
        key = oracle.kth_key(g, k)
        thr_np = np.partition(mag, n - k)[n - k]
        thr_t = torch.topk(torch.from_numpy(mag), k, largest=True, sorted=False)[0].min().item()
        thr = oracle.bf16_bits_to_f32(np.array([key], np.uint16))[0] if dtype == "bf16" else np.array([key], np.uint32).view(np.float32)[0]
        assert thr == thr_np == np.float32(thr_t)
        idx, val = oracle.select(g, key)
        assert np.array_equal(idx, np.flatnonzero((mag >= thr) & (mag != 0)))
        assert np.array_equal(val, g[idx])
        assert len(idx) >= min(k, np.count_nonzero(mag))
        dense, kept = oracle.mask_dense(g, key)
        ref = torch.where(torch.from_numpy(mag) >= float(thr), torch.from_numpy(x if dtype == "f32" else oracle.bf16_bits_to_f32(g)), torch.tensor(0.0)).numpy()
        got = dense if dtype == "f32" else oracle.bf16_bits_to_f32(dense)
        assert np.array_equal(got, ref) and kept == len(idx)


def test_select_ties_kept(oracle):
    g = np.array([0.0, 1.0, -1.0, 0.5, 1.0, -0.25, 2.0, 0.0], np.float32)
    key = oracle.kth_key(g, 2)  # 2nd largest magnitude is 1.0, three ties
    idx, _ = oracle.select(g, key)
    assert idx.tolist() == [1, 2, 4, 6]


# ----------------------------------------------------------------- merge


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_decode_matches_torch_scatter_add(oracle, dtype):
    rng = np.random.default_rng(31)
    n, r = 5000, 20000
    idx = rng.integers(0, n, r).astype(np.int32)
    v = (rng.standard_normal(r) * 1e-3).astype(np.float32)
    if dtype == "bf16":
        vb = oracle.f32_to_bf16_bits(v)
        vt = torch.from_numpy(oracle.bf16_bits_to_f32(vb)).to(torch.bfloat16)
        val = vb
    else:
        vt = torch.from_numpy(v)
        val = v
    it = torch.from_numpy(idx).long()
    # comm.py:36-39 on CPU tensors: sequential, hence deterministic
    native_t = torch.zeros(n, dtype=vt.dtype).scatter_add_(0, it, vt)
    f32_t = torch.zeros(n, dtype=torch.float32).scatter_add_(0, it, vt.float())
    f64_t = torch.zeros(n, dtype=torch.float64).scatter_add_(0, it, vt.double())
    got_native = oracle.decode(idx, val, n, "native")
    if dtype == "bf16":
        # torch's CPU kernel sums bf16 in fp32 and rounds once; the GPU kernel
        # the reference runs rounds after every atomic add.  "native" restates
        # the latter in payload order, so it is pinned by scalar bf16 adds.
        assert np.array_equal(oracle.f32_to_bf16_bits(f32_t.numpy()), native_t.view(torch.int16).numpy().view(np.uint16))
        step = torch.zeros(n, dtype=torch.bfloat16)
        for j in range(r):
            step[idx[j]] = step[idx[j]] + vt[j]
        assert np.array_equal(got_native, step.view(torch.int16).numpy().view(np.uint16))
    else:
        assert np.array_equal(got_native, native_t.numpy())
    assert np.array_equal(oracle.decode(idx, val, n, "f32acc"), f32_t.numpy())
    assert np.array_equal(oracle.decode(idx, val, n, "f64"), f64_t.numpy())
    with pytest.raises(ValueError):
        oracle.decode(np.array([n], np.int32), val[:1], n)


def test_encode_matches_flatnonzero(oracle):
    d = np.array([0.0, 1.5, -0.0, np.nan, 0.0, -3.0], np.float32)
    idx, val = oracle.encode(d)
    assert idx.tolist() == [1, 3, 5] and idx.dtype == np.int64
    assert np.array_equal(val.view(np.uint32), d[[1, 3, 5]].view(np.uint32))
    ti = torch.nonzero(torch.from_numpy(d), as_tuple=True)[0]
    assert ti.tolist() == idx.tolist()


def test_merge_cancellation_vanishes(oracle):
    idx = np.array([4, 9, 4, 2], np.int32)
    val = np.array([1.0, 2.0, -1.0, 3.0], np.float32)
    mi, mv = oracle.merge_sparse(idx, val, 16)
    assert mi.tolist() == [2, 9] and mv.tolist() == [3.0, 2.0]


# --------------------------------------------------------------- mapping


def test_mapping_is_partition_of_range(oracle):
    n, P = 1 << 12, 8
    mp = oracle.mapping(n, P)
    part = oracle.hash_index(n, P)
    assert len(mp) == P
    allidx = np.concatenate(mp)
    assert np.array_equal(np.sort(allidx), np.arange(n))
    for p, lst in enumerate(mp):
        assert (np.diff(lst) > 0).all() and (part[lst] == p).all()
    # n % P != 0: indices whose part is P are in no list
    mp2 = oracle.mapping(1003, 4)
    assert sum(len(x) for x in mp2) == int((oracle.hash_index(1003, 4) < 4).sum())


# ---------------------------------------------------------------- bitmap


def test_bitmap_matches_packbits(oracle):
    n, P = 1 << 12, 8
    mp = oracle.mapping(n, P)[3]
    rng = np.random.default_rng(41)
    pick = np.sort(rng.choice(mp, 100, replace=False))
    bm = oracle.bitmap_encode(mp, pick)
    mask = np.isin(mp, pick).astype(np.uint8)
    assert np.array_equal(bm, np.packbits(mask, bitorder="little"))
    assert np.array_equal(oracle.bitmap_decode(mp, bm), pick)
    assert len(bm) == (len(mp) + 7) // 8


def test_bitmap_of_indices_that_are_no_members(oracle):
    """comm.py:61-63 looks every index up with torch.searchsorted (left side) and sets the bit at that
    position, member or not: an index between two members marks the next member, one below the first member
    marks the first, duplicates mark once, and a position past the end of the list is an error (torch's
    index_put raises).  Pinned against numpy's and torch's searchsorted, not against the oracle's own loop."""
    import torch

    mp = np.array([3, 10, 11, 40, 41, 42, 100, 1000], np.int64)
    idx = np.array([0, 3, 4, 9, 10, 12, 39, 43, 99, 100, 101, 999, 1000, 4, 4], np.int64)
    pos = np.searchsorted(mp, idx, side="left")
    assert np.array_equal(pos, torch.searchsorted(torch.from_numpy(mp), torch.from_numpy(idx)).numpy())
    mask = np.zeros(len(mp), np.uint8)
    mask[pos] = 1
    bm = oracle.bitmap_encode(mp, idx)
    assert np.array_equal(bm, np.packbits(mask, bitorder="little"))
    # decoding gives members only: what was between members has become the next member
    assert np.array_equal(oracle.bitmap_decode(mp, bm), mp[np.unique(pos)])
    # one past the last member: no position in the list
    with pytest.raises(IndexError):
        oracle.bitmap_encode(mp, np.array([3, 1001], np.int64))
    # random case, any order, many non-members
    rng = np.random.default_rng(43)
    mp = np.unique(rng.integers(0, 1 << 20, 5000)).astype(np.int64)
    idx = rng.integers(0, int(mp[-1]) + 1, 3000).astype(np.int64)
    mask = np.zeros(len(mp), np.uint8)
    mask[np.searchsorted(mp, idx, side="left")] = 1
    assert np.array_equal(oracle.bitmap_encode(mp, idx), np.packbits(mask, bitorder="little"))


def test_selection_of_nan_gradients_is_by_bit_pattern(oracle):
    """Where this build and the reference's torch ops part ways, written down: the selection compares
    magnitude BIT PATTERNS, in which a NaN (exponent all ones, mantissa nonzero) ranks above infinity.
    torch.topk also treats NaN as the largest value, so the threshold of train.py:81-82 becomes NaN as soon as
    k reaches into the NaNs, and `tensor_abs >= threshold` (train.py:83) is then false everywhere: the
    reference selects nothing, this build selects the NaNs and whatever else lies at or above the k-th
    pattern.  Without NaNs among the k largest the two agree.  The nonzero predicate of the insert kernel
    (float(x) != 0, functions_cuda_kernel.cu:100) counts NaN as nonzero in both."""
    import torch

    g = np.array([0.5, -2.0, np.nan, 1.0, -np.inf, 0.0, 3.0, -0.25, np.nan, 1e-3, -1e-3, 7.0, 0.125, -4.0, 2.5, 0.75],
                 np.float32)
    t = torch.from_numpy(g)
    # k = 3 reaches two NaNs and the infinity
    key = oracle.kth_key(g, 3)
    assert key == 0x7F800000  # the pattern of infinity: the NaNs rank above it
    masked, kept = oracle.mask_dense(g, key)
    assert kept == 3 and np.isnan(masked[[2, 8]]).all() and masked[4] == -np.inf
    thr = torch.topk(t.abs(), 3, largest=True, sorted=False)[0].min()
    assert torch.isnan(thr) or thr == float("inf")  # torch: NaN is the largest, min() of the top 3 propagates it
    ref = torch.where(t.abs() >= thr, t, torch.zeros(()))
    assert int(torch.count_nonzero(ref)) <= 1  # the reference keeps (almost) nothing where this build keeps 3
    # bf16 likewise
    key16 = oracle.kth_key(oracle.f32_to_bf16_bits(g), 3)
    assert key16 == 0x7F80
    # no NaN among the k largest finite values: agreement with torch (k = 5 of the NaN-free tensor)
    h = np.where(np.isnan(g), 0, g).astype(np.float32)
    key = oracle.kth_key(h, 5)
    th = torch.from_numpy(h)
    thr = torch.topk(th.abs(), 5, largest=True, sorted=False)[0].min()
    masked, kept = oracle.mask_dense(h, key)
    assert np.array_equal(masked, torch.where(th.abs() >= thr, th, torch.zeros(())).numpy())
    # the insert's predicate: NaN is nonzero, -0.0 is zero
    mem, ser, off, st = oracle.sparse_balance(np.array([0.0, np.nan, -0.0, 1.0], np.float32), 4, 0, 1, 3)
    assert sorted(int(x) for x in mem if x) == [1, 3]
