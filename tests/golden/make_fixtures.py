#!/usr/bin/env python3
"""Writes the fixtures in this directory.  The reference ships no golden vectors
for this path, so the expected outputs are computed here by plain-Python models
written from the reference's text (unbounded integers, dict and list state, one
element at a time) that share no code with the C oracle or the HIP kernels:

  hash_kat.json        hash values and partition ids (functions_cuda_kernel.cu:80-93, :169-177)
  insert_dense.npz     ~1K-element insert at load factor 0.6, serial region in use
                       (functions_cuda_kernel.cu:97-167, tensor_load_balance.py:13-51)
  insert_overflow.npz  the same at load factor 1 with one level: the serial region overflows
  select_ties.npz      bf16 top-k with most magnitudes tied at the threshold (train.py:79-84)
  merge_overlap.npz    merge of 4 payloads with shared indices, fp32 sums in arrival order
                       (comm.py:32-50)

    python tests/golden/make_fixtures.py        # rewrites the files; the output is deterministic
"""
import json
import os
import struct

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
MASK = (1 << 32) - 1
D, A, B = 573729859, 0xCC9E2D51, 0x1B873593
SEEDS = (10001861, 100703, 5002639)


def h(k, c):
    return (D * k ** 3 + A * k ** 2 + B * k + c) & MASK


def sizes(n, P, scale=1):
    return int(n * scale // P * P), int(n // P // 10 * P)


def insert(nz, m, P, spp, levels):
    """One element at a time in ascending index order."""
    mem, ser, off, npp, overflow = [0] * m, [0] * (spp * P), [p * spp for p in range(P)], m // P, False
    for t in nz:
        s = h(t, SEEDS[0]) % m
        part = s // npp
        slots = [s] + [part * npp + h(t, SEEDS[lv]) % npp for lv in range(1, levels)]
        for c in slots:
            if mem[c] == 0:
                mem[c] = t
                break
        else:
            i = off[part]
            off[part] += 1
            overflow |= i >= (part + 1) * spp  # the reference writes on, into the next region (.cu:107-108)
            if i < len(ser):
                ser[i] = t
    return mem, ser, off, overflow


def compaction(mem, ser, P):
    """Per partition: table chunk in slot order, then its serial chunk (tensor_load_balance.py:24-51)."""
    npp, spp = len(mem) // P, len(ser) // P
    idx, splits = [], []
    for p in range(P):
        part = [t for t in mem[p * npp:(p + 1) * npp] if t] + [t for t in ser[p * spp:(p + 1) * spp] if t]
        idx += part
        splits.append(len(part))
    return idx, splits


def f32(x):
    return struct.unpack("<f", struct.pack("<f", x))[0]


def bf16_bits(x):
    """Round-to-nearest-even bf16 bit pattern of a python float (finite)."""
    u = struct.unpack("<I", struct.pack("<f", x))[0]
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF


def main():
    rng = np.random.default_rng(20240607)

    keys = [0, 1, 2, 3, 7, 255, 4096, 65535, (1 << 20) - 1, (1 << 24) + 5, (1 << 30) - 1, (1 << 31) - 1]
    kat = {"hash": [{"key": k, "h": [h(k, c) for c in SEEDS]} for k in keys], "part": []}
    for n, P in ((1 << 20, 4), (38597376, 16), (743440384, 16), (1000, 4), (786432000, 64)):
        npp = n // P
        ts = [t for t in keys if t < n - 1] + [n - 1]
        kat["part"].append({"n": n, "P": P, "t": ts, "part": [(h(t, SEEDS[0]) % n) // npp for t in ts]})
    with open(os.path.join(HERE, "hash_kat.json"), "w") as f:
        json.dump(kat, f, indent=1)

    # insert at load factor 0.6 (three levels) and 1.0 (one level: overflows the serial region)
    for name, n, P, density, levels in (("insert_dense", 1200, 4, 0.6, 3), ("insert_overflow", 1000, 5, 1.0, 1)):
        g = np.where(rng.random(n) < density, rng.standard_normal(n) * 1e-3, 0).astype(np.float32)
        g[0] = 1.0  # index 0 can never be told from an empty slot: it is dropped
        m, s = sizes(n, P)
        nz = [int(t) for t in np.flatnonzero(g)]
        mem, ser, off, overflow = insert(nz, m, P, s // P, levels)
        assert overflow == (name == "insert_overflow"), name
        assert any(ser), name
        out = dict(grad=g, partitions=P, levels=levels, memory=np.array(mem, np.int32), overflow=overflow)
        if not overflow:  # past an overflow only the table is well defined
            idx, splits = compaction(mem, ser, P)
            out.update(serial=np.array(ser, np.int32), offset=np.array(off, np.int32),
                       indices=np.array(idx, np.int32), values=g[idx], splits=np.array(splits, np.int64))
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)

    # bf16 select with heavy ties: 3000 elements, magnitudes from 6 levels, signs mixed
    n, k = 3000, 700
    levels = [0.0, 0.25, 0.5, 0.5, 0.5, 1.0, 2.0]
    vals = [levels[i] * (1 if s else -1) for i, s in zip(rng.integers(0, len(levels), n), rng.integers(0, 2, n))]
    bits = [bf16_bits(v) for v in vals]
    mags = sorted((b & 0x7FFF for b in bits), reverse=True)
    key = mags[k - 1]
    sel = [i for i, b in enumerate(bits) if (b & 0x7FFF) >= key and (b & 0x7FFF) != 0]
    assert len(sel) > k  # ties at the threshold are all kept
    np.savez_compressed(os.path.join(HERE, "select_ties.npz"), grad_bits=np.array(bits, np.uint16), k=k, key=key,
                        indices=np.array(sel, np.int64), values_bits=np.array([bits[i] for i in sel], np.uint16))

    # merge: 4 payloads of 300 entries over 5000 positions, 40 % of each from a shared pool, one exact cancellation
    dense_n, peers, per = 5000, 4, 300
    pool = rng.choice(dense_n, 120, replace=False)
    idx, val = [], []
    for q in range(peers):
        own = rng.integers(0, dense_n, per - len(pool))
        i = np.concatenate([pool, own])
        rng.shuffle(i)
        idx.append(i.astype(np.int32))
        val.append((rng.standard_normal(per) * 1e-3).astype(np.float32))
    used = set(np.concatenate(idx).tolist())
    lone = next(i for i in range(dense_n) if i not in used)
    idx.append(np.array([lone, lone], np.int32))  # sums to exactly zero: must not appear in the result
    val.append(np.array([0.125, -0.125], np.float32))
    acc = {}
    for i, v in zip(np.concatenate(idx).tolist(), np.concatenate(val).tolist()):
        acc[i] = f32(acc.get(i, 0.0) + v)  # one fp32 rounding per add, arrival order
    assert acc[lone] == 0.0
    merged = sorted(i for i, v in acc.items() if v != 0.0)
    np.savez_compressed(os.path.join(HERE, "merge_overlap.npz"), dense_n=dense_n, indices=np.concatenate(idx),
                        values=np.concatenate(val), lengths=np.array([len(i) for i in idx]),
                        merged_indices=np.array(merged, np.int64),
                        merged_values=np.array([acc[i] for i in merged], np.float32))


if __name__ == "__main__":
    main()
