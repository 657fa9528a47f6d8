"""The committed fixtures (tests/golden, written by make_fixtures.py from
plain-Python models of the reference's text) against the C oracle on the CPU and
against the HIP library on the GPU."""
import json
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with np.load(os.path.join(GOLDEN, name)) as z:
        return {k: z[k] for k in z.files}


def kat():
    with open(os.path.join(GOLDEN, "hash_kat.json")) as f:
        return json.load(f)


# ------------------------------------------------------------ oracle (CPU)


def test_fixtures_are_what_the_generator_writes(tmp_path, monkeypatch):
    import importlib.util

    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    monkeypatch.setattr(gen, "HERE", str(tmp_path))
    gen.main()
    for name in sorted(os.listdir(GOLDEN)):
        if name.endswith(".npz"):
            a, b = load(name), {k: v for k, v in np.load(tmp_path / name).items()}
            assert a.keys() == b.keys()
            assert all(np.array_equal(a[k], b[k]) for k in a), name
    assert json.load(open(tmp_path / "hash_kat.json")) == kat()


def test_oracle_hash_fixture(oracle):
    k = kat()
    for row in k["hash"]:
        for seed, want in zip((oracle.SEED1, oracle.SEED2, oracle.SEED3), row["h"]):
            assert oracle.hash32(row["key"], seed) == want
    for row in k["part"]:
        if row["n"] > (1 << 26):
            continue  # the oracle's hash_index fills a whole array; large n is covered by the closed form above
        part = oracle.hash_index(row["n"], row["P"])
        assert [int(part[t]) for t in row["t"]] == row["part"]


@pytest.mark.parametrize("name", ["insert_dense.npz", "insert_overflow.npz"])
def test_oracle_insert_fixture(oracle, name):
    z = load(name)
    g, P, levels = z["grad"], int(z["partitions"]), int(z["levels"])
    m, sn = oracle.table_sizes(g.size, P)
    mem, ser, off, st = oracle.sparse_balance(g, m, sn, P, levels)
    assert np.array_equal(mem, z["memory"])
    assert bool(st & oracle.SERIAL_OVERFLOW) == bool(z["overflow"])
    if not z["overflow"]:
        assert np.array_equal(ser, z["serial"]) and np.array_equal(off, z["offset"])
        idx, val, splits, st = oracle.load_balance(g, P, 1, levels)
        assert st == 0
        assert np.array_equal(idx, z["indices"]) and np.array_equal(val, z["values"])
        assert np.array_equal(splits, z["splits"])
        # the same gradient as bf16 bit patterns selects the same indices (all magnitudes are bf16-normal)
        idx16, _, splits16, _ = oracle.load_balance(oracle.f32_to_bf16_bits(g), P, 1, levels)
        assert np.array_equal(idx16, z["indices"]) and np.array_equal(splits16, z["splits"])


def test_oracle_select_fixture(oracle):
    z = load("select_ties.npz")
    g = z["grad_bits"]
    key = oracle.kth_key(g, int(z["k"]))
    assert key == int(z["key"])
    idx, val = oracle.select(g, key)
    assert np.array_equal(idx, z["indices"]) and np.array_equal(val, z["values_bits"])


def test_oracle_merge_fixture(oracle):
    z = load("merge_overlap.npz")
    idx, val = oracle.merge_sparse(z["indices"], z["values"], int(z["dense_n"]))
    assert np.array_equal(idx, z["merged_indices"])
    assert np.array_equal(val.view(np.uint32), z["merged_values"].view(np.uint32))


# ------------------------------------------------------------ HIP library (GPU)


@pytest.fixture(scope="module")
def zen():
    import zen_repro_amd

    zen_repro_amd._lib.lib()
    return zen_repro_amd


def dev(a):
    from gpu_util import to_dev

    return to_dev(a)


def host(t):
    from gpu_util import to_np

    return to_np(t)


@pytest.mark.gpu
def test_hip_hash_fixture(zen):
    for row in kat()["part"]:
        assert max(row["t"]) < row["n"]
        out = torch.empty(row["n"], dtype=torch.int32, device="cuda")
        zen.hash_index(out, row["P"])
        assert out[torch.tensor(row["t"], device="cuda")].tolist() == row["part"]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("name", ["insert_dense.npz", "insert_overflow.npz"])
def test_hip_insert_fixture(zen, oracle, name, dtype):
    z = load(name)
    g, P, levels = z["grad"], int(z["partitions"]), int(z["levels"])
    if dtype == "bf16":
        g = oracle.f32_to_bf16_bits(g)
    m, sn = oracle.table_sizes(g.size, P)
    d = dev(g)
    mem = torch.zeros(m, dtype=torch.int32, device="cuda")
    ser = torch.zeros(sn, dtype=torch.int32, device="cuda")
    assert zen.sparse_balance(d, mem, ser, P, levels) is None  # like the reference's
    pending = zen.last_status()
    assert np.array_equal(host(mem), z["memory"])
    assert bool(pending.status.item() & 1) == bool(z["overflow"])
    tp = zen.TensorPartition(P, 1, levels)
    if z["overflow"]:
        with pytest.raises(RuntimeError):
            tp.load_balance(d)
        return
    assert np.array_equal(host(ser), z["serial"]) and np.array_equal(host(pending.offsets), z["offset"])
    for mode in (0, 1):
        indices, values, splits = tp.load_balance(d, mode=mode)
        assert np.array_equal(host(splits), z["splits"])
        assert np.array_equal(np.concatenate([host(i) for i in indices]), z["indices"])
        got = np.concatenate([host(v) for v in values])
        assert np.array_equal(got, oracle.f32_to_bf16_bits(z["values"]) if dtype == "bf16" else z["values"])


@pytest.mark.gpu
def test_hip_select_fixture(zen):
    z = load("select_ties.npz")
    d = dev(z["grad_bits"])
    thr = zen.topk_threshold(d, int(z["k"]))
    assert int(host(thr)[0]) == int(z["key"]) and int(host(thr)[1]) == len(z["indices"])
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(4), None, None)
    import importlib

    masked = importlib.import_module("zen_repro_amd.compress").mask_below(d, thr)
    idx, val = lba.encode_sparse_tensor(masked)
    assert np.array_equal(host(idx), z["indices"]) and np.array_equal(host(val), z["values_bits"])


@pytest.mark.gpu
@pytest.mark.parametrize("mode", [0, 1])
def test_hip_merge_fixture(zen, mode):
    z = load("merge_overlap.npz")
    lba = zen.LoadBalanceAllreduce(zen.LocalGroup(4), None, None)
    idx, val, cnt, st = lba.merge_sparse_flat(dev(z["indices"]), dev(z["values"]), int(z["dense_n"]), mode=mode)
    u = len(z["merged_indices"])
    assert st.item() == 0 and cnt.item() == u
    assert np.array_equal(host(idx)[:u], z["merged_indices"].astype(np.int32))
    assert np.array_equal(host(val)[:u].view(np.uint32), z["merged_values"].view(np.uint32))
    # list form through decode + encode, as the reference's caller does (comm.py:125-127)
    parts = np.split(np.arange(len(z["indices"])), np.cumsum(z["lengths"])[:-1])
    dense = lba.decode_sparse_tensors([dev(z["indices"][p]) for p in parts], [dev(z["values"][p]) for p in parts],
                                      int(z["dense_n"]))
    i2, v2 = lba.encode_sparse_tensor(dense)
    assert np.array_equal(host(i2), z["merged_indices"])
    assert np.allclose(host(v2), z["merged_values"], rtol=1e-6, atol=0)
