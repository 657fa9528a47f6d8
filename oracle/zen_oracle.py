"""ctypes front end of the CPU oracle (oracle/zen_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg as the checker.  The product package never imports
it.  Arrays are numpy; bf16 tensors travel as uint16 bit patterns.

Reference lines restated by each C function are cited in zen_oracle.h.
"""
import ctypes
import os
import subprocess

import numpy as np

F32, BF16 = 0, 1
SEED1, SEED2, SEED3 = 10001861, 100703, 5002639
SERIAL_OVERFLOW = 1

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libzen_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (seconds)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < max(
        os.path.getmtime(os.path.join(_HERE, f)) for f in ("zen_oracle.c", "zen_oracle.h")
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libzen_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        vp, i32, i64, u32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_uint32
        L.zen_oracle_hash.restype = u32
        L.zen_oracle_hash.argtypes = [ctypes.c_int32, u32]
        L.zen_oracle_hash_index.restype = i32
        L.zen_oracle_hash_index.argtypes = [vp, i64, i32]
        L.zen_oracle_sparse_balance.restype = i32
        L.zen_oracle_sparse_balance.argtypes = [vp, i32, i64, vp, i64, vp, i64, vp, i32, i32]
        L.zen_oracle_load_balance.restype = i32
        L.zen_oracle_load_balance.argtypes = [vp, i32, i64, i64, i32, i32, vp, vp, vp]
        L.zen_oracle_kth_key.restype = u32
        L.zen_oracle_kth_key.argtypes = [vp, i32, i64, i64]
        L.zen_oracle_mask_dense.restype = i64
        L.zen_oracle_mask_dense.argtypes = [vp, i32, i64, u32, vp]
        L.zen_oracle_select.restype = i64
        L.zen_oracle_select.argtypes = [vp, i32, i64, u32, vp, vp]
        for name in ("zen_oracle_decode_f32acc", "zen_oracle_decode_native", "zen_oracle_decode_f64"):
            f = getattr(L, name)
            f.restype = i32
            f.argtypes = [vp, vp, i32, i64, vp, i64]
        L.zen_oracle_encode.restype = i64
        L.zen_oracle_encode.argtypes = [vp, i32, i64, vp, vp]
        L.zen_oracle_mapping.restype = i32
        L.zen_oracle_mapping.argtypes = [i64, i32, vp, vp]
        L.zen_oracle_bitmap_encode.restype = i32
        L.zen_oracle_bitmap_encode.argtypes = [vp, i64, vp, i64, vp]
        L.zen_oracle_bitmap_decode.restype = i64
        L.zen_oracle_bitmap_decode.argtypes = [vp, i64, vp, vp]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _dtype_of(a):
    """numpy float32 -> F32; uint16 (bf16 bit patterns) -> BF16."""
    if a.dtype == np.float32:
        return F32
    if a.dtype == np.uint16:
        return BF16
    raise TypeError(f"oracle takes float32 or uint16(bf16 bits), got {a.dtype}")


def _c(a):
    return np.ascontiguousarray(a)


def hash32(key, seed=SEED1):
    return int(lib().zen_oracle_hash(int(key), int(seed)))


def hash_index(n, partitions):
    out = np.empty(n, np.int32)
    if lib().zen_oracle_hash_index(_p(out), n, partitions) != 0:
        raise ValueError("invalid hash_index arguments")
    return out


def table_sizes(numel, partitions, memory_scale=1):
    """tensor_load_balance.py:14-18: (table size, serial size)."""
    memory_size = numel * memory_scale
    memory_size = int(memory_size // partitions * partitions)
    serial_size = int(numel // partitions // 10 * partitions)
    return memory_size, serial_size


def sparse_balance(g, m, serial_n, partitions, rehash=3):
    """Returns (memory, serial, offset, status) after the sequential insert."""
    g = _c(g)
    memory = np.zeros(m, np.int32)
    serial = np.zeros(max(serial_n, 0), np.int32)
    spp = serial_n // partitions
    offset = np.array([p * spp for p in range(partitions)], np.int32)
    st = lib().zen_oracle_sparse_balance(
        _p(g), _dtype_of(g), g.size, _p(memory), m, _p(serial), serial_n, _p(offset), partitions, rehash
    )
    if st < 0:
        raise ValueError("invalid sparse_balance arguments")
    return memory, serial, offset, st


def load_balance(g, partitions, memory_scale=1, rehash=3):
    """Returns (idx int32[nnz'], val[nnz'], splits int64[P], status)."""
    g = _c(g)
    m, _ = table_sizes(g.size, partitions, memory_scale)
    cap = int(np.count_nonzero(g if g.dtype == np.float32 else (g & 0x7FFF))) + 1
    idx = np.empty(cap, np.int32)
    val = np.empty(cap, g.dtype)
    splits = np.zeros(partitions, np.int64)
    st = lib().zen_oracle_load_balance(
        _p(g), _dtype_of(g), g.size, m, partitions, rehash, _p(idx), _p(val), _p(splits)
    )
    if st < 0:
        raise ValueError("invalid load_balance arguments")
    total = int(splits.sum())
    return idx[:total].copy(), val[:total].copy(), splits, st


def kth_key(g, k):
    g = _c(g)
    key = lib().zen_oracle_kth_key(_p(g), _dtype_of(g), g.size, k)
    if key == 0xFFFFFFFF:
        raise ValueError("invalid kth_key arguments")
    return int(key)


def mask_dense(g, thr_key):
    g = _c(g)
    out = np.empty_like(g)
    kept = lib().zen_oracle_mask_dense(_p(g), _dtype_of(g), g.size, thr_key, _p(out))
    return out, int(kept)


def select(g, thr_key):
    g = _c(g)
    idx = np.empty(g.size, np.int32)
    val = np.empty(g.size, g.dtype)
    cnt = lib().zen_oracle_select(_p(g), _dtype_of(g), g.size, thr_key, _p(idx), _p(val))
    return idx[:cnt].copy(), val[:cnt].copy()


def decode(idx, val, dense_n, mode="f32acc"):
    """mode: 'f32acc' -> float32 out, 'native' -> val dtype out, 'f64' -> float64."""
    idx = _c(idx.astype(np.int32, copy=False))
    val = _c(val)
    if mode == "f32acc":
        out = np.empty(dense_n, np.float32)
        fn = lib().zen_oracle_decode_f32acc
    elif mode == "native":
        out = np.empty(dense_n, val.dtype)
        fn = lib().zen_oracle_decode_native
    elif mode == "f64":
        out = np.empty(dense_n, np.float64)
        fn = lib().zen_oracle_decode_f64
    else:
        raise ValueError(mode)
    if fn(_p(idx), _p(val), _dtype_of(val), idx.size, _p(out), dense_n) != 0:
        raise ValueError("index out of range in decode")
    return out


def encode(dense):
    dense = _c(dense)
    idx = np.empty(dense.size, np.int64)
    val = np.empty(dense.size, dense.dtype)
    cnt = lib().zen_oracle_encode(_p(dense), _dtype_of(dense), dense.size, _p(idx), _p(val))
    return idx[:cnt].copy(), val[:cnt].copy()


def merge_sparse(idx, val, dense_n):
    """decode (fp32 accumulation, payload order) followed by encode."""
    return encode(decode(idx, val, dense_n, "f32acc"))


def mapping(n, partitions):
    out = np.empty(n, np.int64)
    counts = np.zeros(partitions, np.int64)
    if lib().zen_oracle_mapping(n, partitions, _p(out), _p(counts)) != 0:
        raise ValueError("invalid mapping arguments")
    ends = np.cumsum(counts)
    return [out[e - c:e].copy() for c, e in zip(counts, ends)]


def bitmap_encode(mapping_p, idx):
    mapping_p = _c(mapping_p.astype(np.int64, copy=False))
    idx = _c(idx.astype(np.int64, copy=False))
    out = np.empty((mapping_p.size + 7) // 8, np.uint8)
    if lib().zen_oracle_bitmap_encode(_p(mapping_p), mapping_p.size, _p(idx), idx.size, _p(out)) != 0:
        raise IndexError("index beyond the mapping")
    return out


def bitmap_decode(mapping_p, bitmap):
    mapping_p = _c(mapping_p.astype(np.int64, copy=False))
    bitmap = _c(bitmap)
    out = np.empty(mapping_p.size, np.int64)
    cnt = lib().zen_oracle_bitmap_decode(_p(mapping_p), mapping_p.size, _p(bitmap), _p(out))
    return out[:cnt].copy()


# ---------------------------------------------------------------- bf16 helpers


def f32_to_bf16_bits(x):
    """Round-to-nearest-even float32 -> bf16 bit patterns (uint16)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)
