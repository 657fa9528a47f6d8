"""Loader of libzen_hip.so (the C-ABI of include/zen_hip.h) and the small
amount of torch plumbing every wrapper shares: dtype codes, stream handles,
cached workspaces and status words.  There is no fallback: if the library is
missing or a call fails, an exception is raised."""
import ctypes
import threading
import os

import torch  # first: makes the process use torch's HIP runtime for libzen_hip too

F32, BF16 = 0, 1
OK, EINVAL, EHIP, EWORKSPACE = 0, -1, -2, -3
STAT_SERIAL_OVERFLOW, STAT_CAPACITY, STAT_INTERNAL, STAT_BAD_INDEX, STAT_RETRY = 1, 2, 4, 8, 16
MODE_FAST, MODE_GENERAL = 0, 1
MODE_ZEROED = 0x100  # zen_merge: the head of the workspace is zero (and stays so)
MODE_PREPARED, MODE_SECOND, MODE_DISCARD = 0x200, 0x400, 0x800  # zen_load_balance: the sample was taken ahead (zen_load_balance_prepare)
MODE_FLOOR = 0x1000  # zen_load_balance with k > 0: thr holds a key close to the threshold, no sample is taken
MODE_SLABS = 0x2000  # fast mode without the wide-bucket path (bucket slabs where they fit)

_HERE = os.path.dirname(os.path.abspath(__file__))
# ZEN_HIP_LIB names another build of the library (a debug build, a build with other compile-time settings)
LIB_PATH = os.environ.get("ZEN_HIP_LIB") or os.path.join(_HERE, "csrc", "libzen_hip.so")

# ZEN_ABI_VERSION of include/zen_hip.h this loader's signatures and structs are written for
ABI_VERSION = 3

_lib = None


class EncodeMergeArgs(ctypes.Structure):
    """zen_encode_merge_args of include/zen_hip.h."""
    _vp, _i32, _i64, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t
    _fields_ = [
        ("input", _vp), ("dtype", _i32), ("n", _i64), ("m", _i64), ("partitions", _i32), ("rehash", _i32),
        ("thr", _vp), ("k", _i64), ("thr_out", _vp), ("out_idx", _vp), ("out_val", _vp), ("capacity", _i64),
        ("splits", _vp), ("table", _vp), ("mode", _i32), ("workspace", _vp), ("workspace_bytes", _sz),
        ("status", _vp),
        ("recv_idx", _vp), ("recv_idx64", _i32), ("recv_val", _vp), ("r", _i64), ("dense_n", _i64),
        ("merged_idx", _vp), ("merged_idx64", _i32), ("merged_val", _vp), ("merged_capacity", _i64),
        ("merged_count", _vp), ("merge_mode", _i32), ("merge_workspace", _vp), ("merge_workspace_bytes", _sz),
        ("merge_status", _vp),
        ("stream", _vp), ("merge_stream", _vp),
        ("next_input", _vp), ("next_k", _i64), ("next_n", _i64), ("next_m", _i64), ("next_capacity", _i64),
        ("next_table", _vp),
    ]


def build():
    """Compile libzen_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
    import subprocess

    subprocess.check_call(["make", "-C", os.path.join(_HERE, "csrc"), "-B", "-j8", "all"],
                          stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    return LIB_PATH


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C zen_repro_amd/csrc` "
            "(or __graft_entry__.build()); there is no fallback path")
    L = ctypes.CDLL(LIB_PATH)
    vp, i32, i64, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t
    sig = {
        "zen_abi_version": (i32, []),
        "zen_last_error": (ctypes.c_char_p, []),
        "zen_hash_index": (i32, [vp, i64, i32, vp]),
        "zen_mapping_workspace": (sz, [i64, i32]),
        "zen_mapping": (i32, [i64, i32, vp, vp, vp, sz, vp, vp]),
        "zen_bitmap_words": (sz, [i64]),
        "zen_bitmap_rank_words": (sz, [i64]),
        "zen_bitmap_ranks": (i32, [vp, i64, i64, vp, vp]),
        "zen_bitmap_encode": (i32, [vp, i64, vp, i32, i64, vp, vp, i64, vp, vp, vp]),
        "zen_bitmap_decode_workspace": (sz, [i64]),
        "zen_bitmap_decode": (i32, [vp, i64, vp, i64, vp, i64, vp, vp, sz, vp, vp]),
        "zen_sparse_balance": (i32, [vp, i32, i64, vp, i64, vp, i64, vp, i32, i32, vp, vp]),
        "zen_encode_merge_samples_next": (i32, [i64, i64, i32, i64, i32, i64, i32]),
        "zen_topk_threshold_workspace": (sz, []),
        "zen_topk_threshold": (i32, [vp, i32, i64, i64, vp, vp, sz, vp]),
        "zen_topk_threshold_static": (i32, [vp, i32, i64, i64, vp, vp]),
        "zen_round_compact_workspace": (sz, [i64]),
        "zen_round_compact": (i32, [vp, i32, vp, vp, i64, i32, vp, vp, vp, vp, sz, vp, vp]),
        "zen_sample_threshold_workspace": (sz, [i64, i32]),
        "zen_sample_threshold": (i32, [vp, i32, i64, vp, i64, i64, vp, vp, sz, vp, vp]),
        "zen_compress": (i32, [vp, i32, i64, vp, vp, vp]),
        "zen_select_workspace": (sz, [i64, i32]),
        "zen_select": (i32, [vp, i32, i64, vp, vp, i32, vp, i64, vp, vp, sz, vp, vp]),
        "zen_load_balance_workspace": (sz, [i64, i64, i32, i64, i32]),
        "zen_load_balance": (i32, [vp, i32, i64, i64, i32, i32, vp, i64, vp, vp, vp, i64, vp, vp, i32, vp, sz, vp, vp]),
        "zen_load_balance_prepare": (i32, [vp, i32, i64, i64, i32, i64, i64, vp, i32, vp, sz, vp]),
        "zen_load_balance_path": (i32, [i64, i64, i32, i64, i32, i64, i32]),
        "zen_merge_workspace": (sz, [i64, i64]),
        "zen_merge_path": (i32, [i64, i64, i32]),
        "zen_merge_zero_bytes": (sz, []),
        "zen_merge": (i32, [vp, i32, vp, i32, i64, i64, vp, i32, vp, i64, vp, i32, vp, sz, vp, vp]),
        "zen_encode_merge": (i32, [ctypes.POINTER(EncodeMergeArgs)]),
        "zen_decode_dense_workspace": (sz, [i64, i64]),
        "zen_decode_dense": (i32, [vp, i32, vp, i32, i64, vp, i64, i32, vp, sz, vp, vp]),
        "zen_decode_dense_sorted_workspace": (sz, [i64, i32]),
        "zen_decode_dense_sorted": (i32, [vp, i32, vp, i32, ctypes.POINTER(ctypes.c_int64), i32, vp, i64, vp, sz, vp, vp]),
        "zen_bitmap_dense_dict_bytes": (sz, [i64, i32]),
        "zen_bitmap_dense_dict": (i32, [i64, i32, vp, ctypes.POINTER(ctypes.c_int64), vp]),
        "zen_bitmap_dense_workspace": (sz, [i64, i32]),
        "zen_bitmap_dense": (i32, [vp, i64, i32, vp, ctypes.POINTER(ctypes.c_int64), vp, i32,
                                   ctypes.POINTER(ctypes.c_int64), vp, vp, sz, vp, vp]),
        "zen_sort_pairs_workspace": (sz, [i64]),
        "zen_sort_pairs": (i32, [vp, vp, i64, vp, i32, vp, sz, vp, vp]),
        "zen_bucket_sort_fits": (i32, [i64, ctypes.c_uint32]),
        "zen_bucket_sort_pairs": (i32, [vp, vp, i64, vp, ctypes.c_uint32, vp, sz, vp, vp]),
        "zen_stream_read": (i32, [vp, sz, vp, vp]),
        "zen_profile_enable": (i32, [i32]),
        "zen_profile_only": (i32, [i32]),
        "zen_profile_every": (i32, [i32]),
        "zen_profile_tags": (i32, []),
        "zen_profile_name": (ctypes.c_char_p, [i32]),
        "zen_profile_read": (i32, [i32, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_int64)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    if L.zen_abi_version() != ABI_VERSION:
        raise RuntimeError("libzen_hip.so: unexpected ABI version")
    _lib = L
    return L


def check(code, what):
    if code == OK:
        return
    msg = lib().zen_last_error().decode(errors="replace")
    if code == EINVAL:
        raise ValueError(f"{what}: {msg}")
    raise RuntimeError(f"{what} failed ({code}): {msg}")


def dtype_code(t):
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise AssertionError(f"gradient dtype must be bfloat16 or float32, got {t.dtype}")


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def device_index(device):
    """Index of a torch device (or of the current one if it names none)."""
    index = device.index if isinstance(device, torch.device) else torch.device(device).index
    return index if index is not None else torch.cuda.current_device()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_handle(device):
    """The current stream of `device` as an integer handle (hipStream_t).  Asked on every call of the hot
    path: torch's own shortcut, where it has one, is several microseconds quicker than a Stream object."""
    if _raw_stream is not None:
        return _raw_stream(device_index(device))
    return torch.cuda.current_stream(device).cuda_stream


def stream_of(device):
    return ctypes.c_void_p(stream_handle(device))


def require_gpu(t, name):
    # extensions/cuda/functions.py:5-7 asserts; functions_cuda.cpp:11-13 raises RuntimeError
    assert t.is_cuda, f"{name} must be a GPU tensor"
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


class Scratch:
    """Cache of raw byte buffers per device and host thread, grown on demand
    and reused.  A buffer is tied to the stream order of its users, like any
    torch tensor; two threads that enqueue calls side by side (their kernels
    interleave even on one stream) never share one, and a thread's buffers go
    when the thread does."""

    def __init__(self):
        self._local = threading.local()

    def _bufs(self):
        bufs = getattr(self._local, "bufs", None)
        if bufs is None:
            bufs = self._local.bufs = {}
        return bufs

    def get(self, device, name, nbytes, zero=False):
        key = (device_index(device), name)
        bufs = self._bufs()
        buf = bufs.get(key)
        if buf is None or buf.numel() < nbytes:
            alloc = torch.zeros if zero else torch.empty
            buf = alloc(max(int(nbytes), 256), dtype=torch.uint8, device=device)
            bufs[key] = buf
        return buf

    def drop(self):
        """Forget the calling thread's buffers."""
        self._bufs().clear()


scratch = Scratch()


class ZeroPool:
    """Small zeroed device buffers (status words, counters, split sizes).  A
    fill kernel for four bytes costs the device as much as one for a megabyte,
    and a call on the hot path needs two or three such buffers: they are cut
    from a block that one fill zeroed.  Every piece is handed out once (its
    holder may write to it).  A block belongs to the host thread and the stream
    that were current when it was made, so a piece is only ever used in the
    stream order of its block's fill."""

    BLOCK = 1 << 16
    ALIGN = 16

    def __init__(self):
        self._local = threading.local()

    _SIZES = {torch.int32: 4, torch.int64: 8, torch.uint8: 1, torch.float32: 4}

    def take(self, device, count, dtype):
        size = self._SIZES.get(dtype)
        if size is None:
            size = torch.empty((), dtype=dtype).element_size()
        nbytes = count * size
        if nbytes > self.BLOCK // 4:
            return torch.zeros(count, dtype=dtype, device=device)
        blocks = getattr(self._local, "blocks", None)
        if blocks is None:
            blocks = self._local.blocks = {}
        key = (device_index(device), stream_handle(device))
        entry = blocks.get(key)
        if entry is None or entry[1] + nbytes > self.BLOCK:
            # the block, how much of it is handed out, and views of it by element type (made when first asked for)
            entry = blocks[key] = [torch.zeros(self.BLOCK, dtype=torch.uint8, device=device), 0, {}]
        at = entry[1]
        entry[1] = (at + nbytes + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        typed = entry[2].get(dtype)
        if typed is None:
            typed = entry[2][dtype] = entry[0].view(dtype)
        first = at // size  # `at` is a multiple of ALIGN, which every element size divides
        return typed[first:first + count]

    def fresh(self, device):
        """Forget the current stream's block: the next piece comes from a new one.  Call this at the start of
        every HIP graph capture: the block made inside the capture, fill included, then belongs to that graph
        alone (its replays put its own status words and counts back to zero and nobody else's)."""
        blocks = getattr(self._local, "blocks", None)
        if blocks is not None:
            blocks.pop((device_index(device), stream_handle(device)), None)


zeros = ZeroPool()


def status_word(device):
    return zeros.take(device, 1, torch.int32)


def describe_status(bits):
    names = []
    if bits & STAT_SERIAL_OVERFLOW:
        names.append("serial region overflow")
    if bits & STAT_CAPACITY:
        names.append("output capacity exceeded")
    if bits & STAT_INTERNAL:
        names.append("internal wait expired")
    if bits & STAT_BAD_INDEX:
        names.append("index out of range")
    if bits & STAT_RETRY:
        names.append("fast path declined the input (retry in general mode)")
    return ", ".join(names) or "ok"


def profile_enable(on=True, only=None, every=1):
    """Start (or stop) timing the tagged launches; `only` names the one kernel
    tag to time, `every` = n times every n-th launch of a tag."""
    L = lib()
    tag = -1
    if only is not None:
        names = [L.zen_profile_name(t).decode() for t in range(L.zen_profile_tags())]
        tag = names.index(only)
    check(L.zen_profile_only(tag), "profile_only")
    check(L.zen_profile_every(int(every)), "profile_every")
    check(L.zen_profile_enable(1 if on else 0), "profile_enable")


def profile_read():
    """{kernel name: (total ms, launches)} for every tag that recorded a launch."""
    L = lib()
    out = {}
    for tag in range(L.zen_profile_tags()):
        ms, cnt = ctypes.c_double(0), ctypes.c_int64(0)
        check(L.zen_profile_read(tag, ctypes.byref(ms), ctypes.byref(cnt)), "profile_read")
        if cnt.value:
            out[L.zen_profile_name(tag).decode()] = (ms.value, cnt.value)
    return out


# ---------------------------------------------------------------- ranges
# Named ranges around the steps of the path, under the names the reference gives its nvtx ranges (comm.py:66-144,
# tensor_load_balance.py:25-44, train.py:65-69, 176), so that a rocprofv3 --marker-trace run of a training step
# reads like an Nsight trace of the reference.  Off unless ZEN_ROCTX=1 is set or ranges_enable(True) is called:
# the hot calls then pay nothing for them.
import contextlib

_ranges_on = os.environ.get("ZEN_ROCTX", "") not in ("", "0")
_no_range = contextlib.nullcontext()


def ranges_enable(on=True):
    global _ranges_on
    _ranges_on = bool(on)


def annotate(name):
    """Context manager: a roctx range called `name` (torch.cuda.nvtx is roctx on ROCm), or nothing when ranges are off."""
    if not _ranges_on:
        return _no_range
    return torch.cuda.nvtx.range(name)
