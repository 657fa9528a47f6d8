"""Drop-in for the reference's extensions/cuda/functions.py: the two entry
points `sparse_balance` and `hash_index`, same argument order and in-place
semantics, backed by libzen_hip.so instead of the pybind CUDA module."""
import threading

import torch

from . import _lib


def sparse_balance(tensor, memory, serial_memory, partitions, rehash):
    """In-place insert of every nonzero index of `tensor` into the int32 hash
    table `memory` (split into `partitions` equal ranges), overflow into
    `serial_memory` (extensions/cuda/functions.py:4-12).

    Both tables must be zero on entry, as TensorPartition allocates them.  The
    result is deterministic: a slot belongs to the smallest index that probes
    it and each partition's serial entries are ascending.  bfloat16 as in the
    reference, float32 additionally.  Raises RuntimeError when a partition has
    more overflow entries than serial slots (the reference writes out of bounds).
    """
    assert tensor.is_cuda and tensor.dtype in (torch.bfloat16, torch.float32)
    assert memory.is_cuda and memory.dtype == torch.int32
    assert serial_memory.is_cuda and serial_memory.dtype == torch.int32
    for name, t in (("input", tensor), ("memory", memory), ("serial_memory", serial_memory)):
        _lib.require_gpu(t, name)
    numel = serial_memory.numel()
    numel_per_part = numel // partitions
    # serial base offsets, extensions/cuda/functions.py:8-11
    offsets = torch.arange(partitions, dtype=torch.int32, device=tensor.device) * numel_per_part
    status = _lib.status_word(tensor.device)
    rc = _lib.lib().zen_sparse_balance(
        _lib.ptr(tensor), _lib.dtype_code(tensor), tensor.numel(),
        _lib.ptr(memory), memory.numel(), _lib.ptr(serial_memory), numel,
        _lib.ptr(offsets), partitions, rehash, _lib.ptr(status), _lib.stream_of(tensor.device))
    _lib.check(rc, "sparse_balance")
    _last.pending = _PendingStatus(status, offsets)  # the call itself returns None, like the reference's


_last = threading.local()


def last_status():
    """The calling thread's most recent sparse_balance: an object whose
    check() synchronises and raises if the device flagged a condition (a serial
    region that overflowed), with the status word and the final ticket counters
    as attributes.  The reference has no such thing: it writes out of bounds."""
    return getattr(_last, "pending", None)


class _PendingStatus:
    """Kept per host thread after every sparse_balance (see last_status): the
    device status word and final ticket counters, checked only on request so
    the call itself stays asynchronous and returns None as the reference's does."""

    def __init__(self, status, offsets):
        self.status = status
        self.offsets = offsets

    def check(self):
        bits = int(self.status.item())
        if bits:
            raise RuntimeError("sparse_balance: " + _lib.describe_status(bits))


def hash_index(index, partitions):
    """index[t] = partition id of t for every t < index.numel(); the contents
    on entry are ignored (extensions/cuda/functions.py:14-15)."""
    assert index.is_cuda and index.dtype == torch.int32
    _lib.require_gpu(index, "input")
    rc = _lib.lib().zen_hash_index(_lib.ptr(index), index.numel(), partitions, _lib.stream_of(index.device))
    _lib.check(rc, "hash_index")
