"""Magnitude selection: the reference's `compress` (train.py:75-84) and the
exact top-k threshold BASELINE's configurations ask for."""
import math

import torch

from . import _lib


def topk_threshold(tensor, k):
    """Device tensor uint32[2]: [magnitude key of the k-th largest |x|, number
    of elements with key >= it].  The key is the bit pattern of |x| (bf16: 15
    bits, fp32: 31 bits); for non-NaN values key order is magnitude order, so
    this equals topk(|x|, k)[0].min() (train.py:81-82).  No host sync."""
    _lib.require_gpu(tensor, "input")
    flat = tensor.reshape(-1)
    L = _lib.lib()
    thr = torch.empty(2, dtype=torch.int32, device=flat.device)
    nbytes = L.zen_topk_threshold_workspace()
    ws = _lib.scratch.get(flat.device, "topk", nbytes)
    rc = L.zen_topk_threshold(_lib.ptr(flat), _lib.dtype_code(flat), flat.numel(), int(k),
                              _lib.ptr(thr), _lib.ptr(ws), ws.numel(), _lib.stream_of(flat.device))
    _lib.check(rc, "topk_threshold")
    return thr


def sample_threshold(tensor, sample_index, k):
    """(thr, status): thr as topk_threshold returns it for the multiset tensor.reshape(-1)[sample_index] (the
    sample of train.py:78-80), status int32[1] on the device (STAT_BAD_INDEX: a position outside the tensor).
    One gather kernel and the radix select, no intermediate tensor, no host sync."""
    _lib.require_gpu(tensor, "input")
    _lib.require_gpu(sample_index, "sample_index")
    flat = tensor.reshape(-1)
    if sample_index.dtype != torch.int64:
        raise RuntimeError("sample_index must be int64")
    L = _lib.lib()
    dev = flat.device
    s = sample_index.numel()
    code = _lib.dtype_code(flat)
    thr = torch.empty(2, dtype=torch.int32, device=dev)
    status = _lib.status_word(dev)
    ws = _lib.scratch.get(dev, "sample_threshold", L.zen_sample_threshold_workspace(s, code))
    rc = L.zen_sample_threshold(_lib.ptr(flat), code, flat.numel(), _lib.ptr(sample_index.reshape(-1)), s, int(k),
                                _lib.ptr(thr), _lib.ptr(ws), ws.numel(), _lib.ptr(status), _lib.stream_of(dev))
    _lib.check(rc, "sample_threshold")
    return thr, status


def threshold_value(tensor, thr):
    """The threshold as a 0-dim tensor of tensor.dtype (synchronises)."""
    key = int(thr[0].item()) & 0xFFFFFFFF
    if tensor.dtype == torch.bfloat16:
        return torch.tensor([key], dtype=torch.int16).view(torch.bfloat16)[0]
    return torch.tensor([key], dtype=torch.int32).view(torch.float32)[0]


def mask_below(tensor, thr):
    """where(|x| >= threshold, x, 0) as a new dense tensor (train.py:83)."""
    _lib.require_gpu(tensor, "input")
    out = torch.empty_like(tensor)
    rc = _lib.lib().zen_compress(_lib.ptr(tensor), _lib.dtype_code(tensor), tensor.numel(),
                                 _lib.ptr(thr), _lib.ptr(out), _lib.stream_of(tensor.device))
    _lib.check(rc, "compress")
    return out


def compress(top_k, tensor, sample_index=None):
    """Same contract as the reference's compress (train.py:75-84): tensors of
    at most 4096 elements pass through; otherwise the threshold is the
    (n_s*top_k//100)-th largest magnitude of a 1 % sample drawn with
    replacement, and everything below it is zeroed.  `sample_index` (int64
    positions) replaces the reference's device RNG draw so that results can be
    reproduced; None draws it with torch.randint like the reference."""
    numel = tensor.numel()
    if numel <= 4096:
        return tensor
    flat = tensor.reshape(-1)
    if sample_index is None:
        sample_index = torch.randint(0, numel, (math.ceil(0.01 * numel),), device=tensor.device)
    k = sample_index.numel() * top_k // 100
    if k < 1:
        # torch.min of the empty topk result raises in the reference
        raise RuntimeError("compress: top-k of the sample is empty")
    # a position outside the tensor counts as a zero and is flagged in the status word (not waited for here)
    thr, _ = sample_threshold(flat, sample_index, k)
    return mask_below(flat, thr).view_as(tensor)


def threshold_with_allgather(top_k, tensor, pg_group, sample_index=None, all_gather=None):
    """The threshold compress_with_allgather applies (train.py:56-71), as the
    device tensor topk_threshold returns, without the masked copy of the
    tensor: for callers that hand it on to the load balance, which selects
    while it reads the tensor anyway.  None for tensors of at most 4096
    elements (they pass through uncompressed, train.py:58-59)."""
    numel = tensor.numel()
    if numel <= 4096:
        return None
    flat = tensor.reshape(-1)
    if sample_index is None:
        sample_index = torch.randint(0, numel, (math.ceil(0.01 * numel),), device=tensor.device)
    if all_gather is None and pg_group.size() == 1:
        k = sample_index.numel() * top_k // 100
        if k < 1:
            raise RuntimeError("compress_with_allgather: top-k of the samples is empty")
        return sample_threshold(flat, sample_index, k)[0]  # one rank: its own sample is the whole multiset
    if all_gather is None:
        raise RuntimeError("compress_with_allgather needs an all_gather callable for more than one rank")
    sample = flat[sample_index]  # the exchange needs the sample as a tensor of its own
    samples = all_gather(sample)
    if samples.numel() != pg_group.size() * sample.numel():
        raise RuntimeError("compress_with_allgather: the gathered samples have the wrong size")
    k = samples.numel() * top_k // 100
    if k < 1:
        raise RuntimeError("compress_with_allgather: top-k of the samples is empty")
    return topk_threshold(samples.contiguous(), k)


def compress_with_allgather(top_k, tensor, pg_group, sample_index=None, all_gather=None):
    """The reference's compress_with_allgather (train.py:56-73): as compress,
    but the threshold is the (n_all*top_k//100)-th largest magnitude among
    the 1 % samples of every rank of pg_group.  `all_gather(sample)` returns
    the samples of all ranks as one tensor (the reference calls
    dist.all_gather_into_tensor there); this build ships no exchange, so it
    has to be passed in for groups of more than one rank."""
    with _lib.annotate("topk"), _lib.annotate("min"):  # train.py:65-68: one radix select here
        thr = threshold_with_allgather(top_k, tensor, pg_group, sample_index, all_gather)
    if thr is None:
        return tensor
    with _lib.annotate("where"):  # train.py:69
        return mask_below(tensor.reshape(-1), thr).view_as(tensor)
