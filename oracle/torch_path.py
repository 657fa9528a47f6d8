"""CPU baseline: the reference's torch-op sequence for the path, restated on CPU
tensors (TEST / BENCH INFRASTRUCTURE ONLY -- imported by tests and by bench.py's
cpu_baseline leg, never by the product package).

  select   train.py:79-84       abs, topk(sorted=False), min, where
  insert   functions_cuda_kernel.cu:97-167   the reference has no CPU insert:
                                the sequential C oracle stands in for the kernel
  compact  tensor_load_balance.py:24-51      chunk, != 0, boolean index, gather, cat
  merge    comm.py:32-44        cat, .type(int64), zeros, scatter_add_
  encode   comm.py:47-50        nonzero(as_tuple), gather
"""
import time

import numpy as np
import torch

from . import zen_oracle


def select(tensor, k):
    tensor_abs = tensor.abs()
    topk = torch.topk(tensor_abs, k, 0, largest=True, sorted=False)[0]
    threshold = torch.min(topk)
    return torch.where(tensor_abs >= threshold, tensor, torch.tensor(0, dtype=tensor.dtype))


def _as_oracle_array(t):
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def balance_sparse_tensor(tensor, partitions, memory_scale=1, rehash=3):
    numel = tensor.numel()
    m, sn = zen_oracle.table_sizes(numel, partitions, memory_scale)
    memory, serial, _, status = zen_oracle.sparse_balance(_as_oracle_array(tensor), m, sn, partitions, rehash)
    return torch.from_numpy(memory), torch.from_numpy(serial), status


def get_sub_sparse_tensors(tensor, memory, partitions):
    indices, values, splits = [], [], []
    for chunk in memory.chunk(partitions):
        sparse_indices = chunk[chunk != 0]
        sparse_values = tensor[sparse_indices.type(torch.long)]
        indices.append(sparse_indices)
        values.append(sparse_values)
        splits.append(sparse_indices.numel())
    return indices, values, torch.tensor(splits)


def load_balance(tensor, partitions, memory_scale=1, rehash=3):
    memory, serial, status = balance_sparse_tensor(tensor, partitions, memory_scale, rehash)
    indices, values, splits = get_sub_sparse_tensors(tensor, memory, partitions)
    s_indices, s_values, s_splits = get_sub_sparse_tensors(tensor, serial, partitions)
    indices = [torch.cat([a, b]) for a, b in zip(indices, s_indices)]
    values = [torch.cat([a, b]) for a, b in zip(values, s_values)]
    return indices, values, splits + s_splits, status


def decode_sparse_tensors(indices_tensors, values_tensors, dense_size):
    dtype = values_tensors[0].dtype
    dense = torch.zeros(dense_size, dtype=dtype)
    indices = torch.cat(indices_tensors).type(torch.int64)
    values = torch.cat(values_tensors)
    dense.scatter_add_(0, indices, values)
    return dense


def encode_sparse_tensor(tensor):
    sparse_indices = torch.nonzero(tensor, as_tuple=True)[0]
    return sparse_indices, tensor[sparse_indices]


def timed_pass(grad, k, partitions, peer_idx, peer_val):
    """One pass of the whole path on CPU tensors; returns (seconds per stage,
    results).  k == 0 skips the select stage (input already sparse)."""
    t = {}
    t0 = time.perf_counter()
    masked = select(grad, k) if k > 0 else grad
    t["select"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    indices, values, splits, status = load_balance(masked, partitions)
    t["partition"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    dense = decode_sparse_tensors(peer_idx, peer_val, grad.numel())
    m_idx, m_val = encode_sparse_tensor(dense)
    t["merge"] = time.perf_counter() - t0
    return t, (indices, values, splits, status, m_idx, m_val)
