"""Drop-in for the encode / decode / mapping half of the reference's comm.py
(LoadBalanceAllreduce).  The collectives around it are not part of this
package: one GPU computes its own share, the full P-way partition of its
gradient and the merge of P incoming payloads."""
import ctypes
import itertools

import torch

from . import _lib
from .functions import hash_index
from .tensor_load_balance import TensorPartition


class LocalGroup:
    """Stands in for a torch.distributed process group when there is none: it
    only answers size() and rank(), which is all this path asks of a group."""

    def __init__(self, size, rank=0):
        self._size, self._rank = size, rank

    def size(self):
        return self._size

    def rank(self):
        return self._rank


def _select_raw(tensor, thr, idx64, capacity=None):
    """(indices, values, count, status bits) of the selected elements of a flat tensor, ascending; the count
    is that of all elements that pass, also beyond `capacity` (then the bits hold STAT_CAPACITY and the first
    `capacity` entries are there).  Synchronises."""
    flat = tensor.reshape(-1)
    n = flat.numel()
    dev = flat.device
    if capacity is None:
        capacity = n
    L = _lib.lib()
    code = _lib.dtype_code(flat)
    out_idx = torch.empty(capacity, dtype=torch.int64 if idx64 else torch.int32, device=dev)
    out_val = torch.empty(capacity, dtype=flat.dtype, device=dev)
    count = torch.zeros(1, dtype=torch.int64, device=dev)
    status = _lib.status_word(dev)
    ws = _lib.scratch.get(dev, "select", L.zen_select_workspace(n, code))
    rc = L.zen_select(_lib.ptr(flat), code, n, _lib.ptr(thr), _lib.ptr(out_idx), 1 if idx64 else 0,
                      _lib.ptr(out_val), capacity, _lib.ptr(count), _lib.ptr(ws), ws.numel(),
                      _lib.ptr(status), _lib.stream_of(dev))
    _lib.check(rc, "select")
    host = torch.cat([count, status.to(torch.int64)]).tolist()
    kept = min(host[0], capacity)
    return out_idx[:kept], out_val[:kept], host[0], host[1]


def _select(tensor, thr, idx64, capacity=None, grow=False):
    """Ascending (indices, values, count) of the selected elements of a flat tensor.  With `grow`, a selection
    that does not fit `capacity` is taken again with room for exactly what passed (the first call counted
    it); any other trouble raises at once."""
    idx, val, count, bits = _select_raw(tensor, thr, idx64, capacity)
    if bits == _lib.STAT_CAPACITY and grow:
        idx, val, count, bits = _select_raw(tensor, thr, idx64, count)
    if bits:
        raise RuntimeError("select: " + _lib.describe_status(bits))
    return idx, val, count


class LoadBalanceAllreduce:
    """Constructor and method names of the reference class (comm.py:8-56)."""

    def __init__(self, process_group, global_ranks, logger, memory_scale=1, rehash=3):
        self.name = "LoadBalanceAllreduce"
        self.device = torch.cuda.current_device()
        self.process_group = process_group
        self.global_ranks = global_ranks
        self.partitions = process_group.size()
        self.local_rank = process_group.rank() if hasattr(process_group, "rank") else 0
        self.tensor_partition = self.get_tensor_partition_obj(memory_scale, rehash)
        self.logger = logger
        self.mapping = {}
        self._step_sizes = {}    # shape of an encode_merge_flat call -> (table size, workspace bytes, merge workspace bytes)
        self._bitmap_ranks = {}  # numel -> (mapping list of this rank, its rank table)
        self._dense_dicts = {}   # numel -> dictionary of decode_bitmaps_dense

    def get_tensor_partition_obj(self, memory_scale, rehash):
        return TensorPartition(partitions=self.partitions, memory_scale=memory_scale, rehash=rehash)

    def stack_tensors(self, tensors, shape=-1):
        # comm.py:25-29; payloads that already sit back to back in one buffer
        # (what an all-to-all into a single flat buffer leaves) are not copied
        if isinstance(tensors, (list, tuple)):
            flat = _as_one_buffer(tensors)
            return (flat if flat is not None else torch.cat(list(tensors))).reshape(shape)
        return tensors.reshape(shape)

    # ------------------------------------------------------------ merge
    def decode_sparse_tensors(self, indices_tensors, values_tensors, alltoall_dense_size, ascending=False):
        """Dense tensor of `alltoall_dense_size` elements in the value dtype with
        every payload scatter-added into it (comm.py:32-44).  Sums are taken in
        fp32 in payload order and rounded once.  `ascending` says that every
        tensor of the list is a strictly ascending index list (what the second
        exchange and method 1 deliver, comm.py:113-117, 142-145): the dense
        tensor is then built tile by tile without a sort; a list that is not
        ascending after all only costs the time of the attempt."""
        lists = indices_tensors if isinstance(indices_tensors, (list, tuple)) else [indices_tensors]
        sizes = [int(t.numel()) for t in lists]
        indices = self.stack_tensors(indices_tensors)
        values = self.stack_tensors(values_tensors)
        assert indices.dtype in (torch.int32, torch.int64)
        _lib.require_gpu(indices, "indices")
        _lib.require_gpu(values, "values")
        dev = values.device
        L = _lib.lib()
        r = indices.numel()
        dense = torch.empty(alltoall_dense_size, dtype=values.dtype, device=dev)
        if ascending and 1 <= len(sizes) <= 64 and sum(sizes) == r == values.numel():
            starts = (ctypes.c_int64 * (len(sizes) + 1))(0, *itertools.accumulate(sizes))
            ws = _lib.scratch.get(dev, "decode_sorted",
                                  L.zen_decode_dense_sorted_workspace(alltoall_dense_size, len(sizes)))
            status = _lib.status_word(dev)
            rc = L.zen_decode_dense_sorted(_lib.ptr(indices), int(indices.dtype == torch.int64), _lib.ptr(values),
                                           _lib.dtype_code(values), starts, len(sizes), _lib.ptr(dense),
                                           alltoall_dense_size, _lib.ptr(ws), ws.numel(), _lib.ptr(status),
                                           _lib.stream_of(dev))
            _lib.check(rc, "decode_sparse_tensors")
            if not int(status.item()):  # the reference's scatter_add_ raises on a bad index, also a sync
                return dense
        ws = _lib.scratch.get(dev, "decode", L.zen_decode_dense_workspace(r, alltoall_dense_size))
        for mode in self._fast_then_general():
            status = _lib.status_word(dev)
            rc = L.zen_decode_dense(_lib.ptr(indices), int(indices.dtype == torch.int64), _lib.ptr(values),
                                    _lib.dtype_code(values), r, _lib.ptr(dense), alltoall_dense_size, mode,
                                    _lib.ptr(ws), ws.numel(), _lib.ptr(status), _lib.stream_of(dev))
            _lib.check(rc, "decode_sparse_tensors")
            bits = int(status.item())  # the reference's scatter_add_ raises on a bad index, also a sync
            if not bits & _lib.STAT_RETRY:
                break
        if bits:
            raise RuntimeError("decode_sparse_tensors: " + _lib.describe_status(bits))
        return dense

    # OR-ed into the mode of every fast-mode call (_lib.MODE_SLABS keeps the calls off the wide buckets)
    fast_flags = 0

    def _fast_then_general(self):
        """The modes a call that may be declined (STAT_RETRY) goes through: the fast mode, the fast mode on the
        bucket slabs alone, the general mode."""
        fast = _lib.MODE_FAST | self.fast_flags
        return [fast] + ([_lib.MODE_FAST | _lib.MODE_SLABS] if not fast & _lib.MODE_SLABS else []) + [_lib.MODE_GENERAL]

    def encode_sparse_tensor(self, tensor):
        """(ascending int64 indices of the nonzeros, their values), comm.py:47-50."""
        _lib.require_gpu(tensor, "input")
        idx, val, _ = _select(tensor, None, idx64=True)
        return idx, val

    def merge_sparse_flat(self, indices_tensors, values_tensors, dense_size, capacity=None, idx64=False,
                          mode=_lib.MODE_FAST, slot=0):
        """decode_sparse_tensors followed by encode_sparse_tensor (comm.py:125-127)
        without the dense intermediate and without host synchronisation.
        Returns (indices, fp32 sums, count int64[1], status int32[1]); the first
        `count` entries are valid and ascending.  In fast mode a status with
        STAT_RETRY means the outputs are unspecified and the call must be repeated
        with mode=MODE_GENERAL (merge_sparse does that by itself).  Calls that
        may be in flight at the same time must use different `slot` numbers
        (a slot owns its workspace)."""
        indices = self.stack_tensors(indices_tensors)
        values = self.stack_tensors(values_tensors)
        _lib.require_gpu(indices, "indices")
        _lib.require_gpu(values, "values")
        dev = values.device
        L = _lib.lib()
        r = indices.numel()
        if capacity is None:
            capacity = r
        if (mode & 0xff) == _lib.MODE_FAST:
            mode |= self.fast_flags
        out_idx = torch.empty(capacity, dtype=torch.int64 if idx64 else torch.int32, device=dev)
        out_val = torch.empty(capacity, dtype=torch.float32, device=dev)
        count = _lib.zeros.take(dev, 1, torch.int64)
        status = _lib.status_word(dev)
        # The workspace is allocated zeroed and serves zen_merge only, which leaves its head (the counters
        # that must start at zero) zero again: no call spends a kernel on clearing it.
        ws = _lib.scratch.get(dev, f"merge/{slot}", L.zen_merge_workspace(r, dense_size), zero=True)
        rc = L.zen_merge(_lib.ptr(indices), int(indices.dtype == torch.int64), _lib.ptr(values),
                         _lib.dtype_code(values), r, dense_size, _lib.ptr(out_idx), 1 if idx64 else 0,
                         _lib.ptr(out_val), capacity, _lib.ptr(count), mode | _lib.MODE_ZEROED, _lib.ptr(ws),
                         ws.numel(), _lib.ptr(status), _lib.stream_of(dev))
        if rc != _lib.OK:
            ws[:L.zen_merge_zero_bytes()].zero_()
        _lib.check(rc, "merge_sparse")
        return out_idx, out_val, count, status

    def encode_merge_flat(self, partition, tensor, capacity, k, recv_indices, recv_values, dense_size, slot=0,
                          thr_out=None, near=None, merge_stream=None, next_tensor=None, next_k=None,
                          next_capacity=None):
        """One bucket's step in one call of the library: partition.load_balance_flat(tensor, None, capacity,
        k=k, slot=slot, thr_out=thr_out, near=near) of the rank's own gradient and merge_sparse_flat(recv_indices,
        recv_values, dense_size, slot=slot) of the entries it received, whose values have the gradient's type.
        Returns the two calls' tuples.  Everything is enqueued on the current stream unless `merge_stream` (a
        torch stream in whose order the received entries are ready) takes the merge.  A sample taken ahead with
        partition.prepare() is picked up as load_balance_flat would.  `next_tensor` (ready in the current stream's
        order) is the gradient of the call that follows on this slot, `next_k` its k (default: this call's): if
        it has this tensor's type, the pass over this tensor takes the sample of that call along (no kernel of
        its own), as if partition.prepare(next_tensor, next_k, next_capacity, slot) had been called
        (`next_capacity`: that call's capacity, default this call's; gradient buckets differ in size)."""
        from .tensor_load_balance import TensorPartition  # noqa: F401 (the type of `partition`)

        _lib.require_gpu(tensor, "input")
        flat = tensor.reshape(-1)
        indices = self.stack_tensors(recv_indices)
        values = self.stack_tensors(recv_values)
        _lib.require_gpu(indices, "indices")
        _lib.require_gpu(values, "values")
        assert values.dtype == flat.dtype, "received values must have the gradient's type"
        dev = flat.device
        L = _lib.lib()
        n, r = flat.numel(), indices.numel()
        code = _lib.dtype_code(flat)
        P = partition.partitions
        # sizes that only depend on the call's shape are worked out once (three crossings into the library less)
        shape = (n, code, capacity, P, partition.memory_scale, r, dense_size)
        sizes = self._step_sizes.get(shape)
        if sizes is None:
            m = partition.table_sizes(n)[0]
            sizes = self._step_sizes[shape] = (m, L.zen_load_balance_workspace(n, m, code, capacity, P),
                                               L.zen_merge_workspace(r, dense_size))
        m, ws_bytes, mws_bytes = sizes
        mode = _lib.MODE_FAST | partition.fast_flags
        out_idx = torch.empty(capacity, dtype=torch.int32, device=dev)
        out_val = torch.empty(capacity, dtype=flat.dtype, device=dev)
        m_idx = torch.empty(r, dtype=torch.int32, device=dev)
        m_val = torch.empty(r, dtype=torch.float32, device=dev)
        small = _lib.zeros.take(dev, P + 2, torch.int64)  # split sizes, merged count, the two status words
        splits, count = small[:P], small[P:P + 1]
        status2 = small[P + 1:P + 2].view(torch.int32)
        status, m_status = status2[0:1], status2[1:2]
        if next_k is None:
            next_k = k
        if next_capacity is None:
            next_capacity = capacity
        if next_tensor is not None and next_k > 0 and (next_tensor.numel() != n or next_capacity != capacity):
            # the next call shares the slot's workspace: it must not move between the two calls
            n2 = next_tensor.numel()
            shape2 = (n2, code, next_capacity, P, partition.memory_scale)
            bytes2 = self._step_sizes.get(shape2)
            if bytes2 is None:
                bytes2 = self._step_sizes[shape2] = L.zen_load_balance_workspace(
                    n2, partition.table_sizes(n2)[0], code, next_capacity, P)
            ws_bytes = max(ws_bytes, bytes2)
        ws = _lib.scratch.get(dev, f"load_balance/{slot}", ws_bytes)
        mws = _lib.scratch.get(dev, f"merge/{slot}", mws_bytes, zero=True)
        table = partition._table(dev, m, slot)
        flags, used = partition._take_ahead(flat, n, int(k), capacity, ws, slot, mode, None, near)
        thr = None
        if near is not None and k > 0:
            thr, flags = near, flags | _lib.MODE_FLOOR
        nxt, nxt_table = partition._next_sample(flat, next_tensor, int(next_k), capacity, next_capacity, slot,
                                                mode | flags, used)
        other = nxt is not None and nxt_table is not None
        a = _lib.EncodeMergeArgs(
            flat.data_ptr(), code, n, m, P, partition.rehash, thr.data_ptr() if thr is not None else None, int(k),
            thr_out.data_ptr() if thr_out is not None else None, out_idx.data_ptr(), out_val.data_ptr(), capacity,
            splits.data_ptr(), table.data_ptr(), mode | flags, ws.data_ptr(), ws.numel(), status.data_ptr(),
            indices.data_ptr(), int(indices.dtype == torch.int64), values.data_ptr(), r, dense_size,
            m_idx.data_ptr(), 0, m_val.data_ptr(), r, count.data_ptr(),
            _lib.MODE_FAST | self.fast_flags | _lib.MODE_ZEROED, mws.data_ptr(), mws.numel(), m_status.data_ptr(),
            _lib.stream_handle(dev), merge_stream.cuda_stream if merge_stream is not None else None,
            nxt.data_ptr() if nxt is not None else None, int(next_k) if nxt is not None else 0,
            nxt.numel() if other else 0, nxt_table.numel() if other else 0, next_capacity if other else 0,
            nxt_table.data_ptr() if other else None)
        self.last_encode_merge_args = a  # what the library was called with (its buffers live as long as the results)
        rc = L.zen_encode_merge(ctypes.byref(a))
        if rc != _lib.OK:
            mws[:L.zen_merge_zero_bytes()].zero_()
        _lib.check(rc, "encode_merge")
        partition._after_call(dev, slot, int(k), used)
        if nxt is not None:
            partition._sample_taken(nxt, int(next_k), next_capacity, ws, slot, 1 - used)
        return (out_idx, out_val, splits, status), (m_idx, m_val, count, m_status)

    def round_merged_flat(self, indices, sums, count, dtype):
        """What comm.py:125-127 hands to the second exchange, from merge_sparse_flat's output and without host
        synchronisation: the fp32 sums rounded once to `dtype`, the entries that round to zero dropped, the rest
        in their order.  Returns (indices, values, count int64[1], status int32[1])."""
        _lib.require_gpu(indices, "indices")
        dev = indices.device
        L = _lib.lib()
        cap = indices.numel()
        out_idx = torch.empty_like(indices)
        out_val = torch.empty(cap, dtype=dtype, device=dev)
        kept = _lib.zeros.take(dev, 1, torch.int64)
        status = _lib.status_word(dev)
        ws = _lib.scratch.get(dev, "round_compact", L.zen_round_compact_workspace(cap))
        rc = L.zen_round_compact(_lib.ptr(indices), int(indices.dtype == torch.int64), _lib.ptr(sums), _lib.ptr(count),
                                 cap, _lib.dtype_code(out_val), _lib.ptr(out_idx), _lib.ptr(out_val), _lib.ptr(kept),
                                 _lib.ptr(ws), ws.numel(), _lib.ptr(status), _lib.stream_of(dev))
        _lib.check(rc, "round_merged")
        return out_idx, out_val, kept, status

    def merge_rounded(self, indices_tensors, values_tensors, dense_size, dtype):
        """merge_sparse followed by the rounding of round_merged_flat: (int64 indices, values of `dtype`), with
        one host synchronisation (the result's size) instead of three."""
        for mode in self._fast_then_general():
            idx, val, count, status = self.merge_sparse_flat(indices_tensors, values_tensors, dense_size,
                                                             idx64=True, mode=mode)
            r_idx, r_val, kept, r_status = self.round_merged_flat(idx, val, count, dtype)
            host = torch.cat([kept, status.to(torch.int64), r_status.to(torch.int64)]).tolist()
            if host[1] & (_lib.STAT_RETRY | _lib.STAT_INTERNAL):
                self.reset_merge_workspace(idx.device)
            if not host[1] & _lib.STAT_RETRY:
                break
        if host[1] | host[2]:
            raise RuntimeError("merge_rounded: " + _lib.describe_status(host[1] | host[2]))
        return r_idx[:host[0]], r_val[:host[0]]

    def reset_merge_workspace(self, device, slot=0):
        """After a merge_sparse_flat whose status carried STAT_RETRY or
        STAT_INTERNAL: clears the head of the slot's workspace again."""
        L = _lib.lib()
        ws = _lib.scratch.get(device, f"merge/{slot}", 256, zero=True)
        ws[:min(ws.numel(), L.zen_merge_zero_bytes())].zero_()

    def merge_sparse(self, indices_tensors, values_tensors, dense_size):
        """Synchronising form of merge_sparse_flat: (int64 indices, fp32 sums)."""
        for mode in self._fast_then_general():
            idx, val, count, status = self.merge_sparse_flat(indices_tensors, values_tensors, dense_size,
                                                             idx64=True, mode=mode)
            host = torch.cat([count, status.to(torch.int64)]).tolist()
            if host[1] & (_lib.STAT_RETRY | _lib.STAT_INTERNAL):
                self.reset_merge_workspace(idx.device)
            if not host[1] & _lib.STAT_RETRY:
                break
        if host[1]:
            raise RuntimeError("merge_sparse: " + _lib.describe_status(host[1]))
        return idx[:host[0]], val[:host[0]]

    # ---------------------------------------------------------- mapping
    def calculate_mapping(self, numel):
        """List of P ascending int64 tensors: the indices of each partition
        (comm.py:52-56)."""
        L = _lib.lib()
        dev = torch.device("cuda", self.device)
        out = torch.empty(numel, dtype=torch.int64, device=dev)
        counts = torch.zeros(self.partitions, dtype=torch.int64, device=dev)
        ws = _lib.scratch.get(dev, "mapping", L.zen_mapping_workspace(numel, self.partitions))
        status = _lib.status_word(dev)
        rc = L.zen_mapping(numel, self.partitions, _lib.ptr(out), _lib.ptr(counts), _lib.ptr(ws), ws.numel(),
                           _lib.ptr(status), _lib.stream_of(dev))
        _lib.check(rc, "calculate_mapping")
        sizes = torch.cat([counts, status.to(torch.int64)]).tolist()
        if sizes.pop():
            raise RuntimeError("calculate_mapping: " + _lib.describe_status(int(status.item())))
        mapping, at = [], 0
        for c in sizes:
            mapping.append(out[at:at + c])
            at += c
        return mapping

    # ----------------------------------------------------------- bitmap

    def encode_bitmap_flat(self, sparse_indices, numel, count=None):
        """encode_bitmap without host synchronisation: (uint8 bitmap, status
        int32[1]).  `count` (int64[1] on the device) limits the indices that
        are looked at to the first `count`."""
        mapping = self.mapping[numel][self.local_rank]
        _lib.require_gpu(sparse_indices, "sparse_indices")
        if sparse_indices.dtype not in (torch.int32, torch.int64):
            raise RuntimeError("sparse_indices must be int32 or int64")
        dev = sparse_indices.device
        L = _lib.lib()
        members = mapping.numel()
        words = torch.empty(max(1, L.zen_bitmap_words(members)), dtype=torch.int32, device=dev)
        status = _lib.status_word(dev)
        # the rank table lives next to the mapping it belongs to (same cache, same lifetime)
        cached = self._bitmap_ranks.get(numel)
        if cached is None or cached[0] is not mapping:
            rank_at = torch.empty(L.zen_bitmap_rank_words(numel), dtype=torch.int32, device=dev)
            _lib.check(L.zen_bitmap_ranks(_lib.ptr(mapping), members, numel, _lib.ptr(rank_at),
                                          _lib.stream_of(dev)), "encode_bitmap")
            cached = self._bitmap_ranks[numel] = (mapping, rank_at)
        rc = L.zen_bitmap_encode(_lib.ptr(mapping), members, _lib.ptr(sparse_indices),
                                 int(sparse_indices.dtype == torch.int64), sparse_indices.numel(),
                                 _lib.ptr(count) if count is not None else None, _lib.ptr(cached[1]), numel,
                                 _lib.ptr(words), _lib.ptr(status), _lib.stream_of(dev))
        _lib.check(rc, "encode_bitmap")
        return words.view(torch.uint8)[:(members + 7) // 8], status

    def encode_bitmap(self, sparse_indices, numel):
        """One bit per member of this rank's mapping list, set where the member
        is among sparse_indices; least significant bit first, padded to a whole
        byte (comm.py:59-85).  self.mapping[numel] must exist (comm.py:135)."""
        bitmap, status = self.encode_bitmap_flat(sparse_indices, numel)
        bits = int(status.item())
        if bits & _lib.STAT_BAD_INDEX:  # result[indices] = 1 with an index == len(result), comm.py:63
            raise IndexError("encode_bitmap: an index lies beyond the last member of the mapping")
        if bits:
            raise RuntimeError("encode_bitmap: " + _lib.describe_status(bits))
        return bitmap

    def decode_bitmap(self, bitmap_indices, numel):
        """For every rank i the members of mapping[numel][i] whose bit is set in
        bitmap_indices[i], ascending int64 (comm.py:87-99)."""
        mapping_tensor = self.mapping[numel]
        L = _lib.lib()
        outs, counts = [], []
        status = None
        for i, bitmap_tensor in enumerate(bitmap_indices):
            mapping = mapping_tensor[i]
            _lib.require_gpu(bitmap_tensor, "bitmap")
            if bitmap_tensor.dtype != torch.uint8:
                raise RuntimeError("bitmap must be uint8")
            dev = bitmap_tensor.device
            members = mapping.numel()
            if bitmap_tensor.numel() * 8 < members:  # the mask would be shorter than the list it indexes, comm.py:97-98
                raise IndexError("decode_bitmap: bitmap shorter than the mapping")
            if status is None:
                status = _lib.status_word(dev)
            # a set bit costs eight bytes of output: room for every bit that can be set
            capacity = min(members, bitmap_tensor.numel() * 8)
            out = torch.empty(capacity, dtype=torch.int64, device=dev)
            count = torch.zeros(1, dtype=torch.int64, device=dev)
            ws = _lib.scratch.get(dev, "bitmap", L.zen_bitmap_decode_workspace(members))
            rc = L.zen_bitmap_decode(_lib.ptr(mapping), members, _lib.ptr(bitmap_tensor), bitmap_tensor.numel(),
                                     _lib.ptr(out), capacity, _lib.ptr(count), _lib.ptr(ws), ws.numel(),
                                     _lib.ptr(status), _lib.stream_of(dev))
            _lib.check(rc, "decode_bitmap")
            outs.append(out)
            counts.append(count)
        if not outs:
            return []
        host = torch.cat(counts + [status.to(torch.int64)]).tolist()
        if host[-1]:
            raise RuntimeError("decode_bitmap: " + _lib.describe_status(host[-1]))
        return [out[:c] for out, c in zip(outs, host)]

    def decode_bitmaps_dense(self, bitmap_indices, values_tensors, numel):
        """decode_bitmap for every rank followed by decode_sparse_tensors
        (comm.py:136-145) in one pass: bitmap_indices[i] / values_tensors[i] are
        rank i's bitmap over partition i's index list and the values of its set
        bits in order; returns the dense tensor of `numel` elements in the
        values' dtype.  Neither the index lists nor self.mapping are needed: a
        dictionary of two bytes per element (per tile of the dense tensor, the
        places of its indices ordered by partition) is built on first use of a
        `numel` and cached like the reference caches the mapping
        (comm.py:132-134)."""
        if len(bitmap_indices) != self.partitions or len(values_tensors) != self.partitions:
            raise RuntimeError("decode_bitmaps_dense: one bitmap and one value list per rank")
        for t in bitmap_indices:
            _lib.require_gpu(t, "bitmap")
            if t.dtype != torch.uint8:
                raise RuntimeError("bitmap must be uint8")
        L = _lib.lib()
        dev = values_tensors[0].device
        cached = self._dense_dicts.get(numel)
        if cached is None:
            nbytes = L.zen_bitmap_dense_dict_bytes(numel, self.partitions)
            if nbytes == 0:
                raise ValueError("decode_bitmaps_dense: at most 64 partitions, numel below 2^31")
            cached = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            _lib.check(L.zen_bitmap_dense_dict(numel, self.partitions, _lib.ptr(cached), None, _lib.stream_of(dev)),
                       "decode_bitmaps_dense")
            self._dense_dicts[numel] = cached
        bitmaps = self.stack_tensors(list(bitmap_indices))
        values = self.stack_tensors(list(values_tensors))
        _lib.require_gpu(values, "values")
        P = self.partitions
        bm_start = (ctypes.c_int64 * (P + 1))(0, *itertools.accumulate(int(t.numel()) for t in bitmap_indices))
        v_start = (ctypes.c_int64 * (P + 1))(0, *itertools.accumulate(int(t.numel()) for t in values_tensors))
        dense = torch.empty(numel, dtype=values.dtype, device=dev)
        ws = _lib.scratch.get(dev, "bitmap_dense", L.zen_bitmap_dense_workspace(numel, P))
        status = _lib.status_word(dev)
        rc = L.zen_bitmap_dense(_lib.ptr(cached), numel, P, _lib.ptr(bitmaps), bm_start, _lib.ptr(values),
                                _lib.dtype_code(values), v_start, _lib.ptr(dense), _lib.ptr(ws), ws.numel(),
                                _lib.ptr(status), _lib.stream_of(dev))
        _lib.check(rc, "decode_bitmaps_dense")
        bits = int(status.item())  # the reference's masking and scatter_add_ raise on a mismatch, also a sync
        if bits & _lib.STAT_BAD_INDEX:
            raise IndexError("decode_bitmaps_dense: a bitmap is shorter than its partition's index list, or has "
                             "more set bits than values came with it")
        if bits:
            raise RuntimeError("decode_bitmaps_dense: " + _lib.describe_status(bits))
        return dense

    # ------------------------------------------------- the whole exchange

    def zen_sparse_comm(self, tensor, method, thr=None, capacity=None):
        """The reference's driver of one sparse all-reduce (comm.py:101-150):
        method 1 = all-gather of (indices, values); 2 = load balance, exchange of
        the buckets, merge, all-gather of the merged indices; 3 = as 2 with the
        indices travelling as bitmaps.  The exchanges themselves belong to
        `self.ddp`, an object with the reference backend's allgather /
        allgather_padding / alltoallv (DDPbackend.py:13-41, 71-81); this build
        ships none, so the attribute has to be set by the caller.
        The reference is handed a tensor that compress has thresholded already;
        with `thr` (the device tensor topk_threshold returns) the tensor is the
        gradient as it is and everything below that magnitude counts as zero:
        the masked copy and the pass that reads it again fall away.  `capacity`
        then says how many elements are expected to pass."""
        ddp = getattr(self, "ddp", None)
        if ddp is None:
            raise RuntimeError("zen_sparse_comm needs a communication backend in self.ddp")
        numel = tensor.numel()
        ann = _lib.annotate
        if method == 1:
            with ann("encode_sparse_tensor"):
                if thr is None:
                    sparse_indices, sparse_values = self.encode_sparse_tensor(tensor)
                else:
                    _lib.require_gpu(tensor, "input")
                    sparse_indices, sparse_values, _ = _select(tensor, thr, idx64=True, capacity=capacity, grow=True)
            with ann("allgatherv indices"):
                indices_tensors = ddp.allgather_padding(sparse_indices)
            with ann("allgatherv values"):
                values_tensors = ddp.allgather_padding(sparse_values)
            with ann("decode_sparse_tensors"):
                return self.decode_sparse_tensors(indices_tensors, values_tensors, numel, ascending=True)
        with ann("load_balance"):
            indices, values, splits = self.tensor_partition.load_balance(tensor, thr=thr, capacity=capacity,
                                                                         grow=True if thr is not None else None)
        with ann("allgather"):
            gather_splits = ddp.allgather(splits)
        with ann("alltoallv indices"):
            indices_tensors = ddp.alltoallv(indices, gather_splits)
        with ann("alltoallv values"):
            values_tensors = ddp.alltoallv(values, gather_splits)
        # decode_sparse_tensors + encode_sparse_tensor (comm.py:125-127) without the dense tensor in between:
        # fp32 sums in payload order, rounded once to the tensor's type, what rounds to zero dropped (the two
        # ranges of the reference are one step here and carry both names)
        with ann("decode_sparse_tensors"), ann("encode_sparse_tensor"):
            sparse_indices, sparse_values = self.merge_rounded(indices_tensors, values_tensors, numel, tensor.dtype)
        if method == 2:
            with ann("allgather indices"):
                indices_tensors = ddp.allgather_padding(sparse_indices)
        else:
            if numel not in self.mapping:
                with ann("calculate_mapping"):
                    self.mapping[numel] = self.calculate_mapping(numel)
            with ann("allgather_bitmap"):
                with ann("encode_bitmap"):
                    bitmap_indices = self.encode_bitmap(sparse_indices, numel)
                with ann("allgatherv"):
                    bitmap_indices_gather = ddp.allgather_padding(bitmap_indices)
            with ann("allgather indices"):
                values_tensors = ddp.allgather_padding(sparse_values)
            if self.partitions <= 64:
                # decode_bitmap + decode_sparse_tensors (comm.py:140-145) in one pass, without the indices
                with ann("decode_bitmap"), ann("decode_sparse_tensors"):
                    return self.decode_bitmaps_dense(bitmap_indices_gather, values_tensors, numel)
            with ann("decode_bitmap"):
                indices_tensors = self.decode_bitmap(bitmap_indices_gather, numel)
            with ann("decode_sparse_tensors"):
                return self.decode_sparse_tensors(indices_tensors, values_tensors, numel, ascending=True)
        with ann("allgather indices"):
            values_tensors = ddp.allgather_padding(sparse_values)
        with ann("decode_sparse_tensors"):
            return self.decode_sparse_tensors(indices_tensors, values_tensors, numel, ascending=True)


def _as_one_buffer(tensors):
    """If the 1-D tensors are consecutive views of one storage, the covering
    view; else None."""
    if not tensors:
        return None
    first = tensors[0]
    if first.dim() != 1 or not first.is_contiguous():
        return None
    total = 0
    base = first.data_ptr()
    for t in tensors:
        if (t.dim() != 1 or t.dtype != first.dtype or not t.is_contiguous()
                or t.untyped_storage().data_ptr() != first.untyped_storage().data_ptr()
                or t.data_ptr() != base + total * first.element_size()):
            return None
        total += t.numel()
    return torch.as_strided(first, (total,), (1,))
