"""Drop-in for the reference's tensor_load_balance.py.  `load_balance` runs as
one fused device pipeline (select, insert, slot-order compaction) instead of
2P boolean-mask compactions with a host sync each."""
import ctypes

import torch

from . import _lib
from .functions import last_status, sparse_balance


class _Mark:
    """A point in a stream's order that work on other streams may have to wait for.  The event is recorded
    only when another stream asks, at the tail the stream has then (further on in its order than the mark:
    waiting for more is safe, and since every dependency points back in host time no cycle can form), so a
    sequence of calls that stays on one stream puts no event between its kernels: on the device an event
    between two kernels of a stream costs about ten microseconds."""

    def __init__(self, stream):
        self.stream = stream
        self.event = None

    def wait(self, consumer):
        if consumer == self.stream:
            return
        if self.event is None:
            self.event = torch.cuda.Event()
            self.event.record(self.stream)
        consumer.wait_event(self.event)


class TensorPartition:
    """Same constructor and methods as the reference class
    (tensor_load_balance.py:5-51)."""

    # OR-ed into the mode of every fast-mode call (_lib.MODE_SLABS keeps the calls off the wide buckets)
    fast_flags = 0

    def __init__(self, partitions, memory_scale, rehash):
        self.partitions = partitions
        self.memory_scale = memory_scale
        self.rehash = rehash
        self.device = torch.cuda.current_device()
        self._tables = {}
        self._ahead = {}  # (device, slot) -> samples taken ahead of their calls (prepare)
        self._samples_next = {}  # shape of a call -> whether its pass over the tensor can take the next sample along

    # ------------------------------------------------------------ sizes
    def table_sizes(self, numel):
        """(hash table size, serial table size), tensor_load_balance.py:14-18."""
        memory_size = numel * self.memory_scale
        memory_size = int(memory_size // self.partitions * self.partitions)
        serial_memory_size = int(numel // self.partitions // 10 * self.partitions)
        return memory_size, serial_memory_size

    # ------------------------------------------- reference-shaped pieces
    def balance_sparse_tensor(self, tensor):
        """Allocates and fills the two tables (tensor_load_balance.py:13-21)."""
        with _lib.annotate("balance_sparse_tensor"):  # tensor_load_balance.py:44
            memory_size, serial_memory_size = self.table_sizes(tensor.numel())
            memory = torch.zeros(memory_size, dtype=torch.int32, device=tensor.device)
            serial_memory = torch.zeros(serial_memory_size, dtype=torch.int32, device=tensor.device)
            sparse_balance(tensor, memory, serial_memory, self.partitions, rehash=self.rehash)
            last_status().check()
            return memory, serial_memory

    def get_sub_sparse_tensors(self, tensor, memory):
        """Per-partition nonzero entries of a table and the values they point
        at (tensor_load_balance.py:24-40), as one compaction over the table."""
        flat = tensor.reshape(-1)
        found = self._nonzero_int32(memory)
        per_part = memory.numel() // self.partitions if self.partitions else 0
        if per_part == 0:
            bounds = torch.zeros(self.partitions + 1, dtype=torch.int64, device=memory.device)
        else:
            edges = torch.arange(self.partitions + 1, device=memory.device, dtype=torch.int64) * per_part
            bounds = torch.searchsorted(found[0], edges)
        splits = bounds[1:] - bounds[:-1]
        cuts = bounds.tolist()
        idx = found[1]
        indices = [idx[cuts[p]:cuts[p + 1]] for p in range(self.partitions)]
        values = [flat[i.long()] for i in indices]
        return indices, values, splits

    @staticmethod
    def _nonzero_int32(table):
        """(positions, entries) of the nonzero entries of an int32 table.  An
        int32 is nonzero iff its bit pattern read as float32 has a nonzero
        magnitude key, so the float compaction kernel serves."""
        from .comm import _select

        pos, val, _ = _select(table.view(torch.float32), None, idx64=True, capacity=table.numel())
        return pos, val.view(torch.int32)

    # ------------------------------------------------------- fused path
    _MAX_TABLES = 4

    def _table(self, device, m, slot=0):
        """The zeroed int32[m] table of (device, m, slot).  Gradient buckets of a
        few different sizes come round again and again (the hook is called per
        bucket, train.py:167-185), so a handful of tables is kept, least
        recently used first out."""
        key = (device if isinstance(device, torch.device) else torch.device(device), m, slot)
        t = self._tables.pop(key, None)
        if t is None:
            while len(self._tables) >= self._MAX_TABLES:
                self._tables.pop(next(iter(self._tables)))
            t = torch.zeros(m, dtype=torch.int32, device=device)
        self._tables[key] = t  # most recently used last
        return t

    def _honest_capacity(self, flat, thr, k):
        """Room for the selection without guessing `numel` (which would take a
        small selection off the bucket-slab path and size the workspace for the
        whole tensor): from k, from the count the threshold came with, or from
        a count of the nonzeros.  The last two take a pass over the tensor and read a device value."""
        if k > 0:
            return int(k) + int(k) // 4 + 4096  # ties at the threshold
        if thr is not None:
            # thr[1] counts the multiset the threshold was computed on, which may be a sample of the tensor
            # (compress): count what passes it in the tensor itself
            from .comm import _select_raw

            return _select_raw(flat, thr, False, 0)[2] + 1024
        return int(torch.count_nonzero(flat)) + 1024

    def _ahead_state(self, device, slot, create=False):
        # "free": per set of sampling memory, the mark behind the last call that used it; "pending": samples
        # taken and not yet picked up by their calls (tensor, size, k, capacity, workspace, set, mark, type,
        # workspace bytes)
        key = (_lib.device_index(device), slot)
        state = self._ahead.get(key)
        if state is None and create:
            # Calls made before the first prepare left no events behind (a call only keeps this book once
            # samples are taken ahead for its slot): wait for them all, once.
            torch.cuda.synchronize(device)
            state = self._ahead[key] = {"free": [None, None], "pending": []}
        return state

    def prepare(self, tensor, k, capacity, slot=0):
        """Takes the sample of a coming load_balance_flat(tensor, None, capacity,
        k=k, slot=slot) ahead, on the CURRENT stream, which may be another one
        than the call's: the sample then runs beside whatever the call's stream
        is still busy with (the previous bucket's sort and placement) instead of
        in front of the pass over the tensor.  The tensor must be ready in the
        current stream's order.  The call that follows finds the sample by
        itself (same tensor, k, capacity and slot) and waits for it; two samples
        per slot can be ahead of their calls.  Where there is nothing to take
        ahead (k == 0, small tensors) this does nothing."""
        _lib.require_gpu(tensor, "input")
        flat = tensor.reshape(-1)
        n = flat.numel()
        code = _lib.dtype_code(flat)
        m, _ = self.table_sizes(n)
        dev = flat.device
        L = _lib.lib()
        if k <= 0 or L.zen_load_balance_path(n, m, code, capacity, self.partitions, k,
                                             _lib.MODE_FAST | self.fast_flags) not in (2, 3):
            return
        state = self._ahead_state(dev, slot, create=True)
        busy = {entry[5] for entry in state["pending"]}
        if len(busy) >= 2:
            return  # both sets are spoken for
        which = 1 if 1 not in busy else 0  # the second first: a call that samples for itself prefers the first
        stream = torch.cuda.current_stream(dev)
        if state["free"][which] is not None:
            state["free"][which].wait(stream)  # the call that used this set last has finished
        nbytes = L.zen_load_balance_workspace(n, m, code, capacity, self.partitions)
        ws = _lib.scratch.get(dev, f"load_balance/{slot}", nbytes)
        table = self._table(dev, m, slot)
        rc = L.zen_load_balance_prepare(_lib.ptr(flat), code, n, m, self.partitions, int(k), capacity, _lib.ptr(table),
                                        _lib.MODE_FAST | self.fast_flags | (_lib.MODE_SECOND if which else 0),
                                        _lib.ptr(ws), ws.numel(),
                                        _lib.stream_of(dev))
        _lib.check(rc, "load_balance prepare")
        state["pending"].append((flat.data_ptr(), n, int(k), capacity, ws.data_ptr(), which, _Mark(stream), code,
                                 ws.numel()))

    def _next_sample(self, flat, next_tensor, next_k, capacity, next_capacity, slot, mode, used):
        """(flat view of `next_tensor`, its table or None if it has this call's size) if the call that is about
        to be made can take that tensor's sample along (same type, paths that sample, the other set of sampling
        memory free), else (None, None)."""
        if next_tensor is None or next_k <= 0:
            return None, None
        nxt = next_tensor.reshape(-1)
        if (nxt.dtype != flat.dtype or nxt.device != flat.device or not nxt.is_contiguous()
                or (mode & 0xff) != _lib.MODE_FAST):
            return None, None
        n, n2 = flat.numel(), nxt.numel()
        key = (n, n2, flat.dtype, capacity, next_capacity, next_k, mode & (0xff | _lib.MODE_SLABS))
        able = self._samples_next.get(key)
        if able is None:
            L = _lib.lib()
            m, _ = self.table_sizes(n)
            m2, _ = self.table_sizes(n2)
            code = _lib.dtype_code(flat)
            # this call must be on a path whose pass over the tensor samples, the next one on a path that picks
            # a sample up from its table
            able = self._samples_next[key] = bool(
                L.zen_encode_merge_samples_next(n, m, code, capacity, self.partitions, next_k, key[6])
                and L.zen_load_balance_path(n2, m2, code, next_capacity, self.partitions, next_k, key[6]) in (2, 3))
        if not able:
            return None, None
        state = self._ahead_state(flat.device, slot, create=True)
        if any(entry[5] == 1 - used for entry in state["pending"]):
            return None, None  # the other set holds a sample that is still to be picked up
        if state["free"][1 - used] is not None:
            state["free"][1 - used].wait(torch.cuda.current_stream(flat.device))
        if n2 == n and next_capacity == capacity:
            return nxt, None
        return nxt, self._table(flat.device, self.table_sizes(n2)[0], slot)

    def _sample_taken(self, nxt, next_k, capacity, ws, slot, which):
        """Books the sample the last call took along for the call that follows (see _next_sample)."""
        dev = nxt.device
        state = self._ahead_state(dev, slot, create=True)
        state["pending"].append((nxt.data_ptr(), nxt.numel(), next_k, capacity, ws.data_ptr(), which,
                                 _Mark(torch.cuda.current_stream(dev)), _lib.dtype_code(nxt), ws.numel()))

    def _take_ahead(self, flat, n, k, capacity, ws, slot, mode, thr, near):
        """The sample taken ahead for the call that is about to be made, if there is one: (mode flags that tell
        the library, the set of sampling memory the call will use).  Samples taken for other calls stay where
        they are; one that its bucket will never pick up (same tensor and size, other arguments) is dropped."""
        dev = flat.device
        state = self._ahead_state(dev, slot)  # None: no sample was ever taken ahead for this slot
        if state is None or k <= 0:
            return 0, 0
        L = _lib.lib()
        want = (flat.data_ptr(), n, k, capacity, ws.data_ptr())
        ahead = None
        for i, entry in enumerate(state["pending"]):
            if entry[:5] == want:
                ahead = state["pending"].pop(i)
                break
        usable = (mode & 0xff) == _lib.MODE_FAST and thr is None and near is None
        cur = torch.cuda.current_stream(dev)
        if ahead is not None and not usable:
            # taken for this very call, which will not use it: its histogram is cleared again
            self._discard(ahead, slot, dev)
            ahead = None
        if ahead is not None:
            ahead[6].wait(cur)
            return _lib.MODE_PREPARED | (_lib.MODE_SECOND if ahead[5] else 0), ahead[5]
        # the call samples for itself, in a set no pending sample sits in (and whose last user has finished)
        busy = {entry[5] for entry in state["pending"]}
        which = 0 if 0 not in busy else 1
        if which in busy:
            # both sets hold samples of other buckets: the older one gives way
            old = state["pending"].pop(0)
            self._discard(old, slot, dev)
            which = old[5]
        if state["free"][which] is not None:
            state["free"][which].wait(cur)
        return (_lib.MODE_SECOND if which else 0), which

    def _discard(self, entry, slot, dev):
        """Clears the sampling memory of a sample nobody will pick up (with the arguments it was taken with)."""
        L = _lib.lib()
        a_ptr, a_n, a_k, a_cap, a_ws, a_which, a_done, a_code, a_bytes = entry
        a_done.wait(torch.cuda.current_stream(dev))
        a_m, _ = self.table_sizes(a_n)
        _lib.check(L.zen_load_balance_prepare(
            ctypes.c_void_p(a_ptr), a_code, a_n, a_m, self.partitions, a_k, a_cap,
            _lib.ptr(self._table(dev, a_m, slot)), _lib.MODE_FAST | self.fast_flags | _lib.MODE_DISCARD |
            (_lib.MODE_SECOND if a_which else 0), ctypes.c_void_p(a_ws), a_bytes, _lib.stream_of(dev)),
            "load_balance discard")

    def _after_call(self, dev, slot, k, used):
        """The set of sampling memory a top-k call used is free again once the call has finished."""
        state = self._ahead_state(dev, slot)
        if k > 0 and state is not None:
            state["free"][used] = _Mark(torch.cuda.current_stream(dev))

    def load_balance_flat(self, tensor, thr=None, capacity=None, k=0, mode=_lib.MODE_FAST, thr_out=None, slot=0,
                          near=None):
        """Fused path without host synchronisation.  Returns (indices int32
        [capacity], values [capacity], splits int64[P] on device, status int32[1]
        on device); the first splits.sum() entries are valid, partition-major.
        Selection: `k` > 0 keeps the k largest magnitudes (ties kept; `thr_out`,
        an int32[2] device tensor, receives the threshold key and the count);
        else `thr` is the device tensor written by topk_threshold; else the
        nonzeros.  With `k`, `near` may be a device tensor whose first word is
        a key close to the threshold, e.g. the `thr_out` of the previous call
        on this gradient bucket: the call then takes no sample (one kernel
        less) and raises STAT_RETRY if the key was too far off.  A status with
        STAT_RETRY (fast mode only) means the call must be repeated (without
        `near`, or with mode=MODE_GENERAL); load_balance does that.
        Calls that may be in flight at the same time (different streams, e.g.
        one gradient bucket's encode next to the previous bucket's) must use
        different `slot` numbers: a slot owns its workspace and its table."""
        _lib.require_gpu(tensor, "input")
        flat = tensor.reshape(-1)
        n = flat.numel()
        code = _lib.dtype_code(flat)
        m, _ = self.table_sizes(n)
        if capacity is None:
            # no synchronisation here, so no count: the largest the library takes.  A caller that knows a bound
            # should pass it (load_balance works one out): this default sizes everything for the whole tensor.
            capacity = min(n, (1 << 29) - 1)
        if (mode & 0xff) == _lib.MODE_FAST:
            mode |= self.fast_flags
        dev = flat.device
        L = _lib.lib()
        out_idx = torch.empty(capacity, dtype=torch.int32, device=dev)
        out_val = torch.empty(capacity, dtype=flat.dtype, device=dev)
        splits = _lib.zeros.take(dev, self.partitions, torch.int64)
        status = _lib.status_word(dev)
        nbytes = L.zen_load_balance_workspace(n, m, code, capacity, self.partitions)
        ws = _lib.scratch.get(dev, f"load_balance/{slot}", nbytes)
        table = self._table(dev, m, slot)
        flags, used = self._take_ahead(flat, n, int(k), capacity, ws, slot, mode, thr, near)
        if near is not None and k > 0 and thr is None:
            thr, flags = near, flags | _lib.MODE_FLOOR
        rc = L.zen_load_balance(
            _lib.ptr(flat), code, n, m, self.partitions, self.rehash, _lib.ptr(thr), int(k), _lib.ptr(thr_out),
            _lib.ptr(out_idx), _lib.ptr(out_val), capacity, _lib.ptr(splits), _lib.ptr(table), mode | flags,
            _lib.ptr(ws), ws.numel(), _lib.ptr(status), _lib.stream_of(dev))
        if rc != _lib.OK:
            table.zero_()  # a call that failed half way may have left entries behind
        _lib.check(rc, "load_balance")
        self._after_call(dev, slot, int(k), used)
        return out_idx, out_val, splits, status

    def load_balance(self, tensor, thr=None, capacity=None, k=0, mode=None, grow=None):
        """Returns (indices[P], values[P], splits) like the reference
        (tensor_load_balance.py:43-51).  The per-partition tensors are views of
        two contiguous buffers; slicing them needs the split sizes on the
        host, which is this call's only synchronisation.  Without a `capacity`
        one is worked out and the call is repeated with four times as much
        when the selection turns out larger; `grow=True` asks for the same
        with a capacity that is the caller's estimate."""
        flat = tensor.reshape(-1)
        n = flat.numel()
        if grow is None:
            grow = capacity is None
        if capacity is None:
            capacity = min(n, self._honest_capacity(flat, thr, k))
        fast = _lib.MODE_FAST | self.fast_flags
        every = ([fast] + ([_lib.MODE_FAST | _lib.MODE_SLABS] if not fast & _lib.MODE_SLABS else []) +
                 [_lib.MODE_GENERAL]) if mode is None else [mode]
        modes = list(every)
        while modes:
            out_idx, out_val, splits, status = self.load_balance_flat(tensor, thr, capacity, k, modes[0])
            host = torch.cat([splits, status.to(torch.int64)]).tolist()
            bits = host[-1]
            if bits & (_lib.STAT_RETRY | _lib.STAT_INTERNAL):
                # a declined or aborted call may leave entries and counters behind in the table
                m, _ = self.table_sizes(n)
                self._table(tensor.device, m).zero_()
            if bits & _lib.STAT_RETRY:
                modes.pop(0)
            elif bits & _lib.STAT_CAPACITY and grow and capacity < n:
                # more passed than allowed for (a fast path short of room declines, so this is mostly the general
                # mode speaking): with more room the fast modes get their turn again
                capacity = min(n, max(sum(host[:-1]) + 1024, capacity * 4))
                modes = list(every)
            else:
                break
        if bits:
            raise RuntimeError("load_balance: " + _lib.describe_status(bits))
        indices, values, at = [], [], 0
        for p in range(self.partitions):
            indices.append(out_idx[at:at + host[p]])
            values.append(out_val[at:at + host[p]])
            at += host[p]
        return indices, values, splits
