"""The DDP communication hook of the reference's training driver
(train.py:158-185) as a callable object: same arguments, same return value (a
completed torch.futures.Future holding the tensor), same steps in the same
order.  The exchanges belong to the LoadBalanceAllreduce's `ddp` backend, which
this package does not ship: with a group of one rank the hook returns the
compressed bucket, as the reference does when dp_group.size() == 1
(train.py:178); a larger group without a backend is an error.

Stream order: the reference switches to its side stream and completes the
future at once (train.py:165-181), leaving it to host time that the gradients
are written before the hook reads them and that the result is complete before
it is used.  Here the side stream first waits for the caller's current stream
(whatever produced the bucket there has finished before the path reads it), and
the caller's current stream waits for the side stream before the hook returns
(whatever consumes the future's tensor in that stream's order finds it
complete).  Neither wait blocks the host."""
import torch

from ._lib import annotate
from .compress import mask_below, threshold_with_allgather


class SparseCommHook:
    """custom_comm_hook(state, bucket) of train.py:167-183.

    load_balance_allreduce  the LoadBalanceAllreduce of the data-parallel group
    top_k                   args.top_k: per cent of the sample kept (train.py:176)
    method                  args.method: 1, 2 or 3 (comm.py:101-146)
    tp_group                the group whose ranks share a threshold (train.py:176)
    all_gather              callable(sample) -> samples of every rank of tp_group
                            (dist.all_gather_into_tensor in the reference,
                            train.py:63-64); needed only when tp_group has more
                            than one rank
    stream                  the side stream the path runs on (train.py:165);
                            default priority
    fused                   False: the reference's steps one by one (the bucket
                            is thresholded into a dense copy, the all-reduce
                            reads that copy); True (default): the threshold is
                            handed to the all-reduce, which selects while it
                            reads the bucket: same result, two passes over the
                            bucket fewer
    headroom                fused only: the buffers of the selection are sized for
                            top_k per cent of the bucket times this factor (the
                            sampled threshold lets a little more or less than
                            top_k per cent pass); if more pass, the call repeats
                            itself with more room
    The first call passes the bucket through untouched (train.py:170-174)."""

    def __init__(self, load_balance_allreduce, top_k, method, tp_group, all_gather=None, stream=None,
                 sample_index=None, fused=True, headroom=1.5):
        self.lba = load_balance_allreduce
        self.top_k = top_k
        self.method = method
        self.tp_group = tp_group
        self.all_gather = all_gather
        self.stream = stream if stream is not None else torch.cuda.Stream()
        self.sample_index = sample_index  # callable(numel) -> int64 sample positions; None: drawn like the reference
        self.fused = fused
        self.headroom = headroom
        self.skip = True

    def __call__(self, state, bucket):
        tensors = bucket.buffer()
        future = torch.futures.Future()
        if self.skip:
            future.set_result(tensors)
            self.skip = False
            return future
        exchange = self.lba.process_group.size() > 1
        if exchange and getattr(self.lba, "ddp", None) is None:
            raise RuntimeError("SparseCommHook: a group of more than one rank needs a communication backend in "
                               "load_balance_allreduce.ddp")
        caller = torch.cuda.current_stream(tensors.device)
        self.stream.wait_stream(caller)
        with torch.cuda.stream(self.stream):
            index = self.sample_index(tensors.numel()) if self.sample_index is not None else None
            with annotate("compress"):  # train.py:176 (the masked copy, if one is made, comes below)
                thr = threshold_with_allgather(self.top_k, tensors, self.tp_group, sample_index=index,
                                               all_gather=self.all_gather)
            if thr is None:  # a small bucket: not compressed (train.py:58-59)
                if exchange:
                    tensors = self.lba.zen_sparse_comm(tensors, self.method)
            elif exchange and self.fused:
                # about top_k per cent of the bucket pass the sampled threshold; the call grows its buffers if more do
                room = int(tensors.numel() * self.top_k / 100 * self.headroom) + 4096
                tensors = self.lba.zen_sparse_comm(tensors, self.method, thr=thr, capacity=min(room, tensors.numel()))
            else:
                tensors = mask_below(tensors.reshape(-1), thr).view_as(tensors)
                if exchange:
                    tensors = self.lba.zen_sparse_comm(tensors, self.method)
        caller.wait_stream(self.stream)
        # like the reference, the future is completed at once (train.py:181): its tensor is complete in the
        # order of the caller's stream and of `self.stream`
        future.set_result(tensors)
        return future
