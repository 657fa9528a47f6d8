#!/usr/bin/env python3
"""Benchmark of the sparse-gradient encode + decode path on one MI355X.

One step = exact top-k selection fused with the hash partition and slot-order
compaction of the rank's own gradient + merge of the P peer payloads addressed
to rank 0, all inputs resident in HBM.  Prints one JSON line: the step's dense-gradient
throughput, the roofline figures of the kernel that streams the gradient, the stage
times, the CPU baseline on the same workload and whether the HIP path reproduced it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c3] [--shrink S]
"""
import argparse
import ctypes
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by what the
# same counters read for a plain 1 GiB copy: the summaries under profiles/ that hold such figures, by
# (configuration, --shrink).  A summary names the kernel sources it was measured on (a digest of the library's
# source files); a figure measured on other sources is not reported.
TRAFFIC_PROFILES = {("c3", 1): "profiles/c3_select_stage_hbm_traffic.txt"}
HERE = os.path.dirname(os.path.abspath(__file__))


def kernel_sources_digest():
    """sha256 over the library's source files (names and contents, in name order)."""
    import glob
    import hashlib

    h = hashlib.sha256()
    files = sorted(glob.glob(os.path.join(HERE, "zen_repro_amd", "csrc", "*.hip")) +
                   glob.glob(os.path.join(HERE, "zen_repro_amd", "csrc", "*.h")) +
                   glob.glob(os.path.join(HERE, "include", "*.h")))
    for f in files:
        h.update(os.path.basename(f).encode() + b"\0")
        h.update(open(f, "rb").read())
    return h.hexdigest()


def measured_traffic(config, shrink, kernel):
    """(bytes per launch or None, where it comes from or why it is missing) for `kernel` on this workload: read
    from the summary's header lines '# kernel_sources_sha256: <digest>' and
    '# traffic_bytes_per_launch <kernel>: <bytes>'."""
    rel = TRAFFIC_PROFILES.get((config, shrink))
    if rel is None:
        return None, None
    try:
        text = open(os.path.join(HERE, rel)).read()
    except OSError:
        return None, f"{rel} is missing"
    digest = value = None
    for ln in text.splitlines():
        if ln.startswith("# kernel_sources_sha256:"):
            digest = ln.split(":", 1)[1].strip()
        elif ln.startswith(f"# traffic_bytes_per_launch {kernel}:"):
            value = float(ln.split(":", 1)[1].strip())
    if value is None or digest is None:
        return None, f"{rel} holds no figure for {kernel}"
    if digest != kernel_sources_digest():
        return None, f"{rel} was measured on other kernel sources (digest {digest[:12]}): not reported"
    return value, rel


def note(msg):
    """Progress line on stderr (a long CPU leg would otherwise look like a hang to whoever watches the run)."""
    print(f"[bench {time.strftime('%H:%M:%S')}] {msg}", file=sys.stderr, flush=True)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=40)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c3", choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--shrink", type=int, default=1, help="divide the workload size (debugging)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-div", type=int, default=1,
                    help="the CPU baseline runs on 1/div of the workload")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run five device copies of 1 GiB and exit (scale for hardware byte counters)")
    ap.add_argument("--bitmap-codec", action="store_true",
                    help="measure the bitmap index codec of the second exchange instead (prints its own line)")
    ap.add_argument("--phase2-decode", action="store_true",
                    help="measure the decode of the second exchange instead (prints its own line)")
    ap.add_argument("--separate-calls", action="store_true",
                    help="one library call for the encode and one for the merge instead of one per bucket for both "
                         "(zen_encode_merge); the kernels and streams are the same")
    ap.add_argument("--one-stream", action="store_true", help="run encode and merge back to back on one stream")
    ap.add_argument("--prepare-on", choices=["call", "main", "own"], default="call",
                    help="how the next step's sample is taken ahead: by the current step's pass over its tensor (no "
                         "kernel of its own), by a kernel on the step's stream right behind the step, or by one on a "
                         "stream of its own")
    ap.add_argument("--no-prepare", action="store_true",
                    help="do not take the next step's sample ahead on a stream of its own")
    ap.add_argument("--merge-beside", action="store_true",
                    help="with --depth 2 or more: a step's merge runs on a stream of its own beside its encode "
                         "(default there: on its encode's stream, after it; at --depth 1 it always runs beside)")
    ap.add_argument("--depth", type=int, default=1,
                    help="steps in flight in the timed region: 1 = a step starts when the previous one has finished "
                         "(its merge runs beside its encode on a second stream), so that a kernel's events time "
                         "that kernel; 2 or more: step i+1 is enqueued on its own stream next to step i, as a "
                         "training step hands over one gradient bucket after the other (the default run reports "
                         "that rate too, as two_steps_in_flight)")
    ap.add_argument("--rotate", type=int, default=16,
                    help="at most this many copies of the inputs, used in turn (as many as make 512 MB)")
    ap.add_argument("--near-threshold", action="store_true",
                    help="top-k steps are handed the threshold key the warm-up found for their bucket (in training: "
                         "the previous iteration's) and take no sample: one kernel less per bucket")
    ap.add_argument("--graph", action="store_true",
                    help="capture a step (encode, and the merge on its second stream) into a HIP graph per input copy "
                         "and time replays: what a caller gets who hands the library's calls to a graph, without "
                         "the host's share of every launch (matters for small buckets)")
    ap.add_argument("--imbalance", action="store_true", help="report the per-bucket load imbalance (always for c4)")
    ap.add_argument("--time-every", type=int, default=2,
                    help="in the timed region every n-th launch of the roofline kernel carries HIP events")
    ap.add_argument("--stage-steps", type=int, default=20,
                    help="steps of the untimed pass with every stage's events on (the stage table; it also tells "
                         "which kernel is the roofline kernel)")
    ap.add_argument("--no-reference-bucket", action="store_true",
                    help="leave out the sub-record for one bucket of a training run's size (c3 only)")
    ap.add_argument("--no-kernel-timing", action="store_true",
                    help="leave the HIP-event kernel timers off during the timed region")
    return ap.parse_args()


def cpu_pass(buckets, grads, payloads, threads):
    """The reference's torch-op sequence (insert: sequential C oracle) over every gradient bucket on this
    box's host cores: (seconds per stage summed over the buckets, per-bucket results)."""
    import torch

    from oracle import torch_path

    torch.set_num_threads(threads)
    total = {"select": 0.0, "partition": 0.0, "merge": 0.0}
    results = []
    for b, g, (idx_l, val_l) in zip(buckets, grads, payloads):
        note(f"CPU pass over {b.name}: {b.n} elements, {threads} thread(s)")
        times, res = torch_path.timed_pass(g, b.k, b.partitions, idx_l, val_l)
        for key, sec in times.items():
            total[key] += sec
        results.append(res)
    return total, results


def cpu_baseline(buckets, grads_dev, payloads_dev, outs, div):
    """CPU baseline on the whole workload (div == 1: the very tensors and payloads of the timed steps, and the
    last timed step's outputs are what is checked against it) or on the first 1/div of every bucket (then the
    HIP path repeats that sample, untimed, for the check).  A second pass on one host thread runs on a quarter
    of that, to keep the run short."""
    import torch

    from zen_repro_amd import workloads

    all_threads = torch.get_num_threads()
    if div == 1:
        subs = buckets
        grads = [g.cpu() for g in grads_dev]
        payloads = [([t.cpu() for t in idx_l], [t.cpu() for t in val_l]) for idx_l, val_l in payloads_dev]
        hip = outs
    else:
        subs, grads, payloads = [], [], []
        for b, g in zip(buckets, grads_dev):
            n_s = b.n // div // (16 * b.partitions) * (16 * b.partitions)
            sub = workloads.Config(b.name, n_s, b.dtype, b.partitions, b.peers, b.overlap, k=int(b.k * n_s / b.n) if b.k else 0)
            gs = g[:n_s].cpu()
            nnz_est = sub.k if sub.k else int(torch.count_nonzero(gs))
            idx_l, val_l, _, _ = workloads.peer_payloads(sub, workloads.per_peer_entries(sub, nnz_est), device=g.device, seed=1)
            subs.append(sub)
            grads.append(gs)
            payloads.append(([t.cpu() for t in idx_l], [t.cpu() for t in val_l]))
        hip = hip_pass(subs, [g[:s.n] for g, s in zip(grads_dev, subs)],
                       [([t.to(grads_dev[0].device) for t in i], [t.to(grads_dev[0].device) for t in v]) for i, v in payloads])
    times, results = cpu_pass(subs, grads, payloads, all_threads)
    note("checking the HIP outputs against the CPU pass")
    parity = parity_gate(subs, payloads, results, hip, "the last timed step's outputs" if div == 1 else
                         f"an untimed repeat on the first 1/{div} of every bucket")
    nbytes = sum(s.n * g.element_size() for s, g in zip(subs, grads))
    base = {
        "value": nbytes / sum(times.values()) / 1e9,
        "unit": "GB/s",
        "cores": all_threads,
        "kind": "port",
        "sample": f"{'the whole workload' if div == 1 else f'the first 1/{div} of every bucket'}: "
                  f"{sum(s.n for s in subs)} elements in {len(subs)} bucket(s); "
                  f"select {times['select']:.2f}s partition {times['partition']:.2f}s merge {times['merge']:.2f}s; "
                  f"torch ops use {all_threads} threads, the sequential insert 1",
    }
    # one host thread, on the first quarter of that sample
    q_subs, q_grads, q_pay = [], [], []
    for s_, g in zip(subs, grads):
        n_q = s_.n // 4 // (16 * s_.partitions) * (16 * s_.partitions)
        if n_q < 16 * s_.partitions:
            continue
        q = workloads.Config(s_.name, n_q, s_.dtype, s_.partitions, s_.peers, s_.overlap, k=int(s_.k * n_q / s_.n) if s_.k else 0)
        gq = g[:n_q]
        nnz_est = q.k if q.k else int(torch.count_nonzero(gq))
        idx_l, val_l, _, _ = workloads.peer_payloads(q, workloads.per_peer_entries(q, nnz_est), device="cpu", seed=1)
        q_subs.append(q)
        q_grads.append(gq)
        q_pay.append((idx_l, val_l))
    if q_subs:
        note("one host thread on a quarter of the sample")
        t1, _ = cpu_pass(q_subs, q_grads, q_pay, 1)
        base["value_1thread"] = sum(q.n * g.element_size() for q, g in zip(q_subs, q_grads)) / sum(t1.values()) / 1e9
        base["sample_1thread"] = f"the first quarter of that sample ({sum(q.n for q in q_subs)} elements), one host thread"
    torch.set_num_threads(all_threads)
    return parity, base


def hip_pass(buckets, grads, payloads):
    """One untimed pass of the HIP path: per bucket ((idx, val, splits, status), (m_idx, m_val, m_count, status))."""
    from zen_repro_amd import LoadBalanceAllreduce, LocalGroup, TensorPartition

    outs = []
    for b, g, (idx_l, val_l) in zip(buckets, grads, payloads):
        import torch

        capacity = int(b.k * 1.25) + 4096 if b.k else int(torch.count_nonzero(g)) + 16
        enc = TensorPartition(b.partitions, 1, 3).load_balance_flat(g, None, capacity, k=b.k)
        lba = LoadBalanceAllreduce(LocalGroup(b.partitions), None, None)
        flat_i, flat_v = torch.cat(idx_l), torch.cat(val_l)
        mrg = lba.merge_sparse_flat(flat_i, flat_v, b.n, capacity=flat_i.numel())
        outs.append((enc, mrg))
    return outs


def parity_gate(buckets, payloads, cpu_results, hip_outs, what):
    """The HIP path's outputs against the CPU pass on the same inputs: split sizes, the buckets' indices in
    their order and their values bit for bit; the merged indices and fp32 sums bit for bit against a sequential
    fp32 scatter_add_ on the CPU (the baseline itself accumulates in the values' own type, as the reference
    does)."""
    import torch

    encode_ok = merge_ok = True
    selected = merged = 0
    for b, (idx_l, val_l), (c_idx, c_val, c_splits, _, _, _), (enc, mrg) in zip(buckets, payloads, cpu_results, hip_outs):
        g_idx, g_val, g_splits, _ = enc
        count = int(g_splits.sum())
        bits = torch.int16 if g_val.dtype == torch.bfloat16 else torch.int32
        encode_ok = (encode_ok and torch.equal(g_splits.cpu(), c_splits.to(torch.int64))
                     and torch.equal(g_idx[:count].cpu(), torch.cat(c_idx).to(torch.int32))
                     and torch.equal(g_val[:count].cpu().view(bits), torch.cat(c_val).view(bits)))
        m_idx, m_val, m_count, _ = mrg
        u = int(m_count)
        dense = torch.zeros(b.n, dtype=torch.float32)
        dense.scatter_add_(0, torch.cat(idx_l).to(torch.int64), torch.cat(val_l).to(torch.float32))
        want_idx = torch.nonzero(dense, as_tuple=True)[0]
        merge_ok = (merge_ok and u == want_idx.numel() and torch.equal(m_idx[:u].cpu().to(torch.int64), want_idx)
                    and torch.equal(m_val[:u].cpu().view(torch.int32), dense[want_idx].view(torch.int32)))
        selected += count
        merged += u
        del dense
    return {"ok": bool(encode_ok and merge_ok), "encode_bit_exact": bool(encode_ok), "merge_bit_exact": bool(merge_ok),
            "checked": f"{what}: {selected} selected entries, {merged} merged entries"}


def bitmap_codec(args, dev):
    """Rank 0's merged indices -> bitmap over its partition's member list -> indices again (comm.py:59-99):
    one step = one encode_bitmap and one decode_bitmap of that bitmap, no host synchronisation in between.
    Algorithmic bytes: the indices in (8 B each), the bitmap out and in again (members / 8 B each way), the
    indices out (8 B each)."""
    import torch

    from zen_repro_amd import LoadBalanceAllreduce, LocalGroup, _lib, workloads

    cfg, grad = workloads.make(args.config, device=dev, seed=0, shrink=args.shrink)
    del grad
    n, P = cfg.n, cfg.partitions
    lba = LoadBalanceAllreduce(LocalGroup(P, 0), None, None)
    lba.mapping[n] = lba.calculate_mapping(n)
    members = lba.mapping[n][0]
    _, _, flat_idx, flat_val = workloads.peer_payloads(cfg, max(1, (cfg.k or n // 100) // P), device=dev, seed=1)
    m_idx, _ = lba.merge_sparse(flat_idx, flat_val, n)
    L = _lib.lib()
    out = torch.empty(m_idx.numel(), dtype=torch.int64, device=dev)
    count = torch.zeros(1, dtype=torch.int64, device=dev)
    ws = torch.empty(max(256, L.zen_bitmap_decode_workspace(members.numel())), dtype=torch.uint8, device=dev)
    status = _lib.status_word(dev)

    def step():
        bitmap, st = lba.encode_bitmap_flat(m_idx, n)
        _lib.check(L.zen_bitmap_decode(_lib.ptr(members), members.numel(), _lib.ptr(bitmap), bitmap.numel(),
                                       _lib.ptr(out), out.numel(), _lib.ptr(count), _lib.ptr(ws), ws.numel(),
                                       _lib.ptr(status), _lib.stream_of(dev)), "decode_bitmap")
        return st

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    flags = [step() for _ in range(args.steps)]
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    bits = int(status.item())
    for st in flags:
        bits |= int(st.item())
    if bits or int(count.item()) != m_idx.numel() or not torch.equal(out, m_idx):
        print("bench.py: the bitmap round trip did not return the indices", file=sys.stderr)
        sys.exit(1)
    u, nbytes = m_idx.numel(), (members.numel() + 7) // 8
    b_alg = 16 * u + 2 * nbytes
    print(json.dumps({
        "metric": "bitmap index codec, encode + decode of one rank's merged indices", "value": round(u / ms / 1e3, 2),
        "unit": "M indices/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "dtype": "int64", "data": "synthetic",
        "config": {"workload": f"{cfg.name}: {cfg.note}", "elements": n, "partitions": P, "indices": u,
                   "members": members.numel(), "bitmap_bytes": nbytes},
        "algorithmic_bytes": b_alg, "algorithmic_GBps": round(b_alg / (ms * 1e-3) / 1e9, 2)}))


def phase2_decode(args, dev):
    """The second exchange's decode (comm.py:136-145): P pairwise disjoint shards of merged entries (rank p's
    shard holds indices of hash partition p, as many as rank 0 merges in the main benchmark) into the dense
    gradient.  Three ways, each checked against a plain assignment (the shards are disjoint): from the ranks'
    bitmaps and value lists in one pass (decode_bitmaps_dense; the headline figure); from the bitmaps as the
    reference does it, decode_bitmap for every rank and then decode_sparse_tensors; and from index lists
    (method 2's exchange, decode_sparse_tensors(ascending=True))."""
    import torch

    from zen_repro_amd import LoadBalanceAllreduce, LocalGroup, workloads

    cfg, grad = workloads.make(args.config, device=dev, seed=0, shrink=args.shrink)
    dtype = grad.dtype
    del grad
    n, P = cfg.n, cfg.partitions
    lba = LoadBalanceAllreduce(LocalGroup(P, 0), None, None)
    part = torch.empty(n, dtype=torch.int32, device=dev)
    from zen_repro_amd.functions import hash_index
    hash_index(part, P)
    per = max(1, int((cfg.k or n // 100) * 0.766))  # what a rank keeps after merging P payloads that overlap by a quarter
    gen = torch.Generator(device=dev).manual_seed(2)
    weights = torch.tensor([1, 2, 4, 8, 16, 32, 64, 128], dtype=torch.uint8, device=dev)
    idx, val, bitmaps, members_of = [], [], [], []
    for p in range(P):
        members = torch.nonzero(part == p, as_tuple=True)[0]
        pick = torch.randperm(members.numel(), device=dev, generator=gen)[:per].sort().values
        idx.append(members[pick].contiguous())
        val.append((torch.randn(per, device=dev, generator=gen) * 1e-3).to(dtype))
        bits = torch.zeros((members.numel() + 7) // 8 * 8, dtype=torch.uint8, device=dev)
        bits[pick] = 1
        bitmaps.append((bits.view(-1, 8) * weights).sum(1, dtype=torch.uint8))  # comm.py:79-83
        members_of.append(members)
        del pick, bits
    del part
    flat_i, flat_v = torch.cat(idx), torch.cat(val)
    sizes = [t.numel() for t in idx]
    views = list(torch.split(flat_i, sizes)), list(torch.split(flat_v, sizes))  # what an all-gather into one buffer leaves
    flat_b = torch.cat(bitmaps)
    bviews = list(torch.split(flat_b, [t.numel() for t in bitmaps]))
    want = torch.zeros(n, dtype=dtype, device=dev)
    want[flat_i] = flat_v
    bits_t = torch.int16 if dtype == torch.bfloat16 else torch.int32

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            dense = fn()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        if not torch.equal(dense.view(bits_t), want.view(bits_t)):
            print("bench.py: the decoded dense tensor is not the shards' assignment", file=sys.stderr)
            sys.exit(1)
        return ms

    ms_fused = timed(lambda: lba.decode_bitmaps_dense(bviews, views[1], n))
    ms_lists = timed(lambda: lba.decode_sparse_tensors(views[0], views[1], n, ascending=True))
    lba.mapping[n] = members_of  # what calculate_mapping returns (comm.py:52-56)
    ms_two = timed(lambda: lba.decode_sparse_tensors(lba.decode_bitmap(bviews, n), views[1], n, ascending=True))
    r, s_ = flat_i.numel(), flat_v.element_size()
    b_alg = flat_b.numel() + r * s_ + n * s_  # the bitmaps and the values in, the dense tensor out
    print(json.dumps({
        "metric": "phase-2 decode: all ranks' bitmaps and values into the dense gradient, one pass",
        "value": round(b_alg / (ms_fused * 1e-3) / 1e9, 2),
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_fused, 4),
        "higher_is_better": True, "dtype": "bf16" if dtype == torch.bfloat16 else "f32", "data": "synthetic",
        "config": {"workload": f"{cfg.name}: {cfg.note}", "elements": n, "shards": P, "entries": r,
                   "bitmap_bytes": flat_b.numel()},
        "algorithmic_bytes": b_alg,
        "frac_of_hbm_peak": round(b_alg / (ms_fused * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "ms_per_step_two_steps_from_bitmaps": round(ms_two, 4),
        "ms_per_step_from_index_lists": round(ms_lists, 4)}))


def reference_bucket(dev, steps, warmup):
    """The step on ONE gradient bucket of the size a training run hands over (the c3 tensor cut in twelve:
    61,953,360 bf16 elements, the 0.5 % largest kept, P = 16): one call of the library per step, the next step's
    sample taken ahead, the merge beside the encode; then the same with two steps in flight."""
    import torch

    from zen_repro_amd import LoadBalanceAllreduce, LocalGroup, TensorPartition, _lib, workloads

    cfg, grad = workloads.make("c3", device=dev, seed=0, shrink=12)
    b = workloads.buckets(cfg)[0]
    esize, P = grad.element_size(), cfg.partitions
    cap = int(b.k * 1.25) + 4096
    _, _, fi, fv = workloads.peer_payloads(b, workloads.per_peer_entries(b, b.k), device=dev, seed=1)
    copies = max(1, -(-(512 << 20) // (b.n * esize)))  # more bytes than the last-level cache holds
    grads = [grad] + [grad.clone() for _ in range(copies - 1)]
    tp = TensorPartition(P, 1, 3)
    lba = LoadBalanceAllreduce(LocalGroup(P), None, None)
    main = torch.cuda.current_stream(dev)
    second, beside = (torch.cuda.Stream(device=dev) for _ in range(2))

    def run(count, depth, marks=None):
        outs = []
        for s_ in (second, beside):
            s_.wait_stream(main)
        for i in range(count):
            es = second if (depth == 2 and i % 2) else main

            def call():
                outs.append(lba.encode_merge_flat(tp, grads[i % copies], cap, b.k, fi, fv, b.n, slot=i % depth,
                                                  merge_stream=beside if depth == 1 else None,
                                                  next_tensor=grads[(i + 1) % copies] if depth == 1 and i + 1 < count
                                                  else None))

            if es is main:
                call()
            else:
                with torch.cuda.stream(es):
                    call()
            if marks is not None and i % (2 * depth) == 2 * depth - 1:
                pair = [torch.cuda.Event(enable_timing=True)]
                pair[0].record(es)
                if depth == 1:
                    pair.append(torch.cuda.Event(enable_timing=True))
                    pair[1].record(beside)
                marks.append(pair)
        for s_ in (second, beside):
            main.wait_stream(s_)
        return outs

    rec = {"elements": b.n, "k": b.k, "partitions": P, "dtype": "bf16"}
    for depth in (1, 2):
        run(max(1, warmup), depth)
        torch.cuda.synchronize()
        _lib.profile_enable(True)
        run(4, depth)
        torch.cuda.synchronize()
        launches = sum(v[1] for v in _lib.profile_read().values()) // 4
        _lib.profile_enable(False)
        t0 = time.perf_counter()
        outs = run(steps, depth)
        t_enq = time.perf_counter()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        marks = []
        ref = torch.cuda.Event(enable_timing=True)
        ref.record(main)
        run(2 * depth * 22, depth, marks)
        torch.cuda.synchronize()
        ends = [max(ref.elapsed_time(e) for e in pair) for pair in marks]
        per = sorted((ends[i + 1] - ends[i]) / (2 * depth) for i in range(len(ends) - 1))
        call_us = None
        if depth == 1:
            # what the one call of the library costs the host: the last step's call again, a hundred times, timed
            # until the last one returns (nothing waits for the device; the results are the same every time)
            a = lba.last_encode_merge_args
            L = _lib.lib()
            t2 = time.perf_counter()
            for _ in range(100):
                L.zen_encode_merge(ctypes.byref(a))
            call_us = (time.perf_counter() - t2) * 1e4
            torch.cuda.synchronize()
        (_, _, splits, st), (_, _, count, mst) = outs[-1]
        if int(st) | int(mst):
            print("bench.py: reference bucket: device status " + _lib.describe_status(int(st) | int(mst)), file=sys.stderr)
            sys.exit(1)
        b_alg = workloads.algorithmic_bytes(b.n, esize, int(splits.sum()), fi.numel(), int(count))
        rec["one_step_at_a_time" if depth == 1 else "two_steps_in_flight"] = {
            "ms_per_step": round(ms, 4), "ms_per_step_device_median": round(per[len(per) // 2], 4),
            "value": round(b.n * esize / (ms * 1e-3) / 1e9, 2), "unit": "GB/s",
            "path_frac_of_hbm_peak": round(b_alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "host_enqueue_ms_per_step": round((t_enq - t0) * 1e3 / steps, 4), "kernel_launches_per_step": launches}
        if call_us is not None:
            rec["library_call_host_ms"] = round(call_us / 1e3, 4)
    rec["selected"], rec["received"], rec["merged"] = int(splits.sum()), fi.numel(), int(count)
    return rec


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share of the path; --gpus must be 1 "
              "(the exchange between ranks is not part of it)", file=sys.stderr)
        sys.exit(2)

    import torch

    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from zen_repro_amd import LoadBalanceAllreduce, LocalGroup, TensorPartition, _lib, topk_threshold, workloads

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    _lib.lib()

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"bytes_read": src.numel() * 4, "bytes_written": src.numel() * 4,
                                               "copies": 5}}))
        return

    if args.bitmap_codec:
        bitmap_codec(args, dev)
        return
    if args.phase2_decode:
        phase2_decode(args, dev)
        return

    note(f"synthesising {args.config}")
    cfg, grad = workloads.make(args.config, device=dev, seed=0, shrink=args.shrink)
    esize, P = grad.element_size(), cfg.partitions
    buckets = workloads.buckets(cfg)  # the gradient buckets the tensor is handed over in (c2: two; else one)
    tp = TensorPartition(P, 1, 3)
    lba = LoadBalanceAllreduce(LocalGroup(P), None, None)

    # Per bucket: its stretch of the gradient, the capacity of its selection and the payloads the P peers send
    # to rank 0, generated on the device (the CPU baseline gets copies of these very tensors).
    grads, caps, payloads, flats = [], [], [], []
    for b in buckets:
        g = grad[b.offset:b.offset + b.n]
        nnz_guess = b.k if b.k else int(torch.count_nonzero(g))
        caps.append(int(b.k * 1.25) + 4096 if b.k else nnz_guess + 16)  # room for ties at the threshold
        idx_l, val_l, flat_idx, flat_val = workloads.peer_payloads(b, workloads.per_peer_entries(b, nnz_guess), device=dev, seed=1)
        grads.append(g)
        payloads.append((idx_l, val_l))
        flats.append((flat_idx, flat_val))
    received = sum(fi.numel() for fi, _ in flats)
    total_bytes = sum(b.n for b in buckets) * esize

    # Inputs rotate between copies at different addresses so that nothing of a step's input is still in the
    # 256 MB last-level cache when the next step reads it (the copies hold the same values: one check serves).
    def copies_of(nbytes):
        return max(1, min(args.rotate, -(-(512 << 20) // max(1, nbytes))))
    grad_sets = [[g] + [g.clone() for _ in range(copies_of(total_bytes) - 1)] for g in grads]
    pay_bytes = sum(fi.numel() * (4 + esize) for fi, _ in flats)
    flat_sets = [[(fi, fv)] + [(fi.clone(), fv.clone()) for _ in range(copies_of(pay_bytes) - 1)] for fi, fv in flats]

    # By default a step starts when the one before has finished, and its merge, which does not depend on its
    # encode, runs beside it on a second stream.  A training step hands over one gradient bucket after the
    # other (train.py:167-185 is called per bucket), and nothing in bucket i+1 depends on bucket i: with
    # --depth 2 two consecutive steps are in flight, alternating between two streams, workspaces and tables
    # ("slots"), each step's merge behind its encode on the step's own stream, so that the long, memory-bound
    # select of one step runs next to the short, latency-bound kernels of the other (a kernel's events then
    # also time its wait for room on the chip).  All streams have default priority.
    fused = not (args.separate_calls or args.graph)
    depth = 1 if (args.one_stream or args.graph) else max(1, args.depth)
    main = torch.cuda.current_stream(dev)
    enc_streams = [main] + [torch.cuda.Stream(device=dev) for _ in range(depth - 1)]
    merge_follows = depth > 1 and not args.merge_beside
    mrg_streams = [None if (args.one_stream or merge_follows) else torch.cuda.Stream(device=dev)
                   for _ in range(depth)]

    # The sample that gives a top-k call its floor only needs the tensor: the next step's is taken ahead on a
    # stream of its own, beside the current step's sort and placement, instead of in front of the next pass
    # over the tensor (a hook that is called per bucket can do the same as soon as it holds the next bucket).
    prep_stream = (None if (args.one_stream or args.no_prepare or args.graph or args.near_threshold)
                   else torch.cuda.Stream(device=dev))

    warm_thr = [torch.zeros(2, dtype=torch.int32, device=dev) for _ in buckets]
    near_keys = [None for _ in buckets]
    warm = False

    def step(i, more=True, es=None):
        slot = i % depth
        ms_ = mrg_streams[slot]
        if es is None:
            es = enc_streams[slot]
        enc, mrg = [], []

        def encode():
            for j, b in enumerate(buckets):
                g = grad_sets[j][i % len(grad_sets[j])]
                enc.append(tp.load_balance_flat(g, None, caps[j], k=b.k, slot=slot, thr_out=warm_thr[j] if warm else None,
                                                near=near_keys[j]))

        def merge():
            for j, b in enumerate(buckets):
                fi, fv = flat_sets[j][i % len(flat_sets[j])]
                mrg.append(lba.merge_sparse_flat(fi, fv, b.n, capacity=fi.numel(), slot=slot))

        def both():
            along = prep_stream is not None and more and depth == 1 and args.prepare_on == "call"
            for j, b in enumerate(buckets):
                g = grad_sets[j][i % len(grad_sets[j])]
                fi, fv = flat_sets[j][i % len(flat_sets[j])]
                # the bucket that follows this one on the slot: the next bucket of the step, or the next step's first
                nj, ni = (j + 1, i) if j + 1 < len(buckets) else (0, i + 1)
                e_, m_ = lba.encode_merge_flat(tp, g, caps[j], b.k, fi, fv, b.n, slot=slot,
                                               thr_out=warm_thr[j] if warm else None, near=near_keys[j],
                                               merge_stream=ms_,
                                               next_tensor=grad_sets[nj][ni % len(grad_sets[nj])] if along else None,
                                               next_k=buckets[nj].k, next_capacity=caps[nj])
                enc.append(e_)
                mrg.append(m_)

        def on_stream():
            if fused:
                both()
            else:
                encode()
                if ms_ is None:
                    merge()  # behind the encode, on its stream

        if es is main:
            on_stream()  # already the current stream: entering it again costs the host 10 us a step
        else:
            with torch.cuda.stream(es):
                on_stream()
        if prep_stream is not None and more and depth == 1 and not (fused and args.prepare_on == "call"):
            with torch.cuda.stream(prep_stream if args.prepare_on == "own" else es):
                for j, b in enumerate(buckets):
                    tp.prepare(grad_sets[j][(i + 1) % len(grad_sets[j])], b.k, caps[j], slot=slot)
        if ms_ is not None and not fused:
            with torch.cuda.stream(ms_):
                merge()
        return list(zip(enc, mrg))

    side = enc_streams[1:] + [m for m in mrg_streams if m is not None] + ([prep_stream] if prep_stream is not None else [])

    def run(count, marks=None):
        outs = []
        for s_ in side:
            s_.wait_stream(main)  # the inputs were produced on the main stream
        for i in range(count):
            outs.append(step(i, more=i + 1 < count))
            if marks is not None and i % (2 * depth) == 2 * depth - 1:
                # where the step's streams stand once the step is enqueued (the later of the two is the step's
                # end); behind every second step per stream only: an event between two kernels of a stream holds
                # the second one up for microseconds
                pair = [torch.cuda.Event(enable_timing=True)]
                pair[0].record(enc_streams[i % depth])
                if mrg_streams[i % depth] is not None:
                    pair.append(torch.cuda.Event(enable_timing=True))
                    pair[1].record(mrg_streams[i % depth])
                marks.append(pair)
        for s_ in side:
            main.wait_stream(s_)
        return outs

    note("warm-up")
    warm = True
    run(max(1, args.warmup))
    torch.cuda.synchronize()
    warm = False
    if args.near_threshold:
        near_keys = [warm_thr[j].clone() if b.k else None for j, b in enumerate(buckets)]
    note("timing")

    # what a read-only pass over the gradient reaches on this box (plain non-temporal streaming loads)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    ceiling = None
    if total_bytes >= 1 << 26:
        L = _lib.lib()
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(11)]
        for r in range(10):
            evs[r].record()
            for gs in grad_sets:
                g = gs[r % len(gs)]
                _lib.check(L.zen_stream_read(_lib.ptr(g), g.numel() * esize, _lib.ptr(sink), _lib.stream_of(dev)), "stream_read")
        evs[10].record()
        torch.cuda.synchronize()
        per = sorted(evs[r].elapsed_time(evs[r + 1]) for r in range(10))
        ceiling = total_bytes / (per[len(per) // 2] * 1e-3) / 1e9

    # An event between two kernels costs the device a few microseconds, about 40 of them per step with every
    # stage timed.  So the stage breakdown comes from an untimed pass of its own, and in the timed region only
    # the dominant kernel (the one the roofline figure is about) carries events, on every --time-every-th of
    # its launches (the pair of events around one launch holds the stream up for 10 us or so).
    streaming = ("k_select_stage", "k_select_compact", "k_topk_hist")  # kernels that read the dense gradient
    stages, dom = {}, None
    every = 1 if len(buckets) > 1 else max(1, args.time_every)  # several buckets: every launch, or one bucket's only
    if not args.no_kernel_timing:
        _lib.profile_enable(True)
        stage_steps = max(1, args.stage_steps)
        run(stage_steps)
        torch.cuda.synchronize()
        stages = _lib.profile_read()
        cands = [(stages[name][0], name) for name in streaming if name in stages]
        dom = max(cands)[1] if cands else None
        _lib.profile_enable(dom is not None, only=dom, every=every)
    if args.graph:
        # one graph per combination of input copies; a replay is the whole step: the encode on the graph's
        # stream, the merge forked onto the second stream and joined again
        _lib.profile_enable(False)
        lens = [len(gs) for gs in grad_sets] + [len(fs) for fs in flat_sets]
        rounds = max(lens)  # graph r reads copy r % len of every input
        cap = torch.cuda.Stream(device=dev)
        graphs, graph_outs = [], []
        for r in range(rounds):
            g_ = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g_, stream=cap):
                cur = torch.cuda.current_stream(dev)
                _lib.zeros.fresh(dev)  # this graph's status words and counts: a block of its own, zeroed by the graph
                if mrg_streams[0] is not None:
                    mrg_streams[0].wait_stream(cur)
                    with torch.cuda.stream(mrg_streams[0]):
                        _lib.zeros.fresh(dev)
                graph_outs.append(step(r, more=False, es=cur))
                if mrg_streams[0] is not None:
                    cur.wait_stream(mrg_streams[0])
            graphs.append(g_)
        _lib.zeros.fresh(dev)
        with torch.cuda.stream(cap):
            _lib.zeros.fresh(dev)
        if mrg_streams[0] is not None:
            with torch.cuda.stream(mrg_streams[0]):
                _lib.zeros.fresh(dev)  # later eager calls must not take pieces of a graph's block
        for r in range(min(rounds, args.warmup)):
            graphs[r].replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            graphs[i % rounds].replay()
        t_enq = time.perf_counter()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        outs = [graph_outs[(args.steps - 1 - j) % rounds] for j in range(min(rounds, args.steps))][::-1]  # last: the last replay's
        kernels = {dom: stages[dom]} if dom else {}  # the roofline kernel's duration: from the pass with events above
    else:
        t0 = time.perf_counter()
        outs = run(args.steps)
        t_enq = time.perf_counter()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        kernels = _lib.profile_read() if dom else {}
        _lib.profile_enable(False)

    # The same steps once more with an event behind each: the median of the per-step device times does not move
    # with a slow first step or a hiccup of the host as the mean above does.
    device_ms = None
    if not args.graph:
        marks = []
        ref = torch.cuda.Event(enable_timing=True)
        ref.record(main)
        run(2 * depth * 22, marks)
        torch.cuda.synchronize()
        ends = [max(ref.elapsed_time(e) for e in pair) for pair in marks]
        per = sorted((ends[i + 1] - ends[i]) / (2 * depth) for i in range(len(ends) - 1))
        device_ms = {"median": round(per[len(per) // 2], 4), "min": round(per[0], 4), "max": round(per[-1], 4),
                     "samples": len(per), "steps_per_sample": 2 * depth,
                     "what": "device time per step between events recorded behind every second step on the step's "
                             "streams (the later one counts), back to back, in an untimed pass of its own"}

    last = outs[-1]
    nnz = [int(enc[2].sum()) for enc, _ in last]
    merged = [int(mrg[2]) for _, mrg in last]
    flags = 0
    for o in outs:  # every step of the timed region must have gone through cleanly and agree
        for j, (enc, mrg) in enumerate(o):
            flags |= int(enc[3]) | int(mrg[3])
            if int(enc[2].sum()) != nnz[j] or int(mrg[2]) != merged[j]:
                print(f"bench.py: steps disagree on their result sizes (bucket {j}: selected {int(enc[2].sum())} vs "
                      f"{nnz[j]}, merged {int(mrg[2])} vs {merged[j]}, status {int(enc[3])} / {int(mrg[3])})", file=sys.stderr)
                sys.exit(1)
    if flags:
        print("bench.py: device status " + _lib.describe_status(flags), file=sys.stderr)
        sys.exit(1)

    ms = (t1 - t0) * 1e3 / args.steps
    value = total_bytes / (ms * 1e-3) / 1e9
    b_alg = sum(workloads.algorithmic_bytes(b.n, esize, nnz[j], flats[j][0].numel(), merged[j]) for j, b in enumerate(buckets))

    # isolated steps (a step starts when the one before has finished), each bracketed by events: the median
    # tells how a single bucket's latency compares with the pipelined rate above
    lat = []
    for i in range(min(args.steps, 20)):
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for s_ in side:
            s_.wait_stream(main)
        step(i, more=False)
        for s_ in side:
            main.wait_stream(s_)
        e1.record()
        torch.cuda.synchronize()
        lat.append(e0.elapsed_time(e1))
    lat.sort()

    # the rate with two steps in flight (see --depth), when the timed region above ran one at a time
    two = None
    if depth == 1 and not args.one_stream and not args.graph:
        torch.cuda.synchronize()
        second = torch.cuda.Stream(device=dev)

        def pipelined(count):
            second.wait_stream(main)
            for i in range(count):
                with torch.cuda.stream(second if i % 2 else main):
                    if fused:
                        for j, b in enumerate(buckets):
                            fi, fv = flat_sets[j][i % len(flat_sets[j])]
                            lba.encode_merge_flat(tp, grad_sets[j][i % len(grad_sets[j])], caps[j], b.k, fi, fv, b.n,
                                                  slot=i % 2, near=near_keys[j])
                        continue
                    for j, b in enumerate(buckets):
                        tp.load_balance_flat(grad_sets[j][i % len(grad_sets[j])], None, caps[j], k=b.k, slot=i % 2,
                                             near=near_keys[j])
                    for j, b in enumerate(buckets):
                        fi, fv = flat_sets[j][i % len(flat_sets[j])]
                        lba.merge_sparse_flat(fi, fv, b.n, capacity=fi.numel(), slot=i % 2)
            main.wait_stream(second)

        pipelined(4)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        pipelined(args.steps)
        torch.cuda.synchronize()
        ms2 = (time.perf_counter() - t2) * 1e3 / args.steps
        two = {"ms_per_step": round(ms2, 4), "value": round(total_bytes / (ms2 * 1e-3) / 1e9, 2), "unit": "GB/s",
               "path_frac_of_hbm_peak": round(b_alg / (ms2 * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
               "what": "the same steps with two in flight on two streams, a step's merge behind its encode (--depth 2)"}

    # the roofline kernel with the chip to itself: the encodes alone on the main stream (no merge beside them,
    # nothing left over from a step before), events around every launch of that kernel
    alone = None
    if dom and not args.graph:
        torch.cuda.synchronize()
        _lib.profile_enable(True, only=dom, every=1)
        for i in range(12):
            for j, b in enumerate(buckets):
                tp.load_balance_flat(grad_sets[j][i % len(grad_sets[j])], None, caps[j], k=b.k, slot=0, near=near_keys[j])
        torch.cuda.synchronize()
        alone = _lib.profile_read().get(dom)
        _lib.profile_enable(False)

    # dominant kernel: the one with the largest summed duration among the
    # kernels that stream the dense gradient; its algorithmic bytes per launch
    # (several buckets: the mean over the buckets' launches, all of which are timed)
    sel_bytes = sum(b.n * esize + nnz[j] * (4 + esize) for j, b in enumerate(buckets)) / len(buckets)
    per_launch = {"k_select_stage": sel_bytes, "k_select_compact": sel_bytes, "k_topk_hist": total_bytes / len(buckets)}
    roofline = None
    stage_ms = {name: round(total / stage_steps, 4) for name, (total, _) in stages.items()} if stages else {}
    if dom in kernels:
        total_ms, launches = kernels[dom]
        avg_ms = total_ms / launches
        achieved = per_launch[dom] / (avg_ms * 1e-3) / 1e9
        traffic = measured_traffic(cfg.name, args.shrink, dom)
        roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                    "traffic": traffic[0], "traffic_source": traffic[1],
                    "avg_launch_ms": round(avg_ms, 4), "launches_per_step": stages[dom][1] // stage_steps,
                    "timed_launches": launches,
                    "algorithmic_bytes_per_launch": int(per_launch[dom]),
                    "measured_read_ceiling_GBps": round(ceiling, 1) if ceiling else None,
                    "frac_of_read_ceiling": round(achieved / ceiling, 4) if ceiling else None}
        if alone:
            a_ms = alone[0] / alone[1]
            a_rate = per_launch[dom] / (a_ms * 1e-3) / 1e9
            roofline["alone"] = {"avg_launch_ms": round(a_ms, 4), "achieved": round(a_rate, 1),
                                 "frac": round(a_rate / HBM_PEAK_GBS, 4),
                                 "frac_of_read_ceiling": round(a_rate / ceiling, 4) if ceiling else None,
                                 "launches": alone[1],
                                 "what": "the same kernel with the chip to itself (encodes alone on one stream, untimed "
                                         "pass): in a step its launches wait for compute units the merge before them "
                                         "still holds and share the memory system with the merge's scatter"}

    if roofline and args.graph:
        roofline["timed_in"] = "the untimed pass with every stage's events on (graph replays carry no events)"
    line = {
        "metric": "encode+decode dense-gradient GB/s on 1 GPU; % of HBM roofline",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if grad.dtype == torch.bfloat16 else "f32",
        "data": "synthetic",
        "config": {"workload": f"{cfg.name}: {cfg.note}", "elements": cfg.n, "partitions": P,
                   "buckets": [{"name": b.name, "elements": b.n, "k": b.k, "selected": nnz[j],
                                "received": flats[j][0].numel(), "merged": merged[j]} for j, b in enumerate(buckets)],
                   "k": sum(b.k for b in buckets), "selected": sum(nnz), "received": received, "merged": sum(merged),
                   "peers": cfg.peers, "overlap": cfg.overlap, "shrink": args.shrink, "steps_in_flight": depth, "calls_per_bucket": 1 if fused else 2,
                   "merge_runs": "behind its step's encode" if (merge_follows or args.one_stream) else "beside its step's encode",
                   "replayed_from_graph": bool(args.graph),
                   "topk_sample": "none: the warm-up's threshold key is handed over" if args.near_threshold else "taken in every step",
                   "input_copies": {"gradient": len(grad_sets[0]), "payloads": len(flat_sets[0])}},
        "path_algorithmic_GBps": round(b_alg / (ms * 1e-3) / 1e9, 2),
        "path_frac_of_hbm_peak": round(b_alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "ms_per_step_device_median": device_ms["median"] if device_ms else None,
        "path_frac_of_hbm_peak_at_median": (round(b_alg / (device_ms["median"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
                                            if device_ms else None),
        "per_step_device_ms": device_ms,
        "ms_per_step_isolated_median": round(lat[len(lat) // 2], 4),
        "two_steps_in_flight": two,
        "host_enqueue_ms_per_step": round((t_enq - t0) * 1e3 / args.steps, 4),
        "stage_ms_per_step": stage_ms,
        "stage_ms_note": "from an untimed pass with every stage's events on; the timed region times only the "
                         "roofline kernel",
        "roofline": roofline,
        "cpu_baseline": None,
    }
    if cfg.name == "c3" and args.shrink == 1 and not (args.no_reference_bucket or args.graph or args.one_stream):
        note("one bucket of a training run's size")
        line["reference_bucket"] = reference_bucket(dev, args.steps, args.warmup)
    if cfg.name == "c4" or args.imbalance:
        # per-bucket load, max / mean, of the hash partition (the split sizes) and of a plain range partition of
        # the same indices (utils.py:66-88 is the reference's notion of skew)
        enc = last[0][0]
        count = nnz[0]
        by_hash = enc[2].double()
        by_range = torch.bincount(enc[0][:count].to(torch.int64) // -(-buckets[0].n // P), minlength=P).double()
        line["bucket_imbalance"] = {"hash": round((by_hash.max() / by_hash.mean()).item(), 4),
                                    "range": round((by_range.max() / by_range.mean()).item(), 4),
                                    "what": "largest bucket / mean bucket over the P destinations"}
    if not args.no_cpu_baseline:
        note(f"GPU part done: {ms:.4f} ms per step; CPU baseline next")
        line["parity_vs_cpu_baseline"], line["cpu_baseline"] = cpu_baseline(
            buckets, [gs[(args.steps - 1) % len(gs)] for gs in grad_sets],
            [(list(torch.split(fs[(args.steps - 1) % len(fs)][0], [t.numel() for t in payloads[j][0]])),
              list(torch.split(fs[(args.steps - 1) % len(fs)][1], [t.numel() for t in payloads[j][1]])))
             for j, fs in enumerate(flat_sets)], last, args.cpu_sample_div)
    print(json.dumps(line))
    if line.get("parity_vs_cpu_baseline") and not line["parity_vs_cpu_baseline"]["ok"]:
        print("bench.py: the HIP path and the CPU baseline disagree", file=sys.stderr)
        sys.exit(1)


if __name__ == "__main__":
    main()
