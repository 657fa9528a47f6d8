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
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# HBM bytes per launch of the dominant kernel on the full c3 workload, from
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by what the same counters read
# for a plain 1 GiB copy (profiles/c3_select_stage_hbm_traffic.txt).  Other
# workloads report null.
MEASURED_TRAFFIC = {("c3", 1, "k_select_stage"): 1.519e9}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
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
    ap.add_argument("--one-stream", action="store_true", help="run encode and merge back to back on one stream")
    ap.add_argument("--merge-follows", action="store_true",
                    help="with --depth: a step's merge runs on its encode's stream, after it")
    ap.add_argument("--depth", type=int, default=1,
                    help="gradient buckets in flight: step i+1 is enqueued on its own streams next to step i "
                         "(1 = a step starts when the previous one has finished)")
    ap.add_argument("--time-every", type=int, default=4,
                    help="in the timed region every n-th launch of the roofline kernel carries HIP events")
    ap.add_argument("--no-kernel-timing", action="store_true",
                    help="leave the HIP-event kernel timers off during the timed region")
    return ap.parse_args()


def cpu_baseline(cfg, grad_dev, div):
    """The reference's torch-op sequence (insert: sequential C oracle) on this
    box's host cores, on the first 1/div of the gradient."""
    import torch

    from oracle import torch_path
    from zen_repro_amd import workloads

    n_s = cfg.n // div // (16 * cfg.partitions) * (16 * cfg.partitions)
    sub = workloads.Config(cfg.name, n_s, cfg.dtype, cfg.partitions, cfg.peers, cfg.overlap,
                           k=int(cfg.k * n_s / cfg.n) if cfg.k else 0)
    g = grad_dev[:n_s].cpu()
    nnz_est = sub.k if sub.k else int(torch.count_nonzero(g))
    per_peer = max(1, nnz_est // cfg.partitions)
    idx_l, val_l, _, _ = workloads.peer_payloads(sub, per_peer, device="cpu", seed=1)
    times, (c_idx, c_val, c_splits, _, _, _) = torch_path.timed_pass(g, sub.k, cfg.partitions, idx_l, val_l)
    total = sum(times.values())
    parity = parity_gate(sub, grad_dev[:n_s], idx_l, val_l, c_idx, c_val, c_splits)
    return parity, {
        "value": n_s * g.element_size() / total / 1e9,
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"first {n_s} of {cfg.n} elements (1/{div}), k={sub.k}, {cfg.peers} peer payloads of {per_peer}; "
                  f"select {times['select']:.2f}s partition {times['partition']:.2f}s merge {times['merge']:.2f}s; "
                  f"torch ops use {torch.get_num_threads()} threads, the sequential insert 1",
    }


def parity_gate(sub, grad_dev, idx_l, val_l, c_idx, c_val, c_splits):
    """The HIP path on the sample the CPU baseline has just worked through, checked against that pass's
    results (untimed): split sizes, the buckets' indices in their order and their values bit for bit; the
    merged indices and fp32 sums bit for bit against a sequential fp32 scatter_add_ on the CPU (the baseline
    itself accumulates in the values' own type, as the reference does)."""
    import torch

    from zen_repro_amd import LoadBalanceAllreduce, LocalGroup, TensorPartition

    dev, P = grad_dev.device, sub.partitions
    n_s = grad_dev.numel()
    capacity = int(sub.k * 1.25) + 4096 if sub.k else int(sum(t.numel() for t in c_idx)) + 16
    g_idx, g_val, g_splits = TensorPartition(P, 1, 3).load_balance(grad_dev, capacity=capacity, k=sub.k)
    bits = torch.int16 if grad_dev.dtype == torch.bfloat16 else torch.int32
    encode_ok = (torch.equal(g_splits.cpu(), c_splits.to(torch.int64))
                 and torch.equal(torch.cat(g_idx).cpu(), torch.cat(c_idx).to(torch.int32))
                 and torch.equal(torch.cat(g_val).cpu().view(bits), torch.cat(c_val).view(bits)))
    lba = LoadBalanceAllreduce(LocalGroup(P), None, None)
    m_idx, m_val = lba.merge_sparse([t.to(dev) for t in idx_l], [t.to(dev) for t in val_l], n_s)
    dense = torch.zeros(n_s, dtype=torch.float32)
    dense.scatter_add_(0, torch.cat(idx_l).to(torch.int64), torch.cat(val_l).to(torch.float32))
    want_idx = torch.nonzero(dense, as_tuple=True)[0]
    merge_ok = (torch.equal(m_idx.cpu(), want_idx)
                and torch.equal(m_val.cpu().view(torch.int32), dense[want_idx].view(torch.int32)))
    return {"ok": bool(encode_ok and merge_ok), "encode_bit_exact": bool(encode_ok), "merge_bit_exact": bool(merge_ok),
            "checked": f"the CPU baseline's sample: {int(g_splits.sum())} selected entries in {P} buckets, "
                       f"{int(m_idx.numel())} merged entries"}


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
    """The second exchange's decode (comm.py:142-145): P ascending, pairwise disjoint shards of merged entries
    (rank p's shard holds indices of hash partition p, as many as rank 0 merges in the main benchmark) into
    the dense gradient.  One step = one decode_sparse_tensors(ascending=True) of the concatenated shards;
    the result is checked against a plain assignment (the shards are disjoint)."""
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
    idx, val = [], []
    for p in range(P):
        members = torch.nonzero(part == p, as_tuple=True)[0]
        pick = torch.randperm(members.numel(), device=dev, generator=gen)[:per].sort().values
        idx.append(members[pick].contiguous())
        val.append((torch.randn(per, device=dev, generator=gen) * 1e-3).to(dtype))
        del members, pick
    del part
    flat_i, flat_v = torch.cat(idx), torch.cat(val)
    sizes = [t.numel() for t in idx]
    views = list(torch.split(flat_i, sizes)), list(torch.split(flat_v, sizes))  # what an all-gather into one buffer leaves

    def step():
        return lba.decode_sparse_tensors(views[0], views[1], n, ascending=True)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        dense = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    want = torch.zeros(n, dtype=dtype, device=dev)
    want[flat_i] = flat_v
    bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
    if not torch.equal(dense.view(bits), want.view(bits)):
        print("bench.py: the decoded dense tensor is not the shards' assignment", file=sys.stderr)
        sys.exit(1)
    r, s_ = flat_i.numel(), flat_v.element_size()
    b_alg = r * (8 + s_) + n * s_
    print(json.dumps({
        "metric": "phase-2 decode: all ranks' merged shards into the dense gradient", "value": round(b_alg / (ms * 1e-3) / 1e9, 2),
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "dtype": "bf16" if dtype == torch.bfloat16 else "f32", "data": "synthetic",
        "config": {"workload": f"{cfg.name}: {cfg.note}", "elements": n, "shards": P, "entries": r},
        "algorithmic_bytes": b_alg}))


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

    cfg, grad = workloads.make(args.config, device=dev, seed=0, shrink=args.shrink)
    n, esize, P = cfg.n, grad.element_size(), cfg.partitions
    tp = TensorPartition(P, 1, 3)
    lba = LoadBalanceAllreduce(LocalGroup(P), None, None)

    if cfg.k:
        nnz_guess = cfg.k
        capacity = int(cfg.k * 1.25) + 4096  # room for ties at the threshold
    else:
        nnz_guess = int(torch.count_nonzero(grad))
        capacity = nnz_guess + 16
    per_peer = max(1, nnz_guess // P)
    idx_l, val_l, flat_idx, flat_val = workloads.peer_payloads(cfg, per_peer, device=dev, seed=1)
    received = flat_idx.numel()

    # The merge of the received payloads does not depend on this rank's own encode, so it runs on a second
    # stream.  A training step hands over one gradient bucket after the other (train.py:167-185 is called
    # per bucket), and nothing in bucket i+1 depends on bucket i: with --depth 2 consecutive steps alternate
    # between two sets of streams, workspaces and tables ("slots"), so the long, memory-bound select of one
    # step runs next to the short, latency-bound kernels of the other.  All streams have default priority.
    depth = 1 if args.one_stream else max(1, args.depth)
    main = torch.cuda.current_stream(dev)
    enc_streams = [main] + [torch.cuda.Stream(device=dev) for _ in range(depth - 1)]
    mrg_streams = [None if (args.one_stream or args.merge_follows) else torch.cuda.Stream(device=dev)
                   for _ in range(depth)]

    def step(i):
        slot = i % depth
        es, ms_ = enc_streams[slot], mrg_streams[slot]
        with torch.cuda.stream(es):
            enc = tp.load_balance_flat(grad, None, capacity, k=cfg.k, slot=slot)
        with torch.cuda.stream(ms_ if ms_ is not None else es):
            mrg = lba.merge_sparse_flat(flat_idx, flat_val, n, capacity=received, slot=slot)
        return enc, mrg

    def run(count):
        outs = []
        for s_ in enc_streams[1:] + [m for m in mrg_streams if m is not None]:
            s_.wait_stream(main)  # the inputs were produced on the main stream
        for i in range(count):
            outs.append(step(i))
        for s_ in enc_streams[1:] + [m for m in mrg_streams if m is not None]:
            main.wait_stream(s_)
        return outs

    run(args.warmup)
    torch.cuda.synchronize()
    # An event between two kernels costs the device a few microseconds, about 40 of them per step with every
    # stage timed.  So the stage breakdown comes from an untimed pass of its own, and in the timed region only
    # the dominant kernel (the one the roofline figure is about) carries events, on every --time-every-th of
    # its launches (the pair of events around one launch holds the stream up for 10 us or so).
    streaming = ("k_select_stage", "k_select_compact", "k_topk_hist")  # kernels that read the dense gradient
    stages, dom = {}, None
    if not args.no_kernel_timing:
        _lib.profile_enable(True)
        run(args.steps)
        torch.cuda.synchronize()
        stages = _lib.profile_read()
        cands = [(stages[name][0], name) for name in streaming if name in stages]
        dom = max(cands)[1] if cands else None
        _lib.profile_enable(dom is not None, only=dom, every=max(1, args.time_every))
    t0 = time.perf_counter()
    outs = run(args.steps)
    t_enq = time.perf_counter()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    kernels = _lib.profile_read() if dom else {}
    _lib.profile_enable(False)

    (o_idx, o_val, splits, st_enc), (m_idx, m_val, m_count, st_mrg) = outs[-1]
    nnz = int(splits.sum())
    merged = int(m_count)
    flags = 0
    for enc, mrg in outs:  # every step of the timed region must have gone through cleanly and agree
        flags |= int(enc[3]) | int(mrg[3])
        if int(enc[2].sum()) != nnz or int(mrg[2]) != merged:
            print(f"bench.py: steps disagree on their result sizes (selected {int(enc[2].sum())} vs {nnz}, "
                  f"merged {int(mrg[2])} vs {merged}, status {int(enc[3])} / {int(mrg[3])})", file=sys.stderr)
            sys.exit(1)
    if flags:
        print("bench.py: device status " + _lib.describe_status(flags), file=sys.stderr)
        sys.exit(1)

    ms = (t1 - t0) * 1e3 / args.steps
    value = n * esize / (ms * 1e-3) / 1e9
    b_alg = workloads.algorithmic_bytes(n, esize, nnz, received, merged)

    # dominant kernel: the one with the largest summed duration among the
    # kernels that stream the dense gradient; its algorithmic bytes per launch
    per_launch = {
        "k_select_stage": n * esize + nnz * (4 + esize),
        "k_select_compact": n * esize + nnz * (4 + esize),
        "k_topk_hist": n * esize,
    }
    roofline = None
    stage_ms = {name: round(total / args.steps, 4) for name, (total, _) in stages.items()}
    if dom in kernels:
        total_ms, launches = kernels[dom]
        avg_ms = total_ms / launches
        achieved = per_launch[dom] / (avg_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                    "traffic": MEASURED_TRAFFIC.get((cfg.name, args.shrink, dom)),
                    "avg_launch_ms": round(avg_ms, 4), "launches_per_step": stages[dom][1] // args.steps,
                    "timed_launches": launches,
                    "algorithmic_bytes_per_launch": per_launch[dom]}

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
        "config": {"workload": f"{cfg.name}: {cfg.note}", "elements": n, "partitions": P, "k": cfg.k,
                   "selected": nnz, "received": received, "merged": merged, "peers": cfg.peers,
                   "overlap": cfg.overlap, "shrink": args.shrink, "steps_in_flight": depth},
        "path_algorithmic_GBps": round(b_alg / (ms * 1e-3) / 1e9, 2),
        "path_frac_of_hbm_peak": round(b_alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "host_enqueue_ms_per_step": round((t_enq - t0) * 1e3 / args.steps, 4),
        "stage_ms_per_step": stage_ms,
        "stage_ms_note": "from an untimed pass with every stage's events on; the timed region times only the "
                         "roofline kernel",
        "roofline": roofline,
        "cpu_baseline": None,
    }
    if not args.no_cpu_baseline:
        line["parity_vs_cpu_baseline"], line["cpu_baseline"] = cpu_baseline(cfg, grad, args.cpu_sample_div)
    print(json.dumps(line))
    if line.get("parity_vs_cpu_baseline") and not line["parity_vs_cpu_baseline"]["ok"]:
        print("bench.py: the HIP path and the CPU baseline disagree on the sample", file=sys.stderr)
        sys.exit(1)


if __name__ == "__main__":
    main()
