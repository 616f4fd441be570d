#!/usr/bin/env python3
"""Headline benchmark: NN evaluations per second of the 40-block x 256-filter
network, fp16 storage / fp32 accumulate, batch 64, on one MI355X.

A step is one forward pass (residual tower + 1x1 heads) over one batch of 64
synthetic positions that already sit in device memory; `value` is measured over exactly
--steps such steps.  The same JSON line also carries the rate through host buffers (PCIe
inside the timed region), the figure repeated over five blocks of --steps forwards, the
roofline of the GEMM and of the transforms from per-launch device timestamps, what a plain
copy of the same bytes takes on this box, the CPU baseline, the same network in fp32 and
the three smaller configurations.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

PEAK_MFMA_F16 = 2.5e15   # dense fp16 matrix FLOP/s, MI355X
PEAK_MFMA_F32 = 157.3e12
PEAK_HBM = 8.0e12        # bytes/s

# HBM bytes per launch of the Winograd GEMM come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (KiB per dispatch, scaled by what the same counters read for a plain copy kernel of known
# size).  Counters cannot be read from inside this process: the figure is read from the
# tracked summary of those runs, which states it for the workload it was measured on.
PMC_SUMMARY = os.path.join(ROOT, "profiles", "gemm_and_transform_40x256_fp16_b64_pmc.txt")


def measured_gemm_traffic(blocks, filters, precision, batch):
    """`gemm_traffic_bytes_per_launch = N` of the PMC summary, for its own workload only."""
    if (blocks, filters, precision, batch) != (40, 256, "fp16", 64):
        return None
    try:
        for line in open(PMC_SUMMARY):
            if "gemm_traffic_bytes_per_launch" in line and "=" in line:
                return float(line.split("=")[1].split()[0])
    except OSError:
        pass
    return None


def gemm_flops(batch, filters, n_layers):
    """Algorithmic flops of the 36 batched GEMMs of one forward:
    2 * 36 * (25*batch) * F * (18 + (L-1)*F)."""
    return 2.0 * 36 * 25 * batch * filters * (18 + (n_layers - 1) * filters)


def transform_bytes(batch, filters, n_layers, e):
    """Algorithmic HBM bytes per forward of the three transform kernel classes:
    external inputs + outputs of each launch, nothing counted twice.
      in_transform   (layer 0 only): input planes packed to 64 channels + V_0
      out_in         (layers 0..L-2): M_l in, V_{l+1} out, + the activation out on block
                     ends (layer 0 and second convs) + the skip activation in (l >= 2)
      out_transform  (last layer): M in, skip in, activation out"""
    T = 25 * batch
    act = batch * filters * 361 * e
    tiles = 36 * filters * T * e
    bn = 2 * filters * 4
    in_t = batch * 64 * 361 * e + 36 * 64 * T * e
    n_fused = n_layers - 1
    n_block_end = (n_layers - 1) // 2          # l = 0, 2, ..., L-3
    fused = n_fused * (2 * tiles + bn) + n_block_end * act + max(0, n_block_end - 1) * act
    out_t = tiles + act + bn + (act if n_layers >= 3 else 0)
    return in_t, out_t, fused


def cpu_baseline(orc, netgen, net, x, seconds_budget=15.0):
    """CPU oracle timed on this host: independent single-position forwards on all
    the cores this process may use (the shape of the reference's netbench)."""
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    cores = max(1, min(16, cores))
    provider = orc.use_openblas()
    w_ref, _ = netgen.prepare(net, orc.winograd_transform_f, orc.process_bn_var)
    ref = orc.OraclePipe()
    ref.initialize(net.filters)
    ref.push_weights(6, 18, net.filters, w_ref)
    t0 = time.perf_counter()
    ref.forward(x[0])
    one = time.perf_counter() - t0
    per_thread = max(1, min(256, int(seconds_budget / max(one, 1e-3))))
    n = cores * per_thread
    xs = np.concatenate([x] * (n // x.shape[0] + 1))[:n]
    pol, val, secs = ref.forward_many(xs, threads=cores)
    return {
        "value": n / secs, "unit": "evals/s", "cores": cores, "kind": "port",
        "sample": "%d single-position forwards of the same %dx%d net (CPU oracle, fp32, "
                  "Winograd F(4x4,3x3), sgemm=%s, 1 BLAS thread per call) on %d threads, %.1f s"
                  % (n, net.blocks, net.filters, provider, cores, secs),
    }, (pol, val)


def calibrate_heads(pipe, netgen, h, batch):
    """A deep random-init tower feeds the heads planes of magnitude 1e2..1e4, so the
    softmax is one-hot and tanh saturated: every simulation would follow one line and
    the search would degenerate.  The fully connected head weights are rescaled (one
    scalar each, measured on a batch of synthetic positions) so that the policy logits
    have unit spread and the value pre-activation is centred with spread 0.5 -- the
    tower, and therefore the device work per evaluation, is unchanged."""
    import copy
    x = netgen.synthetic_inputs(min(batch, 32), seed=77)
    pol, val = pipe.forward_batch(x)
    relu = lambda a: np.maximum(a, 0.0)
    p = relu((pol.reshape(-1, 2, 361) - h.bn_pol_mean[None, :, None]) * h.bn_pol_scale[None, :, None])
    logits = p.reshape(-1, 722) @ h.ip_pol_w.T + h.ip_pol_b
    v = relu((val - h.bn_val_mean[0]) * h.bn_val_scale[0])
    hid = relu(v @ h.ip1_val_w.T + h.ip1_val_b)
    out = hid @ h.ip2_val_w
    h2 = copy.copy(h)
    h2.ip_pol_w = (h.ip_pol_w / max(float(logits.std()), 1e-6)).astype(np.float32)
    g = 0.5 / max(float(out.std()), 1e-6)
    h2.ip2_val_w = (h.ip2_val_w * g).astype(np.float32)
    h2.ip2_val_b = np.array([-float(out.mean()) * g], np.float32)
    return h2


def search_workload(args, pkg, netgen):
    """The search workload: tree search with `threads` search threads driving the
    scheduler at max batch `batch`; every move `visits` root visits, `moves` moves of
    self-play from the empty board.  Prints one JSON line of its own."""
    B, F, blocks = args.batch, args.filters, args.blocks
    prec = pkg.FP16 if args.precision == "fp16" else pkg.FP32
    net = netgen.make_network(blocks, F, seed=2025)
    w, h = netgen.prepare(net)
    pipe = pkg.HIPScheduler(prec, B, device=0)
    pipe.initialize(F)
    pipe.push_weights(6, 18, F, w)
    h = calibrate_heads(pipe, netgen, h, B)
    dev = 1 if args.device_heads else 0
    if dev:
        pipe.push_heads(h)
    cfg = pkg.SearchConfig.default(threads=args.threads, visits=args.visits, moves=args.moves,
                                   seed=2027, reuse_tree=0 if args.no_tree_reuse else 1,
                                   device_heads=dev)
    warm = pkg.SearchConfig.default(threads=args.threads, visits=min(200, args.visits), moves=1,
                                    seed=1, device_heads=dev)
    pipe.selfplay(h, warm)
    pipe.reset_stats()
    res, moves = pipe.selfplay(h, cfg)
    pipe.close()
    fill = res.sched.requests / max(1, res.sched.batch_slots)
    out = {
        "metric": "search visits/sec and NN batch-fill ratio",
        "value": res.visits_per_s, "unit": "visits/s", "n_gpus": 1, "steps": res.moves_played,
        "warmup": 1, "ms_per_step": res.seconds / max(1, res.moves_played) * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 storage, f32 accumulate" if prec == pkg.FP16 else "f32",
        "data": "synthetic (seeded random weights, FC head weights rescaled to unsaturated "
                "outputs, self-play from the empty board)",
        "config": {"workload": "%d search threads, max batch %d, %dx%d %s, %d visits/move, "
                               "%d moves, heads on the %s"
                               % (args.threads, B, blocks, F, args.precision, args.visits,
                                  res.moves_played, "device" if dev else "search threads")},
        "batch_fill": fill, "mean_batch": res.sched.requests / max(1, res.sched.batches),
        "max_batch_seen": res.sched.max_batch_seen, "batches": res.sched.batches,
        "playouts": res.playouts, "nn_evals": res.evals,
        "nn_evals_per_s": res.sched.requests / res.seconds,
        "cache_hits": res.cache_hits, "halted": res.halted, "wasted": res.wasted,
        "seconds": res.seconds, "moves": moves,
    }
    print(json.dumps(out))


def netbench_workload(args, pkg, netgen):
    """The reference's built-in benchmark of this path (Network::benchmark, GTP `netbench`,
    reference src/Network.cpp:128-149): `threads` threads evaluate the empty board under
    random symmetries, cache off, one blocking request each, `steps` x max batch evaluations.
    Prints one JSON line of its own."""
    B, F, blocks = args.batch, args.filters, args.blocks
    prec = pkg.FP16 if args.precision == "fp16" else pkg.FP32
    if args.weights:
        # a network file, read and prepared by the library as the engine reads it
        pipe = pkg.HIPScheduler.from_file(args.weights, prec, B, device=0)
        h, F, blocks = None, pipe.filters, (pipe.n_layers - 1) // 2
    else:
        net = netgen.make_network(blocks, F, seed=2025)
        w, h = netgen.prepare(net)
        pipe = pkg.HIPScheduler(prec, B, device=0)
        pipe.initialize(F)
        pipe.push_weights(6, 18, F, w)
    boards = np.full((1, 361), pkg.EMPTY, np.uint8)
    pipe.netbench(h, boards, pkg.BLACK, args.threads, max(1, args.warmup) * B)
    pipe.reset_stats()
    done, secs = pipe.netbench(h, boards, pkg.BLACK, args.threads, args.steps * B)
    st = pipe.stats()
    pipe.close()
    out = {
        "metric": "netbench: evaluations/s through the request queue (Network::benchmark)",
        "value": done / secs, "unit": "evals/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": secs / max(1, st["batches"]) * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 storage, f32 accumulate" if prec == pkg.FP16 else "f32",
        "data": ("weights file %s" % args.weights if args.weights else
                 "synthetic (seeded random weights)") + ", the empty board under random symmetries",
        "config": {"workload": "%d threads, max batch %d, %dx%d %s, %d evaluations, heads on "
                               "the calling threads" % (args.threads, B, blocks, F,
                                                        args.precision, done)},
        "batch_fill": st["requests"] / max(1, st["batch_slots"]), "batches": st["batches"],
        "seconds": secs,
    }
    print(json.dumps(out))


def gemm_kernel_name(fp16, Fp, B):
    """The GEMM kernel the library launches for this precision, padded width and batch."""
    if fp16 and Fp in (128, 192, 256):
        return "wino_gemm_stream_k"
    if not fp16 and Fp in (128, 256):
        return "wino_gemm_stream32_k"
    return "wino_gemm_k / wino_gemm_big_k family"


def measure_forward(pkg, netgen, torch, blocks, F, precision, B, steps, warmup, lanes_arg,
                    profile_reps, host_buffers=False, blocks_of_k=0, min_block=200):
    """One network on the device: evaluations/s of `steps` forwards of B device-resident
    positions (all lanes, and one lane), optionally the same through host buffers, and the
    per-kernel-class durations with the roofline figures derived from them."""
    prec = pkg.FP16 if precision == "fp16" else pkg.FP32
    net = netgen.make_network(blocks, F, seed=2025)
    x = netgen.synthetic_inputs(B, seed=2026)
    w, h = netgen.prepare(net)
    pipe = pkg.HIPScheduler(prec, B, device=0)
    pipe.initialize(F)
    pipe.push_weights(6, 18, F, w)
    nl = net.n_layers

    d_in = torch.from_numpy(x).cuda()
    lanes = pipe.lanes() if lanes_arg <= 0 else max(1, min(lanes_arg, pipe.lanes()))
    d_pols = [torch.zeros(B, 722, device="cuda") for _ in range(lanes)]
    d_vals = [torch.zeros(B, 361, device="cuda") for _ in range(lanes)]
    d_pol, d_val = d_pols[0], d_vals[0]
    torch.cuda.synchronize()
    ptrs = (d_in.data_ptr(), d_pol.data_ptr(), d_val.data_ptr())

    # A step is one forward of one batch.  Steps go to the handle's lanes in turn (a lane is
    # a stream with the working buffers of one forward), so that `lanes` batches are on the
    # device side by side, as when the request queue has more callers than one batch holds.
    def timed(n_lanes, n_steps, n_warm):
        for i in range(n_warm):
            k = i % n_lanes
            pipe.forward_batch_device(B, d_in.data_ptr(), d_pols[k].data_ptr(),
                                      d_vals[k].data_ptr(), lane=k)
        pipe.sync()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n_steps):
            k = i % n_lanes
            pipe.forward_batch_device(B, d_in.data_ptr(), d_pols[k].data_ptr(),
                                      d_vals[k].data_ptr(), lane=k)
        pipe.sync()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    dt1 = timed(1, steps, warmup) if lanes > 1 else None
    dt = timed(lanes, steps, warmup)          # the headline figure: exactly `steps` steps
    if dt1 is None:
        dt1 = dt
    res = {"value": B * steps / dt, "ms_per_step": dt / steps * 1e3, "lanes": lanes,
           "one_lane": {"value": B * steps / dt1, "unit": "evals/s",
                        "ms_per_step": dt1 / steps * 1e3,
                        "note": "the same steps one after the other on one stream: the latency "
                                "of one batch"}}
    if blocks_of_k:
        # the same timed region again, blocks_of_k times: spread of the figure on this box
        # (at least min_block forwards a block, whatever --steps asks of the headline figure;
        # the short runs made for a profiler, --headline-only, keep --steps)
        per_block = max(steps, min_block)
        rates = sorted(B * per_block / timed(lanes, per_block, 2) for _ in range(blocks_of_k))
        rates1 = sorted(B * per_block / timed(1, per_block, 2) for _ in range(blocks_of_k))
        res["blocks_of_k"] = {"blocks": blocks_of_k, "forwards_per_block": per_block,
                              "median": rates[len(rates) // 2], "min": rates[0], "max": rates[-1],
                              "one_lane_median": rates1[len(rates1) // 2], "unit": "evals/s"}

    if host_buffers:
        # the same batch handed over as host buffers (pageable numpy arrays in and out): copy
        # to pinned staging, H2D, forward, D2H, copy out -- PCIe inside the timed region
        host_steps = max(steps, min_block)       # at least 200 forwards unless --headline-only
        pipe.forward_batch(x)
        t0 = time.perf_counter()
        for _ in range(host_steps):
            pipe.forward_batch(x)
        host_dt = (time.perf_counter() - t0) / host_steps
        # ... and from as many threads as the handle has lanes, a batch each at a time
        host2_dt = None
        if lanes > 1:
            import threading

            def host_caller():
                for _ in range(host_steps):
                    pipe.forward_batch(x)
            th = [threading.Thread(target=host_caller) for _ in range(lanes)]
            t0 = time.perf_counter()
            for t in th:
                t.start()
            for t in th:
                t.join()
            host2_dt = (time.perf_counter() - t0) / (host_steps * lanes)
        res["host_buffers"] = {
            "value": B / host_dt, "unit": "evals/s", "ms_per_step": host_dt * 1e3,
            "forwards": host_steps,
            "note": "lzhip_forward_batch on pageable host arrays, sequential calls: H2D + tower "
                    "+ 1x1 heads + D2H (PCIe and staging copies inside the timed region)",
            "callers_as_lanes": (None if host2_dt is None else
                                 {"value": B / host2_dt, "callers": lanes,
                                  "note": "one calling thread per lane, a batch each at a time"})}

        # Events on the stream around H2D (pinned) + tower + heads on the device + D2H
        # (pinned), forwards one after the other on one lane: five blocks of at least 200
        # forwards after 20 warm-up forwards, median.
        pipe.push_heads(h)
        per_block = max(steps, min_block)
        pipe.timed_evaluations(x, 20)
        ms_blocks = sorted(pipe.timed_evaluations(x, per_block)[0] for _ in range(5))
        med = ms_blocks[2]
        res["events_h2d_tower_heads_d2h"] = {
            "value": B * per_block / (med * 1e-3), "unit": "evals/s",
            "ms_per_forward": med / per_block, "forwards_per_block": per_block, "blocks": 5,
            "min": B * per_block / (ms_blocks[-1] * 1e-3), "max": B * per_block / (ms_blocks[0] * 1e-3),
            "note": "stream events around (copy of the planes from pinned host memory + tower + "
                    "fully connected heads, softmax and tanh on the device + copy of policy and "
                    "value to pinned host memory), one lane, median of five blocks"}

    # per-kernel-class device time, measured live with HIP events on the pipe's stream
    ms = np.zeros(pkg.K_COUNT)
    cnt = np.zeros(pkg.K_COUNT)
    pipe.profile_forward(B, *ptrs)   # untimed: the first event-timed forward creates its events
    for _ in range(profile_reps):
        m, c = pipe.profile_forward(B, *ptrs)
        ms += m
        cnt += c
    ms /= profile_reps
    cnt /= profile_reps
    # the same event-timed forward on lane 0 while another lane works through forwards of
    # its own: what a launch takes when it shares the device, as in the timed steps above
    ms2 = None
    if lanes > 1:
        ms2 = np.zeros(pkg.K_COUNT)
        for _ in range(profile_reps):
            for _ in range(3):
                pipe.forward_batch_device(B, d_in.data_ptr(), d_pols[1].data_ptr(),
                                          d_vals[1].data_ptr(), lane=1)
            m, _c = pipe.profile_forward(B, *ptrs)
            pipe.sync()
            ms2 += m
        ms2 /= profile_reps
    e = 2 if prec == pkg.FP16 else 4
    gf = gemm_flops(B, F, nl)
    in_b, out_b, fused_b = transform_bytes(B, F, nl, e)
    peak = PEAK_MFMA_F16 if prec == pkg.FP16 else PEAK_MFMA_F32
    gemm_rate = gf / (ms[pkg.K_GEMM] * 1e-3)
    Fp = (F + 63) // 64 * 64
    roofline = {
        "kernel": gemm_kernel_name(prec == pkg.FP16, Fp, B) + " (36-way batched Winograd GEMM)",
        "bound": "mfma", "achieved": gemm_rate / 1e12, "peak": peak / 1e12, "unit": "TFLOP/s",
        "frac": gemm_rate / peak,
        "traffic": measured_gemm_traffic(blocks, F, precision, B),
        "algorithmic_bytes_per_launch": 36.0 * e * (25 * B * F * 2 + F * F),
        "avg_launch_us": ms[pkg.K_GEMM] * 1e3 / cnt[pkg.K_GEMM],
        "launches_per_forward": int(cnt[pkg.K_GEMM]),
        "flops_per_launch": gf / cnt[pkg.K_GEMM],
    }
    roofline["launch_context"] = ("launches that run alone (event-timed forward on one lane, "
                                  "nothing else enqueued)")
    # The events bracket a launch's own execution; what lies between two launches of a chain
    # (the hand-over from one kernel to the next) is not in them, and a kernel trace, whose
    # durations run from one dispatch to the next, reads longer by that much.  The same
    # forward priced launch to launch: the one-lane wall time shared out over the launches
    # in proportion to their event durations.
    wall_ms = res["one_lane"]["ms_per_step"]
    stretch = wall_ms / float(ms.sum())
    roofline["launch_to_launch"] = {
        "avg_launch_us": roofline["avg_launch_us"] * stretch,
        "frac": roofline["frac"] / stretch,
        "note": "one-lane forward wall time (%.3f ms) shared out over its %d launches in "
                "proportion to their event durations: what a kernel trace reads per launch"
                % (wall_ms, int(cnt.sum()))}
    if ms2 is not None:
        roofline["side_by_side"] = {
            "avg_launch_us": ms2[pkg.K_GEMM] * 1e3 / cnt[pkg.K_GEMM],
            "frac": gf / (ms2[pkg.K_GEMM] * 1e-3) / peak,
            "note": "the same launches while another lane's forward shares the device: each "
                    "lasts longer, two are in progress"}
    # the same launch against the HBM roof: at this batch the GEMM's flop-per-byte ratio is below
    # the machine's (peak flops / peak bytes), so HBM, not MFMA, is the roof above it
    alg_bytes = roofline["algorithmic_bytes_per_launch"]
    roofline["flop_per_byte"] = roofline["flops_per_launch"] / alg_bytes
    roofline["machine_flop_per_byte"] = peak / PEAK_HBM
    roofline["hbm_view"] = {
        "achieved": alg_bytes / (roofline["avg_launch_us"] * 1e-6) / 1e9, "peak": PEAK_HBM / 1e9,
        "unit": "GB/s", "frac": alg_bytes / (roofline["avg_launch_us"] * 1e-6) / PEAK_HBM}

    def hbm(nbytes, k):
        if cnt[k] == 0:
            return None
        rate = nbytes / (ms[k] * 1e-3)
        return {"bound": "hbm", "achieved": rate / 1e9, "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                "frac": rate / PEAK_HBM, "bytes_per_launch": nbytes / cnt[k],
                "avg_launch_us": ms[k] * 1e3 / cnt[k], "launches_per_forward": int(cnt[k])}

    res["roofline"] = roofline
    res["roofline_transforms"] = {"out_in_transform": hbm(fused_b, pkg.K_OUTIN),
                                  "in_transform": hbm(in_b, pkg.K_IN),
                                  "out_transform": hbm(out_b, pkg.K_OUT)}
    res["kernel_ms_per_forward"] = {pkg.KERNEL_CLASSES[k]: float(ms[k]) for k in range(pkg.K_COUNT)}
    res["_net"], res["_x"], res["_pol"] = net, x, d_pol.cpu().numpy()
    pipe.close()
    return res


def copy_floor(torch, B, F, e):
    """What a plain device copy of the GEMM's tile arrays takes on this box: V-sized read +
    M-sized write (36 x 25B x F elements each) per launch, launches back to back, timed with
    events on the stream they run on -- at three working sets: two arrays that swap roles
    (resident in the 256 MB memory-side cache), three pairs (the working set of two lanes),
    and enough pairs to pass 1 GB (every byte from and to HBM)."""
    n = 36 * 25 * B * F
    dt = torch.float16 if e == 2 else torch.float32
    nbytes = 2.0 * n * e
    out = {"bytes_per_launch": nbytes, "unit": "GB/s",
           "note": "device-to-device copy of a V-sized array into an M-sized one (the bytes a "
                   "GEMM launch moves, less the filters), launch to launch"}

    def run(pairs, swap):
        src = [torch.ones(n, dtype=dt, device="cuda") for _ in range(pairs)]
        dst = src[::-1] if swap else [torch.empty(n, dtype=dt, device="cuda") for _ in range(pairs)]
        k = len(src)
        into = (lambda i: dst[i % k]) if swap else (lambda i: dst[(i + 1) % k])
        for i in range(2 * k):
            into(i).copy_(src[i % k])
        torch.cuda.synchronize()
        reps = 60
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(reps):
            into(i).copy_(src[i % k])
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / reps
        ws = (k if swap else 2 * k) * n * e
        return {"working_set_mb": ws / 1e6, "us_per_launch": us,
                "achieved": nbytes / (us * 1e-6) / 1e9,
                "frac_of_hbm_peak": nbytes / (us * 1e-6) / PEAK_HBM}

    big_pairs = int(0.55e9 // (n * e)) + 1
    out["cache_resident"] = run(2, True)
    out["two_lanes"] = run(3, False)
    out["hbm_only"] = run(big_pairs, False)
    # the figures earlier versions of this line carried, for the middle working set
    out.update({k: out["two_lanes"][k] for k in ("us_per_launch", "achieved", "frac_of_hbm_peak")})
    return out


def side_config(pkg, netgen, torch, blocks, F, precision, B, args, cpu=False):
    """One line for a configuration beside the headline one."""
    r = measure_forward(pkg, netgen, torch, blocks, F, precision, B, max(20, args.steps // 2),
                        args.warmup, 0, 2)
    net, x = r.pop("_net"), r.pop("_x")
    r.pop("_pol")
    t = r["roofline_transforms"]["out_in_transform"]
    out = {"value": r["value"], "unit": "evals/s", "lanes": r["lanes"],
           "one_lane": r["one_lane"]["value"], "ms_per_batch_one_lane": r["one_lane"]["ms_per_step"],
           "gemm_frac_of_mfma_peak": r["roofline"]["frac"],
           "gemm_us_per_launch": r["roofline"]["avg_launch_us"],
           "transform_frac_of_hbm_peak": t["frac"] if t else None,
           "transform_us_per_launch": t["avg_launch_us"] if t else None}
    if cpu and not args.no_cpu_baseline:
        orc = entry.load_oracle()
        c, _ = cpu_baseline(orc, netgen, net, x, seconds_budget=3.0)
        out["cpu_oracle"] = {"value": c["value"], "cores": c["cores"], "sample": c["sample"]}
    return out


def latency_by_batch(pkg, netgen, torch, blocks, F, precision, args):
    """Forward latency of the headline network at small batches (one lane, device-resident
    inputs, median of three runs of 60 forwards), and at batch 16 -- the batch a search with
    16 threads forms -- also with the forward's launches replayed from a HIP graph."""
    prec = pkg.FP16 if precision == "fp16" else pkg.FP32
    net = netgen.make_network(blocks, F, seed=2025)
    w, _ = netgen.prepare(net)
    out = {}

    def run(B, graph):
        if graph:
            os.environ["LZHIP_GRAPH"] = "1"
        try:
            pipe = pkg.HIPScheduler(prec, B, device=0)
            pipe.initialize(F)
            pipe.push_weights(6, 18, F, w)
        finally:
            os.environ.pop("LZHIP_GRAPH", None)
        d_in = torch.from_numpy(netgen.synthetic_inputs(B, seed=2026)).cuda()
        d_pol = torch.zeros(B, 722, device="cuda")
        d_val = torch.zeros(B, 361, device="cuda")
        torch.cuda.synchronize()
        ts = []
        for _ in range(3):
            for _ in range(10):
                pipe.forward_batch_device(B, d_in.data_ptr(), d_pol.data_ptr(), d_val.data_ptr())
            pipe.sync()
            t0 = time.perf_counter()
            for _ in range(60):
                pipe.forward_batch_device(B, d_in.data_ptr(), d_pol.data_ptr(), d_val.data_ptr())
            pipe.sync()
            ts.append((time.perf_counter() - t0) / 60 * 1e3)
        pipe.close()
        return sorted(ts)[1]

    for B in (1, 4, 8, 16, 32):
        out["b%d_ms" % B] = run(B, False)
    out["b16_graph_replay_ms"] = run(16, True)
    out["note"] = ("one lane, ms per forward of the whole batch; graph replay = the same launches "
                   "captured once and replayed (LZHIP_GRAPH=1)")
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--blocks", type=int, default=40)
    ap.add_argument("--filters", type=int, default=256)
    ap.add_argument("--batch", type=int, default=None,
                    help="max batch: default 64 (forward) or 32 (search)")
    ap.add_argument("--precision", choices=["fp16", "fp32"], default="fp16")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--headline-only", action="store_true",
                    help="forward workload: skip the fp32 run and the smaller configurations")
    ap.add_argument("--profile-reps", type=int, default=5)
    ap.add_argument("--lanes", type=int, default=0,
                    help="forward workload: batches kept on the device side by side; 0 = as "
                         "many as the handle has (2, or 3 up to batch 48)")
    ap.add_argument("--workload", choices=["forward", "search", "netbench"], default="forward",
                    help="forward: the headline metric; search: visits/s of a multi-threaded tree search; netbench: "
                         "the reference's Network::benchmark (threads x single-position requests)")
    ap.add_argument("--threads", type=int, default=16, help="search threads (search workload)")
    ap.add_argument("--visits", type=int, default=1600)
    ap.add_argument("--moves", type=int, default=20)
    ap.add_argument("--no-tree-reuse", action="store_true")
    ap.add_argument("--device-heads", action="store_true",
                    help="search workload: heads computed on the device, not on the search threads")
    ap.add_argument("--weights", default=None, metavar="FILE",
                    help="netbench workload: a Leela Zero weights file instead of the seeded "
                         "random network")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MIB",
                    help="only run a plain device copy kernel of MIB mebibytes three times "
                         "(known traffic, for scaling the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (one replica per GPU, no "
              "collectives); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    pkg = entry.ensure_built()
    import leela_zero_amd.netgen as netgen
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    if args.copy_probe:
        n = args.copy_probe * (1 << 20) // 4
        a = torch.ones(n, device="cuda")
        b = torch.empty(n, device="cuda")
        for _ in range(3):
            torch.mul(a, 1.0, out=b)      # reads n*4 bytes, writes n*4 bytes
        torch.cuda.synchronize()
        print(json.dumps({"copy_probe_mib": args.copy_probe, "bytes_read": n * 4,
                          "bytes_written": n * 4, "launches": 3}))
        return
    if args.batch is None:
        args.batch = 32 if args.workload == "search" else 64
    if args.workload == "search":
        search_workload(args, pkg, netgen)
        return
    if args.workload == "netbench":
        netbench_workload(args, pkg, netgen)
        return

    B, F, blocks = args.batch, args.filters, args.blocks
    head = measure_forward(pkg, netgen, torch, blocks, F, args.precision, B, args.steps,
                           args.warmup, args.lanes, args.profile_reps, host_buffers=True,
                           blocks_of_k=5, min_block=0 if args.headline_only else 200)
    net, x = head.pop("_net"), head.pop("_x")
    pol = head.pop("_pol")

    # parity spot check + CPU baseline (oracle as checker / reported baseline only)
    cpu = None
    if not args.no_cpu_baseline:
        orc = entry.load_oracle()
        cpu, (rpol, rval) = cpu_baseline(orc, netgen, net, x)
        k = min(B, rpol.shape[0])
        rel = float(np.linalg.norm(pol[:k] - rpol[:k]) / max(np.linalg.norm(rpol[:k]), 1e-30))
        cpu["raw_policy_plane_rel_l2_vs_gpu"] = rel

    out = {
        "metric": "NN evals/sec at 40x256 fp16 b64 on 1 MI355X; Winograd GEMM MFMA util %",
        "value": head["value"], "unit": "evals/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": head["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 storage, f32 accumulate" if args.precision == "fp16" else "f32",
        "data": "synthetic",
        "config": {"workload": "%d blocks x %d filters, %s, batch %d (the headline configuration when "
                               "40x256 fp16 b64), %d conv layers + 1x1 heads per step"
                               % (blocks, F, args.precision, B, net.n_layers),
                   "inputs": "device-resident fp32 NCHW [%d][18][361]" % B,
                   "lanes": head["lanes"]},
        "blocks_of_k": head["blocks_of_k"],
        "one_lane": head["one_lane"],
        "host_buffers": head["host_buffers"],
        "roofline": head["roofline"],
        "roofline_transforms": head["roofline_transforms"],
        "kernel_ms_per_forward": head["kernel_ms_per_forward"],
        "gemm_mfma_util_pct": 100.0 * head["roofline"]["frac"],
        "events_h2d_tower_heads_d2h": head["events_h2d_tower_heads_d2h"],
        "hbm_copy_floor": copy_floor(torch, B, F, 2 if args.precision == "fp16" else 4),
        "cpu_baseline": cpu,
    }
    # what this GEMM launch is against the copy rates measured above: the roof that applies
    # to one lane is the cache-resident one (V, M and the activations of a lane are ~100 MB)
    floor = out["hbm_copy_floor"]
    alg = out["roofline"]["algorithmic_bytes_per_launch"]
    us = out["roofline"]["avg_launch_us"]
    out["roofline"]["hbm_view"]["vs_copy_rate"] = {
        k: alg / (us * 1e-6) / 1e9 / floor[k]["achieved"]
        for k in ("cache_resident", "two_lanes", "hbm_only")}
    out["config"]["one_lane_evals_per_s"] = head["one_lane"]["value"]
    out["config"]["events_h2d_tower_heads_d2h_evals_per_s"] = head["events_h2d_tower_heads_d2h"]["value"]
    if not args.headline_only:
        # the same network in fp32, and the three smaller configurations, one line each
        if args.precision == "fp16":
            out["fp32"] = side_config(pkg, netgen, torch, blocks, F, "fp32", B, args)
        out["latency_by_batch"] = latency_by_batch(pkg, netgen, torch, blocks, F, args.precision,
                                                   args)
        out["configs"] = {
            "6x128 fp32 b1": side_config(pkg, netgen, torch, 6, 128, "fp32", 1, args, cpu=True),
            "15x192 fp32 b8": side_config(pkg, netgen, torch, 15, 192, "fp32", 8, args),
            "20x256 fp16 b32": side_config(pkg, netgen, torch, 20, 256, "fp16", 32, args),
        }
    out["environment"] = {"device": torch.cuda.get_device_name(0), "hip": torch.version.hip,
                          "torch": torch.__version__}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
