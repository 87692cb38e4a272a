"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dataflow auto|fod|gms|os] [--no-cpu]

One step = one forward pass of the submanifold 3x3x3 layer of configuration 2 (fp16, 64 -> 64
channels, ~150k voxels of the seeded LiDAR-like cloud) over a cached kernel map, features and map
resident in HBM.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def layer_records(forward, graph_ms, regret=True):
    """One record per distinct convolution of a network forward (fp16): the call's shapes and dataflow, its time
    (10 calls captured into a HIP graph, median of 5 replays), and what that time means against the two roofs --
    the layer's algorithmic bytes (input rows, output rows, residual rows, weights, the pair list) per second
    against the HBM peak, its multiply-accumulates against the dense fp16 MFMA peak.  `n` = how many layers of
    the forward have exactly this shape.  With `regret`, every convolution is also timed in each other dataflow
    that takes it and can be captured (output-stationary, ordered output-stationary, deferred scatter,
    gather-GEMM-scatter; atomic fetch-on-demand allocates its accumulator and is left out): `by_dataflow_ms`,
    `best` and `regret` = picked time / best time."""
    import torch
    from pcengine_amd import backend
    calls = []
    real_conv, real_dense = backend.conv_forward, backend.dense_forward

    def conv(feats, weight, km, dataflow, **kw):
        calls.append(("conv", feats, weight, km, dataflow, kw))
        return real_conv(feats, weight, km, dataflow, **kw)

    def dense(feats, weight, packed=None, **kw):
        calls.append(("dense", feats, weight, None, -1, dict(kw, packed=packed)))
        return real_dense(feats, weight, packed, **kw)
    backend.conv_forward, backend.dense_forward = conv, dense
    try:
        with torch.no_grad():
            forward()
    finally:
        backend.conv_forward, backend.dense_forward = real_conv, real_dense
    names = {backend.DATAFLOW_FOD: "fod", backend.DATAFLOW_GMS: "gms", backend.DATAFLOW_OS: "os", backend.DATAFLOW_FDS: "fds",
             backend.DATAFLOW_OSO: "oso", -1: "gemm"}
    records = {}
    for kind, feats, weight, km, flow, kw in calls:
        w3 = weight if weight.dim() == 3 else weight.unsqueeze(0)
        kv, c_in, c_out = w3.shape
        e = feats.element_size()
        if kind == "dense":
            n_in = n_out = feats.shape[0]
            M, what = 0, "1x1"
            flops = 2.0 * n_in * c_in * c_out
            fn = lambda: real_dense(feats, weight, kw["packed"], bias=kw.get("bias"), residual=kw.get("residual"), act=kw.get("act"))
        else:
            tr = bool(kw.get("transposed", False))
            n_in, n_out = (km.n_out, km.n_in) if tr else (km.n_in, km.n_out)
            M = km.M
            what = ("T" if tr else "") + ("subm" if km.subm else "strided") + "x".join(str(k) for k in km.ks)
            flops = 2.0 * (M + (n_in if km.subm else 0)) * c_in * c_out
            fn = lambda: real_conv(feats, weight, km, flow, **kw)
        res = kw.get("residual") is not None
        key = (what, n_in, n_out, M, c_in, c_out, names[flow], res)
        if key in records:
            records[key]["n"] += 1
            continue
        ms = graph_ms(fn, 10, 2, replays=5)[0]
        nbytes = n_in * c_in * e + n_out * c_out * e * (2 if res else 1) + kv * c_in * c_out * e + 8 * M
        records[key] = {"layer": what, "n_in": n_in, "n_out": n_out, "pairs": M, "c_in": c_in, "c_out": c_out,
                        "dataflow": names[flow], "residual": res, "n": 1, "ms": round(ms, 5),
                        "GBs": round(nbytes / ms / 1e6, 1), "hbm_frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 3),
                        "TFLOPs": round(flops / ms / 1e9, 1), "mfma_frac": round(flops / ms / 1e9 / 2500.0, 3)}
        if regret and kind == "conv":
            tr = bool(kw.get("transposed", False))
            by = {names[flow]: ms}
            for other in (backend.DATAFLOW_OS, backend.DATAFLOW_FDS, backend.DATAFLOW_OSO, backend.DATAFLOW_GMS):
                if other == flow or (other == backend.DATAFLOW_OSO and not backend.oso_takes(km, c_in, c_out, feats.dtype, tr)):
                    continue
                kw2 = dict(kw)
                if other == backend.DATAFLOW_GMS:       # stores dense rows: give it its own output and staging buffer
                    kw2["out"] = None
                    kw2["buffer"] = torch.empty(max(km.qsum * (c_in + c_out), 1), dtype=feats.dtype, device=feats.device)
                    o2 = torch.empty((n_out, c_out), dtype=feats.dtype, device=feats.device)
                    kw2["out"] = o2
                elif kw2.get("buffer") is None and other == backend.DATAFLOW_FDS:
                    kw2["buffer"] = torch.empty(max(km.M * c_out, 1), dtype=feats.dtype, device=feats.device)
                if kw2.get("out") is None:
                    kw2["out"] = torch.empty((n_out, c_out), dtype=feats.dtype, device=feats.device)
                try:
                    by[names[other]] = graph_ms(lambda: real_conv(feats, weight, km, other, **kw2), 10, 2, replays=3)[0]
                except Exception as exc:      # a dataflow that does not take the layer (or cannot be captured) is no candidate
                    print(f"bench.py: {what} {c_in}->{c_out} in {names[other]}: {exc}", file=sys.stderr)
            best = min(by, key=by.get)
            records[key].update({"by_dataflow_ms": {k: round(v, 5) for k, v in by.items()}, "best": best,
                                 "regret": round(ms / by[best], 3)})
    return list(records.values())


def regret_summary(records):
    """Selector regret over the distinct convolutions of a network: the worst layer, and the whole forward's
    convolution time as picked against the same with every layer in its best dataflow."""
    rs = [r for r in records if "regret" in r]
    if not rs:
        return None
    picked = sum(r["ms"] * r["n"] for r in rs)
    best = sum(min(r["by_dataflow_ms"].values()) * r["n"] for r in rs)
    worst = max(rs, key=lambda r: r["regret"])
    return {"layers": len(rs), "max": worst["regret"],
            "max_at": f'{worst["layer"]} {worst["c_in"]}->{worst["c_out"]} rows {worst["n_out"]} pairs {worst["pairs"]}: '
                      f'{worst["dataflow"]} picked, {worst["best"]} best',
            "time_weighted": round(picked / best, 4), "picked_ms": round(picked, 4), "best_ms": round(best, 4)}


def trace_net(config, forwards):
    """Forwards of the network of configuration 4 or 5 on its synthetic cloud: two to warm up (the first builds the
    kernel maps), `forwards` over the kept maps, `forwards` more with the maps built by the native planner."""
    import torch
    import pcengine_amd as pe
    from pcengine_amd import nets, synth
    dev = "cuda:0"
    if config == "cfg4":
        coords, kw, batches = synth.lidar_cloud_100k(), {}, 1
    else:
        coords, kw, batches = synth.indoor_batch(), dict(stem=64, enc=(64, 128, 256, 512), dec=(512, 256, 192, 192)), 8
    feats = torch.as_tensor(synth.features(4, len(coords), 4), device=dev).half()
    cd = torch.as_tensor(coords, device=dev)
    torch.manual_seed(4)
    model = nets.SparseResUNet(4, 20, **kw).to(dev).eval().fuse_bn().half()
    cmax = coords[:, 1:].max(0).tolist()

    def forward(keep=None):
        x = pe.spTensor(feats, cd, None, [0, 0, 0], cmax, batchsize=batches)
        if keep is not None:
            x.kmaps, x.cbook = keep.kmaps, keep.cbook
        with torch.no_grad():
            return model(x)

    def timed(fn):
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(forwards):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / max(forwards, 1)
    y0 = forward()
    forward(y0)
    kept = timed(lambda: forward(y0))
    model.use_planner()
    for _ in range(3):
        forward()
    planned = timed(forward)
    print(json.dumps({"config": config, "voxels": len(coords), "forwards": forwards, "forward_ms_kept_maps": round(kept, 3),
                      "forward_ms_planned_map_build": round(planned, 3)}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--dataflow", default="auto")
    ap.add_argument("--workload", default="cfg2", choices=["cfg2", "cfg2x8", "deep"],
                    help="cfg2: the headline layer; cfg2x8: the same layer on a batch of 8 such scans (1.2 M voxels, a working "
                         "set beyond the last-level cache); deep: a decoder-like layer (dense map, C 256->256) for the MFMA roofline")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-net", action="store_true", help="skip the MinkUNet-style forward (configuration 4)")
    ap.add_argument("--no-layers", action="store_true", help="skip the per-layer record of the configuration-4 network")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip configurations 1 (fp32 C16 layer), 3 (k2s2 down + transposed up) and 5 (8-scene indoor "
                         "batch, widened network), whose timings go to extra.cfg1 / cfg3 / cfg5")
    ap.add_argument("--trace-net", default=None, choices=["cfg4", "cfg5"],
                    help="run only forwards of the configuration-4 / configuration-5 network (what a kernel trace of the "
                         "network is taken from): --forwards of them over kept kernel maps, then as many that build their "
                         "maps through the native planner; prints one line and exits")
    ap.add_argument("--forwards", type=int, default=5)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this engine has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2
    if args.trace_net:
        return trace_net(args.trace_net, args.forwards)

    import numpy as np
    import torch
    from pcengine_amd import _lib, backend, synth
    from pcengine_amd.backend import DATAFLOW_FOD, DATAFLOW_GMS, DATAFLOW_OS, DATAFLOW_FDS, DATAFLOW_OSO

    lib = _lib.load()
    dev = "cuda:0"
    torch.cuda.set_device(0)
    ks = (3, 3, 3)
    if args.workload == "cfg2":
        c_in = c_out = 64
        coords = synth.lidar_cloud()
        what = "cfg2: submanifold 3x3x3 conv, fp16 storage / fp32 accumulate, C 64->64, batch 1, N={n} voxels " \
               "(64x2048 LiDAR-like rays + ground plane @0.1 m), M={M} pairs, cached kernel map"
    elif args.workload == "cfg2x8":
        c_in = c_out = 64
        scans = [synth.lidar_cloud(seed=2 + b) for b in range(8)]
        for b, sc in enumerate(scans):
            sc[:, 0] = b
        coords = np.concatenate(scans, axis=0)
        args.no_net = True
        what = "cfg2x8: the configuration-2 layer (submanifold 3x3x3, fp16, C 64->64) on a batch of 8 LiDAR-like scans, " \
               "N={n} voxels, M={M} pairs, cached kernel map"
    else:
        c_in = c_out = 256
        coords = synth.random_cloud(seed=7, n=90000, extent=58)
        args.no_net = True
        what = "deep: submanifold 3x3x3 conv, fp16 storage / fp32 accumulate, C 256->256, batch 1, N={n} voxels of a " \
               "dense random cloud (the pair density of the decoder layers of configuration 4), M={M} pairs, cached kernel map"
    n = len(coords)
    feats = synth.features(2, n, c_in)
    weight = synth.weights(2, 27, c_in, c_out)
    cd = torch.as_tensor(coords, device=dev)
    fd = torch.as_tensor(feats, device=dev).half()
    wd = torch.as_tensor(weight, device=dev).half()
    cmax = coords[:, 1:].max(0).tolist()

    def ev_ms(fn, steps, warmup):
        """Eager launches: HIP events on the current stream around `steps` calls."""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(steps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / steps

    REPLAYS = 11
    MIN_GRAPH_CALLS = 200

    def graph_ms(fn, steps, warmup, replays=REPLAYS, spread=None, min_calls=0):
        """`steps` calls captured into one HIP graph; the graph is replayed `replays` times, each replay
        between its own pair of HIP events on the current stream (the stream the kernels are launched on);
        the figure is the median replay divided by the calls in the graph (`spread` receives min / median /
        max).  Two or three launches of 5-15 us each are otherwise paced by the host.  With `min_calls` the
        `steps` calls are repeated inside the graph until it holds at least that many: the cost of launching
        a graph (about 20 us) is then spread over as many kernels whatever `steps` is."""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        if min_calls > steps:
            steps *= -(-min_calls // steps)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(steps):
                fn()
        g.replay()
        torch.cuda.synchronize()
        times = []
        for _ in range(replays):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            g.replay()
            b.record()
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b) / steps)
        times.sort()
        if spread is not None:
            spread.update({"min": times[0], "median": times[len(times) // 2], "max": times[-1], "replays": replays,
                           "steps_per_graph": steps})
        return times[len(times) // 2], g

    # ---- kernel map (built once, reused by every step; timed separately) -----------------------
    n_batch = int(coords[:, 0].max()) + 1

    def build_ms(batchsize, want_csr=True):
        """Wall time of one map build (median of 21, each from the call to the end of its work on the GPU).  With the
        batch count stated the sorted coordinates are indexed by column (what the front end does); without it they go
        through the hash table.  want_csr=True: pair lists, CSR views, neighbour table and row order; False: the
        neighbour table, the counts and the row order only (what the output-stationary dataflows read)."""
        build = lambda: backend.build_kernel_map(cd, ks, (1, 1, 1), (0, 0, 0), [0, 0, 0], cmax, True, want_csr=want_csr,
                                                 batchsize=batchsize, want_pairs=want_csr)
        km = build()
        for _ in range(3):
            build()
        torch.cuda.synchronize()
        times = []
        for _ in range(21):
            t0 = time.perf_counter()
            build()
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e3)
        return km, sorted(times)[len(times) // 2]
    km_hash, map_hash_ms = build_ms(0)
    km, map_ms = build_ms(n_batch)
    km_table, map_table_only_ms = build_ms(n_batch, want_csr=False)
    if not (torch.equal(km_table.nbr_out, km.nbr_out) and torch.equal(km_table.kpos, km.kpos) and km_table.M == km.M):
        raise RuntimeError("the map built without pair lists and the full map differ")
    del km_table
    if not (torch.equal(km.imap, km_hash.imap) and torch.equal(km.omap, km_hash.omap) and torch.equal(km.ocsr, km_hash.ocsr)):
        raise RuntimeError("the column-grid map and the hash-table map differ")
    del km_hash
    M = km.M

    names = {DATAFLOW_FOD: "fod", DATAFLOW_GMS: "gms", DATAFLOW_OS: "os", DATAFLOW_FDS: "fds", DATAFLOW_OSO: "oso"}
    packed = backend.pack_weights(wd)     # weights are constants: packed once, outside the timed region
    if args.dataflow == "auto":
        flow = backend.select_dataflow(km, c_in, c_out, torch.float16)
    else:
        flow = {v: k for k, v in names.items()}[args.dataflow]
    buffer = torch.empty(max(km.qsum * (c_in + c_out), 1), dtype=torch.float16, device=dev)
    out_buf = torch.empty((n, c_out), dtype=torch.float16, device=dev)
    step = lambda f=flow: backend.conv_forward(fd, wd, km, f, buffer=buffer, packed=packed, out=out_buf)

    # ---- timed region ---------------------------------------------------------------------------
    # Eager: K calls through the Python front end (what a caller without graphs sees; host paced).
    t_wall = time.perf_counter()
    eager_ms = ev_ms(step, args.steps, args.warmup)
    wall_ms = (time.perf_counter() - t_wall) * 1e3 / (args.steps + args.warmup)
    # Graph: the same K steps as one HIP graph, replayed once between HIP events.  Every replay is
    # checked against the eager result, with eager work and synchronisations between replays.
    want = step().clone()
    launch = "hip_graph"
    spread = {}
    try:
        ms, graph = graph_ms(step, args.steps, args.warmup, spread=spread, min_calls=MIN_GRAPH_CALLS)
        for _ in range(3):
            out_buf.zero_()
            step(DATAFLOW_OS)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            if not torch.equal(out_buf, want):
                raise RuntimeError("a graph replay disagrees with the eager result")
        timer = graph_ms
    except Exception as exc:     # capture not possible: report the eager figure
        print(f"bench.py: HIP graph capture failed ({exc}); timing eager launches", file=sys.stderr)
        launch, ms = "eager", eager_ms
        timer = lambda fn, steps, warmup, **kw: (ev_ms(fn, steps, warmup), None)

    # The same step with nothing left in the 256 MB last-level cache from the step before: twelve pairs of
    # (feature tensor, output tensor), 460 MB together, taken in turn inside one graph.  Between graph replays of
    # the single pair above, the 38 MB of the layer never leave that cache; a layer inside a network sees
    # something in between.  The map, the row order and the weights are shared by all pairs, as the layers of
    # one level of a network share them.
    cold = None
    if args.workload == "cfg2" and launch == "hip_graph":
        pairs = 12
        ins = [fd.clone() for _ in range(pairs)]
        outs = [torch.empty_like(out_buf) for _ in range(pairs)]
        turn = [0]

        def cold_step():
            i = turn[0] % pairs
            turn[0] += 1
            backend.conv_forward(ins[i], wd, km, flow, buffer=buffer, packed=packed, out=outs[i])
        turn[0] = 0
        cold_spread = {}
        cold_ms = graph_ms(cold_step, 20 * pairs, 0, spread=cold_spread)[0]
        if not all(torch.equal(o, want) for o in outs):
            raise RuntimeError("a step over rotated buffers disagrees with the eager result")
        cold = {"ms_per_step": round(cold_ms, 5), "buffer_pairs": pairs,
                "working_set_MB": round(pairs * (fd.numel() + out_buf.numel()) * 2 / 1e6, 1),
                "min": round(cold_spread["min"], 5), "max": round(cold_spread["max"], 5)}
        del ins, outs

    # calibration for hardware counters: a plain copy of known size (2 x 19.2 MB) runs three times, so
    # that a counter run can scale FETCH_SIZE / WRITE_SIZE by what they read for it
    for _ in range(3):
        fd.clone()

    # ---- per-stage durations of the chosen dataflow (stage mask), and the other dataflows -------
    e = 2
    stages = {}
    narrow = c_in <= 64 and c_out <= 64     # the barrier-free kernel takes these layers
    stage_names = {DATAFLOW_FOD: {0: "centre_gemm", 1: "fod_pairs", 2: "convert"},
                   DATAFLOW_GMS: {3: "gather", 1: "grouped_gemm", 0: "centre_gemm", 2: "scatter"},
                   DATAFLOW_FDS: ({1: "pairs_and_centre_gemm", 2: "partial_row_sum"} if narrow else
                                  {1: "fod_pairs_to_buffer", 2: "centre_gemm_then_row_sum"}),
                   DATAFLOW_OS: {1: "os_tile"}, DATAFLOW_OSO: {1: "ordered_rows"}}[flow]
    if flow not in (DATAFLOW_OS, DATAFLOW_OSO):
        # one stage at a time, on the measurement build of the library (the same kernels; the product library has
        # no stage switch)
        with _lib.measurement_build() as mlib:
            for bit, name in stage_names.items():
                mlib.pce_set_stage_mask((1 << bit) | 0xFFFFFFF0)   # bits 4 and up keep the kernel selection of the full run
                stages[name] = timer(step, max(20, args.steps // 4), 5, min_calls=MIN_GRAPH_CALLS)[0]
    else:
        stages[stage_names[1]] = ms       # one kernel is the whole layer
    takes = lambda f: f != DATAFLOW_OSO or backend.oso_takes(km, c_in, c_out, torch.float16)
    others = {names[f]: timer(lambda f=f: step(f), max(20, args.steps // 4), 5)[0]
              for f in names if f != flow and f != DATAFLOW_FOD and takes(f)}
    others[names[DATAFLOW_FOD]] = ev_ms(lambda: step(DATAFLOW_FOD), max(20, args.steps // 4), 5)   # allocates: eager

    # What the platform itself reaches on tensors of this size, in the same graph replays: a device copy of the
    # feature tensor into the output tensor (reads and writes what the layer must at least read and write, with no
    # indices and no arithmetic) and the centre offset's dense GEMM alone (one launch, rows in storage order).
    floors = {}
    if c_in == c_out:
        dst = torch.empty_like(fd)
        floors["device_copy_ms"] = timer(lambda: dst.copy_(fd), max(20, args.steps // 4), 5, min_calls=MIN_GRAPH_CALLS)[0]
        del dst
    w_mid = wd[13].contiguous()
    pk_mid = backend.pack_weights(w_mid)
    floors["centre_gemm_only_ms"] = timer(lambda: backend.dense_forward(fd, w_mid, packed=pk_mid), max(20, args.steps // 4), 5,
                                          min_calls=MIN_GRAPH_CALLS)[0]

    # algorithmic bytes of the layer: every tensor once + the pair list
    b_conv = n * c_in * e + n * c_out * e + 27 * c_in * c_out * e + 8 * M
    flops = 2.0 * (M + n) * c_in * c_out
    # dominant kernel of the chosen dataflow and its own algorithmic bytes
    dom = max(stages, key=stages.get)
    dom_bytes = {
        "centre_gemm": n * c_in * e + n * c_out * (4 if flow == DATAFLOW_FOD else e) + c_in * c_out * e,
        "fod_pairs": M * (c_in * e + c_out * 4) + 8 * M + 26 * c_in * c_out * e,
        "convert": n * c_out * (4 + e),
        "gather": n * c_in * e + M * c_in * e + 4 * M + 4 * (n + 1),
        "grouped_gemm": M * (c_in + c_out) * e + 26 * c_in * c_out * e,
        "scatter": M * c_out * e + 2 * n * c_out * e + 4 * M + 4 * (n + 1),
        "os_tile": b_conv - 8 * M + 4 * 27 * n,
        # every row in and out once, the gathered neighbour rows, the neighbour index of every pair, the order
        # (row index and offset mask of every row), every weight once
        "ordered_rows": n * c_in * e + n * c_out * e + M * c_in * e + 4 * M + 8 * n + 27 * c_in * c_out * e,
        "fod_pairs_to_buffer": M * (c_in + c_out) * e + 4 * M + 26 * c_in * c_out * e,
        "centre_gemm_csr_sum": n * c_in * e + n * c_out * e + c_in * c_out * e + M * c_out * e + 4 * M + 4 * (n + 1),
        # centre rows in and out, pair rows in and partial rows out, the two index lists, every weight once
        "pairs_and_centre_gemm": n * c_in * e + n * c_out * e + M * (c_in + c_out) * e + 8 * M + 27 * c_in * c_out * e,
        "partial_row_sum": 3 * M * c_out * e + 8 * M + 4 * (n + 1),
        "centre_gemm_then_row_sum": n * (c_in + c_out) * e + c_in * c_out * e + 3 * M * c_out * e + 8 * M + 4 * (n + 1),
    }[dom]
    achieved = dom_bytes / (stages[dom] * 1e-3) / 1e9
    # HBM bytes per launch of that kernel: hardware counters cannot be read from inside this process, so the
    # figure comes from the record the last rocprofv3 --pmc runs left in profiles/ (FETCH_SIZE and WRITE_SIZE,
    # scaled by what they read for a plain copy), and only while the kernel sources are the ones it was
    # measured on (the record holds their digest); otherwise null
    traffic = None
    try:
        import hashlib
        with open(os.path.join(ROOT, "profiles", "pmc_traffic.json")) as fh:
            rec = json.load(fh).get(f"{args.workload}/{dom}")
        with open(os.path.join(ROOT, "pcengine_amd", "csrc", "pce_conv.hip"), "rb") as fh:
            src = hashlib.sha256(fh.read()).hexdigest()[:16]
        if rec and rec.get("source_sha16") == src:
            traffic = rec["bytes_per_launch"]
    except (OSError, ValueError, KeyError):
        traffic = None
    if args.workload in ("cfg2", "cfg2x8"):
        roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                    "algorithmic_bytes": dom_bytes, "kernel_ms": round(stages[dom], 5),
                    "layer_bytes": b_conv, "layer_GBs": round(b_conv / (ms * 1e-3) / 1e9, 1),
                    "layer_frac": round(b_conv / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                    "layer_TFLOPs": round(flops / (ms * 1e-3) / 1e12, 2)}
        if cold is not None:
            # the same two fractions on the step over rotated buffers (one kernel is the layer, so the step is the
            # kernel when the ordered dataflow runs)
            cold["layer_frac"] = round(b_conv / (cold["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
            if len(stages) == 1:
                cold["frac"] = round(dom_bytes / (cold["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
    else:
        # flops of the dominant kernel alone: the pair products for the pair-tile kernel, everything for the
        # single-kernel output-stationary dataflow
        dom_flops = {"fod_pairs_to_buffer": 2.0 * M * c_in * c_out, "os_tile": flops,
                     "centre_gemm_then_row_sum": 2.0 * n * c_in * c_out}.get(dom, flops)
        tf = dom_flops / (stages[dom] * 1e-3) / 1e12
        roofline = {"bound": "mfma", "kernel": dom, "achieved": round(tf, 1), "peak": 2500.0, "unit": "TFLOP/s",
                    "frac": round(tf / 2500.0, 4), "traffic": None, "algorithmic_flops": dom_flops,
                    "kernel_ms": round(stages[dom], 5), "layer_flops": flops,
                    "layer_TFLOPs": round(flops / (ms * 1e-3) / 1e12, 1)}

    result = {
        "metric": "subm3_conv_layer_ms", "value": round(ms, 5), "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": what.format(n=n, M=M), "dataflow": names[flow], "selector": args.dataflow == "auto",
                   "launch": launch},
        "roofline": roofline,
        "extra": {"ms_per_step_replays": {k: (round(v, 5) if k not in ("replays", "steps_per_graph") else v) for k, v in spread.items()},
                  **({"cold_ms_per_step": cold["ms_per_step"], "cold": cold} if cold is not None else {}),
                  "eager_ms_per_step": round(eager_ms, 5), "eager_wall_ms_per_step": round(wall_ms, 5),
                  "map_build_ms": round(map_ms, 4), "map_build_hash_table_ms": round(map_hash_ms, 4),
                  "map_build_neighbour_table_and_order_only_ms": round(map_table_only_ms, 4),
                  "stage_ms": {k: round(v, 5) for k, v in stages.items()},
                  "other_dataflows_ms": {k: round(v, 5) for k, v in others.items()},
                  "floors": {**{k: round(v, 5) for k, v in floors.items()},
                             **({"device_copy_frac_of_hbm_peak": round(2 * n * c_in * e / (floors["device_copy_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
                                if "device_copy_ms" in floors else {})}},
    }

    # ---- configuration 4: MinkUNet-style forward, ~100k voxels, fp16, BN folded --------------------
    if not args.no_net:
        import pcengine_amd as pe
        from pcengine_amd import nets
        c4 = synth.lidar_cloud_100k()
        f4 = torch.as_tensor(synth.features(4, len(c4), 4), device=dev).half()
        c4d = torch.as_tensor(c4, device=dev)
        torch.manual_seed(4)
        model = nets.SparseResUNet(4, 20).to(dev).eval().fuse_bn().half()
        cmax4 = c4[:, 1:].max(0).tolist()

        def forward(keep=None):
            x = pe.spTensor(f4, c4d, None, [0, 0, 0], cmax4)
            if keep is not None:          # reuse the kernel maps of an earlier pass
                x.kmaps, x.cbook = keep.kmaps, keep.cbook
            with torch.no_grad():
                return model(x)
        net = {}
        for name in ("auto", "fod", "gms"):
            if name == "auto":
                os.environ.pop("PCENGINE_DATAFLOW", None)
            else:
                os.environ["PCENGINE_DATAFLOW"] = name
            y0 = forward()
            if name == "auto":
                y_auto = y0.feats.clone()
            full = ev_ms(forward, 10, 2)
            cached = ev_ms(lambda: forward(y0), 20, 3)
            net[name] = {"forward_ms_with_map_build": round(full, 4), "forward_ms_cached_maps": round(cached, 4)}
        os.environ.pop("PCENGINE_DATAFLOW", None)
        # the same forward with the maps of every cloud built through the native planner (one allocation for all maps,
        # two library calls) and the layer outputs cut from one arena: no device allocation in a forward
        model.use_planner()
        for _ in range(3):
            forward()
        if not torch.equal(forward().feats, y_auto):
            raise RuntimeError("the planned forward and the plain forward differ")
        net["auto"]["forward_ms_with_map_build_planned"] = round(ev_ms(forward, 20, 3), 4)
        torch.cuda.synchronize()
        n_alloc = torch.cuda.memory_stats()["allocation.all.allocated"]
        forward()
        torch.cuda.synchronize()
        net["auto"]["device_allocations_in_a_planned_forward"] = int(torch.cuda.memory_stats()["allocation.all.allocated"] - n_alloc)
        model.use_planner(False)
        # a serving loop that knows its next cloud: the maps of cloud i+1 are built on a second stream while the
        # network runs cloud i (every forward still builds all nine maps of its own cloud)
        from pcengine_amd.spconv import MapPrefetcher

        def prefetched(n):
            mk = lambda: pe.spTensor(f4, c4d, None, [0, 0, 0], cmax4)
            pf = MapPrefetcher(model.map_plan(), dev)
            nxt = mk()
            pf.submit(nxt)
            for _ in range(n):
                cur, nxt = nxt, mk()
                pf.take(cur)
                with torch.no_grad():
                    model(cur)
                pf.submit(nxt)
        prefetched(3)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        prefetched(10)
        torch.cuda.synchronize()
        net["auto"]["forward_ms_with_map_build_prefetched"] = round((time.perf_counter() - t0) * 1e3 / 11, 4)
        result["extra"]["cfg4_minkunet"] = {"voxels": int(len(c4)), "dtype": "f16", "selector": net["auto"],
                                            "all_fetch_on_demand": net["fod"], "all_gather_gemm_scatter": net["gms"]}
        if not args.no_layers:
            y0 = forward()
            recs4 = layer_records(lambda: forward(y0), graph_ms)
            result["extra"]["cfg4_minkunet"]["layers"] = recs4
            result["extra"].setdefault("selector_regret", {})["cfg4"] = regret_summary(recs4)
        # the same network in training mode (BatchNorm on batch statistics, cross-entropy on random labels):
        # forward + backward with kernel maps built every step, fp16 features and fp32 parameters
        torch.manual_seed(5)
        train_model = nets.SparseResUNet(4, 20).to(dev).train()
        target = torch.randint(0, 20, (len(c4),), device=dev)

        def train_step():
            train_model.zero_grad(set_to_none=True)
            x = pe.spTensor(f4, c4d, None, [0, 0, 0], cmax4)
            loss = torch.nn.functional.cross_entropy(train_model(x).feats.float(), target)
            loss.backward()
        result["extra"]["cfg4_minkunet"]["training_step_ms"] = round(ev_ms(train_step, 5, 2), 3)
        del train_model

    # ---- configurations 1, 3 and 5 ----------------------------------------------------------------------
    if not args.no_other_configs and args.workload == "cfg2":
        import pcengine_amd as pe
        from pcengine_amd import nets
        # cfg1: fp32, C 16 -> 16, ~20 k voxels
        c1 = synth.sphere_plane_cloud()
        f1 = torch.as_tensor(synth.features(1, len(c1), 16), device=dev).float()
        w1 = torch.as_tensor(synth.weights(1, 27, 16, 16), device=dev).float()
        km1 = backend.build_kernel_map(torch.as_tensor(c1, device=dev), ks, (1, 1, 1), (0, 0, 0), [0, 0, 0],
                                       c1[:, 1:].max(0).tolist(), True, want_csr=True)
        o1 = torch.empty((len(c1), 16), dtype=torch.float32, device=dev)
        fl1 = backend.select_dataflow(km1, 16, 16, torch.float32)
        b1 = torch.empty(max(km1.qsum * 32, 1), dtype=torch.float32, device=dev)
        t1 = timer(lambda: backend.conv_forward(f1, w1, km1, fl1, buffer=b1, out=o1), 100, 10)[0]
        result["extra"]["cfg1"] = {"voxels": int(len(c1)), "pairs": int(km1.M), "dtype": "f32", "dataflow": names[fl1],
                                   "layer_ms": round(t1, 5)}
        if not args.no_cpu:     # configuration 1 is the reference's CPU-runnable case: the torch CPU path beside it
            from oracle import cpu_path
            m1, v1, _, _ = cpu_path.time_layer(c1, f1.cpu().numpy(), w1.cpu().numpy(), ks, warmup=3, runs=10)
            result["extra"]["cfg1"]["cpu_map_build_ms"] = round(m1, 3)
            result["extra"]["cfg1"]["cpu_conv_ms"] = round(v1, 3)
            result["extra"]["cfg1"]["cpu_threads"] = torch.get_num_threads()
        # cfg3: k2s2 down 64 -> 128 on the cfg2 cloud, transposed k2s2 128 -> 64 back
        g3 = [(c - 1) // 2 for c in cmax]
        km3 = backend.build_kernel_map(cd, (2, 2, 2), (2, 2, 2), (0, 0, 0), [0, 0, 0], g3, False, want_csr=True,
                                       want_nbr_in=True, batchsize=1)
        wdn = torch.as_tensor(synth.weights(3, 8, 64, 128), device=dev).half()
        wup = torch.as_tensor(synth.weights(3, 8, 128, 64), device=dev).half()
        pdn, pup = backend.pack_weights(wdn), backend.pack_weights(wup)
        mid3 = torch.empty((km3.n_out, 128), dtype=torch.float16, device=dev)
        back3 = torch.empty((n, 64), dtype=torch.float16, device=dev)
        b3 = torch.empty(max(km3.qsum * 192, 1), dtype=torch.float16, device=dev)
        fd3 = backend.select_dataflow(km3, 64, 128, torch.float16)
        fu3 = backend.select_dataflow(km3, 128, 64, torch.float16, transposed=True)

        def down_up():
            backend.conv_forward(fd, wdn, km3, fd3, buffer=b3, packed=pdn, out=mid3)
            backend.conv_forward(mid3, wup, km3, fu3, transposed=True, buffer=b3, packed=pup, out=back3)
        t3 = timer(down_up, 100, 10)[0]
        result["extra"]["cfg3"] = {"voxels_in": int(n), "voxels_out": int(km3.n_out), "pairs": int(km3.M),
                                   "dataflow_down": names[fd3], "dataflow_up": names[fu3], "down_up_ms": round(t3, 5)}
        down = {f: timer(lambda f=f: backend.conv_forward(fd, wdn, km3, f, buffer=b3, packed=pdn, out=mid3), 50, 5)[0]
                for f in (DATAFLOW_OS, DATAFLOW_FDS, DATAFLOW_OSO)}
        result["extra"]["cfg3"]["down_ms_by_dataflow"] = {names[f]: round(t, 5) for f, t in down.items()}
        # the narrow stride-2 layers of a network's first levels on the same map (32 -> 32, 64 -> 64): the dataflow the
        # selector gives them beside the two others that take them
        narrow = {}
        for c3 in (32, 64):
            f3n = fd[:, :c3].contiguous()
            w3n = torch.as_tensor(synth.weights(3, 8, c3, c3), device=dev).half()
            p3n = backend.pack_weights(w3n)
            o3n = torch.empty((km3.n_out, c3), dtype=torch.float16, device=dev)
            pick = backend.select_dataflow(km3, c3, c3, torch.float16)
            flows = {f: timer(lambda f=f: backend.conv_forward(f3n, w3n, km3, f, buffer=b3, packed=p3n, out=o3n), 50, 5)[0]
                     for f in (DATAFLOW_OS, DATAFLOW_FDS, DATAFLOW_OSO)}
            narrow[f"{c3}x{c3}"] = {"selector": names[pick], **{names[f] + "_ms": round(t, 5) for f, t in flows.items()}}
        result["extra"]["cfg3"]["narrow_k2s2_layers"] = narrow
        # cfg5: 8 indoor scenes, the cfg4 network with channels doubled
        c5 = synth.indoor_batch()
        f5 = torch.as_tensor(synth.features(5, len(c5), 4), device=dev).half()
        c5d = torch.as_tensor(c5, device=dev)
        torch.manual_seed(5)
        model5 = nets.SparseResUNet(4, 20, stem=64, enc=(64, 128, 256, 512), dec=(512, 256, 192, 192)).to(dev).eval().fuse_bn().half()
        cmax5 = c5[:, 1:].max(0).tolist()

        def forward5(keep=None):
            x = pe.spTensor(f5, c5d, None, [0, 0, 0], cmax5, batchsize=8)
            if keep is not None:
                x.kmaps, x.cbook = keep.kmaps, keep.cbook
            with torch.no_grad():
                return model5(x)
        y5 = forward5()
        result["extra"]["cfg5"] = {"voxels": int(len(c5)), "scenes": 8, "dtype": "f16",
                                   "forward_ms_with_map_build": round(ev_ms(forward5, 5, 1), 3),
                                   "forward_ms_cached_maps": round(ev_ms(lambda: forward5(y5), 10, 2), 3)}
        if not args.no_layers:
            recs5 = layer_records(lambda: forward5(y5), graph_ms)
            result["extra"]["cfg5"]["layers"] = recs5
            result["extra"].setdefault("selector_regret", {})["cfg5"] = regret_summary(recs5)
        del model5, y5, f5, c5d

    # ---- CPU baseline: the oracle's torch path on this box's host cores, same workload ---------
    if not args.no_cpu:
        from oracle import cpu_path, oracle as orc
        # threads: what torch was given on this host (OMP_NUM_THREADS bounds a one-GPU box's share of the cores),
        # never more than the machine has
        cores = max(1, min(torch.get_num_threads(), os.cpu_count() or 1))
        torch.set_num_threads(cores)
        f16 = fd.float().cpu().numpy()
        w16 = wd.float().cpu().numpy()
        cpu_map_ms, cpu_conv_ms, cpu_out, _ = cpu_path.time_layer(coords, f16, w16, ks, warmup=3, runs=10)
        gpu_out = step().float().cpu().numpy()
        result["cpu_baseline"] = {"value": round(cpu_conv_ms, 3), "unit": "ms", "cores": cores, "kind": "port",
                                  "sample": f"the full {args.workload} layer (same N, M, C), fp32 on fp16-rounded inputs, "
                                            "median of 10 runs after 3 warm-ups; map build timed separately",
                                  "map_build_ms": round(cpu_map_ms, 3), "host_cpus": os.cpu_count()}
        result["extra"]["rel_l2_vs_cpu"] = float(orc.rel_l2(gpu_out, cpu_out))
        if not result["extra"]["rel_l2_vs_cpu"] <= 1e-3:
            raise RuntimeError(f"the timed layer is {result['extra']['rel_l2_vs_cpu']:.3e} (rel-L2) away from the CPU path: bar 1e-3")
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
