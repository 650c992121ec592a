"""Benchmark of the sparse steerable convolution layer on one MI355X.

One step = one forward of ss_conv.convolution.Convolution on the voxelised
batch, with everything the reference runs per training forward: rulebook build
(count + emit), steerable kernel synthesis, and the MFMA sparse convolution.
Inputs (voxel indices and features) are resident in HBM before the timed
region.  Workload: the second benchmark configuration by default (32 clouds x 2048 surface
points, 64^3 grid, irreps (4,4,4,4) -> (8,8,8,8), i.e. 64 -> 128 channels,
kernel 3, stride 1, padding 1, fp32).

Prints one JSON line; see --help for the other workloads.
"""
import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (os.path.join(ROOT, "ss-conv_amd"), os.path.join(ROOT, "oracle")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix peak

# the step is run for this long before the warm-up steps, to bring an idle GPU to its
# sustained clock
CLOCK_WARMUP_MS = 100

# HBM bytes per launch of the convolution kernel (per call for cfg5, whose call is three
# launches) for every workload this script offers, from rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE runs scaled by a copy kernel of known size (the summaries
# profiles/conv_fwd_<workload>_hbm_traffic.md give commands and counter values).
MEASURED_TRAFFIC_BYTES = {"cfg1": 4173070, "cfg2": 346645302, "cfg3": 227819460, "cfg5": 69089450913}
# the same for all kernels of one rulebook call and of one Point2Voxel call
# (profiles/rulebook_hbm_traffic.md, profiles/point_voxel_hbm_traffic.md)
RULEBOOK_TRAFFIC_BYTES = {"cfg2": 37500000, "cfg3": 28600000, "cfg5": 188400000}
P2V_TRAFFIC_BYTES = {"cfg2": 60500000, "cfg5": 119300000}
HBM_PEAK_GBS = 8000.0


def parse_args():
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5"],
                    help="cfg4: the backbone of the fourth configuration (evaluation mode), one "
                         "step = one forward of the whole backbone")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--time-every", type=int, default=0, metavar="N",
                    help="time every N-th launch of the convolution kernel with HIP events "
                         "(default: every fourth one, every launch below 20 steps)")
    ap.add_argument("--calibration-copy", type=int, default=0, metavar="MIB",
                    help="also run one plain device copy of MIB mebibytes before the timed "
                         "region (the known-size kernel that scales rocprofv3's FETCH_SIZE / "
                         "WRITE_SIZE counters)")
    ap.add_argument("--ops", action="store_true",
                    help="also time the other operators of the path (pools, global pools, "
                         "Point2Voxel, Voxel2Point) against their algorithmic HBM bytes; "
                         "table on stderr")
    ap.add_argument("--p2v", action="store_true",
                    help="also time Point2Voxel and Voxel2Point alone on the clouds of cfg2 and "
                         "cfg5; table on stderr")
    ap.add_argument("--backbone", action="store_true",
                    help="also run the backbone of the fourth configuration (Point2Voxel -> four "
                         "[Convolution -> BatchNorm -> gated Activation] stages -> GlobalAvgPool + "
                         "Voxel2Point, evaluation mode) and print, stage by stage, pairs, flops "
                         "and the convolution kernel's time and fraction of the fp32 MFMA peak; "
                         "table on stderr")
    ap.add_argument("--thin-layers", action="store_true",
                    help="also time layers whose last group of 16 output columns would be alone "
                         "in its block of 64 (64->72, 128->136, 152->8, 128->16), with the "
                         "kernel's one-column-group form and without (table on stderr)")
    ap.add_argument("--one-stream", action="store_true",
                    help="queue the index work (rulebooks, plans) on the convolutions' stream "
                         "instead of a second one: a step's kernels one after the other (for "
                         "kernel traces and counters)")
    ap.add_argument("--breakdown", action="store_true",
                    help="also print per-phase timings to stderr")
    return ap.parse_args()


def cpu_baseline(idx, feats, dense_w, cfg, n_out_expected):
    """The CPU restatement of the reference layer (serial rulebook, per-offset
    gather -> BLAS GEMM -> scatter-add) on the full workload, median of 3."""
    import numpy as np
    import oracle as O
    grid = cfg["grid"]
    times = []
    n_out = None
    for _ in range(3):
        t0 = time.perf_counter()
        o_idx, pairs, num, _ = O.rulebook(idx, cfg["batch"], [grid] * 3, cfg["kernel"],
                                          cfg["stride"], cfg["padding"])
        out = O.conv_fwd(feats, dense_w, pairs, num, o_idx.shape[0], matmul=np.matmul)
        times.append(time.perf_counter() - t0)
        n_out = o_idx.shape[0]
        if sum(times) > 40:
            break
    assert n_out == n_out_expected
    t = sorted(times)[len(times) // 2]
    try:
        from threadpoolctl import threadpool_info
        cores = max([p.get("num_threads", 1) for p in threadpool_info()] + [1])
    except Exception:
        cores = os.cpu_count() or 1
    return {"value": n_out / t, "unit": "active output voxels/s", "cores": int(cores),
            "kind": "port",
            "sample": "full %s layer (rulebook + gather/GEMM/scatter conv), median of %d runs, "
                      "%.2f s each; rulebook and gather/scatter single-thread C, GEMM numpy BLAS"
                      % (cfg["name"], len(times), t)}, out


def gpu_span_us(torch, dev, queue, reps=20):
    """GPU time in microseconds of the kernels `queue()` enqueues on the current stream: a
    pair of events around them, behind a fill kernel that keeps the GPU busy while the host
    enqueues (so the span holds no host time), minus what an empty pair of events reads in
    the same position.  queue() returns a function that finishes the call (waits, results),
    run after the second event is recorded.  Medians over `reps` calls; returns
    (span, empty span)."""
    filler = torch.empty(192 << 20, dtype=torch.uint8, device=dev)
    spans, empties = [], []
    for rep in range(reps + 3):
        for what in (0, 1):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            filler.zero_()
            e0.record()
            done = queue() if what else None
            e1.record()
            if done is not None:
                done()
            torch.cuda.synchronize()
            if rep >= 3:
                (spans if what else empties).append(e0.elapsed_time(e1) * 1e3)
    med = lambda v: sorted(v)[len(v) // 2]  # noqa: E731
    return med(spans), med(empties)


def rulebook_figure(torch, _ext, dev, indices, batch, shape, k, stride, pad, workload):
    """The rulebook of the layer by itself: GPU time of its kernels (events on their stream)
    against its algorithmic bytes 16 N_in + 16 N_out + 8 P + 4 K, and the call as the host
    sees it (get_indice_pairs with its wait)."""
    from ss_conv.sp_ops.ops import get_indice_pairs
    K = k ** 3
    out_idx, _, num = get_indice_pairs(indices, batch, shape, k, stride, pad)
    n_in, n_out, P = indices.shape[0], out_idx.shape[0], int(num.sum().item())
    nbytes = 16 * n_in + 16 * n_out + 8 * P + 4 * K

    def queue():
        r = _ext._rulebook_begin(indices, batch, shape, [k] * 3, [stride] * 3, [pad] * 3, [1] * 3,
                                 [0] * 3, 0, 0)
        return lambda: _ext._rulebook_finish(r)
    was = _ext.index_stream(False)  # (the kernels on the stream the events are recorded on)
    try:
        span, empty = gpu_span_us(torch, dev, queue)
    finally:
        _ext.index_stream(was)
    gpu_us = max(span - empty, 1e-3)
    def calls():
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            get_indice_pairs(indices, batch, shape, k, stride, pad)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e6 / 20
    call_us_default = calls()
    was = _ext.index_stream(False)
    try:
        call_us = calls()
    finally:
        _ext.index_stream(was)
    gbs = nbytes / gpu_us / 1e3
    return {"workload": workload, "bytes": nbytes, "gpu_us": gpu_us, "gbs": gbs,
            "frac_hbm": gbs / HBM_PEAK_GBS, "traffic": RULEBOOK_TRAFFIC_BYTES.get(workload),
            "call_us": call_us, "call_us_second_stream": call_us_default, "event_pair_us": empty,
            "n_in": n_in, "n_out": n_out, "pairs": P,
            "how": "HIP events around the kernels of one ssc_rulebook_begin on their stream, "
                   "median of 20, an empty event pair subtracted; call_us: get_indice_pairs "
                   "with its host wait, mean of 20, the kernels on the caller's stream; "
                   "call_us_second_stream: the same call as the library queues it by default, "
                   "on a second stream (built to run beside a convolution, not to return "
                   "sooner)"}


def point2voxel_figure(torch, _ext, synth, dev, workload, seed, channels=64):
    """Point2Voxel on the clouds of a configuration: the module call as the host sees it --
    a first call (a fresh module) and repeated calls -- and the GPU time of its kernels,
    against its algorithmic bytes N (12 + 8 + 4 C) + M (16 + 4 C) + 4 N."""
    from ss_conv.sp_ops.voxelize import Point2Voxel
    cfg = synth.CONFIGS[workload]
    pts, _, ids = synth.config_clouds(workload, seed)
    tp = torch.from_numpy(pts).to(dev)
    tf = torch.randn(tp.shape[0], channels, device=dev)
    ti = torch.from_numpy(ids).to(dev)
    grid = cfg["grid"]
    make = lambda: Point2Voxel([grid] * 3, [2.0 / grid] * 3)  # noqa: E731
    with torch.no_grad():
        p2v = make()
        r = p2v(tp, tf, ti)
        torch.cuda.synchronize()
        firsts = []
        for _ in range(10):
            m = make()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            m(tp, tf, ti)
            firsts.append((time.perf_counter() - t0) * 1e6)
            torch.cuda.synchronize()
        first_path = m.last_path
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(50):
            p2v(tp, tf, ti)
        torch.cuda.synchronize()
        call_us = (time.perf_counter() - t0) * 1e6 / 50

        def queue():
            p2v(tp, tf, ti)
            return None
        span, empty = gpu_span_us(torch, dev, queue)
    N, M = tp.shape[0], r[1].features.shape[0]
    nbytes = N * (12 + 8 + 4 * channels) + M * (16 + 4 * channels) + 4 * N
    gpu_us = max(span - empty, 1e-3)
    gbs = nbytes / gpu_us / 1e3
    return {"workload": workload, "points": N, "voxels": M, "channels": channels, "bytes": nbytes,
            "gpu_us": gpu_us, "gbs": gbs, "frac_hbm": gbs / HBM_PEAK_GBS,
            "traffic": P2V_TRAFFIC_BYTES.get(workload),
            "call_us": call_us, "first_call_us": sorted(firsts)[len(firsts) // 2],
            "path": p2v.last_path, "first_call_path": first_path, "event_pair_us": empty,
            "how": "gpu_us: HIP events around one module call (its one host wait included), "
                   "median of 20, an empty event pair subtracted; call_us: mean of 50 calls of "
                   "one module, host-timed; first_call_us: median of 10 first calls of fresh "
                   "modules on an idle GPU, host-timed like call_us (the call returns after "
                   "its one host wait, its last two kernels still running)"}


def ops_table(torch, _ext, synth, dev, seed):
    """Times the bandwidth-bound operators of the path on synthetic inputs of the
    benchmark shapes and prints time, algorithmic bytes and GB/s (of 8000 GB/s HBM
    peak) for each.  Rulebooks are built outside the timed region, except for the
    "module" rows, which time the user-facing layer as the reference runs it."""
    import numpy as np
    from ss_conv.pool import MaxPool, AvgPool, GlobalAvgPool, GlobalMaxPool
    from ss_conv.sp_ops.ops import get_indice_pairs, get_conv_output_size
    from ss_conv.sp_ops.tensor import SparseTensor
    from ss_conv.sp_ops.voxelize import Point2Voxel, Voxel2Point

    def timed(fn, n=20, warm=3, busy_ms=40.0):
        # (a GPU that has idled runs its first tens of milliseconds at a lower clock: every
        # row is measured behind busy_ms of the same work, as the layer step is)
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        t_busy = time.perf_counter()
        while (time.perf_counter() - t_busy) * 1e3 < busy_ms:
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
        a = time.perf_counter()
        for _ in range(n):
            r = fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - a) * 1e3 / n, r

    rows = []

    def report(name, ms, nbytes, note=""):
        gbs = nbytes / ms / 1e6
        rows.append("%-44s %8.3f ms %9.2f MB %8.1f GB/s %5.1f%% of HBM  %s"
                    % (name, ms, nbytes / 1e6, gbs, gbs / 80.0, note))

    # what a dependent launch costs whatever it does: 200 one-element kernels in a row between
    # two events (the floor under every operator below that is a chain of small kernels)
    one = torch.zeros(1, device=dev)
    for _ in range(20):
        one.add_(1.0)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(200):
        one.add_(1.0)
    e1.record()
    torch.cuda.synchronize()
    rows.append("%-44s %8.2f us each (200 dependent one-element kernels on one stream)"
                % ("dependent launch floor", e0.elapsed_time(e1) * 1e3 / 200))

    # convolution backward on the benchmark layer (cfg2: 64 -> 128 channels)
    cfg = synth.CONFIGS["cfg2"]
    pts, feats, ids = synth.config_clouds("cfg2", seed)
    idx = torch.from_numpy(synth.voxel_indices(pts, ids, cfg["grid"])).to(dev)
    o_idx, pairs, num = get_indice_pairs(idx, cfg["batch"], [cfg["grid"]] * 3, 3, 1, 1)
    cin, cout, K = 64, 128, 27
    f = torch.randn(idx.shape[0], cin, device=dev)
    w = torch.randn(3, 3, 3, cin, cout, device=dev) / (K * cin) ** 0.5
    go = torch.randn(o_idx.shape[0], cout, device=dev)
    P = int(num.sum().item())
    ms, _ = timed(lambda: _ext.indice_conv_backward_fp32(f, w, go, pairs, num, 0, 0), n=10)
    _ext.profile_conv(True)  # the input gradient is the forward kernel on the output gradient
    for _ in range(10):
        _ext.indice_conv_backward_fp32(f, w, go, pairs, num, 0, 0)
    in_ms = _ext.profile_conv_read()
    _ext.profile_conv(False)
    rows.append("%-44s %8.3f ms %9.2f GFLOP %7.1f TFLOP/s %5.1f%% of fp32 MFMA peak"
                % ("conv backward, cfg2 (input + filter gradient)", ms, 4.0 * P * cin * cout / 1e9,
                   4.0 * P * cin * cout / ms / 1e9, 4.0 * P * cin * cout / ms / 1e9 / 1.573))
    t_in = sum(in_ms) / max(len(in_ms), 1)
    rows.append("%-44s %8.3f ms %9.2f GFLOP %7.1f TFLOP/s %5.1f%% of fp32 MFMA peak"
                % ("  of which the input-gradient kernel (128->64)", t_in, 2.0 * P * cin * cout / 1e9,
                   2.0 * P * cin * cout / t_in / 1e9, 2.0 * P * cin * cout / t_in / 1e9 / 1.573))
    # the same layer on half-precision tensors (fp32 arithmetic, half the row bytes)
    fh, wh, goh = f.half(), w.half(), go.half()
    n_out_rows = o_idx.shape[0]
    ms32, _ = timed(lambda: _ext.indice_conv_fp32(f, w, pairs, num, n_out_rows, 0, 0), n=10)
    ms16, _ = timed(lambda: _ext.indice_conv_half(fh, wh, pairs, num, n_out_rows, 0, 0), n=10)
    msb16, _ = timed(lambda: _ext.indice_conv_backward_half(fh, wh, goh, pairs, num, 0, 0), n=10)
    for name, t, fl in (("conv forward call, cfg2, float32", ms32, 2.0), ("conv forward call, cfg2, half", ms16, 2.0),
                        ("conv backward, cfg2, half", msb16, 4.0)):
        rows.append("%-44s %8.3f ms %9.2f GFLOP %7.1f TFLOP/s %5.1f%% of fp32 MFMA peak"
                    % (name, t, fl * P * cin * cout / 1e9, fl * P * cin * cout / t / 1e9,
                       fl * P * cin * cout / t / 1e9 / 1.573))

    # pools on the output of the stride-2 layer: 32 clouds at 32^3, 256 channels
    cfg = synth.CONFIGS["cfg3"]
    pts, feats, ids = synth.config_clouds("cfg3", seed)
    idx = torch.from_numpy(synth.voxel_indices(pts, ids, cfg["grid"])).to(dev)
    shape = [cfg["grid"]] * 3
    o_idx, _, _ = get_indice_pairs(idx, cfg["batch"], shape, 3, 2, 1)
    shape2 = get_conv_output_size(shape, [3] * 3, [2] * 3, [1] * 3, [1] * 3)
    C = 256
    x = torch.randn(o_idx.shape[0], C, device=dev)
    st = SparseTensor(x, o_idx, shape2, cfg["batch"])
    p_idx, p_pairs, p_num = get_indice_pairs(o_idx, cfg["batch"], shape2, 2, 2, 0)
    P = int(p_num.sum().item())
    n_in, n_out = x.shape[0], p_idx.shape[0]
    nbytes = 4 * C * (n_in + n_out) + 8 * P
    ms, _ = timed(lambda: _ext.indice_maxpool_fp32(x, p_pairs, p_num, n_out))
    report("max pool k2 s2 (kernel, %d->%d rows, C=%d)" % (n_in, n_out, C), ms, nbytes)
    rf = _ext.indiceSummaryRF(p_pairs, p_num, n_out)
    ms, _ = timed(lambda: _ext.indice_avgpool_fp32(x, p_pairs, p_num, n_out, rf))
    report("avg pool k2 s2 (kernel)", ms, nbytes)
    mp = MaxPool(2, 2)
    ms, _ = timed(lambda: mp(st))
    report("MaxPool module (rulebook + kernel)", ms, nbytes + 16 * (n_in + n_out), "incl. rulebook")
    xh = x.half()
    hbytes = 2 * C * (n_in + n_out) + 8 * P
    ms, _ = timed(lambda: _ext.indice_maxpool_half(xh, p_pairs, p_num, n_out))
    report("max pool k2 s2, half rows (kernel)", ms, hbytes)
    ms, _ = timed(lambda: _ext.indice_avgpool_half(xh, p_pairs, p_num, n_out, rf))
    report("avg pool k2 s2, half rows (kernel)", ms, hbytes, "a rounding after every operation")

    # global pools: 32 segments over the pooled rows, 512 channels
    C = 512
    f = torch.randn(n_in, C, device=dev)
    offs = st.get_offsets().int().contiguous()
    B = offs.numel() - 1
    nbytes = 4 * C * (n_in + B) + 4 * (B + 1)
    ga, gm = GlobalAvgPool(), GlobalMaxPool()
    ms, _ = timed(lambda: ga(f, offs))
    report("GlobalAvgPool (%d rows, %d segments, C=%d)" % (n_in, B, C), ms, nbytes)
    ms, _ = timed(lambda: gm(f, offs))
    report("GlobalMaxPool", ms, nbytes + 4 * C * B)

    # Point2Voxel on the cfg2 and cfg5 clouds (65536 / 131072 points, 64 channels) and
    # Voxel2Point back
    point_voxel_rows(torch, synth, dev, seed, timed, report)

    # BatchNorm + gated Activation after the cfg2 layer: irrep(8,8,8,8) fields = 128 columns
    # plus 24 gate scalars, on the layer's 600k output rows
    from ss_conv import bnact
    from ss_conv.activation import Activation
    from ss_conv.batchnorm import BatchNorm
    from ss_conv.fused import BatchNormActivation
    Rs = synth.irreps(8, 3)
    n_gates = sum(m for m, l in Rs[1:])
    bn = BatchNorm(Rs + [(n_gates, 0)]).to(dev)
    act = Activation(Rs, (torch.relu, torch.sigmoid)).to(dev)
    fused = BatchNormActivation(bn, act).train()
    n_rows = 600000
    c_in = bn.num_channels
    c_out = c_in - n_gates
    x = torch.randn(n_rows, c_in, device=dev)
    zi = torch.zeros(n_rows, 4, dtype=torch.int32, device=dev)
    with torch.no_grad():
        ms, _ = timed(lambda: fused(SparseTensor(x, zi, [64] * 3, 32)), n=10)
        # statistics: the rows once (sums, sums of squares), the scalar columns a second
        # time (centred squares); then the rows once more for the output
        n_scalar = Rs[0][0] + n_gates
        fwd_cols = 2 * c_in + n_scalar + c_out
        report("BatchNorm+Activation fused, training (%d rows, %d->%d ch)" % (n_rows, c_in, c_out),
               ms, 4 * n_rows * fwd_cols, "statistics read the scalar columns twice")
        fused.eval()
        ms, _ = timed(lambda: fused(SparseTensor(x, zi, [64] * 3, 32)), n=10)
        report("BatchNorm+Activation fused, evaluation", ms, 4 * n_rows * (c_in + c_out))
        fused.train()
        keep = bnact.usable
        bnact.usable = lambda t: False   # the layers' torch code, for comparison
        try:
            ms, _ = timed(lambda: fused(SparseTensor(x, zi, [64] * 3, 32)), n=10)
        finally:
            bnact.usable = keep
        report("same layers as torch ops, training", ms, 4 * n_rows * fwd_cols,
               "same algorithmic bytes")
    # the whole block conv -> bn -> activation on the cfg2 geometry in evaluation mode: one
    # kernel (batch norm constants and gate applied while the rows are stored) against the
    # convolution followed by the fused batch norm + activation pass
    from ss_conv.fused import ConvBatchNormActivation
    from ss_conv.sp_ops.conv import SparseConvolution
    cfg = synth.CONFIGS["cfg2"]
    pts2, _, ids2 = synth.config_clouds("cfg2", seed)
    idx2 = torch.from_numpy(synth.voxel_indices(pts2, ids2, cfg["grid"])).to(dev)
    conv = SparseConvolution(3, 64, c_in, 3, 1, 1, bias=False, indice_key="b").to(dev)
    block = ConvBatchNormActivation(conv, bn, act).eval()
    f2 = torch.randn(idx2.shape[0], 64, device=dev)
    with torch.no_grad():
        st2 = SparseTensor(f2, idx2, [cfg["grid"]] * 3, cfg["batch"])
        y2 = block(st2)  # builds the rulebook, kept under the key

        def again(fn):
            t = SparseTensor(f2, idx2, [cfg["grid"]] * 3, cfg["batch"])
            t.indice_dict = y2.indice_dict
            return fn(t)
        ms_one, _ = timed(lambda: again(block), n=10)
        ms_sep, _ = timed(lambda: again(lambda t: fused.eval()(conv(t))), n=10)
        fused.train()
        # the same block on half-precision rows and filters (the tables stay float32)
        conv.half()
        f2h = f2.half()

        def again_half(fn):
            t = SparseTensor(f2h, idx2, [cfg["grid"]] * 3, cfg["batch"])
            t.indice_dict = y2.indice_dict
            return fn(t)
        block_half = ConvBatchNormActivation(conv, bn, act).eval()
        again_half(block_half)
        ms_half, _ = timed(lambda: again_half(block_half), n=10)
        conv.float()
    rows.append("%-44s %8.3f ms   (cached rulebook and plan, %d rows, 64 -> %d -> %d ch)"
                % ("conv+bn+act block, evaluation, one kernel", ms_one, y2.features.shape[0], c_in,
                   c_out))
    rows.append("%-44s %8.3f ms" % ("  the same as conv, then bn+act pass", ms_sep))
    rows.append("%-44s %8.3f ms" % ("  the one kernel on half rows and filters", ms_half))
    xg = x.clone().requires_grad_(True)
    dy = torch.randn(n_rows, c_out, device=dev)

    def step():
        y = fused(SparseTensor(xg, zi, [64] * 3, 32)).features
        y.backward(dy)
        xg.grad = None
    ms, _ = timed(step, n=10)
    nbytes = 4 * n_rows * (fwd_cols + 2 * (c_in + c_out) + c_in)
    report("BatchNorm+Activation fused, forward + backward", ms, nbytes,
           "backward reads rows and gradients twice")
    keep = bnact.usable
    bnact.usable = lambda t: False
    try:
        ms, _ = timed(step, n=5)
    finally:
        bnact.usable = keep
    report("same layers as torch ops, forward + backward", ms, nbytes, "same algorithmic bytes")

    # the whole backbone of the fourth configuration
    backbone = build_backbone(torch, synth, dev, seed)
    with torch.no_grad():
        ms, r = timed(backbone, n=5, warm=2)
    rows.append("%-44s %8.3f ms   (%d clouds x 1024 points; %d voxels after stage 4, %d channels)"
                % ("backbone forward, 4th configuration (eval)", ms, 32, r[2].features.shape[0],
                   r[2].features.shape[1]))
    print("\n".join(rows), file=sys.stderr)


def point_voxel_rows(torch, synth, dev, seed, timed, report):
    """Point2Voxel (as a module that is called again and again, which is how a training loop
    uses it) and Voxel2Point on the clouds of the second and fifth configuration."""
    from ss_conv.sp_ops.voxelize import Point2Voxel, Voxel2Point
    for name in ("cfg2", "cfg5"):
        cfg = synth.CONFIGS[name]
        pts, feats, ids = synth.config_clouds(name, seed)
        C = 64
        tp = torch.from_numpy(pts).to(dev)
        tf = torch.randn(tp.shape[0], C, device=dev)
        ti = torch.from_numpy(ids).to(dev)
        p2v = Point2Voxel([cfg["grid"]] * 3, [2.0 / cfg["grid"]] * 3)
        with torch.no_grad():
            ms, r = timed(lambda: p2v(tp, tf, ti), n=20)
        N, M = tp.shape[0], r[1].features.shape[0]
        report("Point2Voxel module, %s (%d pts -> %d voxels, C=%d)" % (name, N, M, C), ms,
               N * (12 + 8 + 4 * C) + M * (16 + 4 * C) + 4 * N,
               "path: %s; one host wait" % p2v.last_path)
        v2p = Voxel2Point(unit_voxel_extent=[2.0 / cfg["grid"]] * 3)
        vp, vs, vi = r[0], r[1], r[2]
        with torch.no_grad():
            ms, _ = timed(lambda: v2p(vs, vp, vi), n=20, warm=3)
        n = vp.shape[0]
        report("Voxel2Point module, %s (%d pts, %d voxels, C=%d)" % (name, n, M, C), ms,
               4 * C * 4 * n + 16 * (n + M) + 24 * n, "3-NN search around the query's cell")


def build_backbone(torch, synth, dev, seed):
    """The backbone of the fourth configuration in evaluation mode: inputs, layers and a
    function that runs it and returns (pooled, point features, last SparseTensor, stages),
    stages holding row counts, pair counts and channel counts of every convolution.
    backbone(separate=True) runs convolution, batch norm and activation of a block one
    after the other; by default a block is one fused.ConvBatchNormActivation, whose
    convolution kernel applies the other two while it stores its rows."""
    from ss_conv.activation import Activation
    from ss_conv.batchnorm import BatchNorm
    from ss_conv.convolution import Convolution
    from ss_conv.fused import BatchNormActivation, ConvBatchNormActivation
    from ss_conv.pool import GlobalAvgPool
    from ss_conv.sp_ops.voxelize import Point2Voxel, Voxel2Point
    pts, feats, ids = synth.make_clouds(32, 1024, seed=seed, channels=3)
    tp, tf, ti = [torch.from_numpy(a).to(dev) for a in (pts, feats, ids)]
    p2v = Point2Voxel([64] * 3, [2.0 / 64] * 3)
    layers, rs_in = [], [(3, 0)]
    for mult, stride in ((8, 1), (16, 2), (32, 2), (32, 1)):
        rs = synth.irreps(mult, 3)
        gated = rs + [(sum(m for m, l in rs[1:]), 0)]
        conv = Convolution(rs_in, gated, 3, stride=stride, padding=1)
        bn, act = BatchNorm(gated), Activation(rs, (torch.relu, torch.sigmoid))
        block = ConvBatchNormActivation(conv, bn, act).to(dev).eval()
        layers.append((block, BatchNormActivation(bn, act).to(dev).eval()))
        rs_in = rs
    gap = GlobalAvgPool()

    def backbone(separate=False):
        vp, x, vi, _ = p2v(tp, tf, ti)
        stages = []
        for block, bn_act in layers:
            n_in = x.features.shape[0]
            x = bn_act(block.conv(x)) if separate else block(x)
            stages.append((n_in, x.features.shape[0], x.indice_dict[None][3],
                           block.conv.in_channels, block.conv.out_channels))
        pooled = gap(x.features.contiguous(), x.get_offsets().int().contiguous())
        v2p = Voxel2Point(unit_voxel_extent=[2.0 / s for s in x.spatial_shape])
        return pooled, v2p(x, vp, vi), x, stages
    return backbone


def thin_layer_table(torch, _ext, synth, dev, seed):
    """Layers with Cout = 64 b + (1 ... 16) on the clouds of the second and third
    configuration: the convolution kernel's time (HIP events around its launches) with the
    last column group shared by the four consumer waves (the default: a launch of its own
    for b <= 2, or, with more than 192 input channels, as a fifth group of the last block)
    and with the group in a column block of its own (ssc_conv_tuning flags 2 and 8)."""
    from ss_conv.sp_ops.ops import get_indice_pairs
    rows = []
    for name, cin, cout, k, stride, pad in (("cfg2", 64, 72, 3, 1, 1), ("cfg2", 128, 136, 3, 1, 1),
                                            ("cfg2", 152, 8, 3, 1, 1), ("cfg3", 128, 16, 3, 2, 1),
                                            ("cfg3", 256, 72, 3, 2, 1), ("cfg2", 256, 136, 3, 1, 1)):
        cfg = synth.CONFIGS[name]
        pts, _, ids = synth.config_clouds(name, seed)
        idx = torch.from_numpy(synth.voxel_indices(pts, ids, cfg["grid"])).to(dev)
        o_idx, pairs, num = get_indice_pairs(idx, cfg["batch"], [cfg["grid"]] * 3, k, stride, pad)
        P, K = int(num.sum().item()), k ** 3
        f = torch.randn(idx.shape[0], cin, device=dev)
        w = torch.randn(k, k, k, cin, cout, device=dev) / (K * cin) ** 0.5
        times, outs = [], []
        for flags in (1, 1 | 2 | 8):
            _ext._lib.ssc_conv_tuning(flags)
            pr = pairs.clone()  # a rulebook without a plan of the other form
            try:
                for _ in range(3):
                    out = _ext.indice_conv_fp32(f, w, pr, num, o_idx.shape[0], 0, 0)
                torch.cuda.synchronize()
                _ext.profile_conv(True)
                for _ in range(10):
                    out = _ext.indice_conv_fp32(f, w, pr, num, o_idx.shape[0], 0, 0)
                ms = _ext.profile_conv_read()
            finally:
                _ext.profile_conv(False)
                _ext._lib.ssc_conv_tuning(1)
            times.append(sum(ms) / len(ms))
            outs.append(out)
        err = float((outs[0] - outs[1]).norm() / outs[1].norm())
        gf = 2.0 * P * cin * cout / 1e9
        rows.append("%s clouds, %3d -> %3d ch, k%d s%d: %d pairs, %.3f GFLOP; kernel %.3f ms (%.1f%% "
                    "of fp32 MFMA peak), %.3f ms with the group in a block of its own; rel-L2 "
                    "between the two %.1e"
                    % (name, cin, cout, k, stride, P, gf, times[0], gf / times[0] / 1.573, times[1], err))
    print("\n".join(rows), file=sys.stderr)


def backbone_table(torch, _ext, synth, dev, seed, n=5, warm=2):
    """Runs the backbone of the fourth configuration and prints one row per convolution
    stage: rows, pairs, flops, the MFMA kernel's time (HIP events around its launch) and
    its fraction of the fp32 MFMA peak; then the whole forward."""
    backbone = build_backbone(torch, synth, dev, seed)

    def run(**kw):
        a = time.perf_counter()
        for _ in range(n):
            out = backbone(**kw)
        torch.cuda.synchronize()
        return (time.perf_counter() - a) * 1e3 / n, out

    with torch.no_grad():
        for _ in range(warm):
            backbone(separate=True)
            r = backbone()
        torch.cuda.synchronize()
        ms_sep, _ = run(separate=True)
        _ext.profile_conv(True)
        ms, r = run()
        conv_ms = _ext.profile_conv_read()
        _ext.profile_conv(False)
    stages = r[3]
    rows = ["backbone of the fourth configuration (32 clouds x 1024 points, 64^3, evaluation mode):"]
    for i, (n_in, n_out, num, cin, cout) in enumerate(stages):
        P = int(num.sum().item())
        t = sum(conv_ms[i::len(stages)]) / max(len(conv_ms[i::len(stages)]), 1)
        fl = 2.0 * P * cin * cout
        rows.append("  stage %d: %7d -> %7d rows, %4d -> %4d ch, %9d pairs, %8.3f GFLOP, conv kernel "
                    "%8.3f ms = %6.1f TFLOP/s = %5.1f%% of fp32 MFMA peak"
                    % (i + 1, n_in, n_out, cin, cout, P, fl / 1e9, t, fl / t / 1e9,
                       fl / t / 1e9 / (FP32_MFMA_PEAK_TFLOPS / 100.0)))
    rows.append("  whole forward %.3f ms (%d voxels after stage 4, %d channels); %.3f ms with "
                "convolution, batch norm and activation as separate kernels"
                % (ms, r[2].features.shape[0], r[2].features.shape[1], ms_sep))
    rows.append("  (kernel times: with batch norm and gate applied by the convolution kernel; "
                "flops of the layer's own filter columns, gates included)")
    print("\n".join(rows), file=sys.stderr)


def backbone_line(args, torch, _ext, synth, dev):
    """--workload cfg4: one step = one forward of the backbone of the fourth configuration
    in evaluation mode (Point2Voxel, four [Convolution -> BatchNorm -> gated Activation]
    blocks, GlobalAvgPool, Voxel2Point).  The JSON line carries the whole forward as
    ms_per_step, every stage's convolution kernel time (HIP events around its launches) and,
    as roofline, the flops of the four convolutions over the sum of their kernel times."""
    backbone = build_backbone(torch, synth, dev, args.seed)
    with torch.no_grad():
        t_warm = time.perf_counter()
        while (time.perf_counter() - t_warm) * 1e3 < CLOCK_WARMUP_MS:
            r = backbone()
            torch.cuda.synchronize()
        for _ in range(args.warmup):
            r = backbone()
        torch.cuda.synchronize()
        gc.collect()
        n_st = len(r[3])
        steps = args.steps
        _ext.profile_conv(True, every=1)
        gc.disable()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            r = backbone()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        gc.enable()
        conv_ms = _ext.profile_conv_read()
        _ext.profile_conv(False)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        for _ in range(max(steps // 4, 1)):
            backbone(separate=True)
        torch.cuda.synchronize()
        ms_sep = (time.perf_counter() - t2) * 1e3 / max(steps // 4, 1)
    ms_per_step = (t1 - t0) * 1e3 / steps
    stages, flops_sum, kernel_sum, rows_sum = [], 0.0, 0.0, 0
    conv_ms = conv_ms[len(conv_ms) % n_st:]  # the ring holds whole forwards
    for i, (n_in, n_out, num, cin, cout) in enumerate(r[3]):
        P = int(num.sum().item())
        mine = conv_ms[i::n_st]
        t = sum(mine) / max(len(mine), 1)
        fl = 2.0 * P * cin * cout
        flops_sum += fl
        kernel_sum += t
        rows_sum += n_out
        stages.append({"stage": i + 1, "n_in": int(n_in), "n_out": int(n_out), "c_in": int(cin),
                       "c_out": int(cout), "pairs": P, "gflop": fl / 1e9, "kernel_ms": t,
                       "tflops": fl / t / 1e9 if t > 0 else 0.0,
                       "frac_mfma": fl / t / 1e9 / FP32_MFMA_PEAK_TFLOPS if t > 0 else 0.0})
    achieved = flops_sum / (kernel_sum * 1e-3) / 1e12 if kernel_sum > 0 else 0.0
    result = {
        "metric": "SS-Conv backbone forward: active output voxels/s over its four convolution "
                  "stages (Point2Voxel + 4 x [conv + bn + gate] + GlobalAvgPool + Voxel2Point)",
        "value": rows_sum / (ms_per_step * 1e-3), "unit": "active output voxels/s",
        "n_gpus": 1, "steps": steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "cfg4: backbone, 32 clouds x 1024 pts, 64^3 grid, 3 -> 152 -> 304 "
                               "-> 608 -> 608 filter columns (gates included), strides 1, 2, 2, 1, "
                               "evaluation mode",
                   "stages": stages, "clock_warmup_ms": CLOCK_WARMUP_MS,
                   "timed_region": "cyclic garbage collector off (as timeit does)",
                   "ms_per_step_separate_layers": ms_sep,
                   "voxels_after_stage_4": int(r[2].features.shape[0]),
                   "channels_after_stage_4": int(r[2].features.shape[1])},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": FP32_MFMA_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / FP32_MFMA_PEAK_TFLOPS, "traffic": None,
                     "kernel": "conv_fwd_kernel (the four stages' launches; batch norm and gate "
                               "applied by the kernel)",
                     "kernel_ms": kernel_sum, "kernel_launches_timed": len(conv_ms),
                     "flops_per_launch": flops_sum},
        "cpu_baseline": None,
    }
    print(json.dumps(result))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path uses no second GPU "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import synth
    from ss_conv import _ext
    from ss_conv.convolution import Convolution
    from ss_conv.sp_ops.tensor import SparseTensor
    from ss_conv.sp_ops.voxelize import Point2Voxel

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    if args.one_stream:
        _ext.index_stream(False)
    if args.workload == "cfg4":
        if args.steps == 100 and args.warmup == 20:  # the defaults are sized for a 0.4 ms step
            args.steps, args.warmup = 20, 5
        backbone_line(args, torch, _ext, synth, dev)
        return
    cfg = dict(synth.CONFIGS[args.workload], name=args.workload)
    grid = cfg["grid"]
    rs_in = synth.irreps(cfg["mult_in"], cfg["lmax"])
    rs_out = synth.irreps(cfg["mult_out"], cfg["lmax"])

    torch.manual_seed(args.seed)
    pts, feats, ids = synth.config_clouds(args.workload, args.seed)
    conv = Convolution(rs_in, rs_out, cfg["kernel"], stride=cfg["stride"],
                       padding=cfg["padding"]).to(dev)
    conv.train()  # the kernel is synthesised on every forward, as in a training step
    p2v = Point2Voxel([grid] * 3, [2.0 / grid] * 3)
    with torch.no_grad():
        _, st, _, _ = p2v(torch.from_numpy(pts).to(dev), torch.from_numpy(feats).to(dev),
                          torch.from_numpy(ids).to(dev))
    indices = st.indices.contiguous()
    features = st.features.contiguous()
    n_in, c_in = features.shape
    c_out = conv.out_channels
    K = cfg["kernel"] ** 3

    def step():
        x = SparseTensor(features, indices, st.spatial_shape, st.batch_size)
        with torch.no_grad():
            return conv(x)

    gc.collect()
    # A GPU that has idled while the host prepared the inputs runs its first tens of
    # milliseconds of work at a lower clock (the convolution kernel takes 0.33 ms in a step
    # that follows 2 ms of work, 0.30 ms after 40 ms of it).  The step is therefore run for
    # CLOCK_WARMUP_MS before the warm-up steps proper, so that the timed steps are those of a
    # GPU at its sustained clock; the JSON line says so (config.clock_warmup_ms).
    t_warm = time.perf_counter()
    while (time.perf_counter() - t_warm) * 1e3 < CLOCK_WARMUP_MS:
        for _ in range(10):
            out = step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        out = step()
    torch.cuda.synchronize()
    if args.calibration_copy > 0:
        src = torch.ones(args.calibration_copy << 18, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # every fourth launch of the convolution kernel inside the timed region is timed with HIP
    # events on its stream (a pair of events costs the stream 7-10 us: the kernel behind it
    # cannot be set up while the one before it still runs)
    _ext.profile_conv(True, every=args.time_every or (4 if args.steps >= 20 else 1))
    # The interpreter's cyclic garbage collector stays out of the timed region, as in
    # timeit: a full collection of a process that has imported torch takes 30-40 ms, many
    # times the region itself, and when it falls due depends on allocation counts only.
    # (The one collection that empties the backlog runs before the warm-up steps: the
    # hundred steps after a full collection are each about 15 us slower, collector on or
    # off, than steps that follow other steps.)
    gc.disable()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    gc.enable()
    conv_ms = _ext.profile_conv_read()
    _ext.profile_conv(False)
    # the same region with the collector left on, reported beside the headline figure: what
    # a Python caller that does not manage the collector sees on average
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    ms_gc_on = (time.perf_counter() - t2) * 1e3 / args.steps
    # and with the index work (rulebook, plan) on the convolution's own stream: a step's
    # kernels one after the other, nothing of one step beside the convolution of another
    was = _ext.index_stream(False)
    try:
        for _ in range(3):
            out = step()
        _ext.profile_conv(True, every=args.time_every or (4 if args.steps >= 20 else 1))
        gc.disable()
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        for _ in range(args.steps):
            out = step()
        torch.cuda.synchronize()
        ms_one_stream = (time.perf_counter() - t3) * 1e3 / args.steps
        gc.enable()
        conv_ms_alone = _ext.profile_conv_read()
        _ext.profile_conv(False)
    finally:
        _ext.index_stream(was)

    n_out = out.features.shape[0]
    pair_num = out.indice_dict[None][3] if None in out.indice_dict else None
    x = SparseTensor(features, indices, st.spatial_shape, st.batch_size)
    with torch.no_grad():
        from ss_conv.sp_ops.ops import get_indice_pairs
        _, _, num = get_indice_pairs(indices, st.batch_size, st.spatial_shape, cfg["kernel"],
                                     cfg["stride"], cfg["padding"])
    P = int(num.sum().item())
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    conv_kernel_ms = sum(conv_ms) / max(len(conv_ms), 1)
    flops = 2.0 * P * c_in * c_out
    achieved = flops / (conv_kernel_ms * 1e-3) / 1e12 if conv_kernel_ms > 0 else 0.0

    result = {
        "metric": "SS-Conv layer active output voxels/s (rulebook + kernel synthesis + conv)",
        "value": n_out / (ms_per_step * 1e-3),
        "unit": "active output voxels/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: %d clouds x %d pts, %d^3 grid, %d->%d ch, k=%d s=%d p=%d"
                               % (args.workload, cfg["batch"], cfg["points"], grid, c_in, c_out,
                                  cfg["kernel"], cfg["stride"], cfg["padding"]),
                   "n_in": int(n_in), "n_out": int(n_out), "pairs": P,
                   "input_voxels_per_s": n_in / (ms_per_step * 1e-3),
                   "timed_region": "cyclic garbage collector off (as timeit does)",
                   "clock_warmup_ms": CLOCK_WARMUP_MS,
                   "ms_per_step_gc_on": ms_gc_on,
                   "streams": "rulebook and plan on a second stream of the device (they need "
                              "the voxel indices only): a step's index work runs beside the "
                              "previous step's convolution" if was else "one",
                   "ms_per_step_one_stream": ms_one_stream},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": FP32_MFMA_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / FP32_MFMA_PEAK_TFLOPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
                     "kernel": "conv_fwd_kernel", "kernel_ms": conv_kernel_ms,
                     "kernel_launches_timed": len(conv_ms),
                     "flops_per_launch": flops,
                     # the same kernel with nothing beside it (the one-stream region: in the
                     # timed region the next step's index work shares the CUs with it)
                     "kernel_ms_one_stream": sum(conv_ms_alone) / max(len(conv_ms_alone), 1),
                     "frac_one_stream": (flops / (sum(conv_ms_alone) / max(len(conv_ms_alone), 1)
                                                  * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS)
                     if conv_ms_alone else None},
    }

    # the two bandwidth-bound callers of the layer that the metric names, measured in this
    # process: the rulebook of this workload and Point2Voxel on its clouds
    with torch.no_grad():
        result["rulebook"] = rulebook_figure(torch, _ext, dev, indices, st.batch_size,
                                             list(st.spatial_shape), cfg["kernel"], cfg["stride"],
                                             cfg["padding"], args.workload)
        result["point2voxel"] = point2voxel_figure(torch, _ext, synth, dev, args.workload,
                                                   args.seed)

    if args.breakdown:
        def timed(fn, n=10):
            torch.cuda.synchronize()
            a = time.perf_counter()
            for _ in range(n):
                r = fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - a) * 1e3 / n, r
        with torch.no_grad():
            t_rb, rb = timed(lambda: get_indice_pairs(indices, st.batch_size, st.spatial_shape,
                                                      cfg["kernel"], cfg["stride"], cfg["padding"]))
            t_ks, w = timed(lambda: conv.kernel())
            wv = w.permute(2, 3, 4, 1, 0)
            t_cv, _ = timed(lambda: _ext.indice_conv_fp32(features, wv, rb[1], rb[2], n_out, 0, 0))
        rb_bytes = 16 * n_in + 16 * n_out + 8 * P + 4 * K
        print("breakdown ms: rulebook %.3f (%.1f GB/s algorithmic) | kernel synthesis %.3f | "
              "conv call %.3f (MFMA kernel %.3f)" %
              (t_rb, rb_bytes / t_rb / 1e6, t_ks, t_cv, conv_kernel_ms), file=sys.stderr)

    if args.ops:
        ops_table(torch, _ext, synth, dev, args.seed)
    if args.p2v:
        rows = []

        def timed_pv(fn, n=20, warm=3):
            for _ in range(warm):
                fn()
            torch.cuda.synchronize()
            a = time.perf_counter()
            for _ in range(n):
                r = fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - a) * 1e3 / n, r

        def report_pv(name, ms, nbytes, note=""):
            gbs = nbytes / ms / 1e6
            rows.append("%-58s %8.3f ms %9.2f MB %8.1f GB/s %5.1f%% of HBM  %s"
                        % (name, ms, nbytes / 1e6, gbs, gbs / 80.0, note))
        point_voxel_rows(torch, synth, dev, args.seed, timed_pv, report_pv)
        print("\n".join(rows), file=sys.stderr)
    if args.backbone:
        backbone_table(torch, _ext, synth, dev, args.seed)
    if args.thin_layers:
        thin_layer_table(torch, _ext, synth, dev, args.seed)

    if not args.no_cpu_baseline:
        w = conv.kernel().detach().permute(2, 3, 4, 1, 0).reshape(K, c_in, c_out).cpu().numpy()
        base, ref_out = cpu_baseline(indices.cpu().numpy(), features.cpu().numpy(), w, cfg, n_out)
        result["cpu_baseline"] = base
        # the timed GPU result against the CPU port (first-touch vs key order: compare by key)
        import oracle as O
        o_idx, _, _, o_shape = O.rulebook(indices.cpu().numpy(), cfg["batch"], [grid] * 3,
                                          cfg["kernel"], cfg["stride"], cfg["padding"])
        order = np.argsort(O.flat_key(o_idx, o_shape), kind="stable")
        got = out.features.cpu().numpy()
        err = float(np.linalg.norm(got - ref_out[order]) / np.linalg.norm(ref_out))
        result["parity_rel_l2"] = err
    else:
        result["cpu_baseline"] = None

    print(json.dumps(result))


if __name__ == "__main__":
    main()
