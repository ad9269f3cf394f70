#!/usr/bin/env python3
"""Benchmark of the incremental sparse-convolution inference path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload incr|unet|ssc|cfg1|cfg2]

Prints ONE JSON line.  A step is one pass of the hot path over one batch of seeded synthetic
input that is already resident in HBM when the timed region starts:
  incr (default): workload 5 - one incremental U-Net frame of the 50-frame sensor sweep
         (3k-8k new voxels + 1k-2k re-observed voxels per frame, growing to 150k voxels).
         The LAST K incremental frames of the sweep are timed back to back, whatever K is, so
         that the timed region ends on the 150 000-voxel scene the metric names; frame 0 (full
         forward) and the 49 - K frames before them are untimed (W is a lower bound on those).
         value = mean ms per frame; frame_at_150k_ms = the last frame alone.
  unet : workload 4 - full U-Net forward over the 150k-voxel scene (165k points).
  ssc  : workload 3 - 4 x [SubmanifoldConvolution(3) + BatchNormReLU] at 500k active voxels,
         once at 32 channels and once at 64 (8 convolutions per step); value = Msites/s.
  cfg1 : workload 1 - one SubmanifoldConvolution(3) 16->16 on 20k voxels in 128^3: HIP us per
         call, the CPU oracle's ms, largest absolute / relative error between the two.
  cfg2 : workload 2 - hash grid insert of 200k voxels in 1024^3 (+10 % repeated points), query,
         3^3 rulebook and stride-2 rulebook: Minserts/s, Mqueries/s, GB/s, and whether every
         integer structure equals the CPU oracle's bit for bit (computed in the same run).
`roofline` is measured live on the dominant kernel, the submanifold gather-GEMM-scatter, at
the size the roofline target is stated for (500k voxels, 32 channels), with events on the
launch stream.  `cpu_baseline` times the CPU oracle (a restatement of the reference's CPU
path) on this machine's host cores over a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "ins-conv_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
MFMA_FP32_PEAK_TFLOPS = 157.3


def profile_records(name):
    """Machine-readable lines of a counter summary under profiles/: every line of the form
    `TRAFFIC key=value key=value ...` as a dict.  None if the summary is not there."""
    path = os.path.join(ROOT, "profiles", name)
    if not os.path.isfile(path):
        return None
    out = []
    with open(path) as f:
        for line in f:
            w = line.split()
            if w and w[0] == "TRAFFIC":
                out.append(dict(kv.split("=", 1) for kv in w[1:]))
    return out


def profiled_traffic(name, kernel):
    """HBM bytes per launch of `kernel` as recorded in profiles/<name> (FETCH_SIZE + WRITE_SIZE,
    each scaled by the copy-kernel calibration of the same run).  The summary must be about this
    kernel: a stale file fails loudly instead of lending its number to another kernel."""
    recs = profile_records(name)
    if recs is None:
        return None, "profiles/%s not found" % name
    hit = [r for r in recs if r.get("kernel") == kernel]
    if len(hit) != 1:
        raise SystemExit("bench.py: profiles/%s holds no TRAFFIC record for kernel %s" % (name, kernel))
    r = hit[0]
    fetch, write = float(r["fetch_bytes"]), float(r["write_bytes"])
    return fetch + write, ("HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by what the "
                           "same counter reads for a plain copy of known size: %.1f MB fetched + %.1f MB written, "
                           "profiles/%s" % (fetch / 1e6, write / 1e6, name))


# ---------------------------------------------------------------------------------------------
# workload 3: SSC layer stack at 500k voxels (also the roofline measurement)
# ---------------------------------------------------------------------------------------------
def build_ssc_stack(C, seed, device):
    import torch

    import sparseconvnet as scn

    torch.manual_seed(seed)
    net = scn.Sequential()
    for _ in range(4):
        net.add(scn.SubmanifoldConvolution(3, C, C, 3, False))
        bn = scn.BatchNormReLU(C)
        bn.running_mean.normal_(0, 1)
        bn.running_var.uniform_(0.5, 2.0)
        net.add(bn)
    return net.to(device).eval()


def ssc_workload(device, channels=(32, 64)):
    import numpy as np
    import torch

    from workloads import scenes
    import sparseconvnet as scn

    vox = scenes.indoor_scene(seed=3, n=500000)
    size = torch.LongTensor([4096, 4096, 4096])
    inp = scn.InputLayer(3, size, mode=4)
    rng = np.random.default_rng(3)
    stacks, xs = [], []
    coords = torch.from_numpy(vox.astype(np.int64))
    for C in channels:
        f = torch.from_numpy(rng.normal(size=(len(vox), C)).astype(np.float32)).to(device)
        x = inp([coords, f, 1])
        x.features = x.features.clone()
        xs.append(x)
        stacks.append(build_ssc_stack(C, 3, device))
        sc = x.metadata.ssc_rulebook(size)
    n_rules = x.metadata.n_ssc_rules(sc)

    def step():
        with torch.no_grad():
            for net, x in zip(stacks, xs):
                net(x)

    info = {"sites": len(vox), "rules": n_rules, "convs_per_step": 4 * len(channels)}
    return step, info, (xs[0], stacks[0])


def conv_roofline(device, reps=200, warm=300):
    """Average duration of the 32-channel submanifold convolution kernel at 500k voxels and the
    roofline figures derived from it."""
    import torch

    from sparseconvnet import SCN

    _, info, (x, stack) = ssc_workload(device, channels=(32,))
    n_rules = info["rules"]
    conv = stack[0]
    m = x.metadata
    sc = m.ssc_rulebook(x.spatial_size)
    out = torch.empty((sc.n, conv.nOut), device=device)
    w = conv.weight
    plan = m.ssc_plan(sc)  # built once per rulebook, like the neighbour map and the order
    # Warm-up.  On this part the clocks need some 25 ms of load to settle (the kernel's duration goes
    # 127 -> 145 -> 113 us over its first 200 launches).  The warm-up computes the same layer on the
    # per-tile kernel, so that a profiler's table for the filter-in-LDS kernel holds the timed launches
    # (and ten before them) only and its average can be compared with the figure printed here.
    from sparseconvnet._lib import lib
    lib.insc_conv_set_filter_lds_min_tiles(1 << 40)
    for _ in range(warm):
        SCN.ssc_rows_planned(x.features, out, w, None, sc, plan)
    lib.insc_conv_set_filter_lds_min_tiles(4096)
    for _ in range(10):
        SCN.ssc_rows_planned(x.features, out, w, None, sc, plan)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        SCN.ssc_rows_planned(x.features, out, w, None, sc, plan)
    e1.record()
    torch.cuda.synchronize()
    t = e0.elapsed_time(e1) * 1e-3 / reps
    Cin, Cout = conv.nIn, conv.nOut
    # every gathered row read once per rule (+ its two int32 ids), every output row written
    # once, the weights once
    bytes_alg = n_rules * (4 * Cin + 8) + sc.n * 4 * Cout + 27 * Cin * Cout * 4
    flops = 2.0 * n_rules * Cin * Cout
    achieved = bytes_alg / t / 1e9
    traffic, traffic_note = profiled_traffic("conv_wlds_ssc32_500k.txt", "insc::conv_wlds_kernel")
    return {
        "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
        "bound_in_practice": "mfma issue: `achieved` counts ALGORITHMIC bytes (every gathered row once per rule); the L2 "
                             "serves most of that reuse, so the HBM itself moves `traffic` bytes per launch "
                             "(hbm_GB/s_on_traffic), and what the kernel waits for is matrix-core issue (mfma_frac)",
        "hbm_GB/s_on_traffic": round(traffic / t / 1e9, 1) if traffic else None,
        "hbm_frac_on_traffic": round(traffic / t / 1e9 / HBM_PEAK_GBS, 4) if traffic else None,
        "kernel": "conv_wlds_kernel (SSC 3^3, 32->32, filter in LDS, persistent blocks; 500k sites, %d rules)" % n_rules,
        "avg_us": round(t * 1e6, 1), "algorithmic_bytes": int(bytes_alg),
        "traffic_note": traffic_note,
        "mfma_tflops": round(flops / t / 1e12, 2), "mfma_frac": round(flops / t / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4),
        "ssc_msites_per_s": round(sc.n / t / 1e6, 1),
    }


def wide_conv_row(device, C=64, reps=40, warm=60):
    """The 64-channel submanifold convolution of workload 3 (500k voxels), which is bound by the
    matrix cores rather than by HBM: us per launch and the fraction of the fp32 MFMA peak."""
    import torch

    from sparseconvnet import SCN

    _, info, (x, stack) = ssc_workload(device, channels=(C,))
    conv = stack[0]
    m = x.metadata
    sc = m.ssc_rulebook(x.spatial_size)
    out = torch.empty((sc.n, conv.nOut), device=device)
    plan = m.ssc_plan(sc)
    # (warm-up on another kernel that computes the same layer - the weight-sharing kernel switched off - so
    # that a profiler's table for conv_wshare_kernel holds the timed launches and five before them only)
    from sparseconvnet._lib import lib
    lib.insc_conv_set_shared_weights_min_units(1 << 40)
    for _ in range(warm):
        SCN.ssc_rows_planned(x.features, out, conv.weight, None, sc, plan)
    lib.insc_conv_set_shared_weights_min_units(896)
    for _ in range(5):
        SCN.ssc_rows_planned(x.features, out, conv.weight, None, sc, plan)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        SCN.ssc_rows_planned(x.features, out, conv.weight, None, sc, plan)
    e1.record()
    torch.cuda.synchronize()
    t = e0.elapsed_time(e1) * 1e-3 / reps
    flops = 2.0 * info["rules"] * C * C
    bytes_alg = info["rules"] * (4 * C + 8) + sc.n * 4 * C + 27 * C * C * 4
    return {"kernel": "conv_wshare_kernel<2, 4> (SSC 3^3, %d->%d, persistent blocks of four tiles sharing weight tiles through LDS, two output blocks per gathered chunk; 500k sites)" % (C, C),
            "bound": "mfma", "avg_us": round(t * 1e6, 1), "achieved": round(flops / t / 1e12, 2),
            "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(flops / t / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4),
            "GB/s_on_algorithmic_bytes": round(bytes_alg / t / 1e9, 1)}


def split_layer_row(device, C=96, shift=2, reps=200, warm=200):
    """The kernel the incremental frame spends most of its time in - conv_mfma_kernel<1, 27, 0, 4>,
    the items of a 32-row tile dealt to four wavefronts - on the layer it serves most often: 3^3,
    96 -> 96 channels, at the third scale of the 150 000-voxel scene (10 414 sites), alone in a loop.
    Useful and issued flops against the fp32 MFMA peak."""
    import numpy as np
    import torch

    import sparseconvnet as scn
    from sparseconvnet import SCN
    from workloads import scenes

    _, _, vox = scenes.unet_scene()
    coarse = vox.copy()
    coarse[:, :3] >>= shift
    _, first = np.unique(coarse, axis=0, return_index=True)
    coarse = coarse[np.sort(first)]
    size = torch.LongTensor([4096 >> shift] * 3)
    rng = np.random.default_rng(7)
    f = torch.from_numpy(rng.normal(size=(len(coarse), C)).astype(np.float32)).to(device)
    x = scn.InputLayer(3, size, mode=4)([torch.from_numpy(coarse[:, :3].astype(np.int64)), f, 1])
    m = x.metadata
    sc = m.ssc_rulebook(size)
    plan = m.ssc_plan(sc)
    w = torch.from_numpy((rng.normal(size=(27, C, C)) * (2.0 / C / 27) ** 0.5).astype(np.float32)).to(device)
    out = torch.empty((sc.n, C), device=device)
    for _ in range(warm):
        SCN.ssc_rows_planned(x.features, out, w, None, sc, plan)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        SCN.ssc_rows_planned(x.features, out, w, None, sc, plan)
    e1.record()
    torch.cuda.synchronize()
    t = e0.elapsed_time(e1) * 1e-3 / reps
    rules = m.n_ssc_rules(sc)
    tiles = (sc.n + 31) // 32
    tmask = plan[1][:tiles].cpu().numpy().astype(np.uint32)
    slots = 32 * int(sum(bin(int(v)).count("1") for v in tmask))
    useful, issued = 2.0 * rules * C * C, 2.0 * slots * C * C
    return {"kernel": "conv_mfma_kernel<1, 27, 0, 4> (SSC 3^3, %d->%d, one 32-row tile and output block per block of four "
                      "wavefronts; %d sites = scale %d of the 150 000-voxel scene, %d rules, %d tiles)"
                      % (C, C, sc.n, shift, rules, tiles),
            "bound": "mfma", "avg_us": round(t * 1e6, 1), "unit": "TFLOP/s", "peak": MFMA_FP32_PEAK_TFLOPS,
            "achieved": round(useful / t / 1e12, 2), "frac": round(useful / t / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4),
            "issued_tflops": round(issued / t / 1e12, 2),
            "issued_frac": round(issued / t / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4),
            "rule_slot_fill": round(useful / issued, 3),
            "offsets_used_per_tile": round(slots / 32.0 / tiles, 2),
            "note": "alone in a loop, plain epilogue; inside a frame the same layer also adds the residual, applies the "
                    "next batch norm and writes two outputs"}


# ---------------------------------------------------------------------------------------------
# the bandwidth-bound kernels of the path, one C call each, against the HBM roofline
# ---------------------------------------------------------------------------------------------
def kernel_table(device, reps=20, strict=True):
    """us per call, achieved GB/s on ALGORITHMIC bytes and fraction of the HBM peak for the hash
    grid, the rulebooks, batch norm and the input/output layers, on the workload-2 scene (200k
    voxels, 1024^3, plus 10 % repeated points) and, for the feature kernels, 500k x 32 floats."""
    import ctypes

    import numpy as np
    import torch

    from workloads import scenes
    from sparseconvnet._lib import lib, ptr, stream_ptr

    I64 = ctypes.c_int64
    st = stream_ptr()
    rng = np.random.default_rng(2)
    vox = scenes.planes_boxes_scene(seed=2, n=200000).astype(np.int32)
    pts = np.concatenate([vox, vox[rng.integers(0, len(vox), len(vox) // 10)]])
    pts = pts[rng.permutation(len(pts))]
    if pts.shape[1] == 3:
        pts = np.concatenate([pts, np.zeros((len(pts), 1), np.int32)], 1)
    P, N = len(pts), len(vox)
    c4 = torch.from_numpy(np.ascontiguousarray(pts[:, :4])).to(device)
    sop = torch.empty(P, dtype=torch.int32, device=device)
    grid, coarse = ctypes.c_void_p(), ctypes.c_void_p()
    lib.insc_grid_create(I64(2 * N), ctypes.byref(grid))
    lib.insc_grid_create(I64(N), ctypes.byref(coarse))
    n_sites = I64(0)
    nbr = torch.empty((N, 27), dtype=torch.int32, device=device)
    parent = torch.empty(N, dtype=torch.int32, device=device)
    offset = torch.empty(N, dtype=torch.int32, device=device)
    child = torch.empty((N, 8), dtype=torch.int32, device=device)
    C, NF = 32, 500000
    x = torch.randn(NF, C, device=device)
    y = torch.empty_like(x)
    mean, var = torch.zeros(C, device=device), torch.ones(C, device=device)
    fp = torch.randn(P, C, device=device)
    acc = torch.zeros(N, C, device=device)
    cnt = torch.zeros(N, dtype=torch.int32, device=device)
    outp = torch.empty(P, C, device=device)

    def timed(fn, pre=None):
        for _ in range(2):
            if pre:
                pre()
            fn()
        torch.cuda.synchronize()
        total = 0.0
        for _ in range(reps):
            if pre:
                pre()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            total += e0.elapsed_time(e1)
        return total * 1e-3 / reps

    rows = []
    # HBM bytes per call from the counter summary of this very table (FETCH_SIZE + WRITE_SIZE, calibrated)
    recs = profile_records("path_kernels_cfg2.txt")
    traffic = {r["row"]: float(r["fetch_bytes"]) + float(r["write_bytes"]) for r in recs or [] if "row" in r}
    if recs is not None and strict:  # (--kernels-only, the run a summary is cut from, passes strict=False)
        # a summary that lacks a row, or holds a zero for it (a kernel renamed since the summary was cut),
        # must not pass for a measurement
        for key in ("insert", "query", "ssc", "down", "bn", "input", "output", "labels"):
            if not traffic.get(key, 0.0) > 0.0:
                raise SystemExit("bench.py: profiles/path_kernels_cfg2.txt holds no (or a zero) TRAFFIC record for row "
                                 "'%s': regenerate the summary" % key)

    def add(name, sec, nbytes, note, key=None):
        gbs = nbytes / sec / 1e9
        row = {"kernel": name, "us": round(sec * 1e6, 1), "algorithmic_bytes": int(nbytes),
               "GB/s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4), "units": note}
        if key in traffic:
            row["traffic_bytes"] = int(traffic[key])
            row["traffic_over_algorithmic"] = round(traffic[key] / nbytes, 2)
            row["hbm_GB/s_on_traffic"] = round(traffic[key] / sec / 1e9, 1)
        rows.append(row)

    # the box's own copy bandwidth at this size, as the reference point for the rows below
    t = timed(lambda: y.copy_(x))
    add("device-to-device copy (torch; reference point, not a kernel of the path)", t, NF * C * 8, "%d x %d" % (NF, C))
    t = timed(lambda: lib.insc_grid_insert(grid, ptr(c4), I64(P), ptr(sop), ctypes.byref(n_sites), st),
              pre=lambda: lib.insc_grid_clear(grid, st))
    add("hash grid insert (into an empty grid: rows sorted by table partition, partitions built in LDS, scan, assign; incl. count read-back)", t, P * 32, "%d points -> %d sites" % (P, n_sites.value), key="insert")
    t = timed(lambda: lib.insc_grid_query(grid, ptr(c4), I64(P), ptr(sop), st))
    add("hash grid query", t, P * 28, "%d queries" % P, key="query")
    t = timed(lambda: lib.insc_rulebook_ssc3(grid, I64(0), I64(N), ptr(nbr), 0, st))
    add("SSC 3^3 rulebook (dense neighbour map, 27 probes per site)", t, N * (16 + 27 * 8 + 27 * 4), "%d sites" % N, key="ssc")

    def down():
        lib.insc_rulebook_down2(grid, coarse, I64(0), I64(N), ptr(parent), ptr(offset), ptr(child), I64(N), st)

    def down_pre():
        lib.insc_grid_clear(coarse, st)
        child.fill_(-1)

    t = timed(down, pre=down_pre)
    add("stride-2 rulebook (coarse grid insert + parent/offset/child maps)", t, N * 36, "%d fine sites" % N, key="down")
    t = timed(lambda: lib.insc_bn_leaky(ptr(x), I64(C), ptr(y), I64(C), ptr(mean), ptr(var), None, None,
                                         ctypes.c_float(1e-4), ctypes.c_float(0.0), None, None, I64(NF), C, st))
    add("batch norm + ReLU (eval)", t, NF * C * 8, "%d x %d" % (NF, C), key="bn")

    def inp():
        lib.insc_input_accumulate(ptr(fp), I64(P), C, ptr(sop), 4, ptr(acc), ptr(cnt), I64(N), st)
        lib.insc_input_finish(ptr(acc), ptr(cnt), 4, ptr(y), I64(C), None, None, I64(N), C, st)

    def inp_pre():
        acc.zero_()
        cnt.zero_()

    t = timed(inp, pre=inp_pre)
    add("input layer (mode 4: per-voxel mean)", t, P * (4 * C + 4) + N * 4 * C, "%d points x %d -> %d sites" % (P, C, N), key="input")
    t = timed(lambda: lib.insc_output_gather(ptr(y), I64(C), ptr(sop), I64(P), C, ptr(outp), st))
    add("output layer (row gather)", t, P * (4 * C + 4) + P * 4 * C, "%d points x %d" % (P, C), key="output")
    # label fusion: one frame of 20-class scores folded into the per-voxel (label, confidence) table
    NCLS = 20
    table = ctypes.c_void_p()
    lib.insc_labels_create(I64(2 * N), 0, ctypes.c_float(5.0), ctypes.byref(table))
    scores = torch.rand(P, NCLS, device=device)
    lib.insc_labels_update(table, ptr(c4), ptr(scores), I64(NCLS), I64(P), NCLS, st)  # the voxels exist from here on
    t = timed(lambda: lib.insc_labels_update(table, ptr(c4), ptr(scores), I64(NCLS), I64(P), NCLS, st))
    add("label fusion update (argmax + per-voxel confidence rule)", t, P * (16 + 4 * NCLS + 12) + N * 16,
        "%d points x %d classes -> %d voxels" % (P, NCLS, N), key="labels")
    lib.insc_labels_destroy(table)
    lib.insc_grid_destroy(grid)
    lib.insc_grid_destroy(coarse)
    return rows


# ---------------------------------------------------------------------------------------------
# workloads 4 and 5: the U-Net of the reference's example, through the network executor
# ---------------------------------------------------------------------------------------------
def unet_only(device):
    from workloads.netdefs import NaiveUNet

    return NaiveUNet(m=32, levels=7, seed=4).to(device)


def unet_model(device):
    import sparseconvnet as scn

    model = unet_only(device)
    return model, scn.compile(model.sparseModel, capacity_sites=1 << 18)


def residual_row(model, seq, frames, last, device):
    """For comparison: the reference's own incremental mode (residual features on the frame's sites
    only - an approximation), frame `last` of the sweep against the scene of all earlier frames.
    Its saved state never changes, so the same frame is simply repeated."""
    import numpy as np
    import torch

    import sparseconvnet as scn

    rnet = scn.compile(model.sparseModel, capacity_sites=1 << 18, residual=True)
    seen = to_dev(np.concatenate([p for p, _ in seq[:last]]), np.concatenate([c for _, c in seq[:last]]), device)
    with torch.no_grad():
        rnet(seen, increment=False)
        for _ in range(3):
            model.linear(rnet(frames[last], increment="residual"))
        torch.cuda.synchronize()
        rt = []
        for _ in range(20):
            t1 = time.perf_counter()
            model.linear(rnet(frames[last], increment="residual"))
            torch.cuda.synchronize()
            rt.append((time.perf_counter() - t1) * 1e3)
    return {"residual_frame_ms": round(float(np.median(rt)), 3),
            "residual_frame_note": "reference-style residual frame (Incre_* semantics, approximate), %d points on "
                                   "the %d-voxel saved scene, median of 20"
                                   % (len(seq[last][0]), rnet.sites_per_level()[0])}


def time_sweep(call, frames, first):
    """Frame 0 as a full forward, frames 1 .. first-1 untimed, the rest timed back to back with one
    synchronisation per frame.  `call(frame, increment)` runs one frame including the classifier.
    Returns (per-frame ms of the timed frames, their total in seconds)."""
    import torch

    with torch.no_grad():
        call(frames[0], False)
        for f in range(1, first):
            call(frames[f], True)
        torch.cuda.synchronize()
        per_frame = []
        t0 = time.perf_counter()
        for f in range(first, len(frames)):
            t1 = time.perf_counter()
            call(frames[f], True)
            torch.cuda.synchronize()
            per_frame.append((time.perf_counter() - t1) * 1e3)
        dt = time.perf_counter() - t0
    return per_frame, dt


def sweep_phases(call, net, frames, first):
    """The timed frames once more with the executor's phase events on (five event records per frame):
    median milliseconds per phase - structure (grids, maps, orders, tile plans of the frame's new sites,
    input features), dirty (the sets of rows to recompute), layers, output (rows of the frame's points)."""
    import numpy as np
    import torch

    rows = []
    with torch.no_grad():
        call(frames[0], False)
        for f in range(1, first):
            call(frames[f], True)
        net.profile(True)
        for f in range(first, len(frames)):
            call(frames[f], True)
            torch.cuda.synchronize()
            ph = net.profile(True)
            if ph:
                rows.append(ph)
        net.profile(False)
    return {k: round(float(np.median([r[k] for r in rows])), 3) for k in rows[0]} if rows else None


def to_host_long(pts, rgb, device):
    """A frame as the reference's callers hand it over (ioLayers.py:52-69): coordinates as a CPU
    LongTensor [P,3], features on the GPU, batch size 1."""
    import numpy as np
    import torch

    return [torch.from_numpy(pts[:, :3].astype(np.int64)), torch.from_numpy(rgb).to(device), 1]


def target_frame_rows(model, net, device, reps=10):
    """The frame the latency target is stated on: a full forward over the first 145 000 voxels of the
    room (untimed), then ONE incremental frame of 5 000 new voxels + 1 500 re-observed ones (timed,
    classifier included); median of `reps` such pairs.  Once with the re-observed voxels drawn from
    the whole scene (as in the sweep) and once from the part of the scene nearest the new voxels."""
    import numpy as np
    import torch

    from workloads import scenes

    out = {}
    for key, old_from in (("frame_5k_on_150k_ms", "scene"), ("frame_5k_on_150k_frontier_ms", "frontier")):
        (p0, c0), (p1, c1) = scenes.target_frame(old_from=old_from)
        base, frame = to_dev(p0, c0, device), to_dev(p1, c1, device)
        ts = []
        with torch.no_grad():
            for _ in range(reps + 2):
                net(base, increment=False)
                torch.cuda.synchronize()
                t1 = time.perf_counter()
                model.linear(net(frame, increment=True))
                torch.cuda.synchronize()
                ts.append((time.perf_counter() - t1) * 1e3)
        if net.n_sites != 150000:
            sys.exit("bench.py: the target frame ended on %d voxels, not 150 000" % net.n_sites)
        out[key] = round(float(np.median(ts[2:])), 3)
        if old_from == "scene":
            out["frame_5k_on_150k_dirty_rows"] = [
                {"scale": l, "sites": int(net.sites_per_level()[l]), "min": min(r for _, r in sets),
                 "max": max(r for _, r in sets)} for l, sets in enumerate(net.dirty_rows()) if sets]
            out["frame_5k_on_150k_work"] = frame_work_summary(net, out[key])
    out["frame_5k_on_150k_note"] = ("full forward over 145 000 voxels (untimed), then one incremental frame of 5 000 new "
                                    "voxels + 1 500 re-observed voxels (6 500 points), classifier included; median of %d; "
                                    "'_frontier': the re-observed voxels come from the 10 %% of the scene nearest the new "
                                    "ones instead of from anywhere in it" % reps)
    return out


def frame_work_summary(net, frame_ms):
    """Flop accounting of the frame the executor ran last (insc_net_frame_work): useful flops =
    2 * rules * Cin * Cout summed over its convolutions, issued = 2 * 32 * (offsets used per 32-row
    tile) * Cin * Cout (what the matrix cores are handed, empty rule slots included; the 3-channel
    stem runs on the vector units and counts as issued = useful), both over the whole frame's
    wall time against the fp32 MFMA peak."""
    useful = issued = 0.0
    by_scale = {}
    for w in net.frame_work():
        u = 2.0 * w["rules"] * w["cin"] * w["cout"]
        up32 = lambda c: (c + 31) // 32 * 32
        i = 2.0 * w["slots"] * up32(w["cin"]) * up32(w["cout"]) if w["cin"] >= 16 else u
        useful += u
        issued += i
        b = by_scale.setdefault(w["level"], [0.0, 0.0, 0])
        b[0] += u
        b[1] += i
        b[2] += 1
    t = frame_ms * 1e-3
    return {"useful_gflop": round(useful / 1e9, 2), "issued_gflop": round(issued / 1e9, 2),
            "useful_tflops": round(useful / t / 1e12, 2), "issued_tflops": round(issued / t / 1e12, 2),
            "useful_frac_of_fp32_mfma_peak": round(useful / t / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4),
            "issued_frac_of_fp32_mfma_peak": round(issued / t / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4),
            "rule_slot_fill": round(useful / issued, 3) if issued else None,
            "by_scale": [{"scale": l, "convolutions": b[2], "useful_gflop": round(b[0] / 1e9, 2),
                          "issued_gflop": round(b[1] / 1e9, 2)} for l, b in sorted(by_scale.items())],
            "note": "whole frame: structure, dirty sets, all layers and the classifier are inside the time"}


def to_dev(pts, rgb, device):
    import numpy as np
    import torch

    return [torch.from_numpy(pts.astype(np.int32)).to(device), torch.from_numpy(rgb).to(device), 1]


def cpu_baseline_unet():
    """The CPU oracle running the same U-Net as a FULL forward over the final 150k-voxel scene
    (the reference's CPU path has no incremental mode, so this is what one frame costs there)."""
    import numpy as np
    import torch

    from oracle import oracle_net
    from workloads import scenes
    from workloads.netdefs import NaiveUNet
    from oracle import oracle as orc

    pts, rgb, _ = scenes.unet_scene()
    model = NaiveUNet(m=32, levels=7, seed=4)
    t0 = time.perf_counter()
    feats = oracle_net.forward(model.sparseModel, [pts, rgb, 1])
    with torch.no_grad():
        model.linear(torch.from_numpy(np.ascontiguousarray(feats)))
    dt = time.perf_counter() - t0
    return {
        "value": round(dt * 1e3, 1), "unit": "ms/frame", "cores": orc.num_threads(), "kind": "port",
        "sample": "one full U-Net forward (rulebooks + 53 SSC + 6 conv + 6 deconv + 65 BN) over the final "
                  "150k-voxel scene of the sweep, 165k points; the reference CPU path has no incremental mode.  "
                  "A port, not the reference's speed: the per-offset contraction is a plain OpenMP loop nest where "
                  "the reference calls at::mm (CPU/Convolution.cpp:131-147)",
    }


def cpu_baseline_ssc(n_sample=100000):
    import numpy as np

    from workloads import scenes
    from oracle import oracle as orc

    vox = scenes.indoor_scene(seed=3, n=500000)[:n_sample]
    _, sc, _ = orc.grid_build(vox)
    _, counts, pairs = orc.ssc_rules(sc)
    rng = np.random.default_rng(0)
    t_total, convs = 0.0, 0
    for C in (32, 64):
        x = rng.normal(size=(len(sc), C)).astype(np.float32)
        W = (rng.normal(size=(27, C, C)) * 0.05).astype(np.float32)
        mean, var = np.zeros(C, np.float32), np.ones(C, np.float32)
        orc.conv_forward(x, W, None, pairs, counts, len(sc))  # warm-up
        best = 1e30
        for _ in range(3):
            t0 = time.perf_counter()
            y, _ = orc.conv_forward(x, W, None, pairs, counts, len(sc))
            orc.bn_forward(y, mean, var, None, None, 1e-4, 0.0)
            best = min(best, time.perf_counter() - t0)
        t_total += best
        convs += 1
    return {
        "value": round(len(sc) * convs / t_total / 1e6, 3), "unit": "Msites/s", "cores": orc.num_threads(),
        "kind": "port",
        "sample": "first %d voxels of the workload-3 scene, one SSC(3)+BN+ReLU pair at C=32 and one at C=64"
                  % len(sc),
    }


# ---------------------------------------------------------------------------------------------
# workloads 1 and 2: one convolution against the CPU oracle; the integer structures
# ---------------------------------------------------------------------------------------------
def cfg1_workload(device, K, W):
    """One SubmanifoldConvolution(3), 16 -> 16, on the 20k-voxel box scene in 128^3."""
    import numpy as np
    import torch

    import sparseconvnet as scn
    from oracle import oracle as orc
    from sparseconvnet import SCN
    from workloads import scenes

    vox = scenes.boxes_scene(seed=1, n=20000)
    rng = np.random.default_rng(1)
    f = rng.normal(size=(len(vox), 16)).astype(np.float32)
    Wt = (rng.normal(size=(27, 16, 16)) * (2.0 / 16 / 27) ** 0.5).astype(np.float32)
    size = torch.LongTensor([128, 128, 128])
    x = scn.InputLayer(3, size, mode=4)([torch.from_numpy(vox.astype(np.int64)), torch.from_numpy(f).to(device), 1])
    m = x.metadata
    sc = m.ssc_rulebook(size)
    plan = m.ssc_plan(sc)
    w = torch.from_numpy(Wt).to(device)
    out = torch.empty((sc.n, 16), device=device)
    for _ in range(W):
        SCN.ssc_rows_planned(x.features, out, w, None, sc, plan)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(K):
        SCN.ssc_rows_planned(x.features, out, w, None, sc, plan)
    e1.record()
    torch.cuda.synchronize()
    t = e0.elapsed_time(e1) * 1e-3 / K
    # the oracle on the same sites (same numbering: first appearance), timed on the host cores
    _, osc, _ = orc.grid_build(vox)
    _, counts, pairs = orc.ssc_rules(osc)
    orc.conv_forward(f, Wt, None, pairs, counts, len(osc))
    best = 1e30
    for _ in range(5):
        t0 = time.perf_counter()
        ref, _ = orc.conv_forward(f, Wt, None, pairs, counts, len(osc))
        best = min(best, time.perf_counter() - t0)
    got = out.cpu().numpy()
    err = np.abs(got - ref)
    rel = err / np.maximum(np.abs(ref), 1e-3)
    n_rules = int(counts.sum())
    info = {"hip_us": round(t * 1e6, 2), "oracle_ms": round(best * 1e3, 3), "oracle_threads": orc.num_threads(),
            "max_abs_err": float(err.max()), "max_rel_err": float(rel.max()),
            "max_rel_err_note": "relative to max(|reference|, 1e-3)",
            "within_1e-4_rel_1e-5_abs": bool((err <= 1e-5 + 1e-4 * np.abs(ref)).all()),
            "sites": int(sc.n), "rules": n_rules}
    return t, info


def cfg2_workload(device, K, W):
    """Hash grid + rulebooks of the 200k-voxel scene in 1024^3, timed per C call and compared with the
    CPU oracle bit for bit in the same run."""
    import ctypes

    import numpy as np
    import torch

    from oracle import oracle as orc
    from sparseconvnet._lib import lib, ptr, stream_ptr
    from workloads import scenes

    I64 = ctypes.c_int64
    st = stream_ptr()
    rng = np.random.default_rng(2)
    vox = scenes.planes_boxes_scene(seed=2, n=200000).astype(np.int32)
    pts = np.concatenate([vox, vox[rng.integers(0, len(vox), len(vox) // 10)]])
    pts = np.ascontiguousarray(pts[rng.permutation(len(pts))][:, :4])
    P, N = len(pts), len(vox)
    c4 = torch.from_numpy(pts).to(device)
    sop = torch.empty(P, dtype=torch.int32, device=device)
    q = torch.empty(P, dtype=torch.int32, device=device)
    grid, coarse = ctypes.c_void_p(), ctypes.c_void_p()
    lib.insc_grid_create(I64(2 * N), ctypes.byref(grid))
    lib.insc_grid_create(I64(N), ctypes.byref(coarse))
    n_sites = I64(0)
    nbr = torch.empty((N, 27), dtype=torch.int32, device=device)
    parent = torch.empty(N, dtype=torch.int32, device=device)
    offset = torch.empty(N, dtype=torch.int32, device=device)
    child = torch.empty((N, 8), dtype=torch.int32, device=device)

    def timed(fn, pre=None):
        for _ in range(W):
            if pre:
                pre()
            fn()
        torch.cuda.synchronize()
        total = 0.0
        for _ in range(K):
            if pre:
                pre()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            total += e0.elapsed_time(e1)
        return total * 1e-3 / K

    t_ins = timed(lambda: lib.insc_grid_insert(grid, ptr(c4), I64(P), ptr(sop), ctypes.byref(n_sites), st),
                  pre=lambda: lib.insc_grid_clear(grid, st))
    t_qry = timed(lambda: lib.insc_grid_query(grid, ptr(c4), I64(P), ptr(q), st))
    t_ssc = timed(lambda: lib.insc_rulebook_ssc3(grid, I64(0), I64(N), ptr(nbr), 0, st))

    def down_pre():
        lib.insc_grid_clear(coarse, st)
        child.fill_(-1)

    t_dn = timed(lambda: lib.insc_rulebook_down2(grid, coarse, I64(0), I64(N), ptr(parent), ptr(offset), ptr(child),
                                                 I64(N), st), pre=down_pre)
    nc = I64(0)
    lib.insc_grid_size(coarse, ctypes.byref(nc), st)
    # bit-exactness against the oracle (ids are comparable as they are: both number by first appearance)
    o_sop, o_sc, _ = orc.grid_build(pts)
    o_nbr, _, _ = orc.ssc_rules(o_sc)
    o_parent, o_off, o_cc = orc.down2_rules(o_sc)
    coords = torch.empty((N, 4), dtype=torch.int32, device=device)
    ccoords = torch.empty((nc.value, 4), dtype=torch.int32, device=device)
    hip = ctypes.CDLL("libamdhip64.so")
    torch.cuda.synchronize()
    ok_copy = hip.hipMemcpy(ctypes.c_void_p(coords.data_ptr()), ctypes.c_void_p(lib.insc_grid_coords(grid)),
                            ctypes.c_size_t(N * 16), 3) == 0
    ok_copy = ok_copy and hip.hipMemcpy(ctypes.c_void_p(ccoords.data_ptr()),
                                        ctypes.c_void_p(lib.insc_grid_coords(coarse)),
                                        ctypes.c_size_t(nc.value * 16), 3) == 0
    checks = {
        "site_of_point": bool(np.array_equal(sop.cpu().numpy(), o_sop)),
        "query": bool(np.array_equal(q.cpu().numpy(), o_sop)),
        "site_coords": bool(ok_copy and np.array_equal(coords.cpu().numpy(), o_sc)),
        "ssc_neighbour_map": bool(np.array_equal(nbr.cpu().numpy(), o_nbr)),
        "down2_parent": bool(np.array_equal(parent.cpu().numpy(), o_parent)),
        "down2_offset": bool(np.array_equal(offset.cpu().numpy(), o_off)),
        "coarse_coords": bool(ok_copy and np.array_equal(ccoords.cpu().numpy(), o_cc)),
    }
    lib.insc_grid_destroy(grid)
    lib.insc_grid_destroy(coarse)
    ssc_bytes = N * (16 + 27 * 8 + 27 * 4)
    info = {"points": P, "sites": int(n_sites.value), "coarse_sites": int(nc.value),
            "insert_us": round(t_ins * 1e6, 1), "Minserts_per_s": round(P / t_ins / 1e6, 1),
            "insert_GB/s": round(P * 32 / t_ins / 1e9, 1),
            "query_us": round(t_qry * 1e6, 1), "Mqueries_per_s": round(P / t_qry / 1e6, 1),
            "query_GB/s": round(P * 28 / t_qry / 1e9, 1),
            "ssc_rulebook_us": round(t_ssc * 1e6, 1), "ssc_rulebook_GB/s": round(ssc_bytes / t_ssc / 1e9, 1),
            "ssc_rulebook_frac_of_hbm_peak": round(ssc_bytes / t_ssc / 1e9 / HBM_PEAK_GBS, 4),
            "down2_rulebook_us": round(t_dn * 1e6, 1), "down2_rulebook_GB/s": round(N * 36 / t_dn / 1e9, 1),
            "bit_exact": bool(all(checks.values())), "bit_exact_checks": checks}
    return t_ins + t_qry + t_ssc + t_dn, info


def cpu_baseline_cfg2():
    import numpy as np

    from oracle import oracle as orc
    from workloads import scenes

    rng = np.random.default_rng(2)
    vox = scenes.planes_boxes_scene(seed=2, n=200000).astype(np.int32)
    pts = np.concatenate([vox, vox[rng.integers(0, len(vox), len(vox) // 10)]])
    pts = np.ascontiguousarray(pts[rng.permutation(len(pts))][:, :4])
    best = 1e30
    for _ in range(3):
        t0 = time.perf_counter()
        _, sc, _ = orc.grid_build(pts)
        orc.ssc_rules(sc)
        orc.down2_rules(sc)
        best = min(best, time.perf_counter() - t0)
    return {"value": round(len(pts) / best / 1e6, 3), "unit": "Mpoints/s", "cores": orc.num_threads(), "kind": "port",
            "sample": "the whole workload: grid build of %d points + 3^3 rulebook + stride-2 rulebook, best of 3"
                      % len(pts)}



def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default="incr", choices=["incr", "unet", "ssc", "cfg1", "cfg2"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-residual", action="store_true",
                    help="skip the residual-frame comparison row of the incremental workload")
    ap.add_argument("--residual-only", action="store_true",
                    help="run only the residual-frame comparison row (short; used under rocprofv3)")
    ap.add_argument("--kernels-only", action="store_true",
                    help="print only the table of bandwidth-bound kernels")
    ap.add_argument("--roofline-only", action="store_true",
                    help="run only the dominant-kernel measurement (short; used under rocprofv3)")
    ap.add_argument("--wide-only", action="store_true",
                    help="run only the 64-channel layer at 500k voxels (short; used under rocprofv3)")
    ap.add_argument("--split-only", action="store_true",
                    help="run only the 96-channel layer at the third scale of the U-Net scene (short; used under rocprofv3)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the roofline, wide-layer and kernel-table rows (used under rocprofv3)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collectives, no sharding)"
                 % args.gpus)
    import numpy as np
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)

    if args.kernels_only:
        print(json.dumps({"kernels": kernel_table(device, strict=False)}))
        return
    if args.residual_only:
        from workloads import scenes

        seq = scenes.sweep_sequence()
        model, _ = unet_model(device)
        frames = [to_dev(p, c, device) for p, c in seq]
        print(json.dumps(residual_row(model, seq, frames, len(seq) - 1, device)))
        return
    if args.wide_only:
        print(json.dumps({"wide_layer": wide_conv_row(device)}))
        return
    if args.split_only:
        print(json.dumps({"split_layer": split_layer_row(device)}))
        return
    if args.roofline_only:
        # plus a plain copy of known size (500k x 32 floats: 64 MB read, 64 MB written), the
        # yardstick the FETCH_SIZE / WRITE_SIZE counters of the same run are scaled by
        from sparseconvnet import SCN

        a = torch.randn(500000, 32, device=device)
        b = torch.empty_like(a)
        for _ in range(5):
            SCN.copy_rows(a, b, None, None, a.size(0))
        torch.cuda.synchronize()
        print(json.dumps({"roofline": conv_roofline(device)}))
        return

    extra = {}
    if args.workload == "incr":
        from workloads import scenes

        seq = scenes.sweep_sequence()
        n_inc = len(seq) - 1  # incremental frames of the sweep (frame 0 is the full forward)
        W = 5 if args.warmup is None else args.warmup
        K = 20 if args.steps is None else args.steps
        if K < 1 or K > 40 or W < 0 or W + K > n_inc:
            sys.exit("bench.py: the sweep has %d incremental frames and the LAST --steps of them are timed (the "
                     "scene must have grown to 150k voxels): need 1 <= steps <= 40 and warmup + steps <= %d"
                     % (n_inc, n_inc))
        first = n_inc - K + 1  # first timed frame; frames 1 .. first - 1 (at least W of them) are untimed
        import sparseconvnet as scn

        model, net = unet_model(device)
        frames = [to_dev(p, c, device) for p, c in seq]
        # the logits of a frame's points = Linear(features of those points)
        per_frame, dt = time_sweep(lambda x, inc: model.linear(net(x, increment=inc)), frames, first)
        if net.n_sites != 150000:
            sys.exit("bench.py: the sweep ended on %d voxels, not on the 150 000 the metric names" % net.n_sites)
        seen = np.unique(np.concatenate([p for p, _ in seq[:first]]), axis=0)
        sites_at_start = int(len(seen))
        new_per_frame = []
        have = set(map(tuple, seen[:, :3].tolist()))
        for f in range(first, n_inc + 1):
            pts = set(map(tuple, seq[f][0][:, :3].tolist()))
            new_per_frame.append(len(pts - have))
            have |= pts
        ms = dt * 1e3 / K
        value, metric, unit, hib = round(ms, 3), "incremental frame latency ms (UNet, 150k vox)", "ms", False
        config = {"workload": "cfg5: the last %d incremental U-Net frames (%d..%d) of the 50-frame sweep (m=32, 7 "
                              "levels, InputLayer mode 4 .. OutputLayer + Linear(32,20)); frames 0..%d untimed; the "
                              "scene grows from %d to 150 000 voxels over the timed frames.  The sweep's draws of "
                              "3k-8k new voxels per frame are scaled so that 50 frames end on 150 000 voxels: a "
                              "timed frame really adds %d-%d new voxels (mean %d) plus 1k-2k re-observed ones; "
                              "the frame the latency target names (5 000 new voxels onto a scene that then has "
                              "150 000) is measured separately: frame_5k_on_150k_ms"
                              % (K, first, n_inc, first - 1, sites_at_start, min(new_per_frame), max(new_per_frame),
                                 int(np.mean(new_per_frame))),
                  "points_per_frame_mean": int(np.mean([len(seq[f][0]) for f in range(first, n_inc + 1)])),
                  "new_voxels_per_frame_mean": int(np.mean(new_per_frame)),
                  "points_last_frame": int(len(seq[n_inc][0])),
                  "sites_at_start": sites_at_start, "sites_at_end": net.n_sites,
                  "order_refresh": "library default: an incremental frame re-sorts the processing orders of its "
                                   "scales once 10 % of a large scale has been appended (several of the timed "
                                   "frames do)",
                  "sites_per_level_at_end": net.sites_per_level()[:7]}
        extra = {"frame_at_150k_ms": round(per_frame[-1], 3),
                 "median_ms": round(float(np.median(per_frame)), 3),
                 "p95_ms": round(float(np.percentile(per_frame, 95)), 3),
                 "first_timed_frame_ms": round(per_frame[0], 3)}
        # rows the last timed frame recomputed: per scale, the smallest and the largest dirty set
        # among the tensors of that scale, beside the scale's sites
        sites = net.sites_per_level()
        extra["dirty_rows_last_frame"] = [
            {"scale": l, "sites": int(sites[l]), "min": min(r for _, r in sets), "max": max(r for _, r in sets)}
            for l, sets in enumerate(net.dirty_rows()) if sets]
        # flop accounting of the last timed frame against the fp32 MFMA peak (the frame is bound by
        # matrix-core issue at the coarse scales, not by HBM)
        extra["frame"] = frame_work_summary(net, per_frame[-1])
        extra["frame_phases_ms"] = sweep_phases(lambda x, inc: model.linear(net(x, increment=inc)), net, frames, first)
        if not args.no_extras:
            # (a) the same frames through the reference's own call path: model(x, increment) on the module
            # tree with CPU int64 coordinates (model.py:23-26, ioLayers.py:52-69); the whole-network
            # Sequential hands them to the executor by itself.  (b) the explicit executor fed the same
            # host coordinates.  (c) the module tree layer by layer (one C call per layer from Python).
            hframes = [to_host_long(p, c, device) for p, c in seq]
            model_b = unet_only(device)
            pf, _ = time_sweep(lambda x, inc: model_b(x, increment=inc), hframes, first)
            extra["module_api_frame_ms"] = round(float(np.mean(pf)), 3)
            extra["module_api_frame_at_150k_ms"] = round(pf[-1], 3)
            if model_b.sparseModel.why_not_compiled() is not None or "_exec" not in model_b.sparseModel.__dict__:
                sys.exit("bench.py: the module path did not reach the executor: %s" % model_b.sparseModel.why_not_compiled())
            pf, _ = time_sweep(lambda x, inc: model.linear(net(x, increment=inc)), hframes, first)
            extra["executor_cpu_coords_frame_ms"] = round(float(np.mean(pf)), 3)
            prev = scn.set_auto_compile(False)
            try:
                model_c = unet_only(device)
                pf, _ = time_sweep(lambda x, inc: model_c(x, increment=inc), hframes, first)
            finally:
                scn.set_auto_compile(prev)
            extra["module_api_layer_by_layer_frame_ms"] = round(float(np.mean(pf)), 3)
            extra["module_api_note"] = ("the same %d frames, mean ms per frame, classifier included: module_api = "
                                        "model([coords int64 on the HOST [P,3], features on the GPU, 1], increment) on "
                                        "the module tree, as a user of the reference calls it (the Sequential traces "
                                        "itself into the executor at its first frame); executor_cpu_coords = the explicit "
                                        "scn.compile() object fed the same host coordinates; layer_by_layer = the module "
                                        "tree with the executor switched off (one C call per layer from Python); "
                                        "`value` = the executor fed int32 device coordinates" % K)
            del model_b, model_c
            # (d) full forward over the whole 150k-voxel scene (workload 4), same executor: what a frame
            # costs without the incremental path
            pts4, rgb4, _ = scenes.unet_scene()
            x4 = to_dev(pts4, rgb4, device)
            with torch.no_grad():
                for _ in range(3):
                    model.linear(net(x4, increment=False))
                torch.cuda.synchronize()
                t1 = time.perf_counter()
                for _ in range(10):
                    model.linear(net(x4, increment=False))
                torch.cuda.synchronize()
                extra["full_forward_ms"] = round((time.perf_counter() - t1) * 100.0, 3)
            extra["full_forward_note"] = ("full U-Net forward over the 150 000-voxel scene (165 000 points), mean of 10: an "
                                          "incremental frame of this sweep dirties every row from the second scale on, so "
                                          "it saves the structure phase and part of the input scale, not the layers")
            # (e) the frame the latency target is stated on
            extra.update(target_frame_rows(model, net, device))
        if not args.no_residual:
            extra.update(residual_row(model, seq, frames, n_inc, device))
        cpu_fn = cpu_baseline_unet
    elif args.workload == "unet":
        from workloads import scenes

        W = 3 if args.warmup is None else args.warmup
        K = 20 if args.steps is None else args.steps
        pts, rgb, _ = scenes.unet_scene()
        model, net = unet_model(device)
        x = to_dev(pts, rgb, device)
        with torch.no_grad():
            for _ in range(W):
                model.linear(net(x, increment=False))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(K):
                model.linear(net(x, increment=False))
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
        ms = dt * 1e3 / K
        value, metric, unit, hib = round(ms, 3), "full U-Net forward ms (150k vox)", "ms", False
        config = {"workload": "cfg4: full U-Net forward (grid + rulebooks + all layers), 150k voxels / 165k points",
                  "sites_per_level": net.sites_per_level()[:7]}
        cpu_fn = cpu_baseline_unet
    elif args.workload == "cfg1":
        W = 50 if args.warmup is None else args.warmup
        K = 200 if args.steps is None else args.steps
        t, info = cfg1_workload(device, K, W)
        ms = t * 1e3
        value, metric, unit, hib = round(info["sites"] / t / 1e6, 1), "SSC Msites/s", "Msites/s", True
        config = {"workload": "cfg1: one SubmanifoldConvolution(3) 16->16 on 20 000 voxels (faces of 8 boxes in 128^3)"}
        extra = {"cfg1": info}
        cpu_fn = lambda: {"value": round(info["sites"] / (info["oracle_ms"] * 1e-3) / 1e6, 3), "unit": "Msites/s",
                          "cores": info["oracle_threads"], "kind": "port",
                          "sample": "the whole workload (one convolution over the 20k-voxel scene), best of 5"}
    elif args.workload == "cfg2":
        W = 2 if args.warmup is None else args.warmup
        K = 20 if args.steps is None else args.steps
        t, info = cfg2_workload(device, K, W)
        ms = t * 1e3
        value, metric, unit, hib = info["Minserts_per_s"], "hash grid Minserts/s", "Minserts/s", True
        config = {"workload": "cfg2: hash grid insert of 200 000 voxels in 1024^3 (+10 % repeated points), query, 3^3 "
                              "rulebook, stride-2 size-2 rulebook; one step = the four calls"}
        extra = {"cfg2": info}
        cpu_fn = cpu_baseline_cfg2
    else:
        W = 3 if args.warmup is None else args.warmup
        K = 20 if args.steps is None else args.steps
        step, info, _ = ssc_workload(device)
        for _ in range(W):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(K):
            step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ms = dt * 1e3 / K
        value = round(info["sites"] * info["convs_per_step"] / (dt / K) / 1e6, 1)
        metric, unit, hib = "SSC Msites/s", "Msites/s", True
        config = {"workload": "cfg3: 4x[SSC(3)+BN+ReLU] at 500k voxels, C=32 then C=64 (8 convs/step)",
                  "sites": info["sites"], "rules": info["rules"]}
        cpu_fn = cpu_baseline_ssc

    out = {
        "metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms, 4), "higher_is_better": hib, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic", "config": config,
    }
    out.update(extra)
    if args.workload in ("cfg1", "cfg2"):  # small side workloads: the roofline rows belong to the main ones
        if not args.no_cpu_baseline:
            out["cpu_baseline"] = cpu_fn()
        print(json.dumps(out))
        return
    if not args.no_extras:
        out["roofline"] = conv_roofline(device)
        out["wide_layer"] = wide_conv_row(device)
        if args.workload in ("incr", "unet"):
            out["split_layer"] = split_layer_row(device)
        out["kernels"] = kernel_table(device)
    # the CPU leg comes last: the GPU idles during it, and a measurement taken right after would
    # start at idle clocks
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_fn()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
