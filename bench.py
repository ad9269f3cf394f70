#!/usr/bin/env python3
"""Benchmark of the sparse-convolution inference path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload ssc|unet|incr]

Prints ONE JSON line.  A step is one pass of the hot path over one batch of seeded
synthetic input that is already resident in HBM when the timed region starts:
  ssc  : workload 3 - 4 x [SubmanifoldConvolution(3) + BatchNormReLU] at 500k active voxels,
         once at 32 channels and once at 64 (8 convolutions per step)
  unet : workload 4 - full U-Net forward over a 150k-voxel scene
  incr : workload 5 - one incremental U-Net frame of the 50-frame sweep
The `roofline` object is measured live on the dominant kernel (the submanifold
gather-GEMM-scatter at 500k voxels, 32 channels) with events on the launch stream;
`cpu_baseline` times the CPU oracle (a restatement of the reference's CPU path) on this
machine's host cores over a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests"), os.path.join(ROOT, "ins-conv_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
MFMA_FP32_PEAK_TFLOPS = 157.3


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


def ssc_workload(device):
    """Workload 3: returns (run_step, info)."""
    import numpy as np
    import torch

    import scenes
    import sparseconvnet as scn
    from sparseconvnet import SCN

    vox = scenes.indoor_scene(seed=3, n=500000)
    size = torch.LongTensor([4096, 4096, 4096])
    inp = scn.InputLayer(3, size, mode=4)
    rng = np.random.default_rng(3)
    stacks, xs = [], []
    coords = torch.from_numpy(vox.astype(np.int64))
    for C in (32, 64):
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

    info = {"sites": len(vox), "rules": n_rules, "convs_per_step": 8}
    return step, info, (xs[0], stacks[0])


def conv_roofline(x, stack, n_rules, device, reps=30):
    """Average duration of the 32-channel submanifold convolution kernel and its roofline figures."""
    import torch

    from sparseconvnet import SCN

    conv = stack[0]
    m = x.metadata
    sc = m.ssc_rulebook(x.spatial_size)
    out = torch.empty((sc.n, conv.nOut), device=device)
    w = conv.weight
    for _ in range(3):
        SCN.conv_rows(x.features, out, w, None, sc.nbr.t, 27, sc.order.t, None, sc.n)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        SCN.conv_rows(x.features, out, w, None, sc.nbr.t, 27, sc.order.t, None, sc.n)
    e1.record()
    torch.cuda.synchronize()
    t = e0.elapsed_time(e1) * 1e-3 / reps
    Cin, Cout = conv.nIn, conv.nOut
    # every gathered row read once per rule (+ its two int32 ids), every output row written
    # once, the weights once
    bytes_alg = n_rules * (4 * Cin + 8) + sc.n * 4 * Cout + 27 * Cin * Cout * 4
    flops = 2.0 * n_rules * Cin * Cout
    achieved = bytes_alg / t / 1e9
    return {
        "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
        "kernel": "conv_mfma_kernel<1> (SSC 3^3, 32->32, 500k sites)", "avg_us": round(t * 1e6, 1),
        "algorithmic_bytes": int(bytes_alg),
        "mfma_tflops": round(flops / t / 1e12, 2), "mfma_frac": round(flops / t / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4),
    }


def cpu_baseline_ssc(n_sample=100000):
    """The CPU oracle on a bounded sample of workload 3: one SSC(3)+BN+ReLU pair at 32 and at 64
    channels over the first `n_sample` voxels of the scene."""
    import numpy as np

    import scenes
    from oracle import oracle as orc

    vox = scenes.indoor_scene(seed=3, n=500000)[:n_sample]
    _, sc, _ = orc.grid_build(vox)
    t0 = time.perf_counter()
    _, counts, pairs = orc.ssc_rules(sc)
    t_rules = time.perf_counter() - t0
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
        "sample": "first %d voxels of the workload-3 scene, one SSC(3)+BN+ReLU pair at C=32 and one at C=64 "
                  "(rulebook build %.2f s not included)" % (len(sc), t_rules),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="ssc", choices=["ssc"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--roofline-only", action="store_true",
                    help="run only the dominant-kernel measurement (short; used under rocprofv3)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collectives, no sharding)"
                 % args.gpus)
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)

    step, info, (x0, stack0) = ssc_workload(device)
    if args.roofline_only:
        print(json.dumps({"roofline": conv_roofline(x0, stack0, info["rules"], device, reps=10)}))
        return
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms = dt * 1e3 / args.steps
    msites = info["sites"] * info["convs_per_step"] / (dt / args.steps) / 1e6

    roof = conv_roofline(x0, stack0, info["rules"], device)
    out = {
        "metric": "SSC Msites/s", "value": round(msites, 1), "unit": "Msites/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "cfg3: 4x[SSC(3)+BN+ReLU] at 500k voxels, C=32 then C=64 (8 convs/step)",
                   "sites": info["sites"], "rules": info["rules"]},
        "roofline": roof,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_ssc()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
