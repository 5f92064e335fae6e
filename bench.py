#!/usr/bin/env python3
"""Benchmark of the F3M kernel-matrix-vector product on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--n N] [--dist uniform|normal] [--ls LS]

A step is one complete product out = K(X,X) b through the C ABI (box division + interaction lists +
near field + far field), inputs resident in HBM, like one `FFM(X) @ b` of the reference
(experiments/experiments.py:72-77).  Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_TFLOPS = 157.3      # MI355X fp32 peak
# HBM bytes moved by one near-field launch of the default workload, from the rocprofv3 FETCH_SIZE and
# WRITE_SIZE counter runs summarised in profiles/ (None until measured)
NEAR_TRAFFIC_BYTES = 6.072e9


def cpu_baseline(X, Y, b, ls, budget_s=15.0):
    """Exact tiled PyTorch product on the host cores for a bounded number of target rows against all
    sources (the checker's code, timed only here)."""
    import torch
    from oracle import f3m_oracle as fo
    Xc, bc = X.cpu(), b.cpu()
    Yc = Xc if Y is None else Y.cpu()
    rows = 64
    t0 = time.perf_counter()
    fo.exact_tiled_torch(Xc[:rows], Yc, bc, ls, row_tile=rows, col_tile=1 << 18)
    t1 = time.perf_counter() - t0
    rows2 = int(max(64, min(20000, rows * budget_s / max(t1, 1e-3)))) // 64 * 64
    t0 = time.perf_counter()
    fo.exact_tiled_torch(Xc[:rows2], Yc, bc, ls, row_tile=min(rows2, 256), col_tile=1 << 18)
    t2 = time.perf_counter() - t0
    return {"value": rows2 / t2, "unit": "points/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "%d target rows x all %d sources, exact tiled torch fp32, %.1f s; implied full product %.0f s"
                      % (rows2, Yc.shape[0], t2, Xc.shape[0] / (rows2 / t2)),
            "host_cpu_count": os.cpu_count()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--n", type=int, default=10_000_000)
    ap.add_argument("--d", type=int, default=3)
    ap.add_argument("--dist", default="uniform", choices=["uniform", "normal", "clustered"],
                    help="clustered = the asymmetric benchmark configuration: X from 50 anisotropic Gaussians, Y (n/10 points) uniform over "
                         "X's bounding box, two trees")
    ap.add_argument("--ls", type=float, default=1.0)
    ap.add_argument("--nodes", type=int, default=64)
    ap.add_argument("--subsample", type=int, default=100_000)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-accuracy", action="store_true")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain 1 GiB device copy (a kernel of known HBM traffic, to scale rocprof counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs on ONE GPU (no sharding, no collectives); --gpus %d is not supported. "
              "Run with --gpus 1." % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from f3m_amd import engine

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    g = torch.Generator().manual_seed(1)
    N, d = args.n, args.d
    Y = None
    if args.dist == "clustered":
        mu, sd = 10 * torch.rand(50, d, generator=g), 0.05 + 0.45 * torch.rand(50, d, generator=g)
        comp = torch.arange(N) % 50
        X = (mu[comp] + sd[comp] * torch.randn(N, d, generator=g)).cuda()
        lo, hi = X.min(0).values.cpu(), X.max(0).values.cpu()
        Y = (lo + (hi - lo) * torch.rand(N // 10, d, generator=g)).cuda()
        dist_name = "X: 50 anisotropic Gaussians, Y: %d uniform over the bounding box" % (N // 10)
    else:
        X = (torch.rand(N, d, generator=g) if args.dist == "uniform" else torch.randn(N, d, generator=g)).cuda()
        dist_name = "uniform [0,1]^%d" % d if args.dist == "uniform" else "N(0,I)"
    M = N if Y is None else Y.shape[0]
    b = torch.randn(M, 1, generator=g).cuda()
    prm = dict(ls=args.ls, min_points=1000, nr_of_interpolation=args.nodes, small_field_points=1000)

    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda")
        src.fill_(1.0)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    engine.set_timing(True)
    for _ in range(args.warmup):
        out = engine.kmvm(X, Y, b, **prm)
    torch.cuda.synchronize()
    near_t, near_n, stage = 0.0, 0, {}
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = engine.kmvm(X, Y, b, **prm)
        tm = engine.get_timing()
        near_t += tm["near"][0]
        near_n += tm["near"][1]
        for k, v in tm.items():
            stage[k] = stage.get(k, 0.0) + v[0]
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms = dt / args.steps * 1e3

    plan = engine.Plan(X, Y, **prm)
    work = plan.work()
    depth = plan.depth
    nbx = plan.level_sizes(depth)["nbx"] if depth else 1
    tiles_per_wave = 5 if (N // max(nbx, 1) + 31) // 32 == 5 else 4     # the library's choice (near_field)
    plan.close()
    F = 3 * d + 3                                  # flops per kernel evaluation (d sub, d mul, d-1 add, scale, exp, fma)
    near_flops = F * work["near_pairs"]
    near_per_launch_s = near_t / max(near_n, 1)
    achieved = near_flops * args.steps / max(near_t, 1e-12) / 1e12
    roofline = {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                "frac": achieved / PEAK_FP32_TFLOPS, "traffic": NEAR_TRAFFIC_BYTES if (N == 10_000_000 and d == 3) else None,
                "kernel": "near_g_kernel<%d,%d,1>" % (d, tiles_per_wave),
                "note": "near field: exponents on the f16 matrix pipe (hi/lo-split operands, fp32 accumulate), exp2 + FMA on "
                        "the fp32 vector ALU; priced against the fp32 peak; %d launches/step, %.3f ms per launch, "
                        "%.3e kernel evaluations/step x %d flops; traffic = HBM bytes per launch from rocprofv3 "
                        "FETCH_SIZE + WRITE_SIZE (profiles/)" % (near_n // max(args.steps, 1), near_per_launch_s * 1e3,
                                                               work["near_pairs"], F)}
    res = {
        "metric": "KMVM points/sec at N=1e7 3D Gaussian (1 GPU); rel-L2 error vs fp64 exact",
        "value": N / (dt / args.steps), "unit": "points/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "%dD Gaussian KMVM %s, N=%d %s, b~N(0,1) (%d,1), ls=%g, %d nodes/box, cutoff 1000 "
                               "(BASELINE.json configs[%d])" % (d, "X=Y" if Y is None else "X!=Y", N, dist_name, M, args.ls,
                                                               args.nodes, 2 if Y is not None else (1 if d == 3 else 3)),
                   "N": N, "d": d, "ls": args.ls, "nodes": args.nodes, "tree_depth": depth},
        "roofline": roofline,
        "stage_ms_per_step": {k: v / args.steps * 1e3 for k, v in stage.items()},
        "work": work,
    }
    if not args.no_accuracy:
        rows = torch.from_numpy(np.random.default_rng(1).choice(N, min(args.subsample, N), replace=False)).cuda()
        exact = engine.exact_f64(X[rows].double(), (X if Y is None else Y).double(), b.double(), args.ls)
        diff = (out[rows].double() - exact)
        res["rel_l2_error"] = float(diff.norm() / exact.norm())
        res["rel_l2_rows"] = int(rows.numel())
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(X, Y, b, args.ls)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
