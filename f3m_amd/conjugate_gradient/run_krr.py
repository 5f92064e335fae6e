"""FALKON kernel ridge regression on a synthetic problem (the fifth benchmark configuration of this project).

    python -m f3m_amd.conjugate_gradient.run_krr --n 10000000 --m 100000 --maxiter 20

X ~ U[-1,1]^3, y = sin(3 x1) cos(2 x2) + x3^2 + 0.1 N(0,1), M uniformly chosen Nystrom centres, Gaussian
kernel with ls = 0.5, penalty 1e-6; every K_nm / K_nm^T product goes through the F3M engine in fp32.
Prints one JSON line with the timings and the R^2 of the fit (reference protocol:
experiments/experiments_krr_a.py:19-23,49-97)."""
import argparse
import json
import time

import torch

from . import FalkonOptions, custom_Falkon, custom_GaussianKernel


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--n", type=float, default=1e7)
    ap.add_argument("--m", type=float, default=1e5)
    ap.add_argument("--ls", type=float, default=0.5)
    ap.add_argument("--penalty", type=float, default=1e-6)
    ap.add_argument("--maxiter", type=int, default=20)
    ap.add_argument("--nodes", type=int, default=64)
    ap.add_argument("--var-compression", action="store_true")
    ap.add_argument("--pc-dtype", default="float64", choices=["float32", "float64"])
    ap.add_argument("--pc-blocked", default="auto", choices=["auto", "yes", "no"],
                    help="tile-by-tile fp32 preconditioner (auto: when a whole matrix would exceed the limit for single "
                         "library calls, as with M = 1e5)")
    ap.add_argument("--pc-block-size", type=int, default=8192)
    ap.add_argument("--products-only", action="store_true",
                    help="time only the two engine products of one CG iteration (no preconditioner, no solve)")
    args = ap.parse_args()
    n, m = int(args.n), int(args.m)
    g = torch.Generator().manual_seed(1)
    X = 2 * torch.rand(n, 3, generator=g) - 1
    y = torch.sin(3 * X[:, 0]) * torch.cos(2 * X[:, 1]) + X[:, 2] ** 2 + 0.1 * torch.randn(n, generator=g)
    X, Y = X.cuda(), y[:, None].cuda()
    opt = FalkonOptions(pc_dtype=getattr(torch, args.pc_dtype), pc_block_size=args.pc_block_size,
                        pc_blocked={"auto": None, "yes": True, "no": False}[args.pc_blocked])
    kernel = custom_GaussianKernel(args.ls, opt=opt, var_compression=args.var_compression, interpolation_nr=args.nodes)
    if args.products_only:
        C = X[torch.randperm(n, generator=g)[:m].cuda()].contiguous()
        v = torch.randn(m, 1, generator=g).cuda()
        torch.cuda.synchronize()
        t0 = time.time()
        kernel.dmmv(X, C, v, None)             # builds the plan, then K_nm v and K_nm^T (.)
        torch.cuda.synchronize()
        t_first = time.time() - t0
        times = []
        for _ in range(5):
            t0 = time.time()
            out = kernel.dmmv(X, C, v, None)
            torch.cuda.synchronize()
            times.append(time.time() - t0)
        print(json.dumps({"n": n, "m": m, "ls": args.ls, "first_dmmv_with_plans_s": t_first,
                          "dmmv_s": [round(t, 4) for t in times], "finite": bool(torch.isfinite(out).all())}))
        return
    model = custom_Falkon(kernel, args.penalty, m, maxiter=args.maxiter, seed=1, options=opt)
    torch.cuda.synchronize()
    t0 = time.time()
    model.fit(X, Y)
    torch.cuda.synchronize()
    t_fit = time.time() - t0
    t0 = time.time()
    pred = model.predict(X)
    torch.cuda.synchronize()
    t_pred = time.time() - t0
    mse = float(((pred - Y) ** 2).mean())
    r2 = 1 - mse / float(((Y - Y.mean()) ** 2).mean())
    print(json.dumps({"n": n, "m": m, "ls": args.ls, "penalty": args.penalty, "cg_iterations": model.cg_iterations_,
                      "preconditioner_s": model.fit_times_[0], "cg_s": model.conjugate_gradient_time,
                      "cg_s_per_iteration": model.conjugate_gradient_time / max(1, model.cg_iterations_),
                      "fit_s": t_fit, "predict_s": t_pred, "mse": mse, "r2": r2,
                      "gpu_peak_allocated_gib": torch.cuda.max_memory_allocated() / 2 ** 30,
                      "mmv_s": [round(t, 4) for t in model_optimizer_times(model)]}))


def model_optimizer_times(model):
    return getattr(model, "mmv_times_", [])


if __name__ == "__main__":
    main()
