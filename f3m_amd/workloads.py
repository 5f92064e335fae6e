"""Seeded synthetic point clouds of the benchmark configurations (CPU generators, torch.manual_seed-style
streams), shared by bench.py and the full-size GPU tests so that both measure the same inputs.

Every entry of CONFIGS: name -> dict(d, dist, ls, nodes, m_ratio, ...) with
  dist "uniform"   X = scale * rand(N, d)  (scale 1 unless given)   (X = Y)
       "normal"    X = randn(N, d)                                 (X = Y)
       "clustered" X from 50 anisotropic Gaussians, means 10 rand(50, d), per-dimension std 0.05 + 0.45 rand,
                   Y = N / m_ratio points uniform over X's bounding box (two trees)
The reference draws its benchmark clouds the same way (experiments/experiments.py:45-60,115: seed 1, uniform
and normal clouds, b ~ N(0,1))."""
import torch

CONFIGS = {
    "uniform3_ls1": dict(d=3, dist="uniform", ls=1.0, nodes=64),
    "uniform3_ls0.1": dict(d=3, dist="uniform", ls=0.1, nodes=64),
    "uniform3_ls10": dict(d=3, dist="uniform", ls=10.0, nodes=64),
    "normal3_ls1": dict(d=3, dist="normal", ls=1.0, nodes=64),
    "normal3_ls0.1": dict(d=3, dist="normal", ls=0.1, nodes=64),
    "normal3_ls10": dict(d=3, dist="normal", ls=10.0, nodes=64),
    "clustered3_xy_ls0.5": dict(d=3, dist="clustered", ls=0.5, nodes=64, m_ratio=10),
    "uniform4_81nodes": dict(d=4, dist="uniform", ls=1.0, nodes=81),
    "uniform5_243nodes": dict(d=5, dist="uniform", ls=1.0, nodes=243),
}

# The node grids of the reference's own sweep beyond 4^3 (experiments/experiments.py:47-49: node_list = [4, 5, 6]), on
# the headline cloud, and that sweep's own protocol (:41,:50-69): X uniform on [0, sqrt(12 r2)]^3 with r2 = 1,
# ls = 1/sqrt(2), min_points = 1000, small_field_points = nr_of_interpolation, var_compression with
# eff_var_limit = 0.3 d.
NODE_SWEEP = (64, 125, 216)
MORE_CONFIGS = {
    "uniform3_125nodes": dict(d=3, dist="uniform", ls=1.0, nodes=125),
    "uniform3_216nodes": dict(d=3, dist="uniform", ls=1.0, nodes=216),
}
for _n in NODE_SWEEP:
    MORE_CONFIGS["sweep3_varcomp_%dnodes" % _n] = dict(d=3, dist="uniform", scale=12.0 ** 0.5, ls=0.5 ** 0.5, nodes=_n,
                                                      var_compression=True, eff_var_limit=0.9, small_field_points=_n)
ALL_CONFIGS = dict(CONFIGS, **MORE_CONFIGS)

# configurations whose error at 64 nodes per box is above the 1e-3 target (the algorithm's own error there): the
# benchmark also runs them at the larger grids of NODE_SWEEP and reports the smallest that meets the target
NODE_VARIANTS_OF = ("uniform3_ls0.1", "normal3_ls1", "normal3_ls0.1", "clustered3_xy_ls0.5")


def make(name, n, seed=1, columns=1, device="cuda", nodes=None):
    """-> X, Y (None when X = Y), b, engine parameters; tensors on `device`.  nodes: another node count than the
    configuration's own (same cloud, same weights)."""
    cfg = ALL_CONFIGS[name]
    d = cfg["d"]
    g = torch.Generator().manual_seed(seed)
    Y = None
    if cfg["dist"] == "clustered":
        mu, sd = 10 * torch.rand(50, d, generator=g), 0.05 + 0.45 * torch.rand(50, d, generator=g)
        comp = torch.arange(n) % 50
        X = mu[comp] + sd[comp] * torch.randn(n, d, generator=g)
        lo, hi = X.min(0).values, X.max(0).values
        Y = (lo + (hi - lo) * torch.rand(n // cfg["m_ratio"], d, generator=g)).to(device)
        X = X.to(device)
    elif cfg["dist"] == "uniform":
        X = torch.rand(n, d, generator=g)
        if "scale" in cfg:
            X *= cfg["scale"]
        X = X.to(device)
    else:
        X = torch.randn(n, d, generator=g).to(device)
    m = n if Y is None else Y.shape[0]
    b = torch.randn(m, columns, generator=g).to(device)
    prm = dict(ls=cfg["ls"], min_points=1000, nr_of_interpolation=nodes or cfg["nodes"],
               small_field_points=cfg.get("small_field_points", 1000))
    if cfg.get("var_compression"):
        prm.update(var_compression=True, eff_var_limit=cfg["eff_var_limit"])
    return X, Y, b, prm


def describe(name, n):
    cfg = ALL_CONFIGS[name]
    d = cfg["d"]
    if cfg["dist"] == "clustered":
        return "X: %d points from 50 anisotropic Gaussians in %d-D, Y: %d uniform over X's bounding box" % (n, d, n // cfg["m_ratio"])
    return "%d points %s, X = Y" % (n, "uniform [0,%.4g]^%d" % (cfg.get("scale", 1), d) if cfg["dist"] == "uniform" else "N(0,I_%d)" % d)
