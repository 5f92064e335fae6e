"""Independent numpy restatements used to pin the oracle (and, through it, the HIP engine)."""
import numpy as np

f32 = np.float32


def cell_coords(X, origin, edge0, k):
    """Integer cell of every point at depth k: floor(fl(fl(2^k * fl(x-origin)) / edge0)) in fp32."""
    a = (X.astype(f32) - origin.astype(f32)).astype(f32)
    q = (f32(2.0 ** k) * a).astype(f32)
    q = (q / f32(edge0)).astype(f32)
    return np.floor(q).astype(np.int64)


def morton_codes(G_levels, d):
    """G_levels: list over depth 1..k of (n,d) integer cells.  Code = concatenation over levels
    (coarsest most significant) of the child digit sum_j bit_j << j of that level."""
    code = np.zeros(G_levels[0].shape[0], dtype=object)
    for G in G_levels:
        digit = np.zeros(G.shape[0], dtype=np.int64)
        for j in range(d):
            digit |= (G[:, j] & 1) << j
        code = code * (1 << d) + digit
    return code


def box_ids_by_morton_rank(X, origin, edge0, k):
    d = X.shape[1]
    Gs = [cell_coords(X, origin, edge0, l) for l in range(1, k + 1)]
    codes = morton_codes(Gs, d)
    uniq = sorted(set(codes.tolist()))
    rank = {c: i for i, c in enumerate(uniq)}
    return np.array([rank[c] for c in codes.tolist()], dtype=np.int64), Gs[-1]


def classify_np(cx, cy, nx, ny, edge, nr_interp, small_limit):
    """0 small, 1 far, 2 keep; fp32, left-to-right sum of squares, correctly rounded sqrt."""
    size = nx.astype(np.int64) + ny.astype(np.int64)
    diff = (cy.astype(f32) - cx.astype(f32)).astype(f32)
    acc = np.zeros(diff.shape[0], f32)
    for j in range(diff.shape[1]):
        acc = (acc + (diff[:, j] * diff[:, j]).astype(f32)).astype(f32)
    dist = np.sqrt(acc).astype(f32)
    thr = f32(edge) * f32(2)
    out = np.full(diff.shape[0], 2, np.int64)
    small1 = size < 2 * nr_interp
    far = (~small1) & (dist >= thr)
    small2 = (~small1) & (~far) & (size < 2 * small_limit)
    out[small1 | small2] = 0
    out[far] = 1
    return out


def box_of_point(level, which="x"):
    """Per-point compact box id from a level dict (perm + offsets)."""
    perm = level["perm" + which]
    off = level["off" + which]
    box = np.empty(perm.shape[0], np.int64)
    box[perm] = np.repeat(np.arange(off.shape[0] - 1), np.diff(off))
    return box


def classify_var_comp_np(cx, cy, nx, ny, edge, nr_interp, small_limit, d, lcs, eff_var_limit):
    """var_compression=True predicates (F3M_src/n_tree.cu:727-743, F3M_src/1_d_conv.cu:983-1026), fp32.
    0 small, 1 far, 2 keep, 3 dropped."""
    edge, lcs, eff = f32(edge), f32(lcs), f32(eff_var_limit)
    sq = f32(f32(edge * edge) * lcs)
    do_init = sq <= 5
    quarter = f32(f32(f32(d) * sq) / f32(4))
    en_pair = quarter <= eff
    en_all = quarter <= f32(eff / f32(2))
    crit = np.sqrt(f32(f32(eff * f32(2)) / f32(f32(d) * lcs))).astype(f32)
    size = nx.astype(np.int64) + ny.astype(np.int64)
    diff = (cy.astype(f32) - cx.astype(f32)).astype(f32)
    acc = np.zeros(diff.shape[0], f32)
    for j in range(diff.shape[1]):
        acc = (acc + (diff[:, j] * diff[:, j]).astype(f32)).astype(f32)
    dist = np.sqrt(acc).astype(f32)
    out = np.full(diff.shape[0], -1, np.int64)
    todo = np.ones(diff.shape[0], bool)

    def settle(mask, code):
        nonlocal todo
        m = todo & mask
        out[m] = code
        todo = todo & ~m

    if do_init:
        settle(size < 2 * nr_interp, 0)
    settle(dist >= f32(edge * f32(2)), 1 if do_init else 3)
    if en_pair:
        settle(((dist * dist).astype(f32) * lcs).astype(f32).astype(np.float64) <= 1e-2, 1)
    if en_all:
        settle(dist <= crit, 1)
    settle(size < 2 * small_limit, 0)
    settle(np.ones_like(todo), 2)
    return out
