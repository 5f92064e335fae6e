"""Pins the oracle's box division and interaction lists by brute force and invariants
(reference: F3M_src/n_tree.cu:25-179,594-811,903-969; F3M_src/1_d_conv.cu:887-953,1127-1191)."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from helpers import box_ids_by_morton_rank, box_of_point, cell_coords, classify_np, classify_var_comp_np

f32 = np.float32


def clouds():
    rng = np.random.default_rng(11)
    out = []
    out.append(("uniform3", rng.random((3000, 3), dtype=f32), None))
    out.append(("normal3", rng.standard_normal((3000, 3)).astype(f32), None))
    out.append(("uniform2", rng.random((2500, 2), dtype=f32), None))
    out.append(("uniform1", rng.random((1500, 1), dtype=f32), None))
    out.append(("uniform4", rng.random((4000, 4), dtype=f32), None))
    out.append(("uniform5", rng.random((5000, 5), dtype=f32), None))
    Xc = np.concatenate([rng.normal(m, s, (600, 3)) for m, s in zip(rng.random((5, 3)) * 10, 0.05 + 0.45 * rng.random((5, 3)))]).astype(f32)
    Yc = (Xc.min(0) + (Xc.max(0) - Xc.min(0)) * rng.random((2000, 3))).astype(f32)
    out.append(("clustered_xy", Xc, Yc))
    dup = rng.random((500, 3), dtype=f32)
    out.append(("duplicates", np.concatenate([dup, dup, dup]), None))
    g = (np.stack(np.meshgrid(*[np.arange(9)] * 3, indexing="ij"), -1).reshape(-1, 3) / 8.0).astype(f32)
    out.append(("lattice_on_faces", np.concatenate([g, g[::-1]]), None))
    return out


CLOUDS = clouds()
PARAMS = dict(ls=1.0, min_points=60, nr_of_interpolation=27, small_field_points=40)


@pytest.mark.parametrize("name,X,Y", CLOUDS, ids=[c[0] for c in CLOUDS])
def test_tree_levels_bruteforce(oracle, name, X, Y):
    P = oracle.Plan(X, Y, **PARAMS)
    edge0, xmin, ymin = oracle.root(X, Y)
    # root closed form
    rng_x = (X.max(0) - X.min(0)).max()
    if Y is None:
        assert edge0 == f32(f32(rng_x) * f32(1.01))
    else:
        rng_y = (Y.max(0) - Y.min(0)).max()
        assert edge0 == f32(f32(max(rng_x, rng_y)) * f32(1.01))
        assert np.array_equal(ymin, Y.min(0))
    assert np.array_equal(xmin, X.min(0))
    assert P.nlevels >= 1
    d = X.shape[1]
    prev_box = {"x": None, "y": None}
    for k in range(P.nlevels):
        L = P.level(k)
        assert L["edge"] == f32(edge0 * f32(0.5 ** (k + 1)))
        for which, data, origin in (("x", X, xmin), ("y", X if Y is None else Y, xmin if Y is None else ymin)):
            box = box_of_point(L, which)
            cnt, off, perm, ctr = L["cnt" + which], L["off" + which], L["perm" + which], L["c" + which]
            # Morton-rank invariant: compact id == rank of the Morton code among non-empty boxes
            ref_box, G = box_ids_by_morton_rank(data, origin, edge0, k + 1)
            assert np.array_equal(box, ref_box)
            # counts / offsets / perm consistency
            assert cnt.sum() == data.shape[0] and (cnt > 0).all()
            assert np.array_equal(off, np.concatenate([[0], np.cumsum(cnt)]))
            assert np.array_equal(np.sort(perm), np.arange(data.shape[0]))
            for bidx in range(len(cnt)):
                seg = perm[off[bidx]:off[bidx + 1]]
                assert (np.diff(seg) > 0).all()          # canonical ascending order inside a box
            # centres: closed form origin + (g+1/2)*edge within a few ulps, and membership
            first = perm[off[:-1]]
            closed = origin.astype(np.float64) + (G[first] + 0.5) * np.float64(L["edge"])
            scale = np.abs(origin).max() + edge0
            assert np.abs(ctr - closed).max() <= 8 * np.finfo(f32).eps * scale
            rel = (data.astype(np.float64) - ctr[box].astype(np.float64)) / np.float64(L["edge"])
            assert (rel > -0.5 - 1e-4).all() and (rel < 0.5 + 1e-4).all()
            # nesting: a box's points all lie in one parent box
            if prev_box[which] is not None:
                parent_of_box = np.full(len(cnt), -1)
                parent_of_box[box] = prev_box[which]
                assert (parent_of_box[box] == prev_box[which]).all()
            prev_box[which] = box


@pytest.mark.parametrize("name,X,Y", CLOUDS, ids=[c[0] for c in CLOUDS])
def test_lists_bruteforce_and_coverage(oracle, name, X, Y):
    P = oracle.Plan(X, Y, **PARAMS)
    N, M = X.shape[0], (X.shape[0] if Y is None else Y.shape[0])
    keep_prev = {(0, 0)}
    parent_x = parent_y = None
    covered = 0
    for k in range(P.nlevels):
        L = P.level(k)
        bx_pt, by_pt = box_of_point(L, "x"), box_of_point(L, "y")
        nbx, nby = len(L["cntx"]), len(L["cnty"])
        # parent (compact id at the previous level) of every box
        if k == 0:
            par_x, par_y = np.zeros(nbx, int), np.zeros(nby, int)
        else:
            par_x = np.zeros(nbx, int); par_x[bx_pt] = parent_x
            par_y = np.zeros(nby, int); par_y[by_pt] = parent_y
        # brute force over ALL pairs of non-empty boxes
        BX, BY = np.meshgrid(np.arange(nbx), np.arange(nby), indexing="ij")
        BX, BY = BX.ravel(), BY.ravel()
        alive = np.fromiter(((int(px), int(py)) in keep_prev for px, py in zip(par_x[BX], par_y[BY])), bool, len(BX))
        BX, BY = BX[alive], BY[alive]
        cls = classify_np(L["cx"][BX], L["cy"][BY], L["cntx"][BX], L["cnty"][BY], L["edge"],
                          PARAMS["nr_of_interpolation"], PARAMS["small_field_points"])
        for name_, code in (("small", 0), ("far", 1), ("keep", 2)):
            ref = np.stack([BX[cls == code], BY[cls == code]], 1)
            got = L[name_]
            assert got.shape == ref.shape, (k, name_)
            assert np.array_equal(got, ref), (k, name_)   # meshgrid 'ij' order is lexicographic (bx,by)
        for name_ in ("small", "far"):
            covered += int((L["cntx"][L[name_][:, 0]].astype(np.int64) * L["cnty"][L[name_][:, 1]]).sum())
        keep_prev = set(map(tuple, L["keep"].tolist()))
        parent_x, parent_y = bx_pt, by_pt
    Lk = P.level(P.nlevels - 1)
    covered += int((Lk["cntx"][Lk["keep"][:, 0]].astype(np.int64) * Lk["cnty"][Lk["keep"][:, 1]]).sum())
    assert covered == N * M                              # every point pair is handled exactly once
    assert P.work_near_pairs + sum(
        int((P.level(k)["cntx"][P.level(k)["far"][:, 0]].astype(np.int64) * P.level(k)["cnty"][P.level(k)["far"][:, 1]]).sum())
        for k in range(P.nlevels)) == N * M


def test_loop_guard_and_no_division(oracle):
    rng = np.random.default_rng(5)
    X = rng.random((500, 3), dtype=f32)
    P = oracle.Plan(X, None, ls=1.0, min_points=1000)
    assert P.nlevels == 0                                # N <= min_points: never divides
    b = rng.standard_normal((500, 2)).astype(f32)
    assert np.allclose(P.apply(b), oracle.exact_f64(X, X, b, 1.0), rtol=1e-4, atol=1e-4)
    # stops as soon as the densest box has <= min_points points
    X = rng.random((4000, 2), dtype=f32)
    P = oracle.Plan(X, None, ls=1.0, min_points=300, small_field_points=10, nr_of_interpolation=4)
    for k in range(P.nlevels - 1):
        assert P.level(k)["cntx"].max() > 300
    assert P.level(P.nlevels - 1)["cntx"].max() <= 300 or len(P.level(P.nlevels - 1)["keep"]) == 0


@settings(max_examples=25, deadline=None)
@given(st.integers(0, 10 ** 6), st.integers(1, 3), st.integers(200, 900))
def test_tree_hypothesis_random_clouds(oracle, seed, d, n):
    rng = np.random.default_rng(seed)
    X = rng.random((n, d)).astype(f32)
    X[rng.integers(0, n, n // 10)] = X[rng.integers(0, n, n // 10)]       # duplicates
    X[rng.integers(0, n, n // 10), rng.integers(0, d)] = f32(0.5)          # points on a face
    P = oracle.Plan(X, None, ls=0.5, min_points=30, nr_of_interpolation=8, small_field_points=20)
    edge0, xmin, _ = oracle.root(X)
    for k in range(P.nlevels):
        L = P.level(k)
        ref_box, _ = box_ids_by_morton_rank(X, xmin, edge0, k + 1)
        assert np.array_equal(box_of_point(L, "x"), ref_box)


@pytest.mark.parametrize("ls,eff", [(2.0, 0.3), (0.7, 0.3), (0.25, 0.15), (8.0, 0.5)])
def test_var_compression_lists_bruteforce(oracle, ls, eff):
    """The var_compression=True classification against an independent numpy restatement of its
    predicates, over all pairs of non-empty boxes whose parents were kept."""
    rng = np.random.default_rng(17)
    X = rng.random((3000, 3), dtype=f32)
    prm = dict(ls=ls, min_points=60, nr_of_interpolation=27, small_field_points=40, var_compression=True,
               eff_var_limit=eff)
    P = oracle.Plan(X, None, **prm)
    keep_prev = {(0, 0)}
    parent = None
    seen_shortcut = False
    for k in range(P.nlevels):
        L = P.level(k)
        box = box_of_point(L, "x")
        nb = len(L["cntx"])
        par = np.zeros(nb, int)
        if k > 0:
            par[box] = parent
        BX, BY = np.meshgrid(np.arange(nb), np.arange(nb), indexing="ij")
        BX, BY = BX.ravel(), BY.ravel()
        alive = np.fromiter(((int(a), int(b)) in keep_prev for a, b in zip(par[BX], par[BY])), bool, len(BX))
        BX, BY = BX[alive], BY[alive]
        cls = classify_var_comp_np(L["cx"][BX], L["cx"][BY], L["cntx"][BX], L["cntx"][BY], L["edge"], 27, 40, 3,
                                   P.lcs, eff)
        for name_, code in (("small", 0), ("far", 1), ("keep", 2)):
            ref = np.stack([BX[cls == code], BY[cls == code]], 1)
            assert np.array_equal(L[name_], ref), (k, name_)
        plain = classify_np(L["cx"][BX], L["cx"][BY], L["cntx"][BX], L["cntx"][BY], L["edge"], 27, 40)
        seen_shortcut |= bool((plain != cls).any())
        keep_prev = set(map(tuple, L["keep"].tolist()))
        parent = box
    assert seen_shortcut or ls < 1.0        # smooth kernels must trigger the extra far-field shortcuts


# ------------------------------------------------------------------------------------------------
# key -> value table (F3M_src/linearprobing.cu:18-87)

def test_hash_finaliser_known_answers(oracle):
    """MurmurHash3_x86_32 of the empty string is its finaliser applied to the seed: the published
    vectors 0 -> 0, seed 1 -> 0x514E28B7, seed 0xffffffff -> 0x81F16F39."""
    assert oracle.hash32(0) == 0
    assert oracle.hash32(1) == 0x514E28B7
    assert oracle.hash32(0xFFFFFFFF) == 0x81F16F39
    for key, cap in ((1, 1 << 20), (0xFFFFFFFF, 1024), (123456789, 4096)):
        assert oracle.hash_slot(key, cap) == oracle.hash32(key) % (cap - 1)      # hash_2: modulo capacity-1


def test_hash_table_against_dict(oracle):
    rng = np.random.default_rng(5)
    cap = 256
    keys = rng.choice(1 << 16, 120, replace=False)
    ref = {}
    t = oracle.HashTable(cap)
    for i, k in enumerate(keys.tolist()):
        t.insert(k, i)
        ref[k] = i
    t.insert(int(keys[3]), 999)                       # same key again: value replaced, no second slot
    ref[int(keys[3])] = 999
    for k, v in ref.items():
        assert t.lookup(k) == v
    absent = [k for k in range(1 << 16, (1 << 16) + 50)]
    assert all(t.lookup(k) == -1 for k in absent)     # kEmpty = 0xffffffff = -1 as an int
    used = t.table[0::2] != 0xFFFFFFFF
    assert used.sum() == len(ref) and not used[cap - 1]    # slots run 0 .. capacity-2 only


def test_grid_key_is_the_reference_sum(oracle):
    # sum_j g_j (2^k)^(d-1-j): dimension 0 most significant (F3M_src/1_d_conv.cu:1142-1144)
    assert oracle.grid_key(3, 2, [1, 2, 3]) == 1 * 16 + 2 * 4 + 3
    assert oracle.grid_key(2, 5, [7, 30]) == 7 * 32 + 30
    assert oracle.grid_key(1, 9, [300]) == 300
