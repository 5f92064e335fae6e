"""f3m_plan_apply_noalloc (the entry point that allocates nothing: its temporaries live in static device
memory) against f3m_plan_apply, through the C ABI.  Results must be the same bit for bit: both run the
same kernels in the same order, only the memory of the temporaries differs.  Two calls in a row, the
second on a smaller problem, so that whatever the first call left in the shared scratch array is there
when the second runs."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.fixture(scope="module")
def eng():
    import torch
    assert torch.cuda.is_available(), "these tests need a GPU"
    from f3m_amd import engine
    engine._lib.get()
    return engine


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _reserved(eng):
    import torch
    torch.cuda.synchronize()
    return torch.cuda.memory_reserved()


def test_apply_without_allocation_matches_apply(eng):
    import torch
    from f3m_amd.capi import F3MError
    rng = np.random.default_rng(31)
    print("case no-alloc: 3-D 300000 points, then 4-D 60000 x 20000 points with 3 columns", flush=True)
    X1 = rng.random((300000, 3), dtype=f32)
    b1 = rng.standard_normal((300000, 1)).astype(f32)
    X2 = rng.random((60000, 4), dtype=f32)
    Y2 = rng.random((20000, 4), dtype=f32)
    b2 = rng.standard_normal((20000, 3)).astype(f32)
    p1 = eng.Plan(dev(X1), None, ls=0.7)
    p2 = eng.Plan(dev(X2), dev(Y2), ls=1.0, nr_of_interpolation=81, min_points=500, small_field_points=200)
    assert p1.depth >= 2 and p2.depth >= 1
    b1d, b2d = dev(b1), dev(b2)
    out1 = torch.full((300000, 1), float("nan"), device="cuda")
    # a plan whose tables are not built yet is refused, and nothing is written
    with pytest.raises(F3MError) as e:
        p1.apply_noalloc(b1d, out1)
    assert e.value.code == 41 and torch.isnan(out1).all()
    want1 = p1.apply(b1d)                       # builds the tables of the plan
    want2 = p2.apply(b2d)
    out2 = torch.full((60000, 3), float("nan"), device="cuda")
    eng.release_cache()                         # the library's buffer cache is empty: any allocation would show
    lib = eng._lib.get()
    free0 = torch.cuda.mem_get_info()[0]
    p1.apply_noalloc(b1d, out1)                 # first call
    p2.apply_noalloc(b2d, out2)                 # second call, smaller, same scratch array
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0            # no device memory was taken
    assert np.array_equal(out1.cpu().numpy(), want1.cpu().numpy())
    assert np.array_equal(out2.cpu().numpy(), want2.cpu().numpy())
    # and again in the other order, results unchanged
    out1.fill_(float("nan"))
    p1.apply_noalloc(b1d, out1)
    assert np.array_equal(out1.cpu().numpy(), want1.cpu().numpy())
    del lib


def test_apply_without_allocation_refuses_what_does_not_fit(eng):
    import torch
    from f3m_amd.capi import F3MError
    print("case no-alloc: refusal above the scratch size", flush=True)
    rng = np.random.default_rng(32)
    n = 6_000_000                               # 4 columns: 4 * 4 * (N + M) bytes = 192 MB > 128 MiB
    X = torch.from_numpy(rng.random((n, 3), dtype=f32)).cuda()
    b = torch.from_numpy(rng.standard_normal((n, 4)).astype(f32)).cuda()
    plan = eng.Plan(X, None, ls=1.0)
    plan.apply(b)
    out = torch.full((n, 4), float("nan"), device="cuda")
    with pytest.raises(F3MError) as e:
        plan.apply_noalloc(b, out)
    assert e.value.code == 42 and "scratch" in str(e.value)
    assert torch.isnan(out).all()
    plan.close()


def test_apply_without_allocation_many_columns(eng):
    """The scratch need must not grow with the number of columns: every column group (and every column's far
    field) reuses the memory of the one before.  N = 1e6 with c = 6 and c = 16: the first group of four columns takes
    ~100 MB of the 128 MiB (sorted copies 32 MB, sliced near-field partial sums 67 MB), so a second group that did
    not reuse it could not fit.  Results are those of f3m_plan_apply bit for bit."""
    import torch
    print("case no-alloc: 3-D 1000000 points, 6 and 16 columns", flush=True)
    rng = np.random.default_rng(34)
    n = 1_000_000
    X = dev(rng.random((n, 3), dtype=f32))
    plan = eng.Plan(X, None, ls=1.0)
    for c in (6, 16):
        b = dev(rng.standard_normal((n, c)).astype(f32))
        want = plan.apply(b)
        out = torch.full((n, c), float("nan"), device="cuda")
        plan.apply_noalloc(b, out)
        torch.cuda.synchronize()
        assert torch.equal(out, want), c
    plan.close()


def test_apply_without_allocation_refusal_writes_nothing(eng):
    """A product whose sorted copies fit (64 MB: the check before any work) but whose first column group does not
    (1.5e6 targets in ~13000 pieces of 128, sliced three ways for four columns: ~80 MB of partial sums on top) is
    refused while that group is being queued: error 42, and `out` is untouched."""
    import torch
    from f3m_amd.capi import F3MError
    print("case no-alloc: refusal inside the first column group", flush=True)
    rng = np.random.default_rng(35)
    X = dev(rng.random((1_500_000, 3), dtype=f32))
    Y = dev(rng.random((2_500_000, 3), dtype=f32))
    b = dev(rng.standard_normal((2_500_000, 6)).astype(f32))
    plan = eng.Plan(X, Y, ls=1.0)
    want = plan.apply(b)
    out = torch.full((1_500_000, 6), float("nan"), device="cuda")
    with pytest.raises(F3MError) as e:
        plan.apply_noalloc(b, out)
    torch.cuda.synchronize()
    assert e.value.code == 42 and "scratch" in str(e.value)
    assert torch.isnan(out).all()
    # the library is in order afterwards: the same plan still multiplies, with the same bits
    assert torch.equal(plan.apply(b), want)
    plan.close()


def test_apply_without_allocation_under_graph_capture(eng):
    """One of the callers the entry point is for: a HIP graph.  The call is captured once and replayed with
    the program's own eager products and synchronisations between the replays; every replay must give the
    eager result bit for bit, also after the input buffer's contents changed."""
    import torch
    print("case no-alloc: captured into a graph, 3-D 300000 points, 5 replays", flush=True)
    rng = np.random.default_rng(33)
    n = 300000
    X = dev(rng.random((n, 3), dtype=f32))
    b = dev(rng.standard_normal((n, 2)).astype(f32))
    plan = eng.Plan(X, None, ls=0.7)
    want = plan.apply(b)
    out = torch.full((n, 2), float("nan"), device="cuda")
    plan.apply_noalloc(b, out)                              # scratch address of this device is looked up here
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=torch.cuda.Stream()):
        plan.apply_noalloc(b, out)
    for replay in range(4):
        out.fill_(float("nan"))
        other = plan.apply(b)                               # eager work of the same library between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), replay
        assert torch.equal(other, want)
    b2 = dev(rng.standard_normal((n, 2)).astype(f32))
    want2 = plan.apply(b2)
    b.copy_(b2)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, want2)
    plan.close()


def test_apply_without_allocation_five_dimensions(eng):
    """5-D: the near field takes its factored form, whose weights (the sorted b times exp2(-|y'|^2)) are one more
    temporary per column group; it comes from the static scratch memory like the others.  One and three columns."""
    import torch
    print("case no-alloc: 5-D 200000 points, 243 nodes, 1 and 3 columns", flush=True)
    rng = np.random.default_rng(35)
    X = dev(rng.random((200000, 5), dtype=f32))
    plan = eng.Plan(X, None, ls=1.0, nr_of_interpolation=243, min_points=1000, small_field_points=243)
    assert plan.depth >= 2
    for c in (1, 3):
        b = dev(rng.standard_normal((200000, c)).astype(f32))
        want = plan.apply(b)
        out = torch.full((200000, c), float("nan"), device="cuda")
        # The far field of plan.apply ran on the library's second stream.  Here its kernels run on the caller's stream
        # for the first time, and the 5-D M2L kernel keeps some registers in the runtime's scratch memory, which the
        # runtime reserves per queue when such a kernel first runs there: one product beforehand, as the header says.
        plan.apply_noalloc(b, out)
        torch.cuda.synchronize()
        out.fill_(float("nan"))
        eng.release_cache()
        free0 = torch.cuda.mem_get_info()[0]
        plan.apply_noalloc(b, out)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0
        assert np.array_equal(out.cpu().numpy(), want.cpu().numpy())
