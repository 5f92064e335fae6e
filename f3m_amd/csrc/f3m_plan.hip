// Host orchestration (the level loop of F3M_src/n_tree.cu:1056-1125) and the C ABI of include/f3m.h.
#include "../../include/f3m.h"
#include "f3m_engine.h"

#include <cmath>
#include <cstdlib>
#include <memory>

namespace f3m {

// ---- stage timing ----------------------------------------------------------------------------
#ifndef F3M_CPU_EMU
struct StageTimer {
    bool enabled = false;
    struct Span { int stage; hipEvent_t a, b; };
    std::vector<Span> spans;
    std::vector<hipEvent_t> spare;      // events are kept for the next call
    double t[kNumStages] = {0};
    int n[kNumStages] = {0};
    hipEvent_t take()
    {
        hipEvent_t e = nullptr;
        if (!spare.empty()) { e = spare.back(); spare.pop_back(); }
        else F3M_HIP(hipEventCreate(&e));
        return e;
    }
    void begin(int stage, hipStream_t s)
    {
        if (!enabled) return;
        Span sp{stage, take(), take()};
        F3M_HIP(hipEventRecord(sp.a, s));
        spans.push_back(sp);
    }
    void end(hipStream_t s)
    {
        if (!enabled || spans.empty()) return;
        F3M_HIP(hipEventRecord(spans.back().b, s));
    }
    void reset()
    {
        for (auto &sp : spans) { spare.push_back(sp.a); spare.push_back(sp.b); }
        spans.clear();
        for (int i = 0; i < kNumStages; i++) { t[i] = 0; n[i] = 0; }
    }
    void collect()
    {
        if (!enabled) return;
        for (auto &sp : spans) {
            float ms = 0.f;
            if (hipEventSynchronize(sp.b) == hipSuccess && hipEventElapsedTime(&ms, sp.a, sp.b) == hipSuccess) {
                t[sp.stage] += ms * 1e-3;
                n[sp.stage] += 1;
            }
            spare.push_back(sp.a);
            spare.push_back(sp.b);
        }
        spans.clear();
    }
};
#else
struct StageTimer {
    bool enabled = false;
    double t[kNumStages] = {0};
    int n[kNumStages] = {0};
    void begin(int, hipStream_t) {}
    void end(hipStream_t) {}
    void reset() {}
    void collect() {}
};
#endif
static thread_local StageTimer g_timer;
static thread_local std::string g_error;

struct Scope {
    hipStream_t s;
    Scope(int stage, hipStream_t st) : s(st) { g_timer.begin(stage, s); }
    ~Scope() { g_timer.end(s); }
};

}  // namespace f3m

using namespace f3m;

struct f3m_plan {
    int d = 0;
    bool symmetric = true;
    long long N = 0, M = 0;
    f3m_params prm{};
    float lcs = 0.f;
    Tree tx, ty_;
    Tree *ty = nullptr;
    std::vector<PlanLevel> levels;         // levels[k-1] = depth k
    std::map<int, std::unique_ptr<NodeSet>> nodes;
    DBuf<float> Xraw, Yraw;                // row-major copies, only when no division happened
    // one-shot products: the first column group of b, already in sorted order (gathered while the lists were built)
    DBuf<float> early_bs;
    DBuf<float> early_outs, early_outs_far;   // the result arrays of that column group, cleared beside the last level's lists
    DBuf<long long> early_symfix;             // with them, for a single column on one tree: the cleared fixed-point sums of the
    DBuf<unsigned> early_symmax;              // symmetric near field and the largest |weight| (SymSums)
    const float *early_b = nullptr;
    int early_c = 0, early_ncol = 0;
    float *early_out = nullptr;               // the caller's result array, cleared beside the last level's lists (N x early_c floats)
    std::map<std::pair<int, int>, std::unique_ptr<DBuf<float>>> shift_tabs;   // (parent nodes, child nodes)
    const float *shift_table(int nodes_parent, int nodes_child, hipStream_t s)
    {
        auto key = std::make_pair(nodes_parent, nodes_child);
        auto it = shift_tabs.find(key);
        if (it == shift_tabs.end()) {
            require_tables_may_be_built("a table that moves expansions between levels");
            std::unique_ptr<DBuf<float>> t(new DBuf<float>());
            make_shift_tables(nodeset(nodes_parent, s), nodeset(nodes_child, s), *t, s);
            it = shift_tabs.emplace(key, std::move(t)).first;
        }
        return it->second->get();
    }
    NodeSet &nodeset(int num_nodes, hipStream_t s)
    {
        auto it = nodes.find(num_nodes);
        if (it == nodes.end()) {
            require_tables_may_be_built("a node set");
            std::unique_ptr<NodeSet> ns(new NodeSet());
            make_nodes(*ns, d, num_nodes, s);
            it = nodes.emplace(num_nodes, std::move(ns)).first;
        }
        return *it->second;
    }
};

namespace f3m {

static void check_params(int d, long long N, long long M, bool sym, const f3m_params *p)
{
    F3M_REQUIRE(p != nullptr, 1, "params is NULL");
    F3M_REQUIRE(d >= 1 && d <= kMaxD, 2, "dimension must be 1..10 (got %d)", d);
    F3M_REQUIRE(N >= 1, 3, "X has no rows");
    F3M_REQUIRE(sym || M >= 1, 3, "Y has no rows");
    F3M_REQUIRE(N < (1ll << 31) - 1 && M < (1ll << 31) - 1, 4, "at most 2^31-2 points per side");
    F3M_REQUIRE(p->ls > 0.f && std::isfinite(p->ls), 5, "ls must be positive");
    F3M_REQUIRE(p->nr_of_interpolation >= 1, 6, "nr_of_interpolation must be >= 1");
    F3M_REQUIRE(p->small_field_points >= 0, 7, "small_field_points must be >= 0");
}

static void check_device_ptr(const void *p, const char *name)
{
    F3M_REQUIRE(p != nullptr, 8, "%s is NULL", name);
#ifndef F3M_CPU_EMU
    hipPointerAttribute_t a;
    hipError_t e = hipPointerGetAttributes(&a, p);
    if (e != hipSuccess) { (void)hipGetLastError(); throw Error(9, fmt("%s is not a device pointer", name)); }
    F3M_REQUIRE(a.type == hipMemoryTypeDevice || a.type == hipMemoryTypeManaged, 9, "%s is not device memory", name);
#endif
}

// start of a plan: the root pair (0,0), its row pointers (0,1), and zeroed counters
__global__ void plan_init_kernel(int *__restrict__ pair, int *__restrict__ rowptr, int *__restrict__ counters, int ncounters,
                                 int *__restrict__ stats, int nstats)
{
    const int t = threadIdx.x;
    if (t < 2) { pair[t] = 0; rowptr[t] = t; }
    for (int i = t; i < ncounters; i += blockDim.x) counters[i] = 0;
    for (int i = t; i < nstats; i += blockDim.x) stats[i] = 0;
}

static ClassifyParams classify_params(const f3m_plan &P, float edge)
{
    ClassifyParams cp;
    cp.nr_interp = P.prm.nr_of_interpolation;
    cp.small_limit = P.prm.small_field_points;
    cp.var_comp = P.prm.var_compression ? 1 : 0;
    cp.lcs = P.lcs;
    cp.edge = edge;
    cp.do_init = 1; cp.en_pair = 0; cp.en_all = 0; cp.crit = 0.f;
    if (cp.var_comp) {
        // thresholds of F3M_src/n_tree.cu:728-743; the "ls" there is 1/(2 ls^2) (n_tree.cu:1083)
        float sq = edge * edge * P.lcs;
        float eff = P.prm.eff_var_limit;
        cp.do_init = sq <= 5;
        cp.en_pair = ((float)P.d * sq / 4) <= eff;
        cp.en_all = ((float)P.d * sq / 4) <= (eff / 2);
        cp.crit = sqrtf(eff * 2 / ((float)P.d * P.lcs));
    }
    return cp;
}

// A second stream per device, on which the far field of a product runs beside the near field (which is bound
// by vector-ALU issue and leaves the memory system and the latency-bound far-field kernels room), with the two
// events that fork it from and join it to the caller's stream.  Default priority, kept for the life of the process.
struct SideStream {
    hipStream_t stream = nullptr;
    hipEvent_t fork = nullptr, join = nullptr, tables = nullptr;
};
static SideStream &side_stream()
{
    static std::mutex mu;
    static std::map<int, SideStream> per_device;
    int dev = 0;
    F3M_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> g(mu);
    SideStream &ss = per_device[dev];
    if (ss.stream == nullptr) {
        F3M_HIP(hipStreamCreateWithFlags(&ss.stream, hipStreamNonBlocking));
        F3M_HIP(hipEventCreateWithFlags(&ss.fork, hipEventDisableTiming));
        F3M_HIP(hipEventCreateWithFlags(&ss.join, hipEventDisableTiming));
        F3M_HIP(hipEventCreateWithFlags(&ss.tables, hipEventDisableTiming));
    }
    return ss;
}

// b_early (nullable, with c_early columns): the weights of the product that will follow at once (f3m_kmvm_f32);
// their first column group is put into sorted order while the lists are built.  With b_early the function returns
// when the last kernels of the plan are queued, not when they are done: the product is queued behind them on the
// same stream (every host-side figure of the plan is known by then), so the GPU does not wait for the host in between.
static f3m_plan *plan_create(int d, const float *X, long long N, const float *Y, long long M, const f3m_params *prm,
                             hipStream_t s, const float *b_early = nullptr, int c_early = 0, float *out_early = nullptr)
{
    bool sym = (Y == nullptr || Y == X);
    check_params(d, N, M, sym, prm);
    check_device_ptr(X, "X");
    if (!sym) check_device_ptr(Y, "Y");
    if (out_early != nullptr) check_device_ptr(out_early, "out");       // it is written before the product checks it
    // (a caller that passes overlapping b and out against the interface's rule at least keeps the old order: all of
    // b is read before the first write to out)
    if (out_early != nullptr && b_early != nullptr) {
        const char *b0 = reinterpret_cast<const char *>(b_early), *o0 = reinterpret_cast<const char *>(out_early);
        const size_t bb = sizeof(float) * (size_t)(sym ? N : M) * (size_t)std::max(c_early, 0), ob = sizeof(float) * (size_t)N * (size_t)std::max(c_early, 0);
        if (b0 < o0 + ob && o0 < b0 + bb) out_early = nullptr;
    }
    std::unique_ptr<f3m_plan> P(new f3m_plan());
    P->d = d; P->symmetric = sym; P->N = N; P->M = sym ? N : M; P->prm = *prm;
    P->lcs = 1 / (2 * prm->ls * prm->ls);                        // F3M_src/n_tree.cu:1060
    P->ty = sym ? &P->tx : &P->ty_;
    Scope sc(kPlan, s);

    // The loop of F3M_src/n_tree.cu:1075/:1099 divides only while the fullest box holds more than
    // min_points points, and depth 0 is one box with every point.  A cloud whose points all coincide
    // cannot be divided either (the reference would compute 0/0 cell indices).  Both cases take the
    // exact product and need no tree.
    bool need_tree = (float)N > prm->min_points && (sym || (float)M > prm->min_points);
    Geo gx;
    memset(&gx, 0, sizeof(gx));
    if (need_tree) {
        // Root geometry (F3M_src/n_tree.cu:25-46), reduced on the device: the Morton keys and their sort are queued
        // behind it and run while the same values travel to the host, which needs them from the root level on.
        DBuf<float> partx, party, dgeo((size_t)2 * kMaxD + 1);
        const unsigned npx = bounding_box_launch(X, N, d, partx, s);
        const unsigned npy = sym ? 0u : bounding_box_launch(Y, M, d, party, s);
        root_geometry_launch(partx.get(), npx, sym ? nullptr : party.get(), npy, d, dgeo.get(), s);
        ExportList G;
        G.add(dgeo.get(), 2 * kMaxD + 1, 0);
        SegmentFetch geo_fetch;
        geo_fetch.begin(G, s);
        gx.d = d;
        // key depth: past 31/d levels the reference's int32 grid keys overflow, past 16 its fp32
        // centres stop resolving cells; the tree is never deeper and what is left is summed exactly
        gx.L = std::min(31 / d, 16);
        sort_tree_launch(P->tx, X, N, d, gx.L, dgeo.get(), dgeo.get() + 2 * kMaxD, s);
        if (!sym) sort_tree_launch(P->ty_, Y, M, d, gx.L, dgeo.get() + kMaxD, dgeo.get() + 2 * kMaxD, s);
        float hgeo[2 * kMaxD + 1];
        geo_fetch.wait(hgeo, s);
        gx.edge0 = hgeo[2 * kMaxD];
        F3M_REQUIRE(std::isfinite(gx.edge0), 10, "point coordinates are not finite");
        if (gx.edge0 > 0.f) {
            Geo gy = gx;
            for (int j = 0; j < d; j++) { gx.origin[j] = hgeo[j]; gy.origin[j] = hgeo[kMaxD + j]; }
            root_level_launch(P->tx, gx, s);
            if (!sym) root_level_launch(P->ty_, gy, s);
        } else {
            need_tree = false;      // every point at one place: the sort that was queued is simply not used
        }
    }

    // The root pair (0,0) with its row pointers (0,1), and the counters of the level loop, all cleared by one kernel:
    // [0..1] pair, [2..3] row pointers, [4..19] counters of a level (dres), then eight 64-bit row statistics per level (drow)
    constexpr int kMaxLevels = 40;
    PairList root;
    root.n = 1;
    root.pairs.reset(2);
    root.rowptr.reset(2);
    DBuf<int> dres(16);
    DBuf<long long> drow((size_t)8 * kMaxLevels);
    F3M_LAUNCH(plan_init_kernel, 1, 64, 0, s, root.pairs.get(), root.rowptr.get(), dres.get(), 16,
               reinterpret_cast<int *>(drow.get()), 2 * 8 * kMaxLevels);
    check_launch("plan_init");
    const PairList *keep = &root;
    P->levels.reserve(64);   // `keep` points into this vector: it must not reallocate
    // Loop of F3M_src/n_tree.cu:1075 (one tree) and :1099 (two trees): divide while the keep list is not
    // empty and the fullest box of each tree holds more than min_points points.  The host has to fetch
    // two things per level, the box counts of the division and the list sizes; to wait only once per
    // level, the division of depth k+1 is started together with the list count of depth k whenever the
    // box counts already call for it (it is dropped again if the keep list of depth k turns out empty).
    // Host record of a level, in 32-bit words: [0..5] pairs of the small, far and keep list (64 bits each),
    // [6,7] far pairs outside the sibling-group M2L tables, [8,9] boxes and largest box of the X tree's new level,
    // [10,11] of the Y tree's, [12,13] far pairs outside the M2L tables of the level (must be none), [14,15] fullest
    // cells at the sorted depth (first division only), [16..31] row statistics of the small and the keep list (eight
    // 64-bit words: what the near field needs to shape its launches).  On the device the first three are the last
    // entries of the list builder's scans; the counters behind [6..15] live in dres and are cleared by the readback
    // that fetches them, the row statistics in drow, eight words per level.
    alignas(8) int hres[32];
    SegmentFetch fetch;
    auto fetch_level_begin = [&](const ListsPending *pend, bool division) {
        memset(hres, 0, sizeof(hres));
        ExportList L;
        if (pend != nullptr && pend->active) {
            for (int c = 0; c < 3; c++) L.add(pend->pos.get() + (c + 1) * pend->stride - 1, 2, 2 * c);
            L.add(dres.get() + 6, 2, 6, true);
            L.add(dres.get() + 12, 2, 12, true);
            L.add(drow.get() + 8 * (P->levels.size() - 1), 16, 16);
        }
        if (division) L.add(dres.get() + 8, sym ? 2 : 4, 8, true);
        if (division && pend == nullptr) L.add(dres.get() + 14, 2, 14, true);      // first division: fullest sorted cells
        fetch.begin(L, s);
    };
    auto fetch_level_wait = [&]() { fetch.wait(hres, s); };
    auto wants_division = [&]() {
        return (float)P->tx.lev.back().maxcount > prm->min_points &&
               (sym || (float)P->ty_.lev.back().maxcount > prm->min_points) && (int)P->tx.lev.size() <= gx.L;
    };
    auto finish_division = [&]() {
        divide_finish(P->tx, hres + 8);
        if (!sym) divide_finish(P->ty_, hres + 10);
    };
    // The points (and the weights of a one-shot product) are moved into sorted order on the second stream while the
    // levels and lists are built here: those are many small kernels that leave the memory system idle, the moves are
    // bound by it.  The order of the first sort is final unless a deep level asks for more key bits to be sorted
    // (level_launch); then the moves wait for that and are done again at the end.
    bool early = false;
    // While work is queued on both streams, blocks that host code gives back are parked (a kernel of the other stream
    // may still use them, and the pool would hand them to the next request); they return to the pool at the end.
    ParkingLot lot;
    const bool two_streams = g_arena == nullptr && !(getenv("F3M_OVERLAP") && atoi(getenv("F3M_OVERLAP")) == 0);
    auto start_early_moves = [&]() {
        SideStream &ss = side_stream();
        F3M_HIP(hipEventRecord(ss.fork, s));
        F3M_HIP(hipStreamWaitEvent(ss.stream, ss.fork, 0));
        gather_tree_points(P->tx, X, ss.stream, /*background=*/true);
        if (!sym) gather_tree_points(P->ty_, Y, ss.stream, /*background=*/true);
        if (b_early != nullptr && c_early >= 1) {
            const long long bstride = P->M + 32;
            P->early_ncol = c_early >= 3 ? std::min(c_early, 4) : c_early;
            const int nc = c_early >= 3 ? 4 : c_early;
            P->early_bs.reset((size_t)bstride * (c_early >= 2 ? 4 : 1));
            if (nc > P->early_ncol) dev_fill(P->early_bs.get(), 0, sizeof(float) * (size_t)bstride * nc, ss.stream);
            gather_columns(b_early, P->ty->perm.get(), P->M, c_early, 0, P->early_ncol, P->early_bs.get(), bstride, ss.stream,
                           /*background=*/true);
            P->early_b = b_early;
            P->early_c = c_early;
            // The result arrays of the product that follows are cleared here as well (and, for a single column on one
            // tree, the fixed-point sums of the symmetric near field; the largest |weight| does not depend on the order
            // of the weights): nothing of this waits for the tree, and what is queued after the last level -- the near
            // field's source operands -- is then all that the near field still waits for.
            P->early_outs.reset((size_t)P->N * (c_early >= 2 ? 4 : 1));
            P->early_outs_far.reset((size_t)P->N * (c_early >= 2 ? 4 : 1));
            dev_fill(P->early_outs.get(), 0, sizeof(float) * (size_t)P->N * nc, ss.stream);
            dev_fill(P->early_outs_far.get(), 0, sizeof(float) * (size_t)P->N * P->early_ncol, ss.stream);
            const char *se = getenv("F3M_NEAR_SYM");
            // (wherever near_symmetric may say yes; with variance compression the near lists are short or empty and the
            // product prepares the sums itself if it turns out to need them)
            const bool maybe_sym = sym && c_early == 1 && d <= 5 && !(se && atoi(se) == 0) && !prm->var_compression;
            if (maybe_sym) {
                P->early_symfix.reset((size_t)P->N);
                P->early_symmax.reset(1);
                dev_fill(P->early_symfix.get(), 0, sizeof(long long) * (size_t)P->N, ss.stream);
                sym_absmax(P->early_bs.get(), P->M, P->early_symmax.get(), ss.stream);
            } else if (out_early != nullptr) {   // the caller's array, for a product that adds its results straight into it
                dev_fill(out_early, 0, sizeof(float) * (size_t)P->N * c_early, ss.stream);
                P->early_out = out_early;
            }
        }
        early = true;
        lot.start();
    };
    // before a division sorts more key bits (which replaces the order arrays the moves read), the moves must be done
    auto settle_early = [&]() {
        if (early && (divide_will_sort(P->tx) || (!sym && divide_will_sort(P->ty_)))) {
            F3M_HIP(hipEventRecord(side_stream().join, side_stream().stream));
            F3M_HIP(hipStreamWaitEvent(s, side_stream().join, 0));
            early = false;
            P->early_b = nullptr;
            P->early_bs.free();
            P->early_outs.free();
            P->early_outs_far.free();
            P->early_symfix.free();
            P->early_symmax.free();
        }
    };
    if (need_tree && wants_division()) {
        settle_early();
        {
            ClassifyParams none = classify_params(*P, 0.f);
            ListsPending nopend;
            level_launch(nullptr, P->tx, *P->ty, 0, none, nopend, nullptr, nullptr, true, dres.get() + 8, dres.get() + 10, s);
        }
        // with the first division's counts, the fullest cell at the depth that the sorted key bits resolve
        // (words [14], [15] of the record)
        if (two_streams) {
            max_run_launch(P->tx, dres.get() + 14, s);
            if (!sym) max_run_launch(P->ty_, dres.get() + 15, s);
        }
        fetch_level_begin(nullptr, true);
        fetch_level_wait();
        finish_division();
        if (two_streams) {
            // A tree whose fullest cell at that depth still calls for division will need more key bits sorted: now,
            // rather than in the middle of the level loop, so that the order of the points is final from here on
            // (deeper trees than that sort again later, and the moves below are then repeated).
            if ((float)hres[14] > prm->min_points) sort_more_bits(P->tx, s);
            if (!sym && (float)hres[15] > prm->min_points) sort_more_bits(P->ty_, s);
            start_early_moves();
        }
        for (;;) {
            const int k = (int)P->tx.lev.size() - 1;
            const float e = P->tx.lev[k].edge;
            P->levels.emplace_back();
            PlanLevel &L = P->levels.back();
            ClassifyParams cp = classify_params(*P, e);
            ListsPending pend;
            F3M_REQUIRE((int)P->levels.size() <= kMaxLevels, 23, "tree deeper than %d levels", kMaxLevels);
            const bool ahead = wants_division();
            if (ahead) settle_early();
            level_launch(keep, P->tx, *P->ty, k, cp, pend, reinterpret_cast<long long *>(dres.get()),
                         drow.get() + 8 * (P->levels.size() - 1), ahead, dres.get() + 8, dres.get() + 10, s);
            // The sizes of the lists travel to the host; the pass that writes the lists is queued behind them, before the
            // host has them, wherever an upper bound of the sizes is a modest allocation: it then runs during the wait.
            fetch_level_begin(&pend, ahead);
            lists_write_early(pend, *keep, P->tx, *P->ty, k, cp, L, s);
            // (Queued after this level's own kernels: the host needs a while for these launches, and the caller's stream
            // should not wait for it.)
            // No further division: this is the deepest level, whose near lists will be summed.  Its source operands
            // are prepared on the second stream (behind the moves of the points) while its lists are built here.
            // (The host has seen the counts of this level's division, so the level's arrays are complete.)
            if (!ahead && early) {
                prepare_near_operands(d, *P->ty, P->ty->lev[k], P->lcs, side_stream().stream);
            }
            fetch_level_wait();
            lists_finish(pend, reinterpret_cast<const long long *>(hres), *keep, P->tx, *P->ty, k, cp, L,
                         reinterpret_cast<const long long *>(hres + 16), s);
            if (ahead) finish_division();
            L.num_nodes = prm->nr_of_interpolation;
            if (prm->var_compression && e * e * P->lcs < 0.01f)      // F3M_src/n_tree.cu:971-978,1022-1025
                L.num_nodes = std::min((int)pow(3, d), prm->nr_of_interpolation);
            keep = &L.keep;
            if (getenv("F3M_DEBUG"))
                fprintf(stderr, "level %d: boxes %d far %lld (outliers %lld) small %lld keep %lld\n", k, P->tx.lev[k].nb, L.far.n,
                        L.far.outliers, L.small_.n, L.keep.n);
            if (ahead && keep->n > 0) continue;
            if (ahead) {
                divide_discard(P->tx);
                if (!sym) divide_discard(P->ty_);
            }
            break;
        }
    }
    if (early) {
        F3M_HIP(hipEventRecord(side_stream().join, side_stream().stream));
        F3M_HIP(hipStreamWaitEvent(s, side_stream().join, 0));       // the work of the second stream is part of the plan
    }
    if (need_tree && !early) {
        gather_tree_points(P->tx, X, s);
        if (!sym) gather_tree_points(P->ty_, Y, s);
    }
    if (P->levels.empty()) {
        P->Xraw.reset((size_t)N * d);
        F3M_HIP(hipMemcpyAsync(P->Xraw.get(), X, sizeof(float) * (size_t)N * d, hipMemcpyDeviceToDevice, s));
        if (!sym) {
            P->Yraw.reset((size_t)M * d);
            F3M_HIP(hipMemcpyAsync(P->Yraw.get(), Y, sizeof(float) * (size_t)M * d, hipMemcpyDeviceToDevice, s));
        }
    }
    if (b_early == nullptr) {
        // a plan that is kept: lists written into blocks sized for an upper bound move into blocks of their own size
        for (PlanLevel &L : P->levels) shrink_lists(L, s);
        F3M_HIP(hipStreamSynchronize(s));
    }
    return P.release();
}

static void check_level(const f3m_plan *P, int level)
{
    F3M_REQUIRE(P != nullptr, 1, "plan is NULL");
    F3M_REQUIRE(level >= 1 && level <= (int)P->levels.size(), 11, "level %d out of range 1..%d", level, (int)P->levels.size());
}

static int m2l_mode_env()
{
    // F3M_M2L=direct|separable forces one form of the M2L kernel (default: separable when its tables fit);
    // F3M_M2L=sibling takes the sibling-group kernel wherever it applies, also at levels with few parents
    int mode = 0;
    if (const char *e = getenv("F3M_M2L"))
        mode = !strcmp(e, "direct") ? 1 : (!strcmp(e, "separable") ? 2 : (!strcmp(e, "sibling") ? 3 : 0));
    return mode;
}

static void far_level(f3m_plan *P, int level, const float *bs, float *outs, float *mom, float *loc, hipStream_t s)
{
    PlanLevel &L = P->levels[level - 1];
    if (L.far.n == 0) return;
    NodeSet &ns = P->nodeset(L.num_nodes, s);
    const int mode = m2l_mode_env();
    far_field(P->d, P->tx, P->tx.lev[level], *P->ty, P->ty->lev[level], L.far, ns, bs, outs, P->lcs, mode, mom, loc, s);
}

// Far field of all levels in one upward and one downward sweep: the points are interpolated once, at
// the deepest level with far pairs; moments of shallower levels come from their children and local
// expansions are handed down to the children, level by level, before one evaluation at the points.
// Where a level has more nodes per dimension than the next deeper one (var_compression lowers the node
// count of small boxes, F3M_src/n_tree.cu:971-978) the hand-over would not be exact, and that level
// is interpolated from / evaluated at the points directly, as the reference does for every level.
// direct (nullable): the one evaluation at the points adds into the caller's array (only where the node counts of the
// levels allow the single evaluation)
static void far_tree(f3m_plan *P, bool transposed, const float *bs, float *outs, hipStream_t s, bool beside_near = false,
                     const DirectOut *direct = nullptr)
{
    const int depth = (int)P->levels.size();
    // targets and sources of this product: the X and Y tree, or the other way round for K(X,Y)^T
    const Tree &TX = transposed ? *P->ty : P->tx, &TY = transposed ? P->tx : *P->ty;
    auto far_of = [&](int k) -> const PairList & { return transposed ? P->levels[k - 1].farT : P->levels[k - 1].far; };
    int ku = 0, kd = 0;
    for (int k = 1; k <= depth; k++)
        if (far_of(k).n > 0) { if (!ku) ku = k; kd = k; }
    if (!ku) return;
    const int mode = m2l_mode_env();
    const int d = P->d;
    auto ns_of = [&](int k) -> NodeSet & { return P->nodeset(P->levels[k - 1].num_nodes, s); };
    std::vector<DBuf<float>> mom((size_t)depth + 1);
    // upward
    for (int k = kd; k >= ku; k--) {
        NodeSet &ns = ns_of(k);
        const TreeLevel &ly = TY.lev[k];
        mom[k].reset((size_t)ly.nb * ns.P);
        if (k < kd && nodes_nest(ns, ns_of(k + 1))) {
            const float *tab = P->shift_table(P->levels[k - 1].num_nodes, P->levels[k].num_nodes, s);
            shift_level(false, ly, TY.lev[k + 1], ns, ns_of(k + 1), tab, mom[k + 1].get(), mom[k].get(), s);
        } else {
            p2m_level(d, TY, ly, nullptr, ns, bs, mom[k].get(), s);
        }
    }
    // downward
    DBuf<float> loc, prev;
    int pending = 0;        // level whose local expansions (in prev) still wait to be evaluated
    for (int k = ku; k <= kd; k++) {
        NodeSet &ns = ns_of(k);
        const TreeLevel &lx = TX.lev[k];
        loc.reset((size_t)lx.nb * ns.P);
        m2l_level(d, TX, lx, TY, TY.lev[k], far_of(k), ns, P->lcs, mode, mom[k].get(), loc.get(), s, beside_near);
        mom[k].free();
        if (pending) {
            NodeSet &nsp = ns_of(pending);
            if (nodes_nest(nsp, ns)) {
                const float *tab = P->shift_table(P->levels[pending - 1].num_nodes, P->levels[k - 1].num_nodes, s);
                shift_level(true, TX.lev[pending], lx, nsp, ns, tab, prev.get(), loc.get(), s);
            } else {
                F3M_REQUIRE(direct == nullptr, 36, "direct output with more than one evaluation of the far field");
                l2p_level(d, TX, TX.lev[pending], nullptr, nsp, prev.get(), outs, s);
            }
        }
        std::swap(loc, prev);
        pending = k;
    }
    l2p_level(d, TX, TX.lev[pending], nullptr, ns_of(pending), prev.get(), outs, s, direct);
}

// The lists seen from the Y boxes, for the transposed product (built once, on its first use).
static void ensure_transposed_lists(f3m_plan *P, hipStream_t s)
{
    if (P->symmetric) return;          // one tree: K and every list are symmetric
    for (size_t l = 0; l < P->levels.size(); l++) {
        PlanLevel &L = P->levels[l];
        if (L.haveT) continue;
        require_tables_may_be_built("the transposed lists");
        const TreeLevel &ly = P->ty->lev[l + 1];
        transpose_list(L.far, ly, L.farT, s);
        transpose_list(L.small_, ly, L.smallT, s);
        // only the keep list of the last level is ever summed
        if (l + 1 == P->levels.size()) transpose_list(L.keep, ly, L.keepT, s);
        L.haveT = true;
    }
}

// waits for the stream, except while it is being captured into a graph (where a wait is an error and
// the work has not run anyway)
static void finish_stream(hipStream_t s)
{
#ifndef F3M_CPU_EMU
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone) return;
    (void)hipGetLastError();
#endif
    F3M_HIP(hipStreamSynchronize(s));
}

// out = K(X,Y) b, or with `transposed` out = K(X,Y)^T b (b then has N rows and out M): the same trees
// with the roles of targets and sources swapped and every list seen from its Y boxes.
static void plan_apply(f3m_plan *P, const float *b, int c, float *out, hipStream_t s, bool transposed = false)
{
    F3M_REQUIRE(P != nullptr, 1, "plan is NULL");
    F3M_REQUIRE(c >= 1, 12, "b has no columns");
    check_device_ptr(b, "b");
    check_device_ptr(out, "out");
    if (P->symmetric) transposed = false;           // K(X,X) is symmetric
    if (P->levels.empty()) {
        const float *Yp = P->symmetric ? P->Xraw.get() : P->Yraw.get();
        Scope sc(kNear, s);
        if (transposed) exact_f32(P->d, Yp, P->M, P->Xraw.get(), P->N, b, c, P->prm.ls, false, out, s);
        else exact_f32(P->d, P->Xraw.get(), P->N, Yp, P->M, b, c, P->prm.ls, false, out, s);
        finish_stream(s);
        return;
    }
    if (transposed) ensure_transposed_lists(P, s);
    const Tree &TX = transposed ? *P->ty : P->tx, &TY = transposed ? P->tx : *P->ty;     // targets, sources
    const long long NT = TX.n, NS = TY.n;
    auto small_of = [&](int k) -> const PairList & { return transposed ? P->levels[k - 1].smallT : P->levels[k - 1].small_; };
    auto keep_of = [&](int k) -> const PairList & { return transposed ? P->levels[k - 1].keepT : P->levels[k - 1].keep; };
    // Columns are taken four at a time while at least three are left (the near field then computes every
    // exponential once for the four), two at a time when two are left, else one.  bs columns are padded by one tile:
    // near_g_kernel reads whole tiles.
    const long long bstride = NS + 32, ostride = NT;
    const int width = c >= 2 ? 4 : 1;
    DBuf<float> bs((size_t)bstride * width), outs((size_t)ostride * width);
    const int depth = (int)P->levels.size();
    // F3M_FAR=levels: interpolate every level from the points like the reference (cross-check)
    const char *fe = getenv("F3M_FAR");
    const bool per_level = fe && !strcmp(fe, "levels") && !transposed;
    // The far field runs on a second stream beside the near field and adds its share when the result is
    // scattered (F3M_OVERLAP=0: one stream).  Not for a call whose temporaries come from an arena (it would need
    // one more array of N floats per column) and not for the per-level cross-check.
    bool overlap = false;
    {
        bool any_far = false;
        for (int k = 1; k <= depth; k++) any_far = any_far || (transposed ? P->levels[k - 1].farT.n : P->levels[k - 1].far.n) > 0;
        const char *oe = getenv("F3M_OVERLAP");
        overlap = any_far && !per_level && g_arena == nullptr && !(oe && atoi(oe) == 0);
        // Five dimensions, symmetric near field: the far field follows the near field on the caller's stream.  Both are
        // bound by the vector ALU there (M2L on 3^5 nodes takes 6 ms alone), beside each other they take as long as one
        // after the other, and M2L has its faster form (whole families of siblings per workgroup) only alone on the GPU:
        // N=1e7: 38.3 ms against 45.8 with the far field beside the (shorter) symmetric near field.
        if (overlap && P->symmetric && c == 1 && P->d == 5 &&
            near_symmetric(P->d, TX, TX.lev[depth], TY, small_of(depth), P->lcs, 1))
            overlap = false;
    }
    // Where the whole near field is one launch in which every target belongs to one wavefront, and the far field is
    // evaluated at the points once, both add their sums straight into the caller's array (cleared before; two additions
    // per element, so their order does not matter) and the pass that scatters the sorted results is not needed: the
    // scattered writes happen inside the two long kernels instead of after them.  F3M_DIRECT=0 turns it off.
    bool direct = false;
    const bool b_out_overlap = reinterpret_cast<const char *>(b) < reinterpret_cast<const char *>(out) + sizeof(float) * (size_t)NT * c &&
                               reinterpret_cast<const char *>(out) < reinterpret_cast<const char *>(b) + sizeof(float) * (size_t)NS * c;
    if (overlap && !b_out_overlap && !(getenv("F3M_DIRECT") && atoi(getenv("F3M_DIRECT")) == 0)) {
        int ku = 0, kd = 0;
        bool same_nodes = true;
        for (int k = 1; k <= depth; k++)
            if ((transposed ? P->levels[k - 1].farT.n : P->levels[k - 1].far.n) > 0) {
                if (kd && P->levels[k - 1].num_nodes != P->levels[kd - 1].num_nodes) same_nodes = false;
                if (!ku) ku = k;
                kd = k;
            }
        int nlists = 0;
        direct = same_nodes;
        for (int k = 1; k <= depth && direct; k++) {
            const PairList *ls[2] = {&small_of(k), k == depth ? &keep_of(depth) : nullptr};
            for (const PairList *l : ls) {
                if (l == nullptr || l->n == 0) continue;
                nlists++;
                // every column group of this product (four columns while three or more are left, then two or one)
                for (int left = c; left > 0 && direct;) {
                    const int nc = left >= 3 ? 4 : (left == 2 ? 2 : 1);
                    direct = near_single_pass(P->d, TX, TX.lev[k], *l, P->lcs, nc) &&
                             !near_symmetric(P->d, TX, TX.lev[k], TY, *l, P->lcs, nc);
                    left -= std::min(nc, left);
                }
            }
        }
        direct = direct && nlists == 1;          // (without a near field to hide them, the atomic additions of the far field alone take longer than the pass they replace: 0.50 against 0.13 + 0.17 ms)
    }
    // F3M_DIRECT=2 (testing aid): fail where the results cannot go straight into the caller's array
    F3M_REQUIRE(direct || !(getenv("F3M_DIRECT") && atoi(getenv("F3M_DIRECT")) == 2), 37,
                "F3M_DIRECT=2: this product does not qualify for direct output");
    if (direct) {
        if (!(P->early_out == out && P->early_c == c && !transposed)) {
            Scope sc(kPerm, s);
            dev_fill(out, 0, sizeof(float) * (size_t)NT * c, s);
        }
        P->early_out = nullptr;
    }
    DBuf<float> outs_far;
    if (overlap) {
        if (!direct) outs_far.reset((size_t)ostride * width);
        // The one table that kernels of both streams read has to exist before the streams part: L2P starts from the
        // box table of the deepest level with far pairs (and of every level with far pairs where the node counts
        // change between levels, since such levels are evaluated at the points themselves).
        int ku = 0, kd = 0;
        bool same_nodes = true;
        for (int k = 1; k <= depth; k++)
            if ((transposed ? P->levels[k - 1].farT.n : P->levels[k - 1].far.n) > 0) {
                if (!ku) ku = k;
                if (kd && P->levels[k - 1].num_nodes != P->levels[kd - 1].num_nodes) same_nodes = false;
                kd = k;
            }
        for (int k = same_nodes ? kd : ku; k <= kd; k++) ensure_box_table(TX.lev[k], NT, s);
    }
    // A call whose temporaries come from an arena runs on one stream, so the temporaries of a column group (and of one
    // column's far field) can take the place of the previous one's: the need does not grow with the number of columns,
    // and the first group, which has the most columns, is the one that decides whether the product fits -- before
    // anything has been written to `out`.
    // The symmetric near field (one tree, a single column: half the exponentials) adds the sums of its second direction
    // as fixed-point numbers into an array of their own, which the scatter pass folds in.  With an arena only where
    // that array is a small part of it (a product that fits without must not be refused because of it).
    DBuf<long long> symfix;
    DBuf<unsigned> symmax;
    const size_t group_mark = arena_mark();
    for (int col = 0; col < c;) {
        arena_rewind(group_mark);
        const int left = c - col;
        const int nc = left >= 3 ? 4 : (left == 2 ? 2 : 1);   // columns of this pass (past `left`: zero weights)
        const int ncol = std::min(nc, left);
        bool use_sym = false;
        if (P->symmetric && nc == 1) {
            for (int k = 1; k <= depth && !use_sym; k++)
                use_sym = near_symmetric(P->d, TX, TX.lev[k], TY, small_of(k), P->lcs, nc) ||
                          (k == depth && near_symmetric(P->d, TX, TX.lev[k], TY, keep_of(k), P->lcs, nc));
            if (g_arena != nullptr && sizeof(long long) * (size_t)NT > (g_arena->cap - g_arena->used) / 4) use_sym = false;
        }
        // (prepared while the plan was built, together with this group's weights and cleared result arrays)
        const bool sym_early = use_sym && col == 0 && !transposed && P->early_b == b && P->early_c == c && P->early_ncol == ncol &&
                               P->early_bs.size() > 0 && P->early_outs.size() > 0 && P->early_symfix.size() > 0;
        SymSums symsums;
        if (sym_early) {
            std::swap(symfix, P->early_symfix);
            std::swap(symmax, P->early_symmax);
        } else if (use_sym) {
            symfix.reset((size_t)NT);
            symmax.reset(1);
        }
        P->early_symfix.free();
        P->early_symmax.free();
        if (use_sym) {
            symsums.fix = symfix.get();
            symsums.absmax = symmax.get();
            symsums.nsrc = NS;
            symsums.small_far = true;               // the far field's workgroups are single small wavefronts up to 4 x 4 x 4 nodes
            for (int k = 1; k <= depth; k++)
                if (P->levels[k - 1].far.n > 0 && P->levels[k - 1].num_nodes > 64) symsums.small_far = false;
        }
        const SymSums *sym = use_sym ? &symsums : nullptr;
        {
            Scope sc(kPerm, s);
            bool cleared = false;
            if (col == 0 && !transposed && P->early_b == b && P->early_c == c && P->early_ncol == ncol && P->early_bs.size() > 0) {
                std::swap(bs, P->early_bs);                 // this group's weights were put in order while the plan was built
                P->early_b = nullptr;
                P->early_bs.free();
                if (P->early_outs.size() > 0) {             // and its result arrays cleared
                    std::swap(outs, P->early_outs);
                    if (overlap && !direct) std::swap(outs_far, P->early_outs_far);
                    P->early_outs.free();
                    P->early_outs_far.free();
                    cleared = true;
                }
            } else {
                if (nc > ncol) dev_fill(bs.get(), 0, sizeof(float) * (size_t)bstride * nc, s);
                gather_columns(b, TY.perm.get(), NS, c, col, ncol, bs.get(), bstride, s);
            }
            if (!cleared && !direct) {
                dev_fill(outs.get(), 0, sizeof(float) * (size_t)ostride * nc, s);
                if (overlap) dev_fill(outs_far.get(), 0, sizeof(float) * (size_t)ostride * ncol, s);
            }
            if (use_sym && !sym_early) {
                dev_fill(symfix.get(), 0, sizeof(long long) * (size_t)NT, s);
                sym_absmax(bs.get(), NS, symmax.get(), s);
            }
        }
        // Every temporary that is given back while this column group is being queued is parked until the streams
        // have joined: work queued on one stream may still use a block when host code of the other asks for memory.
        {
            ParkingLot lot;
            lot.start();
            // The lists of the deepest level come first: they are the long launches, and their tables are ready or
            // nearly so (the plan prepared the source operands beside its level loop).  The tables of the shallower
            // levels' lists (kept with the plan from then on) are built on the second stream meanwhile, ahead of the
            // far field; those lists follow on the caller's stream once their tables are there.  The order of the
            // launches, and with it the order in which a target's sums are added, is the same on one stream.
            const bool deepest_only_list = keep_of(depth).n == 0;
            if (overlap) {
                near_field(P->d, TX, TX.lev[depth], TY, TY.lev[depth], small_of(depth), bs.get(), outs.get(), P->lcs, s, nc,
                           bstride, ostride, /*only_list=*/deepest_only_list, /*prepare_only=*/true);
                near_field(P->d, TX, TX.lev[depth], TY, TY.lev[depth], keep_of(depth), bs.get(), outs.get(), P->lcs, s, nc,
                           bstride, ostride, false, /*prepare_only=*/true);
                F3M_HIP(hipEventRecord(side_stream().fork, s));
                F3M_HIP(hipStreamWaitEvent(side_stream().stream, side_stream().fork, 0));
            }
            DirectOut dnear;
            if (direct) { dnear.perm = TX.perm.get(); dnear.out = out; dnear.c = c; dnear.col = col; dnear.ncol = ncol; }
            const DirectOut *dn = direct ? &dnear : nullptr;
            if (per_level) {
                for (int k = 1; k <= depth; k++) {
                    // F3M_src/n_tree.cu:1018-1051: exact sums of the small pairs, then the far field
                    near_field(P->d, TX, TX.lev[k], TY, TY.lev[k], small_of(k), bs.get(), outs.get(), P->lcs, s, nc,
                               bstride, ostride, /*only_list=*/k < depth || deepest_only_list, false, dn, sym);
                    const size_t mark = arena_mark();
                    for (int q = 0; q < ncol; q++) {
                        arena_rewind(mark);
                        far_level(P, k, bs.get() + q * bstride, outs.get() + q * ostride, nullptr, nullptr, s);
                    }
                }
                // F3M_src/n_tree.cu:1092-1094: what is still "keep" after the last division is summed exactly
                near_field(P->d, TX, TX.lev[depth], TY, TY.lev[depth], keep_of(depth), bs.get(),
                           outs.get(), P->lcs, s, nc, bstride, ostride, false, false, dn, sym);
            } else {
                // F3M_src/n_tree.cu:1018-1051 and :1092-1094: exact sums of the small pairs of every level and of what
                // is still "keep" after the last division
                near_field(P->d, TX, TX.lev[depth], TY, TY.lev[depth], small_of(depth), bs.get(), outs.get(), P->lcs, s, nc,
                           bstride, ostride, /*only_list=*/deepest_only_list, false, dn, sym);
                near_field(P->d, TX, TX.lev[depth], TY, TY.lev[depth], keep_of(depth), bs.get(),
                           outs.get(), P->lcs, s, nc, bstride, ostride, false, false, dn, sym);
                if (overlap) {       // (queued after the long launches: the host needs a while for these many small kernels)
                    for (int k = 1; k < depth; k++)
                        near_field(P->d, TX, TX.lev[k], TY, TY.lev[k], small_of(k), bs.get(), outs.get(), P->lcs,
                                   side_stream().stream, nc, bstride, ostride, /*only_list=*/true, /*prepare_only=*/true);
                    F3M_HIP(hipEventRecord(side_stream().tables, side_stream().stream));
                    F3M_HIP(hipStreamWaitEvent(s, side_stream().tables, 0));
                }
                for (int k = 1; k < depth; k++)
                    near_field(P->d, TX, TX.lev[k], TY, TY.lev[k], small_of(k), bs.get(), outs.get(), P->lcs, s, nc,
                               bstride, ostride, /*only_list=*/true, false, dn, sym);
            }
            // the far field: beside the near field on the second stream into its own array, or after it on the one
            // stream; either way a result is (near sums) + (far sum)
            if (!per_level) {
                hipStream_t fs = s;
                float *fo = outs.get();
                if (overlap) { fs = side_stream().stream; fo = outs_far.get(); }
                const size_t mark = arena_mark();
                for (int q = 0; q < ncol; q++) {
                    arena_rewind(mark);
                    DirectOut dfar = dnear;
                    dfar.col = col + q;
                    dfar.ncol = 1;
                    far_tree(P, transposed, bs.get() + q * bstride, fo + q * ostride, fs, overlap, direct ? &dfar : nullptr);
                }
            }
            if (overlap) {
                F3M_HIP(hipEventRecord(side_stream().join, side_stream().stream));
                F3M_HIP(hipStreamWaitEvent(s, side_stream().join, 0));
            }
            Scope sc(kPerm, s);
            if (!direct)
                scatter_columns(outs.get(), overlap ? outs_far.get() : nullptr, ostride, TX.perm.get(), NT, c, col, ncol, out, s, sym);
        }
        col += ncol;
    }
    finish_stream(s);
}

// A call that fails may have queued work on the caller's stream and on the library's second stream, and the
// buffers of that work have gone back to the pool while the error travelled up here: nothing may reuse them before
// the device is idle.  Not while the call's stream is being captured into a graph: nothing has run then, a device-wide
// wait is an error during capture (and would invalidate it), and such a call takes its temporaries from static memory.
static thread_local hipStream_t g_call_stream = nullptr;
static void settle_after_error()
{
#ifndef F3M_CPU_EMU
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    const bool capturing = hipStreamIsCapturing(g_call_stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone;
    (void)hipGetLastError();
    if (capturing) return;
    (void)hipDeviceSynchronize();
    (void)hipGetLastError();
#endif
}

template <typename F>
static int guarded(F f)
{
    try {
        f();
        return 0;
    } catch (const Error &e) {
        g_error = e.what();
        settle_after_error();
        return e.code;
    } catch (const std::exception &e) {
        g_error = e.what();
        settle_after_error();
        return 99;
    }
}

}  // namespace f3m

// timing hooks used by f3m_field.hip
namespace f3m {
void timer_begin(int stage, hipStream_t s) { g_timer.begin(stage, s); }
void timer_end(hipStream_t s) { g_timer.end(s); }
}  // namespace f3m

extern "C" {

int f3m_kmvm_f32(int d, const float *X, int64_t N, const float *Y, int64_t M, const float *b, int c,
                 const f3m_params *params, float *out, void *stream)
{
    return guarded([&] {
        hipStream_t s = (hipStream_t)stream;
        g_timer.reset();
        std::unique_ptr<f3m_plan> P(plan_create(d, X, N, Y, M, params, s, b, c, out));
        plan_apply(P.get(), b, c, out, s);
        g_timer.collect();
    });
}

int f3m_exact_f32(int d, const float *X, int64_t N, const float *Y, int64_t M, const float *b, int c, float ls,
                  float *out, void *stream)
{
    return guarded([&] {
        F3M_REQUIRE(d >= 1 && d <= kMaxD, 2, "dimension must be 1..10 (got %d)", d);
        F3M_REQUIRE(N >= 0 && M >= 0 && c >= 1, 3, "bad shape");
        F3M_REQUIRE(ls > 0.f, 5, "ls must be positive");
        if (N == 0) return;
        check_device_ptr(X, "X"); check_device_ptr(out, "out");
        if (M > 0) { check_device_ptr(Y, "Y"); check_device_ptr(b, "b"); }
        exact_f32(d, X, N, Y, M, b, c, ls, false, out, (hipStream_t)stream);
        F3M_HIP(hipStreamSynchronize((hipStream_t)stream));
    });
}

int f3m_exact_grad_f32(int d, const float *X, int64_t N, const float *Y, int64_t M, const float *b, int c, float ls,
                       float *out, void *stream)
{
    return guarded([&] {
        F3M_REQUIRE(d >= 1 && d <= kMaxD, 2, "dimension must be 1..10 (got %d)", d);
        F3M_REQUIRE(N >= 0 && M >= 0 && c >= 1, 3, "bad shape");
        F3M_REQUIRE(ls > 0.f, 5, "ls must be positive");
        if (N == 0) return;
        check_device_ptr(X, "X"); check_device_ptr(out, "out");
        if (M > 0) { check_device_ptr(Y, "Y"); check_device_ptr(b, "b"); }
        exact_f32(d, X, N, Y, M, b, c, ls, true, out, (hipStream_t)stream);
        F3M_HIP(hipStreamSynchronize((hipStream_t)stream));
    });
}

int f3m_exact_f64(int d, const double *X, int64_t N, const double *Y, int64_t M, const double *b, int c, double ls,
                  double *out, void *stream)
{
    return guarded([&] {
        F3M_REQUIRE(d >= 1 && d <= kMaxD, 2, "dimension must be 1..10 (got %d)", d);
        F3M_REQUIRE(N >= 0 && M >= 0 && c >= 1, 3, "bad shape");
        F3M_REQUIRE(ls > 0., 5, "ls must be positive");
        if (N == 0) return;
        check_device_ptr(X, "X"); check_device_ptr(out, "out");
        if (M > 0) { check_device_ptr(Y, "Y"); check_device_ptr(b, "b"); }
        exact_f64(d, X, N, Y, M, b, c, ls, out, (hipStream_t)stream);
        F3M_HIP(hipStreamSynchronize((hipStream_t)stream));
    });
}

int f3m_plan_create(int d, const float *X, int64_t N, const float *Y, int64_t M, const f3m_params *params, void *stream,
                    f3m_plan **plan)
{
    return guarded([&] {
        F3M_REQUIRE(plan != nullptr, 1, "plan is NULL");
        *plan = nullptr;
        g_timer.reset();
        *plan = plan_create(d, X, N, Y, M, params, (hipStream_t)stream);
        g_timer.collect();
    });
}

int f3m_plan_apply(f3m_plan *plan, const float *b, int c, float *out, void *stream)
{
    return guarded([&] {
        g_timer.reset();
        plan_apply(plan, b, c, out, (hipStream_t)stream);
        g_timer.collect();
    });
}

int f3m_plan_apply_transpose(f3m_plan *plan, const float *u, int c, float *out, void *stream)
{
    return guarded([&] {
        g_timer.reset();
        plan_apply(plan, u, c, out, (hipStream_t)stream, /*transposed=*/true);
        g_timer.collect();
    });
}

// ---- the entry point that allocates nothing ---------------------------------------------------
// Its temporaries (the sorted copies of b and of the result, moments and local expansions, partial sums)
// come from this array, one copy per GPU, which the device holds from the moment the library is loaded.
// In host code the name `scratch` is only a handle for hipGetSymbolAddress: the device address is asked
// for once per device and kept.
constexpr size_t kScratchBytes = (size_t)128 << 20;
#ifndef F3M_CPU_EMU
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
#else
alignas(256) static unsigned char scratch[kScratchBytes];
#endif

namespace f3m {
static void *scratch_address()
{
    static std::mutex mu;
    static std::map<int, void *> addr;        // device -> address of that device's copy of the array
    int dev = 0;
    F3M_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> g(mu);
    auto it = addr.find(dev);
    if (it != addr.end()) return it->second;
    void *ptr = nullptr;
#ifndef F3M_CPU_EMU
    F3M_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
#else
    ptr = scratch;
#endif
    F3M_REQUIRE(ptr != nullptr, 100, "no device address for the static scratch memory");
    addr[dev] = ptr;
    return ptr;
}
}  // namespace f3m

int f3m_plan_apply_noalloc(f3m_plan *plan, const float *b, int c, float *out, void *stream)
{
    g_call_stream = (hipStream_t)stream;
    const int rc = guarded([&] {
        F3M_REQUIRE(plan != nullptr, 1, "plan is NULL");
        F3M_REQUIRE(c >= 1, 12, "b has no columns");
        // what the call needs at the least: the sorted copies of b and of the result
        const size_t width = c >= 2 ? 4 : 1;
        const size_t least = plan->levels.empty() ? 0 : sizeof(float) * width * ((size_t)plan->M + 32 + (size_t)plan->N);
        F3M_REQUIRE(least <= kScratchBytes, 42,
                    "f3m_plan_apply_noalloc: a product with N=%lld, M=%lld, c=%d needs more than %zu MiB of scratch memory; the "
                    "static scratch memory holds %zu MiB (use f3m_plan_apply)", plan->N, plan->M, c, least >> 20, kScratchBytes >> 20);
        Arena arena;
        arena.base = static_cast<char *>(scratch_address());
        arena.cap = kScratchBytes;
        arena.owner = "f3m_plan_apply_noalloc";
        ArenaScope scope(&arena);
        const bool timing = g_timer.enabled;      // stage timing creates events: off for this call
        g_timer.enabled = false;
        try {
            plan_apply(plan, b, c, out, (hipStream_t)stream);
        } catch (...) {
            g_timer.enabled = timing;
            throw;
        }
        g_timer.enabled = timing;
    });
    g_call_stream = nullptr;
    return rc;
}

int f3m_plan_destroy(f3m_plan *plan)
{
    return guarded([&] { delete plan; });
}

int f3m_plan_depth(const f3m_plan *plan) { return plan ? (int)plan->levels.size() : -1; }
int f3m_plan_symmetric(const f3m_plan *plan) { return plan ? (plan->symmetric ? 1 : 0) : -1; }

int f3m_plan_level_sizes(const f3m_plan *plan, int level, int64_t *sizes, float *edge)
{
    return guarded([&] {
        check_level(plan, level);
        const PlanLevel &L = plan->levels[level - 1];
        sizes[0] = plan->tx.lev[level].nb;
        sizes[1] = plan->ty->lev[level].nb;
        sizes[2] = L.far.n;
        sizes[3] = L.small_.n;
        sizes[4] = L.keep.n;
        sizes[5] = L.num_nodes;
        sizes[6] = plan->tx.lev[level].maxcount;
        sizes[7] = plan->ty->lev[level].maxcount;
        if (edge) *edge = plan->tx.lev[level].edge;
    });
}

int f3m_plan_list_rows(const f3m_plan *plan, int level, int64_t *rows)
{
    return guarded([&] {
        check_level(plan, level);
        F3M_REQUIRE(rows != nullptr, 1, "rows is NULL");
        const PlanLevel &L = plan->levels[level - 1];
        const PairList *l[2] = {&L.small_, &L.keep};
        for (int c = 0; c < 2; c++) {
            rows[4 * c + 0] = l[c]->rows, rows[4 * c + 1] = l[c]->row_points;
            rows[4 * c + 2] = l[c]->items128, rows[4 * c + 3] = l[c]->items160;
        }
    });
}

int f3m_plan_level_copy(const f3m_plan *plan, int level, int which, void *dst, void *stream)
{
    return guarded([&] {
        check_level(plan, level);
        F3M_REQUIRE(dst != nullptr, 1, "dst is NULL");
        hipStream_t s = (hipStream_t)stream;
        const PlanLevel &L = plan->levels[level - 1];
        const TreeLevel &lx = plan->tx.lev[level], &ly = plan->ty->lev[level];
        const int d = plan->d;
        switch (which) {
        case F3M_CENTERS_X: d2h((float *)dst, lx.ctr.get(), (size_t)lx.nb * d, s); break;
        case F3M_CENTERS_Y: d2h((float *)dst, ly.ctr.get(), (size_t)ly.nb * d, s); break;
        case F3M_OFFSETS_X: d2h((int *)dst, lx.off.get(), (size_t)lx.nb + 1, s); break;
        case F3M_OFFSETS_Y: d2h((int *)dst, ly.off.get(), (size_t)ly.nb + 1, s); break;
        case F3M_LIST_FAR: if (L.far.n) d2h((int *)dst, L.far.pairs.get(), (size_t)L.far.n * 2, s); break;
        case F3M_LIST_SMALL: if (L.small_.n) d2h((int *)dst, L.small_.pairs.get(), (size_t)L.small_.n * 2, s); break;
        case F3M_LIST_KEEP: if (L.keep.n) d2h((int *)dst, L.keep.pairs.get(), (size_t)L.keep.n * 2, s); break;
        case F3M_PERM_X: d2h((int *)dst, plan->tx.perm.get(), (size_t)plan->N, s); break;
        case F3M_PERM_Y: d2h((int *)dst, plan->ty->perm.get(), (size_t)plan->M, s); break;
        default: throw Error(13, "unknown level array");
        }
    });
}

int f3m_plan_far_level(f3m_plan *plan, int level, const float *b, int c, float *out, float *mom, float *loc, void *stream)
{
    return guarded([&] {
        check_level(plan, level);
        hipStream_t s = (hipStream_t)stream;
        check_device_ptr(b, "b"); check_device_ptr(out, "out");
        DBuf<float> bs((size_t)plan->M + 32), outs((size_t)plan->N);
        PlanLevel &L = plan->levels[level - 1];
        int P = L.far.n ? plan->nodeset(L.num_nodes, s).P : 0;
        for (int col = 0; col < c; col++) {
            gather_column(b, plan->ty->perm.get(), plan->M, c, col, bs.get(), s);
            dev_fill(outs.get(), 0, sizeof(float) * (size_t)plan->N, s);
            far_level(plan, level, bs.get(), outs.get(),
                      mom ? mom + (size_t)col * plan->ty->lev[level].nb * P : nullptr,
                      loc ? loc + (size_t)col * plan->tx.lev[level].nb * P : nullptr, s);
            scatter_column(outs.get(), plan->tx.perm.get(), plan->N, c, col, out, s);
        }
        F3M_HIP(hipStreamSynchronize(s));
    });
}

int f3m_plan_near_level(f3m_plan *plan, int level, int which, const float *b, int c, float *out, void *stream)
{
    return guarded([&] {
        check_level(plan, level);
        F3M_REQUIRE(which == F3M_LIST_SMALL || which == F3M_LIST_KEEP, 13, "which must be F3M_LIST_SMALL or F3M_LIST_KEEP");
        hipStream_t s = (hipStream_t)stream;
        check_device_ptr(b, "b"); check_device_ptr(out, "out");
        DBuf<float> bs((size_t)plan->M + 32), outs((size_t)plan->N);
        PlanLevel &L = plan->levels[level - 1];
        for (int col = 0; col < c; col++) {
            gather_column(b, plan->ty->perm.get(), plan->M, c, col, bs.get(), s);
            dev_fill(outs.get(), 0, sizeof(float) * (size_t)plan->N, s);
            near_field(plan->d, plan->tx, plan->tx.lev[level], *plan->ty, plan->ty->lev[level],
                       which == F3M_LIST_SMALL ? L.small_ : L.keep, bs.get(), outs.get(), plan->lcs, s);
            scatter_column(outs.get(), plan->tx.perm.get(), plan->N, c, col, out, s);
        }
        F3M_HIP(hipStreamSynchronize(s));
    });
}

int f3m_plan_work(const f3m_plan *plan, double *w)
{
    return guarded([&] {
        F3M_REQUIRE(plan != nullptr && w != nullptr, 1, "NULL argument");
        // computed on the host from copies of the lists and offsets
        w[0] = w[1] = w[2] = w[3] = w[4] = 0.0;
        const int depth = (int)plan->levels.size();
        if (depth == 0) { w[0] = (double)plan->N * (double)plan->M; return; }
        hipStream_t s = nullptr;
        for (int k = 1; k <= depth; k++) {
            const PlanLevel &L = plan->levels[k - 1];
            const TreeLevel &lx = plan->tx.lev[k], &ly = plan->ty->lev[k];
            std::vector<int> ox((size_t)lx.nb + 1), oy((size_t)ly.nb + 1);
            d2h(ox.data(), lx.off.get(), ox.size(), s);
            d2h(oy.data(), ly.off.get(), oy.size(), s);
            auto pair_sum = [&](const PairList &l) {
                double acc = 0;
                if (!l.n) return acc;
                std::vector<int> h((size_t)l.n * 2);
                d2h(h.data(), l.pairs.get(), h.size(), s);
                for (long long t = 0; t < l.n; t++)
                    acc += (double)(ox[h[2 * t] + 1] - ox[h[2 * t]]) * (double)(oy[h[2 * t + 1] + 1] - oy[h[2 * t + 1]]);
                return acc;
            };
            w[0] += pair_sum(L.small_);
            if (k == depth) w[0] += pair_sum(L.keep);
            w[1] += (double)L.far.n;
            w[4] += pair_sum(L.far);
            if (L.far.n) {
                std::vector<int> h((size_t)L.far.n * 2);
                d2h(h.data(), L.far.pairs.get(), h.size(), s);
                std::vector<char> ux(lx.nb, 0), uy(ly.nb, 0);
                for (long long t = 0; t < L.far.n; t++) { ux[h[2 * t]] = 1; uy[h[2 * t + 1]] = 1; }
                for (int bx = 0; bx < lx.nb; bx++) if (ux[bx]) w[2] += ox[bx + 1] - ox[bx];
                for (int by = 0; by < ly.nb; by++) if (uy[by]) w[2] += oy[by + 1] - oy[by];
                int P = 1;
                {
                    NodeSet tmp;
                    // node count of the level without touching the device
                    float ref_val = (float)pow((double)L.num_nodes, 1.0 / (double)(float)plan->d);
                    int hi = (int)std::ceil(ref_val), lo = (int)std::floor(ref_val), acc = 1;
                    for (int i = 0; i < plan->d; i++) {
                        int fut = (int)((double)acc * pow((double)lo, (double)(plan->d - (i + 1))) * (double)hi);
                        int pick = fut <= L.num_nodes ? hi : lo;
                        if (pick < 1) pick = 1;
                        acc *= pick;
                    }
                    P = acc;
                }
                w[3] += (double)L.far.n * (double)P * (double)P;
            }
        }
    });
}

int f3m_plan_lookup_boxes(f3m_plan *plan, int level, int tree, const int32_t *cells, int64_t n, int32_t *ids, void *stream)
{
    return guarded([&] {
        check_level(plan, level);
        F3M_REQUIRE(tree == 0 || tree == 1, 13, "tree must be 0 (X) or 1 (Y)");
        F3M_REQUIRE(n >= 0, 13, "negative count");
        hipStream_t s = (hipStream_t)stream;
        if (n > 0) { check_device_ptr(cells, "cells"); check_device_ptr(ids, "ids"); }
        const Tree &t = tree == 0 ? plan->tx : *plan->ty;
        lookup_boxes(t, t.lev[level], cells, n, ids, s);
        F3M_HIP(hipStreamSynchronize(s));
    });
}

uint32_t f3m_hash_slot(uint32_t key, uint32_t capacity) { return capacity > 1 ? hash_slot_host(key, capacity) : 0u; }

int f3m_set_timing(int enabled)
{
    g_timer.enabled = enabled != 0;
    return 0;
}

int f3m_get_timing(double *t, int *n)
{
    for (int i = 0; i < kNumStages; i++) {
        if (t) t[i] = g_timer.t[i];
        if (n) n[i] = g_timer.n[i];
    }
    return 0;
}

const char *f3m_last_error(void) { return g_error.c_str(); }

int f3m_release_cache(void)
{
    return guarded([&] { Pool::get().release_cached(); });
}

const char *f3m_version(void) { return "f3m-gfx950 0.1"; }

}  // extern "C"
