// Internal interfaces between the engine's translation units.
//   f3m_geom.hip  : bounding box, Morton keys, counting sort, tree levels, interaction lists
//                   (compiled with -ffp-contract=off: every fp32 operation rounds once)
//   f3m_field.hip : exact products, near field, P2M / M2L / L2P
//   f3m_plan.hip  : host orchestration and the C ABI
#pragma once
#include "f3m_rt.h"

#include <cmath>

namespace f3m {

struct Geo {
    float origin[kMaxD];
    float edge0;
    int d;
    int L;   // key depth: number of levels encoded in a Morton key (d*L <= 31)
};

struct TreeLevel {
    int depth = 0;
    float edge = 0.f;
    int nb = 0;          // non-empty boxes
    int maxcount = 0;
    DBuf<int> off;       // nb+1 offsets into the Morton-sorted point order
    DBuf<uint32_t> prefix;  // nb Morton prefixes (depth*d bits)
    DBuf<float> ctr;     // nb*d box centres, row-major
    DBuf<int> cell;      // nb*d integer cell coordinates of the box at its depth
    DBuf<uint32_t> cellpack;   // nb: the same coordinates in one word, coordinate j in bits [j*depth, (j+1)*depth)
    DBuf<int> childstart;   // nb+1: compact id at depth+1 of each box's first child (set by the next level)
    DBuf<int> parent;       // nb: compact id at depth-1 of each box's parent (the root: 0)
    // near-field source operands of this level (built on first use by near_field): per point, the
    // split-f16 matrix operand of its coordinates relative to its own box centre, scaled by nearops_sc
    // Two tables, each built at most once and never replaced (a launch recorded into a graph keeps its address):
    // nearops_all holds every box, nearops only the source boxes of the level's one near list.
    mutable DBuf<unsigned char> nearops, nearops_all;
    mutable DBuf<float> nearey, nearey_all;   // factored form only: exp2(-|y'|^2) per point, beside the table of the same slot
    mutable float nearops_sc = 0.f;
    // grid key -> box id table of this level (built on first use by lookup_boxes)
    // box of every 32nd point (npoints/32 + 2 entries, built on first use by box_table): kernels that
    // take points in fixed-size pieces start from here instead of searching the offsets
    mutable DBuf<int> box32;
    mutable DBuf<uint32_t> hashtab;      // hashcap pairs (key, value), empty = 0xffffffff
    mutable uint32_t hashcap = 0;
    // work items of P2M and of the general L2P over every box of this level (chunk offsets per box,
    // built on first use): they depend on the tree only
    mutable DBuf<int> p2m_tiles, l2p_tiles;
    mutable int p2m_bound = -1, l2p_bound = -1;
};

struct Tree {
    Geo geo;
    long long n = 0;
    DBuf<float> pts;     // d*n, dimension-major, Morton-sorted
    DBuf<uint32_t> keys; // n keys, sorted by their bits [sorted_from, d*L)
    int sorted_from = 0;
    DBuf<int> perm;      // sorted position -> original row
    std::vector<TreeLevel> lev;   // lev[0] is the root
};

// work items of the near field over one list: offsets of the target tiles per x box (in the order
// `order`, if any), and the launch bound that goes with them
struct TileTable {
    DBuf<int> tileoff, order;
    int bound = 0;
};

struct PairList {
    long long n = 0;
    DBuf<int> pairs;     // (n,2) int32: (bx, by), sorted by (bx, by)
    DBuf<int> rowptr;    // nbx+1: range of each x box
    // far lists: pairs whose cell offset lies outside the 13 offsets per dimension that the M2L tables of a
    // level hold (m2l_table_omin .. +12).  Cannot happen (a far pair's parents were closer than 2 parent
    // edges); plan creation counts them and fails if there is one, so the M2L kernels never meet one.
    long long beyond_tables = 0;
    // far lists of one tree only: pairs whose y box is neither a child of one of the 3^d parents around
    // the parent of the x box nor a child of a parent two cells away along one axis (a parent pair
    // exactly on the far threshold, kept by rounding); -1 = not counted.  Expected to be 0.
    long long outliers = -1;
    // x boxes with a non-empty row, their points, and the work items they make when cut into pieces of
    // 128 and of 160 targets (near-field launch shapes); rows = -1: not counted
    long long rows = -1, row_points = 0, items128 = 0, items160 = 0;
    // Tables that depend on the plan only, built on first use and kept: near-field tile tables by
    // (targets per work item) * 2 + (longest lists first); for far lists the separable M2L tables of the
    // level and the order of the parents for the sibling-group kernel.
    mutable std::map<int, TileTable> near_tiles;
    mutable DBuf<float> m2l_tab;
    mutable DBuf<int> m2l_order;
};

struct ClassifyParams {
    int omin[kMaxD];     // m2l_table_omin per dimension (set by level_launch)
    int nr_interp;
    int small_limit;
    int var_comp;
    int do_init, en_pair, en_all;
    float crit, lcs, edge;
};

// Lowest cell offset (y cell - x cell) along one dimension in the separable M2L tables of a level.
// Centres of a far pair are less than 5 edges apart along every dimension (their parents were closer
// than 2 parent edges), so offset * edge + (origin_y - origin_x) lies in (-5 edge, 5 edge): at most 11
// integers from ceil(-5 - delta/edge) on; the tables hold 13 from here.
constexpr int kM2LOffsets = 13;
inline int m2l_table_omin(float origin_x, float origin_y, float edge)
{
    const double delta = (double)origin_y - (double)origin_x;
    return (int)std::floor(-5.0 - delta / (double)edge) - 1;
}

struct PlanLevel {
    PairList far, small_, keep;
    // the same lists seen from the Y boxes, (by, bx) sorted by (by, bx) with row pointers over the Y boxes:
    // what the transposed product K(X,Y)^T u walks (built on its first use; plans of two trees only)
    PairList farT, smallT, keepT;
    bool haveT = false;
    int num_nodes = 0;
};

// per-stage timing with HIP events (f3m_plan.hip); no-ops unless enabled through the C ABI
enum Stage { kPlan = 0, kNear, kP2M, kM2L, kL2P, kPerm, kNumStages };
void timer_begin(int stage, hipStream_t s);
void timer_end(hipStream_t s);

// --- f3m_geom.hip ---
// Root geometry without a host wait before the sort: partial minima and maxima per tree (bounding_box_launch), their
// reduction to the minima of X, of Y and the root edge in device memory (root_geometry_launch: 2 kMaxD + 1 floats),
// Morton keys and their sort from those values (sort_tree_launch); the host fetches the same values meanwhile and
// sets up the root level with them (root_level_launch).  The coordinates are gathered by gather_tree_points once
// the order is final (divisions may still refine the order inside the boxes).
unsigned bounding_box_launch(const float *X, long long n, int d, DBuf<float> &part, hipStream_t s);
void root_geometry_launch(const float *partx, unsigned gridx, const float *party, unsigned gridy, int d, float *out, hipStream_t s);
void sort_tree_launch(Tree &t, const float *X, long long n, int d, int L, const float *origin, const float *edge0p, hipStream_t s);
void root_level_launch(Tree &t, const Geo &geo, hipStream_t s);
void gather_tree_points(Tree &t, const float *X, hipStream_t s, bool background = false);
// The division to a new depth is queued by level_launch (below) and appended to the tree with its box count and
// largest count still unknown; divide_finish completes it with the two numbers the kernels left in dstats once the
// host has fetched them; divide_discard drops a level that turned out not to be needed.
// Levels whose boxes the sorted key bits resolve; the count of the fullest cell at that depth (added to *dout by
// atomicMax, *dout zero before): if it exceeds the division threshold the tree will go deeper than the sorted bits
// reach, and sort_more_bits (eight more key bits; the levels built so far stay valid) is due sooner or later.
int sorted_levels(const Tree &t);
void max_run_launch(const Tree &t, int *dout, hipStream_t s);
void sort_more_bits(Tree &t, hipStream_t s);
// whether the next division will first sort more key bits (and thereby replace the key and order arrays)
bool divide_will_sort(const Tree &t);
void divide_finish(Tree &t, const int *hstats);
void divide_discard(Tree &t);
// One step of the level loop, queued as one group of launches: the counting pass of the lists of depth k from the keep
// list of depth k-1 (keep_prev; null or empty: no lists) and, if `divide`, the division of both trees to depth k+1
// (dstats_x, dstats_y: two zeroed words each, to which the kernels add the new level's boxes and largest count).  The
// two are independent, so their kernels share launches: one for the counting pass and the candidates' point ranges,
// one set for all the scans.  After it the sizes of the small, far and keep list are the last entries
// pos[(c+1)*stride - 1] of the three scans; the number of far pairs outside the sibling-group tables has been added to
// dtot[3] and of those outside the M2L tables of the level to dtot[6], which the caller keeps zero between levels; the
// row statistics of the small and the keep list -- x boxes with pairs, their points, their pieces of 128 and of 160
// points -- have been added to the eight zeroed words drow (nullable).  lists_finish allocates from the fetched totals
// htot[0..3], takes the fetched row statistics hrow[0..7] and writes.
struct ListsPending {
    DBuf<long long> pos;
    long long stride = 0;
    unsigned grid = 0;
    bool active = false;
    bool written = false;    // the writing pass has been queued (lists_write_early)
};
void level_launch(const PairList *keep_prev, Tree &tx, Tree &ty, int k, ClassifyParams &cp, ListsPending &pend,
                  long long *dtot, long long *drow, bool divide, int *dstats_x, int *dstats_y, hipStream_t s);
// queues the writing pass before the sizes are known, into lists allocated for an upper bound of the pairs, if that
// bound is modest (returns whether it did; lists_finish then only records the sizes)
bool lists_write_early(ListsPending &pend, const PairList &keep_prev, const Tree &tx, const Tree &ty, int k,
                       const ClassifyParams &cp, PlanLevel &out, hipStream_t s);
void lists_finish(ListsPending &pend, const long long *htot, const PairList &keep_prev, const Tree &tx, const Tree &ty, int k,
                  const ClassifyParams &cp, PlanLevel &out, const long long *hrow /* 8 words or null */, hipStream_t s);
// moves lists that fill a small part of the block they were written into (lists_write_early) into blocks of their size
void shrink_lists(PlanLevel &L, hipStream_t s);
// out = `in` with the two boxes of every pair swapped, sorted by (by, bx) (a stable sort by `by` of a list that is
// sorted by bx), its row pointers over the nby boxes of the Y level, and its row statistics for the near field
void transpose_list(const PairList &in, const TreeLevel &ly, PairList &out, hipStream_t s);
void exclusive_scan_i32(const int *in, long long n, int *out /* n+1 */, hipStream_t s);
void exclusive_scan_i64(const long long *in, long long n, long long *out /* n+1 */, hipStream_t s);
void exclusive_scan_i64_batched(const long long *in, long long n, long long pitch, int nch, long long *out, hipStream_t s);
void build_rowptr(PairList &l, int nbx, hipStream_t s);
// slot of a key in a table of `capacity` slots (host and device use the same function)
uint32_t hash_slot_host(uint32_t key, uint32_t capacity);
// ids[i] = box of depth lev.depth whose integer cell is cells[i*d .. i*d+d), or -1 if that cell is empty
void lookup_boxes(const Tree &t, const TreeLevel &lev, const int *cells, long long n, int *ids, hipStream_t s);

// --- f3m_field.hip ---
struct NodeSet {
    int d = 0, P = 0, S1 = 0;
    int n[kMaxD] = {0};
    int start[kMaxD] = {0};
    DBuf<float> dt, dw;             // concatenated 1-D nodes and barycentric weights
    DBuf<float> noff;               // (P,d) node offsets of a box of the current level
};
void make_nodes(NodeSet &ns, int d, int max_nodes, hipStream_t s);
void set_node_offsets(NodeSet &ns, float edge, hipStream_t s);

// background: the move runs beside latency-bound kernels of another stream and takes one workgroup per compute unit
void gather_points(const float *X, const int *perm, long long n, int d, float *pts, hipStream_t s, bool background = false);
void gather_column(const float *b, const int *perm, long long n, int c, int col, float *bs, hipStream_t s);
void scatter_column(const float *outs, const int *perm, long long n, int c, int col, float *out, hipStream_t s);
// ncol (1..4) neighbouring columns at once, one access per row; the scatter adds outs2 (same layout) if it is given,
// and to its one column the fixed-point sums of a symmetric near field (see SymSums) if those are given
struct SymSums;
void gather_columns(const float *b, const int *perm, long long n, int c, int col, int ncol, float *bs, long long bstride,
                    hipStream_t s, bool background = false);
void scatter_columns(const float *outs, const float *outs2, long long ostride, const int *perm, long long n, int c, int col,
                     int ncol, float *out, hipStream_t s, const SymSums *symsums = nullptr);

// Results added straight into the caller's array instead of the sorted one: out[perm[i] * c + col + q] += value by a
// hardware atomic addition.  The array is cleared before, and at most two values are added to an element (the near
// field's sum and the far field's), so the result does not depend on which comes first: 0 + a + b = 0 + b + a.
struct DirectOut {
    const int *perm = nullptr;
    float *out = nullptr;         // null: not used, results go to the sorted array
    int c = 0, col = 0, ncol = 0; // row length of out, first column and number of columns of this pass
};
// whether near_field would take this list in one launch of the matrix-pipe kernel with one wavefront per work item
// (the condition for DirectOut: every target is then written by exactly one wavefront)
bool near_single_pass(int d, const Tree &tx, const TreeLevel &lx, const PairList &list, float lcs, int nc);
// The symmetric near field (one tree: K is symmetric and the lists name (A,B) exactly when they name (B,A)) evaluates the
// tiles of a pair of boxes once and adds them in both directions.  The sums of the second direction reach a point from
// many wavefronts in no fixed order, so they are added as 64-bit fixed-point numbers (integer addition is associative: the
// result does not depend on the order) with one scale for the whole product: 2^61 over a power of two above
// (number of sources) x (largest |weight|), which no sum can exceed.  One unit is below 1e-18 of that bound, far under
// the rounding of the fp32 sums it joins.  absmax: bit pattern of the largest |weight| (written by sym_absmax; not finite:
// the kernel adds floats atomically instead, the results are not finite anyway).
struct SymSums {
    long long *fix = nullptr;          // one per sorted point, cleared by the caller; null: not used
    const unsigned *absmax = nullptr;
    long long nsrc = 0;
    // factored form only (near_field fills them in): the sorted weights themselves (the kernel's weight argument then holds
    // them times exp2(-|y'|^2)) and that factor per point
    const float *braw = nullptr, *ey = nullptr;
    // set by the caller where the far field that runs beside the near field is made of small one-wavefront workgroups
    // (node grids up to 4 x 4 x 4): the near field then takes workgroups of one wavefront itself (see near_sym_waves)
    bool small_far = false;
};
// scale of the fixed-point sums as a power of two (0: weights not finite)
__host__ __device__ inline float sym_scale(unsigned absmax_bits, long long nsrc)
{
    if (absmax_bits >= 0x7f800000u) return 0.f;
    int lg = 0;
    while ((1ll << lg) < nsrc) lg++;
    const int e = (int)(absmax_bits >> 23) - 127 + 1;          // |w| < 2^e
    int se = 61 - lg - e;
    if (se > 127) se = 127;                                    // (tiny weights: coarser than it could be, still exact enough)
    if (se < -126) se = -126;
    return __builtin_bit_cast(float, (unsigned)(se + 127) << 23);
}
// whether near_field would take this list in the symmetric form, given a place for the sums of the second direction
bool near_symmetric(int d, const Tree &tx, const TreeLevel &lx, const Tree &ty, const PairList &list, float lcs, int nc);
// absmax[0] = bit pattern of the largest |bs[i]|, i < n
void sym_absmax(const float *bs, long long n, unsigned *absmax, hipStream_t s);
// builds the table "box of every 32nd point" of a level now, on stream s, if it does not exist yet (kernels of
// the near field and of L2P start from it; when those run on different streams the table must exist before)
void ensure_box_table(const TreeLevel &lev, long long npoints, hipStream_t s);
// the near field's source operands of every box of a level, ahead of its use (kept with the level)
void prepare_near_operands(int d, const Tree &ty, const TreeLevel &ly, float lcs, hipStream_t s);
// nc = 1 or 4 right-hand sides at a time: columns of bs are bstride floats apart, those of outs ostride;
// only_list: no other near list of this level will be applied with this plan;
// prepare_only: build the tables of the list that are kept with the plan (tile table, source operands), launch nothing else
void near_field(int d, const Tree &tx, const TreeLevel &lx, const Tree &ty, const TreeLevel &ly, const PairList &list,
                const float *bs, float *outs, float lcs, hipStream_t s, int nc = 1, long long bstride = 0,
                long long ostride = 0, bool only_list = false, bool prepare_only = false, const DirectOut *direct = nullptr,
                const SymSums *symsums = nullptr);
void far_field(int d, const Tree &tx, const TreeLevel &lx, const Tree &ty, const TreeLevel &ly, const PairList &far,
               NodeSet &ns, const float *bs, float *outs, float lcs, int m2l_mode,
               float *mom_out, float *loc_out, hipStream_t s);

// the three stages of one level on their own; flag (one int per box, or nullptr = every box) selects
// the boxes whose points are interpolated
void mark_far_boxes(const PairList &far, int nbx, int nby, int *fx, int *fy, hipStream_t s);
void p2m_level(int d, const Tree &ty, const TreeLevel &ly, const int *flag, NodeSet &ns, const float *bs, float *mom,
               hipStream_t s);
// beside_near: the launch will run beside the near field of another stream (small workgroups then)
void m2l_level(int d, const Tree &tx, const TreeLevel &lx, const Tree &ty, const TreeLevel &ly, const PairList &far,
               NodeSet &ns, float lcs, int m2l_mode, const float *mom, float *loc /* overwritten */, hipStream_t s, bool beside_near = false);
// direct (nullable, one column: direct->col is the column): results go to the caller's array
void l2p_level(int d, const Tree &tx, const TreeLevel &lx, const int *flag, NodeSet &ns, const float *loc, float *outs,
               hipStream_t s, const DirectOut *direct = nullptr);
// expansions moved between a level and the next deeper one: moments up (down = false, dst = parent
// moments, overwritten) or local expansions down (down = true, dst = child expansions, added to)
bool nodes_nest(const NodeSet &coarse, const NodeSet &fine);
void make_shift_tables(const NodeSet &nsp, const NodeSet &nsc, DBuf<float> &tab, hipStream_t s);
void shift_level(bool down, const TreeLevel &parent, const TreeLevel &child, const NodeSet &nsp, const NodeSet &nsc,
                 const float *tab, const float *src, float *dst, hipStream_t s);

void exact_f32(int d, const float *X, long long N, const float *Y, long long M, const float *b, int c, float ls,
               bool grad, float *out, hipStream_t s);
void exact_f64(int d, const double *X, long long N, const double *Y, long long M, const double *b, int c, double ls,
               double *out, hipStream_t s);

}  // namespace f3m
