/*
 * C ABI of the MI355X (gfx950) F3M kernel-matrix-vector-product engine.
 *
 * Every pointer named X, Y, b, out is DEVICE memory (fp32 row-major unless stated), borrowed for
 * the duration of the call and never modified except `out`.  `stream` is a hipStream_t passed as
 * void* (NULL = the default stream).  Every function returns 0 on success or a positive error
 * code; f3m_last_error() then returns a message for the calling thread.  Calls are synchronous:
 * the stream is idle when they return.  `out` must not overlap X, Y or b (it may be written before the
 * inputs have been read for the last time).  One call at a time per device (the engine keeps a cache of
 * device buffers, per device, that concurrent calls would share).  The device of the pointers must be
 * the calling thread's current device (hipSetDevice), for plans during create, apply and destroy.
 *
 * The citations name the interface of the upstream reference (repository MrHuff/F3M) that each
 * entry point replaces.
 */
#ifndef F3M_H
#define F3M_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct f3m_plan f3m_plan;

/* Problem parameters = the scalar arguments of FFM_XY<float,nd>
 * (F3M_src/n_tree.cu:1056-1059; Python defaults experiments/FFM_classes.py:9-19). */
typedef struct f3m_params {
    float ls;                   /* lengthscale: K = exp(-r^2 / (2 ls^2)) */
    float min_points;           /* divide while the fullest box holds more points than this */
    int nr_of_interpolation;    /* interpolation nodes per box (upper bound of the tensor grid) */
    int var_compression;        /* 0/1: extra far-field shortcuts of 1_d_conv.cu:955-1029 */
    float eff_var_limit;        /* threshold used by var_compression */
    int small_field_points;     /* box pairs with fewer points than 2*this are summed exactly */
} f3m_params;

/* out(N,c) = K(X,Y) b.  Replaces FFM_XY_FLOAT_{1..10} (F3M_src/pybinder_setup.cu:17-36, C++ body
 * F3M_src/n_tree.cu:1056-1125).  d = columns of X and Y (1..10).  Y == NULL or Y == X selects the
 * symmetric case (the reference tests X.data_ptr()==Y.data_ptr(), n_tree.cu:1072); M is then ignored.
 * b is (M,c).  If no division happens (N <= min_points) the exact product is returned, where the
 * reference reads undefined tensors. */
int f3m_kmvm_f32(int d, const float *X, int64_t N, const float *Y, int64_t M, const float *b, int c,
                 const f3m_params *params, float *out, void *stream);

/* Exact dense products.  Replace rbf_float_{1..10}, rbf_float_{1..10}_grad and rbf_double_{1..10}
 * (F3M_src/pybinder_setup.cu:40-72, bodies F3M_src/n_tree.cu:185-241).  The _grad form returns
 * sum_j exp(-r^2/(2 ls^2)) r^2 b_j / ls^3. */
int f3m_exact_f32(int d, const float *X, int64_t N, const float *Y, int64_t M, const float *b, int c,
                  float ls, float *out, void *stream);
int f3m_exact_grad_f32(int d, const float *X, int64_t N, const float *Y, int64_t M, const float *b, int c,
                       float ls, float *out, void *stream);
int f3m_exact_f64(int d, const double *X, int64_t N, const double *Y, int64_t M, const double *b, int c,
                  double ls, double *out, void *stream);

/* Plan = box division + interaction lists of (X, Y, params), i.e. everything FFM_XY computes that
 * does not depend on b (F3M_src/n_tree.cu:105-179 divide, :903-969 get_field).  f3m_kmvm_f32 is
 * create + apply + destroy; callers that multiply many vectors by the same kernel matrix (the
 * conjugate-gradient drivers, conjugate_gradient/custom_conjugate_gradient_falkon.py:144-160) keep
 * the plan.  The plan holds its own sorted copy of the points: X and Y may be freed after create. */
int f3m_plan_create(int d, const float *X, int64_t N, const float *Y, int64_t M, const f3m_params *params,
                    void *stream, f3m_plan **plan);
int f3m_plan_apply(f3m_plan *plan, const float *b, int c, float *out, void *stream);
/* (Results are reproducible: the same call on the same inputs gives the same bits, whatever the order in which
 * the GPU runs the wavefronts.  Where sums of several wavefronts meet in one element -- the near field of a
 * product on one tree with one column evaluates each pair of boxes once for both directions -- they are added
 * as 64-bit fixed-point numbers scaled by the largest |b|, one unit below 1e-18 of (number of sources) x
 * max |b|.  F3M_NEAR_SYM=0 in the environment selects the one-directional near field for such products.) */
/* out(M,c) = K(X,Y)^T u, u (N,c), with the plan of (X, Y): the two trees swap roles and every interaction
 * list is read from its Y boxes (the lists of (Y, X) are the lists of (X, Y) with the boxes of each pair
 * swapped: the classification of F3M_src/1_d_conv.cu:927-952 depends on n_x + n_y and |c_y - c_x| only).
 * Replaces FFM.chunk_forward_transpose (experiments/FFM_classes.py:54-61: one FFM_XY call per chunk of the
 * rows of X, 48 of them per product at conjugate_gradient/custom_gaussian_kernel.py:85) and a second plan of
 * (Y, X), whose product it equals.  The transposed lists are built by the first call and kept. */
int f3m_plan_apply_transpose(f3m_plan *plan, const float *u, int c, float *out, void *stream);
int f3m_plan_destroy(f3m_plan *plan);
/* f3m_plan_apply without any device allocation.  No counterpart in the reference: it is for callers that
 * cannot allocate (a stream under HIP graph capture, a serving loop that must not touch the allocator, a
 * harness that forbids hipMalloc).  Same arguments and result as f3m_plan_apply.  Its temporaries live in
 * 128 MiB of static device memory that every GPU running the library holds until the process ends.  The
 * need does not grow with c beyond four columns: the sorted copies of b and of the result for one group of
 * columns (4 (N + M) bytes for c = 1, 16 (N + M) bytes for c >= 2), the partial sums of that group's near
 * field, and the moments and local expansions of one column's far field; every further group and column
 * reuses that memory (N = M = 1e7 with one column just fits).  One tree and one column: f3m_plan_apply
 * sums the near field in its symmetric form, which needs 8 N more bytes for fixed-point sums; this call
 * takes that form only where those bytes are at most a quarter of the scratch memory still free (N up
 * to about 3e6: the bits of f3m_plan_apply) and the plain form beyond (same sums in another order: equal
 * to about 1e-6 relative, not bit for bit).  A product that needs more is refused with
 * error 42 while its first column group is being queued, before anything is written to out.  The plan's own
 * tables are built by the first f3m_plan_apply with the same number of columns, which must therefore have
 * run once before (otherwise error 41).  All calls on a GPU share the one scratch array: calls that overlap
 * on one GPU race, also from different plans or threads.  The call waits for the stream like the others,
 * except while the stream is being captured.  A captured call holds the addresses of the plan's tables: its
 * graph may be replayed while the plan lives (a table of a plan is built once and never replaced; destroying the
 * plan frees them); an error raised during capture leaves the capture to the caller (the library then waits
 * for nothing).  The library itself asks for no memory here; the HIP runtime, however, reserves its own
 * per-queue scratch memory the first time a kernel that keeps registers there runs on a queue (some M2L and
 * near-field instances do: a few dozen bytes per lane), and f3m_plan_apply runs the far field on the library's
 * second stream.  A caller that must not see the device's free memory change runs one
 * f3m_plan_apply_noalloc on its stream beforehand. */
int f3m_plan_apply_noalloc(f3m_plan *plan, const float *b, int c, float *out, void *stream);

/* Introspection for parity tests (no counterpart is exported by the reference; the data are its
 * n_tree_cuda members, F3M_src/n_tree.cu:51-78, and the three lists of separate_interactions,
 * :701-787).  Levels are numbered 1..depth. */
int f3m_plan_depth(const f3m_plan *plan);                 /* number of divisions performed */
int f3m_plan_symmetric(const f3m_plan *plan);
/* sizes[0..7] = boxes of X tree, boxes of Y tree, |far|, |small|, |keep|, nodes used, max count X, max count Y */
int f3m_plan_level_sizes(const f3m_plan *plan, int level, int64_t *sizes, float *edge);
/* rows[0..3] = x boxes with pairs in the small list, their points, their pieces of 128 and of 160 points;
 * rows[4..7] = the same for the keep list (what the near field sizes its launches with) */
int f3m_plan_list_rows(const f3m_plan *plan, int level, int64_t *rows);
enum f3m_level_array {
    F3M_CENTERS_X = 0,   /* float (nbx,d) */
    F3M_CENTERS_Y = 1,
    F3M_OFFSETS_X = 2,   /* int32 nbx+1: point ranges of the boxes in sorted order */
    F3M_OFFSETS_Y = 3,
    F3M_LIST_FAR = 4,    /* int32 (n,2) */
    F3M_LIST_SMALL = 5,
    F3M_LIST_KEEP = 6,
    F3M_PERM_X = 7,      /* int32 N: sorted position -> row of X (same at every level) */
    F3M_PERM_Y = 8
};
/* copies one array of a level to HOST memory `dst` (caller sizes it from f3m_plan_level_sizes) */
int f3m_plan_level_copy(const f3m_plan *plan, int level, int which, void *dst, void *stream);
/* far field of one level only: out(N,c) receives its contribution; mom (nby*P*c) and loc (nbx*P*c),
 * device pointers or NULL, receive the moments and local expansions, column-major over c */
int f3m_plan_far_level(f3m_plan *plan, int level, const float *b, int c, float *out, float *mom, float *loc,
                       void *stream);
/* near field of one list of one level: which = F3M_LIST_SMALL or F3M_LIST_KEEP */
int f3m_plan_near_level(f3m_plan *plan, int level, int which, const float *b, int c, float *out, void *stream);
/* work model of the plan: w[0] = point pairs summed exactly, w[1] = far box pairs, w[2] = points
 * interpolated (P2M + L2P passes), w[3] = sum over levels of far pairs * P^2, w[4] = point pairs
 * covered by far box pairs (w[0] + w[4] = N*M: every point pair is handled exactly once) */
int f3m_plan_work(const f3m_plan *plan, double *w);

/* Box lookup by grid cell: ids[i] = compact id, at depth `level`, of the box whose integer cell is
 * cells[i*d .. i*d+d) (device int32, 0 <= cell < 2^level per dimension), or -1 if no point lies in that
 * cell.  tree = 0 for the X tree, 1 for the Y tree.  Replaces the key -> index table of
 * F3M_src/linearprobing.cu:41-87 as box_division_assign_hash uses it (F3M_src/1_d_conv.cu:1127-1191):
 * same slot function (Murmur3 finaliser modulo capacity-1), same probing, same answer for an absent
 * key.  The table of a level lives in device memory and is built on the first lookup. */
int f3m_plan_lookup_boxes(f3m_plan *plan, int level, int tree, const int32_t *cells, int64_t n, int32_t *ids,
                          void *stream);
/* slot of `key` in a table of `capacity` slots (host function; hash_2 of F3M_src/linearprobing.cu:18-26) */
uint32_t f3m_hash_slot(uint32_t key, uint32_t capacity);

/* seconds spent by the last f3m_plan_apply / f3m_kmvm_f32 of this thread in each stage, measured
 * with HIP events on the call's stream when timing is enabled: t[0] plan, t[1] near, t[2] P2M,
 * t[3] M2L, t[4] L2P, t[5] permutations; n[] = kernel launches per stage */
int f3m_set_timing(int enabled);
int f3m_get_timing(double *t, int *n);

const char *f3m_last_error(void);
/* frees the cached device buffers */
int f3m_release_cache(void);
const char *f3m_version(void);

#ifdef __cplusplus
}
#endif
#endif
