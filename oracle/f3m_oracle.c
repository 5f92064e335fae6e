/*
 * CPU ORACLE -- TEST INFRASTRUCTURE ONLY.
 *
 * A scalar restatement, in IEEE fp32 with one rounding per operation (build with
 * -ffp-contract=off, no fast-math), of the F3M kernel-matrix-vector-product algorithm.
 * It is the checker for the HIP engine: only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load it.  Nothing in the product path calls it.
 *
 * Every function cites the reference file:line (under the upstream tree, F3M_src/) whose
 * behaviour it restates.  The reference has no tests or golden vectors; what pins each
 * function is listed in oracle/README.md and exercised by tests/test_oracle_*.py.
 *
 * Parity status of each function (pinned = checked against something other than itself):
 *   fo_nodes_1d, fo_node_counts, fo_node_grid ...... pinned (numpy chebpts1, scipy weights, closed forms)
 *   fo_basis ....................................... pinned (partition of unity, delta property,
 *                                                    polynomial reproduction, scipy barycentric)
 *   tree division (fo_plan levels) ................. pinned (brute-force membership, Morton-rank
 *                                                    invariant, nesting, counts)
 *   interaction lists .............................. pinned (brute force over all box pairs,
 *                                                    partition + coverage invariants)
 *   near field / exact ............................. pinned (dense fp64 product)
 *   M2L ............................................ pinned (dense exp(-lcs*cdist^2) of shifted nodes)
 *   end to end ..................................... pinned (reduces to the dense product when no
 *                                                    pair is far; rel-L2 vs fp64 exact; linearity)
 *   var_compression classification ................. pinned (independent numpy restatement of the
 *                                                    predicates, brute force over all box pairs)
 *   sums for selected target rows (rowsel) ......... pinned (bit-equal to the unrestricted sums on those rows)
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define FO_MAXD 10
#define FO_MAXLEVELS 32

typedef struct {
    int d, p;            /* dimension, 2^d */
    long n;              /* points */
    const float *data;   /* (n,d) row-major, borrowed */
    float origin[FO_MAXD];
    float edge0;         /* root edge */
    int depth;
    float edge;          /* edge at current depth */
    long nb;             /* non-empty boxes at current depth */
    float *centers;      /* (nb,d) */
    int *counts;         /* nb */
    int *offsets;        /* nb+1 */
    int *perm;           /* n: point indices grouped by box, ascending inside a box */
    int *nat2compact;    /* nb_nat: natural child index -> compact id or -1 */
    long nb_nat;
    long maxcount;
} fo_tree;

typedef struct {
    int depth;
    float edge;
    long nbx, nby;
    float *cx, *cy;          /* centres (nb,d) */
    int *cntx, *cnty;
    int *offx, *offy;
    int *permx, *permy;
    long nfar, nsmall, nkeep;
    int *far, *small_, *keep; /* (n,2) int32 */
    int num_nodes;            /* interpolation nodes used for the far field of this level */
} fo_level;

typedef struct {
    int d, symmetric;
    long N, M;
    const float *X, *Y;
    float lcs;                /* 1/(2 ls^2), fp32 */
    int nlevels;              /* number of divisions performed */
    fo_level lev[FO_MAXLEVELS];
    int nr_interp;
    int status;               /* 0 ok; >0 error code */
    char msg[256];
    double work_near_pairs;   /* sum n_x n_y over small lists and the final keep list */
    double work_far_pairs;    /* sum over levels of |far_k| */
    double work_interp_pts;   /* sum over levels with far pairs of participating X + Y points */
} fo_plan;

/* ------------------------------------------------------------------------------------------ */
/* Nodes (n_tree.cu:265-285): first-kind Chebyshev points and barycentric weights, pi as float */

void fo_nodes_1d(int n, float *t, float *w)
{
    /* n_tree.cu:267  float PI = atan(1.)*4.;  the products below follow torch fp32 tensor ops:
     * cos(((i*2.+1.)*PI)/(2*(n-1)+2)) evaluated on a float tensor (n_tree.cu:268-269) */
    float PI = (float)(atan(1.) * 4.);
    for (int i = 0; i < n; i++) {
        float a = (float)i;
        a = a * 2.0f;
        a = a + 1.0f;
        a = a * PI;
        a = a / (float)(2 * (n - 1) + 2);
        t[i] = cosf(a);
        /* n_tree.cu:281  pow(base,i)*sin(((2.*(float)i+1.)*PI)/(2.*(float)(n-1.0)+2.)) is evaluated
         * in double from float inputs and stored to float */
        double s = sin(((2. * (double)(float)i + 1.) * (double)PI) / (2. * (double)(float)(n - 1.0) + 2.));
        double sg = (i % 2 == 0) ? 1.0 : -1.0;
        w[i] = (float)(sg * s);
    }
}

/* n_tree.cu:328-346 (without the random permutation of dims at :347, which is the identity on
 * the value multiset; for perfect d-th powers every entry is equal so order is irrelevant) */
void fo_node_counts(int d, int max_nodes, int *per_dim)
{
    float ref_val = (float)pow((double)max_nodes, 1.0 / (double)(float)d);
    int hi = (int)ceilf(ref_val);
    int lo = (int)floorf(ref_val);
    int acc = 1;
    for (int i = 0; i < d; i++) {
        int fut = (int)((double)acc * pow((double)lo, (double)(d - (i + 1))) * (double)hi);
        if (fut <= max_nodes) { per_dim[i] = hi; acc *= hi; }
        else { per_dim[i] = lo; acc *= lo; }
    }
}

/* tensor grid, dim 0 fastest (1_d_conv.cu:871-883).  idx (P,d) holds positions in the
 * concatenated 1-D node array; coords (P,d) the node coordinates. Returns P. */
int fo_node_grid(int d, const int *per_dim, const float *nodes_cat, int *idx, float *coords)
{
    int P = 1;
    int cum[FO_MAXD];
    for (int j = 0; j < d; j++) { P *= per_dim[j]; cum[j] = P; }
    for (int i = 0; i < P; i++) {
        int acc = 0;
        for (int j = 0; j < d; j++) {
            int tmp = i % cum[j];
            int id = (j == 0) ? tmp : (int)floorf((float)tmp / (float)cum[j - 1]);
            if (j > 0) acc += per_dim[j - 1];
            if (idx) idx[i * d + j] = id + acc;
            if (coords) coords[i * d + j] = nodes_cat[id + acc];
        }
    }
    return P;
}

/* ------------------------------------------------------------------------------------------ */
/* Basis (1_d_conv.cu:418-448 preparation, :217-238 product).                                 */

typedef struct {
    float t[FO_MAXD];    /* local coordinate */
    float lx[FO_MAXD];   /* 1/sum_l w_l/(t - t_l), or 1 on an exact hit */
    int hit[FO_MAXD];
} fo_bprep;

static void fo_basis_prepare(int d, const float *x, const float *center, float factor,
                             const int *per_dim, const float *nodes_cat, const float *w_cat,
                             fo_bprep *bp)
{
    int lo = 0;
    for (int k = 0; k < d; k++) {
        float tk = factor * (x[k] - center[k]);
        float tmp = 0.f;
        int hit = 0;
        for (int l = lo; l < lo + per_dim[k]; l++) {
            if (tk == nodes_cat[l]) { hit = 1; tmp = 1.f; break; }
            tmp += w_cat[l] / (tk - nodes_cat[l]);
        }
        bp->t[k] = tk; bp->hit[k] = hit; bp->lx[k] = 1.f / tmp;
        lo += per_dim[k];
    }
}

static inline float fo_basis_apply(int d, const fo_bprep *bp, const int *comb,
                                   const float *nodes_cat, const float *w_cat, float b)
{
    for (int i = 0; i < d; i++) {
        if (bp->hit[i]) {
            if (bp->t[i] != nodes_cat[comb[i]]) { b = 0.f; break; }
        } else {
            b *= bp->lx[i] * w_cat[comb[i]] / (bp->t[i] - nodes_cat[comb[i]]);
        }
    }
    return b;
}

/* All P basis values of one point (weight 1): out[m] = L_m(x). */
void fo_basis(int d, int nr_interp, const float *x, const float *center, float edge, float *out)
{
    int per_dim[FO_MAXD];
    fo_node_counts(d, nr_interp, per_dim);
    int tot = 0;
    for (int j = 0; j < d; j++) tot += per_dim[j];
    float *nodes = (float *)malloc(sizeof(float) * tot), *w = (float *)malloc(sizeof(float) * tot);
    int lo = 0;
    for (int j = 0; j < d; j++) { fo_nodes_1d(per_dim[j], nodes + lo, w + lo); lo += per_dim[j]; }
    int P = 1;
    for (int j = 0; j < d; j++) P *= per_dim[j];
    int *idx = (int *)malloc(sizeof(int) * P * d);
    fo_node_grid(d, per_dim, nodes, idx, NULL);
    fo_bprep bp;
    float factor = 2 / edge;
    fo_basis_prepare(d, x, center, factor, per_dim, nodes, w, &bp);
    for (int m = 0; m < P; m++) out[m] = fo_basis_apply(d, &bp, idx + m * d, nodes, w, 1.0f);
    free(nodes); free(w); free(idx);
}

/* ------------------------------------------------------------------------------------------ */
/* Root geometry (n_tree.cu:25-46).                                                            */

static void fo_minmax(const float *X, long n, int d, float *mn, float *mx)
{
    for (int j = 0; j < d; j++) { mn[j] = X[j]; mx[j] = X[j]; }
    for (long i = 1; i < n; i++)
        for (int j = 0; j < d; j++) {
            float v = X[i * d + j];
            if (v < mn[j]) mn[j] = v;
            if (v > mx[j]) mx[j] = v;
        }
}

static float fo_maxrange(const float *mn, const float *mx, int d)
{
    float e = mx[0] - mn[0];
    for (int j = 1; j < d; j++) { float r = mx[j] - mn[j]; if (r > e) e = r; }
    return e;
}

/* exported for tests: root edge and origins */
void fo_root(int d, const float *X, long N, const float *Y, long M, float *edge0, float *xmin, float *ymin)
{
    float mn[FO_MAXD], mx[FO_MAXD];
    fo_minmax(X, N, d, mn, mx);
    float xe = fo_maxrange(mn, mx, d);
    memcpy(xmin, mn, sizeof(float) * d);
    if (Y == NULL || Y == X) {
        *edge0 = xe * 1.01f;                   /* n_tree.cu:44-45 */
        if (ymin) memcpy(ymin, mn, sizeof(float) * d);
    } else {
        float ymn[FO_MAXD], ymx[FO_MAXD];
        fo_minmax(Y, M, d, ymn, ymx);
        float ye = fo_maxrange(ymn, ymx, d);
        float e = xe > ye ? xe : ye;           /* n_tree.cu:32-35 */
        *edge0 = e * 1.01f;
        memcpy(ymin, ymn, sizeof(float) * d);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* Tree (n_tree.cu:79-179; kernels 1_d_conv.cu:887-899, 1127-1191, 1056-1077).                 */

static void fo_tree_init(fo_tree *t, int d, const float *data, long n, const float *origin, float edge0)
{
    memset(t, 0, sizeof(*t));
    t->d = d; t->p = 1 << d; t->n = n; t->data = data; t->edge0 = edge0; t->edge = edge0;
    memcpy(t->origin, origin, sizeof(float) * d);
    t->depth = 0; t->nb = 1;
    t->centers = (float *)malloc(sizeof(float) * d);
    float half = 0.5f * edge0;
    for (int j = 0; j < d; j++) t->centers[j] = origin[j] + half;      /* n_tree.cu:93 */
    t->counts = (int *)malloc(sizeof(int));
    t->counts[0] = (int)n;
    t->offsets = (int *)malloc(sizeof(int) * 2);
    t->offsets[0] = 0; t->offsets[1] = (int)n;
    t->perm = (int *)malloc(sizeof(int) * (n > 0 ? n : 1));
    for (long i = 0; i < n; i++) t->perm[i] = (int)i;                  /* n_tree.cu:86 */
    t->maxcount = n;                                                   /* n_tree.cu:87 */
    t->nat2compact = NULL; t->nb_nat = 1;
}

static void fo_tree_free(fo_tree *t)
{
    free(t->centers); free(t->counts); free(t->offsets); free(t->perm); free(t->nat2compact);
}

typedef struct { int64_t key; int nat; } fo_kv;
static int fo_kv_cmp(const void *a, const void *b)
{
    int64_t ka = ((const fo_kv *)a)->key, kb = ((const fo_kv *)b)->key;
    return (ka > kb) - (ka < kb);
}

/* grid key of a position at the given depth (1_d_conv.cu:1142-1144 and :1161-1164):
 * sum_j mult[j] * (int)floor( side * (x_j - origin_j) / edge0 ), mult[j] = side^(d-1-j). */
static int64_t fo_grid_key(const fo_tree *t, const float *x, float side, const int64_t *mult)
{
    int64_t key = 0;
    for (int j = 0; j < t->d; j++) {
        float a = x[j] - t->origin[j];
        float q = side * a;
        q = q / t->edge0;
        key += mult[j] * (int64_t)(int)floorf(q);
    }
    return key;
}

/* one division; returns 0 or an error code */
static int fo_tree_divide(fo_tree *t, char *msg)
{
    int d = t->d, p = t->p;
    long nbp = t->nb;
    long nat = nbp * p;
    /* candidate centres (n_tree.cu:98-104, sign table 1_d_conv.cu:895-897) */
    float *cand = (float *)malloc(sizeof(float) * nat * d);
    float q = 0.25f * t->edge;
    for (long b = 0; b < nbp; b++)
        for (int i = 0; i < p; i++)
            for (int j = 0; j < d; j++) {
                float s = ((i >> j) & 1) ? 1.f : -1.f;
                cand[(b * p + i) * d + j] = t->centers[b * d + j] + q * s;
            }
    t->edge = t->edge * 0.5f;                                          /* n_tree.cu:107 */
    t->depth += 1;
    float side = powf(2.f, (float)t->depth);                           /* n_tree.cu:109 */
    int64_t mult[FO_MAXD];
    for (int j = 0; j < d; j++) {                                      /* n_tree.cu:88,170 */
        int64_t m = 1;
        for (int r = 0; r < d - 1 - j; r++) m *= ((int64_t)1 << t->depth);
        mult[j] = m;
    }
    if ((double)t->depth * d >= 62.0) { snprintf(msg, 256, "grid key overflow at depth %d", t->depth); free(cand); return 3; }
    /* key -> natural index (the reference inserts into a hash table, 1_d_conv.cu:1150-1166) */
    fo_kv *kv = (fo_kv *)malloc(sizeof(fo_kv) * nat);
    for (long c = 0; c < nat; c++) { kv[c].key = fo_grid_key(t, cand + c * d, side, mult); kv[c].nat = (int)c; }
    qsort(kv, nat, sizeof(fo_kv), fo_kv_cmp);
    for (long c = 1; c < nat; c++)
        if (kv[c].key == kv[c - 1].key) { snprintf(msg, 256, "duplicate centre key at depth %d", t->depth); free(cand); free(kv); return 4; }
    /* histogram (1_d_conv.cu:1127-1148) */
    int *natcount = (int *)calloc(nat, sizeof(int));
    int *natof = (int *)malloc(sizeof(int) * (t->n > 0 ? t->n : 1));
    for (long i = 0; i < t->n; i++) {
        int64_t key = fo_grid_key(t, t->data + i * d, side, mult);
        long lo = 0, hi = nat - 1, f = -1;
        while (lo <= hi) {
            long mid = (lo + hi) / 2;
            if (kv[mid].key == key) { f = mid; break; }
            if (kv[mid].key < key) lo = mid + 1; else hi = mid - 1;
        }
        if (f < 0) { snprintf(msg, 256, "point %ld has no candidate box at depth %d", i, t->depth); free(cand); free(kv); free(natcount); free(natof); return 5; }
        natof[i] = kv[f].nat;
        natcount[kv[f].nat]++;
    }
    /* drop empty boxes, natural order kept (n_tree.cu:162-177) */
    long nb = 0;
    for (long c = 0; c < nat; c++) if (natcount[c]) nb++;
    free(t->nat2compact);
    t->nat2compact = (int *)malloc(sizeof(int) * nat);
    float *centers = (float *)malloc(sizeof(float) * (nb > 0 ? nb : 1) * d);
    int *counts = (int *)malloc(sizeof(int) * (nb > 0 ? nb : 1));
    int *offsets = (int *)malloc(sizeof(int) * (nb + 1));
    long k = 0, mx = 0;
    offsets[0] = 0;
    for (long c = 0; c < nat; c++) {
        if (natcount[c]) {
            t->nat2compact[c] = (int)k;
            memcpy(centers + k * d, cand + c * d, sizeof(float) * d);
            counts[k] = natcount[c];
            offsets[k + 1] = offsets[k] + natcount[c];
            if (natcount[c] > mx) mx = natcount[c];
            k++;
        } else t->nat2compact[c] = -1;
    }
    /* counting-sort scatter, canonical (ascending original index) order inside a box
     * (the reference's order is the atomic race order, 1_d_conv.cu:1190) */
    int *fill = (int *)calloc(nb > 0 ? nb : 1, sizeof(int));
    for (long i = 0; i < t->n; i++) {
        int cb = t->nat2compact[natof[i]];
        t->perm[offsets[cb] + fill[cb]++] = (int)i;
    }
    free(fill); free(natof); free(natcount); free(kv); free(cand);
    free(t->centers); free(t->counts); free(t->offsets);
    t->centers = centers; t->counts = counts; t->offsets = offsets;
    t->nb = nb; t->nb_nat = nat; t->maxcount = mx;
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* Interaction lists (n_tree.cu:594-641 expansion, 788-811 filter, 701-787 + 1_d_conv.cu:903-1029
 * classification).                                                                            */

typedef struct {
    int var_comp;
    int nr_interp;
    int small_limit;
    float eff_var_limit;
    float lcs;
} fo_cls_params;

/* 0 = small, 1 = far, 2 = keep */
static int fo_classify(int d, const float *cx, const float *cy, int nx, int ny, float edge,
                       const fo_cls_params *cp)
{
    int size = nx + ny;
    int do_init = 1, en_pair = 0, en_all = 0;
    float crit = 0.f;
    if (cp->var_comp) {
        /* n_tree.cu:728-743 ("ls" there is lcs, see n_tree.cu:1083) */
        float sq = edge * edge * cp->lcs;
        do_init = sq <= 5;
        en_pair = ((float)d * sq / 4) <= cp->eff_var_limit;
        en_all = ((float)d * sq / 4) <= (cp->eff_var_limit / 2);
        crit = sqrtf(cp->eff_var_limit * 2 / ((float)d * cp->lcs));
    }
    if (do_init && size < 2 * cp->nr_interp) return 0;                 /* 1_d_conv.cu:928-934 */
    float acc = 0.f;
    for (int k = 0; k < d; k++) {                                      /* 1_d_conv.cu:243-250,936-940 */
        float dk = cy[k] - cx[k];
        float s = dk * dk;
        acc += s;
    }
    float dist = sqrtf(acc);
    if (dist >= edge * 2) return do_init ? 1 : 3;                      /* 1_d_conv.cu:941-947: dropped if !do_init */
    if (cp->var_comp) {
        if (en_pair && (double)(dist * dist * cp->lcs) <= 1e-2) return 1;     /* 1_d_conv.cu:1006-1012 */
        if (en_all && dist <= crit) return 1;                          /* 1_d_conv.cu:1013-1019 */
    }
    if (size < 2 * cp->small_limit) return 0;                          /* 1_d_conv.cu:948-952 */
    return 2;
}

typedef struct { int *v; long n, cap; } fo_ivec;
static void fo_push2(fo_ivec *a, int x, int y)
{
    if (a->n + 2 > a->cap) { a->cap = a->cap ? a->cap * 2 : 1024; a->v = (int *)realloc(a->v, sizeof(int) * a->cap); }
    a->v[a->n++] = x; a->v[a->n++] = y;
}

static void fo_lists(const fo_tree *tx, const fo_tree *ty, const int *keep_prev, long nkeep_prev,
                     const fo_cls_params *cp, fo_ivec *far, fo_ivec *small_, fo_ivec *keep)
{
    int d = tx->d, p = tx->p;
    long a = 0;
    while (a < nkeep_prev) {
        long b = a;
        int x = keep_prev[2 * a];
        while (b < nkeep_prev && keep_prev[2 * b] == x) b++;
        /* order (x, cx, y, cy): n_tree.cu:604-637 with repeat_within / repeat_add */
        for (int cxi = 0; cxi < p; cxi++) {
            int bx = tx->nat2compact[(long)x * p + cxi];
            if (bx < 0) continue;
            for (long t = a; t < b; t++) {
                int y = keep_prev[2 * t + 1];
                for (int cyi = 0; cyi < p; cyi++) {
                    int by = ty->nat2compact[(long)y * p + cyi];
                    if (by < 0) continue;
                    int cls = fo_classify(d, tx->centers + (long)bx * d, ty->centers + (long)by * d,
                                          tx->counts[bx], ty->counts[by], tx->edge, cp);
                    if (cls == 0) fo_push2(small_, bx, by);
                    else if (cls == 1) fo_push2(far, bx, by);
                    else if (cls == 2) fo_push2(keep, bx, by);
                }
            }
        }
        a = b;
    }
}

/* ------------------------------------------------------------------------------------------ */
/* Plan = all tree levels and lists (n_tree.cu:1056-1125 loop structure).                     */

static void fo_snapshot(fo_level *L, const fo_tree *tx, const fo_tree *ty, int symmetric)
{
    int d = tx->d;
    L->depth = tx->depth; L->edge = tx->edge;
    L->nbx = tx->nb;
    L->cx = (float *)malloc(sizeof(float) * tx->nb * d); memcpy(L->cx, tx->centers, sizeof(float) * tx->nb * d);
    L->cntx = (int *)malloc(sizeof(int) * tx->nb); memcpy(L->cntx, tx->counts, sizeof(int) * tx->nb);
    L->offx = (int *)malloc(sizeof(int) * (tx->nb + 1)); memcpy(L->offx, tx->offsets, sizeof(int) * (tx->nb + 1));
    L->permx = (int *)malloc(sizeof(int) * tx->n); memcpy(L->permx, tx->perm, sizeof(int) * tx->n);
    if (symmetric) {
        L->nby = L->nbx; L->cy = L->cx; L->cnty = L->cntx; L->offy = L->offx; L->permy = L->permx;
    } else {
        L->nby = ty->nb;
        L->cy = (float *)malloc(sizeof(float) * ty->nb * d); memcpy(L->cy, ty->centers, sizeof(float) * ty->nb * d);
        L->cnty = (int *)malloc(sizeof(int) * ty->nb); memcpy(L->cnty, ty->counts, sizeof(int) * ty->nb);
        L->offy = (int *)malloc(sizeof(int) * (ty->nb + 1)); memcpy(L->offy, ty->offsets, sizeof(int) * (ty->nb + 1));
        L->permy = (int *)malloc(sizeof(int) * ty->n); memcpy(L->permy, ty->perm, sizeof(int) * ty->n);
    }
}

fo_plan *fo_plan_create(int d, const float *X, long N, const float *Y, long M, float ls,
                        float min_points, int nr_interp, int var_comp, float eff_var_limit,
                        int small_limit, int max_levels)
{
    fo_plan *P = (fo_plan *)calloc(1, sizeof(fo_plan));
    P->d = d; P->N = N; P->X = X;
    P->symmetric = (Y == NULL || Y == X);
    P->Y = P->symmetric ? X : Y; P->M = P->symmetric ? N : M;
    P->lcs = 1 / (2 * ls * ls);                                         /* n_tree.cu:1060 */
    P->nr_interp = nr_interp;
    if (d < 1 || d > FO_MAXD) { P->status = 1; snprintf(P->msg, 256, "d out of range"); return P; }
    /* depth cap: past floor(31/d) levels the reference's int32 grid keys overflow
     * (1_d_conv.cu:1141-1144) and past ~16 levels fp32 centres no longer resolve cells; the
     * reference's behaviour there is undefined.  Defined behaviour here: stop dividing and sum
     * the remaining keep pairs exactly. */
    int cap = 31 / d < 16 ? 31 / d : 16;
    if (max_levels <= 0 || max_levels > cap) max_levels = cap;
    float edge0, xmin[FO_MAXD], ymin[FO_MAXD];
    fo_root(d, X, N, P->symmetric ? NULL : Y, M, &edge0, xmin, ymin);
    fo_tree tx, ty;
    fo_tree_init(&tx, d, X, N, xmin, edge0);
    if (!P->symmetric) fo_tree_init(&ty, d, P->Y, P->M, ymin, edge0);
    fo_cls_params cp = { var_comp, nr_interp, small_limit, eff_var_limit, P->lcs };
    int *keep = (int *)malloc(sizeof(int) * 2);
    keep[0] = 0; keep[1] = 0;
    long nkeep = 1;
    /* loop guard n_tree.cu:1075 / :1099 */
    while (nkeep > 0 && (float)tx.maxcount > min_points &&
           (P->symmetric || (float)ty.maxcount > min_points) && P->nlevels < max_levels) {
        int rc = fo_tree_divide(&tx, P->msg);
        if (!rc && !P->symmetric) rc = fo_tree_divide(&ty, P->msg);
        if (rc) { P->status = rc; break; }
        fo_level *L = &P->lev[P->nlevels];
        fo_snapshot(L, &tx, P->symmetric ? &tx : &ty, P->symmetric);
        fo_ivec far = {0, 0, 0}, sm = {0, 0, 0}, kp = {0, 0, 0};
        fo_lists(&tx, P->symmetric ? &tx : &ty, keep, nkeep, &cp, &far, &sm, &kp);
        L->far = far.v; L->nfar = far.n / 2;
        L->small_ = sm.v; L->nsmall = sm.n / 2;
        L->keep = kp.v; L->nkeep = kp.n / 2;
        L->num_nodes = nr_interp;
        if (var_comp) {                                                 /* n_tree.cu:971-978,1022-1025 */
            float eff = tx.edge * tx.edge * P->lcs;
            if (eff < 0.01f) { int t3 = (int)pow(3, d); L->num_nodes = t3 < nr_interp ? t3 : nr_interp; }
        }
        free(keep);
        nkeep = L->nkeep;
        keep = (int *)malloc(sizeof(int) * 2 * (nkeep > 0 ? nkeep : 1));
        memcpy(keep, L->keep, sizeof(int) * 2 * nkeep);
        P->nlevels++;
        /* work model */
        for (long t = 0; t < L->nsmall; t++)
            P->work_near_pairs += (double)L->cntx[L->small_[2 * t]] * (double)L->cnty[L->small_[2 * t + 1]];
        P->work_far_pairs += (double)L->nfar;
        if (L->nfar > 0) {
            char *ux = (char *)calloc(L->nbx, 1), *uy = (char *)calloc(L->nby, 1);
            for (long t = 0; t < L->nfar; t++) { ux[L->far[2 * t]] = 1; uy[L->far[2 * t + 1]] = 1; }
            for (long b = 0; b < L->nbx; b++) if (ux[b]) P->work_interp_pts += L->cntx[b];
            for (long b = 0; b < L->nby; b++) if (uy[b]) P->work_interp_pts += L->cnty[b];
            free(ux); free(uy);
        }
    }
    if (P->nlevels > 0) {
        fo_level *L = &P->lev[P->nlevels - 1];
        for (long t = 0; t < L->nkeep; t++)
            P->work_near_pairs += (double)L->cntx[L->keep[2 * t]] * (double)L->cnty[L->keep[2 * t + 1]];
    } else {
        P->work_near_pairs = (double)N * (double)P->M;
    }
    free(keep);
    fo_tree_free(&tx);
    if (!P->symmetric) fo_tree_free(&ty);
    return P;
}

void fo_plan_destroy(fo_plan *P)
{
    if (!P) return;
    for (int k = 0; k < P->nlevels; k++) {
        fo_level *L = &P->lev[k];
        if (!P->symmetric) { free(L->cy); free(L->cnty); free(L->offy); free(L->permy); }
        free(L->cx); free(L->cntx); free(L->offx); free(L->permx);
        free(L->far); free(L->small_); free(L->keep);
    }
    free(P);
}

int fo_plan_status(const fo_plan *P) { return P->status; }
const char *fo_plan_message(const fo_plan *P) { return P->msg; }
int fo_plan_nlevels(const fo_plan *P) { return P->nlevels; }
int fo_plan_symmetric(const fo_plan *P) { return P->symmetric; }
float fo_plan_lcs(const fo_plan *P) { return P->lcs; }
void fo_plan_work(const fo_plan *P, double *w)
{
    w[0] = P->work_near_pairs; w[1] = P->work_far_pairs; w[2] = P->work_interp_pts;
}
/* sizes: nbx, nby, nfar, nsmall, nkeep, num_nodes */
void fo_plan_level_sizes(const fo_plan *P, int k, long *s, float *edge)
{
    const fo_level *L = &P->lev[k];
    s[0] = L->nbx; s[1] = L->nby; s[2] = L->nfar; s[3] = L->nsmall; s[4] = L->nkeep; s[5] = L->num_nodes;
    *edge = L->edge;
}
/* which: 0 cx,1 cy,2 cntx,3 cnty,4 offx,5 offy,6 permx,7 permy,8 far,9 small,10 keep */
const void *fo_plan_level_ptr(const fo_plan *P, int k, int which)
{
    const fo_level *L = &P->lev[k];
    switch (which) {
    case 0: return L->cx; case 1: return L->cy; case 2: return L->cntx; case 3: return L->cnty;
    case 4: return L->offx; case 5: return L->offy; case 6: return L->permx; case 7: return L->permy;
    case 8: return L->far; case 9: return L->small_; case 10: return L->keep;
    }
    return NULL;
}

/* ------------------------------------------------------------------------------------------ */
/* Numerics.                                                                                   */

/* kernel arithmetic 1_d_conv.cu:60-73 */
static inline float fo_rbf(int d, const float *x, const float *y, float lcs)
{
    float dist = 0.f;
    for (int k = 0; k < d; k++) { float t = x[k] - y[k]; float s = t * t; dist += s; }
    return expf(-dist * lcs);
}

/* exact block sums over a box-pair list sorted by bx (1_d_conv.cu:255-335): one accumulator per
 * target over the whole list of its box, then out += acc */
static void fo_near(const fo_plan *P, const fo_level *L, const int *list, long nlist,
                    const float *b, int c, float *out, const char *rowsel)
{
    int d = P->d;
    long ngroups = 0;
    long *gstart = (long *)malloc(sizeof(long) * (nlist + 1));
    for (long t = 0; t < nlist; t++) if (t == 0 || list[2 * t] != list[2 * (t - 1)]) gstart[ngroups++] = t;
    gstart[ngroups] = nlist;
#pragma omp parallel for schedule(dynamic, 8)
    for (long g = 0; g < ngroups; g++) {
        int bx = list[2 * gstart[g]];
        for (int ii = L->offx[bx]; ii < L->offx[bx + 1]; ii++) {
            int i = L->permx[ii];
            if (rowsel && !rowsel[i]) continue;     /* rows that the caller did not ask for stay untouched */
            const float *xi = P->X + (long)i * d;
            for (int col = 0; col < c; col++) {
                float acc = 0.f;
                for (long t = gstart[g]; t < gstart[g + 1]; t++) {
                    int by = list[2 * t + 1];
                    for (int jj = L->offy[by]; jj < L->offy[by + 1]; jj++) {
                        int j = L->permy[jj];
                        acc += fo_rbf(d, xi, P->Y + (long)j * d, P->lcs) * b[(long)j * c + col];
                    }
                }
                out[(long)i * c + col] += acc;
            }
        }
    }
    free(gstart);
}

/* far field of one level (n_tree.cu:489-593): P2M (1_d_conv.cu:451-552), M2L (:741-817),
 * L2P (:554-659).  Optional outputs mom/loc receive the moments of every Y box / local
 * expansions of every X box (zeros for boxes outside the far list).
 * rowsel (nullable, one flag per row of X): the same sums restricted to the flagged target rows --
 * M2L only for the X boxes that hold a flagged row, L2P only for flagged rows; everything else of
 * out and loc stays zero/untouched.  (Sized for clouds whose complete M2L, far pairs x P^2 kernel
 * evaluations, would take minutes on a CPU.) */
static void fo_far(const fo_plan *P, const fo_level *L, const float *b, int c, float *out,
                   float *mom_out, float *loc_out, const char *rowsel)
{
    int d = P->d;
    int per_dim[FO_MAXD];
    fo_node_counts(d, L->num_nodes, per_dim);                           /* n_tree.cu:821 */
    int tot = 0;
    for (int j = 0; j < d; j++) tot += per_dim[j];
    float *nodes = (float *)malloc(sizeof(float) * tot), *w = (float *)malloc(sizeof(float) * tot);
    int lo = 0;
    for (int j = 0; j < d; j++) { fo_nodes_1d(per_dim[j], nodes + lo, w + lo); lo += per_dim[j]; }
    int Pn = 1;
    for (int j = 0; j < d; j++) Pn *= per_dim[j];
    int *idx = (int *)malloc(sizeof(int) * Pn * d);
    float *grid = (float *)malloc(sizeof(float) * Pn * d);
    fo_node_grid(d, per_dim, nodes, idx, grid);
    /* node offsets scaled to the box: cheb*edge/2 + edge/2 (n_tree.cu:510) */
    float *noff = (float *)malloc(sizeof(float) * Pn * d);
    for (int i = 0; i < Pn * d; i++) { float v = grid[i] * L->edge; v = v / 2.f; noff[i] = v + L->edge / 2.f; }
    float factor = 2 / L->edge;                                         /* 1_d_conv.cu:473 */

    char *uy = (char *)calloc(L->nby, 1), *ux = (char *)calloc(L->nbx, 1);
    for (long t = 0; t < L->nfar; t++) { ux[L->far[2 * t]] = 1; uy[L->far[2 * t + 1]] = 1; }
    if (rowsel)
        for (long bx = 0; bx < L->nbx; bx++) {
            char any = 0;
            for (int ii = L->offx[bx]; ii < L->offx[bx + 1] && !any; ii++) any = rowsel[L->permx[ii]];
            if (!any) ux[bx] = 0;
        }
    float *mom = (float *)calloc((size_t)L->nby * Pn * c, sizeof(float));
    float *loc = (float *)calloc((size_t)L->nbx * Pn * c, sizeof(float));

    /* P2M */
#pragma omp parallel for schedule(dynamic, 8)
    for (long by = 0; by < L->nby; by++) {
        if (!uy[by]) continue;
        for (int jj = L->offy[by]; jj < L->offy[by + 1]; jj++) {
            int j = L->permy[jj];
            fo_bprep bp;
            fo_basis_prepare(d, P->Y + (long)j * d, L->cy + by * d, factor, per_dim, nodes, w, &bp);
            for (int col = 0; col < c; col++) {
                float bj = b[(long)j * c + col];
                for (int m = 0; m < Pn; m++)
                    mom[((size_t)by * Pn + m) * c + col] += fo_basis_apply(d, &bp, idx + m * d, nodes, w, bj);
            }
        }
    }
    /* M2L: rows of the far list grouped by bx */
    long ngroups = 0;
    long *gstart = (long *)malloc(sizeof(long) * (L->nfar + 1));
    for (long t = 0; t < L->nfar; t++) if (t == 0 || L->far[2 * t] != L->far[2 * (t - 1)]) gstart[ngroups++] = t;
    gstart[ngroups] = L->nfar;
#pragma omp parallel for schedule(dynamic, 4)
    for (long g = 0; g < ngroups; g++) {
        int bx = L->far[2 * gstart[g]];
        if (!ux[bx]) continue;
        float xi[FO_MAXD], ym[FO_MAXD];
        for (int i = 0; i < Pn; i++) {
            for (int k = 0; k < d; k++) xi[k] = noff[i * d + k] + L->cx[(long)bx * d + k];  /* 1_d_conv.cu:776 */
            for (int col = 0; col < c; col++) {
                float acc = 0.f;
                for (long t = gstart[g]; t < gstart[g + 1]; t++) {
                    int by = L->far[2 * t + 1];
                    for (int m = 0; m < Pn; m++) {
                        for (int k = 0; k < d; k++) ym[k] = noff[m * d + k] + L->cy[(long)by * d + k]; /* :794 */
                        acc += fo_rbf(d, xi, ym, P->lcs) * mom[((size_t)by * Pn + m) * c + col];
                    }
                }
                loc[((size_t)bx * Pn + i) * c + col] = acc;
            }
        }
    }
    free(gstart);
    /* L2P */
#pragma omp parallel for schedule(dynamic, 8)
    for (long bx = 0; bx < L->nbx; bx++) {
        if (!ux[bx]) continue;
        for (int ii = L->offx[bx]; ii < L->offx[bx + 1]; ii++) {
            int i = L->permx[ii];
            if (rowsel && !rowsel[i]) continue;
            fo_bprep bp;
            fo_basis_prepare(d, P->X + (long)i * d, L->cx + bx * d, factor, per_dim, nodes, w, &bp);
            for (int col = 0; col < c; col++) {
                float acc = 0.f;
                for (int m = 0; m < Pn; m++)
                    acc += fo_basis_apply(d, &bp, idx + m * d, nodes, w, loc[((size_t)bx * Pn + m) * c + col]);
                out[(long)i * c + col] += acc;
            }
        }
    }
    if (mom_out) memcpy(mom_out, mom, sizeof(float) * (size_t)L->nby * Pn * c);
    if (loc_out) memcpy(loc_out, loc, sizeof(float) * (size_t)L->nbx * Pn * c);
    free(mom); free(loc); free(ux); free(uy); free(noff); free(grid); free(idx); free(nodes); free(w);
}

/* exact dense product, sequential fp32 accumulation (1_d_conv.cu:171-214) */
void fo_exact_f32(int d, const float *X, long N, const float *Y, long M, const float *b, int c,
                  float ls, float *out)
{
    float lcs = 1 / (2 * ls * ls);                                      /* n_tree.cu:194 */
#pragma omp parallel for schedule(static)
    for (long i = 0; i < N; i++)
        for (int col = 0; col < c; col++) {
            float acc = 0.f;
            for (long j = 0; j < M; j++) acc += fo_rbf(d, X + i * d, Y + j * d, lcs) * b[j * c + col];
            out[i * c + col] = acc;
        }
}

/* d/d ls variant (1_d_conv.cu:76-80,126-169; n_tree.cu:222-239): sum exp(-r^2 lcs) r^2 b / ls^3 */
void fo_exact_grad_f32(int d, const float *X, long N, const float *Y, long M, const float *b, int c,
                       float ls, float *out)
{
    float lcs = 1 / (2 * ls * ls);
    float inv = 1 / (ls * ls * ls);
#pragma omp parallel for schedule(static)
    for (long i = 0; i < N; i++)
        for (int col = 0; col < c; col++) {
            float acc = 0.f;
            for (long j = 0; j < M; j++) {
                float dist = 0.f;
                for (int k = 0; k < d; k++) { float t = X[i * d + k] - Y[j * d + k]; float s = t * t; dist += s; }
                acc += expf(-dist * lcs) * dist * b[j * c + col];
            }
            out[i * c + col] = acc * inv;
        }
}

void fo_exact_f64(int d, const double *X, long N, const double *Y, long M, const double *b, int c,
                  double ls, double *out)
{
    double lcs = 1 / (2 * ls * ls);
#pragma omp parallel for schedule(static)
    for (long i = 0; i < N; i++)
        for (int col = 0; col < c; col++) {
            double acc = 0.;
            for (long j = 0; j < M; j++) {
                double dist = 0.;
                for (int k = 0; k < d; k++) { double t = X[i * d + k] - Y[j * d + k]; dist += t * t; }
                acc += exp(-dist * lcs) * b[j * c + col];
            }
            out[i * c + col] = acc;
        }
}

/* whole product from a plan (n_tree.cu:1075-1094 / 1099-1120) */
static int fo_apply_rows(const fo_plan *P, const float *b, int c, float *out, const char *rowsel)
{
    if (P->status) return P->status;
    memset(out, 0, sizeof(float) * (size_t)P->N * c);
    if (P->nlevels == 0) {
        /* the reference never divides when N <= min_points and then reads undefined tensors
         * (n_tree.cu:1075,1092-1093); the defined behaviour chosen here is the exact product */
        float lcs = P->lcs;
#pragma omp parallel for schedule(static)
        for (long i = 0; i < P->N; i++) {
            if (rowsel && !rowsel[i]) continue;
            for (int col = 0; col < c; col++) {
                float acc = 0.f;
                for (long j = 0; j < P->M; j++)
                    acc += fo_rbf(P->d, P->X + i * P->d, P->Y + j * P->d, lcs) * b[j * c + col];
                out[i * c + col] = acc;
            }
        }
        return 0;
    }
    for (int k = 0; k < P->nlevels; k++) {
        const fo_level *L = &P->lev[k];
        if (L->nsmall > 0) fo_near(P, L, L->small_, L->nsmall, b, c, out, rowsel);     /* n_tree.cu:1018-1020 */
        if (L->nfar > 0) fo_far(P, L, b, c, out, NULL, NULL, rowsel);                  /* n_tree.cu:1021-1051 */
    }
    const fo_level *L = &P->lev[P->nlevels - 1];
    if (L->nkeep > 0) fo_near(P, L, L->keep, L->nkeep, b, c, out, rowsel);             /* n_tree.cu:1092-1094 */
    return 0;
}
int fo_plan_apply(const fo_plan *P, const float *b, int c, float *out) { return fo_apply_rows(P, b, c, out, NULL); }
/* the same product for the target rows flagged in rowsel (N flags) only; the other rows of out are zero */
int fo_plan_apply_rows(const fo_plan *P, const float *b, int c, float *out, const char *rowsel)
{
    return fo_apply_rows(P, b, c, out, rowsel);
}

/* single stages, exported so the GPU stages can be checked one by one */
int fo_plan_far_level_rows(const fo_plan *P, int k, const float *b, int c, float *out_accum, float *mom, float *loc,
                           const char *rowsel)
{
    if (k < 0 || k >= P->nlevels) return 1;
    fo_far(P, &P->lev[k], b, c, out_accum, mom, loc, rowsel);
    return 0;
}
int fo_plan_far_level(const fo_plan *P, int k, const float *b, int c, float *out_accum, float *mom, float *loc)
{
    return fo_plan_far_level_rows(P, k, b, c, out_accum, mom, loc, NULL);
}
int fo_plan_near_level_rows(const fo_plan *P, int k, int which, const float *b, int c, float *out_accum, const char *rowsel)
{
    if (k < 0 || k >= P->nlevels) return 1;
    const fo_level *L = &P->lev[k];
    if (which == 0) fo_near(P, L, L->small_, L->nsmall, b, c, out_accum, rowsel);
    else fo_near(P, L, L->keep, L->nkeep, b, c, out_accum, rowsel);
    return 0;
}
int fo_plan_near_level(const fo_plan *P, int k, int which, const float *b, int c, float *out_accum)
{
    return fo_plan_near_level_rows(P, k, which, b, c, out_accum, NULL);
}

/* M2L block between two boxes: K (P x P) with K[i][m] = exp(-|(n_i+cx)-(n_m+cy)|^2 lcs) */
int fo_m2l_block(int d, int nr_interp, const float *cx, const float *cy, float edge, float lcs, float *K)
{
    int per_dim[FO_MAXD];
    fo_node_counts(d, nr_interp, per_dim);
    int tot = 0;
    for (int j = 0; j < d; j++) tot += per_dim[j];
    float *nodes = (float *)malloc(sizeof(float) * tot), *w = (float *)malloc(sizeof(float) * tot);
    int lo = 0;
    for (int j = 0; j < d; j++) { fo_nodes_1d(per_dim[j], nodes + lo, w + lo); lo += per_dim[j]; }
    int Pn = 1;
    for (int j = 0; j < d; j++) Pn *= per_dim[j];
    float *grid = (float *)malloc(sizeof(float) * Pn * d);
    fo_node_grid(d, per_dim, nodes, NULL, grid);
    float xi[FO_MAXD], ym[FO_MAXD];
    for (int i = 0; i < Pn; i++) {
        for (int k = 0; k < d; k++) { float v = grid[i * d + k] * edge; v = v / 2.f; v = v + edge / 2.f; xi[k] = v + cx[k]; }
        for (int m = 0; m < Pn; m++) {
            for (int k = 0; k < d; k++) { float v = grid[m * d + k] * edge; v = v / 2.f; v = v + edge / 2.f; ym[k] = v + cy[k]; }
            K[i * Pn + m] = fo_rbf(d, xi, ym, lcs);
        }
    }
    free(nodes); free(w); free(grid);
    return Pn;
}

/* ------------------------------------------------------------------------------------------------
 * Open-addressing key -> value table (F3M_src/linearprobing.cu:18-87).  Slot of a key: Murmur3's 32-bit
 * finaliser, reduced modulo capacity-1 (hash_2, :18-26); collisions probe (slot+1) % (capacity-1)
 * (:66,:84); an empty slot holds 0xffffffff in key and value (:47-49), which is also what a lookup of
 * an absent key returns (:80-83).  table = capacity pairs (key, value).
 * Pinned by: MurmurHash3_x86_32 of the empty string is fmix32(seed) -> 0x514E28B7 for seed 1 and
 * 0x81F16F39 for seed 0xffffffff (published test vectors); table semantics against a Python dict. */
uint32_t fo_hash32(uint32_t k)
{
    k ^= k >> 16;
    k *= 0x85ebca6bu;
    k ^= k >> 13;
    k *= 0xc2b2ae35u;
    k ^= k >> 16;
    return k;
}

uint32_t fo_hash_slot(uint32_t key, uint32_t capacity) { return fo_hash32(key) % (capacity - 1u); }

void fo_hash_clear(uint32_t *table, uint32_t capacity) { memset(table, 0xff, sizeof(uint32_t) * 2 * (size_t)capacity); }

void fo_hash_insert(uint32_t *table, uint32_t capacity, uint32_t key, uint32_t value)
{
    uint32_t slot = fo_hash_slot(key, capacity);
    for (;;) {
        uint32_t prev = table[2 * (size_t)slot];
        if (prev == 0xffffffffu || prev == key) {
            table[2 * (size_t)slot] = key;
            table[2 * (size_t)slot + 1] = value;
            return;
        }
        slot = (slot + 1u) % (capacity - 1u);
    }
}

uint32_t fo_hash_lookup(const uint32_t *table, uint32_t capacity, uint32_t key)
{
    uint32_t slot = fo_hash_slot(key, capacity);
    for (;;) {
        if (table[2 * (size_t)slot] == key) return table[2 * (size_t)slot + 1];
        if (table[2 * (size_t)slot] == 0xffffffffu) return 0xffffffffu;
        slot = (slot + 1u) % (capacity - 1u);
    }
}

/* grid key of an integer cell at depth k: sum_j g_j (2^k)^(d-1-j), int32 arithmetic
 * (F3M_src/1_d_conv.cu:1142-1144, stride update F3M_src/n_tree.cu:170) */
int32_t fo_cell_key(int d, int k, const int32_t *cell)
{
    int32_t key = 0;
    for (int j = 0; j < d; j++) {
        int32_t mult = 1;
        for (int l = 0; l < d - 1 - j; l++) mult *= (int32_t)1 << k;
        key += mult * cell[j];
    }
    return key;
}
