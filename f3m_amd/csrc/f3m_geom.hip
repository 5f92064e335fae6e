// Box division and interaction lists for gfx950.
//
// Replaces the reference's per-level hash + atomic histogram + scatter (F3M_src/n_tree.cu:105-179,
// F3M_src/1_d_conv.cu:1127-1191) by one Morton sort: every point gets the key of its finest cell
// once, a wavefront-ballot counting sort orders the points, and the boxes of every depth are the
// runs of equal key prefixes, found by binary search.  The compact box index of the reference
// equals the rank of the Morton prefix among non-empty boxes, so box ids, counts, centres and the
// interaction lists come out identical.
//
// This file is compiled with -ffp-contract=off: every fp32 operation below rounds exactly once,
// in the order the reference's tensor code performs it.
#include "f3m_engine.h"

namespace f3m {

// ------------------------------------------------------------------------------------------------
// exclusive scan (n inputs, n+1 outputs; out[n] is the total)

constexpr int kScanBlock = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanBlock * kScanItems;

// RISE: the scanned element i is 1 where in[i+1] > in[i] (in has n+1 entries), else 0
template <typename Tin, typename Tout, bool RISE = false>
__global__ void scan_tile_kernel(const Tin *__restrict__ in, long long n, Tout *__restrict__ out, Tout *__restrict__ tilesum)
{
    __shared__ Tout sh[kScanBlock];
    const int tid = threadIdx.x;
    const long long base = (long long)blockIdx.x * kScanTile + (long long)tid * kScanItems;
    Tout v[kScanItems];
    Tout sum = 0;
#pragma unroll
    for (int e = 0; e < kScanItems; e++) {
        long long i = base + e;
        if (RISE) v[e] = (i < n && in[i + 1] > in[i]) ? (Tout)1 : (Tout)0;
        else v[e] = (i < n) ? (Tout)in[i] : (Tout)0;   // element n (the extra output slot) reads as 0
        sum += v[e];
    }
    sh[tid] = sum;
    __syncthreads();
    for (int off = 1; off < kScanBlock; off <<= 1) {
        Tout t = (tid >= off) ? sh[tid - off] : (Tout)0;
        __syncthreads();
        sh[tid] += t;
        __syncthreads();
    }
    Tout run = sh[tid] - sum;   // exclusive prefix of this thread inside the tile
#pragma unroll
    for (int e = 0; e < kScanItems; e++) {
        long long i = base + e;
        if (i <= n) out[i] = run;
        run += v[e];
    }
    if (tid == kScanBlock - 1) tilesum[blockIdx.x] = sh[tid];
}

template <typename Tout>
__global__ void scan_add_kernel(Tout *__restrict__ out, long long n1, const Tout *__restrict__ tileoff)
{
    long long i = (long long)blockIdx.x * kScanTile + threadIdx.x;
    Tout add = tileoff[blockIdx.x];
#pragma unroll
    for (int e = 0; e < kScanItems; e++, i += kScanBlock)
        if (i < n1) out[i] += add;
}

template <typename Tin, typename Tout, bool RISE = false>
static void exclusive_scan(const Tin *in, long long n, Tout *out, hipStream_t s)
{
    long long n1 = n + 1;
    unsigned ntiles = cdiv(n1, kScanTile);
    DBuf<Tout> tilesum(ntiles);
    F3M_LAUNCH((scan_tile_kernel<Tin, Tout, RISE>), ntiles, kScanBlock, 0, s, in, n, out, tilesum.get());
    check_launch("scan_tile");
    if (ntiles > 1) {
        DBuf<Tout> tileoff((size_t)ntiles + 1);
        exclusive_scan<Tout, Tout>(tilesum.get(), ntiles, tileoff.get(), s);
        F3M_LAUNCH((scan_add_kernel<Tout>), ntiles, kScanBlock, 0, s, out, n1, tileoff.get());
        check_launch("scan_add");
    }
}

// Batched form: `nch` arrays of n elements each, `pitch` apart in `in` and in `out` (n+1 outputs per
// array), scanned independently with three launches in all (one, if an array fits one tile).
template <typename T>
__global__ void scan_tile_batched_kernel(const T *__restrict__ in, long long n, long long pitch, unsigned ntiles,
                                         T *__restrict__ out, T *__restrict__ tilesum)
{
    __shared__ T sh[kScanBlock];
    const int tid = threadIdx.x;
    const unsigned ch = blockIdx.x / ntiles, tile = blockIdx.x % ntiles;
    in += ch * pitch;
    out += ch * pitch;
    const long long base = (long long)tile * kScanTile + (long long)tid * kScanItems;
    T v[kScanItems];
    T sum = 0;
#pragma unroll
    for (int e = 0; e < kScanItems; e++) {
        long long i = base + e;
        v[e] = (i < n) ? in[i] : (T)0;
        sum += v[e];
    }
    sh[tid] = sum;
    __syncthreads();
    for (int off = 1; off < kScanBlock; off <<= 1) {
        T t = (tid >= off) ? sh[tid - off] : (T)0;
        __syncthreads();
        sh[tid] += t;
        __syncthreads();
    }
    T run = sh[tid] - sum;
#pragma unroll
    for (int e = 0; e < kScanItems; e++) {
        long long i = base + e;
        if (i <= n) out[i] = run;
        run += v[e];
    }
    if (tid == kScanBlock - 1) tilesum[blockIdx.x] = sh[tid];
}

// tile sums of one array (at most kScanTile of them) -> their exclusive prefixes, in place; one workgroup per array
template <typename T>
__global__ void scan_sums_batched_kernel(T *__restrict__ tilesum, unsigned ntiles)
{
    __shared__ T sh[kScanBlock];
    const int tid = threadIdx.x;
    T *ts = tilesum + (size_t)blockIdx.x * ntiles;
    T v[kScanItems];
    T sum = 0;
#pragma unroll
    for (int e = 0; e < kScanItems; e++) {
        unsigned i = (unsigned)tid * kScanItems + e;
        v[e] = (i < ntiles) ? ts[i] : (T)0;
        sum += v[e];
    }
    sh[tid] = sum;
    __syncthreads();
    for (int off = 1; off < kScanBlock; off <<= 1) {
        T t = (tid >= off) ? sh[tid - off] : (T)0;
        __syncthreads();
        sh[tid] += t;
        __syncthreads();
    }
    T run = sh[tid] - sum;
#pragma unroll
    for (int e = 0; e < kScanItems; e++) {
        unsigned i = (unsigned)tid * kScanItems + e;
        if (i < ntiles) ts[i] = run;
        run += v[e];
    }
}

template <typename T>
__global__ void scan_add_batched_kernel(T *__restrict__ out, long long n1, long long pitch, unsigned ntiles,
                                        const T *__restrict__ tileoff)
{
    const unsigned ch = blockIdx.x / ntiles, tile = blockIdx.x % ntiles;
    out += ch * pitch;
    long long i = (long long)tile * kScanTile + threadIdx.x;
    T add = tileoff[blockIdx.x];
#pragma unroll
    for (int e = 0; e < kScanItems; e++, i += kScanBlock)
        if (i < n1) out[i] += add;
}

void exclusive_scan_i64_batched(const long long *in, long long n, long long pitch, int nch, long long *out, hipStream_t s)
{
    const long long n1 = n + 1;
    const unsigned ntiles = cdiv(n1, kScanTile);
    if (ntiles > (unsigned)kScanTile) {              // tile sums of an array would not fit one workgroup
        for (int c = 0; c < nch; c++) exclusive_scan_i64(in + c * pitch, n, out + c * pitch, s);
        return;
    }
    DBuf<long long> tilesum((size_t)ntiles * nch);
    F3M_LAUNCH((scan_tile_batched_kernel<long long>), ntiles * nch, kScanBlock, 0, s, in, n, pitch, ntiles, out, tilesum.get());
    check_launch("scan_tile_batched");
    if (ntiles > 1) {
        F3M_LAUNCH((scan_sums_batched_kernel<long long>), nch, kScanBlock, 0, s, tilesum.get(), ntiles);
        check_launch("scan_sums_batched");
        F3M_LAUNCH((scan_add_batched_kernel<long long>), ntiles * nch, kScanBlock, 0, s, out, n1, pitch, ntiles, tilesum.get());
        check_launch("scan_add_batched");
    }
}

void exclusive_scan_i32(const int *in, long long n, int *out, hipStream_t s) { exclusive_scan<int, int>(in, n, out, s); }
// out[i] = number of j < i with pos[j+1] > pos[j] (pos: n+1 non-decreasing offsets)
static void exclusive_scan_nonempty(const int *pos, long long n, int *out, hipStream_t s) { exclusive_scan<int, int, true>(pos, n, out, s); }
void exclusive_scan_i64(const long long *in, long long n, long long *out, hipStream_t s)
{
    exclusive_scan<long long, long long>(in, n, out, s);
}

// Several independent scans in one set of launches (the level loop's: the three list counts of depth k, and per tree the
// "candidate box is not empty" flags of depth k+1).  A channel of kind 0 scans n 64-bit values into n+1 64-bit
// outputs; a channel of kind 1 scans the flags in[i+1] > in[i] of n+1 non-decreasing 32-bit entries into n+1 32-bit
// outputs.  One tile launch; where a channel has more than one tile, a launch that scans the tile sums (one workgroup
// per channel, so at most kScanTile tiles per channel) and one that adds them.
// Folded in: the row statistics of the small and the keep list (channels rs_ch[0], rs_ch[1] of kind 0, or -1): x boxes
// with pairs, their points, their pieces of 128 and of 160 points, added to rowstat[4c .. 4c+3] (zero before).
constexpr int kMaxScanCh = 5;
struct ScanChannel {
    const void *in;
    void *out;
    long long n;
    int kind;
    unsigned tile0, ntiles;
};
struct ScanJob {
    ScanChannel ch[kMaxScanCh];
    int nch = 0;
    unsigned blocks = 0;
    const int *offx = nullptr;
    unsigned long long *rowstat = nullptr;
    int rs_ch[2] = {-1, -1};
    void add(const void *in, void *out, long long n, int kind)
    {
        if (nch >= kMaxScanCh) throw Error(103, "too many scan channels");
        const unsigned nt = cdiv(n + 1, kScanTile);
        ch[nch++] = ScanChannel{in, out, n, kind, blocks, nt};
        blocks += nt;
    }
};

__global__ void __launch_bounds__(kScanBlock) multi_scan_tile_kernel(ScanJob job, long long *__restrict__ tilesum)
{
    __shared__ long long sh[kScanBlock];
    __shared__ unsigned long long rs[4];
    int c = 0;
    while (c + 1 < job.nch && blockIdx.x >= job.ch[c + 1].tile0) c++;
    const ScanChannel ch = job.ch[c];
    const int tid = threadIdx.x;
    const long long n = ch.n;
    const long long base = (long long)(blockIdx.x - ch.tile0) * kScanTile + (long long)tid * kScanItems;
    const int rsi = (job.rowstat != nullptr && c == job.rs_ch[0]) ? 0 : ((job.rowstat != nullptr && c == job.rs_ch[1]) ? 1 : -1);
    if (tid < 4) rs[tid] = 0;
    long long v[kScanItems];
    long long sum = 0;
    if (ch.kind == 0) {
        const long long *in = static_cast<const long long *>(ch.in);
#pragma unroll
        for (int e = 0; e < kScanItems; e++) { const long long i = base + e; v[e] = i < n ? in[i] : 0; sum += v[e]; }
    } else {
        const int *in = static_cast<const int *>(ch.in);
#pragma unroll
        for (int e = 0; e < kScanItems; e++) { const long long i = base + e; v[e] = (i < n && in[i + 1] > in[i]) ? 1 : 0; sum += v[e]; }
    }
    sh[tid] = sum;
    __syncthreads();
    for (int off = 1; off < kScanBlock; off <<= 1) {
        long long t = (tid >= off) ? sh[tid - off] : 0;
        __syncthreads();
        sh[tid] += t;
        __syncthreads();
    }
    long long run = sh[tid] - sum;
    if (ch.kind == 0) {
        long long *out = static_cast<long long *>(ch.out);
#pragma unroll
        for (int e = 0; e < kScanItems; e++) { const long long i = base + e; if (i <= n) out[i] = run; run += v[e]; }
    } else {
        int *out = static_cast<int *>(ch.out);
#pragma unroll
        for (int e = 0; e < kScanItems; e++) { const long long i = base + e; if (i <= n) out[i] = (int)run; run += v[e]; }
    }
    if (tid == kScanBlock - 1) tilesum[blockIdx.x] = sh[tid];
    if (rsi >= 0) {                                   // uniform over the workgroup
        unsigned long long r0 = 0, r1 = 0, r2 = 0, r3 = 0;
#pragma unroll
        for (int e = 0; e < kScanItems; e++) {
            const long long i = base + e;
            if (i < n && v[e] > 0) {
                const unsigned long long np = (unsigned long long)(job.offx[i + 1] - job.offx[i]);
                r0 += 1; r1 += np; r2 += (np + 127) / 128; r3 += (np + 159) / 160;
            }
        }
        if (r0) { atomicAdd(&rs[0], r0); atomicAdd(&rs[1], r1); atomicAdd(&rs[2], r2); atomicAdd(&rs[3], r3); }
        __syncthreads();
        if (tid < 4 && rs[tid]) atomicAdd(&job.rowstat[4 * rsi + tid], rs[tid]);
    }
}

// tile sums of every channel -> their exclusive prefixes, in place; one workgroup per channel
__global__ void __launch_bounds__(kScanBlock) multi_scan_sums_kernel(ScanJob job, long long *__restrict__ tilesum)
{
    __shared__ long long sh[kScanBlock];
    const ScanChannel ch = job.ch[blockIdx.x];
    const int tid = threadIdx.x;
    long long *ts = tilesum + ch.tile0;
    long long v[kScanItems];
    long long sum = 0;
#pragma unroll
    for (int e = 0; e < kScanItems; e++) {
        const unsigned i = (unsigned)tid * kScanItems + e;
        v[e] = i < ch.ntiles ? ts[i] : 0;
        sum += v[e];
    }
    sh[tid] = sum;
    __syncthreads();
    for (int off = 1; off < kScanBlock; off <<= 1) {
        long long t = (tid >= off) ? sh[tid - off] : 0;
        __syncthreads();
        sh[tid] += t;
        __syncthreads();
    }
    long long run = sh[tid] - sum;
#pragma unroll
    for (int e = 0; e < kScanItems; e++) {
        const unsigned i = (unsigned)tid * kScanItems + e;
        if (i < ch.ntiles) ts[i] = run;
        run += v[e];
    }
}

__global__ void __launch_bounds__(kScanBlock) multi_scan_add_kernel(ScanJob job, const long long *__restrict__ tilesum)
{
    int c = 0;
    while (c + 1 < job.nch && blockIdx.x >= job.ch[c + 1].tile0) c++;
    const ScanChannel ch = job.ch[c];
    if (ch.ntiles == 1) return;                       // nothing to add
    const long long add = tilesum[blockIdx.x];
    long long i = (long long)(blockIdx.x - ch.tile0) * kScanTile + threadIdx.x;
#pragma unroll
    for (int e = 0; e < kScanItems; e++, i += kScanBlock)
        if (i <= ch.n) {
            if (ch.kind == 0) static_cast<long long *>(ch.out)[i] += add;
            else static_cast<int *>(ch.out)[i] += (int)add;
        }
}

// queues the scans of a job; false (nothing queued) if a channel has more tiles than one workgroup can scan
static bool multi_scan(const ScanJob &job, hipStream_t s)
{
    if (job.nch == 0) return true;
    unsigned most = 0;
    for (int c = 0; c < job.nch; c++) most = std::max(most, job.ch[c].ntiles);
    if (most > (unsigned)kScanTile) return false;
    if (const char *e = getenv("F3M_LEVEL_SCANS"))      // F3M_LEVEL_SCANS=separate: the path of levels too large for this one (testing aid)
        if (!strcmp(e, "separate")) return false;
    DBuf<long long> tilesum((size_t)job.blocks);
    F3M_LAUNCH(multi_scan_tile_kernel, job.blocks, kScanBlock, 0, s, job, tilesum.get());
    check_launch("multi_scan_tile");
    if (most > 1) {
        F3M_LAUNCH(multi_scan_sums_kernel, job.nch, kScanBlock, 0, s, job, tilesum.get());
        check_launch("multi_scan_sums");
        F3M_LAUNCH(multi_scan_add_kernel, job.blocks, kScanBlock, 0, s, job, (const long long *)tilesum.get());
        check_launch("multi_scan_add");
    }
    return true;
}

// ------------------------------------------------------------------------------------------------
// bounding box (F3M_src/n_tree.cu:28-31,42-43: per-dimension min and max)

// signed integers ordered like the floats they come from (-0 below +0), and back
__device__ inline int float_order(float v)
{
    const int b = __builtin_bit_cast(int, v);
    return b >= 0 ? b : b ^ 0x7fffffff;
}
__device__ inline float float_unorder(int k) { return __builtin_bit_cast(float, k >= 0 ? k : k ^ 0x7fffffff); }

// X is read as one flat array, four floats per load.  The number of threads is a multiple of d, so the
// elements a thread meets always belong to the same four dimensions and it keeps four running pairs.
constexpr int kBBBlocksPerDim = 192;

// `prefix` (0..3) leading elements come before the first 16-byte boundary and are read one by one.
__global__ void __launch_bounds__(256) minmax_kernel(const float *__restrict__ X, long long total, int d, int prefix,
                                                     float *__restrict__ part)
{
    __shared__ int smin[kMaxD], smax[kMaxD];
    const long long T = (long long)gridDim.x * blockDim.x;            // multiple of d
    const long long g = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    float lo[4], hi[4];
#pragma unroll
    for (int c = 0; c < 4; c++) { lo[c] = INFINITY; hi[c] = -INFINITY; }
    const long long nvec = (total - prefix) / 4;
    const float4 *X4 = reinterpret_cast<const float4 *>(X + prefix);
    for (long long e = g; e < nvec; e += T) {
        const float4 v = X4[e];
        lo[0] = fminf(lo[0], v.x); hi[0] = fmaxf(hi[0], v.x);
        lo[1] = fminf(lo[1], v.y); hi[1] = fmaxf(hi[1], v.y);
        lo[2] = fminf(lo[2], v.z); hi[2] = fmaxf(hi[2], v.z);
        lo[3] = fminf(lo[3], v.w); hi[3] = fmaxf(hi[3], v.w);
    }
    // per-dimension minimum and maximum of the workgroup through integer atomics in LDS on an
    // order-preserving image of the floats (NaNs stay out, as with fminf/fmaxf)
    if ((int)threadIdx.x < kMaxD) { smin[threadIdx.x] = 0x7fffffff; smax[threadIdx.x] = (int)0x80000000; }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const int j = (int)((prefix + 4 * g + c) % d);
        if (lo[c] == lo[c]) atomicMin(&smin[j], float_order(lo[c]));
        if (hi[c] == hi[c]) atomicMax(&smax[j], float_order(hi[c]));
    }
    if (g == 0) {                                                      // the few elements before and after the full loads
        for (long long e = 0; e < prefix && e < total; e++)
            if (X[e] == X[e]) { atomicMin(&smin[e % d], float_order(X[e])); atomicMax(&smax[e % d], float_order(X[e])); }
        for (long long e = prefix + 4 * nvec; e < total; e++)
            if (X[e] == X[e]) { atomicMin(&smin[e % d], float_order(X[e])); atomicMax(&smax[e % d], float_order(X[e])); }
    }
    __syncthreads();
    if ((int)threadIdx.x < d) {
        part[((long long)blockIdx.x * 2 + 0) * kMaxD + threadIdx.x] = float_unorder(smin[threadIdx.x]);
        part[((long long)blockIdx.x * 2 + 1) * kMaxD + threadIdx.x] = float_unorder(smax[threadIdx.x]);
    }
}

// queues the partial minima and maxima of X (per workgroup and dimension) into `part`; returns their number
unsigned bounding_box_launch(const float *X, long long n, int d, DBuf<float> &part, hipStream_t s)
{
    const int prefix = (int)(((16 - reinterpret_cast<uintptr_t>(X) % 16) % 16) / 4);
    unsigned grid = (unsigned)d * kBBBlocksPerDim;                      // threads = 256 * grid: a multiple of d
    const unsigned need = cdiv(cdiv(n * d, 4), 256);
    if (need < grid) grid = (unsigned)d * std::max(1u, cdiv(need, d));
    part.reset((size_t)grid * 2 * kMaxD);
    F3M_LAUNCH(minmax_kernel, grid, 256, 0, s, X, n * d, d, std::min<long long>(prefix, n * d), part.get());
    check_launch("minmax");
    return grid;
}

// Root geometry on the device (F3M_src/n_tree.cu:25-46): per tree and dimension the minimum over the partial
// results, the edge = largest extent over both trees, times 1.01.  out: minima of X (kMaxD), minima of Y (kMaxD; of X
// again for one tree), edge0.  The Morton keys are computed from these values without the host having seen them.
__global__ void __launch_bounds__(2 * kMaxD * 32) root_geometry_kernel(const float *__restrict__ partx, unsigned gridx,
                                                                       const float *__restrict__ party, unsigned gridy, int d,
                                                                       float *__restrict__ out)
{
    // 32 lanes per (tree, dimension): strided over the partial results, then combined inside the half wavefront
    // (minimum and maximum do not depend on the order)
    __shared__ float smn[2][kMaxD], smx[2][kMaxD];
    const int combo = threadIdx.x / 32, sub = threadIdx.x % 32;
    const int tree = combo / kMaxD, j = combo % kMaxD;
    const float *part = (tree && party) ? party : partx;
    const unsigned grid = (tree && party) ? gridy : gridx;
    float mn = part[j < d ? j : 0], mx = part[kMaxD + (j < d ? j : 0)];          // the first block's: every lane starts there
    if (j < d)
        for (unsigned b = sub; b < grid; b += 32) {
            mn = fminf(mn, part[((size_t)b * 2) * kMaxD + j]);
            mx = fmaxf(mx, part[((size_t)b * 2 + 1) * kMaxD + j]);
        }
#pragma unroll
    for (int m = 16; m >= 1; m >>= 1) {
        mn = fminf(mn, wave_shfl_xor_f(mn, m));
        mx = fmaxf(mx, wave_shfl_xor_f(mx, m));
    }
    if (sub == 0 && j < d) {
        smn[tree][j] = mn;
        smx[tree][j] = mx;
        out[tree * kMaxD + j] = mn;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float e = smx[0][0] - smn[0][0];
        for (int k = 1; k < d; k++) { const float r = smx[0][k] - smn[0][k]; if (r > e) e = r; }
        if (party) {
            float ye = smx[1][0] - smn[1][0];
            for (int k = 1; k < d; k++) { const float r = smx[1][k] - smn[1][k]; if (r > ye) ye = r; }
            if (ye > e) e = ye;
        }
        out[2 * kMaxD] = e * 1.01f;
    }
}

void root_geometry_launch(const float *partx, unsigned gridx, const float *party, unsigned gridy, int d, float *out, hipStream_t s)
{
    F3M_LAUNCH(root_geometry_kernel, 1, 2 * kMaxD * 32, 0, s, partx, gridx, party, gridy, d, out);
    check_launch("root_geometry");
}

// ------------------------------------------------------------------------------------------------
// Morton keys.  Cell of a point at the key depth L, per dimension (F3M_src/1_d_conv.cu:1142-1144):
//   g_j = (int) floor( (2^L * (x_j - origin_j)) / edge0 )
// Scaling by a power of two commutes with rounding, so the cell at depth k <= L is g_j >> (L-k):
// one key serves every level.  Key = child digits, coarsest level first; the digit of a level has
// bit j set when the point lies in the upper half along dimension j (sign table of
// F3M_src/1_d_conv.cu:895-897), which makes the natural child index of the reference the digit.

template <int K> struct __attribute__((aligned(4))) point_row { float v[K]; };   // K floats at any 4-byte boundary

// origin (D floats) and edge0 are read from device memory: the root geometry need not have reached the host
template <int D>
__global__ void morton_kernel(const float *__restrict__ X, long long n, const float *__restrict__ origin,
                              const float *__restrict__ edge0p, int L, uint32_t *__restrict__ keys, int *__restrict__ idx)
{
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float edge0 = *edge0p;
    const float side = (float)(1u << L);
    const int top = (1 << L) - 1;
    const point_row<D> row = *reinterpret_cast<const point_row<D> *>(X + i * D);   // the row with one request
    int cell[D];
#pragma unroll
    for (int j = 0; j < D; j++) {
        float a = row.v[j] - origin[j];
        float q = side * a;
        q = q / edge0;
        int c = (int)floorf(q);
        cell[j] = c < 0 ? 0 : (c > top ? top : c);
    }
    uint32_t key = 0;
    for (int l = L - 1; l >= 0; l--) {
        uint32_t digit = 0;
#pragma unroll
        for (int j = 0; j < D; j++) digit |= (uint32_t)((cell[j] >> l) & 1) << j;
        key = (key << D) | digit;
    }
    keys[i] = key;
    idx[i] = (int)i;
}

// ------------------------------------------------------------------------------------------------
// Counting sort by 8-bit digits, least significant first; stable.  A workgroup of four wavefronts
// takes a tile of 8192 keys (2048 per wavefront, in order).  Inside a round of 64 keys the rank of a key
// among equal digits comes from eight ballots; running digit counts per wavefront live in LDS.  The
// tile is first reordered by digit inside LDS and then written out, so that the ~32 keys of a tile that
// share a digit leave as one contiguous run.

constexpr int kSortWaves = 4;
constexpr int kSortRounds = 32;
constexpr int kSortTile = kSortWaves * kWave * kSortRounds;

__global__ void __launch_bounds__(kSortWaves * 64) sort_hist_kernel(const uint32_t *__restrict__ keys, long long n, int shift,
                                                                    int *__restrict__ blockhist, int nblk)
{
    __shared__ int hist[256];
    const int tid = threadIdx.x;
    hist[tid] = 0;
    __syncthreads();
    const long long base = (long long)blockIdx.x * kSortTile;
    for (int r = 0; r < kSortRounds; r++) {
        long long i = base + (long long)r * (kSortWaves * kWave) + tid;
        if (i < n) atomicAdd(&hist[(keys[i] >> shift) & 255u], 1);
    }
    __syncthreads();
    blockhist[(long long)tid * nblk + blockIdx.x] = hist[tid];
}

__global__ void __launch_bounds__(kSortWaves * 64) sort_scatter_kernel(const uint32_t *__restrict__ keys_in,
                                                                       const int *__restrict__ idx_in,
                                                                       uint32_t *__restrict__ keys_out,
                                                                       int *__restrict__ idx_out, long long n, int shift,
                                                                       const int *__restrict__ base, int nblk)
{
    __shared__ int wrun[kSortWaves][256];     // per wavefront: keys of each digit met so far; then its offset
    __shared__ int tstart[256];               // first position of each digit inside the reordered tile
    __shared__ int gdelta[256];               // global position minus tile position, per digit
    __shared__ uint32_t skey[kSortTile];
    __shared__ int sval[kSortTile];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    for (int b = lane; b < 256; b += kWave) wrun[w][b] = 0;
    __syncthreads();
    const long long tile = (long long)blockIdx.x * kSortTile;
    const long long mine = tile + (long long)w * (kWave * kSortRounds);      // this wavefront's 2048 keys
    const unsigned long long below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    // the whole share goes to registers first, so that the loads of all rounds are in flight together
    uint32_t key[kSortRounds];
    int val[kSortRounds];
    int rk[kSortRounds];                      // rank among the keys of the same digit in this wavefront
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        long long i = mine + r * kWave + lane;
        key[r] = (i < n) ? keys_in[i] : 0u;
        val[r] = (i < n) ? idx_in[i] : 0;
    }
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        long long i = mine + r * kWave + lane;
        bool valid = i < n;
        uint32_t digit = (key[r] >> shift) & 255u;
        unsigned long long same = wave_ballot(valid);
#pragma unroll
        for (int bit = 0; bit < 8; bit++) {
            bool one = (digit >> bit) & 1u;
            unsigned long long m = wave_ballot(one);
            same &= one ? m : ~m;
        }
        int rank = __popcll(same & below);
        int start = valid ? wrun[w][digit] : 0;           // only this wavefront touches wrun[w]
        rk[r] = start + rank;
        wave_sync();                                       // every lane has read before the first lane of a digit writes
        if (valid && rank == 0) wrun[w][digit] = start + __popcll(same);
        wave_sync();
    }
    __syncthreads();
    // digit d: counts per wavefront -> offsets of the wavefronts, tile total -> start inside the tile
    {
        int c[kSortWaves], tot = 0;
#pragma unroll
        for (int v = 0; v < kSortWaves; v++) { c[v] = wrun[v][tid]; }
#pragma unroll
        for (int v = 0; v < kSortWaves; v++) { wrun[v][tid] = tot; tot += c[v]; }
        tstart[tid] = tot;
    }
    __syncthreads();
    if (w == 0) {                              // exclusive scan of the 256 totals by one wavefront
        int v[4], sum = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) { v[e] = tstart[lane * 4 + e]; sum += v[e]; }
        int incl = sum;
        for (int off = 1; off < 64; off <<= 1) {
            int t = wave_shfl_i(incl, lane >= off ? lane - off : lane);
            if (lane >= off) incl += t;
        }
        int run = incl - sum;
#pragma unroll
        for (int e = 0; e < 4; e++) { tstart[lane * 4 + e] = run; run += v[e]; }
    }
    __syncthreads();
    gdelta[tid] = base[(long long)tid * nblk + blockIdx.x] - tstart[tid];
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        long long i = mine + r * kWave + lane;
        if (i < n) {
            uint32_t digit = (key[r] >> shift) & 255u;
            int p = tstart[digit] + wrun[w][digit] + rk[r];
            skey[p] = key[r];
            sval[p] = val[r];
        }
    }
    __syncthreads();
    const int cnt = (int)min((long long)kSortTile, n - tile);
    for (int j = tid; j < cnt; j += kSortWaves * kWave) {
        const uint32_t k = skey[j];
        const int g = gdelta[(k >> shift) & 255u] + j;
        keys_out[g] = k;
        idx_out[g] = sval[j];
    }
}

// stable sort by key bits [from, bits), 8 bits per pass
static void radix_sort(DBuf<uint32_t> &keys, DBuf<int> &idx, long long n, int from, int bits, hipStream_t s)
{
    int nblk = (int)cdiv(n, kSortTile);
    DBuf<uint32_t> keys2((size_t)n);
    DBuf<int> idx2((size_t)n);
    DBuf<int> hist((size_t)256 * nblk);
    DBuf<int> base((size_t)256 * nblk + 1);
    for (int shift = from; shift < bits; shift += 8) {
        F3M_LAUNCH(sort_hist_kernel, nblk, kSortWaves * kWave, 0, s, keys.get(), n, shift, hist.get(), nblk);
        check_launch("sort_hist");
        exclusive_scan_i32(hist.get(), (long long)256 * nblk, base.get(), s);
        F3M_LAUNCH(sort_scatter_kernel, nblk, kSortWaves * kWave, 0, s, keys.get(), idx.get(), keys2.get(), idx2.get(), n, shift,
                   base.get(), nblk);
        check_launch("sort_scatter");
        std::swap(keys, keys2);
        std::swap(idx, idx2);
    }
}

// depth 0: one box with every point, centred at origin + edge0/2 (F3M_src/n_tree.cu:86-95)
__global__ void root_level_kernel(Geo g, int n, int *__restrict__ off, uint32_t *__restrict__ prefix, float *__restrict__ ctr,
                                  int *__restrict__ cell, uint32_t *__restrict__ cellpack)
{
    int j = threadIdx.x;
    if (j == 0) { off[0] = 0; off[1] = n; prefix[0] = 0u; cellpack[0] = 0u; }
    if (j < g.d) {
        float half = 0.5f * g.edge0;
        ctr[j] = g.origin[j] + half;
        cell[j] = 0;
    }
}

// keys and their order from the root geometry in device memory (origin: d floats, edge0p: one)
void sort_tree_launch(Tree &t, const float *X, long long n, int d, int L, const float *origin, const float *edge0p, hipStream_t s)
{
    t.n = n;
    t.keys.reset((size_t)n);
    t.perm.reset((size_t)n);
#define F3M_CASE(DD)                                                                                                    \
    case DD:                                                                                                            \
        F3M_LAUNCH((morton_kernel<DD>), cdiv(n, 256), 256, 0, s, X, n, origin, edge0p, L, t.keys.get(), t.perm.get());   \
        break;
    switch (d) {
        F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
        F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
    default: throw Error(2, "dimension must be 1..10");
    }
#undef F3M_CASE
    check_launch("morton");
    // Only the leading 16 key bits are sorted at first: a division at depth k looks at the leading d*k
    // bits, and most trees stop before d*k exceeds 16.  divide_tree sorts further bits when it gets there.
    t.sorted_from = std::max(0, d * L - 16);
    radix_sort(t.keys, t.perm, n, t.sorted_from, d * L, s);
}

// the root level, once the host has the geometry (F3M_src/n_tree.cu:86-95)
void root_level_launch(Tree &t, const Geo &geo, hipStream_t s)
{
    t.geo = geo;
    const long long n = t.n;
    t.lev.clear();
    t.lev.reserve(40);
    t.lev.emplace_back();
    TreeLevel &r = t.lev[0];
    r.depth = 0;
    r.edge = geo.edge0;
    r.nb = 1;
    r.maxcount = (int)n;
    r.off.reset(2);
    r.prefix.reset(1);
    r.ctr.reset(geo.d);
    r.cell.reset(geo.d);
    r.cellpack.reset(1);
    F3M_LAUNCH(root_level_kernel, 1, 64, 0, s, geo, (int)n, r.off.get(), r.prefix.get(), r.ctr.get(), r.cell.get(),
               r.cellpack.get());
    check_launch("root_level");
}

void gather_tree_points(Tree &t, const float *X, hipStream_t s, bool background)
{
    t.pts.reset((size_t)t.n * t.geo.d);
    gather_points(X, t.perm.get(), t.n, t.geo.d, t.pts.get(), s, background);
}

// ------------------------------------------------------------------------------------------------
// One division (F3M_src/n_tree.cu:98-179).  Candidates are the 2^d children of every box, natural
// index = parent*2^d + child; their point ranges are found by binary search in the sorted keys.

// (a device function with its workgroup index as an argument: the level loop launches it together with the list
// builder's counting pass in one grid)
struct BoundsArgs {
    const uint32_t *keys, *prefix_prev;
    const int *off_prev;
    long long ncand, n;
    int d, shift;
    int *natpos;
    unsigned grid;              // workgroups of 256 threads (0: nothing to do)
};
__device__ inline void child_bounds_body(unsigned blk, const BoundsArgs &a)
{
    long long nat = (long long)blk * 256 + threadIdx.x;
    if (nat > a.ncand) return;
    if (nat == a.ncand) { a.natpos[nat] = (int)a.n; return; }
    int q = (int)(nat >> a.d);
    uint32_t target = (a.prefix_prev[q] << a.d) | (uint32_t)(nat & ((1 << a.d) - 1));
    int lo = a.off_prev[q], hi = a.off_prev[q + 1];
    // first position in [lo, hi) whose key is not below the target.  The range is cut in eight per step, seven probes
    // whose loads do not wait for each other, instead of in two: the kernel's time is the chain of dependent loads
    // (23 steps of ~1 us in a parent of 1e7 points, now 8).
    while (hi - lo > 8) {
        const int step = (hi - lo) >> 3;
        bool below[7];
#pragma unroll
        for (int u = 0; u < 7; u++) below[u] = (a.keys[lo + (u + 1) * step] >> a.shift) < target;
        int nb = 0;                                   // probes below the target (they are a prefix: the keys are sorted)
#pragma unroll
        for (int u = 0; u < 7; u++) nb += below[u] ? 1 : 0;
        const int nlo = nb ? lo + nb * step + 1 : lo;
        hi = nb < 7 ? lo + (nb + 1) * step : hi;
        lo = nlo;
    }
    while (lo < hi) {
        int mid = lo + ((hi - lo) >> 1);
        if ((a.keys[mid] >> a.shift) < target) lo = mid + 1; else hi = mid;
    }
    a.natpos[nat] = lo;
}

// stats[0] = number of non-empty children, stats[1] = largest count
__global__ void build_level_kernel(const int *__restrict__ natpos, const int *__restrict__ cid, long long ncand, int d,
                                   const uint32_t *__restrict__ prefix_prev, const float *__restrict__ ctr_prev,
                                   const int *__restrict__ cell_prev, float quarter, int *__restrict__ off,
                                   uint32_t *__restrict__ prefix, float *__restrict__ ctr, int *__restrict__ cell,
                                   uint32_t *__restrict__ cellpack, int depth,
                                   int *__restrict__ childstart_prev, int *__restrict__ parent, int *__restrict__ stats)
{
    long long nat = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (nat > ncand) return;
    int id = cid[nat];
    int q = (int)(nat >> d);
    int child = (int)(nat & ((1 << d) - 1));
    if (nat == ncand) {
        off[id] = natpos[nat];
        childstart_prev[q] = id;
        stats[0] = id;
        return;
    }
    if (child == 0) childstart_prev[q] = id;
    int cnt = natpos[nat + 1] - natpos[nat];
    if (cnt > 0) {
        off[id] = natpos[nat];
        parent[id] = q;
        prefix[id] = (prefix_prev[q] << d) | (uint32_t)child;
        uint32_t pack = 0u;
        for (int j = 0; j < d; j++) {
            float step = ((child >> j) & 1) ? quarter : -quarter;      // 0.25*edge*sign, exact
            ctr[(long long)id * d + j] = ctr_prev[(long long)q * d + j] + step;
            const int cj = 2 * cell_prev[(long long)q * d + j] + ((child >> j) & 1);
            cell[(long long)id * d + j] = cj;
            pack |= (uint32_t)cj << (j * depth);                       // d * depth <= 31
        }
        cellpack[id] = pack;
        atomicMax(&stats[1], cnt);
    }
}

// Count of the fullest cell of the grid that the leading `bits` key bits resolve, added to *out by atomicMax (the
// caller keeps *out zero).  One thread per cell: the range of its keys by two binary searches in the sorted keys.
__global__ void max_run_kernel(const uint32_t *__restrict__ keys, long long n, int shift, unsigned ncell, int *__restrict__ out)
{
    const unsigned p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= ncell) return;
    auto lower = [&](unsigned q) {                   // first index whose prefix is >= q
        long long lo = 0, hi = n;
        while (lo < hi) {
            const long long mid = lo + ((hi - lo) >> 1);
            if ((keys[mid] >> shift) < q) lo = mid + 1; else hi = mid;
        }
        return lo;
    };
    const long long cnt = lower(p + 1) - lower(p);
    if (cnt > 0) atomicMax(out, (int)cnt);
}

int sorted_levels(const Tree &t) { return (t.geo.d * t.geo.L - t.sorted_from) / t.geo.d; }

void max_run_launch(const Tree &t, int *dout, hipStream_t s)
{
    const int bits = t.geo.d * sorted_levels(t), shift = t.geo.d * t.geo.L - bits;     // bits <= 16
    const unsigned ncell = 1u << bits;
    F3M_LAUNCH(max_run_kernel, cdiv(ncell, 256), 256, 0, s, t.keys.get(), t.n, shift, ncell, dout);
    check_launch("max_run");
}

void sort_more_bits(Tree &t, hipStream_t s)
{
    if (t.sorted_from == 0) return;
    t.sorted_from = std::max(0, t.sorted_from - 8);
    radix_sort(t.keys, t.perm, t.n, t.sorted_from, t.geo.d * t.geo.L, s);
}

bool divide_will_sort(const Tree &t)
{
    const int k = (int)t.lev.size();
    return t.geo.d * (t.geo.L - k) < t.sorted_from;
}

// The division to the next depth in three steps, so that the level loop can queue the first two together with the
// list builder's counting pass and scans: divide_prepare sorts further key bits if the depth needs them, allocates
// the new level and describes the search for the candidates' point ranges; (the ranges are found and the "not empty"
// flags scanned by the caller's launches;) divide_build queues the kernel that fills the level and appends it.
struct DividePending {
    DBuf<int> natpos, cid;
    TreeLevel cur;
    long long ncand = 0;
    bool active = false;
};
static BoundsArgs divide_prepare(Tree &t, DividePending &dp, hipStream_t s)
{
    const int d = t.geo.d;
    const int k = (int)t.lev.size();   // depth being built
    F3M_REQUIRE(k <= t.geo.L, 20, "depth %d exceeds the key depth", k);
    int shift = d * (t.geo.L - k);
    if (shift < t.sorted_from) {
        // the points are grouped by the boxes built so far whatever the order inside a box, so the
        // offsets of those levels stay valid when the order is refined
        t.sorted_from = std::max(0, std::min(shift, t.sorted_from - 8));
        radix_sort(t.keys, t.perm, t.n, t.sorted_from, d * t.geo.L, s);
    }
    TreeLevel &prev = t.lev[k - 1];
    const long long ncand = (long long)prev.nb << d;
    F3M_REQUIRE(ncand < (1ll << 31) - 2, 20, "too many candidate boxes at depth %d (%lld)", k, ncand);
    dp.ncand = ncand;
    dp.natpos.reset((size_t)ncand + 1);
    dp.cid.reset((size_t)ncand + 1);
    size_t bound = (size_t)std::min<long long>(ncand, t.n);
    TreeLevel &cur = dp.cur;
    cur.depth = k;
    cur.off.reset(bound + 1);
    cur.prefix.reset(bound);
    cur.ctr.reset(bound * d);
    cur.cell.reset(bound * d);
    cur.cellpack.reset(bound);
    cur.parent.reset(bound);
    prev.childstart.reset((size_t)prev.nb + 1);
    dp.active = true;
    BoundsArgs a;
    a.keys = t.keys.get(); a.prefix_prev = prev.prefix.get(); a.off_prev = prev.off.get();
    a.ncand = ncand; a.n = t.n; a.d = d; a.shift = shift; a.natpos = dp.natpos.get();
    a.grid = cdiv(ncand + 1, 256);
    return a;
}
static void divide_build(Tree &t, DividePending &dp, int *dstats, hipStream_t s)
{
    const int d = t.geo.d;
    const int k = (int)t.lev.size();
    TreeLevel &prev = t.lev[k - 1];
    TreeLevel &cur = dp.cur;
    float quarter = 0.25f * prev.edge;
    F3M_LAUNCH(build_level_kernel, cdiv(dp.ncand + 1, 256), 256, 0, s, dp.natpos.get(), dp.cid.get(), dp.ncand, d, prev.prefix.get(),
               prev.ctr.get(), prev.cell.get(), quarter, cur.off.get(), cur.prefix.get(), cur.ctr.get(), cur.cell.get(),
               cur.cellpack.get(), k, prev.childstart.get(), cur.parent.get(), dstats);
    check_launch("build_level");
    cur.nb = -1;                       // until divide_finish
    cur.maxcount = -1;
    cur.edge = prev.edge * 0.5f;
    t.lev.push_back(std::move(cur));
    dp.active = false;
}

void divide_finish(Tree &t, const int *hstats)
{
    t.lev.back().nb = hstats[0];
    t.lev.back().maxcount = hstats[1];
}

void divide_discard(Tree &t) { t.lev.pop_back(); }

// ------------------------------------------------------------------------------------------------
// Grid key -> box id through an open-addressing table in HBM (F3M_src/linearprobing.cu:18-87, used by
// the reference in box_division_assign_hash, F3M_src/1_d_conv.cu:1127-1191): slot = Murmur3 finaliser
// of the key modulo capacity-1, linear probing (slot+1) % (capacity-1), empty = 0xffffffff, which is
// also the answer for an absent key (-1 as an int).  The engine itself never needs the table -- its
// keys are sorted and its box ids dense -- but callers that hold cell coordinates (a point that is
// not part of the plan, a neighbour cell) get the box id the reference's lookup would give.

__host__ __device__ inline uint32_t hash_slot(uint32_t k, uint32_t capacity)
{
    k ^= k >> 16;
    k *= 0x85ebca6bu;
    k ^= k >> 13;
    k *= 0xc2b2ae35u;
    k ^= k >> 16;
    return k % (capacity - 1u);
}

uint32_t hash_slot_host(uint32_t key, uint32_t capacity) { return hash_slot(key, capacity); }

// the reference's key of a cell: sum_j g_j (2^k)^(d-1-j), int32 (F3M_src/1_d_conv.cu:1142-1144)
__device__ inline uint32_t cell_key(const int *__restrict__ cell, int d, int depth)
{
    int key = 0;
    for (int j = 0; j < d; j++) key = (key << depth) + cell[j];   // Horner form of the same sum
    return (uint32_t)key;
}

__global__ void hash_insert_kernel(const int *__restrict__ cell, int nb, int d, int depth, uint32_t *__restrict__ table,
                                   uint32_t capacity)
{
    int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nb) return;
    const uint32_t key = cell_key(cell + (long long)b * d, d, depth);
    uint32_t slot = hash_slot(key, capacity);
    for (uint32_t tries = 0; tries < capacity; tries++) {           // bounded: the table is at most half full
        const uint32_t prev = atomicCAS(&table[2 * (size_t)slot], 0xffffffffu, key);
        if (prev == 0xffffffffu || prev == key) { table[2 * (size_t)slot + 1] = (uint32_t)b; return; }
        slot = (slot + 1u) % (capacity - 1u);
    }
}

__global__ void hash_lookup_kernel(const int *__restrict__ cells, long long n, int d, int depth,
                                   const uint32_t *__restrict__ table, uint32_t capacity, int *__restrict__ ids)
{
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int side = 1 << depth;
    bool inside = true;
    for (int j = 0; j < d; j++) inside = inside && cells[i * d + j] >= 0 && cells[i * d + j] < side;
    int id = -1;
    if (inside) {
        const uint32_t key = cell_key(cells + i * d, d, depth);
        uint32_t slot = hash_slot(key, capacity);
        for (uint32_t tries = 0; tries < capacity; tries++) {
            const uint32_t k = table[2 * (size_t)slot];
            if (k == key) { id = (int)table[2 * (size_t)slot + 1]; break; }
            if (k == 0xffffffffu) break;
            slot = (slot + 1u) % (capacity - 1u);
        }
    }
    ids[i] = id;
}

void lookup_boxes(const Tree &t, const TreeLevel &lev, const int *cells, long long n, int *ids, hipStream_t s)
{
    const int d = t.geo.d;
    F3M_REQUIRE(d * lev.depth <= 31, 23, "grid keys of depth %d do not fit in 32 bits", lev.depth);
    if (lev.hashcap == 0) {
        // capacity: the power of two that leaves the table at most half full (the reference takes
        // max(2^20, that), F3M_src/n_tree.cu:113-116)
        uint32_t cap = 1024;
        while (cap < 2u * (uint32_t)lev.nb) cap <<= 1;
        lev.hashtab.reset(2 * (size_t)cap);
        dev_fill(lev.hashtab.get(), 0xff, sizeof(uint32_t) * 2 * (size_t)cap, s);
        F3M_LAUNCH(hash_insert_kernel, cdiv(lev.nb, 256), 256, 0, s, lev.cell.get(), lev.nb, d, lev.depth, lev.hashtab.get(),
                   cap);
        check_launch("hash_insert");
        lev.hashcap = cap;
    }
    if (n == 0) return;
    F3M_LAUNCH(hash_lookup_kernel, cdiv(n, 256), 256, 0, s, cells, n, d, lev.depth, lev.hashtab.get(), lev.hashcap, ids);
    check_launch("hash_lookup");
}

// ------------------------------------------------------------------------------------------------
// Interaction lists of depth k from the keep list of depth k-1
// (F3M_src/n_tree.cu:594-641 expansion, 788-811 filter, 701-787 + F3M_src/1_d_conv.cu:903-1029 classes).
// Children of a keep pair (x,y) are enumerated in the reference's order (x, child of x, y, child of
// y); only non-empty children exist here, so the filter step is implicit.

// 0 small, 1 far, 2 keep, 3 dropped (F3M_src/1_d_conv.cu:927-952 and :983-1026)
template <int D>
__device__ inline int classify_pair(const float *__restrict__ cx, const float *__restrict__ cy, int size, const ClassifyParams &cp)
{
    if (cp.do_init && size < 2 * cp.nr_interp) return 0;
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < D; j++) {
        float dk = cy[j] - cx[j];
        float sq = dk * dk;
        acc = acc + sq;
    }
    float dist = sqrtf(acc);
    float thr = cp.edge * 2.f;
    if (dist >= thr) return cp.do_init ? 1 : 3;
    if (cp.var_comp) {
        float v = dist * dist;
        v = v * cp.lcs;
        if (cp.en_pair && (double)v <= 1e-2) return 1;
        if (cp.en_all && dist <= cp.crit) return 1;
    }
    if (size < 2 * cp.small_limit) return 0;
    return 2;
}

// One wavefront per box bx of depth k.  Its candidates are the children of the keep partners of its
// parent; lane l takes partner t0 + l (then t0 + 64 + l, ...) and walks that partner's children, so
// candidates are met in the order (partner, child) = increasing y box, the order of the reference.
// WRITE = false counts the three classes per box; WRITE = true recomputes the classes and writes the
// pairs at the offsets that the scan of those counts gave (which are also the row pointers).
constexpr int kListWaves = 4;   // wavefronts per workgroup

template <bool WRITE, int D>
__device__ inline void lists_body(
    unsigned blk, int nbx, const int *__restrict__ parentx, const int *__restrict__ csy, const int *__restrict__ keep_pairs,
    const int *__restrict__ keep_rowptr, const int *__restrict__ offx, const int *__restrict__ offy,
    const float *__restrict__ ctrx, const float *__restrict__ ctry, ClassifyParams cp,
    const uint32_t *__restrict__ cellx, const uint32_t *__restrict__ celly, int depth, bool one_tree,
    unsigned long long *__restrict__ outliers,
    unsigned long long *__restrict__ beyond,
    long long *__restrict__ cnt /* 3 arrays of nbx+1 */, const long long *__restrict__ pos /* 3 arrays of nbx+1 */,
    int *__restrict__ out_small, int *__restrict__ out_far, int *__restrict__ out_keep, int *__restrict__ rp_small,
    int *__restrict__ rp_far, int *__restrict__ rp_keep)
{
    const int lane = threadIdx.x & 63;
    const int bx = (int)blk * kListWaves + (threadIdx.x >> 6);
    if (bx > nbx) return;
    const long long stride = (long long)nbx + 1;
    if (bx == nbx) {                               // the closing entry of the row pointers
        if (WRITE && lane == 0) {
            rp_small[bx] = (int)pos[bx]; rp_far[bx] = (int)pos[stride + bx]; rp_keep[bx] = (int)pos[2 * stride + bx];
        }
        return;
    }
    const int x = parentx[bx];
    const int t0 = keep_rowptr[x], t1 = keep_rowptr[x + 1];
    const int nx = offx[bx + 1] - offx[bx];
    const uint32_t mycell = WRITE ? 0u : cellx[bx];
    constexpr int d = D;
    float cx[D];
#pragma unroll
    for (int j = 0; j < D; j++) cx[j] = ctrx[(long long)bx * D + j];
    long long base0 = 0, base1 = 0, base2 = 0;
    if (WRITE) {
        base0 = pos[bx]; base1 = pos[stride + bx]; base2 = pos[2 * stride + bx];
        if (lane == 0) { rp_small[bx] = (int)base0; rp_far[bx] = (int)base1; rp_keep[bx] = (int)base2; }
    }
    long long c0 = 0, c1 = 0, c2 = 0;              // candidates of each class met so far (uniform)
    const int nchild = 1 << d;
    const unsigned long long below = (1ull << lane) - 1ull;
    for (int tb = t0; tb < t1; tb += 64) {
        // lane l holds the child range of partner tb + l; then the 64 x 2^d (partner, child) slots are
        // classified 64 at a time, lane = slot, which keeps the order (partner, child)
        int y0 = 0, y1 = 0;
        if (tb + lane < t1) { const int y = keep_pairs[2 * (long long)(tb + lane) + 1]; y0 = csy[y]; y1 = csy[y + 1]; }
        const int nslots = min(64, t1 - tb) << d;
#pragma unroll 2
        for (int s0 = 0; s0 < nslots; s0 += 64) {
            const int slot = s0 + lane;
            const int p = slot >> d, cj = slot & (nchild - 1);
            const int by = wave_shfl_i(y0, p) + cj;
            const bool there = by < wave_shfl_i(y1, p);
            int c = 3;
            if (there) {
                const int size = nx + (offy[by + 1] - offy[by]);
                float cy[D];
#pragma unroll
                for (int j = 0; j < D; j++) cy[j] = ctry[(long long)by * D + j];
                c = classify_pair<D>(cx, cy, size, cp);
                if (!WRITE && c == 1) {
                    // The cell offset of a far pair must lie inside the M2L tables of the level.  One tree: a pair is
                    // regular if every offset from twice the parent's cell is in -2..3, or if it is a child of a
                    // parent two cells away along exactly one axis: -4, -3, 4 or 5 there and 0 or 1 elsewhere.
                    // (cells from one packed word per box: one load per far pair instead of d)
                    const uint32_t wy = celly[by], cmask = (1u << depth) - 1u;
                    bool outside = false;
                    int nout = 0, nmid = 0, nbad = 0;
#pragma unroll
                    for (int j = 0; j < D; j++) {
                        const int yj = (int)((wy >> (j * depth)) & cmask), xj = (int)((mycell >> (j * depth)) & cmask);
                        const int o = yj - xj - cp.omin[j];
                        outside = outside || o < 0 || o >= kM2LOffsets;
                        int u = yj - 2 * (xj >> 1);
                        if (u < -2 || u > 3) {
                            nout++;
                            if (u < -4 || u > 5) nbad++;
                        } else if (u == 0 || u == 1) {
                            nmid++;
                        }
                    }
                    if (outside) atomicAdd(beyond, 1ull);
                    if (one_tree && nout > 0 && (nout > 1 || nbad > 0 || nmid != d - 1)) atomicAdd(outliers, 1ull);
                }
            }
            const unsigned long long m0 = wave_ballot(c == 0), m1 = wave_ballot(c == 1), m2 = wave_ballot(c == 2);
            if (WRITE) {
                if (c == 0) { const long long q = base0 + c0 + __popcll(m0 & below); out_small[2 * q] = bx; out_small[2 * q + 1] = by; }
                else if (c == 1) { const long long q = base1 + c1 + __popcll(m1 & below); out_far[2 * q] = bx; out_far[2 * q + 1] = by; }
                else if (c == 2) { const long long q = base2 + c2 + __popcll(m2 & below); out_keep[2 * q] = bx; out_keep[2 * q + 1] = by; }
            }
            c0 += __popcll(m0); c1 += __popcll(m1); c2 += __popcll(m2);
        }
    }
    if (!WRITE && lane == 0) { cnt[bx] = c0; cnt[stride + bx] = c1; cnt[2 * stride + bx] = c2; }
}

// the writing pass on its own
template <int D>
__global__ void __launch_bounds__(kListWaves * 64) lists_write_kernel(
    int nbx, const int *__restrict__ parentx, const int *__restrict__ csy, const int *__restrict__ keep_pairs,
    const int *__restrict__ keep_rowptr, const int *__restrict__ offx, const int *__restrict__ offy,
    const float *__restrict__ ctrx, const float *__restrict__ ctry, ClassifyParams cp, int depth, bool one_tree,
    const long long *__restrict__ pos, int *__restrict__ out_small, int *__restrict__ out_far, int *__restrict__ out_keep,
    int *__restrict__ rp_small, int *__restrict__ rp_far, int *__restrict__ rp_keep)
{
    lists_body<true, D>(blockIdx.x, nbx, parentx, csy, keep_pairs, keep_rowptr, offx, offy, ctrx, ctry, cp, nullptr, nullptr, depth,
                        one_tree, nullptr, nullptr, nullptr, pos, out_small, out_far, out_keep, rp_small, rp_far, rp_keep);
}

// One launch for the two independent things a step of the level loop starts with: the counting pass of the lists of
// depth k (workgroups [0, la.grid)) and the point ranges of the candidate boxes of depth k+1, for one tree or two
// (workgroups after that).  Either part may be absent (grid 0).
struct ListsCountArgs {
    int nbx;
    const int *parentx, *csy, *keep_pairs, *keep_rowptr, *offx, *offy;
    const float *ctrx, *ctry;
    ClassifyParams cp;
    const uint32_t *cellx, *celly;
    int depth;
    bool one_tree;
    unsigned long long *outliers, *beyond;
    long long *cnt;
    unsigned grid;
};
template <int D>
__global__ void __launch_bounds__(kListWaves * 64) level_count_kernel(ListsCountArgs la, BoundsArgs b0, BoundsArgs b1)
{
    unsigned blk = blockIdx.x;
    if (blk < la.grid) {
        lists_body<false, D>(blk, la.nbx, la.parentx, la.csy, la.keep_pairs, la.keep_rowptr, la.offx, la.offy, la.ctrx, la.ctry,
                             la.cp, la.cellx, la.celly, la.depth, la.one_tree, la.outliers, la.beyond, la.cnt, nullptr, nullptr,
                             nullptr, nullptr, nullptr, nullptr, nullptr);
        return;
    }
    blk -= la.grid;
    if (blk < b0.grid) { child_bounds_body(blk, b0); return; }
    child_bounds_body(blk - b0.grid, b1);
}

// Row statistics of the small and the keep list of a level from the per-box counts of the list builder's counting
// pass (cnt: three arrays of `stride` entries, small, far, keep): out[4c .. 4c+3] (c = 0 small, 1 keep) += x boxes
// with pairs, their points, their pieces of 128 and of 160 points (out is zero before).
constexpr int kRowStatBlock = 256;
__global__ void __launch_bounds__(kRowStatBlock) list_rowstats_kernel(const long long *__restrict__ cnt, long long stride,
                                                                       const int *__restrict__ offx, int nbx,
                                                                       unsigned long long *__restrict__ out)
{
    __shared__ unsigned long long acc[8];
    if (threadIdx.x < 8) acc[threadIdx.x] = 0;
    __syncthreads();
    const int b = blockIdx.x * kRowStatBlock + threadIdx.x;
    if (b < nbx) {
        const unsigned long long n = (unsigned long long)(offx[b + 1] - offx[b]);
        for (int c = 0; c < 2; c++) {
            if (cnt[(c ? 2 : 0) * stride + b] > 0) {
                atomicAdd(&acc[4 * c + 0], 1ull);
                atomicAdd(&acc[4 * c + 1], n);
                atomicAdd(&acc[4 * c + 2], (n + 127) / 128);
                atomicAdd(&acc[4 * c + 3], (n + 159) / 160);
            }
        }
    }
    __syncthreads();
    if (threadIdx.x < 8 && acc[threadIdx.x]) atomicAdd(&out[threadIdx.x], acc[threadIdx.x]);
}

__global__ void rowptr_kernel(const int *__restrict__ pairs, long long n, int nbx, int *__restrict__ rowptr)
{
    int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b > nbx) return;
    long long lo = 0, hi = n;
    while (lo < hi) {
        long long mid = lo + ((hi - lo) >> 1);
        if (pairs[2 * mid] < b) lo = mid + 1; else hi = mid;
    }
    rowptr[b] = (int)lo;
}

void build_rowptr(PairList &l, int nbx, hipStream_t s)
{
    l.rowptr.reset((size_t)nbx + 1);
    F3M_LAUNCH(rowptr_kernel, cdiv((long long)nbx + 1, 256), 256, 0, s, l.pairs.get(), l.n, nbx, l.rowptr.get());
    check_launch("rowptr");
}

// ------------------------------------------------------------------------------------------------
// A list seen from its Y boxes.  The predicates of a pair depend on n_x + n_y and on |c_y - c_x| only
// (F3M_src/1_d_conv.cu:927-952), so the lists of the problem (Y, X) are these lists with the boxes of every pair
// swapped, in the order (by, bx): a stable sort by `by` of pairs that are already sorted by bx.

__global__ void split_pairs_kernel(const int *__restrict__ pairs, long long n, uint32_t *__restrict__ key, int *__restrict__ val)
{
    long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < n) { key[t] = (uint32_t)pairs[2 * t + 1]; val[t] = pairs[2 * t]; }
}
__global__ void join_pairs_kernel(const uint32_t *__restrict__ key, const int *__restrict__ val, long long n, int *__restrict__ pairs)
{
    long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < n) { pairs[2 * t] = (int)key[t]; pairs[2 * t + 1] = val[t]; }
}
// row statistics of one list (the first four words of list_rowstats_kernel's record)
__global__ void __launch_bounds__(kRowStatBlock) one_list_rowstats_kernel(const int *__restrict__ rowptr, const int *__restrict__ off,
                                                                           int nb, unsigned long long *__restrict__ out)
{
    __shared__ unsigned long long acc[4];
    if (threadIdx.x < 4) acc[threadIdx.x] = 0;
    __syncthreads();
    const int b = blockIdx.x * kRowStatBlock + threadIdx.x;
    if (b < nb && rowptr[b + 1] > rowptr[b]) {
        const unsigned long long n = (unsigned long long)(off[b + 1] - off[b]);
        atomicAdd(&acc[0], 1ull);
        atomicAdd(&acc[1], n);
        atomicAdd(&acc[2], (n + 127) / 128);
        atomicAdd(&acc[3], (n + 159) / 160);
    }
    __syncthreads();
    if (threadIdx.x < 4 && acc[threadIdx.x]) atomicAdd(&out[threadIdx.x], acc[threadIdx.x]);
}

void transpose_list(const PairList &in, const TreeLevel &ly, PairList &out, hipStream_t s)
{
    out.n = in.n;
    out.outliers = -1;
    out.beyond_tables = 0;
    out.pairs.reset((size_t)std::max<long long>(1, in.n) * 2);
    if (in.n > 0) {
        DBuf<uint32_t> key((size_t)in.n);
        DBuf<int> val((size_t)in.n);
        F3M_LAUNCH(split_pairs_kernel, cdiv(in.n, 256), 256, 0, s, in.pairs.get(), in.n, key.get(), val.get());
        check_launch("split_pairs");
        int bits = 1;
        while ((1ll << bits) < (long long)ly.nb) bits++;
        radix_sort(key, val, in.n, 0, bits, s);
        F3M_LAUNCH(join_pairs_kernel, cdiv(in.n, 256), 256, 0, s, key.get(), val.get(), in.n, out.pairs.get());
        check_launch("join_pairs");
    }
    build_rowptr(out, ly.nb, s);
    DBuf<unsigned long long> dstat(4);
    dev_fill(dstat.get(), 0, 4 * sizeof(unsigned long long), s);
    F3M_LAUNCH(one_list_rowstats_kernel, cdiv(ly.nb, kRowStatBlock), kRowStatBlock, 0, s, out.rowptr.get(), ly.off.get(), ly.nb,
               dstat.get());
    check_launch("one_list_rowstats");
    unsigned long long h[4];
    fetch_small(h, dstat.get(), 4, s);
    out.rows = (long long)h[0], out.row_points = (long long)h[1], out.items128 = (long long)h[2], out.items160 = (long long)h[3];
}

void level_launch(const PairList *keep_prev, Tree &tx, Tree &ty, int k, ClassifyParams &cp, ListsPending &pend,
                  long long *dtot, long long *drow, bool divide, int *dstats_x, int *dstats_y, hipStream_t s)
{
    const int d = tx.geo.d;
    const bool one_tree = &tx == &ty;
    pend.active = false;
    const bool lists = keep_prev != nullptr && keep_prev->n > 0;
    // the counting pass of the lists of depth k
    ListsCountArgs la;
    memset(&la, 0, sizeof(la));
    DBuf<long long> cnt;
    if (lists) {
        const TreeLevel &py = ty.lev[k - 1];
        const TreeLevel &lx = tx.lev[k], &ly = ty.lev[k];
        F3M_REQUIRE(keep_prev->n < (1ll << 31) - 2, 21, "keep list too long (%lld)", keep_prev->n);
        F3M_REQUIRE((1 << d) < (1 << 21), 21, "too many children per box");
        pend.active = true;
        const int nbx = lx.nb;
        pend.stride = (long long)nbx + 1;
        cnt.reset((size_t)(3 * pend.stride));
        pend.pos.reset((size_t)(3 * pend.stride));
        for (int j = 0; j < kMaxD; j++) cp.omin[j] = j < d ? m2l_table_omin(tx.geo.origin[j], ty.geo.origin[j], lx.edge) : 0;
        pend.grid = (unsigned)cdiv((long long)nbx + 1, kListWaves);
        la.nbx = nbx; la.parentx = lx.parent.get(); la.csy = py.childstart.get();
        la.keep_pairs = keep_prev->pairs.get(); la.keep_rowptr = keep_prev->rowptr.get();
        la.offx = lx.off.get(); la.offy = ly.off.get(); la.ctrx = lx.ctr.get(); la.ctry = ly.ctr.get();
        la.cp = cp; la.cellx = lx.cellpack.get(); la.celly = ly.cellpack.get(); la.depth = k; la.one_tree = one_tree;
        la.outliers = reinterpret_cast<unsigned long long *>(dtot + 3);
        la.beyond = reinterpret_cast<unsigned long long *>(dtot + 6);
        la.cnt = cnt.get();
        la.grid = pend.grid;
    }
    // the division to depth k+1 (the lists above read depth k and k-1 only; the new level is appended at the end)
    DividePending dx, dy;
    BoundsArgs bx, by;
    memset(&bx, 0, sizeof(bx));
    memset(&by, 0, sizeof(by));
    if (divide) {
        bx = divide_prepare(tx, dx, s);
        if (!one_tree) by = divide_prepare(ty, dy, s);
    }
    if (la.grid + bx.grid + by.grid == 0) return;
#define F3M_CASE(DD)                                                                                                          \
    case DD:                                                                                                                  \
        F3M_LAUNCH((level_count_kernel<DD>), la.grid + bx.grid + by.grid, kListWaves * 64, 0, s, la, bx, by);                 \
        break;
    switch (d) {
        F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
        F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
    default: throw Error(2, "dimension must be 1..10");
    }
#undef F3M_CASE
    check_launch("level_count");
    // the scans of both, and the row statistics of the small and the keep list, in one set of launches
    ScanJob job;
    if (lists) {
        for (int c = 0; c < 3; c++) job.add(cnt.get() + c * pend.stride, pend.pos.get() + c * pend.stride, la.nbx, 0);
        if (drow != nullptr) {
            job.offx = la.offx;
            job.rowstat = reinterpret_cast<unsigned long long *>(drow);
            job.rs_ch[0] = 0;
            job.rs_ch[1] = 2;
        }
    }
    if (divide) {
        job.add(dx.natpos.get(), dx.cid.get(), dx.ncand, 1);     // compact id = number of non-empty candidates before
        if (!one_tree) job.add(dy.natpos.get(), dy.cid.get(), dy.ncand, 1);
    }
    if (!multi_scan(job, s)) {
        // a level too large for the joint scans (more than kScanTile tiles per array): one scan after the other
        if (lists) {
            exclusive_scan_i64_batched(cnt.get(), la.nbx, pend.stride, 3, pend.pos.get(), s);
            if (drow != nullptr) {
                F3M_LAUNCH(list_rowstats_kernel, cdiv(la.nbx, kRowStatBlock), kRowStatBlock, 0, s, cnt.get(), pend.stride, la.offx,
                           la.nbx, reinterpret_cast<unsigned long long *>(drow));
                check_launch("list_rowstats");
            }
        }
        if (divide) {
            exclusive_scan_nonempty(dx.natpos.get(), dx.ncand, dx.cid.get(), s);
            if (!one_tree) exclusive_scan_nonempty(dy.natpos.get(), dy.ncand, dy.cid.get(), s);
        }
    }
    if (divide) {
        divide_build(tx, dx, dstats_x, s);
        if (!one_tree) divide_build(ty, dy, dstats_y, s);
    }
}

// allocates the small, far and keep list for cap[0..2] pairs and queues the writing pass
static void lists_write(ListsPending &pend, const long long *cap, const PairList &keep_prev, const Tree &tx, const Tree &ty, int k,
                        const ClassifyParams &cp, PlanLevel &out, hipStream_t s)
{
    const int d = tx.geo.d;
    const TreeLevel &py = ty.lev[k - 1];
    const TreeLevel &lx = tx.lev[k], &ly = ty.lev[k];
    const bool one_tree = &tx == &ty;
    const int nbx = lx.nb;
    out.small_.pairs.reset((size_t)std::max<long long>(1, cap[0]) * 2);
    out.far.pairs.reset((size_t)std::max<long long>(1, cap[1]) * 2);
    out.keep.pairs.reset((size_t)std::max<long long>(1, cap[2]) * 2);
    out.small_.rowptr.reset((size_t)pend.stride);
    out.far.rowptr.reset((size_t)pend.stride);
    out.keep.rowptr.reset((size_t)pend.stride);
#define F3M_CASE(DD)                                                                                                          \
    case DD:                                                                                                                  \
        F3M_LAUNCH((lists_write_kernel<DD>), pend.grid, kListWaves * 64, 0, s, nbx, lx.parent.get(), py.childstart.get(),     \
                   keep_prev.pairs.get(), keep_prev.rowptr.get(), lx.off.get(), ly.off.get(), lx.ctr.get(), ly.ctr.get(), cp, \
                   k, one_tree, (const long long *)pend.pos.get(), out.small_.pairs.get(), out.far.pairs.get(),               \
                   out.keep.pairs.get(), out.small_.rowptr.get(), out.far.rowptr.get(), out.keep.rowptr.get());                \
        break;
    switch (d) {
        F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
        F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
    default: throw Error(2, "dimension must be 1..10");
    }
#undef F3M_CASE
    check_launch("lists_write");
}

// A list cannot be longer than the candidates of the level, at most 4^d children pairs per keep pair of the level
// above, nor than all box pairs.  Where three lists of that many pairs are a modest allocation the writing pass is
// queued before the host has seen the sizes (it runs while the host waits for them).
constexpr long long kEarlyListBytes = 64ll << 20;       // per list
bool lists_write_early(ListsPending &pend, const PairList &keep_prev, const Tree &tx, const Tree &ty, int k,
                       const ClassifyParams &cp, PlanLevel &out, hipStream_t s)
{
    pend.written = false;
    if (!pend.active) return false;
    const int d = tx.geo.d;
    const long long per_keep = d <= 15 ? (1ll << (2 * d)) : (1ll << 30);
    long long cap = (long long)tx.lev[k].nb * (long long)ty.lev[k].nb;
    if (keep_prev.n <= cap / per_keep) cap = keep_prev.n * per_keep;
    if (cap * 8 > kEarlyListBytes) return false;
    const long long caps[3] = {cap, cap, cap};
    lists_write(pend, caps, keep_prev, tx, ty, k, cp, out, s);
    pend.written = true;
    return true;
}

void lists_finish(ListsPending &pend, const long long *tot, const PairList &keep_prev, const Tree &tx, const Tree &ty, int k,
                  const ClassifyParams &cp, PlanLevel &out, const long long *hrow, hipStream_t s)
{
    out.far.n = out.small_.n = out.keep.n = 0;
    if (!pend.active) return;
    if (hrow != nullptr) {
        PairList &sm = out.small_, &kp = out.keep;
        sm.rows = hrow[0], sm.row_points = hrow[1], sm.items128 = hrow[2], sm.items160 = hrow[3];
        kp.rows = hrow[4], kp.row_points = hrow[5], kp.items128 = hrow[6], kp.items160 = hrow[7];
    }
    const bool one_tree = &tx == &ty;
    for (int c = 0; c < 3; c++) F3M_REQUIRE(tot[c] < (1ll << 31) - 2, 22, "interaction list too long (%lld)", tot[c]);
    out.far.outliers = one_tree ? tot[3] : -1;
    out.far.beyond_tables = tot[6];
    F3M_REQUIRE(tot[6] == 0, 24, "%lld far pairs of depth %d lie outside the M2L tables (cell offsets beyond %d per dimension)",
                tot[6], k, kM2LOffsets);
    if (!pend.written) lists_write(pend, tot, keep_prev, tx, ty, k, cp, out, s);
    else {
        // written ahead of the sizes into lists allocated for an upper bound: the bound must have held
        const PairList *wl[3] = {&out.small_, &out.far, &out.keep};
        for (int c = 0; c < 3; c++)
            F3M_REQUIRE((size_t)tot[c] * 2 <= wl[c]->pairs.size(), 25, "interaction list of depth %d longer (%lld pairs) than its bound (%zu)",
                        k, tot[c], wl[c]->pairs.size() / 2);
    }
    out.small_.n = tot[0];
    out.far.n = tot[1];
    out.keep.n = tot[2];
    pend.pos.free();
    pend.active = false;
}

// Lists that were written ahead of their sizes sit in blocks allocated for an upper bound (up to 64 MiB per list).  A
// plan that is kept gives the surplus back: a list that fills less than half of a block of more than 1 MiB moves into
// a block of its own size.
void shrink_lists(PlanLevel &L, hipStream_t s)
{
    PairList *wl[3] = {&L.small_, &L.far, &L.keep};
    for (PairList *l : wl) {
        const size_t need = (size_t)std::max<long long>(1, l->n) * 2;
        if (l->pairs.size() * sizeof(int) <= ((size_t)1 << 20) || need * 2 > l->pairs.size()) continue;
        DBuf<int> fit(need);
        F3M_HIP(hipMemcpyAsync(fit.get(), l->pairs.get(), need * sizeof(int), hipMemcpyDeviceToDevice, s));
        std::swap(l->pairs, fit);       // the old block goes back to the pool; work queued later on this stream may reuse it
    }
}

}  // namespace f3m
