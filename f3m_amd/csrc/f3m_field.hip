// Field kernels for gfx950: exact dense products, the near field, and the far field
// (P2M -> M2L -> L2P) on Morton-sorted, dimension-major point arrays.
#include "f3m_engine.h"

#include <cmath>
#include <type_traits>
#include <cstdlib>
#include <cstring>

namespace f3m {

constexpr float kLog2e = 1.4426950408889634f;

// ------------------------------------------------------------------------------------------------
// permutations between caller order and sorted order

template <int K> struct __attribute__((aligned(4))) fvec { float v[K]; };   // K floats at any 4-byte boundary

// A row of X sits at a random place: it is fetched with one load of D floats, so that the row costs
// one request to the memory system rather than D.
template <int D>
__global__ void gather_points_kernel(const float *__restrict__ X, const int *__restrict__ perm, long long n,
                                     float *__restrict__ pts)
{
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const fvec<D> row = *reinterpret_cast<const fvec<D> *>(X + (long long)perm[i] * D);
#pragma unroll
        for (int j = 0; j < D; j++) pts[(long long)j * n + i] = row.v[j];
    }
}
// Workgroups of a gather: one thread per row, or, for a move that runs in the background beside many small
// latency-bound kernels (the level loop of the plan), one workgroup per compute unit that walks the rows in
// strides: the random reads of a full-size launch fill the memory system's queues and the small kernels'
// dependent loads then take several times as long (plan at N=1e7, 3-D: 1.05 -> 0.90 ms; 64 workgroups no
// longer finish in time, 1024 disturb as much as all).
static unsigned gather_grid(long long n, bool background)
{
    const unsigned full = cdiv(n, 256);
    if (!background) return full;
#ifndef F3M_CPU_EMU
    static std::mutex mu;
    static std::map<int, int> units;          // compute units per device
    int dev = 0, cu = 0;
    F3M_HIP(hipGetDevice(&dev));
    {
        std::lock_guard<std::mutex> g(mu);
        auto it = units.find(dev);
        if (it == units.end()) {
            F3M_HIP(hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev));
            it = units.emplace(dev, std::max(cu, 1)).first;
        }
        cu = it->second;
    }
    return std::min<unsigned>(full, (unsigned)cu);
#else
    return full;
#endif
}
void gather_points(const float *X, const int *perm, long long n, int d, float *pts, hipStream_t s, bool background)
{
#define F3M_CASE(DD)                                                                                  \
    case DD:                                                                                          \
        F3M_LAUNCH((gather_points_kernel<DD>), gather_grid(n, background), 256, 0, s, X, perm, n, pts); \
        break;
    switch (d) {
        F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
        F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
    default: throw Error(2, "dimension must be 1..10");
    }
#undef F3M_CASE
    check_launch("gather_points");
}

// Columns col .. col+NC-1 of row perm[i] of b (row-major, c columns) to NC arrays bstride apart: a row sits at a
// random place, so its NC values are fetched with one load.  VEC: the row slice is read as one vector of NC
// floats (any 4-byte alignment), else value by value.
template <int NC>
__global__ void gather_columns_kernel(const float *__restrict__ b, const int *__restrict__ perm, long long n, int c, int col,
                                      float *__restrict__ bs, long long bstride)
{
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const fvec<NC> row = *reinterpret_cast<const fvec<NC> *>(b + (long long)perm[i] * c + col);
#pragma unroll
        for (int q = 0; q < NC; q++) bs[q * bstride + i] = row.v[q];
    }
}
void gather_columns(const float *b, const int *perm, long long n, int c, int col, int ncol, float *bs, long long bstride,
                    hipStream_t s, bool background)
{
    switch (ncol) {
    case 1: F3M_LAUNCH((gather_columns_kernel<1>), gather_grid(n, background), 256, 0, s, b, perm, n, c, col, bs, bstride); break;
    case 2: F3M_LAUNCH((gather_columns_kernel<2>), gather_grid(n, background), 256, 0, s, b, perm, n, c, col, bs, bstride); break;
    case 3: F3M_LAUNCH((gather_columns_kernel<3>), gather_grid(n, background), 256, 0, s, b, perm, n, c, col, bs, bstride); break;
    case 4: F3M_LAUNCH((gather_columns_kernel<4>), gather_grid(n, background), 256, 0, s, b, perm, n, c, col, bs, bstride); break;
    default: throw Error(34, "1 to 4 columns at a time");
    }
    check_launch("gather_columns");
}
void gather_column(const float *b, const int *perm, long long n, int c, int col, float *bs, hipStream_t s)
{
    gather_columns(b, perm, n, c, col, 1, bs, 0, s, false);
}

// out[perm[i]][col + q] = outs[q][i] (+ outs2[q][i] if outs2 is given: the far field's share when it was computed
// beside the near field), q < NC, one store of NC floats per row
template <int NC>
__global__ void scatter_columns_kernel(const float *__restrict__ outs, const float *__restrict__ outs2, long long ostride,
                                       const int *__restrict__ perm, long long n, int c, int col, float *__restrict__ out,
                                       SymSums sym)
{
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    fvec<NC> row;
#pragma unroll
    for (int q = 0; q < NC; q++) row.v[q] = outs[q * ostride + i] + (outs2 ? outs2[q * ostride + i] : 0.f);
    // the fixed-point sums come last: the far field's share is in outs already when everything ran on one stream, and
    // the bits must not depend on that
    if (NC == 1 && sym.fix != nullptr) {
        const float scale = sym_scale(sym.absmax[0], sym.nsrc);
        if (scale != 0.f) row.v[0] += (float)sym.fix[i] * (1.0f / scale);      // (a power of two: the two steps round once in all)
    }
    *reinterpret_cast<fvec<NC> *>(out + (long long)perm[i] * c + col) = row;
}
void scatter_columns(const float *outs, const float *outs2, long long ostride, const int *perm, long long n, int c, int col,
                     int ncol, float *out, hipStream_t s, const SymSums *symsums)
{
    const SymSums sym = symsums ? *symsums : SymSums();
    F3M_REQUIRE(sym.fix == nullptr || ncol == 1, 34, "fixed-point sums belong to a single column");
    switch (ncol) {
    case 1: F3M_LAUNCH((scatter_columns_kernel<1>), cdiv(n, 256), 256, 0, s, outs, outs2, ostride, perm, n, c, col, out, sym); break;
    case 2: F3M_LAUNCH((scatter_columns_kernel<2>), cdiv(n, 256), 256, 0, s, outs, outs2, ostride, perm, n, c, col, out, sym); break;
    case 3: F3M_LAUNCH((scatter_columns_kernel<3>), cdiv(n, 256), 256, 0, s, outs, outs2, ostride, perm, n, c, col, out, sym); break;
    case 4: F3M_LAUNCH((scatter_columns_kernel<4>), cdiv(n, 256), 256, 0, s, outs, outs2, ostride, perm, n, c, col, out, sym); break;
    default: throw Error(34, "1 to 4 columns at a time");
    }
    check_launch("scatter_columns");
}
// absmax[0] = max(absmax[0], bit pattern of the largest |bs[i]|): one atomic maximum per workgroup (the bit patterns of
// non-negative floats order like the floats, NaN above infinity)
__global__ void __launch_bounds__(256) absmax_kernel(const float *__restrict__ bs, long long n, unsigned *__restrict__ absmax)
{
    __shared__ unsigned wmax[4];
    unsigned m = 0;
    const long long n4 = n / 4, step = (long long)gridDim.x * blockDim.x;
    struct alignas(16) u4 { unsigned x, y, z, w; };
    const u4 *b4 = reinterpret_cast<const u4 *>(bs);                // (bs is the start of a device allocation)
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += step) {
        const u4 v = b4[i];
        m = max(max(m, v.x & 0x7fffffffu), max(max(v.y & 0x7fffffffu, v.z & 0x7fffffffu), v.w & 0x7fffffffu));
    }
    if (blockIdx.x == 0 && threadIdx.x < (unsigned)(n - 4 * n4))
        m = max(m, __builtin_bit_cast(unsigned, bs[4 * n4 + threadIdx.x]) & 0x7fffffffu);
    for (int off = 32; off > 0; off >>= 1) m = max(m, (unsigned)wave_shfl_i((int)m, (int)(lane_id() ^ (unsigned)off)));
    if ((threadIdx.x & 63) == 0) wmax[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) atomicMax(absmax, max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3])));
}
void sym_absmax(const float *bs, long long n, unsigned *absmax, hipStream_t s)
{
    dev_fill(absmax, 0, sizeof(unsigned), s);
    F3M_LAUNCH(absmax_kernel, (unsigned)std::min<long long>(cdiv(n, 4096), 1024), 256, 0, s, bs, n, absmax);
    check_launch("absmax");
}
void scatter_column(const float *outs, const int *perm, long long n, int c, int col, float *out, hipStream_t s)
{
    scatter_columns(outs, nullptr, 0, perm, n, c, col, 1, out, s);
}

// ------------------------------------------------------------------------------------------------
// exact dense product (F3M_src/1_d_conv.cu:171-214; gradient form :126-169): one target per lane,
// source tiles staged through LDS.

template <typename T> __device__ inline T kernel_exp(T negr2_scaled);
template <> __device__ inline float kernel_exp<float>(float v) { return fast_exp2(v); }   // v already times log2(e)
template <> __device__ inline double kernel_exp<double>(double v) { return exp(v); }

template <typename T, int D, bool GRAD>
__global__ void __launch_bounds__(256) exact_kernel(const T *__restrict__ X, long long N, const T *__restrict__ Y, long long M,
                                                     const T *__restrict__ b, int c, int col, T scale, T post,
                                                     T *__restrict__ out)
{
    __shared__ T sy[D][256];
    __shared__ T sb[256];
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    T x[D];
#pragma unroll
    for (int k = 0; k < D; k++) x[k] = (i < N) ? X[i * D + k] : (T)0;
    T acc = 0;
    for (long long j0 = 0; j0 < M; j0 += 256) {
        long long j = j0 + threadIdx.x;
        __syncthreads();
        if (j < M) {
#pragma unroll
            for (int k = 0; k < D; k++) sy[k][threadIdx.x] = Y[j * D + k];
            sb[threadIdx.x] = b[j * c + col];
        }
        __syncthreads();
        int cnt = (int)((M - j0) < 256 ? (M - j0) : 256);
        for (int jj = 0; jj < cnt; jj++) {
            T r2 = 0;
#pragma unroll
            for (int k = 0; k < D; k++) { T t = x[k] - sy[k][jj]; r2 += t * t; }
            T e = kernel_exp<T>(-r2 * scale);
            if (GRAD) e *= r2;
            acc += e * sb[jj];
        }
    }
    if (i < N) out[i * c + col] = GRAD ? acc * post : acc;
}

template <typename T, bool GRAD>
static void exact_dispatch(int d, const T *X, long long N, const T *Y, long long M, const T *b, int c, T scale, T post,
                           T *out, hipStream_t s)
{
    unsigned grid = cdiv(N, 256);
    for (int col = 0; col < c; col++) {
#define F3M_CASE(DD)                                                                                               \
    case DD:                                                                                                       \
        F3M_LAUNCH((exact_kernel<T, DD, GRAD>), grid, 256, 0, s, X, N, Y, M, b, c, col, scale, post, out);         \
        break;
        switch (d) {
            F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
            F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
        default: throw Error(2, "dimension must be 1..10");
        }
#undef F3M_CASE
        check_launch("exact");
    }
}

void exact_f32(int d, const float *X, long long N, const float *Y, long long M, const float *b, int c, float ls, bool grad,
               float *out, hipStream_t s)
{
    if (N == 0) return;
    float lcs = 1 / (2 * ls * ls);              // F3M_src/n_tree.cu:194
    float post = 1 / (ls * ls * ls);            // F3M_src/n_tree.cu:223
    if (grad) exact_dispatch<float, true>(d, X, N, Y, M, b, c, lcs * kLog2e, post, out, s);
    else exact_dispatch<float, false>(d, X, N, Y, M, b, c, lcs * kLog2e, post, out, s);
}

void exact_f64(int d, const double *X, long long N, const double *Y, long long M, const double *b, int c, double ls,
               double *out, hipStream_t s)
{
    if (N == 0) return;
    double lcs = 1 / (2 * ls * ls);
    exact_dispatch<double, false>(d, X, N, Y, M, b, c, lcs, 1.0, out, s);
}

// ------------------------------------------------------------------------------------------------
// tiles: work items (box, tile of `tile` consecutive points) for the boxes with flag != 0

// order (nullable): slot k of the tile offsets stands for box order[k]
// rowptr (nullable, instead of flag): the boxes with a row in that list
__global__ void tiles_per_box_kernel(const int *__restrict__ off, const int *__restrict__ flag, int nb, int tile,
                                     const int *__restrict__ order, int *__restrict__ ntiles,
                                     const int *__restrict__ rowptr)
{
    int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= nb) return;
    const int b = order ? order[k] : k;
    int cnt = off[b + 1] - off[b];
    const bool live = rowptr != nullptr ? rowptr[b + 1] > rowptr[b] : (flag == nullptr || flag[b]);
    ntiles[k] = live ? (cnt + tile - 1) / tile : 0;
}

// Boxes ordered by the length of their list rows, longest first, in 256 classes of `unit` pairs (one
// counting pass; the order inside a class is whatever the atomics give, which does not touch results).
__global__ void row_class_count_kernel(const int *__restrict__ rowptr, int nb, int unit, int *__restrict__ cls,
                                       int *__restrict__ hist)
{
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nb) return;
    const int c = 255 - min(255, (rowptr[b + 1] - rowptr[b]) / unit);
    cls[b] = c;
    atomicAdd(&hist[c], 1);
}
__global__ void class_place_kernel(const int *__restrict__ cls, int n, const int *__restrict__ hist, int *__restrict__ order)
{
    __shared__ int start[256];
    if (threadIdx.x == 0) {                          // 256 classes: a serial scan is enough
        int run = 0;
        for (int c = 0; c < 256; c++) { start[c] = run; run += hist[c]; }
    }
    __syncthreads();
    for (int p = threadIdx.x; p < n; p += blockDim.x) order[atomicAdd(&start[cls[p]], 1)] = p;   // one workgroup: cursors in LDS
}

__global__ void mark_rows_kernel(const int *__restrict__ rowptr, int nb, int *__restrict__ flag)
{
    int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b < nb) flag[b] = rowptr[b + 1] > rowptr[b] ? 1 : 0;
}

__global__ void mark_cols_kernel(const int *__restrict__ pairs, long long n, int *__restrict__ flag)
{
    long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < n) flag[pairs[2 * t + 1]] = 1;
}

// tileoff (nb+1) = exclusive scan of tiles per box.  Returns an upper bound of the number of tiles
// (nb + npoints/tile) to launch with; workgroups past tileoff[nb] exit at once, so the host never
// waits for the exact count.
static int build_tiles(const int *off, const int *flag, int nb, long long npoints, int tile, DBuf<int> &tileoff, hipStream_t s,
                       const int *order = nullptr, const int *rowptr = nullptr)
{
    DBuf<int> nt((size_t)nb);
    tileoff.reset((size_t)nb + 1);
    F3M_LAUNCH(tiles_per_box_kernel, cdiv(nb, 256), 256, 0, s, off, flag, nb, tile, order, nt.get(), rowptr);
    check_launch("tiles_per_box");
    exclusive_scan_i32(nt.get(), nb, tileoff.get(), s);
    long long bound = (long long)nb + npoints / tile;
    F3M_REQUIRE(bound < (1ll << 31) - 1, 32, "too many work items");
    return (int)bound;
}

__device__ inline int find_box(const int *__restrict__ tileoff, int nb, int tileid)
{
    int lo = 0, hi = nb;   // last b with tileoff[b] <= tileid
    while (hi - lo > 1) {
        int mid = lo + ((hi - lo) >> 1);
        if (tileoff[mid] <= tileid) lo = mid; else hi = mid;
    }
    return lo;
}

// box32[k] = box of point 32 k (the last box for k past the end).  A workgroup that owns a fixed-size
// piece of the points would otherwise open with a binary search over the offsets, some 17 dependent
// loads that take longer than the piece's own work.
__global__ void box_table_kernel(const int *__restrict__ off, int nb, long long npoints, int nent, int *__restrict__ box32)
{
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= nent) return;
    const long long p = min((long long)k * 32, npoints - 1);
    box32[k] = find_box(off, nb, (int)max(0ll, p));
}

static const int *box_table(const TreeLevel &lev, long long npoints, hipStream_t s)
{
    const int nent = (int)(npoints / 32) + 2;
    if (lev.box32.size() != (size_t)nent) {
        require_tables_may_be_built("the box table of a level");
        lev.box32.reset((size_t)nent);
        F3M_LAUNCH(box_table_kernel, cdiv(nent, 256), 256, 0, s, lev.off.get(), lev.nb, npoints, nent, lev.box32.get());
        check_launch("box_table");
    }
    return lev.box32.get();
}

void ensure_box_table(const TreeLevel &lev, long long npoints, hipStream_t s) { (void)box_table(lev, npoints, s); }

// ------------------------------------------------------------------------------------------------
// near field (F3M_src/1_d_conv.cu:255-335): out_i += sum over the y boxes listed for the box of i of
// sum_j exp(-|x_i-y_j|^2 lcs) b_j.  All-vector form: one workgroup per (x box, tile of targets); the
// sources of a y box are staged through LDS already shifted to the x box centre and scaled by
// sqrt(lcs*log2 e), together with their weights, and a pair costs D subtractions, D multiply-adds, one
// exp2 and one multiply-add:  exp2(-|x' - y'|^2) b.  The exponent is formed from the coordinate
// differences (not from 2x'.y' - |y'|^2 - |x'|^2, whose cancellation costs about 2^-24 (|x'|^2 + |y'|^2)):
// this is the kernel for boxes that are large against the lengthscale, where those squares reach
// hundreds.

constexpr int kNearCap = 512;   // sources per LDS tile

template <int D, int T>
__global__ void __launch_bounds__(512) near_kernel(const float *__restrict__ xs, long long N, const float *__restrict__ ys,
                                                    long long M, const float *__restrict__ bs, float *__restrict__ outs,
                                                    const int *__restrict__ offx, const int *__restrict__ offy,
                                                    const float *__restrict__ ctrx, const int *__restrict__ pairs,
                                                    const int *__restrict__ rowptr, const int *__restrict__ tileoff,
                                                    int nbx, float sc)
{
    constexpr int NV = (D + 1 + 3) / 4;             // float4 slots per source: D coordinates and the weight
    __shared__ float4 sv[NV][kNearCap];
    const int tid = threadIdx.x, BD = blockDim.x;
    if ((int)blockIdx.x >= tileoff[nbx]) return;    // launched with an upper bound of the tile count
    const int bx = find_box(tileoff, nbx, blockIdx.x);
    const int tile = blockIdx.x - tileoff[bx];
    const int x0 = offx[bx] + tile * BD * T, x1 = offx[bx + 1];
    float cx[D];
#pragma unroll
    for (int k = 0; k < D; k++) cx[k] = ctrx[(long long)bx * D + k];
    float x[T][D], acc[T];
#pragma unroll
    for (int r = 0; r < T; r++) {
        int i = x0 + r * BD + tid;
        acc[r] = 0.f;
#pragma unroll
        for (int k = 0; k < D; k++) {
            float v = (i < x1) ? xs[(long long)k * N + i] : cx[k];
            x[r][k] = sc * (v - cx[k]);
        }
    }
    // a wavefront whose lanes all lie past the end of the box only helps with staging
    const bool wave_live = x0 + (tid & ~(kWave - 1)) < x1;
    const int m0 = rowptr[bx], m1 = rowptr[bx + 1];
    for (int m = m0; m < m1; m++) {
        const int by = pairs[2 * (long long)m + 1];
        const int s0 = offy[by], s1 = offy[by + 1];
        for (int base = s0; base < s1; base += kNearCap) {
            const int cnt = (s1 - base) < kNearCap ? (s1 - base) : kNearCap;
            __syncthreads();
            for (int jj = tid; jj < cnt; jj += BD) {
                float v[NV * 4];
#pragma unroll
                for (int k = 0; k < D; k++) v[k] = sc * (ys[(long long)k * M + base + jj] - cx[k]);
                v[D] = bs[base + jj];
#pragma unroll
                for (int k = D + 1; k < NV * 4; k++) v[k] = 0.f;
#pragma unroll
                for (int q = 0; q < NV; q++) sv[q][jj] = make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
            }
            __syncthreads();
            if (!wave_live) continue;
#pragma unroll 4
            for (int jj = 0; jj < cnt; jj++) {
                float v[NV * 4];
#pragma unroll
                for (int q = 0; q < NV; q++) {
                    float4 f = sv[q][jj];
                    v[4 * q] = f.x; v[4 * q + 1] = f.y; v[4 * q + 2] = f.z; v[4 * q + 3] = f.w;
                }
#pragma unroll
                for (int r = 0; r < T; r++) {
                    float r2 = 0.f;
#pragma unroll
                    for (int k = 0; k < D; k++) { const float df = x[r][k] - v[k]; r2 = fmaf(df, df, r2); }
                    acc[r] = fmaf(fast_exp2(-r2), v[D], acc[r]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < T; r++) {
        int i = x0 + r * BD + tid;
        if (i < x1) outs[i] += acc[r];
    }
}

// Near field with the exponent on the matrix pipe.  The exponent of a pair,
//   t = 2x''.y' - |y'|^2 - |x''|^2   (x'', y' shifted to an anchor near the sources and scaled by sqrt(lcs log2 e)),
// is an inner product over the components (2y'_k, -|y'|^2, 1) . (x''_k, 1, -|x''|^2).
// Every fp32 operand is split into two f16 values, v = hi + lo (|v - hi - lo| <= 2^-22 |v|), and the
// products hi.hi + hi.lo + lo.hi of all components fill the inner slots of one
// v_mfma_f32_32x32x16_f16 (two instructions for D >= 5), accumulated in fp32 from zero.
// The f16 matrix pipe runs beside the vector ALU, which is left with one exp2 and one fused
// multiply-add per pair.  near_operands_kernel prepares the source side once per tree level,
// near_g_kernel streams it against the targets of a wavefront.
// Valid while |x''|, |y'| stay small enough for the split (the host checks the box size against the
// lengthscale and otherwise launches near_kernel).

// Inner slots of the matrix product.  Coordinate k takes slots 3k..3k+2: hi.hi, (source hi).(target lo),
// (source lo).(target hi).  The two scalars need two slots each, because their partner is exactly 1:
// slots 3D, 3D+1 = (hi, lo of the source's -|y'|^2) . 1 and slots 3D+2, 3D+3 = 1 . (hi, lo of the
// target's -|x''|^2).  3D+4 slots in all: one instruction of 16 up to D = 4.
// hi/lo hold C = D+2 values: the coordinates, then on the source side (-|y'|^2, 1), on the target side (1, -|x''|^2).
//
// Factored form (FACT): only the coordinates go through the matrix product, u = 2x''.y' in 3D slots, and
//   exp2(t) b = exp2(-|x''|^2) . exp2(u) . (exp2(-|y'|^2) b):
// the source factor rides on the weight (one multiplication per source and product, near_weights_kernel), the target
// factor multiplies the sum over a run of sources once.  It takes one instruction where 3D+4 slots take two
// (D = 5: 15 against 19 slots), at the price of exponentials whose arguments no longer cancel: |u| <= 10 D S^2 with
// S = (box edge) sqrt(lcs log2 e), so the host takes the form only while that stays far from the exponent range
// (near_factored).
__host__ __device__ constexpr int near_slots(int D, bool fact = false) { return fact ? 3 * D : 3 * D + 4; }
__host__ __device__ constexpr int near_insts(int D, bool fact = false) { return (near_slots(D, fact) + 15) / 16; }
// dimensions whose factored form saves an instruction (the others never take it)
__host__ __device__ constexpr bool near_fact_pays(int D) { return near_insts(D, true) < near_insts(D, false); }
template <int D, bool FACT = false>
__device__ inline h8 split_operand(const half_t *hi, const half_t *lo, int n, int hh, bool source)
{
    h8 v;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const int slot = 16 * n + 8 * hh + e;
        if (slot < 3 * D) {
            const int c = slot / 3, tau = slot % 3;
            v[e] = source ? (tau == 2 ? lo[c] : hi[c]) : (tau == 1 ? lo[c] : hi[c]);
        } else if (slot < near_slots(D, FACT)) {
            const int sl = slot - 3 * D;
            if (source) v[e] = sl == 0 ? hi[D] : (sl == 1 ? lo[D] : hi[D + 1]);
            else v[e] = sl < 2 ? hi[D] : (sl == 2 ? hi[D + 1] : lo[D + 1]);
        } else {
            v[e] = to_half(0.f);
        }
    }
    return v;
}

// Source operands, once per tree level: point i of box b, shifted to the centre of b's parent cell
// (near_anchor; shared by the boxes of that parent, which lets near_g_kernel take neighbouring boxes
// in one go) and scaled, as the rows (2y', -|y'|^2) of the matrix product in split-f16 form.  Layout: ops[(n*2 + h)*stride + i]
// = the eight inner slots of half-wave h of instruction n; stride = npoints + 32 (the tail is zero so
// that a wavefront may read one padded tile past the end).
// need (nullable) = prefix count of the boxes that occur as sources (nb+1 entries): operands are then
// written only for the points of those boxes and for the 31 points after them, which a wavefront may
// read as the padding of a box's last tile.
constexpr int kOpsBlock = 256;

// Reference point of the near-field operands of a box: the centre of its parent cell, computed from
// the integer cell so that every box of the parent (and both kernels) get the same bits.
__device__ __forceinline__ float near_anchor(const Geo &geo, float edge, int cell, int k)
{
    return geo.origin[k] + (float)(2 * (cell >> 1) + 1) * edge;
}

// FACT: the operands of the factored form, and ey[i] = exp2(-|y'_i|^2) (stride floats, zero past the end).
template <int D, bool FACT>
__global__ void __launch_bounds__(kOpsBlock) near_operands_kernel(const float *__restrict__ ys, long long M,
                                                                  const int *__restrict__ off, int nb,
                                                                  const int *__restrict__ cell, Geo geo, float edge,
                                                                  float sc, long long stride,
                                                                  const int *__restrict__ need, const int *__restrict__ box32,
                                                                  h8 *__restrict__ ops, float *__restrict__ ey)
{
    constexpr int C = D + 2;                        // coordinates, -|y'|^2, and a 1 that carries the target's -|x''|^2
    constexpr int NS = near_insts(D, FACT);
    __shared__ int bounds[kOpsBlock];
    const int tid = threadIdx.x;
    const long long i0 = (long long)blockIdx.x * kOpsBlock, i = i0 + tid;
    // boxes of the first point of this workgroup and of the point 31 before it (uniform)
    const long long pm = max(0ll, min(i0, M - 1) - 31);
    int b0 = box32[min(i0, M - 1) / 32], b0m = box32[pm / 32];
    while (off[b0 + 1] <= min(i0, M - 1)) b0++;      // at most the boxes that start inside 32 points
    while (off[b0m + 1] <= pm) b0m++;
    if (need != nullptr) {
        // no box between the one 31 points before this workgroup's first point and the one of its last point is
        // wanted: nothing to do (a list of a shallow level names a few boxes, the launch covers every point)
        const long long il = min(i0 + kOpsBlock - 1, M - 1);
        int bl = box32[il / 32];
        while (off[bl + 1] <= il) bl++;
        if (need[bl + 1] - need[b0m] == 0) return;
    }
    bounds[tid] = off[min(b0 + 1 + tid, nb)];       // starts of the following boxes; off[nb] = M closes the list
    __syncthreads();
    if (i >= stride) return;
    half_t hi[C], lo[C];
    float ny2 = 0.f;
    if (i < M) {
        auto box_of = [&](long long p) {            // p >= i0: number of box starts <= p among the following boxes
            int a = 0, b = kOpsBlock;
            while (a < b) {
                int mid = (a + b) >> 1;
                if (bounds[mid] <= p) a = mid + 1; else b = mid;
            }
            return b0 + a;
        };
        const int box = box_of(i);
        if (need != nullptr) {
            const int first = (i - 31 >= i0) ? box_of(i - 31) : b0m;
            if (need[box + 1] - need[first] == 0) return;
        }
#pragma unroll
        for (int k = 0; k < C; k++) {
            float v;
            if (k < D) {
                float y = sc * (ys[(long long)k * M + i] - near_anchor(geo, edge, cell[(long long)box * D + k], k));
                ny2 -= y * y;
                v = 2.f * y;
            } else if (k == D) {
                v = ny2;
            } else {
                v = 1.f;
            }
            hi[k] = to_half(v);
            lo[k] = to_half(v - half_to_float(hi[k]));
        }
    } else {
#pragma unroll
        for (int k = 0; k < C; k++) { hi[k] = to_half(0.f); lo[k] = to_half(0.f); }
    }
#pragma unroll
    for (int n = 0; n < NS; n++) {
        ops[(long long)(n * 2 + 0) * stride + i] = split_operand<D, FACT>(hi, lo, n, 0, true);
        ops[(long long)(n * 2 + 1) * stride + i] = split_operand<D, FACT>(hi, lo, n, 1, true);
    }
    if (FACT) ey[i] = i < M ? fast_exp2(ny2) : 0.f;
}

// weights of the factored form: ws[c][j] = bs[c][j] exp2(-|y'_j|^2), the padding tile included; columns of bs are
// bstride apart, those of ws stride
__global__ void near_weights_kernel(const float *__restrict__ bs, const float *__restrict__ ey, long long stride, int nc,
                                    long long bstride, float *__restrict__ ws)
{
    const long long j = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= stride) return;
    const float e = ey[j];
    for (int c = 0; c < nc; c++) ws[c * stride + j] = bs[c * bstride + j] * e;
}

// Near field, matrix-pipe form.  One wavefront per TPW*32 targets of an x box (TPW tiles of 32; lanes
// l and l+32 hold the same target and different source rows).  For every run of listed y boxes (boxes
// that follow each other in memory under one parent cell) the targets are re-expressed relative to
// the run's anchor, the centre of that parent cell (x'' = sc (x - anchor)), and split into f16 pairs;
// the per-target constant -|x''|^2 rides in two inner slots (against a source-side 1), so the
// accumulator starts from zero.  The source operands come ready-made from near_operands_kernel and
// are streamed from global memory / L2 in 32-source tiles, together with their weights.  No LDS and
// no barriers: wavefronts are independent.  Rows past the end of a box are neutralised by a zero
// weight (the exponent of any two vectors is -|x''-y'|^2 <= 0, so exp2 stays finite).
constexpr int kNearWavesPerBlock = 2;
// value of sorted point i, column q of the pass, added into the caller's array (see DirectOut)
__device__ __forceinline__ void direct_add(const DirectOut &dout, long long i, int q, float value)
{
    float *p = dout.out + (long long)dout.perm[i] * dout.c + dout.col + q;
#ifdef F3M_CPU_EMU
    *p += value;
#else
    unsafeAtomicAdd(p, value);          // one hardware instruction (no compare-and-swap loop); out is ordinary device memory
#endif
}
struct __attribute__((aligned(4))) float4u { float x, y, z, w; };   // four floats at any 4-byte boundary

// NC right-hand sides at once: the exponential of a pair is computed once and multiplies NC weights
// (columns of bs, bstride apart; results to NC columns of outs, ostride apart).
// FACT: the factored form (see near_slots): bs then holds the weights times exp2(-|y'|^2).
//
// SYM (one tree, X = Y: the list names (A,B) exactly when it names (B,A), and K is symmetric): a wavefront of box A takes
// only the listed boxes B >= A.  The exponentials of a tile of B > A serve both directions: weighted with the sources'
// weights they are summed over the rows into the targets of A as always, and weighted with the targets' weights they are
// summed over the columns into the sources of B -- 16 more accumulators per lane, kept over the target tiles of the
// work item, then added up across the 32 columns through the wavefront's own LDS block and added to the sums of B
// atomically, as fixed-point numbers (SymSums): integer additions give the same result in any order.  Half the
// exponentials per listed pair of points.  With FACT the second direction carries the targets' factor exp2(-|x''|^2) in
// its weights (set up per anchor) and receives the sources' factor exp2(-|y'|^2) after the sum over the columns.
constexpr int kSymRedStride = 33;                  // floats per row of the reduction block (32 columns + 1: no bank conflicts)
__device__ __forceinline__ void atomic_add_i64(long long *p, long long v)
{
#ifdef F3M_CPU_EMU
    *p += v;
#else
    atomicAdd(reinterpret_cast<unsigned long long *>(p), (unsigned long long)v);
#endif
}
__device__ __forceinline__ void atomic_add_f32(float *p, float v)
{
#ifdef F3M_CPU_EMU
    *p += v;
#else
    unsafeAtomicAdd(p, v);
#endif
}
// (The symmetric form is held to 120 registers: four wavefronts per SIMD then leave 32 of its 512 free, as five of the
// plain form's 96 do, and the small workgroups of the far field find room beside a running near field; at 128 they
// wait for its end.)
template <int D, int TPW, int NC, bool FACT, bool SYM, int WPB = kNearWavesPerBlock>
__device__ __forceinline__ void near_g_body(
    const float *__restrict__ xs, long long N, const h8 *__restrict__ ops, long long stride, const float *__restrict__ bs,
    long long bstride, float *__restrict__ outs, long long ostride, const int *__restrict__ offx,
    const int *__restrict__ offy, const int *__restrict__ celly, const Geo &geoy, float edgey,
    const int *__restrict__ pairs, const int *__restrict__ rowptr, const int *__restrict__ tileoff, int nbx, float sc,
    int stripe, int nsplit, float *__restrict__ part, int nitems, const int *__restrict__ order, const DirectOut &dout,
    const SymSums &symsums)
{
    constexpr int C = D + 2;                        // coordinates, the source's -|y'|^2, the target's -|x''|^2
    constexpr int NS = near_insts(D, FACT);
    const int lane = threadIdx.x & 63, half = lane >> 5, col = lane & 31;
    // Workgroups are handed to the 8 XCDs round-robin.  Work items are in Morton order of their x box
    // and neighbouring boxes share their source boxes, so the work items are cut into stripes of
    // `stripe` consecutive workgroups and each stripe runs on one XCD: its L2 then serves the re-reads
    // of the sources.  (gridDim.x is a multiple of 8*stripe.)
    int vblock;
    if (stripe <= 0) vblock = blockIdx.x;
    else {
        const int r = blockIdx.x >> 3, xcd = blockIdx.x & 7;
        vblock = (r / stripe) * (8 * stripe) + xcd * stripe + (r % stripe);
    }
    // work item: TPW*32 targets of one box; with few targets and long lists (nsplit > 1) the list of a
    // work item is cut into nsplit slices, one wavefront each, whose sums go to `part` (nsplit x NC x
    // nitems x TPW*32 floats, indexed by work item) and are added up in a fixed order afterwards
    const int wfull = vblock * WPB + (threadIdx.x >> 6);
    const int wid = wfull / nsplit, slice = wfull % nsplit;
    if (wid >= tileoff[nbx]) return;
    const int slot = find_box(tileoff, nbx, wid);
    const int bx = order ? order[slot] : slot;       // order (nullable): boxes with the longest lists first
    const int x0 = offx[bx] + (wid - tileoff[slot]) * (TPW * 32), x1 = offx[bx + 1];
    int nlive = (x1 - x0 + 31) / 32;                 // tiles with targets (uniform per wavefront)
    if (nlive > TPW) nlive = TPW;
    float xr[SYM ? 1 : TPW][D];                      // (SYM: read again at every new anchor, the registers are needed elsewhere)
    if constexpr (!SYM) {
#pragma unroll
        for (int q = 0; q < TPW; q++) {
            const int i = x0 + q * 32 + col;
#pragma unroll
            for (int k = 0; k < D; k++) xr[q][k] = (i < x1) ? xs[(long long)k * N + i] : 0.f;
        }
    }
    float acc[TPW][NC];
#pragma unroll
    for (int q = 0; q < TPW; q++)
#pragma unroll
        for (int c = 0; c < NC; c++) acc[q][c] = 0.f;
    static_assert(!SYM || NC == 1, "the symmetric form takes one column");
    // SYM: the wavefront's LDS block: 32 rows of the column reduction, then the weights of its targets (one tree: sources
    // and targets are the same points in the same order), kept there to spare registers
    // (factored form: a second copy, the weights times the targets' factor exp2(-|x''|^2) of the current anchor)
    constexpr int kSymBlock = 32 * kSymRedStride + TPW * 32 * (FACT ? 2 : 1);
    __shared__ float red_all[SYM ? WPB * kSymBlock : 1];
    float *const red = red_all + (SYM ? (threadIdx.x >> 6) * kSymBlock : 0);
    float *const btl = red + 32 * kSymRedStride;
    float *const wtl = FACT ? btl + TPW * 32 : btl;
    float fixscale = 0.f;                            // SYM: scale of the fixed-point sums (0: weights not finite)
    if constexpr (SYM) {
#pragma unroll
        for (int q = 0; q < TPW; q++) {
            const int i = x0 + q * 32 + col;
            if (half == 0) btl[q * 32 + col] = i < x1 ? (FACT ? symsums.braw[i] : bs[i]) : 0.f;
        }
        wave_sync();
        fixscale = sym_scale(symsums.absmax[0], symsums.nsrc);
    }
    const int m0 = rowptr[bx], m1 = rowptr[bx + 1];
    // slice of this wavefront, in 32-source tiles counted along the whole row: [tlo, thi)
    int tlo = 0, thi = 0x7fffffff;
    if (nsplit > 1) {
        int ttot = 0;
        for (int mb = m0; mb < m1; mb += 64) {
            int nt = 0;
            if (mb + lane < m1) {
                const int byv = pairs[2 * (long long)(mb + lane) + 1];
                nt = (offy[byv + 1] - offy[byv] + 31) >> 5;
            }
            for (int off = 32; off > 0; off >>= 1) nt += wave_shfl_i(nt, lane ^ off);
            ttot += nt;
        }
        tlo = (int)((long long)ttot * slice / nsplit);
        thi = (int)((long long)ttot * (slice + 1) / nsplit);
    }
    int tcur = 0;                                    // tiles of the row before the current y box
    h8 bop[TPW][NS];                                 // target operands of the current anchor
    float ex[TPW];                                   // factored form: exp2(-|x''|^2)
#pragma unroll
    for (int q = 0; q < TPW; q++) {
        ex[q] = 0.f;
#pragma unroll
        for (int n = 0; n < NS; n++)
#pragma unroll
            for (int e = 0; e < 8; e++) bop[q][n][e] = to_half(0.f);
    }
    // The list is consumed 64 y boxes at a time: every lane fetches the range and the anchor of one y
    // box, then the wavefront walks through them (one round of memory latency per 64 boxes).  Boxes
    // that follow each other in the list, in memory and under one parent share their anchor and are
    // taken as one run of sources: one set of target operands and one padded last tile per run.
    for (int mb = m0; mb < m1; mb += 64) {
      const int mi = mb + lane;
      int s0v = 0, s1v = 0, byv = -2;
      int pcv[D];
      float cyv[D];
#pragma unroll
      for (int k = 0; k < D; k++) { cyv[k] = 0.f; pcv[k] = 0; }
      if (mi < m1) {
          byv = pairs[2 * (long long)mi + 1];
          s0v = offy[byv];
          s1v = offy[byv + 1];
#pragma unroll
          for (int k = 0; k < D; k++) {
              const int cl = celly[(long long)byv * D + k];
              pcv[k] = cl >> 1;
              if constexpr (!SYM) cyv[k] = near_anchor(geoy, edgey, cl, k);   // (SYM reads the cell again at a new anchor: registers)
          }
      }
      // SYM: boxes before this one are left to their own wavefronts (each stays in the walk as a run without sources)
      const bool mine = !SYM || byv >= bx;
      if (SYM && !mine) { s0v = 0; s1v = 0; }
      const int mcnt = min(64, m1 - mb);
      // same: under the parent cell of the lane before (same anchor, the target operands stay as they are);
      // cont: also next to it in memory, i.e. continues its run
      // (sliced lists keep one box per run: slices count tiles per box)
      const int before = (lane + 63) & 63;
      bool same = lane > 0 && mi < m1 && nsplit == 1;
#pragma unroll
      for (int k = 0; k < D; k++) same = (wave_shfl_i(pcv[k], before) == pcv[k]) && same;
      const int byprev = wave_shfl_i(byv, before);   // by every lane: an exchange inside a branch sees the branch's lanes only
      if (SYM) same = same && mine && byprev >= bx;  // the operands of a skipped box were never set up
      // (SYM: the box itself is a run of its own, it takes one direction only)
      const bool cont = same && byprev + 1 == byv && !(SYM && (byprev == bx || byv == bx));
      unsigned long long heads = wave_ballot(mi < m1 && !cont);
      const unsigned long long anchors = wave_ballot(mi < m1 && !same);
      while (heads) {
        const int mj = __builtin_ctzll(heads);
        const bool new_anchor = (anchors >> mj) & 1;   // uniform
        heads &= heads - 1;
        const int mlast = heads ? __builtin_ctzll(heads) - 1 : mcnt - 1;
        int s0 = wave_readlane(s0v, mj), s1 = wave_readlane(s1v, mlast);
        if (nsplit > 1) {                            // keep the part of this box that lies in the slice
            const int nt = (s1 - s0 + 31) >> 5;
            const int a = max(tlo, tcur), b = min(thi, tcur + nt);
            const int first = s0 + 32 * (a - tcur);
            if (b < tcur + nt) s1 = s0 + 32 * (b - tcur);
            s0 = first;
            tcur += nt;
            if (a >= b) continue;                    // uniform
        }
        // (both are the same in every lane, which the compiler cannot see through the slicing above: as scalars they
        // keep the loop over the tiles of the run off the vector ALU)
        s0 = wave_uniform(s0);
        s1 = wave_uniform(s1);
        const int byhead = SYM ? wave_readlane(byv, mj) : 0;
        if (SYM && byhead < bx) continue;            // a skipped box (uniform)
        const bool both = SYM && byhead != bx;       // uniform: the tiles of this run serve both directions
        float run[TPW][NC];                           // factored form: the sums of this run
#pragma unroll
        for (int q = 0; q < TPW; q++)
#pragma unroll
            for (int c = 0; c < NC; c++) run[q][c] = 0.f;
        // target operands relative to the anchor of this run; runs under one parent cell follow each other in the
        // list and share them
        if (new_anchor) {
        float cy[D];
#pragma unroll
        for (int k = 0; k < D; k++) {
            if constexpr (SYM) cy[k] = near_anchor(geoy, edgey, celly[(long long)byhead * D + k], k);
            else cy[k] = __builtin_bit_cast(float, wave_readlane(__builtin_bit_cast(int, cyv[k]), mj));
        }
#pragma unroll
        for (int q = 0; q < TPW; q++) {
            if (q >= nlive) continue;                 // uniform per wavefront: tiles without targets need no operands
            const bool ok = x0 + q * 32 + col < x1;
            half_t hi[C], lo[C];
            float nx2 = 0.f;
#pragma unroll
            for (int k = 0; k < C; k++) {
                float v = 1.f;
                if (k < D) {
                    float xv;
                    if constexpr (SYM) xv = ok ? xs[(long long)k * N + x0 + q * 32 + col] : 0.f;
                    else xv = xr[q][k];
                    v = ok ? sc * (xv - cy[k]) : 0.f;
                    nx2 -= v * v;
                } else if (k == D + 1) {
                    v = nx2;
                }
                hi[k] = to_half(v);
                lo[k] = to_half(v - half_to_float(hi[k]));
            }
#pragma unroll
            for (int n = 0; n < NS; n++) {
                h8 v0 = split_operand<D, FACT>(hi, lo, n, 0, false), v1 = split_operand<D, FACT>(hi, lo, n, 1, false);
                bop[q][n] = half ? v1 : v0;
            }
            if (FACT) ex[q] = fast_exp2(nx2);
            if constexpr (SYM && FACT) {
                if (half == 0) wtl[q * 32 + col] = ex[q] * btl[q * 32 + col];
            }
        }
        if constexpr (SYM && FACT) wave_sync();
        }
        for (int j0 = s0; j0 < s1; j0 += 32) {
            h8 a[NS];
#pragma unroll
            for (int n = 0; n < NS; n++) a[n] = ops[(long long)(n * 2 + half) * stride + j0 + col];
            // weights of the 16 source rows this lane sees: rows 8g + 4 half + e of the tile (bs is
            // padded by one tile, so the loads stay in bounds; rows past the box get weight zero)
            float bq[NC][16];
#pragma unroll
            for (int c = 0; c < NC; c++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const float4u f = *reinterpret_cast<const float4u *>(bs + c * bstride + j0 + 8 * g + 4 * half);
                    bq[c][4 * g + 0] = f.x; bq[c][4 * g + 1] = f.y; bq[c][4 * g + 2] = f.z; bq[c][4 * g + 3] = f.w;
                }
            if (j0 + 32 > s1) {
                const int lim = s1 - j0 - 4 * half;      // rows of this lane's half of the tile that are left in the box
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const bool in = 8 * (r / 4) + (r % 4) < lim;
#pragma unroll
                    for (int c = 0; c < NC; c++) bq[c][r] = in ? bq[c][r] : 0.f;
                }
            }
            auto tile = [&](int q) {
                f32x16 t;
#pragma unroll
                for (int r = 0; r < 16; r++) t[r] = 0.f;
#pragma unroll
                for (int n = 0; n < NS; n++) t = mfma_32x32x16_f16(a[n], bop[q][n], t);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float e = fast_exp2(t[r]);
#pragma unroll
                    for (int c = 0; c < NC; c++) {
                        if (FACT) run[q][c] = fmaf(e, bq[c][r], run[q][c]);
                        else acc[q][c] = fmaf(e, bq[c][r], acc[q][c]);
                    }
                }
            };
            if (both) {
                if constexpr (SYM) {
                    float sacc[16];                  // sums over this lane's column of every target tile, per source row
#pragma unroll
                    for (int r = 0; r < 16; r++) sacc[r] = 0.f;
                    auto tile2 = [&](int q) {
                        const float btq = wtl[q * 32 + col];
                        f32x16 t;
#pragma unroll
                        for (int r = 0; r < 16; r++) t[r] = 0.f;
#pragma unroll
                        for (int n = 0; n < NS; n++) t = mfma_32x32x16_f16(a[n], bop[q][n], t);
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const float e = fast_exp2(t[r]);
                            if (FACT) run[q][0] = fmaf(e, bq[0][r], run[q][0]);
                            else acc[q][0] = fmaf(e, bq[0][r], acc[q][0]);
                            sacc[r] = fmaf(e, btq, sacc[r]);
                        }
                    };
                    if (nlive == TPW) {              // the usual case, free of branches (see below)
#pragma unroll
                        for (int q = 0; q < TPW; q++) tile2(q);
                    } else {
#pragma unroll
                        for (int q = 0; q < TPW; q++)
                            if (q < nlive) tile2(q);     // uniform per wavefront
                    }
                    // across the 32 columns: element r of half h is source row 8(r/4) + 4h + r%4 of the tile
#pragma unroll
                    for (int r = 0; r < 16; r++) red[(half * 16 + r) * kSymRedStride + col] = sacc[r];
                    wave_sync();
                    const int rho = ((col >> 2) & 1) * 16 + 4 * (col >> 3) + (col & 3);   // where source row `col` sits
                    float sum = 0.f;
#pragma unroll
                    for (int k = 0; k < 16; k++) sum += red[rho * kSymRedStride + 16 * half + k];
                    wave_sync();
                    sum += wave_shfl_xor_f(sum, 32);
                    if (half == 0 && j0 + col < s1) {
                        if (FACT) sum *= symsums.ey[j0 + col];       // the sources' factor exp2(-|y'|^2)
                        if (fixscale != 0.f) {
                            // |v| < 2^61, and a float has 24 bits: both halves of the integer from exact float steps
                            // (rounded down to a whole unit, which is below 1e-18 of the bound)
                            const float v = sum * fixscale;
                            const float hf = floorf(v * 2.3283064365386963e-10f);          // v / 2^32
                            const float lf = fmaf(hf, -4294967296.f, v);                     // in [0, 2^32)
                            const long long iv = (long long)(((unsigned long long)(unsigned)(int)hf << 32) | (unsigned)lf);
                            atomic_add_i64(symsums.fix + j0 + col, iv);
                        }
                        else atomic_add_f32(outs + j0 + col, sum);
                    }
                }
            } else if (nlive == TPW) {
                // the usual case, free of branches: the compiler may start the matrix products of the
                // next tiles while the vector ALU works on the exponentials of this one
#pragma unroll
                for (int q = 0; q < TPW; q++) tile(q);
            } else {
#pragma unroll
                for (int q = 0; q < TPW; q++)
                    if (q < nlive) tile(q);              // uniform per wavefront
            }
        }
        if (FACT) {
#pragma unroll
            for (int q = 0; q < TPW; q++)
#pragma unroll
                for (int c = 0; c < NC; c++) acc[q][c] = fmaf(run[q][c], ex[q], acc[q][c]);
        }
      }
    }
#pragma unroll
    for (int q = 0; q < TPW; q++) {
        const int i = x0 + q * 32 + col;
#pragma unroll
        for (int c = 0; c < NC; c++) {
            float total = acc[q][c] + wave_shfl_xor_f(acc[q][c], 32);
            if (half == 0 && i < x1) {
                if (nsplit > 1) part[(((long long)slice * NC + c) * nitems + wid) * (TPW * 32) + q * 32 + col] = total;
                else if (SYM && fixscale == 0.f) atomic_add_f32(outs + c * ostride + i, total);
                else if (dout.out == nullptr) outs[c * ostride + i] += total;
                else if (c < dout.ncol) direct_add(dout, i, c, total);
            }
        }
    }
}

template <int D, int TPW, int NC, bool FACT = false>
__global__ void __launch_bounds__(kNearWavesPerBlock * 64, (D <= 3 && TPW == 4 && NC == 1) ? 5 : 2) near_g_kernel(
    const float *__restrict__ xs, long long N, const h8 *__restrict__ ops, long long stride, const float *__restrict__ bs,
    long long bstride, float *__restrict__ outs, long long ostride, const int *__restrict__ offx,
    const int *__restrict__ offy, const int *__restrict__ celly, Geo geoy, float edgey,
    const int *__restrict__ pairs, const int *__restrict__ rowptr, const int *__restrict__ tileoff, int nbx, float sc,
    int stripe, int nsplit, float *__restrict__ part, int nitems, const int *__restrict__ order, DirectOut dout)
{
    near_g_body<D, TPW, NC, FACT, false>(xs, N, ops, stride, bs, bstride, outs, ostride, offx, offy, celly, geoy, edgey, pairs,
                                         rowptr, tileoff, nbx, sc, stripe, nsplit, part, nitems, order, dout, SymSums());
}

// the symmetric form: four or five target tiles per wavefront, one column, the plain exponent; held to 120 registers, so
// that four wavefronts leave 32 of a SIMD's 512 to the far field's small workgroups on the second stream (the attribute
// counts register pairs on this target; what does not fit is spilled outside the loops over the tiles)
#ifdef F3M_CPU_EMU
#define F3M_NEAR_SYM_REGS
#else
#define F3M_NEAR_SYM_REGS __attribute__((amdgpu_num_vgpr(60)))      // counted in pairs on this target: 120 registers
#endif
// WPB wavefronts per workgroup.  One, up to three dimensions and where the far field beside it consists of small
// workgroups: a freed place is taken at once, not when a second one is free as well (N=1e7 3-D: 8.07 -> 7.9 ms, N(0,I)
// 12.85 -> 12.6).  The far field is pushed back by that: in 4-D, whose M2L is longer, the product gains nothing
// (12.4 -> 12.4-12.7 ms), and the large M2L workgroups of the 5^3 and 6^3 grids come in so late that the products take
// longer (216 nodes: 8.65 -> 9.4 ms): two wavefronts there.
constexpr int near_sym_waves(int d, bool small_far) { return d <= 3 && small_far ? 1 : kNearWavesPerBlock; }
template <int D, int TPW, int WPB>
__global__ void __launch_bounds__(WPB * 64, 4) F3M_NEAR_SYM_REGS near_sym_kernel(
    const float *__restrict__ xs, long long N, const h8 *__restrict__ ops, long long stride, const float *__restrict__ bs,
    long long bstride, float *__restrict__ outs, long long ostride, const int *__restrict__ offx,
    const int *__restrict__ offy, const int *__restrict__ celly, Geo geoy, float edgey,
    const int *__restrict__ pairs, const int *__restrict__ rowptr, const int *__restrict__ tileoff, int nbx, float sc,
    int stripe, int nsplit, float *__restrict__ part, int nitems, const int *__restrict__ order, DirectOut dout,
    SymSums symsums)
{
    near_g_body<D, TPW, 1, false, true, WPB>(xs, N, ops, stride, bs, bstride, outs, ostride, offx, offy, celly, geoy, edgey, pairs,
                                      rowptr, tileoff, nbx, sc, stripe, nsplit, part, nitems, order, dout, symsums);
}

// the symmetric form with the factored exponent (five dimensions): the far field does not run beside it (plan_apply), so
// it keeps the 128 registers of four wavefronts per SIMD
template <int D, int TPW>
__global__ void __launch_bounds__(64, 4) near_symf_kernel(
    const float *__restrict__ xs, long long N, const h8 *__restrict__ ops, long long stride, const float *__restrict__ bs,
    long long bstride, float *__restrict__ outs, long long ostride, const int *__restrict__ offx,
    const int *__restrict__ offy, const int *__restrict__ celly, Geo geoy, float edgey,
    const int *__restrict__ pairs, const int *__restrict__ rowptr, const int *__restrict__ tileoff, int nbx, float sc,
    int stripe, int nsplit, float *__restrict__ part, int nitems, const int *__restrict__ order, DirectOut dout,
    SymSums symsums)
{
    near_g_body<D, TPW, 1, true, true, 1>(xs, N, ops, stride, bs, bstride, outs, ostride, offx, offy, celly, geoy, edgey, pairs,
                                       rowptr, tileoff, nbx, sc, stripe, nsplit, part, nitems, order, dout, symsums);
}

// outs += the slices of a split near field, in slice order; one thread per target slot of a work item
__global__ void near_reduce_kernel(const float *__restrict__ part, int nsplit, int nc, int nitems, int tile,
                                   const int *__restrict__ tileoff, int nbx, const int *__restrict__ offx,
                                   float *__restrict__ outs, long long ostride)
{
    const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const int wid = (int)(e / tile), r = (int)(e % tile);
    if (wid >= nitems || wid >= tileoff[nbx]) return;
    const int bx = find_box(tileoff, nbx, wid);
    const int i = offx[bx] + (wid - tileoff[bx]) * tile + r;
    if (i >= offx[bx + 1]) return;
    for (int c = 0; c < nc; c++) {
        // slices in their order, eight loads in flight at a time (the loads do not depend on each other, the sum does)
        const float *p = part + ((long long)c * nitems + wid) * tile + r;
        const long long step = (long long)nc * nitems * tile;
        float sum = 0.f;
        int sl = 0;
        for (; sl + 8 <= nsplit; sl += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = p[(sl + u) * step];
#pragma unroll
            for (int u = 0; u < 8; u++) sum += v[u];
        }
        for (; sl < nsplit; sl++) sum += p[sl * step];
        outs[c * ostride + i] += sum;
    }
}

// whether the near field of a level goes to the matrix-pipe kernel (see near_field)
static bool near_on_matrix_pipe(int d, float lcs, float edge)
{
    const float sc_edge = sqrtf(lcs * kLog2e) * edge;
    bool use_mfma = 30.f * (float)d * sc_edge * sc_edge <= 1200.f;
    if (const char *env = getenv("F3M_NEAR")) use_mfma = !strcmp(env, "mfma") ? true : (!strcmp(env, "valu") ? false : use_mfma);
    return use_mfma;
}

// whether the near field of a level takes the factored form (see near_slots): only where it saves a matrix
// instruction, and while the exponent 2x''.y' (at most 10 d S^2, targets within five edges of the anchor and sources
// within one) stays below 30: the sum of a run, exp2(2x''.y') times weights, then stays below 2^30 times the weights'
// sum, so that weights up to ~1e28 cannot overflow where the plain form (every term at most its weight) would not.
// F3M_NEAR_FACT=0|1 overrides (1: wherever the form saves an instruction).
static bool near_factored(int d, float lcs, float edge)
{
    const bool pays = d == 5 || d == 10;             // near_fact_pays(d)
    const float S = sqrtf(lcs * kLog2e) * edge;
    bool fact = pays && 10.f * (float)d * S * S <= 30.f;
    if (const char *env = getenv("F3M_NEAR_FACT")) fact = pays && atoi(env) != 0;
    return fact;
}

struct NearOps {
    const h8 *ops;
    const float *ey;       // factored form only
};

// The split-f16 source operands of a level, kept with it.  only (nullable): operands are needed for the source boxes
// of this list alone (at most levels a small part of the boxes); otherwise for every box.
// Returns the table to use: the one of every box if it exists, else (for a list that is the level's only one) the table
// of that list's source boxes; whichever is missing is built, none is ever rebuilt.
static NearOps build_near_operands(int d, const Tree &ty, const TreeLevel &ly, float sc, bool fact, const PairList *only,
                                   hipStream_t s)
{
    const bool only_list = only != nullptr;
    F3M_REQUIRE(ly.nearops_sc == 0.f || ly.nearops_sc == sc, 38, "near-field operands of a level asked for with another lengthscale");
    if (ly.nearops_all.size() != 0) return NearOps{reinterpret_cast<const h8 *>(ly.nearops_all.get()), ly.nearey_all.get()};
    if (only_list && ly.nearops.size() != 0) return NearOps{reinterpret_cast<const h8 *>(ly.nearops.get()), ly.nearey.get()};
    const int NS = near_insts(d, fact);
    const long long stride = ty.n + 32;
    require_tables_may_be_built("the near-field source operands of a level");
    DBuf<unsigned char> &table = only_list ? ly.nearops : ly.nearops_all;
    DBuf<float> &eytab = only_list ? ly.nearey : ly.nearey_all;
    table.reset((size_t)NS * 2 * stride * 16);
    if (fact) {
        eytab.reset((size_t)stride);
        dev_fill(eytab.get(), 0, sizeof(float) * (size_t)stride, s);     // points that the operands skip keep a zero factor
    }
    ly.nearops_sc = sc;
    DBuf<int> need;
    if (only_list) {
        DBuf<int> fy((size_t)ly.nb);
        dev_fill(fy.get(), 0, sizeof(int) * (size_t)ly.nb, s);
        F3M_LAUNCH(mark_cols_kernel, cdiv(only->n, 256), 256, 0, s, only->pairs.get(), only->n, fy.get());
        check_launch("mark_cols");
        need.reset((size_t)ly.nb + 1);
        exclusive_scan_i32(fy.get(), ly.nb, need.get(), s);
    }
    const int *box32 = box_table(ly, ty.n, s);
#define F3M_CASE(DD)                                                                                                  \
    case DD:                                                                                                          \
        if constexpr (near_fact_pays(DD)) {                                                                           \
            if (fact) {                                                                                               \
                F3M_LAUNCH((near_operands_kernel<DD, true>), cdiv(stride, kOpsBlock), kOpsBlock, 0, s, ty.pts.get(),  \
                           ty.n, ly.off.get(), ly.nb, ly.cell.get(), ty.geo, ly.edge, sc, stride,                    \
                           only_list ? need.get() : (const int *)nullptr, box32,                                      \
                           reinterpret_cast<h8 *>(table.get()), eytab.get());                                         \
                break;                                                                                                \
            }                                                                                                         \
        }                                                                                                             \
        F3M_LAUNCH((near_operands_kernel<DD, false>), cdiv(stride, kOpsBlock), kOpsBlock, 0, s, ty.pts.get(), ty.n,   \
                   ly.off.get(), ly.nb, ly.cell.get(), ty.geo, ly.edge, sc, stride,                                  \
                   only_list ? need.get() : (const int *)nullptr, box32,                                              \
                   reinterpret_cast<h8 *>(table.get()), (float *)nullptr);                                            \
        break;
    switch (d) {
        F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
        F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
    default: throw Error(2, "dimension must be 1..10");
    }
#undef F3M_CASE
    check_launch("near_operands");
    return NearOps{reinterpret_cast<const h8 *>(table.get()), fact ? eytab.get() : nullptr};
}

// The operands of every box of a level, ahead of the near field (the plan calls this for its deepest level, beside
// the kernels that build that level's lists); nothing happens where the near field would take the all-vector kernel.
void prepare_near_operands(int d, const Tree &ty, const TreeLevel &ly, float lcs, hipStream_t s)
{
    if (!near_on_matrix_pipe(d, lcs, ly.edge)) return;
    build_near_operands(d, ty, ly, sqrtf(lcs * kLog2e), near_factored(d, lcs, ly.edge), nullptr, s);
}

// the launch shape near_field gives a list: target tiles per wavefront and, where the plan has counted the rows of
// the list, the exact number of work items (else -1)
static void near_shape(const Tree &tx, const TreeLevel &lx, const PairList &list, int nc, int &tpw, long long &items_exact,
                       bool sym_capable = false)
{
    const long long avg_points = list.rows > 0 ? list.row_points / list.rows : tx.n / std::max(1, lx.nb);
    const long long tiles = (avg_points + 31) / 32;
    tpw = (tiles == 5 && nc == 1) ? 5 : 4;
    // (The factored 5-D kernel with a fifth tile, ten tiles of a box as 5 + 5 instead of 4 + 4 + 2, takes 127 registers:
    // four wavefronts then fill the 512 of a SIMD and the far field's wavefronts get in beside them only now and
    // then.  N=1e7: the fastest products 39.8 ms against 40.9, but single products up to 48.9 and means of 40.8-42.8
    // against a steady 41.0 with four tiles, 115 registers.  Four it is.)
    // A list that can take the symmetric form (four wavefronts per SIMD with either shape): five wherever that cuts a
    // typical box into fewer work items, e.g. ten tiles as 5 + 5 instead of 4 + 4 + 2 -- the source tiles are then loaded,
    // and their column sums added up and sent off, twice per box instead of three times (N=1e7, 3-D: 8.47 -> 8.12 ms).
    // Only for a list that will not be cut into slices (whose sums, and so the bits of a column, depend on the number of
    // work items: a column keeps the bits it has inside a group of columns).
    if (sym_capable && nc == 1 && (tiles + 4) / 5 < (tiles + 3) / 4 && list.rows >= 0 && list.items160 >= 16384) tpw = 5;
    if (const char *e = getenv("F3M_NEAR_TPW")) tpw = (atoi(e) == 5 && nc == 1) ? 5 : 4;      // tuning aid
    items_exact = list.rows >= 0 ? (tpw == 5 ? list.items160 : list.items128) : -1;
}

bool near_single_pass(int d, const Tree &tx, const TreeLevel &lx, const PairList &list, float lcs, int nc)
{
    if (list.n == 0 || !near_on_matrix_pipe(d, lcs, lx.edge)) return false;
    int tpw;
    long long items_exact;
    near_shape(tx, lx, list, nc, tpw, items_exact);
    return items_exact >= 16384;          // fewer work items: the lists are cut into slices with partial sums
}

// Whether near_field takes a list in the symmetric form (see near_g_kernel): one tree (then every list of the plan names
// (A,B) exactly when it names (B,A): the class of a pair depends on the distance of the centres and on the sum of the
// two boxes' counts), one column, the matrix-pipe kernel: with the plain exponent up to four dimensions, with the
// factored one in five.
// F3M_NEAR_SYM=0 turns it off.
bool near_symmetric(int d, const Tree &tx, const TreeLevel &lx, const Tree &ty, const PairList &list, float lcs, int nc)
{
    if (&tx != &ty || nc != 1 || d > 5 || list.n == 0) return false;
    if (const char *e = getenv("F3M_NEAR_SYM")) if (atoi(e) == 0) return false;
    // (in five dimensions the factored form only: the plain one has no registers left for it)
    return near_on_matrix_pipe(d, lcs, lx.edge) && (d == 5) == near_factored(d, lcs, lx.edge);
    // (lists cut into slices, see near_field, take the plain form all the same)
}

void near_field(int d, const Tree &tx, const TreeLevel &lx, const Tree &ty, const TreeLevel &ly, const PairList &list,
                const float *bs, float *outs, float lcs, hipStream_t s, int nc, long long bstride, long long ostride,
                bool only_list, bool prepare_only, const DirectOut *direct, const SymSums *symsums)
{
    if (list.n == 0) return;
    F3M_REQUIRE(nc == 1 || nc == 2 || nc == 4, 34, "near field takes 1, 2 or 4 columns at a time");
    // The matrix-pipe kernel splits operands into f16 pairs, which keeps the exponent of a pair accurate to
    // about 2^-22 times the products that enter it, (|x''| + |y'|)^2.  Sources lie within one edge per
    // dimension of their anchor, |y'| <= S sqrt(d) with S = sc edge, and a target at scaled distance r of a
    // source within r + S sqrt(d): a pair that matters (2^(-r^2) not negligible, r of order 1) has an
    // exponent error of about 2^-22 4 S^2 d, and pairs with larger errors have targets several boxes away
    // whose kernel values vanish against the others as S grows.  The kernel is used while 30 d S^2 <= 1200,
    // i.e. a relative error of a term below 3e-5 (box edge up to ~3.6 lengthscales in 3-D; the N(0,I) cloud
    // with ls = 0.1 has the same error against the fp64 product, 1.3968e-3, with either kernel at every
    // level), otherwise the all-vector kernel.  F3M_NEAR=valu|mfma overrides the choice.
    const bool use_mfma = near_on_matrix_pipe(d, lcs, lx.edge);
    constexpr int T = 1;
    // all-vector kernel: whole boxes per workgroup where possible (multiple of the wave size, <= 512 lanes)
    int bd = ((lx.maxcount + kWave - 1) / kWave) * kWave;
    if (bd > 512) bd = 256;
    if (bd < kWave) bd = kWave;
    // target tiles of 32 per wavefront: 4 (2: 10.2 ms, 4: 9.2 ms, 5: 10.2 ms, 8: 9.4 ms at N=1e7, d=3, ten tiles
    // per box), but 5 where a typical box has five tiles and would otherwise be cut into 4 + 1
    // (N=1e7, d=4, 153 points per box: 16.9 -> 15.6 ms at the time)
    // Where the plan has counted the rows of the list, "typical" is the mean over the listed boxes and the
    // number of work items is exact; otherwise the mean over all boxes and an upper bound.
    int tpw;
    long long items_exact;
    // (the shape follows from what the list could take, not from whether this call brings a place for the fixed-point
    // sums: the tile table of a list is then the same for every call)
    const bool sym_capable = near_symmetric(d, tx, lx, ty, list, lcs, nc);
    const bool sym_wanted = sym_capable && symsums != nullptr && symsums->fix != nullptr;
    near_shape(tx, lx, list, nc, tpw, items_exact, sym_capable);
    // From five dimensions on the work items are long and their lists differ a lot in length (3^5 boxes around
    // an interior box, 2^5 around a corner): the boxes with the longest lists go first, which shortens the
    // end of the launch (N=1e7, 5-D: 44.6 -> 43.6 ms; 4-D and 3-D lose the Morton order's cache locality and
    // the time of the ordering itself: 11.7 -> 11.8 ms, 10.5 -> 10.8 ms per product).  Lists that are not
    // sliced only.  F3M_NEAR_ORDER=0|1 overrides.
    bool want_order = d >= 5;
    if (const char *e = getenv("F3M_NEAR_ORDER")) want_order = atoi(e) != 0;
    const bool ordered = use_mfma && want_order && items_exact >= 16384 && lx.nb <= 65536;   // one workgroup places the boxes
    // The tile table of this list (offsets of the work items per box, in launch order) depends on the plan
    // only and is kept with the list.
    const int tilesize = use_mfma ? tpw * 32 : bd * T;
    TileTable &tt = list.near_tiles[tilesize * 2 + (ordered ? 1 : 0)];
    if (tt.tileoff.size() == 0) {
        require_tables_may_be_built("the near-field tile table of a list");
        if (!ordered) {
            // (the rows of the list mark the boxes: no pass of its own for the flags)
            tt.bound = build_tiles(lx.off.get(), nullptr, lx.nb, tx.n, tilesize, tt.tileoff, s, nullptr, list.rowptr.get());
        } else {
        DBuf<int> flag((size_t)lx.nb);
        F3M_LAUNCH(mark_rows_kernel, cdiv(lx.nb, 256), 256, 0, s, list.rowptr.get(), lx.nb, flag.get());
        check_launch("mark_rows");
        if (ordered) {
            DBuf<int> cls((size_t)lx.nb), hist(256);
            tt.order.reset((size_t)lx.nb);
            dev_fill(hist.get(), 0, 256 * sizeof(int), s);
            const int unit = (int)std::max<long long>(1, list.n / std::max<long long>(1, list.rows) / 64);   // mean row = class 64
            F3M_LAUNCH(row_class_count_kernel, cdiv(lx.nb, 256), 256, 0, s, list.rowptr.get(), lx.nb, unit, cls.get(), hist.get());
            check_launch("row_class_count");
            F3M_LAUNCH(class_place_kernel, 1, 1024, 0, s, cls.get(), lx.nb, hist.get(), tt.order.get());
            check_launch("class_place");
        }
        tt.bound = build_tiles(lx.off.get(), flag.get(), lx.nb, tx.n, tilesize, tt.tileoff, s, ordered ? tt.order.get() : nullptr);
        }
    }
    const int *ord = ordered ? tt.order.get() : nullptr;
    const DBuf<int> &tileoff = tt.tileoff;
    int ntiles = tt.bound;
    if (use_mfma && items_exact >= 0) ntiles = (int)std::max<long long>(1, items_exact);
    float sc = sqrtf(lcs * kLog2e);
    if (use_mfma) {
        const long long stride = ty.n + 32;
        // the form of a table is decided when it is built and read off the table afterwards (ey comes with the factored one)
        const NearOps src = build_near_operands(d, ty, ly, sc, near_factored(d, lcs, ly.edge), only_list ? &list : nullptr, s);
        const bool fact = src.ey != nullptr;
        if (prepare_only) return;
        const bool sym = sym_wanted && fact == (d == 5);
        F3M_REQUIRE(!(sym && direct), 35, "direct output and the symmetric near field exclude each other");
        int stripe = 128;   // consecutive workgroups per XCD stripe (0: 9.5 ms, 16: 9.3, 64-256: 9.15, 1024: 9.4 at N=1e7)
        if (const char *env = getenv("F3M_NEAR_STRIPE")) stripe = atoi(env);       // tuning aid
        // Few targets against long lists (the transposed product of a tall kernel matrix): too few work
        // items to fill the GPU, so every list is cut into slices with a wavefront each.
        // (A list that takes the symmetric form stays whole from 4096 work items on: half the tiles outweigh the
        // emptier end of the launch.  Uniform 3-D clouds, whole product with 4096 against 16384: N=6e5 0.82 against 0.86
        // ms, 1.1e6 1.36 / 1.49, 1.5e6 1.81 / 2.01; with 2048 N=3e5 takes 1.05 against 0.83 ms.)
        int single = sym ? 4096 : 16384;
        if (const char *e = getenv("F3M_SYM_SINGLE")) single = sym ? atoi(e) : single;   // tuning aid
        int nsplit = 1;
        if (ntiles < single) {
            int target = 32768;      // wavefronts aimed at (K_nm^T u with 1e7 sources, 2e4 / 1e5 targets: 8192 -> 9.7 / 8.1 ms,
                                     // 16384 -> 7.6 / 6.8, 32768 -> 7.5 / 6.0)
            if (const char *e = getenv("F3M_SPLIT_TARGET")) target = atoi(e);
            nsplit = std::min(128, (int)cdiv(target, std::max(1, ntiles)));
        }
        DBuf<float> part;
        if (nsplit > 1) part.reset((size_t)nsplit * nc * ntiles * tpw * 32);   // every slot of a live work item is written
        F3M_REQUIRE(direct == nullptr || nsplit == 1, 35, "direct output needs a near field of one wavefront per work item");
        const DirectOut dout = direct ? *direct : DirectOut();
        // wavefronts per workgroup (the factored symmetric form, which nothing runs beside: one)
        const int wpb = (sym && nsplit == 1) ? (fact ? 1 : near_sym_waves(d, symsums->small_far)) : kNearWavesPerBlock;
        int nblk = (int)cdiv((long long)ntiles * nsplit, wpb);
        int ngrid = stripe > 0 ? (int)cdiv(nblk, 8 * stripe) * 8 * stripe : nblk;
        timer_begin(kNear, s);
        // weights of the factored form: the sorted weights times exp2(-|y'|^2) of their point (one pass per product)
        DBuf<float> ws;
        const float *wsrc = bs;
        long long wstride = bstride;
        if (fact) {
            ws.reset((size_t)stride * nc);
            wstride = stride;
            F3M_LAUNCH(near_weights_kernel, cdiv(stride, 256), 256, 0, s, bs, src.ey, stride, nc, bstride, ws.get());
            check_launch("near_weights");
            wsrc = ws.get();
        }
        auto go = [&](auto kern) {
            F3M_LAUNCH(kern, ngrid, kNearWavesPerBlock * 64, 0, s, tx.pts.get(), tx.n, src.ops, stride, wsrc, wstride, outs,
                       ostride, lx.off.get(), ly.off.get(), ly.cell.get(), ty.geo, ly.edge, list.pairs.get(),
                       list.rowptr.get(), tileoff.get(), lx.nb, sc, stripe, nsplit, part.get(), ntiles, ord, dout);
        };
        auto go_sym = [&](auto kern) {
            SymSums sums = *symsums;
            sums.braw = bs;
            sums.ey = src.ey;
            F3M_LAUNCH(kern, ngrid, wpb * 64, 0, s, tx.pts.get(), tx.n, src.ops, stride, wsrc, wstride, outs,
                       ostride, lx.off.get(), ly.off.get(), ly.cell.get(), ty.geo, ly.edge, list.pairs.get(),
                       list.rowptr.get(), tileoff.get(), lx.nb, sc, stripe, nsplit, part.get(), ntiles, ord, dout, sums);
        };
#define F3M_NEAR_FORM(DD, FF)                                                                                         \
    if constexpr ((DD <= 4 && !FF) || (DD == 5 && FF)) {                                                              \
        if (sym && nsplit == 1) {                                                                                     \
            if constexpr (FF) {                                                                                       \
                if (tpw == 5) go_sym((near_symf_kernel<DD, 5>));                                                      \
                else go_sym((near_symf_kernel<DD, 4>));                                                               \
            } else {                                                                                                  \
                if constexpr (DD <= 3) {                                                                              \
                    if (wpb == 1) {                                                                                   \
                        if (tpw == 5) go_sym((near_sym_kernel<DD, 5, 1>));                                            \
                        else go_sym((near_sym_kernel<DD, 4, 1>));                                                     \
                        break;                                                                                        \
                    }                                                                                                 \
                }                                                                                                     \
                if (tpw == 5) go_sym((near_sym_kernel<DD, 5, kNearWavesPerBlock>));                                   \
                else go_sym((near_sym_kernel<DD, 4, kNearWavesPerBlock>));                                            \
            }                                                                                                         \
            break;                                                                                                    \
        }                                                                                                             \
    }                                                                                                                 \
    if (tpw == 5) go(near_g_kernel<DD, 5, 1, FF>);                                                                    \
    else if (nc == 4) go(near_g_kernel<DD, 4, 4, FF>);                                                                \
    else if (nc == 2) go(near_g_kernel<DD, 4, 2, FF>);                                                                \
    else go(near_g_kernel<DD, 4, 1, FF>);
#define F3M_CASE(DD)                                                                                                  \
    case DD:                                                                                                          \
        if constexpr (near_fact_pays(DD)) {                                                                           \
            if (fact) {                                                                                               \
                F3M_NEAR_FORM(DD, true)                                                                               \
                break;                                                                                                \
            }                                                                                                         \
        }                                                                                                             \
        F3M_NEAR_FORM(DD, false)                                                                                      \
        break;
        switch (d) {
            F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
            F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
        default: throw Error(2, "dimension must be 1..10");
        }
#undef F3M_CASE
#undef F3M_NEAR_FORM
        if (nsplit > 1) {
            check_launch("near_g");
            F3M_LAUNCH(near_reduce_kernel, cdiv((long long)ntiles * tpw * 32, 256), 256, 0, s, part.get(), nsplit, nc, ntiles,
                       tpw * 32, tileoff.get(), lx.nb, lx.off.get(), outs, ostride);
        }
    } else {
        if (prepare_only) return;
        F3M_REQUIRE(direct == nullptr, 35, "direct output needs the matrix-pipe near field");
        timer_begin(kNear, s);
#define F3M_CASE(DD)                                                                                                  \
    case DD:                                                                                                          \
        for (int c = 0; c < nc; c++)                                                                                  \
            F3M_LAUNCH((near_kernel<DD, T>), ntiles, bd, 0, s, tx.pts.get(), tx.n, ty.pts.get(), ty.n,                \
                       bs + c * bstride, outs + c * ostride, lx.off.get(), ly.off.get(), lx.ctr.get(),                \
                       list.pairs.get(), list.rowptr.get(), tileoff.get(), lx.nb, sc);                                \
        break;
        switch (d) {
            F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
            F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
        default: throw Error(2, "dimension must be 1..10");
        }
#undef F3M_CASE
    }
    timer_end(s);
    check_launch("near_field");
}

// ------------------------------------------------------------------------------------------------
// interpolation nodes (F3M_src/n_tree.cu:265-349, F3M_src/1_d_conv.cu:850-884)

struct NodeMeta {
    int n[kMaxD];
    int start[kMaxD];
    int S1, P;
};

static NodeMeta meta_of(const NodeSet &ns)
{
    NodeMeta nm;
    for (int k = 0; k < kMaxD; k++) { nm.n[k] = ns.n[k] > 0 ? ns.n[k] : 1; nm.start[k] = ns.start[k]; }
    nm.S1 = ns.S1;
    nm.P = ns.P;
    return nm;
}

// 1-D first-kind Chebyshev nodes t_i = cos((2i+1)pi/(2n)) and barycentric weights
// w_i = (-1)^i sin((2i+1)pi/(2n)) of every dimension, pi as a float (F3M_src/n_tree.cu:265-285)
__global__ void nodes_kernel(NodeMeta nm, int d, float *__restrict__ t, float *__restrict__ w)
{
    int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= nm.S1) return;
    int j = 0;
    while (j + 1 < d && e >= nm.start[j + 1]) j++;
    const int i = e - nm.start[j], n = nm.n[j];
    const float PI = 3.14159274101257324f;
    float a = (float)i;
    a = a * 2.0f;
    a = a + 1.0f;
    a = a * PI;
    a = a / (float)(2 * (n - 1) + 2);
    t[e] = cosf(a);
    double sg = (i % 2 == 0) ? 1.0 : -1.0;
    w[e] = (float)(sg * sin(((2. * (double)i + 1.) * (double)PI) / (2. * (double)(n - 1) + 2.)));
}

// node position inside a box relative to its centre: cheb*edge/2 + edge/2 (F3M_src/n_tree.cu:510)
__global__ void node_offsets_kernel(NodeMeta nm, int d, const float *__restrict__ t, float edge, float *__restrict__ noff)
{
    int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= nm.P * d) return;
    int m = e / d, j = e % d, cum = 1;
    for (int k = 0; k < j; k++) cum *= nm.n[k];
    int a = (m / cum) % nm.n[j];
    float v = t[nm.start[j] + a] * edge;
    v = v / 2.f;
    noff[e] = v + edge / 2.f;
}

// tables of the separable M2L: E_j[o][a][q] = exp(-lcs ((t_a - t_q) edge/2 - ((omin_j+o) edge + delta_j))^2)
struct SepGeo {
    double delta[kMaxD];
    int omin[kMaxD];
};
__global__ void sep_tables_kernel(NodeMeta nm, int d, int NT, int noffsets, const float *__restrict__ t, double edge, double lcs,
                                  SepGeo g, float *__restrict__ tab)
{
    int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= d * noffsets * NT * NT) return;
    int q = e % NT, a = (e / NT) % NT, oi = (e / (NT * NT)) % noffsets, j = e / (NT * NT * noffsets);
    float v = 0.f;
    if (a < nm.n[j] && q < nm.n[j]) {
        double shift = (double)(g.omin[j] + oi) * edge + g.delta[j];
        double diff = ((double)t[nm.start[j] + a] - (double)t[nm.start[j] + q]) * (edge / 2) - shift;
        v = (float)exp(-lcs * diff * diff);
    }
    tab[e] = v;
}

void make_nodes(NodeSet &ns, int d, int max_nodes, hipStream_t s)
{
    ns.d = d;
    // node counts per dimension (n_tree.cu:328-346); the reference then shuffles the dimensions
    // at random (:347), which is the identity whenever max_nodes is a perfect d-th power; the order
    // of :328-346 is kept here
    float ref_val = (float)pow((double)max_nodes, 1.0 / (double)(float)d);
    int hi = (int)std::ceil(ref_val), lo = (int)std::floor(ref_val), acc = 1;
    ns.P = 1;
    ns.S1 = 0;
    for (int i = 0; i < d; i++) {
        int fut = (int)((double)acc * pow((double)lo, (double)(d - (i + 1))) * (double)hi);
        int pick = fut <= max_nodes ? hi : lo;
        if (pick < 1) pick = 1;
        ns.n[i] = pick;
        acc *= pick;
        ns.start[i] = ns.S1;
        ns.S1 += pick;
        ns.P *= pick;
    }
    ns.dt.reset(ns.S1);
    ns.dw.reset(ns.S1);
    NodeMeta nm = meta_of(ns);
    F3M_LAUNCH(nodes_kernel, cdiv(ns.S1, 64), 64, 0, s, nm, d, ns.dt.get(), ns.dw.get());
    check_launch("nodes");
    ns.noff.reset((size_t)ns.P * d);
}

void set_node_offsets(NodeSet &ns, float edge, hipStream_t s)
{
    NodeMeta nm = meta_of(ns);
    F3M_LAUNCH(node_offsets_kernel, cdiv((long long)ns.P * ns.d, 256), 256, 0, s, nm, ns.d, ns.dt.get(), edge, ns.noff.get());
    check_launch("node_offsets");
}


// 1-D barycentric basis values of one coordinate (F3M_src/1_d_conv.cu:418-448 and :217-238):
// l_a = (w_a/(t-t_a)) / sum_l w_l/(t-t_l), or the unit vector when t hits a node exactly.
__device__ inline void basis_1d(float t, const float *__restrict__ nt, const float *__restrict__ nw, int n,
                                float *__restrict__ out, float scale)
{
    // out[a] holds w_a/(t-t_a) until the sum is known; reciprocals by v_rcp_f32 (1 ulp)
    float sum = 0.f;
    int hit = -1;
    for (int a = 0; a < n; a++) {
        float diff = t - nt[a];
        if (diff == 0.f) hit = a;
        float q = nw[a] * fast_rcp(diff);
        out[a] = q;
        sum += q;
    }
    if (hit >= 0) {
        for (int a = 0; a < n; a++) out[a] = (a == hit) ? scale : 0.f;
    } else {
        float inv = scale * fast_rcp(sum);
        for (int a = 0; a < n; a++) out[a] *= inv;
    }
}

// ------------------------------------------------------------------------------------------------
// P2M (F3M_src/1_d_conv.cu:451-552): Mom[box][m] = sum_j L_m(y_j) b_j.  One workgroup per
// (box, chunk of points), one lane per node; per-chunk partial sums are combined in a fixed order
// by p2m_reduce_kernel, so the result does not depend on scheduling.

constexpr int kP2MChunk = 512;
constexpr int kP2MSub = 64;

template <int D>
__global__ void __launch_bounds__(1024) p2m_kernel(const float *__restrict__ ys, long long M, const float *__restrict__ bs,
                                                    const int *__restrict__ off, const float *__restrict__ ctr,
                                                    const int *__restrict__ tileoff, int nb, NodeMeta nm,
                                                    const float *__restrict__ nt, const float *__restrict__ nw, float factor,
                                                    float *__restrict__ partial)
{
    F3M_DYN_SHARED(float, smem);
    float *snt = smem;                       // S1
    float *snw = smem + nm.S1;               // S1
    float *sl = smem + 2 * nm.S1;            // kP2MSub * S1: per point, per dimension basis values
    const int tid = threadIdx.x, BD = blockDim.x;
    if ((int)blockIdx.x >= tileoff[nb]) return;     // launched with an upper bound of the chunk count
    const int box = find_box(tileoff, nb, blockIdx.x);
    const int chunk = blockIdx.x - tileoff[box];
    const int p0 = off[box] + chunk * kP2MChunk;
    const int p1 = min(off[box + 1], p0 + kP2MChunk);
    for (int a = tid; a < nm.S1; a += BD) { snt[a] = nt[a]; snw[a] = nw[a]; }
    // LDS offsets of this lane's node along every dimension
    int moff[D];
    {
        int rem = tid;
#pragma unroll
        for (int k = 0; k < D; k++) { moff[k] = nm.start[k] + rem % nm.n[k]; rem /= nm.n[k]; }
    }
    float acc = 0.f;
    for (int s0 = p0; s0 < p1; s0 += kP2MSub) {
        const int cnt = min(kP2MSub, p1 - s0);
        __syncthreads();
        for (int task = tid; task < cnt * D; task += BD) {
            int pt = task % cnt, k = task / cnt;
            float t = factor * (ys[(long long)k * M + s0 + pt] - ctr[(long long)box * D + k]);
            float scale = (k == 0) ? bs[s0 + pt] : 1.f;      // the weight rides on dimension 0
            basis_1d(t, snt + nm.start[k], snw + nm.start[k], nm.n[k], sl + pt * nm.S1 + nm.start[k], scale);
        }
        __syncthreads();
        if (tid < nm.P) {
            for (int pt = 0; pt < cnt; pt++) {
                const float *row = sl + pt * nm.S1;
                float v = row[moff[0]];
#pragma unroll
                for (int k = 1; k < D; k++) v *= row[moff[k]];
                acc += v;
            }
        }
    }
    if (tid < nm.P) partial[(long long)blockIdx.x * nm.P + tid] = acc;
}

// P2M for the 4 x 4 x 4 grid: one wavefront per (box, chunk of points).  64 points at a time: every lane
// prepares one point -- its twelve 1-D basis values in registers, then l0[0..3] and the 16 products
// w[a1 + 4 a2] = l1[a1] l2[a2] b to LDS -- and then lane (g, q), g = lane / 16, adds the points
// 16 g .. 16 g + 15 to its four moments (a0, q): one multiply-add per node and point, where the
// lane-per-node form spends two multiplications and three LDS reads as well.  The four partial sums
// of a node are added across the wavefront at the end.  Same partial-sum layout as p2m_kernel.
__device__ inline void basis4(float t, const float (&nt)[4], const float (&nw)[4], float (&out)[4], float scale)
{
    float sum = 0.f;
    int hit = -1;
#pragma unroll
    for (int a = 0; a < 4; a++) {
        const float diff = t - nt[a];
        if (diff == 0.f) hit = a;
        out[a] = nw[a] * fast_rcp(diff);
        sum += out[a];
    }
    const float inv = scale * fast_rcp(sum);
#pragma unroll
    for (int a = 0; a < 4; a++) out[a] = hit >= 0 ? (a == hit ? scale : 0.f) : out[a] * inv;
}

__global__ void __launch_bounds__(64) p2m_q64_kernel(const float *__restrict__ ys, long long M, const float *__restrict__ bs,
                                                      const int *__restrict__ off, const float *__restrict__ ctr,
                                                      const int *__restrict__ tileoff, int nb, const float *__restrict__ nt,
                                                      const float *__restrict__ nw, float factor, float *__restrict__ partial)
{
    // w of point p at 16 p + 16 (p / 16): the four groups of the accumulation read different banks
    __shared__ __align__(16) float sl0[64 * 4];
    __shared__ __align__(16) float sw[64 * 16 + 64];
    const int lane = threadIdx.x;
    if ((int)blockIdx.x >= tileoff[nb]) return;     // launched with an upper bound of the chunk count
    const int box = find_box(tileoff, nb, blockIdx.x);
    const int chunk = blockIdx.x - tileoff[box];
    const int p0 = off[box] + chunk * kP2MChunk;
    const int p1 = min(off[box + 1], p0 + kP2MChunk);
    float tn[3][4], tw[3][4], c[3];
#pragma unroll
    for (int k = 0; k < 3; k++) {
        c[k] = ctr[(long long)box * 3 + k];
#pragma unroll
        for (int a = 0; a < 4; a++) { tn[k][a] = nt[4 * k + a]; tw[k][a] = nw[4 * k + a]; }
    }
    const int g = lane >> 4, q = lane & 15;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = p0; s0 < p1; s0 += 64) {
        const int i = s0 + lane;
        const bool in = i < p1;
        float l[3][4];
#pragma unroll
        for (int k = 0; k < 3; k++) {
            const float t = in ? factor * (ys[(long long)k * M + i] - c[k]) : 0.f;
            basis4(t, tn[k], tw[k], l[k], 1.f);
        }
        const float b = in ? bs[i] : 0.f;            // lanes past the end add nothing
        __syncthreads();                             // the previous 64 points have been read by every lane
        *reinterpret_cast<float4 *>(sl0 + 4 * lane) = make_float4(l[0][0], l[0][1], l[0][2], l[0][3]);
        float *wrow = sw + 16 * lane + 16 * (lane >> 4);
#pragma unroll
        for (int a2 = 0; a2 < 4; a2++) {
            const float lb = l[2][a2] * b;
            *reinterpret_cast<float4 *>(wrow + 4 * a2) = make_float4(l[1][0] * lb, l[1][1] * lb, l[1][2] * lb, l[1][3] * lb);
        }
        __syncthreads();
#pragma unroll 4
        for (int pt = 0; pt < 16; pt++) {
            const int pp = 16 * g + pt;
            const float4 l0 = *reinterpret_cast<const float4 *>(sl0 + 4 * pp);
            const float w = sw[16 * pp + 16 * g + q];
            acc[0] = fmaf(l0.x, w, acc[0]);
            acc[1] = fmaf(l0.y, w, acc[1]);
            acc[2] = fmaf(l0.z, w, acc[2]);
            acc[3] = fmaf(l0.w, w, acc[3]);
        }
    }
#pragma unroll
    for (int a = 0; a < 4; a++) {
        acc[a] += wave_shfl_xor_f(acc[a], 16);
        acc[a] += wave_shfl_xor_f(acc[a], 32);
    }
    if (g == 0)                                      // node a0 + 4 q
        *reinterpret_cast<float4 *>(partial + (long long)blockIdx.x * 64 + 4 * q) = make_float4(acc[0], acc[1], acc[2], acc[3]);
}

// The same scheme for other tensor grids of N nodes per dimension: a lane holds the N^R moments of the
// first R dimensions for one combination q of the others, Q = N^(D-R) <= 64; lane (g, q), g = lane / Q <
// G = 64 / Q, adds the points of its group.
__host__ __device__ constexpr int ipow(int b, int e) { return e == 0 ? 1 : b * ipow(b, e - 1); }
template <int D, int N, int R>
__global__ void __launch_bounds__(64) p2m_tensor_kernel(const float *__restrict__ ys, long long M, const float *__restrict__ bs,
                                                         const int *__restrict__ off, const float *__restrict__ ctr,
                                                         const int *__restrict__ tileoff, int nb, const float *__restrict__ nt,
                                                         const float *__restrict__ nw, float factor, float *__restrict__ partial)
{
    constexpr int NR = ipow(N, R), Q = ipow(N, D - R), G = 64 / Q, PG = (64 + G - 1) / G, QS = Q | 1, P = Q * NR;   // QS: odd row stride
    static_assert(Q <= 64, "one wavefront holds the nodes of the last D-R dimensions");
    __shared__ float sh[64 * NR];
    __shared__ float sw[64 * QS];
    float *const red = NR <= QS ? sw : sh;          // 64 * NR floats for the closing sum over the groups
    const int lane = threadIdx.x;
    if ((int)blockIdx.x >= tileoff[nb]) return;     // launched with an upper bound of the chunk count
    const int box = find_box(tileoff, nb, blockIdx.x);
    const int chunk = blockIdx.x - tileoff[box];
    const int p0 = off[box] + chunk * kP2MChunk;
    const int p1 = min(off[box + 1], p0 + kP2MChunk);
    const int g = lane / Q, q = lane % Q;
    float acc[NR];
#pragma unroll
    for (int a = 0; a < NR; a++) acc[a] = 0.f;
    for (int s0 = p0; s0 < p1; s0 += 64) {
        const int i = s0 + lane;
        const bool in = i < p1;
        float l[D][N];
#pragma unroll
        for (int k = 0; k < D; k++) {
            const float t = in ? factor * (ys[(long long)k * M + i] - ctr[(long long)box * D + k]) : 0.f;
            basis_1d(t, nt + N * k, nw + N * k, N, l[k], 1.f);
        }
        const float b = in ? bs[i] : 0.f;            // lanes past the end add nothing
        __syncthreads();                             // the previous 64 points have been read by every lane
        // products over a range of dimensions, built dimension by dimension from the last (first one fastest)
        float h[NR], w[Q];
        h[0] = 1.f;
        w[0] = b;
        int len = 1;
#pragma unroll
        for (int k = R - 1; k >= 0; k--) {
#pragma unroll
            for (int j = len - 1; j >= 0; j--)
#pragma unroll
                for (int a = N - 1; a >= 0; a--) h[j * N + a] = h[j] * l[k][a];
            len *= N;
        }
        len = 1;
#pragma unroll
        for (int k = D - 1; k >= R; k--) {
#pragma unroll
            for (int j = len - 1; j >= 0; j--)
#pragma unroll
                for (int a = N - 1; a >= 0; a--) w[j * N + a] = w[j] * l[k][a];
            len *= N;
        }
#pragma unroll
        for (int a = 0; a < NR; a++) sh[NR * lane + a] = h[a];
#pragma unroll
        for (int j = 0; j < Q; j++) sw[QS * lane + j] = w[j];
        __syncthreads();
        if (g < G) {
            for (int pt = 0; pt < PG; pt++) {
                const int pp = PG * g + pt;
                if (pp >= 64) break;
                const float wv = sw[QS * pp + q];
#pragma unroll
                for (int a = 0; a < NR; a++) acc[a] = fmaf(sh[NR * pp + a], wv, acc[a]);
            }
        }
    }
    // add the groups: lanes q, Q + q, 2Q + q, ... hold partial sums of the same nodes
    __syncthreads();
#pragma unroll
    for (int a = 0; a < NR; a++) red[lane * NR + a] = g < G ? acc[a] : 0.f;
    __syncthreads();
    if (lane < Q) {
#pragma unroll
        for (int a = 0; a < NR; a++) {
            float t = 0.f;
            for (int gg = 0; gg < G; gg++) t += red[(gg * Q + lane) * NR + a];
            partial[(long long)blockIdx.x * P + a + NR * lane] = t;
        }
    }
}

__global__ void p2m_reduce_kernel(const float *__restrict__ partial, const int *__restrict__ tileoff, int nb, int P,
                                  float *__restrict__ mom)
{
    long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= (long long)nb * P) return;
    int box = (int)(e / P), m = (int)(e % P);
    float acc = 0.f;
    for (int t = tileoff[box]; t < tileoff[box + 1]; t++) acc += partial[(long long)t * P + m];
    mom[e] = acc;
}

// ------------------------------------------------------------------------------------------------
// M2L, direct form (F3M_src/1_d_conv.cu:741-817): Loc[bx][i] = sum over far y boxes, sum_m
// exp(-|(n_i+c_bx)-(n_m+c_by)|^2 lcs) Mom[by][m].  One workgroup per x box, one lane per node.

template <int D>
__global__ void __launch_bounds__(1024) m2l_direct_kernel(const float *__restrict__ noff, int P, const float *__restrict__ ctrx,
                                                           const float *__restrict__ ctry, const int *__restrict__ pairs,
                                                           const int *__restrict__ rowptr, const float *__restrict__ mom,
                                                           float lcs2, float *__restrict__ loc)
{
    F3M_DYN_SHARED(float, smem);
    float *sy = smem;              // P*D
    float *sm = smem + P * D;      // P
    const int bx = blockIdx.x, tid = threadIdx.x;
    const int m0 = rowptr[bx], m1 = rowptr[bx + 1];
    if (m0 == m1) return;          // uniform over the workgroup
    float x[D], no[D];
#pragma unroll
    for (int k = 0; k < D; k++) {
        no[k] = (tid < P) ? noff[(long long)tid * D + k] : 0.f;
        x[k] = no[k] + ctrx[(long long)bx * D + k];
    }
    float acc = 0.f;
    for (int m = m0; m < m1; m++) {
        const int by = pairs[2 * (long long)m + 1];
        __syncthreads();
        if (tid < P) {
#pragma unroll
            for (int k = 0; k < D; k++) sy[tid * D + k] = no[k] + ctry[(long long)by * D + k];
            sm[tid] = mom[(long long)by * P + tid];
        }
        __syncthreads();
        if (tid < P) {
            for (int j = 0; j < P; j++) {
                float r2 = 0.f;
#pragma unroll
                for (int k = 0; k < D; k++) { float t = x[k] - sy[j * D + k]; r2 = fmaf(t, t, r2); }
                acc = fmaf(fast_exp2(-r2 * lcs2), sm[j], acc);
            }
        }
    }
    if (tid < P) loc[(long long)bx * P + tid] = acc;
}

// ------------------------------------------------------------------------------------------------
// M2L, separable form.  Box centres sit on the regular grid of their depth, so the centre offset of
// a far pair is (integer cell offset)*edge + (origin_y - origin_x), and the Gaussian factorises over
// dimensions: K[(a_0..a_{d-1}),(m_0..m_{d-1})] = prod_j E_j[o_j][a_j][m_j] with
// E_j[o][a][m] = exp(-lcs ((t_a - t_m) edge/2 - (o edge + delta_j))^2).  Applying the d small
// factors one dimension at a time costs sum_j n_j multiply-adds per node and far pair instead of P.
// The tables (a few KB, built on the host in fp64) live in LDS; the moment vector ping-pongs between
// two LDS buffers.  Same sums as m2l_direct_kernel up to rounding.

// kM2LOffsets (f3m_engine.h) = cell offsets per dimension held by the tables; plan creation has checked
// that no far pair lies outside them, the clamps below only keep a table index in bounds whatever happens

struct SepMeta {
    int omin[kMaxD];
    int NT;      // row length of a table (largest per-dimension node count)
};

template <int D>
__global__ void __launch_bounds__(1024) m2l_sep_kernel(const float *__restrict__ tables, int ntab, NodeMeta nm, SepMeta sm,
                                                        const int *__restrict__ cellx, const int *__restrict__ celly,
                                                        const int *__restrict__ pairs, const int *__restrict__ rowptr,
                                                        const float *__restrict__ mom, float *__restrict__ loc)
{
    F3M_DYN_SHARED(float, smem);
    float *tab = smem;                 // ntab
    float *bufA = smem + ntab;         // P
    float *bufB = bufA + nm.P;         // P
    const int bx = blockIdx.x, tid = threadIdx.x, BD = blockDim.x, P = nm.P;
    const int m0 = rowptr[bx], m1 = rowptr[bx + 1];
    if (m0 == m1) return;              // uniform over the workgroup
    for (int e = tid; e < ntab; e += BD) tab[e] = tables[e];
    // digit of this lane's node along every dimension, and the flat index with that digit cleared
    int dig[D], base[D], stride[D];
    {
        int st = 1;
#pragma unroll
        for (int j = 0; j < D; j++) {
            stride[j] = st;
            dig[j] = (tid / st) % nm.n[j];
            base[j] = tid - dig[j] * st;
            st *= nm.n[j];
        }
    }
    int cx[D];
#pragma unroll
    for (int j = 0; j < D; j++) cx[j] = cellx[(long long)bx * D + j] + sm.omin[j];
    const bool live = tid < P;
    float acc = 0.f;
    for (int m = m0; m < m1; m++) {
        const int by = pairs[2 * (long long)m + 1];
        __syncthreads();
        if (live) bufA[tid] = mom[(long long)by * P + tid];
        __syncthreads();
        float *in = bufA, *out = bufB;
#pragma unroll
        for (int j = 0; j < D; j++) {
            int oi = celly[(long long)by * D + j] - cx[j];
            oi = oi < 0 ? 0 : (oi >= kM2LOffsets ? kM2LOffsets - 1 : oi);
            float sum = 0.f;
            if (live) {
                const float *row = tab + ((j * kM2LOffsets + oi) * sm.NT + dig[j]) * sm.NT;
                const float *src = in + base[j];
                for (int q = 0; q < nm.n[j]; q++) sum = fmaf(row[q], src[q * stride[j]], sum);
            }
            if (j == D - 1) {
                acc += sum;
            } else {
                if (live) out[tid] = sum;
                __syncthreads();
                float *t = in; in = out; out = t;
            }
        }
    }
    if (live) loc[(long long)bx * P + tid] = acc;
}

// Separable M2L for the 4 x 4 x 4 node grid (64 nodes, the default), one wavefront per x box, lane =
// node (a0 + 4 a1 + 16 a2).  The far boxes of an x box differ from it by cell offsets (o0, o1, o2).
// Per far box only the first factor is applied (four multiply-adds on values broadcast inside groups of
// four lanes) and the result is added to the LDS slot of its (o1, o2); the second factor is then applied
// once per (o1, o2) slot and the third once per o2, instead of once per far box.  SPAN = number of
// distinct offsets per dimension that can occur: 7 with one tree (-3..3), 10 with two trees.
template <int SPAN>
__global__ void __launch_bounds__(64) m2l_q64_kernel(const float *__restrict__ tables, SepMeta sm, int lo1, int lo2,
                                                      const int *__restrict__ cellx, const int *__restrict__ celly,
                                                      const int *__restrict__ pairs, const int *__restrict__ rowptr,
                                                      const float *__restrict__ mom, float *__restrict__ loc)
{
    constexpr int NTAB = 3 * kM2LOffsets * 16;
    __shared__ __align__(16) float tab[NTAB];
    __shared__ float U[SPAN * SPAN * 64];
    const int bx = blockIdx.x, lane = threadIdx.x;
    const int m0 = rowptr[bx], m1 = rowptr[bx + 1];
    if (m0 == m1) return;
    const int a0 = lane & 3, a1 = (lane >> 2) & 3, a2 = lane >> 4;
    for (int e = lane; e < NTAB; e += 64) tab[e] = tables[e];
    for (int e = lane; e < SPAN * SPAN * 64; e += 64) U[e] = 0.f;
    int cx[3];
#pragma unroll
    for (int j = 0; j < 3; j++) cx[j] = cellx[(long long)bx * 3 + j] + sm.omin[j];
    float extra = 0.f;
    __syncthreads();
    // the far list is consumed 64 boxes at a time: every lane fetches the id and the table indices of one
    // far box, then the wavefront walks through them (four moment vectors in flight at a time)
    for (int mb = m0; mb < m1; mb += 64) {
        const int mi = mb + lane;
        int byv = 0, pk = 0;
        if (mi < m1) {
            byv = pairs[2 * (long long)mi + 1];
            int o0 = celly[(long long)byv * 3 + 0] - cx[0];
            int o1 = celly[(long long)byv * 3 + 1] - cx[1];
            int o2 = celly[(long long)byv * 3 + 2] - cx[2];
            o0 = min(max(o0, 0), kM2LOffsets - 1);
            o1 = min(max(o1, 0), kM2LOffsets - 1);
            o2 = min(max(o2, 0), kM2LOffsets - 1);
            pk = o0 | (o1 << 8) | (o2 << 16);
        }
        const int cnt = min(64, m1 - mb);
        for (int j = 0; j < cnt; j += 4) {
            float v[4];
            int pkj[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int jj = min(j + u, cnt - 1);
                const int by = wave_readlane(byv, jj);
                pkj[u] = wave_readlane(pk, jj);
                v[u] = mom[(long long)by * 64 + lane];
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                if (j + u >= cnt) break;             // uniform over the wavefront
                const int o0 = pkj[u] & 255, o1 = (pkj[u] >> 8) & 255, o2 = pkj[u] >> 16;
                const int g1 = o1 - lo1, g2 = o2 - lo2;
                const float4 r = *reinterpret_cast<const float4 *>(&tab[(0 * kM2LOffsets + o0) * 16 + a0 * 4]);
                float sacc = r.x * quad_bcast<0>(v[u]);
                sacc = fmaf(r.y, quad_bcast<1>(v[u]), sacc);
                sacc = fmaf(r.z, quad_bcast<2>(v[u]), sacc);
                sacc = fmaf(r.w, quad_bcast<3>(v[u]), sacc);
                if (g1 >= 0 && g1 < SPAN && g2 >= 0 && g2 < SPAN) {
                    U[(g1 * SPAN + g2) * 64 + lane] += sacc;
                } else {
                    // An offset outside the expected span (a parent pair that sat exactly on the far
                    // threshold and was decided by rounding): apply the other two factors directly.
                    const float4 r1 = *reinterpret_cast<const float4 *>(&tab[(1 * kM2LOffsets + o1) * 16 + a1 * 4]);
                    float t = r1.x * wave_shfl_f(sacc, (lane & ~12) | 0);
                    t = fmaf(r1.y, wave_shfl_f(sacc, (lane & ~12) | 4), t);
                    t = fmaf(r1.z, wave_shfl_f(sacc, (lane & ~12) | 8), t);
                    t = fmaf(r1.w, wave_shfl_f(sacc, (lane & ~12) | 12), t);
                    const float4 r2 = *reinterpret_cast<const float4 *>(&tab[(2 * kM2LOffsets + o2) * 16 + a2 * 4]);
                    extra = fmaf(r2.x, wave_shfl_f(t, (lane & 15) | 0), extra);
                    extra = fmaf(r2.y, wave_shfl_f(t, (lane & 15) | 16), extra);
                    extra = fmaf(r2.z, wave_shfl_f(t, (lane & 15) | 32), extra);
                    extra = fmaf(r2.w, wave_shfl_f(t, (lane & 15) | 48), extra);
                }
            }
        }
    }
    __syncthreads();
    // second factor: per (o1, o2) slot; lanes that differ in a1 exchange values
    float V[SPAN];
#pragma unroll
    for (int g2 = 0; g2 < SPAN; g2++) V[g2] = 0.f;
    for (int g1 = 0; g1 < SPAN; g1++) {
        const int o1 = min(lo1 + g1, kM2LOffsets - 1);
        const float4 r = *reinterpret_cast<const float4 *>(&tab[(1 * kM2LOffsets + o1) * 16 + a1 * 4]);
#pragma unroll
        for (int g2 = 0; g2 < SPAN; g2++) {
            const float u = U[(g1 * SPAN + g2) * 64 + lane];
            float t = V[g2];
            t = fmaf(r.x, wave_shfl_f(u, (lane & ~12) | 0), t);
            t = fmaf(r.y, wave_shfl_f(u, (lane & ~12) | 4), t);
            t = fmaf(r.z, wave_shfl_f(u, (lane & ~12) | 8), t);
            t = fmaf(r.w, wave_shfl_f(u, (lane & ~12) | 12), t);
            V[g2] = t;
        }
    }
    // third factor: per o2; lanes that differ in a2 exchange values
    float out = 0.f;
#pragma unroll
    for (int g2 = 0; g2 < SPAN; g2++) {
        const int o2 = min(lo2 + g2, kM2LOffsets - 1);
        const float4 r = *reinterpret_cast<const float4 *>(&tab[(2 * kM2LOffsets + o2) * 16 + a2 * 4]);
        out = fmaf(r.x, wave_shfl_f(V[g2], (lane & 15) | 0), out);
        out = fmaf(r.y, wave_shfl_f(V[g2], (lane & 15) | 16), out);
        out = fmaf(r.z, wave_shfl_f(V[g2], (lane & 15) | 32), out);
        out = fmaf(r.w, wave_shfl_f(V[g2], (lane & 15) | 48), out);
    }
    loc[(long long)bx * 64 + lane] = out + extra;
}

// ------------------------------------------------------------------------------------------------
// Separable M2L for d >= 3, one tree, one workgroup per PARENT box (or per group of GS of its 2^d
// children when they do not all fit): the children ("siblings") of a box have almost the same far
// boxes -- the children of the 3^d parents around their parent, 6^d cells, minus each sibling's own
// neighbours -- so a moment vector is fetched once per workgroup and used by every sibling.
//
// Phase A writes the far rows of the siblings into a direct-address table in LDS, indexed by the cell
// offset u = cell_y - 2 cell_parent in -2..3 per dimension (dimension 0 fastest), with a bit mask of
// the siblings that list the box.  A parent pair two cells apart along one axis sits exactly on the
// far threshold (distance = 2 edges) and fp32 rounding decides it; where it was kept, its children
// appear in the far rows with u = -4, -3, 4 or 5 along that axis and 0 or 1 elsewhere.  Those cells
// have a small table of their own.  Phase B walks each table in lexicographic order of the offsets,
// last dimension outermost.  Lane (sibling, r2) owns the n0 x n1 nodes (a0, a1, r2) of one sibling:
//   * per far box: factor 0 in registers (n0^2 n1 multiply-adds on the freshly loaded moments);
//   * when the offsets of dimensions >= 1 change: factor 1 in registers;
//   * when the offsets of dimensions >= j change (j >= 2): factor j, exchanging values between lanes
//     through LDS.
// So every factor beyond the first is applied once per group of far boxes that share the remaining
// offsets instead of once per far box.  The per-sibling offset is u - (child bit), which shifts
// every sibling's offsets by a constant and therefore leaves the walking order valid for all of them.
// Preconditions (checked by the host): n0 = n1 = N, every far pair in one of the two tables.

constexpr int kSibSpan = 6;
__host__ __device__ constexpr int sib_codes(int d) { return d == 0 ? 1 : kSibSpan * sib_codes(d - 1); }
__host__ __device__ constexpr int sib_ext_codes(int d) { return d * 4 * (1 << (d - 1)); }

// table position of a far box from its cell offsets relative to twice the parent's cell, shifted by
// 2 (so the regular range is 0..5): >= 0 regular table, -2 - e extension table entry e, -1 neither
template <int D>
__host__ __device__ inline int sib_code(const int *dg)
{
    int code = 0, mul = 1, nout = 0, jj = 0;
    for (int j = 0; j < D; j++) {
        if (dg[j] < 0 || dg[j] >= kSibSpan) { nout++; jj = j; }
        code += dg[j] * mul;
        mul *= kSibSpan;
    }
    if (nout == 0) return code;
    if (nout > 1) return -1;
    const int w = dg[jj];
    const int v = w == -2 ? 0 : w == -1 ? 1 : w == 6 ? 2 : w == 7 ? 3 : -1;
    if (v < 0) return -1;
    int bits = 0, pos = 0;
    for (int j = 0; j < D; j++) {
        if (j == jj) continue;
        if (dg[j] != 2 && dg[j] != 3) return -1;
        bits |= (dg[j] - 2) << pos;
        pos++;
    }
    return -2 - ((jj * 4 + v) * (1 << (D - 1)) + bits);
}

template <int D>
__device__ inline void sib_ext_digits(int e, int *dg)
{
    constexpr int H = 1 << (D - 1);
    const int jj = e / (4 * H), v = (e / H) % 4, bits = e % H;
    int pos = 0;
#pragma unroll
    for (int j = 0; j < D; j++) {
        if (j == jj) { dg[j] = v == 0 ? -2 : v == 1 ? -1 : v == 2 ? 6 : 7; }
        else { dg[j] = 2 + ((bits >> pos) & 1); pos++; }
    }
}

// Parents ordered by the number of far pairs of their children, longest first, in 256 classes of
// `unit` pairs (one counting pass; the order inside a class is whatever the atomics give, which does not
// touch the results: a workgroup's sums do not depend on when it runs).
__global__ void sib_class_count_kernel(const int *__restrict__ childstart, const int *__restrict__ rowptr, int npar, int unit,
                                       int *__restrict__ cls, int *__restrict__ hist)
{
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= npar) return;
    const int cnt = rowptr[childstart[p + 1]] - rowptr[childstart[p]];
    const int c = 255 - min(255, cnt / unit);
    cls[p] = c;
    atomicAdd(&hist[c], 1);
}
// MAXT: the largest workgroup the instance is launched with.  It sets the registers a lane may use: 128 under the
// general bound of 1024 threads, which a lane's 3 N^2 partial sums and its moments in flight exceed by far at 5 or 6
// nodes per dimension; those grids (3-D only, workgroups of one wavefront) have instances bound to 64 threads.
template <int D, int N, int H, int MAXT>
__global__ void __launch_bounds__(MAXT) m2l_sib_kernel(const float *__restrict__ tables, int ntab, SepMeta sm, NodeMeta nm,
                                                        int R2, int GS, int nsub, int npass, const int *__restrict__ order,
                                                        const int *__restrict__ childstart,
                                                        const int *__restrict__ cell, const int *__restrict__ pairs,
                                                        const int *__restrict__ rowptr, const float *__restrict__ mom,
                                                        float *__restrict__ loc, const unsigned char *__restrict__ taken)
{
    // taken (nullable): one byte per parent and regular table cell, set for the cells that m2l_shared_kernel has summed
    // already (its results are in loc; this kernel then leaves those cells out and adds to loc)
    // H = 2: the n0 x n1 nodes of a lane are shared by two lanes, n1/2 values of a1 each (a workgroup of
    // 2^D siblings x R2 lanes would otherwise fill half a wavefront in 3-D); NN = nodes of a lane
    // W: row length of the padded tables of the first two factors (rows are read as vectors of four)
    constexpr int NCODE = sib_codes(D), NEXT = sib_ext_codes(D), NN = N * N / H, NQ1 = N / H, NB = N <= 3 ? 4 : (D >= 4 ? 1 : 2);
    constexpr int W = N <= 4 ? 4 : 8;
    static_assert(H == 1 || (H == 2 && N % 2 == 0), "the nodes of dimension 1 are split in halves");
    F3M_DYN_SHARED(float, smem);
    // (every lambda below is forced inline: a call would take the partial sums, which are indexed by constants
    // everywhere, out of the registers)
    const int tid = threadIdx.x, BD = blockDim.x, lane = tid & 63;
    // The regular table is filled and walked in npass parts (slabs of the last dimension, which is the
    // outermost of the walk), so that it takes NCODE / npass cells of LDS (the host asks for more than
    // one part only where the whole table does not fit).
    const int chunk = NCODE / npass;
    int *tby = reinterpret_cast<int *>(smem);                       // chunk: y box of a table cell
    unsigned *tmask = reinterpret_cast<unsigned *>(smem) + chunk;   // chunk: siblings that list it
    int *xby = reinterpret_cast<int *>(smem) + 2 * chunk;           // NEXT: the same for the extension cells
    unsigned *xmask = reinterpret_cast<unsigned *>(smem) + 2 * chunk + NEXT;
    int *xord = reinterpret_cast<int *>(smem) + 2 * chunk + 2 * NEXT;   // NEXT: extension cells in walking order
    int *xkey = xord + NEXT;                                        // NEXT
    float *xbuf = smem + 2 * chunk + 4 * NEXT;                      // NN * BD: exchange buffer
    float *tabg = xbuf + NN * BD;                                   // ntab: E_j[o][a][q], row length sm.NT
    float *tab01 = tabg + ((ntab + 3) & ~3);                        // 2 * 13 * N rows of W: E_0, E_1 padded
    float *zrow = tab01 + 2 * kM2LOffsets * N * W;                  // N rows of zeros
    int *sib = reinterpret_cast<int *>(zrow + N * W);               // GS: compact id of each sibling or -1
    // order (nullable): the parents sorted by the length of their far rows, longest first, so that the
    // workgroups that run longest start first
    const int px = order ? order[blockIdx.x / nsub] : blockIdx.x / nsub, sg = blockIdx.x % nsub;
    const int P = nm.P;

    for (int e = tid; e < NEXT; e += BD) {
        xby[e] = 0; xmask[e] = 0u;
        int dg[D], key = 0, mul = 1;
        sib_ext_digits<D>(e, dg);
#pragma unroll
        for (int j = 0; j < D; j++) { key += (dg[j] + 2) * mul; mul *= 10; }
        xkey[e] = key;
    }
    for (int e = tid; e < ntab; e += BD) tabg[e] = tables[e];
    for (int e = tid; e < 2 * kM2LOffsets * N * W; e += BD) {
        const int q = e % W, a = (e / W) % N, o = (e / (W * N)) % kM2LOffsets, j = e / (W * N * kM2LOffsets);
        tab01[e] = q < N ? tables[((j * kM2LOffsets + o) * sm.NT + a) * sm.NT + q] : 0.f;
    }
    for (int e = tid; e < N * W; e += BD) zrow[e] = 0.f;
    if (tid < GS) sib[tid] = -1;
    __syncthreads();
    for (int e = tid; e < NEXT; e += BD) {                 // walking order of the extension cells
        const int key = xkey[e];
        int rank = 0;
        for (int f = 0; f < NEXT; f++) rank += xkey[f] < key;
        xord[rank] = e;
    }
    const int c0 = childstart[px], c1 = childstart[px + 1];
    for (int c = c0 + tid; c < c1; c += BD) {
        int code = 0;
#pragma unroll
        for (int j = 0; j < D; j++) code |= (cell[(long long)c * D + j] & 1) << j;
        const int sl = code - sg * GS;
        if (sl >= 0 && sl < GS) sib[sl] = c;
    }
    int pc[D];
#pragma unroll
    for (int j = 0; j < D; j++) pc[j] = 2 * (cell[(long long)c0 * D + j] >> 1) - 2;
    __syncthreads();
    // fills part `pass` of the regular table (and, with part 0, the extension table) from the far rows
    auto fill_tables = [&](int pass) __attribute__((always_inline)) {
        for (int e = tid; e < chunk; e += BD) { tby[e] = 0; tmask[e] = 0u; }
        __syncthreads();
        for (int s2 = 0; s2 < GS; s2++) {
            const int bx = sib[s2];
            if (bx < 0) continue;                          // uniform over the workgroup
            const int m1 = rowptr[bx + 1];
            for (int m = rowptr[bx] + tid; m < m1; m += BD) {
                const int by = pairs[2 * (long long)m + 1];
                int dg[D];
#pragma unroll
                for (int j = 0; j < D; j++) dg[j] = cell[(long long)by * D + j] - pc[j];
                const int code = sib_code<D>(dg);
                if (code >= 0) {
                    const int c = code - pass * chunk;
                    if (c >= 0 && c < chunk && !(taken != nullptr && taken[(long long)px * NCODE + code])) {
                        tby[c] = by;
                        atomicOr(&tmask[c], 1u << s2);
                    }
                } else if (code <= -2 && pass == 0) { xby[-2 - code] = by; atomicOr(&xmask[-2 - code], 1u << s2); }
            }
        }
        __syncthreads();
    };

    // This lane: sibling sl, position r2 among the nodes of dimensions >= 2.  The siblings are the fast
    // index: the GS lanes of one r2 read the same moments, so a wavefront's load touches 64/GS short
    // runs of memory instead of 64 (the moment loads are what the level-1 cache has to carry here).
    const int sl = tid % GS, r2h = tid / GS;               // r2h = r2 * H + h: half h of the a1 range
    const bool valid = r2h < R2;                           // lanes past the last node only keep step
    const int r2 = r2h / H, h = r2h % H;
    const int mybox = valid ? sib[sl] : -1;
    const bool live = mybox >= 0;
    int cbit[D], dig[D], lstride[D];
    {
        const int code = sg * GS + sl;
        int rem = valid ? r2 : 0, st = GS * H;
#pragma unroll
        for (int j = 0; j < D; j++) {
            cbit[j] = 4 + ((code >> j) & 1) + sm.omin[j];  // table index of dimension j = (digit_j + 2) - cbit[j]
            dig[j] = 0; lstride[j] = 0;
            if (j >= 2) { dig[j] = rem % nm.n[j]; rem /= nm.n[j]; lstride[j] = st; st *= nm.n[j]; }   // lstride: in lanes
        }
    }
    const float *mine = mom + (long long)NN * (live ? r2h : 0);

    // the NN moments of a lane, four floats per load (a copy of the whole vector as one object keeps large ones out
    // of registers)
    auto load_moments = [](const float *src, fvec<NN> &v) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i + 4 <= NN; i += 4) {
            const fvec<4> t = *reinterpret_cast<const fvec<4> *>(src + i);
#pragma unroll
            for (int e = 0; e < 4; e++) v.v[i + e] = t.v[e];
        }
#pragma unroll
        for (int i = NN & ~3; i < NN; i++) v.v[i] = src[i];
    };
    // one padded table row
    auto load_row = [](const float *row, float (&ev)[W]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < W; u += 4) {
            const float4 e = *reinterpret_cast<const float4 *>(row + u);
            ev[u] = e.x; ev[u + 1] = e.y; ev[u + 2] = e.z; ev[u + 3] = e.w;
        }
    };
    float acc[D][NN];
#pragma unroll
    for (int j = 0; j < D; j++)
#pragma unroll
        for (int i = 0; i < NN; i++) acc[j][i] = 0.f;
    // The digits of a far cell travel as one word, four bits each, biased by 2 (extension cells reach
    // -2): the walk is the same in every wavefront, so whatever it costs in scalar instructions per far
    // box is paid by each of them on the compute unit's one scalar unit.
    int curpk = 0;
    bool have = false;
    auto digit2 = [](int pk, int j) __attribute__((always_inline)) { return (pk >> (4 * j)) & 15; };      // digit j + 2

    // applies factor l+1 to acc[l], adds the result to acc[l+1] and clears acc[l]
    auto flush = [&](auto level) __attribute__((always_inline)) {
        constexpr int l = decltype(level)::value, j = l + 1;
        if constexpr (j == 1) {
            int oi = digit2(curpk, 1) - cbit[1];
            oi = min(max(oi, 0), kM2LOffsets - 1);
            const float *T1 = tab01 + ((kM2LOffsets + oi) * N) * W;
            if constexpr (H == 1) {
#pragma unroll
                for (int a1 = 0; a1 < N; a1++) {
                    float ev[W];
                    load_row(T1 + a1 * W, ev);
#pragma unroll
                    for (int a0 = 0; a0 < N; a0++) {
                        float t = acc[1][a0 + N * a1];
#pragma unroll
                        for (int q = 0; q < N; q++) t = fmaf(ev[q], acc[0][a0 + N * q], t);
                        acc[1][a0 + N * a1] = t;
                    }
                }
            } else {
                // this lane holds the q1 of its half: partial sums for every a1, then the half of them that
                // belongs to the partner lane (GS lanes away) is traded for the partner's
                float part[N * N];
#pragma unroll
                for (int a1 = 0; a1 < N; a1++) {
                    float ev[W];
                    load_row(T1 + a1 * W, ev);
#pragma unroll
                    for (int a0 = 0; a0 < N; a0++) {
                        float t = 0.f;
#pragma unroll
                        for (int q = 0; q < NQ1; q++) t = fmaf(h ? ev[NQ1 + q] : ev[q], acc[0][a0 + N * q], t);
                        part[a0 + N * a1] = t;
                    }
                }
#pragma unroll
                for (int a1 = 0; a1 < NQ1; a1++)
#pragma unroll
                    for (int a0 = 0; a0 < N; a0++) {
                        const float lo = part[a0 + N * a1], hi = part[a0 + N * (NQ1 + a1)];
                        const float got = wave_shfl_xor_f(h ? lo : hi, GS);       // what the partner summed for my a1
                        acc[1][a0 + N * a1] += (h ? hi : lo) + got;
                    }
            }
        } else {
            __syncthreads();
#pragma unroll
            for (int i = 0; i < NN; i++) xbuf[i * BD + tid] = acc[l][i];
            __syncthreads();
            if (valid) {
                int oi = digit2(curpk, j) - cbit[j];
                oi = min(max(oi, 0), kM2LOffsets - 1);
                const float *row = tabg + ((j * kM2LOffsets + oi) * sm.NT + dig[j]) * sm.NT;
                for (int q = 0; q < nm.n[j]; q++) {
                    const float w = row[q];
                    const float *src = xbuf + tid + (q - dig[j]) * lstride[j];
#pragma unroll
                    for (int i = 0; i < NN; i++) acc[j][i] = fmaf(w, src[i * BD], acc[j][i]);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < NN; i++) acc[l][i] = 0.f;
    };
    auto flush_upto = [&](int jt) __attribute__((always_inline)) {       // levels 0 .. jt-1, jt uniform over the workgroup
        if (jt > 0) flush(std::integral_constant<int, 0>());
        if constexpr (D > 2) { if (jt > 1) flush(std::integral_constant<int, 1>()); }
        if constexpr (D > 3) { if (jt > 2) flush(std::integral_constant<int, 2>()); }
        if constexpr (D > 4) { if (jt > 3) flush(std::integral_constant<int, 3>()); }
    };
    // one far box: pk = its packed digits (uniform), v = its moments at this lane's nodes
    auto far_box = [&](int pk, unsigned smask, const fvec<NN> &v) __attribute__((always_inline)) {
        if (have) {
            const int diff = (pk ^ curpk) >> 4;             // digits 1.. that change
            flush_upto(diff ? (31 - __builtin_clz(diff)) / 4 + 1 : 0);   // up to the highest of them
        }
        curpk = pk;
        have = true;
        const bool part = live && ((smask >> sl) & 1u);
        int oi = digit2(pk, 0) - cbit[0];
        oi = min(max(oi, 0), kM2LOffsets - 1);
        const float *T0 = part ? tab01 + (oi * N) * W : zrow;
#pragma unroll
        for (int a0 = 0; a0 < N; a0++) {
            float ev[W];
            load_row(T0 + a0 * W, ev);
#pragma unroll
            for (int q1 = 0; q1 < NQ1; q1++) {
                float t = acc[0][a0 + N * q1];
#pragma unroll
                for (int q = 0; q < N; q++) t = fmaf(ev[q], v.v[q + N * q1], t);
                acc[0][a0 + N * q1] = t;
            }
        }
    };
    // walks 64 table cells: ml, byl = this lane's cell; cellid = its id (regular code or extension entry)
    auto walk64 = [&](unsigned ml, int byl, int cellid, auto ext) __attribute__((always_inline)) {
        int pkl = 0;                                       // packed digits of this lane's cell
        {
            int dg[D];
            if constexpr (decltype(ext)::value) {
                sib_ext_digits<D>(cellid, dg);
            } else {
                int rem = cellid;
#pragma unroll
                for (int j = 0; j < D; j++) { dg[j] = rem % kSibSpan; rem /= kSibSpan; }
            }
#pragma unroll
            for (int j = 0; j < D; j++) pkl |= (dg[j] + 2) << (4 * j);
        }
        unsigned long long bal = wave_ballot(ml != 0u);
        while (bal) {                                      // identical in every wavefront of the workgroup
            int ls[NB], cnt = 0;
            fvec<NN> v[NB];
#pragma unroll
            for (int u = 0; u < NB; u++) {
                ls[u] = 0;
                if (bal) { ls[u] = __ffsll(bal) - 1; bal &= bal - 1; cnt++; }
                const int by = wave_readlane(byl, ls[u]);
                load_moments(mine + (long long)by * P, v[u]);
            }
#pragma unroll
            for (int u = 0; u < NB; u++) {
                if (u >= cnt) break;                       // uniform
                const unsigned smask = (unsigned)wave_readlane((int)ml, ls[u]);
                far_box(wave_readlane(pkl, ls[u]), smask, v[u]);
            }
        }
    };

    for (int pass = 0; pass < npass; pass++) {
        if (pass > 0) __syncthreads();                     // every wavefront is done with the previous part
        fill_tables(pass);
        for (int base = 0; base < chunk; base += 64) {
            const int idx = base + lane;
            walk64(idx < chunk ? tmask[idx] : 0u, idx < chunk ? tby[idx] : 0, pass * chunk + idx, std::false_type());
        }
    }
    if (have) flush_upto(D - 1);
    have = false;
    for (int base = 0; base < NEXT; base += 64) {
        const int r = base + lane;
        const int e = r < NEXT ? xord[r] : 0;
        walk64(r < NEXT ? xmask[e] : 0u, xby[e], e, std::true_type());
    }
    if (have) flush_upto(D - 1);
    if (live) {
        float *dst = loc + (long long)mybox * P + (long long)NN * r2h;
        if (taken != nullptr) {
#pragma unroll
            for (int i = 0; i < NN; i++) dst[i] += acc[D - 1][i];
            return;
        }
#pragma unroll
        for (int i = 0; i + 4 <= NN; i += 4) {
            fvec<4> r;
#pragma unroll
            for (int e = 0; e < 4; e++) r.v[e] = acc[D - 1][i + e];
            *reinterpret_cast<fvec<4> *>(dst + i) = r;
        }
#pragma unroll
        for (int i = NN & ~3; i < NN; i++) dst[i] = acc[D - 1][i];
    }
}

// ------------------------------------------------------------------------------------------------
// Sibling-group M2L, the far cells that EVERY child of a parent lists (most of them: all cells that are not next to the
// parent's own block of children).  For such a cell the 2^D siblings differ only in the tables they apply, and the
// table of dimension j depends on the sibling's bit j alone: E_j[u_j - b_j].  So the sums are formed once per
// combination of bits seen so far, not once per sibling: after factor 0 there are two variants (b0), after factor 1
// four (b0, b1), ... and only after the last factor one per sibling.  Lane (b0, c1, .., c_{D-1}) holds, for its b0 and
// its position c_j among the nodes of dimensions >= 1, the N values over the nodes of dimension 0 of every variant
// (b1..bj) of level j: N (2^D - 1) partial sums in registers.  Per far box a lane loads N moments and does N^2
// multiply-adds, where m2l_sib_kernel spends N^2 n1 multiply-adds in each of 2^D siblings' lanes; factor j+1 is applied
// when the offsets of dimensions > j change, with the values exchanged through LDS between the lanes that differ in
// c_{j+1}.  One workgroup per parent, 2 N^(D-1) lanes.  The cells taken are flagged in `taken` (one byte per parent and
// cell) for m2l_sib_kernel, which runs afterwards on the rest -- cells next to the parent's block, cells of the
// extension table -- and adds to loc.  Same sums up to rounding.  Preconditions: N nodes in every dimension, one
// tree, every far pair inside the tables (as for m2l_sib_kernel).
__host__ __device__ constexpr int ipow_c(int b, int e) { return e == 0 ? 1 : b * ipow_c(b, e - 1); }

template <int D, int N>
__global__ void __launch_bounds__(256) m2l_shared_kernel(const float *__restrict__ tables, int ntab, SepMeta sm, int P, int npass,
                                                          const int *__restrict__ order, const int *__restrict__ childstart,
                                                          const int *__restrict__ cell, const int *__restrict__ pairs,
                                                          const int *__restrict__ rowptr, const float *__restrict__ mom,
                                                          float *__restrict__ loc, unsigned char *__restrict__ taken)
{
    constexpr int NCODE = sib_codes(D), NSIB = 1 << D, R = ipow_c(N, D - 1), LANES = 2 * R, NB = 8;
    constexpr int XV = N << (D - 2);                                // most values a lane hands over in one exchange
    constexpr int NACC = N * (NSIB - 1);                            // level j: 2^j variants of N values, from N (2^j - 1) on
    F3M_DYN_SHARED(float, smem);
    const int tid = threadIdx.x, BD = blockDim.x, lane = tid & 63;
    const int chunk = NCODE / npass;
    // chunk: y box of a table cell (below 2^24, checked by the host) + 2^24 times the number of siblings that list it
    // while the table is filled, then the box of a cell that is taken or -1
    int *tby = reinterpret_cast<int *>(smem);
    float *xbuf = smem + chunk;                                     // XV * BD: exchange buffer
    float *tabg = xbuf + XV * BD;                                   // ntab: E_j[o][a][q], row length sm.NT
    int *sib = reinterpret_cast<int *>(tabg + ((ntab + 3) & ~3));   // NSIB: box of each sibling or -1
    const int px = order ? order[blockIdx.x] : blockIdx.x;
    unsigned char *tk = taken + (long long)px * NCODE;

    for (int e = tid; e < ntab; e += BD) tabg[e] = tables[e];
    if (tid < NSIB) sib[tid] = -1;
    __syncthreads();
    const int c0 = childstart[px], c1 = childstart[px + 1];
    for (int c = c0 + tid; c < c1; c += BD) {
        int code = 0;
#pragma unroll
        for (int j = 0; j < D; j++) code |= (cell[(long long)c * D + j] & 1) << j;
        sib[code] = c;
    }
    int pc[D];
#pragma unroll
    for (int j = 0; j < D; j++) pc[j] = 2 * (cell[(long long)c0 * D + j] >> 1) - 2;
    __syncthreads();
    int nlive = 0;
    for (int s2 = 0; s2 < NSIB; s2++) nlive += sib[s2] >= 0 ? 1 : 0;

    // part `pass` of the table from the far rows of every sibling; then only the cells that every sibling lists stay
    auto fill_tables = [&](int pass) __attribute__((always_inline)) {
        for (int e = tid; e < chunk; e += BD) tby[e] = 0;
        __syncthreads();
        for (int s2 = 0; s2 < NSIB; s2++) {
            const int bx = sib[s2];
            if (bx < 0) continue;                          // uniform over the workgroup
            const int m1 = rowptr[bx + 1];
            for (int m = rowptr[bx] + tid; m < m1; m += BD) {
                const int by = pairs[2 * (long long)m + 1];
                int dg[D];
#pragma unroll
                for (int j = 0; j < D; j++) dg[j] = cell[(long long)by * D + j] - pc[j];
                const int code = sib_code<D>(dg);
                const int c = code - pass * chunk;
                if (code >= 0 && c >= 0 && c < chunk) { atomicOr(&tby[c], by); atomicAdd(&tby[c], 1 << 24); }
            }
        }
        __syncthreads();
        for (int e = tid; e < chunk; e += BD) {
            const int w = tby[e];
            const bool full = (w >> 24) == nlive;
            tby[e] = full ? (w & 0xffffff) : -1;
            tk[pass * chunk + e] = full ? 1 : 0;
        }
        __syncthreads();
    };

    // this lane: bit 0 of its siblings, and its position among the nodes of dimensions >= 1
    const bool valid = tid < LANES;
    const int b0 = tid & 1, cidx = valid ? tid >> 1 : 0;
    int cj[D], lstride[D];
    {
        int rem = cidx, st = 2;
        cj[0] = 0; lstride[0] = 0;
#pragma unroll
        for (int j = 1; j < D; j++) { cj[j] = rem % N; rem /= N; lstride[j] = st; st *= N; }     // lstride: in lanes
    }
    const float *mine = mom + (long long)N * cidx;
    float acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; i++) acc[i] = 0.f;
    int curpk = 0;
    bool have = false;
    auto digit2 = [](int pk, int j) __attribute__((always_inline)) { return (pk >> (4 * j)) & 15; };      // digit j + 2
    // table row E_j[o][a][.] for the offset of the current far cell in dimension j and a sibling with bit b
    auto table_row = [&](int pk, int j, int b, int a) __attribute__((always_inline)) {
        int oi = digit2(pk, j) - (4 + b + sm.omin[j]);
        oi = min(max(oi, 0), kM2LOffsets - 1);
        return tabg + ((j * kM2LOffsets + oi) * sm.NT + a) * sm.NT;
    };
    // applies factor l+1 to the 2^l variants of level l, adds the results to the 2^(l+1) variants of level l+1 and
    // clears level l
    auto flush = [&](auto level) __attribute__((always_inline)) {
        constexpr int l = decltype(level)::value, j = l + 1, NV = 1 << l, src0 = N * (NV - 1), dst0 = N * (2 * NV - 1);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < N * NV; i++) xbuf[i * BD + tid] = acc[src0 + i];
        __syncthreads();
        if (valid) {
#pragma unroll
            for (int b = 0; b < 2; b++) {
                const float *row = table_row(curpk, j, b, cj[j]);
                for (int q = 0; q < N; q++) {
                    const float w = row[q];
                    const float *src = xbuf + tid + (q - cj[j]) * lstride[j];
#pragma unroll
                    for (int i = 0; i < N * NV; i++)
                        acc[dst0 + N * NV * b + i] = fmaf(w, src[i * BD], acc[dst0 + N * NV * b + i]);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < N * NV; i++) acc[src0 + i] = 0.f;
    };
    auto flush_upto = [&](int jt) __attribute__((always_inline)) {       // levels 0 .. jt-1, jt uniform over the workgroup
        if (jt > 0) flush(std::integral_constant<int, 0>());
        if constexpr (D > 2) { if (jt > 1) flush(std::integral_constant<int, 1>()); }
        if constexpr (D > 3) { if (jt > 2) flush(std::integral_constant<int, 2>()); }
        if constexpr (D > 4) { if (jt > 3) flush(std::integral_constant<int, 3>()); }
    };
    // one far box: pk = its packed digits (uniform), v = its moments at this lane's nodes of dimension 0
    auto far_box = [&](int pk, const float (&v)[N]) __attribute__((always_inline)) {
        if (have) {
            const int diff = (pk ^ curpk) >> 4;             // digits 1.. that change
            flush_upto(diff ? (31 - __builtin_clz(diff)) / 4 + 1 : 0);   // up to the highest of them
        }
        curpk = pk;
        have = true;
#pragma unroll
        for (int a0 = 0; a0 < N; a0++) {
            const float *row = table_row(pk, 0, b0, a0);
#pragma unroll
            for (int q = 0; q < N; q++) acc[a0] = fmaf(row[q], v[q], acc[a0]);
        }
    };

    for (int pass = 0; pass < npass; pass++) {
        if (pass > 0) __syncthreads();                     // every wavefront is done with the previous part
        fill_tables(pass);
        for (int base = 0; base < chunk; base += 64) {
            const int idx = base + lane;
            const int byl = idx < chunk ? tby[idx] : -1;
            int pkl = 0;                                   // packed digits of this lane's cell
            {
                int rem = pass * chunk + idx;
#pragma unroll
                for (int j = 0; j < D; j++) { pkl |= (rem % kSibSpan + 2) << (4 * j); rem /= kSibSpan; }
            }
            unsigned long long bal = wave_ballot(byl >= 0);
            while (bal) {                                  // identical in every wavefront of the workgroup
                int ls[NB], cnt = 0;
                float v[NB][N];
#pragma unroll
                for (int u = 0; u < NB; u++) {
                    ls[u] = 0;
                    if (bal) { ls[u] = __ffsll(bal) - 1; bal &= bal - 1; cnt++; }
                    // (past the last cell of this round the loads repeat box 0: lane 0's cell may be one not taken, -1)
                    const int by = u < cnt ? wave_readlane(byl, ls[u]) : 0;
#pragma unroll
                    for (int q = 0; q < N; q++) v[u][q] = mine[(long long)by * P + q];
                }
#pragma unroll
                for (int u = 0; u < NB; u++) {
                    if (u >= cnt) break;                   // uniform
                    far_box(wave_readlane(pkl, ls[u]), v[u]);
                }
            }
        }
    }
    if (have) flush_upto(D - 1);
    if (valid) {
        constexpr int last0 = N * ((1 << (D - 1)) - 1);
#pragma unroll
        for (int var = 0; var < (1 << (D - 1)); var++) {
            const int bx = sib[b0 | (var << 1)];
            if (bx < 0) continue;
            float *dst = loc + (long long)bx * P + (long long)N * cidx;
#pragma unroll
            for (int a0 = 0; a0 < N; a0++) dst[a0] = acc[last0 + N * var + a0];
        }
    }
}

// ------------------------------------------------------------------------------------------------
// L2P (F3M_src/1_d_conv.cu:554-659): out_i += sum_m L_m(x_i) Loc[box][m].  One lane per point; the
// product over dimensions >= 1 is reused along dimension 0.

constexpr int kL2PBlock = 128;

template <int D>
__global__ void __launch_bounds__(kL2PBlock) l2p_kernel(const float *__restrict__ xs, long long N, float *__restrict__ outs,
                                                         const int *__restrict__ off, const float *__restrict__ ctr,
                                                         const int *__restrict__ tileoff, int nb, NodeMeta nm,
                                                         const float *__restrict__ nt, const float *__restrict__ nw,
                                                         float factor, const float *__restrict__ loc, DirectOut dout)
{
    F3M_DYN_SHARED(float, smem);
    const int S1p = nm.S1 | 1;               // odd stride: lanes hit distinct LDS banks
    float *snt = smem;
    float *snw = smem + nm.S1;
    float *sloc = smem + 2 * nm.S1;          // P
    float *sl = sloc + nm.P;                 // kL2PBlock * S1p
    const int tid = threadIdx.x;
    if ((int)blockIdx.x >= tileoff[nb]) return;     // launched with an upper bound of the chunk count
    const int box = find_box(tileoff, nb, blockIdx.x);
    const int chunk = blockIdx.x - tileoff[box];
    const int i = off[box] + chunk * kL2PBlock + tid;
    const bool live = i < off[box + 1];
    for (int a = tid; a < nm.S1; a += kL2PBlock) { snt[a] = nt[a]; snw[a] = nw[a]; }
    for (int m = tid; m < nm.P; m += kL2PBlock) sloc[m] = loc[(long long)box * nm.P + m];
    __syncthreads();
    if (!live) return;
    float *mine = sl + tid * S1p;
#pragma unroll
    for (int k = 0; k < D; k++) {
        float t = factor * (xs[(long long)k * N + i] - ctr[(long long)box * D + k]);
        basis_1d(t, snt + nm.start[k], snw + nm.start[k], nm.n[k], mine + nm.start[k], 1.f);
    }
    int idx[D];
#pragma unroll
    for (int k = 0; k < D; k++) idx[k] = 0;
    float acc = 0.f;
    const int n0 = nm.n[0];
    for (int m = 0; m < nm.P; m += n0) {
        float hi = 1.f;
#pragma unroll
        for (int k = 1; k < D; k++) hi *= mine[nm.start[k] + idx[k]];
        float inner = 0.f;
        for (int a = 0; a < n0; a++) inner = fmaf(mine[a], sloc[m + a], inner);
        acc = fmaf(hi, inner, acc);
        // advance the multi-index of dimensions 1..D-1
#pragma unroll
        for (int k = 1; k < D; k++) {
            idx[k]++;
            if (idx[k] < nm.n[k]) break;
            idx[k] = 0;
        }
    }
    if (dout.out == nullptr) outs[i] += acc;
    else direct_add(dout, i, 0, acc);
}

void mark_far_boxes(const PairList &far, int nbx, int nby, int *fx, int *fy, hipStream_t s)
{
    // participating boxes: x boxes with a non-empty far row, y boxes that occur in the far list
    F3M_LAUNCH(mark_rows_kernel, cdiv(nbx, 256), 256, 0, s, far.rowptr.get(), nbx, fx);
    check_launch("mark_rows");
    dev_fill(fy, 0, sizeof(int) * (size_t)nby, s);
    if (far.n > 0) {
        F3M_LAUNCH(mark_cols_kernel, cdiv(far.n, 256), 256, 0, s, far.pairs.get(), far.n, fy);
        check_launch("mark_cols");
    }
}

static void check_nodes(const NodeSet &ns)
{
    F3M_REQUIRE(ns.P <= 1024, 30, "at most 1024 interpolation nodes per box are supported (got %d)", ns.P);
}

void p2m_level(int d, const Tree &ty, const TreeLevel &ly, const int *flag, NodeSet &ns, const float *bs, float *mom,
               hipStream_t s)
{
    check_nodes(ns);
    const int P = ns.P;
    NodeMeta nm = meta_of(ns);
    const float factor = 2 / ly.edge;                  // F3M_src/1_d_conv.cu:473
    // chunks of every box: kept with the level (they depend on the tree only); chunks of flagged boxes: per call
    DBuf<int> tiles_flagged;
    int nty;
    if (flag == nullptr) {
        if (ly.p2m_bound < 0) {
            require_tables_may_be_built("the chunk table of a level");
            ly.p2m_bound = build_tiles(ly.off.get(), nullptr, ly.nb, ty.n, kP2MChunk, ly.p2m_tiles, s);
        }
        nty = ly.p2m_bound;
    } else {
        nty = build_tiles(ly.off.get(), flag, ly.nb, ty.n, kP2MChunk, tiles_flagged, s);
    }
    const DBuf<int> &tiley = flag == nullptr ? ly.p2m_tiles : tiles_flagged;
    DBuf<float> partial((size_t)std::max(1, nty) * P);
    int bdp = ((P + kWave - 1) / kWave) * kWave;
    size_t shp = sizeof(float) * (2 * (size_t)ns.S1 + (size_t)kP2MSub * ns.S1);
#define F3M_CASE(DD)                                                                                                   \
    case DD:                                                                                                           \
        F3M_LAUNCH((p2m_kernel<DD>), nty, bdp, shp, s, ty.pts.get(), ty.n, bs, ly.off.get(), ly.ctr.get(), tiley.get(), \
                   ly.nb, nm, ns.dt.get(), ns.dw.get(), factor, partial.get());                                        \
        break;
    timer_begin(kP2M, s);
    if (nty > 0 && d == 3 && ns.n[0] == 4 && ns.n[1] == 4 && ns.n[2] == 4) {
        F3M_LAUNCH(p2m_q64_kernel, nty, 64, 0, s, ty.pts.get(), ty.n, bs, ly.off.get(), ly.ctr.get(), tiley.get(), ly.nb,
                   ns.dt.get(), ns.dw.get(), factor, partial.get());
        check_launch("p2m_q64");
    } else if (nty > 0 && d == 4 && ns.n[0] == 3 && ns.n[1] == 3 && ns.n[2] == 3 && ns.n[3] == 3) {
        F3M_LAUNCH((p2m_tensor_kernel<4, 3, 1>), nty, 64, 0, s, ty.pts.get(), ty.n, bs, ly.off.get(), ly.ctr.get(), tiley.get(),
                   ly.nb, ns.dt.get(), ns.dw.get(), factor, partial.get());
        check_launch("p2m_tensor");
    } else if (nty > 0 && d == 5 && ns.n[0] == 3 && ns.n[1] == 3 && ns.n[2] == 3 && ns.n[3] == 3 && ns.n[4] == 3) {
        F3M_LAUNCH((p2m_tensor_kernel<5, 3, 2>), nty, 64, 0, s, ty.pts.get(), ty.n, bs, ly.off.get(), ly.ctr.get(), tiley.get(),
                   ly.nb, ns.dt.get(), ns.dw.get(), factor, partial.get());
        check_launch("p2m_tensor");
    } else if (nty > 0 && d == 3 && ns.n[0] == 3 && ns.n[1] == 3 && ns.n[2] == 3) {
        F3M_LAUNCH((p2m_tensor_kernel<3, 3, 1>), nty, 64, 0, s, ty.pts.get(), ty.n, bs, ly.off.get(), ly.ctr.get(), tiley.get(),
                   ly.nb, ns.dt.get(), ns.dw.get(), factor, partial.get());
        check_launch("p2m_tensor");
    } else if (nty > 0 && d == 3 && ns.n[0] == 5 && ns.n[1] == 5 && ns.n[2] == 5) {
        F3M_LAUNCH((p2m_tensor_kernel<3, 5, 2>), nty, 64, 0, s, ty.pts.get(), ty.n, bs, ly.off.get(), ly.ctr.get(), tiley.get(),
                   ly.nb, ns.dt.get(), ns.dw.get(), factor, partial.get());
        check_launch("p2m_tensor");
    } else if (nty > 0 && d == 3 && ns.n[0] == 6 && ns.n[1] == 6 && ns.n[2] == 6) {
        F3M_LAUNCH((p2m_tensor_kernel<3, 6, 2>), nty, 64, 0, s, ty.pts.get(), ty.n, bs, ly.off.get(), ly.ctr.get(), tiley.get(),
                   ly.nb, ns.dt.get(), ns.dw.get(), factor, partial.get());
        check_launch("p2m_tensor");
    } else if (nty > 0) {
        switch (d) {
            F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
            F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
        default: throw Error(2, "dimension must be 1..10");
        }
        check_launch("p2m");
    }
#undef F3M_CASE
    F3M_LAUNCH(p2m_reduce_kernel, cdiv((long long)ly.nb * P, 64), 64, 0, s, partial.get(), tiley.get(), ly.nb, P, mom);
    timer_end(s);
    check_launch("p2m_reduce");
}

void m2l_level(int d, const Tree &tx, const TreeLevel &lx, const Tree &ty, const TreeLevel &ly, const PairList &far,
               NodeSet &ns, float lcs, int m2l_mode, const float *mom, float *loc, hipStream_t s, bool beside_near)
{
    check_nodes(ns);
    const int P = ns.P;
    NodeMeta nm = meta_of(ns);
    int bdp = ((P + kWave - 1) / kWave) * kWave;
    dev_fill(loc, 0, sizeof(float) * (size_t)lx.nb * P, s);
    if (far.n == 0) return;
    int NT = 1;
    for (int j = 0; j < d; j++) NT = std::max(NT, ns.n[j]);
    const int ntab = d * kM2LOffsets * NT * NT;
    const bool sib_forced = m2l_mode == 3;
    if (sib_forced) m2l_mode = 0;
    const bool separable = m2l_mode == 2 || (m2l_mode == 0 && (size_t)(ntab + 2 * P) * sizeof(float) <= 48 * 1024);
    if (separable) {
        F3M_REQUIRE((size_t)(ntab + 2 * P) * sizeof(float) <= 64 * 1024, 31, "separable M2L tables do not fit in LDS");
        SepMeta sm;
        sm.NT = NT;
        SepGeo sg;
        const double edge = (double)lx.edge;
        for (int j = 0; j < kMaxD; j++) { sm.omin[j] = 0; sg.omin[j] = 0; sg.delta[j] = 0; }
        for (int j = 0; j < d; j++) {
            sg.delta[j] = (double)ty.geo.origin[j] - (double)tx.geo.origin[j];
            sm.omin[j] = sg.omin[j] = m2l_table_omin(tx.geo.origin[j], ty.geo.origin[j], lx.edge);
        }
        // the tables of the level depend on the plan only (nodes, edge, lengthscale, origins) and are kept with its far list
        DBuf<float> &dtab = far.m2l_tab;
        if (dtab.size() != (size_t)ntab) {
            require_tables_may_be_built("the M2L tables of a level");
            dtab.reset((size_t)ntab);
            F3M_LAUNCH(sep_tables_kernel, cdiv(ntab, 64), 64, 0, s, nm, d, NT, kM2LOffsets, ns.dt.get(), edge, (double)lcs, sg,
                       dtab.get());
            check_launch("sep_tables");
        }
        size_t shs = sizeof(float) * ((size_t)ntab + 2 * (size_t)P);
        timer_begin(kM2L, s);
        const bool q64 = d == 3 && ns.n[0] == 4 && ns.n[1] == 4 && ns.n[2] == 4 && m2l_mode != 2;
        // sibling-group kernel: one tree, 3 <= d <= 5, n0 = n1 in 2..4, every far pair inside the 6^d cells
        int sibGS = 0, sibR2 = 0, sibPass = 1, sibH = 1;
        size_t shsib = 0;
        // (preferred to the per-box kernel for 4 x 4 x 4 nodes as well once a level has a few hundred
        // parents: 0.30 against 0.55 ms at depth 5 of N=1e7; with fewer parents the per-box kernel has
        // more workgroups to offer)
        const bool enough_parents = sib_forced || !q64 || (lx.depth >= 1 && tx.lev[lx.depth - 1].nb >= 256);
        const bool sib_grid = ns.n[0] == ns.n[1] && ns.n[0] >= 2 && (ns.n[0] <= 4 || (d == 3 && ns.n[0] <= 6 && ns.n[2] == ns.n[0]));
        if (m2l_mode == 0 && enough_parents && &tx == &ty && d >= 3 && d <= 5 && sib_grid && far.outliers == 0 && lx.depth >= 1) {
            const int N = ns.n[0], W = N <= 4 ? 4 : 8;
            sibR2 = P / (N * N);
            if (sibR2 <= 1024) {
                sibGS = 1 << d;
                while (sibGS * sibR2 > 1024) sibGS >>= 1;
                // Beside the near field (whose wavefronts keep every compute unit full) only small workgroups find room:
                // from four dimensions on, groups of four siblings then, one or two wavefronts (N=1e7: 4-D 15.1 -> 14.85 ms,
                // 5-D 53.4 -> 51.8 ms per product; groups of eight: 14.9 and 54.8; alone on the GPU the whole family in
                // one workgroup is faster, 2.1 against 3.0 ms in 4-D).
                if (beside_near && d >= 4)
                    while (sibGS > 4 || (sibGS > 1 && sibGS * sibR2 > 2 * kWave)) sibGS >>= 1;
                // 3-D: 8 siblings x n2 lanes fill at most half a wavefront; two lanes then share a lane's nodes
                const char *nosplit = getenv("F3M_SIB_SPLIT");   // F3M_SIB_SPLIT=0: testing aid
                if (d == 3 && N % 2 == 0 && sibGS * sibR2 <= kWave / 2 && !(nosplit && atoi(nosplit) == 0)) { sibH = 2; sibR2 *= 2; }
                const int bd = ((sibGS * sibR2 + kWave - 1) / kWave) * kWave;
                // table in 1, 2, 3 or 6 parts: the fewest that fit (a second workgroup per compute unit bought
                // with two parts did not pay at 6^5 cells: 7.7 -> 8.2 ms; every part scans the far rows again)
                int forced = 0;                                  // F3M_SIB_PASSES=1|2|3|6: testing aid
                if (const char *e = getenv("F3M_SIB_PASSES")) forced = atoi(e);
                for (int np : {1, 2, 3, 6}) {
                    if (forced > 0 && np != forced && np != 6) continue;
                    sibPass = np;
                    shsib = sizeof(float) * (2 * (size_t)(sib_codes(d) / np) + 4 * (size_t)sib_ext_codes(d) + (size_t)(N * N / sibH) * bd +
                                             (size_t)((ntab + 3) & ~3) + 2 * (size_t)kM2LOffsets * N * W + (size_t)N * W) +
                            sizeof(int) * (size_t)sibGS;
                    if ((shsib <= 150 * 1024 && forced <= 0) || np == forced) break;
                }
                if (shsib > 150 * 1024) sibGS = 0;
            }
        }
        if (getenv("F3M_DEBUG"))
            fprintf(stderr, "m2l depth %d: %s (nodes %d, siblings per workgroup %d, lanes per sibling %d, table parts %d)\n", lx.depth,
                    sibGS > 0 ? "sibling groups" : (q64 ? "4x4x4 per box" : "separable per box"), P, sibGS, sibR2, sibPass);
        if (sibGS > 0) {
            const TreeLevel &par = tx.lev[lx.depth - 1];
            const int nsub = (1 << d) / sibGS;
            const int bd = ((sibGS * sibR2 + kWave - 1) / kWave) * kWave;
            // Long workgroups of very different lengths (d >= 4: a boundary parent has a fraction of the far
            // cells of an interior one): start the longest first (N=1e7: 5-D 7.7 -> 6.1 ms, 4-D 2.30 -> 2.07 ms).
            // In 3-D the workgroups are short and many, and the Morton order of the parents is worth more
            // (0.33 -> 0.35 ms; 0.75 -> 1.5 ms on the normal cloud with its 65 000 parents placed by one
            // workgroup).  F3M_SIB_ORDER=0|1 overrides.
            bool ordered = d >= 4 && par.nb <= 16384;
            if (const char *e = getenv("F3M_SIB_ORDER")) ordered = atoi(e) != 0;
            DBuf<int> &sibOrder = far.m2l_order;
            if (ordered && sibOrder.size() != (size_t)par.nb) {
                require_tables_may_be_built("the M2L parent order of a level");
                DBuf<int> cls((size_t)par.nb), hist(256);
                sibOrder.reset((size_t)par.nb);
                dev_fill(hist.get(), 0, 256 * sizeof(int), s);
                const int unit = (int)std::max<long long>(1, far.n / std::max(1, par.nb) / 64);    // mean row = class 64
                F3M_LAUNCH(sib_class_count_kernel, cdiv(par.nb, 256), 256, 0, s, par.childstart.get(), far.rowptr.get(), par.nb,
                           unit, cls.get(), hist.get());
                check_launch("sib_class_count");
                F3M_LAUNCH(class_place_kernel, 1, 1024, 0, s, cls.get(), par.nb, hist.get(), sibOrder.get());
                check_launch("sib_class_place");
            }
            const int *sibOrd = ordered ? sibOrder.get() : (const int *)nullptr;
            // (instances bound to 128 threads for the groups of four siblings that run beside the near field, 4-D and 5-D,
            // have no spilled values but one wavefront per SIMD less: same time, not kept)
            const int maxt = (d == 3 && ns.n[0] >= 5) ? 64 : 1024;
            // 3^4 grid beside the near field: the cells that every child of a parent lists are summed once per combination
            // of sibling bits first (m2l_shared_kernel); the sibling kernel then takes what is left and adds.  A parent's
            // cells are then walked by one wavefront instead of by three or more, with a sixth of the vector
            // instructions: beside the near field, which is short of exactly those, the product gains (N=1e7, 4-D:
            // 14.2 -> 13.7 ms); alone on the GPU the longer walk costs more than the instructions save (M2L 2.1 -> 2.4
            // ms), and in 5-D, 1024 parents with 7776 cells each, it does not end before the near field does (40.9 ->
            // 47.7 ms).  F3M_M2L_SHARED=0|1 overrides (1: 3^4 and 3^5 grids, in either mode).
            const bool shared_fits = (d == 4 || d == 5) && sibH == 1 && ly.nb < (1 << 24) && ns.n[0] == 3 && ns.n[1] == 3 &&
                                     ns.n[2] == 3 && ns.n[3] == 3 && (d == 4 || ns.n[4] == 3);
            bool shared = shared_fits && d == 4 && beside_near;
            if (const char *e = getenv("F3M_M2L_SHARED")) shared = shared_fits && atoi(e) != 0;
            DBuf<unsigned char> taken;
            if (shared) {
                const int lanes = 2 * P / 3, sbd = ((lanes + kWave - 1) / kWave) * kWave, xv = 3 << (d - 2);
                int spass = 1;
                size_t shs3 = 0;
                for (int np : {1, 2, 3, 6}) {
                    spass = np;
                    shs3 = sizeof(float) * ((size_t)(sib_codes(d) / np) + (size_t)xv * sbd + (size_t)((ntab + 3) & ~3)) +
                           sizeof(int) * ((size_t)1 << d);
                    if (shs3 <= 150 * 1024) break;
                }
                taken.reset((size_t)par.nb * sib_codes(d));
                if (getenv("F3M_DEBUG"))
                    fprintf(stderr, "m2l depth %d: shared sums first (%d lanes per parent, table parts %d, %zu bytes of LDS)\n", lx.depth,
                            lanes, spass, shs3);
#ifndef F3M_CPU_EMU
#define F3M_SHARED_ATTR(DD)                                                                                            \
    F3M_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&m2l_shared_kernel<DD, 3>),                             \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shs3));
#else
#define F3M_SHARED_ATTR(DD)
#endif
#define F3M_SHARED(DD)                                                                                                 \
    if (d == DD) {                                                                                                     \
        F3M_SHARED_ATTR(DD)                                                                                            \
        F3M_LAUNCH((m2l_shared_kernel<DD, 3>), par.nb, sbd, shs3, s, dtab.get(), ntab, sm, P, spass, sibOrd,           \
                   par.childstart.get(), lx.cell.get(), far.pairs.get(), far.rowptr.get(), mom, loc, taken.get());     \
    }
                F3M_SHARED(4) F3M_SHARED(5)
#undef F3M_SHARED
#undef F3M_SHARED_ATTR
                check_launch("m2l_shared");
            }
#ifndef F3M_CPU_EMU
#define F3M_SIB_ATTR(DD, NNODE, HH, MT)                                                                                \
    F3M_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&m2l_sib_kernel<DD, NNODE, HH, MT>),                    \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shsib));
#else
#define F3M_SIB_ATTR(DD, NNODE, HH, MT)
#endif
#define F3M_SIB(DD, NNODE, HH, MT)                                                                                     \
    if (d == DD && ns.n[0] == NNODE && sibH == HH && maxt == MT) {                                                     \
        F3M_SIB_ATTR(DD, NNODE, HH, MT)                                                                                \
        F3M_LAUNCH((m2l_sib_kernel<DD, NNODE, HH, MT>), par.nb * nsub, bd, shsib, s, dtab.get(), ntab, sm, nm, sibR2,  \
                   sibGS, nsub, sibPass, sibOrd, par.childstart.get(), lx.cell.get(), far.pairs.get(),                 \
                   far.rowptr.get(), mom, loc, shared ? taken.get() : (const unsigned char *)nullptr);                 \
    }
            F3M_SIB(3, 2, 2, 1024) F3M_SIB(3, 3, 1, 1024) F3M_SIB(3, 4, 2, 1024) F3M_SIB(3, 2, 1, 1024) F3M_SIB(3, 4, 1, 1024)
            F3M_SIB(3, 5, 1, 64) F3M_SIB(3, 6, 1, 64)
            F3M_SIB(4, 2, 1, 1024) F3M_SIB(4, 3, 1, 1024) F3M_SIB(4, 4, 1, 1024)
            F3M_SIB(5, 2, 1, 1024) F3M_SIB(5, 3, 1, 1024) F3M_SIB(5, 4, 1, 1024)
#undef F3M_SIB
#undef F3M_SIB_ATTR
        } else if (q64) {
            // table index of the lowest expected offset: one tree: cell offsets of far pairs are -3..3; two
            // trees: centre distances stay below 5 edges, i.e. offsets from ceil(-5 - delta/edge) on, at most
            // 11 distinct values.  (Anything outside is still handled, pair by pair.)
            int lo[3];
            for (int j = 0; j < 3; j++)
                lo[j] = (&tx == &ty ? -3 : (int)std::ceil(-5.0 - sg.delta[j] / edge)) - sm.omin[j];
            if (&tx == &ty)
                F3M_LAUNCH((m2l_q64_kernel<7>), lx.nb, 64, 0, s, dtab.get(), sm, lo[1], lo[2], lx.cell.get(), ly.cell.get(),
                           far.pairs.get(), far.rowptr.get(), mom, loc);
            else
                F3M_LAUNCH((m2l_q64_kernel<11>), lx.nb, 64, 0, s, dtab.get(), sm, lo[1], lo[2], lx.cell.get(), ly.cell.get(),
                           far.pairs.get(), far.rowptr.get(), mom, loc);
        } else {
#define F3M_CASE(DD)                                                                                                   \
    case DD:                                                                                                           \
        F3M_LAUNCH((m2l_sep_kernel<DD>), lx.nb, bdp, shs, s, dtab.get(), ntab, nm, sm, lx.cell.get(), ly.cell.get(),   \
                   far.pairs.get(), far.rowptr.get(), mom, loc);                                                       \
        break;
        switch (d) {
            F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
            F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
        default: throw Error(2, "dimension must be 1..10");
        }
#undef F3M_CASE
        }
        timer_end(s);
        check_launch("m2l_sep");
    } else {
        set_node_offsets(ns, lx.edge, s);
        size_t shm = sizeof(float) * (size_t)P * (d + 1);
        timer_begin(kM2L, s);
#define F3M_CASE(DD)                                                                                                   \
    case DD:                                                                                                           \
        F3M_LAUNCH((m2l_direct_kernel<DD>), lx.nb, bdp, shm, s, ns.noff.get(), P, lx.ctr.get(), ly.ctr.get(),          \
                   far.pairs.get(), far.rowptr.get(), mom, lcs * kLog2e, loc);                                         \
        break;
        switch (d) {
            F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
            F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
        default: throw Error(2, "dimension must be 1..10");
        }
#undef F3M_CASE
        timer_end(s);
        check_launch("m2l");
    }
}

// L2P for the 4 x 4 x 4 grid over every box of a level: one lane per point, 128 consecutive points per
// workgroup whatever boxes they belong to (a level of small boxes keeps its lanes busy).  Each lane
// finds its box among the box offsets that start inside the workgroup's range, reads the local expansion
// of that box straight from global memory (lanes of one box read the same 16 bytes) and keeps its twelve
// 1-D basis values in registers.
__global__ void __launch_bounds__(kL2PBlock) l2p_q64_kernel(const float *__restrict__ xs, long long N, float *__restrict__ outs,
                                                             const int *__restrict__ off, const float *__restrict__ ctr,
                                                             int nb, const int *__restrict__ box32,
                                                             const float *__restrict__ nt, const float *__restrict__ nw,
                                                             float factor, const float *__restrict__ loc, DirectOut dout)
{
    __shared__ int bounds[kL2PBlock];
    const int tid = threadIdx.x;
    const long long i0 = (long long)blockIdx.x * kL2PBlock;
    const int b0 = box32[i0 / 32];                  // box of the first point (i0 is a multiple of 32)
    bounds[tid] = off[min(b0 + 1 + tid, nb)];      // starts of the next boxes (off[nb] = N closes the list)
    __syncthreads();
    const long long i = i0 + tid;
    if (i >= N) return;
    // number of those starts that are <= i
    int a = 0, b = kL2PBlock;
    while (a < b) {
        int mid = (a + b) >> 1;
        if (bounds[mid] <= i) a = mid + 1; else b = mid;
    }
    const int box = b0 + a;
    float l[3][4];
#pragma unroll
    for (int k = 0; k < 3; k++) {
        const float t = factor * (xs[(long long)k * N + i] - ctr[(long long)box * 3 + k]);
        basis_1d(t, nt + 4 * k, nw + 4 * k, 4, l[k], 1.f);
    }
    const float4 *lp = reinterpret_cast<const float4 *>(loc + (long long)box * 64);
    float acc = 0.f;
#pragma unroll
    for (int h = 0; h < 16; h++) {
        const float4 r = lp[h];
        float inner = l[0][0] * r.x;
        inner = fmaf(l[0][1], r.y, inner);
        inner = fmaf(l[0][2], r.z, inner);
        inner = fmaf(l[0][3], r.w, inner);
        acc = fmaf(l[1][h & 3] * l[2][h >> 2], inner, acc);
    }
    if (dout.out == nullptr) outs[i] += acc;
    else direct_add(dout, i, 0, acc);
}

// The same for other tensor grids of N nodes per dimension: the weights of the nodes of dimensions >= 1
// are formed once per point, the expansion is read in rows of N.
template <int D, int N>
__global__ void __launch_bounds__(kL2PBlock) l2p_tensor_kernel(const float *__restrict__ xs, long long NP, float *__restrict__ outs,
                                                                const int *__restrict__ off, const float *__restrict__ ctr,
                                                                int nb, const int *__restrict__ box32,
                                                                const float *__restrict__ nt, const float *__restrict__ nw,
                                                                float factor, const float *__restrict__ loc, DirectOut dout)
{
    constexpr int Q = ipow(N, D - 1), P = Q * N;
    __shared__ int bounds[kL2PBlock];
    const int tid = threadIdx.x;
    const long long i0 = (long long)blockIdx.x * kL2PBlock;
    const int b0 = box32[i0 / 32];                  // box of the first point (i0 is a multiple of 32)
    bounds[tid] = off[min(b0 + 1 + tid, nb)];      // starts of the next boxes (off[nb] = NP closes the list)
    __syncthreads();
    const long long i = i0 + tid;
    if (i >= NP) return;
    int a = 0, b = kL2PBlock;                       // number of those starts that are <= i
    while (a < b) {
        int mid = (a + b) >> 1;
        if (bounds[mid] <= i) a = mid + 1; else b = mid;
    }
    const int box = b0 + a;
    float l[D][N];
#pragma unroll
    for (int k = 0; k < D; k++) {
        const float t = factor * (xs[(long long)k * NP + i] - ctr[(long long)box * D + k]);
        basis_1d(t, nt + N * k, nw + N * k, N, l[k], 1.f);
    }
    float w[Q];                                     // w[j] = prod_{k >= 1} l_k[digit_k(j)], dimension 1 fastest
    w[0] = 1.f;
    int len = 1;
#pragma unroll
    for (int k = D - 1; k >= 1; k--) {
#pragma unroll
        for (int j = len - 1; j >= 0; j--)
#pragma unroll
            for (int e = N - 1; e >= 0; e--) w[j * N + e] = w[j] * l[k][e];
        len *= N;
    }
    const float *lp = loc + (long long)box * P;
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < Q; j++) {
        const fvec<N> r = *reinterpret_cast<const fvec<N> *>(lp + N * j);
        float inner = l[0][0] * r.v[0];
#pragma unroll
        for (int e = 1; e < N; e++) inner = fmaf(l[0][e], r.v[e], inner);
        acc = fmaf(w[j], inner, acc);
    }
    if (dout.out == nullptr) outs[i] += acc;
    else direct_add(dout, i, 0, acc);
}

void l2p_level(int d, const Tree &tx, const TreeLevel &lx, const int *flag, NodeSet &ns, const float *loc, float *outs,
               hipStream_t s, const DirectOut *direct)
{
    const DirectOut dout = direct ? *direct : DirectOut();
    check_nodes(ns);
    const int P = ns.P;
    NodeMeta nm = meta_of(ns);
    const float factor = 2 / lx.edge;
    if (flag == nullptr && d == 3 && ns.n[0] == 4 && ns.n[1] == 4 && ns.n[2] == 4) {
        timer_begin(kL2P, s);
        F3M_LAUNCH(l2p_q64_kernel, cdiv(tx.n, kL2PBlock), kL2PBlock, 0, s, tx.pts.get(), tx.n, outs, lx.off.get(),
                   lx.ctr.get(), lx.nb, box_table(lx, tx.n, s), ns.dt.get(), ns.dw.get(), factor, loc, dout);
        timer_end(s);
        check_launch("l2p_q64");
        return;
    }
    if (flag == nullptr && d == 4 && ns.n[0] == 3 && ns.n[1] == 3 && ns.n[2] == 3 && ns.n[3] == 3) {
        timer_begin(kL2P, s);
        F3M_LAUNCH((l2p_tensor_kernel<4, 3>), cdiv(tx.n, kL2PBlock), kL2PBlock, 0, s, tx.pts.get(), tx.n, outs, lx.off.get(),
                   lx.ctr.get(), lx.nb, box_table(lx, tx.n, s), ns.dt.get(), ns.dw.get(), factor, loc, dout);
        timer_end(s);
        check_launch("l2p_tensor");
        return;
    }
    if (flag == nullptr && d == 5 && ns.n[0] == 3 && ns.n[1] == 3 && ns.n[2] == 3 && ns.n[3] == 3 && ns.n[4] == 3) {
        timer_begin(kL2P, s);
        F3M_LAUNCH((l2p_tensor_kernel<5, 3>), cdiv(tx.n, kL2PBlock), kL2PBlock, 0, s, tx.pts.get(), tx.n, outs, lx.off.get(),
                   lx.ctr.get(), lx.nb, box_table(lx, tx.n, s), ns.dt.get(), ns.dw.get(), factor, loc, dout);
        timer_end(s);
        check_launch("l2p_tensor");
        return;
    }
    if (flag == nullptr && d == 3 && ns.n[0] == 3 && ns.n[1] == 3 && ns.n[2] == 3) {
        timer_begin(kL2P, s);
        F3M_LAUNCH((l2p_tensor_kernel<3, 3>), cdiv(tx.n, kL2PBlock), kL2PBlock, 0, s, tx.pts.get(), tx.n, outs, lx.off.get(),
                   lx.ctr.get(), lx.nb, box_table(lx, tx.n, s), ns.dt.get(), ns.dw.get(), factor, loc, dout);
        timer_end(s);
        check_launch("l2p_tensor");
        return;
    }
    if (flag == nullptr && d == 3 && ns.n[0] == 5 && ns.n[1] == 5 && ns.n[2] == 5) {
        timer_begin(kL2P, s);
        F3M_LAUNCH((l2p_tensor_kernel<3, 5>), cdiv(tx.n, kL2PBlock), kL2PBlock, 0, s, tx.pts.get(), tx.n, outs, lx.off.get(),
                   lx.ctr.get(), lx.nb, box_table(lx, tx.n, s), ns.dt.get(), ns.dw.get(), factor, loc, dout);
        timer_end(s);
        check_launch("l2p_tensor");
        return;
    }
    if (flag == nullptr && d == 3 && ns.n[0] == 6 && ns.n[1] == 6 && ns.n[2] == 6) {
        timer_begin(kL2P, s);
        F3M_LAUNCH((l2p_tensor_kernel<3, 6>), cdiv(tx.n, kL2PBlock), kL2PBlock, 0, s, tx.pts.get(), tx.n, outs, lx.off.get(),
                   lx.ctr.get(), lx.nb, box_table(lx, tx.n, s), ns.dt.get(), ns.dw.get(), factor, loc, dout);
        timer_end(s);
        check_launch("l2p_tensor");
        return;
    }
    DBuf<int> tiles_flagged;
    int ntx;
    if (flag == nullptr) {
        if (lx.l2p_bound < 0) {
            require_tables_may_be_built("the chunk table of a level");
            lx.l2p_bound = build_tiles(lx.off.get(), nullptr, lx.nb, tx.n, kL2PBlock, lx.l2p_tiles, s);
        }
        ntx = lx.l2p_bound;
    } else {
        ntx = build_tiles(lx.off.get(), flag, lx.nb, tx.n, kL2PBlock, tiles_flagged, s);
    }
    const DBuf<int> &tilex = flag == nullptr ? lx.l2p_tiles : tiles_flagged;
    size_t shl = sizeof(float) * (2 * (size_t)ns.S1 + (size_t)P + (size_t)kL2PBlock * (ns.S1 | 1));
#define F3M_CASE(DD)                                                                                                   \
    case DD:                                                                                                           \
        F3M_LAUNCH((l2p_kernel<DD>), ntx, kL2PBlock, shl, s, tx.pts.get(), tx.n, outs, lx.off.get(), lx.ctr.get(),     \
                   tilex.get(), lx.nb, nm, ns.dt.get(), ns.dw.get(), factor, loc, dout);                                     \
        break;
    if (ntx > 0) {
        timer_begin(kL2P, s);
        switch (d) {
            F3M_CASE(1) F3M_CASE(2) F3M_CASE(3) F3M_CASE(4) F3M_CASE(5)
            F3M_CASE(6) F3M_CASE(7) F3M_CASE(8) F3M_CASE(9) F3M_CASE(10)
        default: throw Error(2, "dimension must be 1..10");
        }
        timer_end(s);
        check_launch("l2p");
    }
#undef F3M_CASE
}

// the far field of one level on its own, as the reference computes it (F3M_src/n_tree.cu:489-593)
void far_field(int d, const Tree &tx, const TreeLevel &lx, const Tree &ty, const TreeLevel &ly, const PairList &far,
               NodeSet &ns, const float *bs, float *outs, float lcs, int m2l_mode, float *mom_out, float *loc_out,
               hipStream_t s)
{
    if (far.n == 0) return;
    const int P = ns.P;
    DBuf<int> fx((size_t)lx.nb), fy((size_t)ly.nb);
    mark_far_boxes(far, lx.nb, ly.nb, fx.get(), fy.get(), s);
    DBuf<float> mom((size_t)ly.nb * P), loc((size_t)lx.nb * P);
    p2m_level(d, ty, ly, fy.get(), ns, bs, mom.get(), s);
    m2l_level(d, tx, lx, ty, ly, far, ns, lcs, m2l_mode, mom.get(), loc.get(), s);
    l2p_level(d, tx, lx, fx.get(), ns, loc.get(), outs, s);
    if (mom_out) F3M_HIP(hipMemcpyAsync(mom_out, mom.get(), sizeof(float) * (size_t)ly.nb * P, hipMemcpyDeviceToDevice, s));
    if (loc_out) F3M_HIP(hipMemcpyAsync(loc_out, loc.get(), sizeof(float) * (size_t)lx.nb * P, hipMemcpyDeviceToDevice, s));
}

// ------------------------------------------------------------------------------------------------
// Moving expansions between a box and its children (no counterpart in the reference, which
// interpolates every level from the points: F3M_src/n_tree.cu:489-593).  The Lagrange polynomials of
// a box, restricted to a child, are polynomials of the same degree, so interpolation at the child's
// nodes reproduces them exactly when the child has at least as many nodes per dimension:
//     L^parent_m(y) = sum_a L^parent_m(node^child_a) L^child_a(y)   for y in the child.
// Hence  Mom_parent[m] = sum_children sum_a T[m][a] Mom_child[a]   (upward) and the local expansion
// of a parent acts on a child's points as  Loc_child[a] += sum_m T[m][a] Loc_parent[m]  (downward),
// with T = tensor product of 1-D tables T_j[s][m][a] = l_m(s/2 + t_a/2), s = -1/+1 for the lower/upper
// half.  The sums are the same as the reference's up to rounding; the points are read once per product
// instead of once per level.

struct ShiftMeta {
    int np[kMaxD], nc[kMaxD];   // nodes per dimension of the parent's and of the child's node set
    int Pp, Pc, NTp, NTc;
};

__global__ void shift_tables_kernel(ShiftMeta sm, int d, NodeMeta nmp, NodeMeta nmc, const float *__restrict__ tp,
                                    const float *__restrict__ wp, const float *__restrict__ tc, float *__restrict__ tab)
{
    int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= d * 2 * sm.NTp * sm.NTc) return;
    const int a = e % sm.NTc, m = (e / sm.NTc) % sm.NTp, sg = (e / (sm.NTc * sm.NTp)) % 2, j = e / (sm.NTc * sm.NTp * 2);
    float v = 0.f;
    if (m < sm.np[j] && a < sm.nc[j]) {
        const double tau = (sg ? 0.5 : -0.5) + 0.5 * (double)tc[nmc.start[j] + a];
        double sum = 0, mine = 0;
        int hit = -1;
        for (int l = 0; l < sm.np[j]; l++) {
            double diff = tau - (double)tp[nmp.start[j] + l];
            if (diff == 0) { hit = l; continue; }
            double q = (double)wp[nmp.start[j] + l] / diff;
            if (l == m) mine = q;
            sum += q;
        }
        v = hit >= 0 ? (hit == m ? 1.f : 0.f) : (float)(mine / sum);
    }
    tab[e] = v;
}

// One workgroup per parent box.  DOWN = false: dst[parent] = sum over children of T src[child];
// DOWN = true: dst[child] += T^t src[parent].  The d one-dimensional factors are applied one after
// the other through two LDS buffers.
template <bool DOWN>
__global__ void __launch_bounds__(1024) shift_kernel(const float *__restrict__ tables, int ntab, ShiftMeta sm, int d,
                                                      const int *__restrict__ childstart, const int *__restrict__ cellc,
                                                      const float *__restrict__ src, float *__restrict__ dst)
{
    F3M_DYN_SHARED(float, smem);
    float *tab = smem;                     // ntab
    float *bufA = smem + ntab;             // Pc (the larger of the two node counts)
    float *bufB = bufA + sm.Pc;
    float *par = bufB + sm.Pc;             // Pp: the parent's expansion (DOWN only)
    const int b = blockIdx.x, tid = threadIdx.x, BD = blockDim.x;
    for (int e = tid; e < ntab; e += BD) tab[e] = tables[e];
    if (DOWN)
        for (int e = tid; e < sm.Pp; e += BD) par[e] = src[(long long)b * sm.Pp + e];
    const int *nin = DOWN ? sm.np : sm.nc, *nout = DOWN ? sm.nc : sm.np;
    const int Pin = DOWN ? sm.Pp : sm.Pc, Pout = DOWN ? sm.Pc : sm.Pp;
    float acc = 0.f;                       // UP: this lane's element of the parent (BD >= Pp)
    for (int c = childstart[b]; c < childstart[b + 1]; c++) {
        __syncthreads();
        for (int e = tid; e < Pin; e += BD) bufA[e] = DOWN ? par[e] : src[(long long)c * sm.Pc + e];
        __syncthreads();
        float *in = bufA, *out = bufB;
        int lo = 1;                        // product of nout over the dimensions already done
        int hi = Pin;                      // product of nin over the dimensions still to do (incl. j)
        for (int j = 0; j < d; j++) {
            hi /= nin[j];
            const int sg = cellc[(long long)c * d + j] & 1;
            const float *T = tab + (size_t)(j * 2 + sg) * sm.NTp * sm.NTc;
            const int size = lo * nout[j] * hi;
            for (int e = tid; e < size; e += BD) {
                const int l = e % lo, q = (e / lo) % nout[j], h = e / (lo * nout[j]);
                const float *sp = in + l + lo * nin[j] * h;
                float sum = 0.f;
                for (int r = 0; r < nin[j]; r++) {
                    // T[m][a] with m = parent node, a = child node
                    const float t = DOWN ? T[r * sm.NTc + q] : T[q * sm.NTc + r];
                    sum = fmaf(t, sp[lo * r], sum);
                }
                if (j == d - 1) {
                    if (DOWN) dst[(long long)c * sm.Pc + e] += sum;
                    else acc += sum;
                } else {
                    out[e] = sum;
                }
            }
            lo *= nout[j];
            __syncthreads();
            float *t = in; in = out; out = t;
        }
    }
    if (!DOWN && tid < Pout) dst[(long long)b * sm.Pp + tid] = acc;
}

// The same transfer for the 4 x 4 x 4 grid on both levels: one wavefront per parent box, lane = node
// (a0 + 4 a1 + 16 a2); the three 4 x 4 factors are applied with exchanges inside the wavefront (groups of
// four lanes, lanes 4 apart, lanes 16 apart), no LDS traffic besides the 96-entry table, no barriers.
// (workgroups of one wavefront: the far field runs beside the near field, whose wavefronts keep the compute
// units full, and only small workgroups find room there)
constexpr int kShiftQWaves = 1;

template <bool DOWN>
__global__ void __launch_bounds__(kShiftQWaves * 64) shift_q64_kernel(const float *__restrict__ tables, int nbp,
                                                                      const int *__restrict__ childstart,
                                                                      const int *__restrict__ cellc,
                                                                      const float *__restrict__ src, float *__restrict__ dst)
{
    // rows[(j*2+s)*4 + r] = the four table entries lane digit r needs: T[r][*] going up, T[*][r] going down
    __shared__ __align__(16) float rows[3 * 2 * 4 * 4];
    for (int e = threadIdx.x; e < 96; e += blockDim.x) {
        const int q = e & 3, r = (e >> 2) & 3, js = e >> 4;
        rows[e] = DOWN ? tables[(js * 4 + q) * 4 + r] : tables[(js * 4 + r) * 4 + q];
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int b = blockIdx.x * kShiftQWaves + (threadIdx.x >> 6);
    if (b >= nbp) return;
    const int a0 = lane & 3, a1 = (lane >> 2) & 3, a2 = lane >> 4;
    const float v0 = DOWN ? src[(long long)b * 64 + lane] : 0.f;
    float acc = 0.f;
    for (int c = childstart[b]; c < childstart[b + 1]; c++) {
        const int s0 = cellc[(long long)c * 3 + 0] & 1, s1 = cellc[(long long)c * 3 + 1] & 1, s2 = cellc[(long long)c * 3 + 2] & 1;
        float v = DOWN ? v0 : src[(long long)c * 64 + lane];
        const float4 r0 = *reinterpret_cast<const float4 *>(&rows[((0 * 2 + s0) * 4 + a0) * 4]);
        float t = r0.x * quad_bcast<0>(v);
        t = fmaf(r0.y, quad_bcast<1>(v), t);
        t = fmaf(r0.z, quad_bcast<2>(v), t);
        t = fmaf(r0.w, quad_bcast<3>(v), t);
        const float4 r1 = *reinterpret_cast<const float4 *>(&rows[((1 * 2 + s1) * 4 + a1) * 4]);
        float u = r1.x * wave_shfl_f(t, (lane & ~12) | 0);
        u = fmaf(r1.y, wave_shfl_f(t, (lane & ~12) | 4), u);
        u = fmaf(r1.z, wave_shfl_f(t, (lane & ~12) | 8), u);
        u = fmaf(r1.w, wave_shfl_f(t, (lane & ~12) | 12), u);
        const float4 r2 = *reinterpret_cast<const float4 *>(&rows[((2 * 2 + s2) * 4 + a2) * 4]);
        float w = r2.x * wave_shfl_f(u, (lane & 15) | 0);
        w = fmaf(r2.y, wave_shfl_f(u, (lane & 15) | 16), w);
        w = fmaf(r2.z, wave_shfl_f(u, (lane & 15) | 32), w);
        w = fmaf(r2.w, wave_shfl_f(u, (lane & 15) | 48), w);
        if (DOWN) dst[(long long)c * 64 + lane] += w;
        else acc += w;
    }
    if (!DOWN) dst[(long long)b * 64 + lane] = acc;
}

// The same transfer for any grid of N nodes per dimension on both levels, one wavefront per parent box (a workgroup
// of one wavefront finds room beside the near field's wavefronts; the general kernel's workgroup of one lane per node
// does not).  The expansion of a child passes through two LDS buffers, one 1-D factor at a time; lane l owns the
// elements l, l + 64, ... of every stage.
template <bool DOWN, int D, int N>
__global__ void __launch_bounds__(64) shift_tensor_kernel(const float *__restrict__ tables, int nbp,
                                                           const int *__restrict__ childstart, const int *__restrict__ cellc,
                                                           const float *__restrict__ src, float *__restrict__ dst)
{
    constexpr int P = ipow(N, D), K = (P + 63) / 64, NTAB = D * 2 * N * N;
    __shared__ float tab[NTAB];             // T_j[s][m][a], m = parent node, a = child node
    __shared__ float buf[2][P];
    const int lane = threadIdx.x, b = blockIdx.x;
    if (b >= nbp) return;
    for (int e = lane; e < NTAB; e += 64) tab[e] = tables[e];
    float acc[K], par[K];
#pragma unroll
    for (int k = 0; k < K; k++) {
        const int e = lane + 64 * k;
        acc[k] = 0.f;
        par[k] = (DOWN && e < P) ? src[(long long)b * P + e] : 0.f;
    }
    for (int c = childstart[b]; c < childstart[b + 1]; c++) {
        __syncthreads();                    // the previous child's last stage has been read
#pragma unroll
        for (int k = 0; k < K; k++) {
            const int e = lane + 64 * k;
            if (e < P) buf[0][e] = DOWN ? par[k] : src[(long long)c * P + e];
        }
        __syncthreads();
        int stride = 1;
#pragma unroll
        for (int j = 0; j < D; j++) {
            const int sg = cellc[(long long)c * D + j] & 1;
            const float *T = tab + (j * 2 + sg) * N * N;
            const float *in = buf[j & 1];
            float *out = buf[(j & 1) ^ 1];
#pragma unroll
            for (int k = 0; k < K; k++) {
                const int e = lane + 64 * k;
                if (e < P) {
                    const int q = (e / stride) % N;
                    const float *sp = in + (e - q * stride);
                    float sum = 0.f;
#pragma unroll
                    for (int r = 0; r < N; r++) sum = fmaf(DOWN ? T[r * N + q] : T[q * N + r], sp[r * stride], sum);
                    if (j == D - 1) {
                        if (DOWN) dst[(long long)c * P + e] += sum;
                        else acc[k] += sum;
                    } else {
                        out[e] = sum;
                    }
                }
            }
            stride *= N;
            if (j < D - 1) __syncthreads();
        }
    }
    if (!DOWN) {
#pragma unroll
        for (int k = 0; k < K; k++) {
            const int e = lane + 64 * k;
            if (e < P) dst[(long long)b * P + e] = acc[k];
        }
    }
}

bool nodes_nest(const NodeSet &coarse, const NodeSet &fine)
{
    if (coarse.d != fine.d) return false;
    for (int j = 0; j < coarse.d; j++)
        if (coarse.n[j] > fine.n[j]) return false;
    return true;
}

static ShiftMeta shift_meta(const NodeSet &nsp, const NodeSet &nsc)
{
    ShiftMeta sm;
    sm.Pp = nsp.P; sm.Pc = nsc.P; sm.NTp = 1; sm.NTc = 1;
    for (int j = 0; j < kMaxD; j++) {
        sm.np[j] = j < nsp.d ? nsp.n[j] : 1;
        sm.nc[j] = j < nsc.d ? nsc.n[j] : 1;
        sm.NTp = std::max(sm.NTp, sm.np[j]);
        sm.NTc = std::max(sm.NTc, sm.nc[j]);
    }
    return sm;
}

void make_shift_tables(const NodeSet &nsp, const NodeSet &nsc, DBuf<float> &tab, hipStream_t s)
{
    F3M_REQUIRE(nodes_nest(nsp, nsc), 33, "child node set is coarser than the parent's");
    ShiftMeta sm = shift_meta(nsp, nsc);
    const int ntab = nsp.d * 2 * sm.NTp * sm.NTc;
    tab.reset((size_t)ntab);
    F3M_LAUNCH(shift_tables_kernel, cdiv(ntab, 64), 64, 0, s, sm, nsp.d, meta_of(nsp), meta_of(nsc), nsp.dt.get(),
               nsp.dw.get(), nsc.dt.get(), tab.get());
    check_launch("shift_tables");
}

void shift_level(bool down, const TreeLevel &parent, const TreeLevel &child, const NodeSet &nsp, const NodeSet &nsc,
                 const float *tab, const float *src, float *dst, hipStream_t s)
{
    check_nodes(nsc);
    ShiftMeta sm = shift_meta(nsp, nsc);
    const int d = nsp.d, ntab = d * 2 * sm.NTp * sm.NTc;
    const int bd = ((sm.Pc + kWave - 1) / kWave) * kWave;
    size_t sh = sizeof(float) * ((size_t)ntab + 2 * (size_t)sm.Pc + (size_t)sm.Pp);
    timer_begin(down ? kL2P : kP2M, s);
    const bool q64 = d == 3 && sm.Pp == 64 && sm.Pc == 64 && sm.NTp == 4 && sm.NTc == 4 && nsp.n[0] == 4 && nsp.n[1] == 4 &&
                     nsc.n[0] == 4 && nsc.n[1] == 4;
    // the same N nodes along every dimension on both levels: one wavefront per parent
    int same = nsp.n[0];
    for (int j = 0; j < d; j++)
        if (nsp.n[j] != same || nsc.n[j] != same) same = 0;
    bool done = false;
#define F3M_SHIFT_T(DD, NNODE)                                                                                         \
    if (!done && !q64 && d == DD && same == NNODE) {                                                                   \
        if (down)                                                                                                      \
            F3M_LAUNCH((shift_tensor_kernel<true, DD, NNODE>), parent.nb, 64, 0, s, tab, parent.nb,                    \
                       parent.childstart.get(), child.cell.get(), src, dst);                                           \
        else                                                                                                           \
            F3M_LAUNCH((shift_tensor_kernel<false, DD, NNODE>), parent.nb, 64, 0, s, tab, parent.nb,                   \
                       parent.childstart.get(), child.cell.get(), src, dst);                                           \
        done = true;                                                                                                   \
    }
    F3M_SHIFT_T(3, 3) F3M_SHIFT_T(3, 5) F3M_SHIFT_T(3, 6) F3M_SHIFT_T(4, 3) F3M_SHIFT_T(5, 3)
#undef F3M_SHIFT_T
    if (getenv("F3M_DEBUG"))
        fprintf(stderr, "shift %s depth %d: %s\n", down ? "down" : "up", parent.depth, done ? "one wavefront per parent" : (q64 ? "4x4x4" : "general"));
    if (done) {
    } else if (q64 && down)
        F3M_LAUNCH((shift_q64_kernel<true>), cdiv(parent.nb, kShiftQWaves), kShiftQWaves * 64, 0, s, tab, parent.nb,
                   parent.childstart.get(), child.cell.get(), src, dst);
    else if (q64)
        F3M_LAUNCH((shift_q64_kernel<false>), cdiv(parent.nb, kShiftQWaves), kShiftQWaves * 64, 0, s, tab, parent.nb,
                   parent.childstart.get(), child.cell.get(), src, dst);
    else if (down)
        F3M_LAUNCH((shift_kernel<true>), parent.nb, bd, sh, s, tab, ntab, sm, d, parent.childstart.get(), child.cell.get(),
                   src, dst);
    else
        F3M_LAUNCH((shift_kernel<false>), parent.nb, bd, sh, s, tab, ntab, sm, d, parent.childstart.get(), child.cell.get(),
                   src, dst);
    timer_end(s);
    check_launch("shift");
}

}  // namespace f3m
