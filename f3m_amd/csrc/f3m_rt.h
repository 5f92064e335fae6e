// Runtime plumbing shared by the engine's translation units: error reporting, a caching device
// memory pool, launch and wave helpers.  gfx950 / wave64 only.
#pragma once

#ifdef F3M_CPU_EMU
#include "hip_emu.h"   // tests/cpu_emu: CPU build of the same sources for logic tests
#define F3M_LAUNCH(kernel, grid, block, shmem, stream, ...) F3M_EMU_LAUNCH(kernel, grid, block, shmem, stream, __VA_ARGS__)
#define F3M_DYN_SHARED(type, name) type *name = reinterpret_cast<type *>(emu::S().dynshared.data())
#else
#include <hip/hip_runtime.h>
#define F3M_LAUNCH(kernel, grid, block, shmem, stream, ...) \
    hipLaunchKernelGGL(kernel, dim3((unsigned)(grid)), dim3((unsigned)(block)), (size_t)(shmem), stream, __VA_ARGS__)
#define F3M_DYN_SHARED(type, name) extern __shared__ __align__(16) unsigned char name##_raw[]; type *name = reinterpret_cast<type *>(name##_raw)
#endif

#include <algorithm>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

namespace f3m {

constexpr int kMaxD = 10;
constexpr int kWave = 64;

// ---- errors -------------------------------------------------------------------------------
struct Error : std::runtime_error {
    int code;
    Error(int c, const std::string &m) : std::runtime_error(m), code(c) {}
};

inline std::string fmt(const char *f, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, f);
    vsnprintf(buf, sizeof(buf), f, ap);
    va_end(ap);
    return buf;
}

#define F3M_HIP(expr)                                                                             \
    do {                                                                                          \
        hipError_t e_ = (expr);                                                                   \
        if (e_ != hipSuccess)                                                                     \
            throw f3m::Error(100, f3m::fmt("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__)); \
    } while (0)

#define F3M_REQUIRE(cond, code, ...)                          \
    do {                                                      \
        if (!(cond)) throw f3m::Error(code, f3m::fmt(__VA_ARGS__)); \
    } while (0)

// ---- device memory pool --------------------------------------------------------------------
// Blocks are cached after release and reused by later requests of a similar size, so steady-state
// calls make no hipMalloc.  All work of one call runs on one stream and every C-ABI entry point
// synchronises that stream before it returns, so a released block is idle when it is handed out
// again.
//
// While the calling thread has an Arena installed (ArenaScope), every request is carved out of that
// fixed block of device memory instead, in order, and nothing is given back until the scope ends:
// a call that must not allocate takes its temporaries from there.  Tables that outlive the call
// (kept in a plan) cannot come from an arena; code that is about to build one calls
// require_tables_may_be_built() first.
struct Arena {
    char *base = nullptr;
    size_t cap = 0, used = 0;
    const char *owner = "";
};
inline thread_local Arena *g_arena = nullptr;
// While set, blocks given back to the pool are parked in this list instead (ParkingLot): work queued on a
// second stream may still use them, so they return to the pool only once the main stream has been made to wait
// for that work.
inline thread_local std::vector<void *> *g_deferred = nullptr;
struct ArenaScope {
    Arena *prev;
    explicit ArenaScope(Arena *a) : prev(g_arena) { g_arena = a; }
    ~ArenaScope() { g_arena = prev; }
    ArenaScope(const ArenaScope &) = delete;
    ArenaScope &operator=(const ArenaScope &) = delete;
};
// Position of the calling thread's arena, and a return to it: what was handed out since is handed out again.  Only for
// temporaries whose kernels are all queued on one stream (a later kernel then reuses the memory after the earlier ones
// are done) and whose host-side owners are gone.  No-ops without an arena.
inline size_t arena_mark() { return g_arena != nullptr ? g_arena->used : 0; }
inline void arena_rewind(size_t mark) { if (g_arena != nullptr) g_arena->used = mark; }
inline void require_tables_may_be_built(const char *what)
{
    if (g_arena != nullptr)
        throw Error(41, fmt("%s: %s of this plan is not built yet; apply the plan once through f3m_plan_apply with the same "
                            "number of columns first (that call builds the plan's tables)", g_arena->owner, what));
}

class Pool {
public:
    static Pool &get() { static Pool p; return p; }
    void *alloc(size_t bytes)
    {
        if (bytes == 0) bytes = 256;
        bytes = (bytes + 255) & ~size_t(255);
        if (Arena *a = g_arena) {
            if (bytes > a->cap - a->used)
                throw Error(42, fmt("%s: the product needs more than the %zu MiB of static scratch memory (request of %zu bytes "
                                    "after %zu in use)", a->owner, a->cap >> 20, bytes, a->used));
            void *p = a->base + a->used;
            a->used += bytes;
            return p;
        }
        int dev = 0;
        (void)hipGetDevice(&dev);                   // blocks are cached per device
        std::lock_guard<std::mutex> g(mu_);
        auto &fr = free_[dev];
        auto it = fr.lower_bound(bytes);
        if (it != fr.end() && it->first <= bytes * 2 + (1 << 20)) {
            void *p = it->second;
            live_[p] = Block{it->first, dev};
            fr.erase(it);
            return p;
        }
        void *p = nullptr;
        hipError_t e = hipMalloc(&p, bytes);
        if (e != hipSuccess) {
            release_cached_locked();
            e = hipMalloc(&p, bytes);
        }
        if (e != hipSuccess) throw Error(101, fmt("device allocation of %zu bytes failed: %s", bytes, hipGetErrorString(e)));
        live_[p] = Block{bytes, dev};
        reserved_ += bytes;
        return p;
    }
    void release(void *p)
    {
        if (!p) return;
        if (g_deferred != nullptr) { g_deferred->push_back(p); return; }
        std::lock_guard<std::mutex> g(mu_);
        auto it = live_.find(p);
        if (it == live_.end()) return;
        free_[it->second.dev].insert({it->second.bytes, p});
        live_.erase(it);
    }
    void release_cached()
    {
        std::lock_guard<std::mutex> g(mu_);
        release_cached_locked();
    }
    size_t reserved() const { return reserved_; }

private:
    struct Block { size_t bytes; int dev; };
    void release_cached_locked()
    {
        for (auto &d : free_)
            for (auto &kv : d.second) { (void)hipFree(kv.second); reserved_ -= kv.first; }
        free_.clear();
    }
    std::mutex mu_;
    std::map<int, std::multimap<size_t, void *>> free_;
    std::map<void *, Block> live_;
    size_t reserved_ = 0;
};

// Parks the blocks that the calling thread gives back between start() and the end of the object's life, and
// returns them to the pool then (also when an exception ends the scope).
class ParkingLot {
public:
    ParkingLot() = default;
    ParkingLot(const ParkingLot &) = delete;
    ParkingLot &operator=(const ParkingLot &) = delete;
    void start()
    {
        if (active_) return;
        prev_ = g_deferred;
        g_deferred = &held_;
        active_ = true;
    }
    ~ParkingLot();

private:
    std::vector<void *> held_, *prev_ = nullptr;
    bool active_ = false;
};

inline ParkingLot::~ParkingLot()
{
    if (!active_) return;
    g_deferred = prev_;
    for (void *p : held_) Pool::get().release(p);
}

template <typename T>
class DBuf {
public:
    DBuf() = default;
    explicit DBuf(size_t n) { reset(n); }
    DBuf(const DBuf &) = delete;
    DBuf &operator=(const DBuf &) = delete;
    DBuf(DBuf &&o) noexcept : p_(o.p_), n_(o.n_) { o.p_ = nullptr; o.n_ = 0; }
    DBuf &operator=(DBuf &&o) noexcept
    {
        if (this != &o) { free(); p_ = o.p_; n_ = o.n_; o.p_ = nullptr; o.n_ = 0; }
        return *this;
    }
    ~DBuf() { free(); }
    void reset(size_t n) { free(); p_ = static_cast<T *>(Pool::get().alloc(n * sizeof(T))); n_ = n; }
    void free() { if (p_) Pool::get().release(p_); p_ = nullptr; n_ = 0; }
    T *get() const { return p_; }
    size_t size() const { return n_; }
    operator T *() const { return p_; }

private:
    T *p_ = nullptr;
    size_t n_ = 0;
};

template <typename T>
inline void d2h(T *dst, const T *src, size_t n, hipStream_t s)
{
    F3M_HIP(hipMemcpyAsync(dst, src, n * sizeof(T), hipMemcpyDeviceToHost, s));
    F3M_HIP(hipStreamSynchronize(s));
}
// Small results the host waits for (box counts, list sizes): a one-workgroup kernel stores them into
// pinned host memory followed by a sequence number, and the host watches that number instead of
// waiting for the stream (a stream wait costs some 15 us more, a copy into pageable memory a staged
// copy command on top).  After kSpinLimitMs of watching the host falls back to the stream wait, which
// also reports a failed kernel.  Pinned blocks are kept for the life of the process.
// What one readback collects: up to kMaxExportSegs runs of 32-bit words from device memory, each to its
// place in the host record; a run marked `clear` is zeroed after it is read (counters that the next
// round of kernels adds to).
constexpr int kMaxExportSegs = 8;
struct ExportList {
    struct Seg { unsigned *src; int nwords, dst, clear; } seg[kMaxExportSegs];
    int nseg = 0, total = 0;
    void add(void *src, int nwords, int dst_word, bool clear = false)
    {
        if (nseg >= kMaxExportSegs) throw Error(103, "too many readback segments");
        seg[nseg++] = Seg{static_cast<unsigned *>(src), nwords, dst_word, clear ? 1 : 0};
        if (dst_word + nwords > total) total = dst_word + nwords;
    }
};
template <int BLOCK>
__global__ void export_segments_kernel(ExportList L, unsigned *__restrict__ dst)
{
    for (int g = 0; g < L.nseg; g++)
        for (int i = threadIdx.x; i < L.seg[g].nwords; i += BLOCK) {
            dst[L.seg[g].dst + i] = L.seg[g].src[i];
            if (L.seg[g].clear) L.seg[g].src[i] = 0;
        }
}
#ifdef F3M_CPU_EMU
template <typename T>
inline void fetch_small(T *dst, const T *src, size_t n, hipStream_t s) { d2h(dst, src, n, s); }
inline void fetch_segments(const ExportList &L, void *dst, hipStream_t s)
{
    F3M_LAUNCH((export_segments_kernel<64>), 1, 64, 0, s, L, static_cast<unsigned *>(dst));
    F3M_HIP(hipStreamSynchronize(s));
}
// a readback in two steps (the emulation has nothing to overlap: begin does it all)
class SegmentFetch {
public:
    void begin(const ExportList &L, hipStream_t s) { words_ = L.total; buf_.assign((size_t)L.total, 0u); if (L.nseg > 0) fetch_segments(L, buf_.data(), s); }
    void wait(void *dst, hipStream_t) { if (words_ > 0) memcpy(dst, buf_.data(), (size_t)words_ * 4); words_ = 0; }
private:
    std::vector<unsigned> buf_;
    int words_ = 0;
};
#else
constexpr size_t kPinnedBytes = 64 << 10, kPinnedHeader = 64;
constexpr int kSpinLimitMs = 50;
class PinnedBlock {
public:
    PinnedBlock()
    {
        {
            std::lock_guard<std::mutex> g(mu());
            if (!spare().empty()) { p_ = spare().back(); spare().pop_back(); }
        }
        if (!p_) {
            F3M_HIP(hipHostMalloc(&p_, kPinnedBytes + kPinnedHeader, hipHostMallocPortable | hipHostMallocMapped | hipHostMallocCoherent));
            memset(p_, 0, kPinnedHeader);
        }
    }
    ~PinnedBlock()
    {
        std::lock_guard<std::mutex> g(mu());
        spare().push_back(p_);
    }
    PinnedBlock(const PinnedBlock &) = delete;
    PinnedBlock &operator=(const PinnedBlock &) = delete;
    unsigned *flag() const { return static_cast<unsigned *>(p_); }            // written by the GPU
    unsigned next_seq() const { return ++static_cast<unsigned *>(p_)[1]; }    // host only
    void *data() const { return static_cast<char *>(p_) + kPinnedHeader; }

private:
    static std::mutex &mu() { static std::mutex m; return m; }
    static std::vector<void *> &spare() { static std::vector<void *> v; return v; }
    void *p_ = nullptr;
};
template <typename T>
__global__ void export_kernel(const T *__restrict__ src, T *__restrict__ dst, int n, unsigned *flag, unsigned seq)
{
    for (int i = threadIdx.x; i < n; i += blockDim.x) dst[i] = src[i];
    __threadfence_system();
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_store(flag, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
// waits until the GPU has stored seq into *flag
inline void await_flag(const unsigned *flag, unsigned seq, hipStream_t s)
{
    // F3M_SPIN_LIMIT_MS overrides the limit; 0 goes straight to the stream wait (test of that path)
    int limit = kSpinLimitMs;
    if (const char *e = getenv("F3M_SPIN_LIMIT_MS")) limit = atoi(e);
    const auto t0 = std::chrono::steady_clock::now();
    for (unsigned spins = 1; limit > 0; spins++) {
        if (__atomic_load_n(flag, __ATOMIC_ACQUIRE) == seq) return;
        __builtin_ia32_pause();
        if ((spins & 0xfff) == 0 && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(limit)) break;
    }
    F3M_HIP(hipStreamSynchronize(s));
    if (__atomic_load_n(flag, __ATOMIC_ACQUIRE) != seq) throw Error(102, "result of a device kernel did not arrive");
}
template <int BLOCK>
__global__ void export_segments_flag_kernel(ExportList L, unsigned *__restrict__ dst, unsigned *flag, unsigned seq)
{
    for (int g = 0; g < L.nseg; g++)
        for (int i = threadIdx.x; i < L.seg[g].nwords; i += BLOCK) {
            dst[L.seg[g].dst + i] = L.seg[g].src[i];
            if (L.seg[g].clear) L.seg[g].src[i] = 0;
        }
    __threadfence_system();
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_store(flag, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
inline void fetch_segments(const ExportList &L, void *dst, hipStream_t s)
{
    if ((size_t)L.total * 4 > kPinnedBytes) throw Error(103, "readback record too large");
    PinnedBlock blk;
    const unsigned seq = blk.next_seq();
    hipLaunchKernelGGL(export_segments_flag_kernel<64>, dim3(1), dim3(64), 0, s, L, static_cast<unsigned *>(blk.data()), blk.flag(), seq);
    F3M_HIP(hipGetLastError());
    await_flag(blk.flag(), seq, s);
    memcpy(dst, blk.data(), (size_t)L.total * 4);
}
// The same readback in two steps: begin queues the kernel that gathers the words into pinned memory, wait returns
// them; kernels queued on the stream in between run while the host waits.
class SegmentFetch {
public:
    void begin(const ExportList &L, hipStream_t s)
    {
        words_ = 0;
        if (L.nseg == 0) return;
        if ((size_t)L.total * 4 > kPinnedBytes) throw Error(103, "readback record too large");
        blk_.reset(new PinnedBlock());
        memset(blk_->data(), 0, (size_t)L.total * 4);      // words between the segments read as zero, not as what the block held before
        seq_ = blk_->next_seq();
        hipLaunchKernelGGL(export_segments_flag_kernel<64>, dim3(1), dim3(64), 0, s, L, static_cast<unsigned *>(blk_->data()),
                           blk_->flag(), seq_);
        F3M_HIP(hipGetLastError());
        words_ = L.total;
    }
    void wait(void *dst, hipStream_t s)
    {
        if (words_ == 0) return;
        await_flag(blk_->flag(), seq_, s);
        memcpy(dst, blk_->data(), (size_t)words_ * 4);
        words_ = 0;
        blk_.reset();
    }
private:
    std::unique_ptr<PinnedBlock> blk_;
    unsigned seq_ = 0;
    int words_ = 0;
};
template <typename T>
inline void fetch_small(T *dst, const T *src, size_t n, hipStream_t s)
{
    if (n * sizeof(T) > kPinnedBytes) { d2h(dst, src, n, s); return; }
    PinnedBlock blk;
    const unsigned seq = blk.next_seq();
    hipLaunchKernelGGL(export_kernel<T>, dim3(1), dim3(256), 0, s, src, static_cast<T *>(blk.data()), (int)n, blk.flag(), seq);
    F3M_HIP(hipGetLastError());
    await_flag(blk.flag(), seq, s);
    memcpy(dst, blk.data(), n * sizeof(T));
}
#endif

template <typename T>
inline void h2d(T *dst, const T *src, size_t n, hipStream_t s)
{
    F3M_HIP(hipMemcpyAsync(dst, src, n * sizeof(T), hipMemcpyHostToDevice, s));
    F3M_HIP(hipStreamSynchronize(s));   // source is pageable host memory that may go out of scope
}

inline unsigned cdiv(long long a, long long b) { return (unsigned)((a + b - 1) / b); }

inline void check_launch(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) throw Error(102, fmt("launch of %s failed: %s", what, hipGetErrorString(e)));
}

// Fills device memory with a byte value, as a kernel (a memset node recorded into a captured graph has
// given wrong results on replays on this GPU pool, and the engine's fills are small or sit next to
// kernels of the same stream anyway).  p and bytes are multiples of 4.
template <int BLOCK>
__global__ void __launch_bounds__(BLOCK) fill_words_kernel(unsigned *__restrict__ p, size_t n32, unsigned word)
{
    size_t i = (size_t)blockIdx.x * BLOCK + threadIdx.x;
    const size_t step = (size_t)gridDim.x * BLOCK;
    for (; i < n32; i += step) p[i] = word;
}
inline void dev_fill(void *p, int byte, size_t bytes, hipStream_t s)
{
    if (bytes == 0) return;
    if ((reinterpret_cast<uintptr_t>(p) | bytes) & 3) throw Error(104, "fill of a range that is not a multiple of 4 bytes");
    const unsigned b = (unsigned)byte & 255u, word = b * 0x01010101u;
    const size_t n32 = bytes / 4;
    // workgroups of one wavefront: they find room beside a kernel that keeps the compute units full
    const unsigned grid = (unsigned)std::min<size_t>((n32 + 63) / 64, 32768);
    F3M_LAUNCH((fill_words_kernel<64>), grid, 64, 0, s, static_cast<unsigned *>(p), n32, word);
    check_launch("fill");
}

// ---- wave helpers ---------------------------------------------------------------------------
#ifdef F3M_CPU_EMU
// Every wave-wide operation carries the source line of its call: the emulation stops when the lanes of one wavefront
// arrive at operations of different lines, as they do when an exchange sits inside a branch that only some lanes
// take (on the GPU such an exchange sees the lanes of the branch only).
__device__ inline unsigned long long wave_ballot(bool p, int site = __builtin_LINE()) { return emu::ballot(p, site); }
// orders the LDS accesses of the lanes of one wavefront (the lanes run in lockstep on the GPU)
__device__ inline void wave_sync(int site = __builtin_LINE()) { (void)emu::ballot(false, site); }
__device__ inline unsigned lane_id() { return emu::S().cur->tid % 64; }
__device__ inline float fast_exp2(float x) { return exp2f(x); }
__device__ inline float fast_rcp(float x) { return 1.0f / x; }
__device__ inline float wave_shfl_f(float v, int src, int site = __builtin_LINE())
{
    uint32_t u;
    memcpy(&u, &v, 4);
    u = emu::shfl_bits(u, src, site);
    memcpy(&v, &u, 4);
    return v;
}
// value of lane (l & ~3) | K of the same group of four lanes
template <int K> __device__ inline float quad_bcast(float v, int site = __builtin_LINE())
{
    return wave_shfl_f(v, (int)((lane_id() & ~3u) | K), site);
}
__device__ inline int wave_shfl_i(int v, int src, int site = __builtin_LINE()) { return (int)emu::shfl_bits((uint32_t)v, src, site); }
__device__ inline int wave_uniform(int v) { return v; }
__device__ inline int wave_readlane(int v, int src, int site = __builtin_LINE())   // src uniform
{
    return (int)emu::shfl_bits((uint32_t)v, src, site);
}
__device__ inline float wave_shfl_xor_f(float v, int mask, int site = __builtin_LINE())
{
    uint32_t u;
    memcpy(&u, &v, 4);
    u = emu::shfl_bits(u, (int)(lane_id() ^ (unsigned)mask), site);
    memcpy(&v, &u, 4);
    return v;
}
struct f32x16 {
    float v[16];
    float &operator[](int i) { return v[i]; }
    const float &operator[](int i) const { return v[i]; }
};
// IEEE binary16 stand-ins for the CPU build (round to nearest even, subnormals kept)
struct half_t { uint16_t bits; };
__device__ inline half_t to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u, mant = x & 0x7fffffu;
    int exp = (int)((x >> 23) & 0xff) - 127 + 15;
    uint16_t h;
    if (((x >> 23) & 0xff) == 0xff) h = (uint16_t)(sign | 0x7c00u | (mant ? 0x200u : 0));
    else if (exp >= 31) h = (uint16_t)(sign | 0x7c00u);
    else if (exp <= 0) {
        if (exp < -10) h = (uint16_t)sign;
        else {
            mant |= 0x800000u;
            int shift = 14 - exp;
            uint32_t hm = mant >> shift, rem = mant & ((1u << shift) - 1), halfway = 1u << (shift - 1);
            if (rem > halfway || (rem == halfway && (hm & 1))) hm++;
            h = (uint16_t)(sign | hm);
        }
    } else {
        uint32_t hm = mant >> 13, rem = mant & 0x1fffu;
        uint32_t v = ((uint32_t)exp << 10) | hm;
        if (rem > 0x1000u || (rem == 0x1000u && (hm & 1))) v++;
        h = (uint16_t)(sign | v);
    }
    return half_t{h};
}
__device__ inline float half_to_float(half_t hv)
{
    uint32_t h = hv.bits, sign = (h & 0x8000u) << 16, exp = (h >> 10) & 0x1f, mant = h & 0x3ffu, x;
    if (exp == 0) {
        if (mant == 0) x = sign;
        else {
            int e = -1;
            do { e++; mant <<= 1; } while (!(mant & 0x400u));
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | ((mant & 0x3ffu) << 13);
        }
    } else if (exp == 31) x = sign | 0x7f800000u | (mant << 13);
    else x = sign | ((exp - 15 + 127) << 23) | (mant << 13);
    float f;
    memcpy(&f, &x, 4);
    return f;
}
struct h8 {
    half_t v[8];
    half_t &operator[](int i) { return v[i]; }
    const half_t &operator[](int i) const { return v[i]; }
};
// D = A(32x16) B(16x32) + C with f16 inputs and fp32 accumulation: lane l supplies row l%32 of A and
// column l%32 of B for the eight inner indices of its half-wave and holds D[8(r/4) + 4(l/32) + r%4][l%32]
// in element r
__device__ inline f32x16 mfma_32x32x16_f16(h8 a, h8 b, f32x16 c, int site = __builtin_LINE())
{
    uint32_t A[4][64], B[4][64];
    uint32_t wa[4], wb[4];
    memcpy(wa, &a, 16);
    memcpy(wb, &b, 16);
    for (int w = 0; w < 4; w++) { emu::gather_bits(wa[w], A[w], site); emu::gather_bits(wb[w], B[w], site); }
    const unsigned l = lane_id(), j = l & 31, h = l >> 5;
    for (int r = 0; r < 16; r++) {
        unsigned i = 8 * (r / 4) + 4 * h + (r % 4);
        double acc = c.v[r];
        for (int hh = 0; hh < 2; hh++)
            for (int e = 0; e < 8; e++) {
                uint32_t aw = A[e / 2][i + 32 * hh], bw = B[e / 2][j + 32 * hh];
                half_t ah{(uint16_t)((e & 1) ? (aw >> 16) : (aw & 0xffff))}, bh{(uint16_t)((e & 1) ? (bw >> 16) : (bw & 0xffff))};
                acc += (double)half_to_float(ah) * (double)half_to_float(bh);
            }
        c.v[r] = (float)acc;
    }
    return c;
}
#else
__device__ __forceinline__ unsigned long long wave_ballot(bool p) { return __ballot(p); }
// orders the LDS accesses of the lanes of one wavefront (the lanes run in lockstep; this only keeps the
// compiler from moving memory operations across the point)
__device__ __forceinline__ void wave_sync() { __builtin_amdgcn_wave_barrier(); }
__device__ __forceinline__ unsigned lane_id() { return __lane_id(); }
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }   // v_rcp_f32, 1 ulp
__device__ __forceinline__ float wave_shfl_f(float v, int src) { return __shfl(v, src, 64); }
// value of lane (l & ~3) | K of the same group of four lanes (DPP quad_perm:[K,K,K,K], no LDS traffic)
template <int K> __device__ __forceinline__ float quad_bcast(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), K * 0x55, 0xf, 0xf, false));
}
__device__ __forceinline__ int wave_shfl_i(int v, int src) { return __shfl(v, src, 64); }
// value of one lane, the same lane for the whole wavefront (v_readlane_b32: the result is scalar)
__device__ __forceinline__ int wave_readlane(int v, int src) { return __builtin_amdgcn_readlane(v, src); }
// a value that is the same in every lane, as a scalar (no exchange: the first active lane's copy)
__device__ __forceinline__ int wave_uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ float wave_shfl_xor_f(float v, int mask) { return __shfl_xor(v, mask, 64); }
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 half_t;
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
// Rounds the fp32 value it is given.  The empty asm statement hides where f comes from: fused with a
// preceding multiply-add (v_fma_mixlo_f16) the conversion would round the unrounded sum instead, and
// code that also uses the fp32 value (lo = f - hi) would then see two different roundings of f at
// exact ties, an error of one f16 unit in the last place.
__device__ __forceinline__ half_t to_half(float f)
{
    asm("" : "+v"(f));
    return (_Float16)f;
}
__device__ __forceinline__ float half_to_float(half_t h) { return (float)h; }
// D = A(32x16) B(16x32) + C with f16 inputs and fp32 accumulation (v_mfma_f32_32x32x16_f16): lane l
// supplies row l%32 of A and column l%32 of B for the eight inner indices of its half-wave and holds
// D[8(r/4) + 4(l/32) + r%4][l%32] in element r
__device__ __forceinline__ f32x16 mfma_32x32x16_f16(h8 a, h8 b, f32x16 c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
#endif

}  // namespace f3m
