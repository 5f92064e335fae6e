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

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
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
class Pool {
public:
    static Pool &get() { static Pool p; return p; }
    void *alloc(size_t bytes)
    {
        if (bytes == 0) bytes = 256;
        bytes = (bytes + 255) & ~size_t(255);
        std::lock_guard<std::mutex> g(mu_);
        auto it = free_.lower_bound(bytes);
        if (it != free_.end() && it->first <= bytes * 2 + (1 << 20)) {
            void *p = it->second;
            live_[p] = it->first;
            free_.erase(it);
            return p;
        }
        void *p = nullptr;
        hipError_t e = hipMalloc(&p, bytes);
        if (e != hipSuccess) {
            release_cached_locked();
            e = hipMalloc(&p, bytes);
        }
        if (e != hipSuccess) throw Error(101, fmt("device allocation of %zu bytes failed: %s", bytes, hipGetErrorString(e)));
        live_[p] = bytes;
        reserved_ += bytes;
        return p;
    }
    void release(void *p)
    {
        if (!p) return;
        std::lock_guard<std::mutex> g(mu_);
        auto it = live_.find(p);
        if (it == live_.end()) return;
        free_.insert({it->second, p});
        live_.erase(it);
    }
    void release_cached()
    {
        std::lock_guard<std::mutex> g(mu_);
        release_cached_locked();
    }
    size_t reserved() const { return reserved_; }

private:
    void release_cached_locked()
    {
        for (auto &kv : free_) { (void)hipFree(kv.second); reserved_ -= kv.first; }
        free_.clear();
    }
    std::mutex mu_;
    std::multimap<size_t, void *> free_;
    std::map<void *, size_t> live_;
    size_t reserved_ = 0;
};

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

// ---- wave helpers ---------------------------------------------------------------------------
#ifdef F3M_CPU_EMU
__device__ inline unsigned long long wave_ballot(bool p) { return emu::ballot(p); }
__device__ inline unsigned lane_id() { return emu::S().cur->tid % 64; }
__device__ inline float fast_exp2(float x) { return exp2f(x); }
__device__ inline int wave_shfl_i(int v, int src) { return (int)emu::shfl_bits((uint32_t)v, src); }
#else
__device__ __forceinline__ unsigned long long wave_ballot(bool p) { return __ballot(p); }
__device__ __forceinline__ unsigned lane_id() { return __lane_id(); }
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ int wave_shfl_i(int v, int src) { return __shfl(v, src, 64); }
#endif

}  // namespace f3m
