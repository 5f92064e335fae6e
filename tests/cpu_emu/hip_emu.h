// TEST INFRASTRUCTURE ONLY: a minimal single-OS-thread emulation of the HIP execution model, so
// that the engine's kernel sources can be compiled with g++ and run on a CPU for logic tests and
// for debugging with gdb / sanitizers.  The product never links this; the Python package loads only
// the gfx950 library and fails if it is missing.
//
// Model: blocks run one after another; the threads of a block are fibers (ucontext) scheduled
// round-robin; __syncthreads and wave-level operations are generation barriers that yield.
// Wave size is 64.  Only 1-D grids and blocks.
#pragma once
#include <ucontext.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __shared__ static
#define __launch_bounds__(...)
#define __align__(n) alignas(n)

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

typedef int hipError_t;
typedef void *hipStream_t;
enum { hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorOutOfMemory = 2 };
enum hipMemcpyKind { hipMemcpyHostToDevice, hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice, hipMemcpyDefault };

// Streams.  The caller's stream (any handle the program did not create, normally null) runs its work at once, in
// program order.  A stream that the program CREATES is lazy: its work is queued and runs only when something waits
// for it -- an event of that stream that another stream or the host waits for, a synchronisation -- which is the
// latest moment the HIP model allows.  Host code that gives a buffer back, or reuses it on the caller's stream, while
// work of a created stream still needs it therefore computes with the wrong data here, and the tests see it.
// F3M_EMU_STREAMS=eager makes created streams run at once as well (the earliest schedule).
namespace emu {
struct Stream {
    std::deque<std::function<void()>> q;
    size_t queued = 0, done = 0;
    void run_until(size_t target)
    {
        while (done < target && !q.empty()) {
            std::function<void()> f = std::move(q.front());
            q.pop_front();
            done++;
            f();
        }
    }
};
struct Event {
    Stream *stream = nullptr;     // lazy stream the event was recorded on (null: recorded on an eager stream, complete)
    size_t pos = 0;               // work of that stream queued before the event
};
inline std::vector<Stream *> &streams() { static std::vector<Stream *> v; return v; }
inline Stream *lazy(void *s)
{
    for (Stream *t : streams()) if (t == s) return t;
    return nullptr;
}
inline bool eager_streams()
{
    const char *e = getenv("F3M_EMU_STREAMS");
    return e && !strcmp(e, "eager");
}
// runs f now, or queues it if `stream` is a lazy stream
inline void submit(void *stream, std::function<void()> f)
{
    Stream *st = lazy(stream);
    if (st && !eager_streams()) { st->q.push_back(std::move(f)); st->queued++; }
    else f();
}
inline void drain_all() { for (Stream *t : streams()) t->run_until(t->queued); }
}  // namespace emu
typedef emu::Event *hipEvent_t;
enum { hipStreamNonBlocking = 1, hipEventDisableTiming = 2 };

inline hipError_t hipMalloc(void **p, size_t n) { *p = malloc(n ? n : 1); return *p ? hipSuccess : hipErrorOutOfMemory; }
inline hipError_t hipFree(void *p) { free(p); return hipSuccess; }
inline hipError_t hipMemcpy(void *d, const void *s, size_t n, hipMemcpyKind) { emu::drain_all(); memcpy(d, s, n); return hipSuccess; }
inline hipError_t hipMemcpyAsync(void *d, const void *s, size_t n, hipMemcpyKind, hipStream_t st)
{
    emu::submit(st, [=]() { memcpy(d, s, n); });
    return hipSuccess;
}
inline hipError_t hipMemsetAsync(void *d, int v, size_t n, hipStream_t st)
{
    emu::submit(st, [=]() { memset(d, v, n); });
    return hipSuccess;
}
inline hipError_t hipStreamSynchronize(hipStream_t st)
{
    if (emu::Stream *t = emu::lazy(st)) t->run_until(t->queued);
    return hipSuccess;
}
inline hipError_t hipDeviceSynchronize() { emu::drain_all(); return hipSuccess; }
inline hipError_t hipGetLastError() { return hipSuccess; }
inline const char *hipGetErrorString(hipError_t) { return "emu"; }
inline hipError_t hipGetDevice(int *d) { *d = 0; return hipSuccess; }
inline hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned) { emu::Stream *t = new emu::Stream(); emu::streams().push_back(t); *s = t; return hipSuccess; }
inline hipError_t hipEventCreateWithFlags(hipEvent_t *e, unsigned) { *e = new emu::Event(); return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t e, hipStream_t st)
{
    emu::Stream *t = emu::eager_streams() ? nullptr : emu::lazy(st);
    e->stream = t;
    e->pos = t ? t->queued : 0;
    return hipSuccess;
}
// the waiting stream may not pass the event: an eager stream (or the host) makes the event's stream catch up now, a
// lazy stream does so when it gets there
inline hipError_t hipStreamWaitEvent(hipStream_t st, hipEvent_t e, unsigned)
{
    emu::Stream *src = e->stream;
    if (!src) return hipSuccess;
    const size_t pos = e->pos;
    emu::submit(st, [=]() { src->run_until(pos); });
    return hipSuccess;
}

namespace emu {

constexpr int WAVE = 64;
constexpr size_t STACK = 256 * 1024;

struct Wave {
    uint64_t bits[2];
    uint32_t vals[2][WAVE];
    int arrived, gen, alive;
    int site;          // source line of the wave-wide operation that the lanes of this generation are arriving at
};

struct Fiber {
    ucontext_t ctx;
    unsigned tid;
    bool done;
};

struct State {
    ucontext_t main_ctx;
    std::vector<Fiber> fibers;
    std::vector<char *> stacks;
    std::vector<Wave> waves;
    Fiber *cur = nullptr;
    unsigned block = 0, bdim = 1, gdim = 1;
    int bar_arrived = 0, bar_gen = 0, alive = 0;
    std::function<void()> body;
    std::vector<char> dynshared;
};

inline State &S() { static State s; return s; }

inline void yield() { State &s = S(); swapcontext(&s.cur->ctx, &s.main_ctx); }

inline void trampoline()
{
    State &s = S();
    s.body();
    Fiber *f = s.cur;
    f->done = true;
    // leaving threads stop counting towards barriers
    s.alive--;
    if (s.alive > 0 && s.bar_arrived == s.alive) { s.bar_arrived = 0; s.bar_gen++; }
    Wave &w = s.waves[f->tid / WAVE];
    w.alive--;
    if (w.alive > 0 && w.arrived == w.alive) { w.arrived = 0; w.bits[(w.gen & 1) ^ 1] = 0; w.gen++; }
    swapcontext(&f->ctx, &s.main_ctx);
}

inline void launch(unsigned grid, unsigned block, size_t shmem, std::function<void()> body)
{
    State &s = S();
    if (block == 0 || grid == 0) return;
    if (s.fibers.size() < block) {
        size_t old = s.fibers.size();
        s.fibers.resize(block);
        s.stacks.resize(block, nullptr);
        for (size_t i = old; i < block; i++) s.stacks[i] = (char *)malloc(STACK);
    }
    s.dynshared.assign(shmem + 16, 0);
    s.body = body;
    s.bdim = block; s.gdim = grid;
    unsigned nw = (block + WAVE - 1) / WAVE;
    s.waves.resize(nw);
    for (unsigned b = 0; b < grid; b++) {
        s.block = b;
        s.bar_arrived = 0; s.bar_gen = 0; s.alive = (int)block;
        for (unsigned w = 0; w < nw; w++) {
            Wave &W = s.waves[w];
            memset(&W, 0, sizeof(W));
            W.alive = (int)std::min<unsigned>(WAVE, block - w * WAVE);
        }
        for (unsigned t = 0; t < block; t++) {
            Fiber &f = s.fibers[t];
            f.tid = t; f.done = false;
            getcontext(&f.ctx);
            f.ctx.uc_stack.ss_sp = s.stacks[t];
            f.ctx.uc_stack.ss_size = STACK;
            f.ctx.uc_link = &s.main_ctx;
            makecontext(&f.ctx, (void (*)())trampoline, 0);
        }
        int remaining = (int)block;
        long sweeps = 0;
        while (remaining > 0) {
            remaining = 0;
            for (unsigned t = 0; t < block; t++) {
                Fiber &f = s.fibers[t];
                if (f.done) continue;
                s.cur = &f;
                swapcontext(&s.main_ctx, &f.ctx);
                if (!f.done) remaining++;
            }
            if (++sweeps > 100000000L) { fprintf(stderr, "emu: kernel does not terminate (deadlocked barrier?)\n"); abort(); }
        }
    }
    s.cur = nullptr;
}

inline void syncthreads()
{
    State &s = S();
    int my = s.bar_gen;
    if (++s.bar_arrived == s.alive) { s.bar_arrived = 0; s.bar_gen++; }
    else while (s.bar_gen == my) yield();
}

inline Wave &wave() { State &s = S(); return s.waves[s.cur->tid / WAVE]; }

// site: the source line of the calling wave-wide operation.  Lanes of one wavefront that meet here from different
// lines have diverged around an exchange (one sits in a branch that not every lane takes): on the GPU such an exchange
// reads lanes that are switched off, so the emulation refuses to go on.
inline void wave_barrier(Wave &w, int site)
{
    int my = w.gen;
    if (w.arrived == 0) w.site = site;
    else if (w.site != site) {
        fprintf(stderr, "emu: lanes of one wavefront are at different wave-wide operations (source lines %d and %d): "
                        "an exchange inside a branch that only some lanes take?\n", w.site, site);
        abort();
    }
    if (++w.arrived == w.alive) { w.arrived = 0; w.bits[(w.gen & 1) ^ 1] = 0; w.gen++; }
    else while (w.gen == my) yield();
}

inline uint64_t ballot(bool pred, int site)
{
    Wave &w = wave();
    int slot = w.gen & 1;
    unsigned lane = S().cur->tid % WAVE;
    if (pred) w.bits[slot] |= 1ull << lane;
    wave_barrier(w, site);
    return w.bits[slot];
}

inline uint32_t shfl_bits(uint32_t v, int src, int site)
{
    Wave &w = wave();
    int slot = w.gen & 1;
    unsigned lane = S().cur->tid % WAVE;
    w.vals[slot][lane] = v;
    wave_barrier(w, site);
    return w.vals[slot][src & (WAVE - 1)];
}

// every lane's value of the wave (exited lanes keep their last deposit)
inline void gather_bits(uint32_t v, uint32_t *out, int site)
{
    Wave &w = wave();
    int slot = w.gen & 1;
    unsigned lane = S().cur->tid % WAVE;
    w.vals[slot][lane] = v;
    wave_barrier(w, site);
    memcpy(out, w.vals[slot], sizeof(uint32_t) * WAVE);
}

struct Idx { unsigned x; };
struct TidProxy { struct X { operator unsigned() const { return S().cur->tid; } } x; };
struct BidProxy { struct X { operator unsigned() const { return S().block; } } x; };
struct BdimProxy { struct X { operator unsigned() const { return S().bdim; } } x; };
struct GdimProxy { struct X { operator unsigned() const { return S().gdim; } } x; };

}  // namespace emu

static emu::TidProxy threadIdx;
static emu::BidProxy blockIdx;
static emu::BdimProxy blockDim;
static emu::GdimProxy gridDim;

inline void __syncthreads() { emu::syncthreads(); }

template <typename T> inline T atomicAdd(T *p, T v) { T o = *p; *p = o + v; return o; }
template <typename T> inline T atomicMax(T *p, T v) { T o = *p; if (v > o) *p = v; return o; }
template <typename T> inline T atomicMin(T *p, T v) { T o = *p; if (v < o) *p = v; return o; }
template <typename T> inline T atomicCAS(T *p, T cmp, T v) { T o = *p; if (o == cmp) *p = v; return o; }
template <typename T> inline T atomicOr(T *p, T v) { T o = *p; *p = o | v; return o; }

inline int __popcll(unsigned long long v) { return __builtin_popcountll(v); }
inline int __popc(unsigned v) { return __builtin_popcount(v); }
inline int __ffsll(unsigned long long v) { return __builtin_ffsll((long long)v); }
inline int __clz(unsigned v) { return v ? __builtin_clz(v) : 32; }

namespace emu {
template <typename K, typename... A>
inline void launch_k(unsigned grid, unsigned block, size_t shmem, K kernel, A... args)
{
    launch(grid, block, shmem, [=]() { kernel(args...); });
}
template <typename K, typename... A>
inline void launch_on(void *stream, unsigned grid, unsigned block, size_t shmem, K kernel, A... args)
{
    submit(stream, [=]() { launch(grid, block, shmem, [=]() { kernel(args...); }); });
}
}  // namespace emu
#define F3M_EMU_LAUNCH(kernel, grid, block, shmem, stream, ...) \
    emu::launch_on((void *)(stream), (unsigned)(grid), (unsigned)(block), (size_t)(shmem), kernel, __VA_ARGS__)

struct float4 { float x, y, z, w; };
inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
using std::max;
using std::min;
