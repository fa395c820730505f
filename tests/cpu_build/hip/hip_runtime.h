// Stand-in for <hip/hip_runtime.h> that lets g++ compile the BVH builder's kernels for the CPU (test infrastructure:
// bounds and logic of the kernels are checked on the host before they ever run on a GPU).  A launch runs the grid's
// workgroups one after the other; the threads of a workgroup take turns on one OS thread and hand over at barriers,
// wave-wide votes and shuffles, so shared memory, barriers and atomics behave as the kernels expect, every run the
// same.  Only what the builder uses is provided (x86-64).
#pragma once
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __restrict__
#define __shared__ static
#define __launch_bounds__(x)
#define __align__(x) alignas(x)
#define HIP_SYMBOL(x) x

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned a = 1, unsigned b = 1, unsigned c = 1) : x(a), y(b), z(c) {}
};
struct int4 { int x, y, z, w; };
struct int2 { int x, y; };
struct float2 { float x, y; };
struct float4 { float x, y, z, w; };
inline int4 make_int4(int a, int b, int c, int d) { return int4{a, b, c, d}; }
inline int2 make_int2(int a, int b) { return int2{a, b}; }
inline float2 make_float2(float a, float b) { return float2{a, b}; }
inline float4 make_float4(float a, float b, float c, float d) { return float4{a, b, c, d}; }

typedef void *hipStream_t;
typedef int hipError_t;
enum { hipSuccess = 0, hipMemcpyDeviceToHost = 2, hipHostMallocDefault = 0 };
inline const char *hipGetErrorString(hipError_t) { return "cpu build"; }
inline hipError_t hipMalloc(void **p, size_t n) { *p = std::aligned_alloc(256, (n + 255) / 256 * 256 + 256); return *p ? 0 : 1; }
inline hipError_t hipHostMalloc(void **p, size_t n, int) { return hipMalloc(p, n); }
inline hipError_t hipFree(void *p) { std::free(p); return 0; }
inline hipError_t hipHostFree(void *p) { std::free(p); return 0; }
inline hipError_t hipMemset(void *p, int v, size_t n) { std::memset(p, v, n); return 0; }
inline hipError_t hipMemcpyAsync(void *d, const void *s, size_t n, int, hipStream_t) { std::memcpy(d, s, n); return 0; }
inline hipError_t hipMemcpy(void *d, const void *s, size_t n, int) { std::memcpy(d, s, n); return 0; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return 0; }
inline hipError_t hipGetLastError() { return 0; }
template <class T> inline hipError_t hipGetSymbolAddress(void **p, T &sym) { *p = (void *)&sym; return 0; }

namespace cpu_gpu {
// A workgroup's threads are fibers of one OS thread, switched by hand: a fiber runs until it reaches a barrier (of the
// workgroup or of its wave) or the end of the kernel, then the next one runs.  A barrier opens when every fiber that
// is still alive in the workgroup (wave) waits at it - what the hardware does - and a round in which nothing can run
// and no barrier can open is reported as a deadlock (threads of one wave or workgroup waiting at different barriers).
constexpr unsigned kWave = 64, kMaxBlock = 1024, kStackBytes = 256 * 1024;
enum State { kReady, kWaitBlock, kWaitWave, kDone };
struct Fiber { void *sp; State state; };
struct Thread { unsigned x, y, z; };
inline Fiber g_fiber[kMaxBlock];
inline char *g_stacks = nullptr;
inline void *g_main_sp = nullptr;
inline unsigned g_cur = 0, g_block = 0, g_live_block = 0, g_wait_block = 0, g_live_wave[kMaxBlock / kWave], g_wait_wave[kMaxBlock / kWave];
inline dim3 g_bdim, g_gdim;
inline const std::function<void()> *g_body = nullptr;
inline uint64_t g_bits[kMaxBlock];
inline bool g_pred[kMaxBlock];

extern "C" void cpu_gpu_switch(void **save_sp, void *load_sp);
asm(R"(
.text
.globl cpu_gpu_switch
.type cpu_gpu_switch,@function
cpu_gpu_switch:
    pushq %rbp
    pushq %rbx
    pushq %r12
    pushq %r13
    pushq %r14
    pushq %r15
    movq %rsp, (%rdi)
    movq %rsi, %rsp
    popq %r15
    popq %r14
    popq %r13
    popq %r12
    popq %rbx
    popq %rbp
    ret
.size cpu_gpu_switch,.-cpu_gpu_switch
)");

inline void to_scheduler() { cpu_gpu_switch(&g_fiber[g_cur].sp, g_main_sp); }
extern "C" inline void cpu_gpu_entry() {
    (*g_body)();
    g_fiber[g_cur].state = kDone;   // a thread that has left takes no part in later votes or barriers
    g_pred[g_cur] = false;
    --g_live_block;
    --g_live_wave[g_cur / kWave];
    to_scheduler();
    std::abort();   // never resumed
}
template <class F> void launch(dim3 grid, dim3 block, F body_fn) {
    const unsigned nt = block.x;
    if (nt == 0 || nt > kMaxBlock || grid.x == 0) return;
    if (!g_stacks) g_stacks = static_cast<char *>(std::aligned_alloc(4096, (size_t)kMaxBlock * kStackBytes));
    const std::function<void()> body = body_fn;
    g_body = &body;
    g_bdim = block;
    g_gdim = grid;
    for (unsigned b = 0; b < grid.x; ++b) {
        g_block = b;
        g_live_block = nt;
        g_wait_block = 0;
        for (unsigned w = 0; w < kMaxBlock / kWave; ++w) {
            g_live_wave[w] = w * kWave < nt ? std::min(kWave, nt - w * kWave) : 0;
            g_wait_wave[w] = 0;
        }
        for (unsigned t = 0; t < nt; ++t) {
            char *top = g_stacks + (size_t)(t + 1) * kStackBytes;   // 16-byte aligned
            void **sp = reinterpret_cast<void **>(top - 16 - 48);
            for (int k = 0; k < 6; ++k) sp[k] = nullptr;
            sp[6] = reinterpret_cast<void *>(&cpu_gpu_entry);
            g_fiber[t].sp = sp;
            g_fiber[t].state = kReady;
            g_pred[t] = false;
        }
        while (g_live_block != 0) {
            bool progressed = false;
            for (unsigned t = 0; t < nt; ++t) {
                if (g_fiber[t].state != kReady) continue;
                g_cur = t;
                cpu_gpu_switch(&g_main_sp, g_fiber[t].sp);
                progressed = true;
            }
            for (unsigned w = 0; w * kWave < nt; ++w) {
                if (g_wait_wave[w] != 0 && g_wait_wave[w] == g_live_wave[w]) {
                    for (unsigned t = w * kWave; t < std::min(nt, (w + 1) * kWave); ++t)
                        if (g_fiber[t].state == kWaitWave) g_fiber[t].state = kReady;
                    g_wait_wave[w] = 0;
                    progressed = true;
                }
            }
            if (g_wait_block != 0 && g_wait_block == g_live_block) {
                for (unsigned t = 0; t < nt; ++t)
                    if (g_fiber[t].state == kWaitBlock) g_fiber[t].state = kReady;
                g_wait_block = 0;
                progressed = true;
            }
            if (!progressed) {
                std::fprintf(stderr, "cpu build: deadlock in workgroup %u (%u alive, %u at the workgroup barrier)\n", b,
                             g_live_block, g_wait_block);
                std::abort();
            }
        }
    }
    g_body = nullptr;
}
inline void block_barrier() {
    g_fiber[g_cur].state = kWaitBlock;
    ++g_wait_block;
    to_scheduler();
}
inline void wave_barrier() {
    g_fiber[g_cur].state = kWaitWave;
    ++g_wait_wave[g_cur / kWave];
    to_scheduler();
}
inline unsigned lane() { return g_cur % kWave; }
inline Thread tid() { return Thread{g_cur, 0, 0}; }
inline Thread bid() { return Thread{g_block, 0, 0}; }
inline uint64_t exchange(uint64_t v, unsigned from) {
    g_bits[g_cur] = v;
    wave_barrier();
    const uint64_t r = g_bits[(g_cur / kWave) * kWave + from % kWave];
    wave_barrier();
    return r;
}
}  // namespace cpu_gpu

#define threadIdx (cpu_gpu::tid())
#define blockIdx (cpu_gpu::bid())
#define blockDim cpu_gpu::g_bdim
#define gridDim cpu_gpu::g_gdim
#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
    cpu_gpu::launch(grid, block, [&] { kernel(__VA_ARGS__); })

inline void __syncthreads() { cpu_gpu::block_barrier(); }
// The lanes of a wave execute in step on the hardware; where a kernel leans on that (all lanes read a word before one
// of them writes it) it says so with this builtin, which costs nothing there and is a real barrier here.
inline void __builtin_amdgcn_wave_barrier() { cpu_gpu::wave_barrier(); }
inline unsigned __lane_id() { return cpu_gpu::lane(); }
inline uint64_t __ballot(bool p) {
    using namespace cpu_gpu;
    g_pred[g_cur] = p;
    wave_barrier();
    uint64_t m = 0;
    const unsigned base = (g_cur / kWave) * kWave;
    for (unsigned k = 0; k < kWave && base + k < g_bdim.x; ++k)
        if (g_pred[base + k]) m |= 1ull << k;
    wave_barrier();
    g_pred[g_cur] = false;
    return m;
}
template <class T> inline T cpu_bits_exchange(T v, unsigned from) {
    uint64_t b = 0;
    std::memcpy(&b, &v, sizeof(T));
    b = cpu_gpu::exchange(b, from);
    T r;
    std::memcpy(&r, &b, sizeof(T));
    return r;
}
template <class T> inline T __shfl_xor(T v, int mask) { return cpu_bits_exchange(v, cpu_gpu::lane() ^ (unsigned)mask); }
template <class T> inline T __shfl_up(T v, int off) {
    const unsigned l = cpu_gpu::lane();
    return cpu_bits_exchange(v, l >= (unsigned)off ? l - off : l);
}
template <class T> inline T __shfl_down(T v, int off) {
    const unsigned l = cpu_gpu::lane();
    return cpu_bits_exchange(v, l + off < cpu_gpu::kWave ? l + off : l);
}
inline int __popcll(uint64_t v) { return __builtin_popcountll(v); }
inline int __clz(uint32_t v) { return v ? __builtin_clz(v) : 32; }
inline uint32_t __float_as_uint(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float __uint_as_float(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
using std::isfinite;
using std::max;
using std::min;
inline uint32_t min(uint32_t a, int b) { return std::min(a, (uint32_t)b); }
inline uint32_t atomicAdd(uint32_t *p, uint32_t v) { return __atomic_fetch_add(p, v, __ATOMIC_RELAXED); }
inline unsigned long long atomicAdd(unsigned long long *p, unsigned long long v) { return __atomic_fetch_add(p, v, __ATOMIC_RELAXED); }
inline uint32_t atomicOr(uint32_t *p, uint32_t v) { return __atomic_fetch_or(p, v, __ATOMIC_RELAXED); }
inline uint32_t atomicMax(uint32_t *p, uint32_t v) {
    uint32_t old = __atomic_load_n(p, __ATOMIC_RELAXED);
    while (old < v && !__atomic_compare_exchange_n(p, &old, v, false, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) {}
    return old;
}
inline uint32_t atomicMin(uint32_t *p, uint32_t v) {
    uint32_t old = __atomic_load_n(p, __ATOMIC_RELAXED);
    while (old > v && !__atomic_compare_exchange_n(p, &old, v, false, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) {}
    return old;
}
inline void __threadfence() { __atomic_thread_fence(__ATOMIC_SEQ_CST); }
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __HIP_MEMORY_SCOPE_WORKGROUP 0
#define __builtin_amdgcn_fence(order, scope) __atomic_thread_fence(__ATOMIC_SEQ_CST)
template <class T> inline T __hip_atomic_load(const T *p, int, int) { T v; __atomic_load(const_cast<T *>(p), &v, __ATOMIC_SEQ_CST); return v; }
template <class T> inline void __hip_atomic_store(T *p, T v, int, int) { __atomic_store(p, &v, __ATOMIC_SEQ_CST); }
inline uint32_t __hip_atomic_fetch_add(uint32_t *p, uint32_t v, int, int) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
