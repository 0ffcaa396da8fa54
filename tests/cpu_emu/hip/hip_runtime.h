// A small CPU stand-in for the parts of the HIP runtime and of the gfx950 device intrinsics that
// cascade_amd/csrc uses, so that the very same kernel sources can be compiled with g++ and run
// (under AddressSanitizer if wanted) on a machine without a GPU. TEST INFRASTRUCTURE ONLY: the
// product never loads a library built with this header.
//
// Execution model: a launch runs its workgroups one after another, in blockIdx order; the threads of
// a workgroup are fibers of the calling host thread (each with a stack of its own, switched by hand:
// no scheduler, no system call, the same order every run), __syncthreads() is a barrier over them, and
// every wave-level operation (__ballot, __shfl*, wave barrier) is a barrier over the 64 fibers of a wave
// followed by an exchange through a per-wave buffer. A fiber runs until it reaches a barrier (or
// s_sleep) that it cannot pass yet and then hands over to the next one. Kernels must therefore call
// wave operations from all 64 lanes (the kernels here do), and a wait on another thread of the same
// workgroup must go through a barrier or s_sleep (theirs do). One launch at a time per process (the
// LDS arrays are static). "Device memory" is host memory.
#pragma once

#include <atomic>
#include <chrono>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __restrict__
#define __shared__ static
#define __align__(n) __attribute__((aligned(n)))

struct alignas(16) uint4 {
    unsigned x, y, z, w;
};
inline uint4 make_uint4(unsigned x, unsigned y, unsigned z, unsigned w) { return uint4{x, y, z, w}; }

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

#if !defined(__x86_64__)
#error "the fiber switch of the CPU stand-in is written for x86-64"
#endif

// hipemu_switch(save, load): parks the running fiber (its callee-saved registers on its stack, the stack pointer in
// *save) and resumes the one whose stack pointer is `load`.
extern "C" void hipemu_switch(void** save, void* load);
asm(".text\n"
    ".globl hipemu_switch\n"
    ".type hipemu_switch,@function\n"
    "hipemu_switch:\n"
    "    pushq %rbp\n"
    "    pushq %rbx\n"
    "    pushq %r12\n"
    "    pushq %r13\n"
    "    pushq %r14\n"
    "    pushq %r15\n"
    "    movq %rsp, (%rdi)\n"
    "    movq %rsi, %rsp\n"
    "    popq %r15\n"
    "    popq %r14\n"
    "    popq %r13\n"
    "    popq %r12\n"
    "    popq %rbx\n"
    "    popq %rbp\n"
    "    ret\n"
    ".size hipemu_switch,.-hipemu_switch\n");

namespace hipemu {
struct Wave {
    unsigned arrived = 0, phase = 0;
    uint64_t buf[64];
};
struct Fiber {
    void* sp = nullptr;
    unsigned t = 0;
    bool done = false;
};
struct Run {
    std::vector<Fiber> fibers;
    std::vector<Wave> waves;
    unsigned arrived = 0, phase = 0; // the workgroup's barrier
    unsigned current = 0, live = 0;
    void* main_sp = nullptr;
    const std::function<void()>* body = nullptr;
};
inline thread_local Run* run = nullptr;
inline thread_local Wave* wave = nullptr;
inline thread_local unsigned lane = 0;

inline void launch(dim3 grid, dim3 blk, size_t shmem, const std::function<void()>& body);
// dynamic LDS of the running launch (workgroups run one after the other, so one buffer serves them all)
inline std::vector<unsigned long long>& dynamic_lds_storage()
{
    static std::vector<unsigned long long> v;
    return v;
}
inline void* dynamic_lds() { return dynamic_lds_storage().data(); }
} // namespace hipemu
#define HIPEMU 1

inline thread_local dim3 threadIdx, blockIdx, blockDim, gridDim;

namespace hipemu {
constexpr size_t FIBER_STACK = 256 * 1024;
// stacks are kept from launch to launch
inline std::vector<std::unique_ptr<char[]>>& fiber_stacks()
{
    static thread_local std::vector<std::unique_ptr<char[]>> v;
    return v;
}

inline void enter(Fiber& f)
{
    run->current = f.t;
    threadIdx = dim3(f.t);
    lane = f.t % 64;
    wave = &run->waves[f.t / 64];
}

// HIPEMU_LANES_REVERSE=1 hands over from a fiber to the one before it instead of the one after it (and starts with the
// last): what one thread writes and another reads between two barriers without an order of their own shows up under one
// of the two directions.
inline bool lanes_reverse()
{
    static const bool reverse = std::getenv("HIPEMU_LANES_REVERSE") != nullptr;
    return reverse;
}
inline unsigned next_fiber(const Run& r, unsigned n)
{
    do
        n = lanes_reverse() ? (n == 0 ? (unsigned)r.fibers.size() - 1 : n - 1) : (n + 1 == r.fibers.size() ? 0 : n + 1);
    while (r.fibers[n].done);
    return n;
}

// hands over to the next fiber that has not finished; returns when this one is resumed
inline void yield()
{
    Run& r = *run;
    Fiber& me = r.fibers[r.current];
    const unsigned n = next_fiber(r, me.t);
    if (n == me.t)
        return; // alone: whatever it waits for will not come from a switch
    enter(r.fibers[n]);
    hipemu_switch(&me.sp, r.fibers[n].sp);
    enter(me);
}

inline void barrier(unsigned& arrived, unsigned& phase, unsigned count)
{
    const unsigned mine = phase;
    if (++arrived == count) {
        arrived = 0;
        phase = mine + 1; // the last one to arrive goes on; the others find the new phase when they are resumed
        return;
    }
    while (phase == mine)
        yield();
}

inline thread_local dim3 launch_grid;
inline void fiber_main()
{
    Run& r = *run;
    Fiber& me = r.fibers[r.current];
    // HIPEMU_REVERSE=1 runs the workgroups from the last blockIdx to the first: results must not depend on it
    static const bool reverse = std::getenv("HIPEMU_REVERSE") != nullptr;
    const unsigned blocks = launch_grid.x;
    for (unsigned i = 0; i < blocks; ++i) {
        blockIdx = dim3(reverse ? blocks - 1 - i : i);
        (*r.body)();
        barrier(r.arrived, r.phase, (unsigned)r.fibers.size()); // LDS ("static") is reused by the next workgroup
    }
    me.done = true;
    void* unused;
    if (--r.live == 0) {
        hipemu_switch(&unused, r.main_sp);
    } else {
        const unsigned n = next_fiber(r, me.t);
        enter(r.fibers[n]);
        hipemu_switch(&unused, r.fibers[n].sp);
    }
    std::abort(); // a finished fiber is never resumed
}
} // namespace hipemu

inline void hipemu::launch(dim3 grid, dim3 blk, size_t shmem, const std::function<void()>& body)
{
    const unsigned B = blk.x;
    dynamic_lds_storage().assign(shmem / 8 + 2, 0ull);
    if (B % 64 != 0 || run != nullptr)
        std::abort(); // whole waves only; no launch from inside a kernel
    if (grid.x == 0)
        return;
    Run r;
    r.fibers.resize(B);
    r.waves.resize(B / 64);
    r.live = B;
    r.body = &body;
    auto& stacks = fiber_stacks();
    while (stacks.size() < B)
        stacks.emplace_back(new char[FIBER_STACK]);
    for (unsigned t = 0; t < B; ++t) {
        // a fresh fiber's stack: the six registers hipemu_switch pops, then fiber_main as its return address; the
        // stack pointer is 8 below a 16-byte boundary when fiber_main starts, as after a call
        uintptr_t top = (reinterpret_cast<uintptr_t>(stacks[t].get()) + FIBER_STACK) & ~(uintptr_t)15;
        void** sp = reinterpret_cast<void**>(top);
        *--sp = nullptr; // where fiber_main would return to: it never does
        *--sp = reinterpret_cast<void*>(&fiber_main);
        for (int k = 0; k < 6; ++k)
            *--sp = nullptr;
        r.fibers[t].sp = sp;
        r.fibers[t].t = t;
    }
    blockDim = blk;
    gridDim = grid;
    launch_grid = grid;
    const dim3 saved_thread = threadIdx, saved_block = blockIdx;
    run = &r;
    Fiber& first = r.fibers[lanes_reverse() ? B - 1 : 0];
    enter(first);
    hipemu_switch(&r.main_sp, first.sp);
    run = nullptr;
    threadIdx = saved_thread;
    blockIdx = saved_block;
}

#define hipLaunchKernelGGL(kernel, grid, blk, shmem, stream, ...) \
    hipemu::launch((grid), (blk), (shmem), [&] { kernel(__VA_ARGS__); })

// ---- synchronisation and wave operations ----
inline void __syncthreads() { hipemu::barrier(hipemu::run->arrived, hipemu::run->phase, (unsigned)hipemu::run->fibers.size()); }
inline unsigned __lane_id() { return hipemu::lane; }
namespace hipemu {
inline void wave_sync(Wave* w) { barrier(w->arrived, w->phase, 64u); }
} // namespace hipemu
inline void __builtin_amdgcn_wave_barrier() { hipemu::wave_sync(hipemu::wave); }
inline void __builtin_amdgcn_s_sleep(int) { hipemu::yield(); }

inline unsigned long long __ballot(int pred)
{
    hipemu::Wave* w = hipemu::wave;
    w->buf[hipemu::lane] = pred ? 1 : 0;
    hipemu::wave_sync(w);
    unsigned long long m = 0;
    for (int l = 0; l < 64; ++l)
        m |= (unsigned long long)(w->buf[l] & 1) << l;
    hipemu::wave_sync(w);
    return m;
}

template <typename T>
inline T __shfl(T var, unsigned src)
{
    hipemu::Wave* w = hipemu::wave;
    w->buf[hipemu::lane] = (uint64_t)var;
    hipemu::wave_sync(w);
    const T r = (T)w->buf[src & 63u];
    hipemu::wave_sync(w);
    return r;
}

template <typename T>
inline T __shfl_up(T var, unsigned delta)
{
    hipemu::Wave* w = hipemu::wave;
    w->buf[hipemu::lane] = (uint64_t)var;
    hipemu::wave_sync(w);
    const T r = hipemu::lane >= delta ? (T)w->buf[hipemu::lane - delta] : var;
    hipemu::wave_sync(w);
    return r;
}

template <typename T>
inline T __shfl_xor(T var, unsigned mask)
{
    hipemu::Wave* w = hipemu::wave;
    w->buf[hipemu::lane] = (uint64_t)var;
    hipemu::wave_sync(w);
    const T r = (T)w->buf[(hipemu::lane ^ mask) & 63u];
    hipemu::wave_sync(w);
    return r;
}

inline int __popc(unsigned v) { return __builtin_popcount(v); }
inline int __popcll(unsigned long long v) { return __builtin_popcountll(v); }

inline unsigned __builtin_amdgcn_ubfe(unsigned src, unsigned off, unsigned width)
{
    off &= 31u;
    width &= 31u;
    if (width == 0)
        return 0;
    return (src >> off) & (width >= 32 ? 0xFFFFFFFFu : ((1u << width) - 1u));
}

inline int __builtin_amdgcn_sbfe(unsigned src, unsigned off, unsigned width)
{
    const unsigned v = __builtin_amdgcn_ubfe(src, off, width);
    const unsigned sign = 1u << (width - 1);
    return (int)((v ^ sign) - sign);
}

// three-input bit operation: bit i of the result is bit ((a_i << 2) | (b_i << 1) | c_i) of the table
inline unsigned __builtin_amdgcn_bitop3_b32(unsigned a, unsigned b, unsigned c, unsigned table)
{
    unsigned r = 0;
    for (int i = 0; i < 32; ++i) {
        const unsigned sel = (((a >> i) & 1u) << 2) | (((b >> i) & 1u) << 1) | ((c >> i) & 1u);
        r |= ((table >> sel) & 1u) << i;
    }
    return r;
}

inline unsigned __builtin_amdgcn_mbcnt_lo(unsigned mask, unsigned add)
{
    const unsigned l = hipemu::lane;
    const unsigned m = l >= 32 ? mask : (mask & ((1u << l) - 1u));
    return add + (unsigned)__builtin_popcount(m);
}

inline unsigned __builtin_amdgcn_mbcnt_hi(unsigned mask, unsigned add)
{
    const unsigned l = hipemu::lane;
    const unsigned m = l <= 32 ? 0u : (mask & ((1u << (l - 32)) - 1u));
    return add + (unsigned)__builtin_popcount(m);
}

// ---- atomics ----
#define __HIP_MEMORY_SCOPE_AGENT 0
template <typename T>
inline T __hip_atomic_load(const T* p, int, int) { return __atomic_load_n(p, __ATOMIC_SEQ_CST); }
template <typename T>
inline void __hip_atomic_store(T* p, T v, int, int) { __atomic_store_n(p, v, __ATOMIC_SEQ_CST); }
inline unsigned atomicAdd(unsigned* p, unsigned v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
inline unsigned atomicAdd(volatile unsigned* p, unsigned v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
inline unsigned long long atomicAdd(unsigned long long* p, unsigned long long v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
inline unsigned atomicExch(unsigned* p, unsigned v) { return __atomic_exchange_n(p, v, __ATOMIC_SEQ_CST); }
inline unsigned atomicOr(unsigned* p, unsigned v) { return __atomic_fetch_or(p, v, __ATOMIC_SEQ_CST); }
inline unsigned long long atomicCAS(unsigned long long* p, unsigned long long expected, unsigned long long desired)
{
    __atomic_compare_exchange_n(p, &expected, desired, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST);
    return expected; // the value found, as the device function returns it
}
inline unsigned long long __umul64hi(unsigned long long a, unsigned long long b) { return (unsigned long long)(((unsigned __int128)a * b) >> 64); }

// ---- host runtime ----
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
constexpr hipError_t hipErrorOutOfMemory = 2;
typedef void* hipStream_t;
struct hipEmuEvent {
    std::chrono::steady_clock::time_point t;
};
typedef hipEmuEvent* hipEvent_t;
enum hipMemcpyKind { hipMemcpyHostToDevice, hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice };
constexpr unsigned hipHostMallocDefault = 0;

inline const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "success" : "emulated failure"; }
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
// a __device__ array is an ordinary array here, so its name already is its address
#define HIP_SYMBOL(x) (x)
template <typename T>
inline hipError_t hipGetSymbolAddress(void** p, T& symbol) { *p = &symbol; return hipSuccess; }
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 63 };
// one "CU", unless a test has the device claim more (HIPEMU_CU_COUNT): workgroups still run one at a time, which makes it
// the extreme case of a device shared with other launches
inline hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int)
{
    const char* claimed = std::getenv("HIPEMU_CU_COUNT");
    *v = claimed ? std::atoi(claimed) : 1;
    return hipSuccess;
}
inline hipError_t hipMalloc(void** p, size_t bytes)
{
    *p = std::malloc(bytes ? bytes : 1);
    if (!*p)
        return hipErrorOutOfMemory;
    std::memset(*p, 0xA5, bytes); // device memory starts as garbage
    return hipSuccess;
}
inline hipError_t hipFree(void* p) { std::free(p); return hipSuccess; }
inline hipError_t hipHostMalloc(void** p, size_t bytes, unsigned) { return hipMalloc(p, bytes); }
inline hipError_t hipHostFree(void* p) { std::free(p); return hipSuccess; }
inline hipError_t hipMemset(void* p, int v, size_t bytes) { std::memset(p, v, bytes); return hipSuccess; }
inline hipError_t hipMemsetAsync(void* p, int v, size_t bytes, hipStream_t) { return hipMemset(p, v, bytes); }
inline hipError_t hipMemcpy(void* d, const void* s, size_t bytes, hipMemcpyKind) { std::memmove(d, s, bytes); return hipSuccess; }
inline hipError_t hipMemcpyAsync(void* d, const void* s, size_t bytes, hipMemcpyKind k, hipStream_t) { return hipMemcpy(d, s, bytes, k); }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
constexpr unsigned hipStreamNonBlocking = 1;
inline hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned) { *s = nullptr; return hipSuccess; }
inline hipError_t hipStreamDestroy(hipStream_t) { return hipSuccess; }
inline hipError_t hipSetDevice(int) { return hipSuccess; }
inline hipError_t hipDeviceSynchronize() { return hipSuccess; }
inline hipError_t hipEventCreate(hipEvent_t* e) { *e = new hipEmuEvent(); return hipSuccess; }
inline hipError_t hipEventDestroy(hipEvent_t e) { delete e; return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t e, hipStream_t) { e->t = std::chrono::steady_clock::now(); return hipSuccess; }
inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t a, hipEvent_t b)
{
    *ms = std::chrono::duration<float, std::milli>(b->t - a->t).count();
    return hipSuccess;
}
