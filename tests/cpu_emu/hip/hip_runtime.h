// A small CPU stand-in for the parts of the HIP runtime and of the gfx950 device intrinsics that
// cascade_amd/csrc uses, so that the very same kernel sources can be compiled with g++ and run
// (under AddressSanitizer if wanted) on a machine without a GPU. TEST INFRASTRUCTURE ONLY: the
// product never loads a library built with this header.
//
// Execution model: a launch runs its workgroups one after another, in blockIdx order; the threads of
// a workgroup are real host threads, __syncthreads() is a barrier over them, and every wave-level
// operation (__ballot, __shfl*, wave barrier) is a barrier over the 64 threads of a wave followed by an
// exchange through a per-wave buffer. Kernels must therefore call wave operations from all 64 lanes
// (the kernels here do). "Device memory" is host memory.
#pragma once

#include <atomic>
#include <barrier>
#include <chrono>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <thread>
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

namespace hipemu {
struct Wave {
    std::barrier<> bar{64};
    uint64_t buf[64];
};
struct Block {
    std::unique_ptr<std::barrier<>> bar;
    std::vector<std::unique_ptr<Wave>> waves;
};
inline thread_local Wave* wave = nullptr;
inline thread_local Block* block = nullptr;
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

inline void hipemu::launch(dim3 grid, dim3 blk, size_t shmem, const std::function<void()>& body)
{
    const unsigned B = blk.x;
    dynamic_lds_storage().assign(shmem / 8 + 2, 0ull);
    if (B % 64 != 0)
        std::abort();
    // HIPEMU_REVERSE=1 runs the workgroups from the last blockIdx to the first: results must not depend on it
    static const bool reverse = std::getenv("HIPEMU_REVERSE") != nullptr;
    Block b;
    b.bar = std::make_unique<std::barrier<>>(B);
    for (unsigned w = 0; w < B / 64; ++w)
        b.waves.push_back(std::make_unique<Wave>());
    std::vector<std::thread> threads;
    for (unsigned t = 0; t < B; ++t) {
        threads.emplace_back([&, t] {
            hipemu::block = &b;
            hipemu::wave = b.waves[t / 64].get();
            hipemu::lane = t % 64;
            threadIdx = dim3(t);
            blockDim = blk;
            gridDim = grid;
            for (unsigned i = 0; i < grid.x; ++i) {
                const unsigned g = reverse ? grid.x - 1 - i : i;
                blockIdx = dim3(g);
                body();
                b.bar->arrive_and_wait(); // LDS ("static") is reused by the next workgroup
            }
        });
    }
    for (auto& th : threads)
        th.join();
}

#define hipLaunchKernelGGL(kernel, grid, blk, shmem, stream, ...) \
    hipemu::launch((grid), (blk), (shmem), [&] { kernel(__VA_ARGS__); })

// ---- synchronisation and wave operations ----
inline void __syncthreads() { hipemu::block->bar->arrive_and_wait(); }
inline unsigned __lane_id() { return hipemu::lane; }
inline void __builtin_amdgcn_wave_barrier() { hipemu::wave->bar.arrive_and_wait(); }
inline void __builtin_amdgcn_s_sleep(int) { std::this_thread::yield(); }

inline unsigned long long __ballot(int pred)
{
    hipemu::Wave* w = hipemu::wave;
    w->buf[hipemu::lane] = pred ? 1 : 0;
    w->bar.arrive_and_wait();
    unsigned long long m = 0;
    for (int l = 0; l < 64; ++l)
        m |= (unsigned long long)(w->buf[l] & 1) << l;
    w->bar.arrive_and_wait();
    return m;
}

template <typename T>
inline T __shfl(T var, unsigned src)
{
    hipemu::Wave* w = hipemu::wave;
    w->buf[hipemu::lane] = (uint64_t)var;
    w->bar.arrive_and_wait();
    const T r = (T)w->buf[src & 63u];
    w->bar.arrive_and_wait();
    return r;
}

template <typename T>
inline T __shfl_up(T var, unsigned delta)
{
    hipemu::Wave* w = hipemu::wave;
    w->buf[hipemu::lane] = (uint64_t)var;
    w->bar.arrive_and_wait();
    const T r = hipemu::lane >= delta ? (T)w->buf[hipemu::lane - delta] : var;
    w->bar.arrive_and_wait();
    return r;
}

template <typename T>
inline T __shfl_xor(T var, unsigned mask)
{
    hipemu::Wave* w = hipemu::wave;
    w->buf[hipemu::lane] = (uint64_t)var;
    w->bar.arrive_and_wait();
    const T r = (T)w->buf[(hipemu::lane ^ mask) & 63u];
    w->bar.arrive_and_wait();
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
