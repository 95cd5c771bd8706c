/*
 * Test infrastructure, not part of the product: a stand-in for <hip/hip_runtime.h>
 * that lets the product's .hip / .cpp sources be compiled for the HOST, so that the
 * kernels can be executed, bounds-checked and compared with the CPU checker without a
 * GPU (tests/test_kernels_on_cpu.py).
 *
 * Execution model: a launch runs its workgroups one after the other; the work-items of
 * a workgroup are fibers (ucontext) that switch at __syncthreads() and at wavefront
 * collectives (shuffles, MFMA), 64 consecutive work-items forming a wavefront.  Memory
 * from hipMalloc / hipHostMalloc and the dynamic LDS of a launch sit against guard
 * pages, so an out-of-range access raises SIGSEGV at the faulting statement.  The three
 * MFMA instructions the kernels use are computed from their documented lane layouts.
 *
 * The stream is asynchronous as on the GPU: kernel launches and asynchronous copies
 * between hipMalloc / hipHostMalloc blocks are queued (kernel arguments by value) and
 * carried out in order as late as the API allows - at the next wait (stream, device,
 * event), blocking copy, copy to pageable memory or free.  Host code that rewrites or
 * recycles a pinned buffer before the work that reads it has run, or reads results
 * without waiting, therefore misbehaves here as it may on the GPU.  HIPCPU_SYNC=1 runs
 * every operation at once instead.
 */
#ifndef HIPCPU_RUNTIME_H
#define HIPCPU_RUNTIME_H

#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <functional>
#include <tuple>
#include <type_traits>
#include <utility>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (x)
#define __shared__ static

typedef void *hipStream_t;
typedef void *hipEvent_t;
typedef int hipError_t;
enum { hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorOutOfMemory = 2 };
enum hipMemcpyKind { hipMemcpyHostToHost, hipMemcpyHostToDevice, hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice };
enum { hipStreamNonBlocking = 1, hipHostMallocDefault = 0 };
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct uint2 { unsigned x, y; };
struct uint4 { unsigned x, y, z, w; };
struct float2 { float x, y; };
struct float4 { float x, y, z, w; };
static inline uint2 make_uint2(unsigned x, unsigned y) { return uint2{ x, y }; }
static inline uint4 make_uint4(unsigned x, unsigned y, unsigned z, unsigned w) { return uint4{ x, y, z, w }; }
static inline float2 make_float2(float x, float y) { return float2{ x, y }; }
static inline float4 make_float4(float x, float y, float z, float w) { return float4{ x, y, z, w }; }

/* ---- runtime (hipcpu_runtime.cpp) ----------------------------------------------- */
struct HipCpuItem { /* one work-item */
    dim3 tid;
    int linear, wave, lane;
};
extern "C" {
extern HipCpuItem *hipcpu_cur;     /* the running work-item */
extern dim3 hipcpu_block_idx, hipcpu_block_dim, hipcpu_grid_dim;
void *hipcpu_dynamic_lds(void);
void hipcpu_syncthreads(void);
void hipcpu_wave_barrier(void);
/* every live lane of the wavefront deposits n 32-bit words; returns the table
   [64][16] of the wavefront once all have, valid until the next collective */
const uint32_t *hipcpu_wave_exchange(const uint32_t *words, int n);
void hipcpu_launch(dim3 grid, dim3 block, size_t shmem, void (*entry)(void *), void *closure);
hipError_t hipMalloc(void **p, size_t n);
hipError_t hipFree(void *p);
hipError_t hipHostMalloc(void **p, size_t n, unsigned flags);
hipError_t hipHostFree(void *p);
}

#define threadIdx (hipcpu_cur->tid)
#define blockIdx hipcpu_block_idx
#define blockDim hipcpu_block_dim
#define gridDim hipcpu_grid_dim
#define warpSize 64

static inline hipError_t hipGetLastError(void) { return hipSuccess; }
static inline const char *hipGetErrorString(hipError_t) { return "hipcpu"; }
static inline hipError_t hipSetDevice(int) { return hipSuccess; }
static inline hipError_t hipGetDevice(int *d) { *d = 0; return hipSuccess; }
static inline hipError_t hipGetSymbolAddress(void **p, const void *symbol) { *p = const_cast<void *>(symbol); return hipSuccess; }
static inline hipError_t hipGetDeviceCount(int *n) { *n = 1; return hipSuccess; }
static inline hipError_t hipStreamCreate(hipStream_t *s) { *s = (hipStream_t)0x1; return hipSuccess; }
static inline hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned) { *s = (hipStream_t)0x1; return hipSuccess; }
static inline hipError_t hipStreamDestroy(hipStream_t) { return hipSuccess; }
extern "C" hipError_t hipcpu_memcpy_async(void *d, const void *s, size_t n);
extern "C" void hipcpu_flush_copies(void);
static inline hipError_t hipStreamSynchronize(hipStream_t) { hipcpu_flush_copies(); return hipSuccess; }
static inline hipError_t hipDeviceSynchronize(void) { hipcpu_flush_copies(); return hipSuccess; }
static inline hipError_t hipMemcpyAsync(void *d, const void *s, size_t n, hipMemcpyKind, hipStream_t)
{
    return hipcpu_memcpy_async(d, s, n);
}
static inline hipError_t hipMemcpy(void *d, const void *s, size_t n, hipMemcpyKind)
{
    hipcpu_flush_copies();
    memmove(d, s, n);
    return hipSuccess;
}
static inline hipError_t hipEventCreate(hipEvent_t *e) { *e = nullptr; return hipSuccess; }
static inline hipError_t hipEventDestroy(hipEvent_t) { return hipSuccess; }
static inline hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
static inline hipError_t hipEventSynchronize(hipEvent_t) { hipcpu_flush_copies(); return hipSuccess; }
static inline hipError_t hipEventElapsedTime(float *ms, hipEvent_t, hipEvent_t) { *ms = 1e-3f; return hipSuccess; }
static inline hipError_t hipFuncSetAttribute(const void *, hipFuncAttribute, int) { return hipSuccess; }

/* ---- launches ---------------------------------------------------------------------- */
template <typename F, typename Tuple, size_t... I>
static void hipcpu_apply(F f, Tuple &t, std::index_sequence<I...>) { f(std::get<I>(t)...); }

void hipcpu_enqueue(std::function<void()> op);

template <typename F, typename... A>
static void hipcpu_launch_impl(F kernel, dim3 grid, dim3 block, size_t shmem, A... args)
{
    struct Closure { F k; std::tuple<A...> a; };
    Closure c{ kernel, std::tuple<A...>(args...) };
    hipcpu_enqueue([c, grid, block, shmem]() mutable {
        hipcpu_launch(grid, block, shmem, [](void *p) {
            Closure *q = (Closure *)p;
            hipcpu_apply(q->k, q->a, std::index_sequence_for<A...>());
        }, &c);
    });
}
#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
    hipcpu_launch_impl(kernel, dim3(grid), dim3(block), (size_t)(shmem), ##__VA_ARGS__)
#define hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, ev0, ev1, flags, ...) \
    hipcpu_launch_impl(kernel, dim3(grid), dim3(block), (size_t)(shmem), ##__VA_ARGS__)

/* ---- device-side library ------------------------------------------------------------- */
#define __syncthreads() hipcpu_syncthreads()
#define __builtin_amdgcn_wave_barrier() hipcpu_wave_barrier()
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_sched_group_barrier(mask, size, id) ((void)0)
#define __builtin_amdgcn_fence(...) ((void)0)
#define __builtin_amdgcn_s_setprio(x) ((void)0)
static inline long long clock64(void) { return 0; }
static inline long long wall_clock64(void) { return 0; }

static inline unsigned __float_as_uint(float f) { unsigned u; memcpy(&u, &f, 4); return u; }
static inline float __uint_as_float(unsigned u) { float f; memcpy(&f, &u, 4); return f; }
static inline int __float_as_int(float f) { int u; memcpy(&u, &f, 4); return u; }
static inline float __int_as_float(int u) { float f; memcpy(&f, &u, 4); return f; }
#define __expf(x) expf(x) /* glibc declares __expf itself */
static inline float rsqrtf(float x) { return 1.0f / sqrtf(x); }
static inline float __fdividef(float a, float b) { return a / b; }

template <typename T, typename U>
static inline typename std::common_type<T, U>::type min(T a, U b) { return b < a ? b : a; }
template <typename T, typename U>
static inline typename std::common_type<T, U>::type max(T a, U b) { return a < b ? b : a; }

template <typename T>
static inline T hipcpu_shfl_from(T v, int src)
{
    static_assert(sizeof(T) == 4 || sizeof(T) == 8, "shuffles move 4- or 8-byte values");
    uint32_t w[2] = { 0, 0 };
    memcpy(w, &v, sizeof(T));
    const uint32_t *tab = hipcpu_wave_exchange(w, 2);
    T r;
    /* a lane outside the wavefront (or one that has exited) returns the caller's own value */
    if (src < 0 || src >= 64) src = hipcpu_cur->lane;
    memcpy(&r, tab + src * 16, sizeof(T));
    hipcpu_wave_barrier();
    return r;
}
template <typename T> static inline T __shfl(T v, int src, int width = 64)
{
    int lane = hipcpu_cur->lane, base = lane / width * width;
    return hipcpu_shfl_from(v, base + (src % width));
}
template <typename T> static inline T __shfl_xor(T v, int mask, int width = 64)
{
    int lane = hipcpu_cur->lane, base = lane / width * width, s = (lane ^ mask);
    return hipcpu_shfl_from(v, s >= base && s < base + width ? s : lane);
}
template <typename T> static inline T __shfl_up(T v, unsigned d, int width = 64)
{
    int lane = hipcpu_cur->lane, base = lane / width * width, s = lane - (int)d;
    return hipcpu_shfl_from(v, s >= base ? s : lane);
}
template <typename T> static inline T __shfl_down(T v, unsigned d, int width = 64)
{
    int lane = hipcpu_cur->lane, base = lane / width * width, s = lane + (int)d;
    return hipcpu_shfl_from(v, s < base + width ? s : lane);
}

/* ---- MFMA (lane layouts of the CDNA3/4 ISA guide) ------------------------------------ */
typedef float hipcpu_f16v __attribute__((ext_vector_type(16)));
typedef float hipcpu_f4v __attribute__((ext_vector_type(4)));

/* v_mfma_f32_32x32x2_f32: lane l holds A[i = l%32][k = l/32] and B[k = l/32][j = l%32];
   D value r of lane l is D[i = (r/4)*8 + (l/32)*4 + r%4][j = l%32] */
static inline hipcpu_f16v hipcpu_mfma_32x32x2f32(float a, float b, hipcpu_f16v c, int, int, int)
{
    uint32_t w[2] = { __float_as_uint(a), __float_as_uint(b) };
    const uint32_t *tab = hipcpu_wave_exchange(w, 2);
    const int l = hipcpu_cur->lane, j = l & 31;
    for (int r = 0; r < 16; r++) {
        const int i = (r / 4) * 8 + (l / 32) * 4 + r % 4;
        float acc = c[r];
        for (int k = 0; k < 2; k++)
            acc = fmaf(__uint_as_float(tab[(k * 32 + i) * 16]), __uint_as_float(tab[(k * 32 + j) * 16 + 1]), acc);
        c[r] = acc;
    }
    hipcpu_wave_barrier();
    return c;
}
/* v_mfma_f32_16x16x4_f32: A[i = l%16][k = l/16], B[k = l/16][j = l%16];
   D value r of lane l is D[i = (l/16)*4 + r][j = l%16] */
static inline hipcpu_f4v hipcpu_mfma_16x16x4f32(float a, float b, hipcpu_f4v c, int, int, int)
{
    uint32_t w[2] = { __float_as_uint(a), __float_as_uint(b) };
    const uint32_t *tab = hipcpu_wave_exchange(w, 2);
    const int l = hipcpu_cur->lane, j = l & 15;
    for (int r = 0; r < 4; r++) {
        const int i = (l / 16) * 4 + r;
        float acc = c[r];
        for (int k = 0; k < 4; k++)
            acc = fmaf(__uint_as_float(tab[(k * 16 + i) * 16]), __uint_as_float(tab[(k * 16 + j) * 16 + 1]), acc);
        c[r] = acc;
    }
    hipcpu_wave_barrier();
    return c;
}
/* v_mfma_f32_32x32x16_bf16: lane l holds 8 consecutive k = (l/32)*8 .. +7 of row / column
   l%32; D as for 32x32x2 */
static inline float hipcpu_bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
template <typename V>
static inline hipcpu_f16v hipcpu_mfma_32x32x16_bf16(V a, V b, hipcpu_f16v c, int, int, int)
{
    static_assert(sizeof(V) == 16, "8 bf16 values");
    uint32_t w[8];
    memcpy(w, &a, 16);
    memcpy(w + 4, &b, 16);
    const uint32_t *tab = hipcpu_wave_exchange(w, 8);
    const int l = hipcpu_cur->lane, j = l & 31;
    for (int r = 0; r < 16; r++) {
        const int i = (r / 4) * 8 + (l / 32) * 4 + r % 4;
        float acc = c[r];
        for (int kg = 0; kg < 2; kg++) {
            const uint16_t *pa = (const uint16_t *)(tab + (kg * 32 + i) * 16);
            const uint16_t *pb = (const uint16_t *)(tab + (kg * 32 + j) * 16 + 4);
            for (int e = 0; e < 8; e++)
                acc = fmaf(hipcpu_bf16_to_f32(pa[e]), hipcpu_bf16_to_f32(pb[e]), acc);
        }
        c[r] = acc;
    }
    hipcpu_wave_barrier();
    return c;
}
/* v_mfma_f32_16x16x32_bf16: lane l holds 8 consecutive k = (l/16)*8 .. +7 of row / column
   l%16; D as for 16x16x4 */
template <typename V>
static inline hipcpu_f4v hipcpu_mfma_16x16x32_bf16(V a, V b, hipcpu_f4v c, int, int, int)
{
    static_assert(sizeof(V) == 16, "8 bf16 values");
    uint32_t w[8];
    memcpy(w, &a, 16);
    memcpy(w + 4, &b, 16);
    const uint32_t *tab = hipcpu_wave_exchange(w, 8);
    const int l = hipcpu_cur->lane, j = l & 15;
    for (int r = 0; r < 4; r++) {
        const int i = (l / 16) * 4 + r;
        float acc = c[r];
        for (int kg = 0; kg < 4; kg++) {
            const uint16_t *pa = (const uint16_t *)(tab + (kg * 16 + i) * 16);
            const uint16_t *pb = (const uint16_t *)(tab + (kg * 16 + j) * 16 + 4);
            for (int e = 0; e < 8; e++)
                acc = fmaf(hipcpu_bf16_to_f32(pa[e]), hipcpu_bf16_to_f32(pb[e]), acc);
        }
        c[r] = acc;
    }
    hipcpu_wave_barrier();
    return c;
}
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16 hipcpu_mfma_16x16x32_bf16
#define __builtin_amdgcn_mfma_f32_32x32x2f32 hipcpu_mfma_32x32x2f32
#define __builtin_amdgcn_mfma_f32_16x16x4f32 hipcpu_mfma_16x16x4f32
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16 hipcpu_mfma_32x32x16_bf16

#endif /* HIPCPU_RUNTIME_H */
