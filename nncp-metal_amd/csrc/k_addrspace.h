// Pointers that carry the global address space, for device code whose pointers come out of
// a by-value struct, a select between two pointers or a table in device memory.  There the
// compiler cannot tell that the memory is global and emits FLAT loads and stores.  A FLAT
// access counts against the LDS counter as well as the memory counter: every wait for an LDS
// read (`s_waitcnt lgkmcnt(0)`) then also waits for the global loads in flight, which
// serialises a pipeline that means to overlap the two.  (Device pass only; the qualifier
// means nothing to a host compiler.)
#ifndef K_ADDRSPACE_H
#define K_ADDRSPACE_H

#if defined(__HIP_DEVICE_COMPILE__)
#define NCHIP_GLOBAL __attribute__((address_space(1)))
#else
#define NCHIP_GLOBAL
#endif

template <typename T>
__device__ __forceinline__ const T NCHIP_GLOBAL *as_global(const T *p) { return (const T NCHIP_GLOBAL *)p; }
template <typename T>
__device__ __forceinline__ T NCHIP_GLOBAL *as_global(T *p) { return (T NCHIP_GLOBAL *)p; }

#endif
