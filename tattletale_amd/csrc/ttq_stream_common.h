// Primitives shared by the decode GEMVs whose workgroups stream weights HBM -> LDS with global_load_lds requests and
// synchronize by hand (ttq_gemv_q6k_stream.hip, ttq_gemv_q8_stream.hip): waits on the wavefront's own request
// counter, a barrier that leaves outstanding requests alone, and LDS accesses the compiler does not see.
#pragma once

#include "ttq_gemv_mfma_common.h"

namespace ttq {

typedef const __attribute__((address_space(1))) void* sm_gptr_t;
typedef __attribute__((address_space(3))) void* sm_lptr_t;
typedef uint32_t sm_u32x4 __attribute__((ext_vector_type(4)));

// s_waitcnt vmcnt(N) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14).  Requests complete in order, so "all but
// the youngest N have landed" is the only wait there is.
template <int N>
__device__ __forceinline__ void sm_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
  asm volatile("" ::: "memory");
}
// A barrier that leaves the outstanding requests alone (a __syncthreads() would wait for every one of them).
__device__ __forceinline__ void sm_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ uint32_t sm_lds(const void* p) { return (uint32_t)(size_t)(sm_lptr_t)(p); }
// LDS accesses the compiler must not see: it cannot tell them from the asynchronous writes of the requests in
// flight and would wait for every one of those first.
__device__ __forceinline__ sm_u32x4 sm_read16(uint32_t a) {
  sm_u32x4 v;
  asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(a) : "memory");
  return v;
}
__device__ __forceinline__ void sm_write_b32(uint32_t a, uint32_t v) {
  asm volatile("ds_write_b32 %0, %1" ::"v"(a), "v"(v) : "memory");
}
__device__ __forceinline__ void sm_write_b64(uint32_t a, uint32_t lo, uint32_t hi) {
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  const u32x2 v = {lo, hi};
  asm volatile("ds_write_b64 %0, %1" ::"v"(a), "v"(v) : "memory");
}
__device__ __forceinline__ void sm_write_f32(uint32_t a, float v) {
  asm volatile("ds_write_b32 %0, %1" ::"v"(a), "v"(v) : "memory");
}

}  // namespace ttq
