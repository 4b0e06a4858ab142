// Shared helpers for the gfx950 forward-Laplacian kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/folx_hip.h"

#define FOLX_WAVE 64

static inline int folx_launch_status() {
  return hipGetLastError() == hipSuccess ? FOLX_HIP_OK : FOLX_HIP_ELAUNCH;
}

static inline bool folx_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#ifdef __HIPCC__
// Index of the wavefront inside its workgroup, in a scalar register: threadIdx.x / 64 is the same for the lanes of
// a wavefront, but the compiler cannot know that; with the scalar, loops over "this wavefront's rows" have scalar trip
// counts and row addresses take the scalar-base form instead of 64-bit vector arithmetic per access.
__device__ __forceinline__ int folx_wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x / FOLX_WAVE)); }
// Streaming accesses for data that is touched once per launch (Jacobian rows): non-temporal
// loads and stores, which a row-strided copy on this GPU runs 12 % faster with.
typedef float folx_vf4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 folx_ld_stream4(const float* p) {
  const folx_vf4 v = __builtin_nontemporal_load(reinterpret_cast<const folx_vf4*>(p));
  return make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void folx_st_stream4(float* p, float4 v) {
  folx_vf4 t;
  t[0] = v.x; t[1] = v.y; t[2] = v.z; t[3] = v.w;
  __builtin_nontemporal_store(t, reinterpret_cast<folx_vf4*>(p));
}
#endif

// 3-D broadcast index: linear i over (n0, n1, n2) -> offset with strides s[3].
struct Bcast3 {
  int64_t n1, n2;
  int64_t s0, s1, s2;
  __device__ __forceinline__ int64_t off(int64_t i) const {
    if ((((uint64_t)i | (uint64_t)n1 | (uint64_t)n2) >> 32) == 0) {
      // everything fits 32 bits (the usual case): a 64-bit division costs several times a 32-bit one
      const uint32_t j = (uint32_t)i, m1 = (uint32_t)n1, m2 = (uint32_t)n2;
      const uint32_t t = j / m2, i2 = j - t * m2;
      const uint32_t i0 = t / m1, i1 = t - i0 * m1;
      return i0 * s0 + i1 * s1 + i2 * s2;
    }
    int64_t i2 = i % n2;
    int64_t t = i / n2;
    int64_t i1 = t % n1;
    int64_t i0 = t / n1;
    return i0 * s0 + i1 * s1 + i2 * s2;
  }
};
