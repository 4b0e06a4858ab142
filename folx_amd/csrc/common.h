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

// 3-D broadcast index: linear i over (n0, n1, n2) -> offset with strides s[3].
struct Bcast3 {
  int64_t n1, n2;
  int64_t s0, s1, s2;
  __device__ __forceinline__ int64_t off(int64_t i) const {
    int64_t i2 = i % n2;
    int64_t t = i / n2;
    int64_t i1 = t % n1;
    int64_t i0 = t / n1;
    return i0 * s0 + i1 * s1 + i2 * s2;
  }
};
