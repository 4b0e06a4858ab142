// Version and error strings of the C ABI.
#include <atomic>

#include "../../include/folx_hip.h"
#include "split_bf16.h"

extern "C" int folx_hip_version(void) { return 100; }

extern "C" const char* folx_hip_strerror(int code) {
  switch (code) {
    case FOLX_HIP_OK: return "ok";
    case FOLX_HIP_EINVAL: return "invalid argument (null pointer, negative size or inconsistent shape)";
    case FOLX_HIP_ENOTSUP: return "size not supported by the gfx950 kernels";
    case FOLX_HIP_ELAUNCH: return "kernel launch failed (hipGetLastError)";
    case FOLX_HIP_ESCRATCH: return "shape needs more scratch memory than the library's static 64 MiB array";
    default: return "unknown folx_hip error code";
  }
}

// Process-wide choice of the matrix instruction for the wide dense rules.
static std::atomic<int> g_gemm_mode{FOLX_HIP_GEMM_F32};

int folx_gemm_mode() { return g_gemm_mode.load(std::memory_order_relaxed); }

extern "C" int folx_hip_set_gemm_mode(int mode) {
  if (mode != FOLX_HIP_GEMM_F32 && mode != FOLX_HIP_GEMM_BF16X3) return FOLX_HIP_EINVAL;
  g_gemm_mode.store(mode, std::memory_order_relaxed);
  return FOLX_HIP_OK;
}

extern "C" int folx_hip_get_gemm_mode(void) { return folx_gemm_mode(); }
