// Version and error strings of the C ABI.
#include "../../include/folx_hip.h"

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
