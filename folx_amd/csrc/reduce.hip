// Reductions over a middle axis: in [rows][outer][red][inner] -> out [rows][outer][inner].
// The sum rule is linear, so the same kernel serves x, the Jacobian rows and lap.  The
// reduced axis may be a window [lo, hi) of a longer axis (a slice that is summed right away is
// read where it lies): `span` is the full length of that axis in memory.
#include "common.h"

namespace {

// inner >= 2: one thread per output element, consecutive threads on consecutive `inner`
// positions so every step of the loop over `red` is a coalesced read.
template <bool MAX>
__global__ __launch_bounds__(256) void reduce_mid_kernel(const float* __restrict__ in,
                                                         float* __restrict__ out, int64_t total,
                                                         int64_t red, int64_t inner, int64_t span, int64_t lo,
                                                         float alpha) {
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= total) return;
  const int64_t ii = o % inner;
  const int64_t ro = o / inner;  // (row, outer) flattened
  const float* src = in + (ro * span + lo) * inner + ii;
  float acc = MAX ? -INFINITY : 0.0f;
  for (int64_t r = 0; r < red; ++r) {
    const float v = src[r * inner];
    acc = MAX ? fmaxf(acc, v) : acc + v;
  }
  out[o] = MAX ? acc : alpha * acc;
}

// inner a multiple of 4 (and aligned): one thread per four output elements, 128-bit streaming loads,
// four of them in flight per thread (the scalar form above keeps one 4-byte load per thread in
// flight and reaches 3 TB/s on the spin-wise means of a 16-electron layer; this one 5).
template <bool MAX>
__global__ __launch_bounds__(256) void reduce_mid_v4_kernel(const float* __restrict__ in,
                                                            float* __restrict__ out, int64_t total4,
                                                            int64_t red, int64_t inner, int64_t span, int64_t lo,
                                                            float alpha) {
  const int64_t o4 = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o4 >= total4) return;
  const int64_t inner4 = inner / 4;
  const int64_t ii = (o4 % inner4) * 4;
  const int64_t ro = o4 / inner4;  // (row, outer) flattened
  const float* src = in + (ro * span + lo) * inner + ii;
  const float init = MAX ? -INFINITY : 0.0f;
  float4 acc = make_float4(init, init, init, init);
  auto take = [&](const float4& v) {
    if (MAX) { acc.x = fmaxf(acc.x, v.x); acc.y = fmaxf(acc.y, v.y); acc.z = fmaxf(acc.z, v.z); acc.w = fmaxf(acc.w, v.w); }
    else { acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w; }
  };
  int64_t r = 0;
  for (; r + 4 <= red; r += 4) {  // in the order of the scalar kernel: r ascending
    const float4 v0 = folx_ld_stream4(src + (r + 0) * inner), v1 = folx_ld_stream4(src + (r + 1) * inner);
    const float4 v2 = folx_ld_stream4(src + (r + 2) * inner), v3 = folx_ld_stream4(src + (r + 3) * inner);
    take(v0); take(v1); take(v2); take(v3);
  }
  for (; r < red; ++r) take(folx_ld_stream4(src + r * inner));
  if (!MAX) { acc.x *= alpha; acc.y *= alpha; acc.z *= alpha; acc.w *= alpha; }
  *reinterpret_cast<float4*>(out + o4 * 4) = acc;
}

// inner == 1: one wavefront per output element, lanes stride over the reduced axis.
template <bool MAX>
__global__ __launch_bounds__(256) void reduce_last_kernel(const float* __restrict__ in,
                                                          float* __restrict__ out, int64_t total,
                                                          int64_t red, int64_t span, int64_t lo, float alpha) {
  const int lane = threadIdx.x % FOLX_WAVE;
  const int64_t o = (int64_t)blockIdx.x * (256 / FOLX_WAVE) + threadIdx.x / FOLX_WAVE;
  if (o >= total) return;
  const float* src = in + o * span + lo;
  float acc = MAX ? -INFINITY : 0.0f;
  for (int64_t r = lane; r < red; r += FOLX_WAVE) {
    const float v = src[r];
    acc = MAX ? fmaxf(acc, v) : acc + v;
  }
#pragma unroll
  for (int off = FOLX_WAVE / 2; off > 0; off >>= 1) {
    const float v = __shfl_xor(acc, off, FOLX_WAVE);
    acc = MAX ? fmaxf(acc, v) : acc + v;
  }
  if (lane == 0) out[o] = MAX ? acc : alpha * acc;
}

template <bool MAX>
int launch_reduce(hipStream_t st, const float* in, float* out, int64_t rows, int64_t outer,
                  int64_t red, int64_t inner, float alpha, int64_t span, int64_t lo) {
  if (rows < 0 || outer < 0 || red < 0 || inner < 0 || lo < 0 || lo + red > span) return FOLX_HIP_EINVAL;
  const int64_t total = rows * outer * inner;
  if (total == 0) return FOLX_HIP_OK;
  if (!in || !out) return FOLX_HIP_EINVAL;
  if (inner == 1 && red >= 16) {
    const int64_t blocks = (total + 3) / 4;
    if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
    reduce_last_kernel<MAX><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(in, out, total, red, span, lo, alpha);
  } else if (inner % 4 == 0 && folx_aligned16(in) && folx_aligned16(out)) {
    const int64_t blocks = (total / 4 + 255) / 256;
    if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
    reduce_mid_v4_kernel<MAX><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(in, out, total / 4, red, inner, span, lo,
                                                                          alpha);
  } else {
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
    reduce_mid_kernel<MAX><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(in, out, total, red, inner, span, lo, alpha);
  }
  return folx_launch_status();
}

}  // namespace

extern "C" int folx_hip_reduce_sum(void* stream, const float* in, float* out, int64_t rows,
                                   int64_t outer, int64_t red, int64_t inner, float alpha) {
  return launch_reduce<false>((hipStream_t)stream, in, out, rows, outer, red, inner, alpha, red, 0);
}

extern "C" int folx_hip_reduce_sum_window(void* stream, const float* in, float* out, int64_t rows,
                                          int64_t outer, int64_t span, int64_t lo, int64_t hi, int64_t inner,
                                          float alpha) {
  if (hi < lo) return FOLX_HIP_EINVAL;
  return launch_reduce<false>((hipStream_t)stream, in, out, rows, outer, hi - lo, inner, alpha, span, lo);
}

extern "C" int folx_hip_reduce_max(void* stream, const float* in, float* out, int64_t outer,
                                   int64_t red, int64_t inner) {
  return launch_reduce<true>((hipStream_t)stream, in, out, 1, outer, red, inner, 1.0f, red, 0);
}
