// Fused elementwise activation rule:
//   y = f(x);  y_jac[p] = f'(x) * jac[p];  y_lap = f'(x) * lap + f''(x) * sum_p jac[p]^2
// One pass over the Jacobian: every jac element is read once and written once, so the
// kernel moves 8 * (P + 2) * S bytes and is bound by HBM bandwidth.
//
// Work split: a workgroup is 4 wavefronts.  All four look at the same 64 * VEC
// consecutive elements; wavefront w streams the Jacobian rows p = w, w + 4, ... so that
// small S still puts enough loads in flight, and the four partial sums of squares meet
// in LDS.  The barrier before that reduction also makes in-place use safe: x is read by
// every wavefront before any of them writes y.
#include "activations.h"

namespace {

constexpr int PSPLIT = 4;

template <int ACT, int VEC>
__global__ __launch_bounds__(FOLX_WAVE * PSPLIT) void elementwise_kernel(
    const float* x, const float* jac, const float* lap, float* y,
    float* y_jac, float* y_lap, int64_t S, int32_t P, float prm) {
  __shared__ float red[PSPLIT][FOLX_WAVE * VEC];
  const int lane = threadIdx.x % FOLX_WAVE;
  const int w = threadIdx.x / FOLX_WAVE;
  const int64_t e0 = ((int64_t)blockIdx.x * FOLX_WAVE + lane) * VEC;
  const bool active = e0 < S;  // S % VEC == 0 is guaranteed by the launcher

  float yv[VEC], d1[VEC], d2[VEC], sq[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) { sq[v] = 0.0f; yv[v] = d1[v] = d2[v] = 0.0f; }

  if (active) {
    float xv[VEC];
    if constexpr (VEC == 4) {
      float4 t = *reinterpret_cast<const float4*>(x + e0);
      xv[0] = t.x; xv[1] = t.y; xv[2] = t.z; xv[3] = t.w;
    } else {
      xv[0] = x[e0];
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) act_eval<ACT>(xv[v], prm, yv[v], d1[v], d2[v]);

    constexpr int UNROLL = 4;
    int p = w;
    for (; p + (UNROLL - 1) * PSPLIT < P; p += UNROLL * PSPLIT) {
      float jv[UNROLL][VEC];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const float* src = jac + (int64_t)(p + u * PSPLIT) * S + e0;
        if constexpr (VEC == 4) {
          float4 t = folx_ld_stream4(src);
          jv[u][0] = t.x; jv[u][1] = t.y; jv[u][2] = t.z; jv[u][3] = t.w;
        } else {
          jv[u][0] = *src;
        }
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        float* dst = y_jac + (int64_t)(p + u * PSPLIT) * S + e0;
        float o[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) { o[v] = d1[v] * jv[u][v]; sq[v] += jv[u][v] * jv[u][v]; }
        if constexpr (VEC == 4) {
          folx_st_stream4(dst, make_float4(o[0], o[1], o[2], o[3]));
        } else {
          *dst = o[0];
        }
      }
    }
    for (; p < P; p += PSPLIT) {
      const float* src = jac + (int64_t)p * S + e0;
      float* dst = y_jac + (int64_t)p * S + e0;
      if constexpr (VEC == 4) {
        float4 t = folx_ld_stream4(src);
        sq[0] += t.x * t.x; sq[1] += t.y * t.y; sq[2] += t.z * t.z; sq[3] += t.w * t.w;
        folx_st_stream4(dst, make_float4(d1[0] * t.x, d1[1] * t.y, d1[2] * t.z, d1[3] * t.w));
      } else {
        float t = *src;
        sq[0] += t * t;
        *dst = d1[0] * t;
      }
    }
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) red[w][lane * VEC + v] = sq[v];
  __syncthreads();
  if (w == 0 && active) {
    float lv[VEC];
    if constexpr (VEC == 4) {
      float4 t = *reinterpret_cast<const float4*>(lap + e0);
      lv[0] = t.x; lv[1] = t.y; lv[2] = t.z; lv[3] = t.w;
    } else {
      lv[0] = lap[e0];
    }
    float ol[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      float s = red[0][lane * VEC + v];
#pragma unroll
      for (int ww = 1; ww < PSPLIT; ++ww) s += red[ww][lane * VEC + v];
      ol[v] = d1[v] * lv[v] + d2[v] * s;
    }
    if constexpr (VEC == 4) {
      *reinterpret_cast<float4*>(y + e0) = make_float4(yv[0], yv[1], yv[2], yv[3]);
      *reinterpret_cast<float4*>(y_lap + e0) = make_float4(ol[0], ol[1], ol[2], ol[3]);
    } else {
      y[e0] = yv[0];
      y_lap[e0] = ol[0];
    }
  }
}

template <int ACT>
int launch_act(hipStream_t st, const float* x, const float* jac, const float* lap, float* y,
               float* y_jac, float* y_lap, int64_t S, int32_t P, float prm) {
  const bool vec = (S % 4 == 0) && folx_aligned16(x) && folx_aligned16(jac) && folx_aligned16(lap) &&
                   folx_aligned16(y) && folx_aligned16(y_jac) && folx_aligned16(y_lap);
  if (vec) {
    int64_t blocks = (S / 4 + FOLX_WAVE - 1) / FOLX_WAVE;
    elementwise_kernel<ACT, 4><<<dim3((unsigned)blocks), dim3(FOLX_WAVE * PSPLIT), 0, st>>>(
        x, jac, lap, y, y_jac, y_lap, S, P, prm);
  } else {
    int64_t blocks = (S + FOLX_WAVE - 1) / FOLX_WAVE;
    elementwise_kernel<ACT, 1><<<dim3((unsigned)blocks), dim3(FOLX_WAVE * PSPLIT), 0, st>>>(
        x, jac, lap, y, y_jac, y_lap, S, P, prm);
  }
  return folx_launch_status();
}

}  // namespace

extern "C" int folx_hip_elementwise_fwdlap(void* stream, int32_t act, float param, const float* x,
                                           const float* jac, const float* lap, float* y,
                                           float* y_jac, float* y_lap, int64_t S, int32_t P) {
  if (S < 0 || P < 0 || act < 0 || act >= FOLX_ACT_COUNT) return FOLX_HIP_EINVAL;
  if (S == 0) return FOLX_HIP_OK;
  if (!x || !lap || !y || !y_lap || (P > 0 && (!jac || !y_jac))) return FOLX_HIP_EINVAL;
  if ((S + FOLX_WAVE - 1) / FOLX_WAVE > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  hipStream_t st = (hipStream_t)stream;
#define FOLX_CASE(A) \
  case A: return launch_act<A>(st, x, jac, lap, y, y_jac, y_lap, S, P, param);
  switch (act) {
    FOLX_CASE(FOLX_ACT_TANH) FOLX_CASE(FOLX_ACT_SILU) FOLX_CASE(FOLX_ACT_EXP) FOLX_CASE(FOLX_ACT_LOG)
    FOLX_CASE(FOLX_ACT_SQRT) FOLX_CASE(FOLX_ACT_RSQRT) FOLX_CASE(FOLX_ACT_SQUARE)
    FOLX_CASE(FOLX_ACT_LOGISTIC) FOLX_CASE(FOLX_ACT_SOFTPLUS) FOLX_CASE(FOLX_ACT_SIN)
    FOLX_CASE(FOLX_ACT_COS) FOLX_CASE(FOLX_ACT_ABS) FOLX_CASE(FOLX_ACT_LOG1P)
    FOLX_CASE(FOLX_ACT_RECIPROCAL) FOLX_CASE(FOLX_ACT_EXPM1) FOLX_CASE(FOLX_ACT_INTEGER_POW)
    FOLX_CASE(FOLX_ACT_SINH) FOLX_CASE(FOLX_ACT_COSH) FOLX_CASE(FOLX_ACT_TAN) FOLX_CASE(FOLX_ACT_ASIN)
    FOLX_CASE(FOLX_ACT_ACOS) FOLX_CASE(FOLX_ACT_ATAN) FOLX_CASE(FOLX_ACT_ASINH) FOLX_CASE(FOLX_ACT_ACOSH)
    FOLX_CASE(FOLX_ACT_ATANH) FOLX_CASE(FOLX_ACT_ERF) FOLX_CASE(FOLX_ACT_ERFC) FOLX_CASE(FOLX_ACT_ERF_INV)
    FOLX_CASE(FOLX_ACT_CBRT) FOLX_CASE(FOLX_ACT_POW) FOLX_CASE(FOLX_ACT_LGAMMA) FOLX_CASE(FOLX_ACT_DIGAMMA)
  }
#undef FOLX_CASE
  return FOLX_HIP_EINVAL;
}
