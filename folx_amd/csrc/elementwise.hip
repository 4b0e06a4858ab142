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
#include "common.h"

namespace {

template <int ACT>
__device__ __forceinline__ void act_eval(float x, float prm, float& y, float& d1, float& d2) {
  if constexpr (ACT == FOLX_ACT_TANH) {
    float t = tanhf(x);
    y = t; d1 = 1.0f - t * t; d2 = -2.0f * t * d1;
  } else if constexpr (ACT == FOLX_ACT_SILU) {
    float s = 1.0f / (1.0f + expf(-x));
    y = x * s; d1 = s * (1.0f + x * (1.0f - s)); d2 = s * (1.0f - s) * (2.0f + x * (1.0f - 2.0f * s));
  } else if constexpr (ACT == FOLX_ACT_EXP) {
    float e = expf(x);
    y = e; d1 = e; d2 = e;
  } else if constexpr (ACT == FOLX_ACT_LOG) {
    float r = 1.0f / x;
    y = logf(x); d1 = r; d2 = -r * r;
  } else if constexpr (ACT == FOLX_ACT_SQRT) {
    float r = sqrtf(x);
    y = r; d1 = 0.5f / r; d2 = -0.25f / (r * x);
  } else if constexpr (ACT == FOLX_ACT_RSQRT) {
    float r = 1.0f / sqrtf(x);
    y = r; d1 = -0.5f * r / x; d2 = 0.75f * r / (x * x);
  } else if constexpr (ACT == FOLX_ACT_SQUARE) {
    y = x * x; d1 = 2.0f * x; d2 = 2.0f;
  } else if constexpr (ACT == FOLX_ACT_LOGISTIC) {
    float s = 1.0f / (1.0f + expf(-x));
    y = s; d1 = s * (1.0f - s); d2 = d1 * (1.0f - 2.0f * s);
  } else if constexpr (ACT == FOLX_ACT_SOFTPLUS) {
    float s = 1.0f / (1.0f + expf(-x));
    y = fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x))); d1 = s; d2 = s * (1.0f - s);
  } else if constexpr (ACT == FOLX_ACT_SIN) {
    float s, c; sincosf(x, &s, &c);
    y = s; d1 = c; d2 = -s;
  } else if constexpr (ACT == FOLX_ACT_COS) {
    float s, c; sincosf(x, &s, &c);
    y = c; d1 = -s; d2 = -c;
  } else if constexpr (ACT == FOLX_ACT_ABS) {
    y = fabsf(x); d1 = (x > 0.0f) ? 1.0f : ((x < 0.0f) ? -1.0f : 0.0f); d2 = 0.0f;
  } else if constexpr (ACT == FOLX_ACT_LOG1P) {
    float r = 1.0f / (1.0f + x);
    y = log1pf(x); d1 = r; d2 = -r * r;
  } else if constexpr (ACT == FOLX_ACT_RECIPROCAL) {
    float r = 1.0f / x;
    y = r; d1 = -r * r; d2 = 2.0f * r * r * r;
  } else if constexpr (ACT == FOLX_ACT_EXPM1) {
    float e = expf(x);
    y = expm1f(x); d1 = e; d2 = e;
  } else if constexpr (ACT == FOLX_ACT_SINH) {
    float sh = sinhf(x), ch = coshf(x);
    y = sh; d1 = ch; d2 = sh;
  } else if constexpr (ACT == FOLX_ACT_COSH) {
    float sh = sinhf(x), ch = coshf(x);
    y = ch; d1 = sh; d2 = ch;
  } else if constexpr (ACT == FOLX_ACT_TAN) {
    float t = tanf(x);
    y = t; d1 = 1.0f + t * t; d2 = 2.0f * t * d1;
  } else if constexpr (ACT == FOLX_ACT_ASIN) {
    float r = 1.0f / sqrtf(1.0f - x * x);
    y = asinf(x); d1 = r; d2 = x * r * r * r;
  } else if constexpr (ACT == FOLX_ACT_ACOS) {
    float r = 1.0f / sqrtf(1.0f - x * x);
    y = acosf(x); d1 = -r; d2 = -x * r * r * r;
  } else if constexpr (ACT == FOLX_ACT_ATAN) {
    float q = 1.0f / (1.0f + x * x);
    y = atanf(x); d1 = q; d2 = -2.0f * x * q * q;
  } else if constexpr (ACT == FOLX_ACT_ASINH) {
    float r = 1.0f / sqrtf(1.0f + x * x);
    y = asinhf(x); d1 = r; d2 = -x * r * r * r;
  } else if constexpr (ACT == FOLX_ACT_ACOSH) {
    float r = 1.0f / sqrtf(x * x - 1.0f);
    y = acoshf(x); d1 = r; d2 = -x * r * r * r;
  } else if constexpr (ACT == FOLX_ACT_ATANH) {
    float q = 1.0f / (1.0f - x * x);
    y = atanhf(x); d1 = q; d2 = 2.0f * x * q * q;
  } else if constexpr (ACT == FOLX_ACT_ERF) {
    float g = 1.1283791670955126f * expf(-x * x);  // 2 / sqrt(pi)
    y = erff(x); d1 = g; d2 = -2.0f * x * g;
  } else if constexpr (ACT == FOLX_ACT_ERFC) {
    float g = 1.1283791670955126f * expf(-x * x);
    y = erfcf(x); d1 = -g; d2 = 2.0f * x * g;
  } else if constexpr (ACT == FOLX_ACT_ERF_INV) {
    float v = erfinvf(x);
    float g = 0.8862269254527580f * expf(v * v);  // sqrt(pi) / 2
    y = v; d1 = g; d2 = 2.0f * v * g * g;
  } else if constexpr (ACT == FOLX_ACT_CBRT) {
    float c = cbrtf(x);
    y = c; d1 = c / (3.0f * x); d2 = -2.0f * c / (9.0f * x * x);
  } else if constexpr (ACT == FOLX_ACT_POW) {
    float pm2 = powf(x, prm - 2.0f);
    y = pm2 * x * x; d1 = prm * pm2 * x; d2 = prm * (prm - 1.0f) * pm2;
  } else {  // FOLX_ACT_INTEGER_POW
    int n = (int)prm;
    // x^(n-2) by repeated multiplication on |n-2|, then one or two more factors
    int m = n - 2;
    int am = m < 0 ? -m : m;
    float b = x, acc = 1.0f;
    while (am) { if (am & 1) acc *= b; b *= b; am >>= 1; }
    float xm2 = m < 0 ? 1.0f / acc : acc;
    float xm1 = xm2 * x;
    y = xm1 * x; d1 = (float)n * xm1; d2 = (float)n * (float)(n - 1) * xm2;
  }
}

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
          float4 t = *reinterpret_cast<const float4*>(src);
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
          *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
        } else {
          *dst = o[0];
        }
      }
    }
    for (; p < P; p += PSPLIT) {
      const float* src = jac + (int64_t)p * S + e0;
      float* dst = y_jac + (int64_t)p * S + e0;
      if constexpr (VEC == 4) {
        float4 t = *reinterpret_cast<const float4*>(src);
        sq[0] += t.x * t.x; sq[1] += t.y * t.y; sq[2] += t.z * t.z; sq[3] += t.w * t.w;
        *reinterpret_cast<float4*>(dst) = make_float4(d1[0] * t.x, d1[1] * t.y, d1[2] * t.z, d1[3] * t.w);
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
    FOLX_CASE(FOLX_ACT_CBRT) FOLX_CASE(FOLX_ACT_POW)
  }
#undef FOLX_CASE
  return FOLX_HIP_EINVAL;
}
