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

// Exponential envelope, a fused chain of broadcast, scale, exp, scale and sum:
//   y[r][o] = sum_I pi[I][o] exp(-sigma[I][o] d[r][I])
// for a triplet d with few columns I (distances of one electron to the nuclei) and constant
// sigma, pi.  The function is a sum of scalar functions of the single d[r][I], so with
// t = pi exp(-sigma d):
//   y_jac[p] = sum_I (-sigma t) d_jac[p][I],
//   y_lap    = sum_I (-sigma t) d_lap[I] + sum_I sigma^2 t sum_p d_jac[p][I]^2.
// A thread owns four consecutive o of one row r; a wavefront therefore reads the same few d
// values (broadcast loads) and writes 1 KB of every output row.  The kernel reads almost
// nothing and is bound by writing (P + 2) R O floats.
namespace {

constexpr int ENV_MAX_I = 8;

__global__ __launch_bounds__(256) void exp_envelope_kernel(const float* __restrict__ d, const float* __restrict__ dj,
                                                           const float* __restrict__ dl,
                                                           const float* __restrict__ sigma,
                                                           const float* __restrict__ pi, float* __restrict__ y,
                                                           float* __restrict__ yj, float* __restrict__ yl, int64_t R,
                                                           int32_t nI, int32_t O, int32_t P) {
  const int O4 = O / 4;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= R * O4) return;
  const int64_t r = idx / O4;
  const int o = (int)(idx - r * O4) * 4;
  float4 g[ENV_MAX_I];  // -sigma t per column I
  float4 val = make_float4(0.f, 0.f, 0.f, 0.f), lap = val;
#pragma unroll
  for (int I = 0; I < ENV_MAX_I; ++I) {
    g[I] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (I < nI) {
      const float dv = d[r * nI + I], lv = dl[r * nI + I];
      float ss = 0.0f;
      for (int p = 0; p < P; ++p) { const float j = dj[((int64_t)p * R + r) * nI + I]; ss += j * j; }
      const float4 s4 = *reinterpret_cast<const float4*>(sigma + (int64_t)I * O + o);
      const float4 p4 = *reinterpret_cast<const float4*>(pi + (int64_t)I * O + o);
      const float sv[4] = {s4.x, s4.y, s4.z, s4.w}, pv[4] = {p4.x, p4.y, p4.z, p4.w};
      float t[4], gg[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) { t[x] = pv[x] * expf(-sv[x] * dv); gg[x] = -sv[x] * t[x]; }
      g[I] = make_float4(gg[0], gg[1], gg[2], gg[3]);
      val.x += t[0]; val.y += t[1]; val.z += t[2]; val.w += t[3];
      lap.x += gg[0] * lv + sv[0] * sv[0] * t[0] * ss; lap.y += gg[1] * lv + sv[1] * sv[1] * t[1] * ss;
      lap.z += gg[2] * lv + sv[2] * sv[2] * t[2] * ss; lap.w += gg[3] * lv + sv[3] * sv[3] * t[3] * ss;
    }
  }
  *reinterpret_cast<float4*>(y + r * O + o) = val;
  *reinterpret_cast<float4*>(yl + r * O + o) = lap;
  for (int p = 0; p < P; ++p) {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int I = 0; I < ENV_MAX_I; ++I)
      if (I < nI) {
        const float j = dj[((int64_t)p * R + r) * nI + I];
        acc.x += g[I].x * j; acc.y += g[I].y * j; acc.z += g[I].z * j; acc.w += g[I].w * j;
      }
    folx_st_stream4(yj + ((int64_t)p * R + r) * O + o, acc);
  }
}

}  // namespace

extern "C" int folx_hip_exp_envelope_fwdlap(void* stream, const float* d, const float* d_jac, const float* d_lap,
                                            const float* sigma, const float* pi, float* y, float* y_jac,
                                            float* y_lap, int64_t R, int32_t n_cols, int32_t O, int32_t P) {
  if (R < 0 || n_cols <= 0 || O <= 0 || P < 0) return FOLX_HIP_EINVAL;
  if (R == 0) return FOLX_HIP_OK;
  if (!d || !d_lap || !sigma || !pi || !y || !y_lap || (P > 0 && (!d_jac || !y_jac))) return FOLX_HIP_EINVAL;
  if (n_cols > ENV_MAX_I || O % 4 != 0) return FOLX_HIP_ENOTSUP;
  const void* ptrs[] = {sigma, pi, y, y_jac, y_lap};
  for (const void* p : ptrs)
    if (p && !folx_aligned16(p)) return FOLX_HIP_ENOTSUP;
  const int64_t blocks = (R * (O / 4) + 255) / 256;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  exp_envelope_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(d, d_jac, d_lap, sigma, pi, y,
                                                                                      y_jac, y_lap, R, n_cols, O, P);
  return folx_launch_status();
}
