// Scalar functions of the elementwise rule: value, first and second derivative.
#pragma once
#include "common.h"

namespace {

// digamma, trigamma and tetragamma (polygamma of order 0, 1, 2) in one pass: the argument is
// moved to x >= 6 with the recurrences psi_m(x) = psi_m(x + 1) - (-1)^m m! / x^(m+1) and the
// asymptotic series are summed there; x < 0.5 goes through the reflection formulas
//   psi(1-x) - psi(x) = pi cot(pi x),  psi1(1-x) + psi1(x) = pi^2 / sin^2(pi x),
//   psi2(1-x) - psi2(x) = 2 pi^3 cos(pi x) / sin^3(pi x).
__device__ __forceinline__ void polygamma012(float x, float& p0, float& p1, float& p2) {
  const bool reflect = x < 0.5f;
  const float xr = x;
  if (reflect) x = 1.0f - x;
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f;
  while (x < 6.0f) {
    const float r = 1.0f / x;
    s0 -= r;
    s1 += r * r;
    s2 -= 2.0f * r * r * r;
    x += 1.0f;
  }
  const float r = 1.0f / x, r2 = r * r;
  p0 = s0 + logf(x) - 0.5f * r - r2 * (1.0f / 12.0f - r2 * (1.0f / 120.0f - r2 * (1.0f / 252.0f - r2 * (1.0f / 240.0f))));
  p1 = s1 + r + 0.5f * r2 + r * r2 * (1.0f / 6.0f - r2 * (1.0f / 30.0f - r2 * (1.0f / 42.0f - r2 * (1.0f / 30.0f))));
  p2 = s2 - r2 - r * r2 - r2 * r2 * (0.5f - r2 * (1.0f / 6.0f - r2 * (1.0f / 6.0f - r2 * (3.0f / 10.0f))));
  if (reflect) {
    const float pi = 3.14159265358979f;
    float sn, cs;
    sincospif(xr, &sn, &cs);
    const float ct = cs / sn, cc = 1.0f / (sn * sn);
    p0 = p0 - pi * ct;
    p1 = pi * pi * cc - p1;
    p2 = p2 - 2.0f * pi * pi * pi * cc * ct;
  }
}

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
  } else if constexpr (ACT == FOLX_ACT_LGAMMA) {
    float p0, p1, p2;
    polygamma012(x, p0, p1, p2);
    y = lgammaf(x); d1 = p0; d2 = p1;
  } else if constexpr (ACT == FOLX_ACT_DIGAMMA) {
    float p0, p1, p2;
    polygamma012(x, p0, p1, p2);
    y = p0; d1 = p1; d2 = p2;
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

// The functions the fused dense + activation kernels take, chosen at run time.
inline bool act_fused(int act) {
  switch (act) {
    case FOLX_ACT_TANH: case FOLX_ACT_SILU: case FOLX_ACT_LOGISTIC: case FOLX_ACT_SOFTPLUS:
    case FOLX_ACT_EXP: case FOLX_ACT_SIN: case FOLX_ACT_COS: case FOLX_ACT_SQUARE:
      return true;
  }
  return false;
}

__device__ __forceinline__ void act_eval_fused(int act, float x, float prm, float& y, float& d1, float& d2) {
  switch (act) {
    case FOLX_ACT_TANH: act_eval<FOLX_ACT_TANH>(x, prm, y, d1, d2); break;
    case FOLX_ACT_SILU: act_eval<FOLX_ACT_SILU>(x, prm, y, d1, d2); break;
    case FOLX_ACT_LOGISTIC: act_eval<FOLX_ACT_LOGISTIC>(x, prm, y, d1, d2); break;
    case FOLX_ACT_SOFTPLUS: act_eval<FOLX_ACT_SOFTPLUS>(x, prm, y, d1, d2); break;
    case FOLX_ACT_EXP: act_eval<FOLX_ACT_EXP>(x, prm, y, d1, d2); break;
    case FOLX_ACT_SIN: act_eval<FOLX_ACT_SIN>(x, prm, y, d1, d2); break;
    case FOLX_ACT_COS: act_eval<FOLX_ACT_COS>(x, prm, y, d1, d2); break;
    default: act_eval<FOLX_ACT_SQUARE>(x, prm, y, d1, d2); break;
  }
}

}  // namespace
