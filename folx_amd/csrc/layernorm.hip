// Fused LayerNorm rule over the last axis:  y = g * (x - mean) * rsqrt(var + eps) + beta.
//
// With c = x - mean(x), r = rsqrt(mean(c^2) + eps) and, per Jacobian row u = jac[p],
//   a_p = mean(u),  b_p = mean(c u),  s_p = mean(u^2) - a_p^2
// the triplet of y is
//   y_jac[p] = g r (u - a_p - c r^2 b_p)
//   y_lap    = g r (lap - mean(lap) - c r^2 mean(c lap))                      (linear part)
//            + g ( -2 r^3 sum_p b_p (u_p - a_p) + c (3 r^5 sum_p b_p^2 - r^3 sum_p s_p) )
// which is what the chain mean / sub / square / mean / rsqrt / mul of elementwise and
// reduction rules evaluates to.  A workgroup of 4 wavefronts owns one row of F features and
// streams its Jacobian rows once (read once, written once: 8 (P + 2) F bytes per row, HBM
// bound): wavefront w takes the Jacobian rows p = w, w + 4, ..., four of them in flight at a
// time, so consecutive workgroups walk consecutive addresses of every Jacobian row.  The
// three per-row means are butterfly reductions inside the wavefront; the sums over p meet
// in LDS and wavefront 0 writes y and y_lap.
#include "common.h"

namespace {

__device__ __forceinline__ void wave_sum3(float& a, float& b, float& c) {
#pragma unroll
  for (int off = FOLX_WAVE / 2; off > 0; off >>= 1) {
    a += __shfl_xor(a, off, FOLX_WAVE);
    b += __shfl_xor(b, off, FOLX_WAVE);
    c += __shfl_xor(c, off, FOLX_WAVE);
  }
}
__device__ __forceinline__ float wave_sum1(float a) {
#pragma unroll
  for (int off = FOLX_WAVE / 2; off > 0; off >>= 1) a += __shfl_xor(a, off, FOLX_WAVE);
  return a;
}

constexpr int PSPLIT = 4;

// PER_WAVE: for a few Jacobian rows (sparse storage, P <= 8) a whole workgroup per row of features would
// mostly wait at its barrier: each WAVEFRONT owns a row of features then and walks all P Jacobian rows
// itself (four in flight), no LDS and no barrier.
template <int NV, bool PER_WAVE>
__global__ __launch_bounds__(FOLX_WAVE * PSPLIT) void layernorm_kernel(
    const float* __restrict__ x, const float* __restrict__ jac, const float* __restrict__ lap,
    const float* __restrict__ gamma, const float* __restrict__ beta, float* __restrict__ y,
    float* __restrict__ y_jac, float* __restrict__ y_lap, int64_t R, int32_t F, int32_t P, float eps) {
  __shared__ float4 redT[PSPLIT][NV * FOLX_WAVE];
  __shared__ float reds[PSPLIT][2];
  const int lane = threadIdx.x % FOLX_WAVE;
  const int w = threadIdx.x / FOLX_WAVE;
  const int64_t row = PER_WAVE ? (int64_t)blockIdx.x * PSPLIT + w : (int64_t)blockIdx.x;
  if (PER_WAVE && row >= R) return;
  constexpr int PS = PER_WAVE ? 1 : PSPLIT;  // distance between the Jacobian rows of a wavefront
  const int F4 = F / 4;
  const float invF = 1.0f / (float)F;
  const int64_t S = R * (int64_t)F;  // elements per Jacobian row
  const int64_t off = row * (int64_t)F;

  bool ok[NV];
  float4 c[NV], g[NV];
  float sx = 0.0f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int i4 = lane + FOLX_WAVE * v;
    ok[v] = i4 < F4;
    c[v] = make_float4(0.f, 0.f, 0.f, 0.f);
    g[v] = c[v];
    if (ok[v]) {
      c[v] = *reinterpret_cast<const float4*>(x + off + 4 * i4);
      g[v] = gamma ? *reinterpret_cast<const float4*>(gamma + 4 * i4) : make_float4(1.f, 1.f, 1.f, 1.f);
      sx += c[v].x + c[v].y + c[v].z + c[v].w;
    }
  }
  const float mu = wave_sum1(sx) * invF;
  float sv = 0.0f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    if (ok[v]) {
      c[v].x -= mu; c[v].y -= mu; c[v].z -= mu; c[v].w -= mu;
      sv += c[v].x * c[v].x + c[v].y * c[v].y + c[v].z * c[v].z + c[v].w * c[v].w;
    }
  }
  const float var = wave_sum1(sv) * invF;
  const float r = 1.0f / sqrtf(var + eps);
  const float r2 = r * r, r3 = r2 * r, r5 = r3 * r2;

  float4 T[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v) T[v] = make_float4(0.f, 0.f, 0.f, 0.f);
  float sb2 = 0.0f, ss = 0.0f;

  auto load_row = [&](int p, float4* u) {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      u[v] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (ok[v]) u[v] = folx_ld_stream4(jac + (int64_t)p * S + off + 4 * (lane + FOLX_WAVE * v));
    }
  };
  auto partial = [&](const float4* u, float& s1, float& s2, float& s3) {
    s1 = s2 = s3 = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      s1 += u[v].x + u[v].y + u[v].z + u[v].w;
      s2 += c[v].x * u[v].x + c[v].y * u[v].y + c[v].z * u[v].z + c[v].w * u[v].w;
      s3 += u[v].x * u[v].x + u[v].y * u[v].y + u[v].z * u[v].z + u[v].w * u[v].w;
    }
  };
  auto finish_row = [&](int p, const float4* u, float s1, float s2, float s3) {
    const float a = s1 * invF, b = s2 * invF;
    sb2 += b * b;
    ss += s3 * invF - a * a;
    const float cb = r2 * b;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      if (ok[v]) {
        const float dx = u[v].x - a, dy = u[v].y - a, dz = u[v].z - a, dw = u[v].w - a;
        T[v].x += b * dx; T[v].y += b * dy; T[v].z += b * dz; T[v].w += b * dw;
        float4 o;
        o.x = g[v].x * r * (dx - c[v].x * cb);
        o.y = g[v].y * r * (dy - c[v].y * cb);
        o.z = g[v].z * r * (dz - c[v].z * cb);
        o.w = g[v].w * r * (dw - c[v].w * cb);
        folx_st_stream4(y_jac + (int64_t)p * S + off + 4 * (lane + FOLX_WAVE * v), o);
      }
    }
  };

  int p = PER_WAVE ? 0 : w;
  for (; p + 3 * PS < P; p += 4 * PS) {  // four Jacobian rows in flight per wavefront
    float4 u0[NV], u1[NV], u2[NV], u3[NV];
    load_row(p, u0);
    load_row(p + PS, u1);
    load_row(p + 2 * PS, u2);
    load_row(p + 3 * PS, u3);
    float a1, a2, a3, b1, b2, b3, c1, c2, c3, e1, e2, e3;
    partial(u0, a1, a2, a3);
    partial(u1, b1, b2, b3);
    partial(u2, c1, c2, c3);
    partial(u3, e1, e2, e3);
    wave_sum3(a1, a2, a3);
    wave_sum3(b1, b2, b3);
    wave_sum3(c1, c2, c3);
    wave_sum3(e1, e2, e3);
    finish_row(p, u0, a1, a2, a3);
    finish_row(p + PS, u1, b1, b2, b3);
    finish_row(p + 2 * PS, u2, c1, c2, c3);
    finish_row(p + 3 * PS, u3, e1, e2, e3);
  }
  for (; p < P; p += PS) {
    float4 u0[NV];
    load_row(p, u0);
    float a1, a2, a3;
    partial(u0, a1, a2, a3);
    wave_sum3(a1, a2, a3);
    finish_row(p, u0, a1, a2, a3);
  }

  // the sums over p of the four wavefronts meet in LDS (this barrier also orders every
  // wavefront's read of x before the write of y, which makes in-place use safe)
  if constexpr (!PER_WAVE) {
#pragma unroll
    for (int v = 0; v < NV; ++v) redT[w][v * FOLX_WAVE + lane] = T[v];
    if (lane == 0) { reds[w][0] = sb2; reds[w][1] = ss; }
    __syncthreads();
    if (w != 0) return;
    sb2 = reds[0][0]; ss = reds[0][1];
#pragma unroll
    for (int ww = 1; ww < PSPLIT; ++ww) {
      sb2 += reds[ww][0]; ss += reds[ww][1];
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const float4 t = redT[ww][v * FOLX_WAVE + lane];
        T[v].x += t.x; T[v].y += t.y; T[v].z += t.z; T[v].w += t.w;
      }
    }
  }

  // value and Laplacian
  float4 l[NV];
  float sl = 0.0f, scl = 0.0f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    l[v] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (ok[v]) {
      l[v] = *reinterpret_cast<const float4*>(lap + off + 4 * (lane + FOLX_WAVE * v));
      sl += l[v].x + l[v].y + l[v].z + l[v].w;
      scl += c[v].x * l[v].x + c[v].y * l[v].y + c[v].z * l[v].z + c[v].w * l[v].w;
    }
  }
  float dummy = 0.0f;
  wave_sum3(sl, scl, dummy);
  const float ml = sl * invF, mcl = scl * invF;
  const float k2 = 3.0f * r5 * sb2 - r3 * ss;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    if (ok[v]) {
      const int i4 = lane + FOLX_WAVE * v;
      const float4 bt = beta ? *reinterpret_cast<const float4*>(beta + 4 * i4) : make_float4(0.f, 0.f, 0.f, 0.f);
      float4 yo, lo;
      yo.x = g[v].x * r * c[v].x + bt.x; yo.y = g[v].y * r * c[v].y + bt.y;
      yo.z = g[v].z * r * c[v].z + bt.z; yo.w = g[v].w * r * c[v].w + bt.w;
      lo.x = g[v].x * (r * (l[v].x - ml - c[v].x * r2 * mcl) - 2.0f * r3 * T[v].x + c[v].x * k2);
      lo.y = g[v].y * (r * (l[v].y - ml - c[v].y * r2 * mcl) - 2.0f * r3 * T[v].y + c[v].y * k2);
      lo.z = g[v].z * (r * (l[v].z - ml - c[v].z * r2 * mcl) - 2.0f * r3 * T[v].z + c[v].z * k2);
      lo.w = g[v].w * (r * (l[v].w - ml - c[v].w * r2 * mcl) - 2.0f * r3 * T[v].w + c[v].w * k2);
      *reinterpret_cast<float4*>(y + off + 4 * i4) = yo;
      *reinterpret_cast<float4*>(y_lap + off + 4 * i4) = lo;
    }
  }
}

}  // namespace

extern "C" int folx_hip_layernorm_fwdlap(void* stream, const float* x, const float* jac,
                                         const float* lap, const float* gamma, const float* beta,
                                         float* y, float* y_jac, float* y_lap, int64_t R, int32_t F,
                                         int32_t P, float eps) {
  if (R < 0 || F <= 0 || P < 0) return FOLX_HIP_EINVAL;
  if (R == 0) return FOLX_HIP_OK;
  if (!x || !lap || !y || !y_lap || (P > 0 && (!jac || !y_jac))) return FOLX_HIP_EINVAL;
  if (F % 4 != 0 || F > 1024) return FOLX_HIP_ENOTSUP;
  const void* ptrs[] = {x, jac, lap, gamma, beta, y, y_jac, y_lap};
  for (const void* p : ptrs)
    if (p && !folx_aligned16(p)) return FOLX_HIP_ENOTSUP;
  const bool per_wave = P <= 8;
  const int64_t blocks = per_wave ? (R + PSPLIT - 1) / PSPLIT : R;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)blocks), block(FOLX_WAVE * PSPLIT);
  const int nv = (F / 4 + FOLX_WAVE - 1) / FOLX_WAVE;
#define FOLX_LN(NV)                                                                                               \
  if (per_wave) layernorm_kernel<NV, true><<<grid, block, 0, st>>>(x, jac, lap, gamma, beta, y, y_jac, y_lap, R, F, P, eps); \
  else layernorm_kernel<NV, false><<<grid, block, 0, st>>>(x, jac, lap, gamma, beta, y, y_jac, y_lap, R, F, P, eps);
  switch (nv) {
    case 1: FOLX_LN(1) break;
    case 2: FOLX_LN(2) break;
    case 3: FOLX_LN(3) break;
    default: FOLX_LN(4) break;
  }
#undef FOLX_LN
  return folx_launch_status();
}
