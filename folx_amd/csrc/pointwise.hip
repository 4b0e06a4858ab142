// Broadcasting elementwise rules on a shared Jacobian row frame: the binary rule
// (mul / div / add / sub / min / max of two triplets) and the affine map against constants.
// Both are single streaming passes bound by HBM bandwidth.
#include "common.h"

namespace {

constexpr int PSPLIT = 4;

// Binary rule.  A workgroup is 4 wavefronts over the same 64 output elements; wavefront
// w handles Jacobian rows p = w, w + 4, ...; the sums over p meet in LDS.
template <int OP>
__global__ __launch_bounds__(FOLX_WAVE * PSPLIT) void binary_kernel(
    const float* __restrict__ a, const float* __restrict__ aj, const float* __restrict__ al,
    const float* __restrict__ b, const float* __restrict__ bj, const float* __restrict__ bl,
    float* __restrict__ y, float* __restrict__ yj, float* __restrict__ yl, int64_t S, Bcast3 ia,
    Bcast3 ib, int64_t a_S, int64_t b_S, int32_t P) {
  __shared__ float red[2][PSPLIT][FOLX_WAVE];
  const int lane = threadIdx.x % FOLX_WAVE;
  const int w = threadIdx.x / FOLX_WAVE;
  const int64_t i = (int64_t)blockIdx.x * FOLX_WAVE + lane;
  const bool active = i < S;
  float sab = 0.0f, sbb = 0.0f;
  float av = 0.f, bv = 1.f, ca = 0.f, cb = 0.f;
  int64_t oa = 0, ob = 0;
  if (active) {
    oa = ia.off(i);
    ob = ib.off(i);
    av = a[oa];
    bv = b[ob];
    // y_jac = ca * a_jac + cb * b_jac
    if constexpr (OP == FOLX_BIN_MUL) { ca = bv; cb = av; }
    else if constexpr (OP == FOLX_BIN_DIV) { ca = 1.0f / bv; cb = -av * ca * ca; }
    else if constexpr (OP == FOLX_BIN_ADD) { ca = 1.0f; cb = 1.0f; }
    else if constexpr (OP == FOLX_BIN_SUB) { ca = 1.0f; cb = -1.0f; }
    else if constexpr (OP == FOLX_BIN_MIN) { ca = av < bv ? 1.0f : (av == bv ? 0.5f : 0.0f); cb = 1.0f - ca; }
    else { ca = av > bv ? 1.0f : (av == bv ? 0.5f : 0.0f); cb = 1.0f - ca; }
    for (int p = w; p < P; p += PSPLIT) {
      // Jacobian rows are touched once per launch: streaming (non-temporal) accesses
      const float ja = __builtin_nontemporal_load(&aj[(int64_t)p * a_S + oa]);
      const float jb = __builtin_nontemporal_load(&bj[(int64_t)p * b_S + ob]);
      __builtin_nontemporal_store(ca * ja + cb * jb, &yj[(int64_t)p * S + i]);
      if constexpr (OP == FOLX_BIN_MUL || OP == FOLX_BIN_DIV) sab += ja * jb;
      if constexpr (OP == FOLX_BIN_DIV) sbb += jb * jb;
    }
  }
  if constexpr (OP == FOLX_BIN_MUL || OP == FOLX_BIN_DIV) {
    red[0][w][lane] = sab;
    red[1][w][lane] = sbb;
    __syncthreads();
  }
  if (w == 0 && active) {
    float l = ca * al[oa] + cb * bl[ob];
    if constexpr (OP == FOLX_BIN_MUL) {
      float s = red[0][0][lane] + red[0][1][lane] + red[0][2][lane] + red[0][3][lane];
      y[i] = av * bv;
      l += 2.0f * s;
    } else if constexpr (OP == FOLX_BIN_DIV) {
      float s = red[0][0][lane] + red[0][1][lane] + red[0][2][lane] + red[0][3][lane];
      float t = red[1][0][lane] + red[1][1][lane] + red[1][2][lane] + red[1][3][lane];
      const float rb = 1.0f / bv;
      y[i] = av * rb;
      // H_lr = -2 / b^2 (counted once for the pair), H_rr = 2 a / b^3
      l += -2.0f * rb * rb * s + 2.0f * av * rb * rb * rb * t;
    } else if constexpr (OP == FOLX_BIN_ADD) {
      y[i] = av + bv;
    } else if constexpr (OP == FOLX_BIN_SUB) {
      y[i] = av - bv;
    } else if constexpr (OP == FOLX_BIN_MIN) {
      y[i] = fminf(av, bv);
    } else {
      y[i] = fmaxf(av, bv);
    }
    yl[i] = l;
  }
}

// Product of a triplet with a dense Jacobian (P rows) and one of the same shape whose Jacobian
// is sparse (k rows, slot s of element i standing for dense row idx[s][i % S_w]; no row named
// twice per element):
//   y = a b,  y_jac[p] = b a_jac[p] + a sum_{s: idx[s] = p} b_jac[s],
//   y_lap = b a_lap + a b_lap + 2 sum_s a_jac[idx[s]] b_jac[s].
// Same work split as binary_kernel; each lane keeps its k sparse rows and their indices in
// registers, so the dense rows of the sparse operand are never built.
// VEC = 4: a lane owns four consecutive elements (128-bit streaming accesses; S_w % 4 == 0, 16-byte aligned
// operands), VEC = 1: one element.
template <int KMAX, int VEC>
__global__ __launch_bounds__(FOLX_WAVE * PSPLIT) void mul_sparse_kernel(
    const float* __restrict__ a, const float* __restrict__ aj, const float* __restrict__ al,
    const float* __restrict__ b, const float* __restrict__ bj, const float* __restrict__ bl,
    const int32_t* __restrict__ idx, float* __restrict__ y, float* __restrict__ yj, float* __restrict__ yl,
    int64_t S, int64_t S_w, int32_t P, int32_t k) {
  __shared__ float red[PSPLIT][VEC][FOLX_WAVE];
  const int lane = threadIdx.x % FOLX_WAVE;
  const int w = threadIdx.x / FOLX_WAVE;
  const int64_t i = ((int64_t)blockIdx.x * FOLX_WAVE + lane) * VEC;
  const bool active = i < S;
  float sab[VEC], av[VEC], bv[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) sab[v] = av[v] = bv[v] = 0.0f;
  if (active) {
    const int64_t pos = (uint64_t)(i | S_w) >> 32 ? i % S_w : (int64_t)((uint32_t)i % (uint32_t)S_w);
    int32_t ix[KMAX][VEC];
    float bs[KMAX][VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) { av[v] = a[i + v]; bv[v] = b[i + v]; }
#pragma unroll
    for (int s = 0; s < KMAX; ++s)
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        ix[s][v] = s < k ? idx[(int64_t)s * S_w + pos + v] : -1;
        bs[s][v] = ix[s][v] >= 0 ? bj[(int64_t)s * S + i + v] : 0.0f;
      }
    for (int p = w; p < P; p += PSPLIT) {
      float ja[VEC], o[VEC];
      if constexpr (VEC == 4) {
        const float4 t = folx_ld_stream4(aj + (int64_t)p * S + i);
        ja[0] = t.x; ja[1] = t.y; ja[2] = t.z; ja[3] = t.w;
      } else {
        ja[0] = __builtin_nontemporal_load(&aj[(int64_t)p * S + i]);
      }
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        o[v] = bv[v] * ja[v];
#pragma unroll
        for (int s = 0; s < KMAX; ++s)
          if (ix[s][v] == p) { o[v] += av[v] * bs[s][v]; sab[v] += ja[v] * bs[s][v]; }
      }
      if constexpr (VEC == 4) folx_st_stream4(yj + (int64_t)p * S + i, make_float4(o[0], o[1], o[2], o[3]));
      else __builtin_nontemporal_store(o[0], &yj[(int64_t)p * S + i]);
    }
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) red[w][v][lane] = sab[v];
  __syncthreads();
  if (w == 0 && active) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float s = red[0][v][lane] + red[1][v][lane] + red[2][v][lane] + red[3][v][lane];
      y[i + v] = av[v] * bv[v];
      yl[i + v] = bv[v] * al[i + v] + av[v] * bl[i + v] + 2.0f * s;
    }
  }
}

__global__ __launch_bounds__(256) void rows_affine_kernel(const float* __restrict__ in,
                                                          float* __restrict__ out, int64_t rows,
                                                          int64_t in_S, int64_t S,
                                                          const float* __restrict__ c,
                                                          const float* __restrict__ d, float alpha,
                                                          float beta, Bcast3 iin, Bcast3 ic,
                                                          Bcast3 id) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= S) return;
  const int64_t oi = iin.off(i);
  const float cv = c ? alpha * c[ic.off(i)] : alpha;
  const float dv = d ? beta * d[id.off(i)] : 0.0f;
  // blockIdx.y strides over rows so that very tall stacks need no 64-bit grid
  for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) out[r * S + i] = in[r * in_S + oi] * cv + dv;
}

// The same map for index spaces whose inner extent is a multiple of 4 and whose operands are contiguous
// (stride 1) or constant (stride 0) along it, all 16-byte aligned: a thread owns four consecutive
// elements, one 128-bit streaming load and store per row, and its three offsets are computed once --
// in 32-bit arithmetic (S < 2^31), without any division when the index space is flat.
__global__ __launch_bounds__(256) void rows_affine_v4_kernel(const float* __restrict__ in,
                                                             float* __restrict__ out, int64_t rows,
                                                             int64_t in_S, int64_t S,
                                                             const float* __restrict__ c,
                                                             const float* __restrict__ d, float alpha,
                                                             float beta, Bcast3 iin, Bcast3 ic,
                                                             Bcast3 id) {
  const uint32_t i = ((uint32_t)blockIdx.x * 256u + threadIdx.x) * 4u;
  if (i >= (uint32_t)S) return;
  const uint32_t n1 = (uint32_t)iin.n1, n2 = (uint32_t)iin.n2;
  uint32_t i0 = 0, i1 = 0, i2 = i;
  if (n2 < (uint32_t)S) {
    i2 = i % n2;
    const uint32_t t = i / n2;
    i1 = t % n1;
    i0 = t / n1;
  }
  const int64_t oi = i0 * iin.s0 + i1 * iin.s1 + i2 * iin.s2;
  float4 cv = make_float4(alpha, alpha, alpha, alpha);
  float4 dv = make_float4(0.f, 0.f, 0.f, 0.f);
  if (c) {
    const float* p = c + (i0 * ic.s0 + i1 * ic.s1 + i2 * ic.s2);
    const float4 v = ic.s2 ? *reinterpret_cast<const float4*>(p) : make_float4(*p, *p, *p, *p);
    cv = make_float4(alpha * v.x, alpha * v.y, alpha * v.z, alpha * v.w);
  }
  if (d) {
    const float* p = d + (i0 * id.s0 + i1 * id.s1 + i2 * id.s2);
    const float4 v = id.s2 ? *reinterpret_cast<const float4*>(p) : make_float4(*p, *p, *p, *p);
    dv = make_float4(beta * v.x, beta * v.y, beta * v.z, beta * v.w);
  }
  for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
    const float* p = in + r * in_S + oi;
    float4 v;
    if (iin.s2) v = folx_ld_stream4(p);
    else v = make_float4(*p, *p, *p, *p);
    folx_st_stream4(out + r * S + i, make_float4(v.x * cv.x + dv.x, v.y * cv.y + dv.y, v.z * cv.z + dv.z, v.w * cv.w + dv.w));
  }
}

Bcast3 mk(const int64_t* dims, int k) {
  Bcast3 b;
  b.n1 = dims[1]; b.n2 = dims[2];
  b.s0 = dims[3 * k + 0]; b.s1 = dims[3 * k + 1]; b.s2 = dims[3 * k + 2];
  return b;
}

}  // namespace

extern "C" int folx_hip_binary_fwdlap(void* stream, int32_t op, const float* a, const float* a_jac,
                                      const float* a_lap, const float* b, const float* b_jac,
                                      const float* b_lap, float* y, float* y_jac, float* y_lap,
                                      const int64_t* dims, int64_t a_S, int64_t b_S, int32_t P) {
  if (!dims || op < 0 || op >= FOLX_BIN_COUNT || P < 0) return FOLX_HIP_EINVAL;
  if (dims[0] < 0 || dims[1] < 0 || dims[2] < 0) return FOLX_HIP_EINVAL;
  const int64_t S = dims[0] * dims[1] * dims[2];
  if (S == 0) return FOLX_HIP_OK;
  if (!a || !a_lap || !b || !b_lap || !y || !y_lap || (P > 0 && (!a_jac || !b_jac || !y_jac)))
    return FOLX_HIP_EINVAL;
  const int64_t blocks = (S + FOLX_WAVE - 1) / FOLX_WAVE;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  Bcast3 ia = mk(dims, 1), ib = mk(dims, 2);
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)blocks), block(FOLX_WAVE * PSPLIT);
#define FOLX_CASE(OP)                                                                         \
  case OP:                                                                                    \
    binary_kernel<OP><<<grid, block, 0, st>>>(a, a_jac, a_lap, b, b_jac, b_lap, y, y_jac,    \
                                               y_lap, S, ia, ib, a_S, b_S, P);                \
    break;
  switch (op) {
    FOLX_CASE(FOLX_BIN_MUL) FOLX_CASE(FOLX_BIN_DIV) FOLX_CASE(FOLX_BIN_ADD) FOLX_CASE(FOLX_BIN_SUB)
    FOLX_CASE(FOLX_BIN_MIN) FOLX_CASE(FOLX_BIN_MAX)
  }
#undef FOLX_CASE
  return folx_launch_status();
}

extern "C" int folx_hip_rows_affine(void* stream, const float* in, float* out, int64_t rows,
                                    int64_t in_S, const float* c, const float* d, float alpha,
                                    float beta, const int64_t* dims) {
  if (!dims || rows < 0 || in_S < 0) return FOLX_HIP_EINVAL;
  if (dims[0] < 0 || dims[1] < 0 || dims[2] < 0) return FOLX_HIP_EINVAL;
  const int64_t S = dims[0] * dims[1] * dims[2];
  if (S == 0 || rows == 0) return FOLX_HIP_OK;
  if (!in || !out) return FOLX_HIP_EINVAL;
  const int64_t blocks = (S + 255) / 256;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  Bcast3 iin = mk(dims, 1), ic = mk(dims, 2), id = mk(dims, 3);
  const unsigned gy = (unsigned)(rows < 1024 ? rows : 1024);
  // 128-bit form: inner extent a multiple of 4, every operand contiguous or constant along it, every other
  // stride and the row pitch multiples of 4 floats, 16-byte aligned pointers, 32-bit element index
  auto vec_ok = [&](const Bcast3& b, const float* p) {
    if (!p) return true;
    if (b.s2 != 0 && b.s2 != 1) return false;
    if (b.s2 == 0) return true;
    return folx_aligned16(p) && (dims[1] == 1 || b.s1 % 4 == 0) && (dims[0] == 1 || b.s0 % 4 == 0);
  };
  const bool v4 = dims[2] % 4 == 0 && S < 0x7fffffffLL && folx_aligned16(out) && vec_ok(iin, in) && vec_ok(ic, c) &&
                  vec_ok(id, d) && (rows == 1 || iin.s2 == 0 || in_S % 4 == 0);
  if (v4) {
    const int64_t blocks4 = (S / 4 + 255) / 256;
    rows_affine_v4_kernel<<<dim3((unsigned)blocks4, gy), dim3(256), 0, (hipStream_t)stream>>>(
        in, out, rows, in_S, S, c, d, alpha, beta, iin, ic, id);
  } else {
    rows_affine_kernel<<<dim3((unsigned)blocks, gy), dim3(256), 0, (hipStream_t)stream>>>(
        in, out, rows, in_S, S, c, d, alpha, beta, iin, ic, id);
  }
  return folx_launch_status();
}

extern "C" int folx_hip_mul_sparse_fwdlap(void* stream, const float* a, const float* a_jac, const float* a_lap,
                                          const float* b, const float* b_jac, const float* b_lap,
                                          const int32_t* index, float* y, float* y_jac, float* y_lap, int64_t S,
                                          int64_t S_w, int32_t P, int32_t k_rows) {
  if (S < 0 || S_w <= 0 || P < 0 || k_rows < 0) return FOLX_HIP_EINVAL;
  if (S == 0) return FOLX_HIP_OK;
  if (S % S_w != 0) return FOLX_HIP_EINVAL;
  if (!a || !a_lap || !b || !b_lap || !y || !y_lap || (P > 0 && (!a_jac || !y_jac)) ||
      (k_rows > 0 && (!b_jac || !index)))
    return FOLX_HIP_EINVAL;
  if (k_rows > 8) return FOLX_HIP_ENOTSUP;
  const bool vec4 = S_w % 4 == 0 && k_rows <= 4 && folx_aligned16(a) && folx_aligned16(a_jac) && folx_aligned16(a_lap) &&
                    folx_aligned16(b) && folx_aligned16(b_jac) && folx_aligned16(b_lap) && folx_aligned16(y) &&
                    folx_aligned16(y_jac) && folx_aligned16(y_lap);
  const int64_t per_block = FOLX_WAVE * (vec4 ? 4 : 1);
  const int64_t blocks = (S + per_block - 1) / per_block;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  dim3 grid((unsigned)blocks), block(FOLX_WAVE * PSPLIT);
  hipStream_t st = (hipStream_t)stream;
  if (vec4)
    mul_sparse_kernel<4, 4><<<grid, block, 0, st>>>(a, a_jac, a_lap, b, b_jac, b_lap, index, y, y_jac, y_lap, S, S_w, P,
                                                    k_rows);
  else if (k_rows <= 4)
    mul_sparse_kernel<4, 1><<<grid, block, 0, st>>>(a, a_jac, a_lap, b, b_jac, b_lap, index, y, y_jac, y_lap, S, S_w, P,
                                                    k_rows);
  else
    mul_sparse_kernel<8, 1><<<grid, block, 0, st>>>(a, a_jac, a_lap, b, b_jac, b_lap, index, y, y_jac, y_lap, S, S_w, P,
                                                    k_rows);
  return folx_launch_status();
}
