// slogdet rule for many small matrices with dense Jacobians.
//
// One wavefront owns one n x n matrix (n <= 32, padded to NP in {8, 16, 32}):
//   1. Gauss-Jordan with partial pivoting on [A | I] in LDS gives A^-1; the pivots give
//      sign and log|det| (the same pivot sequence as an LU with partial pivoting).
//   2. tr(A^-1 lap_A) by a lane-strided product.
//   3. For every Jacobian row p: stage A_jac[p] in LDS (the next row is prefetched into
//      registers meanwhile), M = A^-1 A_jac[p] with lane (i, column group) holding row i
//      of A^-1 in registers, ld_jac[p] = tr M, and sum_p tr(M M) through an LDS transpose.
// The Jacobian is read exactly once, so the kernel is bound by HBM bandwidth as long as
// the 2 n^3 flops per row stay hidden (they do for n <= 32 on the vector ALUs).
#include "common.h"

namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = FOLX_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, FOLX_WAVE);
  return v;
}

template <int NP>
__global__ __launch_bounds__(FOLX_WAVE) void slogdet_kernel(
    const float* __restrict__ A, const float* __restrict__ AJ, const float* __restrict__ AL,
    float* __restrict__ sign_out, float* __restrict__ logdet_out, float* __restrict__ jac_out,
    float* __restrict__ lap_out, int64_t NM, int32_t n, int32_t P) {
  constexpr int AUGS = 2 * NP + 1;     // row stride of the augmented matrix
  constexpr int G = FOLX_WAVE / NP;    // lane groups per row
  constexpr int CPL = NP / G;          // columns of M per lane
  constexpr int MS = NP + 1;           // row stride of the M staging tile
  constexpr int EPL = NP * NP / FOLX_WAVE;  // Jacobian elements prefetched per lane
  __shared__ float aug[NP * AUGS];
  __shared__ __attribute__((aligned(16))) float jb[2][NP * NP];
  __shared__ float mb[NP * MS];

  const int lane = threadIdx.x;
  const int64_t m = blockIdx.x;
  const int64_t nn = (int64_t)n * n;
  const float* a = A + m * nn;

  // ---- stage [A | I], zero padded (padding rows get a unit diagonal on the A side so
  // the elimination leaves them alone; their inverse block stays zero-coupled) ----------
  for (int e = lane; e < NP * 2 * NP; e += FOLX_WAVE) {
    const int i = e / (2 * NP), j = e % (2 * NP);
    float v;
    if (j < NP) v = (i < n && j < n) ? a[i * n + j] : (i == j ? 1.0f : 0.0f);
    else v = (j - NP == i) ? 1.0f : 0.0f;
    aug[i * AUGS + j] = v;
  }
  __syncthreads();

  float logdet = 0.0f, sgn = 1.0f;
  for (int k = 0; k < n; ++k) {
    // pivot search over rows k..n-1 of column k (first maximum wins, as in idamax)
    float best = -1.0f;
    int bi = k;
    if (lane >= k && lane < n) { best = fabsf(aug[lane * AUGS + k]); bi = lane; }
#pragma unroll
    for (int off = FOLX_WAVE / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, FOLX_WAVE);
      const int oi = __shfl_xor(bi, off, FOLX_WAVE);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    if (bi != k) {
      for (int j = lane; j < 2 * NP; j += FOLX_WAVE) {
        const float t = aug[k * AUGS + j];
        aug[k * AUGS + j] = aug[bi * AUGS + j];
        aug[bi * AUGS + j] = t;
      }
      sgn = -sgn;
      __syncthreads();
    }
    const float pv = aug[k * AUGS + k];
    logdet += logf(fabsf(pv));
    if (pv < 0.0f) sgn = -sgn;
    if (pv == 0.0f) sgn = 0.0f;
    const float rp = 1.0f / pv;
    __syncthreads();
    float rowk[(2 * NP + FOLX_WAVE - 1) / FOLX_WAVE];
#pragma unroll
    for (int c = 0; c < (2 * NP + FOLX_WAVE - 1) / FOLX_WAVE; ++c) {
      const int j = lane + c * FOLX_WAVE;
      if (j < 2 * NP) {
        rowk[c] = aug[k * AUGS + j] * rp;
        aug[k * AUGS + j] = rowk[c];
      }
    }
    __syncthreads();
    for (int i = 0; i < n; ++i) {
      if (i == k) continue;
      const float f = aug[i * AUGS + k];
      __syncthreads();  // everyone has read f before column k of row i is overwritten
#pragma unroll
      for (int c = 0; c < (2 * NP + FOLX_WAVE - 1) / FOLX_WAVE; ++c) {
        const int j = lane + c * FOLX_WAVE;
        if (j < 2 * NP) aug[i * AUGS + j] -= f * rowk[c];
      }
    }
    __syncthreads();
  }

  // ---- tr(A^-1 lap_A) = sum_ij Ainv[j][i] lap[i][j] -----------------------------------
  float tl = 0.0f;
  {
    const float* l = AL + m * nn;
    for (int e = lane; e < nn; e += FOLX_WAVE) {
      const int i = e / n, j = e % n;
      tl += aug[j * AUGS + NP + i] * l[e];
    }
  }

  // ---- row i of A^-1 in registers -------------------------------------------------------
  const int i = lane % NP;
  const int g = lane / NP;
  const int col0 = g * CPL;
  float ainv[NP];
#pragma unroll
  for (int j = 0; j < NP; ++j) ainv[j] = aug[i * AUGS + NP + j];

  float mm = 0.0f;
  float pre[EPL];
  auto prefetch = [&](int p) {
    const float* src = AJ + ((int64_t)p * NM + m) * nn;
#pragma unroll
    for (int c = 0; c < EPL; ++c) {
      const int e = lane + c * FOLX_WAVE;  // index into the padded NP x NP tile
      const int r = e / NP, cc = e % NP;
      pre[c] = (r < n && cc < n) ? src[r * n + cc] : 0.0f;
    }
  };
  if (P > 0) prefetch(0);
  for (int p = 0; p < P; ++p) {
    float* J = jb[p & 1];
#pragma unroll
    for (int c = 0; c < EPL; ++c) J[lane + c * FOLX_WAVE] = pre[c];
    __syncthreads();
    if (p + 1 < P) prefetch(p + 1);

    // trace of M without forming it: sum_{j,i} Ainv[i][j] J[j][i]
    float tr = 0.0f;
#pragma unroll
    for (int c = 0; c < EPL; ++c) {
      const int e = lane + c * FOLX_WAVE;
      const int j = e / NP, ii = e % NP;
      tr += aug[ii * AUGS + NP + j] * J[e];
    }
    tr = wave_sum(tr);
    if (lane == 0) jac_out[(int64_t)p * NM + m] = tr;

    // M[i][col0 .. col0 + CPL)
    float acc[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) acc[c] = 0.0f;
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      if constexpr (CPL % 4 == 0) {
#pragma unroll
        for (int c = 0; c < CPL; c += 4) {
          const float4 v = *reinterpret_cast<const float4*>(&J[j * NP + col0 + c]);
          acc[c + 0] += ainv[j] * v.x; acc[c + 1] += ainv[j] * v.y;
          acc[c + 2] += ainv[j] * v.z; acc[c + 3] += ainv[j] * v.w;
        }
      } else {
#pragma unroll
        for (int c = 0; c < CPL; ++c) acc[c] += ainv[j] * J[j * NP + col0 + c];
      }
    }
#pragma unroll
    for (int c = 0; c < CPL; ++c) mb[i * MS + col0 + c] = acc[c];
    __syncthreads();
#pragma unroll
    for (int c = 0; c < CPL; ++c) mm += acc[c] * mb[(col0 + c) * MS + i];
    // the next iteration writes the other jb buffer; mb is rewritten only after the
    // barrier that follows that write, when every lane is past this read
  }
  mm = wave_sum(mm);
  tl = wave_sum(tl);
  if (lane == 0) {
    sign_out[m] = sgn;
    logdet_out[m] = logdet;
    lap_out[m] = tl - mm;
  }
}

}  // namespace

extern "C" int folx_hip_slogdet_fwdlap(void* stream, const float* A, const float* A_jac,
                                       const float* A_lap, float* sign, float* logdet,
                                       float* ld_jac, float* ld_lap, int64_t NM, int32_t n,
                                       int32_t P) {
  if (NM < 0 || n <= 0 || P < 0) return FOLX_HIP_EINVAL;
  if (NM == 0) return FOLX_HIP_OK;
  if (!A || !A_lap || !sign || !logdet || !ld_lap || (P > 0 && (!A_jac || !ld_jac))) return FOLX_HIP_EINVAL;
  if (n > 32 || NM > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)NM), block(FOLX_WAVE);
  if (n <= 8)
    slogdet_kernel<8><<<grid, block, 0, st>>>(A, A_jac, A_lap, sign, logdet, ld_jac, ld_lap, NM, n, P);
  else if (n <= 16)
    slogdet_kernel<16><<<grid, block, 0, st>>>(A, A_jac, A_lap, sign, logdet, ld_jac, ld_lap, NM, n, P);
  else
    slogdet_kernel<32><<<grid, block, 0, st>>>(A, A_jac, A_lap, sign, logdet, ld_jac, ld_lap, NM, n, P);
  return folx_launch_status();
}
