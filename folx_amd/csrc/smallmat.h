// One-wavefront building blocks for n x n matrices with n <= 32 held in LDS.
#pragma once
#include "common.h"

namespace smallmat {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = FOLX_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, FOLX_WAVE);
  return v;
}

// Row stride of the augmented matrix [A | I] for a padded size NP (odd, so that a column
// walk does not stay in one LDS bank).
template <int NP>
struct Aug {
  static constexpr int stride = 2 * NP + 1;
  static constexpr int size = NP * (2 * NP + 1);
};

// Gauss-Jordan with partial pivoting on [A | I]; afterwards aug[i * stride + NP + j] is
// A^-1[i][j].  The pivots give sign and log|det| (the pivot sequence is the one of an LU
// with partial pivoting, first maximum wins as in idamax).  Padding rows/columns carry a
// unit diagonal, so the elimination leaves them alone.  Called by all 64 lanes of the one
// wavefront of the workgroup.
template <int NP>
__device__ __forceinline__ void gauss_jordan(float* aug, const float* __restrict__ a, int n, int lane,
                                             float& logdet, float& sgn, int64_t row_stride = 0,
                                             const float* __restrict__ factor = nullptr) {
  if (row_stride == 0) row_stride = n;  // rows of the matrix follow each other
  constexpr int AUGS = Aug<NP>::stride;
  constexpr int RK = (2 * NP + FOLX_WAVE - 1) / FOLX_WAVE;
  for (int e = lane; e < NP * 2 * NP; e += FOLX_WAVE) {
    const int i = e / (2 * NP), j = e % (2 * NP);
    float v;
    // with `factor` (same layout as a) the matrix is the elementwise product a * factor
    if (j < NP) v = (i < n && j < n) ? a[i * row_stride + j] * (factor ? factor[i * row_stride + j] : 1.0f)
                                     : (i == j ? 1.0f : 0.0f);
    else v = (j - NP == i) ? 1.0f : 0.0f;
    aug[i * AUGS + j] = v;
  }
  __syncthreads();

  logdet = 0.0f;
  sgn = 1.0f;
  for (int k = 0; k < n; ++k) {
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
    float rowk[RK];
#pragma unroll
    for (int c = 0; c < RK; ++c) {
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
      for (int c = 0; c < RK; ++c) {
        const int j = lane + c * FOLX_WAVE;
        if (j < 2 * NP) aug[i * AUGS + j] -= f * rowk[c];
      }
    }
    __syncthreads();
  }
}

// tr(A^-1 L) = sum_ij A^-1[j][i] L[i][j], partial sum of this lane.
template <int NP>
__device__ __forceinline__ float trace_inv_times(const float* aug, const float* __restrict__ l, int n, int lane,
                                                 int64_t row_stride = 0) {
  if (row_stride == 0) row_stride = n;
  constexpr int AUGS = Aug<NP>::stride;
  float t = 0.0f;
  for (int e = lane; e < n * n; e += FOLX_WAVE) {
    const int i = e / n, j = e % n;
    t += aug[j * AUGS + NP + i] * l[i * row_stride + j];
  }
  return t;
}

}  // namespace smallmat
