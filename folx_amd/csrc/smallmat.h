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
// A^-1[i][j] (the left half of aug is not written).  The pivots give sign and log|det| (the
// pivot sequence is the one of an LU with partial pivoting, first maximum wins as in idamax).
// Padding rows/columns carry a unit diagonal, so the elimination leaves them alone.  Called
// by all 64 lanes of the one wavefront of the workgroup.
//
// The elimination runs in registers: lane j < 2 NP holds column j of [A | I], one register per
// row.  A pivot step reads column k into wave-uniform values (v_readlane, the lane index is a
// compile-time constant because the loop over k is unrolled), picks the pivot among them,
// swaps the two rows in every lane's registers and updates each column with NP multiply-adds:
// no LDS round trip and no barrier inside the chain of NP dependent steps.
template <int NP>
__device__ __forceinline__ void gauss_jordan(float* aug, const float* __restrict__ a, int n, int lane,
                                             float& logdet, float& sgn, int64_t row_stride = 0,
                                             const float* __restrict__ factor = nullptr) {
  static_assert(2 * NP <= FOLX_WAVE, "one lane per column of [A | I]");
  if (row_stride == 0) row_stride = n;  // rows of the matrix follow each other
  constexpr int AUGS = Aug<NP>::stride;
  // All loads are issued before the first one is waited for: lanes and rows outside the
  // matrix ask for element (0, 0) instead of branching around the load.
  float col[NP];
  const bool in_cols = lane < n;
  if (factor) {  // the matrix is the elementwise product a * factor (same layout)
    float fv[NP];
#pragma unroll
    for (int r = 0; r < NP; ++r) {
      const int64_t off = (in_cols && r < n) ? r * row_stride + lane : 0;
      col[r] = a[off];
      fv[r] = factor[off];
    }
#pragma unroll
    for (int r = 0; r < NP; ++r) col[r] *= fv[r];
  } else {
#pragma unroll
    for (int r = 0; r < NP; ++r) col[r] = a[(in_cols && r < n) ? r * row_stride + lane : 0];
  }
#pragma unroll
  for (int r = 0; r < NP; ++r) {
    const float unit = (lane < NP ? lane : lane - NP) == r ? 1.0f : 0.0f;  // padding and the right half
    col[r] = (in_cols && r < n) ? col[r] : unit;
  }
  logdet = 0.0f;
  sgn = 1.0f;
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    if (k < n) {
      float ck[NP];  // column k, the same in every lane
#pragma unroll
      for (int r = 0; r < NP; ++r) ck[r] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(col[r]), k));
      int piv = k;
      float best = fabsf(ck[k]);
#pragma unroll
      for (int r = k + 1; r < NP; ++r)
        if (r < n && fabsf(ck[r]) > best) { best = fabsf(ck[r]); piv = r; }
      if (piv != k) {
        // rows k and piv change places, in column k's copy and in this lane's column
        float ckp = ck[k], mine = col[k];
#pragma unroll
        for (int r = k + 1; r < NP; ++r)
          if (r == piv) {
            const float t = ck[r]; ck[r] = ckp; ckp = t;
            const float u = col[r]; col[r] = mine; mine = u;
          }
        ck[k] = ckp;
        col[k] = mine;
        sgn = -sgn;
      }
      const float pv = ck[k];
      logdet += logf(fabsf(pv));
      if (pv < 0.0f) sgn = -sgn;
      if (pv == 0.0f) sgn = 0.0f;
      const float pr = col[k] * (1.0f / pv);
#pragma unroll
      for (int r = 0; r < NP; ++r)
        if (r != k) col[r] = fmaf(-ck[r], pr, col[r]);
      col[k] = pr;
    }
  }
  if (lane >= NP && lane < 2 * NP) {
#pragma unroll
    for (int r = 0; r < NP; ++r) aug[r * AUGS + lane] = col[r];
  }
  __syncthreads();
}

// The same elimination for G <= 4 matrices with n <= 8 at once: lanes 16 g .. 16 g + 15 hold the
// 16 columns of [A_g | I], one register per row.  The pivot column is fetched from lane 16 g + k
// of the own group (ds_bpermute) and the row exchange is a pair of selects per row, because the
// pivot row differs from group to group.  `a` is this lane's matrix (element (i, j) at
// a[i * row_stride + j]); a lane with `valid` false eliminates a unit matrix and stores nothing.
// A^-1 of group g ends up at aug[g * Aug<NP>::size + i * stride + NP + j]; logdet and sgn are
// those of the lane's own group.
template <int NP, int G>
__device__ __forceinline__ void gauss_jordan_groups(float* aug, const float* __restrict__ a, bool valid, int n,
                                                    int lane, float& logdet, float& sgn, int64_t row_stride,
                                                    const float* __restrict__ factor = nullptr) {
  static_assert(2 * NP == 16, "sixteen lanes per matrix");
  constexpr int AUGS = Aug<NP>::stride;
  const int j = lane % 16, grp = lane / 16;
  const bool in_cols = valid && j < n;
  float col[NP];
  if (factor) {
    float fv[NP];
#pragma unroll
    for (int r = 0; r < NP; ++r) {
      const int64_t off = (in_cols && r < n) ? r * row_stride + j : 0;
      col[r] = a[off];
      fv[r] = factor[off];
    }
#pragma unroll
    for (int r = 0; r < NP; ++r) col[r] *= fv[r];
  } else {
#pragma unroll
    for (int r = 0; r < NP; ++r) col[r] = a[(in_cols && r < n) ? r * row_stride + j : 0];
  }
#pragma unroll
  for (int r = 0; r < NP; ++r) {
    const float unit = (j < NP ? j : j - NP) == r ? 1.0f : 0.0f;
    col[r] = (in_cols && r < n) ? col[r] : unit;
  }
  logdet = 0.0f;
  sgn = 1.0f;
#pragma unroll
  for (int k = 0; k < NP; ++k) {
    if (k < n) {
      float ck[NP];  // column k of the own group's matrix
#pragma unroll
      for (int r = 0; r < NP; ++r) ck[r] = __shfl(col[r], 16 * grp + k, FOLX_WAVE);
      int piv = k;
      float best = fabsf(ck[k]);
#pragma unroll
      for (int r = k + 1; r < NP; ++r) {
        const bool take = r < n && fabsf(ck[r]) > best;
        best = take ? fabsf(ck[r]) : best;
        piv = take ? r : piv;
      }
      float ckp = ck[k], mine = col[k];
#pragma unroll
      for (int r = k + 1; r < NP; ++r) {
        const bool sw = r == piv;
        const float t = ck[r], u = col[r];
        ck[r] = sw ? ckp : t;
        ckp = sw ? t : ckp;
        col[r] = sw ? mine : u;
        mine = sw ? u : mine;
      }
      ck[k] = ckp;
      col[k] = mine;
      sgn = piv != k ? -sgn : sgn;
      const float pv = ck[k];
      logdet += logf(fabsf(pv));
      sgn = pv < 0.0f ? -sgn : sgn;
      sgn = pv == 0.0f ? 0.0f : sgn;
      const float pr = col[k] * (1.0f / pv);
#pragma unroll
      for (int r = 0; r < NP; ++r)
        if (r != k) col[r] = fmaf(-ck[r], pr, col[r]);
      col[k] = pr;
    }
  }
  if (j >= NP && grp < G) {
#pragma unroll
    for (int r = 0; r < NP; ++r) aug[grp * Aug<NP>::size + r * AUGS + j] = col[r];
  }
  __syncthreads();
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
