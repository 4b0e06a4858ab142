// slogdet rule for many small matrices with dense Jacobians.
//
// One wavefront owns one n x n matrix (n <= 32, padded to NP in {8, 16, 32}):
//   1. Gauss-Jordan with partial pivoting on [A | I] in LDS gives A^-1; the pivots give
//      sign and log|det| (the same pivot sequence as an LU with partial pivoting).
//   2. tr(A^-1 lap_A) by a lane-strided product.
//   (The matrices may be strided: a stack [batch][row][member][column] is read in place.)
//   3. For every Jacobian row p: stage A_jac[p] in LDS (the next row is prefetched into
//      registers meanwhile), M = A^-1 A_jac[p] with lane (i, column group) holding row i
//      of A^-1 in registers, ld_jac[p] = tr M, and sum_p tr(M M) through an LDS transpose.
// The Jacobian is read exactly once, so the kernel is bound by HBM bandwidth as long as
// the 2 n^3 flops per row stay hidden (they do for n <= 32 on the vector ALUs).
#include "smallmat.h"

namespace {

using smallmat::wave_sum;

// Optional elementwise factor: the matrices are A * F with F a triplet of A's layout whose
// Jacobian is sparse (kf <= KF rows, slot s of the element at per-walker position q standing for
// dense row fidx[s][q]).  Product rule on load:
//   (A F)_jac[p] = F A_jac[p] + A sum_{s: fidx[s] = p} F_jac[s],
//   (A F)_lap    = F A_lap + A F_lap + 2 sum_s A_jac[fidx[s]] F_jac[s].
struct Factor {
  const float *x, *jac, *lap;   // F [..], F_jac [kf][..] (row stride = `slice`), F_lap [..]
  const int32_t* idx;           // [kf][S_w]
  int64_t S_w;                  // elements per walker
  int32_t kf;
};
constexpr int KF = 4;

template <int NP, bool HAS_F>
__global__ __launch_bounds__(FOLX_WAVE) void slogdet_kernel(
    const float* __restrict__ A, const float* __restrict__ AJ, const float* __restrict__ AL,
    float* __restrict__ sign_out, float* __restrict__ logdet_out, float* __restrict__ jac_out,
    float* __restrict__ lap_out, int64_t NM, int32_t n, int32_t P, int64_t ND, int64_t bstride, int64_t dstride,
    int64_t rstride, int64_t slice, int32_t share, Factor fc) {
  constexpr int AUGS = smallmat::Aug<NP>::stride;  // row stride of the augmented matrix
  constexpr int G = FOLX_WAVE / NP;    // lane groups per row
  constexpr int CPL = NP / G;          // columns of M per lane
  constexpr int MS = NP + 1;           // row stride of the M staging tile
  constexpr int EPL = NP * NP / FOLX_WAVE;  // Jacobian elements prefetched per lane
  __shared__ float aug[NP * AUGS];
  __shared__ __attribute__((aligned(16))) float jb[2][NP * NP];
  __shared__ float mb[NP * MS];

  const int lane = threadIdx.x;
  // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  When `share`
  // neighbouring matrices lie in the same 128-byte lines (rows of n floats side by side), they
  // are given to the same XCD in consecutive slots, so that every line comes from HBM once.
  int64_t m = blockIdx.x;
  if (share > 1) {
    const int64_t chunk = 8 * (int64_t)share;
    const int64_t c = m / chunk, r = m % chunk;
    if ((c + 1) * chunk <= NM) m = c * chunk + (r % 8) * share + r / 8;
  }
  // matrix m = (batch m / ND, member m % ND); element (i, j) at base + i * rstride + j
  const int64_t base = (m / ND) * bstride + (m % ND) * dstride;
  const float* a = A + base;

  float logdet, sgn;
  smallmat::gauss_jordan<NP>(aug, a, n, lane, logdet, sgn, rstride, HAS_F ? fc.x + base : nullptr);
  float tl = HAS_F ? 0.0f : smallmat::trace_inv_times<NP>(aug, AL + base, n, lane, rstride);

  // ---- row i of A^-1 in registers -------------------------------------------------------
  const int i = lane % NP;
  const int g = lane / NP;
  const int col0 = g * CPL;
  float ainv[NP];
#pragma unroll
  for (int j = 0; j < NP; ++j) ainv[j] = aug[i * AUGS + NP + j];

  // this lane's EPL elements of the padded tile; with a factor also its values at them
  constexpr int EF = HAS_F ? EPL : 1;
  float fx[EF], ax[EF], lapx[EF], fj[KF][EF];
  int32_t fidx[KF][EF];
  if constexpr (HAS_F) {
#pragma unroll
    for (int c = 0; c < EPL; ++c) {
      const int e = lane + c * FOLX_WAVE;
      const int r = e / NP, cc = e % NP;
      const bool ok = r < n && cc < n;
      const int64_t off = base + r * rstride + cc;
      fx[c] = ok ? fc.x[off] : 0.0f;
      ax[c] = ok ? A[off] : 0.0f;
      lapx[c] = 0.0f;
#pragma unroll
      for (int sl = 0; sl < KF; ++sl) {
        fidx[sl][c] = (ok && sl < fc.kf) ? fc.idx[(int64_t)sl * fc.S_w + off % fc.S_w] : -1;
        fj[sl][c] = fidx[sl][c] >= 0 ? fc.jac[(int64_t)sl * slice + off] : 0.0f;
      }
    }
  }

  float mm = 0.0f;
  float pre[EPL];
  auto prefetch = [&](int p) {
    const float* src = AJ + (int64_t)p * slice + base;
#pragma unroll
    for (int c = 0; c < EPL; ++c) {
      const int e = lane + c * FOLX_WAVE;  // index into the padded NP x NP tile
      const int r = e / NP, cc = e % NP;
      float v = (r < n && cc < n) ? src[r * rstride + cc] : 0.0f;
      if constexpr (HAS_F) {
        float add = 0.0f;
#pragma unroll
        for (int sl = 0; sl < KF; ++sl)
          if (fidx[sl][c] == p) { add += fj[sl][c]; lapx[c] += 2.0f * v * fj[sl][c]; }
        v = fx[c] * v + ax[c] * add;
      }
      pre[c] = v;
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
  if constexpr (HAS_F) {
#pragma unroll
    for (int c = 0; c < EPL; ++c) {
      const int e = lane + c * FOLX_WAVE;
      const int r = e / NP, cc = e % NP;
      if (r < n && cc < n) {
        const int64_t off = base + r * rstride + cc;
        const float al = fx[c] * AL[off] + ax[c] * fc.lap[off] + lapx[c];
        tl += aug[cc * AUGS + NP + r] * al;  // tr(A^-1 lap A) = sum A^-1[c][r] lap A[r][c]
      }
    }
  }
  mm = wave_sum(mm);
  tl = wave_sum(tl);
  if (lane == 0) {
    sign_out[m] = sgn;
    logdet_out[m] = logdet;
    lap_out[m] = tl - mm;
  }
}

// slogdet rule from rank-one factors of dA/dx_c (sparse Jacobian whose coordinate c touches
// few rows, columns or entries of A).  For coordinate c, factor s collects `width` entries
// dA[r_s][j_l]/dx_c (addresses in `take`, columns j_l in `cols`), `rows[c][t]` is the row of
// factor t, and
//     W_c[s][t] = sum_l dA[r_s][j_l]/dx_c * Ainv[j_l][r_t]
// gives d_c log|det A| = tr W_c and lap = tr(Ainv lap_A) - sum_c sum_st W_c[s][t] W_c[t][s].
// With `transposed` the tables describe A^T: addresses already point into A, and the
// inverse is read transposed.  One wavefront per matrix, tables shared by all matrices.
constexpr int SP_MAX_RANK = 64;       // W_c tile held in LDS: rank^2 floats
constexpr int SP_MAX_FACTOR = 2048;   // staged factor entries per coordinate: rank * width

template <int NP>
__global__ __launch_bounds__(FOLX_WAVE) void sparse_slogdet_kernel(
    const float* __restrict__ A, const float* __restrict__ AJ, const float* __restrict__ AL,
    const int32_t* __restrict__ take, const int32_t* __restrict__ cols, const int32_t* __restrict__ rows,
    float* __restrict__ sign_out, float* __restrict__ logdet_out, float* __restrict__ jac_out,
    float* __restrict__ lap_out, int64_t NM, int32_t n, int32_t n_coords, int32_t rank, int32_t width,
    int32_t transposed) {
  constexpr int AUGS = smallmat::Aug<NP>::stride;
  __shared__ float aug[NP * AUGS];
  __shared__ float wb[SP_MAX_RANK * SP_MAX_RANK];
  __shared__ float vb[SP_MAX_FACTOR];
  __shared__ int32_t cb[SP_MAX_FACTOR];
  __shared__ int32_t rb[SP_MAX_RANK];

  const int lane = threadIdx.x;
  const int64_t m = blockIdx.x;
  const int64_t nn = (int64_t)n * n;
  float logdet, sgn;
  smallmat::gauss_jordan<NP>(aug, A + m * nn, n, lane, logdet, sgn);
  float tl = smallmat::trace_inv_times<NP>(aug, AL + m * nn, n, lane);

  const int rw = rank * width;
  float pair = 0.0f;
  for (int c = 0; c < n_coords; ++c) {
    // stage the factor entries of this coordinate
    for (int e = lane; e < rw; e += FOLX_WAVE) {
      const int32_t t = take[(int64_t)c * rw + e];
      float v = 0.0f;
      if (t >= 0) {
        const int32_t row = t / (int32_t)nn, rem = t % (int32_t)nn;
        v = AJ[((int64_t)row * NM + m) * nn + rem];
      }
      vb[e] = v;
      cb[e] = cols[(int64_t)c * rw + e];
    }
    for (int e = lane; e < rank; e += FOLX_WAVE) rb[e] = rows[(int64_t)c * rank + e];
    __syncthreads();
    for (int e = lane; e < rank * rank; e += FOLX_WAVE) {
      const int s = e / rank, t = e % rank;
      const int rt = rb[t];
      float w = 0.0f;
      for (int l = 0; l < width; ++l) {
        const int j = cb[s * width + l];
        const float ai = transposed ? aug[rt * AUGS + NP + j] : aug[j * AUGS + NP + rt];
        w += vb[s * width + l] * ai;
      }
      wb[e] = w;
    }
    __syncthreads();
    float tr = 0.0f;
    for (int e = lane; e < rank * rank; e += FOLX_WAVE) {
      const int s = e / rank, t = e % rank;
      const float w = wb[e];
      if (s == t) tr += w;
      pair += w * wb[t * rank + s];
    }
    tr = wave_sum(tr);
    if (lane == 0) jac_out[(int64_t)c * NM + m] = tr;
    __syncthreads();  // wb, vb, cb, rb are rewritten by the next coordinate
  }
  pair = wave_sum(pair);
  tl = wave_sum(tl);
  if (lane == 0) {
    sign_out[m] = sgn;
    logdet_out[m] = logdet;
    lap_out[m] = tl - pair;
  }
}

}  // namespace

namespace {

int launch_slogdet(hipStream_t st, const float* A, const float* A_jac, const float* A_lap, float* sign, float* logdet,
                   float* ld_jac, float* ld_lap, int64_t NB, int64_t ND, int32_t n, int32_t P, int64_t batch_stride,
                   int64_t member_stride, int64_t row_stride, int64_t jac_stride, const Factor* fc) {
  const int64_t NM = NB * ND;
  dim3 grid((unsigned)NM), block(FOLX_WAVE);
  // members stored side by side along the rows with rows shorter than a 128-byte line
  int32_t share = 1;
  if (member_stride == n && n * 4 < 128 && ND > 1) {
    share = 128 / (n * 4);
    while (share > 1 && ND % share != 0) share /= 2;
  }
#define FOLX_SLD_LAUNCH(NPV, HASF)                                                                             \
  slogdet_kernel<NPV, HASF><<<grid, block, 0, st>>>(A, A_jac, A_lap, sign, logdet, ld_jac, ld_lap, NM, n, P, ND, \
                                                    batch_stride, member_stride, row_stride, jac_stride, share,  \
                                                    fc ? *fc : Factor{})
  if (fc) {
    if (n <= 8) FOLX_SLD_LAUNCH(8, true);
    else FOLX_SLD_LAUNCH(16, true);
  } else {
    if (n <= 8) FOLX_SLD_LAUNCH(8, false);
    else if (n <= 16) FOLX_SLD_LAUNCH(16, false);
    else FOLX_SLD_LAUNCH(32, false);
  }
#undef FOLX_SLD_LAUNCH
  return folx_launch_status();
}

}  // namespace

extern "C" int folx_hip_slogdet_strided_fwdlap(void* stream, const float* A, const float* A_jac,
                                               const float* A_lap, float* sign, float* logdet,
                                               float* ld_jac, float* ld_lap, int64_t NB, int64_t ND,
                                               int32_t n, int32_t P, int64_t batch_stride,
                                               int64_t member_stride, int64_t row_stride,
                                               int64_t jac_stride) {
  if (NB < 0 || ND <= 0 || n <= 0 || P < 0 || row_stride < n) return FOLX_HIP_EINVAL;
  const int64_t NM = NB * ND;
  if (NM == 0) return FOLX_HIP_OK;
  if (!A || !A_lap || !sign || !logdet || !ld_lap || (P > 0 && (!A_jac || !ld_jac))) return FOLX_HIP_EINVAL;
  if (n > 32 || NM > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  return launch_slogdet((hipStream_t)stream, A, A_jac, A_lap, sign, logdet, ld_jac, ld_lap, NB, ND, n, P,
                        batch_stride, member_stride, row_stride, jac_stride, nullptr);
}

extern "C" int folx_hip_slogdet_scaled_fwdlap(void* stream, const float* A, const float* A_jac, const float* A_lap,
                                              const float* F, const float* F_jac, const float* F_lap,
                                              const int32_t* index, float* sign, float* logdet, float* ld_jac,
                                              float* ld_lap, int64_t NB, int64_t ND, int32_t n, int32_t P,
                                              int64_t batch_stride, int64_t member_stride, int64_t row_stride,
                                              int64_t jac_stride, int64_t walker_elems, int32_t k_rows) {
  if (NB < 0 || ND <= 0 || n <= 0 || P < 0 || row_stride < n || walker_elems <= 0 || k_rows < 0)
    return FOLX_HIP_EINVAL;
  const int64_t NM = NB * ND;
  if (NM == 0) return FOLX_HIP_OK;
  if (!A || !A_lap || !F || !F_lap || !sign || !logdet || !ld_lap || (P > 0 && (!A_jac || !ld_jac)) ||
      (k_rows > 0 && (!F_jac || !index)))
    return FOLX_HIP_EINVAL;
  if (n > 16 || k_rows > KF || NM > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  Factor fc;
  fc.x = F; fc.jac = F_jac; fc.lap = F_lap; fc.idx = index; fc.S_w = walker_elems; fc.kf = k_rows;
  return launch_slogdet((hipStream_t)stream, A, A_jac, A_lap, sign, logdet, ld_jac, ld_lap, NB, ND, n, P,
                        batch_stride, member_stride, row_stride, jac_stride, &fc);
}

extern "C" int folx_hip_slogdet_fwdlap(void* stream, const float* A, const float* A_jac,
                                       const float* A_lap, float* sign, float* logdet,
                                       float* ld_jac, float* ld_lap, int64_t NM, int32_t n,
                                       int32_t P) {
  if (NM < 0 || n <= 0 || P < 0) return FOLX_HIP_EINVAL;
  const int64_t nn = (int64_t)n * n;
  return folx_hip_slogdet_strided_fwdlap(stream, A, A_jac, A_lap, sign, logdet, ld_jac, ld_lap, NM, 1, n, P, nn, 0,
                                         n, NM * nn);
}

extern "C" int folx_hip_sparse_slogdet_fwdlap(void* stream, const float* A, const float* A_jac,
                                              const float* A_lap, const int32_t* take, const int32_t* cols,
                                              const int32_t* rows, float* sign, float* logdet, float* ld_jac,
                                              float* ld_lap, int64_t NM, int32_t n, int32_t k,
                                              int32_t n_coords, int32_t rank, int32_t width,
                                              int32_t transposed) {
  if (NM < 0 || n <= 0 || k <= 0 || n_coords <= 0 || rank <= 0 || width <= 0) return FOLX_HIP_EINVAL;
  if (NM == 0) return FOLX_HIP_OK;
  if (!A || !A_jac || !A_lap || !take || !cols || !rows || !sign || !logdet || !ld_jac || !ld_lap)
    return FOLX_HIP_EINVAL;
  if (n > 32 || NM > 0x7fffffffLL || rank > SP_MAX_RANK || (int64_t)rank * width > SP_MAX_FACTOR ||
      (int64_t)k * n * n > 0x7fffffffLL)
    return FOLX_HIP_ENOTSUP;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)NM), block(FOLX_WAVE);
#define FOLX_SP_LAUNCH(NPV)                                                                          \
  sparse_slogdet_kernel<NPV><<<grid, block, 0, st>>>(A, A_jac, A_lap, take, cols, rows, sign, logdet, \
                                                     ld_jac, ld_lap, NM, n, n_coords, rank, width, transposed)
  if (n <= 8) FOLX_SP_LAUNCH(8);
  else if (n <= 16) FOLX_SP_LAUNCH(16);
  else FOLX_SP_LAUNCH(32);
#undef FOLX_SP_LAUNCH
  return folx_launch_status();
}
