// slogdet rule for many small matrices with dense Jacobians.
//
// One wavefront owns one n x n matrix (n <= 32, padded to NP in {8, 16, 32}):
//   1. Gauss-Jordan with partial pivoting on [A | I] in registers (lane j holds column j,
//      smallmat.h) gives A^-1; the pivots give sign and log|det| (the same pivot sequence
//      as an LU with partial pivoting).
//   2. tr(A^-1 lap_A) by a lane-strided product.
//   (The matrices may be strided: a stack [batch][row][member][column] is read in place.)
//   3. For every Jacobian row p: A_jac[p] goes from global memory straight into MFMA
//      operand registers (the next row is prefetched meanwhile), M = A^-1 A_jac[p] and its
//      transpose are two MFMA products of the same registers (operands swapped),
//      sum_p tr(M M) is the elementwise product of the two accumulators, ld_jac[p] = tr M
//      the lane-wise product of the operands, reduced over the wavefront 16 rows at a time
//      through LDS.
// The Jacobian is read exactly once; 4 n^3 flops per row on the matrix cores.
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

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// One MFMA tile covers the matrix: 16 x 16 (v_mfma_f32_16x16x4_f32) for n <= 16, 32 x 32
// (v_mfma_f32_32x32x2_f32) above.  Lane l holds, for step t, the element (k = KS t + l / MP,
// lr = l % MP) of an operand: as A operand that is row lr, column k; as B operand row k,
// column lr.  With a[t] = Ainv[lr][k] and j[t] = J[k][lr]:
//   mfma(a, j) accumulates M   = Ainv J      (A = Ainv,  B = J)
//   mfma(j, a) accumulates M^T = J^T Ainv^T  (A = J^T,   B = Ainv^T) -- the SAME registers,
// so the transpose that tr(M M) = sum_ab M[a][b] M^T[a][b] needs costs a second product and
// no data movement, and tr M = sum over lanes and steps of a[t] j[t].
template <int MP>
struct Tile;
template <>
struct Tile<16> {
  static constexpr int KS = 4, STEPS = 4, CR = 4;
  typedef floatx4 acc_t;
  static __device__ __forceinline__ acc_t mfma(float a, float b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
};
template <>
struct Tile<32> {
  static constexpr int KS = 2, STEPS = 16, CR = 16;
  typedef floatx16 acc_t;
  static __device__ __forceinline__ acc_t mfma(float a, float b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
};

constexpr int TRB = 16;  // Jacobian rows whose traces are reduced together

// KFT = slots of the factor's sparse Jacobian the kernel keeps in registers (>= fc.kf).
template <int NP, bool HAS_F, int KFT = KF>
__global__ __launch_bounds__(FOLX_WAVE, 3) void slogdet_kernel(
    const float* __restrict__ A, const float* __restrict__ AJ, const float* __restrict__ AL,
    float* __restrict__ sign_out, float* __restrict__ logdet_out, float* __restrict__ jac_out,
    float* __restrict__ lap_out, int64_t NM, int32_t n, int32_t P, int64_t ND, int64_t bstride, int64_t dstride,
    int64_t rstride, int64_t slice, int32_t share, Factor fc) {
  constexpr int AUGS = smallmat::Aug<NP>::stride;  // row stride of the augmented matrix
  constexpr int MP = NP <= 16 ? 16 : 32;
  typedef Tile<MP> T;
  constexpr int STEPS = T::STEPS;  // = elements of the padded MP x MP tile per lane
  __shared__ float aug[NP * AUGS];
  __shared__ float trs[TRB][FOLX_WAVE + 1];

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

  // this lane's elements (k, lr) of the padded tile: A^-1 transposed-in-place as the MFMA
  // operand, and with a factor also F, A and the factor's sparse Jacobian rows at them
  const int lr = lane % MP;
  const int lq = lane / MP;
  float ainv[STEPS];
  bool ok[STEPS];
  int64_t eoff[STEPS];
#pragma unroll
  for (int t = 0; t < STEPS; ++t) {
    const int k = T::KS * t + lq;
    ok[t] = k < n && lr < n;
    // elements of the padding ask for element (0, 0): loads are never branched around, so
    // that all of them are in flight before the first wait
    eoff[t] = ok[t] ? (int64_t)k * rstride + lr : 0;
    ainv[t] = ok[t] ? aug[lr * AUGS + NP + k] : 0.0f;  // Ainv[lr][k]
  }
  constexpr int EF = HAS_F ? STEPS : 1;
  float fx[EF], ax[EF], lapx[EF], fj[KFT][EF];
  int32_t fidx[KFT][EF];
  if constexpr (HAS_F) {
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      const int64_t off = base + eoff[t];
      fx[t] = fc.x[off];
      ax[t] = A[off];
      lapx[t] = 0.0f;
#pragma unroll
      for (int sl = 0; sl < KFT; ++sl) {
        fidx[sl][t] = -1;
        fj[sl][t] = 0.0f;
        if (sl < fc.kf) {  // the same for all lanes
          fidx[sl][t] = fc.idx[(int64_t)sl * fc.S_w + off % fc.S_w];
          fj[sl][t] = fc.jac[(int64_t)sl * slice + off];
        }
      }
    }
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      fx[t] = ok[t] ? fx[t] : 0.0f;
      ax[t] = ok[t] ? ax[t] : 0.0f;
#pragma unroll
      for (int sl = 0; sl < KFT; ++sl) {
        fidx[sl][t] = ok[t] ? fidx[sl][t] : -1;
        fj[sl][t] = fidx[sl][t] >= 0 ? fj[sl][t] : 0.0f;
      }
    }
  }

  // Jacobian rows are requested D rows ahead: with one row in flight per wavefront the kernel
  // would be bound by the latency of its own loads, not by HBM bandwidth.
  constexpr int D = MP == 16 ? ((HAS_F && KFT < KF) ? 6 : 4) : 1;
  float mm = 0.0f;
  float raw[D][STEPS];
  auto request = [&](float (&dst)[STEPS], int p) __attribute__((always_inline)) {
    const float* src = AJ + (int64_t)p * slice + base;
#pragma unroll
    for (int t = 0; t < STEPS; ++t) dst[t] = src[eoff[t]];  // A_jac[p][k][lr], padding masked when used
  };
#pragma unroll
  for (int d = 0; d < D; ++d)
    if (d < P) request(raw[d], d);
  for (int p0 = 0; p0 < P; p0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int p = p0 + d;
      if (p < P) {
        float jv[STEPS];
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
          float v = ok[t] ? raw[d][t] : 0.0f;
          if constexpr (HAS_F) {
            float add = 0.0f;
#pragma unroll
            for (int sl = 0; sl < KFT; ++sl) add += fidx[sl][t] == p ? fj[sl][t] : 0.0f;
            lapx[t] = fmaf(2.0f * v, add, lapx[t]);  // cross term 2 dA . dF of the product's Laplacian
            v = fx[t] * v + ax[t] * add;
          }
          jv[t] = v;
        }
        if (p + D < P) request(raw[d], p + D);
        typename T::acc_t c, ct;
#pragma unroll
        for (int r = 0; r < T::CR; ++r) { c[r] = 0.0f; ct[r] = 0.0f; }
        float tr = 0.0f;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
          c = T::mfma(ainv[t], jv[t], c);    // M   = Ainv J
          ct = T::mfma(jv[t], ainv[t], ct);  // M^T
          tr = fmaf(ainv[t], jv[t], tr);     // this lane's part of tr M
        }
#pragma unroll
        for (int r = 0; r < T::CR; ++r) mm = fmaf(c[r], ct[r], mm);
        trs[p % TRB][lane] = tr;
        if ((p + 1) % TRB == 0 || p + 1 == P) {
          // ld_jac of the last rows: four lanes per row add up 16 of its 64 parts each
          // The workgroup is one wavefront and LDS serves a wavefront's accesses in issue
          // order, so the other lanes' writes above are seen without a barrier; a barrier's
          // fence would also wait for the Jacobian rows requested ahead.
          const int pb = p / TRB * TRB, pe = p + 1 - pb;
          asm volatile("" ::: "memory");
          const int row = lane % TRB, part = lane / TRB;
          float sm = 0.0f;
#pragma unroll
          for (int l = 0; l < FOLX_WAVE / 4; ++l) sm += trs[row][part * (FOLX_WAVE / 4) + l];
          sm += __shfl_xor(sm, 16, FOLX_WAVE);
          sm += __shfl_xor(sm, 32, FOLX_WAVE);
          if (part == 0 && row < pe) jac_out[(int64_t)(pb + row) * NM + m] = sm;
          asm volatile("" ::: "memory");
        }
      }
    }
  }
  if constexpr (HAS_F) {
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      // fx, ax, lapx and ainv are zero at the padding
      const int64_t off = base + eoff[t];
      const float al = fx[t] * AL[off] + ax[t] * fc.lap[off] + lapx[t];
      tl += ainv[t] * al;  // tr(A^-1 lap A) = sum A^-1[lr][k] lap A[k][lr]
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
#define FOLX_SLD_LAUNCH(NPV, HASF, KFV)                                                                   \
  slogdet_kernel<NPV, HASF, KFV><<<grid, block, 0, st>>>(A, A_jac, A_lap, sign, logdet, ld_jac, ld_lap, NM, n, P, \
                                                         ND, batch_stride, member_stride, row_stride, jac_stride, \
                                                         share, fc ? *fc : Factor{})
  if (fc) {
    // three slots (the coordinates of one electron) leave registers for two more rows in flight
    const bool three = fc->kf <= 3;
    if (n <= 8) { if (three) FOLX_SLD_LAUNCH(8, true, 3); else FOLX_SLD_LAUNCH(8, true, KF); }
    else { if (three) FOLX_SLD_LAUNCH(16, true, 3); else FOLX_SLD_LAUNCH(16, true, KF); }
  } else {
    if (n <= 8) FOLX_SLD_LAUNCH(8, false, KF);
    else if (n <= 16) FOLX_SLD_LAUNCH(16, false, KF);
    else FOLX_SLD_LAUNCH(32, false, KF);
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
