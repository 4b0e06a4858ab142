// Inverse and linear-solve rules for many small matrices with dense Jacobians.
//
// One wavefront owns one n x n matrix (n <= 32, padded to NP in {8, 16, 32}); A^-1 = C
// comes from Gauss-Jordan with partial pivoting in LDS and is shared by the value, every
// Jacobian row and the Laplacian.  Each Jacobian row is read from HBM exactly once (the
// next row is prefetched into registers while the current one is being multiplied) and
// each output row is written once, through an LDS tile so that the stores are contiguous.
//
//   inverse:  M_p = C dA_p,   dC_p = -M_p C,   lap C = (2 sum_p M_p M_p - C lap_A) C
//   solve:    y = C b,   dy_p = C (db_p - dA_p y),
//             lap y = C (lap_b - lap_A y - 2 sum_p dA_p dy_p)
#include "smallmat.h"

namespace {

// out[i][c] (+)= sum_j L[i * ls + j] * R[j * rs + c] for the elements this lane owns:
// element e = lane + q * 64 of a row-major NP x MP tile.
template <int NP, int MP>
struct Tile {
  static constexpr int total = NP * MP;
  static constexpr int EO = (total + FOLX_WAVE - 1) / FOLX_WAVE;

  // 64 % MP == 0, so all elements of a lane share their column c = lane % MP: one read of
  // R[j][c] serves every owned row.
  __device__ static __forceinline__ void mm(float (&out)[EO], const float* L, int ls, const float* R, int rs,
                                             int lane, float scale) {
    static_assert(FOLX_WAVE % MP == 0, "column of a lane must not depend on q");
    if (total % FOLX_WAVE != 0 && lane >= total) return;
    const int c = lane % MP;
    const int i0 = lane / MP;
    constexpr int RSTEP = FOLX_WAVE / MP;  // row distance between consecutive owned elements
    float acc[EO];
#pragma unroll
    for (int q = 0; q < EO; ++q) acc[q] = 0.0f;
#pragma unroll 8
    for (int j = 0; j < NP; ++j) {
      const float r = R[j * rs + c];
#pragma unroll
      for (int q = 0; q < EO; ++q) acc[q] += L[(i0 + q * RSTEP) * ls + j] * r;
    }
#pragma unroll
    for (int q = 0; q < EO; ++q) out[q] += scale * acc[q];
  }

  __device__ static __forceinline__ void zero(float (&v)[EO]) {
#pragma unroll
    for (int q = 0; q < EO; ++q) v[q] = 0.0f;
  }

  // global (rows x cols, row-major, unpadded) -> registers, zero padded
  __device__ static __forceinline__ void load(float (&v)[EO], const float* __restrict__ src, int rows, int cols,
                                               int lane) {
#pragma unroll
    for (int q = 0; q < EO; ++q) {
      const int e = lane + q * FOLX_WAVE;
      const int i = e / MP, c = e % MP;
      v[q] = (src != nullptr && e < total && i < rows && c < cols) ? src[i * cols + c] : 0.0f;
    }
  }

  __device__ static __forceinline__ void to_lds(float* dst, int stride, const float (&v)[EO], int lane) {
#pragma unroll
    for (int q = 0; q < EO; ++q) {
      const int e = lane + q * FOLX_WAVE;
      if (total % FOLX_WAVE != 0 && e >= total) continue;
      dst[(e / MP) * stride + e % MP] = v[q];
    }
  }

  __device__ static __forceinline__ void store(float* __restrict__ dst, const float (&v)[EO], int rows, int cols,
                                                int lane) {
#pragma unroll
    for (int q = 0; q < EO; ++q) {
      const int e = lane + q * FOLX_WAVE;
      const int i = e / MP, c = e % MP;
      if (e < total && i < rows && c < cols) dst[i * cols + c] = v[q];
    }
  }
};

template <int NP>
__global__ __launch_bounds__(FOLX_WAVE) void inv_kernel(
    const float* __restrict__ A, const float* __restrict__ AJ, const float* __restrict__ AL,
    float* __restrict__ C_out, float* __restrict__ CJ_out, float* __restrict__ CL_out, int64_t NM, int32_t n,
    int32_t P) {
  using T = Tile<NP, NP>;
  constexpr int AUGS = smallmat::Aug<NP>::stride;
  constexpr int S = NP + 1;
  __shared__ float aug[NP * AUGS];
  __shared__ float jb[NP * S];  // dA_p, later lap_A
  __shared__ float mb[NP * S];  // M_p
  const int lane = threadIdx.x;
  const int64_t m = blockIdx.x;
  const int64_t nn = (int64_t)n * n;
  float logdet, sgn;
  smallmat::gauss_jordan<NP>(aug, A + m * nn, n, lane, logdet, sgn);
  const float* Cm = aug + NP;  // C[i][j] = Cm[i * AUGS + j]

  float v[T::EO], pre[T::EO], sacc[T::EO];
#pragma unroll
  for (int q = 0; q < T::EO; ++q) {
    const int e = lane + q * FOLX_WAVE;
    v[q] = Cm[(e / NP) * AUGS + e % NP];
  }
  T::store(C_out + m * nn, v, n, n, lane);

  T::zero(sacc);
  if (P > 0) T::load(pre, AJ + m * nn, n, n, lane);
  for (int p = 0; p < P; ++p) {
    T::to_lds(jb, S, pre, lane);
    __syncthreads();
    if (p + 1 < P) T::load(pre, AJ + ((int64_t)(p + 1) * NM + m) * nn, n, n, lane);
    T::zero(v);
    T::mm(v, Cm, AUGS, jb, S, lane, 1.0f);  // M = C dA
    T::to_lds(mb, S, v, lane);
    __syncthreads();
    T::mm(sacc, mb, S, mb, S, lane, 1.0f);  // sum M M
    T::zero(v);
    T::mm(v, mb, S, Cm, AUGS, lane, -1.0f);  // dC = -M C
    T::store(CJ_out + ((int64_t)p * NM + m) * nn, v, n, n, lane);
    // jb is rewritten at the top of the next iteration, after every lane has passed the
    // barrier above; mb after the barrier that follows that write
  }
  __syncthreads();
  T::load(pre, AL + m * nn, n, n, lane);
  T::to_lds(jb, S, pre, lane);
  __syncthreads();
  T::zero(v);
  T::mm(v, Cm, AUGS, jb, S, lane, -1.0f);  // -C lap_A
#pragma unroll
  for (int q = 0; q < T::EO; ++q) v[q] += 2.0f * sacc[q];
  __syncthreads();
  T::to_lds(mb, S, v, lane);
  __syncthreads();
  T::zero(v);
  T::mm(v, mb, S, Cm, AUGS, lane, 1.0f);
  T::store(CL_out + m * nn, v, n, n, lane);
}

// MP = 1 for a vector right-hand side, NP for up to NP columns.
template <int NP, int MP>
__global__ __launch_bounds__(FOLX_WAVE) void solve_kernel(
    const float* __restrict__ A, const float* __restrict__ AJ, const float* __restrict__ AL,
    const float* __restrict__ Bv, const float* __restrict__ BJ, const float* __restrict__ BL,
    float* __restrict__ Y, float* __restrict__ YJ, float* __restrict__ YL, int64_t NM, int32_t n, int32_t mc,
    int32_t P) {
  using TA = Tile<NP, NP>;
  using TB = Tile<NP, MP>;
  constexpr int AUGS = smallmat::Aug<NP>::stride;
  constexpr int S = NP + 1;
  constexpr int SB = MP + 1;
  __shared__ float aug[NP * AUGS];
  __shared__ float ja[NP * S];    // dA_p, later lap_A
  __shared__ float yb[NP * SB];   // y
  __shared__ float rb[NP * SB];   // right-hand side of the current solve
  __shared__ float yj[NP * SB];   // dy_p
  const int lane = threadIdx.x;
  const int64_t m = blockIdx.x;
  const int64_t nn = (int64_t)n * n;
  const int64_t nm = (int64_t)n * mc;
  float logdet, sgn;
  smallmat::gauss_jordan<NP>(aug, A + m * nn, n, lane, logdet, sgn);
  const float* Cm = aug + NP;
  // a variable operand always carries a Laplacian; its Jacobian pointer may be null when P = 0
  const bool a_var = AL != nullptr;
  const bool b_var = BL != nullptr;

  float rhs[TB::EO], out[TB::EO], tacc[TB::EO], preb[TB::EO], prea[TA::EO];
  // y = C b
  TB::load(rhs, Bv + m * nm, n, mc, lane);
  TB::to_lds(rb, SB, rhs, lane);
  __syncthreads();
  TB::zero(out);
  TB::mm(out, Cm, AUGS, rb, SB, lane, 1.0f);
  TB::store(Y + m * nm, out, n, mc, lane);
  TB::to_lds(yb, SB, out, lane);
  __syncthreads();

  TB::zero(tacc);
  TA::zero(prea);
  TB::zero(preb);
  if (P > 0) {
    if (a_var) TA::load(prea, AJ + m * nn, n, n, lane);
    if (b_var) TB::load(preb, BJ + m * nm, n, mc, lane);
  }
  for (int p = 0; p < P; ++p) {
    if (a_var) TA::to_lds(ja, S, prea, lane);
#pragma unroll
    for (int q = 0; q < TB::EO; ++q) rhs[q] = preb[q];
    __syncthreads();
    if (p + 1 < P) {
      if (a_var) TA::load(prea, AJ + ((int64_t)(p + 1) * NM + m) * nn, n, n, lane);
      if (b_var) TB::load(preb, BJ + ((int64_t)(p + 1) * NM + m) * nm, n, mc, lane);
    }
    if (a_var) TB::mm(rhs, ja, S, yb, SB, lane, -1.0f);  // db - dA y
    TB::to_lds(rb, SB, rhs, lane);
    __syncthreads();
    TB::zero(out);
    TB::mm(out, Cm, AUGS, rb, SB, lane, 1.0f);  // dy = C rhs
    TB::store(YJ + ((int64_t)p * NM + m) * nm, out, n, mc, lane);
    if (a_var) {
      TB::to_lds(yj, SB, out, lane);
      __syncthreads();
      TB::mm(tacc, ja, S, yj, SB, lane, 1.0f);  // sum dA dy
    }
    // ja, rb and yj are rewritten only after the first barrier of the next iteration
    __syncthreads();
  }
  // lap y = C (lap_b - lap_A y - 2 sum dA dy)
  TB::load(rhs, BL != nullptr ? BL + m * nm : nullptr, n, mc, lane);
  if (a_var) {
    TA::load(prea, AL + m * nn, n, n, lane);
    TA::to_lds(ja, S, prea, lane);
    __syncthreads();
    TB::mm(rhs, ja, S, yb, SB, lane, -1.0f);
#pragma unroll
    for (int q = 0; q < TB::EO; ++q) rhs[q] -= 2.0f * tacc[q];
  }
  TB::to_lds(rb, SB, rhs, lane);
  __syncthreads();
  TB::zero(out);
  TB::mm(out, Cm, AUGS, rb, SB, lane, 1.0f);
  TB::store(YL + m * nm, out, n, mc, lane);
}

}  // namespace

extern "C" int folx_hip_inv_fwdlap(void* stream, const float* A, const float* A_jac, const float* A_lap,
                                   float* C, float* C_jac, float* C_lap, int64_t NM, int32_t n, int32_t P) {
  if (NM < 0 || n <= 0 || P < 0) return FOLX_HIP_EINVAL;
  if (NM == 0) return FOLX_HIP_OK;
  if (!A || !A_lap || !C || !C_lap || (P > 0 && (!A_jac || !C_jac))) return FOLX_HIP_EINVAL;
  if (n > 32 || NM > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)NM), block(FOLX_WAVE);
  if (n <= 8) inv_kernel<8><<<grid, block, 0, st>>>(A, A_jac, A_lap, C, C_jac, C_lap, NM, n, P);
  else if (n <= 16) inv_kernel<16><<<grid, block, 0, st>>>(A, A_jac, A_lap, C, C_jac, C_lap, NM, n, P);
  else inv_kernel<32><<<grid, block, 0, st>>>(A, A_jac, A_lap, C, C_jac, C_lap, NM, n, P);
  return folx_launch_status();
}

extern "C" int folx_hip_solve_fwdlap(void* stream, const float* A, const float* A_jac, const float* A_lap,
                                     const float* b, const float* b_jac, const float* b_lap, float* y,
                                     float* y_jac, float* y_lap, int64_t NM, int32_t n, int32_t m, int32_t P) {
  if (NM < 0 || n <= 0 || m <= 0 || P < 0) return FOLX_HIP_EINVAL;
  if (NM == 0) return FOLX_HIP_OK;
  if (!A || !b || !y || !y_lap || (P > 0 && !y_jac)) return FOLX_HIP_EINVAL;
  // an operand is either constant (no Jacobian, no Laplacian) or carries both
  if (P > 0 && ((A_jac == nullptr) != (A_lap == nullptr))) return FOLX_HIP_EINVAL;
  if (P > 0 && ((b_jac == nullptr) != (b_lap == nullptr))) return FOLX_HIP_EINVAL;
  if (!A_lap && !b_lap) return FOLX_HIP_EINVAL;
  if (n > 32 || m > 32 || NM > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)NM), block(FOLX_WAVE);
#define FOLX_SOLVE_LAUNCH(NPV, MPV)                                                                         \
  solve_kernel<NPV, MPV><<<grid, block, 0, st>>>(A, A_jac, A_lap, b, b_jac, b_lap, y, y_jac, y_lap, NM, n, m, P)
  const int np = n <= 8 ? 8 : (n <= 16 ? 16 : 32);
  if (m == 1) {
    if (np == 8) FOLX_SOLVE_LAUNCH(8, 1);
    else if (np == 16) FOLX_SOLVE_LAUNCH(16, 1);
    else FOLX_SOLVE_LAUNCH(32, 1);
  } else {
    const int mp = m <= 8 ? 8 : (m <= 16 ? 16 : 32);
    const int t = np > mp ? np : mp;  // one padded size for both tile edges
    if (t == 8) FOLX_SOLVE_LAUNCH(8, 8);
    else if (t == 16) FOLX_SOLVE_LAUNCH(16, 16);
    else FOLX_SOLVE_LAUNCH(32, 32);
  }
#undef FOLX_SOLVE_LAUNCH
  return folx_launch_status();
}
