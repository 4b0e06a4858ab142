// Determinant / inverse building blocks for matrices of ANY size.
//
// The slogdet, inverse and solve kernels keep one matrix per wavefront and stop at 32 x 32.
// Beyond that the rules are composed from the batched product kernels and the two kernels
// here (the reference reaches LAPACK through jnp.linalg for every size,
// folx/slogdet.py:296-344, folx/linear_solve.py:54-145):
//
//   inv_values_kernel   A^-1, sign and log|det A| of every matrix: in-place Gauss-Jordan with
//                       partial pivoting (row swaps; the pivot sequence is that of an LU
//                       factorisation with partial pivoting, so the sign is the same), one
//                       workgroup per matrix, the matrix in LDS while it fits and in the output
//                       buffer otherwise.
//   trace_pair_kernel   tr M and tr(M M) = sum_ij M_ij M_ji of every matrix of a stack: the two
//                       numbers the slogdet rule needs of M_c = A^-1 d_c A (folx/slogdet.py:313-316).
#include "common.h"

namespace {

constexpr int AS_NT = 256;
constexpr int AS_LDS_NMAX = 112;  // (n + 1) n + 3 n floats stay below 64 KB of LDS

template <bool IN_LDS>
__global__ __launch_bounds__(AS_NT) void inv_values_kernel(const float* __restrict__ A, float* Ainv,
                                                           float* __restrict__ sign, float* __restrict__ logdet,
                                                           int n) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  __shared__ float red_v[AS_NT];
  __shared__ int red_i[AS_NT];
  const int tid = threadIdx.x;
  const int ld = IN_LDS ? n + 1 : n;  // odd row stride in LDS: a column is read without bank conflicts
  float* W = IN_LDS ? sm : Ainv + (int64_t)blockIdx.x * n * n;
  float* rowk = IN_LDS ? sm + (int64_t)n * ld : sm;
  float* colk = rowk + n;
  int* ipiv = reinterpret_cast<int*>(colk + n);
  const float* Ab = A + (int64_t)blockIdx.x * n * n;
  const int nn = n * n;

  for (int e = tid; e < nn; e += AS_NT) W[(e / n) * ld + e % n] = Ab[e];
  __syncthreads();

  float sgn = 1.0f, ldet = 0.0f;
  bool singular = false;  // a zero (or non-finite) pivot: sign 0 and log|det| = -inf, as numpy.linalg.slogdet reports it
  for (int k = 0; k < n; ++k) {
    // pivot: the largest |W[i][k]|, i >= k, the first one among equals
    float best = -1.0f;
    int bi = k;
    for (int i = k + tid; i < n; i += AS_NT) {
      const float v = fabsf(W[i * ld + k]);
      if (v > best) { best = v; bi = i; }
    }
    red_v[tid] = best;
    red_i[tid] = bi;
    __syncthreads();
    for (int s = AS_NT / 2; s > 0; s >>= 1) {
      if (tid < s) {
        const float v = red_v[tid + s];
        const int i = red_i[tid + s];
        if (v > red_v[tid] || (v == red_v[tid] && i < red_i[tid])) { red_v[tid] = v; red_i[tid] = i; }
      }
      __syncthreads();
    }
    const int p = red_i[0];
    if (tid == 0) ipiv[k] = p;
    if (p != k)
      for (int j = tid; j < n; j += AS_NT) {
        const float a = W[k * ld + j], b = W[p * ld + j];
        W[k * ld + j] = b;
        W[p * ld + j] = a;
      }
    __syncthreads();
    const float piv = W[k * ld + k];  // row k and column k stay as they are until the barrier below
    const float pivinv = 1.0f / piv;
    for (int j = tid; j < n; j += AS_NT) rowk[j] = j == k ? pivinv : W[k * ld + j] * pivinv;
    for (int i = tid; i < n; i += AS_NT) colk[i] = W[i * ld + k];
    __syncthreads();
    for (int e = tid; e < nn; e += AS_NT) {
      const int i = e / n, j = e - i * n;
      if (i == k) {
        W[i * ld + j] = rowk[j];
      } else {
        const float w = j == k ? 0.0f : W[i * ld + j];
        W[i * ld + j] = w - colk[i] * rowk[j];
      }
    }
    __syncthreads();
    if (!(fabsf(piv) > 0.0f) || !(fabsf(piv) < INFINITY)) singular = true;
    sgn *= (piv < 0.0f) != (p != k) ? -1.0f : 1.0f;
    ldet += logf(fabsf(piv));
  }
  // the row swaps of the elimination are column swaps of the inverse, undone last to first
  for (int k = n - 1; k >= 0; --k) {
    const int p = ipiv[k];
    if (p != k) {
      for (int i = tid; i < n; i += AS_NT) {
        const float a = W[i * ld + k], b = W[i * ld + p];
        W[i * ld + k] = b;
        W[i * ld + p] = a;
      }
      __syncthreads();
    }
  }
  if (IN_LDS) {
    float* out = Ainv + (int64_t)blockIdx.x * nn;
    for (int e = tid; e < nn; e += AS_NT) out[e] = W[(e / n) * ld + e % n];
  }
  if (tid == 0) {
    sign[blockIdx.x] = singular ? 0.0f : sgn;
    logdet[blockIdx.x] = singular ? -INFINITY : ldet;
  }
}

__global__ __launch_bounds__(AS_NT) void trace_pair_kernel(const float* __restrict__ M, float* __restrict__ tr,
                                                           float* __restrict__ trsq, int n) {
  __shared__ float r0[AS_NT], r1[AS_NT];
  const int tid = threadIdx.x;
  const float* Mb = M + (int64_t)blockIdx.x * n * n;
  float t = 0.0f, q = 0.0f;
  for (int e = tid; e < n * n; e += AS_NT) {
    const int i = e / n, j = e - i * n;
    const float m = Mb[e];
    q += m * Mb[j * n + i];
    if (i == j) t += m;
  }
  r0[tid] = t;
  r1[tid] = q;
  __syncthreads();
  for (int s = AS_NT / 2; s > 0; s >>= 1) {
    if (tid < s) { r0[tid] += r0[tid + s]; r1[tid] += r1[tid + s]; }
    __syncthreads();
  }
  if (tid == 0) {
    tr[blockIdx.x] = r0[0];
    trsq[blockIdx.x] = r1[0];
  }
}

}  // namespace

extern "C" int folx_hip_inv_values(void* stream, const float* A, float* Ainv, float* sign, float* logdet,
                                   int64_t NM, int32_t n) {
  if (NM < 0 || n < 0) return FOLX_HIP_EINVAL;
  if (NM == 0) return FOLX_HIP_OK;
  if (!sign || !logdet || (n > 0 && (!A || !Ainv))) return FOLX_HIP_EINVAL;
  if (NM > 0x7fffffffLL || n > 16384) return FOLX_HIP_ENOTSUP;
  if (A == Ainv) return FOLX_HIP_EINVAL;  // the elimination runs in the output buffer
  hipStream_t st = (hipStream_t)stream;
  if (n <= AS_LDS_NMAX) {
    const size_t lds = sizeof(float) * ((size_t)n * (n + 1) + 3 * (size_t)n);
    inv_values_kernel<true><<<dim3((unsigned)NM), dim3(AS_NT), lds, st>>>(A, Ainv, sign, logdet, n);
  } else {
    const size_t lds = sizeof(float) * 3 * (size_t)n;
    inv_values_kernel<false><<<dim3((unsigned)NM), dim3(AS_NT), lds, st>>>(A, Ainv, sign, logdet, n);
  }
  return folx_launch_status();
}

extern "C" int folx_hip_trace_pair(void* stream, const float* M, float* tr, float* trsq, int64_t R, int32_t n) {
  if (R < 0 || n < 0) return FOLX_HIP_EINVAL;
  if (R == 0) return FOLX_HIP_OK;
  if (!tr || !trsq || (n > 0 && !M)) return FOLX_HIP_EINVAL;
  if (R > 0x7fffffffLL || n > 16384) return FOLX_HIP_ENOTSUP;
  trace_pair_kernel<<<dim3((unsigned)R), dim3(AS_NT), 0, (hipStream_t)stream>>>(M, tr, trsq, n);
  return folx_launch_status();
}
