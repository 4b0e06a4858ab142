// Dense-layer rule: y = h @ W (+ bias) over the stacked operand [x; J; lap].
//
// All (P + 2) * R rows go through ONE launch of an LDS-tiled FP32-MFMA GEMM
// (v_mfma_f32_32x32x2_f32).  The three operands are separate allocations, so the row
// tiles are laid out per segment (x, jac, lap) and never straddle two of them.
//
// Tiling: a workgroup of 4 wavefronts owns BM = 128 rows x BN columns and walks K in
// chunks of BK = 32 through double-buffered LDS tiles (global -> registers -> LDS, one
// barrier per chunk).  A rows are stored [row][k] with a stride of 36 floats: a lane
// fetches 4 consecutive k with one 128-bit LDS read, and the rows of 8 consecutive lanes
// fall into distinct bank groups.  The MFMA only needs A and B to agree on which k a
// lane holds, so the k order inside a chunk is permuted to fit that read:
//     lane l, register j of group t  <->  k = 8 t + 4 (l / 32) + j.
// W rows are stored [k][n], read with consecutive n across lanes.
//
// Workgroup ids are remapped so that the column tiles of one row tile run back to back
// on the same XCD (ids are dealt round-robin to the 8 XCDs), which keeps the second
// read of an A tile in that XCD's L2.
#include "common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128;
constexpr int BK = 32;
constexpr int AS = BK + 4;  // LDS row stride of the A tile (floats)
constexpr int NXCD = 8;

struct Segs {
  const float* in[3];
  float* out[3];
  int64_t rows[3];
  int64_t tiles[3];
};

template <int BN, int WM, int WN>
__global__ __launch_bounds__(256) void dense_kernel(Segs sg, const float* __restrict__ W,
                                                    const float* __restrict__ bias, int32_t K,
                                                    int32_t N, int64_t row_tiles, int32_t col_tiles,
                                                    int vecA, int vecW) {
  constexpr int WROWS = BM / WM;  // rows per wavefront
  constexpr int WCOLS = BN / WN;  // columns per wavefront
  constexpr int TM = WROWS / 32;
  constexpr int TN = WCOLS / 32;
  static_assert(WM * WN == 4, "4 wavefronts");

  __shared__ __attribute__((aligned(16))) float As[2][BM * AS];
  __shared__ __attribute__((aligned(16))) float Ws[2][BK * BN];

  // XCD-aware id -> (row tile, column tile)
  const int64_t id = blockIdx.x;
  const int64_t xcd = id % NXCD;
  const int64_t slot = id / NXCD;
  const int64_t rt = (slot / col_tiles) * NXCD + xcd;
  const int32_t ct = (int32_t)(slot % col_tiles);
  if (rt >= row_tiles) return;

  int seg = 0;
  int64_t t = rt;
  if (t >= sg.tiles[0]) { t -= sg.tiles[0]; seg = 1; if (t >= sg.tiles[1]) { t -= sg.tiles[1]; seg = 2; } }
  const float* __restrict__ A = sg.in[seg];
  float* __restrict__ C = sg.out[seg];
  const int64_t rows = sg.rows[seg];
  const int64_t row0 = t * BM;
  const int32_t col0 = ct * BN;

  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = tid / 64;
  const int wr = (wave / WN) * WROWS;
  const int wc = (wave % WN) * WCOLS;
  const int l32 = lane % 32;
  const int lh = lane / 32;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  constexpr int A_LD = BM * BK / 4 / 256;  // float4 loads per thread for the A tile
  constexpr int W_LD = BK * BN / 4 / 256;  // float4 loads per thread for the W tile
  float4 ra[A_LD];
  float4 rw[W_LD];

  auto load_global = [&](int kt) {
    const int k0 = kt * BK;
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
      const int idx = tid + 256 * i;
      const int r = idx / (BK / 4);
      const int kq = (idx % (BK / 4)) * 4;
      const int64_t gr = row0 + r;
      const int gk = k0 + kq;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (gr < rows) {
        const float* src = A + gr * (int64_t)K + gk;
        if (vecA && gk + 3 < K) {
          v = *reinterpret_cast<const float4*>(src);
        } else {
          if (gk + 0 < K) v.x = src[0];
          if (gk + 1 < K) v.y = src[1];
          if (gk + 2 < K) v.z = src[2];
          if (gk + 3 < K) v.w = src[3];
        }
      }
      ra[i] = v;
    }
#pragma unroll
    for (int i = 0; i < W_LD; ++i) {
      const int idx = tid + 256 * i;
      const int kk = idx / (BN / 4);
      const int nq = (idx % (BN / 4)) * 4;
      const int gk = k0 + kk;
      const int gn = col0 + nq;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (gk < K) {
        const float* src = W + (int64_t)gk * N + gn;
        if (vecW && gn + 3 < N) {
          v = *reinterpret_cast<const float4*>(src);
        } else {
          if (gn + 0 < N) v.x = src[0];
          if (gn + 1 < N) v.y = src[1];
          if (gn + 2 < N) v.z = src[2];
          if (gn + 3 < N) v.w = src[3];
        }
      }
      rw[i] = v;
    }
  };

  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
      const int idx = tid + 256 * i;
      const int r = idx / (BK / 4);
      const int kq = (idx % (BK / 4)) * 4;
      *reinterpret_cast<float4*>(&As[buf][r * AS + kq]) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < W_LD; ++i) {
      const int idx = tid + 256 * i;
      const int kk = idx / (BN / 4);
      const int nq = (idx % (BN / 4)) * 4;
      *reinterpret_cast<float4*>(&Ws[buf][kk * BN + nq]) = rw[i];
    }
  };

  const int KT = (K + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) load_global(kt + 1);

#pragma unroll
    for (int tg = 0; tg < BK / 8; ++tg) {
      float4 a4[TM];
      float b[TN][4];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        a4[i] = *reinterpret_cast<const float4*>(&As[buf][(wr + i * 32 + l32) * AS + tg * 8 + lh * 4]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) b[j][q] = Ws[buf][(tg * 8 + lh * 4 + q) * BN + wc + j * 32 + l32];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const float av = q == 0 ? a4[i].x : (q == 1 ? a4[i].y : (q == 2 ? a4[i].z : a4[i].w));
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, b[j][q], acc[i][j], 0, 0, 0);
        }
      }
    }

    if (kt + 1 < KT) store_lds(buf ^ 1);
    __syncthreads();
  }

  // Epilogue: register r of a 32x32 tile holds row 8 (r / 4) + 4 (lane / 32) + r % 4,
  // column lane % 32, so each store instruction writes two 128-byte row segments.
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int gc = col0 + wc + j * 32 + l32;
      if (gc < N) {
        const float bv = (seg == 0 && bias != nullptr) ? bias[gc] : 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t gr = row0 + wr + i * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
          if (gr < rows) C[gr * (int64_t)N + gc] = acc[i][j][r] + bv;
        }
      }
    }
  }
}

}  // namespace

extern "C" int folx_hip_dense_fwdlap(void* stream, const float* x, const float* jac,
                                     const float* lap, const float* W, const float* bias,
                                     float* y, float* y_jac, float* y_lap, int64_t R, int32_t P,
                                     int32_t K, int32_t N) {
  if (R < 0 || P < 0 || K <= 0 || N <= 0) return FOLX_HIP_EINVAL;
  if (R == 0) return FOLX_HIP_OK;
  if (!x || !lap || !W || !y || !y_lap || (P > 0 && (!jac || !y_jac))) return FOLX_HIP_EINVAL;
  Segs sg;
  sg.in[0] = x; sg.in[1] = jac; sg.in[2] = lap;
  sg.out[0] = y; sg.out[1] = y_jac; sg.out[2] = y_lap;
  sg.rows[0] = R; sg.rows[1] = (int64_t)P * R; sg.rows[2] = R;
  int64_t row_tiles = 0;
  for (int s = 0; s < 3; ++s) { sg.tiles[s] = (sg.rows[s] + BM - 1) / BM; row_tiles += sg.tiles[s]; }
  const int vecA = (K % 4 == 0) && folx_aligned16(x) && folx_aligned16(jac) && folx_aligned16(lap);
  const int vecW = (N % 4 == 0) && folx_aligned16(W);
  const int BN = N > 64 ? 128 : (N > 32 ? 64 : 32);
  const int32_t col_tiles = (N + BN - 1) / BN;
  const int64_t groups = (row_tiles + NXCD - 1) / NXCD;
  const int64_t blocks = groups * NXCD * col_tiles;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)blocks), block(256);
  if (BN == 128)
    dense_kernel<128, 2, 2><<<grid, block, 0, st>>>(sg, W, bias, K, N, row_tiles, col_tiles, vecA, vecW);
  else if (BN == 64)
    dense_kernel<64, 4, 1><<<grid, block, 0, st>>>(sg, W, bias, K, N, row_tiles, col_tiles, vecA, vecW);
  else
    dense_kernel<32, 4, 1><<<grid, block, 0, st>>>(sg, W, bias, K, N, row_tiles, col_tiles, vecA, vecW);
  return folx_launch_status();
}
