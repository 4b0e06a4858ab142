// Wide dense layer and its activation without the pass over the pre-activation Jacobian:
//   z = x @ W + bias          y     = f(z)
//   zj[p] = jac[p] @ W        yj[p] = f'(z) * zj[p]
//   zl = lap @ W              yl    = f'(z) * zl + f''(z) * sum_p zj[p]^2
// for N > 128 and K a multiple of 16 (the narrow layers have their own kernel).  The Jacobian
// rows are (P * R) x K with R positions; an activation kernel after the GEMM would read and
// write all of zj once more, here zj never reaches HBM.
//
// Three launches on the caller's stream:
//  1. the plain dense kernel on the x and lap rows only (2 R of the (P + 2) R rows): z goes to
//     y, zl to y_lap;
//  2. the Jacobian GEMM below, whose 128-row tiles are cut ACROSS Jacobian rows: a tile holds
//     4 consecutive positions x 32 consecutive p, ordered position-major, so that each 32 x 32
//     accumulator block belongs to ONE position.  f'(z) of a block is then one value per lane
//     (its column), the block is scaled by it on the way out, and the squares of the block sum
//     to one value per column inside the wavefront (16 registers and the two lane halves).
//     These sums go to the workspace, one (R, N) slab per group of 32 Jacobian rows;
//  3. a short elementwise kernel that turns z into f(z) and zl into the lap row, adding the
//     slabs in a fixed order.
//
// The main loop is the one of the dense kernel: K in chunks of 16 through double-buffered LDS
// tiles filled by global_load_lds_dwordx4, a 128 x 256 tile on 8 wavefronts of 64 x 64,
// v_mfma_f32_32x32x2_f32 with the k order inside a group of 8 permuted to fit 128-bit reads
// (lane l, register j of group t <-> k = 8 t + 4 (l / 32) + j), piece c of an A row stored at
// slot c ^ ((row / 2) % 4).  Only the address a lane asks for differs: tile row m is
// Jacobian row p0 + m % 32 of position r0 + m / 32.
#include "activations.h"
#include "dense_act_wide.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

#define FOLX_GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define FOLX_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

constexpr int BK = 16;
constexpr int BM = 128, BN = 256, WM = 2, WN = 4;
constexpr int NT = 64 * WM * WN;
constexpr int WROWS = BM / WM, WCOLS = BN / WN;
constexpr int TM = WROWS / 32, TN = WCOLS / 32;
constexpr int TG = BK / 8;
constexpr int NXCD = 8;
constexpr int PT = 32;       // Jacobian rows of a tile
constexpr int RT = BM / PT;  // positions of a tile
constexpr int A_V4 = BM * BK / 4, W_V4 = BK * BN / 4;
constexpr int A_LD = A_V4 / NT, W_LD = W_V4 / NT;
static_assert(A_V4 % NT == 0 && W_V4 % NT == 0, "every thread loads the same number of pieces");
static_assert(TM * WM == RT, "one accumulator block row per position");

struct WideParams {
  const float* jac;
  const float* W;
  const float* z;  // pre-activation values (R, N), bias included
  float* y_jac;
  float* part;     // (PG, R, N) sums of squares per group of PT Jacobian rows
  int64_t R, row_tiles, pos_tiles;
  int32_t P, K, N, col_tiles, act;
  float prm;
};

__global__ __launch_bounds__(NT, 4) void dense_act_wide_kernel(WideParams a) {
  __shared__ __attribute__((aligned(16))) float As0[BM * BK];
  __shared__ __attribute__((aligned(16))) float As1[BM * BK];
  __shared__ __attribute__((aligned(16))) float Ws0[BK * BN];
  __shared__ __attribute__((aligned(16))) float Ws1[BK * BN];

  // ids are dealt round-robin to the XCDs: the column tiles of a row tile stay on one of them
  const int64_t id = blockIdx.x;
  const int64_t xcd = id % NXCD;
  const int64_t slot = id / NXCD;
  const int64_t rt = (slot / a.col_tiles) * NXCD + xcd;
  const int32_t ct = (int32_t)(slot % a.col_tiles);
  if (rt >= a.row_tiles) return;
  const int32_t pg = (int32_t)(rt / a.pos_tiles);
  const int64_t r0 = (rt % a.pos_tiles) * RT;
  const int32_t p0 = pg * PT;
  const int32_t col0 = ct * BN;
  const int32_t K = a.K, N = a.N, P = a.P;
  const int64_t R = a.R;

  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wrow = wave / WN;
  const int wr = wrow * WROWS;
  const int wc = (wave % WN) * WCOLS;
  const int l32 = lane % 32;
  const int lh = lane / 32;

  const float* a_p[A_LD];
  const float* w_p[W_LD];
#pragma unroll
  for (int i = 0; i < A_LD; ++i) {
    const int idx = tid + NT * i;
    const int m = idx / 4, c = idx % 4;
    const int kc = c ^ ((m / 2) % 4);
    int p = p0 + m % PT;
    if (p >= P) p = P - 1;  // reaches accumulator rows that are neither stored nor summed
    a_p[i] = a.jac + ((int64_t)p * R + r0 + m / PT) * K + kc * 4;
  }
#pragma unroll
  for (int i = 0; i < W_LD; ++i) {
    const int idx = tid + NT * i;
    const int k = (idx / (BN / 4)) % BK;
    int n = col0 + (idx % (BN / 4)) * 4;
    if (n > N - 4) n = N - 4;
    w_p[i] = a.W + (int64_t)k * N + n;
  }
  auto issue = [&](int kt, float* as, float* ws) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < A_LD; ++i)
      __builtin_amdgcn_global_load_lds(FOLX_GPTR(a_p[i] + kt * BK), FOLX_LPTR(&as[(wave * 64 + NT * i) * 4]), 16, 0,
                                       0);
#pragma unroll
    for (int i = 0; i < W_LD; ++i)
      __builtin_amdgcn_global_load_lds(FOLX_GPTR(w_p[i] + (int64_t)kt * BK * N),
                                       FOLX_LPTR(&ws[(wave * 64 + NT * i) * 4]), 16, 0, 0);
  };

  // pre-activation value of this lane's column at the position of each accumulator block
  float zv[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      int gc = col0 + wc + j * 32 + l32;
      if (gc >= N) gc = N - 1;
      zv[i][j] = a.z[(r0 + wrow * TM + i) * N + gc];
    }

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int sw = (l32 / 2) % 4;
  auto compute = [&](const float* as, const float* ws) __attribute__((always_inline)) {
#pragma unroll
    for (int tg = 0; tg < TG; ++tg) {
      float4 a4[TM];
      float b[TN][4];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        a4[i] = *reinterpret_cast<const float4*>(&as[(wr + i * 32 + l32) * BK + (((tg * 2 + lh) ^ sw) * 4)]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) b[j][q] = ws[(tg * 8 + lh * 4 + q) * BN + wc + j * 32 + l32];
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
  };

  // The loads of a chunk are waited for at the end of the chunk before it; the barrier then
  // also says that every wavefront is done reading the buffer that is refilled next.
  const int KT = K / BK;
  issue(0, As0, Ws0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  for (int kt = 0; kt < KT; kt += 2) {
    if (kt + 1 < KT) issue(kt + 1, As1, Ws1);
    compute(As0, Ws0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (kt + 1 < KT) {
      if (kt + 2 < KT) issue(kt + 2, As0, Ws0);
      compute(As1, Ws1);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }
  }

  // Register r of a block is Jacobian row p0 + 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32.
  const int64_t pstride = R * N;  // floats between consecutive Jacobian rows
  const bool full_tile = (p0 + PT <= P) && (col0 + BN <= N);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int64_t pos = r0 + wrow * TM + i;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      float f, d1, d2;
      act_eval_fused(a.act, zv[i][j], a.prm, f, d1, d2);
      const int gc = col0 + wc + j * 32 + l32;
      float* out = a.y_jac + ((int64_t)(p0 + 4 * lh) * R + pos) * N + gc;
      float ss = 0.0f;
      if (full_tile) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float v = acc[i][j][r];
          ss = fmaf(v, v, ss);
          __builtin_nontemporal_store(d1 * v, out + (int64_t)(8 * (r / 4) + r % 4) * pstride);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int pl = 8 * (r / 4) + r % 4;
          if (p0 + 4 * lh + pl < P) {
            const float v = acc[i][j][r];
            ss = fmaf(v, v, ss);
            if (gc < N) out[(int64_t)pl * pstride] = d1 * v;
          }
        }
      }
      ss += __shfl_xor(ss, 32, FOLX_WAVE);
      if (lh == 0 && gc < N) a.part[((int64_t)pg * R + pos) * N + gc] = ss;
    }
  }
}

// y <- f(z), y_lap <- f'(z) zl + f''(z) sum_g part[g]; z and zl are what the first launch left
// in y and y_lap.  One float4 per thread.
__global__ __launch_bounds__(256) void dense_act_wide_finish(float* __restrict__ y, float* __restrict__ y_lap,
                                                             const float* __restrict__ part, int64_t S4,
                                                             int32_t PG, int32_t act, float prm) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= S4) return;
  const float4 z = reinterpret_cast<const float4*>(y)[i];
  const float4 zl = reinterpret_cast<const float4*>(y_lap)[i];
  float4 s = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  for (int g = 0; g < PG; ++g) {
    const float4 t = reinterpret_cast<const float4*>(part)[(int64_t)g * S4 + i];
    s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
  }
  float4 f, l;
  float d1, d2;
  act_eval_fused(act, z.x, prm, f.x, d1, d2); l.x = fmaf(d1, zl.x, d2 * s.x);
  act_eval_fused(act, z.y, prm, f.y, d1, d2); l.y = fmaf(d1, zl.y, d2 * s.y);
  act_eval_fused(act, z.z, prm, f.z, d1, d2); l.z = fmaf(d1, zl.z, d2 * s.z);
  act_eval_fused(act, z.w, prm, f.w, d1, d2); l.w = fmaf(d1, zl.w, d2 * s.w);
  reinterpret_cast<float4*>(y)[i] = f;
  reinterpret_cast<float4*>(y_lap)[i] = l;
}

struct WidePlan {
  int64_t row_tiles, pos_tiles, blocks, ws_bytes;
  int32_t PG, col_tiles;
};

bool plan_wide(int64_t R, int32_t P, int32_t K, int32_t N, WidePlan& pl) {
  if (R <= 0 || R % RT != 0 || P < 1 || K < BK || K % BK != 0 || N <= 128 || N % 4 != 0) return false;
  pl.PG = (P + PT - 1) / PT;
  pl.pos_tiles = R / RT;
  pl.row_tiles = pl.pos_tiles * pl.PG;
  pl.col_tiles = (N + BN - 1) / BN;
  pl.blocks = (pl.row_tiles + NXCD - 1) / NXCD * NXCD * pl.col_tiles;
  if (pl.blocks > 0x7fffffffLL) return false;
  if (R * (int64_t)N / 4 + 255 > 0x7fffffffLL * 256) return false;
  pl.ws_bytes = (int64_t)pl.PG * R * N * 4;
  return true;
}

}  // namespace

int64_t folx_dense_act_wide_ws_bytes(int64_t R, int32_t P, int32_t K, int32_t N) {
  WidePlan pl;
  if (!plan_wide(R, P, K, N, pl)) return FOLX_HIP_ENOTSUP;
  return pl.ws_bytes;
}

int folx_dense_act_wide(hipStream_t st, int32_t act, float param, const float* x, const float* jac, const float* lap,
                        const float* W, const float* bias, float* y, float* y_jac, float* y_lap, int64_t R,
                        int32_t P, int32_t K, int32_t N, void* workspace, int64_t workspace_bytes) {
  WidePlan pl;
  if (!act_fused(act) || !plan_wide(R, P, K, N, pl)) return FOLX_HIP_ENOTSUP;
  if (!x || !jac || !lap || !W || !y || !y_jac || !y_lap) return FOLX_HIP_EINVAL;
  if (!folx_aligned16(jac) || !folx_aligned16(W) || !folx_aligned16(y) || !folx_aligned16(y_lap))
    return FOLX_HIP_ENOTSUP;
  if (!workspace || workspace_bytes < pl.ws_bytes || !folx_aligned16(workspace)) return FOLX_HIP_EINVAL;
  // z and zl through the plain dense kernel: no Jacobian rows, no residual
  int rc = folx_hip_dense_fwdlap(st, x, nullptr, lap, W, bias, nullptr, nullptr, nullptr, y, nullptr, y_lap, R, 0, K,
                                 N);
  if (rc != FOLX_HIP_OK) return rc;
  WideParams a;
  a.jac = jac; a.W = W; a.z = y; a.y_jac = y_jac; a.part = (float*)workspace;
  a.R = R; a.row_tiles = pl.row_tiles; a.pos_tiles = pl.pos_tiles;
  a.P = P; a.K = K; a.N = N; a.col_tiles = pl.col_tiles; a.act = act; a.prm = param;
  dense_act_wide_kernel<<<dim3((unsigned)pl.blocks), dim3(NT), 0, st>>>(a);
  rc = folx_launch_status();
  if (rc != FOLX_HIP_OK) return rc;
  const int64_t S4 = R * (int64_t)N / 4;
  dense_act_wide_finish<<<dim3((unsigned)((S4 + 255) / 256)), dim3(256), 0, st>>>(y, y_lap, (const float*)workspace,
                                                                                  S4, pl.PG, act, param);
  return folx_launch_status();
}
