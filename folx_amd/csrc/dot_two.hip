// Matrix product of two operands that BOTH carry derivatives (attention scores q k^T, p v
// written with plain matmul / einsum):
//
//   y        = a b
//   y_jac[p] = a_jac[p] b + a b_jac[p]
//   y_lap    = a_lap b + a b_lap + 2 sum_p a_jac[p] b_jac[p]
//
// for a batch of small matrices, a (I x Kc), b (Kc x J), every operand addressed through element
// strides so that transposed and head-interleaved views ((walker, electron, head, feature)
// read as (walker, head, electron, feature)) are consumed where they lie.  The
// (batch, i, j, k) intermediate of the multiply-and-sum decomposition is never formed: per
// Jacobian row the kernel reads one (I x Kc) and one (Kc x J) tile and writes one (I x J) tile.
//
// One workgroup of four wavefronts per (batch element, 32 x 32 output tile); wavefront w owns
// the 16 x 16 block (w / 2, w % 2).  a and b tiles stay in LDS for the whole Jacobian loop, the
// row's a_jac[p] / b_jac[p] tiles are fetched into registers one row ahead and handed over
// through LDS; three v_mfma_f32_16x16x4_f32 chains per row (a_jac b, a b_jac into the row's
// accumulator, a_jac b_jac into the Laplacian's).  The Laplacian operands run through the same
// loop body as one more row (p = P) that is left out of the second-order sum.  Inside a group of
// 16 values of k the order is permuted (lane (l16, lg), step r <-> k = 4 lg + r), so the A
// operand is one 128-bit LDS read per four MFMAs.
#include <atomic>

#include "common.h"

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int DT_TILE = 32;    // output tile edge
constexpr int DT_NT = 256;     // threads per workgroup
constexpr int DT_KMAX = 128;   // contracted length the LDS tiles are sized for
constexpr int DT_BS = 48;      // row stride of the (k x 32) tiles: 16 mod 32, two k rows per half wavefront hit disjoint banks

struct DotTwoArgs {
  const float *a, *aj, *al, *b, *bj, *bl;
  float *y, *yj, *yl;
  // element strides: batch index = b0 * NB1 + b1
  int64_t a_sb0, a_sb1, a_si, a_sk, a_sp;
  int64_t b_sb0, b_sb1, b_sk, b_sj, b_sp;
  int64_t y_sp;  // elements between consecutive Jacobian rows of y_jac (= NB * I * J)
  int64_t NB;
  int32_t NB1, I, J, Kc, P, tiles_i, tiles_j;
};

// MAXLD = values per thread of one tile: 32 * Kp / 256 with Kp = Kc rounded up to 16
// CONSTB: b carries no derivatives (a constant with batch axes, e.g. per-head weights): the rule is
// linear in a, y_jac[p] = a_jac[p] b and y_lap = a_lap b, one product chain per row and no b rows.
template <int MAXLD, bool CONSTB>
__global__ __launch_bounds__(DT_NT) void dot_two_kernel(DotTwoArgs g) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int Kc = g.Kc;
  const int Kp = (Kc + 15) / 16 * 16;
  const int AS = Kp + 4;                      // row stride of the (32 x k) tiles
  float* As = sm;                             // a        [32][AS]
  float* AJs = As + DT_TILE * AS;             // a_jac[p] [32][AS]
  float* Bs = AJs + DT_TILE * AS;             // b        [Kp][DT_BS]
  float* BJs = Bs + Kp * DT_BS;               // b_jac[p] [Kp][DT_BS]

  const int tid = threadIdx.x;
  const int lane = tid % FOLX_WAVE, w = tid / FOLX_WAVE;
  const int l16 = lane % 16, lg = lane / 16;
  const int wi = w / 2, wj = w % 2;

  int64_t blk = blockIdx.x;
  const int tj = (int)(blk % g.tiles_j); blk /= g.tiles_j;
  const int ti = (int)(blk % g.tiles_i); blk /= g.tiles_i;
  const int64_t bt = blk;
  const int64_t b0 = bt / g.NB1, b1 = bt % g.NB1;
  const int i0 = ti * DT_TILE, j0 = tj * DT_TILE;
  const int64_t a_off = b0 * g.a_sb0 + b1 * g.a_sb1;
  const int64_t b_off = b0 * g.b_sb0 + b1 * g.b_sb1;
  const int nld = DT_TILE * Kp / DT_NT;       // values per thread and tile (Kp / 8)
  // the unit-stride axis of an operand is walked by consecutive threads
  const bool a_kfast = g.a_sk == 1 || g.a_si != 1;
  const bool b_jfast = g.b_sj == 1 || g.b_sk != 1;

  // element e of thread's r-th value -> (row, k) of the a-type tile, (k, col) of the b-type tile
  auto a_coord = [&](int r, int& i, int& k) {
    const int e = tid + DT_NT * r;
    if (a_kfast) { k = e % Kp; i = e / Kp; } else { i = e % DT_TILE; k = e / DT_TILE; }
  };
  auto b_coord = [&](int r, int& k, int& j) {
    const int e = tid + DT_NT * r;
    if (b_jfast) { j = e % DT_TILE; k = e / DT_TILE; } else { k = e % Kp; j = e / Kp; }
  };
  auto fetch_a = [&](const float* src, float (&reg)[MAXLD]) {
#pragma unroll
    for (int r = 0; r < MAXLD; ++r) {
      reg[r] = 0.0f;
      if (r < nld) {
        int i, k;
        a_coord(r, i, k);
        if (i0 + i < g.I && k < Kc) reg[r] = src[a_off + (int64_t)(i0 + i) * g.a_si + (int64_t)k * g.a_sk];
      }
    }
  };
  auto fetch_b = [&](const float* src, float (&reg)[MAXLD]) {
#pragma unroll
    for (int r = 0; r < MAXLD; ++r) {
      reg[r] = 0.0f;
      if (r < nld) {
        int k, j;
        b_coord(r, k, j);
        if (j0 + j < g.J && k < Kc) reg[r] = src[b_off + (int64_t)k * g.b_sk + (int64_t)(j0 + j) * g.b_sj];
      }
    }
  };
  auto put_a = [&](float* dst, const float (&reg)[MAXLD]) {
#pragma unroll
    for (int r = 0; r < MAXLD; ++r)
      if (r < nld) { int i, k; a_coord(r, i, k); dst[i * AS + k] = reg[r]; }
  };
  auto put_b = [&](float* dst, const float (&reg)[MAXLD]) {
#pragma unroll
    for (int r = 0; r < MAXLD; ++r)
      if (r < nld) { int k, j; b_coord(r, k, j); dst[k * DT_BS + j] = reg[r]; }
  };

  float ra[MAXLD], rb[MAXLD];
  fetch_a(g.a, ra);
  fetch_b(g.b, rb);
  put_a(As, ra);
  put_b(Bs, rb);
  // first row in flight: Jacobian row 0, or the Laplacian operands when there are no rows
  fetch_a(g.P > 0 ? g.aj : g.al, ra);
  if constexpr (!CONSTB) fetch_b(g.P > 0 ? g.bj : g.bl, rb);
  __syncthreads();

  // A operand of step (t, r): tile[16 wi + l16][16 t + 4 lg + r]; B operand: tile[16 t + 4 lg + r][16 wj + l16]
  const float* a_row = As + (16 * wi + l16) * AS + 4 * lg;
  const float* aj_row = AJs + (16 * wi + l16) * AS + 4 * lg;
  const float* b_col = Bs + (4 * lg) * DT_BS + 16 * wj + l16;
  const float* bj_col = BJs + (4 * lg) * DT_BS + 16 * wj + l16;
  const int kt = Kp / 16;

  const int orow = i0 + 16 * wi + 4 * lg, ocol = j0 + 16 * wj + l16;
  auto store_tile = [&](float* dst, const floatx4& c) {
    if (ocol < g.J) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (orow + r < g.I) dst[(bt * g.I + orow + r) * (int64_t)g.J + ocol] = c[r];
    }
  };

  {  // y = a b
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int t = 0; t < kt; ++t) {
      const float4 av = *reinterpret_cast<const float4*>(a_row + 16 * t);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.x, b_col[(16 * t + 0) * DT_BS], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.y, b_col[(16 * t + 1) * DT_BS], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.z, b_col[(16 * t + 2) * DT_BS], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.w, b_col[(16 * t + 3) * DT_BS], acc, 0, 0, 0);
    }
    store_tile(g.y, acc);
  }

  floatx4 lap2 = {0.f, 0.f, 0.f, 0.f};  // sum_p a_jac[p] b_jac[p]
  for (int p = 0; p <= g.P; ++p) {
    put_a(AJs, ra);
    if constexpr (!CONSTB) put_b(BJs, rb);
    __syncthreads();
    if (p < g.P) {  // next row: Jacobian row p + 1, or the Laplacian operands after the last one
      const bool last = p + 1 == g.P;
      fetch_a(last ? g.al : g.aj + (int64_t)(p + 1) * g.a_sp, ra);
      if constexpr (!CONSTB) fetch_b(last ? g.bl : g.bj + (int64_t)(p + 1) * g.b_sp, rb);
    }
    floatx4 acc = {0.f, 0.f, 0.f, 0.f}, cross = {0.f, 0.f, 0.f, 0.f};
    for (int t = 0; t < kt; ++t) {
      const float4 av = *reinterpret_cast<const float4*>(a_row + 16 * t);
      const float4 ajv = *reinterpret_cast<const float4*>(aj_row + 16 * t);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float bv = b_col[(16 * t + r) * DT_BS];
        const float ajr = r == 0 ? ajv.x : (r == 1 ? ajv.y : (r == 2 ? ajv.z : ajv.w));
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ajr, bv, acc, 0, 0, 0);
        if constexpr (!CONSTB) {
          const float bjv = bj_col[(16 * t + r) * DT_BS];
          const float ar = r == 0 ? av.x : (r == 1 ? av.y : (r == 2 ? av.z : av.w));
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ar, bjv, acc, 0, 0, 0);
          cross = __builtin_amdgcn_mfma_f32_16x16x4f32(ajr, bjv, cross, 0, 0, 0);
        }
      }
    }
    if (p < g.P) {
      lap2 += cross;
      store_tile(g.yj + (int64_t)p * g.y_sp, acc);
    } else {
      store_tile(g.yl, acc + 2.0f * lap2);
    }
    __syncthreads();  // everyone is done with this row's tiles
  }
}

}  // namespace

extern "C" int folx_hip_dot_two_fwdlap(void* stream, const float* a, const float* a_jac, const float* a_lap,
                                       const float* b, const float* b_jac, const float* b_lap, float* y,
                                       float* y_jac, float* y_lap, int64_t NB0, int32_t NB1, int32_t I,
                                       int32_t J, int32_t Kc, int32_t P, const int64_t* strides) {
  if (NB0 < 0 || NB1 < 0 || I < 0 || J < 0 || Kc < 0 || P < 0 || !strides) return FOLX_HIP_EINVAL;
  if (Kc > DT_KMAX) return FOLX_HIP_ENOTSUP;
  const int64_t NB = NB0 * NB1;
  if (NB == 0 || I == 0 || J == 0) return FOLX_HIP_OK;
  const bool constb = !b_jac && !b_lap;  // b without derivatives
  if (!a || !a_lap || !b || !y || !y_lap || (P > 0 && (!a_jac || !y_jac))) return FOLX_HIP_EINVAL;
  if (!constb && (!b_lap || (P > 0 && !b_jac))) return FOLX_HIP_EINVAL;
  DotTwoArgs g;
  g.a = a; g.aj = a_jac; g.al = a_lap; g.b = b; g.bj = b_jac; g.bl = b_lap;
  g.y = y; g.yj = y_jac; g.yl = y_lap;
  g.a_sb0 = strides[0]; g.a_sb1 = strides[1]; g.a_si = strides[2]; g.a_sk = strides[3]; g.a_sp = strides[4];
  g.b_sb0 = strides[5]; g.b_sb1 = strides[6]; g.b_sk = strides[7]; g.b_sj = strides[8]; g.b_sp = strides[9];
  for (int i = 0; i < 10; ++i)
    if (strides[i] < 0) return FOLX_HIP_EINVAL;
  g.NB = NB; g.NB1 = NB1; g.I = I; g.J = J; g.Kc = Kc; g.P = P;
  g.y_sp = NB * (int64_t)I * J;
  g.tiles_i = (I + DT_TILE - 1) / DT_TILE;
  g.tiles_j = (J + DT_TILE - 1) / DT_TILE;
  const int64_t blocks = NB * g.tiles_i * g.tiles_j;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  const int Kp = (Kc + 15) / 16 * 16 > 0 ? (Kc + 15) / 16 * 16 : 16;
  g.Kc = Kc;
  const size_t lds = sizeof(float) * (2 * DT_TILE * (Kp + 4) + 2 * Kp * DT_BS);
  hipStream_t st = (hipStream_t)stream;
  const int nld = DT_TILE * Kp / DT_NT;  // 2, 4, ..., 16
  const dim3 grid((unsigned)blocks), block(DT_NT);
  if (nld <= 4) {
    if (constb) dot_two_kernel<4, true><<<grid, block, lds, st>>>(g);
    else dot_two_kernel<4, false><<<grid, block, lds, st>>>(g);
  } else if (nld <= 8) {
    if (constb) dot_two_kernel<8, true><<<grid, block, lds, st>>>(g);
    else dot_two_kernel<8, false><<<grid, block, lds, st>>>(g);
  } else {
    if (lds > 64 * 1024) {
      // raised once per process (not a stream operation, so never issued inside a stream capture twice)
      static std::atomic<bool> granted{false};
      if (!granted.load()) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(dot_two_kernel<16, false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) != hipSuccess ||
            hipFuncSetAttribute(reinterpret_cast<const void*>(dot_two_kernel<16, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) != hipSuccess)
          return FOLX_HIP_ENOTSUP;
        granted.store(true);
      }
    }
    if (constb) dot_two_kernel<16, true><<<grid, block, lds, st>>>(g);
    else dot_two_kernel<16, false><<<grid, block, lds, st>>>(g);
  }
  return folx_launch_status();
}
