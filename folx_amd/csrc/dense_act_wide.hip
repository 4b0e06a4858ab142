// Wide dense layer (N > 128, K a multiple of 16) with the elementwise work around it folded
// into the GEMM over the Jacobian rows, so that neither the pre-activation Jacobian nor a
// normalised copy of the input Jacobian goes through HBM:
//
//   (a) dense + activation                    y = f(x @ W + bias)
//   (b) LayerNorm + dense                     y = LN(x) @ W + bias
//   (c) LayerNorm + dense + activation        y = f(LN(x) @ W + bias)
//
// with LN(x) = gamma * xh + beta, xh = (x - mean) * rs, rs = rsqrt(var + eps) over the K
// features of a position.  The Jacobian rows are (P * R) x K with R positions.
//
// Activation.  With z = ... @ W + bias, zj[p] and zl the pre-activation triplet,
//   y = f(z),  yj[p] = f'(z) zj[p],  yl = f'(z) zl + f''(z) sum_p zj[p]^2.
//
// LayerNorm in front of a matrix product.  For a Jacobian row t (K features of one position)
// with a = mean(t), b = mean(xh t):   LN'[t] = gamma rs (t - a - b xh), hence
//   LN'[t] @ W = rs (t @ Wg - a w1 - b w2),   Wg = diag(gamma) W,  w1 = 1^T Wg,  w2 = xh @ Wg,
// a rank-2 correction of the product of the RAW row with Wg; w2 = z - bias - beta @ W is known
// from the x row.  The second-order term of LayerNorm, summed over Jacobian rows,
//   rs^2 gamma (-2 V + xh (3 sum_p b_p^2 - sum_p q_p)),  V = sum_p b_p (t_p - a_p),
//   q_p = mean(t_p^2) - a_p^2,
// goes through W as  rs^2 (-2 sum_p b_p (t_p @ Wg - a_p w1) + w2 (3 sum b^2 - sum q)).
// a_p, b_p and mean(t_p^2) are summed from the A tile while it feeds the MFMAs.
//
// Launches on the caller's stream:
//  1. (LayerNorm only) fold gamma / beta into the weights (Wg, w1, c0 = bias + beta @ W), and
//     one wavefront per position for xh, rs, LN(x) and the linear part of LN's lap row;
//  2. the plain dense kernel on the x and lap rows only (2 R of the (P + 2) R rows): z goes to
//     y, the linear part of zl to y_lap;
//  3. the Jacobian GEMM below, whose 128-row tiles are cut ACROSS Jacobian rows: a tile holds
//     4 consecutive positions x 32 consecutive p, ordered position-major, so that each 32 x 32
//     accumulator block belongs to ONE position.  f'(z), w1, w2 and rs of a block are then one
//     value per lane (its column), and the sums over p inside a block stay inside the
//     wavefront (16 registers and the two lane halves).  The sums go to the workspace, one
//     (R, N) slab per group of 32 Jacobian rows;
//  4. a short elementwise kernel that finishes y and y_lap, adding the slabs in a fixed order.
//
// Variant (a) also reads a CONCATENATED operand part by part (a chunk of 16 features lies in
// exactly one part; a part may hold one row per walker that all of the walker's positions
// share) and adds a skip connection in its epilogue, so that a layer fed by
// [own features, per-walker means, ...] forms neither the broadcasts nor the concatenation.
//
// The main loop is the one of the dense kernel: K in chunks of 16 through double-buffered LDS
// tiles filled by global_load_lds_dwordx4, a 128 x 256 tile on 8 wavefronts of 64 x 64,
// v_mfma_f32_32x32x2_f32 with the k order inside a group of 8 permuted to fit 128-bit reads
// (lane l, register j of group t <-> k = 8 t + 4 (l / 32) + j), piece c of an A row stored at
// slot c ^ ((row / 2) % 4).  Only the address a lane asks for differs: tile row m is
// Jacobian row p0 + m % 32 of position r0 + m / 32.
#include <mutex>
#include <type_traits>

#include "activations.h"
#include "dense_act_wide.h"
#include "split_bf16.h"

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
constexpr int KMAX_NORM = 512; // xh of a tile's positions sits in LDS
constexpr int KMAX_NORM_SPLIT = 512;  // bf16x3 form: with xh of 4 x 512 features its LDS is exactly half a CU's
constexpr int A_V4 = BM * BK / 4, W_V4 = BK * BN / 4;
constexpr int A_LD = A_V4 / NT, W_LD = W_V4 / NT;
static_assert(A_V4 % NT == 0 && W_V4 % NT == 0, "every thread loads the same number of pieces");

constexpr int MAX_PARTS = 8;

// The Jacobian operand as a concatenation along K of up to MAX_PARTS arrays (widths multiples
// of 16, so that no chunk of K straddles two).  A broadcast part has one row per `group`
// consecutive positions (a per-walker feature shown to every electron).
struct WideParts {
  const float* jac[MAX_PARTS];
  int64_t pstride[MAX_PARTS];  // floats between consecutive Jacobian rows of the part
  int32_t width[MAX_PARTS];
  int32_t kend[MAX_PARTS];     // first k after the part
  int32_t bcast[MAX_PARTS];
  int32_t n, group;
};

struct WideParams {
  const float* jac;
  const float* W;    // Wg with LayerNorm
  const float* z;    // pre-activation values (R, N), bias included
  const float* xhat; // (R, K)           LayerNorm only
  const float* rs;   // (R)
  const float2* wc;  // (N) pairs (w1, c0)
  float* y_jac;
  const float* res_jac;  // optional (P, R, N) added to the activated Jacobian rows     PARTS instances only
  const float* pre_jac;  // optional (P, R / pre_group, N) added to the PRE-activation Jacobian rows: position r takes
  int64_t pre_group;     // row r / pre_group (a per-walker term shared by the walker's positions)   PARTS instances only
  float* ss;         // (PG, R, N) sums of zj^2 per group of PT Jacobian rows     activation only
  float* s1;         // (PG, R, N) sums of b_p (t_p @ Wg - a_p w1)                LayerNorm only
  float* sc;         // (PG, R, 2) sums of b_p^2 and of q_p
  int64_t R, row_tiles, pos_tiles;
  int32_t P, K, N, col_tiles, act;
  float prm;
  WideParts parts;   // PARTS instances only (jac unused then)
};

// PT = Jacobian rows of a tile: 32 (4 positions per tile, one per accumulator block), or 16 for
// the activation alone (8 positions per tile, two per block: registers 0-7 of a block belong
// to the first, 8-15 to the second), which wastes less when P is 16 more than a multiple of 32.
// SPLIT: the products on the bf16 matrix pipe from operands split into three bf16 pieces, with
// the loop of dense_split_kernel: A and W chunks come through registers and every element is
// split once per workgroup on its way into LDS (A stage [piece][g][row][8 bf16], W stage
// [piece][g][kp][col] dwords).  The thread that stages four k of a tile row also has their fp32
// values, so LayerNorm's row sums are taken there (and added over the four threads of a row
// after the loop) instead of from the fragments of chosen wavefronts; the per-column values the
// epilogue needs (z, w1, c0) are fetched from memory after the loop, which leaves LDS for two
// workgroups per CU.  A concatenated operand (PARTS) is staged the same way, the part of a chunk
// and the address inside it found per chunk as in the direct-to-LDS form.
template <bool NORM, bool ACT, int PT, bool PARTS, bool SPLIT>
__global__ __launch_bounds__(NT, 4) void dense_wide_kernel(WideParams a) {
  static_assert(!PARTS || !NORM, "LayerNorm reads one array");
  static_assert(!PARTS || A_LD == 1, "one A piece per thread");
  static_assert(!SPLIT || !NORM || PT == 32, "LayerNorm's row sums assume groups of 32 rows");
  constexpr int A_PLANE = 2 * BM * 16;     // SPLIT: bytes of one piece of an A chunk
  constexpr int W_PLANE = 2 * 4 * BN * 4;  //        and of a W chunk
  constexpr int RT = BM / PT;  // positions of a tile
  constexpr int PB = 32 / PT;  // positions of a 32-row accumulator block
  static_assert(PT == 32 || (PT == 16 && !NORM), "LayerNorm's row sums assume one position per block");
  __shared__ __attribute__((aligned(16))) float As0[SPLIT ? 3 * A_PLANE / 4 : BM * BK];
  __shared__ __attribute__((aligned(16))) float As1[SPLIT ? 3 * A_PLANE / 4 : BM * BK];
  __shared__ __attribute__((aligned(16))) float Ws0[SPLIT ? 3 * W_PLANE / 4 : BK * BN];
  __shared__ __attribute__((aligned(16))) float Ws1[SPLIT ? 3 * W_PLANE / 4 : BK * BN];
  __shared__ __attribute__((aligned(16))) float xhS[NORM ? RT * (SPLIT ? KMAX_NORM_SPLIT : KMAX_NORM) : 4];
  __shared__ float zS[NORM && !SPLIT ? RT * BN : 1];  // pre-activation values of the tile's positions and columns
  __shared__ float2 wcS[NORM && !SPLIT ? BN : 1];     // (w1, c0) of the tile's columns
  __shared__ float rsS[SPLIT ? 1 : RT];  // SPLIT: rs is read from memory in the epilogue

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
  int64_t a_pos = 0, a_posg = 0;  // PARTS: this thread's position, and its row in a broadcast part
  int32_t a_row = 0, a_kc = 0;    //        its Jacobian row and 16-byte piece
#pragma unroll
  for (int i = 0; i < A_LD; ++i) {
    const int idx = tid + NT * i;
    const int m = idx / 4, c = idx % 4;
    const int kc = c ^ ((m / 2) % 4);
    int p = p0 + m % PT;
    if (p >= P) p = P - 1;  // reaches accumulator rows that are neither stored nor summed
    if constexpr (PARTS) {
      a_pos = r0 + m / PT;
      a_posg = a_pos / a.parts.group;
      a_row = p;
      a_kc = kc * 4;
      a_p[i] = nullptr;
    } else {
      a_p[i] = a.jac + ((int64_t)p * R + r0 + m / PT) * K + kc * 4;  // tile row m: position m / PT, row m % PT
    }
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
    if constexpr (PARTS) {
      // the part this chunk of K lies in: the same for the whole workgroup
      const int k0 = kt * BK;
      int sp = 0;
      while (sp + 1 < a.parts.n && k0 >= a.parts.kend[sp]) ++sp;
      const int32_t wd = a.parts.width[sp];
      const float* src = a.parts.jac[sp] + (int64_t)a_row * a.parts.pstride[sp] +
                         (a.parts.bcast[sp] ? a_posg : a_pos) * wd + (k0 - (a.parts.kend[sp] - wd)) + a_kc;
      __builtin_amdgcn_global_load_lds(FOLX_GPTR(src), FOLX_LPTR(&as[(wave * 64) * 4]), 16, 0, 0);
    } else {
#pragma unroll
      for (int i = 0; i < A_LD; ++i)
        __builtin_amdgcn_global_load_lds(FOLX_GPTR(a_p[i] + kt * BK), FOLX_LPTR(&as[(wave * 64 + NT * i) * 4]), 16,
                                         0, 0);
    }
#pragma unroll
    for (int i = 0; i < W_LD; ++i)
      __builtin_amdgcn_global_load_lds(FOLX_GPTR(w_p[i] + (int64_t)kt * BK * N),
                                       FOLX_LPTR(&ws[(wave * 64 + NT * i) * 4]), 16, 0, 0);
  };

  // Without LayerNorm the epilogue only needs f'(z) of this lane's columns at its blocks'
  // positions, and there are registers to spare for it: z is asked for first, then the first
  // chunk, and f' is evaluated while the chunk is on its way.  With LayerNorm what the
  // epilogue needs per position and column is staged in LDS behind the first chunk, and both
  // are waited for together in front of the first barrier.
  float dr[TM][TN][PB];
  if constexpr (!NORM) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        int gc = col0 + wc + j * 32 + l32;
        if (gc >= N) gc = N - 1;
#pragma unroll
        for (int b = 0; b < PB; ++b) dr[i][j][b] = a.z[(r0 + (wrow * TM + i) * PB + b) * N + gc];
      }
  }
  // SPLIT staging: thread t has k quarter t % 4 of tile row t / 4; wavefront w has rows 2 w and
  // 2 w + 1 of the W chunk, lane l their columns 4 l .. 4 l + 3
  const float* sa_src = nullptr;
  const float* sw_src = nullptr;
  int sa_dst = 0, sw_dst = 0;
  float4 ra = make_float4(0.f, 0.f, 0.f, 0.f), rw0 = ra, rw1 = ra;
  if constexpr (SPLIT) {
    const int m = tid / 4, q = tid % 4;
    int p = p0 + m % PT;
    if (p >= P) p = P - 1;
    if constexpr (PARTS) {  // the part and the address inside it are found per chunk
      a_pos = r0 + m / PT;
      a_posg = a_pos / a.parts.group;
      a_row = p;
      a_kc = q * 4;
    } else {
      sa_src = a.jac + ((int64_t)p * R + r0 + m / PT) * K + q * 4;
    }
    sa_dst = ((q / 2) * BM + m) * 16 + (q % 2) * 8;
    int wn = col0 + lane * 4;
    if (wn > N - 4) wn = N - 4;
    sw_src = a.W + (int64_t)(2 * wave) * N + wn;
    sw_dst = (wave * BN + lane * 4) * 4;
  }
  auto fetch = [&](int kt) __attribute__((always_inline)) {
    if constexpr (PARTS) {
      const int k0 = kt * BK;
      int sp = 0;
      while (sp + 1 < a.parts.n && k0 >= a.parts.kend[sp]) ++sp;
      const int32_t wd = a.parts.width[sp];
      ra = *reinterpret_cast<const float4*>(a.parts.jac[sp] + (int64_t)a_row * a.parts.pstride[sp] +
                                            (a.parts.bcast[sp] ? a_posg : a_pos) * wd + (k0 - (a.parts.kend[sp] - wd)) + a_kc);
    } else {
      ra = *reinterpret_cast<const float4*>(sa_src + kt * BK);  // plain: the line's other half follows one chunk later
    }
    rw0 = *reinterpret_cast<const float4*>(sw_src + (int64_t)kt * BK * N);
    rw1 = *reinterpret_cast<const float4*>(sw_src + (int64_t)kt * BK * N + N);
  };
  if constexpr (SPLIT) fetch(0);
  else issue(0, As0, Ws0);
  if constexpr (NORM && !SPLIT) {
    for (int e = tid; e < RT * BN; e += NT) {
      int gc = col0 + e % BN;
      if (gc >= N) gc = N - 1;
      zS[e] = a.z[(r0 + e / BN) * N + gc];
    }
  } else if constexpr (ACT) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int b = 0; b < PB; ++b) {
          float f, d1, d2;
          act_eval_fused(a.act, dr[i][j][b], a.prm, f, d1, d2);
          dr[i][j][b] = d1;
        }
  }
  if constexpr (NORM) {
    // xh of the tile's RT positions: RT * K consecutive floats
    const float4* src = reinterpret_cast<const float4*>(a.xhat + r0 * K);
    for (int e = tid; e < RT * K / 4; e += NT) reinterpret_cast<float4*>(xhS)[e] = src[e];
    if constexpr (!SPLIT)
      if (tid < BN) wcS[tid] = a.wc[col0 + tid < N ? col0 + tid : N - 1];
    if constexpr (!SPLIT)
      if (tid < RT) rsS[tid] = a.rs[r0 + tid];
  }

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  if constexpr (PARTS) {
    // The per-walker pre-activation term is what the accumulators START from (the products are added to it): its
    // loads are in flight with the first chunk, where registers are plentiful, instead of in the epilogue.
    // Register r of a block <-> Jacobian row p0 + 4 (lane / 32) + 8 ((r / 4) % GB) + r % 4 of position (r / 4) / GB.
    if (a.pre_jac) {
      constexpr int GB = PT / 8;
      const int64_t pre_pstride = (R / a.pre_group) * N;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          int gc = col0 + wc + j * 32 + l32;
          if (gc >= N) gc = N - 1;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int g = r / 4, b = g / GB;
            int prow = p0 + 4 * lh + 8 * (g % GB) + r % 4;
            if (prow >= P) prow = P - 1;  // rows past P of a ragged tile are neither stored nor summed
            const int64_t pos = r0 + (wrow * TM + i) * PB + b;
            acc[i][j][r] = a.pre_jac[(int64_t)prow * pre_pstride + (pos / a.pre_group) * N + gc];
          }
        }
    }
  }
  // LayerNorm's row sums are taken by ONE wavefront per tile row block and SIMD: block i of
  // tile row group wrow by the wavefront with column index i + 2 * wrow.  That wavefront runs
  // its own copy of the K loop; the others run the plain one.  Per tile row wr + 32 si + l32,
  // over the k this lane half reads: sum t, sum xh t, sum t^2.
  const int si = NORM ? (wave % WN) - 2 * wrow : -1;
  float sa = 0.0f, sb = 0.0f, s2 = 0.0f;

  const int sw = (l32 / 2) % 4;
  auto compute = [&](const float* as, const float* ws, int kt, auto sblk) __attribute__((always_inline)) {
    constexpr int SI = decltype(sblk)::value;
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
      if constexpr (SI >= 0) {
        const float4 xv = *reinterpret_cast<const float4*>(&xhS[(wrow * TM + SI) * K + kt * BK + (tg * 2 + lh) * 4]);
        const float4 t = a4[SI];
        sa += (t.x + t.y) + (t.z + t.w);
        sb = fmaf(t.x, xv.x, fmaf(t.y, xv.y, fmaf(t.z, xv.z, fmaf(t.w, xv.w, sb))));
        s2 = fmaf(t.x, t.x, fmaf(t.y, t.y, fmaf(t.z, t.z, fmaf(t.w, t.w, s2))));
      }
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

  const int KT = K / BK;
  if constexpr (SPLIT) {
    using namespace folx_split;
    // chunk kt of this thread's registers into a stage; LayerNorm's sums from the fp32 values
    auto put = [&](int kt, float* asf, float* wsf) __attribute__((always_inline)) {
      char* as = reinterpret_cast<char*>(asf);
      char* ws = reinterpret_cast<char*>(wsf);
      if constexpr (NORM) {
        const float4 xv = *reinterpret_cast<const float4*>(&xhS[(tid / (4 * PT)) * K + kt * BK + (tid % 4) * 4]);
        sa += (ra.x + ra.y) + (ra.z + ra.w);
        sb = fmaf(ra.x, xv.x, fmaf(ra.y, xv.y, fmaf(ra.z, xv.z, fmaf(ra.w, xv.w, sb))));
        s2 = fmaf(ra.x, ra.x, fmaf(ra.y, ra.y, fmaf(ra.z, ra.z, fmaf(ra.w, ra.w, s2))));
      }
      unsigned p1a, p2a, p3a, p1b, p2b, p3b;
      split_pair(ra.x, ra.y, p1a, p2a, p3a);
      split_pair(ra.z, ra.w, p1b, p2b, p3b);
      uint2v q;
      q[0] = p1a; q[1] = p1b; *reinterpret_cast<uint2v*>(as + sa_dst) = q;
      q[0] = p2a; q[1] = p2b; *reinterpret_cast<uint2v*>(as + A_PLANE + sa_dst) = q;
      q[0] = p3a; q[1] = p3b; *reinterpret_cast<uint2v*>(as + 2 * A_PLANE + sa_dst) = q;
      unsigned a1[4], a2[4], a3[4];
      split_pair(rw0.x, rw1.x, a1[0], a2[0], a3[0]);
      split_pair(rw0.y, rw1.y, a1[1], a2[1], a3[1]);
      split_pair(rw0.z, rw1.z, a1[2], a2[2], a3[2]);
      split_pair(rw0.w, rw1.w, a1[3], a2[3], a3[3]);
      uint4v q1, q2, q3;
#pragma unroll
      for (int c = 0; c < 4; ++c) { q1[c] = a1[c]; q2[c] = a2[c]; q3[c] = a3[c]; }
      *reinterpret_cast<uint4v*>(ws + sw_dst) = q1;
      *reinterpret_cast<uint4v*>(ws + W_PLANE + sw_dst) = q2;
      *reinterpret_cast<uint4v*>(ws + 2 * W_PLANE + sw_dst) = q3;
    };
    auto products = [&](const float* asf, const float* wsf) __attribute__((always_inline)) {
      const char* as = reinterpret_cast<const char*>(asf);
      const char* ws = reinterpret_cast<const char*>(wsf);
      bf16x8 fb[TN][3];
#pragma unroll
      for (int p = 0; p < 3; ++p)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          uint4v v;
#pragma unroll
          for (int kp = 0; kp < 4; ++kp)
            v[kp] = *reinterpret_cast<const unsigned*>(ws + p * W_PLANE + ((lh * 4 + kp) * BN + wc + j * 32 + l32) * 4);
          fb[j][p] = __builtin_bit_cast(bf16x8, v);
        }
      bf16x8 fa[TM];
#pragma unroll
      for (int q = 0; q < 6; ++q) {
        if (q == 0 || kPieceA[q] != kPieceA[q - 1]) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            fa[i] = *reinterpret_cast<const bf16x8*>(as + kPieceA[q] * A_PLANE + (lh * BM + wr + i * 32 + l32) * 16);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j][kPieceB[q]], acc[i][j], 0, 0, 0);
      }
    };
    __syncthreads();  // xh of the tile's positions is in LDS (the first chunk has landed as well)
    put(0, As0, Ws0);
    if (KT > 1) fetch(1);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    for (int kt = 0; kt < KT; kt += 2) {
      if (kt + 1 < KT) {
        put(kt + 1, As1, Ws1);
        if (kt + 2 < KT) fetch(kt + 2);
      }
      products(As0, Ws0);
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if (kt + 1 < KT) {
        if (kt + 2 < KT) {
          put(kt + 2, As0, Ws0);
          if (kt + 3 < KT) fetch(kt + 3);
        }
        products(As1, Ws1);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      }
    }
  }
  // The loads of a chunk are waited for at the end of the chunk before it; the barrier then
  // also says that every wavefront is done reading the buffer that is refilled next.
  if constexpr (!SPLIT) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }
  auto kloop = [&](auto sblk) __attribute__((always_inline)) {
    for (int kt = 0; kt < KT; kt += 2) {
      if (kt + 1 < KT) issue(kt + 1, As1, Ws1);
      compute(As0, Ws0, kt, sblk);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (kt + 1 < KT) {
        if (kt + 2 < KT) issue(kt + 2, As0, Ws0);
        compute(As1, Ws1, kt + 1, sblk);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
      }
    }
  };
  static_assert(TM == 2, "one loop copy per accumulator block row");
  if constexpr (!SPLIT) {
    if (NORM && si == 0) kloop(std::integral_constant<int, 0>{});
    else if (NORM && si == 1) kloop(std::integral_constant<int, 1>{});
    else kloop(std::integral_constant<int, -1>{});
  }
  // SPLIT: what the epilogue needs per column, asked for while the row sums are put together
  float zpre[TM][TN];
  float2 wcpre[TN];
  if constexpr (NORM && SPLIT) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      int gc = col0 + wc + j * 32 + l32;
      if (gc >= N) gc = N - 1;
      wcpre[j] = a.wc[gc];
#pragma unroll
      for (int i = 0; i < TM; ++i) zpre[i][j] = a.z[(r0 + wrow * TM + i) * N + gc];
    }
  }

  // The row sums go through LDS (the tiles are no longer read: the loop ended with a barrier)
  // to the lanes that hold the rows' accumulators.
  float2* st = reinterpret_cast<float2*>(As0) + wrow * TM * 32;  // [wrow][i][row] (a, b)
  if constexpr (NORM && SPLIT) {
    // the four threads of a tile row add their quarters; thread 4 m keeps row m
    float ta = sa + __shfl_xor(sa, 1, FOLX_WAVE), tb = sb + __shfl_xor(sb, 1, FOLX_WAVE);
    float t2 = s2 + __shfl_xor(s2, 1, FOLX_WAVE);
    ta += __shfl_xor(ta, 2, FOLX_WAVE);
    tb += __shfl_xor(tb, 2, FOLX_WAVE);
    t2 += __shfl_xor(t2, 2, FOLX_WAVE);
    const int m = tid / 4;
    const float invK = 1.0f / (float)K;
    const bool keep = tid % 4 == 0 && p0 + m % PT < P;
    const float av = keep ? ta * invK : 0.0f;
    const float bv = keep ? tb * invK : 0.0f;
    const float qv = keep ? t2 * invK - av * av : 0.0f;
    float2* rowsums = reinterpret_cast<float2*>(As0);   // [tile row]
    float2* wavesums = rowsums + BM;                     // [wavefront]: 16 rows of one position each
    if (tid % 4 == 0) rowsums[m] = make_float2(av, bv);
    if (ct == 0) {  // the two scalar sums of a position: two wavefronts each
      float eb = bv * bv, eq = qv;
#pragma unroll
      for (int off = 32; off >= 4; off >>= 1) {
        eb += __shfl_xor(eb, off, FOLX_WAVE);
        eq += __shfl_xor(eq, off, FOLX_WAVE);
      }
      if (lane == 0) wavesums[wave] = make_float2(eb, eq);
    }
    __syncthreads();
    if (ct == 0 && tid < RT) {
      const float2 u = wavesums[2 * tid], v = wavesums[2 * tid + 1];
      float* o = a.sc + ((int64_t)pg * R + r0 + tid) * 2;
      o[0] = u.x + v.x;
      o[1] = u.y + v.y;
    }
  }
  if constexpr (NORM && !SPLIT) {
    if (si >= 0 && si < TM) {
      const float invK = 1.0f / (float)K;
      const bool pv = p0 + l32 < P;
      const float ta = sa + __shfl_xor(sa, 32, FOLX_WAVE);
      const float tb = sb + __shfl_xor(sb, 32, FOLX_WAVE);
      const float t2 = s2 + __shfl_xor(s2, 32, FOLX_WAVE);
      const float av = pv ? ta * invK : 0.0f;
      const float bv = pv ? tb * invK : 0.0f;
      const float qv = pv ? t2 * invK - av * av : 0.0f;
      if (lh == 0) st[si * 32 + l32] = make_float2(av, bv);
      if (ct == 0) {  // the two scalar sums of the block
        float eb = bv * bv, eq = qv;
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) {
          eb += __shfl_xor(eb, off, FOLX_WAVE);
          eq += __shfl_xor(eq, off, FOLX_WAVE);
        }
        if (lane == 0) {
          float* o = a.sc + ((int64_t)pg * R + r0 + wrow * TM + si) * 2;
          o[0] = eb;
          o[1] = eq;
        }
      }
    }
    __syncthreads();
  }

  // Register r of a block is tile row 8 (r / 4) + 4 (lane / 32) + r % 4 of the block, column
  // lane % 32: Jacobian row p0 + (that row) % PT of the block's position (that row) / PT.
  const int64_t pstride = R * N;  // floats between consecutive Jacobian rows
  const bool full_tile = (p0 + PT <= P) && (col0 + BN <= N);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int64_t pos = r0 + (wrow * TM + i) * PB;
    float rsv = 1.0f;
    if constexpr (NORM) rsv = SPLIT ? a.rs[r0 + wrow * TM + i] : rsS[wrow * TM + i];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int gc = col0 + wc + j * 32 + l32;
      float zv[PB], d1[PB];
#pragma unroll
      for (int b = 0; b < PB; ++b) {
        zv[b] = 0.0f;
        d1[b] = 1.0f;
        if constexpr (NORM) {
          if constexpr (SPLIT) zv[b] = zpre[i][j];
          else zv[b] = zS[(wrow * TM + i) * BN + wc + j * 32 + l32];
          if constexpr (ACT) {
            float f, d2;
            act_eval_fused(a.act, zv[b], a.prm, f, d1[b], d2);
          }
        } else if constexpr (ACT) {
          d1[b] = dr[i][j][b];
        }
      }
      float w1c = 0.0f, w2c = 0.0f;
      if constexpr (NORM) {
        const float2 t = SPLIT ? wcpre[j] : wcS[wc + j * 32 + l32];
        w1c = t.x;
        w2c = zv[0] - t.y;
      }
      float* out = a.y_jac + ((int64_t)(p0 + 4 * lh) * R + pos) * N + gc;
      float ss[PB], s1 = 0.0f;
#pragma unroll
      for (int b = 0; b < PB; ++b) ss[b] = 0.0f;
      const float* resp = nullptr;
      if constexpr (PARTS) resp = a.res_jac ? a.res_jac + ((int64_t)(p0 + 4 * lh) * R + pos) * N + gc : nullptr;
      auto rows = [&](auto full, auto has_res) __attribute__((always_inline)) {
        constexpr int GB = PT / 8;     // register groups per position
        constexpr bool FULL = decltype(full)::value, RES = decltype(has_res)::value;
        // What the epilogue reads from memory (the skip connection) is asked for one register group ahead
        // of its use: the stores of a group cannot be told apart from that array, so a load written after
        // them would wait for them to be issued, and every group would pay a round trip of its own.
        float rbuf[2][4];
        auto fetch = [&](int g, float (&rb)[4]) __attribute__((always_inline)) {
          const int b = g / GB;
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            const int pl = 8 * (g % GB) + rr;
            const int64_t off = (int64_t)pl * pstride + (int64_t)b * N;
            const bool live = FULL || (p0 + 4 * lh + pl < P && gc < N);
            rb[rr] = 0.0f;
            if constexpr (RES) {
              if constexpr (FULL) rb[rr] = __builtin_nontemporal_load(resp + off);
              else if (live) rb[rr] = resp[off];
            }
          }
        };
        if constexpr (RES) fetch(0, rbuf[0]);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int b = g / GB;          // position of this group inside the block
          if constexpr (RES)
            if (g + 1 < 4) fetch(g + 1, rbuf[(g + 1) & 1]);
          float ap[4] = {0.0f, 0.0f, 0.0f, 0.0f}, bp[4] = {0.0f, 0.0f, 0.0f, 0.0f};
          if constexpr (NORM) {
            const float4* sp = reinterpret_cast<const float4*>(st + i * 32 + 8 * g + 4 * lh);
            const float4 u0 = sp[0], u1 = sp[1];
            ap[0] = u0.x; bp[0] = u0.y; ap[1] = u0.z; bp[1] = u0.w;
            ap[2] = u1.x; bp[2] = u1.y; ap[3] = u1.z; bp[3] = u1.w;
          }
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            const int pl = 8 * (g % GB) + rr;
            float v = acc[i][j][4 * g + rr];
            if constexpr (NORM) {
              v = fmaf(-ap[rr], w1c, v);
              s1 = fmaf(bp[rr], v, s1);
              v = fmaf(-bp[rr], w2c, v) * rsv;
            }
            const int64_t off = (int64_t)pl * pstride + (int64_t)b * N;
            float* o = out + off;
            if constexpr (FULL) {
              if constexpr (ACT) ss[b] = fmaf(v, v, ss[b]);
              float w = d1[b] * v;
              if constexpr (RES) w += rbuf[g & 1][rr];
              __builtin_nontemporal_store(w, o);
            } else if (p0 + 4 * lh + pl < P) {
              if constexpr (ACT) ss[b] = fmaf(v, v, ss[b]);
              if (gc < N) *o = d1[b] * v + (RES ? rbuf[g & 1][rr] : 0.0f);
            }
          }
        }
      };
      if (PARTS && resp != nullptr) {
        if (full_tile) rows(std::true_type{}, std::true_type{});
        else rows(std::false_type{}, std::true_type{});
      } else {
        if (full_tile) rows(std::true_type{}, std::false_type{});
        else rows(std::false_type{}, std::false_type{});
      }
      const int64_t so = ((int64_t)pg * R + pos) * N + gc;
      if constexpr (ACT) {
#pragma unroll
        for (int b = 0; b < PB; ++b) {
          const float t = ss[b] + __shfl_xor(ss[b], 32, FOLX_WAVE);
          if (lh == 0 && gc < N) a.ss[so + (int64_t)b * N] = t;
        }
      }
      if constexpr (NORM) {
        s1 += __shfl_xor(s1, 32, FOLX_WAVE);
        if (lh == 0 && gc < N) a.s1[so] = s1;
      }
    }
  }
}

// Finishes the x and lap rows.  On entry y holds z and y_lap the part of zl that is linear in
// the input's lap row (what launch 2 left there).  One float4 per thread.
template <bool NORM, bool ACT>
__global__ __launch_bounds__(256) void dense_wide_finish(float* __restrict__ y, float* __restrict__ y_lap,
                                                         const float* __restrict__ ss, const float* __restrict__ s1,
                                                         const float* __restrict__ sc, const float* __restrict__ rs,
                                                         const float2* __restrict__ wc, int64_t S4, int64_t R,
                                                         int32_t N, int32_t PG, int32_t act, float prm,
                                                         const float* __restrict__ res,
                                                         const float* __restrict__ res_lap) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= S4) return;
  const float4 z = reinterpret_cast<const float4*>(y)[i];
  float4 zl = reinterpret_cast<const float4*>(y_lap)[i];
  if constexpr (NORM) {
    const int64_t pos = i / (N / 4);
    const int32_t n = (int32_t)(i % (N / 4)) * 4;
    float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    float eb = 0.0f, eq = 0.0f;
    for (int g = 0; g < PG; ++g) {
      const float4 t = reinterpret_cast<const float4*>(s1)[(int64_t)g * S4 + i];
      v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
      eb += sc[((int64_t)g * R + pos) * 2];
      eq += sc[((int64_t)g * R + pos) * 2 + 1];
    }
    const float r = rs[pos];
    const float r2 = r * r, e = 3.0f * eb - eq;
    zl.x += r2 * fmaf(z.x - wc[n].y, e, -2.0f * v.x);
    zl.y += r2 * fmaf(z.y - wc[n + 1].y, e, -2.0f * v.y);
    zl.z += r2 * fmaf(z.z - wc[n + 2].y, e, -2.0f * v.z);
    zl.w += r2 * fmaf(z.w - wc[n + 3].y, e, -2.0f * v.w);
  }
  if constexpr (ACT) {
    float4 s = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (int g = 0; g < PG; ++g) {
      const float4 t = reinterpret_cast<const float4*>(ss)[(int64_t)g * S4 + i];
      s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
    }
    float4 f;
    float d1, d2;
    act_eval_fused(act, z.x, prm, f.x, d1, d2); zl.x = fmaf(d1, zl.x, d2 * s.x);
    act_eval_fused(act, z.y, prm, f.y, d1, d2); zl.y = fmaf(d1, zl.y, d2 * s.y);
    act_eval_fused(act, z.z, prm, f.z, d1, d2); zl.z = fmaf(d1, zl.z, d2 * s.z);
    act_eval_fused(act, z.w, prm, f.w, d1, d2); zl.w = fmaf(d1, zl.w, d2 * s.w);
    if (res) {
      const float4 r = reinterpret_cast<const float4*>(res)[i];
      f.x += r.x; f.y += r.y; f.z += r.z; f.w += r.w;
    }
    reinterpret_cast<float4*>(y)[i] = f;
  }
  if (res_lap) {
    const float4 r = reinterpret_cast<const float4*>(res_lap)[i];
    zl.x += r.x; zl.y += r.y; zl.z += r.z; zl.w += r.w;
  }
  reinterpret_cast<float4*>(y_lap)[i] = zl;
}

// Wg = diag(gamma) W and per column the pair (w1, c0) = (1^T Wg, bias + beta @ W).  A block
// takes 64 columns; its 16 wavefronts split the K rows.
__global__ __launch_bounds__(1024) void norm_fold_kernel(const float* __restrict__ W, const float* __restrict__ bias,
                                                         const float* __restrict__ gamma,
                                                         const float* __restrict__ beta, float* __restrict__ Wg,
                                                         float2* __restrict__ wc, int32_t K, int32_t N) {
  __shared__ float ps[16][64], pc[16][64];
  const int c = threadIdx.x % 64, sl = threadIdx.x / 64;
  const int n = blockIdx.x * 64 + c;
  float s = 0.0f, cc = 0.0f;
  if (n < N) {
    for (int k = sl; k < K; k += 16) {
      const float w = W[(int64_t)k * N + n];
      const float wg = gamma ? gamma[k] * w : w;
      Wg[(int64_t)k * N + n] = wg;
      s += wg;
      if (beta) cc = fmaf(beta[k], w, cc);
    }
  }
  ps[sl][c] = s;
  pc[sl][c] = cc;
  __syncthreads();
  if (sl == 0 && n < N) {
    float ts = 0.0f, tc = bias ? bias[n] : 0.0f;
    for (int i = 0; i < 16; ++i) { ts += ps[i][c]; tc += pc[i][c]; }
    wc[n] = make_float2(ts, tc);
  }
}

// One wavefront per position: xh, rs, LN(x) and the part of LN's lap row that is linear in the
// input's lap row, gamma rs (lap - mean(lap) - xh mean(xh lap)).  K <= 512: two float4 per lane.
__global__ __launch_bounds__(256) void norm_rows_kernel(const float* __restrict__ x, const float* __restrict__ lap,
                                                        const float* __restrict__ gamma,
                                                        const float* __restrict__ beta, float* __restrict__ xhat,
                                                        float* __restrict__ rs, float* __restrict__ nx,
                                                        float* __restrict__ nlap, int64_t R, int32_t K, float eps) {
  const int lane = threadIdx.x % 64;
  const int64_t pos = (int64_t)blockIdx.x * 4 + threadIdx.x / 64;
  if (pos >= R) return;
  auto wsum = [](float v) __attribute__((always_inline)) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, FOLX_WAVE);
    return v;
  };
  const int nv = K / 4;
  const float invK = 1.0f / (float)K;
  float4 xv[2], lv[2];
  float s = 0.0f, sl = 0.0f;
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int e = lane + 64 * c;
    xv[c] = lv[c] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (e < nv) {
      xv[c] = reinterpret_cast<const float4*>(x + pos * K)[e];
      lv[c] = reinterpret_cast<const float4*>(lap + pos * K)[e];
    }
    s += (xv[c].x + xv[c].y) + (xv[c].z + xv[c].w);
    sl += (lv[c].x + lv[c].y) + (lv[c].z + lv[c].w);
  }
  const float mean = wsum(s) * invK;
  const float aL = wsum(sl) * invK;
  float sv = 0.0f;
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    if (lane + 64 * c < nv) {
      xv[c].x -= mean; xv[c].y -= mean; xv[c].z -= mean; xv[c].w -= mean;
      sv += xv[c].x * xv[c].x + xv[c].y * xv[c].y + xv[c].z * xv[c].z + xv[c].w * xv[c].w;
    }
  }
  const float r = 1.0f / sqrtf(wsum(sv) * invK + eps);
  float sbl = 0.0f;
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    xv[c].x *= r; xv[c].y *= r; xv[c].z *= r; xv[c].w *= r;
    sbl += xv[c].x * lv[c].x + xv[c].y * lv[c].y + xv[c].z * lv[c].z + xv[c].w * lv[c].w;
  }
  const float bL = wsum(sbl) * invK;
  if (lane == 0) rs[pos] = r;
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int e = lane + 64 * c;
    if (e < nv) {
      const float4 g = gamma ? reinterpret_cast<const float4*>(gamma)[e] : make_float4(1.0f, 1.0f, 1.0f, 1.0f);
      const float4 b = beta ? reinterpret_cast<const float4*>(beta)[e] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      reinterpret_cast<float4*>(xhat + pos * K)[e] = xv[c];
      reinterpret_cast<float4*>(nx + pos * K)[e] =
          make_float4(fmaf(g.x, xv[c].x, b.x), fmaf(g.y, xv[c].y, b.y), fmaf(g.z, xv[c].z, b.z), fmaf(g.w, xv[c].w, b.w));
      reinterpret_cast<float4*>(nlap + pos * K)[e] =
          make_float4(g.x * r * (lv[c].x - aL - bL * xv[c].x), g.y * r * (lv[c].y - aL - bL * xv[c].y),
                      g.z * r * (lv[c].z - aL - bL * xv[c].z), g.w * r * (lv[c].w - aL - bL * xv[c].w));
    }
  }
}

// y[r][c] += pre[r / group][c], y_lap likewise: the per-walker pre-activation term on the x and lap
// rows (one float4 per thread).
__global__ __launch_bounds__(256) void wide_add_pre_kernel(float* __restrict__ y, float* __restrict__ y_lap,
                                                           const float* __restrict__ pre,
                                                           const float* __restrict__ pre_lap, int64_t S4, int32_t N4,
                                                           int64_t group) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= S4) return;
  const int64_t src = (i / N4 / group) * N4 + i % N4;
  float4 a = reinterpret_cast<float4*>(y)[i], b = reinterpret_cast<float4*>(y_lap)[i];
  const float4 p = reinterpret_cast<const float4*>(pre)[src], q = reinterpret_cast<const float4*>(pre_lap)[src];
  a.x += p.x; a.y += p.y; a.z += p.z; a.w += p.w;
  b.x += q.x; b.y += q.y; b.z += q.z; b.w += q.w;
  reinterpret_cast<float4*>(y)[i] = a;
  reinterpret_cast<float4*>(y_lap)[i] = b;
}

// Shapes the path takes, launch sizes and the carve-up of the workspace (offsets in floats,
// every part a multiple of 4 floats).
struct WidePlan {
  int64_t row_tiles, pos_tiles, blocks, ws_bytes;
  int64_t o_ss, o_s1, o_sc, o_xhat, o_rs, o_nx, o_nlap, o_wg, o_wc;
  int32_t PG, PT, col_tiles;
};

bool plan_wide(int64_t R, int32_t P, int32_t K, int32_t N, bool norm, bool act, WidePlan& pl) {
  if (R <= 0 || R % 4 != 0 || P < 1 || K < BK || K % BK != 0 || N <= 128 || N % 4 != 0) return false;
  if (norm && K > KMAX_NORM) return false;
  // groups of 16 Jacobian rows where that leaves fewer empty tile rows
  pl.PT = (!norm && R % 8 == 0 && (P + 15) / 16 * 16 < (P + 31) / 32 * 32) ? 16 : 32;
  pl.PG = (P + pl.PT - 1) / pl.PT;
  pl.pos_tiles = R / (BM / pl.PT);
  pl.row_tiles = pl.pos_tiles * pl.PG;
  pl.col_tiles = (N + BN - 1) / BN;
  pl.blocks = (pl.row_tiles + NXCD - 1) / NXCD * NXCD * pl.col_tiles;
  if (pl.blocks > 0x7fffffffLL) return false;
  if (R * (int64_t)N / 4 / 256 + 1 > 0x7fffffffLL) return false;
  const int64_t slab = (int64_t)pl.PG * R * N;
  int64_t o = 0;
  auto take = [&](int64_t n) { const int64_t at = o; o += (n + 3) / 4 * 4; return at; };
  pl.o_ss = act ? take(slab) : 0;
  if (norm) {
    pl.o_s1 = take(slab);
    pl.o_sc = take((int64_t)pl.PG * R * 2);
    pl.o_xhat = take(R * (int64_t)K);
    pl.o_rs = take(R);
    pl.o_nx = take(R * (int64_t)K);
    pl.o_nlap = take(R * (int64_t)K);
    pl.o_wg = take((int64_t)K * N);
    pl.o_wc = take(2 * (int64_t)N);
  }
  pl.ws_bytes = o * 4;
  return true;
}

template <bool NORM, bool ACT, int PT, bool PARTS = false>
int launch_wide(hipStream_t st, const WideParams& a, const WidePlan& pl, float* y, float* y_lap,
                const float* res = nullptr, const float* res_lap = nullptr) {
  const bool split = folx_gemm_mode() == FOLX_HIP_GEMM_BF16X3 && (!NORM || a.K <= KMAX_NORM_SPLIT);
  if (split) dense_wide_kernel<NORM, ACT, PT, PARTS, true><<<dim3((unsigned)pl.blocks), dim3(NT), 0, st>>>(a);
  if (!split) dense_wide_kernel<NORM, ACT, PT, PARTS, false><<<dim3((unsigned)pl.blocks), dim3(NT), 0, st>>>(a);
  int rc = folx_launch_status();
  if (rc != FOLX_HIP_OK) return rc;
  const int64_t S4 = a.R * (int64_t)a.N / 4;
  dense_wide_finish<NORM, ACT><<<dim3((unsigned)((S4 + 255) / 256)), dim3(256), 0, st>>>(
      y, y_lap, a.ss, a.s1, a.sc, a.rs, a.wc, S4, a.R, a.N, pl.PG, a.act, a.prm, res, res_lap);
  return folx_launch_status();
}

int run_wide(hipStream_t st, bool norm, int32_t act, float param, const float* x, const float* jac, const float* lap,
             const float* gamma, const float* beta, float eps, const float* W, const float* bias, float* y,
             float* y_jac, float* y_lap, int64_t R, int32_t P, int32_t K, int32_t N, void* workspace,
             int64_t workspace_bytes, const WideParts* parts = nullptr, const float* res = nullptr,
             const float* res_jac = nullptr, const float* res_lap = nullptr, const float* pre = nullptr,
             const float* pre_jac = nullptr, const float* pre_lap = nullptr, int64_t pre_group = 1) {
  const bool has_act = act >= 0;
  WidePlan pl;
  if ((has_act && !act_fused(act)) || !plan_wide(R, P, K, N, norm, has_act, pl)) return FOLX_HIP_ENOTSUP;
  if (!norm && !has_act) return FOLX_HIP_ENOTSUP;  // that is the plain dense rule
  if (parts && norm) return FOLX_HIP_ENOTSUP;
  if (!x || (!jac && !parts) || !lap || !W || !y || !y_jac || !y_lap) return FOLX_HIP_EINVAL;
  if (!folx_aligned16(jac) || !folx_aligned16(W) || !folx_aligned16(y) || !folx_aligned16(y_lap))
    return FOLX_HIP_ENOTSUP;
  if (norm && (!folx_aligned16(x) || !folx_aligned16(lap) || !folx_aligned16(gamma) || !folx_aligned16(beta)))
    return FOLX_HIP_ENOTSUP;
  if (!workspace || workspace_bytes < pl.ws_bytes || !folx_aligned16(workspace)) return FOLX_HIP_EINVAL;
  float* ws = (float*)workspace;
  WideParams a;
  a.jac = jac; a.W = W; a.z = y; a.y_jac = y_jac; a.res_jac = res_jac;
  a.pre_jac = pre_jac; a.pre_group = pre_group;
  a.xhat = nullptr; a.rs = nullptr; a.wc = nullptr;
  a.ss = ws + pl.o_ss; a.s1 = nullptr; a.sc = nullptr;
  a.R = R; a.row_tiles = pl.row_tiles; a.pos_tiles = pl.pos_tiles;
  a.P = P; a.K = K; a.N = N; a.col_tiles = pl.col_tiles; a.act = act; a.prm = param;
  const float* in_x = x;
  const float* in_lap = lap;
  if (norm) {
    norm_fold_kernel<<<dim3((unsigned)((N + 63) / 64)), dim3(1024), 0, st>>>(W, bias, gamma, beta, ws + pl.o_wg,
                                                                          (float2*)(ws + pl.o_wc), K, N);
    int rc = folx_launch_status();
    if (rc != FOLX_HIP_OK) return rc;
    norm_rows_kernel<<<dim3((unsigned)((R + 3) / 4)), dim3(256), 0, st>>>(
        x, lap, gamma, beta, ws + pl.o_xhat, ws + pl.o_rs, ws + pl.o_nx, ws + pl.o_nlap, R, K, eps);
    rc = folx_launch_status();
    if (rc != FOLX_HIP_OK) return rc;
    a.W = ws + pl.o_wg; a.xhat = ws + pl.o_xhat; a.rs = ws + pl.o_rs; a.wc = (const float2*)(ws + pl.o_wc);
    a.s1 = ws + pl.o_s1; a.sc = ws + pl.o_sc;
    in_x = ws + pl.o_nx; in_lap = ws + pl.o_nlap;
  }
  // z and the linear part of zl through the plain dense kernel: no Jacobian rows, no residual
  int rc = folx_hip_dense_fwdlap(st, in_x, nullptr, in_lap, W, bias, nullptr, nullptr, nullptr, y, nullptr, y_lap, R,
                                 0, K, N);
  if (rc != FOLX_HIP_OK) return rc;
  if (pre) {
    const int64_t S4 = R * (int64_t)N / 4;
    wide_add_pre_kernel<<<dim3((unsigned)((S4 + 255) / 256)), dim3(256), 0, st>>>(y, y_lap, pre, pre_lap, S4, N / 4,
                                                                              pre_group);
    rc = folx_launch_status();
    if (rc != FOLX_HIP_OK) return rc;
  }
  if (norm)
    return has_act ? launch_wide<true, true, 32>(st, a, pl, y, y_lap) : launch_wide<true, false, 32>(st, a, pl, y, y_lap);
  if (parts) {
    a.parts = *parts;
    return pl.PT == 16 ? launch_wide<false, true, 16, true>(st, a, pl, y, y_lap, res, res_lap)
                       : launch_wide<false, true, 32, true>(st, a, pl, y, y_lap, res, res_lap);
  }
  return pl.PT == 16 ? launch_wide<false, true, 16>(st, a, pl, y, y_lap) : launch_wide<false, true, 32>(st, a, pl, y, y_lap);
}

}  // namespace

int64_t folx_dense_act_wide_ws_bytes(int64_t R, int32_t P, int32_t K, int32_t N) {
  WidePlan pl;
  if (!plan_wide(R, P, K, N, false, true, pl)) return FOLX_HIP_ENOTSUP;
  return pl.ws_bytes;
}

int folx_dense_act_wide(hipStream_t st, int32_t act, float param, const float* x, const float* jac, const float* lap,
                        const float* W, const float* bias, float* y, float* y_jac, float* y_lap, int64_t R,
                        int32_t P, int32_t K, int32_t N, void* workspace, int64_t workspace_bytes) {
  if (act < 0) return FOLX_HIP_ENOTSUP;
  return run_wide(st, false, act, param, x, jac, lap, nullptr, nullptr, 0.0f, W, bias, y, y_jac, y_lap, R, P, K, N,
                  workspace, workspace_bytes);
}

extern "C" int64_t folx_hip_norm_dense_workspace_bytes(int64_t R, int32_t P, int32_t K, int32_t N, int32_t act) {
  if (R < 0 || P < 0 || K <= 0 || N <= 0) return FOLX_HIP_EINVAL;
  WidePlan pl;
  if ((act >= 0 && !act_fused(act)) || !plan_wide(R, P, K, N, true, act >= 0, pl)) return FOLX_HIP_ENOTSUP;
  return pl.ws_bytes;
}

extern "C" int folx_hip_norm_dense_fwdlap(void* stream, int32_t act, float param, const float* x, const float* jac,
                                          const float* lap, const float* gamma, const float* beta, float eps,
                                          const float* W, const float* bias, float* y, float* y_jac, float* y_lap,
                                          int64_t R, int32_t P, int32_t K, int32_t N, void* workspace,
                                          int64_t workspace_bytes) {
  if (R < 0 || P < 0 || K <= 0 || N <= 0) return FOLX_HIP_EINVAL;
  return run_wide((hipStream_t)stream, true, act, param, x, jac, lap, gamma, beta, eps, W, bias, y, y_jac, y_lap, R, P,
                  K, N, workspace, workspace_bytes);
}

extern "C" int folx_hip_dense_act_parts_fwdlap(void* stream, int32_t act, float param, const float* x,
                                               const float* lap, int32_t n_parts, const float* const* jac_parts,
                                               const int32_t* widths, const int32_t* broadcast, int32_t group,
                                               const float* W, const float* bias, const float* res,
                                               const float* res_jac, const float* res_lap, const float* pre,
                                               const float* pre_jac, const float* pre_lap, float* y,
                                               float* y_jac, float* y_lap, int64_t R, int32_t P, int32_t N,
                                               void* workspace, int64_t workspace_bytes) {
  if (R < 0 || P < 0 || N <= 0 || n_parts < 1 || group < 1 || !jac_parts || !widths || !broadcast)
    return FOLX_HIP_EINVAL;
  if ((res != nullptr) != (res_jac != nullptr) || (res != nullptr) != (res_lap != nullptr)) return FOLX_HIP_EINVAL;
  if ((pre != nullptr) != (pre_jac != nullptr) || (pre != nullptr) != (pre_lap != nullptr)) return FOLX_HIP_EINVAL;
  if (!folx_aligned16(res) || !folx_aligned16(res_lap) || !folx_aligned16(pre) || !folx_aligned16(pre_lap))
    return FOLX_HIP_ENOTSUP;
  if (n_parts > MAX_PARTS || act < 0 || R % group != 0) return FOLX_HIP_ENOTSUP;
  WideParts parts;
  parts.n = n_parts;
  parts.group = group;
  int32_t K = 0;
  for (int i = 0; i < n_parts; ++i) {
    if (widths[i] <= 0 || widths[i] % BK != 0) return FOLX_HIP_ENOTSUP;
    if (!jac_parts[i]) return FOLX_HIP_EINVAL;
    if (!folx_aligned16(jac_parts[i])) return FOLX_HIP_ENOTSUP;
    parts.jac[i] = jac_parts[i];
    parts.width[i] = widths[i];
    parts.bcast[i] = broadcast[i] ? 1 : 0;
    parts.pstride[i] = (broadcast[i] ? R / group : R) * (int64_t)widths[i];
    K += widths[i];
    parts.kend[i] = K;
  }
  for (int i = n_parts; i < MAX_PARTS; ++i) {
    parts.jac[i] = nullptr; parts.width[i] = 0; parts.bcast[i] = 0; parts.pstride[i] = 0; parts.kend[i] = K;
  }
  return run_wide((hipStream_t)stream, false, act, param, x, nullptr, lap, nullptr, nullptr, 0.0f, W, bias, y, y_jac,
                  y_lap, R, P, K, N, workspace, workspace_bytes, &parts, res, res_jac, res_lap, pre, pre_jac, pre_lap,
                  group);
}

// ---- folx_hip_norm_dense_fwdlap on the library's own scratch memory -------------------------
//
// For callers that cannot bring a workspace because they cannot allocate one (code under HIP
// graph capture, tight serving loops).  The workspace of run_wide() is a file-scope device
// array; every GPU the library runs on holds its own copy of it, at its own address, until the
// process ends.  In host code the array's name is only a handle of the symbol, so the device
// address is asked for once per device (hipGetSymbolAddress, with that device current) and
// kept; everything below uses the pointer, never the name.
namespace {

constexpr int64_t SCRATCH_BYTES = FOLX_HIP_STATIC_SCRATCH_BYTES;
constexpr int MAX_DEVICES = 64;

}  // namespace

static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

namespace {

void* g_scratch_ptr[MAX_DEVICES];  // device address of `scratch` on each device, once known
std::mutex g_scratch_mutex;

// Address of this device's copy of `scratch`; nullptr when the runtime refuses.
void* scratch_of_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

}  // namespace

extern "C" int folx_hip_norm_dense_static_fwdlap(void* stream, int32_t act, float param, const float* x,
                                                 const float* jac, const float* lap, const float* gamma,
                                                 const float* beta, float eps, const float* W, const float* bias,
                                                 float* y, float* y_jac, float* y_lap, int64_t R, int32_t P,
                                                 int32_t K, int32_t N) {
  if (R < 0 || P < 0 || K <= 0 || N <= 0) return FOLX_HIP_EINVAL;
  WidePlan pl;
  if ((act >= 0 && !act_fused(act)) || !plan_wide(R, P, K, N, true, act >= 0, pl)) return FOLX_HIP_ENOTSUP;
  if (pl.ws_bytes > SCRATCH_BYTES) return FOLX_HIP_ESCRATCH;
  void* ptr = scratch_of_current_device();
  if (!ptr) return FOLX_HIP_ELAUNCH;
  // Nothing in the workspace has to start at zero: every launch of run_wide() writes the part
  // it owns (folded weights, per-position rows, one slab of sums per group of Jacobian rows)
  // in full before a later launch on the same stream reads it.
  return run_wide((hipStream_t)stream, true, act, param, x, jac, lap, gamma, beta, eps, W, bias, y, y_jac, y_lap, R, P,
                  K, N, ptr, SCRATCH_BYTES);
}
