// slogdet rule for many small matrices with dense Jacobians (n <= 32).
//
// A wavefront owns one n x n matrix (two for n <= 8):
//   1. Gauss-Jordan with partial pivoting on [A | I] in registers (lane j holds column j,
//      smallmat.h) gives A^-1; the pivots give sign and log|det| (the same pivot sequence
//      as an LU with partial pivoting).
//   2. For every Jacobian row p: A_jac[p] goes from global memory straight into MFMA
//      operand registers (rows are requested several rows ahead), M = A^-1 A_jac[p] on the
//      matrix cores, ld_jac[p] = tr M from the lane-wise product of the operands, and
//      sum_p tr(M M) from M and its transpose.
//   3. tr(A^-1 lap_A) from the same operand registers.
// The matrices may be strided: a stack [batch][row][member][column] is read in place.
// The Jacobian is read exactly once.
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

constexpr int TRB = 16;  // Jacobian rows whose traces are reduced together

// 16 < n <= 32: one 32 x 32 tile (v_mfma_f32_32x32x2_f32) per wavefront.  Lane l holds, for step
// t, the element (k = 2 t + l / 32, lr = l % 32) of an operand: as A operand that is row lr,
// column k; as B operand row k, column lr.  With a[t] = Ainv[lr][k] and j[t] = J[k][lr]:
//   mfma(a, j) accumulates M = Ainv J      (A = Ainv,  B = J)
// and tr M = sum over lanes and steps of a[t] j[t].  The transpose that tr(M M) = sum_ab M[a][b] M[b][a]
// needs comes back through LDS.  (It could be had as a second product of the SAME registers, mfma(j, a) =
// J^T Ainv^T, without any data movement -- but then the kernel is bound by the matrix pipe: two 32 x 32 x 32
// products per 4 KB row are 64 flop per byte, three times the ridge of the FP32 matrix peak over HBM.)
__global__ __launch_bounds__(FOLX_WAVE, 3) void slogdet32_kernel(
    const float* __restrict__ A, const float* __restrict__ AJ, const float* __restrict__ AL,
    float* __restrict__ sign_out, float* __restrict__ logdet_out, float* __restrict__ jac_out,
    float* __restrict__ lap_out, int64_t NM, int32_t n, int32_t P, int64_t ND, int64_t bstride, int64_t dstride,
    int64_t rstride, int64_t slice) {
  constexpr int NP = 32, STEPS = 16;
  constexpr int AUGS = smallmat::Aug<NP>::stride;  // row stride of the augmented matrix
  constexpr int MTS = 36;  // row stride of the tile that hands M^T back
  __shared__ __attribute__((aligned(16))) float aug[NP * AUGS];
  __shared__ float trs[TRB][FOLX_WAVE + 1];
  static_assert(MTS <= AUGS, "the tile of M reuses the memory of the augmented matrix");
  float* const mt = aug;  // the augmented matrix is dead once Ainv sits in registers

  const int lane = threadIdx.x;
  const int64_t m = blockIdx.x;
  // matrix m = (batch m / ND, member m % ND); element (i, j) at base + i * rstride + j
  const int64_t base = (m / ND) * bstride + (m % ND) * dstride;

  float logdet, sgn;
  smallmat::gauss_jordan<NP>(aug, A + base, n, lane, logdet, sgn, rstride);
  float tl = smallmat::trace_inv_times<NP>(aug, AL + base, n, lane, rstride);

  // this lane's elements (k, lr) of the padded tile
  const int lr = lane % 32;
  const int lq = lane / 32;
  float ainv[STEPS];
  int32_t eoff[STEPS];  // offsets inside one matrix fit 32 bits (checked by the launcher)
#pragma unroll
  for (int t = 0; t < STEPS; ++t) {
    const int k = 2 * t + lq;
    const bool ok = k < n && lr < n;
    // elements of the padding ask for element (0, 0): loads are never branched around, so
    // that all of them are in flight before the first wait.  What they bring in needs no masking:
    // in M = Ainv J it meets the zero rows and columns of the padded Ainv, or lands in columns b >= n
    // of M, which tr(M M) pairs with the zero rows M[b][.] and tr M never reads.
    eoff[t] = ok ? (int32_t)(k * rstride) + lr : 0;
    ainv[t] = ok ? aug[lr * AUGS + NP + k] : 0.0f;  // Ainv[lr][k]
  }

  float mm = 0.0f;
  float raw0[STEPS], raw1[STEPS];  // two Jacobian rows on their way
  auto request = [&](int p, float (&raw)[STEPS]) __attribute__((always_inline)) {
    const float* src = AJ + (int64_t)p * slice + base;
#pragma unroll
    for (int t = 0; t < STEPS; ++t) raw[t] = src[eoff[t]];  // A_jac[p][k][lr], padding masked when used
  };
  // One product per row, M = Ainv J in accumulator layout (lane (b, h), register 4 g + j <-> M[8 g + 4 h + j][b]);
  // tr(M M) = sum_ab M[a][b] M[b][a] takes M^T back from LDS: the tile is written row-major (row stride 36:
  // the 128-bit reads of 16 lanes then fall on distinct banks) and lane (b, h) reads M[b][8 g + 4 h .. + 3].
  // LDS serves a wavefront's accesses in issue order, so the round trip needs no barrier.
  auto do_row = [&](int p, const float (&raw)[STEPS]) __attribute__((always_inline)) {
    floatx16 c;
#pragma unroll
    for (int r = 0; r < 16; ++r) c[r] = 0.0f;
    float tr = 0.0f;
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      c = __builtin_amdgcn_mfma_f32_32x32x2f32(ainv[t], raw[t], c, 0, 0, 0);  // M = Ainv J
      tr = fmaf(ainv[t], raw[t], tr);                                        // this lane's part of tr M
    }
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < 16; ++r) mt[(8 * (r / 4) + 4 * lq + r % 4) * MTS + lr] = c[r];
    asm volatile("" ::: "memory");
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 t4 = *reinterpret_cast<const float4*>(&mt[lr * MTS + 8 * g + 4 * lq]);
      mm = fmaf(c[4 * g + 0], t4.x, mm);
      mm = fmaf(c[4 * g + 1], t4.y, mm);
      mm = fmaf(c[4 * g + 2], t4.z, mm);
      mm = fmaf(c[4 * g + 3], t4.w, mm);
    }
    asm volatile("" ::: "memory");
    return tr;
  };
  if (P > 0) request(0, raw0);
  if (P > 1) request(1, raw1);
  for (int p = 0; p < P; ++p) {
    float tr;
    if (p % 2 == 0) {
      tr = do_row(p, raw0);
      if (p + 2 < P) request(p + 2, raw0);
    } else {
      tr = do_row(p, raw1);
      if (p + 2 < P) request(p + 2, raw1);
    }
    trs[p % TRB][lane] = tr;
    if ((p + 1) % TRB == 0 || p + 1 == P) {
      // ld_jac of the last rows: four lanes per row add up 16 of its 64 parts each.
      // The workgroup is one wavefront and LDS serves a wavefront's accesses in issue
      // order, so the other lanes' writes above are seen without a barrier; a barrier's
      // fence would also wait for the Jacobian row requested ahead.
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
  mm = wave_sum(mm);
  tl = wave_sum(tl);
  if (lane == 0) {
    sign_out[m] = sgn;
    logdet_out[m] = logdet;
    lap_out[m] = tl - mm;
  }
}

// n <= 16: one 16 x 16 MFMA tile per wavefront, holding one matrix (NP = 16) or two 8 x 8 matrices
// on its diagonal blocks (NP = 8: the operands are [Ainv_0; Ainv_1] and [J_0 | J_1], K = 8, and
// only the diagonal blocks of the product are used).  Lane l holds, for step t, the element
// (k = 4 t + l / 16, column l % NP) of matrix (l % 16) / NP.  Per Jacobian row:
//   M = Ainv J      NP / 4 MFMA steps (the matrix pipe and the vector ALU do not overlap on a
//                   SIMD, so the second product M^T of the 32 x 32 kernel above is not formed),
//   tr M            lane-wise products of the operands, summed 16 rows at a time through LDS,
//   tr(M M)         M goes to LDS transposed (one 128-bit write per lane) and comes back as M^T in
//                   the accumulator layout; the product with the previous row's M is taken
//                   while this row's MFMAs run.
// Rows are requested D rows ahead with scalar base + 32-bit lane offset addressing.
constexpr int SLD_WPB = 4;  // wavefronts per workgroup

template <int NP, bool HAS_F, int KFT = KF>
__global__ __launch_bounds__(FOLX_WAVE * SLD_WPB, 4) void slogdet16_kernel(
    const float* __restrict__ A, const float* __restrict__ AJ, const float* __restrict__ AL,
    float* __restrict__ sign_out, float* __restrict__ logdet_out, float* __restrict__ jac_out,
    float* __restrict__ lap_out, int64_t NM, int32_t n, int32_t P, int64_t ND, int64_t bstride, int64_t dstride,
    int64_t rstride, int64_t slice, int32_t share, Factor fc) {
  constexpr int G = 16 / NP;      // matrices per wavefront
  constexpr int STEPS = NP / 4;   // MFMA steps = elements per lane
  constexpr int AUGS = smallmat::Aug<NP>::stride;
  constexpr int TS = 20;          // row stride of the transposed product in LDS (floats)
  constexpr int TRN = 8;          // Jacobian rows whose traces are reduced together
  // per wavefront: [A | I] during the elimination; afterwards the transposed product and the
  // staged trace parts take its place
  constexpr int WS = 16 * TS + TRN * (FOLX_WAVE + 1);
  static_assert(G * smallmat::Aug<NP>::size <= WS && WS % 4 == 0, "LDS overlay");
  __shared__ __attribute__((aligned(16))) float ws_all[SLD_WPB][WS];
  __shared__ float fst_all[HAS_F ? SLD_WPB : 1][HAS_F ? 2 * KFT : 1][STEPS][FOLX_WAVE];

  // The wavefronts of a workgroup work on neighbouring matrices and do not share data; they are
  // one workgroup so that they start together and (with a barrier every D rows) stay together:
  // where members lie side by side along the matrix rows, the pieces of a row that the SLD_WPB
  // wavefronts ask for at about the same time are then one contiguous stretch of memory.
  const int lane = threadIdx.x % FOLX_WAVE, wv = folx_wave_id();
  float* aug = ws_all[wv];
  float* mt = ws_all[wv];
  float (*trs)[FOLX_WAVE + 1] = reinterpret_cast<float (*)[FOLX_WAVE + 1]>(ws_all[wv] + 16 * TS);
  // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  When `share`
  // neighbouring workgroups read the same 128-byte lines (rows of n floats side by side), they
  // are given to the same XCD in consecutive slots, so that every line comes from HBM once.
  const int64_t NW = (NM + G - 1) / G;
  int64_t wg = blockIdx.x;
  if (share > 1) {
    const int64_t chunk = 8 * (int64_t)share;
    const int64_t c = wg / chunk, r = wg % chunk;
    if ((c + 1) * chunk <= gridDim.x) wg = c * chunk + (r % 8) * share + r / 8;
  }
  const int64_t w = wg * SLD_WPB + wv;
  // a wavefront past the end goes through the motions on matrix 0 (it has to meet the others at
  // the barriers) and stores nothing
  const bool wvalid = w < NW;
  const int64_t m0 = wvalid ? w * G : 0;  // first matrix of this wavefront
  auto matrix_base = [&](int64_t m) -> int64_t { return (m / ND) * bstride + (m % ND) * dstride; };
  const int64_t base0 = matrix_base(m0);  // the same for all lanes

  // tile mapping
  const int lr = lane % 16, lq = lane / 16;
  const int g = lr / NP, cl = lr % NP;
  const int64_t mm_ = m0 + g;  // this lane's matrix
  const bool mvalid = wvalid && mm_ < NM;
  const int64_t base = mvalid ? matrix_base(mm_) : base0;
  const uint32_t delta = (uint32_t)(base - base0);  // the launcher checks sign and range
  bool ok[STEPS];
  uint32_t eoff[STEPS], boff[STEPS];  // element offset inside the matrix, byte offset from base0
#pragma unroll
  for (int t = 0; t < STEPS; ++t) {
    const int k = 4 * t + lq;
    ok[t] = mvalid && k < n && cl < n;
    // elements of the padding ask for element (0, 0) of the first matrix: loads are never
    // branched around.  What they bring in meets a zero of A^-1 in every product below.
    eoff[t] = ok[t] ? (uint32_t)(k * rstride + cl) : 0u;
    boff[t] = ok[t] ? 4u * (delta + eoff[t]) : 0u;
  }
  // Jacobian rows are requested D rows ahead: with one row in flight per wavefront the kernel
  // would be bound by the latency of its own loads, not by HBM bandwidth.  The first D rows are
  // asked for before the elimination, which touches no memory after its own loads.
  constexpr int D = 8;
  float raw[D][STEPS];
  auto request = [&](float (&dst)[STEPS], int p) __attribute__((always_inline)) {
    const char* src = reinterpret_cast<const char*>(AJ + (int64_t)p * slice + base0);  // the same for all lanes
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      // the 32-bit offset is made opaque here so that it is widened next to the load, which then
      // takes the scalar base + lane offset form (no 64-bit address arithmetic per load)
      uint32_t o = boff[t];
      asm volatile("" : "+v"(o));
      dst[t] = *reinterpret_cast<const float*>(src + o);  // A_jac[p][k][cl] of this lane's matrix
    }
  };
#pragma unroll
  for (int d = 0; d < D; ++d)
    if (d < P) request(raw[d], d);


  // elimination: lane mapping of smallmat (NP = 8: lanes 16 g .. 16 g + 15 work on matrix g)
  float logdet, sgn;
  if constexpr (G == 1) {
    smallmat::gauss_jordan<NP>(aug, A + base0, n, lane, logdet, sgn, rstride, HAS_F ? fc.x + base0 : nullptr);
  } else {
    const int64_t mg = m0 + lane / 16;
    const bool valid = wvalid && lane / 16 < G && mg < NM;
    const int64_t bg = valid ? matrix_base(mg) : base0;
    smallmat::gauss_jordan_groups<NP, G>(aug, A + bg, valid, n, lane, logdet, sgn, rstride,
                                         HAS_F ? fc.x + bg : nullptr);
    if (valid && lane % 16 == 0) {
      sign_out[mg] = sgn;
      logdet_out[mg] = logdet;
    }
  }

  float ainv[STEPS];
#pragma unroll
  for (int t = 0; t < STEPS; ++t)  // Ainv[cl][k]
    ainv[t] = ok[t] ? aug[g * smallmat::Aug<NP>::size + cl * AUGS + NP + 4 * t + lq] : 0.0f;
  // With a factor: F and A at this lane's elements stay in registers; the factor's sparse Jacobian
  // rows and their dense row numbers, needed for a few rows only, wait in LDS (fst[2 s][t][lane] row
  // number, fst[2 s + 1][t][lane] value).
  constexpr int EF = HAS_F ? STEPS : 1;
  float fx[EF], ax[EF], lapx[EF];
  int flo[EF], fhi[EF];
  if constexpr (HAS_F) {
    float (*fst)[STEPS][FOLX_WAVE] = fst_all[wv];
    const int64_t wpos = base % fc.S_w;  // position of the matrix inside its walker's elements
    float fj[KFT][STEPS];
    int32_t fidx[KFT][STEPS];
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      const int64_t off = base + eoff[t];
      int64_t q = wpos + eoff[t];  // eoff < S_w (checked by the launcher)
      q = q >= fc.S_w ? q - fc.S_w : q;
      fx[t] = fc.x[off];
      ax[t] = A[off];
      lapx[t] = 0.0f;
#pragma unroll
      for (int sl = 0; sl < KFT; ++sl) {
        fidx[sl][t] = -1;
        fj[sl][t] = 0.0f;
        if (sl < fc.kf) {  // the same for all lanes
          fidx[sl][t] = fc.idx[(int64_t)sl * fc.S_w + q];
          fj[sl][t] = fc.jac[(int64_t)sl * slice + off];
        }
      }
    }
#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      fx[t] = ok[t] ? fx[t] : 0.0f;
      ax[t] = ok[t] ? ax[t] : 0.0f;
      int mn = 0x7fffffff, mx = -1;
#pragma unroll
      for (int sl = 0; sl < KFT; ++sl) {
        const int32_t id = ok[t] ? fidx[sl][t] : -1;
        fst[2 * sl][t][lane] = __int_as_float(id);
        fst[2 * sl + 1][t][lane] = id >= 0 ? fj[sl][t] : 0.0f;
        mn = id >= 0 ? min(mn, id) : mn;
        mx = max(mx, id);
      }
      // Rows of the dense Jacobian that the factor's slots of step t stand for, over the whole
      // wavefront: the range test in the loop is scalar, so a row outside [flo, fhi] costs one
      // multiplication per element and no compares.
#pragma unroll
      for (int off = FOLX_WAVE / 2; off > 0; off >>= 1) {
        mn = min(mn, __shfl_xor(mn, off, FOLX_WAVE));
        mx = max(mx, __shfl_xor(mx, off, FOLX_WAVE));
      }
      flo[t] = __builtin_amdgcn_readfirstlane(mn);
      fhi[t] = __builtin_amdgcn_readfirstlane(mx);
    }
  }

  float mm = 0.0f;
  floatx4 cp;  // M of the previous row
#pragma unroll
  for (int r = 0; r < 4; ++r) cp[r] = 0.0f;
  const int mt_w = lr * TS + 4 * lq;   // M[4 lq + r][lr] -> transposed tile, row lr, columns 4 lq + r
  const int mt_r = 4 * lq * TS + lr;   // M^T[4 lq + r][lr] = transposed tile row 4 lq + r, column lr
  // sum_ab M[a][b] M^T[a][b] of the row whose M is in cp (LDS serves the one wavefront's accesses
  // in issue order: no barrier between the write and the reads)
  auto square_trace = [&]() __attribute__((always_inline)) {
    *reinterpret_cast<floatx4*>(&mt[mt_w]) = cp;
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < 4; ++r) mm = fmaf(cp[r], mt[mt_r + r * TS], mm);
    asm volatile("" ::: "memory");
  };
  for (int p0 = 0; p0 < P; p0 += D) {
    __builtin_amdgcn_s_barrier();  // no fence: nothing is shared, and the rows requested ahead stay in flight
#pragma unroll
    for (int d = 0; d < D; ++d) {
      int p = p0 + d;
      asm volatile("" : "+s"(p));  // a scalar of its own: compared with directly, not through p0 - index
      if (p < P) {
        float jv[STEPS];
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
          float v = raw[d][t];
          if constexpr (HAS_F) {
            const float rv = v;
            v = fx[t] * rv;
            if (p >= flo[t] && p <= fhi[t]) {  // the same for all lanes
              float add = 0.0f;
#pragma unroll
              for (int sl = 0; sl < KFT; ++sl)
                add += __float_as_int(fst_all[wv][2 * sl][t][lane]) == p ? fst_all[wv][2 * sl + 1][t][lane] : 0.0f;
              lapx[t] = fmaf(2.0f * rv, add, lapx[t]);  // cross term 2 dA . dF of the product's Laplacian
              v = fmaf(ax[t], add, v);
            }
          }
          jv[t] = v;
        }
        if (p + D < P) request(raw[d], p + D);
        floatx4 c;
#pragma unroll
        for (int r = 0; r < 4; ++r) c[r] = 0.0f;
        float tr = 0.0f;
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(ainv[t], jv[t], c, 0, 0, 0);  // M = Ainv J
          tr = fmaf(ainv[t], jv[t], tr);                                       // this lane's part of tr M
        }
        // tr(M M) of the previous row, while this row's products are in the matrix pipe
        square_trace();
        cp = c;
        trs[p % TRN][lane] = tr;
        if ((p + 1) % TRN == 0 || p + 1 == P) {
          // ld_jac of the last rows: eight lanes per row add up 8 of its 64 parts each; the eight
          // lanes of a part belong to one matrix (NP = 8: part % 2).  LDS serves a wavefront's
          // accesses in issue order, so the other lanes' writes above are seen without a
          // barrier; a barrier's fence would also wait for the rows requested ahead.
          const int pb = p / TRN * TRN, pe = p + 1 - pb;
          asm volatile("" ::: "memory");
          const int row = lane % TRN, part = lane / TRN;
          float sm = 0.0f;
#pragma unroll
          for (int l = 0; l < 8; ++l) sm += trs[row][part * 8 + l];
          if constexpr (G == 1) sm += __shfl_xor(sm, 8, FOLX_WAVE);
          sm += __shfl_xor(sm, 16, FOLX_WAVE);
          sm += __shfl_xor(sm, 32, FOLX_WAVE);
          if (wvalid && part < G && row < pe && m0 + part < NM) jac_out[(int64_t)(pb + row) * NM + m0 + part] = sm;
          asm volatile("" ::: "memory");
        }
      }
    }
  }
  square_trace();  // the last row
  if constexpr (G == 2) mm = (lq / 2 == g) ? mm : 0.0f;  // only the diagonal blocks belong to a matrix

  // tr(A^-1 lap A), with a factor lap (A F) = F lap A + A lap F + the cross term collected above
  float tl = 0.0f;
#pragma unroll
  for (int t = 0; t < STEPS; ++t) {
    const int64_t off = base + eoff[t];
    float al = AL[off];
    if constexpr (HAS_F) al = fx[t] * al + ax[t] * fc.lap[off] + lapx[t];
    tl += ainv[t] * al;  // sum A^-1[cl][k] lap A[k][cl]; ainv is zero at the padding
  }
  float res = tl - mm;
  // sum over the lanes of one matrix: all of them (NP = 16) or those with the same lr / 8
#pragma unroll
  for (int off = 1; off < FOLX_WAVE; off <<= 1)
    if (G == 1 || off != 8) res += __shfl_xor(res, off, FOLX_WAVE);
  if constexpr (G == 1) {
    if (wvalid && lane == 0) {
      sign_out[m0] = sgn;
      logdet_out[m0] = logdet;
      lap_out[m0] = res;
    }
  } else {
    if (lq == 0 && cl == 0 && mvalid) lap_out[mm_] = res;
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
  dim3 block(FOLX_WAVE);
  if (n > 16) {
    if (fc) return FOLX_HIP_ENOTSUP;
    if ((int64_t)(n - 1) * row_stride + n > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
    slogdet32_kernel<<<dim3((unsigned)NM), block, 0, st>>>(A, A_jac, A_lap, sign, logdet, ld_jac, ld_lap, NM, n, P, ND,
                                                           batch_stride, member_stride, row_stride, jac_stride);
    return folx_launch_status();
  }
  // n <= 16: lane offsets inside a wavefront's matrices are 32-bit, counted from its first matrix
  const int G = n <= 8 ? 2 : 1;
  if (row_stride < 0 || (int64_t)n * row_stride >= (1LL << 29)) return FOLX_HIP_ENOTSUP;
  if (G == 2 && (batch_stride < 0 || member_stride < 0 || batch_stride < (ND - 1) * member_stride ||
                 batch_stride + member_stride >= (1LL << 29)))
    return FOLX_HIP_ENOTSUP;
  const int64_t NW = (NM + G - 1) / G;
  dim3 grid((unsigned)((NW + SLD_WPB - 1) / SLD_WPB));
  block = dim3(FOLX_WAVE * SLD_WPB);
  // members stored side by side along the rows with rows shorter than a 128-byte line: the
  // wavefronts that read the same lines run on the same XCD
  int32_t share = 1;
  if (member_stride == n && n * 4 < 128 && ND > 1) {
    share = 128 / (n * 4);
    while (share > 1 && ND % share != 0) share /= 2;
    share /= G * SLD_WPB;
    if (share < 1) share = 1;
  }
#define FOLX_SLD_LAUNCH(NPV, HASF, KFV)                                                                     \
  slogdet16_kernel<NPV, HASF, KFV><<<grid, block, 0, st>>>(A, A_jac, A_lap, sign, logdet, ld_jac, ld_lap, NM, n, P, \
                                                           ND, batch_stride, member_stride, row_stride, jac_stride, \
                                                           share, fc ? *fc : Factor{})
  if (fc) {
    // three slots (the coordinates of one electron) need a quarter less LDS than four
    const bool three = fc->kf <= 3;
    if (n <= 8) { if (three) FOLX_SLD_LAUNCH(8, true, 3); else FOLX_SLD_LAUNCH(8, true, KF); }
    else { if (three) FOLX_SLD_LAUNCH(16, true, 3); else FOLX_SLD_LAUNCH(16, true, KF); }
  } else {
    if (n <= 8) FOLX_SLD_LAUNCH(8, false, KF);
    else FOLX_SLD_LAUNCH(16, false, KF);
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
  if ((int64_t)(n - 1) * row_stride + n > walker_elems) return FOLX_HIP_ENOTSUP;  // a matrix lies inside one walker
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
