// Narrow dense layer and its activation in one pass:
//   z = x @ W + bias          y     = f(z)
//   zj[p] = jac[p] @ W        yj[p] = f'(z) * zj[p]
//   zl = lap @ W              yl    = f'(z) * zl + f''(z) * sum_p zj[p]^2
// for K, N <= 128.  The pre-activation triplet never goes to HBM: the layer reads its input
// triplet once and writes its output triplet once, which is what bounds a layer this narrow.
//
// A workgroup of 4 wavefronts owns BR consecutive rows (positions) and ALL N columns, and walks
// the operand one Jacobian row at a time: x first (which gives f' and f'' for its rows, kept
// in registers), then its Jacobian rows (scaled by f' on the way out, squares summed in
// registers), then lap.  The BR x K input tile of one step is contiguous in memory and goes
// straight into LDS (global_load_lds_dwordx4), double buffered.  W never touches LDS: each
// wavefront owns a strip of 32 columns and keeps its K x 32 slice of W in registers as
// ready-made MFMA operands (v_mfma_f32_32x32x2_f32; lane l, register (j, i) <-> k = 8 j +
// 4 (l / 32) + i, column l % 32, matching the 128-bit reads of the A tile).
//
// LDS layout of the tile: [row][K / 4 pieces of 16 bytes]; piece c of row m sits at slot
// c ^ rot(m), with rot chosen from the power of two in K / 4 so that 16 consecutive rows reading
// the same k land on different banks (no rotation when K / 4 is odd, e.g. K = 100).
//
// When there are few row tiles (a small batch) the Jacobian rows are split over G workgroups
// per row tile in a first launch, each of which leaves its partial sums of squares in the
// workspace; a second, short launch with one workgroup per row tile recomputes f' and f''
// from the x tile, adds the partials in a fixed order and produces the lap row.
#include <type_traits>

#include "activations.h"
#include "dense_act_wide.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(1))) char gchar;    // global memory, so that stores stay global_store
typedef __attribute__((address_space(1))) float gfloat;

#define FOLX_GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define FOLX_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

constexpr int NTHR = 256;
constexpr int TM = 1;                 // 32-row accumulator tiles per wavefront
constexpr int TILE_FLOATS = 4096;     // one LDS buffer
constexpr int MAXLD = TILE_FLOATS / 4 / NTHR;
constexpr int PART_PER_BLOCK = TM * 16 * NTHR;

struct DAParams {
  const float *x, *jac, *lap, *W, *bias;
  const float *res, *res_jac, *res_lap;  // optional triplet of the output's shape added to the activated result
  float *y, *y_jac, *y_lap;
  float* part;
  int64_t R;
  int32_t P, K, N, G, PG, act, mode;  // mode 0: whole rule, 1: x + Jacobian rows of one group, 2: lap from partials
  float prm;
};

struct DAPlan {
  int wc, ks, br;
  int64_t row_tiles;
  int32_t G, PG;
  int64_t ws_bytes;
};

// Returns false when the shape is outside what the kernel is built for.
bool plan_dense_act(int64_t R, int32_t P, int32_t K, int32_t N, DAPlan& pl) {
  if (K < 4 || K > 128 || K % 4 != 0 || N < 1 || N > 128) return false;
  pl.wc = (N <= 32 && K <= 32) ? 1 : ((N <= 64 && K <= 64) ? 2 : 4);
  pl.ks = K <= 8 ? 1 : (K <= 32 ? 4 : (K <= 64 ? 8 : (K <= 104 ? 13 : 16)));
  pl.br = 32 * TM * (4 / pl.wc);
  pl.row_tiles = (R + pl.br - 1) / pl.br;
  int64_t G = 1;
  if (pl.row_tiles > 0 && pl.row_tiles < 384) {
    G = 512 / pl.row_tiles;
    int64_t gmax = P / 8;
    if (G > gmax) G = gmax;
    if (G < 1) G = 1;
  }
  pl.G = (int32_t)G;
  pl.PG = (int32_t)((P + G - 1) / G);
  pl.G = pl.PG > 0 ? (P + pl.PG - 1) / pl.PG : 1;  // no empty group
  if (pl.row_tiles * pl.G > 0x7fffffffLL) return false;
  pl.ws_bytes = pl.G > 1 ? pl.row_tiles * pl.G * (int64_t)PART_PER_BLOCK * 4 : 0;
  return true;
}

template <int KS, int WC>
__global__ __launch_bounds__(NTHR, 2) void dense_act_kernel(DAParams a) {
  constexpr int WR = 4 / WC;
  constexpr int BR = 32 * TM * WR;
  __shared__ __attribute__((aligned(16))) float As0[TILE_FLOATS];
  __shared__ __attribute__((aligned(16))) float As1[TILE_FLOATS];

  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int l32 = lane % 32;
  const int lh = lane / 32;
  const int wrow = (wave / WC) * 32 * TM;
  const int wcol = (wave % WC) * 32;
  const int K = a.K, N = a.N, G = a.G;
  const int npr = K / 4;
  const int64_t R = a.R;
  const int mode = a.mode;
  const int64_t rt = mode == 1 ? blockIdx.x / G : blockIdx.x;
  const int g = mode == 1 ? (int)(blockIdx.x % G) : 0;
  const int64_t r0 = rt * BR;
  const int p0 = g * a.PG;
  const int p1 = mode == 1 ? min(a.P, p0 + a.PG) : a.P;
  const int nJ = mode == 2 ? 0 : p1 - p0;
  const int n_iter = 1 + nJ + (mode != 1 ? 1 : 0);

  // bank rotation of the tile rows
  int sh = __builtin_ctz(npr);
  if (sh > 4) sh = 4;
  const int rshift = 4 - sh;
  const int rmask = (1 << sh) - 1;
  const int sw = (l32 >> rshift) & rmask;

  // which 16 bytes of the tile each lane asks for; lane i of a load lands at slot (wave base + i)
  const int pieces = BR * npr;  // a multiple of 64
  int32_t src_off[MAXLD];
#pragma unroll
  for (int i = 0; i < MAXLD; ++i) {
    const int q = i * NTHR + tid;
    int off = 0;
    if (q < pieces) {
      int m = q / npr;
      const int c = (q - m * npr) ^ ((m >> rshift) & rmask);
      if (r0 + m >= R) m = (int)(R - 1 - r0);
      off = m * K + 4 * c;
    }
    src_off[i] = off;
  }
  auto tile_src = [&](int it) __attribute__((always_inline)) -> const float* {
    if (it == 0) return a.x + r0 * K;
    if (it <= nJ) return a.jac + ((int64_t)(p0 + it - 1) * R + r0) * K;
    return a.lap + r0 * K;
  };
  auto issue = [&](const float* src, float* buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < MAXLD; ++i)
      if (i * NTHR + wave * 64 < pieces)
        __builtin_amdgcn_global_load_lds(FOLX_GPTR(src + src_off[i]), FOLX_LPTR(&buf[(i * NTHR + wave * 64) * 4]),
                                         16, 0, 0);
  };

  // this wavefront's slice of W as MFMA operands
  const int col = wcol + l32;
  const bool col_ok = col < N;
  float wreg[KS][4];
#pragma unroll
  for (int j = 0; j < KS; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = 8 * j + 4 * lh + i;
      wreg[j][i] = (k < K && col_ok) ? a.W[(int64_t)k * N + col] : 0.0f;
    }
  const float bcol = (a.bias != nullptr && col_ok) ? a.bias[col] : 0.0f;

  const int arow0 = (wrow + l32) * K;
  auto compute = [&](const float* buf, floatx16 (&acc)[TM]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < TM; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;
    // Every group of 8 k is multiplied, also past K: a lane whose 4 k lie past K reads the last
    // 4 k of its own row instead and meets zeros in the W registers, so the product is one
    // straight run of LDS reads and MFMAs with no test on the data, and no row ever sees
    // another row's values.  The reads run one group ahead of the MFMAs.
    auto frag = [&](int j, float4 (&av)[TM]) __attribute__((always_inline)) {
      const int ch = min(2 * j + lh, npr - 1);
#pragma unroll
      for (int t = 0; t < TM; ++t)
        av[t] = *reinterpret_cast<const float4*>(&buf[arow0 + t * 32 * K + ((ch ^ sw) * 4)]);
    };
    float4 av[2][TM];
    frag(0, av[0]);
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      if (j + 1 < KS) frag(j + 1, av[(j + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int t = 0; t < TM; ++t) {
          const float4& q = av[j & 1][t];
          const float v = i == 0 ? q.x : (i == 1 ? q.y : (i == 2 ? q.z : q.w));
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(v, wreg[j][i], acc[t], 0, 0, 0);
        }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Register r of a 32x32 accumulator tile holds row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32.
  // The rows are stored in increasing order through one running row pointer: its steps are
  // N and 5 N floats, and the pointer is made opaque after each step so that the 32 row
  // addresses are not turned into 32 loop-invariant offsets held in registers.
  const bool full = r0 + BR <= R;
  const uint32_t voff = (uint32_t)((4 * lh * N + l32) * 4);
  const int64_t step1 = (int64_t)N * 4, step5 = (int64_t)N * 20;
  auto store_impl = [&](float* out_rows /* row r0 of the output */, const float* res_rows, auto&& value, auto has_res)
      __attribute__((always_inline)) {
    if (!col_ok) return;
    gchar* rowp = (gchar*)(out_rows + (int64_t)wrow * N + wcol);
    const gchar* resp = nullptr;
    if constexpr (decltype(has_res)::value) resp = (const gchar*)(res_rows + (int64_t)wrow * N + wcol);
    if (full) {
#pragma unroll
      for (int t = 0; t < TM; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float v = value(t, r);
          if constexpr (decltype(has_res)::value) v += *(const gfloat*)(resp + voff);
          *(gfloat*)(rowp + voff) = v;
          const int64_t st = (r % 4 == 3) ? step5 : step1;
          rowp += st;
          asm volatile("" : "+s"(rowp));
          if constexpr (decltype(has_res)::value) {
            resp += st;
            asm volatile("" : "+s"(resp));
          }
        }
    } else {
#pragma unroll
      for (int t = 0; t < TM; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = t * 32 + 8 * (r / 4) + r % 4;
          if (r0 + wrow + row + 4 * lh < R) {
            float v = value(t, r);
            if constexpr (decltype(has_res)::value) v += *(const gfloat*)(resp + voff);
            *(gfloat*)(rowp + voff) = v;
          }
          const int64_t st = (r % 4 == 3) ? step5 : step1;
          rowp += st;
          asm volatile("" : "+s"(rowp));
          if constexpr (decltype(has_res)::value) {
            resp += st;
            asm volatile("" : "+s"(resp));
          }
        }
    }
  };
  // res_rows = row r0 of the matching residual array, or nullptr (the same for the whole workgroup)
  auto store = [&](float* out_rows, const float* res_rows, auto&& value) __attribute__((always_inline)) {
    if (res_rows != nullptr) store_impl(out_rows, res_rows, value, std::true_type{});
    else store_impl(out_rows, res_rows, value, std::false_type{});
  };

  float d1[TM][16], d2[TM][16], ssq[TM][16];
#pragma unroll
  for (int t = 0; t < TM; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) ssq[t][r] = 0.f;

  // One step: ask for the next tile, multiply the current one, wait for the loads (and for the
  // previous step's stores), and only then store; the barrier also says that every wavefront
  // is done reading the buffer that the step after this one refills.
  auto product = [&](int it, const float* cur, float* nxt, floatx16 (&acc)[TM]) __attribute__((always_inline)) {
    if (it + 1 < n_iter) issue(tile_src(it + 1), nxt);
    compute(cur, acc);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  auto jac_step = [&](int it, const float* cur, float* nxt) __attribute__((always_inline)) {
    floatx16 acc[TM];
    product(it, cur, nxt, acc);
#pragma unroll
    for (int t = 0; t < TM; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) ssq[t][r] += acc[t][r] * acc[t][r];
    const int64_t joff = ((int64_t)(p0 + it - 1) * R + r0) * N;
    store(a.y_jac + joff, a.res_jac ? a.res_jac + joff : nullptr, [&](int t, int r) { return d1[t][r] * acc[t][r]; });
  };
  auto lap_step = [&](const float* cur) __attribute__((always_inline)) {
    floatx16 acc[TM];
    compute(cur, acc);
    store(a.y_lap + r0 * N, a.res_lap ? a.res_lap + r0 * N : nullptr,
          [&](int t, int r) { return d1[t][r] * acc[t][r] + d2[t][r] * ssq[t][r]; });
  };

  issue(tile_src(0), As0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  {
    floatx16 acc[TM];
    product(0, As0, As1, acc);
    float o[TM][16];
#define FOLX_DA_CASE(A)                                                                      \
  case A:                                                                                    \
    _Pragma("unroll") for (int t = 0; t < TM; ++t) _Pragma("unroll") for (int r = 0; r < 16; ++r) \
        act_eval<A>(acc[t][r] + bcol, a.prm, o[t][r], d1[t][r], d2[t][r]);                    \
    break;
    switch (a.act) {
      FOLX_DA_CASE(FOLX_ACT_TANH) FOLX_DA_CASE(FOLX_ACT_SILU) FOLX_DA_CASE(FOLX_ACT_LOGISTIC)
      FOLX_DA_CASE(FOLX_ACT_SOFTPLUS) FOLX_DA_CASE(FOLX_ACT_EXP) FOLX_DA_CASE(FOLX_ACT_SIN)
      FOLX_DA_CASE(FOLX_ACT_COS)
      default:
        _Pragma("unroll") for (int t = 0; t < TM; ++t) _Pragma("unroll") for (int r = 0; r < 16; ++r)
            act_eval<FOLX_ACT_SQUARE>(acc[t][r] + bcol, a.prm, o[t][r], d1[t][r], d2[t][r]);
        break;
    }
#undef FOLX_DA_CASE
    if (mode == 0 || (mode == 1 && g == 0))
      store(a.y + r0 * N, a.res ? a.res + r0 * N : nullptr, [&](int t, int r) { return o[t][r]; });
  }
  // Jacobian rows: odd steps read As1, even steps As0
  int it = 1;
  for (; it + 1 <= nJ; it += 2) {
    jac_step(it, As1, As0);
    jac_step(it + 1, As0, As1);
  }
  const bool odd = it <= nJ;
  if (odd) jac_step(it, As1, As0);
  float* part = a.part + (int64_t)rt * G * PART_PER_BLOCK;
  if (mode == 1) {
#pragma unroll
    for (int t = 0; t < TM; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) part[(int64_t)g * PART_PER_BLOCK + (t * 16 + r) * NTHR + tid] = ssq[t][r];
    return;
  }
  if (mode == 2) {
    for (int gg = 0; gg < G; ++gg)
#pragma unroll
      for (int t = 0; t < TM; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) ssq[t][r] += part[(int64_t)gg * PART_PER_BLOCK + (t * 16 + r) * NTHR + tid];
  }
  // the lap tile was requested by the last step before it and has been waited for
  if (odd) lap_step(As0); else lap_step(As1);
}

template <int KS, int WC>
void launch_da(hipStream_t st, DAParams prm, const DAPlan& pl) {
  if (pl.G == 1) {
    prm.mode = 0;
    dense_act_kernel<KS, WC><<<dim3((unsigned)pl.row_tiles), dim3(NTHR), 0, st>>>(prm);
  } else {
    prm.mode = 1;
    dense_act_kernel<KS, WC><<<dim3((unsigned)(pl.row_tiles * pl.G)), dim3(NTHR), 0, st>>>(prm);
    prm.mode = 2;
    dense_act_kernel<KS, WC><<<dim3((unsigned)pl.row_tiles), dim3(NTHR), 0, st>>>(prm);
  }
}

}  // namespace

extern "C" int64_t folx_hip_dense_act_workspace_bytes(int64_t R, int32_t P, int32_t K, int32_t N) {
  DAPlan pl;
  if (R < 0 || P < 0) return FOLX_HIP_EINVAL;
  if (!plan_dense_act(R, P, K, N, pl)) return folx_dense_act_wide_ws_bytes(R, P, K, N);
  return pl.ws_bytes;
}

extern "C" int folx_hip_dense_act_fwdlap(void* stream, int32_t act, float param, const float* x, const float* jac,
                                         const float* lap, const float* W, const float* bias, const float* res,
                                         const float* res_jac, const float* res_lap, float* y,
                                         float* y_jac, float* y_lap, int64_t R, int32_t P, int32_t K, int32_t N,
                                         void* workspace, int64_t workspace_bytes) {
  if (R < 0 || P < 0 || K <= 0 || N <= 0) return FOLX_HIP_EINVAL;
  if ((res != nullptr) != (res_lap != nullptr) || (P > 0 && (res != nullptr) != (res_jac != nullptr)))
    return FOLX_HIP_EINVAL;
  if (!act_fused(act)) return FOLX_HIP_ENOTSUP;
  DAPlan pl;
  if (!plan_dense_act(R, P, K, N, pl)) {
    if (res) return FOLX_HIP_ENOTSUP;  // the wide path adds a skip connection only when it reads its operand in parts
    return folx_dense_act_wide((hipStream_t)stream, act, param, x, jac, lap, W, bias, y, y_jac, y_lap, R, P, K, N,
                               workspace, workspace_bytes);
  }
  if (R == 0) return FOLX_HIP_OK;
  if (!x || !lap || !W || !y || !y_lap || (P > 0 && (!jac || !y_jac))) return FOLX_HIP_EINVAL;
  if (!folx_aligned16(x) || !folx_aligned16(lap) || (P > 0 && !folx_aligned16(jac))) return FOLX_HIP_ENOTSUP;
  if (pl.ws_bytes > 0 && (!workspace || workspace_bytes < pl.ws_bytes || !folx_aligned16(workspace)))
    return FOLX_HIP_EINVAL;
  DAParams prm;
  prm.x = x; prm.jac = jac; prm.lap = lap; prm.W = W; prm.bias = bias;
  prm.res = res; prm.res_jac = res_jac; prm.res_lap = res_lap;
  prm.y = y; prm.y_jac = y_jac; prm.y_lap = y_lap;
  prm.part = (float*)workspace;
  prm.R = R; prm.P = P; prm.K = K; prm.N = N; prm.G = pl.G; prm.PG = pl.PG; prm.act = act; prm.prm = param; prm.mode = 0;
  hipStream_t st = (hipStream_t)stream;
  const int code = pl.wc * 100 + pl.ks;
  switch (code) {
    case 101: launch_da<1, 1>(st, prm, pl); break;
    case 104: launch_da<4, 1>(st, prm, pl); break;
    case 201: launch_da<1, 2>(st, prm, pl); break;
    case 204: launch_da<4, 2>(st, prm, pl); break;
    case 208: launch_da<8, 2>(st, prm, pl); break;
    case 401: launch_da<1, 4>(st, prm, pl); break;
    case 404: launch_da<4, 4>(st, prm, pl); break;
    case 408: launch_da<8, 4>(st, prm, pl); break;
    case 413: launch_da<13, 4>(st, prm, pl); break;
    case 416: launch_da<16, 4>(st, prm, pl); break;
    default: return FOLX_HIP_ENOTSUP;
  }
  return folx_launch_status();
}
