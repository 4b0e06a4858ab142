// Dense-layer rule: y = h @ W (+ bias) (+ residual) over the stacked operand [x; J; lap].
//
// All (P + 2) * R rows go through ONE launch of an LDS-tiled FP32-MFMA GEMM
// (v_mfma_f32_32x32x2_f32).  The three operands are separate allocations, so the row
// tiles are laid out per segment (x, jac, lap) and never straddle two of them.
//
// Tiling: a workgroup owns BM rows x BN columns and walks K in chunks of BK = 16 through
// double-buffered LDS tiles, one barrier per chunk.  For N > 128 the tile is 128 x 256 on 8
// wavefronts (each 64 x 64), so a layer of width 256 reads its A rows from HBM exactly once
// and two workgroups share a CU; narrower layers use 128 x {128, 64, 32} tiles on 4
// wavefronts.
//
// Main path (K a multiple of 16, 16-byte aligned operands): the chunks go from global memory
// straight into LDS (global_load_lds_dwordx4), no staging registers and no LDS store
// instructions.  Such a load puts the 16 bytes of lane i at LDS slot (wavefront base + i), so
// the tile layout is chosen by which global address each lane asks for: an A tile is
// [row][4 pieces of 4 k], and piece c of a row holds k-chunk c ^ ((row / 2) % 4), which
// spreads the rows of 8 consecutive lanes over all LDS banks for the 128-bit fragment
// reads.  The two buffers are separate LDS arrays, so the compiler's memory-counter waits
// for the buffer being filled do not hold up reads of the buffer being computed on.
// The MFMA only needs A and B to agree on which k a lane holds, so the k order inside a
// group of 8 is permuted to fit the 128-bit read:
//     lane l, register j of group t  <->  k = 8 t + 4 (l / 32) + j.
// W rows are stored [k][n] and read with consecutive n across lanes.
//
// Fallback path (any K, any alignment): global -> registers -> LDS with bounds handled by
// clamped addresses and selects; A rows use a stride of BK + 4 floats instead of the swizzle.
//
// Epilogue: a tile that lies fully inside the matrix is stored without per-element tests,
// with one 32-bit lane offset for all stores and wave-uniform scalar row arithmetic; the
// bias is fetched before the K loop.  Edge tiles take a checked path.
//
// Two more forms of the rule live here: N = 1 (a matrix-vector product, dense_n1_flat_kernel /
// dense_n1_kernel) and, when folx_hip_set_gemm_mode asks for it, the 128 x 256 tile with every
// fp32 product taken as six exact products of bf16 pieces (dense_split_kernel, split_bf16.h).
//
// Workgroup ids are remapped so that the column tiles of one row tile run back to back
// on the same XCD (ids are dealt round-robin to the 8 XCDs), which keeps the second
// read of an A tile in that XCD's L2 when N needs more than one column tile.
#include <algorithm>

#include "common.h"
#include "split_bf16.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BK = 16;
constexpr int AS = BK + 4;  // LDS row stride of the A tile (floats)
constexpr int NXCD = 8;

struct Segs {
  const float* in[3];
  const float* res[3];  // optional residual (same shape as out) added in the epilogue
  float* out[3];
  int64_t rows[3];
  int64_t tiles[3];
  // Input rows may come in groups: logical row r sits at physical row
  // (r / group) * gstride + r % group of its segment (group = 0: contiguous rows).
  int64_t group, gstride;
};

__device__ __forceinline__ int64_t phys_row(const Segs& sg, int64_t r) {
  return sg.group > 0 ? (r / sg.group) * sg.gstride + r % sg.group : r;
}

// Register r of a 32x32 accumulator tile holds row 8 (r / 4) + 4 (lane / 32) + r % 4, column
// lane % 32, so each store instruction writes two 128-byte row segments.
template <int BM, int BN, int TM, int TN, bool HAS_RES>
__device__ __forceinline__ void store_tile(const floatx16 (&acc)[TM][TN], const float (&bvals)[TN],
                                           float* __restrict__ C, const float* __restrict__ Rs, int64_t rows,
                                           int32_t N, int64_t row0, int32_t col0, int wr, int wc, int l32,
                                           int lh) {
  const bool full_tile = (row0 + BM <= rows) && (col0 + BN <= N);
  if (full_tile) {
    const uint32_t voff = (uint32_t)((4 * lh * N + l32) * 4);
    float* cs = C + (row0 + wr) * (int64_t)N + col0 + wc;
    const float* rsb = HAS_RES ? Rs + (row0 + wr) * (int64_t)N + col0 + wc : nullptr;
    // The residuals of four rows are requested together, one group of four rows ahead of their
    // use (across accumulator blocks): the stores cannot be told apart from the residual array,
    // so a load written after a group's stores would wait for them to be issued, and every
    // group would pay a memory round trip of its own.
    float rs[2][4];
    auto fetch = [&](int step, float (&dst)[4]) __attribute__((always_inline)) {
      const int g = step % 4, j = (step / 4) % TN, i = step / (4 * TN);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const char* p = (const char*)(rsb + (int64_t)(i * 32 + 8 * g + r) * N + j * 32);
        dst[r] = __builtin_nontemporal_load((const float*)(p + voff));
      }
    };
    if constexpr (HAS_RES) fetch(0, rs[0]);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int step = (i * TN + j) * 4 + g;
          if constexpr (HAS_RES)
            if (step + 1 < TM * TN * 4) fetch(step + 1, rs[(step + 1) & 1]);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            char* p = (char*)(cs + (int64_t)(i * 32 + 8 * g + r) * N + j * 32);
            float o = acc[i][j][4 * g + r] + bvals[j];
            if constexpr (HAS_RES) o += rs[step & 1][r];
            __builtin_nontemporal_store(o, (float*)(p + voff));  // written once, read by a later launch
          }
        }
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int gc = col0 + wc + j * 32 + l32;
      const bool cok = gc < N;
      if (cok) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t gr = row0 + wr + i * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
          if (gr < rows) {
            float o = acc[i][j][r] + bvals[j];
            if constexpr (HAS_RES) o += Rs[gr * (int64_t)N + gc];
            C[gr * (int64_t)N + gc] = o;
          }
        }
      }
    }
  }
}

#define FOLX_GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define FOLX_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

// Main path: direct-to-LDS loads.  Requires K % 16 == 0, N % 4 == 0, N >= 4 and 16-byte
// aligned operands.  Rows / columns past the end are clamped to valid addresses; what they
// bring in only reaches accumulator rows / columns that are never stored.
template <int BM, int BN, int WM, int WN, bool HAS_RES>
__global__ __launch_bounds__(64 * WM * WN, 4) void dense_dma_kernel(Segs sg, const float* __restrict__ W,
                                                                    const float* __restrict__ bias, int32_t K,
                                                                    int32_t N, int64_t row_tiles,
                                                                    int32_t col_tiles) {
  constexpr int NT = 64 * WM * WN;
  constexpr int WROWS = BM / WM, WCOLS = BN / WN;
  constexpr int TM = WROWS / 32, TN = WCOLS / 32;
  constexpr int TG = BK / 8;
  constexpr int A_V4 = BM * BK / 4, W_V4 = BK * BN / 4;
  static_assert(A_V4 % 64 == 0 && W_V4 % 64 == 0, "whole wavefronts per tile chunk");
  constexpr int A_LD = (A_V4 + NT - 1) / NT, W_LD = (W_V4 + NT - 1) / NT;

  __shared__ __attribute__((aligned(16))) float As0[BM * BK];
  __shared__ __attribute__((aligned(16))) float As1[BM * BK];
  __shared__ __attribute__((aligned(16))) float Ws0[BK * BN];
  __shared__ __attribute__((aligned(16))) float Ws1[BK * BN];

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
  const int64_t rows = sg.rows[seg];
  const int64_t row0 = t * BM;
  const int32_t col0 = ct * BN;

  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wr = (wave / WN) * WROWS;
  const int wc = (wave % WN) * WCOLS;
  const int l32 = lane % 32;
  const int lh = lane / 32;

  const float* a_p[A_LD];
  const float* w_p[W_LD];
#pragma unroll
  for (int i = 0; i < A_LD; ++i) {
    const int idx = tid + NT * i;
    const int r = idx / 4, c = idx % 4;
    const int kc = c ^ ((r / 2) % 4);
    int64_t gr = row0 + r;
    if (gr >= rows) gr = rows - 1;
    a_p[i] = A + phys_row(sg, gr) * (int64_t)K + kc * 4;
  }
#pragma unroll
  for (int i = 0; i < W_LD; ++i) {
    const int idx = tid + NT * i;
    const int k = (idx / (BN / 4)) % BK;
    int n = col0 + (idx % (BN / 4)) * 4;
    if (n > N - 4) n = N - 4;
    w_p[i] = W + (int64_t)k * N + n;
  }
  auto issue = [&](int kt, float* as, float* ws) {
#pragma unroll
    for (int i = 0; i < A_LD; ++i)
      if (A_V4 % NT == 0 || wave * 64 + NT * i < A_V4)
        __builtin_amdgcn_global_load_lds(FOLX_GPTR(a_p[i] + kt * BK), FOLX_LPTR(&as[(wave * 64 + NT * i) * 4]), 16,
                                         0, 0);
#pragma unroll
    for (int i = 0; i < W_LD; ++i)
      if (W_V4 % NT == 0 || wave * 64 + NT * i < W_V4)
        __builtin_amdgcn_global_load_lds(FOLX_GPTR(w_p[i] + (int64_t)kt * BK * N),
                                         FOLX_LPTR(&ws[(wave * 64 + NT * i) * 4]), 16, 0, 0);
  };

  float bvals[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int gc = col0 + wc + j * 32 + l32;
    bvals[j] = (seg == 0 && bias != nullptr && gc < N) ? bias[gc] : 0.0f;
  }

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int sw = (l32 / 2) % 4;
  auto compute = [&](const float* as, const float* ws) {
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
  store_tile<BM, BN, TM, TN, HAS_RES>(acc, bvals, sg.out[seg], HAS_RES ? sg.res[seg] : nullptr, rows, N, row0, col0,
                                      wr, wc, l32, lh);
}

template <int BM, int BN, int WM, int WN, int MINB, bool VEC, bool HAS_RES>
__global__ __launch_bounds__(64 * WM * WN, MINB) void dense_kernel(Segs sg, const float* __restrict__ W,
                                                                   const float* __restrict__ bias,
                                                                   int32_t K, int32_t N,
                                                                   int64_t row_tiles,
                                                                   int32_t col_tiles) {
  constexpr int NT = 64 * WM * WN;
  constexpr int WROWS = BM / WM;  // rows per wavefront
  constexpr int WCOLS = BN / WN;  // columns per wavefront
  constexpr int TM = WROWS / 32;
  constexpr int TN = WCOLS / 32;
  constexpr int TG = BK / 8;
  constexpr int A_V4 = BM * BK / 4;                 // float4 of one A chunk
  constexpr int W_V4 = BK * BN / 4;                 // float4 of one W chunk
  constexpr int A_LD = (A_V4 + NT - 1) / NT;
  constexpr int W_LD = (W_V4 + NT - 1) / NT;

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
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wr = (wave / WN) * WROWS;
  const int wc = (wave % WN) * WCOLS;
  const int l32 = lane % 32;
  const int lh = lane / 32;

  float bvals[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int gc = col0 + wc + j * 32 + l32;
    bvals[j] = (seg == 0 && bias != nullptr && gc < N) ? bias[gc] : 0.0f;
  }

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  float4 ra[A_LD], rw[W_LD];

  // per-thread source rows / columns are fixed over the K loop
  int a_r[A_LD], a_k[A_LD], w_k[W_LD], w_n[W_LD];
  bool a_ok[A_LD], w_ok[W_LD];
  const float* a_p[A_LD];
  const float* w_p[W_LD];
#pragma unroll
  for (int i = 0; i < A_LD; ++i) {
    const int idx = tid + NT * i;
    a_r[i] = idx / (BK / 4);
    a_k[i] = (idx % (BK / 4)) * 4;
    int64_t gr = row0 + a_r[i];
    a_ok[i] = (A_V4 % NT == 0 || idx < A_V4) && gr < rows;
    if (gr >= rows) gr = rows - 1;
    a_p[i] = A + phys_row(sg, gr) * (int64_t)K;
  }
#pragma unroll
  for (int i = 0; i < W_LD; ++i) {
    const int idx = tid + NT * i;
    w_k[i] = idx / (BN / 4);
    w_n[i] = (idx % (BN / 4)) * 4;
    w_ok[i] = (W_V4 % NT == 0 || idx < W_V4) && (col0 + w_n[i] < N);
    w_p[i] = W + (w_ok[i] ? col0 + w_n[i] : 0);
  }

  auto load_global = [&](int kt) {
    const int k0 = kt * BK;
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
      const int gk = k0 + a_k[i];
      if constexpr (VEC) {
        const bool ok = a_ok[i] && gk < K;
        const float4 v = *reinterpret_cast<const float4*>(a_p[i] + (gk < K ? gk : 0));
        ra[i] = ok ? v : make_float4(0.f, 0.f, 0.f, 0.f);
      } else {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (a_ok[i]) {
          const float* src = a_p[i] + gk;
          if (gk + 0 < K) v.x = src[0];
          if (gk + 1 < K) v.y = src[1];
          if (gk + 2 < K) v.z = src[2];
          if (gk + 3 < K) v.w = src[3];
        }
        ra[i] = v;
      }
    }
#pragma unroll
    for (int i = 0; i < W_LD; ++i) {
      const int gk = k0 + w_k[i];
      if constexpr (VEC) {
        const bool ok = w_ok[i] && gk < K;
        const float4 v = *reinterpret_cast<const float4*>(w_p[i] + (int64_t)(gk < K ? gk : 0) * N);
        rw[i] = ok ? v : make_float4(0.f, 0.f, 0.f, 0.f);
      } else {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if ((W_V4 % NT == 0 || tid + NT * i < W_V4) && gk < K) {
          const int gn = col0 + w_n[i];
          const float* src = W + (int64_t)gk * N + gn;
          if (gn + 0 < N) v.x = src[0];
          if (gn + 1 < N) v.y = src[1];
          if (gn + 2 < N) v.z = src[2];
          if (gn + 3 < N) v.w = src[3];
        }
        rw[i] = v;
      }
    }
  };

  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_LD; ++i)
      if (A_V4 % NT == 0 || tid + NT * i < A_V4)
        *reinterpret_cast<float4*>(&As[buf][a_r[i] * AS + a_k[i]]) = ra[i];
#pragma unroll
    for (int i = 0; i < W_LD; ++i)
      if (W_V4 % NT == 0 || tid + NT * i < W_V4)
        *reinterpret_cast<float4*>(&Ws[buf][w_k[i] * BN + w_n[i]]) = rw[i];
  };

  const int KT = (K + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) load_global(kt + 1);

#pragma unroll
    for (int tg = 0; tg < TG; ++tg) {
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

  store_tile<BM, BN, TM, TN, HAS_RES>(acc, bvals, C, HAS_RES ? sg.res[seg] : nullptr, rows, N, row0, col0, wr, wc,
                                      l32, lh);
}

// The 128 x 256 tile of dense_dma_kernel with the products taken on the bf16 matrix pipe from
// operands split into three bf16 pieces each.  A (streamed once) and W (K x N, from L2) both
// come through registers, one chunk of 16 k ahead, and every element is split once per
// workgroup on its way into LDS:
//   A stage: [piece][g][row][8 bf16]      k = 8 g + e, one 16-byte fragment per (g, row)
//   W stage: [piece][g][kp][col] dwords   k = 8 g + 2 kp and + 1, read as four 32-bit values
// (lane l of a 32 x 32 x 16 product holds row or column l % 32 and the 8 k of g = l / 32).
// Thread t stages row t / 4, k quarter t % 4 of the A chunk; wavefront w stages rows 2 w and
// 2 w + 1 of the W chunk, lane l their columns 4 l .. 4 l + 3, so that a pair of k lands in one
// 32-bit word.  The barrier between chunks only waits for LDS, not for the requests of the
// next chunk.  Same epilogue as the fp32 kernel.  Requires K % 16 == 0, N % 4 == 0, N >= 4
// and 16-byte aligned operands.
template <bool HAS_RES>
__global__ __launch_bounds__(512, 4) void dense_split_kernel(Segs sg, const float* __restrict__ W,
                                                             const float* __restrict__ bias, int32_t K, int32_t N,
                                                             int64_t row_tiles, int32_t col_tiles) {
  using namespace folx_split;
  constexpr int BM = 128, BN = 256, WN = 4, TM = 2, TN = 2;
  constexpr int A_PLANE = 2 * BM * 16;     // bytes of one piece of an A chunk
  constexpr int W_PLANE = 2 * 4 * BN * 4;  // and of a W chunk
  __shared__ __attribute__((aligned(16))) char As0[3 * A_PLANE];
  __shared__ __attribute__((aligned(16))) char As1[3 * A_PLANE];
  __shared__ __attribute__((aligned(16))) char Ws0[3 * W_PLANE];
  __shared__ __attribute__((aligned(16))) char Ws1[3 * W_PLANE];

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
  const int64_t rows = sg.rows[seg];
  const int64_t row0 = t * BM;
  const int32_t col0 = ct * BN;

  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wr = (wave / WN) * 64;
  const int wc = (wave % WN) * 64;
  const int l32 = lane % 32;
  const int lh = lane / 32;

  const int a_row = tid / 4, a_q = tid % 4;
  int64_t gr = row0 + a_row;
  if (gr >= rows) gr = rows - 1;  // rows past the end: copies of the last one, never stored
  const float* a_src = A + phys_row(sg, gr) * (int64_t)K + a_q * 4;
  const int a_dst = ((a_q / 2) * BM + a_row) * 16 + (a_q % 2) * 8;
  int wn = col0 + lane * 4;
  if (wn > N - 4) wn = N - 4;  // columns past the end likewise
  const float* w_src = W + (int64_t)(2 * wave) * N + wn;
  const int w_dst = (wave * BN + lane * 4) * 4;  // (g, kp) = (wave / 4, wave % 4)

  auto put_a = [&](const float4& v, char* as) __attribute__((always_inline)) {
    unsigned p1a, p2a, p3a, p1b, p2b, p3b;
    split_pair(v.x, v.y, p1a, p2a, p3a);
    split_pair(v.z, v.w, p1b, p2b, p3b);
    uint2v q;
    q[0] = p1a; q[1] = p1b; *reinterpret_cast<uint2v*>(as + a_dst) = q;
    q[0] = p2a; q[1] = p2b; *reinterpret_cast<uint2v*>(as + A_PLANE + a_dst) = q;
    q[0] = p3a; q[1] = p3b; *reinterpret_cast<uint2v*>(as + 2 * A_PLANE + a_dst) = q;
  };
  auto put_w = [&](const float4& r0, const float4& r1, char* ws) __attribute__((always_inline)) {
    unsigned a1[4], a2[4], a3[4];
    split_pair(r0.x, r1.x, a1[0], a2[0], a3[0]);
    split_pair(r0.y, r1.y, a1[1], a2[1], a3[1]);
    split_pair(r0.z, r1.z, a1[2], a2[2], a3[2]);
    split_pair(r0.w, r1.w, a1[3], a2[3], a3[3]);
    uint4v q1, q2, q3;
#pragma unroll
    for (int c = 0; c < 4; ++c) { q1[c] = a1[c]; q2[c] = a2[c]; q3[c] = a3[c]; }
    *reinterpret_cast<uint4v*>(ws + w_dst) = q1;
    *reinterpret_cast<uint4v*>(ws + W_PLANE + w_dst) = q2;
    *reinterpret_cast<uint4v*>(ws + 2 * W_PLANE + w_dst) = q3;
  };

  float bvals[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int gc = col0 + wc + j * 32 + l32;
    bvals[j] = (seg == 0 && bias != nullptr && gc < N) ? bias[gc] : 0.0f;
  }
  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  auto compute = [&](const char* as, const char* ws) __attribute__((always_inline)) {
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

  const int KT = K / 16;
  float4 ra, rw0, rw1;
  auto fetch = [&](int kt) __attribute__((always_inline)) {
    // (a plain load: the other half of each 128-byte line is asked for one chunk later and
    // should still be in L2 then, which a non-temporal request does not promise)
    ra = *reinterpret_cast<const float4*>(a_src + kt * 16);
    rw0 = *reinterpret_cast<const float4*>(w_src + (int64_t)kt * 16 * N);
    rw1 = *reinterpret_cast<const float4*>(w_src + (int64_t)kt * 16 * N + N);
  };
  // chunk kt + 1 is split into the other stage and chunk kt + 2 requested before the products
  // of chunk kt; the barrier waits for LDS only
  fetch(0);
  put_a(ra, As0);
  put_w(rw0, rw1, Ws0);
  if (KT > 1) fetch(1);
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  for (int kt = 0; kt < KT; kt += 2) {
    if (kt + 1 < KT) {
      put_a(ra, As1);
      put_w(rw0, rw1, Ws1);
      if (kt + 2 < KT) fetch(kt + 2);
    }
    compute(As0, Ws0);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (kt + 1 < KT) {
      if (kt + 2 < KT) {
        put_a(ra, As0);
        put_w(rw0, rw1, Ws0);
        if (kt + 3 < KT) fetch(kt + 3);
      }
      compute(As1, Ws1);
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
  }
  store_tile<BM, BN, TM, TN, HAS_RES>(acc, bvals, sg.out[seg], HAS_RES ? sg.res[seg] : nullptr, rows, N, row0, col0,
                                      wr, wc, l32, lh);
}

// N = 1 (a layer with one output per position, e.g. the last layer of a node-wise network): the
// rule is a matrix-vector product, bound by reading the rows once.  A group of 32 lanes owns a
// row at a time: 128-bit loads of up to 128 features per pass, the weights in registers, the
// sum over the group by lane exchanges.  Rows are in the three segments of the stacked operand.
__global__ __launch_bounds__(256) void dense_n1_kernel(Segs sg, const float* __restrict__ W, const float* __restrict__ bias,
                                                       int32_t K, int64_t total_rows) {
  const int lane32 = threadIdx.x % 32;
  const int64_t g0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) / 32;
  const int64_t ngroups = (int64_t)gridDim.x * 8;
  const int passes = (K + 127) / 128;
  const float b0 = bias != nullptr ? bias[0] : 0.0f;
  auto locate = [&](int64_t r, int& seg, int64_t& t) {
    seg = 0;
    t = r;
    if (t >= sg.rows[0]) { t -= sg.rows[0]; seg = 1; if (t >= sg.rows[1]) { t -= sg.rows[1]; seg = 2; } }
  };
  auto finish = [&](float acc, int seg, int64_t t) {
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 32);
    if (lane32 == 0) {
      float o = acc + (seg == 0 ? b0 : 0.0f);
      if (sg.res[seg] != nullptr) o += sg.res[seg][t];
      sg.out[seg][t] = o;
    }
  };
  if (passes == 1) {
    // Four rows in flight per group of lanes: their loads are all issued before the first sum.
    constexpr int U = 4;
    const int k = 4 * lane32;
    const bool on = k < K;
    const float4 w = on ? *reinterpret_cast<const float4*>(W + k) : make_float4(0.f, 0.f, 0.f, 0.f);
    for (int64_t r = g0; r < total_rows; r += U * ngroups) {
      int seg[U];
      int64_t t[U];
      float4 a[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t ru = r + u * ngroups;
        locate(ru < total_rows ? ru : r, seg[u], t[u]);
        a[u] = on ? folx_ld_stream4(sg.in[seg[u]] + phys_row(sg, t[u]) * (int64_t)K + k) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (r + u * ngroups < total_rows)
          finish(fmaf(a[u].x, w.x, fmaf(a[u].y, w.y, fmaf(a[u].z, w.z, a[u].w * w.w))), seg[u], t[u]);
      }
    }
    return;
  }
  for (int64_t r = g0; r < total_rows; r += ngroups) {
    int seg;
    int64_t t;
    locate(r, seg, t);
    const float* row = sg.in[seg] + phys_row(sg, t) * (int64_t)K;
    float acc = 0.0f;
    for (int ps = 0; ps < passes; ++ps) {
      const int k = ps * 128 + 4 * lane32;
      if (k < K) {
        const float4 a = folx_ld_stream4(row + k);
        const float4 w = *reinterpret_cast<const float4*>(W + k);
        acc = fmaf(a.x, w.x, fmaf(a.y, w.y, fmaf(a.z, w.z, fmaf(a.w, w.w, acc))));
      }
    }
    finish(acc, seg, t);
  }
}

// The same for contiguous rows (no row groups) and K <= 256: the rows of a block are read as ONE
// flat run of 128-bit pieces, consecutive lanes consecutive pieces (every lane busy, whole lines
// per request, a handful of instructions per piece instead of a reduction tree per row).  Piece
// f of the block lies in row f / (K / 4) at k = 4 (f % (K / 4)); its product with the four
// weights goes to LDS, and after a barrier thread r adds the K / 4 partial sums of row r
// (stride K / 4 floats between threads: no bank conflict when K / 4 is odd, e.g. K = 100).
constexpr int N1_ROWS = 64;    // rows per block
constexpr int N1_MAXK4 = 64;   // K <= 256
__global__ __launch_bounds__(256) void dense_n1_flat_kernel(Segs sg, const float* __restrict__ W,
                                                            const float* __restrict__ bias, int32_t K) {
  __shared__ __attribute__((aligned(16))) float wS[4 * N1_MAXK4];
  __shared__ float part[N1_ROWS * N1_MAXK4];
  int seg = 0;
  int64_t t = blockIdx.x;
  if (t >= sg.tiles[0]) { t -= sg.tiles[0]; seg = 1; if (t >= sg.tiles[1]) { t -= sg.tiles[1]; seg = 2; } }
  const int K4 = K / 4;
  const int64_t row0 = t * N1_ROWS;
  const int nrows = (int)(sg.rows[seg] - row0 < N1_ROWS ? sg.rows[seg] - row0 : N1_ROWS);
  const int nf = nrows * K4;
  const float* base = sg.in[seg] + row0 * (int64_t)K;
  const int tid = threadIdx.x;
  if (tid < K4) reinterpret_cast<float4*>(wS)[tid] = *reinterpret_cast<const float4*>(W + 4 * tid);
  // up to 16 pieces per thread, eight requests in flight
  constexpr int U = 8;
  const int step = 256 % K4;
  int k4 = tid % K4;
  __syncthreads();
  for (int f0 = tid; f0 < nf; f0 += U * 256) {
    float4 a[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int f = f0 + u * 256;
      a[u] = folx_ld_stream4(base + 4 * (int64_t)(f < nf ? f : f0));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int f = f0 + u * 256;
      const float4 w = reinterpret_cast<const float4*>(wS)[k4];
      if (f < nf) part[f] = fmaf(a[u].x, w.x, fmaf(a[u].y, w.y, fmaf(a[u].z, w.z, a[u].w * w.w)));
      k4 += step;
      if (k4 >= K4) k4 -= K4;
    }
  }
  __syncthreads();
  if (tid < nrows) {
    const float* pr = part + tid * K4;
    float s0 = 0.0f, s1 = 0.0f;
    int c = 0;
    for (; c + 2 <= K4; c += 2) { s0 += pr[c]; s1 += pr[c + 1]; }
    if (c < K4) s0 += pr[c];
    float o = s0 + s1 + (seg == 0 && bias != nullptr ? bias[0] : 0.0f);
    if (sg.res[seg] != nullptr) o += sg.res[seg][row0 + tid];
    sg.out[seg][row0 + tid] = o;
  }
}

template <int BM, int BN, int WM, int WN, int MINB>
int launch_cfg(hipStream_t st, Segs& sg, const float* W, const float* bias, int32_t K, int32_t N,
               bool vec, bool has_res) {
  int64_t row_tiles = 0;
  for (int s = 0; s < 3; ++s) { sg.tiles[s] = (sg.rows[s] + BM - 1) / BM; row_tiles += sg.tiles[s]; }
  const int32_t col_tiles = (N + BN - 1) / BN;
  const int64_t groups = (row_tiles + NXCD - 1) / NXCD;
  const int64_t blocks = groups * NXCD * col_tiles;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  dim3 grid((unsigned)blocks), block(64 * WM * WN);
  if constexpr (BM == 128 && BN == 256) {
    if (vec && K % BK == 0 && N >= 4 && folx_gemm_mode() == FOLX_HIP_GEMM_BF16X3) {
      if (has_res)
        dense_split_kernel<true><<<grid, block, 0, st>>>(sg, W, bias, K, N, row_tiles, col_tiles);
      else
        dense_split_kernel<false><<<grid, block, 0, st>>>(sg, W, bias, K, N, row_tiles, col_tiles);
      return folx_launch_status();
    }
  }
  if (vec && K % BK == 0 && N >= 4) {
    if (has_res)
      dense_dma_kernel<BM, BN, WM, WN, true><<<grid, block, 0, st>>>(sg, W, bias, K, N, row_tiles, col_tiles);
    else
      dense_dma_kernel<BM, BN, WM, WN, false><<<grid, block, 0, st>>>(sg, W, bias, K, N, row_tiles, col_tiles);
    return folx_launch_status();
  }
  if (vec && has_res)
    dense_kernel<BM, BN, WM, WN, MINB, true, true><<<grid, block, 0, st>>>(sg, W, bias, K, N, row_tiles, col_tiles);
  else if (vec)
    dense_kernel<BM, BN, WM, WN, MINB, true, false><<<grid, block, 0, st>>>(sg, W, bias, K, N, row_tiles, col_tiles);
  else if (has_res)
    dense_kernel<BM, BN, WM, WN, MINB, false, true><<<grid, block, 0, st>>>(sg, W, bias, K, N, row_tiles, col_tiles);
  else
    dense_kernel<BM, BN, WM, WN, MINB, false, false><<<grid, block, 0, st>>>(sg, W, bias, K, N, row_tiles, col_tiles);
  return folx_launch_status();
}

}  // namespace

extern "C" int folx_hip_dense_rows_fwdlap(void* stream, const float* x, const float* jac,
                                          const float* lap, const float* W, const float* bias,
                                          const float* res, const float* res_jac, const float* res_lap,
                                          float* y, float* y_jac, float* y_lap, int64_t R, int32_t P,
                                          int32_t K, int32_t N, int64_t group, int64_t group_stride) {
  if (R < 0 || P < 0 || K <= 0 || N <= 0 || group < 0 || (group > 0 && group_stride < group))
    return FOLX_HIP_EINVAL;
  if (R == 0) return FOLX_HIP_OK;
  if (group > 0 && R % group != 0) return FOLX_HIP_EINVAL;
  if (!x || !lap || !W || !y || !y_lap || (P > 0 && (!jac || !y_jac))) return FOLX_HIP_EINVAL;
  if ((res != nullptr) != (res_lap != nullptr) || (P > 0 && (res != nullptr) != (res_jac != nullptr)))
    return FOLX_HIP_EINVAL;
  Segs sg;
  sg.res[0] = res; sg.res[1] = res_jac; sg.res[2] = res_lap;
  sg.in[0] = x; sg.in[1] = jac; sg.in[2] = lap;
  sg.out[0] = y; sg.out[1] = y_jac; sg.out[2] = y_lap;
  sg.rows[0] = R; sg.rows[1] = (int64_t)P * R; sg.rows[2] = R;
  sg.group = group; sg.gstride = group_stride;
  if (P == 0) { sg.in[1] = x; sg.out[1] = y; sg.res[1] = res; }  // never dereferenced: 0 tiles
  const bool vec = (K % 4 == 0) && (N % 4 == 0) && folx_aligned16(x) && folx_aligned16(jac) &&
                   folx_aligned16(lap) && folx_aligned16(W);
  const bool has_res = res != nullptr;
  hipStream_t st = (hipStream_t)stream;
  if (N == 1 && K % 4 == 0 && folx_aligned16(x) && folx_aligned16(jac) && folx_aligned16(lap) && folx_aligned16(W)) {
    if (group == 0 && K <= 4 * N1_MAXK4) {
      int64_t tiles = 0;
      for (int s = 0; s < 3; ++s) { sg.tiles[s] = (sg.rows[s] + N1_ROWS - 1) / N1_ROWS; tiles += sg.tiles[s]; }
      if (tiles <= 0x7fffffffLL) {
        dense_n1_flat_kernel<<<dim3((unsigned)tiles), dim3(256), 0, st>>>(sg, W, bias, K);
        return folx_launch_status();
      }
    }
    const int64_t total = (int64_t)(P + 2) * R;
    const int64_t blocks = std::min<int64_t>((total + 31) / 32, 256 * 32);
    dense_n1_kernel<<<dim3((unsigned)blocks), dim3(256), 0, st>>>(sg, W, bias, K, total);
    return folx_launch_status();
  }
  if (N > 128) return launch_cfg<128, 256, 2, 4, 2>(st, sg, W, bias, K, N, vec, has_res);
  if (N > 64) return launch_cfg<128, 128, 2, 2, 3>(st, sg, W, bias, K, N, vec, has_res);
  if (N > 32) return launch_cfg<128, 64, 4, 1, 3>(st, sg, W, bias, K, N, vec, has_res);
  return launch_cfg<128, 32, 4, 1, 3>(st, sg, W, bias, K, N, vec, has_res);
}

extern "C" int folx_hip_dense_fwdlap(void* stream, const float* x, const float* jac,
                                     const float* lap, const float* W, const float* bias,
                                     const float* res, const float* res_jac, const float* res_lap,
                                     float* y, float* y_jac, float* y_lap, int64_t R, int32_t P,
                                     int32_t K, int32_t N) {
  return folx_hip_dense_rows_fwdlap(stream, x, jac, lap, W, bias, res, res_jac, res_lap, y, y_jac, y_lap, R, P, K,
                                    N, 0, 0);
}
