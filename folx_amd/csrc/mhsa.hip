// Multi-head self attention with Laplacian:  o = softmax(q k^T) v  and its Jacobian rows
// and Laplacian, one workgroup per (walker, head).
//
// Algebra per Jacobian row c (the factored form of the rule):
//   s'_c = q'_c k^T + q k'_c^T          p'_c = p * (s'_c - rowsum(p * s'_c))
//   o'_c = p v'_c + p'_c v
//   lap_o = p lap_v + pL v                                   (pL: same as p'_c with lap_q, lap_k)
//         + [ X + p * (2 G - u - rowsum(p * 2 G)) ] v + 2 sum_c p'_c v'_c
//   X = sum_c p'_c * (s'_c - rowsum(p s'_c)),  G = sum_c q'_c k'_c^T,  u = sum_c rowsum(p'_c s'_c)
// i.e. six n x n x d matrix products per row, all on v_mfma_f32_16x16x4_f32.  With an edge
// bias e (s = q k^T + e) the rows e'_c and lap_e are added to s'_c and to the Laplacian's
// first-order part; they have no second-order contribution.
//
// Mapping: wavefront w owns query rows [16 w, 16 w + 16) and every key column, so all
// row reductions stay inside 16-lane groups of one wavefront.  k, v and the current
// k'_c, v'_c tiles are shared through LDS (the next pair waits in registers; a single LDS
// copy keeps the workgroup under 40 KB, so four workgroups share a CU); q, q'_c and p live in
// registers in MFMA A-operand layout; p'_c goes through a wavefront-private LDS tile to
// turn the MFMA result layout into the A-operand layout.  As in the GEMM, the k index
// inside a group of 16 is permuted (lane l, register r <-> k = 4 (l / 16) + r) so that A
// operands are fetched with 128-bit reads.
#include "common.h"

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float sum16(float v) {
  v += __shfl_xor(v, 1, FOLX_WAVE); v += __shfl_xor(v, 2, FOLX_WAVE);
  v += __shfl_xor(v, 4, FOLX_WAVE); v += __shfl_xor(v, 8, FOLX_WAVE);
  return v;
}
__device__ __forceinline__ float max16(float v) {
  v = fmaxf(v, __shfl_xor(v, 1, FOLX_WAVE)); v = fmaxf(v, __shfl_xor(v, 2, FOLX_WAVE));
  v = fmaxf(v, __shfl_xor(v, 4, FOLX_WAVE)); v = fmaxf(v, __shfl_xor(v, 8, FOLX_WAVE));
  return v;
}
__device__ __forceinline__ float f4get(const float4& v, int r) {
  return r == 0 ? v.x : (r == 1 ? v.y : (r == 2 ? v.z : v.w));
}

struct MhsaArgs {
  const float *q, *qj, *ql, *k, *kj, *kl, *v, *vj, *vl;
  const float *e, *ej, *el;  // optional edge bias [B][n][H][n] and its Jacobian rows / Laplacian
  const uint8_t *mask, *imask;
  float *o, *oj, *ol;
  int64_t B;
  int32_t n, H, d, P;
};

// FAST: n = 16 NW, d = 16 DT and no masks -- every bounds / mask test folds away.
template <int NW, int DT, bool EDGE, bool FAST>
__global__ __launch_bounds__(FOLX_WAVE * NW) void mhsa_kernel(MhsaArgs a) {
  constexpr int NP = 16 * NW;   // padded sequence length
  constexpr int DP = 16 * DT;   // padded head dim
  constexpr int DS = DP + 4;    // LDS row stride of (n x d) tiles
  constexpr int NS = NP + 4;    // LDS row stride of the per-wavefront (16 x n) tiles
  constexpr int NT = FOLX_WAVE * NW;
  constexpr int TILE4 = NP * DP / 4;                 // float4 per (n x d) tile
  constexpr int LD4 = (TILE4 + NT - 1) / NT;         // float4 per thread per tile
  constexpr float BIG = 1e20f;

  __shared__ __attribute__((aligned(16))) float ks[NP * DS];
  __shared__ __attribute__((aligned(16))) float vs[NP * DS];
  __shared__ __attribute__((aligned(16))) float kjs1[NP * DS];
  __shared__ __attribute__((aligned(16))) float vjs1[NP * DS];
  __shared__ __attribute__((aligned(16))) float pst[NW][16 * NS];

  const int tid = threadIdx.x;
  const int lane = tid % FOLX_WAVE;
  const int w = tid / FOLX_WAVE;
  const int l16 = lane % 16;
  const int lg = lane / 16;
  const int64_t b = blockIdx.x / a.H;
  const int h = blockIdx.x % a.H;
  const int n = a.n, d = a.d, H = a.H, P = a.P;
  const int64_t B = a.B;
  const int64_t tok = (int64_t)H * d;                 // stride between electrons
  const int64_t base = (b * n) * tok + (int64_t)h * d;  // offset of (b, 0, h, 0)
  const int64_t slice = B * n * tok;                  // stride between Jacobian rows

  auto valid = [&](int i) -> bool {
    if constexpr (FAST) return true;
    return i < n && (a.mask == nullptr || a.mask[b * n + i] != 0);
  };
  // edge-bias entries of this lane in result layout: row 16 w + 4 lg + r, column 16 jt + l16
  const int64_t etok = (int64_t)H * n;
  const int64_t ebase = (b * n) * etok + (int64_t)h * n;
  const int64_t eslice = B * n * etok;
  auto edge_add = [&](const float* src, floatx4* acc) {
#pragma unroll
    for (int jt = 0; jt < NW; ++jt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = 16 * w + 4 * lg + r, col = 16 * jt + l16;
        if (FAST || (row < n && col < n)) acc[jt][r] += src[ebase + (int64_t)row * etok + col];
      }
  };

  // cooperative load of an (n x d) tile into LDS, rows of padding electrons zeroed
  float4 rk[LD4], rv[LD4];
  auto tile_load = [&](const float* src, float4* reg, bool mask_rows) {
#pragma unroll
    for (int i = 0; i < LD4; ++i) {
      const int idx = tid + NT * i;
      const int j = idx / (DP / 4);
      const int a4 = (idx % (DP / 4)) * 4;
      float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
      if (FAST || (idx < TILE4 && j < n && a4 < d && (!mask_rows || valid(j))))
        val = folx_ld_stream4(src + base + (int64_t)j * tok + a4);  // every tile is read once
      reg[i] = val;
    }
  };
  auto tile_store = [&](float* dst, const float4* reg) {
#pragma unroll
    for (int i = 0; i < LD4; ++i) {
      const int idx = tid + NT * i;
      const int j = idx / (DP / 4);
      const int a4 = (idx % (DP / 4)) * 4;
      if (FAST || idx < TILE4) *reinterpret_cast<float4*>(dst + j * DS + a4) = reg[i];
    }
  };
  // A-operand registers of this wavefront's 16 rows of an (n x d) array:
  // reg[t] = src[row][4 lg + 16 t .. + 3]
  const int qrow = 16 * w + l16;
  auto rows_load = [&](const float* src, float4* reg, bool mask_rows) {
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      const int a4 = 4 * lg + 16 * t;
      float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
      if (FAST || (qrow < n && a4 < d && (!mask_rows || valid(qrow))))
        val = folx_ld_stream4(src + base + (int64_t)qrow * tok + a4);
      reg[t] = val;
    }
  };

  // ---- forward ---------------------------------------------------------------------------
  tile_load(a.k, rk, false);
  tile_load(a.v, rv, false);
  tile_store(ks, rk);
  tile_store(vs, rv);
  float4 qa[DT];
  rows_load(a.q, qa, false);
  __syncthreads();

  bool rvalid[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) rvalid[r] = valid(16 * w + 4 * lg + r);
  bool cvalid[NW], cexist[NW];
#pragma unroll
  for (int jt = 0; jt < NW; ++jt) { cexist[jt] = FAST || (16 * jt + l16) < n; cvalid[jt] = valid(16 * jt + l16); }

  // s = q k^T  (A = q registers, B = k from LDS)
  auto qk_product = [&](const float4* areg, const float* btile, floatx4* acc) {
#pragma unroll
    for (int jt = 0; jt < NW; ++jt) {
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        const float4 bv = *reinterpret_cast<const float4*>(&btile[(16 * jt + l16) * DS + 4 * lg + 16 * t]);
#pragma unroll
        for (int r = 0; r < 4; ++r)
          acc[jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(f4get(areg[t], r), f4get(bv, r), acc[jt], 0, 0, 0);
      }
    }
  };
  // o = p v  (A = p-like registers [NW float4], B = v-like tile from LDS)
  auto pv_product = [&](const float4* areg, const float* btile, floatx4* acc) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int t = 0; t < NW; ++t) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float bv = btile[(4 * lg + 16 * t + r) * DS + 16 * dt + l16];
          acc[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(f4get(areg[t], r), bv, acc[dt], 0, 0, 0);
        }
      }
    }
  };
  // result layout (row 4 lg + r, column 16 jt + l16) -> A-operand layout through LDS
  auto to_a_layout = [&](const floatx4* c, float4* areg) {
    float* st = pst[w];
#pragma unroll
    for (int jt = 0; jt < NW; ++jt)
#pragma unroll
      for (int r = 0; r < 4; ++r) st[(4 * lg + r) * NS + 16 * jt + l16] = c[jt][r];
    // The tile is private to this wavefront, whose LDS accesses complete in issue order:
    // a wavefront-scope fence (no reordering by the compiler) is all the exchange needs.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int t = 0; t < NW; ++t) areg[t] = *reinterpret_cast<const float4*>(&st[l16 * NS + 4 * lg + 16 * t]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  floatx4 pc[NW];  // softmax probabilities, result layout
  {
    floatx4 s[NW];
#pragma unroll
    for (int jt = 0; jt < NW; ++jt) s[jt] = floatx4{0.f, 0.f, 0.f, 0.f};
    qk_product(qa, ks, s);
    if constexpr (EDGE) edge_add(a.e, s);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float mx = -INFINITY;
#pragma unroll
      for (int jt = 0; jt < NW; ++jt) {
        float sv = s[jt][r];
        if (!cexist[jt]) sv = -INFINITY;
        else if (!(rvalid[r] && cvalid[jt])) sv = -BIG;
        s[jt][r] = sv;
        mx = fmaxf(mx, sv);
      }
      mx = max16(mx);
      float sum = 0.0f;
#pragma unroll
      for (int jt = 0; jt < NW; ++jt) {
        const float e = cexist[jt] ? expf(s[jt][r] - mx) : 0.0f;
        s[jt][r] = e;
        sum += e;
      }
      sum = sum16(sum);
      const float inv = 1.0f / sum;
#pragma unroll
      for (int jt = 0; jt < NW; ++jt) pc[jt][r] = s[jt][r] * inv;
    }
  }
  float4 pa[NW];
  to_a_layout(pc, pa);

  floatx4 oc[DT];  // o, result layout: row 4 lg + r, column 16 dt + l16
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) oc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  pv_product(pa, vs, oc);
  // per-lane offset of (row 16 w + 4 lg, column l16) inside one (n, H, d) slice
  const int64_t out_off = base + (int64_t)(16 * w + 4 * lg) * tok + l16;
  auto out_store = [&](float* dst, const floatx4* c) {
    if constexpr (FAST) {
      float* p = dst + out_off;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) __builtin_nontemporal_store(c[dt][r], &p[16 * dt]);
        p += tok;
      }
    } else {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = 16 * w + 4 * lg + r, col = 16 * dt + l16;
          if (row < n && col < d) dst[base + (int64_t)row * tok + col] = c[dt][r];
        }
    }
  };
  out_store(a.o, oc);

  // ---- Jacobian rows and Laplacian -------------------------------------------------------
  floatx4 G[NW], X[NW], O2[DT], OL[DT];
  float u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int jt = 0; jt < NW; ++jt) { G[jt] = floatx4{0.f, 0.f, 0.f, 0.f}; X[jt] = G[jt]; }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) { O2[dt] = floatx4{0.f, 0.f, 0.f, 0.f}; OL[dt] = O2[dt]; }

  // pass c < P: Jacobian row c; pass c == P: the Laplacians take the place of the row
  auto active = [&](int c) -> bool {
    if constexpr (FAST) return true;
    return c == P || a.imask == nullptr || a.imask[(int64_t)c * B + b] != 0;
  };
  auto src_of = [&](const float* jac, const float* lap, int c) -> const float* {
    return c == P ? lap : jac + (int64_t)c * slice;
  };

  float4 qja[DT];
  if (active(0)) {
    tile_load(src_of(a.kj, a.kl, 0), rk, true);
    tile_load(src_of(a.vj, a.vl, 0), rv, true);
    rows_load(src_of(a.qj, a.ql, 0), qja, true);
    tile_store(kjs1, rk);
    tile_store(vjs1, rv);
  }
  __syncthreads();

  for (int c = 0; c <= P; ++c) {
    const bool act = active(c);
    const bool nact = c < P && active(c + 1);
    float4 qjn[DT];
    if (nact) {
      tile_load(src_of(a.kj, a.kl, c + 1), rk, true);
      tile_load(src_of(a.vj, a.vl, c + 1), rv, true);
      rows_load(src_of(a.qj, a.ql, c + 1), qjn, true);
    }
    if (act) {
      const bool is_lap = c == P;
      // s'_c = q'_c k^T + q k'_c^T ;  G += q'_c k'_c^T
      floatx4 sj[NW];
#pragma unroll
      for (int jt = 0; jt < NW; ++jt) sj[jt] = floatx4{0.f, 0.f, 0.f, 0.f};
      qk_product(qja, ks, sj);
      qk_product(qa, kjs1, sj);
      if constexpr (EDGE) edge_add(is_lap ? a.el : a.ej + (int64_t)c * eslice, sj);
      if (!is_lap) qk_product(qja, kjs1, G);
      // p'_c = p * (s'_c - rowsum(p s'_c))
      floatx4 pj[NW];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float rs = 0.0f;
#pragma unroll
        for (int jt = 0; jt < NW; ++jt) rs += pc[jt][r] * sj[jt][r];
        rs = sum16(rs);
        float us = 0.0f;
#pragma unroll
        for (int jt = 0; jt < NW; ++jt) {
          const float dlt = sj[jt][r] - rs;
          const float pv = pc[jt][r] * dlt;
          pj[jt][r] = pv;
          if (!is_lap) { X[jt][r] += pv * dlt; us += pv * sj[jt][r]; }
        }
        u[r] += us;  // lane-partial; reduced over the 16-lane group at the end
      }
      float4 pja[NW];
      to_a_layout(pj, pja);
      // o'_c = p v'_c + p'_c v ;  O2 += p'_c v'_c
      floatx4 ojc[DT];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) ojc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
      pv_product(pa, vjs1, ojc);
      pv_product(pja, vs, ojc);
      if (!is_lap) {
        pv_product(pja, vjs1, O2);
        out_store(a.oj + (int64_t)c * slice, ojc);
      } else {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) OL[dt] = ojc[dt];
      }
    } else {
      // inactive coordinate: its Jacobian row is zero and it adds nothing to the Laplacian
      floatx4 z[DT];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) z[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
      out_store(a.oj + (int64_t)c * slice, z);
    }
    __syncthreads();  // every wavefront is done with the current k', v' tiles
    if (nact) {
      tile_store(kjs1, rk);
      tile_store(vjs1, rv);
#pragma unroll
      for (int t = 0; t < DT; ++t) qja[t] = qjn[t];
    }
    __syncthreads();
  }

  // ---- second-order part:  [X + p * (2 G - u - rowsum(2 p G))] v + 2 O2 ------------------
  floatx4 pi[NW];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float ur = sum16(u[r]);
    float rs = 0.0f;
#pragma unroll
    for (int jt = 0; jt < NW; ++jt) rs += pc[jt][r] * 2.0f * G[jt][r];
    rs = sum16(rs);
#pragma unroll
    for (int jt = 0; jt < NW; ++jt) pi[jt][r] = X[jt][r] + pc[jt][r] * (2.0f * G[jt][r] - ur - rs);
  }
  float4 pia[NW];
  to_a_layout(pi, pia);
  pv_product(pia, vs, OL);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 4; ++r) OL[dt][r] += 2.0f * O2[dt][r];
  out_store(a.ol, OL);
}

template <int NW, int DT>
int launch_mhsa(hipStream_t st, const MhsaArgs& a) {
  const int64_t blocks = a.B * a.H;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  const bool fast = a.n == 16 * NW && a.d == 16 * DT && a.mask == nullptr && a.imask == nullptr;
  const dim3 grid((unsigned)blocks), block(FOLX_WAVE * NW);
  if (a.e != nullptr) {
    if (fast) mhsa_kernel<NW, DT, true, true><<<grid, block, 0, st>>>(a);
    else mhsa_kernel<NW, DT, true, false><<<grid, block, 0, st>>>(a);
  } else {
    if (fast) mhsa_kernel<NW, DT, false, true><<<grid, block, 0, st>>>(a);
    else mhsa_kernel<NW, DT, false, false><<<grid, block, 0, st>>>(a);
  }
  return folx_launch_status();
}

template <int NW>
int launch_mhsa_d(hipStream_t st, const MhsaArgs& a) {
  const int dt = (a.d + 15) / 16;
  switch (dt) {
    case 1: return launch_mhsa<NW, 1>(st, a);
    case 2: return launch_mhsa<NW, 2>(st, a);
    case 3: return launch_mhsa<NW, 3>(st, a);
    default: return launch_mhsa<NW, 4>(st, a);
  }
}

}  // namespace

static int mhsa_entry(void* stream, const float* q, const float* q_jac, const float* q_lap,
                      const float* k, const float* k_jac, const float* k_lap, const float* v,
                      const float* v_jac, const float* v_lap, const float* e, const float* e_jac,
                      const float* e_lap, const uint8_t* mask, const uint8_t* input_mask, float* o,
                      float* o_jac, float* o_lap, int64_t B, int32_t n, int32_t H, int32_t d,
                      int32_t P) {
  if (B < 0 || n <= 0 || H <= 0 || d <= 0 || P < 0) return FOLX_HIP_EINVAL;
  if (B == 0) return FOLX_HIP_OK;
  if (!q || !q_lap || !k || !k_lap || !v || !v_lap || !o || !o_lap) return FOLX_HIP_EINVAL;
  if (P > 0 && (!q_jac || !k_jac || !v_jac || !o_jac)) return FOLX_HIP_EINVAL;
  if (e != nullptr && (!e_lap || (P > 0 && !e_jac))) return FOLX_HIP_EINVAL;
  if (n > 64 || d > 64 || d % 4 != 0) return FOLX_HIP_ENOTSUP;
  const float* ptrs[] = {q, q_jac, q_lap, k, k_jac, k_lap, v, v_jac, v_lap};
  for (const float* p : ptrs)
    if (p && !folx_aligned16(p)) return FOLX_HIP_ENOTSUP;
  MhsaArgs a{q, q_jac, q_lap, k, k_jac, k_lap, v, v_jac, v_lap, e, e_jac, e_lap, mask, input_mask,
             o, o_jac, o_lap, B, n, H, d, P};
  hipStream_t st = (hipStream_t)stream;
  const int nw = (n + 15) / 16;
  switch (nw) {
    case 1: return launch_mhsa_d<1>(st, a);
    case 2: return launch_mhsa_d<2>(st, a);
    case 3: return launch_mhsa_d<3>(st, a);
    default: return launch_mhsa_d<4>(st, a);
  }
}

extern "C" int folx_hip_mhsa_fwdlap(void* stream, const float* q, const float* q_jac,
                                    const float* q_lap, const float* k, const float* k_jac,
                                    const float* k_lap, const float* v, const float* v_jac,
                                    const float* v_lap, const uint8_t* mask,
                                    const uint8_t* input_mask, float* o, float* o_jac, float* o_lap,
                                    int64_t B, int32_t n, int32_t H, int32_t d, int32_t P) {
  return mhsa_entry(stream, q, q_jac, q_lap, k, k_jac, k_lap, v, v_jac, v_lap, nullptr, nullptr, nullptr,
                    mask, input_mask, o, o_jac, o_lap, B, n, H, d, P);
}

extern "C" int folx_hip_mhsea_fwdlap(void* stream, const float* q, const float* q_jac,
                                     const float* q_lap, const float* k, const float* k_jac,
                                     const float* k_lap, const float* e, const float* e_jac,
                                     const float* e_lap, const float* v, const float* v_jac,
                                     const float* v_lap, const uint8_t* mask,
                                     const uint8_t* input_mask, float* o, float* o_jac, float* o_lap,
                                     int64_t B, int32_t n, int32_t H, int32_t d, int32_t P) {
  if (!e) return FOLX_HIP_EINVAL;
  return mhsa_entry(stream, q, q_jac, q_lap, k, k_jac, k_lap, v, v_jac, v_lap, e, e_jac, e_lap, mask,
                    input_mask, o, o_jac, o_lap, B, n, H, d, P);
}
