// Multi-head self attention with Laplacian for q, k, v whose Jacobians are still sparse by
// position: sequence position e depends on its own few input coordinates only (the first
// attention layer of a PsiFormer, where the inputs of electron e are its three coordinates),
// so the dense Jacobian row c = index[s][e] of q, k and v is zero except in row e.
// The output is dense (every output position depends on every electron), but with
//   a = q'_c[e], b = k'_c[e], w = v'_c[e]     alpha[j] = a . k[j]     beta[i] = q[i] . b
// the rule of the dense kernel (s'_c = q'_c k^T + q k'_c^T, p'_c = p * (s'_c - rowsum(p s'_c)),
// o'_c = p v'_c + p'_c v, ...) collapses to vector work per Jacobian row:
//   s'_c[i][j] = [i = e] alpha[j] + beta[i] [j = e]
//   r_c[i]     = [i = e] rho + p[i][e] beta[i],            rho = sum_j p[e][j] alpha[j]
//   o'_c[i]    = p[i][e] (w + beta[i] (v[e] - o[i])) + [i = e] gamma,
//                gamma = sum_j p[e][j] alpha[j] (v[j] - o[e])
// and the second-order part of the Laplacian needs, besides n x n sums of squares of alpha and
// beta, a single n x n x d product:
//   lap_o = p lap_v + (pL + M) v + 2 sum_c p'_c[:, e] w_c
//   M     = p * (T2 - rowsum(p T2) + 2 g (I - diag(p))),   T2 = sum_c (s'_c - r_c)^2,
//   g[e]  = sum_s a_s . b_s,   pL = p * (sL - rowsum(p sL)),   sL = lap_q k^T + q lap_k^T.
// That is O(n^2 d) work per (walker, head) instead of O(P n^2 d); the kernel is bound by
// writing the dense P x n x d output rows.
//
// One workgroup of 512 threads per (walker, head); q, k, v, o, p and the n x n accumulators
// live in LDS (rows of d + 4 floats, so that 16 threads reading 16 bytes each from 16
// different rows cover all banks); the n x n x d products (scores, alpha, beta, the Laplacian's
// score term) run on the matrix cores from those rows, the sums over j on 128-bit LDS reads; the
// vectors of the next group of positions are fetched while the current one is worked on.
#include <atomic>

#include "common.h"

namespace {

struct SAArgs {
  const float *q, *qs, *ql, *k, *ks, *kl, *v, *vs, *vl;
  const int32_t* index;  // [K][n] dense Jacobian row of slot s at position e, or -1
  float *o, *oj, *ol;
  int64_t B;
  int32_t n, H, d, K;
};

constexpr int SA_NT = 512;  // two workgroups per CU (LDS and 128 registers): four wavefronts per SIMD
constexpr int SA_RP = SA_NT / 16;  // output rows per pass: 16 threads of 16 bytes cover a row of d <= 64

// dot product of two 16-byte aligned LDS vectors of 4 * d4 floats
__device__ __forceinline__ float sa_dot(const float* u, const float* m, int d4) {
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
#pragma unroll 4
  for (int t = 0; t < d4; ++t) {
    const float4 x = *reinterpret_cast<const float4*>(u + 4 * t);
    const float4 y = *reinterpret_cast<const float4*>(m + 4 * t);
    s0 += x.x * y.x; s1 += x.y * y.y; s2 += x.z * y.z; s3 += x.w * y.w;
  }
  return (s0 + s1) + (s2 + s3);
}
constexpr int SA_MAXPASS = 64 / SA_RP;  // n <= 64: rows i = SA_RP pass + tid / 16
constexpr int SA_E = 4;        // sequence positions worked on together

typedef float floatx4 __attribute__((ext_vector_type(4)));

// Workgroup barrier for data exchanged through LDS only.  __syncthreads() also waits for every
// global load and store of the wavefront to complete (its fence covers global memory), which
// here would expose the latency of the vectors requested one group ahead and of the output
// rows just stored, once per group.
__device__ __forceinline__ void sa_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// One 16 x 16 tile of X Y^T on the matrix cores (v_mfma_f32_16x16x4_f32): X and Y are row-major in
// LDS, C[r][c] = sum_k X[r][k] Y[c][k] over k < 4 * d4.  Lane l feeds X[l % 16][4 s + l / 16] and
// Y[l % 16][4 s + l / 16] in step s and receives C[4 (l / 16) + i][l % 16] in register i.  With row
// strides of 4 (mod 32) floats the 64 reads of a step fall on all banks twice, the minimum.  Rows
// past the end of X or Y (still inside the workgroup's LDS: every operand is followed by other
// arrays) only reach tile rows / columns that the caller does not keep.
__device__ __forceinline__ floatx4 sa_tile_nt(const float* X, int ldx, const float* Y, int ldy, int d4, int lane) {
  const float* xp = X + (lane % 16) * ldx + lane / 16;
  const float* yp = Y + (lane % 16) * ldy + lane / 16;
  // four accumulators, steps dealt round: independent chains for the matrix pipe, and a quarter
  // as many roundings in a row for every element (the partial sums are added pairwise)
  floatx4 c0 = {0.0f, 0.0f, 0.0f, 0.0f}, c1 = c0, c2 = c0, c3 = c0;
  int s = 0;
  for (; s + 8 <= d4; s += 8) {  // the operands of eight steps are read before the first product
    float xv[8], yv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) { xv[u] = xp[4 * (s + u)]; yv[u] = yp[4 * (s + u)]; }
#pragma unroll
    for (int u = 0; u < 8; u += 4) {
      c0 = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[u], yv[u], c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[u + 1], yv[u + 1], c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[u + 2], yv[u + 2], c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[u + 3], yv[u + 3], c3, 0, 0, 0);
    }
  }
  for (; s < d4; ++s) c0 = __builtin_amdgcn_mfma_f32_16x16x4f32(xp[4 * s], yp[4 * s], c0, 0, 0, 0);
  return (c0 + c1) + (c2 + c3);
}

// Two products at once, C0 = X0 Y0^T (rows < nr0 of X0, rows < nc0 of Y0) and C1 = X1 Y1^T, their
// 16 x 16 tiles dealt to the workgroup's wavefronts as one list; `put(which, r, c, value)`
// receives every element.  (One product: nr1 = 0.)
template <class Put>
__device__ __forceinline__ void sa_products_nt(const float* X0, int ldx0, int nr0, const float* Y0, int ldy0, int nc0,
                                               const float* X1, int ldx1, int nr1, const float* Y1, int ldy1, int nc1,
                                               int d4, int tid, Put put) {
  const int lane = tid % 64, wave = tid / 64;
  const int tc0 = (nc0 + 15) / 16, t0 = ((nr0 + 15) / 16) * tc0;
  const int tc1 = (nc1 + 15) / 16, t1 = ((nr1 + 15) / 16) * tc1;
  for (int t = wave; t < t0 + t1; t += SA_NT / 64) {
    const bool second = t >= t0;
    const int tt = second ? t - t0 : t, tc = second ? tc1 : tc0;
    const int r0 = (tt / tc) * 16, c0 = (tt % tc) * 16;
    const float* X = second ? X1 : X0;
    const float* Y = second ? Y1 : Y0;
    const int ldx = second ? ldx1 : ldx0, ldy = second ? ldy1 : ldy0;
    const floatx4 c = sa_tile_nt(X + r0 * ldx, ldx, Y + c0 * ldy, ldy, d4, lane);
    const int col = c0 + lane % 16;
    const int nr = second ? nr1 : nr0, nc = second ? nc1 : nc0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = r0 + 4 * (lane / 16) + i;
      if (row < nr && col < nc) put(second, row, col, c[i]);
    }
  }
}

template <class Put>
__device__ __forceinline__ void sa_product_nt(const float* X, int ldx, int nr, const float* Y, int ldy, int nc,
                                              int d4, int tid, Put put) {
  sa_products_nt(X, ldx, nr, Y, ldy, nc, X, ldx, 0, Y, ldy, 0, d4, tid,
                 [&](bool, int r, int c, float v) { put(r, c, v); });
}

__host__ __device__ inline int64_t sa_lds_floats(int n, int d, int K) {
  const int dp = d + 4, np1 = n + 1;
  return 4LL * n * dp + 4LL * n * np1 + SA_E * (2LL * K * dp + 2LL * K * d + 2LL * K * n + 2LL * K) + 5LL * n +
         (int64_t)K * n;
}

__global__ __launch_bounds__(SA_NT, 4) void mhsa_sparse_kernel(SAArgs a) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int n = a.n, d = a.d, K = a.K, H = a.H;
  const int dp = d + 4, np1 = n + 1, d4 = d / 4;
  float* qS = sm;
  float* kS = qS + n * dp;
  float* vS = kS + n * dp;
  float* oS = vS + n * dp;
  float* pS = oS + n * dp;
  float* AA = pS + n * np1;
  float* BB = AA + n * np1;
  float* AR = BB + n * np1;
  float* aS = AR + n * np1;             // [SA_E][K][dp] vectors a, b of the positions in work (MFMA operands)
  float* bS = aS + SA_E * K * dp;
  float* wS = bS + SA_E * K * dp;       // [SA_E][K][d]
  float* gamS = wS + SA_E * K * d;
  float* alS = gamS + SA_E * K * d;     // [SA_E][K][n]
  float* beS = alS + SA_E * K * n;
  float* rhoS = beS + SA_E * K * n;     // [SA_E][K]
  float* gpS = rhoS + SA_E * K;         // [SA_E][K] a_s . b_s
  float* D1 = gpS + SA_E * K;
  float* D2 = D1 + n;
  float* R2a = D2 + n;
  float* gS = R2a + n;
  float* rsum = gS + n;
  int* idxS = reinterpret_cast<int*>(rsum + n);  // [K][n] copy of the index table

  const int tid = threadIdx.x;
  const int64_t b = blockIdx.x / H;
  const int h = (int)(blockIdx.x % H);
  const int64_t Srow = a.B * n * (int64_t)H * d;  // elements per Jacobian row
  auto grow = [&](int i) -> int64_t { return ((b * n + i) * (int64_t)H + h) * d; };
  auto load_tile = [&](const float* src, float* dst) {
    for (int it = tid; it < n * d4; it += SA_NT) {
      const int i = it / d4, t4 = it - i * d4;
      const float4 t = *reinterpret_cast<const float4*>(src + grow(i) + 4 * t4);
      *reinterpret_cast<float4*>(dst + i * dp + 4 * t4) = t;
    }
  };

  load_tile(a.q, qS);
  load_tile(a.k, kS);
  load_tile(a.v, vS);
  for (int it = tid; it < 3 * n * np1; it += SA_NT) AA[it] = 0.0f;  // AA, BB, AR are contiguous
  for (int it = tid; it < K * n; it += SA_NT) idxS[it] = a.index[it];
  sa_barrier();

  // p = softmax(q k^T)
  sa_product_nt(qS, dp, n, kS, dp, n, d4, tid, [&](int i, int j, float v) { pS[i * np1 + j] = v; });
  sa_barrier();
  if (tid < n) {
    float* row = pS + tid * np1;
    float m = row[0];
    for (int j = 1; j < n; ++j) m = fmaxf(m, row[j]);
    float z = 0.0f;
    for (int j = 0; j < n; ++j) { const float ex = expf(row[j] - m); row[j] = ex; z += ex; }
    const float rz = 1.0f / z;
    for (int j = 0; j < n; ++j) row[j] *= rz;
  }
  sa_barrier();
  // o = p v
  for (int it = tid; it < n * d4; it += SA_NT) {
    const int i = it / d4, t4 = it - i * d4;
    // four partial sums (keys j % 4), added pairwise: a quarter as many roundings in a row, which
    // the Jacobian rows feel through v - o
    float4 part[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) part[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    int j = 0;
    for (; j + 4 <= n; j += 4) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float pij = pS[i * np1 + j + u];
        const float4 vv = *reinterpret_cast<const float4*>(vS + (j + u) * dp + 4 * t4);
        part[u].x = fmaf(pij, vv.x, part[u].x); part[u].y = fmaf(pij, vv.y, part[u].y);
        part[u].z = fmaf(pij, vv.z, part[u].z); part[u].w = fmaf(pij, vv.w, part[u].w);
      }
    }
    for (; j < n; ++j) {
      const float pij = pS[i * np1 + j];
      const float4 vv = *reinterpret_cast<const float4*>(vS + j * dp + 4 * t4);
      part[0].x = fmaf(pij, vv.x, part[0].x); part[0].y = fmaf(pij, vv.y, part[0].y);
      part[0].z = fmaf(pij, vv.z, part[0].z); part[0].w = fmaf(pij, vv.w, part[0].w);
    }
    const float4 acc = make_float4((part[0].x + part[1].x) + (part[2].x + part[3].x),
                                   (part[0].y + part[1].y) + (part[2].y + part[3].y),
                                   (part[0].z + part[1].z) + (part[2].z + part[3].z),
                                   (part[0].w + part[1].w) + (part[2].w + part[3].w));
    *reinterpret_cast<float4*>(oS + i * dp + 4 * t4) = acc;
    *reinterpret_cast<float4*>(a.o + grow(i) + 4 * t4) = acc;
  }

  // The vectors (a, b, w) of every slot of SA_E consecutive positions form one group: one
  // float4 per thread and position, requested one group ahead of its use.
  const int nvec = 3 * K * d4;
  const int pf_which = tid / (K * d4), pf_sl = (tid / d4) % K, pf_t4 = tid % d4;
  // this thread's source array and offset inside a position's vectors, in registers (selected once:
  // an array chosen per lane inside the loop would be read from the argument block with a
  // vector load, a memory round trip in front of every request)
  const float* pf_src = a.qs;
  if (pf_which == 1) pf_src = a.ks;
  if (pf_which == 2) pf_src = a.vs;
  pf_src += pf_sl * Srow + 4 * pf_t4;
  auto fetch = [&](int e0, float4 (&pf)[SA_E]) {
#pragma unroll
    for (int ee = 0; ee < SA_E; ++ee) {
      pf[ee] = make_float4(0.f, 0.f, 0.f, 0.f);
      const int e = e0 + ee;
      if (tid < nvec && e < n && idxS[pf_sl * n + e] >= 0)
        pf[ee] = *reinterpret_cast<const float4*>(pf_src + grow(e));
    }
  };
  sa_barrier();  // index table, o and p are in LDS
  float4 pf[SA_E];
  fetch(0, pf);

  float4 t2acc[SA_MAXPASS], oreg[SA_MAXPASS];
  const int orow = tid / 16, ot4 = tid % 16;
#pragma unroll
  for (int ps = 0; ps < SA_MAXPASS; ++ps) {
    t2acc[ps] = make_float4(0.f, 0.f, 0.f, 0.f);
    const int i = ps * SA_RP + orow;
    oreg[ps] = (i < n && ot4 < d4) ? *reinterpret_cast<const float4*>(oS + i * dp + 4 * ot4)
                                   : make_float4(0.f, 0.f, 0.f, 0.f);
  }

  for (int e0 = 0; e0 < n; e0 += SA_E) {
    const int ne = min(SA_E, n - e0);
    sa_barrier();  // everyone is done with the previous group's vectors
    if (tid < nvec) {
      const int ld = pf_which == 2 ? d : dp;
      float* dst = (pf_which == 0 ? aS : (pf_which == 1 ? bS : wS)) + pf_sl * ld + 4 * pf_t4;
#pragma unroll
      for (int ee = 0; ee < SA_E; ++ee) *reinterpret_cast<float4*>(dst + ee * K * ld) = pf[ee];
    }
    sa_barrier();
    if (e0 + SA_E < n) fetch(e0 + SA_E, pf);

    // alpha[e][s][j] = a_es . k[j],  beta[e][s][i] = q[i] . b_es,  gp[e][s] = a_es . b_es
    sa_products_nt(aS, dp, ne * K, kS, dp, n, bS, dp, ne * K, qS, dp, n, d4, tid,
                   [&](bool beta, int es, int x, float v) { (beta ? beS : alS)[es * n + x] = v; });
    if (tid >= SA_NT - ne * K) {  // the last wavefront has no tile when n <= 48
      const int es = SA_NT - 1 - tid;
      gpS[es] = sa_dot(aS + es * dp, bS + es * dp, d4);
    }
    sa_barrier();
    // rho[e][s] = sum_j p[e][j] alpha[e][s][j],  gamma[e][s] = sum_j p[e][j] alpha[e][s][j] (v[j] - o[e])
    for (int it = tid; it < ne * K * d4; it += SA_NT) {
      const int es = it / d4, t4 = it - es * d4;
      const int e = e0 + es / K;
      float rho = 0.0f;
      float4 gm = make_float4(0.f, 0.f, 0.f, 0.f);
      // gamma - rho o[e] summed as sum_j p alpha (v[j] - o[e]): the two parts nearly cancel
      const float4 oe = *reinterpret_cast<const float4*>(oS + e * dp + 4 * t4);
#pragma unroll 8
      for (int j = 0; j < n; ++j) {
        const float pa = pS[e * np1 + j] * alS[es * n + j];
        const float4 vv = *reinterpret_cast<const float4*>(vS + j * dp + 4 * t4);
        rho += pa;
        gm.x += pa * (vv.x - oe.x); gm.y += pa * (vv.y - oe.y);
        gm.z += pa * (vv.z - oe.z); gm.w += pa * (vv.w - oe.w);
      }
      *reinterpret_cast<float4*>(gamS + es * d + 4 * t4) = gm;
      if (t4 == 0) rhoS[es] = rho;
    }
    sa_barrier();

    // output rows of the group's slots, and their part of 2 sum_c p'_c[:, e] w_c
    if (ot4 < d4) {
      for (int ee = 0; ee < ne; ++ee) {
        const int e = e0 + ee;
        const float4 v4 = *reinterpret_cast<const float4*>(vS + e * dp + 4 * ot4);
        float pie[SA_MAXPASS];
#pragma unroll
        for (int ps = 0; ps < SA_MAXPASS; ++ps) pie[ps] = (ps * SA_RP + orow < n) ? pS[(ps * SA_RP + orow) * np1 + e] : 0.0f;
        for (int sl = 0; sl < K; ++sl) {
          const int c = idxS[sl * n + e];
          if (c < 0) continue;
          const int es = ee * K + sl;
          const float rho = rhoS[es];
          const float ale = alS[es * n + e];
          const float4 w4 = *reinterpret_cast<const float4*>(wS + es * d + 4 * ot4);
          const float4 g4 = *reinterpret_cast<const float4*>(gamS + es * d + 4 * ot4);
          float* dst = a.oj + (int64_t)c * Srow + 4 * ot4;
#pragma unroll
          for (int ps = 0; ps < SA_MAXPASS; ++ps) {
            const int i = ps * SA_RP + orow;
            if (i < n) {
              const float bi = beS[es * n + i];
              const float4 oi = oreg[ps];
              float4 r;
              r.x = pie[ps] * (w4.x + bi * (v4.x - oi.x));
              r.y = pie[ps] * (w4.y + bi * (v4.y - oi.y));
              r.z = pie[ps] * (w4.z + bi * (v4.z - oi.z));
              r.w = pie[ps] * (w4.w + bi * (v4.w - oi.w));
              float cf = pie[ps] * bi * (1.0f - pie[ps]);
              if (i == e) {
                r.x += g4.x; r.y += g4.y; r.z += g4.z; r.w += g4.w;
                cf += pie[ps] * (ale - rho);
              }
              folx_st_stream4(dst + grow(i), r);
              t2acc[ps].x += cf * w4.x; t2acc[ps].y += cf * w4.y;
              t2acc[ps].z += cf * w4.z; t2acc[ps].w += cf * w4.w;
            }
          }
        }
      }
    }
    // n x n sums over the slots of each position of the group
    for (int it = tid; it < ne * n; it += SA_NT) {
      const int ee = it / n, j = it - ee * n;
      const int e = e0 + ee;
      const float pee = pS[e * np1 + e];
      float aa = 0.0f, ar = 0.0f, bb = 0.0f;
      for (int sl = 0; sl < K; ++sl) {
        const int es = ee * K + sl;
        const float al = alS[es * n + j], be = beS[es * n + j];
        const float rr = rhoS[es] + pee * beS[es * n + e];
        aa += al * al;
        ar += al * rr;
        bb += be * be;
      }
      AA[e * np1 + j] = aa;
      AR[e * np1 + j] = ar;
      BB[j * np1 + e] = bb;
    }
    if (tid >= SA_NT - ne) {
      const int ee = SA_NT - 1 - tid;
      const int e = e0 + ee;
      const float pee = pS[e * np1 + e];
      float d1 = 0.0f, d2 = 0.0f, r2 = 0.0f, g = 0.0f;
      for (int sl = 0; sl < K; ++sl) {
        const int es = ee * K + sl;
        const float ale = alS[es * n + e], bee = beS[es * n + e], rho = rhoS[es];
        d1 += 2.0f * ale * bee;
        d2 += bee * rho;
        r2 += rho * rho + 2.0f * rho * pee * bee;
        g += gpS[es];
      }
      D1[e] = d1; D2[e] = d2; R2a[e] = r2; gS[e] = g;
    }
  }
  sa_barrier();

  // T2 = S2 - 2 SR + R2, then M (kept in AA)
  if (tid < n) {
    const int i = tid;
    float r2 = R2a[i];
    for (int e = 0; e < n; ++e) { const float pe = pS[i * np1 + e]; r2 += pe * pe * BB[i * np1 + e]; }
    R2a[i] = r2;
  }
  sa_barrier();
  for (int it = tid; it < n * n; it += SA_NT) {
    const int i = it / n, j = it - i * n;
    const int x = i * np1 + j;
    float s2 = AA[x] + BB[x], sr = AR[x] + pS[x] * BB[x];
    if (i == j) { s2 += D1[i]; sr += D2[i]; }
    AA[x] = s2 - 2.0f * sr + R2a[i];
  }
  load_tile(a.ql, oS);  // o is not needed any more
  sa_barrier();
  if (tid < n) {
    const int i = tid;
    float s = 0.0f;
    for (int j = 0; j < n; ++j) s += pS[i * np1 + j] * AA[i * np1 + j];
    rsum[i] = s;
  }
  // sL = lap_q k^T (into BB, whose sums of beta^2 are used up)
  sa_product_nt(oS, dp, n, kS, dp, n, d4, tid, [&](int i, int j, float v) { BB[i * np1 + j] = v; });
  sa_barrier();
  for (int it = tid; it < n * n; it += SA_NT) {
    const int i = it / n, j = it - i * n;
    const int x = i * np1 + j;
    const float pij = pS[x];
    AA[x] = pij * (AA[x] - rsum[i] + 2.0f * gS[i] * ((i == j ? 1.0f : 0.0f) - pS[i * np1 + i]));
  }
  load_tile(a.kl, oS);  // lap_q has been consumed; k itself is not needed any more
  sa_barrier();
  sa_product_nt(qS, dp, n, oS, dp, n, d4, tid, [&](int i, int j, float v) { BB[i * np1 + j] += v; });
  sa_barrier();
  if (tid < n) {
    const int i = tid;
    float s = 0.0f;
    for (int j = 0; j < n; ++j) s += pS[i * np1 + j] * BB[i * np1 + j];
    rsum[i] = s;
  }
  load_tile(a.vl, qS);  // q is not needed any more
  sa_barrier();
  for (int it = tid; it < n * n; it += SA_NT) {
    const int i = it / n, j = it - i * n;
    const int x = i * np1 + j;
    AA[x] += pS[x] * (BB[x] - rsum[i]);  // pL + M
  }
  sa_barrier();
  // lap_o = p lap_v + (pL + M) v + 2 sum_c p'_c[:, e] w_c
  if (ot4 < d4) {
#pragma unroll
    for (int ps = 0; ps < SA_MAXPASS; ++ps) {
      const int i = ps * SA_RP + orow;
      if (i < n) {
        float r[4] = {2.0f * t2acc[ps].x, 2.0f * t2acc[ps].y, 2.0f * t2acc[ps].z, 2.0f * t2acc[ps].w};
#pragma unroll 4
        for (int j = 0; j < n; ++j) {
          const float pij = pS[i * np1 + j], mij = AA[i * np1 + j];
          const float4 vl = *reinterpret_cast<const float4*>(qS + j * dp + 4 * ot4);
          const float4 vv = *reinterpret_cast<const float4*>(vS + j * dp + 4 * ot4);
          r[0] += pij * vl.x + mij * vv.x; r[1] += pij * vl.y + mij * vv.y;
          r[2] += pij * vl.z + mij * vv.z; r[3] += pij * vl.w + mij * vv.w;
        }
        *reinterpret_cast<float4*>(a.ol + grow(i) + 4 * ot4) = make_float4(r[0], r[1], r[2], r[3]);
      }
    }
  }
}

}  // namespace

extern "C" int folx_hip_mhsa_sparse_fwdlap(void* stream, const float* q, const float* q_jac, const float* q_lap,
                                           const float* k, const float* k_jac, const float* k_lap, const float* v,
                                           const float* v_jac, const float* v_lap, const int32_t* index, float* o,
                                           float* o_jac, float* o_lap, int64_t B, int32_t n, int32_t H, int32_t d,
                                           int32_t k_rows) {
  if (B < 0 || n <= 0 || H <= 0 || d <= 0 || k_rows <= 0) return FOLX_HIP_EINVAL;
  if (B == 0) return FOLX_HIP_OK;
  if (!q || !q_jac || !q_lap || !k || !k_jac || !k_lap || !v || !v_jac || !v_lap || !index || !o || !o_jac || !o_lap)
    return FOLX_HIP_EINVAL;
  if (n > SA_RP * SA_MAXPASS || d > 64 || d % 4 != 0 || k_rows > 8 || 3 * k_rows * (d / 4) > SA_NT)
    return FOLX_HIP_ENOTSUP;
  const void* ptrs[] = {q, q_jac, q_lap, k, k_jac, k_lap, v, v_jac, v_lap, o, o_jac, o_lap};
  for (const void* p : ptrs)
    if (!folx_aligned16(p)) return FOLX_HIP_ENOTSUP;
  if (B * H > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  const size_t lds = (size_t)sa_lds_floats(n, d, k_rows) * sizeof(float);
  if (lds > 160 * 1024) return FOLX_HIP_ENOTSUP;
  if (lds > 64 * 1024) {
    // raised once per process to the largest size asked for so far (not a stream operation,
    // and then never issued again inside a stream capture)
    static std::atomic<size_t> granted{0};
    if (lds > granted.load()) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(mhsa_sparse_kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
        return FOLX_HIP_ENOTSUP;
      granted.store(160 * 1024);
    }
  }
  SAArgs a;
  a.q = q; a.qs = q_jac; a.ql = q_lap; a.k = k; a.ks = k_jac; a.kl = k_lap; a.v = v; a.vs = v_jac; a.vl = v_lap;
  a.index = index; a.o = o; a.oj = o_jac; a.ol = o_lap; a.B = B; a.n = n; a.H = H; a.d = d; a.K = k_rows;
  mhsa_sparse_kernel<<<dim3((unsigned)(B * H)), dim3(SA_NT), lds, (hipStream_t)stream>>>(a);
  return folx_launch_status();
}
