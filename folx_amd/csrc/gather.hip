// Re-indexing of sparse Jacobian rows between row frames.  The index masks are static and
// live on the host; the device only sees small int32 tables.  Both kernels stream the
// Jacobian once and are bound by HBM bandwidth.
#include "common.h"

namespace {

// out[t][b][so][si] = sum_s data[take[t][s][so]][b][so][si]   (take < 0: no source)
// Threads run along (so, si) in units of VEC floats so reads and writes are coalesced
// 128-bit accesses when S_inner allows; the table entries are read once per thread and
// reused for the WPT walkers the thread loops over (blockIdx.y selects the walker group).
constexpr int GATHER_WPT = 8;

template <int VEC>
__global__ __launch_bounds__(256) void gather_rows_kernel(const float* __restrict__ data,
                                                          const int32_t* __restrict__ take,
                                                          float* __restrict__ out, int32_t n_slots,
                                                          int64_t B, int64_t S_outer, int64_t S_inner) {
  const int64_t S = S_outer * S_inner;
  const int64_t e = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (e >= S) return;
  const int64_t so = e / S_inner;
  const int32_t t = blockIdx.z;
  int32_t src[8];
  const int32_t ns = n_slots < 8 ? n_slots : 8;
  for (int s = 0; s < ns; ++s) src[s] = take[((int64_t)t * n_slots + s) * S_outer + so];
  const int64_t b0 = (int64_t)blockIdx.y * GATHER_WPT;
  const int64_t b1 = b0 + GATHER_WPT < B ? b0 + GATHER_WPT : B;
  for (int64_t b = b0; b < b1; ++b) {
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
    for (int s = 0; s < n_slots; ++s) {
      const int32_t r = s < 8 ? src[s] : take[((int64_t)t * n_slots + s) * S_outer + so];
      if (r >= 0) {
        const float* p = data + ((int64_t)r * B + b) * S + e;
        if constexpr (VEC == 4) {
          const float4 v = *reinterpret_cast<const float4*>(p);
          acc[0] += v.x; acc[1] += v.y; acc[2] += v.z; acc[3] += v.w;
        } else {
          acc[0] += *p;
        }
      }
    }
    float* q = out + ((int64_t)t * B + b) * S + e;
    if constexpr (VEC == 4) *reinterpret_cast<float4*>(q) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    else *q = acc[0];
  }
}

// The same re-indexing with a SUM OVER AN AXIS of the data folded in: the sources of a target
// row are (row r, entry j of the reduced axis) pairs, encoded r * RED + j, and the data keeps its
// own layout [k][B][O][RED][IV][IC] (the reduced axis in the middle, the table constant along
// IC), so neither a slice of the reduced axis nor a permuted copy is formed:
//   out[t][b][o][iv][ic] = alpha * sum_s data[e / RED][b][o][e % RED][iv][ic],  e = take[t][s][o * IV + iv]
template <int VEC>
__global__ __launch_bounds__(256) void gather_reduce_rows_kernel(const float* __restrict__ data,
                                                                 const int32_t* __restrict__ take,
                                                                 float* __restrict__ out, int32_t n_slots,
                                                                 int64_t B, int64_t O, int32_t RED, int64_t IV,
                                                                 int64_t IC, float alpha) {
  const int64_t S_out = O * IV * IC;          // elements of one output row and walker
  const int64_t S_in = S_out * RED;           // elements of one input row and walker
  // a thread owns VEC consecutive floats of the (walker, o, iv, ic) space of one output row, so that
  // consecutive workgroups write consecutive memory
  const int64_t f = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (f >= B * S_out) return;
  const int64_t b = f / S_out, e = f - b * S_out;
  const int64_t q = e / IC, ic = e % IC;      // q = o * IV + iv
  const int64_t o = q / IV, iv = q % IV;
  const int32_t t = blockIdx.y;
  float acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
  // Eight slots at a time: first their table entries, then all their loads, then the sums in slot
  // order -- a slot-by-slot loop would wait for a table entry and then for its load, eight times over.
  for (int s0 = 0; s0 < n_slots; s0 += 8) {
    int32_t en[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      en[u] = s0 + u < n_slots ? take[((int64_t)t * n_slots + s0 + u) * (O * IV) + q] : -1;
    float val[8][VEC];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) val[u][v] = 0.0f;
      if (en[u] >= 0) {
        const int32_t r = en[u] / RED, j = en[u] % RED;
        const float* p = data + ((int64_t)r * B + b) * S_in + ((o * RED + j) * IV + iv) * IC + ic;
        if constexpr (VEC == 4) {
          const float4 v = folx_ld_stream4(p);
          val[u][0] = v.x; val[u][1] = v.y; val[u][2] = v.z; val[u][3] = v.w;
        } else {
          val[u][0] = *p;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] += val[u][v];
  }
  float* dst = out + ((int64_t)t * B + b) * S_out + e;
  if constexpr (VEC == 4) folx_st_stream4(dst, make_float4(alpha * acc[0], alpha * acc[1], alpha * acc[2], alpha * acc[3]));
  else *dst = alpha * acc[0];
}

// Flat form of gather_rows_kernel: a thread owns VEC consecutive floats of the (walker, so, si)
// space of one output row, so that consecutive workgroups write consecutive memory.
template <int VEC>
__global__ __launch_bounds__(256) void gather_rows_flat_kernel(const float* __restrict__ data,
                                                               const int32_t* __restrict__ take,
                                                               float* __restrict__ out, int32_t n_slots,
                                                               int64_t B, int64_t S_outer, int64_t S_inner) {
  const int64_t S = S_outer * S_inner;
  const int64_t f = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (f >= B * S) return;
  const int64_t b = f / S, e = f - b * S;
  const int64_t so = e / S_inner;
  const int32_t t = blockIdx.y;
  float acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
  for (int s = 0; s < n_slots; ++s) {
    const int32_t r = take[((int64_t)t * n_slots + s) * S_outer + so];
    if (r >= 0) {
      const float* p = data + ((int64_t)r * B + b) * S + e;
      if constexpr (VEC == 4) {
        const float4 v = folx_ld_stream4(p);
        acc[0] += v.x; acc[1] += v.y; acc[2] += v.z; acc[3] += v.w;
      } else {
        acc[0] += *p;
      }
    }
  }
  float* q = out + ((int64_t)t * B + b) * S + e;
  if constexpr (VEC == 4) folx_st_stream4(q, make_float4(acc[0], acc[1], acc[2], acc[3]));
  else *q = acc[0];
}

// out[idx[r][so]][b][so][si] += data[r][b][so][si]   (idx < 0: the entry is skipped)
// A thread owns VEC consecutive floats of one walker and walks the stored rows r in order, so
// every output entry is updated by one thread in a fixed order: no atomics, the same bits on
// every run, also where several stored rows of a position name the same target row.  Eight rows
// at a time: their table entries, then their data and the target values they land on, all in
// flight together; rows of a group that share a target are folded into the first of them.
template <int VEC>
__global__ __launch_bounds__(256) void scatter_add_rows_kernel(const float* __restrict__ data,
                                                               const int32_t* __restrict__ idx,
                                                               float* out, int32_t k_in, int32_t k_out,
                                                               int64_t B, int64_t S_outer, int64_t S_inner) {
  const int64_t S = S_outer * S_inner;
  const int64_t f = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (f >= B * S) return;
  const int64_t b = f / S, e = f - b * S;
  const int64_t so = e / S_inner;
  for (int r0 = 0; r0 < k_in; r0 += 8) {
    int32_t t[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      t[u] = r0 + u < k_in ? idx[(int64_t)(r0 + u) * S_outer + so] : -1;
      if (t[u] >= k_out) t[u] = -1;  // a target outside the output is never written
    }
    float val[8][VEC], cur[8][VEC];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) val[u][v] = cur[u][v] = 0.0f;
      if (t[u] >= 0) {
        const float* p = data + ((int64_t)(r0 + u) * B + b) * S + e;
        const float* q = out + ((int64_t)t[u] * B + b) * S + e;
        if constexpr (VEC == 4) {
          const float4 a = folx_ld_stream4(p);
          val[u][0] = a.x; val[u][1] = a.y; val[u][2] = a.z; val[u][3] = a.w;
          const float4 c = *reinterpret_cast<const float4*>(q);
          cur[u][0] = c.x; cur[u][1] = c.y; cur[u][2] = c.z; cur[u][3] = c.w;
        } else {
          val[u][0] = *p;
          cur[u][0] = *q;
        }
      }
    }
    // the first row of a group that names a target collects the later ones, in row order
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (t[u] < 0) continue;
#pragma unroll
      for (int v = 0; v < VEC; ++v) cur[u][v] += val[u][v];
#pragma unroll
      for (int w = u + 1; w < 8; ++w)
        if (t[w] == t[u]) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) cur[u][v] += val[w][v];
          t[w] = -1;
        }
      float* q = out + ((int64_t)t[u] * B + b) * S + e;
      if constexpr (VEC == 4) *reinterpret_cast<float4*>(q) = make_float4(cur[u][0], cur[u][1], cur[u][2], cur[u][3]);
      else *q = cur[u][0];
    }
  }
}

// Static gather along the position axis with a sum over slots (the transposed form of a
// scatter with static indices: every output position lists the inputs that land on it):
//   out[rb][po][si] = sum_s data[rb][table[po][s]][si]        (table < 0: no source)
// Threads run along (po, si); blockIdx.y strides over the rb = (triplet row, walker) axis.
__global__ __launch_bounds__(256) void gather_cols_kernel(const float* __restrict__ data,
                                                          const int32_t* __restrict__ table,
                                                          float* __restrict__ out, int64_t RB,
                                                          int64_t S_in, int64_t S_out_outer,
                                                          int32_t n_slots, int64_t S_inner) {
  const int64_t S_out = S_out_outer * S_inner;
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= S_out) return;
  const int64_t po = e / S_inner, si = e % S_inner;
  int32_t src[4];
  const int32_t ns = n_slots < 4 ? n_slots : 4;
  for (int s = 0; s < ns; ++s) src[s] = table[po * n_slots + s];
  for (int64_t rb = blockIdx.y; rb < RB; rb += gridDim.y) {
    const float* row = data + rb * S_in;
    float acc = 0.0f;
    for (int s = 0; s < n_slots; ++s) {
      const int32_t t = s < 4 ? src[s] : table[po * n_slots + s];
      if (t >= 0) acc += row[(int64_t)t * S_inner + si];
    }
    out[rb * S_out + e] = acc;
  }
}

}  // namespace

extern "C" int folx_hip_gather_rows(void* stream, const float* data, const int32_t* take, float* out,
                                    int32_t k_in, int32_t k_out, int32_t n_slots, int64_t B,
                                    int64_t S_outer, int64_t S_inner) {
  if (k_in < 0 || k_out < 0 || n_slots < 0 || B < 0 || S_outer < 0 || S_inner < 0) return FOLX_HIP_EINVAL;
  const int64_t S = S_outer * S_inner;
  if (k_out == 0 || B == 0 || S == 0) return FOLX_HIP_OK;
  if (!out || (n_slots > 0 && (!take || (k_in > 0 && !data)))) return FOLX_HIP_EINVAL;
  if (k_out > 65535) return FOLX_HIP_ENOTSUP;
  const int64_t gy = (B + GATHER_WPT - 1) / GATHER_WPT;
  if (gy > 65535) return FOLX_HIP_ENOTSUP;
  const bool vec = (S_inner % 4 == 0) && folx_aligned16(data) && folx_aligned16(out);
  const int64_t blocks = vec ? (S / 4 + 255) / 256 : (S + 255) / 256;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  if (vec) {  // 128-bit accesses: the flat form streams at 5.9 TB/s where the strided one reaches 5.2-5.4
    const int64_t fb = (B * S / 4 + 255) / 256;
    if (fb <= 0x7fffffffLL) {
      gather_rows_flat_kernel<4><<<dim3((unsigned)fb, (unsigned)k_out), dim3(256), 0, (hipStream_t)stream>>>(
          data, take, out, n_slots, B, S_outer, S_inner);
      return folx_launch_status();
    }
  }
  dim3 grid((unsigned)blocks, (unsigned)gy, (unsigned)k_out);
  if (vec)
    gather_rows_kernel<4><<<grid, dim3(256), 0, (hipStream_t)stream>>>(data, take, out, n_slots, B, S_outer, S_inner);
  else
    gather_rows_kernel<1><<<grid, dim3(256), 0, (hipStream_t)stream>>>(data, take, out, n_slots, B, S_outer, S_inner);
  return folx_launch_status();
}

extern "C" int folx_hip_scatter_add_rows(void* stream, const float* data, const int32_t* idx,
                                         float* out, int32_t k_in, int32_t k_out, int64_t B,
                                         int64_t S_outer, int64_t S_inner) {
  if (k_in < 0 || k_out < 0 || B < 0 || S_outer < 0 || S_inner < 0) return FOLX_HIP_EINVAL;
  const int64_t S = S_outer * S_inner;
  if (k_in == 0 || B == 0 || S == 0) return FOLX_HIP_OK;
  if (!data || !idx || !out) return FOLX_HIP_EINVAL;
  const bool vec4 = S_inner % 4 == 0 && folx_aligned16(data) && folx_aligned16(out);
  const int64_t threads = vec4 ? B * S / 4 : B * S;
  const int64_t blocks = (threads + 255) / 256;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  if (vec4)
    scatter_add_rows_kernel<4><<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
        data, idx, out, k_in, k_out, B, S_outer, S_inner);
  else
    scatter_add_rows_kernel<1><<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
        data, idx, out, k_in, k_out, B, S_outer, S_inner);
  return folx_launch_status();
}

extern "C" int folx_hip_gather_cols(void* stream, const float* data, const int32_t* table, float* out,
                                    int64_t RB, int64_t S_in_outer, int64_t S_out_outer, int32_t n_slots,
                                    int64_t S_inner) {
  if (RB < 0 || S_in_outer < 0 || S_out_outer < 0 || n_slots < 0 || S_inner < 0) return FOLX_HIP_EINVAL;
  const int64_t S_out = S_out_outer * S_inner;
  if (RB == 0 || S_out == 0) return FOLX_HIP_OK;
  if (!out || (n_slots > 0 && (!table || (S_in_outer > 0 && !data)))) return FOLX_HIP_EINVAL;
  const int64_t blocks = (S_out + 255) / 256;
  if (blocks > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  const unsigned gy = (unsigned)(RB < 4096 ? RB : 4096);
  gather_cols_kernel<<<dim3((unsigned)blocks, gy), dim3(256), 0, (hipStream_t)stream>>>(
      data, table, out, RB, S_in_outer * S_inner, S_out_outer, n_slots, S_inner);
  return folx_launch_status();
}

extern "C" int folx_hip_gather_reduce_rows(void* stream, const float* data, const int32_t* take, float* out,
                                           int32_t k_in, int32_t k_out, int32_t n_slots, int64_t B, int64_t O,
                                           int32_t RED, int64_t IV, int64_t IC, float alpha) {
  if (k_in < 0 || k_out < 0 || n_slots < 0 || B < 0 || O < 0 || RED < 0 || IV < 0 || IC < 0) return FOLX_HIP_EINVAL;
  const int64_t S_out = O * IV * IC;
  if (k_out == 0 || B == 0 || S_out == 0) return FOLX_HIP_OK;
  if (!take || !out || (k_in > 0 && RED > 0 && !data)) return FOLX_HIP_EINVAL;
  if ((int64_t)k_in * RED > 0x7fffffffLL) return FOLX_HIP_ENOTSUP;
  const bool vec4 = IC % 4 == 0 && folx_aligned16(data) && folx_aligned16(out);
  const int64_t threads = vec4 ? B * S_out / 4 : B * S_out;
  const int64_t gx = (threads + 255) / 256;
  if (gx > 0x7fffffffLL || k_out > 65535) return FOLX_HIP_ENOTSUP;
  dim3 grid((unsigned)gx, (unsigned)k_out);
  hipStream_t st = (hipStream_t)stream;
  if (vec4) gather_reduce_rows_kernel<4><<<grid, dim3(256), 0, st>>>(data, take, out, n_slots, B, O, RED, IV, IC, alpha);
  else gather_reduce_rows_kernel<1><<<grid, dim3(256), 0, st>>>(data, take, out, n_slots, B, O, RED, IV, IC, alpha);
  return folx_launch_status();
}
