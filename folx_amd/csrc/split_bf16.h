// FP32 products on the bf16 matrix pipe: every operand is split into three bf16 pieces,
//     x = x1 + x2 + x3   (x1 = bf16(x), x2 = bf16(x - x1), x3 = bf16(x - x1 - x2), exact: 3 x 8
//                         significand bits cover the 24 of an fp32 number),
// and a product a b is taken as the six piece products of weight >= 2^-16,
//     a3 b1 + a2 b2 + a2 b1 + a1 b3 + a1 b2 + a1 b1,
// each exact in fp32 and summed in the fp32 accumulator of v_mfma_f32_32x32x16_bf16.  The three
// products that are left out (a2 b3, a3 b2, a3 b3) weigh <= 2^-24 of a b, the rounding of one
// fp32 multiply-add.  Six bf16 products of depth 16 take 6 x 8 passes on the matrix pipe for
// the work of 8 v_mfma_f32_32x32x2_f32 (8 x 16 passes): 2.7 times the FP32 rate.
//
// An infinite element (or one that rounds to a bf16 infinity) turns into NaN: x - bf16(x) is
// inf - inf.  Finite inputs, the case the rules are used for, are represented exactly.
//
// The mode is process wide (folx_hip_set_gemm_mode); kernels that have no split form ignore it.
#pragma once
#include "common.h"

// 0: v_mfma_f32_32x32x2_f32 on the fp32 operands; 1: the split above where a kernel has it
int folx_gemm_mode();

#ifdef __HIPCC__
namespace folx_split {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned uint2v __attribute__((ext_vector_type(2)));
typedef unsigned uint4v __attribute__((ext_vector_type(4)));

// Two numbers at once (v_cvt_pk_bf16_f32 rounds a pair to nearest even): piece i of x in the
// low half of pi, of y in the high half.
__device__ __forceinline__ void split_pair(float x, float y, unsigned& p1, unsigned& p2, unsigned& p3) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  auto cvt = [](float a, float b) -> unsigned {
    f2 v;
    v[0] = a;
    v[1] = b;
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf2));
  };
  p1 = cvt(x, y);
  float rx = x - __uint_as_float(p1 << 16), ry = y - __uint_as_float(p1 & 0xffff0000u);
  p2 = cvt(rx, ry);
  rx -= __uint_as_float(p2 << 16);
  ry -= __uint_as_float(p2 & 0xffff0000u);
  p3 = cvt(rx, ry);
}

// The six products in the order they are accumulated: by A piece (one piece of A in
// registers at a time), small terms before the leading one.
constexpr int kPieceA[6] = {2, 1, 1, 0, 0, 0};
constexpr int kPieceB[6] = {0, 1, 0, 2, 1, 0};

}  // namespace folx_split
#endif
