// FP32 numbers as bf16 pieces: x = h + m + l exactly, each piece a bf16 (8 significant bits): h = x cut to its upper 16 bits,
// m = x - h cut likewise, l = the rest. Used by the kernels that run FP32 contractions on v_mfma_f32_32x32x16_bf16
// (six of the nine piece products; the three smallest, below 2^-24 of the whole, are left out).
// The pieces keep FP32's exponent range, so nothing is scaled; an x below 2^-110 has lower pieces that are bf16 denormals.
#pragma once
#include <hip/hip_runtime.h>

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

// which piece of the first and of the second operand each of the six MFMAs takes (0 = h, 1 = m, 2 = l), smallest terms first
#define GT_PIECE_TERMS_A {0, 2, 1, 0, 1, 0}
#define GT_PIECE_TERMS_B {2, 0, 1, 1, 0, 0}

// two consecutive elements' pieces as one register each: (h, m, l) of x0 in the low halves, of x1 in the high halves
__device__ __forceinline__ void split_pair(float x0, float x1, unsigned &h, unsigned &m, unsigned &l) {
  const unsigned h0 = __float_as_uint(x0) & 0xFFFF0000u, h1 = __float_as_uint(x1) & 0xFFFF0000u;
  const float r0 = x0 - __uint_as_float(h0), r1 = x1 - __uint_as_float(h1);
  const unsigned m0 = __float_as_uint(r0) & 0xFFFF0000u, m1 = __float_as_uint(r1) & 0xFFFF0000u;
  const float q0 = r0 - __uint_as_float(m0), q1 = r1 - __uint_as_float(m1);
  h = __builtin_amdgcn_perm(h1, h0, 0x07060302);
  m = __builtin_amdgcn_perm(m1, m0, 0x07060302);
  l = __builtin_amdgcn_perm(__float_as_uint(q1), __float_as_uint(q0), 0x07060302);
}
// the 8 k-slots of one lane for one MFMA: x[0..7] -> out[piece]
__device__ __forceinline__ void cut8(const float (&x)[8], v4u (&out)[3]) {
#pragma unroll
  for (int p = 0; p < 4; p++) {
    unsigned h, m, l;
    split_pair(x[2 * p], x[2 * p + 1], h, m, l);
    out[0][p] = h; out[1][p] = m; out[2][p] = l;
  }
}
