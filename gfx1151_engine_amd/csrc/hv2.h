// hgn v2 rotated weights (dtype 23 "i4r" experts): W = diag(svh) . H . G . H . diag(suh) / 128 with H the 128-block
// Sylvester Hadamard matrix in natural order; the rotation is applied to the activations around each projection
// instead of to the weights (reference: src/gpu/parts/28_kernels_hgn_v2.inc:1-15, fwht128 at
// src/gpu/parts/27_kernels_moe_lut.inc:44-65).
#pragma once
#include "common.h"

constexpr float MOE_RS128 = 0.0883883476483184405f;  // 1 / sqrt(128)

// Unnormalised Hadamard transform of 128 values spread over 16 consecutive lanes (an aligned group of 16), lane j of
// the group holding elements 8j .. 8j+7.  The butterflies (lo + hi, lo - hi) run over strides 1, 2, 4 inside the
// lane and 8 .. 64 across lanes, i.e. in ascending stride order whatever the distribution: the same f32 additions
// as a sequential transform.  All 16 lanes of a group must call it together.
__device__ __forceinline__ void moe_fwht128_r8(float (&v)[8], int lane) {
#pragma unroll
  for (int h = 1; h < 8; h <<= 1)
#pragma unroll
    for (int i = 0; i < 8; i++)
      if (!(i & h)) {
        const float a = v[i], b = v[i | h];
        v[i] = a + b;
        v[i | h] = a - b;
      }
#pragma unroll
  for (int s = 1; s < 16; s <<= 1) {
    const bool hi = (lane & s) != 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const float p = __shfl_xor(v[i], s, 64);
      v[i] = hi ? p - v[i] : v[i] + p;
    }
  }
}
