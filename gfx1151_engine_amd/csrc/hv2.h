// hgn v2 rotated weights (dtype 23 "i4r" experts): W = diag(svh) . H . G . H . diag(suh) / 128 with H the 128-block
// Sylvester Hadamard matrix in natural order; the rotation is applied to the activations around each projection
// instead of to the weights (reference: src/gpu/parts/28_kernels_hgn_v2.inc:1-15, fwht128 at
// src/gpu/parts/27_kernels_moe_lut.inc:44-65).
#pragma once
#include "common.h"
#include "qvec.h"

constexpr float MOE_RS128 = 0.0883883476483184405f;  // 1 / sqrt(128)

// the value of lane (l ^ S) of the same row of 16 lanes, S = 1, 2, 4, 8: data-parallel-primitive moves (no trip
// through the LDS crossbar).  l ^ 4 = half-row mirror followed by a quad reversal; l ^ 8 = rotation of the row by 8.
template <int S>
__device__ __forceinline__ float moe_row_xor(float v) {
  const int b = __float_as_int(v);
  if (S == 1) return __int_as_float(__builtin_amdgcn_update_dpp(0, b, 0xB1, 0xf, 0xf, true));
  if (S == 2) return __int_as_float(__builtin_amdgcn_update_dpp(0, b, 0x4E, 0xf, 0xf, true));
  if (S == 8) return __int_as_float(__builtin_amdgcn_update_dpp(0, b, 0x128, 0xf, 0xf, true));
  const int m = __builtin_amdgcn_update_dpp(0, b, 0x141, 0xf, 0xf, true);
  return __int_as_float(__builtin_amdgcn_update_dpp(0, m, 0x1B, 0xf, 0xf, true));
}

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
#define MOE_FWHT_STEP(S)                                  \
  {                                                       \
    const bool hi = (lane & S) != 0;                      \
    _Pragma("unroll") for (int i = 0; i < 8; i++) {       \
      const float p = moe_row_xor<S>(v[i]);               \
      v[i] = hi ? p - v[i] : v[i] + p;                    \
    }                                                     \
  }
  MOE_FWHT_STEP(1)
  MOE_FWHT_STEP(2)
  MOE_FWHT_STEP(4)
  MOE_FWHT_STEP(8)
#undef MOE_FWHT_STEP
}

// 8 values as f16 in the order the grouped GEMM keeps its activations in: [e0,e4,e1,e5,e2,e6,e3,e7]
__device__ __forceinline__ void moe_st8_f16_ilv(__half* p, const float (&v)[8]) {
  const __half2 a = __floats2half2_rn(v[0], v[4]), b = __floats2half2_rn(v[1], v[5]);
  const __half2 c = __floats2half2_rn(v[2], v[6]), d = __floats2half2_rn(v[3], v[7]);
  uint4 o;
  o.x = *(const uint32_t*)&a; o.y = *(const uint32_t*)&b; o.z = *(const uint32_t*)&c; o.w = *(const uint32_t*)&d;
  *(uint4*)p = o;
}

__device__ __forceinline__ float moe_quad_xor1(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));
}
__device__ __forceinline__ float moe_quad_xor2(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true));
}

// 8 values per lane, the four lanes of a quad = one 32-element group -> the group's four digit planes and (q, q*sum)
// in the form the integer-dot decode kernels read (qvec.h, qvec4): lane j of the quad holds dword j of every plane.
__device__ __forceinline__ void moe_st8_planes(const float (&v)[8], int lane, uint32_t* __restrict__ planes,
                                           float2* __restrict__ meta, size_t gi, bool live) {
  float m = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) m = fmaxf(m, fabsf(v[i]));
  m = fmaxf(m, moe_quad_xor1(m));
  m = fmaxf(m, moe_quad_xor2(m));
  const float inv = m > 0.f ? QV4_XMAX / m : 0.f;
  const float q = m * (1.f / QV4_XMAX);
  uint32_t pl[4] = {0u, 0u, 0u, 0u};
  int sx = 0;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int X = (int)rintf(v[i] * inv);
    sx += X;
    int p0, p1, p2, p3;
    qv4_digits(X, p0, p1, p2, p3);
    pl[0] |= (uint32_t)(p0 & 15) << (4 * i);
    pl[1] |= (uint32_t)(p1 & 15) << (4 * i);
    pl[2] |= (uint32_t)(p2 & 15) << (4 * i);
    pl[3] |= (uint32_t)(p3 & 15) << (4 * i);
  }
  sx += __builtin_amdgcn_update_dpp(0, sx, 0xB1, 0xf, 0xf, true);
  sx += __builtin_amdgcn_update_dpp(0, sx, 0x4E, 0xf, 0xf, true);
  if (live) {
    uint32_t* dst = planes + gi * QV4_GROUP_DW + (lane & 3);
#pragma unroll
    for (int p = 0; p < 4; p++) dst[4 * p] = pl[p];
    if ((lane & 3) == 0) meta[gi] = make_float2(q, q * (float)sx);
  }
}

