// Quantised activation vectors for the integer-dot decode kernels ("qvec"), per group of 32
// elements:
//   planes: 3 x 8 dwords of signed 7-bit digits, x ~= q * (2^14 p0 + 2^7 p1 + p2);
//           q4cp order: dword 2i holds elements 8i+{0,2,4,6}, dword 2i+1 elements 8i+{1,3,5,7}
//           (the order in which `w & 0x0f0f0f0f` / `(w>>4) & 0x0f0f0f0f` deliver the 4-bit codes of
//           a q4cp row); natural order (Q4_K, where the low nibbles of 32 consecutive bytes are one
//           32-element sub-block and the high nibbles the next): dword i holds elements 4i..4i+3
//   meta:   float2 (q, q * sum of the quantised elements)
#pragma once
#include "common.h"

constexpr int QV_GROUP_DW = 24;

// digit plane position of element j (0..31) of a group
__device__ __forceinline__ void qvec_pos(int j, bool natural, int& dw, int& sh) {
  dw = natural ? j >> 2 : 2 * (j >> 3) + (j & 1);
  sh = natural ? 8 * (j & 3) : 8 * ((j & 7) >> 1);
}

// One thread quantises group g of token t.
template <bool NATURAL>
__device__ __forceinline__ void qvec_group_from_f32_t(const float* __restrict__ x, uint64_t x_stride, int G, int t,
                                                      int g, uint32_t* __restrict__ planes,
                                                      float2* __restrict__ meta) {
  const float4* xp = (const float4*)(x + (size_t)t * x_stride + (size_t)g * 32);
  float v[32];
  float m = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const float4 f = xp[i];
    v[4 * i] = f.x; v[4 * i + 1] = f.y; v[4 * i + 2] = f.z; v[4 * i + 3] = f.w;
    m = fmaxf(m, fmaxf(fmaxf(fabsf(f.x), fabsf(f.y)), fmaxf(fabsf(f.z), fabsf(f.w))));
  }
  const float inv = m > 0.f ? 1048576.f / m : 0.f;
  const float q = m * (1.f / 1048576.f);
  uint32_t pl[3][8];
#pragma unroll
  for (int p = 0; p < 3; p++)
#pragma unroll
    for (int i = 0; i < 8; i++) pl[p][i] = 0;
  int sx = 0;
#pragma unroll
  for (int j = 0; j < 32; j++) {
    const int X = (int)rintf(v[j] * inv);
    sx += X;
    const int p2 = ((X + 64) & 127) - 64;
    const int X1 = (X - p2) >> 7;
    const int p1 = ((X1 + 64) & 127) - 64;
    const int p0 = (X1 - p1) >> 7;
    const int dw = NATURAL ? j >> 2 : 2 * (j >> 3) + (j & 1), sh = NATURAL ? 8 * (j & 3) : 8 * ((j & 7) >> 1);
    pl[0][dw] |= (uint32_t)(p0 & 0xff) << sh;
    pl[1][dw] |= (uint32_t)(p1 & 0xff) << sh;
    pl[2][dw] |= (uint32_t)(p2 & 0xff) << sh;
  }
  uint4* dst = (uint4*)(planes + ((size_t)t * G + g) * QV_GROUP_DW);
#pragma unroll
  for (int p = 0; p < 3; p++) {
    dst[2 * p] = make_uint4(pl[p][0], pl[p][1], pl[p][2], pl[p][3]);
    dst[2 * p + 1] = make_uint4(pl[p][4], pl[p][5], pl[p][6], pl[p][7]);
  }
  meta[(size_t)t * G + g] = make_float2(q, q * (float)sx);
}
__device__ __forceinline__ void qvec_group_from_f32(const float* __restrict__ x, uint64_t x_stride, int G, int t,
                                                    int g, uint32_t* __restrict__ planes,
                                                    float2* __restrict__ meta, bool natural = false) {
  if (natural) qvec_group_from_f32_t<true>(x, x_stride, G, t, g, planes, meta);
  else qvec_group_from_f32_t<false>(x, x_stride, G, t, g, planes, meta);
}
