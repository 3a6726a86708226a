// Quantised activation vectors for the integer-dot decode kernels ("qvec"), per group of 32
// elements.  Two forms.
//
// qvec4 (q4cp weights, v_dot8_i32_i4): 4 planes x 4 dwords of balanced base-16 digits in [-8, 7],
//   x ~= q * (4096 p3 + 256 p2 + 16 p1 + p0), |X| <= 30583 (15.9 bits relative to the group maximum);
//   dword i of a plane holds elements 8i..8i+7, element 8i+t in bits 4t..4t+3: the nibble order of a
//   q4cp code word, so one v_dot8 multiplies 8 weights with 8 digits without any unpacking
//   (the unsigned codes n become n - 8 in two's complement by flipping bit 3 of every nibble).
//   meta: float2 (q, q * sum of the quantised elements).
//
// qvec (GGUF Q4_K weights, v_dot4_i32_i8):
//   planes: 3 x 8 dwords of signed 7-bit digits, x ~= q * (2^14 p0 + 2^7 p1 + p2);
//           q4cp order: dword 2i holds elements 8i+{0,2,4,6}, dword 2i+1 elements 8i+{1,3,5,7}
//           (the order in which `w & 0x0f0f0f0f` / `(w>>4) & 0x0f0f0f0f` deliver the 4-bit codes of
//           a q4cp row); natural order (Q4_K, where the low nibbles of 32 consecutive bytes are one
//           32-element sub-block and the high nibbles the next): dword i holds elements 4i..4i+3
//   meta:   float2 (q, q * sum of the quantised elements)
#pragma once
#include "common.h"

constexpr int QV_GROUP_DW = 24;
constexpr int QV4_GROUP_DW = 16;
constexpr float QV4_XMAX = 30583.f;  // 0x7777: every balanced digit at +7

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

// balanced base-16 digits of X (|X| <= 30583), least significant first
__device__ __forceinline__ void qv4_digits(int X, int& p0, int& p1, int& p2, int& p3) {
  p0 = ((X + 8) & 15) - 8;
  const int X1 = (X - p0) >> 4;
  p1 = ((X1 + 8) & 15) - 8;
  const int X2 = (X1 - p1) >> 4;
  p2 = ((X2 + 8) & 15) - 8;
  p3 = (X2 - p2) >> 4;
}

// One thread quantises group g of token t into the qvec4 form.
__device__ __forceinline__ void qvec4_group_from_f32(const float* __restrict__ x, uint64_t x_stride, int G, int t,
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
  const float inv = m > 0.f ? QV4_XMAX / m : 0.f;
  const float q = m * (1.f / QV4_XMAX);
  uint32_t pl[4][4];
#pragma unroll
  for (int p = 0; p < 4; p++)
#pragma unroll
    for (int i = 0; i < 4; i++) pl[p][i] = 0;
  int sx = 0;
#pragma unroll
  for (int j = 0; j < 32; j++) {
    const int X = (int)rintf(v[j] * inv);
    sx += X;
    int p0, p1, p2, p3;
    qv4_digits(X, p0, p1, p2, p3);
    const int dw = j >> 3, sh = 4 * (j & 7);
    pl[0][dw] |= (uint32_t)(p0 & 15) << sh;
    pl[1][dw] |= (uint32_t)(p1 & 15) << sh;
    pl[2][dw] |= (uint32_t)(p2 & 15) << sh;
    pl[3][dw] |= (uint32_t)(p3 & 15) << sh;
  }
  uint4* dst = (uint4*)(planes + ((size_t)t * G + g) * QV4_GROUP_DW);
#pragma unroll
  for (int p = 0; p < 4; p++) dst[p] = make_uint4(pl[p][0], pl[p][1], pl[p][2], pl[p][3]);
  meta[(size_t)t * G + g] = make_float2(q, q * (float)sx);
}
