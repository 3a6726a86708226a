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
//   planes: 2 x 8 dwords of signed 8-bit digits, x ~= q * (256 p0 + p1), |X| <= 32639 (15.99 bits
//           relative to the group maximum, the same resolution as qvec4); natural order: dword i
//           holds elements 4i..4i+3 (in Q4_K the low nibbles of 32 consecutive bytes are one
//           32-element sub-block and the high nibbles the next, so `w & 0x0f0f0f0f` and
//           `(w >> 4) & 0x0f0f0f0f` deliver four consecutive codes of one sub-block each)
//   meta:   float2 (q, q * sum of the quantised elements)
#pragma once
#include "common.h"

constexpr int QV_GROUP_DW = 16;
constexpr int QV4_GROUP_DW = 16;
constexpr float QV_XMAX = 32639.f;   // 0x7f7f: both balanced digits at +127
constexpr float QV4_XMAX = 30583.f;  // 0x7777: every balanced digit at +7

// Cross-row steps of the wave reductions of the decode kernels.  v holds its row's (16 lanes) result
// in every lane; lane reads + scalar operands instead of shuffles through the LDS crossbar.  The
// additions pair the rows as the xor-16 / xor-32 butterfly does: (r0 + r1) + (r2 + r3).
__device__ __forceinline__ float rows_total_add(float v) {
  const int b = __float_as_int(v);
  return (__int_as_float(__builtin_amdgcn_readlane(b, 0)) + __int_as_float(__builtin_amdgcn_readlane(b, 16))) +
         (__int_as_float(__builtin_amdgcn_readlane(b, 32)) + __int_as_float(__builtin_amdgcn_readlane(b, 48)));
}
__device__ __forceinline__ float rows_half_add(float v) {  // lanes < 32: r0 + r1, the others: r2 + r3
  const int b = __float_as_int(v);
  const float lo = __int_as_float(__builtin_amdgcn_readlane(b, 0)) + __int_as_float(__builtin_amdgcn_readlane(b, 16));
  const float hi = __int_as_float(__builtin_amdgcn_readlane(b, 32)) + __int_as_float(__builtin_amdgcn_readlane(b, 48));
  return (threadIdx.x & 32) ? hi : lo;
}
__device__ __forceinline__ float rows_half_max(float v) {
  const int b = __float_as_int(v);
  const float lo = fmaxf(__int_as_float(__builtin_amdgcn_readlane(b, 0)), __int_as_float(__builtin_amdgcn_readlane(b, 16)));
  const float hi = fmaxf(__int_as_float(__builtin_amdgcn_readlane(b, 32)), __int_as_float(__builtin_amdgcn_readlane(b, 48)));
  return (threadIdx.x & 32) ? hi : lo;
}

// balanced base-256 digits of X (|X| <= 32639): X = 256 p0 + p1
__device__ __forceinline__ void qv_digits(int X, int& p0, int& p1) {
  p1 = ((X + 128) & 255) - 128;
  p0 = (X - p1) >> 8;
}

// One thread quantises group g of token t into the qvec form.
__device__ __forceinline__ void qvec_group_from_f32(const float* __restrict__ x, uint64_t x_stride, int G, int t,
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
  const float inv = m > 0.f ? QV_XMAX / m : 0.f;
  const float q = m * (1.f / QV_XMAX);
  uint32_t pl[2][8];
#pragma unroll
  for (int p = 0; p < 2; p++)
#pragma unroll
    for (int i = 0; i < 8; i++) pl[p][i] = 0;
  int sx = 0;
#pragma unroll
  for (int j = 0; j < 32; j++) {
    const int X = (int)rintf(v[j] * inv);
    sx += X;
    int p0, p1;
    qv_digits(X, p0, p1);
    const int dw = j >> 2, sh = 8 * (j & 3);
    pl[0][dw] |= (uint32_t)(p0 & 0xff) << sh;
    pl[1][dw] |= (uint32_t)(p1 & 0xff) << sh;
  }
  uint4* dst = (uint4*)(planes + ((size_t)t * G + g) * QV_GROUP_DW);
#pragma unroll
  for (int p = 0; p < 2; p++) {
    dst[2 * p] = make_uint4(pl[p][0], pl[p][1], pl[p][2], pl[p][3]);
    dst[2 * p + 1] = make_uint4(pl[p][4], pl[p][5], pl[p][6], pl[p][7]);
  }
  meta[(size_t)t * G + g] = make_float2(q, q * (float)sx);
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
