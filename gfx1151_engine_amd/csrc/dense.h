// Dense (non-block-quantised) storage of a weight matrix as the reference's generic matvec reads it
// (src/ref.cpp:68-109, src/hgn.h:2-23,160-202): bf16, f32, q8g64 (per row: cols uint8 codes, then cols/64
// pairs of fp16 (scale, min); w = code * scale + min) and q8g32 (planar over the whole tensor: rows*cols int8
// codes, then rows*cols/32 fp16 scales; w = code * scale; src/hgn.h:18,176-183).  Used for shared-expert matrices
// that are not q4cp / raw GGUF blocks (a bf16 checkpoint, the q8 tensors of overlay files and MTP sidecars).
#pragma once
#include "common.h"

// internal type codes, disjoint from the ggml block types
enum { MOE_T_DENSE = 0x100, MOE_T_BF16 = 0x100, MOE_T_F32 = 0x101, MOE_T_Q8G64 = 0x102, MOE_T_Q8G32 = 0x103 };

__host__ __device__ __forceinline__ bool moe_is_dense_type(int t) { return t >= MOE_T_DENSE; }
// bytes from one row to the next (q8g32: of its code plane)
__host__ __device__ __forceinline__ uint64_t moe_dense_row_bytes(int t, uint64_t k) {
  return t == MOE_T_BF16 ? 2 * k : t == MOE_T_F32 ? 4 * k : t == MOE_T_Q8G32 ? k : k + k / 64 * 4;
}
// hgn dtype (src/hgn.h:2-23) -> internal code, 0 if it is not one of the dense kinds
static inline int moe_dense_type_of_hgn(int dtype) {
  return dtype == MOE_DT_BF16 ? MOE_T_BF16 : dtype == MOE_DT_F32 ? MOE_T_F32 : dtype == MOE_DT_Q8G64 ? MOE_T_Q8G64 :
         dtype == MOE_DT_Q8G32 ? MOE_T_Q8G32 : 0;
}

// elements [32 b, 32 b + 32) of row r of a matrix of nrows x K elements stored at base, as f32 (each value exactly
// what the reference's dequant gives: bf16 widened, f32 as is, q8g64 one multiply and one add in f32, q8g32 one
// multiply)
__device__ __forceinline__ void moe_dense_block(int t, const uint8_t* base, uint64_t nrows, int K, uint64_t r, int b,
                                                float (&w)[32]) {
  const uint8_t* row = base + r * moe_dense_row_bytes(t, (uint64_t)K);
  if (t == MOE_T_Q8G32) {
    const uint32_t* p = (const uint32_t*)(row + (size_t)b * 32);
    const float s = __half2float(*(const __half*)(base + nrows * (uint64_t)K + (r * (uint64_t)K / 32 + b) * 2));
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const uint32_t u = p[i];
#pragma unroll
      for (int j = 0; j < 4; j++) w[4 * i + j] = __fmul_rn((float)(int)(int8_t)(u >> (8 * j)), s);
    }
  } else if (t == MOE_T_BF16) {
    const uint4* p = (const uint4*)(row + (size_t)b * 64);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint4 u = p[i];
      const uint32_t v[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
      for (int j = 0; j < 4; j++) {
        w[8 * i + 2 * j] = __uint_as_float(v[j] << 16);
        w[8 * i + 2 * j + 1] = __uint_as_float(v[j] & 0xffff0000u);
      }
    }
  } else if (t == MOE_T_F32) {
    const float4* p = (const float4*)(row + (size_t)b * 128);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const float4 f = p[i];
      w[4 * i] = f.x; w[4 * i + 1] = f.y; w[4 * i + 2] = f.z; w[4 * i + 3] = f.w;
    }
  } else {  // q8g64
    const uint32_t* p = (const uint32_t*)(row + (size_t)b * 32);         // rows start 4-byte aligned (K % 64 == 0)
    const uint32_t sm = *(const uint32_t*)(row + K + (size_t)(b >> 1) * 4);  // (scale, min) of the 64-group
    const float s = __half2float(__ushort_as_half((uint16_t)(sm & 0xffffu)));
    const float m = __half2float(__ushort_as_half((uint16_t)(sm >> 16)));
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const uint32_t u = p[i];
#pragma unroll
      for (int j = 0; j < 4; j++) w[4 * i + j] = __fadd_rn(__fmul_rn((float)((u >> (8 * j)) & 0xffu), s), m);
    }
  }
}
