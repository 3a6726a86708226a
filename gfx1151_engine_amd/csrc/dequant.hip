// Dequantisation of the two 4-bit expert formats to f32, bit-exact with the CPU formulas.
#include "common.h"

// q4cp: w = cb[nibble] * f32(fp16 scale); one f32 multiply, no contraction possible.
// One thread per 32-bit code word (8 weights).  (reference: src/hgn.h:249-261)
__global__ void __launch_bounds__(256) k_q4cp_dequant(const uint8_t* __restrict__ codes,
                                                      const uint8_t* __restrict__ scales,
                                                      const float* __restrict__ cb, uint64_t cols,
                                                      uint64_t scale_stride, uint64_t row0,
                                                      uint64_t nwords, float* __restrict__ out) {
  __shared__ float cbs[16];
  if (threadIdx.x < 16) cbs[threadIdx.x] = cb[threadIdx.x];
  __syncthreads();
  const uint64_t wpr = cols / 8;  // words per row
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nwords;
       i += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t r = i / wpr, wi = i % wpr, row = row0 + r;
    const uint32_t w = *(const uint32_t*)(codes + row * (cols / 2) + wi * 4);
    const __half sh = *(const __half*)(scales + row * scale_stride + (wi / 4) * 2);
    const float s = __half2float(sh);
    float4 a, b;
    a.x = cbs[w & 0xf] * s;
    a.y = cbs[(w >> 4) & 0xf] * s;
    a.z = cbs[(w >> 8) & 0xf] * s;
    a.w = cbs[(w >> 12) & 0xf] * s;
    b.x = cbs[(w >> 16) & 0xf] * s;
    b.y = cbs[(w >> 20) & 0xf] * s;
    b.z = cbs[(w >> 24) & 0xf] * s;
    b.w = cbs[(w >> 28) & 0xf] * s;
    float4* o = (float4*)(out + r * cols + wi * 8);
    o[0] = a;
    o[1] = b;
  }
}

__device__ __forceinline__ void k4_scale_min(int j, const uint8_t* q, int& sc, int& mn) {
  // get_scale_min_k4 (reference: src/gguf.h:328-336)
  if (j < 4) {
    sc = q[j] & 63;
    mn = q[j + 4] & 63;
  } else {
    sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
    mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
  }
}

// Q4_K: one thread per (super-block, sub-block pair j, byte quad): 4 code bytes -> 4 low-nibble
// and 4 high-nibble weights.  y = (d*sc)*q - dmin*m: both products are exact in f32, so the
// result is a single rounded subtraction.  (reference: src/gguf.h:408-441)
__global__ void __launch_bounds__(256) k_q4k_dequant(const uint8_t* __restrict__ raw, uint64_t cols,
                                                     uint64_t nunits, float* __restrict__ out) {
  const uint64_t bpr = cols / 256;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nunits;
       i += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t blk = i / 32;
    const int u = (int)(i % 32), j = u / 8, q4 = u % 8;  // pair j, bytes 4*q4..4*q4+3
    const uint8_t* src = raw + blk * 144;
    const float d = __half2float(*(const __half*)src), dmin = __half2float(*(const __half*)(src + 2));
    int s0, m0, s1, m1;
    k4_scale_min(2 * j, src + 4, s0, m0);
    k4_scale_min(2 * j + 1, src + 4, s1, m1);
    const float d1 = d * (float)s0, dm1 = dmin * (float)m0, d2 = d * (float)s1, dm2 = dmin * (float)m1;
    const uint32_t w = *(const uint32_t*)(src + 16 + j * 32 + q4 * 4);
    const uint64_t r = blk / bpr, b = blk % bpr;
    float* y = out + r * cols + b * 256 + j * 64 + q4 * 4;
    float4 lo, hi;
    lo.x = d1 * (float)(w & 0xf) - dm1;
    lo.y = d1 * (float)((w >> 8) & 0xf) - dm1;
    lo.z = d1 * (float)((w >> 16) & 0xf) - dm1;
    lo.w = d1 * (float)((w >> 24) & 0xf) - dm1;
    hi.x = d2 * (float)((w >> 4) & 0xf) - dm2;
    hi.y = d2 * (float)((w >> 12) & 0xf) - dm2;
    hi.z = d2 * (float)((w >> 20) & 0xf) - dm2;
    hi.w = d2 * (float)(w >> 28) - dm2;
    *(float4*)y = lo;
    *(float4*)(y + 32) = hi;
  }
}

MOE_API int moe_q4cp_dequant_rows(const uint8_t* blob, uint64_t rows, uint64_t cols, uint64_t row0,
                                  uint64_t nrows, float* out, moe_stream_t st) {
  if (!blob || (!out && nrows)) return MOE_E_INVALID;
  if (cols == 0 || cols % 32 || row0 + nrows > rows) return MOE_E_INVALID;
  if (nrows == 0) return MOE_OK;
  if (!moe_aligned(blob, 4) || !moe_aligned(out, 16)) return MOE_E_INVALID;
  moe_wview v{MOE_DT_Q4CP, blob, rows, cols, 0};
  Q4cpOps o = q4cp_ops(&v);
  const uint64_t nwords = nrows * cols / 8;
  const unsigned grid = (unsigned)((nwords + 255) / 256 > 65535 * 16 ? 65535 * 16 : (nwords + 255) / 256);
  k_q4cp_dequant<<<grid, 256, 0, moe_s(st)>>>(o.codes, o.scales, o.cb, cols, o.scale_stride, row0,
                                              nwords, out);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

MOE_API int moe_q4k_dequant_rows(const uint8_t* raw, uint64_t nrows, uint64_t cols, float* out,
                                 moe_stream_t st) {
  if (!raw || (!out && nrows)) return MOE_E_INVALID;
  if (cols == 0 || cols % 256) return MOE_E_INVALID;
  if (nrows == 0) return MOE_OK;
  if (!moe_aligned(raw, 4) || !moe_aligned(out, 16)) return MOE_E_INVALID;
  const uint64_t nunits = nrows * (cols / 256) * 32;
  const unsigned grid = (unsigned)((nunits + 255) / 256 > 65535 * 16 ? 65535 * 16 : (nunits + 255) / 256);
  k_q4k_dequant<<<grid, 256, 0, moe_s(st)>>>(raw, cols, nunits, out);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}
