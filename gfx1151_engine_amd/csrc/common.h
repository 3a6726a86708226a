// Shared helpers of libmi355moe (gfx950 only, wave64).
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/mi355_moe.h"

#define MOE_API extern "C" __attribute__((visibility("default")))
#define MOE_WAVE 64

static inline hipStream_t moe_s(moe_stream_t s) { return (hipStream_t)s; }

// After a launch: hand a launch error back as a positive hipError_t.
#define MOE_LAUNCH_CHECK()                     \
  do {                                         \
    hipError_t e__ = hipGetLastError();        \
    if (e__ != hipSuccess) return (int)e__;    \
  } while (0)
#define MOE_HIP(call)                          \
  do {                                         \
    hipError_t e__ = (call);                   \
    if (e__ != hipSuccess) return (int)e__;    \
  } while (0)

static inline bool moe_aligned(const void* p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

// Set-up that a launch site needs once per device (hipFuncSetAttribute applies to the current device's copy of the
// kernel): one bit per device ordinal.  moe_dev_pending is true until moe_dev_done has been called with that device
// current; two host threads that arrive together both do the (idempotent) set-up.
struct moe_dev_once {
  std::atomic<uint64_t> bits[4] = {};
};
static inline bool moe_dev_pending(moe_dev_once& o, int* dev_out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 256) dev = 255;  // (unknown ordinal: never marked, set up again every time)
  *dev_out = dev;
  return dev == 255 || !(o.bits[dev >> 6].load(std::memory_order_acquire) & (1ull << (dev & 63)));
}
static inline void moe_dev_done(moe_dev_once& o, int dev) {
  if (dev != 255) o.bits[dev >> 6].fetch_or(1ull << (dev & 63), std::memory_order_release);
}

// q4cp view -> operand pointers (reference: xcodes(), 40_model.inc:1599-1602)
struct Q4cpOps {
  const uint8_t* codes;
  const uint8_t* scales;
  const float* cb;
  uint64_t cols, scale_stride;
};
static inline Q4cpOps q4cp_ops(const moe_wview* w) {
  Q4cpOps o;
  o.cb = (const float*)w->data;
  o.codes = w->data + 64;
  o.scales = w->data + 64 + w->rows * w->cols / 2;
  o.cols = w->cols;
  o.scale_stride = w->scale_stride ? w->scale_stride : (((w->cols / 32 * 2) + 15) & ~15ULL);
  return o;
}

// Block barrier for data exchanged through LDS only.  __syncthreads() carries a workgroup fence that the compiler
// lowers to s_waitcnt vmcnt(0) as well: a kernel that keeps global loads in flight across its barriers (prefetch into
// registers or straight into LDS) would wait for all of them at every barrier.  This one waits for the wave's own LDS
// accesses and synchronises; global memory written before it is NOT made visible to the other waves by it.
__device__ __forceinline__ void moe_lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = 32; o; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
// Range guard of the f16 intermediates of the batch path.  hid = silu(g)*u and the down-projection
// pairs are kept in f16; for weights with large scales (raw Q4_K blocks with big sub-scales) their
// magnitude, ~ C.hi * mean(x^2) with C.hi a per-layer constant from the weights' row norms (the larger of
// hid's and the pairs' typical magnitude at unit activations), can pass 65504.  The gate/up epilogue
// multiplies hid by this power of two (exactly 1 while the estimate stays below 16), the pairs inherit it
// and the combine divides it out in f32: exact.  The other side: with very small weights the smaller of the
// two magnitudes, ~ C.lo * mean(x^2), heads for f16's subnormal range (below 2^-14, where a value keeps fewer
// than 11 bits); under 2^-10 the factor is a power of two above 1 that brings it to about 2^-6, as far as the
// larger magnitude stays below 16.  Exactly 1 for ordinary weights (the benchmark's layers: 4 and 4).
struct moe_cmag {
  float hi, lo;
};
__device__ __forceinline__ float moe_hid_scale(moe_cmag C, float xms) {
  const float est = C.hi * xms;
  int e;
  if (est > 16.f) {
    (void)frexpf(est * 0.0625f, &e);  // est/16 = m * 2^e, m in [0.5, 1)
    return ldexpf(1.f, -e);
  }
  const float lo = C.lo * xms;
  if (lo > 0.f && lo < 0x1p-10f) {
    (void)frexpf(lo, &e);      // lo = m * 2^e, m in [0.5, 1)
    int up = -6 - e;           // lo * 2^up in [2^-7, 2^-6)
    int eh;
    (void)frexpf(est, &eh);    // est < 2^eh
    up = up < 4 - eh ? up : 4 - eh;  // est * 2^up < 16
    return up > 0 ? ldexpf(1.f, up) : 1.f;
  }
  return 1.f;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }
