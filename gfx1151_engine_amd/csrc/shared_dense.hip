// Shared expert whose matrices are stored densely (bf16, f32, q8g64) instead of as q4cp / raw GGUF blocks: the
// reference runs it through its generic gemv / gemm (src/gpu/parts/40_model.inc:1848-1858,4698-4711; CPU:
// src/ref.cpp:623-636).  Small batches: plain f32 GEMV kernels, a wave per weight row, every token of the batch
// against the row while it is in registers; the result is added to y behind the routed experts' kernels.
// (Batches over 32 tokens send these matrices through the general grouped GEMM of gguf_types.hip.)
#include "common.h"
#include "dense.h"
#include "internal.h"

namespace {

constexpr int SD_MAXP = 32;

// hid[t][r] = silu(Wg[r] . x_t) * (Wu[r] . x_t); grid ceil(mid / 4), block 256 (a wave per row)
__global__ void __launch_bounds__(256) k_shd_gu(int type, const uint8_t* __restrict__ Wg, const uint8_t* __restrict__ Wu,
                                                const float* __restrict__ x, int P, int d, int mid,
                                                float* __restrict__ hid) {
  const int lane = threadIdx.x & 63, r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= mid) return;
  float ag[SD_MAXP], au[SD_MAXP];
#pragma unroll
  for (int t = 0; t < SD_MAXP; t++) ag[t] = au[t] = 0.f;
  for (int b = lane; b < d / 32; b += 64) {
    float wg[32], wu[32];
    moe_dense_block(type, Wg, (uint64_t)mid, d, (uint64_t)r, b, wg);
    moe_dense_block(type, Wu, (uint64_t)mid, d, (uint64_t)r, b, wu);
#pragma unroll
    for (int t = 0; t < SD_MAXP; t++) {
      if (t < P) {
        const float4* xp = (const float4*)(x + (size_t)t * d + 32 * b);
        float sg = 0.f, su = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
          const float4 f = xp[i];
          sg = fmaf(wg[4 * i], f.x, sg); sg = fmaf(wg[4 * i + 1], f.y, sg);
          sg = fmaf(wg[4 * i + 2], f.z, sg); sg = fmaf(wg[4 * i + 3], f.w, sg);
          su = fmaf(wu[4 * i], f.x, su); su = fmaf(wu[4 * i + 1], f.y, su);
          su = fmaf(wu[4 * i + 2], f.z, su); su = fmaf(wu[4 * i + 3], f.w, su);
        }
        ag[t] += sg;
        au[t] += su;
      }
    }
  }
#pragma unroll
  for (int t = 0; t < SD_MAXP; t++) {
    if (t < P) {
      const float g = wave_sum(ag[t]), u = wave_sum(au[t]);
      if (lane == 0) hid[(size_t)t * mid + r] = silu_f(g) * u;
    }
  }
}

// y[t][r] += sigmoid(sh_logit[t]) * (Wd[r] . hid[t]); grid ceil(d / 4), block 256
__global__ void __launch_bounds__(256) k_shd_dn_axpy(int type, const uint8_t* __restrict__ Wd,
                                                     const float* __restrict__ hid, const float* __restrict__ sh_logit,
                                                     int P, int d, int mid, float* __restrict__ y) {
  const int lane = threadIdx.x & 63, r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= d) return;
  float acc[SD_MAXP];
#pragma unroll
  for (int t = 0; t < SD_MAXP; t++) acc[t] = 0.f;
  for (int b = lane; b < mid / 32; b += 64) {
    float w[32];
    moe_dense_block(type, Wd, (uint64_t)d, mid, (uint64_t)r, b, w);
#pragma unroll
    for (int t = 0; t < SD_MAXP; t++) {
      if (t < P) {
        const float4* hp = (const float4*)(hid + (size_t)t * mid + 32 * b);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
          const float4 f = hp[i];
          s = fmaf(w[4 * i], f.x, s); s = fmaf(w[4 * i + 1], f.y, s);
          s = fmaf(w[4 * i + 2], f.z, s); s = fmaf(w[4 * i + 3], f.w, s);
        }
        acc[t] += s;
      }
    }
  }
#pragma unroll
  for (int t = 0; t < SD_MAXP; t++) {
    if (t < P) {
      const float v = wave_sum(acc[t]);
      if (lane == 0) y[(size_t)t * d + r] += sigmoid_f(sh_logit[t]) * v;
    }
  }
}

// one row as f32 (registration-time sampling for the f16 range guard)
__global__ void __launch_bounds__(64) k_dense_row(int type, const uint8_t* __restrict__ base, uint64_t nrows, int K,
                                                  uint64_t r, float* __restrict__ out) {
  for (int b = threadIdx.x; b < K / 32; b += 64) {
    float w[32];
    moe_dense_block(type, base, nrows, K, r, b, w);
#pragma unroll
    for (int l = 0; l < 32; l++) out[32 * b + l] = w[l];
  }
}

}  // namespace

bool moe_dense_shared_supported(int type, int d, int mid) {
  if (!moe_is_dense_type(type)) return false;
  if (type == MOE_T_Q8G64) return d % 64 == 0 && mid % 64 == 0;  // (whole 64-groups per row)
  return d % 32 == 0 && mid % 32 == 0;
}

// Internal: y[t] += sigmoid(sh_logit[t]) * down(silu(gate x_t) * (up x_t)) for P <= 32 tokens; hid: f32 [P][mid] scratch.
int moe_launch_dense_shared_small(int type, const uint8_t* g, const uint8_t* u, const uint8_t* dn, const float* sh_logit,
                                  const float* x, int P, int d, int mid, float* hid, float* y, hipStream_t st) {
  if (!g || !u || !dn || !sh_logit || !x || !hid || !y) return MOE_E_INVALID;
  if (P < 1 || P > SD_MAXP || !moe_dense_shared_supported(type, d, mid)) return MOE_E_UNSUPPORTED;
  if (!moe_aligned(g, 16) || !moe_aligned(u, 16) || !moe_aligned(dn, 16) || !moe_aligned(x, 16)) return MOE_E_INVALID;
  k_shd_gu<<<(mid + 3) / 4, 256, 0, st>>>(type, g, u, x, P, d, mid, hid);
  MOE_LAUNCH_CHECK();
  k_shd_dn_axpy<<<(d + 3) / 4, 256, 0, st>>>(type, dn, hid, sh_logit, P, d, mid, y);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_dense_dequant_row(int type, const uint8_t* base, uint64_t nrows, int K, uint64_t r, float* out, hipStream_t st) {
  if (!base || !out || !moe_is_dense_type(type) || K % 32 || r >= nrows) return MOE_E_INVALID;
  k_dense_row<<<1, 64, 0, st>>>(type, base, nrows, K, r, out);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}
