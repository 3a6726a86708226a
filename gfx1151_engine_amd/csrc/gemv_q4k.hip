// Decode / small-batch expert GEMV on GGUF Q4_K raw blocks read in place.
// Unit of work = one sub-block pair (32 code bytes = 64 weights):
//   d*(s0*sum(q_lo*x_lo) + s1*sum(q_hi*x_hi)) - dmin*(m0*sum(x_lo) + m1*sum(x_hi))
// (reference: src/gpu/parts/26_kernels_moe_gguf.inc:527-568,693-756,893-939; src/gguf.h:408-441)
#include "common.h"
#include "internal.h"

namespace {

__device__ __forceinline__ void k4_sm(int j, const uint8_t* q, int& sc, int& mn) {
  if (j < 4) {
    sc = q[j] & 63;
    mn = q[j + 4] & 63;
  } else {
    sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
    mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
  }
}

// sums of x over the low-nibble half (first 32) and the high-nibble half (last 32) of a unit
__device__ __forceinline__ void unit_xsums(const float4* xv, float& sl, float& sh) {
  float a = 0.f, b = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    a += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);
    b += (xv[8 + i].x + xv[8 + i].y) + (xv[8 + i].z + xv[8 + i].w);
  }
  sl = a;
  sh = b;
}

// one unit of one row: blk = the 144-byte super-block, j = pair index, xv = 64 activations
__device__ __forceinline__ float unit_dot(const uint8_t* blk, int j, const float4* xv, float sl, float sh) {
  const float d = __half2float(*(const __half*)blk), dmin = __half2float(*(const __half*)(blk + 2));
  int s0, m0, s1, m1;
  k4_sm(2 * j, blk + 4, s0, m0);
  k4_sm(2 * j + 1, blk + 4, s1, m1);
  const uint4 c0 = *(const uint4*)(blk + 16 + j * 32), c1 = *(const uint4*)(blk + 16 + j * 32 + 16);
  const uint32_t w[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
  float lo = 0.f, hi = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) {  // word i = code bytes 4i..4i+3 -> elements 4i..4i+3 of each half
    const uint32_t v = w[i];
    const float4 xl = xv[i], xh = xv[8 + i];
    lo = fmaf((float)(v & 0xf), xl.x, lo);
    hi = fmaf((float)((v >> 4) & 0xf), xh.x, hi);
    lo = fmaf((float)((v >> 8) & 0xf), xl.y, lo);
    hi = fmaf((float)((v >> 12) & 0xf), xh.y, hi);
    lo = fmaf((float)((v >> 16) & 0xf), xl.z, lo);
    hi = fmaf((float)((v >> 20) & 0xf), xh.z, hi);
    lo = fmaf((float)((v >> 24) & 0xf), xl.w, lo);
    hi = fmaf((float)(v >> 28), xh.w, hi);
  }
  return d * ((float)s0 * lo + (float)s1 * hi) - dmin * ((float)m0 * sl + (float)m1 * sh);
}

template <int LPR>
__device__ __forceinline__ float sub_sum(float v) {
#pragma unroll
  for (int o = LPR / 2; o; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

struct GgArgs {
  const uint8_t *gate, *up, *down;           // routed experts [E][rows][row_bytes]
  const uint8_t *sh_gate, *sh_up, *sh_down;  // optional shared expert (raw rows)
  const float* sh_logit;
  const float *ey, *sg;
};

// grid (mid/ROWS, slots, P): x of the token in LDS as float4 [q][unit] (q-th quad of the unit).
constexpr int KG_ROWS = 32;
template <int LPR>
__global__ void __launch_bounds__(256) k_q4k_gemv_gu(GgArgs A, const float* __restrict__ x,
                                                     const int* __restrict__ ids, int id_stride, int kpt,
                                                     int d, int mid, float* __restrict__ hid) {
  extern __shared__ float4 xs[];
  const int s = blockIdx.y, tok = blockIdx.z;
  const int U = d / 64;
  const float* xt = x + (size_t)tok * d;
  for (int i = threadIdx.x; i < d / 4; i += blockDim.x) xs[(i & 15) * U + (i >> 4)] = ((const float4*)xt)[i];
  __syncthreads();
  const uint64_t rb = (uint64_t)(d / 256) * 144;
  const uint8_t *gbase, *ubase;
  if (s < kpt) {
    const int e = ids[(size_t)tok * id_stride + s];
    gbase = A.gate + (uint64_t)e * mid * rb;
    ubase = A.up + (uint64_t)e * mid * rb;
  } else {
    gbase = A.sh_gate;
    ubase = A.sh_up;
  }
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, sub = lane / LPR, l = lane % LPR;
  constexpr int RPW = 64 / LPR;  // rows per wave step
  const int r0 = blockIdx.x * KG_ROWS;
  const int nrows = min(KG_ROWS, mid - r0);
  float* ho = hid + ((size_t)tok * gridDim.y + s) * mid;
  for (int rr = wv * RPW + sub; rr < nrows; rr += 4 * RPW) {
    const int r = r0 + rr;
    const uint8_t* grow = gbase + (uint64_t)r * rb;
    const uint8_t* urow = ubase + (uint64_t)r * rb;
    float ag = 0.f, au = 0.f;
    for (int u = l; u < U; u += LPR) {
      float4 xv[16];
#pragma unroll
      for (int q = 0; q < 16; q++) xv[q] = xs[q * U + u];
      float sl, sh;
      unit_xsums(xv, sl, sh);
      ag += unit_dot(grow + (u >> 2) * 144, u & 3, xv, sl, sh);
      au += unit_dot(urow + (u >> 2) * 144, u & 3, xv, sl, sh);
    }
    ag = sub_sum<LPR>(ag);
    au = sub_sum<LPR>(au);
    if (l == 0) ho[r] = silu_f(ag) * au;
  }
}

constexpr int KD_ROWS = 32;
template <int LPR, int NS>
__global__ void __launch_bounds__(256) k_q4k_gemv_dn(GgArgs A, const float* __restrict__ hid,
                                                     const int* __restrict__ ids,
                                                     const float* __restrict__ ws, int id_stride, int kpt,
                                                     int d, int mid, float* __restrict__ out) {
  extern __shared__ float4 hs[];  // [slot][q][unit]
  __shared__ int eid[17];
  __shared__ float wgt[17];
  const int tok = blockIdx.y;
  const bool has_shared = A.sh_down != nullptr;
  const int nslots = kpt + (has_shared ? 1 : 0);
  const int U = mid / 64, q4 = mid / 4;
  const float* ht = hid + (size_t)tok * nslots * mid;
  for (int i = threadIdx.x; i < nslots * q4; i += blockDim.x) {
    const int s = i / q4, c = i % q4;
    hs[((size_t)s * 16 + (c & 15)) * U + (c >> 4)] = ((const float4*)ht)[i];
  }
  if (threadIdx.x < nslots) {
    const int s = threadIdx.x;
    if (s < kpt) {
      eid[s] = ids[(size_t)tok * id_stride + s];
      wgt[s] = ws[(size_t)tok * id_stride + s];
    } else {
      eid[s] = 0;
      wgt[s] = sigmoid_f(A.sh_logit[tok]);
    }
  }
  __syncthreads();
  const uint64_t rb = (uint64_t)(mid / 256) * 144;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, sub = lane / LPR, l = lane % LPR;
  constexpr int RPW = 64 / LPR;
  const int r0 = blockIdx.x * KD_ROWS;
  const int nrows = min(KD_ROWS, d - r0);
  for (int rr = wv * RPW + sub; rr < nrows; rr += 4 * RPW) {
    const int r = r0 + rr;
    float acc[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
      acc[s] = 0.f;
      if (s < nslots) {
        const bool sh = has_shared && s == nslots - 1;
        const uint8_t* row = sh ? A.sh_down + (uint64_t)r * rb : A.down + ((uint64_t)eid[s] * d + r) * rb;
        float a = 0.f;
        for (int u = l; u < U; u += LPR) {
          float4 xv[16];
#pragma unroll
          for (int q = 0; q < 16; q++) xv[q] = hs[((size_t)s * 16 + q) * U + u];
          float sl, sh2;
          unit_xsums(xv, sl, sh2);
          a += unit_dot(row + (u >> 2) * 144, u & 3, xv, sl, sh2);
        }
        acc[s] = sub_sum<LPR>(a);
      }
    }
    if (l == 0) {
      float y = 0.f;
#pragma unroll
      for (int s = 0; s < NS; s++)
        if (s < nslots) y += wgt[s] * acc[s];
      if (A.ey) y += sigmoid_f(A.sg[tok]) * A.ey[(size_t)tok * d + r];
      out[(size_t)tok * d + r] = y;
    }
  }
}

}  // namespace

// Internal launcher (shared with the context); shared-expert pointers may be null.
// phase: 0 = gate/up + down, 1 = gate/up only, 2 = down only (the context times them separately).
int moe_launch_q4k_gemv(int phase, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                        const uint8_t* sh_gate, const uint8_t* sh_up, const uint8_t* sh_down,
                        const float* sh_logit, const float* x, const int* ids, const float* ws,
                        float* hid, float* out, int P, int d, int mid, int kpt, int id_stride,
                        hipStream_t st) {
  if (!gate || !up || !down || !x || !ids || !ws || !hid || !out) return MOE_E_INVALID;
  if (P < 0 || kpt < 1 || id_stride < kpt) return MOE_E_INVALID;
  if (d < 256 || d % 256 || mid < 256 || mid % 256) return MOE_E_UNSUPPORTED;
  const bool sh = sh_gate != nullptr;
  if (sh && (!sh_up || !sh_down || !sh_logit)) return MOE_E_INVALID;
  const int nslots = kpt + (sh ? 1 : 0);
  if (nslots > 16 || (size_t)d * 4 > 60 * 1024 || (size_t)nslots * mid * 4 > 60 * 1024) return MOE_E_UNSUPPORTED;
  if (!moe_aligned(gate, 16) || !moe_aligned(up, 16) || !moe_aligned(down, 16) || !moe_aligned(x, 16) ||
      !moe_aligned(hid, 16))
    return MOE_E_INVALID;
  if (P == 0) return MOE_OK;
  GgArgs A{};
  A.gate = gate; A.up = up; A.down = down;
  A.sh_gate = sh_gate; A.sh_up = sh_up; A.sh_down = sh_down; A.sh_logit = sh_logit;
  if (phase != 2) {
    dim3 grid((mid + KG_ROWS - 1) / KG_ROWS, nslots, P);
    const int U = d / 64;
    if (U % 16 == 0) k_q4k_gemv_gu<16><<<grid, 256, (size_t)d * 4, st>>>(A, x, ids, id_stride, kpt, d, mid, hid);
    else if (U % 8 == 0) k_q4k_gemv_gu<8><<<grid, 256, (size_t)d * 4, st>>>(A, x, ids, id_stride, kpt, d, mid, hid);
    else k_q4k_gemv_gu<4><<<grid, 256, (size_t)d * 4, st>>>(A, x, ids, id_stride, kpt, d, mid, hid);
    MOE_LAUNCH_CHECK();
  }
  if (phase != 1) {
    dim3 grid((d + KD_ROWS - 1) / KD_ROWS, P);
    const size_t lds = (size_t)nslots * mid * 4;
    const int U = mid / 64;
#define DN_LAUNCH(LPR)                                                                                        \
  do {                                                                                                        \
    if (nslots <= 4) k_q4k_gemv_dn<LPR, 4><<<grid, 256, lds, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, out); \
    else if (nslots <= 11) k_q4k_gemv_dn<LPR, 11><<<grid, 256, lds, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, out); \
    else k_q4k_gemv_dn<LPR, 16><<<grid, 256, lds, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, out);       \
  } while (0)
    if (U % 16 == 0) DN_LAUNCH(16);
    else if (U % 8 == 0) DN_LAUNCH(8);
    else DN_LAUNCH(4);
#undef DN_LAUNCH
    MOE_LAUNCH_CHECK();
  }
  return MOE_OK;
}

MOE_API int moe_gg_gemv(int tgu, int tdn, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                        const float* x, const int* ids, const float* ws, float* hid, float* out, int P,
                        int d, int mid, int kpt, int id_stride, moe_stream_t st) {
  if (!moe_gg_types_supported(tgu, tdn, d, mid)) return MOE_E_UNSUPPORTED;
  if (tgu != MOE_GGML_Q4_K || tdn != MOE_GGML_Q4_K)  // Q5_K gate/up, Q5_1 / Q8_0 down: the general kernels
    return moe_launch_ggx_gemv(0, tgu, tdn, 0, gate, up, down, nullptr, nullptr, nullptr, nullptr, x, ids, ws, hid, out,
                               P, d, mid, kpt, id_stride, moe_s(st));
  return moe_launch_q4k_gemv(0, gate, up, down, nullptr, nullptr, nullptr, nullptr, x, ids, ws, hid, out, P, d,
                             mid, kpt, id_stride, moe_s(st));
}
