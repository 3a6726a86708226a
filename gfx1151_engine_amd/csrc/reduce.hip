// Activation conversion, tile list with the shared expert appended, and the deterministic
// top-k weighted combine (+ sigmoid-gated shared expert).
// (reference: src/gpu/parts/26_kernels_moe_gguf.inc:389; src/gpu/parts/24_kernels_moe_lt.inc:82-124;
//  src/gpu/parts/40_model.inc:8897)
#include "common.h"
#include "hv2.h"
#include "internal.h"

namespace {

// 8 floats -> 8 f16 (RNE).  ILV: the order the grouped GEMM keeps its activations in,
// [e0,e4,e1,e5,e2,e6,e3,e7] inside every group of 8.
template <bool ILV>
__global__ void __launch_bounds__(256) k_f32_to_f16_v8(const float4* __restrict__ x, uint4* __restrict__ y,
                                                       uint64_t n8) {
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += (uint64_t)gridDim.x * blockDim.x) {
    const float4 u = x[2 * i], v = x[2 * i + 1];
    __half2 a, b, c, d;
    if (ILV) {
      a = __floats2half2_rn(u.x, v.x); b = __floats2half2_rn(u.y, v.y);
      c = __floats2half2_rn(u.z, v.z); d = __floats2half2_rn(u.w, v.w);
    } else {
      a = __floats2half2_rn(u.x, u.y); b = __floats2half2_rn(u.z, u.w);
      c = __floats2half2_rn(v.x, v.y); d = __floats2half2_rn(v.z, v.w);
    }
    uint4 o;
    o.x = *(const uint32_t*)&a; o.y = *(const uint32_t*)&b; o.z = *(const uint32_t*)&c; o.w = *(const uint32_t*)&d;
    y[i] = o;
  }
}

// Layout 2 (raw GGUF Q4_K weights): inside every 64 elements, 16-byte chunk w (0..7) holds
// [4w, 4w+2, 32+4w, 32+4w+2, 4w+1, 4w+3, 32+4w+1, 32+4w+3] - the order in which one 32-bit word of
// a Q4_K block (bytes 4w..4w+3: low nibbles = elements 4w.., high nibbles = elements 32+4w..)
// unpacks.
__global__ void __launch_bounds__(256) k_f32_to_f16_q4k(const float4* __restrict__ x, uint4* __restrict__ y,
                                                        uint64_t n8) {
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t blk = i >> 3, w = i & 7;
    const float4 u = x[blk * 16 + w], v = x[blk * 16 + 8 + w];
    const __half2 a = __floats2half2_rn(u.x, u.z), b = __floats2half2_rn(v.x, v.z);
    const __half2 c = __floats2half2_rn(u.y, u.w), d = __floats2half2_rn(v.y, v.w);
    uint4 o;
    o.x = *(const uint32_t*)&a; o.y = *(const uint32_t*)&b; o.z = *(const uint32_t*)&c; o.w = *(const uint32_t*)&d;
    y[i] = o;
  }
}

// The f16 copy of whole rows in layout 1 or 2 plus each row's mean square (the f16 range guard's input) in
// one pass over x: a wave per row, lanes take the row's 8-element chunks in turn.
template <int LAYOUT>
__global__ void __launch_bounds__(256) k_f32_to_f16_rows(const float* __restrict__ x, uint4* __restrict__ y, int P,
                                                         int d, float* __restrict__ xms) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= P) return;
  const float4* xr = (const float4*)(x + (size_t)t * d);
  uint4* yr = y + (size_t)t * (d / 8);
  float acc = 0.f;
  for (int i = lane; i < d / 8; i += 64) {
    float4 u, v;
    __half2 a, b, c, e;
    if (LAYOUT == 2) {
      const int blk = i >> 3, w = i & 7;
      u = xr[blk * 16 + w];
      v = xr[blk * 16 + 8 + w];
      a = __floats2half2_rn(u.x, u.z); b = __floats2half2_rn(v.x, v.z);
      c = __floats2half2_rn(u.y, u.w); e = __floats2half2_rn(v.y, v.w);
    } else if (LAYOUT == 0) {
      u = xr[2 * i];
      v = xr[2 * i + 1];
      a = __floats2half2_rn(u.x, u.y); b = __floats2half2_rn(u.z, u.w);
      c = __floats2half2_rn(v.x, v.y); e = __floats2half2_rn(v.z, v.w);
    } else {
      u = xr[2 * i];
      v = xr[2 * i + 1];
      a = __floats2half2_rn(u.x, v.x); b = __floats2half2_rn(u.y, v.y);
      c = __floats2half2_rn(u.z, v.z); e = __floats2half2_rn(u.w, v.w);
    }
    acc += ((u.x * u.x + u.y * u.y) + (u.z * u.z + u.w * u.w)) + ((v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w));
    uint4 o;
    o.x = *(const uint32_t*)&a; o.y = *(const uint32_t*)&b; o.z = *(const uint32_t*)&c; o.w = *(const uint32_t*)&e;
    yr[i] = o;
  }
#pragma unroll
  for (int o = 32; o; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (lane == 0) xms[t] = acc / (float)d;
}

// out[t][c] = sum_{s<K} pw[pid_s] * pairs[pid_s][c]  (pid_s = pairids[t*K+s], ascending expert id)
//            + sigmoid(sg[t]) * ey[t][c]             (ey f32, or row `sh_first + t` of pairs)
// One thread per 8 consecutive columns (16-byte loads of f16 pairs); grid (ceil(D/8/256), P).
template <class PT>
struct Ld8;
template <>
struct Ld8<__half> {
  static __device__ __forceinline__ void ld(const __half* p, float* v) {
    const uint4 u = *(const uint4*)p;
    const __half2* h = (const __half2*)&u;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const float2 f = __half22float2(h[i]);
      v[2 * i] = f.x;
      v[2 * i + 1] = f.y;
    }
  }
};
template <>
struct Ld8<float> {
  static __device__ __forceinline__ void ld(const float* p, float* v) {
    const float4 a = ((const float4*)p)[0], b = ((const float4*)p)[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
};

__global__ void __launch_bounds__(256) k_zero_f32(float4* __restrict__ p, uint64_t n4) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (uint64_t)gridDim.x * 256)
    p[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

template <class PT, int KMAX, int KC>  // KC = K when it is one of the instantiated values, else 0
__global__ void __launch_bounds__(128) k_reduce_pw_sg(const PT* __restrict__ pairs,
                                                      const int* __restrict__ pairids,
                                                      const float* __restrict__ pw,
                                                      const float* __restrict__ ey,
                                                      const float* __restrict__ sg, int sh_first,
                                                      float* __restrict__ out, int P, int D, int K,
                                                      moe_hscale hs, moe_hc hc, const float* __restrict__ rot_svh) {
  __shared__ int ids[KMAX];
  __shared__ float w[KMAX];
  const int t = blockIdx.y;
  if (threadIdx.x < K) {
    const int id = pairids[(size_t)t * K + threadIdx.x];
    ids[threadIdx.x] = id;
    w[threadIdx.x] = pw[id];
  }
  __syncthreads();
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (c >= D) return;
  float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (KC > 0) {
    // K known at compile time: all pair rows are requested before the first is used (a load under
    // the run-time `s < K` test is waited for where it is issued), summed in the same slot order
    float v[KC > 0 ? KC : 1][8];
#pragma unroll
    for (int s = 0; s < KC; s++) Ld8<PT>::ld(pairs + (size_t)ids[s] * D + c, v[s]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < KC; s++) {
      const float ww = w[s];
#pragma unroll
      for (int i = 0; i < 8; i++) sum[i] += ww * v[s][i];
    }
  } else {
#pragma unroll
    for (int s = 0; s < KMAX; s++)
      if (s < K) {
        float v[8];
        Ld8<PT>::ld(pairs + (size_t)ids[s] * D + c, v);
        const float ww = w[s];
#pragma unroll
        for (int i = 0; i < 8; i++) sum[i] += ww * v[i];
      }
  }
  // pairs of the batch path carry the f16 range-guard factor of their token: divide it out
  float inv_r = 1.f, inv_s = 1.f;
  if (hs.xms) {
    const float ms = hs.xms[t];
    inv_r = 1.f / moe_hid_scale(hs.c_routed, ms);
    inv_s = 1.f / moe_hid_scale(hs.c_shared, ms);
#pragma unroll
    for (int i = 0; i < 8; i++) sum[i] *= inv_r;
  }
  if (rot_svh) {
    // hgn v2 rotated experts: the weighted sum is still in the rotated domain; svh . H(sum) / sqrt(128) per 128 block
    // before the shared expert is added (reference: k_v2_reduce_rot, src/gpu/parts/28_kernels_hgn_v2.inc:153-187).
    // D % 128 == 0: the 16 lanes of a block are all here.
    moe_fwht128_r8(sum, threadIdx.x);
    const float4 a = ((const float4*)(rot_svh + c))[0], b = ((const float4*)(rot_svh + c))[1];
    const float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int i = 0; i < 8; i++) sum[i] = sum[i] * MOE_RS128 * f[i];
  }
  if (sg) {
    const float g = sigmoid_f(sg[t]) * (ey ? 1.f : inv_s);
    float v[8];
    if (ey) Ld8<float>::ld(ey + (size_t)t * D + c, v);
    else Ld8<PT>::ld(pairs + (size_t)(sh_first + t) * D + c, v);
#pragma unroll
    for (int i = 0; i < 8; i++) sum[i] += g * v[i];
  }
  if (hc.R) {
    // HC write-back fused into the combine (reference: k_moe_reduce_pw_sg_hc, 24_kernels_moe_lt.inc:126-161):
    // the four branches of the bf16 state R[t][b][:] take inj_b * sum, inj_b = 2 * sigmoid(w4[t][b] / 4);
    // bf16 <-> f32 as the reference's bf2f / f2bf (22_kernels_prefill.inc:4-9: round to nearest even)
    float inj[4];
#pragma unroll
    for (int b = 0; b < 4; b++) inj[b] = 2.f / (1.f + expf(-hc.w4[(size_t)t * 4 + b] * 0.25f));
#pragma unroll
    for (int b = 0; b < 4; b++) {
      uint4* Rp = (uint4*)(hc.R + ((size_t)t * 4 + b) * D + c);
      const uint4 rv = *Rp;
      const uint32_t w[4] = {rv.x, rv.y, rv.z, rv.w};
      uint32_t o[4];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const float lo = __uint_as_float(w[i] << 16) + inj[b] * sum[2 * i];
        const float hi = __uint_as_float(w[i] & 0xffff0000u) + inj[b] * sum[2 * i + 1];
        uint32_t ul = __float_as_uint(lo), uh = __float_as_uint(hi);
        ul += 0x7FFFu + ((ul >> 16) & 1u);
        uh += 0x7FFFu + ((uh >> 16) & 1u);
        o[i] = (ul >> 16) | (uh & 0xffff0000u);
      }
      *Rp = make_uint4(o[0], o[1], o[2], o[3]);
    }
    return;
  }
  float4* o = (float4*)(out + (size_t)t * D + c);
  o[0] = make_float4(sum[0], sum[1], sum[2], sum[3]);
  o[1] = make_float4(sum[4], sum[5], sum[6], sum[7]);
}

// Tiles of the routed experts (expert order, <= cap pairs each) followed by the shared expert's
// tiles: pairs [sh_first, sh_first + P) in runs of cap with expert id = n_experts; also fills
// tokidx for those pairs with the identity.
__global__ void __launch_bounds__(1024) k_tiles_shared(const int* __restrict__ eoff,
                                                       moe_tile* __restrict__ tiles, int* __restrict__ total,
                                                       int E, int cap, int P, int sh_first,
                                                       int* __restrict__ tokidx) {
  __shared__ int wsum[16];
  __shared__ int routed_total;
  const int e = threadIdx.x, lane = e & 63, w = e >> 6;
  const int first = e < E ? eoff[e] : 0;
  const int ne = e < E ? eoff[e + 1] - first : 0;
  const int count = (ne + cap - 1) / cap;
  int inc = count;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(inc, o, 64);
    if (lane >= o) inc += v;
  }
  if (lane == 63) wsum[w] = inc;
  __syncthreads();
  int base = 0;
  for (int i = 0; i < w; i++) base += wsum[i];
  const int begin = base + inc - count;
  if (e == 1023) routed_total = begin + count;
  for (int j = 0; j < count; j++) {
    moe_tile t;
    t.expert = e;
    t.first = first + j * cap;
    t.count = min(cap, ne - j * cap);
    tiles[begin + j] = t;
  }
  __syncthreads();
  const int nsh = sh_first >= 0 ? (P + cap - 1) / cap : 0;
  for (int j = e; j < nsh; j += 1024) {
    moe_tile t;
    t.expert = E;
    t.first = sh_first + j * cap;
    t.count = min(cap, P - j * cap);
    tiles[routed_total + j] = t;
  }
  if (e == 0) {
    total[0] = routed_total + nsh;
    total[1] = routed_total;
  }
  if (sh_first >= 0)
    for (int i = e; i < P; i += 1024) tokidx[sh_first + i] = i;
}
// The shared expert's tile list on its own (it does not depend on the routing): tiles over pairs
// [sh_first, sh_first + P) in runs of cap, expert id = n_experts, total = {tiles, 0 routed}; also the
// identity tokidx entries of those pairs.
__global__ void __launch_bounds__(256) k_tiles_only_shared(moe_tile* __restrict__ tiles, int* __restrict__ total,
                                                           int E, int cap, int P, int sh_first,
                                                           int* __restrict__ tokidx) {
  const int nsh = (P + cap - 1) / cap;
  const int i0 = blockIdx.x * 256 + threadIdx.x, stride = gridDim.x * 256;
  for (int j = i0; j < nsh; j += stride) {
    moe_tile t;
    t.expert = E;
    t.first = sh_first + j * cap;
    t.count = min(cap, P - j * cap);
    tiles[j] = t;
  }
  if (i0 == 0) {
    total[0] = nsh;
    total[1] = 0;
  }
  for (int i = i0; i < P; i += stride) tokidx[sh_first + i] = i;
}

}  // namespace

int moe_launch_tiles_only_shared(moe_tile* tiles, int* ntiles, int E, int cap, int P, int sh_first, int* tokidx,
                                 hipStream_t st) {
  const int n = P > (P + cap - 1) / cap ? P : (P + cap - 1) / cap;
  k_tiles_only_shared<<<(n + 255) / 256 > 64 ? 64 : (n + 255) / 256, 256, 0, st>>>(tiles, ntiles, E, cap, P, sh_first, tokidx);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// x16 (layout 1 or 2) and the mean square of every row in one launch
int moe_launch_f16_rows_meansq(const float* x, void* x16, int P, int d, int layout, float* xms, hipStream_t st) {
  if (!x || !x16 || !xms || layout < 0 || layout > 2) return MOE_E_INVALID;
  if (d % 8 || (layout == 2 && d % 64) || !moe_aligned(x, 16) || !moe_aligned(x16, 16)) return MOE_E_INVALID;
  if (P == 0) return MOE_OK;
  if (layout == 0) k_f32_to_f16_rows<0><<<(P + 3) / 4, 256, 0, st>>>(x, (uint4*)x16, P, d, xms);
  else if (layout == 2) k_f32_to_f16_rows<2><<<(P + 3) / 4, 256, 0, st>>>(x, (uint4*)x16, P, d, xms);
  else k_f32_to_f16_rows<1><<<(P + 3) / 4, 256, 0, st>>>(x, (uint4*)x16, P, d, xms);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// per-token mean square from an f16 copy of x (any element order): one wave per token
__global__ void __launch_bounds__(256) k_meansq_f16_rows(const uint4* __restrict__ x16, int P, int d,
                                                         float* __restrict__ xms) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= P) return;
  const uint4* xr = x16 + (size_t)t * (d / 8);
  float acc = 0.f;
  for (int i = lane; i < d / 8; i += 64) {
    const uint4 u = xr[i];
    const __half2* h = (const __half2*)&u;
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const float2 f = __half22float2(h[q]);
      acc += f.x * f.x + f.y * f.y;
    }
  }
#pragma unroll
  for (int o = 32; o; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (lane == 0) xms[t] = acc / (float)d;
}

int moe_launch_meansq_f16(const void* x16, int P, int d, float* xms, hipStream_t st) {
  if (!x16 || !xms || d % 8 || !moe_aligned(x16, 16)) return MOE_E_INVALID;
  if (P <= 0) return MOE_OK;
  k_meansq_f16_rows<<<(P + 3) / 4, 256, 0, st>>>((const uint4*)x16, P, d, xms);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_tiles_shared(const int* eoff, moe_tile* tiles, int* ntiles, int E, int cap, int P,
                            int sh_first, int* tokidx, hipStream_t st) {
  k_tiles_shared<<<1, 1024, 0, st>>>(eoff, tiles, ntiles, E, cap, P, sh_first, tokidx);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_reduce(const void* pairs, bool pairs_f16, const int* pairids, const float* pw,
                      const float* ey, const float* sg, int sh_first, float* out, int P, int D, int K,
                      moe_hscale hs, hipStream_t st, const moe_hc* hcp, const float* rot_svh) {
  moe_hc hc{nullptr, nullptr};
  if (hcp) {  // results go into the bf16 HC state instead of out
    if (!hcp->w4 || !hcp->R || !moe_aligned(hcp->R, 16)) return MOE_E_INVALID;
    hc = *hcp;
  }
  if (!pairs || !pairids || !pw || (!out && !hc.R)) return MOE_E_INVALID;
  if (P < 0 || D < 1 || K < 1) return MOE_E_INVALID;
  if (K > 16 || D % 8) return MOE_E_UNSUPPORTED;
  if (rot_svh && (D % 128 || !moe_aligned(rot_svh, 16))) return MOE_E_INVALID;
  if (!moe_aligned(pairs, 16) || (out && !moe_aligned(out, 16)) || (ey && !moe_aligned(ey, 16))) return MOE_E_INVALID;
  if (P == 0) return MOE_OK;
  dim3 grid((D / 8 + 127) / 128, P);
#define RED_GO(PT, KC) k_reduce_pw_sg<PT, 16, KC><<<grid, 128, 0, st>>>((const PT*)pairs, pairids, pw, ey, sg, sh_first, out, P, D, K, hs, hc, rot_svh)
  if (pairs_f16) {
    if (K == 10) RED_GO(__half, 10); else if (K == 8) RED_GO(__half, 8); else RED_GO(__half, 0);
  } else {
    if (K == 10) RED_GO(float, 10); else if (K == 8) RED_GO(float, 8); else RED_GO(float, 0);
  }
#undef RED_GO
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// Zero fill by a kernel (a memset node in a captured graph is avoided on purpose).
int moe_launch_zero_f32(float* p, uint64_t n, hipStream_t st) {
  if (!p || n % 4 || !moe_aligned(p, 16)) return MOE_E_INVALID;
  if (n == 0) return MOE_OK;
  const uint64_t n4 = n / 4;
  const unsigned grid = (unsigned)((n4 + 255) / 256 > 65536 ? 65536 : (n4 + 255) / 256);
  k_zero_f32<<<grid, 256, 0, st>>>((float4*)p, n4);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

MOE_API int moe_f32_to_f16(const float* x, void* x16, uint64_t n, int layout, moe_stream_t st) {
  if (!x || !x16) return n ? MOE_E_INVALID : MOE_OK;
  if (n % 8 || !moe_aligned(x, 16) || !moe_aligned(x16, 16) || layout < 0 || layout > 2) return MOE_E_INVALID;
  if (layout == 2 && n % 64) return MOE_E_INVALID;
  if (n == 0) return MOE_OK;
  const uint64_t n8 = n / 8;
  const unsigned grid = (unsigned)((n8 + 255) / 256 > 1048576 ? 1048576 : (n8 + 255) / 256);
  if (layout == 2) k_f32_to_f16_q4k<<<grid, 256, 0, moe_s(st)>>>((const float4*)x, (uint4*)x16, n8);
  else if (layout) k_f32_to_f16_v8<true><<<grid, 256, 0, moe_s(st)>>>((const float4*)x, (uint4*)x16, n8);
  else k_f32_to_f16_v8<false><<<grid, 256, 0, moe_s(st)>>>((const float4*)x, (uint4*)x16, n8);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

MOE_API int moe_reduce_pw_sg(const void* pairs, int pairs_f16, const int* pairids, const float* pw,
                             const float* ey, const float* sg, float* out, int P, int D, int K,
                             moe_stream_t st) {
  if ((ey == nullptr) != (sg == nullptr)) return MOE_E_INVALID;
  return moe_launch_reduce(pairs, pairs_f16 != 0, pairids, pw, ey, sg, -1, out, P, D, K, moe_hscale{nullptr, 0.f, 0.f},
                           moe_s(st), nullptr);
}

MOE_API int moe_v2_reduce_rot(const void* pairs, int pairs_f16, const int* pairids, const float* pw, const float* svh,
                              const float* ey, const float* sg, float* out, int P, int D, int K, moe_stream_t st) {
  if ((ey == nullptr) != (sg == nullptr) || !svh) return MOE_E_INVALID;
  return moe_launch_reduce(pairs, pairs_f16 != 0, pairids, pw, ey, sg, -1, out, P, D, K, moe_hscale{nullptr, 0.f, 0.f},
                           moe_s(st), nullptr, svh);
}

MOE_API int moe_reduce_pw_sg_hc(const void* pairs, int pairs_f16, const int* pairids, const float* pw,
                                const float* ey, const float* sg, const float* w4, uint16_t* R, int P, int D, int K,
                                moe_stream_t st) {
  if ((ey == nullptr) != (sg == nullptr) || !w4 || !R) return MOE_E_INVALID;
  const moe_hc hc{w4, R};
  return moe_launch_reduce(pairs, pairs_f16 != 0, pairids, pw, ey, sg, -1, nullptr, P, D, K,
                           moe_hscale{nullptr, 0.f, 0.f}, moe_s(st), &hc);
}
