// Activation conversion, tile list with the shared expert appended, and the deterministic
// top-k weighted combine (+ sigmoid-gated shared expert).
// (reference: src/gpu/parts/26_kernels_moe_gguf.inc:389; src/gpu/parts/24_kernels_moe_lt.inc:82-124;
//  src/gpu/parts/40_model.inc:8897)
#include "common.h"
#include "internal.h"

namespace {

__global__ void __launch_bounds__(256) k_f32_to_f16_v4(const float4* __restrict__ x, uint2* __restrict__ y,
                                                       uint64_t n4) {
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4;
       i += (uint64_t)gridDim.x * blockDim.x) {
    const float4 v = x[i];
    const __half2 a = __floats2half2_rn(v.x, v.y), b = __floats2half2_rn(v.z, v.w);
    uint2 o;
    o.x = *(const uint32_t*)&a;
    o.y = *(const uint32_t*)&b;
    y[i] = o;
  }
}

template <class PT>
__device__ __forceinline__ float ldp(const PT* p, size_t i);
template <>
__device__ __forceinline__ float ldp<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ __forceinline__ float ldp<__half>(const __half* p, size_t i) { return __half2float(p[i]); }

// out[t][c] = sum_{s<K} pw[pid_s] * pairs[pid_s][c]  (pid_s = pairids[t*K+s], ascending expert id)
//            + sigmoid(sg[t]) * ey[t][c]             (ey f32, or row `sh_first + t` of pairs)
template <class PT, int KMAX>
__global__ void __launch_bounds__(256) k_reduce_pw_sg(const PT* __restrict__ pairs,
                                                      const int* __restrict__ pairids,
                                                      const float* __restrict__ pw,
                                                      const float* __restrict__ ey,
                                                      const float* __restrict__ sg, int sh_first,
                                                      float* __restrict__ out, int P, int D, int K) {
  __shared__ int ids[KMAX];
  __shared__ float w[KMAX];
  const int t = blockIdx.y;
  if (threadIdx.x < K) {
    const int id = pairids[(size_t)t * K + threadIdx.x];
    ids[threadIdx.x] = id;
    w[threadIdx.x] = pw[id];
  }
  __syncthreads();
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= D) return;
  float sum = 0.f;
#pragma unroll
  for (int s = 0; s < KMAX; s++)
    if (s < K) sum += w[s] * ldp<PT>(pairs, (size_t)ids[s] * D + c);
  if (sg) {
    const float g = sigmoid_f(sg[t]);
    const float e = ey ? ey[(size_t)t * D + c] : ldp<PT>(pairs, (size_t)(sh_first + t) * D + c);
    sum += g * e;
  }
  out[(size_t)t * D + c] = sum;
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
  if (e == 0) *total = routed_total + nsh;
  if (sh_first >= 0)
    for (int i = e; i < P; i += 1024) tokidx[sh_first + i] = i;
}
}  // namespace

int moe_launch_tiles_shared(const int* eoff, moe_tile* tiles, int* ntiles, int E, int cap, int P,
                            int sh_first, int* tokidx, hipStream_t st) {
  k_tiles_shared<<<1, 1024, 0, st>>>(eoff, tiles, ntiles, E, cap, P, sh_first, tokidx);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_reduce(const void* pairs, bool pairs_f16, const int* pairids, const float* pw,
                      const float* ey, const float* sg, int sh_first, float* out, int P, int D, int K,
                      hipStream_t st) {
  if (!pairs || !pairids || !pw || !out) return MOE_E_INVALID;
  if (P < 0 || D < 1 || K < 1) return MOE_E_INVALID;
  if (K > 16) return MOE_E_UNSUPPORTED;
  if (P == 0) return MOE_OK;
  dim3 grid((D + 255) / 256, P);
  if (pairs_f16)
    k_reduce_pw_sg<__half, 16><<<grid, 256, 0, st>>>((const __half*)pairs, pairids, pw, ey, sg, sh_first, out, P, D, K);
  else
    k_reduce_pw_sg<float, 16><<<grid, 256, 0, st>>>((const float*)pairs, pairids, pw, ey, sg, sh_first, out, P, D, K);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

MOE_API int moe_f32_to_f16(const float* x, void* x16, uint64_t n, moe_stream_t st) {
  if (!x || !x16) return n ? MOE_E_INVALID : MOE_OK;
  if (n % 4 || !moe_aligned(x, 16) || !moe_aligned(x16, 8)) return MOE_E_INVALID;
  if (n == 0) return MOE_OK;
  const uint64_t n4 = n / 4;
  const unsigned grid = (unsigned)((n4 + 255) / 256 > 1048576 ? 1048576 : (n4 + 255) / 256);
  k_f32_to_f16_v4<<<grid, 256, 0, moe_s(st)>>>((const float4*)x, (uint2*)x16, n4);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

MOE_API int moe_reduce_pw_sg(const void* pairs, int pairs_f16, const int* pairids, const float* pw,
                             const float* ey, const float* sg, float* out, int P, int D, int K,
                             moe_stream_t st) {
  if ((ey == nullptr) != (sg == nullptr)) return MOE_E_INVALID;
  return moe_launch_reduce(pairs, pairs_f16 != 0, pairids, pw, ey, sg, -1, out, P, D, K, moe_s(st));
}
