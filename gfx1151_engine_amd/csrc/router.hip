// Router: logits with the CPU path's fp64 accumulation, fp64 softmax, top-k, renormalised weights.
// (reference: src/ref.cpp:68-77,565-594; src/gpu/parts/20_kernels_gemv.inc:1433-1562)
#include "common.h"
#include "qvec.h"

namespace {

template <bool BF16>
__device__ __forceinline__ float load_w(const void* W, uint64_t i) {
  if (BF16) return bf16_bits_to_f32(((const uint16_t*)W)[i]);
  return ((const float*)W)[i];
}

// ---- sequential order: bit-identical to `acc += (double)w*x` for c = 0..d-1 ----
// Block = 128 tokens x 64 weight rows, thread = 8 x 4 independent fp64 chains; operands are
// widened to fp64 once, when they are staged in LDS.  The f32*f32 product is exact in fp64, so
// fma(w, x, acc) equals the reference's multiply-then-add.  Row E (if Wx is given) is the
// shared-expert gate vector: its logit goes to out_x[t].
constexpr int RL_T = 128, RL_E = 64, RL_K = 32;
template <bool BF16>
__global__ void __launch_bounds__(256) k_router_logits_seq(const void* __restrict__ W,
                                                           const float* __restrict__ bias,
                                                           const void* __restrict__ Wx, bool wx_bf16,
                                                           const float* __restrict__ x, int P, int E,
                                                           int d, float* __restrict__ logits,
                                                           float* __restrict__ out_x) {
  __shared__ __attribute__((aligned(16))) double Xs[RL_K][RL_T + 2];
  __shared__ __attribute__((aligned(16))) double Ws[RL_K][RL_E + 2];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int e0 = blockIdx.x * RL_E, t0 = blockIdx.y * RL_T;
  const int Etot = E + (Wx ? 1 : 0);
  double acc[8][4];
#pragma unroll
  for (int j = 0; j < 8; j++)
#pragma unroll
    for (int i = 0; i < 4; i++) acc[j][i] = 0.0;
  const bool vec = (d % 4 == 0);
  for (int c0 = 0; c0 < d; c0 += RL_K) {
    // stage 128 x 32 activations and 64 x 32 weights (zero outside the matrices)
#pragma unroll
    for (int it = 0; it < (RL_T * RL_K / 4) / 256; it++) {
      const int i = tid + it * 256, r = i >> 3, c = (i & 7) * 4;
      const int t = t0 + r, cc = c0 + c;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (t < P) {
        if (vec && cc + 3 < d) {
          const float4 f = *(const float4*)(x + (size_t)t * d + cc);
          v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
        } else {
          for (int q = 0; q < 4; q++) if (cc + q < d) v[q] = x[(size_t)t * d + cc + q];
        }
      }
#pragma unroll
      for (int q = 0; q < 4; q++) Xs[c + q][r] = (double)v[q];
    }
#pragma unroll
    for (int it = 0; it < (RL_E * RL_K / 4) / 256; it++) {
      const int i = tid + it * 256, r = i >> 3, c = (i & 7) * 4;
      const int e = e0 + r, cc = c0 + c;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (e < Etot) {
        const bool ex = e == E;
        const void* src = ex ? Wx : W;
        const uint64_t base = ex ? 0 : (uint64_t)e * d;
        const bool bf = ex ? wx_bf16 : BF16;
        for (int q = 0; q < 4; q++)
          if (cc + q < d) v[q] = bf ? bf16_bits_to_f32(((const uint16_t*)src)[base + cc + q]) : ((const float*)src)[base + cc + q];
      }
#pragma unroll
      for (int q = 0; q < 4; q++) Ws[c + q][r] = (double)v[q];
    }
    __syncthreads();
#pragma unroll 4
    for (int c = 0; c < RL_K; c++) {
      double wv[4], xv[8];
#pragma unroll
      for (int i = 0; i < 4; i++) wv[i] = Ws[c][4 * tx + i];
#pragma unroll
      for (int j = 0; j < 8; j++) xv[j] = Xs[c][8 * ty + j];
#pragma unroll
      for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[j][i] = fma(wv[i], xv[j], acc[j][i]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const int t = t0 + 8 * ty + j;
    if (t >= P) continue;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int e = e0 + 4 * tx + i;
      if (e >= Etot) continue;
      float v = (float)acc[j][i];
      if (e == E) {
        out_x[t] = v;
      } else {
        if (bias) v += bias[e];
        logits[(size_t)t * E + e] = v;
      }
    }
  }
}

// ---- lane-parallel order for small P: one wave (= one block) per weight row, lanes stride the
// columns, four independent fp64 chains per lane and token, fixed combination order.  The fp64
// sum differs from the sequential one only in its last bits, so the f32 logit differs with
// probability ~1e-8 per value.  Row E (if Wx given) is the shared-expert gate vector: out_x[t] =
// its logit.  Blocks past the rows (if planes given) turn x into the digit planes of the
// integer-dot decode kernels, so that work rides along instead of costing a launch.
template <bool BF16, int TT>
__global__ void __launch_bounds__(64) k_router_logits_par(const void* __restrict__ W,
                                                          const float* __restrict__ bias,
                                                          const void* __restrict__ Wx, bool wx_bf16,
                                                          const float* __restrict__ x, int P, int E,
                                                          int d, float* __restrict__ logits,
                                                          float* __restrict__ out_x, int nrows,
                                                          uint32_t* __restrict__ planes,
                                                          float2* __restrict__ meta) {
  const int lane = threadIdx.x;
  const int row = blockIdx.x;
  if (row >= nrows) {
    const int G = d / 32, gb = (G + 63) / 64;
    const int q = row - nrows, t = q / gb, g = (q % gb) * 64 + lane;
    if (t < P && g < G) qvec_group_from_f32(x, (uint64_t)d, G, t, g, planes, meta);
    return;
  }
  const bool extra = row == E;
  const void* Wr = extra ? Wx : W;
  const uint64_t base = extra ? 0 : (uint64_t)row * d;
  const bool bf = extra ? wx_bf16 : BF16;
  for (int t0 = 0; t0 < P; t0 += TT) {
    double acc[TT][4];
#pragma unroll
    for (int i = 0; i < TT; i++)
#pragma unroll
      for (int q = 0; q < 4; q++) acc[i][q] = 0.0;
    for (int c = lane * 4; c < d; c += 256) {
      float w[4];
      if (bf) {
        const uint2 u = *(const uint2*)((const uint16_t*)Wr + base + c);
        w[0] = __uint_as_float(u.x << 16);
        w[1] = __uint_as_float(u.x & 0xffff0000u);
        w[2] = __uint_as_float(u.y << 16);
        w[3] = __uint_as_float(u.y & 0xffff0000u);
      } else {
        const float4 f = *(const float4*)((const float*)Wr + base + c);
        w[0] = f.x; w[1] = f.y; w[2] = f.z; w[3] = f.w;
      }
#pragma unroll
      for (int i = 0; i < TT; i++) {
        if (t0 + i < P) {
          const float4 xv = *(const float4*)(x + (size_t)(t0 + i) * d + c);
          acc[i][0] = fma((double)w[0], (double)xv.x, acc[i][0]);
          acc[i][1] = fma((double)w[1], (double)xv.y, acc[i][1]);
          acc[i][2] = fma((double)w[2], (double)xv.z, acc[i][2]);
          acc[i][3] = fma((double)w[3], (double)xv.w, acc[i][3]);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < TT; i++) {
      const double s = wave_sum((acc[i][0] + acc[i][1]) + (acc[i][2] + acc[i][3]));
      if (lane == 0 && t0 + i < P) {
        float v = (float)s;
        if (extra) out_x[t0 + i] = v;
        else {
          if (bias) v += bias[row];
          logits[(size_t)(t0 + i) * E + row] = v;
        }
      }
    }
  }
}

__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }

// ---- softmax + top-k, one wave per token (E <= 64*NPL) ----
template <int NPL>
__global__ void __launch_bounds__(256) k_router_topk(const float* __restrict__ logits,
                                                     int* __restrict__ ids, float* __restrict__ ws,
                                                     int P, int E, int k, int id_stride) {
  __shared__ float pbuf[4][64 * NPL];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int tok = blockIdx.x * 4 + wv;
  if (tok >= P) return;
  const float* lg = logits + (size_t)tok * E;
  float v[NPL];
  float mxf = -INFINITY;
#pragma unroll
  for (int j = 0; j < NPL; j++) {
    const int e = lane + 64 * j;
    v[j] = e < E ? lg[e] : -INFINITY;
    mxf = fmaxf(mxf, v[j]);
  }
  const double mx = (double)wave_max(mxf);
  // p = (float)exp((double)logit - mx)
  float p[NPL];
  bool exact = true;  // all partial sums representable -> any summation order gives the same fp64
#pragma unroll
  for (int j = 0; j < NPL; j++) {
    const int e = lane + 64 * j;
    p[j] = e < E ? (float)exp((double)v[j] - mx) : 0.f;
    exact = exact && (p[j] == 0.f || p[j] >= 0x1p-20f);
  }
  double se;
  if (__all(exact)) {
    double s = 0.0;
#pragma unroll
    for (int j = 0; j < NPL; j++) s += (double)p[j];
    se = wave_sum(s);
  } else {
    // very wide logit range: replay the reference's index order on one lane
#pragma unroll
    for (int j = 0; j < NPL; j++) pbuf[wv][lane + 64 * j] = p[j];
    __builtin_amdgcn_s_waitcnt(0);
    __builtin_amdgcn_wave_barrier();
    double s = 0.0;
    if (lane == 0)
      for (int e = 0; e < E; e++) s += (double)pbuf[wv][e];
    se = __shfl(s, 0, 64);
  }
  // probabilities are >= 0, so their bit patterns order like unsigned integers; key = bits + 1
  // (0 = not a candidate: past E, or already selected)
  uint32_t key[NPL];
#pragma unroll
  for (int j = 0; j < NPL; j++) {
    const int e = lane + 64 * j;
    key[j] = e < E ? __float_as_uint((float)((double)p[j] / se)) + 1u : 0u;
  }
  // k rounds of arg-max: larger probability first, equal probabilities -> lower index.  The
  // maximum goes through DPP row operations + four lane reads (no LDS round trips); the lowest
  // index holding it is found with ballots: register j holds indices [64j, 64j+63], so the first
  // register with a hit has the lowest index range and its lowest set lane the lowest index.
  double wsum = 0.0;
  float mine = 0.f;  // lane r keeps the r-th selected probability
  for (int r = 0; r < k; r++) {
    uint32_t m = key[0];
#pragma unroll
    for (int j = 1; j < NPL; j++) m = m > key[j] ? m : key[j];
    m = umax(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0xB1, 0xf, 0xf, true));
    m = umax(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x4E, 0xf, 0xf, true));
    m = umax(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x141, 0xf, 0xf, true));
    m = umax(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x140, 0xf, 0xf, true));
    const uint32_t wm = umax(umax((uint32_t)__builtin_amdgcn_readlane((int)m, 0), (uint32_t)__builtin_amdgcn_readlane((int)m, 16)),
                             umax((uint32_t)__builtin_amdgcn_readlane((int)m, 32), (uint32_t)__builtin_amdgcn_readlane((int)m, 48)));
    int bi = -1;
#pragma unroll
    for (int j = 0; j < NPL; j++) {
      const unsigned long long hit = __ballot(key[j] == wm);
      if (bi < 0 && hit) bi = 64 * j + (__ffsll((long long)hit) - 1);
    }
    const float bv = __uint_as_float(wm - 1u);
    wsum += (double)bv;  // selection order, as the reference's loop over idx[0..k)
    if (lane == r) mine = bv;
    if (lane == 0) ids[(size_t)tok * id_stride + r] = bi;
    if ((bi & 63) == lane) {
#pragma unroll
      for (int j = 0; j < NPL; j++)
        if (j == (bi >> 6)) key[j] = 0u;
    }
  }
  if (lane < k) ws[(size_t)tok * id_stride + lane] = (float)((double)mine / wsum);
}

}  // namespace

MOE_API int moe_router_logits(const moe_wview* W, const float* bias, const float* x, int P,
                              float* logits, int mode, moe_stream_t st) {
  if (!W || !W->data || !x || !logits) return MOE_E_INVALID;
  if (W->dtype != MOE_DT_F32 && W->dtype != MOE_DT_BF16) return MOE_E_UNSUPPORTED;
  if (P < 0 || W->rows == 0 || W->cols == 0 || W->rows > (1u << 20) || W->cols > (1u << 24))
    return MOE_E_INVALID;
  if (P == 0) return MOE_OK;
  const int E = (int)W->rows, d = (int)W->cols;
  const bool bf = W->dtype == MOE_DT_BF16;
  const bool par = mode == 0 && P <= 32 && d % 4 == 0 && moe_aligned(x, 16) && moe_aligned(W->data, 16);
  if (par) {
    dim3 g(E);
    if (bf) k_router_logits_par<true, 4><<<g, 64, 0, moe_s(st)>>>(W->data, bias, nullptr, false, x, P, E, d, logits, nullptr, E, nullptr, nullptr);
    else k_router_logits_par<false, 4><<<g, 64, 0, moe_s(st)>>>(W->data, bias, nullptr, false, x, P, E, d, logits, nullptr, E, nullptr, nullptr);
  } else {
    dim3 g((E + RL_E - 1) / RL_E, (P + RL_T - 1) / RL_T);
    if (bf) k_router_logits_seq<true><<<g, 256, 0, moe_s(st)>>>(W->data, bias, nullptr, false, x, P, E, d, logits, nullptr);
    else k_router_logits_seq<false><<<g, 256, 0, moe_s(st)>>>(W->data, bias, nullptr, false, x, P, E, d, logits, nullptr);
  }
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// Internal: sequential-order logits for any P (also used for the one-row shared-expert gate).
int moe_router_logits_seq(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x, int P,
                          float* logits, float* out_x, hipStream_t st) {
  const int E = (int)W->rows, d = (int)W->cols;
  const bool xbf = Wx && Wx->dtype == MOE_DT_BF16;
  const void* wx = Wx ? Wx->data : nullptr;
  dim3 g((E + (Wx ? 1 : 0) + RL_E - 1) / RL_E, (P + RL_T - 1) / RL_T);
  if (W->dtype == MOE_DT_BF16) k_router_logits_seq<true><<<g, 256, 0, st>>>(W->data, bias, wx, xbf, x, P, E, d, logits, out_x);
  else k_router_logits_seq<false><<<g, 256, 0, st>>>(W->data, bias, wx, xbf, x, P, E, d, logits, out_x);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// Internal: small-P logits plus the shared-expert gate row (and, if planes != nullptr, the digit
// planes of x for the integer-dot decode kernels) in the same launch.
int moe_router_logits_small(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x,
                            int P, float* logits, float* out_x, uint32_t* planes, float2* meta,
                            hipStream_t st) {
  const int E = (int)W->rows, d = (int)W->cols;
  const bool bf = W->dtype == MOE_DT_BF16;
  const bool xbf = Wx && Wx->dtype == MOE_DT_BF16;
  const int nrows = E + (Wx ? 1 : 0);
  const int qblocks = planes ? P * ((d / 32 + 63) / 64) : 0;
  dim3 g(nrows + qblocks);
  if (bf) k_router_logits_par<true, 4><<<g, 64, 0, st>>>(W->data, bias, Wx ? Wx->data : nullptr, xbf, x, P, E, d, logits, out_x, nrows, planes, meta);
  else k_router_logits_par<false, 4><<<g, 64, 0, st>>>(W->data, bias, Wx ? Wx->data : nullptr, xbf, x, P, E, d, logits, out_x, nrows, planes, meta);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

MOE_API int moe_router_topk(const float* logits, int* ids, float* ws, int P, int E, int k,
                            int id_stride, moe_stream_t st) {
  if (!logits || !ids || !ws) return MOE_E_INVALID;
  if (P < 0 || E < 1 || k < 1 || k > E || k > 64 || id_stride < k) return MOE_E_INVALID;
  if (E > 1024) return MOE_E_UNSUPPORTED;
  if (P == 0) return MOE_OK;
  dim3 g((P + 3) / 4);
  if (E <= 512) k_router_topk<8><<<g, 256, 0, moe_s(st)>>>(logits, ids, ws, P, E, k, id_stride);
  else k_router_topk<16><<<g, 256, 0, moe_s(st)>>>(logits, ids, ws, P, E, k, id_stride);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}
