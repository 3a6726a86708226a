// Batch router without the dense fp64 pass: bit-exact expert ids at a fraction of the fp64 work.
//
// The reference's router (src/ref.cpp:565-594) needs every logit as a sequential fp64 sum, but only the k
// best logits of a token decide its experts and weights; the other ~500 enter through the softmax
// normaliser alone, which cancels in the renormalised weights up to rounding.  So:
//   1. k_router_approx   all T x E logits on the f16 matrix pipe (f32 accumulation), with the row norms of x and W
//                        (for d a multiple of 128: k_router_w16 + k_router_approx2, the same arithmetic with the
//                        router matrix converted to f16 once per call and a token tile's activations read once);
//   2. k_router_cand     per token a RIGOROUS error bound B_e on each approximate logit (below) gives an interval
//                        [a_e - B_e, a_e + B_e] that holds the exact logit; tau = the k-th largest lower end; every
//                        expert whose upper end reaches tau - 1e-5 is a candidate (the true top k are among them:
//                        at least k exact logits are >= tau, and a true top-k logit is >= the k-th largest exact one);
//   3. k_router_pairs_token the candidates' logits (typically 12-18 of 512) as fp64 dot products, eight lanes per
//                        (token, candidate), written over the approximate values: the reference's float, or in
//                        rare cases its neighbour (the fp64 sum in another order than the reference's sequential
//                        one can fall on the other side of a rounding boundary);
//   4. k_router_topk_mixed  ranks the k + 1 best logits; if every gap between neighbours exceeds 1e-6 plus two ulps
//                        and all lie within 70 of the maximum, the order by logit is the reference's order by f32
//                        probability (no two of them can round to one float) and the ids are final; the weights use
//                        these logits of the selected experts and a normaliser in which the non-candidates' terms
//                        are approximate, which moves a renormalised weight by an ulp or two at most;
//   5. tokens that fail any test (near ties, a logit range where probabilities underflow, more candidates than
//      lanes, non-finite values) are listed and redone exactly: all E logits as sequential fp64 chains (k_router_exact_pairs) and the exact softmax /
//      top-k; when more than T/16 tokens are listed the dense fp64 kernel runs for the whole batch instead.
// Error bound.  a~ = fl32(sum of f16(x_c) * f16(w_c)): |f16(v) - v| <= 2^-11 |v| + 2^-25 (the second term covers
// f16 subnormals), so sum |x~ w~ - x w| <= 1.001 (2^-10 |x||w| + 2^-25 sqrt(d) (|x| + |w|)) by Cauchy-Schwarz, and
// the accumulation adds at most (RA_CHUNK * 2^-22 + (d / RA_CHUNK) * 2^-23) * 1.001 |x||w|: inside a chunk of RA_CHUNK
// columns however the matrix pipe orders and rounds its partial sums (twice the IEEE bound per addition, one addition
// charged per product), plus one IEEE f32 addition per chunk for the running sum.  Non-finite approximations
// (overflow of the f16 conversions) send the token to step 5.
#include "common.h"
#include "internal.h"
#include "topk.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef double double2v __attribute__((ext_vector_type(2)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int RA_BT = 128, RA_BE = 128, RA_K = 32;
constexpr int RA_PITCH = 80;   // bytes per LDS row: 32 f16 + 16 B of padding (the 16-byte fragment reads of 8 rows then cover all banks)
constexpr int RA_CHUNK = 128;  // columns summed in the matrix pipe's f32 accumulators before they are added to the running sums
constexpr int RC_SLOTS = 32;   // at most 31 candidates per token (+ the shared-expert gate row) in the exact pass
constexpr int RC_NC_ULP = 1 << 20;  // flag in nc[t]: one of the token's candidate logits may be an ulp off the reference's float

// ---- 1. approximate logits: block = 128 tokens x 128 experts, 4 waves as 2 x 2, wave = 64 x 64 (2 x 2 MFMA tiles) ----
// The accumulators of the matrix pipe are flushed into running f32 sums every RA_CHUNK columns, which bounds the
// rounding of the accumulation by the chunk length instead of d (see the error bound in moe_router_batch_cand).
template <bool BF16>
__global__ void __launch_bounds__(256, 2) k_router_approx(const void* __restrict__ W, const float* __restrict__ bias,
                                                         const float* __restrict__ x, int P, int E, int d,
                                                         float* __restrict__ alog, float* __restrict__ wnorm,
                                                         float* __restrict__ xnorm, float* __restrict__ out_xms,
                                                         int* __restrict__ counters, int ncol, int ntt) {
  __shared__ __attribute__((aligned(16))) uint8_t Xs[RA_BT * RA_PITCH];
  __shared__ __attribute__((aligned(16))) uint8_t Ws[RA_BE * RA_PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int n = lane & 31, h = lane >> 5, wm = wv >> 1, wn = wv & 1;
  const int b = blockIdx.x, xcd = b & 7, q = b >> 3;
  const int col = q % ncol, tt = (q / ncol) * 8 + xcd;  // the column blocks of a token tile share an XCD (and its L2 copy of x)
  if (b == 0 && tid == 0) {
    counters[0] = 0;  // tokens listed for the exact redo
    counters[1] = 0;  // (spare)                                   (first used by later launches)
  }
  if (tt >= ntt) return;
  const int e0 = col * RA_BE, t0 = tt * RA_BT;
  constexpr int NL = RA_BT * RA_K / 4 / 256;  // float4 loads per thread, slab and operand (8)
  constexpr int TPR = RA_K / 4;               // threads per row (16)

  float4 xr[NL], wr[NL];
  auto fetch = [&](int c0) {
#pragma unroll
    for (int it = 0; it < NL; it++) {
      const int i = tid + it * 256, r = i / TPR, cc = c0 + (i % TPR) * 4;
      const int t = t0 + r, e = e0 + r;
      xr[it] = t < P ? *(const float4*)(x + (size_t)t * d + cc) : float4{0.f, 0.f, 0.f, 0.f};
      if (e < E) {
        if (BF16) {
          const uint2 u = *(const uint2*)((const uint16_t*)W + (size_t)e * d + cc);
          wr[it] = float4{__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                          __uint_as_float(u.y & 0xffff0000u)};
        } else {
          wr[it] = *(const float4*)((const float*)W + (size_t)e * d + cc);
        }
      } else {
        wr[it] = float4{0.f, 0.f, 0.f, 0.f};
      }
    }
  };
  float xs2[NL], ws2[NL];
#pragma unroll
  for (int it = 0; it < NL; it++) xs2[it] = ws2[it] = 0.f;
  auto stage = [&]() {
#pragma unroll
    for (int it = 0; it < NL; it++) {
      const int i = tid + it * 256, r = i / TPR, m = i % TPR;
      const float4 a = xr[it], w = wr[it];
      xs2[it] += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
      ws2[it] += w.x * w.x + w.y * w.y + w.z * w.z + w.w * w.w;
      *(half4v*)(Xs + r * RA_PITCH + m * 8) = half4v{(_Float16)a.x, (_Float16)a.y, (_Float16)a.z, (_Float16)a.w};
      *(half4v*)(Ws + r * RA_PITCH + m * 8) = half4v{(_Float16)w.x, (_Float16)w.y, (_Float16)w.z, (_Float16)w.w};
    }
  };
  floatx16 acc[2][2], run[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = run[i][j][r] = 0.f;

  fetch(0);
  for (int c0 = 0; c0 < d; c0 += RA_K) {
    moe_lds_barrier();  // the previous slab has been read (LDS-only barriers: the next slab's loads stay in flight)
    stage();
    moe_lds_barrier();
    if (c0 + RA_K < d) fetch(c0 + RA_K);
#pragma unroll
    for (int ks = 0; ks < RA_K / 16; ks++) {
      half8 a[2], bq[2];
#pragma unroll
      for (int mf = 0; mf < 2; mf++) a[mf] = *(const half8*)(Xs + (wm * 64 + 32 * mf + n) * RA_PITCH + ks * 32 + h * 16);
#pragma unroll
      for (int nf = 0; nf < 2; nf++) bq[nf] = *(const half8*)(Ws + (wn * 64 + 32 * nf + n) * RA_PITCH + ks * 32 + h * 16);
#pragma unroll
      for (int mf = 0; mf < 2; mf++)
#pragma unroll
        for (int nf = 0; nf < 2; nf++)
          acc[mf][nf] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mf], bq[nf], acc[mf][nf], 0, 0, 0);
    }
    if ((c0 + RA_K) % RA_CHUNK == 0 || c0 + RA_K >= d) {
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            run[i][j][r] += acc[i][j][r];
            acc[i][j][r] = 0.f;
          }
    }
  }
  // D[i][j]: j = lane % 32 (expert), i = 8 * (r / 4) + 4 * (lane / 32) + r % 4 (token)
#pragma unroll
  for (int mf = 0; mf < 2; mf++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int t = t0 + wm * 64 + 32 * mf + 8 * (r >> 2) + 4 * h + (r & 3);
      if (t >= P) continue;
#pragma unroll
      for (int nf = 0; nf < 2; nf++) {
        const int e = e0 + wn * 64 + 32 * nf + n;
        if (e < E) alog[(size_t)t * E + e] = run[mf][nf][r] + (bias ? bias[e] : 0.f);
      }
    }
  // row norms: the TPR threads that share a row are consecutive lanes
#pragma unroll
  for (int it = 0; it < NL; it++) {
    float sx = xs2[it], sw = ws2[it];
#pragma unroll
    for (int o = 1; o < TPR; o <<= 1) {
      sx += __shfl_xor(sx, o, 64);
      sw += __shfl_xor(sw, o, 64);
    }
    const int r = (tid + it * 256) / TPR;
    if (tid % TPR == 0) {
      if (col == 0 && t0 + r < P) {
        xnorm[t0 + r] = sqrtf(sx);
        if (out_xms) out_xms[t0 + r] = sx / (float)d;
      }
      if (tt == 0 && e0 + r < E) wnorm[e0 + r] = sqrtf(sw);
    }
  }
}

// ---- 1'. the same approximate logits with the router matrix converted once per call ----
// k_router_w16: W -> f16 (round to nearest even, the conversion the error bound charges) in scratch, rows padded with
// zeros to a multiple of R2_BE, and the row norms of W (from the unrounded values).  A wave per row.
constexpr int R2_BT = 64, R2_BE = 512, R2_K = 32, R2_NBUF = 4;
constexpr int R2_WBYTES = R2_BE * R2_K * 2, R2_XBYTES = R2_BT * R2_K * 2;  // per slab: 32 KB of W16, 4 KB of x as f16
constexpr int R2_SMEM = R2_NBUF * R2_WBYTES + 2 * R2_XBYTES;

template <bool BF16>
__global__ void __launch_bounds__(256) k_router_w16(const void* __restrict__ W, int E, int Epad, int d,
                                                    __half* __restrict__ W16, float* __restrict__ wnorm,
                                                    int* __restrict__ counters) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int row = blockIdx.x * 4 + wv;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    counters[0] = 0;  // tokens listed for the exact redo
    counters[1] = 0;  // (spare)                                   (first used by later launches)
  }
  if (row >= Epad) return;
  float s2 = 0.f;
  for (int c = 4 * lane; c < d; c += 256) {
    float4 w = float4{0.f, 0.f, 0.f, 0.f};
    if (row < E) {
      if (BF16) {
        const uint2 u = *(const uint2*)((const uint16_t*)W + (size_t)row * d + c);
        w = float4{__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                   __uint_as_float(u.y & 0xffff0000u)};
      } else {
        w = *(const float4*)((const float*)W + (size_t)row * d + c);
      }
    }
    s2 += w.x * w.x + w.y * w.y + w.z * w.z + w.w * w.w;
    // slab-major tiles [column group of R2_BE rows][32-column slab][row][four 16-byte chunks, chunk q in slot
    // q ^ ((row >> 2) & 3)]: a slab of a column group is 32 KB of consecutive bytes in the order the LDS image has
    const int rl = row % R2_BE, sl = c / R2_K, q = (c % R2_K) >> 3;
    __half* dst = W16 + ((size_t)(row / R2_BE) * (d / R2_K) + sl) * (R2_BE * R2_K) + (size_t)rl * R2_K +
                  ((q ^ ((rl >> 2) & 3)) << 3) + (c & 7);
    *(half4v*)dst = half4v{(_Float16)w.x, (_Float16)w.y, (_Float16)w.z, (_Float16)w.w};
  }
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) s2 += __shfl_xor(s2, o, 64);
  if (lane == 0 && row < E) wnorm[row] = sqrtf(s2);
}

// k_router_approx2: block = 64 tokens x 512 experts, 8 waves of 64 x 64 (2 x 2 MFMA tiles); a token tile's activations
// are read and converted once (the first kernel's four column blocks each did it again).  Per 32-column slab the f16
// rows of W go global -> LDS directly (64-byte rows, the 16-byte chunk c of row r in slot c ^ ((r >> 2) & 3): the
// fragment reads of 16 rows then cover all banks), four slab buffers; x is converted by its loader threads into a
// double-buffered tile.  The two operands come from different distances -- W out of L2 (every block reads the same
// 3 MB), x out of HBM -- and a wave's loads retire in order, so the loading is split between the waves: waves 0-3
// fetch x eight slabs ahead (registers), waves 4-7 fetch W three slabs ahead (LDS), each half with a wait count of
// its own.  One block barrier per slab.  Accumulators are flushed into running sums every RA_CHUNK columns, as in
// k_router_approx: the error bound is the same.
constexpr int R2_XD = 8;  // slabs of x in flight
typedef float f32x4_nt __attribute__((ext_vector_type(4)));
// 16 bytes that this kernel reads exactly once: loaded as streaming data, so that they do not push the f16 router
// matrix (read by every block) out of L2
__device__ __forceinline__ float4 ld_stream4(const float* p) {
  const f32x4_nt v = __builtin_nontemporal_load((const f32x4_nt*)p);
  return float4{v.x, v.y, v.z, v.w};
}
__global__ void __launch_bounds__(512, 1) k_router_approx2(const __half* __restrict__ W16, const float* __restrict__ bias,
                                                         const float* __restrict__ x, int P, int E, int d,
                                                         float* __restrict__ alog, float* __restrict__ xnorm,
                                                         float* __restrict__ out_xms) {
  extern __shared__ __attribute__((aligned(16))) uint8_t r2sm[];
  uint8_t* const Wl = r2sm;
  uint8_t* const Xl = r2sm + R2_NBUF * R2_WBYTES;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool xwave = wv < 4;
  const int n = lane & 31, h = lane >> 5;
  const int t0 = blockIdx.x * R2_BT, e0 = blockIdx.y * R2_BE;
  const int nslab = d / R2_K;
  // W16 (waves 4-7): a slab of this column group is 32 KB of consecutive bytes in LDS order (k_router_w16); wave
  // instruction j = 8 (wv - 4) + i copies bytes [1024 j, 1024 j + 1024)
  const int wj0 = 8 * (wv & 3);
  const uint8_t* const wsrc = (const uint8_t*)W16 + (size_t)blockIdx.y * nslab * R2_WBYTES + wj0 * 1024 + lane * 16;
  auto issue_w = [&](int s) {
    uint8_t* dst = Wl + (s % R2_NBUF) * R2_WBYTES + wj0 * 1024;
#pragma unroll
    for (int i = 0; i < 8; i++)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(wsrc + (size_t)s * R2_WBYTES + i * 1024),
                                       (__attribute__((address_space(3))) void*)(dst + i * 1024), 16, 0, 0);
  };
  // x (waves 0-3): thread -> float4 f = tid + 256 j (j = 0, 1) of the slab: token row f / 8, columns 4 (f % 8) .. + 3
  const float* xsrc[2];
  uint8_t* xdst[2];
  bool xlive[2];
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int f = (tid & 255) + 256 * j, row = f >> 3, p = f & 7;
    xlive[j] = t0 + row < P;
    xsrc[j] = x + (size_t)(xlive[j] ? t0 + row : 0) * d + 4 * p;
    xdst[j] = Xl + row * 64 + (((p >> 1) ^ ((row >> 2) & 3)) << 4) + (p & 1) * 8;
  }
  float4 xq[R2_XD][2];
  float xs2[2] = {0.f, 0.f};
  floatx16 acc[2][2], run[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = run[i][j][r] = 0.f;
  if (xwave) {
#pragma unroll
    for (int s = 0; s < R2_XD; s++)
      if (s < nslab) {
#pragma unroll
        for (int j = 0; j < 2; j++) xq[s][j] = ld_stream4(xsrc[j] + (size_t)s * R2_K);
      }
  } else {
#pragma unroll
    for (int s = 0; s < 3; s++)
      if (s < nslab) issue_w(s);
  }
  for (int s0 = 0; s0 < nslab; s0 += R2_XD) {
#pragma unroll
    for (int u = 0; u < R2_XD; u++) {
      const int s = s0 + u;
      if (s >= nslab) break;
      if (xwave) {
        // (the compiler waits for xq[u]: the seven later slabs' loads stay in flight)
#pragma unroll
        for (int j = 0; j < 2; j++) {
          const float4 a = xlive[j] ? xq[u][j] : float4{0.f, 0.f, 0.f, 0.f};
          xs2[j] += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
          *(half4v*)(xdst[j] + (s & 1) * R2_XBYTES) = half4v{(_Float16)a.x, (_Float16)a.y, (_Float16)a.z, (_Float16)a.w};
        }
      } else {
        // slab s has landed when at most the loads of the (up to two) later slabs in flight are outstanding
        const int later = nslab - 1 - s < 2 ? nslab - 1 - s : 2;
        if (later == 2) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        else if (later == 1) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      // slab s of W (its loaders waited for it) and of x is in LDS; slab s - 1 has been read by all.  An LDS-only
      // barrier: __syncthreads() would wait for every load in flight
      moe_lds_barrier();
      if (xwave) {
        if (s + R2_XD < nslab) {
#pragma unroll
          for (int j = 0; j < 2; j++) xq[u][j] = ld_stream4(xsrc[j] + (size_t)(s + R2_XD) * R2_K);
        }
      } else if (s + 3 < nslab) {
        issue_w(s + 3);
      }
      const uint8_t* Wb = Wl + (s % R2_NBUF) * R2_WBYTES;
      const uint8_t* Xb = Xl + (s & 1) * R2_XBYTES;
#pragma unroll
      for (int ks = 0; ks < R2_K / 16; ks++) {
        half8 a[2], b[2];
#pragma unroll
        for (int mf = 0; mf < 2; mf++) {
          const int row = 32 * mf + n;
          a[mf] = *(const half8*)(Xb + row * 64 + (((2 * ks + h) ^ ((row >> 2) & 3)) << 4));
        }
#pragma unroll
        for (int nf = 0; nf < 2; nf++) {
          const int row = 64 * wv + 32 * nf + n;
          b[nf] = *(const half8*)(Wb + row * 64 + (((2 * ks + h) ^ ((row >> 2) & 3)) << 4));
        }
#pragma unroll
        for (int mf = 0; mf < 2; mf++)
#pragma unroll
          for (int nf = 0; nf < 2; nf++)
            acc[mf][nf] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mf], b[nf], acc[mf][nf], 0, 0, 0);
      }
      if (((s + 1) * R2_K) % RA_CHUNK == 0 || s + 1 == nslab) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
              run[i][j][r] += acc[i][j][r];
              acc[i][j][r] = 0.f;
            }
      }
    }
  }
  // D[i][j]: j = lane % 32 (expert), i = 8 * (r / 4) + 4 * (lane / 32) + r % 4 (token)
#pragma unroll
  for (int mf = 0; mf < 2; mf++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int t = t0 + 32 * mf + 8 * (r >> 2) + 4 * h + (r & 3);
      if (t >= P) continue;
#pragma unroll
      for (int nf = 0; nf < 2; nf++) {
        const int e = e0 + 64 * wv + 32 * nf + n;
        if (e < E) alog[(size_t)t * E + e] = run[mf][nf][r] + (bias ? bias[e] : 0.f);
      }
    }
  // row norms of x: the 8 threads of a row are consecutive lanes of the loading waves
  if (xwave) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      float v = xs2[j];
      v += __shfl_xor(v, 1, 64);
      v += __shfl_xor(v, 2, 64);
      v += __shfl_xor(v, 4, 64);
      const int f = (tid & 255) + 256 * j, row = f >> 3;
      if (blockIdx.y == 0 && (f & 7) == 0 && xlive[j]) {
        xnorm[t0 + row] = sqrtf(v);
        if (out_xms) out_xms[t0 + row] = v / (float)d;
      }
    }
  }
}

// ---- 2. candidates: one wave per token, lane l holds experts NPL*l .. NPL*l + NPL - 1 ----
template <int NPL>
__global__ void __launch_bounds__(1024) k_router_cand(const float* __restrict__ alog, const float* __restrict__ wnorm,
                                                     const float* __restrict__ xnorm, int P, int E, int k, float eps,
                                                     float dterm, uint32_t* __restrict__ pairs, int* __restrict__ nc,
                                                     int* __restrict__ fb_list, int* __restrict__ counters, int gate_row) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int t = blockIdx.x * 16 + wv;
  const bool tok = t < P;
  const float xn = xnorm[tok ? t : 0];
  float U[NPL], L[NPL];
  bool fin = isfinite(xn);
  float maxU = -INFINITY;
#pragma unroll
  for (int j = 0; j < NPL; j++) {
    const int e = NPL * lane + j;
    if (e < E && tok) {
      const float a = alog[(size_t)t * E + e], wn = wnorm[e];
      const float B = eps * xn * wn + dterm * (xn + wn) + 1e-6f * (1.f + fabsf(a));
      fin = fin && isfinite(a) && isfinite(B);
      U[j] = a + B;
      L[j] = a - B;
    } else {
      U[j] = L[j] = -INFINITY;
    }
    maxU = fmaxf(maxU, U[j]);
  }
  maxU = wave_fmax_dpp(maxU);
  // tau = the k-th largest lower end
  float tau = -INFINITY;
  for (int r = 0; r < k; r++) {
    float m = L[0];
#pragma unroll
    for (int j = 1; j < NPL; j++) m = fmaxf(m, L[j]);
    const float wmx = wave_fmax_dpp(m);
    const int owner = __builtin_ctzll(__ballot(m == wmx) | (1ull << 63));
    tau = wmx;
    if (lane == owner) {  // drop one instance
      bool done = false;
#pragma unroll
      for (int j = 0; j < NPL; j++) {
        const bool hit = !done && L[j] == wmx;
        L[j] = hit ? -INFINITY : L[j];
        done = done || hit;
      }
    }
  }
  const float thr = tau - 1e-5f;
  int mine = 0;
#pragma unroll
  for (int j = 0; j < NPL; j++) mine += (U[j] >= thr) ? 1 : 0;
  int inc = mine;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(inc, o, 64);
    if (lane >= o) inc += v;
  }
  const int total = __shfl(inc, 63, 64);
  const bool ok = __all(fin) && total <= RC_SLOTS - 1 && total >= 1 && (maxU - thr) < 60.f && isfinite(tau);
  // The rows whose exact dot products step 3 computes for this token: pairs[t][0 .. n), the shared-expert gate vector
  // (row E) first where there is one, then the candidates; nc[t] = the number of candidates, -1 for a listed token.
  if (!tok) return;
  uint32_t* mine_out = pairs + (size_t)t * RC_SLOTS;
  if (gate_row && lane == 0) mine_out[0] = (uint32_t)E;
  if (!ok) {
    if (lane == 0) {
      nc[t] = -1;
      fb_list[atomicAdd(&counters[0], 1)] = t;
    }
    return;
  }
  int pos = gate_row + inc - mine;
#pragma unroll
  for (int j = 0; j < NPL; j++)
    if (U[j] >= thr) mine_out[pos++] = (uint32_t)(NPL * lane + j);
  if (lane == 0) nc[t] = total;
}

// One sequential fp64 chain over c = 0..d-1 per lane: acc = fma((double)w[c], (double)x[c], acc); the f32 x f32
// product is exact in fp64, so this is the reference's `acc += (double)w * x` bit for bit.  Every lane streams its
// own weight row, 128 bytes (a cache line) at a time, the next 32 columns in flight while the current ones are used.
template <bool BF16>
__device__ __forceinline__ double chain_row(const void* wrow, const float* xrow, int d) {
  double acc = 0.0;
  float4 wq[8], xq[8];
  auto load = [&](int c) {
    if (BF16) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint4 u = *(const uint4*)((const uint16_t*)wrow + c + 8 * i);
        wq[2 * i] = float4{__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                           __uint_as_float(u.y & 0xffff0000u)};
        wq[2 * i + 1] = float4{__uint_as_float(u.z << 16), __uint_as_float(u.z & 0xffff0000u),
                               __uint_as_float(u.w << 16), __uint_as_float(u.w & 0xffff0000u)};
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) wq[i] = *(const float4*)((const float*)wrow + c + 4 * i);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) xq[i] = *(const float4*)(xrow + c + 4 * i);
  };
  load(0);
  for (int c = 0; c < d; c += 32) {
    float4 w[8], xv[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      w[i] = wq[i];
      xv[i] = xq[i];
    }
    if (c + 32 < d) load(c + 32);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      acc = fma((double)w[i].x, (double)xv[i].x, acc);
      acc = fma((double)w[i].y, (double)xv[i].y, acc);
      acc = fma((double)w[i].z, (double)xv[i].z, acc);
      acc = fma((double)w[i].w, (double)xv[i].w, acc);
    }
  }
  return acc;
}

// ---- 5. exact logits of the listed tokens, every expert: a lane per (token, row) pair, 64 pairs per wave ----
// f32 weights: a wave stages the 64 weight-row pieces of an iteration (32 columns = one 128-byte line per row)
// through LDS, so that a load instruction fetches 8 whole lines (8 lanes per row) instead of 16 bytes of 64
// different lines; lane l of instruction i takes row 8i + l/8, piece (l%8 + l/8) % 8, which lands at byte 16 l of
// the instruction's 1 KB image, and a lane reads its own row's piece j from slot 8a + (j - a) % 8, a = row % 8:
// the 8 lanes of an LDS phase then hit 8 different 16-byte bank groups.  The pairs are (listed token, expert) for
// every expert, taken from the list of tokens (fb_list, counters[0] entries; nothing to do when the dense kernel
// takes over).
// A block is one wave = one listed token and 64 of its experts: with the few tokens that are listed in practice (near
// ties: a couple in ten thousand) the launch is a handful of waves, and what it takes is the latency of one chain --
// d / 32 steps of 32 columns, each a trip to L2, 64 f32 -> f64 conversions (quarter rate) and 32 dependent fp64 FMAs.
// A step's operands are requested three steps ahead: the weight-row pieces (8 KB) and the token's 128 bytes of
// activations (one load by eight lanes) go global -> LDS, three step buffers, and a step's buffer is re-filled as
// soon as its operands are in registers.  (Six steps ahead with the next step's operands read during the current
// step's FMAs measured slower, 65 against 54 us for a handful of tokens: the chain is bound by its own instructions,
// not by the trips to memory any more; raising the wave's priority changes nothing either.)
template <bool BF16>
__global__ void __launch_bounds__(64) k_router_exact_pairs(const void* __restrict__ W, const float* __restrict__ bias,
                                                           const float* __restrict__ x, int E, int d,
                                                           const int* __restrict__ counters, float* __restrict__ logits,
                                                           const int* __restrict__ fb_list, int dense_above, int wpt) {
  constexpr int XD = 3;           // steps in flight
  constexpr int SB = 8192 + 128;  // bytes of a step buffer: 64 rows x 128 B of weights, 128 B of activations
  __shared__ __attribute__((aligned(16))) uint8_t img[XD * SB];
  const int nl = counters[0];
  if (nl == 0 || nl > dense_above) return;
  const int lane = threadIdx.x;
  const int tl = (int)blockIdx.x / wpt;  // wpt = waves per token = ceil(E / 64)
  if (tl >= nl) return;
  const int e_raw = ((int)blockIdx.x - tl * wpt) * 64 + lane;
  const bool live = e_raw < E;
  const int t = fb_list[tl], e = live ? e_raw : E - 1;  // (idle lanes repeat the last row)
  const uint8_t* wrow = (const uint8_t*)W + (size_t)e * d * (BF16 ? 2 : 4);
  const float* xrow = x + (size_t)t * d;
  double acc = 0.0;
  if constexpr (BF16) {
    acc = chain_row<true>(wrow, xrow, d);
  } else {
    // row pointers of the 8 rows this lane fetches pieces of
    const uint8_t* src[8];
    const int a = lane >> 3, piece = ((lane & 7) + a) & 7;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const uint64_t pw = (uint64_t)wrow;
      const int from = 8 * i + a;
      const uint32_t lo = (uint32_t)__shfl((int)(uint32_t)pw, from, 64), hi = (uint32_t)__shfl((int)(uint32_t)(pw >> 32), from, 64);
      src[i] = (const uint8_t*)(((uint64_t)hi << 32) | lo) + piece * 16;
    }
    auto issue = [&](int step, int buf) {  // nine loads
      const int c = step * 32;
#pragma unroll
      for (int i = 0; i < 8; i++)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src[i] + (size_t)c * 4),
                                         (__attribute__((address_space(3))) void*)(&img[buf * SB + i * 1024]), 16, 0, 0);
      if (lane < 8)  // lane l: columns c + 4 l .. of the token's activations, to byte 16 l behind the weights
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xrow + c + 4 * lane),
                                         (__attribute__((address_space(3))) void*)(&img[buf * SB + 8192]), 16, 0, 0);
    };
    const int ar = lane & 7;
    const int rd_w = (lane >> 3) * 1024 + ar * 128;  // this lane's row inside a step's weight image
    const int n = d / 32;
    for (int st = 0; st < XD && st < n; st++) issue(st, st);
    int buf = 0;
    for (int it = 0; it < n; it++) {
      // the loads of the steps behind this one stay in flight (nine per step; they retire in order)
      const int behind = n - 1 - it < XD - 1 ? n - 1 - it : XD - 1;
      if (behind >= 2) asm volatile("s_waitcnt vmcnt(18)" ::: "memory");
      else if (behind == 1) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      float4 w[8], xv[8];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        w[j] = *(const float4*)(&img[buf * SB + rd_w + (((j - ar) & 7) << 4)]);
        xv[j] = *(const float4*)(&img[buf * SB + 8192 + 16 * j]);
      }
      if (it + XD < n) {
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the step's operands are in registers, its buffer is free
        issue(it + XD, buf);
      }
#pragma unroll
      for (int i = 0; i < 8; i++) {
        acc = fma((double)w[i].x, (double)xv[i].x, acc);
        acc = fma((double)w[i].y, (double)xv[i].y, acc);
        acc = fma((double)w[i].z, (double)xv[i].z, acc);
        acc = fma((double)w[i].w, (double)xv[i].w, acc);
      }
      buf = buf + 1 == XD ? 0 : buf + 1;
    }
  }
  if (!live) return;
  float v = (float)acc;
  if (bias) v += bias[e];
  logits[(size_t)t * E + e] = v;
}

// ---- 3. the candidates' logits: a wave per token, eight lanes per (token, row) pair ----
// What step 4 needs from a candidate's logit is the fp64 dot product rounded to f32.  Summed in any order the fp64
// value lies within delta = 2 (d + 8) 2^-53 |w||x| of the reference's sequential sum, so it rounds to the reference's
// float unless a rounding boundary lies within delta of it; the kernel tests exactly that and marks the token
// (RC_NC_ULP in nc[t], a few in ten thousand pairs) so that step 4 allows for an ulp in that token's gap test.  So
// the candidates do not need the sequential chain (the listed tokens of step 5, whose ids hang on the last bit, keep it).
// A wave takes one token and eight of its rows at a time; lane j of a row's eight takes the 16-byte piece j of every
// 128-byte line of the row, so that a load instruction covers eight whole lines, with no trip through LDS for the
// weights.  The token's activations are the same for all rows: the wave fetches them once per pass, 256 columns per
// load instruction, and hands them round through LDS -- loaded per lane like the weights they were half of the load
// instructions, and the rate of those is what bounds this kernel.  The next chunk's weights are requested before the
// current chunk is summed.  Two accumulators per lane, a three-step reduction; the order is fixed.
template <bool BF16>
__global__ void __launch_bounds__(256) k_router_pairs_token(const void* __restrict__ W, const float* __restrict__ bias,
                                                            const void* __restrict__ Wx, const float* __restrict__ x,
                                                            int P, int E, int d, const uint32_t* __restrict__ pairs,
                                                            float* __restrict__ logits, float* __restrict__ out_x,
                                                            const float* __restrict__ wnorm, const float* __restrict__ xnorm,
                                                            int* __restrict__ nc, int gate_row) {
  constexpr int CH = 256;                    // columns of x per wave load
  constexpr int LINE = BF16 ? 64 : 32;       // columns per 128-byte line of a weight row
  constexpr int NL = CH / LINE;              // lines per chunk
  constexpr int ESZ = BF16 ? 2 : 4;
  // (the activations lie in LDS widened to f64: f32 -> f64 conversions run at a quarter of the FMA rate, and a lane
  //  would otherwise convert the same 4 activations per line that the 63 other lanes convert too)
  __shared__ double2v xl[4][2][128];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int t = blockIdx.x * 4 + wv;
  if (t >= P) return;
  const int ncv = nc[t];
  const int cnt = (ncv < 0 ? 0 : ncv) + gate_row;  // (the marks of this launch are set after every wave's own read)
  const int slot = lane >> 3, j = lane & 7;
  const float* xrow = x + (size_t)t * d;
  const uint32_t* mine = pairs + (size_t)t * RC_SLOTS;
  const int nchunk = (d + CH - 1) / CH;
  // (d is a multiple of 32 columns; a piece past the row's end is read from the row's last 16 bytes instead and meets
  //  zeros in the activations' chunk)
  const int last_piece = d * ESZ - 16;
  for (int p0 = 0; p0 < cnt; p0 += 8) {
    const bool live = p0 + slot < cnt;
    const int e = (int)mine[live ? p0 + slot : p0];  // idle slots repeat the pass's first row (no extra traffic)
    const bool gate = e == E;
    const uint8_t* wrow = gate ? (const uint8_t*)Wx : (const uint8_t*)W + (size_t)e * d * ESZ;
    double a0 = 0.0, a1 = 0.0;
    uint4 wc[NL], wn[NL];
    auto load_w = [&](int g, uint4* w) {
#pragma unroll
      for (int l = 0; l < NL; l++) {
        const int off = (g * CH + l * LINE) * ESZ + 16 * j;
        w[l] = *(const uint4*)(wrow + (off < last_piece ? off : last_piece));
      }
    };
    load_w(0, wc);
    float4 xn = 4 * lane < d ? *(const float4*)(xrow + 4 * lane) : float4{0.f, 0.f, 0.f, 0.f};
    int buf = 0;
    for (int g = 0; g < nchunk; g++) {
      xl[wv][buf][2 * lane] = double2v{(double)xn.x, (double)xn.y};
      xl[wv][buf][2 * lane + 1] = double2v{(double)xn.z, (double)xn.w};
      if (g + 1 < nchunk) {
        const int c1 = (g + 1) * CH + 4 * lane;
        xn = c1 < d ? *(const float4*)(xrow + c1) : float4{0.f, 0.f, 0.f, 0.f};
        load_w(g + 1, wn);
      }
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the wave's own LDS writes
      __builtin_amdgcn_wave_barrier();
      const double2v* xs = &xl[wv][buf][0];
#pragma unroll
      for (int l = 0; l < NL; l++) {
        double& acc = (l & 1) ? a1 : a0;
        const uint4 u = wc[l];
        if (BF16) {
          const double2v xa = xs[l * 32 + 4 * j], xb = xs[l * 32 + 4 * j + 1], xc = xs[l * 32 + 4 * j + 2], xd = xs[l * 32 + 4 * j + 3];
          struct { double x, y, z, w; } x0{xa.x, xa.y, xb.x, xb.y}, x1{xc.x, xc.y, xd.x, xd.y};
          acc = fma((double)__uint_as_float(u.x << 16), (double)x0.x, acc);
          acc = fma((double)__uint_as_float(u.x & 0xffff0000u), (double)x0.y, acc);
          acc = fma((double)__uint_as_float(u.y << 16), (double)x0.z, acc);
          acc = fma((double)__uint_as_float(u.y & 0xffff0000u), (double)x0.w, acc);
          acc = fma((double)__uint_as_float(u.z << 16), (double)x1.x, acc);
          acc = fma((double)__uint_as_float(u.z & 0xffff0000u), (double)x1.y, acc);
          acc = fma((double)__uint_as_float(u.w << 16), (double)x1.z, acc);
          acc = fma((double)__uint_as_float(u.w & 0xffff0000u), (double)x1.w, acc);
        } else {
          const double2v xa = xs[l * 16 + 2 * j], xb = xs[l * 16 + 2 * j + 1];
          acc = fma((double)__uint_as_float(u.x), xa.x, acc);
          acc = fma((double)__uint_as_float(u.y), xa.y, acc);
          acc = fma((double)__uint_as_float(u.z), xb.x, acc);
          acc = fma((double)__uint_as_float(u.w), xb.y, acc);
        }
      }
#pragma unroll
      for (int l = 0; l < NL; l++) wc[l] = wn[l];
      buf ^= 1;
    }
    double acc = a0 + a1;
#pragma unroll
    for (int o = 1; o < 8; o <<= 1) acc += __shfl_xor(acc, o, 64);
    if (live && j == 0) {
      if (gate) out_x[t] = (float)acc;
      else {
        float v = (float)acc;
        const double delta = (double)(2.f * (float)(d + 8) * 0x1p-53f * 1.01f) * (double)wnorm[e] * (double)xnorm[t];
        if ((float)(acc - delta) != v || (float)(acc + delta) != v) atomicOr(&nc[t], RC_NC_ULP);
        if (bias) v += bias[e];
        logits[(size_t)t * E + e] = v;
      }
    }
  }
}

// ---- 4. ids and weights from the mixed logits (exact for the candidates) ----
template <int NPL>
__global__ void __launch_bounds__(256) k_router_topk_mixed(const float* __restrict__ lg, int* __restrict__ ids,
                                                           float* __restrict__ ws, int P, int E, int k, int id_stride,
                                                           const int* __restrict__ nc, int* __restrict__ fb_list,
                                                           int* __restrict__ counters, float bias_max) {
  static_assert(NPL <= 8, "4-bit index fields in one 32-bit word");
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int t = blockIdx.x * 4 + wv;
  if (t >= P || nc[t] < 0) return;  // listed already
  float v[NPL];
  uint32_t key[NPL], jj[NPL];
#pragma unroll
  for (int j = 0; j < NPL; j++) {
    const int e = NPL * lane + j;
    v[j] = e < E ? lg[(size_t)t * E + e] : -INFINITY;
    const uint32_t u = __float_as_uint(v[j]);
    key[j] = e < E ? ((u & 0x80000000u) ? ~u : (u | 0x80000000u)) : 0u;  // unsigned keys that order like the floats
    jj[j] = (uint32_t)j;
  }
#pragma unroll
  for (int pass = 0; pass < NPL; pass++) {
#pragma unroll
    for (int i = pass & 1; i + 1 < NPL; i += 2) {
      const uint32_t ka = key[i], kb = key[i + 1], ia = jj[i], ib = jj[i + 1];
      const bool sw = kb > ka;
      key[i] = umax(ka, kb); key[i + 1] = umin(ka, kb);
      jj[i] = sw ? ib : ia; jj[i + 1] = sw ? ia : ib;
    }
  }
  uint32_t jw = 0;
#pragma unroll
  for (int j = 0; j < NPL; j++) jw |= jj[j] << (4 * j);
  uint32_t mykey = 0;
  int myid = 0;
  for (int r = 0; r <= k; r++) {  // k + 1 rounds: the runner-up is needed for the gap test
    const uint32_t wmx = wave_umax(key[0]);
    const int wl = __builtin_ctzll(__ballot(key[0] == wmx) | (1ull << 63));
    const int wj = __builtin_amdgcn_readlane((int)jw, wl) & 15;
    if (lane == r) {
      mykey = wmx;
      myid = NPL * wl + wj;
    }
    const bool me = lane == wl;
#pragma unroll
    for (int j = 0; j + 1 < NPL; j++) {
      const uint32_t cur = key[j], nxt = key[j + 1];
      key[j] = me ? nxt : cur;
    }
    const uint32_t last = key[NPL - 1], jsh = jw >> 4;
    key[NPL - 1] = me ? 0u : last;
    jw = me ? jsh : jw;
  }
  const uint32_t nk = (uint32_t)__shfl_down((int)mykey, 1, 64);
  const float la = __uint_as_float((mykey & 0x80000000u) ? (mykey ^ 0x80000000u) : ~mykey);
  const float lb = __uint_as_float((nk & 0x80000000u) ? (nk ^ 0x80000000u) : ~nk);
  const float lmax = __shfl(la, 0, 64);
  // (a marked token: either logit's dot product can be an ulp off the reference's float, see step 3; |dot| <= |logit| + |bias|)
  const float ulp2 = (nc[t] & RC_NC_ULP) ? 0x1p-22f * (fmaxf(fabsf(la), fabsf(lb)) + bias_max) : 0.f;
  const bool good = lane >= k || (mykey != 0u && nk != 0u && la - lb > 1e-6f + ulp2 && lmax - lb < 70.f);  // false for NaNs
  if (!__all(good)) {
    if (lane == 0) fb_list[atomicAdd(&counters[0], 1)] = t;
    return;
  }
  // softmax terms of every expert (the non-candidates' are approximate: they only enter the normaliser)
  const double mx = (double)lmax;
  double s = 0.0;
#pragma unroll
  for (int j = 0; j < NPL; j++) s += (double)(NPL * lane + j < E ? (float)exp((double)v[j] - mx) : 0.f);
  const double se = wave_dsum_dpp(s);
  const float sc = lane < k ? (float)((double)(float)exp((double)la - mx) / se) : 0.f;
  double wsum = 0.0;
  for (int r = 0; r < k; r++) wsum += (double)__shfl(sc, r, 64);  // selection order, as the reference's loop
  if (lane < k) {
    ids[(size_t)t * id_stride + lane] = myid;
    ws[(size_t)t * id_stride + lane] = (float)((double)sc / wsum);
  }
}

// ---- 5. listed tokens: every logit as an fp64 chain = k_router_exact_pairs<., true> above, unless the dense kernel takes over ----
// exact softmax / top-k of the listed tokens (of every token when the dense kernel ran)
template <int NPL>
__global__ void __launch_bounds__(256) k_router_topk_listed(const float* __restrict__ logits, int* __restrict__ ids,
                                                            float* __restrict__ ws, int P, int E, int k, int id_stride,
                                                            const int* __restrict__ fb_list,
                                                            const int* __restrict__ counters, int dense_above) {
  __shared__ float pbuf[4][64 * NPL];
  const int nl = counters[0];
  if (nl == 0) return;
  const int wv = threadIdx.x >> 6;
  const int w = blockIdx.x * 4 + wv;
  int tok;
  if (nl > dense_above) {
    if (w >= P) return;
    tok = w;
  } else {
    if (w >= nl) return;
    tok = fb_list[w];
  }
  topk_wave<NPL>(logits + (size_t)tok * E, ids + (size_t)tok * id_stride, ws + (size_t)tok * id_stride, E, k, pbuf[wv]);
}

}  // namespace

bool moe_router_cand_supported(const moe_wview* W, const moe_wview* Wx, int P, int k) {
  const int E = (int)W->rows, d = (int)W->cols;
  if (P < 1 || d % RA_K || d < RA_K || E > 512 || k + 1 > RC_SLOTS - 1 || k >= E) return false;
  if (Wx && (Wx->dtype == MOE_DT_BF16) != (W->dtype == MOE_DT_BF16)) return false;
  return moe_aligned(W->data, 16) && (!Wx || moe_aligned(Wx->data, 16));
}

static size_t rc_epad(int experts) { return ((size_t)experts + R2_BE - 1) / R2_BE * R2_BE; }
size_t moe_router_cand_scratch_bytes(int max_tokens, int experts, int d) {
  // counters [16], pairs [T][32] u32, nc [T], fb_list [T], xnorm [T], wnorm [E], the router matrix as f16 (rows padded)
  return (size_t)max_tokens * (RC_SLOTS * 4 + 4 + 4 + 4) + rc_epad(experts) * 4 + 64 + 256 + 256 + rc_epad(experts) * (size_t)d * 2;
}

// Internal: ids / ws (and the shared-expert gate logit, the per-token mean square of x) of a batch; `logits` ends
// up holding exact values for each token's candidates and approximate ones elsewhere.
int moe_router_batch_cand(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x, int P,
                          float* logits, float* out_x, float* out_xms, int* ids, float* ws, int k, int id_stride,
                          void* scratch, hipStream_t st, float bias_max) {
  const int E = (int)W->rows, d = (int)W->cols;
  if (!moe_router_cand_supported(W, Wx, P, k) || !moe_aligned(x, 16)) return MOE_E_UNSUPPORTED;
  uint8_t* sp = (uint8_t*)scratch;
  int* counters = (int*)sp; sp += 64;
  uint32_t* pairs = (uint32_t*)sp; sp += (size_t)P * RC_SLOTS * 4;
  int* nc = (int*)sp; sp += (size_t)P * 4;
  int* fb_list = (int*)sp; sp += (size_t)P * 4;
  float* xnorm = (float*)sp; sp += (size_t)P * 4;
  float* wnorm = (float*)sp; sp += rc_epad(E) * 4;
  __half* W16 = (__half*)(((uintptr_t)sp + 255) & ~(uintptr_t)255);
  const bool bf = W->dtype == MOE_DT_BF16;
  const int ncol = (E + RA_BE - 1) / RA_BE, ntt = (P + RA_BT - 1) / RA_BT;
  const unsigned grid_a = (unsigned)(((ntt + 7) / 8) * 8 * ncol);
  // 1.002: second-order terms; 1.01: the f32 norms' own rounding
  const float eps = (0x1p-10f + (float)RA_CHUNK * 0x1p-22f + (float)(d / RA_CHUNK + 1) * 0x1p-23f) * 1.002f * 1.01f;
  const float dterm = 0x1p-25f * 1.01f * sqrtf((float)d);
  const int dense_above = P / 16;
  const void* wx = Wx ? Wx->data : nullptr;
  const unsigned gtok = (unsigned)((P + 3) / 4), gtok16 = (unsigned)((P + 15) / 16);
  if (d % RA_CHUNK == 0) {
    // the router matrix as f16 once per call (a few microseconds), then the approximate logits with a token tile's
    // activations read and converted once
    const int Epad = (int)rc_epad(E);
    if (bf) k_router_w16<true><<<(Epad + 3) / 4, 256, 0, st>>>(W->data, E, Epad, d, W16, wnorm, counters);
    else k_router_w16<false><<<(Epad + 3) / 4, 256, 0, st>>>(W->data, E, Epad, d, W16, wnorm, counters);
    MOE_LAUNCH_CHECK();
    static moe_dev_once attr_once;
    int dev_now;
    if (moe_dev_pending(attr_once, &dev_now)) {
      MOE_HIP(hipFuncSetAttribute((const void*)k_router_approx2, hipFuncAttributeMaxDynamicSharedMemorySize, R2_SMEM));
      moe_dev_done(attr_once, dev_now);
    }
    const dim3 g2((unsigned)((P + R2_BT - 1) / R2_BT), (unsigned)(Epad / R2_BE));
    k_router_approx2<<<g2, 512, R2_SMEM, st>>>(W16, bias, x, P, E, d, logits, xnorm, out_xms);
  } else if (bf) {
    k_router_approx<true><<<grid_a, 256, 0, st>>>(W->data, bias, x, P, E, d, logits, wnorm, xnorm, out_xms, counters, ncol, ntt);
  } else {
    k_router_approx<false><<<grid_a, 256, 0, st>>>(W->data, bias, x, P, E, d, logits, wnorm, xnorm, out_xms, counters, ncol, ntt);
  }
  MOE_LAUNCH_CHECK();
  k_router_cand<8><<<gtok16, 1024, 0, st>>>(logits, wnorm, xnorm, P, E, k, eps, dterm, pairs, nc, fb_list, counters,
                                         wx ? 1 : 0);
  MOE_LAUNCH_CHECK();
  // at most 32 rows per token (31 candidates + the gate row): a wave per token, eight rows a pass
  if (bf) k_router_pairs_token<true><<<gtok, 256, 0, st>>>(W->data, bias, wx, x, P, E, d, pairs, logits, out_x, wnorm, xnorm, nc, wx ? 1 : 0);
  else k_router_pairs_token<false><<<gtok, 256, 0, st>>>(W->data, bias, wx, x, P, E, d, pairs, logits, out_x, wnorm, xnorm, nc, wx ? 1 : 0);
  MOE_LAUNCH_CHECK();
  k_router_topk_mixed<8><<<gtok, 256, 0, st>>>(logits, ids, ws, P, E, k, id_stride, nc, fb_list, counters, bias_max);
  MOE_LAUNCH_CHECK();
  // the exact redo of the listed tokens: three launches that return at once when nothing is listed
  // (sized for the most tokens the listed path takes, dense_above of them; surplus blocks return at once)
  const int wpt = (E + 63) / 64;  // a wave per token and 64 experts
  const unsigned glist = (unsigned)((dense_above > 0 ? dense_above : 1) * wpt);
  if (bf) k_router_exact_pairs<true><<<glist, 64, 0, st>>>(W->data, bias, x, E, d, counters, logits, fb_list, dense_above, wpt);
  else k_router_exact_pairs<false><<<glist, 64, 0, st>>>(W->data, bias, x, E, d, counters, logits, fb_list, dense_above, wpt);
  MOE_LAUNCH_CHECK();
  int rc = moe_router_logits_seq_if(W, bias, nullptr, x, P, logits, nullptr, nullptr, counters, dense_above, st);
  if (rc) return rc;
  k_router_topk_listed<8><<<gtok, 256, 0, st>>>(logits, ids, ws, P, E, k, id_stride, fb_list, counters, dense_above);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}
