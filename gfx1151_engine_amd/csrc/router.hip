// Router: logits with the CPU path's fp64 accumulation, fp64 softmax, top-k, renormalised weights.
// (reference: src/ref.cpp:68-77,565-594; src/gpu/parts/20_kernels_gemv.inc:1433-1562)
#include "common.h"
#include "hv2.h"
#include "internal.h"
#include "qvec.h"
#include "topk.h"

namespace {

template <bool BF16>
__device__ __forceinline__ float load_w(const void* W, uint64_t i) {
  if (BF16) return bf16_bits_to_f32(((const uint16_t*)W)[i]);
  return ((const float*)W)[i];
}

// ---- sequential order: bit-identical to `acc += (double)w*x` for c = 0..d-1 ----
// The f32*f32 product is exact in fp64, so a chain of fp64 FMAs over c = 0..d-1 equals the
// reference's multiply-then-add.  v_mfma_f64_16x16x4_f64 is such a chain: it adds its four k
// slices to the accumulator one after the other, each with a single FMA rounding (lane group
// l/16 supplies slice k; checked bit for bit against host fma chains over 3072-long sums with
// heavy cancellation), so successive MFMAs over ascending c reproduce the CPU sum exactly while
// the fp64 work runs on the matrix pipe.
// Block = BT tokens x 128 weight rows, 4 waves as 2 x 2, wave = BT/2 tokens x 64 rows.  Operands
// are staged in LDS as f32 (k permuted so that one 16-byte read feeds four MFMAs) and widened in
// registers; the next K slab is fetched into registers while the current one is consumed.
// D layout: value r of lane l is token 4r + l/16, weight row l%16 of the 16 x 16 tile.
// The shared-expert gate vector (Wx), if given, is one more plain FMA chain per token in the first
// column block: its logit goes to out_x[t].  Block ids are dealt so that the column blocks of one
// token tile run on the same XCD (ids that differ by 8) and share its L2 copy of the activations.
typedef double double4v __attribute__((ext_vector_type(4)));
constexpr int RS_E = 128, RS_K = 32, RS_PITCH = 36;
template <bool BF16, int BT>
__global__ void __launch_bounds__(256, 2) k_router_logits_seq(const void* __restrict__ W,
                                                           const float* __restrict__ bias,
                                                           const void* __restrict__ Wx, bool wx_bf16,
                                                           const float* __restrict__ x, int P, int E,
                                                           int d, float* __restrict__ logits,
                                                           float* __restrict__ out_x,
                                                           float* __restrict__ out_xms, int ncol, int ntt,
                                                           const int* __restrict__ run_if_above, int run_thr) {
  // (a launch that is only needed when many tokens were listed for an exact redo returns at once otherwise)
  if (run_if_above && *run_if_above <= run_thr) return;
  constexpr int MT = BT / 32;                 // 16-token MFMA tiles per wave
  constexpr int XL = (BT * RS_K / 4) / 256;   // float4 loads per thread and slab (activations)
  constexpr int WL = (RS_E * RS_K / 4) / 256; // (weights)
  __shared__ __attribute__((aligned(16))) float Xs[BT][RS_PITCH];
  __shared__ __attribute__((aligned(16))) float Ws[RS_E][RS_PITCH];
  __shared__ float Wxs[RS_K];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int li = lane & 15, lg = lane >> 4, wm = wv >> 1, wn = wv & 1;
  const int b = blockIdx.x, xcd = b & 7, q = b >> 3;
  const int col = q % ncol, tt = (q / ncol) * 8 + xcd;
  if (tt >= ntt) return;
  const int e0 = col * RS_E, t0 = tt * BT;
  const bool extra = Wx != nullptr && col == 0;
  const bool want_ms = out_xms != nullptr && col == 0;
  const bool vec = (d % 4 == 0);

  auto fetch_x = [&](int c0, float4* v) {
#pragma unroll
    for (int it = 0; it < XL; it++) {
      const int i = tid + it * 256, r = i >> 3, cc = c0 + (i & 7) * 4;
      const int t = t0 + r;
      float4 f = {0.f, 0.f, 0.f, 0.f};
      if (t < P) {
        const float* src = x + (size_t)t * d + cc;
        if (vec && cc + 3 < d) f = *(const float4*)src;
        else {
          if (cc < d) f.x = src[0];
          if (cc + 1 < d) f.y = src[1];
          if (cc + 2 < d) f.z = src[2];
          if (cc + 3 < d) f.w = src[3];
        }
      }
      v[it] = f;
    }
  };
  auto fetch_w = [&](int c0, float4* v) {
#pragma unroll
    for (int it = 0; it < WL; it++) {
      const int i = tid + it * 256, r = i >> 3, cc = c0 + (i & 7) * 4;
      const int e = e0 + r;
      float4 f = {0.f, 0.f, 0.f, 0.f};
      if (e < E) {
        const uint64_t o = (uint64_t)e * d + cc;
        if (vec && cc + 3 < d) {
          if (BF16) {
            const uint2 u = *(const uint2*)((const uint16_t*)W + o);
            f.x = __uint_as_float(u.x << 16); f.y = __uint_as_float(u.x & 0xffff0000u);
            f.z = __uint_as_float(u.y << 16); f.w = __uint_as_float(u.y & 0xffff0000u);
          } else {
            f = *(const float4*)((const float*)W + o);
          }
        } else {
          if (cc < d) f.x = load_w<BF16>(W, o);
          if (cc + 1 < d) f.y = load_w<BF16>(W, o + 1);
          if (cc + 2 < d) f.z = load_w<BF16>(W, o + 2);
          if (cc + 3 < d) f.w = load_w<BF16>(W, o + 3);
        }
      }
      v[it] = f;
    }
  };
  auto fetch_wx = [&](int c0) -> float {
    const int cc = c0 + tid;
    if (!extra || tid >= RS_K || cc >= d) return 0.f;
    return wx_bf16 ? bf16_bits_to_f32(((const uint16_t*)Wx)[cc]) : ((const float*)Wx)[cc];
  };
  // slab element k (0..31) of a row sits at [ (k & 3) * 8 + (k >> 2) ]: lane group g reads its
  // slices k = 4*kk + g for kk = 0..7 as two float4
  auto stage = [&](float (*dst)[RS_PITCH], const float4* v, int n) {
#pragma unroll
    for (int it = 0; it < n; it++) {
      const int i = tid + it * 256, r = i >> 3, m = i & 7;
      dst[r][m] = v[it].x; dst[r][8 + m] = v[it].y; dst[r][16 + m] = v[it].z; dst[r][24 + m] = v[it].w;
    }
  };

  double4v acc[MT][4];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = double4v{0.0, 0.0, 0.0, 0.0};
  double accx = 0.0;
  float accms = 0.f;
  const bool do_x = extra && tid < BT;    // this thread also carries token t0 + tid of the gate row
  const bool do_ms = want_ms && tid < BT;  // ... and that token's sum of squares

  float4 xr[XL], wr[WL];
  float wxr;
  fetch_x(0, xr);
  fetch_w(0, wr);
  wxr = fetch_wx(0);
  for (int c0 = 0; c0 < d; c0 += RS_K) {
    moe_lds_barrier();  // everybody is done reading the previous slab (LDS-only barriers: the next slab's loads stay in flight)
    stage(Xs, xr, XL);
    stage(Ws, wr, WL);
    if (tid < RS_K) Wxs[tid] = wxr;
    moe_lds_barrier();
    if (c0 + RS_K < d) {
      fetch_x(c0 + RS_K, xr);
      fetch_w(c0 + RS_K, wr);
      wxr = fetch_wx(c0 + RS_K);
    }
#pragma unroll
    for (int half = 0; half < 2; half++) {
      float4 xa[MT], wb[4];
#pragma unroll
      for (int mt = 0; mt < MT; mt++) xa[mt] = *(const float4*)&Xs[wm * (BT / 2) + 16 * mt + li][lg * 8 + 4 * half];
#pragma unroll
      for (int nt = 0; nt < 4; nt++) wb[nt] = *(const float4*)&Ws[wn * 64 + 16 * nt + li][lg * 8 + 4 * half];
#pragma unroll
      for (int kk = 0; kk < 4; kk++) {
        double a[MT], bq[4];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) a[mt] = (double)(kk == 0 ? xa[mt].x : kk == 1 ? xa[mt].y : kk == 2 ? xa[mt].z : xa[mt].w);
#pragma unroll
        for (int nt = 0; nt < 4; nt++) bq[nt] = (double)(kk == 0 ? wb[nt].x : kk == 1 ? wb[nt].y : kk == 2 ? wb[nt].z : wb[nt].w);
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
          for (int nt = 0; nt < 4; nt++)
            acc[mt][nt] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[mt], bq[nt], acc[mt][nt], 0, 0, 0);
      }
    }
    if (do_x) {
#pragma unroll 8
      for (int k = 0; k < RS_K; k++) accx = fma((double)Wxs[k], (double)Xs[tid][(k & 3) * 8 + (k >> 2)], accx);
    }
    if (do_ms) {
#pragma unroll 8
      for (int k = 0; k < RS_K; k++) accms = fmaf(Xs[tid][k], Xs[tid][k], accms);
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int t = t0 + wm * (BT / 2) + 16 * mt + 4 * r + lg;
      if (t >= P) continue;
#pragma unroll
      for (int nt = 0; nt < 4; nt++) {
        const int e = e0 + wn * 64 + 16 * nt + li;
        if (e >= E) continue;
        float v = (float)acc[mt][nt][r];
        if (bias) v += bias[e];
        logits[(size_t)t * E + e] = v;
      }
    }
  }
  if (do_x && t0 + tid < P) out_x[t0 + tid] = (float)accx;
  if (do_ms && t0 + tid < P) out_xms[t0 + tid] = accms / (float)d;
}

// The blocks past the rows of the small-batch router launches: the digit planes of x for the integer-dot decode
// kernels (a thread per 32-element group) and, for hgn v2 layers, the planes of rot_in(x, pre) = H(pre . x) / sqrt(128)
// (a thread per 8 elements, 16 lanes per 128-block) -- work that rides along instead of costing a launch.
// q = index among these blocks, bs = block size.
__device__ __forceinline__ void router_plane_blocks(int q, int bs, int tid, const float* __restrict__ x, int P, int d,
                                                    uint32_t* __restrict__ planes, float2* __restrict__ meta,
                                                    bool planes_natural, const moe_rot_planes& R) {
  const int G = d / 32, gb = (G + bs - 1) / bs;
  const int nq = planes ? P * gb : 0;
  if (q < nq) {
    const int t = q / gb, g = (q % gb) * bs + tid;
    if (t < P && g < G) {
      if (planes_natural) qvec_group_from_f32(x, (uint64_t)d, G, t, g, planes, meta);  // Q4_K kernels
      else qvec4_group_from_f32(x, (uint64_t)d, G, t, g, planes, meta);                       // q4cp kernels
    }
    return;
  }
  if (!R.planes) return;
  q -= nq;
  const int per_row = d / 8, rb = (per_row + bs - 1) / bs;
  const int t = q / rb, c8 = (q % rb) * bs + tid;
  const bool live = t < P && c8 < per_row;  // (whole groups of 16 lanes: d % 128 == 0)
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] = 0.f;
  if (live) {
    const float4* xp = (const float4*)(x + (size_t)t * d + 8 * c8);
    const float4* pp = (const float4*)(R.pre + 8 * c8);
    const float4 a = xp[0], b = xp[1], e = pp[0], f = pp[1];
    v[0] = a.x * e.x; v[1] = a.y * e.y; v[2] = a.z * e.z; v[3] = a.w * e.w;
    v[4] = b.x * f.x; v[5] = b.y * f.y; v[6] = b.z * f.z; v[7] = b.w * f.w;
  }
  moe_fwht128_r8(v, tid);
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] *= MOE_RS128;
  moe_st8_planes(v, tid, R.planes, R.meta, (size_t)t * G + (c8 >> 2), live);
}

// ---- lane-parallel order for small P: one wave per weight row (four rows per block), lanes stride
// the columns, four independent fp64 chains per lane and token, fixed combination order.  The fp64
// sum differs from the sequential one only in its last bits, so the f32 logit differs with
// probability ~1e-8 per value.  Row E (if Wx given) is the shared-expert gate vector: out_x[t] =
// its logit.  Blocks past the rows (if planes given) turn x into the digit planes of the
// integer-dot decode kernels, so that work rides along instead of costing a launch.
// If `counter` is given, the block that finishes last (an atomic ticket per row block; the logits
// cross as device-scope stores that have completed before the ticket, and device-scope loads after
// it) runs the softmax / top-k of every token as well and re-arms the counter: one launch instead
// of two on the latency-bound decode path.
template <bool BF16, int TT, int NPL>
__global__ void __launch_bounds__(256) k_router_small(const void* __restrict__ W,
                                                      const float* __restrict__ bias,
                                                      const void* __restrict__ Wx, bool wx_bf16,
                                                      const float* __restrict__ x, int P, int E, int d,
                                                      float* __restrict__ logits, float* __restrict__ out_x,
                                                      int nrows, uint32_t* __restrict__ planes,
                                                      float2* __restrict__ meta, bool planes_natural,
                                                      unsigned* counter, int* __restrict__ ids,
                                                      float* __restrict__ ws, int k, int id_stride, moe_rot_planes rot,
                                                      float* __restrict__ tol_out, float tol_scale) {
  __shared__ int s_last;
  // the wave index as a scalar: row, weight type and base address are then wave-uniform values
  // and the bf16 / f32 choice below is a scalar branch, not a divergent one around every load
  const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int rpb = blockDim.x >> 6;  // rows per block: one per wave
  const int nrb = (nrows + rpb - 1) / rpb;
  if ((int)blockIdx.x >= nrb) {
    router_plane_blocks((int)blockIdx.x - nrb, (int)blockDim.x, (int)threadIdx.x, x, P, d, planes, meta, planes_natural, rot);
    return;
  }
  const int row = blockIdx.x * rpb + wv;
  if (row < nrows) {
    const bool extra = row == E;
    const void* Wr = extra ? Wx : W;
    const uint64_t base = extra ? 0 : (uint64_t)row * d;
    const bool bf = extra ? wx_bf16 : BF16;
    // the wave of row 0 also takes |x|^2 of every token: the selection that follows needs a bound on how far these
    // sums (lanes, then a tree) can lie from the reference's sequential ones, tol_scale * |x|
    const bool norms = tol_out && row == 0;
    for (int t0 = 0; t0 < P; t0 += TT) {
      double acc[TT][4];
      float xs[TT];
#pragma unroll
      for (int i = 0; i < TT; i++) {
        xs[i] = 0.f;
#pragma unroll
        for (int q = 0; q < 4; q++) acc[i][q] = 0.0;
      }
#pragma unroll 12
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
            if (norms) xs[i] += xv.x * xv.x + xv.y * xv.y + xv.z * xv.z + xv.w * xv.w;
          }
        }
      }
      if (norms) {
#pragma unroll
        for (int i = 0; i < TT; i++) {
          const float n2 = wave_sum(xs[i]);
          if (lane == 0 && t0 + i < P) {
            float tl = tol_scale * sqrtf(n2) * 1.01f;
            tol_out[t0 + i] = tl >= 0.f ? tl : INFINITY;  // (NaN: nothing is certain)
          }
        }
      }
#pragma unroll
      for (int i = 0; i < TT; i++) {
        const double sum = wave_sum((acc[i][0] + acc[i][1]) + (acc[i][2] + acc[i][3]));
        if (lane == 0 && t0 + i < P) {
          float v = (float)sum;
          if (extra) out_x[t0 + i] = v;
          else {
            if (bias) v += bias[row];
            // device-scope store: written through to where every XCD's loads of that scope see it
            __hip_atomic_store(&logits[(size_t)(t0 + i) * E + row], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      }
    }
  }
  if (!counter) return;
  // Hand-over to the block that draws the last ticket (possibly on another XCD).  The logits above are
  // device-scope atomic stores (written through to the device's coherence point, not left in this XCD's
  // L2), and every storing wave waits here until the memory system has acknowledged all of them
  // (vmcnt = 0) before it reaches the barrier; only then does thread 0 take the ticket.  The reader
  // (topk_block<.., true>) uses device-scope atomic loads issued after its own ticket came back, which
  // read at that same point.  No cache-wide write-back or invalidate is involved on either side.
  __builtin_amdgcn_s_waitcnt(0);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned ticket = atomicAdd(counter, 1u);
    s_last = ticket == (unsigned)nrb - 1u;
  }
  __syncthreads();
  if (!s_last) return;
  for (int t = 0; t < P; t++)
    topk_block<NPL, true>(logits + (size_t)t * E, ids + (size_t)t * id_stride, ws + (size_t)t * id_stride, E, k);
  if (threadIdx.x == 0) *counter = 0u;  // re-armed for the next launch on the stream
}

// ---- lane-parallel order for 5..32 tokens: four weight rows per block (a wave each); the tokens'
// activations are widened to fp64 ONCE per block and 128-column slab (in LDS) instead of once per
// row, and every weight is read once for all tokens.  Lane l owns columns 2l, 2l+1 of each slab:
// two fp64 chains per token, combined in a fixed order, then the wave sum.  Same accuracy
// statement as k_router_small.  Blocks past the rows build the digit planes of x.
constexpr int RM_C = 128, RM_D = 4;
template <bool BF16, int PMAX>  // PMAX 8 / 16 / 24
__global__ void __launch_bounds__(256) k_router_mid(const void* __restrict__ W, const float* __restrict__ bias,
                                                    const void* __restrict__ Wx, bool wx_bf16,
                                                    const float* __restrict__ x, int P, int E, int d,
                                                    float* __restrict__ logits, float* __restrict__ out_x,
                                                    int nrows, uint32_t* __restrict__ planes,
                                                    float2* __restrict__ meta, bool planes_natural, moe_rot_planes rot) {
  __shared__ __attribute__((aligned(16))) double Xd[2][PMAX][RM_C];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int nrb = (nrows + 3) >> 2;
  if ((int)blockIdx.x >= nrb) {
    router_plane_blocks((int)blockIdx.x - nrb, 256, tid, x, P, d, planes, meta, planes_natural, rot);
    return;
  }
  // the wave's row as scalar values: the bf16 / f32 choice is then a scalar branch
  const int row = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(wv);
  // (without a gate vector row E is padding like every row past it: it must not take Wx, a null pointer then)
  const bool live = row < nrows, extra = Wx != nullptr && row == E;
  const void* Wr = extra ? Wx : W;
  const uint64_t base = (extra || !live) ? 0 : (uint64_t)row * d;  // rows past the matrix read row 0, never stored
  const bool bf = extra ? wx_bf16 : BF16;
  constexpr int XR = PMAX * RM_C / 256;  // staged activations per thread and slab
  // Register ring of RM_D slabs: slot j holds slab s with s % RM_D == j and is refilled for slab
  // s + RM_D as soon as slab s has gone to LDS, so every load has RM_D slab times to arrive
  // (one slab ahead left the loop waiting a full memory latency per 128 columns).
  // All loads are unconditional (clamped address, value times 0 or 1) and weights stay as raw
  // bits until they are used: a load under a divergent branch, or converted where it is issued,
  // makes the wave wait for every load in flight.  (d is even: c + 1 < d whenever c < d.)
  float xr[RM_D][XR];
  uint2 wr[RM_D];
  auto fetch = [&](int j, int c0) {
#pragma unroll
    for (int i = 0; i < XR; i++) {
      const int e = tid + 256 * i, t = e / RM_C, c = c0 + e % RM_C;
      const bool ok = t < P && c < d;
      xr[j][i] = x[ok ? (size_t)t * d + c : 0] * (ok ? 1.f : 0.f);
    }
    const int c = c0 + 2 * lane;
    const int cc = c < d ? c : 0;
    // two 32-bit loads in either format (bf16: the same word twice), so no branch surrounds them
    const uint8_t* p0 = (const uint8_t*)Wr + (base + cc) * (bf ? 2 : 4);
    wr[j].x = *(const uint32_t*)p0;
    wr[j].y = *(const uint32_t*)(p0 + (bf ? 0 : 4));
  };
  auto weights = [&](int j, int c0, double& w0, double& w1) {
    const float m = c0 + 2 * lane < d ? 1.f : 0.f;
    const float f0 = bf ? __uint_as_float(wr[j].x << 16) : __uint_as_float(wr[j].x);
    const float f1 = bf ? __uint_as_float(wr[j].x & 0xffff0000u) : __uint_as_float(wr[j].y);
    w0 = (double)(f0 * m);
    w1 = (double)(f1 * m);
  };
  double acc[PMAX][2];
#pragma unroll
  for (int t = 0; t < PMAX; t++) acc[t][0] = acc[t][1] = 0.0;
#pragma unroll
  for (int j = 0; j < RM_D; j++) fetch(j, j * RM_C);
  int buf = 0;
  for (int cg = 0; cg < d; cg += RM_D * RM_C) {
#pragma unroll
    for (int j = 0; j < RM_D; j++) {
      const int c0 = cg + j * RM_C;
      if (c0 < d) {  // block-uniform
        // Xd[buf] was last read two slabs ago; every wave has passed the barrier of the slab in
        // between, so it is free
#pragma unroll
        for (int i = 0; i < XR; i++) {
          const int e = tid + 256 * i;
          Xd[buf][e / RM_C][e % RM_C] = (double)xr[j][i];
        }
        double w0, w1;
        weights(j, c0, w0, w1);
        fetch(j, c0 + RM_D * RM_C);  // slabs past d load column 0 and count as zeros
        moe_lds_barrier();  // (LDS only: the ring's loads stay in flight across it)
        // rows past P hold zeros: no predicate, so the LDS reads of a slab go out back to back
#pragma unroll
        for (int t = 0; t < PMAX; t++) {
          const double2 xv = *(const double2*)&Xd[buf][t][2 * lane];
          acc[t][0] = fma(w0, xv.x, acc[t][0]);
          acc[t][1] = fma(w1, xv.y, acc[t][1]);
        }
        buf ^= 1;
      }
    }
  }
#pragma unroll
  for (int t = 0; t < PMAX; t++) {
    if (t < P) {
      const double sum = wave_sum(acc[t][0] + acc[t][1]);
      if (lane == 0 && live) {
        float v = (float)sum;
        if (extra) out_x[t] = v;
        else {
          if (bias) v += bias[row];
          logits[(size_t)t * E + row] = v;
        }
      }
    }
  }
}

// ---- softmax + top-k, one wave per token (E <= 64*NPL): topk_wave in topk.h ----
template <int NPL>
__global__ void __launch_bounds__(256) k_router_topk(const float* __restrict__ logits,
                                                     int* __restrict__ ids, float* __restrict__ ws,
                                                     int P, int E, int k, int id_stride) {
  __shared__ float pbuf[4][64 * NPL];
  const int wv = threadIdx.x >> 6;
  const int tok = blockIdx.x * 4 + wv;
  if (tok >= P) return;
  topk_wave<NPL>(logits + (size_t)tok * E, ids + (size_t)tok * id_stride, ws + (size_t)tok * id_stride, E, k, pbuf[wv]);
}

template <int NPL>
__global__ void __launch_bounds__(256) k_router_topk_block(const float* __restrict__ logits, int* __restrict__ ids,
                                                           float* __restrict__ ws, int E, int k, int id_stride, moe_rfix RF) {
  __shared__ int sel_ids[64];
  __shared__ float sel_ws[64];
  const int t = blockIdx.x;
  if (!RF.W) {
    topk_block<NPL, false>(logits + (size_t)t * E, ids + (size_t)t * id_stride, ws + (size_t)t * id_stride, E, k);
    return;
  }
  select_certain<NPL, 256>(logits + (size_t)t * E, RF, t, sel_ids, sel_ws, E, k, true);
  __syncthreads();
  if ((int)threadIdx.x < k) {
    ids[(size_t)t * id_stride + threadIdx.x] = sel_ids[threadIdx.x];
    ws[(size_t)t * id_stride + threadIdx.x] = sel_ws[threadIdx.x];
  }
}

// |row|_2 of every row, the maximum as the bits of a non-negative float
__global__ void __launch_bounds__(256) k_row_norm_max(const void* __restrict__ W, int bf16, int E, int d, unsigned* __restrict__ out) {
  const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= E) return;
  float a = 0.f;
  for (int c = lane; c < d; c += 64) {
    const float w = bf16 ? bf16_bits_to_f32(((const uint16_t*)W)[(size_t)row * d + c]) : ((const float*)W)[(size_t)row * d + c];
    a += w * w;
  }
  a = wave_sum(a);
  if (lane == 0) atomicMax(out, __float_as_uint(a >= 0.f ? sqrtf(a) : INFINITY));
}

// Launch of the sequential-order kernel: 128-token tiles when there are enough of them to fill the
// chip, 64-token tiles otherwise.
void launch_seq(const void* W, bool bf, const float* bias, const void* wx, bool xbf, const float* x, int P,
                int E, int d, float* logits, float* out_x, float* out_xms, hipStream_t st,
                const int* run_if_above = nullptr, int run_thr = 0) {
  const int ncol = (E + RS_E - 1) / RS_E;
  const bool big = (int64_t)((P + 127) / 128) * ncol >= 512;
  const int bt = big ? 128 : 64;
  const int ntt = (P + bt - 1) / bt;
  const unsigned grid = (unsigned)(((ntt + 7) / 8) * 8 * ncol);
#define RS_GO(BF, BT) k_router_logits_seq<BF, BT><<<grid, 256, 0, st>>>(W, bias, wx, xbf, x, P, E, d, logits, out_x, out_xms, ncol, ntt, run_if_above, run_thr)
  if (bf) { if (big) RS_GO(true, 128); else RS_GO(true, 64); }
  else { if (big) RS_GO(false, 128); else RS_GO(false, 64); }
#undef RS_GO
}


// ---- 5..32 tokens on the f64 matrix pipe: a block = 16 weight rows x all tokens x one column split,
// its eight waves each take one eighth of the block's columns and the partial 16 x 16 tiles are added in
// wave order (fixed, so the result does not depend on timing; same accuracy statement as k_router_small).
// v_mfma_f64_16x16x4_f64: lane l supplies A[row l%16][k l/16] and B[k l/16][token l%16]; a 16-byte load
// per lane (4 consecutive columns 4*(l/16)..+3 of its row / token) therefore feeds four MFMAs.
// Every weight is read once, activations come from L2; loads run through a register ring of
// RD 16-column steps.  Needs d % (128 * KS) == 0.  Blocks past the rows build the digit planes of x.
// KS > 1 (needs gpart and tickets): the columns are split over KS blocks per row group as well, so that
// 16 rows x d columns, one block's work with KS = 1 and the whole time of the launch, become KS blocks on KS
// CUs.  Each block leaves its fp64 partial tile in gpart and takes a ticket of its row group; the block that
// draws the last one adds the KS partial tiles in split order (fixed again) and writes the logits.  Partial
// tiles go out and come back as device-scope accesses, the ticket counters rest at 0 between launches.
template <bool BF16, int NTT, int RD>  // NTT = token tiles of 16 (1 or 2)
__global__ void __launch_bounds__(512, 2) k_router_mfma(const void* __restrict__ W, const float* __restrict__ bias,
                                                        const void* __restrict__ Wx, bool wx_bf16,
                                                        const float* __restrict__ x, int P, int E, int d,
                                                        float* __restrict__ logits, float* __restrict__ out_x,
                                                        int nrows, uint32_t* __restrict__ planes,
                                                        float2* __restrict__ meta, bool planes_natural, int KS,
                                                        double* gpart, unsigned* tickets, moe_rot_planes rot) {
  __shared__ double part[8][NTT][64][4];
  __shared__ int s_last;
  const int tid = threadIdx.x, lane = tid & 63, wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nrt = (nrows + 15) >> 4;
  if ((int)blockIdx.x >= nrt * KS) {
    router_plane_blocks((int)blockIdx.x - nrt * KS, 512, tid, x, P, d, planes, meta, planes_natural, rot);
    return;
  }
  const int rg = (int)blockIdx.x % nrt, ks = (int)blockIdx.x / nrt;  // row group, column split
  const int li = lane & 15, lg = lane >> 4;
  const int row = rg * 16 + li;
  const bool rlive = row < nrows, extra = Wx != nullptr && row == E;
  // per-lane weight row (rows past the end read row 0 and are never stored); all loads unconditional
  const bool wbf = extra ? wx_bf16 : BF16;
  const uint8_t* wrow = extra ? (const uint8_t*)Wx : (const uint8_t*)W + (rlive ? (uint64_t)row : 0) * d * (BF16 ? 2 : 4);
  const float* xrow[NTT];
  float xm[NTT];
#pragma unroll
  for (int tt = 0; tt < NTT; tt++) {
    const int t = 16 * tt + li;
    xrow[tt] = x + (size_t)(t < P ? t : 0) * d;
    xm[tt] = t < P ? 1.f : 0.f;
  }
  const int kper = d / (8 * KS), k0 = (ks * 8 + wv) * kper + 4 * lg;  // this lane's first column
  const int nit = kper / 16;
  uint4 wr[RD];
  float4 xr[RD][NTT];
  auto fetch = [&](int j, int it) {
    const int c = k0 + 16 * (it < nit ? it : nit - 1);  // past the end: a repeat that is never used
    // 16 bytes in either format (bf16: 8 bytes twice), so no branch surrounds the load
    const uint8_t* p = wrow + (size_t)c * (wbf ? 2 : 4);
    const uint2 lo = *(const uint2*)p, hi = *(const uint2*)(p + (wbf ? 0 : 8));
    wr[j] = make_uint4(lo.x, lo.y, hi.x, hi.y);
#pragma unroll
    for (int tt = 0; tt < NTT; tt++) xr[j][tt] = *(const float4*)(xrow[tt] + c);
  };
  double4v acc[NTT];
#pragma unroll
  for (int tt = 0; tt < NTT; tt++) acc[tt] = double4v{0.0, 0.0, 0.0, 0.0};
#pragma unroll
  for (int j = 0; j < RD; j++) fetch(j, j);
  for (int ib = 0; ib < nit; ib += RD) {
#pragma unroll
    for (int j = 0; j < RD; j++) {
      if (ib + j < nit) {  // block-uniform
        float w[4];
        if (wbf) {
          w[0] = __uint_as_float(wr[j].x << 16); w[1] = __uint_as_float(wr[j].x & 0xffff0000u);
          w[2] = __uint_as_float(wr[j].y << 16); w[3] = __uint_as_float(wr[j].y & 0xffff0000u);
        } else {
          w[0] = __uint_as_float(wr[j].x); w[1] = __uint_as_float(wr[j].y);
          w[2] = __uint_as_float(wr[j].z); w[3] = __uint_as_float(wr[j].w);
        }
        float4 xv[NTT];
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) xv[tt] = xr[j][tt];
        fetch(j, ib + j + RD);
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const double a = (double)w[q];
#pragma unroll
          for (int tt = 0; tt < NTT; tt++) {
            const float xq = q == 0 ? xv[tt].x : q == 1 ? xv[tt].y : q == 2 ? xv[tt].z : xv[tt].w;
            acc[tt] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, (double)(xq * xm[tt]), acc[tt], 0, 0, 0);
          }
        }
      }
    }
  }
#pragma unroll
  for (int tt = 0; tt < NTT; tt++)
#pragma unroll
    for (int r = 0; r < 4; r++) part[wv][tt][lane][r] = acc[tt][r];
  __syncthreads();
  // D value r of lane l = [row 4r + l/16][token l%16]; one thread per (tile, lane, r) adds the eight partials
  auto emit = [&](int i, double sum) {
    const int tt = i >> 8, l = (i >> 2) & 63, r = i & 3;
    const int orow = rg * 16 + 4 * r + (l >> 4), t = 16 * tt + (l & 15);
    if (orow < nrows && t < P) {
      float v = (float)sum;
      if (orow == E) out_x[t] = v;
      else {
        if (bias) v += bias[orow];
        logits[(size_t)t * E + orow] = v;
      }
    }
  };
  constexpr int NV = NTT * 256;
  for (int i = tid; i < NV; i += 512) {
    const int tt = i >> 8, l = (i >> 2) & 63, r = i & 3;
    double sum = part[0][tt][l][r];
#pragma unroll
    for (int w = 1; w < 8; w++) sum += part[w][tt][l][r];
    if (KS == 1) emit(i, sum);
    else __hip_atomic_store(&gpart[((size_t)ks * nrt + rg) * NV + i], sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (KS == 1) return;
  // Hand-over of the partial tiles to the block that draws the row group's last ticket (possibly on another
  // XCD): the tiles are device-scope atomic stores, every storing thread waits until all of its stores have
  // been acknowledged (vmcnt = 0) before the barrier, thread 0 takes the device-scope ticket after the
  // barrier, and the last block reads the tiles back with device-scope atomic loads issued after its own
  // ticket returned.  Both sides go to the device's coherence point; no cache-wide write-back / invalidate.
  __builtin_amdgcn_s_waitcnt(0);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (tid == 0) {
    const unsigned ticket = __hip_atomic_fetch_add(&tickets[rg], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = ticket == (unsigned)KS - 1u;
    if (s_last) __hip_atomic_store(&tickets[rg], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // re-armed
  }
  __syncthreads();
  if (!s_last) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  for (int i = tid; i < NV; i += 512) {
    double v[8];  // KS <= 8: all partials requested before the first is used
#pragma unroll
    for (int q = 0; q < 8; q++)
      v[q] = __hip_atomic_load(&gpart[((size_t)(q < KS ? q : 0) * nrt + rg) * NV + i], __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    double sum = v[0];
#pragma unroll
    for (int q = 1; q < 8; q++)
      if (q < KS) sum += v[q];
    emit(i, sum);
  }
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
    return moe_router_logits_small(W, bias, nullptr, x, P, logits, nullptr, nullptr, nullptr, false, nullptr, nullptr,
                                   nullptr, 0, 0, nullptr, moe_s(st), nullptr, nullptr);
  } else {
    launch_seq(W->data, bf, bias, nullptr, false, x, P, E, d, logits, nullptr, nullptr, moe_s(st));
  }
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// Internal: sequential-order logits for any P (also used for the one-row shared-expert gate).
int moe_router_logits_seq(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x, int P,
                          float* logits, float* out_x, float* out_xms, hipStream_t st) {
  const int E = (int)W->rows, d = (int)W->cols;
  const bool xbf = Wx && Wx->dtype == MOE_DT_BF16;
  const void* wx = Wx ? Wx->data : nullptr;
  launch_seq(W->data, W->dtype == MOE_DT_BF16, bias, wx, xbf, x, P, E, d, logits, out_x, out_xms, st);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// Internal: the same launch, doing its work only if *run_if_above > run_thr when it starts (device memory).
int moe_router_logits_seq_if(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x, int P,
                             float* logits, float* out_x, float* out_xms, const int* run_if_above, int run_thr,
                             hipStream_t st) {
  const int E = (int)W->rows, d = (int)W->cols;
  const bool xbf = Wx && Wx->dtype == MOE_DT_BF16;
  launch_seq(W->data, W->dtype == MOE_DT_BF16, bias, Wx ? Wx->data : nullptr, xbf, x, P, E, d, logits, out_x, out_xms, st,
             run_if_above, run_thr);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// Internal: small-P logits plus the shared-expert gate row (and, if planes != nullptr, the digit
// planes of x for the integer-dot decode kernels) in the same launch.  With a counter (device
// memory holding 0) and P <= 4 the launch also does the softmax / top-k: *fused_topk says so.
int moe_router_logits_small(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x,
                            int P, float* logits, float* out_x, uint32_t* planes, float2* meta,
                            bool planes_natural, unsigned* counter, int* ids, float* ws, int k, int id_stride, bool* fused_topk,
                            hipStream_t st, double* kpart, unsigned* ktickets, const moe_rot_planes* rotp,
                            float* tol_out, float tol_scale) {
  const int E = (int)W->rows, d = (int)W->cols;
  moe_rot_planes rot{nullptr, nullptr, nullptr};
  if (rotp) {  // hgn v2: the planes of rot_in(x, pre) in the same launch
    if (!rotp->pre || !rotp->planes || !rotp->meta || d % 128 || !moe_aligned(rotp->pre, 16) || !moe_aligned(x, 16)) return MOE_E_INVALID;
    rot = *rotp;
  }
  // The f64 matrix pipe kernel (d a multiple of 128, one weight format).  With the caller's scratch for
  // partial tiles the columns are split over up to eight blocks per 16 rows and it serves 5..32 tokens;
  // without it one block per 16 rows leaves most CUs idle (38 us at 32 tokens), which only beats
  // k_router_mid above 24 tokens.
  const bool one_fmt = !Wx || (Wx->dtype == MOE_DT_BF16) == (W->dtype == MOE_DT_BF16);
  int KS = 1;
  if (kpart && ktickets && one_fmt && P > 4 && E + 1 <= MOE_ROUTER_KSPLIT_ROWS)
    for (int s = 8; s > 1; s >>= 1)
      if (d % (128 * s) == 0) {
        KS = s;
        break;
      }
  const bool mfma_ok = (P > 24 || KS > 1) && d % 128 == 0 && one_fmt;
  if (P > 24 && !mfma_ok) {
    // more than 24 tokens per block cost the kernel its second wave per SIMD (accumulators):
    // two launches of at most 16 tokens read the router matrix twice (L2 / MALL) and are faster
    const int P0 = 16, G = d / 32;
    const size_t pdw = planes_natural ? QV_GROUP_DW : QV4_GROUP_DW;
    int rc = moe_router_logits_small(W, bias, Wx, x, P0, logits, out_x, planes, meta, planes_natural, nullptr, nullptr,
                                     nullptr, k, id_stride, nullptr, st, nullptr, nullptr, rotp);
    if (rc) return rc;
    if (fused_topk) *fused_topk = false;
    moe_rot_planes rot2 = rot;
    if (rotp) {
      rot2.planes += (size_t)P0 * G * QV4_GROUP_DW;
      rot2.meta += (size_t)P0 * G;
    }
    return moe_router_logits_small(W, bias, Wx, x + (size_t)P0 * d, P - P0, logits + (size_t)P0 * E,
                                   out_x ? out_x + P0 : nullptr, planes ? planes + (size_t)P0 * G * pdw : nullptr,
                                   meta ? meta + (size_t)P0 * G : nullptr, planes_natural, nullptr, nullptr, nullptr, k,
                                   id_stride, nullptr, st, nullptr, nullptr, rotp ? &rot2 : nullptr);
  }
  const bool bf = W->dtype == MOE_DT_BF16;
  const bool xbf = Wx && Wx->dtype == MOE_DT_BF16;
  const int nrows = E + (Wx ? 1 : 0);
  const bool fuse = counter && ids && ws && P <= 4 && E <= 1024;
  if (fused_topk) *fused_topk = fuse;
  unsigned* cn = fuse ? counter : nullptr;
  // one token, no top-k in this launch: two rows per block so that the rows cover every CU
  // (the fused top-k needs its 256 threads)
  const int bs = (P == 1 && !fuse && E <= 512) ? 128 : 256, rpb = bs / 64;
  const int qblocks = (planes ? P * ((d / 32 + bs - 1) / bs) : 0) + (rot.planes ? P * ((d / 8 + bs - 1) / bs) : 0);
  dim3 g((nrows + rpb - 1) / rpb + qblocks);
  const void* wx = Wx ? Wx->data : nullptr;
#define RSM_GO(BF, TT, NPL) k_router_small<BF, TT, NPL><<<g, bs, 0, st>>>(W->data, bias, wx, xbf, x, P, E, d, logits, out_x, nrows, planes, meta, planes_natural, cn, ids, ws, k, id_stride, rot, tol_out, tol_scale)
  if (P == 1 && E <= 512) {
    if (bf) RSM_GO(true, 1, 8); else RSM_GO(false, 1, 8);
  } else if (P <= 4) {
    if (E <= 512) { if (bf) RSM_GO(true, 4, 8); else RSM_GO(false, 4, 8); }
    else { if (bf) RSM_GO(true, 4, 16); else RSM_GO(false, 4, 16); }
  } else {
    if (mfma_ok) {
      // the f64 matrix pipe: 16 rows per block, columns split over KS blocks and their eight waves
      const int qb = (planes ? P * ((d / 32 + 511) / 512) : 0) + (rot.planes ? P * ((d / 8 + 511) / 512) : 0);
      dim3 gx((nrows + 15) / 16 * KS + qb);
#define RX_GO(BF, NTT, RD) k_router_mfma<BF, NTT, RD><<<gx, 512, 0, st>>>(W->data, bias, wx, xbf, x, P, E, d, logits, out_x, nrows, planes, meta, planes_natural, KS, kpart, ktickets, rot)
      const int nit = d / (8 * KS) / 16;  // ring steps a wave walks
      if (nit <= 3) {
        if (P <= 16) { if (bf) RX_GO(true, 1, 3); else RX_GO(false, 1, 3); }
        else { if (bf) RX_GO(true, 2, 3); else RX_GO(false, 2, 3); }
      } else {
        if (P <= 16) { if (bf) RX_GO(true, 1, 12); else RX_GO(false, 1, 12); }
        else { if (bf) RX_GO(true, 2, 12); else RX_GO(false, 2, 12); }
      }
#undef RX_GO
      MOE_LAUNCH_CHECK();
      return MOE_OK;
    }
#define RMD_GO(BF, PM) k_router_mid<BF, PM><<<g, 256, 0, st>>>(W->data, bias, wx, xbf, x, P, E, d, logits, out_x, nrows, planes, meta, planes_natural, rot)
    if (P <= 8) { if (bf) RMD_GO(true, 8); else RMD_GO(false, 8); }
    else if (P <= 16) { if (bf) RMD_GO(true, 16); else RMD_GO(false, 16); }
    else { if (bf) RMD_GO(true, 24); else RMD_GO(false, 24); }  // P <= 24 (larger batches were split above)
#undef RMD_GO
  }
#undef RSM_GO
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_router_topk_small(const float* logits, int* ids, float* ws, int P, int E, int k, int id_stride,
                                 const moe_rfix* rf, hipStream_t st) {
  const moe_rfix R = rf ? *rf : moe_rfix{};
  if (E <= 512) k_router_topk_block<8><<<P, 256, 0, st>>>(logits, ids, ws, E, k, id_stride, R);
  else k_router_topk_block<16><<<P, 256, 0, st>>>(logits, ids, ws, E, k, id_stride, R);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_router_row_norm_max(const moe_wview* W, float* scratch, float* out_host) {
  if (!W || !W->data || !scratch || !out_host) return MOE_E_INVALID;
  MOE_HIP(hipMemset(scratch, 0, 4));
  k_row_norm_max<<<(unsigned)((W->rows + 3) / 4), 256, 0, nullptr>>>(W->data, W->dtype == MOE_DT_BF16 ? 1 : 0, (int)W->rows,
                                                                     (int)W->cols, (unsigned*)scratch);
  MOE_LAUNCH_CHECK();
  MOE_HIP(hipMemcpy(out_host, scratch, 4, hipMemcpyDeviceToHost));
  return MOE_OK;
}

MOE_API int moe_router_topk(const float* logits, int* ids, float* ws, int P, int E, int k,
                            int id_stride, moe_stream_t st) {
  if (!logits || !ids || !ws) return MOE_E_INVALID;
  if (P < 0 || E < 1 || k < 1 || k > E || k > 64 || id_stride < k) return MOE_E_INVALID;
  if (E > 1024) return MOE_E_UNSUPPORTED;
  if (P == 0) return MOE_OK;
  if (P <= 32)  // few tokens: a block per token, the fp64 exps spread over its threads
    return moe_launch_router_topk_small(logits, ids, ws, P, E, k, id_stride, nullptr, moe_s(st));
  dim3 g((P + 3) / 4);
  if (E <= 512) k_router_topk<8><<<g, 256, 0, moe_s(st)>>>(logits, ids, ws, P, E, k, id_stride);
  else k_router_topk<16><<<g, 256, 0, moe_s(st)>>>(logits, ids, ws, P, E, k, id_stride);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}
