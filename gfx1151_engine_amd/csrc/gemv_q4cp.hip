// Decode / small-batch expert GEMV on q4cp weights read in place: fused gate+up+SwiGLU, and the
// down projection with the top-k weighted combine (and the shared expert) folded into its epilogue.
// (reference: src/gpu/parts/20_kernels_gemv.inc:1608-1835, src/gpu/parts/40_model.inc:1832-1858)
#include "common.h"

namespace {

// Codebook handling: cb[n] = a*n + b for all 16 codes (e.g. zero-point 8: n - 8) lets a group's
// dot product be a*sum(n*x) + b*sum(x); any other codebook goes through a 16-entry LDS table.
struct CbInfo {
  float a, b;
  bool affine;
};
__device__ __forceinline__ CbInfo load_cb(const float* __restrict__ cb, float* cbs) {
  // every wave evaluates the same test; result is wave-uniform
  const int lane = threadIdx.x & 63;
  const float c0 = cb[0], c1 = cb[1];
  const float a = c1 - c0;
  bool ok = true;
  if (lane < 16) {
    const float v = cb[lane];
    ok = (v == fmaf((float)lane, a, c0));
    if (threadIdx.x < 16) cbs[lane] = v;
  }
  CbInfo r;
  r.a = a;
  r.b = c0;
  r.affine = __all(ok);
  return r;
}

// dot of 32 weights (16 B of codes) with 32 activations held as 8 float4
template <bool AFFINE>
__device__ __forceinline__ float dot32(const uint4 pk, const float4* xv, const float* cbs) {
  const uint32_t w[4] = {pk.x, pk.y, pk.z, pk.w};
  float a0 = 0.f, a1 = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t v = w[i];
    const float4 x0 = xv[2 * i], x1 = xv[2 * i + 1];
    if (AFFINE) {
      // even and odd nibbles as bytes: two masks, then one byte-to-float conversion per weight
      const uint32_t lo = v & 0x0f0f0f0fu, hi = (v >> 4) & 0x0f0f0f0fu;
      a0 = fmaf((float)(lo & 0xff), x0.x, a0);
      a1 = fmaf((float)(hi & 0xff), x0.y, a1);
      a0 = fmaf((float)((lo >> 8) & 0xff), x0.z, a0);
      a1 = fmaf((float)((hi >> 8) & 0xff), x0.w, a1);
      a0 = fmaf((float)((lo >> 16) & 0xff), x1.x, a0);
      a1 = fmaf((float)((hi >> 16) & 0xff), x1.y, a1);
      a0 = fmaf((float)(lo >> 24), x1.z, a0);
      a1 = fmaf((float)(hi >> 24), x1.w, a1);
    } else {
      a0 = fmaf(cbs[v & 0xf], x0.x, a0);
      a1 = fmaf(cbs[(v >> 4) & 0xf], x0.y, a1);
      a0 = fmaf(cbs[(v >> 8) & 0xf], x0.z, a0);
      a1 = fmaf(cbs[(v >> 12) & 0xf], x0.w, a1);
      a0 = fmaf(cbs[(v >> 16) & 0xf], x1.x, a0);
      a1 = fmaf(cbs[(v >> 20) & 0xf], x1.y, a1);
      a0 = fmaf(cbs[(v >> 24) & 0xf], x1.z, a0);
      a1 = fmaf(cbs[v >> 28], x1.w, a1);
    }
  }
  return a0 + a1;
}
// Pair tables (table codebooks, batches of more than a few tokens: the launch is bound by vector instructions): a code
// byte holds two neighbouring weights; a 256-entry table of (cb[b & 15], cb[b >> 4]) gives both with one 8-byte LDS
// read.  Sixteen copies side by side (entry b, copy c at dword 32 b + 2 c: 32 KB), a lane reads copy lane % 16: the
// sixteen lanes that an 8-byte read serves together sit on sixteen different bank pairs whatever their bytes are.
constexpr int PT_DW = 256 * 32;
typedef float float2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void build_ptab(float* tab, const float* __restrict__ cb) {
  for (int i = threadIdx.x; i < 256 * 16; i += blockDim.x) {
    const int b = i >> 4, c = i & 15;
    *(float2v*)(tab + b * 32 + c * 2) = float2v{cb[b & 15], cb[b >> 4]};
  }
}
__device__ __forceinline__ float dot32_pairs(const uint4 pk, const float4* xv, const float* tab_lane) {
  const uint32_t w[4] = {pk.x, pk.y, pk.z, pk.w};
  float a0 = 0.f, a1 = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t v = w[i];
    const float4 x0 = xv[2 * i], x1 = xv[2 * i + 1];
    const float2v t0 = *(const float2v*)(tab_lane + (v & 0xff) * 32);
    const float2v t1 = *(const float2v*)(tab_lane + ((v >> 8) & 0xff) * 32);
    const float2v t2 = *(const float2v*)(tab_lane + ((v >> 16) & 0xff) * 32);
    const float2v t3 = *(const float2v*)(tab_lane + (v >> 24) * 32);
    a0 = fmaf(t0.x, x0.x, a0);
    a1 = fmaf(t0.y, x0.y, a1);
    a0 = fmaf(t1.x, x0.z, a0);
    a1 = fmaf(t1.y, x0.w, a1);
    a0 = fmaf(t2.x, x1.x, a0);
    a1 = fmaf(t2.y, x1.y, a1);
    a0 = fmaf(t3.x, x1.z, a0);
    a1 = fmaf(t3.y, x1.w, a1);
  }
  return a0 + a1;
}

struct GuArgs {
  const uint8_t *codes, *scales;  // routed experts: fused gate_up [E*2*mid][d]
  const float* cb;
  uint64_t scale_stride;
  // optional shared expert as slot kpt of every token: separate gate / up tensors [mid][d]
  const uint8_t *sh_gcodes, *sh_gscales, *sh_ucodes, *sh_uscales;
  const float *sh_gcb, *sh_ucb;
  uint64_t sh_scale_stride;
};

// grid (mid / rows, slots per token incl. shared, P); block 256 = 4 waves.
// x of the token lies in LDS as float4 [j][g] (j-th quad of group g) so that lanes of
// consecutive groups read consecutive 16-byte words.
// A wave works on two gate rows (and their up rows) at a time: the 2 G groups of the pair are dealt to the lanes as
// units (unit u = row u / G, group u % G; 192 units = three per lane and pass), so that a row of 96 groups fills
// all 64 lanes.  The loads of the next step are in flight while the current one is summed, and a block's first
// loads leave before it stages x: at one token the launch is a few short blocks per CU, and what bounds it is how
// many bytes are in flight, not arithmetic.
constexpr int GU_NI = 3;
struct GuUnit {
  uint4 pg, pu;
  __half sg, su;  // (converted where they are used: a conversion at the load would wait for it there)
  float m;        // 0 for a unit past the pair's end
};

__global__ void __launch_bounds__(256) k_q4cp_gemv_gu(GuArgs A, const float* __restrict__ x,
                                                      uint64_t x_stride, const int* __restrict__ ids,
                                                      int id_stride, int kpt, int d, int mid, int rows_per_block,
                                                      float* __restrict__ hid) {
  extern __shared__ float4 xs[];  // d/4 float4, then d/32 group sums of x
  __shared__ float cbg[16], cbu[16];
  const int s = blockIdx.y, tok = blockIdx.z;
  const bool shared = s >= kpt;
  const int G = d / 32;
  float* const xsum = (float*)(xs + d / 4);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int r0 = blockIdx.x * rows_per_block;
  const int nrows = min(rows_per_block, mid - r0);
  float* ho = hid + ((size_t)tok * gridDim.y + s) * mid;
  const uint8_t *gc, *gs, *uc, *us;
  uint64_t ss;
  const float *cbgp, *cbup;
  if (!shared) {
    const int e = ids[(size_t)tok * id_stride + s];
    const uint64_t gr = (uint64_t)e * 2 * mid;
    gc = A.codes + gr * (d / 2);
    gs = A.scales + gr * A.scale_stride;
    uc = A.codes + (gr + mid) * (d / 2);
    us = A.scales + (gr + mid) * A.scale_stride;
    ss = A.scale_stride;
    cbgp = cbup = A.cb;
  } else {
    gc = A.sh_gcodes; gs = A.sh_gscales; uc = A.sh_ucodes; us = A.sh_uscales;
    ss = A.sh_scale_stride;
    cbgp = A.sh_gcb;
    cbup = A.sh_ucb;
  }
  // steps of this wave: (row pair q, pass p) with the pair at rows 2 wv + 8 q, units 192 p .. 192 p + 191
  const int npass = (2 * G + 64 * GU_NI - 1) / (64 * GU_NI);
  const int npairs = nrows > 2 * wv ? (nrows - 2 * wv + 7) / 8 : 0;
  const int nsteps = npairs * npass;
  auto load = [&](int st, GuUnit* u) {
    const int q = st / npass, p = st - q * npass;
    const int rr = 2 * wv + 8 * q;
    const int lim = min(2, nrows - rr) * G;
#pragma unroll
    for (int i = 0; i < GU_NI; i++) {
      // branch-free: a unit past the pair's end reads unit 0 and gets zero scales (loads under a divergent branch
      // are waited for one by one; in straight-line code they are all in flight together)
      const int idx0 = (p * GU_NI + i) * 64 + lane;
      const bool ok = idx0 < lim;
      const int idx = ok ? idx0 : 0;
      const float m = ok ? 1.f : 0.f;
      const int row = idx >= G ? 1 : 0, g = idx - row * G;
      const uint64_t r = (uint64_t)(r0 + rr + row);
      u[i].pg = *(const uint4*)(gc + r * (d / 2) + (size_t)g * 16);
      u[i].pu = *(const uint4*)(uc + r * (d / 2) + (size_t)g * 16);
      u[i].sg = ((const __half*)(gs + r * ss))[g];
      u[i].su = ((const __half*)(us + r * ss))[g];
      u[i].m = m;
    }
  };
  GuUnit cur[GU_NI], nxt[GU_NI];
  if (nsteps > 0) load(0, cur);
  const float* xt = x + (size_t)tok * x_stride;
  // (d / 4 is a multiple of 8: the eight quads of a group lie with eight neighbouring lanes)
  for (int i = threadIdx.x; i < d / 4; i += blockDim.x) {
    const float4 v = ((const float4*)xt)[i];
    xs[(i & 7) * G + (i >> 3)] = v;
    float t = (v.x + v.y) + (v.z + v.w);
    t += __shfl_xor(t, 1, 64);
    t += __shfl_xor(t, 2, 64);
    t += __shfl_xor(t, 4, 64);
    if ((i & 7) == 0) xsum[i >> 3] = t;
  }
  const CbInfo cg = load_cb(cbgp, cbg), cu = load_cb(cbup, cbu);
  __syncthreads();
  const bool affine = cg.affine && cu.affine;
  float ag0 = 0.f, au0 = 0.f, ag1 = 0.f, au1 = 0.f;
  for (int st = 0; st < nsteps; st++) {
    if (st + 1 < nsteps) load(st + 1, nxt);
    const int q = st / npass, p = st - q * npass;
#pragma unroll
    for (int i = 0; i < GU_NI; i++) {
      const int idx = (p * GU_NI + i) * 64 + lane;
      const int row = idx >= G ? 1 : 0;
      const int g = min(idx - row * G, G - 1);  // (a unit past the pair's end has zero scales)
      float4 xv[8];
#pragma unroll
      for (int j = 0; j < 8; j++) xv[j] = xs[j * G + g];
      float dg, du;
      if (affine) {
        const float sx = xsum[g];
        dg = fmaf(cg.a, dot32<true>(cur[i].pg, xv, cbg), cg.b * sx);
        du = fmaf(cu.a, dot32<true>(cur[i].pu, xv, cbu), cu.b * sx);
      } else {
        dg = dot32<false>(cur[i].pg, xv, cbg);
        du = dot32<false>(cur[i].pu, xv, cbu);
      }
      dg *= __half2float(cur[i].sg) * cur[i].m;
      du *= __half2float(cur[i].su) * cur[i].m;
      ag0 += row ? 0.f : dg;
      au0 += row ? 0.f : du;
      ag1 += row ? dg : 0.f;
      au1 += row ? du : 0.f;
    }
    if (p == npass - 1) {
      const int rr = 2 * wv + 8 * q;
      ag0 = wave_sum(ag0); au0 = wave_sum(au0); ag1 = wave_sum(ag1); au1 = wave_sum(au1);
      if (lane == 0) {
        ho[r0 + rr] = silu_f(ag0) * au0;
        if (rr + 1 < nrows) ho[r0 + rr + 1] = silu_f(ag1) * au1;
      }
      ag0 = au0 = ag1 = au1 = 0.f;
    }
#pragma unroll
    for (int i = 0; i < GU_NI; i++) cur[i] = nxt[i];
  }
}

struct DnArgs {
  const uint8_t *codes, *scales;  // routed experts down [E*d][mid]
  const float* cb;
  uint64_t scale_stride;
  const uint8_t *sh_codes, *sh_scales;  // optional shared expert down [d][mid]
  const float* sh_cb;
  uint64_t sh_scale_stride;
  const float* sh_logit;  // [P] shared-expert gate logit (weight = sigmoid)
  const float *ey, *sg;   // alternative: precomputed shared-expert output [P][d] and gate logit [P]
};

// Few tokens: grid (d / 8, P); block 256.  hid of all the token's slots in LDS as float4 [slot][j][g].
// A half-wave per output row, a lane per group (32 groups a pass); a lane has the codes and scales of all the
// row's slots in flight at once, and a block's first loads leave before it stages hid.  Every slot's partial
// stays in a register and the weighted sum runs in slot order (= descending router probability), then the shared
// expert.
constexpr int DNF_ROWS = 8;

__device__ __forceinline__ float half_wave_sum(float v) {
#pragma unroll
  for (int o = 16; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

template <int NS>
__global__ void __launch_bounds__(256) k_q4cp_gemv_dn_few(DnArgs A, const float* __restrict__ hid,
                                                      const int* __restrict__ ids,
                                                      const float* __restrict__ ws, int id_stride,
                                                      int kpt, int d, int mid, int rows_per_block,
                                                      float* __restrict__ out, uint64_t out_stride) {
  extern __shared__ float4 hs[];  // nslots * mid/4 float4, then nslots * mid/32 group sums
  __shared__ float cbr[16], cbsh[16];
  const int tok = blockIdx.y;
  const bool has_shared = A.sh_codes != nullptr;
  const int nslots = kpt + (has_shared ? 1 : 0);
  const int G = mid / 32, q = mid / 4;
  float* const hsum = (float*)(hs + (size_t)nslots * q);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, l32 = lane & 31;
  const int rb = blockIdx.x * rows_per_block + 2 * wv + (lane >> 5);  // this half-wave's first row; then every 8th
  const int rend = min(d, (int)(blockIdx.x + 1) * rows_per_block);
  const int npass = (G + 31) / 32;
  // steps of this wave: (row pair it, pass p); the wave's lower half decides how many there are
  const int rb0 = blockIdx.x * rows_per_block + 2 * wv;
  const int npairs = rend > rb0 ? (rend - rb0 + 7) / 8 : 0;
  const int nsteps = npairs * npass;
  uint4 pk[NS];
  __half sc[NS];  // (converted where they are used: a conversion at the load would wait for it there)
  auto load = [&](int st) {
    // branch-free (loads under a divergent branch are waited for one by one): a lane past the row's end, a row past
    // the block's and a slot past the token's reads a valid address and gets a zero scale
    const int it = st / npass, p = st - it * npass;
    const int r = rb + 8 * it;
    const bool live = r < rend;
    const int g0 = p * 32 + l32;
    const int g = g0 < G ? g0 : 0;
    const uint64_t rr = live ? (uint64_t)r : 0;
#pragma unroll
    for (int s = 0; s < NS; s++) {
      const int se = s < nslots ? s : 0;
      const bool sh = has_shared && se == nslots - 1;
      const uint64_t row = sh ? rr : (uint64_t)ids[(size_t)tok * id_stride + (sh ? 0 : se)] * d + rr;
      pk[s] = *(const uint4*)((sh ? A.sh_codes : A.codes) + row * (mid / 2) + (size_t)g * 16);
      sc[s] = ((const __half*)((sh ? A.sh_scales : A.scales) + row * (sh ? A.sh_scale_stride : A.scale_stride)))[g];
    }
  };
  if (nsteps > 0) load(0);
  const float* ht = hid + (size_t)tok * nslots * mid;
  for (int s = 0; s < nslots; s++)
    for (int c = threadIdx.x; c < q; c += blockDim.x) {  // (q is a multiple of 8: a group's quads lie with eight neighbouring lanes)
      const float4 v = ((const float4*)ht)[(size_t)s * q + c];
      hs[((size_t)s * 8 + (c & 7)) * G + (c >> 3)] = v;
      float t = (v.x + v.y) + (v.z + v.w);
      t += __shfl_xor(t, 1, 64);
      t += __shfl_xor(t, 2, 64);
      t += __shfl_xor(t, 4, 64);
      if ((c & 7) == 0) hsum[s * G + (c >> 3)] = t;
    }
  const CbInfo cr = load_cb(A.cb, cbr);
  CbInfo cs = cr;
  if (has_shared) cs = load_cb(A.sh_cb, cbsh);
  __syncthreads();
  const bool affine = cr.affine && cs.affine;
  float acc[NS];
#pragma unroll
  for (int s = 0; s < NS; s++) acc[s] = 0.f;
  for (int st = 0; st < nsteps; st++) {
    const int it = st / npass, p = st - it * npass;
    const int g = min(p * 32 + l32, G - 1);
    const float m = (rb + 8 * it < rend && p * 32 + l32 < G) ? 1.f : 0.f;  // a lane past the row's end, a row past the block's
#pragma unroll
    for (int s = 0; s < NS; s++) {
      if (s < nslots) {
        const bool sh = has_shared && s == nslots - 1;
        float4 xv[8];
#pragma unroll
        for (int j = 0; j < 8; j++) xv[j] = hs[((size_t)s * 8 + j) * G + g];
        float dv;
        if (affine) {
          const CbInfo c = sh ? cs : cr;
          dv = fmaf(c.a, dot32<true>(pk[s], xv, cbr), c.b * hsum[s * G + g]);
        } else {
          dv = dot32<false>(pk[s], xv, sh ? cbsh : cbr);
        }
        acc[s] = fmaf(dv, __half2float(sc[s]) * m, acc[s]);
      }
    }
    if (st + 1 < nsteps) load(st + 1);
    if (p == npass - 1) {
      const int r = rb + 8 * it;
      float y = 0.f;
#pragma unroll
      for (int s = 0; s < NS; s++) {
        if (s < nslots) {
          const float a = half_wave_sum(acc[s]);
          const float w = s < kpt ? ws[(size_t)tok * id_stride + s] : sigmoid_f(A.sh_logit[tok]);
          y += w * a;
        }
        acc[s] = 0.f;
      }
      if (r < rend && l32 == 0) {
        if (A.ey) y += sigmoid_f(A.sg[tok]) * A.ey[(size_t)tok * d + r];
        out[(size_t)tok * out_stride + r] = y;
      }
    }
  }
}

__device__ __forceinline__ float sum32(const float4* xv) {
  float s0 = 0.f, s1 = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i += 2) {
    s0 += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);
    s1 += (xv[i + 1].x + xv[i + 1].y) + (xv[i + 1].z + xv[i + 1].w);
  }
  return s0 + s1;
}

// grid (d / ROWS, P); block 256.  hid of all the token's slots in LDS as float4 [slot][j][g].
// Eight lanes per output row; every slot's partial stays in a register and the weighted sum runs
// in slot order (= descending router probability), then the shared expert.
constexpr int DN_ROWS = 32, DN_MAXSLOTS = 17;
// PAIR (not with AFFINE): the routed slots' look-ups through the pair table `ptab` (the shared expert's slot, one of
// eleven and with a codebook of its own, stays on the 16-entry table)
template <bool AFFINE, int NS, bool PAIR = false>
__device__ __forceinline__ void dn_rows(const DnArgs& A, const int* eid, const float* wgt, int nslots,
                                        bool has_shared, int d, int mid, int r0, int nrows, CbInfo cr,
                                        CbInfo cs, const float* cbr, const float* cbsh,
                                        const float4* hs, int tok, float* out, const float* ptab = nullptr) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, sub = lane >> 3, l8 = lane & 7;
  const int G = mid / 32;
  const float* const tab_lane = PAIR ? ptab + 2 * (lane & 15) : nullptr;
  for (int rr = wv * 8 + sub; rr < nrows; rr += (int)(blockDim.x >> 3)) {
    const int r = r0 + rr;
    float acc[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
      acc[s] = 0.f;
      if (s < nslots) {
        const bool sh = has_shared && s == nslots - 1;
        const uint64_t row = sh ? (uint64_t)r : (uint64_t)eid[s] * d + r;
        const uint8_t* rc = (sh ? A.sh_codes : A.codes) + row * (mid / 2);
        const __half* rs = (const __half*)((sh ? A.sh_scales : A.scales) + row * (sh ? A.sh_scale_stride : A.scale_stride));
        const CbInfo c = sh ? cs : cr;
        const float* cbl = sh ? cbsh : cbr;
        float a = 0.f;
        for (int g = l8; g < G; g += 8) {
          const uint4 pk = *(const uint4*)(rc + (size_t)g * 16);
          const float sc = __half2float(rs[g]);
          float4 xv[8];
#pragma unroll
          for (int j = 0; j < 8; j++) xv[j] = hs[((size_t)s * 8 + j) * G + g];
          float dv;
          if (PAIR && !sh) dv = dot32_pairs(pk, xv, tab_lane);
          else dv = dot32<AFFINE>(pk, xv, cbl);
          if (AFFINE) dv = fmaf(c.a, dv, c.b * sum32(xv));
          a = fmaf(dv, sc, a);
        }
        a += __shfl_xor(a, 4, 64);
        a += __shfl_xor(a, 2, 64);
        a += __shfl_xor(a, 1, 64);
        acc[s] = a;
      }
    }
    if (l8 == 0) {
      float y = 0.f;
#pragma unroll
      for (int s = 0; s < NS; s++)
        if (s < nslots) y += wgt[s] * acc[s];
      if (A.ey) y += sigmoid_f(A.sg[tok]) * A.ey[(size_t)tok * d + r];
      out[r] = y;
    }
  }
}

// PAIR: 512 threads and 64 rows per block, the routed experts' pair table behind hid in LDS (for codebooks that are not
// a*n + b; the launcher picks it for batches past the few-token sizes)
template <int NS, bool PAIR = false>
__global__ void __launch_bounds__(PAIR ? 512 : 256) k_q4cp_gemv_dn(DnArgs A, const float* __restrict__ hid,
                                                      const int* __restrict__ ids,
                                                      const float* __restrict__ ws, int id_stride,
                                                      int kpt, int d, int mid, float* __restrict__ out,
                                                      uint64_t out_stride) {
  extern __shared__ float4 hs[];  // nslots * mid/4 float4 (PAIR: then the pair table)
  __shared__ float cbr[16], cbsh[16];
  __shared__ int eid[DN_MAXSLOTS];
  __shared__ float wgt[DN_MAXSLOTS];
  const int tok = blockIdx.y;
  const bool has_shared = A.sh_codes != nullptr;
  const int nslots = kpt + (has_shared ? 1 : 0);
  const int G = mid / 32, q = mid / 4;
  const float* ht = hid + (size_t)tok * nslots * mid;
  for (int i = threadIdx.x; i < nslots * q; i += blockDim.x) {
    const int s = i / q, c = i % q;
    hs[((size_t)s * 8 + (c & 7)) * G + (c >> 3)] = ((const float4*)ht)[i];
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
  const CbInfo cr = load_cb(A.cb, cbr);
  CbInfo cs = cr;
  if (has_shared) cs = load_cb(A.sh_cb, cbsh);
  float* const ptab = (float*)(hs + (size_t)nslots * q);
  if (PAIR) build_ptab(ptab, A.cb);
  __syncthreads();
  const int rows_pb = (int)(blockDim.x >> 3);  // 8 lanes per row: 32 rows (256 threads) or 64 (512)
  const int r0 = blockIdx.x * rows_pb;
  const int nrows = min(rows_pb, d - r0);
  float* o = out + (size_t)tok * out_stride;
  if (PAIR)
    dn_rows<false, NS, true>(A, eid, wgt, nslots, has_shared, d, mid, r0, nrows, cr, cs, cbr, cbsh, hs, tok, o, ptab);
  else if (cr.affine && cs.affine)
    dn_rows<true, NS>(A, eid, wgt, nslots, has_shared, d, mid, r0, nrows, cr, cs, cbr, cbsh, hs, tok, o);
  else
    dn_rows<false, NS>(A, eid, wgt, nslots, has_shared, d, mid, r0, nrows, cr, cs, cbr, cbsh, hs, tok, o);
}

}  // namespace

static int check_q4cp(const moe_wview* w) {
  if (!w || !w->data) return MOE_E_INVALID;
  if (w->dtype != MOE_DT_Q4CP) return MOE_E_UNSUPPORTED;
  if (w->cols == 0 || w->cols % 32 || !moe_aligned(w->data, 16) || (w->cols / 2) % 16) return MOE_E_INVALID;
  // codes and scale records must stay 16-byte / 2-byte aligned behind the 64-byte codebook
  if ((w->rows * w->cols / 2) % 2) return MOE_E_INVALID;
  return MOE_OK;
}

// Internal launchers (shared with the context).  sh_* may be null.
int moe_launch_gemv_gu(const moe_wview* gu, const moe_wview* sh_gate, const moe_wview* sh_up,
                       const float* x, uint64_t x_stride, const int* ids, int id_stride, int kpt, int P,
                       int mid, float* hid, hipStream_t st) {
  int rc = check_q4cp(gu);
  if (rc) return rc;
  const int d = (int)gu->cols;
  if (P < 0 || kpt < 1 || mid < 1 || gu->rows % (2 * (uint64_t)mid)) return MOE_E_INVALID;
  if (d % 32 || (size_t)d * 4 > 48 * 1024) return MOE_E_UNSUPPORTED;
  if (!moe_aligned(x, 16) || x_stride % 4) return MOE_E_INVALID;
  if (P == 0) return MOE_OK;
  Q4cpOps o = q4cp_ops(gu);
  GuArgs A{};
  A.codes = o.codes; A.scales = o.scales; A.cb = o.cb; A.scale_stride = o.scale_stride;
  int nslots = kpt;
  if (sh_gate) {
    if ((rc = check_q4cp(sh_gate)) || (rc = check_q4cp(sh_up))) return rc;
    if ((int)sh_gate->cols != d || (int)sh_up->cols != d || (int)sh_gate->rows != mid || (int)sh_up->rows != mid)
      return MOE_E_INVALID;
    Q4cpOps g = q4cp_ops(sh_gate), u = q4cp_ops(sh_up);
    A.sh_gcodes = g.codes; A.sh_gscales = g.scales; A.sh_gcb = g.cb;
    A.sh_ucodes = u.codes; A.sh_uscales = u.scales; A.sh_ucb = u.cb;
    A.sh_scale_stride = g.scale_stride;
    nslots++;
  }
  // one row pair per wave where the launch would otherwise leave most of the device idle; more rows per block (one
  // staging of x for all of them) once there are blocks enough
  const int rows = (size_t)((mid + 7) / 8) * nslots * P <= 4096 ? 8 : 32;
  dim3 grid((mid + rows - 1) / rows, nslots, P);
  k_q4cp_gemv_gu<<<grid, 256, (size_t)d * 4 + (size_t)d / 8, st>>>(A, x, x_stride, ids, id_stride, kpt, d, mid, rows, hid);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_gemv_dn(const moe_wview* dn, const moe_wview* sh_down, const float* sh_logit,
                       const float* ey, const float* sg, const float* hid, const int* ids,
                       const float* ws, int id_stride, int kpt, int P, int d, float* out,
                       uint64_t out_stride, hipStream_t st, bool pair_tables) {
  int rc = check_q4cp(dn);
  if (rc) return rc;
  const int mid = (int)dn->cols;
  if (P < 0 || kpt < 1 || d < 1 || dn->rows % (uint64_t)d) return MOE_E_INVALID;
  const int nslots = kpt + (sh_down ? 1 : 0);
  if (nslots > 16) return MOE_E_UNSUPPORTED;
  if ((size_t)nslots * mid * 4 > 60 * 1024) return MOE_E_UNSUPPORTED;
  if (!moe_aligned(hid, 16)) return MOE_E_INVALID;
  if ((ey == nullptr) != (sg == nullptr)) return MOE_E_INVALID;
  if (P == 0) return MOE_OK;
  Q4cpOps o = q4cp_ops(dn);
  DnArgs A{};
  A.codes = o.codes; A.scales = o.scales; A.cb = o.cb; A.scale_stride = o.scale_stride;
  A.ey = ey; A.sg = sg;
  if (sh_down) {
    if ((rc = check_q4cp(sh_down))) return rc;
    if ((int)sh_down->cols != mid || (int)sh_down->rows != d || !sh_logit) return MOE_E_INVALID;
    Q4cpOps s = q4cp_ops(sh_down);
    A.sh_codes = s.codes; A.sh_scales = s.scales; A.sh_cb = s.cb; A.sh_scale_stride = s.scale_stride;
    A.sh_logit = sh_logit;
  }
  if ((size_t)((d + DNF_ROWS - 1) / DNF_ROWS) * P <= 1024) {
    // few tokens: 32-row blocks would leave most of the device idle
    dim3 grid((d + DNF_ROWS - 1) / DNF_ROWS, P);
    const size_t lds = (size_t)nslots * mid * 4 + (size_t)nslots * mid / 8;
    if (nslots <= 4) k_q4cp_gemv_dn_few<4><<<grid, 256, lds, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, DNF_ROWS, out, out_stride);
    else if (nslots <= 11) k_q4cp_gemv_dn_few<11><<<grid, 256, lds, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, DNF_ROWS, out, out_stride);
    else k_q4cp_gemv_dn_few<16><<<grid, 256, lds, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, DNF_ROWS, out, out_stride);
    MOE_LAUNCH_CHECK();
    return MOE_OK;
  }
  if (pair_tables) {
    // (the caller vouches that the routed experts' codebook is a table; 64 rows per block of 512 threads)
    const size_t ldp = (size_t)nslots * mid * 4 + (size_t)PT_DW * 4;
    if (ldp > 96 * 1024) return MOE_E_UNSUPPORTED;
    dim3 gp((d + 63) / 64, P);
#define DN_PAIR(N)                                                                                                     \
  do {                                                                                                                 \
    static moe_dev_once once;                                                                                          \
    int dev_now;                                                                                                       \
    if (moe_dev_pending(once, &dev_now)) {                                                                             \
      MOE_HIP(hipFuncSetAttribute((const void*)k_q4cp_gemv_dn<N, true>, hipFuncAttributeMaxDynamicSharedMemorySize,   \
                                  96 * 1024));                                                                         \
      moe_dev_done(once, dev_now);                                                                                     \
    }                                                                                                                  \
    k_q4cp_gemv_dn<N, true><<<gp, 512, ldp, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, out, out_stride);           \
  } while (0)
    if (nslots <= 4) DN_PAIR(4);
    else if (nslots <= 11) DN_PAIR(11);
    else DN_PAIR(16);
#undef DN_PAIR
    MOE_LAUNCH_CHECK();
    return MOE_OK;
  }
  dim3 grid((d + DN_ROWS - 1) / DN_ROWS, P);
  const size_t lds = (size_t)nslots * mid * 4;
  if (nslots <= 4) k_q4cp_gemv_dn<4><<<grid, 256, lds, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, out, out_stride);
  else if (nslots <= 11) k_q4cp_gemv_dn<11><<<grid, 256, lds, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, out, out_stride);
  else k_q4cp_gemv_dn<16><<<grid, 256, lds, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, out, out_stride);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

MOE_API int moe_q4cp_gemv_gate_up(const moe_wview* gu, const float* x, uint64_t x_stride,
                                  const int* ids, int id_stride, int kpt, int P, int mid, float* hid,
                                  moe_stream_t st) {
  if (!x || !ids || !hid) return MOE_E_INVALID;
  return moe_launch_gemv_gu(gu, nullptr, nullptr, x, x_stride, ids, id_stride, kpt, P, mid, hid, moe_s(st));
}

MOE_API int moe_q4cp_gemv_down_topk(const moe_wview* dn, const float* hid, const int* ids,
                                    const float* ws, int id_stride, int kpt, int P, int d,
                                    const float* ey, const float* sg, float* out, uint64_t out_stride,
                                    moe_stream_t st) {
  if (!hid || !ids || !ws || !out) return MOE_E_INVALID;
  return moe_launch_gemv_dn(dn, nullptr, nullptr, ey, sg, hid, ids, ws, id_stride, kpt, P, d, out, out_stride, moe_s(st), false);
}
