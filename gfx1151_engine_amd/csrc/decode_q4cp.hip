// Decode (T <= 32): bandwidth-bound expert GEMV on q4cp weights read in place, integer dot products.
// The activation vector is turned once per token into four planes of balanced base-16 digits per
// 32-element group (x ~= q_g * (4096 p3 + 256 p2 + 16 p1 + p0), 15.9 significant bits relative to the
// group maximum), stored in the nibble order of a q4cp code word.  A 16-byte load of 32 codes then
// costs 4 XORs (unsigned code n -> n - 8 in two's complement) and 16 v_dot8_i32_i4 instead of ~100
// float operations: the VALU keeps up with HBM.  Weights stay exact (codes are integers; the group
// scale, the codebook slope / offset and q_g are applied in f32 after the integer sum, the offset
// through the group sum of the activations).
// (reference: src/gpu/parts/20_kernels_gemv.inc:1608-1835 — same contract: per-slot gate/up with
//  SwiGLU, then the down projection with the top-k weighted combine in slot order, no atomics)
#include "common.h"
#include "internal.h"
#include "qvec.h"
#include "topk.h"

namespace {

__device__ __forceinline__ float dpp_max_row(float v) {  // max over each row of 16 lanes
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true)));
  return v;
}
// sum over each half-wave of 32 lanes; every lane of the half gets the result
__device__ __forceinline__ float sum32(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));   // xor 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true));   // xor 2
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true));  // mirror in 8
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true));  // mirror in 16
  return rows_half_add(v);
}
__device__ __forceinline__ float sum64(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true));
  return rows_total_add(v);
}

// Quantise 32 floats held one per lane by lanes [0,32) of a half-wave (j = lane & 31) into the qvec4
// form: returns this lane's four digits, q and q*sum(X).
__device__ __forceinline__ void quant32_lane(float x, int& p0, int& p1, int& p2, int& p3, float& q, float& qsx) {
  float m = dpp_max_row(fabsf(x));
  m = rows_half_max(m);
  const float inv = m > 0.f ? QV4_XMAX / m : 0.f;
  q = m * (1.f / QV4_XMAX);
  const int X = (int)rintf(x * inv);
  qv4_digits(X, p0, p1, p2, p3);
  qsx = q * sum32((float)X);
}

// One thread per group: x (f32, K elements) -> qvec4.  Blocks of 64.
__global__ void __launch_bounds__(64) k_qvec_from_f32(const float* __restrict__ x, uint64_t x_stride,
                                                      int G, uint32_t* __restrict__ planes,
                                                      float2* __restrict__ meta) {
  const int t = blockIdx.y, g = blockIdx.x * 64 + threadIdx.x;
  if (g < G) qvec4_group_from_f32(x, x_stride, G, t, g, planes, meta);
}

struct XG {  // one group's activation planes in registers
  uint32_t p[4][4];
  float q, qsx;
};
__device__ __forceinline__ void load_xg(XG& x, const uint32_t* planes, const float2* meta, size_t gi) {
  const uint4* s = (const uint4*)(planes + gi * QV4_GROUP_DW);
#pragma unroll
  for (int p = 0; p < 4; p++) {
    const uint4 a = s[p];
    x.p[p][0] = a.x; x.p[p][1] = a.y; x.p[p][2] = a.z; x.p[p][3] = a.w;
  }
  const float2 m = meta[gi];
  x.q = m.x;
  x.qsx = m.y;
}

// sum_k cb[n_k] * x_k over one group, cb = a*n + b = a*(n-8) + (8a+b):
//   a * q * (4096 D3 + 256 D2 + 16 D1 + D0) + (8a + b) * q * sum(X),  D_j = sum_k (n_k - 8) * p_j,k
__device__ __forceinline__ float chunk_dot(const uint4 cw, const XG& x, float cb_a, float cb_b8) {
  const uint32_t w[4] = {cw.x ^ 0x88888888u, cw.y ^ 0x88888888u, cw.z ^ 0x88888888u, cw.w ^ 0x88888888u};
  int d0 = 0, d1 = 0, d2 = 0, d3 = 0;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    d0 = __builtin_amdgcn_sdot8((int)w[i], (int)x.p[0][i], d0, false);
    d1 = __builtin_amdgcn_sdot8((int)w[i], (int)x.p[1][i], d1, false);
    d2 = __builtin_amdgcn_sdot8((int)w[i], (int)x.p[2][i], d2, false);
    d3 = __builtin_amdgcn_sdot8((int)w[i], (int)x.p[3][i], d3, false);
  }
  const int D = ((d3 * 16 + d2) * 16 + d1) * 16 + d0;  // |D| < 2^24: exact as f32
  return fmaf(cb_a * x.q, (float)D, cb_b8 * x.qsx);
}

struct DecW {  // one q4cp tensor's planes
  const uint8_t *codes, *scales;
  const float* cb;
  uint64_t ss;
  int gsh;  // 32-element groups per scale = 1 << gsh (q4cp: 0; hgn v2 i4r, one scale per 128 columns: 2)
};

// ---- codebooks that are not a*n + b (the reference converter's fixed non-uniform table, trained tables): the same
// kernels with a look-up instead of the integer dots, all in f32 (no quantised activations: the result differs
// from the f32 GEMV kernels only by the order of the additions).  The 16 codebook entries lie in LDS 32 times
// side by side (entry n, copy c at dword 32 n + c), so that lane l always reads bank l % 32: no conflicts,
// whatever the codes are.  A weight costs one bit-field extract, one address operation, one LDS read and one
// FMA; a lane keeps the 32 activations of the group it is working on in registers.
constexpr int LUT_DW = 16 * 32;  // dwords per table (2 KB)

struct XF {  // one group's activations
  float v[32];
};
constexpr int XF_PITCH = 36;  // floats between two groups' activations in LDS (see the staging in k_dec_gu)
__device__ __forceinline__ void load_xf(XF& x, const float* src) {  // src: global or LDS, 16-byte aligned
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const float4 f = ((const float4*)src)[i];
    x.v[4 * i] = f.x; x.v[4 * i + 1] = f.y; x.v[4 * i + 2] = f.z; x.v[4 * i + 3] = f.w;
  }
}
// the block fills one table
__device__ __forceinline__ void build_lut(float* lut, const float* __restrict__ cb) {
  for (int i = threadIdx.x; i < LUT_DW; i += blockDim.x) lut[i] = cb[i >> 5];
}
// sum_k cb[n_k] * x_k over one group (16 code bytes, low nibble = the earlier element); lut_lane = table + (lane & 31)
__device__ __forceinline__ float lut_dot(const uint4 cw, const XF& x, const float* lut_lane) {
  const uint32_t w[4] = {cw.x, cw.y, cw.z, cw.w};
  const uint32_t base = (uint32_t)(uintptr_t)lut_lane;  // LDS byte address of this lane's copy of entry 0
  float a0 = 0.f, a1 = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    // (an opaque copy of the word, pinned between this step's neighbours: otherwise the compiler works out the
    // addresses of a whole launch's look-ups ahead of the first one and spills hundreds of registers)
    uint32_t wi = w[i];
    asm volatile("" : "+v"(wi));
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      // entry n of this lane's copy: base + 128 n, two instructions (left to itself the compiler takes three:
      // shift, mask, add)
      uint32_t n_lo, n_hi, a_lo, a_hi;
      asm("v_bfe_u32 %0, %1, %2, 4" : "=v"(n_lo) : "v"(wi), "n"(4 * j));
      asm("v_bfe_u32 %0, %1, %2, 4" : "=v"(n_hi) : "v"(wi), "n"(4 * j + 4));
      asm("v_lshl_add_u32 %0, %1, 7, %2" : "=v"(a_lo) : "v"(n_lo), "v"(base));
      asm("v_lshl_add_u32 %0, %1, 7, %2" : "=v"(a_hi) : "v"(n_hi), "v"(base));
      const float t0 = *(const __attribute__((address_space(3))) float*)(uintptr_t)a_lo;
      const float t1 = *(const __attribute__((address_space(3))) float*)(uintptr_t)a_hi;
      a0 = fmaf(t0, x.v[8 * i + j], a0);
      a1 = fmaf(t1, x.v[8 * i + j + 1], a1);
    }
    if (i & 1) __builtin_amdgcn_sched_barrier(0);  // sixteen look-ups in flight at a time, not a whole row's
  }
  return a0 + a1;
}

// The same kernels once more for codebooks a*n + b in plain f32 arithmetic (the integer-dot kernels switched off):
// sum_k n_k * x_k over one group -- two masks per code word turn its even and odd nibbles into bytes, then a
// byte-to-float conversion and an FMA per weight; the caller adds b * sum(x).
__device__ __forceinline__ float aff_dot(const uint4 cw, const XF& x) {
  const uint32_t w[4] = {cw.x, cw.y, cw.z, cw.w};
  float a0 = 0.f, a1 = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t lo = w[i] & 0x0f0f0f0fu, hi = (w[i] >> 4) & 0x0f0f0f0fu;
    a0 = fmaf((float)(lo & 0xff), x.v[8 * i], a0);
    a1 = fmaf((float)(hi & 0xff), x.v[8 * i + 1], a1);
    a0 = fmaf((float)((lo >> 8) & 0xff), x.v[8 * i + 2], a0);
    a1 = fmaf((float)((hi >> 8) & 0xff), x.v[8 * i + 3], a1);
    a0 = fmaf((float)((lo >> 16) & 0xff), x.v[8 * i + 4], a0);
    a1 = fmaf((float)((hi >> 16) & 0xff), x.v[8 * i + 5], a1);
    a0 = fmaf((float)(lo >> 24), x.v[8 * i + 6], a0);
    a1 = fmaf((float)(hi >> 24), x.v[8 * i + 7], a1);
  }
  return a0 + a1;
}
__device__ __forceinline__ float xf_sum(const XF& x) {
  float s0 = 0.f, s1 = 0.f;
#pragma unroll
  for (int i = 0; i < 32; i += 2) {
    s0 += x.v[i];
    s1 += x.v[i + 1];
  }
  return s0 + s1;
}
// MODE 1: the look-up (any codebook); MODE 2: cb[n] = a n + b0 in f32, sx = the sum of the group's activations
template <int MODE>
__device__ __forceinline__ float f32_dot(const uint4 cw, const XF& x, const float* lut_lane, float a, float b0, float sx) {
  if (MODE == 2) return fmaf(a, aff_dot(cw, x), b0 * sx);
  return lut_dot(cw, x, lut_lane);
}

struct GuArgs2 {
  DecW gu;           // fused gate_up [E*2*mid][d]
  DecW shg, shu;     // shared expert gate / up [mid][d] (codes == nullptr: none)
  // hgn v2 rotated experts (not with UQ / LUT): the routed slots read the rotated activations' planes and write
  // their gate | up sums as they are, zraw[token][slot][2 mid] (the rotation back comes before SwiGLU); the shared
  // expert's slot is untouched by this
  float* zraw;
  const uint32_t* xplanes_rot;
  const float2* xmeta_rot;
};

// grid (mid/32, slots incl. shared, P); block 512.  Wave w: gate rows 4w..4w+3 and the matching up
// rows of this block's 32; lane L holds activation groups L and 64 + (L & 31).  Rows are taken two
// at a time with three 16-byte loads per lane: (row0, group L), (row1, group L), and the tail group
// of row0 (lanes < 32) or row1 (lanes >= 32); all twelve loads of a wave are in flight together.
// UQ ("unique experts", verify batches): grid (mid/32, tiles) instead; a tile = one expert with the
// (token, expert) pairs routed to it (expert-sorted lists of the routing permutation; the shared
// expert is the tile with expert id >= n_experts over all tokens).  The block reads its weight rows
// once and walks the tile's pairs; hid planes are then indexed by pair position.
// NPL > 0 (E <= 64*NPL, not with UQ): the router launch only left the logits; every block of a
// routed slot runs the softmax / top-k of its token itself (the same code and therefore the same
// ids and weights in every block; cheaper than a last-block ticket in the router launch plus a
// dependent load of the ids here) and block (0, 0, token) writes ids / weights out for the down
// kernel.  The shared expert's blocks skip it and have the CU to themselves meanwhile.
// LUT = 1 (not with UQ): table look-up arithmetic (above) for any codebook; xf32 = the tokens' activations [P][d],
// dynamic LDS = two tables (gate rows', up rows') and the token's d activations, hid goes out as f32 only.
// LUT = 2: the same data flow with f32 arithmetic for codebooks a*n + b (no tables).
constexpr int GU2_ROWS = 32;
template <bool UQ, int NPL, int LUT>
__global__ void __launch_bounds__(512, 4) k_dec_gu(GuArgs2 A, const uint32_t* __restrict__ xplanes,
                                                const float2* __restrict__ xmeta,
                                                const int* __restrict__ ids, int id_stride, int kpt, int d,
                                                int mid, uint32_t* __restrict__ hplanes,
                                                float2* __restrict__ hmeta, float* __restrict__ hid_f32,
                                                const moe_tile* __restrict__ tiles, const int* __restrict__ ntiles,
                                                const int* __restrict__ tokidx, int n_experts,
                                                const float* __restrict__ logits, int* __restrict__ ids_out,
                                                float* __restrict__ ws_out, const float* __restrict__ xf32, moe_rfix RF) {
  extern __shared__ float lutmem[];
  __shared__ float gs[GU2_ROWS], us[GU2_ROWS];
  __shared__ uint32_t pk[QV4_GROUP_DW];
  __shared__ int sel_ids[64];
  __shared__ float sel_ws[64];
  const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // (a scalar: see e)
  const int G = d / 32;
  int s = blockIdx.y, nslots = gridDim.y - (NPL > 0 ? 1 : 0), e = 0, first = 0, npairs = 1;
  if (NPL > 0 && s == nslots) {
    // one block of the extra grid row: the exact softmax / top-k (ids, renormalised weights) for the down
    // launch, next to the blocks that stream the weights and only need the ids
    if (blockIdx.x == 0) {
      select_certain<NPL ? NPL : 8, 512>(logits + (size_t)blockIdx.z * n_experts, RF, (int)blockIdx.z, sel_ids, sel_ws, n_experts, kpt, true);
      __syncthreads();
      if ((int)threadIdx.x < kpt) {
        ids_out[(size_t)blockIdx.z * id_stride + threadIdx.x] = sel_ids[threadIdx.x];
        ws_out[(size_t)blockIdx.z * id_stride + threadIdx.x] = sel_ws[threadIdx.x];
      }
    }
    return;
  }
  bool shared;
  if (UQ) {
    if ((int)blockIdx.y >= ntiles[0]) return;
    const moe_tile tile = tiles[blockIdx.y];
    shared = tile.expert >= n_experts;
    e = shared ? 0 : tile.expert;
    first = tile.first;
    npairs = tile.count;
  } else if (NPL > 0) {
    shared = s >= kpt;
    if (!shared) {
      // the ids by logit order (no exps, no sums); the exact selection only when two of the best logits
      // are too close for that to be certain
      const float* lg = logits + (size_t)blockIdx.z * n_experts;
      if (!select_certain<NPL ? NPL : 8, 512>(lg, RF, (int)blockIdx.z, sel_ids, sel_ws, n_experts, kpt, false)) __syncthreads();
      e = sel_ids[s];
    }
  } else {
    shared = s >= kpt;
    e = shared ? 0 : ids[(size_t)blockIdx.z * id_stride + s];
  }
  // the expert number is the same in every lane: as a scalar, the row and byte offsets that follow from it are scalar
  // arithmetic instead of 64-bit products per lane (quarter-rate instructions between the selection and the first load)
  e = __builtin_amdgcn_readfirstlane(e);
  const DecW Wg = shared ? A.shg : A.gu;  // block-uniform choice, by value
  const DecW Wu = shared ? A.shu : A.gu;
  const float *lutg = lutmem + (lane & 31), *lutu = lutg;
  if (LUT) {
    if (LUT == 1) {
      build_lut(lutmem, Wg.cb);
      if (Wu.cb != Wg.cb) {  // (block-uniform) the shared expert's up_proj is a tensor with a codebook of its own
        build_lut(lutmem + LUT_DW, Wu.cb);
        lutu += LUT_DW;
      }
    }
    // the token's activations, staged once per block: a lane fetches a group's 32 values when it starts on it.
    // A group's 128 bytes lie at a pitch of 144: lanes read different groups 16 bytes at a time, and at a pitch of
    // 128 every lane of such a read would sit on the same four banks (measured: 6.4 times the LDS time of this pitch).
    const float4* xr = (const float4*)(xf32 + (size_t)blockIdx.z * d);
    for (int i = threadIdx.x; i < d / 4; i += blockDim.x)
      ((float4*)(lutmem + (LUT == 1 ? 2 * LUT_DW : 0)))[(i >> 3) * (XF_PITCH / 4) + (i & 7)] = xr[i];
    __syncthreads();
  }
  const float* xs = lutmem + (LUT == 1 ? 2 * LUT_DW : 0);
  const uint64_t grow0 = shared ? 0 : (uint64_t)e * 2 * mid;
  const uint64_t urow0 = shared ? 0 : (uint64_t)e * 2 * mid + mid;
  const int r0 = blockIdx.x * GU2_ROWS + 4 * wv;  // first of this wave's 4 gate rows

  // Branch-free loads: a lane whose group lies past the row reads group 0 instead and gets a zero
  // scale.  (Loads inside divergent branches make the compiler wait for each of them where it is
  // issued; in straight-line code all of a wave's loads are in flight together.)
  const bool vA = lane < G, vB = 64 + (lane & 31) < G;
  const int gA = vA ? lane : 0, gB = vB ? 64 + (lane & 31) : 0;
  const float mA = vA ? 1.f : 0.f, mB = vB ? 1.f : 0.f;
  const size_t rb = (size_t)d / 2;
  // the activation planes and codebook constants are requested first: loads return in order, so
  // the dot products of the first row pair can start while the later rows are still in flight
  XG xa, xb;
  const bool raw = !UQ && !LUT && A.zraw && !shared;  // (block-uniform)
  if (!LUT && !UQ) {
    const size_t xbase = (size_t)blockIdx.z * G;
    const uint32_t* xp = raw ? A.xplanes_rot : xplanes;
    const float2* xm = raw ? A.xmeta_rot : xmeta;
    load_xg(xa, xp, xm, xbase + gA);
    load_xg(xb, xp, xm, xbase + gB);
  }
  const float ga = Wg.cb[1] - Wg.cb[0], gb = fmaf(8.f, ga, Wg.cb[0]), ua = Wu.cb[1] - Wu.cb[0], ub = fmaf(8.f, ua, Wu.cb[0]);
  // pairs 0,1: gate rows (r0+2p, r0+2p+1); pairs 2,3: the up rows
  uint4 ca[4], cb[4], ct[4];
  __half sa[4], sb[4], st[4];
#pragma unroll
  for (int p = 0; p < 4; p++) {
    const DecW W = p >= 2 ? Wu : Wg;
    const uint64_t row = (p >= 2 ? urow0 : grow0) + r0 + 2 * (p & 1);
    const uint8_t* c0 = W.codes + row * rb;
    const uint8_t* s0 = W.scales + row * W.ss;
    const uint64_t trow = lane < 32 ? 0 : 1;
    ca[p] = *(const uint4*)(c0 + (size_t)gA * 16);
    cb[p] = *(const uint4*)(c0 + rb + (size_t)gA * 16);
    sa[p] = *(const __half*)(s0 + (gA >> W.gsh) * 2);
    sb[p] = *(const __half*)(s0 + W.ss + (gA >> W.gsh) * 2);
    ct[p] = *(const uint4*)(c0 + trow * rb + (size_t)gB * 16);
    st[p] = *(const __half*)(s0 + trow * W.ss + (gB >> W.gsh) * 2);
  }
  __builtin_amdgcn_sched_barrier(0);  // every load above is issued before the first dot product
  for (int pi = 0; pi < npairs; pi++) {
  const int tok = UQ ? tokidx[first + pi] : (int)blockIdx.z;
  if (UQ) {
    const size_t xbase = (size_t)tok * G;
    load_xg(xa, xplanes, xmeta, xbase + gA);
    load_xg(xb, xplanes, xmeta, xbase + gB);
  }

  float acc[8];
  if (LUT) {
    // group gA of all eight rows first, then the tail group: one group's activations in registers at a time
    XF xf;
    load_xf(xf, xs + (size_t)gA * XF_PITCH);
    const float g0 = Wg.cb[0], u0 = Wu.cb[0];
    float sx = LUT == 2 ? xf_sum(xf) : 0.f;
#pragma unroll
    for (int p = 0; p < 4; p++) {
      const float* lt = p >= 2 ? lutu : lutg;
      const float a = p >= 2 ? ua : ga, b0 = p >= 2 ? u0 : g0;
      acc[2 * p] = __half2float(sa[p]) * mA * f32_dot<LUT>(ca[p], xf, lt, a, b0, sx);
      acc[2 * p + 1] = __half2float(sb[p]) * mA * f32_dot<LUT>(cb[p], xf, lt, a, b0, sx);
    }
    load_xf(xf, xs + (size_t)gB * XF_PITCH);
    sx = LUT == 2 ? xf_sum(xf) : 0.f;
#pragma unroll
    for (int p = 0; p < 4; p++) {
      const float vt = __half2float(st[p]) * mB * f32_dot<LUT>(ct[p], xf, p >= 2 ? lutu : lutg, p >= 2 ? ua : ga, p >= 2 ? u0 : g0, sx);
      if (lane < 32) acc[2 * p] += vt;
      else acc[2 * p + 1] += vt;
    }
  } else {
#pragma unroll
  for (int p = 0; p < 4; p++) {
    const float a = p >= 2 ? ua : ga, b = p >= 2 ? ub : gb;
    // (a multiplication, not a select: a select lets the compiler move the load back under a branch)
    const float fa = __half2float(sa[p]) * mA, fb = __half2float(sb[p]) * mA, ft = __half2float(st[p]) * mB;
    float v0 = fa * chunk_dot(ca[p], xa, a, b);
    float v1 = fb * chunk_dot(cb[p], xa, a, b);
    const float vt = ft * chunk_dot(ct[p], xb, a, b);
    if (lane < 32) v0 += vt;
    else v1 += vt;
    acc[2 * p] = v0;
    acc[2 * p + 1] = v1;
    __builtin_amdgcn_sched_barrier(0);  // row pair p is finished before the wait for pair p + 1
  }
  }
#pragma unroll
  for (int i = 0; i < 8; i++) acc[i] = sum64(acc[i]);
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      gs[4 * wv + i] = acc[i];
      us[4 * wv + i] = acc[4 + i];
    }
  }
  __syncthreads();
  if (raw) {
    if (threadIdx.x < 32) {
      float* zr = A.zraw + ((size_t)tok * kpt + s) * 2 * mid + blockIdx.x * GU2_ROWS + threadIdx.x;
      zr[0] = gs[threadIdx.x];
      zr[mid] = us[threadIdx.x];
    }
    return;
  }
  // SwiGLU on the block's 32 rows = one group of the down projection's input; quantise it
  if (wv == 0) {
    const int j = lane & 31;
    const float g = gs[j], u = us[j];
    const float hv = g / (1.f + expf(-g)) * u;
    const size_t slot = UQ ? (size_t)(first + pi) : (size_t)tok * nslots + s;
    if (hid_f32 && lane < 32) hid_f32[slot * mid + blockIdx.x * GU2_ROWS + j] = hv;
    if (LUT) return;  // (the down kernel of this arithmetic reads hid as f32)
    int p0, p1, p2, p3;
    float q, qsx;
    quant32_lane(hv, p0, p1, p2, p3, q, qsx);
    if (lane < QV4_GROUP_DW) pk[lane] = 0;
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_wave_barrier();
    if (lane < 32) {
      const int dw = j >> 3, sh = 4 * (j & 7);
      atomicOr(&pk[dw], (uint32_t)(p0 & 15) << sh);
      atomicOr(&pk[4 + dw], (uint32_t)(p1 & 15) << sh);
      atomicOr(&pk[8 + dw], (uint32_t)(p2 & 15) << sh);
      atomicOr(&pk[12 + dw], (uint32_t)(p3 & 15) << sh);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_wave_barrier();
    const size_t gi = slot * (mid / 32) + blockIdx.x;
    if (lane < QV4_GROUP_DW) hplanes[gi * QV4_GROUP_DW + lane] = pk[lane];
    if (lane == 0) hmeta[gi] = make_float2(q, qsx);
  }
  if (UQ) __syncthreads();  // gs / us / pk are reused by the next pair
  }
}

struct DnArgs2 {
  DecW dn;   // routed down [E*d][mid]
  DecW shd;  // shared expert down [d][mid] (codes == nullptr: none)
  const float* sh_logit;
  float* out_sh;  // != nullptr: the shared expert's gated rows go here instead of into the sum (same strides as out)
};

// grid (d/ROWS, P); block = 64 x ceil(slots/2).  Wave = one slot pair, half-wave = one slot: lane
// (L & 31) holds that slot's activation group (K/32 <= 32 groups) in registers for all the block's
// rows.  The weighted combine runs afterwards in slot order (descending router probability), then
// the shared expert: deterministic, no atomics.
constexpr int DN2_MAXSLOTS = 16;
#ifndef MOE_DN_ROWS
#define MOE_DN_ROWS 6
#endif
// LUT = 1: table look-up arithmetic for any codebook; hid_f32 = [P][slots][mid], dynamic LDS = two tables (the routed
// experts' tensor, the shared expert's).  LUT = 2: f32 arithmetic for codebooks a*n + b, no tables.
template <int ROWS, int LUT>
__global__ void __launch_bounds__(512) k_dec_dn(DnArgs2 A, const uint32_t* __restrict__ hplanes,
                                                const float2* __restrict__ hmeta,
                                                const int* __restrict__ ids, const float* __restrict__ ws,
                                                int id_stride, int kpt, int d, int mid,
                                                float* __restrict__ out, uint64_t out_stride,
                                                const float* __restrict__ hid_f32) {
  extern __shared__ float lutmem[];
  __shared__ float part[DN2_MAXSLOTS][ROWS];
  __shared__ float wsm[DN2_MAXSLOTS];
  const int tok = blockIdx.y;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const bool has_shared = A.shd.codes != nullptr;
  const int nslots = kpt + (has_shared ? 1 : 0);
  const int G = mid / 32, half = lane >> 5;
  const int r0 = blockIdx.x * ROWS;
  const size_t rb = (size_t)mid / 2;
  if (LUT == 1) {
    build_lut(lutmem, A.dn.cb);
    if (has_shared) build_lut(lutmem + LUT_DW, A.shd.cb);
    __syncthreads();
  }
  // combine weights of the token, fetched while the weight rows are in flight
  float wmine = 0.f;
  if ((int)threadIdx.x < nslots)
    wmine = (int)threadIdx.x < kpt ? ws[(size_t)tok * id_stride + threadIdx.x] : A.sh_logit[tok];
  {
    // Branch-free loads: lanes past the slots or past the row's groups read slot 0 / group 0 and
    // get a zero factor, so that all of a wave's loads are in flight together.
    const int s_raw = 2 * wv + half, g_raw = lane & 31;
    const bool live = s_raw < nslots && g_raw < G;
    const int s = live ? s_raw : 0, g = live ? g_raw : 0;
    const float m = live ? 1.f : 0.f;
    const bool shared = has_shared && s == nslots - 1;
    // per-lane choice of tensor: pick the members by value (a reference to one of two kernel
    // arguments would be re-read from memory in front of every load)
    const uint8_t* wcodes = shared ? A.shd.codes : A.dn.codes;
    const uint8_t* wscales = shared ? A.shd.scales : A.dn.scales;
    const float* wcb = shared ? A.shd.cb : A.dn.cb;
    const uint64_t wss = shared ? A.shd.ss : A.dn.ss;
    const int wgsh = shared ? A.shd.gsh : A.dn.gsh;
    // (an unconditional load -- the shared expert's lanes read slot 0's id and drop it: under a per-lane branch the
    // compiler waits for the id before it issues anything else.  Indices in 32 bits: a 64-bit product per lane is two
    // quarter-rate instructions.)
    const int e_any = ids[tok * id_stride + (shared ? 0 : s)];
    const uint32_t e = shared ? 0u : (uint32_t)e_any;
    XG x;
    XF xh;
    if (LUT) load_xf(xh, hid_f32 + ((size_t)tok * nslots + s) * mid + (size_t)g * 32);
    else load_xg(x, hplanes, hmeta, (size_t)((tok * nslots + s) * G + g));
    const float* lt = lutmem + (shared ? LUT_DW : 0) + (lane & 31);
    const float a = wcb[1] - wcb[0], b = fmaf(8.f, a, wcb[0]);
    const uint32_t row0 = e * (uint32_t)d + (uint32_t)r0;  // < experts * d: the launcher checks that it fits
    const uint8_t* cp = wcodes + (uint64_t)row0 * (uint32_t)rb + (uint32_t)g * 16;
    const uint8_t* sp = wscales + (uint64_t)row0 * (uint32_t)wss + (uint32_t)(g >> wgsh) * 2;
    uint4 cw[ROWS];
    __half sc[ROWS];
    {
      // (row addresses by repeated addition: wss is a per-lane value, and r * wss as a 64-bit product costs two
      // quarter-rate instructions per row)
      const uint8_t *cpr = cp, *spr = sp;
#pragma unroll
      for (int r = 0; r < ROWS; r++) {
        cw[r] = *(const uint4*)cpr;
        sc[r] = *(const __half*)spr;
        cpr += rb;
        spr += wss;
      }
    }
    __builtin_amdgcn_sched_barrier(0);  // every load is issued before the first dot product
    const float b0 = LUT == 2 ? wcb[0] : 0.f, sxh = LUT == 2 ? xf_sum(xh) : 0.f;
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
      float v = __half2float(sc[r]) * m * (LUT ? f32_dot<LUT>(cw[r], xh, lt, a, b0, sxh) : chunk_dot(cw[r], x, a, b));
      v = sum32(v);
      if (g_raw == 0 && s_raw < nslots) part[s_raw][r] = v;
      if ((r & 1) == 1) __builtin_amdgcn_sched_barrier(0);  // rows are consumed in arrival order
    }
  }
  if ((int)threadIdx.x < nslots) wsm[threadIdx.x] = (int)threadIdx.x < kpt ? wmine : sigmoid_f(wmine);
  __syncthreads();
  if (threadIdx.x < ROWS) {
    const int r = threadIdx.x;
    float y = 0.f;
    for (int s = 0; s < kpt; s++) y += wsm[s] * part[s][r];
    if (has_shared) {
      const float shv = wsm[kpt] * part[kpt][r];
      if (A.out_sh) A.out_sh[(size_t)tok * out_stride + r0 + r] = shv;
      else y += shv;
    }
    out[(size_t)tok * out_stride + r0 + r] = y;
  }
}

// Down projection of the unique-expert path: grid (d/DU_ROWS, tiles), block 256 = 8 half-waves of
// DU_HW rows.  Lane g of a half-wave holds group g of its weight rows and walks the tile's pairs; the
// unweighted row results go to pairs[pair][row] (f32) for the weighted combine that follows.
// All loads are unconditional (a lane past the last group reads group 0 and contributes 0) and are
// requested before the first is used: activation planes of the first pair, then the rows.
constexpr int DU_HW = 8, DU_ROWS = 8 * DU_HW;
__global__ void __launch_bounds__(256) k_dec_dn_uq(DnArgs2 A, const uint32_t* __restrict__ hplanes,
                                                   const float2* __restrict__ hmeta,
                                                   const moe_tile* __restrict__ tiles,
                                                   const int* __restrict__ ntiles, int n_experts, int d, int mid,
                                                   float* __restrict__ pairs) {
  if ((int)blockIdx.y >= ntiles[0]) return;
  const moe_tile tile = tiles[blockIdx.y];
  const bool shared = tile.expert >= n_experts;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int G = mid / 32, g_raw = lane & 31, hw = 2 * wv + (lane >> 5);
  const int g = g_raw < G ? g_raw : 0;
  const float live = g_raw < G ? 1.f : 0.f;
  const size_t rb = (size_t)mid / 2;
  const DecW W = shared ? A.shd : A.dn;  // block-uniform, by value
  const int r0 = blockIdx.x * DU_ROWS + DU_HW * hw;
  const uint64_t row0 = (shared ? 0 : (uint64_t)tile.expert * d) + r0;
  const uint8_t* cp = W.codes + row0 * rb + (size_t)g * 16;
  const uint8_t* sp = W.scales + row0 * W.ss + (g >> W.gsh) * 2;
  XG x;
  load_xg(x, hplanes, hmeta, (size_t)tile.first * G + g);
  const float c0 = W.cb[0], c1 = W.cb[1];
  uint4 cw[DU_HW];
  uint16_t sr[DU_HW];
#pragma unroll
  for (int r = 0; r < DU_HW; r++) {
    cw[r] = *(const uint4*)(cp + r * rb);
    sr[r] = *(const uint16_t*)(sp + r * W.ss);
  }
  __builtin_amdgcn_sched_barrier(0);
  const float a = c1 - c0, b = fmaf(8.f, a, c0);
  for (int pi = 0; pi < tile.count; pi++) {
    const size_t pr = (size_t)tile.first + pi;
    XG xn;  // the next pair's planes are requested before this pair's dot products (the last pair repeats itself)
    load_xg(xn, hplanes, hmeta, (pr + (pi + 1 < tile.count ? 1 : 0)) * G + g);
    float v[DU_HW];
#pragma unroll
    for (int r = 0; r < DU_HW; r++)
      v[r] = sum32(live * __half2float(__ushort_as_half(sr[r])) * chunk_dot(cw[r], x, a, b));
    if (g_raw == 0) {
      float4* o = (float4*)(pairs + pr * d + r0);
#pragma unroll
      for (int r = 0; r < DU_HW; r += 4) o[r / 4] = make_float4(v[r], v[r + 1], v[r + 2], v[r + 3]);
    }
    x = xn;
  }
}

DecW decw(const moe_wview* w) {
  DecW o{};
  if (w && w->dtype == MOE_DT_I4R) {  // codes, then one fp16 scale per 128 columns, rows unpadded; codebook n - 8
    o.codes = w->data;
    o.scales = w->data + w->rows * w->cols / 2;
    o.cb = moe_i4r_codebook();
    o.ss = w->cols / 128 * 2;
    o.gsh = 2;
  } else if (w) {
    Q4cpOps q = q4cp_ops(w);
    o.codes = q.codes; o.scales = q.scales; o.cb = q.cb; o.ss = q.scale_stride;
  }
  return o;
}

}  // namespace

size_t moe_qvec_plane_bytes(int K) { return (size_t)(K / 32) * QV_GROUP_DW * 4; }
size_t moe_qvec_meta_bytes(int K) { return (size_t)(K / 32) * sizeof(float2); }

// Supported shapes of the integer-dot decode kernels (otherwise the caller uses the f32 kernels).
bool moe_dec_supported(int d, int mid, int nslots) {
  return d % 32 == 0 && d / 32 <= 96 && mid % 32 == 0 && mid / 32 <= 32 && nslots <= DN2_MAXSLOTS &&
         mid % GU2_ROWS == 0;  // (d % 32 == 0 covers the 8-row down blocks)
}
// the unique-expert kernels on top of that: whole row blocks of the down kernel
bool moe_dec_uq_supported(int d) { return d % DU_ROWS == 0; }

int moe_launch_qvec(const float* x, uint64_t x_stride, int P, int K, uint32_t* planes, float2* meta,
                    hipStream_t st) {
  const int G = K / 32;
  dim3 grid((G + 63) / 64, P);
  k_qvec_from_f32<<<grid, 64, 0, st>>>(x, x_stride, G, planes, meta);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_dec_gu(const moe_wview* gu, const moe_wview* sh_gate, const moe_wview* sh_up,
                      const uint32_t* xplanes, const float2* xmeta, const int* ids, int id_stride, int kpt,
                      int P, int d, int mid, uint32_t* hplanes, float2* hmeta, float* hid_f32,
                      hipStream_t st, const moe_dec_v2* v2) {
  GuArgs2 A{};
  A.gu = decw(gu);
  A.shg = decw(sh_gate);
  A.shu = decw(sh_up);
  if (v2) {
    if (!v2->zraw || !v2->xplanes_rot || !v2->xmeta_rot) return MOE_E_INVALID;
    A.zraw = v2->zraw;
    A.xplanes_rot = v2->xplanes_rot;
    A.xmeta_rot = v2->xmeta_rot;
  }
  if (!A.gu.cb) return MOE_E_STATE;
  dim3 grid(mid / GU2_ROWS, kpt + (sh_gate ? 1 : 0), P);
  k_dec_gu<false, 0, 0><<<grid, 512, 0, st>>>(A, xplanes, xmeta, ids, id_stride, kpt, d, mid, hplanes, hmeta, hid_f32,
                                                  nullptr, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, moe_rfix{});
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// The same with the softmax / top-k of every token done inside the launch: logits [P][n_experts] in,
// ids / ws rows (id_stride wide) out.
bool moe_dec_gu_topk_supported(int n_experts, int kpt) { return n_experts <= 1024 && kpt <= 64 && kpt <= n_experts; }
int moe_launch_dec_gu_topk(const moe_wview* gu, const moe_wview* sh_gate, const moe_wview* sh_up,
                           const uint32_t* xplanes, const float2* xmeta, const float* logits, int n_experts,
                           int* ids, float* ws, int id_stride, int kpt, int P, int d, int mid,
                           uint32_t* hplanes, float2* hmeta, float* hid_f32, hipStream_t st, const moe_dec_v2* v2,
                           const moe_rfix* rf) {
  const moe_rfix RFV = rf ? *rf : moe_rfix{};
  GuArgs2 A{};
  A.gu = decw(gu);
  A.shg = decw(sh_gate);
  A.shu = decw(sh_up);
  if (v2) {
    if (!v2->zraw || !v2->xplanes_rot || !v2->xmeta_rot) return MOE_E_INVALID;
    A.zraw = v2->zraw;
    A.xplanes_rot = v2->xplanes_rot;
    A.xmeta_rot = v2->xmeta_rot;
  }
  if (!A.gu.cb) return MOE_E_STATE;
  dim3 grid(mid / GU2_ROWS, kpt + (sh_gate ? 1 : 0) + 1, P);  // + the row of the exact top-k block
  if (n_experts <= 512)
    k_dec_gu<false, 8, 0><<<grid, 512, 0, st>>>(A, xplanes, xmeta, nullptr, id_stride, kpt, d, mid, hplanes, hmeta,
                                                    hid_f32, nullptr, nullptr, nullptr, n_experts, logits, ids, ws, nullptr, RFV);
  else
    k_dec_gu<false, 16, 0><<<grid, 512, 0, st>>>(A, xplanes, xmeta, nullptr, id_stride, kpt, d, mid, hplanes, hmeta,
                                                     hid_f32, nullptr, nullptr, nullptr, n_experts, logits, ids, ws, nullptr, RFV);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// The look-up kernels (any codebook): x f32 [P][d] in, hid f32 [P][kpt + shared][mid] out; softmax / top-k inside
// the launch as above.
// (affine: every codebook involved is a*n + b -- the f32 arithmetic instead of the look-up.  logits == nullptr: the
//  ids are given and no selection runs inside the launch.)
int moe_launch_dec_gu_lut(const moe_wview* gu, const moe_wview* sh_gate, const moe_wview* sh_up, const float* x,
                          const float* logits, int n_experts, int* ids, float* ws, int id_stride, int kpt, int P, int d,
                          int mid, float* hid_f32, hipStream_t st, const moe_rfix* rf, bool affine) {
  if (!x || !hid_f32 || !ids || (logits && !moe_dec_gu_topk_supported(n_experts, kpt))) return MOE_E_INVALID;
  const moe_rfix RFV = rf ? *rf : moe_rfix{};
  GuArgs2 A{};
  A.gu = decw(gu);
  A.shg = decw(sh_gate);
  A.shu = decw(sh_up);
  dim3 grid(mid / GU2_ROWS, kpt + (sh_gate ? 1 : 0) + (logits ? 1 : 0), P);
  const int lds = (affine ? 0 : 2 * LUT_DW * 4) + d / 32 * XF_PITCH * 4;
  if (lds > 64 * 1024) return MOE_E_UNSUPPORTED;
#define DEC_GU_F32(NPL, MODE)                                                                                          \
  k_dec_gu<false, NPL, MODE><<<grid, 512, lds, st>>>(A, nullptr, nullptr, NPL ? nullptr : ids, id_stride, kpt, d, mid, nullptr, \
                                                     nullptr, hid_f32, nullptr, nullptr, nullptr, n_experts, logits, ids, ws, x, RFV)
  if (!logits) {
    if (affine) DEC_GU_F32(0, 2);
    else DEC_GU_F32(0, 1);
  } else if (n_experts <= 512) {
    if (affine) DEC_GU_F32(8, 2);
    else DEC_GU_F32(8, 1);
  } else {
    if (affine) DEC_GU_F32(16, 2);
    else DEC_GU_F32(16, 1);
  }
#undef DEC_GU_F32
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_dec_dn_lut(const moe_wview* dn, const moe_wview* sh_down, const float* sh_logit, const float* hid_f32,
                          const int* ids, const float* ws, int id_stride, int kpt, int P, int d, int mid, float* out,
                          uint64_t out_stride, hipStream_t st, bool affine) {
  DnArgs2 A{};
  A.dn = decw(dn);
  A.shd = decw(sh_down);
  A.sh_logit = sh_logit;
  if (dn->rows > 0xffffffffull) return MOE_E_UNSUPPORTED;  // (row numbers are 32-bit in the kernel)
  const int nslots = kpt + (sh_down ? 1 : 0), bs = 64 * ((nslots + 1) / 2);
  constexpr int lds = 2 * LUT_DW * 4;
#define DEC_DN_F32(ROWS, MODE)                                                                                          \
  k_dec_dn<ROWS, MODE><<<dim3(d / ROWS, P), bs, MODE == 1 ? lds : 0, st>>>(A, nullptr, nullptr, ids, ws, id_stride, kpt, d, mid, \
                                                                           out, out_stride, hid_f32)
  if (d % MOE_DN_ROWS == 0) {
    if (affine) DEC_DN_F32(MOE_DN_ROWS, 2);
    else DEC_DN_F32(MOE_DN_ROWS, 1);
  } else {
    if (affine) DEC_DN_F32(8, 2);
    else DEC_DN_F32(8, 1);
  }
#undef DEC_DN_F32
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// Unique-expert variants: tiles / ntiles / tokidx from the routing permutation (tiles of <= 32 pairs,
// the shared expert as expert id n_experts); hplanes / hmeta and pairs are indexed by pair position.
int moe_launch_dec_gu_uq(const moe_wview* gu, const moe_wview* sh_gate, const moe_wview* sh_up,
                         const uint32_t* xplanes, const float2* xmeta, const moe_tile* tiles, const int* ntiles,
                         int max_tiles, const int* tokidx, int n_experts, int d, int mid, uint32_t* hplanes,
                         float2* hmeta, hipStream_t st) {
  GuArgs2 A{};
  A.gu = decw(gu);
  A.shg = decw(sh_gate);
  A.shu = decw(sh_up);
  if (max_tiles <= 0) return MOE_OK;
  dim3 grid(mid / GU2_ROWS, max_tiles);
  k_dec_gu<true, 0, 0><<<grid, 512, 0, st>>>(A, xplanes, xmeta, nullptr, 0, 0, d, mid, hplanes, hmeta, nullptr, tiles,
                                                 ntiles, tokidx, n_experts, nullptr, nullptr, nullptr, nullptr, moe_rfix{});
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_dec_dn_uq(const moe_wview* dn, const moe_wview* sh_down, const uint32_t* hplanes,
                         const float2* hmeta, const moe_tile* tiles, const int* ntiles, int max_tiles,
                         int n_experts, int d, int mid, float* pairs, hipStream_t st) {
  DnArgs2 A{};
  A.dn = decw(dn);
  A.shd = decw(sh_down);
  if (max_tiles <= 0) return MOE_OK;
  dim3 grid(d / DU_ROWS, max_tiles);
  k_dec_dn_uq<<<grid, 256, 0, st>>>(A, hplanes, hmeta, tiles, ntiles, n_experts, d, mid, pairs);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_dec_dn(const moe_wview* dn, const moe_wview* sh_down, const float* sh_logit,
                      const uint32_t* hplanes, const float2* hmeta, const int* ids, const float* ws,
                      int id_stride, int kpt, int P, int d, int mid, float* out, uint64_t out_stride,
                      hipStream_t st, float* out_sh) {
  DnArgs2 A{};
  A.dn = decw(dn);
  A.shd = decw(sh_down);
  A.sh_logit = sh_logit;
  A.out_sh = out_sh;
  if (!A.dn.cb) return MOE_E_STATE;
  if (dn->rows > 0xffffffffull) return MOE_E_UNSUPPORTED;  // (row numbers are 32-bit in the kernel)
  const int nslots = kpt + (sh_down ? 1 : 0), bs = 64 * ((nslots + 1) / 2);
  // MOE_DN_ROWS rows per block where that divides d (d = 3072: 512 blocks, two per CU), else 8
  if (d % MOE_DN_ROWS == 0)
    k_dec_dn<MOE_DN_ROWS, 0><<<dim3(d / MOE_DN_ROWS, P), bs, 0, st>>>(A, hplanes, hmeta, ids, ws, id_stride, kpt, d, mid, out, out_stride, nullptr);
  else
    k_dec_dn<8, 0><<<dim3(d / 8, P), bs, 0, st>>>(A, hplanes, hmeta, ids, ws, id_stride, kpt, d, mid, out, out_stride, nullptr);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}
