// The further ggml block types of GGUF expert tensors, read in place: Q5_K (gate/up), Q5_1 and Q8_0 (down),
// IQ4_NL and IQ4_XS next to Q4_K — the mix of the reference's GGUF checkpoints (src/gpu/parts/30_host_util.inc:399-405,
// src/gpu/parts/26_kernels_moe_gguf.inc:32-48).  Dequantisation (bit-exact with gguf::dequant_row,
// src/gguf.h:339-445) and plain f32 GEMV kernels for any mix of these types: one wave per weight row,
// one lane per 32-element block.  These are the general kernels; Q4_K alone has the tuned ones
// (gemv_q4k.hip, decode_q4k.hip, the Q4_K instantiation of the grouped GEMM).
#include "common.h"
#include "dense.h"
#include "internal.h"
#include "iq4.h"

namespace {

__device__ __host__ __forceinline__ uint64_t gg_row_bytes(int t, uint64_t k) {
  if (moe_is_dense_type(t)) return moe_dense_row_bytes(t, k);
  switch (t) {
    case MOE_GGML_Q4_K: return k / 256 * 144;
    case MOE_GGML_Q5_K: return k / 256 * 176;
    case MOE_GGML_Q8_0: return k / 32 * 34;
    case MOE_GGML_Q5_1: return k / 32 * 24;
    case MOE_GGML_IQ4_NL: return k / 32 * 18;
    case MOE_GGML_IQ4_XS: return k / 256 * 136;
    default: return 0;
  }
}
__host__ size_t gg_align(int t) {  // widest load used
  return (t == MOE_GGML_Q8_0 || t == MOE_GGML_IQ4_NL) ? 2 : (t == MOE_GGML_Q5_1 || t == MOE_GGML_IQ4_XS) ? 8 : 16;
}
__host__ bool gg_type_ok(int t, int k) {
  if (t == MOE_GGML_Q4_K || t == MOE_GGML_Q5_K || t == MOE_GGML_IQ4_XS) return k >= 256 && k % 256 == 0;
  if (t == MOE_GGML_Q8_0 || t == MOE_GGML_Q5_1 || t == MOE_GGML_IQ4_NL) return k >= 32 && k % 32 == 0;
  return false;
}

__device__ __forceinline__ void k4_sm(int j, const uint8_t* q, int& sc, int& mn) {  // gguf.h:328-336
  if (j < 4) {
    sc = q[j] & 63;
    mn = q[j + 4] & 63;
  } else {
    sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
    mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
  }
}
__device__ __forceinline__ float h2f_bits(uint32_t h) { return __half2float(__ushort_as_half((uint16_t)h)); }

// Block b (32 consecutive elements) of a row: the 32 integer codes q[] in element order and the two
// constants of w = a*q + c (a, c and a*q are exact in f32: fp16 fields times integers of at most 8 bits).
// Loads are as wide as the block layouts allow: K-quant super-blocks (144 / 176 bytes) keep their fields
// 16-byte aligned, Q5_1 blocks (24 bytes) 8-byte aligned, Q8_0 blocks (34 bytes) 2-byte aligned; rows
// start on 32-byte boundaries in a GGUF file and on allocation boundaries in device memory.
__device__ __forceinline__ void gg_block(int t, const uint8_t* row, int b, int (&q)[32], float& a, float& c) {
  if (t == MOE_GGML_Q4_K || t == MOE_GGML_Q5_K) {
    const bool k5 = t == MOE_GGML_Q5_K;
    const uint8_t* sb = row + (size_t)(b >> 3) * (k5 ? 176 : 144);
    const int j = b & 7;  // sub-block: pair j/2, low nibbles if j even
    const uint4 hd = *(const uint4*)sb;  // d, dmin, scales[12]
    const uint8_t sc12[12] = {(uint8_t)hd.y, (uint8_t)(hd.y >> 8), (uint8_t)(hd.y >> 16), (uint8_t)(hd.y >> 24),
                              (uint8_t)hd.z, (uint8_t)(hd.z >> 8), (uint8_t)(hd.z >> 16), (uint8_t)(hd.z >> 24),
                              (uint8_t)hd.w, (uint8_t)(hd.w >> 8), (uint8_t)(hd.w >> 16), (uint8_t)(hd.w >> 24)};
    int sc, mn;
    k4_sm(j, sc12, sc, mn);
    a = h2f_bits(hd.x & 0xffffu) * (float)sc;
    c = -(h2f_bits(hd.x >> 16) * (float)mn);
    const uint4* ql = (const uint4*)(sb + (k5 ? 48 : 16) + 32 * (j >> 1));
    const uint4 l0 = ql[0], l1 = ql[1];
    const uint32_t lw[8] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w};
    uint32_t hw[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (k5) {
      const uint4* qh = (const uint4*)(sb + 16);
      const uint4 h0 = qh[0], h1 = qh[1];
      hw[0] = h0.x; hw[1] = h0.y; hw[2] = h0.z; hw[3] = h0.w;
      hw[4] = h1.x; hw[5] = h1.y; hw[6] = h1.z; hw[7] = h1.w;
    }
    const int nsh = (j & 1) ? 4 : 0;
#pragma unroll
    for (int l = 0; l < 32; l++) {
      const uint32_t byte = (lw[l >> 2] >> (8 * (l & 3))) & 0xffu, hb = (hw[l >> 2] >> (8 * (l & 3))) & 0xffu;
      q[l] = (int)(((byte >> nsh) & 0xFu) | (((hb >> j) & 1u) << 4));
    }
  } else if (t == MOE_GGML_Q8_0) {
    const uint16_t* p = (const uint16_t*)(row + (size_t)b * 34);
    uint16_t w[17];
#pragma unroll
    for (int i = 0; i < 17; i++) w[i] = p[i];
    a = h2f_bits(w[0]);
    c = 0.f;
#pragma unroll
    for (int l = 0; l < 16; l++) {
      q[2 * l] = (int)(int8_t)(w[1 + l] & 0xff);
      q[2 * l + 1] = (int)(int8_t)(w[1 + l] >> 8);
    }
  } else if (t == MOE_GGML_IQ4_NL || t == MOE_GGML_IQ4_XS) {
    // non-linear 4-bit codes (src/gguf.h:376-407): q = kv[nibble]; IQ4_XS adds a 6-bit scale per 32 elements
    uint16_t w[8];
    if (t == MOE_GGML_IQ4_NL) {
      const uint16_t* p = (const uint16_t*)(row + (size_t)b * 18);
      a = h2f_bits(p[0]);
#pragma unroll
      for (int i = 0; i < 8; i++) w[i] = p[1 + i];
    } else {
      const uint8_t* sb = row + (size_t)(b >> 3) * 136;
      const int ib = b & 7;
      const uint2 hd = *(const uint2*)sb;  // d, scales_h, scales_l[4]
      const uint32_t sh = hd.x >> 16, sl = (hd.y >> (8 * (ib >> 1))) & 0xffu;
      const int ls = (int)(((sl >> (4 * (ib & 1))) & 0xFu) | (((sh >> (2 * ib)) & 3u) << 4));
      a = h2f_bits(hd.x & 0xffffu) * (float)(ls - 32);
      const uint2* qs = (const uint2*)(sb + 8 + 16 * ib);
      const uint2 q0 = qs[0], q1 = qs[1];
      w[0] = (uint16_t)q0.x; w[1] = (uint16_t)(q0.x >> 16); w[2] = (uint16_t)q0.y; w[3] = (uint16_t)(q0.y >> 16);
      w[4] = (uint16_t)q1.x; w[5] = (uint16_t)(q1.x >> 16); w[6] = (uint16_t)q1.y; w[7] = (uint16_t)(q1.y >> 16);
    }
    c = 0.f;
    // kv = {-127,-104,-83,-65,-49,-35,-22,-10,1,13,25,38,53,69,89,113} as bytes of four words
    const uint32_t kv[4] = {0xbfad9881u, 0xf6eaddcfu, 0x26190d01u, 0x71594535u};
#pragma unroll
    for (int l = 0; l < 16; l++) {
      const uint32_t byte = (w[l >> 1] >> (8 * (l & 1))) & 0xffu, lo = byte & 0xFu, hi = byte >> 4;
      q[l] = (int)(int8_t)(kv[lo >> 2] >> (8 * (lo & 3)));
      q[l + 16] = (int)(int8_t)(kv[hi >> 2] >> (8 * (hi & 3)));
    }
  } else {  // Q5_1
    const uint2* p = (const uint2*)(row + (size_t)b * 24);
    const uint2 p0 = p[0], p1 = p[1], p2 = p[2];
    a = h2f_bits(p0.x & 0xffffu);
    c = h2f_bits(p0.x >> 16);
    const uint32_t qh = p0.y;
    const uint32_t qs[4] = {p1.x, p1.y, p2.x, p2.y};
#pragma unroll
    for (int l = 0; l < 16; l++) {
      const uint32_t byte = (qs[l >> 2] >> (8 * (l & 3))) & 0xffu;
      q[l] = (int)((byte & 0xFu) | (((qh >> l) & 1u) << 4));
      q[l + 16] = (int)((byte >> 4) | (((qh >> (l + 16)) & 1u) << 4));
    }
  }
}

// one thread per 32-element block
__global__ void __launch_bounds__(256) k_gg_dequant(int t, const uint8_t* __restrict__ raw, uint64_t cols,
                                                    uint64_t nblocks, float* __restrict__ out) {
  const uint64_t bpr = cols / 32, rbytes = gg_row_bytes(t, cols);
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nblocks; i += (uint64_t)gridDim.x * blockDim.x) {
    const uint64_t r = i / bpr;
    const int b = (int)(i % bpr);
    int q[32];
    float a, c;
    gg_block(t, raw + r * rbytes, b, q, a, c);
    float* y = out + r * cols + (uint64_t)b * 32;
#pragma unroll
    for (int l = 0; l < 32; l++) {
      const float prod = __fmul_rn(a, (float)q[l]);  // exact
      // Q8_0 / IQ4 have no constant term (keeps -0.0); else one rounded add
      y[l] = (t == MOE_GGML_Q8_0 || t == MOE_GGML_IQ4_NL || t == MOE_GGML_IQ4_XS) ? prod : __fadd_rn(prod, c);
    }
  }
}

__device__ __forceinline__ float wave_sum_f(float v) {
#pragma unroll
  for (int o = 32; o; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Activations sit in LDS with one float of padding per 32 (element i at GX_PAD(i)): lanes work on different
// 32-element blocks at the same offset, which without the padding is the same bank for every lane.
#define GX_PAD(i) ((i) + ((i) >> 5))
constexpr int GX_PITCH = 33;  // floats per 32-element block in LDS
                              // (128-bit reads at a pitch of 36 floats were measured: no faster, and the 32 extra registers cost occupancy)

// four bits b0..b3 of x to bit 0 of bytes 0..3
__device__ __forceinline__ uint32_t spread4(uint32_t x) { return ((x & 0xFu) * 0x00204081u) & 0x01010101u; }

// The same block for the dot products: the codes as unsigned bytes, four to a word (byte i of word w = element
// 4w + i), so that unpacking is a few word operations and a byte-to-float conversion per element; w = a*q + c
// with the constants adjusted where the stored codes are signed (Q8_0: q + 128).  Q4_K, Q5_K, Q8_0, Q5_1.
__device__ __forceinline__ void gg_block_packed(int t, const uint8_t* row, int b, uint32_t (&qp)[8], float& a, float& c) {
  if (t == MOE_GGML_Q4_K || t == MOE_GGML_Q5_K) {
    const bool k5 = t == MOE_GGML_Q5_K;
    const uint8_t* sb = row + (size_t)(b >> 3) * (k5 ? 176 : 144);
    const int j = b & 7;
    const uint4 hd = *(const uint4*)sb;
    const uint8_t sc12[12] = {(uint8_t)hd.y, (uint8_t)(hd.y >> 8), (uint8_t)(hd.y >> 16), (uint8_t)(hd.y >> 24),
                              (uint8_t)hd.z, (uint8_t)(hd.z >> 8), (uint8_t)(hd.z >> 16), (uint8_t)(hd.z >> 24),
                              (uint8_t)hd.w, (uint8_t)(hd.w >> 8), (uint8_t)(hd.w >> 16), (uint8_t)(hd.w >> 24)};
    int sc, mn;
    k4_sm(j, sc12, sc, mn);
    a = h2f_bits(hd.x & 0xffffu) * (float)sc;
    c = -(h2f_bits(hd.x >> 16) * (float)mn);
    const uint4* ql = (const uint4*)(sb + (k5 ? 48 : 16) + 32 * (j >> 1));
    const uint4 l0 = ql[0], l1 = ql[1];
    const uint32_t lw[8] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w};
    uint32_t hw[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (k5) {
      const uint4* qh = (const uint4*)(sb + 16);
      const uint4 h0 = qh[0], h1 = qh[1];
      hw[0] = h0.x; hw[1] = h0.y; hw[2] = h0.z; hw[3] = h0.w;
      hw[4] = h1.x; hw[5] = h1.y; hw[6] = h1.z; hw[7] = h1.w;
    }
    const int nsh = (j & 1) ? 4 : 0;
#pragma unroll
    for (int w = 0; w < 8; w++) qp[w] = ((lw[w] >> nsh) & 0x0f0f0f0fu) | (((hw[w] >> j) & 0x01010101u) << 4);
  } else if (t == MOE_GGML_Q8_0) {
    const uint16_t* p = (const uint16_t*)(row + (size_t)b * 34);
    uint16_t w16[17];
#pragma unroll
    for (int i = 0; i < 17; i++) w16[i] = p[i];
    a = h2f_bits(w16[0]);
    c = -128.f * a;
#pragma unroll
    for (int w = 0; w < 8; w++) qp[w] = ((uint32_t)w16[1 + 2 * w] | ((uint32_t)w16[2 + 2 * w] << 16)) ^ 0x80808080u;
  } else {  // Q5_1
    const uint2* p = (const uint2*)(row + (size_t)b * 24);
    const uint2 p0 = p[0], p1 = p[1], p2 = p[2];
    a = h2f_bits(p0.x & 0xffffu);
    c = h2f_bits(p0.x >> 16);
    const uint32_t qh = p0.y;
    const uint32_t qs[4] = {p1.x, p1.y, p2.x, p2.y};
#pragma unroll
    for (int w = 0; w < 4; w++) {
      qp[w] = (qs[w] & 0x0f0f0f0fu) | (spread4(qh >> (4 * w)) << 4);
      qp[4 + w] = ((qs[w] >> 4) & 0x0f0f0f0fu) | (spread4(qh >> (16 + 4 * w)) << 4);
    }
  }
}

// dot product of one row with x (K floats in LDS, padded; xsum[b] = sum of block b's activations): lanes take the
// 32-element blocks in turn
__device__ __forceinline__ float gg_unit_dot(int t, const uint8_t* row, int b, const float* xb, float sx) {
  float a, c, sq = 0.f;
  if (t == MOE_GGML_IQ4_NL || t == MOE_GGML_IQ4_XS) {
    int q[32];
    gg_block(t, row, b, q, a, c);
#pragma unroll
    for (int l = 0; l < 32; l++) sq = fmaf((float)q[l], xb[l], sq);
  } else {
    uint32_t qp[8];
    gg_block_packed(t, row, b, qp, a, c);
#pragma unroll
    for (int w = 0; w < 8; w++) {
      sq = fmaf((float)(qp[w] & 0xffu), xb[4 * w], sq);
      sq = fmaf((float)((qp[w] >> 8) & 0xffu), xb[4 * w + 1], sq);
      sq = fmaf((float)((qp[w] >> 16) & 0xffu), xb[4 * w + 2], sq);
      sq = fmaf((float)(qp[w] >> 24), xb[4 * w + 3], sq);
    }
  }
  return a * sq + c * sx;
}
// Gate and up row of one wave against x: the block type is a compile-time constant here and the loop body is
// straight-line code over two blocks per lane and row (lanes past the row work on block 0 and count as zero: no
// load sits under a branch), so the compiler issues the four blocks' loads together instead of one memory
// round trip after the other.
template <int T>
__device__ __forceinline__ void gg_rowpair_dot(const uint8_t* grow, const uint8_t* urow, const float* x,
                                               const float* xsum, int K, int lane, float& g, float& u) {
  const int nb = K / 32;
  float ag = 0.f, au = 0.f;
  for (int base = 0; base < nb; base += 128) {
    const int r0 = base + lane, r1 = base + 64 + lane;
    const int b0 = r0 < nb ? r0 : 0, b1 = r1 < nb ? r1 : 0;
    const float m0 = r0 < nb ? 1.f : 0.f, m1 = r1 < nb ? 1.f : 0.f;
    const float g0 = gg_unit_dot(T, grow, b0, x + GX_PITCH * b0, xsum[b0]);
    const float u0 = gg_unit_dot(T, urow, b0, x + GX_PITCH * b0, xsum[b0]);
    const float g1 = gg_unit_dot(T, grow, b1, x + GX_PITCH * b1, xsum[b1]);
    const float u1 = gg_unit_dot(T, urow, b1, x + GX_PITCH * b1, xsum[b1]);
    ag += m0 * g0 + m1 * g1;
    au += m0 * u0 + m1 * u1;
  }
  g = wave_sum_f(ag);
  u = wave_sum_f(au);
}
// the same for GG_DN_UNITS (slot, block) units of one output row of the down projection; unit = base + lane + 64 i
constexpr int GG_DN_UNITS = 2;  // (four at a time need more than 170 registers: fewer waves per CU, slower)
template <int T>
__device__ __forceinline__ float gg_down_units(const uint8_t* down, uint64_t rb, const int* eid, const float* wgt,
                                               int d, int r, int nb, int nunits, int base, int lane, const float* hs,
                                               const float* hsum) {
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < GG_DN_UNITS; i++) {
    const int uraw = base + lane + 64 * i;
    const bool ok = uraw < nunits;
    const int un = ok ? uraw : 0;
    const int s = un / nb, b = un - s * nb;
    const uint8_t* row = down + ((uint64_t)eid[s] * d + r) * rb;
    acc += (ok ? wgt[s] : 0.f) * gg_unit_dot(T, row, b, hs + GX_PITCH * un, hsum[un]);
  }
  return acc;
}
// dispatch on a block-uniform type: one scalar branch outside the loads
#define GG_TYPE_SWITCH(t, CALL)                                   \
  switch (t) {                                                    \
    case MOE_GGML_Q4_K: { constexpr int T = MOE_GGML_Q4_K; CALL; } break;   \
    case MOE_GGML_Q5_K: { constexpr int T = MOE_GGML_Q5_K; CALL; } break;   \
    case MOE_GGML_Q8_0: { constexpr int T = MOE_GGML_Q8_0; CALL; } break;   \
    case MOE_GGML_Q5_1: { constexpr int T = MOE_GGML_Q5_1; CALL; } break;   \
    case MOE_GGML_IQ4_NL: { constexpr int T = MOE_GGML_IQ4_NL; CALL; } break; \
    default: { constexpr int T = MOE_GGML_IQ4_XS; CALL; } break;            \
  }

struct GgxArgs {
  const uint8_t *gate, *up, *down;           // routed experts [E][rows][row bytes]
  const uint8_t *sh_gate, *sh_up, *sh_down;  // optional shared expert (raw rows of type tsh)
  int tgu, tdn, tsh;
  const float* sh_logit;
};

#ifndef MOE_GX_ROWS
#define MOE_GX_ROWS 8
#endif
#ifndef MOE_GX_THREADS
#define MOE_GX_THREADS 256
#endif
constexpr int GX_ROWS = MOE_GX_ROWS;        // gate rows per block of k_ggx_gu (16 measured the same; 32 rows in 256 or 512 threads 1.5x slower:
                                            // a wave's row pairs are sequential memory round trips)
constexpr int GX_THREADS = MOE_GX_THREADS;  // its block size (a wave takes every GX_THREADS/64-th row)
constexpr int GX_DN_ROWS = 4;   // output rows per block of k_ggx_dn: one per wave, d / 4 blocks fill the chip
// grid (ceil(mid/GX_ROWS), slots incl. shared, P), block GX_THREADS: hid[token][slot][row] = silu(gate.x) * (up.x)
__global__ void __launch_bounds__(GX_THREADS) k_ggx_gu(GgxArgs A, const float* __restrict__ x, const int* __restrict__ ids,
                                                int id_stride, int kpt, int d, int mid, float* __restrict__ hid) {
  extern __shared__ float xs[];
  const int s = blockIdx.y, tok = blockIdx.z;
  for (int i = threadIdx.x; i < d; i += blockDim.x) xs[GX_PAD(i)] = x[(size_t)tok * d + i];
  __syncthreads();
  float* xsum = xs + d / 32 * GX_PITCH;  // per-block sums of the activations, behind the padded activations
  for (int b = threadIdx.x; b < d / 32; b += blockDim.x) {
    float sx = 0.f;
    for (int l = 0; l < 32; l++) sx += xs[GX_PITCH * b + l];
    xsum[b] = sx;
  }
  __syncthreads();
  const bool shared = s >= kpt;
  const int t = shared ? A.tsh : A.tgu;
  const uint64_t rb = gg_row_bytes(t, d);
  const uint64_t e = shared ? 0 : (uint64_t)ids[(size_t)tok * id_stride + s];
  const uint8_t* gbase = shared ? A.sh_gate : A.gate + e * mid * rb;
  const uint8_t* ubase = shared ? A.sh_up : A.up + e * mid * rb;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  float* ho = hid + ((size_t)tok * gridDim.y + s) * mid;
  for (int rr = wv; rr < GX_ROWS; rr += GX_THREADS / 64) {
    const int r = blockIdx.x * GX_ROWS + rr;
    if (r >= mid) break;  // wave-uniform
    float g, u;
    GG_TYPE_SWITCH(t, gg_rowpair_dot<T>(gbase + (uint64_t)r * rb, ubase + (uint64_t)r * rb, xs, xsum, d, lane, g, u));
    if (lane == 0) ho[r] = silu_f(g) * u;
  }
}

// grid (ceil(d/GX_DN_ROWS), P), block 256: y[token][row] = sum over slots of w_s * (down_s . hid_s)
// + sigmoid(shared gate logit) * (shared down . hid_shared)
__global__ void __launch_bounds__(256) k_ggx_dn(GgxArgs A, const float* __restrict__ hid, const int* __restrict__ ids,
                                                const float* __restrict__ ws, int id_stride, int kpt, int d, int mid,
                                                float* __restrict__ out) {
  extern __shared__ float hs[];  // [slot][mid], padded
  __shared__ int eid[17];
  __shared__ float wgt[17];
  const int tok = blockIdx.y;
  const bool has_shared = A.sh_down != nullptr;
  const int nslots = kpt + (has_shared ? 1 : 0);
  for (int i = threadIdx.x; i < nslots * mid; i += blockDim.x) hs[GX_PAD(i)] = hid[(size_t)tok * nslots * mid + i];
  if ((int)threadIdx.x < nslots) {
    const int s = threadIdx.x;
    eid[s] = s < kpt ? ids[(size_t)tok * id_stride + s] : 0;
    wgt[s] = s < kpt ? ws[(size_t)tok * id_stride + s] : sigmoid_f(A.sh_logit[tok]);
  }
  __syncthreads();
  float* hsum = hs + nslots * mid / 32 * GX_PITCH;  // per-block sums, behind the padded activations
  for (int b = threadIdx.x; b < nslots * mid / 32; b += blockDim.x) {
    float sx = 0.f;
    for (int l = 0; l < 32; l++) sx += hs[GX_PITCH * b + l];
    hsum[b] = sx;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  // a wave per row; its lanes take the (slot, 32-element block) units in turn, each weighted by the slot's
  // combine weight, so a row needs one wave-wide sum (a fixed order: the result does not depend on timing)
  const int nb = mid / 32;
  for (int rr = wv; rr < GX_DN_ROWS; rr += 4) {
    const int r = blockIdx.x * GX_DN_ROWS + rr;
    if (r >= d) break;
    float acc = 0.f;
    {  // routed slots: one block type, GG_DN_UNITS units per lane and pass with all their loads in flight together
      const uint64_t rb = gg_row_bytes(A.tdn, mid);
      for (int base = 0; base < kpt * nb; base += 64 * GG_DN_UNITS)
        GG_TYPE_SWITCH(A.tdn, acc += gg_down_units<T>(A.down, rb, eid, wgt, d, r, nb, kpt * nb, base, lane, hs, hsum));
    }
    if (has_shared) {  // the shared expert's row: its own type; eid[kpt] = 0 and its rows start at sh_down
      const uint64_t rb = gg_row_bytes(A.tsh, mid);
      for (int base = 0; base < nb; base += 64 * GG_DN_UNITS) {
        float v = 0.f;
        GG_TYPE_SWITCH(A.tsh, v = gg_down_units<T>(A.sh_down, rb, eid + kpt, wgt + kpt, d, r, nb, nb, base, lane,
                                                   hs + GX_PITCH * (kpt * nb), hsum + kpt * nb));
        acc += v;
      }
    }
    acc = wave_sum_f(acc);
    if (lane == 0) out[(size_t)tok * d + r] = acc;
  }
}


// ---- grouped GEMM on MFMA for any of these block types (batches; src/gpu/parts/26_kernels_moe_gguf.inc:81-386) ----
// The general form of the batch path: a block = one tile of up to 128 (token, expert) pairs x 128 weight rows
// (gate/up: 64 gate rows and the matching 64 up rows, SwiGLU on the accumulators).  Per 64-wide K stage every
// thread dequantises one 32-element block of one weight row (gg_block: the ggml formula in f32, rounded to f16)
// into an f16 tile in LDS and copies four 16-byte pieces of the activation tile; the four waves (2 x 2, each
// 64 pairs x 64 rows = 2 x 2 tiles of v_mfma_f32_32x32x16_f16) read both operands from LDS.  Two stage buffers;
// the next stage is dequantised behind the current stage's MFMAs.  Activations and hid are f16 in natural element
// order.  The Q4_K-only layers keep the tuned kernel (gemm_q4cp.hip), which dequantises in registers.
typedef _Float16 gg_half8 __attribute__((ext_vector_type(8)));
typedef float gg_floatx16 __attribute__((ext_vector_type(16)));
constexpr int GG_BM = 128, GG_BN = 128, GG_BK = 64, GG_PITCH = 144;  // bytes per LDS row: 64 f16 + 16 (bank spread)
constexpr int GG_TILE_BYTES = GG_BM * GG_PITCH;                       // 18 KB per operand and stage
constexpr int GG_SMEM = 4 * GG_TILE_BYTES + GG_BM * 8;                // A, B x 2 stages + row indices + row scales

struct GgGemmW {
  const uint8_t *w, *w_up;  // expert tensors [E][M rows][row bytes] (gate / down, and up for the gate/up launch)
  int type;
};

// PK != 0: every tensor of the launch is Q8_0 (PK = 1), Q5_1 (PK = 2) -- the reference checkpoints' down tensors and MTP
// sidecar --, IQ4_NL (PK = 3) or IQ4_XS (PK = 4).  Those launches keep the raw bytes of three stages in flight in
// registers (a thread's block as dwords -- nine from the 4-byte boundary at or below a 34-byte Q8_0 block, the six of a
// 24-byte Q5_1 block, five around an 18-byte IQ4_NL block, an IQ4_XS super-block's header and the block's 16 code bytes
// -- and its four activation pieces) and turn the codes into f16 with byte permutes into the 1024 + u form and two or
// three packed operations per pair: the plain form below waits for a trip to memory in every stage.
constexpr int GQ_D = 3;
constexpr int GG_PK_Q8_0 = 1, GG_PK_Q5_1 = 2, GG_PK_IQ4_NL = 3, GG_PK_IQ4_XS = 4;
struct GgRawQ8 {
  uint32_t w[9];
};

template <bool UP, int PK = 0>
__global__ void __launch_bounds__(256, 2) k_moe_gemm_gg(GgGemmW R, GgGemmW Sh, int n_experts,
                                                       const __half* __restrict__ x16, const int* __restrict__ tokidx,
                                                       const moe_tile* __restrict__ tiles,
                                                       const int* __restrict__ ntiles, __half* __restrict__ out, int M,
                                                       int K, moe_hscale hs, int a_layout) {
  extern __shared__ __attribute__((aligned(16))) uint8_t gsm[];
  uint8_t* const As = gsm;
  uint8_t* const Bs = gsm + 2 * GG_TILE_BYTES;
  int* rowidx = (int*)(gsm + 4 * GG_TILE_BYTES);
  float* rowscale = (float*)(rowidx + GG_BM);
  const int ti = blockIdx.y;
  if (ti >= ntiles[0]) return;
  const moe_tile tile = tiles[ti];
  const bool shared = tile.expert >= n_experts;
  const GgGemmW& G = shared ? Sh : R;
  const int e = shared ? 0 : tile.expert, nb = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int n = lane & 31, h = lane >> 5, wm = wv >> 1, wn = wv & 1;
  if (tid < GG_BM) {
    const int m = tid < tile.count ? tid : 0;  // rows past the tile repeat row 0, never stored
    const int ri = tokidx ? tokidx[tile.first + m] : tile.first + m;
    rowidx[tid] = ri;
    rowscale[tid] = (UP && hs.xms) ? moe_hid_scale(shared ? hs.c_shared : hs.c_routed, hs.xms[ri]) : 1.f;
  }
  // this thread's weight row (half of each 64-wide stage of it)
  const int brow = tid >> 1, half = tid & 1;
  const uint64_t rb = gg_row_bytes(G.type, (uint64_t)K);
  int wr;
  const uint8_t* wbase;
  if (UP) {
    wr = nb * 64 + (brow & 63);
    wbase = brow < 64 ? G.w : G.w_up;
  } else {
    wr = nb * GG_BN + brow;
    wbase = G.w;
  }
  wr = wr < M ? wr : M - 1;  // clamped rows are computed and never stored
  const uint8_t* wrow = wbase + ((uint64_t)e * M + wr) * rb;
  __syncthreads();
  const __half* arow[4];
#pragma unroll
  for (int it = 0; it < 4; it++) arow[it] = x16 + (size_t)rowidx[(tid + 256 * it) >> 3] * K + ((tid + 256 * it) & 7) * 8;

  auto fill = [&](int s, int buf) {
#pragma unroll
    for (int it = 0; it < 4; it++) {
      const int i = tid + 256 * it;
      uint4 v = *(const uint4*)(arow[it] + (size_t)s * GG_BK);
      if (a_layout == 1) {
        // the q4cp GEMM's order inside a group of 8, [e0,e4,e1,e5,e2,e6,e3,e7], back to natural order
        const uint4 w = v;
        v.x = __builtin_amdgcn_perm(w.y, w.x, 0x05040100u);
        v.y = __builtin_amdgcn_perm(w.w, w.z, 0x05040100u);
        v.z = __builtin_amdgcn_perm(w.y, w.x, 0x07060302u);
        v.w = __builtin_amdgcn_perm(w.w, w.z, 0x07060302u);
      }
      if (a_layout == 2) {
        // the Q4_K / Q5_K GEMM's order inside a block of 64: chunk w = [4w, 4w+2, 32+4w, 32+4w+2, 4w+1, 4w+3, 32+4w+1,
        // 32+4w+3] -> elements 4w..4w+3 and 32+4w..32+4w+3 in natural order, two 8-byte pieces
        const int w = i & 7;
        uint8_t* rowp = As + buf * GG_TILE_BYTES + (i >> 3) * GG_PITCH;
        uint2 lo, hi;
        lo.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);  // (e4w, e4w+1)
        lo.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);  // (e4w+2, e4w+3)
        hi.x = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
        hi.y = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
        *(uint2*)(rowp + 8 * w) = lo;
        *(uint2*)(rowp + 64 + 8 * w) = hi;
        continue;
      }
      *(uint4*)(As + buf * GG_TILE_BYTES + (i >> 3) * GG_PITCH + (i & 7) * 16) = v;
    }
    uint8_t* dst = Bs + buf * GG_TILE_BYTES + brow * GG_PITCH + half * 64;
    if (moe_is_dense_type(G.type)) {
      float w[32];
      // (dense storage is the shared expert's: one matrix of M rows, e = 0; the planar q8g32 form needs the row count)
      moe_dense_block(G.type, wbase, (uint64_t)M, K, (uint64_t)e * M + wr, 2 * s + half, w);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        gg_half8 v;
#pragma unroll
        for (int l = 0; l < 8; l++) v[l] = (_Float16)w[8 * j + l];
        *(gg_half8*)(dst + 16 * j) = v;
      }
    } else {
      int q[32];
      float a, c;
      gg_block(G.type, wrow, 2 * s + half, q, a, c);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        gg_half8 v;
#pragma unroll
        for (int l = 0; l < 8; l++) v[l] = (_Float16)fmaf(a, (float)q[8 * j + l], c);
        *(gg_half8*)(dst + 16 * j) = v;
      }
    }
  };
  gg_floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  const int nstage = K / GG_BK;
  auto mfmas = [&](int buf) {
    const uint8_t* Ab = As + buf * GG_TILE_BYTES;
    const uint8_t* Bb = Bs + buf * GG_TILE_BYTES;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      gg_half8 a[2], b[2];
#pragma unroll
      for (int mf = 0; mf < 2; mf++) a[mf] = *(const gg_half8*)(Ab + (wm * 64 + 32 * mf + n) * GG_PITCH + ks * 32 + h * 16);
#pragma unroll
      for (int nf = 0; nf < 2; nf++) {
        const int br = UP ? 64 * nf + 32 * wn + n : 64 * wn + 32 * nf + n;
        b[nf] = *(const gg_half8*)(Bb + br * GG_PITCH + ks * 32 + h * 16);
      }
#pragma unroll
      for (int mf = 0; mf < 2; mf++)
#pragma unroll
        for (int nf = 0; nf < 2; nf++)
          acc[mf][nf] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mf], b[nf], acc[mf][nf], 0, 0, 0);
    }
  };
  if constexpr (PK != 0) {
    GgRawQ8 rw[GQ_D];
    uint4 ra[GQ_D][4];
    // block 2 s + half of the row: 34 bytes; odd blocks start 2 bytes past a 4-byte boundary (rows are whole pairs of
    // blocks), so nine dwords from the boundary at or below cover the block and never pass the row's end
    auto fetch = [&](int st, GgRawQ8& r, uint4 (&a4)[4]) {
      const int sc = st < nstage ? st : nstage - 1;  // (past the end: a repeat that is never used)
      if constexpr (PK == GG_PK_Q8_0) {
        const uint32_t* b4 = (const uint32_t*)(wrow + (size_t)(2 * sc + half) * 34 - 2 * half);
#pragma unroll
        for (int i = 0; i < 9; i++) r.w[i] = b4[i];
      } else if constexpr (PK == GG_PK_Q5_1) {  // d | m, qh, 16 bytes of nibbles
        const uint32_t* b4 = (const uint32_t*)(wrow + (size_t)(2 * sc + half) * 24);
#pragma unroll
        for (int i = 0; i < 6; i++) r.w[i] = b4[i];
      } else if constexpr (PK == GG_PK_IQ4_NL) {  // 18 bytes: d, 16 bytes of nibbles; odd blocks start 2 bytes past a boundary
        const uint32_t* b4 = (const uint32_t*)(wrow + (size_t)(2 * sc + half) * 18 - 2 * half);
#pragma unroll
        for (int i = 0; i < 5; i++) r.w[i] = b4[i];
      } else {  // IQ4_XS: the super-block's d | scales_h, scales_l and sub-block (2 sc + half) % 8's 16 bytes of nibbles
        const uint32_t* sb = (const uint32_t*)(wrow + (size_t)(sc >> 2) * 136);
        r.w[0] = sb[0];
        r.w[1] = sb[1];
        const uint32_t* q4 = sb + 2 + 4 * ((2 * sc + half) & 7);
#pragma unroll
        for (int i = 0; i < 4; i++) r.w[2 + i] = q4[i];
      }
#pragma unroll
      for (int it = 0; it < 4; it++) a4[it] = *(const uint4*)(arow[it] + (size_t)sc * GG_BK);
    };
    auto decode = [&](const GgRawQ8& r, const uint4 (&a4)[4], int buf, int stg) {
#pragma unroll
      for (int it = 0; it < 4; it++) {
        const int i = tid + 256 * it;
        uint4 v = a4[it];
        uint8_t* rowp = As + buf * GG_TILE_BYTES + (i >> 3) * GG_PITCH;
        if (a_layout == 2) {
          const int w = i & 7;
          uint2 lo, hi;
          lo.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
          lo.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
          hi.x = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
          hi.y = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
          *(uint2*)(rowp + 8 * w) = lo;
          *(uint2*)(rowp + 64 + 8 * w) = hi;
          continue;
        }
        if (a_layout == 1) {
          const uint4 w = v;
          v.x = __builtin_amdgcn_perm(w.y, w.x, 0x05040100u);
          v.y = __builtin_amdgcn_perm(w.w, w.z, 0x05040100u);
          v.z = __builtin_amdgcn_perm(w.y, w.x, 0x07060302u);
          v.w = __builtin_amdgcn_perm(w.w, w.z, 0x07060302u);
        }
        *(uint4*)(rowp + (i & 7) * 16) = v;
      }
      typedef _Float16 h2 __attribute__((ext_vector_type(2)));
      uint8_t* dst = Bs + buf * GG_TILE_BYTES + brow * GG_PITCH + half * 64;
      if constexpr (PK == GG_PK_Q5_1) {
        // w = d * q + m, q = nibble | fifth bit << 4 (element j: low nibble of byte j, bit j of qh; element 16 + j: high
        // nibble, bit 16 + j).  Four codes per dword as bytes; their fifth bits come out of qh with one multiply:
        // (u << 4) * (1 + 2^7 + 2^14 + 2^21) puts bit i of the 4-bit field u on bit 4 of byte i (all partial products
        // fall on distinct bits).  The f16 of d * q + m is one fused packed operation on the exact integer q.
        union { uint16_t u; _Float16 f; } dv, mv;
        dv.u = (uint16_t)(r.w[0] & 0xffffu);
        mv.u = (uint16_t)(r.w[0] >> 16);
        const h2 d2 = {dv.f, dv.f}, m2 = {mv.f, mv.f}, k1024 = {(_Float16)1024.f, (_Float16)1024.f};
        const uint32_t qh = r.w[1];
        uint32_t o[16];
#pragma unroll
        for (int cq = 0; cq < 4; cq++) {
          const uint32_t w = r.w[2 + cq];
          const uint32_t f_lo = (cq == 0 ? qh << 4 : qh >> (4 * cq - 4)) & 0xf0u;
          const uint32_t f_hi = (qh >> (12 + 4 * cq)) & 0xf0u;
          const uint32_t lo = ((f_lo * 0x204081u) & 0x10101010u) | (w & 0x0f0f0f0fu);
          const uint32_t hi = ((f_hi * 0x204081u) & 0x10101010u) | ((w >> 4) & 0x0f0f0f0fu);
          union { uint32_t u; h2 v; } p;
          p.u = __builtin_amdgcn_perm(0x64646464u, lo, 0x05010400u);  // (1024 + q0, 1024 + q1)
          p.v = (p.v - k1024) * d2 + m2;
          o[2 * cq] = p.u;
          p.u = __builtin_amdgcn_perm(0x64646464u, lo, 0x05030402u);
          p.v = (p.v - k1024) * d2 + m2;
          o[2 * cq + 1] = p.u;
          p.u = __builtin_amdgcn_perm(0x64646464u, hi, 0x05010400u);
          p.v = (p.v - k1024) * d2 + m2;
          o[8 + 2 * cq] = p.u;
          p.u = __builtin_amdgcn_perm(0x64646464u, hi, 0x05030402u);
          p.v = (p.v - k1024) * d2 + m2;
          o[8 + 2 * cq + 1] = p.u;
        }
#pragma unroll
        for (int j = 0; j < 4; j++) *(uint4*)(dst + 16 * j) = make_uint4(o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]);
        return;
      }
      if constexpr (PK == GG_PK_IQ4_NL || PK == GG_PK_IQ4_XS) {
        // w = dl * kv[n] (element j: low nibble of code byte j, element 16 + j: its high nibble), dl = d (IQ4_NL) or
        // d * (ls - 32) with the sub-block's 6-bit scale ls (IQ4_XS).  kv + 128 comes out of the register table as
        // bytes, becomes the f16 1024 + u by a byte permute, and (u - 128) * dl is a packed f16 product: the f16 of the
        // exact product for IQ4_NL; for IQ4_XS dl (17 significant bits) goes in as an f16 pair hi + lo with
        // fma(kv, hi, kv * lo), whose only early rounding is in the 2^-11 times smaller term.
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        uint32_t qd[4];
        h2 dh, dlo = {(_Float16)0.f, (_Float16)0.f};
        if constexpr (PK == GG_PK_IQ4_NL) {
          union { uint16_t u; _Float16 f; } dv;
          dv.u = (uint16_t)(half ? r.w[0] >> 16 : r.w[0] & 0xffffu);
          dh = h2{dv.f, dv.f};
#pragma unroll
          for (int i = 0; i < 4; i++) qd[i] = half ? r.w[i + 1] : __builtin_amdgcn_alignbit(r.w[i + 1], r.w[i], 16);
        } else {
          union { uint16_t u; _Float16 f; } dv;
          dv.u = (uint16_t)(r.w[0] & 0xffffu);
          const uint32_t sh = r.w[0] >> 16;
          const int sub = (2 * stg + half) & 7;  // sub-block within the super-block
          const uint32_t slb = (r.w[1] >> (8 * (sub >> 1))) & 0xffu;
          const int ls = (int)(((sub & 1) ? slb >> 4 : slb & 0xfu) | (((sh >> (2 * sub)) & 3u) << 4)) - 32;
          const float dl = (float)dv.f * (float)ls;  // exact in f32
          const _Float16 hi = (_Float16)dl, lo = (_Float16)(dl - (float)hi);
          dh = h2{hi, hi};
          dlo = h2{lo, lo};
#pragma unroll
          for (int i = 0; i < 4; i++) qd[i] = r.w[2 + i];
        }
        const h2 k1152 = {(_Float16)1152.f, (_Float16)1152.f};
        uint32_t o[16];
#pragma unroll
        for (int cq = 0; cq < 4; cq++) {
#pragma unroll
          for (int hn = 0; hn < 2; hn++) {  // low nibbles: elements 4 cq .. 4 cq + 3; high nibbles: 16 + the same
            const uint32_t ub = moe_iq4_lookup4<128>(qd[cq], 4 * hn);
#pragma unroll
            for (int l = 0; l < 2; l++) {
              union { uint32_t u; h2 v; } p;
              p.u = __builtin_amdgcn_perm(0x64646464u, ub, l ? 0x05030402u : 0x05010400u);
              const h2 kv = p.v - k1152;
              if constexpr (PK == GG_PK_IQ4_NL) p.v = kv * dh;
              else p.v = kv * dh + kv * dlo;
              o[8 * hn + 2 * cq + l] = p.u;
            }
          }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) *(uint4*)(dst + 16 * j) = make_uint4(o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]);
        return;
      }
      // Q8_0: d and the 32 codes, at byte 0 / 2 of the dwords (even block) or at byte 2 / 4 (odd block)
      union { uint16_t u; _Float16 f; } dv;
      dv.u = (uint16_t)(half ? r.w[0] >> 16 : r.w[0] & 0xffffu);
      const h2 d2 = {dv.f, dv.f}, k1152 = {(_Float16)1152.f, (_Float16)1152.f};
#pragma unroll
      for (int j = 0; j < 4; j++) {
        uint32_t o[4];
#pragma unroll
        for (int l = 0; l < 2; l++) {
          const int i = 2 * j + l;
          const uint32_t cd = (half ? r.w[i + 1] : __builtin_amdgcn_alignbit(r.w[i + 1], r.w[i], 16)) ^ 0x80808080u;
          union { uint32_t u; h2 v; } p0, p1;
          p0.u = __builtin_amdgcn_perm(0x64646464u, cd, 0x05010400u);  // (1024 + u0, 1024 + u1), u = code + 128
          p1.u = __builtin_amdgcn_perm(0x64646464u, cd, 0x05030402u);
          p0.v = (p0.v - k1152) * d2;  // code * d, one rounding: the f16 of the exact product
          p1.v = (p1.v - k1152) * d2;
          o[2 * l] = p0.u;
          o[2 * l + 1] = p1.u;
        }
        *(uint4*)(dst + 16 * j) = make_uint4(o[0], o[1], o[2], o[3]);
      }
    };
#pragma unroll
    for (int i = 0; i < GQ_D; i++) fetch(i, rw[i], ra[i]);
    decode(rw[0], ra[0], 0, 0);
    moe_lds_barrier();  // (every barrier of this loop: the raw blocks of the next stages stay in flight across it)
    for (int s0 = 0; s0 < nstage; s0 += GQ_D) {
#pragma unroll
      for (int u = 0; u < GQ_D; u++) {
        const int s = s0 + u;
        if (s < nstage) {
          const int buf = s & 1;
          // stage s is in LDS; the registers hold stages s + 1 and s + 2; slot u takes stage s + 3
          fetch(s + GQ_D, rw[u], ra[u]);
          mfmas(buf);
          if (s + 1 < nstage) decode(rw[(u + 1) % GQ_D], ra[(u + 1) % GQ_D], buf ^ 1, s + 1);
          moe_lds_barrier();
        }
      }
    }
  } else {
    fill(0, 0);
    __syncthreads();
    for (int s = 0; s < nstage; s++) {
      const int buf = s & 1;
      mfmas(buf);
      if (s + 1 < nstage) fill(s + 1, buf ^ 1);  // behind the MFMAs just issued; the other buffer was read a stage ago
      __syncthreads();
    }
  }
  // D[i][j]: j = lane % 32 (weight row), i = 8 * (r / 4) + 4 * (lane / 32) + r % 4 (pair)
  if constexpr (!UP) {
    // down launches: a wave's 64 x 64 results are 128 contiguous bytes of each of its 64 output rows.  Stored straight
    // from the accumulators they leave as 2-byte pieces, 64 bytes per half-wave and instruction; through a patch of the
    // wave's own in LDS (the operand tiles are dead: every wave is past the loop's last barrier) they leave as 16-byte
    // pieces, eight lanes to a whole line.  Rows at a pitch of 144 bytes: the two lane halves write rows m and m + 4,
    // which then lie 16 banks apart.
    static_assert(4 * 64 * GG_PITCH <= 4 * GG_TILE_BYTES, "four per-wave patches fit the operand tiles");
    uint8_t* const patch = gsm + wv * (64 * GG_PITCH);
#pragma unroll
    for (int mf = 0; mf < 2; mf++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int ml = 32 * mf + 8 * (r >> 2) + 4 * h + (r & 3);
#pragma unroll
        for (int nf = 0; nf < 2; nf++) *(__half*)(patch + ml * GG_PITCH + (32 * nf + n) * 2) = __float2half(acc[mf][nf][r]);
      }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the wave's own writes
    __builtin_amdgcn_wave_barrier();
    const int c8 = lane & 7, col = nb * GG_BN + 64 * wn + 8 * c8;
#pragma unroll
    for (int it = 0; it < 8; it++) {
      const int ml = 8 * it + (lane >> 3), m = wm * 64 + ml;
      const uint4 v = *(const uint4*)(patch + ml * GG_PITCH + c8 * 16);
      if (m < tile.count && col < M) *(uint4*)(out + (size_t)(tile.first + m) * M + col) = v;
    }
    return;
  }
#pragma unroll
  for (int mf = 0; mf < 2; mf++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int m = wm * 64 + 32 * mf + 8 * (r >> 2) + 4 * h + (r & 3);
      if (m >= tile.count) continue;
      __half* orow = out + (size_t)(tile.first + m) * M;
      if (UP) {
        const int col = nb * 64 + 32 * wn + n;
        const float g = acc[mf][0][r], u = acc[mf][1][r];
        if (col < M) orow[col] = __float2half(g / (1.f + __expf(-g)) * u * rowscale[m]);
      } else {
#pragma unroll
        for (int nf = 0; nf < 2; nf++) {
          const int col = nb * GG_BN + 64 * wn + 32 * nf + n;
          if (col < M) orow[col] = __float2half(acc[mf][nf][r]);
        }
      }
    }
}

}  // namespace

bool moe_gg_types_supported(int tgu, int tdn, int d, int mid) { return gg_type_ok(tgu, d) && gg_type_ok(tdn, mid); }
uint64_t moe_gg_row_bytes(int type, uint64_t k) { return gg_row_bytes(type, k); }

MOE_API int moe_gg_dequant_rows(int type, const uint8_t* raw, uint64_t nrows, uint64_t cols, float* out,
                                moe_stream_t st) {
  if (!raw || (!out && nrows)) return MOE_E_INVALID;
  if (cols == 0 || cols > (1ull << 31)) return MOE_E_INVALID;
  if (!gg_type_ok(type, (int)cols)) return MOE_E_UNSUPPORTED;
  if (nrows == 0) return MOE_OK;
  if (!moe_aligned(raw, gg_align(type)) || !moe_aligned(out, 4)) return MOE_E_INVALID;
  const uint64_t nblocks = nrows * (cols / 32);
  const unsigned grid = (unsigned)((nblocks + 255) / 256 > 65535 * 16 ? 65535 * 16 : (nblocks + 255) / 256);
  k_gg_dequant<<<grid, 256, 0, moe_s(st)>>>(type, raw, cols, nblocks, out);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// Internal launcher (shared with the context); shared-expert pointers may be null, tsh is their ggml type.
// phase: 0 = gate/up + down, 1 = gate/up only, 2 = down only.
int moe_launch_ggx_gemv(int phase, int tgu, int tdn, int tsh, const uint8_t* gate, const uint8_t* up,
                        const uint8_t* down, const uint8_t* sh_gate, const uint8_t* sh_up, const uint8_t* sh_down,
                        const float* sh_logit, const float* x, const int* ids, const float* ws, float* hid,
                        float* out, int P, int d, int mid, int kpt, int id_stride, hipStream_t st) {
  if (!gate || !up || !down || !x || !ids || !ws || !hid || !out) return MOE_E_INVALID;
  if (P < 0 || kpt < 1 || id_stride < kpt) return MOE_E_INVALID;
  if (!moe_gg_types_supported(tgu, tdn, d, mid)) return MOE_E_UNSUPPORTED;
  const bool sh = sh_gate != nullptr;
  if (sh && (!sh_up || !sh_down || !sh_logit)) return MOE_E_INVALID;
  if (sh && !(gg_type_ok(tsh, d) && gg_type_ok(tsh, mid))) return MOE_E_UNSUPPORTED;
  if (!moe_aligned(gate, gg_align(tgu)) || !moe_aligned(up, gg_align(tgu)) || !moe_aligned(down, gg_align(tdn)) ||
      (sh && (!moe_aligned(sh_gate, gg_align(tsh)) || !moe_aligned(sh_up, gg_align(tsh)) ||
              !moe_aligned(sh_down, gg_align(tsh)))))
    return MOE_E_INVALID;
  const int nslots = kpt + (sh ? 1 : 0);
  // LDS: the activations with one float of padding and one block sum per 32
  if (nslots > 16 || (size_t)d / 32 * (GX_PITCH + 1) * 4 > 60 * 1024 || (size_t)nslots * mid / 32 * (GX_PITCH + 1) * 4 > 60 * 1024)
    return MOE_E_UNSUPPORTED;
  if (P == 0) return MOE_OK;
  GgxArgs A{};
  A.gate = gate; A.up = up; A.down = down;
  A.sh_gate = sh_gate; A.sh_up = sh_up; A.sh_down = sh_down;
  A.tgu = tgu; A.tdn = tdn; A.tsh = tsh;
  A.sh_logit = sh_logit;
  if (phase != 2) {
    dim3 grid((mid + GX_ROWS - 1) / GX_ROWS, nslots, P);
    k_ggx_gu<<<grid, GX_THREADS, (size_t)d / 32 * (GX_PITCH + 1) * 4, st>>>(A, x, ids, id_stride, kpt, d, mid, hid);
    MOE_LAUNCH_CHECK();
  }
  if (phase != 1) {
    dim3 grid((d + GX_DN_ROWS - 1) / GX_DN_ROWS, P);
    k_ggx_dn<<<grid, 256, (size_t)nslots * mid / 32 * (GX_PITCH + 1) * 4, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, out);
    MOE_LAUNCH_CHECK();
  }
  return MOE_OK;
}

// Internal: grouped GEMM over tiles of <= 128 pairs for raw GGUF expert tensors of any supported block type
// (routed experts of type `type`, optional shared expert of type `tsh`; tile.expert >= n_experts selects it).
// `type` / `tsh` may also be a dense code of dense.h (bf16 / f32 / q8g64 rows).
// up: gate/up + SwiGLU -> hid f16 [pairs][m]; else down -> pairs f16 [pairs][m].  x / hid: f16, natural order
// (a_layout = 1 / 2: x is in the q4cp / Q4_K GEMM's order and is put back in natural order on its way into LDS).
int moe_launch_gemm_gg(bool up, int type, const uint8_t* w, const uint8_t* w_up, int tsh, const uint8_t* sh_w,
                       const uint8_t* sh_w_up, int n_experts, const __half* x16, const int* tokidx,
                       const moe_tile* tiles, const int* ntiles, int max_tiles, __half* out, int m, int k,
                       moe_hscale hs, hipStream_t st, int a_layout) {
  if (!w || (up && !w_up) || !x16 || !tiles || !ntiles || !out || max_tiles < 0) return MOE_E_INVALID;
  auto type_ok = [&](int t) { return moe_is_dense_type(t) ? k % 64 == 0 : gg_type_ok(t, k); };
  auto align_of = [&](int t) -> size_t { return moe_is_dense_type(t) ? 16 : gg_align(t); };
  if (!type_ok(type) || (sh_w && !type_ok(tsh)) || k % GG_BK || m < 1 || a_layout < 0 || a_layout > 2)
    return MOE_E_UNSUPPORTED;
  if (!moe_aligned(w, align_of(type)) || (up && !moe_aligned(w_up, align_of(type))) || !moe_aligned(x16, 16) ||
      (sh_w && (!moe_aligned(sh_w, align_of(tsh)) || (up && (!sh_w_up || !moe_aligned(sh_w_up, align_of(tsh)))))))
    return MOE_E_INVALID;
  if (!up && (m % 8 || !moe_aligned(out, 16))) return MOE_E_UNSUPPORTED;  // (down results leave as 16-byte pieces)
  if (max_tiles == 0) return MOE_OK;
  GgGemmW R{w, w_up, type}, S{sh_w ? sh_w : w, sh_w ? sh_w_up : w_up, sh_w ? tsh : type};
  const dim3 grid((unsigned)(up ? (m + 63) / 64 : (m + GG_BN - 1) / GG_BN), (unsigned)max_tiles);
  static moe_dev_once attr_once;
  int dev_now;
  if (moe_dev_pending(attr_once, &dev_now)) {
    MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_gg<true>, hipFuncAttributeMaxDynamicSharedMemorySize, GG_SMEM));
    MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_gg<false>, hipFuncAttributeMaxDynamicSharedMemorySize, GG_SMEM));
    MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_gg<true, GG_PK_Q8_0>, hipFuncAttributeMaxDynamicSharedMemorySize, GG_SMEM));
    MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_gg<false, GG_PK_Q8_0>, hipFuncAttributeMaxDynamicSharedMemorySize, GG_SMEM));
    MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_gg<true, GG_PK_Q5_1>, hipFuncAttributeMaxDynamicSharedMemorySize, GG_SMEM));
    MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_gg<false, GG_PK_Q5_1>, hipFuncAttributeMaxDynamicSharedMemorySize, GG_SMEM));
    MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_gg<true, GG_PK_IQ4_NL>, hipFuncAttributeMaxDynamicSharedMemorySize, GG_SMEM));
    MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_gg<false, GG_PK_IQ4_NL>, hipFuncAttributeMaxDynamicSharedMemorySize, GG_SMEM));
    MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_gg<true, GG_PK_IQ4_XS>, hipFuncAttributeMaxDynamicSharedMemorySize, GG_SMEM));
    MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_gg<false, GG_PK_IQ4_XS>, hipFuncAttributeMaxDynamicSharedMemorySize, GG_SMEM));
    moe_dev_done(attr_once, dev_now);
  }
  // all-Q8_0 / all-Q5_1 launches (4-byte aligned rows: whole pairs of 34-byte blocks, or 24-byte blocks, from a 4-byte
  // aligned base)
  const bool al4 = moe_aligned(w, 4) && (!up || moe_aligned(w_up, 4)) &&
                   (!sh_w || (moe_aligned(sh_w, 4) && (!up || moe_aligned(sh_w_up, 4))));
  const bool one_type = !sh_w || tsh == type;
  if (type == MOE_GGML_Q8_0 && one_type && al4) {
    if (up) k_moe_gemm_gg<true, GG_PK_Q8_0><<<grid, 256, GG_SMEM, st>>>(R, S, n_experts, x16, tokidx, tiles, ntiles, out, m, k, hs, a_layout);
    else k_moe_gemm_gg<false, GG_PK_Q8_0><<<grid, 256, GG_SMEM, st>>>(R, S, n_experts, x16, tokidx, tiles, ntiles, out, m, k, hs, a_layout);
  } else if (type == MOE_GGML_Q5_1 && one_type && al4) {
    if (up) k_moe_gemm_gg<true, GG_PK_Q5_1><<<grid, 256, GG_SMEM, st>>>(R, S, n_experts, x16, tokidx, tiles, ntiles, out, m, k, hs, a_layout);
    else k_moe_gemm_gg<false, GG_PK_Q5_1><<<grid, 256, GG_SMEM, st>>>(R, S, n_experts, x16, tokidx, tiles, ntiles, out, m, k, hs, a_layout);
  } else if (type == MOE_GGML_IQ4_NL && one_type && al4) {
    if (up) k_moe_gemm_gg<true, GG_PK_IQ4_NL><<<grid, 256, GG_SMEM, st>>>(R, S, n_experts, x16, tokidx, tiles, ntiles, out, m, k, hs, a_layout);
    else k_moe_gemm_gg<false, GG_PK_IQ4_NL><<<grid, 256, GG_SMEM, st>>>(R, S, n_experts, x16, tokidx, tiles, ntiles, out, m, k, hs, a_layout);
  } else if (type == MOE_GGML_IQ4_XS && one_type && al4) {
    if (up) k_moe_gemm_gg<true, GG_PK_IQ4_XS><<<grid, 256, GG_SMEM, st>>>(R, S, n_experts, x16, tokidx, tiles, ntiles, out, m, k, hs, a_layout);
    else k_moe_gemm_gg<false, GG_PK_IQ4_XS><<<grid, 256, GG_SMEM, st>>>(R, S, n_experts, x16, tokidx, tiles, ntiles, out, m, k, hs, a_layout);
  } else if (up) k_moe_gemm_gg<true><<<grid, 256, GG_SMEM, st>>>(R, S, n_experts, x16, tokidx, tiles, ntiles, out, m, k, hs, a_layout);
  else k_moe_gemm_gg<false><<<grid, 256, GG_SMEM, st>>>(R, S, n_experts, x16, tokidx, tiles, ntiles, out, m, k, hs, a_layout);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}
