// The further ggml block types of GGUF expert tensors, read in place: Q5_K (gate/up), Q5_1 and Q8_0 (down),
// IQ4_NL and IQ4_XS next to Q4_K — the mix of the reference's GGUF checkpoints (src/gpu/parts/30_host_util.inc:399-405,
// src/gpu/parts/26_kernels_moe_gguf.inc:32-48).  Dequantisation (bit-exact with gguf::dequant_row,
// src/gguf.h:339-445) and plain f32 GEMV kernels for any mix of these types: one wave per weight row,
// one lane per 32-element block.  These are the general kernels; Q4_K alone has the tuned ones
// (gemv_q4k.hip, decode_q4k.hip, the Q4_K instantiation of the grouped GEMM).
#include "common.h"
#include "internal.h"

namespace {

__device__ __host__ __forceinline__ uint64_t gg_row_bytes(int t, uint64_t k) {
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
__device__ __forceinline__ float gg_row_dot(int t, const uint8_t* row, const float* x, const float* xsum, int K,
                                            int lane) {
  float acc = 0.f;
  for (int b = lane; b < K / 32; b += 64) acc += gg_unit_dot(t, row, b, x + 33 * b, xsum[b]);
  return wave_sum_f(acc);
}

struct GgxArgs {
  const uint8_t *gate, *up, *down;           // routed experts [E][rows][row bytes]
  const uint8_t *sh_gate, *sh_up, *sh_down;  // optional shared expert (raw rows of type tsh)
  int tgu, tdn, tsh;
  const float* sh_logit;
};

constexpr int GX_ROWS = 8;      // gate rows per block of k_ggx_gu (a wave takes every fourth)
constexpr int GX_DN_ROWS = 4;   // output rows per block of k_ggx_dn: one per wave, d / 4 blocks fill the chip
// grid (ceil(mid/GX_ROWS), slots incl. shared, P), block 256: hid[token][slot][row] = silu(gate.x) * (up.x)
__global__ void __launch_bounds__(256) k_ggx_gu(GgxArgs A, const float* __restrict__ x, const int* __restrict__ ids,
                                                int id_stride, int kpt, int d, int mid, float* __restrict__ hid) {
  extern __shared__ float xs[];
  const int s = blockIdx.y, tok = blockIdx.z;
  for (int i = threadIdx.x; i < d; i += blockDim.x) xs[GX_PAD(i)] = x[(size_t)tok * d + i];
  __syncthreads();
  float* xsum = xs + d / 32 * 33;  // per-block sums of the activations, behind the padded activations
  for (int b = threadIdx.x; b < d / 32; b += blockDim.x) {
    float sx = 0.f;
    for (int l = 0; l < 32; l++) sx += xs[33 * b + l];
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
  for (int rr = wv; rr < GX_ROWS; rr += 4) {
    const int r = blockIdx.x * GX_ROWS + rr;
    if (r >= mid) break;  // wave-uniform
    const float g = gg_row_dot(t, gbase + (uint64_t)r * rb, xs, xsum, d, lane);
    const float u = gg_row_dot(t, ubase + (uint64_t)r * rb, xs, xsum, d, lane);
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
  float* hsum = hs + nslots * mid / 32 * 33;  // per-block sums, behind the padded activations
  for (int b = threadIdx.x; b < nslots * mid / 32; b += blockDim.x) {
    float sx = 0.f;
    for (int l = 0; l < 32; l++) sx += hs[33 * b + l];
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
    for (int u = lane; u < nslots * nb; u += 64) {
      const int s = u / nb, b = u - s * nb;
      const bool sh = has_shared && s == nslots - 1;
      const int t = sh ? A.tsh : A.tdn;
      const uint64_t rb = gg_row_bytes(t, mid);
      const uint8_t* row = sh ? A.sh_down + (uint64_t)r * rb : A.down + ((uint64_t)eid[s] * d + r) * rb;
      acc += wgt[s] * gg_unit_dot(t, row, b, hs + 33 * (s * nb + b), hsum[s * nb + b]);
    }
    acc = wave_sum_f(acc);
    if (lane == 0) out[(size_t)tok * d + r] = acc;
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
  if (nslots > 16 || (size_t)d / 32 * 34 * 4 > 60 * 1024 || (size_t)nslots * mid / 32 * 34 * 4 > 60 * 1024)
    return MOE_E_UNSUPPORTED;
  if (P == 0) return MOE_OK;
  GgxArgs A{};
  A.gate = gate; A.up = up; A.down = down;
  A.sh_gate = sh_gate; A.sh_up = sh_up; A.sh_down = sh_down;
  A.tgu = tgu; A.tdn = tdn; A.tsh = tsh;
  A.sh_logit = sh_logit;
  if (phase != 2) {
    dim3 grid((mid + GX_ROWS - 1) / GX_ROWS, nslots, P);
    k_ggx_gu<<<grid, 256, (size_t)d / 32 * 34 * 4, st>>>(A, x, ids, id_stride, kpt, d, mid, hid);
    MOE_LAUNCH_CHECK();
  }
  if (phase != 1) {
    dim3 grid((d + GX_DN_ROWS - 1) / GX_DN_ROWS, P);
    k_ggx_dn<<<grid, 256, (size_t)nslots * mid / 32 * 34 * 4, st>>>(A, hid, ids, ws, id_stride, kpt, d, mid, out);
    MOE_LAUNCH_CHECK();
  }
  return MOE_OK;
}
