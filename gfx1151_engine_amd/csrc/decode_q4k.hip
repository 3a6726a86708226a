// Decode (T <= 32) on raw GGUF Q4_K blocks read in place, integer dot products: the Q4_K twin of
// the q4cp decode kernels.  Unit of work = one 32-byte run of code bytes = 64 weights = two
// 32-element sub-blocks (low nibbles / high nibbles), each with its own 6-bit scale and min:
//   sum_k w_k x_k = d * (sc0 * qA * VA + sc1 * qB * VB) - dmin * (m0 * qA * SA + m1 * qB * SB)
// with V = integer dot product of the codes with the activation group's two 8-bit digit planes
// (natural element order) and q * S = the group's quantised sum.  A lane owns one unit of a row;
// rows of 3072 are 48 units (lanes 48..63 idle: the kernels are bandwidth-bound), rows of 768 are
// 12 units (four slots per wave).
// (reference: src/gpu/parts/26_kernels_moe_gguf.inc:527-568,693-756,893-939; src/gguf.h:328-336,408-441)
#include "common.h"
#include "internal.h"
#include "iq4.h"
#include "qvec.h"
#include "topk.h"

namespace {

__device__ __forceinline__ float dpp_add_row(float v) {  // sum over each row of 16 lanes, in every lane
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true));
  return v;
}
__device__ __forceinline__ float dpp_max_row(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, true)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, true)));
  return v;
}
__device__ __forceinline__ float sum64(float v) {
  return rows_total_add(dpp_add_row(v));
}

// activation planes of one unit: two groups (A = low nibbles, B = high nibbles)
struct XU {
  uint32_t a[2][8], b[2][8];
  float qa, qsa, qb, qsb;
};
__device__ __forceinline__ void load_xu(XU& x, const uint32_t* planes, const float2* meta, size_t g0) {
  const uint4* s = (const uint4*)(planes + g0 * QV_GROUP_DW);
#pragma unroll
  for (int p = 0; p < 2; p++) {
    const uint4 a0 = s[2 * p], a1 = s[2 * p + 1], b0 = s[4 + 2 * p], b1 = s[4 + 2 * p + 1];
    x.a[p][0] = a0.x; x.a[p][1] = a0.y; x.a[p][2] = a0.z; x.a[p][3] = a0.w;
    x.a[p][4] = a1.x; x.a[p][5] = a1.y; x.a[p][6] = a1.z; x.a[p][7] = a1.w;
    x.b[p][0] = b0.x; x.b[p][1] = b0.y; x.b[p][2] = b0.z; x.b[p][3] = b0.w;
    x.b[p][4] = b1.x; x.b[p][5] = b1.y; x.b[p][6] = b1.z; x.b[p][7] = b1.w;
  }
  const float2 ma = meta[g0], mb = meta[g0 + 1];
  x.qa = ma.x; x.qsa = ma.y; x.qb = mb.x; x.qsb = mb.y;
}

// gguf scale_min_k4 for sub-blocks 2jj and 2jj+1 of a super-block whose header words are hd
// (hd.x = d | dmin << 16, hd.y/z/w = the 12 packed bytes q[0..11]).  Sub-blocks j < 4 keep their
// 6-bit scale in q[j] and min in q[4+j]; j >= 4 keep 4 bits of each in q[4+j] and the top 2 bits in
// the upper bits of q[j-4] / q[j].  jj differs per lane, so both forms are one sequence of
// bit-field extracts whose source word and widths are per-lane values (a width of 0 extracts 0).
__device__ __forceinline__ void k4_pair(const uint4 hd, int jj, float& a0, float& b0, float& a1, float& b1) {
  union { uint32_t u; __half2 h; } dd;
  dd.u = hd.x;
  const float d = __low2float(dd.h), dmin = __high2float(dd.h);
  const bool lo = jj < 2;
  const uint32_t sh = 16u * (jj & 1), wid = lo ? 6u : 4u, wid2 = lo ? 0u : 2u;
  const uint32_t y = hd.y, z = hd.z, w = hd.w;
  const uint32_t A = lo ? y : w, B = lo ? z : w >> 4;
  const uint32_t sc0 = __builtin_amdgcn_ubfe(A, sh, wid) | (__builtin_amdgcn_ubfe(y, sh + 6, wid2) << 4);
  const uint32_t sc1 = __builtin_amdgcn_ubfe(A, sh + 8, wid) | (__builtin_amdgcn_ubfe(y, sh + 14, wid2) << 4);
  const uint32_t m0 = __builtin_amdgcn_ubfe(B, sh, wid) | (__builtin_amdgcn_ubfe(z, sh + 6, wid2) << 4);
  const uint32_t m1 = __builtin_amdgcn_ubfe(B, sh + 8, wid) | (__builtin_amdgcn_ubfe(z, sh + 14, wid2) << 4);
  a0 = d * (float)sc0;
  a1 = d * (float)sc1;
  b0 = dmin * (float)m0;
  b1 = dmin * (float)m1;
}

// The four lanes that work on one super-block (a quad: units 4b .. 4b+3) each load one dword of its 16-byte
// header and hand the others theirs when the row is computed: 1 register per row in flight instead of 4.
__device__ __forceinline__ uint4 quad_header(uint32_t mine) {
  uint4 hd;
  hd.x = (uint32_t)__builtin_amdgcn_mov_dpp((int)mine, 0x00, 0xf, 0xf, true);  // quad_perm [0,0,0,0]
  hd.y = (uint32_t)__builtin_amdgcn_mov_dpp((int)mine, 0x55, 0xf, 0xf, true);  // [1,1,1,1]
  hd.z = (uint32_t)__builtin_amdgcn_mov_dpp((int)mine, 0xAA, 0xf, 0xf, true);  // [2,2,2,2]
  hd.w = (uint32_t)__builtin_amdgcn_mov_dpp((int)mine, 0xFF, 0xf, 0xf, true);  // [3,3,3,3]
  return hd;
}

// one unit of one row: c0, c1 = its 32 code bytes, hd = the super-block header
__device__ __forceinline__ float unit_dot(const uint4 c0, const uint4 c1, const uint4 hd, int jj, const XU& x) {
  const uint32_t w[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
  int a0 = 0, a1 = 0, b0 = 0, b1 = 0;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int lo = (int)(w[i] & 0x0f0f0f0fu), hi = (int)((w[i] >> 4) & 0x0f0f0f0fu);
    a0 = __builtin_amdgcn_sdot4(lo, (int)x.a[0][i], a0, false);
    a1 = __builtin_amdgcn_sdot4(lo, (int)x.a[1][i], a1, false);
    b0 = __builtin_amdgcn_sdot4(hi, (int)x.b[0][i], b0, false);
    b1 = __builtin_amdgcn_sdot4(hi, (int)x.b[1][i], b1, false);
  }
  // |a0| <= 32 * 15 * 128: the integer sum stays below 2^24 and converts exactly
  const float va = (float)(a0 * 256 + a1);
  const float vb = (float)(b0 * 256 + b1);
  float sa, ma, sb, mb;
  k4_pair(hd, jj, sa, ma, sb, mb);
  return (sa * x.qa * va + sb * x.qb * vb) - (ma * x.qsa + mb * x.qsb);
}

struct Gu4kArgs {
  const uint8_t *gate, *up;        // routed experts [E][mid rows][d/256 blocks]
  const uint8_t *sh_gate, *sh_up;  // shared expert rows (nullptr: none)
};

// grid (mid/32, slots incl. shared, P); block 512.  Wave w: gate rows 4w..4w+3 and the matching up
// rows of this block's 32; lane = unit (d/64 <= 64 units per row).  All 24 loads of a lane (8 rows x
// two code halves + its dword of the header) are in flight together, in under 128 registers: two blocks fit
// a CU, so the grid's 265 blocks are all resident at once (with one block per CU the last nine waited for a
// second round).
// NPL > 0 (E <= 64*NPL): only the logits are given; the blocks of the routed slots run the softmax /
// top-k of their token themselves and block (0, 0, token) writes ids / weights out for the down
// kernel (as in the q4cp gate/up kernel).
constexpr int G4_ROWS = 32;
template <int NPL>
__global__ void __launch_bounds__(512, 4) k_dec4k_gu(Gu4kArgs A, const uint32_t* __restrict__ xplanes,
                                                     const float2* __restrict__ xmeta,
                                                     const int* __restrict__ ids, int id_stride, int kpt, int d,
                                                     int mid, uint32_t* __restrict__ hplanes,
                                                     float2* __restrict__ hmeta, const float* __restrict__ logits,
                                                     int n_experts, int* __restrict__ ids_out,
                                                     float* __restrict__ ws_out, moe_rfix RF) {
  __shared__ float gs[G4_ROWS], us[G4_ROWS];
  __shared__ uint32_t pk[QV_GROUP_DW];
  __shared__ int sel_ids[64];
  __shared__ float sel_ws[64];
  const int s = blockIdx.y, tok = blockIdx.z, nslots = gridDim.y - (NPL > 0 ? 1 : 0);
  if (NPL > 0 && s == nslots) {
    // one block of the extra grid row: the exact softmax / top-k (ids, renormalised weights) for the down
    // launch, next to the blocks that stream the weights and only need the ids
    if (blockIdx.x == 0) {
      select_certain<NPL ? NPL : 8, 512>(logits + (size_t)tok * n_experts, RF, (int)tok, sel_ids, sel_ws, n_experts, kpt, true);
      __syncthreads();
      if ((int)threadIdx.x < kpt) {
        ids_out[(size_t)tok * id_stride + threadIdx.x] = sel_ids[threadIdx.x];
        ws_out[(size_t)tok * id_stride + threadIdx.x] = sel_ws[threadIdx.x];
      }
    }
    return;
  }
  const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int U = d / 64;
  const bool shared = s >= kpt;
  const uint64_t rb = (uint64_t)(d / 256) * 144;
  int e = 0;
  if (NPL > 0) {
    if (!shared) {
      // the ids by logit order; the exact selection only when two of the best logits are too close
      const float* lg = logits + (size_t)tok * n_experts;
      if (!select_certain<NPL ? NPL : 8, 512>(lg, RF, (int)tok, sel_ids, sel_ws, n_experts, kpt, false)) __syncthreads();
      e = sel_ids[s];
    }
  } else if (!shared) {
    e = ids[(size_t)tok * id_stride + s];
  }
  e = __builtin_amdgcn_readfirstlane(e);  // (the same in every lane: as a scalar, the offsets below are scalar arithmetic)
  const uint8_t* gbase = shared ? A.sh_gate : A.gate + (uint64_t)e * mid * rb;
  const uint8_t* ubase = shared ? A.sh_up : A.up + (uint64_t)e * mid * rb;
  const int r0 = blockIdx.x * G4_ROWS + 4 * wv;
  // branch-free loads: lanes past the row's units read a unit of the first super-block (their quad then still
  // assembles a real header) and count as zero
  const bool live = lane < U;
  const int ul = live ? lane : (lane & 3);
  const float mlive = live ? 1.f : 0.f;
  const int jj = ul & 3;
  const size_t uoff = (size_t)(ul >> 2) * 144;  // this lane's super-block inside a row
  XU x;
  load_xu(x, xplanes, xmeta, ((size_t)tok * U + ul) * 2);
  uint4 c0[8], c1[8];
  uint32_t hw[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const uint8_t* row = (i < 4 ? gbase : ubase) + (uint64_t)(r0 + (i & 3)) * rb + uoff;
    hw[i] = *(const uint32_t*)(row + 4 * jj);
    c0[i] = *(const uint4*)(row + 16 + jj * 32);
    c1[i] = *(const uint4*)(row + 32 + jj * 32);
  }
  __builtin_amdgcn_sched_barrier(0);  // every load is issued before the first dot product
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    acc[i] = sum64(unit_dot(c0[i], c1[i], quad_header(hw[i]), jj, x) * mlive);
    if (i & 1) __builtin_amdgcn_sched_barrier(0);  // rows are consumed in arrival order
  }
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      gs[4 * wv + i] = acc[i];
      us[4 * wv + i] = acc[4 + i];
    }
  }
  __syncthreads();
  // SwiGLU on the block's 32 rows = one sub-block of the down projection's input; quantise it
  if (wv == 0) {
    const int j = lane & 31;
    const float g = gs[j], u = us[j];
    const float hv = g / (1.f + expf(-g)) * u;
    float m = dpp_max_row(fabsf(hv));
    m = rows_half_max(m);
    const float inv = m > 0.f ? QV_XMAX / m : 0.f;
    const float q = m * (1.f / QV_XMAX);
    const int X = (int)rintf(hv * inv);
    int p0, p1;
    qv_digits(X, p0, p1);
    float sx = dpp_add_row((float)X);
    sx = rows_half_add(sx);
    if (lane < QV_GROUP_DW) pk[lane] = 0;
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_wave_barrier();
    if (lane < 32) {
      const int dw = j >> 2, sh = 8 * (j & 3);  // natural order
      atomicOr(&pk[dw], (uint32_t)(p0 & 0xff) << sh);
      atomicOr(&pk[8 + dw], (uint32_t)(p1 & 0xff) << sh);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_wave_barrier();
    const size_t gi = ((size_t)tok * nslots + s) * (mid / 32) + blockIdx.x;
    if (lane < QV_GROUP_DW) hplanes[gi * QV_GROUP_DW + lane] = pk[lane];
    if (lane == 0) hmeta[gi] = make_float2(q, q * sx);
  }
}

struct Dn4kArgs {
  const uint8_t *down, *sh_down;  // [E][d rows][mid/256 blocks]; shared expert rows (nullptr: none)
  const float* sh_logit;
};

// grid (d/ROWS, P); block = 64 x ceil(slots/4).  A row of 16 lanes = one slot (mid/64 <= 16 units),
// holding that slot's hid planes in registers for all the block's rows.  The weighted combine runs
// afterwards in slot order (descending router probability), then the shared expert.
constexpr int D4_ROWS = 8, D4_MAXSLOTS = 16;
__global__ void __launch_bounds__(256) k_dec4k_dn(Dn4kArgs A, const uint32_t* __restrict__ hplanes,
                                                  const float2* __restrict__ hmeta, const int* __restrict__ ids,
                                                  const float* __restrict__ ws, int id_stride, int kpt, int d,
                                                  int mid, float* __restrict__ out, uint64_t out_stride) {
  __shared__ float part[D4_MAXSLOTS][D4_ROWS];
  __shared__ float wsm[D4_MAXSLOTS];
  const int tok = blockIdx.y;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const bool has_shared = A.sh_down != nullptr;
  const int nslots = kpt + (has_shared ? 1 : 0);
  const int U = mid / 64, u_raw = lane & 15, s_raw = 4 * wv + (lane >> 4);
  const int r0 = blockIdx.x * D4_ROWS;
  const uint64_t rb = (uint64_t)(mid / 256) * 144;
  // combine weights of the token, fetched while the weight rows are in flight
  float wmine = 0.f;
  if ((int)threadIdx.x < nslots)
    wmine = (int)threadIdx.x < kpt ? ws[(size_t)tok * id_stride + threadIdx.x] : A.sh_logit[tok];
  {
    // branch-free loads: lanes past the slots or the row's units read slot 0 / unit 0 and count as zero
    const bool live = s_raw < nslots && u_raw < U;
    const int s = live ? s_raw : 0, u = live ? u_raw : 0;
    const float mlive = live ? 1.f : 0.f;
    const bool shared = has_shared && s == nslots - 1;
    // (an unconditional load: under a per-lane branch the compiler waits for the id before it issues anything else)
    const int e_any = ids[tok * id_stride + (shared ? 0 : s)];
    const uint32_t e = shared ? 0u : (uint32_t)e_any;
    const uint8_t* base = (shared ? A.sh_down : A.down + (uint64_t)(e * (uint32_t)d) * rb) + (uint64_t)r0 * rb + (uint32_t)(u >> 2) * 144;
    const int jj = u & 3;
    XU x;
    load_xu(x, hplanes, hmeta, (((size_t)tok * nslots + s) * U + u) * 2);
    uint4 c0[D4_ROWS], c1[D4_ROWS], hd[D4_ROWS];
#pragma unroll
    for (int r = 0; r < D4_ROWS; r++) {
      const uint8_t* row = base + (uint64_t)r * rb;
      hd[r] = *(const uint4*)row;
      c0[r] = *(const uint4*)(row + 16 + jj * 32);
      c1[r] = *(const uint4*)(row + 32 + jj * 32);
    }
    __builtin_amdgcn_sched_barrier(0);  // every load is issued before the first dot product
#pragma unroll
    for (int r = 0; r < D4_ROWS; r++) {
      const float v = dpp_add_row(unit_dot(c0[r], c1[r], hd[r], jj, x) * mlive);
      if (u_raw == 0 && s_raw < nslots) part[s_raw][r] = v;
      if (r & 1) __builtin_amdgcn_sched_barrier(0);  // rows are consumed in arrival order
    }
  }
  if ((int)threadIdx.x < nslots) wsm[threadIdx.x] = (int)threadIdx.x < kpt ? wmine : sigmoid_f(wmine);
  __syncthreads();
  if (threadIdx.x < D4_ROWS) {
    const int r = threadIdx.x;
    float y = 0.f;
    for (int i = 0; i < kpt; i++) y += wsm[i] * part[i][r];
    if (has_shared) y += wsm[kpt] * part[kpt][r];
    out[(size_t)tok * out_stride + r0 + r] = y;
  }
}

// ---------------------------------------------------------------------------------------------------------------
// The same launches for the other block types of the reference's GGUF checkpoints (Q5_K gate/up, Q5_1 / Q8_0 down,
// a Q8_0 shared expert; src/gpu/parts/30_host_util.inc:399-405, src/gguf_map.h:212-214), any mix of them with Q4_K.
// A lane still owns one unit of 64 weights = two activation groups with their two 8-bit digit planes; what differs
// per type is what a unit's bytes are and how its integer sums are scaled:
//   Q5_K  (176 B / 256): Q4_K plus a fifth bit per code; unit jj of a super-block takes bits 2jj and 2jj+1 of the 32
//         qh bytes; the four lanes of the super-block load 8 qh bytes each and hand them round by DPP
//   Q8_0  (34 B / 32):   two blocks = 68 bytes starting on a 4-byte boundary: fp16 d, 32 int8 codes (2 bytes off the
//         dword grid in the first block: one v_alignbit per word), d, 32 codes; w = d q
//   Q5_1  (24 B / 32):   two blocks = 48 bytes: fp16 d, m, 32 fifth bits, 16 code bytes (low nibbles = elements
//         0..15, high nibbles = 16..31); w = d q + m
//   IQ4_NL (18 B / 32):  two blocks = 36 bytes from a 4-byte boundary: fp16 d, 16 code bytes (2 bytes off the dword
//         grid in the first block), d, 16 code bytes; w = d kv[n] with the 16-entry int8 table of src/gguf.h:376-379,
//         looked up four codes at a time with byte permutes (iq4.h): the table is four registers of constants
//   IQ4_XS (136 B / 256): fp16 d, 8 x 6-bit sub-block scales (scales_h, scales_l), 128 code bytes; a unit = the
//         8-byte header + the 32 code bytes of sub-blocks 2jj, 2jj+1; w = d (ls - 32) kv[n]
// The type of a block (gate/up launch: one slot) or of a wave (down launch: the shared expert has a wave of its
// own) is uniform, so it is one scalar branch outside the loads.  A wave's eight rows are fetched in two batches of
// four.
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

template <int T> struct GgU;
template <> struct GgU<MOE_GGML_Q4_K> { uint4 c0, c1; uint32_t hw; };
template <> struct GgU<MOE_GGML_Q5_K> { uint4 c0, c1; uint2 qh; uint32_t hw; };
template <> struct GgU<MOE_GGML_Q8_0> { uint32_t w[17]; };
template <> struct GgU<MOE_GGML_Q5_1> { uint4 a, b, c; };
template <> struct GgU<MOE_GGML_IQ4_NL> { uint32_t w[9]; };
template <> struct GgU<MOE_GGML_IQ4_XS> { uint2 hd; uint4 c0, c1; };

__host__ __device__ constexpr uint64_t ggu_row_bytes(int t, uint64_t k) {
  return t == MOE_GGML_Q4_K   ? k / 256 * 144
         : t == MOE_GGML_Q5_K ? k / 256 * 176
         : t == MOE_GGML_Q8_0 ? k / 32 * 34
         : t == MOE_GGML_IQ4_NL ? k / 32 * 18
         : t == MOE_GGML_IQ4_XS ? k / 256 * 136
                                : k / 32 * 24;
}

__device__ __forceinline__ int iq4_lookup4(uint32_t q, int shift) { return (int)moe_iq4_lookup4<0>(q, shift); }
// rows in flight together: four (eight Q4_K rows of nine registers spill next to the kernel's other state and measured
// 1.4 us slower per token than two batches of four)
template <int T> constexpr int ggu_batch() { return 4; }

template <int T>
__device__ __forceinline__ void ggu_fetch(const uint8_t* row, int ul, GgU<T>& o) {
  const int jj = ul & 3;
  if constexpr (T == MOE_GGML_Q4_K) {
    const uint8_t* sb = row + (size_t)(ul >> 2) * 144;
    o.hw = *(const uint32_t*)(sb + 4 * jj);
    o.c0 = *(const uint4*)(sb + 16 + jj * 32);
    o.c1 = *(const uint4*)(sb + 32 + jj * 32);
  } else if constexpr (T == MOE_GGML_Q5_K) {
    const uint8_t* sb = row + (size_t)(ul >> 2) * 176;
    o.hw = *(const uint32_t*)(sb + 4 * jj);
    o.qh = *(const uint2*)(sb + 16 + 8 * jj);
    o.c0 = *(const uint4*)(sb + 48 + jj * 32);
    o.c1 = *(const uint4*)(sb + 64 + jj * 32);
  } else if constexpr (T == MOE_GGML_Q8_0) {
    const uint8_t* p = row + (size_t)ul * 68;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const u32x4_a4 v = *(const u32x4_a4*)(p + 16 * i);
      o.w[4 * i] = v.x; o.w[4 * i + 1] = v.y; o.w[4 * i + 2] = v.z; o.w[4 * i + 3] = v.w;
    }
    o.w[16] = *(const uint32_t*)(p + 64);
  } else if constexpr (T == MOE_GGML_IQ4_NL) {
    const uint32_t* p = (const uint32_t*)(row + (size_t)ul * 36);
    const u32x4_a4 v0 = *(const u32x4_a4*)p, v1 = *(const u32x4_a4*)(p + 4);
    o.w[0] = v0.x; o.w[1] = v0.y; o.w[2] = v0.z; o.w[3] = v0.w;
    o.w[4] = v1.x; o.w[5] = v1.y; o.w[6] = v1.z; o.w[7] = v1.w;
    o.w[8] = p[8];
  } else if constexpr (T == MOE_GGML_IQ4_XS) {
    const uint8_t* sb = row + (size_t)(ul >> 2) * 136;
    o.hd = *(const uint2*)sb;
    const u32x4_a4 v0 = *(const u32x4_a4*)(sb + 8 + jj * 32), v1 = *(const u32x4_a4*)(sb + 24 + jj * 32);
    o.c0 = uint4{v0.x, v0.y, v0.z, v0.w};
    o.c1 = uint4{v1.x, v1.y, v1.z, v1.w};
  } else {
    const uint4* p = (const uint4*)(row + (size_t)ul * 48);
    o.a = p[0]; o.b = p[1]; o.c = p[2];
  }
}

// integer sum of a group against both digit planes -> float (the sums can exceed 2^24 for 5- and 8-bit codes: two
// exact conversions and one rounded fma instead of an integer combine)
__device__ __forceinline__ float planes_val(int hi, int lo) { return fmaf((float)hi, 256.f, (float)lo); }

template <int T>
__device__ __forceinline__ float ggu_dot(const GgU<T>& o, int jj, const XU& x) {
  if constexpr (T == MOE_GGML_Q4_K) {
    return unit_dot(o.c0, o.c1, quad_header(o.hw), jj, x);
  } else if constexpr (T == MOE_GGML_Q5_K) {
    const uint4 hd = quad_header(o.hw);
    const uint32_t w[8] = {o.c0.x, o.c0.y, o.c0.z, o.c0.w, o.c1.x, o.c1.y, o.c1.z, o.c1.w};
    // qh word i (bytes 4i..4i+3) sits in lane i/2 of the quad, register i%2
    uint32_t qh[8];
    qh[0] = (uint32_t)__builtin_amdgcn_mov_dpp((int)o.qh.x, 0x00, 0xf, 0xf, true);
    qh[1] = (uint32_t)__builtin_amdgcn_mov_dpp((int)o.qh.y, 0x00, 0xf, 0xf, true);
    qh[2] = (uint32_t)__builtin_amdgcn_mov_dpp((int)o.qh.x, 0x55, 0xf, 0xf, true);
    qh[3] = (uint32_t)__builtin_amdgcn_mov_dpp((int)o.qh.y, 0x55, 0xf, 0xf, true);
    qh[4] = (uint32_t)__builtin_amdgcn_mov_dpp((int)o.qh.x, 0xAA, 0xf, 0xf, true);
    qh[5] = (uint32_t)__builtin_amdgcn_mov_dpp((int)o.qh.y, 0xAA, 0xf, 0xf, true);
    qh[6] = (uint32_t)__builtin_amdgcn_mov_dpp((int)o.qh.x, 0xFF, 0xf, 0xf, true);
    qh[7] = (uint32_t)__builtin_amdgcn_mov_dpp((int)o.qh.y, 0xFF, 0xf, 0xf, true);
    int a0 = 0, a1 = 0, b0 = 0, b1 = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const uint32_t hb = qh[i] >> (2 * jj);
      const int lo = (int)((w[i] & 0x0f0f0f0fu) | ((hb & 0x01010101u) << 4));
      const int hi = (int)(((w[i] >> 4) & 0x0f0f0f0fu) | (((hb >> 1) & 0x01010101u) << 4));
      a0 = __builtin_amdgcn_sdot4(lo, (int)x.a[0][i], a0, false);
      a1 = __builtin_amdgcn_sdot4(lo, (int)x.a[1][i], a1, false);
      b0 = __builtin_amdgcn_sdot4(hi, (int)x.b[0][i], b0, false);
      b1 = __builtin_amdgcn_sdot4(hi, (int)x.b[1][i], b1, false);
    }
    float sa, ma, sb, mb;
    k4_pair(hd, jj, sa, ma, sb, mb);
    return (sa * x.qa * planes_val(a0, a1) + sb * x.qb * planes_val(b0, b1)) - (ma * x.qsa + mb * x.qsb);
  } else if constexpr (T == MOE_GGML_Q8_0) {
    int a0 = 0, a1 = 0, b0 = 0, b1 = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int ca = (int)__builtin_amdgcn_alignbit(o.w[i + 1], o.w[i], 16);  // the first block's codes: 2 bytes off the dword grid
      const int cb = (int)o.w[9 + i];
      a0 = __builtin_amdgcn_sdot4(ca, (int)x.a[0][i], a0, false);
      a1 = __builtin_amdgcn_sdot4(ca, (int)x.a[1][i], a1, false);
      b0 = __builtin_amdgcn_sdot4(cb, (int)x.b[0][i], b0, false);
      b1 = __builtin_amdgcn_sdot4(cb, (int)x.b[1][i], b1, false);
    }
    union { uint16_t u; __half h; } d0, d1;
    d0.u = (uint16_t)(o.w[0] & 0xffffu);
    d1.u = (uint16_t)(o.w[8] >> 16);
    return __half2float(d0.h) * x.qa * planes_val(a0, a1) + __half2float(d1.h) * x.qb * planes_val(b0, b1);
  } else if constexpr (T == MOE_GGML_IQ4_NL || T == MOE_GGML_IQ4_XS) {
    uint32_t qa[4], qb[4];  // the 16 code bytes of the unit's two 32-element blocks
    float da, db;           // their scales
    if constexpr (T == MOE_GGML_IQ4_NL) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        qa[i] = __builtin_amdgcn_alignbit(o.w[i + 1], o.w[i], 16);  // the first block's codes: 2 bytes off the dword grid
        qb[i] = o.w[5 + i];
      }
      union { uint16_t u; __half h; } d0, d1;
      d0.u = (uint16_t)(o.w[0] & 0xffffu);
      d1.u = (uint16_t)(o.w[4] >> 16);
      da = __half2float(d0.h);
      db = __half2float(d1.h);
    } else {
      qa[0] = o.c0.x; qa[1] = o.c0.y; qa[2] = o.c0.z; qa[3] = o.c0.w;
      qb[0] = o.c1.x; qb[1] = o.c1.y; qb[2] = o.c1.z; qb[3] = o.c1.w;
      // sub-blocks 2jj, 2jj+1: 6-bit scales = a nibble of scales_l[jj] | two bits of scales_h << 4, minus 32
      union { uint16_t u; __half h; } dv;
      dv.u = (uint16_t)(o.hd.x & 0xffffu);
      const uint32_t sh = o.hd.x >> 16, sl = (o.hd.y >> (8 * jj)) & 0xffu;
      const int la = (int)((sl & 0xfu) | (((sh >> (4 * jj)) & 3u) << 4)) - 32;
      const int lb = (int)((sl >> 4) | (((sh >> (4 * jj + 2)) & 3u) << 4)) - 32;
      const float dd = __half2float(dv.h);
      da = dd * (float)la;
      db = dd * (float)lb;
    }
    int a0 = 0, a1 = 0, b0 = 0, b1 = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int al = iq4_lookup4(qa[i], 0), ah = iq4_lookup4(qa[i], 4);
      const int bl = iq4_lookup4(qb[i], 0), bh = iq4_lookup4(qb[i], 4);
      a0 = __builtin_amdgcn_sdot4(al, (int)x.a[0][i], a0, false);
      a1 = __builtin_amdgcn_sdot4(al, (int)x.a[1][i], a1, false);
      a0 = __builtin_amdgcn_sdot4(ah, (int)x.a[0][4 + i], a0, false);
      a1 = __builtin_amdgcn_sdot4(ah, (int)x.a[1][4 + i], a1, false);
      b0 = __builtin_amdgcn_sdot4(bl, (int)x.b[0][i], b0, false);
      b1 = __builtin_amdgcn_sdot4(bl, (int)x.b[1][i], b1, false);
      b0 = __builtin_amdgcn_sdot4(bh, (int)x.b[0][4 + i], b0, false);
      b1 = __builtin_amdgcn_sdot4(bh, (int)x.b[1][4 + i], b1, false);
    }
    return da * x.qa * planes_val(a0, a1) + db * x.qb * planes_val(b0, b1);
  } else {  // Q5_1
    const uint32_t dw[12] = {o.a.x, o.a.y, o.a.z, o.a.w, o.b.x, o.b.y, o.b.z, o.b.w, o.c.x, o.c.y, o.c.z, o.c.w};
    float r = 0.f;
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
      const uint32_t dm = dw[6 * blk], qh = dw[6 * blk + 1];
      int v0 = 0, v1 = 0;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t q = dw[6 * blk + 2 + i];
        // four bits of qh -> bit 4 of four bytes
        const uint32_t hl = ((((qh >> (4 * i)) & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
        const uint32_t hh = ((((qh >> (16 + 4 * i)) & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
        const int lo = (int)((q & 0x0f0f0f0fu) | hl), hi = (int)(((q >> 4) & 0x0f0f0f0fu) | hh);
        const uint32_t* p0 = blk ? x.b[0] : x.a[0];
        const uint32_t* p1 = blk ? x.b[1] : x.a[1];
        v0 = __builtin_amdgcn_sdot4(lo, (int)p0[i], v0, false);
        v1 = __builtin_amdgcn_sdot4(lo, (int)p1[i], v1, false);
        v0 = __builtin_amdgcn_sdot4(hi, (int)p0[4 + i], v0, false);
        v1 = __builtin_amdgcn_sdot4(hi, (int)p1[4 + i], v1, false);
      }
      union { uint32_t u; __half2 h; } cv;
      cv.u = dm;
      r += __low2float(cv.h) * (blk ? x.qb : x.qa) * planes_val(v0, v1) + __high2float(cv.h) * (blk ? x.qsb : x.qsa);
    }
    return r;
  }
}

// eight rows of one wave (gate/up launch: four gate rows and the matching up rows): acc[i] = wave sum of row i
template <int T>
__device__ __forceinline__ void ggu_gu_rows(const uint8_t* gbase, const uint8_t* ubase, int r0, int d, int ul,
                                            float mlive, const XU& x, float (&acc)[8]) {
  constexpr int RB = ggu_batch<T>();
  const uint64_t rb = ggu_row_bytes(T, (uint64_t)d);
  const int jj = ul & 3;
#pragma unroll
  for (int h = 0; h < 8; h += RB) {
    GgU<T> u[RB];
#pragma unroll
    for (int i = 0; i < RB; i++)
      ggu_fetch<T>(((i + h) < 4 ? gbase : ubase) + (uint64_t)(r0 + ((i + h) & 3)) * rb, ul, u[i]);
    __builtin_amdgcn_sched_barrier(0);  // every load of the batch is issued before the first dot product
#pragma unroll
    for (int i = 0; i < RB; i++) {
      acc[i + h] = sum64(ggu_dot<T>(u[i], jj, x) * mlive);
      if (i & 1) __builtin_amdgcn_sched_barrier(0);  // rows are consumed in arrival order
    }
  }
}

#define GGU_SWITCH(t, CALL)                                                       \
  switch (t) {                                                                    \
    case MOE_GGML_Q4_K: { constexpr int T = MOE_GGML_Q4_K; CALL; } break;          \
    case MOE_GGML_Q5_K: { constexpr int T = MOE_GGML_Q5_K; CALL; } break;          \
    case MOE_GGML_Q8_0: { constexpr int T = MOE_GGML_Q8_0; CALL; } break;          \
    case MOE_GGML_IQ4_NL: { constexpr int T = MOE_GGML_IQ4_NL; CALL; } break;      \
    case MOE_GGML_IQ4_XS: { constexpr int T = MOE_GGML_IQ4_XS; CALL; } break;      \
    default: { constexpr int T = MOE_GGML_Q5_1; CALL; } break;                    \
  }

struct GuGgArgs {
  const uint8_t *gate, *up, *sh_gate, *sh_up;
  int tgu, tsh;
};

// grid (mid/32, slots incl. shared + the exact top-k row, P); block 512: k_dec4k_gu<NPL> for any of the four types
template <int NPL>
__global__ void __launch_bounds__(512, 4) k_decgg_gu(GuGgArgs A, const uint32_t* __restrict__ xplanes,
                                                     const float2* __restrict__ xmeta, int id_stride, int kpt, int d,
                                                     int mid, uint32_t* __restrict__ hplanes,
                                                     float2* __restrict__ hmeta, const float* __restrict__ logits,
                                                     int n_experts, int* __restrict__ ids_out,
                                                     float* __restrict__ ws_out, const int* __restrict__ ids_in, moe_rfix RF) {
  __shared__ float gs[G4_ROWS], us[G4_ROWS];
  __shared__ uint32_t pk[QV_GROUP_DW];
  __shared__ int sel_ids[64];
  __shared__ float sel_ws[64];
  const int s = blockIdx.y, tok = blockIdx.z, nslots = gridDim.y - (NPL > 0 ? 1 : 0);
  if (NPL > 0 && s == nslots) {  // the extra grid row: exact softmax / top-k for the down launch
    if (blockIdx.x == 0) {
      select_certain<NPL ? NPL : 8, 512>(logits + (size_t)tok * n_experts, RF, (int)tok, sel_ids, sel_ws, n_experts, kpt, true);
      __syncthreads();
      if ((int)threadIdx.x < kpt) {
        ids_out[(size_t)tok * id_stride + threadIdx.x] = sel_ids[threadIdx.x];
        ws_out[(size_t)tok * id_stride + threadIdx.x] = sel_ws[threadIdx.x];
      }
    }
    return;
  }
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int U = d / 64;
  const bool shared = s >= kpt;
  int e = 0;
  if (!shared) {
    if (NPL > 0) {
      const float* lg = logits + (size_t)tok * n_experts;
      if (!select_certain<NPL ? NPL : 8, 512>(lg, RF, (int)tok, sel_ids, sel_ws, n_experts, kpt, false)) __syncthreads();
      e = sel_ids[s];
    } else {
      e = ids_in[(size_t)tok * id_stride + s];  // (NPL == 0: the ids come from the router's launches)
    }
  }
  e = __builtin_amdgcn_readfirstlane(e);  // (the same in every lane: as a scalar, the offsets below are scalar arithmetic)
  const int t = shared ? A.tsh : A.tgu;
  const uint64_t rb = ggu_row_bytes(t, (uint64_t)d);
  const uint8_t* gbase = shared ? A.sh_gate : A.gate + (uint64_t)e * mid * rb;
  const uint8_t* ubase = shared ? A.sh_up : A.up + (uint64_t)e * mid * rb;
  const int r0 = blockIdx.x * G4_ROWS + 4 * wv;
  const bool live = lane < U;
  const int ul = live ? lane : (lane & 3);
  const float mlive = live ? 1.f : 0.f;
  XU x;
  load_xu(x, xplanes, xmeta, ((size_t)tok * U + ul) * 2);
  float acc[8];
  GGU_SWITCH(t, ggu_gu_rows<T>(gbase, ubase, r0, d, ul, mlive, x, acc));
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      gs[4 * wv + i] = acc[i];
      us[4 * wv + i] = acc[4 + i];
    }
  }
  __syncthreads();
  if (wv == 0) {  // SwiGLU on the block's 32 rows = one activation group of the down projection; quantise it
    const int j = lane & 31;
    const float g = gs[j], u = us[j];
    const float hv = g / (1.f + expf(-g)) * u;
    float m = dpp_max_row(fabsf(hv));
    m = rows_half_max(m);
    const float inv = m > 0.f ? QV_XMAX / m : 0.f;
    const float q = m * (1.f / QV_XMAX);
    const int X = (int)rintf(hv * inv);
    int p0, p1;
    qv_digits(X, p0, p1);
    float sx = dpp_add_row((float)X);
    sx = rows_half_add(sx);
    if (lane < QV_GROUP_DW) pk[lane] = 0;
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_wave_barrier();
    if (lane < 32) {
      const int dw = j >> 2, sh = 8 * (j & 3);
      atomicOr(&pk[dw], (uint32_t)(p0 & 0xff) << sh);
      atomicOr(&pk[8 + dw], (uint32_t)(p1 & 0xff) << sh);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_wave_barrier();
    const size_t gi = ((size_t)tok * nslots + s) * (mid / 32) + blockIdx.x;
    if (lane < QV_GROUP_DW) hplanes[gi * QV_GROUP_DW + lane] = pk[lane];
    if (lane == 0) hmeta[gi] = make_float2(q, q * sx);
  }
}

struct DnGgArgs {
  const uint8_t *down, *sh_down;
  const float* sh_logit;
  int tdn, tsh;
};

// D4_ROWS output rows of one wave's slots: a row of 16 lanes = one slot
template <int T>
__device__ __forceinline__ void ggu_dn_rows(const uint8_t* base, int mid, int ul, float mlive, const XU& x, bool store,
                                            float* part_s) {
  constexpr int RB = ggu_batch<T>();
  const uint64_t rb = ggu_row_bytes(T, (uint64_t)mid);
  const int jj = ul & 3;
#pragma unroll
  for (int h = 0; h < D4_ROWS; h += RB) {
    GgU<T> u[RB];
#pragma unroll
    for (int r = 0; r < RB; r++) ggu_fetch<T>(base + (uint64_t)(h + r) * rb, ul, u[r]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < RB; r++) {
      const float v = dpp_add_row(ggu_dot<T>(u[r], jj, x) * mlive);
      if (store) part_s[h + r] = v;
      if (r & 1) __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// grid (d/D4_ROWS, P); block = 64 x (ceil(kpt/4) + 1 with a shared expert): waves 0.. hold four routed slots each (a row
// of 16 lanes per slot), the last wave the shared expert alone, so that a wave's block type is uniform.
__global__ void __launch_bounds__(320) k_decgg_dn(DnGgArgs A, const uint32_t* __restrict__ hplanes,
                                                  const float2* __restrict__ hmeta, const int* __restrict__ ids,
                                                  const float* __restrict__ ws, int id_stride, int kpt, int d, int mid,
                                                  float* __restrict__ out, uint64_t out_stride) {
  __shared__ float part[D4_MAXSLOTS + 1][D4_ROWS];
  __shared__ float wsm[D4_MAXSLOTS + 1];
  const int tok = blockIdx.y;
  const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const bool has_shared = A.sh_down != nullptr;
  const int nslots = kpt + (has_shared ? 1 : 0), rw = (kpt + 3) >> 2;  // rw: waves of routed slots
  const int U = mid / 64, u_raw = lane & 15;
  const int r0 = blockIdx.x * D4_ROWS;
  float wmine = 0.f;
  if ((int)threadIdx.x < nslots)
    wmine = (int)threadIdx.x < kpt ? ws[(size_t)tok * id_stride + threadIdx.x] : A.sh_logit[tok];
  {
    const bool shw = wv >= rw;  // the shared expert's wave (its slot in lanes 0..15)
    const int s_raw = shw ? kpt + (lane >> 4) * D4_MAXSLOTS : 4 * wv + (lane >> 4);  // lanes 16.. of that wave: no slot
    const bool okslot = shw ? (lane >> 4) == 0 : s_raw < kpt;
    const bool live = okslot && u_raw < U;
    const int s = okslot ? s_raw : (shw ? kpt : 0);
    const int ul = u_raw < U ? u_raw : (u_raw & 3);
    const float mlive = live ? 1.f : 0.f;
    const int t = shw ? A.tsh : A.tdn;
    const uint64_t rb = ggu_row_bytes(t, (uint64_t)mid);
    // (an unconditional load: under a per-lane branch the compiler waits for the id before it issues anything else)
    const int e_any = ids[tok * id_stride + (shw ? 0 : s)];
    const uint32_t e = shw ? 0u : (uint32_t)e_any;
    const uint8_t* base = (shw ? A.sh_down : A.down + (uint64_t)(e * (uint32_t)d) * rb) + (uint64_t)r0 * rb;
    XU x;
    load_xu(x, hplanes, hmeta, (((size_t)tok * nslots + s) * U + ul) * 2);
    GGU_SWITCH(t, ggu_dn_rows<T>(base, mid, ul, mlive, x, u_raw == 0 && okslot, part[s]));
  }
  if ((int)threadIdx.x < nslots) wsm[threadIdx.x] = (int)threadIdx.x < kpt ? wmine : sigmoid_f(wmine);
  __syncthreads();
  if (threadIdx.x < D4_ROWS) {
    const int r = threadIdx.x;
    float y = 0.f;
    for (int i = 0; i < kpt; i++) y += wsm[i] * part[i][r];
    if (has_shared) y += wsm[kpt] * part[kpt][r];
    out[(size_t)tok * out_stride + r0 + r] = y;
  }
}

// ---- distinct experts of a small batch (verify-size batches: tokens share experts) ----
// The expert-sorted pair lists of the routing permutation, cut into tiles of at most GGQ_PAIRS pairs of one expert
// (the shared expert: expert id >= n_experts, over all tokens): a block fetches its weight rows once and walks the
// tile's pairs, so every distinct expert's bytes are read once per batch instead of once per token
// (reference: the _uq kernels, src/gpu/parts/26_kernels_moe_gguf.inc:758-886).
constexpr int GGQ_PAIRS = 4;  // pairs per tile (the tile lists are built with this cap)
// rows fetched together: two (with a pair's activation planes next to them the kernels stay under 128 registers,
// two blocks per CU; four rows spill)
template <int T>
__device__ __host__ constexpr int ggq_batch() { return T == MOE_GGML_Q8_0 ? 4 : 8; }
template <int T>
__device__ __host__ constexpr int ggq_dn_batch() { return T == MOE_GGML_Q8_0 ? 2 : 4; }
constexpr int GGQ_DR = 4, GGQ_DROWS = 16 * GGQ_DR;  // down: output rows per row of 16 lanes, per block

// eight rows of one wave in batches of GGQ_RB, each batch against every pair of the tile; gs / us: [pair][32] rows of
// the block in LDS, already offset to this wave's four
template <int T>
__device__ __forceinline__ void ggq_gu_rows(const uint8_t* gbase, const uint8_t* ubase, int r0, uint64_t rb, int ul, int jj,
                                            float mlive, const uint32_t* __restrict__ xplanes,
                                            const float2* __restrict__ xmeta, const int (&toks)[GGQ_PAIRS], int npairs,
                                            int U, bool writer, float* gs, float* us) {
  constexpr int RB = ggq_batch<T>();
#pragma unroll
  for (int h = 0; h < 8; h += RB) {
    GgU<T> u[RB];
#pragma unroll
    for (int i = 0; i < RB; i++)
      ggu_fetch<T>(((i + h) < 4 ? gbase : ubase) + (uint64_t)(r0 + ((i + h) & 3)) * rb, ul, u[i]);
    __builtin_amdgcn_sched_barrier(0);  // every load of the batch is issued before the first dot product
#pragma unroll 1
    for (int pi = 0; pi < npairs; pi++) {
      XU x;
      load_xu(x, xplanes, xmeta, ((size_t)toks[pi] * U + ul) * 2);
#pragma unroll
      for (int i = 0; i < RB; i++) {
        const float v = sum64(ggu_dot<T>(u[i], jj, x) * mlive);
        if (writer) {
          if (i + h < 4) gs[pi * G4_ROWS + i + h] = v;
          else us[pi * G4_ROWS + i + h - 4] = v;
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);  // the next batch's loads stay behind this batch's pairs
  }
}

// GGQ_DR output rows of one row of 16 lanes against every pair of the tile; out: pairs + first pair's row + r0
template <int T>
__device__ __forceinline__ void ggq_dn_rows(const uint8_t* base, uint64_t rb, int ul, int jj, float mlive,
                                            const uint32_t* __restrict__ hplanes, const float2* __restrict__ hmeta,
                                            size_t first, int npairs, int U, bool writer, float* out, int d);

// gate/up: grid (mid/32, tiles), block 512 (wave w: gate rows 4w..4w+3 and the matching up rows of the block's 32);
// hid planes go out by pair position, [pair][mid/32 groups]
__global__ void __launch_bounds__(512, 2) k_decgg_gu_uq(GuGgArgs A, const uint32_t* __restrict__ xplanes,
                                                        const float2* __restrict__ xmeta,
                                                        const moe_tile* __restrict__ tiles,
                                                        const int* __restrict__ ntiles, const int* __restrict__ tokidx,
                                                        int n_experts, int d, int mid, uint32_t* __restrict__ hplanes,
                                                        float2* __restrict__ hmeta) {
  __shared__ float gs[GGQ_PAIRS][G4_ROWS], us[GGQ_PAIRS][G4_ROWS];
  __shared__ uint32_t pk[GGQ_PAIRS][QV_GROUP_DW];
  if ((int)blockIdx.y >= ntiles[0]) return;
  const moe_tile tile = tiles[blockIdx.y];
  const bool shared = tile.expert >= n_experts;
  const int npairs = tile.count < GGQ_PAIRS ? tile.count : GGQ_PAIRS;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int U = d / 64;
  const int t = shared ? A.tsh : A.tgu;
  const uint64_t rb = ggu_row_bytes(t, (uint64_t)d);
  const uint8_t* gbase = shared ? A.sh_gate : A.gate + (uint64_t)tile.expert * mid * rb;
  const uint8_t* ubase = shared ? A.sh_up : A.up + (uint64_t)tile.expert * mid * rb;
  const int r0 = blockIdx.x * G4_ROWS + 4 * wv;
  const bool live = lane < U;
  const int ul = live ? lane : (lane & 3);
  const float mlive = live ? 1.f : 0.f;
  const int jj = ul & 3;
  int toks[GGQ_PAIRS];
#pragma unroll
  for (int pi = 0; pi < GGQ_PAIRS; pi++) toks[pi] = tokidx[tile.first + (pi < npairs ? pi : 0)];
  GGU_SWITCH(t, ggq_gu_rows<T>(gbase, ubase, r0, rb, ul, jj, mlive, xplanes, xmeta, toks, npairs, U, lane == 0,
                               &gs[0][4 * wv], &us[0][4 * wv]));
  __syncthreads();
  if (wv < npairs) {  // wave pi: SwiGLU on pair pi's 32 rows = one activation group of the down projection; quantise it
    const int j = lane & 31;
    const float g = gs[wv][j], u = us[wv][j];
    const float hv = g / (1.f + expf(-g)) * u;
    float m = dpp_max_row(fabsf(hv));
    m = rows_half_max(m);
    const float inv = m > 0.f ? QV_XMAX / m : 0.f;
    const float q = m * (1.f / QV_XMAX);
    const int X = (int)rintf(hv * inv);
    int p0, p1;
    qv_digits(X, p0, p1);
    float sx = dpp_add_row((float)X);
    sx = rows_half_add(sx);
    if (lane < QV_GROUP_DW) pk[wv][lane] = 0;
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_wave_barrier();
    if (lane < 32) {
      const int dw = j >> 2, sh = 8 * (j & 3);
      atomicOr(&pk[wv][dw], (uint32_t)(p0 & 0xff) << sh);
      atomicOr(&pk[wv][8 + dw], (uint32_t)(p1 & 0xff) << sh);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_wave_barrier();
    const size_t gi = (size_t)(tile.first + wv) * (mid / 32) + blockIdx.x;
    if (lane < QV_GROUP_DW) hplanes[gi * QV_GROUP_DW + lane] = pk[wv][lane];
    if (lane == 0) hmeta[gi] = make_float2(q, q * sx);
  }
}

// down: grid (d/GGQ_DROWS, tiles), block 256 = 16 rows of 16 lanes, each with GGQ_DR output rows; the unweighted row
// results go to pairs[pair][row] (f32) for the weighted combine that follows
template <int T>
__device__ __forceinline__ void ggq_dn_rows(const uint8_t* base, uint64_t rb, int ul, int jj, float mlive,
                                            const uint32_t* __restrict__ hplanes, const float2* __restrict__ hmeta,
                                            size_t first, int npairs, int U, bool writer, float* out, int d) {
  constexpr int RB = ggq_dn_batch<T>();
#pragma unroll
  for (int h = 0; h < GGQ_DR; h += RB) {
    GgU<T> u[RB];
#pragma unroll
    for (int r = 0; r < RB; r++) ggu_fetch<T>(base + (uint64_t)(h + r) * rb, ul, u[r]);
    __builtin_amdgcn_sched_barrier(0);
    for (int pi = 0; pi < npairs; pi++) {
      XU x;
      load_xu(x, hplanes, hmeta, ((first + pi) * U + ul) * 2);
#pragma unroll
      for (int r = 0; r < RB; r++) {
        const float v = dpp_add_row(ggu_dot<T>(u[r], jj, x) * mlive);
        if (writer) out[(size_t)pi * d + h + r] = v;
      }
    }
  }
}

__global__ void __launch_bounds__(256) k_decgg_dn_uq(DnGgArgs A, const uint32_t* __restrict__ hplanes,
                                                     const float2* __restrict__ hmeta,
                                                     const moe_tile* __restrict__ tiles, const int* __restrict__ ntiles,
                                                     int n_experts, int d, int mid, float* __restrict__ pairs) {
  if ((int)blockIdx.y >= ntiles[0]) return;
  const moe_tile tile = tiles[blockIdx.y];
  const bool shared = tile.expert >= n_experts;
  const int npairs = tile.count < GGQ_PAIRS ? tile.count : GGQ_PAIRS;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int U = mid / 64, u_raw = lane & 15;
  const bool live = u_raw < U;
  const int ul = live ? u_raw : (u_raw & 3);
  const float mlive = live ? 1.f : 0.f;
  const int jj = ul & 3;
  const int t = shared ? A.tsh : A.tdn;
  const uint64_t rb = ggu_row_bytes(t, (uint64_t)mid);
  const int r0 = blockIdx.x * GGQ_DROWS + (4 * wv + (lane >> 4)) * GGQ_DR;
  const uint8_t* base = (shared ? A.sh_down : A.down + (uint64_t)tile.expert * d * rb) + (uint64_t)r0 * rb;
  GGU_SWITCH(t, ggq_dn_rows<T>(base, rb, ul, jj, mlive, hplanes, hmeta, (size_t)tile.first, npairs, U, u_raw == 0,
                               pairs + (size_t)tile.first * d + r0, d));
}

}  // namespace

bool moe_dec4k_supported(int d, int mid, int nslots) {
  return d % 256 == 0 && d / 64 <= 64 && mid % 256 == 0 && mid / 64 <= 16 && nslots <= D4_MAXSLOTS &&
         mid % G4_ROWS == 0 && d % D4_ROWS == 0;
}

int moe_launch_dec4k_gu(const uint8_t* gate, const uint8_t* up, const uint8_t* sh_gate, const uint8_t* sh_up,
                        const uint32_t* xplanes, const float2* xmeta, const int* ids, int id_stride, int kpt,
                        int P, int d, int mid, uint32_t* hplanes, float2* hmeta, hipStream_t st) {
  if (!gate || !up || !xplanes || !xmeta || !ids || !hplanes || !hmeta) return MOE_E_INVALID;
  if (!moe_aligned(gate, 16) || !moe_aligned(up, 16) || (sh_gate && (!sh_up || !moe_aligned(sh_gate, 16) || !moe_aligned(sh_up, 16))))
    return MOE_E_INVALID;
  Gu4kArgs A{gate, up, sh_gate, sh_up};
  dim3 grid(mid / G4_ROWS, kpt + (sh_gate ? 1 : 0), P);
  k_dec4k_gu<0><<<grid, 512, 0, st>>>(A, xplanes, xmeta, ids, id_stride, kpt, d, mid, hplanes, hmeta, nullptr, 0,
                                      nullptr, nullptr, moe_rfix{});
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// The same with the softmax / top-k of every token done inside the launch: logits [P][n_experts] in,
// ids / ws rows (id_stride wide) out.
int moe_launch_dec4k_gu_topk(const uint8_t* gate, const uint8_t* up, const uint8_t* sh_gate, const uint8_t* sh_up,
                             const uint32_t* xplanes, const float2* xmeta, const float* logits, int n_experts,
                             int* ids, float* ws, int id_stride, int kpt, int P, int d, int mid,
                             uint32_t* hplanes, float2* hmeta, hipStream_t st, const moe_rfix* rf) {
  const moe_rfix RFV = rf ? *rf : moe_rfix{};
  if (!gate || !up || !xplanes || !xmeta || !logits || !ids || !ws || !hplanes || !hmeta || (!sh_gate != !sh_up))
    return MOE_E_INVALID;
  if (!moe_aligned(gate, 16) || !moe_aligned(up, 16) || (sh_gate && (!moe_aligned(sh_gate, 16) || !moe_aligned(sh_up, 16))))
    return MOE_E_INVALID;
  Gu4kArgs A{gate, up, sh_gate, sh_up};
  dim3 grid(mid / G4_ROWS, kpt + (sh_gate ? 1 : 0) + 1, P);  // + the row of the exact top-k block
  if (n_experts <= 512)
    k_dec4k_gu<8><<<grid, 512, 0, st>>>(A, xplanes, xmeta, nullptr, id_stride, kpt, d, mid, hplanes, hmeta, logits,
                                        n_experts, ids, ws, RFV);
  else
    k_dec4k_gu<16><<<grid, 512, 0, st>>>(A, xplanes, xmeta, nullptr, id_stride, kpt, d, mid, hplanes, hmeta, logits,
                                         n_experts, ids, ws, RFV);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_dec4k_dn(const uint8_t* down, const uint8_t* sh_down, const float* sh_logit,
                        const uint32_t* hplanes, const float2* hmeta, const int* ids, const float* ws,
                        int id_stride, int kpt, int P, int d, int mid, float* out, uint64_t out_stride,
                        hipStream_t st) {
  if (!down || !hplanes || !hmeta || !ids || !ws || !out || (sh_down && !sh_logit)) return MOE_E_INVALID;
  if (!moe_aligned(down, 16) || (sh_down && !moe_aligned(sh_down, 16))) return MOE_E_INVALID;
  Dn4kArgs A{down, sh_down, sh_logit};
  const int nslots = kpt + (sh_down ? 1 : 0);
  dim3 grid(d / D4_ROWS, P);
  k_dec4k_dn<<<grid, 64 * ((nslots + 3) / 4), 0, st>>>(A, hplanes, hmeta, ids, ws, id_stride, kpt, d, mid, out, out_stride);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// ---- any mix of Q4_K / Q5_K / Q8_0 / Q5_1 / IQ4_NL / IQ4_XS (integer-dot kernels above) ----
static bool ggu_type(int t) {
  return t == MOE_GGML_Q4_K || t == MOE_GGML_Q5_K || t == MOE_GGML_Q8_0 || t == MOE_GGML_Q5_1 || t == MOE_GGML_IQ4_NL ||
         t == MOE_GGML_IQ4_XS;
}
bool moe_decgg_supported(int tgu, int tdn, int tsh, bool has_shared, int d, int mid, int kpt, int n_experts) {
  if (!ggu_type(tgu) || !ggu_type(tdn) || (has_shared && !ggu_type(tsh))) return false;
  // (whole 256-element super-blocks in both directions also cover the 64-weight units of the 32-element types)
  return d % 256 == 0 && d / 64 <= 64 && mid % 256 == 0 && mid / 64 <= 16 && kpt + 1 <= D4_MAXSLOTS &&
         mid % G4_ROWS == 0 && d % D4_ROWS == 0 && ((kpt + 3) / 4 + 1) * 64 <= 320 && n_experts <= 1024 && kpt <= 64 &&
         kpt <= n_experts;
}
static size_t ggu_align(int t) { return t == MOE_GGML_Q8_0 || t == MOE_GGML_IQ4_NL ? 4 : 16; }

int moe_launch_decgg_gu_topk(int tgu, int tsh, const uint8_t* gate, const uint8_t* up, const uint8_t* sh_gate,
                             const uint8_t* sh_up, const uint32_t* xplanes, const float2* xmeta, const float* logits,
                             int n_experts, int* ids, float* ws, int id_stride, int kpt, int P, int d, int mid,
                             uint32_t* hplanes, float2* hmeta, hipStream_t st, const moe_rfix* rf) {
  const moe_rfix RFV = rf ? *rf : moe_rfix{};
  if (!gate || !up || !xplanes || !xmeta || !logits || !ids || !ws || !hplanes || !hmeta || (!sh_gate != !sh_up))
    return MOE_E_INVALID;
  if (!moe_decgg_supported(tgu, tgu, tsh, sh_gate != nullptr, d, mid, kpt, n_experts)) return MOE_E_UNSUPPORTED;
  if (!moe_aligned(gate, ggu_align(tgu)) || !moe_aligned(up, ggu_align(tgu)) ||
      (sh_gate && (!moe_aligned(sh_gate, ggu_align(tsh)) || !moe_aligned(sh_up, ggu_align(tsh)))))
    return MOE_E_INVALID;
  GuGgArgs A{gate, up, sh_gate, sh_up, tgu, tsh};
  dim3 grid(mid / G4_ROWS, kpt + (sh_gate ? 1 : 0) + 1, P);
  if (n_experts <= 512)
    k_decgg_gu<8><<<grid, 512, 0, st>>>(A, xplanes, xmeta, id_stride, kpt, d, mid, hplanes, hmeta, logits, n_experts, ids, ws, nullptr, RFV);
  else
    k_decgg_gu<16><<<grid, 512, 0, st>>>(A, xplanes, xmeta, id_stride, kpt, d, mid, hplanes, hmeta, logits, n_experts, ids, ws, nullptr, RFV);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// the same with the ids already there (the router's launches made them)
int moe_launch_decgg_gu(int tgu, int tsh, const uint8_t* gate, const uint8_t* up, const uint8_t* sh_gate,
                        const uint8_t* sh_up, const uint32_t* xplanes, const float2* xmeta, const int* ids, int n_experts,
                        int id_stride, int kpt, int P, int d, int mid, uint32_t* hplanes, float2* hmeta, hipStream_t st) {
  if (!gate || !up || !xplanes || !xmeta || !ids || !hplanes || !hmeta || (!sh_gate != !sh_up)) return MOE_E_INVALID;
  if (!moe_decgg_supported(tgu, tgu, tsh, sh_gate != nullptr, d, mid, kpt, n_experts)) return MOE_E_UNSUPPORTED;
  if (!moe_aligned(gate, ggu_align(tgu)) || !moe_aligned(up, ggu_align(tgu)) ||
      (sh_gate && (!moe_aligned(sh_gate, ggu_align(tsh)) || !moe_aligned(sh_up, ggu_align(tsh)))))
    return MOE_E_INVALID;
  GuGgArgs A{gate, up, sh_gate, sh_up, tgu, tsh};
  dim3 grid(mid / G4_ROWS, kpt + (sh_gate ? 1 : 0), P);
  k_decgg_gu<0><<<grid, 512, 0, st>>>(A, xplanes, xmeta, id_stride, kpt, d, mid, hplanes, hmeta, nullptr, n_experts, nullptr,
                                      nullptr, ids, moe_rfix{});
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_decgg_dn(int tdn, int tsh, const uint8_t* down, const uint8_t* sh_down, const float* sh_logit,
                        const uint32_t* hplanes, const float2* hmeta, const int* ids, const float* ws, int id_stride,
                        int kpt, int P, int d, int mid, float* out, uint64_t out_stride, hipStream_t st) {
  if (!down || !hplanes || !hmeta || !ids || !ws || !out || (sh_down && !sh_logit)) return MOE_E_INVALID;
  if (!moe_aligned(down, ggu_align(tdn)) || (sh_down && !moe_aligned(sh_down, ggu_align(tsh)))) return MOE_E_INVALID;
  DnGgArgs A{down, sh_down, sh_logit, tdn, tsh};
  dim3 grid(d / D4_ROWS, P);
  k_decgg_dn<<<grid, 64 * ((kpt + 3) / 4 + (sh_down ? 1 : 0)), 0, st>>>(A, hplanes, hmeta, ids, ws, id_stride, kpt, d, mid,
                                                                        out, out_stride);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// Distinct-expert variants: tiles (at most 4 pairs each; the shared expert as expert id n_experts) / ntiles / tokidx
// from the routing permutation; hplanes / hmeta and pairs are indexed by pair position.
bool moe_decgg_uq_supported(int d) { return d % GGQ_DROWS == 0; }
int moe_decgg_uq_tile_cap() { return GGQ_PAIRS; }

int moe_launch_decgg_gu_uq(int tgu, int tsh, const uint8_t* gate, const uint8_t* up, const uint8_t* sh_gate,
                           const uint8_t* sh_up, const uint32_t* xplanes, const float2* xmeta, const moe_tile* tiles,
                           const int* ntiles, int max_tiles, const int* tokidx, int n_experts, int d, int mid,
                           uint32_t* hplanes, float2* hmeta, hipStream_t st) {
  if (!gate || !up || !xplanes || !xmeta || !tiles || !ntiles || !tokidx || !hplanes || !hmeta || (!sh_gate != !sh_up))
    return MOE_E_INVALID;
  if (!moe_decgg_supported(tgu, tgu, tsh, sh_gate != nullptr, d, mid, 1, n_experts < 1024 ? n_experts : 1024))
    return MOE_E_UNSUPPORTED;
  if (!moe_aligned(gate, ggu_align(tgu)) || !moe_aligned(up, ggu_align(tgu)) ||
      (sh_gate && (!moe_aligned(sh_gate, ggu_align(tsh)) || !moe_aligned(sh_up, ggu_align(tsh)))))
    return MOE_E_INVALID;
  if (max_tiles <= 0) return MOE_OK;
  GuGgArgs A{gate, up, sh_gate, sh_up, tgu, tsh};
  k_decgg_gu_uq<<<dim3(mid / G4_ROWS, max_tiles), 512, 0, st>>>(A, xplanes, xmeta, tiles, ntiles, tokidx, n_experts, d, mid,
                                                                hplanes, hmeta);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_decgg_dn_uq(int tdn, int tsh, const uint8_t* down, const uint8_t* sh_down, const uint32_t* hplanes,
                           const float2* hmeta, const moe_tile* tiles, const int* ntiles, int max_tiles, int n_experts,
                           int d, int mid, float* pairs, hipStream_t st) {
  if (!down || !hplanes || !hmeta || !tiles || !ntiles || !pairs) return MOE_E_INVALID;
  if (!moe_decgg_uq_supported(d) || mid % 256 || mid / 64 > 16) return MOE_E_UNSUPPORTED;
  if (!moe_aligned(down, ggu_align(tdn)) || (sh_down && !moe_aligned(sh_down, ggu_align(tsh))) || !moe_aligned(pairs, 16))
    return MOE_E_INVALID;
  if (max_tiles <= 0) return MOE_OK;
  DnGgArgs A{down, sh_down, nullptr, tdn, tsh};
  k_decgg_dn_uq<<<dim3(d / GGQ_DROWS, max_tiles), 256, 0, st>>>(A, hplanes, hmeta, tiles, ntiles, n_experts, d, mid, pairs);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}
