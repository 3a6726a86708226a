// hgn v2 routed experts (dtype 23 "i4r"): 4-bit codes n with w = (n - 8) * fp16 scale per 128 columns, stored in the
// rotated domain G of W = diag(svh) . H . G . H . diag(suh) / 128 (H = 128-block Hadamard).  The rotation moves onto
// the activations:
//   rot_in   x^ = H(suh . x) / sqrt(128)          per 128 block of the input
//   GEMV     z  = G . x^
//   rot_out  y  = svh . H(z) / sqrt(128)          per 128 block of the output
// so a layer is rot_in(x, su) -> gate_up -> [rot_out(svh_gu), SwiGLU, rot_in(suh_dn)] -> down -> weighted sum over the
// experts -> rot_out(svh_dn) (svh_dn is shared by all experts of a layer, so the last rotation runs once on the sum).
// (reference: src/gpu/parts/28_kernels_hgn_v2.inc:1-15 format notes, :62-98 k_v2_rot, :105-150 k_i4r_mid;
//  src/gpu/parts/40_model.inc:1638-1656 moe_v2_1, :4570-4686 moe_b_v2; CPU dequantisation tools/moe_lut_test.cu:936-948)
// The kernels here are the pieces around the projections; the projections themselves run on the q4cp kernels with
// one scale per 128 columns (decode_q4cp.hip, gemm_q4cp.hip).  A lane holds 8 consecutive elements, 16 lanes one
// 128-block: 16-byte accesses, and the f16 / digit-plane outputs need no exchange beyond a quad.
#include <mutex>

#include "common.h"
#include "hv2.h"
#include "internal.h"
#include "qvec.h"

namespace {

__device__ __forceinline__ void ld8(const float* p, float (&v)[8]) {
  const float4 a = ((const float4*)p)[0], b = ((const float4*)p)[1];
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void ld8(const __half* p, float (&v)[8]) {
  const uint4 u = *(const uint4*)p;
  const __half2* h = (const __half2*)&u;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const float2 f = __half22float2(h[i]);
    v[2 * i] = f.x;
    v[2 * i + 1] = f.y;
  }
}
__device__ __forceinline__ void st8(float* p, const float (&v)[8]) {
  ((float4*)p)[0] = make_float4(v[0], v[1], v[2], v[3]);
  ((float4*)p)[1] = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void st8_f16_ilv(__half* p, const float (&v)[8]) { moe_st8_f16_ilv(p, v); }
// y[p][i] = post[i] * H(pre . x[p])[i] / sqrt(128) (+ add[p][i]) per 128 block; pre / post / add optional.
// P rows of n values (n % 128 == 0), n/8 lanes per row.  MODE 0: f32 rows; 1: f16 rows in the grouped GEMM's order;
// 2: digit planes of the decode kernels (planes / meta indexed [p][n/32]).  In place (MODE 0, y == x) is fine.
template <int MODE>
__global__ void __launch_bounds__(256) k_v2_rot(const float* x, uint64_t xs, void* y, uint64_t ys,
                                                const float* __restrict__ pre, const float* __restrict__ post,
                                                const float* add, uint64_t adds, int n, int P,
                                                uint32_t* __restrict__ planes, float2* __restrict__ meta) {
  const int lane = threadIdx.x & 63;
  const int per_row = n >> 3;
  const int64_t gl = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int p = (int)(gl / per_row), c = (int)(gl - (int64_t)p * per_row) * 8;
  const bool live = p < P;  // (whole groups of 16 lanes are live or not: n % 128 == 0)
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] = 0.f;
  if (live) {
    ld8(x + (size_t)p * xs + c, v);
    if (pre) {
      float s[8];
      ld8(pre + c, s);
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] *= s[i];
    }
  }
  moe_fwht128_r8(v, lane);
  float s[8];
#pragma unroll
  for (int i = 0; i < 8; i++) s[i] = 1.f;
  if (live && post) ld8(post + c, s);
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] = v[i] * MOE_RS128 * s[i];
  if (MODE == 0) {
    if (!live) return;
    if (add) {
      float a[8];
      ld8(add + (size_t)p * adds + c, a);
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] += a[i];
    }
    st8((float*)y + (size_t)p * ys + c, v);
  } else if (MODE == 1) {
    if (live) st8_f16_ilv((__half*)y + (size_t)p * ys + c, v);
  } else {
    moe_st8_planes(v, lane, planes, meta, (size_t)p * (n >> 5) + (c >> 5), live);
  }
}

// The middle of an i4r expert, per (token, expert) slot:
//   g | u = svh_gu . H(z) / sqrt(128)      z = the slot's rotated gate_up output [2 mid]
//   h     = silu(g) * u
//   out   = H(suh_dn . h) / sqrt(128)      the rotated input of down_proj [mid]
// Sixteen lanes per 128-block b of the slot: they rotate block b of the gate half and block b of the up half (each
// lane then holds g and u of its 8 columns), apply SwiGLU and rotate the result.  No LDS, no block barrier.
// MODE 0: f32 rows, 1: f16 rows in the grouped GEMM's order, 2: digit planes; slot s of the launch goes to output
// row (s / k) * row_slots + s % k (the decode path keeps a token's slots next to its shared-expert slot).
// MODE 1 (batches: the result is rounded to f16) takes the hardware's exp2 / reciprocal approximations (1 ulp) in
// SwiGLU, as the grouped GEMM's fused epilogue does; the other modes the exact expf and division.
// xms (MODE 1, may be null): the f16 range guard of the batch path -- slot s belongs to token tokidx[s], whose row is
// multiplied by moe_hid_scale(C, xms[token]) in front of the rotation (a power of two; the combine divides it out).
template <class TG, int MODE>
__global__ void __launch_bounds__(256) k_i4r_mid(const TG* __restrict__ z, uint64_t zs, void* out, uint64_t os,
                                                 const float* __restrict__ svh_gu, const float* __restrict__ suh_dn,
                                                 int mid, int nslots, int k, int row_slots,
                                                 uint32_t* __restrict__ planes, float2* __restrict__ meta,
                                                 const float* __restrict__ xms, moe_cmag C,
                                                 const int* __restrict__ tokidx) {
  const int lane = threadIdx.x & 63;
  const int nb = mid >> 7;
  const int64_t grp = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 4;
  const int slot = (int)(grp / nb), b = (int)(grp - (int64_t)slot * nb);
  const bool live = slot < nslots;
  const int c = b * 128 + (lane & 15) * 8;  // this lane's 8 columns of each half
  float g[8], u[8], fg[8], fu[8], sd[8];
#pragma unroll
  for (int i = 0; i < 8; i++) g[i] = u[i] = fg[i] = fu[i] = sd[i] = 0.f;
  if (live) {
    ld8(z + (size_t)slot * zs + c, g);
    ld8(z + (size_t)slot * zs + mid + c, u);
    ld8(svh_gu + c, fg);
    ld8(svh_gu + mid + c, fu);
    ld8(suh_dn + c, sd);
    if (MODE == 1 && xms) {
      const float f = moe_hid_scale(C, xms[tokidx[slot]]);
#pragma unroll
      for (int i = 0; i < 8; i++) sd[i] *= f;
    }
  }
  moe_fwht128_r8(g, lane);
  moe_fwht128_r8(u, lane);
  float h[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const float gv = g[i] * MOE_RS128 * fg[i], uv = u[i] * MOE_RS128 * fu[i];
    if (MODE == 1) h[i] = gv * __builtin_amdgcn_rcpf(1.f + __expf(-gv)) * uv * sd[i];
    else h[i] = gv / (1.f + expf(-gv)) * uv * sd[i];
  }
  moe_fwht128_r8(h, lane);
#pragma unroll
  for (int i = 0; i < 8; i++) h[i] *= MOE_RS128;
  const size_t row = live ? (size_t)(slot / k) * row_slots + slot % k : 0;
  if (MODE == 0) {
    if (live) st8((float*)out + row * os + c, h);
  } else if (MODE == 1) {
    if (live) st8_f16_ilv((__half*)out + row * os + c, h);
  } else {
    moe_st8_planes(h, lane, planes, meta, row * (mid >> 5) + (c >> 5), live);
  }
}

// rows [row0, row0 + nrows) of an i4r tensor as f32 (bit-exact: (n - 8) * fp16 scale, one rounding);
// a thread per 8 elements
__global__ void __launch_bounds__(256) k_i4r_rows(const uint8_t* __restrict__ data, uint64_t rows, uint64_t cols,
                                                  uint64_t row0, uint64_t nrows, float* __restrict__ out) {
  const uint64_t per_row = cols / 8;
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < nrows * per_row; i += (uint64_t)gridDim.x * 256) {
    const uint64_t r = i / per_row, c = (i - r * per_row) * 8, gr = row0 + r;
    const uint32_t w = *(const uint32_t*)(data + gr * (cols / 2) + c / 2);
    const __half sc = *(const __half*)(data + rows * (cols / 2) + gr * (cols / 128 * 2) + (c >> 7) * 2);
    const float sf = __half2float(sc);
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = (float)((int)((w >> (4 * j)) & 15u) - 8) * sf;
    st8(out + r * cols + c, v);
  }
}

}  // namespace

// (not const and not in the unnamed namespace: a device variable that no kernel names must survive into the code
// object for the host to look its address up)
static __device__ __align__(64) float g_i4r_cb[16] = {-8.f, -7.f, -6.f, -5.f, -4.f, -3.f, -2.f, -1.f,
                                                       0.f,  1.f,  2.f,  3.f,  4.f,  5.f,  6.f,  7.f};
static std::mutex g_i4r_cb_mu;

// The linear codebook -8..7 of the i4r codes as a device array (the q4cp-style kernels read their codebook from
// memory; reference: g_i4r_cb, src/gpu/parts/30_host_util.inc:790,863-866).  One copy per device, looked up once.
const float* moe_i4r_codebook() {
  static const float* ptr[64] = {};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  std::lock_guard<std::mutex> lock(g_i4r_cb_mu);
  if (!ptr[dev]) {
    float* p = nullptr;
    if (hipGetSymbolAddress((void**)&p, HIP_SYMBOL(g_i4r_cb)) != hipSuccess) return nullptr;
    ptr[dev] = p;
  }
  return ptr[dev];
}

bool moe_v2_shapes_ok(int d, int mid) { return d % 128 == 0 && mid % 128 == 0 && 2 * mid <= 2048; }

// mode 0: f32 rows (y, ys; + add), 1: f16 rows in the grouped GEMM's order (y, ys), 2: digit planes (planes, meta)
int moe_launch_v2_rot(const float* x, uint64_t xs, int P, int n, const float* pre, const float* post, int mode, void* y,
                      uint64_t ys, const float* add, uint64_t adds, uint32_t* planes, float2* meta, hipStream_t st) {
  if (!x || P < 0 || n < 128 || n % 128 || mode < 0 || mode > 2) return MOE_E_INVALID;
  if (mode == 2 ? (!planes || !meta) : !y) return MOE_E_INVALID;
  if (!moe_aligned(x, 16) || xs % 4 || (y && !moe_aligned(y, 16)) || ys % 8 || (add && (!moe_aligned(add, 16) || adds % 4)) ||
      (pre && !moe_aligned(pre, 16)) || (post && !moe_aligned(post, 16)))
    return MOE_E_INVALID;
  if (P == 0) return MOE_OK;
  const int64_t lanes = (int64_t)P * (n / 8);
  const unsigned grid = (unsigned)((lanes + 255) / 256);
  if (mode == 0) k_v2_rot<0><<<grid, 256, 0, st>>>(x, xs, y, ys, pre, post, add, adds, n, P, nullptr, nullptr);
  else if (mode == 1) k_v2_rot<1><<<grid, 256, 0, st>>>(x, xs, y, ys, pre, post, nullptr, 0, n, P, nullptr, nullptr);
  else k_v2_rot<2><<<grid, 256, 0, st>>>(x, xs, nullptr, 0, pre, post, nullptr, 0, n, P, planes, meta);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// z: [nslots][zs] f32 or f16; output row of slot s: (s / k) * row_slots + s % k (k = row_slots = 1: row s)
int moe_launch_i4r_mid(const void* z, bool z_f16, uint64_t zs, int nslots, int mid, const float* svh_gu,
                       const float* suh_dn, int mode, void* out, uint64_t os, int k, int row_slots, uint32_t* planes,
                       float2* meta, hipStream_t st, const float* xms, moe_cmag C, const int* tokidx) {
  if (xms && (mode != 1 || !tokidx)) return MOE_E_INVALID;
  if (!z || !svh_gu || !suh_dn || nslots < 0 || mode < 0 || mode > 2 || k < 1 || row_slots < k) return MOE_E_INVALID;
  if (mode == 2 ? (!planes || !meta) : !out) return MOE_E_INVALID;
  if (mid < 128 || mid % 128 || 2 * mid > 2048) return MOE_E_UNSUPPORTED;
  if (!moe_aligned(z, 16) || zs % 8 || (out && !moe_aligned(out, 16)) || os % 8 || !moe_aligned(svh_gu, 16) ||
      !moe_aligned(suh_dn, 16))
    return MOE_E_INVALID;
  if (nslots == 0) return MOE_OK;
  const int64_t threads = (int64_t)nslots * (mid / 128) * 16;
  const unsigned grid = (unsigned)((threads + 255) / 256);
#define MID_GO(TG, M) \
  k_i4r_mid<TG, M><<<grid, 256, 0, st>>>((const TG*)z, zs, out, os, svh_gu, suh_dn, mid, nslots, k, row_slots, planes, meta, \
                                         xms, C, tokidx)
  if (z_f16) {
    if (mode == 0) MID_GO(__half, 0); else if (mode == 1) MID_GO(__half, 1); else MID_GO(__half, 2);
  } else {
    if (mode == 0) MID_GO(float, 0); else if (mode == 1) MID_GO(float, 1); else MID_GO(float, 2);
  }
#undef MID_GO
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// ---- hgn v2 dense tensors ("ht", dtype 16; q6g64, dtype 24) -> bf16 W[rows][cols] ----
// The matrix the reference's prefill GEMM reads for such a tensor (v2_deq_bf16, src/gpu/parts/30_host_util.inc:1019-1031).
// The loader runs this once per tensor; the router and shared-expert kernels then see a bf16 matrix.

// ht value of a 16-bit window (28_kernels_hgn_v2.inc:19-25): byte sum of w16 * 0x83dcd12d, f32 fma, rounded to f16
__device__ __forceinline__ float ht_val(uint32_t w16) {
  const uint32_t s = __builtin_amdgcn_sad_u8(w16 * 0x83dcd12du, 0u, 0u);
  return (float)(_Float16)fmaf((float)(1024u + s), 1.732421875f / 256.f, -10.3828125f);
}
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {  // the reference's f2bf bit trick
  const uint32_t u = __float_as_uint(f);
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

// One block per 128 x 128 tile of 8 KiB (format: k_ht_deq_bf16, 28_kernels_hgn_v2.inc:386-440).  Seen from the matrix
// side, the tile is 128 rows x 16 column octets and every (row, octet) pair owns exactly one 32-bit word: octet o =
// columns 8o .. 8o+7 lies in the 1 KiB granule o / 2, a granule holds eight 128-byte groups of 16 rows, and inside a
// group the words of the even octet come first (word = row % 16), then the odd octet's.  The eight values of a word
// are 16-bit windows that slide a nibble at a time over the word and its predecessor in the group (cyclically): column
// 8o + 7 - s is the window at bit 4s of predecessor:word.  A thread takes one row and walks the octets.
// The tile goes to LDS as f32 (element (r, c) at r * 128 + (c ^ (r >> 3)): the column pass reads rows 8 apart), is
// transformed down the columns, then along the rows -- W = diag(svh) . H . G . H . diag(suh) / 128 with the
// butterflies in ascending stride order, as the reference's fwht128 -- and leaves as bf16(v * (svh[R] / 128) * suh[C]).
__global__ void __launch_bounds__(256) k_ht_to_bf16(const uint8_t* __restrict__ codes, const float* __restrict__ suh,
                                                    const float* __restrict__ svh, uint16_t* __restrict__ out, int K) {
  __shared__ float t[128 * 128];
  const int tiles_across = K / 128;
  const int ty = (int)blockIdx.x / tiles_across, tx = (int)blockIdx.x % tiles_across;
  const uint32_t* words = (const uint32_t*)(codes + (size_t)blockIdx.x * 8192);
  const int tid = threadIdx.x;
  {
    const int row = tid & 127;
    const uint32_t* group = words + (row >> 4) * 32;  // this row's 128-byte group inside a granule
    for (int octet = tid >> 7; octet < 16; octet += 2) {
      const uint32_t* gw = group + (octet >> 1) * 256;
      const int slot = (row & 15) | ((octet & 1) << 4);
      const uint32_t cur = gw[slot], prev = gw[(slot - 1) & 31];
      float* dst = t + row * 128;
      const int swz = row >> 3;
#pragma unroll
      for (int sft = 0; sft < 8; sft++) {
        const uint32_t window = __builtin_amdgcn_alignbit(prev, cur, 4 * sft) & 0xffffu;
        dst[(8 * octet + 7 - sft) ^ swz] = ht_val(window);
      }
    }
  }
  __syncthreads();
  const int j = tid & 15, vec = tid >> 4;  // 16 lanes per 128-vector, 8 elements each
  float v[8];
  for (int pass = 0; pass < 8; pass++) {  // H down the columns
    const int c = pass * 16 + vec;
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = t[(8 * j + i) * 128 + (c ^ j)];
    moe_fwht128_r8(v, tid);
#pragma unroll
    for (int i = 0; i < 8; i++) t[(8 * j + i) * 128 + (c ^ j)] = v[i];
  }
  __syncthreads();
  for (int pass = 0; pass < 8; pass++) {  // H along the rows, the planes, bf16
    const int r = pass * 16 + vec;
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = t[r * 128 + ((8 * j + i) ^ (r >> 3))];
    moe_fwht128_r8(v, tid);
    const size_t R = (size_t)ty * 128 + r;
    const float sv = svh[R] * (1.f / 128.f);
    const int C = tx * 128 + 8 * j;
    uint32_t pk[4];
#pragma unroll
    for (int i = 0; i < 8; i += 2)
      pk[i / 2] = (uint32_t)f32_to_bf16_rne(v[i] * sv * suh[C + i]) | ((uint32_t)f32_to_bf16_rne(v[i + 1] * sv * suh[C + i + 1]) << 16);
    *(uint4*)(out + R * K + C) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
  }
}

// q6g64 (k_q6g64_deq_bf16, 28_kernels_hgn_v2.inc:442-447,604-634): row r at r * align16(13 C / 16) = C/2 bytes of low
// nibbles (even column = low nibble), C/4 bytes of the codes' two high bits (column k: byte k/4, bits 2 (k % 4)),
// C/64 x (f16 scale, f16 bias); W = bf16(fma(code, scale, bias)).  One thread per eight columns.
__global__ void __launch_bounds__(256) k_q6g64_to_bf16(const uint8_t* __restrict__ wq, uint16_t* __restrict__ out, uint64_t R,
                                                       int C, uint64_t st) {
  const uint64_t n8 = R * (uint64_t)(C >> 3);
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (uint64_t)gridDim.x * 256) {
    const uint64_t r = i / (C >> 3);
    const int c = (int)(i - r * (C >> 3)) * 8;
    const uint8_t* row = wq + r * st;
    const uint32_t lo = *(const uint32_t*)(row + (c >> 1));
    const uint32_t hi = *(const uint16_t*)(row + C / 2 + (c >> 2));
    const uint32_t sb = *(const uint32_t*)(row + 3 * (C / 4) + (c >> 6) * 4);
    const float sc = (float)__builtin_bit_cast(_Float16, (uint16_t)(sb & 0xffffu));
    const float bi = (float)__builtin_bit_cast(_Float16, (uint16_t)(sb >> 16));
    uint32_t pk[4];
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      const uint32_t c0 = ((lo >> (4 * e)) & 15u) | (((hi >> (2 * e)) & 3u) << 4);
      const uint32_t c1 = ((lo >> (4 * e + 4)) & 15u) | (((hi >> (2 * e + 2)) & 3u) << 4);
      pk[e / 2] = (uint32_t)f32_to_bf16_rne(fmaf((float)c0, sc, bi)) | ((uint32_t)f32_to_bf16_rne(fmaf((float)c1, sc, bi)) << 16);
    }
    *(uint4*)(out + r * C + c) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
  }
}

MOE_API int moe_v2_dense_to_bf16(int dtype, const uint8_t* data, const float* suh, const float* svh, uint64_t rows,
                                 uint64_t cols, uint16_t* out, moe_stream_t st) {
  if (!data || !out || rows == 0 || cols == 0 || cols > (1u << 30)) return MOE_E_INVALID;
  if (!moe_aligned(data, 16) || !moe_aligned(out, 16)) return MOE_E_INVALID;
  if (dtype == MOE_DT_HT) {
    if (rows % 128 || cols % 128 || !suh || !svh) return MOE_E_INVALID;
    const uint64_t tiles = (rows / 128) * (cols / 128);
    if (tiles > 0x7fffffffu) return MOE_E_INVALID;
    k_ht_to_bf16<<<(unsigned)tiles, 256, 0, moe_s(st)>>>(data, suh, svh, out, (int)cols);
  } else if (dtype == MOE_DT_Q6G64) {
    if (cols % 64) return MOE_E_INVALID;
    const uint64_t stride = ((13 * cols / 16) + 15) & ~15ull, n = (rows * (cols / 8) + 255) / 256;
    k_q6g64_to_bf16<<<(unsigned)(n > 65536 ? 65536 : n), 256, 0, moe_s(st)>>>(data, out, rows, (int)cols, stride);
  } else {
    return MOE_E_UNSUPPORTED;
  }
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

MOE_API int moe_i4r_dequant_rows(const uint8_t* data, uint64_t rows, uint64_t cols, uint64_t row0, uint64_t nrows,
                                 float* out, moe_stream_t st) {
  if (!data || !out || cols == 0 || cols % 128 || row0 + nrows > rows) return MOE_E_INVALID;
  if (!moe_aligned(data, 4) || !moe_aligned(out, 16)) return MOE_E_INVALID;
  if (nrows == 0) return MOE_OK;
  const uint64_t n = nrows * (cols / 8);
  const unsigned grid = (unsigned)((n + 255) / 256 > 65536 ? 65536 : (n + 255) / 256);
  k_i4r_rows<<<grid, 256, 0, moe_s(st)>>>(data, rows, cols, row0, nrows, out);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

MOE_API int moe_v2_rot(const float* x, uint64_t xs, void* y, uint64_t ys, const float* pre, const float* post, int n,
                       int P, int out_f16, moe_stream_t st) {
  return moe_launch_v2_rot(x, xs, P, n, pre, post, out_f16 ? 1 : 0, y, ys, nullptr, 0, nullptr, nullptr, moe_s(st));
}

MOE_API int moe_i4r_mid(const void* guv, int guv_f16, uint64_t gs, void* out, int out_f16, uint64_t os,
                        const float* svh_gu, const float* suh_dn, int mid, int nslots, moe_stream_t st) {
  return moe_launch_i4r_mid(guv, guv_f16 != 0, gs, nslots, mid, svh_gu, suh_dn, out_f16 ? 1 : 0, out, os, 1, 1, nullptr,
                            nullptr, moe_s(st));
}
