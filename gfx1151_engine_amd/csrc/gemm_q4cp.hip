// Prefill: grouped expert GEMM on q4cp weights with CDNA4 MFMA (v_mfma_f32_32x32x16_f16).
//
// One block = one tile of up to 128 (token, expert) pairs of ONE expert x one block of weight
// rows.  Activations (f16) are gathered through tokidx into LDS; raw 4-bit codes and fp16 scales
// are staged in LDS as they lie in the blob and dequantised in registers straight into the MFMA
// B-operand layout: one 32-bit code word = 8 consecutive K of one weight row = one lane's operand.
// The unpack yields the K order [0,4,1,5,2,6,3,7] inside each group of 8, so the activation tile
// is written to LDS in that same order (a dot product does not care, as long as both sides agree).
// gate/up: both row sets are accumulated by the same wave, SwiGLU runs on the accumulators.
// (reference: src/gpu/parts/27_kernels_moe_lut.inc:75-83,110-640,660-821; weights are
//  w = f16(cb[n] * scale), F32 accumulation over the whole K, as in :16)
#include "common.h"
#include "internal.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128;        // pairs per tile (4 MFMA row fragments)
constexpr int BK = 64;         // K per stage
constexpr int A_LD = BK + 8;   // f16 elements per LDS activation row (144 B: conflict-free b128 reads)
constexpr int WROWS = 256;     // weight rows per block (up: 128 gate + 128 up)

struct LutDev {
  const uint8_t *w, *w_up, *sc, *sc_up;
  const float* cb;
  int sstride, e_rows, up_off;
};

union H8 {
  half8 v;
  uint32_t u[4];
  half2v h[4];
};

__device__ __forceinline__ half2v as_h2(uint32_t u) {
  union { uint32_t u; half2v h; } c;
  c.u = u;
  return c.h;
}

// 8 codes of one 32-bit word -> 8 f16 weights (a*n + b) * s, order [n0,n4,n1,n5,n2,n6,n3,n7].
// 0x6400|n is the f16 1024+n, 0x5400|(n<<4) is 64+n: subtracting the magic leaves n exactly;
// for the zero-point-8 codebook (a=1, b=-8) fma(n, s, -8s) rounds (n-8)*s once.
__device__ __forceinline__ half8 deq8_affine(uint32_t w, half2v as2, half2v bs2) {
  const half2v k1024 = {(_Float16)1024.f, (_Float16)1024.f}, k64 = {(_Float16)64.f, (_Float16)64.f};
  H8 r;
  const uint32_t w8 = w >> 8;
  r.h[0] = (as_h2((w & 0x000f000fu) | 0x64006400u) - k1024) * as2 + bs2;
  r.h[1] = (as_h2((w & 0x00f000f0u) | 0x54005400u) - k64) * as2 + bs2;
  r.h[2] = (as_h2((w8 & 0x000f000fu) | 0x64006400u) - k1024) * as2 + bs2;
  r.h[3] = (as_h2((w8 & 0x00f000f0u) | 0x54005400u) - k64) * as2 + bs2;
  return r.v;
}
// any codebook: 16-entry f32 table in LDS, w = f16(cb[n] * s)
__device__ __forceinline__ half8 deq8_table(uint32_t w, float s, const float* cbs) {
  H8 r;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    half2v h;
    h.x = (_Float16)(cbs[(w >> (4 * i)) & 0xf] * s);
    h.y = (_Float16)(cbs[(w >> (4 * i + 16)) & 0xf] * s);
    r.h[i] = h;
  }
  return r.v;
}

template <bool UP, bool F16OUT>
__global__ void __launch_bounds__(256, 2)
k_moe_gemm_q4cp(LutDev R, LutDev Sh, int n_experts, const __half* __restrict__ x,
                const int* __restrict__ tokidx, const moe_tile* __restrict__ tiles,
                const int* __restrict__ ntiles, void* __restrict__ out, int M, int K, int nblk_n) {
  __shared__ __attribute__((aligned(16))) _Float16 As[BM * A_LD];
  __shared__ __attribute__((aligned(16))) uint8_t Ws[WROWS * 32];
  __shared__ __attribute__((aligned(4))) _Float16 Ss[WROWS * 2];
  __shared__ float cbs[16];
  __shared__ int rowidx[BM];

  // XCD-aware order: consecutive workgroup ids go round-robin over the 8 XCDs; give each XCD a
  // contiguous run of tiles so that tiles of one expert share that XCD's L2.
  const int nt = *ntiles;
  const int wg = blockIdx.x, xcd = wg & 7, j = wg >> 3;
  const int per_xcd = (nt + 7) >> 3;
  const int tl = j / nblk_n, nb = j - tl * nblk_n;
  const int ti = xcd * per_xcd + tl;
  if (tl >= per_xcd || ti >= nt) return;
  const moe_tile tile = tiles[ti];
  const bool shared = tile.expert >= n_experts;
  const LutDev& L = shared ? Sh : R;
  const int e = shared ? 0 : tile.expert;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;

  // codebook: affine (a*n+b) or table
  const float c0 = L.cb[0], c1 = L.cb[1];
  bool aff = true;
  if (lane < 16) {
    const float v = L.cb[lane];
    aff = v == fmaf((float)lane, c1 - c0, c0);
    if (tid < 16) cbs[lane] = v;
  }
  const bool affine = __all(aff);
  const float cb_a = c1 - c0, cb_b = c0;

  if (tid < BM) {
    const int m = tid < tile.count ? tid : 0;  // rows past the tile read a valid row, never stored
    rowidx[tid] = tokidx ? tokidx[tile.first + m] : tile.first + m;
  }
  __syncthreads();

  // per-thread global sources
  const int a_c = tid & 7;  // 16-byte chunk of the 128-byte stage row
  const __half* a_src[4];
#pragma unroll
  for (int i = 0; i < 4; i++) a_src[i] = x + (size_t)rowidx[(tid >> 3) + 32 * i] * K + a_c * 8;
  const uint8_t* w_src[2];
  const int w_half = tid & 1;
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int lr = (tid >> 1) + 128 * i;
    size_t grow;
    const uint8_t* base;
    if (UP) {
      base = i == 0 ? L.w : L.w_up;
      grow = (size_t)e * L.e_rows + (i == 0 ? 0 : L.up_off) + (size_t)nb * 128 + (lr & 127);
    } else {
      base = L.w;
      grow = (size_t)e * L.e_rows + (size_t)nb * 256 + lr;
    }
    w_src[i] = base + grow * (size_t)(K / 2) + w_half * 16;
  }
  const uint8_t* s_src;
  {
    const int lr = tid;
    size_t grow;
    const uint8_t* base;
    if (UP) {
      base = lr < 128 ? L.sc : L.sc_up;
      grow = (size_t)e * L.e_rows + (lr < 128 ? 0 : L.up_off) + (size_t)nb * 128 + (lr & 127);
    } else {
      base = L.sc;
      grow = (size_t)e * L.e_rows + (size_t)nb * 256 + lr;
    }
    s_src = base + grow * (size_t)L.sstride;
  }

  floatx16 acc[4][2];
#pragma unroll
  for (int mf = 0; mf < 4; mf++)
#pragma unroll
    for (int nf = 0; nf < 2; nf++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[mf][nf][i] = 0.f;

  const int nfrag_m = (tile.count + 31) >> 5;  // live 32-row fragments of this tile
  const int n = lane & 31, h = lane >> 5;
  // LDS rows of this wave's two weight fragments
  const int wrow0 = UP ? 32 * wv + n : 64 * wv + n;
  const int wrow1 = UP ? 128 + 32 * wv + n : 64 * wv + 32 + n;

  uint4 ra[4], rw[2];
  uint32_t rs;
  auto gload = [&](int s) {
#pragma unroll
    for (int i = 0; i < 4; i++) ra[i] = *(const uint4*)(a_src[i] + (size_t)s * BK);
#pragma unroll
    for (int i = 0; i < 2; i++) rw[i] = *(const uint4*)(w_src[i] + (size_t)s * 32);
    rs = *(const uint32_t*)(s_src + (size_t)s * 4);
  };
  const int nstage = K / BK;
  gload(0);
  for (int s = 0; s < nstage; s++) {
    // registers -> LDS (activations re-ordered inside each group of 8: [0,4,1,5,2,6,3,7])
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint4 p;
      p.x = (ra[i].x & 0xffffu) | (ra[i].z << 16);
      p.y = (ra[i].x >> 16) | (ra[i].z & 0xffff0000u);
      p.z = (ra[i].y & 0xffffu) | (ra[i].w << 16);
      p.w = (ra[i].y >> 16) | (ra[i].w & 0xffff0000u);
      *(uint4*)(As + ((tid >> 3) + 32 * i) * A_LD + a_c * 8) = p;
    }
#pragma unroll
    for (int i = 0; i < 2; i++) *(uint4*)(Ws + ((tid >> 1) + 128 * i) * 32 + w_half * 16) = rw[i];
    *(uint32_t*)(Ss + tid * 2) = rs;
    __syncthreads();
    if (s + 1 < nstage) gload(s + 1);

    // dequantise this wave's 2 x (32 rows x 64 K): lane (n, h) owns K [32h, 32h+32) of row n
    half8 bfrag[2][4];
#pragma unroll
    for (int nf = 0; nf < 2; nf++) {
      const int wr = nf == 0 ? wrow0 : wrow1;
      const uint4 cw = *(const uint4*)(Ws + wr * 32 + h * 16);
      const float sc = (float)Ss[wr * 2 + h];
      const uint32_t cwv[4] = {cw.x, cw.y, cw.z, cw.w};
      if (affine) {
        const _Float16 as = (_Float16)(cb_a * sc), bs = (_Float16)(cb_b * sc);
        const half2v as2 = {as, as}, bs2 = {bs, bs};
#pragma unroll
        for (int q = 0; q < 4; q++) bfrag[nf][q] = deq8_affine(cwv[q], as2, bs2);
      } else {
#pragma unroll
        for (int q = 0; q < 4; q++) bfrag[nf][q] = deq8_table(cwv[q], sc, cbs);
      }
    }
#pragma unroll
    for (int q = 0; q < 4; q++) {
#pragma unroll
      for (int mf = 0; mf < 4; mf++) {
        if (mf < nfrag_m) {
          const half8 a = *(const half8*)(As + (32 * mf + n) * A_LD + 32 * h + 8 * q);
          acc[mf][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bfrag[0][q], acc[mf][0], 0, 0, 0);
          acc[mf][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bfrag[1][q], acc[mf][1], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }

  // epilogue.  D[i][j]: j = lane%32 (weight row), i = 8*(r/4) + 4*(lane/32) + r%4 (pair)
#pragma unroll
  for (int mf = 0; mf < 4; mf++) {
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int m = 32 * mf + 8 * (r >> 2) + 4 * h + (r & 3);
      if (m >= tile.count) continue;
      const size_t row = (size_t)(tile.first + m);
      if (UP) {
        const float g = acc[mf][0][r], u = acc[mf][1][r];
        const float hv = g / (1.f + __expf(-g)) * u;
        ((__half*)out)[row * M + nb * 128 + 32 * wv + n] = __float2half(hv);
      } else {
#pragma unroll
        for (int nf = 0; nf < 2; nf++) {
          const size_t col = (size_t)nb * 256 + 64 * wv + 32 * nf + n;
          if (F16OUT) ((__half*)out)[row * M + col] = __float2half(acc[mf][nf][r]);
          else ((float*)out)[row * M + col] = acc[mf][nf][r];
        }
      }
    }
  }
}

LutDev to_dev(const moe_lutw* p) {
  LutDev d{};
  if (p) {
    d.w = p->w; d.w_up = p->w_up; d.sc = p->sc; d.sc_up = p->sc_up; d.cb = p->cb;
    d.sstride = p->sstride; d.e_rows = p->e_rows; d.up_off = p->up_off;
  }
  return d;
}

bool lut_ok(const moe_lutw* p, bool pair, int k) {
  if (!p || !p->w || !p->sc || !p->cb) return false;
  if (pair && (!p->w_up || !p->sc_up)) return false;
  if (k < 64 || k % 64) return false;
  if (!moe_aligned(p->w, 16) || !moe_aligned(p->sc, 4) || p->sstride % 4 || p->sstride < k / 32 * 2) return false;
  if (pair && (!moe_aligned(p->w_up, 16) || !moe_aligned(p->sc_up, 4))) return false;
  return true;
}

}  // namespace

// Internal: routed + (optional) shared expert in one launch; tile.expert >= n_experts selects Sh.
int moe_launch_gemm_q4cp(bool up, const moe_lutw* routed, const moe_lutw* sh, int n_experts,
                         const __half* x, const int* tokidx, const moe_tile* tiles, const int* ntiles,
                         int max_tiles, void* out, int m, int k, bool f16out, hipStream_t st) {
  if (!x || !tiles || !ntiles || !out || max_tiles < 0) return MOE_E_INVALID;
  if (!lut_ok(routed, up, k) || (sh && !lut_ok(sh, up, k))) return MOE_E_UNSUPPORTED;
  if (up ? (m % 128 != 0) : (m % 256 != 0)) return MOE_E_UNSUPPORTED;
  if (!moe_aligned(x, 16) || !moe_aligned(out, 4)) return MOE_E_INVALID;
  if (max_tiles == 0) return MOE_OK;
  const int nblk_n = up ? m / 128 : m / 256;
  const int per_xcd = (max_tiles + 7) / 8;
  const unsigned grid = (unsigned)(per_xcd * nblk_n * 8);
  LutDev R = to_dev(routed), S = to_dev(sh ? sh : routed);
  if (up)
    k_moe_gemm_q4cp<true, true><<<grid, 256, 0, st>>>(R, S, n_experts, x, tokidx, tiles, ntiles, out, m, k, nblk_n);
  else if (f16out)
    k_moe_gemm_q4cp<false, true><<<grid, 256, 0, st>>>(R, S, n_experts, x, tokidx, tiles, ntiles, out, m, k, nblk_n);
  else
    k_moe_gemm_q4cp<false, false><<<grid, 256, 0, st>>>(R, S, n_experts, x, tokidx, tiles, ntiles, out, m, k, nblk_n);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

MOE_API int moe_lut_q4cp_view(const uint8_t* data, uint64_t rows, uint64_t cols, uint64_t scale_stride,
                              int e_rows, int up_off, moe_lutw* out) {
  if (!data || !out || cols == 0 || cols % 32) return MOE_E_INVALID;
  out->cb = (const float*)data;
  out->w = out->w_up = data + 64;
  out->sc = out->sc_up = data + 64 + rows * cols / 2;
  out->sstride = (int)(scale_stride ? scale_stride : (((cols / 32 * 2) + 15) & ~15ULL));
  out->e_rows = e_rows;
  out->up_off = up_off;
  return MOE_OK;
}

MOE_API int moe_lut_up(int type, const moe_lutw* p, const void* x16, const int* tokidx,
                       const moe_tile* tiles, const int* ntiles, int max_tiles, void* hid16, int m, int k,
                       moe_stream_t st) {
  if (type != MOE_LUT_Q4CP) return MOE_E_UNSUPPORTED;
  if (!tokidx) return MOE_E_INVALID;
  return moe_launch_gemm_q4cp(true, p, nullptr, 1 << 30, (const __half*)x16, tokidx, tiles, ntiles, max_tiles,
                              hid16, m, k, true, moe_s(st));
}

MOE_API int moe_lut_down(int type, const moe_lutw* p, const void* hid16, const moe_tile* tiles,
                         const int* ntiles, int max_tiles, void* pairs, int m, int k, int f16,
                         moe_stream_t st) {
  if (type != MOE_LUT_Q4CP) return MOE_E_UNSUPPORTED;
  return moe_launch_gemm_q4cp(false, p, nullptr, 1 << 30, (const __half*)hid16, nullptr, tiles, ntiles,
                              max_tiles, pairs, m, k, f16 != 0, moe_s(st));
}
