// Prefill: grouped expert GEMM on q4cp weights with CDNA4 MFMA (v_mfma_f32_32x32x16_f16).
//
// One block (4 waves) = one tile of up to 128 (token, expert) pairs of ONE expert x 256 weight rows
// (gate/up: 128 gate + the matching 128 up rows, SwiGLU on the accumulators).  Each wave owns
// 128 pairs x 64 weight rows = 8 accumulators.  Two such blocks share a CU (2 x 77 KB of LDS, one
// wave of each per SIMD): they pass their barriers, prologues and epilogues independently, so the
// matrix pipe has the other block's MFMAs to run meanwhile (8-wave blocks of 512 rows, one per
// CU, measured 4 % (q4cp) to 10 % (Q4_K) slower).
// Activations (f16), raw 4-bit codes and fp16 scales go global -> LDS directly (no registers),
// three stage buffers, one barrier per 64-wide K stage.  Codes are dequantised in registers straight
// into the MFMA B-operand layout: one 32-bit code word = 8 consecutive K of one weight row = one
// lane's operand.  The unpack yields the K order [0,4,1,5,2,6,3,7] inside each group of 8, so
// f16 activations are kept in that same "interleaved" order (a dot product does not care as long
// as both sides agree): moe_f32_to_f16(layout 1) and the gate/up epilogue write it.
// (reference: src/gpu/parts/27_kernels_moe_lut.inc:75-83,110-640,660-821; weights are
//  w = f16(cb[n] * scale), F32 accumulation over the whole K, as in :16)
//
// Q4K = true reads raw GGUF Q4_K super-blocks in place instead (144 B per 256 elements:
// d, dmin, 12 packed bytes of 6-bit sub-scales / mins, 128 code bytes; src/gguf.h:408-441,
// src/gpu/parts/26_kernels_moe_gguf.inc:81-485).  One 64-wide K stage is one 32-byte run of code
// bytes (low nibbles = elements 0..31, high nibbles = elements 32..63 of the stage), so a 32-bit
// code word unpacks to [4w, 4w+2, 32+4w, 32+4w+2, 4w+1, 4w+3, 32+4w+1, 32+4w+3]: activations are kept
// in that order (layout 2), and the pairs of one word alternate between the stage's two sub-blocks,
// each with its own w = (d*sc)*n - dmin*m as one packed f16 FMA.  The 16-byte block header takes
// the place of q4cp's 8 staged scales (one per row and four stages).
//
// Q5 (with Q4K): raw GGUF Q5_K super-blocks (176 B: the Q4_K header, 32 bytes qh, 128 code bytes; src/gguf.h:421-441):
// the same stages with a fifth bit per code -- bit 2jj of qh byte l for the low nibble of code byte l in stage jj of the
// super-block, bit 2jj+1 for the high nibble.  A lane fetches the 16 qh bytes of its half of each fragment row straight
// into registers, together with the header's load one super-block ahead (through LDS they would take 8 KB more, one
// block per CU instead of two), keeps them for the four stages and ORs the bit into the magic-number form of each code
// pair (1024 + n and 64 + n stay exact for n < 32).
//
// GS = 2: one scale per 128 columns instead of 32 (hgn v2 i4r experts, reference kI4R,
// src/gpu/parts/27_kernels_moe_lut.inc:23-29): the four stages between two scale refreshes span exactly two scales,
// fetched as one 4-byte load per row.
#include "common.h"
#include "hv2.h"
#include "internal.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#ifndef MOE_GEMM_NF
#define MOE_GEMM_NF 2
#endif
#ifndef MOE_GEMM_WALK
#define MOE_GEMM_WALK 3  // column blocks that a block of a down launch walks (at most)
#endif
#ifndef MOE_GEMM_WROWS
#define MOE_GEMM_WROWS 256
#endif
constexpr int NF = MOE_GEMM_NF;          // weight fragments (32 rows) per wave
constexpr int WROWS = MOE_GEMM_WROWS;    // weight rows per block (up: WROWS/2 gate + the matching WROWS/2 up rows)
constexpr int HALF = WROWS / 2;
constexpr int NW = WROWS / 32 / NF;       // waves per block
constexpr int NT = 64 * NW;               // each wave: 128 pairs x 32*NF weight rows
#ifndef MOE_GEMM_BM
#define MOE_GEMM_BM 128
#endif
constexpr int BM = MOE_GEMM_BM;  // pairs per tile (32-row MFMA fragments: 4, or 8 with one block per CU and accumulators in AGPRs)
constexpr int WPE = BM > 128 ? 1 : NT * (WROWS == 512 ? 1 : 2) / 256;  // waves per SIMD: 256-row blocks of 128 pairs run two to a CU
constexpr int BK = 64;         // K per stage
constexpr int A_BYTES = BM * BK * 2;      // 16 KB  [row][8 chunks of 16 B], chunk c of row m at slot c ^ ((m >> 1) & 7): conflict-free for the 128-bit fragment reads
constexpr int W_BYTES = WROWS * 32;       // [row][32 B]
constexpr int S_BYTES = WROWS * 16;       // [row][8 scales], refreshed every 4 stages
// scale buffers: two, or one whose four stages' worth a lane keeps in registers (two 256-row
// blocks then fit the CU's 160 KB)
constexpr int NSB = WROWS == 512 ? 2 : 1;
#ifndef MOE_GEMM_NBUF
#define MOE_GEMM_NBUF 3
#endif
constexpr int NBUF = MOE_GEMM_NBUF;       // activation / code buffers; loads run NBUF-1 stages ahead
constexpr int AHEAD = NBUF - 1;
constexpr int SMEM_BYTES = NBUF * (A_BYTES + W_BYTES) + NSB * S_BYTES + 128 + BM * 4 + BM * 4;  // + two 16-entry codebooks, row indices, row scales
// NAT (table codebooks in natural K order): two 256-entry tables of f16 pairs behind the rest, indexed by a whole code
// byte = two neighbouring weights (the (gate) rows' codebook and the up rows')
constexpr int PT_BYTES = 2 * 256 * 4;

struct LutDev {
  const uint8_t *w, *w_up, *sc, *sc_up;
  const float *cb, *cb_up;  // codebook of the (gate) rows and of the up rows (the same for a fused gate_up tensor)
  int sstride, e_rows, up_off;
  // per expert: the power of two P of the scaled dequantisation (DN below), or MOE_PEXP_NONE; nullptr = none
  const int8_t* pexp;
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

// position of element e (0..7) inside its interleaved group of 8
__device__ __forceinline__ int ilv_pos(int e) { return ((e & 3) << 1) | (e >> 2); }

// position of element c (0..63) of a 64-element block in layout 2
__device__ __forceinline__ int q4k_pos(int c) {
  const int e = c & 31, w = e >> 2, r = e & 3;
  return 8 * w + ((r & 1) << 2) + ((c >> 5) << 1) + (r >> 1);
}

__device__ __forceinline__ void mfma16(floatx16& acc, const half8& a, const half8& b) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
}

#define LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
// 64 lanes x 16 B: global (per-lane address) -> LDS (wave-uniform base, lane l lands at base + 16 l)
__device__ __forceinline__ void g2l16(const void* g, uint8_t* lds_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g, LDS_PTR(lds_base), 16, 0, 0);
}
// 64 lanes x 4 B: lane l lands at base + 4 l
__device__ __forceinline__ void g2l4(const void* g, uint8_t* lds_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g, LDS_PTR(lds_base), 4, 0, 0);
}

// MF = live 32-row fragments of the tile (1 .. 4); AFFINE = codebook a*n+b.
// NF = weight fragments (32 rows) per wave: the block's 16 fragments are split over NW = 16/NF
// waves, each wave multiplying all MF pair fragments with its own NF weight fragments.
// DN (affine q4cp codebooks, a power of two P known for the expert): two instructions per weight pair instead of three.
// A masked code pair IS a pair of f16 denormals, n * 2^-24 (nibbles at bits 0-3) or n * 2^-20 (bits 4-7), so one packed
// FMA with a = f16(cb_a * scale) * 2^(24+P) (or 2^(20+P)) and b = f16(cb_b * scale) * 2^P gives 2^P * f16(n*a' + b'):
// the weights of the three-instruction form times 2^P, bit for bit wherever the scaled weight is a normal f16 (the
// product is exact inside the FMA, one rounding).  P is chosen when the weights are registered, from the expert's
// largest scale, so that the scaled slope stays below 2^15 (an f16 can hold it); the accumulators carry the factor
// 2^P and the epilogue takes it out (exact).  v_pk_fma_f16 takes denormal operands at full rate on gfx950.
constexpr bool NH_OK = NF == 2;
template <bool UP, bool F16OUT, int MF, bool AFFINE, bool Q4K, int GS, bool Q5, bool NAT = false, bool DN = false, bool ROT = false>
__device__ __forceinline__ void gemm_tile(uint8_t* smem, const LutDev& L, int e, const moe_tile tile, int nb,
                                          const __half* __restrict__ x, void* __restrict__ out, int M,
                                          int K, float cb_a, float cb_b, float cb_a_up, float cb_b_up, int ri,
                                          const float* __restrict__ xms,
                                          moe_cmag cmag, const moe_comb& cmb, bool shared, int pexp = 0, int npass = 1,
                                          moe_rotv rot = moe_rotv{nullptr, nullptr}) {
  static_assert(!ROT || (UP && F16OUT && GS == 2 && AFFINE && !DN && HALF == 128 && NH_OK), "rotated experts: gate/up rows of one 128-block per block");
  // npass > 1 (down launches with f16 results): the block walks npass neighbouring column blocks of its pair tile.  The
  // K stages of all passes form one pipeline -- the first stages of the next column block are requested while the
  // current one's last stages run, so only the first pass pays for the trip to memory -- and the epilogue of a pass
  // uses the stage buffer that the pipeline has just left.
  constexpr bool WALK = !UP && F16OUT && !Q5 && AHEAD == 2;
  if (!WALK) npass = 1;
  static_assert(!DN || (AFFINE && !Q4K && !Q5 && !NAT), "scaled dequantisation: affine q4cp-style planes");
  if (DN) {  // the codebook in the scaled units
    const float s24 = __builtin_ldexpf(1.f, 24 + pexp), sp = __builtin_ldexpf(1.f, pexp);
    cb_a *= s24; cb_a_up *= s24;
    cb_b *= sp; cb_b_up *= sp;
  }
  const float oscale = DN ? __builtin_ldexpf(1.f, -pexp) : 1.f;  // takes 2^P out of the accumulators
  constexpr int NH = NF / 2;  // gate/up: fragments per half
  static_assert(GS == 0 || (GS == 2 && !Q4K && NSB == 1), "one scale per 128 columns: q4cp-style planes, single scale buffer");
  static_assert(!Q5 || (Q4K && NSB == 1), "Q5_K: the Q4_K stages plus a fifth bit");
  static_assert(!NAT || (!AFFINE && !Q4K && GS == 0), "pair tables: q4cp planes with a table codebook");
  const uint32_t* const ptab = (const uint32_t*)(smem + SMEM_BYTES);
  constexpr int KBLK = Q5 ? 176 : 144;   // bytes per super-block
  constexpr int KQS = Q5 ? 48 : 16;      // offset of the code bytes in it
  // loads per row group behind the scale buffer's: the header's 16 bytes go to LDS; Q5_K adds two 8-byte register loads
  // per weight fragment of the lane (its half of the row's 32 qh bytes; pairs of registers are easier to place than
  // quadruples in a kernel this close to the register limit), issued in the same place so that the count of outstanding
  // loads the waits rely on is the same for every wave
  constexpr int SP = Q5 ? 1 + 2 * NF : 1;
  static_assert(!Q5 || (WROWS / 64 + NW - 1) / NW == 1, "Q5_K: one row group per wave in the scale buffer");
  uint8_t* const A0 = smem;
  uint8_t* const W0 = smem + NBUF * A_BYTES;
  uint8_t* const S0 = W0 + NBUF * W_BYTES;
  const float* cbs = (const float*)(S0 + NSB * S_BYTES);
  int* rowidx = (int*)(cbs + 32);  // cbs[16..31]: the up rows' codebook
  float* rowscale = (float*)(rowidx + BM);  // f16 range guard of each pair row (gate/up only)
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave index, kept scalar
  const int n = lane & 31, h = lane >> 5;

  // LDS row -> global weight row (rows past the matrix are clamped: loaded, never stored)
  auto wrow_ptrs = [&](int lr, const uint8_t*& cw, const uint8_t*& sw) {
    size_t grow;
    const uint8_t *cb0, *sb0;
    if (UP) {
      const bool up = lr >= HALF;
      int r = nb * HALF + (lr & (HALF - 1));
      r = r < M ? r : M - 1;
      cb0 = up ? L.w_up : L.w;
      sb0 = up ? L.sc_up : L.sc;
      grow = (size_t)e * L.e_rows + (up ? L.up_off : 0) + r;
    } else {
      int r = nb * WROWS + lr;
      r = r < M ? r : M - 1;
      cb0 = L.w;
      sb0 = L.sc;
      grow = (size_t)e * L.e_rows + r;
    }
    if (Q4K) {
      cw = cb0 + grow * (size_t)(K / 256 * KBLK);  // raw row: K/256 super-blocks
      sw = cw;                                    // block header (d, dmin, packed scales) leads each block
    } else {
      cw = cb0 + grow * (size_t)(K / 2);
      sw = sb0 + grow * (size_t)L.sstride;
    }
  };

  // per-lane global sources of the direct-to-LDS loads (wave-load j of a buffer = LDS bytes [1024 j, +1024))
  // activations: rows 8j..8j+7, lane -> (row 8j + lane/8, slot lane%8 holding chunk slot ^ ((row >> 1) & 7)).
  // The 4*MF row groups are dealt to the waves; with more waves than groups some load a group twice
  // (same bytes to the same place) so that every wave issues the same number of loads.
  constexpr int A_GROUPS = 4 * MF;
  constexpr int A_LOADS = (A_GROUPS + NW - 1) / NW;
  constexpr int W_LOADS = WROWS / 32 / NW, S_ROWG = (WROWS / 64 + NW - 1) / NW, S_LOADS = S_ROWG * SP;
  const __half* a_src[A_LOADS];
  int a_grp[A_LOADS];
#pragma unroll
  for (int i = 0; i < A_LOADS; i++) a_grp[i] = (A_LOADS * wv + i) % A_GROUPS;  // a_src: once the row indices are in LDS
  // codes: rows 32j..32j+31, lane -> (row 32j + lane/2, half lane%2); scales: rows 64j.., lane -> row
  const uint8_t *w_src[W_LOADS], *s_src[S_ROWG];
  // Q5_K keeps 32-bit byte offsets from wave-uniform bases instead of per-lane pointers (the launcher checks that the
  // tensors and the activation rows stay below 4 GB): the registers that saves are what lets two blocks share a CU.
  // A wave's code and header rows lie in one half of the block's rows: gate rows for the first NW / 2 waves, up rows
  // for the others.
  uint32_t a_off[Q5 ? A_LOADS : 1], w_off[Q5 ? W_LOADS : 1], s_off = 0, qh_off0 = 0, qh_off1 = 0;
  const uint8_t* const wave_w = Q5 ? (wv >= NW / 2 ? L.w_up : L.w) : nullptr;
  auto wrow_off = [&](int lr) -> uint32_t {  // Q5_K gate/up: byte offset of LDS row lr's weight row in its tensor
    int r = nb * HALF + (lr & (HALF - 1));
    r = r < M ? r : M - 1;
    const uint32_t grow = (uint32_t)e * (uint32_t)L.e_rows + (lr >= HALF ? (uint32_t)L.up_off : 0u) + (uint32_t)r;
    return grow * (uint32_t)(K / 256 * KBLK);
  };
  if (Q5) {
#pragma unroll
    for (int i = 0; i < W_LOADS; i++) w_off[i] = wrow_off(32 * (W_LOADS * wv + i) + (lane >> 1)) + (lane & 1) * 16;
    s_off = wrow_off(64 * wv + lane);
  } else {
#pragma unroll
    for (int i = 0; i < W_LOADS; i++) {
      const uint8_t* sw;
      wrow_ptrs(32 * (W_LOADS * wv + i) + (lane >> 1), w_src[i], sw);
      w_src[i] += (lane & 1) * 16;
    }
#pragma unroll
    for (int i = 0; i < S_ROWG; i++) {
      const uint8_t* cw;
      wrow_ptrs(64 * (S_ROWG * wv + i) + lane, cw, s_src[i]);
    }
  }
  // LDS rows of this wave's weight fragments (gate/up: NH gate + the NH matching up fragments).
  // Q4_K gate/up with one fragment per half: hid is written in 64-element blocks whose 16-byte
  // chunks mix elements c and 32+c, so the fragment takes rows {16q..16q+15} and {32+16q..} of
  // its 64-row block (q = wave parity): four whole chunks per wave.
  int wrow[NF];
#pragma unroll
  for (int nf = 0; nf < NF; nf++) {
    if (!UP) wrow[nf] = 32 * NF * wv + 32 * nf + n;
    else if (Q4K && NH == 1) wrow[nf] = nf * HALF + 64 * (wv >> 1) + 16 * (wv & 1) + (n & 15) + 2 * (n & 16);
    else wrow[nf] = (nf / NH) * HALF + 32 * NH * wv + 32 * (nf % NH) + n;
  }

  // Q5_K: the lane's half (code bytes 16 h .. 16 h + 15) of its fragment rows' 32 qh bytes, fetched into registers one
  // super-block ahead
  static_assert(!Q5 || (UP && NF == 2 && W_LOADS * 32 * (NW / 2) == HALF), "Q5_K: gate/up, a gate and an up fragment per wave");
  uint2 qhn[4] = {{0u, 0u}, {0u, 0u}, {0u, 0u}, {0u, 0u}};
  if (Q5) {
    qh_off0 = wrow_off(wrow[0]) + 16 + 16 * h;        // fragment 0: a gate row (base L.w)
    qh_off1 = wrow_off(wrow[NF - 1]) + 16 + 16 * h;   // fragment 1: the matching up row (base L.w_up)
  }
  const int nstage = K / BK, ngroups = K / 32;
  constexpr int NLOADS = A_LOADS + W_LOADS;  // per stage (+S_LOADS scale loads on every fourth stage)
  // one direct-to-LDS load of stage s: u < A_LOADS activations, then the code loads, then the scale loads
  // bytes from one column block's rows to the next one's (passes of a walk)
  const size_t wpass = WALK ? (size_t)WROWS * (Q4K ? (size_t)(K / 256 * KBLK) : (size_t)(K / 2)) : 0;
  const size_t spass = WALK ? (Q4K ? wpass : (size_t)WROWS * (size_t)L.sstride) : 0;
  // stage s of a pass into buffer b; pw / ps: byte offsets of the pass's code and scale rows from the first pass's
  auto issue_unit = [&](int s, int b, size_t pw, size_t ps, int u) {
    if (u < A_LOADS) {
      if (Q5) g2l16((const uint8_t*)x + (a_off[Q5 ? u : 0] + (uint32_t)s * (BK * 2)), A0 + b * A_BYTES + a_grp[u] * 1024);
      else g2l16(a_src[u] + (size_t)s * BK, A0 + b * A_BYTES + a_grp[u] * 1024);
    } else if (u < NLOADS) {
      const int i = u - A_LOADS;
      const size_t off = Q4K ? (size_t)(s >> 2) * KBLK + KQS + (size_t)(s & 3) * 32 : (size_t)s * 32;
      if (Q5) g2l16(wave_w + (w_off[Q5 ? i : 0] + (uint32_t)off), W0 + b * W_BYTES + (W_LOADS * wv + i) * 1024);
      else g2l16(w_src[i] + (off + pw), W0 + b * W_BYTES + (W_LOADS * wv + i) * 1024);
    } else {
      // 8 scales (16 B) per row for stages s..s+3; at the end of K the window is pulled back inside the row
      const int i = (u - NLOADS) / SP, pc = (u - NLOADS) % SP;  // row group, 16-byte piece of the row's record
      int g0 = 2 * s;
      g0 = g0 + 8 <= ngroups ? g0 : ngroups - 8;
      const size_t off = (Q4K ? (size_t)(s >> 2) * KBLK : (size_t)g0 * 2) + ps;
      if (Q5 && pc == 1)  // this lane's 16 qh bytes of each fragment, into registers
        qhn[0] = *(const uint2*)(L.w + (qh_off0 + (uint32_t)off));
      else if (Q5 && pc == 2)
        qhn[1] = *(const uint2*)(L.w + (qh_off0 + (uint32_t)off + 8u));
      else if (Q5 && pc == 3)
        qhn[2] = *(const uint2*)(L.w_up + (qh_off1 + (uint32_t)off));
      else if (Q5 && pc == 4)
        qhn[3] = *(const uint2*)(L.w_up + (qh_off1 + (uint32_t)off + 8u));
      else if (Q5)
        g2l16(wave_w + (s_off + (uint32_t)off), S0 + wv * 1024);
      else if (GS == 2)  // the two scales of stages s..s+3 (s % 4 == 0: columns 64 s .. 64 s + 255), [row][4 B]
        g2l4(s_src[i] + ((size_t)s + ps), S0 + (S_ROWG * wv + i) * 256);
      else  // piece pc of every row: a region of its own, [row][16 B]
        g2l16(s_src[i] + off, S0 + ((s >> 2) & (NSB - 1)) * S_BYTES + (S_ROWG * wv + i) * 1024);
    }
  };
  auto issue_a = [&](int s) {
#pragma unroll
    for (int u = 0; u < A_LOADS; u++) issue_unit(s, s % NBUF, 0, 0, u);
  };
  auto issue_w = [&](int s) {  // codes, and the scales on every fourth stage
#pragma unroll
    for (int u = A_LOADS; u < NLOADS; u++) issue_unit(s, s % NBUF, 0, 0, u);
    if ((s & 3) == 0) {
#pragma unroll
      for (int u = 0; u < S_LOADS; u++) issue_unit(s, s % NBUF, 0, 0, NLOADS + u);
    }
  };
  // s_waitcnt vmcnt(N), N = loads allowed to stay in flight (loads retire in order)
  // (the immediate must be a constant: one case per count of outstanding loads)
  auto wait_vm = [&](int n) {
    switch (n) {
#define VM_CASE(N) case N: __builtin_amdgcn_s_waitcnt(0x0F70 | ((N) & 15) | (((N) >> 4) << 14)); break;
      VM_CASE(0) VM_CASE(1) VM_CASE(2) VM_CASE(3) VM_CASE(4) VM_CASE(5) VM_CASE(6) VM_CASE(7) VM_CASE(8)
      VM_CASE(9) VM_CASE(10) VM_CASE(11) VM_CASE(12) VM_CASE(13) VM_CASE(14) VM_CASE(15) VM_CASE(16)
      VM_CASE(17) VM_CASE(18) VM_CASE(19) VM_CASE(20) VM_CASE(21) VM_CASE(22) VM_CASE(23) VM_CASE(24)
      VM_CASE(25) VM_CASE(26) VM_CASE(27) VM_CASE(28) VM_CASE(29) VM_CASE(30) VM_CASE(31) VM_CASE(32)
#undef VM_CASE
      default: __builtin_amdgcn_s_waitcnt(0x0F70); break;
    }
  };
  // wait until the loads of every stage before `first` have landed; stages first .. first+AHEAD-2
  // (those that exist) may still be in flight
  // (more: that later stage exists -- in this pass or, on a walk, in the next)
  auto wait_loads_before = [&](int first, bool more) {
    if (AHEAD == 2) {
      // one later stage can be in flight: none, its NLOADS loads, or those and the scale loads -- three immediates
      // (the general count below compiles to a search tree of scalar branches in every stage)
      if (!more) __builtin_amdgcn_s_waitcnt(0x0F70);
      else if ((first & 3) == 0) __builtin_amdgcn_s_waitcnt(0x0F70 | ((NLOADS + S_LOADS) & 15) | (((NLOADS + S_LOADS) >> 4) << 14));
      else __builtin_amdgcn_s_waitcnt(0x0F70 | (NLOADS & 15) | ((NLOADS >> 4) << 14));
      return;
    }
    int n = 0;
    for (int t = first; t < first + AHEAD - 1; t++)
      if (t < nstage) n += NLOADS + ((t & 3) == 0 ? S_LOADS : 0);
    wait_vm(n);
  };

  floatx16 acc[MF][NF];
#pragma unroll
  for (int mf = 0; mf < MF; mf++)
#pragma unroll
    for (int nf = 0; nf < NF; nf++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[mf][nf][i] = 0.f;

  // Software pipeline with a hand-placed instruction order.  Inside a stage (four 16-wide K
  // steps) every MFMA of step q is followed by one "unit" of step q+1's preparation: one
  // activation fragment read from LDS, or one pair of weights dequantised (3-4 VALU ops), fenced
  // so the compiler keeps the interleave.  The matrix pipe takes a new MFMA every 32 cycles and a
  // unit issues in about 20, so the VALU / LDS work hides behind the MFMAs.  Across stages, the
  // barrier sits in front of the LAST step: by then nobody reads the current LDS buffer any more
  // (step 3's operands are already in registers), so the loads of stage s+2 can overwrite it, and
  // step 0 of stage s+1 is prepared from the other buffer while step 3's MFMAs run.
  half8 a[2][MF];
  H8 b[2][NF];
  uint4 cw[NF], cw8[NF];  // code words of the stage and the same shifted right by 8 (parts 2, 3)
  constexpr int NS = Q4K ? 2 : 1;  // scale sets per stage (Q4_K: the two sub-blocks of the stage)
  half2v as2[NF][NS], bs2[NF][NS];
  half2v as20[DN ? NF : 1];  // DN: the slope for code pairs at bits 4-7 (n * 2^-20): as2 / 16
  float scf[NF];
  uint4 hdr[NF];
  uint4 qh4[Q5 ? NF : 1];  // Q5_K: this lane's 16 qh bytes of the current super-block (code bytes 16 h .. 16 h + 15)
  int q5sh = 0;            // Q5_K: 2 * (stage within the super-block) = the bit of a qh byte that belongs to the stage's low nibbles
  uint32_t k4w[Q4K ? NF : 1][6];  // Q4_K: the current super-block's scale / min fields and (d, d), (-dmin, -dmin)
  const uint8_t* Ab = A0;
  auto load_a1 = [&](int q, int mf, half8* dst) {
    const int m = 32 * mf + n;
    dst[mf] = *(const half8*)(Ab + m * 128 + (((4 * h + q) ^ ((m >> 1) & 7)) << 4));
  };
  // single scale buffer: this lane's scales of four stages, f16 bits packed two to a word (stages 0 | 1, 2 | 3); a
  // stage takes its own with one 64-bit shift (a choice between four registers by the wave-uniform stage index
  // compiles to a tree of scalar branches in every stage)
  uint32_t scp[NSB == 1 ? NF : 1][2];
  auto load_codes = [&](int s, int b) {  // raw codes + this lane's scale of stage s, which lies in buffer b
    if (Q5) q5sh = 2 * (s & 3);
    const uint8_t* Wb = W0 + b * W_BYTES;
    const uint8_t* Sb = S0 + ((s >> 2) & (NSB - 1)) * S_BYTES;
    int g0 = 2 * (s & ~3);
    g0 = g0 + 8 <= ngroups ? g0 : ngroups - 8;
    const int sidx = 2 * s + h - g0;  // this lane's scale inside the staged 8
#pragma unroll
    for (int nf = 0; nf < NF; nf++) {
      cw[nf] = *(const uint4*)(Wb + wrow[nf] * 32 + h * 16);
      if (AFFINE && !Q5) cw8[nf] = uint4{cw[nf].x >> 8, cw[nf].y >> 8, cw[nf].z >> 8, cw[nf].w >> 8};
      if (NSB == 1) {
        // the buffer is rewritten while its stages are still being worked on: take all four
        // stages' values when the first of them is prepared (every wave has by the next barrier;
        // the loads that overwrite it are issued two barriers later)
        if (Q4K) {
          if ((s & 3) == 0) {
            hdr[nf] = *(const uint4*)(Sb + wrow[nf] * 16);
            if (Q5) qh4[nf] = uint4{qhn[2 * nf].x, qhn[2 * nf].y, qhn[2 * nf + 1].x, qhn[2 * nf + 1].y};  // (requested with the header's load, two stages ago)
          }
        } else {
          if (GS == 2) {
            if ((s & 3) == 0) {
              const uint32_t w = *(const uint32_t*)(Sb + wrow[nf] * 4);
              scp[nf][0] = __builtin_amdgcn_perm(w, w, 0x01000100u);  // (lo, lo)
              scp[nf][1] = __builtin_amdgcn_perm(w, w, 0x03020302u);  // (hi, hi)
            }
          } else if ((s & 3) == 0) {
            const uint4 w = *(const uint4*)(Sb + wrow[nf] * 16);
            const uint32_t sel = h ? 0x07060302u : 0x05040100u;  // this lane's half of each word
            scp[nf][0] = __builtin_amdgcn_perm(w.y, w.x, sel);
            scp[nf][1] = __builtin_amdgcn_perm(w.w, w.z, sel);
          }
          const int wi = GS == 2 ? (s & 3) : (sidx - h) >> 1;  // wave-uniform
          const uint64_t both = ((uint64_t)scp[nf][1] << 32) | scp[nf][0];
          union { uint16_t u; _Float16 f; } cv;
          cv.u = (uint16_t)(both >> (16 * wi));
          scf[nf] = (float)cv.f;
        }
      } else {
        if (Q4K) {
          if ((s & 3) == 0) hdr[nf] = *(const uint4*)(Sb + wrow[nf] * 16);
        } else {
          scf[nf] = (float)*(const _Float16*)(Sb + wrow[nf] * 16 + sidx * 2);
        }
      }
    }
  };
  auto scale_consts = [&](int s) {
    if (Q4K) {
      // sub-blocks 2jj and 2jj+1 of the super-block: 6-bit (scale, min) pairs, gguf scale_min_k4.
      // At the first stage of a super-block its 12 packed bytes are spread into four words of byte
      // fields (scales 0-3, scales 4-7, mins 0-3, mins 4-7: nine bit operations for all sixteen)
      // and (d, d), (-dmin, -dmin) are kept as packed halves.  A stage then takes its two bytes of
      // each word straight into the f16 "1024 + n" form with one byte permute, and d * sc, dmin * m
      // are packed f16 products: exact integers times an f16, one rounding, the same values as
      // f16(f32(d) * sc).
      const int jj = s & 3;
      const uint32_t selb = (jj & 1) ? 0x04030402u : 0x04010400u;  // bytes 2,3 or 0,1 of the word | 0x64 above each
#pragma unroll
      for (int nf = 0; nf < NF; nf++) {
        if (jj == 0) {
          const uint4 hd = hdr[nf];
          k4w[nf][0] = hd.y & 0x3f3f3f3fu;
          k4w[nf][1] = (hd.w & 0x0f0f0f0fu) | ((hd.y >> 2) & 0x30303030u);
          k4w[nf][2] = hd.z & 0x3f3f3f3fu;
          k4w[nf][3] = ((hd.w >> 4) & 0x0f0f0f0fu) | ((hd.z >> 2) & 0x30303030u);
          k4w[nf][4] = __builtin_amdgcn_perm(hd.x, hd.x, 0x01000100u);                 // (d, d)
          k4w[nf][5] = __builtin_amdgcn_perm(hd.x, hd.x, 0x03020302u) ^ 0x80008000u;  // (-dmin, -dmin)
        }
        const uint32_t wsc = jj < 2 ? k4w[nf][0] : k4w[nf][1], wmn = jj < 2 ? k4w[nf][2] : k4w[nf][3];
        const half2v k1024 = half2v{(_Float16)1024.f, (_Float16)1024.f};
        const half2v sc = as_h2(__builtin_amdgcn_perm(0x64646464u, wsc, selb)) - k1024;
        const half2v mn = as_h2(__builtin_amdgcn_perm(0x64646464u, wmn, selb)) - k1024;
        union { half2v h; uint32_t u; } a, b;
        a.h = sc * as_h2(k4w[nf][4]);
        b.h = mn * as_h2(k4w[nf][5]);
        as2[nf][0] = as_h2(__builtin_amdgcn_perm(a.u, a.u, 0x01000100u));
        bs2[nf][0] = as_h2(__builtin_amdgcn_perm(b.u, b.u, 0x01000100u));
        as2[nf][NS - 1] = as_h2(__builtin_amdgcn_perm(a.u, a.u, 0x03020302u));
        bs2[nf][NS - 1] = as_h2(__builtin_amdgcn_perm(b.u, b.u, 0x03020302u));
      }
    } else {
#pragma unroll
      for (int nf = 0; nf < NF; nf++) {
        const bool upf = UP && nf >= NH;  // the up half may come from a tensor with a codebook of its own
        if (NAT) {
          const _Float16 sh = (_Float16)scf[nf];  // (exact: the scale is an f16)
          as2[nf][0] = half2v{sh, sh};
          continue;
        }
        const _Float16 as = (_Float16)((upf ? cb_a_up : cb_a) * scf[nf]), bs = (_Float16)((upf ? cb_b_up : cb_b) * scf[nf]);
        as2[nf][0] = half2v{as, as};
        bs2[nf][0] = half2v{bs, bs};
        if (DN) as20[nf] = as2[nf][0] * half2v{(_Float16)0.0625f, (_Float16)0.0625f};  // (exact: a power of two, far from underflow)
      }
    }
  };
  // unit u (0..4*NF-1) of step q: weight fragment nf = u/4, code pair part = u%4 -> one half2 of b
  constexpr int NU = 4 * NF;
  auto deq_unit = [&](int q, int u, H8* dst) {
    const int nf = u >> 2, part = u & 3;
    const uint32_t w = q == 0 ? cw[nf].x : q == 1 ? cw[nf].y : q == 2 ? cw[nf].z : cw[nf].w;
    if (DN) {
      const uint32_t w8 = q == 0 ? cw8[nf].x : q == 1 ? cw8[nf].y : q == 2 ? cw8[nf].z : cw8[nf].w;
      const uint32_t ws = part >= 2 ? w8 : w;
      if ((part & 1) == 0) dst[nf].h[part] = as_h2(ws & 0x000f000fu) * as2[nf][0] + bs2[nf][0];
      else dst[nf].h[part] = as_h2(ws & 0x00f000f0u) * as20[DN ? nf : 0] + bs2[nf][0];
    } else if (AFFINE) {
      // (Q5_K shifts on the spot: it has no registers to spare for the shifted copies)
      const uint32_t w8 = Q5 ? w >> 8 : q == 0 ? cw8[nf].x : q == 1 ? cw8[nf].y : q == 2 ? cw8[nf].z : cw8[nf].w;
      const uint32_t ws = part >= 2 ? w8 : w;
      const int ss = Q4K ? (part & 1) : 0;  // Q4_K: odd parts are the high nibbles = the stage's second sub-block
      uint32_t t;
      // Q5_K: the qh word of these four code bytes; the pair's two fifth bits go to bit 4 / 20 (low nibbles: value 16
      // on top of 1024 + n) or bit 8 / 24 (high nibbles: 16 on top of 64 + n, whose unit is bit 4)
      uint32_t q5 = 0;
      if (Q5) {
        const uint32_t qw = q == 0 ? qh4[nf].x : q == 1 ? qh4[nf].y : q == 2 ? qh4[nf].z : qh4[nf].w;
        // bytes 0, 2 (parts 0, 1) or 1, 3 (parts 2, 3); bit 2 jj (low nibbles) or 2 jj + 1 (high nibbles) of each
        const int from = (part >= 2 ? 8 : 0) + q5sh + (part & 1), to = (part & 1) ? 8 : 4;
        q5 = __builtin_amdgcn_alignbit(qw, qw, (uint32_t)(from - to) & 31u);  // rotate: the mask below drops the rest
      }
      if ((part & 1) == 0) {
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(t) : "v"(ws), "s"(0x000f000fu), "v"(0x64006400u));
        if (Q5) asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(t) : "v"(q5), "s"(0x00100010u), "v"(t));
        dst[nf].h[part] = (as_h2(t) - half2v{(_Float16)1024.f, (_Float16)1024.f}) * as2[nf][ss] + bs2[nf][ss];
      } else {
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(t) : "v"(ws), "s"(0x00f000f0u), "v"(0x54005400u));
        if (Q5) asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(t) : "v"(q5), "s"(0x01000100u), "v"(t));
        dst[nf].h[part] = (as_h2(t) - half2v{(_Float16)64.f, (_Float16)64.f}) * as2[nf][ss] + bs2[nf][ss];
      }
    } else {
      if (NAT) {
        // byte `part` of the word = weights 2 part, 2 part + 1 of the step in natural order: one look-up gives both as
        // f16(cb), one packed product applies the scale: w = f16(f16(cb[n]) * scale), the reference kernel's contract
        // (src/gpu/parts/27_kernels_moe_lut.inc:16)
        const uint32_t* pt = (UP && nf >= NH) ? ptab + 256 : ptab;
        dst[nf].h[part] = as_h2(pt[(w >> (8 * part)) & 0xffu]) * as2[nf][0];
      } else {
        half2v hv;
        const float* tb = (UP && nf >= NH) ? cbs + 16 : cbs;
        hv.x = (_Float16)(tb[(w >> (4 * part)) & 0xf] * scf[nf]);
        hv.y = (_Float16)(tb[(w >> (4 * part + 16)) & 0xf] * scf[nf]);
        dst[nf].h[part] = hv;
      }
    }
    // The unit stays where it is written: without a use in its own block the compiler moves a unit's instructions down
    // into the block of the MFMA that reads them (past the branches of the load slots, past the stage barrier), where
    // they run in a row in front of that MFMA instead of one by one behind the earlier ones.
    asm volatile("" : "+v"(dst[nf].u[part]));
  };
  constexpr int NM = NF * MF;                     // MFMAs per K step
  constexpr int UPM = (NU + NM - 1) / NM;         // dequant units behind each MFMA (steps 0-2)
  constexpr int X0 = NM >= 8 ? NM / 4 : 1;        // step 3: first MFMA slot that dequantises
  constexpr int XPM = (NU + NM - X0 - 1) / (NM - X0);

  // Loads run AHEAD stages ahead of the MFMAs.  The first stages' weight loads go out before the
  // tile's row indices (a dependent global load made by the caller, `ri`) are needed: the weights'
  // trip to HBM then overlaps the index fetch instead of following it.
#pragma unroll
  for (int t = 0; t < AHEAD; t++)
    if (t < nstage) issue_w(t);
  float xms_v = 1.f;
  if (tid < BM) {
    rowidx[tid] = ri;
    if (UP && xms) xms_v = xms[ri];  // for the epilogue; the wait for it comes after the K loop
  }
  // barrier for the LDS row indices only: __syncthreads() would also wait for the weight loads
  // just issued (its fence drains the vector memory counter), a full trip to HBM
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
#pragma unroll
  for (int i = 0; i < A_LOADS; i++) {
    const int m = 8 * a_grp[i] + (lane >> 3);
    a_src[i] = x + (size_t)rowidx[m] * K + (((lane & 7) ^ ((m >> 1) & 7)) << 3);
    if (Q5) a_off[Q5 ? i : 0] = ((uint32_t)rowidx[m] * (uint32_t)K + (((lane & 7) ^ ((m >> 1) & 7)) << 3)) * 2u;
  }
#pragma unroll
  for (int t = 0; t < AHEAD; t++)
    if (t < nstage) issue_a(t);
  // stage 0 must have landed; only the activation loads of the later stages may still be in flight
  wait_vm(nstage > 1 ? A_LOADS * (AHEAD - 1) : 0);
  moe_lds_barrier();  // the later stages' loads stay in flight
  load_codes(0, 0);
#pragma unroll
  for (int mf = 0; mf < MF; mf++) load_a1(0, mf, a[0]);
  scale_consts(0);
#pragma unroll
  for (int u = 0; u < NU; u++) deq_unit(0, u, b[0]);

  // `epilogue` (below the loop in the source) writes one column block's results; cbuf = the stage buffer that the
  // pipeline has just left (a walk's patch lives there)
  auto run = [&](auto&& epilogue) {
  int s = 0, p = 0, cbuf = 0;  // stage within the pass, pass, the stage's LDS buffer
  const int nvs = nstage * npass;
  for (int v = 0; v < nvs; v++) {
    Ab = A0 + cbuf * A_BYTES;
    // the stage whose loads go out during step 0: AHEAD stages on, in the next pass where this one ends before
    int is = s + AHEAD, ip = p;
    if (is >= nstage) { is -= nstage; ip++; }
    const bool pf = ip < npass;
    const bool pf_s = pf && (is & 3) == 0;
    const int ib = cbuf + AHEAD >= NBUF ? cbuf + AHEAD - NBUF : cbuf + AHEAD;
    const size_t ipw = (size_t)ip * wpass, ips = (size_t)ip * spass;
#pragma unroll
    for (int q = 0; q < 3; q++) {
      const int cur = q & 1, nxt = cur ^ 1;
#pragma unroll
      for (int i = 0; i < NM; i++) {
        const int mf = i / NF, nf = i % NF;
        mfma16(acc[mf][nf], a[cur][mf], b[cur][nf].v);
        __builtin_amdgcn_sched_barrier(0);
        if (i < MF) load_a1(q + 1, i, a[nxt]);
#pragma unroll
        for (int k = 0; k < UPM; k++)
          if (i * UPM + k < NU) deq_unit(q + 1, i * UPM + k, b[nxt]);
        if (q == 0) {
          // buffer ib was last read in the stage before this one: free since the previous barrier
          constexpr int LPS = (NLOADS + S_LOADS + NM - 1) / NM;  // loads per MFMA slot
#pragma unroll
          for (int k = 0; k < LPS; k++) {
            const int u = i * LPS + k;
            if (u < NLOADS) { if (pf) issue_unit(is, ib, ipw, ips, u); }
            else if (u < NLOADS + S_LOADS) { if (pf_s) issue_unit(is, ib, ipw, ips, u); }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // last step: a[1], b[1] hold its operands.  Step 0 of the next stage is prepared from the next
    // buffer meanwhile, so that buffer must be complete and visible: loads of the next stage done
    // (the one after it may still fly), then the block barrier.
    const int sn = s + 1 == nstage ? 0 : s + 1;            // the next stage (on a walk: of the next pass after the last)
    const int nbuf = cbuf + 1 == NBUF ? 0 : cbuf + 1;
    wait_loads_before(s + 2, v + 2 < nvs);
    moe_lds_barrier();  // (not __syncthreads(): its fence would wait for the loads just issued two stages ahead)
    Ab = A0 + nbuf * A_BYTES;
#pragma unroll
    for (int i = 0; i < NM; i++) {
      const int mf = i / NF, nf = i % NF;
      mfma16(acc[mf][nf], a[1][mf], b[1][nf].v);
      __builtin_amdgcn_sched_barrier(0);
      // (past the last stage of the last pass this reads stale LDS and the result is never used)
      if (i == 0) load_codes(sn, nbuf);
      if (i < MF) load_a1(0, i, a[0]);
      if (i == X0) scale_consts(sn);
      if (i >= X0) {
#pragma unroll
        for (int k = 0; k < XPM; k++)
          if ((i - X0) * XPM + k < NU) deq_unit(0, (i - X0) * XPM + k, b[0]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (WALK && sn == 0) {  // a pass ends: its column block goes out, the accumulators start over
      epilogue(nb + p, cbuf);
      p++;
      // The patch is the wave's quarter of the buffer.  With all four row fragments live those are exactly the bytes
      // that the wave's own loads write (activation row groups 4 wv .. 4 wv + 3), so whoever runs ahead cannot touch
      // another wave's patch; a tile with fewer fragments deals its row groups to the waves differently, and the
      // block has to meet before the next loads into this buffer go out.
      if (MF < 4 && p < npass) moe_lds_barrier();
#pragma unroll
      for (int mf = 0; mf < MF; mf++)
#pragma unroll
        for (int nf = 0; nf < NF; nf++)
#pragma unroll
          for (int i = 0; i < 16; i++) acc[mf][nf][i] = 0.f;
    }
    s = sn;
    cbuf = nbuf;
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // no LDS-bound load may outlive the block
  if (!WALK) {
    if (UP) {
      if (tid < BM) rowscale[tid] = xms ? moe_hid_scale(cmag, xms_v) : 1.f;
      __syncthreads();
    }
    epilogue(nb, 0);
  }
  };

  // epilogue.  D[i][j]: j = lane%32 (weight row), i = 8*(r/4) + 4*(lane/32) + r%4 (pair).
  // f16 results go through a per-wave LDS patch (the stage buffers are dead by now) so that global
  // stores are 16 bytes per lane and whole rows are contiguous.
  constexpr int NC = UP ? 32 * NH : 32 * NF;  // output columns of this wave
  auto epilogue = [&](int nb, int cbuf) {     // nb: the column block that the accumulators hold
  const int colbase = UP ? nb * HALF + NC * wv : nb * WROWS + NC * wv;
  if constexpr (ROT) {
    // hgn v2 rotated experts: the block holds the raw sums of one 128-block of gate columns and of the matching up
    // columns for its pairs, which is what the slot-wise middle works on -- rot_out, SwiGLU, rot_in of the block
    // (hgn_v2.hip, k_i4r_mid) -- so it runs here instead of as a launch of its own behind a round trip of the sums
    // through memory.  The sums cross the waves through LDS as f16 (the rounding that the unfused form's f16 rows
    // in memory have), then 16 lanes take a pair row each, 8 columns a lane.
    constexpr int BP = 2 * HALF * 2 + 16;  // [128 gate | 128 up] f16 + padding: rows m and m + 4 on different banks
    static_assert(BM * BP <= NBUF * (A_BYTES + W_BYTES), "the patch fits the stage buffers");
    uint8_t* patch = smem;
#pragma unroll
    for (int mf = 0; mf < MF; mf++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int ml = 8 * (r >> 2) + 4 * h + (r & 3);
        uint8_t* prow = patch + (32 * mf + ml) * BP + (NC * wv + n) * 2;
        *(__half*)prow = __float2half(acc[mf][0][r]);
        *(__half*)(prow + HALF * 2) = __float2half(acc[mf][1][r]);
      }
    }
    __syncthreads();
    const int j = tid & 15;
    const int c = nb * HALF + 8 * j;  // this lane's 8 columns of the expert's hid
    float fg[8], fu[8], sd[8];
    {
      const int cc = c < M ? c : 0;
      const float4* pg = (const float4*)(rot.svh_gu + cc);
      const float4* pu = (const float4*)(rot.svh_gu + M + cc);
      const float4* pd = (const float4*)(rot.suh_dn + cc);
      const float4 a0 = pg[0], a1 = pg[1], b0 = pu[0], b1 = pu[1], d0 = pd[0], d1 = pd[1];
      fg[0] = a0.x; fg[1] = a0.y; fg[2] = a0.z; fg[3] = a0.w; fg[4] = a1.x; fg[5] = a1.y; fg[6] = a1.z; fg[7] = a1.w;
      fu[0] = b0.x; fu[1] = b0.y; fu[2] = b0.z; fu[3] = b0.w; fu[4] = b1.x; fu[5] = b1.y; fu[6] = b1.z; fu[7] = b1.w;
      sd[0] = d0.x; sd[1] = d0.y; sd[2] = d0.z; sd[3] = d0.w; sd[4] = d1.x; sd[5] = d1.y; sd[6] = d1.z; sd[7] = d1.w;
    }
#pragma unroll 1
    for (int m = tid >> 4; m < 32 * MF; m += NT / 16) {
      const uint4 gq = *(const uint4*)(patch + m * BP + j * 16), uq = *(const uint4*)(patch + m * BP + HALF * 2 + j * 16);
      const __half2* gh = (const __half2*)&gq;
      const __half2* uh = (const __half2*)&uq;
      float g[8], u[8], hv[8];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const float2 a = __half22float2(gh[i]), b = __half22float2(uh[i]);
        g[2 * i] = a.x; g[2 * i + 1] = a.y; u[2 * i] = b.x; u[2 * i + 1] = b.y;
      }
      moe_fwht128_r8(g, lane);
      moe_fwht128_r8(u, lane);
      const float rs = rowscale[m];
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const float gv = g[i] * MOE_RS128 * fg[i], uv = u[i] * MOE_RS128 * fu[i];  // (the slot-wise middle's own arithmetic)
        hv[i] = gv * __builtin_amdgcn_rcpf(1.f + __expf(-gv)) * uv * (sd[i] * rs);
      }
      moe_fwht128_r8(hv, lane);
#pragma unroll
      for (int i = 0; i < 8; i++) hv[i] *= MOE_RS128;
      if (m < tile.count && c < M) moe_st8_f16_ilv((__half*)out + (size_t)(tile.first + m) * M + c, hv);
    }
  } else if constexpr (UP) {
    // gate/up: a wave holds 32 of the block's HALF hid columns, 64 bytes of a row -- stored per wave, the two halves of
    // a 128-byte line reach memory separately (measured: 2.3 times the payload written).  So the block's waves put
    // their columns into one patch of whole rows and every store instruction writes complete lines.
    constexpr int BP = HALF * 2 + 16;  // row pitch of the block-wide patch in bytes
    uint8_t* patch = smem;
#pragma unroll
    for (int mf = 0; mf < MF; mf++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int ml = 8 * (r >> 2) + 4 * h + (r & 3);
#pragma unroll
        for (int f = 0; f < NH; f++) {
          const float g = DN ? acc[mf][f][r] * oscale : acc[mf][f][r], u = DN ? acc[mf][NH + f][r] * oscale : acc[mf][NH + f][r];
          // hardware reciprocal (1 ulp) instead of the IEEE division sequence: the result is rounded
          // to f16 below, and this epilogue is VALU time during which the matrix pipe idles
          const float hv = g * __builtin_amdgcn_rcpf(1.f + __expf(-g)) * u * rowscale[32 * mf + ml];
          // hid feeds the down GEMM: permuted order inside groups of 8 (q4cp) / blocks of 64 (Q4_K)
          int pos;
          if (NAT) {
            pos = 32 * f + n;  // natural order
          } else if (!Q4K) {
            const int c = 32 * f + n;
            pos = (c & ~7) + ilv_pos(c & 7);
          } else if (NH == 1) {
            // lane n holds row 16q + (n&15) + 2*(n&16) of the block: chunks 4q..4q+3 -> local 0..31
            pos = q4k_pos((n & 15) + 2 * (n & 16));
          } else {
            pos = q4k_pos(32 * f + n);
          }
          *(__half*)(patch + (32 * mf + ml) * BP + (NC * wv + pos) * 2) = __float2half(hv);
        }
      }
    }
    __syncthreads();
    constexpr int CH = HALF / 8;  // 16-byte chunks per row
#pragma unroll
    for (int it = 0; it < (32 * MF * CH + NT - 1) / NT; it++) {
      const int c = it * NT + tid, m = c / CH, c8 = c % CH;
      if (c < 32 * MF * CH) {
        const uint4 v = *(const uint4*)(patch + m * BP + c8 * 16);
        const int col = nb * HALF + c8 * 8;
        if (m < tile.count && col < M) *(uint4*)((__half*)out + (size_t)(tile.first + m) * M + col) = v;
      }
    }
  } else if constexpr (F16OUT) {
    // down: a wave's 64 columns are whole 128-byte lines of a row; a per-wave patch turns the accumulators' layout into
    // 16-byte stores.  The patch is the wave's own quarter of the activation buffer that the pipeline has just left,
    // 32 rows of NC f16 without padding; rows 4..7 of every eight swap their row halves, which puts the two lane
    // halves of a store (rows m and m + 4, same columns) on different banks.
    // (Measured and dropped: the two MFMA operands exchanged, which transposes the accumulators so that, after one
    //  v_permlane32_swap between the lane halves, a lane holds 8 neighbouring f16 of one row and stores them without
    //  LDS -- 32 bytes of a row per lane pair and instruction: 4 % slower than this patch, whose stores are whole lines.)
#if MOE_GEMM_NF == 2 && MOE_GEMM_WROWS == 256
    static_assert(32 * NC * 2 * NW <= A_BYTES && NC * 2 == 128, "the patch is a wave's share of one activation buffer");
    uint8_t* patch = A0 + cbuf * A_BYTES + wv * (32 * NC * 2);
    // (the lane's coordinates pass through an opaque copy: on a walk the epilogue sits inside the K loop, and address
    //  terms derived from the plain values would be computed ahead of the loop and held in registers through it)
    int lq = lane;
    asm volatile("" : "+v"(lq));
    const int nq = lq & 31, hq = lq >> 5;
#pragma unroll
    for (int mf = 0; mf < MF; mf++) {
      // row 4 h + ..., column 32 nf + n at byte 2 n + 64 (nf ^ h) of the row
      static_assert(NF == 2, "two 32-column halves per wave");
      uint8_t* const wr0 = patch + (4 * hq) * 128 + nq * 2 + 64 * hq;
      uint8_t* const wr1 = patch + (4 * hq) * 128 + nq * 2 + 64 * (1 - hq);
#pragma unroll
      for (int r = 0; r < 16; r++) {
#pragma unroll
        for (int nf = 0; nf < NF; nf++)
          *(__half*)((nf ? wr1 : wr0) + (8 * (r >> 2) + (r & 3)) * 128) = __float2half(DN ? acc[mf][nf][r] * oscale : acc[mf][nf][r]);
      }
      // 32 rows x NC columns -> NC/8 16-byte chunks per row
      constexpr int CPR = NC / 8;
      constexpr int ITS = (32 * CPR + 63) / 64;
      static_assert(CPR == 8 && ITS == 4, "eight 16-byte chunks per row, eight rows per instruction");
      const int ml0 = lq >> 3, c8 = lq & 7;
      const uint8_t* const rd = patch + ml0 * 128 + ((c8 * 16) ^ (((ml0 >> 2) & 1) << 6));
      __half* const orow = (__half*)out + (size_t)(tile.first + 32 * mf + ml0) * M + (colbase + c8 * 8);
#pragma unroll
      for (int it = 0; it < ITS; it++) {
        const uint4 v = *(const uint4*)(rd + it * 8 * 128);  // rows ml0 + 8 it: the same halves swapped
        const int m = 32 * mf + ml0 + 8 * it;
        if (m < tile.count && colbase + c8 * 8 < M) *(uint4*)(orow + (size_t)(8 * it) * M) = v;
      }
    }
#endif  // (other fragment counts per wave: timing experiments of the gate/up launch only)
  } else if (cmb.y) {
    // fused weighted combine: the tile's rows are added straight into their tokens' output rows
    // (f32 atomics executed in L2, no value returned), weight = the pair's routing weight (the
    // shared expert's: sigmoid of its gate logit) over the f16 range-guard factor of the token.
    // A half-wave covers 32 consecutive floats of one output row per instruction.
    __syncthreads();  // every wave is past its last use of rowidx
    if (tid < BM) {
      const int p = tile.first + (tid < tile.count ? tid : 0);
      const int t = cmb.tokidx[p];
      float w = shared ? sigmoid_f(cmb.sg[t]) : cmb.pw[p];
      if (xms) w /= moe_hid_scale(cmag, xms[t]);
      rowidx[tid] = t;
      rowscale[tid] = w;
    }
    __syncthreads();
#pragma unroll
    for (int mf = 0; mf < MF; mf++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int m = 32 * mf + 8 * (r >> 2) + 4 * h + (r & 3);
        if (m >= tile.count) continue;
        float* yrow = cmb.y + (size_t)rowidx[m] * M;
        const float w = rowscale[m] * oscale;
#pragma unroll
        for (int nf = 0; nf < NF; nf++) {
          const int col = colbase + 32 * nf + n;
          if (col < M) unsafeAtomicAdd(yrow + col, w * acc[mf][nf][r]);
        }
      }
    }
  } else {
#pragma unroll
    for (int mf = 0; mf < MF; mf++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int m = 32 * mf + 8 * (r >> 2) + 4 * h + (r & 3);
        if (m >= tile.count) continue;
#pragma unroll
        for (int nf = 0; nf < NF; nf++) {
          const int col = colbase + 32 * nf + n;
          if (col < M) ((float*)out)[(size_t)(tile.first + m) * M + col] = DN ? acc[mf][nf][r] * oscale : acc[mf][nf][r];
        }
      }
    }
  }
  };
  run(epilogue);
}

template <bool UP, bool F16OUT, bool Q4K, int GS, bool Q5 = false, bool NAT = false, bool ROT = false>
__global__ void __launch_bounds__(NT, WPE)
k_moe_gemm_q4cp(LutDev R, LutDev Sh, int n_experts, const __half* __restrict__ x,
                const int* __restrict__ tokidx, const moe_tile* __restrict__ tiles,
                const int* __restrict__ ntiles, void* __restrict__ out, int M, int K, int nblk_n, int split,
                moe_hscale hs, moe_comb cmb, int npass, moe_rotv rot) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  float* cbs = (float*)(smem + NBUF * (A_BYTES + W_BYTES) + NSB * S_BYTES);
  // XCD-aware order: consecutive workgroup ids go round-robin over the 8 XCDs; give each XCD a
  // contiguous run of tiles so that tiles of one expert share that XCD's L2.
  // Routed tiles and shared-expert tiles (all full) are dealt out separately, or the XCD that
  // gets the tail of the list would carry every shared tile.
  const int nt = ntiles[0];
  const int nr = split ? ntiles[1] : nt;  // routed tiles come first in the list
  const int wg = blockIdx.x, xcd = wg & 7, j = wg >> 3;
  const int per_r = (nr + 7) >> 3, per_s = (nt - nr + 7) >> 3;
  const int tl = j / nblk_n, nb = (j - tl * nblk_n) * npass;  // (nblk_n: groups of npass column blocks per tile)
  int ti;
  if (tl < per_r) {
    ti = xcd * per_r + tl;
    if (ti >= nr) return;
  } else {
    const int k2 = tl - per_r;
    ti = nr + xcd * per_s + k2;
    if (k2 >= per_s || ti >= nt) return;
  }
  const moe_tile tile = tiles[ti];
  const bool shared = tile.expert >= n_experts;
  // (field by field: a reference to one of the two argument structs would put both on the stack)
  LutDev L;
  L.w = shared ? Sh.w : R.w;
  L.w_up = shared ? Sh.w_up : R.w_up;
  L.sc = shared ? Sh.sc : R.sc;
  L.sc_up = shared ? Sh.sc_up : R.sc_up;
  L.cb = shared ? Sh.cb : R.cb;
  L.cb_up = shared ? Sh.cb_up : R.cb_up;
  L.sstride = shared ? Sh.sstride : R.sstride;
  L.e_rows = shared ? Sh.e_rows : R.e_rows;
  L.up_off = shared ? Sh.up_off : R.up_off;
  L.pexp = shared ? Sh.pexp : R.pexp;
  const int e = shared ? 0 : tile.expert;
  // scaled dequantisation: the expert's power of two (requested here, used after the first loads have gone out)
  int pexp = MOE_PEXP_NONE;
  if (!Q4K && GS == 0 && !NAT && L.pexp) pexp = L.pexp[e];
  const int tid = threadIdx.x, lane = tid & 63;

  // the tile's row indices: requested before the codebook is looked at, so that the two round trips
  // overlap; used inside gemm_tile, after its first weight loads
  int ri = 0;
  if (tid < BM) {
    const int m = tid < tile.count ? tid : 0;  // rows past the tile read a valid row, never stored
    ri = tokidx ? tokidx[tile.first + m] : tile.first + m;
  }

  // q4cp codebook: affine (a*n+b) or table.  Q4_K has no codebook (w = (d*sc)*n - dmin*m).
  bool affine = true;
  float cb_a = 1.f, cb_b = 0.f, cb_a_up = 1.f, cb_b_up = 0.f;
  if (NAT) {
    // pair tables: entry b = (f16(cb[b & 15]), f16(cb[b >> 4])) = the two weights of code byte b before scaling
    uint32_t* pt = (uint32_t*)(smem + SMEM_BYTES);
    const float* cbu = UP ? L.cb_up : L.cb;
    for (int i = tid; i < 256; i += NT) {
      union { half2v h; uint32_t u; } g, u;
      g.h = half2v{(_Float16)L.cb[i & 15], (_Float16)L.cb[i >> 4]};
      u.h = half2v{(_Float16)cbu[i & 15], (_Float16)cbu[i >> 4]};
      pt[i] = g.u;
      pt[256 + i] = u.u;
    }
    affine = false;
  } else if (!Q4K) {
    // lanes 0..15: the (gate) rows' codebook, lanes 16..31: the up rows' (the same table unless the two
    // halves come from separately quantised tensors, as a shared expert's gate_proj / up_proj do)
    const float* cbu = UP ? L.cb_up : L.cb;
    const float c0 = L.cb[0], c1 = L.cb[1], u0 = cbu[0], u1 = cbu[1];
    bool aff = true;
    if (lane < 32) {
      const int nn = lane & 15;
      const bool upl = lane >= 16;
      const float v = upl ? cbu[nn] : L.cb[nn];
      aff = v == fmaf((float)nn, upl ? u1 - u0 : c1 - c0, upl ? u0 : c0);
      if (tid < 32) cbs[lane] = v;
    }
    affine = __all(aff);
    cb_a = c1 - c0;
    cb_b = c0;
    cb_a_up = u1 - u0;
    cb_b_up = u0;
  }

  const moe_cmag cmag = shared ? hs.c_shared : hs.c_routed;
  __syncthreads();  // cbs
  const int mfn = (tile.count + 31) >> 5;
#define GEMM_ARGS smem, L, e, tile, nb, x, out, M, K, cb_a, cb_b, cb_a_up, cb_b_up, ri, hs.xms, cmag, cmb, shared
#define GEMM_TAIL 0, npass
#define GEMM_GO(MF)                                                                                     \
  do {                                                                                                  \
    if constexpr (ROT) gemm_tile<UP, F16OUT, MF, true, false, GS, false, false, false, true>(GEMM_ARGS, GEMM_TAIL, rot); \
    else if constexpr (NAT) gemm_tile<UP, F16OUT, MF, false, false, 0, false, true>(GEMM_ARGS, GEMM_TAIL);   \
    else {                                                                                              \
      bool scaled = false;                                                                              \
      if constexpr (!Q4K && GS == 0) {                                                                  \
        if (affine && pexp != MOE_PEXP_NONE) {                                                          \
          gemm_tile<UP, F16OUT, MF, true, false, 0, false, false, true>(GEMM_ARGS, pexp, npass);        \
          scaled = true;                                                                                \
        }                                                                                               \
      }                                                                                                 \
      if (!scaled) {                                                                                    \
        if (Q4K || affine) gemm_tile<UP, F16OUT, MF, true, Q4K, GS, Q5>(GEMM_ARGS, GEMM_TAIL);          \
        else gemm_tile<UP, F16OUT, MF, false, false, GS, false>(GEMM_ARGS, GEMM_TAIL);                  \
      }                                                                                                 \
    }                                                                                                   \
  } while (0)
  if (mfn <= 1) GEMM_GO(1);
  else if (mfn == 2) GEMM_GO(2);
  else if (mfn == 3) GEMM_GO(3);
  else if (BM <= 128 || mfn == 4) GEMM_GO(4);
  else if constexpr (BM > 128) {
    if (mfn <= 6) GEMM_GO(6);
    else GEMM_GO(8);
  }
#undef GEMM_ARGS
#undef GEMM_TAIL
#undef GEMM_GO
}

LutDev to_dev(const moe_lutw* p, const float* cb_up, const int8_t* pexp) {
  LutDev d{};
  d.pexp = pexp;
  if (p) {
    d.w = p->w; d.w_up = p->w_up; d.sc = p->sc; d.sc_up = p->sc_up; d.cb = p->cb;
    d.cb_up = cb_up ? cb_up : p->cb;
    d.sstride = p->sstride; d.e_rows = p->e_rows; d.up_off = p->up_off;
  }
  return d;
}

bool lut_ok(const moe_lutw* p, bool pair, int k, bool q4k, int gs = 0) {
  if (gs == 2) {  // one scale per 128 columns, unpadded scale rows; whole 256-column scale windows
    if (q4k || !p || !p->w || !p->sc || !p->cb || k < 256 || k % 256) return false;
    if (pair && (!p->w_up || !p->sc_up || !moe_aligned(p->w_up, 16) || !moe_aligned(p->sc_up, 4))) return false;
    return moe_aligned(p->w, 16) && moe_aligned(p->sc, 4) && p->sstride % 4 == 0 && p->sstride >= k / 128 * 2;
  }
  if (q4k) {  // raw Q4_K rows: only the code pointers are used
    if (!p || !p->w || (pair && !p->w_up) || k < 256 || k % 256) return false;
    return moe_aligned(p->w, 16) && (!pair || moe_aligned(p->w_up, 16));
  }
  if (!p || !p->w || !p->sc || !p->cb) return false;
  if (pair && (!p->w_up || !p->sc_up)) return false;
  if (k < 256 || k % 128) return false;
  if (!moe_aligned(p->w, 16) || !moe_aligned(p->sc, 4) || p->sstride % 4 || p->sstride < k / 32 * 2) return false;
  if (pair && (!moe_aligned(p->w_up, 16) || !moe_aligned(p->sc_up, 4))) return false;
  return true;
}

}  // namespace

namespace {
// One block per expert: hi = exponent of |slope| * (largest |scale| of the expert), lo = exponent of |slope| * (the
// smallest of the rows' largest scales; rows of zeros left out), as frexp gives them; hi = 127: the scaled
// dequantisation does not apply (a scale or the slope not finite, slope zero); hi = -127: every scale is zero.
__global__ void __launch_bounds__(256) k_q4cp_scale_span(const uint8_t* __restrict__ sc, const float* __restrict__ cb,
                                                         int sstride, int rows, int groups, int8_t* __restrict__ span) {
  __shared__ float s_hi[256], s_lo[256];
  __shared__ int s_bad[256];
  const int e = blockIdx.x, tid = threadIdx.x;
  const uint8_t* base = sc + (size_t)e * rows * sstride;
  float hi = 0.f, lo = INFINITY;
  int bad = 0;
  for (int r = tid; r < rows; r += 256) {
    const __half* row = (const __half*)(base + (size_t)r * sstride);
    float rm = 0.f;
    for (int g = 0; g < groups; g++) {
      const float v = fabsf(__half2float(row[g]));
      if (!(v <= 65504.f)) bad = 1;
      rm = fmaxf(rm, v);
    }
    hi = fmaxf(hi, rm);
    if (rm > 0.f) lo = fminf(lo, rm);
  }
  s_hi[tid] = hi; s_lo[tid] = lo; s_bad[tid] = bad;
  __syncthreads();
  for (int o = 128; o; o >>= 1) {
    if (tid < o) {
      s_hi[tid] = fmaxf(s_hi[tid], s_hi[tid + o]);
      s_lo[tid] = fminf(s_lo[tid], s_lo[tid + o]);
      s_bad[tid] |= s_bad[tid + o];
    }
    __syncthreads();
  }
  if (tid == 0) {
    const float a = fabsf(cb[1] - cb[0]);
    int h = 127, l = 127;
    if (!s_bad[0] && a > 0.f && a <= 3.0e38f) {
      if (s_hi[0] == 0.f) {
        h = l = -127;
      } else {
        int eh, el;
        (void)frexpf(a * s_hi[0], &eh);
        (void)frexpf(a * s_lo[0], &el);
        if (a * s_hi[0] <= 3.0e38f && a * s_lo[0] > 0.f && eh < 100 && el > -100) { h = eh; l = el; }
      }
    }
    span[2 * e] = (int8_t)h;
    span[2 * e + 1] = (int8_t)l;
  }
}
}  // namespace

int moe_q4cp_scale_span(const moe_wview* w, int n_experts, int8_t* span_dev, hipStream_t st) {
  if (!w || !w->data || !span_dev || n_experts < 1 || w->rows % (uint64_t)n_experts || w->cols % 32) return MOE_E_INVALID;
  const Q4cpOps o = q4cp_ops(w);
  k_q4cp_scale_span<<<n_experts, 256, 0, st>>>(o.scales, o.cb, (int)o.scale_stride, (int)(w->rows / n_experts),
                                               (int)(w->cols / 32), span_dev);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

// hi_lo_b may be null (one tensor)
int moe_pexp_from_span(const int8_t* a, const int8_t* b) {
  int hi = a[0], lo = a[1];
  if (hi == 127) return MOE_PEXP_NONE;
  if (b) {
    if (b[0] == 127) return MOE_PEXP_NONE;
    if (hi == -127) { hi = b[0]; lo = b[1]; }
    else if (b[0] != -127) { hi = b[0] > hi ? b[0] : hi; lo = b[1] < lo ? b[1] : lo; }
  }
  if (hi == -127) return 0;          // nothing but zeros: any power will do
  if (hi - lo > 5) return MOE_PEXP_NONE;
  const int P = -9 - hi;             // |slope| * scale * 2^(24+P) < 2^15
  return P < -100 || P > 100 ? MOE_PEXP_NONE : P;
}

bool moe_gemm_q5k_fits(uint64_t rows, uint64_t x_rows, int k) {
  const uint64_t lim = (1ull << 32) - (1ull << 16);
  return k > 0 && k % 256 == 0 && rows * (uint64_t)(k / 256 * 176) < lim && x_rows * (uint64_t)k * 2 < lim;
}

// Internal: routed + (optional) shared expert in one launch; tile.expert >= n_experts selects Sh.
// sh_cb_up: codebook of the shared expert's up rows when they are a tensor of their own (nullptr: sh->cb).
// q4k: the views hold raw GGUF Q4_K rows (w / w_up only) instead of q4cp planes.
int moe_launch_gemm_q4cp(bool up, const moe_lutw* routed, const moe_lutw* sh, int n_experts,
                         const __half* x, const int* tokidx, const moe_tile* tiles, const int* ntiles,
                         int max_tiles, void* out, int m, int k, bool f16out, bool q4k, moe_hscale hs,
                         hipStream_t st, const moe_comb* comb, const float* sh_cb_up, int gs, bool q5k, bool nat,
                         const int8_t* pexp_routed, const int8_t* pexp_sh, const moe_rotv* rot) {
  if (!x || !tiles || !ntiles || !out || max_tiles < 0) return MOE_E_INVALID;
  // (the rotated experts' fused form: gate/up rows with one scale per 128 columns, whole 128-blocks of hid, no shared
  //  expert's tiles in the same launch)
  if (rot && (!up || gs != 2 || sh || comb || !f16out || m % 128 || !rot->svh_gu || !rot->suh_dn ||
              !moe_aligned(rot->svh_gu, 16) || !moe_aligned(rot->suh_dn, 16)))
    return MOE_E_INVALID;
  if (up && gs == 2 && !rot) return MOE_E_UNSUPPORTED;
  if (nat && (q4k || q5k || gs != 0)) return MOE_E_UNSUPPORTED;  // (natural K order: q4cp planes through pair tables)
  if (q5k && (!q4k || !up || comb)) return MOE_E_UNSUPPORTED;  // (Q5_K: gate/up tensors, the reference checkpoints' use of it)
  // (Q5_K: 32-bit byte offsets into the tensors; the caller vouches for the activation rows, moe_gemm_q5k_fits)
  if (q5k && routed && !moe_gemm_q5k_fits((uint64_t)(sh == routed ? 1 : n_experts) * (uint64_t)routed->e_rows + (uint64_t)routed->up_off + (uint64_t)m, 0, k))
    return MOE_E_UNSUPPORTED;
  if (q5k && sh && sh != routed && !moe_gemm_q5k_fits((uint64_t)sh->e_rows + (uint64_t)sh->up_off + (uint64_t)m, 0, k))
    return MOE_E_UNSUPPORTED;
  if (gs != 0 && (gs != 2 || (up && !rot) || !f16out || q4k || sh || comb)) return MOE_E_UNSUPPORTED;
  moe_comb cmb{};
  if (comb) {  // fused combine: down launch with f32 results, out = the (zeroed) token rows
    if (up || f16out || !comb->tokidx || !comb->pw || (sh && !comb->sg) || comb->y != out) return MOE_E_INVALID;
    cmb = *comb;
  }
  if (!lut_ok(routed, up, k, q4k, gs) || (sh && !lut_ok(sh, up, k, q4k))) return MOE_E_UNSUPPORTED;
  if (m < 32 || m % 32) return MOE_E_UNSUPPORTED;
  if (q4k && up && m % 64) return MOE_E_UNSUPPORTED;  // hid is written in whole 64-element blocks
  if (!moe_aligned(x, 16) || !moe_aligned(out, 4)) return MOE_E_INVALID;
  if (max_tiles == 0) return MOE_OK;
  int nblk_n = up ? (m + HALF - 1) / HALF : (m + WROWS - 1) / WROWS;
  // down launches with f16 results: a block walks npass neighbouring column blocks of its pair tile (whole column
  // blocks and whole scale windows only); the largest divisor of the column block count up to the wanted length
  // (measured at 163840 pairs, K = 768, 12 column blocks: 0.938 / 0.921 / 0.912 / 0.921 / 0.943 / 1.015 ms for walks of
  //  1 / 2 / 3 / 4 / 6 / 12; a launch with few tiles keeps its blocks short: the shared expert's 1536 blocks next to the
  //  router's launches took longer as 512 blocks of three passes)
  int npass = 1;
  if (!up && f16out && !q5k && !comb && NBUF == 3 && m % WROWS == 0 && k % 256 == 0)
    for (int c = 1; c <= MOE_GEMM_WALK && c <= nblk_n; c++)
      if (nblk_n % c == 0 && (int64_t)max_tiles * (nblk_n / c) >= 4096) npass = c;
  nblk_n /= npass;
  // per XCD: ceil(routed/8) + ceil(shared/8) <= max_tiles/8 + 2 tile slots
  const int per_xcd = (max_tiles + 7) / 8 + 1;
  const unsigned grid = (unsigned)(per_xcd * nblk_n * 8);
  LutDev R = to_dev(routed, nullptr, pexp_routed), S = to_dev(sh ? sh : routed, sh ? sh_cb_up : nullptr, sh ? pexp_sh : pexp_routed);
  const int split = sh ? 1 : 0;
#define GEMM_LAUNCH(UPK, F16, Q, G)                                                                              \
  do {                                                                                                           \
    static moe_dev_once attr_once;                                                                               \
    int dev_now;                                                                                                 \
    if (moe_dev_pending(attr_once, &dev_now)) {                                                                  \
      MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_q4cp<UPK, F16, Q, G>,                                  \
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM_BYTES));                 \
      moe_dev_done(attr_once, dev_now);                                                                          \
    }                                                                                                            \
    k_moe_gemm_q4cp<UPK, F16, Q, G><<<grid, NT, SMEM_BYTES, st>>>(R, S, n_experts, x, tokidx, tiles, ntiles, out, \
                                                                  m, k, nblk_n, split, hs, cmb, npass, moe_rotv{nullptr, nullptr}); \
  } while (0)
#define GEMM_LAUNCH_NAT(UPK, F16)                                                                                \
  do {                                                                                                           \
    static moe_dev_once attr_once;                                                                               \
    int dev_now;                                                                                                 \
    if (moe_dev_pending(attr_once, &dev_now)) {                                                                  \
      MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_q4cp<UPK, F16, false, 0, false, true>,                 \
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)(SMEM_BYTES + PT_BYTES)));    \
      moe_dev_done(attr_once, dev_now);                                                                          \
    }                                                                                                            \
    k_moe_gemm_q4cp<UPK, F16, false, 0, false, true><<<grid, NT, SMEM_BYTES + PT_BYTES, st>>>(                    \
        R, S, n_experts, x, tokidx, tiles, ntiles, out, m, k, nblk_n, split, hs, cmb, npass, moe_rotv{nullptr, nullptr}); \
  } while (0)
  if (nat) {
    if (up) GEMM_LAUNCH_NAT(true, true);
    else if (f16out) GEMM_LAUNCH_NAT(false, true);
    else GEMM_LAUNCH_NAT(false, false);
#if MOE_GEMM_NF == 2 && MOE_GEMM_WROWS == 256  // (other block shapes: timing experiments of the q4cp / Q4_K launches only)
  } else if (q5k) {
    static moe_dev_once attr5;
    int dev_now;
    if (moe_dev_pending(attr5, &dev_now)) {
      MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_q4cp<true, true, true, 0, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM_BYTES));
      moe_dev_done(attr5, dev_now);
    }
    k_moe_gemm_q4cp<true, true, true, 0, true><<<grid, NT, SMEM_BYTES, st>>>(R, S, n_experts, x, tokidx, tiles, ntiles, out,
                                                                             m, k, nblk_n, split, hs, cmb, npass, moe_rotv{nullptr, nullptr});
  } else if (gs == 2 && up) {
    static moe_dev_once attr_rot;
    int dev_now;
    if (moe_dev_pending(attr_rot, &dev_now)) {
      MOE_HIP(hipFuncSetAttribute((const void*)k_moe_gemm_q4cp<true, true, false, 2, false, false, true>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)SMEM_BYTES));
      moe_dev_done(attr_rot, dev_now);
    }
    k_moe_gemm_q4cp<true, true, false, 2, false, false, true><<<grid, NT, SMEM_BYTES, st>>>(
        R, S, n_experts, x, tokidx, tiles, ntiles, out, m, k, nblk_n, split, hs, cmb, npass, *rot);
  } else if (gs == 2) {
    GEMM_LAUNCH(false, true, false, 2);
#endif
  } else if (q4k) {
    if (up) GEMM_LAUNCH(true, true, true, 0);
    else if (f16out) GEMM_LAUNCH(false, true, true, 0);
    else GEMM_LAUNCH(false, false, true, 0);
  } else {
    if (up) GEMM_LAUNCH(true, true, false, 0);
    else if (f16out) GEMM_LAUNCH(false, true, false, 0);
    else GEMM_LAUNCH(false, false, false, 0);
  }
#undef GEMM_LAUNCH
#undef GEMM_LAUNCH_NAT
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

// hgn v2 i4r tensor [codes][scales], no header: the reference's lut_i4r_view (27_kernels_moe_lut.inc:823-834)
MOE_API int moe_lut_i4r_view(const uint8_t* data, uint64_t rows, uint64_t cols, int e_rows, int up_off, moe_lutw* out) {
  if (!data || !out || cols == 0 || cols % 128) return MOE_E_INVALID;
  out->cb = moe_i4r_codebook();
  if (!out->cb) return MOE_E_STATE;
  out->w = out->w_up = data;
  out->sc = out->sc_up = data + rows * cols / 2;
  out->sstride = (int)(cols / 128 * 2);
  out->e_rows = e_rows;
  out->up_off = up_off;
  return MOE_OK;
}

// gate | up unfused, f16 [slot][2 m] (the rotation back comes before SwiGLU): the reference's moe_lut_up_raw
// (27_kernels_moe_lut.inc:677-685).  x16 in the grouped GEMM's activation order, as for moe_lut_up.
MOE_API int moe_lut_up_raw(int type, const moe_lutw* p, const void* x16, const int* tokidx, const moe_tile* tiles,
                           const int* ntiles, int max_tiles, void* guv16, int m, int k, moe_stream_t st) {
  if (type != MOE_LUT_I4R) return MOE_E_UNSUPPORTED;
  if (!tokidx || !p) return MOE_E_INVALID;
  moe_lutw q = *p;
  q.e_rows = 2 * m;  // the fused tensor's rows of one expert, walked as plain rows
  return moe_launch_gemm_q4cp(false, &q, nullptr, 1 << 30, (const __half*)x16, tokidx, tiles, ntiles, max_tiles, guv16,
                              2 * m, k, true, false, moe_hscale{nullptr, 0.f, 0.f}, moe_s(st), nullptr, nullptr, 2);
}

MOE_API int moe_lut_up(int type, const moe_lutw* p, const void* x16, const int* tokidx,
                       const moe_tile* tiles, const int* ntiles, int max_tiles, void* hid16, int m, int k,
                       moe_stream_t st) {
  if (type != MOE_LUT_Q4CP) return MOE_E_UNSUPPORTED;
  if (!tokidx) return MOE_E_INVALID;
  return moe_launch_gemm_q4cp(true, p, nullptr, 1 << 30, (const __half*)x16, tokidx, tiles, ntiles, max_tiles,
                              hid16, m, k, true, false, moe_hscale{nullptr, 0.f, 0.f}, moe_s(st), nullptr, nullptr);
}

MOE_API int moe_lut_down(int type, const moe_lutw* p, const void* hid16, const moe_tile* tiles,
                         const int* ntiles, int max_tiles, void* pairs, int m, int k, int f16,
                         moe_stream_t st) {
  if (type == MOE_LUT_I4R) {  // (f16 pairs only, the reference's default for hgn v2: 40_model.inc:4619-4631)
    if (!f16) return MOE_E_UNSUPPORTED;
    return moe_launch_gemm_q4cp(false, p, nullptr, 1 << 30, (const __half*)hid16, nullptr, tiles, ntiles, max_tiles, pairs,
                                m, k, true, false, moe_hscale{nullptr, 0.f, 0.f}, moe_s(st), nullptr, nullptr, 2);
  }
  if (type != MOE_LUT_Q4CP) return MOE_E_UNSUPPORTED;
  return moe_launch_gemm_q4cp(false, p, nullptr, 1 << 30, (const __half*)hid16, nullptr, tiles, ntiles,
                              max_tiles, pairs, m, k, f16 != 0, false, moe_hscale{nullptr, 0.f, 0.f}, moe_s(st), nullptr, nullptr);
}

// moe_gg_up / moe_gg_down: raw GGUF blocks, expert e's rows start at row e * m of each tensor
MOE_API int moe_gg_up(int type, const uint8_t* gate, const uint8_t* up, const void* x16, const int* tokidx,
                      const moe_tile* tiles, const int* ntiles, int max_tiles, void* hid16, int m, int k,
                      moe_stream_t st) {
  if (type != MOE_GGML_Q4_K) return MOE_E_UNSUPPORTED;
  if (!tokidx) return MOE_E_INVALID;
  moe_lutw p{};
  p.w = gate;
  p.w_up = up;
  p.e_rows = m;
  return moe_launch_gemm_q4cp(true, &p, nullptr, 1 << 30, (const __half*)x16, tokidx, tiles, ntiles, max_tiles,
                              hid16, m, k, true, true, moe_hscale{nullptr, 0.f, 0.f}, moe_s(st), nullptr, nullptr);
}

MOE_API int moe_gg_down(int type, const uint8_t* down, const void* hid16, const moe_tile* tiles,
                        const int* ntiles, int max_tiles, void* pairs, int m, int k, int f16,
                        moe_stream_t st) {
  if (type != MOE_GGML_Q4_K) return MOE_E_UNSUPPORTED;
  moe_lutw p{};
  p.w = down;
  p.e_rows = m;
  return moe_launch_gemm_q4cp(false, &p, nullptr, 1 << 30, (const __half*)hid16, nullptr, tiles, ntiles,
                              max_tiles, pairs, m, k, f16 != 0, true, moe_hscale{nullptr, 0.f, 0.f}, moe_s(st), nullptr, nullptr);
}

// pairs per tile of the grouped GEMM launches (the cap of the tile lists that moe_forward builds)
int moe_gemm_tile_cap() { return BM; }
