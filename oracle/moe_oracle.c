/*
 * moe_oracle.c — CPU oracle for the routed-expert MoE layer.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the arithmetic of
 * the reference engine's CPU path so that the HIP kernels can be checked
 * against it.  Nothing in the product library links, loads or calls it; only
 * tests, the smoke check and the benchmark's cpu_baseline leg do.
 *
 * Reference files followed (paths relative to the reference tree):
 *   src/hgn.h:77-84      fp16 -> f32
 *   src/hgn.h:219-261    q4cp blob layout, q4cp_parse / q4cp_row
 *   src/gguf.h:328-336   scale_min_k4
 *   src/gguf.h:408-441   Q4_K / Q5_K dequant_row
 *   src/gguf.h:352-375   Q8_0 / Q5_1 dequant_row
 *   src/gguf.h:376-407   IQ4_NL / IQ4_XS dequant_row
 *   src/ref.cpp:55-56    sigmoid / silu
 *   src/ref.cpp:68-77    matvec: fp64 sequential accumulate, f32 result
 *   src/ref.cpp:563-637  Model::moe (router, top-k, experts, shared expert)
 *   src/gpu/parts/10_ple_io.inc:784-825  expert-sorted permutation + tiles
 *   src/gpu/parts/24_kernels_moe_lt.inc:126-161  HC write-back folded into the combine
 *   tools/moe_lut_test.cu:936-948, tools/v2repro/v2enc.py:87-101  hgn v2 i4r rows: (nibble - 8) * fp16 scale per 128
 *   src/gpu/parts/27_kernels_moe_lut.inc:44-65, 28_kernels_hgn_v2.inc:62-150, 40_model.inc:1638-1656
 *                        hgn v2 rotated experts: 128-block Hadamard on the activations around each projection
 *   src/gpu/parts/28_kernels_hgn_v2.inc:19-25,226-231,386-440,442-447,604-634, 30_host_util.inc:1019-1031,
 *   tools/v2repro/v2enc.py:48-84  hgn v2 dense tensors: ht (hashed-trellis) values, tile layout and un-rotation
 *                        to bf16; q6g64 rows to bf16
 *
 * Pinning status of every function is listed in oracle/README.md; each one is
 * checked in tests/ against the reference's own code built under oracle/_ref
 * and against closed forms / brute force.  One form is "parity unpinned": a shared
 * expert stored as planar q8g32 (hgn dtype 8).  Its dequantisation (mat_row) is pinned
 * against the reference's Checkpoint::dequant, but the reference's CPU matvec has no
 * branch for that dtype (src/ref.cpp:68-109 throws), so the layer form used here -- the
 * dequantised row in the generic fp64 dot product -- is confirmed by no run of the
 * reference.  Everything else is pinned; the hgn v2 functions (i4r rows, the 128-block
 * rotation, the rotated layer) by closed forms and by a float64 evaluation of the same
 * layer on the un-rotated weights, because the reference has no CPU code for that format.
 *
 * One deliberate addition: std::partial_sort in src/ref.cpp:587 leaves the
 * order of equal probabilities unspecified.  The oracle fixes it to "lowest
 * expert index first", the rule the reference's GPU router states
 * (src/gpu/parts/20_kernels_gemv.inc:1488-1494,1545).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ---- weight format tags (shared with the library header by value) ---- */
enum { ORC_F32 = 1, ORC_BF16 = 0, ORC_Q4CP = 5, ORC_Q4K = 12, ORC_Q5K = 13, ORC_Q5_1 = 7, ORC_Q8_0 = 8,
       ORC_IQ4_NL = 20, ORC_IQ4_XS = 23,
       ORC_Q8G64 = 107 /* hgn dtype 7; the tag is moved off ggml's Q5_1 = 7 */,
       ORC_Q8G32 = 108 /* hgn dtype 8 (moved off ggml's Q8_0 = 8) */,
       ORC_I4R = 123 /* hgn v2 dtype 23 (moved off ggml's IQ4_XS = 23) */ };

/* src/hgn.h:77-84 and src/gguf.h:318-325 (same function twice in the reference) */
ORC_API float orc_fp16_to_f32(uint16_t h) {
  uint32_t s = (h >> 15) & 1u, e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
  float v;
  if (e == 0) v = (float)m * 0x1p-24f;
  else if (e == 31) v = m ? NAN : INFINITY;
  else v = ldexpf((float)(1024 + m), (int)e - 25);
  return s ? -v : v;
}

static inline float bf16_to_f32(uint16_t b) { /* src/hgn.h:86-91 */
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* ---- q4cp: [64 B codebook][rows*cols/2 codes][rows x scale_stride] ---- */
ORC_API uint64_t orc_q4cp_scale_stride(uint64_t cols) { /* src/hgn.h:231 */
  return ((cols / 32 * 2) + 15) & ~15ULL;
}
ORC_API uint64_t orc_q4cp_blob_bytes(uint64_t rows, uint64_t cols) { /* src/hgn.h:232 */
  return 64 + rows * cols / 2 + rows * orc_q4cp_scale_stride(cols);
}

/* src/hgn.h:249-261: one row -> out[cols] */
ORC_API void orc_q4cp_row(const uint8_t* blob, uint64_t rows, uint64_t cols, uint64_t row,
                          float* out) {
  const float* cb = (const float*)blob;
  const uint8_t* codes = blob + 64 + row * (cols / 2);
  const uint64_t ss = orc_q4cp_scale_stride(cols);
  const uint8_t* srec = blob + 64 + rows * cols / 2 + row * ss;
  for (uint64_t g = 0; g < cols / 32; g++) {
    uint16_t sh;
    memcpy(&sh, srec + 2 * g, 2);
    const float s = orc_fp16_to_f32(sh);
    for (uint64_t j = 0; j < 32; j++) {
      const uint64_t i = g * 32 + j;
      const uint8_t byte = codes[i / 2];
      const uint8_t nib = (j % 2 == 0) ? (byte & 0xf) : (byte >> 4);
      out[i] = cb[nib] * s;
    }
  }
}

ORC_API void orc_q4cp_rows(const uint8_t* blob, uint64_t rows, uint64_t cols, uint64_t row0,
                           uint64_t nrows, float* out) {
  for (uint64_t r = 0; r < nrows; r++) orc_q4cp_row(blob, rows, cols, row0 + r, out + r * cols);
}

/* ---- GGUF Q4_K: 144-byte super-blocks of 256 elements ---- */
ORC_API void orc_scale_min_k4(int j, const uint8_t* q, uint8_t* d, uint8_t* m) { /* gguf.h:328-336 */
  if (j < 4) {
    *d = q[j] & 63;
    *m = q[j + 4] & 63;
  } else {
    *d = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
    *m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
  }
}

/* src/gguf.h:408-441, Q4_K branch.  The products d*sc, dmin*m and (d*sc)*q are
 * exact in f32 (11-bit fp16 significand times a 6-bit and a 4-bit integer), so
 * the value is one correctly rounded f32 subtraction whatever the contraction
 * setting of the compiler. */
ORC_API void orc_q4k_row(const uint8_t* src, float* y, uint64_t k) {
  for (uint64_t b = 0; b < k / 256; b++, src += 144) {
    uint16_t dh, mh;
    memcpy(&dh, src, 2);
    memcpy(&mh, src + 2, 2);
    const float d = orc_fp16_to_f32(dh), dmin = orc_fp16_to_f32(mh);
    const uint8_t* sc = src + 4;
    const uint8_t* ql = src + 16;
    float* yy = y + b * 256;
    int is = 0;
    for (int j = 0; j < 256; j += 64) {
      uint8_t s0, m0, s1, m1;
      orc_scale_min_k4(is + 0, sc, &s0, &m0);
      orc_scale_min_k4(is + 1, sc, &s1, &m1);
      const float d1 = d * s0, dm1 = dmin * m0, d2 = d * s1, dm2 = dmin * m1;
      for (int l = 0; l < 32; l++) *yy++ = d1 * (float)(ql[l] & 0xF) - dm1;
      for (int l = 0; l < 32; l++) *yy++ = d2 * (float)(ql[l] >> 4) - dm2;
      ql += 32;
      is += 2;
    }
  }
}
ORC_API uint64_t orc_q4k_row_bytes(uint64_t k) { return k / 256 * 144; } /* gguf.h:79-84 */

/* src/gguf.h:408-441, Q5_K branch: 176-byte super-blocks {d, dmin, scales[12], qh[32], ql[128]}; bit 2j of
 * qh[l] is the fifth bit of the low-nibble element l of pair j, bit 2j+1 that of the high-nibble element.
 * (d*sc)*q with q <= 31 is still exact in f32 (11 + 6 + 5 bits): one rounded subtraction. */
static void orc_q5k_row(const uint8_t* src, float* y, uint64_t k) {
  for (uint64_t b = 0; b < k / 256; b++, src += 176) {
    uint16_t dh, mh;
    memcpy(&dh, src, 2);
    memcpy(&mh, src + 2, 2);
    const float d = orc_fp16_to_f32(dh), dmin = orc_fp16_to_f32(mh);
    const uint8_t* sc = src + 4;
    const uint8_t* qh = src + 16;
    const uint8_t* ql = src + 48;
    float* yy = y + b * 256;
    for (int j = 0; j < 4; j++) {
      uint8_t s0, m0, s1, m1;
      orc_scale_min_k4(2 * j, sc, &s0, &m0);
      orc_scale_min_k4(2 * j + 1, sc, &s1, &m1);
      const float d1 = d * s0, dm1 = dmin * m0, d2 = d * s1, dm2 = dmin * m1;
      for (int l = 0; l < 32; l++) *yy++ = d1 * (float)((ql[l] & 0xF) + (((qh[l] >> (2 * j)) & 1) << 4)) - dm1;
      for (int l = 0; l < 32; l++) *yy++ = d2 * (float)((ql[l] >> 4) + (((qh[l] >> (2 * j + 1)) & 1) << 4)) - dm2;
      ql += 32;
    }
  }
}
/* src/gguf.h:352-359: 34-byte blocks {d fp16, 32 x int8}; d*q is exact (11 + 8 bits) */
static void orc_q8_0_row(const uint8_t* src, float* y, uint64_t k) {
  for (uint64_t b = 0; b < k / 32; b++, src += 34) {
    uint16_t dh;
    memcpy(&dh, src, 2);
    const float d = orc_fp16_to_f32(dh);
    for (int j = 0; j < 32; j++) y[b * 32 + j] = d * (float)(int8_t)src[2 + j];
  }
}
/* src/gguf.h:360-375: 24-byte blocks {d, m fp16, qh u32, qs[16]}; element j = low nibble of qs[j] + bit j of
 * qh, element j + 16 = high nibble + bit j + 16; x*d is exact (5 + 11 bits), so x*d + m is one rounded add
 * with or without contraction. */
static void orc_q5_1_row(const uint8_t* src, float* y, uint64_t k) {
  for (uint64_t b = 0; b < k / 32; b++, src += 24) {
    uint16_t dh, mh;
    uint32_t qh;
    memcpy(&dh, src, 2);
    memcpy(&mh, src + 2, 2);
    memcpy(&qh, src + 4, 4);
    const float d = orc_fp16_to_f32(dh), mn = orc_fp16_to_f32(mh);
    const uint8_t* qs = src + 8;
    for (int j = 0; j < 16; j++) {
      const int x0 = (qs[j] & 0xF) | (((qh >> j) & 1) << 4);
      const int x1 = (qs[j] >> 4) | (((qh >> (j + 16)) & 1) << 4);
      y[b * 32 + j] = (float)x0 * d + mn;
      y[b * 32 + j + 16] = (float)x1 * d + mn;
    }
  }
}
/* src/gguf.h:376-407: the non-linear 4-bit codebook of IQ4_NL / IQ4_XS */
static const int8_t orc_iq4_kv[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
/* IQ4_NL: 18-byte blocks {d fp16, qs[16]}; element j = kv[low nibble of qs[j]], element j + 16 = kv[high] */
static void orc_iq4_nl_row(const uint8_t* src, float* y, uint64_t k) {
  for (uint64_t b = 0; b < k / 32; b++, src += 18) {
    uint16_t dh;
    memcpy(&dh, src, 2);
    const float d = orc_fp16_to_f32(dh);
    for (int j = 0; j < 16; j++) {
      y[b * 32 + j] = d * orc_iq4_kv[src[2 + j] & 0xF];
      y[b * 32 + j + 16] = d * orc_iq4_kv[src[2 + j] >> 4];
    }
  }
}
/* IQ4_XS: 136-byte super-blocks {d fp16, scales_h u16, scales_l[4], qs[128]}: eight 32-element sub-blocks with
 * 6-bit scales ls (low 4 bits in scales_l, high 2 in scales_h), dl = d*(ls - 32), elements as IQ4_NL.
 * d*(ls-32) and dl*kv are exact in f32 (11 + 6 + 7 bits). */
static void orc_iq4_xs_row(const uint8_t* src, float* y, uint64_t k) {
  for (uint64_t b = 0; b < k / 256; b++, src += 136) {
    uint16_t dh, sh;
    memcpy(&dh, src, 2);
    memcpy(&sh, src + 2, 2);
    const float d = orc_fp16_to_f32(dh);
    const uint8_t* sl = src + 4;
    const uint8_t* qs = src + 8;
    for (int ib = 0; ib < 8; ib++, qs += 16) {
      const int ls = ((sl[ib / 2] >> (4 * (ib % 2))) & 0xF) | (((sh >> (2 * ib)) & 3) << 4);
      const float dl = d * (float)(ls - 32);
      float* yy = y + b * 256 + ib * 32;
      for (int j = 0; j < 16; j++) {
        yy[j] = dl * orc_iq4_kv[qs[j] & 0xF];
        yy[j + 16] = dl * orc_iq4_kv[qs[j] >> 4];
      }
    }
  }
}
/* src/gguf.h:42-84: bytes of one row of k elements */
ORC_API uint64_t orc_gg_row_bytes(int type, uint64_t k) {
  switch (type) {
    case ORC_Q4K: return k / 256 * 144;
    case ORC_Q5K: return k / 256 * 176;
    case ORC_Q8_0: return k / 32 * 34;
    case ORC_Q5_1: return k / 32 * 24;
    case ORC_IQ4_NL: return k / 32 * 18;
    case ORC_IQ4_XS: return k / 256 * 136;
    default: return 0;
  }
}
ORC_API int orc_gg_row(int type, const uint8_t* src, float* y, uint64_t k) {
  switch (type) {
    case ORC_Q4K: orc_q4k_row(src, y, k); return 0;
    case ORC_Q5K: orc_q5k_row(src, y, k); return 0;
    case ORC_Q8_0: orc_q8_0_row(src, y, k); return 0;
    case ORC_Q5_1: orc_q5_1_row(src, y, k); return 0;
    case ORC_IQ4_NL: orc_iq4_nl_row(src, y, k); return 0;
    case ORC_IQ4_XS: orc_iq4_xs_row(src, y, k); return 0;
    default: return -1;
  }
}

/* ---- generic "row r of a weight matrix" in any supported storage ---- */
typedef struct {
  int dtype;            /* ORC_F32 / ORC_BF16 / ORC_Q4CP / ORC_Q4K / ORC_Q5K / ORC_Q8_0 / ORC_Q5_1 */
  const uint8_t* data;  /* f32/bf16: row-major; q4cp: whole blob; q4k: row-major raw blocks */
  uint64_t rows, cols;  /* logical matrix (q4cp: rows of the whole blob) */
} orc_mat;

static void mat_row(const orc_mat* W, uint64_t r, float* out) {
  switch (W->dtype) {
    case ORC_F32: memcpy(out, W->data + r * W->cols * 4, W->cols * 4); break;
    case ORC_BF16: {
      const uint16_t* p = (const uint16_t*)W->data + r * W->cols;
      for (uint64_t c = 0; c < W->cols; c++) out[c] = bf16_to_f32(p[c]);
      break;
    }
    case ORC_Q4CP: orc_q4cp_row(W->data, W->rows, W->cols, r, out); break;
    case ORC_Q4K: orc_q4k_row(W->data + r * orc_q4k_row_bytes(W->cols), out, W->cols); break;
    case ORC_Q5K: case ORC_Q8_0: case ORC_Q5_1: case ORC_IQ4_NL: case ORC_IQ4_XS:
      orc_gg_row(W->dtype, W->data + r * orc_gg_row_bytes(W->dtype, W->cols), out, W->cols);
      break;
    case ORC_Q8G64: { /* src/hgn.h:189-202: per row [cols uint8][cols/64 x (fp16 scale, fp16 min)], w = code * s + m */
      const uint8_t* rp = W->data + r * (W->cols + W->cols / 64 * 4);
      const uint16_t* sm = (const uint16_t*)(rp + W->cols);
      for (uint64_t g = 0; g < W->cols / 64; g++) {
        const float s = orc_fp16_to_f32(sm[g * 2]), m = orc_fp16_to_f32(sm[g * 2 + 1]);
        for (uint64_t j = 0; j < 64; j++) out[g * 64 + j] = rp[g * 64 + j] * s + m;
      }
      break;
    }
    case ORC_Q8G32: { /* src/hgn.h:176-183: planar [rows*cols int8][rows*cols/32 fp16 scales], w = q[i] * s[i / 32] */
      const int8_t* q = (const int8_t*)W->data;
      const uint16_t* sc = (const uint16_t*)(W->data + W->rows * W->cols);
      for (uint64_t c = 0; c < W->cols; c++) {
        const uint64_t i = r * W->cols + c;
        out[c] = q[i] * orc_fp16_to_f32(sc[i / 32]);
      }
      break;
    }
    case ORC_I4R: { /* tools/moe_lut_test.cu:936-948: [rows][cols/2] codes (byte b = element 2b | 2b+1 << 4), then
                       [rows][cols/128] fp16 scales, rows unpadded; w = (nibble - 8) * scale */
      const uint8_t* codes = W->data + r * (W->cols / 2);
      const uint16_t* sc = (const uint16_t*)(W->data + W->rows * (W->cols / 2) + r * (W->cols / 128 * 2));
      for (uint64_t c = 0; c < W->cols; c++) {
        const uint8_t b = codes[c >> 1];
        const int nib = (c & 1) ? b >> 4 : b & 15;
        out[c] = (float)(nib - 8) * orc_fp16_to_f32(sc[c >> 7]);
      }
      break;
    }
    default: memset(out, 0, W->cols * 4);
  }
}

/* ---- hgn v2 rotation (src/gpu/parts/27_kernels_moe_lut.inc:44-65, 28_kernels_hgn_v2.inc:62-98) ----
 * y[i] = post[i] * H(pre . x)[i] / sqrt(128) per block of 128, H the Sylvester Hadamard matrix in natural order;
 * the butterflies run over strides 1, 2, ..., 64 with (lo + hi, lo - hi) in f32, the order of the reference's fwht128.
 * pre / post may be NULL (= 1).  In place is fine. */
static const float kRs128 = 0.0883883476483184405f;
static void fwht128(float* v) {
  for (int h = 1; h < 128; h <<= 1)
    for (int i = 0; i < 128; i += 2 * h)
      for (int j = i; j < i + h; j++) {
        const float a = v[j], b = v[j + h];
        v[j] = a + b;
        v[j + h] = a - b;
      }
}
ORC_API void orc_v2_rot(const float* x, float* y, const float* pre, const float* post, int n) {
  float v[128];
  for (int b = 0; b < n / 128; b++) {
    for (int i = 0; i < 128; i++) v[i] = x[b * 128 + i] * (pre ? pre[b * 128 + i] : 1.f);
    fwht128(v);
    for (int i = 0; i < 128; i++) y[b * 128 + i] = v[i] * kRs128 * (post ? post[b * 128 + i] : 1.f);
  }
}
static inline uint16_t f2bf_ref(float f);
/* ---- hgn v2 dense tensors: "ht" (dtype 16) and q6g64 (dtype 24) -> the bf16 matrix the reference's prefill GEMM
 * reads (v2_deq_bf16, src/gpu/parts/30_host_util.inc:1019-1031) ----
 *
 * ht value of a 16-bit trellis window (28_kernels_hgn_v2.inc:19-25; tools/v2repro/v2enc.py:48-61): the byte sum s of
 * w16 * 0x83dcd12d (mod 2^32), then f16(fma(1024 + s, 1.732421875 / 256, -10.3828125)) with the fma in f32. */
static inline uint16_t f32_to_fp16_rne(float f) { /* round to nearest even; finite |f| < 65520 */
  uint32_t u;
  memcpy(&u, &f, 4);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t a = u & 0x7fffffffu;
  if (a < 0x38800000u) { /* below the smallest normal f16: a subnormal, in units of 2^-24 */
    float m;
    memcpy(&m, &a, 4);
    return sign | (uint16_t)lrintf(m * 16777216.f); /* lrintf: nearest even in the default rounding mode */
  }
  const uint32_t r = a + 0xfffu + ((a >> 13) & 1u); /* drop 13 mantissa bits */
  return sign | (uint16_t)((r - 0x38000000u) >> 13);
}
ORC_API float orc_ht_value(uint32_t w16) {
  const uint32_t t = (w16 & 0xffffu) * 0x83dcd12du;
  const uint32_t s = (t & 0xff) + ((t >> 8) & 0xff) + ((t >> 16) & 0xff) + (t >> 24);
  const float v = fmaf((float)(1024u + s), 1.732421875f / 256.f, -10.3828125f);
  return orc_fp16_to_f32(f32_to_fp16_rne(v));
}
/* The code stream of an ht tensor [O][K] -> its values G[O][K] in the rotated domain.  Layout
 * (28_kernels_hgn_v2.inc:226-231,386-412; v2enc.py:67-84): tiles of 128 x 128, tile (ty, tx) = 8 granules of 1 KiB at
 * ((ty * K/128 + tx) * 8 + g) * 1024; granule g = tile columns 16g .. 16g+15; its 128-byte block q = tile rows
 * 16q .. 16q+15; in a block, 32-bit word L (little endian) belongs to row L % 16 and column half L / 16 and carries 8
 * values: value e = the 16 bits of (word L-1 mod 32 : word L) that start 28 - 4e bits above the low end of word L. */
ORC_API void orc_ht_decode(const uint8_t* codes, uint64_t O, uint64_t K, float* G) {
  const uint64_t ntx = K / 128;
  for (uint64_t ty = 0; ty < O / 128; ty++)
    for (uint64_t tx = 0; tx < ntx; tx++)
      for (int g = 0; g < 8; g++)
        for (int q = 0; q < 8; q++) {
          const uint8_t* blk = codes + ((ty * ntx + tx) * 8 + g) * 1024 + q * 128;
          uint32_t w[32];
          memcpy(w, blk, 128);
          for (int L = 0; L < 32; L++) {
            const uint64_t V = ((uint64_t)w[(L + 31) & 31] << 32) | w[L];
            const uint64_t r = ty * 128 + q * 16 + (L & 15), c0 = tx * 128 + g * 16 + (L >> 4) * 8;
            for (int e = 0; e < 8; e++) G[r * K + c0 + e] = orc_ht_value((uint32_t)(V >> (28 - 4 * e)) & 0xffffu);
          }
        }
}
/* k_ht_deq_bf16 (28_kernels_hgn_v2.inc:386-440): per tile, the unnormalised Hadamard transform down the columns, then
 * along the rows, then bf16(v * (svh[R] / 128) * suh[C]) -- W = diag(svh) . H . G . H . diag(suh) / 128.
 * k_q6g64_deq_bf16 (28_kernels_hgn_v2.inc:442-447,604-634): row r at r * align16(13 C / 16): C/2 bytes of low
 * nibbles (even column = low nibble), C/4 bytes of the codes' two high bits (column k: byte k/4, bits 2(k%4)),
 * C/64 x (f16 scale, f16 bias); W = bf16(fma(code, scale, bias)).
 * suh [cols] / svh [rows]: the f16 planes as f32 (ht only).  Returns 0, or -1 for a dtype / shape outside the two. */
ORC_API int orc_v2_dense_bf16(int dtype, const uint8_t* data, const float* suh, const float* svh, uint64_t rows,
                              uint64_t cols, uint16_t* out) {
  if (dtype == 16) {
    if (rows % 128 || cols % 128 || !suh || !svh) return -1;
    float* G = (float*)malloc(rows * cols * 4);
    orc_ht_decode(data, rows, cols, G);
    float v[128];
    for (uint64_t ty = 0; ty < rows / 128; ty++)
      for (uint64_t tx = 0; tx < cols / 128; tx++) {
        float* t = G + ty * 128 * cols + tx * 128;
        for (int c = 0; c < 128; c++) {
          for (int r = 0; r < 128; r++) v[r] = t[(uint64_t)r * cols + c];
          fwht128(v);
          for (int r = 0; r < 128; r++) t[(uint64_t)r * cols + c] = v[r];
        }
        for (int r = 0; r < 128; r++) {
          fwht128(t + (uint64_t)r * cols);
          const uint64_t R = ty * 128 + r;
          const float sv = svh[R] * (1.f / 128.f);
          for (int c = 0; c < 128; c++) {
            const uint64_t C = tx * 128 + c;
            out[R * cols + C] = f2bf_ref(t[(uint64_t)r * cols + c] * sv * suh[C]);
          }
        }
      }
    free(G);
    return 0;
  }
  if (dtype == 24) {
    if (cols % 64) return -1;
    const uint64_t st = ((13 * cols / 16) + 15) & ~15ull;
    for (uint64_t r = 0; r < rows; r++) {
      const uint8_t* row = data + r * st;
      for (uint64_t c = 0; c < cols; c++) {
        const uint32_t lo = (row[c >> 1] >> (4 * (c & 1))) & 15u;
        const uint32_t hi = (row[cols / 2 + (c >> 2)] >> (2 * (c & 3))) & 3u;
        uint16_t sb[2];
        memcpy(sb, row + 3 * cols / 4 + (c >> 6) * 4, 4);
        out[r * cols + c] = f2bf_ref(fmaf((float)(lo | (hi << 4)), orc_fp16_to_f32(sb[0]), orc_fp16_to_f32(sb[1])));
      }
    }
    return 0;
  }
  return -1;
}

ORC_API void orc_mat_rows(const orc_mat* W, uint64_t row0, uint64_t nrows, float* out) {
  for (uint64_t r = 0; r < nrows; r++) mat_row(W, row0 + r, out + r * W->cols);
}

/* src/ref.cpp:75-77,85-87: acc (double) += (double)w * x, c ascending, then (float) */
static inline float dot_f64(const float* w, const float* x, uint64_t n) {
  double acc = 0;
  for (uint64_t c = 0; c < n; c++) acc += (double)w[c] * x[c];
  return (float)acc;
}

/* One output of the reference's matvec (src/ref.cpp:68-109) for row r of W, whose dequantised row is wr.  q8g64 does
 * not go through the dequantised row: per 64-group it sums code * x and x in fp64 and adds a2 * s + mn * csum
 * (ref.cpp:91-106). */
static inline float mat_dot(const orc_mat* W, uint64_t r, const float* wr, const float* x) {
  if (W->dtype != ORC_Q8G64) return dot_f64(wr, x, W->cols);
  const uint8_t* codes = W->data + r * (W->cols + W->cols / 64 * 4);
  const uint16_t* sm = (const uint16_t*)(codes + W->cols);
  double acc = 0;
  for (uint64_t g = 0; g < W->cols / 64; g++) {
    const float s = orc_fp16_to_f32(sm[g * 2]), mn = orc_fp16_to_f32(sm[g * 2 + 1]);
    double a2 = 0, csum = 0;
    for (int j = 0; j < 64; j++) {
      a2 += (double)codes[g * 64 + j] * x[g * 64 + j];
      csum += x[g * 64 + j];
    }
    acc += a2 * s + mn * csum;
  }
  return (float)acc;
}

static inline float sigmoidf_ref(float x) { return 1.f / (1.f + expf(-x)); } /* ref.cpp:55 */
static inline float siluf_ref(float x) { return x / (1.f + expf(-x)); }      /* ref.cpp:56 */

/* ---- router: src/ref.cpp:565-594 -------------------------------------- */
/* logits[E] (f32, already the (float) of the fp64 dot) -> probs, ids, weights.
 * ids are in selection order (descending probability, ties -> lowest index). */
ORC_API void orc_softmax_topk(const float* logits, int E, int k, float* probs, int* ids,
                              float* ws) {
  double mx = -1e300;
  for (int i = 0; i < E; i++) mx = fmax(mx, (double)logits[i]);
  double se = 0;
  for (int i = 0; i < E; i++) {
    probs[i] = (float)exp((double)logits[i] - mx);
    se += probs[i];
  }
  for (int i = 0; i < E; i++) probs[i] = (float)(probs[i] / se);
  /* k rounds of arg-max over what is left; strict '>' keeps the lowest index */
  uint8_t* taken = (uint8_t*)calloc((size_t)E, 1);
  for (int j = 0; j < k; j++) {
    int best = -1;
    for (int i = 0; i < E; i++)
      if (!taken[i] && (best < 0 || probs[i] > probs[best])) best = i;
    ids[j] = best;
    taken[best] = 1;
  }
  free(taken);
  double wsum = 0;
  for (int j = 0; j < k; j++) wsum += probs[ids[j]];
  for (int j = 0; j < k; j++) ws[j] = (float)(probs[ids[j]] / wsum);
}

/* router logits for T tokens: logits[t][e] = (float) sum_c (double)W[e][c]*x[t][c] */
ORC_API void orc_router_logits(const orc_mat* Wr, const float* x, int T, float* logits) {
  const int E = (int)Wr->rows;
  const uint64_t d = Wr->cols;
#pragma omp parallel
  {
    float* wr = (float*)malloc(d * 4);
#pragma omp for schedule(static)
    for (int e = 0; e < E; e++) {
      mat_row(Wr, (uint64_t)e, wr);
      for (int t = 0; t < T; t++) logits[(size_t)t * E + e] = dot_f64(wr, x + (size_t)t * d, d);
    }
    free(wr);
  }
}

/* ids/ws rows are id_stride wide (the reference pads to 16), first k valid. */
ORC_API void orc_router(const orc_mat* Wr, const float* bias, const float* x, int T, int k,
                        int id_stride, float* logits_out, int* ids, float* ws) {
  const int E = (int)Wr->rows;
  float* logits = logits_out ? logits_out : (float*)malloc((size_t)T * E * 4);
  orc_router_logits(Wr, x, T, logits);
  if (bias) /* synthetic skew only: added in f32 to the f32 logit */
    for (int t = 0; t < T; t++)
      for (int e = 0; e < E; e++) logits[(size_t)t * E + e] += bias[e];
#pragma omp parallel
  {
    float* probs = (float*)malloc((size_t)E * 4);
#pragma omp for schedule(static)
    for (int t = 0; t < T; t++)
      orc_softmax_topk(logits + (size_t)t * E, E, k, probs, ids + (size_t)t * id_stride,
                       ws + (size_t)t * id_stride);
    free(probs);
  }
  if (!logits_out) free(logits);
}

/* ---- expert-sorted permutation: 10_ple_io.inc:784-811 (stable sort by expert) ---- */
ORC_API void orc_route(const int* ids, const float* ws, int P, int k, int E, int id_stride,
                       int* tokidx, float* pw, int* eoff, int* pairids) {
  int* cnt = (int*)calloc((size_t)E + 1, sizeof(int));
  for (int p = 0; p < P * k; p++) cnt[ids[(p / k) * id_stride + p % k] + 1]++;
  eoff[0] = 0;
  for (int e = 0; e < E; e++) eoff[e + 1] = eoff[e] + cnt[e + 1];
  int* cur = (int*)malloc((size_t)E * sizeof(int));
  memcpy(cur, eoff, (size_t)E * sizeof(int));
  for (int p = 0; p < P * k; p++) { /* ascending original pair index = stable */
    const int t = p / k, s = p % k, e = ids[t * id_stride + s];
    const int q = cur[e]++;
    tokidx[q] = t;
    pw[q] = ws[t * id_stride + s];
    if (pairids) {
      int rank = 0;
      for (int j = 0; j < k; j++) rank += ids[t * id_stride + j] < e;
      pairids[t * k + rank] = q;
    }
  }
  free(cur);
  free(cnt);
}

/* 10_ple_io.inc:813-825: split every expert's run into <=cap slot tiles */
ORC_API int orc_tiles(const int* eoff, int E, int cap, int* tiles /* [n][3] */) {
  int n = 0;
  for (int e = 0; e < E; e++) {
    const int first = eoff[e], ne = eoff[e + 1] - first;
    for (int j = 0; j * cap < ne; j++) {
      tiles[3 * n + 0] = e;
      tiles[3 * n + 1] = first + j * cap;
      tiles[3 * n + 2] = ne - j * cap < cap ? ne - j * cap : cap;
      n++;
    }
  }
  return n;
}

/* ---- the layer: src/ref.cpp:596-636 ----------------------------------- */
typedef struct {
  int d, mid, E, k;
  orc_mat router;          /* [E][d] */
  const float* router_bias;/* optional [E] synthetic skew, may be NULL */
  /* routed experts: either fused gate_up [E*2*mid][d] (q4cp) or separate gate/up [E*mid][d] */
  orc_mat gate_up;         /* dtype<0 => use gate/up */
  orc_mat gate, up;
  orc_mat down;            /* [E*d][mid] */
  /* shared expert (dense, one expert's shape) */
  orc_mat sh_gate, sh_up, sh_down; /* [mid][d],[mid][d],[d][mid] */
  orc_mat sh_sg;           /* [1][d] */
  int has_shared;
  /* hgn v2 rotated routed experts (all four NULL otherwise): input / output sign-scale planes of the two expert
   * tensors, f32: su_gu [d], svh_gu [2*mid], suh_dn [mid], svh_dn [d] */
  const float *su_gu, *svh_gu, *suh_dn, *svh_dn;
} orc_layer;

static void expert_rows_gate_up(const orc_layer* L, int e, int r, float* out) {
  /* row r in [0, 2*mid): gate rows first, then up rows (ref.cpp:613-615) */
  if (L->gate_up.data) mat_row(&L->gate_up, (uint64_t)e * 2 * L->mid + r, out);
  else if (r < L->mid) mat_row(&L->gate, (uint64_t)e * L->mid + r, out);
  else mat_row(&L->up, (uint64_t)e * L->mid + (r - L->mid), out);
}

/*
 * y[T][d] for the tokens listed in tok_list (n_list of them; NULL => all T).
 * Per token the arithmetic is exactly Model::moe's; the loops are reordered
 * (expert-major, each weight row dequantised once and used for every token
 * routed to it) which changes no value: every dot product is an independent
 * fp64 chain, and each token's f32 accumulation still runs in rank order.
 * ids/ws are outputs ([T][id_stride]); hid_out (optional) is [T][k][mid].
 * hgn v2 layers (rotation planes set; 40_model.inc:1638-1656): the routed experts see rot_in(x, su_gu); their
 * gate|up outputs go through rot_out(svh_gu) before SwiGLU and the result through rot_in(suh_dn)
 * (k_i4r_mid, 28_kernels_hgn_v2.inc:105-150); the weighted sum over the experts through rot_out(svh_dn); the
 * shared expert reads the plain x.  hid_out then holds the rotated down-projection inputs.
 */
ORC_API void orc_moe_layer(const orc_layer* L, const float* x, int T, const int* tok_list,
                           int n_list, int id_stride, int* ids, float* ws, float* hid_out,
                           float* y) {
  const int d = L->d, mid = L->mid, E = L->E, k = L->k;
  orc_router(&L->router, L->router_bias, x, T, k, id_stride, NULL, ids, ws);
  const int n = tok_list ? n_list : T;
  const int v2 = L->su_gu != NULL;
  const float* xe = x; /* what the routed experts read */
  float* xrot = NULL;
  if (v2) {
    xrot = (float*)malloc((size_t)T * d * 4);
    for (int i = 0; i < n; i++) {
      const int t = tok_list ? tok_list[i] : i;
      orc_v2_rot(x + (size_t)t * d, xrot + (size_t)t * d, L->su_gu, NULL, d);
    }
    xe = xrot;
  }
  /* pair list grouped by expert (only tokens in the list) */
  int* cnt = (int*)calloc((size_t)E + 1, sizeof(int));
  for (int i = 0; i < n; i++) {
    const int t = tok_list ? tok_list[i] : i;
    for (int s = 0; s < k; s++) cnt[ids[t * id_stride + s] + 1]++;
  }
  for (int e = 0; e < E; e++) cnt[e + 1] += cnt[e];
  int* cur = (int*)malloc((size_t)E * sizeof(int));
  memcpy(cur, cnt, (size_t)E * sizeof(int));
  int* pair_i = (int*)malloc((size_t)n * k * sizeof(int)); /* list index */
  int* pair_s = (int*)malloc((size_t)n * k * sizeof(int)); /* rank */
  for (int i = 0; i < n; i++) {
    const int t = tok_list ? tok_list[i] : i;
    for (int s = 0; s < k; s++) {
      const int q = cur[ids[t * id_stride + s]]++;
      pair_i[q] = i;
      pair_s[q] = s;
    }
  }
  free(cur);
  /* per (list index, rank): guv[2*mid], hid[mid], dn[d] */
  float* guv = (float*)malloc((size_t)n * k * 2 * mid * 4);
  float* hid = (float*)malloc((size_t)n * k * mid * 4);
  float* dn = (float*)malloc((size_t)n * k * d * 4);
#pragma omp parallel
  {
    float* wr = (float*)malloc((size_t)(d > mid ? d : mid) * 4);
#pragma omp for schedule(dynamic, 16) collapse(2)
    for (int e = 0; e < E; e++)
      for (int r = 0; r < 2 * mid; r++) {
        if (cnt[e] == cnt[e + 1]) continue;
        expert_rows_gate_up(L, e, r, wr);
        for (int q = cnt[e]; q < cnt[e + 1]; q++) {
          const int i = pair_i[q], t = tok_list ? tok_list[i] : i;
          guv[((size_t)i * k + pair_s[q]) * 2 * mid + r] = dot_f64(wr, xe + (size_t)t * d, d);
        }
      }
#pragma omp for schedule(static)
    for (int i = 0; i < n * k; i++) {
      float* z = guv + (size_t)i * 2 * mid;
      if (v2) orc_v2_rot(z, z, NULL, L->svh_gu, 2 * mid);
      for (int r = 0; r < mid; r++) hid[(size_t)i * mid + r] = siluf_ref(z[r]) * z[mid + r];
      if (v2) orc_v2_rot(hid + (size_t)i * mid, hid + (size_t)i * mid, L->suh_dn, NULL, mid);
    }
#pragma omp for schedule(dynamic, 16) collapse(2)
    for (int e = 0; e < E; e++)
      for (int r = 0; r < d; r++) {
        if (cnt[e] == cnt[e + 1]) continue;
        mat_row(&L->down, (uint64_t)e * d + r, wr);
        for (int q = cnt[e]; q < cnt[e + 1]; q++) {
          const size_t ps = (size_t)pair_i[q] * k + pair_s[q];
          dn[ps * d + r] = dot_f64(wr, hid + ps * mid, mid);
        }
      }
    free(wr);
  }
  /* ref.cpp:621: acc[r] += w * (float)a2, ranks in order, f32 */
#pragma omp parallel for schedule(static)
  for (int i = 0; i < n; i++) {
    const int t = tok_list ? tok_list[i] : i;
    float* yt = y + (size_t)t * d;
    for (int r = 0; r < d; r++) {
      float acc = 0.f;
      for (int s = 0; s < k; s++) acc += ws[t * id_stride + s] * dn[((size_t)i * k + s) * d + r];
      yt[r] = acc;
    }
    if (v2) orc_v2_rot(yt, yt, NULL, L->svh_dn, d);
  }
  free(xrot);
  if (hid_out)
    for (int i = 0; i < n; i++) {
      const int t = tok_list ? tok_list[i] : i;
      memcpy(hid_out + (size_t)t * k * mid, hid + (size_t)i * k * mid, (size_t)k * mid * 4);
    }
  free(guv);
  free(hid);
  free(dn);
  free(pair_i);
  free(pair_s);
  free(cnt);
  if (!L->has_shared) return;
  /* shared expert, ref.cpp:623-636 */
  float* g1 = (float*)malloc((size_t)n * mid * 4);
  float* u1 = (float*)malloc((size_t)n * mid * 4);
  float* sg = (float*)malloc((size_t)n * 4);
#pragma omp parallel
  {
    float* wr = (float*)malloc((size_t)(d > mid ? d : mid) * 4);
#pragma omp for schedule(static)
    for (int r = 0; r < mid; r++) {
      mat_row(&L->sh_gate, (uint64_t)r, wr);
      for (int i = 0; i < n; i++) {
        const int t = tok_list ? tok_list[i] : i;
        g1[(size_t)i * mid + r] = mat_dot(&L->sh_gate, (uint64_t)r, wr, x + (size_t)t * d);
      }
      mat_row(&L->sh_up, (uint64_t)r, wr);
      for (int i = 0; i < n; i++) {
        const int t = tok_list ? tok_list[i] : i;
        u1[(size_t)i * mid + r] = mat_dot(&L->sh_up, (uint64_t)r, wr, x + (size_t)t * d);
      }
    }
#pragma omp single
    {
      mat_row(&L->sh_sg, 0, wr);
      for (int i = 0; i < n; i++) {
        const int t = tok_list ? tok_list[i] : i;
        sg[i] = sigmoidf_ref(mat_dot(&L->sh_sg, 0, wr, x + (size_t)t * d));
      }
    }
#pragma omp for schedule(static)
    for (int i = 0; i < n * mid; i++) g1[i] = siluf_ref(g1[i]) * u1[i];
#pragma omp for schedule(static)
    for (int r = 0; r < d; r++) {
      mat_row(&L->sh_down, (uint64_t)r, wr);
      for (int i = 0; i < n; i++) {
        const int t = tok_list ? tok_list[i] : i;
        const float ey = mat_dot(&L->sh_down, (uint64_t)r, wr, g1 + (size_t)i * mid);
        y[(size_t)t * d + r] = y[(size_t)t * d + r] + sg[i] * ey; /* ref.cpp:636 */
      }
    }
    free(wr);
  }
  free(g1);
  free(u1);
  free(sg);
}

ORC_API int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
ORC_API void orc_set_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* ---- HC write-back of the combine: src/gpu/parts/24_kernels_moe_lt.inc:126-161 ----
 * R[t][b][c] = f2bf(bf2f(R[t][b][c]) + inj_b * y[t][c]), inj_b = 2 / (1 + expf(-w4[t][b] * 0.25f)), b = 0..3;
 * f2bf = round to nearest even by the bit trick of src/gpu/parts/22_kernels_prefill.inc:4-9.  The reference
 * expression is compiled for the GPU with contraction on, i.e. as one fused multiply-add: fmaf here. */
static inline uint16_t f2bf_ref(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7FFF + ((u >> 16) & 1);
  return (uint16_t)(u >> 16);
}
ORC_API void orc_hc_writeback(const float* y, const float* w4, uint16_t* R, int P, int D) {
  for (int t = 0; t < P; t++)
    for (int b = 0; b < 4; b++) {
      const float inj = 2.f / (1.f + expf(-w4[(size_t)t * 4 + b] * 0.25f));
      uint16_t* Rt = R + ((size_t)t * 4 + b) * D;
      for (int c = 0; c < D; c++) Rt[c] = f2bf_ref(fmaf(inj, y[(size_t)t * D + c], bf16_to_f32(Rt[c])));
    }
}
