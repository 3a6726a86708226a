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
      a0 = fmaf((float)(v & 0xf), x0.x, a0);
      a1 = fmaf((float)((v >> 4) & 0xf), x0.y, a1);
      a0 = fmaf((float)((v >> 8) & 0xf), x0.z, a0);
      a1 = fmaf((float)((v >> 12) & 0xf), x0.w, a1);
      a0 = fmaf((float)((v >> 16) & 0xf), x1.x, a0);
      a1 = fmaf((float)((v >> 20) & 0xf), x1.y, a1);
      a0 = fmaf((float)((v >> 24) & 0xf), x1.z, a0);
      a1 = fmaf((float)(v >> 28), x1.w, a1);
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
__device__ __forceinline__ float sum32(const float4* xv) {
  float s0 = 0.f, s1 = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i += 2) {
    s0 += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);
    s1 += (xv[i + 1].x + xv[i + 1].y) + (xv[i + 1].z + xv[i + 1].w);
  }
  return s0 + s1;
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

// grid (mid / ROWS, slots per token incl. shared, P); block 256 = 4 waves.
// x of the token lies in LDS as float4 [j][g] (j-th quad of group g) so that lanes of
// consecutive groups read consecutive 16-byte words.
constexpr int GU_ROWS = 32;  // gate rows per block (and as many up rows)
template <bool AFFINE>
__device__ __forceinline__ void gu_rows(const uint8_t* gc, const uint8_t* gs, const uint8_t* uc,
                                        const uint8_t* us, uint64_t ss, int d, int r0, int nrows,
                                        CbInfo cg, CbInfo cu, const float* cbg, const float* cbu,
                                        const float4* xs, float* hid_out) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int G = d / 32;
  for (int rr = wv; rr < nrows; rr += 4) {
    const int r = r0 + rr;
    const uint8_t* grow = gc + (uint64_t)r * (d / 2);
    const uint8_t* urow = uc + (uint64_t)r * (d / 2);
    const __half* gsc = (const __half*)(gs + (uint64_t)r * ss);
    const __half* usc = (const __half*)(us + (uint64_t)r * ss);
    float ag = 0.f, au = 0.f;
    for (int g = lane; g < G; g += 64) {
      const uint4 pg = *(const uint4*)(grow + (size_t)g * 16);
      const uint4 pu = *(const uint4*)(urow + (size_t)g * 16);
      const float sg = __half2float(gsc[g]), su = __half2float(usc[g]);
      float4 xv[8];
#pragma unroll
      for (int j = 0; j < 8; j++) xv[j] = xs[j * G + g];
      float dg = dot32<AFFINE>(pg, xv, cbg), du = dot32<AFFINE>(pu, xv, cbu);
      if (AFFINE) {
        const float sx = sum32(xv);
        dg = fmaf(cg.a, dg, cg.b * sx);
        du = fmaf(cu.a, du, cu.b * sx);
      }
      ag = fmaf(dg, sg, ag);
      au = fmaf(du, su, au);
    }
    ag = wave_sum(ag);
    au = wave_sum(au);
    if (lane == 0) hid_out[r] = silu_f(ag) * au;
  }
}

__global__ void __launch_bounds__(256) k_q4cp_gemv_gu(GuArgs A, const float* __restrict__ x,
                                                      uint64_t x_stride, const int* __restrict__ ids,
                                                      int id_stride, int kpt, int d, int mid,
                                                      float* __restrict__ hid) {
  extern __shared__ float4 xs[];  // d/4 float4
  __shared__ float cbg[16], cbu[16];
  const int s = blockIdx.y, tok = blockIdx.z;
  const bool shared = s >= kpt;
  const int G = d / 32;
  const float* xt = x + (size_t)tok * x_stride;
  for (int i = threadIdx.x; i < d / 4; i += blockDim.x) xs[(i & 7) * G + (i >> 3)] = ((const float4*)xt)[i];
  const int r0 = blockIdx.x * GU_ROWS;
  const int nrows = min(GU_ROWS, mid - r0);
  float* ho = hid + ((size_t)tok * gridDim.y + s) * mid;
  const uint8_t *gc, *gs, *uc, *us;
  uint64_t ss;
  CbInfo cg, cu;
  if (!shared) {
    const int e = ids[(size_t)tok * id_stride + s];
    const uint64_t gr = (uint64_t)e * 2 * mid;
    gc = A.codes + gr * (d / 2);
    gs = A.scales + gr * A.scale_stride;
    uc = A.codes + (gr + mid) * (d / 2);
    us = A.scales + (gr + mid) * A.scale_stride;
    ss = A.scale_stride;
    cg = load_cb(A.cb, cbg);
    cu = cg;
    if (threadIdx.x < 16) cbu[threadIdx.x] = A.cb[threadIdx.x];
  } else {
    gc = A.sh_gcodes; gs = A.sh_gscales; uc = A.sh_ucodes; us = A.sh_uscales;
    ss = A.sh_scale_stride;
    cg = load_cb(A.sh_gcb, cbg);
    cu = load_cb(A.sh_ucb, cbu);
    if (threadIdx.x < 16) cbu[threadIdx.x] = A.sh_ucb[threadIdx.x];
  }
  __syncthreads();
  if (cg.affine && cu.affine) gu_rows<true>(gc, gs, uc, us, ss, d, r0, nrows, cg, cu, cbg, cbu, xs, ho);
  else gu_rows<false>(gc, gs, uc, us, ss, d, r0, nrows, cg, cu, cbg, cbu, xs, ho);
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

// grid (d / ROWS, P); block 256.  hid of all the token's slots in LDS as float4 [slot][j][g].
// Eight lanes per output row; every slot's partial stays in a register and the weighted sum runs
// in slot order (= descending router probability), then the shared expert.
constexpr int DN_ROWS = 32, DN_MAXSLOTS = 17;
template <bool AFFINE, int NS>
__device__ __forceinline__ void dn_rows(const DnArgs& A, const int* eid, const float* wgt, int nslots,
                                        bool has_shared, int d, int mid, int r0, int nrows, CbInfo cr,
                                        CbInfo cs, const float* cbr, const float* cbsh,
                                        const float4* hs, int tok, float* out) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, sub = lane >> 3, l8 = lane & 7;
  const int G = mid / 32;
  for (int rr = wv * 8 + sub; rr < nrows; rr += 32) {
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
          float dv = dot32<AFFINE>(pk, xv, cbl);
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

template <int NS>
__global__ void __launch_bounds__(256) k_q4cp_gemv_dn(DnArgs A, const float* __restrict__ hid,
                                                      const int* __restrict__ ids,
                                                      const float* __restrict__ ws, int id_stride,
                                                      int kpt, int d, int mid, float* __restrict__ out,
                                                      uint64_t out_stride) {
  extern __shared__ float4 hs[];  // nslots * mid/4 float4
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
  __syncthreads();
  const int r0 = blockIdx.x * DN_ROWS;
  const int nrows = min(DN_ROWS, d - r0);
  float* o = out + (size_t)tok * out_stride;
  if (cr.affine && cs.affine)
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
  dim3 grid((mid + GU_ROWS - 1) / GU_ROWS, nslots, P);
  k_q4cp_gemv_gu<<<grid, 256, (size_t)d * 4, st>>>(A, x, x_stride, ids, id_stride, kpt, d, mid, hid);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

int moe_launch_gemv_dn(const moe_wview* dn, const moe_wview* sh_down, const float* sh_logit,
                       const float* ey, const float* sg, const float* hid, const int* ids,
                       const float* ws, int id_stride, int kpt, int P, int d, float* out,
                       uint64_t out_stride, hipStream_t st) {
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
  return moe_launch_gemv_dn(dn, nullptr, nullptr, ey, sg, hid, ids, ws, id_stride, kpt, P, d, out, out_stride, moe_s(st));
}
