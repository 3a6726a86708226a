// Model-level entry points: a context owns the scratch, layers hold borrowed weight views, and
// moe_forward picks the path by batch size.
// (reference: GpuModel::moe / moe_b / moe_gguf / moe_q4w_run, src/gpu/parts/40_model.inc:1664-1861,4018-4157)
#include <cmath>
#include <new>
#include <vector>

#include "common.h"
#include "dense.h"
#include "internal.h"

struct MoeLayer {
  bool has_router = false, has_q4cp = false, has_gguf = false, has_shared = false;
  moe_wview router{};
  const float* router_bias = nullptr;
  float router_wmax = 0.f;  // the largest row norm of the router matrix (the bound of the small-batch selection, moe_rfix)
  float router_bmax = 0.f;  // the largest |bias| (how far a logit's dot product can lie above the logit itself)
  moe_wview gate_up{}, down{};
  moe_gg_experts gg{};
  moe_wview sh_gate{}, sh_up{}, sh_down{}, sh_sg{};
  int sh_gguf_type = 0;
  int sh_dense = 0;  // != 0: gate/up/down of the shared expert are dense rows of this kind (dense.h), in launches of their own
  // every q4cp codebook of the layer is affine (cb[n] = a*n + b): the integer-dot decode kernels apply
  bool experts_affine = false, shared_affine = false;
  // f16 range guard of the batch path: typical |hid| (and |pair|) per unit mean-square activation,
  // estimated from sampled weight rows when the weights are registered
  moe_cmag c_routed{0.f, 0.f}, c_shared{0.f, 0.f};  // f16 range guard constants (common.h), 0 = no guard
  // hgn v2 rotated experts (gate_up / down are MOE_DT_I4R views): the sign-scale planes of the two tensors, f32
  bool has_i4r = false;
  const float *v2_su = nullptr, *v2_svh_gu = nullptr, *v2_suh_dn = nullptr, *v2_svh_dn = nullptr;
};

// cb[n] == a*n + b for all 16 codes?  Reads the 64-byte codebook back from the device: weight
// registration is set-up work, not part of the enqueue-only forward path.
static int codebook_affine(const moe_wview* w, bool* out) {
  float cb[16];
  MOE_HIP(hipMemcpy(cb, w->data, sizeof cb, hipMemcpyDeviceToHost));
  bool ok = true;
  for (int n = 0; n < 16; n++) ok = ok && cb[n] == fmaf((float)n, cb[1] - cb[0], cb[0]);
  *out = ok;
  return MOE_OK;
}

struct moe_ctx;
static int pexp_register(moe_ctx* c, int layer, int slot0, const moe_wview* a, const moe_wview* b, int n_experts);
static int magnitude_constant(moe_ctx* c, int tgu, int tdn, const moe_wview* gate, uint64_t gate_stride,
                              const moe_wview* up, uint64_t up_first, const moe_wview* down, int n_experts,
                              moe_cmag* out);
static int magnitude_constant_i4r(moe_ctx* c, const moe_wview* gu, const moe_wview* dn, const float* su,
                                  const float* svh_gu, const float* suh_dn, int n_experts, moe_cmag* out);

struct moe_ctx {
  moe_config cfg;
  std::vector<MoeLayer> layers;
  // scratch (device), sized for cfg.max_tokens rows
  float* logits = nullptr;    // [T][E]
  int* ids = nullptr;         // [T][id_stride]
  float* ws = nullptr;        // [T][id_stride]
  float* sh_logit = nullptr;  // [T]
  float* rtol = nullptr;      // [min(T, small_max)]: per token, how far the small-batch router's logits can lie from the reference's
  unsigned* ticket = nullptr; // block counter of the fused small-batch router launch (rests at 0)
  double* kpart = nullptr;    // partial tiles and per-row-group tickets (resting at 0) of the column-split router launch
  unsigned* ktickets = nullptr;
  float* xms = nullptr;       // [T] mean square of each token's activations (batch path)
  float* sample = nullptr;    // 96 dequantised weight rows (registration-time magnitude estimate)
  float* hid32 = nullptr;     // [min(T,small_max)][k+1][mid] f32 (small-batch path)
  uint32_t *xplanes = nullptr, *hplanes = nullptr;  // integer digit planes of x / hid (decode kernels)
  float2 *xmeta = nullptr, *hmeta = nullptr;
#ifndef MOE_SMALL_MAX
#define MOE_SMALL_MAX 32
#endif
  int small_max = MOE_SMALL_MAX;         // batches up to this size take the in-place GEMV path
  bool int_decode = true;     // small batches: integer-dot kernels where they apply (else f32 kernels)
  // expert-sorted permutation (batch path; small batches that de-duplicate experts)
  moe_routing* routing = nullptr;
  __half* x16 = nullptr;      // [T][d]
  int* tokidx = nullptr;      // [(k+1)T] routed pairs then the shared expert's P pairs
  float* pw = nullptr;        // [(k+1)T]
  int* eoff = nullptr;        // [E+1]
  int* pairids = nullptr;     // [T*k]
  moe_tile* tiles = nullptr;  // [max_tiles]
  int* ntiles = nullptr;
  int max_tiles = 0;
  __half* hid16 = nullptr;    // [(k+1)T][mid]
  __half* pairs16 = nullptr;  // [(k+1)T][d]
  // scaled dequantisation of the grouped GEMM (internal.h): per layer [E gate_up | E down | shared gate/up | shared down]
  // powers of two, MOE_PEXP_NONE where the form does not apply; span_tmp: the scan's (hi, lo) pairs of one tensor
  int8_t* pexp = nullptr;
  int8_t* span_tmp = nullptr;
  float* pairs32 = nullptr;   // [(k+1)min(T,small_max)][d] unweighted pair rows of the unique-expert small-batch path
  bool fused_combine = false; // batch path: the down GEMM adds its weighted rows into y with f32 atomics (no pairs buffer, no reduce launch)
  int uq_min = 24;            // > 0: small batches of at least this many tokens read every distinct expert once
  int lut_max = 5;            // q4cp layers off the integer-dot kernels: batches up to this size take the register-resident f32 down kernel
  int gu_topk_max = 4;        // batches up to this size run the softmax / top-k inside the gate/up launch (else in the router's launches)
  bool uq_gguf = false;       // the same for GGUF layers (off: their per-token kernels measure faster unless most tokens share experts)
  // per-stage timing (the reference's KP("moe:route|up|down|reduce") tags, 07_kprof.inc)
  bool profile = false;
  int skip_stage = 0;      // MOE_OPT_TIMING_SKIP_STAGE: 1 + the stage whose launches are left out (0 = none; builds with MOE_TIMING_HOOKS only)
  int ran_complete = 0;    // the largest batch of at most small_max tokens that ran with every stage on this context
  hipEvent_t ev[MOE_PROF_STAGES + 1] = {};
  int ev_n = 0;            // events recorded by the last call
  int ev_stage[MOE_PROF_STAGES] = {};
  // batch path: the f32 -> f16 copy of x runs on a side stream next to the latency-bound top-k and
  // permutation launches (forked after the logits launch, joined in front of the gate/up GEMM)
  hipStream_t side = nullptr;
  hipEvent_t ev_fork = nullptr, ev_join = nullptr, ev_x16 = nullptr;
  // batch path, shared expert on the side stream: its tile list and the switch
  moe_tile* tiles_sh = nullptr;
  int* ntiles_sh = nullptr;
  const moe_hc* hc = nullptr;  // set for the duration of moe_forward_hc: the combine writes into the HC state
  const __half* x16_ext = nullptr;  // set for the duration of moe_forward_x16: the caller's f16 copy of x
  bool shared_aside = true;
  bool v2_fused_mid = true;   // hgn v2 batches: the slot-wise middle in the gate/up launch's epilogue
  bool pair_tables = true;    // table codebooks, 6..32 tokens: look-ups through pair tables
  int last_path = MOE_PATH_NONE;  // which path the last successful moe_forward* call took (moe_last_path)
  // batch router through candidate selection (exact ids at a fraction of the fp64 work); its scratch
  bool router_cand = true;
  void* rc_scratch = nullptr;
  // hgn v2 layers (allocated when the first one is registered): unfused gate | up sums and the rotated activations'
  // planes of the small-batch path, the routed sum and the shared expert's rows ahead of the last rotation; the
  // rotated f16 activations and the unfused f16 gate | up rows of the batch path
  float* v2_zraw = nullptr;      // [min(T,small_max)][k][2 mid]
  uint32_t* v2_xplanes = nullptr;
  float2* v2_xmeta = nullptr;
  float *v2_acc = nullptr, *v2_ey = nullptr;  // [min(T,small_max)][d] each
  __half* v2_x16 = nullptr;      // [T][d]
  __half* v2_z16 = nullptr;      // [kT][2 mid]
};

// Scaled dequantisation of the grouped GEMM: the powers of two of the experts of tensor a (and, for a launch that reads
// two tensors -- a shared expert's gate_proj and up_proj --, of a and b together) into slots slot0 .. of the layer's
// table.  a == nullptr: the form is switched off for these slots.  Set-up work (a scan of the scale planes, a read-back).
static int8_t* pexp_slot(moe_ctx* c, int layer, int slot0) {
  return c->pexp ? c->pexp + (size_t)layer * (2 * (size_t)c->cfg.experts + 2) + slot0 : nullptr;
}
static int pexp_register(moe_ctx* c, int layer, int slot0, const moe_wview* a, const moe_wview* b, int n_experts) {
  int8_t* dst = pexp_slot(c, layer, slot0);
  if (!dst) return MOE_OK;  // contexts for small batches only have no grouped GEMM
  std::vector<int8_t> out((size_t)n_experts, (int8_t)MOE_PEXP_NONE);
  if (a) {
    std::vector<int8_t> sa((size_t)2 * n_experts), sb;
    int rc = moe_q4cp_scale_span(a, n_experts, c->span_tmp, nullptr);
    if (rc) return rc;
    MOE_HIP(hipMemcpy(sa.data(), c->span_tmp, sa.size(), hipMemcpyDeviceToHost));
    if (b) {
      sb.resize(sa.size());
      if ((rc = moe_q4cp_scale_span(b, n_experts, c->span_tmp, nullptr))) return rc;
      MOE_HIP(hipMemcpy(sb.data(), c->span_tmp, sb.size(), hipMemcpyDeviceToHost));
    }
    for (int e = 0; e < n_experts; e++) out[e] = (int8_t)moe_pexp_from_span(&sa[2 * e], b ? &sb[2 * e] : nullptr);
  }
  MOE_HIP(hipMemcpy(dst, out.data(), out.size(), hipMemcpyHostToDevice));
  return MOE_OK;
}

static void prof_mark(moe_ctx* c, int stage_done, hipStream_t st) {
  // event i closes stage ev_stage[i-1]; event 0 opens the call
  if (!c->profile || c->ev_n > MOE_PROF_STAGES) return;
  if (hipEventRecord(c->ev[c->ev_n], st) != hipSuccess) return;
  if (c->ev_n > 0) c->ev_stage[c->ev_n - 1] = stage_done;
  c->ev_n++;
}

MOE_API const char* moe_version(void) { return "mi355moe 0.1 (gfx950)"; }

MOE_API const char* moe_status_string(int status) {
  switch (status) {
    case MOE_OK: return "ok";
    case MOE_E_UNSUPPORTED: return "unsupported shape or type";
    case MOE_E_INVALID: return "invalid argument";
    case MOE_E_STATE: return "context not ready or capacity exceeded";
    default: return status > 0 ? hipGetErrorString((hipError_t)status) : "unknown status";
  }
}

MOE_API int moe_destroy(moe_ctx* c) {
  if (!c) return MOE_OK;
  int rc = MOE_OK;
  if (c->routing) rc = moe_routing_destroy(c->routing);
  for (hipEvent_t e : c->ev)
    if (e) (void)hipEventDestroy(e);
  if (c->ev_fork) (void)hipEventDestroy(c->ev_fork);
  if (c->ev_join) (void)hipEventDestroy(c->ev_join);
  if (c->ev_x16) (void)hipEventDestroy(c->ev_x16);
  if (c->side) (void)hipStreamDestroy(c->side);
  void* bufs[] = {c->logits, c->ids, c->ws, c->sh_logit, c->ticket, c->kpart, c->ktickets, c->xms, c->sample, c->hid32, c->xplanes, c->hplanes, c->xmeta, c->hmeta, c->x16, c->tokidx, c->pw, c->eoff,
                  c->pairids, c->tiles, c->ntiles, c->tiles_sh, c->ntiles_sh, c->hid16, c->pairs16, c->pairs32, c->rc_scratch,
                  c->v2_zraw, c->v2_xplanes, c->v2_xmeta, c->v2_acc, c->v2_ey, c->v2_x16, c->v2_z16, c->pexp, c->span_tmp, c->rtol};
  for (void* b : bufs)
    if (b) {
      hipError_t e = hipFree(b);
      if (e != hipSuccess && rc == MOE_OK) rc = (int)e;
    }
  delete c;
  return rc;
}

MOE_API int moe_create(const moe_config* cfg, moe_ctx** out) {
  if (!cfg || !out) return MOE_E_INVALID;
  if (cfg->d < 32 || cfg->d % 32 || cfg->mid < 32 || cfg->mid % 32 || cfg->experts < 1 ||
      cfg->topk < 1 || cfg->topk > cfg->experts || cfg->layers < 1 || cfg->max_tokens < 1)
    return MOE_E_INVALID;
  if (cfg->experts > 1024 || cfg->topk > 15) return MOE_E_UNSUPPORTED;
  moe_ctx* c = new (std::nothrow) moe_ctx();
  if (!c) return (int)hipErrorOutOfMemory;
  c->cfg = *cfg;
  if (c->cfg.id_stride == 0) c->cfg.id_stride = 16;
  if (c->cfg.id_stride < cfg->topk) {
    delete c;
    return MOE_E_INVALID;
  }
  c->layers.resize(cfg->layers);
  const size_t T = (size_t)cfg->max_tokens, E = cfg->experts, S = c->cfg.id_stride;
  hipError_t e = hipMalloc(&c->logits, T * E * 4);
  // (index-like scratch starts at zero: expert ids, offsets and tile counts are addresses in the making, and nothing
  //  but a complete call fills them)
  if (e == hipSuccess) e = hipMalloc(&c->ids, T * S * 4);
  if (e == hipSuccess) e = hipMemset(c->ids, 0, T * S * 4);
  if (e == hipSuccess) e = hipMalloc(&c->ws, T * S * 4);
  if (e == hipSuccess) e = hipMemset(c->ws, 0, T * S * 4);
  if (e == hipSuccess) e = hipMalloc(&c->sh_logit, T * 4);
  if (e == hipSuccess) e = hipMalloc(&c->rtol, (T < (size_t)c->small_max ? T : (size_t)c->small_max) * 4);
  if (e == hipSuccess) e = hipMalloc(&c->ticket, 256);
  if (e == hipSuccess) e = hipMemset(c->ticket, 0, 256);
  if (e == hipSuccess) e = hipMalloc(&c->kpart, MOE_ROUTER_KPART_BYTES);
  if (e == hipSuccess) e = hipMalloc(&c->ktickets, MOE_ROUTER_KTICKET_BYTES);
  if (e == hipSuccess) e = hipMemset(c->ktickets, 0, MOE_ROUTER_KTICKET_BYTES);
  if (e == hipSuccess) e = hipMalloc(&c->xms, T * 4);
  if (e == hipSuccess) e = hipMalloc(&c->sample, (size_t)96 * (cfg->d > cfg->mid ? cfg->d : cfg->mid) * 4);
  const size_t Ts = T < (size_t)c->small_max ? T : (size_t)c->small_max;
  if (e == hipSuccess) e = hipMalloc(&c->hid32, Ts * (size_t)(cfg->topk + 1) * cfg->mid * 4);
  if (e == hipSuccess) e = hipMalloc(&c->xplanes, Ts * moe_qvec_plane_bytes(cfg->d));
  if (e == hipSuccess) e = hipMalloc(&c->xmeta, Ts * moe_qvec_meta_bytes(cfg->d));
  if (e == hipSuccess) e = hipMalloc(&c->hplanes, Ts * (size_t)(cfg->topk + 1) * moe_qvec_plane_bytes(cfg->mid));
  if (e == hipSuccess) e = hipMalloc(&c->hmeta, Ts * (size_t)(cfg->topk + 1) * moe_qvec_meta_bytes(cfg->mid));
  const size_t k1 = (size_t)cfg->topk + 1;
  if (e == hipSuccess) {
    // expert-sorted permutation: the batch path, and small batches that de-duplicate shared experts
    const size_t batch_tiles = (T * cfg->topk + 127) / 128 + E + (T + 127) / 128, uq_tiles = Ts * cfg->topk + (Ts + 3) / 4;
    c->max_tiles = (int)(batch_tiles > uq_tiles ? batch_tiles : uq_tiles);
    int rc = moe_routing_create((int)(T * cfg->topk), cfg->experts, &c->routing);
    if (rc != MOE_OK) {
      moe_destroy(c);
      return rc;
    }
    e = hipMalloc(&c->tokidx, k1 * T * 4);
    if (e == hipSuccess) e = hipMemset(c->tokidx, 0, k1 * T * 4);
    if (e == hipSuccess) e = hipMalloc(&c->pw, k1 * T * 4);
    if (e == hipSuccess) e = hipMalloc(&c->eoff, (E + 2) * 4);
    if (e == hipSuccess) e = hipMemset(c->eoff, 0, (E + 2) * 4);
    if (e == hipSuccess) e = hipMalloc(&c->pairids, T * cfg->topk * 4);
    if (e == hipSuccess) e = hipMemset(c->pairids, 0, T * cfg->topk * 4);
    if (e == hipSuccess) e = hipMalloc(&c->tiles, (size_t)c->max_tiles * sizeof(moe_tile));
    if (e == hipSuccess) e = hipMemset(c->tiles, 0, (size_t)c->max_tiles * sizeof(moe_tile));
    if (e == hipSuccess) e = hipMalloc(&c->ntiles, 8);
    if (e == hipSuccess) e = hipMemset(c->ntiles, 0, 8);
    if (e == hipSuccess) e = hipMalloc(&c->tiles_sh, ((T + 127) / 128 + 1) * sizeof(moe_tile));
    if (e == hipSuccess) e = hipMemset(c->tiles_sh, 0, ((T + 127) / 128 + 1) * sizeof(moe_tile));
    if (e == hipSuccess) e = hipMalloc(&c->ntiles_sh, 8);
    if (e == hipSuccess) e = hipMemset(c->ntiles_sh, 0, 8);
    if (e == hipSuccess) e = hipMalloc(&c->pairs32, k1 * Ts * (size_t)cfg->d * 4);
  }
  if (e == hipSuccess && T > (size_t)c->small_max) {
    const size_t d = cfg->d, mid = cfg->mid;
    e = hipMalloc(&c->rc_scratch, moe_router_cand_scratch_bytes(cfg->max_tokens, cfg->experts, cfg->d));
    if (e == hipSuccess) e = hipMalloc(&c->x16, T * d * 2);
    const size_t pe_bytes = (size_t)cfg->layers * (2 * E + 2);
    if (e == hipSuccess) e = hipMalloc(&c->pexp, pe_bytes);
    if (e == hipSuccess) e = hipMemset(c->pexp, 0x80, pe_bytes);  // MOE_PEXP_NONE
    if (e == hipSuccess) e = hipMalloc(&c->span_tmp, 2 * E);
    if (e == hipSuccess) e = hipMalloc(&c->hid16, k1 * T * mid * 2);
    if (e == hipSuccess) e = hipMalloc(&c->pairs16, k1 * T * d * 2);
  }
  for (int i = 0; i <= MOE_PROF_STAGES && e == hipSuccess; i++) e = hipEventCreate(&c->ev[i]);
  if (e == hipSuccess && c->x16) {
    e = hipStreamCreateWithFlags(&c->side, hipStreamNonBlocking);  // default priority
    if (e == hipSuccess) e = hipEventCreateWithFlags(&c->ev_fork, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&c->ev_join, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&c->ev_x16, hipEventDisableTiming);
  }
  if (e != hipSuccess) {
    moe_destroy(c);
    return (int)e;
  }
  *out = c;
  return MOE_OK;
}

static MoeLayer* layer_of(moe_ctx* c, int l) {
  if (!c || l < 0 || l >= (int)c->layers.size()) return nullptr;
  return &c->layers[l];
}

MOE_API int moe_set_router(moe_ctx* c, int layer, const moe_wview* w, const float* bias) {
  MoeLayer* L = layer_of(c, layer);
  if (!L || !w || !w->data) return MOE_E_INVALID;
  if (w->dtype != MOE_DT_F32 && w->dtype != MOE_DT_BF16) return MOE_E_UNSUPPORTED;
  if ((int)w->rows != c->cfg.experts || (int)w->cols != c->cfg.d) return MOE_E_INVALID;
  const int rn = moe_router_row_norm_max(w, c->sample, &L->router_wmax);
  if (rn) return rn;
  L->router_bmax = 0.f;
  if (bias) {
    std::vector<float> hb((size_t)w->rows);
    MOE_HIP(hipMemcpy(hb.data(), bias, hb.size() * 4, hipMemcpyDeviceToHost));
    for (float b : hb) L->router_bmax = fmaxf(L->router_bmax, fabsf(b));
  }
  L->router = *w;
  L->router_bias = bias;
  L->has_router = true;
  return MOE_OK;
}

MOE_API int moe_set_experts_q4cp(moe_ctx* c, int layer, const moe_wview* gu, const moe_wview* dn) {
  MoeLayer* L = layer_of(c, layer);
  if (!L || !gu || !dn || !gu->data || !dn->data) return MOE_E_INVALID;
  if (gu->dtype != MOE_DT_Q4CP || dn->dtype != MOE_DT_Q4CP) return MOE_E_UNSUPPORTED;
  const moe_config& g = c->cfg;
  if (gu->rows != (uint64_t)g.experts * 2 * g.mid || (int)gu->cols != g.d ||
      dn->rows != (uint64_t)g.experts * g.d || (int)dn->cols != g.mid)
    return MOE_E_INVALID;
  bool a1 = false, a2 = false;
  int rc;
  if ((rc = codebook_affine(gu, &a1)) || (rc = codebook_affine(dn, &a2))) return rc;
  L->experts_affine = a1 && a2;
  if ((rc = magnitude_constant(c, 0, 0, gu, (uint64_t)2 * g.mid, gu, (uint64_t)g.mid, dn, g.experts, &L->c_routed)))
    return rc;
  if ((rc = pexp_register(c, layer, 0, a1 ? gu : nullptr, nullptr, g.experts)) ||
      (rc = pexp_register(c, layer, g.experts, a2 ? dn : nullptr, nullptr, g.experts)))
    return rc;
  L->gate_up = *gu;
  L->down = *dn;
  L->has_q4cp = true;
  L->has_gguf = false;
  L->has_i4r = false;
  return MOE_OK;
}

// hgn v2 routed experts (reference: v2_init, src/gpu/parts/30_host_util.inc:818-870; moe_b_v2's shape checks,
// 40_model.inc:4574-4576)
MOE_API int moe_set_experts_i4r(moe_ctx* c, int layer, const moe_wview* gu, const moe_wview* dn, const float* su,
                                const float* svh_gu, const float* suh_dn, const float* svh_dn) {
  MoeLayer* L = layer_of(c, layer);
  if (!L || !gu || !dn || !gu->data || !dn->data || !su || !svh_gu || !suh_dn || !svh_dn) return MOE_E_INVALID;
  if (gu->dtype != MOE_DT_I4R || dn->dtype != MOE_DT_I4R) return MOE_E_UNSUPPORTED;
  const moe_config& g = c->cfg;
  if (gu->rows != (uint64_t)g.experts * 2 * g.mid || (int)gu->cols != g.d || dn->rows != (uint64_t)g.experts * g.d ||
      (int)dn->cols != g.mid)
    return MOE_E_INVALID;
  if (!moe_v2_shapes_ok(g.d, g.mid) || !moe_dec_supported(g.d, g.mid, g.topk + 1) ||
      !moe_dec_gu_topk_supported(g.experts, g.topk))
    return MOE_E_UNSUPPORTED;
  if (!moe_aligned(gu->data, 16) || !moe_aligned(dn->data, 16) || !moe_aligned(su, 16) || !moe_aligned(svh_gu, 16) ||
      !moe_aligned(suh_dn, 16) || !moe_aligned(svh_dn, 16))
    return MOE_E_INVALID;
  if (!moe_i4r_codebook()) return MOE_E_STATE;
  if (!c->v2_zraw) {  // set-up work: the scratch of these layers
    const size_t T = (size_t)g.max_tokens, Ts = T < (size_t)c->small_max ? T : (size_t)c->small_max;
    hipError_t e = hipMalloc(&c->v2_zraw, Ts * g.topk * 2 * g.mid * 4);
    if (e == hipSuccess) e = hipMalloc(&c->v2_xplanes, Ts * moe_qvec_plane_bytes(g.d));
    if (e == hipSuccess) e = hipMalloc(&c->v2_xmeta, Ts * moe_qvec_meta_bytes(g.d));
    if (e == hipSuccess) e = hipMalloc(&c->v2_acc, Ts * (size_t)g.d * 4);
    if (e == hipSuccess) e = hipMalloc(&c->v2_ey, Ts * (size_t)g.d * 4);
    if (e == hipSuccess && c->x16) {
      e = hipMalloc(&c->v2_x16, T * (size_t)g.d * 2);
      if (e == hipSuccess) e = hipMalloc(&c->v2_z16, T * g.topk * 2 * (size_t)g.mid * 2);
    }
    if (e != hipSuccess) {
      void* bufs[] = {c->v2_zraw, c->v2_xplanes, c->v2_xmeta, c->v2_acc, c->v2_ey, c->v2_x16, c->v2_z16};
      for (void* b : bufs)
        if (b) (void)hipFree(b);
      c->v2_zraw = nullptr; c->v2_xplanes = nullptr; c->v2_xmeta = nullptr; c->v2_acc = c->v2_ey = nullptr;
      c->v2_x16 = c->v2_z16 = nullptr;
      return (int)e;
    }
  }
  L->gate_up = *gu;
  L->down = *dn;
  L->v2_su = su; L->v2_svh_gu = svh_gu; L->v2_suh_dn = suh_dn; L->v2_svh_dn = svh_dn;
  L->c_routed = moe_cmag{0.f, 0.f};
  if (c->v2_x16) {  // (the batch path's f16 range guard; the small-batch kernels keep f32 between the projections)
    const int rm = magnitude_constant_i4r(c, gu, dn, su, svh_gu, suh_dn, g.experts, &L->c_routed);
    if (rm) return rm;
  }
  L->experts_affine = true;
  L->has_i4r = true;
  L->has_q4cp = false;
  L->has_gguf = false;
  return MOE_OK;
}

MOE_API int moe_get_config(const moe_ctx* c, moe_config* out) {
  if (!c || !out) return MOE_E_INVALID;
  *out = c->cfg;
  return MOE_OK;
}

MOE_API int moe_set_experts_gguf(moe_ctx* c, int layer, const moe_gg_experts* gg) {
  MoeLayer* L = layer_of(c, layer);
  if (!L || !gg || !gg->gate || !gg->up || !gg->down) return MOE_E_INVALID;
  if (!moe_gg_types_supported(gg->tgu, gg->tdn, c->cfg.d, c->cfg.mid)) return MOE_E_UNSUPPORTED;
  L->c_routed = moe_cmag{0.f, 0.f};
  {  // constant of the f16 range guard of the grouped GEMMs
    const moe_config& g = c->cfg;
    moe_wview gv{0, gg->gate, (uint64_t)g.experts * g.mid, (uint64_t)g.d, 0};
    moe_wview uv{0, gg->up, (uint64_t)g.experts * g.mid, (uint64_t)g.d, 0};
    moe_wview dv{0, gg->down, (uint64_t)g.experts * g.d, (uint64_t)g.mid, 0};
    int rc = magnitude_constant(c, gg->tgu, gg->tdn, &gv, (uint64_t)g.mid, &uv, 0, &dv, g.experts, &L->c_routed);
    if (rc) return rc;
  }
  L->gg = *gg;
  L->has_gguf = true;
  L->has_q4cp = false;
  L->has_i4r = false;
  return MOE_OK;
}

MOE_API int moe_set_shared(moe_ctx* c, int layer, const moe_wview* g, const moe_wview* u,
                           const moe_wview* dn, const moe_wview* sg, int sh_gguf_type) {
  MoeLayer* L = layer_of(c, layer);
  if (!L || !g || !u || !dn || !sg || !g->data || !u->data || !dn->data || !sg->data) return MOE_E_INVALID;
  const moe_config& cf = c->cfg;
  if ((int)g->rows != cf.mid || (int)g->cols != cf.d || (int)u->rows != cf.mid || (int)u->cols != cf.d ||
      (int)dn->rows != cf.d || (int)dn->cols != cf.mid || (int)sg->rows != 1 || (int)sg->cols != cf.d)
    return MOE_E_INVALID;
  if (sg->dtype != MOE_DT_F32 && sg->dtype != MOE_DT_BF16) return MOE_E_UNSUPPORTED;
  int dense = 0;
  if (sh_gguf_type == 0) {
    if (g->dtype != u->dtype || g->dtype != dn->dtype) return MOE_E_UNSUPPORTED;
    if (g->dtype != MOE_DT_Q4CP) {
      dense = moe_dense_type_of_hgn(g->dtype);
      if (!dense || !moe_dense_shared_supported(dense, cf.d, cf.mid)) return MOE_E_UNSUPPORTED;
    }
  } else if (!moe_gg_types_supported(sh_gguf_type, sh_gguf_type, cf.d, cf.mid)) {
    return MOE_E_UNSUPPORTED;
  }
  L->shared_affine = false;
  if (sh_gguf_type == 0 && !dense) {
    bool a1 = false, a2 = false, a3 = false;
    int rc;
    if ((rc = codebook_affine(g, &a1)) || (rc = codebook_affine(u, &a2)) || (rc = codebook_affine(dn, &a3))) return rc;
    L->shared_affine = a1 && a2 && a3;
    if ((rc = pexp_register(c, layer, 2 * cf.experts, a1 && a2 ? g : nullptr, u, 1)) ||
        (rc = pexp_register(c, layer, 2 * cf.experts + 1, a3 ? dn : nullptr, nullptr, 1)))
      return rc;
  } else {
    int rc;
    if ((rc = pexp_register(c, layer, 2 * cf.experts, nullptr, nullptr, 1)) ||
        (rc = pexp_register(c, layer, 2 * cf.experts + 1, nullptr, nullptr, 1)))
      return rc;
  }
  L->c_shared = moe_cmag{0.f, 0.f};
  {
    const int t = dense ? dense : sh_gguf_type;
    int rc = magnitude_constant(c, t, t, g, (uint64_t)cf.mid, u, 0, dn, 1, &L->c_shared);
    if (rc) return rc;
  }
  L->sh_dense = dense;
  L->sh_gate = *g;
  L->sh_up = *u;
  L->sh_down = *dn;
  L->sh_sg = *sg;
  L->sh_gguf_type = sh_gguf_type;
  L->has_shared = true;
  return MOE_OK;
}

// Typical |silu(g)*u| (times the growth through the down projection, if that is > 1) for
// activations of unit mean square: sigma_gate * sigma_up * max(1, sigma_down), sigma^2 = mean
// squared row norm over two sampled rows, maximum over up to 16 evenly spaced experts (out->hi); and the smaller of
// the two magnitudes, sigma_gate * sigma_up * min(1, sigma_down), minimum over those experts (out->lo).  Expert e's
// gate rows start at row e*gate_stride of `gate`, its up rows at e*gate_stride + up_first of `up`
// (the same fused tensor for hgn, a tensor of its own for GGUF), its down rows at e*down->rows/n.
// Set-up work: dequantises 6 rows per sampled expert on the device and reads them back.
// tgu / tdn: ggml block types of raw GGUF rows (gate and up; down), a dense code of dense.h, or 0 = q4cp views.
static int magnitude_constant(moe_ctx* c, int tgu, int tdn, const moe_wview* gate, uint64_t gate_stride,
                              const moe_wview* up, uint64_t up_first, const moe_wview* down, int n_experts,
                              moe_cmag* out) {
  const int ns = n_experts < 16 ? n_experts : 16;
  const uint64_t d = gate->cols, mid = down->cols, drows = down->rows / (uint64_t)n_experts;
  const uint64_t pitch = d > mid ? d : mid;
  auto deq = [&](const moe_wview* w, uint64_t row, float* dst) -> int {
    const int t = w == down ? tdn : tgu;
    if (moe_is_dense_type(t))
      return moe_dense_dequant_row(t, w->data, w->rows, (int)w->cols, row, dst, nullptr);
    if (t) return moe_gg_dequant_rows(t, w->data + row * moe_gg_row_bytes(t, w->cols), 1, w->cols, dst, nullptr);
    return moe_q4cp_dequant_rows(w->data, w->rows, w->cols, row, 1, dst, nullptr);
  };
  int rc;
  for (int i = 0; i < ns; i++) {
    const uint64_t e = (uint64_t)i * n_experts / ns;
    float* base = c->sample + (size_t)i * 6 * pitch;
    const uint64_t g0 = e * gate_stride, u0 = e * gate_stride + up_first, d0 = e * drows;
    if ((rc = deq(gate, g0, base)) || (rc = deq(gate, g0 + mid / 2, base + pitch)) ||
        (rc = deq(up, u0, base + 2 * pitch)) || (rc = deq(up, u0 + mid / 2, base + 3 * pitch)) ||
        (rc = deq(down, d0, base + 4 * pitch)) || (rc = deq(down, d0 + drows / 2, base + 5 * pitch)))
      return rc;
  }
  std::vector<float> h((size_t)ns * 6 * pitch);
  MOE_HIP(hipMemcpy(h.data(), c->sample, h.size() * 4, hipMemcpyDeviceToHost));
  double best = 0.0, least = 1e300;
  for (int i = 0; i < ns; i++) {
    double n2[6];
    for (int r = 0; r < 6; r++) {
      const float* v = h.data() + ((size_t)i * 6 + r) * pitch;
      const uint64_t n = r < 4 ? d : mid;
      double s = 0.0;
      for (uint64_t j = 0; j < n; j++) s += (double)v[j] * v[j];
      n2[r] = s;
    }
    const double sg = std::sqrt(0.5 * (n2[0] + n2[1])), su = std::sqrt(0.5 * (n2[2] + n2[3])),
                 sd = std::sqrt(0.5 * (n2[4] + n2[5]));
    const double cst = sg * su * (sd > 1.0 ? sd : 1.0);
    if (cst > best) best = cst;
    // the smaller of the two magnitudes (hid, pairs), smallest over the sampled experts: what can underflow
    const double low = sg * su * (sd < 1.0 ? sd : 1.0);
    if (low < least) least = low;
  }
  out->hi = (float)best;
  out->lo = least < 1e300 ? (float)least : 0.f;
  return MOE_OK;
}

// The same two magnitudes for hgn v2 rotated experts, as the batch path's f16 buffers see them: hid in the rotated
// domain of down_proj, ~ sigma_gate * sigma_up * rms(suh_dn) per unit mean square of x, and the pairs, that times the
// row norm of the stored down matrix.  The block Hadamard rotations are orthogonal, so the mean squared row norm of
// W = diag(svh) H G H diag(suh) / 128 is that of the stored G times the mean squares of the two vectors (to the
// accuracy a guard with factor-of-many margins needs).  Set-up work like magnitude_constant.
static int magnitude_constant_i4r(moe_ctx* c, const moe_wview* gu, const moe_wview* dn, const float* su,
                                  const float* svh_gu, const float* suh_dn, int n_experts, moe_cmag* out) {
  const int ns = n_experts < 16 ? n_experts : 16;
  const uint64_t d = gu->cols, mid = dn->cols;
  const uint64_t pitch = d > mid ? d : mid;
  int rc;
  for (int i = 0; i < ns; i++) {
    const uint64_t e = (uint64_t)i * n_experts / ns;
    float* base = c->sample + (size_t)i * 6 * pitch;
    const uint64_t g0 = e * 2 * mid, u0 = g0 + mid, d0 = e * d;
    const uint64_t rows[6] = {g0, g0 + mid / 2, u0, u0 + mid / 2, d0, d0 + d / 2};
    for (int r = 0; r < 6; r++) {
      const moe_wview* w = r < 4 ? gu : dn;
      if ((rc = moe_i4r_dequant_rows(w->data, w->rows, w->cols, rows[r], 1, base + (size_t)r * pitch, nullptr))) return rc;
    }
  }
  std::vector<float> h((size_t)ns * 6 * pitch), vsu(d), vgu(2 * mid), vdn(mid);
  MOE_HIP(hipMemcpy(h.data(), c->sample, h.size() * 4, hipMemcpyDeviceToHost));
  MOE_HIP(hipMemcpy(vsu.data(), su, d * 4, hipMemcpyDeviceToHost));
  MOE_HIP(hipMemcpy(vgu.data(), svh_gu, 2 * mid * 4, hipMemcpyDeviceToHost));
  MOE_HIP(hipMemcpy(vdn.data(), suh_dn, mid * 4, hipMemcpyDeviceToHost));
  auto rms = [](const float* v, uint64_t n) {
    double s = 0.0;
    for (uint64_t j = 0; j < n; j++) s += (double)v[j] * v[j];
    return std::sqrt(s / (double)n);
  };
  const double r_su = rms(vsu.data(), d), r_g = rms(vgu.data(), mid), r_u = rms(vgu.data() + mid, mid), r_dn = rms(vdn.data(), mid);
  double best = 0.0, least = 1e300;
  for (int i = 0; i < ns; i++) {
    double n2[6];
    for (int r = 0; r < 6; r++) {
      const float* v = h.data() + ((size_t)i * 6 + r) * pitch;
      const uint64_t n = r < 4 ? d : mid;
      double s = 0.0;
      for (uint64_t j = 0; j < n; j++) s += (double)v[j] * v[j];
      n2[r] = s;
    }
    const double sg = std::sqrt(0.5 * (n2[0] + n2[1])) * r_su * r_g, sup = std::sqrt(0.5 * (n2[2] + n2[3])) * r_su * r_u,
                 sd = std::sqrt(0.5 * (n2[4] + n2[5]));
    const double hid = sg * sup * r_dn;
    const double cst = hid * (sd > 1.0 ? sd : 1.0), low = hid * (sd < 1.0 ? sd : 1.0);
    if (cst > best) best = cst;
    if (low < least) least = low;
  }
  if (!(best < 1e30)) best = 0.0;  // (non-finite vectors: no guard rather than a factor of zero)
  out->hi = (float)best;
  out->lo = least < 1e300 && best > 0.0 ? (float)least : 0.f;
  return MOE_OK;
}

MOE_API int moe_clear_layer(moe_ctx* c, int layer) {
  MoeLayer* L = layer_of(c, layer);
  if (!L) return MOE_E_INVALID;
  *L = MoeLayer();
  return MOE_OK;
}

MOE_API int moe_set_option(moe_ctx* c, int option, int value) {
  if (!c) return MOE_E_INVALID;
  switch (option) {
    case MOE_OPT_INT_DECODE: c->int_decode = value != 0; return MOE_OK;
    case MOE_OPT_UNIQUE_MIN_TOKENS:
      if (value < 0) return MOE_E_INVALID;
      c->uq_min = value;
      return MOE_OK;
    case MOE_OPT_FUSED_COMBINE: c->fused_combine = value != 0; return MOE_OK;
    case MOE_OPT_SHARED_ASIDE: c->shared_aside = value != 0; return MOE_OK;
    case MOE_OPT_ROUTER_CANDIDATES: c->router_cand = value != 0; return MOE_OK;
    case MOE_OPT_UNIQUE_GGUF: c->uq_gguf = value != 0; return MOE_OK;
    case MOE_OPT_V2_FUSED_MIDDLE: c->v2_fused_mid = value != 0; return MOE_OK;
    case MOE_OPT_PAIR_TABLES: c->pair_tables = value != 0; return MOE_OK;
    case MOE_OPT_F32_DECODE_MAX_TOKENS:
      if (value < 0 || value > c->small_max) return MOE_E_INVALID;
      c->lut_max = value;
      return MOE_OK;
    case MOE_OPT_GU_TOPK_MAX_TOKENS:
      if (value < 0) return MOE_E_INVALID;
      c->gu_topk_max = value;
      return MOE_OK;
    case MOE_OPT_TIMING_SKIP_STAGE:
#ifdef MOE_TIMING_HOOKS
      // (the timing twin of the library only; and only once a complete call has filled the scratch that the stages
      //  behind the skipped one take their indices from)
      if (value < 0 || value > MOE_PROF_STAGES) return MOE_E_INVALID;
      if (value != 0 && c->ran_complete == 0) return MOE_E_STATE;
      c->skip_stage = value;
      return MOE_OK;
#else
      return MOE_E_UNSUPPORTED;  // not part of this build: a call with a stage left out returns wrong results
#endif
    default: return MOE_E_INVALID;
  }
}

MOE_API int moe_profile_enable(moe_ctx* c, int on) {
  if (!c) return MOE_E_INVALID;
  c->profile = on != 0;
  c->ev_n = 0;
  return MOE_OK;
}

MOE_API int moe_profile_read(moe_ctx* c, float* ms) {
  if (!c || !ms) return MOE_E_INVALID;
  for (int i = 0; i < MOE_PROF_STAGES; i++) ms[i] = 0.f;
  if (c->ev_n < 2) return MOE_E_STATE;
  MOE_HIP(hipEventSynchronize(c->ev[c->ev_n - 1]));
  for (int i = 1; i < c->ev_n; i++) {
    float t = 0.f;
    MOE_HIP(hipEventElapsedTime(&t, c->ev[i - 1], c->ev[i]));
    ms[c->ev_stage[i - 1]] += t;
  }
  return MOE_OK;
}

MOE_API int moe_get_routing(moe_ctx* c, int P, int* ids_out, float* ws_out, moe_stream_t st) {
  if (!c || P < 0 || P > c->cfg.max_tokens) return MOE_E_INVALID;
  const size_t n = (size_t)P * c->cfg.id_stride * 4;
  if (n == 0) return MOE_OK;
  if (ids_out) MOE_HIP(hipMemcpyAsync(ids_out, c->ids, n, hipMemcpyDeviceToDevice, moe_s(st)));
  if (ws_out) MOE_HIP(hipMemcpyAsync(ws_out, c->ws, n, hipMemcpyDeviceToDevice, moe_s(st)));
  return MOE_OK;
}

// Small batches: every (token, expert) slot reads its expert in place.  Four launches:
// logits (+ shared-gate logit), top-k, gate/up/SwiGLU (shared expert as one more slot),
// down + weighted combine + shared expert.
static int forward_small_routed(moe_ctx* c, MoeLayer& L, const float* x, int P, float* y, hipStream_t st);

static int forward_small_v2(moe_ctx* c, MoeLayer& L, const float* x, int P, float* y, hipStream_t st);

static int forward_small(moe_ctx* c, MoeLayer& L, const float* x, int P, float* y, hipStream_t st) {
  const int rc = L.has_i4r ? forward_small_v2(c, L, x, P, y, st) : forward_small_routed(c, L, x, P, y, st);
  if (rc || !L.has_shared || !L.sh_dense) return rc;
  // a densely stored shared expert: added to y behind the routed experts' kernels (its gate logit is in
  // sh_logit since the router launch); scratch: the shared slot's part of hid32
  const moe_config& g = c->cfg;
  return moe_launch_dense_shared_small(L.sh_dense, L.sh_gate.data, L.sh_up.data, L.sh_down.data, c->sh_logit, x, P, g.d,
                                       g.mid, c->hid32 + (size_t)(g.max_tokens < c->small_max ? g.max_tokens : c->small_max) * g.topk * g.mid,
                                       y, st);
}

// What the selection of a small batch needs to be certain of its expert ids (topk.h, select_certain): the router
// launch sums the products in a parallel order; |that fp64 sum - the reference's sequential one| <= 2 gamma_d |w||x|
// for any row w (gamma_d = d u / (1 - d u), u = 2^-53), so tol_scale * |x| bounds it for every logit of a token.
static moe_rfix router_fix(const moe_ctx* c, const MoeLayer& L, const float* x, bool tol_from_router) {
  moe_rfix R{};
  R.W = L.router.data;
  R.bias = L.router_bias;
  R.x = x;
  R.tol = tol_from_router ? c->rtol : nullptr;
  R.tol_scale = 2.f * (float)(c->cfg.d + 4) * 0x1p-53f * L.router_wmax * 1.05f;
  R.bf16 = L.router.dtype == MOE_DT_BF16 ? 1 : 0;
  R.d = c->cfg.d;
  return R;
}

// the router and the routed experts (and the shared expert where the kernels take it along as one more slot)
static int forward_small_routed(moe_ctx* c, MoeLayer& L, const float* x, int P, float* y, hipStream_t st) {
  const moe_config& g = c->cfg;
  int rc;
  c->ev_n = 0;
  prof_mark(c, 0, st);
  // A stage = the launches between two profile events.  MOE_OPT_TIMING_SKIP_STAGE leaves one stage's launches
  // out (timing experiments only: the output is then meaningless).
  auto stage = [&](int tag, auto&& launch) -> int {
    if (c->skip_stage != tag + 1) {
      const int e = launch();
      if (e) return e;
    }
    prof_mark(c, tag, st);
    return MOE_OK;
  };
  const bool sh = L.has_shared && !L.sh_dense;  // the shared expert rides in these kernels as one more slot
  const int nslots_d = g.topk + (sh ? 1 : 0);
  const bool use_int = L.has_q4cp && c->int_decode && L.experts_affine && (!sh || L.shared_affine) &&
                       (!sh || L.sh_gguf_type == 0) && moe_dec_supported(g.d, g.mid, nslots_d);
  const bool use_int4k = L.has_gguf && c->int_decode && L.gg.tgu == MOE_GGML_Q4_K && L.gg.tdn == MOE_GGML_Q4_K &&
                         (!sh || L.sh_gguf_type == MOE_GGML_Q4_K) && moe_dec4k_supported(g.d, g.mid, nslots_d);
  // q4cp codebooks that are not affine (the reference converter's fixed table, trained tables): the same launch
  // structure with look-up arithmetic
  // (the gate/up launch at every small-batch size -- 138 against 151 us at 20 tokens --, the down launch up to
  //  lut_max tokens: 35 against 38 us at 4 tokens, but 135 against 91 at 20)
  const bool use_lut = L.has_q4cp && c->int_decode && !use_int && (!sh || L.sh_gguf_type == 0) &&
                       moe_dec_supported(g.d, g.mid, nslots_d) && moe_dec_gu_topk_supported(g.experts, g.topk);
  // the integer-dot kernels switched off: for a*n + b codebooks the same launches with f32 arithmetic (every weight a
  // conversion and an FMA on the f32 activations; against the plain f32 kernels below, a lane keeps its group's
  // activations in registers over the block's rows and the top-k rides in the gate/up launch)
  const bool use_f32a = L.has_q4cp && !c->int_decode && L.experts_affine && (!sh || L.shared_affine) &&
                        (!sh || L.sh_gguf_type == 0) && moe_dec_supported(g.d, g.mid, nslots_d) &&
                        moe_dec_gu_topk_supported(g.experts, g.topk);
  // GGUF layers in other mixes of Q4_K / Q5_K / Q8_0 / Q5_1 (the reference checkpoints' types): the same integer-dot
  // launches, generalised over the block type
  const bool use_intgg = L.has_gguf && c->int_decode && !use_int4k &&
                         moe_decgg_supported(L.gg.tgu, L.gg.tdn, L.sh_gguf_type, sh, g.d, g.mid, g.topk, g.experts) &&
                         (!sh || L.sh_gguf_type != 0);
  const bool use_uq = use_int && c->uq_min > 0 && P >= c->uq_min && moe_dec_uq_supported(g.d);
  // the same for GGUF layers on the integer-dot kernels (any mix of their four block types)
  const bool use_uq_gg = (use_int4k || use_intgg) && c->uq_gguf && c->uq_min > 0 && P >= c->uq_min && moe_decgg_uq_supported(g.d) &&
                         moe_decgg_supported(L.gg.tgu, L.gg.tdn, L.sh_gguf_type, sh, g.d, g.mid, g.topk, g.experts) &&
                         (!sh || L.sh_gguf_type != 0);
  // integer-dot kernels: the gate/up launch runs the softmax / top-k itself (one launch less on the
  // latency-bound path than a top-k kernel, no last-block ticket in the logits launch)
  const bool gu_topk = (((use_int && !use_uq) || ((use_int4k || use_intgg) && !use_uq_gg) || use_lut || use_f32a) && P <= c->gu_topk_max) &&
                       moe_dec_gu_topk_supported(g.experts, g.topk);
  // (up to 4 tokens the router launch leaves each token's bound for the selection; larger batches: the selecting
  //  block takes the norm of x itself)
  const moe_rfix rf = router_fix(c, L, x, P <= 4);
  if ((rc = stage(MOE_PROF_ROUTER, [&]() -> int {
         bool fused = false;
         // (the selection runs in launches of its own here, so that it can be made certain: no top-k inside the logits launch)
         int e = moe_router_logits_small(&L.router, L.router_bias, L.has_shared ? &L.sh_sg : nullptr, x, P, c->logits,
                                         c->sh_logit, (use_int || use_int4k || use_intgg) ? c->xplanes : nullptr, c->xmeta,
                                         use_int4k || use_intgg, nullptr, c->ids, c->ws, g.topk,
                                         g.id_stride, &fused, st, c->kpart, c->ktickets, nullptr, P <= 4 && rf.W ? c->rtol : nullptr,
                                         rf.tol_scale);
         if (!e && !gu_topk)
           e = moe_launch_router_topk_small(c->logits, c->ids, c->ws, P, g.experts, g.topk, g.id_stride, &rf, st);
         return e;
       })))
    return rc;
  const moe_wview *shg = sh ? &L.sh_gate : nullptr, *shu = sh ? &L.sh_up : nullptr, *shd = sh ? &L.sh_down : nullptr;
  const uint8_t *rg = sh ? L.sh_gate.data : nullptr, *ru = sh ? L.sh_up.data : nullptr, *rd = sh ? L.sh_down.data : nullptr;
  if (L.has_q4cp) {
    if (sh && L.sh_gguf_type != 0) return MOE_E_UNSUPPORTED;
    if (use_uq) {
      // verify-size batches: tokens share experts; walk the expert-sorted pair lists so that every
      // distinct expert's weights are read once (reference: the _uq kernels, 26_kernels_moe_gguf.inc:758-877)
      const int sh_first = sh ? P * g.topk : -1;
      const int max_tiles = P * g.topk + (sh ? (P + 3) / 4 : 0);  // tiles of <= 4 pairs
      if ((rc = stage(MOE_PROF_ROUTE, [&]() -> int {
             if (moe_route_small_supported(P, g.topk, g.experts))  // permutation and tiles in one launch
               return moe_launch_route_small(c->ids, c->ws, c->tokidx, c->pw, c->eoff, c->pairids, P, g.topk,
                                             g.experts, g.id_stride, c->tiles, c->ntiles, 4, sh_first, st);
             const int e = moe_routing_run(c->routing, c->ids, c->ws, c->tokidx, c->pw, c->eoff, c->pairids, P,
                                           g.topk, g.experts, g.id_stride, st);
             return e ? e : moe_launch_tiles_shared(c->eoff, c->tiles, c->ntiles, g.experts, 4, P, sh_first, c->tokidx, st);
           })))
        return rc;
      if ((rc = stage(MOE_PROF_UP, [&]() -> int {
             return moe_launch_dec_gu_uq(&L.gate_up, shg, shu, c->xplanes, c->xmeta, c->tiles, c->ntiles, max_tiles,
                                         c->tokidx, g.experts, g.d, g.mid, c->hplanes, c->hmeta, st);
           })))
        return rc;
      if ((rc = stage(MOE_PROF_DOWN, [&]() -> int {
             return moe_launch_dec_dn_uq(&L.down, shd, c->hplanes, c->hmeta, c->tiles, c->ntiles, max_tiles, g.experts,
                                         g.d, g.mid, c->pairs32, st);
           })))
        return rc;
      return stage(MOE_PROF_REDUCE, [&]() -> int {
        return moe_launch_reduce(c->pairs32, false, c->pairids, c->pw, nullptr, sh ? c->sh_logit : nullptr, sh_first, y,
                                 P, g.d, g.topk, moe_hscale{nullptr, 0.f, 0.f}, st, nullptr);
      });
    }
    if (use_int) {
      // integer-dot kernels: activations as digit planes (made by the logits launch above)
      if ((rc = stage(MOE_PROF_UP, [&]() -> int {
             return gu_topk ? moe_launch_dec_gu_topk(&L.gate_up, shg, shu, c->xplanes, c->xmeta, c->logits, g.experts,
                                                     c->ids, c->ws, g.id_stride, g.topk, P, g.d, g.mid, c->hplanes,
                                                     c->hmeta, nullptr, st, nullptr, &rf)
                            : moe_launch_dec_gu(&L.gate_up, shg, shu, c->xplanes, c->xmeta, c->ids, g.id_stride, g.topk,
                                                P, g.d, g.mid, c->hplanes, c->hmeta, nullptr, st);
           })))
        return rc;
      return stage(MOE_PROF_DOWN, [&]() -> int {
        return moe_launch_dec_dn(&L.down, shd, c->sh_logit, c->hplanes, c->hmeta, c->ids, c->ws, g.id_stride, g.topk, P,
                                 g.d, g.mid, y, (uint64_t)g.d, st);
      });
    }
    if (use_lut || use_f32a) {
      // table codebooks past the few-token sizes: the plain f32 down kernel looks the routed experts' weights up two
      // at a time in a pair table (the gate/up kernel was measured with one as well: no gain, its LDS traffic per
      // weight stays what it is)
      const bool pair_tabs = use_lut && !use_f32a && c->pair_tables && P > c->lut_max;
      if ((rc = stage(MOE_PROF_UP, [&]() -> int {
             return moe_launch_dec_gu_lut(&L.gate_up, shg, shu, x, gu_topk ? c->logits : nullptr, g.experts, c->ids, c->ws,
                                          g.id_stride, g.topk, P, g.d, g.mid, c->hid32, st, &rf, use_f32a);
           })))
        return rc;
      return stage(MOE_PROF_DOWN, [&]() -> int {
        // (the down projection of more than a few tokens: the plain f32 kernel's blocks of 32 rows read a token's
        //  hidden rows once for all of them and measure faster from about 6 tokens on)
        if (P > c->lut_max)
          return moe_launch_gemv_dn(&L.down, shd, c->sh_logit, nullptr, nullptr, c->hid32, c->ids, c->ws, g.id_stride,
                                    g.topk, P, g.d, y, (uint64_t)g.d, st, pair_tabs);
        return moe_launch_dec_dn_lut(&L.down, shd, c->sh_logit, c->hid32, c->ids, c->ws, g.id_stride, g.topk, P, g.d,
                                     g.mid, y, (uint64_t)g.d, st, use_f32a);
      });
    }
    if ((rc = stage(MOE_PROF_UP, [&]() -> int {
           return moe_launch_gemv_gu(&L.gate_up, shg, shu, x, (uint64_t)g.d, c->ids, g.id_stride, g.topk, P, g.mid,
                                     c->hid32, st);
         })))
      return rc;
    return stage(MOE_PROF_DOWN, [&]() -> int {
      return moe_launch_gemv_dn(&L.down, shd, c->sh_logit, nullptr, nullptr, c->hid32, c->ids, c->ws, g.id_stride,
                                g.topk, P, g.d, y, (uint64_t)g.d, st, false);
    });
  }
  if (sh && L.sh_gguf_type == 0) return MOE_E_UNSUPPORTED;
  if (use_uq_gg) {
    // verify-size batches of a GGUF layer: every distinct expert's rows read once (reference: the _uq kernels,
    // 26_kernels_moe_gguf.inc:758-886)
    const int cap = moe_decgg_uq_tile_cap();
    const int sh_first = sh ? P * g.topk : -1;
    const int max_tiles = P * g.topk + (sh ? (P + cap - 1) / cap : 0);
    if ((rc = stage(MOE_PROF_ROUTE, [&]() -> int {
           if (moe_route_small_supported(P, g.topk, g.experts))
             return moe_launch_route_small(c->ids, c->ws, c->tokidx, c->pw, c->eoff, c->pairids, P, g.topk, g.experts,
                                           g.id_stride, c->tiles, c->ntiles, cap, sh_first, st);
           const int e = moe_routing_run(c->routing, c->ids, c->ws, c->tokidx, c->pw, c->eoff, c->pairids, P, g.topk,
                                         g.experts, g.id_stride, st);
           return e ? e : moe_launch_tiles_shared(c->eoff, c->tiles, c->ntiles, g.experts, cap, P, sh_first, c->tokidx, st);
         })))
      return rc;
    if ((rc = stage(MOE_PROF_UP, [&]() -> int {
           return moe_launch_decgg_gu_uq(L.gg.tgu, L.sh_gguf_type, L.gg.gate, L.gg.up, rg, ru, c->xplanes, c->xmeta, c->tiles,
                                         c->ntiles, max_tiles, c->tokidx, g.experts, g.d, g.mid, c->hplanes, c->hmeta, st);
         })))
      return rc;
    if ((rc = stage(MOE_PROF_DOWN, [&]() -> int {
           return moe_launch_decgg_dn_uq(L.gg.tdn, L.sh_gguf_type, L.gg.down, rd, c->hplanes, c->hmeta, c->tiles, c->ntiles,
                                         max_tiles, g.experts, g.d, g.mid, c->pairs32, st);
         })))
      return rc;
    return stage(MOE_PROF_REDUCE, [&]() -> int {
      return moe_launch_reduce(c->pairs32, false, c->pairids, c->pw, nullptr, sh ? c->sh_logit : nullptr, sh_first, y, P,
                               g.d, g.topk, moe_hscale{nullptr, 0.f, 0.f}, st, nullptr);
    });
  }
  if (use_intgg) {
    if ((rc = stage(MOE_PROF_UP, [&]() -> int {
           return gu_topk ? moe_launch_decgg_gu_topk(L.gg.tgu, L.sh_gguf_type, L.gg.gate, L.gg.up, rg, ru, c->xplanes,
                                                     c->xmeta, c->logits, g.experts, c->ids, c->ws, g.id_stride, g.topk,
                                                     P, g.d, g.mid, c->hplanes, c->hmeta, st, &rf)
                          : moe_launch_decgg_gu(L.gg.tgu, L.sh_gguf_type, L.gg.gate, L.gg.up, rg, ru, c->xplanes, c->xmeta,
                                                c->ids, g.experts, g.id_stride, g.topk, P, g.d, g.mid, c->hplanes, c->hmeta,
                                                st);
         })))
      return rc;
    return stage(MOE_PROF_DOWN, [&]() -> int {
      return moe_launch_decgg_dn(L.gg.tdn, L.sh_gguf_type, L.gg.down, rd, c->sh_logit, c->hplanes, c->hmeta, c->ids, c->ws,
                                 g.id_stride, g.topk, P, g.d, g.mid, y, (uint64_t)g.d, st);
    });
  }
  if (L.gg.tgu != MOE_GGML_Q4_K || L.gg.tdn != MOE_GGML_Q4_K || (sh && L.sh_gguf_type != MOE_GGML_Q4_K)) {
    // Q5_K gate/up, Q5_1 / Q8_0 down (or such a shared expert): the general kernels
    for (int phase = 1; phase <= 2; phase++)
      if ((rc = stage(phase == 1 ? MOE_PROF_UP : MOE_PROF_DOWN, [&]() -> int {
             return moe_launch_ggx_gemv(phase, L.gg.tgu, L.gg.tdn, L.sh_gguf_type, L.gg.gate, L.gg.up, L.gg.down, rg, ru,
                                        rd, c->sh_logit, x, c->ids, c->ws, c->hid32, y, P, g.d, g.mid, g.topk,
                                        g.id_stride, st);
           })))
        return rc;
    return MOE_OK;
  }
  if (use_int4k) {
    if ((rc = stage(MOE_PROF_UP, [&]() -> int {
           return gu_topk ? moe_launch_dec4k_gu_topk(L.gg.gate, L.gg.up, rg, ru, c->xplanes, c->xmeta, c->logits,
                                                     g.experts, c->ids, c->ws, g.id_stride, g.topk, P, g.d, g.mid,
                                                     c->hplanes, c->hmeta, st, &rf)
                          : moe_launch_dec4k_gu(L.gg.gate, L.gg.up, rg, ru, c->xplanes, c->xmeta, c->ids, g.id_stride,
                                                g.topk, P, g.d, g.mid, c->hplanes, c->hmeta, st);
         })))
      return rc;
    return stage(MOE_PROF_DOWN, [&]() -> int {
      return moe_launch_dec4k_dn(L.gg.down, rd, c->sh_logit, c->hplanes, c->hmeta, c->ids, c->ws, g.id_stride, g.topk, P,
                                 g.d, g.mid, y, (uint64_t)g.d, st);
    });
  }
  for (int phase = 1; phase <= 2; phase++)
    if ((rc = stage(phase == 1 ? MOE_PROF_UP : MOE_PROF_DOWN, [&]() -> int {
           return moe_launch_q4k_gemv(phase, L.gg.gate, L.gg.up, L.gg.down, rg, ru, rd, c->sh_logit, x, c->ids, c->ws,
                                      c->hid32, y, P, g.d, g.mid, g.topk, g.id_stride, st);
         })))
      return rc;
  return MOE_OK;
}

// hgn v2 rotated experts, small batches (reference: moe_v2_1, 40_model.inc:1638-1656): the integer-dot launches of
// the q4cp path with the rotations in between --
//   router logits (+ planes of x for the shared expert's slot) -> planes of rot_in(x, su)
//   -> gate | up sums of the routed slots, unfused (the shared expert's slot as usual)
//   -> per slot rot_out(svh_gu), SwiGLU, rot_in(suh_dn) -> planes
//   -> down + weighted sum (the shared expert's rows aside) -> rot_out(svh_dn) + shared expert.
static int forward_small_v2(moe_ctx* c, MoeLayer& L, const float* x, int P, float* y, hipStream_t st) {
  const moe_config& g = c->cfg;
  int rc;
  c->ev_n = 0;
  prof_mark(c, 0, st);
  auto stage = [&](int tag, auto&& launch) -> int {
    if (c->skip_stage != tag + 1) {
      const int e = launch();
      if (e) return e;
    }
    prof_mark(c, tag, st);
    return MOE_OK;
  };
  const bool sh = L.has_shared && !L.sh_dense;  // a q4cp shared expert rides in these kernels as one more slot
  if (sh && (L.sh_gguf_type != 0 || !L.shared_affine)) return MOE_E_UNSUPPORTED;
  const int nslots_d = g.topk + (sh ? 1 : 0);
  const bool gu_topk = P <= c->gu_topk_max;
  const moe_rfix rf = router_fix(c, L, x, P <= 4);
  if ((rc = stage(MOE_PROF_ROUTER, [&]() -> int {
         bool fused = false;
         // (the planes of rot_in(x, su) ride in the router launch's spare blocks)
         const moe_rot_planes rot{L.v2_su, c->v2_xplanes, c->v2_xmeta};
         int e = moe_router_logits_small(&L.router, L.router_bias, L.has_shared ? &L.sh_sg : nullptr, x, P, c->logits,
                                         c->sh_logit, sh ? c->xplanes : nullptr, c->xmeta, false,
                                         nullptr, c->ids, c->ws, g.topk, g.id_stride, &fused, st,
                                         c->kpart, c->ktickets, &rot, P <= 4 && rf.W ? c->rtol : nullptr, rf.tol_scale);
         if (!e && !gu_topk) e = moe_launch_router_topk_small(c->logits, c->ids, c->ws, P, g.experts, g.topk, g.id_stride, &rf, st);
         return e;
       })))
    return rc;
  const moe_wview *shg = sh ? &L.sh_gate : nullptr, *shu = sh ? &L.sh_up : nullptr, *shd = sh ? &L.sh_down : nullptr;
  if ((rc = stage(MOE_PROF_UP, [&]() -> int {
         const moe_dec_v2 v2{c->v2_zraw, c->v2_xplanes, c->v2_xmeta};
         const int e = gu_topk ? moe_launch_dec_gu_topk(&L.gate_up, shg, shu, c->xplanes, c->xmeta, c->logits, g.experts,
                                                        c->ids, c->ws, g.id_stride, g.topk, P, g.d, g.mid, c->hplanes,
                                                        c->hmeta, nullptr, st, &v2, &rf)
                               : moe_launch_dec_gu(&L.gate_up, shg, shu, c->xplanes, c->xmeta, c->ids, g.id_stride, g.topk,
                                                   P, g.d, g.mid, c->hplanes, c->hmeta, nullptr, st, &v2);
         return e ? e : moe_launch_i4r_mid(c->v2_zraw, false, (uint64_t)2 * g.mid, P * g.topk, g.mid, L.v2_svh_gu,
                                           L.v2_suh_dn, 2, nullptr, 0, g.topk, nslots_d, c->hplanes, c->hmeta, st);
       })))
    return rc;
  return stage(MOE_PROF_DOWN, [&]() -> int {
    const int e = moe_launch_dec_dn(&L.down, shd, c->sh_logit, c->hplanes, c->hmeta, c->ids, c->ws, g.id_stride, g.topk, P,
                                    g.d, g.mid, c->v2_acc, (uint64_t)g.d, st, sh ? c->v2_ey : nullptr);
    return e ? e : moe_launch_v2_rot(c->v2_acc, (uint64_t)g.d, P, g.d, nullptr, L.v2_svh_dn, 0, y, (uint64_t)g.d,
                                     sh ? c->v2_ey : nullptr, (uint64_t)g.d, nullptr, nullptr, st);
  });
}

// Which grouped GEMM each of a GGUF layer's four launches takes.  The tuned kernel (gemm_q4cp.hip: raw K-quant blocks
// dequantised in registers, activations in the order the unpack produces) has gate/up forms for Q4_K and Q5_K and a
// down form for Q4_K, which reads the hid rows its own gate/up form wrote; everything else (Q8_0, Q5_1, IQ4 types,
// densely stored shared experts) goes through the general kernel (gguf_types.hip), which puts activations of either
// order back into natural order on their way into LDS.
struct GgKinds {
  bool r_gu, r_dn, s_gu, s_dn;  // tuned? (routed gate/up, routed down, shared gate/up, shared down)
  bool any_tuned() const { return r_gu || s_gu; }
  // routed and shared tiles can share a launch when they take the same kernel with the same block type (the general
  // kernel reads any two types in one launch, but its pipelined Q8_0 / Q5_1 forms want one type per launch)
  bool uniform(const MoeLayer& L) const {
    if (!L.has_shared) return true;
    if (L.sh_dense) return false;
    return r_gu == s_gu && r_dn == s_dn && L.gg.tgu == L.sh_gguf_type && L.gg.tdn == L.sh_gguf_type;
  }
};
static GgKinds gg_kinds(const MoeLayer& L, const moe_config& g) {
  const int d = g.d, mid = g.mid;
  GgKinds k{false, false, false, false};
  if (!L.has_gguf) return k;
  // (the Q5_K form wants tensors and activation rows below 4 GB: 32-bit byte offsets)
  auto gu_ok = [&](int t, uint64_t rows) {
    return t == MOE_GGML_Q4_K || (t == MOE_GGML_Q5_K && moe_gemm_q5k_fits(rows, (uint64_t)g.max_tokens, d));
  };
  const bool shapes = d % 256 == 0 && mid % 256 == 0;
  k.r_gu = shapes && gu_ok(L.gg.tgu, (uint64_t)g.experts * mid);
  k.r_dn = k.r_gu && L.gg.tdn == MOE_GGML_Q4_K;
  if (L.has_shared && !L.sh_dense) {
    k.s_gu = shapes && gu_ok(L.sh_gguf_type, (uint64_t)mid);
    k.s_dn = k.s_gu && L.sh_gguf_type == MOE_GGML_Q4_K;
  }
  return k;
}
// the order of the f16 activations a layer's grouped GEMMs read (moe_f32_to_f16's layout)
// q4cp experts whose codebook is a table (not a*n + b): the grouped GEMMs of the whole layer then run in natural K
// order and dequantise through pair tables (gemm_q4cp.hip, NAT); affine experts keep the interleaved order
static bool batch_nat(const MoeLayer& L) { return L.has_q4cp && !L.has_i4r && !L.experts_affine; }
static int batch_x16_layout(const MoeLayer& L, const moe_config& g) {
  if (!L.has_gguf) return batch_nat(L) ? 0 : 1;
  return gg_kinds(L, g).any_tuned() ? 2 : 0;
}

// Router of a batch: ids / ws, the shared-expert gate logit and (if asked) the per-token mean square of x.
// By default through candidate selection (router_cand.hip); MOE_OPT_ROUTER_CANDIDATES = 0, or a shape it does not
// take, runs the dense fp64 launch and the exact softmax / top-k over all experts.
static int router_batch(moe_ctx* c, MoeLayer& L, const float* x, int P, float* out_xms, hipStream_t st) {
  const moe_config& g = c->cfg;
  const moe_wview* wx = L.has_shared ? &L.sh_sg : nullptr;
  if (c->router_cand && c->rc_scratch && moe_router_cand_supported(&L.router, wx, P, g.topk))
    return moe_router_batch_cand(&L.router, L.router_bias, wx, x, P, c->logits, c->sh_logit, out_xms, c->ids, c->ws,
                                 g.topk, g.id_stride, c->rc_scratch, st, L.router_bmax);
  int rc = moe_router_logits_seq(&L.router, L.router_bias, wx, x, P, c->logits, c->sh_logit, out_xms, st);
  if (!rc) rc = moe_router_topk(c->logits, c->ids, c->ws, P, g.experts, g.topk, g.id_stride, st);
  return rc;
}

// Batches: expert-sorted permutation, MFMA grouped GEMMs over <=128-pair tiles (the shared expert
// rides along as expert index E over all tokens), f16 pair buffer, deterministic weighted combine.
// Returns MOE_E_UNSUPPORTED (before enqueuing anything) for shapes / formats the GEMM does not cover.
static int forward_batch_impl(moe_ctx* c, MoeLayer& L, const float* x, int P, float* y, hipStream_t st, bool* enqueued);

static int forward_batch(moe_ctx* c, MoeLayer& L, const float* x, int P, float* y, hipStream_t st) {
  bool enqueued = false;
  const int rc = forward_batch_impl(c, L, x, P, y, st, &enqueued);
  // "unsupported" promises the caller that nothing ran; past the first launch it is a broken call instead
  return rc == MOE_E_UNSUPPORTED && enqueued ? MOE_E_STATE : rc;
}

static int forward_batch_impl(moe_ctx* c, MoeLayer& L, const float* x, int P, float* y, hipStream_t st, bool* enqueued) {
  const moe_config& g = c->cfg;
  const bool q4k = L.has_gguf;  // raw GGUF blocks
  // hgn v2 rotated experts (reference: moe_b_v2, 40_model.inc:4570-4686): the routed launches read rot_in(x, su),
  // leave gate | up unfused for the rotations around SwiGLU, and the combine rotates the weighted sum
  const bool v2 = L.has_i4r;
  if (v2 && (!c->v2_x16 || g.d % 256 || g.mid % 256)) return MOE_E_UNSUPPORTED;
  // GGUF layers: each launch on the tuned kernel where it has a form for the block type, else on the general one
  const GgKinds kd = gg_kinds(L, g);
  const bool shd = L.has_shared && L.sh_dense;  // shared expert stored densely: the general GEMM, launches of its own
  const bool split = shd || (q4k && !kd.uniform(L));  // routed and shared experts in launches of their own
  if (L.has_shared && !shd && (L.sh_gguf_type != 0) != q4k) return MOE_E_UNSUPPORTED;  // one format family per layer
  if (q4k ? (g.d % 64 || g.mid % 64) : (g.d % 128 || g.mid % 128 || g.mid < 256 || g.d < 256))
    return MOE_E_UNSUPPORTED;  // the caller walks the batch through the small path
  moe_lutw gu{}, dn{}, sgu{}, sdn{};
  const float* sh_cb_up = nullptr;
  if (q4k) {
    gu.w = L.gg.gate; gu.w_up = L.gg.up; gu.e_rows = g.mid;
    dn.w = L.gg.down; dn.e_rows = g.d;
    if (L.has_shared && !shd) {
      sgu.w = L.sh_gate.data; sgu.w_up = L.sh_up.data; sgu.e_rows = g.mid;
      sdn.w = L.sh_down.data; sdn.e_rows = g.d;
    }
  } else if (v2) {
    int e = moe_lut_i4r_view(L.gate_up.data, L.gate_up.rows, L.gate_up.cols, 2 * g.mid, 0, &gu);
    if (!e) e = moe_lut_i4r_view(L.down.data, L.down.rows, L.down.cols, g.d, 0, &dn);
    if (e) return e;
  } else {
    moe_lut_q4cp_view(L.gate_up.data, L.gate_up.rows, L.gate_up.cols, L.gate_up.scale_stride, 2 * g.mid, g.mid, &gu);
    moe_lut_q4cp_view(L.down.data, L.down.rows, L.down.cols, L.down.scale_stride, g.d, 0, &dn);
  }
  if (L.has_shared && !q4k && !shd) {
    moe_lutw t;
    moe_lut_q4cp_view(L.sh_gate.data, L.sh_gate.rows, L.sh_gate.cols, L.sh_gate.scale_stride, g.mid, 0, &sgu);
    moe_lut_q4cp_view(L.sh_up.data, L.sh_up.rows, L.sh_up.cols, L.sh_up.scale_stride, g.mid, 0, &t);
    sgu.w_up = t.w;
    sgu.sc_up = t.sc;
    sh_cb_up = t.cb;  // up_proj is a tensor of its own, with its own codebook (the converter trains one per tensor)
    moe_lut_q4cp_view(L.sh_down.data, L.sh_down.rows, L.sh_down.cols, L.sh_down.scale_stride, g.d, 0, &sdn);
  }
  int rc;
  const moe_hscale hs{c->xms, L.c_routed, L.c_shared};
  const __half* xh = c->x16_ext ? c->x16_ext : c->x16;  // f16 activations in the GEMM's order
  const int xl = batch_x16_layout(L, g);       // that order (moe_f32_to_f16's layout)
  const bool nat = batch_nat(L);               // table codebooks: natural K order, pair tables
  // scaled dequantisation (affine q4cp codebooks): the powers of two found when the weights were registered
  const bool pe_r = L.has_q4cp && !v2 && L.experts_affine, pe_s = L.has_shared && !shd && !q4k && L.shared_affine;
  const int8_t* pe_gu = pe_r ? pexp_slot(c, (int)(&L - c->layers.data()), 0) : nullptr;
  const int8_t* pe_dn = pe_r ? pexp_slot(c, (int)(&L - c->layers.data()), g.experts) : nullptr;
  const int8_t* pe_sgu = pe_s ? pexp_slot(c, (int)(&L - c->layers.data()), 2 * g.experts) : nullptr;
  const int8_t* pe_sdn = pe_s ? pexp_slot(c, (int)(&L - c->layers.data()), 2 * g.experts + 1) : nullptr;
  // gate/up (+ SwiGLU) and down launches over a tile list: routed experts, with_sh: the shared expert as well
  // (tiles whose expert index is >= n_experts)
  // dry: the launchers run their shape / type / alignment checks and return in front of the launch (a tile capacity
  // of 0), so that every reason to decline is found before anything is enqueued
  bool dry = true;
  auto gemm_up = [&](bool with_sh, const moe_tile* tl, const int* ntl, int mt, hipStream_t s2) -> int {
    if (dry) mt = 0;
    if (shd && with_sh)  // the shared expert's own tile list
      return moe_launch_gemm_gg(true, L.sh_dense, L.sh_gate.data, L.sh_up.data, 0, nullptr, nullptr, g.experts, xh,
                                c->tokidx, tl, ntl, mt, c->hid16, g.mid, g.d, hs, s2, xl);
    if (q4k && split) {  // one class per launch: the shared expert's tiles (with_sh) or the routed experts'
      if (with_sh ? kd.s_gu : kd.r_gu)
        return moe_launch_gemm_q4cp(true, with_sh ? &sgu : &gu, with_sh ? &sgu : nullptr, g.experts, xh, c->tokidx, tl, ntl,
                                    mt, c->hid16, g.mid, g.d, true, true, hs, s2, nullptr, nullptr, 0,
                                    (with_sh ? L.sh_gguf_type : L.gg.tgu) == MOE_GGML_Q5_K);
      return with_sh ? moe_launch_gemm_gg(true, L.sh_gguf_type, L.sh_gate.data, L.sh_up.data, L.sh_gguf_type,
                                          L.sh_gate.data, L.sh_up.data, g.experts, xh, c->tokidx, tl, ntl, mt, c->hid16,
                                          g.mid, g.d, hs, s2, xl)
                     : moe_launch_gemm_gg(true, L.gg.tgu, L.gg.gate, L.gg.up, 0, nullptr, nullptr, g.experts, xh,
                                          c->tokidx, tl, ntl, mt, c->hid16, g.mid, g.d, hs, s2, xl);
    }
    if (q4k && !kd.r_gu)
      return moe_launch_gemm_gg(true, L.gg.tgu, L.gg.gate, L.gg.up, L.sh_gguf_type, with_sh ? L.sh_gate.data : nullptr,
                                with_sh ? L.sh_up.data : nullptr, g.experts, xh, c->tokidx, tl, ntl, mt, c->hid16, g.mid,
                                g.d, hs, s2, xl);
    if (v2 && !with_sh) {
      // the routed experts' tiles: gate rows and their up rows in one block, the slot-wise middle (rotation back,
      // SwiGLU, rotation for down_proj) in the launch's epilogue
      if (c->v2_fused_mid) {
        moe_lutw gf = gu;
        gf.up_off = g.mid;
        const moe_rotv rv{L.v2_svh_gu, L.v2_suh_dn};
        return moe_launch_gemm_q4cp(true, &gf, nullptr, g.experts, c->v2_x16, c->tokidx, tl, ntl, mt, c->hid16, g.mid, g.d,
                                    true, false, hs, s2, nullptr, nullptr, 2, false, false, nullptr, nullptr, &rv);
      }
      // (the earlier form: plain rows of the fused tensor as f16 sums, then the middle as a launch of its own)
      const int e = moe_launch_gemm_q4cp(false, &gu, nullptr, g.experts, c->v2_x16, c->tokidx, tl, ntl, mt, c->v2_z16,
                                         2 * g.mid, g.d, true, false, moe_hscale{nullptr, 0.f, 0.f}, s2, nullptr, nullptr, 2);
      return e || dry ? e : moe_launch_i4r_mid(c->v2_z16, true, (uint64_t)2 * g.mid, P * g.topk, g.mid, L.v2_svh_gu, L.v2_suh_dn,
                                        1, c->hid16, (uint64_t)g.mid, 1, 1, nullptr, nullptr, s2, c->xms, L.c_routed, c->tokidx);
    }
    if (v2)  // the shared expert's own tile list (q4cp, not rotated; every tile's expert index is >= n_experts)
      return moe_launch_gemm_q4cp(true, &sgu, &sgu, g.experts, xh, c->tokidx, tl, ntl, mt, c->hid16, g.mid, g.d, true,
                                  false, hs, s2, nullptr, sh_cb_up, 0, false, false, pe_sgu, pe_sgu);
    return moe_launch_gemm_q4cp(true, &gu, with_sh ? &sgu : nullptr, g.experts, xh, c->tokidx, tl, ntl, mt, c->hid16,
                                g.mid, g.d, true, q4k, hs, s2, nullptr, sh_cb_up, 0, q4k && L.gg.tgu == MOE_GGML_Q5_K, nat,
                                pe_gu, pe_sgu);
  };
  auto gemm_dn = [&](bool with_sh, const moe_tile* tl, const int* ntl, int mt, hipStream_t s2, const moe_comb* cmb) -> int {
    if (dry) mt = 0;
    if (shd && with_sh)  // (hid rows of the shared tiles were written in natural order by the launch above)
      return moe_launch_gemm_gg(false, L.sh_dense, L.sh_down.data, nullptr, 0, nullptr, nullptr, g.experts, c->hid16,
                                nullptr, tl, ntl, mt, c->pairs16, g.d, g.mid, hs, s2, 0);
    if (q4k && split) {
      // (hid rows are in the tuned kernel's order where its gate/up form wrote them, else in natural order)
      if (with_sh ? kd.s_dn : kd.r_dn)
        return moe_launch_gemm_q4cp(false, with_sh ? &sdn : &dn, with_sh ? &sdn : nullptr, g.experts, c->hid16, nullptr, tl,
                                    ntl, mt, c->pairs16, g.d, g.mid, true, true, hs, s2, nullptr);
      return with_sh ? moe_launch_gemm_gg(false, L.sh_gguf_type, L.sh_down.data, nullptr, L.sh_gguf_type, L.sh_down.data,
                                          nullptr, g.experts, c->hid16, nullptr, tl, ntl, mt, c->pairs16, g.d, g.mid, hs, s2,
                                          kd.s_gu ? 2 : 0)
                     : moe_launch_gemm_gg(false, L.gg.tdn, L.gg.down, nullptr, 0, nullptr, nullptr, g.experts, c->hid16,
                                          nullptr, tl, ntl, mt, c->pairs16, g.d, g.mid, hs, s2, kd.r_gu ? 2 : 0);
    }
    if (q4k && !kd.r_dn)
      return moe_launch_gemm_gg(false, L.gg.tdn, L.gg.down, nullptr, L.sh_gguf_type, with_sh ? L.sh_down.data : nullptr,
                                nullptr, g.experts, c->hid16, nullptr, tl, ntl, mt, c->pairs16, g.d, g.mid, hs, s2,
                                kd.r_gu ? 2 : 0);
    if (v2 && !with_sh)
      return moe_launch_gemm_q4cp(false, &dn, nullptr, g.experts, c->hid16, nullptr, tl, ntl, mt, c->pairs16, g.d, g.mid,
                                  true, false, moe_hscale{nullptr, 0.f, 0.f}, s2, nullptr, nullptr, 2);
    if (v2)
      return moe_launch_gemm_q4cp(false, &sdn, &sdn, g.experts, c->hid16, nullptr, tl, ntl, mt, c->pairs16, g.d, g.mid,
                                  true, false, hs, s2, nullptr, nullptr, 0, false, false, pe_sdn, pe_sdn);
    return moe_launch_gemm_q4cp(false, &dn, with_sh ? &sdn : nullptr, g.experts, c->hid16, nullptr, tl, ntl, mt,
                                cmb ? (void*)cmb->y : (void*)c->pairs16, g.d, g.mid, cmb == nullptr, q4k, hs, s2, cmb, nullptr,
                                0, false, nat, pe_dn, pe_sdn);
  };
  const bool fused = c->fused_combine && !c->hc && !(q4k && !kd.r_dn) && !split && !v2;  // the HC write-back belongs to the ordered combine
  const bool aside = v2 || (L.has_shared && (split || (c->shared_aside && !fused)));
  {
    const moe_comb cmb0{y, c->tokidx, c->pw, L.has_shared ? c->sh_logit : nullptr};
    int pre = MOE_OK;
    if (aside) {
      if (L.has_shared) {
        pre = gemm_up(true, c->tiles_sh, c->ntiles_sh, 0, st);
        if (!pre) pre = gemm_dn(true, c->tiles_sh, c->ntiles_sh, 0, st, nullptr);
      }
      if (!pre) pre = gemm_up(false, c->tiles, c->ntiles, 0, st);
      if (!pre) pre = gemm_dn(false, c->tiles, c->ntiles, 0, st, nullptr);
    } else {
      pre = gemm_up(L.has_shared, c->tiles, c->ntiles, 0, st);
      if (!pre) pre = gemm_dn(L.has_shared, c->tiles, c->ntiles, 0, st, fused ? &cmb0 : nullptr);
    }
    if (pre) return pre;  // nothing has been enqueued
    dry = false;
  }
  *enqueued = true;
  c->ev_n = 0;
  prof_mark(c, 0, st);
  if (aside) {
    // The shared expert does not depend on the routing: its two GEMMs run on the side stream from the start
    // of the call, next to the fp64 router launch and the latency-bound top-k / permutation launches.  The
    // side stream also makes what both streams need first: the per-token mean square of x (range guard) and
    // the f16 copy of x.  Joins: in front of the routed gate/up GEMM (x16, xms) and in front of the combine.
    const int sh_first = P * g.topk;
    const int max_tiles_sh = (P + 127) / 128;
    const int max_tiles = (P * g.topk + 127) / 128 + g.experts;
    MOE_HIP(hipEventRecord(c->ev_fork, st));
    MOE_HIP(hipStreamWaitEvent(c->side, c->ev_fork, 0));
    int rs = MOE_OK;
    if (v2) rs = moe_launch_v2_rot(x, (uint64_t)g.d, P, g.d, L.v2_su, nullptr, 1, c->v2_x16, (uint64_t)g.d, nullptr, 0, nullptr, nullptr, c->side);
    if (!rs)
      rs = c->x16_ext ? moe_launch_meansq_f16(xh, P, g.d, c->xms, c->side)
                      : moe_launch_f16_rows_meansq(x, c->x16, P, g.d, xl, c->xms, c->side);
    hipError_t ee = hipEventRecord(c->ev_x16, c->side);
    if (!rs && ee != hipSuccess) rs = (int)ee;
    if (L.has_shared) {
      if (!rs) rs = moe_launch_tiles_only_shared(c->tiles_sh, c->ntiles_sh, g.experts, moe_gemm_tile_cap(), P, sh_first, c->tokidx, c->side);
      if (!rs) rs = gemm_up(true, c->tiles_sh, c->ntiles_sh, max_tiles_sh, c->side);
      if (!rs) rs = gemm_dn(true, c->tiles_sh, c->ntiles_sh, max_tiles_sh, c->side, nullptr);
    }
    // caller's stream: router, top-k, permutation, the routed experts' GEMMs
    rc = router_batch(c, L, x, P, nullptr, st);
    prof_mark(c, MOE_PROF_ROUTER, st);
    if (!rc)
      rc = moe_routing_run(c->routing, c->ids, c->ws, c->tokidx, c->pw, c->eoff, c->pairids, P, g.topk, g.experts,
                           g.id_stride, st);
    if (!rc) rc = moe_launch_tiles_shared(c->eoff, c->tiles, c->ntiles, g.experts, moe_gemm_tile_cap(), P, -1, c->tokidx, st);
    ee = hipStreamWaitEvent(st, c->ev_x16, 0);
    if (!rc && ee != hipSuccess) rc = (int)ee;
    prof_mark(c, MOE_PROF_ROUTE, st);
    if (!rc && !rs) rc = gemm_up(false, c->tiles, c->ntiles, max_tiles, st);
    prof_mark(c, MOE_PROF_UP, st);
    if (!rc && !rs) rc = gemm_dn(false, c->tiles, c->ntiles, max_tiles, st, nullptr);
    // the side stream is joined on every path out of here (a capture on `st` must not end with it forked)
    ee = hipEventRecord(c->ev_join, c->side);
    if (ee == hipSuccess) ee = hipStreamWaitEvent(st, c->ev_join, 0);
    prof_mark(c, MOE_PROF_DOWN, st);
    if (rc) return rc;
    if (rs) return rs;
    if (ee != hipSuccess) return (int)ee;
    rc = moe_launch_reduce(c->pairs16, true, c->pairids, c->pw, nullptr, L.has_shared ? c->sh_logit : nullptr,
                           L.has_shared ? sh_first : -1, y, P, g.d, g.topk,
                           hs, st, c->hc,
                           v2 ? L.v2_svh_dn : nullptr);
    prof_mark(c, MOE_PROF_REDUCE, st);
    return rc;
  }
  if ((rc = router_batch(c, L, x, P, c->xms, st))) return rc;
  // x -> f16 (HBM-bound) on the side stream while top-k, counting, scan and scatter (small dependent
  // launches that leave the memory system idle) run on the caller's stream
  MOE_HIP(hipEventRecord(c->ev_fork, st));
  MOE_HIP(hipStreamWaitEvent(c->side, c->ev_fork, 0));
  int rc16 = c->x16_ext ? MOE_OK : moe_f32_to_f16(x, c->x16, (uint64_t)P * g.d, xl, c->side);
  if (fused && !rc16) rc16 = moe_launch_zero_f32(y, (uint64_t)P * g.d, c->side);  // after the last read of x
  // the side stream is joined on every path out of here (a capture on `st` must not end with it forked)
  auto join = [&]() -> int {
    hipError_t e = hipEventRecord(c->ev_join, c->side);
    if (e == hipSuccess) e = hipStreamWaitEvent(st, c->ev_join, 0);
    return (int)e;
  };
  const int sh_first = L.has_shared ? P * g.topk : -1;
  rc = rc16;
  prof_mark(c, MOE_PROF_ROUTER, st);
  if (!rc)
    rc = moe_routing_run(c->routing, c->ids, c->ws, c->tokidx, c->pw, c->eoff, c->pairids, P, g.topk, g.experts,
                         g.id_stride, st);
  if (!rc) rc = moe_launch_tiles_shared(c->eoff, c->tiles, c->ntiles, g.experts, moe_gemm_tile_cap(), P, sh_first, c->tokidx, st);
  const int jrc = join();
  if (rc) return rc;
  if (jrc) return jrc;
  prof_mark(c, MOE_PROF_ROUTE, st);
  const int max_tiles = (P * g.topk + 127) / 128 + g.experts + (L.has_shared ? (P + 127) / 128 : 0);
  if ((rc = gemm_up(L.has_shared, c->tiles, c->ntiles, max_tiles, st))) return rc;
  prof_mark(c, MOE_PROF_UP, st);
  if (fused) {
    const moe_comb cmb{y, c->tokidx, c->pw, L.has_shared ? c->sh_logit : nullptr};
    rc = gemm_dn(L.has_shared, c->tiles, c->ntiles, max_tiles, st, &cmb);
    prof_mark(c, MOE_PROF_DOWN, st);
    return rc;
  }
  if ((rc = gemm_dn(L.has_shared, c->tiles, c->ntiles, max_tiles, st, nullptr))) return rc;
  prof_mark(c, MOE_PROF_DOWN, st);
  rc = moe_launch_reduce(c->pairs16, true, c->pairids, c->pw, nullptr, L.has_shared ? c->sh_logit : nullptr,
                         sh_first, y, P, g.d, g.topk, hs, st, c->hc);
  prof_mark(c, MOE_PROF_REDUCE, st);
  return rc;
}

MOE_API int moe_forward(moe_ctx* c, int layer, const float* x, int P, float* y, moe_stream_t st) {
  MoeLayer* L = layer_of(c, layer);
  if (!L || !x || !y || P < 0) return MOE_E_INVALID;
  if (!L->has_router || !(L->has_q4cp || L->has_gguf || L->has_i4r)) return MOE_E_STATE;
  if (P > c->cfg.max_tokens) return MOE_E_STATE;
  if (!moe_aligned(x, 16) || !moe_aligned(y, 16)) return MOE_E_INVALID;
  if (P == 0) return MOE_OK;
  if (P <= c->small_max) {
#ifdef MOE_TIMING_HOOKS
    if (c->skip_stage != 0 && P > c->ran_complete) return MOE_E_STATE;  // the scratch of a call this size is not filled yet
#endif
    const int rs = forward_small(c, *L, x, P, y, moe_s(st));
    if (rs == MOE_OK && c->skip_stage == 0 && P > c->ran_complete) c->ran_complete = P;
    if (rs == MOE_OK) c->last_path = MOE_PATH_SMALL;
    return rs;
  }
  const int rc = forward_batch(c, *L, x, P, y, moe_s(st));
  if (rc == MOE_OK) c->last_path = MOE_PATH_BATCH;
  if (rc != MOE_E_UNSUPPORTED) return rc;
  // formats the grouped GEMM does not cover yet: the in-place path, 32 rows at a time.  Every chunk leaves its
  // router output in the first rows of ids / ws; the walk runs from the last chunk to the first and moves each
  // chunk's rows to their place, so that moe_get_routing sees the whole batch afterwards.
  const size_t stride = (size_t)c->cfg.id_stride;
  for (int t0 = (P - 1) / c->small_max * c->small_max; t0 >= 0; t0 -= c->small_max) {
    const int n = P - t0 < c->small_max ? P - t0 : c->small_max;
    const int r2 = forward_small(c, *L, x + (size_t)t0 * c->cfg.d, n, y + (size_t)t0 * c->cfg.d, moe_s(st));
    if (r2) return r2;
    if (t0 > 0) {
      MOE_HIP(hipMemcpyAsync(c->ids + t0 * stride, c->ids, n * stride * 4, hipMemcpyDeviceToDevice, moe_s(st)));
      MOE_HIP(hipMemcpyAsync(c->ws + t0 * stride, c->ws, n * stride * 4, hipMemcpyDeviceToDevice, moe_s(st)));
    }
  }
  c->last_path = MOE_PATH_WALKED;
  return MOE_OK;
}

MOE_API int moe_last_path(const moe_ctx* c) { return c ? c->last_path : MOE_E_INVALID; }

// GpuModel::moe_b(l, P, try_hcw = true) (src/gpu/parts/40_model.inc:4018,4082-4094): the batch call with the HC
// write-back fused into the combine.  MOE_E_UNSUPPORTED (nothing enqueued) where the reference returns false:
// batches of at most 32 tokens and formats outside the grouped GEMM; the caller then runs moe_forward and its own
// write-back.
MOE_API int moe_forward_hc(moe_ctx* c, int layer, const float* x, int P, const float* w4, uint16_t* R,
                           moe_stream_t st) {
  MoeLayer* L = layer_of(c, layer);
  if (!L || !x || !w4 || !R || P < 0) return MOE_E_INVALID;
  if (!L->has_router || !(L->has_q4cp || L->has_gguf || L->has_i4r)) return MOE_E_STATE;
  if (P > c->cfg.max_tokens) return MOE_E_STATE;
  if (!moe_aligned(x, 16) || !moe_aligned(R, 16)) return MOE_E_INVALID;
  if (P <= c->small_max) return MOE_E_UNSUPPORTED;
  const moe_hc hc{w4, R};
  c->hc = &hc;
  const int rc = forward_batch(c, *L, x, P, nullptr, moe_s(st));
  c->hc = nullptr;
  if (rc == MOE_OK) c->last_path = MOE_PATH_BATCH;
  return rc;
}

// The layout of the f16 activations the grouped GEMM of a layer reads (moe_f32_to_f16's `layout`): 1 for q4cp
// experts, 2 for raw GGUF Q4_K blocks, 0 (natural order) for GGUF layers with other block types; MOE_E_STATE
// without expert weights.
MOE_API int moe_x16_layout(moe_ctx* c, int layer) {
  MoeLayer* L = layer_of(c, layer);
  if (!L) return MOE_E_INVALID;
  if (!(L->has_q4cp || L->has_gguf || L->has_i4r)) return MOE_E_STATE;
  return batch_x16_layout(*L, c->cfg);
}

// moe_forward for a batch whose f16 copy the caller has already made (its HC-read epilogue can write it next to
// the f32 rows, src/gpu/parts/40_model.inc:2556-2565,4817): the library's own conversion pass is left out.
MOE_API int moe_forward_x16(moe_ctx* c, int layer, const float* x, const void* x16, int P, float* y, moe_stream_t st) {
  MoeLayer* L = layer_of(c, layer);
  if (!L || !x || !x16 || !y || P < 0) return MOE_E_INVALID;
  if (!L->has_router || !(L->has_q4cp || L->has_gguf || L->has_i4r)) return MOE_E_STATE;
  if (P > c->cfg.max_tokens) return MOE_E_STATE;
  if (!moe_aligned(x, 16) || !moe_aligned(y, 16) || !moe_aligned(x16, 16)) return MOE_E_INVALID;
  if (P <= c->small_max) return MOE_E_UNSUPPORTED;  // small batches never use an f16 copy
  if (L->has_i4r) return MOE_E_UNSUPPORTED;  // (these layers read the rotated activations, made from the f32 rows)
  c->x16_ext = (const __half*)x16;
  const int rc = forward_batch(c, *L, x, P, y, moe_s(st));
  c->x16_ext = nullptr;
  if (rc == MOE_OK) c->last_path = MOE_PATH_BATCH;
  return rc;
}
