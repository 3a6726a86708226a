// Model-level entry points: a context owns the scratch, layers hold borrowed weight views, and
// moe_forward picks the path by batch size.
// (reference: GpuModel::moe / moe_b / moe_gguf / moe_q4w_run, src/gpu/parts/40_model.inc:1664-1861,4018-4157)
#include <new>
#include <vector>

#include "common.h"
#include "internal.h"

struct MoeLayer {
  bool has_router = false, has_q4cp = false, has_gguf = false, has_shared = false;
  moe_wview router{};
  const float* router_bias = nullptr;
  moe_wview gate_up{}, down{};
  moe_gg_experts gg{};
  moe_wview sh_gate{}, sh_up{}, sh_down{}, sh_sg{};
  int sh_gguf_type = 0;
};

struct moe_ctx {
  moe_config cfg;
  std::vector<MoeLayer> layers;
  // scratch (device), sized for cfg.max_tokens rows
  float* logits = nullptr;    // [T][E]
  int* ids = nullptr;         // [T][id_stride]
  float* ws = nullptr;        // [T][id_stride]
  float* sh_logit = nullptr;  // [T]
  float* hid32 = nullptr;     // [T][k+1][mid] f32 (small-batch path)
  int small_max = 32;         // batches up to this size take the in-place GEMV path
};

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
  void* bufs[] = {c->logits, c->ids, c->ws, c->sh_logit, c->hid32};
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
  if (e == hipSuccess) e = hipMalloc(&c->ids, T * S * 4);
  if (e == hipSuccess) e = hipMalloc(&c->ws, T * S * 4);
  if (e == hipSuccess) e = hipMalloc(&c->sh_logit, T * 4);
  if (e == hipSuccess) e = hipMalloc(&c->hid32, T * (size_t)(cfg->topk + 1) * cfg->mid * 4);
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
  L->gate_up = *gu;
  L->down = *dn;
  L->has_q4cp = true;
  L->has_gguf = false;
  return MOE_OK;
}

MOE_API int moe_set_experts_gguf(moe_ctx* c, int layer, const moe_gg_experts* gg) {
  MoeLayer* L = layer_of(c, layer);
  if (!L || !gg || !gg->gate || !gg->up || !gg->down) return MOE_E_INVALID;
  if (gg->tgu != MOE_GGML_Q4_K || gg->tdn != MOE_GGML_Q4_K) return MOE_E_UNSUPPORTED;
  if (c->cfg.d % 256 || c->cfg.mid % 256) return MOE_E_UNSUPPORTED;
  L->gg = *gg;
  L->has_gguf = true;
  L->has_q4cp = false;
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
  if (sh_gguf_type == 0) {
    if (g->dtype != MOE_DT_Q4CP || u->dtype != MOE_DT_Q4CP || dn->dtype != MOE_DT_Q4CP) return MOE_E_UNSUPPORTED;
  } else if (sh_gguf_type != MOE_GGML_Q4_K) {
    return MOE_E_UNSUPPORTED;
  }
  L->sh_gate = *g;
  L->sh_up = *u;
  L->sh_down = *dn;
  L->sh_sg = *sg;
  L->sh_gguf_type = sh_gguf_type;
  L->has_shared = true;
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
static int forward_small(moe_ctx* c, MoeLayer& L, const float* x, int P, float* y, hipStream_t st) {
  const moe_config& g = c->cfg;
  int rc;
  if ((rc = moe_router_logits_small(&L.router, L.router_bias, L.has_shared ? &L.sh_sg : nullptr, x, P,
                                    c->logits, c->sh_logit, st)))
    return rc;
  if ((rc = moe_router_topk(c->logits, c->ids, c->ws, P, g.experts, g.topk, g.id_stride, st))) return rc;
  if (L.has_q4cp) {
    if (L.has_shared && L.sh_gguf_type != 0) return MOE_E_UNSUPPORTED;
    if ((rc = moe_launch_gemv_gu(&L.gate_up, L.has_shared ? &L.sh_gate : nullptr,
                                 L.has_shared ? &L.sh_up : nullptr, x, (uint64_t)g.d, c->ids, g.id_stride,
                                 g.topk, P, g.mid, c->hid32, st)))
      return rc;
    return moe_launch_gemv_dn(&L.down, L.has_shared ? &L.sh_down : nullptr, c->sh_logit, nullptr, nullptr,
                              c->hid32, c->ids, c->ws, g.id_stride, g.topk, P, g.d, y, (uint64_t)g.d, st);
  }
  if (L.has_shared && L.sh_gguf_type != MOE_GGML_Q4_K) return MOE_E_UNSUPPORTED;
  return moe_launch_q4k_gemv(L.gg.gate, L.gg.up, L.gg.down, L.has_shared ? L.sh_gate.data : nullptr,
                             L.has_shared ? L.sh_up.data : nullptr, L.has_shared ? L.sh_down.data : nullptr,
                             c->sh_logit, x, c->ids, c->ws, c->hid32, y, P, g.d, g.mid, g.topk, g.id_stride, st);
}

MOE_API int moe_forward(moe_ctx* c, int layer, const float* x, int P, float* y, moe_stream_t st) {
  MoeLayer* L = layer_of(c, layer);
  if (!L || !x || !y || P < 0) return MOE_E_INVALID;
  if (!L->has_router || !(L->has_q4cp || L->has_gguf)) return MOE_E_STATE;
  if (P > c->cfg.max_tokens) return MOE_E_STATE;
  if (!moe_aligned(x, 16) || !moe_aligned(y, 16)) return MOE_E_INVALID;
  if (P == 0) return MOE_OK;
  return forward_small(c, *L, x, P, y, moe_s(st));
}
