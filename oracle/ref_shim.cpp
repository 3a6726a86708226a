// ref_shim.cpp — builds the reference's OWN CPU code (src/ref.cpp, src/hgn.h,
// src/gguf.h, compiled where they lie in the reference tree) into
// oracle/_ref/libmoe_ref.so so the restated oracle can be checked against it.
//
// TEST INFRASTRUCTURE ONLY.  No reference source is copied: the files are
// #included from REF_ROOT at build time (see oracle/Makefile).  The shim only
// feeds the reference's Model::moe synthetic tensors through the reference's
// own Checkpoint::add_view and exposes plain C entry points.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#define main ref_cli_main  // the reference's CLI entry point is not used
#include REF_CPP           // <REF_ROOT>/src/ref.cpp (pulls in hgn.h, rope.h)
#undef main
#include REF_GGUF_H        // <REF_ROOT>/src/gguf.h

namespace {
hgn::Tensor mk(const char* name, uint32_t dtype, uint64_t rows, uint64_t cols,
               const uint8_t* data, uint64_t bytes) {
  hgn::Tensor t;
  t.name = name;
  t.dtype = dtype;
  t.ndims = 2;
  t.dims[0] = rows;
  t.dims[1] = cols;
  t.data = data;
  t.data_size = bytes;
  return t;
}
uint64_t dense_bytes(uint32_t dtype, uint64_t rows, uint64_t cols) {
  if (dtype == 0) return rows * cols * 2;  // bf16
  if (dtype == 5) return 64 + rows * cols / 2 + rows * (((cols / 32 * 2) + 15) & ~15ULL);
  if (dtype == 7) return rows * (cols + cols / 64 * 4);  // q8g64
  if (dtype == 8) return rows * cols + rows * cols / 32 * 2;  // q8g32 planar
  return 0;
}
}  // namespace

extern "C" {

__attribute__((visibility("default"))) float ref_fp16_to_f32(uint16_t h) {
  return hgn::fp16_to_f32(h);
}

// hgn::Checkpoint::q4cp_parse + q4cp_row on a blob of `rows` x `cols`
__attribute__((visibility("default"))) int ref_q4cp_rows(const uint8_t* blob, uint64_t rows,
                                                         uint64_t cols, uint64_t row0,
                                                         uint64_t nrows, float* out) {
  try {
    hgn::Tensor t = mk("w", 5, rows, cols, blob, dense_bytes(5, rows, cols));
    auto q = hgn::Checkpoint::q4cp_parse(t);
    for (uint64_t r = 0; r < nrows; r++) hgn::Checkpoint::q4cp_row(q, row0 + r, out + r * cols);
    return 0;
  } catch (...) {
    return -1;
  }
}

// hgn::Checkpoint::dequant (src/hgn.h:165-207) of a whole tensor of `rows` x `cols` stored as `dtype` (0 bf16, 7 q8g64)
__attribute__((visibility("default"))) int ref_dequant_tensor(uint32_t dtype, uint64_t rows, uint64_t cols,
                                                              const uint8_t* data, float* out) {
  try {
    hgn::Checkpoint ck;
    ck.dequant(mk("w", dtype, rows, cols, data, dense_bytes(dtype, rows, cols)), out);
    return 0;
  } catch (...) {
    return -1;
  }
}

__attribute__((visibility("default"))) void ref_scale_min_k4(int j, const uint8_t* q, uint8_t* d,
                                                             uint8_t* m) {
  gguf::scale_min_k4(j, q, *d, *m);
}

// gguf::dequant_row for type Q4_K (12)
__attribute__((visibility("default"))) int ref_q4k_row(const uint8_t* src, float* y, uint64_t k) {
  try {
    gguf::dequant_row(gguf::Q4_K, src, y, k);
    return 0;
  } catch (...) {
    return -1;
  }
}
// gguf::dequant_row / gguf::row_bytes for any ggml type id
__attribute__((visibility("default"))) int ref_gg_row(uint32_t type, const uint8_t* src, float* y, uint64_t k) {
  try {
    gguf::dequant_row(type, src, y, k);
    return 0;
  } catch (...) {
    return -1;
  }
}
__attribute__((visibility("default"))) uint64_t ref_gg_row_bytes(uint32_t type, uint64_t k) {
  return gguf::row_bytes(type, k);
}
__attribute__((visibility("default"))) uint64_t ref_q4k_row_bytes(uint64_t k) {
  return gguf::row_bytes(gguf::Q4_K, k);
}

// The reference's Model::moe for ONE token on a one-layer synthetic checkpoint.
// router / shared-expert tensors: dtype 0 (bf16), 5 (q4cp) or 7 (q8g64) as the reference's
// matvec supports; routed experts: q4cp blobs [E*2*mid, d] and [E*d, mid].
__attribute__((visibility("default"))) int ref_moe_token(
    int d, int mid, int E, int k, uint32_t router_dtype, const uint8_t* router,
    const uint8_t* gate_up_blob, const uint8_t* down_blob, uint32_t sh_dtype,
    const uint8_t* sh_gate, const uint8_t* sh_up, const uint8_t* sh_down, uint32_t sg_dtype,
    const uint8_t* sh_sg, const float* x, float* y) {
  try {
    g_cfg.d = d;
    g_cfg.moe_mid = mid;
    g_cfg.experts = E;
    g_cfg.topk = k;
    g_cfg.layers = 1;
    hgn::Checkpoint ck;
    // tensors Model's constructor insists on (PLE, unrelated to this path): tiny placeholders
    static uint8_t zeros[256] = {0};
    static uint8_t fp8tab[8] = {0, 0, 0, 0, 0, 0, 0x80, 0x3f};  // 4 codes + f32 scale 1.0
    const char* ple_bf16[] = {"key_proj.weight", "value_proj.weight", "conv1d.weight",
                              "norm_key.weight", "norm_query.weight", "norm_conv.weight"};
    for (const char* n : ple_bf16)
      ck.add_view(mk((std::string("layers.1.ple.") + n).c_str(), 0, 1, 4, zeros, 8));
    ck.add_view(mk("layers.1.ple.ple_embedding.layer_multipliers", 4, 1, 3, zeros, 24));
    ck.add_view(mk("layers.1.ple.ple_embedding.ngram_heads_vocab_sizes", 4, 1, 16, zeros, 128));
    ck.add_view(mk("layers.1.ple.ple_embedding.ngram_heads_offsets", 4, 1, 16, zeros, 128));
    ck.add_view(mk("layers.1.ple.ngram_embedding.weight", 10, 1, 4, fp8tab, 8));
    // the MoE tensors of layer 0
    ck.add_view(mk("layers.0.mlp.gate.weight", router_dtype, E, d, router,
                   dense_bytes(router_dtype, E, d)));
    ck.add_view(mk("layers.0.mlp.experts.gate_up_proj.weight", 5, (uint64_t)E * 2 * mid, d,
                   gate_up_blob, dense_bytes(5, (uint64_t)E * 2 * mid, d)));
    ck.add_view(mk("layers.0.mlp.experts.down_proj.weight", 5, (uint64_t)E * d, mid, down_blob,
                   dense_bytes(5, (uint64_t)E * d, mid)));
    ck.add_view(mk("layers.0.mlp.shared_expert_gate.weight", sg_dtype, 1, d, sh_sg,
                   dense_bytes(sg_dtype, 1, d)));
    ck.add_view(mk("layers.0.mlp.shared_expert.gate_proj.weight", sh_dtype, mid, d, sh_gate,
                   dense_bytes(sh_dtype, mid, d)));
    ck.add_view(mk("layers.0.mlp.shared_expert.up_proj.weight", sh_dtype, mid, d, sh_up,
                   dense_bytes(sh_dtype, mid, d)));
    ck.add_view(mk("layers.0.mlp.shared_expert.down_proj.weight", sh_dtype, d, mid, sh_down,
                   dense_bytes(sh_dtype, d, mid)));
    Model m(ck);
    m.moe(0, x, y);
    return 0;
  } catch (const std::exception& e) {
    fprintf(stderr, "ref_moe_token: %s\n", e.what());
    return -1;
  }
}

// --- the reference's file readers (checks of the .hgn / GGUF writers and of the library's parser) ---
// Looks `name` up through hgn::Checkpoint(path) (src/hgn.h:103-106,294-363).  Returns 0, 1 if the file
// has no such tensor, -1 if the reader throws.  Copies min(nbytes, cap) data bytes to out.
__attribute__((visibility("default"))) int ref_hgn_tensor(const char* path, const char* name, uint32_t* dtype,
                                                          uint32_t* ndims, uint64_t* dims, uint64_t* nbytes,
                                                          uint8_t* out, uint64_t cap) {
  try {
    hgn::Checkpoint ck(path);
    const hgn::Tensor* t = ck.find(name);
    if (!t) return 1;
    *dtype = t->dtype;
    *ndims = t->ndims;
    for (int k = 0; k < 4; k++) dims[k] = t->dims[k];
    *nbytes = t->data_size;
    if (out && cap) memcpy(out, t->data, t->data_size < cap ? t->data_size : cap);
    return 0;
  } catch (const std::exception& e) {
    fprintf(stderr, "ref_hgn_tensor: %s\n", e.what());
    return -1;
  }
}

// Same through gguf::File(path) (src/gguf.h:119-160,225-314); dims are ne[].
__attribute__((visibility("default"))) int ref_gguf_tensor(const char* path, const char* name, uint32_t* dtype,
                                                           uint32_t* ndims, uint64_t* dims, uint64_t* nbytes,
                                                           uint8_t* out, uint64_t cap) {
  try {
    gguf::File f(path);
    const gguf::Tensor* t = f.find(name);
    if (!t) return 1;
    *dtype = t->type;
    *ndims = t->nd;
    for (int k = 0; k < 4; k++) dims[k] = t->ne[k];
    *nbytes = t->nbytes;
    if (out && cap) memcpy(out, t->data, t->nbytes < cap ? t->nbytes : cap);
    return 0;
  } catch (const std::exception& e) {
    fprintf(stderr, "ref_gguf_tensor: %s\n", e.what());
    return -1;
  }
}

__attribute__((visibility("default"))) int64_t ref_gguf_kv_i(const char* path, const char* key, int64_t def) {
  try {
    gguf::File f(path);
    return f.kv_i(key, def);
  } catch (const std::exception& e) {
    fprintf(stderr, "ref_gguf_kv_i: %s\n", e.what());
    return def;
  }
}
}
