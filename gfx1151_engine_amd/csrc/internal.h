// Launchers shared between the translation units of libmi355moe (not exported).
#pragma once
#include "common.h"

// f16 range guard of the batch path: per-token mean square of x and the per-class constants
// (routed experts, shared expert); xms == nullptr switches it off (scale 1).
struct moe_hscale {
  const float* xms;
  moe_cmag c_routed, c_shared;
};

// Fused weighted combine of the down launch (f32 results): rows are added into y[tokidx[pair]] with the
// weight pw[pair] (shared expert: sigmoid(sg[token])); y holds zeros when the launch starts.
struct moe_comb {
  float* y;
  const int* tokidx;
  const float* pw;
  const float* sg;
};

// HC write-back fused into the combine: w4 = inject gate logits [P][4], R = bf16 state [P][4][d]
struct moe_hc {
  const float* w4;
  uint16_t* R;
};

// What the small-batch selection needs to make the expert ids certain: the router's operands and the bound tol.
struct moe_rfix {
  const void* W;      // router matrix [E][d], f32 or bf16 (nullptr: no check, the logits are taken as they are)
  const float* bias;  // [E] or nullptr
  const float* x;     // activations [P][d]
  const float* tol;   // [P]: bound on |fp64 sum in the router launch's order - the reference's sequential sum| (any logit
                      // of the token), written by the router launch; nullptr: the selecting block takes the norm of x itself
  float tol_scale;    // the bound = tol_scale * |x_token|_2: 2 (d + 4) 2^-53 * the largest row norm of W, with a margin
  int bf16, d;
};
// the largest row norm of a router matrix (set-up work: one launch and a read-back through `scratch`, a device float)
int moe_router_row_norm_max(const moe_wview* W, float* scratch, float* out_host);
// softmax / top-k of at most 32 tokens, a block per token, with the expert ids made certain (rf may be null)
int moe_launch_router_topk_small(const float* logits, int* ids, float* ws, int P, int E, int k, int id_stride,
                                 const moe_rfix* rf, hipStream_t st);

// hgn v2 layers: the small-batch router launch also leaves the digit planes of rot_in(x, pre) (planes / meta [P][d/32])
struct moe_rot_planes {
  const float* pre;
  uint32_t* planes;
  float2* meta;
};
int moe_router_logits_small(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x,
                            int P, float* logits, float* out_x, uint32_t* planes, float2* meta,
                            bool planes_natural, unsigned* counter, int* ids, float* ws, int k, int id_stride, bool* fused_topk,
                            hipStream_t st, double* kpart, unsigned* ktickets, const moe_rot_planes* rot = nullptr,
                            float* tol_out = nullptr, float tol_scale = 0.f);
// scratch of the column-split router launch (5..32 tokens): fp64 partial tiles of up to 8 splits x 32 tokens
// for at most MOE_ROUTER_KSPLIT_ROWS rows, and one ticket counter (resting at 0) per 16 rows
constexpr int MOE_ROUTER_KSPLIT_ROWS = 1040;
constexpr size_t MOE_ROUTER_KPART_BYTES = (size_t)8 * (MOE_ROUTER_KSPLIT_ROWS / 16) * 512 * sizeof(double);
constexpr size_t MOE_ROUTER_KTICKET_BYTES = (MOE_ROUTER_KSPLIT_ROWS / 16) * sizeof(unsigned);
int moe_launch_gemv_gu(const moe_wview* gu, const moe_wview* sh_gate, const moe_wview* sh_up,
                       const float* x, uint64_t x_stride, const int* ids, int id_stride, int kpt, int P,
                       int mid, float* hid, hipStream_t st);
int moe_launch_gemv_dn(const moe_wview* dn, const moe_wview* sh_down, const float* sh_logit,
                       const float* ey, const float* sg, const float* hid, const int* ids,
                       const float* ws, int id_stride, int kpt, int P, int d, float* out,
                       uint64_t out_stride, hipStream_t st, bool pair_tables = false);
int moe_launch_q4k_gemv(int phase, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                        const uint8_t* sh_gate, const uint8_t* sh_up, const uint8_t* sh_down,
                        const float* sh_logit, const float* x, const int* ids, const float* ws,
                        float* hid, float* out, int P, int d, int mid, int kpt, int id_stride,
                        hipStream_t st);
// hgn v2 rotated experts, gate/up launch with the slot-wise middle in its epilogue (gs = 2, up): svh_gu [2 m], suh_dn [m]
struct moe_rotv {
  const float *svh_gu, *suh_dn;
};
int moe_launch_gemm_q4cp(bool up, const moe_lutw* routed, const moe_lutw* sh, int n_experts,
                         const __half* x, const int* tokidx, const moe_tile* tiles, const int* ntiles,
                         int max_tiles, void* out, int m, int k, bool f16out, bool q4k, moe_hscale hs,
                         hipStream_t st, const moe_comb* comb, const float* sh_cb_up = nullptr, int gs = 0,
                         bool q5k = false, bool nat = false, const int8_t* pexp_routed = nullptr,
                         const int8_t* pexp_sh = nullptr, const moe_rotv* rot = nullptr);
// Scaled dequantisation of the grouped GEMM (affine q4cp codebooks): per expert the power of two P with
// |cb slope| * (largest scale of the expert) * 2^(24+P) in [2^14, 2^15), or MOE_PEXP_NONE where the form does not apply
// (a scale that is not finite, a zero slope, rows whose largest scale lies more than 2^5 below the expert's: their
// weights would fall into the f16 denormals of the scaled units).  moe_q4cp_scale_span fills one (hi, lo) pair of
// exponents per expert for a tensor; moe_pexp_from_span combines the spans of the tensors one launch reads.
constexpr int MOE_PEXP_NONE = -128;
int moe_q4cp_scale_span(const moe_wview* w, int n_experts, int8_t* span_dev, hipStream_t st);
int moe_pexp_from_span(const int8_t* hi_lo_a, const int8_t* hi_lo_b);
// The Q5_K form addresses weights and activations with 32-bit byte offsets: true when a tensor of `rows` rows of k
// columns and an activation buffer of `x_rows` rows of k f16 values both stay below 4 GB (the caller of
// moe_launch_gemm_q4cp(q5k = true) checks it; other layers take the general kernel)
bool moe_gemm_q5k_fits(uint64_t rows, uint64_t x_rows, int k);
int moe_gemm_tile_cap();
int moe_launch_zero_f32(float* p, uint64_t n, hipStream_t st);
int moe_launch_tiles_only_shared(moe_tile* tiles, int* ntiles, int E, int cap, int P, int sh_first, int* tokidx,
                                 hipStream_t st);
int moe_launch_meansq_f16(const void* x16, int P, int d, float* xms, hipStream_t st);
int moe_launch_f16_rows_meansq(const float* x, void* x16, int P, int d, int layout, float* xms, hipStream_t st);
// permutation (+ tile list with tiles != nullptr) of a batch of at most 32 tokens in one launch
bool moe_route_small_supported(int P, int k, int experts);
int moe_launch_route_small(const int* ids, const float* ws, int* tokidx, float* pw, int* eoff, int* pairids,
                           int P, int k, int experts, int id_stride, moe_tile* tiles, int* ntiles, int cap,
                           int sh_first, hipStream_t st);
int moe_launch_tiles_shared(const int* eoff, moe_tile* tiles, int* ntiles, int E, int cap, int P,
                            int sh_first, int* tokidx, hipStream_t st);
int moe_launch_reduce(const void* pairs, bool pairs_f16, const int* pairids, const float* pw,
                      const float* ey, const float* sg, int sh_first, float* out, int P, int D, int K,
                      moe_hscale hs, hipStream_t st, const moe_hc* hc, const float* rot_svh = nullptr);
int moe_router_logits_seq(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x, int P,
                          float* logits, float* out_x, float* out_xms, hipStream_t st);

int moe_router_logits_seq_if(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x, int P,
                             float* logits, float* out_x, float* out_xms, const int* run_if_above, int run_thr,
                             hipStream_t st);
// batch router through candidate selection (router_cand.hip): bit-exact ids, weights within an ulp or two
bool moe_router_cand_supported(const moe_wview* W, const moe_wview* Wx, int P, int k);
size_t moe_router_cand_scratch_bytes(int max_tokens, int experts, int d);
int moe_router_batch_cand(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x, int P,
                          float* logits, float* out_x, float* out_xms, int* ids, float* ws, int k, int id_stride,
                          void* scratch, hipStream_t st, float bias_max);

size_t moe_qvec_plane_bytes(int K);
size_t moe_qvec_meta_bytes(int K);
bool moe_dec_supported(int d, int mid, int nslots);
bool moe_dec_uq_supported(int d);
int moe_launch_qvec(const float* x, uint64_t x_stride, int P, int K, uint32_t* planes, float2* meta,
                    hipStream_t st);
// hgn v2 rotated experts in the gate/up launch: the routed slots read the rotated activations' planes and leave
// their gate | up sums unfused in zraw [P][kpt][2 mid]
struct moe_dec_v2 {
  float* zraw;
  const uint32_t* xplanes_rot;
  const float2* xmeta_rot;
};
bool moe_dec_gu_topk_supported(int n_experts, int kpt);
int moe_launch_dec_gu_topk(const moe_wview* gu, const moe_wview* sh_gate, const moe_wview* sh_up,
                           const uint32_t* xplanes, const float2* xmeta, const float* logits, int n_experts,
                           int* ids, float* ws, int id_stride, int kpt, int P, int d, int mid,
                           uint32_t* hplanes, float2* hmeta, float* hid_f32, hipStream_t st,
                           const moe_dec_v2* v2 = nullptr, const moe_rfix* rf = nullptr);
int moe_launch_dec_gu(const moe_wview* gu, const moe_wview* sh_gate, const moe_wview* sh_up,
                      const uint32_t* xplanes, const float2* xmeta, const int* ids, int id_stride, int kpt,
                      int P, int d, int mid, uint32_t* hplanes, float2* hmeta, float* hid_f32,
                      hipStream_t st, const moe_dec_v2* v2 = nullptr);
int moe_launch_dec_gu_lut(const moe_wview* gu, const moe_wview* sh_gate, const moe_wview* sh_up, const float* x,
                          const float* logits, int n_experts, int* ids, float* ws, int id_stride, int kpt, int P, int d,
                          int mid, float* hid_f32, hipStream_t st, const moe_rfix* rf = nullptr, bool affine = false);
int moe_launch_dec_dn_lut(const moe_wview* dn, const moe_wview* sh_down, const float* sh_logit, const float* hid_f32,
                          const int* ids, const float* ws, int id_stride, int kpt, int P, int d, int mid, float* out,
                          uint64_t out_stride, hipStream_t st, bool affine = false);
int moe_launch_dec_gu_uq(const moe_wview* gu, const moe_wview* sh_gate, const moe_wview* sh_up,
                         const uint32_t* xplanes, const float2* xmeta, const moe_tile* tiles, const int* ntiles,
                         int max_tiles, const int* tokidx, int n_experts, int d, int mid, uint32_t* hplanes,
                         float2* hmeta, hipStream_t st);
int moe_launch_dec_dn_uq(const moe_wview* dn, const moe_wview* sh_down, const uint32_t* hplanes,
                         const float2* hmeta, const moe_tile* tiles, const int* ntiles, int max_tiles,
                         int n_experts, int d, int mid, float* pairs, hipStream_t st);
// the same for raw GGUF Q4_K rows (activation planes in natural order)
bool moe_dec4k_supported(int d, int mid, int nslots);
bool moe_decgg_supported(int tgu, int tdn, int tsh, bool has_shared, int d, int mid, int kpt, int n_experts);
int moe_launch_decgg_gu_topk(int tgu, int tsh, const uint8_t* gate, const uint8_t* up, const uint8_t* sh_gate,
                             const uint8_t* sh_up, const uint32_t* xplanes, const float2* xmeta, const float* logits,
                             int n_experts, int* ids, float* ws, int id_stride, int kpt, int P, int d, int mid,
                             uint32_t* hplanes, float2* hmeta, hipStream_t st, const moe_rfix* rf = nullptr);
int moe_launch_decgg_gu(int tgu, int tsh, const uint8_t* gate, const uint8_t* up, const uint8_t* sh_gate,
                        const uint8_t* sh_up, const uint32_t* xplanes, const float2* xmeta, const int* ids, int n_experts,
                        int id_stride, int kpt, int P, int d, int mid, uint32_t* hplanes, float2* hmeta, hipStream_t st);
int moe_launch_decgg_dn(int tdn, int tsh, const uint8_t* down, const uint8_t* sh_down, const float* sh_logit,
                        const uint32_t* hplanes, const float2* hmeta, const int* ids, const float* ws, int id_stride,
                        int kpt, int P, int d, int mid, float* out, uint64_t out_stride, hipStream_t st);
bool moe_decgg_uq_supported(int d);
int moe_decgg_uq_tile_cap();
int moe_launch_decgg_gu_uq(int tgu, int tsh, const uint8_t* gate, const uint8_t* up, const uint8_t* sh_gate,
                           const uint8_t* sh_up, const uint32_t* xplanes, const float2* xmeta, const moe_tile* tiles,
                           const int* ntiles, int max_tiles, const int* tokidx, int n_experts, int d, int mid,
                           uint32_t* hplanes, float2* hmeta, hipStream_t st);
int moe_launch_decgg_dn_uq(int tdn, int tsh, const uint8_t* down, const uint8_t* sh_down, const uint32_t* hplanes,
                           const float2* hmeta, const moe_tile* tiles, const int* ntiles, int max_tiles, int n_experts,
                           int d, int mid, float* pairs, hipStream_t st);
int moe_launch_dec4k_gu_topk(const uint8_t* gate, const uint8_t* up, const uint8_t* sh_gate, const uint8_t* sh_up,
                             const uint32_t* xplanes, const float2* xmeta, const float* logits, int n_experts,
                             int* ids, float* ws, int id_stride, int kpt, int P, int d, int mid,
                             uint32_t* hplanes, float2* hmeta, hipStream_t st, const moe_rfix* rf = nullptr);
int moe_launch_dec4k_gu(const uint8_t* gate, const uint8_t* up, const uint8_t* sh_gate, const uint8_t* sh_up,
                        const uint32_t* xplanes, const float2* xmeta, const int* ids, int id_stride, int kpt,
                        int P, int d, int mid, uint32_t* hplanes, float2* hmeta, hipStream_t st);
int moe_launch_dec4k_dn(const uint8_t* down, const uint8_t* sh_down, const float* sh_logit,
                        const uint32_t* hplanes, const float2* hmeta, const int* ids, const float* ws,
                        int id_stride, int kpt, int P, int d, int mid, float* out, uint64_t out_stride,
                        hipStream_t st);
int moe_launch_dec_dn(const moe_wview* dn, const moe_wview* sh_down, const float* sh_logit,
                      const uint32_t* hplanes, const float2* hmeta, const int* ids, const float* ws,
                      int id_stride, int kpt, int P, int d, int mid, float* out, uint64_t out_stride,
                      hipStream_t st, float* out_sh = nullptr);
// hgn v2 (hgn_v2.hip)
const float* moe_i4r_codebook();
bool moe_v2_shapes_ok(int d, int mid);
int moe_launch_v2_rot(const float* x, uint64_t xs, int P, int n, const float* pre, const float* post, int mode, void* y,
                      uint64_t ys, const float* add, uint64_t adds, uint32_t* planes, float2* meta, hipStream_t st);
int moe_launch_i4r_mid(const void* z, bool z_f16, uint64_t zs, int nslots, int mid, const float* svh_gu,
                       const float* suh_dn, int mode, void* out, uint64_t os, int k, int row_slots, uint32_t* planes,
                       float2* meta, hipStream_t st, const float* xms = nullptr, moe_cmag C = moe_cmag{0.f, 0.f},
                       const int* tokidx = nullptr);
// general GEMV kernels for any supported mix of ggml block types (gguf_types.hip)
int moe_launch_gemm_gg(bool up, int type, const uint8_t* w, const uint8_t* w_up, int tsh, const uint8_t* sh_w,
                       const uint8_t* sh_w_up, int n_experts, const __half* x16, const int* tokidx,
                       const moe_tile* tiles, const int* ntiles, int max_tiles, __half* out, int m, int k,
                       moe_hscale hs, hipStream_t st, int a_layout = 0);
// shared expert stored densely (bf16 / f32 / q8g64; type codes of dense.h)
bool moe_dense_shared_supported(int type, int d, int mid);
int moe_launch_dense_shared_small(int type, const uint8_t* g, const uint8_t* u, const uint8_t* dn, const float* sh_logit,
                                  const float* x, int P, int d, int mid, float* hid, float* y, hipStream_t st);
int moe_dense_dequant_row(int type, const uint8_t* base, uint64_t nrows, int K, uint64_t r, float* out, hipStream_t st);
bool moe_gg_types_supported(int tgu, int tdn, int d, int mid);
uint64_t moe_gg_row_bytes(int type, uint64_t k);
int moe_launch_ggx_gemv(int phase, int tgu, int tdn, int tsh, const uint8_t* gate, const uint8_t* up,
                        const uint8_t* down, const uint8_t* sh_gate, const uint8_t* sh_up, const uint8_t* sh_down,
                        const float* sh_logit, const float* x, const int* ids, const float* ws, float* hid,
                        float* out, int P, int d, int mid, int kpt, int id_stride, hipStream_t st);
