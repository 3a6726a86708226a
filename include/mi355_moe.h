/*
 * mi355_moe.h — C ABI of libmi355moe.so: the routed-expert MoE layer of gfx1151-engine
 * (router top-k, 4-bit expert GEMV / grouped GEMM, SwiGLU, weighted combine, shared expert)
 * for one AMD Instinct MI355X (gfx950).
 *
 * Every entry point names the reference symbol it stands in for (file:line inside the reference
 * tree).  Conventions kept from the reference:
 *   - the caller owns every buffer; weights are borrowed, read-only device memory in the
 *     engine's on-disk byte layouts (hgn q4cp blobs, GGUF raw blocks);
 *   - every call only enqueues work on the given HIP stream, never synchronises the host, never
 *     allocates (contexts allocate once, at creation) and is safe under HIP graph capture;
 *   - router rows are `id_stride` ints/floats wide, the first k valid (the engine uses 16);
 *   - one host thread drives a context at a time (contexts share scratch between calls).
 * Return value: 0 = ok, < 0 = moe_status (unsupported / invalid arguments: nothing was enqueued),
 * > 0 = a hipError_t from the runtime.  Nothing throws across this boundary.
 */
#ifndef MI355_MOE_H
#define MI355_MOE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef void* moe_stream_t; /* hipStream_t */

enum moe_status {
  MOE_OK = 0,
  MOE_E_UNSUPPORTED = -1, /* shape / type the kernels do not cover (reference: `return false`) */
  MOE_E_INVALID = -2,     /* null pointer, misaligned pointer, inconsistent sizes */
  MOE_E_STATE = -3        /* context not ready (weights missing, capacity exceeded) */
};

/* hgn tensor dtypes (src/hgn.h:2-23) and ggml types (src/gguf.h:42-64) used on this path */
enum { MOE_DT_BF16 = 0, MOE_DT_F32 = 1, MOE_DT_F16 = 2, MOE_DT_Q4CP = 5, MOE_DT_Q8G64 = 7, MOE_DT_Q8G32 = 8,
       /* hgn v2 routed experts (src/gpu/parts/28_kernels_hgn_v2.inc:1-15): data = [rows*cols/2 codes][rows x cols/128
        * fp16 scales], no header, w = (nibble - 8) * scale, stored in the Hadamard-rotated domain */
       MOE_DT_I4R = 23,
       /* hgn v2 dense tensors (28_kernels_hgn_v2.inc:1-15,226-231,442-447): "ht" = 4-bit hashed-trellis codes in
        * 128 x 128 tiles, Hadamard-rotated domain, with f16 planes <name>.suh [cols] / <name>.svh [rows]; q6g64 = 6-bit
        * codes with (fp16 scale, fp16 bias) per 64 columns.  Accepted by moe_v2_dense_to_bf16 and by the file loader
        * (which converts them), not by moe_set_router / moe_set_shared. */
       MOE_DT_HT = 16, MOE_DT_Q6G64 = 24 };
/* Q4_K: every kernel of the path.  Q5_K (gate/up), Q5_1 and Q8_0 (down) — the mix of the reference's GGUF
 * checkpoints (src/gpu/parts/30_host_util.inc:399-405) — and IQ4_NL / IQ4_XS (src/gguf.h:376-407):
 * bit-exact dequantisation, the stateless general GEMV kernels (moe_gg_gemv), and inside moe_forward integer-dot
 * decode kernels and grouped GEMMs for any mix of the six. */
enum { MOE_GGML_Q5_1 = 7, MOE_GGML_Q8_0 = 8, MOE_GGML_Q4_K = 12, MOE_GGML_Q5_K = 13, MOE_GGML_IQ4_NL = 20,
       MOE_GGML_IQ4_XS = 23 };

/* WView (src/gpu/parts/30_host_util.inc:772-780): a weight tensor as it lies in memory.
 * q4cp: data = [64 B codebook][rows*cols/2 codes][rows x scale_stride]. */
typedef struct moe_wview {
  int dtype;
  const uint8_t* data;
  uint64_t rows, cols, scale_stride;
} moe_wview;

/* GgExperts (30_host_util.inc:348-351): GGUF ffn_{gate,up,down}_exps raw blocks, [K,N,E]. */
typedef struct moe_gg_experts {
  const uint8_t *gate, *up, *down;
  int tgu, tdn; /* ggml types */
} moe_gg_experts;

/* MoeTile (src/gpu/parts/10_ple_io.inc:813) */
typedef struct moe_tile {
  int expert, first, count;
} moe_tile;

const char* moe_version(void);
const char* moe_status_string(int status);

/* ---- weights: dequantisation (bit-exact with the reference's CPU formulas) ---- */

/* hgn::Checkpoint::q4cp_row (src/hgn.h:249-261) for rows [row0, row0+nrows) of a q4cp blob:
 * out[r][c] = cb[nibble] * f32(fp16 scale[r][c/32]).  out: f32 [nrows][cols]. */
int moe_q4cp_dequant_rows(const uint8_t* blob, uint64_t rows, uint64_t cols, uint64_t row0,
                          uint64_t nrows, float* out, moe_stream_t st);
/* gguf::dequant_row, Q4_K branch (src/gguf.h:408-441) for nrows raw rows of `cols` elements. */
int moe_q4k_dequant_rows(const uint8_t* raw, uint64_t nrows, uint64_t cols, float* out,
                         moe_stream_t st);
/* gguf::dequant_row (src/gguf.h:339-445) for nrows raw rows of `cols` elements of ggml type
 * MOE_GGML_Q4_K / Q5_K / IQ4_XS (cols % 256 == 0) or Q5_1 / Q8_0 / IQ4_NL (cols % 32 == 0); bit-exact. */
int moe_gg_dequant_rows(int type, const uint8_t* raw, uint64_t nrows, uint64_t cols, float* out,
                        moe_stream_t st);

/* ---- router ---- */

/* Router logits, the reference CPU arithmetic (src/ref.cpp:70-77 via :566): per (token, expert)
 * one fp64 accumulation over c = 0..d-1 rounded to f32; replaces gemv()/gemm() on
 * mlp.gate.weight (src/gpu/parts/40_model.inc:1809,4023).  W: [E][d] f32 or bf16.
 * bias (optional, [E]) is added in f32 afterwards.  mode 0 = automatic (exact sequential order
 * for P > 32, lane-parallel fp64 order for P <= 32), 1 = force the sequential order. */
int moe_router_logits(const moe_wview* W, const float* bias, const float* x, int P, float* logits,
                      int mode, moe_stream_t st);
/* k_router_topk / k_router_topk_w32 (src/gpu/parts/20_kernels_gemv.inc:1433,1496) with the CPU
 * path's arithmetic (src/ref.cpp:575-594): fp64 softmax -> f32 probabilities, k rounds of
 * arg-max (ties -> lowest index), weights renormalised over the selected k. */
int moe_router_topk(const float* logits, int* ids, float* ws, int P, int E, int k, int id_stride,
                    moe_stream_t st);

/* ---- expert-sorted token permutation ---- */

/* GpuMoeRouting (10_ple_io.inc:827-861): init() -> create, run() -> run.  Stable by expert:
 * tokidx[p] token of pair p, pw[p] its router weight, eoff[e]..eoff[e+1] expert e's pairs,
 * pairids[t*k+rank] pair of token t's rank-th expert in ascending expert id (may be NULL). */
typedef struct moe_routing moe_routing;
int moe_routing_create(int capacity_pairs, int experts, moe_routing** out);
int moe_routing_destroy(moe_routing* r);
int moe_routing_run(moe_routing* r, const int* ids, const float* ws, int* tokidx, float* pw,
                    int* eoff, int* pairids, int P, int k, int experts, int id_stride,
                    moe_stream_t st);
/* moe_routing_run for callers that cannot allocate and hold no moe_routing object (code under HIP graph
 * capture, serving loops and harnesses that forbid hipMalloc).  No counterpart in the reference, whose
 * GpuMoeRouting::init allocates.  Same arguments, results and launches as moe_routing_run; the per-block
 * histograms live in a fixed 1 MiB array inside the library's device image (one copy per GPU, kept until the
 * process ends), so nothing is allocated or freed, at the first call or later.  P <= MOE_ROUTING_STATIC_MAX_TOKENS
 * (MOE_E_STATE beyond it), experts <= 1024.  Every call on a GPU uses that GPU's one array: calls that
 * overlap on the same GPU (two streams or two host threads) race; calls on one stream are ordered.
 * The first call on each GPU looks the array's address up (hipGetSymbolAddress, under a mutex: host work, not a
 * stream operation); make that call outside any stream capture -- one with P = 0 is enough -- and every later
 * call, captured or not, only launches kernels. */
enum { MOE_ROUTING_STATIC_MAX_TOKENS = 32768 };
int moe_routing_run_static(const int* ids, const float* ws, int* tokidx, float* pw, int* eoff, int* pairids,
                           int P, int k, int experts, int id_stride, moe_stream_t st);
/* k_moe_tiles (10_ple_io.inc:815): split each expert's run into <= cap pair tiles, expert order.
 * tiles must hold (pairs+cap-1)/cap + experts entries. */
int moe_tiles(const int* eoff, moe_tile* tiles, int* ntiles, int experts, int cap, moe_stream_t st);

/* ---- decode / small-batch path (P*k slots, each token's experts read in place) ---- */

/* k_q4cp_gemv_gg + k_silu_mul_g (20_kernels_gemv.inc:1608,1680) fused: for slot = (tok, s),
 * expert e = ids[tok*id_stride+s]: hid[slot][r] = silu(W_e[r].x_tok) * (W_e[mid+r].x_tok).
 * gu: q4cp view of the fused gate_up tensor [E*2*mid][d].  x: f32 [P][x_stride]. */
int moe_q4cp_gemv_gate_up(const moe_wview* gu, const float* x, uint64_t x_stride, const int* ids,
                          int id_stride, int kpt, int P, int mid, float* hid, moe_stream_t st);
/* k_q4cp_gemv_gd_topk_h16 (20_kernels_gemv.inc:1771): out[tok][r] = sum_s ws[tok][s] *
 * (W_{e_s}[r] . hid[tok*kpt+s]) in slot order, overwriting out (no atomics).  If ey/sg are given,
 * k_axpy_sg (40_model.inc:8897) is folded in: out += sigmoid(sg[tok]) * ey[tok]. */
int moe_q4cp_gemv_down_topk(const moe_wview* dn, const float* hid, const int* ids, const float* ws,
                            int id_stride, int kpt, int P, int d, const float* ey, const float* sg,
                            float* out, uint64_t out_stride, moe_stream_t st);
/* moe_gg_gemv (src/gpu/parts/26_kernels_moe_gguf.inc:893): GGUF raw-block experts, small P.
 * Supported: tgu and tdn each one of Q4_K, Q5_K, IQ4_XS (row length % 256 == 0), Q5_1, Q8_0, IQ4_NL (% 32 == 0);
 * tgu = tdn = Q4_K with d % 256 == 0 and mid % 256 == 0 takes the tuned kernels, any other mix the general ones.
 * MOE_E_UNSUPPORTED for other types, as the reference's wrapper returns false. */
int moe_gg_gemv(int tgu, int tdn, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                const float* x, const int* ids, const float* ws, float* hid, float* out, int P,
                int d, int mid, int kpt, int id_stride, moe_stream_t st);

/* ---- prefill path: grouped GEMM on MFMA over expert-sorted tiles ---- */

/* LutW (src/gpu/parts/27_kernels_moe_lut.inc:75-83): q4cp operand planes of an expert tensor.
 * Expert e's gate rows start at row e*e_rows of (w, sc), its up rows at row e*e_rows + up_off of
 * (w_up, sc_up); down tensors use (w, sc) only. */
typedef struct moe_lutw {
  const uint8_t *w, *w_up, *sc, *sc_up;
  const float* cb;
  int sstride, e_rows, up_off;
} moe_lutw;
enum { MOE_LUT_Q4CP = 100,  /* moelut::kQ4CP (27_kernels_moe_lut.inc:33) */
       MOE_LUT_I4R = 101 }; /* moelut::kI4R (27_kernels_moe_lut.inc:34): one scale per 128 columns, codebook n - 8 */
/* lut_q4cp_view (27_kernels_moe_lut.inc:811) */
int moe_lut_q4cp_view(const uint8_t* data, uint64_t rows, uint64_t cols, uint64_t scale_stride,
                      int e_rows, int up_off, moe_lutw* out);
/* lut_i4r_view (27_kernels_moe_lut.inc:823-834): the planes of an hgn v2 i4r tensor (MOE_DT_I4R layout); the linear
 * codebook is a device array the library owns */
int moe_lut_i4r_view(const uint8_t* data, uint64_t rows, uint64_t cols, int e_rows, int up_off, moe_lutw* out);
/* moe_lut_up_raw (27_kernels_moe_lut.inc:677-685), type MOE_LUT_I4R: guv16[pair][2 m] = gate | up rows of the fused
 * tensor times x16[tokidx[pair]], unfused (hgn v2: the rotation back comes before SwiGLU, moe_i4r_mid), f16 in natural
 * order; x16 in layout 1 (moe_v2_rot writes it so); m % 16 == 0, k % 256 == 0 */
int moe_lut_up_raw(int type, const moe_lutw* p, const void* x16, const int* tokidx, const moe_tile* tiles,
                   const int* ntiles, int max_tiles, void* guv16, int m, int k, moe_stream_t st);
/* k_f32_to_f16_v4 (26_kernels_moe_gguf.inc:389): round-to-nearest-even, n % 8 == 0.
 * layout 0 = natural order; layout 1 = the order the grouped GEMM reads its f16 activations in:
 * inside every group of 8 consecutive elements, [e0,e4,e1,e5,e2,e6,e3,e7] (matches the order the
 * 4-bit unpack produces, so no shuffle is needed on the weight side).  moe_lut_up expects x16 in
 * layout 1 and writes hid16 in layout 1 for moe_lut_down.
 * layout 2 = the order for raw Q4_K weights (moe_gg_up / moe_gg_down), n % 64 == 0: inside every
 * 64 elements, 16-byte chunk w = [4w, 4w+2, 32+4w, 32+4w+2, 4w+1, 4w+3, 32+4w+1, 32+4w+3]. */
int moe_f32_to_f16(const float* x, void* x16, uint64_t n, int layout, moe_stream_t st);
/* moe_lut_up (27_kernels_moe_lut.inc:660): hid16[pair][m] = f16(silu(gate) * up) for every tile
 * (tiles hold <= 128 pairs); x16: f16 [P][k] (layout 1) gathered through tokidx; m % 32 == 0, k % 128 == 0, k >= 256. */
int moe_lut_up(int type, const moe_lutw* p, const void* x16, const int* tokidx,
               const moe_tile* tiles, const int* ntiles, int max_tiles, void* hid16, int m, int k,
               moe_stream_t st);
/* moe_lut_down (27_kernels_moe_lut.inc:765): pairs[pair][m] (unweighted; f32, or f16 if f16 != 0)
 * = W_e[m][k] . hid16[pair] (hid16 in layout 1); m % 32 == 0, k % 128 == 0, k >= 256.
 * type MOE_LUT_I4R: f16 pairs only, k % 256 == 0. */
int moe_lut_down(int type, const moe_lutw* p, const void* hid16, const moe_tile* tiles,
                 const int* ntiles, int max_tiles, void* pairs, int m, int k, int f16,
                 moe_stream_t st);
/* moe_gg_up / moe_gg_down (src/gpu/parts/26_kernels_moe_gguf.inc:456,473): the same grouped GEMMs
 * on raw GGUF blocks read in place.  type: ggml type of the tensors (supported: MOE_GGML_Q4_K).
 * gate / up: ffn_gate_exps / ffn_up_exps [E][m rows][k]; down: ffn_down_exps [E][m rows][k].
 * x16 / hid16 are f16 in layout 2 (see moe_f32_to_f16); moe_gg_up writes hid16 in layout 2.
 * k % 256 == 0; m % 64 == 0 (up), m % 32 == 0 (down); tiles hold <= 128 pairs. */
int moe_gg_up(int type, const uint8_t* gate, const uint8_t* up, const void* x16, const int* tokidx,
              const moe_tile* tiles, const int* ntiles, int max_tiles, void* hid16, int m, int k,
              moe_stream_t st);
int moe_gg_down(int type, const uint8_t* down, const void* hid16, const moe_tile* tiles,
                const int* ntiles, int max_tiles, void* pairs, int m, int k, int f16, moe_stream_t st);
/* k_moe_reduce_pw / k_moe_reduce_pw_sg (src/gpu/parts/24_kernels_moe_lt.inc:82,104):
 * out[t] = sum_s pw[pid_s] * pairs[pid_s] in pairids order (+ sigmoid(sg[t]) * ey[t] if given). */
int moe_reduce_pw_sg(const void* pairs, int pairs_f16, const int* pairids, const float* pw,
                     const float* ey, const float* sg, float* out, int P, int D, int K,
                     moe_stream_t st);
/* k_moe_reduce_pw_sg_hc (src/gpu/parts/24_kernels_moe_lt.inc:126-161): the same combine with the HC write-back
 * folded in - instead of storing the f32 result, the four branches of the bf16 state take it:
 * R[t][b][c] = bf16(f32(R[t][b][c]) + inj_b * sum), inj_b = 2 / (1 + exp(-w4[t][b] / 4)), b = 0..3.
 * w4: f32 [P][4] (inject gate logits), R: bf16 [P][4][D] (16-byte aligned), D % 8 == 0. */
int moe_reduce_pw_sg_hc(const void* pairs, int pairs_f16, const int* pairids, const float* pw,
                        const float* ey, const float* sg, const float* w4, uint16_t* R, int P, int D, int K,
                        moe_stream_t st);

/* ---- model level ---- */

typedef struct moe_config {
  int d, mid, experts, topk;
  int layers;     /* number of layer slots */
  int max_tokens; /* scratch is sized for this many rows (reference: maxbatch_cap) */
  int id_stride;  /* 0 -> 16 */
} moe_config;

typedef struct moe_ctx moe_ctx;
int moe_create(const moe_config* cfg, moe_ctx** out);
/* The configuration the context was created with (no counterpart in the reference: its g_cfg is a global). */
int moe_get_config(const moe_ctx* ctx, moe_config* out);
int moe_destroy(moe_ctx* ctx);
/* weights of one layer; all pointers are device memory owned by the caller.
 * router: mlp.gate.weight [E][d] (f32 / bf16); router_bias optional (synthetic skew).
 * hgn: gate_up [E*2*mid][d] and down [E*d][mid] q4cp views (40_model.inc:1826-1829).
 * gguf: GgExperts (40_model.inc:1823).  Exactly one of hgn / gguf per layer.
 * shared expert: gate_proj/up_proj [mid][d], down_proj [d][mid], shared_expert_gate [1][d]
 * (40_model.inc:1848-1857).  gate_proj / up_proj / down_proj: q4cp (each tensor with its own codebook); or one of
 * the dense dtypes of the reference's generic matvec (src/ref.cpp:68-109) for all three: bf16, f32, q8g64 (dtype 7:
 * per row cols uint8 codes then cols/64 x (fp16 scale, fp16 min)), and q8g32 (dtype 8, the quality overlay's dense
 * tensors: rows*cols int8 codes then rows*cols/32 fp16 scales over the whole tensor, src/hgn.h:18,176-183); or, with
 * sh_gguf_type != 0, raw GGUF rows of that one ggml type.  shared_expert_gate: f32 or bf16.
 * MOE_E_UNSUPPORTED for other matrix dtypes.  A densely stored shared expert of a q4cp layer runs in launches of its
 * own next to the routed experts' kernels. */
int moe_set_router(moe_ctx* ctx, int layer, const moe_wview* gate_w, const float* router_bias);
int moe_set_experts_q4cp(moe_ctx* ctx, int layer, const moe_wview* gate_up, const moe_wview* down);
int moe_set_experts_gguf(moe_ctx* ctx, int layer, const moe_gg_experts* gg);
int moe_set_shared(moe_ctx* ctx, int layer, const moe_wview* gate_proj, const moe_wview* up_proj,
                   const moe_wview* down_proj, const moe_wview* shared_gate, int sh_gguf_type);
/* hgn v2 routed experts of a layer (GpuModel::moe_v2_1 / moe_b_v2, 40_model.inc:1638-1656,4570-4686): gate_up
 * [E*2*mid][d] and down [E*d][mid] as MOE_DT_I4R views, and the four sign-scale planes of the two tensors as f32
 * device arrays (the reference uploads the f16 sidecars .su / .svh / .suh as f32, 30_host_util.inc:818-861):
 * su [d] (input plane of gate_up, "experts.su"), svh_gu [2*mid], suh_dn [mid], svh_dn [d].
 * d % 128 == 0, mid % 128 == 0, 2*mid <= 2048 (as the reference); batches above 32 tokens also need d % 256 == 0 and
 * mid % 256 == 0 (else they are walked through the small-batch path).  The shared expert of such a layer is not
 * rotated: moe_set_shared as usual (q4cp with affine codebooks, or dense).  The first call allocates the scratch
 * these layers need on top of the context's. */
int moe_set_experts_i4r(moe_ctx* ctx, int layer, const moe_wview* gate_up, const moe_wview* down, const float* su,
                        const float* svh_gu, const float* suh_dn, const float* svh_dn);
/* GpuModel::moe (40_model.inc:1806) for P == 1 and GpuModel::moe_b (40_model.inc:4018) for a
 * batch: y[P][d] = routed experts (top-k, renormalised) + sigmoid-gated shared expert.
 * x, y: f32 [P][d]; y is fully overwritten.
 * Everything is enqueued, nothing waits on the host and nothing is allocated.  Batches above 32 tokens also
 * use one stream that the context owns (default priority): it is forked from st and joined back into st by
 * events inside the call, so work queued on st after the call is ordered after all of it, and a stream
 * capture on st takes that stream in and closes it again. */
int moe_forward(moe_ctx* ctx, int layer, const float* x, int P, float* y, moe_stream_t st);
/* GpuModel::moe_b(l, P, try_hcw = true) (40_model.inc:4018,4082-4094): the batch call with the HC write-back fused
 * into the combine (moe_reduce_pw_sg_hc above); no f32 output is written.  Returns MOE_E_UNSUPPORTED, with nothing
 * enqueued, where the reference's call returns false (P <= 32, formats outside the grouped GEMM): the caller then
 * runs moe_forward and its own write-back. */
int moe_forward_hc(moe_ctx* ctx, int layer, const float* x, int P, const float* w4, uint16_t* R, moe_stream_t st);
/* moe_forward for a caller that already holds the batch as f16 in the order the grouped GEMM reads (the reference's
 * callers write a 16-bit copy of x in the epilogue that produces x, src/gpu/parts/40_model.inc:2556-2565; its
 * moe_q4w_run / moe_gguf convert once more, :1762, :1703).  x16: f16 [P][d] as moe_f32_to_f16(x, ., layout) makes it,
 * layout = moe_x16_layout(ctx, layer) (q4cp experts: 1, or 0 = natural order when their codebook is a table rather than
 * a*n + b; GGUF layers: 2 when the launches that read x run Q4_K / Q5_K tensors on the tuned kernel, else 0).  x (f32) is still read by the router.
 * The library's own conversion pass is left out.  P > 32 only (MOE_E_UNSUPPORTED below: the small-batch kernels do
 * not use an f16 copy; call moe_forward there), and a format outside the grouped GEMM returns MOE_E_UNSUPPORTED. */
int moe_x16_layout(moe_ctx* ctx, int layer);
int moe_forward_x16(moe_ctx* ctx, int layer, const float* x, const void* x16, int P, float* y, moe_stream_t st);
/* Switches in the spirit of the reference's QWENOX_* opt-outs (src/gpu/parts/40_model.inc:1959-1996):
 * every fast path is on by default and can be turned off to fall back to the plainer kernel.
 * MOE_OPT_INT_DECODE (default 1): small batches use the integer-dot GEMV kernels (activations as
 * digit planes per 32-group, 16 significant bits relative to the group maximum) instead of the f32 FMA kernels. */
/* MOE_OPT_UNIQUE_MIN_TOKENS (default 24; 0 = off): q4cp batches of at least this many tokens (and at most 32)
 * walk the expert-sorted pair lists, so that an expert shared by several tokens is read once
 * (the reference's _uq decode kernels, src/gpu/parts/26_kernels_moe_gguf.inc:758-877).  One extra launch
 * builds the permutation and the tile list and a reduce launch follows; measured on verify batches with 30 % of the
 * expert picks shared, against the per-token kernels: 163 against 160 us at 20 tokens, 223 against 234 us at 32 (the
 * per-token kernels find shared experts in L2).  The pairs are then combined in ascending expert order, as on the
 * batch path. */
/* MOE_OPT_FUSED_COMBINE (default 0): batches over 32 tokens fold the top-k weighted combine into the epilogue of
 * the down GEMM (the reference keeps pairs + k_moe_reduce_pw_sg, src/gpu/parts/24_kernels_moe_lt.inc:104): a tile's
 * weighted rows are added into y with f32 atomics, y is zeroed on the context's side stream, no pairs buffer is
 * written and no reduce launch follows.  The order of the k+1 additions per element then depends on timing, so
 * results can differ in their last bits from run to run; 0 keeps the ordered two-step form. */
/* MOE_OPT_SHARED_ASIDE (default 1): batches over 32 tokens run the shared expert's two GEMMs (which do not depend
 * on the routing) on the context's side stream from the start of the call, next to the router launch; 0 = the shared
 * expert's tiles ride in the routed experts' launches.  Same arithmetic either way. */
/* MOE_OPT_ROUTER_CANDIDATES (default 1): batches over 32 tokens find each token's experts without the dense fp64
 * pass over all experts: approximate logits on the f16 matrix pipe with a rigorous error bound select the experts
 * that can be among the k best, whose logits are then computed as the reference's sequential fp64 sums
 * (src/ref.cpp:70-77); tokens with near ties or a logit range in which probabilities underflow are redone with the
 * exact arithmetic over all experts.  Expert ids and their order are the reference's bit for bit; the renormalised
 * weights can differ from it in the last bit or two (the softmax normaliser, which cancels in them up to rounding,
 * contains approximate terms for the experts that were not candidates).  0 = dense fp64 logits and exact weights. */
/* MOE_OPT_TIMING_SKIP_STAGE (default 0): NOT in the library's default build, where it returns MOE_E_UNSUPPORTED; only a
 * build with -DMOE_TIMING_HOOKS (the benchmark's timing twin of the library) takes it.  value = 1 + MOE_PROF_* stage:
 * calls with at most 32 tokens leave that stage's launches out (the later stages then work on the scratch of the last
 * complete call and the output is meaningless).  Refused with MOE_E_STATE until a complete call of at least that many
 * tokens has run on the context.  The difference between the times of a loop of calls without and with the skip is
 * that stage's cost inside the pipelined stream, without the dispatch latency that an event pair around a 10 us
 * kernel adds. */
/* MOE_OPT_GU_TOPK_MAX_TOKENS (default 4: the measured crossover on every weight format): batches of at most this many tokens run the softmax / top-k inside the gate/up launch
 * (every block of a routed slot selects its token's experts itself: one launch less on the latency-bound path);
 * larger batches of the integer-dot kernels take the ids from the router's launches, so that the thousands of blocks
 * of such a launch do not each repeat the selection. */
/* MOE_OPT_F32_DECODE_MAX_TOKENS (default 5; 0 .. 32): q4cp layers that do not run on the integer-dot kernels (a codebook
 * that is not a*n + b, or MOE_OPT_INT_DECODE = 0) use f32 kernels in which a lane keeps its group's activations in
 * registers over a block's rows (a look-up per weight for table codebooks, a conversion and an FMA for a*n + b); for
 * batches of more than this many tokens the down projection goes to the plain f32 GEMV kernel instead, whose blocks of
 * 32 rows read a token's hidden rows once (the measured crossover is between 4 and 6 tokens). */
/* MOE_OPT_UNIQUE_GGUF (default 0): 1 = GGUF layers on the integer-dot kernels also take the distinct-expert path for
 * batches of MOE_OPT_UNIQUE_MIN_TOKENS .. 32 tokens (the reference's _uq kernels, 26_kernels_moe_gguf.inc:758-886:
 * every distinct expert's rows are read once per batch).  Off by default: at the benchmark's verify batch (20 tokens,
 * 30 % of the expert picks shared) the per-token kernels measure faster; it pays when most tokens share their experts. */
/* MOE_OPT_V2_FUSED_MIDDLE (default 1): hgn v2 layers, batches over 32 tokens: the routed experts' gate/up launch takes
 * an expert's gate rows and the matching up rows into one block and runs the slot-wise middle (rotation back, SwiGLU,
 * rotation for down_proj) in its epilogue; 0 = the gate | up sums as f16 rows in memory and the middle as a launch of
 * its own (the reference's moe_lut_up_raw + k_i4r_mid, 40_model.inc:4600-4618). */
/* MOE_OPT_PAIR_TABLES (default 1): q4cp layers whose codebook is a table (not a*n + b), batches above
 * MOE_OPT_F32_DECODE_MAX_TOKENS and up to 32 tokens: the f32 kernels look two neighbouring weights up at a time in
 * 256-entry pair tables (one per code byte); 0 = one look-up per weight in the 16-entry table, as at a few tokens. */
enum { MOE_OPT_INT_DECODE = 1, MOE_OPT_UNIQUE_MIN_TOKENS = 2, MOE_OPT_FUSED_COMBINE = 3, MOE_OPT_SHARED_ASIDE = 4,
       MOE_OPT_TIMING_SKIP_STAGE = 5, MOE_OPT_ROUTER_CANDIDATES = 6, MOE_OPT_UNIQUE_GGUF = 7,
       MOE_OPT_GU_TOPK_MAX_TOKENS = 8, MOE_OPT_F32_DECODE_MAX_TOKENS = 9,
       MOE_OPT_V2_FUSED_MIDDLE = 10, MOE_OPT_PAIR_TABLES = 11 };
int moe_set_option(moe_ctx* ctx, int option, int value);
/* Per-stage timing of the last moe_forward, the reference's KP("moe:route|up|down|reduce") tags
 * (src/gpu/parts/07_kprof.inc, 40_model.inc:1749-1782).  While enabled moe_forward records HIP
 * events between its stages; moe_profile_read waits for the last one and fills
 * ms[MOE_PROF_STAGES] (router = logits + top-k; route = permutation + tiles + f16 conversion;
 * up / down = the expert GEMM or GEMV kernels; reduce = weighted combine). */
enum { MOE_PROF_ROUTER = 0, MOE_PROF_ROUTE = 1, MOE_PROF_UP = 2, MOE_PROF_DOWN = 3, MOE_PROF_REDUCE = 4,
       MOE_PROF_STAGES = 5 };
int moe_profile_enable(moe_ctx* ctx, int on);
int moe_profile_read(moe_ctx* ctx, float* ms);
/* Copy the last call's router output (the reference keeps it in d_topids / d_topw,
 * 40_model.inc:1811) into caller buffers [P][id_stride] (device memory; async on st). */
int moe_get_routing(moe_ctx* ctx, int P, int* ids_out, float* ws_out, moe_stream_t st);
/* Which path the last successful moe_forward / moe_forward_hc / moe_forward_x16 call on the context took (no
 * counterpart in the reference, whose callers pick the path themselves: 40_model.inc:1959-1996 moe / moe_b).
 * MOE_PATH_SMALL: the in-place kernels for at most 32 tokens; MOE_PATH_BATCH: the grouped GEMM; MOE_PATH_WALKED: a
 * batch over 32 tokens of a shape or format outside the grouped GEMM, run through the in-place kernels 32 rows at a
 * time -- correct, and several times slower than the grouped GEMM, which is why a caller may want to know. */
enum { MOE_PATH_NONE = 0, MOE_PATH_SMALL = 1, MOE_PATH_BATCH = 2, MOE_PATH_WALKED = 3 };
int moe_last_path(const moe_ctx* ctx);

/* ---- hgn v2 rotated experts: the stages around the projections ---- */
/* rows [row0, row0 + nrows) of an i4r tensor as f32, bit-exact (tools/moe_lut_test.cu:936-948) */
int moe_i4r_dequant_rows(const uint8_t* data, uint64_t rows, uint64_t cols, uint64_t row0, uint64_t nrows, float* out,
                         moe_stream_t st);
/* k_v2_rot (28_kernels_hgn_v2.inc:62-98): y[p][i] = post[i] * H(pre . x[p])[i] / sqrt(128) per block of 128, H the
 * Sylvester Hadamard matrix in natural order; pre / post may be NULL (= 1).  P rows of n values (n % 128 == 0), row
 * strides xs / ys in elements.  out_f16 = 0: f32 rows (in place is fine); 1: f16 rows in layout 1 of moe_f32_to_f16
 * (what moe_lut_up_raw reads). */
int moe_v2_rot(const float* x, uint64_t xs, void* y, uint64_t ys, const float* pre, const float* post, int n, int P,
               int out_f16, moe_stream_t st);
/* v2_deq_bf16 (src/gpu/parts/30_host_util.inc:1019-1031; k_ht_deq_bf16 / k_q6g64_deq_bf16, 28_kernels_hgn_v2.inc:386-440,
 * 604-634): an hgn v2 dense tensor (MOE_DT_HT or MOE_DT_Q6G64) as the bf16 matrix out[rows][cols] the reference's prefill
 * GEMM reads, bit for bit.  ht: rows % 128 == 0, cols % 128 == 0, suh [cols] / svh [rows] = the tensor's f16 planes as
 * f32; q6g64: cols % 64 == 0, planes unused (may be NULL).  data and out 16-byte aligned. */
int moe_v2_dense_to_bf16(int dtype, const uint8_t* data, const float* suh, const float* svh, uint64_t rows,
                         uint64_t cols, uint16_t* out, moe_stream_t st);
/* k_i4r_mid (28_kernels_hgn_v2.inc:105-150): per slot, g | u = svh_gu . H(guv) / sqrt(128), h = silu(g) * u,
 * out = H(suh_dn . h) / sqrt(128).  guv: [nslots][gs] f32 or f16 (2*mid used), out: [nslots][os] f32, or f16 in
 * layout 1 (what moe_lut_down reads).  mid % 128 == 0, 2*mid <= 2048. */
int moe_i4r_mid(const void* guv, int guv_f16, uint64_t gs, void* out, int out_f16, uint64_t os, const float* svh_gu,
                const float* suh_dn, int mid, int nslots, moe_stream_t st);
/* k_v2_reduce_rot (28_kernels_hgn_v2.inc:153-187): moe_reduce_pw_sg with svh . H(sum) / sqrt(128) applied to the
 * weighted sum before the shared expert's rows are added; D % 128 == 0. */
int moe_v2_reduce_rot(const void* pairs, int pairs_f16, const int* pairids, const float* pw, const float* svh,
                      const float* ey, const float* sg, float* out, int P, int D, int K, moe_stream_t st);

/* ---- checkpoint files -> HBM ---- */

/* hgn::Checkpoint (src/hgn.h:48-76,295-363: HGN1 header + 160-byte records) and gguf::File
 * (src/gguf.h:225-314: GGUF v2/v3 header, key-value section, tensor infos, aligned data) for the tensors
 * of this path.  The file is mapped read-only; tensor data pointers are host pointers into the mapping,
 * valid until moe_file_close.  hgn dims are outermost first (cols last); GGUF dims are ggml's ne[]
 * (cols first).  dtype is the hgn dtype or the ggml type.  Host-only calls: no GPU needed. */
enum { MOE_FILE_HGN = 1, MOE_FILE_GGUF = 2 };
typedef struct moe_file moe_file;
typedef struct moe_tensor_info {
  int dtype;
  uint32_t ndims;
  uint64_t dims[4];
  const uint8_t* data;
  uint64_t nbytes;
} moe_tensor_info;
/* A GGUF path of the form <stem>-<5 digits>-of-<5 digits>.gguf opens every shard of that model, whichever shard is
 * named (gguf::File::open, src/gguf.h:133-150): tensors of all shards are indexed, integer metadata of the first
 * shard wins. */
int moe_file_open(const char* path, moe_file** out);
int moe_file_close(moe_file* f);
/* Maps a second .hgn file whose tensors replace those of the same name (hgn::Checkpoint::add_overlay,
 * src/hgn.h:108-121: the "quality overlay" that stores dense tensors, the shared expert among them, in another
 * dtype).  MOE_OK: applied.  MOE_E_STATE: the file was left out as a whole, as the reference leaves it out -- it is
 * already mapped, or one of its tensors would replace an hgn v2 tensor (dtype 16 / 23 / 24).  The overlay stays
 * mapped until moe_file_close. */
int moe_file_add_overlay(moe_file* f, const char* path);
int moe_file_format(const moe_file* f);
int64_t moe_file_tensor_count(const moe_file* f);
/* MOE_E_STATE if the file has no tensor of that name */
int moe_file_find(const moe_file* f, const char* name, moe_tensor_info* out);
/* MOE_FILE_OPT_GGUF_F32_ROUTER (default 0): moe_load_layers registers the F32 tensors ffn_gate_inp and
 * ffn_gate_inp_shexp of a GGUF file rounded to bf16 (nearest even), as the reference does when it maps a GGUF
 * file (src/gguf_map.h:9,66-72,145-157,210-211), so that a layer routes exactly like the engine it drops into;
 * 1 keeps them F32.  No effect on .hgn files (their tensors are registered in the dtype they are stored in). */
enum { MOE_FILE_OPT_GGUF_F32_ROUTER = 1 };
int moe_file_set_option(moe_file* f, int option, int value);
/* d, mid, experts read off the expert tensors of layer `layer`, layers = consecutive layers from there
 * on that carry them; topk only from the standard GGUF
 * key "<arch>.expert_used_count" (a .hgn file does not store it).  Other fields untouched. */
int moe_file_config(const moe_file* f, int layer, moe_config* cfg);
/* Copies the MoE tensors of n_layers file layers (layers.<l>.mlp.{gate,experts.*,shared_expert*} in a .hgn
 * file, src/gpu/parts/40_model.inc:1808-1857; blk.<l>.ffn_{gate_inp,gate_exps,up_exps,down_exps,*_shexp}
 * in a GGUF file, src/gpu/parts/30_host_util.inc:384-412, src/gguf_map.h:210-214) to device memory, bytes
 * unchanged, and registers them as context layers ctx_layer0...  On the reference's APU the experts are
 * read in place from registered host memory (30_host_util.inc:552-573); here they become resident in HBM.
 * The returned object owns the device copies: free it after the context (or after moe_clear_layer).
 * MOE_E_UNSUPPORTED: a tensor type outside this path (the layers registered so far are cleared again). */
typedef struct moe_weights moe_weights;
int moe_load_layers(moe_ctx* ctx, const moe_file* f, int file_layer0, int ctx_layer0, int n_layers,
                    moe_weights** out, moe_stream_t st);
/* The MoE of the MTP draft layer(s) (GpuModel::mtp_moe / mtp_moe_b, src/gpu/parts/40_model.inc:5546,5892): the same
 * computation on the tensors mtp.layers.<i>.mlp.* of a .hgn file, registered as context layer ctx_layer0 + i (create
 * the context with one layer slot more per MTP layer and call moe_forward on that slot).  In a GGUF file the MTP
 * layer is an ordinary block (blk.<n_layers>.*, the sidecar of src/gguf_map.h:3): use moe_load_layers for it; this
 * call does the same there. */
int moe_load_mtp_layers(moe_ctx* ctx, const moe_file* f, int mtp_layer0, int ctx_layer0, int n_layers,
                        moe_weights** out, moe_stream_t st);
uint64_t moe_weights_bytes(const moe_weights* w);
int moe_weights_free(moe_weights* w);
/* Forget the weights registered for a layer (moe_forward on it returns MOE_E_STATE until it is set again). */
int moe_clear_layer(moe_ctx* ctx, int layer);

#ifdef __cplusplus
}
#endif
#endif
