// Launchers shared between the translation units of libmi355moe (not exported).
#pragma once
#include "common.h"

int moe_router_logits_small(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x,
                            int P, float* logits, float* out_x, hipStream_t st);
int moe_launch_gemv_gu(const moe_wview* gu, const moe_wview* sh_gate, const moe_wview* sh_up,
                       const float* x, uint64_t x_stride, const int* ids, int id_stride, int kpt, int P,
                       int mid, float* hid, hipStream_t st);
int moe_launch_gemv_dn(const moe_wview* dn, const moe_wview* sh_down, const float* sh_logit,
                       const float* ey, const float* sg, const float* hid, const int* ids,
                       const float* ws, int id_stride, int kpt, int P, int d, float* out,
                       uint64_t out_stride, hipStream_t st);
int moe_launch_q4k_gemv(const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                        const uint8_t* sh_gate, const uint8_t* sh_up, const uint8_t* sh_down,
                        const float* sh_logit, const float* x, const int* ids, const float* ws,
                        float* hid, float* out, int P, int d, int mid, int kpt, int id_stride,
                        hipStream_t st);
int moe_launch_gemm_q4cp(bool up, const moe_lutw* routed, const moe_lutw* sh, int n_experts,
                         const __half* x, const int* tokidx, const moe_tile* tiles, const int* ntiles,
                         int max_tiles, void* out, int m, int k, bool f16out, hipStream_t st);
int moe_launch_tiles_shared(const int* eoff, moe_tile* tiles, int* ntiles, int E, int cap, int P,
                            int sh_first, int* tokidx, hipStream_t st);
int moe_launch_reduce(const void* pairs, bool pairs_f16, const int* pairids, const float* pw,
                      const float* ey, const float* sg, int sh_first, float* out, int P, int D, int K,
                      hipStream_t st);
int moe_router_logits_seq(const moe_wview* W, const float* bias, const moe_wview* Wx, const float* x, int P,
                          float* logits, float* out_x, hipStream_t st);
