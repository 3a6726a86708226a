/* Plain C caller of libmi355moe.so: loads the MoE layers of a .hgn / GGUF file into HBM and runs one
 * token through layer 0.  Shows the boundary as the engine's C++ host code would use it: device
 * pointers, sizes, an int status; nothing else crosses it.
 *
 *   gcc -std=c99 -D__HIP_PLATFORM_AMD__ -I/opt/rocm/include -Iinclude examples/forward.c \
 *       -Lgfx1151_engine_amd -lmi355moe -L/opt/rocm/lib -lamdhip64 \
 *       -Wl,-rpath,$PWD/gfx1151_engine_amd -Wl,-rpath,/opt/rocm/lib -o forward && ./forward model.hgn 10
 */
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

#include "mi355_moe.h"

#define CK(e)                                                                          \
  do {                                                                                 \
    int rc_ = (e);                                                                     \
    if (rc_) {                                                                         \
      fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, moe_status_string(rc_));      \
      return 1;                                                                        \
    }                                                                                  \
  } while (0)

int main(int argc, char** argv) {
  if (argc < 3) {
    fprintf(stderr, "usage: %s <model.hgn|model.gguf> <topk>\n", argv[0]);
    return 2;
  }
  moe_file* f = NULL;
  CK(moe_file_open(argv[1], &f));
  moe_config cfg = {0};
  CK(moe_file_config(f, 0, &cfg)); /* d, mid, experts, layers (topk only from GGUF metadata) */
  if (cfg.topk <= 0) cfg.topk = atoi(argv[2]);
  cfg.max_tokens = 32;
  cfg.id_stride = 16;
  moe_ctx* ctx = NULL;
  CK(moe_create(&cfg, &ctx));
  moe_weights* w = NULL;
  CK(moe_load_layers(ctx, f, 0, 0, cfg.layers, &w, NULL));
  CK(moe_file_close(f));
  printf("%s: d=%d mid=%d experts=%d topk=%d layers=%d, %.2f GB resident\n", moe_version(), cfg.d, cfg.mid,
         cfg.experts, cfg.topk, cfg.layers, (double)moe_weights_bytes(w) / 1e9);

  float *x = NULL, *y = NULL, *hx = (float*)malloc(sizeof(float) * (size_t)cfg.d);
  for (int i = 0; i < cfg.d; i++) hx[i] = (float)((i * 37) % 101 - 50) / 50.f;
  CK((int)hipMalloc((void**)&x, sizeof(float) * (size_t)cfg.d));
  CK((int)hipMalloc((void**)&y, sizeof(float) * (size_t)cfg.d));
  CK((int)hipMemcpy(x, hx, sizeof(float) * (size_t)cfg.d, hipMemcpyHostToDevice));
  CK(moe_forward(ctx, 0, x, 1, y, NULL)); /* enqueue only, on the default stream */
  CK((int)hipMemcpy(hx, y, sizeof(float) * (size_t)cfg.d, hipMemcpyDeviceToHost));
  printf("y[0..3] = %g %g %g %g\n", hx[0], hx[1], hx[2], hx[3]);

  CK(moe_destroy(ctx));
  CK(moe_weights_free(w));
  hipFree(x);
  hipFree(y);
  free(hx);
  return 0;
}
