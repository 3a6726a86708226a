// The 16-entry int8 table of ggml's non-linear 4-bit types IQ4_NL / IQ4_XS (reference: kvalues_iq4nl,
// src/gguf.h:376-379): -127 -104 -83 -65 -49 -35 -22 -10 1 13 25 38 53 69 89 113, looked up in registers.
#pragma once
#include <stdint.h>
#include <hip/hip_runtime.h>

// kv[n] (BIAS = 0: int8 bytes) or kv[n] + 128 (BIAS = 128: unsigned bytes, for the f16 "1024 + u" form) for the four
// 4-bit codes in the low nibbles of q's bytes (shift = 0) or in the high nibbles (shift = 4): entries 0-7 and 8-15 of
// the table through one byte permute each (selector = the code's low three bits), then a third permute takes byte j
// from the first or the second result by the code's bit 3.
template <int BIAS>
__device__ __forceinline__ uint32_t moe_iq4_lookup4(uint32_t q, int shift) {
  static_assert(BIAS == 0 || BIAS == 128, "signed bytes or bytes + 128");
  const uint32_t i7 = (q >> shift) & 0x07070707u;
  const uint32_t flip = BIAS ? 0x80808080u : 0u;  // + 128 on an int8 byte = its top bit flipped
  const uint32_t lo = __builtin_amdgcn_perm(0xF6EADDCFu ^ flip, 0xBFAD9881u ^ flip, i7);  // -127 -104 -83 -65 | -49 -35 -22 -10
  const uint32_t hi = __builtin_amdgcn_perm(0x71594535u ^ flip, 0x26190D01u ^ flip, i7);  // 1 13 25 38 | 53 69 89 113
  const uint32_t sel = ((q >> (shift + 1)) & 0x04040404u) | 0x03020100u;
  return __builtin_amdgcn_perm(hi, lo, sel);
}
