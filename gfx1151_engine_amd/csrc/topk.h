// Softmax + top-k selection shared by the router kernels and the decode gate/up kernel.
// (reference: src/ref.cpp:565-594 — fp64 softmax over f32 logits, k rounds of arg-max with ties to
//  the lower index, weights renormalised over the selected k)
#pragma once
#include "common.h"
#include "internal.h"

__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }
__device__ __forceinline__ uint32_t umin(uint32_t a, uint32_t b) { return a < b ? a : b; }
__device__ __forceinline__ uint32_t wave_umax(uint32_t m) {
  m = umax(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0xB1, 0xf, 0xf, true));
  m = umax(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x4E, 0xf, 0xf, true));
  m = umax(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x141, 0xf, 0xf, true));
  m = umax(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x140, 0xf, 0xf, true));
  return umax(umax((uint32_t)__builtin_amdgcn_readlane((int)m, 0), (uint32_t)__builtin_amdgcn_readlane((int)m, 16)),
              umax((uint32_t)__builtin_amdgcn_readlane((int)m, 32), (uint32_t)__builtin_amdgcn_readlane((int)m, 48)));
}
__device__ __forceinline__ uint32_t wave_umin(uint32_t m) {
  m = umin(m, (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)m, 0xB1, 0xf, 0xf, false));
  m = umin(m, (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)m, 0x4E, 0xf, 0xf, false));
  m = umin(m, (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)m, 0x141, 0xf, 0xf, false));
  m = umin(m, (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)m, 0x140, 0xf, 0xf, false));
  return umin(umin((uint32_t)__builtin_amdgcn_readlane((int)m, 0), (uint32_t)__builtin_amdgcn_readlane((int)m, 16)),
              umin((uint32_t)__builtin_amdgcn_readlane((int)m, 32), (uint32_t)__builtin_amdgcn_readlane((int)m, 48)));
}

// Wave-wide maximum / fp64 sum through DPP row operations and four lane reads: a butterfly of
// __shfl_xor steps goes through the LDS crossbar six times, each a dependent round trip.
__device__ __forceinline__ float wave_fmax_dpp(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, false)));
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, false)));
  const int b = __float_as_int(v);
  return fmaxf(fmaxf(__int_as_float(__builtin_amdgcn_readlane(b, 0)), __int_as_float(__builtin_amdgcn_readlane(b, 16))),
               fmaxf(__int_as_float(__builtin_amdgcn_readlane(b, 32)), __int_as_float(__builtin_amdgcn_readlane(b, 48))));
}
__device__ __forceinline__ double dpp_f64(double v, int ctrl_sel) {
  union { double d; int i[2]; } a, r;
  a.d = v;
  switch (ctrl_sel) {
    case 0: r.i[0] = __builtin_amdgcn_update_dpp(0, a.i[0], 0xB1, 0xf, 0xf, false); r.i[1] = __builtin_amdgcn_update_dpp(0, a.i[1], 0xB1, 0xf, 0xf, false); break;
    case 1: r.i[0] = __builtin_amdgcn_update_dpp(0, a.i[0], 0x4E, 0xf, 0xf, false); r.i[1] = __builtin_amdgcn_update_dpp(0, a.i[1], 0x4E, 0xf, 0xf, false); break;
    case 2: r.i[0] = __builtin_amdgcn_update_dpp(0, a.i[0], 0x141, 0xf, 0xf, false); r.i[1] = __builtin_amdgcn_update_dpp(0, a.i[1], 0x141, 0xf, 0xf, false); break;
    default: r.i[0] = __builtin_amdgcn_update_dpp(0, a.i[0], 0x140, 0xf, 0xf, false); r.i[1] = __builtin_amdgcn_update_dpp(0, a.i[1], 0x140, 0xf, 0xf, false); break;
  }
  return r.d;
}
__device__ __forceinline__ double readlane_f64(double v, int l) {
  union { double d; int i[2]; } a, r;
  a.d = v;
  r.i[0] = __builtin_amdgcn_readlane(a.i[0], l);
  r.i[1] = __builtin_amdgcn_readlane(a.i[1], l);
  return r.d;
}
// (the order of the additions differs from a plain loop: callers use it where every partial sum is exact)
__device__ __forceinline__ double wave_dsum_dpp(double v) {
  v += dpp_f64(v, 0);
  v += dpp_f64(v, 1);
  v += dpp_f64(v, 2);
  v += dpp_f64(v, 3);
  return (readlane_f64(v, 0) + readlane_f64(v, 16)) + (readlane_f64(v, 32) + readlane_f64(v, 48));
}

// k rounds of arg-max by one wave over keys held NPL per lane (key[j] of lane l = expert l + 64 j;
// key = probability bits + 1, probabilities are >= 0 so the bit patterns order like unsigned
// integers; 0 = not a candidate).  Larger probability first, equal probabilities -> lower index.
// Each lane tracks its own best (value, lowest register holding it); a round is a wave-wide
// maximum of the values, then a wave-wide minimum of the expert index over the lanes that hold
// that value, both through DPP row operations and four lane reads.  The selected ids and values
// stay in registers (lane r keeps round r) and are written once at the end.
template <int NPL>
__device__ __forceinline__ void topk_select(uint32_t (&key)[NPL], int lane, int k, int* ids_row,
                                            float* ws_row) {
  double wsum = 0.0;
  float mine = 0.f;
  int myid = 0;
  for (int r = 0; r < k; r++) {
    uint32_t m = key[0];
    int jm = 0;
#pragma unroll
    for (int j = 1; j < NPL; j++) {
      const bool gt = key[j] > m;  // strict: the lowest register (= lowest expert index) wins a tie
      m = gt ? key[j] : m;
      jm = gt ? j : jm;
    }
    const uint32_t wm = wave_umax(m);
    const uint32_t bi = wave_umin(m == wm ? (uint32_t)(64 * jm + lane) : 0xffffffffu);
    const float bv = __uint_as_float(wm - 1u);
    wsum += (double)bv;  // selection order, as the reference's loop over idx[0..k)
    if (lane == r) {
      mine = bv;
      myid = (int)bi;
    }
    if ((int)(bi & 63u) == lane) {
#pragma unroll
      for (int j = 0; j < NPL; j++)
        if (j == (int)(bi >> 6)) key[j] = 0u;
    }
  }
  if (lane < k) {
    ids_row[lane] = myid;
    ws_row[lane] = (float)((double)mine / wsum);
  }
}

// The same with the keys held lane-major (key[j] of lane l = expert NPL*l + j): among equal keys
// the lowest expert is then in the lowest lane, so the second wave-wide reduction becomes a ballot
// and a find-first-one, and the winner's register index is one lane read.
template <int NPL>
__device__ __forceinline__ void topk_select_lm(uint32_t (&key)[NPL], int lane, int k, int* ids_row, float* ws_row) {
  double wsum = 0.0;
  float mine = 0.f;
  int myid = 0;
  for (int r = 0; r < k; r++) {
    uint32_t m = key[0];
    int jm = 0;
#pragma unroll
    for (int j = 1; j < NPL; j++) {
      const bool gt = key[j] > m;  // strict: the lowest register (= lowest expert index) wins a tie
      m = gt ? key[j] : m;
      jm = gt ? j : jm;
    }
    const uint32_t wm = wave_umax(m);
    const int wl = __builtin_ctzll(__ballot(m == wm));          // lowest lane holding the maximum
    const int wj = __builtin_amdgcn_readlane(jm, wl);           // its register
    const float bv = __uint_as_float(wm - 1u);
    wsum += (double)bv;  // selection order, as the reference's loop over idx[0..k)
    if (lane == r) {
      mine = bv;
      myid = NPL * wl + wj;
    }
    const bool me = lane == wl;
#pragma unroll
    for (int j = 0; j < NPL; j++) key[j] = (me && j == wj) ? 0u : key[j];
  }
  if (lane < k) {
    ids_row[lane] = myid;
    ws_row[lane] = (float)((double)mine / wsum);
  }
}

// Lane-major keys again, each lane's keys sorted first (descending, equal keys keep their index
// order: an odd-even transposition sort with strict compares never lets equal keys pass each other).
// A round is then the wave-wide maximum of the lanes' heads and a pop in the winning lane — the
// per-lane scan over NPL registers, a chain of dependent compares and selects, leaves the
// rounds.  The keys' original register indices travel in 4-bit fields of one word.
// runner_up (optional): the expert ranked k + 1, or -1 when there is none, the same in every lane.
template <int NPL>
__device__ __forceinline__ void topk_select_sorted(uint32_t (&key)[NPL], int lane, int k, int* ids_row,
                                                   float* ws_row, int* runner_up = nullptr) {
  static_assert(NPL <= 8, "4-bit index fields in one 32-bit word");
  uint32_t jj[NPL];
#pragma unroll
  for (int j = 0; j < NPL; j++) jj[j] = (uint32_t)j;
#pragma unroll
  for (int pass = 0; pass < NPL; pass++) {
#pragma unroll
    for (int i = pass & 1; i + 1 < NPL; i += 2) {
      const uint32_t ka = key[i], kb = key[i + 1], ia = jj[i], ib = jj[i + 1];  // values, not lvalues:
      const bool sw = kb > ka;                                                   // see the note below
      key[i] = umax(ka, kb); key[i + 1] = umin(ka, kb);
      jj[i] = sw ? ib : ia; jj[i + 1] = sw ? ia : ib;
    }
  }
  // (a conditional between two array elements, `c ? key[j + 1] : key[j]`, is compiled as a load
  //  through a selected address, i.e. a computed index into the register array, which costs a
  //  chain of selects per access: the operands are copied to plain values first)
  uint32_t jw = 0;
#pragma unroll
  for (int j = 0; j < NPL; j++) jw |= jj[j] << (4 * j);
  double wsum = 0.0;
  float mine = 0.f;
  int myid = 0;
  for (int r = 0; r < k; r++) {
    const uint32_t wm = wave_umax(key[0]);
    const int wl = __builtin_ctzll(__ballot(key[0] == wm));        // lowest lane whose head is the maximum
    const int wj = __builtin_amdgcn_readlane((int)jw, wl) & 15;    // the head's register before the sort
    const float bv = __uint_as_float(wm - 1u);
    wsum += (double)bv;  // selection order, as the reference's loop over idx[0..k)
    if (lane == r) {
      mine = bv;
      myid = NPL * wl + wj;
    }
    const bool me = lane == wl;
#pragma unroll
    for (int j = 0; j + 1 < NPL; j++) {
      const uint32_t cur = key[j], nxt = key[j + 1];
      key[j] = me ? nxt : cur;
    }
    const uint32_t last = key[NPL - 1], jsh = jw >> 4;
    key[NPL - 1] = me ? 0u : last;
    jw = me ? jsh : jw;
  }
  if (lane < k) {
    ids_row[lane] = myid;
    ws_row[lane] = (float)((double)mine / wsum);
  }
  if (runner_up) {
    const uint32_t wm = wave_umax(key[0]);
    const int wl = __builtin_ctzll(__ballot(key[0] == wm));
    const int wj = __builtin_amdgcn_readlane((int)jw, wl) & 15;
    *runner_up = wm != 0u ? NPL * wl + wj : -1;
  }
}

// Gap that two neighbours among the k + 1 best logits must exceed for their order to be the reference's: 1e-6 (below
// it two probabilities can round to one float, where the reference orders by index) + twice what a logit can lie
// from the reference's value (tol: the two fp64 summation orders; 2 ulp: the roundings to f32 and the bias addition).
// (ulps = 0 for logits that are the reference's own)
__device__ __forceinline__ float topk_gap_needed(float la, float lb, float tol, float ulps = 4.8e-7f) {
  return 1e-6f + 2.f * tol + ulps * fmaxf(fabsf(la), fabsf(lb));
}
// rows that the ranking by logit handles (block-uniform)
template <int NPL>
__device__ __forceinline__ bool topk_fast_handled(const float* lg, int E, int k) {
  if constexpr (NPL == 8) return E % 4 == 0 && E >= 4 && k < E && k < 63 && ((uintptr_t)lg & 15) == 0;
  return false;
}

// The softmax / top-k of one token by one wave (E <= 64 * NPL): lane l holds experts NPL*l .. NPL*l + NPL - 1
// (lane-major), so that among equal keys the lowest expert sits in the lowest lane and register, and the
// selection can pre-sort each lane's keys.  pbuf: 64 * NPL floats of LDS owned by this wave.
template <int NPL>
__device__ __forceinline__ void topk_wave(const float* __restrict__ lg, int* __restrict__ ids_row,
                                          float* __restrict__ ws_row, int E, int k, float* pbuf) {
  const int lane = threadIdx.x & 63;
  float v[NPL];
  float mxf = -INFINITY;
#pragma unroll
  for (int j = 0; j < NPL; j++) {
    const int e = NPL * lane + j;
    v[j] = e < E ? lg[e] : -INFINITY;
    mxf = fmaxf(mxf, v[j]);
  }
  const double mx = (double)wave_max(mxf);
  // p = (float)exp((double)logit - mx)
  float p[NPL];
  bool exact = true;  // all partial sums representable -> any summation order gives the same fp64
#pragma unroll
  for (int j = 0; j < NPL; j++) {
    const int e = NPL * lane + j;
    p[j] = e < E ? (float)exp((double)v[j] - mx) : 0.f;
    exact = exact && (p[j] == 0.f || p[j] >= 0x1p-20f);
  }
  double se;
  if (__all(exact)) {
    double s = 0.0;
#pragma unroll
    for (int j = 0; j < NPL; j++) s += (double)p[j];
    se = wave_sum(s);
  } else {
    // very wide logit range: replay the reference's index order on one lane
#pragma unroll
    for (int j = 0; j < NPL; j++) pbuf[NPL * lane + j] = p[j];
    __builtin_amdgcn_s_waitcnt(0);
    __builtin_amdgcn_wave_barrier();
    double s = 0.0;
    if (lane == 0)
      for (int e = 0; e < E; e++) s += (double)pbuf[e];
    se = __shfl(s, 0, 64);
  }
  // probabilities are >= 0, so their bit patterns order like unsigned integers; key = bits + 1
  // (0 = not a candidate: past E, or already selected)
  uint32_t key[NPL];
#pragma unroll
  for (int j = 0; j < NPL; j++) {
    const int e = NPL * lane + j;
    key[j] = e < E ? __float_as_uint((float)((double)p[j] / se)) + 1u : 0u;
  }
  if constexpr (NPL <= 8) topk_select_sorted<NPL>(key, lane, k, ids_row, ws_row);
  else topk_select_lm<NPL>(key, lane, k, ids_row, ws_row);
}

// The softmax / top-k of one token by one block of NT threads (E <= 64*NPL): the fp64 exps, the
// costly part, are spread over the block; wave 0 then runs the k selection rounds on the keys in
// LDS.  COH: the logits were written by other blocks of the same launch: read them with
// device-scope loads.  ids_row / ws_row may point to global memory or LDS.
// CHECK: also returns (to every thread; one more barrier) the slack of the k + 1 best logits: the smallest gap between
// neighbours minus what topk_gap_needed asks for at tol = 0 (-inf: a logit range in which probabilities underflow, or
// NaNs).  The selection is certain when the slack exceeds 2 tol -- the verdict of topk_ids_by_logit below on the same
// row, so that blocks which rank by logit and a block which runs this function agree on when to fall back.  Rows
// that ranking does not handle return +inf (taken as they are).
template <int NPL, bool COH, int NT = 256, bool CHECK = false>
__device__ float topk_block(const float* lg, int* ids_row, float* ws_row, int E, int k, float ulps = 4.8e-7f) {
  constexpr int NPT = (64 * NPL + NT - 1) / NT;  // values per thread
  constexpr int NW = NT / 64;
  __shared__ float pb[64 * NPL];
  __shared__ uint32_t keys[64 * NPL];
  __shared__ double red[NW];
  __shared__ float redf[NW];
  __shared__ int redx[NW];
  __shared__ float slack;
  __shared__ float lgs[CHECK ? 64 * NPL : 1];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  __syncthreads();  // LDS of a previous token is no longer read
  float v[NPT];
  float mxf = -INFINITY;
#pragma unroll
  for (int j = 0; j < NPT; j++) {
    const int e = tid + NT * j;
    v[j] = -INFINITY;
    if (e < E) v[j] = COH ? __hip_atomic_load(&lg[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : lg[e];
    if (CHECK && e < 64 * NPL) lgs[e] = v[j];
    mxf = fmaxf(mxf, v[j]);
  }
  // The maximum: every wave reads the whole row itself (NPL values per lane, 16-byte loads; rows
  // past the end re-read the last four values) and needs no exchange with the other waves.
  // Otherwise (unaligned rows, logits written by this launch) it goes through LDS and a barrier.
  const bool wide = !COH && NPL % 4 == 0 && E % 4 == 0 && E >= 4 && ((uintptr_t)lg & 15) == 0;
  float mxa;
  if (wide) {
    float m = -INFINITY;
#pragma unroll
    for (int q = 0; q < NPL / 4; q++) {
      int idx = NPL * lane + 4 * q;
      idx = idx < E ? idx : E - 4;
      const float4 f = *(const float4*)(lg + idx);
      m = fmaxf(fmaxf(m, fmaxf(f.x, f.y)), fmaxf(f.z, f.w));
    }
    mxa = wave_fmax_dpp(m);
  } else {
    mxf = wave_fmax_dpp(mxf);
    if (lane == 0) redf[wv] = mxf;
    __syncthreads();
    mxa = redf[0];
#pragma unroll
    for (int w = 1; w < NW; w++) mxa = fmaxf(mxa, redf[w]);
  }
  const double mx = (double)mxa;
  float p[NPT];
  bool exact = true;
  double sloc = 0.0;
#pragma unroll
  for (int j = 0; j < NPT; j++) {
    const int e = tid + NT * j;
    p[j] = e < E ? (float)exp((double)v[j] - mx) : 0.f;
    exact = exact && (p[j] == 0.f || p[j] >= 0x1p-20f);
    sloc += (double)p[j];
    if (e < 64 * NPL) pb[e] = p[j];
  }
  // wave sums and "every term exact" flags cross the block together, behind one barrier
  sloc = wave_dsum_dpp(sloc);
  const int wex = __all(exact);
  if (lane == 0) {
    red[wv] = sloc;
    redx[wv] = wex;
  }
  __syncthreads();
  bool all_exact = true;
#pragma unroll
  for (int w = 0; w < NW; w++) all_exact = all_exact && redx[w] != 0;
  double se;
  if (all_exact) {  // every partial sum is representable: any order gives the reference's fp64 sum
    se = red[0];
#pragma unroll
    for (int w = 1; w < NW; w++) se += red[w];
  } else {          // very wide logit range: replay the reference's index order on one thread
    __syncthreads();  // red[] has been read
    if (tid == 0) {
      double t = 0.0;
      for (int e = 0; e < E; e++) t += (double)pb[e];
      red[0] = t;
    }
    __syncthreads();
    se = red[0];
  }
#pragma unroll
  for (int j = 0; j < NPT; j++) {
    const int e = tid + NT * j;
    if (e < 64 * NPL) keys[e] = e < E ? __float_as_uint((float)((double)p[j] / se)) + 1u : 0u;
  }
  __syncthreads();
  if (wv == 0) {
    uint32_t key[NPL];
#pragma unroll
    for (int j = 0; j < NPL; j++) key[j] = keys[NPL * lane + j];
    if constexpr (NPL <= 8) {
      int ru = -1;
      topk_select_sorted<NPL>(key, lane, k, ids_row, ws_row, CHECK ? &ru : nullptr);
      if constexpr (CHECK) {
        float sl = INFINITY;
        if (topk_fast_handled<NPL>(lg, E, k)) {
          // lane r < k: the expert of rank r (its own write), lane k: the runner-up; each against the next rank
          const int idr = lane < k ? ids_row[lane] : lane == k ? ru : -1;
          const float la = idr >= 0 ? lgs[idr] : -INFINITY;
          const float lb = __shfl_down(la, 1, 64);
          const float lmax = __shfl(la, 0, 64);
          float mine = INFINITY;
          if (lane < k) {
            const bool fine = idr >= 0 && lb > -INFINITY && lmax - lb < 70.f;  // false for NaNs
            mine = fine ? (la - lb) - topk_gap_needed(la, lb, 0.f, ulps) : -INFINITY;
            if (!(mine == mine)) mine = -INFINITY;
          }
          sl = -wave_fmax_dpp(-mine);
        }
        if (lane == 0) slack = sl;
      }
    } else {
      topk_select_lm<NPL>(key, lane, k, ids_row, ws_row);
      if (CHECK && lane == 0) slack = INFINITY;
    }
  }
  if constexpr (CHECK) {
    __syncthreads();
    return slack;
  }
  return INFINITY;
}

// The k best experts of one token by their LOGITS, without the softmax: wave 0 of the block selects,
// all threads return the verdict (the call contains block barriers).  The probabilities of the
// reference, p = (float)((float)exp(l - max) / sum), are a non-decreasing function of the logit l, so
// the order by logit is the order by probability unless two probabilities round to the same float,
// where the reference order falls back to the expert index.  Two logits more than 1e-6 apart give
// probabilities whose ratio exceeds 1 + 2^-23 after both roundings, i.e. different floats in the same
// order.  The function therefore checks the k + 1 best logits: every gap between neighbours above
// 1e-6 and all of them within 70 of the maximum (probabilities that are normal floats) -> ids_row[0..k) (LDS)
// holds the reference's ranking and 1 is returned; 0: the ranking is not certain (also NaNs); -1: a row this
// function does not handle; in both cases the caller runs the exact selection.
// tol: how far a logit as it stands in lg can lie from the reference's value (the small-batch router sums the
// products in a parallel order: a bound on the difference of the two fp64 sums, from the norms of the operands; the
// roundings to f32 on top are charged here).  Gaps of the k + 1 best above 1e-6 + 2 (tol + 2 ulp) mean that the
// reference's own logits are more than 1e-6 apart and in the same order.
template <int NPL>
__device__ int topk_ids_by_logit(const float* lg, int* ids_row, int E, int k, float tol = 0.f, float ulps = 4.8e-7f) {
  __shared__ int fast_ok;
  const int tid = threadIdx.x, lane = tid & 63;
  bool handled = false;
  handled = topk_fast_handled<NPL>(lg, E, k);
  if (!handled) return -1;  // block-uniform
  if constexpr (NPL == 8) {
    if (tid < 64) {
      // lane-major keys: key[j] of lane l = expert 8 l + j; unsigned keys that order like the floats
      uint32_t key[8], jj[8];
#pragma unroll
      for (int q = 0; q < 2; q++) {
        const int idx = 8 * lane + 4 * q;
        const float4 f = *(const float4*)(lg + (idx < E ? idx : 0));
        const float fv[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const uint32_t u = __float_as_uint(fv[i]);
          const uint32_t o = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
          key[4 * q + i] = idx < E ? o : 0u;
        }
      }
#pragma unroll
      for (int j = 0; j < 8; j++) jj[j] = (uint32_t)j;
#pragma unroll
      for (int pass = 0; pass < 8; pass++) {
#pragma unroll
        for (int i = pass & 1; i + 1 < 8; i += 2) {
          const uint32_t ka = key[i], kb = key[i + 1], ia = jj[i], ib = jj[i + 1];
          const bool sw = kb > ka;
          key[i] = umax(ka, kb); key[i + 1] = umin(ka, kb);
          jj[i] = sw ? ib : ia; jj[i + 1] = sw ? ia : ib;
        }
      }
      uint32_t jw = 0;
#pragma unroll
      for (int j = 0; j < 8; j++) jw |= jj[j] << (4 * j);
      uint32_t mykey = 0;
      int myid = 0;
      for (int r = 0; r <= k; r++) {  // k + 1 rounds: the runner-up is needed for the gap test
        const uint32_t wm = wave_umax(key[0]);
        const int wl = __builtin_ctzll(__ballot(key[0] == wm));
        const int wj = __builtin_amdgcn_readlane((int)jw, wl) & 15;
        if (lane == r) {
          mykey = wm;
          myid = 8 * wl + wj;
        }
        const bool me = lane == wl;
#pragma unroll
        for (int j = 0; j + 1 < 8; j++) {
          const uint32_t cur = key[j], nxt = key[j + 1];
          key[j] = me ? nxt : cur;
        }
        const uint32_t last = key[7], jsh = jw >> 4;
        key[7] = me ? 0u : last;
        jw = me ? jsh : jw;
      }
      // lane r holds rank r: its logit against the next rank's (the subtraction of close floats is exact)
      const uint32_t nk = (uint32_t)__shfl_down((int)mykey, 1, 64);
      const float la = __uint_as_float((mykey & 0x80000000u) ? (mykey ^ 0x80000000u) : ~mykey);
      const float lb = __uint_as_float((nk & 0x80000000u) ? (nk ^ 0x80000000u) : ~nk);
      // The gap argument needs normal floats: a probability keeps 24 significant bits while exp(l - max) / sum
      // stays above the smallest normal float, i.e. while l - max > -70 (exp(-70) / 1024 = 4e-34).  Further down
      // the probabilities go subnormal or to zero, the reference sees ties there and orders them by index, so
      // such rows take the exact selection as well.
      const float lmax = __shfl(la, 0, 64);
      const bool good = lane >= k || (mykey != 0u && nk != 0u && (la - lb) - topk_gap_needed(la, lb, 0.f, ulps) > 2.f * tol && lmax - lb < 70.f);  // false for NaNs; the same arithmetic as topk_block's slack
      const int ok = __all(good);
      if (lane < k) ids_row[lane] = myid;
      if (lane == 0) fast_ok = ok;
    }
    __syncthreads();
    return fast_ok != 0 ? 1 : 0;
  }
  return -1;
}

// Every logit of token `tok` as the reference computes it (src/ref.cpp:70-77: one fp64 chain over the columns in
// order, rounded to f32, + bias), a thread per expert, into out[0..E).  The slow, certain path: a block reads the
// whole router matrix.
template <int NT>
__device__ void exact_logits_block(const moe_rfix& R, int tok, int E, float* out) {
  // Two experts per thread (e and e + NT) as two interleaved chains, 32 columns per step with all of the step's
  // loads requested before the first of its additions: the chains are bound by the latency of their loads, a thread's
  // row being read 16 (f32) or 8 (bf16) bytes at a time out of L2.  d % 32 == 0 (moe_create).
  const float* xr = R.x + (size_t)tok * R.d;
  for (int e0 = threadIdx.x; e0 < E; e0 += 2 * NT) {
    const int e1 = e0 + NT < E ? e0 + NT : e0;  // (no second expert: the first again, dropped below)
    double a0 = 0.0, a1 = 0.0;
    for (int c = 0; c < R.d; c += 32) {
      float w0[32], w1[32];
      if (R.bf16) {
        const uint16_t* r0 = (const uint16_t*)R.W + (size_t)e0 * R.d + c;
        const uint16_t* r1 = (const uint16_t*)R.W + (size_t)e1 * R.d + c;
        uint4 u0[4], u1[4];
#pragma unroll
        for (int i = 0; i < 4; i++) { u0[i] = ((const uint4*)r0)[i]; u1[i] = ((const uint4*)r1)[i]; }
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const uint32_t p0[4] = {u0[i].x, u0[i].y, u0[i].z, u0[i].w}, p1[4] = {u1[i].x, u1[i].y, u1[i].z, u1[i].w};
#pragma unroll
          for (int j = 0; j < 4; j++) {
            w0[8 * i + 2 * j] = __uint_as_float(p0[j] << 16);
            w0[8 * i + 2 * j + 1] = __uint_as_float(p0[j] & 0xffff0000u);
            w1[8 * i + 2 * j] = __uint_as_float(p1[j] << 16);
            w1[8 * i + 2 * j + 1] = __uint_as_float(p1[j] & 0xffff0000u);
          }
        }
      } else {
        const float4* r0 = (const float4*)((const float*)R.W + (size_t)e0 * R.d + c);
        const float4* r1 = (const float4*)((const float*)R.W + (size_t)e1 * R.d + c);
        float4 f0[8], f1[8];
#pragma unroll
        for (int i = 0; i < 8; i++) { f0[i] = r0[i]; f1[i] = r1[i]; }
#pragma unroll
        for (int i = 0; i < 8; i++) {
          w0[4 * i] = f0[i].x; w0[4 * i + 1] = f0[i].y; w0[4 * i + 2] = f0[i].z; w0[4 * i + 3] = f0[i].w;
          w1[4 * i] = f1[i].x; w1[4 * i + 1] = f1[i].y; w1[4 * i + 2] = f1[i].z; w1[4 * i + 3] = f1[i].w;
        }
      }
#pragma unroll
      for (int i = 0; i < 32; i++) {
        const double xv = (double)xr[c + i];
        a0 = fma((double)w0[i], xv, a0);
        a1 = fma((double)w1[i], xv, a1);
      }
    }
    float v0 = (float)a0, v1 = (float)a1;
    if (R.bias) { v0 += R.bias[e0]; v1 += R.bias[e1]; }
    out[e0] = v0;
    if (e1 != e0) out[e1] = v1;
  }
}

// One logit as the reference computes it, by one thread (32 columns per step, the step's loads requested together).
__device__ __forceinline__ float exact_logit(const moe_rfix& R, int tok, int e) {
  const float* xr = R.x + (size_t)tok * R.d;
  double a0 = 0.0;
  for (int c = 0; c < R.d; c += 32) {
    float w0[32];
    if (R.bf16) {
      const uint4* r0 = (const uint4*)((const uint16_t*)R.W + (size_t)e * R.d + c);
      uint4 u0[4];
#pragma unroll
      for (int i = 0; i < 4; i++) u0[i] = r0[i];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t p0[4] = {u0[i].x, u0[i].y, u0[i].z, u0[i].w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
          w0[8 * i + 2 * j] = __uint_as_float(p0[j] << 16);
          w0[8 * i + 2 * j + 1] = __uint_as_float(p0[j] & 0xffff0000u);
        }
      }
    } else {
      const float4* r0 = (const float4*)((const float*)R.W + (size_t)e * R.d + c);
      float4 f0[8];
#pragma unroll
      for (int i = 0; i < 8; i++) f0[i] = r0[i];
#pragma unroll
      for (int i = 0; i < 8; i++) { w0[4 * i] = f0[i].x; w0[4 * i + 1] = f0[i].y; w0[4 * i + 2] = f0[i].z; w0[4 * i + 3] = f0[i].w; }
    }
#pragma unroll
    for (int i = 0; i < 32; i++) a0 = fma((double)w0[i], (double)xr[c + i], a0);
  }
  float v = (float)a0;
  if (R.bias) v += R.bias[e];
  return v;
}

// The selection of one token by one block, certain to be the reference's: ids by logit order where the k + 1 best
// are far enough apart for that (returns true; sel_ws untouched unless want_ws), else the exact softmax / top-k.
// Where the gaps are within what the router launch's summation order can differ from the reference's by, the logits
// that can reach the top k are recomputed in the reference's order first; if their exact values are more than 1e-6
// apart, that settles it, and only a true near tie (where the reference's f32 probabilities decide, and with them
// the exact normaliser) has the block recompute every logit.  All threads of the block call it; sel_ids / sel_ws are
// LDS rows of the caller.  Every block of a launch that calls this for a token reaches the same verdicts: they see
// the same logits and run the same arithmetic.
template <int NPL, int NT>
__device__ bool select_certain(const float* lg, const moe_rfix& R, int tok, int* sel_ids, float* sel_ws, int E, int k,
                               bool want_ws) {
  __shared__ __attribute__((aligned(16))) float lgfix[64 * NPL];
  __shared__ float xsq[NT / 64];
  float tol = 0.f;
  if (!want_ws) {
    tol = R.W && R.tol ? R.tol[tok] : 0.f;  // (blocks that only rank take the bound from the router launch)
    const int r = topk_ids_by_logit<NPL>(lg, sel_ids, E, k, tol);
    if (r == 1) return true;
    if (r != 0 || !R.W) {  // rows the ranking does not handle, or no router operands: the logits as they stand
      topk_block<NPL, false, NT>(lg, sel_ids, sel_ws, E, k);
      return false;
    }
  } else {
    if (!R.W) {
      topk_block<NPL, false, NT>(lg, sel_ids, sel_ws, E, k);
      return false;
    }
    // The exact selection on the logits as they stand, with the slack of the k + 1 best on the side.  Without a
    // bound from the router launch the block takes |x| itself: the loads go out first and are summed after the
    // selection, whose own loads and barriers they then overlap.
    constexpr int PRE = 4;  // 16-byte loads per thread held in registers
    float4 xv[PRE];
    const bool own = R.tol == nullptr;
    const float* xr = R.x + (size_t)tok * R.d;
    if (own) {
#pragma unroll
      for (int i = 0; i < PRE; i++) {
        const int c = 4 * ((int)threadIdx.x + NT * i);
        xv[i] = c < R.d ? *(const float4*)(xr + c) : float4{0.f, 0.f, 0.f, 0.f};
      }
    }
    const float sl = topk_block<NPL, false, NT, true>(lg, sel_ids, sel_ws, E, k);
    if (own) {
      float a = 0.f;
#pragma unroll
      for (int i = 0; i < PRE; i++) a += xv[i].x * xv[i].x + xv[i].y * xv[i].y + xv[i].z * xv[i].z + xv[i].w * xv[i].w;
      for (int c = 4 * ((int)threadIdx.x + NT * PRE); c < R.d; c += 4 * NT) {
        const float4 v = *(const float4*)(xr + c);
        a += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
      }
      a = wave_sum(a);
      if ((threadIdx.x & 63) == 0) xsq[threadIdx.x >> 6] = a;
      __syncthreads();
      float t = 0.f;
#pragma unroll
      for (int w = 0; w < NT / 64; w++) t += xsq[w];
      tol = R.tol_scale * sqrtf(t) * 1.01f;
      if (!(tol >= 0.f)) tol = INFINITY;  // (NaN / overflow: nothing is certain, take the slow path)
    } else {
      tol = R.tol[tok];
    }
    if (sl > 2.f * tol) return false;
  }
  // Not certain (block-uniform from here on).  sel_ids[k - 1] is the k-th best by the logits as they stand; an expert
  // whose logit lies further below it than the margin cannot be among the reference's k best, nor come within 1e-6
  // of them.
  __syncthreads();
  const float lk = lg[sel_ids[k - 1]];
  const float margin = topk_gap_needed(lk, lk, tol) + 4.8e-7f * 70.f;  // (logits up to 70 above the k-th: their ulps)
  bool full = !(lk == lk) || !(margin < INFINITY);
  if (!full) {
    for (int e = threadIdx.x; e < E; e += NT) {
      const float v = lg[e];
      lgfix[e] = v >= lk - margin ? exact_logit(R, tok, e) : v;  // (NaNs stay as they are)
    }
    __syncthreads();
    if (!want_ws) {
      if (topk_ids_by_logit<NPL>(lgfix, sel_ids, E, k, 0.f, 0.f) == 1) return true;
      full = true;
    } else {
      if (topk_block<NPL, false, NT, true>(lgfix, sel_ids, sel_ws, E, k, 0.f) > 0.f) return false;
      full = true;
    }
  }
  exact_logits_block<NT>(R, tok, E, lgfix);
  __syncthreads();
  topk_block<NPL, false, NT>(lgfix, sel_ids, sel_ws, E, k);
  return false;
}
