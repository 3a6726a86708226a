// Expert-sorted token permutation: wavefront ballots build, per 64-token wave, one membership
// bit mask per expert in LDS; popcounts of those masks give counts, and prefix sums over
// waves / blocks / experts give every pair its slot.  Stable: inside an expert pairs are in
// ascending token order, exactly what the reference's stable radix sort yields.
// (reference: src/gpu/parts/10_ple_io.inc:784-861)
#include <mutex>
#include <new>

#include "common.h"
#include "internal.h"

struct moe_routing {
  int capacity_pairs, experts, max_blocks;
  int* blockcnt;  // [max_blocks][experts] pairs of block b that go to expert e
  int* blockoff;  // [max_blocks][experts] exclusive prefix over blocks
};

namespace {
constexpr int RT_WAVES = 4, RT_TOK = 64 * RT_WAVES, RT_MAXE = 1024;

// masks[w][e]: bit l set <=> token (block*256 + w*64 + l) routes to expert e.
__device__ __forceinline__ void build_masks(const int* __restrict__ ids, int P, int k, int E,
                                            int id_stride, int nbits,
                                            unsigned long long (*masks)[RT_MAXE]) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < RT_WAVES * E; i += blockDim.x) masks[i / E][i % E] = 0ull;
  __syncthreads();
  const int tok = blockIdx.x * RT_TOK + threadIdx.x;
  for (int s = 0; s < k; s++) {
    const int key = tok < P ? ids[(size_t)tok * id_stride + s] : -1;
    const bool valid = key >= 0 && key < E;
    unsigned long long eq = __ballot(valid);
    for (int b = 0; b < nbits; b++) {
      const bool bit = (key >> b) & 1;
      const unsigned long long bal = __ballot(bit);
      eq &= bit ? bal : ~bal;
    }
    // the lowest lane of every equal-key set records the set; keys differ between leaders
    if (valid && (unsigned)lane == (unsigned)__ffsll((long long)eq) - 1u) masks[w][key] |= eq;
  }
  __syncthreads();
}

__global__ void __launch_bounds__(256) k_route_count(const int* __restrict__ ids, int P, int k, int E,
                                                     int id_stride, int nbits,
                                                     int* __restrict__ blockcnt) {
  __shared__ unsigned long long masks[RT_WAVES][RT_MAXE];
  build_masks(ids, P, k, E, id_stride, nbits, masks);
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    int c = 0;
#pragma unroll
    for (int w = 0; w < RT_WAVES; w++) c += __popcll(masks[w][e]);
    blockcnt[(size_t)blockIdx.x * E + e] = c;
  }
}

// One block, one thread per expert: prefix over blocks, then an LDS prefix scan over experts.
__global__ void __launch_bounds__(RT_MAXE) k_route_scan(const int* __restrict__ blockcnt,
                                                        int* __restrict__ blockoff,
                                                        int* __restrict__ eoff, int nblk, int E) {
  __shared__ int wsum[RT_MAXE / 64];
  const int e = threadIdx.x, lane = e & 63, w = e >> 6;
  int run = 0;
  if (e < E) {
    // eight block counts are requested together: one at a time the loop is a chain of L2 round trips
    int b = 0;
    for (; b + 8 <= nblk; b += 8) {
      int c[8];
#pragma unroll
      for (int i = 0; i < 8; i++) c[i] = blockcnt[(size_t)(b + i) * E + e];
#pragma unroll
      for (int i = 0; i < 8; i++) {
        blockoff[(size_t)(b + i) * E + e] = run;
        run += c[i];
      }
    }
    for (; b < nblk; b++) {
      const int c = blockcnt[(size_t)b * E + e];
      blockoff[(size_t)b * E + e] = run;
      run += c;
    }
  }
  // inclusive scan inside the wave
  int inc = run;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(inc, o, 64);
    if (lane >= o) inc += v;
  }
  if (lane == 63) wsum[w] = inc;
  __syncthreads();
  int base = 0;
  for (int i = 0; i < w; i++) base += wsum[i];
  if (e < E) eoff[e] = base + inc - run;
  if (e == E - 1) eoff[E] = base + inc;
}

__global__ void __launch_bounds__(256) k_route_scatter(const int* __restrict__ ids,
                                                       const float* __restrict__ ws, int P, int k,
                                                       int E, int id_stride, int nbits,
                                                       const int* __restrict__ blockoff,
                                                       const int* __restrict__ eoff,
                                                       int* __restrict__ tokidx, float* __restrict__ pw,
                                                       int* __restrict__ pairids) {
  __shared__ unsigned long long masks[RT_WAVES][RT_MAXE];
  build_masks(ids, P, k, E, id_stride, nbits, masks);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int tok = blockIdx.x * RT_TOK + threadIdx.x;
  if (tok >= P) return;
  const unsigned long long below = lane ? (~0ull >> (64 - lane)) : 0ull;
  // the token's slots four at a time: ids and weights first, then the offsets they index, so that
  // each step of the dependent chain ids -> eoff / blockoff is one round trip for four slots
  for (int s0 = 0; s0 < k; s0 += 4) {
    int key[4], base[4];
    float wv[4];
    bool ok[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int s = s0 + i < k ? s0 + i : k - 1;
      key[i] = ids[(size_t)tok * id_stride + s];
      wv[i] = ws[(size_t)tok * id_stride + s];
      ok[i] = s0 + i < k && key[i] >= 0 && key[i] < E;
      key[i] = ok[i] ? key[i] : 0;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) base[i] = eoff[key[i]] + blockoff[(size_t)blockIdx.x * E + key[i]];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      if (!ok[i]) continue;
      int pos = base[i];
      for (int j = 0; j < w; j++) pos += __popcll(masks[j][key[i]]);
      pos += __popcll(masks[w][key[i]] & below);
      tokidx[pos] = tok;
      pw[pos] = wv[i];
      if (pairids) {
        int rank = 0;
        for (int j = 0; j < k; j++) rank += ids[(size_t)tok * id_stride + j] < key[i];
        pairids[(size_t)tok * k + rank] = pos;
      }
    }
  }
}

// Tiles in expert order: thread e owns expert e, LDS scan of the per-expert tile counts.
__global__ void __launch_bounds__(RT_MAXE) k_tiles(const int* __restrict__ eoff,
                                                   moe_tile* __restrict__ tiles,
                                                   int* __restrict__ total, int E, int cap) {
  __shared__ int wsum[RT_MAXE / 64];
  const int e = threadIdx.x, lane = e & 63, w = e >> 6;
  const int first = e < E ? eoff[e] : 0;
  const int ne = e < E ? eoff[e + 1] - first : 0;
  const int count = (ne + cap - 1) / cap;
  int inc = count;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(inc, o, 64);
    if (lane >= o) inc += v;
  }
  if (lane == 63) wsum[w] = inc;
  __syncthreads();
  int base = 0;
  for (int i = 0; i < w; i++) base += wsum[i];
  const int begin = base + inc - count;
  if (e == RT_MAXE - 1) *total = begin + count;
  for (int j = 0; j < count; j++) {
    moe_tile t;
    t.expert = e;
    t.first = first + j * cap;
    t.count = min(cap, ne - j * cap);
    tiles[begin + j] = t;
  }
}
// Batches of at most 32 tokens: the whole permutation in one block and one launch.  An expert's
// members are a 32-bit token mask in LDS (a token picks an expert at most once), so a pair's slot
// is its expert's offset plus the count of lower tokens in the mask: the same stable order as the
// general kernels.  With `tiles` the tile list (routed experts in runs of `cap`, then the shared
// expert's runs over all tokens, whose tokidx entries are the identity) comes out of the same launch.
__global__ void __launch_bounds__(RT_MAXE) k_route_small(const int* __restrict__ ids, const float* __restrict__ ws,
                                                         int P, int k, int E, int id_stride,
                                                         int* __restrict__ tokidx, float* __restrict__ pw,
                                                         int* __restrict__ eoff, int* __restrict__ pairids,
                                                         moe_tile* __restrict__ tiles, int* __restrict__ total,
                                                         int cap, int sh_first) {
  __shared__ uint32_t mask[RT_MAXE];
  __shared__ int eo[RT_MAXE];
  __shared__ int wsum[RT_MAXE / 64], tsum[RT_MAXE / 64];
  __shared__ int routed_total;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  mask[tid] = 0u;
  __syncthreads();
  const int n = P * k;
  int tok = 0, key = -1;
  float wt = 0.f;
  if (tid < n) {
    tok = tid / k;
    const int s = tid - tok * k;
    key = ids[(size_t)tok * id_stride + s];
    wt = ws[(size_t)tok * id_stride + s];
    if (key < 0 || key >= E) key = -1;
    else atomicOr(&mask[key], 1u << tok);
  }
  __syncthreads();
  const int e = tid;
  const int ne = e < E ? __popc(mask[e]) : 0;
  const int nt = tiles ? (ne + cap - 1) / cap : 0;
  int incE = ne, incT = nt;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(incE, o, 64), u = __shfl_up(incT, o, 64);
    if (lane >= o) {
      incE += v;
      incT += u;
    }
  }
  if (lane == 63) {
    wsum[w] = incE;
    tsum[w] = incT;
  }
  __syncthreads();
  int baseE = 0, baseT = 0;
  for (int i = 0; i < w; i++) {
    baseE += wsum[i];
    baseT += tsum[i];
  }
  const int first = baseE + incE - ne, begin = baseT + incT - nt;
  eo[e] = first;
  if (e < E) eoff[e] = first;
  if (e == E - 1) eoff[E] = first + ne;
  if (e == RT_MAXE - 1) routed_total = begin + nt;
  for (int j = 0; j < nt; j++) {
    moe_tile t;
    t.expert = e;
    t.first = first + j * cap;
    t.count = min(cap, ne - j * cap);
    tiles[begin + j] = t;
  }
  __syncthreads();
  if (key >= 0) {
    const int pos = eo[key] + __popc(mask[key] & ((1u << tok) - 1u));
    tokidx[pos] = tok;
    pw[pos] = wt;
    if (pairids) {
      int rank = 0;
      for (int j = 0; j < k; j++) rank += ids[(size_t)tok * id_stride + j] < key;
      pairids[(size_t)tok * k + rank] = pos;
    }
  }
  if (tiles) {
    const int nsh = sh_first >= 0 ? (P + cap - 1) / cap : 0;
    for (int j = tid; j < nsh; j += RT_MAXE) {
      moe_tile t;
      t.expert = E;
      t.first = sh_first + j * cap;
      t.count = min(cap, P - j * cap);
      tiles[routed_total + j] = t;
    }
    if (tid == 0) {
      total[0] = routed_total + nsh;
      total[1] = routed_total;
    }
    if (sh_first >= 0)
      for (int i = tid; i < P; i += RT_MAXE) tokidx[sh_first + i] = i;
  }
}
}  // namespace

bool moe_route_small_supported(int P, int k, int experts) {
  return P >= 1 && P <= 32 && k >= 1 && P * k <= RT_MAXE && experts >= 1 && experts <= RT_MAXE;
}

// Internal: permutation (and, with tiles != nullptr, the tile list incl. the shared expert's) of a
// batch of at most 32 tokens in one launch.
int moe_launch_route_small(const int* ids, const float* ws, int* tokidx, float* pw, int* eoff, int* pairids,
                           int P, int k, int experts, int id_stride, moe_tile* tiles, int* ntiles, int cap,
                           int sh_first, hipStream_t st) {
  if (!ids || !ws || !tokidx || !pw || !eoff || (tiles && (!ntiles || cap < 1))) return MOE_E_INVALID;
  if (!moe_route_small_supported(P, k, experts) || id_stride < k) return MOE_E_UNSUPPORTED;
  k_route_small<<<1, RT_MAXE, 0, st>>>(ids, ws, P, k, experts, id_stride, tokidx, pw, eoff, pairids, tiles, ntiles,
                                       cap, sh_first);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}

MOE_API int moe_routing_create(int capacity_pairs, int experts, moe_routing** out) {
  if (!out || capacity_pairs < 1 || experts < 1) return MOE_E_INVALID;
  if (experts > RT_MAXE) return MOE_E_UNSUPPORTED;
  moe_routing* r = new (std::nothrow) moe_routing();
  if (!r) return (int)hipErrorOutOfMemory;
  r->capacity_pairs = capacity_pairs;
  r->experts = experts;
  r->max_blocks = (capacity_pairs + RT_TOK - 1) / RT_TOK;  // >= ceil(P/256) for any k >= 1
  r->blockcnt = r->blockoff = nullptr;
  const size_t bytes = (size_t)r->max_blocks * experts * sizeof(int);
  hipError_t e = hipMalloc(&r->blockcnt, bytes);
  if (e == hipSuccess) e = hipMalloc(&r->blockoff, bytes);
  if (e != hipSuccess) {
    if (r->blockcnt) (void)hipFree(r->blockcnt);
    delete r;
    return (int)e;
  }
  *out = r;
  return MOE_OK;
}

MOE_API int moe_routing_destroy(moe_routing* r) {
  if (!r) return MOE_OK;
  hipError_t e1 = hipFree(r->blockcnt), e2 = hipFree(r->blockoff);
  delete r;
  return e1 != hipSuccess ? (int)e1 : (int)e2;
}

// Counting, scan and scatter launches of a batch of more than 32 tokens; blockcnt / blockoff hold
// [ceil(P/256)][experts] ints each.
static int routing_launch(int* blockcnt, int* blockoff, const int* ids, const float* ws, int* tokidx, float* pw,
                          int* eoff, int* pairids, int P, int k, int experts, int id_stride, hipStream_t st) {
  int nbits = 0;
  for (int v = experts - 1; v; v >>= 1) nbits++;
  const int nblk = (P + RT_TOK - 1) / RT_TOK;
  if (nblk > 0) {
    k_route_count<<<nblk, 256, 0, st>>>(ids, P, k, experts, id_stride, nbits, blockcnt);
    MOE_LAUNCH_CHECK();
  }
  k_route_scan<<<1, RT_MAXE, 0, st>>>(blockcnt, blockoff, eoff, nblk, experts);
  MOE_LAUNCH_CHECK();
  if (nblk > 0) {
    k_route_scatter<<<nblk, 256, 0, st>>>(ids, ws, P, k, experts, id_stride, nbits, blockoff, eoff, tokidx, pw,
                                          pairids);
    MOE_LAUNCH_CHECK();
  }
  return MOE_OK;
}

MOE_API int moe_routing_run(moe_routing* r, const int* ids, const float* ws, int* tokidx, float* pw,
                            int* eoff, int* pairids, int P, int k, int experts, int id_stride,
                            moe_stream_t st) {
  if (!r || !eoff || (P > 0 && (!ids || !ws || !tokidx || !pw))) return MOE_E_INVALID;
  if (P < 0 || k < 1 || id_stride < k || experts != r->experts) return MOE_E_INVALID;
  if ((int64_t)P * k > r->capacity_pairs) return MOE_E_STATE;
  if (moe_route_small_supported(P, k, experts))
    return moe_launch_route_small(ids, ws, tokidx, pw, eoff, pairids, P, k, experts, id_stride, nullptr, nullptr, 0,
                                  -1, moe_s(st));
  return routing_launch(r->blockcnt, r->blockoff, ids, ws, tokidx, pw, eoff, pairids, P, k, experts, id_stride,
                        moe_s(st));
}

// ---- the permutation for callers that cannot allocate ----
// The per-block histograms and their prefix sums live in a file-scope device array instead of a
// moe_routing object's allocations: MOE_ROUTING_STATIC_MAX_TOKENS / 256 blocks x 1024 experts x 2 arrays
// of ints = 1 MiB per GPU, held until the process ends.  Every kernel of a call writes the part of the
// array it later reads (nothing has to start at zero), and every call on a GPU uses the same array:
// calls that overlap on one GPU (two streams, two threads) race.
namespace {
constexpr int RT_STATIC_BLOCKS = MOE_ROUTING_STATIC_MAX_TOKENS / RT_TOK;
constexpr int RT_MAX_DEVICES = 64;
}  // namespace
static __device__ __align__(256) int scratch[2 * RT_STATIC_BLOCKS * RT_MAXE];
static int* g_scratch_ptr[RT_MAX_DEVICES];  // device address of `scratch` on each GPU (its name is no address on the host)
static std::mutex g_scratch_mu;

// The address of this GPU's copy of `scratch`, looked up once per device with that device current.
static int scratch_of_current_device(int** out) {
  int dev = -1;
  MOE_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= RT_MAX_DEVICES) return MOE_E_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    int* p = nullptr;
    MOE_HIP(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
    if (!p) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return MOE_OK;
}

MOE_API int moe_routing_run_static(const int* ids, const float* ws, int* tokidx, float* pw, int* eoff, int* pairids,
                                   int P, int k, int experts, int id_stride, moe_stream_t st) {
  if (!eoff || (P > 0 && (!ids || !ws || !tokidx || !pw))) return MOE_E_INVALID;
  if (P < 0 || k < 1 || id_stride < k || experts < 1) return MOE_E_INVALID;
  if (experts > RT_MAXE) return MOE_E_UNSUPPORTED;
  if (P > MOE_ROUTING_STATIC_MAX_TOKENS) return MOE_E_STATE;  // beyond the fixed scratch: use moe_routing_create / run
  // (the look-up comes first, whatever the batch size: any call made outside a capture, P = 0 included, sets the
  //  device up for later calls inside one)
  int* base = nullptr;
  const int rc = scratch_of_current_device(&base);
  if (rc) return rc;
  if (moe_route_small_supported(P, k, experts))
    return moe_launch_route_small(ids, ws, tokidx, pw, eoff, pairids, P, k, experts, id_stride, nullptr, nullptr, 0,
                                  -1, moe_s(st));
  return routing_launch(base, base + (size_t)RT_STATIC_BLOCKS * RT_MAXE, ids, ws, tokidx, pw, eoff, pairids, P, k,
                        experts, id_stride, moe_s(st));
}

MOE_API int moe_tiles(const int* eoff, moe_tile* tiles, int* ntiles, int experts, int cap,
                      moe_stream_t st) {
  if (!eoff || !tiles || !ntiles || cap < 1 || experts < 1) return MOE_E_INVALID;
  if (experts > RT_MAXE) return MOE_E_UNSUPPORTED;
  k_tiles<<<1, RT_MAXE, 0, moe_s(st)>>>(eoff, tiles, ntiles, experts, cap);
  MOE_LAUNCH_CHECK();
  return MOE_OK;
}
