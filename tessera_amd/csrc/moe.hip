// C ABI: MoE routing metadata, dispatch / combine, grouped GEMM and the fused
// SwiGLU expert block.
//
// Routing follows distributed.moe.route_tokens + the slot sort of
// nn.functional.moe_layer, expressed directly in the int32 transport ABI
// (token_of_slot, expert_of_slot, combine_weights, group_sizes, group_offsets):
//
//   topk_kernel    one wavefront per token: f32 max-subtracted softmax over the
//                  experts, k rounds of (max value, lowest index) selection,
//                  optional renormalisation of the k weights.
//   count_kernel   per-chunk histogram of the selected experts.
//   scan_kernel    per-expert exclusive scan over chunks (= each chunk's first
//                  rank inside every expert, in token-major order), capacity
//                  clamp, group sizes and offsets.
//   place_kernel   every kept slot lands at offsets[e] + (its token-major rank
//                  inside expert e): a stable sort by expert without sorting.
// A slot is kept iff its rank inside its expert is below the capacity, which is
// the reference's first-come rule (earlier tokens win, slot-minor inside a token).
#include <algorithm>
#include <mutex>
#include "../../include/tessera_gfx950.h"
#include "gemm16_launch.h"
#include "host_util.h"

// Routing temporaries of the entry point that allocates nothing: device memory that is
// part of the library image, one copy per GPU, held until the process ends.  Host code
// reaches it only through the address hipGetSymbolAddress returns for the current device.
constexpr size_t kRouteScratchBytes = size_t(4) << 20;
static __device__ __align__(256) unsigned char scratch[kRouteScratchBytes];

namespace tsr950 {
namespace {

constexpr int kSlotsPerChunk = 512;   // slots handled by one wavefront in count/place
constexpr int kMaxExperts = 1024;

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Selection key of a score: an unsigned integer ordered like the float, with every NaN
// below every number (numpy's stable descending sort leaves NaNs last) and 0 kept free as
// the "already taken" marker.  A row of NaN probabilities (a NaN or +inf logit, or a row of
// -inf, turns the whole softmax into NaN, in numpy as here) is then a row of equal keys and
// takes experts 0..k-1: every selected id stays inside [0, E).
__device__ __forceinline__ uint32_t select_key(float v) {
  if (v != v) return 1u;
  const uint32_t u = __float_as_uint(v + 0.f);     // -0 and +0 are one key, as they compare equal
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Router variants.  kRouterSoftmaxAll: distributed.moe.route_tokens — softmax over all
// experts, top-k of the probabilities, weights = those probabilities (renormalised over
// the k when asked).  kRouterSoftmaxSelected / kRouterUniform: models.moe_routing.route_top_k
// — top-k of the logits themselves, weights = softmax over the k selected logits, or 1/k.
constexpr int kRouterSoftmaxAll = 0;
constexpr int kRouterSoftmaxSelected = 1;
constexpr int kRouterUniform = 2;

// One wavefront per token.  Lane l owns experts l, l+64, ... (EPL of them).
template <int EPL>
__global__ __launch_bounds__(256) void topk_kernel(const float* scores, int T, int E, int k, int normalize, int router,
                                                   int32_t* expert_ids, float* weights) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  const float* row = scores + (long)t * E;
  float pr[EPL];                 // the values the selection ranks: probabilities or logits
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int e = lane + 64 * i;
    pr[i] = e < E ? row[e] : -INFINITY;
  }
  if (router == kRouterSoftmaxAll) {
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < EPL; ++i) mx = fmaxf(mx, pr[i]);
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const int e = lane + 64 * i;
      pr[i] = e < E ? expf(pr[i] - mx) : 0.f;
      sum += pr[i];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int i = 0; i < EPL; ++i) pr[i] = __fdiv_rn(pr[i], sum);
  }
  uint32_t key[EPL];
#pragma unroll
  for (int i = 0; i < EPL; ++i) key[i] = lane + 64 * i < E ? select_key(pr[i]) : 0u;
  float wsum = 0.f;
  float my_w = 0.f;       // lane j keeps the j-th selected value
  int my_e = -1;
  for (int j = 0; j < k; ++j) {
    // best (key desc, index asc) among this lane's experts, then across lanes
    uint32_t bk = 0u;
    int be = 0x7fffffff;
    float bv = 0.f;
#pragma unroll
    for (int i = 0; i < EPL; ++i)
      if (key[i] > bk) { bk = key[i]; be = lane + 64 * i; bv = pr[i]; }   // ascending e inside a lane: first max wins
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint32_t ok = __shfl_xor(bk, o, 64);
      const int oe = __shfl_xor(be, o, 64);
      const float ov = __shfl_xor(bv, o, 64);
      if (ok > bk || (ok == bk && oe < be)) { bk = ok; be = oe; bv = ov; }
    }
#pragma unroll
    for (int i = 0; i < EPL; ++i)
      if (lane + 64 * i == be) key[i] = 0u;        // remove the winner
    if (lane == (j & 63)) { my_w = bv; my_e = be; }
    wsum += bv;
    if ((j & 63) == 63 || j == k - 1) {
      // flush up to 64 selections (k <= 64 in practice; the loop form keeps it general)
      const int base = j - (j & 63);
      float w_out = my_w;
      if (router != kRouterSoftmaxAll) {
        // (the launcher admits these routers for k <= 64 only: one flush holds the whole row)
        const bool mine = lane < k;
        const float top = wave_max(mine ? my_w : -INFINITY);
        const float ex = mine ? expf(my_w - top) : 0.f;
        const float tot = wave_sum(ex);
        w_out = router == kRouterUniform ? __fdiv_rn(1.0f, (float)k) : __fdiv_rn(ex, tot);
      }
      if (lane <= (j & 63)) {
        expert_ids[(long)t * k + base + lane] = my_e;
        weights[(long)t * k + base + lane] = w_out;
      }
    }
  }
  if (router == kRouterSoftmaxAll && normalize && k > 1) {
    const float d = wsum > 0.f ? wsum : 1.f;
    for (int j = lane; j < k; j += 64) weights[(long)t * k + j] = __fdiv_rn(weights[(long)t * k + j], d);
  }
}

__global__ __launch_bounds__(64) void count_kernel(const int32_t* expert_ids, int S, int E, int32_t* chunk_counts) {
  __shared__ int hist[kMaxExperts];
  for (int e = threadIdx.x; e < E; e += 64) hist[e] = 0;
  __syncthreads();
  const int base = blockIdx.x * kSlotsPerChunk;
  for (int i = threadIdx.x; i < kSlotsPerChunk; i += 64) {
    const int s = base + i;
    if (s < S) {
      const int e = expert_ids[s];
      if ((unsigned)e < (unsigned)E) atomicAdd(&hist[e], 1);
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 64) chunk_counts[(long)blockIdx.x * E + e] = hist[e];
}

// One workgroup.  chunk_counts[c][e] becomes the rank of chunk c's first slot in
// expert e; group sizes (capacity clamped) and offsets follow.
__global__ __launch_bounds__(256) void scan_kernel(int32_t* chunk_counts, int chunks, int E, int capacity,
                                                   int32_t* group_sizes, int32_t* group_offsets,
                                                   int32_t* num_slots) {
  __shared__ int sz[kMaxExperts];
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    int run = 0;
    for (int c0 = 0; c0 < chunks; c0 += 16) {          // 16 independent loads per round trip
      int v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = c0 + u < chunks ? chunk_counts[(long)(c0 + u) * E + e] : 0;
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        if (c0 + u < chunks) chunk_counts[(long)(c0 + u) * E + e] = run;
        run += v[u];
      }
    }
    sz[e] = (capacity > 0 && run > capacity) ? capacity : run;
    group_sizes[e] = sz[e];
  }
  __syncthreads();
  // offsets: the first wave scans the sizes from LDS, a run of consecutive experts per
  // lane (one thread summing them from global memory, a store between every two loads,
  // took E dependent memory round trips)
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    const int per = (E + 63) / 64;
    const int lo = min(lane * per, E), hi = min(lo + per, E);
    int sum = 0;
    for (int e = lo; e < hi; ++e) sum += sz[e];
    int incl = sum;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int u = __shfl_up(incl, d, 64);
      if (lane >= d) incl += u;
    }
    int run = incl - sum;
    for (int e = lo; e < hi; ++e) {
      group_offsets[e] = run;
      run += sz[e];
    }
    if (lane == 63) {
      group_offsets[E] = incl;
      if (num_slots) *num_slots = incl;
    }
  }
}

__global__ __launch_bounds__(64) void place_kernel(const int32_t* expert_ids, const float* weights, int S, int E,
                                                   int k, int capacity, const int32_t* chunk_base,
                                                   const int32_t* group_offsets, int32_t* token_of_slot,
                                                   int32_t* expert_of_slot, float* combine_weights,
                                                   int32_t* sort_perm, int32_t* inverse_perm, uint8_t* kept_mask) {
  __shared__ int cursor[kMaxExperts];
  const int lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) cursor[e] = chunk_base[(long)blockIdx.x * E + e];
  __syncthreads();
  const int base = blockIdx.x * kSlotsPerChunk;
  for (int i0 = 0; i0 < kSlotsPerChunk; i0 += 64) {
    const int s = base + i0 + lane;
    int e = s < S ? expert_ids[s] : -1;
    const bool valid = (unsigned)e < (unsigned)E;     // an id outside [0, E) is dropped, never an index
    if (!valid) e = -1;
    // Rank inside the expert in slot order.  `same` = the lanes that hold this lane's
    // expert, built from one ballot per bit of the expert index (all lanes at once, no
    // loop over the experts present); lower lanes are earlier slots.
    unsigned long long same = __ballot(valid);
    for (int bit = 0; (1 << bit) < E; ++bit) {
      const unsigned long long set = __ballot(valid && ((e >> bit) & 1));
      same &= ((e >> bit) & 1) ? set : ~set;
    }
    int rank = 0;
    if (valid) rank = cursor[e] + __popcll(same & ((1ull << lane) - 1ull));
    // (the workgroup is one wave: its LDS operations execute in program order, so the
    // update below comes after every lane's read above and before the next round's)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    // the last lane of every expert present advances that expert's cursor
    if (valid && (same >> lane) == 1ull) cursor[e] += __popcll(same);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const bool kept = valid && (capacity <= 0 || rank < capacity);
    int pos = -1;
    if (kept) {
      pos = group_offsets[e] + rank;
      if (token_of_slot) token_of_slot[pos] = s / k;
      if (expert_of_slot) expert_of_slot[pos] = e;
      if (combine_weights) combine_weights[pos] = weights[s];
      if (sort_perm) sort_perm[pos] = s;
    }
    // the packing plan in the token-major view: where a slot went (-1 = dropped)
    if (s < S) {
      if (inverse_perm) inverse_perm[s] = pos;
      if (kept_mask) kept_mask[s] = kept ? 1 : 0;
    }
  }
}

// Bytes of temporaries one routing call needs: the token-major expert ids and weights
// (S = T * k each) and the per-chunk histograms.
size_t route_workspace_bytes(int S, int E) {
  const size_t slot_bytes = ((size_t)S * 4 + 255) & ~(size_t)255;
  return 2 * slot_bytes + (size_t)ceil_div(S, kSlotsPerChunk) * E * 4;
}

bool bad_route(const float* scores, int T, int E, int k, const int32_t* token_of_slot, const int32_t* expert_of_slot,
               const float* combine_weights, const int32_t* group_sizes, const int32_t* group_offsets) {
  if (T <= 0 || E <= 0 || k <= 0 || k > E || E > kMaxExperts || !scores || !token_of_slot || !expert_of_slot ||
      !combine_weights || !group_sizes || !group_offsets)
    return true;
  return (long)T * k > 0x7fffffffL;      // int32 device ABI
}

// Extra outputs of the packing plan in the token-major view (stdlib.moe.plan_dispatch,
// models.moe_routing.plan_packing); each may be null.
struct PlanOutputs {
  int32_t* expert_ids = nullptr;     // (T, k) selected experts, rank order
  float* weights = nullptr;          // (T, k) route weights, rank order
  uint8_t* kept_mask = nullptr;      // (T, k) 1 = kept, 0 = dropped over capacity
  int32_t* sort_perm = nullptr;      // [S] kept token-major slot ids, expert-sorted
  int32_t* inverse_perm = nullptr;   // [T k] position of a slot in the packed order, -1 = dropped
};

// The routing kernels on stream `s`, their temporaries in `ws` (device memory of at
// least route_workspace_bytes(T * k, E) bytes; every byte a kernel reads is written by an
// earlier kernel of the same call, so `ws` needs no clearing).  `scores` null: the
// selection is given (given_ids / given_weights, (T, k)) and only the plan is built.
int route_launch(const float* scores, int T, int E, int k, int normalize, int capacity, int router,
                 int32_t* token_of_slot, int32_t* expert_of_slot, float* combine_weights, int32_t* group_sizes,
                 int32_t* group_offsets, int32_t* num_slots, char* ws, hipStream_t s,
                 const PlanOutputs& plan = PlanOutputs{}, const int32_t* given_ids = nullptr,
                 const float* given_weights = nullptr) {
  const int S = T * k;
  const int chunks = ceil_div(S, kSlotsPerChunk);
  const size_t slot_bytes = ((size_t)S * 4 + 255) & ~(size_t)255;
  // the token-major selection goes straight to the caller's arrays when it wants them
  int32_t* ids = plan.expert_ids ? plan.expert_ids : reinterpret_cast<int32_t*>(ws);
  float* w = plan.weights ? plan.weights : reinterpret_cast<float*>(ws + slot_bytes);
  int32_t* counts = reinterpret_cast<int32_t*>(ws + 2 * slot_bytes);
  if (scores) {
    const dim3 tgrid(ceil_div(T, 4));
    const int epl = ceil_div(E, 64);
    if (epl <= 1) hipLaunchKernelGGL((topk_kernel<1>), tgrid, dim3(256), 0, s, scores, T, E, k, normalize, router, ids, w);
    else if (epl <= 2) hipLaunchKernelGGL((topk_kernel<2>), tgrid, dim3(256), 0, s, scores, T, E, k, normalize, router, ids, w);
    else if (epl <= 4) hipLaunchKernelGGL((topk_kernel<4>), tgrid, dim3(256), 0, s, scores, T, E, k, normalize, router, ids, w);
    else hipLaunchKernelGGL((topk_kernel<16>), tgrid, dim3(256), 0, s, scores, T, E, k, normalize, router, ids, w);
  } else {
    ids = const_cast<int32_t*>(given_ids);
    w = const_cast<float*>(given_weights);
  }
  hipLaunchKernelGGL(count_kernel, dim3(chunks), dim3(64), 0, s, ids, S, E, counts);
  hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(256), 0, s, counts, chunks, E, capacity, group_sizes, group_offsets,
                     num_slots);
  hipLaunchKernelGGL(place_kernel, dim3(chunks), dim3(64), 0, s, ids, w, S, E, k, capacity, counts, group_offsets,
                     token_of_slot, expert_of_slot, combine_weights, plan.sort_perm, plan.inverse_perm,
                     plan.kept_mask);
  return launch_status();
}

int route_dev(const float* scores, int T, int E, int k, int normalize, int capacity, int32_t* token_of_slot,
              int32_t* expert_of_slot, float* combine_weights, int32_t* group_sizes, int32_t* group_offsets,
              int32_t* num_slots, hipStream_t s) {
  if (bad_route(scores, T, E, k, token_of_slot, expert_of_slot, combine_weights, group_sizes, group_offsets))
    return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  // The temporaries are carved from the stream's own workspace (work on one stream runs in
  // order and the placement kernel is their last reader): no allocation once it has grown,
  // and three stream-ordered allocate / free pairs less on the host side of a call.
  char* ws = static_cast<char*>(stream_workspace(s, route_workspace_bytes(T * k, E)));
  if (!ws) return kDeviceFailed;
  return route_launch(scores, T, E, k, normalize, capacity, kRouterSoftmaxAll, token_of_slot, expert_of_slot,
                      combine_weights, group_sizes, group_offsets, num_slots, ws, s);
}

// route_top_k (or a given selection) + the packing plan with its token-major outputs.
int plan_dev(const float* logits, const int32_t* given_ids, const float* given_weights, int T, int E, int k,
             int router, int capacity, const PlanOutputs& plan, int32_t* token_of_slot, int32_t* expert_of_slot,
             float* combine_weights, int32_t* group_sizes, int32_t* group_offsets, int32_t* num_slots, hipStream_t s,
             int renormalize = 0) {
  if (T <= 0 || E <= 0 || k <= 0 || k > E || E > kMaxExperts || (long)T * k > 0x7fffffffL || !group_sizes ||
      !group_offsets)
    return kBadShape;
  if (logits ? (router != kRouterSoftmaxAll && k > 64) : (!given_ids || (combine_weights && !given_weights)))
    return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  char* ws = static_cast<char*>(stream_workspace(s, route_workspace_bytes(T * k, E)));
  if (!ws) return kDeviceFailed;
  return route_launch(logits, T, E, k, renormalize, capacity, router, token_of_slot, expert_of_slot, combine_weights,
                      group_sizes, group_offsets, num_slots, ws, s, plan, given_ids, given_weights);
}

// The `normalize` argument of the plan entry points: 0 = 1/k each, 1 = softmax over the selected
// logits (both route_top_k), 2 / 3 = route_tokens' router (softmax over all experts, the k
// largest probabilities), renormalised over the k (2) or as they are (3).
bool plan_router(int normalize, int* router, int* renormalize) {
  *renormalize = normalize == 2;
  switch (normalize) {
    case 0: *router = kRouterUniform; return true;
    case 1: *router = kRouterSoftmaxSelected; return true;
    case 2: case 3: *router = kRouterSoftmaxAll; return true;
    default: return false;
  }
}

// Device address of `scratch` on the current device, looked up once per device.
int route_scratch(char** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static char* ptrs[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return kDeviceFailed; }
  if (dev < 0 || dev >= kMaxDevices) return kDeviceFailed;
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
      (void)hipGetLastError();
      return kDeviceFailed;
    }
    ptrs[dev] = static_cast<char*>(p);
  }
  *out = ptrs[dev];
  return kOk;
}

}  // namespace
int route_scratch_warm() {
  char* unused = nullptr;
  return route_scratch(&unused);
}
namespace {

// ---- dispatch: exact row gather, 16 bytes per lane -------------------------------
__global__ __launch_bounds__(256) void dispatch_kernel(const char* x, const int32_t* token_of_slot, char* x_perm,
                                                       int T, int S, long row_bytes) {
  const int s = blockIdx.x;
  if (s >= S) return;
  const int t = token_of_slot[s];
  if (t < 0 || t >= T) return;
  const char* src = x + (long)t * row_bytes;
  char* dst = x_perm + (long)s * row_bytes;
  if ((row_bytes & 15) == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(x_perm)) & 15) == 0) {
    for (long o = (long)threadIdx.x * 16; o < row_bytes; o += 256 * 16)
      *reinterpret_cast<uint4*>(dst + o) = *reinterpret_cast<const uint4*>(src + o);
  } else {
    for (long o = threadIdx.x; o < row_bytes; o += 256) dst[o] = src[o];
  }
}

// ---- combine ------------------------------------------------------------------------
// The slots of a token are found by sorting slot ids by token (count, scan,
// fill); each token then adds its slots in ascending slot order — the order of
// the reference's unbuffered scatter-add — so the f32 result is reproducible.
// (n_dev, when given, is the device-side number of valid slots: the host then only
// knows the upper bound S)
__global__ void combine_count_kernel(const int32_t* token_of_slot, int S, int T, int32_t* cnt, const int32_t* n_dev) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= S || (n_dev && s >= *n_dev)) return;
  const int t = token_of_slot[s];
  if (t >= 0 && t < T) atomicAdd(&cnt[t], 1);
}
// Single workgroup exclusive scan of cnt[T] -> off[T+1]; cnt is zeroed for reuse as cursors.
__global__ __launch_bounds__(1024) void combine_scan_kernel(int32_t* cnt, int T, int32_t* off) {
  __shared__ int wave_total[16];
  const int per = (T + 1023) / 1024;
  const int lo = min((int)threadIdx.x * per, T), hi = min(lo + per, T);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int sum = 0;
  // (eight counts per round trip here as well: the loop is not unrolled on its own)
  for (int i0 = lo; i0 < hi; i0 += 8) {
    int v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = i0 + u < hi ? cnt[i0 + u] : 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) sum += v[u];
  }
  // inclusive scan of the 1024 partial sums: inside each wave by shuffles, then over the
  // 16 wave totals (two barriers in all)
  int incl = sum;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int u = __shfl_up(incl, d, 64);
    if (lane >= d) incl += u;
  }
  if (lane == 63) wave_total[wave] = incl;
  __syncthreads();
  int before = 0, total = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    const int v = wave_total[w];
    before += w < wave ? v : 0;
    total += v;
  }
  if (threadIdx.x == 0) off[T] = total;
  int run = before + incl - sum;
  // (the counts of a batch are fetched before the first store: a store between every two
  // loads would make each of them a separate round trip)
  for (int i0 = lo; i0 < hi; i0 += 8) {
    int v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = i0 + u < hi ? cnt[i0 + u] : 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (i0 + u < hi) {
        off[i0 + u] = run;
        cnt[i0 + u] = 0;
      }
      run += v[u];
    }
  }
}
__global__ void combine_fill_kernel(const int32_t* token_of_slot, int S, int T, const int32_t* off, int32_t* cursor,
                                    int32_t* list, const int32_t* n_dev) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= S || (n_dev && s >= *n_dev)) return;
  const int t = token_of_slot[s];
  if (t >= 0 && t < T) list[off[t] + atomicAdd(&cursor[t], 1)] = s;
}
// acc + (v * w) with the product rounded to f32 before the add — the reference
// scales the rows first and scatter-adds afterwards, so no fused multiply-add.
__device__ __forceinline__ float add_rounded_product(float acc, float v, float w) {
#pragma clang fp contract(off)
  const float prod = v * w;
  return acc + prod;
}

// One workgroup per token.  VEC: every thread owns runs of 16 bytes of y (8 storage
// or 4 f32 columns), so a slot row is read with 16-byte loads; needs N a multiple of
// the run and 16-byte aligned rows.  The sum over a token's slots runs in ascending
// slot order for every column either way.
// `ranked` > 0: the token's slots are not taken from the lists but from the routing's own
// token-major table, list[t ranked + j] = packed position of the token's j-th choice or -1 for a
// dropped one (ranked <= 256); off is not read.
template <class YT, bool VEC>
__global__ __launch_bounds__(256) void combine_kernel(const YT* y, const float* w, const int32_t* off,
                                                      const int32_t* list, float* out, int N, int ranked) {
  constexpr int kMaxSorted = 256;
  constexpr int RUN = VEC ? 16 / (int)sizeof(YT) : 1;
  __shared__ int sorted[kMaxSorted];
  __shared__ float sw[kMaxSorted];
  const int t = blockIdx.x;
  const int lo = ranked > 0 ? t * ranked : off[t], hi = ranked > 0 ? lo + ranked : off[t + 1];
  int len = hi - lo;
  const bool small = len <= kMaxSorted;
  if (small) {
    // rank of every slot id inside the token's list -> ascending order in LDS
    int kept = 0;
    for (int i = 0; i < len; ++i) kept += list[lo + i] >= 0;
    for (int j = threadIdx.x; j < len; j += 256) {
      const int sl = list[lo + j];
      if (sl < 0) continue;
      int rank = 0;
      for (int i = 0; i < len; ++i) {
        const int other = list[lo + i];
        rank += other >= 0 && other < sl;
      }
      sorted[rank] = sl;
      sw[rank] = w[sl];
    }
    len = kept;
    __syncthreads();
  }
  for (int n = threadIdx.x * RUN; n < N; n += 256 * RUN) {
    float acc[RUN];
#pragma unroll
    for (int e = 0; e < RUN; ++e) acc[e] = 0.f;
    auto add_row = [&](const uint4& raw, float wt) {
      const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int e = 0; e < RUN; ++e) {
        float v;
        if constexpr (sizeof(YT) == 2) v = __uint_as_float((e & 1) ? (u[e >> 1] & 0xffff0000u) : (u[e >> 1] << 16));
        else v = __uint_as_float(u[e]);
        acc[e] = add_rounded_product(acc[e], v, wt);
      }
    };
    if (VEC && small) {
      // four rows are requested before the first is added (the order of the adds stays)
      int i = 0;
      for (; i + 4 <= len; i += 4) {
        uint4 raw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) raw[u] = *reinterpret_cast<const uint4*>(y + (long)sorted[i + u] * N + n);
#pragma unroll
        for (int u = 0; u < 4; ++u) add_row(raw[u], sw[i + u]);
      }
      for (; i < len; ++i) add_row(*reinterpret_cast<const uint4*>(y + (long)sorted[i] * N + n), sw[i]);
    } else {
      int prev = -1;
      for (int i = 0; i < len; ++i) {
        int slot;
        float wt;
        if (small) {
          slot = sorted[i];
          wt = sw[i];
        } else {
          // next slot in ascending order: smallest id greater than the previous one
          int best = 0x7fffffff;
          for (int j = lo; j < hi; ++j) {
            const int sl = list[j];
            if (sl > prev && sl < best) best = sl;
          }
          prev = slot = best;
          wt = w[best];
        }
        const YT* src = y + (long)slot * N + n;
        if constexpr (VEC) {
          add_row(*reinterpret_cast<const uint4*>(src), wt);
        } else {
          float v;
          if constexpr (sizeof(YT) == 2) v = bf16_bits_to_f32(src[0]);
          else v = src[0];
          acc[0] = add_rounded_product(acc[0], v, wt);
        }
      }
    }
    if constexpr (VEC) {
#pragma unroll
      for (int e = 0; e < RUN; e += 4)
        *reinterpret_cast<float4*>(out + (long)t * N + n + e) = make_float4(acc[e], acc[e + 1], acc[e + 2], acc[e + 3]);
    } else {
      out[(long)t * N + n] = acc[0];
    }
  }
}

// models.moe_routing.unpack_combine: out[t, :] = sum over the token's k slots, in rank
// order j = 0..k-1, of y[inverse_perm[t k + j], :] * w[t, j]; the product is rounded before
// the add, like numpy's (y_slots * w).sum(axis=1).  A dropped slot (inverse_perm < 0)
// adds nothing.  One workgroup per token, 16-byte loads when the rows allow.
template <class YT, bool VEC>
__global__ __launch_bounds__(256) void unpack_combine_kernel(const YT* y, const int32_t* inverse_perm, const float* w,
                                                             float* out, int k, int N, int S) {
  constexpr int RUN = VEC ? 16 / (int)sizeof(YT) : 1;
  const int t = blockIdx.x;
  for (int n = threadIdx.x * RUN; n < N; n += 256 * RUN) {
    float acc[RUN];
#pragma unroll
    for (int e = 0; e < RUN; ++e) acc[e] = 0.f;
    for (int j = 0; j < k; ++j) {
      const int pos = inverse_perm[(long)t * k + j];
      if (pos < 0 || pos >= S) continue;
      const float wt = w[(long)t * k + j];
      const YT* src = y + (long)pos * N + n;
      if constexpr (VEC) {
        const uint4 raw = *reinterpret_cast<const uint4*>(src);
        const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int e = 0; e < RUN; ++e) {
          float v;
          if constexpr (sizeof(YT) == 2) v = __uint_as_float((e & 1) ? (u[e >> 1] & 0xffff0000u) : (u[e >> 1] << 16));
          else v = __uint_as_float(u[e]);
          acc[e] = add_rounded_product(acc[e], v, wt);
        }
      } else {
        float v;
        if constexpr (sizeof(YT) == 2) v = bf16_bits_to_f32(src[0]);
        else v = src[0];
        acc[0] = add_rounded_product(acc[0], v, wt);
      }
    }
    if constexpr (VEC) {
#pragma unroll
      for (int e = 0; e < RUN; e += 4)
        *reinterpret_cast<float4*>(out + (long)t * N + n + e) = make_float4(acc[e], acc[e + 1], acc[e + 2], acc[e + 3]);
    } else {
      out[(long)t * N + n] = acc[0];
    }
  }
}

template <class YT>
int unpack_combine_dev(const void* y, const int32_t* inverse_perm, const float* w, float* out, int T, int k, int S,
                       int N, hipStream_t s) {
  if (T <= 0 || k <= 0 || S < 0 || N <= 0 || !out || !inverse_perm || !w || (S > 0 && !y)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const bool vec = N % (16 / (int)sizeof(YT)) == 0 && aligned16(y) && aligned16(out);
  if (vec)
    hipLaunchKernelGGL((unpack_combine_kernel<YT, true>), dim3(T), dim3(256), 0, s, static_cast<const YT*>(y),
                       inverse_perm, w, out, k, N, S);
  else
    hipLaunchKernelGGL((unpack_combine_kernel<YT, false>), dim3(T), dim3(256), 0, s, static_cast<const YT*>(y),
                       inverse_perm, w, out, k, N, S);
  return launch_status();
}

// `positions` (with k = `ranked`): the routing's token-major table of packed positions; the
// per-token lists are then not built.
template <class YT>
int combine_dev(const void* y, const int32_t* token_of_slot, const float* w, float* out, int T, int S, int N,
                hipStream_t s, const int32_t* n_dev = nullptr, const int32_t* positions = nullptr, int ranked = 0) {
  if (T <= 0 || S < 0 || N <= 0 || !out || (S > 0 && (!y || !token_of_slot || !w))) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  if (positions && ranked > 0 && ranked <= 256) {
    const bool vec = N % (16 / (int)sizeof(YT)) == 0 && aligned16(y) && aligned16(out);
    if (vec)
      hipLaunchKernelGGL((combine_kernel<YT, true>), dim3(T), dim3(256), 0, s, static_cast<const YT*>(y), w, nullptr, positions, out, N, ranked);
    else
      hipLaunchKernelGGL((combine_kernel<YT, false>), dim3(T), dim3(256), 0, s, static_cast<const YT*>(y), w, nullptr, positions, out, N, ranked);
    return launch_status();
  }
  // the per-token slot lists live in the stream's own workspace (the combine kernel below
  // is their last reader; work on one stream runs in order)
  const size_t tok_bytes = ((size_t)(T + 1) * 4 + 255) & ~(size_t)255;
  char* ws = static_cast<char*>(stream_workspace(s, 2 * tok_bytes + (size_t)(S > 0 ? S : 1) * 4));
  if (!ws) return kDeviceFailed;
  int32_t* cnt = reinterpret_cast<int32_t*>(ws);
  int32_t* off = reinterpret_cast<int32_t*>(ws + tok_bytes);
  int32_t* list = reinterpret_cast<int32_t*>(ws + 2 * tok_bytes);
  zero_words(cnt, (size_t)T, s);
  if (S > 0) hipLaunchKernelGGL(combine_count_kernel, dim3(ceil_div(S, 256)), dim3(256), 0, s, token_of_slot, S, T, cnt, n_dev);
  hipLaunchKernelGGL(combine_scan_kernel, dim3(1), dim3(1024), 0, s, cnt, T, off);
  if (S > 0) hipLaunchKernelGGL(combine_fill_kernel, dim3(ceil_div(S, 256)), dim3(256), 0, s, token_of_slot, S, T, off, cnt, list, n_dev);
  const bool vec = N % (16 / (int)sizeof(YT)) == 0 && aligned16(y) && aligned16(out);
  if (vec)
    hipLaunchKernelGGL((combine_kernel<YT, true>), dim3(T), dim3(256), 0, s, static_cast<const YT*>(y), w, off, list, out, N, 0);
  else
    hipLaunchKernelGGL((combine_kernel<YT, false>), dim3(T), dim3(256), 0, s, static_cast<const YT*>(y), w, off, list, out, N, 0);
  return launch_status();
}

int dispatch_dev(const void* x, const int32_t* token_of_slot, void* x_perm, int T, int S, int H, int elem_bytes,
                 hipStream_t s) {
  if (T <= 0 || S < 0 || H <= 0 || (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) || !x ||
      (S > 0 && (!token_of_slot || !x_perm)))
    return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  if (S == 0) return kOk;
  hipLaunchKernelGGL(dispatch_kernel, dim3(S), dim3(256), 0, s, static_cast<const char*>(x), token_of_slot,
                     static_cast<char*>(x_perm), T, S, (long)H * elem_bytes);
  return launch_status();
}

// out[r, :] = y[r, :] * scale[e] for the rows r of group e (offsets[e] <= r < offsets[e + 1]): the
// per-tensor scales of a quantised grouped product, applied to the f32 result of the product of
// the unscaled grid values.  One workgroup per row.  OUT16: the result is rounded to bf16.
template <bool OUT16>
__global__ __launch_bounds__(256) void scale_groups_kernel(const float* __restrict__ y, const int32_t* __restrict__ offsets,
                                                           const float* __restrict__ scale, int E, int N,
                                                           void* __restrict__ out) {
  const int r = blockIdx.x;
  int lo = 0, hi = E - 1;                                  // the last group whose first row is <= r
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (offsets[mid] <= r) lo = mid; else hi = mid - 1;
  }
  const float sc = scale[lo];
  const float* src = y + (long)r * N;
  for (int n = threadIdx.x; n < N; n += 256) {
    const float v = src[n] * sc;
    if constexpr (OUT16) static_cast<uint16_t*>(out)[(long)r * N + n] = f32_to_bf16_bits(v);
    else static_cast<float*>(out)[(long)r * N + n] = v;
  }
}

int scale_groups_dev(const float* y, const int32_t* offsets, const float* scale, void* out, int out_bf16, int S, int N,
                     int E, hipStream_t s) {
  if (S < 0 || N <= 0 || E <= 0 || !offsets || !scale || (S > 0 && (!y || !out))) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  if (S == 0) return kOk;
  if (out_bf16)
    hipLaunchKernelGGL((scale_groups_kernel<true>), dim3(S), dim3(256), 0, s, y, offsets, scale, E, N, out);
  else
    hipLaunchKernelGGL((scale_groups_kernel<false>), dim3(S), dim3(256), 0, s, y, offsets, scale, E, N, out);
  return launch_status();
}

bool bad_grouped(int S, int K, int N, int E) { return S < 0 || K <= 0 || N <= 0 || E <= 0; }

// A gathered row of the (rows, K) 16-bit activation is fetched by a buffer load whose
// offset is counted from the start of x, and the buffer resource spans kBufferRange
// bytes: an offset at or past the range reads as zero without an error, so the whole
// activation has to lie inside it.
bool gather_out_of_buffer_range(int rows, int K) { return (long)rows * K * 2 > (long)kBufferRange - 16; }

template <int EPI, class T = BF16>
int grouped_dev(const void* x, const void* w, const int32_t* offsets, void* y, int S, int K, int N, int E,
                hipStream_t s) {
  if (bad_grouped(S, K, N, E) || !w || !offsets || (S > 0 && (!x || !y))) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  if (S == 0) return kOk;
  Gemm16Params p{};
  p.A = static_cast<const uint16_t*>(x);
  p.B = static_cast<const uint16_t*>(w);
  p.D = y;
  p.M = S; p.N = N; p.K = K;
  p.lda = K; p.ldb = N; p.ldd = N;
  p.strideB = (long)K * N;
  p.offsets = offsets;
  p.groups = E;
  return launch_gemm16_grouped<T, EPI>(p, s);
}

// `gather` (device int32[S], or null): row m of the block's input is x[gather[m]], i.e.
// x is the unpermuted (T, K) activation and the dispatch is part of the first GEMM's
// operand load.  x_rows = number of rows of x (T with a gather, else S).
int swiglu_dev(const void* x, const void* wg, const void* wu, const void* wd, const int32_t* offsets, void* y,
               void* hidden, int S, int K, int F, int N, int E, hipStream_t s, const int32_t* gather = nullptr,
               int x_rows = 0) {
  if (bad_grouped(S, K, N, E) || F <= 0 || !wg || !wu || !wd || !offsets || (S > 0 && (!x || !y))) return kBadShape;
  // (the kernels address a gathered row with a buffer load off x)
  if (gather && (x_rows <= 0 || gather_out_of_buffer_range(x_rows, K))) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  if (S == 0) return kOk;
  void* h = hidden;
  if (!h && hipMallocAsync(&h, (size_t)S * F * 2, s) != hipSuccess) return kDeviceFailed;
  Gemm16Params p{};
  p.A = static_cast<const uint16_t*>(x);
  p.B = static_cast<const uint16_t*>(wg);
  p.B2 = static_cast<const uint16_t*>(wu);
  p.D = h;
  p.M = S; p.N = F; p.K = K;
  p.lda = K; p.ldb = F; p.ldd = F;
  p.strideB = (long)K * F;
  p.offsets = offsets;
  p.gather = gather;
  p.groups = E;
  int rc = launch_gemm16_grouped<BF16, EPI_SWIGLU16>(p, s);
  if (rc == kOk) rc = grouped_dev<EPI_STORE16>(h, wd, offsets, y, S, F, N, E, s);
  if (!hidden && hipFreeAsync(h, s) != hipSuccess) rc = kDeviceFailed;
  return rc;
}

// bf16 bit patterns -> f32 (exact widening), 8 per thread.
__global__ __launch_bounds__(256) void widen_bf16_kernel(const uint16_t* __restrict__ in, float* __restrict__ out, long n) {
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i + 8 <= n) {
    const uint4 v = *reinterpret_cast<const uint4*>(in + i);
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
    float4 lo, hi;
    lo.x = __uint_as_float(u[0] << 16); lo.y = __uint_as_float(u[0] & 0xffff0000u);
    lo.z = __uint_as_float(u[1] << 16); lo.w = __uint_as_float(u[1] & 0xffff0000u);
    hi.x = __uint_as_float(u[2] << 16); hi.y = __uint_as_float(u[2] & 0xffff0000u);
    hi.z = __uint_as_float(u[3] << 16); hi.w = __uint_as_float(u[3] & 0xffff0000u);
    *reinterpret_cast<float4*>(out + i) = lo;
    *reinterpret_cast<float4*>(out + i + 4) = hi;
  } else {
    for (long j = i; j < n; ++j) out[j] = bf16_bits_to_f32(in[j]);
  }
}

inline size_t round256(size_t b) { return (b + 255) & ~(size_t)255; }

// Device scratch of the whole layer: router scores (bf16) and logits (f32), the hidden
// activation h [T k, F] and the expert output y [T k, N] (both bf16).
struct LayerScratch {
  size_t scores, logits, hidden, y, positions, route, total;
};
LayerScratch layer_scratch(int T, int F, int N, int E, int k) {
  LayerScratch w{};
  const size_t S = (size_t)T * k;
  w.scores = 0;
  w.logits = w.scores + round256((size_t)T * E * 2);
  w.hidden = w.logits + round256((size_t)T * E * 4);
  w.y = w.hidden + round256(S * F * 2);
  w.positions = w.y + round256(S * N * 2);      // token-major packed positions, for the combine
  w.route = w.positions + round256(S * 4);      // the routing kernels' temporaries
  w.total = w.route + round256(route_workspace_bytes((int)S, E));
  return w;
}

bool bad_layer(int T, int H, int F, int N, int E, int k) {
  return T <= 0 || H <= 0 || F <= 0 || N <= 0 || E <= 0 || k <= 0 || k > E || E > kMaxExperts ||
         (long)T * k > 0x7fffffffL;
}

// nn.functional.moe_layer on one stream, no host hop: (router GEMM ->) route -> expert
// block reading x through the dispatch map -> combine.  With a capacity the number of
// kept slots is only known on the device (*num_slots): every later stage is launched
// for the upper bound T k and takes its real extent from the device-side offsets / count.
int moe_layer_dev(const void* x, const void* w_router, const float* router_logits, const void* wg, const void* wu,
                  const void* wd, float* out, void* workspace, size_t workspace_bytes, int T, int H, int F, int N,
                  int E, int k, int normalize, int capacity, int32_t* token_of_slot, int32_t* expert_of_slot,
                  float* combine_weights, int32_t* group_sizes, int32_t* group_offsets, int32_t* num_slots,
                  hipStream_t s) {
  if (bad_layer(T, H, F, N, E, k) || !x || (!w_router && !router_logits) || !wg || !wu || !wd || !out ||
      !workspace || !token_of_slot || !expert_of_slot || !combine_weights || !group_sizes || !group_offsets ||
      !num_slots || !aligned16(workspace))
    return kBadShape;
  const LayerScratch w = layer_scratch(T, F, N, E, k);
  if (workspace_bytes < w.total) return kBadShape;
  if (gather_out_of_buffer_range(T, H)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  char* ws = static_cast<char*>(workspace);
  const float* logits = router_logits;
  if (w_router) {
    // scores = ops.gemm(x, W_router): stored in bf16 like every reduced-precision
    // product, then read as f32 (nn/functional.py:453)
    Gemm16Params g{};
    g.A = static_cast<const uint16_t*>(x);
    g.B = static_cast<const uint16_t*>(w_router);
    g.D = ws + w.scores;
    g.M = T; g.N = E; g.K = H;
    g.lda = H; g.ldb = E; g.ldd = E;
    g.strideA = (long)T * H; g.strideB = (long)H * E; g.strideD = (long)T * E;
    g.groups = 1;
    if (const int rc = launch_gemm16<BF16, EPI_STORE16>(g, s); rc != kOk) return rc;
    const long n = (long)T * E;
    hipLaunchKernelGGL(widen_bf16_kernel, dim3((unsigned)((n + 2047) / 2048)), dim3(256), 0, s,
                       reinterpret_cast<const uint16_t*>(ws + w.scores), reinterpret_cast<float*>(ws + w.logits), n);
    logits = reinterpret_cast<const float*>(ws + w.logits);
  }
  // (the placement pass also leaves each token's packed positions, so the combine need not
  // rebuild per-token slot lists from token_of_slot)
  PlanOutputs plan;
  plan.inverse_perm = reinterpret_cast<int32_t*>(ws + w.positions);
  // (the routing temporaries, too, come from the caller's workspace: with the logits given the
  // layer touches no memory of the library's)
  if (bad_route(logits, T, E, k, token_of_slot, expert_of_slot, combine_weights, group_sizes, group_offsets))
    return kBadShape;
  int rc = route_launch(logits, T, E, k, normalize, capacity, kRouterSoftmaxAll, token_of_slot, expert_of_slot,
                        combine_weights, group_sizes, group_offsets, num_slots, ws + w.route, s, plan);
  if (rc != kOk) return rc;
  const int S = T * k;
  rc = swiglu_dev(x, wg, wu, wd, group_offsets, ws + w.y, ws + w.hidden, S, H, F, N, E, s, token_of_slot, T);
  if (rc != kOk) return rc;
  return combine_dev<uint16_t>(ws + w.y, token_of_slot, combine_weights, out, T, S, N, s, num_slots,
                               plan.inverse_perm, k);
}

// Host-pointer form of the layer: upload, run moe_layer_dev, download.
int moe_layer_host(const void* x, const void* w_router, const float* router_logits, const void* wg, const void* wu,
                   const void* wd, float* out, int T, int H, int F, int N, int E, int k, int normalize, int capacity,
                   int32_t* token_of_slot, int32_t* expert_of_slot, float* combine_weights, int32_t* group_sizes,
                   int32_t* group_offsets, float* logits_out) {
  if (bad_layer(T, H, F, N, E, k) || !x || (!w_router && !router_logits) || !wg || !wu || !wd || !out)
    return kBadShape;
  if (gather_out_of_buffer_range(T, H)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const size_t S = (size_t)T * k;
  const LayerScratch w = layer_scratch(T, F, N, E, k);
  DeviceScope scope;
  void* dx = scope.alloc((size_t)T * H * 2, x);
  void* dr = w_router ? scope.alloc((size_t)H * E * 2, w_router) : nullptr;
  float* dl = router_logits && !w_router ? static_cast<float*>(scope.alloc((size_t)T * E * 4, router_logits)) : nullptr;
  void* dg = scope.alloc((size_t)E * H * F * 2, wg);
  void* du = scope.alloc((size_t)E * H * F * 2, wu);
  void* dd = scope.alloc((size_t)E * F * N * 2, wd);
  int32_t* dt = static_cast<int32_t*>(scope.alloc(S * 4));
  int32_t* de = static_cast<int32_t*>(scope.alloc(S * 4));
  float* dw = static_cast<float*>(scope.alloc(S * 4));
  int32_t* dgs = static_cast<int32_t*>(scope.alloc((size_t)E * 4));
  int32_t* dof = static_cast<int32_t*>(scope.alloc((size_t)(E + 1) * 4));
  int32_t* dn = static_cast<int32_t*>(scope.alloc(4));
  void* dws = scope.alloc(w.total);
  float* dout = static_cast<float*>(scope.alloc((size_t)T * N * 4));
  if (scope.failed()) return kDeviceFailed;
  int rc = moe_layer_dev(dx, dr, dl, dg, du, dd, dout, dws, w.total, T, H, F, N, E, k, normalize, capacity, dt, de,
                         dw, dgs, dof, dn, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  int32_t n = 0;                       // kept slots (a capacity may drop some)
  if (!scope.download(&n, dn, 4) || !scope.download(out, dout, (size_t)T * N * 4)) return kDeviceFailed;
  if (token_of_slot && !scope.download(token_of_slot, dt, (size_t)n * 4)) return kDeviceFailed;
  if (expert_of_slot && !scope.download(expert_of_slot, de, (size_t)n * 4)) return kDeviceFailed;
  if (combine_weights && !scope.download(combine_weights, dw, (size_t)n * 4)) return kDeviceFailed;
  if (group_sizes && !scope.download(group_sizes, dgs, (size_t)E * 4)) return kDeviceFailed;
  if (group_offsets && !scope.download(group_offsets, dof, (size_t)(E + 1) * 4)) return kDeviceFailed;
  if (logits_out && w_router &&
      !scope.download(logits_out, static_cast<char*>(dws) + w.logits, (size_t)T * E * 4))
    return kDeviceFailed;
  return kOk;
}

int combine_host(const void* y_perm, const int32_t* token_of_slot, const float* weights, float* out, int T,
                        int S, int N, int ysz) {
  if (T <= 0 || S < 0 || N <= 0 || !out || (S > 0 && (!y_perm || !token_of_slot || !weights))) return kBadShape;
  for (int s = 0; s < S; ++s)
    if (token_of_slot[s] < 0 || token_of_slot[s] >= T) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  DeviceScope scope;
  void* dy = scope.alloc((size_t)S * N * ysz, y_perm);
  int32_t* dt = static_cast<int32_t*>(scope.alloc((size_t)S * 4, token_of_slot));
  float* dw = static_cast<float*>(scope.alloc((size_t)S * 4, weights));
  float* dout = static_cast<float*>(scope.alloc((size_t)T * N * 4));
  if (scope.failed()) return kDeviceFailed;
  int rc = ysz == 2 ? combine_dev<uint16_t>(dy, dt, dw, dout, T, S, N, nullptr)
                    : combine_dev<float>(dy, dt, dw, dout, T, S, N, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  return scope.download(out, dout, (size_t)T * N * 4) ? kOk : kDeviceFailed;
}
// offsets must be non-decreasing, start at 0 and end at S.
bool bad_offsets(const int32_t* offsets, int E, int S) {
  if (offsets[0] != 0 || offsets[E] != S) return true;
  for (int e = 0; e < E; ++e)
    if (offsets[e + 1] < offsets[e]) return true;
  return false;
}

template <int EPI, class T = BF16>
int grouped_host(const void* x, const void* w, const int32_t* offsets, void* y, int S, int K, int N, int E) {
  if (bad_grouped(S, K, N, E) || !w || !offsets || (S > 0 && (!x || !y))) return kBadShape;
  if (bad_offsets(offsets, E, S)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  if (S == 0) return kOk;
  const size_t dsz = EPI == EPI_F32 ? 4 : 2;
  DeviceScope scope;
  void* dx = scope.alloc((size_t)S * K * 2, x);
  void* dw = scope.alloc((size_t)E * K * N * 2, w);
  int32_t* dof = static_cast<int32_t*>(scope.alloc((size_t)(E + 1) * 4, offsets));
  void* dy = scope.alloc((size_t)S * N * dsz);
  if (scope.failed()) return kDeviceFailed;
  int rc = grouped_dev<EPI, T>(dx, dw, dof, dy, S, K, N, E, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  return scope.download(y, dy, (size_t)S * N * dsz) ? kOk : kDeviceFailed;
}
// out = storage(silu(a) * b) elementwise on 16-bit storage, eight elements per thread in the body.
template <class T>
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b,
                                                       uint16_t* __restrict__ out, long n) {
  auto one = [](uint16_t ga, uint16_t ub) -> uint16_t {
    const float g = from_storage<T>(ga), u = from_storage<T>(ub);
    return to_storage<T>((g / (1.0f + __expf(-g))) * u);
  };
  const long tid = (long)blockIdx.x * 256 + threadIdx.x, nth = (long)gridDim.x * 256;
  const bool vec = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
  const long n8 = vec ? n / 8 : 0;
  for (long i = tid; i < n8; i += nth) {
    const uint4 va = reinterpret_cast<const uint4*>(a)[i], vb = reinterpret_cast<const uint4*>(b)[i];
    const uint32_t wa[4] = {va.x, va.y, va.z, va.w}, wb[4] = {vb.x, vb.y, vb.z, vb.w};
    uint32_t wo[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      wo[e] = (uint32_t)one((uint16_t)(wa[e] & 0xffff), (uint16_t)(wb[e] & 0xffff)) |
              ((uint32_t)one((uint16_t)(wa[e] >> 16), (uint16_t)(wb[e] >> 16)) << 16);
    reinterpret_cast<uint4*>(out)[i] = make_uint4(wo[0], wo[1], wo[2], wo[3]);
  }
  for (long i = n8 * 8 + tid; i < n; i += nth) out[i] = one(a[i], b[i]);
}

template <class T>
int silu_mul_dev(const void* a, const void* b, void* out, int64_t n, hipStream_t s) {
  if (n <= 0 || !a || !b || !out) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const long blocks = std::min<long>((n / 8 + 255) / 256 + 1, 8192);
  hipLaunchKernelGGL(silu_mul_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<const uint16_t*>(a),
                     static_cast<const uint16_t*>(b), static_cast<uint16_t*>(out), (long)n);
  return launch_status();
}

template <class T>
int silu_mul_host(const void* a, const void* b, void* out, int64_t n) {
  if (n <= 0 || !a || !b || !out) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  DeviceScope scope;
  void* da = scope.alloc((size_t)n * 2, a);
  void* db = scope.alloc((size_t)n * 2, b);
  void* dout = scope.alloc((size_t)n * 2);
  if (scope.failed()) return kDeviceFailed;
  int rc = silu_mul_dev<T>(da, db, dout, n, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  return scope.download(out, dout, (size_t)n * 2) ? kOk : kDeviceFailed;
}
}  // namespace
}  // namespace tsr950

using namespace tsr950;

extern "C" {

int tessera_gfx950_silu_mul_bf16(const void* a, const void* b, void* out, int64_t n) { return silu_mul_host<BF16>(a, b, out, n); }
int tessera_gfx950_silu_mul_f16(const void* a, const void* b, void* out, int64_t n) { return silu_mul_host<F16>(a, b, out, n); }
int tessera_gfx950_silu_mul_bf16_dev(const void* a, const void* b, void* out, int64_t n, void* stream) {
  return silu_mul_dev<BF16>(a, b, out, n, as_stream(stream));
}
int tessera_gfx950_silu_mul_f16_dev(const void* a, const void* b, void* out, int64_t n, void* stream) {
  return silu_mul_dev<F16>(a, b, out, n, as_stream(stream));
}


int tessera_gfx950_moe_route_f32_dev(const float* scores, int T, int E, int k, int normalize, int capacity,
                                     int32_t* token_of_slot, int32_t* expert_of_slot, float* combine_weights,
                                     int32_t* group_sizes, int32_t* group_offsets, int32_t* num_slots,
                                     void* stream) {
  return route_dev(scores, T, E, k, normalize, capacity, token_of_slot, expert_of_slot, combine_weights,
                   group_sizes, group_offsets, num_slots, as_stream(stream));
}

int tessera_gfx950_moe_route_f32_noalloc_dev(const float* scores, int T, int E, int k, int normalize, int capacity,
                                             int32_t* token_of_slot, int32_t* expert_of_slot,
                                             float* combine_weights, int32_t* group_sizes, int32_t* group_offsets,
                                             int32_t* num_slots, void* stream) {
  if (bad_route(scores, T, E, k, token_of_slot, expert_of_slot, combine_weights, group_sizes, group_offsets))
    return kBadShape;
  if (route_workspace_bytes(T * k, E) > kRouteScratchBytes) return kBadShape;    // beyond the fixed scratch
  if (probe_device() != kOk) return kNoDevice;
  char* ws = nullptr;
  if (const int rc = route_scratch(&ws); rc != kOk) return rc;
  return route_launch(scores, T, E, k, normalize, capacity, kRouterSoftmaxAll, token_of_slot, expert_of_slot,
                      combine_weights, group_sizes, group_offsets, num_slots, ws, as_stream(stream));
}

int tessera_gfx950_moe_route_f32(const float* scores, int T, int E, int k, int normalize, int capacity,
                                 int32_t* token_of_slot, int32_t* expert_of_slot, float* combine_weights,
                                 int32_t* group_sizes, int32_t* group_offsets, int32_t* num_slots) {
  if (T <= 0 || E <= 0 || k <= 0 || k > E || E > kMaxExperts || !scores || !token_of_slot || !expert_of_slot ||
      !combine_weights || !group_sizes || !group_offsets)
    return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  const size_t S = (size_t)T * k;
  DeviceScope scope;
  float* ds = static_cast<float*>(scope.alloc((size_t)T * E * 4, scores));
  int32_t* dt = static_cast<int32_t*>(scope.alloc(S * 4));
  int32_t* de = static_cast<int32_t*>(scope.alloc(S * 4));
  float* dw = static_cast<float*>(scope.alloc(S * 4));
  int32_t* dg = static_cast<int32_t*>(scope.alloc((size_t)E * 4));
  int32_t* dof = static_cast<int32_t*>(scope.alloc((size_t)(E + 1) * 4));
  int32_t* dn = static_cast<int32_t*>(scope.alloc(4));
  if (scope.failed()) return kDeviceFailed;
  int rc = route_dev(ds, T, E, k, normalize, capacity, dt, de, dw, dg, dof, dn, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  int32_t n = 0;
  if (!scope.download(&n, dn, 4)) return kDeviceFailed;
  if (!scope.download(token_of_slot, dt, (size_t)n * 4) || !scope.download(expert_of_slot, de, (size_t)n * 4) ||
      !scope.download(combine_weights, dw, (size_t)n * 4) || !scope.download(group_sizes, dg, (size_t)E * 4) ||
      !scope.download(group_offsets, dof, (size_t)(E + 1) * 4))
    return kDeviceFailed;
  if (num_slots) *num_slots = n;
  return kOk;
}

int tessera_gfx950_moe_plan_f32_dev(const float* router_logits, const int32_t* given_expert_ids,
                                    const float* given_weights, int T, int E, int k, int normalize, int capacity,
                                    int32_t* expert_ids, float* weights, uint8_t* kept_mask, int32_t* sort_perm,
                                    int32_t* inverse_perm, int32_t* token_of_slot, int32_t* expert_of_slot,
                                    float* combine_weights, int32_t* group_sizes, int32_t* group_offsets,
                                    int32_t* num_slots, void* stream) {
  PlanOutputs plan;
  plan.expert_ids = router_logits ? expert_ids : nullptr;
  plan.weights = router_logits ? weights : nullptr;
  plan.kept_mask = kept_mask;
  plan.sort_perm = sort_perm;
  plan.inverse_perm = inverse_perm;
  int router = 0, renorm = 0;
  if (!plan_router(normalize, &router, &renorm)) return kBadShape;
  return plan_dev(router_logits, given_expert_ids, given_weights, T, E, k, router, capacity, plan, token_of_slot,
                  expert_of_slot, combine_weights, group_sizes, group_offsets, num_slots, as_stream(stream), renorm);
}

int tessera_gfx950_moe_plan_f32(const float* router_logits, const int32_t* given_expert_ids,
                                const float* given_weights, int T, int E, int k, int normalize, int capacity,
                                int32_t* expert_ids, float* weights, uint8_t* kept_mask, int32_t* sort_perm,
                                int32_t* inverse_perm, int32_t* token_of_slot, int32_t* expert_of_slot,
                                float* combine_weights, int32_t* group_sizes, int32_t* group_offsets,
                                int32_t* num_slots) {
  if (T <= 0 || E <= 0 || k <= 0 || k > E || E > kMaxExperts || (long)T * k > 0x7fffffffL || !group_sizes ||
      !group_offsets)
    return kBadShape;
  if (router_logits ? (normalize < 0 || normalize > 3 || (normalize < 2 && k > 64)) : !given_expert_ids) return kBadShape;
  const size_t S = (size_t)T * k;
  if (!router_logits)
    for (size_t i = 0; i < S; ++i)
      if (given_expert_ids[i] < 0 || given_expert_ids[i] >= E) return kBadShape;     // "expert id out of range"
  if (probe_device() != kOk) return kNoDevice;
  DeviceScope scope;
  float* dl = router_logits ? static_cast<float*>(scope.alloc((size_t)T * E * 4, router_logits)) : nullptr;
  int32_t* dgi = router_logits ? nullptr : static_cast<int32_t*>(scope.alloc(S * 4, given_expert_ids));
  // (a plan built from ids alone carries no weights: zeros, as plan_packing's placeholder)
  float* dgw = router_logits ? nullptr : static_cast<float*>(scope.alloc(S * 4, given_weights));
  if (dgw && !given_weights && hipMemset(dgw, 0, S * 4) != hipSuccess) return kDeviceFailed;
  int32_t* dids = static_cast<int32_t*>(scope.alloc(S * 4));
  float* dw = static_cast<float*>(scope.alloc(S * 4));
  uint8_t* dkm = static_cast<uint8_t*>(scope.alloc(S));
  int32_t* dsp = static_cast<int32_t*>(scope.alloc(S * 4));
  int32_t* dip = static_cast<int32_t*>(scope.alloc(S * 4));
  int32_t* dt = static_cast<int32_t*>(scope.alloc(S * 4));
  int32_t* de = static_cast<int32_t*>(scope.alloc(S * 4));
  float* dcw = static_cast<float*>(scope.alloc(S * 4));
  int32_t* dg = static_cast<int32_t*>(scope.alloc((size_t)E * 4));
  int32_t* dof = static_cast<int32_t*>(scope.alloc((size_t)(E + 1) * 4));
  int32_t* dn = static_cast<int32_t*>(scope.alloc(4));
  if (scope.failed()) return kDeviceFailed;
  int rc = tessera_gfx950_moe_plan_f32_dev(dl, dgi, dgw, T, E, k, normalize, capacity, dids, dw, dkm, dsp, dip, dt,
                                           de, dcw, dg, dof, dn, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  int32_t n = 0;
  if (!scope.download(&n, dn, 4)) return kDeviceFailed;
  const size_t kept = (size_t)n * 4;
  if ((expert_ids && router_logits && !scope.download(expert_ids, dids, S * 4)) ||
      (weights && router_logits && !scope.download(weights, dw, S * 4)) ||
      (kept_mask && !scope.download(kept_mask, dkm, S)) || (sort_perm && !scope.download(sort_perm, dsp, kept)) ||
      (inverse_perm && !scope.download(inverse_perm, dip, S * 4)) ||
      (token_of_slot && !scope.download(token_of_slot, dt, kept)) ||
      (expert_of_slot && !scope.download(expert_of_slot, de, kept)) ||
      (combine_weights && !scope.download(combine_weights, dcw, kept)) ||
      !scope.download(group_sizes, dg, (size_t)E * 4) || !scope.download(group_offsets, dof, (size_t)(E + 1) * 4))
    return kDeviceFailed;
  if (num_slots) *num_slots = n;
  return kOk;
}

int tessera_gfx950_moe_unpack_combine_bf16_dev(const void* y_packed, const int32_t* inverse_perm,
                                               const float* weights, float* out, int T, int k, int S, int N,
                                               void* stream) {
  return unpack_combine_dev<uint16_t>(y_packed, inverse_perm, weights, out, T, k, S, N, as_stream(stream));
}
int tessera_gfx950_moe_unpack_combine_f32_dev(const void* y_packed, const int32_t* inverse_perm,
                                              const float* weights, float* out, int T, int k, int S, int N,
                                              void* stream) {
  return unpack_combine_dev<float>(y_packed, inverse_perm, weights, out, T, k, S, N, as_stream(stream));
}
static int unpack_combine_host(const void* y_packed, const int32_t* inverse_perm, const float* weights, float* out,
                               int T, int k, int S, int N, int ysz) {
  if (T <= 0 || k <= 0 || S < 0 || N <= 0 || !out || !inverse_perm || !weights || (S > 0 && !y_packed))
    return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  DeviceScope scope;
  void* dy = scope.alloc((size_t)S * N * ysz, y_packed);
  int32_t* dip = static_cast<int32_t*>(scope.alloc((size_t)T * k * 4, inverse_perm));
  float* dw = static_cast<float*>(scope.alloc((size_t)T * k * 4, weights));
  float* dout = static_cast<float*>(scope.alloc((size_t)T * N * 4));
  if (scope.failed()) return kDeviceFailed;
  int rc = ysz == 2 ? unpack_combine_dev<uint16_t>(dy, dip, dw, dout, T, k, S, N, nullptr)
                    : unpack_combine_dev<float>(dy, dip, dw, dout, T, k, S, N, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  return scope.download(out, dout, (size_t)T * N * 4) ? kOk : kDeviceFailed;
}
int tessera_gfx950_moe_unpack_combine_bf16(const void* y_packed, const int32_t* inverse_perm, const float* weights,
                                           float* out, int T, int k, int S, int N) {
  return unpack_combine_host(y_packed, inverse_perm, weights, out, T, k, S, N, 2);
}
int tessera_gfx950_moe_unpack_combine_f32(const void* y_packed, const int32_t* inverse_perm, const float* weights,
                                          float* out, int T, int k, int S, int N) {
  return unpack_combine_host(y_packed, inverse_perm, weights, out, T, k, S, N, 4);
}

int tessera_gfx950_moe_dispatch_dev(const void* x, const int32_t* token_of_slot, void* x_perm, int T, int S, int H,
                                    int elem_bytes, void* stream) {
  return dispatch_dev(x, token_of_slot, x_perm, T, S, H, elem_bytes, as_stream(stream));
}

int tessera_gfx950_moe_dispatch(const void* x, const int32_t* token_of_slot, void* x_perm, int T, int S, int H,
                                int elem_bytes) {
  if (T <= 0 || S < 0 || H <= 0 || (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) || !x ||
      (S > 0 && (!token_of_slot || !x_perm)))
    return kBadShape;
  for (int s = 0; s < S; ++s)
    if (token_of_slot[s] < 0 || token_of_slot[s] >= T) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  if (S == 0) return kOk;
  const size_t row = (size_t)H * elem_bytes;
  DeviceScope scope;
  void* dx = scope.alloc((size_t)T * row, x);
  int32_t* dt = static_cast<int32_t*>(scope.alloc((size_t)S * 4, token_of_slot));
  void* dp = scope.alloc((size_t)S * row);
  if (scope.failed()) return kDeviceFailed;
  int rc = dispatch_dev(dx, dt, dp, T, S, H, elem_bytes, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  return scope.download(x_perm, dp, (size_t)S * row) ? kOk : kDeviceFailed;
}

int tessera_gfx950_moe_combine_bf16_dev(const void* y_perm, const int32_t* token_of_slot, const float* weights,
                                        float* out, int T, int S, int N, void* stream) {
  return combine_dev<uint16_t>(y_perm, token_of_slot, weights, out, T, S, N, as_stream(stream));
}
int tessera_gfx950_moe_combine_f32_dev(const void* y_perm, const int32_t* token_of_slot, const float* weights,
                                       float* out, int T, int S, int N, void* stream) {
  return combine_dev<float>(y_perm, token_of_slot, weights, out, T, S, N, as_stream(stream));
}

int tessera_gfx950_moe_combine_bf16(const void* y_perm, const int32_t* token_of_slot, const float* weights,
                                    float* out, int T, int S, int N) {
  return combine_host(y_perm, token_of_slot, weights, out, T, S, N, 2);
}
int tessera_gfx950_moe_combine_f32(const void* y_perm, const int32_t* token_of_slot, const float* weights,
                                   float* out, int T, int S, int N) {
  return combine_host(y_perm, token_of_slot, weights, out, T, S, N, 4);
}

int tessera_gfx950_grouped_gemm_bf16_dev(const void* x, const void* w, const int32_t* offsets, void* y, int S,
                                         int K, int N, int E, void* stream) {
  return grouped_dev<EPI_STORE16>(x, w, offsets, y, S, K, N, E, as_stream(stream));
}
int tessera_gfx950_grouped_gemm_bf16_f32_dev(const void* x, const void* w, const int32_t* offsets, void* y, int S,
                                             int K, int N, int E, void* stream) {
  return grouped_dev<EPI_F32>(x, w, offsets, y, S, K, N, E, as_stream(stream));
}

int tessera_gfx950_grouped_gemm_bf16(const void* x, const void* w, const int32_t* offsets, void* y, int S, int K,
                                     int N, int E) {
  return grouped_host<EPI_STORE16>(x, w, offsets, y, S, K, N, E);
}
int tessera_gfx950_grouped_gemm_bf16_f32(const void* x, const void* w, const int32_t* offsets, void* y, int S, int K,
                                         int N, int E) {
  return grouped_host<EPI_F32>(x, w, offsets, y, S, K, N, E);
}

int tessera_gfx950_grouped_gemm_f16_dev(const void* x, const void* w, const int32_t* offsets, void* y, int S, int K,
                                        int N, int E, void* stream) {
  return grouped_dev<EPI_STORE16, F16>(x, w, offsets, y, S, K, N, E, as_stream(stream));
}
int tessera_gfx950_grouped_gemm_f16_f32_dev(const void* x, const void* w, const int32_t* offsets, void* y, int S,
                                            int K, int N, int E, void* stream) {
  return grouped_dev<EPI_F32, F16>(x, w, offsets, y, S, K, N, E, as_stream(stream));
}
int tessera_gfx950_grouped_gemm_f16(const void* x, const void* w, const int32_t* offsets, void* y, int S, int K, int N,
                                    int E) {
  return grouped_host<EPI_STORE16, F16>(x, w, offsets, y, S, K, N, E);
}
int tessera_gfx950_grouped_gemm_f16_f32(const void* x, const void* w, const int32_t* offsets, void* y, int S, int K,
                                        int N, int E) {
  return grouped_host<EPI_F32, F16>(x, w, offsets, y, S, K, N, E);
}

int tessera_gfx950_scale_groups_f32_dev(const float* y, const int32_t* offsets, const float* scale, void* out,
                                        int out_bf16, int S, int N, int E, void* stream) {
  return scale_groups_dev(y, offsets, scale, out, out_bf16, S, N, E, as_stream(stream));
}
int tessera_gfx950_scale_groups_f32(const float* y, const int32_t* offsets, const float* scale, void* out, int out_bf16,
                                    int S, int N, int E) {
  if (S < 0 || N <= 0 || E <= 0 || !offsets || !scale || (S > 0 && (!y || !out))) return kBadShape;
  if (bad_offsets(offsets, E, S)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  if (S == 0) return kOk;
  const size_t ob = (size_t)S * N * (out_bf16 ? 2 : 4);
  DeviceScope scope;
  float* dy = static_cast<float*>(scope.alloc((size_t)S * N * 4, y));
  int32_t* dof = static_cast<int32_t*>(scope.alloc((size_t)(E + 1) * 4, offsets));
  float* dsc = static_cast<float*>(scope.alloc((size_t)E * 4, scale));
  void* dout = scope.alloc(ob);
  if (scope.failed()) return kDeviceFailed;
  int rc = scale_groups_dev(dy, dof, dsc, dout, out_bf16, S, N, E, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  return scope.download(out, dout, ob) ? kOk : kDeviceFailed;
}

int tessera_gfx950_moe_swiglu_block_bf16_dev(const void* x, const void* wg, const void* wu, const void* wd,
                                             const int32_t* offsets, void* y, void* hidden, int S, int K, int F,
                                             int N, int E, void* stream) {
  return swiglu_dev(x, wg, wu, wd, offsets, y, hidden, S, K, F, N, E, as_stream(stream));
}

int tessera_gfx950_moe_swiglu_block_bf16(const void* x, const void* wg, const void* wu, const void* wd,
                                         const int32_t* offsets, void* y, int S, int K, int F, int N, int E) {
  if (bad_grouped(S, K, N, E) || F <= 0 || !wg || !wu || !wd || !offsets || (S > 0 && (!x || !y))) return kBadShape;
  if (bad_offsets(offsets, E, S)) return kBadShape;
  if (probe_device() != kOk) return kNoDevice;
  if (S == 0) return kOk;
  DeviceScope scope;
  void* dx = scope.alloc((size_t)S * K * 2, x);
  void* dg = scope.alloc((size_t)E * K * F * 2, wg);
  void* du = scope.alloc((size_t)E * K * F * 2, wu);
  void* dd = scope.alloc((size_t)E * F * N * 2, wd);
  int32_t* dof = static_cast<int32_t*>(scope.alloc((size_t)(E + 1) * 4, offsets));
  void* dh = scope.alloc((size_t)S * F * 2);
  void* dy = scope.alloc((size_t)S * N * 2);
  if (scope.failed()) return kDeviceFailed;
  int rc = swiglu_dev(dx, dg, du, dd, dof, dy, dh, S, K, F, N, E, nullptr);
  if (rc != kOk) return rc;
  if (hipDeviceSynchronize() != hipSuccess) return kDeviceFailed;
  return scope.download(y, dy, (size_t)S * N * 2) ? kOk : kDeviceFailed;
}

int tessera_gfx950_moe_swiglu_block_gather_bf16_dev(const void* x, const int32_t* token_of_slot, const void* wg,
                                                    const void* wu, const void* wd, const int32_t* offsets, void* y,
                                                    void* hidden, int T, int S, int K, int F, int N, int E,
                                                    void* stream) {
  if (S > 0 && !token_of_slot) return kBadShape;       // (no slots: no map to read)
  return swiglu_dev(x, wg, wu, wd, offsets, y, hidden, S, K, F, N, E, as_stream(stream), token_of_slot, T);
}

int tessera_gfx950_moe_layer_bf16(const void* x, const float* router_logits, const void* wg, const void* wu,
                                  const void* wd, float* out, int T, int H, int F, int N, int E, int k,
                                  int normalize, int capacity, int32_t* token_of_slot, int32_t* expert_of_slot,
                                  float* combine_weights, int32_t* group_sizes, int32_t* group_offsets) {
  if (!router_logits) return kBadShape;
  return moe_layer_host(x, nullptr, router_logits, wg, wu, wd, out, T, H, F, N, E, k, normalize, capacity,
                        token_of_slot, expert_of_slot, combine_weights, group_sizes, group_offsets, nullptr);
}

int tessera_gfx950_moe_layer_router_bf16(const void* x, const void* w_router, const void* wg, const void* wu,
                                         const void* wd, float* out, int T, int H, int F, int N, int E, int k,
                                         int normalize, int capacity, int32_t* token_of_slot,
                                         int32_t* expert_of_slot, float* combine_weights, int32_t* group_sizes,
                                         int32_t* group_offsets, float* router_logits_out) {
  if (!w_router) return kBadShape;
  return moe_layer_host(x, w_router, nullptr, wg, wu, wd, out, T, H, F, N, E, k, normalize, capacity,
                        token_of_slot, expert_of_slot, combine_weights, group_sizes, group_offsets,
                        router_logits_out);
}

int tessera_gfx950_moe_layer_workspace_bytes(int T, int H, int F, int N, int E, int k, size_t* bytes) {
  if (bad_layer(T, H, F, N, E, k) || !bytes) return kBadShape;
  *bytes = layer_scratch(T, F, N, E, k).total;
  return kOk;
}

int tessera_gfx950_moe_layer_bf16_dev(const void* x, const void* w_router, const float* router_logits,
                                      const void* wg, const void* wu, const void* wd, float* out,
                                      void* workspace, size_t workspace_bytes, int T, int H, int F, int N, int E,
                                      int k, int normalize, int capacity, int32_t* token_of_slot,
                                      int32_t* expert_of_slot, float* combine_weights, int32_t* group_sizes,
                                      int32_t* group_offsets, int32_t* num_slots, void* stream) {
  return moe_layer_dev(x, w_router, router_logits, wg, wu, wd, out, workspace, workspace_bytes, T, H, F, N, E, k,
                       normalize, capacity, token_of_slot, expert_of_slot, combine_weights, group_sizes,
                       group_offsets, num_slots, as_stream(stream));
}

}  // extern "C"
