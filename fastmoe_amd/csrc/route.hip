// Routing metadata on gfx950: per-expert histogram, exclusive scan and stable
// position assignment (a counting sort of the routed slots by expert), plus
// the capacity kernels that share its ranks.
//
// Three launches on the caller's stream:
//   hist   one block per 2048 slots, LDS-privatised counters  -> block_hist[b][e]
//   scan   one block: per-expert exclusive scan over the blocks, then a
//          wave64 scan over the experts                       -> seg_off, counts
//   place  one block per 2048 slots: per-wave LDS counters give every slot its
//          rank among the earlier slots of the same expert    -> pos / inv / mask
// No arrival-order atomics touch the result, so positions and drop masks are
// the ones a sequential sweep over the slots would produce.  Up to 4096 slots
// and 512 experts fmoe_route runs the same three steps as ONE workgroup
// (route_single_kernel): one launch instead of three.
//
// Semantics follow cuda/local_exchange.cuh:5-16,36-69 and
// cuda/balancing.cuh:5-21,32-45 of the reference.
#include "common.h"

namespace fmoe {

constexpr int kRouteThreads = 256;
constexpr int kRouteWaves = kRouteThreads / kWave;
constexpr int kRowsPerWave = 8;                               // 64-slot rows
constexpr int kRouteChunk = kRouteThreads * kRowsPerWave;     // slots per block
constexpr int kScanThreads = 1024;

enum { MODE_ROUTE = 0, MODE_ASSIGN = 1, MODE_PRUNE = 2 };

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// ---------------------------------------------------------------- histogram
__global__ __launch_bounds__(kRouteThreads) void route_hist_kernel(
    const int64_t* __restrict__ gate, int64_t n, int n_expert,
    int32_t* __restrict__ block_hist, int32_t* __restrict__ direct_count) {
  extern __shared__ int32_t lds_hist[];
  for (int e = threadIdx.x; e < n_expert; e += kRouteThreads) lds_hist[e] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kRouteChunk;
#pragma unroll
  for (int it = 0; it < kRowsPerWave; ++it) {
    const int64_t i = base + it * kRouteThreads + threadIdx.x;
    if (i < n) {
      const int64_t g = gate[i];
      if (g >= 0 && g < n_expert) atomicAdd(&lds_hist[(int)g], 1);
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_expert; e += kRouteThreads) {
    const int32_t c = lds_hist[e];
    if (block_hist) block_hist[(int64_t)blockIdx.x * n_expert + e] = c;
    if (direct_count && c) atomicAdd(&direct_count[e], c);
  }
}

// Expert sets too large for LDS: plain global atomics (integer, exact).
__global__ __launch_bounds__(kRouteThreads) void route_hist_global_kernel(
    const int64_t* __restrict__ gate, int64_t n, int64_t n_expert,
    int32_t* __restrict__ count) {
  const int64_t i = (int64_t)blockIdx.x * kRouteThreads + threadIdx.x;
  if (i < n) {
    const int64_t g = gate[i];
    if (g >= 0 && g < n_expert) atomicAdd(&count[g], 1);
  }
}

// --------------------------------------------------------------------- scan
constexpr int kScanChunk = 8;   // per-block counters a thread loads before it sums them
template <int MODE>
__global__ __launch_bounds__(kScanThreads) void route_scan_kernel(
    int32_t* __restrict__ block_hist, int n_blocks, int n_expert,
    int64_t* __restrict__ count64, int32_t* __restrict__ seg_off,
    int32_t* __restrict__ cum_or_cap, int32_t* __restrict__ cap_copy) {
  extern __shared__ int32_t lds_scan[];
  int32_t* cnt = lds_scan;                  // [E]
  int32_t* off = lds_scan + n_expert;       // [E+1]
  // exclusive scan over the blocks, one expert per thread
  // (kScanChunk loads in flight at a time: one memory round trip per chunk
  // instead of one per block)
  for (int e = threadIdx.x; e < n_expert; e += kScanThreads) {
    int32_t run = 0;
    for (int b0 = 0; b0 < n_blocks; b0 += kScanChunk) {
      int32_t v[kScanChunk];
#pragma unroll
      for (int u = 0; u < kScanChunk; ++u)
        v[u] = b0 + u < n_blocks ? block_hist[(int64_t)(b0 + u) * n_expert + e] : 0;
#pragma unroll
      for (int u = 0; u < kScanChunk; ++u) {
        if (b0 + u < n_blocks) block_hist[(int64_t)(b0 + u) * n_expert + e] = run;
        run += v[u];
      }
    }
    cnt[e] = run;
  }
  __syncthreads();
  if (MODE == MODE_ROUTE) {
    // exclusive scan over the experts by wave 0, 64 experts per step
    if (threadIdx.x < kWave) {
      const int lane = threadIdx.x;
      int32_t carry = 0;
      for (int base = 0; base < n_expert; base += kWave) {
        const int e = base + lane;
        const int32_t v = e < n_expert ? cnt[e] : 0;
        int32_t incl = v;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
          const int32_t t = __shfl_up(incl, d, kWave);
          if (lane >= d) incl += t;
        }
        if (e < n_expert) off[e] = carry + incl - v;
        carry += __shfl(incl, kWave - 1, kWave);
      }
      if (lane == 0) off[n_expert] = carry;
    }
    __syncthreads();
  }
  for (int e = threadIdx.x; e < n_expert; e += kScanThreads) {
    const int32_t c = cnt[e];
    if (MODE == MODE_ROUTE) {
      if (count64) count64[e] = c;
      seg_off[e] = off[e];
    } else if (MODE == MODE_ASSIGN) {
      // inclusive cumulative count in, exclusive one out
      cum_or_cap[e] = cum_or_cap[e] - c;
    } else {
      const int32_t cap = cum_or_cap[e];
      cap_copy[e] = cap;
      cum_or_cap[e] = cap - c;
    }
  }
  if (MODE == MODE_ROUTE && threadIdx.x == 0) seg_off[n_expert] = off[n_expert];
}

// -------------------------------------------------------------------- place
// MODE_ROUTE / MODE_ASSIGN: pos[base_off[e] + rank] = slot, inv[slot] = row.
// MODE_PRUNE: new_gate[slot] = rank < cap[e] ? e : -1.
template <int MODE>
__global__ __launch_bounds__(kRouteThreads) void route_place_kernel(
    const int64_t* __restrict__ gate, int64_t n, int n_expert,
    const int32_t* __restrict__ block_hist, const int32_t* __restrict__ base_off,
    int64_t* __restrict__ pos, int32_t* __restrict__ inv,
    int64_t* __restrict__ new_gate, const int32_t* __restrict__ cap) {
  extern __shared__ int32_t wave_cnt[];  // [kRouteWaves][E]
  const int w = threadIdx.x / kWave;
  const int lane = lane_id();
  for (int x = threadIdx.x; x < kRouteWaves * n_expert; x += kRouteThreads)
    wave_cnt[x] = 0;
  __syncthreads();

  const int64_t base = (int64_t)blockIdx.x * kRouteChunk;
  int32_t keys[kRowsPerWave];
#pragma unroll
  for (int s = 0; s < kRowsPerWave; ++s) {
    const int64_t i = base + (int64_t)(w * kRowsPerWave + s) * kWave + lane;
    int32_t key = -1;
    if (i < n) {
      const int64_t g = gate[i];
      if (g >= 0 && g < n_expert) key = (int32_t)g;
    }
    keys[s] = key;
    if (key >= 0) atomicAdd(&wave_cnt[w * n_expert + key], 1);
  }
  __syncthreads();
  // per-expert start of every wave: block base (+ segment start) + earlier waves
  for (int e = threadIdx.x; e < n_expert; e += kRouteThreads) {
    int32_t run = block_hist[(int64_t)blockIdx.x * n_expert + e];
    if (MODE != MODE_PRUNE) run += base_off[e];
#pragma unroll
    for (int w2 = 0; w2 < kRouteWaves; ++w2) {
      const int32_t t = wave_cnt[w2 * n_expert + e];
      wave_cnt[w2 * n_expert + e] = run;
      run += t;
    }
  }
  __syncthreads();

  const uint64_t lt_mask = ((uint64_t)1 << lane) - 1;
  const int key_bits = 32 - __clz(max(n_expert - 1, 1));
#pragma unroll
  for (int s = 0; s < kRowsPerWave; ++s) {
    const int64_t i = base + (int64_t)(w * kRowsPerWave + s) * kWave + lane;
    const int32_t key = keys[s];
    const bool valid = key >= 0;
    // lanes of this row with the same key: one ballot per bit of the key
    uint64_t same = __ballot(valid);
    for (int bit = 0; bit < key_bits; ++bit) {
      const uint64_t vote = __ballot(valid && ((key >> bit) & 1));
      same &= ((key >> bit) & 1) ? vote : ~vote;
    }
    const int rank = __popcll(same & lt_mask);
    const int cnt = __popcll(same);
    const bool first = valid && (same & lt_mask) == 0;
    int32_t p = 0;
    if (valid) p = wave_cnt[w * n_expert + key] + rank;
    // every lane of the wave has read its counter before the leader of each
    // expert advances it (one wave issues its LDS operations in order)
    if (valid && first) wave_cnt[w * n_expert + key] = p + cnt;
    if (MODE == MODE_PRUNE) {
      if (i < n) new_gate[i] = valid ? (p < cap[key] ? (int64_t)key : (int64_t)-1)
                                     : gate[i];
    } else {
      if (valid) pos[p] = i;
      if (inv != nullptr && i < n) inv[i] = valid ? p : -1;
    }
  }
}

// ------------------------------------------------------------- single launch
// The three steps above in ONE workgroup of 16 waves, for problems small enough
// that three launches (and their gaps) cost more than the work: up to 4096 slots
// and 512 experts (512 tokens, top-2: 22 -> 12 us per call; from 16384 slots on one
// CU alone takes longer over the slots than three launches that use all of them:
// 25 vs 19 us).  Wave w takes the w-th sixteenth of the 64-slot rows, so the
// order of slots inside an expert is the ascending one of the three-kernel path
// and the results are the same bit for bit.  A wave loads all its rows (at most
// ROWS, kept in registers) in one go: with a load per loop trip the memory
// latency of the dependent trips adds up.
constexpr int kSingleThreads = 1024;
constexpr int kSingleWaves = kSingleThreads / kWave;
constexpr int kSingleMaxSlots = 4096;
constexpr int kSingleRows = kSingleMaxSlots / kSingleThreads;   // 64-slot rows per wave
constexpr int kSingleMaxExperts = 512;

template <int ROWS>
__global__ __launch_bounds__(kSingleThreads) void route_single_kernel(
    const int64_t* __restrict__ gate, int64_t n, int n_expert, int64_t* __restrict__ count64,
    int32_t* __restrict__ seg_off, int64_t* __restrict__ pos, int32_t* __restrict__ inv) {
  extern __shared__ int32_t lds_single[];
  int32_t* wave_cnt = lds_single;                            // [kSingleWaves][E]
  int32_t* cnt = lds_single + kSingleWaves * n_expert;       // [E]
  int32_t* off = cnt + n_expert;                             // [E+1]
  const int w = threadIdx.x / kWave;
  const int lane = lane_id();
  for (int x = threadIdx.x; x < kSingleWaves * n_expert; x += kSingleThreads) wave_cnt[x] = 0;
  __syncthreads();

  const int rows = (int)((n + kWave - 1) / kWave);
  const int rows_per_wave = (rows + kSingleWaves - 1) / kSingleWaves;
  const int row_lo = w * rows_per_wave, row_hi = min(rows, row_lo + rows_per_wave);
  int32_t keys[ROWS];
#pragma unroll
  for (int u = 0; u < ROWS; ++u) {
    const int64_t i = (int64_t)(row_lo + u) * kWave + lane;
    int32_t key = -1;
    if (row_lo + u < row_hi && i < n) {
      const int64_t g = gate[i];
      if (g >= 0 && g < n_expert) key = (int32_t)g;
    }
    keys[u] = key;
  }
#pragma unroll
  for (int u = 0; u < ROWS; ++u)
    if (keys[u] >= 0) atomicAdd(&wave_cnt[w * n_expert + keys[u]], 1);
  __syncthreads();
  // per expert: its total, and where every wave's share starts inside its segment
  for (int e = threadIdx.x; e < n_expert; e += kSingleThreads) {
    int32_t run = 0;
#pragma unroll
    for (int w2 = 0; w2 < kSingleWaves; ++w2) {
      const int32_t t = wave_cnt[w2 * n_expert + e];
      wave_cnt[w2 * n_expert + e] = run;
      run += t;
    }
    cnt[e] = run;
  }
  __syncthreads();
  if (threadIdx.x < kWave) {   // exclusive scan over the experts, 64 per step
    int32_t carry = 0;
    for (int base = 0; base < n_expert; base += kWave) {
      const int e = base + lane;
      const int32_t v = e < n_expert ? cnt[e] : 0;
      int32_t incl = v;
#pragma unroll
      for (int d = 1; d < kWave; d <<= 1) {
        const int32_t t = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += t;
      }
      if (e < n_expert) off[e] = carry + incl - v;
      carry += __shfl(incl, kWave - 1, kWave);
    }
    if (lane == 0) off[n_expert] = carry;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_expert; e += kSingleThreads) {
    const int32_t o = off[e];
#pragma unroll
    for (int w2 = 0; w2 < kSingleWaves; ++w2) wave_cnt[w2 * n_expert + e] += o;
    if (count64) count64[e] = cnt[e];
    seg_off[e] = o;
  }
  if (threadIdx.x == 0) seg_off[n_expert] = off[n_expert];
  __syncthreads();

  const uint64_t lt_mask = ((uint64_t)1 << lane) - 1;
  const int key_bits = 32 - __clz(max(n_expert - 1, 1));
#pragma unroll
  for (int u = 0; u < ROWS; ++u) {
    if (row_lo + u >= row_hi) break;   // the same for the whole wave
    const int64_t i = (int64_t)(row_lo + u) * kWave + lane;
    const int32_t key = keys[u];
    const bool valid = key >= 0;
    uint64_t same = __ballot(valid);
    for (int bit = 0; bit < key_bits; ++bit) {
      const uint64_t vote = __ballot(valid && ((key >> bit) & 1));
      same &= ((key >> bit) & 1) ? vote : ~vote;
    }
    const int rank = __popcll(same & lt_mask);
    const bool first = valid && (same & lt_mask) == 0;
    int32_t p = 0;
    if (valid) p = wave_cnt[w * n_expert + key] + rank;
    // every lane has read its counter before the leader of each expert advances it
    if (valid && first) wave_cnt[w * n_expert + key] = p + __popcll(same);
    if (valid) pos[p] = i;
    if (inv != nullptr && i < n) inv[i] = valid ? p : -1;
  }
}

// ------------------------------------------------------------------- limit
// One thread per expert walks the workers in ascending order.
__global__ __launch_bounds__(256) void limit_by_capacity_kernel(
    const int64_t* __restrict__ ec, int32_t* __restrict__ cap,
    int64_t* __restrict__ eca, int64_t n_expert, int64_t n_worker) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n_expert) return;
  int32_t left = cap[e];
  for (int64_t w = 0; w < n_worker; ++w) {
    const int32_t proposal = (int32_t)ec[w * n_expert + e];
    int64_t grant;
    if (left >= proposal) grant = proposal;
    else if (left >= 0) grant = left;
    else grant = 0;
    eca[w * n_expert + e] = grant;
    left -= proposal;
  }
  cap[e] = left;
}

// --------------------------------------------------------------- host side
// Scratch of the entry point that allocates nothing (fmoe_route_static): the
// per-block histograms live in this array instead of a caller's workspace.
// Every GPU the library runs on holds its own copy until the process ends.
constexpr int64_t kStaticScratchBytes = FMOE_ROUTE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxRouteDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxRouteDevices];   // device address of `scratch`, per GPU

// Device address of the current GPU's copy of `scratch` (looked up once per GPU).
static int static_scratch(void** out) {
  int dev = 0;
  FMOE_HIP_CHECK(hipGetDevice(&dev));
  FMOE_REQUIRE(dev >= 0 && dev < kMaxRouteDevices, FMOE_ERR_UNSUPPORTED,
               "route_static: device %d", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    FMOE_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    FMOE_REQUIRE(p != nullptr, FMOE_ERR_HIP, "route_static: scratch has no device address");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return FMOE_OK;
}

// The routing share of fmoe_init(): looks up the current GPU's copy of the static
// buffer, so that fmoe_route_static has no runtime query left to make.
int route_static_init() {
  void* p = nullptr;
  return static_scratch(&p);
}

struct RouteWs {
  int32_t* block_hist;
  int32_t* cap_copy;
  int n_blocks;
};

static int64_t route_ws_bytes(int64_t numel, int32_t n_expert) {
  const int64_t n_blocks = (numel + kRouteChunk - 1) / kRouteChunk;
  int64_t ints = n_blocks * n_expert + n_expert + 64;
  return ((ints * 4 + 255) / 256) * 256;
}

static int carve_ws(void* ws, int64_t ws_bytes, int64_t numel, int32_t n_expert,
                    RouteWs* out) {
  const int64_t need = route_ws_bytes(numel, n_expert);
  FMOE_REQUIRE(ws != nullptr && ws_bytes >= need, FMOE_ERR_WORKSPACE,
               "routing workspace too small: need %lld bytes, got %lld",
               (long long)need, (long long)ws_bytes);
  out->n_blocks = (int)((numel + kRouteChunk - 1) / kRouteChunk);
  out->block_hist = (int32_t*)ws;
  out->cap_copy = out->block_hist + (int64_t)out->n_blocks * n_expert;
  return FMOE_OK;
}

static int check_route_args(int64_t numel, int64_t n_expert) {
  FMOE_REQUIRE(numel >= 0, FMOE_ERR_INVALID, "numel must be >= 0");
  FMOE_REQUIRE(numel < ((int64_t)1 << 31), FMOE_ERR_UNSUPPORTED,
               "numel %lld does not fit the int32 positions", (long long)numel);
  FMOE_REQUIRE(n_expert >= 1, FMOE_ERR_INVALID, "n_expert must be >= 1");
  FMOE_REQUIRE(n_expert <= FMOE_MAX_EXPERTS, FMOE_ERR_UNSUPPORTED,
               "n_expert %lld exceeds FMOE_MAX_EXPERTS (%d)",
               (long long)n_expert, FMOE_MAX_EXPERTS);
  return FMOE_OK;
}

}  // namespace fmoe

using namespace fmoe;

extern "C" int fmoe_expert_count(const int64_t* gate_idx, int64_t numel,
                                 int32_t* expert_count, int32_t n_expert,
                                 void* stream) {
  FMOE_REQUIRE(numel >= 0 && n_expert >= 1, FMOE_ERR_INVALID,
               "expert_count: bad sizes numel=%lld n_expert=%d",
               (long long)numel, n_expert);
  if (numel == 0) return FMOE_OK;
  FMOE_REQUIRE(gate_idx && expert_count, FMOE_ERR_INVALID,
               "expert_count: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if (n_expert <= FMOE_MAX_EXPERTS) {
    const int blocks = ceil_div(numel, kRouteChunk);
    hipLaunchKernelGGL(route_hist_kernel, dim3(blocks), dim3(kRouteThreads),
                       n_expert * sizeof(int32_t), s, gate_idx, numel,
                       (int)n_expert, (int32_t*)nullptr, expert_count);
  } else {
    const int blocks = ceil_div(numel, kRouteThreads);
    hipLaunchKernelGGL(route_hist_global_kernel, dim3(blocks),
                       dim3(kRouteThreads), 0, s, gate_idx, numel,
                       (int64_t)n_expert, expert_count);
  }
  FMOE_LAUNCH_CHECK("expert_count");
  return FMOE_OK;
}

extern "C" int64_t fmoe_route_workspace_bytes(int64_t numel, int32_t n_expert) {
  if (numel < 0 || n_expert < 1) return FMOE_ERR_INVALID;
  return route_ws_bytes(numel, n_expert);
}

// `single_launch`: small problems may run as one workgroup without the workspace.
static int route_impl(const int64_t* gate, int64_t numel, int32_t n_expert,
                      int64_t* count64, int32_t* seg_off, int64_t* pos,
                      int32_t* inv, void* workspace, int64_t workspace_bytes,
                      void* stream, bool single_launch) {
  int rc = check_route_args(numel, n_expert);
  if (rc) return rc;
  FMOE_REQUIRE(seg_off != nullptr, FMOE_ERR_INVALID, "route: seg_off is null");
  FMOE_REQUIRE(numel == 0 || (gate && pos), FMOE_ERR_INVALID,
               "route: null gate/pos");
  RouteWs ws;
  rc = carve_ws(workspace, workspace_bytes, numel, n_expert, &ws);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (single_launch && numel <= kSingleMaxSlots && n_expert <= kSingleMaxExperts) {
    const size_t lds = ((kSingleWaves + 2) * n_expert + 1) * sizeof(int32_t);
    hipLaunchKernelGGL(route_single_kernel<kSingleRows>, dim3(1), dim3(kSingleThreads), lds, s,
                       gate, numel, (int)n_expert, count64, seg_off, pos, inv);
    FMOE_LAUNCH_CHECK("route_single");
    return FMOE_OK;
  }
  if (ws.n_blocks > 0) {
    hipLaunchKernelGGL(route_hist_kernel, dim3(ws.n_blocks), dim3(kRouteThreads),
                       n_expert * sizeof(int32_t), s, gate, numel, (int)n_expert,
                       ws.block_hist, (int32_t*)nullptr);
    FMOE_LAUNCH_CHECK("route_hist");
  }
  hipLaunchKernelGGL(route_scan_kernel<MODE_ROUTE>, dim3(1), dim3(kScanThreads),
                     (2 * n_expert + 1) * sizeof(int32_t), s, ws.block_hist,
                     ws.n_blocks, (int)n_expert, count64, seg_off,
                     (int32_t*)nullptr, (int32_t*)nullptr);
  FMOE_LAUNCH_CHECK("route_scan");
  if (ws.n_blocks > 0) {
    hipLaunchKernelGGL(route_place_kernel<MODE_ROUTE>, dim3(ws.n_blocks),
                       dim3(kRouteThreads),
                       kRouteWaves * n_expert * sizeof(int32_t), s, gate, numel,
                       (int)n_expert, ws.block_hist, seg_off, pos, inv,
                       (int64_t*)nullptr, (const int32_t*)nullptr);
    FMOE_LAUNCH_CHECK("route_place");
  }
  return FMOE_OK;
}

extern "C" int fmoe_route(const int64_t* gate, int64_t numel, int32_t n_expert,
                          int64_t* count64, int32_t* seg_off, int64_t* pos,
                          int32_t* inv, void* workspace, int64_t workspace_bytes,
                          void* stream) {
  return route_impl(gate, numel, n_expert, count64, seg_off, pos, inv, workspace,
                    workspace_bytes, stream, true);
}

extern "C" int fmoe_route_static(const int64_t* gate, int64_t numel, int32_t n_expert,
                                 int64_t* count64, int32_t* seg_off, int64_t* pos,
                                 int32_t* inv, void* stream) {
  int rc = check_route_args(numel, n_expert);
  if (rc) return rc;
  const int64_t need = route_ws_bytes(numel, n_expert);
  FMOE_REQUIRE(need <= kStaticScratchBytes, FMOE_ERR_WORKSPACE,
               "route_static: %lld slots x %d experts need %lld bytes of scratch, the "
               "built-in buffer holds %lld; use fmoe_route with a workspace",
               (long long)numel, n_expert, (long long)need, (long long)kStaticScratchBytes);
  void* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc) return rc;
  // every block of the histogram kernel overwrites its whole row of the table
  // before anything reads it, so what the last call left behind needs no clearing
  // (always the three-kernel form: it is the one that uses the scratch buffer)
  return route_impl(gate, numel, n_expert, count64, seg_off, pos, inv, ws, kStaticScratchBytes,
                    stream, false);
}

extern "C" int fmoe_assign_pos(int32_t* cum_count, const int64_t* gate,
                               int64_t* pos, int64_t numel, int32_t n_expert,
                               void* workspace, int64_t workspace_bytes,
                               void* stream) {
  int rc = check_route_args(numel, n_expert);
  if (rc) return rc;
  if (numel == 0) return FMOE_OK;
  FMOE_REQUIRE(cum_count && gate && pos, FMOE_ERR_INVALID,
               "assign_pos: null pointer");
  RouteWs ws;
  rc = carve_ws(workspace, workspace_bytes, numel, n_expert, &ws);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(route_hist_kernel, dim3(ws.n_blocks), dim3(kRouteThreads),
                     n_expert * sizeof(int32_t), s, gate, numel, (int)n_expert,
                     ws.block_hist, (int32_t*)nullptr);
  FMOE_LAUNCH_CHECK("route_hist");
  hipLaunchKernelGGL(route_scan_kernel<MODE_ASSIGN>, dim3(1), dim3(kScanThreads),
                     (2 * n_expert + 1) * sizeof(int32_t), s, ws.block_hist,
                     ws.n_blocks, (int)n_expert, (int64_t*)nullptr,
                     (int32_t*)nullptr, cum_count, (int32_t*)nullptr);
  FMOE_LAUNCH_CHECK("route_scan");
  hipLaunchKernelGGL(route_place_kernel<MODE_ASSIGN>, dim3(ws.n_blocks),
                     dim3(kRouteThreads),
                     kRouteWaves * n_expert * sizeof(int32_t), s, gate, numel,
                     (int)n_expert, ws.block_hist, cum_count, pos,
                     (int32_t*)nullptr, (int64_t*)nullptr,
                     (const int32_t*)nullptr);
  FMOE_LAUNCH_CHECK("route_place");
  return FMOE_OK;
}

extern "C" int fmoe_limit_by_capacity(const int64_t* ec, int32_t* cap,
                                      int64_t* eca, int64_t n_expert,
                                      int64_t n_worker, void* stream) {
  FMOE_REQUIRE(n_expert >= 0 && n_worker >= 0, FMOE_ERR_INVALID,
               "limit_by_capacity: negative size");
  if (n_expert == 0 || n_worker == 0) return FMOE_OK;
  FMOE_REQUIRE(ec && cap && eca, FMOE_ERR_INVALID,
               "limit_by_capacity: null pointer");
  hipLaunchKernelGGL(limit_by_capacity_kernel, dim3(ceil_div(n_expert, 256)),
                     dim3(256), 0, (hipStream_t)stream, ec, cap, eca, n_expert,
                     n_worker);
  FMOE_LAUNCH_CHECK("limit_by_capacity");
  return FMOE_OK;
}

extern "C" int fmoe_prune_gate_by_capacity(const int64_t* gate_idx,
                                           int64_t* new_gate_idx, int32_t* ec,
                                           int64_t numel, int64_t n_expert,
                                           int64_t n_worker, void* workspace,
                                           int64_t workspace_bytes,
                                           void* stream) {
  FMOE_REQUIRE(n_expert >= 1 && n_worker >= 1, FMOE_ERR_INVALID,
               "prune_gate_by_capacity: bad expert/worker count");
  const int64_t bins = n_expert * n_worker;
  int rc = check_route_args(numel, bins);
  if (rc) return rc;
  if (numel == 0) return FMOE_OK;
  FMOE_REQUIRE(gate_idx && new_gate_idx && ec, FMOE_ERR_INVALID,
               "prune_gate_by_capacity: null pointer");
  RouteWs ws;
  rc = carve_ws(workspace, workspace_bytes, numel, (int32_t)bins, &ws);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  const int E = (int)bins;
  hipLaunchKernelGGL(route_hist_kernel, dim3(ws.n_blocks), dim3(kRouteThreads),
                     E * sizeof(int32_t), s, gate_idx, numel, E, ws.block_hist,
                     (int32_t*)nullptr);
  FMOE_LAUNCH_CHECK("route_hist");
  hipLaunchKernelGGL(route_scan_kernel<MODE_PRUNE>, dim3(1), dim3(kScanThreads),
                     (2 * E + 1) * sizeof(int32_t), s, ws.block_hist, ws.n_blocks,
                     E, (int64_t*)nullptr, (int32_t*)nullptr, ec, ws.cap_copy);
  FMOE_LAUNCH_CHECK("route_scan");
  hipLaunchKernelGGL(route_place_kernel<MODE_PRUNE>, dim3(ws.n_blocks),
                     dim3(kRouteThreads), kRouteWaves * E * sizeof(int32_t), s,
                     gate_idx, numel, E, ws.block_hist, (const int32_t*)nullptr,
                     (int64_t*)nullptr, (int32_t*)nullptr, new_gate_idx,
                     ws.cap_copy);
  FMOE_LAUNCH_CHECK("route_place");
  return FMOE_OK;
}
