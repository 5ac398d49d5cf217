// Token dispatch: stable counting sort of the flat expert ids.
// Replaces the E boolean-mask gathers of MOEFeedForwardSwiGLU.forward
// (/root/reference/comfy/ldm/hidream/model.py:313-318), which pick, for expert i,
// the flat slots p = 2t+s with topk_idx[p] == i in ascending p.
//
// Two launches over chunks of 256 flat slots (2048 above 2^16 slots):
//   count:   per-chunk expert histogram from wave ballots        -> chunk_counts[chunk][E]
//   scatter: every block sums the histograms of the chunks before it (and all of
//            them for the global counts/offsets), then ranks its own slots with
//            ballot prefix counts inside a wave and an LDS scan across waves, and
//            writes perm / inv_perm.
// No atomics, so the result does not depend on scheduling.
// Traffic: 2T*4 bytes read twice, 2*2T*4 bytes written.
// Inside the one-call layer the gate kernel does the counting (its blocks own contiguous token ranges and leave
// one histogram each) and only the scatter launch remains.
#include <mutex>

#include "common.h"

namespace {

constexpr int THREADS = 256;
constexpr int WAVES = THREADS / 64;
// A block handles THREADS * ITEMS flat slots. Few items per block keep the serial part of a block short (this
// stage is latency bound at the sizes of one layer); many items bound the number of per-chunk histograms every
// block has to sum at very large T.
constexpr int ITEMS_SMALL = 1, ITEMS_LARGE = 8;
constexpr int SMALL_MAX_SLOTS = 1 << 16;
inline int items_for(size_t n) { return n <= (size_t)SMALL_MAX_SLOTS ? ITEMS_SMALL : ITEMS_LARGE; }

template <int ITEMS>
__global__ __launch_bounds__(THREADS) void dispatch_count_kernel(const int32_t* __restrict__ flat, int n,
                                                                 int E, int32_t* __restrict__ chunk_counts) {
  __shared__ int32_t wave_cnt[WAVES][HDMOE_MAX_EXPERTS];
  constexpr int CHUNK = THREADS * ITEMS;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int base = blockIdx.x * CHUNK;
  int32_t cnt = 0;  // lane e (< E) of each wave accumulates the wave's count for expert e
  for (int it = 0; it < ITEMS; ++it) {
    const int p = base + it * THREADS + threadIdx.x;
    const int e = p < n ? flat[p] : -1;  // ids outside [0,E) match no ballot and are dropped
    for (int q = 0; q < E; ++q) {
      const unsigned long long m = __ballot(e == q);
      if (lane == q) cnt += __popcll(m);
    }
  }
  if (lane < E) wave_cnt[wave][lane] = cnt;
  __syncthreads();
  if (threadIdx.x < E) {
    int32_t s = 0;
    for (int w = 0; w < WAVES; ++w) s += wave_cnt[w][threadIdx.x];
    chunk_counts[(size_t)blockIdx.x * E + threadIdx.x] = s;
  }
}

template <int ITEMS>
__global__ __launch_bounds__(THREADS) void dispatch_scatter_kernel(
    const int32_t* __restrict__ flat, int n, int E, int nhist, int hist_per_chunk, int chunk_slots,
    const int32_t* __restrict__ chunk_counts, int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
    int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm) {
  __shared__ int32_t total[HDMOE_MAX_EXPERTS];
  __shared__ int32_t before[HDMOE_MAX_EXPERTS];
  __shared__ int32_t cursor[HDMOE_MAX_EXPERTS];  // next sorted row per expert for this block
  __shared__ int32_t wave_cnt[WAVES][HDMOE_MAX_EXPERTS];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  // per expert: rows in earlier chunks, rows overall. Wave w handles experts w, w+WAVES, ... The histograms may be
  // finer than the chunks (hist_per_chunk consecutive ones make up a chunk: those of the gate kernel's blocks).
  const int first_mine = (int)blockIdx.x * hist_per_chunk;
  for (int e = wave; e < E; e += WAVES) {
    int32_t tot = 0, bef = 0;
    for (int c = lane; c < nhist; c += 64) {
      const int32_t v = chunk_counts[(size_t)c * E + e];
      tot += v;
      if (c < first_mine) bef += v;
    }
    for (int off = 32; off >= 1; off >>= 1) {
      tot += __shfl_xor(tot, off, 64);
      bef += __shfl_xor(bef, off, 64);
    }
    if (lane == 0) { total[e] = tot; before[e] = bef; }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t run = 0;
    for (int e = 0; e < E; ++e) {
      cursor[e] = run + before[e];
      if (blockIdx.x == 0) { counts[e] = total[e]; offsets[e] = run; }
      run += total[e];
    }
    if (blockIdx.x == 0) offsets[E] = run;
  }
  __syncthreads();

  // a block's chunk: chunk_slots flat slots (at most THREADS * ITEMS; fewer when the histograms' granularity asks)
  const int base = blockIdx.x * chunk_slots;
  const int end = min(n, base + chunk_slots);
  const unsigned long long lt = (1ull << lane) - 1ull;
  for (int it = 0; it < ITEMS; ++it) {
    const int p = base + it * THREADS + threadIdx.x;
    int e = p < end ? flat[p] : -1;
    if (e >= E) e = -1;  // never index the LDS tables with a bad id
    int32_t rank = 0;   // slots of my expert in lower lanes of my wave
    int32_t mine = 0;   // lane q holds the wave's count for expert q
    for (int q = 0; q < E; ++q) {
      const unsigned long long m = __ballot(e == q);
      if (e == q) rank = __popcll(m & lt);
      if (lane == q) mine = __popcll(m);
    }
    if (lane < E) wave_cnt[wave][lane] = mine;
    __syncthreads();
    if (e >= 0) {
      int32_t pos = cursor[e] + rank;
      for (int w = 0; w < wave; ++w) pos += wave_cnt[w][e];
      perm[pos] = p;
      inv_perm[p] = pos;
    }
    __syncthreads();
    if (threadIdx.x < E) {
      int32_t s = 0;
      for (int w = 0; w < WAVES; ++w) s += wave_cnt[w][threadIdx.x];
      cursor[threadIdx.x] += s;
    }
    __syncthreads();
  }
}

}  // namespace

extern "C" size_t hdmoe_dispatch_workspace_bytes(int T, int E) {
  if (T < 0 || E < 1) return 0;
  const size_t n = (size_t)T * HDMOE_TOPK;
  const size_t chunk = (size_t)THREADS * items_for(n);
  const size_t nchunks = (n + chunk - 1) / chunk;
  return hdmoe_align_up((nchunks > 0 ? nchunks : 1) * (size_t)E * sizeof(int32_t), 256);
}

namespace {

// Shared by the two entry points: argument checks and the two launches; cc holds the per-chunk histograms.
int dispatch_enqueue(const char* what, const int32_t* topk_idx, int T, int E, int32_t* counts, int32_t* offsets,
                     int32_t* perm, int32_t* inv_perm, int32_t* cc, hipStream_t s) {
  const int n = T * HDMOE_TOPK;
  const int items = items_for((size_t)n);
  const int chunk = THREADS * items;
  int nchunks = (n + chunk - 1) / chunk;
  if (nchunks < 1) nchunks = 1;  // T == 0 still writes counts = 0 and offsets = 0
  if (items == ITEMS_SMALL) {
    hipLaunchKernelGGL(dispatch_count_kernel<ITEMS_SMALL>, dim3(nchunks), dim3(THREADS), 0, s, topk_idx, n, E, cc);
    hipLaunchKernelGGL(dispatch_scatter_kernel<ITEMS_SMALL>, dim3(nchunks), dim3(THREADS), 0, s, topk_idx, n, E,
                       nchunks, 1, chunk, cc, counts, offsets, perm, inv_perm);
  } else {
    hipLaunchKernelGGL(dispatch_count_kernel<ITEMS_LARGE>, dim3(nchunks), dim3(THREADS), 0, s, topk_idx, n, E, cc);
    hipLaunchKernelGGL(dispatch_scatter_kernel<ITEMS_LARGE>, dim3(nchunks), dim3(THREADS), 0, s, topk_idx, n, E,
                       nchunks, 1, chunk, cc, counts, offsets, perm, inv_perm);
  }
  return hdmoe_check_launch(what);
}

// Second pass alone: the histograms come from the gate kernel, one per block of tokens_per_hist tokens
// (hdmoe_gate_tokens_per_block). A chunk is as many whole histograms as fit 128 tokens, or one histogram of up to
// 1024 tokens.
int dispatch_scatter_enqueue(const char* what, const int32_t* topk_idx, int T, int E, int32_t* counts,
                             int32_t* offsets, int32_t* perm, int32_t* inv_perm, const int32_t* block_hist,
                             int tokens_per_hist, hipStream_t s) {
  const int n = T * HDMOE_TOPK;
  const int small_tokens = THREADS * ITEMS_SMALL / HDMOE_TOPK, large_tokens = THREADS * ITEMS_LARGE / HDMOE_TOPK;
  if (tokens_per_hist < 1 || tokens_per_hist > large_tokens)
    return hdmoe_fail(HDMOE_E_SHAPE, "%s: histograms of %d tokens (1 to %d)", what, tokens_per_hist, large_tokens);
  const int per_chunk = tokens_per_hist <= small_tokens ? small_tokens / tokens_per_hist : 1;
  const int chunk_tokens = per_chunk * tokens_per_hist;
  const int chunk = chunk_tokens * HDMOE_TOPK;
  int nchunks = (n + chunk - 1) / chunk;
  if (nchunks < 1) nchunks = 1;
  const int nhist = T > 0 ? (T + tokens_per_hist - 1) / tokens_per_hist : 0;
  if (chunk <= THREADS * ITEMS_SMALL)
    hipLaunchKernelGGL(dispatch_scatter_kernel<ITEMS_SMALL>, dim3(nchunks), dim3(THREADS), 0, s, topk_idx, n, E, nhist,
                       per_chunk, chunk, block_hist, counts, offsets, perm, inv_perm);
  else
    hipLaunchKernelGGL(dispatch_scatter_kernel<ITEMS_LARGE>, dim3(nchunks), dim3(THREADS), 0, s, topk_idx, n, E, nhist,
                       per_chunk, chunk, block_hist, counts, offsets, perm, inv_perm);
  return hdmoe_check_launch(what);
}

int dispatch_check_sizes(const char* what, int T, int E) {
  if (T < 0 || E < 1 || E > HDMOE_MAX_EXPERTS)
    return hdmoe_fail(HDMOE_E_SHAPE, "%s: T=%d E=%d (1 <= E <= %d)", what, T, E, HDMOE_MAX_EXPERTS);
  if ((size_t)T * HDMOE_TOPK > (size_t)INT32_MAX) return hdmoe_fail(HDMOE_E_SHAPE, "%s: T=%d too large", what, T);
  return HDMOE_OK;
}

}  // namespace

// The dispatch of the one-call layer: the gate kernel has already counted.
int hdmoe_launch_dispatch_scatter(const int32_t* topk_idx, int T, int E, int32_t* counts, int32_t* offsets,
                                  int32_t* perm, int32_t* inv_perm, const int32_t* block_hist, int tokens_per_hist,
                                  hipStream_t s, const char* what) {
  if (int rc = dispatch_check_sizes(what, T, E)) return rc;
  return dispatch_scatter_enqueue(what, topk_idx, T, E, counts, offsets, perm, inv_perm, block_hist, tokens_per_hist, s);
}

extern "C" int hdmoe_dispatch(const int32_t* topk_idx, int T, int E, int32_t* counts, int32_t* offsets,
                              int32_t* perm, int32_t* inv_perm, void* workspace, size_t workspace_bytes,
                              hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(topk_idx);
  HDMOE_REQUIRE_PTR(counts);
  HDMOE_REQUIRE_PTR(offsets);
  HDMOE_REQUIRE_PTR(perm);
  HDMOE_REQUIRE_PTR(inv_perm);
  HDMOE_REQUIRE_PTR(workspace);
  if (int rc = dispatch_check_sizes("hdmoe_dispatch", T, E)) return rc;
  if (workspace_bytes < hdmoe_dispatch_workspace_bytes(T, E) || (reinterpret_cast<uintptr_t>(workspace) & 3))
    return hdmoe_fail(HDMOE_E_WORKSPACE, "hdmoe_dispatch: workspace %zu bytes, need %zu (4-byte aligned)",
                      workspace_bytes, hdmoe_dispatch_workspace_bytes(T, E));
  return dispatch_enqueue("hdmoe_dispatch", topk_idx, T, E, counts, offsets, perm, inv_perm,
                          static_cast<int32_t*>(workspace), static_cast<hipStream_t>(stream));
}

// ---- the same dispatch for callers that cannot allocate ------------------------------------------------------
// The per-chunk histograms live in a device array that is part of the library image (every GPU the library runs
// on holds its own copy until the process ends). Host code must not use the array's name as an address: the
// device address is asked for once per device and kept.
namespace {

constexpr size_t STATIC_SCRATCH_BYTES = 64 * 1024;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
void* scratch_dev_ptr[MAX_DEVICES] = {};

// Device address of `scratch` on the current device (looked up on the first call per device), nullptr on failure.
void* scratch_address(const char* what, int* rc) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess || device < 0 || device >= MAX_DEVICES) {
    *rc = hdmoe_fail(HDMOE_E_LAUNCH, "%s: hipGetDevice: %s (device %d)", what, hipGetErrorString(e), device);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_dev_ptr[device] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      *rc = hdmoe_fail(HDMOE_E_LAUNCH, "%s: hipGetSymbolAddress: %s", what, hipGetErrorString(e));
      return nullptr;
    }
    scratch_dev_ptr[device] = p;
  }
  return scratch_dev_ptr[device];
}

}  // namespace

extern "C" int hdmoe_dispatch_static_max_tokens(int E) {
  if (E < 1 || E > HDMOE_MAX_EXPERTS) return 0;
  // chunks of THREADS * ITEMS_LARGE flat slots above SMALL_MAX_SLOTS; E counters per chunk
  const size_t max_chunks = STATIC_SCRATCH_BYTES / (sizeof(int32_t) * (size_t)E);
  const size_t tokens = max_chunks * (size_t)(THREADS * ITEMS_LARGE) / HDMOE_TOPK;
  return tokens > (size_t)(INT32_MAX / HDMOE_TOPK) ? INT32_MAX / HDMOE_TOPK : (int)tokens;
}

extern "C" int hdmoe_dispatch_static(const int32_t* topk_idx, int T, int E, int32_t* counts, int32_t* offsets,
                                     int32_t* perm, int32_t* inv_perm, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(topk_idx);
  HDMOE_REQUIRE_PTR(counts);
  HDMOE_REQUIRE_PTR(offsets);
  HDMOE_REQUIRE_PTR(perm);
  HDMOE_REQUIRE_PTR(inv_perm);
  if (int rc = dispatch_check_sizes("hdmoe_dispatch_static", T, E)) return rc;
  const size_t need = hdmoe_dispatch_workspace_bytes(T, E);
  if (need > STATIC_SCRATCH_BYTES)
    return hdmoe_fail(HDMOE_E_WORKSPACE,
                      "hdmoe_dispatch_static: T=%d E=%d needs %zu bytes of histograms, the built-in buffer holds %zu "
                      "(at most %d tokens for this E); use hdmoe_dispatch with a workspace",
                      T, E, need, STATIC_SCRATCH_BYTES, hdmoe_dispatch_static_max_tokens(E));
  int rc = HDMOE_OK;
  void* cc = scratch_address("hdmoe_dispatch_static", &rc);
  if (cc == nullptr) return rc;
  // every chunk histogram the scatter kernel reads is written by the count kernel of the same call: nothing of
  // the previous call's contents is used, so nothing has to be cleared
  return dispatch_enqueue("hdmoe_dispatch_static", topk_idx, T, E, counts, offsets, perm, inv_perm,
                          static_cast<int32_t*>(cc), static_cast<hipStream_t>(stream));
}
