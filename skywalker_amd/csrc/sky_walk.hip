// Biased walk on prebuilt alias tables (replaces sample_kernel_static / _buffer / sample_kernel and
// OfflineWalk of the reference, src/offline_walk.cu:10-230), with the PPR stop test the reference
// only has in its online kernel (src/online_walk.cu:109-110).
//
// One walker per lane.  Step s of walker i draws r = Philox(seed; i, s, 0, DOM_WALK):
//   stop when stop_prob > 0 and u24(r.z) < stop_prob, or the vertex has no out-edge,
//   col = mulhi(r.x, deg); cand = u24(r.y) < prob[off+col] ? col : alias[off+col];
//   stop when cand == SKY_INVALID (row of zero total weight); next = adjncy[off + cand].
// The result depends on (seed, i, s) only, never on scheduling.
#include "sky_graph.h"

namespace sky {

constexpr int WALK_BLOCK = 256;

__global__ __launch_bounds__(WALK_BLOCK) void walk_offline_kernel(
    const uint32_t* __restrict__ xadj, const uint32_t* __restrict__ adjncy,
    const AliasEntry* __restrict__ table, const uint32_t* __restrict__ seeds, uint32_t N, uint32_t V, uint32_t len,
    float stop_prob, uint64_t seed, uint32_t* __restrict__ paths, uint32_t* __restrict__ lengths,
    unsigned long long* __restrict__ sampled, unsigned long long* __restrict__ block_partials) {
  __shared__ unsigned long long s_part[WALK_BLOCK / 64];
  const uint32_t i = blockIdx.x * WALK_BLOCK + threadIdx.x;
  uint32_t s = 0;
  if (i < N) {
    uint32_t* path = paths + (size_t)i * (len + 1);
    uint32_t v = seeds[i];
    path[0] = v;
    for (; s < len && v < V; ++s) {  // a start vertex that does not exist is recorded and never left
      const u32x4 r = philox(seed, i, s, 0, DOM_WALK);
      if (stop_prob > 0.0f && u24(r.z) < stop_prob) break;
      const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
      if (deg == 0) break;
      const uint32_t col = __umulhi(r.x, deg);
      const AliasEntry e = table[off + col];
      const uint32_t cand = u24(r.y) < e.prob ? col : e.alias;
      if (cand == SKY_INVALID) break;
      v = adjncy[off + cand];
      path[s + 1] = v;
    }
    lengths[i] = s;
  }
  // exact 64-bit count of sampled edges (the reference reduces lengths through float, sampler_result.cuh:57-67)
  unsigned long long t = s;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) t += shfl_xor_u64(t, m);
  if (block_partials) {  // one sum per workgroup, added up by reduce_partials_kernel: no counter to clear
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = t;
    __syncthreads();
    if (threadIdx.x == 0) {
      unsigned long long b = 0;
#pragma unroll
      for (int w = 0; w < WALK_BLOCK / 64; ++w) b += s_part[w];
      block_partials[blockIdx.x] = b;
    }
  } else if ((threadIdx.x & 63) == 0 && t) {
    atomicAdd(sampled, t);
  }
}

int walk_offline(sky_graph* g, const uint32_t* seeds, uint32_t N, uint32_t len, float stop_prob, uint64_t seed,
                 uint32_t* paths, uint32_t* lengths, uint64_t* sampled, double* seconds) {
  hipStream_t st = g->stream;
  unsigned long long* d_sampled = nullptr;
  SKY_TRY(pool_get(g, sky_graph::POOL_COUNTERS, 64, (void**)&d_sampled));
  SKY_HIP(hipMemsetAsync(d_sampled, 0, 8, st));
  EventTimer tm(g);
  SKY_TRY(tm.mark("start", 0));
  if (N)
    hipLaunchKernelGGL(walk_offline_kernel, dim3((N + WALK_BLOCK - 1) / WALK_BLOCK), dim3(WALK_BLOCK), 0, st, g->xadj,
                       g->adjncy, g->table, seeds, N, g->V, len, stop_prob, seed, paths, lengths, d_sampled,
                       (unsigned long long*)nullptr);
  SKY_TRY(tm.mark("walk", 0));
  SKY_TRY(tm.finish(nullptr, seconds));
  unsigned long long h = 0;
  SKY_HIP(hipMemcpy(&h, d_sampled, 8, hipMemcpyDeviceToHost));
  if (sampled) *sampled = h;
  return SKY_OK;
}

// ---------------------------------------------------------------- the same walk without any allocation
// For callers that cannot allocate (HIP graph capture, serving loops): the per-workgroup counts of sampled
// edges go to a file-scope device array instead of a counter from hipMalloc, a second kernel adds them up into
// the caller's own device word, no event is created and nothing is copied to the host.  Every call on a GPU
// shares that GPU's array: calls that overlap on one GPU race.  Nothing in it needs clearing (each workgroup of
// a call writes its own element before the sum reads it).
constexpr uint32_t NOALLOC_MAX_BLOCKS = 16384;  // 128 KiB of device memory per GPU, held until the process ends
constexpr int NOALLOC_MAX_DEVICES = 64;
static __device__ __align__(256) unsigned long long scratch[NOALLOC_MAX_BLOCKS];
static unsigned long long* g_scratch_ptr[NOALLOC_MAX_DEVICES];  // device address of `scratch` on each GPU

__global__ __launch_bounds__(1024) void reduce_partials_kernel(const unsigned long long* __restrict__ partials,
                                                               uint32_t n, unsigned long long* __restrict__ out) {
  __shared__ unsigned long long s_w[16];
  unsigned long long t = 0;
  for (uint32_t k = threadIdx.x; k < n; k += 1024u) t += partials[k];
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) t += shfl_xor_u64(t, m);
  if ((threadIdx.x & 63) == 0) s_w[threadIdx.x >> 6] = t;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long b = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) b += s_w[w];
    *out = b;
  }
}

int walk_offline_noalloc(sky_graph* g, const uint32_t* seeds, uint32_t N, uint32_t len, float stop_prob,
                         uint64_t seed, uint32_t* paths, uint32_t* lengths, uint64_t* sampled_device) {
  const uint64_t max_walkers = (uint64_t)NOALLOC_MAX_BLOCKS * WALK_BLOCK;
  if (N > max_walkers)
    return fail(SKY_ERR_LIMIT, "sky_walk_offline_noalloc: " + std::to_string(N) + " walkers, the static scratch holds " +
                                   std::to_string(max_walkers) + " (split the batch)");
  int dev = 0;
  SKY_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return fail(SKY_ERR_LIMIT, "sky_walk_offline_noalloc: device index beyond 63");
  if (!g_scratch_ptr[dev]) {  // once per device, with that device current: each GPU holds its own copy of the array
    unsigned long long* p = nullptr;
    SKY_HIP(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
    g_scratch_ptr[dev] = p;
  }
  unsigned long long* const partials = g_scratch_ptr[dev];
  hipStream_t st = g->stream;
  const uint32_t blocks = (N + WALK_BLOCK - 1) / WALK_BLOCK;
  if (blocks)
    hipLaunchKernelGGL(walk_offline_kernel, dim3(blocks), dim3(WALK_BLOCK), 0, st, g->xadj, g->adjncy, g->table, seeds,
                       N, g->V, len, stop_prob, seed, paths, lengths, (unsigned long long*)nullptr, partials);
  if (sampled_device)
    hipLaunchKernelGGL(reduce_partials_kernel, dim3(1), dim3(1024), 0, st, partials, blocks,
                       reinterpret_cast<unsigned long long*>(sampled_device));
  SKY_HIP(hipGetLastError());
  return SKY_OK;
}

// ---------------------------------------------------------------- node2vec by rejection
// The second-order law of a step, w(v,x) * f(x) with f = 1/p for the previous vertex, 1 for its
// neighbours and 1/q for the rest (src/api/bias_node2vec.cu:15-27), is sampled without building the
// step's table: trial t draws a candidate from the first-order table of the current vertex with
// r_t = Philox(seed; i, s, t, DOM_WALK) (trial 0 shares the counter of the stop test) and keeps it when
// u24(r_t.w) * fmax < f(candidate), fmax = max(1/p, 1, 1/q); the 65537th candidate is kept whatever
// it is.  One membership search in the previous vertex's sorted row per trial, instead of one
// per neighbour of the current vertex.  The reference's unbiased node2vec walker rejects the same way
// (src/unbiased_walk.cu:14-60).  One walker per lane.
__device__ __forceinline__ bool row_has(const uint32_t* __restrict__ row, uint32_t n, uint32_t key) {
  uint32_t lo = 0;
  while (n > 1) {  // invariant: if key is in the row it is in [lo, lo + n)
    const uint32_t half = n >> 1;
    lo = row[lo + half] <= key ? lo + half : lo;
    n -= half;
  }
  return n == 1 && row[lo] == key;
}

__global__ __launch_bounds__(WALK_BLOCK) void walk_n2v_reject_kernel(
    const uint32_t* __restrict__ xadj, const uint32_t* __restrict__ adjncy,
    const AliasEntry* __restrict__ table, const uint32_t* __restrict__ seeds, uint32_t N, uint32_t V, uint32_t len,
    float fp, float fq, float fmax, float stop_prob, uint64_t seed, uint32_t* __restrict__ paths,
    uint32_t* __restrict__ lengths, unsigned long long* __restrict__ sampled) {
  const uint32_t i = blockIdx.x * WALK_BLOCK + threadIdx.x;
  uint32_t s = 0;
  if (i < N) {
    uint32_t* path = paths + (size_t)i * (len + 1);
    uint32_t v = seeds[i], prev = 0, prev_off = 0, prev_deg = 0;
    path[0] = v;
    for (; s < len && v < V; ++s) {
      u32x4 r = philox(seed, i, s, 0, DOM_WALK);
      if (stop_prob > 0.0f && u24(r.z) < stop_prob) break;
      const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
      if (deg == 0) break;
      uint32_t next = 0;
      bool dead = false;
      for (uint32_t t = 0;; ++t) {
        if (t) r = philox(seed, i, s, t, DOM_WALK);
        const uint32_t col = __umulhi(r.x, deg);
        const AliasEntry e = table[off + col];
        const uint32_t cand = u24(r.y) < e.prob ? col : e.alias;
        if (cand == SKY_INVALID) {
          dead = true;
          break;
        }
        next = adjncy[off + cand];
        if (s == 0 || t >= 65536u) break;
        const float f = next == prev ? fp : (row_has(adjncy + prev_off, prev_deg, next) ? 1.0f : fq);
        if (u24(r.w) * fmax < f) break;
      }
      if (dead) break;
      prev = v;
      prev_off = off;
      prev_deg = deg;
      v = next;
      path[s + 1] = v;
    }
    lengths[i] = s;
  }
  unsigned long long t = s;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) t += shfl_xor_u64(t, m);
  if ((threadIdx.x & 63) == 0 && t) atomicAdd(sampled, t);
}

int walk_node2vec_reject(sky_graph* g, float p, float q, const uint32_t* seeds, uint32_t N, uint32_t len,
                         float stop_prob, uint64_t seed, uint32_t* paths, uint32_t* lengths, uint64_t* sampled,
                         double* seconds) {
  hipStream_t st = g->stream;
  double build_sec = 0;
  if (!g->has_tables) SKY_TRY(build_all_tables(g, &build_sec));  // first-order tables, built on demand
  const float fp = 1.0f / p, fq = 1.0f / q;
  const float fmax = fmaxf(1.0f, fmaxf(fp, fq));
  unsigned long long* d_sampled = nullptr;
  auto body = [&]() -> int {
    SKY_TRY(pool_get(g, sky_graph::POOL_COUNTERS, 64, (void**)&d_sampled));
    SKY_HIP(hipMemsetAsync(d_sampled, 0, 8, st));
    EventTimer tm(g);
    SKY_TRY(tm.mark("start", 0));
    if (N)
      hipLaunchKernelGGL(walk_n2v_reject_kernel, dim3((N + WALK_BLOCK - 1) / WALK_BLOCK), dim3(WALK_BLOCK), 0, st,
                         g->xadj, g->adjncy, g->table, seeds, N, g->V, len, fp, fq, fmax, stop_prob, seed, paths, lengths,
                         d_sampled);
    SKY_TRY(tm.mark("walk", 0));
    double sec = 0;
    SKY_TRY(tm.finish(nullptr, &sec));
    SKY_HIP(hipGetLastError());
    unsigned long long h = 0;
    SKY_HIP(hipMemcpy(&h, d_sampled, 8, hipMemcpyDeviceToHost));
    if (sampled) *sampled = h;
    if (seconds) *seconds = sec + build_sec;
    return SKY_OK;
  };
  return body();
}

}  // namespace sky
