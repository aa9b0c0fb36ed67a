// Walks that build the alias table of the current vertex on the fly (replaces OnlineWalkKernel /
// OnlineWalkShMem / OnlineWalkGMem of src/online_walk.cu:82-166,245-327 and online_walk_gmem.cu).
//
// Static bias (DeepWalk, PPR): the table of a vertex does not depend on the walker, so each
// step builds, once, the tables of the distinct vertices the live walkers stand on that were
// not built earlier in the call, through the kernels of the offline build, and then advances
// every walker by one draw.  The draws, and so the paths, are those of the offline walk.
//
// node2vec: the weights of a step depend on the walker's previous vertex
// (src/api/bias_node2vec.cu:15-27), so each (walker, step) builds its own table.
#include "sky_graph.h"
#include "sky_step_draw.h"

namespace sky {

__global__ __launch_bounds__(256) void walk_init_kernel(const uint32_t* __restrict__ seeds, uint32_t N, uint32_t len,
                                                        uint32_t V, uint32_t* __restrict__ paths,
                                                        uint32_t* __restrict__ lengths) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= N) return;
  const uint32_t v = seeds[i];
  paths[(size_t)i * (len + 1)] = v;
  // "still walking"; a walker that stops at step s stores s < len.  A start vertex that does not exist
  // is recorded and never left.
  lengths[i] = v < V ? len : 0u;
}

// Stop test and dead-end test of step s; collects the vertices whose table is still missing.
// counters[0] = new vertices appended to list, counters[1] = walkers that will draw.
__global__ __launch_bounds__(256) void walk_collect_kernel(const uint32_t* __restrict__ xadj, uint32_t N, uint32_t len,
                                                           uint32_t s, float stop_prob, uint64_t seed,
                                                           const uint32_t* __restrict__ paths,
                                                           uint32_t* __restrict__ lengths,
                                                           uint32_t* __restrict__ bitmap, uint32_t* __restrict__ list,
                                                           uint32_t* __restrict__ counters) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  bool draws = false, fresh = false;
  uint32_t v = 0;
  if (i < N && lengths[i] == len) {
    const u32x4 r = philox(seed, i, s, 0, DOM_WALK);
    v = paths[(size_t)i * (len + 1) + s];
    if ((stop_prob > 0.0f && u24(r.z) < stop_prob) || xadj[v + 1] == xadj[v]) {
      lengths[i] = s;
    } else {
      draws = true;
      const uint32_t bit = 1u << (v & 31);
      fresh = !(atomicOr(&bitmap[v >> 5], bit) & bit);
    }
  }
  // one counter update per wavefront and counter
  const int lane = threadIdx.x & 63;
  const unsigned long long md = __ballot(draws), mf = __ballot(fresh);
  if (md && lane == __ffsll((long long)md) - 1) atomicAdd(&counters[1], (uint32_t)__popcll(md));
  if (mf) {
    const int first = __ffsll((long long)mf) - 1;
    uint32_t base = 0;
    if (lane == first) base = atomicAdd(&counters[0], (uint32_t)__popcll(mf));
    base = (uint32_t)__shfl((int)base, first, 64);
    if (fresh) list[base + (uint32_t)__popcll(mf & ((1ull << lane) - 1ull))] = v;
  }
}

__global__ __launch_bounds__(256) void walk_step_kernel(const uint32_t* __restrict__ xadj,
                                                        const uint32_t* __restrict__ adjncy,
                                                        const AliasEntry* __restrict__ table, uint32_t N, uint32_t len,
                                                        uint32_t s, uint64_t seed, uint32_t* __restrict__ paths,
                                                        uint32_t* __restrict__ lengths) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= N || lengths[i] != len) return;
  const u32x4 r = philox(seed, i, s, 0, DOM_WALK);
  uint32_t* path = paths + (size_t)i * (len + 1);
  const uint32_t v = path[s];
  const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
  const uint32_t col = __umulhi(r.x, deg);
  const AliasEntry e = table[off + col];
  const uint32_t cand = u24(r.y) < e.prob ? col : e.alias;
  if (cand == SKY_INVALID) {
    lengths[i] = s;
    return;
  }
  path[s + 1] = adjncy[off + cand];
}

__global__ __launch_bounds__(256) void sum_lengths_kernel(const uint32_t* __restrict__ lengths, uint32_t N,
                                                          unsigned long long* __restrict__ out) {
  unsigned long long t = 0;
  for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < N; i += gridDim.x * 256u) t += lengths[i];
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) t += shfl_xor_u64(t, m);
  if ((threadIdx.x & 63) == 0 && t) atomicAdd(out, t);
}

int walk_online_node2vec(sky_graph* g, float p, float q, const uint32_t* seeds, uint32_t N, uint32_t len,
                         float stop_prob, uint64_t seed, uint32_t* paths, uint32_t* lengths, uint64_t* sampled,
                         double* seconds);

// Option online_full_build: -1: decide by the estimate below; 0: always build lazily, step by step; 1: always build
// every row first.

// Estimated milliseconds of the two ways to serve a static-bias online walk.  A lazy round costs a
// host round trip and a handful of small launches (about 1/8 ms measured), and the rounds together
// build at most min(N * len, V) rows; the full build runs at about 1.3e8 edges per millisecond.
static bool online_prefers_full_build(const sky_graph* g, uint32_t N, uint32_t len) {
  const long long mode = option(g, OPT_ONLINE_FULL_BUILD);
  if (mode >= 0) return mode != 0;
  const double all_ms = (double)g->E / 1.3e8;
  const double visited = std::min(1.0, (double)N * len / std::max(1u, g->V));
  return 0.4 + all_ms < 0.125 * len + visited * all_ms;
}

int walk_online(sky_graph* g, int bias_kind, float p, float q, const uint32_t* seeds, uint32_t N, uint32_t len,
                float stop_prob, uint64_t seed, uint32_t* paths, uint32_t* lengths, uint64_t* sampled,
                double* seconds) {
  if (bias_kind == SKY_BIAS_NODE2VEC_REJECT)
    return walk_node2vec_reject(g, p, q, seeds, N, len, stop_prob, seed, paths, lengths, sampled, seconds);
  if (bias_kind == SKY_BIAS_NODE2VEC)
    return walk_online_node2vec(g, p, q, seeds, N, len, stop_prob, seed, paths, lengths, sampled, seconds);
  // Tables that already exist are used as they are.  Otherwise one build of every row, then the
  // offline kernel, is taken when it is expected to cost less than len rounds of lazy builds, each
  // of which waits for the host; the paths are the same either way.
  double build_sec = 0;
  if (!g->has_tables && N && len && online_prefers_full_build(g, N, len)) SKY_TRY(build_all_tables(g, &build_sec));
  if (g->has_tables) {
    SKY_TRY(walk_offline(g, seeds, N, len, stop_prob, seed, paths, lengths, sampled, seconds));
    if (seconds) *seconds += build_sec;
    return SKY_OK;
  }
  hipStream_t st = g->stream;
  unsigned long long* d_sampled = nullptr;
  uint32_t *bitmap = nullptr, *list = nullptr, *d_cnt = nullptr;
  const uint32_t words = (g->V + 31) / 32;
  // Without a row too long for the streaming kernel, no step waits for the device: the size of a step's list stays
  // there (build_rows_dev), and whether any walker still walks comes back through pinned host words that the host
  // reads as they arrive, some steps behind what it has enqueued; the steps enqueued past the last walker's end find
  // nothing to do.
  const bool dev_sized = build_rows_dev_possible(g) && option(g, OPT_ONLINE_DEVICE_SIZED) != 0;
  auto body = [&]() -> int {
    SKY_TRY(ensure_table_storage(g));
    if (dev_sized) {
      SKY_TRY(ensure_class_census(g));
      if (g->live_report_cap < len) {
        if (g->live_report) SKY_HIP(hipHostFree(g->live_report));
        g->live_report = nullptr;
        g->live_report_cap = 0;
        SKY_HIP(hipHostMalloc((void**)&g->live_report, (size_t)len * 4, hipHostMallocDefault));
        g->live_report_cap = len;
      }
      for (uint32_t s = 0; s < len; ++s) g->live_report[s] = 0xFFFFFFFFu;  // "not reported yet"
    }
    SKY_TRY(prepare_build_scratch(g, std::min(N, g->V)));
    SKY_TRY(pool_get(g, sky_graph::POOL_COUNTERS, 64, (void**)&d_sampled));
    d_cnt = reinterpret_cast<uint32_t*>(d_sampled + 1);
    SKY_TRY(pool_get(g, sky_graph::POOL_BITMAP, (size_t)words * 4, (void**)&bitmap));
    SKY_TRY(pool_get(g, sky_graph::POOL_LIST, (size_t)std::min(N, g->V) * 4, (void**)&list));
    SKY_HIP(hipMemsetAsync(d_sampled, 0, 8, st));
    EventTimer tm(g);
    SKY_TRY(tm.mark("start", 0));
    const uint32_t blocks = (N + 255) / 256;
    if (N) {
      SKY_HIP(hipMemsetAsync(bitmap, 0, (size_t)words * 4, st));
      hipLaunchKernelGGL(walk_init_kernel, dim3(blocks), dim3(256), 0, st, seeds, N, len, g->V, paths, lengths);
      for (uint32_t s = 0; s < len; ++s) {
        SKY_HIP(hipMemsetAsync(d_cnt, 0, 8, st));
        hipLaunchKernelGGL(walk_collect_kernel, dim3(blocks), dim3(256), 0, st, g->xadj, N, len, s, stop_prob, seed,
                           paths, lengths, bitmap, list, d_cnt);
        if (dev_sized) {
          SKY_HIP(hipMemcpyAsync(&g->live_report[s], d_cnt + 1, 4, hipMemcpyDeviceToHost, st));
          bool ended = false;
          for (uint32_t k = 0; k < s && !ended; ++k) ended = *(volatile uint32_t*)&g->live_report[k] == 0;
          if (ended) break;  // a step that has run found no walker left
          SKY_TRY(build_rows_dev(g, list, d_cnt, std::min(N, g->V)));
        } else {
          uint32_t cnt[2] = {0, 0};
          SKY_HIP(hipMemcpyAsync(cnt, d_cnt, 8, hipMemcpyDeviceToHost, st));
          SKY_HIP(hipStreamSynchronize(st));
          if (cnt[1] == 0) break;  // every walker has stopped
          SKY_TRY(build_rows(g, list, cnt[0], nullptr));
        }
        hipLaunchKernelGGL(walk_step_kernel, dim3(blocks), dim3(256), 0, st, g->xadj, g->adjncy, g->table, N,
                           len, s, seed, paths, lengths);
      }
      hipLaunchKernelGGL(sum_lengths_kernel, dim3(std::min<uint32_t>(blocks, 1024)), dim3(256), 0, st, lengths, N,
                         d_sampled);
    }
    SKY_TRY(tm.mark("walk", 0));
    SKY_TRY(tm.finish(nullptr, seconds));
    unsigned long long h = 0;
    SKY_HIP(hipMemcpy(&h, d_sampled, 8, hipMemcpyDeviceToHost));
    if (sampled) *sampled = h;
    return SKY_OK;
  };
  return body();
}

// ---------------------------------------------------------------- node2vec
// One workgroup per (walker, step) evaluates the one entry of the step's second-order table that the draw
// reads (step_draw_slot of sky_step_draw.h).
struct N2vRow {
  const float* w;
  const uint32_t* nbr;
  const uint32_t* prow;
  uint32_t pdeg, prev;
  bool has_prev;
  float p, q;
  // weight of the edge in slot k after the second-order factor (src/api/bias_node2vec.cu:15-27)
  __device__ __forceinline__ float operator()(uint32_t k) const {
    float x = w[k];
    if (has_prev) {
      const uint32_t t = nbr[k];
      if (t == prev) x = __fdiv_rn(x, p);
      else if (!row_contains(prow, pdeg, t)) x = __fdiv_rn(x, q);
    }
    return clamp_weight(x);
  }
};

__global__ __launch_bounds__(N2V_T) void n2v_step_kernel(const uint32_t* __restrict__ xadj,
                                                         const uint32_t* __restrict__ adjncy,
                                                         const float* __restrict__ wgt, uint32_t len, uint32_t s,
                                                         float p, float q, float stop_prob, uint64_t seed,
                                                         uint32_t* __restrict__ paths,
                                                         uint32_t* __restrict__ lengths) {
  const uint32_t i = blockIdx.x;
  const int tid = threadIdx.x;
  if (lengths[i] != len) return;  // stopped at an earlier step
  const u32x4 r = philox(seed, i, s, 0, DOM_WALK);
  uint32_t* path = paths + (size_t)i * (len + 1);
  const uint32_t v = path[s];
  const uint32_t off = xadj[v], d = xadj[v + 1] - off;
  if ((stop_prob > 0.0f && u24(r.z) < stop_prob) || d == 0) {
    if (tid == 0) lengths[i] = s;
    return;
  }
  N2vRow row;
  row.w = wgt + off;
  row.nbr = adjncy + off;
  row.has_prev = s > 0;
  row.prev = s > 0 ? path[s - 1] : 0;
  row.prow = adjncy + xadj[row.prev];
  row.pdeg = xadj[row.prev + 1] - xadj[row.prev];
  row.p = p;
  row.q = q;
  const uint32_t cand = step_draw_slot(row, d, r);
  if (tid == 0) {
    if (cand == NONE_SLOT) lengths[i] = s;
    else path[s + 1] = row.nbr[cand];
  }
}

int walk_online_node2vec(sky_graph* g, float p, float q, const uint32_t* seeds, uint32_t N, uint32_t len,
                         float stop_prob, uint64_t seed, uint32_t* paths, uint32_t* lengths, uint64_t* sampled,
                         double* seconds) {
  hipStream_t st = g->stream;
  unsigned long long* d_sampled = nullptr;
  auto body = [&]() -> int {
    SKY_TRY(pool_get(g, sky_graph::POOL_COUNTERS, 64, (void**)&d_sampled));
    SKY_HIP(hipMemsetAsync(d_sampled, 0, 8, st));
    EventTimer tm(g);
    SKY_TRY(tm.mark("start", 0));
    if (N) {
      const uint32_t blocks = (N + 255) / 256;
      hipLaunchKernelGGL(walk_init_kernel, dim3(blocks), dim3(256), 0, st, seeds, N, len, g->V, paths, lengths);
      for (uint32_t s = 0; s < len; ++s)
        hipLaunchKernelGGL(n2v_step_kernel, dim3(N), dim3(N2V_T), 0, st, g->xadj, g->adjncy, g->adjwgt, len, s, p, q,
                           stop_prob, seed, paths, lengths);
      hipLaunchKernelGGL(sum_lengths_kernel, dim3(std::min<uint32_t>(blocks, 1024)), dim3(256), 0, st, lengths, N,
                         d_sampled);
    }
    SKY_TRY(tm.mark("walk", 0));
    SKY_TRY(tm.finish(nullptr, seconds));
    unsigned long long h = 0;
    SKY_HIP(hipMemcpy(&h, d_sampled, 8, hipMemcpyDeviceToHost));
    if (sampled) *sampled = h;
    return SKY_OK;
  };
  return body();
}

}  // namespace sky
