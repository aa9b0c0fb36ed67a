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

namespace sky {

__global__ __launch_bounds__(256) void walk_init_kernel(const uint32_t* __restrict__ seeds, uint32_t N, uint32_t len,
                                                        uint32_t* __restrict__ paths, uint32_t* __restrict__ lengths) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= N) return;
  paths[(size_t)i * (len + 1)] = seeds[i];
  lengths[i] = len;  // "still walking"; a walker that stops at step s stores s < len
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
  if (i >= N || lengths[i] != len) return;
  const u32x4 r = philox(seed, i, s, 0, DOM_WALK);
  const uint32_t v = paths[(size_t)i * (len + 1) + s];
  if ((stop_prob > 0.0f && u24(r.z) < stop_prob) || xadj[v + 1] == xadj[v]) {
    lengths[i] = s;
    return;
  }
  atomicAdd(&counters[1], 1u);
  const uint32_t bit = 1u << (v & 31);
  if (atomicOr(&bitmap[v >> 5], bit) & bit) return;
  list[atomicAdd(&counters[0], 1u)] = v;
}

__global__ __launch_bounds__(256) void walk_step_kernel(const uint32_t* __restrict__ xadj,
                                                        const uint32_t* __restrict__ adjncy,
                                                        const float* __restrict__ prob,
                                                        const uint32_t* __restrict__ alias, uint32_t N, uint32_t len,
                                                        uint32_t s, uint64_t seed, uint32_t* __restrict__ paths,
                                                        uint32_t* __restrict__ lengths) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= N || lengths[i] != len) return;
  const u32x4 r = philox(seed, i, s, 0, DOM_WALK);
  uint32_t* path = paths + (size_t)i * (len + 1);
  const uint32_t v = path[s];
  const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
  const uint32_t col = __umulhi(r.x, deg);
  const uint32_t cand = u24(r.y) < prob[off + col] ? col : alias[off + col];
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

int walk_online(sky_graph* g, int bias_kind, float p, float q, const uint32_t* seeds, uint32_t N, uint32_t len,
                float stop_prob, uint64_t seed, uint32_t* paths, uint32_t* lengths, uint64_t* sampled,
                double* seconds) {
  if (bias_kind == SKY_BIAS_NODE2VEC)
    return walk_online_node2vec(g, p, q, seeds, N, len, stop_prob, seed, paths, lengths, sampled, seconds);
  hipStream_t st = g->stream;
  unsigned long long* d_sampled = nullptr;
  uint32_t *bitmap = nullptr, *list = nullptr, *d_cnt = nullptr;
  const uint32_t words = (g->V + 31) / 32;
  auto cleanup = [&]() {
    if (d_sampled) (void)hipFree(d_sampled);
    if (bitmap) (void)hipFree(bitmap);
    if (list) (void)hipFree(list);
    if (d_cnt) (void)hipFree(d_cnt);
  };
  auto body = [&]() -> int {
    SKY_TRY(ensure_table_storage(g));
    SKY_TRY(prepare_build_scratch(std::min(N, g->V)));
    SKY_HIP(hipMalloc((void**)&d_sampled, 8));
    SKY_HIP(hipMalloc((void**)&bitmap, (size_t)words * 4 + 16));
    SKY_HIP(hipMalloc((void**)&list, (size_t)std::min(N, g->V) * 4 + 16));
    SKY_HIP(hipMalloc((void**)&d_cnt, 8));
    SKY_HIP(hipMemsetAsync(d_sampled, 0, 8, st));
    EventTimer tm(st);
    SKY_TRY(tm.mark("start", 0));
    const uint32_t blocks = (N + 255) / 256;
    if (N) {
      SKY_HIP(hipMemsetAsync(bitmap, 0, (size_t)words * 4, st));
      hipLaunchKernelGGL(walk_init_kernel, dim3(blocks), dim3(256), 0, st, seeds, N, len, paths, lengths);
      for (uint32_t s = 0; s < len; ++s) {
        SKY_HIP(hipMemsetAsync(d_cnt, 0, 8, st));
        hipLaunchKernelGGL(walk_collect_kernel, dim3(blocks), dim3(256), 0, st, g->xadj, N, len, s, stop_prob, seed,
                           paths, lengths, bitmap, list, d_cnt);
        uint32_t cnt[2] = {0, 0};
        SKY_HIP(hipMemcpyAsync(cnt, d_cnt, 8, hipMemcpyDeviceToHost, st));
        SKY_HIP(hipStreamSynchronize(st));
        if (cnt[1] == 0) break;  // every walker has stopped
        SKY_TRY(build_rows(g, list, cnt[0], nullptr));
        hipLaunchKernelGGL(walk_step_kernel, dim3(blocks), dim3(256), 0, st, g->xadj, g->adjncy, g->prob, g->alias, N,
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
  const int rc = body();
  cleanup();
  return rc;
}

int walk_online_node2vec(sky_graph*, float, float, const uint32_t*, uint32_t, uint32_t, float, uint64_t, uint32_t*,
                         uint32_t*, uint64_t*, double*) {
  return fail(SKY_ERR_STATE, "sky_walk_online: node2vec bias is not available in this build");
}

}  // namespace sky
