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
    const AliasEntry* __restrict__ table, const uint32_t* __restrict__ seeds, uint32_t N, uint32_t len,
    float stop_prob, uint64_t seed, uint32_t* __restrict__ paths, uint32_t* __restrict__ lengths,
    unsigned long long* __restrict__ sampled) {
  const uint32_t i = blockIdx.x * WALK_BLOCK + threadIdx.x;
  uint32_t s = 0;
  if (i < N) {
    uint32_t* path = paths + (size_t)i * (len + 1);
    uint32_t v = seeds[i];
    path[0] = v;
    for (; s < len; ++s) {
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
  if ((threadIdx.x & 63) == 0 && t) atomicAdd(sampled, t);
}

int walk_offline(sky_graph* g, const uint32_t* seeds, uint32_t N, uint32_t len, float stop_prob, uint64_t seed,
                 uint32_t* paths, uint32_t* lengths, uint64_t* sampled, double* seconds) {
  hipStream_t st = g->stream;
  unsigned long long* d_sampled = nullptr;
  SKY_HIP(hipMalloc((void**)&d_sampled, 8));
  SKY_HIP(hipMemsetAsync(d_sampled, 0, 8, st));
  hipEvent_t e0, e1;
  SKY_HIP(hipEventCreate(&e0));
  SKY_HIP(hipEventCreate(&e1));
  SKY_HIP(hipEventRecord(e0, st));
  if (N)
    hipLaunchKernelGGL(walk_offline_kernel, dim3((N + WALK_BLOCK - 1) / WALK_BLOCK), dim3(WALK_BLOCK), 0, st, g->xadj,
                       g->adjncy, g->table, seeds, N, len, stop_prob, seed, paths, lengths, d_sampled);
  SKY_HIP(hipEventRecord(e1, st));
  SKY_HIP(hipStreamSynchronize(st));
  SKY_HIP(hipGetLastError());
  float ms = 0;
  SKY_HIP(hipEventElapsedTime(&ms, e0, e1));
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  unsigned long long h = 0;
  SKY_HIP(hipMemcpy(&h, d_sampled, 8, hipMemcpyDeviceToHost));
  SKY_HIP(hipFree(d_sampled));
  if (sampled) *sampled = h;
  if (seconds) *seconds = ms * 1e-3;
  return SKY_OK;
}

}  // namespace sky
