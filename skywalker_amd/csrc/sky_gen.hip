// Synthetic inputs generated on the device: R-MAT CSR, per-slot weights, start vertices.
// The reference reads Galois .gr files (include/graph.cuh:164-327) and draws random weights with
// srand/rand (:210-219); graphs of the benchmark sizes are produced here instead so that they
// never cross PCIe.  Every value is a function of (seed, index) through Philox4x32-10.
#include <hipcub/hipcub.hpp>

#include "sky_graph.h"

namespace sky {

// Edge i: one 16-bit uniform per level (level 0 = most significant bit), eight levels per
// Philox call; quadrant thresholds a=.57 b=.19 c=.19 d=.05 on a 65536 grid.
__global__ __launch_bounds__(256) void rmat_keys_kernel(uint32_t scale, uint64_t E, uint64_t seed,
                                                        uint64_t* __restrict__ keys) {
  const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (i >= E) return;
  const uint32_t A = 37355u, AB = 49807u, ABC = 62259u;
  uint32_t s = 0, d = 0;
  for (uint32_t blk = 0; blk * 8 < scale; ++blk) {
    const u32x4 r = philox(seed, (uint32_t)i, (uint32_t)(i >> 32), blk, DOM_RMAT);
    const uint32_t words[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (uint32_t j = 0; j < 8; ++j) {
      if (blk * 8 + j >= scale) break;
      const uint32_t word = words[j >> 1];
      const uint32_t x = (j & 1u) ? (word >> 16) : (word & 0xFFFFu);
      const uint32_t sb = x >= AB ? 1u : 0u;
      const uint32_t db = ((x >= A && x < AB) || x >= ABC) ? 1u : 0u;
      s = (s << 1) | sb;
      d = (d << 1) | db;
    }
  }
  keys[i] = ((uint64_t)s << 32) | d;
}

// From keys sorted by (src, dst): adjncy[i] = dst, and xadj[v] = first slot whose src >= v.
__global__ __launch_bounds__(256) void csr_from_keys_kernel(const uint64_t* __restrict__ keys, uint64_t E, uint32_t V,
                                                            uint32_t* __restrict__ xadj,
                                                            uint32_t* __restrict__ adjncy) {
  const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (i > E) return;
  const int64_t prev = i == 0 ? -1 : (int64_t)(keys[i - 1] >> 32);
  int64_t cur = V;
  if (i < E) {
    const uint64_t k = keys[i];
    cur = (int64_t)(k >> 32);
    adjncy[i] = (uint32_t)k;
  }
  for (int64_t v = prev + 1; v <= cur; ++v) xadj[v] = (uint32_t)i;
}

__global__ __launch_bounds__(256) void weights_kernel(int kind, uint64_t seed, uint64_t E, float a, float b,
                                                      float* __restrict__ w) {
  const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (i >= E) return;
  const u32x4 r = philox(seed, (uint32_t)i, (uint32_t)(i >> 32), 0, DOM_WEIGHT);
  float x;
  if (kind == SKY_W_UNIFORM) {
    x = __fmaf_rn(b - a, u24(r.x), a);
  } else if (kind == SKY_W_UNIT) {
    x = (float)((r.x >> 8) + 1u) * (1.0f / 16777216.0f);
  } else {
    const float u1 = (float)((r.x >> 8) + 1u) * (1.0f / 16777216.0f);
    const float u2 = u24(r.y);
    const float z = sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
    x = expf(a + b * z);
  }
  w[i] = x;
}

__global__ __launch_bounds__(256) void seeds_kernel(uint64_t seed, uint32_t V, uint32_t N, uint32_t* __restrict__ out) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= N) return;
  out[i] = __umulhi(philox(seed, i, 0, 0, DOM_SEEDS).x, V);
}

__global__ __launch_bounds__(256) void max_degree_kernel(const uint32_t* __restrict__ xadj, uint32_t V,
                                                         uint32_t* __restrict__ out) {
  uint32_t m = 0;
  for (uint32_t v = blockIdx.x * 256u + threadIdx.x; v < V; v += gridDim.x * 256u)
    m = max(m, xadj[v + 1] - xadj[v]);
#pragma unroll
  for (int k = 32; k >= 1; k >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, k, 64));
  if ((threadIdx.x & 63) == 0 && m) atomicMax(out, m);
}

__global__ void philox_selftest_kernel(const uint32_t* ctr, const uint32_t* key, uint32_t n, uint32_t* out) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const u32x4 r = philox4x32_10(ctr[4 * i], ctr[4 * i + 1], ctr[4 * i + 2], ctr[4 * i + 3], key[2 * i], key[2 * i + 1]);
  out[4 * i] = r.x;
  out[4 * i + 1] = r.y;
  out[4 * i + 2] = r.z;
  out[4 * i + 3] = r.w;
}

int compute_max_degree(sky_graph* g) {
  uint32_t* d_m = nullptr;
  SKY_HIP(hipMalloc((void**)&d_m, 4));
  SKY_HIP(hipMemsetAsync(d_m, 0, 4, g->stream));
  if (g->V) {
    const uint32_t grid = std::min<uint32_t>((g->V + 255) / 256, 4096);
    hipLaunchKernelGGL(max_degree_kernel, dim3(grid), dim3(256), 0, g->stream, g->xadj, g->V, d_m);
  }
  SKY_HIP(hipMemcpy(&g->max_degree, d_m, 4, hipMemcpyDeviceToHost));
  SKY_HIP(hipFree(d_m));
  return SKY_OK;
}

int generate_rmat(uint32_t scale, uint32_t edge_factor, uint64_t graph_seed, int weight_kind, float wa, float wb,
                  uint64_t weight_seed, sky_graph** out) {
  if (!out || scale == 0 || scale > 31 || edge_factor == 0) return fail(SKY_ERR_ARG, "generate_rmat: bad arguments");
  const uint64_t V = 1ull << scale, E = (uint64_t)edge_factor << scale;
  if (E >= 0xFFFFFFFFull) return fail(SKY_ERR_LIMIT, "generate_rmat: edge count does not fit 32-bit offsets");
  if (weight_kind < SKY_W_UNIFORM || weight_kind > SKY_W_LOGNORMAL)
    return fail(SKY_ERR_ARG, "generate_rmat: unknown weight kind");
  sky_graph* g = new sky_graph();
  (void)hipGetDevice(&g->device);
  g->V = (uint32_t)V;
  g->E = (uint32_t)E;
  hipStream_t st = g->stream;
  uint64_t *keys_a = nullptr, *keys_b = nullptr;
  void* temp = nullptr;
  size_t temp_bytes = 0;
  auto cleanup = [&]() {
    if (keys_a) (void)hipFree(keys_a);
    if (keys_b) (void)hipFree(keys_b);
    if (temp) (void)hipFree(temp);
  };
#define GEN_HIP(expr)                                                                              \
  do {                                                                                             \
    hipError_t _e = (expr);                                                                        \
    if (_e != hipSuccess) {                                                                        \
      cleanup();                                                                                   \
      sky_graph_free(g);                                                                           \
      return fail(SKY_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(_e));                 \
    }                                                                                              \
  } while (0)
  GEN_HIP(hipMalloc((void**)&keys_a, E * 8));
  GEN_HIP(hipMalloc((void**)&keys_b, E * 8));
  const uint32_t eblocks = (uint32_t)((E + 255) / 256);
  hipLaunchKernelGGL(rmat_keys_kernel, dim3(eblocks), dim3(256), 0, st, scale, E, graph_seed, keys_a);
  GEN_HIP(hipcub::DeviceRadixSort::SortKeys(nullptr, temp_bytes, keys_a, keys_b, E, 0, (int)(32 + scale), st));
  GEN_HIP(hipMalloc(&temp, temp_bytes ? temp_bytes : 16));
  GEN_HIP(hipcub::DeviceRadixSort::SortKeys(temp, temp_bytes, keys_a, keys_b, E, 0, (int)(32 + scale), st));
  GEN_HIP(hipMalloc((void**)&g->xadj, (V + 1) * 4 + 16));
  GEN_HIP(hipMalloc((void**)&g->adjncy, E * 4 + 16));
  hipLaunchKernelGGL(csr_from_keys_kernel, dim3((uint32_t)((E + 1 + 255) / 256)), dim3(256), 0, st, keys_b, E,
                     (uint32_t)V, g->xadj, g->adjncy);
  GEN_HIP(hipStreamSynchronize(st));
  GEN_HIP(hipFree(keys_a));
  keys_a = nullptr;
  GEN_HIP(hipFree(keys_b));
  keys_b = nullptr;
  GEN_HIP(hipFree(temp));
  temp = nullptr;
  GEN_HIP(hipMalloc((void**)&g->adjwgt, E * 4 + 16));
  hipLaunchKernelGGL(weights_kernel, dim3(eblocks), dim3(256), 0, st, weight_kind, weight_seed, E, wa, wb, g->adjwgt);
  GEN_HIP(hipStreamSynchronize(st));
  GEN_HIP(hipGetLastError());
#undef GEN_HIP
  int rc = compute_max_degree(g);
  if (rc != SKY_OK) {
    sky_graph_free(g);
    return rc;
  }
  *out = g;
  return SKY_OK;
}

// Neighbour ids uniform over [0, V), one Philox counter per slot (domain of the R-MAT generator, third counter
// word 1 so that no counter is shared with it).  Rows come out unsorted.
__global__ __launch_bounds__(256) void random_adjncy_kernel(uint64_t seed, uint32_t V, uint64_t E,
                                                            uint32_t* __restrict__ adjncy) {
  const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (i >= E) return;
  adjncy[i] = __umulhi(philox(seed, (uint32_t)i, (uint32_t)(i >> 32), 1, DOM_RMAT).x, V);
}

int generate_from_degrees(const uint32_t* xadj_host, uint32_t V, uint64_t graph_seed, int weight_kind, float wa, float wb,
                          uint64_t weight_seed, sky_graph** out) {
  if (!out || !xadj_host) return fail(SKY_ERR_ARG, "generate_from_degrees: null pointer");
  if (weight_kind < SKY_W_UNIFORM || weight_kind > SKY_W_LOGNORMAL)
    return fail(SKY_ERR_ARG, "generate_from_degrees: unknown weight kind");
  if (xadj_host[0] != 0) return fail(SKY_ERR_ARG, "generate_from_degrees: xadj[0] != 0");
  for (uint32_t v = 0; v < V; ++v)
    if (xadj_host[v] > xadj_host[v + 1]) return fail(SKY_ERR_ARG, "generate_from_degrees: xadj is not monotone");
  const uint64_t E = xadj_host[V];
  if (E && V == 0) return fail(SKY_ERR_ARG, "generate_from_degrees: edges without vertices");
  sky_graph* g = new sky_graph();
  (void)hipGetDevice(&g->device);
  g->V = V;
  g->E = (uint32_t)E;
  hipStream_t st = g->stream;
  auto body = [&]() -> int {
    SKY_TRY(alloc_padded(&g->xadj, (size_t)V + 1));
    SKY_TRY(alloc_padded(&g->adjncy, (size_t)E));
    SKY_TRY(alloc_padded(&g->adjwgt, (size_t)E));
    SKY_HIP(hipMemcpy(g->xadj, xadj_host, ((size_t)V + 1) * 4, hipMemcpyHostToDevice));
    if (E) {
      const uint32_t eblocks = (uint32_t)((E + 255) / 256);
      hipLaunchKernelGGL(random_adjncy_kernel, dim3(eblocks), dim3(256), 0, st, graph_seed, V, E, g->adjncy);
      hipLaunchKernelGGL(weights_kernel, dim3(eblocks), dim3(256), 0, st, weight_kind, weight_seed, E, wa, wb, g->adjwgt);
    }
    SKY_HIP(hipStreamSynchronize(st));
    SKY_HIP(hipGetLastError());
    return compute_max_degree(g);
  };
  const int rc = body();
  if (rc != SKY_OK) {
    sky_graph_free(g);
    return rc;
  }
  *out = g;
  return SKY_OK;
}

int gen_seeds(uint64_t seed, uint32_t V, uint32_t N, uint32_t* seeds_device) {
  if (N) hipLaunchKernelGGL(seeds_kernel, dim3((N + 255) / 256), dim3(256), 0, nullptr, seed, V, N, seeds_device);
  SKY_HIP(hipStreamSynchronize(nullptr));
  SKY_HIP(hipGetLastError());
  return SKY_OK;
}

int philox_selftest(const uint32_t* ctr, const uint32_t* key, uint32_t n, uint32_t* out) {
  uint32_t *d_c = nullptr, *d_k = nullptr, *d_o = nullptr;
  SKY_HIP(hipMalloc((void**)&d_c, (size_t)n * 16));
  SKY_HIP(hipMalloc((void**)&d_k, (size_t)n * 8));
  SKY_HIP(hipMalloc((void**)&d_o, (size_t)n * 16));
  SKY_HIP(hipMemcpy(d_c, ctr, (size_t)n * 16, hipMemcpyHostToDevice));
  SKY_HIP(hipMemcpy(d_k, key, (size_t)n * 8, hipMemcpyHostToDevice));
  hipLaunchKernelGGL(philox_selftest_kernel, dim3((n + 63) / 64), dim3(64), 0, nullptr, d_c, d_k, n, d_o);
  SKY_HIP(hipMemcpy(out, d_o, (size_t)n * 16, hipMemcpyDeviceToHost));
  SKY_HIP(hipFree(d_c));
  SKY_HIP(hipFree(d_k));
  SKY_HIP(hipFree(d_o));
  return SKY_OK;
}

}  // namespace sky
