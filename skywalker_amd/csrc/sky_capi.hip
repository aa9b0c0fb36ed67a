// extern "C" surface of libskywalker_hip.so (declared in include/skywalker_hip.h).
#include <cstring>

#include "sky_graph.h"

namespace sky {

static thread_local std::string g_last_error;

void set_error(const std::string& msg) { g_last_error = msg; }
int fail(int code, const std::string& msg) {
  g_last_error = msg;
  return code;
}

static int ensure_device() {
  static thread_local bool checked = false;
  if (checked) return SKY_OK;
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    return fail(SKY_ERR_NO_GPU, "no HIP device is visible to this process");
  }
  checked = true;
  return SKY_OK;
}

}  // namespace sky

using namespace sky;

namespace {
// The table as two arrays and back, on the device: a host loop over a table of a billion entries takes seconds.
__global__ __launch_bounds__(256) void split_table_kernel(const sky::AliasEntry* __restrict__ table, size_t lo, size_t n,
                                                          float* __restrict__ prob, uint32_t* __restrict__ alias) {
  const size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
  if (i >= n) return;
  const sky::AliasEntry e = table[lo + i];
  prob[i] = e.prob;
  alias[i] = e.alias;
}
__global__ __launch_bounds__(256) void join_table_kernel(const float* __restrict__ prob, const uint32_t* __restrict__ alias,
                                                         size_t lo, size_t n, sky::AliasEntry* __restrict__ table) {
  const size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
  if (i >= n) return;
  table[lo + i] = sky::AliasEntry{prob[i], alias[i]};
}
constexpr size_t TABLE_PIECE = 64u << 20;  // entries moved per round: 512 MB of staging on the device
}  // namespace

namespace sky {
// process-wide values of the tuning knobs, in the order of SkyOpt (sky_set_option changes them)
long long g_option_value[OPT_COUNT] = {
    1ll << 22,                             // tiled_max_tiles: no limit
    1,                                     // row_merge
    4000000,                               // stream_min_edges
    512ll * (sky::STREAM_MAX_DEG / 2),     // stream_wide_min_edges: 512 workgroups run at a time
    -1,                                    // walk_read_once: by the size of the tables
    0,                                     // sample_distinct
    -1,                                    // small_in_place: builds of at least 2^25 rows
    1,                                     // build_streams
    0,                                     // build_profile
    0,                                     // walk_compact_every
    -1,                                    // online_full_build: by estimate
    1,                                     // online_device_sized
};
}  // namespace sky

extern "C" {

const char* sky_last_error(void) { return g_last_error.c_str(); }
const char* sky_version(void) { return "skywalker_hip 0.1 (gfx950)"; }

int sky_device_malloc(size_t bytes, void** out) {
  if (!out) return fail(SKY_ERR_ARG, "sky_device_malloc: null output");
  SKY_TRY(ensure_device());
  SKY_HIP(hipMalloc(out, bytes + 16));  // 16 spare bytes, as every array of the library has: kernels read whole vectors
  return SKY_OK;
}
int sky_device_free(void* p) {
  if (p) SKY_HIP(hipFree(p));
  return SKY_OK;
}
int sky_memcpy_h2d(void* dst, const void* src, size_t bytes) {
  if (bytes && (!dst || !src)) return fail(SKY_ERR_ARG, "sky_memcpy_h2d: null pointer");
  if (bytes) SKY_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
  return SKY_OK;
}
int sky_memcpy_d2h(void* dst, const void* src, size_t bytes) {
  if (bytes && (!dst || !src)) return fail(SKY_ERR_ARG, "sky_memcpy_d2h: null pointer");
  if (bytes) SKY_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
  return SKY_OK;
}

__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}
int sky_device_fill_u32(void* dst, uint32_t value, size_t count) {
  if (count && !dst) return fail(SKY_ERR_ARG, "sky_device_fill_u32: null pointer");
  if (count) {
    const unsigned grid = (unsigned)std::min<size_t>((count + 255) / 256, 65536);
    hipLaunchKernelGGL(fill_u32_kernel, dim3(grid), dim3(256), 0, nullptr, (uint32_t*)dst, value, count);
    SKY_HIP(hipStreamSynchronize(nullptr));
    SKY_HIP(hipGetLastError());
  }
  return SKY_OK;
}
__global__ void copy_u32_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ src, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}
int sky_device_copy_u32(void* dst, const void* src, size_t count) {
  if (count && (!dst || !src)) return fail(SKY_ERR_ARG, "sky_device_copy_u32: null pointer");
  if (count) {
    const unsigned grid = (unsigned)std::min<size_t>((count + 255) / 256, 65536);
    hipLaunchKernelGGL(copy_u32_kernel, dim3(grid), dim3(256), 0, nullptr, (uint32_t*)dst, (const uint32_t*)src,
                       count);
    SKY_HIP(hipStreamSynchronize(nullptr));
    SKY_HIP(hipGetLastError());
  }
  return SKY_OK;
}
int sky_device_mem_info(size_t* free_bytes, size_t* total_bytes) {
  SKY_TRY(ensure_device());
  size_t f = 0, t = 0;
  SKY_HIP(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = f;
  if (total_bytes) *total_bytes = t;
  return SKY_OK;
}
int sky_device_synchronize(void) {
  SKY_HIP(hipDeviceSynchronize());
  return SKY_OK;
}
int sky_device_name(char* buf, size_t buflen, int* compute_units) {
  SKY_TRY(ensure_device());
  hipDeviceProp_t prop;
  int dev = 0;
  SKY_HIP(hipGetDevice(&dev));
  SKY_HIP(hipGetDeviceProperties(&prop, dev));
  if (buf && buflen) {
    std::string s = std::string(prop.name) + " (" + prop.gcnArchName + ")";
    strncpy(buf, s.c_str(), buflen - 1);
    buf[buflen - 1] = 0;
  }
  if (compute_units) *compute_units = prop.multiProcessorCount;
  return SKY_OK;
}

static int check_csr(const uint32_t* xadj, uint32_t V, uint32_t E) {
  if (xadj[0] != 0 || xadj[V] != E) return fail(SKY_ERR_ARG, "sky_graph_upload: xadj[0] != 0 or xadj[V] != E");
  for (uint32_t v = 0; v < V; ++v)
    if (xadj[v] > xadj[v + 1]) return fail(SKY_ERR_ARG, "sky_graph_upload: xadj is not monotone");
  return SKY_OK;
}

int sky_graph_upload(const uint32_t* xadj, const uint32_t* adjncy, const float* adjwgt, uint32_t V, uint32_t E,
                     sky_graph** out) {
  if (!out || !xadj || (E && !adjncy)) return fail(SKY_ERR_ARG, "sky_graph_upload: null pointer");
  SKY_TRY(ensure_device());
  SKY_TRY(check_csr(xadj, V, E));
  for (uint32_t i = 0; i < E; ++i)
    if (adjncy[i] >= V) return fail(SKY_ERR_ARG, "sky_graph_upload: neighbour id out of range");
  sky_graph* g = new sky_graph();
  (void)hipGetDevice(&g->device);
  g->V = V;
  g->E = E;
  int rc = SKY_OK;
  auto body = [&]() -> int {
    SKY_TRY(alloc_padded(&g->xadj, (size_t)V + 1));
    SKY_TRY(alloc_padded(&g->adjncy, (size_t)E));
    SKY_TRY(alloc_padded(&g->adjwgt, (size_t)E));
    SKY_HIP(hipMemcpy(g->xadj, xadj, ((size_t)V + 1) * 4, hipMemcpyHostToDevice));
    if (E) SKY_HIP(hipMemcpy(g->adjncy, adjncy, (size_t)E * 4, hipMemcpyHostToDevice));
    if (E) {
      if (adjwgt) {
        SKY_HIP(hipMemcpy(g->adjwgt, adjwgt, (size_t)E * 4, hipMemcpyHostToDevice));
      } else {
        SKY_TRY(sky_device_fill_u32(g->adjwgt, 0x3F800000u, E));  // 1.0f
      }
    }
    return compute_max_degree(g);
  };
  rc = body();
  if (rc != SKY_OK) {
    std::string keep = g_last_error;
    sky_graph_free(g);
    g_last_error = keep;
    return rc;
  }
  *out = g;
  return SKY_OK;
}

int sky_graph_generate_rmat(uint32_t scale, uint32_t edge_factor, uint64_t graph_seed, int weight_kind, float wa,
                            float wb, uint64_t weight_seed, sky_graph** out) {
  SKY_TRY(ensure_device());
  return generate_rmat(scale, edge_factor, graph_seed, weight_kind, wa, wb, weight_seed, out);
}

int sky_graph_generate_from_degrees(const uint32_t* xadj, uint32_t V, uint64_t graph_seed, int weight_kind, float wa,
                                    float wb, uint64_t weight_seed, sky_graph** out) {
  SKY_TRY(ensure_device());
  return generate_from_degrees(xadj, V, graph_seed, weight_kind, wa, wb, weight_seed, out);
}

int sky_graph_info(const sky_graph* g, uint32_t* V, uint32_t* E, uint32_t* max_degree) {
  if (!g) return fail(SKY_ERR_ARG, "sky_graph_info: null graph");
  if (V) *V = g->V;
  if (E) *E = g->E;
  if (max_degree) *max_degree = g->max_degree;
  return SKY_OK;
}

int sky_graph_download(const sky_graph* g, uint32_t* xadj, uint32_t* adjncy, float* adjwgt) {
  if (!g) return fail(SKY_ERR_ARG, "sky_graph_download: null graph");
  if (xadj) SKY_HIP(hipMemcpy(xadj, g->xadj, ((size_t)g->V + 1) * 4, hipMemcpyDeviceToHost));
  if (adjncy && g->E) SKY_HIP(hipMemcpy(adjncy, g->adjncy, (size_t)g->E * 4, hipMemcpyDeviceToHost));
  if (adjwgt && g->E) SKY_HIP(hipMemcpy(adjwgt, g->adjwgt, (size_t)g->E * 4, hipMemcpyDeviceToHost));
  return SKY_OK;
}

int sky_graph_device_ptrs(const sky_graph* g, const uint32_t** xadj, const uint32_t** adjncy, const float** adjwgt,
                          const sky_alias_entry** table, const int8_t** valid) {
  if (!g) return fail(SKY_ERR_ARG, "sky_graph_device_ptrs: null graph");
  if (xadj) *xadj = g->xadj;
  if (adjncy) *adjncy = g->adjncy;
  if (adjwgt) *adjwgt = g->adjwgt;
  if (table) *table = reinterpret_cast<const sky_alias_entry*>(g->table);
  if (valid) *valid = g->valid;
  return SKY_OK;
}

int sky_graph_free(sky_graph* g) {
  if (!g) return SKY_OK;
  void* ptrs[] = {g->xadj, g->adjncy, g->adjwgt, g->table, g->valid, g->walk_index, g->wgt_copy};
  for (void* p : ptrs)
    if (p) (void)hipFree(p);
  pool_release(g);
  free_build_scratch(g);
  free_tiled_scratch(g);
  if (g->live_report) (void)hipHostFree(g->live_report);
  delete g;
  return SKY_OK;
}

int sky_alias_build_all(sky_graph* g, double* seconds) {
  if (!g) return fail(SKY_ERR_ARG, "sky_alias_build_all: null graph");
  if (g->E && !g->adjwgt) return fail(SKY_ERR_STATE, "sky_alias_build_all: graph has no weights");
  return build_all_tables(g, seconds);
}

// Whether `bytes + 16` bytes are known to be readable from p on: the build kernels read whole 16-byte vectors.
static bool padded_allocation(const void* p, size_t bytes) {
  void* abase = nullptr;
  size_t asize = 0;
  if (hipMemGetAddressRange(reinterpret_cast<hipDeviceptr_t*>(&abase), &asize,
                            reinterpret_cast<hipDeviceptr_t>(const_cast<void*>(p))) != hipSuccess || !abase) {
    (void)hipGetLastError();
    return false;
  }
  const size_t before = (size_t)(static_cast<const char*>(p) - static_cast<const char*>(abase));
  return before <= asize && asize - before >= bytes + 16;
}

// A caller's array of E weights as the build kernels can read it: the array itself when its allocation is known to
// hold 16 more bytes, else a copy in a padded array that stays with the graph.
static int readable_weights(sky_graph* g, const float* weights_device, const float** use) {
  *use = weights_device;
  if (!g->E || !weights_device || padded_allocation(weights_device, (size_t)g->E * 4)) return SKY_OK;
  if (g->wgt_copy_cap < g->E) {
    if (g->wgt_copy) SKY_HIP(hipFree(g->wgt_copy));
    g->wgt_copy = nullptr;
    g->wgt_copy_cap = 0;
    SKY_TRY(alloc_padded(&g->wgt_copy, (size_t)g->E));
    g->wgt_copy_cap = g->E;
  }
  SKY_HIP(hipMemcpyAsync(g->wgt_copy, weights_device, (size_t)g->E * 4, hipMemcpyDeviceToDevice, g->stream));
  *use = g->wgt_copy;
  return SKY_OK;
}

int sky_alias_build_from_weights(sky_graph* g, const float* weights_device, double* seconds) {
  if (!g) return fail(SKY_ERR_ARG, "sky_alias_build_from_weights: null graph");
  if (g->E && !weights_device) return fail(SKY_ERR_ARG, "sky_alias_build_from_weights: null weights");
  // The build kernels read whole 16-byte vectors that may reach up to 12 bytes past the last weight.  The
  // caller's array is used where it lies only when its allocation is known to hold those bytes; otherwise the
  // weights are copied into a padded array that stays with the graph.
  const float* use = weights_device;
  SKY_TRY(readable_weights(g, weights_device, &use));
  float* const own = g->adjwgt;
  g->adjwgt = const_cast<float*>(use);  // the build only reads it
  const int rc = build_all_tables(g, seconds);
  g->adjwgt = own;
  return rc;
}

int sky_alias_download(const sky_graph* g, float* prob, uint32_t* alias, int8_t* valid) {
  if (!g) return fail(SKY_ERR_ARG, "sky_alias_download: null graph");
  if (!g->has_tables) return fail(SKY_ERR_STATE, "sky_alias_download: tables have not been built");
  if ((prob || alias) && g->E) {
    const size_t piece = std::min<size_t>(g->E, TABLE_PIECE);
    float* d_prob = nullptr;
    uint32_t* d_alias = nullptr;
    SKY_HIP(hipMalloc((void**)&d_prob, piece * 4));
    if (hipMalloc((void**)&d_alias, piece * 4) != hipSuccess) {
      (void)hipFree(d_prob);
      return fail(SKY_ERR_HIP, "sky_alias_download: no device memory for the staging arrays");
    }
    int rc = SKY_OK;
    for (size_t lo = 0; lo < g->E && rc == SKY_OK; lo += piece) {
      const size_t n = std::min(piece, (size_t)g->E - lo);
      hipLaunchKernelGGL(split_table_kernel, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, g->stream, g->table, lo, n,
                         d_prob, d_alias);
      if (prob && hipMemcpy(prob + lo, d_prob, n * 4, hipMemcpyDeviceToHost) != hipSuccess) rc = SKY_ERR_HIP;
      if (alias && hipMemcpy(alias + lo, d_alias, n * 4, hipMemcpyDeviceToHost) != hipSuccess) rc = SKY_ERR_HIP;
    }
    (void)hipFree(d_prob);
    (void)hipFree(d_alias);
    if (rc != SKY_OK) return fail(rc, "sky_alias_download: copy to host failed");
  }
  if (valid && g->V) SKY_HIP(hipMemcpy(valid, g->valid, (size_t)g->V, hipMemcpyDeviceToHost));
  return SKY_OK;
}

// A table from outside is data the walk and sample kernels index with: every alias must stay inside its row
// (or be SKY_INVALID in a row flagged invalid), every prob must be a probability.
static int check_tables(const uint32_t* xadj, uint32_t V, const float* prob, const uint32_t* alias,
                        const int8_t* valid) {
  for (uint32_t v = 0; v < V; ++v) {
    const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
    if (valid[v] != 0 && valid[v] != 1)
      return fail(SKY_ERR_ARG, "sky_alias_upload: valid[" + std::to_string(v) + "] is neither 0 nor 1");
    if (deg == 0 && valid[v])
      return fail(SKY_ERR_ARG, "sky_alias_upload: vertex " + std::to_string(v) + " has no edge but is flagged valid");
    for (uint32_t i = 0; i < deg; ++i) {
      const float p = prob[off + i];
      const uint32_t a = alias[off + i];
      if (!(p >= 0.0f && p <= 1.0f))
        return fail(SKY_ERR_ARG, "sky_alias_upload: prob of slot " + std::to_string(off + i) + " is not in [0, 1]");
      if (valid[v] ? a >= deg : a != SKY_INVALID)
        return fail(SKY_ERR_ARG, "sky_alias_upload: alias of slot " + std::to_string(off + i) + " (row of " +
                                     std::to_string(deg) + " entries, valid " + std::to_string((int)valid[v]) +
                                     ") is " + std::to_string(a));
    }
  }
  return SKY_OK;
}

int sky_alias_upload(sky_graph* g, const float* prob, const uint32_t* alias, const int8_t* valid) {
  if (!g || (g->E && (!prob || !alias)) || (g->V && !valid)) return fail(SKY_ERR_ARG, "sky_alias_upload: null pointer");
  {
    std::vector<uint32_t> xadj((size_t)g->V + 1);
    SKY_HIP(hipMemcpy(xadj.data(), g->xadj, xadj.size() * 4, hipMemcpyDeviceToHost));
    SKY_TRY(check_tables(xadj.data(), g->V, prob, alias, valid));
  }
  if (!g->table) SKY_TRY(alloc_padded(&g->table, (size_t)g->E));
  if (!g->valid) SKY_TRY(alloc_padded(&g->valid, (size_t)g->V));
  if (g->E) {
    const size_t piece = std::min<size_t>(g->E, TABLE_PIECE);
    float* d_prob = nullptr;
    uint32_t* d_alias = nullptr;
    SKY_HIP(hipMalloc((void**)&d_prob, piece * 4));
    if (hipMalloc((void**)&d_alias, piece * 4) != hipSuccess) {
      (void)hipFree(d_prob);
      return fail(SKY_ERR_HIP, "sky_alias_upload: no device memory for the staging arrays");
    }
    int rc = SKY_OK;
    for (size_t lo = 0; lo < g->E && rc == SKY_OK; lo += piece) {
      const size_t n = std::min(piece, (size_t)g->E - lo);
      if (hipMemcpy(d_prob, prob + lo, n * 4, hipMemcpyHostToDevice) != hipSuccess ||
          hipMemcpy(d_alias, alias + lo, n * 4, hipMemcpyHostToDevice) != hipSuccess)
        rc = SKY_ERR_HIP;
      else
        hipLaunchKernelGGL(join_table_kernel, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, g->stream, d_prob, d_alias, lo,
                           n, g->table);
    }
    if (rc == SKY_OK && hipStreamSynchronize(g->stream) != hipSuccess) rc = SKY_ERR_HIP;
    (void)hipFree(d_prob);
    (void)hipFree(d_alias);
    if (rc != SKY_OK) return fail(rc, "sky_alias_upload: copy to the device failed");
  }
  if (g->V) SKY_HIP(hipMemcpy(g->valid, valid, (size_t)g->V, hipMemcpyHostToDevice));
  g->has_tables = true;
  g->has_walk_index = false;
  return SKY_OK;
}

int sky_gen_seeds(uint64_t seed, uint32_t V, uint32_t N, uint32_t* seeds_device) {
  if (N && !seeds_device) return fail(SKY_ERR_ARG, "sky_gen_seeds: null pointer");
  if (V == 0) return fail(SKY_ERR_ARG, "sky_gen_seeds: empty graph");
  SKY_TRY(ensure_device());
  return gen_seeds(seed, V, N, seeds_device);
}

static int check_walk_args(const char* who, sky_graph* g, const uint32_t* seeds, uint32_t N, uint32_t len,
                           float stop_prob, const uint32_t* paths, const uint32_t* lengths) {
  if (!g) return fail(SKY_ERR_ARG, std::string(who) + ": null graph");
  if (N && (!seeds || !paths || !lengths)) return fail(SKY_ERR_ARG, std::string(who) + ": null pointer");
  if (!(stop_prob >= 0.0f && stop_prob <= 1.0f)) return fail(SKY_ERR_ARG, std::string(who) + ": stop_prob not in [0,1]");
  if ((uint64_t)N * ((uint64_t)len + 1) > (1ull << 40)) return fail(SKY_ERR_LIMIT, std::string(who) + ": output too large");
  return SKY_OK;
}

int sky_walk_offline(sky_graph* g, const uint32_t* seeds_device, uint32_t N, uint32_t len, float stop_prob,
                     uint64_t philox_seed, uint32_t* paths_device, uint32_t* lengths_device, uint64_t* sampled,
                     double* seconds) {
  SKY_TRY(check_walk_args("sky_walk_offline", g, seeds_device, N, len, stop_prob, paths_device, lengths_device));
  if (!g->has_tables) return fail(SKY_ERR_STATE, "sky_walk_offline: alias tables have not been built");
  return walk_offline(g, seeds_device, N, len, stop_prob, philox_seed, paths_device, lengths_device, sampled, seconds);
}

int sky_walk_index_build(sky_graph* g, double* seconds) {
  if (!g) return fail(SKY_ERR_ARG, "sky_walk_index_build: null graph");
  if (!g->has_tables) return fail(SKY_ERR_STATE, "sky_walk_index_build: alias tables have not been built");
  return build_walk_index(g, seconds);
}

int sky_walk_offline_noalloc(sky_graph* g, const uint32_t* seeds_device, uint32_t N, uint32_t len, float stop_prob,
                             uint64_t philox_seed, uint32_t* paths_device, uint32_t* lengths_device,
                             uint64_t* sampled_device) {
  SKY_TRY(check_walk_args("sky_walk_offline_noalloc", g, seeds_device, N, len, stop_prob, paths_device, lengths_device));
  if (!g->has_tables) return fail(SKY_ERR_STATE, "sky_walk_offline_noalloc: alias tables have not been built");
  return walk_offline_noalloc(g, seeds_device, N, len, stop_prob, philox_seed, paths_device, lengths_device,
                              sampled_device);
}

int sky_walk_online(sky_graph* g, int bias_kind, float p, float q, const uint32_t* seeds_device, uint32_t N,
                    uint32_t len, float stop_prob, uint64_t philox_seed, uint32_t* paths_device,
                    uint32_t* lengths_device, uint64_t* sampled, double* seconds) {
  SKY_TRY(check_walk_args("sky_walk_online", g, seeds_device, N, len, stop_prob, paths_device, lengths_device));
  if (bias_kind != SKY_BIAS_STATIC && bias_kind != SKY_BIAS_NODE2VEC && bias_kind != SKY_BIAS_NODE2VEC_REJECT)
    return fail(SKY_ERR_ARG, "sky_walk_online: unknown bias kind");
  if (bias_kind != SKY_BIAS_STATIC && !(p > 0.0f && q > 0.0f))
    return fail(SKY_ERR_ARG, "sky_walk_online: node2vec needs p > 0 and q > 0");
  return walk_online(g, bias_kind, p, q, seeds_device, N, len, stop_prob, philox_seed, paths_device, lengths_device,
                     sampled, seconds);
}

int sky_sample_layout(const uint32_t* fanout, uint32_t hops, uint64_t* length_per_sample,
                      uint64_t* size_of_sample_lengths) {
  if (!fanout || hops < 2 || hops > 8 || fanout[0] != 1)
    return fail(SKY_ERR_ARG, "sky_sample_layout: need 2..8 hops with fanout[0] == 1");
  uint64_t width = 1, lps = 0, slen = 0;
  for (uint32_t h = 0; h < hops; ++h) {
    if (fanout[h] == 0) return fail(SKY_ERR_ARG, "sky_sample_layout: zero fanout");
    width *= fanout[h];
    if (width > (1ull << 32)) return fail(SKY_ERR_LIMIT, "sky_sample_layout: fanout product too large");
    lps += width;
    if (h + 1 < hops) slen += width;
  }
  if (length_per_sample) *length_per_sample = lps;
  if (size_of_sample_lengths) *size_of_sample_lengths = slen;
  return SKY_OK;
}

static int sample_common(const char* who, bool online, sky_graph* g, const uint32_t* seeds, uint32_t N,
                         const uint32_t* fanout, uint32_t hops, uint64_t seed, uint32_t* data, uint32_t* sl,
                         uint64_t* sampled, double* seconds) {
  if (!g) return fail(SKY_ERR_ARG, std::string(who) + ": null graph");
  if (N && (!seeds || !data || !sl)) return fail(SKY_ERR_ARG, std::string(who) + ": null pointer");
  uint64_t lps = 0, slen = 0;
  SKY_TRY(sky_sample_layout(fanout, hops, &lps, &slen));
  if (!online && !g->has_tables) return fail(SKY_ERR_STATE, std::string(who) + ": alias tables have not been built");
  return sample_khop(g, online, seeds, N, fanout, hops, seed, data, sl, sampled, seconds);
}

struct sky_sample_session {
  sky::SampleSession* s;
  sky_graph* g;
};

int sky_sample_session_begin(sky_graph* g, const uint32_t* seeds_device, uint32_t N, const uint32_t* fanout, uint32_t hops,
                             uint64_t philox_seed, uint32_t* data_device, uint32_t* sample_lengths_device,
                             sky_sample_session** out) {
  if (!g || !out) return fail(SKY_ERR_ARG, "sky_sample_session_begin: null pointer");
  if (N && (!seeds_device || !data_device || !sample_lengths_device))
    return fail(SKY_ERR_ARG, "sky_sample_session_begin: null pointer");
  uint64_t lps = 0, slen = 0;
  SKY_TRY(sky_sample_layout(fanout, hops, &lps, &slen));
  g->has_tables = false;  // the rows are rebuilt from the caller's weights, hop by hop
  sky::SampleSession* s = nullptr;
  SKY_TRY(sample_session_begin(g, seeds_device, N, fanout, hops, philox_seed, data_device, sample_lengths_device, &s));
  *out = new sky_sample_session{s, g};
  return SKY_OK;
}
int sky_sample_session_frontier(sky_sample_session* s, uint32_t hop, const uint32_t** list_device,
                                const uint32_t** count_device, uint32_t* upper) {
  if (!s) return fail(SKY_ERR_ARG, "sky_sample_session_frontier: null session");
  return sample_session_frontier(s->s, hop, list_device, count_device, upper);
}
int sky_sample_session_hop(sky_sample_session* s, uint32_t hop, const float* weights_device) {
  if (!s) return fail(SKY_ERR_ARG, "sky_sample_session_hop: null session");
  const float* use = weights_device;
  SKY_TRY(readable_weights(s->g, weights_device, &use));
  return sample_session_hop(s->s, hop, use);
}
int sky_sample_session_end(sky_sample_session* s, uint64_t* sampled, double* seconds) {
  if (!s) return fail(SKY_ERR_ARG, "sky_sample_session_end: null session");
  const int rc = sample_session_end(s->s, sampled, seconds);
  delete s;
  return rc;
}

int sky_sample_offline(sky_graph* g, const uint32_t* seeds_device, uint32_t N, const uint32_t* fanout, uint32_t hops,
                       uint64_t philox_seed, uint32_t* data_device, uint32_t* sample_lengths_device,
                       uint64_t* sampled, double* seconds) {
  return sample_common("sky_sample_offline", false, g, seeds_device, N, fanout, hops, philox_seed, data_device,
                       sample_lengths_device, sampled, seconds);
}
int sky_sample_online(sky_graph* g, const uint32_t* seeds_device, uint32_t N, const uint32_t* fanout, uint32_t hops,
                      uint64_t philox_seed, uint32_t* data_device, uint32_t* sample_lengths_device, uint64_t* sampled,
                      double* seconds) {
  return sample_common("sky_sample_online", true, g, seeds_device, N, fanout, hops, philox_seed, data_device,
                       sample_lengths_device, sampled, seconds);
}

int sky_philox_selftest(const uint32_t* ctr_host, const uint32_t* key_host, uint32_t n, uint32_t* out_host) {
  if (n && (!ctr_host || !key_host || !out_host)) return fail(SKY_ERR_ARG, "sky_philox_selftest: null pointer");
  SKY_TRY(ensure_device());
  if (n == 0) return SKY_OK;
  return philox_selftest(ctr_host, key_host, n, out_host);
}

// name, smallest and largest accepted value of every knob, in the order of SkyOpt
struct OptionSpec {
  const char* name;
  long long lo, hi;
};
static const OptionSpec g_option_spec[OPT_COUNT] = {
    {"tiled_max_tiles", 1, 1ll << 22},
    {"row_merge", 0, 1},
    {"stream_min_edges", 0, 1ll << 40},
    {"stream_wide_min_edges", 0, 1ll << 40},
    {"walk_read_once", -1, 1},
    {"sample_distinct", 0, 1},
    {"small_in_place", -1, 1},
    {"build_streams", 0, 1},
    {"build_profile", 0, 1},
    {"walk_compact_every", 0, 1ll << 31},
    {"online_full_build", -1, 1},
    {"online_device_sized", 0, 1},
};
static int parse_option(const char* who, const char* name, long value, int* index, long long* stored) {
  if (!name) return fail(SKY_ERR_ARG, std::string(who) + ": null name");
  for (int i = 0; i < OPT_COUNT; ++i) {
    if (strcmp(name, g_option_spec[i].name)) continue;
    const OptionSpec& sp = g_option_spec[i];
    long long v = value;
    if (sp.lo == 0 && sp.hi == 1) v = value != 0;  // switches take any non-zero value as "on"
    if (i == OPT_TILED_MAX_TILES && v > sp.hi) v = sp.hi;
    if (v < sp.lo || v > sp.hi)
      return fail(SKY_ERR_ARG, std::string(who) + ": " + name + " takes " + std::to_string(sp.lo) + " .. " +
                                   std::to_string(sp.hi));
    *index = i;
    *stored = v;
    return SKY_OK;
  }
  return fail(SKY_ERR_ARG, std::string(who) + ": unknown option " + name);
}

int sky_set_option(const char* name, long value) {
  int i = 0;
  long long v = 0;
  SKY_TRY(parse_option("sky_set_option", name, value, &i, &v));
  g_option_value[i] = v;
  return SKY_OK;
}
int sky_graph_set_option(sky_graph* g, const char* name, long value) {
  if (!g) return fail(SKY_ERR_ARG, "sky_graph_set_option: null graph");
  int i = 0;
  long long v = 0;
  SKY_TRY(parse_option("sky_graph_set_option", name, value, &i, &v));
  g->opt_value[i] = v;
  g->opt_own[i] = true;
  return SKY_OK;
}
int sky_graph_unset_option(sky_graph* g, const char* name) {
  if (!g) return fail(SKY_ERR_ARG, "sky_graph_unset_option: null graph");
  if (!name) return fail(SKY_ERR_ARG, "sky_graph_unset_option: null name");
  for (int i = 0; i < OPT_COUNT; ++i)
    if (!strcmp(name, g_option_spec[i].name)) {
      g->opt_own[i] = false;
      return SKY_OK;
    }
  return fail(SKY_ERR_ARG, std::string("sky_graph_unset_option: unknown option ") + name);
}

int sky_last_build_profile(const sky_graph* g, const char** names, float* ms, uint64_t* edges, int max_entries) {
  if (!g) return 0;
  int n = 0;
  for (const auto& e : g->build_profile) {
    if (n >= max_entries) break;
    if (names) names[n] = e.name;
    if (ms) ms[n] = e.ms;
    if (edges) edges[n] = e.edges;
    ++n;
  }
  return n;
}

}  // extern "C"
