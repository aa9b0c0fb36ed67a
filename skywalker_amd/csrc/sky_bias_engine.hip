// The kernels that call a bias operator (include/skywalker_bias.h).  This file is compiled with -fgpu-rdc and
// linked with exactly one plug-in source, which defines sky_get_bias and sky_update_walker_state, into
// libskywalker_bias_<name>.so.  It works on graphs of libskywalker_hip.so through that library's C-ABI.
//
//   sky_bias_build_all    one lane per CSR slot evaluates the operator into a weight array, then the offline
//                         build of libskywalker_hip runs on that array (ConstructTable, src/createTable.cu:119-179)
//   sky_bias_walk_online  one workgroup per (walker, step) draws from the table of the current vertex under the
//                         walker's state without building it (OnlineWalkShMem, src/online_walk.cu:97-132)
#include <algorithm>
#include <string>

#include "../../include/skywalker_bias.h"
#include "sky_step_draw.h"

namespace {

thread_local std::string g_err;
int fail_hip(const char* what, hipError_t e) {
  g_err = std::string(what) + ": " + hipGetErrorString(e);
  return SKY_ERR_HIP;
}
#define BIAS_HIP(expr)                                   \
  do {                                                   \
    hipError_t _e = (expr);                              \
    if (_e != hipSuccess) return fail_hip(#expr, _e);    \
  } while (0)
#define BIAS_TRY(expr)             \
  do {                             \
    int _rc = (expr);              \
    if (_rc != SKY_OK) return _rc; \
  } while (0)

struct View {
  const uint32_t* xadj;
  const uint32_t* adjncy;
  const float* adjwgt;
  uint32_t V, E;
};
int view_of(sky_graph* g, View* v) {
  BIAS_TRY(sky_graph_info(g, &v->V, &v->E, nullptr));
  return sky_graph_device_ptrs(g, &v->xadj, &v->adjncy, &v->adjwgt, nullptr, nullptr);
}

// The operator's weights of a row as the step draw wants them: clamped, by slot.
struct OperatorRow {
  sky_row_view view;
  const sky_walker_state* st;
  const uint32_t* nbr;
  __device__ __forceinline__ float operator()(uint32_t k) const {
    return sky::clamp_weight(sky_get_bias(&view, k, nbr[k], st));
  }
};

// weights[slot] = operator(row of the slot, slot) with an empty walker state; one workgroup per 1024 vertices,
// each lane walks the rows of its vertices (rows are short on average; long rows are shared by the wavefront)
__global__ __launch_bounds__(256) void bias_weights_kernel(View g, float p, float q, float* __restrict__ out) {
  sky_walker_state st{};
  st.p = p;
  st.q = q;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = (blockIdx.x * 256u + threadIdx.x) >> 6;
  for (uint32_t k = 0; k < 64u; ++k) {  // the wavefront's 64 vertices in turn, its lanes side by side in the row
    const uint32_t v = wave * 64u + k;
    if (v >= g.V) break;
    sky_row_view row{g.xadj, g.adjncy, g.adjwgt, g.V, v, g.xadj[v], g.xadj[v + 1] - g.xadj[v]};
    for (uint32_t s = lane; s < row.deg; s += 64u) out[row.off + s] = sky_get_bias(&row, s, g.adjncy[row.off + s], &st);
  }
}

// The operator's weights of the rows listed in list[0 .. *count): one wavefront per row at a time, its lanes side
// by side in the row; the grid strides over the list, whose length only the device knows.
__global__ __launch_bounds__(256) void bias_frontier_weights_kernel(View g, float p, float q,
                                                                    const uint32_t* __restrict__ list,
                                                                    const uint32_t* __restrict__ count,
                                                                    float* __restrict__ out) {
  sky_walker_state st{};
  st.p = p;
  st.q = q;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t n = *count, waves = gridDim.x * 4u;
  for (uint32_t i = (blockIdx.x * 256u + threadIdx.x) >> 6; i < n; i += waves) {
    const uint32_t v = list[i];
    sky_row_view row{g.xadj, g.adjncy, g.adjwgt, g.V, v, g.xadj[v], g.xadj[v + 1] - g.xadj[v]};
    for (uint32_t s = lane; s < row.deg; s += 64u) out[row.off + s] = sky_get_bias(&row, s, g.adjncy[row.off + s], &st);
  }
}

__global__ __launch_bounds__(256) void bias_init_kernel(const uint32_t* __restrict__ seeds, uint32_t N, uint32_t len,
                                                        uint32_t V, float p, float q, uint32_t* __restrict__ paths,
                                                        uint32_t* __restrict__ lengths,
                                                        sky_walker_state* __restrict__ states) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= N) return;
  const uint32_t v = seeds[i];
  paths[(size_t)i * (len + 1)] = v;
  lengths[i] = v < V ? len : 0u;  // "still walking"; a walker that stops at step s stores s < len
  sky_walker_state st{};
  st.walker = i;
  st.p = p;
  st.q = q;
  states[i] = st;
}

// One workgroup per walker that is still walking: `live` lists them (null: walkers 0 .. gridDim.x - 1), *n_live says
// how many they are (the grid covers an upper bound that the host knows).
__global__ __launch_bounds__(sky::N2V_T) void bias_step_kernel(View g, uint32_t len, uint32_t s, float stop_prob,
                                                               uint64_t seed, const uint32_t* __restrict__ live,
                                                               const uint32_t* __restrict__ n_live,
                                                               uint32_t* __restrict__ paths,
                                                               uint32_t* __restrict__ lengths,
                                                               sky_walker_state* __restrict__ states) {
  if (live && blockIdx.x >= *n_live) return;
  const uint32_t i = live ? live[blockIdx.x] : blockIdx.x;
  const int tid = threadIdx.x;
  if (lengths[i] != len) return;  // stopped at an earlier step
  const sky::u32x4 r = sky::philox(seed, i, s, 0, sky::DOM_WALK);
  uint32_t* path = paths + (size_t)i * (len + 1);
  const uint32_t v = path[s];
  const uint32_t off = g.xadj[v], d = g.xadj[v + 1] - off;
  if ((stop_prob > 0.0f && sky::u24(r.z) < stop_prob) || d == 0) {
    if (tid == 0) lengths[i] = s;
    return;
  }
  OperatorRow row;
  row.view = sky_row_view{g.xadj, g.adjncy, g.adjwgt, g.V, v, off, d};
  row.st = states + i;
  row.nbr = g.adjncy + off;
  const uint32_t cand = sky::step_draw_slot(row, d, r);
  __syncthreads();  // every lane has read the state before it moves on
  if (tid == 0) {
    if (cand == sky::NONE_SLOT) {
      lengths[i] = s;
    } else {
      path[s + 1] = row.nbr[cand];
      sky_walker_state st = states[i];
      st.last = v;
      st.has_last = 1;
      sky_update_walker_state(&st, v);
      states[i] = st;
    }
  }
}

// The walkers of `in` (null: 0 .. n_first - 1) that still walk after the step, appended to `out`: one counter
// update per workgroup of 1024 lanes (every append goes through one word, which serves its atomics one by one).
__global__ __launch_bounds__(1024) void bias_compact_kernel(const uint32_t* __restrict__ in,
                                                            const uint32_t* __restrict__ n_in, uint32_t n_first,
                                                            const uint32_t* __restrict__ lengths, uint32_t len,
                                                            uint32_t* __restrict__ out, uint32_t* __restrict__ n_out) {
  __shared__ uint32_t s_n[16];
  __shared__ uint32_t s_base;
  const uint32_t n = in ? *n_in : n_first;
  const uint32_t idx = blockIdx.x * 1024u + threadIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t i = 0;
  bool alive = false;
  if (idx < n) {
    i = in ? in[idx] : idx;
    alive = lengths[i] == len;
  }
  const unsigned long long m = __ballot(alive);
  if (lane == 0) s_n[wave] = (uint32_t)__popcll(m);
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t t = 0;
    for (int w = 0; w < 16; ++w) t += s_n[w];
    s_base = t ? atomicAdd(n_out, t) : 0u;
  }
  __syncthreads();
  if (alive) {
    uint32_t base = s_base;
    for (int w = 0; w < wave; ++w) base += s_n[w];
    out[base + (uint32_t)__popcll(m & ((1ull << lane) - 1ull))] = i;
  }
}

__global__ __launch_bounds__(256) void bias_sum_kernel(const uint32_t* __restrict__ lengths, uint32_t N,
                                                       unsigned long long* __restrict__ out) {
  unsigned long long t = 0;
  for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < N; i += gridDim.x * 256u) t += lengths[i];
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) t += sky::shfl_xor_u64(t, m);
  if ((threadIdx.x & 63) == 0 && t) atomicAdd(out, t);
}

}  // namespace

extern "C" {

const char* sky_bias_last_error(void) { return g_err.c_str(); }

int sky_bias_build_all(sky_graph* g, float p, float q, double* seconds) {
  View v{};
  BIAS_TRY(view_of(g, &v));
  float* w = nullptr;
  BIAS_TRY(sky_device_malloc((size_t)v.E * 4 + 16, (void**)&w));
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int rc = SKY_OK;
  auto body = [&]() -> int {
    BIAS_HIP(hipEventCreate(&e0));
    BIAS_HIP(hipEventCreate(&e1));
    BIAS_HIP(hipEventRecord(e0, nullptr));
    if (v.V)
      hipLaunchKernelGGL(bias_weights_kernel, dim3((v.V + 255) / 256), dim3(256), 0, nullptr, v, p, q, w);
    BIAS_HIP(hipEventRecord(e1, nullptr));
    BIAS_HIP(hipStreamSynchronize(nullptr));
    BIAS_HIP(hipGetLastError());
    float ms = 0;
    BIAS_HIP(hipEventElapsedTime(&ms, e0, e1));
    double build_sec = 0;
    BIAS_TRY(sky_alias_build_from_weights(g, w, &build_sec));
    if (seconds) *seconds = ms * 1e-3 + build_sec;
    return SKY_OK;
  };
  rc = body();
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)sky_device_free(w);
  return rc;
}

int sky_bias_sample_online(sky_graph* g, float p, float q, const uint32_t* seeds, uint32_t N, const uint32_t* fanout,
                           uint32_t hops, uint64_t philox_seed, uint32_t* data, uint32_t* sample_lengths,
                           uint64_t* sampled, double* seconds) {
  if (!g) {
    g_err = "sky_bias_sample_online: null graph";
    return SKY_ERR_ARG;
  }
  View v{};
  BIAS_TRY(view_of(g, &v));
  float* w = nullptr;  // weights of the rows built so far, in their CSR slots; every other slot is never read
  BIAS_TRY(sky_device_malloc((size_t)v.E * 4 + 16, (void**)&w));
  sky_sample_session* s = nullptr;
  auto body = [&]() -> int {
    BIAS_TRY(sky_sample_session_begin(g, seeds, N, fanout, hops, philox_seed, data, sample_lengths, &s));
    for (uint32_t h = 0; h + 1 < hops; ++h) {
      const uint32_t *list = nullptr, *count = nullptr;
      uint32_t upper = 0;
      BIAS_TRY(sky_sample_session_frontier(s, h, &list, &count, &upper));
      if (upper) {
        const uint32_t blocks = std::min<uint32_t>((upper + 3) / 4, 8192u);
        hipLaunchKernelGGL(bias_frontier_weights_kernel, dim3(blocks), dim3(256), 0, nullptr, v, p, q, list, count, w);
        BIAS_HIP(hipGetLastError());
      }
      BIAS_TRY(sky_sample_session_hop(s, h, w));
    }
    return SKY_OK;
  };
  int rc = body();
  if (s) {
    const int rc_end = sky_sample_session_end(s, sampled, seconds);
    if (rc == SKY_OK) rc = rc_end;
  }
  (void)sky_device_free(w);
  return rc;
}

int sky_bias_walk_online(sky_graph* g, float p, float q, const uint32_t* seeds, uint32_t N, uint32_t len,
                         float stop_prob, uint64_t philox_seed, uint32_t* paths, uint32_t* lengths, uint64_t* sampled,
                         double* seconds) {
  if (!g || (N && (!seeds || !paths || !lengths))) {
    g_err = "sky_bias_walk_online: null pointer";
    return SKY_ERR_ARG;
  }
  if (!(stop_prob >= 0.0f && stop_prob <= 1.0f) || !(p > 0.0f) || !(q > 0.0f)) {
    g_err = "sky_bias_walk_online: need 0 <= stop_prob <= 1, p > 0, q > 0";
    return SKY_ERR_ARG;
  }
  View v{};
  BIAS_TRY(view_of(g, &v));
  sky_walker_state* states = nullptr;
  unsigned long long* d_sampled = nullptr;
  uint32_t *lists = nullptr, *counts = nullptr, *report = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  auto body = [&]() -> int {
    BIAS_TRY(sky_device_malloc((size_t)N * sizeof(sky_walker_state) + 16, (void**)&states));
    BIAS_TRY(sky_device_malloc(8, (void**)&d_sampled));
    BIAS_HIP(hipMemsetAsync(d_sampled, 0, 8, nullptr));
    BIAS_TRY(sky_device_malloc((size_t)2 * N * 4 + 16, (void**)&lists));
    BIAS_TRY(sky_device_malloc(((size_t)len + 2) * 4, (void**)&counts));
    BIAS_HIP(hipMemsetAsync(counts, 0, ((size_t)len + 2) * 4, nullptr));
    BIAS_HIP(hipHostMalloc((void**)&report, ((size_t)len + 1) * 4, hipHostMallocDefault));
    for (uint32_t k = 0; k <= len; ++k) report[k] = 0xFFFFFFFFu;  // "not reported yet"
    BIAS_HIP(hipEventCreate(&e0));
    BIAS_HIP(hipEventCreate(&e1));
    BIAS_HIP(hipEventRecord(e0, nullptr));
    if (N) {
      const uint32_t blocks = (N + 255) / 256;
      hipLaunchKernelGGL(bias_init_kernel, dim3(blocks), dim3(256), 0, nullptr, seeds, N, len, v.V, p, q, paths,
                         lengths, states);
      // A step launches workgroups for the walkers that still walk, not for all N: after every step the survivors
      // are appended to a list the next step reads (the reference's walker queue, include/sampler_result.cuh:646-669).
      // The list's length stays on the device; the host sizes the next launches from the lengths that have come back
      // so far through pinned memory (they can only shrink), reads them without waiting, and stops once one is 0.
      uint32_t upper = N;
      for (uint32_t s = 0; s < len && upper; ++s) {
        const uint32_t* in = s ? lists + (size_t)((s - 1) & 1) * N : nullptr;
        uint32_t* out = lists + (size_t)(s & 1) * N;
        hipLaunchKernelGGL(bias_step_kernel, dim3(upper), dim3(sky::N2V_T), 0, nullptr, v, len, s, stop_prob, philox_seed,
                           in, s ? counts + s : nullptr, paths, lengths, states);
        hipLaunchKernelGGL(bias_compact_kernel, dim3((upper + 1023) / 1024), dim3(1024), 0, nullptr, in,
                           s ? counts + s : nullptr, N, lengths, len, out, counts + s + 1);
        BIAS_HIP(hipMemcpyAsync(&report[s], counts + s + 1, 4, hipMemcpyDeviceToHost, nullptr));
        for (uint32_t k = 0; k <= s; ++k) {
          const uint32_t seen = *(volatile uint32_t*)&report[k];
          if (seen != 0xFFFFFFFFu && seen < upper) upper = seen;
        }
      }
      hipLaunchKernelGGL(bias_sum_kernel, dim3(blocks < 1024 ? blocks : 1024), dim3(256), 0, nullptr, lengths, N,
                         d_sampled);
    }
    BIAS_HIP(hipEventRecord(e1, nullptr));
    BIAS_HIP(hipStreamSynchronize(nullptr));
    BIAS_HIP(hipGetLastError());
    float ms = 0;
    BIAS_HIP(hipEventElapsedTime(&ms, e0, e1));
    unsigned long long h = 0;
    BIAS_HIP(hipMemcpy(&h, d_sampled, 8, hipMemcpyDeviceToHost));
    if (sampled) *sampled = h;
    if (seconds) *seconds = ms * 1e-3;
    return SKY_OK;
  };
  const int rc = body();
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (states) (void)sky_device_free(states);
  if (d_sampled) (void)sky_device_free(d_sampled);
  if (lists) (void)sky_device_free(lists);
  if (counts) (void)sky_device_free(counts);
  if (report) (void)hipHostFree(report);
  return rc;
}

}  // extern "C"
