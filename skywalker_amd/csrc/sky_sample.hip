// k-hop neighbour sampling (replaces the fused sample_kernel and OfflineSample of
// src/offline_sample.cu:72-141,443-513, and sample_kernel / OnlineGBSampleNew of
// src/online_sample_new.cu:191-270,459-547).
//
// Output layout (include/sampler_result.cuh:226-260,421-426): per seed, hop h occupies
// width[h] = prod fanout[0..h] slots starting at offsets[h]; the children of slot s of hop h are
// slots s*fanout[h+1].. of hop h+1; sample_lengths holds one count per parent slot of every hop
// but the last.  A parent of degree deg with fanout k contributes all its neighbours when
// k >= deg, else k alias draws with replacement; draw i of slot s uses
// Philox(seed; seed index, s*k + i, h, DOM_SAMPLE).  One lane per (seed, slot, draw), one launch
// per hop: no device-side queues, and the result does not depend on scheduling.
//
// Online mode builds the table of every distinct frontier vertex, once, through the same
// kernels as the offline build (into the graph's table storage), then samples the hop.
#include <algorithm>
#include <vector>

#include "sky_graph.h"

namespace sky {

struct HopGeom {
  uint32_t h, k, fan_h;          // hop index, fanout of the next hop, fanout of this hop
  uint64_t width, off, off_next; // slots of hop h, where they start, where hop h+1 starts
  uint64_t loff, loff_prev;      // sample_lengths offsets of hop h and h-1
  uint64_t lps, slen;            // per-seed strides of data and sample_lengths
};

__device__ __forceinline__ bool slot_filled(const HopGeom& g, const uint32_t* sl, uint64_t si, uint64_t s) {
  if (g.h == 0) return true;
  // slots of a hop fit 32 bits (sky_sample_layout checks the fanout product)
  const uint32_t s32 = (uint32_t)s;
  return sl[si * g.slen + g.loff_prev + s32 / g.fan_h] > s32 % g.fan_h;
}

// One lane per (seed, slot, draw).  `narrow` (N * width * k below 2^32, the usual case) keeps the index
// arithmetic in 32 bits: three 64-bit divisions per lane cost more than the draw itself.
__global__ __launch_bounds__(256) void sample_hop_kernel(const uint32_t* __restrict__ xadj,
                                                         const uint32_t* __restrict__ adjncy,
                                                         const AliasEntry* __restrict__ table,
                                                         const int8_t* __restrict__ valid, uint64_t total,
                                                         uint32_t V, HopGeom g, uint64_t seed, bool narrow,
                                                         uint32_t* __restrict__ data,
                                                         uint32_t* __restrict__ sl) {
  const uint64_t tid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (tid < total) {
    uint64_t si, s;
    uint32_t i;
    if (narrow) {
      const uint32_t t32 = (uint32_t)tid, width = (uint32_t)g.width;
      const uint32_t parent = t32 / g.k;
      i = t32 - parent * g.k;
      const uint32_t si32 = parent / width;
      si = si32;
      s = parent - si32 * width;
    } else {
      const uint64_t per_seed = g.width * g.k;
      const uint64_t rem = tid % per_seed;
      si = tid / per_seed;
      s = rem / g.k;
      i = (uint32_t)(rem % g.k);
    }
    if (slot_filled(g, sl, si, s)) {
      const uint32_t v = data[si * g.lps + g.off + s];
      uint32_t o = 0, deg = 0;
      if (v < V && valid[v]) {  // a seed that does not exist, or a row without weight, has no children
        o = xadj[v];
        deg = xadj[v + 1] - o;
      }
      if (deg != 0) {
        uint32_t* out = data + si * g.lps + g.off_next + s * g.k;
        uint32_t cnt;
        if (g.k >= deg) {
          cnt = deg;
          if (i < deg) out[i] = adjncy[o + i];
        } else {
          cnt = g.k;
          const u32x4 r = philox(seed, (uint32_t)si, (uint32_t)(s * g.k + i), g.h, DOM_SAMPLE);
          const uint32_t col = __umulhi(r.x, deg);
          const AliasEntry e = table[o + col];
          const uint32_t cand = u24(r.y) < e.prob ? col : e.alias;
          out[i] = adjncy[o + cand];
        }
        if (i == 0) sl[si * g.slen + g.loff + s] = cnt;
      }
    }
  }
}

// Distinct children (the rule of the reference's online sampler, roll_atomic / roll_once of
// src/online_sample_new.cu:72-105: up to 11 rounds, a candidate whose slot of the row is already selected is
// dropped, a parent may end with fewer than k children), made sequential so that the result does not depend on
// scheduling: draw i of slot s tries Philox(seed; seed index, s*k + i, h + 256 t, DOM_SAMPLE) for t = 0..10 and
// keeps the first candidate slot that no earlier draw of this parent kept; the children are written densely in
// the order of i.  One lane per (seed, slot); the slots it has kept so far sit in LDS, one column per lane.
constexpr int DISTINCT_T = 128;          // threads per workgroup
constexpr uint32_t DISTINCT_MAX_K = 64;  // largest fanout of this rule
constexpr uint32_t DISTINCT_ROUNDS = 11;
__global__ __launch_bounds__(DISTINCT_T) void sample_hop_distinct_kernel(
    const uint32_t* __restrict__ xadj, const uint32_t* __restrict__ adjncy, const AliasEntry* __restrict__ table,
    const int8_t* __restrict__ valid, uint64_t total, uint32_t V, HopGeom g, uint64_t seed,
    uint32_t* __restrict__ data, uint32_t* __restrict__ sl) {
  __shared__ uint32_t s_taken[DISTINCT_MAX_K][DISTINCT_T];
  const uint64_t tid = (uint64_t)blockIdx.x * DISTINCT_T + threadIdx.x;
  if (tid >= total) return;
  const uint64_t si = tid / g.width, s = tid % g.width;
  if (!slot_filled(g, sl, si, s)) return;
  const uint32_t v = data[si * g.lps + g.off + s];
  if (v >= V || !valid[v]) return;
  const uint32_t o = xadj[v], deg = xadj[v + 1] - o;
  if (deg == 0) return;
  uint32_t* out = data + si * g.lps + g.off_next + s * g.k;
  uint32_t cnt = 0;
  if (g.k >= deg) {
    for (; cnt < deg; ++cnt) out[cnt] = adjncy[o + cnt];
  } else {
    for (uint32_t i = 0; i < g.k; ++i)
      for (uint32_t t = 0; t < DISTINCT_ROUNDS; ++t) {
        const u32x4 r = philox(seed, (uint32_t)si, (uint32_t)(s * g.k + i), g.h + 256u * t, DOM_SAMPLE);
        const uint32_t col = __umulhi(r.x, deg);
        const AliasEntry e = table[o + col];
        const uint32_t cand = u24(r.y) < e.prob ? col : e.alias;
        bool seen = false;
        for (uint32_t j = 0; j < cnt; ++j) seen = seen || s_taken[j][threadIdx.x] == cand;
        if (seen) continue;
        s_taken[cnt][threadIdx.x] = cand;
        out[cnt++] = adjncy[o + cand];
        break;
      }
  }
  sl[si * g.slen + g.loff + s] = cnt;
}

// Sampled edges of the call = sum of sample_lengths (as the reference counts them, src/main.cu:378-394): one pass
// at the end, one atomic per workgroup; a counter bumped by every wavefront of every hop is a hot spot.
__global__ __launch_bounds__(256) void sum_u32_kernel(const uint32_t* __restrict__ x, uint64_t n,
                                                      unsigned long long* __restrict__ out) {
  __shared__ unsigned long long s_w[4];
  unsigned long long t = 0;
  for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256u) t += x[i];
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) t += shfl_xor_u64(t, m);
  if ((threadIdx.x & 63) == 0) s_w[threadIdx.x >> 6] = t;
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned long long b = s_w[0] + s_w[1] + s_w[2] + s_w[3];
    if (b) atomicAdd(out, b);
  }
}

// Collects the distinct vertices of the filled slots of hop h whose table has not been built
// during this call: first setter of the vertex's bit appends it.  One counter update per workgroup of 1024
// lanes: every append of a launch goes through one word, and a word serves its atomics one after another
// (one update per wavefront made this kernel as long as the build it feeds).
constexpr int COLLECT_T = 1024;
__global__ __launch_bounds__(COLLECT_T) void frontier_collect_kernel(const uint32_t* __restrict__ data,
                                                                     const uint32_t* __restrict__ sl, uint64_t total,
                                                                     uint32_t V, HopGeom g, uint32_t* __restrict__ bitmap,
                                                                     uint32_t* __restrict__ list,
                                                                     uint32_t* __restrict__ count) {
  __shared__ uint32_t s_n[COLLECT_T / 64];
  __shared__ uint32_t s_base;
  const uint64_t tid = (uint64_t)blockIdx.x * COLLECT_T + threadIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  bool fresh = false, live = false;
  uint32_t v = 0;
  if (tid < total) {
    uint64_t si, s;
    if (total <= 0xFFFFFFFFull) {
      const uint32_t si32 = (uint32_t)tid / (uint32_t)g.width;
      si = si32;
      s = (uint32_t)tid - si32 * (uint32_t)g.width;
    } else {
      si = tid / g.width;
      s = tid % g.width;
    }
    if (slot_filled(g, sl, si, s)) {
      v = data[si * g.lps + g.off + s];
      live = v < V;
    }
  }
  // The draws of a hop land on a few well-connected vertices again and again: the lanes of the wavefront that hold
  // the same vertex send one atomic between them (the lanes take turns by distinct vertex, at most 64 short rounds).
  {
    unsigned long long todo = __ballot(live);
    while (todo) {
      const int first = __ffsll((long long)todo) - 1;
      const uint32_t v0 = (uint32_t)__shfl((int)v, first, 64);
      const unsigned long long same = __ballot(live && v == v0);
      if (lane == first) {
        const uint32_t bit = 1u << (v & 31);
        fresh = !(atomicOr(&bitmap[v >> 5], bit) & bit);
      }
      todo &= ~same;
    }
  }
  const unsigned long long m = __ballot(fresh);
  if (lane == 0) s_n[wave] = (uint32_t)__popcll(m);
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t n = 0;
#pragma unroll
    for (int w = 0; w < COLLECT_T / 64; ++w) n += s_n[w];
    s_base = n ? atomicAdd(count, n) : 0u;
  }
  __syncthreads();
  if (fresh) {
    uint32_t base = s_base;
    for (int w = 0; w < wave; ++w) base += s_n[w];
    list[base + (uint32_t)__popcll(m & ((1ull << lane) - 1ull))] = v;
  }
}

__global__ __launch_bounds__(256) void sample_init_kernel(const uint32_t* __restrict__ seeds, uint32_t N, uint64_t lps,
                                                          uint32_t* __restrict__ data) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i < N) data[(uint64_t)i * lps] = seeds[i];
}


// One call of the k-hop sampler, taken apart hop by hop: begin (outputs cleared, start vertices in place), then for
// every hop frontier (online: the distinct parents whose rows are not built yet), build (online: their rows) and
// draw, then end (count, time).  sample_khop runs the steps in turn; sky_sample_session_* hands them to callers that
// supply the weights of a frontier's rows themselves.
struct SampleSession {
  sky_graph* g = nullptr;
  bool online = false, dev_sized = false, distinct = false;
  const uint32_t* seeds = nullptr;
  uint32_t N = 0, hops = 0;
  uint64_t seed = 0;
  uint32_t *data = nullptr, *sample_lengths = nullptr;
  std::vector<uint32_t> fanout;
  std::vector<uint64_t> width, off, loff;
  uint64_t lps = 0, slen = 0;
  unsigned long long* d_sampled = nullptr;
  uint32_t *bitmap = nullptr, *list = nullptr, *d_count = nullptr;
  uint32_t frontier_upper = 0;   // most rows the last frontier can hold
  uint32_t frontier_count = 0;   // its size, when the host has read it (dev_sized false)
  EventTimer tm;
  explicit SampleSession(sky_graph* g_) : g(g_), tm(g_) {}

  HopGeom geom(uint32_t h) const {
    HopGeom hg;
    hg.h = h;
    hg.k = fanout[h + 1];
    hg.fan_h = fanout[h];
    hg.width = width[h];
    hg.off = off[h];
    hg.off_next = off[h + 1];
    hg.loff = loff[h];
    hg.loff_prev = h ? loff[h - 1] : 0;
    hg.lps = lps;
    hg.slen = slen;
    return hg;
  }

  int begin(bool online_, const uint32_t* seeds_, uint32_t N_, const uint32_t* fanout_, uint32_t hops_, uint64_t seed_,
            uint32_t* data_, uint32_t* sl_) {
    hipStream_t st = g->stream;
    online = online_;
    seeds = seeds_;
    N = N_;
    hops = hops_;
    seed = seed_;
    data = data_;
    sample_lengths = sl_;
    distinct = option(g, OPT_SAMPLE_DISTINCT) != 0;
    fanout.assign(fanout_, fanout_ + hops);
    if (distinct) {
      if (hops > 256) return fail(SKY_ERR_LIMIT, "sample: distinct children need at most 256 hops");
      for (uint32_t h = 1; h < hops; ++h)
        if (fanout[h] > DISTINCT_MAX_K) return fail(SKY_ERR_LIMIT, "sample: distinct children need fanouts of at most 64");
    }
    if (g->has_tables) online = false;  // every row is already there: nothing to build on the way
    // Without the option the host reads the size of every frontier and sizes the launches of its build exactly;
    // with it (the default) nothing inside the call waits for the device.
    dev_sized = online && build_rows_dev_possible(g) && option(g, OPT_ONLINE_DEVICE_SIZED) != 0;
    width.assign(hops, 0);
    off.assign(hops, 0);
    loff.assign(hops, 0);
    uint64_t wd = 1;
    for (uint32_t h = 0; h < hops; ++h) {
      wd *= fanout[h];
      width[h] = wd;
      off[h] = lps;
      lps += wd;
      if (h + 1 < hops) {
        loff[h] = slen;
        slen += wd;
      }
    }
    if ((uint64_t)N * lps > (1ull << 40)) return fail(SKY_ERR_LIMIT, "sample: output too large");
    const uint32_t words = (g->V + 31) / 32;
    SKY_TRY(pool_get(g, sky_graph::POOL_COUNTERS, 64, (void**)&d_sampled));
    d_count = reinterpret_cast<uint32_t*>(d_sampled + 1);
    SKY_HIP(hipMemsetAsync(d_sampled, 0, 8, st));
    if (N && slen) SKY_HIP(hipMemsetAsync(sample_lengths, 0, (size_t)N * slen * 4, st));
    if (online) {
      SKY_TRY(ensure_table_storage(g));
      if (dev_sized) SKY_TRY(ensure_class_census(g));  // once per graph
      SKY_TRY(prepare_build_scratch(g, g->V));
      SKY_TRY(pool_get(g, sky_graph::POOL_BITMAP, (size_t)words * 4, (void**)&bitmap));
      SKY_TRY(pool_get(g, sky_graph::POOL_LIST, (size_t)g->V * 4, (void**)&list));
    }
    SKY_TRY(tm.mark("start", 0));
    if (online) SKY_HIP(hipMemsetAsync(bitmap, 0, (size_t)words * 4, st));
    if (N) hipLaunchKernelGGL(sample_init_kernel, dim3((N + 255) / 256), dim3(256), 0, st, seeds, N, lps, data);
    return SKY_OK;
  }

  // Online: the distinct parents of hop h whose rows this call has not built yet, into `list`; their number stays in
  // the device word d_count (and is read by the host only when the build needs it there).
  int frontier(uint32_t h) {
    frontier_upper = frontier_count = 0;
    if (!online || !N) return SKY_OK;
    hipStream_t st = g->stream;
    const HopGeom hg = geom(h);
    const uint64_t slots = (uint64_t)N * hg.width;
    SKY_HIP(hipMemsetAsync(d_count, 0, 4, st));
    hipLaunchKernelGGL(frontier_collect_kernel, dim3((uint32_t)((slots + COLLECT_T - 1) / COLLECT_T)), dim3(COLLECT_T), 0,
                       st, data, sample_lengths, slots, g->V, hg, bitmap, list, d_count);
    frontier_upper = (uint32_t)std::min<uint64_t>(slots, g->V);
    if (!dev_sized) {
      SKY_HIP(hipMemcpyAsync(&frontier_count, d_count, 4, hipMemcpyDeviceToHost, st));
      SKY_HIP(hipStreamSynchronize(st));
    }
    return SKY_OK;
  }

  // Online: the rows of the last frontier, from `weights` (null: the graph's own).  The length of the list stays
  // on the device where it can: the kernels of the build find it there, and the host goes on to enqueue the hop
  // without waiting (the reference's sampler never leaves the device either, src/online_sample_new.cu:191-270).
  int build(const float* weights) {
    if (!online || !N || !frontier_upper) return SKY_OK;
    float* const own = g->adjwgt;
    if (weights) g->adjwgt = const_cast<float*>(weights);  // the build only reads it
    const int rc = dev_sized ? build_rows_dev(g, list, d_count, frontier_upper) : build_rows(g, list, frontier_count, nullptr);
    g->adjwgt = own;
    return rc;
  }

  int draw(uint32_t h) {
    if (!N) return SKY_OK;
    hipStream_t st = g->stream;
    const HopGeom hg = geom(h);
    const uint64_t total = (uint64_t)N * hg.width * hg.k;
    if (total > 0xFFFFFFFFull * 256ull) return fail(SKY_ERR_LIMIT, "sample: hop too large for one launch");
    if (distinct) {
      const uint64_t slots = (uint64_t)N * hg.width;
      hipLaunchKernelGGL(sample_hop_distinct_kernel, dim3((uint32_t)((slots + DISTINCT_T - 1) / DISTINCT_T)),
                         dim3(DISTINCT_T), 0, st, g->xadj, g->adjncy, g->table, g->valid, slots, g->V, hg, seed, data,
                         sample_lengths);
      return SKY_OK;
    }
    hipLaunchKernelGGL(sample_hop_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, st, g->xadj, g->adjncy,
                       g->table, g->valid, total, g->V, hg, seed, total <= 0xFFFFFFFFull, data, sample_lengths);
    return SKY_OK;
  }

  int end(uint64_t* sampled, double* seconds) {
    hipStream_t st = g->stream;
    if (N && slen) {
      const uint64_t n = (uint64_t)N * slen;
      hipLaunchKernelGGL(sum_u32_kernel, dim3((uint32_t)std::min<uint64_t>((n + 255) / 256, 1024)), dim3(256), 0, st,
                         sample_lengths, n, d_sampled);
    }
    SKY_TRY(tm.mark("sample", 0));
    SKY_TRY(tm.finish(nullptr, seconds));
    unsigned long long hcount = 0;
    SKY_HIP(hipMemcpy(&hcount, d_sampled, 8, hipMemcpyDeviceToHost));
    if (sampled) *sampled = hcount;
    return SKY_OK;
  }
};

int sample_khop(sky_graph* g, bool online, const uint32_t* seeds, uint32_t N, const uint32_t* fanout, uint32_t hops,
                uint64_t seed, uint32_t* data, uint32_t* sample_lengths, uint64_t* sampled, double* seconds) {
  SampleSession s(g);
  SKY_TRY(s.begin(online, seeds, N, fanout, hops, seed, data, sample_lengths));
  for (uint32_t h = 0; h + 1 < hops; ++h) {
    SKY_TRY(s.frontier(h));
    SKY_TRY(s.build(nullptr));
    SKY_TRY(s.draw(h));
  }
  return s.end(sampled, seconds);
}

// The same steps behind the C interface (sky_sample_session_*).
int sample_session_begin(sky_graph* g, const uint32_t* seeds, uint32_t N, const uint32_t* fanout, uint32_t hops,
                         uint64_t seed, uint32_t* data, uint32_t* sample_lengths, SampleSession** out) {
  SampleSession* s = new SampleSession(g);
  const int rc = s->begin(true, seeds, N, fanout, hops, seed, data, sample_lengths);
  if (rc != SKY_OK) {
    delete s;
    return rc;
  }
  *out = s;
  return SKY_OK;
}
int sample_session_frontier(SampleSession* s, uint32_t hop, const uint32_t** list, const uint32_t** count,
                            uint32_t* upper) {
  if (hop + 1 >= s->hops) return fail(SKY_ERR_ARG, "sky_sample_session_frontier: no such hop");
  SKY_TRY(s->frontier(hop));
  if (list) *list = s->list;
  if (count) *count = s->d_count;
  if (upper) *upper = s->frontier_upper;
  return SKY_OK;
}
int sample_session_hop(SampleSession* s, uint32_t hop, const float* weights) {
  if (hop + 1 >= s->hops) return fail(SKY_ERR_ARG, "sky_sample_session_hop: no such hop");
  SKY_TRY(s->build(weights));
  return s->draw(hop);
}
int sample_session_end(SampleSession* s, uint64_t* sampled, double* seconds) {
  const int rc = s->end(sampled, seconds);
  delete s;
  return rc;
}
bool sample_session_online(const SampleSession* s) { return s->online; }

}  // namespace sky
