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
constexpr int WALK_STAGE = 4;  // steps whose vertices leave together as one 16-byte store

typedef uint32_t path4u __attribute__((ext_vector_type(4), aligned(4)));

// One draw from the row of v.  With the walk index one 16-byte entry holds both possible next vertices (two
// cache lines per step: xadj and the entry); without it the neighbour id is a third gather.
template <bool INDEXED, bool ONCE>
__device__ __forceinline__ bool walk_draw(const uint32_t* __restrict__ xadj, const uint32_t* __restrict__ adjncy,
                                          const AliasEntry* __restrict__ table, const WalkEntry* __restrict__ index,
                                          const u32x4& r, uint32_t v, uint32_t& next) {
  const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
  if (deg == 0) return false;
  const uint32_t col = __umulhi(r.x, deg);
  if (INDEXED) {
    // like the table entry below: read once, so it should not push the row offsets out of L2
    typedef uint32_t idx4 __attribute__((ext_vector_type(4)));
    const idx4* ep = reinterpret_cast<const idx4*>(index + off + col);
    const idx4 eb = ONCE ? __builtin_nontemporal_load(ep) : *ep;
    WalkEntry e;
    e.prob = __uint_as_float(eb.x);
    e.alias = eb.y;
    e.nbr_col = eb.z;
    e.nbr_alias = eb.w;
    const bool keep = u24(r.y) < e.prob;
    if (!keep && e.alias == SKY_INVALID) return false;
    next = keep ? e.nbr_col : e.nbr_alias;
  } else {
    // On a graph whose tables are far larger than the caches the entry and the neighbour id are read once per
    // step, the row offsets of the well-connected vertices many times by many walkers: the two gathers then go
    // past the cache's usual replacement order so that they do not evict the offsets (1 M walkers x 80 steps on the
    // scale-26 graph: 2.16 -> 1.86 ms).  On a small graph the entries are hit again and stay ordinary loads.
    const AliasEntry e = ONCE ? load_entry_once(table + off + col) : table[off + col];
    const uint32_t cand = u24(r.y) < e.prob ? col : e.alias;
    if (cand == SKY_INVALID) return false;
    next = ONCE ? __builtin_nontemporal_load(adjncy + off + cand) : adjncy[off + cand];
  }
  return true;
}

// Steps [s_begin, s_end) of the walkers listed in `live` (null: walkers 0..n_live-1, which then also record
// their start vertex).  A walker that is still walking at s_end is appended to `next_live` when that list is
// given: the next launch then runs on full wavefronts again (walkers that reached a vertex without out-edges
// or stopped no longer hold a lane).  The vertices of WALK_STAGE steps leave as one store.
template <bool INDEXED, bool ONCE>
__global__ __launch_bounds__(WALK_BLOCK) void walk_offline_kernel(
    const uint32_t* __restrict__ xadj, const uint32_t* __restrict__ adjncy, const AliasEntry* __restrict__ table,
    const WalkEntry* __restrict__ index, const uint32_t* __restrict__ seeds, const uint32_t* __restrict__ live,
    const uint32_t* __restrict__ n_live_dev, uint32_t n_live, uint32_t V, uint32_t len, uint32_t s_begin,
    uint32_t s_end, float stop_prob, uint64_t seed, uint32_t* __restrict__ paths, uint32_t* __restrict__ lengths,
    uint32_t* __restrict__ next_live, uint32_t* __restrict__ n_next, unsigned long long* __restrict__ sampled,
    unsigned long long* __restrict__ block_partials) {
  __shared__ unsigned long long s_part[WALK_BLOCK / 64];
  const uint32_t t = blockIdx.x * WALK_BLOCK + threadIdx.x;
  if (n_live_dev) n_live = min(n_live, *n_live_dev);  // the list's length is only known on the device
  uint32_t steps = 0;
  bool walking = false;
  uint32_t i = 0;
  if (t < n_live) {
    i = live ? live[t] : t;
    uint32_t* path = paths + (size_t)i * (len + 1);
    uint32_t v;
    if (s_begin == 0) {
      v = seeds[i];
      path[0] = v;
    } else {
      v = path[s_begin];
    }
    uint32_t s = s_begin;
    walking = v < V;  // a start vertex that does not exist is recorded and never left
    while (walking && s < s_end) {
      uint32_t b[WALK_STAGE];
      uint32_t got = 0;
#pragma unroll
      for (int k = 0; k < WALK_STAGE; ++k) {
        b[k] = 0;
        if (walking && s + got < s_end) {
          const u32x4 r = philox(seed, i, s + got, 0, DOM_WALK);
          uint32_t nx = 0;
          if ((stop_prob > 0.0f && u24(r.z) < stop_prob) || !walk_draw<INDEXED, ONCE>(xadj, adjncy, table, index, r, v, nx)) {
            walking = false;
          } else {
            v = nx;
            b[k] = nx;
            got = k + 1;
          }
        }
      }
      uint32_t* dst = path + s + 1;
      if (got == WALK_STAGE) {
        path4u o;
        o.x = b[0]; o.y = b[1]; o.z = b[2]; o.w = b[3];
        *reinterpret_cast<path4u*>(dst) = o;
      } else {
#pragma unroll
        for (int k = 0; k < WALK_STAGE - 1; ++k)
          if ((uint32_t)k < got) dst[k] = b[k];
      }
      s += got;
    }
    steps = s - s_begin;
    if (!walking || s_end == len) lengths[i] = s;
    walking = walking && s_end < len;
  }
  if (next_live) {  // survivors, one atomic per wavefront
    const unsigned long long m = __ballot(walking);
    if (m) {
      const int lane = threadIdx.x & 63;
      uint32_t base = 0;
      if (lane == __ffsll((long long)m) - 1) base = atomicAdd(n_next, (uint32_t)__popcll(m));
      base = (uint32_t)__shfl((int)base, __ffsll((long long)m) - 1, 64);
      if (walking) next_live[base + (uint32_t)__popcll(m & ((1ull << lane) - 1ull))] = i;
    }
  }
  // exact 64-bit count of sampled edges (the reference reduces lengths through float, sampler_result.cuh:57-67)
  unsigned long long tot = steps;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) tot += shfl_xor_u64(tot, m);
  if (block_partials) {  // one sum per workgroup, added up by reduce_partials_kernel: no counter to clear
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = tot;
    __syncthreads();
    if (threadIdx.x == 0) {
      unsigned long long b = 0;
#pragma unroll
      for (int w = 0; w < WALK_BLOCK / 64; ++w) b += s_part[w];
      block_partials[blockIdx.x] = b;
    }
  } else if ((threadIdx.x & 63) == 0 && tot) {
    atomicAdd(sampled, tot);
  }
}

// Options walk_compact_every (0: one launch, every walker keeps its lane for the whole walk) and walk_read_once
// (-1: by the size of the tables, 0 / 1: never / always load entries as read-once data).
// Tables of more than 2 GiB (the last-level cache holds 256 MiB) are gathered from as read-once data.
static bool walk_reads_once(const sky_graph* g) {
  const long long mode = option(g, OPT_WALK_READ_ONCE);
  return mode < 0 ? (uint64_t)g->E * sizeof(AliasEntry) > (2ull << 30) : mode != 0;
}

template <bool INDEXED>
static void launch_walk(sky_graph* g, const uint32_t* seeds, const uint32_t* live, const uint32_t* n_live_dev,
                        uint32_t n_live, uint32_t len, uint32_t s_begin, uint32_t s_end, float stop_prob, uint64_t seed,
                        uint32_t* paths, uint32_t* lengths, uint32_t* next_live, uint32_t* n_next,
                        unsigned long long* sampled, unsigned long long* partials) {
  const dim3 grid((n_live + WALK_BLOCK - 1) / WALK_BLOCK), block(WALK_BLOCK);
  if (walk_reads_once(g))
    hipLaunchKernelGGL((walk_offline_kernel<INDEXED, true>), grid, block, 0, g->stream, g->xadj, g->adjncy, g->table,
                       INDEXED ? g->walk_index : nullptr, seeds, live, n_live_dev, n_live, g->V, len, s_begin, s_end, stop_prob,
                       seed, paths, lengths, next_live, n_next, sampled, partials);
  else
    hipLaunchKernelGGL((walk_offline_kernel<INDEXED, false>), grid, block, 0, g->stream, g->xadj, g->adjncy, g->table,
                       INDEXED ? g->walk_index : nullptr, seeds, live, n_live_dev, n_live, g->V, len, s_begin, s_end, stop_prob,
                       seed, paths, lengths, next_live, n_next, sampled, partials);
}

int walk_offline(sky_graph* g, const uint32_t* seeds, uint32_t N, uint32_t len, float stop_prob, uint64_t seed,
                 uint32_t* paths, uint32_t* lengths, uint64_t* sampled, double* seconds) {
  hipStream_t st = g->stream;
  unsigned long long* d_sampled = nullptr;
  SKY_TRY(pool_get(g, sky_graph::POOL_COUNTERS, 64, (void**)&d_sampled));
  const uint32_t every = (uint32_t)option(g, OPT_WALK_COMPACT_EVERY);
  const bool segmented = every > 0 && every < len && N > 0;
  const uint32_t nseg = segmented ? (len + every - 1) / every : 1;
  uint32_t *lists = nullptr, *counts = nullptr;
  if (segmented) {  // two lists of walker numbers used in turn, one survivor count per segment
    SKY_TRY(pool_get(g, sky_graph::POOL_LIST, (size_t)2 * N * 4, (void**)&lists));
    SKY_TRY(pool_get(g, sky_graph::POOL_BITMAP, (size_t)(nseg + 1) * 4, (void**)&counts));
    SKY_HIP(hipMemsetAsync(counts, 0, (size_t)(nseg + 1) * 4, st));
  }
  SKY_HIP(hipMemsetAsync(d_sampled, 0, 8, st));
  EventTimer tm(g);
  SKY_TRY(tm.mark("start", 0));
  auto run = [&](auto... a) {
    if (g->has_walk_index) launch_walk<true>(g, a...);
    else launch_walk<false>(g, a...);
  };
  if (N && !segmented) {
    run(seeds, (const uint32_t*)nullptr, (const uint32_t*)nullptr, N, len, 0u, len, stop_prob, seed, paths, lengths,
        (uint32_t*)nullptr, (uint32_t*)nullptr, d_sampled, (unsigned long long*)nullptr);
  } else if (N) {
    for (uint32_t k = 0; k < nseg; ++k) {
      const uint32_t s0 = k * every, s1 = std::min(len, s0 + every);
      const uint32_t* in = k ? lists + (size_t)((k - 1) & 1) * N : nullptr;
      uint32_t* out = s1 < len ? lists + (size_t)(k & 1) * N : nullptr;
      // the survivors of segment k - 1 are counted in counts[k]; the grid covers all N, blocks past the count leave
      run(seeds, in, k ? counts + k : (const uint32_t*)nullptr, N, len, s0, s1, stop_prob, seed, paths, lengths, out,
          counts + k + 1, d_sampled, (unsigned long long*)nullptr);
    }
  }
  SKY_TRY(tm.mark("walk", 0));
  SKY_TRY(tm.finish(nullptr, seconds));
  unsigned long long h = 0;
  SKY_HIP(hipMemcpy(&h, d_sampled, 8, hipMemcpyDeviceToHost));
  if (sampled) *sampled = h;
  return SKY_OK;
}

// ---------------------------------------------------------------- walk index
// Optional 16-byte entries {prob, alias, neighbour of this slot, neighbour of the alias slot} beside the 8-byte
// table: a step then reads one entry and needs no gather from adjncy.  Built from the finished tables by one pass
// over the slots; a tile of 1024 slots finds its rows through the row that holds the tile's first slot.
constexpr uint32_t IDX_TILE = 1024;
constexpr uint32_t IDX_ROWS = 4096;  // row offsets of a tile kept in LDS; tiles that span more rows search xadj itself

__global__ __launch_bounds__(256) void index_tile_rows_kernel(const uint32_t* __restrict__ xadj, uint32_t V,
                                                              uint32_t* __restrict__ row_of_tile) {
  const uint32_t v = blockIdx.x * 256u + threadIdx.x;
  if (v >= V) return;
  const uint32_t lo = xadj[v], hi = xadj[v + 1];
  for (uint64_t t = ((uint64_t)lo + IDX_TILE - 1) / IDX_TILE; t * IDX_TILE < hi; ++t) row_of_tile[t] = v;
}

__global__ __launch_bounds__(256) void index_fill_kernel(const uint32_t* __restrict__ xadj,
                                                         const uint32_t* __restrict__ adjncy,
                                                         const AliasEntry* __restrict__ table,
                                                         const uint32_t* __restrict__ row_of_tile, uint32_t ntiles,
                                                         uint32_t V, uint32_t E, WalkEntry* __restrict__ index) {
  __shared__ uint32_t s_x[IDX_ROWS];
  const uint32_t t = blockIdx.x;
  const uint32_t v0 = row_of_tile[t], v1 = t + 1 < ntiles ? row_of_tile[t + 1] : V - 1;
  const uint32_t rows = v1 - v0 + 1;  // rows v0..v1 hold every slot of the tile
  const bool in_lds = rows <= IDX_ROWS;
  if (in_lds)
    for (uint32_t k = threadIdx.x; k < rows; k += 256u) s_x[k] = xadj[v0 + k];
  __syncthreads();
  const uint32_t* x = in_lds ? s_x : xadj + v0;
#pragma unroll
  for (int k = 0; k < (int)(IDX_TILE / 256); ++k) {
    const uint32_t i = t * IDX_TILE + k * 256u + threadIdx.x;
    if (i >= E) continue;
    // the last row of v0..v1 that starts at or before slot i (rows without entries share their start with the
    // next row and are passed over)
    uint32_t lo = 0, n = rows;
    while (n > 1) {
      const uint32_t half = n >> 1;
      lo = x[lo + half] <= i ? lo + half : lo;
      n -= half;
    }
    const uint32_t off = x[lo];
    const AliasEntry e = table[i];
    WalkEntry w;
    w.prob = e.prob;
    w.alias = e.alias;
    w.nbr_col = adjncy[i];
    w.nbr_alias = e.alias == SKY_INVALID ? SKY_INVALID : adjncy[off + e.alias];
    index[i] = w;
  }
}

int build_walk_index(sky_graph* g, double* seconds) {
  hipStream_t st = g->stream;
  if (seconds) *seconds = 0;
  if (!g->walk_index) SKY_TRY(alloc_padded(&g->walk_index, (size_t)g->E));
  if (g->E == 0) return SKY_OK;
  const uint32_t ntiles = (g->E + IDX_TILE - 1) / IDX_TILE;
  uint32_t* row_of_tile = nullptr;
  SKY_TRY(pool_get(g, sky_graph::POOL_LIST, (size_t)ntiles * 4, (void**)&row_of_tile));
  EventTimer tm(g);
  SKY_TRY(tm.mark("start", 0));
  hipLaunchKernelGGL(index_tile_rows_kernel, dim3((g->V + 255) / 256), dim3(256), 0, st, g->xadj, g->V, row_of_tile);
  hipLaunchKernelGGL(index_fill_kernel, dim3(ntiles), dim3(256), 0, st, g->xadj, g->adjncy, g->table, row_of_tile,
                     ntiles, g->V, g->E, g->walk_index);
  SKY_TRY(tm.mark("index", 0));
  SKY_TRY(tm.finish(nullptr, seconds));
  g->has_walk_index = true;
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
  if (dev != g->device)  // the scratch array of the current device would be handed to kernels that read another device's graph
    return fail(SKY_ERR_STATE, "sky_walk_offline_noalloc: the graph lives on device " + std::to_string(g->device) +
                                   ", the current device is " + std::to_string(dev));
  if (!g_scratch_ptr[dev]) {  // once per device, with that device current: each GPU holds its own copy of the array
    unsigned long long* p = nullptr;
    SKY_HIP(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
    g_scratch_ptr[dev] = p;
  }
  unsigned long long* const partials = g_scratch_ptr[dev];
  hipStream_t st = g->stream;
  const uint32_t blocks = (N + WALK_BLOCK - 1) / WALK_BLOCK;
  if (blocks) {
    if (g->has_walk_index)
      launch_walk<true>(g, seeds, nullptr, nullptr, N, len, 0u, len, stop_prob, seed, paths, lengths, nullptr, nullptr,
                        nullptr, partials);
    else
      launch_walk<false>(g, seeds, nullptr, nullptr, N, len, 0u, len, stop_prob, seed, paths, lengths, nullptr, nullptr,
                         nullptr, partials);
  }
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
    float fp, float fq, float fmax, float stop_prob, uint64_t seed, bool once, uint32_t* __restrict__ paths,
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
        const AliasEntry e = once ? load_entry_once(table + off + col) : table[off + col];
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

// The same walk with 8 lanes per walker, for batches too small to fill the GPU with one walker per lane (a
// batch then lasts as long as its longest walker: steps x the chain of dependent loads of one step).  The lanes
// of a group hold the walker's state alike and search the previous row together: 8 probes per round narrow
// the range 9-fold, so a row of 100,000 entries takes 6 dependent loads instead of 17.  Same draws, same paths.
constexpr int N2V_G = 8;  // a batch of 40,000 walkers x 80 steps on the scale-24 graph, tables built inside: 2.81 ms with one lane per
                          // walker, 2.35 with 4, 2.25 with 8, 2.45 with 16, 2.59 with 32, 2.68 with 64
constexpr uint32_t N2V_GROUP_MAX_WALKERS = 1u << 18;
__device__ __forceinline__ unsigned long long group_ballot(bool p) {
  const unsigned long long b = __ballot(p) >> (lane_id() & (64u - N2V_G));
  return N2V_G == 64 ? b : b & ((1ull << (N2V_G & 63)) - 1ull);
}
// Every lane of the group must call this together with the same row, n and key.
// The first round's probes depend on the row alone: group_first_probe loads them as soon as the row is known
// (a step before the key is), and group_row_has takes the value.
__device__ __forceinline__ uint32_t group_first_probe(const uint32_t* __restrict__ row, uint32_t n) {
  const uint32_t gl = lane_id() & (N2V_G - 1);
  if (n <= (uint32_t)N2V_G) return 0xFFFFFFFFu;
  const uint32_t p = (gl + 1) * (n / (N2V_G + 1) + 1) - 1;
  return p < n ? row[p] : 0xFFFFFFFFu;
}
__device__ __forceinline__ bool group_row_has(const uint32_t* __restrict__ row, uint32_t n, uint32_t key, uint32_t x0) {
  const uint32_t gl = lane_id() & (N2V_G - 1);
  uint32_t lo = 0, len = n;  // if the key is in the row it is in [lo, lo + len)
  bool first_round = true;
  while (len > (uint32_t)N2V_G) {
    const uint32_t step = len / (N2V_G + 1) + 1, end = lo + len;
    const uint32_t p = lo + (gl + 1) * step - 1;           // probe gl: last element of part gl
    const uint32_t x = first_round ? x0 : (p < end ? row[p] : 0xFFFFFFFFu);  // no vertex has this id
    first_round = false;
    const uint32_t c = (uint32_t)__popcll(group_ballot(x < key));  // parts that lie wholly below the key
    lo += c * step;
    len = min(step, end - lo);
  }
  return group_ballot(gl < len && row[lo + gl] == key) != 0;
}

__global__ __launch_bounds__(WALK_BLOCK) void walk_n2v_reject_group_kernel(
    const uint32_t* __restrict__ xadj, const uint32_t* __restrict__ adjncy,
    const AliasEntry* __restrict__ table, const uint32_t* __restrict__ seeds, uint32_t N, uint32_t V, uint32_t len,
    float fp, float fq, float fmax, float stop_prob, uint64_t seed, bool once, uint32_t* __restrict__ paths,
    uint32_t* __restrict__ lengths, unsigned long long* __restrict__ sampled) {
  const uint32_t i = (blockIdx.x * WALK_BLOCK + threadIdx.x) / N2V_G;
  const bool first = (threadIdx.x & (N2V_G - 1)) == 0;  // the lane that writes for the group
  uint32_t s = 0;
  if (i < N) {
    uint32_t* path = paths + (size_t)i * (len + 1);
    uint32_t v = seeds[i], prev = 0, prev_off = 0, prev_deg = 0;
    if (first) path[0] = v;
    for (; s < len && v < V; ++s) {
      const uint32_t x0 = group_first_probe(adjncy + prev_off, prev_deg);  // in flight during the loads below
      u32x4 r = philox(seed, i, s, 0, DOM_WALK);
      if (stop_prob > 0.0f && u24(r.z) < stop_prob) break;
      const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
      if (deg == 0) break;
      uint32_t next = 0;
      bool dead = false;
      for (uint32_t t = 0;; ++t) {
        if (t) r = philox(seed, i, s, t, DOM_WALK);
        const uint32_t col = __umulhi(r.x, deg);
        const AliasEntry e = once ? load_entry_once(table + off + col) : table[off + col];
        const uint32_t cand = u24(r.y) < e.prob ? col : e.alias;
        if (cand == SKY_INVALID) {
          dead = true;
          break;
        }
        next = adjncy[off + cand];
        if (s == 0 || t >= 65536u) break;
        const float f = next == prev ? fp : (group_row_has(adjncy + prev_off, prev_deg, next, x0) ? 1.0f : fq);
        if (u24(r.w) * fmax < f) break;
      }
      if (dead) break;
      prev = v;
      prev_off = off;
      prev_deg = deg;
      v = next;
      if (first) path[s + 1] = v;
    }
    if (first) lengths[i] = s;
  }
  unsigned long long t = first ? s : 0u;
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
    if (N && N <= N2V_GROUP_MAX_WALKERS)
      hipLaunchKernelGGL(walk_n2v_reject_group_kernel,
                         dim3((uint32_t)(((uint64_t)N * N2V_G + WALK_BLOCK - 1) / WALK_BLOCK)), dim3(WALK_BLOCK), 0, st,
                         g->xadj, g->adjncy, g->table, seeds, N, g->V, len, fp, fq, fmax, stop_prob, seed, walk_reads_once(g), paths,
                         lengths, d_sampled);
    else if (N)
      hipLaunchKernelGGL(walk_n2v_reject_kernel, dim3((N + WALK_BLOCK - 1) / WALK_BLOCK), dim3(WALK_BLOCK), 0, st,
                         g->xadj, g->adjncy, g->table, seeds, N, g->V, len, fp, fq, fmax, stop_prob, seed, walk_reads_once(g), paths,
                         lengths, d_sampled);
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
