// Alias tables of rows of 8190..65533 entries: one workgroup streams the row three times and
// keeps the row's heavies in LDS.
//
// The table is the same pure function of the weights as everywhere else (see sky_build.hip).
// Only the heavies of a row need random access: a light's alias is the first heavy whose surplus
// prefix exceeds the light's exclusive deficit prefix, and a heavy's residual probability belongs
// to the one light whose deficit interval (SL - D, SL] contains the heavy's surplus prefix.  So
//   pass A  exact sum of the weights -> ledger
//   pass B  classify, running surplus prefix; heavies compacted into LDS in slot order:
//           {surplus prefix, slot}, 10 bytes each
//   pass C  classify again, running deficit prefix; every light searches the heavy list once
//           (alias) and finishes the heavies whose prefix falls into its interval (usually none,
//           sometimes one); every heavy takes the next heavy of the list as alias, or {1, itself}
//           when it is the last heavy or no light reaches it.
// A heavy's probability and alias are separate 4-byte stores by different threads of the workgroup.
// The second and third pass read the weights from L2.  Rows with more heavies than the LDS list
// holds are appended to `deferred` and left untouched (the tile-parallel path builds them).
#include "sky_build_common.h"
#include "sky_graph.h"

namespace sky {

constexpr int ST_T = 512;                 // threads per row
constexpr int ST_PER = 8;                 // consecutive slots per thread and chunk
constexpr int ST_CH = ST_T * ST_PER;      // slots per chunk
constexpr int ST_NW = ST_T / 64;
constexpr uint32_t ST_CAP = 8063;         // heavies per row kept in LDS (and one sentinel): two workgroups share a CU's 160 KB
static_assert(STREAM_MAX_DEG + 3 <= 65536, "heavy slots are stored as 16-bit numbers");

struct StreamRow {
  uint32_t base, lead, span;
};

// The 8 weights of this thread in chunk c (span slots c*ST_CH + 8*tid ...) as loaded; zeros past the row.
// Whether any slot of wavefront `wave` in chunk c lies inside the row's span.
__device__ __forceinline__ bool wave_in_row(const StreamRow& r, uint32_t c, int wave) {
  return c * ST_CH + (uint32_t)(ST_PER * 64) * (uint32_t)wave < r.span;
}

struct RawChunk {
  float4 q[ST_PER / 4];
};
__device__ __forceinline__ RawChunk fetch_chunk(const float* __restrict__ wgt, const StreamRow& r, uint32_t c,
                                                int tid) {
  RawChunk x;
#pragma unroll
  for (int q = 0; q < ST_PER / 4; ++q) {
    const uint32_t pos = c * ST_CH + (uint32_t)ST_PER * tid + 4u * q;
    x.q[q] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (pos < r.span) x.q[q] = *reinterpret_cast<const float4*>(wgt + r.base + pos);
  }
  return x;
}
// Clamped weights as doubles (0 outside the row) and the mask of slots that belong to the row.
__device__ __forceinline__ uint32_t unpack_chunk(const RawChunk& x, const StreamRow& r, uint32_t c, int tid,
                                                 double (&wd)[ST_PER]) {
  uint32_t live = 0;
#pragma unroll
  for (int q = 0; q < ST_PER / 4; ++q) {
    const uint32_t pos = c * ST_CH + (uint32_t)ST_PER * tid + 4u * q;
    const float xs[4] = {x.q[q].x, x.q[q].y, x.q[q].z, x.q[q].w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t idx = pos + k;
      const bool in = idx >= r.lead && idx < r.span;
      if (in) live |= 1u << (q * 4 + k);
      wd[q * 4 + k] = (double)(in ? clamp_weight(xs[k]) : 0.0f);
    }
  }
  return live;
}

// Exclusive prefix over the workgroup (thread order) of one u64 and one u32 per thread, plus totals.
// One barrier: consecutive calls must alternate between two sets of s_a / s_c (a wavefront may start
// the next call while others still read this one's sums; it cannot start the one after that before
// every wavefront has passed the next call's barrier).
__device__ __forceinline__ void stream_excl(uint64_t a, uint32_t c, uint64_t* s_a, uint32_t* s_c, uint64_t& ex_a,
                                            uint32_t& ex_c, uint64_t& tot_a, uint32_t& tot_c) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint64_t ia = group_scan_u64<64>(a);
  const uint32_t ic = group_scan_u32<64>(c);
  if (lane == 63) {
    s_a[wave] = ia;
    s_c[wave] = ic;
  }
  __syncthreads();
  uint64_t ra = 0;
  uint32_t rc = 0;
  ex_a = ia - a;
  ex_c = ic - c;
#pragma unroll
  for (int w = 0; w < ST_NW; ++w) {
    if (w == wave) {
      ex_a += ra;
      ex_c += rc;
    }
    ra += s_a[w];
    rc += s_c[w];
  }
  tot_a = ra;
  tot_c = rc;
}

// For M keys at once: number of entries of the sorted LDS array a[0..n), n >= 1, that are <= key[m].
// The M chains of dependent LDS reads advance in lockstep, so their latencies overlap.
template <int M>
__device__ __forceinline__ void count_le(const uint64_t* a, uint32_t n, const uint64_t (&key)[M], uint32_t (&out)[M]) {
  const uint32_t hb = 1u << (31 - __clz((int)n));
  uint32_t cur[M];
  {
    const uint64_t v = a[hb - 1];
#pragma unroll
    for (int m = 0; m < M; ++m) cur[m] = v <= key[m] ? n - hb : 0u;
  }
  for (uint32_t step = hb >> 1; step >= 1; step >>= 1) {
    uint64_t v[M];
#pragma unroll
    for (int m = 0; m < M; ++m) v[m] = a[cur[m] + step - 1];
#pragma unroll
    for (int m = 0; m < M; ++m) cur[m] = v[m] <= key[m] ? cur[m] + step : cur[m];
  }
  uint64_t v[M];
#pragma unroll
  for (int m = 0; m < M; ++m) v[m] = a[cur[m]];
#pragma unroll
  for (int m = 0; m < M; ++m) out[m] = cur[m] + (v[m] <= key[m] ? 1u : 0u);
}

__global__ __launch_bounds__(ST_T) void build_stream_kernel(const RowRef* __restrict__ vlist,
                                                            const float* __restrict__ wgt,
                                                            AliasEntry* __restrict__ table,
                                                            int8_t* __restrict__ valid,
                                                            RowRef* __restrict__ deferred,
                                                            uint32_t* __restrict__ n_deferred) {
  __shared__ uint64_t s_sh[ST_CAP + 1];    // surplus prefix of the row's h-th heavy
  __shared__ uint16_t s_slot[ST_CAP + 1];  // its span slot
  __shared__ WSum3 s_w[ST_NW];
  __shared__ uint64_t s_a[2][ST_NW];  // two sets of wavefront sums, used alternately
  __shared__ uint32_t s_c[2][ST_NW];
  const RowRef rr = vlist[blockIdx.x];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  StreamRow r;
  r.base = rr.off & ~3u;
  r.lead = rr.off - r.base;
  r.span = r.lead + rr.d;
  const uint32_t nch = (r.span + ST_CH - 1) / ST_CH;

  // ---- pass A: exact sum
  WSum3 sum{0.0, 0.0, 0.0};
  RawChunk nx = fetch_chunk(wgt, r, 0, tid);  // every loop below requests chunk c + 1 before it works on chunk c
  for (uint32_t c = 0; c < nch; ++c) {
    const RawChunk cur = nx;
    if (c + 1 < nch) nx = fetch_chunk(wgt, r, c + 1, tid);
    if (!wave_in_row(r, c, wave)) continue;
    double wd[ST_PER];
    unpack_chunk(cur, r, c, tid, wd);
#pragma unroll
    for (int j = 0; j < ST_PER; ++j) wsum3_add(sum, wd[j]);
  }
  nx = fetch_chunk(wgt, r, 0, tid);
  sum = group_sum_wsum3<64>(sum);
  if (lane == 0) s_w[wave] = sum;
  __syncthreads();
  sum = s_w[0];
#pragma unroll
  for (int i = 1; i < ST_NW; ++i) {
    sum.top += s_w[i].top;
    sum.mid += s_w[i].mid;
    sum.low += s_w[i].low;
  }
  if (sum.top + sum.mid + sum.low == 0.0) {
    for (uint32_t c = 0; c < nch; ++c)
#pragma unroll
      for (int j = 0; j < ST_PER; ++j) {
        const uint32_t idx = c * ST_CH + (uint32_t)ST_PER * tid + j;
        if (idx >= r.lead && idx < r.span) table[r.base + idx] = AliasEntry{0.0f, SKY_INVALID};
      }
    if (tid == 0) valid[rr.v] = 0;
    return;
  }
  const Ledger L = make_ledger_small(rr.d, wsum3_to_double(sum));

  // ---- pass B: the heavies, in slot order.  Whether an entry is heavy is a monotone function of its
  // clamped weight (p = fl(w * scale) and t = fma(p, 2^F, -2^F) are monotone, heavy iff t >= 0.5), so one
  // compare against the smallest heavy weight of this row decides it; the surplus is then computed for the
  // heavies alone, from the compacted list.
  uint32_t thr_bits;  // bit pattern of the smallest clamped weight that is heavy (above 2^32: none is)
  {
    auto is_heavy = [&](uint32_t bits) {
      const double p = (double)__uint_as_float(bits) * L.scale;
      return fma(p, L.fs, -L.fs) >= 0.5;
    };
    const double est = (1.0 + 0.5 * L.inv_fs) / L.scale;
    constexpr uint32_t MAXW = 0x4F800000u;  // 2^32
    uint32_t bits = est >= 4294967296.0 ? MAXW : __float_as_uint((float)est);
    int guard = 0;
    while (bits > 0 && is_heavy(bits - 1) && guard < 64) {
      --bits;
      ++guard;
    }
    while (bits <= MAXW && !is_heavy(bits) && guard < 64) {
      ++bits;
      ++guard;
    }
    if (guard >= 64) {  // the estimate is within a step or two of the boundary; anything else: leave the row
      if (tid == 0) deferred[atomicAdd(n_deferred, 1u)] = rr;
      return;
    }
    thr_bits = bits;
  }
  float* s_w32 = reinterpret_cast<float*>(s_sh);  // weight of heavy h in the low half of s_sh[h], until its prefix replaces it
  uint32_t carry_c = 0;
  bool overflow = false;
  for (uint32_t c = 0; c < nch; ++c) {
    const RawChunk cur = nx;
    if (c + 1 < nch) nx = fetch_chunk(wgt, r, c + 1, tid);
    float cw[ST_PER];
    uint32_t heavy = 0;
    if (wave_in_row(r, c, wave))
#pragma unroll
    for (int q = 0; q < ST_PER / 4; ++q) {
      const uint32_t pos = c * ST_CH + (uint32_t)ST_PER * tid + 4u * q;
      const float xs[4] = {cur.q[q].x, cur.q[q].y, cur.q[q].z, cur.q[q].w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t idx = pos + k;
        cw[q * 4 + k] = clamp_weight(xs[k]);
        if (idx >= r.lead && idx < r.span && __float_as_uint(cw[q * 4 + k]) >= thr_bits) heavy |= 1u << (q * 4 + k);
      }
    }
    uint64_t ex_u, tot_u;
    uint32_t ex_c, tot_c;
    stream_excl(0ull, (uint32_t)__popc(heavy), s_a[c & 1], s_c[c & 1], ex_u, ex_c, tot_u, tot_c);
    if (carry_c + tot_c > ST_CAP) {  // uniform
      overflow = true;
      break;
    }
    uint32_t rank = carry_c + ex_c;
#pragma unroll
    for (int j = 0; j < ST_PER; ++j)
      if ((heavy >> j) & 1) {
        s_w32[2 * rank] = cw[j];
        s_slot[rank] = (uint16_t)(c * ST_CH + (uint32_t)ST_PER * tid + j);
        ++rank;
      }
    carry_c += tot_c;
  }
  if (overflow) {
    if (tid == 0) deferred[atomicAdd(n_deferred, 1u)] = rr;
    return;
  }
  __syncthreads();  // the heavy list is complete
  const uint32_t nh = carry_c;
  {
    // surplus prefix of the list: 16 consecutive heavies per thread
    constexpr int HP = 16;
    static_assert(ST_CAP < (uint32_t)ST_T * HP, "one round covers the list");
    uint64_t u[HP];
    uint64_t su = 0;
#pragma unroll
    for (int k = 0; k < HP; ++k) {
      const uint32_t h = (uint32_t)HP * tid + k;
      if (h < nh) su += classify_fast((double)s_w32[2 * h], true, L).amount;
      u[k] = su;
    }
    uint64_t ex_u, tot_u;
    uint32_t ex_c, tot_c;
    stream_excl(su, 0u, s_a[0], s_c[0], ex_u, ex_c, tot_u, tot_c);
#pragma unroll
    for (int k = 0; k < HP; ++k) {
      const uint32_t h = (uint32_t)HP * tid + k;
      if (h < nh) s_sh[h] = ex_u + u[k];
    }
  }
  __syncthreads();
  if (tid == 0) {  // sentinel after the list; the first barrier of pass C publishes it
    s_sh[nh] = ~0ull;
    s_slot[nh] = nh ? s_slot[nh - 1] : (uint16_t)0;
  }

  // ---- pass C: every entry
  uint64_t carry_d = 0;  // deficits so far; the row's total deficit after the last chunk
  carry_c = 0;
  nx = fetch_chunk(wgt, r, 0, tid);
  for (uint32_t c = 0; c < nch; ++c) {
    const RawChunk cur = nx;
    if (c + 1 < nch) nx = fetch_chunk(wgt, r, c + 1, tid);
    const bool on = wave_in_row(r, c, wave);  // a wavefront past the row's end only takes part in the scan
    uint32_t live = 0;
    float op[ST_PER];
    uint64_t dl[ST_PER];
    uint32_t heavy = 0;
    uint64_t run = 0;
    if (on) {
      double wd[ST_PER];
      live = unpack_chunk(cur, r, c, tid, wd);
#pragma unroll
      for (int j = 0; j < ST_PER; ++j) {
        const Entry e = classify_fast(wd[j], (live >> j) & 1, L);
        op[j] = (float)e.p;
        dl[j] = e.heavy ? 0 : e.amount;
        run += dl[j];
        if (e.heavy) heavy |= 1u << j;
      }
    }
    uint64_t ex_d, tot_d;
    uint32_t ex_c, tot_c;
    stream_excl(run, (uint32_t)__popc(heavy), s_a[c & 1], s_c[c & 1], ex_d, ex_c, tot_d, tot_c);
    if (!on) {
      carry_d += tot_d;
      carry_c += tot_c;
      continue;
    }
    // b = heavies whose surplus prefix is <= the deficits before this thread's slots: one search; from
    // there the thread's lights walk the list, each stopping at its own deficit prefix
    uint64_t sl = carry_d + ex_d;
    uint32_t b = 0;
    if (nh) {
      const uint64_t k1[1] = {sl};
      uint32_t o1[1];
      count_le<1>(s_sh, nh, k1, o1);
      b = o1[0];
    }
    uint64_t hv = s_sh[b];          // ~0 once the list is exhausted
    uint32_t hslot = s_slot[b];     // then: the last heavy
    const uint32_t pos0 = c * ST_CH + (uint32_t)ST_PER * tid;
#pragma unroll
    for (int j = 0; j < ST_PER; ++j) {
      if (!((live >> j) & 1)) continue;
      const uint32_t idx = pos0 + j;
      if ((heavy >> j) & 1) {
        const uint32_t hr = carry_c + ex_c + (uint32_t)__popc(heavy & ((1u << j) - 1));
        if (hr + 1 >= nh) {
          table[r.base + idx] = AliasEntry{1.0f, idx - r.lead};
        } else {
          table[r.base + idx].alias = (uint32_t)s_slot[hr + 1] - r.lead;
        }
      } else {
        table[r.base + idx] = AliasEntry{op[j], (nh ? hslot : idx) - r.lead};
        // heavies whose surplus prefix lies in (sl, sl + D]: this light finishes them
        sl += dl[j];
        while (hv <= sl) {
          if (b + 1 < nh) table[r.base + hslot].prob = residual_prob(L.one + hv - sl, L);
          ++b;
          hv = s_sh[b];
          hslot = s_slot[b];
        }
      }
    }
    carry_d += tot_d;
    carry_c += tot_c;
  }
  // heavies no light has reached (surplus prefix beyond the row's total deficit) keep their bucket
  __syncthreads();
  for (uint32_t h = tid; h + 1 < nh; h += ST_T)
    if (s_sh[h] > carry_d) {
      const uint32_t slot = s_slot[h];
      table[r.base + slot] = AliasEntry{1.0f, slot - r.lead};
    }
}

namespace {
struct StreamScratch {
  RowRef* deferred = nullptr;
  uint32_t* n_deferred = nullptr;
  uint32_t cap = 0;
};
StreamScratch g_stream;
}  // namespace

// Builds the n rows of `rows_list` (8190..STREAM_MAX_DEG entries each).  Rows whose heavies do not fit the
// LDS list are returned in *deferred (device array owned by this file, valid until the next call).
int build_rows_stream(sky_graph* g, const RowRef* rows_list, uint32_t n, const RowRef** deferred,
                      uint32_t* n_deferred) {
  StreamScratch& sc = g_stream;
  *deferred = nullptr;
  *n_deferred = 0;
  if (n == 0) return SKY_OK;
  hipStream_t st = g->stream;
  if (sc.cap < n) {
    if (sc.deferred) SKY_HIP(hipFree(sc.deferred));
    sc.deferred = nullptr;
    sc.cap = 0;
    SKY_HIP(hipMalloc((void**)&sc.deferred, (size_t)n * sizeof(RowRef)));
    sc.cap = n;
  }
  if (!sc.n_deferred) SKY_HIP(hipMalloc((void**)&sc.n_deferred, 4));
  SKY_HIP(hipMemsetAsync(sc.n_deferred, 0, 4, st));
  hipLaunchKernelGGL(build_stream_kernel, dim3(n), dim3(ST_T), 0, st, rows_list, g->adjwgt, g->table, g->valid,
                     sc.deferred, sc.n_deferred);
  *deferred = sc.deferred;
  return SKY_OK;
}

// Number of rows the last build_rows_stream call deferred (synchronises the stream).
int stream_deferred_count(sky_graph* g, uint32_t* n_deferred) {
  *n_deferred = 0;
  if (!g_stream.n_deferred) return SKY_OK;
  SKY_HIP(hipMemcpyAsync(n_deferred, g_stream.n_deferred, 4, hipMemcpyDeviceToHost, g->stream));
  SKY_HIP(hipStreamSynchronize(g->stream));
  return SKY_OK;
}

}  // namespace sky
