// Alias tables of rows of 8190..524287 entries: one workgroup streams the row and keeps a window of
// the row's heavies in LDS.  (Rows of 5118..8189 entries: build_hold_kernel at the end of this file, which keeps
// the row itself in registers.)
//
// The table is the same pure function of the weights as everywhere else (see sky_build.hip).
// Only the heavies of a row need random access: a light's alias is the first heavy whose surplus
// prefix exceeds the light's exclusive deficit prefix, and a heavy's residual probability belongs
// to the one light whose deficit interval (SL - D, SL] contains the heavy's surplus prefix.  So
//   pass A   exact sum of the weights -> ledger
//   collect  the next ST_CAP heavies in slot order into LDS, {surplus prefix, slot, residual}, 16 bytes
//            each, and the slot of the heavy after them, if there is one
//   emit     classify every entry, running deficit prefix; a light whose alias lies in the window
//            gets its entry, and every light leaves the residual of the window's heavies that fall
//            into its deficit interval (usually none, sometimes one) in the window; entries go out
//            four at a time as two 16-byte stores, heavy slots among them carry a placeholder
//   sweep    every heavy of the window gets its final entry from the window: {residual, next heavy}
//            when a light reached it and it is not the row's last heavy, {1, itself} otherwise
// Rows with more heavies than one window holds repeat collect, emit and sweep: all move through
// the row in slot order and only come back to the chunk in which the previous window ended, because
// the alias ranks of the lights and the slots of the heavies both grow along the row.  An emit pass
// leaves alone what belongs to another window: lights whose alias lies outside this one, and heavies of
// earlier windows, whose final entries are already written.  After the first pass the weights come from L2.
#include <type_traits>

#include "sky_build_common.h"
#include "sky_graph.h"

namespace sky {

constexpr int ST_T = 512;                 // threads per row
constexpr int ST_PER = 8;                 // consecutive slots per thread and chunk
constexpr int ST_CH = ST_T * ST_PER;      // slots per chunk
constexpr int ST_NW = ST_T / 64;
constexpr uint32_t ST_CAP = 5080;         // heavies per row kept in LDS (and one sentinel): two workgroups share a CU's 160 KB
static_assert(STREAM_MAX_DEG + 3 < (1u << 20), "the three-limb sum is exact for rows of fewer than 2^20 entries");

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
// Makes the wavefront wait, here, until the chunk's loads have arrived.
__device__ __forceinline__ void wait_for_chunk(const RawChunk& x) {
#pragma unroll
  for (int q = 0; q < ST_PER / 4; ++q) asm volatile("" ::"v"(x.q[q].x), "v"(x.q[q].y), "v"(x.q[q].z), "v"(x.q[q].w));
}
// Whether every slot of wavefront `wave` in chunk c lies inside the row: true for all but the row's first wavefront
// (when the row starts after its 16-byte aligned base) and the one that holds its end.  Such a wavefront needs
// no per-slot masks.
__device__ __forceinline__ bool wave_inside_row(const StreamRow& r, uint32_t c, int wave) {
  const uint32_t w0 = c * ST_CH + (uint32_t)(ST_PER * 64) * (uint32_t)wave;
  return w0 >= r.lead && w0 + (uint32_t)(ST_PER * 64) <= r.span;
}
// Clamped weights (0 outside the row) and the mask of slots that belong to the row.  EDGE false: the caller
// knows that every slot does.
template <bool EDGE>
__device__ __forceinline__ uint32_t unpack_chunk(const RawChunk& x, const StreamRow& r, uint32_t c, int tid,
                                                 float (&cw)[ST_PER]) {
  uint32_t live = EDGE ? 0u : (1u << ST_PER) - 1u;
#pragma unroll
  for (int q = 0; q < ST_PER / 4; ++q) {
    const uint32_t pos = c * ST_CH + (uint32_t)ST_PER * tid + 4u * q;
    const float xs[4] = {x.q[q].x, x.q[q].y, x.q[q].z, x.q[q].w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if constexpr (EDGE) {
        const uint32_t idx = pos + k;
        const bool in = idx - r.lead < r.span - r.lead;
        if (in) live |= 1u << (q * 4 + k);
        cw[q * 4 + k] = masked_weight(xs[k], in);
      } else {
        cw[q * 4 + k] = clamp_weight(xs[k]);
      }
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

// The same for one u32 per thread alone.
__device__ __forceinline__ void stream_excl_c(uint32_t c, uint32_t* s_c, uint32_t& ex_c, uint32_t& tot_c) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint32_t ic = group_scan_u32<64>(c);
  if (lane == 63) s_c[wave] = ic;
  __syncthreads();
  uint32_t rc = 0;
  ex_c = ic - c;
#pragma unroll
  for (int w = 0; w < ST_NW; ++w) {
    if (w == wave) ex_c += rc;
    rc += s_c[w];
  }
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

// Values that every lane holds alike, moved to scalar registers (the compiler cannot see that sums read
// back from LDS are the same in every lane).
__device__ __forceinline__ uint32_t uniform_u32(uint32_t x) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); }
__device__ __forceinline__ uint64_t uniform_u64(uint64_t x) {
  return ((uint64_t)uniform_u32((uint32_t)(x >> 32)) << 32) | uniform_u32((uint32_t)x);
}

template <bool DEV>
__global__ __launch_bounds__(ST_T, 4) void build_stream_kernel(const RowRef* __restrict__ first_list, uint32_t n_first,
                                                            const RowRef* __restrict__ vlist, uint32_t n_rows,
                                                            const uint32_t* __restrict__ dev, int dev_ncls,
                                                            const float* __restrict__ wgt,
                                                            AliasEntry* __restrict__ table,
                                                            int8_t* __restrict__ valid) {
  __shared__ uint64_t s_sh[ST_CAP + 2];    // surplus prefix of the window's h-th heavy, then two sentinels
  __shared__ float s_prob[ST_CAP + 2];     // its residual probability, left by the light that reaches it
  __shared__ uint32_t s_slot[ST_CAP + 2];  // its span slot; after them the slot lights beyond the window take
  __shared__ WSum3 s_w[ST_NW];
  __shared__ double s_fsum[ST_NW];
  __shared__ uint32_t s_mn[ST_NW];
  __shared__ uint64_t s_a[2][ST_NW];  // two sets of wavefront sums, used alternately
  __shared__ uint32_t s_c[2][ST_NW];
  __shared__ uint32_t s_next;  // slot of the first heavy after the window
  // Class sizes known to the host (dev null): one workgroup per row, the first n_first take the rows of first_list
  // (the longest ones), the others those of vlist.  Sizes known to the device alone: the rows of the first dev_ncls
  // streaming classes lie back to back in vlist, after those of the classes before them, and the grid strides over them.
  uint32_t start = 0, count = n_first + n_rows;
  if (DEV) {
    for (int c = 0; c < CLS_STREAM; ++c) start += dev[c];
    count = 0;
    for (int c = CLS_STREAM; c < CLS_STREAM + dev_ncls; ++c) count += dev[c];
  }
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  // DEV false: one row per workgroup, and the loop is none
  for (uint32_t row = blockIdx.x; DEV ? row < count : row == blockIdx.x; row += DEV ? gridDim.x : 1u) {
  if (DEV && row != blockIdx.x) __syncthreads();  // the window and the sums in LDS are about to be rewritten
  const RowRef rr = DEV ? vlist[start + row] : (row < n_first ? first_list[row] : vlist[row - n_first]);
  StreamRow r;
  r.base = rr.off & ~3u;
  r.lead = rr.off - r.base;
  r.span = r.lead + rr.d;
  const uint32_t nch = (r.span + ST_CH - 1) / ST_CH;

  // ---- pass A: the sum of the row, as a plain fp64 sum when that is exact (see plain_sum_is_exact)
  double row_sum;
  RawChunk nx = fetch_chunk(wgt, r, 0, tid);  // every loop below requests chunk c + 1 before it works on chunk c
  {
    double fsum = 0.0;
    uint32_t mn = 0xFFFFFFFFu;
    for (uint32_t c = 0; c < nch; ++c) {
      const RawChunk cur = nx;
      if (c + 1 < nch) nx = fetch_chunk(wgt, r, c + 1, tid);
      if (!wave_in_row(r, c, wave)) continue;
      float cw[ST_PER];
      if (wave_inside_row(r, c, wave))
        unpack_chunk<false>(cur, r, c, tid, cw);
      else
        unpack_chunk<true>(cur, r, c, tid, cw);
#pragma unroll
      for (int j = 0; j < ST_PER; j += 2) {
        fsum += (double)cw[j];
        fsum += (double)cw[j + 1];
        mn = min(mn, min(__float_as_uint(cw[j]) - 1u, __float_as_uint(cw[j + 1]) - 1u));
      }
    }
    fsum = group_sum_f64<64>(fsum);
    mn = wave_min_u32(mn);
    if (lane == 0) {
      s_fsum[wave] = fsum;
      s_mn[wave] = mn;
    }
    __syncthreads();
    fsum = s_fsum[0];
    mn = s_mn[0];
#pragma unroll
    for (int i = 1; i < ST_NW; ++i) {
      fsum += s_fsum[i];
      mn = min(mn, s_mn[i]);
    }
    row_sum = fsum;
    if (!plain_sum_is_exact(fsum, uniform_u32(mn))) {  // uniform: the three-limb sum, from a second pass over the row
      WSum3 sum{0.0, 0.0, 0.0};
      nx = fetch_chunk(wgt, r, 0, tid);
      for (uint32_t c = 0; c < nch; ++c) {
        const RawChunk cur = nx;
        if (c + 1 < nch) nx = fetch_chunk(wgt, r, c + 1, tid);
        if (!wave_in_row(r, c, wave)) continue;
        float cw[ST_PER];
        unpack_chunk<true>(cur, r, c, tid, cw);
#pragma unroll
        for (int j = 0; j < ST_PER; ++j) wsum3_add(sum, (double)cw[j]);
      }
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
      row_sum = sum.top + sum.mid + sum.low == 0.0 ? 0.0 : wsum3_to_double(sum);
    }
  }
  if (row_sum == 0.0) {
    for (uint32_t c = 0; c < nch; ++c)
#pragma unroll
      for (int j = 0; j < ST_PER; ++j) {
        const uint32_t idx = c * ST_CH + (uint32_t)ST_PER * tid + j;
        if (idx >= r.lead && idx < r.span) table[r.base + idx] = AliasEntry{0.0f, SKY_INVALID};
      }
    if (tid == 0) valid[rr.v] = 0;
    continue;
  }
  const Ledger L = make_ledger_small(rr.d, row_sum);

  // Whether an entry is heavy is a monotone function of its clamped weight (p = fl(w * scale) and
  // t = fma(p, 2^F, -2^F) are monotone, heavy iff t >= 0.5), so one compare against the smallest heavy weight
  // of this row decides it; the surplus is then computed for the heavies alone, from the compacted list.
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
    while (bits > 0 && is_heavy(bits - 1) && guard < 8) {
      --bits;
      ++guard;
    }
    while (bits <= MAXW && !is_heavy(bits) && guard < 8) {
      ++bits;
      ++guard;
    }
    if (guard >= 8) {  // the estimate is normally within a step or two of the boundary; if not, bisect for it
      uint32_t lo = 0, hi = MAXW + 1;  // smallest pattern in [0, MAXW + 1) that is heavy, MAXW + 1 if none
      while (lo < hi) {
        const uint32_t mid = lo + (hi - lo) / 2;
        if (is_heavy(mid)) hi = mid; else lo = mid + 1;
      }
      bits = lo;
    }
    thr_bits = bits;
  }
  float* s_w32 = reinterpret_cast<float*>(s_sh);  // weight of heavy h in the low half of s_sh[h], until its prefix replaces it
  const double neg_fs = -L.fs;

  // window state: collecting resumes at chunk cb (cnt_cb heavies lie before it), emitting at chunk cc
  // (def_cc deficits and hc_cc heavies lie before it)
  uint32_t hb = 0;     // rank of the window's first heavy
  uint64_t sh_lo = 0;  // surplus prefix of the heavies before the window
  uint32_t cb = 0, cnt_cb = 0, cc = 0, hc_cc = 0;
  uint64_t def_cc = 0;
  for (;;) {
    // ---- collect: heavies of ranks [hb, hb + ST_CAP) and the slot of rank hb + ST_CAP
    bool more = false;
    uint32_t cnt = cnt_cb, next_cb = nch, next_cnt_cb = 0;
    nx = fetch_chunk(wgt, r, cb, tid);
    for (uint32_t c = cb; c < nch; ++c) {
      const RawChunk cur = nx;
      if (c + 1 < nch) nx = fetch_chunk(wgt, r, c + 1, tid);
      float cw[ST_PER];
      uint32_t heavy = 0;
      if (wave_in_row(r, c, wave)) {
        uint32_t live;
        if (wave_inside_row(r, c, wave))
          live = unpack_chunk<false>(cur, r, c, tid, cw);
        else
          live = unpack_chunk<true>(cur, r, c, tid, cw);
#pragma unroll
        for (int j = 0; j < ST_PER; ++j)
          if (__float_as_uint(cw[j]) >= thr_bits) heavy |= 1u << j;
        heavy &= live;
      }
      uint32_t ex_c, tot_c;
      stream_excl_c((uint32_t)__popc(heavy), s_c[c & 1], ex_c, tot_c);
      uint32_t rank = cnt + ex_c;
#pragma unroll
      for (int j = 0; j < ST_PER; ++j)
        if ((heavy >> j) & 1) {
          const uint32_t slot = c * ST_CH + (uint32_t)ST_PER * tid + j;
          if (rank >= hb && rank < hb + ST_CAP) {
            s_w32[2 * (rank - hb)] = cw[j];
            s_slot[rank - hb] = slot;
          } else if (rank == hb + ST_CAP) {
            s_next = slot;
          }
          ++rank;
        }
      tot_c = uniform_u32(tot_c);
      if (cnt + tot_c > hb + ST_CAP) {  // uniform: the window is full and another heavy follows in this chunk
        more = true;
        next_cb = c;
        next_cnt_cb = cnt;
        break;
      }
      cnt += tot_c;
    }
    const uint32_t nw = more ? ST_CAP : cnt - hb;
    __syncthreads();  // the window's weights and slots, and s_next, are complete
    const uint32_t next_slot = more ? uniform_u32(s_next) : NONE32;
    uint64_t sh_hi;  // surplus prefix of the window's last heavy
    {
      // surplus prefix of the window: HP consecutive heavies per thread; the surplus takes the weight's place
      // in s_sh first, the prefix takes the surplus's place after the scan
      constexpr int HP = 12;
      static_assert(ST_CAP < (uint32_t)ST_T * HP, "one round covers the window");
      uint64_t su = 0;
#pragma unroll
      for (int k = 0; k < HP; ++k) {
        const uint32_t h = (uint32_t)HP * tid + k;
        if (h < nw) {
          const uint64_t a = classify_fast((double)s_w32[2 * h], true, L).amount;
          s_sh[h] = a;
          su += a;
        }
      }
      uint64_t ex_u, tot_u;
      uint32_t ex_c, tot_c;
      stream_excl(su, 0u, s_a[0], s_c[0], ex_u, ex_c, tot_u, tot_c);
      uint64_t acc = sh_lo + ex_u;
#pragma unroll
      for (int k = 0; k < HP; ++k) {
        const uint32_t h = (uint32_t)HP * tid + k;
        if (h < nw) {
          acc += s_sh[h];
          s_sh[h] = acc;
        }
      }
      sh_hi = sh_lo + uniform_u64(tot_u);
    }
    const bool any_heavy = hb + nw != 0;
    const bool whole_row = hb == 0 && !more;  // the usual case: one window holds every heavy of the row
    if (tid == 0) {  // after the list: two sentinels, and the slot that lights beyond the window's last heavy take
      s_sh[nw] = ~0ull;
      s_sh[nw + 1] = ~0ull;
      s_slot[nw] = more ? next_slot : (nw ? s_slot[nw - 1] : 0u);
      s_slot[nw + 1] = 0u;
    }
    __syncthreads();

    // ---- emit: chunks from cc on, until the deficits before a chunk reach the window's last surplus prefix
    uint64_t carry_d = def_cc;
    uint32_t carry_c = hc_cc;    // heavies before the chunk
    uint32_t last_c = cc;        // the last chunk worked on, where the next window starts again
    uint64_t last_def = def_cc;  // deficits before it
    uint32_t last_hc = hc_cc;    // heavies before it
    nx = fetch_chunk(wgt, r, cc, tid);
    for (uint32_t c = cc; c < nch; ++c) {
      if (more && carry_d >= sh_hi) break;  // uniform: the lights from here on belong to later windows
      last_c = c;
      last_def = carry_d;
      last_hc = carry_c;
      const RawChunk cur = nx;
      if (c + 1 < nch) nx = fetch_chunk(wgt, r, c + 1, tid);
      const bool on = wave_in_row(r, c, wave);  // a wavefront past the row's end only takes part in the scan
      const bool inside = wave_inside_row(r, c, wave);
      uint32_t live = (1u << ST_PER) - 1u;
      // op[j]: float(p) of a light, -1 of a heavy (the sign carries "heavy" to the walk below); dl[j]: the
      // deficit of a light of the row, 0 for any other slot
      float op[ST_PER];
      uint64_t dl[ST_PER];
      uint32_t nheavy = 0;
      uint64_t run = 0;
      auto classify_chunk = [&](auto edge) {
        constexpr bool EDGE = decltype(edge)::value;
        float cw[ST_PER];
        live = unpack_chunk<EDGE>(cur, r, c, tid, cw);
#pragma unroll
        for (int j = 0; j < ST_PER; ++j) {
          // only the lights' amounts are used here: |t| <= 2^F, so the sum with 2^52 holds rint(|t|) in its low bits
          // (0 for a light with 0 < t < 0.5).  Heavy slots and slots outside the row come out as anything and are dropped.
          const double pj = (double)cw[j] * L.scale;
          const double t = fma(pj, L.fs, neg_fs);  // = (pj - 1) * 2^F rounded once: the product with 2^F is exact
          const uint64_t d = (uint64_t)__double_as_longlong(fabs(t) + 4503599627370496.0) & 0x000FFFFFFFFFFFFFull;
          const bool lv = !EDGE || ((live >> j) & 1);
          const bool hj = lv && __float_as_uint(cw[j]) >= thr_bits;
          op[j] = hj ? -1.0f : (float)pj;
          dl[j] = (lv && !hj) ? d : 0;
          nheavy += hj ? 1u : 0u;
          run += dl[j];
        }
      };
      if (on) {
        if (inside) classify_chunk(std::false_type{});
        else classify_chunk(std::true_type{});
      } else {
#pragma unroll
        for (int j = 0; j < ST_PER; ++j) {
          op[j] = 0.0f;
          dl[j] = 0;
        }
      }
      uint64_t ex_d, tot_d;
      uint32_t ex_c, tot_c;
      stream_excl(run, nheavy, s_a[c & 1], s_c[c & 1], ex_d, ex_c, tot_d, tot_c);
      const uint32_t pos0 = c * ST_CH + (uint32_t)ST_PER * tid;
      uint32_t oa[ST_PER];
      uint32_t wr = 0;  // entries this window writes: its lights, and heavies as placeholders unless an earlier window owns them
      if (on) {
        // b = window heavies whose surplus prefix is <= the deficits before this thread's slots: one search;
        // from there the thread's lights walk the list, each stopping at its own deficit prefix.  The list
        // entry after the current one is requested a hit ahead, so that a hit does not wait for local memory.
        uint64_t sl = carry_d + ex_d;
        uint32_t b = 0;
        if (nw) {
          const uint64_t k1[1] = {sl};
          uint32_t o1[1];
          count_le<1>(s_sh, nw, k1, o1);
          b = o1[0];
        }
        uint64_t hv = s_sh[b], hvn = s_sh[b + 1];  // ~0 once the window is exhausted
        // alias value of the current list entry (then: of the first heavy after the window, or the row's last heavy)
        uint32_t hal = s_slot[b] - r.lead, haln = s_slot[b + 1] - r.lead;
        const uint32_t self0 = pos0 - r.lead;
        uint32_t hrank = carry_c + ex_c;
        // One path for every slot: a heavy slot, or one outside the row, adds no deficit, so the list does not move.
#pragma unroll
        for (int j = 0; j < ST_PER; ++j) {
          const bool lv = (live >> j) & 1, hj = op[j] < 0.0f;
          if (!whole_row) {
            // a light's alias is the first heavy whose surplus prefix exceeds sl: in this window iff
            // sh_lo <= sl < sh_hi, or beyond every heavy of the row
            const bool w = hj ? hrank >= hb : lv && sl >= sh_lo && (sl < sh_hi || !more);
            if (w) wr |= 1u << j;
            hrank += hj ? 1u : 0u;
          }
          oa[j] = (lv && !hj && any_heavy) ? hal : self0 + (uint32_t)j;
          op[j] = fabsf(op[j]);
          // heavies of the window whose surplus prefix lies in (sl, sl + D]: this light finishes them
          sl += dl[j];
          if (hv <= sl) {
            do {
              s_prob[b] = residual_below(sl - hv);
              ++b;
              hv = hvn;
              hal = haln;
              hvn = s_sh[b + 1];
              haln = s_slot[b + 1] - r.lead;
            } while (hv <= sl);
          }
        }
        if (whole_row) wr = live;
      }
      // The weights of the next chunk, requested at the top of this iteration, are waited for here, before this
      // chunk's stores are issued: loads and stores complete in one in-order count, so a wait for the load placed
      // after the stores (at its first use in the next iteration) would wait for the stores as well.
      wait_for_chunk(nx);
      if (wr) {
        AliasEntry* const t0 = table + r.base + pos0;
#pragma unroll
        for (int q = 0; q < ST_PER / 4; ++q) {
          const uint32_t m = (wr >> (4 * q)) & 15u;
          AliasEntry* t = t0 + 4 * q;
          if (m == 15u) {
            const float p4[4] = {op[4 * q], op[4 * q + 1], op[4 * q + 2], op[4 * q + 3]};
            const uint32_t a4[4] = {oa[4 * q], oa[4 * q + 1], oa[4 * q + 2], oa[4 * q + 3]};
            store_entries4(t, p4, a4);
          } else if (m) {
#pragma unroll
            for (int k = 0; k < 4; ++k)
              if ((m >> k) & 1) t[k] = AliasEntry{op[4 * q + k], oa[4 * q + k]};
          }
        }
      }
      carry_d += uniform_u64(tot_d);
      carry_c += uniform_u32(tot_c);
    }
    // ---- sweep: the final entry of every heavy of the window.  A light reached it iff its surplus prefix is
    // within the deficits seen (all of them when the pass stopped early: it stops once they cover the window).
    __syncthreads();  // also orders the placeholders before the entries that replace them: the barrier's release waits for this wavefront's stores
    for (uint32_t h = tid; h < nw; h += ST_T) {
      const uint32_t slot = s_slot[h];
      const uint32_t nxt = h + 1 < nw ? (uint32_t)s_slot[h + 1] : next_slot;
      const bool fin = nxt != NONE32 && s_sh[h] <= carry_d;
      table[r.base + slot] = fin ? AliasEntry{s_prob[h], nxt - r.lead} : AliasEntry{1.0f, slot - r.lead};
    }
    if (!more) break;
    hb += nw;
    sh_lo = sh_hi;
    cb = next_cb;
    cnt_cb = next_cnt_cb;
    cc = last_c;
    def_cc = last_def;
    hc_cc = last_hc;
    __syncthreads();  // the lists are rewritten by the next window, whose stores must not overtake this sweep's
  }
  }  // rows of this workgroup
}

// ---------------------------------------------------------------- rows held in registers
// Rows of 5118..8189 entries: one workgroup of 512 threads holds the whole row, 16 consecutive slots per thread, so
// the weights are read once and every entry is classified once.  As in the streaming kernel only the heavies go to
// LDS, {surplus prefix, slot, residual} of each in slot order, 14 bytes; a thread knows the rank and the surplus
// prefix of its own heavies from one scan over the workgroup, so the list needs no second pass.  Then one list
// search per thread, its lights walk the list from there and leave the residual of every heavy they finish in the
// list; after a barrier every thread completes its own heavies from the list and writes its 16 entries as whole
// quads: each entry is written once.  A row with more heavies than the list holds repeats list, walk and completion
// for the next ranks; everything it needs is still in registers.  (2.1 TB/s on such rows against 1.9 for the
// streaming kernel.  The same with 1024 threads for rows of up to 16381 entries leaves one workgroup per CU, all
// of whose wavefronts wait at the same barriers: 1.7 TB/s.)
constexpr int HOLD_PER = 16;
constexpr int HOLD_T = 512;
constexpr uint32_t HOLD_CAP = 5632;  // heavies per list: two workgroups fill a CU's LDS
constexpr size_t HOLD_LDS_BYTES = (size_t)(HOLD_CAP + 2) * 14;
static_assert(HOLD_T * HOLD_PER >= HOLD_MAX_DEG + 3, "the row fits from any 16-byte phase");

template <bool DEV>
__global__ __launch_bounds__(HOLD_T, 4) void build_hold_kernel(const RowRef* __restrict__ vlist, uint32_t count,
                                                       const uint32_t* __restrict__ dev, int cls,
                                                       const float* __restrict__ wgt, AliasEntry* __restrict__ table,
                                                       int8_t* __restrict__ valid) {
  constexpr int PER = HOLD_PER, T = HOLD_T, NW = T / 64;
  constexpr uint32_t CAPH = HOLD_CAP;
  extern __shared__ uint64_t smem[];
  uint64_t* s_sh = smem;                                              // [CAPH + 2] surplus prefix of the list's h-th heavy, then two sentinels
  float* s_prob = reinterpret_cast<float*>(smem + CAPH + 2);          // [CAPH + 2] its residual probability
  uint16_t* s_slot = reinterpret_cast<uint16_t*>(s_prob + CAPH + 2);  // [CAPH + 2] its slot; after them the slot lights beyond the list take
  __shared__ WSum3 s_wsum[NW];
  __shared__ double s_fsum[NW];
  __shared__ uint32_t s_mn[NW];
  __shared__ uint64_t s_ex[3 * NW];

  uint32_t start = 0;
  if (DEV) {  // the class's rows start after those of the classes before it; the grid is an upper bound
    for (int c = 0; c < cls; ++c) start += dev[c];
    count = dev[cls];
  }
  if (blockIdx.x >= count) return;
  const RowRef rr = vlist[start + blockIdx.x];
  const uint32_t d = rr.d;
  const uint32_t base = rr.off & ~3u, lead = rr.off - base, span = lead + d;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const uint32_t pos0 = (uint32_t)PER * (uint32_t)tid;
  const bool wave_on = (uint32_t)(PER * 64 * wave) < span;

  float cw[PER];
  uint32_t live = 0;  // bit j: slot pos0 + j belongs to the row
  double rsum = 0.0;
  uint32_t mn = 0xFFFFFFFFu;
  if (wave_on) {
#pragma unroll
    for (int q = 0; q < PER / 4; ++q) {
      const uint32_t pos = pos0 + 4u * q;
      float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
      if (pos < span) x = *reinterpret_cast<const float4*>(wgt + base + pos);
      const float xs[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const bool in = pos + k - lead < d;  // one unsigned compare: slots before the row wrap around
        if (in) live |= 1u << (q * 4 + k);
        cw[q * 4 + k] = masked_weight(xs[k], in);
        rsum += (double)cw[q * 4 + k];
        mn = min(mn, __float_as_uint(cw[q * 4 + k]) - 1u);
      }
    }
    rsum = group_sum_f64<64>(rsum);
    mn = wave_min_u32(mn);
  } else {
#pragma unroll
    for (int j = 0; j < PER; ++j) cw[j] = 0.0f;
  }
  if (lane == 0) {
    s_fsum[wave] = rsum;
    s_mn[wave] = mn;
  }
  __syncthreads();
  rsum = s_fsum[0];
  mn = s_mn[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) {
    rsum += s_fsum[i];
    mn = min(mn, s_mn[i]);
  }
  if (!plain_sum_is_exact(rsum, uniform_u32(mn))) {  // uniform over the workgroup: the three-limb sum instead
    WSum3 sum{0.0, 0.0, 0.0};
    if (wave_on) {
#pragma unroll
      for (int j = 0; j < PER; ++j) wsum3_add(sum, (double)cw[j]);
      sum = group_sum_wsum3<64>(sum);
    }
    if (lane == 0) s_wsum[wave] = sum;
    __syncthreads();
    sum = s_wsum[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) {
      sum.top += s_wsum[i].top;
      sum.mid += s_wsum[i].mid;
      sum.low += s_wsum[i].low;
    }
    rsum = sum.top + sum.mid + sum.low != 0.0 ? wsum3_to_double(sum) : 0.0;
  }
  if (rsum == 0.0) {
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if ((live >> j) & 1) table[base + pos0 + j] = AliasEntry{0.0f, SKY_INVALID};
    if (tid == 0) valid[rr.v] = 0;
    return;
  }
  const Ledger L = make_ledger_small(d, rsum);
  const double neg_fs = -L.fs;

  // classify once: op = float(p); amt = deficit of a light, surplus of a heavy, 0 outside the row
  float op[PER];
  uint64_t amt[PER];
  uint32_t heavy = 0;
  uint64_t run_d = 0, run_u = 0;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const bool in = (live >> j) & 1;
    const double pj = (double)cw[j] * L.scale;
    const double t = fma(pj, L.fs, neg_fs);  // = (pj - 1) * 2^F rounded once: the product with 2^F is exact
    const bool hj = in && t >= 0.5;
    const double a = fmax(fabs(t), hj ? 1.0 : 0.0);  // |t| < 0.5 for a light with t > 0: rounds to the deficit 0
    uint64_t x;
    if (a < 4503599627370496.0)
      x = (uint64_t)__double_as_longlong(a + 4503599627370496.0) & 0x000FFFFFFFFFFFFFull;
    else
      x = (uint64_t)a;  // a surplus of 2^52 units and more is an integer already
    amt[j] = in ? x : 0;
    op[j] = (float)pj;
    if (hj) heavy |= 1u << j;
    run_d += hj ? 0 : amt[j];
    run_u += hj ? amt[j] : 0;
  }
  // exclusive prefixes over the workgroup of deficits, surpluses and heavy counts, and their totals
  uint64_t ex_d, ex_u, tot_d;
  uint32_t ex_c, nh;
  {
    const uint32_t c = (uint32_t)__popc(heavy);
    const uint64_t id = group_scan_u64<64>(run_d), iu = group_scan_u64<64>(run_u);
    const uint32_t ic = group_scan_u32<64>(c);
    if (lane == 63) {
      s_ex[3 * wave] = id;
      s_ex[3 * wave + 1] = iu;
      s_ex[3 * wave + 2] = ic;
    }
    __syncthreads();
    // the wavefronts' sums, one per lane of the first row of 16 lanes, scanned there
    uint64_t wd = 0, wu = 0;
    uint32_t wc = 0;
    if (lane < NW) {
      wd = s_ex[3 * lane];
      wu = s_ex[3 * lane + 1];
      wc = (uint32_t)s_ex[3 * lane + 2];
    }
    wd = group_scan_u64<16>(wd);
    wu = group_scan_u64<16>(wu);
    wc = group_scan_u32<16>(wc);
    const int prev = max(wave - 1, 0);
    uint64_t bd = shfl_u64(wd, prev), bu = shfl_u64(wu, prev);
    uint32_t bc = (uint32_t)__shfl((int)wc, prev, 64);
    if (wave == 0) {
      bd = bu = 0;
      bc = 0;
    }
    tot_d = shfl_u64(wd, NW - 1);
    nh = (uint32_t)__shfl((int)wc, NW - 1, 64);
    ex_d = bd + id - run_d;
    ex_u = bu + iu - run_u;
    ex_c = bc + ic - c;
  }
  nh = uniform_u32(nh);
  tot_d = uniform_u64(tot_d);

  uint32_t oa[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) oa[j] = pos0 + (uint32_t)j - lead;  // a light of a row without heavies, and a heavy nobody finishes, point at themselves
  uint64_t sh_lo = 0;  // surplus prefix of the heavies before the list
  for (uint32_t hb = 0; hb < nh; hb += CAPH) {
    const uint32_t nw = min(CAPH, nh - hb);
    const bool more = hb + nw < nh;
    const bool whole_row = hb == 0 && !more;  // the usual case: one list holds every heavy of the row
    if (hb) __syncthreads();                  // the previous list is read until its heavies are complete
    // ---- list: this thread's heavies of ranks [hb, hb + nw], the last one only when more follow (its slot is what
    // the list's last heavy points at); without more, the slot after the list repeats the last heavy's
    if (heavy) {
      uint32_t r = ex_c - hb;
      uint64_t su = ex_u;
#pragma unroll
      for (int j = 0; j < PER; ++j)
        if ((heavy >> j) & 1) {
          su += amt[j];
          if (r <= nw) {  // ranks before the list wrap around
            if (r < nw) s_sh[r] = su;
            s_slot[r] = (uint16_t)(pos0 + j);
            if (!more && r + 1 == nw) s_slot[nw] = (uint16_t)(pos0 + j);
          }
          ++r;
        }
    }
    if (tid == 0) {
      s_sh[nw] = ~0ull;
      s_sh[nw + 1] = ~0ull;
      s_slot[nw + 1] = 0;
    }
    __syncthreads();
    const uint64_t sh_hi = uniform_u64(s_sh[nw - 1]);  // surplus prefix of the list's last heavy
    // ---- walk: one search, then every light of this thread takes the list entry it stands at as its alias and
    // finishes the heavies whose surplus prefix its deficit reaches
    if (wave_on) {
      uint64_t sl = ex_d;
      const uint64_t k1[1] = {sl};
      uint32_t o1[1];
      count_le<1>(s_sh, nw, k1, o1);
      uint32_t b = o1[0];
      uint64_t hv = s_sh[b], hvn = s_sh[b + 1];  // ~0 once the list is exhausted
      uint32_t hal = (uint32_t)s_slot[b] - lead, haln = (uint32_t)s_slot[b + 1] - lead;
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        const bool lt = ((live & ~heavy) >> j) & 1;  // a light of the row
        // its alias is the first heavy whose surplus prefix exceeds sl: in this list iff sh_lo <= sl < sh_hi, or
        // beyond every heavy of the row
        if (lt && (whole_row || (sl >= sh_lo && (sl < sh_hi || !more)))) oa[j] = hal;
        sl += ((heavy >> j) & 1) ? 0 : amt[j];
        if (hv <= sl) {
          do {
            s_prob[b] = residual_below(sl - hv);
            ++b;
            hv = hvn;
            hal = haln;
            hvn = s_sh[b + 1];
            haln = (uint32_t)s_slot[b + 1] - lead;
          } while (hv <= sl);
        }
      }
    }
    __syncthreads();
    // ---- this thread's heavies of the list: {residual, next heavy} when a light reached it and it is not the row's
    // last heavy, {1, itself} otherwise
    if (heavy) {
      uint32_t r = ex_c - hb;
      uint64_t su = ex_u;
#pragma unroll
      for (int j = 0; j < PER; ++j)
        if ((heavy >> j) & 1) {
          su += amt[j];
          if (r < nw) {
            const bool fin = (r + 1 < nw || more) && su <= tot_d;
            op[j] = fin ? s_prob[r] : 1.0f;
            if (fin) oa[j] = (uint32_t)s_slot[r + 1] - lead;
          }
          ++r;
        }
    }
    sh_lo = sh_hi;
  }

  if (pos0 < span) {
#pragma unroll
    for (int q = 0; q < PER / 4; ++q) {
      const uint32_t pos = pos0 + 4u * q;
      if (pos >= lead && pos + 4 <= span) {
        const float p4[4] = {op[4 * q], op[4 * q + 1], op[4 * q + 2], op[4 * q + 3]};
        const uint32_t a4[4] = {oa[4 * q], oa[4 * q + 1], oa[4 * q + 2], oa[4 * q + 3]};
        store_entries4(table + base + pos, p4, a4);
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if ((live >> (4 * q + k)) & 1) table[base + pos + k] = AliasEntry{op[4 * q + k], oa[4 * q + k]};
      }
    }
  }
}

static bool g_hold_lds_enabled = false;
// The n rows of `rows` (5118..HOLD_MAX_DEG entries each), or with `dev` the rows of class `cls` of a list whose class
// sizes only the device knows (n is then an upper bound of their number).
int build_rows_hold(sky_graph* g, const RowRef* rows, uint32_t n, const uint32_t* dev, int cls) {
  if (n == 0) return SKY_OK;
  if (!g_hold_lds_enabled) {
    SKY_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(build_hold_kernel<false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)HOLD_LDS_BYTES));
    SKY_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(build_hold_kernel<true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)HOLD_LDS_BYTES));
    g_hold_lds_enabled = true;
  }
  if (dev)
    hipLaunchKernelGGL(build_hold_kernel<true>, dim3(n), dim3(HOLD_T), HOLD_LDS_BYTES, g->stream, rows, n, dev, cls,
                       g->adjwgt, g->table, g->valid);
  else
    hipLaunchKernelGGL(build_hold_kernel<false>, dim3(n), dim3(HOLD_T), HOLD_LDS_BYTES, g->stream, rows, n, dev, cls,
                       g->adjwgt, g->table, g->valid);
  return SKY_OK;
}

// Builds the n_first rows of `first_list` and the n rows of `rows_list` (8190..STREAM_MAX_DEG entries each) in one
// launch that starts with the former.
int build_rows_stream(sky_graph* g, const RowRef* first_list, uint32_t n_first, const RowRef* rows_list, uint32_t n) {
  if (n + n_first == 0) return SKY_OK;
  hipLaunchKernelGGL(build_stream_kernel<false>, dim3(n + n_first), dim3(ST_T), 0, g->stream, first_list, n_first, rows_list, n,
                     (const uint32_t*)nullptr, 0, g->adjwgt, g->table, g->valid);
  return SKY_OK;
}

// The rows of the first ncls streaming classes of a list whose class sizes only the device knows (`dev`: the counter
// block of the binning pass): `grid` workgroups stride over them.
int build_rows_stream_dev(sky_graph* g, const RowRef* vlist, const uint32_t* dev, int ncls, uint32_t grid) {
  if (grid == 0) return SKY_OK;
  hipLaunchKernelGGL(build_stream_kernel<true>, dim3(grid), dim3(ST_T), 0, g->stream, (const RowRef*)nullptr, 0u, vlist, 0u, dev,
                     ncls, g->adjwgt, g->table, g->valid);
  return SKY_OK;
}

}  // namespace sky
