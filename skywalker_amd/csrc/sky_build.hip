// Offline alias-table construction for every vertex (replaces ConstructAliasTableKernel /
// ConstructTable of the reference, src/createTable.cu:48-179, and the constructors of
// include/alias_table_new.cuh it calls).
//
// The table of a row is a pure function of its weights, defined with exact integer
// prefix sums so that no kernel below can change a bit of it by changing how it
// parallelises:
//   S     = sum floor(w_i 2^64)  (128 bit)        scale = deg / double(S)      p_i = w_i * scale
//   F     = 40 fraction bits (62 - floor(log2 deg) for rows of 2^22 entries and more)
//   t_i   = (p_i - 1) 2^F  ;  heavy iff t_i >= 0.5 : surplus U_i = max(rint(t_i), 1)
//                             light otherwise      : deficit D_i = rint(-t_i)      (ties to even)
//   SL(i) = inclusive prefix sum of deficits over slots <= i,  SH(i) likewise of surpluses
//   light i : prob = float(p_i), alias = first slot m with SH(m) > SL(i) - D_i
//             (the last heavy if there is none; itself if the row has no heavy)
//   heavy j : last heavy of the row -> prob 1, alias itself; otherwise with y = SH(j):
//             l = first slot with SL(l) >= y;  found -> prob = (2^F + y - SL(l)) 2^-F, alias = next heavy
//                                              none  -> prob 1, alias itself
// This is the pairing a sequential two-pointer Vose sweep over (lights in slot order,
// heavies in slot order) produces, written so that every entry is resolved by two
// prefix sums and a binary search: no queues, no float atomics, no rollback.
//
// Dispatch is by degree class (sky_graph.h): one lane per vertex while binning (deg <= 2),
// 4/8/16/32/64 lanes per vertex with the prefix arrays in a per-wave LDS strip,
// 64 to 512 threads per vertex with the row's prefix arrays in LDS (rows up to 4093 entries),
// and the tile-parallel path of sky_build_tiled.hip for longer rows.
#include <algorithm>
#include <functional>
#include <utility>
#include <vector>

#include "sky_build_common.h"
#include "sky_graph.h"

namespace sky {

__host__ __device__ __forceinline__ int degree_class(uint32_t d) {
  if (d == 0) return CLS_EMPTY;
  if (d <= 2) return CLS_TINY;
  // rows of the group kernels start at any slot (their vector loads and stores only need 4-byte alignment)
  if (d <= 8) return CLS_G2;
  if (d <= 16) return CLS_G4;
  if (d <= 32) return CLS_G8;
  if (d <= 64) return CLS_G16;
  if (d <= 128) return CLS_G32;
  if (d <= 160) return CLS_G32S;
  if (d <= 192) return CLS_G32X;
  if (d <= 253) return CLS_LDS_W1;
  // These kernels are bound by instruction issue: a row pays for the slots of its class, not for its entries.  The
  // two classes whose rows differ most in length (by a factor of two) are halved: 6 instead of 8 slots per thread
  // for their shorter rows.
  if (d <= 381) return CLS_LDS_W6;
  if (d <= 509) return CLS_LDS_W2;
  if (d <= 765) return CLS_MW2_6;
  const uint32_t nw = (d + 3 + 511) / 512;  // wavefronts of 512 slots that hold the row from any 16-byte phase
  // The arrays of a longer row (14 bytes of LDS per slot) would leave room for one workgroup per CU only: such a row
  // keeps its heavies alone in LDS, and its entries in registers as long as 512 threads can hold them (1024 threads
  // for rows of up to 16381 entries, one workgroup per CU, ran at 1.7 TB/s where the streaming kernel reaches 1.95).
  if (nw <= MERGE_MAX_NW) return CLS_MW2 + (int)nw - 2;
  if (d <= HOLD_MAX_DEG) return CLS_HOLD;
  if (d > STREAM_MAX_DEG) return CLS_HUGE;
  if (d > 65533u) return CLS_STREAM_WIDE;
  return d > 24576u ? CLS_STREAM : CLS_STREAM_LAST;
}

// Vectors that are only 4-byte aligned: global loads and stores of 8 and 16 bytes need no more on gfx950.
typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));
typedef float float2u __attribute__((ext_vector_type(2), aligned(4)));
typedef uint32_t uint4u __attribute__((ext_vector_type(4), aligned(4)));

// ---------------------------------------------------------------- 2..32 lanes per row
// G lanes share one row of at most PER * G slots; every lane holds PER consecutive weights, so a
// wavefront carries 64 / G rows and the per-row steps that do not depend on the row length (exact
// sum, ledger, scans) are paid once per 64 / G rows.  Prefix sums run over the group by DPP; SL and
// SH of every slot go to a per-group LDS strip padded to PER * G slots (slots outside the row add
// nothing), which each entry then searches once with a fixed number of probes; the heavies' slots,
// compacted by rank, give "next heavy" and "last heavy".  The rank rides in bits 52..63 of the SH scan.
// Every lane of the wavefront must call this together (DPP); a group without a row passes d = 0.
// s_pre: [2 * BLOCK * PER] u64 ([0, BLK): SL of every slot of the block; [BLK, 2 * BLK): SH), s_hs: [BLOCK * PER]
// (per group: row-local slot of its h-th heavy).  Returns false for a row whose weights sum to zero.
constexpr uint64_t GROUP_CNT = 1ull << 52;

template <int G, int PER, int BLOCK = 256>
__device__ __forceinline__ bool group_build_row(uint32_t off, uint32_t d, const float* __restrict__ wgt,
                                                AliasEntry* __restrict__ table, uint64_t* __restrict__ s_pre,
                                                uint8_t* __restrict__ s_hs, uint32_t tid = threadIdx.x) {
  static_assert(PER >= 4 && PER <= 6, "a lane loads one float4 (and one float), or three float2");
  constexpr uint32_t SLOTS = PER * G;
  constexpr uint32_t HB = PER == 4 ? SLOTS : PER == 5 ? SLOTS / 5 * 4 : SLOTS / 3 * 2;  // largest power of two <= SLOTS
  static_assert((HB & (HB - 1)) == 0 && HB <= SLOTS && 2 * HB > SLOTS && SLOTS <= 256, "G is a power of two");
  constexpr uint32_t BLK = BLOCK * PER;                      // slots of one block's strips (BLOCK threads)
  const int gl = tid & (G - 1);
  const int lane = tid & 63;
  const uint32_t gbase = (uint32_t)PER * (tid - gl);  // first LDS slot of the group
  const uint32_t pos = (uint32_t)PER * gl;

  float xs[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) xs[k] = 0.0f;
  if (PER == 4 || PER == 5) {
    if (pos < d) {
      const float4u x = *reinterpret_cast<const float4u*>(wgt + off + pos);
      xs[0] = x.x; xs[1] = x.y; xs[2] = x.z; xs[3] = x.w;
    }
  } else {
#pragma unroll
    for (int h = 0; h < PER / 2; ++h)
      if (pos + 2 * h < d) {
        const float2u x = *reinterpret_cast<const float2u*>(wgt + off + pos + 2 * h);
        xs[2 * h] = x.x;
        xs[2 * h + 1] = x.y;
      }
  }
  if (PER % 2 == 1 && pos + PER - 1 < d) xs[PER - 1] = wgt[off + pos + PER - 1];
  double wd[PER];
  uint32_t live = 0;
  // the sum of the row as a plain fp64 sum where that is exact (plain_sum_is_exact); a wavefront in which some
  // group's is not falls back to the three-limb sum for all of its groups
  double Sd = 0.0;
  uint32_t mn = 0xFFFFFFFFu;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const bool in = pos + k < d;
    if (in) live |= 1u << k;
    const float cw = masked_weight(xs[k], in);
    wd[k] = (double)cw;
    Sd += wd[k];
    mn = min(mn, __float_as_uint(cw) - 1u);
  }
  Sd = group_sum_f64<G>(Sd);
  mn = group_min_u32<G>(mn);
  const bool plain = plain_sum_is_exact(Sd, mn);
  if (__any(!plain)) {
    WSum3 S{0.0, 0.0, 0.0};
#pragma unroll
    for (int k = 0; k < PER; ++k) wsum3_add(S, wd[k]);
    S = group_sum_wsum3<G>(S);
    if (!plain) Sd = S.top + S.mid + S.low != 0.0 ? wsum3_to_double(S) : 0.0;
  }
  const bool row_ok = Sd != 0.0;
  Ledger L = make_ledger_small(d, Sd);
  if (!row_ok) L.scale = 0.0;
  const double neg_fs = -L.fs;

  uint64_t dl[PER], sl[PER], sh[PER];
  float op[PER];
  uint32_t heavy = 0;
  uint64_t ra = 0, rb = 0;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const Entry e = classify_small_fma(wd[k], L, neg_fs);
    dl[k] = (e.heavy || !((live >> k) & 1)) ? 0 : e.amount;
    ra += dl[k];
    rb += e.heavy ? (e.amount | GROUP_CNT) : 0;
    sl[k] = ra;
    sh[k] = rb;
    op[k] = (float)e.p;
    if (e.heavy) heavy |= 1u << k;
  }
  const uint64_t ia = group_scan_u64<G>(ra), ib = group_scan_u64<G>(rb);
  const uint32_t nh = (uint32_t)(shfl_u64(ib, (lane - gl) + G - 1) >> 52);
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    sl[k] += ia - ra;
    sh[k] += ib - rb;
    s_pre[gbase + pos + k] = sl[k];
    s_pre[BLK + gbase + pos + k] = sh[k] & (GROUP_CNT - 1);
    if ((heavy >> k) & 1) s_hs[gbase + (uint32_t)(sh[k] >> 52) - 1] = (uint8_t)(pos + k);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  // light: first slot with SH > SL - D.  heavy: first slot with SL >= SH, i.e. SL > SH - 1.
  // The first probe narrows the answer to a window of HB slots that ends inside the strip.
  uint32_t arr[PER], at[PER];
  uint64_t key[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const bool hv = (heavy >> k) & 1;
    arr[k] = gbase + (hv ? 0u : BLK);
    key[k] = hv ? (sh[k] & (GROUP_CNT - 1)) - 1 : sl[k] - dl[k];
    at[k] = HB == SLOTS ? 0u : (s_pre[arr[k] + HB - 1] <= key[k] ? SLOTS - HB : 0u);
  }
#pragma unroll
  for (uint32_t step = HB / 2; step >= 1; step >>= 1) {
    uint64_t v[PER];
#pragma unroll
    for (int k = 0; k < PER; ++k) v[k] = s_pre[arr[k] + at[k] + step - 1];
#pragma unroll
    for (int k = 0; k < PER; ++k) at[k] += v[k] <= key[k] ? step : 0u;
  }
  uint32_t oa[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const uint64_t v = s_pre[arr[k] + at[k]];
    const bool found = v > key[k];
    const uint32_t self = pos + k;
    if (!((heavy >> k) & 1)) {
      oa[k] = found ? at[k] : (nh ? (uint32_t)s_hs[gbase + nh - 1] : self);
    } else {
      const uint32_t hc = (uint32_t)(sh[k] >> 52);
      if (hc < nh && found) {
        op[k] = residual_prob(L.one + key[k] + 1 - v, L);
        oa[k] = s_hs[gbase + hc];
      } else {
        op[k] = 1.0f;
        oa[k] = self;
      }
    }
    if (!row_ok) {
      op[k] = 0.0f;
      oa[k] = SKY_INVALID;
    }
  }
  // the next row of this group reuses the strips: its writes must stay behind these reads
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int h = 0; h < PER / 2; ++h) {
    const uint32_t m = (live >> (2 * h)) & 3u;
    AliasEntry* t = table + off + pos + 2 * h;
    if (m == 3u) {
      uint4u o;
      o.x = __float_as_uint(op[2 * h]); o.y = oa[2 * h]; o.z = __float_as_uint(op[2 * h + 1]); o.w = oa[2 * h + 1];
      *reinterpret_cast<uint4u*>(t) = o;
    } else if (m == 1u) {
      t[0] = AliasEntry{op[2 * h], oa[2 * h]};
    }
  }
  if (PER % 2 == 1 && ((live >> (PER - 1)) & 1)) table[off + pos + PER - 1] = AliasEntry{op[PER - 1], oa[PER - 1]};
  return row_ok || d == 0;
}

// Where a class kernel finds its rows.  A build whose class sizes the host knows passes the class's segment of the
// row list and its length, and launches exactly the workgroups the rows need (dev null).  A build whose sizes only
// the device knows (the rows of a frontier that the host never waits for) passes the whole list and the counter
// block of the binning pass: the class's rows start after those of the classes before it, and a grid of fixed
// size strides over them.
__device__ __forceinline__ void class_segment(const uint32_t* __restrict__ dev, int cls, int ncls, uint32_t& start,
                                              uint32_t& count) {
  if (!dev) return;
  uint32_t st = 0;
  for (int c = 0; c < cls; ++c) st += dev[c];
  uint32_t n = 0;
  for (int c = cls; c < cls + ncls; ++c) n += dev[c];
  start = st;
  count = n;
}

template <int G, int PER, bool DEV = false>
__global__ __launch_bounds__(256) void build_group_kernel(const RowRef* __restrict__ vlist, uint32_t count,
                                                          const uint32_t* __restrict__ dev, int cls,
                                                          const float* __restrict__ wgt,
                                                          AliasEntry* __restrict__ table,
                                                          int8_t* __restrict__ valid) {
  __shared__ uint64_t s_pre[2 * 256 * PER];
  __shared__ uint8_t s_hs[256 * PER];
  uint32_t start = 0;
  if (DEV) class_segment(dev, cls, 1, start, count);
  constexpr uint32_t ROWS = 256 / G;  // rows per workgroup and round
  // DEV false: one round per workgroup, and the loop is none
  for (uint32_t b = blockIdx.x; DEV ? b * ROWS < count : b == blockIdx.x; b += DEV ? gridDim.x : 1u) {
    const uint32_t grp = b * ROWS + threadIdx.x / G;
    RowRef rr{0, 0, 0, 0};
    if (grp < count) rr = vlist[start + grp];
    const bool ok = group_build_row<G, PER>(rr.off, rr.d, wgt, table, s_pre, s_hs);
    if ((threadIdx.x & (G - 1)) == 0 && !ok) valid[rr.v] = 0;  // the binning pass has set it
  }
}

// ---------------------------------------------------------------- binning
// `src` lists the vertices to bin (n of them); a null src means vertices 0..n-1.  Block b of the
// count and scatter kernels owns the items [b * per_block, (b + 1) * per_block): the count kernel
// leaves one row of class counts per block, bin_offsets_kernel turns the rows into each block's
// first position inside every class segment, and the scatter kernel hands out positions from
// cursors it keeps in LDS, so no global atomic is involved and the lists come out grouped by block.
constexpr int BIN_BLOCKS = 4096;  // most blocks a binning pass uses
constexpr int BIN_ITEMS = 4;      // vertices per thread and step

__global__ __launch_bounds__(256) void bin_count_kernel(const uint32_t* __restrict__ xadj,
                                                        const uint32_t* __restrict__ src, uint32_t n,
                                                        const uint32_t* __restrict__ n_dev,
                                                        uint32_t per_block, int listed_from,
                                                        uint32_t* __restrict__ blk_cnt,
                                                        unsigned long long* __restrict__ class_edges) {
  __shared__ uint32_t s_cnt[CLS_COUNT];
  __shared__ unsigned long long s_edges[CLS_COUNT];
  if (threadIdx.x < CLS_COUNT) {
    s_cnt[threadIdx.x] = 0;
    s_edges[threadIdx.x] = 0;
  }
  __syncthreads();
  if (n_dev) n = min(n, *n_dev);  // the host passed an upper bound
  const uint32_t lo = blockIdx.x * per_block, hi = min(n, lo + per_block);
  uint32_t tiny_edges = 0;  // rows of 1..2 entries, the commonest kind of a power-law graph, stay out of the LDS atomics
  // four vertices per thread and step: their loads are in flight together (one at a time, the loop waits a
  // memory round trip per vertex)
  for (uint32_t chunk = lo; chunk < hi; chunk += 256u * BIN_ITEMS) {
    uint32_t d[BIN_ITEMS];
#pragma unroll
    for (int k = 0; k < BIN_ITEMS; ++k) {
      const uint32_t i = chunk + k * 256u + threadIdx.x;
      d[k] = 0;
      if (i < hi) {
        const uint32_t v = src ? src[i] : i;
        d[k] = xadj[v + 1] - xadj[v];
      }
    }
#pragma unroll
    for (int k = 0; k < BIN_ITEMS; ++k) {
      const int c = degree_class(d[k]);
      if (c >= CLS_G2) {
        if (c >= listed_from) atomicAdd(&s_cnt[c], 1u);  // classes below get no list: small_rows_kernel builds them
        atomicAdd(&s_edges[c], (unsigned long long)d[k]);
      } else {
        tiny_edges += d[k];  // 0 for an empty row
      }
    }
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) tiny_edges += (uint32_t)__shfl_xor((int)tiny_edges, m, 64);
  if ((threadIdx.x & 63) == 0 && tiny_edges) atomicAdd(&s_edges[CLS_TINY], (unsigned long long)tiny_edges);
  __syncthreads();
  if (threadIdx.x < CLS_COUNT) {
    blk_cnt[blockIdx.x * CLS_COUNT + threadIdx.x] = s_cnt[threadIdx.x];
    if (s_edges[threadIdx.x]) atomicAdd(&class_edges[threadIdx.x], s_edges[threadIdx.x]);
  }
}

// One workgroup per class: exclusive prefix of the class's per-block counts (in place), total to counts[c].
// Thread t owns a run of consecutive blocks: its loads do not wait for one another.
__global__ __launch_bounds__(256) void bin_offsets_kernel(uint32_t* __restrict__ blk_cnt, uint32_t blocks,
                                                          uint32_t* __restrict__ counts) {
  __shared__ uint32_t s_w[4];
  const uint32_t c = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr uint32_t RUN = (BIN_BLOCKS + 255) / 256;
  const uint32_t b0 = tid * RUN;
  uint32_t x[RUN], sum = 0;
#pragma unroll
  for (uint32_t k = 0; k < RUN; ++k) {
    x[k] = b0 + k < blocks ? blk_cnt[(b0 + k) * CLS_COUNT + c] : 0u;
    sum += x[k];
  }
  const uint32_t inc = group_scan_u32<64>(sum);
  if (lane == 63) s_w[wave] = inc;
  __syncthreads();
  uint32_t run = inc - sum;
  for (uint32_t w = 0; w < wave; ++w) run += s_w[w];
#pragma unroll
  for (uint32_t k = 0; k < RUN; ++k) {
    if (b0 + k < blocks) blk_cnt[(b0 + k) * CLS_COUNT + c] = run;
    run += x[k];
  }
  if (tid == 0) counts[c] = s_w[0] + s_w[1] + s_w[2] + s_w[3];
}

// A row of one or two entries in closed form.
__device__ __forceinline__ bool tiny_row(uint32_t off, uint32_t d, const float* __restrict__ wgt,
                                         AliasEntry* __restrict__ table) {
  // a weight adds to the exact sum iff it is at least 2^-64
  constexpr float UNIT = 5.421010862427522170037e-20f;  // 2^-64
  const float w0 = clamp_weight(wgt[off]);
  if (d == 1) {
    const bool ok = w0 >= UNIT;
    table[off] = AliasEntry{ok ? 1.0f : 0.0f, ok ? 0u : SKY_INVALID};
    return ok;
  }
  const float w1 = clamp_weight(wgt[off + 1]);
  const bool ok = w0 >= UNIT || w1 >= UNIT;
  AliasEntry a{0.0f, SKY_INVALID}, b{0.0f, SKY_INVALID};
  if (ok) {
    WSum3 S{0.0, 0.0, 0.0};
    wsum3_add(S, (double)w0);
    wsum3_add(S, (double)w1);
    const Ledger L = make_ledger_small(2, wsum3_to_double(S));
    const Entry e0 = classify_small((double)w0, true, L), e1 = classify_small((double)w1, true, L);
    // a lone heavy is the last heavy: it keeps its bucket and tops up the light
    a = AliasEntry{e0.heavy ? 1.0f : (float)e0.p, (!e0.heavy && e1.heavy) ? 1u : 0u};
    b = AliasEntry{e1.heavy ? 1.0f : (float)e1.p, (!e1.heavy && e0.heavy) ? 0u : 1u};
  }
  uint4u o;
  o.x = __float_as_uint(a.prob); o.y = a.alias; o.z = __float_as_uint(b.prob); o.w = b.alias;
  *reinterpret_cast<uint4u*>(table + off) = o;
  return ok;
}

// Writes each row of class >= CLS_G2 into its class segment of vlist, and finishes
// the classes that need no cooperation: deg 0 (valid = 0) and deg 1..2 (closed form).  The rows of one
// or two entries that a wavefront meets in a step go to a list of its own in LDS first and are then
// built with its lanes side by side (they are a fifth of the vertices of a power-law graph: built where
// they are met, every step would pay for them with most lanes idle).
__global__ __launch_bounds__(256) void bin_scatter_kernel(const uint32_t* __restrict__ xadj,
                                                          const float* __restrict__ wgt,
                                                          const uint32_t* __restrict__ src, uint32_t n,
                                                          const uint32_t* __restrict__ n_dev,
                                                          uint32_t per_block, int listed_from,
                                                          const uint32_t* __restrict__ counts,
                                                          const uint32_t* __restrict__ blk_off,
                                                          RowRef* __restrict__ vlist,
                                                          AliasEntry* __restrict__ table,
                                                          int8_t* __restrict__ valid) {
  __shared__ uint32_t s_cur[CLS_COUNT];
  __shared__ uint2 s_tiny[4][64 * BIN_ITEMS];  // per wavefront: {offset, vertex} of its rows of 1..2 entries
  __shared__ uint8_t s_tiny_d[4][64 * BIN_ITEMS];
  if (threadIdx.x < CLS_COUNT) {  // the class lists lie back to back in class order
    uint32_t start = 0;
    for (uint32_t c = 0; c < threadIdx.x; ++c) start += counts[c];
    s_cur[threadIdx.x] = start + blk_off[blockIdx.x * CLS_COUNT + threadIdx.x];
  }
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (n_dev) n = min(n, *n_dev);
  const uint32_t lo = blockIdx.x * per_block, hi = min(n, lo + per_block);
  for (uint32_t chunk = lo; chunk < hi; chunk += 256u * BIN_ITEMS) {
    uint32_t nt = 0;  // wave-uniform: rows in this wavefront's list
#pragma unroll
    for (int i = 0; i < BIN_ITEMS; ++i) {
      const uint32_t item = chunk + i * 256u + threadIdx.x;
      int c = -1;
      uint32_t v = 0, off = 0, d = 0;
      if (item < hi) {
        v = src ? src[item] : item;
        off = xadj[v];
        d = xadj[v + 1] - off;
        c = degree_class(d);
      }
      // listed_from > CLS_G2: the rows of the classes below it, empty rows included, belong to small_rows_kernel
      const bool tiny_here = c == CLS_TINY && listed_from == CLS_G2;
      const unsigned long long m = __ballot(tiny_here);
      if (tiny_here) {
        const uint32_t p = nt + (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
        s_tiny[wave][p] = make_uint2(off, v);
        s_tiny_d[wave][p] = (uint8_t)d;
      } else if (c >= listed_from) {
        vlist[atomicAdd(&s_cur[c], 1u)] = RowRef{v, off, d, 0};
      }
      nt += (uint32_t)__popcll(m);
      // written here, next to its neighbours' flags; a row without weight clears it later
      if (c >= listed_from || (c >= 0 && listed_from == CLS_G2)) valid[v] = c != CLS_EMPTY;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (uint32_t t = lane; t < nt; t += 64u) {
      const uint2 rec = s_tiny[wave][t];
      if (!tiny_row(rec.x, s_tiny_d[wave][t], wgt, table)) valid[rec.y] = 0;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // the next step's list entries stay behind these reads
    __builtin_amdgcn_wave_barrier();
  }
}

// ---------------------------------------------------------------- rows of at most 32 entries, where they lie
// One wavefront walks a contiguous range of vertices, 64 at a time, and builds every row of 1..32 entries it
// meets: the rows of a class queue up in LDS until they fill the wavefront (64 rows of 1..2 entries, 32 of 3..8 with
// 2 lanes each, 16 of 9..16 with 4, 8 of 17..32 with 8) and are then built by the same code as in the class kernels.
// Neighbouring rows of different classes share their cache lines, and here the same wavefront touches them within a
// few steps; no row list is written or read for these classes.  Also sets valid[] of the vertices it owns (rows of
// 0..32 entries).  Workgroups are single wavefronts: nothing in here waits for another wavefront.
// Queue capacities (128, 96, 80, 72): less than one batch left over plus the 64 vertices of a step
// (64 + 63, 64 + 31, 64 + 15, 64 + 7), rounded up.  A queue entry is the row's offset and, in 16 bits, its degree (6 bits) above the vertex's position in
// the wavefront's range (10 bits): the vertex id itself is only needed for a row without weight, whose flag is
// cleared.  6.5 KB of LDS per wavefront, so that six of them fit every SIMD (the kernel's registers allow six).
constexpr uint32_t SMALL_RANGE = 1024;  // most vertices per wavefront
constexpr uint32_t SMALL_QBASE[4] = {0, 128, 224, 304};
constexpr uint32_t SMALL_QTOTAL = 376;
__global__ __launch_bounds__(64) void small_rows_kernel(const uint32_t* __restrict__ xadj,
                                                        const float* __restrict__ wgt,
                                                        const uint32_t* __restrict__ src, uint32_t n,
                                                        uint32_t per_wave, AliasEntry* __restrict__ table,
                                                        int8_t* __restrict__ valid) {
  __shared__ uint64_t s_pre[2 * 64 * 4];
  __shared__ uint8_t s_hs[64 * 4];
  __shared__ uint32_t q_off[SMALL_QTOTAL];
  __shared__ uint16_t q_it[SMALL_QTOTAL];
  const uint32_t lane = threadIdx.x;
  const uint32_t lo = blockIdx.x * per_wave, hi = min(n, lo + per_wave);
  uint32_t cnt[4] = {0, 0, 0, 0};  // wave-uniform queue lengths: rows of 1..2, 3..8, 9..16, 17..32 entries

  // the last `rows` entries of queue q, one per group of G lanes; d = 0 for a group without a row.  `t` is the lane
  // number behind an empty asm statement: it keeps what depends on the lane number inside one batch (hoisted
  // out of the loop for all four row sizes at once, those values double the registers of the kernel).
  auto take = [&](int q, uint32_t rows, uint32_t G, uint32_t& t, uint32_t& off, uint32_t& it, uint32_t& d) {
    t = lane;
    asm volatile("" : "+v"(t));
    const uint32_t r = t / G;
    off = it = d = 0;
    if (r < rows) {
      const uint32_t k = SMALL_QBASE[q] + cnt[q] - rows + r;
      off = q_off[k];
      const uint32_t x = q_it[k];
      it = x & (SMALL_RANGE - 1);
      d = x >> 10;
    }
  };
  auto clear_valid = [&](uint32_t it) {  // a row whose weights sum to zero (rare)
    const uint32_t item = lo + it;
    valid[src ? src[item] : item] = 0;
  };
  auto build_tiny = [&](uint32_t rows) {
    uint32_t t, off, it, d;
    take(0, rows, 1, t, off, it, d);
    if (d && !tiny_row(off, d, wgt, table)) clear_valid(it);
    cnt[0] -= rows;
  };
  auto build_g2 = [&](uint32_t rows) {
    uint32_t t, off, it, d;
    take(1, rows, 2, t, off, it, d);
    const bool ok = group_build_row<2, 4, 64>(off, d, wgt, table, s_pre, s_hs, t);
    if ((t & 1) == 0 && !ok) clear_valid(it);
    cnt[1] -= rows;
  };
  auto build_g4 = [&](uint32_t rows) {
    uint32_t t, off, it, d;
    take(2, rows, 4, t, off, it, d);
    const bool ok = group_build_row<4, 4, 64>(off, d, wgt, table, s_pre, s_hs, t);
    if ((t & 3) == 0 && !ok) clear_valid(it);
    cnt[2] -= rows;
  };
  auto build_g8 = [&](uint32_t rows) {
    uint32_t t, off, it, d;
    take(3, rows, 8, t, off, it, d);
    const bool ok = group_build_row<8, 4, 64>(off, d, wgt, table, s_pre, s_hs, t);
    if ((t & 7) == 0 && !ok) clear_valid(it);
    cnt[3] -= rows;
  };

  // the row offsets of step i + 1 are requested before the batches of step i are built
  auto fetch = [&](uint32_t base, uint32_t& v, uint32_t& off, uint32_t& end) {
    const uint32_t item = base + lane;
    v = 0xFFFFFFFFu;
    off = end = 0;
    if (item < hi) {
      v = src ? src[item] : item;
      off = xadj[v];
      end = xadj[v + 1];
    }
  };
  uint32_t nv, noff, nend;
  fetch(lo, nv, noff, nend);
  for (uint32_t base = lo; base < hi; base += 64u) {
    const uint32_t v = nv, off = noff, d = nend - noff;
    if (base + 64u < hi) fetch(base + 64u, nv, noff, nend);
    int q = -1;
    if (v != 0xFFFFFFFFu && d <= 32u) {
      valid[v] = d != 0;  // a row without weight clears it when it is built
      q = d == 0 ? -1 : d <= 2 ? 0 : d <= 8 ? 1 : d <= 16 ? 2 : 3;
    }
    const uint32_t packed = (d << 10) | (base - lo + lane);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const unsigned long long m = __ballot(q == c);
      if (q == c) {
        const uint32_t p = SMALL_QBASE[c] + cnt[c] + (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
        q_off[p] = off;
        q_it[p] = (uint16_t)packed;
      }
      cnt[c] += (uint32_t)__popcll(m);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    while (cnt[0] >= 64u) build_tiny(64);
    while (cnt[1] >= 32u) build_g2(32);
    while (cnt[2] >= 16u) build_g4(16);
    while (cnt[3] >= 8u) build_g8(8);
    // the next step's queue entries stay behind this step's reads of the queues
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  if (cnt[0]) build_tiny(cnt[0]);
  if (cnt[1]) build_g2(cnt[1]);
  if (cnt[2]) build_g4(cnt[2]);
  if (cnt[3]) build_g8(cnt[3]);
}

// ---------------------------------------------------------------- one row per workgroup, prefix arrays in LDS
// ROWT threads cooperate on one row of at most ROWT*4*T slots (counted from the row's 16-byte
// aligned start).  Weights are read once as aligned float4 quads; every entry is classified once
// and keeps its search key in registers; SL and SH of every slot live in LDS.  Each entry then
// does exactly one binary search, lights in SH and heavies in SL, four searches interleaved; the
// next heavy after each heavy and the last heavy of the row come from a suffix scan, not a search.
template <int ROWT, int T>
__global__ __launch_bounds__(ROWT) void build_lds_kernel(const RowRef* __restrict__ vlist,
                                                         const uint32_t* __restrict__ xadj,
                                                         const float* __restrict__ wgt,
                                                         AliasEntry* __restrict__ table, int8_t* __restrict__ valid) {
  constexpr int CAP = ROWT * 4 * T;
  constexpr int NW = ROWT / 64;
  extern __shared__ uint64_t smem[];
  uint64_t* s_sl = smem;
  uint64_t* s_sh = smem + CAP;
  __shared__ u128 s_wsum[NW];
  __shared__ uint64_t s_ex[2 * T * NW];
  __shared__ uint32_t s_fh[T][NW], s_lh[T][NW];

  const RowRef rr = vlist[blockIdx.x];
  const uint32_t v = rr.v, off = rr.off, d = rr.d;
  const uint32_t base = off & ~3u, lead = off - base, span = lead + d;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;

  float w[T][4];
  u128 sum{0, 0};
  uint32_t live = 0;       // bit q*4+k: slot belongs to the row
  uint32_t wave_live = 0;  // bit t: some slot of this wave's strip of sub-tile t belongs to the row
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const uint32_t pos = 4u * (t * ROWT + tid);
    if (4u * (t * ROWT + wave * 64) >= span) {  // wave-uniform: nothing of the row here
#pragma unroll
      for (int k = 0; k < 4; ++k) w[t][k] = 0.0f;
      continue;
    }
    wave_live |= 1u << t;
    float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
    if (pos < span) x = *reinterpret_cast<const float4*>(wgt + base + pos);
    const float xs[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t idx = pos + k;
      const bool in = idx - lead < d;  // one unsigned compare: slots before the row wrap around
      if (in) live |= 1u << (t * 4 + k);
      w[t][k] = in ? clamp_weight(xs[k]) : 0.0f;
      sum = add128(sum, weight_fixed(w[t][k]));
    }
  }
  sum = group_sum_u128<64>(sum);
  if (NW > 1) {
    if (lane == 0) s_wsum[wave] = sum;
    __syncthreads();
    sum = s_wsum[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) sum = add128(sum, s_wsum[i]);
  }
  if ((sum.lo | sum.hi) == 0) {
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if ((live >> (t * 4 + k)) & 1) {
          const uint32_t idx = 4u * (t * ROWT + tid) + k;
          table[base + idx] = AliasEntry{0.0f, SKY_INVALID};
        }
    if (tid == 0) valid[v] = 0;
    return;
  }
  const Ledger L = make_ledger(d, sum);

  // classify once; amounts -> prefix sums; first / last heavy of every (sub-tile, wave)
  uint64_t dl[T][4], dh[T][4], sl[T][4], sh[T][4];
  float op[T][4];
  uint32_t heavy = 0;
  uint64_t hb_mask[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    if (!((wave_live >> t) & 1)) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        dl[t][k] = dh[t][k] = 0;
        op[t][k] = 0.0f;
      }
      hb_mask[t] = 0;
      if (lane == 0) {
        s_fh[t][wave] = NONE32;
        s_lh[t][wave] = 0;
      }
      continue;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int b = t * 4 + k;
      const Entry e = classify(w[t][k], L);
      const bool in = (live >> b) & 1;
      dl[t][k] = (in && !e.heavy) ? e.amount : 0;
      dh[t][k] = (in && e.heavy) ? e.amount : 0;
      op[t][k] = e.heavy ? 1.0f : (float)e.p;
      if (in && e.heavy) heavy |= 1u << b;
    }
    // first and last heavy slot of this (sub-tile, wave), from a ballot over the quads that hold a heavy
    const uint32_t m = (heavy >> (t * 4)) & 15u;
    const uint64_t bal = __ballot(m != 0);
    hb_mask[t] = bal;
    // readlane must see every lane's m: keep it out of divergent code
    uint32_t fh = NONE32, lh = 0;  // lh holds index + 1, 0 = none
    if (bal) {
      const int l0 = __ffsll((unsigned long long)bal) - 1, l1 = 63 - __clzll((long long)bal);
      const uint32_t m0 = (uint32_t)__builtin_amdgcn_readlane((int)m, l0);
      const uint32_t m1 = (uint32_t)__builtin_amdgcn_readlane((int)m, l1);
      fh = 4u * (t * ROWT + wave * 64 + l0) + (uint32_t)(__ffs((int)m0) - 1);
      lh = 4u * (t * ROWT + wave * 64 + l1) + (uint32_t)(31 - __clz((int)m1)) + 1;
    }
    if (lane == 0) {
      s_fh[t][wave] = fh;
      s_lh[t][wave] = lh;
    }
  }
  uint64_t total_l, total_h;
  block_scan2<ROWT, T>(dl, dh, s_ex, sl, sh, total_l, total_h, wave_live);  // its barrier also publishes s_fh / s_lh
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const uint32_t pos = 4u * (t * ROWT + tid);
    if (!((wave_live >> t) & 1)) continue;  // slots beyond the row are never searched
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      s_sl[pos + k] = sl[t][k];
      s_sh[pos + k] = sh[t][k];
    }
  }
  // next heavy after each quad: later lanes of the wave, later waves of the sub-tile, later sub-tiles
  uint32_t last_heavy = 0;
  uint32_t nh_after[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    // next quad of this wave that holds a heavy: first ballot bit above this lane
    const uint32_t m = (heavy >> (t * 4)) & 15u;
    const uint64_t above = hb_mask[t] & ~((2ull << lane) - 1);
    const int ln = above ? __ffsll((unsigned long long)above) - 1 : lane;
    const uint32_t mn = (uint32_t)__shfl((int)m, ln, 64);
    uint32_t nx = above ? 4u * (t * ROWT + wave * 64 + ln) + (uint32_t)(__ffs((int)mn) - 1) : NONE32;
#pragma unroll
    for (int wv = 0; wv < NW; ++wv) {
      if (wv > wave) nx = min(nx, s_fh[t][wv]);
#pragma unroll
      for (int t2 = t + 1; t2 < T; ++t2) nx = min(nx, s_fh[t2][wv]);
      last_heavy = max(last_heavy, s_lh[t][wv]);
    }
    nh_after[t] = nx;
  }
  __syncthreads();  // s_sl / s_sh are complete

  const uint64_t* a_l = s_sl + lead;
  const uint32_t off_l = lead * 8u, off_h = (CAP + lead) * 8u;  // byte offsets of the row inside smem
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const uint32_t pos = 4u * (t * ROWT + tid);
    if (pos >= span) continue;
    uint32_t arr[4];
    uint64_t key[4];
    uint32_t nh[4], oa[4], at[4];
    uint32_t nxt = nh_after[t];
#pragma unroll
    for (int k = 3; k >= 0; --k) {
      nh[k] = nxt;
      if ((heavy >> (t * 4 + k)) & 1) nxt = pos + k;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bool hv = (heavy >> (t * 4 + k)) & 1;
      arr[k] = hv ? off_l : off_h;                          // a heavy looks for its retiring light in SL
      key[k] = hv ? sh[t][k] - 1 : sl[t][k] - dl[t][k];      // first SL >= y  <=>  first SL > y - 1
    }
    search4(smem, arr, key, d, at);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bool hv = (heavy >> (t * 4 + k)) & 1;
      const uint32_t self = pos + k - lead;
      if (!hv) {
        oa[k] = at[k] < d ? at[k] : (last_heavy ? last_heavy - 1 - lead : self);
      } else if (nh[k] != NONE32 && at[k] < d) {
        op[t][k] = residual_prob(L.one + sh[t][k] - a_l[at[k]], L);
        oa[k] = nh[k] - lead;
      } else {
        oa[k] = self;  // op is already 1
      }
    }
    if (pos >= lead && pos + 4 <= span) {
      store_entries4(table + base + pos, op[t], oa);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if ((live >> (t * 4 + k)) & 1) {
          table[base + pos + k] = AliasEntry{op[t][k], oa[k]};
        }
    }
  }
}

// ---------------------------------------------------------------- one row per workgroup, pairing by merge
// Same table as build_lds_kernel, reached without a binary search per entry.  Lights and heavies
// are compacted by rank into one LDS array (inclusive SL of the lights from the front, inclusive
// SH of the heavies from the back, a sentinel after each).  In the order of the merged sequence,
// ties heavy first,
//   the alias of light r is the heavy rank reached when light r - 1 is taken (rank 0 for r = 0),
//   the light that finishes heavy h is the light rank reached when heavy h is taken,
// so each thread finds where its share of PER merged elements starts (one diagonal search) and
// walks it.  The heavy count rides in bits 52..63 of the SH scan: a row of at most 4093 entries
// keeps its sums below 2^52.
constexpr uint64_t MERGE_CNT = 1ull << 52;
constexpr uint32_t MERGE_SELF = 0x80000000u;  // "prob 1, alias self" in the per-heavy result word

template <int ROWT, int PER, int MINW = 4, int DEV = 0>  // DEV 1: segment from the device, one row per workgroup; 2: striding grid
__global__ __launch_bounds__(ROWT, MINW) void build_merge_kernel(const RowRef* __restrict__ vlist, uint32_t count,
                                                           const uint32_t* __restrict__ dev, int cls,
                                                           const float* __restrict__ wgt,
                                                           AliasEntry* __restrict__ table, int8_t* __restrict__ valid) {
  // PER consecutive slots per thread, counted from the row's 16-byte aligned start; a thread moves them as
  // quads when PER is a multiple of 4, as pairs otherwise (its first slot is then only 8-byte aligned)
  constexpr int VEC = PER % 4 == 0 ? 4 : 2;
  static_assert(PER % VEC == 0 && PER <= 16, "whole vectors, and `live` has one bit per slot");
  constexpr int CAP = ROWT * PER;
  constexpr int NW = ROWT / 64;
  constexpr uint32_t TOP = CAP + 1;  // heavy h lives at index TOP - h of the value array and of the result array
  constexpr bool PACKED = CAP <= 4096;  // the heavy count rides in the SH scan; larger rows scan it separately
  static_assert(CAP <= 8192, "sums and shifts below assume rows of fewer than 2^13 entries");
  extern __shared__ uint64_t smem[];
  uint64_t* s_v = smem;                                             // [CAP + 2]
  uint32_t* s_res = reinterpret_cast<uint32_t*>(smem + CAP + 2);  // [CAP + 2]
  uint16_t* s_hs = reinterpret_cast<uint16_t*>(s_res + CAP + 2);   // [CAP + 2] row-local slot of heavy h
  __shared__ WSum3 s_wsum[NW];
  __shared__ double s_fsum[NW];
  __shared__ uint32_t s_mn[NW];
  __shared__ uint64_t s_ex[3 * NW];

  uint32_t start = 0;
  if (DEV) class_segment(dev, cls, 1, start, count);
  if (DEV == 1 && blockIdx.x >= count) return;
  // DEV 0 and 1: one row per workgroup, and the loop is none
  for (uint32_t row = blockIdx.x; DEV == 2 ? row < count : row == blockIdx.x; row += DEV == 2 ? gridDim.x : 1u) {
  if (DEV == 2 && row != blockIdx.x) __syncthreads();  // the arrays in LDS are about to be rewritten
  const RowRef rr = vlist[start + row];
  const uint32_t v = rr.v, off = rr.off, d = rr.d;
  const uint32_t base = off & ~3u, lead = off - base, span = lead + d;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const uint32_t pos0 = (uint32_t)PER * (uint32_t)tid;
  const bool wave_on = (uint32_t)(PER * 64 * wave) < span;

  double wd[PER];
  uint32_t live = 0;  // bit j: slot pos0 + j belongs to the row
  // the sum of the row as a plain fp64 sum where that is exact (plain_sum_is_exact), else as three limbs
  double rsum = 0.0;
  uint32_t mn = 0xFFFFFFFFu;
  if (wave_on) {
#pragma unroll
    for (int t = 0; t < PER / VEC; ++t) {
      const uint32_t pos = pos0 + (uint32_t)(VEC * t);
      float xs[4] = {0.f, 0.f, 0.f, 0.f};
      if (pos < span) {
        if constexpr (VEC == 4) {
          const float4 x = *reinterpret_cast<const float4*>(wgt + base + pos);
          xs[0] = x.x; xs[1] = x.y; xs[2] = x.z; xs[3] = x.w;
        } else {
          const float2 x = *reinterpret_cast<const float2*>(wgt + base + pos);
          xs[0] = x.x; xs[1] = x.y;
        }
      }
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const uint32_t idx = pos + k;
        const bool in = idx - lead < d;  // one unsigned compare: slots before the row wrap around
        if (in) live |= 1u << (t * VEC + k);
        const float cw = masked_weight(xs[k], in);
        wd[t * VEC + k] = (double)cw;
        rsum += wd[t * VEC + k];
        mn = min(mn, __float_as_uint(cw) - 1u);
      }
    }
    rsum = group_sum_f64<64>(rsum);
    mn = wave_min_u32(mn);
  } else {
#pragma unroll
    for (int j = 0; j < PER; ++j) wd[j] = 0.0;
  }
  if (NW > 1) {
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
  }
  if (!plain_sum_is_exact(rsum, (uint32_t)__builtin_amdgcn_readfirstlane((int)mn))) {  // uniform over the workgroup
    WSum3 sum{0.0, 0.0, 0.0};
    if (wave_on) {
#pragma unroll
      for (int j = 0; j < PER; ++j) wsum3_add(sum, wd[j]);
      sum = group_sum_wsum3<64>(sum);
    }
    if (NW > 1) {
      if (lane == 0) s_wsum[wave] = sum;
      __syncthreads();
      sum = s_wsum[0];
#pragma unroll
      for (int i = 1; i < NW; ++i) {
        sum.top += s_wsum[i].top;
        sum.mid += s_wsum[i].mid;
        sum.low += s_wsum[i].low;
      }
    }
    rsum = sum.top + sum.mid + sum.low != 0.0 ? wsum3_to_double(sum) : 0.0;
  }
  if (rsum == 0.0) {
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if ((live >> j) & 1) table[base + pos0 + j] = AliasEntry{0.0f, SKY_INVALID};
    if (tid == 0) valid[v] = 0;
    continue;
  }
  const Ledger L = make_ledger_small(d, rsum);
  const double neg_fs = -L.fs;

  float op[PER];
  uint32_t hcnt[PER];  // heavies up to and including this slot
  uint32_t heavy = 0;
  uint32_t nh, nl;
  {
    uint64_t dl[PER], dh[PER], sl[PER], sh[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const bool in = (live >> j) & 1;
      const Entry e = PACKED ? classify_small_fma(wd[j], L, neg_fs) : classify_fast(wd[j], in, L);
      dl[j] = (e.heavy || !in) ? 0 : e.amount;
      dh[j] = e.heavy ? (PACKED ? (e.amount | MERGE_CNT) : e.amount) : 0;
      op[j] = (float)e.p;
      if (e.heavy) heavy |= 1u << j;
    }
    uint64_t total_l, total_h;
    uint32_t ex_c = 0;
    if constexpr (PACKED) {
      block_scan2_flat<ROWT, PER>(dl, dh, s_ex, sl, sh, total_l, total_h, wave_on);
      nh = (uint32_t)(total_h >> 52);
    } else {
      block_scan2c_flat<ROWT, PER>(dl, dh, (uint32_t)__popc(heavy), s_ex, sl, sh, ex_c, total_l, total_h, nh, wave_on);
    }
    nl = d - nh;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const uint32_t hc = PACKED ? (uint32_t)(sh[j] >> 52) : ex_c + (uint32_t)__popc(heavy & ((2u << j) - 1));
      hcnt[j] = hc;
      if (!((live >> j) & 1)) continue;
      const uint32_t li = pos0 + j - lead;
      const bool hv = (heavy >> j) & 1;
      s_v[hv ? TOP + 1 - hc : li - hc] = hv ? (PACKED ? (sh[j] & (MERGE_CNT - 1)) : sh[j]) : sl[j];
      if (hv) s_hs[hc - 1] = (uint16_t)li;
    }
  }
  if (tid == 0) {
    s_v[nl] = ~0ull;
    s_v[TOP - nh] = ~0ull;
  }
  __syncthreads();

  if (nh) {
    if (tid == 0) s_res[0] = s_hs[0];  // the first light starts in the first heavy
    // merged positions [k0, k0 + PER) belong to this thread; a lights and k0 - a heavies come before them
    const uint32_t k0 = pos0;
    if (k0 < d) {
      uint32_t lo = k0 > nh ? k0 - nh : 0u, hi = min(k0, nl);
      while (lo < hi) {
        const uint32_t mid = (lo + hi + 1) >> 1;
        if (s_v[mid - 1] < s_v[TOP - (k0 - mid)]) lo = mid; else hi = mid - 1;
      }
      uint32_t a = lo, b = k0 - lo;
      const uint32_t steps = min((uint32_t)PER, d - k0);
      uint64_t va = s_v[a], vb = s_v[TOP - b];  // heads of the two sequences: only the one taken is read again
#pragma unroll
      for (int s = 0; s < PER; ++s) {
        if ((uint32_t)s < steps) {
          if (vb <= va) {
            s_res[TOP - b] = a;
            ++b;
            vb = s_v[TOP - b];
          } else {
            ++a;
            if (a < nl) s_res[a] = s_hs[min(b, nh - 1)];
            va = s_v[a];
          }
        }
      }
    }
    __syncthreads();
    // heavies, densely by rank: residual probability from the light that finishes them
    for (uint32_t h = tid; h < nh; h += ROWT) {
      const uint32_t r = s_res[TOP - h];
      uint32_t out = MERGE_SELF;
      if (h + 1 < nh && r < nl) out = __float_as_uint(residual_prob(L.one + s_v[TOP - h] - s_v[r], L));
      s_res[TOP - h] = out;
    }
    __syncthreads();
  }

  if (pos0 < span) {
    uint32_t oa[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const uint32_t li = pos0 + j - lead;
      const uint32_t hc = hcnt[j];
      oa[j] = li;
      if (nh && ((live >> j) & 1)) {
        if ((heavy >> j) & 1) {
          const uint32_t x = s_res[TOP - (hc - 1)];
          op[j] = x == MERGE_SELF ? 1.0f : __uint_as_float(x);
          if (x != MERGE_SELF) oa[j] = s_hs[hc];
        } else {
          oa[j] = s_res[li - hc];
        }
      }
    }
#pragma unroll
    for (int t = 0; t < PER / VEC; ++t) {
      const uint32_t pos = pos0 + (uint32_t)(VEC * t);
      if (pos >= lead && pos + VEC <= span) {
        if constexpr (VEC == 4) {
          const float p4[4] = {op[4 * t], op[4 * t + 1], op[4 * t + 2], op[4 * t + 3]};
          const uint32_t a4[4] = {oa[4 * t], oa[4 * t + 1], oa[4 * t + 2], oa[4 * t + 3]};
          store_entries4(table + base + pos, p4, a4);
        } else {
          *reinterpret_cast<uint4*>(table + base + pos) =
              make_uint4(__float_as_uint(op[2 * t]), oa[2 * t], __float_as_uint(op[2 * t + 1]), oa[2 * t + 1]);
        }
      } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          if ((live >> (t * VEC + k)) & 1) table[base + pos + k] = AliasEntry{op[VEC * t + k], oa[VEC * t + k]};
      }
    }
  }
  }  // rows of this workgroup
}

// ---------------------------------------------------------------- rows beyond LDS: global scratch
// 1024 threads stream one row three times: exact sum; prefix sums written to a scratch
// region private to the row (16 bytes per slot); searches over that scratch.
constexpr int HUGE_T = 1024;

__device__ __forceinline__ u128 block_sum_u128(u128 v, u128* s_tmp) {
  v = group_sum_u128<64>(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) s_tmp[wave] = v;
  __syncthreads();
  u128 r = s_tmp[0];
  for (int i = 1; i < HUGE_T / 64; ++i) r = add128(r, s_tmp[i]);
  return r;
}

__device__ __forceinline__ bool streaming_row(uint32_t off, uint32_t d, uint32_t max_tiles) {
  return ((off & 3u) + d + TILED_TILE - 1) / TILED_TILE > max_tiles;  // rows the tile-parallel path leaves alone
}

__global__ __launch_bounds__(HUGE_T) void build_huge_kernel(const RowRef* __restrict__ vlist, uint32_t count,
                                                            uint32_t max_tiles,
                                                            const uint64_t* __restrict__ scratch_off,
                                                            const uint32_t* __restrict__ xadj,
                                                            const float* __restrict__ wgt,
                                                            uint64_t* __restrict__ scratch,
                                                            AliasEntry* __restrict__ table,
                                                            int8_t* __restrict__ valid) {
  constexpr int NW = HUGE_T / 64;
  __shared__ u128 s_tmp[NW];
  __shared__ uint64_t s_wl[NW], s_wh[NW];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  for (uint32_t r = blockIdx.x; r < count; r += gridDim.x) {
    const uint32_t v = vlist[r].v;
    const uint32_t off = xadj[v], d = xadj[v + 1] - off;
    if (!streaming_row(off, d, max_tiles)) continue;
    const float* wr = wgt + off;
    uint64_t* g_sl = scratch + 2 * scratch_off[r];
    uint64_t* g_sh = g_sl + d;

    u128 sum{0, 0};
    for (uint32_t i = tid; i < d; i += HUGE_T) sum = add128(sum, weight_fixed(clamp_weight(wr[i])));
    sum = block_sum_u128(sum, s_tmp);
    if ((sum.lo | sum.hi) == 0) {
      for (uint32_t i = tid; i < d; i += HUGE_T) {
        table[off + i] = AliasEntry{0.0f, SKY_INVALID};
      }
      if (tid == 0) valid[v] = 0;
      continue;
    }
    const Ledger L = make_ledger(d, sum);

    uint64_t carry_l = 0, carry_h = 0;
    for (uint32_t tile = 0; tile < d; tile += HUGE_T) {
      const uint32_t i = tile + tid;
      uint64_t dl = 0, dh = 0;
      if (i < d) {
        const Entry e = classify(clamp_weight(wr[i]), L);
        if (e.heavy) dh = e.amount; else dl = e.amount;
      }
      const uint64_t il = group_scan_u64<64>(dl), ih = group_scan_u64<64>(dh);
      __syncthreads();
      if (lane == 63) { s_wl[wave] = il; s_wh[wave] = ih; }
      __syncthreads();
      uint64_t bl = carry_l, bh = carry_h, tl = 0, th = 0;
      for (int k = 0; k < NW; ++k) {
        if (k == wave) { bl += tl; bh += th; }
        tl += s_wl[k];
        th += s_wh[k];
      }
      if (i < d) {
        g_sl[i] = bl + il;
        g_sh[i] = bh + ih;
      }
      carry_l += tl;
      carry_h += th;
    }
    const uint64_t total_h = carry_h;
    __threadfence();
    __syncthreads();

    for (uint32_t i = tid; i < d; i += HUGE_T) {
      const Entry e = classify(clamp_weight(wr[i]), L);
      float op;
      uint32_t oa;
      if (!e.heavy) {
        const uint64_t x = g_sl[i] - e.amount;
        const uint32_t m = first_greater(g_sh, 0, d, x);
        op = (float)e.p;
        if (m < d) oa = m;
        else if (total_h) oa = first_greater(g_sh, 0, d, total_h - 1);
        else oa = i;
      } else {
        const uint64_t y = g_sh[i];
        const uint32_t nxt = first_greater(g_sh, i + 1, d, y);
        const uint32_t li = nxt < d ? first_greater(g_sl, 0, d, y - 1) : d;
        if (li < d) {
          op = residual_prob(L.one + y - g_sl[li], L);
          oa = nxt;
        } else {
          op = 1.0f;
          oa = i;
        }
      }
      table[off + i] = AliasEntry{op, oa};
    }
    __syncthreads();
  }
}

// Exclusive prefix sum of the degrees of the huge rows (a few thousand at most per launch of
// 1024 threads; longer lists are walked in chunks by the same block).
__global__ __launch_bounds__(1024) void huge_prefix_kernel(const RowRef* __restrict__ vlist, uint32_t count,
                                                           uint32_t max_tiles, const uint32_t* __restrict__ xadj,
                                                           uint64_t* __restrict__ scratch_off,
                                                           uint64_t* __restrict__ total) {
  __shared__ uint64_t s_w[16];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  uint64_t carry = 0;
  for (uint32_t chunk = 0; chunk < count; chunk += 1024) {
    const uint32_t r = chunk + tid;
    uint64_t d = 0;
    if (r < count) {
      const uint32_t v = vlist[r].v;
      d = xadj[v + 1] - xadj[v];
      if (!streaming_row(xadj[v], (uint32_t)d, max_tiles)) d = 0;
    }
    const uint64_t inc = group_scan_u64<64>(d);
    __syncthreads();
    if (lane == 63) s_w[wave] = inc;
    __syncthreads();
    uint64_t b = carry, t = 0;
    for (int k = 0; k < 16; ++k) {
      if (k == wave) b += t;
      t += s_w[k];
    }
    if (r < count) scratch_off[r] = b + inc - d;
    carry += t;
  }
  if (tid == 0) *total = carry;
}

// ---------------------------------------------------------------- host driver
namespace {

constexpr size_t COUNTER_BYTES = 2 * CLS_COUNT * 4 + CLS_COUNT * 8;

struct BuildScratch {
  RowRef* vlist = nullptr;       // [vcap]
  uint32_t* counters = nullptr;  // [2*CLS_COUNT] class counts (the second half is unused), then CLS_COUNT 64-bit edge totals
  uint32_t* blk_cnt = nullptr;   // [BIN_BLOCKS * CLS_COUNT] class counts of every binning block, then their prefixes
  uint64_t* huge_off = nullptr;  // [huge_cap + 1], last = total
  uint64_t* huge_scratch = nullptr;
  uint32_t vcap = 0, huge_cap = 0;
  uint64_t huge_scratch_cap = 0;
};
bool g_lds_enabled = false;  // the kernels' LDS limits are raised once per process

template <class K>
int enable_big_lds(K kernel, size_t bytes) {
  SKY_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)bytes));
  return SKY_OK;
}

// The graph's build scratch, created on first use.
BuildScratch& scratch_of(sky_graph* g) {
  if (!g->build_scratch) g->build_scratch = new BuildScratch();
  return *static_cast<BuildScratch*>(g->build_scratch);
}

}  // namespace

void free_build_scratch(sky_graph* g) {
  if (!g->build_scratch) return;
  BuildScratch* sc = static_cast<BuildScratch*>(g->build_scratch);
  void* ptrs[] = {sc->vlist, sc->counters, sc->blk_cnt, sc->huge_off, sc->huge_scratch};
  for (void* p : ptrs)
    if (p) (void)hipFree(p);
  delete sc;
  g->build_scratch = nullptr;
}

EventTimer::EventTimer(sky_graph* g) : stream(g->stream), pooled(g->ev), npooled(2) {}

int pool_get(sky_graph* g, int slot, size_t bytes, void** out) {
  sky_graph::PoolBuf& b = g->pool[slot];
  if (b.cap < bytes) {
    if (b.p) SKY_HIP(hipFree(b.p));
    b.p = nullptr;
    b.cap = 0;
    SKY_HIP(hipMalloc(&b.p, bytes + 16));
    b.cap = bytes;
  }
  *out = b.p;
  return SKY_OK;
}
void pool_release(sky_graph* g) {
  for (auto& b : g->pool) {
    if (b.p) (void)hipFree(b.p);
    b.p = nullptr;
    b.cap = 0;
  }
  for (hipEvent_t& e : g->ev) {
    if (e) (void)hipEventDestroy(e);
    e = nullptr;
  }
  for (hipStream_t& s : g->side) {
    if (s) (void)hipStreamDestroy(s);
    s = nullptr;
  }
  for (hipEvent_t& e : g->join_ev) {
    if (e) (void)hipEventDestroy(e);
    e = nullptr;
  }
  if (g->fork_ev) (void)hipEventDestroy(g->fork_ev);
  g->fork_ev = nullptr;
}

// The class kernels of one build are independent of one another once the binning pass has run.  A small build is
// bound by launching them one after another (a class of a few hundred rows takes as long as one row), so it sends
// them out in turn over the graph's stream and three side streams; the graph's stream waits for the others at
// the end.  Not used when every kernel is timed on its own, nor for builds so large that each kernel fills the GPU.
constexpr uint64_t FAN_MIN_EDGES = 2000000, FAN_MAX_EDGES = 1ull << 30;
struct StreamFan {
  sky_graph* g;
  hipStream_t main;
  bool on = false, joinable = false, used[sky_graph::SIDE_STREAMS] = {false, false, false};
  int turn = 0;
  StreamFan(sky_graph* g_, hipStream_t m) : g(g_), main(m) {}
  int ensure() {
    for (int k = 0; k < sky_graph::SIDE_STREAMS; ++k) {
      if (!g->side[k]) SKY_HIP(hipStreamCreateWithFlags(&g->side[k], hipStreamNonBlocking));
      if (!g->join_ev[k]) SKY_HIP(hipEventCreateWithFlags(&g->join_ev[k], hipEventDisableTiming));
    }
    if (!g->fork_ev) SKY_HIP(hipEventCreateWithFlags(&g->fork_ev, hipEventDisableTiming));
    return SKY_OK;
  }
  // One side stream that starts from the present end of the graph's stream, whatever start() does later; join()
  // waits for it.
  int branch(int k, hipStream_t* out) {
    SKY_TRY(ensure());
    SKY_HIP(hipEventRecord(g->fork_ev, main));
    SKY_HIP(hipStreamWaitEvent(g->side[k], g->fork_ev, 0));
    used[k] = true;
    joinable = true;
    *out = g->side[k];
    return SKY_OK;
  }
  int start() {  // after the binning pass has been enqueued on the graph's stream
    SKY_TRY(ensure());
    SKY_HIP(hipEventRecord(g->fork_ev, main));
    for (int k = 0; k < sky_graph::SIDE_STREAMS; ++k) SKY_HIP(hipStreamWaitEvent(g->side[k], g->fork_ev, 0));
    on = true;
    joinable = true;
    return SKY_OK;
  }
  hipStream_t next() {
    if (!on) return main;
    const int k = turn++ % (sky_graph::SIDE_STREAMS + 1);
    if (k == sky_graph::SIDE_STREAMS) return main;
    used[k] = true;
    return g->side[k];
  }
  // The stream that carries the least work so far (`work`: the launch's entries, weighted by the caller where a
  // kernel is slow): a kernel queued behind a long one waits for it while other streams run dry.
  uint64_t load[sky_graph::SIDE_STREAMS + 1] = {0, 0, 0, 0};
  hipStream_t next(uint64_t work) {
    if (!on) return main;
    int k = 0;
    for (int i = 1; i <= sky_graph::SIDE_STREAMS; ++i)
      if (load[i] < load[k]) k = i;
    load[k] += work + 1;
    if (k == sky_graph::SIDE_STREAMS) return main;
    used[k] = true;
    return g->side[k];
  }
  int join() {
    if (!joinable) return SKY_OK;
    on = joinable = false;
    for (int k = 0; k < sky_graph::SIDE_STREAMS; ++k)
      if (used[k]) {
        used[k] = false;
        SKY_HIP(hipEventRecord(g->join_ev[k], g->side[k]));
        SKY_HIP(hipStreamWaitEvent(main, g->join_ev[k], 0));
      }
    return SKY_OK;
  }
  ~StreamFan() { (void)join(); }  // an error in between still leaves the graph's stream behind every kernel
};
// The graph's stream replaced for the duration of a call that takes it from the graph.
struct StreamSwap {
  sky_graph* g;
  hipStream_t saved;
  StreamSwap(sky_graph* g_, hipStream_t s) : g(g_), saved(g_->stream) { g->stream = s; }
  ~StreamSwap() { g->stream = saved; }
};

int EventTimer::mark(const char* name, uint64_t e) {
  hipEvent_t x;
  if (ev.size() < npooled) {
    if (!pooled[ev.size()]) SKY_HIP(hipEventCreate(&pooled[ev.size()]));
    x = pooled[ev.size()];
  } else {
    SKY_HIP(hipEventCreate(&x));
  }
  SKY_HIP(hipEventRecord(x, stream));
  ev.push_back(x);
  names.push_back(name);
  edges.push_back(e);
  return SKY_OK;
}
int EventTimer::finish(std::vector<sky_graph::ProfileEntry>* profile, double* seconds) {
  SKY_HIP(hipStreamSynchronize(stream));
  SKY_HIP(hipGetLastError());
  if (profile) profile->clear();
  for (size_t i = 1; i < ev.size(); ++i) {
    float ms = 0;
    SKY_HIP(hipEventElapsedTime(&ms, ev[i - 1], ev[i]));
    if (profile) profile->push_back({names[i], ms, edges[i]});
  }
  float total_ms = 0;
  if (ev.size() >= 2) SKY_HIP(hipEventElapsedTime(&total_ms, ev.front(), ev.back()));
  if (seconds) *seconds = total_ms * 1e-3;
  return SKY_OK;
}
EventTimer::~EventTimer() {
  for (size_t i = npooled; i < ev.size(); ++i) (void)hipEventDestroy(ev[i]);
}

int ensure_table_storage(sky_graph* g) {
  if (!g->table) SKY_TRY(alloc_padded(&g->table, (size_t)g->E));
  if (!g->valid) SKY_TRY(alloc_padded(&g->valid, (size_t)g->V));
  return SKY_OK;
}

int prepare_build_scratch(sky_graph* g, uint32_t max_rows) {
  BuildScratch& sc = scratch_of(g);
  if (sc.vcap < max_rows) {
    if (sc.vlist) SKY_HIP(hipFree(sc.vlist));
    sc.vlist = nullptr;
    sc.vcap = 0;
    SKY_HIP(hipMalloc((void**)&sc.vlist, (size_t)max_rows * sizeof(RowRef) + 16));
    sc.vcap = max_rows;
  }
  if (!sc.counters) SKY_HIP(hipMalloc((void**)&sc.counters, COUNTER_BYTES));
  if (!sc.blk_cnt) SKY_HIP(hipMalloc((void**)&sc.blk_cnt, (size_t)BIN_BLOCKS * CLS_COUNT * 4));
  if (!g_lds_enabled) {
    SKY_TRY(enable_big_lds(build_lds_kernel<512, 2>, 512 * 4 * 2 * 16));
    SKY_TRY(enable_big_lds(build_merge_kernel<512, 10>, (512 * 10 + 2) * 14));
    SKY_TRY(enable_big_lds(build_merge_kernel<768, 6>, (768 * 6 + 2) * 14));
    SKY_TRY(enable_big_lds((build_merge_kernel<512, 10, 4, 1>), (512 * 10 + 2) * 14));
    SKY_TRY(enable_big_lds((build_merge_kernel<768, 6, 4, 1>), (768 * 6 + 2) * 14));
    g_lds_enabled = true;
  }
  return SKY_OK;
}

// Builds the rows listed in `src` (device array of n vertex ids; null = vertices 0..n-1).
// prepare_build_scratch(n) and ensure_table_storage must have been called.
int build_rows(sky_graph* g, const uint32_t* src, uint32_t n, EventTimer* tm) {
  hipStream_t st = g->stream;
  g->has_walk_index = false;  // the table entries it was made from are about to change
  BuildScratch& sc = scratch_of(g);
  uint32_t counts[CLS_COUNT] = {0}, starts[CLS_COUNT] = {0};
  struct {
    uint32_t counts[2 * CLS_COUNT];
    unsigned long long edges[CLS_COUNT];
  } host = {};
  static_assert(sizeof(host) == COUNTER_BYTES, "counter block layout");
  // A large build leaves its rows of at most 32 entries to small_rows_kernel, which builds them where they lie,
  // without lists.  Taken alone it is slower than the class kernels of these rows (1.39 against 1.12 ms on the
  // scale-26 graph), but it does not depend on the binning pass: on a side stream it runs beside the binning and
  // the kernels of the long rows (it waits on memory, they on the vector ALU): 10.2 -> 9.95 ms for the whole build.
  // Smaller builds, whose class kernels already overlap, gain nothing (scale 24: 3 % slower).
  const long long sip = option(g, OPT_SMALL_IN_PLACE);
  const bool small_in_place = sip < 0 ? n >= (1u << 25) : sip != 0;
  const int listed_from = small_in_place ? CLS_G16 : CLS_G2;
  StreamFan fan(g, st);
  auto launch_small = [&](hipStream_t s) {
    const uint32_t per_wave = std::max(256u, std::min(SMALL_RANGE, n / 16384u / 64u * 64u));
    hipLaunchKernelGGL(small_rows_kernel, dim3((n + per_wave - 1) / per_wave), dim3(64), 0, s, g->xadj, g->adjwgt, src, n,
                       per_wave, g->table, g->valid);
  };
  if (n > 0) {
    if (small_in_place && !tm) {
      hipStream_t side;
      SKY_TRY(fan.branch(sky_graph::SIDE_STREAMS - 1, &side));
      launch_small(side);
    }
    SKY_HIP(hipMemsetAsync(sc.counters, 0, COUNTER_BYTES, st));
    // at most BIN_BLOCKS blocks, each a multiple of one scatter step
    const uint32_t step = 256u * BIN_ITEMS;
    const uint32_t per_block = ((n + BIN_BLOCKS - 1) / BIN_BLOCKS + step - 1) / step * step;
    const uint32_t blocks = (n + per_block - 1) / per_block;
    hipLaunchKernelGGL(bin_count_kernel, dim3(blocks), dim3(256), 0, st, g->xadj, src, n, (const uint32_t*)nullptr,
                       per_block, listed_from, sc.blk_cnt,
                       reinterpret_cast<unsigned long long*>(sc.counters + 2 * CLS_COUNT));
    hipLaunchKernelGGL(bin_offsets_kernel, dim3(CLS_COUNT), dim3(256), 0, st, sc.blk_cnt, blocks, sc.counters);
    hipLaunchKernelGGL(bin_scatter_kernel, dim3(blocks), dim3(256), 0, st, g->xadj, g->adjwgt, src, n,
                       (const uint32_t*)nullptr, per_block, listed_from, sc.counters, sc.blk_cnt, sc.vlist, g->table,
                       g->valid);
    // The class sizes decide the launches that follow.  Those of all vertices depend on xadj alone and are kept
    // with the graph after the first time; any other list of rows is waited for.
    const bool all_rows = src == nullptr && n == g->V;
    if (all_rows && g->bin_known && g->bin_listed_from == listed_from) {
      for (int c = 0; c < CLS_COUNT; ++c) {
        host.counts[c] = g->bin_counts[c];
        host.edges[c] = g->bin_edges[c];
      }
    } else {
      SKY_HIP(hipMemcpyAsync(&host, sc.counters, COUNTER_BYTES, hipMemcpyDeviceToHost, st));
      SKY_HIP(hipStreamSynchronize(st));
      if (all_rows) {
        for (int c = 0; c < CLS_COUNT; ++c) {
          g->bin_counts[c] = host.counts[c];
          g->bin_edges[c] = host.edges[c];
        }
        g->bin_known = true;
        g->bin_listed_from = listed_from;
      }
    }
    for (int c = 0; c < CLS_COUNT; ++c) counts[c] = host.counts[c];
    uint32_t acc = 0;
    for (int c = 0; c < CLS_COUNT; ++c) {
      starts[c] = acc;
      acc += counts[c];
    }
  }
  const uint64_t small_edges = host.edges[CLS_TINY] + host.edges[CLS_G2] + host.edges[CLS_G4] + host.edges[CLS_G8];
  if (tm) SKY_TRY(tm->mark("bin", small_in_place ? 0 : host.edges[CLS_TINY]));
  if (tm && small_in_place && n > 0) {
    launch_small(st);
    SKY_TRY(tm->mark("small", small_edges));
  }
  RowRef* const vlist = sc.vlist;
  uint64_t call_edges = 0;
  for (int c = 0; c < CLS_COUNT; ++c) call_edges += host.edges[c];
  if (!tm && option(g, OPT_BUILD_STREAMS) && call_edges >= FAN_MIN_EDGES && call_edges < FAN_MAX_EDGES) SKY_TRY(fan.start());

  auto grp = [&](int cls, auto kernel, int G, const char* name) -> int {
    const uint32_t cnt = counts[cls];
    if (cnt) {
      const uint32_t per_block = 256 / G;
      hipLaunchKernelGGL(kernel, dim3((cnt + per_block - 1) / per_block), dim3(256), 0, fan.next(host.edges[cls]), vlist + starts[cls],
                         cnt, (const uint32_t*)nullptr, 0, g->adjwgt, g->table, g->valid);
    }
    return (tm && cnt) ? tm->mark(name, host.edges[cls]) : SKY_OK;  // no bracket for an empty class
  };
  const bool row_merge = option(g, OPT_ROW_MERGE) != 0;
  // Rows of 8190..STREAM_MAX_DEG entries: one workgroup streams a row.  A small streaming class is not worth its
  // own launch (too few workgroups to fill the GPU): its rows then go to the tile-parallel path together with the
  // HUGE class.  The rows above 65533 entries keep one workgroup busy for up to 1.5 ms; they join the launch (and
  // start first) only when it holds enough other rows to run that long anyway, else they are built tile by tile.
  // The lists lie back to back: STREAM, STREAM_LAST, STREAM_WIDE, HUGE.
  const uint32_t narrow_rows = counts[CLS_STREAM] + counts[CLS_STREAM_LAST];
  const uint64_t narrow_edges = host.edges[CLS_STREAM] + host.edges[CLS_STREAM_LAST];
  const uint64_t all_stream_edges = narrow_edges + host.edges[CLS_STREAM_WIDE];
  const bool stream_to_tiled = !row_merge || all_stream_edges <= (uint64_t)option(g, OPT_STREAM_MIN_EDGES);
  const bool wide_streamed = !stream_to_tiled && all_stream_edges >= (uint64_t)option(g, OPT_STREAM_WIDE_MIN_EDGES);
  const uint32_t wide_rows = wide_streamed ? counts[CLS_STREAM_WIDE] : 0;
  if (!stream_to_tiled && narrow_rows + wide_rows) {
    // the streaming kernel takes three times as long for an entry as the others when it shares the GPU with them
    StreamSwap sw(g, fan.next(3 * (narrow_edges + (wide_streamed ? host.edges[CLS_STREAM_WIDE] : 0))));
    SKY_TRY(build_rows_stream(g, vlist + starts[CLS_STREAM_WIDE], wide_rows, vlist + starts[CLS_STREAM], narrow_rows));
    if (tm) SKY_TRY(tm->mark("stream", narrow_edges + (wide_streamed ? host.edges[CLS_STREAM_WIDE] : 0)));
  }
  // Rows of 5118..8189 entries: one workgroup holds the row (without row_merge they are built tile by tile).
  if (row_merge && counts[CLS_HOLD]) {
    {
      StreamSwap sw(g, fan.next(2 * host.edges[CLS_HOLD]));
      SKY_TRY(build_rows_hold(g, vlist + starts[CLS_HOLD], counts[CLS_HOLD], nullptr, 0));
    }
    if (tm) SKY_TRY(tm->mark("hold", host.edges[CLS_HOLD]));
  }
  auto lds = [&](int cls, auto kernel, int rowt, int t, const char* name) -> int {
    const uint32_t cnt = counts[cls];
    if (cnt) {
      const size_t bytes = (size_t)rowt * 4 * t * 16;
      hipLaunchKernelGGL(kernel, dim3(cnt), dim3(rowt), bytes, fan.next(host.edges[cls]), vlist + starts[cls], g->xadj, g->adjwgt,
                         g->table, g->valid);
    }
    return (tm && cnt) ? tm->mark(name, host.edges[cls]) : SKY_OK;  // no bracket for an empty class
  };
  auto mrg = [&](int cls, auto kernel, int rowt, int per, const char* name) -> int {
    const uint32_t cnt = counts[cls];
    if (cnt) {
      const size_t bytes = ((size_t)rowt * per + 2) * 14;
      hipLaunchKernelGGL(kernel, dim3(cnt), dim3(rowt), bytes, fan.next(host.edges[cls]), vlist + starts[cls], cnt,
                         (const uint32_t*)nullptr, 0, g->adjwgt, g->table, g->valid);
    }
    return (tm && cnt) ? tm->mark(name, host.edges[cls]) : SKY_OK;  // no bracket for an empty class
  };
  static const char* const mw_name[9] = {"mw2", "mw3", "mw4", "mw5", "mw6", "mw7", "mw8", "mw9", "mw10"};
  if (row_merge) {
    SKY_TRY(mrg(CLS_LDS_W1, build_merge_kernel<64, 4>, 64, 4, "lds_w1"));
    SKY_TRY(mrg(CLS_LDS_W6, build_merge_kernel<64, 6>, 64, 6, "lds_w6"));
    SKY_TRY(mrg(CLS_LDS_W2, build_merge_kernel<64, 8>, 64, 8, "lds_w2"));
    SKY_TRY(mrg(CLS_MW2_6, build_merge_kernel<128, 6>, 128, 6, "mw2_6"));
#define SKY_MW(NW) SKY_TRY(mrg(CLS_MW2 + NW - 2, build_merge_kernel<64 * NW, 8>, 64 * NW, 8, mw_name[NW - 2]))
    // Class nw holds rows that fit 512 nw slots.  Where a shape with an even number of slots per thread and a
    // multiple of 4 wavefronts covers that span exactly, it is used instead of nw wavefronts of 8 slots: every
    // SIMD of the CU then carries the same number of a workgroup's wavefronts, and 6..10 slots per thread need
    // 70..110 registers (measured on rows of one class each: 13 % faster for nw = 3, 24 % for 5, 41 % for 6,
    // 2 % for 7, 31 % for 9, 28 % for 10, where 10 wavefronts of 8 slots also spill).
    SKY_MW(2);
    SKY_TRY(mrg(CLS_MW2 + 1, build_merge_kernel<256, 6>, 256, 6, mw_name[1]));
    SKY_MW(4);
    SKY_TRY(mrg(CLS_MW2 + 3, build_merge_kernel<256, 10>, 256, 10, mw_name[3]));
    SKY_TRY(mrg(CLS_MW2 + 4, build_merge_kernel<512, 6>, 512, 6, mw_name[4]));
    SKY_TRY(mrg(CLS_MW2 + 5, build_merge_kernel<256, 14>, 256, 14, mw_name[5]));
    SKY_MW(8);
    SKY_TRY(mrg(CLS_MW2 + 7, build_merge_kernel<768, 6>, 768, 6, mw_name[7]));
    SKY_TRY(mrg(CLS_MW2 + 8, build_merge_kernel<512, 10>, 512, 10, mw_name[8]));
#undef SKY_MW
  } else {
    SKY_TRY(lds(CLS_LDS_W1, build_lds_kernel<64, 1>, 64, 1, "lds_w1"));
    SKY_TRY(lds(CLS_LDS_W6, build_lds_kernel<64, 2>, 64, 2, "lds_w6"));
    SKY_TRY(lds(CLS_LDS_W2, build_lds_kernel<64, 2>, 64, 2, "lds_w2"));
    SKY_TRY(lds(CLS_MW2_6, build_lds_kernel<128, 2>, 128, 2, "mw2_6"));
    for (int nw = 2; nw <= MERGE_MAX_NW; ++nw) {
      const int cls = CLS_MW2 + nw - 2;
      if (nw <= 2) SKY_TRY(lds(cls, build_lds_kernel<128, 2>, 128, 2, mw_name[nw - 2]));
      else if (nw <= 4) SKY_TRY(lds(cls, build_lds_kernel<256, 2>, 256, 2, mw_name[nw - 2]));
      else if (nw <= 8) SKY_TRY(lds(cls, build_lds_kernel<512, 2>, 512, 2, mw_name[nw - 2]));
      else {  // this variant has no kernel for rows of 4094..5117 entries: tile-parallel path
        if (counts[cls]) {
          uint32_t skipped = 0;
          SKY_TRY(fan.join());  // the tile-parallel path's scratch serves one call at a time
          SKY_TRY(build_rows_tiled(g, vlist + starts[cls], counts[cls], &skipped, nullptr, 0));
          if (skipped) return fail(SKY_ERR_STATE, "tiled_max_tiles below 9 needs row_merge");
        }
        if (tm) SKY_TRY(tm->mark(mw_name[nw - 2], host.edges[cls]));
      }
    }
  }

  SKY_TRY(grp(CLS_G2, build_group_kernel<2, 4>, 2, "g2"));
  SKY_TRY(grp(CLS_G4, build_group_kernel<4, 4>, 4, "g4"));
  SKY_TRY(grp(CLS_G8, build_group_kernel<8, 4>, 8, "g8"));
  SKY_TRY(grp(CLS_G16, build_group_kernel<16, 4>, 16, "g16"));
  SKY_TRY(grp(CLS_G32, build_group_kernel<32, 4>, 32, "g32"));
  SKY_TRY(grp(CLS_G32S, build_group_kernel<32, 5>, 32, "g32s"));
  SKY_TRY(grp(CLS_G32X, build_group_kernel<32, 6>, 32, "g32x"));

  // the lists HOLD, STREAM, STREAM_LAST, STREAM_WIDE, HUGE lie back to back (the class numbers between are unused)
  const uint32_t held_rows = row_merge ? 0 : counts[CLS_HOLD];
  const uint32_t tiled_rows =
      counts[CLS_HUGE] + (wide_streamed ? 0 : counts[CLS_STREAM_WIDE]) + (stream_to_tiled ? narrow_rows : 0) + held_rows;
  const uint64_t tiled_edges = host.edges[CLS_HUGE] + (wide_streamed ? 0 : host.edges[CLS_STREAM_WIDE]) +
                               (stream_to_tiled ? narrow_edges : 0) +
                               (row_merge ? 0 : host.edges[CLS_HOLD]);
  const RowRef* tiled_list =
      vlist + (held_rows ? starts[CLS_HOLD]
                         : stream_to_tiled ? starts[CLS_STREAM] : (wide_streamed ? starts[CLS_HUGE] : starts[CLS_STREAM_WIDE]));
  if (tiled_rows) {
    const uint32_t cnt = tiled_rows;
    uint32_t skipped = 0;
    {
      StreamSwap sw(g, fan.next(2 * tiled_edges));
      SKY_TRY(build_rows_tiled(g, tiled_list, cnt, &skipped, tm, tiled_edges));
    }
    SKY_TRY(fan.join());
    if (skipped) {  // rows with more tiles than the tile-parallel path takes: one workgroup streams each
      const uint32_t max_tiles = tiled_max_tiles(g);
      if (sc.huge_cap < cnt) {
        if (sc.huge_off) SKY_HIP(hipFree(sc.huge_off));
        sc.huge_off = nullptr;
        sc.huge_cap = 0;
        SKY_HIP(hipMalloc((void**)&sc.huge_off, ((size_t)cnt + 1) * 8));
        sc.huge_cap = cnt;
      }
      hipLaunchKernelGGL(huge_prefix_kernel, dim3(1), dim3(1024), 0, st, tiled_list, cnt, max_tiles,
                         g->xadj, sc.huge_off, sc.huge_off + cnt);
      uint64_t total = 0;
      SKY_HIP(hipMemcpyAsync(&total, sc.huge_off + cnt, 8, hipMemcpyDeviceToHost, st));
      SKY_HIP(hipStreamSynchronize(st));
      if (sc.huge_scratch_cap < total) {
        if (sc.huge_scratch) SKY_HIP(hipFree(sc.huge_scratch));
        sc.huge_scratch = nullptr;
        sc.huge_scratch_cap = 0;
        SKY_HIP(hipMalloc((void**)&sc.huge_scratch, total * 16));
        sc.huge_scratch_cap = total;
      }
      hipLaunchKernelGGL(build_huge_kernel, dim3(std::min<uint32_t>(cnt, 512)), dim3(HUGE_T), 0, st,
                         tiled_list, cnt, max_tiles, sc.huge_off, g->xadj, g->adjwgt, sc.huge_scratch,
                         g->table, g->valid);
      if (tm) SKY_TRY(tm->mark("streamed", 0));
    }
  }
  return fan.join();
}

// ---------------------------------------------------------------- builds that never wait for the device
// The rows of a frontier: how many there are, and how many fall into each degree class, is known on the device
// only.  The binning kernels take the length of the list from a device word, every class kernel finds its segment
// of the row list through the counter block (class_segment) and strides over it with a grid of fixed size.  Which
// classes can hold a row at all depends on the graph alone: a census of all vertices, taken once per graph, lets
// the host skip the launches of the classes the graph does not populate.
// Most workgroups of a launch, by workgroup size: enough to fill every CU several times over (a class that
// turns out small leaves most of them with nothing to do, which costs microseconds).
constexpr uint32_t DEV_GRID_STREAM = 512;
constexpr uint32_t dev_grid_cap(int threads) { return threads <= 64 ? 16384u : threads <= 256 ? 8192u : 2048u; }

bool build_rows_dev_possible(const sky_graph* g) { return option(g, OPT_ROW_MERGE) != 0 && tiled_max_tiles(g) == (1u << 22); }

int ensure_class_census(sky_graph* g) {
  if (g->bin_known || g->V == 0) return SKY_OK;
  hipStream_t st = g->stream;
  SKY_TRY(prepare_build_scratch(g, 1));
  BuildScratch& sc = scratch_of(g);
  struct {
    uint32_t counts[2 * CLS_COUNT];
    unsigned long long edges[CLS_COUNT];
  } host = {};
  const uint32_t n = g->V, step = 256u * BIN_ITEMS;
  const uint32_t per_block = ((n + BIN_BLOCKS - 1) / BIN_BLOCKS + step - 1) / step * step;
  const uint32_t blocks = (n + per_block - 1) / per_block;
  SKY_HIP(hipMemsetAsync(sc.counters, 0, COUNTER_BYTES, st));
  hipLaunchKernelGGL(bin_count_kernel, dim3(blocks), dim3(256), 0, st, g->xadj, (const uint32_t*)nullptr, n,
                     (const uint32_t*)nullptr, per_block, (int)CLS_G2, sc.blk_cnt,
                     reinterpret_cast<unsigned long long*>(sc.counters + 2 * CLS_COUNT));
  hipLaunchKernelGGL(bin_offsets_kernel, dim3(CLS_COUNT), dim3(256), 0, st, sc.blk_cnt, blocks, sc.counters);
  SKY_HIP(hipMemcpyAsync(&host, sc.counters, COUNTER_BYTES, hipMemcpyDeviceToHost, st));
  SKY_HIP(hipStreamSynchronize(st));
  for (int c = 0; c < CLS_COUNT; ++c) {
    g->bin_counts[c] = host.counts[c];
    g->bin_edges[c] = host.edges[c];
  }
  g->bin_known = true;
  g->bin_listed_from = CLS_G2;
  return SKY_OK;
}

int build_rows_dev(sky_graph* g, const uint32_t* src, const uint32_t* n_dev, uint32_t n_upper) {
  if (n_upper == 0) return SKY_OK;
  if (!build_rows_dev_possible(g) || !g->bin_known)
    return fail(SKY_ERR_STATE, "build_rows_dev: needs the class census and rows the streaming kernel takes");
  hipStream_t st = g->stream;
  g->has_walk_index = false;
  BuildScratch& sc = scratch_of(g);
  const uint32_t step = 256u * BIN_ITEMS;
  const uint32_t per_block = ((n_upper + BIN_BLOCKS - 1) / BIN_BLOCKS + step - 1) / step * step;
  const uint32_t blocks = (n_upper + per_block - 1) / per_block;
  SKY_HIP(hipMemsetAsync(sc.counters, 0, COUNTER_BYTES, st));
  hipLaunchKernelGGL(bin_count_kernel, dim3(blocks), dim3(256), 0, st, g->xadj, src, n_upper, n_dev, per_block,
                     (int)CLS_G2, sc.blk_cnt, reinterpret_cast<unsigned long long*>(sc.counters + 2 * CLS_COUNT));
  hipLaunchKernelGGL(bin_offsets_kernel, dim3(CLS_COUNT), dim3(256), 0, st, sc.blk_cnt, blocks, sc.counters);
  hipLaunchKernelGGL(bin_scatter_kernel, dim3(blocks), dim3(256), 0, st, g->xadj, g->adjwgt, src, n_upper, n_dev,
                     per_block, (int)CLS_G2, sc.counters, sc.blk_cnt, sc.vlist, g->table, g->valid);
  // a class of the graph holds bin_counts[c] rows at most (bin_edges tells whether it holds any: the counts of the
  // census leave out the classes that a large full build does not list)
  auto rows_of = [&](int cls) -> uint32_t {
    if (g->bin_edges[cls] == 0) return 0;
    const uint32_t in_graph = g->bin_listed_from <= cls ? g->bin_counts[cls] : n_upper;
    return std::min(n_upper, std::max(1u, in_graph));
  };
  const uint32_t* const dev = sc.counters;
  const RowRef* const vlist = sc.vlist;
  // the class kernels are independent of one another: they go out in turn over the graph's stream and its side streams
  StreamFan fan(g, st);
  if (option(g, OPT_BUILD_STREAMS) && n_upper >= 4096) SKY_TRY(fan.start());
  // Rows of 8190 entries and more first, because theirs is the longest chain of launches.  The classes STREAM,
  // STREAM_LAST, STREAM_WIDE, HUGE lie back to back.  What the graph holds of them decides, as in a build of all
  // rows, which go to the streaming kernel (one workgroup per row) and which are built tile by tile by the whole
  // GPU: the two longest classes always are (a frontier holds a few such rows at most, and one workgroup would need
  // a millisecond for one), the other two when the graph has too few of their rows to fill the GPU with one
  // workgroup each.
  static_assert(CLS_STREAM_LAST == CLS_STREAM + 1 && CLS_STREAM_WIDE == CLS_STREAM + 2 && CLS_HUGE == CLS_STREAM + 3,
                "the lists of the long rows lie back to back");
  const bool narrow_tiled = g->bin_edges[CLS_STREAM] + g->bin_edges[CLS_STREAM_LAST] <= (uint64_t)option(g, OPT_STREAM_MIN_EDGES);
  const uint32_t stream_rows = narrow_tiled ? 0 : rows_of(CLS_STREAM) + rows_of(CLS_STREAM_LAST);
  const int t_first = narrow_tiled ? CLS_STREAM : CLS_STREAM_WIDE;
  uint32_t tiled_rows = 0;
  uint64_t tiled_edges = 0;
  for (int c = t_first; c <= CLS_HUGE; ++c) {
    tiled_rows += rows_of(c);
    tiled_edges += g->bin_edges[c];
  }
  // A stream is chosen by the work it already carries; the work of a class is what the graph holds of it (a
  // frontier mirrors the graph), weighted for the kernels of the long rows, which are slow beside the others.
  if (tiled_rows) {
    StreamSwap sw(g, fan.next(2 * tiled_edges));
    SKY_TRY(build_rows_tiled_dev(g, vlist, dev, t_first, CLS_HUGE - t_first + 1, tiled_rows, tiled_edges));
  }
  // the streaming kernel fills the LDS of every CU it reaches: the tile-parallel path, whose first kernels are small,
  // is enqueued before it
  if (stream_rows) {
    StreamSwap sw(g, fan.next(3 * (g->bin_edges[CLS_STREAM] + g->bin_edges[CLS_STREAM_LAST])));
    SKY_TRY(build_rows_stream_dev(g, vlist, dev, 2, std::min(DEV_GRID_STREAM, stream_rows)));
  }
  auto grp = [&](int cls, auto kernel, int G) {
    const uint32_t rows = rows_of(cls);
    if (!rows) return;
    const uint32_t per = 256 / G;
    hipLaunchKernelGGL(kernel, dim3(std::min(dev_grid_cap(256), (rows + per - 1) / per)), dim3(256), 0,
                       fan.next(g->bin_edges[cls]), vlist, 0u, dev, cls, g->adjwgt, g->table, g->valid);
  };
  auto mrg = [&](int cls, auto kernel, int rowt, int per) {
    const uint32_t rows = rows_of(cls);
    if (!rows) return;
    const size_t bytes = ((size_t)rowt * per + 2) * 14;
    // one wavefront per row: a striding grid; larger workgroups: one per row the class can hold (the code of a
    // loop over rows costs these kernels registers they do not have)
    hipLaunchKernelGGL(kernel, dim3(rowt <= 64 ? std::min(dev_grid_cap(rowt), rows) : rows), dim3(rowt), bytes,
                       fan.next(g->bin_edges[cls]), vlist, 0u, dev, cls, g->adjwgt, g->table, g->valid);
  };
  // The class kernels go out in the order of the classes' sizes in the graph, the largest first: a frontier mirrors
  // the graph, and the streams should not end on a long kernel that started last.
  std::vector<std::pair<unsigned long long, std::function<void()>>> queue;
#define SKY_Q(CLS, CALL) queue.emplace_back(g->bin_edges[CLS], [&] { CALL; })
  SKY_Q(CLS_G2, grp(CLS_G2, (build_group_kernel<2, 4, true>), 2));
  SKY_Q(CLS_G4, grp(CLS_G4, (build_group_kernel<4, 4, true>), 4));
  SKY_Q(CLS_G8, grp(CLS_G8, (build_group_kernel<8, 4, true>), 8));
  SKY_Q(CLS_G16, grp(CLS_G16, (build_group_kernel<16, 4, true>), 16));
  SKY_Q(CLS_G32, grp(CLS_G32, (build_group_kernel<32, 4, true>), 32));
  SKY_Q(CLS_G32S, grp(CLS_G32S, (build_group_kernel<32, 5, true>), 32));
  SKY_Q(CLS_G32X, grp(CLS_G32X, (build_group_kernel<32, 6, true>), 32));
  SKY_Q(CLS_LDS_W1, mrg(CLS_LDS_W1, (build_merge_kernel<64, 4, 4, 2>), 64, 4));
  SKY_Q(CLS_LDS_W6, mrg(CLS_LDS_W6, (build_merge_kernel<64, 6, 4, 2>), 64, 6));
  SKY_Q(CLS_LDS_W2, mrg(CLS_LDS_W2, (build_merge_kernel<64, 8, 4, 2>), 64, 8));
  SKY_Q(CLS_MW2_6, mrg(CLS_MW2_6, (build_merge_kernel<128, 6, 4, 1>), 128, 6));
#define SKY_MW(NW) SKY_Q(CLS_MW2 + NW - 2, mrg(CLS_MW2 + NW - 2, (build_merge_kernel<64 * NW, 8, 4, 1>), 64 * NW, 8))
  SKY_MW(2);
  SKY_Q(CLS_MW2 + 1, mrg(CLS_MW2 + 1, (build_merge_kernel<256, 6, 4, 1>), 256, 6));
  SKY_MW(4);
  SKY_Q(CLS_MW2 + 3, mrg(CLS_MW2 + 3, (build_merge_kernel<256, 10, 4, 1>), 256, 10));
  SKY_Q(CLS_MW2 + 4, mrg(CLS_MW2 + 4, (build_merge_kernel<512, 6, 4, 1>), 512, 6));
  SKY_Q(CLS_MW2 + 5, mrg(CLS_MW2 + 5, (build_merge_kernel<256, 14, 4, 1>), 256, 14));
  SKY_MW(8);
  SKY_Q(CLS_MW2 + 7, mrg(CLS_MW2 + 7, (build_merge_kernel<768, 6, 4, 1>), 768, 6));
  SKY_Q(CLS_MW2 + 8, mrg(CLS_MW2 + 8, (build_merge_kernel<512, 10, 4, 1>), 512, 10));
#undef SKY_MW
  auto hold = [&](int cls) -> int {
    const uint32_t rows = rows_of(cls);
    if (!rows) return SKY_OK;
    StreamSwap sw(g, fan.next(2 * g->bin_edges[cls]));
    return build_rows_hold(g, vlist, rows, dev, cls);
  };
  int hold_rc = SKY_OK;
  SKY_Q(CLS_HOLD, { const int rc = hold(CLS_HOLD); if (rc != SKY_OK) hold_rc = rc; });
#undef SKY_Q
  std::stable_sort(queue.begin(), queue.end(), [](const auto& a, const auto& b) { return a.first > b.first; });
  for (auto& q : queue) q.second();
  SKY_TRY(fan.join());
  if (hold_rc != SKY_OK) return hold_rc;
  SKY_HIP(hipGetLastError());
  return SKY_OK;
}

int build_all_tables(sky_graph* g, double* seconds) {
  SKY_TRY(ensure_table_storage(g));
  SKY_TRY(prepare_build_scratch(g, g->V));
  EventTimer tm(g);
  SKY_TRY(tm.mark("start", 0));
  if (option(g, OPT_BUILD_PROFILE)) {
    SKY_TRY(build_rows(g, nullptr, g->V, &tm));
  } else {  // one bracket around the whole build: no event between the kernels
    SKY_TRY(build_rows(g, nullptr, g->V, nullptr));
    SKY_TRY(tm.mark("build", g->E));
  }
  SKY_TRY(tm.finish(&g->build_profile, seconds));
  g->has_tables = true;
  return SKY_OK;
}

}  // namespace sky
