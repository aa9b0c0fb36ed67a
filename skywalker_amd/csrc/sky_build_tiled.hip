// Alias tables of rows too long for one workgroup's LDS, built tile by tile by the whole GPU.
//
// A row is cut into tiles of 1024 slots counted from its 16-byte aligned start.  The table is the
// same pure function of the weights as everywhere else (see sky_build.hip); only the evaluation
// order changes:
//   tiled_sum_kernel      per tile   exact 128-bit partial sum of the weights
//   tiled_ledger_kernel   per row    total -> scale and fraction bits
//   tiled_totals_kernel   per tile   sum of deficits, sum of surpluses, first and last heavy
//   tiled_scan_kernel     per row    exclusive prefix of the tile totals (BL, BH), next heavy after each tile
//   tiled_emit_kernel     per tile   every entry of the tile
// In the last step a light with exclusive deficit prefix x needs the first slot whose surplus prefix
// exceeds x.  The tile holding that slot ("partner") follows from BH; its per-slot prefix is
// recomputed from the weights into LDS and searched there.  Heavies look up their retiring
// light the same way against BL.  Lights and heavies of a tile are monotone in their keys, so the
// partners of one tile are a contiguous run and the total number of (tile, partner) pairs of a row
// is at most twice its tile count: no per-slot scratch in global memory, O(1) passes over the weights.
#include <algorithm>

#include "sky_build_common.h"
#include "sky_graph.h"

namespace sky {

constexpr int TL_T = 256;                // threads per tile
constexpr int TL_Q = 1;                  // float4 quads per thread
constexpr int TILE = TL_T * 4 * TL_Q;    // slots per tile
static_assert(TILE == (int)TILED_TILE, "tile size is part of the dispatch contract");
constexpr uint32_t TILED_MAX_TILES = 1u << 22;  // rows of more tiles (4G entries) cannot exist with 32-bit offsets

struct TiledRow {
  uint32_t v, off, d, base, lead, span, ntiles, tile0, bofs;  // tile0: first tile id; bofs: first slot of the row's BL/BH
  double scale, fs, inv_fs;
  uint64_t one, total_h;
  uint32_t ok, last_heavy;  // last_heavy: span index
};
struct TileTotals {
  uint64_t d, u;
  uint32_t first_heavy, last_heavy;  // span indices, NONE32 when the tile has no heavy
};

// Where a tile lies, one aligned record per tile: a tile's weights can be requested after one
// dependent load instead of two (tile -> row -> geometry).
struct __attribute__((aligned(32))) TileGeom {
  uint32_t row, T, base, lead, span, pad[3];  // row: index into the row array; T: tile number inside the row
};
__device__ __forceinline__ TiledRow geom_row(const TileGeom& tg, uint32_t tile) {
  TiledRow r = {};
  r.base = tg.base;
  r.lead = tg.lead;
  r.span = tg.span;
  r.tile0 = tile - tg.T;
  return r;
}

__device__ __forceinline__ Ledger row_ledger(const TiledRow& r) {
  Ledger L;
  L.scale = r.scale;
  L.fs = r.fs;
  L.inv_fs = r.inv_fs;
  L.one = r.one;
  return L;
}

// Weights of tile `t` of a row: quad q of thread tid covers span slots 4*(q*TL_T + tid) + t*TILE ...+3.
__device__ __forceinline__ void load_tile(const float* __restrict__ wgt, const TiledRow& r, uint32_t t, int tid,
                                          float (&w)[TL_Q][4]) {
#pragma unroll
  for (int q = 0; q < TL_Q; ++q) {
    const uint32_t pos = t * TILE + 4u * (q * TL_T + tid);
    float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
    if (pos < r.span) x = *reinterpret_cast<const float4*>(wgt + r.base + pos);
    const float xs[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t idx = pos + k;
      w[q][k] = idx - r.lead < r.span - r.lead ? clamp_weight(xs[k]) : 0.0f;
    }
  }
}
__device__ __forceinline__ bool in_row(const TiledRow& r, uint32_t idx) { return idx - r.lead < r.span - r.lead; }

// ---------------------------------------------------------------- row and tile bookkeeping
struct TiledCounters {
  unsigned long long next;  // low 32 bits: tiles handed out; high 32 bits: rows handed out
  uint32_t skipped;         // rows with more tiles than the path accepts (left to the streaming kernel)
  uint32_t pad;
};

// Geometry of every row; each block reserves a run of tile ids (and of prefix-array slots) for its
// rows with one atomic.  Tile numbering therefore depends on scheduling; no result does.
// `dev` (may be null): the counter block of a binning pass whose class sizes the host does not know.  The rows are
// then those of the classes cls .. cls + ncls - 1, which lie back to back in vlist after the rows of the classes
// before them; `count` is an upper bound, and the rows between the true number and the bound are recorded as rows
// without tiles, which every later kernel passes over.
__global__ __launch_bounds__(256) void tiled_rows_kernel(const RowRef* __restrict__ vlist, uint32_t count,
                                                         const uint32_t* __restrict__ dev, int cls, int ncls,
                                                         const uint32_t* __restrict__ xadj, uint32_t max_tiles,
                                                         TiledRow* __restrict__ rows,
                                                         TiledCounters* __restrict__ ctr) {
  __shared__ uint32_t s_w[4];
  __shared__ unsigned long long s_base;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const uint32_t r = blockIdx.x * 256u + tid;
  const uint32_t bound = count;
  if (dev) {
    uint32_t st = 0, n = 0;
    for (int c = 0; c < cls; ++c) st += dev[c];
    for (int c = cls; c < cls + ncls; ++c) n += dev[c];
    vlist += st;
    count = min(count, n);
  }
  TiledRow row = {};
  uint32_t nt = 0;
  bool skip = false;
  if (r < count) {
    row.v = vlist[r].v;
    row.off = xadj[row.v];
    row.d = xadj[row.v + 1] - row.off;
    row.base = row.off & ~3u;
    row.lead = row.off - row.base;
    row.span = row.lead + row.d;
    nt = (row.span + TILE - 1) / TILE;
    if (nt > max_tiles) {
      nt = 0;
      skip = true;
    }
    row.ntiles = nt;
  }
  const uint32_t inc = group_scan_u32<64>(nt);
  const uint32_t nskip = __popcll(__ballot(skip));
  if (lane == 63) s_w[wave] = inc;
  __syncthreads();
  uint32_t before = 0, total = 0;
  for (int k = 0; k < 4; ++k) {
    if (k == wave) before = total;
    total += s_w[k];
  }
  if (tid == 0) s_base = atomicAdd(&ctr->next, ((unsigned long long)256u << 32) | total);
  if (lane == 0 && nskip) atomicAdd(&ctr->skipped, nskip);
  __syncthreads();
  if (r < count) {
    row.tile0 = (uint32_t)s_base + before + inc - nt;
    row.bofs = row.tile0 + (uint32_t)(s_base >> 32) + tid;  // every row owns ntiles + 1 prefix slots
    rows[r] = row;
  } else if (r < bound) {
    rows[r] = row;  // no tiles
  }
}

__global__ __launch_bounds__(256) void tiled_map_kernel(const TiledRow* __restrict__ rows, uint32_t count,
                                                        TileGeom* __restrict__ geom) {
  const uint32_t r = blockIdx.x;
  if (r >= count) return;
  const TiledRow row = rows[r];
  for (uint32_t t = threadIdx.x; t < row.ntiles; t += 256)
    geom[row.tile0 + t] = TileGeom{r, t, row.base, row.lead, row.span, {0, 0, 0}};
}

// ---------------------------------------------------------------- pass 1: exact sums
__global__ __launch_bounds__(TL_T) void tiled_sum_kernel(const TileGeom* __restrict__ geom,
                                                         const float* __restrict__ wgt, u128* __restrict__ tsum) {
  __shared__ WSum3 s_w[TL_T / 64];
  const uint32_t tile = blockIdx.x;
  const TileGeom tg = geom[tile];
  if (tg.span == 0) return;  // the grid may be larger than the number of tiles
  const TiledRow r = geom_row(tg, tile);
  const int tid = threadIdx.x;
  float w[TL_Q][4];
  load_tile(wgt, r, tg.T, tid, w);
  WSum3 sum{0.0, 0.0, 0.0};  // exact: a tile adds at most 1024 limbs below 2^32 + 1
#pragma unroll
  for (int q = 0; q < TL_Q; ++q)
#pragma unroll
    for (int k = 0; k < 4; ++k) wsum3_add(sum, (double)w[q][k]);
  sum = group_sum_wsum3<64>(sum);
  if ((tid & 63) == 0) s_w[tid >> 6] = sum;
  __syncthreads();
  if (tid == 0) {
    WSum3 s = s_w[0];
    for (int i = 1; i < TL_T / 64; ++i) {
      s.top += s_w[i].top;
      s.mid += s_w[i].mid;
      s.low += s_w[i].low;
    }
    tsum[tile] = wsum3_to_u128(s);
  }
}

__global__ __launch_bounds__(64) void tiled_ledger_kernel(TiledRow* __restrict__ rows, uint32_t count,
                                                          const u128* __restrict__ tsum) {
  const uint32_t r = blockIdx.x;
  if (r >= count) return;
  const uint32_t t0 = rows[r].tile0, nt = rows[r].ntiles, d = rows[r].d;
  if (nt == 0) return;
  u128 sum{0, 0};
  for (uint32_t t = threadIdx.x; t < nt; t += 64) sum = add128(sum, tsum[t0 + t]);
  sum = group_sum_u128<64>(sum);
  if (threadIdx.x == 0) {
    const bool ok = (sum.lo | sum.hi) != 0;
    rows[r].ok = ok;
    if (ok) {
      const Ledger L = make_ledger(d, sum);
      rows[r].scale = L.scale;
      rows[r].fs = L.fs;
      rows[r].inv_fs = L.inv_fs;
      rows[r].one = L.one;
    }
  }
}

// ---------------------------------------------------------------- pass 2: tile totals
__global__ __launch_bounds__(TL_T) void tiled_totals_kernel(const TileGeom* __restrict__ geom,
                                                            const TiledRow* __restrict__ rows,
                                                            const float* __restrict__ wgt,
                                                            TileTotals* __restrict__ ttot) {
  __shared__ uint64_t s_d[TL_T / 64], s_u[TL_T / 64];
  __shared__ uint32_t s_f[TL_T / 64], s_l[TL_T / 64];
  const uint32_t tile = blockIdx.x;
  const TileGeom tg = geom[tile];
  if (tg.span == 0) return;
  const int tid = threadIdx.x;
  const uint32_t t = tg.T;
  float w[TL_Q][4];
  load_tile(wgt, geom_row(tg, tile), t, tid, w);  // requested before the row's ledger arrives
  const TiledRow r = rows[tg.row];
  if (!r.ok) return;
  const Ledger L = row_ledger(r);
  uint64_t sd = 0, su = 0;
  uint32_t fh = NONE32, lh = 0;  // lh holds idx + 1 so that 0 means none
#pragma unroll
  for (int q = 0; q < TL_Q; ++q)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t idx = t * TILE + 4u * (q * TL_T + tid) + k;
      if (!in_row(r, idx)) continue;
      const Entry e = classify_fast((double)w[q][k], true, L);
      if (e.heavy) {
        su += e.amount;
        fh = min(fh, idx);
        lh = max(lh, idx + 1);
      } else {
        sd += e.amount;
      }
    }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    sd += shfl_xor_u64(sd, m);
    su += shfl_xor_u64(su, m);
    fh = min(fh, (uint32_t)__shfl_xor((int)fh, m, 64));
    lh = max(lh, (uint32_t)__shfl_xor((int)lh, m, 64));
  }
  if ((tid & 63) == 0) {
    s_d[tid >> 6] = sd;
    s_u[tid >> 6] = su;
    s_f[tid >> 6] = fh;
    s_l[tid >> 6] = lh;
  }
  __syncthreads();
  if (tid == 0) {
    TileTotals o{0, 0, NONE32, 0};
    for (int i = 0; i < TL_T / 64; ++i) {
      o.d += s_d[i];
      o.u += s_u[i];
      o.first_heavy = min(o.first_heavy, s_f[i]);
      o.last_heavy = max(o.last_heavy, s_l[i]);
    }
    o.last_heavy = o.last_heavy ? o.last_heavy - 1 : NONE32;
    ttot[tile] = o;
  }
}

// first t in [0, nt) with B[t + 1] > key (nt if none)
__device__ __forceinline__ uint32_t first_tile_above(const uint64_t* B, uint32_t nt, uint64_t key) {
  return first_greater(B + 1, 0, nt, key);
}

// Per row: BL[t], BH[t] = deficits / surpluses before tile t (t = 0..ntiles, the last entry is the
// row total), stored at index tile0 + row + t; nfh[tile] = first heavy in any later tile.  One workgroup
// of 1024 threads per row: a row of a million entries has a thousand tiles, and one wavefront walking
// them 64 at a time with dependent loads was a sixth of a millisecond on the critical path.
constexpr int TS_T = 1024;
__global__ __launch_bounds__(TS_T) void tiled_scan_kernel(TiledRow* __restrict__ rows, uint32_t count,
                                                          const TileTotals* __restrict__ ttot,
                                                          uint64_t* __restrict__ BL, uint64_t* __restrict__ BH,
                                                          uint32_t* __restrict__ nfh, uint4* __restrict__ ranges) {
  constexpr int NW = TS_T / 64;
  __shared__ uint64_t s_wl[NW], s_wh[NW];
  __shared__ uint32_t s_wm[NW];
  const uint32_t r = blockIdx.x;
  if (r >= count) return;
  const uint32_t t0 = rows[r].tile0, nt = rows[r].ntiles;
  if (nt == 0 || !rows[r].ok) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t b0 = rows[r].bofs;
  uint64_t cl = 0, ch = 0;
  uint32_t last = NONE32;
  for (uint32_t c = 0; c < nt; c += TS_T) {
    const uint32_t t = c + tid;
    uint64_t d = 0, u = 0;
    uint32_t lh = 0;
    if (t < nt) {
      const TileTotals x = ttot[t0 + t];
      d = x.d;
      u = x.u;
      lh = x.last_heavy == NONE32 ? 0 : x.last_heavy + 1;
    }
    const uint64_t il = group_scan_u64<64>(d), ih = group_scan_u64<64>(u);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) lh = max(lh, (uint32_t)__shfl_xor((int)lh, m, 64));
    if (lane == 63) {
      s_wl[wave] = il;
      s_wh[wave] = ih;
      s_wm[wave] = lh;
    }
    __syncthreads();
    uint64_t bl = cl, bh = ch, tl = 0, th = 0;
    uint32_t lm = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      if (w == wave) {
        bl += tl;
        bh += th;
      }
      tl += s_wl[w];
      th += s_wh[w];
      lm = max(lm, s_wm[w]);
    }
    if (t < nt) {
      BL[b0 + t] = bl + il - d;
      BH[b0 + t] = bh + ih - u;
    }
    cl += tl;
    ch += th;
    if (lm) last = lm - 1;
    __syncthreads();  // the wavefront totals are rewritten by the next round
  }
  // next first heavy: the tiles backwards, exclusive suffix minimum of first_heavy
  uint32_t carry = NONE32;
  for (int32_t c = (int32_t)((nt - 1) / TS_T * TS_T); c >= 0; c -= TS_T) {
    const uint32_t t = (uint32_t)c + tid;
    const uint32_t fh = t < nt ? ttot[t0 + t].first_heavy : NONE32;
    uint32_t suf = fh;  // inclusive suffix minimum over the lanes of the wavefront
#pragma unroll
    for (int dlt = 1; dlt < 64; dlt <<= 1) {
      const uint32_t o = (uint32_t)__shfl_down((int)suf, dlt, 64);
      if (lane + dlt < 64) suf = min(suf, o);
    }
    uint32_t excl = (uint32_t)__shfl_down((int)suf, 1, 64);
    if (lane == 63) excl = NONE32;
    if (lane == 0) s_wm[wave] = suf;  // minimum of the wavefront
    __syncthreads();
    uint32_t later = carry, all = carry;  // minimum over the later wavefronts of this round and the later rounds
#pragma unroll
    for (int w = NW - 1; w >= 0; --w) {
      if (w == wave) later = all;
      all = min(all, s_wm[w]);
    }
    if (t < nt) nfh[t0 + t] = min(excl, later);
    carry = all;
    __syncthreads();
  }
  if (tid == 0) {
    BL[b0 + nt] = cl;
    BH[b0 + nt] = ch;
    rows[r].total_h = ch;
    rows[r].last_heavy = last;
  }
  // partner tiles of every tile: lights of tile t (keys in [BL[t], BL[t+1]]) meet the tiles whose surplus
  // range holds those keys; heavies (y in (BH[t], BH[t+1]]) the tiles whose deficit range holds y
  __threadfence_block();
  __syncthreads();
  const uint64_t* rl = BL + b0;
  const uint64_t* rh = BH + b0;
  for (uint32_t t = tid; t < nt; t += TS_T) {
    uint4 g;
    g.x = first_tile_above(rh, nt, rl[t]);
    g.y = min(first_tile_above(rh, nt, rl[t + 1]), nt - 1);
    if (rh[t + 1] != rh[t]) {
      g.z = first_tile_above(rl, nt, rh[t]);
      g.w = min(first_tile_above(rl, nt, rh[t + 1] - 1), nt - 1);
    } else {
      g.z = 1;
      g.w = 0;
    }
    ranges[t0 + t] = g;
  }
}

// ---------------------------------------------------------------- pass 3: every entry of a tile
// Resolves the own entries of one kind whose key lies in [lo, hi) against the per-slot prefix of tile
// `pt` held in smem[0..TILE).  OWN_HEAVY = false: lights, key = exclusive deficit prefix, prefix = surplus.
// OWN_HEAVY = true: heavies, key = y - 1, prefix = deficit.
template <bool OWN_HEAVY>
__device__ __forceinline__ void resolve_in_tile(const TiledRow& r, const Ledger& L, const uint64_t* smem, uint32_t pt,
                                                uint64_t lo, uint64_t hi, uint32_t heavy_mask, uint32_t live_mask,
                                                const uint32_t (&nh_after)[TL_Q], uint32_t T,
                                                const uint64_t (&key)[TL_Q][4], float (&op)[TL_Q][4],
                                                uint32_t (&oa)[TL_Q][4]) {
  const int tid = threadIdx.x;
#pragma unroll
  for (int q = 0; q < TL_Q; ++q) {
    uint32_t mine = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int b = q * 4 + k;
      const bool kind = ((live_mask >> b) & 1) && (((heavy_mask >> b) & 1) != 0) == OWN_HEAVY;
      if (kind && key[q][k] >= lo && key[q][k] < hi) mine |= 1u << k;
    }
    if (!mine) continue;
    const uint32_t base[4] = {0, 0, 0, 0};
    uint32_t pos[4];
    search4(smem, base, key[q], (uint32_t)TILE, pos);
    if (OWN_HEAVY) {
      // next heavy after each slot of the quad; the row's last heavy never retires
      uint32_t nxt = nh_after[q];
#pragma unroll
      for (int k = 3; k >= 0; --k) {
        if (((mine >> k) & 1) && nxt != NONE32) {
          op[q][k] = residual_prob(L.one + key[q][k] + 1 - smem[pos[k]], L);
          oa[q][k] = nxt - r.lead;
        }
        if ((heavy_mask >> (q * 4 + k)) & 1) nxt = T * TILE + 4u * (q * TL_T + tid) + k;
      }
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if ((mine >> k) & 1) oa[q][k] = pt * TILE + pos[k] - r.lead;
    }
  }
}

// One pass over the partner tiles of one kind other than the own tile T: their per-slot prefix is
// recomputed from the weights into LDS.
template <bool OWN_HEAVY>
__device__ __forceinline__ void partner_pass(const TiledRow& r, const Ledger& L, const float* __restrict__ wgt,
                                             const uint64_t* __restrict__ B, uint32_t t_lo, uint32_t t_hi,
                                             uint64_t* smem,
                                             uint64_t* s_ex, uint32_t heavy_mask, uint32_t live_mask,
                                             const uint32_t (&nh_after)[TL_Q], uint32_t T,
                                             const uint64_t (&key)[TL_Q][4], float (&op)[TL_Q][4],
                                             uint32_t (&oa)[TL_Q][4]) {
  const int tid = threadIdx.x;
  const uint32_t nt = r.ntiles;
  for (uint32_t pt = t_lo; pt <= t_hi && pt < nt; ++pt) {
    const uint64_t lo = B[pt], hi = B[pt + 1];
    if (hi == lo || pt == T) continue;
    float pw[TL_Q][4];
    load_tile(wgt, r, pt, tid, pw);
    uint64_t pv[TL_Q][4], ps[TL_Q][4];
#pragma unroll
    for (int q = 0; q < TL_Q; ++q)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t idx = pt * TILE + 4u * (q * TL_T + tid) + k;
        const Entry e = classify_fast((double)pw[q][k], in_row(r, idx), L);
        pv[q][k] = e.heavy != OWN_HEAVY ? e.amount : 0;
      }
    __syncthreads();  // searches of the previous partner are done: s_ex and the prefix may be overwritten
    block_scan1<TL_T, TL_Q>(pv, s_ex, lo, ps);
#pragma unroll
    for (int q = 0; q < TL_Q; ++q)
#pragma unroll
      for (int k = 0; k < 4; ++k) smem[4u * (q * TL_T + tid) + k] = ps[q][k];
    __syncthreads();
    resolve_in_tile<OWN_HEAVY>(r, L, smem, pt, lo, hi, heavy_mask, live_mask, nh_after, T, key, op, oa);
  }
}

__global__ __launch_bounds__(TL_T) void tiled_emit_kernel(const TileGeom* __restrict__ geom,
                                                          const TiledRow* __restrict__ rows,
                                                          const float* __restrict__ wgt,
                                                          const uint64_t* __restrict__ gBL,
                                                          const uint64_t* __restrict__ gBH,
                                                          const uint32_t* __restrict__ nfh,
                                                          const uint4* __restrict__ ranges,
                                                          AliasEntry* __restrict__ table,
                                                          int8_t* __restrict__ valid) {
  constexpr int NW = TL_T / 64;
  __shared__ uint64_t smem[TILE];      // per-slot prefix of the current partner tile
  __shared__ uint64_t s_ex[2 * TL_Q * NW];
  __shared__ uint32_t s_fh[TL_Q][NW];
  const uint32_t tile = blockIdx.x;
  const TileGeom tg = geom[tile];
  if (tg.span == 0) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const uint32_t T = tg.T;

  float w[TL_Q][4];
  load_tile(wgt, geom_row(tg, tile), T, tid, w);  // requested before the row record arrives
  const TiledRow r = rows[tg.row];
  if (!r.ok) {
#pragma unroll
    for (int q = 0; q < TL_Q; ++q)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t idx = T * TILE + 4u * (q * TL_T + tid) + k;
        if (in_row(r, idx)) {
          table[r.base + idx] = AliasEntry{0.0f, SKY_INVALID};
        }
      }
    if (T == 0 && tid == 0) valid[r.v] = 0;
    return;
  }
  const Ledger L = row_ledger(r);
  const uint64_t* BL = gBL + r.bofs;  // tile prefixes of this row
  const uint64_t* BH = gBH + r.bofs;
  const uint64_t bl = BL[T], bl1 = BL[T + 1], bh = BH[T], bh1 = BH[T + 1];
  const uint4 rg = ranges[tile];

  // own tile: class and amount of every slot, both prefixes, search key of the own kind
  uint64_t key[TL_Q][4], sl[TL_Q][4], sh[TL_Q][4];
  float op[TL_Q][4];
  uint32_t oa[TL_Q][4];
  uint32_t heavy_mask = 0, live_mask = 0;
  uint64_t hb_mask[TL_Q];
  {
    uint64_t dl[TL_Q][4], dh[TL_Q][4];
#pragma unroll
    for (int q = 0; q < TL_Q; ++q) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t idx = T * TILE + 4u * (q * TL_T + tid) + k;
        const bool in = in_row(r, idx);
        const Entry e = classify_fast((double)w[q][k], in, L);
        dl[q][k] = e.heavy ? 0 : e.amount;
        dh[q][k] = e.heavy ? e.amount : 0;
        op[q][k] = e.heavy ? 1.0f : (float)e.p;
        if (in) live_mask |= 1u << (q * 4 + k);
        if (e.heavy) heavy_mask |= 1u << (q * 4 + k);
      }
      const uint32_t m = (heavy_mask >> (q * 4)) & 15u;
      const uint64_t bal = __ballot(m != 0);
      hb_mask[q] = bal;
      uint32_t fh = NONE32;
      if (bal) {
        const int l0 = __ffsll((unsigned long long)bal) - 1;
        const uint32_t m0 = (uint32_t)__builtin_amdgcn_readlane((int)m, l0);
        fh = T * TILE + 4u * (q * TL_T + wave * 64 + l0) + (uint32_t)(__ffs((int)m0) - 1);
      }
      if (lane == 0) s_fh[q][wave] = fh;
    }
    uint64_t tl, th;
    block_scan2<TL_T, TL_Q>(dl, dh, s_ex, sl, sh, tl, th);  // its barrier also publishes s_fh
#pragma unroll
    for (int q = 0; q < TL_Q; ++q)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        sl[q][k] += bl;
        sh[q][k] += bh;
        key[q][k] = ((heavy_mask >> (q * 4 + k)) & 1) ? sh[q][k] - 1 : sl[q][k] - dl[q][k];
      }
  }
  // next heavy after each quad (span index): later lanes, later waves, later sub-tiles, later tiles
  uint32_t nh_after[TL_Q];
  {
    const uint32_t later_tiles = nfh[tile];
#pragma unroll
    for (int q = 0; q < TL_Q; ++q) {
      const uint32_t m = (heavy_mask >> (q * 4)) & 15u;
      const uint64_t above = hb_mask[q] & ~((2ull << lane) - 1);
      const int ln = above ? __ffsll((unsigned long long)above) - 1 : lane;
      const uint32_t mn = (uint32_t)__shfl((int)m, ln, 64);
      uint32_t nx = above ? T * TILE + 4u * (q * TL_T + wave * 64 + ln) + (uint32_t)(__ffs((int)mn) - 1) : later_tiles;
#pragma unroll
      for (int wv = 0; wv < NW; ++wv) {
        if (wv > wave) nx = min(nx, s_fh[q][wv]);
#pragma unroll
        for (int q2 = q + 1; q2 < TL_Q; ++q2) nx = min(nx, s_fh[q2][wv]);
      }
      nh_after[q] = nx;
    }
  }
  // defaults: a light without donor takes the last heavy (itself if the row has none);
  // a heavy that is last, or that no light retires, keeps {1, itself}
#pragma unroll
  for (int q = 0; q < TL_Q; ++q)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t idx = T * TILE + 4u * (q * TL_T + tid) + k;
      const bool heavy = (heavy_mask >> (q * 4 + k)) & 1;
      oa[q][k] = (!heavy && r.total_h) ? r.last_heavy - r.lead : idx - r.lead;
    }
  // the own tile is usually its own main partner, and its prefixes are already in registers
#pragma unroll
  for (int q = 0; q < TL_Q; ++q)
#pragma unroll
    for (int k = 0; k < 4; ++k) smem[4u * (q * TL_T + tid) + k] = sh[q][k];
  __syncthreads();
  resolve_in_tile<false>(r, L, smem, T, bh, bh1, heavy_mask, live_mask, nh_after, T, key, op, oa);
  __syncthreads();
#pragma unroll
  for (int q = 0; q < TL_Q; ++q)
#pragma unroll
    for (int k = 0; k < 4; ++k) smem[4u * (q * TL_T + tid) + k] = sl[q][k];
  __syncthreads();
  resolve_in_tile<true>(r, L, smem, T, bl, bl1, heavy_mask, live_mask, nh_after, T, key, op, oa);

  // the other partner tiles (ranges precomputed per tile by tiled_scan_kernel)
  partner_pass<false>(r, L, wgt, BH, rg.x, rg.y, smem, s_ex, heavy_mask, live_mask, nh_after, T, key, op, oa);
  partner_pass<true>(r, L, wgt, BL, rg.z, rg.w, smem, s_ex, heavy_mask, live_mask, nh_after, T, key, op, oa);

#pragma unroll
  for (int q = 0; q < TL_Q; ++q) {
    const uint32_t pos = T * TILE + 4u * (q * TL_T + tid);
    if (pos >= r.span) continue;
    if (pos >= r.lead && pos + 4 <= r.span) {
      store_entries4(table + r.base + pos, op[q], oa[q]);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (in_row(r, pos + k)) {
          table[r.base + pos + k] = AliasEntry{op[q][k], oa[q][k]};
        }
    }
  }
}

// ---------------------------------------------------------------- host driver
namespace {
struct TiledScratch {
  TiledRow* rows = nullptr;
  TiledCounters* totals = nullptr;
  TileGeom* geom = nullptr;
  u128* tsum = nullptr;
  TileTotals* ttot = nullptr;
  uint64_t *BL = nullptr, *BH = nullptr;
  uint32_t* nfh = nullptr;
  uint4* ranges = nullptr;
  uint32_t row_cap = 0, tile_cap = 0;
  size_t b_cap = 0;  // entries of BL and BH
};
TiledScratch& tiled_of(sky_graph* g) {
  if (!g->tiled_scratch) g->tiled_scratch = new TiledScratch();
  return *static_cast<TiledScratch*>(g->tiled_scratch);
}
}  // namespace

void free_tiled_scratch(sky_graph* g) {
  if (!g->tiled_scratch) return;
  TiledScratch* sc = static_cast<TiledScratch*>(g->tiled_scratch);
  void* ptrs[] = {sc->rows, sc->totals, sc->geom, sc->tsum, sc->ttot, sc->BL, sc->BH, sc->nfh, sc->ranges};
  for (void* p : ptrs)
    if (p) (void)hipFree(p);
  delete sc;
  g->tiled_scratch = nullptr;
}

uint32_t tiled_max_tiles(const sky_graph* g) {
  const long long n = option(g, OPT_TILED_MAX_TILES);
  return (uint32_t)std::min<long long>(std::max<long long>(n, 1), TILED_MAX_TILES);
}

// Builds the rows of `rows_list` (device, n entries) that have at most the configured number of
// tiles; *skipped receives how many rows were left for the streaming kernel.  `edges` is the number of
// entries of the listed rows when the caller knows it (0 otherwise): the tile grids are then sized by
// the bound edges / TILE + 2 n, with empty records for the tiles that do not exist, and the host does
// not wait for the device to count them.
// dev non-null: see tiled_rows_kernel; n and edges are then upper bounds, and the call never waits for the device.
static int build_rows_tiled_any(sky_graph* g, const RowRef* rows_list, uint32_t n, const uint32_t* dev, int cls, int ncls,
                                uint32_t* skipped, EventTimer* tm, uint64_t edges) {
  hipStream_t st = g->stream;
  TiledScratch& sc = tiled_of(g);
  const uint32_t max_tiles = tiled_max_tiles(g);
  *skipped = 0;
  if (n == 0) return SKY_OK;
  if (sc.row_cap < n) {
    if (sc.rows) SKY_HIP(hipFree(sc.rows));
    sc.rows = nullptr;
    sc.row_cap = 0;
    SKY_HIP(hipMalloc((void**)&sc.rows, (size_t)n * sizeof(TiledRow)));
    sc.row_cap = n;
  }
  if (!sc.totals) SKY_HIP(hipMalloc((void**)&sc.totals, sizeof(TiledCounters)));
  SKY_HIP(hipMemsetAsync(sc.totals, 0, sizeof(TiledCounters), st));
  hipLaunchKernelGGL(tiled_rows_kernel, dim3((n + 255) / 256), dim3(256), 0, st, rows_list, n, dev, cls, ncls, g->xadj,
                     max_tiles, sc.rows, sc.totals);
  const bool bounded = edges != 0 && max_tiles == TILED_MAX_TILES && edges / TILE + 2ull * n < (1ull << 31);
  uint32_t ntiles, nslots;
  if (bounded) {
    ntiles = (uint32_t)(edges / TILE + 2ull * n);
    nslots = 256u * ((n + 255) / 256);
  } else {
    TiledCounters totals = {};
    SKY_HIP(hipMemcpyAsync(&totals, sc.totals, sizeof(totals), hipMemcpyDeviceToHost, st));
    SKY_HIP(hipStreamSynchronize(st));
    ntiles = (uint32_t)totals.next;
    nslots = (uint32_t)(totals.next >> 32);  // 256 per block of rows
    *skipped = totals.skipped;
  }
  if (ntiles == 0) return SKY_OK;
  if (sc.tile_cap < ntiles) {
    void* olds[] = {sc.geom, sc.tsum, sc.ttot, sc.nfh, sc.ranges};
    for (void* p : olds)
      if (p) SKY_HIP(hipFree(p));
    sc.geom = nullptr; sc.tsum = nullptr; sc.ttot = nullptr; sc.nfh = nullptr; sc.ranges = nullptr;
    sc.tile_cap = 0;
    const size_t cap = (size_t)ntiles + ntiles / 4 + 1024;
    SKY_HIP(hipMalloc((void**)&sc.geom, cap * sizeof(TileGeom)));
    SKY_HIP(hipMalloc((void**)&sc.tsum, cap * sizeof(u128)));
    SKY_HIP(hipMalloc((void**)&sc.ttot, cap * sizeof(TileTotals)));
    SKY_HIP(hipMalloc((void**)&sc.nfh, cap * 4));
    SKY_HIP(hipMalloc((void**)&sc.ranges, cap * sizeof(uint4)));
    sc.tile_cap = (uint32_t)cap;
  }
  // prefix arrays hold ntiles + one extra entry per row
  const size_t b_need = (size_t)ntiles + nslots;
  if (sc.b_cap < b_need) {
    if (sc.BL) SKY_HIP(hipFree(sc.BL));
    if (sc.BH) SKY_HIP(hipFree(sc.BH));
    sc.BL = sc.BH = nullptr;
    sc.b_cap = 0;
    SKY_HIP(hipMalloc((void**)&sc.BL, (b_need + b_need / 4 + 1024) * 8));
    SKY_HIP(hipMalloc((void**)&sc.BH, (b_need + b_need / 4 + 1024) * 8));
    sc.b_cap = b_need + b_need / 4 + 1024;
  }
  if (bounded) SKY_HIP(hipMemsetAsync(sc.geom, 0, (size_t)ntiles * sizeof(TileGeom), st));  // span 0: no such tile
  hipLaunchKernelGGL(tiled_map_kernel, dim3(n), dim3(256), 0, st, sc.rows, n, sc.geom);
  if (tm) SKY_TRY(tm->mark("tiled_rows", 0));
  hipLaunchKernelGGL(tiled_sum_kernel, dim3(ntiles), dim3(TL_T), 0, st, sc.geom, g->adjwgt, sc.tsum);
  if (tm) SKY_TRY(tm->mark("tiled_sum", edges));
  hipLaunchKernelGGL(tiled_ledger_kernel, dim3(n), dim3(64), 0, st, sc.rows, n, sc.tsum);
  hipLaunchKernelGGL(tiled_totals_kernel, dim3(ntiles), dim3(TL_T), 0, st, sc.geom, sc.rows, g->adjwgt, sc.ttot);
  if (tm) SKY_TRY(tm->mark("tiled_totals", edges));
  hipLaunchKernelGGL(tiled_scan_kernel, dim3(n), dim3(TS_T), 0, st, sc.rows, n, sc.ttot, sc.BL, sc.BH, sc.nfh, sc.ranges);
  hipLaunchKernelGGL(tiled_emit_kernel, dim3(ntiles), dim3(TL_T), 0, st, sc.geom, sc.rows, g->adjwgt, sc.BL,
                     sc.BH, sc.nfh, sc.ranges, g->table, g->valid);
  if (tm) SKY_TRY(tm->mark("tiled_emit", edges));
  return SKY_OK;
}

int build_rows_tiled(sky_graph* g, const RowRef* rows_list, uint32_t n, uint32_t* skipped, EventTimer* tm,
                     uint64_t edges) {
  return build_rows_tiled_any(g, rows_list, n, nullptr, 0, 0, skipped, tm, edges);
}

int build_rows_tiled_dev(sky_graph* g, const RowRef* vlist, const uint32_t* dev, int cls, int ncls, uint32_t n_upper,
                         uint64_t edges_upper) {
  if (tiled_max_tiles(g) != TILED_MAX_TILES || edges_upper == 0 || edges_upper / TILE + 2ull * n_upper >= (1ull << 31))
    return fail(SKY_ERR_STATE, "build_rows_tiled_dev: the number of tiles has no usable bound");
  uint32_t skipped = 0;
  return build_rows_tiled_any(g, vlist, n_upper, dev, cls, ncls, &skipped, nullptr, edges_upper);
}

}  // namespace sky
