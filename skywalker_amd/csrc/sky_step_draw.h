// The draw of one (walker, step) from a table that is never built: only entry `col` of the step's table is ever
// read, so one workgroup evaluates that entry alone, from the same prefix-sum definition the offline build uses:
//   pass 1  exact sum of the row's weights -> ledger, class of entry col
//           (a light col whose own share accepts the draw needs nothing more)
//   pass 2  prefix of deficits (or surpluses) up to col
//   pass 3  first slot whose running prefix crosses it (and the last / next heavy)
// The result is bit for bit the draw from the fully built table.  The row's weights come from a functor, so the
// same code serves node2vec's second-order weights and the weights of a bias operator linked in from outside.
#pragma once
#include "sky_common.h"

namespace sky {

constexpr int N2V_T = 256;
constexpr uint32_t N2V_CACHE = 4096;  // second-order weights of rows up to this degree stay in LDS between passes

__device__ __forceinline__ bool row_contains(const uint32_t* __restrict__ row, uint32_t n, uint32_t key) {
  uint32_t lo = 0, len = n;
  while (len > 0) {
    const uint32_t half = len >> 1;
    const uint32_t x = row[lo + half];
    if (x == key) return true;
    if (x < key) {
      lo += half + 1;
      len -= half + 1;
    } else {
      len = half;
    }
  }
  return false;
}

template <class T>
__device__ __forceinline__ T block_bcast_min(T v, T* s_tmp) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    const T o = (T)shfl_xor_u64((uint64_t)v, m);
    v = o < v ? o : v;
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) s_tmp[threadIdx.x >> 6] = v;
  __syncthreads();
  T r = s_tmp[0];
  for (int i = 1; i < N2V_T / 64; ++i) r = s_tmp[i] < r ? s_tmp[i] : r;
  return r;
}
__device__ __forceinline__ uint64_t block_bcast_sum(uint64_t v, uint64_t* s_tmp) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += shfl_xor_u64(v, m);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) s_tmp[threadIdx.x >> 6] = v;
  __syncthreads();
  uint64_t r = 0;
  for (int i = 0; i < N2V_T / 64; ++i) r += s_tmp[i];
  return r;
}


constexpr uint32_t NONE_SLOT = 0xFFFFFFFFu;

// Row-local slot that (walker, step) with random numbers r draws from the row of d >= 1 entries whose clamped
// weights are row(0..d-1), or NONE_SLOT when they sum to zero.  Called by every thread of a workgroup of N2V_T.
template <class RowFn>
__device__ uint32_t step_draw_slot(const RowFn& row, uint32_t d, const u32x4& r) {
  __shared__ float s_w[N2V_CACHE];
  __shared__ uint64_t s_tmp[N2V_T / 64];
  __shared__ u128 s_sum[N2V_T / 64];
  const int tid = threadIdx.x;
  const bool cached = d <= N2V_CACHE;
  auto weight = [&](uint32_t k) -> float { return cached ? s_w[k] : row(k); };

  // pass 1: exact total
  u128 sum{0, 0};
  for (uint32_t k = tid; k < d; k += N2V_T) {
    const float x = row(k);
    if (cached) s_w[k] = x;
    sum = add128(sum, weight_fixed(x));
  }
  sum = group_sum_u128<64>(sum);
  if ((tid & 63) == 0) s_sum[tid >> 6] = sum;
  __syncthreads();
  sum = s_sum[0];
  for (int k = 1; k < N2V_T / 64; ++k) sum = add128(sum, s_sum[k]);
  if ((sum.lo | sum.hi) == 0) return NONE_SLOT;
  const Ledger L = make_ledger(d, sum);
  const uint32_t col = __umulhi(r.x, d);
  const float u = u24(r.y);
  const Entry ec = classify(weight(col), L);
  if (!ec.heavy && u < (float)ec.p) return col;  // the light keeps the draw: its alias is never read

  // pass 2: prefix up to col of the amounts of col's own kind (exclusive for a light, inclusive for a heavy)
  uint64_t part = 0;
  const uint32_t upto = ec.heavy ? col + 1 : col;
  for (uint32_t k = tid; k < upto; k += N2V_T) {
    const Entry e = classify(weight(k), L);
    if (e.heavy == ec.heavy) part += e.amount;
  }
  const uint64_t key = block_bcast_sum(part, s_tmp);  // x of a light, y of a heavy

  // pass 3: running prefix of the other kind until it crosses the key
  uint32_t cand;
  if (!ec.heavy) {
    // first heavy m with SH(m) > x; the last heavy if none; col itself if the row has no heavy
    uint64_t carry = 0;
    uint32_t found = 0xFFFFFFFFu, last_heavy = 0xFFFFFFFFu;
    for (uint32_t base = 0; base < d && found == 0xFFFFFFFFu; base += N2V_T) {
      const uint32_t k = base + tid;
      uint64_t amt = 0;
      bool heavy = false;
      if (k < d) {
        const Entry e = classify(weight(k), L);
        heavy = e.heavy;
        amt = heavy ? e.amount : 0;
      }
      const uint64_t inc = group_scan_u64<64>(amt);
      __syncthreads();
      if ((tid & 63) == 63) s_tmp[tid >> 6] = inc;
      __syncthreads();
      uint64_t before = carry, total = 0;
      for (int wv = 0; wv < N2V_T / 64; ++wv) {
        if (wv == (tid >> 6)) before += total;
        total += s_tmp[wv];
      }
      const uint32_t hit = (heavy && before + inc > key) ? k : 0xFFFFFFFFu;
      const uint32_t lh = heavy ? ~k : 0xFFFFFFFFu;  // min of ~k = max of k
      found = block_bcast_min<uint32_t>(hit, reinterpret_cast<uint32_t*>(s_tmp));
      const uint32_t lhm = block_bcast_min<uint32_t>(lh, reinterpret_cast<uint32_t*>(s_tmp));
      if (lhm != 0xFFFFFFFFu) last_heavy = ~lhm;
      carry += total;
    }
    cand = found != 0xFFFFFFFFu ? found : (last_heavy != 0xFFFFFFFFu ? last_heavy : col);
  } else {
    // next heavy after col (none: col is the last heavy and keeps the draw), then the first light l
    // with SL(l) >= y: prob = (one + y - SL(l)) / one
    uint32_t nxt = 0xFFFFFFFFu;
    for (uint32_t base = col + 1; base < d && nxt == 0xFFFFFFFFu; base += N2V_T) {
      const uint32_t k = base + tid;
      uint32_t hit = 0xFFFFFFFFu;
      if (k < d && classify(weight(k), L).heavy) hit = k;
      nxt = block_bcast_min<uint32_t>(hit, reinterpret_cast<uint32_t*>(s_tmp));
    }
    cand = col;
    if (nxt != 0xFFFFFFFFu) {
      uint64_t carry = 0, best = ~0ull;  // best = (index << 0) encoded below
      uint32_t li = 0xFFFFFFFFu;
      uint64_t sl_at = 0;
      for (uint32_t base = 0; base < d && li == 0xFFFFFFFFu; base += N2V_T) {
        const uint32_t k = base + tid;
        uint64_t amt = 0;
        bool light = false;
        if (k < d) {
          const Entry e = classify(weight(k), L);
          light = !e.heavy;
          amt = light ? e.amount : 0;
        }
        const uint64_t inc = group_scan_u64<64>(amt);
        __syncthreads();
        if ((tid & 63) == 63) s_tmp[tid >> 6] = inc;
        __syncthreads();
        uint64_t before = carry, total = 0;
        for (int wv = 0; wv < N2V_T / 64; ++wv) {
          if (wv == (tid >> 6)) before += total;
          total += s_tmp[wv];
        }
        const uint64_t mine = before + inc;
        const uint32_t hit = (light && mine >= key) ? k : 0xFFFFFFFFu;
        li = block_bcast_min<uint32_t>(hit, reinterpret_cast<uint32_t*>(s_tmp));
        if (li != 0xFFFFFFFFu) {
          // the owner of slot li publishes its prefix
          __syncthreads();
          if (k == li) s_tmp[0] = mine;
          __syncthreads();
          sl_at = s_tmp[0];
        }
        carry += total;
      }
      (void)best;
      if (li != 0xFFFFFFFFu) {
        const float pr = residual_prob(L.one + key - sl_at, L);
        cand = u < pr ? col : nxt;
      }
    }
  }
  return cand;
}


}  // namespace sky
