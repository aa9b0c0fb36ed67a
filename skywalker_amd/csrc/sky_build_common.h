// Block-level building blocks shared by the alias-build kernels: prefix sums over a tile held as
// [Q][4] slots per thread, and interleaved binary searches over prefix arrays kept in LDS.
#pragma once
#include "sky_common.h"

namespace sky {

constexpr uint32_t NONE32 = 0xFFFFFFFFu;

// Inclusive prefixes of two quantities over the slots of a tile held as [Q][4] per thread (slot order:
// quad q of thread tid, then thread tid + 1; sub-tile q before q + 1).  One barrier.
// Bit q of `wave_live` (wave-uniform) clear means every value of this wave in sub-tile q is zero:
// the wave then skips that sub-tile's scan.
template <int ROWT, int Q>
__device__ __forceinline__ void block_scan2(const uint64_t (&a)[Q][4], const uint64_t (&b)[Q][4],
                                            uint64_t* __restrict__ s_ex /* [2 * Q * ROWT/64] */,
                                            uint64_t (&oa)[Q][4], uint64_t (&ob)[Q][4], uint64_t& tot_a,
                                            uint64_t& tot_b, uint32_t wave_live = 0xFFFFFFFFu) {
  constexpr int NW = ROWT / 64;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  uint64_t ia[Q], ib[Q];
#pragma unroll
  for (int q = 0; q < Q; ++q) {
    if (!((wave_live >> q) & 1)) {
#pragma unroll
      for (int k = 0; k < 4; ++k) oa[q][k] = ob[q][k] = 0;
      ia[q] = ib[q] = 0;
      if (lane == 63) s_ex[(q * NW + wave) * 2] = s_ex[(q * NW + wave) * 2 + 1] = 0;
      continue;
    }
    uint64_t ra = 0, rb = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      ra += a[q][k];
      rb += b[q][k];
      oa[q][k] = ra;
      ob[q][k] = rb;
    }
    ia[q] = group_scan_u64<64>(ra);
    ib[q] = group_scan_u64<64>(rb);
    if (lane == 63) {
      s_ex[(q * NW + wave) * 2] = ia[q];
      s_ex[(q * NW + wave) * 2 + 1] = ib[q];
    }
    ia[q] -= ra;  // exclusive over the lanes of this wave
    ib[q] -= rb;
  }
  __syncthreads();
  uint64_t run_a = 0, run_b = 0;
#pragma unroll
  for (int q = 0; q < Q; ++q) {
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      if (w == wave) {
        ia[q] += run_a;
        ib[q] += run_b;
      }
      run_a += s_ex[(q * NW + w) * 2];
      run_b += s_ex[(q * NW + w) * 2 + 1];
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      oa[q][k] += ia[q];
      ob[q][k] += ib[q];
    }
  }
  tot_a = run_a;
  tot_b = run_b;
}

// Inclusive prefixes of two quantities over PER consecutive slots per thread (thread tid owns slots
// PER * tid ..).  One barrier.  Waves whose `wave_on` is false hold zeros only and skip their scan.
template <int ROWT, int PER>
__device__ __forceinline__ void block_scan2_flat(const uint64_t (&a)[PER], const uint64_t (&b)[PER],
                                                 uint64_t* __restrict__ s_ex /* [2 * ROWT/64] */,
                                                 uint64_t (&oa)[PER], uint64_t (&ob)[PER], uint64_t& tot_a,
                                                 uint64_t& tot_b, bool wave_on) {
  constexpr int NW = ROWT / 64;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  uint64_t ia = 0, ib = 0;
  if (wave_on) {
    uint64_t ra = 0, rb = 0;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      ra += a[k];
      rb += b[k];
      oa[k] = ra;
      ob[k] = rb;
    }
    ia = group_scan_u64<64>(ra);
    ib = group_scan_u64<64>(rb);
    if (NW > 1 && lane == 63) {
      s_ex[wave * 2] = ia;
      s_ex[wave * 2 + 1] = ib;
    }
    if (NW == 1) {
      tot_a = shfl_u64(ia, 63);
      tot_b = shfl_u64(ib, 63);
    }
    ia -= ra;
    ib -= rb;
  } else {
#pragma unroll
    for (int k = 0; k < PER; ++k) oa[k] = ob[k] = 0;
    if (NW > 1 && lane == 63) s_ex[wave * 2] = s_ex[wave * 2 + 1] = 0;
    if (NW == 1) tot_a = tot_b = 0;
  }
  if (NW > 1) {
    __syncthreads();
    uint64_t run_a = 0, run_b = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      if (w == wave) {
        ia += run_a;
        ib += run_b;
      }
      run_a += s_ex[w * 2];
      run_b += s_ex[w * 2 + 1];
    }
    tot_a = run_a;
    tot_b = run_b;
  }
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    oa[k] += ia;
    ob[k] += ib;
  }
}

// block_scan2_flat plus an exclusive prefix (and total) of one 32-bit count per thread, same barrier.
template <int ROWT, int PER>
__device__ __forceinline__ void block_scan2c_flat(const uint64_t (&a)[PER], const uint64_t (&b)[PER], uint32_t c,
                                                  uint64_t* __restrict__ s_ex /* [3 * ROWT/64] */,
                                                  uint64_t (&oa)[PER], uint64_t (&ob)[PER], uint32_t& ex_c,
                                                  uint64_t& tot_a, uint64_t& tot_b, uint32_t& tot_c, bool wave_on) {
  constexpr int NW = ROWT / 64;
  static_assert(NW > 1, "multi-wave rows only");
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  uint64_t ia = 0, ib = 0;
  uint32_t ic = 0;
  if (wave_on) {
    uint64_t ra = 0, rb = 0;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      ra += a[k];
      rb += b[k];
      oa[k] = ra;
      ob[k] = rb;
    }
    ia = group_scan_u64<64>(ra);
    ib = group_scan_u64<64>(rb);
    ic = group_scan_u32<64>(c);
    if (lane == 63) {
      s_ex[wave * 3] = ia;
      s_ex[wave * 3 + 1] = ib;
      s_ex[wave * 3 + 2] = ic;
    }
    ia -= ra;
    ib -= rb;
    ic -= c;
  } else {
#pragma unroll
    for (int k = 0; k < PER; ++k) oa[k] = ob[k] = 0;
    if (lane == 63) s_ex[wave * 3] = s_ex[wave * 3 + 1] = s_ex[wave * 3 + 2] = 0;
  }
  __syncthreads();
  uint64_t run_a = 0, run_b = 0;
  uint32_t run_c = 0;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    if (w == wave) {
      ia += run_a;
      ib += run_b;
      ic += run_c;
    }
    run_a += s_ex[w * 3];
    run_b += s_ex[w * 3 + 1];
    run_c += (uint32_t)s_ex[w * 3 + 2];
  }
  tot_a = run_a;
  tot_b = run_b;
  tot_c = run_c;
  ex_c = ic;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    oa[k] += ia;
    ob[k] += ib;
  }
}

// For four keys at once: number of entries of the sorted array that starts `base_k` bytes into the LDS
// block `s` and has n >= 1 entries that are <= key_k.  The first probe narrows the answer to a window
// of hb = 2^floor(log2 n) entries that ends inside the array, so no later probe needs a bound check.
// Everything is kept as 32-bit byte offsets from `s` so that the probes stay LDS reads.
__device__ __forceinline__ uint64_t lds_u64(const uint64_t* s, uint32_t byte_off) {
  return *reinterpret_cast<const uint64_t*>(reinterpret_cast<const char*>(s) + byte_off);
}
__device__ __forceinline__ void search4(const uint64_t* s, const uint32_t (&base)[4], const uint64_t (&key)[4],
                                        uint32_t n, uint32_t (&pos)[4]) {
  const uint32_t hb = 1u << (31 - __clz((int)n));
  uint32_t cur[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) cur[k] = base[k] + (lds_u64(s, base[k] + (hb - 1) * 8u) <= key[k] ? (n - hb) * 8u : 0u);
  for (uint32_t step = hb * 4u; step >= 8u; step >>= 1) {  // step in bytes: hb/2 entries first
    uint64_t v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = lds_u64(s, cur[k] + step - 8u);
#pragma unroll
    for (int k = 0; k < 4; ++k) cur[k] = v[k] <= key[k] ? cur[k] + step : cur[k];
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) pos[k] = (cur[k] - base[k]) / 8u + (lds_u64(s, cur[k]) <= key[k] ? 1u : 0u);
}


// Single-quantity form of block_scan2.
template <int ROWT, int Q>
__device__ __forceinline__ void block_scan1(const uint64_t (&a)[Q][4], uint64_t* __restrict__ s_ex /* [Q * ROWT/64] */,
                                            uint64_t base, uint64_t (&oa)[Q][4]) {
  constexpr int NW = ROWT / 64;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  uint64_t ia[Q];
#pragma unroll
  for (int q = 0; q < Q; ++q) {
    uint64_t ra = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      ra += a[q][k];
      oa[q][k] = ra;
    }
    ia[q] = group_scan_u64<64>(ra);
    if (lane == 63) s_ex[q * NW + wave] = ia[q];
    ia[q] -= ra;
  }
  __syncthreads();
  uint64_t run = base;
#pragma unroll
  for (int q = 0; q < Q; ++q) {
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      if (w == wave) ia[q] += run;
      run += s_ex[q * NW + w];
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) oa[q][k] += ia[q];
  }
}

}  // namespace sky
