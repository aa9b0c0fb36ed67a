// Shared device/host helpers of libskywalker_hip (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

#include "../../include/skywalker_hip.h"

namespace sky {

// ---------------------------------------------------------------- error plumbing
void set_error(const std::string& msg);
int fail(int code, const std::string& msg);

#define SKY_HIP(expr)                                                                                 \
  do {                                                                                                \
    hipError_t _e = (expr);                                                                           \
    if (_e != hipSuccess)                                                                             \
      return ::sky::fail(SKY_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(_e) + " (" +      \
                                          __FILE__ + ":" + std::to_string(__LINE__) + ")");           \
  } while (0)

#define SKY_TRY(expr)         \
  do {                        \
    int _rc = (expr);         \
    if (_rc != SKY_OK) return _rc; \
  } while (0)

// ---------------------------------------------------------------- Philox4x32-10
// Counter = (a, b, c, domain), key = 64-bit seed.  Domains separate the streams of
// the generators and of the samplers so that no two consumers share a counter.
enum : uint32_t { DOM_RMAT = 1, DOM_WEIGHT = 2, DOM_SEEDS = 3, DOM_WALK = 4, DOM_SAMPLE = 5 };

struct u32x4 {
  uint32_t x, y, z, w;
};

__device__ __forceinline__ u32x4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                               uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    c0 = hi1 ^ c1 ^ k0;
    c1 = lo1;
    c2 = hi0 ^ c3 ^ k1;
    c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return u32x4{c0, c1, c2, c3};
}
__device__ __forceinline__ u32x4 philox(uint64_t seed, uint32_t a, uint32_t b, uint32_t c, uint32_t dom) {
  return philox4x32_10(a, b, c, dom, (uint32_t)seed, (uint32_t)(seed >> 32));
}
// 24-bit uniform in [0,1): every value and the comparison against an fp32 prob are exact.
__device__ __forceinline__ float u24(uint32_t r) { return (float)(r >> 8) * (1.0f / 16777216.0f); }

// ---------------------------------------------------------------- exact weight arithmetic
// The build sums weights as 128-bit fixed point (grid 2^-64) so that the total, and with it
// every table entry, does not depend on the order of the parallel reduction.
struct u128 {
  uint64_t lo, hi;
};
__device__ __forceinline__ u128 add128(u128 a, u128 b) {
  u128 r;
  r.lo = a.lo + b.lo;
  r.hi = a.hi + b.hi + (r.lo < a.lo ? 1ull : 0ull);
  return r;
}
__device__ __forceinline__ float clamp_weight(float w) {
  // median of (w, 0, 2^32): zero, negatives and NaN give +0 (a NaN operand makes the instruction return the
  // smallest of the other two), values above 2^32 give 2^32
  return __builtin_amdgcn_fmed3f(w, 0.0f, 4294967296.0f);
}
// The clamped weight of a slot of the row, +0 for a slot outside it: the upper bound carries the mask, which
// costs one 32-bit select instead of two on the converted double.
__device__ __forceinline__ float masked_weight(float w, bool in) {
  return __builtin_amdgcn_fmed3f(w, 0.0f, in ? 4294967296.0f : 0.0f);
}
// floor(w * 2^64) of a clamped weight.
__device__ __forceinline__ u128 weight_fixed(float w) {
  const uint32_t bits = __float_as_uint(w);
  const uint32_t e = (bits >> 23) & 0xFFu;
  const uint64_t m = (bits & 0x7FFFFFu) | 0x800000u;
  const int sh = (int)e - 86;
  u128 r{0, 0};
  if (e == 0 || sh <= -24) return r;
  if (sh < 0) {
    r.lo = m >> (-sh);
  } else if (sh < 64) {
    r.lo = m << sh;
    r.hi = sh ? (m >> (64 - sh)) : 0;
  } else {
    r.hi = m << (sh - 64);
  }
  return r;
}
__device__ __forceinline__ double fixed_to_double(u128 s) {
  const uint32_t l0 = (uint32_t)s.lo, l1 = (uint32_t)(s.lo >> 32), l2 = (uint32_t)s.hi, l3 = (uint32_t)(s.hi >> 32);
  const double hi = (double)l3 * 4294967296.0 + (double)l2;
  const double lo = (double)l1 * (1.0 / 4294967296.0) + (double)l0 * (1.0 / 18446744073709551616.0);
  return hi + lo;
}

// The same exact sum without 128-bit integer work per entry: floor(w * 2^64) of a clamped weight is
// top * 2^64 + mid * 2^32 + low with three integers of at most 2^32, here kept as doubles.  Sums of up
// to 2^20 such terms stay below 2^53, so fp64 additions of them are exact in any order.
struct WSum3 {
  double top, mid, low;
};
__device__ __forceinline__ void wsum3_add(WSum3& s, double wd /* (double) clamped weight */) {
  const double top = trunc(wd);
  const double m = (wd - top) * 4294967296.0;  // exact: wd carries 24 significant bits
  const double mid = trunc(m);
  s.top += top;
  s.mid += mid;
  s.low += floor((m - mid) * 4294967296.0);
}
// double(S) exactly as fixed_to_double gives it for the u128 S = top * 2^64 + mid * 2^32 + low
// (needs top + carries < 2^53: rows of fewer than 2^20 entries).  Returns 0 for the zero sum.
__device__ __forceinline__ double wsum3_to_double(const WSum3& s) {
  const double c0 = floor(s.low * (1.0 / 4294967296.0));
  const double l0 = s.low - c0 * 4294967296.0;
  const double m = s.mid + c0;
  const double c1 = floor(m * (1.0 / 4294967296.0));
  const double l1 = m - c1 * 4294967296.0;
  const double hi = s.top + c1;  // = l3 * 2^32 + l2, exact
  const double lo = l1 * (1.0 / 4294967296.0) + l0 * (1.0 / 18446744073709551616.0);
  return hi + lo;
}

// The integer ledger of a row keeps F fraction bits: 40, fewer only for rows of 2^22 entries
// and more so that the row's prefix sums stay below 2^63.
struct Ledger {
  double scale;   // deg / sum(w): p = w * scale
  double fs;      // 2^F
  double inv_fs;  // 2^-F
  uint64_t one;   // 2^F
};
__device__ __forceinline__ Ledger make_ledger(uint32_t deg, u128 sum) {
  const int F = deg < (1u << 22) ? 40 : 62 - (31 - __clz((int)deg));
  Ledger L;
  L.scale = (double)deg / fixed_to_double(sum);
  L.one = 1ull << F;
  L.fs = (double)L.one;
  L.inv_fs = 1.0 / L.fs;
  return L;
}
// Per-entry classification: t = (p - 1) * 2^F; heavy iff t >= 0.5; amount = max(rint(|t|), 1 if heavy).
struct Entry {
  double p;
  uint64_t amount;  // surplus (heavy) or deficit (light), units of 2^-F
  bool heavy;
};
// |t| rounded to the nearest integer, ties to even.  Below 2^52 adding 2^52 leaves the rounded integer in
// the low mantissa bits (two instructions); from 2^52 on a double is an integer already.
__device__ __forceinline__ uint64_t round_to_u64(double x) {
  if (x < 4503599627370496.0) return (uint64_t)__double_as_longlong(x + 4503599627370496.0) - 0x4330000000000000ull;
  return (uint64_t)x;
}
__device__ __forceinline__ Entry classify(float w, const Ledger& L) {
  Entry e;
  e.p = (double)w * L.scale;
  const double t = (e.p - 1.0) * L.fs;
  e.heavy = t >= 0.5;
  e.amount = round_to_u64(fmax(e.heavy ? t : -t, 0.0));  // a light with 0 < t < 0.5 has deficit 0
  if (e.heavy && e.amount == 0) e.amount = 1;  // t = 0.5 exactly rounds to even 0: a heavy always has surplus >= 1
  return e;
}
__device__ __forceinline__ Ledger make_ledger_small(uint32_t deg, double sum /* double(S), deg < 2^22 */) {
  Ledger L;
  L.scale = (double)deg / sum;
  L.one = 1ull << 40;
  L.fs = 1099511627776.0;
  L.inv_fs = 1.0 / 1099511627776.0;
  return L;
}
// classify for rows of fewer than 2^12 entries (|t| < 2^52, F = 40): same values as classify, fewer
// instructions.  `in` false gives a light of deficit 0.  max(t, 1) before rounding == max(rint(t), 1) for a
// heavy.  (p - 1) * fs as written: the product with a power of two is exact, so one rounding as in classify;
// a subtraction with an inline constant and a multiplication, where a fused form needs its addend moved
// into the destination first.
__device__ __forceinline__ Entry classify_small(double wd, bool in, const Ledger& L) {
  Entry e;
  e.p = in ? wd * L.scale : 1.0;
  const double t = (e.p - 1.0) * L.fs;
  e.heavy = t >= 0.5;
  const double a = fmax(fabs(t), e.heavy ? 1.0 : 0.0);  // |t| < 0.5 for a light with t > 0: rounds to the deficit 0
  e.amount = (uint64_t)__double_as_longlong(a + 4503599627370496.0) - 0x4330000000000000ull;
  return e;
}
// classify_small without the row mask: a slot outside the row arrives with weight +0 and comes out as a
// light with a deficit of 2^F, which the caller drops (two selects on a double saved per entry; the
// caller's own selects take the mask for free, as a scalar AND of lane masks).
__device__ __forceinline__ Entry classify_small_unmasked(double wd, const Ledger& L) {
  Entry e;
  e.p = wd * L.scale;
  const double t = (e.p - 1.0) * L.fs;
  e.heavy = t >= 0.5;
  const double a = fmax(fabs(t), e.heavy ? 1.0 : 0.0);  // |t| < 0.5 for a light with t > 0: rounds to the deficit 0
  e.amount = (uint64_t)__double_as_longlong(a + 4503599627370496.0) - 0x4330000000000000ull;
  return e;
}
// classify with fewer instructions for any row: same values.  The 2^52 rounding shortcut covers every
// amount below 2^52; larger ones are integers already and take the (rare, branched) general conversion.
__device__ __forceinline__ Entry classify_fast(double wd, bool in, const Ledger& L) {
  Entry e;
  e.p = in ? wd * L.scale : 1.0;
  const double t = (e.p - 1.0) * L.fs;
  e.heavy = t >= 0.5;
  const double a = fmax(fabs(t), e.heavy ? 1.0 : 0.0);  // |t| < 0.5 for a light with t > 0: rounds to the deficit 0
  if (a < 4503599627370496.0)
    e.amount = (uint64_t)__double_as_longlong(a + 4503599627370496.0) - 0x4330000000000000ull;
  else
    e.amount = (uint64_t)a;
  return e;
}
// u128 value of an exact three-limb sum (limbs below 2^53).
__device__ __forceinline__ u128 wsum3_to_u128(const WSum3& s) {
  const uint64_t top = (uint64_t)s.top, mid = (uint64_t)s.mid, low = (uint64_t)s.low;
  u128 r{low, top};
  r = add128(r, u128{mid << 32, mid >> 32});
  return r;
}
__device__ __forceinline__ float residual_prob(uint64_t r_units, const Ledger& L) {
  return (float)((double)r_units * L.inv_fs);
}

// first m in [lo, n) with a[m] > key, else n
__device__ __forceinline__ uint32_t first_greater(const uint64_t* a, uint32_t lo, uint32_t n, uint64_t key) {
  uint32_t len = n - lo;
  while (len > 0) {
    const uint32_t half = len >> 1;
    if (a[lo + half] <= key) {
      lo += half + 1;
      len -= half + 1;
    } else {
      len = half;
    }
  }
  return lo;
}

// ---------------------------------------------------------------- alias table entries
// The table keeps {prob, alias} of a slot side by side: a draw reads one 8-byte entry, not two
// arrays (one cache line less per walk step).  Same definition as sky_alias_entry of the C header.
struct AliasEntry {
  float prob;
  uint32_t alias;
};
// A table entry that is read once (a draw of a walk or a sample): loaded past the cache's usual replacement
// order, so that the gathers of a walk do not evict what is read again and again (the row offsets).
__device__ __forceinline__ AliasEntry load_entry_once(const AliasEntry* p) {
  const unsigned long long b = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long*>(p));
  return AliasEntry{__uint_as_float((uint32_t)b), (uint32_t)(b >> 32)};
}
// Entry of the optional walk index: the table entry of a slot together with the neighbour ids of the slot
// itself and of its alias slot, so that a step needs no gather from the adjacency array.
struct WalkEntry {
  float prob;
  uint32_t alias;
  uint32_t nbr_col, nbr_alias;
};
// Four consecutive entries starting at a 32-byte aligned slot, as two 16-byte stores.
__device__ __forceinline__ void store_entries4(AliasEntry* t, const float (&p)[4], const uint32_t (&a)[4]) {
  uint4* o = reinterpret_cast<uint4*>(t);
  o[0] = make_uint4(__float_as_uint(p[0]), a[0], __float_as_uint(p[1]), a[1]);
  o[1] = make_uint4(__float_as_uint(p[2]), a[2], __float_as_uint(p[3]), a[3]);
}

// ---------------------------------------------------------------- wave64 primitives
__device__ __forceinline__ unsigned lane_id() { return __lane_id(); }

__device__ __forceinline__ uint64_t shfl_u64(uint64_t v, int src) {
  const uint32_t lo = __shfl((int)(uint32_t)v, src, 64);
  const uint32_t hi = __shfl((int)(uint32_t)(v >> 32), src, 64);
  return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int mask) {
  const uint32_t lo = __shfl_xor((int)(uint32_t)v, mask, 64);
  const uint32_t hi = __shfl_xor((int)(uint32_t)(v >> 32), mask, 64);
  return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ uint64_t shfl_up_u64(uint64_t v, int delta) {
  const uint32_t lo = __shfl_up((int)(uint32_t)v, delta, 64);
  const uint32_t hi = __shfl_up((int)(uint32_t)(v >> 32), delta, 64);
  return ((uint64_t)hi << 32) | lo;
}
// ---- DPP building blocks.  A wave is four rows of 16 lanes; row_shr:n moves data n lanes up inside a
// row, row_bcast15 / row_bcast31 carry the last lane of a row (of the first half) to the next row(s).
// Lanes without a source, and rows masked off, receive 0.  Callers must be convergent (all 64 lanes
// active): a DPP read from a disabled lane is not defined.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp0(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xF, true);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint64_t dpp0_u64(uint64_t v) {
  // the 64-bit form keeps the two moved halves a register pair, so that the addition that follows is one
  // instruction (halves joined by shift and or end up as two additions)
  return (uint64_t)__builtin_amdgcn_update_dpp((uint64_t)0, v, CTRL, ROW_MASK, 0xF, true);
}
constexpr int DPP_ROW_SHR1 = 0x111, DPP_ROW_SHR2 = 0x112, DPP_ROW_SHR4 = 0x114, DPP_ROW_SHR8 = 0x118;
constexpr int DPP_ROW_BCAST15 = 0x142, DPP_ROW_BCAST31 = 0x143;
constexpr int DPP_QUAD_XOR1 = 0xB1 /* quad_perm [1,0,3,2] */, DPP_QUAD_XOR2 = 0x4E /* quad_perm [2,3,0,1] */;
constexpr int DPP_ROW_HALF_MIRROR = 0x141, DPP_ROW_MIRROR = 0x140;

// Inclusive prefix sum over aligned groups of G lanes (G = 4, 8, 16, 32, 64).
template <int G>
__device__ __forceinline__ uint64_t group_scan_u64(uint64_t v) {
  const int gl = lane_id() & (G - 1);
  if (G >= 16) {
    v += dpp0_u64<DPP_ROW_SHR1, 0xF>(v);
    v += dpp0_u64<DPP_ROW_SHR2, 0xF>(v);
    v += dpp0_u64<DPP_ROW_SHR4, 0xF>(v);
    v += dpp0_u64<DPP_ROW_SHR8, 0xF>(v);
    if (G >= 32) v += dpp0_u64<DPP_ROW_BCAST15, 0xA>(v);
    if (G >= 64) v += dpp0_u64<DPP_ROW_BCAST31, 0xC>(v);
  } else {
    uint64_t o = dpp0_u64<DPP_ROW_SHR1, 0xF>(v);
    v += gl >= 1 ? o : 0;
    if (G >= 4) {
      o = dpp0_u64<DPP_ROW_SHR2, 0xF>(v);
      v += gl >= 2 ? o : 0;
    }
    if (G >= 8) {
      o = dpp0_u64<DPP_ROW_SHR4, 0xF>(v);
      v += gl >= 4 ? o : 0;
    }
  }
  return v;
}
template <int G>
__device__ __forceinline__ uint32_t group_scan_u32(uint32_t v) {
  const int gl = lane_id() & (G - 1);
  if (G >= 16) {
    v += dpp0<DPP_ROW_SHR1, 0xF>(v);
    v += dpp0<DPP_ROW_SHR2, 0xF>(v);
    v += dpp0<DPP_ROW_SHR4, 0xF>(v);
    v += dpp0<DPP_ROW_SHR8, 0xF>(v);
    if (G >= 32) v += dpp0<DPP_ROW_BCAST15, 0xA>(v);
    if (G >= 64) v += dpp0<DPP_ROW_BCAST31, 0xC>(v);
  } else {
    uint32_t o = dpp0<DPP_ROW_SHR1, 0xF>(v);
    v += gl >= 1 ? o : 0;
    o = dpp0<DPP_ROW_SHR2, 0xF>(v);
    v += gl >= 2 ? o : 0;
    if (G >= 8) {
      o = dpp0<DPP_ROW_SHR4, 0xF>(v);
      v += gl >= 4 ? o : 0;
    }
  }
  return v;
}
// Sum over aligned groups of G lanes; every lane of the group receives the total.
// Butterfly inside a row of 16 by DPP (xor 1, xor 2, half mirror, mirror), then across rows.
template <int G>
__device__ __forceinline__ u128 group_sum_u128(u128 v) {
  auto mix = [&](auto get) {
    u128 o;
    o.lo = get(v.lo);
    o.hi = get(v.hi);
    v = add128(v, o);
  };
  mix([](uint64_t x) { return dpp0_u64<DPP_QUAD_XOR1, 0xF>(x); });
  mix([](uint64_t x) { return dpp0_u64<DPP_QUAD_XOR2, 0xF>(x); });
  if (G >= 8) mix([](uint64_t x) { return dpp0_u64<DPP_ROW_HALF_MIRROR, 0xF>(x); });
  if (G >= 16) mix([](uint64_t x) { return dpp0_u64<DPP_ROW_MIRROR, 0xF>(x); });
  if (G >= 32) mix([](uint64_t x) { return shfl_xor_u64(x, 16); });
  if (G >= 64) mix([](uint64_t x) { return shfl_xor_u64(x, 32); });
  return v;
}

// Sum of a double over aligned groups of G lanes; every lane receives the total.
template <int G>
__device__ __forceinline__ double group_sum_f64(double v) {
  auto get = [](double x, auto f) {
    const uint64_t b = (uint64_t)__double_as_longlong(x);
    return __longlong_as_double((long long)f(b));
  };
  v += get(v, [](uint64_t b) { return dpp0_u64<DPP_QUAD_XOR1, 0xF>(b); });
  if (G >= 4) v += get(v, [](uint64_t b) { return dpp0_u64<DPP_QUAD_XOR2, 0xF>(b); });
  if (G >= 8) v += get(v, [](uint64_t b) { return dpp0_u64<DPP_ROW_HALF_MIRROR, 0xF>(b); });
  if (G >= 16) v += get(v, [](uint64_t b) { return dpp0_u64<DPP_ROW_MIRROR, 0xF>(b); });
  if (G >= 32) v += get(v, [](uint64_t b) { return shfl_xor_u64(b, 16); });
  if (G >= 64) v += get(v, [](uint64_t b) { return shfl_xor_u64(b, 32); });
  return v;
}
template <int G>
__device__ __forceinline__ WSum3 group_sum_wsum3(WSum3 s) {
  s.top = group_sum_f64<G>(s.top);
  s.mid = group_sum_f64<G>(s.mid);
  s.low = group_sum_f64<G>(s.low);
  return s;
}

// Minimum over the wavefront; every lane receives it.
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
  v = min(v, dpp0<DPP_QUAD_XOR1, 0xF>(v));
  v = min(v, dpp0<DPP_QUAD_XOR2, 0xF>(v));
  v = min(v, dpp0<DPP_ROW_HALF_MIRROR, 0xF>(v));
  v = min(v, dpp0<DPP_ROW_MIRROR, 0xF>(v));
  v = min(v, (uint32_t)__shfl_xor((int)v, 16, 64));
  v = min(v, (uint32_t)__shfl_xor((int)v, 32, 64));
  return v;
}

// Residual probability of a heavy whose surplus prefix lies d units (d < 2^40) below the deficit prefix of the
// light that finishes it: (2^40 - d) * 2^-40, the value residual_prob gives for 2^40 + SH - SL.  d below 2^52
// becomes a double by the 2^52 trick; 1 - d * 2^-40 is a multiple of 2^-40 in (0, 1] and therefore exact.
__device__ __forceinline__ float residual_below(uint64_t d) {
  const double x = __longlong_as_double((long long)(d | 0x4330000000000000ull)) - 4503599627370496.0;
  return (float)fma(x, -1.0 / 1099511627776.0, 1.0);
}

// The exact sum of a row without 128-bit work per entry.  Every clamped weight is a multiple of
// u = 2^(e - 150), e the smallest exponent field among the nonzero ones; when e >= 86 no weight loses anything
// to the floor of w * 2^64, and when the fp64 sum of the weights stays below 2^53 u every partial sum of
// the (positive) terms is a multiple of u below 2^53 u, so every addition was exact in whatever order the lanes
// added: the fp64 sum then equals double(S) of the 128-bit definition bit for bit.  (A sum that was rounded
// somewhere is at least 2^53 u, because rounding is monotone and 2^53 u is representable: the test cannot pass
// by accident.)  `mn` = min over the row of (weight bits - 1), unsigned: zero weights wrap to 2^32 - 1 and drop
// out, a weight of the form 2^k counts with the exponent below its own, which only makes the test stricter.
__device__ __forceinline__ bool plain_sum_is_exact(double sum, uint32_t mn) {
  const int e = (int)(mn >> 23);  // 511 for a row without a nonzero weight
  return e >= 86 && sum < ldexp(1.0, e - 97);
}

// Minimum of a 32-bit value over aligned groups of G lanes; every lane of the group receives it.
template <int G>
__device__ __forceinline__ uint32_t group_min_u32(uint32_t v) {
  v = min(v, dpp0<DPP_QUAD_XOR1, 0xF>(v));
  if (G >= 4) v = min(v, dpp0<DPP_QUAD_XOR2, 0xF>(v));
  if (G >= 8) v = min(v, dpp0<DPP_ROW_HALF_MIRROR, 0xF>(v));
  if (G >= 16) v = min(v, dpp0<DPP_ROW_MIRROR, 0xF>(v));
  if (G >= 32) v = min(v, (uint32_t)__shfl_xor((int)v, 16, 64));
  if (G >= 64) v = min(v, (uint32_t)__shfl_xor((int)v, 32, 64));
  return v;
}

// classify_small_unmasked with one instruction less per step: t by one fused multiply-add (the product with 2^F
// is exact, so the result is rounded once, as (p - 1) * 2^F is), the amount cut out of the 2^52 sum by a mask.
__device__ __forceinline__ Entry classify_small_fma(double wd, const Ledger& L, double neg_fs) {
  Entry e;
  e.p = wd * L.scale;
  const double t = fma(e.p, L.fs, neg_fs);
  e.heavy = t >= 0.5;
  const double a = fmax(fabs(t), e.heavy ? 1.0 : 0.0);  // |t| < 0.5 for a light with t > 0: rounds to the deficit 0
  e.amount = (uint64_t)__double_as_longlong(a + 4503599627370496.0) & 0x000FFFFFFFFFFFFFull;
  return e;
}

}  // namespace sky
