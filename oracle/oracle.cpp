// CPU oracle for the alias-method hot path.  TEST INFRASTRUCTURE ONLY.
//
// This file is the checker, never the product: only tests/, the smoke test and
// the benchmark's cpu_baseline leg may load it.  Nothing under skywalker_amd/
// links, includes or calls it, and the product has no CPU fallback.
//
// It restates, for a host CPU, what the reference's CUDA kernels compute:
//   * per-vertex alias tables            (include/alias_table_new.cuh:1077-1132 normalise,
//                                         :1211-1316 small/large pairing; src/createTable.cu:3-46
//                                         table slot = CSR edge slot, valid flag)
//   * biased walk on prebuilt tables     (src/offline_walk.cu:75-124)
//   * online walk / PPR / node2vec       (src/online_walk.cu:10-40,97-132; src/api/bias_node2vec.cu:15-27;
//                                         include/gpu_graph.cuh:204-238 sorted-row membership)
//   * k-hop neighbour sampling           (src/offline_sample.cu:72-141; include/sampler_result.cuh:226-260,334-352
//                                         output layout, child slot = parent_slot*fanout + i)
// The reference's RNG (cuRAND XORWOW, closed source) is replaced by Philox4x32-10
// keyed by (seed, walker, step, hop): "parity unpinned" against XORWOW-exact
// paths, by design.  The reference's pairing ORDER (speculative float atomics,
// non-deterministic even on its own hardware) is likewise not reproduced; what
// is pinned is the distribution every table must encode.
//
// Pinned by (tests/test_oracle_*.py):
//   philox4x32_10      Random123 known-answer vectors.
//   alias build        reconstruction invariant q_i == w_i/sum(w) (1e-6 rel) on every row,
//                      closed forms (deg 1, equal weights, two weights, 35x0.5+5x2.0 toy of test/tmp.cu:30-52),
//                      textbook stack-based Vose (orc_vose_row) on random rows: same distribution.
//   walks / samples    chi-square of next-hop frequencies, truncated-geometric PPR lengths,
//                      star/path/complete closed forms, brute-force node2vec factors on tiny graphs.
//
// ---------------------------------------------------------------------------
// Arithmetic contract shared with the GPU library (so results are bit-exact and
// do not depend on how either side parallelises):
//   w'   = w if 0 < w <= 2^32 ; 2^32 if w > 2^32 ; 0 if w <= 0 or NaN
//   S    = sum_i floor(w'_i * 2^64)          exact, 128-bit unsigned integer
//   Sd   = ((double)l3*2^32 + (double)l2) + ((double)l1*2^-32 + (double)l0*2^-64)   (l0..l3 = 32-bit limbs of S)
//   scale= (double)deg / Sd ;  p_i = (double)w'_i * scale
//   F    = 40 if deg < 2^22, else 62 - floor(log2(deg))    (fraction bits of the integer ledger)
//   t_i  = (p_i - 1.0) * 2^F
//   heavy iff t_i >= 0.5, with surplus U_i = max(rint(t_i), 1)                     (64-bit unsigned,
//   light otherwise, with deficit D_i = rint(-t_i)                                  rint = nearest, ties to even)
//   lights and heavies are taken in CSR slot order.  A sweep lets heavy j fill
//   lights while its residual r (units of 2^-F) exceeds 2^F; when r <= 2^F the
//   heavy becomes a bucket {prob = r*2^-F, alias = next heavy} and the next
//   heavy inherits r + U.  The last heavy always ends {prob 1, alias self};
//   lights left without a donor take the last heavy; a row without heavies is
//   {prob (float)p, alias self}.  A light stores prob = (float)p_i.
//   Rows with S == 0 (or deg 0) are invalid: valid=0, prob=0, alias=0xFFFFFFFF.
//   Compiled with -ffp-contract=off; no fast-math.
// ---------------------------------------------------------------------------
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef unsigned __int128 u128;

static const uint32_t ORC_INVALID = 0xFFFFFFFFu;

// Philox counter domains (word 3 of the counter).
enum : uint32_t {
  DOM_RMAT = 1,
  DOM_WEIGHT = 2,
  DOM_SEEDS = 3,
  DOM_WALK = 4,
  DOM_SAMPLE = 5,
};

extern "C" {

// ---------------------------------------------------------------- Philox4x32-10
// Salmon et al., "Parallel random numbers: as easy as 1, 2, 3" (SC'11).
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u;
  const uint32_t W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)M0 * c0;
    uint64_t p1 = (uint64_t)M1 * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += W0; k1 += W1;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

}  // extern "C"

static inline void philox(uint64_t seed, uint32_t a, uint32_t b, uint32_t c, uint32_t dom, uint32_t out[4]) {
  uint32_t ctr[4] = {a, b, c, dom};
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  orc_philox4x32_10(ctr, key, out);
}
// 24-bit uniform in [0,1): exact in fp32.
static inline float u24(uint32_t r) { return (float)(r >> 8) * (1.0f / 16777216.0f); }
static inline uint32_t mulhi32(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * b) >> 32); }

// ---------------------------------------------------------------- synthetic inputs
extern "C" {

// R-MAT edge i of a 2^scale-vertex graph: one 16-bit uniform per level, eight
// levels per Philox call.  Thresholds a=.57 b=.19 c=.19 d=.05 on a 65536 grid.
// Level L (0 = most significant bit) uses call L/8, 16-bit lane L%8.
static inline void rmat_edge(uint64_t seed, uint64_t i, uint32_t scale, uint32_t* src, uint32_t* dst) {
  const uint32_t A = 37355u, AB = 49807u, ABC = 62259u;
  uint32_t s = 0, d = 0, r[4] = {0, 0, 0, 0};
  for (uint32_t lvl = 0; lvl < scale; ++lvl) {
    if ((lvl & 7u) == 0) philox(seed, (uint32_t)i, (uint32_t)(i >> 32), lvl >> 3, DOM_RMAT, r);
    uint32_t word = r[(lvl & 7u) >> 1];
    uint32_t x = (lvl & 1u) ? (word >> 16) : (word & 0xFFFFu);
    uint32_t sb = x >= AB ? 1u : 0u;
    uint32_t db = (x >= A && x < AB) || x >= ABC ? 1u : 0u;
    s = (s << 1) | sb;
    d = (d << 1) | db;
  }
  *src = s; *dst = d;
}

// CSR of the R-MAT multigraph: all E = edge_factor << scale edges, duplicates and
// self loops kept, sorted by (src, dst).
int orc_rmat_csr(uint32_t scale, uint32_t edge_factor, uint64_t seed, uint32_t* xadj, uint32_t* adjncy) {
  if (scale == 0 || scale > 31) return -1;
  const uint64_t V = 1ull << scale, E = (uint64_t)edge_factor << scale;
  if (E > 0xFFFFFFFFull) return -1;
  std::vector<uint64_t> keys(E);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)E; ++i) {
    uint32_t s, d;
    rmat_edge(seed, (uint64_t)i, scale, &s, &d);
    keys[i] = ((uint64_t)s << 32) | d;
  }
  std::sort(keys.begin(), keys.end());
  std::fill(xadj, xadj + V + 1, 0u);
  for (uint64_t i = 0; i < E; ++i) {
    xadj[(keys[i] >> 32) + 1]++;
    adjncy[i] = (uint32_t)keys[i];
  }
  for (uint64_t v = 0; v < V; ++v) xadj[v + 1] += xadj[v];
  return 0;
}

// Per-slot weights.  kind 0: U[lo,hi) = fmaf(hi-lo, u, lo), u = 24-bit uniform in [0,1)
//                    kind 1: U(0,1]  = (k+1) * 2^-24
//                    kind 2: log-normal exp(mu + sigma*z), z by Box-Muller (libm: not bit-portable)
int orc_gen_weights(int kind, uint64_t seed, uint64_t E, float a, float b, float* w) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)E; ++i) {
    uint32_t r[4];
    philox(seed, (uint32_t)i, (uint32_t)((uint64_t)i >> 32), 0, DOM_WEIGHT, r);
    if (kind == 0) {
      w[i] = fmaf(b - a, u24(r[0]), a);
    } else if (kind == 1) {
      w[i] = (float)((r[0] >> 8) + 1u) * (1.0f / 16777216.0f);
    } else {
      float u1 = (float)((r[0] >> 8) + 1u) * (1.0f / 16777216.0f);
      float u2 = u24(r[1]);
      float z = sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
      w[i] = expf(a + b * z);
    }
  }
  return 0;
}

// Start vertices: uniform over [0,V) from Philox(seed, i).
int orc_gen_seeds(uint64_t seed, uint32_t V, uint32_t N, uint32_t* seeds) {
  for (uint32_t i = 0; i < N; ++i) {
    uint32_t r[4];
    philox(seed, i, 0, 0, DOM_SEEDS, r);
    seeds[i] = mulhi32(r[0], V);
  }
  return 0;
}

}  // extern "C"

// ---------------------------------------------------------------- alias tables
static inline float clamp_weight(float w) {
  if (!(w > 0.0f)) return 0.0f;  // negatives, zero, NaN
  if (w > 4294967296.0f) return 4294967296.0f;
  return w;
}
// floor(w * 2^64) for a clamped weight, exactly.
static inline u128 weight_fixed(float w) {
  uint32_t bits;
  memcpy(&bits, &w, 4);
  uint32_t e = (bits >> 23) & 0xFFu;
  if (e == 0) return 0;  // zero and subnormals: below the grid
  u128 m = (bits & 0x7FFFFFu) | 0x800000u;
  int sh = (int)e - 86;  // value = m * 2^(e-150); times 2^64
  if (sh >= 0) return m << sh;
  if (sh <= -24) return 0;
  return m >> (-sh);
}
static inline double fixed_to_double(u128 S) {
  uint32_t l0 = (uint32_t)S, l1 = (uint32_t)(S >> 32), l2 = (uint32_t)(S >> 64), l3 = (uint32_t)(S >> 96);
  double hi = (double)l3 * 4294967296.0 + (double)l2;
  double lo = (double)l1 * (1.0 / 4294967296.0) + (double)l0 * (1.0 / 18446744073709551616.0);
  return hi + lo;
}

static inline int frac_bits(uint32_t deg) {
  if (deg < (1u << 22)) return 40;
  int lg = 0;
  while ((deg >> (lg + 1)) != 0) ++lg;
  return 62 - lg;
}

// One row by the two-pointer sweep.  getw(i) yields the raw weight of slot i.
// Returns 1 if the row is valid.
template <class GetW>
static int alias_row_sweep(uint32_t deg, GetW getw, float* prob, uint32_t* alias,
                           std::vector<double>& p, std::vector<uint32_t>& heavy) {
  u128 S = 0;
  for (uint32_t i = 0; i < deg; ++i) S += weight_fixed(clamp_weight(getw(i)));
  if (deg == 0) return 0;
  if (S == 0) {
    for (uint32_t i = 0; i < deg; ++i) { prob[i] = 0.0f; alias[i] = ORC_INVALID; }
    return 0;
  }
  const double scale = (double)deg / fixed_to_double(S);
  p.resize(deg);
  heavy.clear();
  const int F = frac_bits(deg);
  const double FS = std::ldexp(1.0, F), INV_FS = std::ldexp(1.0, -F);
  auto excess = [&](uint32_t i) -> double { return (p[i] - 1.0) * FS; };
  for (uint32_t i = 0; i < deg; ++i) {
    p[i] = (double)clamp_weight(getw(i)) * scale;
    if (excess(i) >= 0.5) heavy.push_back(i);
  }
  const size_t nH = heavy.size();
  auto surplus = [&](uint32_t j) -> uint64_t {
    const uint64_t u = (uint64_t)std::nearbyint(excess(heavy[j]));  // default rounding mode: ties to even
    return u ? u : 1;
  };
  const uint64_t ONE = 1ull << F;
  if (nH == 0) {
    for (uint32_t i = 0; i < deg; ++i) { prob[i] = (float)p[i]; alias[i] = i; }
    return 1;
  }
  size_t j = 0;
  uint64_t r = ONE + surplus(0);  // residual of the current heavy, units of 2^-32
  for (uint32_t i = 0; i < deg; ++i) {
    if (excess(i) >= 0.5) continue;
    // retire heavies that can no longer donate
    while (r <= ONE && j + 1 < nH) {
      prob[heavy[j]] = (float)((double)r * INV_FS);
      alias[heavy[j]] = heavy[j + 1];
      r += surplus(j + 1);
      ++j;
    }
    const uint64_t D = (uint64_t)std::nearbyint(-excess(i));
    prob[i] = (float)p[i];
    alias[i] = heavy[j];  // the last heavy also absorbs lights left without a donor
    // a heavy that is not the last has r > 2^32 > D here; the last heavy's r is never read again
    if (j + 1 < nH) r -= D;
  }
  // lights are done: retire the chain of heavies whose residual is spent
  while (r <= ONE && j + 1 < nH) {
    prob[heavy[j]] = (float)((double)r * INV_FS);
    alias[heavy[j]] = heavy[j + 1];
    r += surplus(j + 1);
    ++j;
  }
  // current heavy and every heavy never reached keep their own bucket whole
  for (; j < nH; ++j) { prob[heavy[j]] = 1.0f; alias[heavy[j]] = heavy[j]; }
  return 1;
}

extern "C" {

// Build one row from explicit weights.  Returns valid (0/1).
int orc_alias_build_row(const float* w, uint32_t deg, float* prob, uint32_t* alias) {
  std::vector<double> p;
  std::vector<uint32_t> heavy;
  return alias_row_sweep(deg, [&](uint32_t i) { return w[i]; }, prob, alias, p, heavy);
}

// Offline build for every vertex (what ConstructTable produces, src/createTable.cu:119-179).
int orc_alias_build(const uint32_t* xadj, const float* w, uint32_t V, float* prob, uint32_t* alias, int8_t* valid,
                    int nthreads) {
#ifdef _OPENMP
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#endif
#pragma omp parallel num_threads(nthreads > 0 ? nthreads : 1)
  {
    std::vector<double> p;
    std::vector<uint32_t> heavy;
#pragma omp for schedule(dynamic, 4096)
    for (int64_t v = 0; v < (int64_t)V; ++v) {
      const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
      const float* wr = w + off;
      valid[v] = (int8_t)alias_row_sweep(deg, [&](uint32_t i) { return wr[i]; }, prob + off, alias + off, p, heavy);
    }
  }
  return 0;
}

// Textbook Vose (stacks of small and large, fp64) for cross-checking the sweep:
// the two must encode the same distribution, not the same table.
int orc_vose_row(const float* w, uint32_t deg, double* prob, uint32_t* alias) {
  double sum = 0;
  for (uint32_t i = 0; i < deg; ++i) sum += (double)clamp_weight(w[i]);
  if (deg == 0 || sum == 0) return 0;
  std::vector<double> p(deg);
  std::vector<uint32_t> small, large;
  for (uint32_t i = 0; i < deg; ++i) {
    p[i] = (double)clamp_weight(w[i]) * deg / sum;
    (p[i] < 1.0 ? small : large).push_back(i);
  }
  while (!small.empty() && !large.empty()) {
    uint32_t s = small.back(); small.pop_back();
    uint32_t l = large.back(); large.pop_back();
    prob[s] = p[s]; alias[s] = l;
    p[l] = (p[l] + p[s]) - 1.0;
    (p[l] < 1.0 ? small : large).push_back(l);
  }
  for (uint32_t l : large) { prob[l] = 1.0; alias[l] = l; }
  for (uint32_t s : small) { prob[s] = 1.0; alias[s] = s; }
  return 1;
}

// Distribution encoded by a table row: q_i = (prob_i + sum_{j: alias_j = i} (1 - prob_j)) / deg, in fp64.
void orc_alias_reconstruct_row(const float* prob, const uint32_t* alias, uint32_t deg, double* q) {
  for (uint32_t i = 0; i < deg; ++i) q[i] = 0;
  for (uint32_t i = 0; i < deg; ++i) {
    q[i] += (double)prob[i];
    if (alias[i] < deg) q[alias[i]] += 1.0 - (double)prob[i];
  }
  for (uint32_t i = 0; i < deg; ++i) q[i] /= deg;
}

// Check every row of a table against the weights it was built from.
//   stats[0] max relative error of q_i vs w_i/sum(w) over valid rows (fp64)
//   stats[1] rows whose valid flag disagrees with (sum(w) > 0)
//   stats[2] entries with prob outside [0,1] or alias >= deg on valid rows
//   stats[3] entries of invalid rows that are not {0, 0xFFFFFFFF}
//   stats[4] vertex of the worst row
int orc_alias_check(const uint32_t* xadj, const float* w, const float* prob, const uint32_t* alias, const int8_t* valid,
                    uint32_t V, double* stats) {
  double worst = 0;
  uint64_t bad_valid = 0, bad_range = 0, bad_invalid = 0;
  uint32_t worst_v = 0;
#pragma omp parallel
  {
    std::vector<double> q;
    double lworst = 0;
    uint32_t lworst_v = 0;
    uint64_t lbv = 0, lbr = 0, lbi = 0;
#pragma omp for schedule(dynamic, 4096)
    for (int64_t v = 0; v < (int64_t)V; ++v) {
      const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
      long double sum = 0;
      u128 fixed = 0;  // a row is valid iff its exact 2^-64 fixed-point sum is not zero (weights below 2^-64 add nothing)
      for (uint32_t i = 0; i < deg; ++i) {
        sum += (long double)clamp_weight(w[off + i]);
        fixed += weight_fixed(clamp_weight(w[off + i]));
      }
      const bool ok = deg > 0 && fixed != 0;
      if ((valid[v] != 0) != ok) ++lbv;
      if (!ok) {
        for (uint32_t i = 0; i < deg; ++i)
          if (prob[off + i] != 0.0f || alias[off + i] != ORC_INVALID) ++lbi;
        continue;
      }
      bool range_ok = true;
      for (uint32_t i = 0; i < deg; ++i)
        if (!(prob[off + i] >= 0.0f && prob[off + i] <= 1.0f) || alias[off + i] >= deg) { ++lbr; range_ok = false; }
      if (!range_ok) continue;
      q.resize(deg);
      orc_alias_reconstruct_row(prob + off, alias + off, deg, q.data());
      for (uint32_t i = 0; i < deg; ++i) {
        double t = (double)((long double)clamp_weight(w[off + i]) / sum);
        // shares of a bucket below 1e-30 are at the edge of what a float probability can hold (denormals,
        // then zero): there only an absolute bound can be asked for
        double err;
        if (t * deg < 1e-30) err = q[i] * deg < 2e-30 ? 0.0 : 1.0;
        else err = std::fabs(q[i] - t) / t;
        if (err > lworst) { lworst = err; lworst_v = (uint32_t)v; }
      }
    }
#pragma omp critical
    {
      if (lworst > worst) { worst = lworst; worst_v = lworst_v; }
      bad_valid += lbv; bad_range += lbr; bad_invalid += lbi;
    }
  }
  stats[0] = worst; stats[1] = (double)bad_valid; stats[2] = (double)bad_range; stats[3] = (double)bad_invalid;
  stats[4] = (double)worst_v;
  return 0;
}

// ---------------------------------------------------------------- walks on prebuilt tables
// Step rule (src/offline_walk.cu:89-120) with the stop test of the online kernel
// (src/online_walk.cu:109-110) placed before the step:
//   r = Philox(seed; walker, step, 0, DOM_WALK)
//   stop if stop_prob > 0 and u24(r[2]) < stop_prob          -> length = step
//   stop if deg == 0                                          -> length = step
//   col = mulhi(r[0], deg); cand = u24(r[1]) < prob[col] ? col : alias[col]
//   stop if cand == 0xFFFFFFFF (row with zero total weight)   -> length = step
//   next = adjncy[off + cand]
// paths is walker-major, N x (len+1) (sampler_result.cuh:607-612); slots past
// length[i] are not written.
int orc_walk_offline(const uint32_t* xadj, uint32_t V, const uint32_t* adjncy, const float* prob, const uint32_t* alias,
                     const uint32_t* seeds, uint32_t N, uint32_t len, float stop_prob, uint64_t seed, uint32_t* paths,
                     uint32_t* lengths, uint64_t* sampled) {
  uint64_t total = 0;
#pragma omp parallel for schedule(dynamic, 256) reduction(+ : total)
  for (int64_t i = 0; i < (int64_t)N; ++i) {
    uint32_t* path = paths + (size_t)i * (len + 1);
    uint32_t v = seeds[i];
    path[0] = v;
    uint32_t s = 0;
    for (; s < len && v < V; ++s) {  // a start vertex that does not exist is recorded and never left
      uint32_t r[4];
      philox(seed, (uint32_t)i, s, 0, DOM_WALK, r);
      if (stop_prob > 0.0f && u24(r[2]) < stop_prob) break;
      const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
      if (deg == 0) break;
      const uint32_t col = mulhi32(r[0], deg);
      const uint32_t cand = u24(r[1]) < prob[off + col] ? col : alias[off + col];
      if (cand == ORC_INVALID) break;
      v = adjncy[off + cand];
      path[s + 1] = v;
    }
    lengths[i] = s;
    total += s;
  }
  if (sampled) *sampled = total;
  return 0;
}

// ---------------------------------------------------------------- online walks (table per step)
// Second-order factor of node2vec (src/api/bias_node2vec.cu:15-27): weight of the edge to
// `nbr` is divided by p when nbr is the previous vertex, kept when nbr is adjacent
// to the previous vertex (sorted-row membership, gpu_graph.cuh:204-238), divided by
// q otherwise.  On the first step there is no previous vertex: factor 1.
// The weight is the edge slot's own weight (the reference indexes adjwgt by the
// neighbour's vertex id, a quirk that is not kept).
static inline float node2vec_weight(const uint32_t* xadj, const uint32_t* adjncy, float w, uint32_t nbr, bool has_prev,
                                    uint32_t prev, float p, float q) {
  if (!has_prev) return w;
  if (nbr == prev) return w / p;
  const uint32_t* b = adjncy + xadj[prev];
  const uint32_t* e = adjncy + xadj[prev + 1];
  if (std::binary_search(b, e, nbr)) return w;
  return w / q;
}

// bias_kind 0: static edge weights (DeepWalk / PPR); 1: node2vec second order.
int orc_walk_online(const uint32_t* xadj, uint32_t V, const uint32_t* adjncy, const float* w, int bias_kind, float p, float q,
                    const uint32_t* seeds, uint32_t N, uint32_t len, float stop_prob, uint64_t seed, uint32_t* paths,
                    uint32_t* lengths, uint64_t* sampled) {
  uint64_t total = 0;
#pragma omp parallel reduction(+ : total)
  {
    std::vector<float> rw, prob;
    std::vector<uint32_t> alias, heavy;
    std::vector<double> pp;
#pragma omp for schedule(dynamic, 64)
    for (int64_t i = 0; i < (int64_t)N; ++i) {
      uint32_t* path = paths + (size_t)i * (len + 1);
      uint32_t v = seeds[i], prev = 0;
      bool has_prev = false;
      path[0] = v;
      uint32_t s = 0;
      for (; s < len && v < V; ++s) {
        uint32_t r[4];
        philox(seed, (uint32_t)i, s, 0, DOM_WALK, r);
        if (stop_prob > 0.0f && u24(r[2]) < stop_prob) break;
        const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
        if (deg == 0) break;
        rw.resize(deg); prob.resize(deg); alias.resize(deg);
        for (uint32_t k = 0; k < deg; ++k)
          rw[k] = bias_kind == 1 ? node2vec_weight(xadj, adjncy, w[off + k], adjncy[off + k], has_prev, prev, p, q)
                                 : w[off + k];
        if (!alias_row_sweep(deg, [&](uint32_t k) { return rw[k]; }, prob.data(), alias.data(), pp, heavy)) break;
        const uint32_t col = mulhi32(r[0], deg);
        const uint32_t cand = u24(r[1]) < prob[col] ? col : alias[col];
        prev = v; has_prev = true;
        v = adjncy[off + cand];
        path[s + 1] = v;
      }
      lengths[i] = s;
      total += s;
    }
  }
  if (sampled) *sampled = total;
  return 0;
}

// node2vec by rejection on the first-order tables (the "second-order rejection" of KnightKing-style
// walkers; the reference's own unbiased node2vec, src/unbiased_walk.cu:14-60, uses the same idea).
// Step s of walker i with a previous vertex: trial t draws a candidate from the first-order table of
// the current vertex with r_t = Philox(seed; i, s, t, DOM_WALK) (t = 0 shares the step's counter with the
// stop test), cand = u24(r_t[1]) < prob[col] ? col : alias[col], col = mulhi(r_t[0], deg), and accepts
// it when u24(r_t[3]) * fmax < f(nbr), f = 1/p if nbr is the previous vertex, 1 if adjacent to it, 1/q
// otherwise, fmax = max(1/p, 1, 1/q).  After 65536 rejections the last candidate is taken.  The law of
// the accepted neighbour is w * f / sum(w * f), the same as a draw from the second-order table.
int orc_walk_node2vec_reject(const uint32_t* xadj, uint32_t V, const uint32_t* adjncy, const float* prob, const uint32_t* alias,
                             float p, float q, const uint32_t* seeds, uint32_t N, uint32_t len, float stop_prob,
                             uint64_t seed, uint32_t* paths, uint32_t* lengths, uint64_t* sampled) {
  const float fp = 1.0f / p, fq = 1.0f / q;
  const float fmax = std::max(1.0f, std::max(fp, fq));
  uint64_t total = 0;
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : total)
  for (int64_t i = 0; i < (int64_t)N; ++i) {
    uint32_t* path = paths + (size_t)i * (len + 1);
    uint32_t v = seeds[i], prev = 0;
    bool has_prev = false;
    path[0] = v;
    uint32_t s = 0;
    for (; s < len && v < V; ++s) {
      uint32_t r[4];
      philox(seed, (uint32_t)i, s, 0, DOM_WALK, r);
      if (stop_prob > 0.0f && u24(r[2]) < stop_prob) break;
      const uint32_t off = xadj[v], deg = xadj[v + 1] - off;
      if (deg == 0) break;
      uint32_t next = 0;
      bool dead = false;
      for (uint32_t t = 0;; ++t) {
        if (t) philox(seed, (uint32_t)i, s, t, DOM_WALK, r);
        const uint32_t col = mulhi32(r[0], deg);
        const uint32_t cand = u24(r[1]) < prob[off + col] ? col : alias[off + col];
        if (cand == ORC_INVALID) { dead = true; break; }
        next = adjncy[off + cand];
        if (!has_prev || t >= 65536) break;
        float f;
        if (next == prev) f = fp;
        else if (std::binary_search(adjncy + xadj[prev], adjncy + xadj[prev + 1], next)) f = 1.0f;
        else f = fq;
        if (u24(r[3]) * fmax < f) break;
      }
      if (dead) break;
      prev = v; has_prev = true;
      v = next;
      path[s + 1] = v;
    }
    lengths[i] = s;
    total += s;
  }
  if (sampled) *sampled = total;
  return 0;
}

// ---------------------------------------------------------------- k-hop neighbour sampling
// Layout (sampler_result.cuh:226-260,421-426): per seed, data holds
// length_per_sample = sum_h prod_{g<=h} fanout[g] vertex ids (fanout[0] = 1 is the seed
// itself); hop h starts at offsets[h]; the children of the vertex in slot s of hop h
// occupy slots s*fanout[h+1] .. of hop h+1.  sample_lengths per seed holds
// 1 + sum_{h=1}^{hops-2} ... one count per parent slot of every hop but the last:
// entry loff[h] + s is the number of children written for slot s of hop h.
// Per parent of degree deg and fanout k (src/offline_sample.cu:109-133): if k >= deg
// every neighbour is copied (count = deg), else k alias draws with replacement
// (count = k).  Draw i of the parent in slot s of hop h uses
//   r = Philox(seed; seed_index, s*k + i, h, DOM_SAMPLE); col = mulhi(r[0],deg); u24(r[1]) < prob[col]
// A parent with an invalid row (zero total weight) yields no children (CheckValid, offline_sample.cu:86).
// Slots that receive no vertex are not written.
// online != 0 rebuilds each parent's table from w with the sweep instead of reading prob/alias.
// distinct != 0 is the rule of the reference's online sampler (roll_atomic / roll_once, src/online_sample_new.cu:72-105:
// up to 11 rounds of draws, a candidate whose slot of the row is already selected is dropped, so a parent may end
// with fewer than k children), made sequential so that it does not depend on scheduling: draw i tries
//   r = Philox(seed; seed_index, s*k + i, h + 256 t, DOM_SAMPLE), t = 0..10
// and takes the first candidate slot that no earlier draw of this parent took; a draw whose 11 candidates were
// all taken yields nothing.  The children are written densely in the order of i.  Needs k <= 64 and hops <= 256.
constexpr uint32_t SAMPLE_ROUNDS = 11;
static int sample_impl(const uint32_t* xadj, uint32_t V, const uint32_t* adjncy, const float* w, const float* prob,
                       const uint32_t* alias, int online, int distinct, const uint32_t* seeds, uint32_t N,
                       const uint32_t* fanout, uint32_t hops, uint64_t seed, uint32_t* data, uint32_t* sample_lengths,
                       uint64_t* sampled) {
  if (distinct) {
    if (hops > 256) return -1;
    for (uint32_t h = 1; h < hops; ++h)
      if (fanout[h] > 64) return -1;
  }
  // fanout[0..hops-1], fanout[0] == 1
  std::vector<uint64_t> width(hops), off(hops), loff(hops);
  uint64_t lps = 0, slen = 0, wd = 1;
  for (uint32_t h = 0; h < hops; ++h) {
    wd *= fanout[h];
    width[h] = wd; off[h] = lps; lps += wd;
    if (h + 1 < hops) { loff[h] = slen; slen += wd; }
  }
  uint64_t total = 0;
#pragma omp parallel reduction(+ : total)
  {
    std::vector<float> rprob;
    std::vector<uint32_t> ralias, heavy;
    std::vector<double> pp;
    std::vector<uint8_t> filled, nfilled;
#pragma omp for schedule(dynamic, 16)
    for (int64_t si = 0; si < (int64_t)N; ++si) {
      uint32_t* d = data + (size_t)si * lps;
      uint32_t* sl = sample_lengths + (size_t)si * slen;
      for (uint64_t k = 0; k < slen; ++k) sl[k] = 0;
      d[0] = seeds[si];
      filled.assign(1, 1);
      for (uint32_t h = 0; h + 1 < hops; ++h) {
        const uint32_t k = fanout[h + 1];
        nfilled.assign(width[h + 1], 0);
        for (uint64_t s = 0; s < width[h]; ++s) {
          if (!filled[s]) continue;
          const uint32_t v = d[off[h] + s];
          if (v >= V) continue;  // a seed that does not exist has no children
          const uint32_t o = xadj[v], deg = xadj[v + 1] - o;
          if (deg == 0) continue;
          const float* pr = prob ? prob + o : nullptr;
          const uint32_t* al = alias ? alias + o : nullptr;
          if (online) {
            rprob.resize(deg); ralias.resize(deg);
            const float* wr = w + o;
            if (!alias_row_sweep(deg, [&](uint32_t i) { return wr[i]; }, rprob.data(), ralias.data(), pp, heavy))
              continue;
            pr = rprob.data(); al = ralias.data();
          } else if (al[0] == ORC_INVALID) {
            continue;
          }
          uint32_t cnt;
          uint32_t* out = d + off[h + 1] + s * k;
          if (k >= deg) {
            cnt = deg;
            for (uint32_t i = 0; i < deg; ++i) out[i] = adjncy[o + i];
          } else if (distinct) {
            uint32_t taken[64];
            cnt = 0;
            for (uint32_t i = 0; i < k; ++i)
              for (uint32_t t = 0; t < SAMPLE_ROUNDS; ++t) {
                uint32_t r[4];
                philox(seed, (uint32_t)si, (uint32_t)(s * k + i), h + 256u * t, DOM_SAMPLE, r);
                const uint32_t col = mulhi32(r[0], deg);
                const uint32_t cand = u24(r[1]) < pr[col] ? col : al[col];
                bool seen = false;
                for (uint32_t j = 0; j < cnt; ++j) seen = seen || taken[j] == cand;
                if (seen) continue;
                taken[cnt] = cand;
                out[cnt++] = adjncy[o + cand];
                break;
              }
          } else {
            cnt = k;
            for (uint32_t i = 0; i < k; ++i) {
              uint32_t r[4];
              philox(seed, (uint32_t)si, (uint32_t)(s * k + i), h, DOM_SAMPLE, r);
              const uint32_t col = mulhi32(r[0], deg);
              const uint32_t cand = u24(r[1]) < pr[col] ? col : al[col];
              out[i] = adjncy[o + cand];
            }
          }
          for (uint32_t i = 0; i < cnt; ++i) nfilled[s * k + i] = 1;
          sl[loff[h] + s] = cnt;
          total += cnt;
        }
        filled.swap(nfilled);
      }
    }
  }
  if (sampled) *sampled = total;
  return 0;
}

int orc_sample_offline(const uint32_t* xadj, uint32_t V, const uint32_t* adjncy, const float* prob, const uint32_t* alias,
                       const uint32_t* seeds, uint32_t N, const uint32_t* fanout, uint32_t hops, uint64_t seed,
                       uint32_t* data, uint32_t* sample_lengths, uint64_t* sampled) {
  return sample_impl(xadj, V, adjncy, nullptr, prob, alias, 0, 0, seeds, N, fanout, hops, seed, data, sample_lengths,
                     sampled);
}
int orc_sample_online(const uint32_t* xadj, uint32_t V, const uint32_t* adjncy, const float* w, const uint32_t* seeds, uint32_t N,
                      const uint32_t* fanout, uint32_t hops, uint64_t seed, uint32_t* data, uint32_t* sample_lengths,
                      uint64_t* sampled) {
  return sample_impl(xadj, V, adjncy, w, nullptr, nullptr, 1, 0, seeds, N, fanout, hops, seed, data, sample_lengths,
                     sampled);
}
// The same two with distinct children per parent (see sample_impl); -1 for a fanout above 64 or more than 256 hops.
int orc_sample_offline_distinct(const uint32_t* xadj, uint32_t V, const uint32_t* adjncy, const float* prob,
                                const uint32_t* alias, const uint32_t* seeds, uint32_t N, const uint32_t* fanout,
                                uint32_t hops, uint64_t seed, uint32_t* data, uint32_t* sample_lengths, uint64_t* sampled) {
  return sample_impl(xadj, V, adjncy, nullptr, prob, alias, 0, 1, seeds, N, fanout, hops, seed, data, sample_lengths,
                     sampled);
}
int orc_sample_online_distinct(const uint32_t* xadj, uint32_t V, const uint32_t* adjncy, const float* w,
                               const uint32_t* seeds, uint32_t N, const uint32_t* fanout, uint32_t hops, uint64_t seed,
                               uint32_t* data, uint32_t* sample_lengths, uint64_t* sampled) {
  return sample_impl(xadj, V, adjncy, w, nullptr, nullptr, 1, 1, seeds, N, fanout, hops, seed, data, sample_lengths,
                     sampled);
}

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

}  // extern "C"
