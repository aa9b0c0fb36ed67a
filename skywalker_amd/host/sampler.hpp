// Orchestration objects and host entry functions with the reference's names and calling
// conventions (include/sampler.cuh:43-529): Sampler, Sampler_new, Walker, and
//   float ConstructTable(Sampler&, uint ngpu = 1, uint index = 0)
//   float OfflineWalk(Walker&)            float OnlineWalkShMem(Walker&)   float OnlineWalkGMem(Walker&)
//   float OfflineSample(Sampler_new&)     float OnlineGBSampleNew(Sampler_new&)
// Each returns the elapsed seconds of its kernel region and sets sampled_edges; results stay
// in device memory.  Errors print file:line and exit, as the reference does.
#pragma once
#include <dlfcn.h>

#include <cstdint>
#include <cstring>
#include <vector>

#include "../../include/skywalker_bias.h"
#include "gpu_graph.hpp"

DECLARE_bool(itl);
DECLARE_bool(replica);
DECLARE_bool(printresult);
DECLARE_bool(node2vec);
DECLARE_bool(n2v_table);
DECLARE_double(p);
DECLARE_double(q);
DECLARE_double(tp);
DECLARE_int32(seed);
DECLARE_string(biasplugin);

// The reference links one bias plug-in into every executable (src/api/bias_*.cu, CMakeLists.txt:54-57,84-87).
// Here the plug-in is a shared library named at run time (--biasplugin); without one the built-in biases run.
struct BiasPluginLib {
  void* handle = nullptr;
  decltype(&sky_bias_name) name = nullptr;
  decltype(&sky_bias_last_error) last_error = nullptr;
  decltype(&sky_bias_build_all) build_all = nullptr;
  decltype(&sky_bias_walk_online) walk_online = nullptr;
  decltype(&sky_bias_sample_online) sample_online = nullptr;
  bool Load(const std::string& path) {
    handle = dlopen(path.c_str(), RTLD_NOW | RTLD_GLOBAL);
    if (!handle) {
      fprintf(stderr, "cannot load bias plug-in %s: %s\n", path.c_str(), dlerror());
      return false;
    }
    name = (decltype(name))dlsym(handle, "sky_bias_name");
    last_error = (decltype(last_error))dlsym(handle, "sky_bias_last_error");
    build_all = (decltype(build_all))dlsym(handle, "sky_bias_build_all");
    walk_online = (decltype(walk_online))dlsym(handle, "sky_bias_walk_online");
    sample_online = (decltype(sample_online))dlsym(handle, "sky_bias_sample_online");
    if (!name || !last_error || !build_all || !walk_online || !sample_online) {
      fprintf(stderr, "%s does not export the entry points of include/skywalker_bias.h\n", path.c_str());
      return false;
    }
    return true;
  }
};
inline BiasPluginLib& BiasPlugin() {
  static BiasPluginLib lib;
  return lib;
}
#define SKY_PLUGIN_CALL(call)                                                                              \
  do {                                                                                                     \
    int _status = (call);                                                                                  \
    if (_status != 0) {                                                                                    \
      const char* _m = BiasPlugin().last_error();                                                          \
      fprintf(stderr, "ERROR: %s:%d, error %d: %s\n", __FILE__, __LINE__, _status, _m[0] ? _m : sky_last_error()); \
      exit(_status < 0 ? -_status : _status);                                                              \
    }                                                                                                      \
  } while (0)

#define LOG(...)                                           \
  do {                                                     \
    if (FLAGS_v) {                                         \
      fprintf(stdout, "%s:%d HOST: ", __FILE__, __LINE__); \
      fprintf(stdout, __VA_ARGS__);                        \
    }                                                      \
  } while (0)

struct DeviceBuffer {
  void* ptr = nullptr;
  size_t bytes = 0;
  void Allocate(size_t n) {
    Free();
    SKY_RT_CALL(sky_device_malloc(n, &ptr));
    bytes = n;
  }
  void Free() {
    if (ptr) SKY_RT_CALL(sky_device_free(ptr));
    ptr = nullptr;
    bytes = 0;
  }
};

// Result of a walk: data[size * hop_num] walker-major, length[size] (include/sampler_result.cuh:456-612).
struct WalkResult {
  uint64_t size = 0;
  uint hop_num = 0;
  uint* data = nullptr;
  uint* length = nullptr;
  DeviceBuffer data_buf, length_buf, seed_buf;
  void init(uint _size, uint _hop_num, const uint* seeds) {
    size = _size;
    hop_num = _hop_num;
    data_buf.Allocate((size_t)size * hop_num * 4);
    length_buf.Allocate((size_t)size * 4);
    seed_buf.Allocate((size_t)size * 4);
    data = (uint*)data_buf.ptr;
    length = (uint*)length_buf.ptr;
    SKY_RT_CALL(sky_device_fill_u32(data, SKY_INVALID, (size_t)size * hop_num));
    SKY_RT_CALL(sky_memcpy_h2d(seed_buf.ptr, seeds, (size_t)size * 4));
  }
  void Free() {
    data_buf.Free();
    length_buf.Free();
    seed_buf.Free();
  }
  // First paths, in the format of Jobs_result<RW>::PrintResult (sampler_result.cuh:592-606).
  void PrintResult() const {
    const uint64_t n = size < 3 ? size : 3;
    std::vector<uint> d(n * hop_num), l(n);
    if (!n) return;
    SKY_RT_CALL(sky_memcpy_d2h(d.data(), data, d.size() * 4));
    SKY_RT_CALL(sky_memcpy_d2h(l.data(), length, l.size() * 4));
    for (uint64_t j = 0; j < n; ++j) {
      printf("\n%drd path len %u \n", (int)j, l[j]);
      for (uint i = 0; i < (l[j] < hop_num ? l[j] : hop_num); ++i) printf("%u \t", d[j * hop_num + i]);
      printf("\n");
    }
  }
};

// Result of k-hop sampling (include/sampler_result.cuh:150-454).
struct SampleResult {
  uint64_t size = 0;
  uint hop_num = 0;
  std::vector<uint> hops_h;
  uint64_t length_per_sample = 0, size_of_sample_lengths = 0;
  uint* data = nullptr;
  uint* sample_lengths = nullptr;
  DeviceBuffer data_buf, len_buf, seed_buf;
  void init(uint _size, uint _hop_num, const uint* _hops, const uint* seeds) {
    size = _size;
    hop_num = _hop_num;
    hops_h.assign(_hops, _hops + _hop_num);
    SKY_RT_CALL(sky_sample_layout(hops_h.data(), hop_num, &length_per_sample, &size_of_sample_lengths));
    data_buf.Allocate((size_t)size * length_per_sample * 4);
    len_buf.Allocate((size_t)size * size_of_sample_lengths * 4);
    seed_buf.Allocate((size_t)size * 4);
    data = (uint*)data_buf.ptr;
    sample_lengths = (uint*)len_buf.ptr;
    SKY_RT_CALL(sky_device_fill_u32(data, SKY_INVALID, (size_t)size * length_per_sample));
    SKY_RT_CALL(sky_memcpy_h2d(seed_buf.ptr, seeds, (size_t)size * 4));
  }
  void Free() {
    data_buf.Free();
    len_buf.Free();
    seed_buf.Free();
  }
  // First samples, in the format of Jobs_result<NS>::PrintResult (sampler_result.cuh:399-420).
  void PrintResult() const {
    if (hop_num < 2) return;
    const uint64_t n = size < 4 ? size : 4;
    if (!n) return;
    std::vector<uint> d(n * length_per_sample), l(n * size_of_sample_lengths);
    SKY_RT_CALL(sky_memcpy_d2h(d.data(), data, d.size() * 4));
    SKY_RT_CALL(sky_memcpy_d2h(l.data(), sample_lengths, l.size() * 4));
    for (uint64_t j = 0; j < n; ++j) {
      const uint* dj = d.data() + j * length_per_sample;
      const uint* lj = l.data() + j * size_of_sample_lengths;
      printf("\n%dth sample src: %u, 1-hop len: %u \n", (int)j, dj[0], lj[0]);
      printf("\t 1-hop : ");
      for (uint k = 0; k < (lj[0] < 30 ? lj[0] : 30); ++k) printf("%u \t", dj[1 + k]);
      printf("\n");
      if (hop_num < 3) continue;
      for (uint i = 0; i < lj[0]; ++i) {
        printf("\t %u th 2-hop [%u]: ", i, dj[1 + i]);
        for (uint k = 0; k < (lj[1 + i] < 30 ? lj[1 + i] : 30); ++k) printf("%u \t", dj[1 + hops_h[1] + k + i * hops_h[2]]);
        printf("\n");
      }
    }
  }
};

class Sampler {
 public:
  gpu_graph ggraph;
  uint num_seed = 0;
  std::vector<uint> seeds, hops;
  uint hop_num = 0;
  const sky_alias_entry* alias_table = nullptr;
  const int8_t* valid = nullptr;
  uint device_id = 0;
  size_t sampled_edges = 0;

  Sampler() {}
  Sampler(gpu_graph graph, uint _device_id = 0) : ggraph(graph), device_id(_device_id) {}
  // Seeds are dev_id + n * dev_num, i.e. 0..N-1 on one GPU (include/sampler.cuh:308-321).
  void SetSeed(uint _num_seed, uint _hop_num, uint* _hops, uint dev_num = 1, uint dev_id = 0) {
    num_seed = _num_seed;
    hop_num = _hop_num;
    hops.assign(_hops, _hops + _hop_num);
    seeds.resize(num_seed);
    for (uint n = 0; n < num_seed; ++n) seeds[n] = (FLAGS_replica ? n : dev_id + n * dev_num) % ggraph.vtx_num;
  }
  void InitFullForConstruction(uint = 1, uint = 0) {}  // the build takes every vertex; nothing to stage
  void Free(bool = false) {}                            // tables belong to the graph handle
};

class Sampler_new {
 public:
  gpu_graph ggraph;
  SampleResult result;
  uint num_seed = 0;
  uint device_id = 0;
  size_t sampled_edges = 0;
  Sampler_new() {}
  Sampler_new(Sampler& old) { *this = old; }
  Sampler_new& operator=(Sampler& old) {
    ggraph = old.ggraph;
    num_seed = old.num_seed;
    device_id = old.device_id;
    sampled_edges = old.sampled_edges;
    result.init(num_seed, old.hop_num, old.hops.data(), old.seeds.data());
    return *this;
  }
  void Free(bool = false) { result.Free(); }
};

class Walker {
 public:
  gpu_graph ggraph;
  uint num_seed = 0;
  WalkResult result;
  uint device_id = 0;
  size_t sampled_edges = 0;
  Walker(gpu_graph graph, uint _device_id = 0) : ggraph(graph), device_id(_device_id) {}
  Walker(Sampler& sampler) : ggraph(sampler.ggraph), device_id(sampler.device_id) {}
  void Free() { result.Free(); }
  // --itl: seeds dev_id + n * dev_num, else a contiguous block (include/sampler.cuh:494-503).
  void SetSeed(uint _num_seed, uint _hop_num, uint dev_num = 1, uint dev_id = 0) {
    num_seed = _num_seed;
    std::vector<uint> seeds(num_seed);
    for (uint n = 0; n < num_seed; ++n)
      seeds[n] = (FLAGS_itl ? dev_id + n * dev_num : n + dev_id * num_seed) % ggraph.vtx_num;
    result.init(num_seed, _hop_num, seeds.data());
  }
};

inline float ConstructTable(Sampler& sampler, uint ngpu = 1, uint index = 0) {
  LOG("%s\n", __FUNCTION__);
  (void)ngpu;
  (void)index;
  double sec = 0;
  if (BiasPlugin().handle)
    SKY_PLUGIN_CALL(BiasPlugin().build_all(sampler.ggraph.handle, (float)FLAGS_p, (float)FLAGS_q, &sec));
  else
    SKY_RT_CALL(sky_alias_build_all(sampler.ggraph.handle, &sec));
  sampler.ggraph.Refresh();
  sampler.alias_table = sampler.ggraph.alias_table;
  sampler.valid = sampler.ggraph.valid;
  LOG("Construct table time:\t%.6f\n", sec);
  return (float)sec;
}

// Table persistence (the reference has none: every run rebuilds).  File: "SKYTBL02", V, E, fingerprint (u64 each),
// then prob f32[E], alias u32[E], valid i8[V], little endian.  The fingerprint is FNV-1a over the graph's row
// offsets and edge weights: every R-MAT graph of one scale and edge factor has the same V and E, so those two
// alone would let the tables of another graph in.  sky_alias_upload checks the arrays themselves.
inline bool GraphFingerprint(const gpu_graph& g, uint64_t* out) {
  std::vector<uint32_t> xadj((size_t)g.vtx_num + 1);
  std::vector<float> w(g.edge_num);
  if (sky_graph_download(g.handle, xadj.data(), nullptr, w.data()) != 0) return false;
  uint64_t h = 1469598103934665603ull;
  auto mix = [&](const void* p, size_t bytes) {
    const unsigned char* b = static_cast<const unsigned char*>(p);
    for (size_t i = 0; i < bytes; ++i) h = (h ^ b[i]) * 1099511628211ull;
  };
  mix(xadj.data(), xadj.size() * 4);
  mix(w.data(), w.size() * 4);
  *out = h;
  return true;
}
inline bool SaveTable(Sampler& sampler, const std::string& path) {
  const uint64_t V = sampler.ggraph.vtx_num, E = sampler.ggraph.edge_num;
  uint64_t fp = 0;
  if (!GraphFingerprint(sampler.ggraph, &fp)) return false;
  std::vector<float> prob(E);
  std::vector<uint32_t> alias(E);
  std::vector<int8_t> valid(V);
  SKY_RT_CALL(sky_alias_download(sampler.ggraph.handle, prob.data(), alias.data(), valid.data()));
  FILE* f = fopen(path.c_str(), "wb");
  if (!f) return false;
  bool ok = fwrite("SKYTBL02", 1, 8, f) == 8 && fwrite(&V, 8, 1, f) == 1 && fwrite(&E, 8, 1, f) == 1 &&
            fwrite(&fp, 8, 1, f) == 1;
  ok = ok && fwrite(prob.data(), 4, E, f) == E && fwrite(alias.data(), 4, E, f) == E;
  ok = ok && fwrite(valid.data(), 1, V, f) == V;
  return fclose(f) == 0 && ok;
}
inline bool LoadTable(Sampler& sampler, const std::string& path) {
  const uint64_t V = sampler.ggraph.vtx_num, E = sampler.ggraph.edge_num;
  uint64_t fp = 0;
  if (!GraphFingerprint(sampler.ggraph, &fp)) return false;
  FILE* f = fopen(path.c_str(), "rb");
  if (!f) return false;
  char magic[8];
  uint64_t fv = 0, fe = 0, ffp = 0;
  bool ok = fread(magic, 1, 8, f) == 8 && !memcmp(magic, "SKYTBL02", 8) && fread(&fv, 8, 1, f) == 1 &&
            fread(&fe, 8, 1, f) == 1 && fread(&ffp, 8, 1, f) == 1 && fv == V && fe == E && ffp == fp;
  std::vector<float> prob(ok ? E : 0);
  std::vector<uint32_t> alias(ok ? E : 0);
  std::vector<int8_t> valid(ok ? V : 0);
  ok = ok && fread(prob.data(), 4, E, f) == E && fread(alias.data(), 4, E, f) == E && fread(valid.data(), 1, V, f) == V;
  ok = ok && fgetc(f) == EOF;  // nothing may follow
  fclose(f);
  if (!ok) return false;
  if (sky_alias_upload(sampler.ggraph.handle, prob.data(), alias.data(), valid.data()) != 0) {
    fprintf(stderr, "%s\n", sky_last_error());
    return false;  // a damaged table: an alias outside its row, a prob that is no probability
  }
  sampler.ggraph.Refresh();
  sampler.alias_table = sampler.ggraph.alias_table;
  sampler.valid = sampler.ggraph.valid;
  return true;
}

inline float walk_common(Walker& walker, bool online, const char* who) {
  LOG("%s\n", who);
  double sec = 0;
  uint64_t sampled = 0;
  const uint len = walker.result.hop_num - 1;
  const uint* seeds = (const uint*)walker.result.seed_buf.ptr;
  if (online && BiasPlugin().handle) {
    SKY_PLUGIN_CALL(BiasPlugin().walk_online(walker.ggraph.handle, (float)FLAGS_p, (float)FLAGS_q, seeds, walker.num_seed,
                                             len, (float)FLAGS_tp, (uint64_t)FLAGS_seed, walker.result.data,
                                             walker.result.length, &sampled, &sec));
  } else if (online) {
    SKY_RT_CALL(sky_walk_online(walker.ggraph.handle, !FLAGS_node2vec  ? SKY_BIAS_STATIC
                                : FLAGS_n2v_table ? SKY_BIAS_NODE2VEC
                                                  : SKY_BIAS_NODE2VEC_REJECT,
                                (float)FLAGS_p, (float)FLAGS_q, seeds, walker.num_seed, len, (float)FLAGS_tp,
                                (uint64_t)FLAGS_seed, walker.result.data, walker.result.length, &sampled, &sec));
  } else {
    SKY_RT_CALL(sky_walk_offline(walker.ggraph.handle, seeds, walker.num_seed, len, (float)FLAGS_tp,
                                 (uint64_t)FLAGS_seed, walker.result.data, walker.result.length, &sampled, &sec));
  }
  walker.sampled_edges = sampled;
  LOG("Device %d sampling time:\t%.6f ratio:\t %.2f MSEPS\n", 0, sec, (float)(sampled / sec / 1000000));
  LOG("sampled_edges %lu\n", (unsigned long)sampled);
  if (FLAGS_printresult) walker.result.PrintResult();
  return (float)sec;
}
inline float OfflineWalk(Walker& walker) { return walk_common(walker, false, "OfflineWalk"); }
inline float OnlineWalkShMem(Walker& walker) { return walk_common(walker, true, "OnlineWalkShMem"); }
// The reference's --gmem twin differs only in where its per-block queues live; there are no such queues here.
inline float OnlineWalkGMem(Walker& walker) { return walk_common(walker, true, "OnlineWalkGMem"); }

inline float sample_common(Sampler_new& sampler, bool online, const char* who) {
  LOG("%s\n", who);
  double sec = 0;
  uint64_t sampled = 0;
  const uint* seeds = (const uint*)sampler.result.seed_buf.ptr;
  if (online && BiasPlugin().handle) {
    SKY_PLUGIN_CALL(BiasPlugin().sample_online(sampler.ggraph.handle, (float)FLAGS_p, (float)FLAGS_q, seeds, sampler.num_seed,
                                               sampler.result.hops_h.data(), sampler.result.hop_num, (uint64_t)FLAGS_seed,
                                               sampler.result.data, sampler.result.sample_lengths, &sampled, &sec));
  } else if (online) {
    SKY_RT_CALL(sky_sample_online(sampler.ggraph.handle, seeds, sampler.num_seed, sampler.result.hops_h.data(),
                                  sampler.result.hop_num, (uint64_t)FLAGS_seed, sampler.result.data,
                                  sampler.result.sample_lengths, &sampled, &sec));
  } else {
    SKY_RT_CALL(sky_sample_offline(sampler.ggraph.handle, seeds, sampler.num_seed, sampler.result.hops_h.data(),
                                   sampler.result.hop_num, (uint64_t)FLAGS_seed, sampler.result.data,
                                   sampler.result.sample_lengths, &sampled, &sec));
  }
  sampler.sampled_edges = sampled;
  LOG("Device %d sampling time:\t%.2f ms ratio:\t %.1f MSEPS\n", 0, sec * 1000, (float)(sampled / sec / 1000000));
  LOG("sampled_edges %lu\n", (unsigned long)sampled);
  if (FLAGS_printresult) sampler.result.PrintResult();
  return (float)sec;
}
inline float OfflineSample(Sampler_new& sampler) { return sample_common(sampler, false, "OfflineSample"); }
inline float OnlineGBSampleNew(Sampler_new& sampler) { return sample_common(sampler, true, "OnlineGBSampleNew"); }
