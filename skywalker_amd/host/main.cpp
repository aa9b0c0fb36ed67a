// `skywalker`: the reference's command line (src/main.cu:32-109 flags, :111-421 flow and output)
// on top of libskywalker_hip.  One GPU; the flags of the multi-GPU and of the unified / host-mapped
// memory tiers are accepted and ignored so that the reference's scripts keep working.
#include <algorithm>
#include <cstdio>
#include <string>

#include "sampler.hpp"

DEFINE_string(input, "/home/pywang/data/lj.w.gr", "input");
DEFINE_int32(ngpu, 1, "number of GPUs ");
DEFINE_bool(s, true, "single run");
DEFINE_int32(n, 4000, "sample size");
DEFINE_int32(k, 2, "neightbor");
DEFINE_int32(d, 2, "depth");
DEFINE_double(hd, 1, "high degree ratio");
DEFINE_bool(ol, false, "online alias table building");
DEFINE_bool(rw, false, "Random walk specific");
DEFINE_bool(dw, false, "using degree as weight");
DEFINE_bool(randomweight, false, "generate random weight with range");
DEFINE_int32(weightrange, 2, "generate random weight with range from 0 to ");
DEFINE_bool(sage, false, "GraphSage");
DEFINE_bool(deepwalk, false, "deepwalk");
DEFINE_bool(node2vec, false, "node2vec");
DEFINE_bool(n2v_table, false, "node2vec: build the second-order table of every step instead of rejection sampling");
DEFINE_bool(ppr, false, "ppr");
DEFINE_double(p, 2.0, "hyper-parameter p for node2vec");
DEFINE_double(q, 0.5, "hyper-parameter q for node2vec");
DEFINE_double(tp, 0.0, "terminate probabiility");
DEFINE_bool(hmtable, false, "using host mapped mem for alias table");
DEFINE_bool(dt, true, "using duplicated table on each GPU");
DEFINE_bool(umgraph, true, "using UM for graph");
DEFINE_bool(hmgraph, false, "using host registered mem for graph");
DEFINE_bool(gmgraph, false, "using GPU mem for graph");
DEFINE_int32(gmid, 1, "using mem of GPU gmid for graph");
DEFINE_bool(umtable, false, "using UM for alias table");
DEFINE_bool(umresult, false, "using UM for result");
DEFINE_bool(umbuf, false, "using UM for global buffer");
DEFINE_bool(cache, false, "cache alias table for online");
DEFINE_bool(debug, false, "debug");
DEFINE_bool(bias, true, "biased or unbiased sampling");
DEFINE_bool(full, false, "sample over all node");
DEFINE_bool(stream, false, "streaming sample over all node");
DEFINE_bool(v, false, "verbose");
DEFINE_bool(printresult, false, "printresult");
DEFINE_bool(edgecut, true, "edgecut");
DEFINE_bool(itl, true, "interleave");
DEFINE_bool(twc, false, "using twc");
DEFINE_bool(static, true, "using static scheduling");
DEFINE_bool(buffer, false, "buffered write for memory (problem-prone)");
DEFINE_int32(m, 4, "block per sm");
DEFINE_bool(peritr, false, "invoke kernel for each itr");
DEFINE_bool(sp, false, "using spliced buffer");
DEFINE_bool(pf, true, "using UM prefetching");
DEFINE_bool(ab, true, "using UM AB hint");
DEFINE_double(pfr, 1.0, "UM prefetching ratio");
DEFINE_bool(async, false, "using async execution");
DEFINE_bool(replica, false, "same task for all gpus");
DEFINE_bool(built, false, "has built table");
DEFINE_string(savetable, "", "write the alias tables to this file after building them");
DEFINE_string(loadtable, "", "read the alias tables from this file instead of building them");
DEFINE_bool(gmem, false, "do not use shmem as buffer");
DEFINE_bool(newsampler, true, "use new sampler");
DEFINE_bool(csv, false, "CSV output");
// defined by the bias plugin in the reference (src/api/bias_static.cu:9, bias_node2vec.cu:11)
DEFINE_bool(weight, true, "load edge weight from file");
// new here: the bias operator as a shared library (include/skywalker_bias.h) instead of a link-time choice
DEFINE_string(biasplugin, "", "bias plug-in library, e.g. libskywalker_bias_degree.so (default: built-in static / node2vec bias)");
// new here: the reference's online sampler never takes a slot of a row twice (roll_once, online_sample_new.cu:83-105),
// its offline sampler may; here one flag selects the rule for both
DEFINE_bool(replace, true, "k-hop sampling draws with replacement; 0: distinct neighbours (fanouts of at most 64)");
// new here: key of the Philox streams (the reference seeds cuRAND with the thread id)
DEFINE_int32(seed, 0, "Philox seed of the samplers");

int main(int argc, char* argv[]) {
  // an explicit --d on the command line wins over the app presets (the reference overwrites it)
  bool d_given = false;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    if (a == "--d" || a == "-d" || a.rfind("--d=", 0) == 0 || a.rfind("-d=", 0) == 0) d_given = true;
  }
  if (skyflags::ParseCommandLineFlags(&argc, &argv)) return 1;
  if (FLAGS_ngpu != 1) {
    fprintf(stderr, "skywalker: this build runs on one GPU; --ngpu %d is not supported\n", FLAGS_ngpu);
    return 1;
  }
  if (FLAGS_node2vec || FLAGS_deepwalk || FLAGS_ppr) {
    FLAGS_rw = true;
    FLAGS_k = 1;
    if (!d_given) FLAGS_d = 100;
    if (FLAGS_ppr) FLAGS_tp = 0.15;
  }
  if (FLAGS_sage) {
    FLAGS_rw = false;
    FLAGS_d = 2;
  }
  if (!FLAGS_bias) {
    FLAGS_weight = false;
    FLAGS_randomweight = false;
  }
  if (!FLAGS_biasplugin.empty() && !BiasPlugin().Load(FLAGS_biasplugin)) return 1;
  if (FLAGS_node2vec && !FLAGS_ol) {
    LOG("node2vec is second-order: switching to --ol=1\n");
    FLAGS_ol = true;
  }
  // the reference takes these as they come (a negative depth indexes hops out of bounds, main.cu:177-186)
  if (FLAGS_d < 1 || FLAGS_k < 1 || FLAGS_n < 0) {
    fprintf(stderr, "skywalker: need --d >= 1, --k >= 1 and -n >= 0 (got d=%d k=%d n=%d)\n", FLAGS_d, FLAGS_k, FLAGS_n);
    return 1;
  }
  if (!(FLAGS_tp >= 0.0 && FLAGS_tp <= 1.0) || !(FLAGS_p > 0.0) || !(FLAGS_q > 0.0)) {
    fprintf(stderr, "skywalker: need 0 <= --tp <= 1, --p > 0 and --q > 0\n");
    return 1;
  }
  if (!FLAGS_replace && sky_set_option("sample_distinct", 1) != SKY_OK) {
    fprintf(stderr, "skywalker: %s\n", sky_last_error());
    return 1;
  }
  int sample_size = FLAGS_n;
  const int NeighborSize = FLAGS_k, Depth = FLAGS_d;
  std::vector<uint> hops(Depth + 1, (uint)NeighborSize);
  hops[0] = 1;
  if (FLAGS_sage) {
    hops[1] = 25;
    hops[2] = 10;
  }
  Graph* ginst = new Graph();
  if (!ginst->ok) return 1;
  if (ginst->numNode == 0) {  // start vertices are taken modulo the vertex count
    fprintf(stderr, "skywalker: %s has no vertices\n", FLAGS_input.c_str());
    return 1;
  }
  if (FLAGS_full && !FLAGS_stream) {
    sample_size = (int)ginst->numNode;
    FLAGS_n = sample_size;
  }
  gpu_graph ggraph(ginst, 0);
  Sampler sampler(ggraph, 0);
  Sampler_new sampler_new;
  float time = 0, table_time = 0;
  size_t sampled = 0;
  // unbiased runs go through the same tables with every weight equal to 1
  const bool online = FLAGS_ol;
  if (!online) {
    sampler.InitFullForConstruction(1, 0);
    if (!FLAGS_loadtable.empty()) {
      if (!LoadTable(sampler, FLAGS_loadtable)) {
        fprintf(stderr, "cannot use table file %s (missing, damaged, or of another graph)\n", FLAGS_loadtable.c_str());
        return 1;
      }
    } else {
      table_time = ConstructTable(sampler, 1, 0) * 1000;
      LOG("Max construction time with %u gpu \t%.2f ms\n", 1, table_time);
    }
    if (!FLAGS_savetable.empty() && !SaveTable(sampler, FLAGS_savetable)) {
      fprintf(stderr, "cannot write table file %s\n", FLAGS_savetable.c_str());
      return 1;
    }
    FLAGS_built = true;
  }
  if (!FLAGS_rw) {
    sampler.SetSeed(sample_size, Depth + 1, hops.data(), 1, 0);
    sampler_new = sampler;
    time = online ? OnlineGBSampleNew(sampler_new) : OfflineSample(sampler_new);
    sampled = sampler_new.sampled_edges;
    sampler_new.Free();
  } else {
    Walker walker(sampler);
    walker.SetSeed(sample_size, Depth + 1, 1, 0);
    if (online)
      time = FLAGS_gmem ? OnlineWalkGMem(walker) : OnlineWalkShMem(walker);
    else
      time = OfflineWalk(walker);
    sampled = walker.sampled_edges;
    walker.Free();
  }
  ggraph.Free();
  const float ms = time * 1000, tp = sampled / time / 1000000;
  const bool show_table = !FLAGS_ol && FLAGS_bias;
  if (FLAGS_csv) {
    if (show_table) printf("%0.2f,\t", table_time);
    printf("%0.2f,\t", ms);
    printf("%0.2f,\n", tp);
  } else {
    if (show_table) printf("%0.2f\t", table_time);
    printf("\n");
    printf("%0.2f\t", ms);
    printf("\n");
    printf("%0.2f\t", tp);
    printf("\n");
  }
  return 0;
}
