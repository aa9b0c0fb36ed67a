// Host graph: Galois .gr (version 1) reader and writer with the reference's weight options
// (include/graph.cuh:164-327).  File layout: 4 x u64 header {version = 1, sizeof(edge data), V, E};
// V x u64 row END offsets; E x u32 destinations; 4 bytes of padding when E is odd; E x u32 edge data
// (weights, converted to float).
#pragma once
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "flags.hpp"

typedef unsigned int uint;
typedef uint edge_t;
typedef uint vtx_t;
typedef float weight_t;

DECLARE_string(input);
DECLARE_bool(v);
DECLARE_bool(csv);
DECLARE_bool(bias);
DECLARE_bool(weight);
DECLARE_bool(randomweight);
DECLARE_int32(weightrange);
DECLARE_bool(dw);

class Graph {
 public:
  std::string graphFilePath;
  uint64_t numNode = 0, numEdge = 0, sizeEdgeTy = 0;
  std::vector<edge_t> xadj;
  std::vector<vtx_t> adjncy;
  std::vector<weight_t> adjwgt;  // empty when the run is unbiased: every edge then weighs 1
  std::vector<uint> outDegree;
  uint MaxDegree = 0;
  bool weighted = false, ok = false;

  Graph() {
    graphFilePath = FLAGS_input;
    ok = ReadGraphGR();
  }
  explicit Graph(const std::string& path) : graphFilePath(path) { ok = ReadGraphGR(); }

  bool ReadGraphGR() {
    FILE* f = fopen(graphFilePath.c_str(), "rb");
    if (!f) {
      fprintf(stderr, "ReadGraphGR: cannot open %s\n", graphFilePath.c_str());
      return false;
    }
    uint64_t hdr[4];
    if (fread(hdr, 8, 4, f) != 4) {
      fprintf(stderr, "Unable to read header\n");
      fclose(f);
      return false;
    }
    if (hdr[0] != 1) fprintf(stderr, "Unknown file version\n");
    sizeEdgeTy = hdr[1];
    numNode = hdr[2];
    numEdge = hdr[3];
    if (numNode >= 0xFFFFFFFFull || numEdge >= 0xFFFFFFFFull) {
      fprintf(stderr, "ReadGraphGR: graph does not fit 32-bit offsets\n");
      fclose(f);
      return false;
    }
    if (FLAGS_v) {
      printf("%s has %lu nodes and %lu  edges\n", graphFilePath.c_str(), (unsigned long)numNode,
             (unsigned long)numEdge);
    } else {
      const std::string token = graphFilePath.substr(graphFilePath.rfind('/') + 1);
      printf(FLAGS_csv ? "%s," : "%s\n", token.c_str());
    }
    xadj.assign(numNode + 1, 0);
    std::vector<uint64_t> ends(numNode);
    if (fread(ends.data(), 8, numNode, f) != numNode) {
      fprintf(stderr, "Error: Partial read of node data\n");
      fclose(f);
      return false;
    }
    for (uint64_t i = 0; i < numNode; ++i) xadj[i + 1] = (edge_t)ends[i];
    adjncy.resize(numEdge);
    if (fread(adjncy.data(), 4, numEdge, f) != numEdge) {
      fprintf(stderr, "Error: Partial read of edge destinations\n");
      fclose(f);
      return false;
    }
    outDegree.resize(numNode);
    for (uint64_t i = 0; i < numNode; ++i) outDegree[i] = xadj[i + 1] - xadj[i];
    MaxDegree = numNode ? *std::max_element(outDegree.begin(), outDegree.end()) : 0;
    if (FLAGS_bias && (FLAGS_weight || FLAGS_randomweight)) {
      adjwgt.resize(numEdge);
      if (!sizeEdgeTy || FLAGS_randomweight) {
        printf("generating random weight\n");
        srand(0u);
        for (uint64_t i = 0; i < numEdge; ++i)
          adjwgt[i] = static_cast<float>(rand()) / (static_cast<float>(RAND_MAX / FLAGS_weightrange));
      } else {
        if (numEdge % 2) fseek(f, 4, SEEK_CUR);
        std::vector<uint> tmp(numEdge);
        if (fread(tmp.data(), 4, numEdge, f) != numEdge) {
          fprintf(stderr, "Error: Partial read of edge data\n");
          fclose(f);
          return false;
        }
        if (!FLAGS_dw) {
          for (uint64_t i = 0; i < numEdge; ++i) adjwgt[i] = static_cast<float>(tmp[i]);
        } else {
          for (uint64_t v = 0; v < numNode; ++v)
            for (uint64_t j = xadj[v]; j < xadj[v + 1]; ++j) adjwgt[j] = static_cast<float>(outDegree[v]);
        }
        weighted = true;
      }
    }
    fclose(f);
    // node2vec's membership test needs rows sorted by neighbour id (include/gpu_graph.cuh:204-238)
    return true;
  }

  static bool WriteGraphGR(const std::string& path, const std::vector<edge_t>& xadj, const std::vector<vtx_t>& adjncy,
                           const std::vector<uint>& weights) {
    FILE* f = fopen(path.c_str(), "wb");
    if (!f) return false;
    const uint64_t V = xadj.size() - 1, E = adjncy.size();
    uint64_t hdr[4] = {1, weights.empty() ? 0u : 4u, V, E};
    fwrite(hdr, 8, 4, f);
    for (uint64_t i = 0; i < V; ++i) {
      uint64_t e = xadj[i + 1];
      fwrite(&e, 8, 1, f);
    }
    fwrite(adjncy.data(), 4, E, f);
    if (!weights.empty()) {
      if (E % 2) {
        uint pad = 0;
        fwrite(&pad, 4, 1, f);
      }
      fwrite(weights.data(), 4, E, f);
    }
    fclose(f);
    return true;
  }
};
