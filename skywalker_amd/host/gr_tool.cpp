// gr_tool: checks the flag parser and the Galois .gr reader on the CPU (no GPU needed).
//   gr_tool info <file.gr>            prints "V E maxdeg sum(adjncy) sum(weights)"
//   gr_tool flags <args...>           parses the arguments and prints a few flags
#include <cstdio>
#include <string>

#include "graph.hpp"

DEFINE_string(input, "", "input");
DEFINE_bool(v, false, "verbose");
DEFINE_bool(csv, false, "CSV output");
DEFINE_bool(bias, true, "biased or unbiased sampling");
DEFINE_bool(weight, true, "load edge weight from file");
DEFINE_bool(randomweight, false, "generate random weight with range");
DEFINE_int32(weightrange, 2, "generate random weight with range from 0 to ");
DEFINE_bool(dw, false, "using degree as weight");
DEFINE_int32(n, 4000, "sample size");
DEFINE_double(tp, 0.0, "terminate probabiility");
DEFINE_bool(ol, false, "online alias table building");

int main(int argc, char** argv) {
  if (argc < 2) return 2;
  const std::string mode = argv[1];
  if (mode == "info" && argc >= 3) {
    FLAGS_csv = true;
    Graph g(argv[2]);
    if (!g.ok) return 1;
    unsigned long long sa = 0;
    double sw = 0;
    for (auto a : g.adjncy) sa += a;
    for (auto w : g.adjwgt) sw += w;
    printf("\n%lu %lu %u %llu %.1f\n", (unsigned long)g.numNode, (unsigned long)g.numEdge, g.MaxDegree, sa, sw);
    return 0;
  }
  if (mode == "flags") {
    int ac = argc - 1;
    char** av = argv + 1;
    if (skyflags::ParseCommandLineFlags(&ac, &av)) return 1;
    printf("input=%s n=%d tp=%g ol=%d bias=%d v=%d\n", FLAGS_input.c_str(), FLAGS_n, FLAGS_tp, (int)FLAGS_ol,
           (int)FLAGS_bias, (int)FLAGS_v);
    return 0;
  }
  return 2;
}
