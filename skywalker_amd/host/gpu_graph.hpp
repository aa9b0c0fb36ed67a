// Device graph object with the reference's name and fields (include/gpu_graph.cuh:32-117,164-177),
// backed by a sky_graph handle of libskywalker_hip.  Everything is resident in HBM: the reference's
// unified / host-mapped placements (--umgraph, --hmgraph, --gmgraph) are accepted and ignored.
#pragma once
#include <cstdio>
#include <cstdlib>

#include "../../include/skywalker_hip.h"
#include "graph.hpp"

// Print-and-exit error policy of the reference (CUDA_RT_CALL, include/util.cuh:112-124).
#define SKY_RT_CALL(call)                                                                      \
  do {                                                                                         \
    int _status = (call);                                                                      \
    if (_status != 0) {                                                                        \
      fprintf(stderr, "ERROR: %s:%d, error %d: %s\n", __FILE__, __LINE__, _status, sky_last_error()); \
      exit(_status < 0 ? -_status : _status);                                                  \
    }                                                                                          \
  } while (0)

class gpu_graph {
 public:
  sky_graph* handle = nullptr;
  const vtx_t* adjncy = nullptr;
  const weight_t* adjwgt = nullptr;
  const edge_t* xadj = nullptr;
  const sky_alias_entry* alias_table = nullptr;  // {prob, alias} per CSR slot (the reference's prob_array / alias_array)
  const int8_t* valid = nullptr;
  edge_t vtx_num = 0, edge_num = 0, avg_degree = 0;
  uint MaxDegree = 0, device_id = 0;
  uint local_vtx_offset = 0, local_edge_offset = 0, local_vtx_num = 0, local_edge_num = 0;

  gpu_graph() {}
  gpu_graph(Graph* ginst, uint _device_id = 0) : device_id(_device_id) {
    vtx_num = (edge_t)ginst->numNode;
    edge_num = (edge_t)ginst->numEdge;
    avg_degree = vtx_num ? edge_num / vtx_num : 0;
    SKY_RT_CALL(sky_graph_upload(ginst->xadj.data(), ginst->adjncy.data(),
                                 ginst->adjwgt.empty() ? nullptr : ginst->adjwgt.data(), vtx_num, edge_num, &handle));
    MaxDegree = ginst->MaxDegree;
    local_vtx_num = vtx_num;
    local_edge_num = edge_num;
    Refresh();
  }
  // Re-reads the device addresses after the library allocated tables.
  void Refresh() {
    SKY_RT_CALL(sky_graph_device_ptrs(handle, &xadj, &adjncy, &adjwgt, &alias_table, &valid));
  }
  void Free() {
    if (handle) SKY_RT_CALL(sky_graph_free(handle));
    handle = nullptr;
  }
};
