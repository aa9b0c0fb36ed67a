/*
 * Bias operator of libskywalker_hip: the user-supplied weight of an edge, evaluated on the device.
 *
 * In the reference the bias is a link-time plug-in: exactly one src/api/bias_*.cu per executable defines
 *   __device__ float gpu_graph::getBias(edge_t dst, uint src, uint idx)     (include/gpu_graph.cuh:189)
 *   __device__ void  gpu_graph::UpdateWalkerState(uint idx, uint info)      (include/gpu_graph.cuh:255)
 * and CMake builds one program per plug-in (CMakeLists.txt:54-57,84-87).  Here a plug-in is one HIP source
 * file that defines the two device functions below.  It is compiled with -fgpu-rdc and linked with
 * skywalker_amd/csrc/sky_bias_engine.hip into one shared library per plug-in (skywalker_amd/build.py,
 * build_plugins): libskywalker_bias_<name>.so, which exports the three host entry points at the end of this
 * file and works on graphs of libskywalker_hip.so.  The enum sky_bias of skywalker_hip.h stays as the fast path
 * for the two biases the reference ships kernels for.
 *
 * Shipped plug-ins (skywalker_amd/plugins): bias_static.hip (src/api/bias_static.cu:12-14),
 * bias_node2vec.hip (src/api/bias_node2vec.cu:15-27), bias_degree.hip (src/api/bias_degree.cu:12-16).
 */
#ifndef SKYWALKER_BIAS_H_
#define SKYWALKER_BIAS_H_

#include <stdint.h>

#include "skywalker_hip.h"

/* The row a weight is asked for, and the graph around it (device pointers). */
typedef struct sky_row_view {
  const uint32_t* xadj;   /* [V+1] */
  const uint32_t* adjncy; /* [E], rows sorted by neighbour id */
  const float* adjwgt;    /* [E] */
  uint32_t V;
  uint32_t src;           /* the vertex whose row this is */
  uint32_t off, deg;      /* its first CSR slot and its degree */
} sky_row_view;

/* Per-walker state, the reference's sample_result::state[idx] (include/sampler_result.cuh).  has_last == 0 until
 * the walker has left its first vertex, and in table builds that are not tied to a walker. */
typedef struct sky_walker_state {
  uint32_t last;     /* vertex visited before the current one */
  uint32_t has_last;
  uint32_t walker;   /* index of the walker in its batch */
  float p, q;        /* hyper-parameters of the call */
  uint32_t user[2];  /* free for the plug-in */
} sky_walker_state;

#if defined(__HIPCC__)
/* Weight of the edge in CSR slot row->off + slot, which leads to vertex dst; replaces gpu_graph::getBias.
 * Must be a pure function of its arguments.  Values that are not positive finite numbers count as 0. */
__device__ float sky_get_bias(const sky_row_view* row, uint32_t slot, uint32_t dst, const sky_walker_state* st);
/* Called once per step, after the draw, with the vertex the walker leaves; replaces gpu_graph::UpdateWalkerState.
 * The engine has already stored that vertex in st->last. */
__device__ void sky_update_walker_state(sky_walker_state* st, uint32_t left);

/* gpu_graph::CheckConnect (include/gpu_graph.cuh:204-238): whether b is a neighbour of a. */
__device__ inline bool sky_connected(const sky_row_view* row, uint32_t a, uint32_t b) {
  const uint32_t* r = row->adjncy + row->xadj[a];
  uint32_t lo = 0, n = row->xadj[a + 1] - row->xadj[a];
  while (n > 0) {
    const uint32_t half = n >> 1;
    const uint32_t x = r[lo + half];
    if (x == b) return true;
    if (x < b) {
      lo += half + 1;
      n -= half + 1;
    } else {
      n = half;
    }
  }
  return false;
}
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* ---- what every plug-in library exports (host side) ---- */
const char* sky_bias_name(void);
const char* sky_bias_last_error(void); /* message of the last failure inside the plug-in library on this thread */
/* ConstructTable under the operator (src/createTable.cu:119-179 calls getBias through the constructors): the weight
 * of every slot is evaluated with a walker state whose has_last is 0, the tables of all vertices are built from
 * those weights by libskywalker_hip and stay in the graph for sky_walk_offline / sky_sample_offline. */
int sky_bias_build_all(sky_graph* g, float p, float q, double* seconds);
/* OnlineWalkShMem under the operator (src/online_walk.cu:97-132): every (walker, step) draws from the table of the
 * current vertex under the walker's state; arguments as sky_walk_online. */
int sky_bias_walk_online(sky_graph* g, float p, float q, const uint32_t* seeds_device, uint32_t N, uint32_t len,
                         float stop_prob, uint64_t philox_seed, uint32_t* paths_device, uint32_t* lengths_device,
                         uint64_t* sampled, double* seconds);

/* OnlineGBSampleNew under the operator (src/online_sample_new.cu:459-547; its constructors ask getBias for every
 * weight of every frontier row, include/alias_table_new.cuh:1090-1091): hop by hop, the operator is evaluated for
 * the rows of the distinct frontier vertices alone (walker state with has_last 0), their tables are built from those
 * weights by libskywalker_hip, and the hop is drawn; arguments as sky_sample_online. */
int sky_bias_sample_online(sky_graph* g, float p, float q, const uint32_t* seeds_device, uint32_t N,
                           const uint32_t* fanout, uint32_t hops, uint64_t philox_seed, uint32_t* data_device,
                           uint32_t* sample_lengths_device, uint64_t* sampled, double* seconds);

#ifdef __cplusplus
}
#endif
#endif /* SKYWALKER_BIAS_H_ */
