// node2vec second-order bias (src/api/bias_node2vec.cu:15-27): the edge weight divided by p when the edge leads
// back to the vertex the walker came from, kept when it leads to a neighbour of that vertex, divided by q otherwise.
#include "../../include/skywalker_bias.h"

__device__ float sky_get_bias(const sky_row_view* row, uint32_t slot, uint32_t dst, const sky_walker_state* st) {
  const float w = row->adjwgt[row->off + slot];
  if (!st->has_last) return w;
  if (st->last == dst) return __fdiv_rn(w, st->p);
  if (sky_connected(row, st->last, dst)) return w;
  return __fdiv_rn(w, st->q);
}
// the engine keeps st->last; nothing else to remember (the reference's plug-in stores it itself, :24-26)
__device__ void sky_update_walker_state(sky_walker_state*, uint32_t) {}

extern "C" const char* sky_bias_name(void) { return "node2vec"; }
