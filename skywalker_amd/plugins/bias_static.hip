// Static bias: the weight of an edge is the weight stored with it (src/api/bias_static.cu:12-14; the reference
// indexes adjwgt with the neighbour's vertex id, here it is the edge's own slot).
#include "../../include/skywalker_bias.h"

__device__ float sky_get_bias(const sky_row_view* row, uint32_t slot, uint32_t, const sky_walker_state*) {
  return row->adjwgt[row->off + slot];
}
__device__ void sky_update_walker_state(sky_walker_state*, uint32_t) {}

extern "C" const char* sky_bias_name(void) { return "static"; }
