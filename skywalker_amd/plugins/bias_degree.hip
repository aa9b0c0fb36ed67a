// Degree bias (src/api/bias_degree.cu:12-16): an edge weighs as much as its end vertex has out-edges.
#include "../../include/skywalker_bias.h"

__device__ float sky_get_bias(const sky_row_view* row, uint32_t, uint32_t dst, const sky_walker_state*) {
  return (float)(row->xadj[dst + 1] - row->xadj[dst]);
}
__device__ void sky_update_walker_state(sky_walker_state*, uint32_t) {}

extern "C" const char* sky_bias_name(void) { return "degree"; }
