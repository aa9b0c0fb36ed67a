// Internal definition of the opaque sky_graph handle.
#pragma once
#include <vector>

#include "sky_common.h"

// The tuning knobs of sky_set_option / sky_graph_set_option.  A graph reads a knob through option(g, ...): its own
// value when sky_graph_set_option has given it one, the process-wide value otherwise.
enum SkyOpt : int {
  OPT_TILED_MAX_TILES = 0,
  OPT_ROW_MERGE,
  OPT_STREAM_MIN_EDGES,
  OPT_STREAM_WIDE_MIN_EDGES,
  OPT_WALK_READ_ONCE,
  OPT_SAMPLE_DISTINCT,
  OPT_SMALL_IN_PLACE,
  OPT_BUILD_STREAMS,
  OPT_BUILD_PROFILE,
  OPT_WALK_COMPACT_EVERY,
  OPT_ONLINE_FULL_BUILD,
  OPT_ONLINE_DEVICE_SIZED,
  OPT_COUNT
};

struct sky_graph {
  uint32_t V = 0, E = 0, max_degree = 0;
  long long opt_value[OPT_COUNT] = {0};
  bool opt_own[OPT_COUNT] = {false};  // the graph has a value of its own for the knob
  // scratch memory of the table builds on this graph (allocated on first use, reused by every later build, freed
  // with the graph): row lists and counters of the binning pass, and the arrays of the tile-parallel path
  void* build_scratch = nullptr;
  void* tiled_scratch = nullptr;
  int device = 0;  // the device that was current when the graph was created: its arrays live there
  // CSR, device resident.  Arrays are allocated with 16 spare bytes so that kernels may
  // read whole aligned float4/uint4 quads that straddle the end.
  uint32_t* xadj = nullptr;    // [V+1]
  uint32_t* adjncy = nullptr;  // [E]
  float* adjwgt = nullptr;     // [E]
  // padded copy of a caller's weight array (sky_alias_build_from_weights) whose allocation has no spare bytes
  float* wgt_copy = nullptr;
  size_t wgt_copy_cap = 0;
  // alias table: entry i belongs to CSR slot i; alias holds a row-local index
  sky::AliasEntry* table = nullptr;  // [E] {prob, alias}
  int8_t* valid = nullptr;    // [V]
  bool has_tables = false;
  // optional walk index: one 16-byte entry per CSR slot that also holds the two neighbour ids a draw can
  // lead to; null unless sky_walk_index_build has run since the tables were last written
  sky::WalkEntry* walk_index = nullptr;  // [E] storage, kept once allocated
  bool has_walk_index = false;           // its contents match the tables
  hipStream_t stream = nullptr;  // null stream, like the reference ("0 stream everywhere")

  struct ProfileEntry {
    const char* name;
    float ms;
    uint64_t edges;
  };
  std::vector<ProfileEntry> build_profile;

  // Device buffers that calls on this graph reuse instead of allocating each time (they only grow), and the two
  // events that bracket a call's kernel region.
  enum PoolSlot { POOL_COUNTERS = 0, POOL_BITMAP, POOL_LIST, POOL_SLOTS };
  struct PoolBuf {
    void* p = nullptr;
    size_t cap = 0;
  };
  PoolBuf pool[POOL_SLOTS];
  hipEvent_t ev[2] = {nullptr, nullptr};
  // Pinned host words into which the device reports, step by step, how many walkers of an online walk still walk;
  // the host reads them without waiting (they lag behind the enqueued steps) to stop enqueuing once none does.
  uint32_t* live_report = nullptr;
  size_t live_report_cap = 0;
  // Side streams (default priority) over which a small build spreads its class kernels, the event they wait for
  // and the events the graph's stream waits for afterwards; created on first use.
  static constexpr int SIDE_STREAMS = 3;
  hipStream_t side[SIDE_STREAMS] = {nullptr, nullptr, nullptr};
  hipEvent_t fork_ev = nullptr;
  hipEvent_t join_ev[SIDE_STREAMS] = {nullptr, nullptr, nullptr};

  // Class sizes of the last binning of all vertices.  They depend on xadj alone, which never changes, so a
  // later build of all vertices sizes its launches from them without waiting for the device.
  bool bin_known = false;
  int bin_listed_from = 0;  // first class that the binning pass behind these sizes gave a list
  uint32_t bin_counts[32] = {0};
  unsigned long long bin_edges[32] = {0};
};

namespace sky {

// Degree classes of the offline build.  Upper bounds are inclusive.
enum BuildClass : int {
  CLS_EMPTY = 0,    // deg 0            handled while binning
  CLS_TINY = 1,     // deg 1..2         one lane per vertex, handled while binning
  CLS_G2 = 2,       // deg 3..8         2 lanes per row, 4 slots per lane
  CLS_G4 = 3,       // deg <= 16        4 lanes
  CLS_G8 = 4,       // deg <= 32        8 lanes
  CLS_G16 = 5,      // deg <= 64        16 lanes
  CLS_G32 = 6,      // deg <= 128       32 lanes
  CLS_G32X = 7,     // deg 161..192     32 lanes, 6 slots per lane
  CLS_LDS_W1 = 8,   // deg <= 253       one wavefront per row, 4 slots per lane
  CLS_LDS_W2 = 9,   // deg 382..509     one wavefront per row, 8 slots per lane
  CLS_MW2 = 10,     // deg 766.. for nw = 2, then <= 512 * nw - 3, nw = 2..10 (class CLS_MW2 + nw - 2, up to 18): one workgroup per row whose
                    //                  threads cover 512 * nw slots (the numbers 22..24 are not used)
  CLS_LDS_W6 = 19,  // deg 254..381     one wavefront per row, 6 slots per lane (the lower half of what CLS_LDS_W2 would hold)
  CLS_MW2_6 = 20,   // deg 510..765     two wavefronts per row, 6 slots per lane (the lower half of what CLS_MW2 would hold)
  CLS_HOLD = 21,         // deg 5118..8189     one workgroup holds the row in registers, its heavies in LDS
  CLS_STREAM = 25,       // deg 24577..65533   one workgroup streams the row, a window of its heavies stays in LDS.
  CLS_STREAM_LAST = 26,  // deg 8190..24576    Three classes built by one launch that takes the longest rows first
  CLS_STREAM_WIDE = 27,  // deg 65534..524287  and so
                    //                  does not end on its longest rows
  CLS_HUGE = 28,    // above            built tile by tile by the whole GPU
  CLS_G32S = 29,    // deg 129..160     32 lanes, 5 slots per lane (the lower half of what CLS_G32X would hold;
                    //                  3 slots per lane for rows of 33..48 entries gained nothing over CLS_G16)
  CLS_COUNT = 30
};

// One listed row of a degree class: the build kernels read where the row lies from the list itself
// instead of chasing xadj[v] after the list entry (one dependent global load less at every row start).
struct RowRef {
  uint32_t v, off, d, pad;
};

// Sequence of HIP events on one stream; consecutive marks bracket one kernel (or group).
struct EventTimer {
  hipStream_t stream;
  std::vector<hipEvent_t> ev;
  std::vector<const char*> names;
  std::vector<uint64_t> edges;
  hipEvent_t* pooled = nullptr;  // events that exist already are used first and are not destroyed
  size_t npooled = 0;
  explicit EventTimer(hipStream_t s) : stream(s) {}
  EventTimer(sky_graph* g);  // on the graph's stream, with the graph's two events for the first two marks
  ~EventTimer();
  int mark(const char* name, uint64_t edges);
  // synchronises, then fills `profile` (may be null) and the time from first to last mark
  int finish(std::vector<sky_graph::ProfileEntry>* profile, double* seconds);
};

// A device buffer of at least `bytes` bytes that belongs to the graph; its contents do not survive a larger request.
int pool_get(sky_graph* g, int slot, size_t bytes, void** out);
void pool_release(sky_graph* g);
int ensure_table_storage(sky_graph* g);
int prepare_build_scratch(sky_graph* g, uint32_t max_rows);
int build_rows(sky_graph* g, const uint32_t* src, uint32_t n, EventTimer* tm);
int build_all_tables(sky_graph* g, double* seconds);
// rows of more than 4093 entries: tile-parallel path, and how many tiles per row it accepts
constexpr uint32_t TILED_TILE = 1024;  // slots per tile of the tile-parallel path
int build_rows_tiled(sky_graph* g, const RowRef* rows_list, uint32_t n, uint32_t* skipped, EventTimer* tm,
                     uint64_t edges);
int build_rows_tiled_dev(sky_graph* g, const RowRef* vlist, const uint32_t* dev, int cls, int ncls, uint32_t n_upper,
                         uint64_t edges_upper);
constexpr int MERGE_MAX_NW = 10;  // rows of at most 512 * 10 - 3 = 5117 entries pair by merge in LDS
constexpr uint32_t HOLD_MAX_DEG = 8189;  // 512 threads x 16 slots hold such a row from any 16-byte phase
constexpr uint32_t STREAM_MAX_DEG = 524287;  // longest row of the streaming classes (one workgroup takes 1.5 ms for it)
int build_rows_stream(sky_graph* g, const RowRef* first_list, uint32_t n_first, const RowRef* rows_list, uint32_t n);
int build_rows_stream_dev(sky_graph* g, const RowRef* vlist, const uint32_t* dev, int ncls, uint32_t grid);
int build_rows_hold(sky_graph* g, const RowRef* rows, uint32_t n, const uint32_t* dev, int cls);
// Builds the rows listed in src[0 .. *n_dev) (n_dev: a device word the host never reads; n_upper: what it cannot
// exceed) without waiting for the device at any point.  Needs the graph's class census and a longest row the
// streaming kernel takes (build_rows_dev_possible).
bool build_rows_dev_possible(const sky_graph* g);
int ensure_class_census(sky_graph* g);
int build_rows_dev(sky_graph* g, const uint32_t* src, const uint32_t* n_dev, uint32_t n_upper);
int build_walk_index(sky_graph* g, double* seconds);
uint32_t tiled_max_tiles(const sky_graph* g);
// process-wide values of the knobs (sky_capi.hip) and the accessor every use goes through
extern long long g_option_value[OPT_COUNT];
inline long long option(const sky_graph* g, SkyOpt o) { return g && g->opt_own[o] ? g->opt_value[o] : g_option_value[o]; }
void free_build_scratch(sky_graph* g);
void free_tiled_scratch(sky_graph* g);
int walk_offline(sky_graph* g, const uint32_t* seeds, uint32_t N, uint32_t len, float stop_prob, uint64_t seed,
                 uint32_t* paths, uint32_t* lengths, uint64_t* sampled, double* seconds);
int walk_offline_noalloc(sky_graph* g, const uint32_t* seeds, uint32_t N, uint32_t len, float stop_prob, uint64_t seed,
                         uint32_t* paths, uint32_t* lengths, uint64_t* sampled_device);
int walk_online(sky_graph* g, int bias_kind, float p, float q, const uint32_t* seeds, uint32_t N, uint32_t len,
                float stop_prob, uint64_t seed, uint32_t* paths, uint32_t* lengths, uint64_t* sampled,
                double* seconds);
int walk_node2vec_reject(sky_graph* g, float p, float q, const uint32_t* seeds, uint32_t N, uint32_t len,
                         float stop_prob, uint64_t seed, uint32_t* paths, uint32_t* lengths, uint64_t* sampled,
                         double* seconds);
int sample_khop(sky_graph* g, bool online, const uint32_t* seeds, uint32_t N, const uint32_t* fanout, uint32_t hops,
                uint64_t seed, uint32_t* data, uint32_t* sample_lengths, uint64_t* sampled, double* seconds);
struct SampleSession;
int sample_session_begin(sky_graph* g, const uint32_t* seeds, uint32_t N, const uint32_t* fanout, uint32_t hops,
                         uint64_t seed, uint32_t* data, uint32_t* sample_lengths, SampleSession** out);
int sample_session_frontier(SampleSession* s, uint32_t hop, const uint32_t** list, const uint32_t** count, uint32_t* upper);
int sample_session_hop(SampleSession* s, uint32_t hop, const float* weights);
int sample_session_end(SampleSession* s, uint64_t* sampled, double* seconds);
int generate_rmat(uint32_t scale, uint32_t edge_factor, uint64_t graph_seed, int weight_kind, float wa, float wb,
                  uint64_t weight_seed, sky_graph** out);
int generate_from_degrees(const uint32_t* xadj_host, uint32_t V, uint64_t graph_seed, int weight_kind, float wa, float wb,
                          uint64_t weight_seed, sky_graph** out);
int gen_seeds(uint64_t seed, uint32_t V, uint32_t N, uint32_t* seeds_device);
int philox_selftest(const uint32_t* ctr, const uint32_t* key, uint32_t n, uint32_t* out);
int compute_max_degree(sky_graph* g);

// Device allocation with the spare bytes described above.
template <class T>
int alloc_padded(T** p, size_t count) {
  SKY_HIP(hipMalloc((void**)p, count * sizeof(T) + 16));
  return SKY_OK;
}

}  // namespace sky
