/*
 * C-ABI of libskywalker_hip.so: the alias-method hot path of Skywalker on one MI355X.
 *
 * The reference has no FFI; its host boundary is the set of `float f(Obj&)` entry
 * functions declared in include/sampler.cuh:510-529 plus the gpu_graph / Sampler /
 * Walker objects they take.  Each entry point below names the reference interface
 * it replaces.  The C++ facade in skywalker_amd/host keeps the reference's class
 * and function names on top of this ABI.
 *
 * Conventions
 *   - every function returns 0 on success or a negative sky_status; the message of
 *     the last failure on the calling thread is available from sky_last_error().
 *   - a sky_graph owns the device-resident CSR and, after sky_alias_build_all, the
 *     alias tables.  One host thread per sky_graph; calls are synchronous.  The scratch memory of the table
 *     builds belongs to the graph (allocated on first use, freed with it), and so can the tuning knobs
 *     (sky_graph_set_option).  Every graph works on the null stream, like the reference's entry functions.
 *   - "device pointer" arguments are HIP device addresses on the current device
 *     (from sky_device_malloc, or any other allocator of the same process).
 *   - `seconds` outputs report the kernel region only (launch to completion,
 *     measured with HIP events on the stream the kernels run on), like the
 *     gettimeofday bracket of the reference (src/util.cu:35-44).
 *   - unreached output slots are never written; callers that want a sentinel
 *     pre-fill with sky_device_fill_u32.
 */
#ifndef SKYWALKER_HIP_H_
#define SKYWALKER_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct sky_graph sky_graph;

/* One slot of an alias table: draw col uniformly, keep it when u < prob, else take alias (a row-local index).
 * The reference keeps two arrays (prob_array, alias_array; include/gpu_graph.cuh:41-43); here the pair is
 * interleaved so that a draw touches one cache line instead of two. */
typedef struct sky_alias_entry {
  float prob;
  uint32_t alias;
} sky_alias_entry;

enum sky_status {
  SKY_OK = 0,
  SKY_ERR_ARG = -1,     /* null pointer, zero size, inconsistent CSR */
  SKY_ERR_HIP = -2,     /* a HIP runtime call failed */
  SKY_ERR_STATE = -3,   /* e.g. walk on tables that were never built */
  SKY_ERR_NO_GPU = -4,  /* no usable device */
  SKY_ERR_LIMIT = -5    /* size beyond what the entry point supports */
};

/* SKY_BIAS_NODE2VEC builds the second-order table of every (walker, step) and draws from it, as the reference
 * does; SKY_BIAS_NODE2VEC_REJECT samples the same law by rejection on the first-order tables (built by the call
 * when the graph has none): one membership search per trial instead of one per neighbour. */
enum sky_bias { SKY_BIAS_STATIC = 0, SKY_BIAS_NODE2VEC = 1, SKY_BIAS_NODE2VEC_REJECT = 2 };
enum sky_weight_kind { SKY_W_UNIFORM = 0, SKY_W_UNIT = 1, SKY_W_LOGNORMAL = 2 };

#define SKY_INVALID 0xFFFFFFFFu /* alias value of rows whose total weight is zero */

const char* sky_last_error(void);
const char* sky_version(void);

/* ---- device memory helpers (replace the cudaMalloc/cudaMemcpy calls scattered through
 *      include/sampler_result.cuh:490-566 and include/gpu_graph.cuh:68-117).  sky_device_malloc allocates 16 bytes
 *      more than asked for: the build kernels read weights as whole 16-byte vectors, and an array from here can be
 *      handed to them where it lies ---- */
int sky_device_malloc(size_t bytes, void** out);
int sky_device_free(void* p);
int sky_memcpy_h2d(void* dst_device, const void* src_host, size_t bytes);
int sky_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes);
int sky_device_fill_u32(void* dst_device, uint32_t value, size_t count);
/* Plain device-to-device copy kernel of `count` 32-bit words: the known-size reference for calibrating
 * HBM traffic counters. */
int sky_device_copy_u32(void* dst_device, const void* src_device, size_t count);
int sky_device_synchronize(void);
/* Free and total device memory of the current device as the HIP runtime reports them (hipMemGetInfo); either
 * output may be NULL.  Lets a caller check that a call allocated nothing. */
int sky_device_mem_info(size_t* free_bytes, size_t* total_bytes);
int sky_device_name(char* buf, size_t buflen, int* compute_units);

/* ---- graph residency: replaces gpu_graph::gpu_graph(Graph*, uint) (include/gpu_graph.cuh:68-117).
 *      xadj[V+1], adjncy[E], adjwgt[E] are host arrays; rows must be sorted by neighbour id for
 *      node2vec (gpu_graph.cuh:204-238 assumes the same). adjwgt may be NULL (all weights 1). ---- */
int sky_graph_upload(const uint32_t* xadj, const uint32_t* adjncy, const float* adjwgt, uint32_t V, uint32_t E,
                     sky_graph** out);
/* Synthetic R-MAT graph (a,b,c,d = .57,.19,.19,.05) generated and sorted on the device; no counterpart in the
 * reference, which reads Galois .gr files (include/graph.cuh:164-327).  weight_kind: sky_weight_kind with
 * parameters (wa, wb) = (lo, hi) for UNIFORM, ignored for UNIT, (mu, sigma) for LOGNORMAL. */
int sky_graph_generate_rmat(uint32_t scale, uint32_t edge_factor, uint64_t graph_seed, int weight_kind, float wa,
                            float wb, uint64_t weight_seed, sky_graph** out);
/* Synthetic graph with the row lengths the caller chooses: xadj[V+1] is a host array (row offsets), every neighbour id
 * is drawn uniformly over [0, V) and every weight as in sky_graph_generate_rmat, both on the device, so that a graph of
 * a billion edges needs no host arrays of that size.  No counterpart in the reference.  Rows are NOT sorted by
 * neighbour id: fine for table builds, first-order walks and sampling, not for node2vec.  Made for measuring the
 * build on degree distributions that an R-MAT generator does not produce. */
int sky_graph_generate_from_degrees(const uint32_t* xadj, uint32_t V, uint64_t graph_seed, int weight_kind, float wa,
                                    float wb, uint64_t weight_seed, sky_graph** out);
int sky_graph_info(const sky_graph* g, uint32_t* V, uint32_t* E, uint32_t* max_degree);
/* Copies to host; any destination may be NULL. */
int sky_graph_download(const sky_graph* g, uint32_t* xadj, uint32_t* adjncy, float* adjwgt);
/* Device addresses of the resident arrays (xadj, adjncy, adjwgt, table[E], valid); any output may be NULL. */
int sky_graph_device_ptrs(const sky_graph* g, const uint32_t** xadj, const uint32_t** adjncy, const float** adjwgt,
                          const sky_alias_entry** table, const int8_t** valid);
/* Replaces gpu_graph::Free + Sampler::Free (gpu_graph.cuh:164-177, sampler.cuh:65-81). */
int sky_graph_free(sky_graph* g);

/* ---- offline alias tables for every vertex: replaces ConstructTable(Sampler&, ngpu=1, index=0)
 *      (src/createTable.cu:119-179, kernel :48-108).  Allocates table[E] ({prob f32, alias u32}: row-local
 *      index, same slot as the CSR edge) and valid[V] i8 inside the graph.  Unlike the reference the
 *      edge weights are kept (createTable.cu:175-177 frees them). ---- */
int sky_alias_build_all(sky_graph* g, double* seconds);
/* The same build from a weight array of the caller (E floats in device memory, CSR slot order) instead of the graph's
 * own weights, which are left as they are: for weights that a bias operator computes (include/skywalker_bias.h), as
 * the reference's constructors take them from gpu_graph::getBias (include/alias_table_new.cuh:1090-1091).
 * An array of exactly E floats is accepted.  The build kernels read whole 16-byte vectors that may reach up to 12
 * bytes past the last weight: when the array's device allocation holds at least 16 readable bytes after the E floats
 * (the library asks the HIP runtime for the allocation's extent) it is read where it lies; otherwise the call first
 * copies it into a padded array that stays with the graph (E * 4 + 16 bytes more device memory, one device-to-device
 * copy before the kernel region that `seconds` reports).  Allocate E * 4 + 16 bytes to avoid the copy. */
int sky_alias_build_from_weights(sky_graph* g, const float* weights_device, double* seconds);
/* Copies the table to host as two arrays (any destination may be NULL). */
int sky_alias_download(const sky_graph* g, float* prob, uint32_t* alias, int8_t* valid);
/* Installs caller-built tables (host arrays) instead of building: for tests and table persistence.  The arrays are
 * checked before they are used: valid[v] is 0 or 1 (0 for a vertex without edges); every prob lies in [0, 1];
 * in a valid row every alias is below the row's degree, in an invalid row every alias is SKY_INVALID.
 * SKY_ERR_ARG otherwise, and the graph keeps the tables it had. */
int sky_alias_upload(sky_graph* g, const float* prob, const uint32_t* alias, const int8_t* valid);

/* ---- start vertices uniform over [0,V): Philox(seed; i). seeds_device[N]. The reference uses 0..N-1
 *      (include/sampler.cuh:494-503); sequential seeds are simply uploaded by the caller.  The walk and
 *      sample calls below accept any 32-bit value as a start vertex: one that is not below V is recorded in its
 *      slot and never left (length 0, no children), it is not an error. ---- */
int sky_gen_seeds(uint64_t seed, uint32_t V, uint32_t N, uint32_t* seeds_device);

/* ---- biased walk on prebuilt tables: replaces OfflineWalk(Walker&) (src/offline_walk.cu:181-230, kernels
 *      :10-175); stop_prob > 0 adds the PPR stop test the reference only has online (online_walk.cu:109-110).
 *      paths_device[N*(len+1)] walker-major, lengths_device[N]; *sampled = sum of lengths. ---- */
int sky_walk_offline(sky_graph* g, const uint32_t* seeds_device, uint32_t N, uint32_t len, float stop_prob,
                     uint64_t philox_seed, uint32_t* paths_device, uint32_t* lengths_device, uint64_t* sampled,
                     double* seconds);

/* ---- optional index for the walks on prebuilt tables (no counterpart in the reference, whose walk kernels gather
 *      prob_array, alias_array and adjncy separately, src/offline_walk.cu:100-120): one 16-byte entry per CSR slot,
 *      {prob, alias, neighbour of the slot, neighbour of its alias slot}, so that a step reads two cache lines
 *      (xadj, entry) instead of three.  Costs 16 bytes per edge of device memory and one pass over the tables;
 *      sky_walk_offline, sky_walk_offline_noalloc and the walks that end in them use it while it is current.  Any
 *      call that rewrites table entries (sky_alias_build_all, sky_alias_upload, the online modes) makes it stale:
 *      it is then ignored until it is built again.  Paths are the same with and without it. ---- */
int sky_walk_index_build(sky_graph* g, double* seconds);

/* ---- sky_walk_offline for callers that cannot allocate (code under HIP graph capture, serving loops, harnesses
 *      that forbid hipMalloc).  No counterpart in the reference.  Same kernel, same paths and lengths; the
 *      per-workgroup counts of sampled edges go to a static device array of the library (128 KiB per GPU, held
 *      until the process ends) instead of an allocated counter, and their sum is written by a second kernel to
 *      sampled_device, a device word of the caller (may be NULL).  The call allocates nothing, creates no event,
 *      copies nothing to the host and does not wait: the kernels are enqueued on the graph's stream (the null
 *      stream) and the caller synchronises (sky_device_synchronize) before reading the outputs.  At most
 *      4,194,304 walkers per call (SKY_ERR_LIMIT beyond).  Every call on a GPU shares that GPU's array, so calls
 *      that overlap on one GPU race. ---- */
#define SKY_WALK_NOALLOC_MAX_WALKERS 4194304u
int sky_walk_offline_noalloc(sky_graph* g, const uint32_t* seeds_device, uint32_t N, uint32_t len, float stop_prob,
                             uint64_t philox_seed, uint32_t* paths_device, uint32_t* lengths_device,
                             uint64_t* sampled_device);

/* ---- walk that rebuilds the table of the current vertex at every step: replaces OnlineWalkShMem(Walker&) /
 *      OnlineWalkGMem(Walker&) (src/online_walk.cu:245-327, online_walk_gmem.cu); bias SKY_BIAS_NODE2VEC applies
 *      the second-order factors of src/api/bias_node2vec.cu:15-27 with (p, q); SKY_BIAS_NODE2VEC_REJECT reaches
 *      the same distribution by rejection, the way src/unbiased_walk.cu:14-60 does for unit weights. ---- */
int sky_walk_online(sky_graph* g, int bias_kind, float p, float q, const uint32_t* seeds_device, uint32_t N,
                    uint32_t len, float stop_prob, uint64_t philox_seed, uint32_t* paths_device,
                    uint32_t* lengths_device, uint64_t* sampled, double* seconds);

/* ---- k-hop neighbour sampling: replaces OfflineSample(Sampler_new&) (src/offline_sample.cu:443-513) and
 *      OnlineGBSampleNew(Sampler_new&) (src/online_sample_new.cu:459-547).  fanout[hops] with fanout[0] == 1
 *      (host array, e.g. {1,25,10}); data_device[N*length_per_sample], sample_lengths_device[N*size_of_lengths]
 *      in the layout of include/sampler_result.cuh:226-260 (see sky_sample_layout). ---- */
int sky_sample_layout(const uint32_t* fanout, uint32_t hops, uint64_t* length_per_sample,
                      uint64_t* size_of_sample_lengths);
int sky_sample_offline(sky_graph* g, const uint32_t* seeds_device, uint32_t N, const uint32_t* fanout, uint32_t hops,
                       uint64_t philox_seed, uint32_t* data_device, uint32_t* sample_lengths_device,
                       uint64_t* sampled, double* seconds);
/* By default sky_sample_online draws WITH replacement, like sky_sample_offline and the reference's offline kernel
 * (src/offline_sample.cu:109-133): a parent of more than fanout neighbours yields exactly fanout children, which may
 * repeat, and sample_lengths holds fanout.  The reference's OnlineGBSampleNew draws distinct neighbours by retrying
 * against a selected[] set and may return fewer than fanout (src/online_sample_new.cu:83-105): the option
 * "sample_distinct" of sky_set_option (below) switches both sample calls to a rule of distinct children.  That rule
 * is a deterministic variant, not the reference's law: here draw i of a parent tries up to 11 candidates in turn,
 * there up to 11 rounds per parent run with 32 lanes drawing at once, so the expected number of children of a
 * parent differs; the variant's own law is pinned by enumeration in the tests, its agreement with the reference's
 * is unpinned.  Online and offline results of this library are identical under either setting. */
int sky_sample_online(sky_graph* g, const uint32_t* seeds_device, uint32_t N, const uint32_t* fanout, uint32_t hops,
                      uint64_t philox_seed, uint32_t* data_device, uint32_t* sample_lengths_device, uint64_t* sampled,
                      double* seconds);

/* ---- sky_sample_online taken apart hop by hop, for callers that compute the weights of the rows a hop builds
 *      themselves: a bias operator (include/skywalker_bias.h).  The reference's online sampler builds every frontier
 *      row through a constructor that asks gpu_graph::getBias for each weight
 *      (include/alias_table_new.cuh:1090-1091, called from src/online_sample_new.cu:3-70); here the operator lives in
 *      another library, so the sampler hands out the frontier and takes the weights back:
 *        begin     outputs cleared, start vertices in place; the graph's tables count as not built
 *        frontier  the distinct parents of `hop` (0 .. hops - 2) whose rows this session has not built: their vertex
 *                  ids in *list_device, their number in the device word *count_device (the host is not told it),
 *                  at most *upper of them
 *        hop       builds those rows from weights_device (E floats in CSR slot order, of which only the slots of
 *                  the listed rows are read; an array whose allocation does not hold 16 more bytes, which
 *                  sky_device_malloc always adds, is copied first, as in sky_alias_build_from_weights; NULL: the
 *                  graph's own weights), then draws the children of `hop`
 *        end       sampled edges and kernel-region seconds; frees the session
 *      Calls come in that order, frontier and hop once per hop, on one host thread.  Results are those of
 *      sky_sample_online on a graph whose weights are the ones supplied. ---- */
typedef struct sky_sample_session sky_sample_session;
int sky_sample_session_begin(sky_graph* g, const uint32_t* seeds_device, uint32_t N, const uint32_t* fanout, uint32_t hops,
                             uint64_t philox_seed, uint32_t* data_device, uint32_t* sample_lengths_device,
                             sky_sample_session** out);
int sky_sample_session_frontier(sky_sample_session* s, uint32_t hop, const uint32_t** list_device,
                                const uint32_t** count_device, uint32_t* upper);
int sky_sample_session_hop(sky_sample_session* s, uint32_t hop, const float* weights_device);
int sky_sample_session_end(sky_sample_session* s, uint64_t* sampled, double* seconds);

/* ---- self-test hook: runs Philox4x32-10 on the device for n (counter, key) pairs.
 *      ctr_host[4n], key_host[2n] -> out_host[4n]. ---- */
int sky_philox_selftest(const uint32_t* ctr_host, const uint32_t* key_host, uint32_t n, uint32_t* out_host);

/* ---- tuning knobs (no counterpart in the reference).  "tiled_max_tiles": rows too long for one workgroup are
 *      built tile by tile (1024 entries per tile) up to this many tiles (default: no limit); longer rows
 *      fall to a kernel in which one workgroup walks the whole row.  Tests lower it to exercise that kernel.
 *      "row_merge" (default 1): rows of 193..5117 entries pair lights and heavies by a merge of their prefix
 *      sums, rows of 5118..8189 entries are held by one workgroup; 0 selects the kernel that does one binary search per
 *      entry (the tile-parallel path from 4094 entries on).  Both give the same table.
 *      "stream_min_edges" (default 4000000): rows of 8190..524287 entries have a kernel of their own (one workgroup
 *      streams a row); when a build holds no more than this many entries in such rows, too few to fill the GPU
 *      with one workgroup each, they go to the tile-parallel path instead.  Tests set 0.
 *      "stream_wide_min_edges" (default 134217216): the rows of more than 65533 entries among them keep a workgroup
 *      busy for up to 1.5 ms; they join that kernel only when the build holds at least this many entries in rows
 *      of 8190..524287 entries (the launch then runs that long anyway), else they are built tile by tile.  Tests set 0.
 *      "walk_read_once" (default -1): 1 makes the walks load a step's table entry and neighbour id as read-once
 *      data, which keeps the row offsets of the well-connected vertices in L2 on a graph whose tables are far larger
 *      than the caches; 0 loads them as ordinary data (better when the tables fit the caches); -1 decides by the size of
 *      the tables (read-once above 2 GiB).  Same paths.
 *      "sample_distinct" (default 0): 1 makes sky_sample_offline and sky_sample_online give every parent distinct
 *      children, the rule of the reference's online sampler (roll_atomic / roll_once, src/online_sample_new.cu:72-105),
 *      in a form that does not depend on scheduling: draw i of a parent tries up to 11 candidates (Philox counter
 *      word 2 = hop + 256 * try) and keeps the first slot of the row that no earlier draw of the parent kept; a draw
 *      whose candidates were all kept already adds nothing, so sample_lengths may be below the fanout.  Fanouts of
 *      at most 64, at most 256 hops (SKY_ERR_LIMIT otherwise).
 *      "small_in_place" (default -1): 1 builds the rows of at most 32 entries in one kernel that walks the vertices
 *      in order and needs no row lists (it runs beside the binning pass and the kernels of the long rows); 0 builds
 *      them by degree class like all other rows; -1 takes the former for builds of at least 2^25 rows.  Same tables.
 *      "build_streams" (default 1): a build of 2 M .. 1 G entries without per-kernel timing sends the kernels of
 *      its degree classes out over the graph's stream and three side streams (small builds are bound by one
 *      kernel waiting for the one before); 0 keeps every kernel on the graph's stream.  Same tables.
 *      "build_profile" (default 0): 1 records a HIP event after every kernel of sky_alias_build_all for
 *      sky_last_build_profile (about 3 microseconds each; a small graph pays 20 % of its build for them).
 *      "online_full_build" (default -1): how sky_walk_online serves a static bias on a graph without tables:
 *      0 builds, before every step, the rows the walkers stand on; 1 builds every row first and walks as
 *      sky_walk_offline does; -1 takes whichever is estimated to be faster.  The paths are the same.
 *      "online_device_sized" (default 1): sky_sample_online and the step-by-step form of sky_walk_online build the
 *      rows of a frontier without the host ever learning how many they are: the length of the list and the sizes of
 *      its degree classes stay on the device, every build kernel finds its rows through them, and the call waits for
 *      the device only once, at its end (a walk also learns that no walker is left through pinned host words that it
 *      reads without waiting).  0 makes the host read the size of every frontier and size the launches exactly, which
 *      waits twice per hop or step.  Same results.
 *      "walk_compact_every" (default 0): k > 0 makes sky_walk_offline run k steps per launch and hand the next
 *      launch the list of walkers that are still walking (the reference's walker queue,
 *      include/sampler_result.cuh:646-669), so that walkers that have stopped no longer hold a lane; 0 keeps every
 *      walker on its lane for the whole walk in one launch.  The paths are the same. ---- */
int sky_set_option(const char* name, long value);
/* The same knobs for one graph: sky_graph_set_option gives the graph a value of its own, which the calls on that graph
 * use instead of the process-wide one that sky_set_option sets; sky_graph_unset_option returns the graph to the
 * process-wide value.  Two graphs of one process can so be built and walked under different settings. */
int sky_graph_set_option(sky_graph* g, const char* name, long value);
int sky_graph_unset_option(sky_graph* g, const char* name);

/* ---- per-kernel timing of the last sky_alias_build_all on this graph, for roofline reporting:
 *      names[i] is a static string, ms[i] its HIP-event duration.  Returns the number of entries: one
 *      ("build") unless the option "build_profile" was 1 during the build. ---- */
int sky_last_build_profile(const sky_graph* g, const char** names, float* ms, uint64_t* edges, int max_entries);

#ifdef __cplusplus
}
#endif
#endif /* SKYWALKER_HIP_H_ */
