// Internal declarations shared by the translation units of libflowwalker_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "flowwalker.h"

// A vertex that walkers are parked on: its CSR range, so that building batch tasks is a streaming pass.
struct fw_hub_info {
  int32_t v;
  uint32_t off;  // xadj[v]
  uint32_t deg;
  uint32_t row;  // two-pass steps: first row of this list's groups (times the labels per hub), FW_NO_ROWS: none
};
constexpr uint32_t FW_NO_ROWS = 0xFFFFFFFFu;

// Device CSR mirror (include/gpu_graph.cuh:28-36 in the reference).  Edge arrays are allocated with
// FW_EDGE_PAD extra elements so that aligned 16-byte loads of the last quartet stay in bounds.
struct fw_graph {
  int32_t V = 0;
  uint64_t E = 0;
  uint32_t* xadj = nullptr;
  int32_t* adjncy = nullptr;
  float* weight = nullptr;
  int32_t* label = nullptr;
  int owns = 1;
  int host_edges = 0;  // edge arrays live in pinned host memory (FW_GRAPH_HOST_PINNED) and are read over the bus
  int device = 0;
  int32_t max_degree = -1;  // lazily computed
  int32_t max_degree_vertex = -1;
  int sorted = -1;          // lazily computed
  // lazily built index of the vertices whose degree exceeds hub_index_threshold (hub parking)
  int32_t hub_index_threshold = -1;
  int32_t n_hubs = 0;
  uint32_t hub_rows = 0;              // rows the hubs with rows need together, per label
  int32_t* hub_index = nullptr;       // int32[V]: position in hub_info, -1 (not parked on) or -2 (degree 0)
  int2* adj_hub = nullptr;            // int2[E]: {adjncy[e], hub_index[adjncy[e]]}, so that a hub step learns its new
                                      // vertex and that vertex's parking index with one memory request instead of two;
                                      // NULL when the edge arrays live in host memory or there was no room
  struct fw_hub_info* hub_info = nullptr;  // [n_hubs]
  void* park_cache = nullptr;         // the parking lists of the last fw_walk_device call, kept for the next one
  void* batch_cache = nullptr;        // the device buffers of the last fw_walk_batch call, kept for the next one
  void* call_scratch = nullptr;       // launch record (dispenser word + counters) of fw_walk_device, allocated once
  hipEvent_t call_ev[2] = {nullptr, nullptr};  // and its two timing events
  std::atomic<int> busy{0};           // a walk call is running on this graph (the caches above are per graph)
};

constexpr int FW_EDGE_PAD = 4;

// A walker in transit between kernels (parked on a hub, or resuming after its hub step): 16 bytes.
struct fw_walker_rec {
  int32_t q;     // query index inside the launch (walker id = walker_base + q)
  int32_t cur;   // current vertex; in a parked record: the bucket (hub index * labels + label slot) it waits in
  int32_t prev;  // previous vertex or -1; in a parked record: its position inside the bucket of `cur`
  int32_t len;   // path entries written so far
};

// Arguments of one walk-kernel launch.
struct fw_kargs {
  const uint32_t* xadj;
  const int32_t* adjncy;
  const float* weight;
  const int32_t* label;
  const int32_t* starts;
  int32_t* paths;
  uint32_t* dispenser;          // one zeroed word per launch: the global query dispenser
  unsigned long long* counters; // [0] steps, [1] sum of source degrees (walk kernel); [2], [3] the same for the hub batch kernel
  int32_t V;
  int32_t n;
  int32_t max_depth;
  int32_t hub_threshold;
  int32_t slot_limit;           // task slots a workgroup may fill (small batches are spread over the grid)
  uint32_t seed_lo, seed_hi;
  uint32_t walker_base;
  float tp, inv_p, inv_q;
  float n2v_fmax;                    // F = max(1, 1/q): the envelope of node2vec's acceptance test
  float n2v_extra;                   // 1/p - F when positive, else 0: the return edge's excess over the envelope, a
                                     // component of its own of the trial
  int32_t schema_len;
  int32_t schema[FW_MAX_SCHEMA];
  // hub parking (park_threshold = INT32_MAX switches it off)
  int32_t park_threshold;            // a walker that arrives on a vertex of larger degree is parked
  int32_t n_labels_per_hub;          // buckets per hub: 1, or schema_len for metapath (walkers wanting one label share a scan)
  const int32_t* hub_index;          // int32[V]: index of the vertex among the parked-on ones, -1, or -2 = degree 0
  const int2* adj_hub;               // int2[E] or NULL: every adjacency entry with the parking index of its vertex
  fw_walker_rec* parked;             // out: parked[i] = the walker of entry i of the launch's input if it was parked, else a hole (q = -1)
  uint32_t* parked_count;            // += walkers parked (one update per workgroup)
  uint32_t* bucket_count;            // [n_hubs * n_labels_per_hub]
  const fw_walker_rec* resume;       // in: walkers to continue instead of fresh queries (NULL: use starts)
  const uint32_t* n_dev;             // in: when not NULL, the number of entries is read here (n is an upper bound
                                     // the grid was sized for) and slot_limit follows from it
};

// Tag in fw_walker_rec::len of a batch-kernel output record whose vertex is parked on again (stripped by readers).
constexpr int32_t FW_REC_PARK = 0x40000000;
// node2vec records: bits 0..15 of len hold the path length, bits 16..29 the rejected trials of the walker's current
// step (a parked walker whose proposal is rejected waits on the same vertex for another round); prev is the previous
// vertex in every record (its acceptance test searches N(prev)), so positions inside a bucket are handed out by the
// scatter kernel, never carried in the record.
constexpr int FW_REC_TRIAL_SHIFT = 16;
constexpr int32_t FW_REC_TRIAL_MASK = 0x3FFF;
constexpr int32_t FW_REC_LEN_MASK = 0xFFFF;

// A parked walker in the sorted list, for every application but node2vec: the bucket follows from the position and
// the previous vertex is not needed, so 8 bytes are enough -- half the scattered bytes of the counting sort, whose
// time follows the bytes it scatters (node2vec keeps whole records: its acceptance test needs the previous vertex).
struct fw_parked_rec {
  int32_t q;
  int32_t len;
};

// The counters of a parking round sit one to a 64-byte line (counter k at word k * FW_CTR_STRIDE): atomic updates of
// one line complete one after the other wherever they come from, and several kernels update several of them at once.
constexpr int FW_CTR_STRIDE = 16;

// One batch: up to 64 walkers parked on vertex v, records sorted[rec_base .. rec_base + count).  32 bytes.
struct fw_batch_task {
  int32_t v;
  uint32_t off;       // xadj[v]
  uint32_t deg;
  uint32_t rec_base;
  int32_t count;
  int32_t slot;       // metapath: position in the schema of the label these walkers want
  uint32_t row;       // two-pass steps: first row of the list's groups
  int32_t pad;
};

// Arguments of the hub batch kernel: up to 64 walkers parked on one vertex are served with one scan of its list,
// by a workgroup (degree above hub_threshold: workgroup-granularity sampling) or by a single wave.
struct fw_hub_args {
  const void* sorted;                // parked records grouped by bucket: fw_parked_rec, node2vec fw_walker_rec
  const fw_batch_task* tasks;        // workgroup tasks, handed out through task_next to the last dynamic_wgs workgroups
  uint32_t* task_next;
  uint32_t dynamic_wgs;              // set by the launch: the workgroups of one resident set
  const uint32_t* ntasks;
  const fw_batch_task* wtasks;       // wave tasks, wave i of the grid takes i, i + waves, ...
  const uint32_t* nwtasks;
  // out[rec_base + i] = walker i of the batch after its step: q = -1 when its walk is over, len tagged with
  // FW_REC_PARK when its new vertex is parked on again (bucket_out counts those, prev = position inside the
  // bucket), untagged otherwise
  fw_walker_rec* out;
  uint32_t* bucket_out;
  uint32_t* out_counts;              // [0] += records that resume, [FW_CTR_STRIDE] += records parked again
  // Two-pass steps of crowded hubs.  The scan launch works through stasks (rec_base = first group of the run,
  // count = one past its last, row = the list's first row) and fills, per group of a list, totals[row],
  // rows[row * 128 ..] (64 running maxima, 64 prefixes) and lastpos[row]; the batch launch then serves ttasks
  // (a batch task plus row = the list's first row) from them.
  const fw_batch_task* stasks;
  const uint32_t* nstasks;
  const fw_batch_task* ttasks;
  const uint32_t* nttasks;
  // Quad tasks: at most 16 walkers on a list of at most 64 aligned quartets (one group whose lanes hold one quartet
  // each).  A wave serves four of them at once, one per 16-lane row: wave i of the grid takes tasks 4i .. 4i + 3,
  // then 4 (i + waves) ..
  const fw_batch_task* qtasks;
  const uint32_t* nqtasks;
  float* totals;
  float* rows;
  int32_t* lastpos;
};

#ifdef __HIPCC__
// counter[key] += 1 for every lane with pred; returns the value the lane's own increment found (its rank among the
// increments of that counter).  When several lanes of the wave share the first active lane's key (then the first
// remaining lane's), they are served by one atomic of their count: a wave whose walkers mostly move to one vertex
// would otherwise update that vertex's counter 64 times in a row, and updates of one address cost about 13 ns
// each wherever they come from.  Call from wave-uniform control flow.
template <bool kReturn>
__device__ __forceinline__ uint32_t fw_wave_count_keys(uint32_t* counter, uint32_t key, bool pred) {
  const int lane = (int)__lane_id();
  uint32_t rank = 0u;
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const uint64_t m = __ballot(pred);
    if (m == 0ull) break;
    const int leader = __builtin_ctzll(m);
    const uint32_t k = (uint32_t)__builtin_amdgcn_readlane((int)key, leader);
    const bool same = pred && key == k;
    const uint64_t ms = __ballot(same);
    const uint32_t cnt = (uint32_t)__builtin_popcountll(ms);
    if (cnt < 4u) break;
    uint32_t old = 0u;
    if (lane == leader) {
      if (kReturn) old = atomicAdd(&counter[k], cnt);
      else atomicAdd(&counter[k], cnt);
    }
    if (kReturn) {
      old = (uint32_t)__builtin_amdgcn_readlane((int)old, leader);
      if (same) rank = old + (uint32_t)__builtin_popcountll(ms & ((1ull << lane) - 1ull));
    }
    pred = pred && !same;
  }
  if (pred) {
    if (kReturn) rank = atomicAdd(&counter[key], 1u);
    else atomicAdd(&counter[key], 1u);
  }
  return rank;
}
#endif

void fw_set_error(const char* fmt, ...);
int fw_check_hip(hipError_t e, const char* what, const char* file, int line);
#define FW_HIP(call)                                                  \
  do {                                                                \
    int fw_rc_ = fw_check_hip((call), #call, __FILE__, __LINE__);     \
    if (fw_rc_ != FW_OK) return fw_rc_;                               \
  } while (0)

// Launches the walk kernel for (app, sampler, wg_threads) on `stream`.  grid = 0: fill the device.
// Returns the grid used through *grid_used.
// entries_hint: launches of the parking pipeline say about how many entries they will find (sizes the grid when
// grid <= 0); 0 for a launch whose walkers run their whole walks.
int fw_launch_walk(const fw_kargs& a, int app, int sampler, int wg_threads, int grid, uint32_t entries_hint,
                   hipStream_t stream, int* grid_used);

// Launches the reference's walk engine restated for 64-lane waves (sampler = FW_SAMPLER_REF_ZPRS / _DPRS, optionally
// with FW_SAMPLER_REF_STATIC).  grid = 0: twice the resident set.
int fw_launch_ref_walk(const fw_kargs& a, int app, int sampler, int wg_threads, int grid, hipStream_t stream,
                       int* grid_used);

// Launches the hub batch kernel.  tasks_hint: about how many wave-sized pieces of work it will find (sizes the grid;
// 0 = no idea: one resident set).
int fw_launch_hub_batch(const fw_kargs& a, const fw_hub_args& h, int app, int wg_threads, uint32_t tasks_hint,
                        hipStream_t stream);
int fw_launch_hub_quad(const fw_kargs& a, const fw_hub_args& h, int app, uint32_t quads_hint, hipStream_t stream);
// Launches the scan kernel of the two-pass steps (it finds its task count in h.nstasks on the device).
// tasks_hint: about how many scan tasks to expect, to size the grid (0 = no idea: a full resident set).
int fw_launch_hub_scan(const fw_kargs& a, const fw_hub_args& h, int app, uint32_t tasks_hint, hipStream_t stream);
