/*
 * flowwalker.h -- C ABI of libflowwalker_hip.so, the MI355X (gfx950) walk engine.
 *
 * The reference (junyimei/flowwalker-artifact) has no FFI; its seam is the pair of in-process host
 * entry points walk_test / walk_batch (include/walker.cuh:49-57) that src/main.cu:346-357 calls
 * with a device graph (include/gpu_graph.cuh:28-78) and gflags globals for the application
 * parameters (src/walk.cu:36-44).  Every function below names the reference interface it replaces.
 *
 * Conventions: plain pointers and sizes; every function returns an fw_status (0 = ok) and never
 * calls exit(); fw_last_error() describes the last failure on the calling thread.  "d_" pointers
 * are device memory of the current HIP device, "h_" pointers are host memory.  Output buffers are
 * caller-owned (the reference allocates result_pool inside the callee and never frees it:
 * src/walk.cu:536, :586).
 */
#ifndef FLOWWALKER_H_
#define FLOWWALKER_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FW_MAX_SCHEMA 64
#define FW_WAVE 64

typedef enum {
  FW_OK = 0,
  FW_ERR_INVALID = 1,   /* bad argument (message says which) */
  FW_ERR_HIP = 2,       /* a HIP runtime call failed */
  FW_ERR_NO_DEVICE = 3, /* no gfx950 device visible */
  FW_ERR_IO = 4,        /* file missing / short / inconsistent */
  FW_ERR_NOMEM = 5
} fw_status;

/* Application selector: --deepwalk / --ppr / --node2vec / --metapath (src/main.cu:50-53);
 * functors of include/app.cuh:58-152. */
typedef enum { FW_APP_DEEPWALK = 0, FW_APP_PPR = 1, FW_APP_NODE2VEC = 2, FW_APP_METAPATH = 3 } fw_app;

/*
 * Sampler selector: ZPRS kernel (include/walker.cuh:1307) or DPRS kernel (:1444, --dprs).  Both name this
 * library's one-pass sampler (it evaluates every bias once, which is what the reference's DPRS kernel exists for).
 * FW_SAMPLER_REF_ZPRS / FW_SAMPLER_REF_DPRS run the reference's own algorithms instead, restated for 64-lane waves:
 * sampler_warp / sampler_block (include/sampler.cuh:46-127: two passes, one uniform per neighbour, key max-reduce)
 * and sampler_warp_oneloop / sampler_block_oneloop (:129-200: chunked scan with carry) inside the reference's round
 * structure (64 task slots per workgroup, include/walker.cuh:1357-1438).  They are the ablation baselines of
 * README.md:152-163 and the columns of the sampler micro-benchmark; same sampling law, their own random streams, no
 * parking.  OR FW_SAMPLER_REF_STATIC into either for the reference's static query assignment (src/walk.cu:46-61)
 * instead of the global dispenser.
 * With FW_SAMPLER_REF_STATIC, OR in FW_SAMPLER_REF_RNG_GLOBAL or FW_SAMPLER_REF_RNG_LDS for generators that belong to
 * the threads, as the reference's do, instead of draws addressed by (walker, step, element): thread `gid` takes its
 * uniforms one after the other from its own stream, with the generator's state in device memory, read and written
 * around every draw (cuRAND states, walker_wb_dprs_curand, include/walker.cuh:1584-1696: the "FW" level of
 * README.md:152-163), or in LDS as a structure of arrays (include/myrand.cuh:83-86, :174-186: the "+ RNG" level).  The
 * walks are then a function of (seed, queries, grid, wg_threads) -- the same for both placements -- and the law is
 * unchanged.  FW_ERR_INVALID without FW_SAMPLER_REF_STATIC (with the dispenser the thread that serves a query changes
 * from run to run).
 */
typedef enum {
  FW_SAMPLER_ZPRS = 0,
  FW_SAMPLER_DPRS = 1,
  FW_SAMPLER_REF_ZPRS = 2,
  FW_SAMPLER_REF_DPRS = 3,
  FW_SAMPLER_REF_STATIC = 0x100,
  FW_SAMPLER_REF_RNG_LDS = 0x200,
  FW_SAMPLER_REF_RNG_GLOBAL = 0x400
} fw_sampler;

/*
 * Walk parameters.  Replaces the gflags globals read by src/walk.cu:36-44 (FLAGS_tp, FLAGS_p,
 * FLAGS_q, app booleans) and the schema / schema_len / max_depth arguments of walk_test /
 * walk_batch.  Fill with fw_walk_params_default() and override.
 */
typedef struct {
  int32_t app;           /* fw_app */
  int32_t sampler;       /* fw_sampler */
  int32_t max_depth;     /* path row length = --d + 1 (src/main.cu:342) */
  int32_t wg_threads;    /* lanes of the workgroup sampler: 256, 512 or 1024 */
  int32_t hub_threshold; /* degree > hub_threshold uses the workgroup sampler (THRESHOLD, include/walker.cuh:29) */
  int32_t schema_len;    /* metapath: number of labels in the schema (src/main.cu:226-242) */
  int32_t schema[FW_MAX_SCHEMA];
  float tp;              /* PPR termination probability (--tp) */
  float p;               /* node2vec return parameter (--p) */
  float q;               /* node2vec in-out parameter (--q) */
  uint32_t walker_base;  /* global walker id of query 0: keys the RNG, so batches do not repeat streams */
  uint64_t seed;         /* RNG seed (the reference hard-codes 1337: include/walker.cuh:1324) */
  int32_t grid;          /* workgroups to launch; 0 = library default (src/walk.cu:84-92 analogue) */
  int32_t park_threshold; /* hub parking, an execution strategy that never changes results: walkers that arrive on a
                            vertex of larger degree wait there and are served 64 at a time by one shared scan of its
                            list (by a workgroup above hub_threshold, by one wave below).  0 = library default (on
                            for batches >= 65536 queries), < 0 = off, > 0 = degree.  node2vec: the shared scan
                            proposes, each walker accepts with its own adjacency test (max_depth <= 65535). */
  /* node2vec is sampled in two stages: a neighbour is proposed with probability w / sum w and accepted with
   * probability f / F, f = 1 (common neighbour of the previous vertex) or 1/q, F = max(1, 1/q); a rejected walker
   * proposes again.  The return edge (f = 1/p) is accepted with probability (1/p) / F when that is at most 1; when 1/p
   * is larger, a trial first takes the return edge outright with the probability its excess (1/p - F) w has in the
   * envelope F sum w + (1/p - F) w, and otherwise accepts it whenever it is proposed.  The accepted neighbour has the
   * reference's law w f / sum w f (include/app.cuh:97-127) exactly.  The work per step does not depend on p, but it
   * follows q: the expected number of proposals is about F sum w / sum w f (1.3 at p = 2, q = 0.5 on the R-MAT
   * benchmark graph, where few proposals are common neighbours; about q for q > 1: 4 at q = 4), where the reference's
   * one pass over the biases costs the same whatever p and q.  After 16,383 rejections of one step the next proposal
   * is taken unconditionally (the trial count travels in 14 bits of a record): at acceptance probabilities this library
   * is meant for that never happens (0.94^16383), and where it could (q above about 1000) that step follows w / sum w
   * instead of the node2vec law. */
  int32_t time_kernels;  /* != 0: fw_walk_stats.walk_kernel_ms / hub_kernel_ms are measured too (two more events on the
                            stream per launch; an event costs the stream about 5 us, which is 3 - 5 % of a pass made of
                            many short launches).  0 (default): they stay 0, kernel_ms is measured as always. */
  int32_t reserved;      /* 0 */
} fw_walk_params;

/* What src/main.cu:82-113 (calculate_workload) and the timing code of src/walk.cu report. */
typedef struct {
  double kernel_ms;       /* sum of walk-kernel durations (HIP events on the launch stream) */
  double total_ms;        /* wall time of the call, transfers included (src/walk.cu:388,459,465) */
  uint64_t steps;         /* "Total sampled vertex" */
  uint64_t sampled_edges; /* "Total sampled edge": sum over steps of deg(source) */
  int32_t launches;       /* fw_walk_batch: batches; fw_walk_device: walk + hub-batch kernel launches */
  int32_t grid;           /* workgroups per launch actually used */
  /* per-kernel breakdown of kernel_ms / steps / sampled_edges (hub parking splits a pass over two kernels) */
  double walk_kernel_ms;      /* sum over fw_walk_zprs launches (with fw_walk_params.time_kernels, else 0) */
  double hub_kernel_ms;       /* sum over the hub launches of every round: fw_hub_scan, fw_hub_batch, fw_hub_quad
                                 (with fw_walk_params.time_kernels, else 0) */
  uint64_t hub_steps;         /* steps taken in the hub launches (included in steps) */
  uint64_t hub_sampled_edges; /* their source degrees (included in sampled_edges) */
  /* What the call's kernels asked of the memory, MODELLED from the run's own counters (steps, records moved, list
   * quartets streamed): requested_bytes = list_bytes + 128 * scattered_reads + 32 * scattered_writes + record_bytes.
   * list_bytes: every list pass in 16-byte quartets (a list is read once per walker step by the walk kernel, once per
   * batch of up to 64 walkers or once per call by the hub kernels); scattered_reads: reads of one 128-byte block each
   * (CSR offset pair, parking index, selected neighbour; node2vec: 4 per step for the searches of its acceptance tests);
   * scattered_writes: stores of one 32-byte write request each (path entry, scattered record); record_bytes: walker
   * records, tasks and bucket tables that are streamed.  Tables that stay in the L2 are not priced.  This sits
   * between the algorithmic bytes of src/main.cu:93-111 (4 * sampled_edges + ...) and what a profiler's HBM counters
   * see; it is an estimate, the counters are the measurement. */
  uint64_t requested_bytes;
  uint64_t list_bytes;
  uint64_t scattered_reads;
  uint64_t scattered_writes;
  uint64_t record_bytes;
} fw_walk_stats;

typedef struct fw_graph fw_graph; /* device CSR mirror: include/gpu_graph.cuh:28-78 */

/* ---- library ---------------------------------------------------------------------------------- */

/* Thread-local text of the last error; replaces the print-and-exit of CUDA_RT_CALL (include/util.cuh:56-68). */
const char* fw_last_error(void);

/* Number of usable devices (0 when there is no GPU); never fails. */
int fw_device_count(void);

/* Free / total device memory in bytes: get_avail_mem (src/util.cu:50-65). */
int fw_device_mem_info(size_t* free_bytes, size_t* total_bytes);

/* Fills defaults: app DeepWalk, d = 80, tp 0.2, p 2.0, q 0.5, schema 0,1,2,3,4, seed 1337 (src/main.cu:40-80). */
void fw_walk_params_default(fw_walk_params* p);

/* The same defaults with `app` set and whatever the library would choose differently for that application (the
 * reference picks node2vec's kernel by application, src/walk.cu:403; this library's choices are the same for all
 * four today). */
void fw_walk_params_default_for(fw_walk_params* p, int app);

/*
 * Autobatch rule of adjust_flags (src/main.cu:259-271):
 *   bs = min((free - headroom_mb * 2^20) / (4 * (d + 2)), INT_MAX); halved unless sync; min(bs, n_queries).
 * d = max_depth - 1.  Returns 0 on invalid input (free <= headroom).
 */
uint32_t fw_autobatch_size(size_t free_bytes, int32_t headroom_mb, int32_t max_depth, int sync, uint32_t n_queries);

/* ---- device buffers (so hosts without a HIP binding can keep inputs resident) ------------------ */

int fw_dev_alloc(size_t bytes, void** d_ptr);
int fw_dev_free(void* d_ptr);
int fw_dev_upload(void* d_dst, const void* h_src, size_t bytes);
int fw_dev_download(void* h_dst, const void* d_src, size_t bytes);
int fw_dev_fill_i32(int32_t* d_dst, int32_t value, size_t count);
/* Plain device-to-device copy kernel (16-byte granularity); also the known-size kernel that HBM traffic
 * counters are calibrated against. */
int fw_dev_copy(void* d_dst, const void* d_src, size_t bytes);
int fw_dev_sync(void);
/*
 * Calibration, no counterpart in the reference: scattered accesses per second over d_buf (at least 1 MiB, 128-byte
 * aligned and sized).  mode 0: 4-byte reads of pseudo-random 64-byte lines; 1 / 2 / 3: 4- / 8- / 16-byte stores into
 * them (a store that does not cover its line costs the memory a read-modify-write); 4 / 5: pairs of 4-byte reads, from
 * the two 64-byte halves of one random 128-byte block / from two random blocks, loads per second (the two rates tell
 * whether the memory is asked for 64 or for 128 bytes at a time).  bench.py reports these next to the walk pipeline's
 * own transaction rate.
 */
int fw_dev_random_access_rate(void* d_buf, size_t bytes, int mode, double* accesses_per_s);

/* ---- graph ------------------------------------------------------------------------------------ */

/*
 * Uploads a host CSR: replaces gpu_graph::gpu_graph(graph*) (include/gpu_graph.cuh:39-78).
 * xadj: uint32[V+1], xadj[0] = 0, xadj[V] = E; adjncy: int32[E]; weight: float32[E] or NULL;
 * label: int32[E] or NULL (the reference uploads weights XOR labels, :50-76; here both may be given).
 * Weights must be finite and >= 0 (checked).  Fails with FW_ERR_INVALID on inconsistent input.
 */
int fw_graph_create(int32_t V, uint64_t E, const uint32_t* h_xadj, const int32_t* h_adjncy,
                    const float* h_weight, const int32_t* h_label, fw_graph** out);

/*
 * Where the edge arrays (adjncy, weight, label) of a graph live.  Replaces FLAGS_umgraph
 * (src/main.cu:48, include/gpu_graph.cuh:46-54: cudaMallocManaged instead of cudaMalloc, for graphs
 * that do not fit the device).  FW_GRAPH_HOST_PINNED keeps them in pinned host memory mapped into the
 * device's address space: the kernels read them over the bus, 64 bytes per request, nothing migrates
 * and nothing has to fit the device except xadj, the parking index (4 bytes per vertex) and the walk
 * buffers.  Results are identical to FW_GRAPH_DEVICE; throughput is bounded by the bus, which hub
 * parking (one read of a hub's list per 64 walkers) relieves.
 */
enum { FW_GRAPH_DEVICE = 0, FW_GRAPH_HOST_PINNED = 1 };
int fw_graph_create_placed(int32_t V, uint64_t E, const uint32_t* h_xadj, const int32_t* h_adjncy,
                           const float* h_weight, const int32_t* h_label, int placement, fw_graph** out);

/*
 * Adopts device arrays that already hold a CSR (e.g. produced by fw_gen_rmat).  The arrays must
 * stay valid until fw_graph_destroy and must be readable 12 bytes past their last element
 * (the kernels use aligned 16-byte loads).  take_ownership != 0: destroy frees them with hipFree.
 */
int fw_graph_adopt_device(int32_t V, uint64_t E, uint32_t* d_xadj, int32_t* d_adjncy, float* d_weight,
                          int32_t* d_label, int take_ownership, fw_graph** out);

int fw_graph_destroy(fw_graph* g);

/* V, E and the maximum degree / its vertex (graph::print_max_degree, include/graph.cuh:209-220). */
int fw_graph_info(const fw_graph* g, int32_t* V, uint64_t* E, int32_t* max_degree, int32_t* max_degree_vertex);

/* 1 when every neighbour list is ascending (equal neighbours allowed; needed by node2vec: include/gpu_graph.cuh:97-118; the walk
 * entry points return FW_ERR_INVALID for FW_APP_NODE2VEC on a graph where this is 0). */
int fw_graph_is_sorted(const fw_graph* g, int* sorted);

/* Copies the device CSR back (any output pointer may be NULL). */
int fw_graph_download(const fw_graph* g, uint32_t* h_xadj, int32_t* h_adjncy, float* h_weight, int32_t* h_label);

/* ---- on-disk CSR: <prefix>_xadj.bin / _edge.bin / _weight.bin / _label.bin ---------------------- */

/*
 * Replaces graph::load_graph (include/graph.cuh:93-190); the layout is the one
 * data/EdgeListToCSR.cpp:216-251 writes: _xadj.bin = int32 V, uint32 E, uint32 xadj[V+1]; _edge.bin =
 * int32 adjncy[E]; _weight.bin = float32[E]; _label.bin = int32[E].  The reference's asserts
 * (:113, :119, :135-136, :155, :176) become FW_ERR_IO with a message.
 */
int fw_csr_read_header(const char* prefix, int32_t* V, uint64_t* E);
/* Reads into caller-owned arrays sized from the header; h_weight / h_label may be NULL (not read). */
int fw_csr_load(const char* prefix, int32_t V, uint64_t E, uint32_t* h_xadj, int32_t* h_adjncy, float* h_weight,
                int32_t* h_label);
/* Writes the four files (weight / label only when given). */
int fw_csr_write(const char* prefix, int32_t V, uint64_t E, const uint32_t* h_xadj, const int32_t* h_adjncy,
                 const float* h_weight, const int32_t* h_label);
/*
 * Host-side: sorts every neighbour list that is not ascending, weight and label moving with their edges
 * (any of the two may be NULL); *lists_sorted (may be NULL) = number of lists that were changed.  The reference's
 * converter writes lists in insertion order (data/EdgeListToCSR.cpp:182-191) although its node2vec binary-searches
 * them (include/gpu_graph.cuh:97-118); the sampling law does not depend on the order inside a list.
 */
int fw_csr_sort_neighbours(int32_t V, const uint32_t* h_xadj, int32_t* h_adjncy, float* h_weight, int32_t* h_label,
                           int64_t* lists_sorted);
/* load + fw_graph_create: graph::graph(...) followed by gpu_graph::gpu_graph(graph*) (src/main.cu:312-325). */
int fw_graph_load(const char* prefix, int want_weight, int want_label, fw_graph** out);
/* The same with the edge arrays placed as fw_graph_create_placed does (--umgraph, src/main.cu:48). */
int fw_graph_load_placed(const char* prefix, int want_weight, int want_label, int placement, fw_graph** out);

/* ---- walks ------------------------------------------------------------------------------------ */

/*
 * One kernel launch over device-resident queries: replaces walk_test + timing<App>() for
 * walk_mode wb_dynamic (src/walk.cu:527-574, :222-248), i.e. kernels walker_wb_dynamic_zprs /
 * _dprs (include/walker.cuh:1307, :1444).
 * d_starts: int32[n]; d_paths: int32[n][max_depth], written completely (-1 padded; the caller does
 * not have to pre-fill it, unlike src/walk.cu:536).  stream: hipStream_t or NULL.  Synchronous:
 * returns after the kernel has finished; stats may be NULL.
 * One walk call at a time per graph: the graph keeps the parking lists, the table of parked-on vertices and the
 * launch record between calls, so a second fw_walk_device / fw_walk_batch on the same fw_graph while one is running
 * (another host thread, whatever the stream) returns FW_ERR_INVALID.  Different graphs are independent.
 */
int fw_walk_device(const fw_graph* g, const fw_walk_params* p, const int32_t* d_starts, int32_t n,
                   int32_t* d_paths, void* stream, fw_walk_stats* stats);

/*
 * fw_walk_device for callers that cannot allocate device memory: tight serving loops that must not touch the allocator,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference (walk_test allocates on every
 * call, src/walk.cu:535-536).  Same arguments, same walks and same counters as fw_walk_device with
 * park_threshold < 0 (one launch, walkers run their whole walks; parking never changes results, so the paths also
 * equal fw_walk_device's under any park_threshold).  The launch scratch (query dispenser word and workload
 * counters, 48 bytes) lives in a 256-byte array inside the library's device image, one copy per device, held
 * until the process ends; the call makes no hipMalloc / hipFree / event creation after its first call on a
 * device.  Like fw_walk_device it is synchronous (it waits for its launch and copies the counters back), so it cannot
 * be recorded into a HIP graph.  n is limited to FW_WALK_NOALLOC_MAX_QUERIES, the largest batch fw_walk_device itself
 * serves with a single launch under its default rule (larger batches are what its parking pipeline and the lists it
 * allocates are for): FW_ERR_INVALID beyond it.  All calls on one device share the array: a call made while another
 * one is running on the same device (two host threads) returns FW_ERR_INVALID; calls one after the other are
 * independent.
 */
#define FW_WALK_NOALLOC_MAX_QUERIES 65535
int fw_walk_device_noalloc(const fw_graph* g, const fw_walk_params* p, const int32_t* d_starts, int32_t n,
                           int32_t* d_paths, void* stream, fw_walk_stats* stats);

/*
 * Batched walk over host queries: replaces walk_batch (src/walk.cu:576-649) with
 * timing_batch_async (two streams, double-buffered H2D / kernel / D2H, :373-466) or, when
 * sync != 0, timing_batch_sync (:468-523).  h_starts: int32[n]; h_paths: int32[n][max_depth],
 * caller-owned (pinned memory gives overlap, pageable works).  batch_size = 0: autobatch.
 * Walker ids are walker_base + query index, whatever the batch size.
 * The device buffers of a call (start vertices, the path matrices of the one or two batches in flight, their parking
 * lists) stay with the graph for the next call and are freed by fw_graph_destroy (the reference allocates and frees
 * them per call, src/walk.cu:586-649): memory that was freed a moment ago keeps the device's copy engines busy, and
 * the next call's path matrix would cross the bus at half its rate.  Autobatch counts them as free memory.
 */
int fw_walk_batch(const fw_graph* g, const fw_walk_params* p, const int32_t* h_starts, int32_t n,
                  uint32_t batch_size, int sync, int32_t* h_paths, fw_walk_stats* stats);

/* Pinned host memory for start points / paths: cudaMallocHost in src/main.cu:275, src/walk.cu:586. */
int fw_host_alloc_pinned(size_t bytes, void** h_ptr);
int fw_host_free_pinned(void* h_ptr);

/* ---- synthetic graphs (the build's own generator; output format of data/EdgeListToCSR.cpp:216-251) */

typedef struct {
  int32_t scale;        /* V = 2^scale */
  int32_t edge_factor;  /* generated edges = edge_factor * V (before dedupe) */
  float a, b, c;        /* R-MAT quadrant probabilities; d = 1 - a - b - c.  a = b = c = 0.25: uniform */
  int32_t symmetrise;   /* insert both directions */
  float w_lo, w_hi;     /* weights uniform in [w_lo, w_hi), equal on both directions */
  int32_t n_labels;     /* labels uniform in [0, n_labels); 0 = no labels */
  int32_t make_weights; /* 0 = no weights */
  uint64_t seed;
} fw_rmat_params;

/*
 * Generates a deduplicated, self-loop-free R-MAT CSR with ascending neighbour lists directly in
 * device memory.  Deterministic in (params).  The CSR has V = 2^scale vertices (isolated vertices kept).
 */
int fw_gen_rmat(const fw_rmat_params* rp, fw_graph** out);

/* ---- sampler micro-benchmark baselines ----------------------------------------------------------- */

/*
 * The three textbook samplers that the reference's sampler test compares its reservoir samplers with
 * (src/sampler_test.cu:290-410 and :561-712; include/sampler.cuh:850-884, :934-968 inverse transform sampling,
 * :970-1100 rejection sampling, :559-790 the alias method), for 64-lane waves.  They are a measuring stick, not part of the walk path.
 * d_weights: float[elements]; task position i draws ONE index from the list_len weights that start at
 * d_tasks[i] * list_len (d_tasks NULL: at i * list_len; every slice must lie inside the array) and writes it to
 * d_out[i] (-1 when no weight of the slice is positive).  workgroup = 0: one wave per task; 1: one workgroup of
 * wg_threads (256, 512 or 1024) per task.  Inverse transform sampling allocates its prefix-sum scratch
 * (list_len floats per resident worker) for the call, the alias method six times as much.  kernel_ms (may be NULL): duration of the one launch.
 */
typedef enum { FW_BASELINE_ITS = 0, FW_BASELINE_RJS = 1, FW_BASELINE_ALS = 2 } fw_baseline_sampler;
int fw_sampler_baseline_run(int type, int workgroup, const float* d_weights, uint64_t elements, uint32_t list_len,
                            const uint32_t* d_tasks, uint32_t n_tasks, int wg_threads, uint64_t seed, int32_t* d_out,
                            double* kernel_ms);

#ifdef __cplusplus
}
#endif
#endif /* FLOWWALKER_H_ */
