// fw_shim.cpp -- drop-in for the reference's src/walk.cu: keeps its two host entry points
//   double walk_test(...), double walk_batch(...)   (include/walker.cuh:49-57)
// and its device graph type, and runs them on libflowwalker_hip.so.  A maintainer of the reference compiles this
// file instead of walk.cu / walker.cuh / sampler.cuh / myrand.cuh / gpu_graph.cuh and links -lflowwalker_hip.
// tests/test_shim.py compiles it against stand-ins of <gflags/gflags.h> and graph.cuh that declare only what it uses,
// together with a driver that holds the reference's prototypes.
#include <stdio.h>
#include <stdlib.h>

#include <gflags/gflags.h>
#include "flowwalker.h"
#include "graph.cuh"            // host CSR loader of the reference (include/graph.cuh)

DECLARE_bool(deepwalk); DECLARE_bool(ppr); DECLARE_bool(node2vec); DECLARE_bool(metapath);
DECLARE_bool(dprs); DECLARE_bool(syn);
DECLARE_double(p); DECLARE_double(q); DECLARE_double(tp);

struct gpu_graph {               // replaces include/gpu_graph.cuh:28-78
  fw_graph* h = nullptr;
  explicit gpu_graph(graph* g) {
    if (fw_graph_create(g->vert_count, g->edge_count, g->xadj, g->adjncy,
                        FLAGS_metapath ? nullptr : g->weight, FLAGS_metapath ? g->edge_label : nullptr, &h))
      { fprintf(stderr, "%s\n", fw_last_error()); exit(1); }
  }
  ~gpu_graph() { fw_graph_destroy(h); }
};

static fw_walk_params params_from_flags(int max_depth, int* schema, int schema_len) {
  fw_walk_params P;  // the library's choices for the application
  fw_walk_params_default_for(&P, FLAGS_deepwalk ? FW_APP_DEEPWALK : FLAGS_ppr ? FW_APP_PPR
                                 : FLAGS_node2vec ? FW_APP_NODE2VEC : FW_APP_METAPATH);
  P.sampler = FLAGS_dprs ? FW_SAMPLER_DPRS : FW_SAMPLER_ZPRS;
  P.max_depth = max_depth; P.tp = FLAGS_tp; P.p = FLAGS_p; P.q = FLAGS_q;
  P.schema_len = schema_len; for (int i = 0; i < schema_len; i++) P.schema[i] = schema[i];
  return P;
}

// src/walk.cu:576-649.  result_pool: pinned host matrix, allocated here as the reference does.
double walk_batch(vtx_t*& result_pool, gpu_graph* g, vtx_t* start_points, int max_depth, int num_walkers,
                  int batch_size, int* schema, int schema_len) {
  fw_walk_params P = params_from_flags(max_depth, schema, schema_len);
  fw_host_alloc_pinned((size_t)num_walkers * max_depth * sizeof(vtx_t), (void**)&result_pool);
  fw_walk_stats st;
  if (fw_walk_batch(g->h, &P, start_points, num_walkers, batch_size, FLAGS_syn, result_pool, &st))
    { fprintf(stderr, "%s\n", fw_last_error()); exit(1); }
  return st.total_ms;             // milliseconds, transfers included (src/walk.cu:465)
}

// src/walk.cu:527-574.  result_pool_ptr: device matrix, as in the reference (print_res copies it back).
double walk_test(vtx_t*& result_pool_ptr, gpu_graph* g, vtx_t* start_points, int max_depth, int num_walkers,
                 walk_mode /*wb_dynamic only*/, int* schema, int schema_len) {
  fw_walk_params P = params_from_flags(max_depth, schema, schema_len);
  void *d_starts, *d_paths;
  fw_dev_alloc((size_t)num_walkers * 4, &d_starts);
  fw_dev_alloc((size_t)num_walkers * max_depth * 4, &d_paths);
  fw_dev_upload(d_starts, start_points, (size_t)num_walkers * 4);
  fw_walk_stats st;
  if (fw_walk_device(g->h, &P, (int32_t*)d_starts, num_walkers, (int32_t*)d_paths, nullptr, &st))
    { fprintf(stderr, "%s\n", fw_last_error()); exit(1); }
  result_pool_ptr = (vtx_t*)d_paths;
  return st.kernel_ms;
}

// for callers that only see gpu_graph as an incomplete type
gpu_graph* shim_make_gpu_graph(graph* g) { return new gpu_graph(g); }
