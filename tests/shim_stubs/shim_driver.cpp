// Driver for fw_shim.cpp: the prototypes below are the reference's (include/walker.cuh:49-57, default arguments
// included); the flag variables are what its src/main.cu:40-80 DEFINEs.  Builds a small CSR, calls both entry points the
// way src/main.cu:346-357 does and writes the two path matrices to the files named on the command line.
#include <stdio.h>
#include <stdlib.h>
#include <algorithm>
#include <vector>

#include "flowwalker.h"
#include "graph.cuh"

struct gpu_graph;
gpu_graph* shim_make_gpu_graph(graph* g);
double walk_test(vtx_t*& result_pool_ptr, gpu_graph* graph, vtx_t* start_points, int max_depth, int num_walkers,
                 walk_mode type, int* schema = NULL, int schema_len = 0);
double walk_batch(vtx_t*& result_pool, gpu_graph* graph, vtx_t* start_points, int max_depth, int num_walkers,
                  int batch_size, int* schema = NULL, int schema_len = 0);

bool FLAGS_deepwalk = true, FLAGS_ppr = false, FLAGS_node2vec = false, FLAGS_metapath = false;
bool FLAGS_dprs = false, FLAGS_syn = false;
double FLAGS_p = 2.0, FLAGS_q = 0.5, FLAGS_tp = 0.2;

int main(int argc, char** argv) {
  if (argc < 3) return 2;
  const int V = 2000, deg = 12, depth = 21, n = 500;
  std::vector<edge_t> xadj(V + 1);
  std::vector<vtx_t> adj((size_t)V * deg);
  std::vector<weight_t> w((size_t)V * deg);
  for (int v = 0; v <= V; ++v) xadj[v] = (edge_t)(v * deg);
  for (int v = 0; v < V; ++v)
    for (int k = 0; k < deg; ++k) {  // ascending neighbour lists, no self-loops
      adj[(size_t)v * deg + k] = (v + 1 + k * 37) % V;
      w[(size_t)v * deg + k] = 1.0f + (float)((v * 31 + k * 17) % 97);
    }
  for (int v = 0; v < V; ++v) std::sort(adj.begin() + (size_t)v * deg, adj.begin() + (size_t)(v + 1) * deg);
  graph g = {xadj.data(), adj.data(), w.data(), nullptr, V, (edge_t)adj.size()};
  gpu_graph* gg = shim_make_gpu_graph(&g);
  std::vector<vtx_t> starts(n);
  for (int i = 0; i < n; ++i) starts[i] = (i * 7) % V;

  vtx_t* d_res = nullptr;
  const double ms_test = walk_test(d_res, gg, starts.data(), depth, n, wb_dynamic);
  std::vector<vtx_t> from_test((size_t)n * depth);
  if (fw_dev_download(from_test.data(), d_res, from_test.size() * sizeof(vtx_t)) != FW_OK) return 3;
  vtx_t* h_res = nullptr;
  const double ms_batch = walk_batch(h_res, gg, starts.data(), depth, n, 128);
  FILE* f = fopen(argv[1], "wb");
  fwrite(from_test.data(), sizeof(vtx_t), from_test.size(), f);
  fclose(f);
  f = fopen(argv[2], "wb");
  fwrite(h_res, sizeof(vtx_t), (size_t)n * depth, f);
  fclose(f);
  printf("walk_test %.3f ms, walk_batch %.3f ms\n", ms_test, ms_batch);
  return 0;
}
