// Stand-in for the reference's include/graph.cuh + include/util.cuh, declaring only what fw_shim.cpp touches: the
// scalar types (include/util.cuh:38-40), the host CSR object's public fields (include/graph.cuh:38-60) and the
// walk_mode enumeration (include/walker.cuh:30-45).
#pragma once
#include <stdint.h>
typedef int vtx_t;
typedef unsigned int edge_t;
typedef float weight_t;
struct graph {
  edge_t* xadj;
  vtx_t* adjncy;
  weight_t* weight;
  vtx_t* edge_label;
  vtx_t vert_count;
  edge_t edge_count;
};
enum walk_mode { wp, wb, twb, queue, tw, twb_dynamic, wb_dynamic, w_dynamic, b_dynamic, wb_curand, wb_dprs, wb_dynamic_dprs,
                 wb_curand_zprs };
