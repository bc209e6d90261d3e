// fw_gen -- writes synthetic graphs in the reference's on-disk CSR layout
// (<prefix>_xadj.bin / _edge.bin / _weight.bin / _label.bin, data/EdgeListToCSR.cpp:216-251).
//
//   fw_gen --out PREFIX --kind rmat --scale 22 [--edgefactor 16] [--a .57 --b .19 --c .19] [--sym]
//          [--wlo 1 --whi 100] [--labels 5] [--seed 1]          (generated on the GPU)
//   fw_gen --out PREFIX --kind uniform --vertices 7115 --edges 103689 [--wlo 1 --whi 5] [--labels 5] [--seed 1]
//                                                               (generated on the host)

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <random>
#include <string>
#include <vector>

#include "flowwalker.h"

static int fail(const char* what) {
  fprintf(stderr, "fw_gen: %s: %s\n", what, fw_last_error());
  return 1;
}

int main(int argc, char** argv) {
  std::string out, kind = "rmat";
  int scale = 16, ef = 16, labels = 5, sym = 0;
  long long vertices = 7115, edges = 103689;
  double a = 0.57, b = 0.19, c = 0.19, wlo = 1.0, whi = 100.0;
  unsigned long long seed = 1;
  for (int i = 1; i < argc; ++i) {
    const std::string k = argv[i];
    auto val = [&]() -> const char* { if (i + 1 >= argc) { fprintf(stderr, "fw_gen: %s needs a value\n", k.c_str()); exit(2); } return argv[++i]; };
    if (k == "--out") out = val();
    else if (k == "--kind") kind = val();
    else if (k == "--scale") scale = atoi(val());
    else if (k == "--edgefactor") ef = atoi(val());
    else if (k == "--a") a = atof(val());
    else if (k == "--b") b = atof(val());
    else if (k == "--c") c = atof(val());
    else if (k == "--sym") sym = 1;
    else if (k == "--wlo") wlo = atof(val());
    else if (k == "--whi") whi = atof(val());
    else if (k == "--labels") labels = atoi(val());
    else if (k == "--seed") seed = strtoull(val(), nullptr, 10);
    else if (k == "--vertices") vertices = atoll(val());
    else if (k == "--edges") edges = atoll(val());
    else { fprintf(stderr, "fw_gen: unknown flag %s\n", k.c_str()); return 2; }
  }
  if (out.empty()) { fprintf(stderr, "fw_gen: --out PREFIX is required\n"); return 2; }

  if (kind == "rmat") {
    fw_rmat_params rp;
    memset(&rp, 0, sizeof(rp));
    rp.scale = scale; rp.edge_factor = ef; rp.a = (float)a; rp.b = (float)b; rp.c = (float)c;
    rp.symmetrise = sym; rp.w_lo = (float)wlo; rp.w_hi = (float)whi; rp.n_labels = labels; rp.make_weights = 1;
    rp.seed = seed;
    fw_graph* g = nullptr;
    if (fw_gen_rmat(&rp, &g) != FW_OK) return fail("generating");
    int32_t V = 0; uint64_t E = 0;
    fw_graph_info(g, &V, &E, nullptr, nullptr);
    std::vector<uint32_t> xadj((size_t)V + 1);
    std::vector<int32_t> adj((size_t)E), lab(labels > 0 ? (size_t)E : 0);
    std::vector<float> w((size_t)E);
    if (fw_graph_download(g, xadj.data(), adj.data(), w.data(), labels > 0 ? lab.data() : nullptr) != FW_OK) return fail("downloading");
    if (fw_csr_write(out.c_str(), V, E, xadj.data(), adj.data(), w.data(), labels > 0 ? lab.data() : nullptr) != FW_OK) return fail("writing");
    printf("fw_gen: R-MAT scale %d: %d vertices, %llu CSR entries -> %s_*.bin\n", scale, V, (unsigned long long)E, out.c_str());
    fw_graph_destroy(g);
    return 0;
  }
  if (kind == "uniform") {
    if (vertices < 2 || edges < 1 || edges > vertices * (vertices - 1)) { fprintf(stderr, "fw_gen: impossible vertex / edge counts\n"); return 2; }
    std::mt19937_64 rng(seed);
    std::vector<uint64_t> keys;
    keys.reserve((size_t)edges * 2);
    while ((long long)keys.size() < edges) {  // distinct (src != dst) pairs, exactly `edges` of them
      const long long need = edges - (long long)keys.size();
      for (long long i = 0; i < need + need / 4 + 16; ++i) {
        const uint64_t s = rng() % (uint64_t)vertices, d = rng() % (uint64_t)vertices;
        if (s != d) keys.push_back((s << 32) | d);
      }
      std::sort(keys.begin(), keys.end());
      keys.erase(std::unique(keys.begin(), keys.end()), keys.end());
    }
    while ((long long)keys.size() > edges) {
      keys.erase(keys.begin() + (long long)(rng() % keys.size()));
    }
    const int32_t V = (int32_t)vertices;
    const uint64_t E = keys.size();
    std::vector<uint32_t> xadj((size_t)V + 1, 0);
    std::vector<int32_t> adj(E), lab(E);
    std::vector<float> w(E);
    std::uniform_real_distribution<float> wd((float)wlo, (float)whi);
    for (uint64_t i = 0; i < E; ++i) {
      xadj[(keys[i] >> 32) + 1]++;
      adj[i] = (int32_t)(keys[i] & 0xFFFFFFFFu);
      float x = wd(rng);
      if (x >= (float)whi) x = (float)wlo;
      w[i] = x;
      lab[i] = labels > 0 ? (int32_t)(rng() % (uint64_t)labels) : 0;
    }
    for (int32_t v = 0; v < V; ++v) xadj[v + 1] += xadj[v];
    if (fw_csr_write(out.c_str(), V, E, xadj.data(), adj.data(), w.data(), labels > 0 ? lab.data() : nullptr) != FW_OK) return fail("writing");
    printf("fw_gen: uniform graph: %d vertices, %llu CSR entries -> %s_*.bin\n", V, (unsigned long long)E, out.c_str());
    return 0;
  }
  fprintf(stderr, "fw_gen: --kind must be rmat or uniform\n");
  return 2;
}
