// fw_convert -- ASCII edge list -> the on-disk CSR layout the walk engine loads.
//
// Same conversion as the reference's data/EdgeListToCSR.cpp (GetEdgeList :22-65, WriteCSR :132-268):
//   * lines starting with '#' are comments; every other line holds "u v";
//   * the graph becomes undirected: (u, v) and (v, u) are one edge, self loops are dropped, duplicates are dropped;
//   * the normalised pairs (min, max) are sorted, and vertices are renumbered 0, 1, ... in the order in which they
//     first appear in that sorted list (so vertices without edges disappear);
//   * every edge gets ONE label in [0, num_labels) and ONE weight in [1, 5) that both directions share;
//   * neighbour lists keep the order of the sorted pair list;
//   * files: PREFIX_xadj.bin (int32 V, int32 E, uint32 xadj[V+1]), PREFIX_edge.bin, PREFIX_label.bin,
//     PREFIX_weight.bin (E entries each) and PREFIX.edgelist (the renumbered directed pairs, "u v" per line).
// Differences: the random stream is seeded (--seed, default 1; the reference seeds from the OS entropy source, so its
// labels and weights are not reproducible), and --sorted writes ascending neighbour lists, which node2vec needs
// (the reference's order is ascending only for graphs whose renumbering happens to be monotone).
//
//   fw_convert INPUT PREFIX NUM_LABELS [--seed S] [--sorted] [--wlo 1 --whi 5]

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <fstream>
#include <numeric>
#include <random>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "flowwalker.h"

int main(int argc, char** argv) {
  if (argc < 4) {
    fprintf(stderr, "usage: fw_convert INPUT PREFIX NUM_LABELS [--seed S] [--sorted] [--wlo 1 --whi 5]\n");
    return 2;
  }
  const std::string input = argv[1], prefix = argv[2];
  const int num_labels = atoi(argv[3]);
  unsigned long long seed = 1;
  bool sorted = false;
  double wlo = 1.0, whi = 5.0;
  for (int i = 4; i < argc; ++i) {
    const std::string k = argv[i];
    auto val = [&]() -> const char* {
      if (i + 1 >= argc) { fprintf(stderr, "fw_convert: %s needs a value\n", k.c_str()); exit(2); }
      return argv[++i];
    };
    if (k == "--seed") seed = strtoull(val(), nullptr, 10);
    else if (k == "--sorted") sorted = true;
    else if (k == "--wlo") wlo = atof(val());
    else if (k == "--whi") whi = atof(val());
    else { fprintf(stderr, "fw_convert: unknown flag %s\n", k.c_str()); return 2; }
  }
  if (num_labels < 1) { fprintf(stderr, "fw_convert: NUM_LABELS must be at least 1\n"); return 2; }
  if (!(wlo >= 0.0) || !(whi > wlo)) { fprintf(stderr, "fw_convert: need 0 <= wlo < whi\n"); return 2; }

  // read and normalise
  std::ifstream ifs(input);
  if (!ifs.good()) { fprintf(stderr, "fw_convert: cannot open %s\n", input.c_str()); return 1; }
  std::vector<std::pair<int64_t, int64_t>> pairs;
  std::string line;
  size_t line_no = 0;
  while (std::getline(ifs, line)) {
    ++line_no;
    if (line.empty() || line[0] == '#') continue;
    char* end = nullptr;
    const long long u = strtoll(line.c_str(), &end, 10);
    if (end == line.c_str()) continue;  // no number on the line
    char* end2 = nullptr;
    const long long v = strtoll(end, &end2, 10);
    if (end2 == end) { fprintf(stderr, "fw_convert: line %zu has one number only\n", line_no); return 1; }
    if (u < 0 || v < 0 || u >= INT32_MAX || v >= INT32_MAX) {
      fprintf(stderr, "fw_convert: line %zu: vertex id out of range\n", line_no);
      return 1;
    }
    if (u == v) continue;
    pairs.emplace_back(std::min(u, v), std::max(u, v));
  }
  std::sort(pairs.begin(), pairs.end());
  pairs.erase(std::unique(pairs.begin(), pairs.end()), pairs.end());
  if (pairs.size() * 2 > 0xFFFFFFF0ull) { fprintf(stderr, "fw_convert: too many edges for 32-bit CSR offsets\n"); return 1; }

  // renumber in order of first appearance
  std::unordered_map<int64_t, int32_t> renum;
  renum.reserve(pairs.size());
  auto id_of = [&](int64_t x) -> int32_t {
    auto it = renum.find(x);
    if (it != renum.end()) return it->second;
    const int32_t id = (int32_t)renum.size();
    renum.emplace(x, id);
    return id;
  };
  std::vector<std::pair<int32_t, int32_t>> edges(pairs.size());
  for (size_t i = 0; i < pairs.size(); ++i) {
    const int32_t a = id_of(pairs[i].first);  // src first, then dst: the reference's order of assignment
    const int32_t b = id_of(pairs[i].second);
    edges[i] = {a, b};
  }
  const int32_t V = (int32_t)renum.size();
  const uint64_t E = 2ull * edges.size();

  // one label and one weight per undirected edge
  std::mt19937_64 gen(seed);
  std::uniform_int_distribution<int> dl(0, num_labels - 1);
  std::uniform_real_distribution<double> dw(wlo, whi);
  std::vector<int32_t> elabel(edges.size());
  std::vector<float> eweight(edges.size());
  for (size_t i = 0; i < edges.size(); ++i) {
    elabel[i] = dl(gen);
    float w = (float)dw(gen);
    if (!(w < (float)whi)) w = (float)wlo;  // the float rounding of a double just below whi
    eweight[i] = w;
  }

  // CSR by counting; lists keep the order of the pair list
  std::vector<uint32_t> xadj((size_t)V + 1, 0u);
  for (const auto& e : edges) { ++xadj[(size_t)e.first + 1]; ++xadj[(size_t)e.second + 1]; }
  for (int32_t v = 0; v < V; ++v) xadj[(size_t)v + 1] += xadj[v];
  std::vector<int32_t> adj(E), lab(E);
  std::vector<float> wgt(E);
  {
    std::vector<uint32_t> fill(xadj.begin(), xadj.end() - 1);
    for (size_t i = 0; i < edges.size(); ++i) {
      const int32_t a = edges[i].first, b = edges[i].second;
      const uint32_t pa = fill[a]++, pb = fill[b]++;
      adj[pa] = b; lab[pa] = elabel[i]; wgt[pa] = eweight[i];
      adj[pb] = a; lab[pb] = elabel[i]; wgt[pb] = eweight[i];
    }
  }
  if (sorted) {
    std::vector<uint32_t> order;
    std::vector<int32_t> ta, tl;
    std::vector<float> tw;
    for (int32_t v = 0; v < V; ++v) {
      const uint32_t b = xadj[v], n = xadj[(size_t)v + 1] - b;
      order.resize(n);
      std::iota(order.begin(), order.end(), 0u);
      std::sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) { return adj[b + x] < adj[b + y]; });
      ta.resize(n); tl.resize(n); tw.resize(n);
      for (uint32_t i = 0; i < n; ++i) { ta[i] = adj[b + order[i]]; tl[i] = lab[b + order[i]]; tw[i] = wgt[b + order[i]]; }
      std::copy(ta.begin(), ta.end(), adj.begin() + b);
      std::copy(tl.begin(), tl.end(), lab.begin() + b);
      std::copy(tw.begin(), tw.end(), wgt.begin() + b);
    }
  }

  if (fw_csr_write(prefix.c_str(), V, E, xadj.data(), adj.data(), wgt.data(), lab.data()) != FW_OK) {
    fprintf(stderr, "fw_convert: writing %s: %s\n", prefix.c_str(), fw_last_error());
    return 1;
  }
  {
    FILE* f = fopen((prefix + ".edgelist").c_str(), "w");
    if (!f) { fprintf(stderr, "fw_convert: cannot write %s.edgelist\n", prefix.c_str()); return 1; }
    for (int32_t v = 0; v < V; ++v)
      for (uint32_t i = xadj[v]; i < xadj[(size_t)v + 1]; ++i) fprintf(f, "%d %d\n", v, adj[i]);
    fclose(f);
  }
  printf("vertices: %d\nCSR entries: %llu (undirected edges: %zu)\nneighbour lists: %s\n", V, (unsigned long long)E,
         edges.size(), sorted ? "ascending" : "order of the sorted pair list");
  return 0;
}
