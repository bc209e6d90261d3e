// On-disk CSR in the reference's layout (written by data/EdgeListToCSR.cpp:216-251, read by
// graph::load_graph, include/graph.cuh:93-190), little-endian:
//   <prefix>_xadj.bin   int32 V, uint32 E, uint32 xadj[V+1]      (file size 4 * (V + 3))
//   <prefix>_edge.bin   int32 adjncy[E]
//   <prefix>_weight.bin float32 weight[E]   (read unless metapath: include/graph.cuh:163-185)
//   <prefix>_label.bin  int32 label[E]      (read only for metapath: include/graph.cuh:145-162)
// Host-only code; failures are status codes with a message instead of the reference's asserts.

#include <stdio.h>
#include <string.h>
#include <sys/stat.h>

#include <algorithm>
#include <string>
#include <vector>

#include "fw_internal.h"

namespace {

long long file_size(const std::string& path) {
  struct stat st;
  if (stat(path.c_str(), &st) != 0) return -1;
  return (long long)st.st_size;
}

int read_exact(const std::string& path, long long offset, void* dst, size_t bytes) {
  FILE* f = fopen(path.c_str(), "rb");
  if (!f) { fw_set_error("cannot open %s", path.c_str()); return FW_ERR_IO; }
  if (offset && fseek(f, (long)offset, SEEK_SET) != 0) { fclose(f); fw_set_error("cannot seek in %s", path.c_str()); return FW_ERR_IO; }
  const size_t got = fread(dst, 1, bytes, f);
  fclose(f);
  if (got != bytes) { fw_set_error("%s is short: wanted %zu bytes, got %zu", path.c_str(), bytes, got); return FW_ERR_IO; }
  return FW_OK;
}

int write_all(const std::string& path, const void* a, size_t abytes, const void* b, size_t bbytes) {
  FILE* f = fopen(path.c_str(), "wb");
  if (!f) { fw_set_error("cannot create %s", path.c_str()); return FW_ERR_IO; }
  bool ok = (abytes == 0 || fwrite(a, 1, abytes, f) == abytes) && (bbytes == 0 || fwrite(b, 1, bbytes, f) == bbytes);
  ok = (fclose(f) == 0) && ok;
  if (!ok) { fw_set_error("short write to %s", path.c_str()); return FW_ERR_IO; }
  return FW_OK;
}

}  // namespace

extern "C" int fw_csr_read_header(const char* prefix, int32_t* V, uint64_t* E) {
  if (!prefix || !V || !E) { fw_set_error("fw_csr_read_header: NULL argument"); return FW_ERR_INVALID; }
  const std::string xf = std::string(prefix) + "_xadj.bin";
  const std::string ef = std::string(prefix) + "_edge.bin";
  const long long xs = file_size(xf), es = file_size(ef);
  if (xs < 0) { fw_set_error("xadj file cannot open: %s", xf.c_str()); return FW_ERR_IO; }
  if (es < 0) { fw_set_error("CSR file cannot open: %s", ef.c_str()); return FW_ERR_IO; }
  if (xs < 12 || (xs % 4) != 0 || (es % 4) != 0) { fw_set_error("%s / %s: sizes are not whole 32-bit words", xf.c_str(), ef.c_str()); return FW_ERR_IO; }
  struct { int32_t v; uint32_t e; } hdr;
  int rc = read_exact(xf, 0, &hdr, sizeof(hdr));
  if (rc != FW_OK) return rc;
  // include/graph.cuh:99-100: the sizes are derived from the files first, then the header overrides V
  const long long v_from_size = xs / 4 - 3;
  const long long e_from_size = es / 4;
  if ((long long)hdr.v != v_from_size) {
    fw_set_error("%s: header says %d vertices, file size says %lld", xf.c_str(), hdr.v, v_from_size);
    return FW_ERR_IO;
  }
  if ((long long)hdr.e != e_from_size) {
    fw_set_error("%s: header says %u edges, %s holds %lld", xf.c_str(), hdr.e, ef.c_str(), e_from_size);
    return FW_ERR_IO;
  }
  if (hdr.v <= 0 || hdr.e == 0) { fw_set_error("%s: empty graph", xf.c_str()); return FW_ERR_IO; }
  *V = hdr.v;
  *E = hdr.e;
  return FW_OK;
}

extern "C" int fw_csr_load(const char* prefix, int32_t V, uint64_t E, uint32_t* h_xadj, int32_t* h_adjncy,
                           float* h_weight, int32_t* h_label) {
  if (!prefix || !h_xadj || !h_adjncy) { fw_set_error("fw_csr_load: NULL argument"); return FW_ERR_INVALID; }
  int32_t hv = 0;
  uint64_t he = 0;
  int rc = fw_csr_read_header(prefix, &hv, &he);
  if (rc != FW_OK) return rc;
  if (hv != V || he != E) { fw_set_error("fw_csr_load: V/E do not match the header (%d, %llu)", hv, (unsigned long long)he); return FW_ERR_INVALID; }
  const std::string p(prefix);
  if ((rc = read_exact(p + "_xadj.bin", 8, h_xadj, (size_t)(V + 1) * 4)) != FW_OK) return rc;
  if ((uint64_t)h_xadj[V] != E) {  // include/graph.cuh:135-136
    fw_set_error("%s_xadj.bin: xadj[V] = %u but the edge file holds %llu entries", prefix, h_xadj[V], (unsigned long long)E);
    return FW_ERR_IO;
  }
  if ((rc = read_exact(p + "_edge.bin", 0, h_adjncy, (size_t)E * 4)) != FW_OK) return rc;
  if (h_weight) {
    if (file_size(p + "_weight.bin") != (long long)E * 4) { fw_set_error("File cannot open or has the wrong size: %s_weight.bin", prefix); return FW_ERR_IO; }
    if ((rc = read_exact(p + "_weight.bin", 0, h_weight, (size_t)E * 4)) != FW_OK) return rc;
  }
  if (h_label) {
    if (file_size(p + "_label.bin") != (long long)E * 4) { fw_set_error("File cannot open or has the wrong size: %s_label.bin", prefix); return FW_ERR_IO; }
    if ((rc = read_exact(p + "_label.bin", 0, h_label, (size_t)E * 4)) != FW_OK) return rc;
  }
  return FW_OK;
}

extern "C" int fw_csr_write(const char* prefix, int32_t V, uint64_t E, const uint32_t* h_xadj, const int32_t* h_adjncy,
                            const float* h_weight, const int32_t* h_label) {
  if (!prefix || !h_xadj || !h_adjncy || V <= 0 || E == 0 || E > 0xFFFFFFF0ull) {
    fw_set_error("fw_csr_write: bad argument");
    return FW_ERR_INVALID;
  }
  const std::string p(prefix);
  struct { int32_t v; uint32_t e; } hdr = {V, (uint32_t)E};
  int rc;
  if ((rc = write_all(p + "_xadj.bin", &hdr, sizeof(hdr), h_xadj, (size_t)(V + 1) * 4)) != FW_OK) return rc;
  if ((rc = write_all(p + "_edge.bin", h_adjncy, (size_t)E * 4, nullptr, 0)) != FW_OK) return rc;
  if (h_weight && (rc = write_all(p + "_weight.bin", h_weight, (size_t)E * 4, nullptr, 0)) != FW_OK) return rc;
  if (h_label && (rc = write_all(p + "_label.bin", h_label, (size_t)E * 4, nullptr, 0)) != FW_OK) return rc;
  return FW_OK;
}

// Sorts every neighbour list that is not ascending, carrying weight and label with their edges.  The reference's
// converter writes lists in insertion order (data/EdgeListToCSR.cpp:182-191) while node2vec's adjacency test
// binary-searches them (include/gpu_graph.cuh:97-118); the sampling law does not depend on the order of a list.
extern "C" int fw_csr_sort_neighbours(int32_t V, const uint32_t* h_xadj, int32_t* h_adjncy, float* h_weight,
                                      int32_t* h_label, int64_t* lists_sorted) {
  if (V <= 0 || !h_xadj || !h_adjncy) { fw_set_error("fw_csr_sort_neighbours: bad argument"); return FW_ERR_INVALID; }
  int64_t touched = 0;
  std::vector<uint32_t> perm;
  std::vector<int32_t> ta, tl;
  std::vector<float> tw;
  for (int32_t v = 0; v < V; ++v) {
    const uint32_t b = h_xadj[v], e = h_xadj[v + 1];
    bool ascending = true;
    for (uint32_t i = b + 1; i < e && ascending; ++i) ascending = h_adjncy[i - 1] <= h_adjncy[i];
    if (ascending) continue;
    ++touched;
    const uint32_t d = e - b;
    perm.resize(d);
    for (uint32_t i = 0; i < d; ++i) perm[i] = i;
    std::stable_sort(perm.begin(), perm.end(), [&](uint32_t x, uint32_t y) { return h_adjncy[b + x] < h_adjncy[b + y]; });
    ta.resize(d);
    for (uint32_t i = 0; i < d; ++i) ta[i] = h_adjncy[b + perm[i]];
    std::copy(ta.begin(), ta.end(), h_adjncy + b);
    if (h_weight) {
      tw.resize(d);
      for (uint32_t i = 0; i < d; ++i) tw[i] = h_weight[b + perm[i]];
      std::copy(tw.begin(), tw.end(), h_weight + b);
    }
    if (h_label) {
      tl.resize(d);
      for (uint32_t i = 0; i < d; ++i) tl[i] = h_label[b + perm[i]];
      std::copy(tl.begin(), tl.end(), h_label + b);
    }
  }
  if (lists_sorted) *lists_sorted = touched;
  return FW_OK;
}

extern "C" int fw_graph_load(const char* prefix, int want_weight, int want_label, fw_graph** out) {
  return fw_graph_load_placed(prefix, want_weight, want_label, FW_GRAPH_DEVICE, out);
}

extern "C" int fw_graph_load_placed(const char* prefix, int want_weight, int want_label, int placement,
                                    fw_graph** out) {
  if (!out) { fw_set_error("fw_graph_load: out is NULL"); return FW_ERR_INVALID; }
  *out = nullptr;
  int32_t V = 0;
  uint64_t E = 0;
  int rc = fw_csr_read_header(prefix, &V, &E);
  if (rc != FW_OK) return rc;
  std::vector<uint32_t> xadj((size_t)V + 1);
  std::vector<int32_t> adj((size_t)E);
  std::vector<float> w(want_weight ? (size_t)E : 0);
  std::vector<int32_t> lab(want_label ? (size_t)E : 0);
  rc = fw_csr_load(prefix, V, E, xadj.data(), adj.data(), want_weight ? w.data() : nullptr,
                   want_label ? lab.data() : nullptr);
  if (rc != FW_OK) return rc;
  return fw_graph_create_placed(V, E, xadj.data(), adj.data(), want_weight ? w.data() : nullptr,
                                want_label ? lab.data() : nullptr, placement, out);
}
