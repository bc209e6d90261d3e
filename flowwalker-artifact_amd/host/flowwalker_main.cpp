// flowwalker -- command-line front end with the reference's flag surface (src/main.cu:40-80, :298-384),
// calling the HIP engine through the C ABI of libflowwalker_hip.so.
//
//   flowwalker --input PREFIX (--deepwalk | --ppr | --node2vec | --metapath)
//              [--n N | --all] [--seq] [--d D] [--batch] [--batchsize B] [--autobatch] [--headroom MB] [--syn]
//              [--tp T] [--p P] [--q Q] [--schema 0,1,2] [--dprs] [--printresult] [--printworkload]
//              [--seed S] [--pprstart maxdeg|seq] [--hub_threshold T] [--wg_threads W] [--park_threshold P]
//              [--walkmode M] [--savepaths FILE]
//
// Flags follow gflags syntax: --flag, --flag=value, --flag value, --noflag.  Differences from the
// reference, on purpose: random start vertices come from --seed instead of time(NULL) (src/main.cu:284),
// the first min(100, n) walkers are printed (the reference always prints 100 and reads out of bounds for
// smaller n: src/main.cu:165), errors return a non-zero status with a message instead of exit() inside a
// macro, --lognorm draws its weights from a seeded host generator, --umgraph keeps the edge arrays in pinned host
// memory that the kernels read over the bus (the reference uses managed memory that migrates by page,
// include/gpu_graph.cuh:46-54).  --walkmode keeps the reference's ablation levels (README.md:152-163), run by the
// reference's own algorithms restated for 64-lane waves (FW_SAMPLER_REF_*: two-pass ZPRS / chunked DPRS, 64 task
// slots per workgroup), and adds this engine's own levels:
//   --walkmode=9       "FW": the reference's DPRS samplers, static query assignment, generators that belong to the threads
//                      with their state in device memory (cuRAND's place: walker_wb_dprs_curand, include/walker.cuh:1584)
//   --walkmode=10      "FW + RNG": the same with the generators' state in LDS, structure of arrays (include/myrand.cuh:83-86;
//                      walker_wb_dprs, include/walker.cuh:1813): the same walks as 9, cheaper draws
//   --walkmode=1       "FW + ZPRS": the reference's ZPRS samplers, static query assignment, generators in LDS (walker_wb, :172)
//   --walkmode=6       "FW + DS": the reference's ZPRS samplers with the global query dispenser (its default kernel, :1307);
//                      draws addressed by (walker, step, element), because a generator owned by a thread gives other
//                      walks on every run once the queries are handed out dynamically
//   --walkmode=20      this engine's walk kernel alone, every list sampled by one wave (no workgroup sampler, no parking)
//   --walkmode=21      + the workgroup sampler for lists above --hub_threshold
//   --walkmode=22      + parking: walkers waiting on the same vertex share one scan of its list (the default)
// --park_threshold passes fw_walk_params.park_threshold through (0 library rule, < 0 off, > 0 explicit degree).

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <chrono>
#include <map>
#include <random>
#include <string>
#include <vector>

#include "flowwalker.h"

namespace {

struct Flags {
  std::string input = "../data/wiki-Vote";
  std::string b_file = "../res/bucket.csv";
  int n = 4000;
  bool seq = false, all = false;
  int d = 80;
  bool umgraph = false;
  bool deepwalk = false, node2vec = false, ppr = false, metapath = false;
  bool dprs = false;
  double p = 2.0, q = 0.5, tp = 0.2;
  int schemalen = 5;
  std::string schema = "0,1,2,3,4";
  bool printresult = false, printworkload = false, save_degree = false;
  bool autobatch = false, batch = false, syn = false;
  unsigned batchsize = 10000000;
  int headroom = 512;
  int walkmode = -1;
  bool lognorm = false;
  // additions of this build
  long long seed = 1337;
  std::string pprstart = "maxdeg";
  int hub_threshold = -1;
  int wg_threads = 0;
  int park_threshold = 0;
  std::string savepaths;
};

enum Kind { kBool, kInt, kUint, kLong, kDouble, kString };
struct Spec { Kind kind; void* ptr; };

int fail(const char* what) {
  fprintf(stderr, "flowwalker: %s: %s\n", what, fw_last_error());
  return 1;
}

bool parse_flags(int argc, char** argv, Flags* f) {
  const std::map<std::string, Spec> specs = {
      {"input", {kString, &f->input}},       {"b_file", {kString, &f->b_file}},
      {"n", {kInt, &f->n}},                  {"seq", {kBool, &f->seq}},
      {"all", {kBool, &f->all}},             {"d", {kInt, &f->d}},
      {"umgraph", {kBool, &f->umgraph}},     {"deepwalk", {kBool, &f->deepwalk}},
      {"node2vec", {kBool, &f->node2vec}},   {"ppr", {kBool, &f->ppr}},
      {"metapath", {kBool, &f->metapath}},   {"dprs", {kBool, &f->dprs}},
      {"p", {kDouble, &f->p}},               {"q", {kDouble, &f->q}},
      {"tp", {kDouble, &f->tp}},             {"schemalen", {kInt, &f->schemalen}},
      {"schema", {kString, &f->schema}},     {"printresult", {kBool, &f->printresult}},
      {"printworkload", {kBool, &f->printworkload}}, {"save_degree", {kBool, &f->save_degree}},
      {"autobatch", {kBool, &f->autobatch}}, {"batch", {kBool, &f->batch}},
      {"syn", {kBool, &f->syn}},             {"batchsize", {kUint, &f->batchsize}},
      {"headroom", {kInt, &f->headroom}},    {"walkmode", {kInt, &f->walkmode}},
      {"lognorm", {kBool, &f->lognorm}},     {"seed", {kLong, &f->seed}},
      {"pprstart", {kString, &f->pprstart}}, {"hub_threshold", {kInt, &f->hub_threshold}},
      {"wg_threads", {kInt, &f->wg_threads}}, {"savepaths", {kString, &f->savepaths}},
      {"park_threshold", {kInt, &f->park_threshold}},
  };
  for (int i = 1; i < argc; ++i) {
    std::string arg = argv[i];
    if (arg.size() < 2 || arg[0] != '-') { fprintf(stderr, "flowwalker: unexpected argument '%s'\n", arg.c_str()); return false; }
    arg = arg.substr(arg[1] == '-' ? 2 : 1);
    std::string value;
    bool has_value = false;
    const size_t eq = arg.find('=');
    if (eq != std::string::npos) { value = arg.substr(eq + 1); arg = arg.substr(0, eq); has_value = true; }
    auto it = specs.find(arg);
    bool negated = false;
    if (it == specs.end() && arg.compare(0, 2, "no") == 0) {
      it = specs.find(arg.substr(2));
      negated = it != specs.end() && it->second.kind == kBool;
      if (!negated) it = specs.end();
    }
    if (it == specs.end()) { fprintf(stderr, "flowwalker: unknown command line flag '%s'\n", arg.c_str()); return false; }
    const Spec& s = it->second;
    if (s.kind == kBool) {
      bool v = !negated;
      if (has_value) v = (value == "true" || value == "1" || value == "yes" || value == "t" || value == "y") != negated;
      *static_cast<bool*>(s.ptr) = v;
      continue;
    }
    if (!has_value) {
      if (i + 1 >= argc) { fprintf(stderr, "flowwalker: flag '--%s' is missing its argument\n", arg.c_str()); return false; }
      value = argv[++i];
    }
    char* endp = nullptr;
    switch (s.kind) {
      case kInt: *static_cast<int*>(s.ptr) = (int)strtol(value.c_str(), &endp, 10); break;
      case kUint: *static_cast<unsigned*>(s.ptr) = (unsigned)strtoul(value.c_str(), &endp, 10); break;
      case kLong: *static_cast<long long*>(s.ptr) = strtoll(value.c_str(), &endp, 10); break;
      case kDouble: *static_cast<double*>(s.ptr) = strtod(value.c_str(), &endp); break;
      default: *static_cast<std::string*>(s.ptr) = value; break;
    }
    if (s.kind != kString && (endp == value.c_str() || *endp != '\0')) {
      fprintf(stderr, "flowwalker: illegal value '%s' for flag '--%s'\n", value.c_str(), arg.c_str());
      return false;
    }
  }
  return true;
}

// src/main.cu:226-242
bool parse_schema(const std::string& text, std::vector<int>* out) {
  size_t pos = 0;
  while (pos <= text.size()) {
    const size_t comma = text.find(',', pos);
    const std::string tok = text.substr(pos, comma == std::string::npos ? std::string::npos : comma - pos);
    char* endp = nullptr;
    const long v = strtol(tok.c_str(), &endp, 10);
    if (tok.empty() || *endp != '\0') return false;
    out->push_back((int)v);
    if (comma == std::string::npos) break;
    pos = comma + 1;
  }
  return !out->empty();
}

double now_s() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

// src/main.cu:151-181
void print_res(int n, int max_depth, const int32_t* result) {
  unsigned long long sampled = 0;
  const int shown = std::min(n, 100);
  for (int i = 0; i < shown; i++) {
    printf("----------------------\nWalker %d:\n", i);
    int len = max_depth;
    for (int j = 0; j < max_depth; j++) {
      const int32_t v = result[(size_t)i * max_depth + j];
      if (v == -1) { len = j; break; }
      if (j > 0) sampled++;
      printf("%d\t", v);
    }
    printf("\nTotal length=%d\n", len);
  }
  printf("Total sampled: %llu\n", sampled);
}

// src/main.cu:183-224
void print_res_metapath(int n, int max_depth, const int32_t* result, const uint32_t* xadj, const int32_t* adjncy,
                        const int32_t* label) {
  unsigned long long sampled = 0;
  for (int i = 0; i < n; i++) {
    printf("----------------------\nWalker %llu:\n", (unsigned long long)i);
    int len = max_depth;
    int pre = -1;
    for (int j = 0; j < max_depth; j++) {
      const int32_t v = result[(size_t)i * max_depth + j];
      if (v == -1) { len = j; break; }
      if (pre != -1) {
        for (uint32_t k = xadj[pre]; k < xadj[pre + 1]; k++) {
          if (adjncy[k] == v) { printf("[%d]\t", label[k]); break; }
        }
      }
      if (j > 0) sampled++;
      pre = v;
      printf("%d\t", v);
    }
    printf("\nTotal length=%d\n", len);
  }
  printf("Total sampled: %llu\n", sampled);
}

}  // namespace

int main(int argc, char** argv) {
  printf("\n---------------------------------------------------------------------"
         "------------------------------------\n");
  Flags F;
  if (!parse_flags(argc, argv, &F)) return 2;
  if (F.umgraph) printf("umgraph: edge arrays stay in pinned host memory and are read over the bus\n");
  if (F.walkmode >= 0 && F.walkmode != 1 && F.walkmode != 6 && F.walkmode != 9 && F.walkmode != 10 &&
      (F.walkmode < 20 || F.walkmode > 22)) {
    fprintf(stderr, "flowwalker: --walkmode must be 9, 10, 1, 6 (the reference's ablation levels) or 20, 21, 22 (this "
                    "engine's); %d ignored\n", F.walkmode);
    F.walkmode = -1;
  }
  if (!(F.deepwalk || F.ppr || F.node2vec || F.metapath)) {  // src/walk.cu:565-568
    printf("Please choose a walk mode\n");
    return 0;
  }
  if (fw_device_count() < 1) {
    fprintf(stderr, "flowwalker: no HIP device visible; the walk engine has no CPU fallback\n");
    return 3;
  }

  // ---- graph (src/main.cu:304-325) ----
  const double t_load = now_s();
  int32_t V = 0;
  uint64_t E = 0;
  if (fw_csr_read_header(F.input.c_str(), &V, &E) != FW_OK) return fail("reading the graph header");
  printf("Vertex count:%d Expected edge count: %llu\n", V, (unsigned long long)E);
  std::vector<uint32_t> xadj((size_t)V + 1);
  std::vector<int32_t> adjncy((size_t)E);
  std::vector<float> weight(F.metapath ? 0 : (size_t)E);
  std::vector<int32_t> label(F.metapath ? (size_t)E : 0);
  if (fw_csr_load(F.input.c_str(), V, E, xadj.data(), adjncy.data(), F.metapath ? nullptr : weight.data(),
                  F.metapath ? label.data() : nullptr) != FW_OK)
    return fail("loading the graph");
  if (F.lognorm && !F.metapath) {
    // include/graph.cuh:79-91, :164-165: the weights of the file are replaced by log-normal(0, 3) draws (the
    // reference draws them with cuRAND, seed 1234; here a seeded host generator: same law, other numbers)
    std::mt19937_64 gen(1234ULL);
    std::lognormal_distribution<float> dist(0.0f, 3.0f);
    for (size_t i = 0; i < weight.size(); ++i) weight[i] = dist(gen);
  }
  if (F.node2vec) {
    // the adjacency test binary-searches neighbour lists (include/gpu_graph.cuh:97-118), but the reference's own
    // converter writes them in insertion order (data/EdgeListToCSR.cpp:182-191, its shipped wiki-Vote files
    // included): lists that do not ascend are sorted here, weights moving with their edges (same sampling law)
    int64_t changed = 0;
    if (fw_csr_sort_neighbours(V, xadj.data(), adjncy.data(), weight.data(), nullptr, &changed) != FW_OK)
      return fail("sorting neighbour lists");
    if (changed) printf("node2vec: %lld neighbour lists were not ascending and have been sorted\n", (long long)changed);
  }
  printf("Graph load (success): %d verts, %llu edges %g second(s)\n", V, (unsigned long long)E, now_s() - t_load);
  printf("Read Graph!\n");
  int32_t max_deg = 0, max_idx = 0;
  for (int32_t v = 0; v < V; ++v) {  // include/graph.cuh:209-220
    const int32_t deg = (int32_t)(xadj[v + 1] - xadj[v]);
    if (deg > max_deg) { max_deg = deg; max_idx = v; }
  }
  printf("Max degree: %d, idx: %d\n", max_deg, max_idx);
  fw_graph* g = nullptr;
  if (fw_graph_create_placed(V, E, xadj.data(), adjncy.data(), F.metapath ? nullptr : weight.data(),
                             F.metapath ? label.data() : nullptr, F.umgraph ? FW_GRAPH_HOST_PINNED : FW_GRAPH_DEVICE,
                             &g) != FW_OK)
    return fail("uploading the graph");

  fw_walk_params P;
  fw_walk_params_default_for(&P, F.deepwalk ? FW_APP_DEEPWALK : F.ppr ? FW_APP_PPR : F.node2vec ? FW_APP_NODE2VEC : FW_APP_METAPATH);
  std::vector<int> schema;
  if (F.metapath) {
    if (!parse_schema(F.schema, &schema) || schema.size() > FW_MAX_SCHEMA) {
      fprintf(stderr, "flowwalker: cannot parse --schema '%s' (1..%d comma-separated labels)\n", F.schema.c_str(), FW_MAX_SCHEMA);
      return 2;
    }
    F.schemalen = (int)schema.size();
    printf("schema len=%d\n", F.schemalen);
    for (int s : schema) printf("%d ", s);
    printf("\n");
    P.schema_len = F.schemalen;
    for (size_t i = 0; i < schema.size(); ++i) P.schema[i] = schema[i];
  }

  // ---- adjust_flags (src/main.cu:244-272) ----
  int sample_size = F.all ? V : F.n;
  if (sample_size <= 0) { fprintf(stderr, "flowwalker: --n must be positive\n"); return 2; }
  if (F.metapath) F.d = F.schemalen;
  if (F.all) { F.seq = true; F.batch = true; F.autobatch = true; }
  if (F.autobatch) {
    F.batch = true;
    size_t free_b = 0, total_b = 0;
    if (fw_device_mem_info(&free_b, &total_b) != FW_OK) return fail("querying device memory");
    const double gib = 1024.0 * 1024.0 * 1024.0;
    printf("Amount of total memory: %g GB, avail memory: %g GB, take up: %g GB, %g MB, %g KB\n", total_b / gib,
           free_b / gib, (total_b - free_b) / gib, (total_b - free_b) / (1024.0 * 1024.0), (total_b - free_b) / 1024.0);
    F.batchsize = fw_autobatch_size(free_b, F.headroom, F.d + 1, F.syn ? 1 : 0, (uint32_t)sample_size);
    if (F.batchsize == 0) { fprintf(stderr, "flowwalker: not enough free device memory for autobatch\n"); return 4; }
    printf("batch size=%u\n", F.batchsize);
  }
  const int depth = F.d + 1;

  // ---- start vertices (src/main.cu:273-296) ----
  int32_t* starts = nullptr;
  if (fw_host_alloc_pinned((size_t)sample_size * sizeof(int32_t), reinterpret_cast<void**>(&starts)) != FW_OK)
    return fail("allocating start points");
  if (F.ppr && F.pprstart != "seq") {
    for (int i = 0; i < sample_size; ++i) starts[i] = max_idx;  // src/main.cu:277-281
  } else {
    unsigned int local_seed = (unsigned int)F.seed;
    for (int i = 0; i < sample_size; ++i) starts[i] = F.seq ? (i % V) : (int32_t)(rand_r(&local_seed) % V);
  }

  P.app = F.deepwalk ? FW_APP_DEEPWALK : F.ppr ? FW_APP_PPR : F.node2vec ? FW_APP_NODE2VEC : FW_APP_METAPATH;
  P.sampler = F.dprs ? FW_SAMPLER_DPRS : FW_SAMPLER_ZPRS;
  P.max_depth = depth;
  P.tp = (float)F.tp;
  P.p = (float)F.p;
  P.q = (float)F.q;
  P.seed = (uint64_t)F.seed;
  if (F.hub_threshold >= 0) P.hub_threshold = F.hub_threshold;
  if (F.wg_threads > 0) P.wg_threads = F.wg_threads;
  P.park_threshold = F.park_threshold;
  if (F.walkmode >= 20) {  // this engine's levels, lowest first
    if (F.walkmode == 20) P.hub_threshold = 0x7FFFFFFF;
    if (F.walkmode != 22) P.park_threshold = -1;
    printf("ablation level %d: %s\n", F.walkmode,
           F.walkmode == 22 ? "workgroup sampler and parking (the full engine)"
                            : F.walkmode == 21 ? "workgroup sampler, no parking" : "wave sampler only, no parking");
  } else if (F.walkmode >= 0) {  // the reference's levels (README.md:152-163), its algorithms on 64-lane waves
    const bool dprs = F.walkmode == 9 || F.walkmode == 10;
    const bool is_static = F.walkmode != 6;
    const int rng = F.walkmode == 9 ? FW_SAMPLER_REF_RNG_GLOBAL : (is_static ? FW_SAMPLER_REF_RNG_LDS : 0);
    P.sampler = (dprs ? FW_SAMPLER_REF_DPRS : FW_SAMPLER_REF_ZPRS) | (is_static ? FW_SAMPLER_REF_STATIC : 0) | rng;
    if (F.hub_threshold < 0) P.hub_threshold = 1024;  // THRESHOLD, include/walker.cuh:29
    printf("ablation level %d: the reference's %s samplers on 64-lane waves, %s, %s\n", F.walkmode, dprs ? "DPRS" : "ZPRS",
           is_static ? "static query assignment" : "global query dispenser",
           rng == FW_SAMPLER_REF_RNG_GLOBAL ? "thread-owned generators in device memory"
           : rng == FW_SAMPLER_REF_RNG_LDS  ? "thread-owned generators in LDS"
                                            : "draws addressed by walker, step and element");
  }

  // ---- walk (src/main.cu:346-357) ----
  int32_t* paths = nullptr;
  const size_t path_bytes = (size_t)sample_size * (size_t)depth * sizeof(int32_t);
  if (fw_host_alloc_pinned(path_bytes, reinterpret_cast<void**>(&paths)) != FW_OK) return fail("allocating the path matrix");
  fw_walk_stats st;
  memset(&st, 0, sizeof(st));
  printf("========start timing\n");
  if (F.batch) {
    if (fw_walk_batch(g, &P, starts, sample_size, F.batchsize, F.syn ? 1 : 0, paths, &st) != FW_OK) return fail("walk_batch");
    if (F.syn) printf("compute time=%.6f ms, transfer time=%.6f ms\n", st.kernel_ms, st.total_ms - st.kernel_ms);
  } else {
    void* d_starts = nullptr;
    void* d_paths = nullptr;
    if (fw_dev_alloc((size_t)sample_size * 4, &d_starts) != FW_OK || fw_dev_alloc(path_bytes, &d_paths) != FW_OK)
      return fail("allocating device buffers");
    if (fw_dev_upload(d_starts, starts, (size_t)sample_size * 4) != FW_OK) return fail("uploading start points");
    if (fw_walk_device(g, &P, static_cast<int32_t*>(d_starts), sample_size, static_cast<int32_t*>(d_paths), nullptr, &st) != FW_OK)
      return fail("walk_test");
    if (fw_dev_download(paths, d_paths, path_bytes) != FW_OK) return fail("downloading paths");
    fw_dev_free(d_starts);
    fw_dev_free(d_paths);
  }
  const double sample_ms = F.batch ? st.total_ms : st.kernel_ms;  // src/walk.cu:368, :465
  printf("flowwalker HOST: grid:%d,block:%d,sampling time:%.6f ms\n", st.grid, P.wg_threads, sample_ms);

  if (F.printresult) {
    if (F.metapath) print_res_metapath(sample_size, depth, paths, xadj.data(), adjncy.data(), label.data());
    else print_res(sample_size, depth, paths);
  }
  if (F.printworkload) {  // src/main.cu:82-113; the reference divides by milliseconds and prints "per s"
    printf("Total sampled vertex: %llu\n", (unsigned long long)st.steps);
    printf("Total sampled edge: %llu,throughput: %f edges per s\n", (unsigned long long)st.sampled_edges,
           (double)st.sampled_edges / (sample_ms * 1e-3));
    printf("walk steps per s: %f (kernel only: %f)\n", (double)st.steps / (sample_ms * 1e-3),
           (double)st.steps / (st.kernel_ms * 1e-3));
  }
  if (F.save_degree) {  // src/main.cu:115-149, :373: how many steps left a vertex of each degree, "degree,count" per line
    std::map<uint32_t, uint64_t> hist;
    for (int i = 0; i < sample_size; ++i) {
      const int32_t* row = paths + (size_t)i * (size_t)depth;
      for (int j = 1; j < depth && row[j] != -1; ++j) ++hist[xadj[(size_t)row[j - 1] + 1] - xadj[(size_t)row[j - 1]]];
    }
    FILE* f = fopen(F.b_file.c_str(), "w");
    if (!f) { fprintf(stderr, "flowwalker: cannot write %s\n", F.b_file.c_str()); return 4; }
    for (const auto& kv : hist) fprintf(f, "%u,%llu\n", kv.first, (unsigned long long)kv.second);
    fclose(f);
  }
  if (!F.savepaths.empty()) {
    FILE* f = fopen(F.savepaths.c_str(), "wb");
    if (!f || fwrite(paths, 1, path_bytes, f) != path_bytes) { fprintf(stderr, "flowwalker: cannot write %s\n", F.savepaths.c_str()); return 4; }
    fclose(f);
  }
  fw_host_free_pinned(paths);
  fw_host_free_pinned(starts);
  fw_graph_destroy(g);
  return 0;
}
