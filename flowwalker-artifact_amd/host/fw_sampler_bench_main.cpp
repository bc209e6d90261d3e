// fw_sampler_bench -- throughput of ONE sampling step at fixed list lengths, the counterpart of the reference's
// TestSampler (src/sampler_test.cu: every worker samples one index from a slice of a large array of random weights,
// slices visited in shuffled order).
//
// Two command lines.
//
// 1. The reference's (src/sampler_test.cu:33-35, README.md:125-150), gflags spelling:
//      fw_sampler_bench --groupsize=S --gran=32|512 --type=N
//    --type: 1 / 2 = ZPRS by a wave / by a workgroup (warp_myrand / block_myrand, src/sampler_test.cu:798-813),
//    3 / 4 = DPRS (warp_oneloop / block_oneloop, :814-819), 5 / 6 = inverse transform sampling (:820-825), 7 / 8 = the
//    alias method (:826-833), 13 / 14 = rejection sampling (:843-862); 0 / 100 = this engine's own sampler by a wave / a
//    workgroup (the reference's 0 is its one-thread sampler, which has no counterpart here).  Odd types sample with one
//    wave, even ones with a workgroup of 512.
//    The reference's source and its README name the two size flags the other way round: sampler_test.cu:33-34 calls
//    --groupsize "the number of threads in a sampler" and --gran "the number of elements processed by each sampler",
//    README.md:128-149 runs `--groupsize=$SAMPLING_SIZE --gran=32` (wave) / `--gran=512` (workgroup).  The lanes of a
//    sampler follow from --type here (64-lane waves stand in for 32-lane warps), so whichever of the two values is
//    that type's lane count (32 or 64 for the wave types, 512 for the workgroup types) names the lanes and the other one
//    is the list length; when both are lane counts the source's reading holds (--gran is the list length).  Both
//    spellings of the README's and of the source's commands therefore measure what their authors meant.
//    As in the reference, the weight array has 512 Mi elements (--elements overrides), every slice is sampled once,
//    in shuffled order, and the output ends with "Elapsed time: %.3f ms" (src/sampler_test.cu:915).
//
// 2. This tool's own sweep:
//      fw_sampler_bench [--elements 268435456] [--lengths 16,64,256,1024,4096,16384,65536] [--samples 4194304]
//                       [--granularity wave|workgroup|both] [--type native,zprs,dprs,its,rjs,als] [--wg_threads 512]
//                       [--reps 3] [--seed 1]
//    One line per (list length, type, granularity): samples/s and GB/s of weights (4 bytes per element and sample; the
//    two-pass ZPRS reads them twice, which is not counted).
//
// In both, the slices are the neighbour lists of a regular graph (vertex v owns weights[v*len, (v+1)*len)), a sample of
// native / zprs / dprs is a one-step walk (max_depth 2) through the C ABI -- the engine's kernels are measured as they
// are -- and its / rjs / als run on the same slices of the weight array (fw_sampler_baseline_run).  Flags may be written
// `--flag value` or `--flag=value`.

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
  fprintf(stderr, "fw_sampler_bench: %s: %s\n", what, fw_last_error());
  return 1;
}

struct Type {
  const char* name;
  int sampler;  // fw_sampler, or -1 - fw_baseline_sampler
};

static bool type_by_name(const std::string& t, Type* out) {
  if (t == "native") *out = {"native", FW_SAMPLER_ZPRS};
  else if (t == "zprs") *out = {"zprs", FW_SAMPLER_REF_ZPRS};
  else if (t == "dprs") *out = {"dprs", FW_SAMPLER_REF_DPRS};
  else if (t == "its") *out = {"its", -1 - FW_BASELINE_ITS};
  else if (t == "rjs") *out = {"rjs", -1 - FW_BASELINE_RJS};
  else if (t == "als") *out = {"als", -1 - FW_BASELINE_ALS};
  else return false;
  return true;
}

// TestSampler's numeric types (src/sampler_test.cu:789-895): the algorithm and whether a workgroup samples.
static bool type_by_number(int n, Type* out, int* workgroup) {
  switch (n) {
    case 0: *out = {"native", FW_SAMPLER_ZPRS}; *workgroup = 0; return true;
    case 100: *out = {"native", FW_SAMPLER_ZPRS}; *workgroup = 1; return true;
    case 1: case 2: *out = {"zprs", FW_SAMPLER_REF_ZPRS}; break;
    case 3: case 4: *out = {"dprs", FW_SAMPLER_REF_DPRS}; break;
    case 5: case 6: *out = {"its", -1 - FW_BASELINE_ITS}; break;
    case 7: case 8: *out = {"als", -1 - FW_BASELINE_ALS}; break;
    case 13: case 14: *out = {"rjs", -1 - FW_BASELINE_RJS}; break;
    default: return false;
  }
  *workgroup = (n & 1) ? 0 : 1;
  return true;
}

// The lists of one length, ready to be sampled: a regular graph over the weight array and a task list on the device.
struct Lists {
  fw_graph* g = nullptr;
  void* d_starts = nullptr;
  void* d_paths = nullptr;
  long long samples = 0;
  void release() {
    fw_dev_free(d_starts);
    fw_dev_free(d_paths);
    fw_graph_destroy(g);
    g = nullptr;
    d_starts = d_paths = nullptr;
  }
};

// every_list: the task list is a shuffle of all lists (the reference's), else `samples` lists drawn at random.
static int make_lists(const std::vector<float>& w, std::vector<int32_t>& adj, unsigned long long elements, long long len,
                      long long samples, bool every_list, std::mt19937_64& rng, Lists* out) {
  const long long V = (long long)(elements / (unsigned long long)len);
  std::vector<uint32_t> xadj((size_t)V + 1);
  for (long long v = 0; v <= V; ++v) xadj[(size_t)v] = (uint32_t)(v * len);
  for (unsigned long long i = 0; i < (unsigned long long)V * (unsigned long long)len; ++i) adj[i] = (int32_t)(i % (unsigned long long)V);
  if (fw_graph_create((int32_t)V, (uint64_t)V * (uint64_t)len, xadj.data(), adj.data(), w.data(), nullptr, &out->g) != FW_OK)
    return fail("uploading");
  std::vector<int32_t> starts;
  if (every_list) {  // src/sampler_test.cu:746-755
    starts.resize((size_t)V);
    for (long long i = 0; i < V; ++i) starts[(size_t)i] = (int32_t)i;
    std::shuffle(starts.begin(), starts.end(), rng);
  } else {
    starts.resize((size_t)samples);
    for (long long i = 0; i < samples; ++i) starts[(size_t)i] = (int32_t)(rng() % (uint64_t)V);
  }
  out->samples = (long long)starts.size();
  if (fw_dev_alloc(starts.size() * 4, &out->d_starts) != FW_OK || fw_dev_alloc(starts.size() * 8, &out->d_paths) != FW_OK)
    return fail("allocating");
  if (fw_dev_upload(out->d_starts, starts.data(), starts.size() * 4) != FW_OK) return fail("uploading queries");
  return 0;
}

// One measurement: `reps` timed launches after a warm-up, the best one counts.  Returns its milliseconds in *best_ms,
// the samples taken in *taken and the weights they covered in *edges.
static int measure(const Lists& L, const Type& type, int workgroup, const void* d_w, unsigned long long elements,
                   long long len, int wg_threads, int reps, unsigned long long seed, double* best_ms,
                   unsigned long long* taken, unsigned long long* edges) {
  double best = 0.0;
  if (type.sampler < 0) {
    double ms = 0.0;
    for (int r = 0; r <= reps; ++r) {
      if (fw_sampler_baseline_run(-1 - type.sampler, workgroup, (const float*)d_w, elements, (uint32_t)len,
                                  (const uint32_t*)L.d_starts, (uint32_t)L.samples, wg_threads, seed, (int32_t*)L.d_paths,
                                  &ms) != FW_OK)
        return fail("sampling");
      if (r > 0 && (best == 0.0 || ms < best)) best = ms;
    }
    *taken = (unsigned long long)L.samples;
    *edges = (unsigned long long)L.samples * (unsigned long long)len;
  } else {
    fw_walk_params p;
    fw_walk_params_default(&p);
    p.app = FW_APP_DEEPWALK;
    p.sampler = type.sampler;
    p.max_depth = 2;                 // the start vertex and one sampled neighbour
    p.wg_threads = wg_threads;
    p.hub_threshold = workgroup ? 0 : 0x7FFFFFFF;  // every list by the workgroup / by one wave
    p.park_threshold = -1;           // the plain sampler, no sharing of scans between walkers
    p.seed = seed;
    fw_walk_stats st;
    memset(&st, 0, sizeof(st));
    for (int r = 0; r <= reps; ++r) {  // first run warms up
      if (fw_walk_device(L.g, &p, (const int32_t*)L.d_starts, (int32_t)L.samples, (int32_t*)L.d_paths, nullptr, &st) != FW_OK)
        return fail("sampling");
      if (r > 0 && (best == 0.0 || st.kernel_ms < best)) best = st.kernel_ms;
    }
    *taken = st.steps;
    *edges = st.sampled_edges;
  }
  *best_ms = best;
  return 0;
}

int main(int argc, char** argv) {
  unsigned long long elements = 0, seed = 1;
  long long samples = 1ll << 22;
  std::string lengths = "16,64,256,1024,4096,16384,65536", granularity = "both", types = "native,zprs,dprs";
  int wg_threads = 512, reps = 3;
  long long groupsize = -1, gran = -1;  // the reference's two size flags
  for (int i = 1; i < argc; ++i) {
    std::string k = argv[i];
    std::string inline_val;
    bool has_inline = false;
    const size_t eq = k.find('=');
    if (k.rfind("--", 0) == 0 && eq != std::string::npos) {
      inline_val = k.substr(eq + 1);
      k = k.substr(0, eq);
      has_inline = true;
    }
    auto val = [&]() -> std::string {
      if (has_inline) return inline_val;
      if (i + 1 >= argc) { fprintf(stderr, "fw_sampler_bench: %s needs a value\n", k.c_str()); exit(2); }
      return argv[++i];
    };
    if (k == "--elements") elements = strtoull(val().c_str(), nullptr, 10);
    else if (k == "--lengths") lengths = val();
    else if (k == "--gran") gran = atoll(val().c_str());
    else if (k == "--groupsize") groupsize = atoll(val().c_str());
    else if (k == "--samples") samples = atoll(val().c_str());
    else if (k == "--granularity") granularity = val();
    else if (k == "--type") types = val();
    else if (k == "--wg_threads") wg_threads = atoi(val().c_str());
    else if (k == "--reps") reps = atoi(val().c_str());
    else if (k == "--seed") seed = strtoull(val().c_str(), nullptr, 10);
    else { fprintf(stderr, "fw_sampler_bench: unknown flag %s\n", k.c_str()); return 2; }
  }
  const bool numeric_type = !types.empty() && types.find_first_not_of("0123456789") == std::string::npos;
  const bool reference_cli = numeric_type || groupsize >= 0 || gran >= 0;
  if (reference_cli && !numeric_type) {
    fprintf(stderr, "fw_sampler_bench: --groupsize / --gran belong to the reference's command line and go with a numeric "
                    "--type (0..8, 13, 14, 100); this tool's own sweep takes --lengths\n");
    return 2;
  }
  if (granularity != "wave" && granularity != "workgroup" && granularity != "both") {
    fprintf(stderr, "fw_sampler_bench: --granularity must be wave, workgroup or both\n");
    return 2;
  }
  if (elements == 0) elements = reference_cli ? 512ull * 1024ull * 1024ull : 1ull << 28;  // src/sampler_test.cu:923
  if (elements < 1024 || elements > 0xFFFFFFF0ull || samples < 1 || samples > 0x7FFFFFFF || reps < 1) {
    fprintf(stderr, "fw_sampler_bench: sizes out of range\n");
    return 2;
  }

  // the reference's command line: one type, one list length
  Type ref_type = {"", 0};
  int ref_workgroup = 0;
  long long ref_len = 0;
  if (reference_cli) {
    const int tn = atoi(types.c_str());
    if (!type_by_number(tn, &ref_type, &ref_workgroup)) {
      fprintf(stderr, "fw_sampler_bench: --type=%d is not built (1/2 ZPRS, 3/4 DPRS, 5/6 ITS, 7/8 ALS, 13/14 RJS by a wave / a "
                      "workgroup; 0/100 this engine's sampler)\n", tn);
      return 2;
    }
    if (groupsize < 0) groupsize = 32;  // the reference's defaults, src/sampler_test.cu:33-34
    if (gran < 0) gran = 32;
    auto is_lanes = [&](long long v) { return ref_workgroup ? v == 512 : (v == 32 || v == 64); };
    // --gran is the list length (the source's reading) unless only --gran can be the lane count (the README's)
    ref_len = (is_lanes(gran) && !is_lanes(groupsize)) ? groupsize : gran;
    if (ref_len < 1 || (unsigned long long)ref_len > elements) {
      fprintf(stderr, "fw_sampler_bench: list length %lld out of range\n", ref_len);
      return 2;
    }
    if (ref_workgroup) wg_threads = 512;  // TEST_BLOCK_SIZE, src/sampler_test.cu:30
  }
  if (fw_device_count() < 1) { fprintf(stderr, "fw_sampler_bench: no HIP device\n"); return 1; }

  // one array of random weights for all list lengths (the lists are cut out of it); neighbour ids are refilled per
  // list length so that they name existing vertices
  std::mt19937_64 rng(seed);
  std::vector<float> w(elements);
  std::vector<int32_t> adj(elements);
  if (reference_cli) {  // uniform in (0, 1], as curandGenerateUniform gives them (src/sampler_test.cu:945)
    for (unsigned long long i = 0; i < elements; ++i) w[i] = (float)(((rng() >> 40) + 1) * (1.0 / 16777216.0));
  } else {
    for (unsigned long long i = 0; i < elements; ++i) w[i] = 1.0f + 99.0f * (float)((rng() >> 40) * (1.0 / 16777216.0));
  }

  if (reference_cli) {
    const long long V = (long long)(elements / (unsigned long long)ref_len);
    if (V > 0x7FFFFFF0ll) { fprintf(stderr, "fw_sampler_bench: too many lists\n"); return 2; }
    printf("\n\n-----------------------------------------------------------------"
           "----------------------------------------\n");
    printf("Test config: {Num of Elements: %llu, Block Size: %d, Number of Threads in a Sampler: %d, Sampler Type: %s "
           "(%s), Number of Elements Processed by a Sampler: %lld, Number of tasks: %lld}\n",
           elements, 512, ref_workgroup ? 512 : 64, types.c_str(), ref_type.name, ref_len, V);
    void* d_w = nullptr;
    if (ref_type.sampler < 0 &&
        (fw_dev_alloc((size_t)elements * 4, &d_w) != FW_OK || fw_dev_upload(d_w, w.data(), (size_t)elements * 4) != FW_OK))
      return fail("uploading the weight array");
    Lists L;
    if (make_lists(w, adj, elements, ref_len, 0, true, rng, &L) != 0) return 1;
    double ms = 0.0;
    unsigned long long taken = 0, edges = 0;
    if (measure(L, ref_type, ref_workgroup, d_w, elements, ref_len, wg_threads, 1, seed, &ms, &taken, &edges) != 0) return 1;
    L.release();
    if (d_w) fw_dev_free(d_w);
    printf("Samples: %llu, %.4g samples/s, %.1f GB/s of weights\n", taken, (double)taken / (ms * 1e-3),
           4.0 * (double)edges / (ms * 1e-3) / 1e9);
    printf("Elapsed time: %.3f ms\n", ms);  // src/sampler_test.cu:915
    return 0;
  }

  std::vector<Type> run_types;
  for (size_t tp = 0; tp < types.size();) {
    size_t c = types.find(',', tp);
    if (c == std::string::npos) c = types.size();
    const std::string t = types.substr(tp, c - tp);
    tp = c + 1;
    Type ty;
    if (!type_by_name(t, &ty)) {
      fprintf(stderr, "fw_sampler_bench: --type takes native, zprs, dprs, its, rjs, als (got %s)\n", t.c_str());
      return 2;
    }
    run_types.push_back(ty);
  }
  void* d_w = nullptr;  // the baselines read the weight array itself, not a graph
  for (const Type& type : run_types)
    if (type.sampler < 0 && !d_w) {
      if (fw_dev_alloc((size_t)elements * 4, &d_w) != FW_OK || fw_dev_upload(d_w, w.data(), (size_t)elements * 4) != FW_OK)
        return fail("uploading the weight array");
    }
  printf("%-10s %-8s %-10s %12s %14s %12s %10s\n", "length", "type", "sampler", "samples", "samples/s", "GB/s", "ms");
  size_t pos = 0;
  while (pos < lengths.size()) {
    size_t comma = lengths.find(',', pos);
    if (comma == std::string::npos) comma = lengths.size();
    const long long len = atoll(lengths.substr(pos, comma - pos).c_str());
    pos = comma + 1;
    if (len < 1 || (unsigned long long)len > elements) continue;
    if ((long long)(elements / (unsigned long long)len) > 0x7FFFFFF0ll) {
      fprintf(stderr, "fw_sampler_bench: length %lld gives too many lists, skipped\n", len);
      continue;
    }
    Lists L;
    if (make_lists(w, adj, elements, len, samples, false, rng, &L) != 0) return 1;
    for (const Type& type : run_types) {
      for (int mode = 0; mode < 2; ++mode) {
        const char* name = mode == 0 ? "wave" : "workgroup";
        if (granularity != "both" && granularity != name) continue;
        double ms = 0.0;
        unsigned long long taken = 0, edges = 0;
        if (measure(L, type, mode, d_w, elements, len, wg_threads, reps, seed, &ms, &taken, &edges) != 0) return 1;
        printf("%-10lld %-8s %-10s %12llu %14.4g %12.1f %10.3f\n", len, type.name, name, taken,
               (double)taken / (ms * 1e-3), 4.0 * (double)edges / (ms * 1e-3) / 1e9, ms);
        fflush(stdout);
      }
    }
    L.release();
  }
  if (d_w) fw_dev_free(d_w);
  return 0;
}
