// fw_sampler_bench -- throughput of ONE sampling step at fixed list lengths, the counterpart of the reference's
// TestSampler (src/sampler_test.cu: every worker samples one index from a `gran`-element slice of a large array of
// random weights, slices visited in shuffled order; flags --gran / --groupsize, :33-35).
//
// Here the slices are the neighbour lists of a regular graph (vertex v owns weights[v*gran, (v+1)*gran)), a sample is
// a one-step walk (max_depth 2) started on a shuffled vertex list, and the granularity is chosen the way the walk
// engine chooses it: --granularity wave (every list by one wave; lists of at most 64 elements four or two per wave)
// or workgroup (every list by a whole workgroup of --wg_threads).  The engine's kernels are measured as they
// are, through the C ABI; nothing is re-implemented here.
//
// --type picks the algorithm, as TestSampler's --type does (src/sampler_test.cu:789-895): `native` = this engine's
// one-pass group reservoir; `zprs` / `dprs` = the reference's own samplers restated for 64-lane waves
// (include/sampler.cuh:46-127 and :129-200, FW_SAMPLER_REF_ZPRS / _DPRS: TestSampler types 1 / 2 and 3 / 4), run
// on the same lists so that the columns can be compared; `its` / `rjs` / `als` = inverse transform sampling,
// rejection sampling and the alias method on the same slices of the weight array (TestSampler types 5 / 6, its RJS
// kernels and types 7 / 8; fw_sampler_baseline_run).
//
//   fw_sampler_bench [--elements 268435456] [--gran 16,64,256,1024,4096,16384,65536] [--samples 4194304]
//                    [--granularity wave|workgroup|both] [--type native,zprs,dprs,its,rjs,als] [--wg_threads 512] [--reps 3]
//                    [--seed 1]
// Output: one line per (gran, type, granularity): samples/s and GB/s of weights (4 bytes per element and sample;
// the two-pass ZPRS reads them twice, which is not counted).

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

int main(int argc, char** argv) {
  unsigned long long elements = 1ull << 28, seed = 1;
  long long samples = 1ll << 22;
  std::string grans = "16,64,256,1024,4096,16384,65536", granularity = "both", types = "native,zprs,dprs";
  int wg_threads = 512, reps = 3;
  for (int i = 1; i < argc; ++i) {
    const std::string k = argv[i];
    auto val = [&]() -> const char* {
      if (i + 1 >= argc) { fprintf(stderr, "fw_sampler_bench: %s needs a value\n", k.c_str()); exit(2); }
      return argv[++i];
    };
    if (k == "--elements") elements = strtoull(val(), nullptr, 10);
    else if (k == "--gran") grans = val();
    else if (k == "--samples") samples = atoll(val());
    else if (k == "--granularity") granularity = val();
    else if (k == "--type") types = val();
    else if (k == "--wg_threads") wg_threads = atoi(val());
    else if (k == "--reps") reps = atoi(val());
    else if (k == "--seed") seed = strtoull(val(), nullptr, 10);
    else { fprintf(stderr, "fw_sampler_bench: unknown flag %s\n", k.c_str()); return 2; }
  }
  if (granularity != "wave" && granularity != "workgroup" && granularity != "both") {
    fprintf(stderr, "fw_sampler_bench: --granularity must be wave, workgroup or both\n");
    return 2;
  }
  if (elements < 1024 || elements > 0xFFFFFFF0ull || samples < 1 || samples > 0x7FFFFFFF || reps < 1) {
    fprintf(stderr, "fw_sampler_bench: sizes out of range\n");
    return 2;
  }
  if (fw_device_count() < 1) { fprintf(stderr, "fw_sampler_bench: no HIP device\n"); return 1; }

  // one array of random weights for all list lengths (the lists are cut out of it); neighbour ids are refilled per
  // list length so that they name existing vertices
  std::mt19937_64 rng(seed);
  std::vector<float> w(elements);
  std::vector<int32_t> adj(elements);
  for (unsigned long long i = 0; i < elements; ++i) {
    w[i] = 1.0f + 99.0f * (float)((rng() >> 40) * (1.0 / 16777216.0));
    adj[i] = 0;
  }

  struct Type { const char* name; int sampler; };
  std::vector<Type> run_types;
  for (size_t tp = 0; tp < types.size();) {
    size_t c = types.find(',', tp);
    if (c == std::string::npos) c = types.size();
    const std::string t = types.substr(tp, c - tp);
    tp = c + 1;
    if (t == "native") run_types.push_back({"native", FW_SAMPLER_ZPRS});
    else if (t == "zprs") run_types.push_back({"zprs", FW_SAMPLER_REF_ZPRS});
    else if (t == "dprs") run_types.push_back({"dprs", FW_SAMPLER_REF_DPRS});
    else if (t == "its") run_types.push_back({"its", -1 - FW_BASELINE_ITS});
    else if (t == "rjs") run_types.push_back({"rjs", -1 - FW_BASELINE_RJS});
    else if (t == "als") run_types.push_back({"als", -1 - FW_BASELINE_ALS});
    else { fprintf(stderr, "fw_sampler_bench: --type takes native, zprs, dprs, its, rjs, als (got %s)\n", t.c_str()); return 2; }
  }
  void* d_w = nullptr;  // the baselines read the weight array itself, not a graph
  for (const Type& type : run_types)
    if (type.sampler < 0 && !d_w) {
      if (fw_dev_alloc((size_t)elements * 4, &d_w) != FW_OK || fw_dev_upload(d_w, w.data(), (size_t)elements * 4) != FW_OK)
        return fail("uploading the weight array");
    }
  printf("%-10s %-8s %-10s %12s %14s %12s %10s\n", "gran", "type", "sampler", "samples", "samples/s", "GB/s", "ms");
  size_t pos = 0;
  while (pos < grans.size()) {
    size_t comma = grans.find(',', pos);
    if (comma == std::string::npos) comma = grans.size();
    const long long gran = atoll(grans.substr(pos, comma - pos).c_str());
    pos = comma + 1;
    if (gran < 1 || (unsigned long long)gran > elements) continue;
    const long long V = (long long)(elements / (unsigned long long)gran);
    if (V > 0x7FFFFFF0ll) { fprintf(stderr, "fw_sampler_bench: gran %lld gives too many lists, skipped\n", gran); continue; }
    std::vector<uint32_t> xadj((size_t)V + 1);
    for (long long v = 0; v <= V; ++v) xadj[(size_t)v] = (uint32_t)(v * gran);
    for (unsigned long long i = 0; i < (unsigned long long)V * (unsigned long long)gran; ++i) adj[i] = (int32_t)(i % (unsigned long long)V);
    fw_graph* g = nullptr;
    if (fw_graph_create((int32_t)V, (uint64_t)V * (uint64_t)gran, xadj.data(), adj.data(), w.data(), nullptr, &g) != FW_OK)
      return fail("uploading");
    // shuffled task list (src/sampler_test.cu visits its slices through a shuffled list too)
    std::vector<int32_t> starts((size_t)samples);
    for (long long i = 0; i < samples; ++i) starts[(size_t)i] = (int32_t)(rng() % (uint64_t)V);
    void* d_starts = nullptr;
    void* d_paths = nullptr;
    if (fw_dev_alloc((size_t)samples * 4, &d_starts) != FW_OK || fw_dev_alloc((size_t)samples * 8, &d_paths) != FW_OK)
      return fail("allocating");
    if (fw_dev_upload(d_starts, starts.data(), (size_t)samples * 4) != FW_OK) return fail("uploading queries");

    for (const Type& type : run_types) {
      for (int mode = 0; mode < 2; ++mode) {
        const char* name = mode == 0 ? "wave" : "workgroup";
        if (granularity != "both" && granularity != name) continue;
        if (type.sampler < 0) {
          double best = 0.0, ms = 0.0;
          for (int r = 0; r <= reps; ++r) {
            if (fw_sampler_baseline_run(-1 - type.sampler, mode, (const float*)d_w, elements, (uint32_t)gran,
                                        (const uint32_t*)d_starts, (uint32_t)samples, wg_threads, seed, (int32_t*)d_paths,
                                        &ms) != FW_OK)
              return fail("sampling");
            if (r > 0 && (best == 0.0 || ms < best)) best = ms;
          }
          printf("%-10lld %-8s %-10s %12lld %14.4g %12.1f %10.3f\n", gran, type.name, name, samples,
                 (double)samples / (best * 1e-3), 4.0 * (double)samples * (double)gran / (best * 1e-3) / 1e9, best);
          fflush(stdout);
          continue;
        }
        fw_walk_params p;
        fw_walk_params_default(&p);
        p.app = FW_APP_DEEPWALK;
        p.sampler = type.sampler;
        p.max_depth = 2;                 // the start vertex and one sampled neighbour
        p.wg_threads = wg_threads;
        p.hub_threshold = mode == 0 ? 0x7FFFFFFF : 0;  // every list by one wave / by the workgroup
        p.park_threshold = -1;           // the plain sampler, no sharing of scans between walkers
        p.seed = seed;
        double best = 0.0;
        fw_walk_stats st;
        for (int r = 0; r <= reps; ++r) {  // first run warms up
          if (fw_walk_device(g, &p, (const int32_t*)d_starts, (int32_t)samples, (int32_t*)d_paths, nullptr, &st) != FW_OK)
            return fail("sampling");
          if (r > 0 && (best == 0.0 || st.kernel_ms < best)) best = st.kernel_ms;
        }
        printf("%-10lld %-8s %-10s %12llu %14.4g %12.1f %10.3f\n", gran, type.name, name, (unsigned long long)st.steps,
               (double)st.steps / (best * 1e-3), 4.0 * (double)st.sampled_edges / (best * 1e-3) / 1e9, best);
        fflush(stdout);
      }
    }
    fw_dev_free(d_starts);
    fw_dev_free(d_paths);
    fw_graph_destroy(g);
  }
  if (d_w) fw_dev_free(d_w);
  return 0;
}
