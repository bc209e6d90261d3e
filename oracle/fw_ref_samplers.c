/*
 * fw_ref_samplers.c -- the reference's own samplers, restated on the CPU.  TEST INFRASTRUCTURE ONLY.
 *
 * Part of the checker (libfw_oracle.so): only tests/ may build, load or call it.  The shipped library never links
 * it.
 *
 * The walk engine of this build samples with a different algorithm than the reference (one pass, a reservoir over
 * groups of 1024 biases, see fw_oracle.c), so what it has to share with the reference is the LAW of a sampling
 * step, P(i) = w_i / sum w, and the special cases (no positive bias: -1; zero biases never taken).  The functions
 * here restate the reference's samplers thread by thread so that tests can check that claim against the
 * reference's algorithm itself and not only against the formula:
 *
 *   fw_ref_sampler_thread   include/sampler.cuh:26-44    sequential weighted reservoir sampling
 *   fw_ref_sampler_zprs     include/sampler.cuh:46-85    (warp, W = 32) and :87-127 (block, W = 512):
 *                           two passes, lane-strided elements, exclusive prefix over lane totals, i64 key
 *                           i + size * lane, max-reduce (include/util.cuh:104-109), key % size
 *   fw_ref_sampler_dprs     include/sampler.cuh:129-155  (warp) and :157-200 (block): one pass in chunks of W,
 *                           inclusive scan inside the chunk + carry, running max of the accepted indices
 *
 * Random numbers.  In the reference every thread owns an XORWOW stream (include/myrand.cuh) and draws from it in
 * program order.  Here the uniform a thread draws for element i is u[i]: every element is visited by exactly
 * one thread exactly once in the drawing pass, so this is a relabelling of the threads' streams, and i.i.d.
 * uniforms stay i.i.d. under it.  Uniforms lie in (0, 1] as cuRAND's do (include/myrand.cuh:213-215).
 *
 * Float arithmetic follows the reference's expressions (f32 sums, `u < w / weight_sum` with a division).  The
 * exclusive prefix over the lane totals is the Hillis-Steele network of :62-68 for any power-of-two W (the block
 * sampler's cub::BlockScan has no documented association; tests that need equality use integer-valued biases, whose
 * sums are exact in any order).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

void fw_oracle_wave_scan(float x[64]);                                                          /* fw_oracle.c */
void fw_oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);    /* fw_oracle.c */

/* include/sampler.cuh:26-44 */
int32_t fw_ref_sampler_thread(const float* w, int32_t n, const float* u) {
  int32_t selected = -1;
  float weight_sum = 0.0f;
  for (int32_t i = 0; i < n; ++i) {
    const float x = w[i];
    weight_sum += x;
    if (x > 0.0f) {
      if (selected == -1) selected = 0; /* :37 */
      if (u[i] < x / weight_sum) selected = i;
    }
  }
  return selected;
}

/* inclusive Hillis-Steele scan over W lanes, as the shuffles of include/sampler.cuh:63-66 and :146-148 */
static void hillis_steele(float* v, int W) {
  float* t = (float*)malloc(sizeof(float) * (size_t)W);
  for (int mask = 1; mask < W; mask <<= 1) {
    for (int l = 0; l < W; ++l) t[l] = l >= mask ? v[l - mask] : 0.0f;
    for (int l = 0; l < W; ++l)
      if (l >= mask) v[l] += t[l];
  }
  free(t);
}

/* include/sampler.cuh:46-85 (W = 32) / :87-127 (W = 512).  W must be a power of two. */
int32_t fw_ref_sampler_zprs(const float* w, int32_t n, int32_t W, const float* u) {
  float* sum = (float*)calloc((size_t)W, sizeof(float));
  float* local = (float*)malloc(sizeof(float) * (size_t)W);
  for (int l = 0; l < W; ++l)
    for (int32_t i = l; i < n; i += W) sum[l] += w[i]; /* :56-59 */
  for (int l = 0; l < W; ++l) local[l] = sum[l];
  hillis_steele(sum, W);                              /* :62-66 */
  for (int l = 0; l < W; ++l) sum[l] -= local[l];     /* :68: exclusive prefix of the lane */
  long long best = -1;
  for (int l = 0; l < W; ++l) {
    long long selected = -1;
    float weight_sum = sum[l];
    for (int32_t i = l; i < n; i += W) { /* :70-80 */
      const float x = w[i];
      weight_sum += x;
      if (x > 0.0f) {
        if (selected == -1) selected = 0;
        if (u[i] < x / weight_sum) selected = (long long)i + (long long)n * l;
      }
    }
    if (selected > best) best = selected; /* warpReduceMax, :82 */
  }
  free(sum);
  free(local);
  return best == -1 ? -1 : (int32_t)(best % n); /* :84 */
}

/* include/sampler.cuh:129-155 (W = 32) / :157-200 (W = 512).  W must be a power of two. */
int32_t fw_ref_sampler_dprs(const float* w, int32_t n, int32_t W, const float* u) {
  float* v = (float*)malloc(sizeof(float) * (size_t)W);
  float* x = (float*)malloc(sizeof(float) * (size_t)W);
  float prev_ite_sum = 0.0f;
  int32_t selected = -1; /* every lane holds the maximum after each chunk (:151) */
  const int32_t bound = n + W - n % W; /* :138: one extra all-zero chunk when n % W == 0 */
  for (int32_t base = 0; base < bound; base += W) {
    for (int l = 0; l < W; ++l) {
      const int32_t i = base + l;
      x[l] = i < n ? w[i] : 0.0f;
      v[l] = x[l];
    }
    int32_t chunk_max = selected;
    for (int l = 0; l < W; ++l)
      if (x[l] > 0.0f && selected == -1 && chunk_max < 0) chunk_max = 0; /* :142 */
    hillis_steele(v, W);                                                 /* :143-148 */
    for (int l = 0; l < W; ++l) {
      const int32_t i = base + l;
      const float weight_sum = v[l] + prev_ite_sum; /* :149 */
      if (i < n && u[i] < x[l] / weight_sum && i > chunk_max) chunk_max = i; /* :150 */
    }
    prev_ite_sum = v[W - 1] + prev_ite_sum; /* :151: lane W-1 broadcasts its inclusive sum */
    selected = chunk_max;
  }
  free(v);
  free(x);
  return selected;
}

/*
 * m independent sampling steps over the same n biases: row r of `u` (n uniforms) drives step r.
 * kind 0 = thread, 1 = zprs, 2 = dprs, 3 = zprs on 64-lane waves, 4 = dprs on 64-lane waves.  out[r] = selected index or -1.
 */
int32_t fw_ref64_zprs(const float* w, int32_t n, int32_t W, const float* u);
int32_t fw_ref64_dprs(const float* w, int32_t n, int32_t W, const float* u);

int fw_ref_sample_many(int kind, const float* w, int32_t n, int32_t W, const float* u, int64_t m, int32_t* out) {
  if (kind < 0 || kind > 4 || n < 0 || W < 1 || (W & (W - 1)) != 0) return 1;
  if (kind >= 3 && W % 64 != 0) return 1;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < m; ++r) {
    const float* ur = u + r * (int64_t)n;
    out[r] = kind == 0 ? fw_ref_sampler_thread(w, n, ur)
             : kind == 1 ? fw_ref_sampler_zprs(w, n, W, ur)
             : kind == 2 ? fw_ref_sampler_dprs(w, n, W, ur)
             : kind == 3 ? fw_ref64_zprs(w, n, W, ur) : fw_ref64_dprs(w, n, W, ur);
  }
  return 0;
}

/* ---- the same two samplers for groups of 64-lane wavefronts (what FW_SAMPLER_REF_ZPRS / _DPRS run on the GPU) ----
 *
 * W = 64 (one wave) or a multiple of it (a workgroup of W / 64 waves).  Everything follows the functions above except
 * the inclusive scan over the W lanes, which is the one a 64-lane machine has: the wave scan tree of fw_oracle.c inside
 * each wave, the waves' totals added one after the other in front of it (starting from `carry`).  The reference never
 * ran with 64 lanes, so this is this build's definition of "the reference's sampler on wave64"; what pins it is what
 * pins the functions above (equality with the sequential reservoir over the sampler's element order, the law).
 */
static void scan64(float* v, int W, float carry) {
  float off = carry;
  for (int w = 0; w < W / 64; ++w) {
    fw_oracle_wave_scan(v + 64 * w);
    const float T = v[64 * w + 63];
    for (int l = 0; l < 64; ++l) v[64 * w + l] = off + v[64 * w + l];
    off = off + T;
  }
}

int32_t fw_ref64_zprs(const float* w, int32_t n, int32_t W, const float* u) {
  float* sum = (float*)calloc((size_t)W, sizeof(float));
  float* local = (float*)malloc(sizeof(float) * (size_t)W);
  for (int l = 0; l < W; ++l)
    for (int64_t i = l; i < n; i += W) sum[l] += w[i];
  memcpy(local, sum, sizeof(float) * (size_t)W);
  scan64(sum, W, 0.0f);
  for (int l = 0; l < W; ++l) sum[l] = sum[l] - local[l];
  long long best = -1;
  for (int l = 0; l < W; ++l) {
    long long selected = -1;
    float weight_sum = sum[l];
    for (int64_t i = l; i < n; i += W) {
      const float x = w[i];
      weight_sum += x;
      if (x > 0.0f) {
        if (selected == -1) selected = 0;
        if (u[i] < x / weight_sum) selected = (long long)i + (long long)n * l;
      }
    }
    if (selected > best) best = selected;
  }
  free(sum);
  free(local);
  return best == -1 ? -1 : (int32_t)(best % n);
}

int32_t fw_ref64_dprs(const float* w, int32_t n, int32_t W, const float* u) {
  if (n <= 0) return -1;
  float* v = (float*)malloc(sizeof(float) * (size_t)W);
  float* x = (float*)malloc(sizeof(float) * (size_t)W);
  float carry = 0.0f;
  int32_t selected = -1;
  const int64_t bound = (int64_t)n + W - n % W;
  for (int64_t base = 0; base < bound; base += W) {
    int32_t chunk_max = selected;
    for (int l = 0; l < W; ++l) {
      const int64_t i = base + l;
      x[l] = i < n ? w[i] : 0.0f;
      v[l] = x[l];
      if (x[l] > 0.0f && chunk_max < 0) chunk_max = 0;
    }
    scan64(v, W, carry);
    for (int l = 0; l < W; ++l) {
      const int64_t i = base + l;
      if (i < n && x[l] > 0.0f && u[i] < x[l] / v[l] && (int32_t)i > chunk_max) chunk_max = (int32_t)i;
    }
    carry = v[W - 1];
    selected = chunk_max;
  }
  free(v);
  free(x);
  return selected;
}

/* The uniform of element i of a list sampled by a group of W lanes at (walker, step): lane t = i % W draws it as its
 * j-th, j = i / W: word j & 3 of Philox block (j >> 2) * W + t of stream 0x20000000, mapped to (0, 1]. */
float fw_ref64_uniform(uint64_t seed, uint32_t walker, uint32_t step, uint32_t i, uint32_t W) {
  const uint32_t t = i % W, j = i / W;
  const uint32_t ctr[4] = {walker, step, 0x20000000u, (j >> 2) * W + t};
  const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t out[4];
  fw_oracle_philox4x32_10(ctr, key, out);
  return (float)((out[j & 3] >> 8) + 1u) * 0x1p-24f;
}
