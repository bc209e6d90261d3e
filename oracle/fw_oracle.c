/*
 * fw_oracle.c -- CPU oracle for the FlowWalker walk path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, not the product: only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may build, load or call it.  The shipped library never links it
 * and has no CPU fallback.
 *
 * It restates, in plain C, the algorithm of the reference's sampler-centric walk engine and fixes
 * every detail the reference leaves to thread scheduling, so that the HIP kernels can be compared
 * bit for bit.  The reference itself cannot be built here (CUDA + CUB + cuRAND + gflags) and is not
 * a bitwise oracle anyway: its RNG streams belong to threads and its query->slot assignment is an
 * atomic race (include/walker.cuh:1323-1324, :1339).
 *
 * What follows the reference, and where:
 *   - walk control flow (start write, step commit, dead end, stop, -1 padded rows):
 *       include/walker.cuh:1338-1350, :1357-1438; include/gpu_task.cuh:52-77
 *   - sampler: parallel weighted reservoir sampling over lane-strided elements with a prefix scan
 *       over lane totals: include/sampler.cuh:46-85 (warp), :87-127 (block), chunk carry of
 *       :129-155, :157-200; sequential ground truth include/sampler.cuh:26-44
 *   - bias functors and stop rules: include/app.cuh:58-71 (DeepWalk), :73-95 (PPR),
 *       :97-127 (node2vec), :129-152 (MetaPath); adjacency test include/gpu_graph.cuh:97-118
 *   - workload counters (steps, sum of source degrees): src/main.cu:82-113
 *
 * What this build defines differently from the reference (documented, deliberate):
 *   - RNG: Philox4x32-10 (Salmon et al., SC'11), keyed by the 64-bit seed, counter =
 *       (walker id, step, stream, block).  Replaces the stateful XORWOW of include/myrand.cuh.
 *       Pinned by the Random123 known-answer vectors (tests/golden/philox4x32_10_kat.json).
 *   - the sampler is one pass and evaluates every bias once.  The neighbour list is cut into groups
 *       of FW_GROUP_QUARTETS * 64 quartets (1024 elements); each wave runs a sequential weighted
 *       reservoir over the groups it owns, where "element" = a whole group with its total as weight
 *       (the prefix / carry structure of include/sampler.cuh:139-152), and inside an accepted group
 *       the element is picked by inverse transform on the same wave-scan prefix.  The law of the
 *       winner is unchanged: P(i) = (T_g / sum T) * (w_i / T_g) = w_i / sum w.
 *   - reservoir acceptance uses the telescoping identity
 *       P(no accept in (j,k]) = prod S_{i-1}/S_i = S_j/S_k,
 *       so one uniform u decides the NEXT accepted group (first k with S_k*u > S_j) instead of one
 *       uniform per element (include/sampler.cuh:76).  O(log n) draws per step, all wave-uniform.
 *   - no division anywhere: tests are u*S < w-shaped products, never FMA-contracted.
 *   - uniforms are (x >> 8) * 2^-24 in [0,1), exact in f32.
 *   - elements are grouped in 4-element quartets aligned to the absolute CSR index (16-byte
 *       aligned vector loads on the GPU).
 *   - PPR stop draw is made once per completed step of a live walk, from its own stream
 *       (the reference also draws for empty slots, include/walker.cuh:1422-1431).
 *   - node2vec samples in two stages.  The reference evaluates the bias w * f (f = 1/p for the return edge, 1 for a
 *       common neighbour of prev and cur, 1/q otherwise; include/app.cuh:108-123) of EVERY neighbour, one binary
 *       search each, inside its one-pass sampler.  Here a trial proposes a neighbour with probability w_i / sum w
 *       through the same sampler DeepWalk uses (no adjacency test at all) and accepts it with probability f_i / F,
 *       F = max(1, 1/q), which takes ONE adjacency test (include/gpu_graph.cuh:97-118); a rejected trial is
 *       followed by another with its own draws.  P(i) = (w_i / sum w)(f_i / F) / sum_j (w_j / sum w)(f_j / F) =
 *       w_i f_i / sum_j w_j f_j: the reference's law exactly (its own rejection sampler has the same structure,
 *       include/sampler.cuh:202-266).  When 1/p exceeds F, the return edge is the one neighbour the envelope w F does
 *       not cover, and raising F to 1/p would make every other proposal 1/(p F) times less likely to be accepted.
 *       Its excess is a component of its own instead: with T the list's total as the sampler adds it up and R the
 *       weights of the entries that lead back to prev (f32, list order), a trial takes the return edge outright when
 *       u0 (F T + (1/p - F) R) < (1/p - F) R, and otherwise runs as above with the return edge always accepted
 *       (envelope w F for every entry plus (1/p - F) w for the return entries: total mass of an entry w f, as above).
 *       So the number of trials does not depend on p.  Draws of trial t use the streams of a plain step offset by
 *       t << 8; the acceptance uniform is word 0 and u0 word 1 of block 0 of stream FW_STREAM_ACCEPT | t << 8; trial
 *       FW_MAX_TRIALS - 1 is accepted unconditionally (never reached in practice: the acceptance probability is at
 *       least min(1, 1/q) / F).  f uses host-computed f32 reciprocals 1/p and 1/q; the tests are u * F < f and the
 *       one above, no division.
 *   - --dprs selects nothing different: the one sampler already has DPRS's property (one bias
 *       evaluation per neighbour, include/sampler.cuh:129-200), so FW_SAMPLER_DPRS is an alias.
 *
 * Build: make -C oracle   (gcc -O2 -ffp-contract=off -fopenmp)
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define FW_WAVE 64
#define FW_QUAD 4
#define FW_GROUP_QUARTETS 4 /* quartets per lane per group: a group spans 64 * 4 * 4 = 1024 elements */
#define FW_MAX_SCHEMA 64
#define FW_MAX_GROUP 1024

enum { FW_APP_DEEPWALK = 0, FW_APP_PPR = 1, FW_APP_NODE2VEC = 2, FW_APP_METAPATH = 3 };
enum { FW_SAMPLER_ZPRS = 0, FW_SAMPLER_DPRS = 1, FW_SAMPLER_REF_ZPRS = 2, FW_SAMPLER_REF_DPRS = 3 };

/* fw_ref_samplers.c */
int32_t fw_ref64_zprs(const float* w, int32_t n, int32_t W, const float* u);
int32_t fw_ref64_dprs(const float* w, int32_t n, int32_t W, const float* u);
float fw_ref64_uniform(uint64_t seed, uint32_t walker, uint32_t step, uint32_t i, uint32_t W);

#define FW_STREAM_WAVE 0x40000000u   /* workgroup-level combine draw */
#define FW_STREAM_STOP 0x80000000u   /* PPR stop draw */
#define FW_STREAM_ACCEPT 0x10000000u /* node2vec acceptance draw of a trial */
#define FW_MAX_TRIALS 16384u         /* node2vec: trials per step (the trial index travels in 14 bits) */

typedef struct {
  int32_t app;           /* FW_APP_* */
  int32_t sampler;       /* FW_SAMPLER_* */
  int32_t max_depth;     /* path row length = steps + 1 */
  int32_t wg_threads;    /* lanes of the workgroup sampler (multiple of 64, <= 1024) */
  int32_t hub_threshold; /* degree > hub_threshold -> workgroup sampler */
  int32_t schema_len;
  int32_t schema[FW_MAX_SCHEMA];
  float tp;
  float inv_p;
  float inv_q;
  uint32_t walker_base; /* global walker id of query 0 */
  uint64_t seed;
} fw_oracle_params;

typedef struct {
  int32_t V;
  const uint32_t* xadj;
  const int32_t* adjncy;
  const float* weight;  /* NULL for metapath */
  const int32_t* label; /* NULL unless metapath */
} fw_oracle_graph;

/* ---- Philox4x32-10 ------------------------------------------------------------------------ */

void fw_oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* n-th 32-bit draw of stream `stream` at (walker, step): word n&3 of Philox block n>>2. */
static uint32_t draw_bits(uint64_t seed, uint32_t walker, uint32_t step, uint32_t stream, uint32_t n) {
  uint32_t ctr[4] = {walker, step, stream, n >> 2};
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t out[4];
  fw_oracle_philox4x32_10(ctr, key, out);
  return out[n & 3];
}

static float u24(uint32_t bits) { return (float)(bits >> 8) * 0x1p-24f; }

float fw_oracle_uniform(uint64_t seed, uint32_t walker, uint32_t step, uint32_t stream, uint32_t n) {
  return u24(draw_bits(seed, walker, step, stream, n));
}

/* ---- scan trees (mirror of the wave64 DPP scan: row_shr 1,2,4,8; row_bcast15; row_bcast31) - */

/* In-place inclusive scan of 64 floats with the exact association order of the GPU wave scan. */
void fw_oracle_wave_scan(float x[FW_WAVE]) {
  float t[FW_WAVE];
  for (int off = 1; off < 16; off <<= 1) {
    for (int l = 0; l < FW_WAVE; ++l) t[l] = ((l & 15) >= off) ? x[l] + x[l - off] : x[l];
    memcpy(x, t, sizeof(t));
  }
  /* row_bcast:15, rows 1 and 3 */
  {
    float r0 = x[15], r2 = x[47];
    for (int l = 16; l < 32; ++l) x[l] = x[l] + r0;
    for (int l = 48; l < 64; ++l) x[l] = x[l] + r2;
  }
  /* row_bcast:31, rows 2 and 3 */
  {
    float h = x[31];
    for (int l = 32; l < 64; ++l) x[l] = x[l] + h;
  }
}

/* Inclusive scan of m <= 16 floats: one DPP row (row_shr 1,2,4,8). */
static void row_scan(float* x, int m) {
  float t[16];
  for (int off = 1; off < 16; off <<= 1) {
    for (int l = 0; l < m; ++l) t[l] = (l >= off) ? x[l] + x[l - off] : x[l];
    memcpy(x, t, sizeof(float) * m);
  }
}

/* ---- bias functors (include/app.cuh) -------------------------------------------------------- */

typedef struct {
  const fw_oracle_graph* g;
  const fw_oracle_params* p;
  int32_t prev;       /* -1 on the first step */
  uint32_t prev_off;  /* CSR range of prev (node2vec) */
  int32_t prev_deg;
  int32_t want_label; /* metapath: schema[step % schema_len] */
  int n2v_full;       /* node2vec: 1 = the full bias w * f of every neighbour (the reference's samplers), 0 = the plain
                         weight (proposal stage of this build's two-stage step) */
  uint32_t stream_base; /* added to every stream of the step's sampler draws: trial << 8 */
  /* exhaustive tests only (fw_oracle_enumerate_draw): draw (force_stream, force_index) of the step takes
   * force_value instead of its Philox word, and the walker-independent rows of a group are kept between calls */
  int force;
  uint32_t force_stream, force_index;
  float force_value;
  struct group_rows* cache;
  uint64_t cache_groups;
} bias_ctx;

enum { FW_EL = FW_GROUP_QUARTETS * FW_QUAD };
/* What a group's part of the sampler computes before any draw: the 16 biases of every lane, the lane totals and
 * their wave scan. */
typedef struct group_rows {
  float x[FW_WAVE][FW_EL];
  float q[FW_WAVE], I[FW_WAVE];
  int valid;
} group_rows;

/* n-th uniform of stream `stream` at (walker, step) */
static float step_draw(const bias_ctx* c, uint32_t walker, uint32_t step, uint32_t stream, uint32_t n) {
  if (c->force && stream == c->force_stream && n == c->force_index) return c->force_value;
  return u24(draw_bits(c->p->seed, walker, step, stream | c->stream_base, n));
}

/* include/gpu_graph.cuh:97-112 */
static int sorted_contains(const int32_t* arr, int32_t size, int32_t target) {
  int32_t l = 0, r = size - 1;
  while (l <= r) {
    int32_t m = l + (r - l) / 2;
    if (arr[m] == target) return 1;
    if (arr[m] < target) l = m + 1; else r = m - 1;
  }
  return 0;
}

/* Bias of CSR entry `a` (absolute index).  include/app.cuh:64-66, :86-88, :108-123, :141-146. */
static float bias_at(const bias_ctx* c, uint64_t a) {
  switch (c->p->app) {
    case FW_APP_METAPATH:
      return c->g->label[a] == c->want_label ? 1.0f : 0.0f;
    case FW_APP_NODE2VEC: {
      float w = c->g->weight[a];
      if (c->prev == -1 || !c->n2v_full) return w;
      int32_t post = c->g->adjncy[a];
      if (post == c->prev) return w * c->p->inv_p;
      if (!sorted_contains(c->g->adjncy + c->prev_off, c->prev_deg, post)) return w * c->p->inv_q;
      return w;
    }
    default:
      return c->g->weight[a];
  }
}

/* ---- one-pass zero-preprocessing parallel reservoir sampler ------------------------------------- */

/* first i in [0,n) with v[i] > 0 and prefix[i] > target; if there is none, the last i with v[i] > 0
 * (rounding in the prefix tree may leave no crossing); -1 when no v[i] is positive. */
static int pick_by_prefix(const float* v, const float* prefix, int n, float target) {
  int last = -1;
  for (int i = 0; i < n; ++i) {
    if (v[i] > 0.0f) {
      if (prefix[i] > target) return i;
      last = i;
    }
  }
  return last;
}

/*
 * Samples one local index in [0,deg) with probability bias_i / sum(bias), or -1 when no bias is
 * positive.  nw waves of 64 lanes (1 = wave granularity, wg_threads / 64 = workgroup).
 *
 * Quartet k of the list (aligned to the absolute CSR index) belongs to group k / (64 * U), U =
 * FW_GROUP_QUARTETS; inside group g, lane l owns quartets g*64*U + j*64 + l, j = 0..U-1.  Wave w owns
 * groups w, w + nw, ...  For each owned group: lane totals q (sequential f32 adds in (j, element)
 * order), wave scan I of q, group total T = I[63], running sum S += T; the group is accepted iff
 * S * u > Sj.  On acceptance: target = draw * T; lane = pick_by_prefix(q, I); inside the lane the
 * running sum starts at I[lane] - q[lane] and the element is pick_by_prefix again; then Sj = S and
 * u = next draw.  Draws of wave w at (walker, step) are consecutive words of Philox stream w.
 * Waves are combined by one more inverse transform on the row scan of the wave totals.
 */
static int32_t group_sample(const bias_ctx* c, uint32_t off, int32_t deg, int nw, uint32_t walker,
                            uint32_t step, float* total_out) {
  if (total_out) *total_out = 0.0f;
  if (deg <= 0) return -1;
  enum { U = FW_GROUP_QUARTETS, EL = FW_EL, G = FW_WAVE * FW_GROUP_QUARTETS };
  const uint64_t a0 = (uint64_t)off & ~(uint64_t)(FW_QUAD - 1);
  const uint64_t end = (uint64_t)off + (uint64_t)deg;
  const uint64_t nq = (end - a0 + FW_QUAD - 1) / FW_QUAD;
  const uint64_t ngroups = (nq + G - 1) / G;

  float W[16];
  int32_t wsel[16];
  for (int wv = 0; wv < nw; ++wv) {
    float S = 0.0f, Sj = 0.0f, u = 1.0f;
    int32_t sel = -1;
    uint32_t nd = 0;
    for (uint64_t g = (uint64_t)wv; g < ngroups; g += (uint64_t)nw) {
      group_rows local;
      group_rows* r = (c->cache && g < c->cache_groups) ? &c->cache[g] : &local;
      if (r == &local || !r->valid) {
        for (int l = 0; l < FW_WAVE; ++l) {
          float s = 0.0f;
          for (int j = 0; j < U; ++j) {
            const uint64_t k = g * G + (uint64_t)j * FW_WAVE + (uint64_t)l;
            for (int e = 0; e < FW_QUAD; ++e) {
              const uint64_t a = a0 + FW_QUAD * k + (uint64_t)e;
              const float b = (k < nq && a >= off && a < end) ? bias_at(c, a) : 0.0f;
              r->x[l][j * FW_QUAD + e] = b;
              s = s + b;
            }
          }
          r->q[l] = s;
          r->I[l] = s;
        }
        fw_oracle_wave_scan(r->I);
        r->valid = 1;
      }
      const float* q = r->q;
      const float* I = r->I;
      const float T = I[FW_WAVE - 1];
      const float Snew = S + T;
      const float lhs = Snew * u;
      if (lhs > Sj) {
        const float u2 = step_draw(c, walker, step, (uint32_t)wv, nd++);
        const float target = u2 * T;
        const int lane = pick_by_prefix(q, I, FW_WAVE, target);
        /* lane >= 0: acceptance implies T > 0, hence some q > 0 */
        float pre[EL];
        float e = I[lane] - q[lane];
        for (int i = 0; i < EL; ++i) {
          e = e + r->x[lane][i];
          pre[i] = e;
        }
        const int pick = pick_by_prefix(r->x[lane], pre, EL, target);
        const uint64_t k = g * G + (uint64_t)(pick / FW_QUAD) * FW_WAVE + (uint64_t)lane;
        sel = (int32_t)(a0 + FW_QUAD * k + (uint64_t)(pick % FW_QUAD) - off);
        Sj = Snew;
        u = step_draw(c, walker, step, (uint32_t)wv, nd++);
      }
      S = Snew;
    }
    W[wv] = S;
    wsel[wv] = sel;
  }
  if (nw == 1) {
    if (total_out) *total_out = W[0];
    return wsel[0];
  }

  float J[16];
  for (int wv = 0; wv < nw; ++wv) J[wv] = W[wv];
  row_scan(J, nw);
  if (total_out) *total_out = J[nw - 1];
  const float u3 = step_draw(c, walker, step, FW_STREAM_WAVE, 0u);
  const float target = u3 * J[nw - 1];
  const int wv = pick_by_prefix(W, J, nw, target);
  return wv < 0 ? -1 : wsel[wv];
}

/* One sampling step, exposed for sampler-level tests.  Granularity by degree as in
 * include/walker.cuh:1362 (degree <= threshold -> wave, else workgroup). */
int32_t fw_oracle_sample(const fw_oracle_graph* g, const fw_oracle_params* p, int32_t cur,
                         int32_t prev, uint32_t walker, uint32_t step) {
  bias_ctx c;
  c.g = g; c.p = p; c.prev = prev;
  c.prev_off = 0; c.prev_deg = 0;
  c.force = 0; c.cache = NULL; c.cache_groups = 0;
  c.n2v_full = 0; c.stream_base = 0;
  if (prev >= 0) { c.prev_off = g->xadj[prev]; c.prev_deg = (int32_t)(g->xadj[prev + 1] - g->xadj[prev]); }
  c.want_label = (p->app == FW_APP_METAPATH && p->schema_len > 0) ? p->schema[step % (uint32_t)p->schema_len] : 0;
  uint32_t off = g->xadj[cur];
  int32_t deg = (int32_t)(g->xadj[cur + 1] - off);
  const int nw = (deg > p->hub_threshold) ? p->wg_threads / FW_WAVE : 1;
  const int kind = p->sampler & 0xFF;
  if (kind == FW_SAMPLER_REF_ZPRS || kind == FW_SAMPLER_REF_DPRS) {
    /* the reference's own samplers on 64-lane waves (fw_ref_samplers.c), fed with this build's biases and uniforms */
    if (deg <= 0) return -1;
    c.n2v_full = 1;
    const int32_t W = nw * FW_WAVE;
    float* w = (float*)malloc(sizeof(float) * (size_t)deg);
    float* u = (float*)malloc(sizeof(float) * (size_t)deg);
    for (int32_t i = 0; i < deg; ++i) {
      w[i] = bias_at(&c, (uint64_t)off + (uint32_t)i);
      u[i] = fw_ref64_uniform(p->seed, walker, step, (uint32_t)i, (uint32_t)W);
    }
    const int32_t sel = kind == FW_SAMPLER_REF_ZPRS ? fw_ref64_zprs(w, deg, W, u) : fw_ref64_dprs(w, deg, W, u);
    free(w);
    free(u);
    return sel;
  }
  if (p->app != FW_APP_NODE2VEC || prev < 0) return group_sample(&c, off, deg, nw, walker, step, NULL);
  /* node2vec after the first step: propose by weight, accept by f / F (include/app.cuh:108-123 for f).  F covers the
   * common neighbours and the others; the return edge's excess over it is a component of its own (header). */
  float F = 1.0f;
  if (p->inv_q > F) F = p->inv_q;
  const float extra = p->inv_p > F ? p->inv_p - F : 0.0f;
  float w_ret = 0.0f;     /* weights of the entries of N(cur) that lead back to prev, in list order */
  int32_t first_ret = -1;
  if (extra > 0.0f) {
    for (int32_t i = 0; i < deg; ++i) {
      if (g->adjncy[(uint64_t)off + (uint32_t)i] == prev) {
        if (first_ret < 0) first_ret = i;
        w_ret = w_ret + bias_at(&c, (uint64_t)off + (uint32_t)i);
      }
    }
  }
  for (uint32_t trial = 0;; ++trial) {
    c.stream_base = trial << 8;
    float T = 0.0f;
    const int32_t sel = group_sample(&c, off, deg, nw, walker, step, &T);
    if (sel < 0) return -1; /* no positive weight: dead end, whatever the trial */
    if (trial == FW_MAX_TRIALS - 1u) return sel;
    const int32_t post = g->adjncy[(uint64_t)off + (uint32_t)sel];
    if (extra > 0.0f) {
      const float u0 = u24(draw_bits(p->seed, walker, step, FW_STREAM_ACCEPT | (trial << 8), 1u));
      const float gx = extra * w_ret;
      const float gb = F * T;
      const float lhs0 = u0 * (gb + gx);
      if (lhs0 < gx) return first_ret; /* the return edge's own component (gx > 0: there is such an entry) */
      if (post == prev) return sel;    /* its share of the proposals is never turned down */
    }
    float f;
    if (post == prev) f = p->inv_p;
    else if (sorted_contains(g->adjncy + c.prev_off, c.prev_deg, post)) f = 1.0f;
    else f = p->inv_q;
    const float u = u24(draw_bits(p->seed, walker, step, FW_STREAM_ACCEPT | (trial << 8), 0u));
    const float lhs = u * F;
    if (lhs < f) return sel;
  }
}

/* ---- whole walks (include/walker.cuh:1338-1438) --------------------------------------------- */

static void walk_one(const fw_oracle_graph* g, const fw_oracle_params* p, int32_t start, uint32_t walker,
                     int32_t* row, uint64_t* steps, uint64_t* edges) {
  const int md = p->max_depth;
  for (int i = 0; i < md; ++i) row[i] = -1;
  if (md <= 0) return;
  row[0] = start;
  if (start < 0 || start >= g->V) return;
  int32_t cur = start, prev = -1;
  int len = 1;
  while (len < md) {
    uint32_t step = (uint32_t)(len - 1);
    uint32_t off = g->xadj[cur];
    int32_t deg = (int32_t)(g->xadj[cur + 1] - off);
    int32_t s = fw_oracle_sample(g, p, cur, prev, walker, step);
    if (s < 0) break; /* dead end: include/walker.cuh:1373-1374 */
    int32_t v = g->adjncy[(uint64_t)off + (uint32_t)s];
    row[len] = v;
    *steps += 1;
    *edges += (uint64_t)deg; /* src/main.cu:101-103 */
    prev = cur;
    cur = v;
    ++len;
    if (p->app == FW_APP_PPR) { /* include/app.cuh:88-94 */
      float r = u24(draw_bits(p->seed, walker, step, FW_STREAM_STOP, 0u));
      if (r < p->tp) break;
    }
  }
}

/*
 * Runs n queries; paths is int32[n][max_depth], -1 padded, column 0 = start vertex
 * (include/walker.cuh:1342, :1379-1381).  steps / edges as src/main.cu:93-104.
 * nthreads <= 0: all cores (OpenMP schedule(dynamic) over walkers).
 */
static int walk_many(const fw_oracle_graph* g, const fw_oracle_params* p, const int32_t* starts,
                     const uint32_t* walker_ids, int64_t n, int32_t* paths, uint64_t* steps_out, uint64_t* edges_out,
                     int nthreads) {
  if (p->wg_threads % FW_WAVE != 0 || p->wg_threads > FW_MAX_GROUP || p->wg_threads < FW_WAVE) return -1;
  if (p->app == FW_APP_METAPATH && (p->schema_len <= 0 || p->schema_len > FW_MAX_SCHEMA)) return -1;
  uint64_t steps = 0, edges = 0;
#ifdef _OPENMP
  if (nthreads > 0) omp_set_num_threads(nthreads);
#else
  (void)nthreads;
#endif
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : steps, edges)
  for (int64_t q = 0; q < n; ++q) {
    uint64_t s = 0, e = 0;
    const uint32_t walker = walker_ids ? walker_ids[q] : p->walker_base + (uint32_t)q;
    walk_one(g, p, starts[q], walker, paths + (uint64_t)q * p->max_depth, &s, &e);
    steps += s;
    edges += e;
  }
  if (steps_out) *steps_out = steps;
  if (edges_out) *edges_out = edges;
  return 0;
}

int fw_oracle_walk(const fw_oracle_graph* g, const fw_oracle_params* p, const int32_t* starts, int64_t n,
                   int32_t* paths, uint64_t* steps_out, uint64_t* edges_out, int nthreads) {
  return walk_many(g, p, starts, NULL, n, paths, steps_out, edges_out, nthreads);
}

/* The same for chosen rows of a larger job: query i is the walk of global walker id walker_ids[i] (draws are
 * addressed by walker id, so row r of a job equals this walk with walker_ids[i] = walker_base + r). */
int fw_oracle_walk_ids(const fw_oracle_graph* g, const fw_oracle_params* p, const int32_t* starts,
                       const uint32_t* walker_ids, int64_t n, int32_t* paths, uint64_t* steps_out,
                       uint64_t* edges_out, int nthreads) {
  return walk_many(g, p, starts, walker_ids, n, paths, steps_out, edges_out, nthreads);
}

int fw_oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---- the reference's engine with thread-owned generators, replayed thread by thread -------------------------------
 *
 * FW_SAMPLER_REF_ZPRS / _DPRS with static query assignment and FW_SAMPLER_REF_RNG_LDS / _GLOBAL (the "FW" and "+ RNG"
 * levels of the reference's ablation, README.md:152-163): the generators belong to the threads, as the reference's do
 * (include/myrand.cuh:271-292: sequence = global thread id; walker_wb_dprs_curand, include/walker.cuh:1584-1696), so a
 * walk is no longer a function of the walker alone.  With static assignment it is still a function of the launch:
 *   - workgroup b of `grid` owns queries [b * per, (b + 1) * per), per = ceil(n / grid) (src/walk.cu:46-61), and
 *     grid is cut to ceil(n / 64) workgroups; it has 64 task slots (TASK_NUM, include/walker.cuh:28) and
 *     W = wg_threads threads in W / 64 waves;
 *   - slots take the next queries in slot order (at the start, and after a round for the slots whose walk ended);
 *   - a round (include/walker.cuh:1357-1438): wave v steps slots v, v + W/64, ... whose degree is at most
 *     hub_threshold with the wave sampler (its 64 threads draw), then the deferred slots are stepped in slot order by
 *     the workgroup sampler (all W threads draw), then the stop rule (PPR's stop draw is addressed by the walker:
 *     stream FW_STREAM_STOP);
 *   - thread gid = b * W + t takes as its k-th uniform word k & 3 of Philox block (gid, k >> 2, 0x08000000, 0),
 *     mapped to (0, 1]; a DPRS step costs every thread of the group one draw per chunk (also the lanes past the end
 *     of the list, include/sampler.cuh:139-152), a ZPRS step one draw per element the thread owns.
 * The samplers themselves are fw_ref64_zprs / fw_ref64_dprs, fed with these uniforms.
 */
typedef struct {
  uint64_t seed;
  uint32_t gid0;     /* global id of the workgroup's thread 0 */
  uint32_t* count;   /* [W] draws taken so far by each thread */
} thread_rngs;

static float thread_draw(thread_rngs* r, uint32_t t) {
  const uint32_t k = r->count[t]++;
  const uint32_t ctr[4] = {r->gid0 + t, k >> 2, 0x08000000u, 0u};
  const uint32_t key[2] = {(uint32_t)r->seed, (uint32_t)(r->seed >> 32)};
  uint32_t out[4];
  fw_oracle_philox4x32_10(ctr, key, out);
  return (float)((out[k & 3] >> 8) + 1u) * 0x1p-24f;
}

/* One step of slot state (cur, prev) at `step` by the threads t0 .. t0 + W - 1 of the workgroup. */
static int32_t thread_rng_step(const fw_oracle_graph* g, const fw_oracle_params* p, int32_t cur, int32_t prev,
                               uint32_t step, thread_rngs* r, uint32_t t0, int32_t W) {
  bias_ctx c;
  c.g = g; c.p = p; c.prev = prev;
  c.prev_off = 0; c.prev_deg = 0;
  c.force = 0; c.cache = NULL; c.cache_groups = 0;
  c.n2v_full = 1; c.stream_base = 0;
  if (prev >= 0) { c.prev_off = g->xadj[prev]; c.prev_deg = (int32_t)(g->xadj[prev + 1] - g->xadj[prev]); }
  c.want_label = (p->app == FW_APP_METAPATH && p->schema_len > 0) ? p->schema[step % (uint32_t)p->schema_len] : 0;
  const uint32_t off = g->xadj[cur];
  const int32_t deg = (int32_t)(g->xadj[cur + 1] - off);
  if (deg <= 0) return -1;
  float* w = (float*)malloc(sizeof(float) * (size_t)deg);
  float* u = (float*)malloc(sizeof(float) * (size_t)deg);
  for (int32_t i = 0; i < deg; ++i) w[i] = bias_at(&c, (uint64_t)off + (uint32_t)i);
  int32_t sel;
  if ((p->sampler & 0xFF) == FW_SAMPLER_REF_DPRS) {
    const int64_t bound = (int64_t)deg + W - deg % W; /* include/sampler.cuh:138, :167 */
    for (int64_t base = 0; base < bound; base += W)
      for (int32_t l = 0; l < W; ++l) {
        const float d = thread_draw(r, t0 + (uint32_t)l);
        if (base + l < deg) u[base + l] = d;
      }
    sel = fw_ref64_dprs(w, deg, W, u);
  } else {
    for (int32_t l = 0; l < W; ++l)
      for (int64_t i = l; i < deg; i += W) u[i] = thread_draw(r, t0 + (uint32_t)l);
    sel = fw_ref64_zprs(w, deg, W, u);
  }
  free(w);
  free(u);
  return sel;
}

int fw_oracle_walk_ref_threads(const fw_oracle_graph* g, const fw_oracle_params* p, const int32_t* starts, int64_t n,
                               int32_t grid, int32_t* paths, uint64_t* steps_out, uint64_t* edges_out) {
  enum { SLOTS = 64 };
  const int32_t W = p->wg_threads;
  const int kind = p->sampler & 0xFF;
  if (W % FW_WAVE != 0 || W > FW_MAX_GROUP || W < FW_WAVE || grid < 1 || n < 1) return -1;
  if (kind != FW_SAMPLER_REF_ZPRS && kind != FW_SAMPLER_REF_DPRS) return -1;
  const int64_t needed = (n + SLOTS - 1) / SLOTS;
  if (grid > needed) grid = (int32_t)needed;
  const int md = p->max_depth;
  const int nw = W / FW_WAVE;
  const int64_t per = (n + grid - 1) / grid;
  uint64_t steps = 0, edges = 0;
  for (int64_t i = 0; i < n * (int64_t)md; ++i) paths[i] = -1;
#pragma omp parallel for schedule(dynamic, 1) reduction(+ : steps, edges)
  for (int32_t b = 0; b < grid; ++b) {
    const int64_t lo = (int64_t)b * per < n ? (int64_t)b * per : n;
    const int64_t hi = lo + per < n ? lo + per : n;
    int64_t cursor = lo;
    thread_rngs r;
    r.seed = p->seed;
    r.gid0 = (uint32_t)b * (uint32_t)W;
    r.count = (uint32_t*)calloc((size_t)W, sizeof(uint32_t));
    int64_t q_of[SLOTS];
    int32_t cur[SLOTS], prev[SLOTS], len[SLOTS], moved[SLOTS];
    int large[SLOTS];
    int active = 0;
    for (int s = 0; s < SLOTS; ++s) { len[s] = -1; large[s] = 0; }
    /* Task::init (include/gpu_task.cuh:52-68) */
#define FW_TAKE_QUERY(s)                                                   \
    do {                                                                   \
      if (cursor < hi) {                                                   \
        const int64_t q = cursor++;                                        \
        q_of[s] = q;                                                       \
        cur[s] = starts[q];                                                \
        prev[s] = -1;                                                      \
        moved[s] = 0;                                                      \
        paths[q * md] = starts[q];                                         \
        len[s] = (starts[q] >= 0 && starts[q] < g->V) ? 1 : md;            \
        ++active;                                                          \
      } else {                                                             \
        len[s] = -1;                                                       \
      }                                                                    \
    } while (0)
    for (int s = 0; s < SLOTS; ++s) FW_TAKE_QUERY(s);
    while (active > 0) {
      for (int pass = 0; pass < 2; ++pass) {
        /* pass 0: the waves step their slots (wave v: slots v, v + nw, ... in this order; the waves do not share
         * threads, so their order among each other does not matter); pass 1: the deferred slots, by the workgroup */
        for (int v = 0; v < (pass == 0 ? nw : 1); ++v)
          for (int s = (pass == 0 ? v : 0); s < SLOTS; s += (pass == 0 ? nw : 1)) {
            if (pass == 0) {
              if (len[s] < 0 || len[s] >= md) continue;
              const int32_t deg = (int32_t)(g->xadj[cur[s] + 1] - g->xadj[cur[s]]);
              if (deg > p->hub_threshold) { large[s] = 1; continue; }
            } else {
              if (!large[s]) continue;
            }
            const uint32_t off = g->xadj[cur[s]];
            const int32_t deg = (int32_t)(g->xadj[cur[s] + 1] - off);
            const int32_t sel = pass == 0
                ? thread_rng_step(g, p, cur[s], prev[s], (uint32_t)(len[s] - 1), &r, (uint32_t)v * FW_WAVE, FW_WAVE)
                : thread_rng_step(g, p, cur[s], prev[s], (uint32_t)(len[s] - 1), &r, 0u, W);
            if (sel < 0) { /* include/walker.cuh:1373-1374 */
              len[s] = md;
              moved[s] = 0;
              continue;
            }
            const int32_t nv = g->adjncy[(uint64_t)off + (uint32_t)sel];
            paths[q_of[s] * md + len[s]] = nv;
            prev[s] = cur[s];
            cur[s] = nv;
            len[s] += 1;
            moved[s] = 1;
            steps += 1;
            edges += (uint64_t)deg;
          }
      }
      for (int s = 0; s < SLOTS; ++s) { /* include/walker.cuh:1422-1432, on live slots only */
        large[s] = 0;
        if (len[s] < 0) continue;
        int stop = len[s] >= md || g->xadj[cur[s] + 1] == g->xadj[cur[s]];
        if (p->app == FW_APP_PPR && !stop && moved[s]) { /* include/app.cuh:88-94 */
          const uint32_t walker = p->walker_base + (uint32_t)q_of[s];
          stop = u24(draw_bits(p->seed, walker, (uint32_t)(len[s] - 2), FW_STREAM_STOP, 0u)) < p->tp;
        }
        moved[s] = 0;
        if (stop) {
          --active;
          FW_TAKE_QUERY(s);
        }
      }
    }
#undef FW_TAKE_QUERY
    free(r.count);
  }
  if (steps_out) *steps_out = steps;
  if (edges_out) *edges_out = edges;
  return 0;
}

/* ---- sequential ground truth (include/sampler.cuh:26-44), for brute-force equivalence tests -- */

/*
 * Textbook sequential weighted reservoir sampling over `n` biases in the given order with one
 * uniform per positive element: accept i iff u_i * S_i < w_i.  Returns the last accepted index.
 */
int32_t fw_oracle_sequential_reservoir(const float* w, const float* u, int32_t n) {
  float S = 0.0f;
  int32_t pick = -1;
  for (int32_t i = 0; i < n; ++i) {
    S = S + w[i];
    if (w[i] > 0.0f) {
      float lhs = u[i] * S;
      if (lhs < w[i]) pick = i;
    }
  }
  return pick;
}

/* ---- exhaustive enumeration of one draw (tests only) ------------------------------------------ */

/*
 * A sampling step is a deterministic function of its uniforms, and a uniform has only 2^24 values.  For a list
 * of `deg` biases whose first element sits at absolute CSR index `off` (0..3: only the alignment matters), sampled by `nw`
 * waves, this runs the step once for every value v * 2^-24 of draw number `index` of stream `stream` (stream w =
 * the draws of wave w: target of its first accepted group, jump uniform, target of the next accepted group, ...;
 * FW_STREAM_WAVE, index 0 = the draw that combines the waves) while all other draws keep their Philox words for
 * (seed, walker, step), and counts how often each local index is returned: counts[i + 1] for index i, counts[0]
 * for -1.  The exact law of those counts follows from the prefix sums of the biases alone.
 */
int fw_oracle_enumerate_draw(const float* bias, int32_t deg, uint32_t off, int32_t nw, uint32_t stream, uint32_t index,
                             uint64_t seed, uint32_t walker, uint32_t step, uint64_t* counts) {
  if (deg <= 0 || nw < 1 || nw > 16 || off > 3u) return -1; /* only off mod 4 matters: pass 0..3 */
  float* padded = (float*)calloc((size_t)off + (size_t)deg + FW_QUAD, sizeof(float));
  if (!padded) return -1;
  memcpy(padded + off, bias, (size_t)deg * sizeof(float));
  fw_oracle_params p;
  memset(&p, 0, sizeof(p));
  p.app = FW_APP_DEEPWALK;
  p.seed = seed;
  /* a graph whose weight array is addressed like a CSR that holds this list at `off` */
  fw_oracle_graph g;
  g.V = 1; g.xadj = NULL; g.adjncy = NULL; g.label = NULL;
  g.weight = padded;
  const uint64_t ngroups = (((uint64_t)(off & 3u) + (uint64_t)deg + 3u) / 4u + FW_WAVE * FW_GROUP_QUARTETS - 1) /
                           (FW_WAVE * FW_GROUP_QUARTETS);
  for (int32_t i = 0; i <= deg; ++i) counts[i] = 0;
  int failed = 0;
#pragma omp parallel
  {
    group_rows* cache = (group_rows*)calloc((size_t)ngroups, sizeof(group_rows));
    uint64_t* mine = (uint64_t*)calloc((size_t)deg + 1, sizeof(uint64_t));
    if (!cache || !mine) {
#pragma omp atomic write
      failed = 1;
    } else {
      bias_ctx c;
      memset(&c, 0, sizeof(c));
      c.g = &g; c.p = &p; c.prev = -1;
      c.force = 1; c.force_stream = stream; c.force_index = index;
      c.cache = cache; c.cache_groups = ngroups;
#pragma omp for schedule(static)
      for (int64_t v = 0; v < (1 << 24); ++v) {
        c.force_value = (float)v * 0x1p-24f;
        const int32_t s = group_sample(&c, off, deg, nw, walker, step, NULL);
        mine[s + 1] += 1;
      }
#pragma omp critical
      for (int32_t i = 0; i <= deg; ++i) counts[i] += mine[i];
    }
    free(cache);
    free(mine);
  }
  free(padded);
  return failed ? -1 : 0;
}

/* The same step for one forced value of that draw: the local index it returns (-1: none). */
int32_t fw_oracle_sample_forced(const float* bias, int32_t deg, uint32_t off, int32_t nw, uint32_t stream, uint32_t index,
                                float value, uint64_t seed, uint32_t walker, uint32_t step) {
  if (deg <= 0 || nw < 1 || nw > 16 || off > 3u) return -2;
  float* padded = (float*)calloc((size_t)off + (size_t)deg + FW_QUAD, sizeof(float));
  if (!padded) return -2;
  memcpy(padded + off, bias, (size_t)deg * sizeof(float));
  fw_oracle_params p;
  memset(&p, 0, sizeof(p));
  p.app = FW_APP_DEEPWALK;
  p.seed = seed;
  fw_oracle_graph g;
  g.V = 1; g.xadj = NULL; g.adjncy = NULL; g.label = NULL;
  g.weight = padded;
  bias_ctx c;
  memset(&c, 0, sizeof(c));
  c.g = &g; c.p = &p; c.prev = -1;
  c.force = 1; c.force_stream = stream; c.force_index = index; c.force_value = value;
  const int32_t sel = group_sample(&c, off, deg, nw, walker, step, NULL);
  free(padded);
  return sel;
}
