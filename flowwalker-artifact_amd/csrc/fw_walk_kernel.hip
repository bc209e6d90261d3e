// Sampler-centric random-walk kernel for gfx950 (MI355X): persistent workgroups, an LDS task table,
// a global atomic query dispenser, a one-pass zero-preprocessing parallel reservoir sampler at
// wavefront (64 lanes) and workgroup granularity, Philox4x32-10 counter-based draws, and the
// DeepWalk / PPR / node2vec / MetaPath bias functors.
//
// Reference behaviour this replaces: walker_wb_dynamic_zprs / _dprs (include/walker.cuh:1307-1580),
// sampler_warp / sampler_block and their one-loop forms (include/sampler.cuh:46-200), Task
// (include/gpu_task.cuh:24-78), the functors of include/app.cuh:58-152 and check_connect
// (include/gpu_graph.cuh:97-118).
//
// Sampler.  A neighbour list is cut into groups of 64 lanes x 4 quartets x 4 elements = 1024 biases.
// A wave streams the groups it owns: four aligned 16-byte loads per lane, 16 adds, one DPP scan of the
// lane totals.  The group totals feed a sequential weighted reservoir whose acceptance test
// "S * u > Sj" uses one uniform per ACCEPTED group (the probability of no acceptance between two
// groups telescopes to a ratio of running sums), so the common iteration has no random draw and no
// divergent branch.  Inside an accepted group the element is found by inverse transform on the scan
// prefix.  All draws of a step are wave-uniform, so Philox runs on the scalar unit.
//
// Round structure of one workgroup (WGT threads, WGT task slots in LDS, SoA):
//   B  every hub slot (degree > hub_threshold) is streamed by the whole workgroup, wave w taking
//      groups w, w + NW, ...; per-wave (selection, total) pairs are parked in LDS; one barrier per
//      chunk of hubs, then one wave per hub picks the winning wave and commits the step.
//   A  waves claim the remaining slots one by one from an LDS counter and sample them alone.
//   C  one thread per slot: reload the CSR range of the new vertex, stop test, refill from the
//      global dispenser (one atomic per wave per refill round), classify into next round's lists.
//
// Results depend only on (seed, walker id, graph, parameters): every random draw is addressed by
// (walker, step, stream, draw index), never by which wave or workgroup happens to run the slot.

#include <mutex>
#include "fw_internal.h"
#include "fw_device_util.h"

namespace {

constexpr int kPipelineInFlight = 4;            // bundles of short lists a wave loads per turn in launches of the parking pipeline
constexpr uint32_t kStreamWave = 0x40000000u;  // workgroup-level combine draw
constexpr uint32_t kStreamStop = 0x80000000u;  // PPR stop draw
constexpr uint32_t kStreamAccept = 0x10000000u;  // node2vec acceptance draw of a trial
constexpr uint32_t kMaxTrials = 16384u;          // node2vec: trials per step (the trial index travels in 14 bits)
constexpr int kHubChunk = 32;                  // hub tasks whose wave partials are parked in LDS at once
constexpr int kGroupQuartets = 4;              // quartets per lane per group (part of the sampler's definition)
constexpr int kFlagMoved = 1;
constexpr int kFlagDead = 2;
constexpr int kFlagRetry = 4;                  // node2vec: the proposal was rejected, the slot samples again

// ---- per-step context (wave-uniform) -----------------------------------------------------------

struct StepCtx {
  uint32_t off;
  int32_t deg;
  int32_t prev;
  uint32_t prev_off;
  int32_t prev_deg;
  int32_t want;  // metapath label of this step
  uint32_t walker;
  uint32_t step;
  uint32_t sbase;  // added to every stream of the step's sampler draws: node2vec's trial << 8, else 0
};

// ---- node2vec: two-stage step -----------------------------------------------------------------------
// The reference evaluates the bias w * f of every neighbour (f = 1/p for the return edge, 1 for a common neighbour
// of prev and cur, 1/q otherwise: include/app.cuh:108-123), one binary search each.  Here a trial proposes a
// neighbour with probability w_i / sum w through the sampler every application shares -- no adjacency test, and
// walkers that stand on the same vertex can share the pass over its list -- and accepts it with probability
// f_i / F, F = max(1, 1/p, 1/q): ONE search in N(prev) (include/gpu_graph.cuh:97-112).  A rejected trial is
// followed by another with draws of its own (streams offset by trial << 8).  The accepted neighbour has the
// reference's law, w_i f_i / sum_j w_j f_j.

// is `target` in the ascending arr[0, size)?  (one lane on its own: the hub batch kernel, where every lane serves
// another walker)
__device__ __forceinline__ bool sorted_contains(const int32_t* __restrict__ arr, int32_t size, int32_t target) {
  int32_t l = 0, r = size - 1;
  while (l <= r) {
    const int32_t m = l + ((r - l) >> 1);
    const int32_t x = arr[m];
    if (x == target) return true;
    if (x < target) l = m + 1; else r = m - 1;
  }
  return false;
}

// Sum of the weights of the entries of the ascending list adj[0, size) that equal `target`, added in list order
// (0 when there is none): the return edges of a node2vec step.
__device__ __forceinline__ float return_weight(const int32_t* __restrict__ adj, const float* __restrict__ w, uint32_t size,
                                               int32_t target) {
  uint32_t lo = 0u, hi = size;  // first entry that is not smaller
  while (lo < hi) {
    const uint32_t mid = (lo + hi) >> 1;
    if (adj[mid] < target) lo = mid + 1u; else hi = mid;
  }
  float sum = 0.0f;
  while (lo < size && adj[lo] == target) {
    sum = sum + w[lo];
    ++lo;
  }
  return sum;
}

// The same question answered by a whole wave for one (wave-uniform) list and target: 64 probes per round instead
// of one, so a list of 100,000 entries takes three dependent loads instead of seventeen.  Lane l probes the last
// entry of the l-th of 64 chunks; the entries ascend, so the lanes whose probe is smaller than the target form a
// prefix and the first entry that is not smaller lies in the chunk after it.
__device__ __forceinline__ bool wave_contains(const int32_t* __restrict__ arr, uint32_t size, int32_t target, int lane) {
  uint32_t lo = 0u, hi = size;
  while (hi - lo > 64u) {  // wave-uniform
    const uint32_t chunk = (hi - lo + 63u) >> 6;
    uint32_t idx = lo + ((uint32_t)lane + 1u) * chunk - 1u;
    idx = idx < hi ? idx : hi - 1u;
    const uint32_t cnt = (uint32_t)__builtin_popcountll(__ballot(arr[idx] < target));
    if (cnt == 64u) return false;  // every entry is smaller
    lo += cnt * chunk;
    hi = lo + chunk < hi ? lo + chunk : hi;
  }
  const uint32_t i = lo + (uint32_t)lane;
  return __ballot(i < hi && arr[i] == target) != 0ull;
}

// And by the kSeg lanes of a segment of a wave, every segment for a list and a target of its own (size 0: nothing
// to look for): kSeg probes per round.  All lanes of the wave call it together.
template <int kSeg>
__device__ __forceinline__ bool segment_contains(const int32_t* __restrict__ arr, uint32_t size, int32_t target,
                                                 int lane) {
  constexpr uint32_t kS = (uint32_t)kSeg;
  constexpr uint32_t kShift = kSeg == 32 ? 5u : 4u;
  const uint32_t c = (uint32_t)lane & (kS - 1u);
  const int seg_first = lane & ~(kSeg - 1);
  const uint32_t seg_mask = kSeg == 32 ? 0xFFFFFFFFu : 0xFFFFu;
  uint32_t lo = 0u, hi = size;
  for (;;) {
    const bool big = hi - lo > kS;  // uniform in the segment
    if (__ballot(big) == 0ull) break;
    const uint32_t chunk = (hi - lo + kS - 1u) >> kShift;
    uint32_t idx = lo + (c + 1u) * chunk - 1u;
    idx = idx < hi ? idx : hi - 1u;
    const bool less = big && arr[idx] < target;
    const uint32_t cnt = (uint32_t)__builtin_popcount((uint32_t)(__ballot(less) >> seg_first) & seg_mask);
    if (big) {
      if (cnt == kS) {
        lo = hi;  // every entry is smaller
      } else {
        lo += cnt * chunk;
        hi = lo + chunk < hi ? lo + chunk : hi;
      }
    }
  }
  const uint32_t i = lo + c;
  const uint64_t m = __ballot(i < hi && arr[i] == target);
  return ((uint32_t)(m >> seg_first) & seg_mask) != 0u;
}

// The acceptance test u * F < f of trial `trial` at (walker, step) in two halves, so that the search for the proposal
// in N(prev) is only made when its answer matters: f is 1/p for the return edge, else 1 (common neighbour) or 1/q, so a
// threshold u * F below both is accepted and one that reaches both is rejected whichever it is.  F = max(1, 1/q).
// When 1/p is larger than that (a.n2v_extra = 1/p - F > 0) the return edge's excess is a component of its own: with T
// the list's total as the sampler added it up and w_ret the weights of the entries that lead back to prev, the trial
// takes the return edge outright when u0 (F T + extra w_ret) < extra w_ret (take_prev), and otherwise the return
// edge among the proposals is always accepted.  The number of trials then does not depend on p.
struct N2vTest {
  float uF;          // u * F
  bool decided;      // no search needed
  bool accept;       // the decision when decided
  bool take_prev;    // the step goes back to the previous vertex whatever was proposed
};

__device__ __forceinline__ N2vTest n2v_test(const fw_kargs& a, int32_t post, int32_t prev, uint32_t walker, uint32_t step,
                                            uint32_t trial, float T, float w_ret) {
  N2vTest t;
  t.uF = 0.0f;
  t.decided = true;
  t.accept = true;
  t.take_prev = false;
  if (prev == -1 || trial == kMaxTrials - 1u) return t;
  const uint4 bits = philox4x32_10(walker, step, kStreamAccept | (trial << 8), 0u, a.seed_lo, a.seed_hi);
  t.uF = u24(bits.x) * a.n2v_fmax;
  if (a.n2v_extra > 0.0f) {
    const float gx = a.n2v_extra * w_ret;
    const float gb = a.n2v_fmax * T;
    const float lhs0 = u24(bits.y) * (gb + gx);
    t.take_prev = lhs0 < gx;
    if (t.take_prev || post == prev) return t;
  } else if (post == prev) {
    t.accept = t.uF < a.inv_p;
    return t;
  }
  const float f_lo = a.inv_q < 1.0f ? a.inv_q : 1.0f;
  const float f_hi = a.inv_q < 1.0f ? 1.0f : a.inv_q;
  if (t.uF < f_lo) return t;            // accepted as a common neighbour and as any other
  t.accept = false;
  if (!(t.uF < f_hi)) return t;         // rejected as either
  t.decided = false;
  return t;
}

// the other half: `common` = the proposal is a neighbour of prev
__device__ __forceinline__ bool n2v_finish(const fw_kargs& a, const N2vTest& t, bool common) {
  return t.decided ? t.accept : t.uF < (common ? 1.0f : a.inv_q);
}

// Wave-uniform queue of Philox words: draw n of a stream is word n & 3 of block n >> 2.
struct DrawQueue {
  uint32_t q0 = 0, q1 = 0, q2 = 0, q3 = 0;
  uint32_t avail = 0;
  uint32_t blk = 0;
};

__device__ __forceinline__ float next_uniform(DrawQueue& d, const fw_kargs& a, const StepCtx& c, uint32_t stream) {
  if (d.avail == 0u) {
    const uint4 b = philox4x32_10(c.walker, c.step, stream | c.sbase, d.blk, a.seed_lo, a.seed_hi);
    d.q0 = b.x; d.q1 = b.y; d.q2 = b.z; d.q3 = b.w;
    d.avail = 4u;
    ++d.blk;
  }
  const float u = u24(d.q0);
  d.q0 = d.q1; d.q1 = d.q2; d.q2 = d.q3;
  --d.avail;
  return u;
}

// One wave streams the groups w, w + nw, ... of a neighbour list and keeps a reservoir over them.
// kJ = quartets per lane per group that can exist (kGroupQuartets, or 1 when the caller knows that the
// list has at most 64 quartets).  kTrackV: also load the adjacency quartet and return the selected
// vertex.  Outputs: running total S of the wave's groups, selected local index (or -1), its vertex.
template <int kApp, int kJ, bool kTrackV>
__device__ __forceinline__ void wave_stream(const fw_kargs& a, const StepCtx& c, const int lane, const uint32_t w,
                                            const uint32_t nw, const DrawQueue& dq0, float& S_out,
                                            int32_t& sel_out, int32_t& selv_out) {
  constexpr uint32_t kG = 64u * kGroupQuartets;  // quartets per group
  constexpr int kEl = 4 * kJ;
  const uint32_t a0 = c.off & ~3u;
  const uint32_t end = c.off + (uint32_t)c.deg;
  const uint32_t nq = (end - a0 + 3u) >> 2;
  const uint32_t ngroups = (nq + kG - 1u) / kG;
  const uint32_t* __restrict__ bias =
      reinterpret_cast<const uint32_t*>(kApp == FW_APP_METAPATH ? (const void*)a.label : (const void*)a.weight);
  constexpr bool need_adj = kTrackV;

  float S = 0.0f, Sj = 0.0f, u = 1.0f;
  int32_t sel = -1, selv = -1;
  DrawQueue dq = dq0;  // empty, or block 0 of this wave's stream computed ahead by the slot's own thread

  for (uint32_t g = w; g < ngroups; g += nw) {
    const uint32_t kb = g * kG + (uint32_t)lane;  // this lane's quartet for j = 0
    uint4 raw[kJ];
    int4 adj[kJ];
    float x[kEl];
    const bool interior = g > 0u && (g + 1u) * kG < nq;  // no head / tail quartet, every quartet exists
    if (interior) {
#pragma unroll
      for (int j = 0; j < kJ; ++j) {
        const uint32_t base = a0 + 4u * (kb + 64u * (uint32_t)j);
        raw[j] = *reinterpret_cast<const uint4*>(bias + base);
        adj[j] = make_int4(-1, -1, -1, -1);
        if (need_adj) adj[j] = *reinterpret_cast<const int4*>(a.adjncy + base);
      }
    } else {
#pragma unroll
      for (int j = 0; j < kJ; ++j) {
        const uint32_t k = kb + 64u * (uint32_t)j;
        const uint32_t base = a0 + 4u * k;
        raw[j] = make_uint4(0, 0, 0, 0);
        adj[j] = make_int4(-1, -1, -1, -1);
        if (k < nq) {
          raw[j] = *reinterpret_cast<const uint4*>(bias + base);
          if (need_adj) adj[j] = *reinterpret_cast<const int4*>(a.adjncy + base);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < kJ; ++j) {
      if (kApp == FW_APP_METAPATH) {  // include/app.cuh:141-146
        x[4 * j + 0] = (int32_t)raw[j].x == c.want ? 1.0f : 0.0f;
        x[4 * j + 1] = (int32_t)raw[j].y == c.want ? 1.0f : 0.0f;
        x[4 * j + 2] = (int32_t)raw[j].z == c.want ? 1.0f : 0.0f;
        x[4 * j + 3] = (int32_t)raw[j].w == c.want ? 1.0f : 0.0f;
      } else {
        x[4 * j + 0] = __uint_as_float(raw[j].x);
        x[4 * j + 1] = __uint_as_float(raw[j].y);
        x[4 * j + 2] = __uint_as_float(raw[j].z);
        x[4 * j + 3] = __uint_as_float(raw[j].w);
      }
    }
    if (!interior) {  // entries outside [off, end) (head / tail quartet, quartets past the list) have no bias
#pragma unroll
      for (int j = 0; j < kJ; ++j) {
        // local index of the quartet's first slot; it wraps below 0 for the head quartet, and quartets past
        // the list start at or beyond deg, so one unsigned compare per slot decides membership
        const uint32_t li = a0 + 4u * (kb + 64u * (uint32_t)j) - c.off;
        const bool in0 = li < (uint32_t)c.deg;
        const bool in1 = li + 1u < (uint32_t)c.deg;
        const bool in2 = li + 2u < (uint32_t)c.deg;
        const bool in3 = li + 3u < (uint32_t)c.deg;
        x[4 * j + 0] = in0 ? x[4 * j + 0] : 0.0f;
        x[4 * j + 1] = in1 ? x[4 * j + 1] : 0.0f;
        x[4 * j + 2] = in2 ? x[4 * j + 2] : 0.0f;
        x[4 * j + 3] = in3 ? x[4 * j + 3] : 0.0f;
      }
    }
    float q = 0.0f;
#pragma unroll
    for (int i = 0; i < kEl; ++i) q = q + x[i];
    const float I = wave_scan(q);
    const float T = readlane_f(I, 63);
    const float Snew = S + T;
    if (Snew * u > Sj) {  // wave-uniform: the reservoir accepts this group
      const float target = next_uniform(dq, a, c, w) * T;
      const bool pos = q > 0.0f;
      const uint64_t m = __ballot(pos && I > target);
      int l;
      if (m != 0ull) {
        l = __builtin_ctzll(m);
      } else {  // rounding in the scan tree left no crossing: last lane with a positive total
        l = 63 - __builtin_clzll(__ballot(pos));
      }
      // Every lane resolves its own elements; the answer of lane l is the one that is read.  The running sum
      // e never decreases (the biases are not negative), so "first positive element whose running sum exceeds
      // the target" is the first positive element at or after position #(sums <= target); none: last positive.
      float e = I - q;
      uint32_t cnt = 0u, pm = 0u;
#pragma unroll
      for (int i = 0; i < kEl; ++i) {
        e = e + x[i];
        cnt += e <= target ? 1u : 0u;
        pm |= (x[i] > 0.0f ? 1u : 0u) << i;
      }
      const uint32_t cand = pm >> cnt;
      const int pick = cand != 0u ? (int)cnt + __builtin_ctz(cand) : 31 - __builtin_clz(pm | 1u);
      const uint32_t abs_idx = a0 + 4u * kb + 256u * (uint32_t)(pick >> 2) + (uint32_t)(pick & 3);
      sel = __builtin_amdgcn_readlane((int32_t)(abs_idx - c.off), l);
      if (kTrackV) {
        int32_t v = adj[0].x;
#pragma unroll
        for (int j = 0; j < kJ; ++j) {
          v = (pick == 4 * j + 0) ? adj[j].x : v;
          v = (pick == 4 * j + 1) ? adj[j].y : v;
          v = (pick == 4 * j + 2) ? adj[j].z : v;
          v = (pick == 4 * j + 3) ? adj[j].w : v;
        }
        selv = __builtin_amdgcn_readlane(v, l);
      }
      Sj = Snew;
      u = next_uniform(dq, a, c, w);
    }
    S = Snew;
  }
  S_out = S;
  sel_out = sel;
  selv_out = selv;
}

// ---- LDS task table ----------------------------------------------------------------------------

template <int kWGT, int kApp>
struct TaskTable {
  // include/gpu_task.cuh:24-33, as structure of arrays; len < 0 marks an empty slot.
  int32_t walker[kWGT];
  int32_t cur[kWGT];
  int32_t prev[kWGT];
  uint32_t off[kWGT];
  int32_t deg[kWGT];
  int32_t len[kWGT];
  uint32_t prev_off[kWGT];
  int32_t prev_deg[kWGT];
  int32_t flag[kWGT];
  // Philox block 0 of stream 0 for the slot's next step, computed by the slot's own thread in phase C (64 blocks
  // per vector instruction instead of one block per scalar instruction stream)
  uint32_t draw[4][kWGT];
  // per-round work lists, double buffered by round parity.  Lists of at most 16 (32) quartets use one (two) 16-lane
  // rows of a wave, so four (two) of them are sampled by one wave at the same time; the others take a whole wave
  // (small) or the whole workgroup (hub).
  uint16_t tiny_list[2][kWGT];
  uint16_t half_list[2][kWGT];
  uint16_t small_list[2][kWGT];
  uint16_t hub_list[2][kWGT];
  int32_t tiny_count[2];
  int32_t half_count[2];
  int32_t small_count[2];
  int32_t hub_count[2];
  int32_t claim_tiny[2];
  int32_t claim_half[2];
  int32_t claim[2];
  int32_t exhausted;
  uint32_t cursor;            // resume lists: entries of this workgroup's share handed out so far
  uint32_t entry[kWGT];       // parking: the slot's walker came in as entry number ... of the launch's input
  uint32_t n_parked;          // walkers this workgroup has parked
  unsigned long long acc[2];  // steps, sum of source degrees of this workgroup
  // wave partials of the hub chunk in flight
  float hub_w[kHubChunk][16];
  int32_t hub_sel[kHubChunk][16];
  // node2vec only: trials of the slot's current step that were rejected so far
  int32_t trial[kApp == FW_APP_NODE2VEC ? kWGT : 1];
  // metapath only: the schema, so that the per-step label is an LDS read (a dynamic index into the
  // by-value kernel arguments would force a private copy of the whole array)
  int32_t schema[kApp == FW_APP_METAPATH ? FW_MAX_SCHEMA : 1];
  int32_t want[kApp == FW_APP_METAPATH ? kWGT : 1];  // the label the slot's next step looks for
};

// The slot index is wave-uniform; readfirstlane tells the compiler so (scalar registers, scalar Philox).
template <int kWGT, int kApp>
__device__ __forceinline__ StepCtx load_ctx(const fw_kargs& a, const TaskTable<kWGT, kApp>& tt, int slot) {
  StepCtx c;
  c.off = (uint32_t)__builtin_amdgcn_readfirstlane((int)tt.off[slot]);
  c.deg = __builtin_amdgcn_readfirstlane(tt.deg[slot]);
  c.prev = __builtin_amdgcn_readfirstlane(tt.prev[slot]);
  c.prev_off = (uint32_t)__builtin_amdgcn_readfirstlane((int)tt.prev_off[slot]);
  c.prev_deg = __builtin_amdgcn_readfirstlane(tt.prev_deg[slot]);
  c.walker = a.walker_base + (uint32_t)__builtin_amdgcn_readfirstlane(tt.walker[slot]);
  c.step = (uint32_t)(__builtin_amdgcn_readfirstlane(tt.len[slot]) - 1);
  c.want = 0;
  c.sbase = kApp == FW_APP_NODE2VEC ? (uint32_t)__builtin_amdgcn_readfirstlane(tt.trial[slot]) << 8 : 0u;
  return c;
}

// node2vec, all lanes of the wave: is the (wave-uniform) proposal v of the step accepted?  The lanes look it up in
// N(prev) together when the answer matters.
// T: the list's total as the step's sampler added it up.  v becomes the previous vertex when the trial takes the
// return edge's own component.
template <int kApp>
__device__ __forceinline__ bool n2v_wave_accept(const fw_kargs& a, const StepCtx& c, int32_t& v, bool ok, int lane,
                                                float T) {
  if (kApp != FW_APP_NODE2VEC || !ok) return true;
  float w_ret = 0.0f;
  if (a.n2v_extra > 0.0f && c.prev >= 0)  // wave-uniform: every lane walks the same few entries
    w_ret = return_weight(a.adjncy + c.off, a.weight + c.off, (uint32_t)c.deg, c.prev);
  const N2vTest t = n2v_test(a, v, c.prev, c.walker, c.step, c.sbase >> 8, T, w_ret);  // wave-uniform
  if (t.take_prev) {
    v = c.prev;
    return true;
  }
  bool common = false;
  if (!t.decided) common = wave_contains(a.adjncy + c.prev_off, (uint32_t)c.prev_deg, v, lane);
  return n2v_finish(a, t, common);
}

// Step commit by one lane: include/walker.cuh:1372-1385 and Task::update (include/gpu_task.cuh:70-77).
// The CSR range of the new vertex is reloaded in phase C by the slot's own thread.  node2vec: the wave has made
// the acceptance test of the proposal before (n2v_wave_accept).
template <int kWGT, int kApp>
__device__ __forceinline__ void commit(const fw_kargs& a, TaskTable<kWGT, kApp>& tt, int slot, const StepCtx& c, int32_t v,
                                       bool ok, bool accepted, unsigned long long& n_steps,
                                       unsigned long long& n_edges) {
  if (!ok) {
    tt.flag[slot] = kFlagDead;
    return;
  }
  if (kApp == FW_APP_NODE2VEC) {  // v is a proposal: accepted, or the slot samples again next round
    const uint32_t trial = c.sbase >> 8;
    if (!accepted) {
      tt.trial[slot] = (int32_t)trial + 1;
      tt.flag[slot] = kFlagRetry;
      return;
    }
    tt.trial[slot] = 0;
  }
  const int32_t len = (int32_t)c.step + 1;
  a.paths[(uint64_t)(uint32_t)tt.walker[slot] * (uint64_t)a.max_depth + (uint64_t)len] = v;
  tt.prev[slot] = tt.cur[slot];
  tt.prev_off[slot] = c.off;
  tt.prev_deg[slot] = c.deg;
  tt.cur[slot] = v;
  tt.len[slot] = len + 1;
  tt.flag[slot] = kFlagMoved;
  n_steps += 1ull;
  n_edges += (unsigned long long)(uint32_t)c.deg;
}

// One sampling step for 64 / kSeg task slots at once: slot s of the bundle owns the kSeg lanes starting at
// s * kSeg (kSeg = 16 or 32, lists of at most kSeg quartets, one quartet per lane).  The arithmetic is the wave
// sampler's: inside a 16-lane row the scan network is the same, row_bcast:15 joins the two rows of a 32-lane
// segment exactly as it joins rows 0 and 1 of a whole wave, and the steps of the whole-wave scan that are left out
// only ever add zeros for such a list, so every slot gets the element it would get from a wave of its own.
// `slot` is this lane's slot or -1.  Not for node2vec (its biases need the adjacency test).
// What a packed step keeps between its two halves: the loads are started for several bundles before the first one
// is finished, so that a wave waits for memory once per pair of bundles instead of once per bundle.
struct PackedBundle {
  int slot;
  uint32_t off, deg, d0;
  int32_t len, want;
  bool have;
  uint4 raw;
  int4 adj;
};

template <int kApp, int kSeg, int kWGT>
__device__ __forceinline__ void packed_load(const fw_kargs& a, TaskTable<kWGT, kApp>& tt, const int lane,
                                            const int slot, PackedBundle& b) {
  static_assert(kSeg == 16 || kSeg == 32, "a segment is one or two DPP rows");
  const bool active = slot >= 0;
  const int c = lane & (kSeg - 1);
  b.slot = slot;
  b.off = 0u; b.deg = 0u; b.d0 = 0u; b.len = 1; b.want = 0;
  if (active) {
    b.off = tt.off[slot];
    b.deg = (uint32_t)tt.deg[slot];
    b.len = tt.len[slot];
    b.d0 = tt.draw[0][slot];
    if (kApp == FW_APP_METAPATH) b.want = tt.want[slot];
  }
  const uint32_t a0 = b.off & ~3u;
  const uint32_t nq = (b.off + b.deg - a0 + 3u) >> 2;
  b.have = active && (uint32_t)c < nq;
  const uint32_t base = a0 + 4u * (uint32_t)c;
  const uint32_t* __restrict__ bias =
      reinterpret_cast<const uint32_t*>(kApp == FW_APP_METAPATH ? (const void*)a.label : (const void*)a.weight);
  b.raw = make_uint4(0, 0, 0, 0);
  b.adj = make_int4(-1, -1, -1, -1);
  if (b.have) {
    b.raw = *reinterpret_cast<const uint4*>(bias + base);
    b.adj = *reinterpret_cast<const int4*>(a.adjncy + base);
  }
}

template <int kApp, int kSeg, int kWGT>
__device__ __forceinline__ void packed_finish(const fw_kargs& a, TaskTable<kWGT, kApp>& tt, const int lane,
                                              const PackedBundle& b, unsigned long long& n_steps,
                                              unsigned long long& n_edges) {
  const int slot = b.slot;
  const bool active = slot >= 0;
  const int c = lane & (kSeg - 1);
  const int seg_first = lane & ~(kSeg - 1);
  const uint32_t off = b.off, deg = b.deg, d0 = b.d0;
  const int32_t len = b.len, want = b.want;
  const bool have = b.have;
  const uint4 raw = b.raw;
  const int4 adj = b.adj;
  const uint32_t a0 = off & ~3u;
  const uint32_t base = a0 + 4u * (uint32_t)c;
  float x[4];
  if (kApp == FW_APP_METAPATH) {  // include/app.cuh:141-146
    x[0] = (int32_t)raw.x == want ? 1.0f : 0.0f;
    x[1] = (int32_t)raw.y == want ? 1.0f : 0.0f;
    x[2] = (int32_t)raw.z == want ? 1.0f : 0.0f;
    x[3] = (int32_t)raw.w == want ? 1.0f : 0.0f;
  } else {
    x[0] = __uint_as_float(raw.x);
    x[1] = __uint_as_float(raw.y);
    x[2] = __uint_as_float(raw.z);
    x[3] = __uint_as_float(raw.w);
  }
  const uint32_t li = base - off;  // local index of the quartet's first slot (wraps below 0 for the head quartet)
  const uint32_t lim = have ? deg : 0u;
  x[0] = li < lim ? x[0] : 0.0f;
  x[1] = li + 1u < lim ? x[1] : 0.0f;
  x[2] = li + 2u < lim ? x[2] : 0.0f;
  x[3] = li + 3u < lim ? x[3] : 0.0f;
  float q = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i) q = q + x[i];
  float I = row_scan(q);
  if (kSeg == 32) I = dpp_add_bcast15(I);
  const float T = bperm_f((lane | (kSeg - 1)) << 2, I);  // the segment's total
  const bool accept = T > 0.0f;                          // first group of an empty reservoir: S * 1 > 0
  const float target = u24(d0) * T;
  const bool pos = q > 0.0f;
  const uint64_t mhit = __ballot(pos && I > target);
  const uint64_t mpos = __ballot(pos);
  const uint32_t seg_mask = kSeg == 32 ? 0xFFFFFFFFu : 0xFFFFu;
  const uint32_t hit = (uint32_t)(mhit >> seg_first) & seg_mask;
  const uint32_t any = (uint32_t)(mpos >> seg_first) & seg_mask;
  // first lane of the segment with a positive total whose prefix exceeds the target, else the last positive one
  const int l = hit != 0u ? __builtin_ctz(hit) : 31 - __builtin_clz(any | 1u);
  // every lane resolves its own four elements; the answer of lane l of the segment is the one that is read
  float e = I - q;
  uint32_t cnt = 0u, pm = 0u;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    e = e + x[i];
    cnt += e <= target ? 1u : 0u;
    pm |= (x[i] > 0.0f ? 1u : 0u) << i;
  }
  const uint32_t cand = pm >> cnt;
  const int pick = cand != 0u ? (int)cnt + __builtin_ctz(cand) : 31 - __builtin_clz(pm | 1u);
  int32_t v = adj.x;
  v = pick == 1 ? adj.y : v;
  v = pick == 2 ? adj.z : v;
  v = pick == 3 ? adj.w : v;
  int32_t selv = __builtin_amdgcn_ds_bpermute((seg_first + l) << 2, v);
  bool n2v_ok = true;
  if (kApp == FW_APP_NODE2VEC) {  // selv is a proposal: the acceptance test, its search made by the segment's lanes together
    N2vTest t;
    t.uF = 0.0f; t.decided = true; t.accept = true; t.take_prev = false;
    uint32_t psize = 0u;
    const int32_t* plist = a.adjncy;
    float w_ret = 0.0f;
    if (a.n2v_extra > 0.0f) {
      // The weights of the entries that lead back to the previous vertex, added in list order.  The entries are in
      // the lanes' registers (lane k of the segment holds quartet k); they follow each other in the list, so they sit
      // in one lane or in a few neighbouring ones, which are visited in order.
      const int32_t pv = active ? tt.prev[slot] : -1;
      uint32_t mine = 0u;  // which of this lane's four entries lead back
      mine |= (li < lim && adj.x == pv) ? 1u : 0u;
      mine |= (li + 1u < lim && adj.y == pv) ? 2u : 0u;
      mine |= (li + 2u < lim && adj.z == pv) ? 4u : 0u;
      mine |= (li + 3u < lim && adj.w == pv) ? 8u : 0u;
      uint32_t rest = (uint32_t)(__ballot(mine != 0u) >> seg_first) & seg_mask;
      while (__ballot(rest != 0u) != 0ull) {
        const int from = (seg_first + (rest != 0u ? __builtin_ctz(rest) : 0)) << 2;
        const uint32_t their = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)mine);
        const float y0 = bperm_f(from, x[0]), y1 = bperm_f(from, x[1]);
        const float y2 = bperm_f(from, x[2]), y3 = bperm_f(from, x[3]);
        if (rest != 0u) {
          if (their & 1u) w_ret = w_ret + y0;
          if (their & 2u) w_ret = w_ret + y1;
          if (their & 4u) w_ret = w_ret + y2;
          if (their & 8u) w_ret = w_ret + y3;
          rest &= rest - 1u;
        }
      }
    }
    if (active && accept) {
      t = n2v_test(a, selv, tt.prev[slot], a.walker_base + (uint32_t)tt.walker[slot], (uint32_t)(len - 1),
                   (uint32_t)tt.trial[slot], T, w_ret);  // the same in every lane of the segment
      if (t.take_prev) selv = tt.prev[slot];
      if (!t.decided) {
        plist = a.adjncy + tt.prev_off[slot];
        psize = (uint32_t)tt.prev_deg[slot];
      }
    }
    const bool common = segment_contains<kSeg>(plist, psize, selv, lane);
    n2v_ok = n2v_finish(a, t, common);
  }
  if (active && c == 0) {  // commit (include/walker.cuh:1372-1385, Task::update include/gpu_task.cuh:70-77)
    bool rejected = false;
    if (kApp == FW_APP_NODE2VEC && accept) {  // accept the proposal or sample again next round
      const uint32_t trial = (uint32_t)tt.trial[slot];
      rejected = !n2v_ok;
      tt.trial[slot] = rejected ? (int32_t)trial + 1 : 0;
    }
    if (!accept) {
      tt.flag[slot] = kFlagDead;
    } else if (rejected) {
      tt.flag[slot] = kFlagRetry;
    } else {
      a.paths[(uint64_t)(uint32_t)tt.walker[slot] * (uint64_t)a.max_depth + (uint64_t)len] = selv;
      tt.prev[slot] = tt.cur[slot];
      if (kApp == FW_APP_NODE2VEC) {
        tt.prev_off[slot] = off;
        tt.prev_deg[slot] = (int32_t)deg;
      }
      tt.cur[slot] = selv;
      tt.len[slot] = len + 1;
      tt.flag[slot] = kFlagMoved;
      n_steps += 1ull;
      n_edges += (unsigned long long)deg;
    }
  }
}

template <int kApp, int kSeg, int kWGT>
__device__ __forceinline__ void packed_step(const fw_kargs& a, TaskTable<kWGT, kApp>& tt, const int lane,
                                            const int slot, unsigned long long& n_steps,
                                            unsigned long long& n_edges) {
  PackedBundle b;
  packed_load<kApp, kSeg, kWGT>(a, tt, lane, slot, b);
  packed_finish<kApp, kSeg, kWGT>(a, tt, lane, b, n_steps, n_edges);
}

// ---- the kernel --------------------------------------------------------------------------------

// kPackedInFlight: bundles of short lists a wave loads per turn.  1 for launches whose walkers run whole walks (80
// VGPRs, three workgroups of 512 per CU: such launches live on streaming long lists and want every wave they can
// get); kPipelineInFlight for the launches of the parking pipeline, which are rounds of refills and packed steps
// on short lists and wait for one bundle's loads after the other otherwise (110 VGPRs, two workgroups per CU).
template <int kApp, int kWGT, int kPackedInFlight>
__global__ __launch_bounds__(kWGT, kPackedInFlight == 1 ? 8 : 4) void fw_walk_zprs(
    const fw_kargs a) {
  constexpr int kNW = kWGT / 64;
  __shared__ TaskTable<kWGT, kApp> tt;

  const int tid = (int)threadIdx.x;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  unsigned long long n_steps = 0ull, n_edges = 0ull;
  uint32_t my_parked = 0u;  // walkers parked, counted by the leading lanes of the parking waves
  // entries of this launch and the slots a workgroup fills: from the host, or (a launch queued before its input's
  // size was known to the host) from the device, with the same rule: small inputs are spread over the grid
  uint32_t n_entries = (uint32_t)a.n;
  int32_t slot_limit = a.slot_limit;
  if (a.n_dev != nullptr) {
    n_entries = *a.n_dev;
    const uint32_t per_wg = (n_entries + gridDim.x - 1u) / gridDim.x;
    slot_limit = (int32_t)(per_wg < (uint32_t)kWGT ? (per_wg > 0u ? per_wg : 1u) : (uint32_t)kWGT);
  }

  tt.len[tid] = -1;
  tt.flag[tid] = 0;
  if (kApp == FW_APP_NODE2VEC) tt.trial[tid] = 0;
  if (kApp == FW_APP_METAPATH && tid == 0) {
#pragma unroll
    for (int i = 0; i < FW_MAX_SCHEMA; ++i) tt.schema[i] = a.schema[i];
  }
  if (tid == 0) {
    tt.tiny_count[0] = tt.tiny_count[1] = 0;
    tt.half_count[0] = tt.half_count[1] = 0;
    tt.small_count[0] = tt.small_count[1] = 0;
    tt.hub_count[0] = tt.hub_count[1] = 0;
    tt.claim_tiny[0] = tt.claim_tiny[1] = 0;
    tt.claim_half[0] = tt.claim_half[1] = 0;
    tt.claim[0] = tt.claim[1] = 0;
    tt.exhausted = 0;
    tt.cursor = 0u;
    tt.n_parked = 0u;
    tt.acc[0] = tt.acc[1] = 0ull;
  }
  __syncthreads();

  int parity = 0;  // lists[parity] are consumed this round, lists[parity ^ 1] are produced by phase C
  bool first = true;
  for (;;) {
    if (!first) {
      const int nh = tt.hub_count[parity];
      const int ns = tt.small_count[parity];
      const int nt = tt.tiny_count[parity];
      const int nf = tt.half_count[parity];
      if (nh + ns + nt + nf == 0) break;  // uniform: read after the barrier that closed phase C

      // ---- phase B: hubs, whole workgroup ----
      for (int hb = 0; hb < nh; hb += kHubChunk) {
        const int cnt = min(kHubChunk, nh - hb);
        for (int h = 0; h < cnt; ++h) {
          const int slot = tt.hub_list[parity][hb + h];
          StepCtx c = load_ctx(a, tt, slot);
          if (kApp == FW_APP_METAPATH) c.want = tt.schema[c.step % (uint32_t)a.schema_len];
          float W;
          int32_t sel, selv;
          wave_stream<kApp, kGroupQuartets, false>(a, c, lane, (uint32_t)wave, (uint32_t)kNW, DrawQueue(), W, sel,
                                                   selv);
          if (lane == 0) {
            tt.hub_w[h][wave] = W;
            tt.hub_sel[h][wave] = sel;
          }
        }
        __syncthreads();
        for (int h = wave; h < cnt; h += kNW) {
          const int slot = tt.hub_list[parity][hb + h];
          const StepCtx c = load_ctx(a, tt, slot);
          float W = 0.0f;
          int32_t s = -1;
          if (lane < kNW) {
            W = tt.hub_w[h][lane];
            s = tt.hub_sel[h][lane];
          }
          // inverse transform over the wave totals (lanes >= kNW hold 0 and never qualify)
          const float J = row_scan(W);
          const float total = readlane_f(J, kNW - 1);
          const uint32_t bits = philox4x32_10(c.walker, c.step, kStreamWave | c.sbase, 0u, a.seed_lo, a.seed_hi).x;
          const float target = u24(bits) * total;
          const bool pos = W > 0.0f;
          uint64_t m = __ballot(pos && J > target);
          int32_t pick = -1;
          if (m != 0ull) {
            pick = __builtin_amdgcn_readlane(s, __builtin_ctzll(m));
          } else {
            m = __ballot(pos);
            if (m != 0ull) pick = __builtin_amdgcn_readlane(s, 63 - __builtin_clzll(m));
          }
          int32_t v = -1;
          if (pick >= 0) v = a.adjncy[c.off + (uint32_t)pick];  // wave-uniform
          const bool accepted = n2v_wave_accept<kApp>(a, c, v, pick >= 0, lane, total);
          if (lane == 0) commit(a, tt, slot, c, v, pick >= 0, accepted, n_steps, n_edges);
        }
        if (hb + kHubChunk < nh) __syncthreads();  // the partial buffers are reused by the next chunk
      }

      // ---- phase A: remaining slots, claimed dynamically: four or two short lists per wave, else one ----
      {
        // kPackedInFlight bundles per turn: their loads are in flight together, so a wave waits for memory once per
        // turn instead of once per bundle (the registers are there: two workgroups per CU fit with up to 128)
        for (;;) {
          int idx = 0;
          if (lane == 0) idx = atomicAdd(&tt.claim_tiny[parity], 4 * kPackedInFlight);
          idx = __builtin_amdgcn_readfirstlane(idx);
          if (idx >= nt) break;
          PackedBundle b[kPackedInFlight];
#pragma unroll
          for (int k = 0; k < kPackedInFlight; ++k) {
            const int e = idx + 4 * k + (lane >> 4);
            packed_load<kApp, 16, kWGT>(a, tt, lane, e < nt ? (int)tt.tiny_list[parity][e] : -1, b[k]);
          }
#pragma unroll
          for (int k = 0; k < kPackedInFlight; ++k)
            if (idx + 4 * k < nt) packed_finish<kApp, 16, kWGT>(a, tt, lane, b[k], n_steps, n_edges);
        }
        for (;;) {
          int idx = 0;
          if (lane == 0) idx = atomicAdd(&tt.claim_half[parity], 2 * kPackedInFlight);
          idx = __builtin_amdgcn_readfirstlane(idx);
          if (idx >= nf) break;
          PackedBundle b[kPackedInFlight];
#pragma unroll
          for (int k = 0; k < kPackedInFlight; ++k) {
            const int e = idx + 2 * k + (lane >> 5);
            packed_load<kApp, 32, kWGT>(a, tt, lane, e < nf ? (int)tt.half_list[parity][e] : -1, b[k]);
          }
#pragma unroll
          for (int k = 0; k < kPackedInFlight; ++k)
            if (idx + 2 * k < nf) packed_finish<kApp, 32, kWGT>(a, tt, lane, b[k], n_steps, n_edges);
        }
      }
      for (;;) {
        int idx = 0;
        if (lane == 0) idx = atomicAdd(&tt.claim[parity], 1);
        idx = __builtin_amdgcn_readfirstlane(idx);
        if (idx >= ns) break;
        const int slot = tt.small_list[parity][idx];
        StepCtx c = load_ctx(a, tt, slot);
        if (kApp == FW_APP_METAPATH) c.want = tt.schema[c.step % (uint32_t)a.schema_len];
        float W;
        int32_t sel, selv;
        const uint32_t nq = ((c.off + (uint32_t)c.deg) - (c.off & ~3u) + 3u) >> 2;
        int32_t v = -1;
        DrawQueue dq0;
        dq0.q0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)tt.draw[0][slot]);
        dq0.q1 = (uint32_t)__builtin_amdgcn_readfirstlane((int)tt.draw[1][slot]);
        dq0.q2 = (uint32_t)__builtin_amdgcn_readfirstlane((int)tt.draw[2][slot]);
        dq0.q3 = (uint32_t)__builtin_amdgcn_readfirstlane((int)tt.draw[3][slot]);
        dq0.avail = 4u;
        dq0.blk = 1u;
        if (nq <= 64u) {  // one quartet per lane: fetch the adjacency with the biases, no dependent load
          wave_stream<kApp, 1, true>(a, c, lane, 0u, 1u, dq0, W, sel, selv);
          v = selv;
        } else {
          wave_stream<kApp, kGroupQuartets, false>(a, c, lane, 0u, 1u, dq0, W, sel, selv);
          if (sel >= 0) v = a.adjncy[c.off + (uint32_t)sel];
        }
        const bool accepted = n2v_wave_accept<kApp>(a, c, v, sel >= 0, lane, W);
        if (lane == 0) commit(a, tt, slot, c, v, sel >= 0, accepted, n_steps, n_edges);
      }
      __syncthreads();
      if (tid == 0) {  // this round's lists are drained; they become the lists produced two rounds later
        tt.tiny_count[parity] = 0;
        tt.half_count[parity] = 0;
        tt.small_count[parity] = 0;
        tt.hub_count[parity] = 0;
        tt.claim_tiny[parity] = 0;
        tt.claim_half[parity] = 0;
        tt.claim[parity] = 0;
      }
      parity ^= 1;
    }

    // ---- phase C: one thread per slot (include/walker.cuh:1421-1432; Task::init/update) ----
    {
      const int np = first ? 0 : parity;  // lists to fill for the next round
      first = false;
      int32_t len = tt.len[tid];
      bool need = tid < slot_limit;  // slot wants a new walker
      bool park = false;               // the slot's walker has reached a hub that is served by the batch kernel
      int32_t hidx = -1;               // that vertex's index among the parked-on ones (read together with its CSR range)
      const bool parking = a.park_threshold != 0x7FFFFFFF;
      const bool by_position = parking || a.resume != nullptr;
      int32_t deg = 0;
      if (len >= 0) {
        if (tt.flag[tid] == kFlagMoved) {
          const int32_t v = tt.cur[tid];
          const uint32_t o = a.xadj[v];
          const uint32_t e = a.xadj[v + 1];
          if (parking) hidx = a.hub_index[v];
          deg = (int32_t)(e - o);
          tt.off[tid] = o;
          tt.deg[tid] = deg;
          bool stop = len >= a.max_depth || deg == 0;
          if (kApp == FW_APP_PPR && !stop) {  // include/app.cuh:88-94: one draw per completed step
            const uint32_t w = a.walker_base + (uint32_t)tt.walker[tid];
            const uint32_t bits = philox4x32_10(w, (uint32_t)(len - 2), kStreamStop, 0u, a.seed_lo, a.seed_hi).x;
            stop = u24(bits) < a.tp;
          }
          need = stop;
          park = !stop && hidx >= 0;  // same as deg > park_threshold
        } else if (kApp == FW_APP_NODE2VEC && tt.flag[tid] == kFlagRetry) {
          need = false;  // the proposal was rejected: the walker stays and samples again (tt.trial counts)
          deg = tt.deg[tid];
        }
        // kFlagDead: dead end (no neighbour with positive bias), include/walker.cuh:1373-1374
      }
      bool exhausted = tt.exhausted != 0;
      for (;;) {
        // park first: the record leaves the slot, which then asks for the next walker
        const uint64_t pm = __ballot(park);
        if (pm != 0ull) {
          // The record goes to the position of the walker's entry in the launch's input (every entry is parked at most
          // once), not to the end of a list: appending would take an update of one list counter per wave and round, and
          // updates of one address complete one after the other -- with some 2,800 waves per launch that chain was as
          // long as the rounds themselves.  The positions of walkers that are not parked hold holes (q = -1, written
          // when the entry is taken).
          if (lane == __builtin_ctzll(pm)) my_parked += (uint32_t)__builtin_popcountll(pm);
          const uint32_t label_slot =
              kApp == FW_APP_METAPATH ? (uint32_t)(len - 1) % (uint32_t)a.n_labels_per_hub : 0u;
          const uint32_t bucket = (uint32_t)hidx * (uint32_t)a.n_labels_per_hub + label_slot;
          // counted only: the wave does not wait for a position inside the bucket (the counters of the busiest
          // vertices are contended); the counting sort hands the positions out later
          fw_wave_count_keys<false>(a.bucket_count, bucket, park);
          if (park) {
            const uint32_t at = tt.entry[tid];
            fw_walker_rec rec;
            rec.q = tt.walker[tid];
            rec.cur = (int32_t)bucket;  // the vertex follows from the bucket
            rec.prev = tt.prev[tid];
            rec.len = len;
            a.parked[at] = rec;
            park = false;
            need = true;
            len = -1;
          }
        }
        const bool want = need && !exhausted;
        const uint64_t m = __ballot(want);
        if (m == 0ull) break;
        uint32_t base = 0;
        const int leader = __builtin_ctzll(m);
        if (lane == leader) {
          // Without parking a walker stays in its slot for its whole walk, and queries come from the global
          // dispenser (include/walker.cuh:1339,1423) so that the workgroups balance.  With parking every launch
          // is short and there are many: the entries (fresh queries or a resume list) are dealt out by position
          // -- the workgroups take interleaved chunks of slot_limit entries -- with a workgroup-local cursor,
          // because a global counter is contended (about 13 ns per update).
          base = by_position ? atomicAdd(&tt.cursor, (uint32_t)__builtin_popcountll(m))
                             : atomicAdd(a.dispenser, (uint32_t)__builtin_popcountll(m));
        }
        base = (uint32_t)__builtin_amdgcn_readlane((int)base, leader);
        if (want) {
          uint32_t q = base + (uint32_t)__builtin_popcountll(m & ((1ull << lane) - 1ull));
          if (by_position) {
            const uint32_t chunk = q / (uint32_t)slot_limit;
            const uint64_t pos = ((uint64_t)chunk * gridDim.x + blockIdx.x) * (uint64_t)slot_limit +
                                 (q - chunk * (uint32_t)slot_limit);
            q = pos < (uint64_t)n_entries ? (uint32_t)pos : 0xFFFFFFFFu;
          }
          if (q < n_entries) {
            if (parking) {  // the entry's place in the list of parked walkers: a hole until its walker is parked
              a.parked[q].q = -1;
              tt.entry[tid] = q;
            }
            int32_t wq, sp, pv, ln, tr = 0;
            if (a.resume != nullptr) {  // a walker coming back from its batch step
              const fw_walker_rec rec = a.resume[q];
              wq = rec.q; sp = rec.cur; pv = rec.prev; ln = rec.len;
              // the list has holes: walks that ended, and walkers that wait on their next vertex already
              if (rec.q < 0 || (rec.len & FW_REC_PARK) != 0) sp = -1;
              if (kApp == FW_APP_NODE2VEC) {  // the rejected trials of the walker's current step travel with its length
                tr = (ln >> FW_REC_TRIAL_SHIFT) & FW_REC_TRIAL_MASK;
                ln &= FW_REC_LEN_MASK;
              }
            } else {                    // a fresh query (include/walker.cuh:1340-1343)
              wq = (int32_t)q; sp = a.starts[q]; pv = -1; ln = 1;
              a.paths[(uint64_t)q * (uint64_t)a.max_depth] = sp;
            }
            if ((uint32_t)sp < (uint32_t)a.V && ln < a.max_depth) {
              const uint32_t o = a.xadj[sp];
              const uint32_t e = a.xadj[sp + 1];
              // (a walker that resumes stands on a vertex nobody is parked on: the batch kernel looked it up)
              hidx = parking && a.resume == nullptr ? a.hub_index[sp] : -1;
              deg = (int32_t)(e - o);
              if (deg > 0) {
                tt.walker[tid] = wq;
                tt.cur[tid] = sp;
                tt.prev[tid] = pv;
                tt.off[tid] = o;
                tt.deg[tid] = deg;
                tt.prev_off[tid] = 0;
                tt.prev_deg[tid] = 0;
                if (kApp == FW_APP_NODE2VEC) {
                  tt.trial[tid] = tr;
                  if (pv >= 0) {  // the acceptance test searches N(prev)
                    const uint32_t po = a.xadj[pv];
                    tt.prev_off[tid] = po;
                    tt.prev_deg[tid] = (int32_t)(a.xadj[pv + 1] - po);
                  }
                }
                len = ln;
                need = false;
                park = hidx >= 0;  // same as deg > park_threshold
              }
            }
          } else {
            exhausted = true;
            tt.exhausted = 1;
          }
        }
      }
      if (need || len < 0) {  // nothing to run in this slot (finished / parked / never filled / beyond slot_limit)
        tt.len[tid] = -1;
      } else {
        tt.len[tid] = len;
        tt.flag[tid] = 0;
        if (deg > a.hub_threshold) {
          tt.hub_list[np][atomicAdd(&tt.hub_count[np], 1)] = (uint16_t)tid;
        } else {
          const uint32_t o = tt.off[tid];
          const uint32_t nq = (o + (uint32_t)deg - (o & ~3u) + 3u) >> 2;
          if (nq <= 16u) {
            tt.tiny_list[np][atomicAdd(&tt.tiny_count[np], 1)] = (uint16_t)tid;
          } else if (nq <= 32u) {
            tt.half_list[np][atomicAdd(&tt.half_count[np], 1)] = (uint16_t)tid;
          } else {
            tt.small_list[np][atomicAdd(&tt.small_count[np], 1)] = (uint16_t)tid;
          }
          if (kApp == FW_APP_METAPATH) tt.want[tid] = tt.schema[(uint32_t)(len - 1) % (uint32_t)a.schema_len];
          const uint32_t sbase = kApp == FW_APP_NODE2VEC ? (uint32_t)tt.trial[tid] << 8 : 0u;
          const uint4 b = philox4x32_10(a.walker_base + (uint32_t)tt.walker[tid], (uint32_t)(len - 1), sbase, 0u,
                                        a.seed_lo, a.seed_hi);
          tt.draw[0][tid] = b.x;
          tt.draw[1][tid] = b.y;
          tt.draw[2][tid] = b.z;
          tt.draw[3][tid] = b.w;
        }
      }
      parity = np;
    }
    __syncthreads();
  }

  // workload counters: summed inside the workgroup first, the global counters are contended
  if (n_steps != 0ull) {
    atomicAdd(&tt.acc[0], n_steps);
    atomicAdd(&tt.acc[1], n_edges);
  }
  if (my_parked != 0u) atomicAdd(&tt.n_parked, my_parked);
  __syncthreads();
  if (tid == 0 && tt.acc[0] != 0ull) {
    atomicAdd(&a.counters[0], tt.acc[0]);
    atomicAdd(&a.counters[1], tt.acc[1]);
  }
  if (tid == 0 && tt.n_parked != 0u) atomicAdd(a.parked_count, tt.n_parked);
}

// ---- hub batch kernel -----------------------------------------------------------------------------
//
// Many walkers stand on the same high-degree vertex at the same time (visits are proportional to degree), and
// for DeepWalk / PPR / MetaPath the biases of a list do not depend on the walker.  One workgroup therefore
// serves up to 64 parked walkers of one hub with ONE pass over its list: lane i of every wave carries walker
// i's reservoir (Sj, u, selection, its own Philox stream), while the group loads, the 16 adds, the DPP scan and
// the running total S are shared by all 64.  The sampling definition is the workgroup sampler's, unchanged:
// wave w owns groups w, w + NW, ..., the wave totals are combined by inverse transform, every draw is
// addressed by (walker, step, stream, index).  Each walker gets exactly the vertex it would have got alone.

// per-lane Philox word queue (same addressing as DrawQueue, different walker in every lane)
struct LaneDraw {
  uint32_t q0 = 0, q1 = 0, q2 = 0, q3 = 0;
  uint32_t avail = 0;
  uint32_t blk = 0;
};

__device__ __forceinline__ float next_uniform_lane(LaneDraw& d, const fw_kargs& a, uint32_t walker, uint32_t step,
                                                   uint32_t stream) {
  if (d.avail == 0u) {
    const uint4 b = philox4x32_10(walker, step, stream, d.blk, a.seed_lo, a.seed_hi);
    d.q0 = b.x; d.q1 = b.y; d.q2 = b.z; d.q3 = b.w;
    d.avail = 4u;
    ++d.blk;
  }
  const float u = u24(d.q0);
  d.q0 = d.q1; d.q1 = d.q2; d.q2 = d.q3;
  --d.avail;
  return u;
}

// The groups w, w + nw, ... of one list for up to 64 walkers at once (lane i = walker i).  Outputs the total S
// of those groups (the same in every lane) and each walker's selected local index (or -1).
template <int kApp>
__device__ __forceinline__ void batch_stream(const fw_kargs& a, const uint32_t* __restrict__ bias, const uint32_t off,
                                             const uint32_t deg, const int32_t want, const uint32_t w,
                                             const uint32_t nw, const bool have, const uint32_t walker,
                                             const uint32_t step, const uint32_t sbase, const int lane, float& S_out,
                                             int32_t& sel_out) {
  constexpr uint32_t kG = 64u * kGroupQuartets;
  constexpr int kEl = 4 * kGroupQuartets;
  const uint32_t a0 = off & ~3u;
  const uint32_t nq = (off + deg - a0 + 3u) >> 2;
  const uint32_t ngroups = (nq + kG - 1u) / kG;

  float S = 0.0f;             // shared: running total of this wave's groups
  float Sj = 0.0f, u = 1.0f;  // per walker
  int32_t sel = -1;
  LaneDraw dq;

  for (uint32_t g = w; g < ngroups; g += nw) {
    const uint32_t kb = g * kG + (uint32_t)lane;
    const bool interior = g > 0u && (g + 1u) * kG < nq;
    uint4 raw[kGroupQuartets];
    float x[kEl];
    if (interior) {
#pragma unroll
      for (int j = 0; j < kGroupQuartets; ++j)
        raw[j] = *reinterpret_cast<const uint4*>(bias + a0 + 4u * (kb + 64u * (uint32_t)j));
    } else {
#pragma unroll
      for (int j = 0; j < kGroupQuartets; ++j) {
        const uint32_t k = kb + 64u * (uint32_t)j;
        raw[j] = make_uint4(0, 0, 0, 0);
        if (k < nq) raw[j] = *reinterpret_cast<const uint4*>(bias + a0 + 4u * k);
      }
    }
#pragma unroll
    for (int j = 0; j < kGroupQuartets; ++j) {
      if (kApp == FW_APP_METAPATH) {
        x[4 * j + 0] = (int32_t)raw[j].x == want ? 1.0f : 0.0f;
        x[4 * j + 1] = (int32_t)raw[j].y == want ? 1.0f : 0.0f;
        x[4 * j + 2] = (int32_t)raw[j].z == want ? 1.0f : 0.0f;
        x[4 * j + 3] = (int32_t)raw[j].w == want ? 1.0f : 0.0f;
      } else {
        x[4 * j + 0] = __uint_as_float(raw[j].x);
        x[4 * j + 1] = __uint_as_float(raw[j].y);
        x[4 * j + 2] = __uint_as_float(raw[j].z);
        x[4 * j + 3] = __uint_as_float(raw[j].w);
      }
    }
    if (!interior) {
#pragma unroll
      for (int j = 0; j < kGroupQuartets; ++j) {
        const uint32_t li = a0 + 4u * (kb + 64u * (uint32_t)j) - off;  // wraps below 0 for the head quartet
        x[4 * j + 0] = li < deg ? x[4 * j + 0] : 0.0f;
        x[4 * j + 1] = li + 1u < deg ? x[4 * j + 1] : 0.0f;
        x[4 * j + 2] = li + 2u < deg ? x[4 * j + 2] : 0.0f;
        x[4 * j + 3] = li + 3u < deg ? x[4 * j + 3] : 0.0f;
      }
    }
    float q = 0.0f;
#pragma unroll
    for (int i = 0; i < kEl; ++i) q = q + x[i];
    const float I = wave_scan(q);
    const float T = readlane_f(I, 63);
    const float Snew = S + T;

    const bool acc = have && (Snew * u > Sj);  // per walker: this group enters its reservoir
    const uint64_t macc = __ballot(acc);
    if (macc != 0ull) {
      float target = 0.0f;
      if (acc) target = next_uniform_lane(dq, a, walker, step, w | sbase) * T;
      // which lane's biases hold the target of walker k: first lane with a positive total whose prefix
      // exceeds it, else the last lane with a positive total
      const bool pos = q > 0.0f;
      const uint64_t mpos = __ballot(pos);
      // M = running maximum of the positive lanes' prefixes.  It never decreases, and the first lane where it
      // exceeds a target is the first positive lane whose own prefix does (a lane without positive total adds 0,
      // which exceeds no target), so every walker finds its lane with a binary search across the lanes.
      const float M = wave_prefix_max(pos ? I : 0.0f);
      int src = 0;
#pragma unroll
      for (int s = 32; s >= 1; s >>= 1) {
        const float Mp = bperm_f((src + s - 1) << 2, M);
        src = Mp > target ? src : src + s;
      }
      if (!(bperm_f(src << 2, M) > target)) src = 63 - __builtin_clzll(mpos | 1ull);  // no crossing: last positive lane
      // Every walker resolves its own target on the 16 biases of its source lane (fetched across lanes, all
      // fetches in flight together).  The running sum never decreases, so the element is the first positive one
      // at or after position #(sums <= target); none: the last positive one.
      const int addr = src << 2;
      float xs[kEl];
      float e = bperm_f(addr, I - q);
#pragma unroll
      for (int i = 0; i < kEl; ++i) xs[i] = bperm_f(addr, x[i]);
      uint32_t cnt = 0u, pm = 0u;
#pragma unroll
      for (int i = 0; i < kEl; ++i) {
        e = e + xs[i];
        cnt += e <= target ? 1u : 0u;
        pm |= (xs[i] > 0.0f ? 1u : 0u) << i;
      }
      const uint32_t cand = pm >> cnt;
      const int pick = cand != 0u ? (int)cnt + __builtin_ctz(cand) : 31 - __builtin_clz(pm | 1u);
      if (acc) {
        const uint32_t abs_idx = a0 + 4u * (g * kG + (uint32_t)src) + 256u * (uint32_t)(pick >> 2) + (uint32_t)(pick & 3);
        sel = (int32_t)(abs_idx - off);
        Sj = Snew;
        u = next_uniform_lane(dq, a, walker, step, w | sbase);
      }
    }
    S = Snew;
  }
  S_out = S;
  sel_out = sel;
}

// ---- Two-pass steps for crowded hubs ----------------------------------------------------------------------------------
// A hub with many parked walkers is scanned once per 64 of them by the batches above.  Nothing in a group's part
// of the sampler depends on the walker except two uniforms, so the walker-independent part can be made once per
// hub and round: for every group its total T, the running maximum M of its positive lanes' prefixes, every
// lane's prefix before its own 16 biases (E), and its last positive lane.  A walker then runs its reservoir over
// the totals alone (same additions, same tests, same draws in the same order) and resolves its final target
// inside one group from M, E and the 16 biases of one lane.  Same vertex as from the full stream, bit for bit.

// The 16 biases of this lane in group g of a list (elements outside the list read as 0).
template <int kApp>
__device__ __forceinline__ void group_load(const uint32_t* __restrict__ bias, const uint32_t off, const uint32_t deg,
                                           const int32_t want, const uint32_t g, const int lane, float* x) {
  constexpr uint32_t kG = 64u * kGroupQuartets;
  const uint32_t a0 = off & ~3u;
  const uint32_t nq = (off + deg - a0 + 3u) >> 2;
  const uint32_t kb = g * kG + (uint32_t)lane;
  const bool interior = g > 0u && (g + 1u) * kG < nq;
  uint4 raw[kGroupQuartets];
  if (interior) {
#pragma unroll
    for (int j = 0; j < kGroupQuartets; ++j)
      raw[j] = *reinterpret_cast<const uint4*>(bias + a0 + 4u * (kb + 64u * (uint32_t)j));
  } else {
#pragma unroll
    for (int j = 0; j < kGroupQuartets; ++j) {
      const uint32_t k = kb + 64u * (uint32_t)j;
      raw[j] = make_uint4(0, 0, 0, 0);
      if (k < nq) raw[j] = *reinterpret_cast<const uint4*>(bias + a0 + 4u * k);
    }
  }
#pragma unroll
  for (int j = 0; j < kGroupQuartets; ++j) {
    if (kApp == FW_APP_METAPATH) {
      x[4 * j + 0] = (int32_t)raw[j].x == want ? 1.0f : 0.0f;
      x[4 * j + 1] = (int32_t)raw[j].y == want ? 1.0f : 0.0f;
      x[4 * j + 2] = (int32_t)raw[j].z == want ? 1.0f : 0.0f;
      x[4 * j + 3] = (int32_t)raw[j].w == want ? 1.0f : 0.0f;
    } else {
      x[4 * j + 0] = __uint_as_float(raw[j].x);
      x[4 * j + 1] = __uint_as_float(raw[j].y);
      x[4 * j + 2] = __uint_as_float(raw[j].z);
      x[4 * j + 3] = __uint_as_float(raw[j].w);
    }
  }
  if (!interior) {
#pragma unroll
    for (int j = 0; j < kGroupQuartets; ++j) {
      const uint32_t li = a0 + 4u * (kb + 64u * (uint32_t)j) - off;  // wraps below 0 for the head quartet
      x[4 * j + 0] = li < deg ? x[4 * j + 0] : 0.0f;
      x[4 * j + 1] = li + 1u < deg ? x[4 * j + 1] : 0.0f;
      x[4 * j + 2] = li + 2u < deg ? x[4 * j + 2] : 0.0f;
      x[4 * j + 3] = li + 3u < deg ? x[4 * j + 3] : 0.0f;
    }
  }
}

// First pass, one wave, one group: rows[0..63] = M, rows[64..127] = E, *total = T, *lastpos = last positive lane.
template <int kApp>
__device__ __forceinline__ void group_rows(const uint32_t* __restrict__ bias, const uint32_t off, const uint32_t deg,
                                           const int32_t want, const uint32_t g, const int lane, float* rows,
                                           float* total, int32_t* lastpos) {
  constexpr int kEl = 4 * kGroupQuartets;
  float x[kEl];
  group_load<kApp>(bias, off, deg, want, g, lane, x);
  float q = 0.0f;
#pragma unroll
  for (int i = 0; i < kEl; ++i) q = q + x[i];
  const float I = wave_scan(q);
  const float T = readlane_f(I, 63);
  const bool pos = q > 0.0f;
  const uint64_t mpos = __ballot(pos);
  const float M = wave_prefix_max(pos ? I : 0.0f);
  rows[lane] = M;
  rows[64 + lane] = I - q;
  if (lane == 0) {
    *total = T;
    *lastpos = 63 - __builtin_clzll(mpos | 1ull);
  }
}

// Second half of a two-pass step: lane and element of a walker's target `t` inside group `g` of the list, from the
// rows group_rows left behind and the 16 biases of the lane that holds the target -- the same arithmetic on the
// same values as batch_stream's search and pick.  Every lane works for its own walker (no cross-lane operations).
// Returns the local index of the selected neighbour.
template <int kApp>
__device__ __forceinline__ int32_t resolve_pick(const uint32_t* __restrict__ bias, const uint32_t off, const uint32_t deg,
                                                const int32_t want, const float* rows, const int32_t* lastpos,
                                                const int32_t g, const float t) {
  constexpr int kEl = 4 * kGroupQuartets;
  const uint32_t a0 = off & ~3u;
  const uint32_t nq = (off + deg - a0 + 3u) >> 2;
  const float* M = rows + (size_t)(uint32_t)g * 128u;
  // M never decreases: three pivots name the quarter of the lanes, its 16 entries the lane
  const float p15 = M[15], p31 = M[31], p47 = M[47];
  const int quarter = p15 > t ? 0 : (p31 > t ? 1 : (p47 > t ? 2 : 3));
  const float4* Mq = reinterpret_cast<const float4*>(M + 16 * quarter);
  const float4 m0 = Mq[0], m1 = Mq[1], m2 = Mq[2], m3 = Mq[3];
  const float m[16] = {m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w, m2.x, m2.y, m2.z, m2.w, m3.x, m3.y, m3.z, m3.w};
  int below = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) below += m[i] <= t ? 1 : 0;
  // first lane whose running maximum exceeds the target; none (rounding in the scan tree): the last positive lane
  const int src = below < 16 ? 16 * quarter + below : lastpos[g];
  float e = M[64 + src];
  const uint32_t kb = (uint32_t)g * (64u * kGroupQuartets) + (uint32_t)src;
  uint4 raw[kGroupQuartets];
#pragma unroll
  for (int j = 0; j < kGroupQuartets; ++j) {
    const uint32_t k = kb + 64u * (uint32_t)j;
    raw[j] = make_uint4(0, 0, 0, 0);
    if (k < nq) raw[j] = *reinterpret_cast<const uint4*>(bias + a0 + 4u * k);
  }
  float x[kEl];
#pragma unroll
  for (int j = 0; j < kGroupQuartets; ++j) {
    if (kApp == FW_APP_METAPATH) {
      x[4 * j + 0] = (int32_t)raw[j].x == want ? 1.0f : 0.0f;
      x[4 * j + 1] = (int32_t)raw[j].y == want ? 1.0f : 0.0f;
      x[4 * j + 2] = (int32_t)raw[j].z == want ? 1.0f : 0.0f;
      x[4 * j + 3] = (int32_t)raw[j].w == want ? 1.0f : 0.0f;
    } else {
      x[4 * j + 0] = __uint_as_float(raw[j].x);
      x[4 * j + 1] = __uint_as_float(raw[j].y);
      x[4 * j + 2] = __uint_as_float(raw[j].z);
      x[4 * j + 3] = __uint_as_float(raw[j].w);
    }
    const uint32_t li = a0 + 4u * (kb + 64u * (uint32_t)j) - off;  // wraps below 0 for the head quartet
    x[4 * j + 0] = li < deg ? x[4 * j + 0] : 0.0f;
    x[4 * j + 1] = li + 1u < deg ? x[4 * j + 1] : 0.0f;
    x[4 * j + 2] = li + 2u < deg ? x[4 * j + 2] : 0.0f;
    x[4 * j + 3] = li + 3u < deg ? x[4 * j + 3] : 0.0f;
  }
  uint32_t cnt = 0u, pm = 0u;
#pragma unroll
  for (int i = 0; i < kEl; ++i) {
    e = e + x[i];
    cnt += e <= t ? 1u : 0u;
    pm |= (x[i] > 0.0f ? 1u : 0u) << i;
  }
  const uint32_t cand = pm >> cnt;
  const int pick = cand != 0u ? (int)cnt + __builtin_ctz(cand) : 31 - __builtin_clz(pm | 1u);
  const uint32_t abs_idx = a0 + 4u * kb + 256u * (uint32_t)(pick >> 2) + (uint32_t)(pick & 3);
  return (int32_t)(abs_idx - off);
}

// A walker's reservoir over the totals of sequence `seq` of a list (groups seq, seq + nw, ...): the group it ends
// up in (-1: none) and its target there.  Totals past the end read as 0, which changes nothing: S stays, and a
// test that failed on S fails again.
__device__ __forceinline__ void table_reservoir(const fw_kargs& a, const float* totals, const uint32_t ngroups,
                                                const uint32_t seq, const uint32_t nw, const uint32_t walker,
                                                const uint32_t step, const uint32_t sbase, int32_t& gsel, float& tsel,
                                                float& S_out) {
  float S = 0.0f, Sj = 0.0f, u = 1.0f;
  LaneDraw dq;
  gsel = -1;
  tsel = 0.0f;
  for (uint32_t g0 = seq; g0 < ngroups; g0 += 4u * nw) {
    float t4[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t g = g0 + (uint32_t)j * nw;
      t4[j] = g < ngroups ? totals[g] : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float Snew = S + t4[j];
      if (Snew * u > Sj) {
        tsel = next_uniform_lane(dq, a, walker, step, seq | sbase) * t4[j];
        gsel = (int32_t)(g0 + (uint32_t)j * nw);
        Sj = Snew;
        u = next_uniform_lane(dq, a, walker, step, seq | sbase);
      }
      S = Snew;
    }
  }
  S_out = S;
}

// A step of up to 64 walkers (lane i = walker i) on a hub whose rows are made: returns each walker's local index
// (or -1).  wg: the list is sampled at workgroup granularity (kNW sequences combined by inverse transform).
template <int kApp, int kNW>
__device__ __forceinline__ int32_t table_sample(const fw_kargs& a, const uint32_t* __restrict__ bias, const uint32_t off,
                                                const uint32_t deg, const int32_t want, const bool wg, const bool have,
                                                const uint32_t walker, const uint32_t step, const uint32_t sbase,
                                                const int lane, const float* totals, const float* rows,
                                                const int32_t* lastpos, float& total_out) {
  constexpr uint32_t kG = 64u * kGroupQuartets;
  const uint32_t nq = (off + deg - (off & ~3u) + 3u) >> 2;
  const uint32_t ngroups = (nq + kG - 1u) / kG;
  const uint32_t nw = wg ? (uint32_t)kNW : 1u;
  int wsel = 0;
  total_out = 0.0f;
  if (wg) {
    // the sequences' totals, each added up in its own order by one lane, then the inverse transform over them
    float Wl = 0.0f;
    if ((uint32_t)lane < nw) {
      for (uint32_t g0 = (uint32_t)lane; g0 < ngroups; g0 += 8u * nw) {
        float t8[8];  // eight loads in flight, added in order; + 0 past the end changes nothing
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint32_t g = g0 + (uint32_t)j * nw;
          t8[j] = g < ngroups ? totals[g] : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) Wl = Wl + t8[j];
      }
    }
    const float J = row_scan(Wl);
    const float total = readlane_f(J, kNW - 1);
    total_out = total;
    const float target = u24(philox4x32_10(walker, step, kStreamWave | sbase, 0u, a.seed_lo, a.seed_hi).x) * total;
    int wlast = -1;
    wsel = -1;
#pragma unroll
    for (int w = 0; w < kNW; ++w) {
      const float Ww = readlane_f(Wl, w);
      const float Jw = readlane_f(J, w);
      if (Ww > 0.0f) {
        wsel = (wsel < 0 && Jw > target) ? w : wsel;
        wlast = w;
      }
    }
    wsel = wsel < 0 ? wlast : wsel;
  }
  // only the sequence the walker ends up in needs running: the draws of a sequence are addressed by the sequence
  int32_t gsel = -1;
  float tsel = 0.0f;
  float S_seq = 0.0f;  // the total of the sequence the reservoir ran over: the list's total at wave granularity
  if (have && wsel >= 0) table_reservoir(a, totals, ngroups, (uint32_t)wsel, nw, walker, step, sbase, gsel, tsel, S_seq);
  if (!wg) total_out = S_seq;
  int32_t pick = -1;
  if (gsel >= 0) pick = resolve_pick<kApp>(bias, off, deg, want, rows, lastpos, gsel, tsel);
  return pick;
}

// Step commit of a batch by one wave (lane i = walker i; include/walker.cuh:1410-1417).  Every walker's record
// goes back to its own position of the output list, so no list counter is contended: finished walks are marked
// (q = -1), walkers whose new vertex is parked on again are tagged and carry their position inside that vertex's
// bucket, the others are picked up from the same list by the next walk launch.
// node2vec: `pick` is a proposal.  A walker whose proposal is rejected stays parked on v with one more trial on its
// record; records carry the previous vertex instead of a position (the scatter kernel hands the positions out).
// Record `at` of the sorted list of parked walkers (the walker stands on v, the vertex of its task).
template <int kApp>
__device__ __forceinline__ fw_walker_rec load_parked(const void* sorted, uint32_t at, int32_t v) {
  if (kApp == FW_APP_NODE2VEC) return static_cast<const fw_walker_rec*>(sorted)[at];
  const fw_parked_rec p = static_cast<const fw_parked_rec*>(sorted)[at];
  fw_walker_rec r;
  r.q = p.q; r.cur = v; r.prev = -1; r.len = p.len;
  return r;
}

// v, off, deg: the list the lane's walker stands on (the same in every lane, or one list per 16-lane row with
// kPerLane, where every lane then counts its own step); out_at: the walker's position in the output list.
// T (node2vec): the list's total as the step's sampler added it up.
template <int kApp, bool kPerLane = false>
__device__ __forceinline__ void batch_commit(const fw_kargs& a, const fw_hub_args& h, const int32_t v,
                                             const uint32_t off, const uint32_t deg, const uint32_t out_at,
                                             const fw_walker_rec rec, const uint32_t trial, const bool have,
                                             const int32_t pick, const uint32_t walker, const uint32_t step,
                                             const int lane, unsigned long long& n_steps,
                                             unsigned long long& n_edges, uint32_t (&n_out)[2], const float T = 0.0f) {
  bool moved = have && pick >= 0;
  bool retry = false;
  bool go_on = false;
  int32_t nv = -1;
  int32_t nv_hidx = -1;  // the parking index of nv when it came with the adjacency entry
  if (moved) {
    if (a.adj_hub != nullptr) {
      const int2 e = a.adj_hub[off + (uint32_t)pick];
      nv = e.x;
      nv_hidx = e.y;
    } else {
      nv = a.adjncy[off + (uint32_t)pick];
    }
    if (kApp == FW_APP_NODE2VEC && rec.prev >= 0) {
      float w_ret = 0.0f;  // T: the list's total as the step's sampler added it up
      if (a.n2v_extra > 0.0f) w_ret = return_weight(a.adjncy + off, a.weight + off, deg, rec.prev);
      const N2vTest t = n2v_test(a, nv, rec.prev, walker, step, trial, T, w_ret);
      if (t.take_prev) {  // the return edge's own component: back to the previous vertex
        nv = rec.prev;
        if (a.adj_hub != nullptr) nv_hidx = a.hub_index[nv];
      } else {
        bool common = false;
        if (!t.decided) {
          const uint32_t po = a.xadj[rec.prev];
          common = sorted_contains(a.adjncy + po, (int32_t)(a.xadj[rec.prev + 1] - po), nv);
        }
        if (!n2v_finish(a, t, common)) {
          moved = false;
          retry = true;
        }
      }
    }
  }
  if (moved) {
    go_on = rec.len + 1 < a.max_depth;
    if (kApp == FW_APP_PPR && go_on) {
      const uint32_t bits = philox4x32_10(walker, step, kStreamStop, 0u, a.seed_lo, a.seed_hi).x;
      go_on = !(u24(bits) < a.tp);
    }
  }
  if (kPerLane) {
    if (moved) {
      n_steps += 1ull;
      n_edges += (unsigned long long)deg;
    }
  } else {
    const uint64_t mmoved = __ballot(moved);
    if (lane == 0) {
      const unsigned long long c = (unsigned long long)__builtin_popcountll(mmoved);
      n_steps += c;
      n_edges += c * (unsigned long long)deg;
    }
  }
  bool park = false;
  int32_t hidx = -1;
  if (go_on) {
    // one look-up tells both what the step commit needs to know about the new vertex: parked on (index >= 0),
    // a dead end that finishes the walk (-2, include/walker.cuh:1373-1374), or neither
    hidx = a.adj_hub != nullptr ? nv_hidx : a.hub_index[nv];
    go_on = hidx != -2;
    park = hidx >= 0;
  }
  if (kApp == FW_APP_NODE2VEC && retry) {  // back into the bucket it came from
    hidx = a.hub_index[v];
    go_on = true;
    park = true;
  }
  if (have && !retry) {
    // Path entries are written in aligned pairs where that is possible: a scattered 4-byte store costs the memory
    // system a read-modify-write of its line, and a pair costs the same.  The walker stands on v = entry len - 1 and
    // moves to nv = entry len.  When entry len is the upper half of an aligned pair, both are stored together.  When
    // it is the lower half and the walker is parked again, nothing is stored: its next step is taken here too and
    // stores the pair (the last few walkers that leave the parking loop instead have their latest entry written by
    // fw_bucket_to_vertex_kernel).  A walk that ends here without a step stores a lower-half v that may be pending.
    int32_t* const at = a.paths + ((uint64_t)(uint32_t)rec.q * (uint64_t)a.max_depth + (uint64_t)rec.len);
    const bool upper = (reinterpret_cast<uintptr_t>(at) & 4u) != 0u;
    if (moved) {
      // (non-temporal: nobody reads a path entry before the call ends, and the line is not worth an L2 slot)
      if (upper) {
        const unsigned long long both = ((unsigned long long)(uint32_t)nv << 32) | (unsigned long long)(uint32_t)v;
        __builtin_nontemporal_store((long long)both, reinterpret_cast<long long*>(at - 1));
      } else if (!(go_on && park)) {
        __builtin_nontemporal_store(nv, at);
      }
    } else if (upper) {
      at[-1] = v;
    }
  }
  const uint32_t label_slot = kApp == FW_APP_METAPATH ? (uint32_t)rec.len % (uint32_t)a.n_labels_per_hub : 0u;
  const uint32_t bucket = (uint32_t)hidx * (uint32_t)a.n_labels_per_hub + label_slot;
  uint32_t rank = 0u;
  if (kApp == FW_APP_NODE2VEC) fw_wave_count_keys<false>(h.bucket_out, bucket, go_on && park);
  else rank = fw_wave_count_keys<true>(h.bucket_out, bucket, go_on && park);
  if (have) {
    fw_walker_rec out;
    out.q = go_on ? rec.q : -1;
    out.cur = nv;
    out.prev = v;
    out.len = rec.len + 1;
    if (kApp == FW_APP_NODE2VEC && retry) {
      out.cur = (int32_t)bucket;
      out.prev = rec.prev;
      out.len = rec.len | (int32_t)((trial + 1u) << FW_REC_TRIAL_SHIFT) | FW_REC_PARK;
    } else if (go_on && park) {
      out.cur = (int32_t)bucket;  // the vertex follows from the bucket
      if (kApp != FW_APP_NODE2VEC) out.prev = (int32_t)rank;
      out.len |= FW_REC_PARK;
    }
    h.out[out_at] = out;
  }
  const uint64_t mpark = __ballot(go_on && park);
  const uint64_t mres = __ballot(go_on && !park);
  if (lane == 0) {
    n_out[0] += (uint32_t)__builtin_popcountll(mres);
    n_out[1] += (uint32_t)__builtin_popcountll(mpark);
  }
}

template <int kApp, int kWGT>
__global__ __launch_bounds__(kWGT, 8) void fw_hub_batch(const fw_kargs a, const fw_hub_args h) {
  constexpr int kNW = kWGT / 64;
  __shared__ int32_t s_sel[kNW][64];
  __shared__ float s_w[16];
  __shared__ uint32_t s_task;
  __shared__ int32_t s_schema[kApp == FW_APP_METAPATH ? FW_MAX_SCHEMA : 1];
  __shared__ unsigned long long s_acc[2];
  __shared__ uint32_t s_out[2];

  const int tid = (int)threadIdx.x;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (tid == 0) {
    s_acc[0] = s_acc[1] = 0ull;
    s_out[0] = s_out[1] = 0u;
  }
  if (kApp == FW_APP_METAPATH && threadIdx.x == 0) {
#pragma unroll
    for (int i = 0; i < FW_MAX_SCHEMA; ++i) s_schema[i] = a.schema[i];
  }
  const uint32_t ntasks = *h.ntasks;
  const uint32_t nwtasks = *h.nwtasks;
  const uint32_t* __restrict__ bias =
      reinterpret_cast<const uint32_t*>(kApp == FW_APP_METAPATH ? (const void*)a.label : (const void*)a.weight);
  unsigned long long n_steps = 0ull, n_edges = 0ull;
  uint32_t n_out[2] = {0u, 0u};  // walkers that resume / that are parked again

  __syncthreads();  // the shared initialisation above is visible

  // ---- table tasks first: 64 walkers of a crowded hub whose rows the scan launch has made; one wave each,
  //      dealt out by position like the wave tasks ----
  const uint32_t nwaves = gridDim.x * (uint32_t)kNW;
  const uint32_t nttasks = *h.nttasks;
  for (uint32_t t = blockIdx.x * (uint32_t)kNW + (uint32_t)wave; t < nttasks; t += nwaves) {
    const fw_batch_task* tp = h.ttasks + t;
    const int32_t v = __builtin_amdgcn_readfirstlane(tp->v);
    const uint32_t off = (uint32_t)__builtin_amdgcn_readfirstlane((int)tp->off);
    const uint32_t deg = (uint32_t)__builtin_amdgcn_readfirstlane((int)tp->deg);
    const uint32_t rec_base = (uint32_t)__builtin_amdgcn_readfirstlane((int)tp->rec_base);
    const int count = __builtin_amdgcn_readfirstlane(tp->count);
    const uint32_t row_base = (uint32_t)__builtin_amdgcn_readfirstlane((int)tp->row);
    const int32_t want = kApp == FW_APP_METAPATH ? s_schema[__builtin_amdgcn_readfirstlane(tp->slot)] : 0;

    const bool have = lane < count;
    fw_walker_rec rec;
    rec.q = 0; rec.cur = v; rec.prev = -1; rec.len = 1;
    if (have) rec = load_parked<kApp>(h.sorted, rec_base + (uint32_t)lane, v);
    uint32_t trial = 0u;
    if (kApp == FW_APP_NODE2VEC) {
      trial = (uint32_t)((rec.len >> FW_REC_TRIAL_SHIFT) & FW_REC_TRIAL_MASK);
      rec.len &= FW_REC_LEN_MASK;
    }
    const uint32_t walker = a.walker_base + (uint32_t)rec.q;
    const uint32_t step = (uint32_t)(rec.len - 1);

    float T = 0.0f;
    const int32_t sel = table_sample<kApp, kNW>(a, bias, off, deg, want, (int32_t)deg > a.hub_threshold, have, walker,
                                               step, trial << 8, lane, h.totals + row_base,
                                               h.rows + (size_t)row_base * 128u, h.lastpos + row_base, T);
    batch_commit<kApp>(a, h, v, off, deg, rec_base + (uint32_t)lane, rec, trial, have, sel, walker, step, lane, n_steps,
                       n_edges, n_out, T);
  }

  // ---- then wave tasks: lists up to hub_threshold, sampled at wave granularity, one batch per wave; the tasks are
  //      short and many, so they are dealt out by position instead of through a contended counter ----
  for (uint32_t t = blockIdx.x * (uint32_t)kNW + (uint32_t)wave; t < nwtasks; t += nwaves) {
    const fw_batch_task* tp = h.wtasks + t;
    const int32_t v = __builtin_amdgcn_readfirstlane(tp->v);
    const uint32_t off = (uint32_t)__builtin_amdgcn_readfirstlane((int)tp->off);
    const uint32_t deg = (uint32_t)__builtin_amdgcn_readfirstlane((int)tp->deg);
    const uint32_t rec_base = (uint32_t)__builtin_amdgcn_readfirstlane((int)tp->rec_base);
    const int count = __builtin_amdgcn_readfirstlane(tp->count);
    const int32_t want = kApp == FW_APP_METAPATH ? s_schema[__builtin_amdgcn_readfirstlane(tp->slot)] : 0;

    const bool have = lane < count;
    fw_walker_rec rec;
    rec.q = 0; rec.cur = v; rec.prev = -1; rec.len = 1;
    if (have) rec = load_parked<kApp>(h.sorted, rec_base + (uint32_t)lane, v);
    uint32_t trial = 0u;
    if (kApp == FW_APP_NODE2VEC) {
      trial = (uint32_t)((rec.len >> FW_REC_TRIAL_SHIFT) & FW_REC_TRIAL_MASK);
      rec.len &= FW_REC_LEN_MASK;
    }
    const uint32_t walker = a.walker_base + (uint32_t)rec.q;
    const uint32_t step = (uint32_t)(rec.len - 1);

    float S;
    int32_t sel;
    batch_stream<kApp>(a, bias, off, deg, want, 0u, 1u, have, walker, step, trial << 8, lane, S, sel);
    batch_commit<kApp>(a, h, v, off, deg, rec_base + (uint32_t)lane, rec, trial, have, sel, walker, step, lane, n_steps,
                       n_edges, n_out, S);
  }

  // ---- then workgroup tasks: lists above hub_threshold, sampled at workgroup granularity.  They are few, long and
  //      uneven, so they are handed out through a counter -- to the last resident set of workgroups only: the
  //      rest of an oversized grid exists to even out the wave tasks (one counter update per workgroup of it
  //      would cost more than these tasks), and the workgroups that start last hold nobody up while they work
  //      through long lists ----
  for (;;) {
    if (blockIdx.x + h.dynamic_wgs < gridDim.x) break;
    if (tid == 0) s_task = atomicAdd(h.task_next, 1u);
    __syncthreads();
    const uint32_t t = s_task;
    __syncthreads();  // everyone has read s_task before it is overwritten; also fences s_sel / s_w reuse
    if (t >= ntasks) break;

    const fw_batch_task task = h.tasks[t];
    const int32_t want = kApp == FW_APP_METAPATH ? s_schema[task.slot] : 0;

    // lane i carries walker i of the batch
    const bool have = lane < task.count;
    fw_walker_rec rec;
    rec.q = 0; rec.cur = task.v; rec.prev = -1; rec.len = 1;
    if (have) rec = load_parked<kApp>(h.sorted, task.rec_base + (uint32_t)lane, task.v);
    uint32_t trial = 0u;
    if (kApp == FW_APP_NODE2VEC) {
      trial = (uint32_t)((rec.len >> FW_REC_TRIAL_SHIFT) & FW_REC_TRIAL_MASK);
      rec.len &= FW_REC_LEN_MASK;
    }
    const uint32_t walker = a.walker_base + (uint32_t)rec.q;
    const uint32_t step = (uint32_t)(rec.len - 1);

    float S;
    int32_t sel;
    batch_stream<kApp>(a, bias, task.off, task.deg, want, (uint32_t)wave, (uint32_t)kNW, have, walker, step, trial << 8,
                       lane, S, sel);
    s_sel[wave][lane] = sel;
    if (lane == 0) s_w[wave] = S;
    __syncthreads();

    if (wave == 0) {
      // inverse transform over the wave totals, per walker (include/sampler.cuh:118-126 is the max-reduce analogue)
      const float Wl = lane < kNW ? s_w[lane] : 0.0f;
      const float J = row_scan(Wl);
      const float total = readlane_f(J, kNW - 1);
      int32_t pick = -1;
      if (have) {
        const float target = u24(philox4x32_10(walker, step, kStreamWave | (trial << 8), 0u, a.seed_lo, a.seed_hi).x) * total;
        int wsel = -1, wlast = -1;
#pragma unroll
        for (int w = 0; w < kNW; ++w) {
          const float Ww = readlane_f(Wl, w);
          const float Jw = readlane_f(J, w);
          if (Ww > 0.0f) {
            wsel = (wsel < 0 && Jw > target) ? w : wsel;
            wlast = w;
          }
        }
        wsel = wsel < 0 ? wlast : wsel;
        if (wsel >= 0) pick = s_sel[wsel][lane];
      }
      batch_commit<kApp>(a, h, task.v, task.off, task.deg, task.rec_base + (uint32_t)lane, rec, trial, have, pick, walker,
                         step, lane, n_steps, n_edges, n_out, total);
    }
  }

  // counters: summed inside the workgroup first (the global ones are contended); the batch kernel's share of the
  // workload is counted apart and added up by the host
  if (n_steps != 0ull) {
    atomicAdd(&s_acc[0], n_steps);
    atomicAdd(&s_acc[1], n_edges);
  }
  // (a wave of node2vec walkers whose proposals were all rejected has walkers to hand on and no steps)
  if (n_out[0] != 0u) atomicAdd(&s_out[0], n_out[0]);
  if (n_out[1] != 0u) atomicAdd(&s_out[1], n_out[1]);
  __syncthreads();
  if (tid == 0) {
    if (s_acc[0] != 0ull) {
      atomicAdd(&a.counters[2], s_acc[0]);
      atomicAdd(&a.counters[3], s_acc[1]);
    }
    if (s_out[0] != 0u) atomicAdd(&h.out_counts[0], s_out[0]);
    if (s_out[1] != 0u) atomicAdd(&h.out_counts[FW_CTR_STRIDE], s_out[1]);
  }
}

// Quad tasks: lists of at most 64 aligned quartets with at most 16 walkers, four tasks per wave, one per 16-lane row
// (most parked-on lists are short and hold a few walkers: a wave of its own would leave most of its lanes idle
// through the per-walker part of the step).  Such a list is one group whose lane L holds quartet L alone; lane i of a
// row stands in for lanes i, 16 + i, 32 + i and 48 + i of that group, one after the other, and puts their prefixes
// together exactly as the whole-wave scan does: row_bcast:15 adds the last prefix of row 0 to row 1 and that of row 2
// to row 3, row_bcast:31 then adds lane 31's sum to rows 2 and 3.  The walkers then resolve their targets as the table
// tasks do, from rows that the wave keeps in LDS.  A kernel of its own, so that its registers are not the batch
// kernel's.
template <int kApp>
__global__ __launch_bounds__(256, 8) void fw_hub_quad(const fw_kargs a, const fw_hub_args h) {
  constexpr int kNW = 4;
  __shared__ __align__(16) float s_qrows[kNW][4][128];  // per wave and row: 64 running maxima, 64 prefixes
  __shared__ int32_t s_schema[kApp == FW_APP_METAPATH ? FW_MAX_SCHEMA : 1];
  __shared__ unsigned long long s_acc[2];
  __shared__ uint32_t s_out[2];
  const int tid = (int)threadIdx.x;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (tid == 0) {
    s_acc[0] = s_acc[1] = 0ull;
    s_out[0] = s_out[1] = 0u;
  }
  if (kApp == FW_APP_METAPATH && threadIdx.x == 0) {
#pragma unroll
    for (int i = 0; i < FW_MAX_SCHEMA; ++i) s_schema[i] = a.schema[i];
  }
  const uint32_t* __restrict__ bias =
      reinterpret_cast<const uint32_t*>(kApp == FW_APP_METAPATH ? (const void*)a.label : (const void*)a.weight);
  unsigned long long n_steps = 0ull, n_edges = 0ull;
  uint32_t n_out[2] = {0u, 0u};
  const uint32_t nwaves = gridDim.x * (uint32_t)kNW;
  __syncthreads();
  {
    const int row = lane >> 4;
    const int rl = lane & 15;
    const uint32_t nqtasks = *h.nqtasks;
    float* const myM = &s_qrows[wave][row][0];
    float* const myE = &s_qrows[wave][row][64];
    const int row_last = (lane | 15) << 2;  // byte address of the row's lane 15 for ds_bpermute
    for (uint32_t t4 = 4u * (blockIdx.x * (uint32_t)kNW + (uint32_t)wave); t4 < nqtasks; t4 += 4u * nwaves) {
      const uint32_t t = t4 + (uint32_t)row;
      const bool live = t < nqtasks;
      fw_batch_task task;
      task.v = 0; task.off = 0; task.deg = 0; task.rec_base = 0; task.count = 0; task.slot = 0; task.row = 0; task.pad = 0;
      if (live) task = h.qtasks[t];
      const int32_t want = kApp == FW_APP_METAPATH ? s_schema[task.slot] : 0;
      const bool have = rl < task.count;
      fw_walker_rec rec;
      rec.q = 0; rec.cur = task.v; rec.prev = -1; rec.len = 1;
      if (have) rec = load_parked<kApp>(h.sorted, task.rec_base + (uint32_t)rl, task.v);
      uint32_t trial = 0u;
      if (kApp == FW_APP_NODE2VEC) {
        trial = (uint32_t)((rec.len >> FW_REC_TRIAL_SHIFT) & FW_REC_TRIAL_MASK);
        rec.len &= FW_REC_LEN_MASK;
      }
      const uint32_t walker = a.walker_base + (uint32_t)rec.q;
      const uint32_t step = (uint32_t)(rec.len - 1);

      const uint32_t a0 = task.off & ~3u;
      const uint32_t nq = (task.off + task.deg - a0 + 3u) >> 2;
      float x[4][4];
      float q[4];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const uint32_t k = 16u * (uint32_t)s + (uint32_t)rl;
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (live && k < nq) raw = *reinterpret_cast<const uint4*>(bias + a0 + 4u * k);
        if (kApp == FW_APP_METAPATH) {
          x[s][0] = (int32_t)raw.x == want ? 1.0f : 0.0f;
          x[s][1] = (int32_t)raw.y == want ? 1.0f : 0.0f;
          x[s][2] = (int32_t)raw.z == want ? 1.0f : 0.0f;
          x[s][3] = (int32_t)raw.w == want ? 1.0f : 0.0f;
        } else {
          x[s][0] = __uint_as_float(raw.x);
          x[s][1] = __uint_as_float(raw.y);
          x[s][2] = __uint_as_float(raw.z);
          x[s][3] = __uint_as_float(raw.w);
        }
        const uint32_t li = a0 + 4u * k - task.off;  // wraps below 0 for the head quartet
        x[s][0] = live && k < nq && li < task.deg ? x[s][0] : 0.0f;
        x[s][1] = live && k < nq && li + 1u < task.deg ? x[s][1] : 0.0f;
        x[s][2] = live && k < nq && li + 2u < task.deg ? x[s][2] : 0.0f;
        x[s][3] = live && k < nq && li + 3u < task.deg ? x[s][3] : 0.0f;
        q[s] = (((0.0f + x[s][0]) + x[s][1]) + x[s][2]) + x[s][3];  // the lane's other twelve biases are zeros
      }
      // prefixes of the 64 lanes of the group, put together as wave_scan does
      float I[4];
      I[0] = row_scan(q[0]);
      const float p1 = row_scan(q[1]);
      const float p2 = row_scan(q[2]);
      const float p3 = row_scan(q[3]);
      const float R0 = bperm_f(row_last, I[0]);
      I[1] = p1 + R0;
      const float C1 = bperm_f(row_last, I[1]);
      const float R2 = bperm_f(row_last, p2);
      I[2] = p2 + C1;
      I[3] = (p3 + R2) + C1;
      const float T = bperm_f(row_last, I[3]);
      // running maximum of the positive lanes' prefixes, and the last positive lane
      float M[4];
      uint32_t carry = 0u;
      int lastpos = 0;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const bool pos = q[s] > 0.0f;
        float m = pos ? I[s] : 0.0f;
        m = dpp_max<0x111, 0xF>(m);
        m = dpp_max<0x112, 0xF>(m);
        m = dpp_max<0x114, 0xF>(m);
        m = dpp_max<0x118, 0xF>(m);
        const uint32_t mi = __float_as_uint(m);
        M[s] = __uint_as_float(mi > carry ? mi : carry);
        carry = __float_as_uint(bperm_f(row_last, M[s]));
        const uint32_t mrow = (uint32_t)(__ballot(pos) >> (16 * row)) & 0xFFFFu;
        if (mrow != 0u) lastpos = 16 * s + 31 - __builtin_clz(mrow);
      }
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        myM[16 * s + rl] = M[s];
        myE[16 * s + rl] = I[s] - q[s];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

      // per walker: one group, so the reservoir accepts it as soon as its total is positive (S * 1 > 0)
      const bool acc = have && (T * 1.0f > 0.0f);
      int32_t sel = -1;
      {
        LaneDraw dq;
        float target = 0.0f;
        if (acc) target = next_uniform_lane(dq, a, walker, step, trial << 8) * T;
        const float p15 = myM[15], p31 = myM[31], p47 = myM[47];
        const int quarter = p15 > target ? 0 : (p31 > target ? 1 : (p47 > target ? 2 : 3));
        const float4* Mq = reinterpret_cast<const float4*>(myM + 16 * quarter);
        const float4 m0 = Mq[0], m1 = Mq[1], m2 = Mq[2], m3 = Mq[3];
        const float mm[16] = {m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w, m2.x, m2.y, m2.z, m2.w, m3.x, m3.y, m3.z, m3.w};
        int below = 0;
#pragma unroll
        for (int i = 0; i < 16; ++i) below += mm[i] <= target ? 1 : 0;
        const int src = below < 16 ? 16 * quarter + below : lastpos;
        float e = myE[src];
        // the quartet of lane src: held by the row's lane src & 15 in its pass src >> 4
        const int from = ((lane & 48) | (src & 15)) << 2;
        const int pass = src >> 4;
        float xs[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const float y0 = bperm_f(from, x[0][c]), y1 = bperm_f(from, x[1][c]);
          const float y2 = bperm_f(from, x[2][c]), y3 = bperm_f(from, x[3][c]);
          xs[c] = pass == 0 ? y0 : (pass == 1 ? y1 : (pass == 2 ? y2 : y3));
        }
        uint32_t cnt = 0u, pm = 0u;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          e = e + xs[c];
          cnt += e <= target ? 1u : 0u;
          pm |= (xs[c] > 0.0f ? 1u : 0u) << c;
        }
        cnt += e <= target ? 12u : 0u;  // the twelve zeros that follow leave the sum where it is
        const uint32_t cand = pm >> cnt;
        const int pick = cand != 0u ? (int)cnt + __builtin_ctz(cand) : 31 - __builtin_clz(pm | 1u);
        if (acc) sel = (int32_t)(a0 + 4u * (uint32_t)src + (uint32_t)pick - task.off);
      }
      __builtin_amdgcn_wave_barrier();  // the rows are rewritten by the wave's next four tasks
      batch_commit<kApp, true>(a, h, task.v, task.off, task.deg, task.rec_base + (uint32_t)rl, rec, trial, have, sel, walker,
                               step, lane, n_steps, n_edges, n_out, T);
    }
  }

  if (n_steps != 0ull) {
    atomicAdd(&s_acc[0], n_steps);
    atomicAdd(&s_acc[1], n_edges);
  }
  if (n_out[0] != 0u) atomicAdd(&s_out[0], n_out[0]);
  if (n_out[1] != 0u) atomicAdd(&s_out[1], n_out[1]);
  __syncthreads();
  if (tid == 0) {
    if (s_acc[0] != 0ull) {
      atomicAdd(&a.counters[2], s_acc[0]);
      atomicAdd(&a.counters[3], s_acc[1]);
    }
    if (s_out[0] != 0u) atomicAdd(&h.out_counts[0], s_out[0]);
    if (s_out[1] != 0u) atomicAdd(&h.out_counts[FW_CTR_STRIDE], s_out[1]);
  }
}

// First pass of the two-pass steps: the rows of every crowded hub of the round.  A scan task is a run of groups
// of one list (rec_base = first group, count = one past the last, row = the list's first row); one wave per
// task, tasks dealt out by position.
template <int kApp>
__global__ __launch_bounds__(256) void fw_hub_scan(const fw_kargs a, const fw_hub_args h) {
  __shared__ int32_t s_schema[kApp == FW_APP_METAPATH ? FW_MAX_SCHEMA : 1];
  if (kApp == FW_APP_METAPATH) {
    if (threadIdx.x == 0) {
#pragma unroll
      for (int i = 0; i < FW_MAX_SCHEMA; ++i) s_schema[i] = a.schema[i];
    }
    __syncthreads();
  }
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const uint32_t nstasks = *h.nstasks;
  const uint32_t* __restrict__ bias =
      reinterpret_cast<const uint32_t*>(kApp == FW_APP_METAPATH ? (const void*)a.label : (const void*)a.weight);
  const uint32_t nwaves = gridDim.x * 4u;
  for (uint32_t t = blockIdx.x * 4u + (uint32_t)wave; t < nstasks; t += nwaves) {
    const fw_batch_task* tp = h.stasks + t;
    const uint32_t off = (uint32_t)__builtin_amdgcn_readfirstlane((int)tp->off);
    const uint32_t deg = (uint32_t)__builtin_amdgcn_readfirstlane((int)tp->deg);
    const uint32_t g0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)tp->rec_base);
    const uint32_t g1 = (uint32_t)__builtin_amdgcn_readfirstlane(tp->count);
    const uint32_t row_base = (uint32_t)__builtin_amdgcn_readfirstlane((int)tp->row);
    const int32_t want = kApp == FW_APP_METAPATH ? s_schema[__builtin_amdgcn_readfirstlane(tp->slot)] : 0;
    for (uint32_t g = g0; g < g1; ++g) {
      const size_t r = (size_t)row_base + g;
      group_rows<kApp>(bias, off, deg, want, g, lane, h.rows + r * 128u, h.totals + r, h.lastpos + r);
    }
  }
}

// tasks_hint: about how many scan tasks to expect (the launch works through any number; 0 = no idea)
template <int kApp>
int launch_hub_scan_app(const fw_kargs& a, const fw_hub_args& h, uint32_t tasks_hint, hipStream_t stream) {
  int dev = 0, cus = 0;
  FW_HIP(hipGetDevice(&dev));
  FW_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  uint32_t grid = (uint32_t)cus * 8u;  // one resident set
  if (tasks_hint != 0u && tasks_hint / 2u + 32u < grid) grid = tasks_hint / 2u + 32u;  // 4 waves a workgroup, room to grow
  hipLaunchKernelGGL((fw_hub_scan<kApp>), dim3(grid), dim3(256), 0, stream, a, h);
  FW_HIP(hipGetLastError());
  return FW_OK;
}

// quads_hint: about how many quad tasks to expect (the launch works through any number; 0 = no idea).  Four tasks per
// wave and turn, about kQuadTurns turns per wave, up to eight resident sets (see launch_hub_one).
constexpr uint32_t kQuadTurns = 4;
template <int kApp>
int launch_hub_quad_app(const fw_kargs& a, const fw_hub_args& h, uint32_t quads_hint, hipStream_t stream) {
  int dev = 0, cus = 0;
  FW_HIP(hipGetDevice(&dev));
  FW_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  const uint32_t resident = (uint32_t)cus * 8u;  // workgroups of four waves, eight waves per SIMD
  uint32_t grid = resident;
  if (quads_hint != 0u) {
    const uint32_t wanted = quads_hint / (4u * 4u * kQuadTurns) + 1u;
    grid = wanted < 8u * resident ? wanted : 8u * resident;
  }
  hipLaunchKernelGGL((fw_hub_quad<kApp>), dim3(grid), dim3(256), 0, stream, a, h);
  FW_HIP(hipGetLastError());
  return FW_OK;
}

// Compute units of the current device and workgroups of `kernel` that fit one of them; asked once per kernel and
// device (the answers do not change, and the questions are slow enough to matter in rounds of 0.3 ms).
template <typename Kernel>
int resident_set(Kernel kernel, int wg_threads, int* cus_out, int* per_cu_out) {
  struct Entry {
    const void* kernel;
    int dev, cus, per_cu;
  };
  constexpr int kEntries = 64;
  static Entry s_entries[kEntries];
  static int s_count = 0;
  static std::mutex s_lock;
  int dev = 0;
  FW_HIP(hipGetDevice(&dev));
  const void* key = reinterpret_cast<const void*>(kernel);
  {
    std::lock_guard<std::mutex> guard(s_lock);
    for (int i = 0; i < s_count; ++i)
      if (s_entries[i].kernel == key && s_entries[i].dev == dev) {
        *cus_out = s_entries[i].cus;
        *per_cu_out = s_entries[i].per_cu;
        return FW_OK;
      }
  }
  int cus = 0, per_cu = 0;
  FW_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  FW_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, wg_threads, 0));
  if (per_cu < 1) per_cu = 1;
  {
    std::lock_guard<std::mutex> guard(s_lock);
    if (s_count < kEntries) s_entries[s_count++] = Entry{key, dev, cus, per_cu};
  }
  *cus_out = cus;
  *per_cu_out = per_cu;
  return FW_OK;
}

// tasks_hint: about how many wave-sized pieces of work the launch will find (wave tasks + table tasks + waves of
// workgroup tasks; 0 = no idea).  All tasks are dealt out by position, so the grid may be larger than what is
// resident: the hardware then starts a workgroup wherever one has finished, which evens out the uneven shares
// without any counter.  About kTasksPerWave tasks per wave, between one and eight resident sets.
constexpr uint32_t kTasksPerWave = 4;

template <int kApp, int kWGT>
int launch_hub_one(const fw_kargs& a, const fw_hub_args& h, uint32_t tasks_hint, hipStream_t stream) {
  int cus = 0, per_cu = 0;
  const int rc = resident_set(fw_hub_batch<kApp, kWGT>, kWGT, &cus, &per_cu);
  if (rc != FW_OK) return rc;
  const int resident = cus * per_cu;
  fw_hub_args hh = h;
  hh.dynamic_wgs = (uint32_t)resident;
  int grid = resident;
  if (tasks_hint != 0u) {
    const uint32_t wanted = tasks_hint / ((uint32_t)(kWGT / 64) * kTasksPerWave);
    if (wanted > (uint32_t)grid) grid = wanted < 8u * (uint32_t)resident ? (int)wanted : 8 * resident;
  }
  hipLaunchKernelGGL((fw_hub_batch<kApp, kWGT>), dim3(grid), dim3(kWGT), 0, stream, a, hh);
  FW_HIP(hipGetLastError());
  return FW_OK;
}

template <int kApp>
int launch_hub_app(const fw_kargs& a, const fw_hub_args& h, int wg_threads, uint32_t tasks_hint, hipStream_t stream) {
  switch (wg_threads) {
    case 256: return launch_hub_one<kApp, 256>(a, h, tasks_hint, stream);
    case 512: return launch_hub_one<kApp, 512>(a, h, tasks_hint, stream);
    case 1024: return launch_hub_one<kApp, 1024>(a, h, tasks_hint, stream);
    default:
      fw_set_error("wg_threads must be 256, 512 or 1024 (got %d)", wg_threads);
      return FW_ERR_INVALID;
  }
}

// entries_hint (launches of the parking pipeline; 0 otherwise): about how many entries the launch will find.  Their
// walkers are short-lived (a step or two until they are parked again), so a launch is a few rounds of refills plus
// a tail of sparse rounds that every workgroup pays.  kEntriesPerWorkgroup entries per workgroup, at least one
// workgroup per compute unit and at most a resident set: large launches fill the device, small ones (the later rounds,
// the smaller batches) take as many workgroups as give each about a refill and a half of its task table.
constexpr int kEntriesPerWorkgroup = 700;

template <int kApp, int kWGT>
int launch_one(fw_kargs a, int grid, uint32_t entries_hint, hipStream_t stream, int* grid_used) {
  // launches of the parking pipeline (they park, or they continue parked walkers) take the variant with several
  // bundles in flight
  constexpr int kFlight = kPipelineInFlight;
  const bool pipeline = kFlight != 1 && (a.park_threshold != 0x7FFFFFFF || a.resume != nullptr);
  if (grid <= 0) {
    int cus = 0, per_cu = 0;
    const int rc = pipeline ? resident_set(fw_walk_zprs<kApp, kWGT, kFlight>, kWGT, &cus, &per_cu)
                            : resident_set(fw_walk_zprs<kApp, kWGT, 1>, kWGT, &cus, &per_cu);
    if (rc != FW_OK) return rc;
    grid = cus * per_cu;
    if (entries_hint != 0u) {
      const int wanted = (int)(entries_hint / (uint32_t)kEntriesPerWorkgroup);
      if (wanted < grid) grid = wanted > cus ? wanted : cus;
    }
  }
  // a small batch is spread over the grid (down to one query per workgroup) instead of filling the
  // task table of a few workgroups: fewer slots per workgroup, same persistent grid
  if (grid > a.n) grid = a.n;
  const long long per_wg = ((long long)a.n + grid - 1) / grid;
  a.slot_limit = (int32_t)(per_wg < kWGT ? per_wg : kWGT);
  if (pipeline)
    hipLaunchKernelGGL((fw_walk_zprs<kApp, kWGT, kFlight>), dim3(grid), dim3(kWGT), 0, stream, a);
  else
    hipLaunchKernelGGL((fw_walk_zprs<kApp, kWGT, 1>), dim3(grid), dim3(kWGT), 0, stream, a);
  FW_HIP(hipGetLastError());
  if (grid_used) *grid_used = grid;
  return FW_OK;
}

template <int kApp>
int launch_app(const fw_kargs& a, int wg_threads, int grid, uint32_t entries_hint, hipStream_t stream,
               int* grid_used) {
  switch (wg_threads) {
    case 256: return launch_one<kApp, 256>(a, grid, entries_hint, stream, grid_used);
    case 512: return launch_one<kApp, 512>(a, grid, entries_hint, stream, grid_used);
    case 1024: return launch_one<kApp, 1024>(a, grid, entries_hint, stream, grid_used);
    default:
      fw_set_error("wg_threads must be 256, 512 or 1024 (got %d)", wg_threads);
      return FW_ERR_INVALID;
  }
}

}  // namespace

int fw_launch_hub_scan(const fw_kargs& a, const fw_hub_args& h, int app, uint32_t tasks_hint, hipStream_t stream) {
  switch (app) {
    case FW_APP_DEEPWALK: return launch_hub_scan_app<FW_APP_DEEPWALK>(a, h, tasks_hint, stream);
    case FW_APP_PPR: return launch_hub_scan_app<FW_APP_PPR>(a, h, tasks_hint, stream);
    case FW_APP_NODE2VEC: return launch_hub_scan_app<FW_APP_DEEPWALK>(a, h, tasks_hint, stream);  // the same rows: plain weights
    case FW_APP_METAPATH: return launch_hub_scan_app<FW_APP_METAPATH>(a, h, tasks_hint, stream);
    default:
      fw_set_error("unknown app %d", app);
      return FW_ERR_INVALID;
  }
}

int fw_launch_hub_quad(const fw_kargs& a, const fw_hub_args& h, int app, uint32_t quads_hint, hipStream_t stream) {
  switch (app) {
    case FW_APP_DEEPWALK: return launch_hub_quad_app<FW_APP_DEEPWALK>(a, h, quads_hint, stream);
    case FW_APP_PPR: return launch_hub_quad_app<FW_APP_PPR>(a, h, quads_hint, stream);
    case FW_APP_NODE2VEC: return launch_hub_quad_app<FW_APP_NODE2VEC>(a, h, quads_hint, stream);
    case FW_APP_METAPATH: return launch_hub_quad_app<FW_APP_METAPATH>(a, h, quads_hint, stream);
    default:
      fw_set_error("unknown app %d", app);
      return FW_ERR_INVALID;
  }
}

int fw_launch_hub_batch(const fw_kargs& a, const fw_hub_args& h, int app, int wg_threads, uint32_t tasks_hint,
                        hipStream_t stream) {
  switch (app) {
    case FW_APP_DEEPWALK: return launch_hub_app<FW_APP_DEEPWALK>(a, h, wg_threads, tasks_hint, stream);
    case FW_APP_PPR: return launch_hub_app<FW_APP_PPR>(a, h, wg_threads, tasks_hint, stream);
    case FW_APP_NODE2VEC: return launch_hub_app<FW_APP_NODE2VEC>(a, h, wg_threads, tasks_hint, stream);
    case FW_APP_METAPATH: return launch_hub_app<FW_APP_METAPATH>(a, h, wg_threads, tasks_hint, stream);
    default:
      fw_set_error("unknown app %d", app);
      return FW_ERR_INVALID;
  }
}

int fw_launch_walk(const fw_kargs& a, int app, int sampler, int wg_threads, int grid, uint32_t entries_hint,
                   hipStream_t stream, int* grid_used) {
  // FW_SAMPLER_DPRS is an alias: the one sampler already evaluates every bias exactly once, which is
  // what the reference's DPRS kernel (include/walker.cuh:1444) exists for.
  constexpr int kRefFlags = FW_SAMPLER_REF_STATIC | FW_SAMPLER_REF_RNG_LDS | FW_SAMPLER_REF_RNG_GLOBAL;
  if ((sampler & ~kRefFlags) == FW_SAMPLER_REF_ZPRS || (sampler & ~kRefFlags) == FW_SAMPLER_REF_DPRS)
    return fw_launch_ref_walk(a, app, sampler, wg_threads, grid, stream, grid_used);
  if (sampler != FW_SAMPLER_ZPRS && sampler != FW_SAMPLER_DPRS) {
    fw_set_error("unknown sampler %d", sampler);
    return FW_ERR_INVALID;
  }
  switch (app) {
    case FW_APP_DEEPWALK: return launch_app<FW_APP_DEEPWALK>(a, wg_threads, grid, entries_hint, stream, grid_used);
    case FW_APP_PPR: return launch_app<FW_APP_PPR>(a, wg_threads, grid, entries_hint, stream, grid_used);
    case FW_APP_NODE2VEC: return launch_app<FW_APP_NODE2VEC>(a, wg_threads, grid, entries_hint, stream, grid_used);
    case FW_APP_METAPATH: return launch_app<FW_APP_METAPATH>(a, wg_threads, grid, entries_hint, stream, grid_used);
    default:
      fw_set_error("unknown app %d", app);
      return FW_ERR_INVALID;
  }
}
