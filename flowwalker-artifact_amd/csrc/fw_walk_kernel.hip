// Sampler-centric random-walk kernel for gfx950 (MI355X): persistent workgroups, an LDS task table,
// a global atomic query dispenser, a one-pass zero-preprocessing parallel reservoir sampler (ZPRS)
// at wavefront (64 lanes) and workgroup granularity, Philox4x32-10 counter-based draws, and the
// DeepWalk / PPR / node2vec / MetaPath bias functors.
//
// Reference behaviour this replaces: walker_wb_dynamic_zprs / _dprs (include/walker.cuh:1307-1580),
// sampler_warp / sampler_block (include/sampler.cuh:46-127), Task (include/gpu_task.cuh:24-78),
// the functors of include/app.cuh:58-152 and check_connect (include/gpu_graph.cuh:97-118).
//
// Round structure of one workgroup (WGT threads, WGT task slots in LDS, SoA):
//   B  every hub slot (degree > hub_threshold) is streamed by the whole workgroup: lane-local
//      reservoirs, per-wave combine, partial (selection, total) pairs parked in LDS; one barrier per
//      chunk of hubs, then one wave per hub combines the wave partials and commits the step.
//   A  waves claim the remaining slots one by one from an LDS counter and sample them alone.
//   C  one thread per slot: reload the CSR range of the new vertex, stop test, refill from the
//      global dispenser (one atomic per wave per refill round), classify into next round's lists.
//
// Results depend only on (seed, walker id, graph, parameters): every random draw is addressed by
// (walker, step, lane stream, draw index), never by which wave or workgroup happens to run the slot.

#include "fw_internal.h"

namespace {

constexpr uint32_t kStreamWave = 0x40000000u;  // | wave index: workgroup-level combine draws
constexpr uint32_t kStreamStop = 0x80000000u;  // PPR stop draw
constexpr int kHubChunk = 32;                  // hub tasks whose wave partials are parked in LDS at once
constexpr int kFlagMoved = 1;
constexpr int kFlagDead = 2;
#ifndef FW_STREAM_UNROLL
#define FW_STREAM_UNROLL 4
#endif

// ---- Philox4x32-10 ---------------------------------------------------------------------------

__device__ __forceinline__ uint4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                               uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    const uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return make_uint4(c0, c1, c2, c3);
}

__device__ __forceinline__ float u24(uint32_t bits) { return (float)(bits >> 8) * 0x1p-24f; }

// ---- wave64 scans on the DPP network -----------------------------------------------------------

// x + (value of the lane selected by the DPP control, 0 where the control has no source lane or the
// row is masked off).
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_add(float x) {
  const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(x), kCtrl, kRowMask, 0xF, false);
  return x + __int_as_float(moved);
}

// Inclusive scan over the 64 lanes: Kogge-Stone inside each 16-lane row (row_shr 1,2,4,8), then
// row_bcast:15 into rows 1 and 3, then row_bcast:31 into rows 2 and 3.  The association order is part
// of the sampler's definition.
__device__ __forceinline__ float wave_scan(float x) {
  x = dpp_add<0x111, 0xF>(x);
  x = dpp_add<0x112, 0xF>(x);
  x = dpp_add<0x114, 0xF>(x);
  x = dpp_add<0x118, 0xF>(x);
  x = dpp_add<0x142, 0xA>(x);
  x = dpp_add<0x143, 0xC>(x);
  return x;
}

// Inclusive scan inside each 16-lane row only.
__device__ __forceinline__ float row_scan(float x) {
  x = dpp_add<0x111, 0xF>(x);
  x = dpp_add<0x112, 0xF>(x);
  x = dpp_add<0x114, 0xF>(x);
  x = dpp_add<0x118, 0xF>(x);
  return x;
}

__device__ __forceinline__ int lane_id() { return (int)__lane_id(); }

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
};

// include/gpu_graph.cuh:97-112
__device__ __forceinline__ bool sorted_contains(const int32_t* __restrict__ arr, int32_t size, int32_t target) {
  int32_t lo = 0, hi = size;
  while (lo < hi) {
    const int32_t mid = (int32_t)(((uint32_t)lo + (uint32_t)hi) >> 1);
    const int32_t v = arr[mid];
    if (v == target) return true;
    if (v < target) lo = mid + 1; else hi = mid;
  }
  return false;
}

// Per-lane reservoir state while a neighbour list streams by.
struct LaneState {
  float S = 0.0f;    // running sum of biases seen by this lane
  float Sj = 0.0f;   // running sum at the last acceptance
  float u = 1.0f;    // uniform that decides the next acceptance: first element with S * u > Sj
  // unread words of the lane's Philox stream, next one first; draw n of the stream is word n & 3 of
  // block n >> 2, and draw 0 is the lane's combine draw, so block 0 leaves three words for jumps
  uint32_t q0 = 0, q1 = 0, q2 = 0, q3 = 0;
  uint32_t avail = 0;  // unread words in the queue
  uint32_t blk = 0;    // index of the block the queue came from
  int32_t sel = -1;  // local index of the last accepted element
  int32_t selv = -1; // its vertex id (only tracked when the adjacency quartet is loaded alongside)
};

// Feeds one quartet (absolute CSR index base..base+3, raw 32-bit words of the bias array and, when
// needed, of the adjacency array) to the lane's reservoir.
template <int kApp, bool kTrackV>
__device__ __forceinline__ void consume_quartet(LaneState& st, const fw_kargs& a, const StepCtx& c, const int t,
                                                const uint32_t base, const bool edge, const uint32_t end, uint4 raw,
                                                int4 adj) {
  float w0, w1, w2, w3;
  if (kApp == FW_APP_METAPATH) {  // include/app.cuh:141-146
    w0 = (int32_t)raw.x == c.want ? 1.0f : 0.0f;
    w1 = (int32_t)raw.y == c.want ? 1.0f : 0.0f;
    w2 = (int32_t)raw.z == c.want ? 1.0f : 0.0f;
    w3 = (int32_t)raw.w == c.want ? 1.0f : 0.0f;
  } else {
    w0 = __uint_as_float(raw.x); w1 = __uint_as_float(raw.y);
    w2 = __uint_as_float(raw.z); w3 = __uint_as_float(raw.w);
  }
  if (edge) {  // head / tail quartet: entries outside [off, end) have no bias
    const bool in0 = base >= c.off && base < end;
    const bool in1 = base + 1u >= c.off && base + 1u < end;
    const bool in2 = base + 2u >= c.off && base + 2u < end;
    const bool in3 = base + 3u >= c.off && base + 3u < end;
    w0 = in0 ? w0 : 0.0f;
    w1 = in1 ? w1 : 0.0f;
    w2 = in2 ? w2 : 0.0f;
    w3 = in3 ? w3 : 0.0f;
    if (kApp == FW_APP_NODE2VEC) {  // never search for an entry of a foreign list
      adj.x = in0 ? adj.x : c.prev; adj.y = in1 ? adj.y : c.prev;
      adj.z = in2 ? adj.z : c.prev; adj.w = in3 ? adj.w : c.prev;
    }
  }
  if (kApp == FW_APP_NODE2VEC && c.prev != -1) {  // include/app.cuh:108-123
    const int32_t* __restrict__ plist = a.adjncy + c.prev_off;
    w0 = (adj.x == c.prev) ? w0 * a.inv_p : (sorted_contains(plist, c.prev_deg, adj.x) ? w0 : w0 * a.inv_q);
    w1 = (adj.y == c.prev) ? w1 * a.inv_p : (sorted_contains(plist, c.prev_deg, adj.y) ? w1 : w1 * a.inv_q);
    w2 = (adj.z == c.prev) ? w2 * a.inv_p : (sorted_contains(plist, c.prev_deg, adj.z) ? w2 : w2 * a.inv_q);
    w3 = (adj.w == c.prev) ? w3 * a.inv_p : (sorted_contains(plist, c.prev_deg, adj.w) ? w3 : w3 * a.inv_q);
  }

  const float s1 = st.S + w0;
  const float s2 = s1 + w1;
  const float s3 = s2 + w2;
  const float s4 = s3 + w3;
  // S is non-decreasing, so the next acceptance lies in this quartet iff it triggers at its end.
  if (s4 * st.u > st.Sj) {
#define FW_ELEM(sj_, vj_, j_)                                                                        \
  if ((sj_) * st.u > st.Sj) {                                                                        \
    st.sel = (int32_t)(base + (j_) - c.off);                                                         \
    if (kTrackV) st.selv = (vj_);                                                                    \
    st.Sj = (sj_);                                                                                   \
    if (st.avail == 0u) {                                                                            \
      ++st.blk;                                                                                      \
      const uint4 nb = philox4x32_10(c.walker, c.step, (uint32_t)t, st.blk, a.seed_lo, a.seed_hi);   \
      st.q0 = nb.x; st.q1 = nb.y; st.q2 = nb.z; st.q3 = nb.w;                                        \
      st.avail = 4u;                                                                                 \
    }                                                                                                \
    st.u = u24(st.q0);                                                                               \
    st.q0 = st.q1; st.q1 = st.q2; st.q2 = st.q3;                                                     \
    --st.avail;                                                                                      \
  }
    FW_ELEM(s1, adj.x, 0u)
    FW_ELEM(s2, adj.y, 1u)
    FW_ELEM(s3, adj.z, 2u)
    FW_ELEM(s4, adj.w, 3u)
#undef FW_ELEM
  }
  st.S = s4;
}

// Lane-local reservoir over quartets t, t+P, t+2P, ... of the neighbour list, kU quartets in flight.
// Outputs the lane total L, the lane's selected local index (or -1), the vertex behind it when
// kTrackV (the adjacency quartet is then loaded alongside), and the lane's combine draw.
template <int kApp, int kP, bool kTrackV, int kU>
__device__ __forceinline__ void lane_pass(const fw_kargs& a, const StepCtx& c, const int t, float& L, int32_t& sel,
                                          int32_t& selv, uint32_t& bern) {
  const uint32_t a0 = c.off & ~3u;
  const uint32_t end = c.off + (uint32_t)c.deg;
  const uint32_t nq = (end - a0 + 3u) >> 2;
  const uint32_t* __restrict__ bias =
      reinterpret_cast<const uint32_t*>(kApp == FW_APP_METAPATH ? (const void*)a.label : (const void*)a.weight);
  const bool need_adj = kTrackV || (kApp == FW_APP_NODE2VEC && c.prev != -1);

  LaneState st;
  bern = 0;
  if ((uint32_t)t < nq) {
    const uint4 b0 = philox4x32_10(c.walker, c.step, (uint32_t)t, 0u, a.seed_lo, a.seed_hi);
    bern = b0.x;
    st.q0 = b0.y; st.q1 = b0.z; st.q2 = b0.w;
    st.avail = 3u;
  }

  uint32_t k = (uint32_t)t;
  if (kU > 1) {
    // all kU quartets of the group exist for this lane: issue the loads together, then consume in order
    for (; k + (uint32_t)((kU - 1) * kP) < nq; k += (uint32_t)(kU * kP)) {
      uint4 raw[kU];
      int4 adj[kU];
#pragma unroll
      for (int j = 0; j < kU; ++j) {
        const uint32_t base = a0 + 4u * (k + (uint32_t)(j * kP));
        raw[j] = *reinterpret_cast<const uint4*>(bias + base);
        adj[j] = make_int4(-1, -1, -1, -1);
        if (need_adj) adj[j] = *reinterpret_cast<const int4*>(a.adjncy + base);
      }
#pragma unroll
      for (int j = 0; j < kU; ++j) {
        const uint32_t kk = k + (uint32_t)(j * kP);
        consume_quartet<kApp, kTrackV>(st, a, c, t, a0 + 4u * kk, kk == 0u || kk == nq - 1u, end, raw[j], adj[j]);
      }
    }
  }
  for (; k < nq; k += (uint32_t)kP) {
    const uint32_t base = a0 + 4u * k;
    const uint4 raw = *reinterpret_cast<const uint4*>(bias + base);
    int4 adj = make_int4(-1, -1, -1, -1);
    if (need_adj) adj = *reinterpret_cast<const int4*>(a.adjncy + base);
    consume_quartet<kApp, kTrackV>(st, a, c, t, base, k == 0u || k == nq - 1u, end, raw, adj);
  }
  L = st.S;
  sel = st.sel;
  selv = st.selv;
}

// Combines the 64 lane reservoirs of one wave: lane l is accepted iff L > 0 and bern * prefix < L;
// the last accepted lane wins (include/sampler.cuh:82-84 takes the max over lane-tagged keys).
// Returns the winning lane or -1; W = wave total.
__device__ __forceinline__ int wave_combine(float L, uint32_t bern, float& W) {
  const float I = wave_scan(L);
  const bool acc = (L > 0.0f) && (u24(bern) * I < L);
  const uint64_t m = __ballot(acc);
  W = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(I), 63));
  if (m == 0ull) return -1;
  return 63 - __builtin_clzll(m);
}

// ---- LDS task table ----------------------------------------------------------------------------

template <int kWGT>
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
  // per-round work lists, double buffered by round parity
  int32_t small_list[2][kWGT];
  int32_t hub_list[2][kWGT];
  int32_t small_count[2];
  int32_t hub_count[2];
  int32_t claim[2];
  int32_t exhausted;
  // wave partials of the hub chunk in flight
  float hub_w[kHubChunk][16];
  int32_t hub_sel[kHubChunk][16];
};

template <int kWGT>
__device__ __forceinline__ StepCtx load_ctx(const fw_kargs& a, const TaskTable<kWGT>& tt, int slot) {
  StepCtx c;
  c.off = tt.off[slot];
  c.deg = tt.deg[slot];
  c.prev = tt.prev[slot];
  c.prev_off = tt.prev_off[slot];
  c.prev_deg = tt.prev_deg[slot];
  c.walker = a.walker_base + (uint32_t)tt.walker[slot];
  c.step = (uint32_t)(tt.len[slot] - 1);
  c.want = 0;
  return c;
}

// Step commit by one lane: include/walker.cuh:1372-1385 and Task::update (include/gpu_task.cuh:70-77).
// The CSR range of the new vertex is reloaded in phase C by the slot's own thread.
template <int kWGT>
__device__ __forceinline__ void commit(const fw_kargs& a, TaskTable<kWGT>& tt, int slot, const StepCtx& c, int32_t v,
                                       bool ok, unsigned long long& n_steps, unsigned long long& n_edges) {
  if (!ok) {
    tt.flag[slot] = kFlagDead;
    return;
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

// ---- the kernel --------------------------------------------------------------------------------

template <int kApp, int kWGT>
__global__ __launch_bounds__(kWGT) void fw_walk_zprs(const fw_kargs a) {
  constexpr int kNW = kWGT / 64;
  // quartets in flight per lane while streaming; node2vec is bound by its adjacency probes instead
  constexpr int kUnroll = (kApp == FW_APP_NODE2VEC) ? 1 : FW_STREAM_UNROLL;
  __shared__ TaskTable<kWGT> tt;

  const int tid = (int)threadIdx.x;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  unsigned long long n_steps = 0ull, n_edges = 0ull;

  tt.len[tid] = -1;
  tt.flag[tid] = 0;
  if (tid == 0) {
    tt.small_count[0] = tt.small_count[1] = 0;
    tt.hub_count[0] = tt.hub_count[1] = 0;
    tt.claim[0] = tt.claim[1] = 0;
    tt.exhausted = 0;
  }
  __syncthreads();

  int parity = 0;  // lists[parity] are consumed this round, lists[parity ^ 1] are produced by phase C
  bool first = true;
  for (;;) {
    if (!first) {
      const int nh = tt.hub_count[parity];
      const int ns = tt.small_count[parity];
      if (nh + ns == 0) break;  // uniform: read after the barrier that closed phase C

      // ---- phase B: hubs, whole workgroup ----
      for (int hb = 0; hb < nh; hb += kHubChunk) {
        const int cnt = min(kHubChunk, nh - hb);
        for (int h = 0; h < cnt; ++h) {
          const int slot = tt.hub_list[parity][hb + h];
          StepCtx c = load_ctx(a, tt, slot);
          if (kApp == FW_APP_METAPATH) c.want = a.schema[c.step % (uint32_t)a.schema_len];
          float L, W;
          int32_t sel, selv;
          uint32_t bern;
          lane_pass<kApp, kWGT, false, kUnroll>(a, c, tid, L, sel, selv, bern);
          const int win = wave_combine(L, bern, W);
          const int32_t wsel = (win >= 0) ? __builtin_amdgcn_readlane(sel, win) : -1;
          if (lane == 0) {
            tt.hub_w[h][wave] = W;
            tt.hub_sel[h][wave] = wsel;
          }
        }
        __syncthreads();
        for (int h = wave; h < cnt; h += kNW) {
          const int slot = tt.hub_list[parity][hb + h];
          const StepCtx c = load_ctx(a, tt, slot);
          float W = 0.0f;
          int32_t s = -1;
          uint32_t bits = 0;
          if (lane < kNW) {
            W = tt.hub_w[h][lane];
            s = tt.hub_sel[h][lane];
            bits = philox4x32_10(c.walker, c.step, kStreamWave | (uint32_t)lane, 0u, a.seed_lo, a.seed_hi).x;
          }
          const float J = row_scan(W);
          const bool acc = (lane < kNW) && (W > 0.0f) && (u24(bits) * J < W);
          const uint64_t m = __ballot(acc);
          int32_t pick = -1;
          if (m != 0ull) pick = __builtin_amdgcn_readlane(s, 63 - __builtin_clzll(m));
          if (lane == 0) {
            int32_t v = -1;
            if (pick >= 0) v = a.adjncy[c.off + (uint32_t)pick];
            commit(a, tt, slot, c, v, pick >= 0, n_steps, n_edges);
          }
        }
        if (hb + kHubChunk < nh) __syncthreads();  // the partial buffers are reused by the next chunk
      }

      // ---- phase A: remaining slots, one wave each, claimed dynamically ----
      for (;;) {
        int idx = 0;
        if (lane == 0) idx = atomicAdd(&tt.claim[parity], 1);
        idx = __builtin_amdgcn_readfirstlane(idx);
        if (idx >= ns) break;
        const int slot = tt.small_list[parity][idx];
        StepCtx c = load_ctx(a, tt, slot);
        if (kApp == FW_APP_METAPATH) c.want = a.schema[c.step % (uint32_t)a.schema_len];
        float L, W;
        int32_t sel, selv;
        uint32_t bern;
        const uint32_t nq = ((c.off + (uint32_t)c.deg) - (c.off & ~3u) + 3u) >> 2;
        int win;
        int32_t v = -1;
        if (nq <= 64u) {  // one quartet per lane: fetch the adjacency with the weights, no dependent load
          lane_pass<kApp, 64, true, 1>(a, c, lane, L, sel, selv, bern);
          win = wave_combine(L, bern, W);
          if (win >= 0) v = __builtin_amdgcn_readlane(selv, win);
        } else {
          lane_pass<kApp, 64, false, kUnroll>(a, c, lane, L, sel, selv, bern);
          win = wave_combine(L, bern, W);
          if (win >= 0) {
            const int32_t pick = __builtin_amdgcn_readlane(sel, win);
            v = a.adjncy[c.off + (uint32_t)pick];
          }
        }
        if (lane == 0) commit(a, tt, slot, c, v, win >= 0, n_steps, n_edges);
      }
      __syncthreads();
      if (tid == 0) {  // this round's lists are drained; they become the lists produced two rounds later
        tt.small_count[parity] = 0;
        tt.hub_count[parity] = 0;
        tt.claim[parity] = 0;
      }
      parity ^= 1;
    }

    // ---- phase C: one thread per slot (include/walker.cuh:1421-1432; Task::init/update) ----
    {
      const int np = first ? 0 : parity;  // lists to fill for the next round
      first = false;
      int32_t len = tt.len[tid];
      bool need = true;  // slot wants a new query
      int32_t deg = 0;
      if (len >= 0) {
        if (tt.flag[tid] == kFlagMoved) {
          const int32_t v = tt.cur[tid];
          const uint32_t o = a.xadj[v];
          const uint32_t e = a.xadj[v + 1];
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
        }
        // kFlagDead: dead end (no neighbour with positive bias), include/walker.cuh:1373-1374
      }
      bool exhausted = tt.exhausted != 0;
      for (;;) {
        const bool want = need && !exhausted;
        const uint64_t m = __ballot(want);
        if (m == 0ull) break;
        uint32_t base = 0;
        const int leader = __builtin_ctzll(m);
        if (lane == leader) base = atomicAdd(a.dispenser, (uint32_t)__builtin_popcountll(m));
        base = (uint32_t)__builtin_amdgcn_readlane((int)base, leader);
        if (want) {
          const uint32_t q = base + (uint32_t)__builtin_popcountll(m & ((1ull << lane) - 1ull));
          if (q < (uint32_t)a.n) {
            const int32_t sp = a.starts[q];
            a.paths[(uint64_t)q * (uint64_t)a.max_depth] = sp;  // include/walker.cuh:1342
            if ((uint32_t)sp < (uint32_t)a.V && a.max_depth > 1) {
              const uint32_t o = a.xadj[sp];
              const uint32_t e = a.xadj[sp + 1];
              deg = (int32_t)(e - o);
              if (deg > 0) {
                tt.walker[tid] = (int32_t)q;
                tt.cur[tid] = sp;
                tt.prev[tid] = -1;
                tt.off[tid] = o;
                tt.deg[tid] = deg;
                tt.prev_off[tid] = 0;
                tt.prev_deg[tid] = 0;
                len = 1;
                need = false;
              }
            }
          } else {
            exhausted = true;
            tt.exhausted = 1;
          }
        }
      }
      if (need) {
        tt.len[tid] = -1;
      } else {
        tt.len[tid] = len;
        tt.flag[tid] = 0;
        if (deg > a.hub_threshold) {
          tt.hub_list[np][atomicAdd(&tt.hub_count[np], 1)] = tid;
        } else {
          tt.small_list[np][atomicAdd(&tt.small_count[np], 1)] = tid;
        }
      }
      parity = np;
    }
    __syncthreads();
  }

  if (n_steps != 0ull) {
    atomicAdd(&a.counters[0], n_steps);
    atomicAdd(&a.counters[1], n_edges);
  }
}

template <int kApp, int kWGT>
int launch_one(const fw_kargs& a, int grid, hipStream_t stream, int* grid_used) {
  if (grid <= 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    FW_HIP(hipGetDevice(&dev));
    FW_HIP(hipGetDeviceProperties(&prop, dev));
    int per_cu = 0;
    FW_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fw_walk_zprs<kApp, kWGT>, kWGT, 0));
    if (per_cu < 1) per_cu = 1;
    grid = prop.multiProcessorCount * per_cu;
  }
  // no more workgroups than there are slots to fill
  const long long max_useful = ((long long)a.n + kWGT - 1) / kWGT;
  if ((long long)grid > max_useful) grid = (int)(max_useful > 0 ? max_useful : 1);
  hipLaunchKernelGGL((fw_walk_zprs<kApp, kWGT>), dim3(grid), dim3(kWGT), 0, stream, a);
  FW_HIP(hipGetLastError());
  if (grid_used) *grid_used = grid;
  return FW_OK;
}

template <int kApp>
int launch_app(const fw_kargs& a, int wg_threads, int grid, hipStream_t stream, int* grid_used) {
  switch (wg_threads) {
    case 256: return launch_one<kApp, 256>(a, grid, stream, grid_used);
    case 512: return launch_one<kApp, 512>(a, grid, stream, grid_used);
    case 1024: return launch_one<kApp, 1024>(a, grid, stream, grid_used);
    default:
      fw_set_error("wg_threads must be 256, 512 or 1024 (got %d)", wg_threads);
      return FW_ERR_INVALID;
  }
}

}  // namespace

int fw_launch_walk(const fw_kargs& a, int app, int sampler, int wg_threads, int grid, hipStream_t stream,
                   int* grid_used) {
  if (sampler != FW_SAMPLER_ZPRS) {
    fw_set_error("sampler %d is not available in this build", sampler);
    return FW_ERR_INVALID;
  }
  switch (app) {
    case FW_APP_DEEPWALK: return launch_app<FW_APP_DEEPWALK>(a, wg_threads, grid, stream, grid_used);
    case FW_APP_PPR: return launch_app<FW_APP_PPR>(a, wg_threads, grid, stream, grid_used);
    case FW_APP_NODE2VEC: return launch_app<FW_APP_NODE2VEC>(a, wg_threads, grid, stream, grid_used);
    case FW_APP_METAPATH: return launch_app<FW_APP_METAPATH>(a, wg_threads, grid, stream, grid_used);
    default:
      fw_set_error("unknown app %d", app);
      return FW_ERR_INVALID;
  }
}
