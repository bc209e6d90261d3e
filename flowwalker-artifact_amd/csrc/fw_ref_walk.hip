// The reference's own walk engine, restated for 64-lane wavefronts: ablation baseline and micro-benchmark column.
//
// fw_walk_zprs (fw_walk_kernel.hip) samples with a different algorithm than the reference.  This file keeps the
// reference's algorithm itself runnable on gfx950 so that the two can be measured side by side on the same lists:
//   * walker_wb_dynamic_zprs / _dprs (include/walker.cuh:1307-1580): 64 task slots per workgroup, every wave steps
//     its slots with the wave sampler, slots above the threshold are deferred and stepped by the whole workgroup,
//     then threads 0..63 apply the stop rule and claim the next query;
//   * static query assignment (init_taskassignment, src/walk.cu:46-61; walker_wb, include/walker.cuh:170) or the
//     global dispenser (include/walker.cuh:1339, :1423);
//   * sampler_warp / sampler_block (ZPRS, include/sampler.cuh:46-127): two passes over lane-strided elements, one
//     uniform per neighbour with positive bias, accept `u < w / S`, 64-bit key `i + size * lane`, max-reduce;
//   * sampler_warp_oneloop / sampler_block_oneloop (DPRS, include/sampler.cuh:129-200): one pass in chunks of the
//     group's width, inclusive scan + carry, running maximum of the accepted indices;
//   * the functors of include/app.cuh:58-152, node2vec with one binary search per neighbour
//     (include/gpu_graph.cuh:97-118).
// What is this build's and not the reference's: 64 lanes per wave (the scans are the DPP network of fw_device_util.h),
// workgroups of wg_threads, and the random numbers: Philox4x32-10, the uniform of element i of a list sampled by a
// group of W lanes at (walker, step) is word j & 3 of block (j >> 2) * W + t of stream kStreamRef, t = i % W,
// j = i / W, mapped to (0, 1] as cuRAND's uniforms are (include/myrand.cuh:213-215).  Walks are therefore a function
// of (seed, walker id, graph, parameters) and can be compared bit for bit with a CPU restatement.
//
// Thread-owned generators (FW_SAMPLER_REF_RNG_LDS / _GLOBAL, static assignment only).  The reference's ablation
// (README.md:152-163) starts from generators that belong to the threads: cuRAND states in device memory, read and
// written around every draw (walker_wb_dprs_curand, include/walker.cuh:1584-1696, `state + gid`), then its own
// generator with the states of a block in shared memory, structure of arrays (include/myrand.cuh:83-86, :174-186;
// walker_wb_dprs, include/walker.cuh:1813).  Both are restated here with one generator: thread `gid` (global thread id,
// the reference's sequence number, include/myrand.cuh:271-292) draws word n & 3 of Philox block n >> 2 of its own
// stream (counter (gid, n >> 2, kStreamThread, 0)) as its n-th uniform, whatever list it is working on; the state (the
// current block and n) lives in LDS or in device memory.  With static assignment every step of the launch is a
// function of (seed, grid, wg_threads, queries): slots take their queries in slot order, deferred lists are stepped in
// slot order, so the CPU restatement replays a workgroup thread by thread and the walks compare bit for bit.  Both
// placements give the same walks; they differ in what a draw costs.

#include "fw_internal.h"
#include "fw_device_util.h"

namespace {

constexpr uint32_t kStreamRef = 0x20000000u;
constexpr uint32_t kStreamThread = 0x08000000u;   // thread-owned generators: counter (gid, block, kStreamThread, 0)
constexpr uint32_t kStreamStopRef = 0x80000000u;  // PPR stop draw: the same stream the walk kernel uses
constexpr int kRefTasks = 64;                      // TASK_NUM, include/walker.cuh:28

__device__ __forceinline__ float ref_u(uint32_t bits) { return (float)((bits >> 8) + 1u) * 0x1p-24f; }

// max over the wave of a per-lane 64-bit key (the reference's warpReduceMax on `ll`, include/util.cuh:104-109)
__device__ __forceinline__ long long wave_max_i64(long long v) {
  constexpr int kHiMin = (int)0x80000000;
#define FW_STEP(ctrl, rowmask)                                                                          \
  {                                                                                                     \
    const int hi = __builtin_amdgcn_update_dpp(kHiMin, (int)(v >> 32), ctrl, rowmask, 0xF, false);      \
    const int lo = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)v, ctrl, rowmask, 0xF, false);         \
    const long long o = (long long)(((unsigned long long)(uint32_t)hi << 32) | (uint32_t)lo);           \
    v = o > v ? o : v;                                                                                  \
  }
  FW_STEP(0x111, 0xF)
  FW_STEP(0x112, 0xF)
  FW_STEP(0x114, 0xF)
  FW_STEP(0x118, 0xF)
  FW_STEP(0x142, 0xA)
  FW_STEP(0x143, 0xC)
#undef FW_STEP
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, 63);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(v >> 32), 63);
  return (long long)(((unsigned long long)hi << 32) | lo);
}

// What a sampling step needs to know about its slot (wave- or workgroup-uniform).
struct RefStep {
  uint32_t off;
  int32_t deg;
  int32_t prev;
  uint32_t prev_off;
  int32_t prev_deg;
  int32_t want;
  uint32_t walker, step;
};

// include/gpu_graph.cuh:97-112
__device__ __forceinline__ bool ref_contains(const int32_t* __restrict__ arr, int32_t size, int32_t target) {
  int32_t l = 0, r = size - 1;
  while (l <= r) {
    const int32_t m = l + (r - l) / 2;
    const int32_t x = arr[m];
    if (x == target) return true;
    if (x < target) l = m + 1; else r = m - 1;
  }
  return false;
}

// App::get_weight (include/app.cuh:64-66, :86-88, :108-123, :141-146); node2vec multiplies by the reciprocals the
// host computed, as the rest of this library does
template <int kApp>
__device__ __forceinline__ float ref_bias(const fw_kargs& a, const RefStep& s, uint32_t i) {
  const uint32_t e = s.off + i;
  if (kApp == FW_APP_METAPATH) return a.label[e] == s.want ? 1.0f : 0.0f;
  const float w = a.weight[e];
  if (kApp == FW_APP_NODE2VEC && s.prev != -1) {
    const int32_t post = a.adjncy[e];
    if (post == s.prev) return w * a.inv_p;
    if (!ref_contains(a.adjncy + s.prev_off, s.prev_deg, post)) return w * a.inv_q;
  }
  return w;
}

// State of a thread-owned generator in device memory (the place of cuRAND's `state + gid`).
struct RefThreadState {
  uint32_t w[4];
  uint32_t n;
  uint32_t pad[3];
};

// Where the calling thread's generator lives (kRng 1: LDS, structure of arrays; 2: device memory).
struct RefRng {
  uint32_t* lds_w;  // [4][blockDim.x]
  uint32_t* lds_n;  // [blockDim.x]
  RefThreadState* dev;  // this thread's state
  uint32_t tid, threads, gid;
};

// kRng 0: the uniforms of one lane of a group of W lanes, its j-th element takes word j & 3 of block (j >> 2) * W + t.
// kRng 1 / 2: the thread's own generator, its draws one after the other.
template <int kRng>
struct RefDraws {
  uint4 blk;
  __device__ __forceinline__ float next(const fw_kargs& a, const RefStep& s, const RefRng& r, uint32_t W, uint32_t t,
                                        uint32_t j) {
    if (kRng == 0) {
      if ((j & 3u) == 0u) blk = philox4x32_10(s.walker, s.step, kStreamRef, (j >> 2) * W + t, a.seed_lo, a.seed_hi);
      const uint32_t k = j & 3u;
      const uint32_t bits = k == 0u ? blk.x : (k == 1u ? blk.y : (k == 2u ? blk.z : blk.w));
      return ref_u(bits);
    }
    uint32_t bits;
    if (kRng == 1) {
      const uint32_t n = r.lds_n[r.tid];
      if ((n & 3u) == 0u) {
        const uint4 b = philox4x32_10(r.gid, n >> 2, kStreamThread, 0u, a.seed_lo, a.seed_hi);
        r.lds_w[0u * r.threads + r.tid] = b.x;
        r.lds_w[1u * r.threads + r.tid] = b.y;
        r.lds_w[2u * r.threads + r.tid] = b.z;
        r.lds_w[3u * r.threads + r.tid] = b.w;
      }
      bits = r.lds_w[(n & 3u) * r.threads + r.tid];
      r.lds_n[r.tid] = n + 1u;
    } else {
      volatile RefThreadState* st = r.dev;  // every draw goes to memory and back, as a cuRAND state does
      const uint32_t n = st->n;
      if ((n & 3u) == 0u) {
        const uint4 b = philox4x32_10(r.gid, n >> 2, kStreamThread, 0u, a.seed_lo, a.seed_hi);
        st->w[0] = b.x;
        st->w[1] = b.y;
        st->w[2] = b.z;
        st->w[3] = b.w;
      }
      bits = st->w[n & 3u];
      st->n = n + 1u;
    }
    return ref_u(bits);
  }
};

// sampler_warp (include/sampler.cuh:46-85) for a 64-lane wave
template <int kApp, int kRng>
__device__ __forceinline__ int32_t ref_zprs_wave(const fw_kargs& a, const RefStep& s, const RefRng& r, const int lane) {
  const uint32_t deg = (uint32_t)s.deg;
  float L = 0.0f;
  for (uint32_t i = (uint32_t)lane; i < deg; i += 64u) L += ref_bias<kApp>(a, s, i);  // :56-59
  const float I = wave_scan(L);                                                       // :62-66
  float S = I - L;                                                                    // :68
  long long key = -1;
  RefDraws<kRng> d;
  uint32_t j = 0u;
  for (uint32_t i = (uint32_t)lane; i < deg; i += 64u, ++j) {  // :70-80
    const float w = ref_bias<kApp>(a, s, i);
    S += w;
    const float u = d.next(a, s, r, 64u, (uint32_t)lane, j);
    if (w > 0.0f) {
      if (key == -1) key = 0;
      if (u < w / S) key = (long long)i + (long long)deg * (long long)lane;
    }
  }
  key = wave_max_i64(key);                                   // :82
  return key == -1 ? -1 : (int32_t)(key % (long long)deg);   // :84
}

// sampler_warp_oneloop (include/sampler.cuh:129-155) for a 64-lane wave
template <int kApp, int kRng>
__device__ __forceinline__ int32_t ref_dprs_wave(const fw_kargs& a, const RefStep& s, const RefRng& r, const int lane) {
  const uint32_t deg = (uint32_t)s.deg;
  if (deg == 0u) return -1;
  float carry = 0.0f;
  int32_t sel = -1;
  RefDraws<kRng> d;
  const uint64_t bound = (uint64_t)deg + 64u - deg % 64u;  // :138
  uint32_t j = 0u;
  for (uint64_t base = 0; base < bound; base += 64u, ++j) {
    const uint64_t i = base + (uint64_t)lane;
    const float x = i < deg ? ref_bias<kApp>(a, s, (uint32_t)i) : 0.0f;
    if (x > 0.0f && sel == -1) sel = 0;                        // :142
    const float Sl = carry + wave_scan(x);                     // :143-149
    const float u = d.next(a, s, r, 64u, (uint32_t)lane, j);
    if (i < deg && x > 0.0f && u < x / Sl) sel = (int32_t)i;   // :150
    carry = readlane_f(Sl, 63);                                // :151
    sel = wave_max_i32(sel);                                   // :152
  }
  return sel;
}

// Scratch of the workgroup samplers.
struct RefBlockScratch {
  float tot[16];
  long long key[16];
};

// sampler_block (include/sampler.cuh:87-127) for a workgroup of W = blockDim.x threads.  The exclusive prefix over the
// threads' totals is: wave scan inside each wave, the waves' totals added up one after the other, minus the thread's
// own total (the reference's cub::BlockScan has no documented association).
template <int kApp, int kRng>
__device__ __forceinline__ int32_t ref_zprs_block(const fw_kargs& a, const RefStep& s, const RefRng& r, RefBlockScratch& scr,
                                                  const int tid, const int lane, const int wave, const int nw) {
  const uint32_t deg = (uint32_t)s.deg;
  const uint32_t W = (uint32_t)nw * 64u;
  float L = 0.0f;
  for (uint32_t i = (uint32_t)tid; i < deg; i += W) L += ref_bias<kApp>(a, s, i);  // :96-99
  const float I = wave_scan(L);
  if (lane == 63) scr.tot[wave] = I;
  __syncthreads();
  float off = 0.0f;
  for (int v = 0; v < wave; ++v) off = off + scr.tot[v];
  float S = (off + I) - L;  // :102-104
  long long key = -1;
  RefDraws<kRng> d;
  uint32_t j = 0u;
  for (uint32_t i = (uint32_t)tid; i < deg; i += W, ++j) {  // :106-116
    const float w = ref_bias<kApp>(a, s, i);
    S += w;
    const float u = d.next(a, s, r, W, (uint32_t)tid, j);
    if (w > 0.0f) {
      if (key == -1) key = 0;
      if (u < w / S) key = (long long)i + (long long)deg * (long long)tid;
    }
  }
  key = wave_max_i64(key);
  if (lane == 0) scr.key[wave] = key;
  __syncthreads();  // :121
  long long best = -1;
  for (int v = 0; v < nw; ++v) best = scr.key[v] > best ? scr.key[v] : best;  // (kept 64-bit: :118-124 truncates to 32)
  __syncthreads();  // :124: the scratch is reused by the next list
  return best == -1 ? -1 : (int32_t)(best % (long long)deg);
}

// sampler_block_oneloop (include/sampler.cuh:157-200) for a workgroup of W = blockDim.x threads
template <int kApp, int kRng>
__device__ __forceinline__ int32_t ref_dprs_block(const fw_kargs& a, const RefStep& s, const RefRng& r, RefBlockScratch& scr,
                                                  const int tid, const int lane, const int wave, const int nw) {
  const uint32_t deg = (uint32_t)s.deg;
  if (deg == 0u) return -1;
  const uint32_t W = (uint32_t)nw * 64u;
  float carry = 0.0f;  // prefix_sum, :163-164
  int32_t sel = -1;
  RefDraws<kRng> d;
  const uint64_t bound = (uint64_t)deg + W - deg % W;  // :167
  uint32_t j = 0u;
  for (uint64_t base = 0; base < bound; base += W, ++j) {
    const uint64_t i = base + (uint64_t)tid;
    const float x = i < deg ? ref_bias<kApp>(a, s, (uint32_t)i) : 0.0f;
    const float I = wave_scan(x);  // :175-178
    if (lane == 63) scr.tot[wave] = I;
    __syncthreads();
    float off = carry;
    for (int v = 0; v < wave; ++v) off = off + scr.tot[v];
    float next_carry = carry;
    for (int v = 0; v < nw; ++v) next_carry = next_carry + scr.tot[v];  // :194-196
    const float Sl = off + I;
    int32_t local = -1;
    const float u = d.next(a, s, r, W, (uint32_t)tid, j);
    if (x > 0.0f && i < deg) {  // :181-184
      local = 0;
      if (u < x / Sl) local = (int32_t)i;
    }
    local = wave_max_i32(local);
    if (lane == 0) scr.key[wave] = (long long)local;
    __syncthreads();
    int32_t m = -1;
    for (int v = 0; v < nw; ++v) m = (int32_t)scr.key[v] > m ? (int32_t)scr.key[v] : m;
    sel = m > sel ? m : sel;  // :190-192
    carry = next_carry;
    __syncthreads();  // :197
  }
  return sel;
}

// walker_wb_dynamic_zprs / _dprs (include/walker.cuh:1307-1580) and their statically assigned forms.
// kRng: 0 = every draw addressed by (walker, step, element); 1 / 2 = thread-owned generators with their state in LDS /
// in device memory (rng_dev, one RefThreadState per thread of the grid), static assignment only.
template <int kApp, bool kDprs, int kRng>
__global__ __launch_bounds__(1024) void fw_walk_ref(const fw_kargs a, const int static_assignment, RefThreadState* rng_dev) {
  static_assert(kRefTasks == 64, "the task slots are claimed and refilled by the lanes of wave 0");
  __shared__ int32_t t_walker[kRefTasks], t_cur[kRefTasks], t_prev[kRefTasks], t_len[kRefTasks], t_deg[kRefTasks];
  __shared__ int32_t t_prev_deg[kRefTasks], t_moved[kRefTasks];
  __shared__ uint32_t t_off[kRefTasks], t_prev_off[kRefTasks];
  __shared__ int32_t is_large[kRefTasks];
  __shared__ int32_t num_active;
  __shared__ uint32_t s_cursor;
  __shared__ int32_t s_schema[kApp == FW_APP_METAPATH ? FW_MAX_SCHEMA : 1];
  __shared__ RefBlockScratch scr;
  __shared__ unsigned long long s_acc[2];
  __shared__ uint32_t s_rng_w[kRng == 1 ? 4 * 1024 : 1];  // include/myrand.cuh:83-86: the block's states, structure of arrays
  __shared__ uint32_t s_rng_n[kRng == 1 ? 1024 : 1];

  const int tid = (int)threadIdx.x;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nw = (int)(blockDim.x >> 6);
  // static assignment: an even split of the queries over the workgroups (src/walk.cu:46-61)
  const uint32_t n = (uint32_t)a.n;
  const uint32_t per = (n + gridDim.x - 1u) / gridDim.x;
  const uint32_t lo = blockIdx.x * per < n ? blockIdx.x * per : n;
  const uint32_t hi = lo + per < n ? lo + per : n;

  RefRng rng;
  rng.lds_w = s_rng_w;
  rng.lds_n = s_rng_n;
  rng.tid = (uint32_t)tid;
  rng.threads = blockDim.x;
  rng.gid = blockIdx.x * blockDim.x + (uint32_t)tid;
  rng.dev = kRng == 2 ? rng_dev + rng.gid : nullptr;
  if (kRng == 1) s_rng_n[tid] = 0u;  // myrand_init (include/myrand.cuh:271-292): sequence = global thread id
  if (kRng == 2) rng.dev->n = 0u;    // curand_init(1337, gid, 0, state + gid), include/walker.cuh:1597

  if (tid == 0) {
    num_active = kRefTasks;
    s_cursor = 0u;
    s_acc[0] = s_acc[1] = 0ull;
  }
  if (tid < kRefTasks) {
    t_len[tid] = -1;
    is_large[tid] = 0;
  }
  if (kApp == FW_APP_METAPATH && tid == 0) {
#pragma unroll
    for (int i = 0; i < FW_MAX_SCHEMA; ++i) s_schema[i] = a.schema[i];
  }
  __syncthreads();

  // Wave 0, all lanes: the slots with `want` take the next queries (include/walker.cuh:1339, :1423), in slot order --
  // the lowest slot gets the lowest query, so that a statically assigned launch is the same every time it runs.
  // Task::init (include/gpu_task.cuh:52-68), include/walker.cuh:1340-1349.
  auto refill = [&](bool want) {
    const uint64_t m = __ballot(want);
    if (m == 0ull) return;
    const uint32_t rank = (uint32_t)__builtin_popcountll(m & ((1ull << lane) - 1ull));
    const uint32_t cnt = (uint32_t)__builtin_popcountll(m);
    uint32_t base = 0u;
    if (static_assignment) {
      base = s_cursor;  // only wave 0 touches it
      if (lane == 0) s_cursor = base + cnt;
    } else {
      if (lane == __builtin_ctzll(m)) base = atomicAdd(a.dispenser, cnt);
      base = (uint32_t)__builtin_amdgcn_readlane((int)base, __builtin_ctzll(m));
    }
    if (!want) return;
    const uint32_t q = static_assignment ? lo + base + rank : base + rank;
    const int slot = tid;
    if (q >= (static_assignment ? hi : n)) {
      t_len[slot] = -1;
      atomicSub(&num_active, 1);
      return;
    }
    const int32_t start = a.starts[q];
    a.paths[(uint64_t)q * (uint64_t)a.max_depth] = start;
    t_walker[slot] = (int32_t)q;
    t_cur[slot] = start;
    t_prev[slot] = -1;
    t_prev_off[slot] = 0u;
    t_prev_deg[slot] = 0;
    t_moved[slot] = 0;
    if ((uint32_t)start < (uint32_t)a.V) {
      const uint32_t o = a.xadj[start];
      t_off[slot] = o;
      t_deg[slot] = (int32_t)(a.xadj[start + 1] - o);
      t_len[slot] = 1;
    } else {  // not a vertex: the walk is its start entry
      t_off[slot] = 0u;
      t_deg[slot] = 0;
      t_len[slot] = a.max_depth;
    }
  };
  if (wave == 0) refill(true);
  __syncthreads();

  unsigned long long n_steps = 0ull, n_edges = 0ull;
  auto load_step = [&](int slot) -> RefStep {
    RefStep s;
    s.off = t_off[slot];
    s.deg = t_deg[slot];
    s.prev = t_prev[slot];
    s.prev_off = t_prev_off[slot];
    s.prev_deg = t_prev_deg[slot];
    s.walker = a.walker_base + (uint32_t)t_walker[slot];
    s.step = (uint32_t)(t_len[slot] - 1);
    s.want = kApp == FW_APP_METAPATH ? s_schema[s.step % (uint32_t)a.schema_len] : 0;
    return s;
  };
  // include/walker.cuh:1372-1385 and Task::update (include/gpu_task.cuh:70-77), by one thread
  auto commit = [&](int slot, const RefStep& s, int32_t sel) {
    if (sel == -1) {
      t_len[slot] = a.max_depth;  // :1373-1374
      t_moved[slot] = 0;
      return;
    }
    const int32_t v = a.adjncy[s.off + (uint32_t)sel];
    const int32_t len = t_len[slot];
    a.paths[(uint64_t)(uint32_t)t_walker[slot] * (uint64_t)a.max_depth + (uint64_t)len] = v;
    t_prev[slot] = t_cur[slot];
    t_prev_off[slot] = s.off;
    t_prev_deg[slot] = s.deg;
    t_cur[slot] = v;
    const uint32_t o = a.xadj[v];
    t_off[slot] = o;
    t_deg[slot] = (int32_t)(a.xadj[v + 1] - o);
    t_len[slot] = len + 1;
    t_moved[slot] = 1;
    n_steps += 1ull;
    n_edges += (unsigned long long)(uint32_t)s.deg;
  };

  while (num_active > 0) {  // :1357 (read after a barrier)
    for (int slot = wave; slot < kRefTasks; slot += nw) {  // :1358
      if (t_len[slot] < 0 || t_len[slot] >= a.max_depth) continue;
      const RefStep s = load_step(slot);
      if (s.deg <= a.hub_threshold) {  // :1362
        const int32_t sel = kDprs ? ref_dprs_wave<kApp, kRng>(a, s, rng, lane) : ref_zprs_wave<kApp, kRng>(a, s, rng, lane);
        if (lane == 0) commit(slot, s, sel);
      } else if (lane == 0) {
        is_large[slot] = 1;  // :1386-1391 (a flag per slot instead of a list: the deferred lists are stepped in slot order)
      }
    }
    __syncthreads();  // :1395
    for (int slot = 0; slot < kRefTasks; ++slot) {  // :1397-1419
      if (is_large[slot] == 0) continue;  // uniform in the workgroup
      const RefStep s = load_step(slot);
      const int32_t sel = kDprs ? ref_dprs_block<kApp, kRng>(a, s, rng, scr, tid, lane, wave, nw)
                                : ref_zprs_block<kApp, kRng>(a, s, rng, scr, tid, lane, wave, nw);
      if (tid == 0) commit(slot, s, sel);
    }
    __syncthreads();
    if (wave == 0) {  // :1422-1432, on live slots only
      bool stop = false;
      if (t_len[tid] >= 0) {
        const int32_t len = t_len[tid];
        stop = len >= a.max_depth || t_deg[tid] == 0;
        if (kApp == FW_APP_PPR && !stop && t_moved[tid]) {  // include/app.cuh:88-94: one draw per completed step
          const uint32_t w = a.walker_base + (uint32_t)t_walker[tid];
          const uint32_t bits = philox4x32_10(w, (uint32_t)(len - 2), kStreamStopRef, 0u, a.seed_lo, a.seed_hi).x;
          stop = u24(bits) < a.tp;
        }
        t_moved[tid] = 0;
      }
      is_large[tid] = 0;
      refill(stop);
    }
    __syncthreads();  // :1433-1437
  }

  if (n_steps != 0ull) {
    atomicAdd(&s_acc[0], n_steps);
    atomicAdd(&s_acc[1], n_edges);
  }
  __syncthreads();
  if (tid == 0 && s_acc[0] != 0ull) {
    atomicAdd(&a.counters[0], s_acc[0]);
    atomicAdd(&a.counters[1], s_acc[1]);
  }
}

// Workgroups of a launch of the reference's engine: `grid` when given, else twice the resident set (src/walk.cu:84-92),
// never more than there are groups of kRefTasks queries.
template <int kApp, bool kDprs, int kRng>
int launch_ref(const fw_kargs& a, int wg_threads, int grid, int static_assignment, hipStream_t stream, int* grid_used) {
  if (wg_threads != 256 && wg_threads != 512 && wg_threads != 1024) {
    fw_set_error("wg_threads must be 256, 512 or 1024 (got %d)", wg_threads);
    return FW_ERR_INVALID;
  }
  if (grid <= 0) {
    int dev = 0, cus = 0, per_cu = 0;
    FW_HIP(hipGetDevice(&dev));
    FW_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    FW_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fw_walk_ref<kApp, kDprs, kRng>, wg_threads, 0));
    grid = cus * (per_cu > 0 ? per_cu : 1) * 2;
  }
  const int needed = (a.n + kRefTasks - 1) / kRefTasks;
  if (grid > needed) grid = needed;
  RefThreadState* rng_dev = nullptr;
  if (kRng == 2) FW_HIP(hipMalloc(reinterpret_cast<void**>(&rng_dev), (size_t)grid * (size_t)wg_threads * sizeof(RefThreadState)));
  hipLaunchKernelGGL((fw_walk_ref<kApp, kDprs, kRng>), dim3(grid), dim3(wg_threads), 0, stream, a, static_assignment, rng_dev);
  int rc = fw_check_hip(hipGetLastError(), "fw_walk_ref", __FILE__, __LINE__);
  if (kRng == 2) {  // the states are the launch's own: wait for it and give them back
    if (rc == FW_OK) rc = fw_check_hip(hipStreamSynchronize(stream), "hipStreamSynchronize", __FILE__, __LINE__);
    (void)hipFree(rng_dev);
  }
  if (rc != FW_OK) return rc;
  if (grid_used) *grid_used = grid;
  return FW_OK;
}

template <int kApp, int kRng>
int launch_ref_rng(const fw_kargs& a, bool dprs, int wg_threads, int grid, int static_assignment, hipStream_t stream,
                   int* grid_used) {
  return dprs ? launch_ref<kApp, true, kRng>(a, wg_threads, grid, static_assignment, stream, grid_used)
              : launch_ref<kApp, false, kRng>(a, wg_threads, grid, static_assignment, stream, grid_used);
}

template <int kApp>
int launch_ref_app(const fw_kargs& a, bool dprs, int rng, int wg_threads, int grid, int static_assignment, hipStream_t stream,
                   int* grid_used) {
  switch (rng) {
    case 0: return launch_ref_rng<kApp, 0>(a, dprs, wg_threads, grid, static_assignment, stream, grid_used);
    case 1: return launch_ref_rng<kApp, 1>(a, dprs, wg_threads, grid, static_assignment, stream, grid_used);
    default: return launch_ref_rng<kApp, 2>(a, dprs, wg_threads, grid, static_assignment, stream, grid_used);
  }
}

}  // namespace

int fw_launch_ref_walk(const fw_kargs& a, int app, int sampler, int wg_threads, int grid, hipStream_t stream,
                       int* grid_used) {
  const bool dprs = (sampler & 0xFF) == FW_SAMPLER_REF_DPRS;
  const int static_assignment = (sampler & FW_SAMPLER_REF_STATIC) ? 1 : 0;
  const int rng = (sampler & FW_SAMPLER_REF_RNG_LDS) ? 1 : ((sampler & FW_SAMPLER_REF_RNG_GLOBAL) ? 2 : 0);
  if ((sampler & FW_SAMPLER_REF_RNG_LDS) && (sampler & FW_SAMPLER_REF_RNG_GLOBAL)) {
    fw_set_error("FW_SAMPLER_REF_RNG_LDS and FW_SAMPLER_REF_RNG_GLOBAL exclude each other");
    return FW_ERR_INVALID;
  }
  if (rng != 0 && !static_assignment) {
    fw_set_error("thread-owned generators (FW_SAMPLER_REF_RNG_*) need FW_SAMPLER_REF_STATIC: with the global query "
                 "dispenser the thread that serves a query changes from run to run");
    return FW_ERR_INVALID;
  }
  switch (app) {
    case FW_APP_DEEPWALK: return launch_ref_app<FW_APP_DEEPWALK>(a, dprs, rng, wg_threads, grid, static_assignment, stream, grid_used);
    case FW_APP_PPR: return launch_ref_app<FW_APP_PPR>(a, dprs, rng, wg_threads, grid, static_assignment, stream, grid_used);
    case FW_APP_NODE2VEC: return launch_ref_app<FW_APP_NODE2VEC>(a, dprs, rng, wg_threads, grid, static_assignment, stream, grid_used);
    case FW_APP_METAPATH: return launch_ref_app<FW_APP_METAPATH>(a, dprs, rng, wg_threads, grid, static_assignment, stream, grid_used);
    default:
      fw_set_error("unknown app %d", app);
      return FW_ERR_INVALID;
  }
}
