// Baseline samplers of the sampler micro-benchmark, restated for 64-lane waves: inverse transform sampling (ITS),
// rejection sampling (RJS) and the alias method (ALS).  The reference's TestSampler compares its reservoir samplers with them on slices of one large
// array of weights (src/sampler_test.cu:290-410, :561-712; samplers include/sampler.cuh:792-1100); they are not part
// of the walk path.  A "worker" is a wave (or a workgroup) that draws ONE index from the `list_len` weights of a task;
// tasks name their slice (task t owns weights[t * list_len, (t + 1) * list_len)) and are visited in the order of a task
// list, as the reference's shuffled task_list does.  Random numbers: Philox4x32-10 keyed by (seed, task position).
//
//   ITS  its_warp_sampler_direct / its_block_sampler_direct (include/sampler.cuh:850-884, :934-968): inclusive prefix
//        sums of the weights written to a scratch slice (chunks of the group's width, scan + carry), one uniform scaled by
//        the total, binary search for the first prefix above it.
//   RJS  rjs_warp_sampler / rjs_block_sampler (include/sampler.cuh:970-1100): maximum weight by a reduction, then
//        (index, height) proposals until one falls under its weight.  Here every lane of the group proposes per round
//        and the first lane that hits wins: proposals are independent and identically distributed, so taking the first
//        success in a fixed order is the same law as the reference's one-proposal-at-a-time loop.
//   ALS  naive_alias_warp_sampler / _block_sampler (include/sampler.cuh:559-790; kernels src/sampler_test.cu:348-410): an
//        alias table built for the list, then one (slot, height) draw.  The reference pairs small and large entries
//        through lock-free work lists; here the table is built from prefix sums, with no loop whose end depends on another
//        lane: with p_i = w_i * n / sum w, lights (p < 1) and heavies (p >= 1) in list order, D_i = the lights' cumulative
//        deficit and E_j = the heavies' cumulative excess, the ordered two-pointer sweep of the textbook construction gives
//        light i the alias heavy min{j : E_j >= D_(i-1)}, and heavy j ends with probability 1 + E_j - D_i* (i* = the first
//        light with D_i > E_j) and the next heavy as its alias.  Two compactions, two scans and two binary searches per
//        entry; the table is exact up to f32 rounding like any alias table.

#include <algorithm>

#include "fw_internal.h"
#include "fw_device_util.h"

namespace {

constexpr uint32_t kStreamBench = 0x08000000u;

__device__ __forceinline__ float wave_max_f32(float v) {  // non-negative floats order like their bit patterns
  return __int_as_float(wave_max_i32(__float_as_int(v)));
}

struct BenchArgs {
  const float* weights;
  const uint32_t* tasks;  // slice of every task position (NULL: position p owns slice p)
  uint32_t n_tasks;
  uint32_t list_len;
  uint32_t n_slices;      // elements / list_len: a task that names a slice beyond it is answered -1, not read
  float* scratch;         // ITS: list_len floats per worker; ALS: 6 * list_len words per worker
  int32_t* out;           // out[position] = sampled index in [0, list_len), -1 when no weight is positive
  uint32_t seed_lo, seed_hi;
};

// ---- ITS ------------------------------------------------------------------------------------------------------

// one wave per task
__global__ __launch_bounds__(256) void fw_bench_its_wave(const BenchArgs a) {
  const int lane = lane_id();
  const uint32_t worker = blockIdx.x * 4u + (threadIdx.x >> 6);
  const uint32_t nworkers = gridDim.x * 4u;
  float* const prefix = a.scratch + (size_t)worker * a.list_len;
  for (uint32_t p = worker; p < a.n_tasks; p += nworkers) {
    const uint32_t slice = a.tasks ? a.tasks[p] : p;
    if (slice >= a.n_slices) {
      if (lane == 0) a.out[p] = -1;
      continue;
    }
    const float* w = a.weights + (size_t)slice * a.list_len;
    float carry = 0.0f;
    for (uint32_t base = 0; base < a.list_len; base += 64u) {  // :858-866
      const uint32_t i = base + (uint32_t)lane;
      const float x = i < a.list_len ? w[i] : 0.0f;
      const float s = carry + wave_scan(x);
      if (i < a.list_len) prefix[i] = s;
      carry = readlane_f(s, 63);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (lane == 0) {  // :875-880 (the division by the total is folded into the target)
      int32_t sel = -1;
      if (carry > 0.0f) {
        const float target = u24(philox4x32_10(p, 0u, kStreamBench, 0u, a.seed_lo, a.seed_hi).x) * carry;
        uint32_t lo = 0u, hi = a.list_len;  // first prefix above the target
        while (lo < hi) {
          const uint32_t mid = (lo + hi) >> 1;
          if (prefix[mid] > target) hi = mid; else lo = mid + 1u;
        }
        sel = (int32_t)(lo < a.list_len ? lo : a.list_len - 1u);
        while (sel > 0 && w[sel] <= 0.0f) --sel;  // rounding left the target on a zero weight's flat stretch
      }
      a.out[p] = sel;
    }
    __builtin_amdgcn_wave_barrier();  // the scratch slice is reused by the worker's next task
  }
}

// one workgroup per task
__global__ __launch_bounds__(1024) void fw_bench_its_block(const BenchArgs a) {
  __shared__ float s_tot[16];
  const int lane = lane_id();
  const int wave = (int)(threadIdx.x >> 6);
  const int nw = (int)(blockDim.x >> 6);
  float* const prefix = a.scratch + (size_t)blockIdx.x * a.list_len;
  for (uint32_t p = blockIdx.x; p < a.n_tasks; p += gridDim.x) {
    const uint32_t slice = a.tasks ? a.tasks[p] : p;
    if (slice >= a.n_slices) {  // the same in every thread
      if (threadIdx.x == 0) a.out[p] = -1;
      continue;
    }
    const float* w = a.weights + (size_t)slice * a.list_len;
    float carry = 0.0f;
    for (uint32_t base = 0; base < a.list_len; base += blockDim.x) {  // :939-953
      const uint32_t i = base + threadIdx.x;
      const float x = i < a.list_len ? w[i] : 0.0f;
      const float I = wave_scan(x);
      if (lane == 63) s_tot[wave] = I;
      __syncthreads();
      float off = carry, next = carry;
      for (int v = 0; v < nw; ++v) {
        if (v < wave) off += s_tot[v];
        next += s_tot[v];
      }
      if (i < a.list_len) prefix[i] = off + I;
      carry = next;
      __syncthreads();
    }
    if (threadIdx.x == 0) {
      int32_t sel = -1;
      if (carry > 0.0f) {
        const float target = u24(philox4x32_10(p, 0u, kStreamBench, 0u, a.seed_lo, a.seed_hi).x) * carry;
        uint32_t lo = 0u, hi = a.list_len;
        while (lo < hi) {
          const uint32_t mid = (lo + hi) >> 1;
          if (prefix[mid] > target) hi = mid; else lo = mid + 1u;
        }
        sel = (int32_t)(lo < a.list_len ? lo : a.list_len - 1u);
        while (sel > 0 && w[sel] <= 0.0f) --sel;
      }
      a.out[p] = sel;
    }
    __syncthreads();
  }
}

// ---- RJS ------------------------------------------------------------------------------------------------------

// Proposals of one round: lane-th (index, height) pair of round r of task position p.
__device__ __forceinline__ bool rjs_try(const BenchArgs& a, const float* w, uint32_t p, uint32_t round, uint32_t t,
                                        float wmax, uint32_t* idx_out) {
  const uint4 b = philox4x32_10(p, round, kStreamBench + 1u, t, a.seed_lo, a.seed_hi);
  const uint32_t x = (uint32_t)(((uint64_t)b.x * a.list_len) >> 32);  // uniform index
  const float y = u24(b.y) * wmax;
  *idx_out = x;
  return y < w[x];
}

constexpr uint32_t kRjsMaxRounds = 1u << 20;  // every wave leaves the loop: a task whose weights are all tiny next to
                                              // one huge one stops proposing after this many rounds and reports -1

__global__ __launch_bounds__(256) void fw_bench_rjs_wave(const BenchArgs a) {
  const int lane = lane_id();
  const uint32_t worker = blockIdx.x * 4u + (threadIdx.x >> 6);
  const uint32_t nworkers = gridDim.x * 4u;
  for (uint32_t p = worker; p < a.n_tasks; p += nworkers) {
    const uint32_t slice = a.tasks ? a.tasks[p] : p;
    if (slice >= a.n_slices) {
      if (lane == 0) a.out[p] = -1;
      continue;
    }
    const float* w = a.weights + (size_t)slice * a.list_len;
    float m = 0.0f;
    for (uint32_t i = (uint32_t)lane; i < a.list_len; i += 64u) m = fmaxf(m, w[i]);  // :975-981
    const float wmax = wave_max_f32(m);
    int32_t sel = -1;
    if (wmax > 0.0f) {
      for (uint32_t round = 0; round < kRjsMaxRounds; ++round) {  // :984-991
        uint32_t x;
        const bool hit = rjs_try(a, w, p, round, (uint32_t)lane, wmax, &x);
        const uint64_t mh = __ballot(hit);
        if (mh != 0ull) {
          sel = __builtin_amdgcn_readlane((int)x, __builtin_ctzll(mh));
          break;
        }
      }
    }
    if (lane == 0) a.out[p] = sel;
  }
}

__global__ __launch_bounds__(1024) void fw_bench_rjs_block(const BenchArgs a) {
  __shared__ float s_max[16];
  __shared__ int32_t s_hit[16];
  const int lane = lane_id();
  const int wave = (int)(threadIdx.x >> 6);
  const int nw = (int)(blockDim.x >> 6);
  for (uint32_t p = blockIdx.x; p < a.n_tasks; p += gridDim.x) {
    const uint32_t slice = a.tasks ? a.tasks[p] : p;
    if (slice >= a.n_slices) {  // the same in every thread
      if (threadIdx.x == 0) a.out[p] = -1;
      continue;
    }
    const float* w = a.weights + (size_t)slice * a.list_len;
    float m = 0.0f;
    for (uint32_t i = threadIdx.x; i < a.list_len; i += blockDim.x) m = fmaxf(m, w[i]);
    m = wave_max_f32(m);
    if (lane == 0) s_max[wave] = m;
    __syncthreads();
    float wmax = 0.0f;
    for (int v = 0; v < nw; ++v) wmax = fmaxf(wmax, s_max[v]);
    int32_t sel = -1;
    if (wmax > 0.0f) {
      for (uint32_t round = 0; round < kRjsMaxRounds; ++round) {
        uint32_t x;
        const bool hit = rjs_try(a, w, p, round, threadIdx.x, wmax, &x);
        const uint64_t mh = __ballot(hit);
        if (lane == 0) s_hit[wave] = mh != 0ull ? __builtin_amdgcn_readlane((int)x, (int)__builtin_ctzll(mh | (1ull << 63))) : -1;
        __syncthreads();
        for (int v = 0; v < nw && sel < 0; ++v) sel = s_hit[v];  // first wave, first lane that hit
        __syncthreads();
        if (sel >= 0) break;  // the same in every thread
      }
    }
    if (threadIdx.x == 0) a.out[p] = sel;
    __syncthreads();
  }
}


// ---- ALS ------------------------------------------------------------------------------------------------------

// Scratch of one worker: six arrays of list_len words.
struct AliasScratch {
  float* prob;      // [n] probability of keeping the slot's own index
  uint32_t* alias;  // [n]
  uint32_t* light;  // [a] indices with p < 1, in list order
  uint32_t* heavy;  // [b] indices with p >= 1
  float* D;         // [a] inclusive cumulative deficit of the lights
  float* E;         // [b] inclusive cumulative excess of the heavies
};
__device__ __forceinline__ AliasScratch alias_scratch(float* base, uint32_t n) {
  AliasScratch s;
  s.prob = base;
  s.alias = reinterpret_cast<uint32_t*>(base + n);
  s.light = reinterpret_cast<uint32_t*>(base + 2 * (size_t)n);
  s.heavy = reinterpret_cast<uint32_t*>(base + 3 * (size_t)n);
  s.D = base + 4 * (size_t)n;
  s.E = base + 5 * (size_t)n;
  return s;
}

// Second half of the construction, for entries first, first + step, ...: aliases and probabilities from D and E.
__device__ __forceinline__ void alias_assign(const AliasScratch& t, const float* w, float scale, uint32_t a, uint32_t b,
                                             uint32_t first, uint32_t step) {
  for (uint32_t i = first; i < a; i += step) {  // light i: served by the first heavy that still holds 1 when it comes up
    const float before = i == 0u ? 0.0f : t.D[i - 1u];
    uint32_t lo = 0u, hi = b;  // first j with E_j >= before
    while (lo < hi) {
      const uint32_t mid = (lo + hi) >> 1;
      if (t.E[mid] >= before) hi = mid; else lo = mid + 1u;
    }
    const uint32_t idx = t.light[i];
    t.prob[idx] = w[idx] * scale;
    t.alias[idx] = b != 0u ? t.heavy[lo < b ? lo : b - 1u] : idx;  // (no heavy at all: rounding only; the entry keeps itself)
    if (b == 0u) t.prob[idx] = 1.0f;
  }
  for (uint32_t j = first; j < b; j += step) {  // heavy j: drops below 1 at the first light whose cumulative deficit exceeds E_j
    const float e = t.E[j];
    uint32_t lo = 0u, hi = a;  // first i with D_i > e
    while (lo < hi) {
      const uint32_t mid = (lo + hi) >> 1;
      if (t.D[mid] > e) hi = mid; else lo = mid + 1u;
    }
    const uint32_t idx = t.heavy[j];
    float pr = 1.0f;
    if (lo < a && j + 1u < b) {
      pr = 1.0f + e - t.D[lo];
      pr = pr < 0.0f ? 0.0f : (pr > 1.0f ? 1.0f : pr);
    }
    t.prob[idx] = pr;
    t.alias[idx] = j + 1u < b ? t.heavy[j + 1u] : idx;
  }
}

__device__ __forceinline__ int32_t alias_draw(const BenchArgs& a, const AliasScratch& t, uint32_t p) {
  const uint4 r = philox4x32_10(p, 0u, kStreamBench + 2u, 0u, a.seed_lo, a.seed_hi);
  const uint32_t slot = (uint32_t)(((uint64_t)r.x * a.list_len) >> 32);
  return u24(r.y) < t.prob[slot] ? (int32_t)slot : (int32_t)t.alias[slot];
}

__global__ __launch_bounds__(256) void fw_bench_als_wave(const BenchArgs a) {
  const int lane = lane_id();
  const uint32_t worker = blockIdx.x * 4u + (threadIdx.x >> 6);
  const uint32_t nworkers = gridDim.x * 4u;
  const uint32_t n = a.list_len;
  const AliasScratch t = alias_scratch(a.scratch + (size_t)worker * 6u * n, n);
  for (uint32_t p = worker; p < a.n_tasks; p += nworkers) {
    const uint32_t slice = a.tasks ? a.tasks[p] : p;
    if (slice >= a.n_slices) {
      if (lane == 0) a.out[p] = -1;
      continue;
    }
    const float* w = a.weights + (size_t)slice * n;
    float sum = 0.0f;
    for (uint32_t i = (uint32_t)lane; i < n; i += 64u) sum += w[i];
    sum = readlane_f(wave_scan(sum), 63);
    if (!(sum > 0.0f)) {
      if (lane == 0) a.out[p] = -1;
      continue;
    }
    const float scale = (float)n / sum;
    // lights and heavies in list order, with their cumulative deficit / excess
    uint32_t na = 0u, nb = 0u;  // the same in every lane
    float cd = 0.0f, ce = 0.0f;
    for (uint32_t base = 0; base < n; base += 64u) {
      const uint32_t i = base + (uint32_t)lane;
      const bool in = i < n;
      const float pi = in ? w[i] * scale : 1.0f;
      const bool is_light = in && pi < 1.0f;
      const bool is_heavy = in && !is_light;
      const uint64_t ml = __ballot(is_light), mh = __ballot(is_heavy);
      const uint64_t below = (1ull << lane) - 1ull;
      const float d = cd + wave_scan(is_light ? 1.0f - pi : 0.0f);
      const float e = ce + wave_scan(is_heavy ? pi - 1.0f : 0.0f);
      if (is_light) {
        const uint32_t at = na + (uint32_t)__builtin_popcountll(ml & below);
        t.light[at] = i;
        t.D[at] = d;
      }
      if (is_heavy) {
        const uint32_t at = nb + (uint32_t)__builtin_popcountll(mh & below);
        t.heavy[at] = i;
        t.E[at] = e;
      }
      na += (uint32_t)__builtin_popcountll(ml);
      nb += (uint32_t)__builtin_popcountll(mh);
      cd = readlane_f(d, 63);
      ce = readlane_f(e, 63);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    alias_assign(t, w, scale, na, nb, (uint32_t)lane, 64u);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (lane == 0) a.out[p] = alias_draw(a, t, p);
    __builtin_amdgcn_wave_barrier();  // the scratch is reused by the worker's next task
  }
}

__global__ __launch_bounds__(1024) void fw_bench_als_block(const BenchArgs a) {
  __shared__ float s_f[2][16];
  __shared__ uint32_t s_c[2][16];
  const int lane = lane_id();
  const int wave = (int)(threadIdx.x >> 6);
  const int nw = (int)(blockDim.x >> 6);
  const uint32_t n = a.list_len;
  const AliasScratch t = alias_scratch(a.scratch + (size_t)blockIdx.x * 6u * n, n);
  for (uint32_t p = blockIdx.x; p < a.n_tasks; p += gridDim.x) {
    const uint32_t slice = a.tasks ? a.tasks[p] : p;
    if (slice >= a.n_slices) {  // the same in every thread
      if (threadIdx.x == 0) a.out[p] = -1;
      continue;
    }
    const float* w = a.weights + (size_t)slice * n;
    float sum = 0.0f;
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) sum += w[i];
    sum = readlane_f(wave_scan(sum), 63);
    if (lane == 0) s_f[0][wave] = sum;
    __syncthreads();
    sum = 0.0f;
    for (int v = 0; v < nw; ++v) sum += s_f[0][v];
    __syncthreads();
    if (!(sum > 0.0f)) {
      if (threadIdx.x == 0) a.out[p] = -1;
      continue;
    }
    const float scale = (float)n / sum;
    uint32_t na = 0u, nb = 0u;
    float cd = 0.0f, ce = 0.0f;
    for (uint32_t base = 0; base < n; base += blockDim.x) {
      const uint32_t i = base + threadIdx.x;
      const bool in = i < n;
      const float pi = in ? w[i] * scale : 1.0f;
      const bool is_light = in && pi < 1.0f;
      const bool is_heavy = in && !is_light;
      const uint64_t ml = __ballot(is_light), mh = __ballot(is_heavy);
      const uint64_t below = (1ull << lane) - 1ull;
      const float dw = wave_scan(is_light ? 1.0f - pi : 0.0f);
      const float ew = wave_scan(is_heavy ? pi - 1.0f : 0.0f);
      if (lane == 63) {
        s_f[0][wave] = dw;
        s_f[1][wave] = ew;
        s_c[0][wave] = (uint32_t)__builtin_popcountll(ml);
        s_c[1][wave] = (uint32_t)__builtin_popcountll(mh);
      }
      __syncthreads();
      float d0 = cd, e0 = ce, dall = cd, eall = ce;
      uint32_t a0 = na, b0 = nb, aall = na, ball = nb;
      for (int v = 0; v < nw; ++v) {
        if (v < wave) { d0 += s_f[0][v]; e0 += s_f[1][v]; a0 += s_c[0][v]; b0 += s_c[1][v]; }
        dall += s_f[0][v]; eall += s_f[1][v]; aall += s_c[0][v]; ball += s_c[1][v];
      }
      if (is_light) {
        const uint32_t at = a0 + (uint32_t)__builtin_popcountll(ml & below);
        t.light[at] = i;
        t.D[at] = d0 + dw;
      }
      if (is_heavy) {
        const uint32_t at = b0 + (uint32_t)__builtin_popcountll(mh & below);
        t.heavy[at] = i;
        t.E[at] = e0 + ew;
      }
      cd = dall; ce = eall; na = aall; nb = ball;
      __syncthreads();
    }
    __threadfence_block();
    __syncthreads();
    alias_assign(t, w, scale, na, nb, threadIdx.x, blockDim.x);
    __threadfence_block();
    __syncthreads();
    if (threadIdx.x == 0) a.out[p] = alias_draw(a, t, p);
    __syncthreads();
  }
}

}  // namespace

extern "C" int fw_sampler_baseline_run(int type, int workgroup, const float* d_weights, uint64_t elements,
                                       uint32_t list_len, const uint32_t* d_tasks, uint32_t n_tasks, int wg_threads,
                                       uint64_t seed, int32_t* d_out, double* kernel_ms) {
  if (!d_weights || !d_out || list_len == 0u || n_tasks == 0u || (uint64_t)list_len > elements) {
    fw_set_error("fw_sampler_baseline_run: bad argument");
    return FW_ERR_INVALID;
  }
  if (type != FW_BASELINE_ITS && type != FW_BASELINE_RJS && type != FW_BASELINE_ALS) {
    fw_set_error("fw_sampler_baseline_run: type must be FW_BASELINE_ITS, FW_BASELINE_RJS or FW_BASELINE_ALS (got %d)", type);
    return FW_ERR_INVALID;
  }
  if (workgroup && wg_threads != 256 && wg_threads != 512 && wg_threads != 1024) {
    fw_set_error("wg_threads must be 256, 512 or 1024 (got %d)", wg_threads);
    return FW_ERR_INVALID;
  }
  int dev = 0, cus = 0;
  FW_HIP(hipGetDevice(&dev));
  FW_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  // workers: one resident set, fewer when the tasks are few or the ITS scratch of a worker is large
  uint32_t grid = (uint32_t)cus * (workgroup ? 2u : 8u);
  const uint32_t per_block = workgroup ? 1u : 4u;
  if ((uint64_t)grid * per_block > n_tasks) grid = (n_tasks + per_block - 1u) / per_block;
  BenchArgs a;
  a.weights = d_weights;
  a.tasks = d_tasks;
  a.n_tasks = n_tasks;
  a.list_len = list_len;
  a.n_slices = (uint32_t)std::min<uint64_t>(elements / list_len, 0xFFFFFFFFull);
  a.scratch = nullptr;
  a.out = d_out;
  a.seed_lo = (uint32_t)seed;
  a.seed_hi = (uint32_t)(seed >> 32);
  if (type == FW_BASELINE_ITS || type == FW_BASELINE_ALS) {
    const uint64_t words = type == FW_BASELINE_ITS ? 1u : 6u;  // per list element and worker
    const uint64_t limit = (uint64_t)2 << 30;  // at most 2 Gi words of scratch
    while ((uint64_t)grid * per_block * list_len * words > limit && grid > 1u) grid /= 2u;
    if ((uint64_t)per_block * list_len * words > limit) {
      fw_set_error("fw_sampler_baseline_run: list_len %u needs more scratch than the 8 GiB this entry point allows", list_len);
      return FW_ERR_INVALID;
    }
    FW_HIP(hipMalloc(reinterpret_cast<void**>(&a.scratch), (size_t)grid * per_block * list_len * words * sizeof(float)));
  }
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int rc = fw_check_hip(hipEventCreate(&e0), "hipEventCreate", __FILE__, __LINE__);
  if (rc == FW_OK) rc = fw_check_hip(hipEventCreate(&e1), "hipEventCreate", __FILE__, __LINE__);
  if (rc == FW_OK) {
    (void)hipEventRecord(e0, nullptr);
    if (type == FW_BASELINE_ITS) {
      if (workgroup) hipLaunchKernelGGL(fw_bench_its_block, dim3(grid), dim3(wg_threads), 0, nullptr, a);
      else hipLaunchKernelGGL(fw_bench_its_wave, dim3(grid), dim3(256), 0, nullptr, a);
    } else if (type == FW_BASELINE_RJS) {
      if (workgroup) hipLaunchKernelGGL(fw_bench_rjs_block, dim3(grid), dim3(wg_threads), 0, nullptr, a);
      else hipLaunchKernelGGL(fw_bench_rjs_wave, dim3(grid), dim3(256), 0, nullptr, a);
    } else {
      if (workgroup) hipLaunchKernelGGL(fw_bench_als_block, dim3(grid), dim3(wg_threads), 0, nullptr, a);
      else hipLaunchKernelGGL(fw_bench_als_wave, dim3(grid), dim3(256), 0, nullptr, a);
    }
    rc = fw_check_hip(hipGetLastError(), "baseline sampler launch", __FILE__, __LINE__);
    (void)hipEventRecord(e1, nullptr);
    if (rc == FW_OK) rc = fw_check_hip(hipEventSynchronize(e1), "hipEventSynchronize", __FILE__, __LINE__);
    float ms = 0.0f;
    if (rc == FW_OK) rc = fw_check_hip(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime", __FILE__, __LINE__);
    if (kernel_ms) *kernel_ms = ms;
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (a.scratch) (void)hipFree(a.scratch);
  return rc;
}
