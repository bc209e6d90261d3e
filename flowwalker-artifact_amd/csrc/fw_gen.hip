// Synthetic R-MAT graphs generated directly in device memory.
//
// The reference ships one example graph and an offline converter (data/EdgeListToCSR.cpp); the
// measured configurations need R-MAT graphs of up to 2^26 vertices, which are generated here:
// edges from Philox4x32-10 draws, self-loops dropped, duplicates removed, optional symmetrisation,
// ascending neighbour lists, weights / labels keyed by the unordered endpoint pair (so both
// directions of an edge agree, as data/EdgeListToCSR.cpp:185-191 does).
//
// Everything is integer arithmetic on counter-based draws, so a host program can reproduce the same
// graph: edge k, level i uses word (i & 3) of Philox(ctr = (k_lo, k_hi, i >> 2, 'RMAT'), key = seed)
// and compares it against floor(a * 2^32), floor((a+b) * 2^32), floor((a+b+c) * 2^32).

#include <cstring>

#include <rocprim/rocprim.hpp>

#include "fw_internal.h"

namespace {

constexpr uint32_t kTagRmat = 0x524D4154u;  // 'RMAT'
constexpr uint32_t kTagEdge = 0x45444745u;  // 'EDGE'
constexpr uint64_t kDropped = ~0ull;

__device__ __forceinline__ uint4 philox(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
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

__global__ void gen_edges_kernel(uint64_t* keys, uint64_t n_edges, int scale, uint32_t ta, uint32_t tab,
                                 uint32_t tabc, int symmetrise, uint32_t k0, uint32_t k1) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t e = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n_edges; e += stride) {
    uint32_t src = 0, dst = 0;
    uint4 r = make_uint4(0, 0, 0, 0);
    for (int i = 0; i < scale; ++i) {
      if ((i & 3) == 0) r = philox((uint32_t)e, (uint32_t)(e >> 32), (uint32_t)(i >> 2), kTagRmat, k0, k1);
      const uint32_t x = (i & 3) == 0 ? r.x : (i & 3) == 1 ? r.y : (i & 3) == 2 ? r.z : r.w;
      // quadrants in the order a (0,0), b (0,1), c (1,0), d (1,1); thresholds are cumulative
      const uint32_t row = (x >= tab) ? 1u : 0u;
      const uint32_t col = (x >= ta && x < tab) || (x >= tabc) ? 1u : 0u;
      src = (src << 1) | row;
      dst = (dst << 1) | col;
    }
    const bool loop = src == dst;
    const uint64_t fwd = loop ? kDropped : (((uint64_t)src << 32) | dst);
    if (symmetrise) {
      keys[2 * e] = fwd;
      keys[2 * e + 1] = loop ? kDropped : (((uint64_t)dst << 32) | src);
    } else {
      keys[e] = fwd;
    }
  }
}

// xadj[v] = number of keys with source < v  (keys are sorted and unique)
__global__ void build_xadj_kernel(const uint64_t* __restrict__ keys, uint64_t n, uint32_t* xadj, int32_t V) {
  const int stride = gridDim.x * blockDim.x;
  for (int v = blockIdx.x * blockDim.x + threadIdx.x; v <= V; v += stride) {
    const uint64_t target = (uint64_t)(uint32_t)v << 32;
    uint64_t lo = 0, hi = n;
    while (lo < hi) {
      const uint64_t mid = (lo + hi) >> 1;
      if (keys[mid] < target) lo = mid + 1; else hi = mid;
    }
    xadj[v] = (uint32_t)lo;
  }
}

__global__ void fill_edges_kernel(const uint64_t* __restrict__ keys, uint64_t n, int32_t* adjncy, float* weight,
                                  int32_t* label, float w_lo, float w_span, uint32_t n_labels, uint32_t k0,
                                  uint32_t k1) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const uint64_t key = keys[i];
    const uint32_t s = (uint32_t)(key >> 32), d = (uint32_t)key;
    adjncy[i] = (int32_t)d;
    if (weight || label) {
      const uint32_t lo = s < d ? s : d, hi = s < d ? d : s;
      const uint4 r = philox(lo, hi, 0u, kTagEdge, k0, k1);
      if (weight) {
        const float u = (float)(r.x >> 8) * 0x1p-24f;
        const float scaled = w_span * u;
        weight[i] = w_lo + scaled;
      }
      if (label) label[i] = (int32_t)(((uint64_t)r.y * (uint64_t)n_labels) >> 32);
    }
  }
}

__global__ void count_valid_kernel(const uint64_t* __restrict__ keys, uint64_t n, unsigned long long* out) {
  // keys are sorted; the dropped sentinel, if present, is the single last key after unique
  if (blockIdx.x == 0 && threadIdx.x == 0) *out = (n > 0 && keys[n - 1] == kDropped) ? n - 1 : n;
}

struct DevBuf {
  void* p = nullptr;
  ~DevBuf() { if (p) (void)hipFree(p); }
  void* release() { void* r = p; p = nullptr; return r; }
};

}  // namespace

extern "C" int fw_gen_rmat(const fw_rmat_params* rp, fw_graph** out) {
  if (!rp || !out) { fw_set_error("fw_gen_rmat: NULL argument"); return FW_ERR_INVALID; }
  *out = nullptr;
  if (rp->scale < 1 || rp->scale > 30 || rp->edge_factor < 1) {
    fw_set_error("fw_gen_rmat: scale must be in [1,30] and edge_factor >= 1");
    return FW_ERR_INVALID;
  }
  const double a = rp->a, b = rp->b, c = rp->c;
  if (!(a >= 0 && b >= 0 && c >= 0 && a + b + c <= 1.0)) {
    fw_set_error("fw_gen_rmat: need a,b,c >= 0 and a+b+c <= 1");
    return FW_ERR_INVALID;
  }
  if (rp->make_weights && !(rp->w_lo >= 0.0f && rp->w_hi >= rp->w_lo)) {
    fw_set_error("fw_gen_rmat: need 0 <= w_lo <= w_hi");
    return FW_ERR_INVALID;
  }
  if (fw_device_count() <= 0) { fw_set_error("no HIP device is visible"); return FW_ERR_NO_DEVICE; }

  const int32_t V = (int32_t)(1u << rp->scale);
  const uint64_t n_gen = (uint64_t)rp->edge_factor << rp->scale;
  const uint64_t n_keys = rp->symmetrise ? 2 * n_gen : n_gen;
  if (n_keys > 0xFFFFFFF0ull) { fw_set_error("fw_gen_rmat: too many edges for 32-bit CSR offsets"); return FW_ERR_INVALID; }
  auto thr = [](double x) { double t = x * 4294967296.0; return t >= 4294967295.0 ? 0xFFFFFFFFu : (uint32_t)t; };
  const uint32_t ta = thr(a), tab = thr(a + b), tabc = thr(a + b + c);
  const uint32_t k0 = (uint32_t)rp->seed, k1 = (uint32_t)(rp->seed >> 32);

  DevBuf keys_a, keys_b, temp, d_count;
  FW_HIP(hipMalloc(&keys_a.p, n_keys * sizeof(uint64_t)));
  FW_HIP(hipMalloc(&keys_b.p, n_keys * sizeof(uint64_t)));
  FW_HIP(hipMalloc(&d_count.p, 2 * sizeof(unsigned long long)));
  uint64_t* ka = static_cast<uint64_t*>(keys_a.p);
  uint64_t* kb = static_cast<uint64_t*>(keys_b.p);
  unsigned long long* dcount = static_cast<unsigned long long*>(d_count.p);

  hipLaunchKernelGGL(gen_edges_kernel, dim3(8192), dim3(256), 0, 0, ka, n_gen, rp->scale, ta, tab, tabc,
                     rp->symmetrise, k0, k1);
  FW_HIP(hipGetLastError());

  // sort (only the bits that can be set; the sentinel has all bits set, so keep 64 when it may occur)
  size_t temp_bytes = 0;
  FW_HIP(rocprim::radix_sort_keys(nullptr, temp_bytes, ka, kb, (size_t)n_keys, 0, 64, 0));
  FW_HIP(hipMalloc(&temp.p, temp_bytes ? temp_bytes : 1));
  FW_HIP(rocprim::radix_sort_keys(temp.p, temp_bytes, ka, kb, (size_t)n_keys, 0, 64, 0));
  FW_HIP(hipFree(temp.release()));

  // unique: kb -> ka
  size_t temp2 = 0;
  FW_HIP(rocprim::unique(nullptr, temp2, kb, ka, dcount, (size_t)n_keys, rocprim::equal_to<uint64_t>(), 0));
  FW_HIP(hipMalloc(&temp.p, temp2 ? temp2 : 1));
  FW_HIP(rocprim::unique(temp.p, temp2, kb, ka, dcount, (size_t)n_keys, rocprim::equal_to<uint64_t>(), 0));
  unsigned long long n_unique = 0;
  FW_HIP(hipMemcpy(&n_unique, dcount, sizeof(n_unique), hipMemcpyDeviceToHost));
  hipLaunchKernelGGL(count_valid_kernel, dim3(1), dim3(1), 0, 0, ka, (uint64_t)n_unique, dcount + 1);
  unsigned long long E = 0;
  FW_HIP(hipMemcpy(&E, dcount + 1, sizeof(E), hipMemcpyDeviceToHost));
  FW_HIP(hipFree(temp.release()));
  FW_HIP(hipFree(keys_b.release()));
  if (E == 0) { fw_set_error("fw_gen_rmat: the generated graph has no edges"); return FW_ERR_INVALID; }

  DevBuf xadj, adjncy, weight, label;
  const size_t ebytes = (size_t)(E + FW_EDGE_PAD) * 4;
  FW_HIP(hipMalloc(&xadj.p, (size_t)(V + 1) * sizeof(uint32_t)));
  FW_HIP(hipMalloc(&adjncy.p, ebytes));
  FW_HIP(hipMemset(adjncy.p, 0, ebytes));
  if (rp->make_weights) {
    FW_HIP(hipMalloc(&weight.p, ebytes));
    FW_HIP(hipMemset(weight.p, 0, ebytes));
  }
  if (rp->n_labels > 0) {
    FW_HIP(hipMalloc(&label.p, ebytes));
    FW_HIP(hipMemset(label.p, 0, ebytes));
  }
  hipLaunchKernelGGL(build_xadj_kernel, dim3(4096), dim3(256), 0, 0, ka, (uint64_t)E,
                     static_cast<uint32_t*>(xadj.p), V);
  FW_HIP(hipGetLastError());
  hipLaunchKernelGGL(fill_edges_kernel, dim3(8192), dim3(256), 0, 0, ka, (uint64_t)E,
                     static_cast<int32_t*>(adjncy.p), static_cast<float*>(weight.p),
                     static_cast<int32_t*>(label.p), rp->w_lo, rp->w_hi - rp->w_lo, (uint32_t)rp->n_labels, k0, k1);
  FW_HIP(hipGetLastError());
  FW_HIP(hipDeviceSynchronize());

  int rc = fw_graph_adopt_device(V, (uint64_t)E, static_cast<uint32_t*>(xadj.p), static_cast<int32_t*>(adjncy.p),
                                 static_cast<float*>(weight.p), static_cast<int32_t*>(label.p), 1, out);
  if (rc != FW_OK) return rc;
  xadj.release(); adjncy.release(); weight.release(); label.release();
  (*out)->sorted = 1;
  return FW_OK;
}
