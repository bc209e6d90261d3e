// C ABI of libflowwalker_hip.so: errors, device buffers, graph mirror, walk drivers.
// Host-side counterpart of src/walk.cu (walk_test, walk_batch, timing_batch_async/sync),
// include/gpu_graph.cuh (device CSR mirror) and adjust_flags' autobatch rule (src/main.cu:244-272).

#include <limits.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <cstring>

#include <chrono>
#include <mutex>
#include <new>
#include <vector>

#include <rocprim/rocprim.hpp>

#include "fw_internal.h"

// ---- errors --------------------------------------------------------------------------------------

static thread_local char g_err[512] = "";

void fw_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int fw_check_hip(hipError_t e, const char* what, const char* file, int line) {
  if (e == hipSuccess) return FW_OK;
  fw_set_error("%s:%d HIP call \"%s\" failed with %s (%d)", file, line, what, hipGetErrorString(e), (int)e);
  (void)hipGetLastError();
  return FW_ERR_HIP;
}

extern "C" const char* fw_last_error(void) { return g_err; }

extern "C" int fw_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

static int require_device() {
  if (fw_device_count() <= 0) {
    fw_set_error("no HIP device is visible; the walk engine has no CPU fallback");
    return FW_ERR_NO_DEVICE;
  }
  return FW_OK;
}

extern "C" int fw_device_mem_info(size_t* free_bytes, size_t* total_bytes) {
  int rc = require_device();
  if (rc != FW_OK) return rc;
  size_t f = 0, t = 0;
  FW_HIP(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = f;
  if (total_bytes) *total_bytes = t;
  return FW_OK;
}

extern "C" void fw_walk_params_default(fw_walk_params* p) {
  if (!p) return;
  memset(p, 0, sizeof(*p));
  p->app = FW_APP_DEEPWALK;
  p->sampler = FW_SAMPLER_ZPRS;
  p->max_depth = 81;
  p->wg_threads = 512;
  p->hub_threshold = 16384;
  p->schema_len = 5;
  for (int i = 0; i < 5; ++i) p->schema[i] = i;
  p->tp = 0.2f;
  p->p = 2.0f;
  p->q = 0.5f;
  p->walker_base = 0;
  p->seed = 1337;
  p->grid = 0;
}

extern "C" void fw_walk_params_default_for(fw_walk_params* p, int app) {
  if (!p) return;
  fw_walk_params_default(p);
  p->app = app;
}

extern "C" uint32_t fw_autobatch_size(size_t free_bytes, int32_t headroom_mb, int32_t max_depth, int sync,
                                      uint32_t n_queries) {
  const size_t headroom = (size_t)(headroom_mb > 0 ? headroom_mb : 0) * 1024u * 1024u;
  if (max_depth < 1 || free_bytes <= headroom) return 0;
  const int d = max_depth - 1;
  size_t bs = (free_bytes - headroom) / (4u * (size_t)(d + 2));
  if (bs > (size_t)INT_MAX) bs = (size_t)INT_MAX;
  if (!sync) bs /= 2;
  if (bs > (size_t)n_queries) bs = n_queries;
  return (uint32_t)bs;
}

// ---- device buffers ------------------------------------------------------------------------------

extern "C" int fw_dev_alloc(size_t bytes, void** d_ptr) {
  if (!d_ptr) { fw_set_error("fw_dev_alloc: d_ptr is NULL"); return FW_ERR_INVALID; }
  *d_ptr = nullptr;
  int rc = require_device();
  if (rc != FW_OK) return rc;
  FW_HIP(hipMalloc(d_ptr, bytes ? bytes : 1));
  return FW_OK;
}
extern "C" int fw_dev_free(void* d_ptr) {
  if (!d_ptr) return FW_OK;
  FW_HIP(hipFree(d_ptr));
  return FW_OK;
}
extern "C" int fw_dev_upload(void* d_dst, const void* h_src, size_t bytes) {
  if (bytes == 0) return FW_OK;
  FW_HIP(hipMemcpy(d_dst, h_src, bytes, hipMemcpyHostToDevice));
  return FW_OK;
}
extern "C" int fw_dev_download(void* h_dst, const void* d_src, size_t bytes) {
  if (bytes == 0) return FW_OK;
  FW_HIP(hipMemcpy(h_dst, d_src, bytes, hipMemcpyDeviceToHost));
  return FW_OK;
}

__global__ void fw_fill_i32_kernel(int32_t* dst, int32_t value, size_t count) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) dst[i] = value;
}
extern "C" int fw_dev_fill_i32(int32_t* d_dst, int32_t value, size_t count) {
  if (count == 0) return FW_OK;
  size_t blocks = (count + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(fw_fill_i32_kernel, dim3((unsigned)blocks), dim3(256), 0, 0, d_dst, value, count);
  FW_HIP(hipGetLastError());
  FW_HIP(hipDeviceSynchronize());
  return FW_OK;
}
__global__ void fw_copy_u32x4_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t count) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) dst[i] = src[i];
}
extern "C" int fw_dev_copy(void* d_dst, const void* d_src, size_t bytes) {
  if (bytes == 0) return FW_OK;
  if ((bytes & 15u) || (((uintptr_t)d_dst | (uintptr_t)d_src) & 15u)) {
    fw_set_error("fw_dev_copy: pointers and size must be multiples of 16 bytes");
    return FW_ERR_INVALID;
  }
  const size_t count = bytes / 16;
  size_t blocks = (count + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL(fw_copy_u32x4_kernel, dim3((unsigned)blocks), dim3(256), 0, 0, static_cast<uint4*>(d_dst),
                     static_cast<const uint4*>(d_src), count);
  FW_HIP(hipGetLastError());
  FW_HIP(hipDeviceSynchronize());
  return FW_OK;
}
// Calibration: how many scattered accesses per second the memory delivers.  Every thread touches `per_thread`
// pseudo-random 64-byte lines of a buffer: mode 0 reads 4 bytes of each, mode 1 / 2 / 3 store 4 / 8 / 16 bytes into
// each (a store that does not cover its line costs the memory a read-modify-write).  Modes 4 and 5 settle the size of
// a read request: both read two words per access, mode 4 from the two 64-byte halves of one random 128-byte block,
// mode 5 from two different random blocks.  If the memory is asked for 128 bytes at a time, mode 4 costs one request
// per pair and runs at about twice mode 5's rate of loads; if for 64, both cost two.  The walk pipeline's kernels are
// priced against these rates.
__device__ __forceinline__ uint64_t fw_probe_mix(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
template <int kMode>
__global__ __launch_bounds__(256) void fw_random_access_kernel(uint32_t* arr, uint64_t n_lines, uint32_t per_thread,
                                                               uint32_t* sink) {
  const uint64_t tid = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x;
  uint32_t acc = 0u;
  for (uint32_t i = 0; i < per_thread; i += 4u) {
    uint64_t w[4], w2[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint64_t r = fw_probe_mix(tid * per_thread + i + (uint32_t)j);
      if (kMode >= 4) {  // n_lines counts 64-byte lines: blocks of 128 bytes are pairs of them
        w[j] = (r % (n_lines >> 1)) * 32u;
        w2[j] = kMode == 4 ? w[j] + 16u : (fw_probe_mix(r) % (n_lines >> 1)) * 32u;
      } else {
        w[j] = (r % n_lines) * 16u;
        w2[j] = 0u;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (kMode == 0) acc += arr[w[j] + (tid & 15u)];
      else if (kMode == 1) arr[w[j] + (tid & 15u)] = i;
      else if (kMode == 2) *reinterpret_cast<uint2*>(arr + w[j] + (tid & 14u)) = make_uint2(i, 1u);
      else if (kMode == 3) *reinterpret_cast<uint4*>(arr + w[j] + (tid & 12u)) = make_uint4(i, 1u, 2u, 3u);
      else acc += arr[w[j] + (tid & 15u)] + arr[w2[j] + (tid & 15u)];
    }
  }
  if (acc == 0x12345678u) *sink = acc;  // keeps the loads
}
extern "C" int fw_dev_random_access_rate(void* d_buf, size_t bytes, int mode, double* accesses_per_s) {
  if (!d_buf || !accesses_per_s || bytes < ((size_t)1 << 20) || (bytes & 127u) || ((uintptr_t)d_buf & 127u) || mode < 0 ||
      mode > 5) {
    fw_set_error("fw_dev_random_access_rate: buffer of at least 1 MiB, 128-byte aligned and sized; mode 0..5");
    return FW_ERR_INVALID;
  }
  const uint64_t n_lines = bytes / 64u;  // > 0: every index below stays inside the buffer
  const uint32_t per_thread = 256u;
  const unsigned grid = 8192u;
  uint32_t* sink = nullptr;
  FW_HIP(hipMalloc(reinterpret_cast<void**>(&sink), 64));
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int rc = fw_check_hip(hipEventCreate(&e0), "hipEventCreate", __FILE__, __LINE__);
  if (rc == FW_OK) rc = fw_check_hip(hipEventCreate(&e1), "hipEventCreate", __FILE__, __LINE__);
  float best = 0.0f;
  for (int rep = 0; rc == FW_OK && rep < 3; ++rep) {
    (void)hipEventRecord(e0, nullptr);
    uint32_t* arr = static_cast<uint32_t*>(d_buf);
    switch (mode) {
      case 0: hipLaunchKernelGGL(fw_random_access_kernel<0>, dim3(grid), dim3(256), 0, nullptr, arr, n_lines, per_thread, sink); break;
      case 1: hipLaunchKernelGGL(fw_random_access_kernel<1>, dim3(grid), dim3(256), 0, nullptr, arr, n_lines, per_thread, sink); break;
      case 2: hipLaunchKernelGGL(fw_random_access_kernel<2>, dim3(grid), dim3(256), 0, nullptr, arr, n_lines, per_thread, sink); break;
      case 3: hipLaunchKernelGGL(fw_random_access_kernel<3>, dim3(grid), dim3(256), 0, nullptr, arr, n_lines, per_thread, sink); break;
      case 4: hipLaunchKernelGGL(fw_random_access_kernel<4>, dim3(grid), dim3(256), 0, nullptr, arr, n_lines, per_thread, sink); break;
      default: hipLaunchKernelGGL(fw_random_access_kernel<5>, dim3(grid), dim3(256), 0, nullptr, arr, n_lines, per_thread, sink); break;
    }
    rc = fw_check_hip(hipGetLastError(), "fw_random_access_kernel", __FILE__, __LINE__);
    (void)hipEventRecord(e1, nullptr);
    if (rc == FW_OK) rc = fw_check_hip(hipEventSynchronize(e1), "hipEventSynchronize", __FILE__, __LINE__);
    float ms = 0.0f;
    if (rc == FW_OK) rc = fw_check_hip(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime", __FILE__, __LINE__);
    if (rep > 0 && (best == 0.0f || ms < best)) best = ms;
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(sink);
  // modes 4 and 5 make two loads per access: the rate counts loads
  if (rc == FW_OK) *accesses_per_s = (double)grid * 256.0 * (double)per_thread * (mode >= 4 ? 2.0 : 1.0) / ((double)best * 1e-3);
  return rc;
}
extern "C" int fw_dev_sync(void) {
  FW_HIP(hipDeviceSynchronize());
  return FW_OK;
}

extern "C" int fw_host_alloc_pinned(size_t bytes, void** h_ptr) {
  if (!h_ptr) { fw_set_error("fw_host_alloc_pinned: h_ptr is NULL"); return FW_ERR_INVALID; }
  *h_ptr = nullptr;
  int rc = require_device();
  if (rc != FW_OK) return rc;
  FW_HIP(hipHostMalloc(h_ptr, bytes ? bytes : 1, hipHostMallocDefault));
  return FW_OK;
}
extern "C" int fw_host_free_pinned(void* h_ptr) {
  if (!h_ptr) return FW_OK;
  FW_HIP(hipHostFree(h_ptr));
  return FW_OK;
}

// ---- graph ---------------------------------------------------------------------------------------

static int validate_csr_host(int32_t V, uint64_t E, const uint32_t* xadj, const int32_t* adjncy, const float* weight) {
  if (V <= 0) { fw_set_error("V must be positive (got %d)", V); return FW_ERR_INVALID; }
  if (E == 0 || E > 0xFFFFFFF0ull) { fw_set_error("E must be in [1, 2^32-16] (got %llu)", (unsigned long long)E); return FW_ERR_INVALID; }
  if (!xadj || !adjncy) { fw_set_error("xadj and adjncy are required"); return FW_ERR_INVALID; }
  if (xadj[0] != 0u) { fw_set_error("xadj[0] must be 0"); return FW_ERR_INVALID; }
  if ((uint64_t)xadj[V] != E) {  // include/graph.cuh:135-136
    fw_set_error("xadj[V] = %u does not match E = %llu", xadj[V], (unsigned long long)E);
    return FW_ERR_INVALID;
  }
  for (int32_t v = 0; v < V; ++v) {
    if (xadj[v + 1] < xadj[v]) { fw_set_error("xadj is not non-decreasing at vertex %d", v); return FW_ERR_INVALID; }
  }
  for (uint64_t i = 0; i < E; ++i) {
    if ((uint32_t)adjncy[i] >= (uint32_t)V) {
      fw_set_error("adjncy[%llu] = %d is outside [0, V)", (unsigned long long)i, adjncy[i]);
      return FW_ERR_INVALID;
    }
  }
  if (weight) {
    for (uint64_t i = 0; i < E; ++i) {
      const float w = weight[i];
      if (!(w >= 0.0f) || isinf(w)) {
        fw_set_error("weight[%llu] = %g is not a finite non-negative number", (unsigned long long)i, (double)w);
        return FW_ERR_INVALID;
      }
    }
  }
  return FW_OK;
}

// One edge array with FW_EDGE_PAD zeroed elements behind it, filled from the host copy.  In pinned host memory the
// array is mapped into the device's address space: the kernels use the same pointer and every read crosses the bus.
template <typename T>
static int alloc_edge_array(T** out, uint64_t E, const T* h_src, int host_pinned) {
  const size_t bytes = (size_t)(E + FW_EDGE_PAD) * sizeof(T);
  if (host_pinned) {
    FW_HIP(hipHostMalloc(reinterpret_cast<void**>(out), bytes, hipHostMallocDefault));
    memcpy(*out, h_src, (size_t)E * sizeof(T));
    memset(reinterpret_cast<char*>(*out) + (size_t)E * sizeof(T), 0, FW_EDGE_PAD * sizeof(T));
    return FW_OK;
  }
  FW_HIP(hipMalloc(reinterpret_cast<void**>(out), bytes));
  FW_HIP(hipMemset(reinterpret_cast<char*>(*out) + (size_t)E * sizeof(T), 0, FW_EDGE_PAD * sizeof(T)));
  FW_HIP(hipMemcpy(*out, h_src, (size_t)E * sizeof(T), hipMemcpyHostToDevice));
  return FW_OK;
}

static void release_park_cache(fw_graph* g);  // defined with the parking buffers below
static void release_batch_cache(fw_graph* g);

extern "C" int fw_graph_destroy(fw_graph* g) {
  if (!g) return FW_OK;
  int rc = FW_OK;
  if (g->owns) {
    if (g->xadj && hipFree(g->xadj) != hipSuccess) { (void)hipGetLastError(); rc = FW_ERR_HIP; }
    void* ptrs[3] = {g->adjncy, g->weight, g->label};
    for (void* p : ptrs) {
      if (p && (g->host_edges ? hipHostFree(p) : hipFree(p)) != hipSuccess) { (void)hipGetLastError(); rc = FW_ERR_HIP; }
    }
  }
  release_park_cache(g);
  release_batch_cache(g);
  for (hipEvent_t e : g->call_ev) if (e) (void)hipEventDestroy(e);
  void* index_ptrs[4] = {g->hub_index, g->hub_info, g->call_scratch, g->adj_hub};
  for (void* p : index_ptrs) {
    if (p && hipFree(p) != hipSuccess) { (void)hipGetLastError(); rc = FW_ERR_HIP; }
  }
  delete g;
  return rc;
}

extern "C" int fw_graph_create_placed(int32_t V, uint64_t E, const uint32_t* h_xadj, const int32_t* h_adjncy,
                                      const float* h_weight, const int32_t* h_label, int placement, fw_graph** out) {
  if (!out) { fw_set_error("fw_graph_create: out is NULL"); return FW_ERR_INVALID; }
  *out = nullptr;
  if (placement != FW_GRAPH_DEVICE && placement != FW_GRAPH_HOST_PINNED) {
    fw_set_error("fw_graph_create_placed: unknown placement %d", placement);
    return FW_ERR_INVALID;
  }
  int rc = validate_csr_host(V, E, h_xadj, h_adjncy, h_weight);
  if (rc != FW_OK) return rc;
  rc = require_device();
  if (rc != FW_OK) return rc;
  fw_graph* g = new (std::nothrow) fw_graph();
  if (!g) { fw_set_error("out of host memory"); return FW_ERR_NOMEM; }
  g->V = V;
  g->E = E;
  g->owns = 1;
  g->host_edges = placement == FW_GRAPH_HOST_PINNED;
  auto fail = [&](int code) { fw_graph_destroy(g); return code; };
  if (hipGetDevice(&g->device) != hipSuccess) return fail(FW_ERR_HIP);
  const size_t xbytes = (size_t)(V + 1) * sizeof(uint32_t);
  if ((rc = fw_check_hip(hipMalloc(reinterpret_cast<void**>(&g->xadj), xbytes), "hipMalloc(xadj)", __FILE__, __LINE__))) return fail(rc);
  if ((rc = fw_check_hip(hipMemcpy(g->xadj, h_xadj, xbytes, hipMemcpyHostToDevice), "hipMemcpy(xadj)", __FILE__, __LINE__))) return fail(rc);
  if ((rc = alloc_edge_array(&g->adjncy, E, h_adjncy, g->host_edges))) return fail(rc);
  if (h_weight && (rc = alloc_edge_array(&g->weight, E, h_weight, g->host_edges))) return fail(rc);
  if (h_label && (rc = alloc_edge_array(&g->label, E, h_label, g->host_edges))) return fail(rc);
  *out = g;
  return FW_OK;
}

extern "C" int fw_graph_create(int32_t V, uint64_t E, const uint32_t* h_xadj, const int32_t* h_adjncy,
                               const float* h_weight, const int32_t* h_label, fw_graph** out) {
  return fw_graph_create_placed(V, E, h_xadj, h_adjncy, h_weight, h_label, FW_GRAPH_DEVICE, out);
}

extern "C" int fw_graph_adopt_device(int32_t V, uint64_t E, uint32_t* d_xadj, int32_t* d_adjncy, float* d_weight,
                                     int32_t* d_label, int take_ownership, fw_graph** out) {
  if (!out) { fw_set_error("fw_graph_adopt_device: out is NULL"); return FW_ERR_INVALID; }
  *out = nullptr;
  if (V <= 0 || E == 0 || E > 0xFFFFFFF0ull || !d_xadj || !d_adjncy) {
    fw_set_error("fw_graph_adopt_device: need V > 0, 0 < E <= 2^32-16, xadj and adjncy");
    return FW_ERR_INVALID;
  }
  if ((((uintptr_t)d_adjncy) | ((uintptr_t)d_weight) | ((uintptr_t)d_label)) & 15u) {
    fw_set_error("fw_graph_adopt_device: edge arrays must be 16-byte aligned");
    return FW_ERR_INVALID;
  }
  int rc = require_device();
  if (rc != FW_OK) return rc;
  fw_graph* g = new (std::nothrow) fw_graph();
  if (!g) { fw_set_error("out of host memory"); return FW_ERR_NOMEM; }
  g->V = V; g->E = E;
  g->xadj = d_xadj; g->adjncy = d_adjncy; g->weight = d_weight; g->label = d_label;
  g->owns = take_ownership ? 1 : 0;
  if (hipGetDevice(&g->device) != hipSuccess) { (void)hipGetLastError(); }
  *out = g;
  return FW_OK;
}

// max degree with the smallest vertex among ties: key = degree << 32 | ~vertex
__global__ void fw_max_degree_kernel(const uint32_t* __restrict__ xadj, int32_t V, unsigned long long* best) {
  unsigned long long local = 0ull;
  const int stride = gridDim.x * blockDim.x;
  for (int v = blockIdx.x * blockDim.x + threadIdx.x; v < V; v += stride) {
    const unsigned long long d = xadj[v + 1] - xadj[v];
    const unsigned long long key = (d << 32) | (unsigned long long)(0xFFFFFFFFu - (uint32_t)v);
    local = key > local ? key : local;
  }
  atomicMax(best, local);
}

__global__ void fw_sorted_kernel(const uint32_t* __restrict__ xadj, const int32_t* __restrict__ adjncy, int32_t V,
                                 int* unsorted) {
  const int stride = gridDim.x * blockDim.x;
  for (int v = blockIdx.x * blockDim.x + threadIdx.x; v < V; v += stride) {
    const uint32_t b = xadj[v], e = xadj[v + 1];
    for (uint32_t i = b + 1; i < e; ++i) {
      if (adjncy[i] < adjncy[i - 1]) { *unsorted = 1; break; }  // equal neighbours (a multigraph) are in order
    }
  }
}

extern "C" int fw_graph_info(const fw_graph* g, int32_t* V, uint64_t* E, int32_t* max_degree,
                             int32_t* max_degree_vertex) {
  if (!g) { fw_set_error("fw_graph_info: graph is NULL"); return FW_ERR_INVALID; }
  if (V) *V = g->V;
  if (E) *E = g->E;
  if (max_degree || max_degree_vertex) {
    fw_graph* mg = const_cast<fw_graph*>(g);
    if (mg->max_degree < 0) {
      unsigned long long* d_best = nullptr;
      FW_HIP(hipMalloc(reinterpret_cast<void**>(&d_best), sizeof(unsigned long long)));
      FW_HIP(hipMemset(d_best, 0, sizeof(unsigned long long)));
      hipLaunchKernelGGL(fw_max_degree_kernel, dim3(1024), dim3(256), 0, 0, g->xadj, g->V, d_best);
      unsigned long long best = 0;
      FW_HIP(hipMemcpy(&best, d_best, sizeof(best), hipMemcpyDeviceToHost));
      FW_HIP(hipFree(d_best));
      mg->max_degree = (int32_t)(best >> 32);
      mg->max_degree_vertex = (int32_t)(0xFFFFFFFFu - (uint32_t)(best & 0xFFFFFFFFull));
    }
    if (max_degree) *max_degree = mg->max_degree;
    if (max_degree_vertex) *max_degree_vertex = mg->max_degree_vertex;
  }
  return FW_OK;
}

// d_flag: one int of device memory to use (the caller's), or NULL: allocated and freed here.
static int graph_sorted(const fw_graph* g, int* sorted, int* d_flag_in) {
  fw_graph* mg = const_cast<fw_graph*>(g);
  if (mg->sorted < 0) {
    int* d_flag = d_flag_in;
    if (!d_flag) FW_HIP(hipMalloc(reinterpret_cast<void**>(&d_flag), sizeof(int)));
    int flag = 0;
    int rc = fw_check_hip(hipMemset(d_flag, 0, sizeof(int)), "hipMemset(sorted flag)", __FILE__, __LINE__);
    if (rc == FW_OK) {
      hipLaunchKernelGGL(fw_sorted_kernel, dim3(2048), dim3(256), 0, 0, g->xadj, g->adjncy, g->V, d_flag);
      rc = fw_check_hip(hipMemcpy(&flag, d_flag, sizeof(flag), hipMemcpyDeviceToHost), "hipMemcpy(sorted flag)", __FILE__, __LINE__);
    }
    if (!d_flag_in) (void)hipFree(d_flag);
    if (rc != FW_OK) return rc;
    mg->sorted = flag ? 0 : 1;
  }
  *sorted = mg->sorted;
  return FW_OK;
}

extern "C" int fw_graph_is_sorted(const fw_graph* g, int* sorted) {
  if (!g || !sorted) { fw_set_error("fw_graph_is_sorted: NULL argument"); return FW_ERR_INVALID; }
  return graph_sorted(g, sorted, nullptr);
}

extern "C" int fw_graph_download(const fw_graph* g, uint32_t* h_xadj, int32_t* h_adjncy, float* h_weight,
                                 int32_t* h_label) {
  if (!g) { fw_set_error("fw_graph_download: graph is NULL"); return FW_ERR_INVALID; }
  if (h_xadj) FW_HIP(hipMemcpy(h_xadj, g->xadj, (size_t)(g->V + 1) * 4, hipMemcpyDeviceToHost));
  const hipMemcpyKind edge_kind = g->host_edges ? hipMemcpyHostToHost : hipMemcpyDeviceToHost;
  if (h_adjncy) FW_HIP(hipMemcpy(h_adjncy, g->adjncy, (size_t)g->E * 4, edge_kind));
  if (h_weight) {
    if (!g->weight) { fw_set_error("graph has no weights"); return FW_ERR_INVALID; }
    FW_HIP(hipMemcpy(h_weight, g->weight, (size_t)g->E * 4, edge_kind));
  }
  if (h_label) {
    if (!g->label) { fw_set_error("graph has no labels"); return FW_ERR_INVALID; }
    FW_HIP(hipMemcpy(h_label, g->label, (size_t)g->E * 4, edge_kind));
  }
  return FW_OK;
}

// ---- walks ---------------------------------------------------------------------------------------

// d_flag: one int of device memory for the neighbour-order check of node2vec (NULL: allocated when needed).
static int check_walk_args(const fw_graph* g, const fw_walk_params* p, const void* starts, int32_t n,
                           const void* paths, int* d_flag = nullptr) {
  if (!g || !p || !starts || !paths) { fw_set_error("walk: NULL argument"); return FW_ERR_INVALID; }
  if (n <= 0) { fw_set_error("walk: n must be positive (got %d)", n); return FW_ERR_INVALID; }
  if (p->max_depth < 1) { fw_set_error("walk: max_depth must be >= 1 (got %d)", p->max_depth); return FW_ERR_INVALID; }
  if (p->hub_threshold < 0) { fw_set_error("walk: hub_threshold must be >= 0"); return FW_ERR_INVALID; }
  switch (p->app) {
    case FW_APP_DEEPWALK:
    case FW_APP_PPR:
    case FW_APP_NODE2VEC:
      if (!g->weight) { fw_set_error("walk: this application needs edge weights"); return FW_ERR_INVALID; }
      break;
    case FW_APP_METAPATH:
      if (!g->label) { fw_set_error("walk: metapath needs edge labels"); return FW_ERR_INVALID; }
      if (p->schema_len < 1 || p->schema_len > FW_MAX_SCHEMA) {
        fw_set_error("walk: schema_len must be in [1, %d] (got %d)", FW_MAX_SCHEMA, p->schema_len);
        return FW_ERR_INVALID;
      }
      break;
    default:
      fw_set_error("walk: unknown app %d", p->app);
      return FW_ERR_INVALID;
  }
  if (p->app == FW_APP_PPR && !(p->tp >= 0.0f && p->tp <= 1.0f)) {
    fw_set_error("walk: tp must be in [0,1]");
    return FW_ERR_INVALID;
  }
  if (p->app == FW_APP_NODE2VEC && !(p->p > 0.0f && p->q > 0.0f)) {
    fw_set_error("walk: p and q must be positive");
    return FW_ERR_INVALID;
  }
  if (p->app == FW_APP_NODE2VEC) {  // the adjacency test searches ascending lists (include/gpu_graph.cuh:97-118)
    int sorted = 0;
    const int rc = graph_sorted(g, &sorted, d_flag);  // one pass over the adjacency the first time, then cached
    if (rc != FW_OK) return rc;
    if (!sorted) {
      fw_set_error("walk: node2vec needs ascending neighbour lists and this graph has others "
                   "(fw_csr_sort_neighbours sorts a host CSR before the upload)");
      return FW_ERR_INVALID;
    }
  }
  return FW_OK;
}

static void fill_kargs(fw_kargs* a, const fw_graph* g, const fw_walk_params* p) {
  memset(a, 0, sizeof(*a));
  a->xadj = g->xadj;
  a->adjncy = g->adjncy;
  a->weight = g->weight;
  a->label = g->label;
  a->V = g->V;
  a->max_depth = p->max_depth;
  a->hub_threshold = p->hub_threshold;
  a->seed_lo = (uint32_t)p->seed;
  a->seed_hi = (uint32_t)(p->seed >> 32);
  a->walker_base = p->walker_base;
  a->tp = p->tp;
  a->inv_p = 1.0f / p->p;
  a->inv_q = 1.0f / p->q;
  a->n2v_fmax = 1.0f;
  if (a->inv_q > a->n2v_fmax) a->n2v_fmax = a->inv_q;
  a->n2v_extra = a->inv_p > a->n2v_fmax ? a->inv_p - a->n2v_fmax : 0.0f;
  a->schema_len = p->schema_len;
  for (int i = 0; i < FW_MAX_SCHEMA; ++i) a->schema[i] = (i < p->schema_len) ? p->schema[i] : 0;
  a->park_threshold = INT_MAX;
  a->n_labels_per_hub = 1;
}

// ---- hub parking: walkers that reach a very-high-degree vertex wait there and are served in batches -------
//
// Execution strategy only: every walker still gets the vertex that the sampling definition gives it for
// (seed, walker id, step), so results are identical with and without parking.  The walk kernel parks a walker
// when it arrives on a vertex whose degree exceeds park_threshold; the parked records are grouped by hub
// (counting sort on the device), the hub batch kernel serves up to 64 walkers of a hub with one pass over its
// list, and the survivors resume in the next walk launch.  Loop until nobody is parked.

// Two-pass steps: buckets with more than kTwoPassWalkers walkers on lists of at least kTwoPassDegree elements.
// Every such list has rows of its own (520 bytes per 1024 elements and label a walker can want), set aside when
// the lists are numbered, so that nothing has to be handed out while the walks run; kMaxHubRows bounds them
// (lists past it are served by batches, however crowded).
constexpr uint32_t kTwoPassWalkers = 128;
constexpr uint32_t kTwoPassDegree = 2048;
constexpr uint32_t kMaxHubRows = 1u << 21;             // per label: 1 GiB of rows
constexpr uint64_t kMaxRows = (4ull << 30) / 520u;     // all labels together: 4 GiB

__global__ void fw_hub_count_kernel(const uint32_t* __restrict__ xadj, int32_t V, int32_t threshold, unsigned* count) {
  const int stride = gridDim.x * blockDim.x;
  unsigned local = 0;
  for (int v = blockIdx.x * blockDim.x + threadIdx.x; v < V; v += stride)
    local += (int32_t)(xadj[v + 1] - xadj[v]) > threshold ? 1u : 0u;
  if (local) atomicAdd(count, local);
}

// Hub numbers are spread: hub k of the order in which the vertices come up gets number k * spread mod n_hubs (spread is a
// prime that does not divide n_hubs, so this is a permutation).  Vertices that come up together are often busy together
// (in an R-MAT graph the busiest vertices have the lowest ids), and the counters of buckets whose numbers are neighbours
// share a 64-byte line, on which atomic updates queue behind each other.
// next[0]: the next hub number; next[1]: the next free row.  A hub of at least rows_degree elements gets rows for its
// groups (1024 elements each, from the list's first aligned quartet on) while fewer than rows_limit are taken.
__global__ void fw_hub_index_kernel(const uint32_t* __restrict__ xadj, int32_t V, int32_t threshold, unsigned* next,
                                    int32_t* hub_index, fw_hub_info* hub_info, uint32_t rows_degree,
                                    uint32_t rows_limit, uint32_t n_hubs, uint32_t spread) {
  const int stride = gridDim.x * blockDim.x;
  for (int v = blockIdx.x * blockDim.x + threadIdx.x; v < V; v += stride) {
    int32_t idx = -1;
    if ((int32_t)(xadj[v + 1] - xadj[v]) > threshold) {
      idx = (int32_t)(((unsigned long long)atomicAdd(next, 1u) * spread) % n_hubs);  // a permutation: spread is coprime with n_hubs
      fw_hub_info hi;
      hi.v = v;
      hi.off = xadj[v];
      hi.deg = xadj[v + 1] - hi.off;
      hi.row = FW_NO_ROWS;
      if (hi.deg >= rows_degree) {
        const uint32_t ngroups = ((((hi.off & 3u) + hi.deg + 3u) >> 2) + 255u) / 256u;
        const uint32_t row = atomicAdd(&next[1], ngroups);
        if (row < rows_limit && ngroups <= rows_limit - row) hi.row = row;
      }
      hub_info[idx] = hi;
    }
    // -1: not parked on; -2: no neighbours at all (a walker that arrives there is finished)
    hub_index[v] = idx >= 0 ? idx : (xadj[v + 1] == xadj[v] ? -2 : -1);
  }
}

// Every adjacency entry next to the parking index of the vertex it names.  A hub step needs both (the vertex for the
// path, the index to park the walker again), and what the kernels pay for is the number of memory requests: the pair
// sits in one 128-byte block, the entry and a look-up in hub_index are two.
__global__ void fw_adj_hub_kernel(const int32_t* __restrict__ adjncy, const int32_t* __restrict__ hub_index, uint64_t E,
                                  int2* __restrict__ adj_hub) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t e = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; e < E; e += stride) {
    const int32_t v = adjncy[e];
    adj_hub[e] = make_int2(v, hub_index[v]);
  }
}

// (Re)builds g->hub_index / hub_info / adj_hub for `threshold`; cached in the graph.
static int ensure_hub_index(fw_graph* g, int32_t threshold) {
  if (g->hub_index_threshold == threshold && g->hub_index) return FW_OK;
  if (g->hub_index) { (void)hipFree(g->hub_index); g->hub_index = nullptr; }
  if (g->hub_info) { (void)hipFree(g->hub_info); g->hub_info = nullptr; }
  if (g->adj_hub) { (void)hipFree(g->adj_hub); g->adj_hub = nullptr; }
  g->hub_index_threshold = -1;
  g->n_hubs = 0;
  unsigned* d_cnt = nullptr;
  FW_HIP(hipMalloc(reinterpret_cast<void**>(&d_cnt), 3 * sizeof(unsigned)));
  FW_HIP(hipMemset(d_cnt, 0, 3 * sizeof(unsigned)));
  hipLaunchKernelGGL(fw_hub_count_kernel, dim3(1024), dim3(256), 0, 0, g->xadj, g->V, threshold, d_cnt);
  unsigned n_hubs = 0;
  int rc = fw_check_hip(hipMemcpy(&n_hubs, d_cnt, sizeof(unsigned), hipMemcpyDeviceToHost), "hipMemcpy(hub count)", __FILE__, __LINE__);
  if (rc == FW_OK) rc = fw_check_hip(hipMalloc(reinterpret_cast<void**>(&g->hub_index), (size_t)g->V * sizeof(int32_t)), "hipMalloc(hub_index)", __FILE__, __LINE__);
  if (rc == FW_OK) rc = fw_check_hip(hipMalloc(reinterpret_cast<void**>(&g->hub_info), (size_t)(n_hubs ? n_hubs : 1) * sizeof(fw_hub_info)), "hipMalloc(hub_info)", __FILE__, __LINE__);
  uint32_t spread = 1u;
  for (uint32_t prime : {1000003u, 999983u, 999979u}) if (n_hubs > 64u && n_hubs % prime != 0u) { spread = prime; break; }
  if (rc == FW_OK) {
    hipLaunchKernelGGL(fw_hub_index_kernel, dim3(1024), dim3(256), 0, 0, g->xadj, g->V, threshold, d_cnt + 1,
                       g->hub_index, g->hub_info, kTwoPassDegree, kMaxHubRows, n_hubs ? n_hubs : 1u, spread);
    rc = fw_check_hip(hipDeviceSynchronize(), "hub index", __FILE__, __LINE__);
  }
  unsigned rows_taken = 0;
  if (rc == FW_OK) rc = fw_check_hip(hipMemcpy(&rows_taken, d_cnt + 2, sizeof(unsigned), hipMemcpyDeviceToHost), "hipMemcpy(hub rows)", __FILE__, __LINE__);
  (void)hipFree(d_cnt);
  if (rc != FW_OK) return rc;
  // the annotated adjacency is an extra: without room for it (or with the edges in host memory, where it would be
  // read over the bus) the hub kernels look the index up
  if (n_hubs != 0u && !g->host_edges) {
    if (hipMalloc(reinterpret_cast<void**>(&g->adj_hub), (size_t)g->E * sizeof(int2)) == hipSuccess) {
      hipLaunchKernelGGL(fw_adj_hub_kernel, dim3(8192), dim3(256), 0, 0, g->adjncy, g->hub_index, g->E, g->adj_hub);
      rc = fw_check_hip(hipDeviceSynchronize(), "adjacency with parking indices", __FILE__, __LINE__);
      if (rc != FW_OK) return rc;
    } else {
      (void)hipGetLastError();
      g->adj_hub = nullptr;
    }
  }
  g->n_hubs = (int32_t)n_hubs;
  g->hub_rows = rows_taken < kMaxHubRows ? rows_taken : kMaxHubRows;  // rows past the limit were not handed out
  g->hub_index_threshold = threshold;
  return FW_OK;
}

// Default parking rule (batches of at least kMinParkBatch queries): park on vertices where about kParkMeet or more
// walkers of the batch stand at the same time.  With n walkers spread in proportion to degree over E adjacency
// entries, a vertex of degree d holds about n * d / E of them, so the threshold is kParkMeet * E / n, not below
// kMinDefaultPark (shorter lists cost less to read than a record costs to move).  Edge arrays in host memory are
// read over the bus, where every shared read counts: vertices where one walker is expected, not below kMinHostPark.
constexpr int32_t kMinParkBatch = 65536;
constexpr uint32_t kParkTail = 32768;  // fewer walkers than this finish in one walk launch without parking
constexpr double kParkMeet = 4.0;
constexpr int32_t kMinDefaultPark = 64;
constexpr int32_t kMinHostPark = 16;
constexpr int32_t kMinParkThreshold = 1;
constexpr int kParkCtrs = 16;                    // counters of a parking round

// Cuts the round's buckets into tasks.  A bucket with more than two_pass_walkers walkers on a list that has rows
// is served in two passes (scan tasks of up to kScanRun groups that make the list's rows, one table task per 64
// walkers); every other bucket gets one batch task per 64 walkers:
// a workgroup task when its vertex is sampled at workgroup granularity (degree above hub_threshold), a wave task
// otherwise -- or, on a list of at most 64 aligned quartets, one quad task per 16 walkers (four of those share a
// wave).  ctrs (out): [3] workgroup tasks, [4] their dispenser, [5] wave tasks, [7] table tasks, [8] scan tasks, [9] quad tasks,
// [12] walkers in the fullest bucket when that is more than half of kTwoPassWalkers, [13] walkers served by table
// tasks, [14..15] (one 64-bit word) 16-byte quartets the round's batch and scan tasks stream.
constexpr uint32_t kScanRun = 16;

struct TaskPlan {
  int32_t hub_threshold;
  uint32_t two_pass_walkers;  // 0xFFFFFFFF: never
  int32_t quad_tasks;         // lists of at most 64 aligned quartets are served four to a wave
};

__global__ __launch_bounds__(1024) void fw_bucket_tasks_kernel(const uint32_t* __restrict__ bucket_count,
                                       const uint32_t* __restrict__ bucket_offset, int n_buckets, int labels,
                                       const fw_hub_info* __restrict__ hub_info, const TaskPlan plan,
                                       fw_batch_task* tasks, fw_batch_task* wtasks, fw_batch_task* ttasks,
                                       fw_batch_task* stasks, fw_batch_task* qtasks, uint32_t* rows_made,
                                       uint32_t* ctrs) {
  // slots and rows: one update of the (contended) global counters per workgroup and kind; inside the workgroup
  // they are dealt out by a scan over the waves' totals
  constexpr int kKinds = 5;  // workgroup, wave, table, scan, quad
  __shared__ uint32_t s_tot[kKinds][16];
  __shared__ unsigned long long s_q[16];
  __shared__ uint32_t s_base[kKinds];
  __shared__ uint32_t s_cmax;
  if (threadIdx.x == 0) s_cmax = 0u;
  __syncthreads();
  const int stride = gridDim.x * blockDim.x;
  const int lane = (int)(threadIdx.x & 63u);
  const int wave = (int)(threadIdx.x >> 6);
  const int rounds = (n_buckets + stride - 1) / stride;  // every thread runs every round: scans and barriers
  unsigned long long my_quartets = 0ull;  // traffic figures of the round: summed per thread, one update per workgroup
  uint32_t my_table_walkers = 0u;

  for (int r = 0; r < rounds; ++r) {
    const int b = r * stride + (int)(blockIdx.x * blockDim.x + threadIdx.x);
    const uint32_t c = b < n_buckets ? bucket_count[b] : 0u;
    fw_batch_task t;
    t.v = 0; t.off = 0; t.deg = 0; t.slot = 0; t.rec_base = 0; t.count = 0; t.row = 0; t.pad = 0;
    uint32_t ngroups = 0u, hub_row = FW_NO_ROWS;
    if (c != 0u) {
      const fw_hub_info hi = hub_info[b / labels];
      t.v = hi.v;
      t.off = hi.off;
      t.deg = hi.deg;
      t.slot = b % labels;
      hub_row = hi.row;
      ngroups = ((((t.off & 3u) + t.deg + 3u) >> 2) + 255u) / 256u;
    }
    {
      // the fullest bucket, for the host's decision about the next round
      uint32_t cmax = c;
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) {
        const uint32_t o = __shfl_xor(cmax, d);
        cmax = o > cmax ? o : cmax;
      }
      if (lane == 0 && cmax * 2u > kTwoPassWalkers) atomicMax(&s_cmax, cmax);  // smaller ones do not matter
    }
    const bool two_pass = c > plan.two_pass_walkers && hub_row != FW_NO_ROWS;
    if (two_pass) t.row = hub_row * (uint32_t)labels + (uint32_t)t.slot * ngroups;
    // the rows of a list do not depend on the walkers: they are made in the first round that wants them and serve
    // every later round of the call
    const bool scan = two_pass && rows_made[b] == 0u;
    if (scan) rows_made[b] = 1u;
    const bool wg = (int32_t)t.deg > plan.hub_threshold;
    const uint32_t nq_list = c != 0u ? (((t.off & 3u) + t.deg + 3u) >> 2) : 0u;
    const bool quad = plan.quad_tasks != 0 && c != 0u && !two_pass && !wg && nq_list <= 64u;
    const uint32_t per_task = quad ? 16u : 64u;
    const uint32_t nb = (c + per_task - 1u) / per_task;
    {
      // what the round's hub launches will stream: a list once per batch task, or once by the scan tasks
      const unsigned long long nq = c != 0u ? (((t.off & 3u) + t.deg + 3u) >> 2) : 0u;
      my_quartets += two_pass ? (scan ? nq : 0ull) : nq * nb;
      my_table_walkers += two_pass ? c : 0u;
    }
    uint32_t x[kKinds];
    x[0] = !two_pass && wg ? nb : 0u;
    x[1] = !two_pass && !wg && !quad ? nb : 0u;
    x[2] = two_pass ? nb : 0u;
    x[4] = quad ? nb : 0u;
    x[3] = scan ? (ngroups + kScanRun - 1u) / kScanRun : 0u;
    uint32_t inc[kKinds];
#pragma unroll
    for (int k = 0; k < kKinds; ++k) inc[k] = x[k];
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
#pragma unroll
      for (int k = 0; k < kKinds; ++k) {
        const uint32_t up = __shfl_up(inc[k], d);
        if (lane >= d) inc[k] += up;
      }
    }
    if (lane == 63) {
#pragma unroll
      for (int k = 0; k < kKinds; ++k) s_tot[k][wave] = inc[k];
    }
    __syncthreads();
    if (threadIdx.x == kKinds && s_cmax != 0u) {  // one update of the global maximum per workgroup
      atomicMax(&ctrs[12 * FW_CTR_STRIDE], s_cmax);
      s_cmax = 0u;
    }
    if (threadIdx.x < kKinds) {
      uint32_t total = 0u;
      for (int w = 0; w < 16; ++w) {  // exclusive prefix over the waves, in place
        const uint32_t v = s_tot[threadIdx.x][w];
        s_tot[threadIdx.x][w] = total;
        total += v;
      }
      const int ctr = threadIdx.x == 0 ? 3 : (threadIdx.x == 1 ? 5 : (threadIdx.x == 2 ? 7 : (threadIdx.x == 3 ? 8 : 9)));
      s_base[threadIdx.x] = total != 0u ? atomicAdd(&ctrs[ctr * FW_CTR_STRIDE], total) : 0u;
    }
    __syncthreads();
    const int kind = two_pass ? 2 : (wg ? 0 : (quad ? 4 : 1));
    // (selected, not indexed: the arrays stay in registers)
    const uint32_t mine = two_pass ? inc[2] - x[2] : (wg ? inc[0] - x[0] : (quad ? inc[4] - x[4] : inc[1] - x[1]));
    const uint32_t t0 = s_base[kind] + s_tot[kind][wave] + mine;
    const uint32_t base = c != 0u ? bucket_offset[b] : 0u;
    // a crowded bucket has thousands of tasks: those are written by the whole wave, one bucket after the other
    constexpr uint32_t kOwnTasks = 8;
    for (uint64_t big = __ballot(nb > kOwnTasks); big != 0ull; big &= big - 1ull) {
      const int l = __builtin_ctzll(big);
      fw_batch_task bt;
      bt.v = __shfl(t.v, l); bt.off = __shfl(t.off, l); bt.deg = __shfl(t.deg, l); bt.slot = __shfl(t.slot, l);
      bt.row = __shfl(t.row, l); bt.pad = 0;
      const uint32_t bc = __shfl(c, l), bbase = __shfl(base, l), bt0 = __shfl(t0, l), bnb = __shfl(nb, l);
      const int bkind = __shfl(kind, l);
      const uint32_t bper = bkind == 4 ? 16u : 64u;
      fw_batch_task* bout = bkind == 0 ? tasks : (bkind == 1 ? wtasks : (bkind == 2 ? ttasks : qtasks));
      for (uint32_t k = (uint32_t)lane; k < bnb; k += 64u) {
        bt.rec_base = bbase + bper * k;
        bt.count = (int32_t)(bc - bper * k < bper ? bc - bper * k : bper);
        bout[bt0 + k] = bt;
      }
    }
    if (c != 0u) {
      fw_batch_task* out = kind == 0 ? tasks : (kind == 1 ? wtasks : (kind == 2 ? ttasks : qtasks));
      for (uint32_t k = 0; k < (nb > kOwnTasks ? 0u : nb); ++k) {
        t.rec_base = base + per_task * k;
        t.count = (int32_t)(c - per_task * k < per_task ? c - per_task * k : per_task);
        out[t0 + k] = t;
      }
      if (scan) {
        const uint32_t s0 = s_base[3] + s_tot[3][wave] + inc[3] - x[3];
        for (uint32_t k = 0; k < x[3]; ++k) {
          t.rec_base = k * kScanRun;
          t.count = (int32_t)((k + 1u) * kScanRun < ngroups ? (k + 1u) * kScanRun : ngroups);
          stasks[s0 + k] = t;
        }
      }
    }
    __syncthreads();  // s_tot / s_base are reused by the next round
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    my_quartets += __shfl_xor(my_quartets, d);
    my_table_walkers += __shfl_xor(my_table_walkers, d);
  }
  if (lane == 0) {
    s_q[wave] = my_quartets;
    s_tot[2][wave] = my_table_walkers;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long q = 0ull;
    uint32_t tw = 0u;
    for (int w = 0; w < (int)(blockDim.x >> 6); ++w) {
      q += s_q[w];
      tw += s_tot[2][w];
    }
    if (q != 0ull) atomicAdd(reinterpret_cast<unsigned long long*>(ctrs + 14 * FW_CTR_STRIDE), q);
    if (tw != 0u) atomicAdd(&ctrs[13 * FW_CTR_STRIDE], tw);
  }
}

// Zeroes what a parking round starts from, in one launch: the round's counters, the next round's bucket counts, the
// fill positions the scatter above has used, and the query dispenser.
__global__ void fw_round_reset_kernel(uint32_t* ctrs, int n_ctrs, uint32_t* count_next, uint32_t* fill, int n_buckets,
                                      uint32_t* dispenser) {
  const int stride = gridDim.x * blockDim.x;
  const int i0 = blockIdx.x * blockDim.x + threadIdx.x;
  if (i0 < n_ctrs) ctrs[i0] = 0u;
  if (i0 == 0) *dispenser = 0u;
  for (int i = i0; i < n_buckets; i += stride) {
    count_next[i] = 0u;
    fill[i] = 0u;
  }
}

// A record read that is not worth an L2 slot: the lists of records are streamed once per round, and what the L2
// should keep are the small tables the same kernels look up per record (bucket offsets, counters).
typedef int fw_v4i __attribute__((ext_vector_type(4)));
__device__ __forceinline__ fw_walker_rec load_rec_streaming(const fw_walker_rec* p) {
  const fw_v4i v = __builtin_nontemporal_load(reinterpret_cast<const fw_v4i*>(p));
  fw_walker_rec r;
  r.q = v.x; r.cur = v.y; r.prev = v.z; r.len = v.w;
  return r;
}

// Counting-sort scatter of a round's parked walkers into `sorted`.  Two sources share a bucket's range:
//  * the previous batch launch's output list, of which only the records tagged FW_REC_PARK are parked; they carry
//    their bucket and their position inside it (taken when they were parked) and fill the range from its start;
//  * the walk kernel's list, whose records were only counted; they take positions from the end of the range here.
__global__ void fw_scatter_tagged_kernel(const fw_walker_rec* __restrict__ src, uint32_t m,
                                         const uint32_t* __restrict__ bucket_offset,
                                         fw_parked_rec* __restrict__ sorted) {
  const uint32_t stride = gridDim.x * blockDim.x;
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < m; i += stride) {
    const fw_walker_rec r = load_rec_streaming(src + i);
    if (r.q < 0 || (r.len & FW_REC_PARK) == 0) continue;
    fw_parked_rec p;
    p.q = r.q;
    p.len = r.len & ~FW_REC_PARK;
    sorted[bucket_offset[r.cur] + (uint32_t)r.prev] = p;
  }
}

// tagged_only (node2vec, whose records carry the previous vertex instead of a position): src is a batch launch's
// output list, of which only the records tagged FW_REC_PARK take part.  whole (node2vec): the sorted list holds
// fw_walker_rec, otherwise fw_parked_rec.
// m_dev: when not NULL the number of entries is read there (m is an upper bound the grid was sized for): the launch
// is queued before the host has seen the counters of the round that made the list.
__global__ void fw_scatter_counted_kernel(const fw_walker_rec* __restrict__ src, uint32_t m,
                                          const uint32_t* __restrict__ m_dev,
                                          const uint32_t* __restrict__ bucket_count,
                                          const uint32_t* __restrict__ bucket_offset, uint32_t* bucket_fill,
                                          void* __restrict__ sorted, int tagged_only, int whole) {
  if (m_dev != nullptr) m = *m_dev < m ? *m_dev : m;
  const uint32_t stride = gridDim.x * blockDim.x;
  for (uint32_t i0 = blockIdx.x * blockDim.x; i0 < m; i0 += stride) {  // uniform in the wave: the ranks are taken together
    const uint32_t i = i0 + threadIdx.x;
    bool have = i < m;
    fw_walker_rec r;
    r.q = 0; r.cur = 0; r.prev = 0; r.len = 0;
    if (have) r = load_rec_streaming(src + i);
    have = have && r.q >= 0;  // both lists have holes
    if (tagged_only) {
      have = have && (r.len & FW_REC_PARK) != 0;
      r.len &= ~FW_REC_PARK;
    }
    const uint32_t b = (uint32_t)r.cur;
    const uint32_t rank = fw_wave_count_keys<true>(bucket_fill, b, have);
    if (have) {
      const uint32_t at = bucket_offset[b] + bucket_count[b] - 1u - rank;
      if (whole) {  // node2vec
        static_cast<fw_walker_rec*>(sorted)[at] = r;
      } else {
        fw_parked_rec p;
        p.q = r.q;
        p.len = r.len;
        static_cast<fw_parked_rec*>(sorted)[at] = p;
      }
    }
  }
}

// Copies the records of a batch launch's output list that continue in the walk kernel (not finished, not parked
// again) to a dense list, so that the walk kernel's refill rounds do not scan the holes.  One update of the
// (contended) list counter per 4096 records.
__global__ __launch_bounds__(1024) void fw_compact_resume_kernel(const fw_walker_rec* __restrict__ out, uint32_t m,
                                                                 fw_walker_rec* __restrict__ resume, uint32_t* count) {
  __shared__ uint32_t s_wave[16];
  __shared__ uint32_t s_base;
  const int lane = (int)(threadIdx.x & 63u);
  const int wave = (int)(threadIdx.x >> 6);
  for (uint32_t base = blockIdx.x * 4096u; base < m; base += gridDim.x * 4096u) {  // uniform per workgroup
    fw_walker_rec r[4];
    uint32_t n = 0u;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t i = base + (uint32_t)k * 1024u + threadIdx.x;
      r[k].q = -1; r[k].cur = 0; r[k].prev = 0; r[k].len = 0;
      if (i < m) r[k] = out[i];
      if (r[k].q < 0 || (r[k].len & FW_REC_PARK) != 0) r[k].q = -1;
      n += r[k].q >= 0 ? 1u : 0u;
    }
    uint32_t incl = n;  // inclusive wave scan
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const uint32_t up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t total = 0u;
      for (int w = 0; w < 16; ++w) {
        const uint32_t v = s_wave[w];
        s_wave[w] = total;
        total += v;
      }
      s_base = total != 0u ? atomicAdd(count, total) : 0u;
    }
    __syncthreads();
    uint32_t at = s_base + s_wave[wave] + incl - n;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (r[k].q >= 0) resume[at++] = r[k];
    }
    __syncthreads();  // s_wave / s_base are reused by the next chunk
  }
}

// When the last few walkers leave the park / batch loop they take their next steps in the walk kernel, which wants
// whole records that name the vertex.  Sorted record i belongs to the last bucket whose offset is at most i (empty
// buckets share their offset with the next one that is not); node2vec's records name their bucket themselves.  The
// batch kernel may have left the path entry of a walker it parked again to the walker's next step there (entries are
// stored in pairs), so the entry is stored here.
__global__ void fw_bucket_to_vertex_kernel(const void* sorted, uint32_t m, const uint32_t* __restrict__ bucket_offset,
                                           int n_buckets, const fw_hub_info* __restrict__ hub_info, int labels,
                                           int32_t* __restrict__ paths, int32_t max_depth, int n2v,
                                           fw_walker_rec* __restrict__ whole) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= m) return;
  fw_walker_rec r;
  uint32_t bucket;
  if (n2v != 0) {
    r = static_cast<const fw_walker_rec*>(sorted)[i];
    bucket = (uint32_t)r.cur;
  } else {
    const fw_parked_rec p = static_cast<const fw_parked_rec*>(sorted)[i];
    uint32_t lo = 0u, hi = (uint32_t)n_buckets;  // first bucket whose offset is above i
    while (lo < hi) {
      const uint32_t mid = (lo + hi) >> 1;
      if (bucket_offset[mid] > i) hi = mid; else lo = mid + 1u;
    }
    bucket = lo - 1u;  // lo >= 1: offset[0] = 0 <= i
    r.q = p.q; r.prev = -1; r.len = p.len;
  }
  const int32_t v = hub_info[bucket / (uint32_t)labels].v;
  r.cur = v;
  whole[i] = r;
  const int32_t len = n2v != 0 ? (r.len & FW_REC_LEN_MASK) : r.len;
  if (r.q >= 0 && len >= 1) paths[(uint64_t)(uint32_t)r.q * (uint64_t)max_depth + (uint64_t)(len - 1)] = v;
}

// Device buffers of one park / batch / resume loop (one per stream in flight).  Three record lists: `walked`
// (walkers parked by the walk kernel), `sorted` (a round's parked walkers grouped by bucket, the batch kernel's
// input) and `out` (the batch kernel's output, one record per input record: finished / resumes / parked again).
// The bucket counts are double buffered: a round's batch and walk launches count the next round's walkers.
struct ParkBuffers {
  size_t cap = 0;       // walkers
  int n_buckets = 0;
  fw_walker_rec* walked = nullptr;
  fw_walker_rec* sorted = nullptr;
  fw_walker_rec* out = nullptr;
  fw_walker_rec* resume = nullptr;    // the records of `out` that continue in the walk kernel, dense
  uint32_t* buckets = nullptr;        // [5 * n_buckets]: count of round parity 0, of parity 1, offset, fill, and
                                      // whether the bucket's rows have been made in this call
  fw_batch_task* tasks = nullptr;
  fw_batch_task* wtasks = nullptr;
  fw_batch_task* qtasks = nullptr;    // quad tasks: up to 16 walkers each
  uint32_t* ctrs = nullptr;           // [0] walkers in `walked`, [1] records of `out` that resume, [2] that are parked
                                      // again, [3] workgroup tasks, [4] their dispenser, [5] wave tasks, [6] records in
                                      // `resume`, [7] table tasks, [8] scan tasks, [12] walkers in the fullest bucket
  fw_batch_task* ttasks = nullptr;    // two-pass steps: table tasks, scan tasks and the rows between them
  fw_batch_task* stasks = nullptr;
  float* totals = nullptr;
  float* rows = nullptr;
  int32_t* lastpos = nullptr;
  uint32_t rows_cap = 0;              // rows allocated (0: no two-pass steps)
  uint32_t* h_ctrs = nullptr;         // pinned mirror
  void* tmp = nullptr;                // scan temporary storage
  size_t scan_bytes = 0;
  hipEvent_t ev[4] = {nullptr, nullptr, nullptr, nullptr};  // timing events of the walk and the hub launches
  hipStream_t side = nullptr;          // the quad launch of a round runs beside the batch launch
  hipEvent_t fork = nullptr, join = nullptr;
  hipEvent_t copied = nullptr;         // the round's counters have reached the host

  uint32_t* count(int parity) const { return buckets + (size_t)parity * n_buckets; }
  uint32_t* offset() const { return buckets + (size_t)2 * n_buckets; }
  uint32_t* fill() const { return buckets + (size_t)3 * n_buckets; }
  uint32_t* rows_made() const { return buckets + (size_t)4 * n_buckets; }

  int alloc(size_t walkers, int n, uint64_t rows_wanted) {
    cap = walkers;
    n_buckets = n;
    const size_t ntask = cap / 64 + (size_t)n + 1;
    FW_HIP(hipMalloc(reinterpret_cast<void**>(&walked), cap * sizeof(fw_walker_rec)));
    FW_HIP(hipMalloc(reinterpret_cast<void**>(&sorted), cap * sizeof(fw_walker_rec)));
    FW_HIP(hipMalloc(reinterpret_cast<void**>(&out), cap * sizeof(fw_walker_rec)));
    FW_HIP(hipMalloc(reinterpret_cast<void**>(&resume), cap * sizeof(fw_walker_rec)));
    FW_HIP(hipMalloc(reinterpret_cast<void**>(&buckets), (size_t)5 * n * sizeof(uint32_t)));
    FW_HIP(hipMalloc(reinterpret_cast<void**>(&tasks), ntask * sizeof(fw_batch_task)));
    FW_HIP(hipMalloc(reinterpret_cast<void**>(&wtasks), ntask * sizeof(fw_batch_task)));
    FW_HIP(hipMalloc(reinterpret_cast<void**>(&qtasks), (cap / 16 + (size_t)n + 1) * sizeof(fw_batch_task)));
    FW_HIP(hipMalloc(reinterpret_cast<void**>(&ctrs), kParkCtrs * FW_CTR_STRIDE * sizeof(uint32_t)));
    FW_HIP(hipHostMalloc(reinterpret_cast<void**>(&h_ctrs), kParkCtrs * FW_CTR_STRIDE * sizeof(uint32_t), hipHostMallocDefault));
    for (hipEvent_t& e : ev) FW_HIP(hipEventCreate(&e));
    FW_HIP(hipStreamCreateWithFlags(&side, hipStreamNonBlocking));
    FW_HIP(hipEventCreateWithFlags(&fork, hipEventDisableTiming));
    FW_HIP(hipEventCreateWithFlags(&join, hipEventDisableTiming));
    FW_HIP(hipEventCreateWithFlags(&copied, hipEventDisableTiming));
    // the rows are an extra: without room for them every bucket is served by batch tasks
    if (rows_wanted != 0u) {
      // scan tasks: a list of G groups is cut into at most G / kScanRun + 1 runs, and no more lists are scanned in
      // a round than there are buckets or walkers
      const size_t nscan = (size_t)(rows_wanted / kScanRun) + ((size_t)n < cap ? (size_t)n : cap) + 1;
      if (hipMalloc(reinterpret_cast<void**>(&ttasks), ntask * sizeof(fw_batch_task)) == hipSuccess &&
          hipMalloc(reinterpret_cast<void**>(&stasks), nscan * sizeof(fw_batch_task)) == hipSuccess &&
          hipMalloc(reinterpret_cast<void**>(&totals), (size_t)rows_wanted * sizeof(float)) == hipSuccess &&
          hipMalloc(reinterpret_cast<void**>(&lastpos), (size_t)rows_wanted * sizeof(int32_t)) == hipSuccess &&
          hipMalloc(reinterpret_cast<void**>(&rows), (size_t)rows_wanted * 128 * sizeof(float)) == hipSuccess) {
        rows_cap = (uint32_t)rows_wanted;
      } else {
        (void)hipGetLastError();
        release_rows();
      }
    }
    FW_HIP(rocprim::exclusive_scan(nullptr, scan_bytes, count(0), offset(), 0u, (size_t)n,
                                   rocprim::plus<uint32_t>(), (hipStream_t)0));
    FW_HIP(hipMalloc(&tmp, scan_bytes ? scan_bytes : 16));
    return FW_OK;
  }
  void release_rows() {
    void* dev[5] = {ttasks, stasks, totals, lastpos, rows};
    for (void* p : dev) if (p) (void)hipFree(p);
    ttasks = stasks = nullptr;
    totals = rows = nullptr;
    lastpos = nullptr;
    rows_cap = 0;
  }
  void release() {
    release_rows();
    void* dev[10] = {walked, sorted, out, resume, buckets, tasks, wtasks, qtasks, ctrs, tmp};
    for (void* p : dev) if (p) (void)hipFree(p);
    if (h_ctrs) (void)hipHostFree(h_ctrs);
    for (hipEvent_t& e : ev) {
      if (e) (void)hipEventDestroy(e);
      e = nullptr;
    }
    if (side) (void)hipStreamDestroy(side);
    if (fork) (void)hipEventDestroy(fork);
    if (join) (void)hipEventDestroy(join);
    if (copied) (void)hipEventDestroy(copied);
    side = nullptr;
    fork = join = copied = nullptr;
    walked = sorted = out = resume = nullptr;
    buckets = ctrs = h_ctrs = nullptr;
    tasks = wtasks = qtasks = nullptr;
    tmp = nullptr;
  }
};

static void release_park_cache(fw_graph* g) {
  ParkBuffers* c = static_cast<ParkBuffers*>(g->park_cache);
  if (c) {
    c->release();
    delete c;
  }
  g->park_cache = nullptr;
}

// The parking lists for a call over n queries with n_buckets buckets: the graph keeps the last set (a call pays ten
// allocations otherwise, which is a fifth of a 7 ms pass); it is replaced when it is too small or shaped differently.
// NULL when the memory is not there (the caller then walks without parking).
static ParkBuffers* cached_park_buffers(fw_graph* g, size_t n, int n_buckets, uint64_t rows_wanted) {
  ParkBuffers* c = static_cast<ParkBuffers*>(g->park_cache);
  if (c && c->cap >= n && c->n_buckets == n_buckets && c->rows_cap >= rows_wanted) return c;
  release_park_cache(g);
  c = new (std::nothrow) ParkBuffers;
  if (!c) return nullptr;
  if (c->alloc(n, n_buckets, rows_wanted) != FW_OK) {
    c->release();
    delete c;
    (void)hipGetLastError();
    return nullptr;
  }
  g->park_cache = c;
  return c;
}

struct Scratch {  // dispenser word + workload counters of the two kernels, 48 bytes per launch slot
  uint32_t dispenser;
  uint32_t pad;
  unsigned long long counters[4];
  unsigned long long pad2;
};

// The device side of fw_walk_batch: start vertices and path matrices of the batches in flight, their parking lists,
// launch records, streams and events.  Kept with the graph from one call to the next and only ever grown.  A call that
// allocated and freed them itself would cost the NEXT call's copy of the path matrix half its rate: memory that was
// just freed keeps the device's copy engines busy for a few hundred milliseconds (measured: the 5.4 GB path matrix
// of the largest benchmark configuration crosses the bus in 95 ms, and in 178 ms when 14 GB were freed 125 ms before).
struct BatchCache {
  int32_t* d_starts = nullptr;
  int32_t* d_paths = nullptr;
  Scratch* d_scr = nullptr;
  size_t starts_cap = 0, paths_cap = 0, scr_cap = 0;  // elements
  ParkBuffers pbs[2];
  hipStream_t streams[2] = {nullptr, nullptr};
  std::vector<hipEvent_t> events;
  size_t bytes() const {
    size_t b = starts_cap * sizeof(int32_t) + paths_cap * sizeof(int32_t) + scr_cap * sizeof(Scratch);
    for (const ParkBuffers& pb : pbs) b += pb.cap * 72u;  // about what the lists of a query take
    return b;
  }
  void release() {
    if (d_starts) (void)hipFree(d_starts);
    if (d_paths) (void)hipFree(d_paths);
    if (d_scr) (void)hipFree(d_scr);
    d_starts = d_paths = nullptr;
    d_scr = nullptr;
    starts_cap = paths_cap = scr_cap = 0;
    for (ParkBuffers& pb : pbs) pb.release();
    for (hipStream_t& s : streams) {
      if (s) (void)hipStreamDestroy(s);
      s = nullptr;
    }
    for (hipEvent_t e : events) (void)hipEventDestroy(e);
    events.clear();
  }
};

static void release_batch_cache(fw_graph* g) {
  BatchCache* c = static_cast<BatchCache*>(g->batch_cache);
  if (c) {
    c->release();
    delete c;
  }
  g->batch_cache = nullptr;
}

// Rows the two-pass steps of a call need: every hub that has rows, once per label a walker can want.
static uint64_t two_pass_rows(const fw_graph* g, int labels) {
  const uint64_t rows = (uint64_t)g->hub_rows * (uint64_t)labels;
  return rows <= kMaxRows ? rows : 0;  // too many: no two-pass steps in this call
}

// Decides whether a call parks walkers, and at which degree.  Returns INT_MAX for "no".
static int32_t resolve_park_threshold(const fw_graph* g, const fw_walk_params* p, int32_t n) {
  // node2vec's proposals do not depend on the walker, so its walkers share scans like the others; their records keep
  // the path length in 16 bits
  if (p->app == FW_APP_NODE2VEC && p->max_depth > FW_REC_LEN_MASK) return INT_MAX;
  if (p->sampler != FW_SAMPLER_ZPRS && p->sampler != FW_SAMPLER_DPRS) return INT_MAX;  // the reference's engine: one launch
  if (p->park_threshold < 0) return INT_MAX;
  if (p->park_threshold == 0) {
    if (n < kMinParkBatch) return INT_MAX;  // too few walkers to meet
    const double t = (g->host_edges ? 1.0 : kParkMeet) * (double)g->E / (double)n;
    if (t >= 2.0e9) return INT_MAX;
    const int32_t floor_deg = g->host_edges ? kMinHostPark : kMinDefaultPark;
    return t < (double)floor_deg ? floor_deg : (int32_t)t;
  }
  return p->park_threshold < kMinParkThreshold ? kMinParkThreshold : p->park_threshold;
}

// Runs all walks of one batch on `stream`: a single walk launch, or the park / batch / resume loop.
// `a` is complete except for the parking fields; a.dispenser / a.counters point at zeroed memory.
struct KernelTimes {
  double walk_ms = 0.0;
  double hub_ms = 0.0;
  // what the parking pipeline asked of the memory system beyond the walk launches' own steps (see requested_bytes)
  uint64_t hub_quartets = 0;     // 16-byte quartets streamed by batch and scan tasks
  uint64_t table_walkers = 0;    // walkers served from a crowded hub's rows
  uint64_t parked_records = 0;   // records parked by walk launches
  uint64_t resume_entries = 0;   // records read back by walk launches
  uint64_t sorted_records = 0;   // records moved by the counting sort (one per walker and round)
  uint64_t bucket_passes = 0;    // buckets x rounds (scan, reset, task list)
};

// Records one event pair around a launch and adds its duration to *acc after the next stream sync.  The events belong
// to the parking buffers (created once with them, not per launch).
struct TimedLaunch {
  hipEvent_t e0 = nullptr, e1 = nullptr;
  bool enabled = true;  // an event costs the stream about 5 us: the per-kernel split is measured on request only
  bool open = false;
  int begin(hipStream_t s) {
    if (!enabled) return FW_OK;
    FW_HIP(hipEventRecord(e0, s));
    open = true;
    return FW_OK;
  }
  int end(hipStream_t s) {
    if (enabled) FW_HIP(hipEventRecord(e1, s));
    return FW_OK;
  }
  void collect(double* acc) {  // call after the stream has been synchronised
    float ms = 0.0f;
    if (open && hipEventElapsedTime(&ms, e0, e1) == hipSuccess) *acc += ms;
    else (void)hipGetLastError();
    open = false;
  }
};

static int run_walk_launches(const fw_graph* g, const fw_walk_params* p, fw_kargs a, int32_t park_threshold,
                             ParkBuffers* pb, hipStream_t stream, int* grid_used, int* launches,
                             KernelTimes* times) {
  *launches = 0;
  if (park_threshold == INT_MAX || g->n_hubs == 0 || pb == nullptr) {
    *launches = 1;
    return fw_launch_walk(a, p->app, p->sampler, p->wg_threads, p->grid, 0u, stream, grid_used);
  }
  const int labels = p->app == FW_APP_METAPATH ? p->schema_len : 1;
  a.park_threshold = park_threshold;
  a.n_labels_per_hub = labels;
  a.hub_index = g->hub_index;
  a.adj_hub = g->adj_hub;
  a.parked = pb->walked;
  a.parked_count = &pb->ctrs[0 * FW_CTR_STRIDE];
  fw_hub_args h;
  h.sorted = pb->sorted;
  h.tasks = pb->tasks;
  h.ntasks = &pb->ctrs[3 * FW_CTR_STRIDE];
  h.task_next = &pb->ctrs[4 * FW_CTR_STRIDE];
  h.dynamic_wgs = 0u;
  h.wtasks = pb->wtasks;
  h.nwtasks = &pb->ctrs[5 * FW_CTR_STRIDE];
  h.out = pb->out;
  h.out_counts = &pb->ctrs[1 * FW_CTR_STRIDE];
  h.stasks = pb->stasks;
  h.nstasks = &pb->ctrs[8 * FW_CTR_STRIDE];
  h.ttasks = pb->ttasks;
  h.nttasks = &pb->ctrs[7 * FW_CTR_STRIDE];
  h.qtasks = pb->qtasks;
  h.nqtasks = &pb->ctrs[9 * FW_CTR_STRIDE];
  h.totals = pb->totals;
  h.rows = pb->rows;
  h.lastpos = pb->lastpos;
  TaskPlan plan;
  plan.hub_threshold = p->hub_threshold;
  plan.quad_tasks = 1;
  // Two-pass steps cost a launch per round that looks for scan tasks, so a round only gets them when the round
  // before had a bucket at least half as full as they need (the first round always does): a bucket may then miss
  // them for a round and is served by batches, with the same results.
  const bool two_pass_possible = pb->rows_cap != 0u;
  plan.two_pass_walkers = two_pass_possible ? kTwoPassWalkers : 0xFFFFFFFFu;

  // Queues one walk launch (timed); the caller reads the counters back.
  TimedLaunch tw;
  tw.e0 = pb->ev[0];
  tw.e1 = pb->ev[1];
  tw.enabled = p->time_kernels != 0;
  uint32_t entries_hint = 0u;  // set before every queue_walk
  // the hint counts entries of the kind the grid rule was made for, lists of up to 124 neighbours (four or two to a
  // wave); with a higher parking threshold an entry is more work, about in proportion
  auto hint_for = [&](uint64_t entries) -> uint32_t {
    const uint64_t scaled = park_threshold > 124 ? entries * (uint64_t)park_threshold / 124u : entries;
    return scaled < 0x7FFFFFFFull ? (uint32_t)scaled : 0x7FFFFFFFu;
  };
  auto queue_walk = [&](int* grid_out) -> int {
    int rc = tw.begin(stream);
    if (rc != FW_OK) return rc;
    rc = fw_launch_walk(a, p->app, p->sampler, p->wg_threads, p->grid, entries_hint, stream, grid_out);
    if (rc != FW_OK) return rc;
    if ((rc = tw.end(stream)) != FW_OK) return rc;
    ++*launches;
    return FW_OK;
  };
  // The counters of a round go to the host once per round.  Behind the copy, before the host waits for it, the part of
  // the next round that needs nothing from the host is queued already -- the bucket scan, the counting sort of the
  // parked walkers and the reset of the round's counters -- so the device works through the host's round trip.
  auto copy_counters = [&]() -> int {
    FW_HIP(hipMemcpyAsync(pb->h_ctrs, pb->ctrs, kParkCtrs * FW_CTR_STRIDE * sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
    FW_HIP(hipEventRecord(pb->copied, stream));
    return FW_OK;
  };
  auto wait_counters = [&]() -> int {
    FW_HIP(hipEventSynchronize(pb->copied));
    return FW_OK;
  };
  auto read_back = [&]() -> int {  // for the last launch of a call: nothing follows
    int rc_ = copy_counters();
    return rc_ != FW_OK ? rc_ : wait_counters();
  };
  unsigned rblocks = ((unsigned)pb->n_buckets + 255u) / 256u;
  if (rblocks > 2048u) rblocks = 2048u;
  if (rblocks == 0u) rblocks = 1u;
  auto blocks_for = [](uint32_t cnt) {
    unsigned blocks = (cnt + 255u) / 256u;
    return blocks > 8192u ? 8192u : (blocks ? blocks : 1u);
  };
  // The sort of the walkers parked for the coming round (bucket counts in array `cnt`): n_tagged records of the last
  // batch launch's output list (0: there was none) and the last walk launch's list of n_entries positions at most (the
  // exact number on the device at entries_dev when not NULL); then the counters start the round at zero and array
  // `nxt` is cleared for the walkers the round will park.
  auto queue_sort = [&](int cnt, int nxt, uint32_t n_tagged, uint32_t n_entries, const uint32_t* entries_dev) -> int {
    FW_HIP(rocprim::exclusive_scan(pb->tmp, pb->scan_bytes, pb->count(cnt), pb->offset(), 0u, (size_t)pb->n_buckets,
                                   rocprim::plus<uint32_t>(), stream));
    if (n_tagged != 0u) {
      if (p->app == FW_APP_NODE2VEC)
        hipLaunchKernelGGL(fw_scatter_counted_kernel, dim3(blocks_for(n_tagged)), dim3(256), 0, stream, pb->out, n_tagged,
                           static_cast<const uint32_t*>(nullptr), pb->count(cnt), pb->offset(), pb->fill(), pb->sorted, 1, 1);
      else
        hipLaunchKernelGGL(fw_scatter_tagged_kernel, dim3(blocks_for(n_tagged)), dim3(256), 0, stream, pb->out, n_tagged,
                           pb->offset(), reinterpret_cast<fw_parked_rec*>(pb->sorted));
    }
    if (n_entries != 0u)  // the walk launch's list has one position per entry of its input: parked walkers and holes
      hipLaunchKernelGGL(fw_scatter_counted_kernel, dim3(blocks_for(n_entries)), dim3(256), 0, stream, pb->walked,
                         n_entries, entries_dev, pb->count(cnt), pb->offset(), pb->fill(), pb->sorted, 0,
                         p->app == FW_APP_NODE2VEC ? 1 : 0);
    hipLaunchKernelGGL(fw_round_reset_kernel, dim3(rblocks), dim3(256), 0, stream, pb->ctrs, kParkCtrs * FW_CTR_STRIDE, pb->count(nxt),
                       pb->fill(), pb->n_buckets, a.dispenser);
    FW_HIP(hipGetLastError());
    return FW_OK;
  };

  if (two_pass_possible) {  // no bucket has rows yet
    hipLaunchKernelGGL(fw_fill_i32_kernel, dim3(rblocks), dim3(256), 0, stream, reinterpret_cast<int32_t*>(pb->rows_made()),
                       0, (size_t)pb->n_buckets);
    FW_HIP(hipGetLastError());
  }
  // first walk launch: fresh queries; the walkers it parks are counted in bucket array 0
  int cur = 0;
  hipLaunchKernelGGL(fw_round_reset_kernel, dim3(rblocks), dim3(256), 0, stream, pb->ctrs, kParkCtrs * FW_CTR_STRIDE, pb->count(0),
                     pb->fill(), pb->n_buckets, a.dispenser);
  FW_HIP(hipGetLastError());
  a.resume = nullptr;
  a.n_dev = nullptr;
  a.bucket_count = pb->count(0);
  entries_hint = hint_for((uint64_t)a.n);
  int rc = queue_walk(grid_used);
  if (rc != FW_OK) return rc;
  if ((rc = copy_counters()) != FW_OK) return rc;
  if ((rc = queue_sort(0, 1, 0u, (uint32_t)a.n, nullptr)) != FW_OK) return rc;
  if ((rc = wait_counters()) != FW_OK) return rc;
  tw.collect(&times->walk_ms);
  times->parked_records += pb->h_ctrs[0 * FW_CTR_STRIDE];
  uint32_t n_out = 0;  // records in `out` (the previous batch launch's input size)
  uint32_t walk_entries = (uint32_t)a.n;  // entries of the last walk launch's input = positions of its list of parked walkers
  uint32_t fullest = 0;  // walkers in the fullest bucket of the previous round
  uint32_t scan_tasks = 0;  // and its scan tasks
  uint32_t quad_tasks = 0;  // and its quad tasks
  uint32_t resumed = 0;     // and the walkers that went on in its walk launch
  uint32_t batch_tasks = 0; // and its batch tasks, in waves
  uint32_t wg_task_waves = 0;  // of which workgroup tasks
  for (;;) {
    // one round: the walkers parked by the last walk launch and by the last batch launch are grouped by bucket, the
    // batch launch moves each of them one step, and the walk launch queued right behind it takes those that are
    // not parked again as far as their next parking.  The host looks at the counters once per round.
    const uint32_t n_walked = pb->h_ctrs[0 * FW_CTR_STRIDE];                 // parked by the walk launch
    const uint32_t n_again = n_out ? pb->h_ctrs[2 * FW_CTR_STRIDE] : 0u;     // parked again by the previous batch launch
    const uint64_t m = (uint64_t)n_walked + n_again;
    if (m == 0u) break;
    if (m > pb->cap) { fw_set_error("internal: %llu walkers parked, capacity %zu", (unsigned long long)m, pb->cap); return FW_ERR_INVALID; }
    const int nxt = cur ^ 1;
    // (the scan of this round's buckets, the sort of its walkers and the reset of its counters are queued already)
    if (p->park_threshold == 0 && m < kParkTail) {
      // default rule only (an explicit threshold keeps every round in the loop): too few walkers are left to
      // meet anywhere, so they finish in one walk launch that does not park
      hipLaunchKernelGGL(fw_bucket_to_vertex_kernel, dim3(((unsigned)m + 255u) / 256u), dim3(256), 0, stream,
                         pb->sorted, (uint32_t)m, pb->offset(), pb->n_buckets, g->hub_info, labels, a.paths,
                         a.max_depth, p->app == FW_APP_NODE2VEC ? 1 : 0, pb->resume);
      FW_HIP(hipGetLastError());
      a.resume = pb->resume;
      a.n_dev = nullptr;
      a.n = (int32_t)m;
      a.park_threshold = INT_MAX;
      entries_hint = 0u;  // these walkers run to the end of their walks: every workgroup is wanted
      if ((rc = queue_walk(nullptr)) != FW_OK) return rc;
      if ((rc = read_back()) != FW_OK) return rc;
      tw.collect(&times->walk_ms);
      times->resume_entries += m;
      times->sorted_records += m;
      times->bucket_passes += (uint64_t)pb->n_buckets;
      return FW_OK;
    }
    plan.two_pass_walkers = two_pass_possible && (n_out == 0u || fullest * 2u > kTwoPassWalkers) ? kTwoPassWalkers : 0xFFFFFFFFu;
    unsigned tblocks = ((unsigned)pb->n_buckets + 1023u) / 1024u;
    if (tblocks > 1024u) tblocks = 1024u;
    hipLaunchKernelGGL(fw_bucket_tasks_kernel, dim3(tblocks), dim3(1024), 0, stream, pb->count(cur), pb->offset(),
                       pb->n_buckets, labels, g->hub_info, plan, pb->tasks, pb->wtasks, pb->ttasks, pb->stasks,
                       pb->qtasks, pb->rows_made(), pb->ctrs);
    FW_HIP(hipGetLastError());
    h.bucket_out = pb->count(nxt);
    TimedLaunch th;
    th.e0 = pb->ev[2];
    th.e1 = pb->ev[3];
    th.enabled = p->time_kernels != 0;
    if ((rc = th.begin(stream)) != FW_OK) return rc;
    if (plan.two_pass_walkers != 0xFFFFFFFFu) {
      // finds its task count on the device; sized by the round before (twice that many tasks still get a wave each)
      rc = fw_launch_hub_scan(a, h, p->app, n_out != 0u ? scan_tasks * 4u + 1u : 0u, stream);
      if (rc != FW_OK) return rc;
    }
    // The grid follows the number of tasks: about as many as a round ago, scaled by the walkers (the first round
    // has nothing to go by and takes one resident set).  Not when workgroup tasks are more than a sixteenth of the
    // work: an oversized grid puts them behind all wave tasks, and they are better spread among those.
    uint32_t tasks_hint = n_out != 0u ? (uint32_t)((uint64_t)batch_tasks * m / n_out) + 1u : 0u;
    if ((uint64_t)wg_task_waves * 16u > batch_tasks) tasks_hint = 0u;
    // the short lists with few walkers, four to a wave (about as many as a round ago, scaled by the walkers): beside
    // the batch launch on a stream of their own -- the two work on different tasks and meet only in counters
    FW_HIP(hipEventRecord(pb->fork, stream));
    FW_HIP(hipStreamWaitEvent(pb->side, pb->fork, 0));
    rc = fw_launch_hub_quad(a, h, p->app, n_out != 0u ? (uint32_t)((uint64_t)quad_tasks * m / n_out) + 1u : 0u, pb->side);
    if (rc != FW_OK) return rc;
    FW_HIP(hipEventRecord(pb->join, pb->side));
    rc = fw_launch_hub_batch(a, h, p->app, p->wg_threads, tasks_hint, stream);
    if (rc != FW_OK) return rc;
    FW_HIP(hipStreamWaitEvent(stream, pb->join, 0));
    if ((rc = th.end(stream)) != FW_OK) return rc;
    ++*launches;
    {
      unsigned cblocks = ((unsigned)m + 4095u) / 4096u;
      if (cblocks > 1024u) cblocks = 1024u;
      hipLaunchKernelGGL(fw_compact_resume_kernel, dim3(cblocks), dim3(1024), 0, stream, pb->out, (uint32_t)m,
                         pb->resume, pb->ctrs + 6 * FW_CTR_STRIDE);
      FW_HIP(hipGetLastError());
    }
    // the walkers on vertices below the threshold continue in the walk kernel, which counts the walkers it parks in
    // the same bucket array as the batch launch did; how many they are is only known on the device yet
    a.resume = pb->resume;
    a.n_dev = pb->ctrs + 6 * FW_CTR_STRIDE;
    a.n = (int32_t)m;
    a.bucket_count = pb->count(nxt);
    entries_hint = hint_for(n_out != 0u ? (uint64_t)resumed + 1u : m / 4u + 1u);  // about as many as a round ago
    if ((rc = queue_walk(nullptr)) != FW_OK) return rc;
    if ((rc = copy_counters()) != FW_OK) return rc;
    // the next round: this round's m records of the batch launches' output list, and the walk launch's list (as many
    // positions as walkers resumed, which the device knows)
    if ((rc = queue_sort(nxt, cur, (uint32_t)m, (uint32_t)m, pb->ctrs + 6 * FW_CTR_STRIDE)) != FW_OK) return rc;
    if ((rc = wait_counters()) != FW_OK) return rc;
    th.collect(&times->hub_ms);
    tw.collect(&times->walk_ms);
    times->hub_quartets += *reinterpret_cast<const uint64_t*>(pb->h_ctrs + 14 * FW_CTR_STRIDE);
    times->table_walkers += pb->h_ctrs[13 * FW_CTR_STRIDE];
    times->parked_records += pb->h_ctrs[0 * FW_CTR_STRIDE];
    times->resume_entries += pb->h_ctrs[6 * FW_CTR_STRIDE];
    times->sorted_records += m;
    times->bucket_passes += (uint64_t)pb->n_buckets;
    n_out = (uint32_t)m;
    fullest = pb->h_ctrs[12 * FW_CTR_STRIDE];
    resumed = pb->h_ctrs[6 * FW_CTR_STRIDE];
    walk_entries = resumed;
    wg_task_waves = pb->h_ctrs[3 * FW_CTR_STRIDE] * (uint32_t)(p->wg_threads / 64);
    batch_tasks = pb->h_ctrs[5 * FW_CTR_STRIDE] + pb->h_ctrs[7 * FW_CTR_STRIDE] + wg_task_waves;
    quad_tasks = pb->h_ctrs[9 * FW_CTR_STRIDE];
    scan_tasks = pb->h_ctrs[8 * FW_CTR_STRIDE];
    cur = nxt;
  }
  return FW_OK;
}

// What a call's kernels ask of the memory, modelled from the run's own counters (steps, records, list quartets, table
// walkers): the lists as often as they were actually streamed, the scattered reads (one 128-byte block each: that is
// what the L2 asks the memory for, a pair of reads from the two halves of a block costs what one read costs), the
// scattered stores (one 32-byte write request each: a path entry or pair, a record) and the records and tasks that are
// streamed.  Tables that stay in the L2s (bucket counters, bucket offsets: 4 bytes per parked-on vertex) are not
// priced.  A model, not a measurement: the profiler's FETCH_SIZE / WRITE_SIZE are the measurement.
struct TrafficModel {
  uint64_t list_bytes = 0;
  uint64_t scattered_reads = 0;
  uint64_t scattered_writes = 0;
  uint64_t record_bytes = 0;
  uint64_t total() const { return list_bytes + 128u * scattered_reads + 32u * scattered_writes + record_bytes; }
};

// annotated: the hub kernels read the new vertex and its parking index from one annotated adjacency entry.
static TrafficModel traffic_model(const fw_walk_params* p, int32_t n, bool parked, int32_t park_threshold, bool annotated,
                                  uint64_t walk_steps, uint64_t walk_edges, uint64_t hub_steps, const KernelTimes& t) {
  constexpr uint64_t kRec = 16;
  const bool n2v = p->app == FW_APP_NODE2VEC;
  TrafficModel m;
  // walk launches.  A list is read from its first aligned quartet on (about 12 bytes of padding per step); lists of
  // up to 64 quartets bring their neighbours along with the biases, longer ones fetch the selected neighbour alone.
  const bool short_lists = parked && park_threshold <= 252;
  m.list_bytes += (short_lists ? 2u : 1u) * (4 * walk_edges + 12 * walk_steps);
  if (!short_lists) m.scattered_reads += walk_steps;             // adjncy[off + sel]
  m.scattered_reads += (parked ? 2u : 1u) * walk_steps;          // xadj pair, parking index
  m.scattered_writes += walk_steps;                              // path entry
  if (n2v) m.scattered_reads += 4 * (walk_steps + hub_steps);    // the searches in N(prev): about four blocks per step
  m.record_bytes += 4 * (uint64_t)n;                             // start vertices
  m.scattered_reads += (parked ? 2u : 1u) * (uint64_t)n;         // xadj pair, parking index
  m.scattered_writes += (uint64_t)n;                             // path[0]
  if (parked) {
    m.scattered_writes += t.parked_records;                      // record out (the bucket counter stays in the L2)
    m.record_bytes += kRec * t.resume_entries;                   // record in
    m.scattered_reads += t.resume_entries;                       // xadj pair
    // hub launches: the lists, and per walker its record in and out, the selected neighbour, the parking index of
    // the new vertex and the path entry
    m.list_bytes += 16 * t.hub_quartets;
    m.record_bytes += ((n2v ? kRec : kRec / 2) + kRec) * hub_steps;
    m.scattered_reads += (annotated ? 1u : 2u) * hub_steps;
    m.scattered_writes += hub_steps;
    m.scattered_reads += 7 * t.table_walkers;                    // pivots, lane row, prefix, four quartets of one lane
    // counting sort (record in, scattered record out), compaction (in, out), task list, reset, bucket scan
    m.record_bytes += 3 * kRec * t.sorted_records;
    m.scattered_writes += t.sorted_records;
    m.record_bytes += (12 + 8 + 8) * t.bucket_passes;
  }
  return m;
}


// One walk call at a time per graph: the parking index, the parking lists and the launch record are cached in the
// graph, so a second call that started while one is running would rebuild or overwrite them under it.
struct BusyGuard {
  fw_graph* g;
  bool held;
  explicit BusyGuard(const fw_graph* graph) : g(const_cast<fw_graph*>(graph)), held(false) {
    int expected = 0;
    held = g->busy.compare_exchange_strong(expected, 1);
    if (!held) fw_set_error("walk: another walk call is running on this fw_graph (one call at a time per graph; "
                            "make a second fw_graph to walk concurrently)");
  }
  bool ok() const { return held; }
  ~BusyGuard() { if (held) g->busy.store(0); }
};

static double now_ms() {
  using clk = std::chrono::steady_clock;
  return std::chrono::duration<double, std::milli>(clk::now().time_since_epoch()).count();
}

extern "C" int fw_walk_device(const fw_graph* g, const fw_walk_params* p, const int32_t* d_starts, int32_t n,
                              int32_t* d_paths, void* stream_v, fw_walk_stats* stats) {
  int rc = check_walk_args(g, p, d_starts, n, d_paths);
  if (rc != FW_OK) return rc;
  BusyGuard busy(g);
  if (!busy.ok()) return FW_ERR_INVALID;
  hipStream_t stream = reinterpret_cast<hipStream_t>(stream_v);
  const double t0 = now_ms();

  const int32_t park_threshold = resolve_park_threshold(g, p, n);
  ParkBuffers* pb = nullptr;
  bool use_pb = false;
  if (park_threshold != INT_MAX) {
    rc = ensure_hub_index(const_cast<fw_graph*>(g), park_threshold);
    if (rc != FW_OK) return rc;
    // buckets = parked-on vertices x labels must stay a 30-bit count (bucket ids travel in 32-bit record fields)
    use_pb = g->n_hubs > 0 &&
             (int64_t)g->n_hubs * (p->app == FW_APP_METAPATH ? p->schema_len : 1) <= ((int64_t)1 << 30);
  }
  if (use_pb) {
    const int labels = p->app == FW_APP_METAPATH ? p->schema_len : 1;
    pb = cached_park_buffers(const_cast<fw_graph*>(g), (size_t)n, g->n_hubs * labels, two_pass_rows(g, labels));
    use_pb = pb != nullptr;  // no room for the parking lists: walk without parking (same results, one launch)
  }
  // the launch record and the two timing events are the graph's, made once
  fw_graph* mg = const_cast<fw_graph*>(g);
  if (!mg->call_scratch) FW_HIP(hipMalloc(&mg->call_scratch, sizeof(Scratch)));
  for (hipEvent_t& e : mg->call_ev) if (!e) FW_HIP(hipEventCreate(&e));
  Scratch* const d_scr = static_cast<Scratch*>(mg->call_scratch);
  const hipEvent_t ev0 = mg->call_ev[0], ev1 = mg->call_ev[1];
  auto cleanup = [&]() {};
#define FW_TRY(call)                                                 \
  do {                                                               \
    int rc_ = fw_check_hip((call), #call, __FILE__, __LINE__);       \
    if (rc_ != FW_OK) { cleanup(); return rc_; }                     \
  } while (0)
  FW_TRY(hipMemsetAsync(d_scr, 0, sizeof(Scratch), stream));
  // -1 fill of the path matrix: src/walk.cu:398, :536
  FW_TRY(hipMemsetAsync(d_paths, 0xFF, (size_t)n * (size_t)p->max_depth * sizeof(int32_t), stream));

  fw_kargs a;
  fill_kargs(&a, g, p);
  a.starts = d_starts;
  a.paths = d_paths;
  a.n = n;
  a.dispenser = &d_scr->dispenser;
  a.counters = d_scr->counters;
  int grid_used = 0, launches = 0;
  KernelTimes times;
  FW_TRY(hipEventRecord(ev0, stream));
  rc = run_walk_launches(g, p, a, park_threshold, use_pb ? pb : nullptr, stream, &grid_used, &launches, &times);
  if (rc != FW_OK) { cleanup(); return rc; }
  FW_TRY(hipEventRecord(ev1, stream));
  FW_TRY(hipStreamSynchronize(stream));
  float ms = 0.0f;
  FW_TRY(hipEventElapsedTime(&ms, ev0, ev1));
  Scratch h;
  FW_TRY(hipMemcpy(&h, d_scr, sizeof(h), hipMemcpyDeviceToHost));
  cleanup();
  if (stats) {
    stats->kernel_ms = ms;
    stats->total_ms = now_ms() - t0;
    stats->steps = h.counters[0] + h.counters[2];
    stats->sampled_edges = h.counters[1] + h.counters[3];
    stats->launches = launches;
    stats->grid = grid_used;
    stats->walk_kernel_ms = launches == 1 ? (double)ms : times.walk_ms;  // the split: with time_kernels only
    stats->hub_kernel_ms = times.hub_ms;
    stats->hub_steps = h.counters[2];
    stats->hub_sampled_edges = h.counters[3];
    const TrafficModel tm = traffic_model(p, n, launches > 1, park_threshold, g->adj_hub != nullptr, h.counters[0],
                                          h.counters[1], h.counters[2], times);
    stats->requested_bytes = tm.total();
    stats->list_bytes = tm.list_bytes;
    stats->scattered_reads = tm.scattered_reads;
    stats->scattered_writes = tm.scattered_writes;
    stats->record_bytes = tm.record_bytes;
  }
  return FW_OK;
}

// ---- fw_walk_device_noalloc: the single-launch walk for callers that cannot allocate -----------------------
//
// fw_walk_device allocates its launch scratch (query dispenser word + workload counters) and two events per call.
// This variant keeps that scratch in a file-scope device array and creates its events once per device, so a call
// makes no hipMalloc / hipFree / hipEventCreate.  Every device holds its own copy of the array at its own address;
// the address is looked up once per device (the array's name is only a host-side handle, never a kernel argument).
// All calls on a device share the array, so a call that starts while another one is running on the same device is
// refused.  The call is synchronous like fw_walk_device (it waits for its launch and reads the counters back), so it is
// not a call to make while a stream is being captured into a graph.

static __device__ __align__(256) unsigned char scratch[256];
static_assert(sizeof(Scratch) <= 128 && sizeof(scratch) >= 128 + sizeof(int), "launch record in the first half, flag behind it");

namespace {
constexpr int kNoAllocMaxDevices = 64;
struct NoAllocDevice {
  Scratch* ptr = nullptr;  // device address of `scratch` on this device
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  std::atomic<int> busy{0};  // a call is using this device's array
};
// One call at a time per device: the array is shared by every call on the device.
struct NoAllocGuard {
  NoAllocDevice* d;
  bool held;
  explicit NoAllocGuard(NoAllocDevice* dev) : d(dev), held(false) {
    int expected = 0;
    held = d->busy.compare_exchange_strong(expected, 1);
    if (!held) fw_set_error("fw_walk_device_noalloc: another call is running on this device (all calls on a device share "
                            "one launch record inside the library; run them one after the other)");
  }
  bool ok() const { return held; }
  ~NoAllocGuard() { if (held) d->busy.store(0); }
};
NoAllocDevice g_noalloc[kNoAllocMaxDevices];
std::mutex g_noalloc_lock;

// Set-up of the current device, once: the array's address on this device and the two timing events.
int noalloc_device(NoAllocDevice** out) {
  int dev = 0;
  FW_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kNoAllocMaxDevices) {
    fw_set_error("fw_walk_device_noalloc: device %d is beyond the %d devices it keeps state for", dev, kNoAllocMaxDevices);
    return FW_ERR_INVALID;
  }
  std::lock_guard<std::mutex> guard(g_noalloc_lock);
  NoAllocDevice& d = g_noalloc[dev];
  if (d.ptr == nullptr) {
    void* p = nullptr;
    FW_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (p == nullptr) { fw_set_error("fw_walk_device_noalloc: the scratch array has no address on device %d", dev); return FW_ERR_HIP; }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    FW_HIP(hipEventCreate(&e0));
    if (fw_check_hip(hipEventCreate(&e1), "hipEventCreate", __FILE__, __LINE__) != FW_OK) {
      (void)hipEventDestroy(e0);
      return FW_ERR_HIP;
    }
    d.ev0 = e0;
    d.ev1 = e1;
    d.ptr = static_cast<Scratch*>(p);
  }
  *out = &d;
  return FW_OK;
}
}  // namespace

extern "C" int fw_walk_device_noalloc(const fw_graph* g, const fw_walk_params* p, const int32_t* d_starts, int32_t n,
                                      int32_t* d_paths, void* stream_v, fw_walk_stats* stats) {
  NoAllocDevice* d = nullptr;
  int rc = noalloc_device(&d);
  if (rc != FW_OK) return rc;
  NoAllocGuard guard(d);
  if (!guard.ok()) return FW_ERR_INVALID;
  // (the neighbour-order check of a graph's first node2vec call keeps its flag behind the launch record)
  rc = check_walk_args(g, p, d_starts, n, d_paths, reinterpret_cast<int*>(reinterpret_cast<unsigned char*>(d->ptr) + 128));
  if (rc != FW_OK) return rc;
  if (n > FW_WALK_NOALLOC_MAX_QUERIES) {
    fw_set_error("fw_walk_device_noalloc: n = %d exceeds FW_WALK_NOALLOC_MAX_QUERIES = %d (split the batch and advance "
                 "walker_base, or use fw_walk_device)", n, FW_WALK_NOALLOC_MAX_QUERIES);
    return FW_ERR_INVALID;
  }
  hipStream_t stream = reinterpret_cast<hipStream_t>(stream_v);
  const double t0 = now_ms();
  Scratch* const scr = d->ptr;  // the device address; never the array's name

  // the array keeps the last call's contents: the dispenser word and the counters start at zero
  hipLaunchKernelGGL(fw_fill_i32_kernel, dim3(1), dim3(64), 0, stream, reinterpret_cast<int32_t*>(scr), 0,
                     sizeof(Scratch) / sizeof(int32_t));
  FW_HIP(hipGetLastError());
  {
    const size_t count = (size_t)n * (size_t)p->max_depth;  // -1 fill of the path matrix: src/walk.cu:398, :536
    size_t blocks = (count + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(fw_fill_i32_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, d_paths, -1, count);
    FW_HIP(hipGetLastError());
  }
  fw_kargs a;
  fill_kargs(&a, g, p);  // park_threshold stays INT_MAX: one launch, walkers run whole walks
  a.starts = d_starts;
  a.paths = d_paths;
  a.n = n;
  a.dispenser = &scr->dispenser;
  a.counters = scr->counters;
  int grid_used = 0;
  FW_HIP(hipEventRecord(d->ev0, stream));
  rc = fw_launch_walk(a, p->app, p->sampler, p->wg_threads, p->grid, 0u, stream, &grid_used);
  if (rc != FW_OK) return rc;
  FW_HIP(hipEventRecord(d->ev1, stream));
  FW_HIP(hipStreamSynchronize(stream));
  float ms = 0.0f;
  FW_HIP(hipEventElapsedTime(&ms, d->ev0, d->ev1));
  Scratch h;
  FW_HIP(hipMemcpy(&h, scr, sizeof(h), hipMemcpyDeviceToHost));
  if (stats) {
    stats->kernel_ms = ms;
    stats->total_ms = now_ms() - t0;
    stats->steps = h.counters[0];
    stats->sampled_edges = h.counters[1];
    stats->launches = 1;
    stats->grid = grid_used;
    stats->walk_kernel_ms = ms;
    stats->hub_kernel_ms = 0.0;
    stats->hub_steps = 0;
    stats->hub_sampled_edges = 0;
    const TrafficModel tm = traffic_model(p, n, false, INT_MAX, false, h.counters[0], h.counters[1], 0, KernelTimes());
    stats->requested_bytes = tm.total();
    stats->list_bytes = tm.list_bytes;
    stats->scattered_reads = tm.scattered_reads;
    stats->scattered_writes = tm.scattered_writes;
    stats->record_bytes = tm.record_bytes;
  }
  return FW_OK;
}

extern "C" int fw_walk_batch(const fw_graph* g, const fw_walk_params* p, const int32_t* h_starts, int32_t n,
                             uint32_t batch_size, int sync, int32_t* h_paths, fw_walk_stats* stats) {
  int rc = check_walk_args(g, p, h_starts, n, h_paths);
  if (rc != FW_OK) return rc;
  BusyGuard busy(g);
  if (!busy.ok()) return FW_ERR_INVALID;
  fw_graph* const mg = const_cast<fw_graph*>(g);
  if (!mg->batch_cache) mg->batch_cache = new (std::nothrow) BatchCache;
  BatchCache* const bc = static_cast<BatchCache*>(mg->batch_cache);
  if (!bc) { fw_set_error("fw_walk_batch: out of host memory"); return FW_ERR_NOMEM; }
  if (batch_size == 0) {  // autobatch, src/main.cu:259-271 with the default 512 MB headroom
    size_t free_b = 0, total_b = 0;
    rc = fw_device_mem_info(&free_b, &total_b);
    if (rc != FW_OK) return rc;
    free_b += bc->bytes();  // what the last call left with the graph is this call's to use
    batch_size = fw_autobatch_size(free_b, 512, p->max_depth, sync, (uint32_t)n);
    if (batch_size == 0) { fw_set_error("autobatch: not enough free device memory"); return FW_ERR_NOMEM; }
    if (resolve_park_threshold(g, p, (int32_t)batch_size) != INT_MAX) {
      // the reference's rule counts the path matrix only; the parking lists take about 72 bytes per query more
      const size_t per_query = 4u * ((size_t)p->max_depth + 1u) + 72u;
      size_t bs2 = (free_b > ((size_t)512 << 20) ? free_b - ((size_t)512 << 20) : 0) / per_query;
      if (!sync) bs2 /= 2;
      if (bs2 >= 1 && bs2 < (size_t)batch_size) batch_size = (uint32_t)bs2;
    }
  }
  if (batch_size > (uint32_t)n) batch_size = (uint32_t)n;
  const size_t bs = batch_size;
  const size_t md = (size_t)p->max_depth;
  const int nbatch = (int)(((size_t)n + bs - 1) / bs);
  const int nbuf = sync || nbatch == 1 ? 1 : 2;  // buffers in flight

  const int32_t park_threshold = resolve_park_threshold(g, p, (int32_t)bs);
  bool use_pb = false;
  if (park_threshold != INT_MAX) {
    rc = ensure_hub_index(mg, park_threshold);
    if (rc != FW_OK) return rc;
    // buckets = parked-on vertices x labels must stay a 30-bit count (bucket ids travel in 32-bit record fields)
    use_pb = g->n_hubs > 0 &&
             (int64_t)g->n_hubs * (p->app == FW_APP_METAPATH ? p->schema_len : 1) <= ((int64_t)1 << 30);
  }
  // The buffers stay with the graph (see BatchCache); a failed call gives them up.
  auto cleanup = [&]() { release_batch_cache(mg); };
  if (bc->starts_cap < bs * (size_t)nbuf) {
    if (bc->d_starts) (void)hipFree(bc->d_starts);
    bc->d_starts = nullptr;
    bc->starts_cap = 0;
    FW_TRY(hipMalloc(reinterpret_cast<void**>(&bc->d_starts), bs * (size_t)nbuf * sizeof(int32_t)));
    bc->starts_cap = bs * (size_t)nbuf;
  }
  if (bc->paths_cap < bs * (size_t)nbuf * md) {
    if (bc->d_paths) (void)hipFree(bc->d_paths);
    bc->d_paths = nullptr;
    bc->paths_cap = 0;
    FW_TRY(hipMalloc(reinterpret_cast<void**>(&bc->d_paths), bs * (size_t)nbuf * md * sizeof(int32_t)));
    bc->paths_cap = bs * (size_t)nbuf * md;
  }
  if (use_pb) {
    const int n_buckets = g->n_hubs * (p->app == FW_APP_METAPATH ? p->schema_len : 1);
    const uint64_t rows = two_pass_rows(g, p->app == FW_APP_METAPATH ? p->schema_len : 1);
    for (int i = 0; i < nbuf && use_pb; ++i) {
      ParkBuffers& pb = bc->pbs[i];
      if (pb.cap >= bs && pb.n_buckets == n_buckets && pb.rows_cap >= rows) continue;
      pb.release();
      if (pb.alloc(bs, n_buckets, rows) != FW_OK) {  // no room for the parking lists: walk without parking (same results)
        bc->pbs[0].release();
        bc->pbs[1].release();
        use_pb = false;
        (void)hipGetLastError();
      }
    }
  }
  if (bc->scr_cap < (size_t)nbatch) {
    if (bc->d_scr) (void)hipFree(bc->d_scr);
    bc->d_scr = nullptr;
    bc->scr_cap = 0;
    FW_TRY(hipMalloc(reinterpret_cast<void**>(&bc->d_scr), sizeof(Scratch) * (size_t)nbatch));
    bc->scr_cap = (size_t)nbatch;
  }
  FW_TRY(hipMemset(bc->d_scr, 0, sizeof(Scratch) * (size_t)nbatch));
  for (int i = 0; i < nbuf; ++i) if (!bc->streams[i]) FW_TRY(hipStreamCreate(&bc->streams[i]));
  while (bc->events.size() < (size_t)nbatch * 2) {
    hipEvent_t e = nullptr;
    FW_TRY(hipEventCreate(&e));
    bc->events.push_back(e);
  }
  ParkBuffers* const pbs = bc->pbs;
  int32_t* const d_starts = bc->d_starts;
  int32_t* const d_paths = bc->d_paths;
  Scratch* const d_scr = bc->d_scr;
  hipStream_t* const streams = bc->streams;
  std::vector<hipEvent_t>& events = bc->events;

  fw_kargs a;
  fill_kargs(&a, g, p);
  int grid_used = 0;
  KernelTimes times;
  const double t0 = now_ms();
  for (int b = 0; b < nbatch; ++b) {
    const int s = b % nbuf;
    const size_t first = (size_t)b * bs;
    const int32_t cnt = (int32_t)(((size_t)n - first) < bs ? ((size_t)n - first) : bs);
    int32_t* ds = d_starts + (size_t)s * bs;
    int32_t* dp = d_paths + (size_t)s * bs * md;
    FW_TRY(hipMemcpyAsync(ds, h_starts + first, (size_t)cnt * sizeof(int32_t), hipMemcpyHostToDevice, streams[s]));
    FW_TRY(hipMemsetAsync(dp, 0xFF, (size_t)cnt * md * sizeof(int32_t), streams[s]));
    a.starts = ds;
    a.paths = dp;
    a.n = cnt;
    a.walker_base = p->walker_base + (uint32_t)first;
    a.dispenser = &d_scr[b].dispenser;
    a.counters = d_scr[b].counters;
    FW_TRY(hipEventRecord(events[2 * b], streams[s]));
    int launches = 0;
    rc = run_walk_launches(g, p, a, park_threshold, use_pb ? &pbs[s] : nullptr, streams[s], &grid_used, &launches,
                           &times);
    if (rc != FW_OK) { cleanup(); return rc; }
    FW_TRY(hipEventRecord(events[2 * b + 1], streams[s]));
    FW_TRY(hipMemcpyAsync(h_paths + first * md, dp, (size_t)cnt * md * sizeof(int32_t), hipMemcpyDeviceToHost, streams[s]));
    if (sync) FW_TRY(hipStreamSynchronize(streams[s]));
  }
  for (int i = 0; i < nbuf; ++i) FW_TRY(hipStreamSynchronize(streams[i]));
  const double total = now_ms() - t0;

  double kernel_ms = 0.0;
  for (int b = 0; b < nbatch; ++b) {
    float ms = 0.0f;
    FW_TRY(hipEventElapsedTime(&ms, events[2 * b], events[2 * b + 1]));
    kernel_ms += ms;
  }
  std::vector<Scratch> h((size_t)nbatch);
  FW_TRY(hipMemcpy(h.data(), d_scr, sizeof(Scratch) * (size_t)nbatch, hipMemcpyDeviceToHost));
  if (stats) {
    stats->kernel_ms = kernel_ms;
    stats->total_ms = total;
    stats->steps = 0;
    stats->sampled_edges = 0;
    stats->hub_steps = 0;
    stats->hub_sampled_edges = 0;
    for (const Scratch& s : h) {
      stats->steps += s.counters[0] + s.counters[2];
      stats->sampled_edges += s.counters[1] + s.counters[3];
      stats->hub_steps += s.counters[2];
      stats->hub_sampled_edges += s.counters[3];
    }
    stats->launches = nbatch;
    stats->grid = grid_used;
    stats->walk_kernel_ms = stats->hub_steps == 0 ? kernel_ms : times.walk_ms;  // the split: with time_kernels only
    stats->hub_kernel_ms = times.hub_ms;
    const TrafficModel tm = traffic_model(p, n, times.sorted_records != 0, park_threshold, g->adj_hub != nullptr,
                                          stats->steps - stats->hub_steps,
                                          stats->sampled_edges - stats->hub_sampled_edges, stats->hub_steps, times);
    stats->requested_bytes = tm.total();
    stats->list_bytes = tm.list_bytes;
    stats->scattered_reads = tm.scattered_reads;
    stats->scattered_writes = tm.scattered_writes;
    stats->record_bytes = tm.record_bytes;
  }
  return FW_OK;
}
#undef FW_TRY
