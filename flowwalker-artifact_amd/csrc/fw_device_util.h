// Device helpers shared by the kernels of libflowwalker_hip.so: Philox4x32-10, the uniform conversion, and the
// wave64 scan / max networks on the DPP unit.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

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

// x + (value of the lane selected by the DPP control; lanes without a source lane add 0).  For values that are
// not -0 (sums of non-negative biases never are) x + 0 == x bit for bit.
template <int kCtrl>
__device__ __forceinline__ float dpp_add(float x) {
  const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(x), kCtrl, 0xF, 0xF, true);
  return x + __int_as_float(moved);
}

// x += (lane 15 of the previous row) in rows 1 and 3; x += (lane 31) in rows 2 and 3.  The other rows keep x: the
// instruction does not write them.  (Written out because the compiler only folds a lane movement into an add
// when the skipped lanes can be given the operation's identity, which it does not do for float adds.)
__device__ __forceinline__ float dpp_add_bcast15(float x) {
  asm volatile("s_nop 1\n\tv_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf" : "+v"(x));
  return x;
}
__device__ __forceinline__ float dpp_add_bcast31(float x) {
  asm volatile("s_nop 1\n\tv_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf" : "+v"(x));
  return x;
}

// Inclusive scan over the 64 lanes: Kogge-Stone inside each 16-lane row (row_shr 1,2,4,8), then
// row_bcast:15 into rows 1 and 3, then row_bcast:31 into rows 2 and 3.  The association order is part
// of the sampler's definition.
__device__ __forceinline__ float wave_scan(float x) {
  x = dpp_add<0x111>(x);
  x = dpp_add<0x112>(x);
  x = dpp_add<0x114>(x);
  x = dpp_add<0x118>(x);
  x = dpp_add_bcast15(x);
  x = dpp_add_bcast31(x);
  return x;
}

// Inclusive prefix maximum over the 64 lanes of non-negative floats (same network as wave_scan).  Non-negative
// floats order like their bit patterns, so the maximum is taken on the integers (exact, no NaN handling).
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_max(float x) {
  const uint32_t xi = __float_as_uint(x);
  const uint32_t moved = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)xi, kCtrl, kRowMask, 0xF, false);
  return __uint_as_float(xi > moved ? xi : moved);
}

__device__ __forceinline__ float wave_prefix_max(float x) {
  x = dpp_max<0x111, 0xF>(x);
  x = dpp_max<0x112, 0xF>(x);
  x = dpp_max<0x114, 0xF>(x);
  x = dpp_max<0x118, 0xF>(x);
  x = dpp_max<0x142, 0xA>(x);
  x = dpp_max<0x143, 0xC>(x);
  return x;
}

// Inclusive scan inside each 16-lane row only.
__device__ __forceinline__ float row_scan(float x) {
  x = dpp_add<0x111>(x);
  x = dpp_add<0x112>(x);
  x = dpp_add<0x114>(x);
  x = dpp_add<0x118>(x);
  return x;
}

__device__ __forceinline__ int lane_id() { return (int)__lane_id(); }

__device__ __forceinline__ float readlane_f(float x, int l) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), l));
}

// Value of x in the lane whose number is byte_addr / 4 (any lane may read any lane).
__device__ __forceinline__ float bperm_f(int byte_addr, float x) {
  return __int_as_float(__builtin_amdgcn_ds_bpermute(byte_addr, __float_as_int(x)));
}

// max over the wave of a per-lane int (INT_MIN where a lane has nothing), result in every lane
__device__ __forceinline__ int32_t wave_max_i32(int32_t v) {
  constexpr int kMin = (int)0x80000000;
  v = max(v, __builtin_amdgcn_update_dpp(kMin, v, 0x111, 0xF, 0xF, false));
  v = max(v, __builtin_amdgcn_update_dpp(kMin, v, 0x112, 0xF, 0xF, false));
  v = max(v, __builtin_amdgcn_update_dpp(kMin, v, 0x114, 0xF, 0xF, false));
  v = max(v, __builtin_amdgcn_update_dpp(kMin, v, 0x118, 0xF, 0xF, false));
  v = max(v, __builtin_amdgcn_update_dpp(kMin, v, 0x142, 0xA, 0xF, false));
  v = max(v, __builtin_amdgcn_update_dpp(kMin, v, 0x143, 0xC, 0xF, false));
  return __builtin_amdgcn_readlane(v, 63);
}

}  // namespace
