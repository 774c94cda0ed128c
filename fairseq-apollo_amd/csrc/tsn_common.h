// Device helpers shared by the TimestepNorm kernels: lane-group reductions and scans of Welford
// states with DPP, packed 16-bit dot products, and the tagged 64-bit words tiles publish for each other.
#pragma once
#include "common.h"

namespace mega {
namespace {

struct TsnHeader {
  uint32_t epoch;        // bumped by the last workgroup of every launch
  uint32_t done2;        // second-level retire counter
  uint32_t error;        // set when a bounded wait gave up
  uint32_t pad;
  uint32_t done1[32];    // first-level retire counters (workgroup id mod 32)
};

// a bounded wait gave up: the workspace header and the device's host-mapped status word say so
__device__ __forceinline__ void report_give_up(TsnHeader* hdr, uint32_t* status) {
  publish_u32(&hdr->error, 1u);
  if (status) __hip_atomic_store(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// ---- lane-group primitives (DPP inside rows of 16 lanes)
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
constexpr int kXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kHalfMirror = 0x141;
constexpr int kRowMirror = 0x140;

// sum over LPG adjacent lanes (LPG a power of two <= 64); every lane of the group gets the sum
template <int LPG>
__device__ __forceinline__ float group_sum(float v) {
  if (LPG >= 2) v += dpp_f<kXor1>(v);
  if (LPG >= 4) v += dpp_f<kXor2>(v);
  if (LPG >= 8) v += dpp_f<kHalfMirror>(v);
  if (LPG >= 16) v += dpp_f<kRowMirror>(v);
  if (LPG >= 32) v += __shfl_xor(v, 16);
  if (LPG >= 64) v += __shfl_xor(v, 32);
  return v;
}

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;

// acc + x0 + x1 and acc + x0^2 + x1^2 for a packed pair of 16-bit values
template <typename T>
__device__ __forceinline__ float dot2_ones(uint32_t w, float acc) {
  if constexpr (sizeof(T) == 2 && !__is_same(T, f16_t)) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w), __builtin_bit_cast(bf16x2_t, 0x3f803f80u),
                                           acc, false);
  } else {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, w), __builtin_bit_cast(f16x2_t, 0x3c003c00u), acc, false);
  }
}
template <typename T>
__device__ __forceinline__ float dot2_self(uint32_t w, float acc) {
  if constexpr (sizeof(T) == 2 && !__is_same(T, f16_t)) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w), __builtin_bit_cast(bf16x2_t, w), acc, false);
  } else {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, w), __builtin_bit_cast(f16x2_t, w), acc, false);
  }
}

// merge of two sets of equally weighted steps; one reciprocal per merge.  Two empty sets keep the first one's
// mean and variance: a row that has seen no valid step yet still carries the caller's prior statistics, which
// the reference hands back unchanged (timestep_norm.cc:283-311: u, v only move on unmasked steps).
__device__ __forceinline__ Moments merge(Moments a, Moments b) {
  const float n = a.n + b.n;
  const float rn = n > 0.f ? __builtin_amdgcn_rcpf(n) : 0.f;
  const float cb = b.n * rn, ca = a.n * rn;
  const float d = b.mean - a.mean;
  Moments r;
  r.n = n;
  r.mean = a.mean + cb * d;
  r.var = n > 0.f ? ca * a.var + cb * b.var + (ca * d) * (cb * d) : a.var;
  return r;
}

template <int CTRL>
__device__ __forceinline__ Moments dpp_m(Moments m) {
  return Moments{dpp_f<CTRL>(m.n), dpp_f<CTRL>(m.mean), dpp_f<CTRL>(m.var)};
}

// all 16 lanes of a row get the merge of the row
__device__ __forceinline__ Moments row_reduce(Moments m) {
  m = merge(m, dpp_m<kXor1>(m));
  m = merge(m, dpp_m<kXor2>(m));
  m = merge(m, dpp_m<kHalfMirror>(m));
  m = merge(m, dpp_m<kRowMirror>(m));
  return m;
}

// inclusive scan over the 16 lanes of a row (lanes shifted in from outside the row are empty sets)
__device__ __forceinline__ Moments row_scan(Moments m) {
  m = merge(dpp_m<0x111>(m), m);
  m = merge(dpp_m<0x112>(m), m);
  m = merge(dpp_m<0x114>(m), m);
  m = merge(dpp_m<0x118>(m), m);
  return m;
}

__device__ __forceinline__ uint32_t row_sum_u32(uint32_t v) {
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kXor1, 0xf, 0xf, true);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kXor2, 0xf, 0xf, true);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kHalfMirror, 0xf, 0xf, true);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kRowMirror, 0xf, 0xf, true);
  return v;
}

__device__ __forceinline__ unsigned long long tagged(uint32_t v, uint32_t tag) {
  return ((unsigned long long)tag << 32) | v;
}
__device__ __forceinline__ void put_rec(unsigned long long* p, unsigned long long v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long get_rec(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace
}  // namespace mega
