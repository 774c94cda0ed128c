// Shared host/device helpers for libmega_hip (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/mega_hip.h"

namespace mega {

// ---------------------------------------------------------------- errors
void set_error(const char* fmt, ...);

// ---- give-ups of the bounded waits between workgroups (look-back of the streaming kernels).
// A kernel that gives up writes NaN into what depended on the missing words and sets two words: `error` of its
// workspace header and the host-mapped status word of its device, which the host reads without synchronising.
struct LookbackLaunch {
  uint32_t* status;      // device address of the device's host-mapped status word (null: none could be set up)
  uint32_t spin_limit;   // polls before a wait gives up
  int withhold_first;    // test hook: the first tile of every row publishes nothing
};
// `may_allocate`: the status word may be created (pinned host memory) if the device has none yet
LookbackLaunch lookback_launch(bool may_allocate);
// MEGA_ERR_LAUNCH (message set, word cleared) when a launch on the current device has given up since the last check
int lookback_pending(const char* entry);
// checked mode (mega_lookback_checked / MEGA_LOOKBACK_CHECKED=1): waits for the stream and reports a give-up of the
// launch just made; MEGA_OK at once when the mode is off
int lookback_verify(const char* entry, hipStream_t stream);

#define MEGA_REQUIRE(cond, code, ...)  \
  do {                                 \
    if (!(cond)) {                     \
      ::mega::set_error(__VA_ARGS__);  \
      return (code);                   \
    }                                  \
  } while (0)

#define MEGA_CHECK_LAUNCH(what)                                           \
  do {                                                                    \
    hipError_t e__ = hipGetLastError();                                   \
    if (e__ != hipSuccess) {                                              \
      ::mega::set_error("%s: launch failed: %s", what, hipGetErrorString(e__)); \
      return MEGA_ERR_LAUNCH;                                             \
    }                                                                     \
  } while (0)

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Function attributes (the dynamic shared memory limit of a kernel) belong to a device: a call site sets them the
// first time it launches on each device.  `seen` is the call site's own mask of devices.
static inline bool first_on_device(uint64_t* seen) {
  int d = 0;
  if (hipGetDevice(&d) != hipSuccess) {
    (void)hipGetLastError();
    d = 0;
  }
  const uint64_t bit = 1ull << (d & 63);
  return !(__atomic_fetch_or(seen, bit, __ATOMIC_RELAXED) & bit);
}

// Compute units of the current device, queried once per device (256 when the query fails).
static inline int device_cu_count() {
  static int cu_count[64] = {0};
  int d = 0;
  if (hipGetDevice(&d) != hipSuccess || d < 0 || d >= 64) {
    (void)hipGetLastError();
    return 256;
  }
  int n = __atomic_load_n(&cu_count[d], __ATOMIC_RELAXED);
  if (n == 0) {
    n = (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, d) == hipSuccess && n > 0) ? n : 256;
    __atomic_store_n(&cu_count[d], n, __ATOMIC_RELAXED);
  }
  return n;
}

// ---- address audit (host only).  Between mega_audit_begin() and mega_audit_end() the entry points that take part
// launch nothing: they compute, for every launch they would make, the last byte each operand is addressed at (from
// the same sizes and strides the kernel gets) and check that it lies inside one of the byte ranges registered with
// mega_audit_add (the caller's tensors and workspace, at made-up addresses: no GPU is needed).
bool audit_on();
// [p, p + bytes) must lie inside one registered range; records a violation (and returns false) otherwise
bool audit_use(const void* p, size_t bytes, const char* what);

// Clears `bytes` (a multiple of 4) with a small kernel (elementwise.hip).  Used instead of a memset
// node so that a caller may record any entry point into a HIP graph.
void zero_async(void* p, size_t bytes, hipStream_t s);
static inline size_t align_up(size_t a, size_t b) { return (a + b - 1) / b * b; }
// do the byte ranges [a, a + na) and [b, b + nb) share a byte?
static inline bool ranges_overlap(const void* a, size_t na, const void* b, size_t nb) {
  const uintptr_t ua = (uintptr_t)a, ub = (uintptr_t)b;
  return ua < ub + nb && ub < ua + na;
}

// ---------------------------------------------------------------- row tiling of [tokens, H] tiles
// How the channel vectors of one token are spread over threads in the kernels that walk
// [tokens, H] tiles with per-group reductions: LPG consecutive lanes (a power of two) share one
// (token, group) and move PER vectors of `vec` channels each; `slots` = lanes per token.
struct RowTiling {
  int LPG, PER, slots;
  int lpg_shift;     // log2(LPG)
  int slots_shift;   // log2(slots), or -1 when slots is not a power of two
};

static inline RowTiling make_row_tiling(int64_t G, int64_t Dg, int vec) {
  RowTiling R;
  const int64_t vecs = Dg / vec;          // vectors per (token, group)
  int lpg = 1;
  while (lpg < 64 && vecs % (2 * lpg) == 0) lpg *= 2;
  R.LPG = lpg;
  R.PER = (int)(vecs / lpg);
  R.slots = (int)G * lpg;
  R.lpg_shift = 0;
  while ((1 << R.lpg_shift) < R.LPG) ++R.lpg_shift;
  R.slots_shift = -1;
  if ((R.slots & (R.slots - 1)) == 0) {
    R.slots_shift = 0;
    while ((1 << R.slots_shift) < R.slots) ++R.slots_shift;
  }
  return R;
}

// item -> (token, slot): a shift when the lane count per token is a power of two
__device__ __forceinline__ void split_item(const RowTiling& R, int i, int& tok, int& slot) {
  if (R.slots_shift >= 0) {
    tok = i >> R.slots_shift;
    slot = i & (R.slots - 1);
  } else {
    tok = i / R.slots;
    slot = i - tok * R.slots;
  }
}

// ---------------------------------------------------------------- element types
struct bf16_t { uint16_t u; };
struct f16_t { _Float16 h; };

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(((uint32_t)v.u) << 16); }
__device__ __forceinline__ float to_float(f16_t v) { return (float)v.h; }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) {
  // round to nearest even in hardware (v_cvt_pk_bf16_f32 on gfx950)
  const __bf16 h = (__bf16)v;
  bf16_t r;
  r.u = __builtin_bit_cast(uint16_t, h);
  return r;
}
template <> __device__ __forceinline__ f16_t from_float<f16_t>(float v) {
  f16_t r;
  r.h = (_Float16)v;
  return r;
}

// VEC consecutive fp32 parameters (16-byte pieces when VEC is a multiple of 4 and p is aligned to it)
template <int VEC>
__device__ __forceinline__ void load_params(const float* __restrict__ p, float (&out)[VEC]) {
  if constexpr (VEC % 4 == 0) {
#pragma unroll
    for (int i = 0; i < VEC / 4; ++i) {
      const float4 v = ((const float4*)p)[i];
      out[4 * i] = v.x; out[4 * i + 1] = v.y; out[4 * i + 2] = v.z; out[4 * i + 3] = v.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) out[i] = p[i];
  }
}

// a naturally aligned vector of VEC elements, moved with one memory instruction
template <typename T, int VEC>
struct alignas(sizeof(T) * VEC) Vec {
  T v[VEC];
};

// ---------------------------------------------------------------- counter-based random numbers
// Uniform number in [0, 1) that depends only on (seed, idx): the 64-bit finaliser of splitmix64 on
// seed + (idx + 1) * golden ratio, top 24 bits.  Every kernel that drops keys calls it with the
// element's position in the [B, Nh, L, L] weight tensor, so the fused and the unfused attention
// draw the same mask from the same seed, and a mask can be restated on the host bit for bit.
__host__ __device__ inline float hash_uniform(uint64_t seed, uint64_t idx) {
  uint64_t z = seed + (idx + 1) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}

// ---------------------------------------------------------------- complex
struct cfloat {
  float re, im;
};
__device__ __forceinline__ cfloat cmul(cfloat a, cfloat b) {
  return {a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
}
__device__ __forceinline__ cfloat cadd(cfloat a, cfloat b) { return {a.re + b.re, a.im + b.im}; }

// q^e for a non-negative integer e by binary exponentiation (double precision)
__host__ __device__ inline void cpow_int(double qr, double qi, int64_t e, double* rr, double* ri) {
  double ar = 1.0, ai = 0.0;
  double br = qr, bi = qi;
  while (e > 0) {
    if (e & 1) {
      const double t = ar * br - ai * bi;
      ai = ar * bi + ai * br;
      ar = t;
    }
    const double t = br * br - bi * bi;
    bi = 2.0 * br * bi;
    br = t;
    e >>= 1;
  }
  *rr = ar;
  *ri = ai;
}

// ---------------------------------------------------------------- Welford
// state: n elements' worth of weight, their mean and their biased variance
// (the combine operator of the streaming norm; equal weights merge exactly as
// WelfordCombine does for counts).
struct Moments {
  float n, mean, var;
};
__device__ __forceinline__ Moments combine(Moments a, Moments b) {
  const float n = a.n + b.n;
  if (n == 0.f) return {0.f, 0.f, 0.f};
  const float ca = a.n / n, cb = b.n / n;
  const float d = b.mean - a.mean;
  Moments r;
  r.n = n;
  r.mean = ca * a.mean + cb * b.mean;
  r.var = ca * a.var + cb * b.var + (ca * d) * (cb * d);
  return r;
}

// ---------------------------------------------------------------- cross-workgroup signalling
// Values that one workgroup publishes for another travel through these (device scope)
// atomics so that they are coherent across the per-XCD L2 caches.
__device__ __forceinline__ void publish_f32(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float fetch_f32(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void publish_u32(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t fetch_u32(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void release_flag(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t acquire_flag(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace mega
