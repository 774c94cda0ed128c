// SwiGLU gate y = silu(a) * b and the plain activation y = silu(a) (elementwise, streamed with 16-byte accesses).
#include "common.h"

namespace mega {
namespace {

// x sigmoid(x) with the hardware reciprocal (1 ulp) in the place of a full division: the division's ten
// instructions per element made these kernels instruction-bound
__device__ __forceinline__ float silu_f(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

template <typename T, int VEC>
__global__ __launch_bounds__(256) void swiglu_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                     T* __restrict__ y, int64_t n) {
  using V = Vec<T, VEC>;
  const int64_t nv = n / VEC;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nv; i += stride) {
    const V av = ((const V*)a)[i];
    const V bv = ((const V*)b)[i];
    V o;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      const float x = to_float(av.v[k]);
      const float s = silu_f(x);
      o.v[k] = from_float<T>(s * to_float(bv.v[k]));
    }
    ((V*)y)[i] = o;
  }
  // tail
  const int64_t t = nv * VEC + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) {
    const float x = to_float(a[t]);
    y[t] = from_float<T>(silu_f(x) * to_float(b[t]));
  }
}

template <typename T>
int launch_swiglu(const void* a, const void* b, void* y, int64_t n, hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool aligned = (((uintptr_t)a | (uintptr_t)b | (uintptr_t)y) % 16) == 0;
  int64_t blocks = ceil_div(ceil_div(n, VEC), 256);
  if (blocks > 256 * 16) blocks = 256 * 16;
  if (blocks < 1) blocks = 1;
  if (aligned)
    hipLaunchKernelGGL((swiglu_kernel<T, VEC>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)a, (const T*)b,
                       (T*)y, n);
  else
    hipLaunchKernelGGL((swiglu_kernel<T, 1>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)a, (const T*)b,
                       (T*)y, n);
  MEGA_CHECK_LAUNCH("swiglu_fwd");
  return MEGA_OK;
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void silu_kernel(const T* __restrict__ a, T* __restrict__ y, int64_t n) {
  using V = Vec<T, VEC>;
  const int64_t nv = n / VEC;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nv; i += stride) {
    const V av = ((const V*)a)[i];
    V o;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      const float x = to_float(av.v[k]);
      o.v[k] = from_float<T>(silu_f(x));
    }
    ((V*)y)[i] = o;
  }
  const int64_t t = nv * VEC + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) {
    const float x = to_float(a[t]);
    y[t] = from_float<T>(silu_f(x));
  }
}

template <typename T>
int launch_silu(const void* a, void* y, int64_t n, hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool aligned = (((uintptr_t)a | (uintptr_t)y) % 16) == 0;
  int64_t blocks = ceil_div(ceil_div(n, VEC), 256);
  if (blocks > 256 * 16) blocks = 256 * 16;
  if (blocks < 1) blocks = 1;
  if (aligned)
    hipLaunchKernelGGL((silu_kernel<T, VEC>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)a, (T*)y, n);
  else
    hipLaunchKernelGGL((silu_kernel<T, 1>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)a, (T*)y, n);
  MEGA_CHECK_LAUNCH("silu_fwd");
  return MEGA_OK;
}

// zeros for small outputs of degenerate calls
__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t* __restrict__ p, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0u;
}

}  // namespace

void zero_async(void* p, size_t bytes, hipStream_t s) {
  const size_t n = bytes / 4;
  if (n == 0) return;
  hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)ceil_div((int64_t)n, 256)), dim3(256), 0, s, (uint32_t*)p, n);
}

}  // namespace mega

using namespace mega;

extern "C" int mega_swiglu_fwd(const void* a, const void* b, void* y, int dtype, int64_t n, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "swiglu_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(n >= 0, MEGA_ERR_ARG, "swiglu_fwd: negative size");
  if (n == 0) return MEGA_OK;
  MEGA_REQUIRE(a && b && y, MEGA_ERR_ARG, "swiglu_fwd: null pointer argument");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MEGA_F32: return launch_swiglu<float>(a, b, y, n, s);
    case MEGA_BF16: return launch_swiglu<bf16_t>(a, b, y, n, s);
    default: return launch_swiglu<f16_t>(a, b, y, n, s);
  }
}

extern "C" int mega_silu_fwd(const void* a, void* y, int dtype, int64_t n, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "silu_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(n >= 0, MEGA_ERR_ARG, "silu_fwd: negative size");
  if (n == 0) return MEGA_OK;
  MEGA_REQUIRE(a && y, MEGA_ERR_ARG, "silu_fwd: null pointer argument");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MEGA_F32: return launch_silu<float>(a, y, n, s);
    case MEGA_BF16: return launch_silu<bf16_t>(a, y, n, s);
    default: return launch_silu<f16_t>(a, y, n, s);
  }
}
