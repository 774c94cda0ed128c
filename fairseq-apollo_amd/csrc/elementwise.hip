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

// dx = dy silu'(x),  silu'(x) = s (1 + x (1 - s)), s = sigmoid(x)
template <typename T, int VEC>
__global__ __launch_bounds__(256) void silu_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ a,
                                                       T* __restrict__ dx, int64_t n) {
  using V = Vec<T, VEC>;
  const int64_t nv = n / VEC;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  auto f = [](float g, float x) {
    const float sg = __builtin_amdgcn_rcpf(1.0f + __expf(-x));
    return g * sg * fmaf(x, 1.0f - sg, 1.0f);
  };
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nv; i += stride) {
    const V gv = ((const V*)dy)[i];
    const V av = ((const V*)a)[i];
    V o;
#pragma unroll
    for (int k = 0; k < VEC; ++k) o.v[k] = from_float<T>(f(to_float(gv.v[k]), to_float(av.v[k])));
    ((V*)dx)[i] = o;
  }
  const int64_t t = nv * VEC + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) dx[t] = from_float<T>(f(to_float(dy[t]), to_float(a[t])));
}

template <typename T>
int launch_silu_bwd(const void* dy, const void* a, void* dx, int64_t n, hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool aligned = (((uintptr_t)dy | (uintptr_t)a | (uintptr_t)dx) % 16) == 0;
  int64_t blocks = ceil_div(ceil_div(n, VEC), 256);
  if (blocks > 256 * 16) blocks = 256 * 16;
  if (blocks < 1) blocks = 1;
  if (aligned)
    hipLaunchKernelGGL((silu_bwd_kernel<T, VEC>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)dy, (const T*)a,
                       (T*)dx, n);
  else
    hipLaunchKernelGGL((silu_bwd_kernel<T, 1>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)dy, (const T*)a,
                       (T*)dx, n);
  MEGA_CHECK_LAUNCH("silu_bwd");
  return MEGA_OK;
}

// Column sums of a [T, W] matrix (the bias gradient of a projection: the sum of its output's gradient over the
// tokens).  A workgroup owns kColBlock columns (a lane VEC adjacent ones) and one slab of rows; its four waves take
// every fourth row of the slab, four rows in flight per wave, and add up through LDS in wave order; one row of
// partial sums per slab of 256 rows goes to the workspace, and colsum_finish_kernel adds the slabs in order: the
// same bits on every run.
constexpr int kColSlabRows = 256;

template <typename T, int VEC>
__global__ __launch_bounds__(256) void colsum_partial_kernel(const T* __restrict__ x, int64_t rs, int64_t T_, int W,
                                                             float* __restrict__ part) {
  using V = Vec<T, VEC>;
  __shared__ float s_acc[3][64 * VEC];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c0 = ((int)blockIdx.x * 64 + lane) * VEC;
  const int64_t r0 = (int64_t)blockIdx.y * kColSlabRows;
  const int64_t r1 = r0 + kColSlabRows < T_ ? r0 + kColSlabRows : T_;
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
  if (c0 < W) {
    for (int64_t r = r0 + wave; r < r1; r += 16) {
      V v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t rr = r + 4 * u;
        if (rr < r1) {
          v[u] = *(const V*)(x + rr * rs + c0);
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e) v[u].v[e] = from_float<T>(0.f);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] += to_float(v[u].v[e]);
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) s_acc[wave - 1][lane * VEC + e] = acc[e];
  }
  __syncthreads();
  if (wave == 0 && c0 < W) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float t = acc[e];
      for (int w = 0; w < 3; ++w) t += s_acc[w][lane * VEC + e];
      part[(int64_t)blockIdx.y * W + c0 + e] = t;
    }
  }
}

template <typename TOut>
__global__ __launch_bounds__(64) void colsum_finish_kernel(const float* __restrict__ part, int nslab, int W,
                                                            TOut* __restrict__ out) {
  const int c = (int)blockIdx.x * 64 + (int)threadIdx.x;
  if (c >= W) return;
  float t = 0.f;
  for (int s0 = 0; s0 < nslab; s0 += 8) {          // eight slabs requested together, added in slab order
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = s0 + u < nslab ? part[(int64_t)(s0 + u) * W + c] : 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) t += v[u];
  }
  out[c] = from_float<TOut>(t);
}

template <typename T>
int launch_colsum(const void* x, int64_t rs, int64_t T_, int64_t W, void* out, int out_dtype, float* part,
                  hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const int nslab = (int)ceil_div(T_, kColSlabRows);
  const dim3 grid((unsigned)ceil_div(W, 64 * VEC), (unsigned)nslab);
  hipLaunchKernelGGL((colsum_partial_kernel<T, VEC>), grid, dim3(256), 0, s, (const T*)x, rs, T_, (int)W, part);
  MEGA_CHECK_LAUNCH("colsum");
  const dim3 g2((unsigned)ceil_div(W, 64));
  if (out_dtype == MEGA_F32)
    hipLaunchKernelGGL(colsum_finish_kernel<float>, g2, dim3(64), 0, s, part, nslab, (int)W, (float*)out);
  else if (out_dtype == MEGA_BF16)
    hipLaunchKernelGGL(colsum_finish_kernel<bf16_t>, g2, dim3(64), 0, s, part, nslab, (int)W, (bf16_t*)out);
  else
    hipLaunchKernelGGL(colsum_finish_kernel<f16_t>, g2, dim3(64), 0, s, part, nslab, (int)W, (f16_t*)out);
  MEGA_CHECK_LAUNCH("colsum (slabs)");
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

extern "C" int mega_silu_bwd(const void* y_grad, const void* a, void* a_grad, int dtype, int64_t n, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "silu_bwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(n >= 0, MEGA_ERR_ARG, "silu_bwd: negative size");
  if (n == 0) return MEGA_OK;
  MEGA_REQUIRE(y_grad && a && a_grad, MEGA_ERR_ARG, "silu_bwd: null pointer argument");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MEGA_F32: return launch_silu_bwd<float>(y_grad, a, a_grad, n, s);
    case MEGA_BF16: return launch_silu_bwd<bf16_t>(y_grad, a, a_grad, n, s);
    default: return launch_silu_bwd<f16_t>(y_grad, a, a_grad, n, s);
  }
}

extern "C" size_t mega_colsum_workspace_bytes(int64_t T_, int64_t W) {
  if (T_ <= 0 || W <= 0) return 256;
  return (size_t)ceil_div(T_, kColSlabRows) * (size_t)W * 4;
}

namespace mega {
namespace {

// out[b][c][r] = in[b][r'][c'] with r' = r or rows - 1 - r, c' = c or cols - 1 - c: tiles of 64 x 64 elements
// through LDS, rows of the tile read and written as whole runs of 64 neighbouring elements.  E: the element as an
// unsigned integer of its size.
template <typename E>
__global__ __launch_bounds__(256) void transpose_tile_kernel(const E* __restrict__ in, E* __restrict__ out, int64_t rows,
                                                             int64_t cols, int tiles_r, int tiles_c, int rev_r, int rev_c) {
  __shared__ E tile[64][64 + (sizeof(E) == 4 ? 1 : 2)];
  const int t = (int)blockIdx.x;
  const int tc = t % tiles_c, rest = t / tiles_c;
  const int tr = rest % tiles_r;
  const int64_t b = rest / tiles_r;
  const int64_t r0 = (int64_t)tr * 64, c0 = (int64_t)tc * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const E* src = in + b * rows * cols;
  E* dst = out + b * rows * cols;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t r = r0 + ty + 4 * i, c = c0 + tx;
    if (r < rows && c < cols) tile[ty + 4 * i][tx] = src[(rev_r ? rows - 1 - r : r) * cols + (rev_c ? cols - 1 - c : c)];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t c = c0 + ty + 4 * i, r = r0 + tx;
    if (c < cols && r < rows) dst[c * rows + r] = tile[tx][ty + 4 * i];
  }
}

}  // namespace
}  // namespace mega

extern "C" int mega_transpose_2d(const void* in, void* out, int elem_bytes, int64_t batch, int64_t rows, int64_t cols,
                                 int reverse_rows, int reverse_cols, void* stream) {
  MEGA_REQUIRE(elem_bytes == 2 || elem_bytes == 4, MEGA_ERR_ARG, "transpose_2d: elements of 2 or 4 bytes, got %d",
               elem_bytes);
  MEGA_REQUIRE(batch >= 0 && rows >= 0 && cols >= 0, MEGA_ERR_ARG, "transpose_2d: bad sizes %lld x %lld x %lld",
               (long long)batch, (long long)rows, (long long)cols);
  if (batch == 0 || rows == 0 || cols == 0) return MEGA_OK;
  MEGA_REQUIRE(in && out && in != out, MEGA_ERR_ARG, "transpose_2d: null or aliased pointer argument");
  const int64_t tr = (rows + 63) / 64, tc = (cols + 63) / 64;
  MEGA_REQUIRE(batch * tr * tc < ((int64_t)1 << 31), MEGA_ERR_UNSUPPORTED, "transpose_2d: too many tiles");
  const dim3 grid((unsigned)(batch * tr * tc));
  hipStream_t s = (hipStream_t)stream;
  if (elem_bytes == 4)
    hipLaunchKernelGGL((mega::transpose_tile_kernel<uint32_t>), grid, dim3(256), 0, s, (const uint32_t*)in, (uint32_t*)out,
                       rows, cols, (int)tr, (int)tc, reverse_rows ? 1 : 0, reverse_cols ? 1 : 0);
  else
    hipLaunchKernelGGL((mega::transpose_tile_kernel<uint16_t>), grid, dim3(256), 0, s, (const uint16_t*)in, (uint16_t*)out,
                       rows, cols, (int)tr, (int)tc, reverse_rows ? 1 : 0, reverse_cols ? 1 : 0);
  MEGA_CHECK_LAUNCH("transpose_2d");
  return MEGA_OK;
}

extern "C" int mega_colsum(const void* x, int64_t row_stride, int dtype, int64_t T_, int64_t W, void* out,
                           int out_dtype, void* workspace, size_t workspace_bytes, void* stream) {
  MEGA_REQUIRE((dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16) &&
                   (out_dtype == MEGA_F32 || out_dtype == MEGA_BF16 || out_dtype == MEGA_F16),
               MEGA_ERR_ARG, "colsum: unknown dtype %d / %d", dtype, out_dtype);
  MEGA_REQUIRE(T_ >= 0 && W >= 1 && W < (1ll << 30) && row_stride >= W, MEGA_ERR_ARG,
               "colsum: bad sizes T=%lld W=%lld row stride %lld", (long long)T_, (long long)W, (long long)row_stride);
  MEGA_REQUIRE(out, MEGA_ERR_ARG, "colsum: null pointer argument");
  hipStream_t s = (hipStream_t)stream;
  const size_t esz = dtype == MEGA_F32 ? 4 : 2;
  if (T_ == 0) {
    MEGA_REQUIRE(out_dtype == MEGA_F32 ? true : (W % 2 == 0), MEGA_ERR_UNSUPPORTED,
                 "colsum: an empty matrix with an odd number of 16-bit columns");
    zero_async(out, (size_t)W * (out_dtype == MEGA_F32 ? 4 : 2), s);
    return MEGA_OK;
  }
  MEGA_REQUIRE(x, MEGA_ERR_ARG, "colsum: null pointer argument");
  // whole 16-byte pieces per lane: the width, the row pitch and the base address in pieces
  MEGA_REQUIRE((W * esz) % 16 == 0 && (row_stride * esz) % 16 == 0 && ((uintptr_t)x % 16) == 0, MEGA_ERR_UNSUPPORTED,
               "colsum: rows of whole 16-byte pieces only (W=%lld, row stride %lld)", (long long)W, (long long)row_stride);
  const size_t need = mega_colsum_workspace_bytes(T_, W);
  MEGA_REQUIRE(workspace && workspace_bytes >= need, MEGA_ERR_WORKSPACE, "colsum: workspace of %zu bytes needed", need);
  switch (dtype) {
    case MEGA_F32: return launch_colsum<float>(x, row_stride, T_, W, out, out_dtype, (float*)workspace, s);
    case MEGA_BF16: return launch_colsum<bf16_t>(x, row_stride, T_, W, out, out_dtype, (float*)workspace, s);
    default: return launch_colsum<f16_t>(x, row_stride, T_, W, out, out_dtype, (float*)workspace, s);
  }
}
