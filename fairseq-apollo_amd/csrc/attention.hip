// Attention softmax (right-aligned causal mask, fully masked rows -> zeros) and the fused
// attention op y = softmax_causal(scale q k^T) v.
//
// Semantics: fairseq/csrc/softmax.cuh:90-153 (row r of an [outer, inner] matrix keeps the
// first inner - outer + r + 1 columns; a row whose maximum is -inf, or whose sum is zero,
// becomes zeros) and fairseq/csrc/ops/attention_kernel.cu:40-131 (q, k: [B,L,Nh,H1],
// v: [B,L,Nh,H2]).
#include "common.h"

namespace mega {

// matrix-core path (attention_mfma.hip)
bool attention_mfma_covers(int dtype, const void* q, const void* k, const void* v, int64_t B, int64_t L, int64_t Nh,
                           int64_t H1, int64_t H2);
size_t attention_mfma_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t Nh, int64_t H2);
int attention_mfma_run(const void* q, const void* k, const void* v, void* y, void* w, int dtype, int64_t B, int64_t L,
                       int64_t Nh, int64_t H1, int64_t H2, float scale, int causal, float dropout, uint64_t seed,
                       void* ws, hipStream_t s);
bool attention_mfma_bwd_covers(int dtype, const void* dy, const void* q, const void* k, const void* v, const void* dq,
                               const void* dk, const void* dv, int64_t B, int64_t L, int64_t Nh, int64_t H1,
                               int64_t H2);
size_t attention_mfma_bwd_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t Nh, int64_t H1, int64_t H2);
int attention_mfma_bwd_run(const void* dy, const void* q, const void* k, const void* v, const void* w, const void* y,
                           void* dq, void* dk, void* dv, int dtype, int64_t B, int64_t L, int64_t Nh, int64_t H1, int64_t H2,
                           float scale, int causal, void* ws, hipStream_t s);

namespace {

constexpr int kBlock = 256;

__device__ __forceinline__ float block_reduce(float v, float* red, bool is_max) {
  for (int m = 32; m >= 1; m >>= 1) {
    const float o = __shfl_xor(v, m);
    v = is_max ? fmaxf(v, o) : v + o;
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float r = red[0];
  for (int i = 1; i < kBlock / 64; ++i) r = is_max ? fmaxf(r, red[i]) : r + red[i];
  return r;
}

// DropKey (fairseq/csrc/softmax.cuh:157-185): a score whose uniform draw falls below `dropout` is
// replaced by -inf before the softmax, so the surviving keys of the row still sum to one.
__device__ __forceinline__ float drop_key(float v, float dropout, uint64_t seed, uint64_t idx) {
  return (dropout > 0.f && hash_uniform(seed, idx) < dropout) ? -INFINITY : v;
}

// one workgroup per row
template <typename T>
__global__ __launch_bounds__(kBlock) void softmax_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                         int64_t outer, int64_t inner, int causal, float dropout,
                                                         uint64_t seed) {
  __shared__ float red[kBlock / 64];
  const int64_t row = blockIdx.x;
  const int64_t r = row % outer;
  int64_t n = causal ? inner - outer + r + 1 : inner;
  if (n < 0) n = 0;
  const T* xp = x + row * inner;
  T* yp = y + row * inner;
  const uint64_t e0 = (uint64_t)row * (uint64_t)inner;
  float m = -INFINITY;
  for (int64_t j = threadIdx.x; j < n; j += kBlock) m = fmaxf(m, drop_key(to_float(xp[j]), dropout, seed, e0 + j));
  m = block_reduce(m, red, true);
  const bool dead = !(m > -INFINITY) || !(m < INFINITY);
  float s = 0.f;
  if (!dead)
    for (int64_t j = threadIdx.x; j < n; j += kBlock)
      s += __expf(drop_key(to_float(xp[j]), dropout, seed, e0 + j) - m);
  s = block_reduce(s, red, false);
  const float c = (dead || s == 0.f) ? 0.f : 1.0f / s;
  for (int64_t j = threadIdx.x; j < inner; j += kBlock) {
    const float e = (j < n && !dead) ? __expf(drop_key(to_float(xp[j]), dropout, seed, e0 + j) - m) * c : 0.f;
    yp[j] = from_float<T>(e);
  }
}

// Plain attention: one workgroup per (b, head, query row); scores of the row live in LDS.
template <typename T>
__global__ __launch_bounds__(kBlock) void attention_row_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                               const T* __restrict__ v, T* __restrict__ y,
                                                               T* __restrict__ w, int B, int L, int Nh, int H1,
                                                               int H2, float scale, int causal, float dropout,
                                                               uint64_t seed) {
  extern __shared__ float sc[];     // [L] scores, then [H1] the query row
  __shared__ float red[kBlock / 64];
  float* qs = sc + L;
  const int l = blockIdx.x % L;
  const int n = (blockIdx.x / L) % Nh;
  const int b = blockIdx.x / (L * Nh);
  const int nk = causal ? l + 1 : L;
  const T* qp = q + (((size_t)b * L + l) * Nh + n) * H1;
  const uint64_t e0 = (((uint64_t)b * Nh + n) * L + l) * L;     // the row's place in the [B,Nh,L,L] weights
  for (int i = threadIdx.x; i < H1; i += kBlock) qs[i] = to_float(qp[i]);
  __syncthreads();
  float m = -INFINITY;
  for (int j = threadIdx.x; j < nk; j += kBlock) {
    const T* kp = k + (((size_t)b * L + j) * Nh + n) * H1;
    float s = 0.f;
    for (int i = 0; i < H1; ++i) s += qs[i] * to_float(kp[i]);
    s = drop_key(s * scale, dropout, seed, e0 + j);
    sc[j] = s;
    m = fmaxf(m, s);
  }
  m = block_reduce(m, red, true);
  const bool dead = !(m > -INFINITY) || !(m < INFINITY);
  float s = 0.f;
  for (int j = threadIdx.x; j < nk; j += kBlock) {
    const float e = dead ? 0.f : __expf(sc[j] - m);     // exp(-inf - m) = 0 for a dropped key
    sc[j] = e;
    s += e;
  }
  s = block_reduce(s, red, false);
  const float c = (dead || s == 0.f) ? 0.f : 1.0f / s;
  __syncthreads();
  if (w) {
    T* wp = w + (((size_t)b * Nh + n) * L + l) * L;
    for (int j = threadIdx.x; j < L; j += kBlock) wp[j] = from_float<T>(j < nk ? sc[j] * c : 0.f);
  }
  T* yp = y + (((size_t)b * L + l) * Nh + n) * H2;
  for (int f = threadIdx.x; f < H2; f += kBlock) {
    float acc = 0.f;
    for (int j = 0; j < nk; ++j) acc += sc[j] * to_float(v[(((size_t)b * L + j) * Nh + n) * H2 + f]);
    yp[f] = from_float<T>(acc * c);
  }
}

// Softmax backward (fairseq/csrc/softmax.cuh AttentionSoftmaxBwdKernel, called from
// ops/attention_softmax_kernel.cu and ops/attention_kernel.cu:195-203):
//   dx[r, c] = scale * y[r, c] * (dy[r, c] - sum_c' y[r, c'] dy[r, c']).
// One wave per row, four rows per workgroup; columns behind the causal limit hold y = 0 and are
// written as zeros without being read.  dx may alias dy.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void softmax_bwd_kernel(const T* dy, const T* __restrict__ y,
                                                          T* dx, int64_t rows, int outer, int inner, int causal,
                                                          float scale) {
  using V = Vec<T, VEC>;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int r = (int)(row % outer);
  int limit = causal ? inner - outer + r + 1 : inner;     // columns that can be non-zero
  if (limit < 0) limit = 0;
  if (limit > inner) limit = inner;
  const T* dyr = dy + row * inner;
  const T* yr = y + row * inner;
  T* dxr = dx + row * inner;
  float dot = 0.f;
  for (int c = lane * VEC; c < limit; c += 64 * VEC) {
    const V a = *(const V*)(dyr + c);
    const V b = *(const V*)(yr + c);
#pragma unroll
    for (int e = 0; e < VEC; ++e)
      if (c + e < limit) dot = fmaf(to_float(a.v[e]), to_float(b.v[e]), dot);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) dot += __shfl_xor(dot, o);
  for (int c = lane * VEC; c < inner; c += 64 * VEC) {
    V o;
    if (c < limit) {
      const V a = *(const V*)(dyr + c);
      const V b = *(const V*)(yr + c);
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        o.v[e] = from_float<T>(c + e < limit ? scale * to_float(b.v[e]) * (to_float(a.v[e]) - dot) : 0.f);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) o.v[e] = from_float<T>(0.f);
    }
    *(V*)(dxr + c) = o;
  }
}

template <typename T>
int launch_softmax_bwd(const void* dy, const void* y, void* dx, int64_t rows, int64_t outer, int64_t inner, int causal,
                       float scale, hipStream_t s) {
  constexpr int FULL = 16 / (int)sizeof(T);
  const dim3 grid((unsigned)ceil_div(rows, 4));
  const bool vec = inner % FULL == 0 && ((((uintptr_t)dy | (uintptr_t)y | (uintptr_t)dx) % 16) == 0);
  if (vec)
    hipLaunchKernelGGL((softmax_bwd_kernel<T, FULL>), grid, dim3(256), 0, s, (const T*)dy, (const T*)y, (T*)dx, rows,
                       (int)outer, (int)inner, causal, scale);
  else
    hipLaunchKernelGGL((softmax_bwd_kernel<T, 1>), grid, dim3(256), 0, s, (const T*)dy, (const T*)y, (T*)dx, rows,
                       (int)outer, (int)inner, causal, scale);
  MEGA_CHECK_LAUNCH("attention_softmax_bwd");
  return MEGA_OK;
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_attention_softmax_fwd(const void* x, void* y, int dtype, int64_t batch, int64_t outer,
                                          int64_t inner, int causal, float dropout, uint64_t seed, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "attention_softmax_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(batch >= 0 && outer >= 0 && inner >= 0, MEGA_ERR_ARG, "attention_softmax_fwd: negative size");
  MEGA_REQUIRE(dropout >= 0.f && dropout <= 1.f, MEGA_ERR_ARG, "attention_softmax_fwd: dropout %g outside [0, 1]",
               (double)dropout);
  const int64_t rows = batch * outer;
  if (rows == 0 || inner == 0) return MEGA_OK;
  MEGA_REQUIRE(x && y, MEGA_ERR_ARG, "attention_softmax_fwd: null pointer argument");
  MEGA_REQUIRE(rows < (int64_t)1 << 31, MEGA_ERR_UNSUPPORTED, "attention_softmax_fwd: too many rows");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)rows);
  switch (dtype) {
    case MEGA_F32:
      hipLaunchKernelGGL(softmax_kernel<float>, grid, dim3(kBlock), 0, s, (const float*)x, (float*)y, outer, inner, causal,
                         dropout, seed);
      break;
    case MEGA_BF16:
      hipLaunchKernelGGL(softmax_kernel<bf16_t>, grid, dim3(kBlock), 0, s, (const bf16_t*)x, (bf16_t*)y, outer, inner, causal,
                         dropout, seed);
      break;
    default:
      hipLaunchKernelGGL(softmax_kernel<f16_t>, grid, dim3(kBlock), 0, s, (const f16_t*)x, (f16_t*)y, outer, inner, causal,
                         dropout, seed);
      break;
  }
  MEGA_CHECK_LAUNCH("attention_softmax_fwd");
  return MEGA_OK;
}

extern "C" size_t mega_attention_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t Nh, int64_t H1,
                                                 int64_t H2) {
  if (B <= 0 || L <= 0 || Nh <= 0 || H1 <= 0 || H2 <= 0 || dtype == MEGA_F32 || H1 % 8 != 0) return 0;
  return attention_mfma_workspace_bytes(dtype, B, L, Nh, H2);
}

extern "C" int mega_attention_fwd(const void* q, const void* k, const void* v, void* y, void* w, int dtype,
                                  int64_t B, int64_t L, int64_t Nh, int64_t H1, int64_t H2, float scale,
                                  int causal, float dropout, uint64_t seed, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "attention_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(dropout >= 0.f && dropout <= 1.f, MEGA_ERR_ARG, "attention_fwd: dropout %g outside [0, 1]",
               (double)dropout);
  MEGA_REQUIRE(B >= 0 && L >= 0 && Nh > 0 && H1 > 0 && H2 > 0, MEGA_ERR_ARG, "attention_fwd: bad shape");
  if (B == 0 || L == 0) return MEGA_OK;
  MEGA_REQUIRE(q && k && v && (y || w), MEGA_ERR_ARG, "attention_fwd: null pointer argument");
  MEGA_REQUIRE(y || attention_mfma_covers(dtype, q, k, v, B, L, Nh, H1, H2), MEGA_ERR_UNSUPPORTED,
               "attention_fwd: the weights alone (y = NULL) are formed on the matrix-core path only");
  MEGA_REQUIRE(B * L * Nh < (int64_t)1 << 31, MEGA_ERR_UNSUPPORTED, "attention_fwd: too many rows");
  if (attention_mfma_covers(dtype, q, k, v, B, L, Nh, H1, H2)) {
    const size_t need = attention_mfma_workspace_bytes(dtype, B, L, Nh, H2);
    MEGA_REQUIRE(workspace && workspace_bytes >= need && ((uintptr_t)workspace % 256) == 0, MEGA_ERR_WORKSPACE,
                 "attention_fwd: workspace of %zu bytes (256-byte aligned) needed", need);
    return attention_mfma_run(q, k, v, y, w, dtype, B, L, Nh, H1, H2, scale, causal, dropout, seed, workspace,
                              (hipStream_t)stream);
  }
  const size_t smem = (size_t)(L + H1) * 4;
  MEGA_REQUIRE(smem <= 150 * 1024, MEGA_ERR_UNSUPPORTED, "attention_fwd: L=%ld too long for one chunk", (long)L);
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)(B * L * Nh));
#define LAUNCH_ATT(T)                                                                                      \
  do {                                                                                                     \
    if (smem > 64 * 1024)                                                                                  \
      hipFuncSetAttribute((const void*)attention_row_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                          (int)smem);                                                                      \
    hipLaunchKernelGGL(attention_row_kernel<T>, grid, dim3(kBlock), smem, s, (const T*)q, (const T*)k,     \
                       (const T*)v, (T*)y, (T*)w, (int)B, (int)L, (int)Nh, (int)H1, (int)H2, scale, causal,  \
                       dropout, seed);                                                                     \
  } while (0)
  switch (dtype) {
    case MEGA_F32: LAUNCH_ATT(float); break;
    case MEGA_BF16: LAUNCH_ATT(bf16_t); break;
    default: LAUNCH_ATT(f16_t); break;
  }
#undef LAUNCH_ATT
  MEGA_CHECK_LAUNCH("attention_fwd");
  return MEGA_OK;
}

extern "C" int mega_attention_softmax_bwd(const void* y_grad, const void* y, void* x_grad, int dtype, int64_t batch,
                                          int64_t outer, int64_t inner, int causal, float scale, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "attention_softmax_bwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(batch >= 0 && outer >= 0 && inner >= 0, MEGA_ERR_ARG, "attention_softmax_bwd: negative size");
  const int64_t rows = batch * outer;
  if (rows == 0 || inner == 0) return MEGA_OK;
  MEGA_REQUIRE(y_grad && y && x_grad, MEGA_ERR_ARG, "attention_softmax_bwd: null pointer argument");
  MEGA_REQUIRE(rows < (int64_t)1 << 33 && inner < (int64_t)1 << 30 && outer < (int64_t)1 << 30, MEGA_ERR_UNSUPPORTED,
               "attention_softmax_bwd: shape too large");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MEGA_F32: return launch_softmax_bwd<float>(y_grad, y, x_grad, rows, outer, inner, causal, scale, s);
    case MEGA_BF16: return launch_softmax_bwd<bf16_t>(y_grad, y, x_grad, rows, outer, inner, causal, scale, s);
    default: return launch_softmax_bwd<f16_t>(y_grad, y, x_grad, rows, outer, inner, causal, scale, s);
  }
}

extern "C" size_t mega_attention_bwd_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t Nh, int64_t H1,
                                                     int64_t H2) {
  if (B <= 0 || L <= 0 || Nh <= 0 || H1 <= 0 || H2 <= 0 || dtype == MEGA_F32 || H1 % 8 != 0 || H2 % 8 != 0) return 0;
  if (B * Nh > 65535 || L >= (int64_t)1 << 15) return 0;
  return attention_mfma_bwd_workspace_bytes(dtype, B, L, Nh, H1, H2);
}

extern "C" int mega_attention_bwd(const void* y_grad, const void* q, const void* k, const void* v, const void* w,
                                  const void* y, void* q_grad, void* k_grad, void* v_grad, int dtype, int64_t B, int64_t L,
                                  int64_t Nh, int64_t H1, int64_t H2, float scale, int causal, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_BF16 || dtype == MEGA_F16, dtype == MEGA_F32 ? MEGA_ERR_UNSUPPORTED : MEGA_ERR_ARG,
               "attention_bwd: 16-bit activations only (dtype %d)", dtype);
  MEGA_REQUIRE(B >= 0 && L >= 0 && Nh > 0 && H1 > 0 && H2 > 0, MEGA_ERR_ARG, "attention_bwd: bad shape");
  if (B == 0 || L == 0) return MEGA_OK;
  MEGA_REQUIRE(y_grad && q && k && v && w && q_grad && k_grad && v_grad, MEGA_ERR_ARG,
               "attention_bwd: null pointer argument");
  MEGA_REQUIRE(attention_mfma_bwd_covers(dtype, y_grad, q, k, v, q_grad, k_grad, v_grad, B, L, Nh, H1, H2),
               MEGA_ERR_UNSUPPORTED,
               "attention_bwd: needs H1 %% 8 == 0, H2 %% 8 == 0, 16-byte aligned tensors, B * Nh <= 65535, L < 32768");
  const size_t need = attention_mfma_bwd_workspace_bytes(dtype, B, L, Nh, H1, H2);
  MEGA_REQUIRE(workspace && workspace_bytes >= need && ((uintptr_t)workspace % 256) == 0, MEGA_ERR_WORKSPACE,
               "attention_bwd: workspace of %zu bytes (256-byte aligned) needed", need);
  return attention_mfma_bwd_run(y_grad, q, k, v, w, y, q_grad, k_grad, v_grad, dtype, B, L, Nh, H1, H2, scale, causal,
                                workspace, (hipStream_t)stream);
}
