// Long convolution with an explicit time-domain kernel k[K, Lk]:
//   causal         y[b,d,t] = sum_{j<Lk} k[d,j] x[b,d,t-j]
//   bidirectional  + sum_{m>=1} k[D+d,m-1] x[b,d,t+m]            (shift)
//                  + sum_{m>=0} k[D+d,m]   x[b,d,t+m]            (no shift)
// i.e. what fftconv / bidirectional_fftconv return
// (fairseq/modules/fused_ops/fftconv.py:45-61, 85-100), evaluated directly in the time
// domain with fp32 accumulation: a workgroup owns 256 outputs of one row and walks the lags
// in blocks of 256 staged through LDS.
#include "common.h"

namespace mega {
namespace {

constexpr int kT = 256;

template <typename T>
__global__ __launch_bounds__(kT) void long_conv_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                       const float* __restrict__ k, int D, int L, int Lk,
                                                       int bidirectional, int shift) {
  __shared__ float ks[kT];
  __shared__ float xs[2 * kT];
  const int row = blockIdx.x;             // b*D + d
  const int d = row % D;
  const int t0 = blockIdx.y * kT;
  const int t = t0 + threadIdx.x;
  const T* xr = x + (size_t)row * L;
  float acc = 0.f;
  // causal half: lags j in [0, min(Lk, t0 + kT))
  const int jmax = min(Lk, t0 + kT);
  for (int j0 = 0; j0 < jmax; j0 += kT) {
    __syncthreads();
    ks[threadIdx.x] = (j0 + threadIdx.x < Lk) ? k[(size_t)d * Lk + j0 + threadIdx.x] : 0.f;
    // x window: indices t0 - j0 - (kT-1) ... t0 - j0 + (kT-1)
    const int base = t0 - j0 - (kT - 1);
    for (int i = threadIdx.x; i < 2 * kT - 1; i += kT) {
      const int xi = base + i;
      xs[i] = (xi >= 0 && xi < L) ? to_float(xr[xi]) : 0.f;
    }
    __syncthreads();
    // y[t] += sum_jj ks[jj] * x[t - j0 - jj];  x index in window = threadIdx.x + kT-1 - jj
#pragma unroll 8
    for (int jj = 0; jj < kT; ++jj) acc += ks[jj] * xs[threadIdx.x + kT - 1 - jj];
  }
  if (bidirectional) {
    // anti-causal half: offsets m; tap index m-1 (shift) or m (no shift)
    const float* k2 = k + (size_t)(D + d) * Lk;
    const int mlo = shift ? 1 : 0;
    const int mhi = min(shift ? Lk : Lk - 1, L - 1 - t0);     // largest useful offset
    for (int m0 = mlo; m0 <= mhi; m0 += kT) {
      __syncthreads();
      const int tap = m0 + threadIdx.x - (shift ? 1 : 0);
      ks[threadIdx.x] = (tap >= 0 && tap < Lk) ? k2[tap] : 0.f;
      // x window: indices t0 + m0 ... t0 + m0 + 2kT-2
      for (int i = threadIdx.x; i < 2 * kT - 1; i += kT) {
        const int xi = t0 + m0 + i;
        xs[i] = (xi < L) ? to_float(xr[xi]) : 0.f;
      }
      __syncthreads();
#pragma unroll 8
      for (int mm = 0; mm < kT; ++mm) acc += ks[mm] * xs[threadIdx.x + mm];
    }
  }
  if (t < L) y[(size_t)row * L + t] = from_float<T>(acc);
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_long_conv_fwd(const void* x, void* y, int dtype, const float* k, int64_t B, int64_t D,
                                  int64_t L, int64_t Lk, int bidirectional, int shift, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "long_conv_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && D > 0 && L >= 0 && Lk > 0, MEGA_ERR_ARG, "long_conv_fwd: bad shape");
  MEGA_REQUIRE(Lk <= L || L == 0, MEGA_ERR_ARG, "long_conv_fwd: kernel length %ld exceeds sequence length %ld",
               (long)Lk, (long)L);
  if (B == 0 || L == 0) return MEGA_OK;
  MEGA_REQUIRE(x && y && k, MEGA_ERR_ARG, "long_conv_fwd: null pointer argument");
  MEGA_REQUIRE(B * D < (int64_t)1 << 31 && L < (int64_t)65535 * kT, MEGA_ERR_UNSUPPORTED, "long_conv_fwd: shape too large");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)(B * D), (unsigned)ceil_div(L, kT));
  switch (dtype) {
    case MEGA_F32:
      hipLaunchKernelGGL(long_conv_kernel<float>, grid, dim3(kT), 0, s, (const float*)x, (float*)y, k, (int)D, (int)L,
                         (int)Lk, bidirectional, shift);
      break;
    case MEGA_BF16:
      hipLaunchKernelGGL(long_conv_kernel<bf16_t>, grid, dim3(kT), 0, s, (const bf16_t*)x, (bf16_t*)y, k, (int)D,
                         (int)L, (int)Lk, bidirectional, shift);
      break;
    default:
      hipLaunchKernelGGL(long_conv_kernel<f16_t>, grid, dim3(kT), 0, s, (const f16_t*)x, (f16_t*)y, k, (int)D, (int)L,
                         (int)Lk, bidirectional, shift);
      break;
  }
  MEGA_CHECK_LAUNCH("long_conv_fwd");
  return MEGA_OK;
}
