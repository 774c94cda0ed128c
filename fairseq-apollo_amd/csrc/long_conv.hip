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

// ---- the same convolutions through a Fourier transform held in LDS, O(M log M) per row instead of
// O(L Lk): the reference's route (fftconv_kernel.cu:40-78 with the shuffle FFT of fft.cuh:461-533; n = 2 *
// pow2ceil(L), fused_ops/fftconv.py:45-61).  M = pow2ceil(L + Lk) points, complex fp32, one workgroup of 1024
// threads per channel: the (real) kernel row is transformed once and its spectrum kept in registers; the
// batch rows of the channel go through in pairs, row b in the real and row b + 1 in the imaginary part (the
// kernel is real, so the two convolutions do not mix).  Forward transform by decimation in frequency (natural
// order in, bit-reversed out), product with the spectrum in that order, inverse by decimation in time
// (bit-reversed in, natural out): no reordering pass.
// A pass takes three stages at once (radix 8; the remainder of the stages as one pass of radix 2 or 4): a thread
// holds the eight points of a butterfly group in registers, so the buffer in LDS is read and written, and the
// workgroup meets at a barrier, once per three stages.  One twiddle factor per group comes from v_sin_f32 /
// v_cos_f32 (argument in revolutions, an exact fraction), the factors of the other two stages are its squares and
// the fixed eighth roots of unity are written out.  Point i of the buffer lives at slot i + (i >> 3): with one
// spare slot per eight points the eight-point groups of the last passes (64 contiguous bytes per thread) spread
// over the banks.
#ifndef MEGA_LC_FFT_MIN
#define MEGA_LC_FFT_MIN 512        // shortest kernel that takes the transform
#endif
constexpr int kFT = 1024;
constexpr int kFftMaxLog = 14;            // M <= 16384: 144 KB of LDS with the spare slots

__device__ __forceinline__ int fslot(int i) { return i + (i >> 3); }

__device__ __forceinline__ float2 cmulf(float2 a, float2 b) {
  return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x);
}
__device__ __forceinline__ float2 caddf(float2 a, float2 b) { return make_float2(a.x + b.x, a.y + b.y); }
__device__ __forceinline__ float2 csubf(float2 a, float2 b) { return make_float2(a.x - b.x, a.y - b.y); }
// v * exp(-+ 2 pi i k / 8), k = 0..3 (SIGN = -1: forward, +1: inverse)
template <int K8, int SIGN>
__device__ __forceinline__ float2 rot8(float2 v) {
  constexpr float h = 0.70710678118654752440f;
  if (K8 == 0) return v;
  if (K8 == 2) return SIGN < 0 ? make_float2(v.y, -v.x) : make_float2(-v.y, v.x);
  if (K8 == 1) return SIGN < 0 ? make_float2((v.x + v.y) * h, (v.y - v.x) * h) : make_float2((v.x - v.y) * h, (v.x + v.y) * h);
  return SIGN < 0 ? make_float2((v.y - v.x) * h, -(v.x + v.y) * h) : make_float2(-(v.x + v.y) * h, (v.x - v.y) * h);
}

// One pass of the forward transform over stages s, s - 1, ..., s - R + 1 (stage t pairs points 2^t apart).
// A group: the 2^R points base + q h, h = 2^(s - R + 1), of one block of 2^(s + 1) points.
template <int R>
__device__ __forceinline__ void dif_pass(float2* buf, const int s, const int M) {
  constexpr int N = 1 << R;
  const int lh = s - R + 1, h = 1 << lh;
  const float inv = 1.0f / (float)(2 << s);
  for (int g = threadIdx.x; g < (M >> R); g += kFT) {
    const int pos = g & (h - 1);
    const int base = ((g >> lh) << (s + 1)) + pos;
    float2 v[N];
#pragma unroll
    for (int q = 0; q < N; ++q) v[q] = buf[fslot(base + q * h)];
    const float fr = (float)pos * inv;                                       // pos / 2^(s+1) revolutions
    float2 w = make_float2(__builtin_amdgcn_cosf(fr), -__builtin_amdgcn_sinf(fr));
#pragma unroll
    for (int l = 0; l < R; ++l) {
      const int dist = N >> (l + 1);
      // the twiddle of stage s - l for point base' + q' h: w^(2^l) times exp(-2 pi i q' / (2 dist))
#pragma unroll
      for (int q = 0; q < N; ++q) {
        if (q & dist) continue;
        const int qp = q & (dist - 1);
        const float2 a = v[q], b = v[q + dist];
        v[q] = caddf(a, b);
        float2 d = cmulf(csubf(a, b), w);
        // eighth roots: k8 = qp * 8 / (2 dist)
        const int k8 = qp * 4 / dist;
        d = k8 == 0 ? d : k8 == 1 ? rot8<1, -1>(d) : k8 == 2 ? rot8<2, -1>(d) : rot8<3, -1>(d);
        v[q + dist] = d;
      }
      w = cmulf(w, w);
    }
#pragma unroll
    for (int q = 0; q < N; ++q) buf[fslot(base + q * h)] = v[q];
  }
}

// One pass of the inverse transform over stages s, s + 1, ..., s + R - 1.  A group: the 2^R points base + q 2^s of
// one block of 2^(s + R) points.
template <int R>
__device__ __forceinline__ void dit_pass(float2* buf, const int s, const int M) {
  constexpr int N = 1 << R;
  const int h = 1 << s;
  const float inv = 1.0f / (float)(h << R);
  for (int g = threadIdx.x; g < (M >> R); g += kFT) {
    const int pos = g & (h - 1);
    const int base = ((g >> s) << (s + R)) + pos;
    float2 v[N];
#pragma unroll
    for (int q = 0; q < N; ++q) v[q] = buf[fslot(base + q * h)];
    // twiddles of the R stages: the smallest angle from the hardware, the others by squaring
    float2 w[R];
    const float fr = (float)pos * inv;                                       // pos / 2^(s+R) revolutions
    w[R - 1] = make_float2(__builtin_amdgcn_cosf(fr), __builtin_amdgcn_sinf(fr));
#pragma unroll
    for (int l = R - 2; l >= 0; --l) w[l] = cmulf(w[l + 1], w[l + 1]);
#pragma unroll
    for (int l = 0; l < R; ++l) {
      const int dist = 1 << l;
#pragma unroll
      for (int q = 0; q < N; ++q) {
        if (q & dist) continue;
        const int qp = q & (dist - 1);
        float2 t = cmulf(v[q + dist], w[l]);
        const int k8 = qp * 4 / dist;
        t = k8 == 0 ? t : k8 == 1 ? rot8<1, 1>(t) : k8 == 2 ? rot8<2, 1>(t) : rot8<3, 1>(t);
        const float2 a = v[q];
        v[q] = caddf(a, t);
        v[q + dist] = csubf(a, t);
      }
    }
#pragma unroll
    for (int q = 0; q < N; ++q) buf[fslot(base + q * h)] = v[q];
  }
}

// forward: natural order -> bit-reversed order
__device__ __forceinline__ void fft_dif(float2* buf, int logm) {
  const int M = 1 << logm;
  int s = logm - 1;
  for (; s >= 2; s -= 3) {
    __syncthreads();
    dif_pass<3>(buf, s, M);
  }
  if (s >= 0) {
    __syncthreads();
    if (s == 1) dif_pass<2>(buf, s, M);
    else dif_pass<1>(buf, s, M);
  }
  __syncthreads();
}

// inverse (unscaled): bit-reversed order -> natural order
__device__ __forceinline__ void fft_dit_inverse(float2* buf, int logm) {
  const int M = 1 << logm;
  int s = 0;
  const int rem = logm % 3;
  if (rem) {
    __syncthreads();
    if (rem == 2) dit_pass<2>(buf, 0, M);
    else dit_pass<1>(buf, 0, M);
    s = rem;
  }
  for (; s < logm; s += 3) {
    __syncthreads();
    dit_pass<3>(buf, s, M);
  }
  __syncthreads();
}

template <typename T>
__global__ __launch_bounds__(kFT) void long_conv_fft_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                            const float* __restrict__ k, int B, int D, int L, int Lk,
                                                            int logm, int bidirectional, int shift) {
  extern __shared__ float2 fbuf[];                   // M complex values at slots i + (i >> 3)
  const int M = 1 << logm;
  const int d = blockIdx.x;
  constexpr int kPer = (1 << kFftMaxLog) / kFT;      // spectrum values per thread at the largest M
  // ---- the kernel row(s) of the channel as one sequence of period M: lags 0 .. Lk - 1 at the front, the
  // anti-causal taps of the second row at the back (offset m at index M - m)
  for (int i = threadIdx.x; i < M; i += kFT) fbuf[fslot(i)] = make_float2(i < Lk ? k[(size_t)d * Lk + i] : 0.f, 0.f);
  if (bidirectional) {
    __syncthreads();
    const float* k2 = k + (size_t)(D + d) * Lk;
    for (int tap = threadIdx.x; tap < Lk; tap += kFT) {
      const int m = tap + (shift ? 1 : 0);           // x[t + m] meets tap m - 1 (shift) or m
      const int idx = (M - m) & (M - 1);
      fbuf[fslot(idx)].x += k2[tap];
    }
  }
  fft_dif(fbuf, logm);
  float2 Kf[kPer];
  const float scale = 1.0f / (float)M;
#pragma unroll
  for (int e = 0; e < kPer; ++e) {
    const int i = threadIdx.x + e * kFT;
    Kf[e] = i < M ? make_float2(fbuf[fslot(i)].x * scale, fbuf[fslot(i)].y * scale) : make_float2(0.f, 0.f);
  }
  // ---- the rows of the channel, two at a time
  for (int b = blockIdx.y * 2; b < B; b += 2 * gridDim.y) {
    const bool two = b + 1 < B;
    const T* x0 = x + ((size_t)b * D + d) * L;
    const T* x1 = x + ((size_t)(b + 1) * D + d) * L;
    __syncthreads();
    for (int i = threadIdx.x; i < M; i += kFT)
      fbuf[fslot(i)] = i < L ? make_float2(to_float(x0[i]), two ? to_float(x1[i]) : 0.f) : make_float2(0.f, 0.f);
    fft_dif(fbuf, logm);
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
      const int i = threadIdx.x + e * kFT;
      if (i < M) fbuf[fslot(i)] = cmulf(fbuf[fslot(i)], Kf[e]);
    }
    fft_dit_inverse(fbuf, logm);
    T* y0 = y + ((size_t)b * D + d) * L;
    T* y1 = y + ((size_t)(b + 1) * D + d) * L;
    for (int i = threadIdx.x; i < L; i += kFT) {
      const float2 v = fbuf[fslot(i)];
      y0[i] = from_float<T>(v.x);
      if (two) y1[i] = from_float<T>(v.y);
    }
  }
}

// the transform pays off once the kernel is long; it needs M = pow2ceil(L + Lk) complex values in LDS
bool long_conv_fft_plan(int64_t L, int64_t Lk, int* logm) {
  if (Lk < MEGA_LC_FFT_MIN) return false;
  int lg = 0;
  while (((int64_t)1 << lg) < L + Lk) ++lg;
  if (lg > kFftMaxLog || lg < 11) return false;
  *logm = lg;
  return true;
}

template <typename T>
int launch_long_conv_fft(const void* x, void* y, const float* k, int64_t B, int64_t D, int64_t L, int64_t Lk, int logm,
                         int bidirectional, int shift, hipStream_t s) {
  auto kern = long_conv_fft_kernel<T>;
  const size_t smem = ((size_t)9) << logm;             // M + M / 8 slots of 8 bytes
  static uint64_t attr_seen = 0;
  if (first_on_device(&attr_seen)) {
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 9 << kFftMaxLog);
  }
  // enough workgroups to fill the chip: split the batch when there are few channels
  int64_t nb = 1;
  while (D * nb < 512 && nb * 2 <= (B + 1) / 2) nb *= 2;
  hipLaunchKernelGGL(kern, dim3((unsigned)D, (unsigned)nb), dim3(kFT), smem, s, (const T*)x, (T*)y, k, (int)B, (int)D,
                     (int)L, (int)Lk, logm, bidirectional, shift);
  MEGA_CHECK_LAUNCH("long_conv_fwd (transform path)");
  return MEGA_OK;
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
  int logm = 0;
  if (D < 65536 && long_conv_fft_plan(L, Lk, &logm)) {
    switch (dtype) {
      case MEGA_F32: return launch_long_conv_fft<float>(x, y, k, B, D, L, Lk, logm, bidirectional, shift, s);
      case MEGA_BF16: return launch_long_conv_fft<bf16_t>(x, y, k, B, D, L, Lk, logm, bidirectional, shift, s);
      default: return launch_long_conv_fft<f16_t>(x, y, k, B, D, L, Lk, logm, bidirectional, shift, s);
    }
  }
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
