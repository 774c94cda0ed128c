// Parameter-gradient sums of the moving-average layer (unidirectional, no carried state).
//
// The reference forms the kernel gradient dk[d, l] = sum_{b,t} dy[b,d,t] x[b,d,t-l] with FFTs
// (fairseq/modules/fused_ops/fftconv.py:66-88, csrc/ops/fftconv_kernel.cu backward) and then
// reduces it against the powers of q (csrc/ops/ema_parameters.cc:80-97):
//     sum2[d,n] = sum_l dk[d,l] q^l,      sum1[d,n] = sum_l dk[d,l] l q^(l-1)
//     dp = Re(sum2 gamma),  dq = conj(sum1 p gamma),  dgamma = conj(sum2 p).
// Here dk is never formed: with the unscaled state s[t] = q s[t-1] + x[t] and its derivative
// g[t] = q g[t-1] + s[t-1],
//     sum2 = sum_{b,t} dy[t] s[t],        sum1 = sum_{b,t} dy[t] g[t],
// two recurrences of the forward kind run next to each other.  One workgroup owns 16 channels of
// one batch row: thread = (channel, state n), 12 fused multiply-adds per token on the vector
// ALUs; x and dy tiles pass through LDS so that every layout is read with its own coalescing.
// Output: per batch row (the sum over rows is left to the caller: B terms, deterministic)
//   sums [B, D, N, 4] = (Re sum2, Im sum2, Re sum1, Im sum1),  dyx [B, D] = sum_t dy x (for omega).
#include "common.h"

namespace mega {
namespace {

constexpr int kCh = 16;        // channels per workgroup
constexpr int kNs = 16;        // state lanes per channel
constexpr int kTk = 128;       // tokens per LDS tile
constexpr int kBwdThreads = kCh * kNs;
constexpr int kPerThread = kCh * kTk / kBwdThreads;   // elements of one tile a thread moves

struct EmaGradArgs {
  const void* dy;
  const void* x;
  int64_t sgb, sgd, sgl;    // dy strides (elements)
  int64_t sxb, sxd, sxl;    // x strides
  const float* q;           // [D, N, 2]
  const uint8_t* mask;      // [B, L] or null
  float* sums;              // [B, D, N, 4]
  float* dyx;               // [B, D]
  int B, D, N, L;
};

template <typename T>
__global__ __launch_bounds__(kBwdThreads) void ema_param_grad_kernel(const EmaGradArgs A) {
  __shared__ float s_x[kCh][kTk + 4];
  __shared__ float s_g[kCh][kTk + 4];
  __shared__ float s_keep[kTk];
  const int tid = threadIdx.x;
  const int ncb = (A.D + kCh - 1) / kCh;
  const int b = blockIdx.x / ncb;
  const int c0 = (blockIdx.x - b * ncb) * kCh;
  const int ch = tid / kNs, n = tid % kNs;
  const bool state_lane = n < A.N && c0 + ch < A.D;
  const T* xg = (const T*)A.x + b * A.sxb;
  const T* gg = (const T*)A.dy + b * A.sgb;
  // tile-load mapping: consecutive lanes follow whichever axis is contiguous in memory
  const bool x_chan_fast = A.sxd == 1, g_chan_fast = A.sgd == 1;

  float qr = 0.f, qi = 0.f;
  if (state_lane) {
    qr = A.q[((size_t)(c0 + ch) * A.N + n) * 2];
    qi = A.q[((size_t)(c0 + ch) * A.N + n) * 2 + 1];
  }
  float sr = 0.f, si = 0.f, gr = 0.f, gi = 0.f;          // s[t], g[t]
  float a2r = 0.f, a2i = 0.f, a1r = 0.f, a1i = 0.f, ax = 0.f;

  // Tile moves are branch-free (clamped addresses, validity applied when the value is parked in
  // LDS) so that all loads of a tile are in flight together and stay in flight across the
  // arithmetic of the previous tile.
  float px[kPerThread], pg[kPerThread];
  int ex[kPerThread], eg[kPerThread];       // (channel << 16 | token) of every element this thread moves
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    const int e = tid + k * kBwdThreads;
    ex[k] = x_chan_fast ? ((e % kCh) << 16 | (e / kCh)) : ((e / kTk) << 16 | (e % kTk));
    eg[k] = g_chan_fast ? ((e % kCh) << 16 | (e / kCh)) : ((e / kTk) << 16 | (e % kTk));
  }
  const int dmax = A.D - 1 - c0, lmax = A.L - 1;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int k = 0; k < kPerThread; ++k) {
      const int cx = min(ex[k] >> 16, dmax), tx = min(t0 + (ex[k] & 0xffff), lmax);
      const int cg = min(eg[k] >> 16, dmax), tg = min(t0 + (eg[k] & 0xffff), lmax);
      px[k] = to_float(xg[(int64_t)(c0 + cx) * A.sxd + (int64_t)tx * A.sxl]);
      pg[k] = to_float(gg[(int64_t)(c0 + cg) * A.sgd + (int64_t)tg * A.sgl]);
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < A.L; t0 += kTk) {
    __syncthreads();    // the previous tile has been consumed
#pragma unroll
    for (int k = 0; k < kPerThread; ++k) {
      const int cx = ex[k] >> 16, tx = ex[k] & 0xffff, cg = eg[k] >> 16, tg = eg[k] & 0xffff;
      s_x[cx][tx] = (cx <= dmax && t0 + tx <= lmax) ? px[k] : 0.f;
      s_g[cg][tg] = (cg <= dmax && t0 + tg <= lmax) ? pg[k] : 0.f;
    }
    if (tid < kTk) {
      const int tm = min(t0 + tid, lmax);
      const uint8_t mk = A.mask ? A.mask[(size_t)b * A.L + tm] : (uint8_t)0;
      s_keep[tid] = mk ? 0.f : 1.f;
    }
    __syncthreads();
    fetch(t0 + kTk);    // the next tile (clamped past the end) is in flight while this one is worked through
#pragma unroll 4
    for (int t = 0; t < kTk; t += 4) {
      const float4 xv = *(const float4*)&s_x[ch][t];
      const float4 gv = *(const float4*)&s_g[ch][t];
      const float4 kv = *(const float4*)&s_keep[t];
      const float xs[4] = {xv.x, xv.y, xv.z, xv.w}, ds[4] = {gv.x, gv.y, gv.z, gv.w}, ks[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // g[t] = q g[t-1] + s[t-1];  s[t] = q s[t-1] + x[t] (masked tokens enter as zero)
        const float ngr = fmaf(qr, gr, fmaf(-qi, gi, sr));
        const float ngi = fmaf(qr, gi, fmaf(qi, gr, si));
        const float nsr = fmaf(qr, sr, fmaf(-qi, si, xs[j] * ks[j]));
        const float nsi = fmaf(qr, si, qi * sr);
        gr = ngr; gi = ngi; sr = nsr; si = nsi;
        a2r = fmaf(ds[j], sr, a2r);
        a2i = fmaf(ds[j], si, a2i);
        a1r = fmaf(ds[j], gr, a1r);
        a1i = fmaf(ds[j], gi, a1i);
        ax = fmaf(ds[j], xs[j], ax);
      }
    }
  }
  if (state_lane) {
    float4* dst = (float4*)A.sums + ((size_t)b * A.D + c0 + ch) * A.N + n;
    *dst = make_float4(a2r, a2i, a1r, a1i);
    if (n == 0) A.dyx[(size_t)b * A.D + c0 + ch] = ax;
  }
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_ema_param_grad(const void* dy, const void* x, int dtype, int64_t sgb, int64_t sgd, int64_t sgl,
                                   int64_t sxb, int64_t sxd, int64_t sxl, const float* q, const uint8_t* mask,
                                   int64_t B, int64_t D, int64_t N, int64_t L, float* sums, float* dyx,
                                   void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "ema_param_grad: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && D > 0 && N > 0 && L >= 0, MEGA_ERR_ARG, "ema_param_grad: bad shape B=%ld D=%ld N=%ld L=%ld",
               (long)B, (long)D, (long)N, (long)L);
  MEGA_REQUIRE(N <= kNs, MEGA_ERR_UNSUPPORTED, "ema_param_grad: ndim=%ld > %d is not supported", (long)N, kNs);
  MEGA_REQUIRE(B * ceil_div(D, kCh) < (int64_t)1 << 31 && L < (int64_t)1 << 30, MEGA_ERR_UNSUPPORTED,
               "ema_param_grad: shape too large");
  if (B == 0) return MEGA_OK;
  MEGA_REQUIRE(q && sums && dyx && (L == 0 || (dy && x)), MEGA_ERR_ARG, "ema_param_grad: null pointer argument");
  if (L == 0) {
    hipMemsetAsync(sums, 0, (size_t)B * D * N * 16, (hipStream_t)stream);
    hipMemsetAsync(dyx, 0, (size_t)B * D * 4, (hipStream_t)stream);
    return MEGA_OK;
  }
  MEGA_REQUIRE(((uintptr_t)sums % 16) == 0, MEGA_ERR_ARG, "ema_param_grad: sums must be 16-byte aligned");
  EmaGradArgs A;
  A.dy = dy; A.x = x; A.sgb = sgb; A.sgd = sgd; A.sgl = sgl; A.sxb = sxb; A.sxd = sxd; A.sxl = sxl;
  A.q = q; A.mask = mask; A.sums = sums; A.dyx = dyx;
  A.B = (int)B; A.D = (int)D; A.N = (int)N; A.L = (int)L;
  const dim3 grid((unsigned)(B * ceil_div(D, kCh)));
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MEGA_F32: hipLaunchKernelGGL(ema_param_grad_kernel<float>, grid, dim3(kBwdThreads), 0, s, A); break;
    case MEGA_BF16: hipLaunchKernelGGL(ema_param_grad_kernel<bf16_t>, grid, dim3(kBwdThreads), 0, s, A); break;
    default: hipLaunchKernelGGL(ema_param_grad_kernel<f16_t>, grid, dim3(kBwdThreads), 0, s, A); break;
  }
  MEGA_CHECK_LAUNCH("ema_param_grad");
  return MEGA_OK;
}
