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
// Per batch row the kernel leaves sums [B, D, N, 4] = (Re sum2, Im sum2, Re sum1, Im sum1) and
// dyx [B, D] = sum_t dy x in the workspace; ema_grad_finalize_kernel adds the rows up in a fixed
// order and forms dp, dq, dgamma and domega.
#include <type_traits>

#include "common.h"

namespace mega {

// matrix-core form of the sums (ema_bwd_tile.hip)
bool ema_param_grad_tile_covers(int dtype, const void* dy, const void* x, int64_t sgb, int64_t sgd, int64_t sgl,
                                int64_t sxb, int64_t sxd, int64_t sxl, const uint8_t* mask, int64_t B, int64_t D,
                                int64_t N, int64_t L, int lag_one);
void ema_param_grad_tile_launch(const void* dy, const void* x, int64_t sgb, int64_t sgd, int64_t sgl, int64_t sxb,
                                int64_t sxd, int64_t sxl, const float* q, int64_t B, int64_t D, int64_t N, int64_t L,
                                float* sums, float* dyx, hipStream_t s);

namespace {

constexpr int kNs = 16;        // state lanes per channel
constexpr int kTk = 128;       // tokens per LDS tile


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
  int reverse;   // walk the tokens from the last to the first (the backward half of a two-sided layer)
};

// LAG1: the sums pair dy[t] with the state before token t (kernel lags start at 1: the backward
// half of a two-sided layer with shift).  A.reverse: x and dy arrive with negated token strides and
// pointers at the last token; only the mask needs the index turned round here.
// CH channels per workgroup (16, or 8 when 16 would leave compute units without a workgroup).
// ROLES = 2: a second set of CH * 16 threads shares the tiles; the first set runs s and the sum2
// pair, the second s, g and the sum1 pair.  That is 17 instead of 13 multiply-adds per token and
// state, but two waves per SIMD issue about 1.6 times faster than one wave alone, so it pays
// whenever the grid would otherwise leave every SIMD with a single wave.
template <typename T, bool MASKED, bool LAG1, int CH, int ROLES>
__global__ __launch_bounds__(CH * kNs * ROLES) void ema_param_grad_kernel(const EmaGradArgs A) {
  constexpr int kCh = CH;
  constexpr int kBwdThreads = CH * kNs * ROLES;
  constexpr int kPerThread = kTk / kNs / ROLES;   // elements of one tile a thread moves
  __shared__ float s_x[kCh][kTk + 4];
  __shared__ float s_g[kCh][kTk + 4];
  __shared__ float s_keep[kTk];
  const int tid = threadIdx.x;
  const int ncb = (A.D + kCh - 1) / kCh;
  const int b = blockIdx.x / ncb;
  const int c0 = (blockIdx.x - b * ncb) * kCh;
  const int role = tid / (CH * kNs);             // wave-uniform
  const int ch = (tid % (CH * kNs)) / kNs, n = tid % kNs;
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
  // per element: pointer at tile 0 and pointer of the row's last token (what a token past the end reads)
  const T* bx[kPerThread]; const T* lx[kPerThread];
  const T* bg[kPerThread]; const T* lg[kPerThread];
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    const int cx = min(ex[k] >> 16, dmax), cg = min(eg[k] >> 16, dmax);
    bx[k] = xg + (int64_t)(c0 + cx) * A.sxd + (int64_t)(ex[k] & 0xffff) * A.sxl;
    lx[k] = xg + (int64_t)(c0 + cx) * A.sxd + (int64_t)lmax * A.sxl;
    bg[k] = gg + (int64_t)(c0 + cg) * A.sgd + (int64_t)(eg[k] & 0xffff) * A.sgl;
    lg[k] = gg + (int64_t)(c0 + cg) * A.sgd + (int64_t)lmax * A.sgl;
  }
  auto fetch = [&](int t0) {
    const int64_t ox = (int64_t)t0 * A.sxl, og = (int64_t)t0 * A.sgl;
#pragma unroll
    for (int k = 0; k < kPerThread; ++k) {
      px[k] = to_float(*(t0 + (ex[k] & 0xffff) <= lmax ? bx[k] + ox : lx[k]));
      pg[k] = to_float(*(t0 + (eg[k] & 0xffff) <= lmax ? bg[k] + og : lg[k]));
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
    if (MASKED && tid < kTk) {
      const int tm = min(t0 + tid, lmax);
      s_keep[tid] = A.mask[(size_t)b * A.L + (A.reverse ? lmax - tm : tm)] ? 0.f : 1.f;
    }
    __syncthreads();
    fetch(t0 + kTk);    // the next tile (clamped past the end) is in flight while this one is worked through
    auto work = [&](auto do_a2, auto do_g) {
      constexpr bool A2 = decltype(do_a2)::value, G = decltype(do_g)::value;
#pragma unroll 4
      for (int t = 0; t < kTk; t += 4) {
        const float4 xv = *(const float4*)&s_x[ch][t];
        const float4 gv = *(const float4*)&s_g[ch][t];
        float4 kv = make_float4(1.f, 1.f, 1.f, 1.f);
        if (MASKED) kv = *(const float4*)&s_keep[t];
        const float xs[4] = {xv.x, xv.y, xv.z, xv.w}, ds[4] = {gv.x, gv.y, gv.z, gv.w}, ks[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // g[t] = q g[t-1] + s[t-1];  s[t] = q s[t-1] + x[t] (masked tokens enter as zero)
          float ngr = 0.f, ngi = 0.f;
          if (G) {
            ngr = fmaf(qr, gr, fmaf(-qi, gi, sr));
            ngi = fmaf(qr, gi, fmaf(qi, gr, si));
          }
          const float nsr = fmaf(qr, sr, fmaf(-qi, si, MASKED ? xs[j] * ks[j] : xs[j]));
          const float nsi = fmaf(qr, si, qi * sr);
          if (LAG1) {
            if (A2) { a2r = fmaf(ds[j], sr, a2r); a2i = fmaf(ds[j], si, a2i); }
            if (G) { a1r = fmaf(ds[j], gr, a1r); a1i = fmaf(ds[j], gi, a1i); }
          }
          gr = ngr; gi = ngi; sr = nsr; si = nsi;
          if (!LAG1) {
            if (A2) { a2r = fmaf(ds[j], sr, a2r); a2i = fmaf(ds[j], si, a2i); }
            if (G) { a1r = fmaf(ds[j], gr, a1r); a1i = fmaf(ds[j], gi, a1i); }
          }
          if (A2) ax = fmaf(ds[j], xs[j], ax);
        }
      }
    };
    using Yes = std::integral_constant<bool, true>;
    using No = std::integral_constant<bool, false>;
    if (ROLES == 1) work(Yes{}, Yes{});
    else if (role == 0) work(Yes{}, No{});
    else work(No{}, Yes{});
  }
  if (state_lane) {
    float2* dst = (float2*)A.sums + (((size_t)b * A.D + c0 + ch) * A.N + n) * 2;
    if (ROLES == 1 || role == 0) {
      dst[0] = make_float2(a2r, a2i);
      if (n == 0) A.dyx[(size_t)b * A.D + c0 + ch] = ax;
    }
    if (ROLES == 1 || role == 1) dst[1] = make_float2(a1r, a1i);
  }
}

// thread = (channel, state): rows summed in order, then the products of ema_parameters.cc:95-96
__global__ void ema_grad_finalize_kernel(const float* __restrict__ sums, const float* __restrict__ dyx,
                                         const float* __restrict__ p, const float* __restrict__ gamma, int B, int D,
                                         int N, float* __restrict__ dp, float* __restrict__ dq,
                                         float* __restrict__ dgamma, float* __restrict__ domega) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;   // over D * N
  if (i >= D * N) return;
  float s2r = 0.f, s2i = 0.f, s1r = 0.f, s1i = 0.f;
  for (int b = 0; b < B; ++b) {
    const float4 v = ((const float4*)sums)[(size_t)b * D * N + i];
    s2r += v.x; s2i += v.y; s1r += v.z; s1i += v.w;
  }
  const float pr = p[i], gr = gamma[2 * i], gi = gamma[2 * i + 1];
  dp[i] = s2r * gr - s2i * gi;                       // Re(sum2 gamma)
  dq[2 * i] = pr * (s1r * gr - s1i * gi);            // conj(sum1 p gamma)
  dq[2 * i + 1] = -pr * (s1r * gi + s1i * gr);
  dgamma[2 * i] = pr * s2r;                          // conj(sum2 p)
  dgamma[2 * i + 1] = -pr * s2i;
  if (i % N == 0) {
    const int d = i / N;
    float o = 0.f;
    for (int b = 0; b < B; ++b) o += dyx[(size_t)b * D + d];
    domega[d] = o;
  }
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" size_t mega_ema_param_grad_workspace_bytes(int64_t B, int64_t D, int64_t N) {
  if (B <= 0 || D <= 0 || N <= 0) return 256;
  return align_up((size_t)B * D * N * 16, 256) + align_up((size_t)B * D * 4, 256);
}

extern "C" int mega_ema_param_grad(const void* dy, const void* x, int dtype, int64_t sgb, int64_t sgd, int64_t sgl,
                                   int64_t sxb, int64_t sxd, int64_t sxl, const float* p, const float* q,
                                   const float* gamma, const uint8_t* mask, int64_t B, int64_t D, int64_t N,
                                   int64_t L, int reverse_time, int lag_one, float* dp, float* dq, float* dgamma,
                                   float* domega, void* workspace, size_t workspace_bytes, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "ema_param_grad: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && D > 0 && N > 0 && L >= 0, MEGA_ERR_ARG, "ema_param_grad: bad shape B=%ld D=%ld N=%ld L=%ld",
               (long)B, (long)D, (long)N, (long)L);
  MEGA_REQUIRE(N <= kNs, MEGA_ERR_UNSUPPORTED, "ema_param_grad: ndim=%ld > %d is not supported", (long)N, kNs);
  MEGA_REQUIRE(B * ceil_div(D, 8) < (int64_t)1 << 31 && L < (int64_t)1 << 30 && D * N < (int64_t)1 << 31,
               MEGA_ERR_UNSUPPORTED, "ema_param_grad: shape too large");
  MEGA_REQUIRE(p && q && gamma && dp && dq && dgamma && domega, MEGA_ERR_ARG, "ema_param_grad: null pointer argument");
  hipStream_t s = (hipStream_t)stream;
  if (B == 0 || L == 0) {
    zero_async(dp, (size_t)D * N * 4, s);
    zero_async(dq, (size_t)D * N * 8, s);
    zero_async(dgamma, (size_t)D * N * 8, s);
    zero_async(domega, (size_t)D * 4, s);
    return MEGA_OK;
  }
  MEGA_REQUIRE(dy && x, MEGA_ERR_ARG, "ema_param_grad: null dy / x");
  const size_t need = mega_ema_param_grad_workspace_bytes(B, D, N);
  MEGA_REQUIRE(workspace && workspace_bytes >= need && ((uintptr_t)workspace % 16) == 0, MEGA_ERR_WORKSPACE,
               "ema_param_grad: workspace of %zu bytes (16-byte aligned) needed", need);
  EmaGradArgs A;
  A.dy = dy; A.x = x; A.sgb = sgb; A.sgd = sgd; A.sgl = sgl; A.sxb = sxb; A.sxd = sxd; A.sxl = sxl;
  A.q = q; A.mask = mask; A.reverse = reverse_time ? 1 : 0;
  if (reverse_time) {
    const int64_t es = dtype == MEGA_F32 ? 4 : 2;
    A.dy = (const char*)dy + (L - 1) * sgl * es;
    A.x = (const char*)x + (L - 1) * sxl * es;
    A.sgl = -sgl;
    A.sxl = -sxl;
  }
  A.sums = (float*)workspace;
  A.dyx = (float*)((char*)workspace + align_up((size_t)B * D * N * 16, 256));
  A.B = (int)B; A.D = (int)D; A.N = (int)N; A.L = (int)L;
  if (audit_on()) {
    // both forms of the kernel leave (b, channel, state) -> 4 floats and (b, channel) -> 1 float; the activations are
    // addressed from the first token of the walk to the last (the walk may run backwards in memory)
    const int64_t es = dtype == MEGA_F32 ? 4 : 2;
    audit_use(A.sums, (size_t)B * D * N * 16, "ema_param_grad: sums");
    audit_use(A.dyx, (size_t)B * D * 4, "ema_param_grad: dy x");
    const int64_t hi_g = (B - 1) * sgb + (D - 1) * sgd + (L - 1) * sgl, hi_x = (B - 1) * sxb + (D - 1) * sxd + (L - 1) * sxl;
    audit_use(dy, (size_t)(hi_g + 1) * es, "ema_param_grad: dy");
    audit_use(x, (size_t)(hi_x + 1) * es, "ema_param_grad: x");
    audit_use(dp, (size_t)D * N * 4, "ema_param_grad: dp");
    audit_use(dq, (size_t)D * N * 8, "ema_param_grad: dq");
    audit_use(dgamma, (size_t)D * N * 8, "ema_param_grad: dgamma");
    audit_use(domega, (size_t)D * 4, "ema_param_grad: domega");
    return MEGA_OK;
  }
  if (ema_param_grad_tile_covers(dtype, A.dy, A.x, A.sgb, A.sgd, A.sgl, A.sxb, A.sxd, A.sxl, mask, B, D, N, L,
                                 lag_one)) {
    ema_param_grad_tile_launch(A.dy, A.x, A.sgb, A.sgd, A.sgl, A.sxb, A.sxd, A.sxl, q, B, D, N, L, A.sums, A.dyx, s);
    MEGA_CHECK_LAUNCH("ema_param_grad (matrix-core form)");
    hipLaunchKernelGGL(ema_grad_finalize_kernel, dim3((unsigned)ceil_div(D * N, 256)), dim3(256), 0, s, A.sums, A.dyx,
                       p, gamma, (int)B, (int)D, (int)N, dp, dq, dgamma, domega);
    MEGA_CHECK_LAUNCH("ema_param_grad (finalize)");
    return MEGA_OK;
  }
  // 16 channels per workgroup, 8 when that would leave compute units idle
  const int cus = device_cu_count();
  // one role set per workgroup only when the grid fills every SIMD with several waves anyway
  const bool narrow = B * ceil_div(D, 16) < cus;
  const int ch = narrow ? 8 : 16;
  const int64_t wgs = B * ceil_div(D, ch);
  const bool split = wgs * (ch * kNs / 64) <= (int64_t)cus * 4;     // at most one wave per SIMD without it
  const dim3 grid((unsigned)wgs);
#define LAUNCH_PG(T)                                                                                          \
  do {                                                                                                        \
    typedef void (*Kern)(const EmaGradArgs);                                                                 \
    static const Kern table[16] = {                                                                           \
        ema_param_grad_kernel<T, false, false, 16, 1>, ema_param_grad_kernel<T, false, true, 16, 1>,          \
        ema_param_grad_kernel<T, true, false, 16, 1>,  ema_param_grad_kernel<T, true, true, 16, 1>,           \
        ema_param_grad_kernel<T, false, false, 8, 1>,  ema_param_grad_kernel<T, false, true, 8, 1>,           \
        ema_param_grad_kernel<T, true, false, 8, 1>,   ema_param_grad_kernel<T, true, true, 8, 1>,            \
        ema_param_grad_kernel<T, false, false, 16, 2>, ema_param_grad_kernel<T, false, true, 16, 2>,          \
        ema_param_grad_kernel<T, true, false, 16, 2>,  ema_param_grad_kernel<T, true, true, 16, 2>,           \
        ema_param_grad_kernel<T, false, false, 8, 2>,  ema_param_grad_kernel<T, false, true, 8, 2>,           \
        ema_param_grad_kernel<T, true, false, 8, 2>,   ema_param_grad_kernel<T, true, true, 8, 2>};           \
    hipLaunchKernelGGL(table[(split ? 8 : 0) + (narrow ? 4 : 0) + (mask ? 2 : 0) + (lag_one ? 1 : 0)], grid,  \
                       dim3(ch * kNs * (split ? 2 : 1)), 0, s, A);                                            \
  } while (0)
  switch (dtype) {
    case MEGA_F32: LAUNCH_PG(float); break;
    case MEGA_BF16: LAUNCH_PG(bf16_t); break;
    default: LAUNCH_PG(f16_t); break;
  }
#undef LAUNCH_PG
  MEGA_CHECK_LAUNCH("ema_param_grad");
  hipLaunchKernelGGL(ema_grad_finalize_kernel, dim3((unsigned)ceil_div(D * N, 256)), dim3(256), 0, s, A.sums, A.dyx, p,
                     gamma, (int)B, (int)D, (int)N, dp, dq, dgamma, domega);
  MEGA_CHECK_LAUNCH("ema_param_grad (finalize)");
  return MEGA_OK;
}
