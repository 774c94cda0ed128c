// One decode step of the norm -> moving-average pair: streaming TimestepNorm of one token
// (fairseq/modules/norm_layer/timestep_norm.py:100-139 with L = 1: the WelfordCombine of
// fairseq/csrc/utils.h:66-76 on the carried (count, mean, var)) followed by the single-step state
// update h' = q h + p xn, y = Re sum gamma h' + omega xn
// (fairseq/modules/base_moving_average.py:105-118, 144-160).  One launch per step; a workgroup
// owns one (stream, group): it reads its slice of x once, the state h once, and writes both back.
// Traffic per step is the state: 2 * B * D * N * 8 bytes.
#include "common.h"

namespace mega {
namespace {

constexpr int kT = 128;

struct StepArgs {
  const void* x;
  void* xn;
  void* y;
  const int64_t* prev_count;
  const float* prev_mean;
  const float* prev_var;
  int64_t* count;
  float* mean;
  float* var;
  const float* nw;       // gamma of the norm (weight + 1)
  const float* nb;
  const float* p;        // [D, N]
  const float* q;        // [D, N, 2]
  const float* g;        // [D, N, 2]
  const float* omega;    // [D]
  const float* h_in;     // [B, D, N, 2] or null
  float* h_out;
  int B, D, G, N;
  int K;                 // tokens per stream in this launch (the multi-token kernel)
  int MB;                // tokens per batch staged in LDS
  float eps;
};

__device__ __forceinline__ float block_sum(float v, float* red) {
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < kT / 64; ++i) t += red[i];
  return t;
}

template <typename T, bool CPLX>
__global__ __launch_bounds__(kT) void norm_ema_step_kernel(const StepArgs A) {
  __shared__ float red[kT / 64];
  const int g = blockIdx.x % A.G, b = blockIdx.x / A.G;
  const int dg = A.D / A.G;
  const T* xr = (const T*)A.x + (size_t)b * A.D + (size_t)g * dg;
  // moments of this token's group
  float s = 0.f;
  for (int f = threadIdx.x; f < dg; f += kT) s += to_float(xr[f]);
  const float gm = block_sum(s, red) / (float)dg;
  float s2 = 0.f;
  for (int f = threadIdx.x; f < dg; f += kT) {
    const float d = to_float(xr[f]) - gm;
    s2 += d * d;
  }
  const float gv = block_sum(s2, red) / (float)dg;
  // fold into the carried state (one step of weight 1)
  const int64_t c0 = A.prev_count[b];
  const float u0 = A.prev_mean[(size_t)b * A.G + g], v0 = A.prev_var[(size_t)b * A.G + g];
  const float c1 = (float)c0 / (float)(c0 + 1), c2 = 1.0f / (float)(c0 + 1);
  const float dl = gm - u0;
  const float u1 = c1 * u0 + c2 * gm;
  const float v1 = c1 * v0 + c2 * gv + (c1 * dl) * (c2 * dl);
  const float rstd = 1.0f / sqrtf(v1 + A.eps);
  __syncthreads();                               // every thread has read the old state
  if (threadIdx.x == 0) {
    A.mean[(size_t)b * A.G + g] = u1;
    A.var[(size_t)b * A.G + g] = v1;
    if (g == 0) A.count[b] = c0 + 1;
  }
  for (int f = threadIdx.x; f < dg; f += kT) {
    const int d = g * dg + f;
    const size_t o = (size_t)b * A.D + d;
    const float xnv_full = (to_float(xr[f]) - u1) * rstd * A.nw[d] + A.nb[d];
    const T xn_t = from_float<T>(xnv_full);
    ((T*)A.xn)[o] = xn_t;
    const float xv = to_float(xn_t);             // the moving average sees the rounded activation
    float acc = 0.f;
    const size_t ho = o * A.N * 2;
    const size_t co = (size_t)d * A.N;
    for (int n = 0; n < A.N; ++n) {
      const float qr = A.q[(co + n) * 2], qi = CPLX ? A.q[(co + n) * 2 + 1] : 0.f;
      const float gr = A.g[(co + n) * 2], gi = CPLX ? A.g[(co + n) * 2 + 1] : 0.f;
      float hr = 0.f, hi = 0.f;
      if (A.h_in) {
        hr = A.h_in[ho + 2 * n];
        hi = CPLX ? A.h_in[ho + 2 * n + 1] : 0.f;
      }
      const float nr = qr * hr - qi * hi + A.p[co + n] * xv;
      const float ni = qr * hi + qi * hr;
      A.h_out[ho + 2 * n] = nr;
      A.h_out[ho + 2 * n + 1] = ni;
      acc += gr * nr - gi * ni;
    }
    ((T*)A.y)[o] = from_float<T>(acc + A.omega[d] * xv);
  }
}

// Same step with the state streamed as 32-byte pieces: NP = N / 4 adjacent lanes own one channel,
// each lane four states (two 16-byte loads of h, q, gamma, one of p), so a wave reads and writes
// the state as one contiguous 2 KB block; the output sum is finished across the NP lanes.
constexpr int kTV = 256;

template <typename T, int NP>
__global__ __launch_bounds__(kTV) void norm_ema_step_vec_kernel(const StepArgs A) {
  __shared__ float red[kTV / 64];
  const int g = blockIdx.x % A.G, b = blockIdx.x / A.G;
  const int dg = A.D / A.G;
  const T* xr = (const T*)A.x + (size_t)b * A.D + (size_t)g * dg;
  const int64_t c0 = A.prev_count[b];
  const float u0 = A.prev_mean[(size_t)b * A.G + g], v0 = A.prev_var[(size_t)b * A.G + g];
  auto wg_sum = [&](float v) {
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < kTV / 64; ++i) t += red[i];
    return t;
  };
  float s = 0.f;
  for (int f = threadIdx.x; f < dg; f += kTV) s += to_float(xr[f]);
  const float gm = wg_sum(s) / (float)dg;
  float s2 = 0.f;
  for (int f = threadIdx.x; f < dg; f += kTV) {
    const float d = to_float(xr[f]) - gm;
    s2 += d * d;
  }
  const float gv = wg_sum(s2) / (float)dg;
  const float c1 = (float)c0 / (float)(c0 + 1), c2 = 1.0f / (float)(c0 + 1);
  const float dl = gm - u0;
  const float u1 = c1 * u0 + c2 * gm;
  const float v1 = c1 * v0 + c2 * gv + (c1 * dl) * (c2 * dl);
  const float rstd = 1.0f / sqrtf(v1 + A.eps);
  __syncthreads();                               // every thread has read the old state
  if (threadIdx.x == 0) {
    A.mean[(size_t)b * A.G + g] = u1;
    A.var[(size_t)b * A.G + g] = v1;
    if (g == 0) A.count[b] = c0 + 1;
  }
  const int items = dg * NP;                     // a multiple of NP, so the lanes of a channel stay together
  for (int it0 = 0; it0 < items; it0 += kTV) {
    const int it = it0 + threadIdx.x;
    const bool ok = it < items;
    const int f = ok ? it / NP : 0, part = it % NP;
    const int d = g * dg + f;
    const size_t o = (size_t)b * A.D + d;
    const float xnv_full = (to_float(xr[f]) - u1) * rstd * A.nw[d] + A.nb[d];
    const T xn_t = from_float<T>(xnv_full);
    const float xv = to_float(xn_t);             // the moving average sees the rounded activation
    const size_t ho = (o * A.N + 4 * part) * 2;
    const size_t co = (size_t)d * A.N + 4 * part;
    float4 h0 = make_float4(0.f, 0.f, 0.f, 0.f), h1 = h0;
    if (A.h_in) {
      h0 = *(const float4*)(A.h_in + ho);
      h1 = *(const float4*)(A.h_in + ho + 4);
    }
    const float4 q0 = *(const float4*)(A.q + co * 2), q1 = *(const float4*)(A.q + co * 2 + 4);
    const float4 g0 = *(const float4*)(A.g + co * 2), g1 = *(const float4*)(A.g + co * 2 + 4);
    const float4 pp = *(const float4*)(A.p + co);
    float4 n0, n1;
    n0.x = q0.x * h0.x - q0.y * h0.y + pp.x * xv;  n0.y = q0.x * h0.y + q0.y * h0.x;
    n0.z = q0.z * h0.z - q0.w * h0.w + pp.y * xv;  n0.w = q0.z * h0.w + q0.w * h0.z;
    n1.x = q1.x * h1.x - q1.y * h1.y + pp.z * xv;  n1.y = q1.x * h1.y + q1.y * h1.x;
    n1.z = q1.z * h1.z - q1.w * h1.w + pp.w * xv;  n1.w = q1.z * h1.w + q1.w * h1.z;
    float acc = (g0.x * n0.x - g0.y * n0.y) + (g0.z * n0.z - g0.w * n0.w) + (g1.x * n1.x - g1.y * n1.y) +
                (g1.z * n1.z - g1.w * n1.w);
#pragma unroll
    for (int m = 1; m < NP; m <<= 1) acc += __shfl_xor(acc, m);
    if (ok) {
      *(float4*)(A.h_out + ho) = n0;
      *(float4*)(A.h_out + ho + 4) = n1;
      if (part == 0) {
        ((T*)A.xn)[o] = xn_t;
        ((T*)A.y)[o] = from_float<T>(acc + A.omega[d] * xv);
      }
    }
  }
}

// K consecutive tokens of every stream in one launch: x, xn, y are [B, K, D].  The state h of a channel stays in
// registers over the K tokens (read once, written once per launch instead of once per token), the norm
// statistics of the (stream, group) advance token by token exactly as K single steps would advance them.
// Tokens are taken in batches of A.MB that fit in LDS: the group's slice of the batch is staged there with its
// moments (one wave per token, no workgroup barrier per token), every thread then walks the batch for its
// channels out of LDS (no global access inside the token loop), and xn, y leave as whole rows.
constexpr int kStepsLdsBytes = 32 * 1024;     // per workgroup, so that four of them share a CU
constexpr int kStepsIT = 2;                     // channels-parts a thread advances side by side

struct StepMoments {
  float n, mean, var;
};
// Welford merge of two runs (fairseq/csrc/utils.h:66-76 for general weights)
__device__ __forceinline__ StepMoments step_merge(StepMoments a, StepMoments b) {
  const float n = a.n + b.n;
  const float rn = n > 0.f ? 1.0f / n : 0.f;
  const float ca = a.n * rn, cb = b.n * rn;
  const float d = b.mean - a.mean;
  return StepMoments{n, a.mean + cb * d, ca * a.var + cb * b.var + (ca * d) * (cb * d)};
}

template <typename T, int NP>
__global__ __launch_bounds__(kTV) void norm_ema_steps_kernel(const StepArgs A) {
  extern __shared__ float s_dyn[];
  const int dg = A.D / A.G;
  const int MB = A.MB;                           // <= 64
  float* s_mu = s_dyn;                           // [MB] group mean of the token, then running mean
  float* s_rs = s_mu + MB;                       // [MB] group variance, then running 1 / sqrt(var + eps)
  float* s_x = s_rs + MB;                        // [MB][dg] x, then xn (as rounded to T)
  float* s_y = s_x + (size_t)MB * dg;            // [MB][dg] y
  const int g = blockIdx.x % A.G, b = blockIdx.x / A.G;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* xb = (const T*)A.x + (size_t)b * A.K * A.D + (size_t)g * dg;
  T* xnb = (T*)A.xn + (size_t)b * A.K * A.D + (size_t)g * dg;
  T* yb = (T*)A.y + (size_t)b * A.K * A.D + (size_t)g * dg;
  const int64_t c_in = A.prev_count[b];
  // the statistics carried into the current batch (every thread keeps a copy)
  StepMoments carry = {(float)c_in, A.prev_mean[(size_t)b * A.G + g], A.prev_var[(size_t)b * A.G + g]};
  const float inv_dg = 1.0f / (float)dg;
  const int items = dg * NP;                     // a multiple of NP, so the lanes of a channel stay together
  for (int k0 = 0; k0 < A.K; k0 += MB) {
    const int nk = min(MB, A.K - k0);
    __syncthreads();                             // the previous batch has left LDS
    for (int k = wave; k < nk; k += kTV / 64) {
      const T* xr = xb + (size_t)(k0 + k) * A.D;
      float* sx = s_x + (size_t)k * dg;
      float s = 0.f;
      for (int f = lane; f < dg; f += 64) {
        const float xv = to_float(xr[f]);
        sx[f] = xv;
        s += xv;
      }
      for (int m = 32; m >= 1; m >>= 1) s += __shfl_xor(s, m);
      const float gm = s * inv_dg;
      float s2 = 0.f;
      for (int f = lane; f < dg; f += 64) {
        const float d = sx[f] - gm;              // this lane's own stores
        s2 += d * d;
      }
      for (int m = 32; m >= 1; m >>= 1) s2 += __shfl_xor(s2, m);
      if (lane == 0) {
        s_mu[k] = gm;
        s_rs[k] = s2 * inv_dg;
      }
    }
    __syncthreads();
    // running statistics after every token of the batch: an inclusive scan of Welford merges over the tokens
    // (lane = token), every wave for itself; the same merge tree for every wave, so all threads agree
    StepMoments m = {0.f, 0.f, 0.f};
    if (lane < nk) m = StepMoments{1.f, s_mu[lane], s_rs[lane]};
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const StepMoments p = {__shfl_up(m.n, o), __shfl_up(m.mean, o), __shfl_up(m.var, o)};
      if (lane >= o) m = step_merge(p, m);
    }
    const StepMoments run = step_merge(carry, m);
    __syncthreads();                             // every wave has read the group moments
    if (wave == 0 && lane < nk) {
      s_mu[lane] = run.mean;
      s_rs[lane] = 1.0f / sqrtf(run.var + A.eps);
    }
    {
      const StepMoments last = {__shfl(run.n, nk - 1), __shfl(run.mean, nk - 1), __shfl(run.var, nk - 1)};
      carry = last;
    }
    __syncthreads();
    for (int it0 = 0; it0 < items; it0 += kTV * kStepsIT) {
      bool ok[kStepsIT];
      int f[kStepsIT], part[kStepsIT];
      size_t ho[kStepsIT];
      float4 h0[kStepsIT], h1[kStepsIT], q0[kStepsIT], q1[kStepsIT], g0[kStepsIT], g1[kStepsIT], pp[kStepsIT];
      float nw[kStepsIT], nb[kStepsIT], om[kStepsIT];
      const float* hsrc = k0 == 0 ? A.h_in : A.h_out;          // later batches continue from what this thread wrote
#pragma unroll
      for (int i = 0; i < kStepsIT; ++i) {
        const int it = it0 + i * kTV + threadIdx.x;
        ok[i] = it < items;
        f[i] = ok[i] ? it / NP : 0;
        part[i] = it % NP;
        const int d = g * dg + f[i];
        ho[i] = (((size_t)b * A.D + d) * A.N + 4 * part[i]) * 2;
        const size_t co = (size_t)d * A.N + 4 * part[i];
        h0[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        h1[i] = h0[i];
        if (hsrc) {
          h0[i] = *(const float4*)(hsrc + ho[i]);
          h1[i] = *(const float4*)(hsrc + ho[i] + 4);
        }
        q0[i] = *(const float4*)(A.q + co * 2);
        q1[i] = *(const float4*)(A.q + co * 2 + 4);
        g0[i] = *(const float4*)(A.g + co * 2);
        g1[i] = *(const float4*)(A.g + co * 2 + 4);
        pp[i] = *(const float4*)(A.p + co);
        nw[i] = A.nw[d];
        nb[i] = A.nb[d];
        om[i] = A.omega[d];
      }
      for (int k = 0; k < nk; ++k) {
        const float mu = s_mu[k], rs = s_rs[k];
#pragma unroll
        for (int i = 0; i < kStepsIT; ++i) {
          float* sx = s_x + (size_t)k * dg + f[i];
          const T xn_t = from_float<T>((*sx - mu) * rs * nw[i] + nb[i]);
          const float xv = to_float(xn_t);         // the moving average sees the rounded activation
          float4 n0, n1;
          n0.x = q0[i].x * h0[i].x - q0[i].y * h0[i].y + pp[i].x * xv;  n0.y = q0[i].x * h0[i].y + q0[i].y * h0[i].x;
          n0.z = q0[i].z * h0[i].z - q0[i].w * h0[i].w + pp[i].y * xv;  n0.w = q0[i].z * h0[i].w + q0[i].w * h0[i].z;
          n1.x = q1[i].x * h1[i].x - q1[i].y * h1[i].y + pp[i].z * xv;  n1.y = q1[i].x * h1[i].y + q1[i].y * h1[i].x;
          n1.z = q1[i].z * h1[i].z - q1[i].w * h1[i].w + pp[i].w * xv;  n1.w = q1[i].z * h1[i].w + q1[i].w * h1[i].z;
          h0[i] = n0;
          h1[i] = n1;
          float acc = (g0[i].x * n0.x - g0[i].y * n0.y) + (g0[i].z * n0.z - g0[i].w * n0.w) +
                      (g1[i].x * n1.x - g1[i].y * n1.y) + (g1[i].z * n1.z - g1[i].w * n1.w);
#pragma unroll
          for (int mm = 1; mm < NP; mm <<= 1) acc += __shfl_xor(acc, mm);
          if (ok[i] && part[i] == 0) {             // the NP lanes of the channel have read *sx (same wave)
            *sx = xv;
            s_y[(size_t)k * dg + f[i]] = acc + om[i] * xv;
          }
        }
      }
#pragma unroll
      for (int i = 0; i < kStepsIT; ++i) {
        if (ok[i]) {
          *(float4*)(A.h_out + ho[i]) = h0[i];
          *(float4*)(A.h_out + ho[i] + 4) = h1[i];
        }
      }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nk * dg; i += kTV) {
      const int k = i / dg, f = i - k * dg;
      const size_t o = (size_t)(k0 + k) * A.D + f;
      xnb[o] = from_float<T>(s_x[i]);              // exact: the value was rounded to T before it was stored
      yb[o] = from_float<T>(s_y[i]);
    }
  }
  if (threadIdx.x == 0) {
    A.mean[(size_t)b * A.G + g] = carry.mean;
    A.var[(size_t)b * A.G + g] = carry.var;
    if (g == 0) A.count[b] = c_in + (int64_t)A.K;
  }
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_norm_ema_step(const void* x, void* xn, void* y, int dtype, const int64_t* prev_count,
                                  const float* prev_mean, const float* prev_var, int64_t* count, float* mean,
                                  float* var, const float* norm_gamma, const float* norm_beta, double eps,
                                  const float* p, const float* q, const float* gamma, int is_complex,
                                  const float* omega, const float* h_in, float* h_out, int64_t B, int64_t D,
                                  int64_t G, int64_t N, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "norm_ema_step: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && D > 0 && G > 0 && N > 0 && D % G == 0, MEGA_ERR_ARG,
               "norm_ema_step: bad shape B=%ld D=%ld G=%ld N=%ld", (long)B, (long)D, (long)G, (long)N);
  MEGA_REQUIRE(N <= 32, MEGA_ERR_UNSUPPORTED, "norm_ema_step: ndim=%ld > 32 is not supported", (long)N);
  MEGA_REQUIRE(B * G < (int64_t)1 << 31, MEGA_ERR_UNSUPPORTED, "norm_ema_step: too many streams");
  if (B == 0) return MEGA_OK;
  MEGA_REQUIRE(x && xn && y && prev_count && prev_mean && prev_var && count && mean && var && norm_gamma && norm_beta &&
                   p && q && gamma && omega && h_out,
               MEGA_ERR_ARG, "norm_ema_step: null pointer argument");
  // Every workgroup (stream, group) of a launch reads prev_count[stream] and the workgroup of group 0 writes
  // count[stream]: with the two in one buffer a late workgroup could read the count of the step being
  // written.  mean / var words and the state h have one owning workgroup each, so those may be updated in place.
  MEGA_REQUIRE(!ranges_overlap(prev_count, (size_t)B * 8, count, (size_t)B * 8), MEGA_ERR_ARG,
               "norm_ema_step: count must not overlap prev_count (every group of a stream reads prev_count "
               "while one of them writes count); alternate between two count buffers");
  StepArgs A;
  A.x = x; A.xn = xn; A.y = y; A.prev_count = prev_count; A.prev_mean = prev_mean; A.prev_var = prev_var;
  A.count = count; A.mean = mean; A.var = var; A.nw = norm_gamma; A.nb = norm_beta; A.p = p; A.q = q; A.g = gamma;
  A.omega = omega; A.h_in = h_in; A.h_out = h_out; A.B = (int)B; A.D = (int)D; A.G = (int)G; A.N = (int)N;
  A.K = 1;
  A.eps = (float)eps;
  const dim3 grid((unsigned)(B * G));
  hipStream_t s = (hipStream_t)stream;
  // vector path: complex coefficient storage (always), 4 | N, N / 4 a power of two, aligned pointers
  const int np = (int)(N / 4);
  if (is_complex && N % 4 == 0 && (np & (np - 1)) == 0 && ((uintptr_t)h_out % 16) == 0 && (!h_in || ((uintptr_t)h_in % 16) == 0) &&
      ((uintptr_t)q % 16) == 0 && ((uintptr_t)gamma % 16) == 0 && ((uintptr_t)p % 16) == 0) {
#define LAUNCH_NV(T)                                                                                     \
  switch (np) {                                                                                          \
    case 1: hipLaunchKernelGGL((norm_ema_step_vec_kernel<T, 1>), grid, dim3(kTV), 0, s, A); break;       \
    case 2: hipLaunchKernelGGL((norm_ema_step_vec_kernel<T, 2>), grid, dim3(kTV), 0, s, A); break;       \
    case 4: hipLaunchKernelGGL((norm_ema_step_vec_kernel<T, 4>), grid, dim3(kTV), 0, s, A); break;       \
    default: hipLaunchKernelGGL((norm_ema_step_vec_kernel<T, 8>), grid, dim3(kTV), 0, s, A); break;      \
  }
    if (dtype == MEGA_F32) { LAUNCH_NV(float) }
    else if (dtype == MEGA_BF16) { LAUNCH_NV(bf16_t) }
    else { LAUNCH_NV(f16_t) }
#undef LAUNCH_NV
    MEGA_CHECK_LAUNCH("norm_ema_step");
    return MEGA_OK;
  }
#define LAUNCH_NS(T, C) hipLaunchKernelGGL((norm_ema_step_kernel<T, C>), grid, dim3(kT), 0, s, A)
  if (is_complex) {
    if (dtype == MEGA_F32) LAUNCH_NS(float, true);
    else if (dtype == MEGA_BF16) LAUNCH_NS(bf16_t, true);
    else LAUNCH_NS(f16_t, true);
  } else {
    if (dtype == MEGA_F32) LAUNCH_NS(float, false);
    else if (dtype == MEGA_BF16) LAUNCH_NS(bf16_t, false);
    else LAUNCH_NS(f16_t, false);
  }
#undef LAUNCH_NS
  MEGA_CHECK_LAUNCH("norm_ema_step");
  return MEGA_OK;
}

extern "C" int mega_norm_ema_steps(const void* x, void* xn, void* y, int dtype, int64_t K, const int64_t* prev_count,
                                   const float* prev_mean, const float* prev_var, int64_t* count, float* mean,
                                   float* var, const float* norm_gamma, const float* norm_beta, double eps,
                                   const float* p, const float* q, const float* gamma, int is_complex,
                                   const float* omega, const float* h_in, float* h_out, int64_t B, int64_t D,
                                   int64_t G, int64_t N, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "norm_ema_steps: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && K >= 0 && D > 0 && G > 0 && N > 0 && D % G == 0, MEGA_ERR_ARG,
               "norm_ema_steps: bad shape B=%ld K=%ld D=%ld G=%ld N=%ld", (long)B, (long)K, (long)D, (long)G, (long)N);
  MEGA_REQUIRE(B * G < (int64_t)1 << 31 && K < (int64_t)1 << 24 && B * K * D < (int64_t)1 << 40, MEGA_ERR_UNSUPPORTED,
               "norm_ema_steps: shape too large");
  const int np = (int)(N / 4);
  MEGA_REQUIRE(is_complex && N % 4 == 0 && N <= 32 && (np & (np - 1)) == 0, MEGA_ERR_UNSUPPORTED,
               "norm_ema_steps: complex coefficient storage with ndim in {4, 8, 16, 32} only (ndim=%ld, is_complex=%d); "
               "call mega_norm_ema_step once per token",
               (long)N, is_complex);
  if (B == 0 || K == 0) return MEGA_OK;
  MEGA_REQUIRE(x && xn && y && prev_count && prev_mean && prev_var && count && mean && var && norm_gamma && norm_beta &&
                   p && q && gamma && omega && h_out,
               MEGA_ERR_ARG, "norm_ema_steps: null pointer argument");
  MEGA_REQUIRE(((uintptr_t)h_out % 16) == 0 && (!h_in || ((uintptr_t)h_in % 16) == 0) && ((uintptr_t)q % 16) == 0 &&
                   ((uintptr_t)gamma % 16) == 0 && ((uintptr_t)p % 16) == 0,
               MEGA_ERR_ARG, "norm_ema_steps: h, p, q, gamma must be 16-byte aligned");
  MEGA_REQUIRE(!ranges_overlap(prev_count, (size_t)B * 8, count, (size_t)B * 8), MEGA_ERR_ARG,
               "norm_ema_steps: count must not overlap prev_count (every group of a stream reads prev_count "
               "while one of them writes count); alternate between two count buffers");
  StepArgs A;
  A.x = x; A.xn = xn; A.y = y; A.prev_count = prev_count; A.prev_mean = prev_mean; A.prev_var = prev_var;
  A.count = count; A.mean = mean; A.var = var; A.nw = norm_gamma; A.nb = norm_beta; A.p = p; A.q = q; A.g = gamma;
  A.omega = omega; A.h_in = h_in; A.h_out = h_out; A.B = (int)B; A.D = (int)D; A.G = (int)G; A.N = (int)N;
  A.K = (int)K;
  A.eps = (float)eps;
  // tokens per batch: what fits in LDS beside the moments (x / xn and y of the group's slice as fp32)
  const int64_t dg = D / G;
  int64_t mb = (kStepsLdsBytes - 0) / (dg * 8 + 8);
  MEGA_REQUIRE(mb >= 1, MEGA_ERR_UNSUPPORTED, "norm_ema_steps: %ld channels per group do not fit in LDS", (long)dg);
  if (mb > 64) mb = 64;
  if (mb > K) mb = K;
  A.MB = (int)mb;
  const size_t smem = (size_t)mb * (dg * 8 + 8);
  const dim3 grid((unsigned)(B * G));
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH_NK(T)                                                                                  \
  switch (np) {                                                                                       \
    case 1: hipLaunchKernelGGL((norm_ema_steps_kernel<T, 1>), grid, dim3(kTV), smem, s, A); break;       \
    case 2: hipLaunchKernelGGL((norm_ema_steps_kernel<T, 2>), grid, dim3(kTV), smem, s, A); break;       \
    case 4: hipLaunchKernelGGL((norm_ema_steps_kernel<T, 4>), grid, dim3(kTV), smem, s, A); break;       \
    default: hipLaunchKernelGGL((norm_ema_steps_kernel<T, 8>), grid, dim3(kTV), smem, s, A); break;      \
  }
  if (dtype == MEGA_F32) { LAUNCH_NK(float) }
  else if (dtype == MEGA_BF16) { LAUNCH_NK(bf16_t) }
  else { LAUNCH_NK(f16_t) }
#undef LAUNCH_NK
  MEGA_CHECK_LAUNCH("norm_ema_steps");
  return MEGA_OK;
}
