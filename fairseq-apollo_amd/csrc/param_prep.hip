// The small per-parameter formulas in front of the kernels, one launch each way instead of a chain of
// element-wise launches per formula step:
//   moving-average coefficients from the stored parameters
//     (fairseq/modules/complex_exponential_moving_average.py:79-96, exponential_moving_average.py:71-80) and
//   the TimestepNorm operands (weight + 1, bias, the prior mean and exp(prior log-variance) expanded over the
//     batch; fairseq/modules/norm_layer/timestep_norm.py:118-131),
// each with its backward pass.  Parameters are read in their storage type (fp32, bf16, fp16) and their gradients
// written in it; everything the other kernels consume is fp32.
#include "common.h"

namespace mega {
namespace {

__device__ __forceinline__ float ld(const void* p, int dtype, int64_t i) {
  if (dtype == MEGA_F32) return ((const float*)p)[i];
  if (dtype == MEGA_BF16) return to_float(((const bf16_t*)p)[i]);
  return to_float(((const f16_t*)p)[i]);
}
__device__ __forceinline__ void st(void* p, int dtype, int64_t i, float v) {
  if (dtype == MEGA_F32) ((float*)p)[i] = v;
  else if (dtype == MEGA_BF16) ((bf16_t*)p)[i] = from_float<bf16_t>(v);
  else ((f16_t*)p)[i] = from_float<f16_t>(v);
}
__device__ __forceinline__ float sigm(float x) { return 1.0f / (1.0f + expf(-x)); }

struct CoeffArgs {
  const void* alpha;   // [K, N]
  const void* delta;   // [K, N]
  const void* third;   // complex: theta [K]; real: beta [K, N]
  const void* gamma;   // complex: [K, N, 2]; real: [K, N]
  const void* omega;   // [D]
  int dtype, is_complex, K, N, D;
  float scale, turn;   // sqrt(1 / N), 2 pi / N
  // forward results (fp32, the layout every kernel of the library takes)
  float* p;            // [K, N]
  float* q;            // [K, N, 2]
  float* g;            // [K, N, 2]
  float* om;           // [D]
  // backward: gradients of the forward results in, gradients of the parameters out (storage type)
  const float* dp;
  const float* dq;
  const float* dg;
  const float* dom;
  void* dalpha;
  void* ddelta;
  void* dthird;
  void* dgamma;
  void* domega;
};

// one thread per (row, state)
__global__ __launch_bounds__(256) void ema_coeffs_fwd_kernel(const CoeffArgs A) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < A.D) A.om[i] = ld(A.omega, A.dtype, i);
  if (i >= (int64_t)A.K * A.N) return;
  const int k = (int)(i / A.N), n = (int)(i - (int64_t)k * A.N);
  const float a = sigm(ld(A.alpha, A.dtype, i)), d = sigm(ld(A.delta, A.dtype, i));
  const float r = 1.0f - a * d;
  if (A.is_complex) {
    const float ang = (float)(n + 1) * (sigm(ld(A.third, A.dtype, k)) * A.turn);
    float sn, cs;
    sincosf(ang, &sn, &cs);
    A.p[i] = a;
    A.q[2 * i] = r * cs;
    A.q[2 * i + 1] = r * sn;
    A.g[2 * i] = ld(A.gamma, A.dtype, 2 * i) * A.scale;
    A.g[2 * i + 1] = ld(A.gamma, A.dtype, 2 * i + 1) * A.scale;
  } else {
    A.p[i] = a * ld(A.third, A.dtype, i);
    A.q[2 * i] = r;
    A.q[2 * i + 1] = 0.f;
    A.g[2 * i] = ld(A.gamma, A.dtype, i) * A.scale;
    A.g[2 * i + 1] = 0.f;
  }
}

// one lane per (row, state), 64 / N rows per wave (N <= 64): the gradient of theta, a sum over the row's states, is
// collected from the row's lanes.  Rows of more than 64 states: one lane per row walking its states (rpw = 0).
__global__ __launch_bounds__(256) void ema_coeffs_bwd_kernel(const CoeffArgs A, const int rpw) {
  const int lane = (int)threadIdx.x & 63, wave = (int)threadIdx.x >> 6;
  const int gid = (int)blockIdx.x * 256 + (int)threadIdx.x;
  if (gid < A.D) st(A.domega, A.dtype, gid, A.dom[gid]);
  int k, n0, n1;
  bool live;
  if (rpw > 0) {
    const int r = lane / A.N;
    k = ((int)blockIdx.x * 4 + wave) * rpw + r;
    n0 = lane - r * A.N;
    n1 = n0 + 1;
    live = r < rpw && k < A.K;
  } else {
    k = gid;
    n0 = 0;
    n1 = A.N;
    live = k < A.K;
  }
  float tsum = 0.f, st0 = 0.f;
  if (live) {
    if (A.is_complex) st0 = sigm(ld(A.third, A.dtype, k));
    for (int n = n0; n < n1; ++n) {
      const int64_t i = (int64_t)k * A.N + n;
      const float a = sigm(ld(A.alpha, A.dtype, i)), d = sigm(ld(A.delta, A.dtype, i));
      float da, dr;
      if (A.is_complex) {
        const float r = 1.0f - a * d;
        const float ang = (float)(n + 1) * (st0 * A.turn);
        float sn, cs;
        sincosf(ang, &sn, &cs);
        const float gr = A.dq[2 * i], gi = A.dq[2 * i + 1];      // dL/dRe q, dL/dIm q
        dr = gr * cs + gi * sn;
        tsum = fmaf((float)(n + 1), r * (gi * cs - gr * sn), tsum);
        da = A.dp[i];
        st(A.dgamma, A.dtype, 2 * i, A.dg[2 * i] * A.scale);
        st(A.dgamma, A.dtype, 2 * i + 1, A.dg[2 * i + 1] * A.scale);
      } else {
        const float b = ld(A.third, A.dtype, i);
        dr = A.dq[i];                                            // real layer: [K, N] gradients, no pairs
        da = A.dp[i] * b;
        st(A.dthird, A.dtype, i, A.dp[i] * a);
        st(A.dgamma, A.dtype, i, A.dg[i] * A.scale);
      }
      // r = 1 - a d
      st(A.dalpha, A.dtype, i, (da - dr * d) * a * (1.0f - a));
      st(A.ddelta, A.dtype, i, -dr * a * d * (1.0f - d));
    }
  }
  if (!A.is_complex) return;
  if (rpw > 0) {
    // the row's states in order, the same sum every run: lane n0 = 0 of the row adds the others' terms
    const int base = lane - n0;
    float total = 0.f;
    for (int j = 0; j < A.N; ++j) total += __shfl(tsum, base + j, 64);
    tsum = total;
    live = live && n0 == 0;
  }
  if (live) st(A.dthird, A.dtype, k, tsum * A.turn * st0 * (1.0f - st0));
}

struct NormParamArgs {
  const void* weight;      // [H]
  const void* bias;        // [H]
  const void* prior_mean;  // [G]
  const void* prior_logv;  // [G]
  int wdtype, pdtype, H, G, B;
  float* gamma;            // [H] weight + 1
  float* beta;             // [H]
  float* prev_mean;        // [B, G]
  float* prev_var;         // [B, G]
  const float* dgamma;     // backward: gradients of the four results
  const float* dbeta;
  const float* dprev_mean;
  const float* dprev_var;
  void* dweight;
  void* dbias;
  void* dprior_mean;       // null: the prior is a buffer
  void* dprior_logv;
};

__global__ __launch_bounds__(256) void norm_params_fwd_kernel(const NormParamArgs A) {
  const int i = (int)blockIdx.x * 256 + (int)threadIdx.x;
  if (i < A.H) {
    A.gamma[i] = ld(A.weight, A.wdtype, i) + 1.0f;
    A.beta[i] = ld(A.bias, A.wdtype, i);
  }
  if (i < A.B * A.G) {
    const int g = i % A.G;
    A.prev_mean[i] = ld(A.prior_mean, A.pdtype, g);
    A.prev_var[i] = expf(ld(A.prior_logv, A.pdtype, g));
  }
}

__global__ __launch_bounds__(256) void norm_params_bwd_kernel(const NormParamArgs A) {
  const int i = (int)blockIdx.x * 256 + (int)threadIdx.x;
  if (i < A.H) {
    st(A.dweight, A.wdtype, i, A.dgamma[i]);
    st(A.dbias, A.wdtype, i, A.dbeta[i]);
  }
  if (i < A.G && A.dprior_mean) {
    float sm = 0.f, sv = 0.f;
    for (int b = 0; b < A.B; ++b) {            // batch rows in order: the same sum every run
      sm += A.dprev_mean[b * A.G + i];
      sv += A.dprev_var[b * A.G + i];
    }
    st(A.dprior_mean, A.pdtype, i, sm);
    st(A.dprior_logv, A.pdtype, i, sv * expf(ld(A.prior_logv, A.pdtype, i)));
  }
}

bool known(int dtype) { return dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16; }

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_ema_coeffs_fwd(const void* alpha, const void* delta, const void* theta_or_beta, const void* gamma,
                                   const void* omega, int dtype, int is_complex, int64_t K, int64_t N, int64_t D,
                                   float* p, float* q, float* gamma_out, float* omega_out, void* stream) {
  MEGA_REQUIRE(known(dtype), MEGA_ERR_ARG, "ema_coeffs_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(K > 0 && N > 0 && D > 0 && K * N < (1ll << 30) && (K == D || K == 2 * D), MEGA_ERR_ARG,
               "ema_coeffs_fwd: bad sizes K=%lld N=%lld D=%lld", (long long)K, (long long)N, (long long)D);
  MEGA_REQUIRE(alpha && delta && theta_or_beta && gamma && omega && p && q && gamma_out && omega_out, MEGA_ERR_ARG,
               "ema_coeffs_fwd: null pointer argument");
  CoeffArgs A = {};
  A.alpha = alpha; A.delta = delta; A.third = theta_or_beta; A.gamma = gamma; A.omega = omega;
  A.dtype = dtype; A.is_complex = is_complex ? 1 : 0; A.K = (int)K; A.N = (int)N; A.D = (int)D;
  A.scale = (float)sqrt(1.0 / (double)N); A.turn = (float)(2.0 * 3.14159265358979323846 / (double)N);
  A.p = p; A.q = q; A.g = gamma_out; A.om = omega_out;
  const int64_t n = K * N > D ? K * N : D;
  hipLaunchKernelGGL(ema_coeffs_fwd_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, A);
  MEGA_CHECK_LAUNCH("ema_coeffs_fwd");
  return MEGA_OK;
}

extern "C" int mega_ema_coeffs_bwd(const float* p_grad, const float* q_grad, const float* gamma_out_grad,
                                   const float* omega_out_grad, const void* alpha, const void* delta,
                                   const void* theta_or_beta, int dtype, int is_complex, int64_t K, int64_t N,
                                   int64_t D, void* alpha_grad, void* delta_grad, void* theta_or_beta_grad,
                                   void* gamma_grad, void* omega_grad, void* stream) {
  MEGA_REQUIRE(known(dtype), MEGA_ERR_ARG, "ema_coeffs_bwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(K > 0 && N > 0 && D > 0 && K * N < (1ll << 30) && (K == D || K == 2 * D), MEGA_ERR_ARG,
               "ema_coeffs_bwd: bad sizes K=%lld N=%lld D=%lld", (long long)K, (long long)N, (long long)D);
  MEGA_REQUIRE(p_grad && q_grad && gamma_out_grad && omega_out_grad && alpha && delta && theta_or_beta && alpha_grad &&
                   delta_grad && theta_or_beta_grad && gamma_grad && omega_grad,
               MEGA_ERR_ARG, "ema_coeffs_bwd: null pointer argument");
  CoeffArgs A = {};
  A.alpha = alpha; A.delta = delta; A.third = theta_or_beta;
  A.dtype = dtype; A.is_complex = is_complex ? 1 : 0; A.K = (int)K; A.N = (int)N; A.D = (int)D;
  A.scale = (float)sqrt(1.0 / (double)N); A.turn = (float)(2.0 * 3.14159265358979323846 / (double)N);
  A.dp = p_grad; A.dq = q_grad; A.dg = gamma_out_grad; A.dom = omega_out_grad;
  A.dalpha = alpha_grad; A.ddelta = delta_grad; A.dthird = theta_or_beta_grad; A.dgamma = gamma_grad;
  A.domega = omega_grad;
  const int rpw = N <= 64 ? (int)(64 / N) : 0;                   // rows per wave, one lane per (row, state)
  int64_t blocks = rpw > 0 ? ceil_div(K, 4 * rpw) : ceil_div(K, 256);
  if (blocks * 256 < D) blocks = ceil_div(D, 256);               // the first D threads also copy omega's gradient
  hipLaunchKernelGGL(ema_coeffs_bwd_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, A, rpw);
  MEGA_CHECK_LAUNCH("ema_coeffs_bwd");
  return MEGA_OK;
}

extern "C" int mega_norm_params_fwd(const void* weight, const void* bias, int dtype, const void* prior_mean,
                                    const void* prior_logv, int prior_dtype, int64_t H, int64_t G, int64_t B,
                                    float* gamma, float* beta, float* prev_mean, float* prev_var, void* stream) {
  MEGA_REQUIRE(known(dtype) && known(prior_dtype), MEGA_ERR_ARG, "norm_params_fwd: unknown dtype %d / %d", dtype,
               prior_dtype);
  MEGA_REQUIRE(H > 0 && G > 0 && B > 0 && H < (1ll << 30) && B * G < (1ll << 30), MEGA_ERR_ARG,
               "norm_params_fwd: bad sizes H=%lld G=%lld B=%lld", (long long)H, (long long)G, (long long)B);
  MEGA_REQUIRE(weight && bias && prior_mean && prior_logv && gamma && beta && prev_mean && prev_var, MEGA_ERR_ARG,
               "norm_params_fwd: null pointer argument");
  NormParamArgs A = {};
  A.weight = weight; A.bias = bias; A.prior_mean = prior_mean; A.prior_logv = prior_logv;
  A.wdtype = dtype; A.pdtype = prior_dtype; A.H = (int)H; A.G = (int)G; A.B = (int)B;
  A.gamma = gamma; A.beta = beta; A.prev_mean = prev_mean; A.prev_var = prev_var;
  const int64_t n = H > B * G ? H : B * G;
  hipLaunchKernelGGL(norm_params_fwd_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, A);
  MEGA_CHECK_LAUNCH("norm_params_fwd");
  return MEGA_OK;
}

extern "C" int mega_norm_params_bwd(const float* gamma_grad, const float* beta_grad, const float* prev_mean_grad,
                                    const float* prev_var_grad, const void* prior_logv, int dtype, int prior_dtype,
                                    int64_t H, int64_t G, int64_t B, void* weight_grad, void* bias_grad,
                                    void* prior_mean_grad, void* prior_logv_grad, void* stream) {
  MEGA_REQUIRE(known(dtype) && known(prior_dtype), MEGA_ERR_ARG, "norm_params_bwd: unknown dtype %d / %d", dtype,
               prior_dtype);
  MEGA_REQUIRE(H > 0 && G > 0 && B > 0 && H < (1ll << 30) && B * G < (1ll << 30), MEGA_ERR_ARG,
               "norm_params_bwd: bad sizes H=%lld G=%lld B=%lld", (long long)H, (long long)G, (long long)B);
  MEGA_REQUIRE(gamma_grad && beta_grad && weight_grad && bias_grad, MEGA_ERR_ARG,
               "norm_params_bwd: null pointer argument");
  MEGA_REQUIRE((prior_mean_grad == nullptr) == (prior_logv_grad == nullptr), MEGA_ERR_ARG,
               "norm_params_bwd: the two prior gradients go together");
  MEGA_REQUIRE(!prior_mean_grad || (prev_mean_grad && prev_var_grad && prior_logv), MEGA_ERR_ARG,
               "norm_params_bwd: the prior's gradients need prev_mean_grad, prev_var_grad and prior_logv");
  NormParamArgs A = {};
  A.prior_logv = prior_logv; A.wdtype = dtype; A.pdtype = prior_dtype; A.H = (int)H; A.G = (int)G; A.B = (int)B;
  A.dgamma = gamma_grad; A.dbeta = beta_grad; A.dprev_mean = prev_mean_grad; A.dprev_var = prev_var_grad;
  A.dweight = weight_grad; A.dbias = bias_grad; A.dprior_mean = prior_mean_grad; A.dprior_logv = prior_logv_grad;
  const int64_t n = H > G ? H : G;
  hipLaunchKernelGGL(norm_params_bwd_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, A);
  MEGA_CHECK_LAUNCH("norm_params_bwd");
  return MEGA_OK;
}
