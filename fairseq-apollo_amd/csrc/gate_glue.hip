// Elementwise and per-token glue of the gated-attention layer
// (fairseq/modules/moving_average_gated_attention.py:322-330, 407-412): the pieces between the
// projections and the attention product.  Every kernel is a single streaming pass in fp32
// registers with one rounding at the store; operands are rows of a wider projection output, so
// each takes its own row stride and the split of that output never needs a copy.
//
//   rms_norm   y = x / sqrt(mean(x^2) + eps) * weight                      (one wave per token)
//   gate_qk    q, k = rotary(normalize(z) * gamma[i] + beta[i])             (one wave per token)
//   gate_mul   y = a * silu(r)
//   gate_out   y = residual + sigmoid(u) * (silu(hx + hp) - residual)
#include "common.h"

namespace mega {
namespace {

constexpr int kRowThreads = 256;                 // 4 waves, one token each
constexpr int kRowsPerWg = kRowThreads / 64;

// hardware reciprocal (1 ulp) in the place of a full division
__device__ __forceinline__ float silu_f(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// ---------------------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(kRowThreads) void rms_norm_kernel(const T* __restrict__ x, int64_t xs,
                                                               const float* __restrict__ w, T* __restrict__ y,
                                                               int64_t T_, int D, float eps) {
  using V = Vec<T, VEC>;
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
  if (t >= T_) return;
  const T* row = x + t * xs;
  float ss = 0.f;
  for (int j = lane * VEC; j < D; j += 64 * VEC) {
    const V v = *(const V*)(row + j);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float f = to_float(v.v[i]);
      ss = fmaf(f, f, ss);
    }
  }
  const float r = rsqrtf(wave_sum(ss) / (float)D + eps);
  T* out = y + t * (int64_t)D;
  for (int j = lane * VEC; j < D; j += 64 * VEC) {
    const V v = *(const V*)(row + j);   // second read of a row this wave has just pulled in
    V o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float g = w ? w[j + i] : 1.0f;
      o.v[i] = from_float<T>(to_float(v.v[i]) * r * g);
    }
    *(V*)(out + j) = o;
  }
}

// ---------------------------------------------------------------------------------------------
// One wave per token: L2 norm over the S features, the two affine maps, then the rotation of
// feature pairs (2i, 2i+1) of each head by pos * freqs[i]  (relative_positional_bias.py:86-92),
// pos = pos0 + token index within its chunk.
template <typename T, int VEC>
__global__ __launch_bounds__(kRowThreads) void gate_qk_kernel(const T* __restrict__ z, int64_t zs,
                                                              const float* __restrict__ gamma,
                                                              const float* __restrict__ beta,
                                                              const float* __restrict__ freqs, T* __restrict__ q,
                                                              T* __restrict__ k, int64_t T_, int S, int Hd,
                                                              int64_t chunk, int64_t pos0, float eps) {
  using V = Vec<T, VEC>;
  static_assert(VEC % 2 == 0, "pairs of features stay inside one vector");
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
  if (t >= T_) return;
  const T* row = z + t * zs;
  float ss = 0.f;
  for (int j = lane * VEC; j < S; j += 64 * VEC) {
    const V v = *(const V*)(row + j);
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float f = to_float(v.v[i]);
      ss = fmaf(f, f, ss);
    }
  }
  const float inv = 1.0f / fmaxf(sqrtf(wave_sum(ss)), eps);   // F.normalize: x / max(|x|, eps)
  const float pos = (float)(pos0 + t % chunk);
  T* qo = q + t * (int64_t)S;
  T* ko = k + t * (int64_t)S;
  for (int j = lane * VEC; j < S; j += 64 * VEC) {
    const V v = *(const V*)(row + j);
    V oq, ok;
#pragma unroll
    for (int i = 0; i < VEC; i += 2) {
      const int f = j + i;
      float sn, cs;
      sincosf(pos * freqs[(f % Hd) >> 1], &sn, &cs);
      const float z0 = to_float(v.v[i]) * inv, z1 = to_float(v.v[i + 1]) * inv;
      const float q0 = fmaf(z0, gamma[f], beta[f]), q1 = fmaf(z1, gamma[f + 1], beta[f + 1]);
      const float k0 = fmaf(z0, gamma[S + f], beta[S + f]), k1 = fmaf(z1, gamma[S + f + 1], beta[S + f + 1]);
      oq.v[i] = from_float<T>(q0 * cs - q1 * sn);
      oq.v[i + 1] = from_float<T>(q0 * sn + q1 * cs);
      ok.v[i] = from_float<T>(k0 * cs - k1 * sn);
      ok.v[i + 1] = from_float<T>(k0 * sn + k1 * cs);
    }
    *(V*)(qo + j) = oq;
    *(V*)(ko + j) = ok;
  }
}

// Backward of the q / k map.  One wave per token, a wave walks tokens t, t + waves, ...; lane l owns
// the same NV vectors of features at every token, so the four parameter sums (d gamma, d beta of the
// q and of the k map) stay in registers until the end:
//   dq_pre = rot^T(dq), dk_pre = rot^T(dk)                         (rotation by -pos * freq)
//   dbeta_q += dq_pre, dgamma_q += dq_pre zn   (and the same for k)
//   dzn = dq_pre gamma_q + dk_pre gamma_k
//   dz  = (dzn - zn (zn . dzn)) / |z|      (|z| > eps)      or      dzn / eps      (|z| <= eps)
// The workgroup's four waves then add their sums in LDS, one after the other, and leave one row
// per workgroup in `part` [workgroups][4][S]; gate_qk_param_kernel adds the rows in order.
template <typename T, int VEC, int NV>
__global__ __launch_bounds__(kRowThreads) void gate_qk_bwd_kernel(
    const T* __restrict__ dq, const T* __restrict__ dk, const T* __restrict__ z, int64_t zs,
    const float* __restrict__ gamma, const float* __restrict__ freqs, T* __restrict__ dz, int64_t dzs,
    float* __restrict__ part, int64_t T_, int S, int Hd, int64_t chunk, int64_t pos0, float eps) {
  using V = Vec<T, VEC>;
  static_assert(VEC % 2 == 0, "pairs of features stay inside one vector");
  extern __shared__ float s_acc[];                     // [4][S]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float agq[NV][VEC], abq[NV][VEC], agk[NV][VEC], abk[NV][VEC];
  float gq[NV][VEC], gk[NV][VEC], fr[NV][VEC / 2];
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int j = (u * 64 + lane) * VEC;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      agq[u][i] = abq[u][i] = agk[u][i] = abk[u][i] = 0.f;
      gq[u][i] = j + i < S ? gamma[j + i] : 0.f;
      gk[u][i] = j + i < S ? gamma[S + j + i] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < VEC / 2; ++i) fr[u][i] = j + 2 * i < S ? freqs[((j + 2 * i) % Hd) >> 1] : 0.f;
  }
  const int64_t stride = (int64_t)gridDim.x * kRowsPerWg;
  for (int64_t t = (int64_t)blockIdx.x * kRowsPerWg + wave; t < T_; t += stride) {
    const T* row = z + t * zs;
    float zf[NV][VEC], aq[NV][VEC], ak[NV][VEC];
    float ss = 0.f;
    const float pos = (float)(pos0 + t % chunk);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int j = (u * 64 + lane) * VEC;
      if (j < S) {
        const V v = *(const V*)(row + j);
        const V a = *(const V*)(dq + t * (int64_t)S + j);
        const V b = *(const V*)(dk + t * (int64_t)S + j);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          zf[u][i] = to_float(v.v[i]);
          ss = fmaf(zf[u][i], zf[u][i], ss);
        }
#pragma unroll
        for (int i = 0; i < VEC; i += 2) {
          float sn, cs;
          sincosf(pos * fr[u][i >> 1], &sn, &cs);
          const float a0 = to_float(a.v[i]), a1 = to_float(a.v[i + 1]);
          const float b0 = to_float(b.v[i]), b1 = to_float(b.v[i + 1]);
          aq[u][i] = a0 * cs + a1 * sn;
          aq[u][i + 1] = a1 * cs - a0 * sn;
          ak[u][i] = b0 * cs + b1 * sn;
          ak[u][i + 1] = b1 * cs - b0 * sn;
        }
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) zf[u][i] = aq[u][i] = ak[u][i] = 0.f;
      }
    }
    const float nrm = sqrtf(wave_sum(ss));
    const bool clamped = !(nrm > eps);
    const float inv = 1.0f / fmaxf(nrm, eps);
    float dot = 0.f;
    float dzn[NV][VEC];
#pragma unroll
    for (int u = 0; u < NV; ++u)
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float zn = zf[u][i] * inv;
        abq[u][i] += aq[u][i];
        agq[u][i] = fmaf(aq[u][i], zn, agq[u][i]);
        abk[u][i] += ak[u][i];
        agk[u][i] = fmaf(ak[u][i], zn, agk[u][i]);
        dzn[u][i] = fmaf(aq[u][i], gq[u][i], ak[u][i] * gk[u][i]);
        dot = fmaf(zn, dzn[u][i], dot);
        zf[u][i] = zn;
      }
    dot = clamped ? 0.f : wave_sum(dot);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int j = (u * 64 + lane) * VEC;
      if (j < S) {
        V o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) o.v[i] = from_float<T>((dzn[u][i] - zf[u][i] * dot) * inv);
        *(V*)(dz + t * dzs + j) = o;
      }
    }
  }
  // the four waves add up in a fixed order
  for (int turn = 0; turn < kRowsPerWg; ++turn) {
    if (wave == turn) {
#pragma unroll
      for (int u = 0; u < NV; ++u) {
        const int j = (u * 64 + lane) * VEC;
#pragma unroll
        for (int i = 0; i < VEC; ++i)
          if (j + i < S) {
            if (turn == 0) {
              s_acc[j + i] = agq[u][i]; s_acc[S + j + i] = agk[u][i];
              s_acc[2 * S + j + i] = abq[u][i]; s_acc[3 * S + j + i] = abk[u][i];
            } else {
              s_acc[j + i] += agq[u][i]; s_acc[S + j + i] += agk[u][i];
              s_acc[2 * S + j + i] += abq[u][i]; s_acc[3 * S + j + i] += abk[u][i];
            }
          }
      }
    }
    __syncthreads();
  }
  float* dst = part + (size_t)blockIdx.x * 4 * S;
  for (int i = threadIdx.x; i < 4 * S; i += kRowThreads) dst[i] = s_acc[i];
}

// dgamma [2, S] = rows 0, 1 of the sums, dbeta [2, S] = rows 2, 3.  A workgroup owns 64 adjacent
// columns; its 16 waves each add every 16th row (independent loads in flight, a fixed order inside
// the wave), then the 16 sums of a column are added in wave order.
constexpr int kParamSlices = 16;
__global__ __launch_bounds__(64 * kParamSlices) void gate_qk_param_kernel(const float* __restrict__ part, int rows,
                                                                          int S, float* __restrict__ dgamma,
                                                                          float* __restrict__ dbeta) {
  __shared__ float s_sum[kParamSlices][64];
  const int lane = threadIdx.x & 63, slice = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + lane;
  const size_t W = (size_t)4 * S;
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  if (i < 4 * S) {
    int r = slice;
    for (; r + 3 * kParamSlices < rows; r += 4 * kParamSlices) {
      a0 += part[(size_t)r * W + i];
      a1 += part[(size_t)(r + kParamSlices) * W + i];
      a2 += part[(size_t)(r + 2 * kParamSlices) * W + i];
      a3 += part[(size_t)(r + 3 * kParamSlices) * W + i];
    }
    for (; r < rows; r += kParamSlices) a0 += part[(size_t)r * W + i];
  }
  s_sum[slice][lane] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  if (slice == 0 && i < 4 * S) {
    float a = 0.f;
#pragma unroll
    for (int w = 0; w < kParamSlices; ++w) a += s_sum[w][lane];
    if (i < 2 * S) dgamma[i] = a;
    else dbeta[i - 2 * S] = a;
  }
}

// ---------------------------------------------------------------------------------------------
// Row-strided elementwise kernels: blockIdx.x walks rows, threads walk the row in vectors.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void gate_mul_kernel(const T* __restrict__ a, int64_t as, const T* __restrict__ r,
                                                       int64_t rs, T* __restrict__ y, int64_t T_, int E) {
  using V = Vec<T, VEC>;
  for (int64_t t = blockIdx.x; t < T_; t += gridDim.x) {
    const T* ar = a + t * as;
    const T* rr = r + t * rs;
    T* yr = y + t * (int64_t)E;
    for (int j = threadIdx.x * VEC; j < E; j += 256 * VEC) {
      const V av = *(const V*)(ar + j);
      const V rv = *(const V*)(rr + j);
      V o;
#pragma unroll
      for (int i = 0; i < VEC; ++i) o.v[i] = from_float<T>(to_float(av.v[i]) * silu_f(to_float(rv.v[i])));
      *(V*)(yr + j) = o;
    }
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void gate_out_kernel(const T* __restrict__ res, int64_t ress,
                                                       const T* __restrict__ u, int64_t us, const T* __restrict__ hx,
                                                       int64_t hxs, const T* __restrict__ hp, int64_t hps,
                                                       T* __restrict__ y, int64_t T_, int D) {
  using V = Vec<T, VEC>;
  for (int64_t t = blockIdx.x; t < T_; t += gridDim.x) {
    const T* r0 = res + t * ress;
    const T* u0 = u + t * us;
    const T* x0 = hx + t * hxs;
    const T* p0 = hp + t * hps;
    T* yr = y + t * (int64_t)D;
    for (int j = threadIdx.x * VEC; j < D; j += 256 * VEC) {
      const V rv = *(const V*)(r0 + j);
      const V uv = *(const V*)(u0 + j);
      const V xv = *(const V*)(x0 + j);
      const V pv = *(const V*)(p0 + j);
      V o;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float rr = to_float(rv.v[i]);
        const float h = silu_f(to_float(xv.v[i]) + to_float(pv.v[i]));
        o.v[i] = from_float<T>(fmaf(sigmoid_f(to_float(uv.v[i])), h - rr, rr));
      }
      *(V*)(yr + j) = o;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Backward of the three element-wise gates.  silu'(a) = s (1 + a (1 - s)), s = sigmoid(a).
__device__ __forceinline__ float dsilu_f(float a) {
  const float sg = sigmoid_f(a);
  return sg * fmaf(a, 1.0f - sg, 1.0f);
}

// y = a * silu(r):  da = dy silu(r),  dr = dy a silu'(r)
template <typename T, int VEC>
__global__ __launch_bounds__(256) void gate_mul_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ a,
                                                           int64_t as, const T* __restrict__ r, int64_t rs,
                                                           T* __restrict__ da, T* __restrict__ dr, int64_t drs,
                                                           int64_t T_, int E) {
  using V = Vec<T, VEC>;
  for (int64_t t = blockIdx.x; t < T_; t += gridDim.x) {
    for (int j = threadIdx.x * VEC; j < E; j += 256 * VEC) {
      const V gv = *(const V*)(dy + t * (int64_t)E + j);
      const V av = *(const V*)(a + t * as + j);
      const V rv = *(const V*)(r + t * rs + j);
      V oa, orr;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float g = to_float(gv.v[i]), rr = to_float(rv.v[i]);
        oa.v[i] = from_float<T>(g * silu_f(rr));
        orr.v[i] = from_float<T>(g * to_float(av.v[i]) * dsilu_f(rr));
      }
      *(V*)(da + t * (int64_t)E + j) = oa;
      *(V*)(dr + t * drs + j) = orr;
    }
  }
}

// y = res + sigmoid(u) (silu(hx + hp) - res):
//   dres = dy (1 - s),  du = dy (h - res) s (1 - s),  da = dy s silu'(hx + hp)  (da serves hx and hp)
template <typename T, int VEC>
__global__ __launch_bounds__(256) void gate_out_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ res,
                                                           int64_t ress, const T* __restrict__ u, int64_t us,
                                                           const T* __restrict__ hx, int64_t hxs,
                                                           const T* __restrict__ hp, int64_t hps, T* __restrict__ dres,
                                                           T* __restrict__ du, int64_t dus, T* __restrict__ da,
                                                           int64_t das, int64_t T_, int D) {
  using V = Vec<T, VEC>;
  for (int64_t t = blockIdx.x; t < T_; t += gridDim.x) {
    for (int j = threadIdx.x * VEC; j < D; j += 256 * VEC) {
      const V gv = *(const V*)(dy + t * (int64_t)D + j);
      const V rv = *(const V*)(res + t * ress + j);
      const V uv = *(const V*)(u + t * us + j);
      const V xv = *(const V*)(hx + t * hxs + j);
      const V pv = *(const V*)(hp + t * hps + j);
      V o0, o1, o2;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float g = to_float(gv.v[i]), rr = to_float(rv.v[i]);
        const float sg = sigmoid_f(to_float(uv.v[i]));
        const float a = to_float(xv.v[i]) + to_float(pv.v[i]);
        o0.v[i] = from_float<T>(g * (1.0f - sg));
        o1.v[i] = from_float<T>(g * (silu_f(a) - rr) * sg * (1.0f - sg));
        o2.v[i] = from_float<T>(g * sg * dsilu_f(a));
      }
      *(V*)(dres + t * (int64_t)D + j) = o0;
      *(V*)(du + t * dus + j) = o1;
      *(V*)(da + t * das + j) = o2;
    }
  }
}

// y = silu(a) * b:  da = dy b silu'(a),  db = dy silu(a)   (contiguous operands)
template <typename T, int VEC>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ a,
                                                         const T* __restrict__ b, T* __restrict__ da,
                                                         T* __restrict__ db, int64_t n) {
  using V = Vec<T, VEC>;
  const int64_t nv = n / VEC;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nv; i += stride) {
    const V gv = ((const V*)dy)[i];
    const V av = ((const V*)a)[i];
    const V bv = ((const V*)b)[i];
    V oa, ob;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      const float g = to_float(gv.v[k]), aa = to_float(av.v[k]);
      oa.v[k] = from_float<T>(g * to_float(bv.v[k]) * dsilu_f(aa));
      ob.v[k] = from_float<T>(g * silu_f(aa));
    }
    ((V*)da)[i] = oa;
    ((V*)db)[i] = ob;
  }
  const int64_t t = nv * VEC + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) {
    const float g = to_float(dy[t]), aa = to_float(a[t]);
    da[t] = from_float<T>(g * to_float(b[t]) * dsilu_f(aa));
    db[t] = from_float<T>(g * silu_f(aa));
  }
}

// ---------------------------------------------------------------------------------------------
inline bool vec_ok(const void* p, int64_t stride, size_t elem, int vec) {
  return ((uintptr_t)p % (elem * vec)) == 0 && stride % vec == 0;
}

inline unsigned row_grid(int64_t T_) {
  const int64_t cap = 256 * 16;
  return (unsigned)(T_ < cap ? T_ : cap);
}

template <typename T>
int launch_rms_norm(const void* x, int64_t xs, const float* w, void* y, int64_t T_, int64_t D, float eps,
                    hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const unsigned grid = (unsigned)ceil_div(T_, kRowsPerWg);
  if (D % VEC == 0 && vec_ok(x, xs, sizeof(T), VEC) && vec_ok(y, D, sizeof(T), VEC))
    hipLaunchKernelGGL((rms_norm_kernel<T, VEC>), dim3(grid), dim3(kRowThreads), 0, s, (const T*)x, xs, w, (T*)y, T_,
                       (int)D, eps);
  else
    hipLaunchKernelGGL((rms_norm_kernel<T, 1>), dim3(grid), dim3(kRowThreads), 0, s, (const T*)x, xs, w, (T*)y, T_,
                       (int)D, eps);
  MEGA_CHECK_LAUNCH("rms_norm_fwd");
  return MEGA_OK;
}

template <typename T>
int launch_gate_qk(const void* z, int64_t zs, const float* gamma, const float* beta, const float* freqs, void* q,
                   void* k, int64_t T_, int64_t S, int64_t Hd, int64_t chunk, int64_t pos0, float eps,
                   hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const unsigned grid = (unsigned)ceil_div(T_, kRowsPerWg);
  if (S % VEC == 0 && vec_ok(z, zs, sizeof(T), VEC) && vec_ok(q, S, sizeof(T), VEC) && vec_ok(k, S, sizeof(T), VEC))
    hipLaunchKernelGGL((gate_qk_kernel<T, VEC>), dim3(grid), dim3(kRowThreads), 0, s, (const T*)z, zs, gamma, beta,
                       freqs, (T*)q, (T*)k, T_, (int)S, (int)Hd, chunk, pos0, eps);
  else {
    MEGA_REQUIRE(vec_ok(z, zs, sizeof(T), 2) && vec_ok(q, S, sizeof(T), 2) && vec_ok(k, S, sizeof(T), 2), MEGA_ERR_ARG,
                 "gate_qk_fwd: rows must start on an even element (feature pairs are moved together)");
    hipLaunchKernelGGL((gate_qk_kernel<T, 2>), dim3(grid), dim3(kRowThreads), 0, s, (const T*)z, zs, gamma, beta,
                       freqs, (T*)q, (T*)k, T_, (int)S, (int)Hd, chunk, pos0, eps);
  }
  MEGA_CHECK_LAUNCH("gate_qk_fwd");
  return MEGA_OK;
}

constexpr int kQkBwdMaxWgs = 512;

inline int64_t gate_qk_bwd_wgs(int64_t T_) {
  const int64_t w = ceil_div(T_, kRowsPerWg);
  return w < kQkBwdMaxWgs ? w : kQkBwdMaxWgs;
}

template <typename T>
int launch_gate_qk_bwd(const void* dq, const void* dk, const void* z, int64_t zs, const float* gamma,
                       const float* freqs, void* dz, int64_t dzs, float* dgamma, float* dbeta, float* part, int64_t T_,
                       int64_t S, int64_t Hd, int64_t chunk, int64_t pos0, float eps, hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  MEGA_REQUIRE(S % VEC == 0 && S <= 2 * 64 * VEC && vec_ok(z, zs, sizeof(T), VEC) && vec_ok(dq, S, sizeof(T), VEC) &&
                   vec_ok(dk, S, sizeof(T), VEC) && vec_ok(dz, dzs, sizeof(T), VEC),
               MEGA_ERR_UNSUPPORTED,
               "gate_qk_bwd: S=%lld must be a multiple of %d, at most %d, with 16-byte aligned rows", (long long)S, VEC,
               2 * 64 * VEC);
  const unsigned grid = (unsigned)gate_qk_bwd_wgs(T_);
  const size_t lds = (size_t)4 * S * sizeof(float);
  if (audit_on()) {
    // every workgroup leaves one row of 4 S sums; rows of T tokens of S (z: pitch zs) elements on the tensors
    audit_use(part, (size_t)grid * 4 * S * 4, "gate_qk_bwd: rows of parameter sums");
    audit_use(dq, (size_t)T_ * S * sizeof(T), "gate_qk_bwd: q_grad");
    audit_use(dk, (size_t)T_ * S * sizeof(T), "gate_qk_bwd: k_grad");
    audit_use(dz, (size_t)((T_ - 1) * dzs + S) * sizeof(T), "gate_qk_bwd: z_grad");
    audit_use(z, (size_t)((T_ - 1) * zs + S) * sizeof(T), "gate_qk_bwd: z");
    audit_use(dgamma, (size_t)2 * S * 4, "gate_qk_bwd: gamma_grad");
    audit_use(dbeta, (size_t)2 * S * 4, "gate_qk_bwd: beta_grad");
    return MEGA_OK;
  }
  if (S <= 64 * VEC)
    hipLaunchKernelGGL((gate_qk_bwd_kernel<T, VEC, 1>), dim3(grid), dim3(kRowThreads), lds, s, (const T*)dq,
                       (const T*)dk, (const T*)z, zs, gamma, freqs, (T*)dz, dzs, part, T_, (int)S, (int)Hd, chunk, pos0, eps);
  else
    hipLaunchKernelGGL((gate_qk_bwd_kernel<T, VEC, 2>), dim3(grid), dim3(kRowThreads), lds, s, (const T*)dq,
                       (const T*)dk, (const T*)z, zs, gamma, freqs, (T*)dz, dzs, part, T_, (int)S, (int)Hd, chunk, pos0, eps);
  MEGA_CHECK_LAUNCH("gate_qk_bwd");
  hipLaunchKernelGGL(gate_qk_param_kernel, dim3((unsigned)ceil_div(4 * S, 64)), dim3(64 * kParamSlices), 0, s, part,
                     (int)grid,
                     (int)S, dgamma, dbeta);
  MEGA_CHECK_LAUNCH("gate_qk_bwd (parameter sums)");
  return MEGA_OK;
}

template <typename T>
int launch_gate_mul(const void* a, int64_t as, const void* r, int64_t rs, void* y, int64_t T_, int64_t E,
                    hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  if (E % VEC == 0 && vec_ok(a, as, sizeof(T), VEC) && vec_ok(r, rs, sizeof(T), VEC) && vec_ok(y, E, sizeof(T), VEC))
    hipLaunchKernelGGL((gate_mul_kernel<T, VEC>), dim3(row_grid(T_)), dim3(256), 0, s, (const T*)a, as, (const T*)r,
                       rs, (T*)y, T_, (int)E);
  else
    hipLaunchKernelGGL((gate_mul_kernel<T, 1>), dim3(row_grid(T_)), dim3(256), 0, s, (const T*)a, as, (const T*)r, rs,
                       (T*)y, T_, (int)E);
  MEGA_CHECK_LAUNCH("gate_mul_fwd");
  return MEGA_OK;
}

template <typename T>
int launch_gate_out(const void* res, int64_t ress, const void* u, int64_t us, const void* hx, int64_t hxs,
                    const void* hp, int64_t hps, void* y, int64_t T_, int64_t D, hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  if (D % VEC == 0 && vec_ok(res, ress, sizeof(T), VEC) && vec_ok(u, us, sizeof(T), VEC) &&
      vec_ok(hx, hxs, sizeof(T), VEC) && vec_ok(hp, hps, sizeof(T), VEC) && vec_ok(y, D, sizeof(T), VEC))
    hipLaunchKernelGGL((gate_out_kernel<T, VEC>), dim3(row_grid(T_)), dim3(256), 0, s, (const T*)res, ress,
                       (const T*)u, us, (const T*)hx, hxs, (const T*)hp, hps, (T*)y, T_, (int)D);
  else
    hipLaunchKernelGGL((gate_out_kernel<T, 1>), dim3(row_grid(T_)), dim3(256), 0, s, (const T*)res, ress, (const T*)u,
                       us, (const T*)hx, hxs, (const T*)hp, hps, (T*)y, T_, (int)D);
  MEGA_CHECK_LAUNCH("gate_out_fwd");
  return MEGA_OK;
}

template <typename T>
int launch_gate_mul_bwd(const void* dy, const void* a, int64_t as, const void* r, int64_t rs, void* da, void* dr,
                        int64_t drs, int64_t T_, int64_t E, hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool v = E % VEC == 0 && vec_ok(dy, E, sizeof(T), VEC) && vec_ok(a, as, sizeof(T), VEC) &&
                 vec_ok(r, rs, sizeof(T), VEC) && vec_ok(da, E, sizeof(T), VEC) && vec_ok(dr, drs, sizeof(T), VEC);
  if (v)
    hipLaunchKernelGGL((gate_mul_bwd_kernel<T, VEC>), dim3(row_grid(T_)), dim3(256), 0, s, (const T*)dy, (const T*)a,
                       as, (const T*)r, rs, (T*)da, (T*)dr, drs, T_, (int)E);
  else
    hipLaunchKernelGGL((gate_mul_bwd_kernel<T, 1>), dim3(row_grid(T_)), dim3(256), 0, s, (const T*)dy, (const T*)a, as,
                       (const T*)r, rs, (T*)da, (T*)dr, drs, T_, (int)E);
  MEGA_CHECK_LAUNCH("gate_mul_bwd");
  return MEGA_OK;
}

template <typename T>
int launch_gate_out_bwd(const void* dy, const void* res, int64_t ress, const void* u, int64_t us, const void* hx,
                        int64_t hxs, const void* hp, int64_t hps, void* dres, void* du, int64_t dus, void* da,
                        int64_t das, int64_t T_, int64_t D, hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool v = D % VEC == 0 && vec_ok(dy, D, sizeof(T), VEC) && vec_ok(res, ress, sizeof(T), VEC) &&
                 vec_ok(u, us, sizeof(T), VEC) && vec_ok(hx, hxs, sizeof(T), VEC) && vec_ok(hp, hps, sizeof(T), VEC) &&
                 vec_ok(dres, D, sizeof(T), VEC) && vec_ok(du, dus, sizeof(T), VEC) && vec_ok(da, das, sizeof(T), VEC);
  if (v)
    hipLaunchKernelGGL((gate_out_bwd_kernel<T, VEC>), dim3(row_grid(T_)), dim3(256), 0, s, (const T*)dy, (const T*)res,
                       ress, (const T*)u, us, (const T*)hx, hxs, (const T*)hp, hps, (T*)dres, (T*)du, dus, (T*)da, das,
                       T_, (int)D);
  else
    hipLaunchKernelGGL((gate_out_bwd_kernel<T, 1>), dim3(row_grid(T_)), dim3(256), 0, s, (const T*)dy, (const T*)res,
                       ress, (const T*)u, us, (const T*)hx, hxs, (const T*)hp, hps, (T*)dres, (T*)du, dus, (T*)da, das,
                       T_, (int)D);
  MEGA_CHECK_LAUNCH("gate_out_bwd");
  return MEGA_OK;
}

template <typename T>
int launch_swiglu_bwd(const void* dy, const void* a, const void* b, void* da, void* db, int64_t n, hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool aligned = (((uintptr_t)dy | (uintptr_t)a | (uintptr_t)b | (uintptr_t)da | (uintptr_t)db) % 16) == 0;
  int64_t blocks = ceil_div(ceil_div(n, VEC), 256);
  if (blocks > 256 * 16) blocks = 256 * 16;
  if (blocks < 1) blocks = 1;
  if (aligned)
    hipLaunchKernelGGL((swiglu_bwd_kernel<T, VEC>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)dy, (const T*)a,
                       (const T*)b, (T*)da, (T*)db, n);
  else
    hipLaunchKernelGGL((swiglu_bwd_kernel<T, 1>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)dy, (const T*)a,
                       (const T*)b, (T*)da, (T*)db, n);
  MEGA_CHECK_LAUNCH("swiglu_bwd");
  return MEGA_OK;
}

bool known_dtype(int dtype) { return dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16; }

}  // namespace
}  // namespace mega

using namespace mega;

#define MEGA_GLUE_DISPATCH(fn, ...)                 \
  switch (dtype) {                                  \
    case MEGA_F32: return fn<float>(__VA_ARGS__);   \
    case MEGA_BF16: return fn<bf16_t>(__VA_ARGS__); \
    default: return fn<f16_t>(__VA_ARGS__);         \
  }

extern "C" int mega_rms_norm_fwd(const void* x, int64_t x_stride, const float* weight, void* y, int dtype, int64_t T_,
                                 int64_t D, double eps, void* stream) {
  MEGA_REQUIRE(known_dtype(dtype), MEGA_ERR_ARG, "rms_norm_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(T_ >= 0 && D >= 1 && D < (1ll << 30), MEGA_ERR_ARG, "rms_norm_fwd: bad sizes T=%lld D=%lld",
               (long long)T_, (long long)D);
  if (T_ == 0) return MEGA_OK;
  MEGA_REQUIRE(x && y, MEGA_ERR_ARG, "rms_norm_fwd: null pointer argument");
  MEGA_REQUIRE(x_stride >= D, MEGA_ERR_ARG, "rms_norm_fwd: row stride %lld below the row length %lld",
               (long long)x_stride, (long long)D);
  MEGA_REQUIRE(ceil_div(T_, kRowsPerWg) < (1ll << 31), MEGA_ERR_ARG, "rms_norm_fwd: too many rows");
  hipStream_t s = (hipStream_t)stream;
  MEGA_GLUE_DISPATCH(launch_rms_norm, x, x_stride, weight, y, T_, D, (float)eps, s);
}

extern "C" int mega_gate_qk_fwd(const void* z, int64_t z_stride, const float* gamma, const float* beta,
                                const float* freqs, void* q, void* k, int dtype, int64_t T_, int64_t S,
                                int64_t heads, int64_t chunk, int64_t pos0, double eps, void* stream) {
  MEGA_REQUIRE(known_dtype(dtype), MEGA_ERR_ARG, "gate_qk_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(T_ >= 0 && S >= 2 && S < (1ll << 30) && heads >= 1 && chunk >= 1 && pos0 >= 0, MEGA_ERR_ARG,
               "gate_qk_fwd: bad sizes T=%lld S=%lld heads=%lld chunk=%lld pos0=%lld", (long long)T_, (long long)S,
               (long long)heads, (long long)chunk, (long long)pos0);
  MEGA_REQUIRE(S % heads == 0 && (S / heads) % 2 == 0, MEGA_ERR_ARG,
               "gate_qk_fwd: S=%lld must split into %lld heads of even size", (long long)S, (long long)heads);
  if (T_ == 0) return MEGA_OK;
  MEGA_REQUIRE(z && gamma && beta && freqs && q && k, MEGA_ERR_ARG, "gate_qk_fwd: null pointer argument");
  MEGA_REQUIRE(z_stride >= S, MEGA_ERR_ARG, "gate_qk_fwd: row stride %lld below the row length %lld",
               (long long)z_stride, (long long)S);
  MEGA_REQUIRE(ceil_div(T_, kRowsPerWg) < (1ll << 31), MEGA_ERR_ARG, "gate_qk_fwd: too many rows");
  hipStream_t s = (hipStream_t)stream;
  MEGA_GLUE_DISPATCH(launch_gate_qk, z, z_stride, gamma, beta, freqs, q, k, T_, S, S / heads, chunk, pos0, (float)eps,
                     s);
}

extern "C" size_t mega_gate_qk_bwd_workspace_bytes(int64_t T_, int64_t S) {
  if (T_ <= 0 || S <= 0) return 256;
  return align_up((size_t)gate_qk_bwd_wgs(T_) * 4 * (size_t)S * sizeof(float), 256);
}

extern "C" int mega_gate_qk_bwd_strided(const void* q_grad, const void* k_grad, const void* z, int64_t z_stride,
                                        const float* gamma, const float* freqs, void* z_grad, int64_t z_grad_stride,
                                        float* gamma_grad, float* beta_grad, int dtype, int64_t T_, int64_t S,
                                        int64_t heads, int64_t chunk, int64_t pos0, double eps, void* workspace,
                                        size_t workspace_bytes, void* stream) {
  MEGA_REQUIRE(known_dtype(dtype), MEGA_ERR_ARG, "gate_qk_bwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(T_ >= 0 && S >= 2 && S < (1ll << 30) && heads >= 1 && chunk >= 1 && pos0 >= 0, MEGA_ERR_ARG,
               "gate_qk_bwd: bad sizes T=%lld S=%lld heads=%lld chunk=%lld pos0=%lld", (long long)T_, (long long)S,
               (long long)heads, (long long)chunk, (long long)pos0);
  MEGA_REQUIRE(S % heads == 0 && (S / heads) % 2 == 0, MEGA_ERR_ARG,
               "gate_qk_bwd: S=%lld must split into %lld heads of even size", (long long)S, (long long)heads);
  MEGA_REQUIRE(gamma_grad && beta_grad, MEGA_ERR_ARG, "gate_qk_bwd: null pointer argument");
  hipStream_t s = (hipStream_t)stream;
  if (T_ == 0) {
    zero_async(gamma_grad, (size_t)2 * S * 4, s);
    zero_async(beta_grad, (size_t)2 * S * 4, s);
    return MEGA_OK;
  }
  MEGA_REQUIRE(q_grad && k_grad && z && gamma && freqs && z_grad, MEGA_ERR_ARG, "gate_qk_bwd: null pointer argument");
  MEGA_REQUIRE(z_stride >= S && z_grad_stride >= S, MEGA_ERR_ARG,
               "gate_qk_bwd: row stride %lld / %lld below the row length %lld", (long long)z_stride,
               (long long)z_grad_stride, (long long)S);
  const size_t need = mega_gate_qk_bwd_workspace_bytes(T_, S);
  MEGA_REQUIRE(workspace && workspace_bytes >= need && ((uintptr_t)workspace % 16) == 0, MEGA_ERR_WORKSPACE,
               "gate_qk_bwd: workspace of %zu bytes (16-byte aligned) needed", need);
  MEGA_GLUE_DISPATCH(launch_gate_qk_bwd, q_grad, k_grad, z, z_stride, gamma, freqs, z_grad, z_grad_stride, gamma_grad,
                     beta_grad, (float*)workspace, T_, S, S / heads, chunk, pos0, (float)eps, s);
}

extern "C" int mega_gate_qk_bwd(const void* q_grad, const void* k_grad, const void* z, int64_t z_stride,
                                const float* gamma, const float* freqs, void* z_grad, float* gamma_grad,
                                float* beta_grad, int dtype, int64_t T_, int64_t S, int64_t heads, int64_t chunk,
                                int64_t pos0, double eps, void* workspace, size_t workspace_bytes, void* stream) {
  return mega_gate_qk_bwd_strided(q_grad, k_grad, z, z_stride, gamma, freqs, z_grad, S, gamma_grad, beta_grad, dtype,
                                  T_, S, heads, chunk, pos0, eps, workspace, workspace_bytes, stream);
}

extern "C" int mega_gate_mul_fwd(const void* a, int64_t a_stride, const void* r, int64_t r_stride, void* y, int dtype,
                                 int64_t T_, int64_t E, void* stream) {
  MEGA_REQUIRE(known_dtype(dtype), MEGA_ERR_ARG, "gate_mul_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(T_ >= 0 && E >= 1 && E < (1ll << 30), MEGA_ERR_ARG, "gate_mul_fwd: bad sizes T=%lld E=%lld",
               (long long)T_, (long long)E);
  if (T_ == 0) return MEGA_OK;
  MEGA_REQUIRE(a && r && y, MEGA_ERR_ARG, "gate_mul_fwd: null pointer argument");
  MEGA_REQUIRE(a_stride >= E && r_stride >= E, MEGA_ERR_ARG, "gate_mul_fwd: a row stride is below the row length");
  hipStream_t s = (hipStream_t)stream;
  MEGA_GLUE_DISPATCH(launch_gate_mul, a, a_stride, r, r_stride, y, T_, E, s);
}

extern "C" int mega_gate_out_fwd(const void* residual, int64_t residual_stride, const void* u, int64_t u_stride,
                                 const void* hx, int64_t hx_stride, const void* hp, int64_t hp_stride, void* y,
                                 int dtype, int64_t T_, int64_t D, void* stream) {
  MEGA_REQUIRE(known_dtype(dtype), MEGA_ERR_ARG, "gate_out_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(T_ >= 0 && D >= 1 && D < (1ll << 30), MEGA_ERR_ARG, "gate_out_fwd: bad sizes T=%lld D=%lld",
               (long long)T_, (long long)D);
  if (T_ == 0) return MEGA_OK;
  MEGA_REQUIRE(residual && u && hx && hp && y, MEGA_ERR_ARG, "gate_out_fwd: null pointer argument");
  MEGA_REQUIRE(residual_stride >= D && u_stride >= D && hx_stride >= D && hp_stride >= D, MEGA_ERR_ARG,
               "gate_out_fwd: a row stride is below the row length");
  hipStream_t s = (hipStream_t)stream;
  MEGA_GLUE_DISPATCH(launch_gate_out, residual, residual_stride, u, u_stride, hx, hx_stride, hp, hp_stride, y, T_, D,
                     s);
}

extern "C" int mega_gate_mul_bwd_strided(const void* y_grad, const void* a, int64_t a_stride, const void* r,
                                         int64_t r_stride, void* a_grad, void* r_grad, int64_t r_grad_stride,
                                         int dtype, int64_t T_, int64_t E, void* stream) {
  MEGA_REQUIRE(known_dtype(dtype), MEGA_ERR_ARG, "gate_mul_bwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(T_ >= 0 && E >= 1 && E < (1ll << 30), MEGA_ERR_ARG, "gate_mul_bwd: bad sizes T=%lld E=%lld",
               (long long)T_, (long long)E);
  if (T_ == 0) return MEGA_OK;
  MEGA_REQUIRE(y_grad && a && r && a_grad && r_grad, MEGA_ERR_ARG, "gate_mul_bwd: null pointer argument");
  MEGA_REQUIRE(a_stride >= E && r_stride >= E && r_grad_stride >= E, MEGA_ERR_ARG,
               "gate_mul_bwd: a row stride is below the row length");
  hipStream_t s = (hipStream_t)stream;
  MEGA_GLUE_DISPATCH(launch_gate_mul_bwd, y_grad, a, a_stride, r, r_stride, a_grad, r_grad, r_grad_stride, T_, E, s);
}

extern "C" int mega_gate_mul_bwd(const void* y_grad, const void* a, int64_t a_stride, const void* r, int64_t r_stride,
                                 void* a_grad, void* r_grad, int dtype, int64_t T_, int64_t E, void* stream) {
  return mega_gate_mul_bwd_strided(y_grad, a, a_stride, r, r_stride, a_grad, r_grad, E, dtype, T_, E, stream);
}

extern "C" int mega_gate_out_bwd_strided(const void* y_grad, const void* residual, int64_t residual_stride,
                                         const void* u, int64_t u_stride, const void* hx, int64_t hx_stride,
                                         const void* hp, int64_t hp_stride, void* residual_grad, void* u_grad,
                                         int64_t u_grad_stride, void* h_grad, int64_t h_grad_stride, int dtype,
                                         int64_t T_, int64_t D, void* stream) {
  MEGA_REQUIRE(known_dtype(dtype), MEGA_ERR_ARG, "gate_out_bwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(T_ >= 0 && D >= 1 && D < (1ll << 30), MEGA_ERR_ARG, "gate_out_bwd: bad sizes T=%lld D=%lld",
               (long long)T_, (long long)D);
  if (T_ == 0) return MEGA_OK;
  MEGA_REQUIRE(y_grad && residual && u && hx && hp && residual_grad && u_grad && h_grad, MEGA_ERR_ARG,
               "gate_out_bwd: null pointer argument");
  MEGA_REQUIRE(residual_stride >= D && u_stride >= D && hx_stride >= D && hp_stride >= D && u_grad_stride >= D &&
                   h_grad_stride >= D,
               MEGA_ERR_ARG, "gate_out_bwd: a row stride is below the row length");
  hipStream_t s = (hipStream_t)stream;
  MEGA_GLUE_DISPATCH(launch_gate_out_bwd, y_grad, residual, residual_stride, u, u_stride, hx, hx_stride, hp, hp_stride,
                     residual_grad, u_grad, u_grad_stride, h_grad, h_grad_stride, T_, D, s);
}

extern "C" int mega_gate_out_bwd(const void* y_grad, const void* residual, int64_t residual_stride, const void* u,
                                 int64_t u_stride, const void* hx, int64_t hx_stride, const void* hp,
                                 int64_t hp_stride, void* residual_grad, void* u_grad, void* h_grad, int dtype,
                                 int64_t T_, int64_t D, void* stream) {
  return mega_gate_out_bwd_strided(y_grad, residual, residual_stride, u, u_stride, hx, hx_stride, hp, hp_stride,
                                   residual_grad, u_grad, D, h_grad, D, dtype, T_, D, stream);
}

extern "C" int mega_swiglu_bwd(const void* y_grad, const void* a, const void* b, void* a_grad, void* b_grad, int dtype,
                               int64_t n, void* stream) {
  MEGA_REQUIRE(known_dtype(dtype), MEGA_ERR_ARG, "swiglu_bwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(n >= 0, MEGA_ERR_ARG, "swiglu_bwd: negative size");
  if (n == 0) return MEGA_OK;
  MEGA_REQUIRE(y_grad && a && b && a_grad && b_grad, MEGA_ERR_ARG, "swiglu_bwd: null pointer argument");
  hipStream_t s = (hipStream_t)stream;
  MEGA_GLUE_DISPATCH(launch_swiglu_bwd, y_grad, a, b, a_grad, b_grad, n, s);
}
