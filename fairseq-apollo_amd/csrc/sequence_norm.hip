// SequenceNorm forward (group and per-feature variants, [B, L, H] and [B, H, L] layouts):
// the statistics of one (batch row, group) are the mean and the biased variance over all unmasked
// tokens and the group's channels; y = (x - mean) * rstd * gamma + beta, masked tokens become 0.
// Reference: fairseq/csrc/ops/sequence_norm.cc:258-372 (per feature), :531-656 (groups); the
// per-feature form is the group form with one channel per group.
//
// Three launches, all deterministic (no floating-point atomics):
//   1. moments: partial (count, mean, M2) per (row, token tile, group) for [B, L, H], per
//      (row, channel) for [B, H, L]  (sums of x and x^2 over at most a tile in fp32);
//   2. combine: one wave per (row, group) merges the partials pairwise (Chan et al.) and writes
//      mean, rstd and the row's token count;
//   3. apply: the same tiling as 1, one streaming pass.
// HBM traffic: x twice, y once.
#include "common.h"

namespace mega {
namespace {

constexpr int kThreads = 256;        // [B, H, L] kernels: one workgroup per row, rows are plentiful
constexpr int kTileThreads = 512;    // [B, L, H] tile kernel: two tiles per compute unit, four waves per SIMD
constexpr int kMaxCells = 4096;     // tokens-per-tile * groups held in LDS

struct SeqNormParams {
  const void* x;
  void* y;
  const float* gamma;
  const float* beta;
  const uint8_t* mask;
  float* part;        // [B, np, G, 3] ([B, L, H]) or [B, H, 3] ([B, H, L]): (n, mean, M2)
  int64_t* count;
  float* mean;
  float* rstd;
  int B, L, H, G, Dg, TT, nt;
  RowTiling R;
  float eps;
};

// Chan et al.: (na, ma, Ma) + (nb, mb, Mb)
__device__ __forceinline__ void merge3(float& n, float& m, float& M2, float nb, float mb, float Mb) {
  const float nt = n + nb;
  if (nt > 0.f) {
    const float d = mb - m, f = nb / nt;
    m = fmaf(d, f, m);
    M2 = M2 + Mb + d * d * n * f;
  }
  n = nt;
}

// ---------------------------------------------------------------- [B, L, H]: channels contiguous
// APPLY = false: partial moments of the tile; APPLY = true: normalise the tile.
template <typename T, int VEC, bool APPLY>
__global__ __launch_bounds__(kTileThreads) void seqnorm_blh_kernel(const SeqNormParams P) {
  using V = Vec<T, VEC>;
  extern __shared__ float smem[];
  const int G = P.G, H = P.H, TT = P.TT, Dg = P.Dg;
  float* s_a = smem;                  // moments: sum per (token, group);  apply: mean per group
  float* s_b = s_a + (APPLY ? G : TT * G);   // moments: sum of squares;  apply: rstd per group
  int* s_mask = (int*)(s_b + (APPLY ? G : TT * G));
  const int tid = threadIdx.x;
  const int tile = blockIdx.x % P.nt, b = blockIdx.x / P.nt;
  const int t0 = tile * TT;
  const int ntok = min(TT, P.L - t0);
  const T* x = (const T*)P.x + ((size_t)b * P.L + t0) * H;
  for (int tok = tid; tok < TT; tok += kTileThreads)
    s_mask[tok] = (tok >= ntok) || (P.mask && P.mask[(size_t)b * P.L + t0 + tok]);
  if (APPLY)
    for (int g = tid; g < G; g += kTileThreads) {
      s_a[g] = P.mean[(size_t)b * G + g];
      s_b[g] = P.rstd[(size_t)b * G + g];
    }
  __syncthreads();
  const int items = ntok * P.R.slots;
  const int span = VEC * P.R.PER;
  for (int i0 = 0; i0 < items; i0 += kTileThreads) {
    const int i = i0 + tid;
    const bool live = i < items;
    int tok, slot;
    split_item(P.R, live ? i : 0, tok, slot);
    const int g = slot >> P.R.lpg_shift;
    const int c0 = g * Dg + (slot - (g << P.R.lpg_shift)) * span;
    if (APPLY) {
      if (live) {
        const float mu = s_a[g], r = s_b[g];
        const bool keep = !s_mask[tok];
        T* y = (T*)P.y + ((size_t)b * P.L + t0 + tok) * H;
        for (int k = 0; k < P.R.PER; ++k) {
          const int c = c0 + k * VEC;
          const V xv = *(const V*)(x + (size_t)tok * H + c);
          float gw[VEC], bw[VEC];
          load_params<VEC>(P.gamma + c, gw);
          load_params<VEC>(P.beta + c, bw);
          V o;
#pragma unroll
          for (int e = 0; e < VEC; ++e)
            o.v[e] = from_float<T>(keep ? fmaf((to_float(xv.v[e]) - mu) * r, gw[e], bw[e]) : 0.f);
          *(V*)(y + c) = o;
        }
      }
    } else {
      float s1 = 0.f, s2 = 0.f;
      if (live && !s_mask[tok]) {
        for (int k = 0; k < P.R.PER; ++k) {
          const V xv = *(const V*)(x + (size_t)tok * H + c0 + k * VEC);
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const float f = to_float(xv.v[e]);
            s1 += f;
            s2 = fmaf(f, f, s2);
          }
        }
      }
      for (int o = 1; o < P.R.LPG; o <<= 1) {
        s1 += __shfl_xor(s1, o);
        s2 += __shfl_xor(s2, o);
      }
      if (live && slot == (g << P.R.lpg_shift)) {
        s_a[tok * G + g] = s1;
        s_b[tok * G + g] = s2;
      }
    }
  }
  if (!APPLY) {
    __syncthreads();
    int nkeep = 0;
    for (int tok = 0; tok < ntok; ++tok) nkeep += s_mask[tok] ? 0 : 1;
    for (int g = tid; g < G; g += kTileThreads) {
      float s1 = 0.f, s2 = 0.f;
      for (int tok = 0; tok < ntok; ++tok) {      // masked tokens hold zeros
        s1 += s_a[tok * G + g];
        s2 += s_b[tok * G + g];
      }
      const float n = (float)nkeep * (float)Dg;
      const float m = n > 0.f ? s1 / n : 0.f;
      float* dst = P.part + (((size_t)b * P.nt + tile) * G + g) * 3;
      dst[0] = n;
      dst[1] = m;
      dst[2] = fmaxf(s2 - n * m * m, 0.f);
    }
  }
}

// ---------------------------------------------------------------- [B, H, L]: time contiguous
// one workgroup per (row, channel)
template <typename T, int VEC, bool APPLY>
__global__ __launch_bounds__(kThreads) void seqnorm_bhl_kernel(const SeqNormParams P) {
  using V = Vec<T, VEC>;
  __shared__ float s_red[2][kThreads / 64];
  __shared__ int s_cnt[kThreads / 64];
  const int tid = threadIdx.x;
  const int c = blockIdx.x % P.H, b = blockIdx.x / P.H;
  const T* x = (const T*)P.x + ((size_t)b * P.H + c) * P.L;
  const uint8_t* mk = P.mask ? P.mask + (size_t)b * P.L : nullptr;
  if (APPLY) {
    const int g = c / P.Dg;
    const float mu = P.mean[(size_t)b * P.G + g], r = P.rstd[(size_t)b * P.G + g];
    const float w = P.gamma[c] * r, sh = P.beta[c] - mu * w;
    T* y = (T*)P.y + ((size_t)b * P.H + c) * P.L;
    for (int t = tid * VEC; t < P.L; t += kThreads * VEC) {
      const V xv = *(const V*)(x + t);
      V o;
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        o.v[e] = from_float<T>((mk && mk[t + e]) ? 0.f : fmaf(to_float(xv.v[e]), w, sh));
      *(V*)(y + t) = o;
    }
    return;
  }
  float s1 = 0.f, s2 = 0.f;
  int n = 0;
  for (int t = tid * VEC; t < P.L; t += kThreads * VEC) {
    const V xv = *(const V*)(x + t);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      if (!(mk && mk[t + e])) {
        const float f = to_float(xv.v[e]);
        s1 += f;
        s2 = fmaf(f, f, s2);
        ++n;
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    s1 += __shfl_xor(s1, o);
    s2 += __shfl_xor(s2, o);
    n += __shfl_xor(n, o);
  }
  if ((tid & 63) == 0) { s_red[0][tid >> 6] = s1; s_red[1][tid >> 6] = s2; s_cnt[tid >> 6] = n; }
  __syncthreads();
  if (tid == 0) {
    float a1 = 0.f, a2 = 0.f;
    int nn = 0;
    for (int k = 0; k < kThreads / 64; ++k) { a1 += s_red[0][k]; a2 += s_red[1][k]; nn += s_cnt[k]; }
    const float fn = (float)nn, m = nn > 0 ? a1 / fn : 0.f;
    float* dst = P.part + ((size_t)b * P.H + c) * 3;
    dst[0] = fn;
    dst[1] = m;
    dst[2] = fmaxf(a2 - fn * m * m, 0.f);
  }
}

// one wave per (row, group): partial p of the group sits at part[(b * np_outer + p_outer) ...];
// both layouts are walked with (first, stride, count).
__global__ __launch_bounds__(64) void seqnorm_combine_kernel(const SeqNormParams P, int np, int64_t row_stride,
                                                            int64_t g_stride, int64_t p_stride) {
  const int i = blockIdx.x;
  const int b = i / P.G, g = i - b * P.G;
  const int lane = threadIdx.x;
  const float* base = P.part + (size_t)b * row_stride + (size_t)g * g_stride;
  float n = 0.f, m = 0.f, M2 = 0.f;
  for (int p = lane; p < np; p += 64) {
    const float* q = base + (size_t)p * p_stride;
    merge3(n, m, M2, q[0], q[1], q[2]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float nb = __shfl_xor(n, o), mb = __shfl_xor(m, o), Mb = __shfl_xor(M2, o);
    // both partners must end with the same bits: merge in a fixed (low lane, high lane) order
    float an = (lane & o) ? nb : n, am = (lane & o) ? mb : m, aM = (lane & o) ? Mb : M2;
    const float bn = (lane & o) ? n : nb, bm = (lane & o) ? m : mb, bM = (lane & o) ? M2 : Mb;
    merge3(an, am, aM, bn, bm, bM);
    n = an; m = am; M2 = aM;
  }
  if (lane == 0) {
    const float var = n > 0.f ? M2 / n : 0.f;
    P.mean[i] = m;
    P.rstd[i] = rsqrtf(var + P.eps);
    if (g == 0) P.count[b] = (int64_t)llrintf(n / (float)P.Dg);
  }
}

// ---------------------------------------------------------------- backward, [B, H, L]
// Reference: sequence_norm.cc:756-842 (groups, time last), :459-529 (per feature).  Per (row, channel)
// ds = sum dy x, db = sum dy over the unmasked tokens; per (row, group) dsw = sum ds gamma,
// dbw = sum db gamma, n = count * D, dv = r^3 (u dbw - dsw) / 2, du = -r dbw;
// dx = r gamma dy + (2 (x - u) dv + du) / n;  dgamma = sum_rows r (ds - u db), dbeta = sum_rows db.
struct SeqBwdParams {
  const void* dy;
  const void* x;
  void* dx;
  const int64_t* count;
  const float* mean;
  const float* rstd;
  const float* gamma;
  const uint8_t* mask;
  float* part;     // [B, H, 2]  (ds, db)
  float* coef;     // [B, G, 2]  (2 dv / n, du / n)
  float* gamma_grad;
  float* beta_grad;
  int B, L, H, G, Dg;
};

template <typename T, int VEC, bool APPLY>
__global__ __launch_bounds__(kThreads) void seqnorm_bwd_bhl_kernel(const SeqBwdParams P) {
  using V = Vec<T, VEC>;
  __shared__ float s_red[2][kThreads / 64];
  const int tid = threadIdx.x;
  const int c = blockIdx.x % P.H, b = blockIdx.x / P.H;
  const T* x = (const T*)P.x + ((size_t)b * P.H + c) * P.L;
  const T* dy = (const T*)P.dy + ((size_t)b * P.H + c) * P.L;
  const uint8_t* mk = P.mask ? P.mask + (size_t)b * P.L : nullptr;
  if (APPLY) {
    const int g = c / P.Dg;
    const float u = P.mean[(size_t)b * P.G + g], r = P.rstd[(size_t)b * P.G + g];
    const float a1 = P.coef[((size_t)b * P.G + g) * 2], a0 = P.coef[((size_t)b * P.G + g) * 2 + 1];
    const float rw = r * P.gamma[c], sh = a0 - a1 * u;
    T* dx = (T*)P.dx + ((size_t)b * P.H + c) * P.L;
    for (int t = tid * VEC; t < P.L; t += kThreads * VEC) {
      const V xv = *(const V*)(x + t);
      const V gv = *(const V*)(dy + t);
      V o;
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        o.v[e] = from_float<T>((mk && mk[t + e]) ? 0.f : fmaf(rw, to_float(gv.v[e]), fmaf(a1, to_float(xv.v[e]), sh)));
      *(V*)(dx + t) = o;
    }
    return;
  }
  float ds = 0.f, db = 0.f;
  for (int t = tid * VEC; t < P.L; t += kThreads * VEC) {
    const V xv = *(const V*)(x + t);
    const V gv = *(const V*)(dy + t);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      if (!(mk && mk[t + e])) {
        const float d = to_float(gv.v[e]);
        ds = fmaf(d, to_float(xv.v[e]), ds);
        db += d;
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    ds += __shfl_xor(ds, o);
    db += __shfl_xor(db, o);
  }
  if ((tid & 63) == 0) { s_red[0][tid >> 6] = ds; s_red[1][tid >> 6] = db; }
  __syncthreads();
  if (tid == 0) {
    float a = 0.f, d = 0.f;
    for (int k = 0; k < kThreads / 64; ++k) { a += s_red[0][k]; d += s_red[1][k]; }
    P.part[((size_t)b * P.H + c) * 2] = a;
    P.part[((size_t)b * P.H + c) * 2 + 1] = d;
  }
}

// one wave per (row, group): the two coefficients of dx
__global__ __launch_bounds__(64) void seqnorm_bwd_combine_kernel(const SeqBwdParams P) {
  const int i = blockIdx.x;
  const int b = i / P.G, g = i - b * P.G;
  const int lane = threadIdx.x;
  float dsw = 0.f, dbw = 0.f;
  for (int k = lane; k < P.Dg; k += 64) {
    const int c = g * P.Dg + k;
    const float w = P.gamma[c];
    dsw = fmaf(P.part[((size_t)b * P.H + c) * 2], w, dsw);
    dbw = fmaf(P.part[((size_t)b * P.H + c) * 2 + 1], w, dbw);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    dsw += __shfl_xor(dsw, o);
    dbw += __shfl_xor(dbw, o);
  }
  if (lane == 0) {
    const float n = (float)P.count[b] * (float)P.Dg;
    const float u = P.mean[i], r = P.rstd[i];
    const float dv = 0.5f * r * r * r * (u * dbw - dsw), du = -r * dbw;
    P.coef[(size_t)i * 2] = n > 0.f ? 2.0f * dv / n : 0.f;
    P.coef[(size_t)i * 2 + 1] = n > 0.f ? du / n : 0.f;
  }
}

// thread per channel: parameter gradients summed over the rows in order
__global__ void seqnorm_bwd_param_kernel(const SeqBwdParams P) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= P.H) return;
  const int g = c / P.Dg;
  float gw = 0.f, gb = 0.f;
  for (int b = 0; b < P.B; ++b) {
    const float ds = P.part[((size_t)b * P.H + c) * 2], db = P.part[((size_t)b * P.H + c) * 2 + 1];
    gw = fmaf(P.rstd[(size_t)b * P.G + g], ds - P.mean[(size_t)b * P.G + g] * db, gw);
    gb += db;
  }
  P.gamma_grad[c] = gw;
  P.beta_grad[c] = gb;
}

template <typename T>
int launch_seqnorm_bwd(const SeqBwdParams& P, bool vec, hipStream_t s) {
  constexpr int FULL = 16 / (int)sizeof(T);
  const dim3 grid((unsigned)(P.B * P.H));
  if (vec) hipLaunchKernelGGL((seqnorm_bwd_bhl_kernel<T, FULL, false>), grid, dim3(kThreads), 0, s, P);
  else hipLaunchKernelGGL((seqnorm_bwd_bhl_kernel<T, 1, false>), grid, dim3(kThreads), 0, s, P);
  MEGA_CHECK_LAUNCH("sequence_norm_bwd (sums)");
  hipLaunchKernelGGL(seqnorm_bwd_combine_kernel, dim3((unsigned)(P.B * P.G)), dim3(64), 0, s, P);
  MEGA_CHECK_LAUNCH("sequence_norm_bwd (combine)");
  hipLaunchKernelGGL(seqnorm_bwd_param_kernel, dim3((unsigned)ceil_div(P.H, 256)), dim3(256), 0, s, P);
  MEGA_CHECK_LAUNCH("sequence_norm_bwd (parameters)");
  if (vec) hipLaunchKernelGGL((seqnorm_bwd_bhl_kernel<T, FULL, true>), grid, dim3(kThreads), 0, s, P);
  else hipLaunchKernelGGL((seqnorm_bwd_bhl_kernel<T, 1, true>), grid, dim3(kThreads), 0, s, P);
  MEGA_CHECK_LAUNCH("sequence_norm_bwd (dx)");
  return MEGA_OK;
}

struct SeqGeom {
  int tt, nt, vec;
  size_t part_bytes;
};

bool seq_geometry(int dtype, int64_t B, int64_t L, int64_t H, int64_t G, int length_last, SeqGeom* g) {
  if (B * L >= (int64_t)1 << 31 || B * H >= (int64_t)1 << 31 || G > kMaxCells) return false;
  const int full = dtype == MEGA_F32 ? 4 : 8;
  if (length_last) {
    g->vec = (L % full == 0) ? full : 1;
    g->tt = 0; g->nt = 0;
    g->part_bytes = align_up((size_t)B * H * 12, 256);
    return true;
  }
  const int64_t Dg = H / G;
  g->vec = (Dg % full == 0) ? full : 1;
  int tt = (int)(kMaxCells / G);
  if (tt > 16) tt = 16;
  if (tt < 1) tt = 1;
  g->tt = tt;
  g->nt = (int)ceil_div(L, tt);
  if (B * g->nt >= (int64_t)1 << 31) return false;
  g->part_bytes = align_up((size_t)B * g->nt * G * 12, 256);
  return true;
}

template <typename T>
int launch_seqnorm(SeqNormParams P, const SeqGeom& g, int length_last, bool aligned, hipStream_t s) {
  constexpr int FULL = 16 / (int)sizeof(T);
  const bool vec = g.vec == FULL && aligned;
  if (length_last) {
    const dim3 grid((unsigned)(P.B * P.H));
    if (vec) hipLaunchKernelGGL((seqnorm_bhl_kernel<T, FULL, false>), grid, dim3(kThreads), 0, s, P);
    else hipLaunchKernelGGL((seqnorm_bhl_kernel<T, 1, false>), grid, dim3(kThreads), 0, s, P);
    MEGA_CHECK_LAUNCH("sequence_norm_fwd (moments)");
    hipLaunchKernelGGL(seqnorm_combine_kernel, dim3((unsigned)(P.B * P.G)), dim3(64), 0, s, P, P.Dg,
                       (int64_t)P.H * 3, (int64_t)P.Dg * 3, (int64_t)3);
    MEGA_CHECK_LAUNCH("sequence_norm_fwd (combine)");
    if (vec) hipLaunchKernelGGL((seqnorm_bhl_kernel<T, FULL, true>), grid, dim3(kThreads), 0, s, P);
    else hipLaunchKernelGGL((seqnorm_bhl_kernel<T, 1, true>), grid, dim3(kThreads), 0, s, P);
    MEGA_CHECK_LAUNCH("sequence_norm_fwd (apply)");
    return MEGA_OK;
  }
  const dim3 grid((unsigned)(P.B * P.nt));
  const size_t lds_m = ((size_t)2 * P.TT * P.G + P.TT) * 4, lds_a = ((size_t)2 * P.G + P.TT) * 4;
  if (vec) hipLaunchKernelGGL((seqnorm_blh_kernel<T, FULL, false>), grid, dim3(kTileThreads), lds_m, s, P);
  else hipLaunchKernelGGL((seqnorm_blh_kernel<T, 1, false>), grid, dim3(kTileThreads), lds_m, s, P);
  MEGA_CHECK_LAUNCH("sequence_norm_fwd (moments)");
  hipLaunchKernelGGL(seqnorm_combine_kernel, dim3((unsigned)(P.B * P.G)), dim3(64), 0, s, P, P.nt,
                     (int64_t)P.nt * P.G * 3, (int64_t)3, (int64_t)P.G * 3);
  MEGA_CHECK_LAUNCH("sequence_norm_fwd (combine)");
  if (vec) hipLaunchKernelGGL((seqnorm_blh_kernel<T, FULL, true>), grid, dim3(kTileThreads), lds_a, s, P);
  else hipLaunchKernelGGL((seqnorm_blh_kernel<T, 1, true>), grid, dim3(kTileThreads), lds_a, s, P);
  MEGA_CHECK_LAUNCH("sequence_norm_fwd (apply)");
  return MEGA_OK;
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" size_t mega_sequence_norm_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t H, int64_t G,
                                                     int length_last) {
  SeqGeom g;
  if (B <= 0 || L <= 0 || H <= 0 || G <= 0 || H % G != 0 || !seq_geometry(dtype, B, L, H, G, length_last, &g))
    return 256;
  return g.part_bytes;
}

extern "C" int mega_group_sequence_norm_fwd(const void* x, void* y, int dtype, const float* gamma, const float* beta,
                                            const uint8_t* mask, int64_t B, int64_t L, int64_t H, int64_t G,
                                            double eps, int length_last, int64_t* count, float* mean, float* rstd,
                                            void* workspace, size_t workspace_bytes, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "sequence_norm_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && L >= 0 && H > 0 && G > 0 && H % G == 0, MEGA_ERR_ARG,
               "sequence_norm_fwd: bad shape B=%ld L=%ld H=%ld G=%ld", (long)B, (long)L, (long)H, (long)G);
  if (B == 0) return MEGA_OK;
  MEGA_REQUIRE(gamma && beta && count && mean && rstd && (L == 0 || (x && y)), MEGA_ERR_ARG,
               "sequence_norm_fwd: null pointer argument");
  SeqGeom g;
  MEGA_REQUIRE(seq_geometry(dtype, B, L > 0 ? L : 1, H, G, length_last, &g), MEGA_ERR_UNSUPPORTED,
               "sequence_norm_fwd: shape outside the supported envelope (G <= %d)", kMaxCells);
  MEGA_REQUIRE(L > 0, MEGA_ERR_UNSUPPORTED, "sequence_norm_fwd: empty sequences have no statistics");
  MEGA_REQUIRE(workspace && workspace_bytes >= g.part_bytes, MEGA_ERR_WORKSPACE,
               "sequence_norm_fwd: workspace of %zu bytes needed", g.part_bytes);
  SeqNormParams P;
  P.x = x; P.y = y; P.gamma = gamma; P.beta = beta; P.mask = mask; P.part = (float*)workspace;
  P.count = count; P.mean = mean; P.rstd = rstd;
  P.B = (int)B; P.L = (int)L; P.H = (int)H; P.G = (int)G; P.Dg = (int)(H / G); P.TT = g.tt; P.nt = g.nt;
  P.eps = (float)eps;
  const bool aligned = ((((uintptr_t)x | (uintptr_t)y | (uintptr_t)gamma | (uintptr_t)beta) % 16) == 0);
  if (!aligned) g.vec = 1;                 // element-wise tiling when a buffer is not 16-byte aligned
  P.R = make_row_tiling(G, H / G, length_last ? 1 : g.vec);
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MEGA_F32: return launch_seqnorm<float>(P, g, length_last, aligned, s);
    case MEGA_BF16: return launch_seqnorm<bf16_t>(P, g, length_last, aligned, s);
    default: return launch_seqnorm<f16_t>(P, g, length_last, aligned, s);
  }
}

extern "C" int mega_sequence_norm_fwd(const void* x, void* y, int dtype, const float* gamma, const float* beta,
                                      const uint8_t* mask, int64_t B, int64_t L, int64_t H, double eps,
                                      int length_last, int64_t* count, float* mean, float* rstd, void* workspace,
                                      size_t workspace_bytes, void* stream) {
  return mega_group_sequence_norm_fwd(x, y, dtype, gamma, beta, mask, B, L, H, H, eps, length_last, count, mean,
                                      rstd, workspace, workspace_bytes, stream);
}

extern "C" size_t mega_sequence_norm_bwd_workspace_bytes(int64_t B, int64_t H, int64_t G) {
  if (B <= 0 || H <= 0 || G <= 0) return 256;
  return align_up((size_t)B * H * 8, 256) + align_up((size_t)B * G * 8, 256);
}

extern "C" int mega_group_sequence_norm_bwd(const void* y_grad, const void* x, int dtype, const int64_t* count,
                                            const float* mean, const float* rstd, const float* gamma,
                                            const uint8_t* mask, int64_t B, int64_t L, int64_t H, int64_t G,
                                            void* x_grad, float* gamma_grad, float* beta_grad, void* workspace,
                                            size_t workspace_bytes, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "sequence_norm_bwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && L > 0 && H > 0 && G > 0 && H % G == 0, MEGA_ERR_ARG,
               "sequence_norm_bwd: bad shape B=%ld L=%ld H=%ld G=%ld", (long)B, (long)L, (long)H, (long)G);
  MEGA_REQUIRE(B * H < (int64_t)1 << 31 && L < (int64_t)1 << 30, MEGA_ERR_UNSUPPORTED,
               "sequence_norm_bwd: shape too large");
  MEGA_REQUIRE(gamma_grad && beta_grad, MEGA_ERR_ARG, "sequence_norm_bwd: null gradient output");
  hipStream_t s = (hipStream_t)stream;
  if (B == 0) {
    zero_async(gamma_grad, (size_t)H * 4, s);
    zero_async(beta_grad, (size_t)H * 4, s);
    return MEGA_OK;
  }
  MEGA_REQUIRE(y_grad && x && x_grad && count && mean && rstd && gamma, MEGA_ERR_ARG,
               "sequence_norm_bwd: null pointer argument");
  const size_t need = mega_sequence_norm_bwd_workspace_bytes(B, H, G);
  MEGA_REQUIRE(workspace && workspace_bytes >= need, MEGA_ERR_WORKSPACE,
               "sequence_norm_bwd: workspace of %zu bytes needed", need);
  SeqBwdParams P;
  P.dy = y_grad; P.x = x; P.dx = x_grad; P.count = count; P.mean = mean; P.rstd = rstd; P.gamma = gamma; P.mask = mask;
  P.part = (float*)workspace;
  P.coef = (float*)((char*)workspace + align_up((size_t)B * H * 8, 256));
  P.gamma_grad = gamma_grad; P.beta_grad = beta_grad;
  P.B = (int)B; P.L = (int)L; P.H = (int)H; P.G = (int)G; P.Dg = (int)(H / G);
  const int full = dtype == MEGA_F32 ? 4 : 8;
  const bool vec = L % full == 0 && ((((uintptr_t)y_grad | (uintptr_t)x | (uintptr_t)x_grad) % 16) == 0);
  switch (dtype) {
    case MEGA_F32: return launch_seqnorm_bwd<float>(P, vec, s);
    case MEGA_BF16: return launch_seqnorm_bwd<bf16_t>(P, vec, s);
    default: return launch_seqnorm_bwd<f16_t>(P, vec, s);
  }
}
