// TimestepNorm forward (group variant): cumulative per-group mean / variance over time
// with a carried (count, mean, var) state, one pass over x.
//
// Semantics follow the CPU implementation of the reference,
// fairseq/csrc/ops/timestep_norm.cc:218-316 (moments of each (token, group), then a
// WelfordCombine of the running state with one step per unmasked token,
// fairseq/csrc/utils.h:66-76).
//
// Design (one launch):
//   * a workgroup owns one tile = TT consecutive tokens of one batch row, i.e. one
//     contiguous block of TT*H elements that it reads once into registers;
//   * it reduces the block to per-(token, group) moments in LDS, scans them over its
//     TT tokens from a zero state and publishes the tile aggregate;
//   * it then waits until every earlier tile of the same batch row has published,
//     folds prior state + earlier aggregates into its carry-in, finishes the
//     per-token running statistics and writes the normalised block.
//   Tiles are handed out by an atomic ticket in time-major order, so a tile only ever
//   waits for tiles whose workgroups are already resident; the wait is bounded and
//   sets an error word instead of spinning forever.
#include "common.h"

namespace mega {

namespace {

constexpr int kThreads = 256;
constexpr int kNV = 16;                       // vectors kept in registers per thread
constexpr int kPartCap = kThreads * kNV;      // vectors per tile
constexpr uint32_t kSpinLimit = 1u << 22;

struct TsnHeader {
  uint32_t ticket;
  uint32_t done;
  uint32_t error;
  uint32_t pad;
};

struct TsnParams {
  const void* x;
  void* y;
  const int64_t* prev_count;
  const float* prev_mean;
  const float* prev_var;
  const float* gamma;
  const float* beta;
  const uint8_t* mask;
  int64_t* count;
  float* mean;
  float* var;
  float* group_mean;
  float* cummean;
  float* cumrstd;
  TsnHeader* hdr;
  uint32_t* flags;   // [B*ntiles]
  uint32_t* tcnt;    // [B*ntiles] unmasked tokens per tile
  float* agg;        // [B*ntiles*G*2] (mean, var) of the tile
  int B, L, H, G;
  int TT, ntiles;
  int TPT;           // vectors per token
  int LPG;           // vectors per group
  float eps;
};

template <typename T, int VEC, bool HOIST>
__global__ __launch_bounds__(kThreads) void group_tsn_kernel(const TsnParams P) {
  extern __shared__ float smem[];
  float* part = smem;                              // [kPartCap]
  float* s_mean = part + kPartCap;                 // [TT*G]
  float* s_var = s_mean + (size_t)P.TT * P.G;      // [TT*G]
  float* s_carry = s_var + (size_t)P.TT * P.G;     // [3*G]
  float* s_slot = s_carry + 3 * (size_t)P.G;       // [3*max(G,256)]
  float* s_lcnt = s_slot + 3 * (size_t)(P.G > kThreads ? P.G : kThreads);  // [TT]
  uint8_t* s_mask = (uint8_t*)(s_lcnt + P.TT);     // [TT]
  __shared__ uint32_t s_ticket;
  __shared__ uint32_t s_prevcnt;
  __shared__ uint32_t s_last;

  const int tid = threadIdx.x;
  if (tid == 0) {
    s_ticket = atomicAdd(&P.hdr->ticket, 1u);
    s_prevcnt = 0;
  }
  __syncthreads();
  const int ticket = (int)s_ticket;
  const int tile = ticket / P.B;
  const int b = ticket - tile * P.B;
  const int t0 = tile * P.TT;
  const int nt = min(P.TT, P.L - t0);
  const int nvec = nt * P.TPT;
  const int G = P.G, TPT = P.TPT, LPG = P.LPG;
  const float inv_dg = 1.0f / (float)(LPG * VEC);

  using V = Vec<T, VEC>;
  const V* xin = (const V*)P.x + ((size_t)b * P.L + t0) * TPT;
  V* yout = (V*)P.y + ((size_t)b * P.L + t0) * TPT;

  // ---- load the tile (one contiguous block) and the mask bytes
  V xv[kNV];
#pragma unroll
  for (int j = 0; j < kNV; ++j) {
    const int v = j * kThreads + tid;
    if (v < nvec) xv[j] = xin[v];
  }
  for (int t = tid; t < nt; t += kThreads)
    s_mask[t] = P.mask ? (P.mask[(size_t)b * P.L + t0 + t] != 0) : 0;

  // ---- phase 1: group means
#pragma unroll
  for (int j = 0; j < kNV; ++j) {
    const int v = j * kThreads + tid;
    if (v < nvec) {
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < VEC; ++i) s += to_float(xv[j].v[i]);
      part[v] = s;
    }
  }
  __syncthreads();
  for (int item = tid; item < nt * G; item += kThreads) {
    const int tok = item / G, g = item - tok * G;
    const float* pp = part + tok * TPT + g * LPG;
    float s = 0.f;
    for (int i = 0; i < LPG; ++i) s += pp[i];
    s_mean[item] = s * inv_dg;
  }
  __syncthreads();
  // ---- phase 2: group variances around the group mean
#pragma unroll
  for (int j = 0; j < kNV; ++j) {
    const int v = j * kThreads + tid;
    if (v < nvec) {
      const int tok = v / TPT;
      const int g = (v - tok * TPT) / LPG;
      const float m = s_mean[tok * G + g];
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float d = to_float(xv[j].v[i]) - m;
        s += d * d;
      }
      part[v] = s;
    }
  }
  __syncthreads();
  for (int item = tid; item < nt * G; item += kThreads) {
    const int tok = item / G, g = item - tok * G;
    const float* pp = part + tok * TPT + g * LPG;
    float s = 0.f;
    for (int i = 0; i < LPG; ++i) s += pp[i];
    s_var[item] = s * inv_dg;
  }
  __syncthreads();

  // ---- phase 3: scan over the tile's tokens from a zero state; publish the aggregate
  const size_t tslot = (size_t)b * P.ntiles + tile;
  for (int g = tid; g < G; g += kThreads) {
    Moments st = {0.f, 0.f, 0.f};
    for (int tok = 0; tok < nt; ++tok) {
      const float gm = s_mean[tok * G + g];
      const float gv = s_var[tok * G + g];
      if (P.group_mean) P.group_mean[((size_t)b * P.L + t0 + tok) * G + g] = gm;
      if (!s_mask[tok]) st = combine(st, Moments{1.f, gm, gv});
      s_mean[tok * G + g] = st.mean;
      s_var[tok * G + g] = st.var;
      if (g == 0) s_lcnt[tok] = st.n;
    }
    publish_f32(&P.agg[(tslot * G + g) * 2 + 0], st.mean);
    publish_f32(&P.agg[(tslot * G + g) * 2 + 1], st.var);
    if (g == 0) publish_u32(&P.tcnt[tslot], (uint32_t)st.n);
  }
  __threadfence();
  __syncthreads();
  if (tid == 0) release_flag(&P.flags[tslot], 1u);

  // ---- phase 4: wait for the earlier tiles of this row, fold them into the carry-in
  for (int p = tid; p < tile; p += kThreads) {
    const uint32_t* f = &P.flags[(size_t)b * P.ntiles + p];
    uint32_t spins = 0;
    while (acquire_flag(f) == 0u) {
      __builtin_amdgcn_s_sleep(2);
      if (++spins > kSpinLimit) {
        publish_u32(&P.hdr->error, 1u);
        break;
      }
    }
    atomicAdd(&s_prevcnt, fetch_u32(&P.tcnt[(size_t)b * P.ntiles + p]));
  }
  __syncthreads();
  const int NS = G >= kThreads ? 1 : kThreads / G;
  for (int item = tid; item < G * NS; item += kThreads) {
    const int slot = item / G, g = item - slot * G;
    Moments st = {0.f, 0.f, 0.f};
    for (int p = slot; p < tile; p += NS) {
      const size_t ps = (size_t)b * P.ntiles + p;
      Moments a;
      a.n = (float)fetch_u32(&P.tcnt[ps]);
      a.mean = fetch_f32(&P.agg[(ps * G + g) * 2 + 0]);
      a.var = fetch_f32(&P.agg[(ps * G + g) * 2 + 1]);
      st = combine(st, a);
    }
    s_slot[item * 3 + 0] = st.n;
    s_slot[item * 3 + 1] = st.mean;
    s_slot[item * 3 + 2] = st.var;
  }
  __syncthreads();
  for (int g = tid; g < G; g += kThreads) {
    Moments st = {(float)P.prev_count[b], P.prev_mean[(size_t)b * G + g], P.prev_var[(size_t)b * G + g]};
    for (int slot = 0; slot < NS; ++slot) {
      const int item = slot * G + g;
      st = combine(st, Moments{s_slot[item * 3 + 0], s_slot[item * 3 + 1], s_slot[item * 3 + 2]});
    }
    s_carry[g * 3 + 0] = st.n;
    s_carry[g * 3 + 1] = st.mean;
    s_carry[g * 3 + 2] = st.var;
  }
  __syncthreads();

  // ---- phase 5: running statistics of every token of the tile
  const bool last_tile = tile == P.ntiles - 1;
  for (int item = tid; item < nt * G; item += kThreads) {
    const int tok = item / G, g = item - tok * G;
    const Moments c = {s_carry[g * 3 + 0], s_carry[g * 3 + 1], s_carry[g * 3 + 2]};
    const Moments st = combine(c, Moments{s_lcnt[tok], s_mean[item], s_var[item]});
    const float rstd = 1.0f / sqrtf(st.var + P.eps);
    s_mean[item] = st.mean;
    s_var[item] = rstd;
    const size_t o = ((size_t)b * P.L + t0 + tok) * G + g;
    if (P.cummean) P.cummean[o] = st.mean;
    if (P.cumrstd) P.cumrstd[o] = rstd;
    if (last_tile && tok == nt - 1) {
      P.mean[(size_t)b * G + g] = st.mean;
      P.var[(size_t)b * G + g] = st.var;
    }
  }
  if (last_tile && tid == 0)
    P.count[b] = P.prev_count[b] + (int64_t)s_prevcnt + (int64_t)s_lcnt[nt - 1];
  __syncthreads();

  // ---- phase 6: normalise and store
  float gam[VEC], bet[VEC];
  if (HOIST) {
    const int f0 = (tid % TPT) * VEC;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      gam[i] = P.gamma[f0 + i];
      bet[i] = P.beta[f0 + i];
    }
  }
#pragma unroll
  for (int j = 0; j < kNV; ++j) {
    const int v = j * kThreads + tid;
    if (v < nvec) {
      const int tok = v / TPT;
      const int vi = v - tok * TPT;
      const int g = vi / LPG;
      const float m = s_mean[tok * G + g];
      const float r = s_var[tok * G + g];
      const bool masked = s_mask[tok] != 0;
      if (!HOIST) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          gam[i] = P.gamma[vi * VEC + i];
          bet[i] = P.beta[vi * VEC + i];
        }
      }
      V out;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float val = (to_float(xv[j].v[i]) - m) * r * gam[i] + bet[i];
        out.v[i] = from_float<T>(masked ? 0.f : val);
      }
      yout[v] = out;
    }
  }

  // ---- retire: the last workgroup to finish leaves the workspace zero-filled
  __syncthreads();
  if (tid == 0) {
    const uint32_t total = (uint32_t)(P.B * P.ntiles);
    const uint32_t prev = atomicAdd(&P.hdr->done, 1u);
    s_last = (prev == total - 1) ? 1u : 0u;
  }
  __syncthreads();
  if (s_last) {
    for (int i = tid; i < P.B * P.ntiles; i += kThreads) publish_u32(&P.flags[i], 0u);
    if (tid == 0) {
      publish_u32(&P.hdr->ticket, 0u);
      publish_u32(&P.hdr->done, 0u);
    }
  }
}

// Per-feature variant (every feature its own group): the running state is updated with
// WelfordUpdate per element, fairseq/csrc/ops/timestep_norm.cc:23-103
// (fairseq/csrc/utils.h:55-64).  One thread per (batch row, feature) walks the time axis;
// consecutive threads read consecutive features, so every access is coalesced.
template <typename T>
__global__ __launch_bounds__(kThreads) void feature_tsn_kernel(
    const T* __restrict__ x, T* __restrict__ y, const int64_t* __restrict__ prev_count,
    const float* __restrict__ prev_mean, const float* __restrict__ prev_var,
    const float* __restrict__ gamma, const float* __restrict__ beta,
    const uint8_t* __restrict__ mask, int B, int L, int H, float eps, int64_t* count,
    float* mean, float* var, float* cummean, float* cumrstd) {
  const int h = blockIdx.x * kThreads + threadIdx.x;
  const int b = blockIdx.y;
  if (h >= H) return;
  int64_t m0 = prev_count[b];
  float u = prev_mean[(size_t)b * H + h];
  float v = prev_var[(size_t)b * H + h];
  const float w = gamma[h], bb = beta[h];
  for (int t = 0; t < L; ++t) {
    const size_t o = ((size_t)b * L + t) * H + h;
    const bool masked = mask && mask[(size_t)b * L + t];
    const float xv = to_float(x[o]);
    const float coef = 1.0f / (float)(m0 + 1);
    const float d1 = xv - u;
    const float m1 = u + coef * d1;
    const float m2 = v + coef * (d1 * (xv - m1) - v);
    const float rstd = 1.0f / sqrtf(m2 + eps);
    y[o] = from_float<T>(masked ? 0.f : (xv - m1) * rstd * w + bb);
    if (!masked) {
      u = m1;
      v = m2;
      ++m0;
    }
    if (cummean) cummean[o] = masked ? u : m1;
    if (cumrstd) cumrstd[o] = masked ? 1.0f / sqrtf(v + eps) : rstd;
  }
  mean[(size_t)b * H + h] = u;
  var[(size_t)b * H + h] = v;
  if (h == 0) count[b] = m0;
}

struct TsnGeom {
  int vec, tpt, lpg, tt, ntiles;
  size_t smem;
};

bool tsn_geometry(int dtype, int64_t B, int64_t L, int64_t H, int64_t G, TsnGeom* g) {
  const int esize = dtype == MEGA_F32 ? 4 : 2;
  const int64_t dg = H / G;
  int vec = 16 / esize;
  while (vec > 1 && dg % vec != 0) vec /= 2;
  const int64_t tpt = H / vec;
  if (tpt > kPartCap) return false;
  int tt = (int)(kPartCap / tpt);
  if (tt > 64) tt = 64;
  while (tt > 8 && B * ceil_div(L, tt) < 512) tt /= 2;
  if (tt > L) tt = (int)L;
  if (tt < 1) tt = 1;
  g->vec = vec;
  g->tpt = (int)tpt;
  g->lpg = (int)(dg / vec);
  g->tt = tt;
  g->ntiles = (int)ceil_div(L, tt);
  const size_t floats = (size_t)kPartCap + 2 * (size_t)tt * G + 3 * (size_t)G +
                        3 * (size_t)(G > kThreads ? G : kThreads) + (size_t)tt;
  g->smem = floats * 4 + align_up((size_t)tt, 16);
  return g->smem <= 150 * 1024;
}

template <typename T, int VEC>
int launch_group_tsn(const TsnParams& P, const TsnGeom& g, hipStream_t stream) {
  const bool hoist = (kThreads % g.tpt) == 0;
  const dim3 grid((unsigned)(P.B * P.ntiles));
  auto kern = hoist ? group_tsn_kernel<T, VEC, true> : group_tsn_kernel<T, VEC, false>;
  if (g.smem > 64 * 1024) {
    hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)g.smem);
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), g.smem, stream, P);
  MEGA_CHECK_LAUNCH("group_timestep_norm_fwd");
  return MEGA_OK;
}

template <typename T>
int dispatch_vec(const TsnParams& P, const TsnGeom& g, hipStream_t s) {
  if constexpr (sizeof(T) == 2) {
    if (g.vec == 8) return launch_group_tsn<T, 8>(P, g, s);
  }
  if (g.vec == 4) return launch_group_tsn<T, 4>(P, g, s);
  if (g.vec == 2) return launch_group_tsn<T, 2>(P, g, s);
  return launch_group_tsn<T, 1>(P, g, s);
}

size_t tsn_workspace_bytes(int64_t B, int64_t G, int ntiles) {
  const size_t n = (size_t)B * ntiles;
  return align_up(sizeof(TsnHeader), 256) + align_up(n * 4, 256) * 2 + align_up(n * G * 2 * 4, 256);
}

}  // namespace

}  // namespace mega

using namespace mega;

extern "C" size_t mega_timestep_norm_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t H, int64_t G) {
  TsnGeom g;
  if (B <= 0 || L <= 0 || H <= 0 || G <= 0 || H % G != 0 || !tsn_geometry(dtype, B, L, H, G, &g)) return 256;
  return tsn_workspace_bytes(B, G, g.ntiles);
}

extern "C" int mega_group_timestep_norm_fwd(const void* x, void* y, int dtype,
                                            const int64_t* prev_count, const float* prev_mean,
                                            const float* prev_var, const float* gamma,
                                            const float* beta, const uint8_t* mask, int64_t B,
                                            int64_t L, int64_t H, int64_t G, double eps,
                                            int64_t* count, float* mean, float* var,
                                            float* group_mean, float* cummean, float* cumrstd,
                                            void* workspace, size_t workspace_bytes, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "group_timestep_norm_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && L >= 0 && H > 0 && G > 0, MEGA_ERR_ARG,
               "group_timestep_norm_fwd: bad shape B=%ld L=%ld H=%ld G=%ld", (long)B, (long)L, (long)H, (long)G);
  MEGA_REQUIRE(H % G == 0, MEGA_ERR_ARG, "group_timestep_norm_fwd: H=%ld is not a multiple of num_groups=%ld",
               (long)H, (long)G);
  MEGA_REQUIRE(B * L < (int64_t)1 << 31 && H < (int64_t)1 << 24, MEGA_ERR_UNSUPPORTED,
               "group_timestep_norm_fwd: B*L or H too large");
  if (B == 0) return MEGA_OK;
  MEGA_REQUIRE(prev_count && prev_mean && prev_var && gamma && beta && count && mean && var, MEGA_ERR_ARG,
               "group_timestep_norm_fwd: null state / parameter pointer");
  hipStream_t s = (hipStream_t)stream;
  if (L == 0) {
    hipMemcpyAsync(count, prev_count, (size_t)B * 8, hipMemcpyDeviceToDevice, s);
    hipMemcpyAsync(mean, prev_mean, (size_t)B * G * 4, hipMemcpyDeviceToDevice, s);
    hipMemcpyAsync(var, prev_var, (size_t)B * G * 4, hipMemcpyDeviceToDevice, s);
    return MEGA_OK;
  }
  MEGA_REQUIRE(x && y, MEGA_ERR_ARG, "group_timestep_norm_fwd: null x / y");
  MEGA_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)y % 16) == 0, MEGA_ERR_ARG,
               "group_timestep_norm_fwd: x / y must be 16-byte aligned");
  TsnGeom g;
  MEGA_REQUIRE(tsn_geometry(dtype, B, L, H, G, &g), MEGA_ERR_UNSUPPORTED,
               "group_timestep_norm_fwd: H=%ld G=%ld outside the supported envelope", (long)H, (long)G);
  MEGA_REQUIRE(workspace != nullptr && workspace_bytes >= tsn_workspace_bytes(B, G, g.ntiles),
               MEGA_ERR_WORKSPACE, "group_timestep_norm_fwd: workspace of %zu bytes needed",
               tsn_workspace_bytes(B, G, g.ntiles));
  const size_t n = (size_t)B * g.ntiles;
  char* w = (char*)workspace;
  TsnParams P;
  P.x = x; P.y = y; P.prev_count = prev_count; P.prev_mean = prev_mean; P.prev_var = prev_var;
  P.gamma = gamma; P.beta = beta; P.mask = mask; P.count = count; P.mean = mean; P.var = var;
  P.group_mean = group_mean; P.cummean = cummean; P.cumrstd = cumrstd;
  P.hdr = (TsnHeader*)w; w += align_up(sizeof(TsnHeader), 256);
  P.flags = (uint32_t*)w; w += align_up(n * 4, 256);
  P.tcnt = (uint32_t*)w; w += align_up(n * 4, 256);
  P.agg = (float*)w;
  P.B = (int)B; P.L = (int)L; P.H = (int)H; P.G = (int)G;
  P.TT = g.tt; P.ntiles = g.ntiles; P.TPT = g.tpt; P.LPG = g.lpg; P.eps = (float)eps;
  switch (dtype) {
    case MEGA_F32: return dispatch_vec<float>(P, g, s);
    case MEGA_BF16: return dispatch_vec<bf16_t>(P, g, s);
    default: return dispatch_vec<f16_t>(P, g, s);
  }
}

extern "C" int mega_timestep_norm_fwd(const void* x, void* y, int dtype, const int64_t* prev_count,
                                      const float* prev_mean, const float* prev_var,
                                      const float* gamma, const float* beta, const uint8_t* mask,
                                      int64_t B, int64_t L, int64_t H, double eps, int64_t* count,
                                      float* mean, float* var, float* cummean, float* cumrstd,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  (void)workspace;
  (void)workspace_bytes;
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "timestep_norm_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && L >= 0 && H > 0, MEGA_ERR_ARG, "timestep_norm_fwd: bad shape");
  MEGA_REQUIRE(B < 65536 && B * L * H < (int64_t)1 << 40, MEGA_ERR_UNSUPPORTED, "timestep_norm_fwd: too large");
  if (B == 0) return MEGA_OK;
  MEGA_REQUIRE(prev_count && prev_mean && prev_var && gamma && beta && count && mean && var, MEGA_ERR_ARG,
               "timestep_norm_fwd: null state / parameter pointer");
  MEGA_REQUIRE(L == 0 || (x && y), MEGA_ERR_ARG, "timestep_norm_fwd: null x / y");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)ceil_div(H, kThreads), (unsigned)B);
#define LAUNCH_FTSN(T)                                                                            \
  hipLaunchKernelGGL(feature_tsn_kernel<T>, grid, dim3(kThreads), 0, s, (const T*)x, (T*)y,       \
                     prev_count, prev_mean, prev_var, gamma, beta, mask, (int)B, (int)L, (int)H,  \
                     (float)eps, count, mean, var, cummean, cumrstd)
  switch (dtype) {
    case MEGA_F32: LAUNCH_FTSN(float); break;
    case MEGA_BF16: LAUNCH_FTSN(bf16_t); break;
    default: LAUNCH_FTSN(f16_t); break;
  }
#undef LAUNCH_FTSN
  MEGA_CHECK_LAUNCH("timestep_norm_fwd");
  return MEGA_OK;
}
