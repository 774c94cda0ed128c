// TimestepNorm backward (group and per-feature variants).
//
// Reference recurrences: fairseq/csrc/ops/timestep_norm.cc:318-450 (group) and :104-217
// (per-feature, which is the group form with one channel per group and group_mean = x).
// Walking the tokens of one (batch row, group) from the last to the first, the pair
// (u_grad, v_grad) is carried; at an unmasked token with running count n, c1 = (n-1)/n, c2 = 1/n,
// delta = group_mean - previous cumulative mean, r = cumrstd, ds = sum dy (x - cummean) w,
// db = sum dy w over the group's channels:
//     du = u_grad - r db,  dv = v_grad - r^3 ds / 2
//     dux = c2 du + 2 c1 c2 dv delta,  dvx = c2 dv
//     dx = dy r w + (dux + 2 dvx (x - group_mean)) / D
//     u_grad <- c1 du - 2 c1 c2 dv delta,  v_grad <- c1 dv
// The update of (u_grad, v_grad) is an affine map [[a, m], [0, a]] (.) + (bu, bv); such maps
// compose into maps of the same shape, so the walk is split over token tiles:
//   1. tsn_bwd_tile_kernel<.., 0>: per tile, ds / db per (token, group), the tile's composed map,
//      and the tile's share of the gamma / beta gradients;
//   2. tsn_bwd_carry_kernel: one wave per (row, group) scans the tile maps from the last tile
//      to the first and leaves the pair that enters every tile (and the prev_mean / prev_var
//      gradients at the end);
//   3. tsn_bwd_tile_kernel<.., 1>: per tile, the same ds / db again, the walk inside the tile from
//      its entering pair, then dx;
//   4. tsn_bwd_param_kernel: sums the per-tile gamma / beta shares.
// One launch instead of 1 - 3 (tsn_bwd_onepass_kernel: 16-bit activations in 16-byte vectors, at most 16 groups, a
// tile's dy and x held in registers): every tile publishes its map as tagged words, composes the maps of the tiles
// behind it in walk order (block records of 32 tiles for rows of more than 128 tiles, bounded waits) and goes on to dx with the dy and
// x it already holds, so both are read once.
// The per-feature norm with an even number of channels takes the same three steps with the channels across the
// lanes (tsn_bwd_feature_kernel: a thread owns two channels and walks its tile's 64 tokens itself).
// Masked tokens are skipped by the walk (identity map, dx = 0).  "Previous cumulative mean" is
// cummean[t-1]; the forward kernels of this library store the carried mean at masked tokens, so
// this is the state before token t also behind a masked token.
#include <atomic>

#include "common.h"
#include "tsn_common.h"

namespace mega {
namespace {

constexpr int kThreads = 512;
constexpr int kMaxTileCells = 4096;   // tokens-per-tile * groups held in LDS

struct TsnBwdParams {
  const void* dy;
  const void* x;
  void* dx;
  const float* mean_grad;
  const float* var_grad;
  const float* prev_mean;
  const int64_t* count;
  const float* group_mean;
  const float* cummean;
  const float* cumrstd;
  const float* gamma;
  const uint8_t* mask;
  float* agg;     // [B, nt, G, 4]  composed map of every tile
  float* state;   // [B, nt, G, 2]  (u_grad, v_grad) entering every tile (from the right)
  float* part;    // [B * nt, 2, H] gamma / beta shares
  float* prev_mean_grad;
  float* prev_var_grad;
  float* gamma_grad;
  float* beta_grad;
  int B, L, H, G, Dg, TT, nt;
  RowTiling R;
  // one-launch form: [B * nt][G][4] tagged words, a tile's map, and [B * nblk][G][4], the map of kOpBlock tiles
  unsigned long long* rec;
  unsigned long long* brec;
  int nblk;
  LookbackLaunch lb;
};

struct TileMap { float a, m, bu, bv; };
// first `f`, then `s`
__device__ __forceinline__ TileMap then(const TileMap f, const TileMap s) {
  return TileMap{s.a * f.a, fmaf(s.a, f.m, s.m * f.a), fmaf(s.a, f.bu, fmaf(s.m, f.bv, s.bu)), fmaf(s.a, f.bv, s.bv)};
}

__device__ __forceinline__ TileMap shfl_up32(const TileMap v, int o) {
  return TileMap{__shfl_up(v.a, o, 32), __shfl_up(v.m, o, 32), __shfl_up(v.bu, o, 32), __shfl_up(v.bv, o, 32)};
}

// PHASE 0: tile maps + parameter shares; PHASE 1: dx.
// FIXED (PHASE 0 only): slots divides the workgroup size and every lane moves one vector, so a
// thread meets the same VEC channels at every token it visits and keeps their gamma / beta shares
// in registers; otherwise tsn_bwd_shares_kernel forms the shares (a thread per vector of channels).
template <typename T, int VEC, int PHASE, bool FIXED = false>
__global__ __launch_bounds__(kThreads) void tsn_bwd_tile_kernel(const TsnBwdParams P) {
  using V = Vec<T, VEC>;
  extern __shared__ float smem[];
  const int G = P.G, H = P.H, TT = P.TT, Dg = P.Dg;
  const int cells = TT * G;
  float* s_r = smem;
  float* s_u = s_r + cells;
  float* s_ux = s_u + cells;
  float* s_ds = s_ux + cells;    // PHASE 1: dux after the walk
  float* s_db = s_ds + cells;    // PHASE 1: dvx after the walk
  float* s_up0 = s_db + cells;   // [G] cumulative mean before the tile's first token
  float* s_wg = s_up0 + G;       // [H] PHASE 0 only
  float* s_bg = s_wg + H;
  int* s_mask = (int*)(PHASE == 0 ? s_bg + H : s_up0 + G);   // [TT] + 1 counter
  const int tid = threadIdx.x;
  const int tile = blockIdx.x % P.nt;
  const int b = blockIdx.x / P.nt;
  const int t0 = tile * TT;
  const int ntok = min(TT, P.L - t0);
  const T* dy = (const T*)P.dy + ((size_t)b * P.L + t0) * H;
  const T* x = (const T*)P.x + ((size_t)b * P.L + t0) * H;

  // ---- statistics of the tile, mask, tokens that count after the tile
  for (int i = tid; i < cells; i += kThreads) {
    const int tok = i / G;
    if (tok < ntok) {
      const size_t o = ((size_t)b * P.L + t0) * G + i;
      s_r[i] = P.cumrstd[o];
      s_u[i] = P.cummean[o];
      s_ux[i] = P.group_mean ? P.group_mean[o] : 0.f;
    }
  }
  for (int g = tid; g < G; g += kThreads)
    s_up0[g] = t0 == 0 ? P.prev_mean[(size_t)b * G + g] : P.cummean[((size_t)b * P.L + t0 - 1) * G + g];
  if (PHASE == 0)
    for (int c = tid; c < H; c += kThreads) { s_wg[c] = 0.f; s_bg[c] = 0.f; }
  if (tid == 0) s_mask[TT] = 0;
  for (int tok = tid; tok < TT; tok += kThreads)
    s_mask[tok] = (tok >= ntok) || (P.mask && P.mask[(size_t)b * P.L + t0 + tok]);
  __syncthreads();
  if (P.mask) {
    int later = 0;   // unmasked tokens behind this tile
    for (int t = t0 + TT + tid; t < P.L; t += kThreads) later += P.mask[(size_t)b * P.L + t] ? 0 : 1;
    if (later) atomicAdd(&s_mask[TT], later);
  }

  // ---- ds, db (and the group mean when it was not handed in) per (token, group)
  const int items = ntok * P.R.slots;
  const int span = VEC * P.R.PER;          // channels per lane
  float rw[VEC], rb[VEC];                // FIXED: this thread's gamma / beta shares
#pragma unroll
  for (int e = 0; e < VEC; ++e) { rw[e] = 0.f; rb[e] = 0.f; }
  if (P.R.PER == 1) {
    // one vector per lane: four items per thread are loaded before any of them is used
    constexpr int U = 4;
    for (int i0 = 0; i0 < items; i0 += U * kThreads) {
      V dvv[U], xvv[U];
      int tokk[U], cc[U], cellk[U];
      bool livek[U], leadk[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = i0 + u * kThreads + tid;
        livek[u] = i < items;
        int tok, slot;
        split_item(P.R, livek[u] ? i : 0, tok, slot);
        const int g = slot >> P.R.lpg_shift;
        tokk[u] = tok;
        cc[u] = g * Dg + (slot - (g << P.R.lpg_shift)) * VEC;
        cellk[u] = tok * G + g;
        leadk[u] = livek[u] && slot == (g << P.R.lpg_shift);
        dvv[u] = *(const V*)(dy + (size_t)tok * H + cc[u]);
        xvv[u] = *(const V*)(x + (size_t)tok * H + cc[u]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float u_ = s_u[cellk[u]], r = s_r[cellk[u]];
        const bool keep = livek[u] && !s_mask[tokk[u]];
        float ds = 0.f, db = 0.f, sx = 0.f;
        float gw[VEC];
        load_params<VEC>(P.gamma + cc[u], gw);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float d = livek[u] ? to_float(dvv[u].v[e]) : 0.f, xe = to_float(xvv[u].v[e]), w = gw[e];
          ds = fmaf(d * (xe - u_), w, ds);
          db = fmaf(d, w, db);
          sx += xe;
          if (PHASE == 0 && keep) {
            if (FIXED) {
              rw[e] = fmaf(d * (xe - u_), r, rw[e]);
              rb[e] += d;
            }
          }
        }
        for (int o = 1; o < P.R.LPG; o <<= 1) {
          ds += __shfl_xor(ds, o);
          db += __shfl_xor(db, o);
          sx += __shfl_xor(sx, o);
        }
        if (leadk[u]) {
          s_ds[cellk[u]] = ds;
          s_db[cellk[u]] = db;
          if (!P.group_mean) s_ux[cellk[u]] = sx / (float)Dg;
        }
      }
    }
  } else {
  for (int i0 = 0; i0 < items; i0 += kThreads) {
    const int i = i0 + tid;
    const bool live = i < items;
    const int tok = live ? i / P.R.slots : 0;
    const int slot = live ? i - tok * P.R.slots : 0;
    const int g = slot / P.R.LPG;
    const int c0 = g * Dg + (slot - g * P.R.LPG) * span;
    const int cell = tok * G + g;
    float ds = 0.f, db = 0.f, sx = 0.f;
    if (live) {
      const float u = s_u[cell], r = s_r[cell];
      const bool keep = !s_mask[tok];
      for (int k = 0; k < P.R.PER; ++k) {
        const int c = c0 + k * VEC;
        const V dv = *(const V*)(dy + (size_t)tok * H + c);
        const V xv = *(const V*)(x + (size_t)tok * H + c);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float d = to_float(dv.v[e]), xe = to_float(xv.v[e]), w = P.gamma[c + e];
          ds = fmaf(d * (xe - u), w, ds);
          db = fmaf(d, w, db);
          sx += xe;
        }
      }
    }
    for (int o = 1; o < P.R.LPG; o <<= 1) {
      ds += __shfl_xor(ds, o);
      db += __shfl_xor(db, o);
      sx += __shfl_xor(sx, o);
    }
    if (live && slot == g * P.R.LPG) {
      s_ds[cell] = ds;
      s_db[cell] = db;
      if (!P.group_mean) s_ux[cell] = sx / (float)Dg;
    }
  }
  }
  __syncthreads();

  // ---- the walk over the tile's tokens, last to first, one thread per group
  const int64_t n_end = P.count[b] - (P.mask ? s_mask[TT] : max(0, P.L - t0 - TT));
  if (TT >= 16) {
    // 32 lanes per group, lane = position in walk order (0 = the tile's last token): every token's
    // map at once, then a scan over the positions
    const int pos = tid & 31;
    const int tok = ntok - 1 - pos;
    for (int g0 = 0; g0 < G; g0 += kThreads / 32) {
      const int g = g0 + (tid >> 5);
      const bool valid = g < G;
      const bool has = valid && tok >= 0 && !s_mask[max(tok, 0)];
      const unsigned long long bal = __ballot(has);
      const unsigned half = (unsigned)(bal >> (tid & 32));
      const int64_t n = n_end - __popc(half & ((1u << pos) - 1u));
      const int cell = max(tok, 0) * G + (valid ? g : 0);
      float c2 = 0.f, e = 0.f, rdb = 0.f, mj = 0.f;
      TileMap own{1.f, 0.f, 0.f, 0.f};
      if (has) {
        c2 = 1.0f / (float)n;
        const float c1 = (float)(n - 1) * c2;
        const float r = s_r[cell];
        const float up = tok == 0 ? s_up0[g] : s_u[cell - G];
        const float delta = s_ux[cell] - up;
        e = 0.5f * r * r * r * s_ds[cell];
        rdb = r * s_db[cell];
        mj = -2.0f * c1 * c2 * delta;
        own = TileMap{c1, mj, -c1 * rdb - mj * e, -c1 * e};
      }
      TileMap inc = own;
#pragma unroll
      for (int o = 1; o < 32; o <<= 1) {
        const TileMap prev = shfl_up32(inc, o);
        if (pos >= o) inc = then(prev, inc);
      }
      if (PHASE == 0) {
        if (valid && pos == 31) ((float4*)P.agg)[((size_t)b * P.nt + tile) * G + g] = make_float4(inc.a, inc.m, inc.bu, inc.bv);
      } else {
        TileMap exc = shfl_up32(inc, 1);
        if (pos == 0) exc = TileMap{1.f, 0.f, 0.f, 0.f};
        if (valid && tok >= 0) {
          const size_t so = (((size_t)b * P.nt + tile) * G + g) * 2;
          const float u0 = P.state[so], v0 = P.state[so + 1];
          const float ug = fmaf(exc.a, u0, fmaf(exc.m, v0, exc.bu));
          const float vg = fmaf(exc.a, v0, exc.bv);
          const float du = ug - rdb, dv = vg - e;
          s_ds[cell] = has ? c2 * du - mj * dv : 0.f;      // dux
          s_db[cell] = has ? c2 * dv : 0.f;                // dvx
        }
      }
    }
  } else
  for (int g = tid; g < G; g += kThreads) {
    int64_t n = n_end;                         // running count at the tile's last unmasked token
    float a = 1.f, m = 0.f, bu = 0.f, bv = 0.f;
    float ug = 0.f, vg = 0.f;
    if (PHASE == 1) {
      const size_t so = (((size_t)b * P.nt + tile) * G + g) * 2;
      ug = P.state[so];
      vg = P.state[so + 1];
    }
    for (int tok = ntok - 1; tok >= 0; --tok) {
      const int cell = tok * G + g;
      if (s_mask[tok]) {
        if (PHASE == 1) { s_ds[cell] = 0.f; s_db[cell] = 0.f; }
        continue;
      }
      const float c2 = 1.0f / (float)n, c1 = (float)(n - 1) * c2;
      --n;
      const float r = s_r[cell];
      const float up = tok == 0 ? s_up0[g] : s_u[cell - G];
      const float delta = s_ux[cell] - up;
      const float e = 0.5f * r * r * r * s_ds[cell];
      const float rdb = r * s_db[cell];
      const float mj = -2.0f * c1 * c2 * delta;
      if (PHASE == 0) {
        const float buj = -c1 * rdb - mj * e, bvj = -c1 * e;
        // this token's map after the maps of the tokens behind it
        const float na = c1 * a, nm = c1 * m + mj * a;
        const float nbu = c1 * bu + mj * bv + buj, nbv = c1 * bv + bvj;
        a = na; m = nm; bu = nbu; bv = nbv;
      } else {
        const float du = ug - rdb, dv = vg - e;
        s_ds[cell] = c2 * du - mj * dv;      // dux = c2 du + 2 c1 c2 dv delta
        s_db[cell] = c2 * dv;                // dvx
        ug = c1 * du + mj * dv;
        vg = c1 * dv;
      }
    }
    if (PHASE == 0) {
      float4* dst = (float4*)P.agg + ((size_t)b * P.nt + tile) * G + g;
      *dst = make_float4(a, m, bu, bv);
    }
  }
  __syncthreads();

  if (PHASE == 0) {
    if (FIXED) {
      // the kThreads / slots threads of one slot add up in a fixed order
      const int slot = tid % P.R.slots;
      const int g = slot / P.R.LPG;
      const int c0 = g * Dg + (slot - g * P.R.LPG) * VEC;
      for (int turn = 0; turn < kThreads / P.R.slots; ++turn) {
        if (tid / P.R.slots == turn) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) { s_wg[c0 + e] += rw[e]; s_bg[c0 + e] += rb[e]; }
        }
        __syncthreads();
      }
    }
    if (FIXED) {
      float* dst = P.part + ((size_t)b * P.nt + tile) * 2 * H;
      for (int c = tid; c < H; c += kThreads) { dst[c] = s_wg[c]; dst[H + c] = s_bg[c]; }
    }
  } else {
    T* dx = (T*)P.dx + ((size_t)b * P.L + t0) * H;
    const float cg = 1.0f / (float)Dg;
    if (P.R.PER == 1) {
      constexpr int U = 4;
      for (int i0 = 0; i0 < items; i0 += U * kThreads) {
        V dvv[U], xvv[U];
        int tokk[U], cc[U], cellk[U];
        bool livek[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i = i0 + u * kThreads + tid;
          livek[u] = i < items;
          int tok, slot;
          split_item(P.R, livek[u] ? i : 0, tok, slot);
          const int g = slot >> P.R.lpg_shift;
          tokk[u] = tok;
          cc[u] = g * Dg + (slot - (g << P.R.lpg_shift)) * VEC;
          cellk[u] = tok * G + g;
          dvv[u] = *(const V*)(dy + (size_t)tok * H + cc[u]);
          xvv[u] = *(const V*)(x + (size_t)tok * H + cc[u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const float r = s_r[cellk[u]], ux = s_ux[cellk[u]];
          const float a0 = s_ds[cellk[u]] * cg, a1 = 2.0f * s_db[cellk[u]] * cg;
          const bool keep = !s_mask[tokk[u]];
          V o;
          float gw[VEC];
          load_params<VEC>(P.gamma + cc[u], gw);
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const float v = fmaf(to_float(dvv[u].v[e]) * r, gw[e],
                                 fmaf(a1, to_float(xvv[u].v[e]) - ux, a0));
            o.v[e] = from_float<T>(keep ? v : 0.f);
          }
          if (livek[u]) *(V*)(dx + (size_t)tokk[u] * H + cc[u]) = o;
        }
      }
    } else {
      for (int i = tid; i < items; i += kThreads) {
        const int tok = i / P.R.slots;
        const int slot = i - tok * P.R.slots;
        const int g = slot / P.R.LPG;
        const int c0 = g * Dg + (slot - g * P.R.LPG) * span;
        const int cell = tok * G + g;
        const float r = s_r[cell], ux = s_ux[cell];
        const float a0 = s_ds[cell] * cg, a1 = 2.0f * s_db[cell] * cg;
        const bool keep = !s_mask[tok];
        for (int k = 0; k < P.R.PER; ++k) {
          const int c = c0 + k * VEC;
          const V dv = *(const V*)(dy + (size_t)tok * H + c);
          const V xv = *(const V*)(x + (size_t)tok * H + c);
          V o;
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const float v = fmaf(to_float(dv.v[e]) * r, P.gamma[c + e], fmaf(a1, to_float(xv.v[e]) - ux, a0));
            o.v[e] = from_float<T>(keep ? v : 0.f);
          }
          *(V*)(dx + (size_t)tok * H + c) = o;
        }
      }
    }
  }
}

// ---- per-feature statistics (one channel per group, group_mean = x): a thread owns two neighbouring channels and
// walks the tokens of its tile itself, from the last to the first; the tiles' maps are carried per channel.
// The same three steps as above (maps, carry, dx) with the channels, not the groups, across the lanes: every load is
// a row of neighbouring channels.  kFbT tokens per tile, kFbThreads x 2 channels per workgroup.
constexpr int kFbT = 64;
constexpr int kFbThreads = 256;
constexpr int kFbU = 8;            // tokens whose loads are in flight together

template <typename T>
__device__ __forceinline__ float2 load2(const T* p) {
  if constexpr (sizeof(T) == 4) {
    return *(const float2*)p;
  } else {
    const uint32_t w = *(const uint32_t*)p;
    T lo, hi;
    const uint16_t l16 = (uint16_t)(w & 0xffffu), h16 = (uint16_t)(w >> 16);
    __builtin_memcpy(&lo, &l16, 2);
    __builtin_memcpy(&hi, &h16, 2);
    return make_float2(to_float(lo), to_float(hi));
  }
}
template <typename T>
__device__ __forceinline__ void store2(T* p, float a, float b) {
  if constexpr (sizeof(T) == 4) {
    *(float2*)p = make_float2(a, b);
  } else {
    const T lo = from_float<T>(a), hi = from_float<T>(b);
    uint16_t l16, h16;
    __builtin_memcpy(&l16, &lo, 2);
    __builtin_memcpy(&h16, &hi, 2);
    *(uint32_t*)p = (uint32_t)l16 | ((uint32_t)h16 << 16);
  }
}

// PHASE 0: the tile's map of every channel and its gamma / beta shares; PHASE 1: dx from the pair entering the tile
template <typename T, int PHASE>
__global__ __launch_bounds__(kFbThreads) void tsn_bwd_feature_kernel(const TsnBwdParams P) {
  __shared__ float s_c1[kFbT], s_c2[kFbT];
  __shared__ int s_keep[kFbT];
  __shared__ int s_later;
  const int H = P.H, tid = threadIdx.x;
  const int cblocks = (H + 2 * kFbThreads - 1) / (2 * kFbThreads);
  const int cblk = (int)blockIdx.x % cblocks;
  const int rest = (int)blockIdx.x / cblocks;
  const int tile = rest % P.nt, b = rest / P.nt;
  const int t0 = tile * kFbT;
  const int ntok = min(kFbT, P.L - t0);
  const int c = cblk * 2 * kFbThreads + 2 * tid;      // H is even: a thread's two channels are both inside or outside
  const bool live = c < H;

  // ---- the running count at every token of the tile (the same for all channels)
  if (tid == 0) s_later = 0;
  __syncthreads();
  if (P.mask) {
    int later = 0;
    for (int t = t0 + kFbT + tid; t < P.L; t += kFbThreads) later += P.mask[(size_t)b * P.L + t] ? 0 : 1;
    if (later) atomicAdd(&s_later, later);
  }
  __syncthreads();
  if (tid < kFbT) {
    const bool has = tid < ntok && !(P.mask && P.mask[(size_t)b * P.L + t0 + tid]);
    const unsigned long long bal = __ballot(has);
    const int after = tid >= 63 ? 0 : __popcll(bal >> (tid + 1));     // unmasked tokens of the tile behind this one
    const int64_t n_end = P.count[b] - (P.mask ? (int64_t)s_later : (int64_t)max(0, P.L - t0 - kFbT));
    const float n = (float)(n_end - after);
    const float c2 = has ? 1.0f / n : 0.f;
    s_c2[tid] = c2;
    s_c1[tid] = has ? (n - 1.0f) * c2 : 1.f;
    s_keep[tid] = has ? 1 : 0;
  }
  __syncthreads();
  if (!live) return;

  const size_t row = ((size_t)b * P.L + t0) * H + c;
  const T* dy = (const T*)P.dy + row;
  const T* x = (const T*)P.x + row;
  const float* cm = P.cummean + row;
  const float* cr = P.cumrstd + row;
  const float2 w = *(const float2*)(P.gamma + c);
  // cumulative mean before the tile's first token
  const float2 up0 = t0 == 0 ? *(const float2*)(P.prev_mean + (size_t)b * H + c) : *(const float2*)(cm - H);

  float2 ug = make_float2(0.f, 0.f), vg = make_float2(0.f, 0.f);     // PHASE 1: the carried pair
  float2 ma = make_float2(1.f, 1.f), mm = make_float2(0.f, 0.f);     // PHASE 0: the composed map
  float2 mbu = make_float2(0.f, 0.f), mbv = make_float2(0.f, 0.f);
  float2 gwv = make_float2(0.f, 0.f), gbv = make_float2(0.f, 0.f);
  if (PHASE == 1) {
    const float4 st = *(const float4*)(P.state + (((size_t)b * P.nt + tile) * H + c) * 2);   // (u, v) of both channels
    ug = make_float2(st.x, st.z);
    vg = make_float2(st.y, st.w);
  }
  T* dx = PHASE == 1 ? (T*)P.dx + row : nullptr;
  for (int hi = ntok; hi > 0; hi -= kFbU) {
    // tokens hi - 1 down to hi - kFbU (those below 0 repeat token 0 and are dropped)
    float2 d[kFbU], xv[kFbU], m_[kFbU + 1], r_[kFbU];
#pragma unroll
    for (int k = 0; k < kFbU; ++k) {
      const int t = max(hi - 1 - k, 0);
      d[k] = load2<T>(dy + (size_t)t * H);
      xv[k] = load2<T>(x + (size_t)t * H);
      m_[k] = *(const float2*)(cm + (size_t)t * H);
      r_[k] = *(const float2*)(cr + (size_t)t * H);
    }
    {
      const int t = hi - 1 - kFbU;                    // the token before the batch: its cumulative mean
      m_[kFbU] = t >= 0 ? *(const float2*)(cm + (size_t)t * H) : up0;
    }
#pragma unroll
    for (int k = 0; k < kFbU; ++k) {
      const int t = hi - 1 - k;
      if (t < 0) break;
      const bool keep = s_keep[t] != 0;
      const float c1 = s_c1[t], c2 = s_c2[t];
      const float2 up = t == 0 ? up0 : m_[k + 1];
      float dxv[2];
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const float dq = q ? d[k].y : d[k].x, xq = q ? xv[k].y : xv[k].x, mq = q ? m_[k].y : m_[k].x;
        const float rq = q ? r_[k].y : r_[k].x, wq = q ? w.y : w.x, upq = q ? up.y : up.x;
        const float ds = dq * (xq - mq) * wq, db = dq * wq;
        const float e = 0.5f * rq * rq * rq * ds, rdb = rq * db;
        const float mj = -2.0f * c1 * c2 * (xq - upq);
        float& a_ = q ? ma.y : ma.x; float& m2 = q ? mm.y : mm.x; float& bu = q ? mbu.y : mbu.x; float& bv = q ? mbv.y : mbv.x;
        float& u_ = q ? ug.y : ug.x; float& v_ = q ? vg.y : vg.x;
        float& gw_ = q ? gwv.y : gwv.x; float& gb_ = q ? gbv.y : gbv.x;
        dxv[q] = 0.f;
        if (keep) {
          if (PHASE == 0) {
            // this token's map after the maps of the tokens behind it
            const float buj = -c1 * rdb - mj * e, bvj = -c1 * e;
            const float na = c1 * a_, nm = fmaf(c1, m2, mj * a_);
            const float nbu = fmaf(c1, bu, fmaf(mj, bv, buj)), nbv = fmaf(c1, bv, bvj);
            a_ = na; m2 = nm; bu = nbu; bv = nbv;
            gw_ = fmaf(dq * (xq - mq), rq, gw_);
            gb_ += dq;
          } else {
            const float du = u_ - rdb, dv = v_ - e;
            dxv[q] = fmaf(dq * rq, wq, c2 * du - mj * dv);      // group_mean = x: the dvx term vanishes
            u_ = fmaf(c1, du, mj * dv);
            v_ = c1 * dv;
          }
        }
      }
      if (PHASE == 1) store2<T>(dx + (size_t)t * H, dxv[0], dxv[1]);
    }
  }
  if (PHASE == 0) {
    float4* dst = (float4*)P.agg + ((size_t)b * P.nt + tile) * H + c;
    dst[0] = make_float4(ma.x, mm.x, mbu.x, mbv.x);
    dst[1] = make_float4(ma.y, mm.y, mbu.y, mbv.y);
    float* pt = P.part + ((size_t)b * P.nt + tile) * 2 * H;
    *(float2*)(pt + c) = gwv;
    *(float2*)(pt + H + c) = gbv;
  }
}

// one thread per (row, channel): the tiles' maps from the last tile to the first, eight maps in flight
__global__ __launch_bounds__(kFbThreads) void tsn_bwd_feature_carry_kernel(const TsnBwdParams P) {
  const int H = P.H;
  const int i = (int)blockIdx.x * kFbThreads + (int)threadIdx.x;      // (row, channel)
  if (i >= P.B * H) return;
  const int b = i / H, c = i - b * H;
  float ug = P.mean_grad ? P.mean_grad[i] : 0.f;
  float vg = P.var_grad ? P.var_grad[i] : 0.f;
  const float4* agg = (const float4*)P.agg + (size_t)b * P.nt * H + c;
  float2* st = (float2*)P.state + (size_t)b * P.nt * H + c;
  for (int hi = P.nt; hi > 0; hi -= 8) {
    float4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = agg[(size_t)max(hi - 1 - k, 0) * H];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int tile = hi - 1 - k;
      if (tile < 0) break;
      st[(size_t)tile * H] = make_float2(ug, vg);
      const float nu = fmaf(v[k].x, ug, fmaf(v[k].y, vg, v[k].z));
      vg = fmaf(v[k].x, vg, v[k].w);
      ug = nu;
    }
  }
  P.prev_mean_grad[i] = ug;
  P.prev_var_grad[i] = vg;
}

// ---- one launch: tile maps, look-back over the tiles behind, dx
constexpr int kOpThreads = 512;  // 8 waves; two workgroups share a compute unit (128 registers a lane)
constexpr int kOpNV = 8;        // 16-byte vectors of dy (and of x) a thread holds
constexpr int kOpBlock = 32;    // tiles per block record
constexpr int kOpDirect = 128;  // rows of up to this many tiles look back over the tiles themselves: one stage of
                                // waiting instead of two
constexpr uint32_t kOpTag = 1u; // the records are cleared before every launch

__device__ __forceinline__ TileMap shfl32(const TileMap v, int l) {
  return TileMap{__shfl(v.a, l, 32), __shfl(v.m, l, 32), __shfl(v.bu, l, 32), __shfl(v.bv, l, 32)};
}

// Workgroups are handed out in the order of their ids, so tile = nt - 1 - id / B: whatever a tile waits for was
// started before it.  512 threads: for the loads thread = (token of a round, slot of 8 channels), always the same
// channels; for the walk thread = (group, position in walk order).
template <typename T>
__global__ __launch_bounds__(kOpThreads, 4) void tsn_bwd_onepass_kernel(const TsnBwdParams P) {
  constexpr int VEC = 8;
  using V = Vec<T, VEC>;
  extern __shared__ float smem[];
  const int G = P.G, H = P.H, TT = P.TT, Dg = P.Dg;
  const int cells = TT * G;
  float* s_r = smem;
  float* s_u = s_r + cells;
  float* s_ux = s_u + cells;
  float* s_ds = s_ux + cells;    // dux after the walk
  float* s_db = s_ds + cells;    // dvx after the walk
  float* s_up0 = s_db + cells;   // [G] cumulative mean before the tile's first token
  float* s_wg = s_up0 + G;       // [H]
  float* s_bg = s_wg + H;
  int* s_mask = (int*)(s_bg + H);   // [TT] + counter of later unmasked tokens + give-up flag
  const int tid = threadIdx.x;
  const int ticket = (int)blockIdx.x;
  const int tile = P.nt - 1 - ticket / P.B;
  const int b = ticket % P.B;
  const int t0 = tile * TT;
  const int ntok = min(TT, P.L - t0);
  const T* dy = (const T*)P.dy + ((size_t)b * P.L + t0) * H;
  const T* x = (const T*)P.x + ((size_t)b * P.L + t0) * H;

  // ---- the tile's dy and x are requested first: thread = (token tokb + j * tps, slot)
  const int slots = P.R.slots, tps = kOpThreads / slots;
  const int slot = tid % slots, tokb = tid / slots;
  const int gs = slot >> P.R.lpg_shift;
  const int cc = gs * Dg + (slot - (gs << P.R.lpg_shift)) * VEC;
  static_assert(sizeof(V) == 16, "a vector is 16 bytes");
  uint4 dq[kOpNV], xq[kOpNV];             // kept packed: the values are unpacked where they are used, twice
#pragma unroll
  for (int j = 0; j < kOpNV; ++j) {
    // rounds beyond the tile's last token read that token again: whatever they compute is dropped (no branch here,
    // so that the sixteen words of a round stay sixteen registers)
    const int tok = min(tokb + j * tps, ntok - 1);
    dq[j] = *(const uint4*)(dy + (size_t)tok * H + cc);
    xq[j] = *(const uint4*)(x + (size_t)tok * H + cc);
  }
  float gw[VEC];
  load_params<VEC>(P.gamma + cc, gw);

  // ---- statistics of the tile, mask, tokens that count after the tile
  for (int i = tid; i < cells; i += kOpThreads) {
    const int tok = i / G;
    if (tok < ntok) {
      const size_t o = ((size_t)b * P.L + t0) * G + i;
      s_r[i] = P.cumrstd[o];
      s_u[i] = P.cummean[o];
      s_ux[i] = P.group_mean ? P.group_mean[o] : 0.f;
    }
  }
  for (int g = tid; g < G; g += kOpThreads)
    s_up0[g] = t0 == 0 ? P.prev_mean[(size_t)b * G + g] : P.cummean[((size_t)b * P.L + t0 - 1) * G + g];
  for (int c = tid; c < H; c += kOpThreads) { s_wg[c] = 0.f; s_bg[c] = 0.f; }
  if (tid == 0) { s_mask[TT] = 0; s_mask[TT + 1] = 0; }
  for (int tok = tid; tok < TT; tok += kOpThreads)
    s_mask[tok] = (tok >= ntok) || (P.mask && P.mask[(size_t)b * P.L + t0 + tok]);
  __syncthreads();
  if (P.mask) {
    int later = 0;   // unmasked tokens behind this tile
    for (int t = t0 + TT + tid; t < P.L; t += kOpThreads) later += P.mask[(size_t)b * P.L + t] ? 0 : 1;
    if (later) atomicAdd(&s_mask[TT], later);
  }

  // ---- ds, db (and the group mean when it was not handed in) per (token, group)
#pragma unroll
  for (int j = 0; j < kOpNV; ++j) {
    int tok = tokb + j * tps;
    asm volatile("" : "+v"(tok));
    const bool live = tok < ntok;
    const int cell = live ? tok * G + gs : gs;
    const float u_ = s_u[cell];
    float ds = 0.f, db = 0.f, sx = 0.f;
    asm volatile("" : "+v"(dq[j].x), "+v"(dq[j].y), "+v"(dq[j].z), "+v"(dq[j].w));
    asm volatile("" : "+v"(xq[j].x), "+v"(xq[j].y), "+v"(xq[j].z), "+v"(xq[j].w));
    const V dvj = __builtin_bit_cast(V, dq[j]), xvj = __builtin_bit_cast(V, xq[j]);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float d = to_float(dvj.v[e]), xe = to_float(xvj.v[e]), w = gw[e];
      ds = fmaf(d * (xe - u_), w, ds);
      db = fmaf(d, w, db);
      sx += xe;
    }
    for (int o = 1; o < P.R.LPG; o <<= 1) {
      ds += __shfl_xor(ds, o);
      db += __shfl_xor(db, o);
      sx += __shfl_xor(sx, o);
    }
    if (live && slot == (gs << P.R.lpg_shift)) {
      s_ds[cell] = ds;
      s_db[cell] = db;
      if (!P.group_mean) s_ux[cell] = sx / (float)Dg;
    }
    __builtin_amdgcn_sched_barrier(0);      // one token's temporaries at a time: the tile itself fills half the registers
  }
  __syncthreads();

  // ---- every token's map and the scan over the positions: 32 lanes per group, lane = position in walk order
  {
  const int64_t n_end = P.count[b] - (P.mask ? s_mask[TT] : max(0, P.L - t0 - TT));
  const int pos = tid & 31, grp = tid >> 5;
  const bool valid = grp < G;
  const int g = valid ? grp : 0;
  const int tok = ntok - 1 - pos;
  const bool has = valid && tok >= 0 && !s_mask[max(tok, 0)];
  const unsigned long long bal = __ballot(has);
  const unsigned half = (unsigned)(bal >> (tid & 32));
  const int64_t n = n_end - __popc(half & ((1u << pos) - 1u));
  const int cell = max(tok, 0) * G + g;
  float c2 = 0.f, e = 0.f, rdb = 0.f, mj = 0.f;
  TileMap own{1.f, 0.f, 0.f, 0.f};
  if (has) {
    c2 = 1.0f / (float)n;
    const float c1 = (float)(n - 1) * c2;
    const float r = s_r[cell];
    const float up = tok == 0 ? s_up0[g] : s_u[cell - G];
    const float delta = s_ux[cell] - up;
    e = 0.5f * r * r * r * s_ds[cell];
    rdb = r * s_db[cell];
    mj = -2.0f * c1 * c2 * delta;
    own = TileMap{c1, mj, -c1 * rdb - mj * e, -c1 * e};
  }
  TileMap inc = own;
#pragma unroll
  for (int o = 1; o < 32; o <<= 1) {
    const TileMap prev = shfl_up32(inc, o);
    if (pos >= o) inc = then(prev, inc);
  }
  TileMap exc = shfl_up32(inc, 1);
  if (pos == 0) exc = TileMap{1.f, 0.f, 0.f, 0.f};
  const TileMap tmap = shfl32(inc, 31);           // the tile's map, in every lane of the group

  // ---- publish it (lanes 0..3 of the group: one word each)
  auto word_of = [&](const TileMap& m_) -> uint32_t {
    return __float_as_uint(pos == 0 ? m_.a : pos == 1 ? m_.m : pos == 2 ? m_.bu : m_.bv);
  };
  if (valid && pos < 4 && !(P.lb.withhold_first && tile == P.nt - 1))
    put_rec(P.rec + (((size_t)b * P.nt + tile) * G + g) * 4 + pos, tagged(word_of(tmap), kOpTag));

  // ---- the maps of everything behind the tile, in walk order: the later blocks from the row's last one down, then
  // the later tiles of the tile's own block.  Lane i of a group fetches record i of a round of 32; the round is
  // composed in order by a scan over the lanes.
  const bool blocks = P.nt > kOpDirect;
  const int lbb = blocks ? kOpBlock : P.nt;
  const int kb = tile / lbb;
  const int bend = min(P.nt, (kb + 1) * lbb);     // one past the block's last tile
  const int nb = blocks ? P.nblk - 1 - kb : 0;    // later blocks
  const int nown = bend - 1 - tile;               // later tiles of the own block
  bool gave = false;
  auto fetch = [&](const int i0, const int i1) -> TileMap {
    TileMap acc{1.f, 0.f, 0.f, 0.f};
    for (int r0 = i0; r0 < i1; r0 += 32) {
      const int i = r0 + pos;
      TileMap v{1.f, 0.f, 0.f, 0.f};
      if (valid && i < i1) {
        const unsigned long long* src =
            i < nb ? P.brec + (((size_t)b * P.nblk + (P.nblk - 1 - i)) * G + g) * 4
                   : P.rec + (((size_t)b * P.nt + (bend - 1 - (i - nb))) * G + g) * 4;
        // the four words are asked for together; those that are not there yet are asked for again together
        unsigned long long w[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) w[u] = get_rec(src + u);
        uint32_t spins = 0;
        for (;;) {
          bool pending = false;
#pragma unroll
          for (int u = 0; u < 4; ++u) pending |= (uint32_t)(w[u] >> 32) != kOpTag;
          if (!pending) break;
          if (++spins > P.lb.spin_limit) {
            gave = true;
            break;
          }
          __builtin_amdgcn_s_sleep(1);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if ((uint32_t)(w[u] >> 32) != kOpTag) w[u] = get_rec(src + u);
        }
        v = TileMap{__uint_as_float((uint32_t)w[0]), __uint_as_float((uint32_t)w[1]), __uint_as_float((uint32_t)w[2]),
                    __uint_as_float((uint32_t)w[3])};
      }
      TileMap sc = v;
#pragma unroll
      for (int o = 1; o < 32; o <<= 1) {
        const TileMap prev = shfl_up32(sc, o);
        if (pos >= o) sc = then(prev, sc);
      }
      acc = then(acc, shfl32(sc, 31));
    }
    return acc;
  };
  // a group whose wait gave up: every lane of the group knows (and nothing is built on the missing words)
  auto group_gave = [&]() -> bool {
    const unsigned long long gb = __ballot(gave);
    return ((unsigned)(gb >> (tid & 32))) != 0u;
  };
  const TileMap own_blk = fetch(nb, nb + nown);
  bool lost = group_gave();
  if (blocks && tile == kb * lbb && valid && pos < 4 && !lost)
    put_rec(P.brec + (((size_t)b * P.nblk + kb) * G + g) * 4 + pos, tagged(word_of(then(own_blk, tmap)), kOpTag));
  const TileMap ent = then(fetch(0, nb), own_blk);
  lost = group_gave();
  if (lost && pos == 0) {
    s_mask[TT + 1] = 1;
    if (P.lb.status) __hip_atomic_store(P.lb.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }

  // ---- the pair that enters the tile, the pairs at its tokens, dux / dvx
  const float u0 = P.mean_grad ? P.mean_grad[(size_t)b * G + g] : 0.f;
  const float v0 = P.var_grad ? P.var_grad[(size_t)b * G + g] : 0.f;
  float ug0 = fmaf(ent.a, u0, fmaf(ent.m, v0, ent.bu));
  const float vg0 = fmaf(ent.a, v0, ent.bv);
  if (lost) ug0 = __builtin_nanf("");
  if (valid && tok >= 0) {
    const float ug = fmaf(exc.a, ug0, fmaf(exc.m, vg0, exc.bu));
    const float vg = fmaf(exc.a, vg0, exc.bv);
    const float du = ug - rdb, dv = vg - e;
    s_ds[cell] = has ? c2 * du - mj * dv : 0.f;      // dux
    s_db[cell] = has ? c2 * dv : 0.f;                // dvx
  }
  if (tile == 0 && valid && pos == 31) {
    const TileMap full = then(ent, tmap);
    const size_t i = (size_t)b * G + g;
    P.prev_mean_grad[i] = lost ? __builtin_nanf("") : fmaf(full.a, u0, fmaf(full.m, v0, full.bu));
    P.prev_var_grad[i] = lost ? __builtin_nanf("") : fmaf(full.a, v0, full.bv);
  }
  }
  __syncthreads();

  // ---- dx from the dy and x the thread holds, and the thread's gamma / beta shares (always the same channels)
  float rw[VEC], rb[VEC];
#pragma unroll
  for (int q = 0; q < VEC; ++q) { rw[q] = 0.f; rb[q] = 0.f; }
  {
    // the channels' weights again (out of the cache) rather than eight registers held across the look-back
    const float* gp = P.gamma + cc;
    asm volatile("" : "+v"(gp));
    load_params<VEC>(gp, gw);
    T* dx = (T*)P.dx + ((size_t)b * P.L + t0) * H;
    const float cg = 1.0f / (float)Dg;
    const bool poison = s_mask[TT + 1] != 0;
#pragma unroll
    for (int j = 0; j < kOpNV; ++j) {
      int tk = tokb + j * tps;
      asm volatile("" : "+v"(tk));      // addresses and cells are formed again here, not kept from the loads
      // the packed words are taken as they are (no unpacked copy is carried over from the first use)
      asm volatile("" : "+v"(dq[j].x), "+v"(dq[j].y), "+v"(dq[j].z), "+v"(dq[j].w));
      asm volatile("" : "+v"(xq[j].x), "+v"(xq[j].y), "+v"(xq[j].z), "+v"(xq[j].w));
      const V dvj = __builtin_bit_cast(V, dq[j]), xvj = __builtin_bit_cast(V, xq[j]);
      if (tk < ntok) {
        const int cl = tk * G + gs;
        const float r = s_r[cl], ux = s_ux[cl], um = s_u[cl];
        const float a0 = s_ds[cl] * cg, a1 = 2.0f * s_db[cl] * cg;
        const bool keep = !s_mask[tk];
        V o;
#pragma unroll
        for (int q = 0; q < VEC; ++q) {
          const float d = to_float(dvj.v[q]), xe = to_float(xvj.v[q]);
          float v = fmaf(d * r, gw[q], fmaf(a1, xe - ux, a0));
          if (poison) v = __builtin_nanf("");
          o.v[q] = from_float<T>(keep ? v : 0.f);
          if (keep) {
            rw[q] = fmaf(d * (xe - um), r, rw[q]);
            rb[q] += d;
          }
        }
        *(V*)(dx + (size_t)tk * H + cc) = o;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- the tile's share of the gamma / beta gradients: the threads of one slot add up in a fixed order
  for (int turn = 0; turn < tps; ++turn) {
    if (tokb == turn) {
#pragma unroll
      for (int q = 0; q < VEC; ++q) { s_wg[cc + q] += rw[q]; s_bg[cc + q] += rb[q]; }
    }
    __syncthreads();
  }
  float* dst = P.part + ((size_t)b * P.nt + tile) * 2 * H;
  for (int c = tid; c < H; c += kOpThreads) { dst[c] = s_wg[c]; dst[H + c] = s_bg[c]; }
}

// The gamma / beta shares of a tile where the tile kernel's threads do not keep to the same channels (group sizes
// that are not a power of two of vectors, more vectors per token than threads): a thread owns one vector of
// channels and walks the tile's tokens, four tokens' loads in flight.  Same output as the tile kernel's:
// part[row, tile][2][H].
template <typename T, int VEC>
__global__ __launch_bounds__(256) void tsn_bwd_shares_kernel(const TsnBwdParams P) {
  using V = Vec<T, VEC>;
  const int H = P.H, G = P.G, TT = P.TT;
  const int nvec = H / VEC;
  const int cblocks = (nvec + 255) / 256;
  const int cblk = (int)blockIdx.x % cblocks, rt = (int)blockIdx.x / cblocks;    // rt = row * nt + tile
  const int tile = rt % P.nt, b = rt / P.nt;
  const int v = cblk * 256 + (int)threadIdx.x;
  if (v >= nvec) return;
  const int c = v * VEC, g = c / P.Dg;
  const int t0 = tile * TT, ntok = min(TT, P.L - t0);
  const T* dy = (const T*)P.dy + ((size_t)b * P.L + t0) * H + c;
  const T* x = (const T*)P.x + ((size_t)b * P.L + t0) * H + c;
  const float* cm = P.cummean + ((size_t)b * P.L + t0) * G + g;
  const float* cr = P.cumrstd + ((size_t)b * P.L + t0) * G + g;
  const uint8_t* mk = P.mask ? P.mask + (size_t)b * P.L + t0 : nullptr;
  float rw[VEC], rb[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) { rw[e] = 0.f; rb[e] = 0.f; }
  for (int tb = 0; tb < ntok; tb += 4) {
    V dv[4], xv[4];
    float u[4], r[4];
    bool keep[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int t = min(tb + k, ntok - 1);
      dv[k] = *(const V*)(dy + (size_t)t * H);
      xv[k] = *(const V*)(x + (size_t)t * H);
      u[k] = cm[(size_t)t * G];
      r[k] = cr[(size_t)t * G];
      keep[k] = tb + k < ntok && !(mk && mk[t]);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (keep[k]) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float d = to_float(dv[k].v[e]);
          rw[e] = fmaf(d * (to_float(xv[k].v[e]) - u[k]), r[k], rw[e]);
          rb[e] += d;
        }
      }
    }
  }
  float* dst = P.part + (size_t)rt * 2 * H + c;
#pragma unroll
  for (int e = 0; e < VEC; ++e) { dst[e] = rw[e]; dst[H + e] = rb[e]; }
}

// One wave per (row, group).  The tiles are walked from the last to the first; lane l owns the
// l-th run of `per` tiles in that order, composes its run, the runs are combined by a scan over
// the lanes, and every lane then replays its run from the pair that enters it.
__global__ __launch_bounds__(64) void tsn_bwd_carry_kernel(const TsnBwdParams P) {
  const int i = blockIdx.x;               // (row, group)
  const int b = i / P.G, g = i - b * P.G;
  const int lane = threadIdx.x;
  const int per = (P.nt + 63) / 64;
  const int first = lane * per;           // position in walk order; tile = nt - 1 - position
  const float4* agg = (const float4*)P.agg + (size_t)b * P.nt * P.G + g;
  TileMap run{1.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < per; ++k) {
    const int pos = first + k;
    if (pos < P.nt) {
      const float4 v = agg[(size_t)(P.nt - 1 - pos) * P.G];
      run = then(run, TileMap{v.x, v.y, v.z, v.w});
    }
  }
  TileMap inc = run;                      // inclusive scan over the lanes
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    TileMap prev{__shfl_up(inc.a, o), __shfl_up(inc.m, o), __shfl_up(inc.bu, o), __shfl_up(inc.bv, o)};
    if (lane >= o) inc = then(prev, inc);
  }
  TileMap exc{__shfl_up(inc.a, 1), __shfl_up(inc.m, 1), __shfl_up(inc.bu, 1), __shfl_up(inc.bv, 1)};
  if (lane == 0) exc = TileMap{1.f, 0.f, 0.f, 0.f};
  const float u0 = P.mean_grad ? P.mean_grad[i] : 0.f;
  const float v0 = P.var_grad ? P.var_grad[i] : 0.f;
  float ug = fmaf(exc.a, u0, fmaf(exc.m, v0, exc.bu));
  float vg = fmaf(exc.a, v0, exc.bv);
  for (int k = 0; k < per; ++k) {
    const int pos = first + k;
    if (pos < P.nt) {
      const size_t o = ((size_t)b * P.nt + (P.nt - 1 - pos)) * P.G + g;
      P.state[o * 2] = ug;
      P.state[o * 2 + 1] = vg;
      const float4 v = ((const float4*)P.agg)[o];
      const float nu = fmaf(v.x, ug, fmaf(v.y, vg, v.z));
      vg = fmaf(v.x, vg, v.w);
      ug = nu;
    }
  }
  if (lane == 63) {
    P.prev_mean_grad[i] = fmaf(inc.a, u0, fmaf(inc.m, v0, inc.bu));
    P.prev_var_grad[i] = fmaf(inc.a, v0, inc.bv);
  }
}

// gamma / beta: 32 columns x 8 tile lanes per workgroup
__global__ __launch_bounds__(256) void tsn_bwd_param_kernel(const TsnBwdParams P) {
  __shared__ float s_acc[8][33];
  const int cl = threadIdx.x & 31, tl = threadIdx.x >> 5;
  const int c = blockIdx.x * 32 + cl;     // over 2 * H
  const int ntile = P.B * P.nt;
  float s = 0.f;
  if (c < 2 * P.H) {
    int t = tl;
    for (; t + 56 < ntile; t += 64) {       // eight loads in flight
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = P.part[(size_t)(t + 8 * k) * 2 * P.H + c];
#pragma unroll
      for (int k = 0; k < 8; ++k) s += v[k];
    }
    for (; t < ntile; t += 8) s += P.part[(size_t)t * 2 * P.H + c];
  }
  s_acc[tl][cl] = s;
  __syncthreads();
  if (tl == 0 && c < 2 * P.H) {
    float r = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) r += s_acc[k][cl];
    if (c < P.H) P.gamma_grad[c] = r;
    else P.beta_grad[c - P.H] = r;
  }
}

struct BwdGeom {
  int tt, nt, vec;
  size_t agg_bytes, state_bytes, part_bytes;
  // the one-launch form (onepass): its own tile length and records
  bool onepass;
  int op_tt, op_nt, op_nblk;
  size_t op_rec_bytes, op_brec_bytes, op_part_bytes;
  // per-feature statistics with an even number of channels: the channel-parallel form
  bool feature;
  int fb_nt;
  size_t fb_agg_bytes, fb_state_bytes, fb_part_bytes;
};

std::atomic<int> g_onepass{1};     // test hook: 0 keeps every call on the three-pass form

bool bwd_geometry(int dtype, int64_t B, int64_t L, int64_t H, int64_t G, BwdGeom* g) {
  if (G > kMaxTileCells || H > 8192 || B * L >= (int64_t)1 << 31) return false;
  const int64_t Dg = H / G;
  const int full = dtype == MEGA_F32 ? 4 : 8;
  g->vec = (Dg % full == 0) ? full : 1;
  int tt = (int)(kMaxTileCells / G);
  if (tt > 32) tt = 32;
  if (tt < 1) tt = 1;
  g->tt = tt;
  g->nt = (int)ceil_div(L, tt);
  if (B * g->nt >= (int64_t)1 << 31) return false;
  g->agg_bytes = align_up((size_t)B * g->nt * G * 16, 256);
  g->state_bytes = align_up((size_t)B * g->nt * G * 8, 256);
  g->part_bytes = align_up((size_t)B * g->nt * 2 * H * 4, 256);
  // one launch: 16-bit activations as 16-byte vectors, one vector per lane and token, at most 16 groups, and a tile
  // of at most kOpNV rounds of the workgroup's threads
  g->onepass = false;
  g->op_rec_bytes = g->op_brec_bytes = g->op_part_bytes = 0;
  if (dtype != MEGA_F32 && g->vec == 8 && G <= 16) {
    const RowTiling R = make_row_tiling(G, Dg, 8);
    if (R.PER == 1 && R.slots <= kOpThreads && kOpThreads % R.slots == 0) {
      const int per_round = kOpThreads / R.slots;
      const int ott = per_round * kOpNV < 32 ? per_round * kOpNV : 32;
      const int64_t ont = ceil_div(L, ott);
      if (ott >= 8 && B * ont < (int64_t)1 << 31) {
        g->onepass = true;
        g->op_tt = ott;
        g->op_nt = (int)ont;
        g->op_nblk = ont > kOpDirect ? (int)ceil_div(ont, kOpBlock) : 0;
        g->op_rec_bytes = align_up((size_t)B * ont * G * 32, 256);
        g->op_brec_bytes = align_up((size_t)B * g->op_nblk * G * 32, 256);
        g->op_part_bytes = align_up((size_t)B * ont * 2 * H * 4, 256);
      }
    }
  }
  g->feature = G == H && H % 2 == 0 && B * H < (int64_t)1 << 31;
  g->fb_nt = (int)ceil_div(L, kFbT);
  g->fb_agg_bytes = g->fb_state_bytes = g->fb_part_bytes = 0;
  if (g->feature) {
    g->fb_agg_bytes = align_up((size_t)B * g->fb_nt * H * 16, 256);
    g->fb_state_bytes = align_up((size_t)B * g->fb_nt * H * 8, 256);
    g->fb_part_bytes = align_up((size_t)B * g->fb_nt * 2 * H * 4, 256);
  }
  return true;
}

size_t bwd_workspace_need(const BwdGeom& g) {
  const size_t three = g.agg_bytes + g.state_bytes + g.part_bytes;
  const size_t one = g.op_rec_bytes + g.op_brec_bytes + g.op_part_bytes;
  const size_t feat = g.fb_agg_bytes + g.fb_state_bytes + g.fb_part_bytes;
  size_t need = three > one ? three : one;
  return need > feat ? need : feat;
}

template <typename T, int VEC>
int launch_tiles(const TsnBwdParams& P, hipStream_t s) {
  const size_t cells = (size_t)P.TT * P.G;
  const size_t lds0 = (5 * cells + P.G + 2 * (size_t)P.H) * 4 + (P.TT + 1) * 4;
  const size_t lds1 = (5 * cells + P.G) * 4 + (P.TT + 1) * 4;
  static uint64_t seen0 = 0, seen1 = 0;
  if (first_on_device(&seen0)) {
    (void)hipFuncSetAttribute((const void*)tsn_bwd_tile_kernel<T, VEC, 0, false>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    (void)hipFuncSetAttribute((const void*)tsn_bwd_tile_kernel<T, VEC, 0, true>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  }
  if (first_on_device(&seen1)) {
    (void)hipFuncSetAttribute((const void*)tsn_bwd_tile_kernel<T, VEC, 1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              160 * 1024);
  }
  const dim3 grid((unsigned)(P.B * P.nt));
  const bool fixed = P.R.PER == 1 && P.R.slots <= kThreads && kThreads % P.R.slots == 0;
  if (fixed) {
    hipLaunchKernelGGL((tsn_bwd_tile_kernel<T, VEC, 0, true>), grid, dim3(kThreads), lds0, s, P);
  } else {
    hipLaunchKernelGGL((tsn_bwd_tile_kernel<T, VEC, 0, false>), grid, dim3(kThreads), lds0, s, P);
    MEGA_CHECK_LAUNCH("timestep_norm_bwd (tile maps)");
    const int64_t cblocks = ceil_div((int64_t)P.H / VEC, 256);
    hipLaunchKernelGGL((tsn_bwd_shares_kernel<T, VEC>), dim3((unsigned)(P.B * P.nt * cblocks)), dim3(256), 0, s, P);
  }
  MEGA_CHECK_LAUNCH("timestep_norm_bwd (tile maps)");
  hipLaunchKernelGGL(tsn_bwd_carry_kernel, dim3((unsigned)(P.B * P.G)), dim3(64), 0, s, P);
  MEGA_CHECK_LAUNCH("timestep_norm_bwd (carry)");
  hipLaunchKernelGGL((tsn_bwd_tile_kernel<T, VEC, 1>), grid, dim3(kThreads), lds1, s, P);
  MEGA_CHECK_LAUNCH("timestep_norm_bwd (dx)");
  hipLaunchKernelGGL(tsn_bwd_param_kernel, dim3((unsigned)ceil_div(2 * (int64_t)P.H, 32)), dim3(256), 0, s, P);
  MEGA_CHECK_LAUNCH("timestep_norm_bwd (parameters)");
  return MEGA_OK;
}

template <typename T>
int launch_feature(const TsnBwdParams& P, hipStream_t s) {
  const int cblocks = (P.H + 2 * kFbThreads - 1) / (2 * kFbThreads);
  const dim3 grid((unsigned)((int64_t)P.B * P.nt * cblocks));
  hipLaunchKernelGGL((tsn_bwd_feature_kernel<T, 0>), grid, dim3(kFbThreads), 0, s, P);
  MEGA_CHECK_LAUNCH("timestep_norm_bwd (per-feature maps)");
  hipLaunchKernelGGL(tsn_bwd_feature_carry_kernel, dim3((unsigned)ceil_div((int64_t)P.B * P.H, kFbThreads)),
                     dim3(kFbThreads), 0, s, P);
  MEGA_CHECK_LAUNCH("timestep_norm_bwd (per-feature carry)");
  hipLaunchKernelGGL((tsn_bwd_feature_kernel<T, 1>), grid, dim3(kFbThreads), 0, s, P);
  MEGA_CHECK_LAUNCH("timestep_norm_bwd (per-feature dx)");
  hipLaunchKernelGGL(tsn_bwd_param_kernel, dim3((unsigned)ceil_div(2 * (int64_t)P.H, 32)), dim3(256), 0, s, P);
  MEGA_CHECK_LAUNCH("timestep_norm_bwd (parameters)");
  return MEGA_OK;
}

template <typename T>
int launch_onepass(const TsnBwdParams& P, size_t rec_bytes, hipStream_t s) {
  if constexpr (sizeof(T) != 2) {
    return MEGA_ERR_UNSUPPORTED;
  } else {
    const size_t cells = (size_t)P.TT * P.G;
    const size_t lds = (5 * cells + P.G + 2 * (size_t)P.H) * 4 + (P.TT + 2) * 4;
    static uint64_t seen = 0;
    if (first_on_device(&seen))
      (void)hipFuncSetAttribute((const void*)tsn_bwd_onepass_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                160 * 1024);
    zero_async(P.rec, rec_bytes, s);       // tile and block records (one range): no word carries the tag
    hipLaunchKernelGGL((tsn_bwd_onepass_kernel<T>), dim3((unsigned)(P.B * P.nt)), dim3(kOpThreads), lds, s, P);
    MEGA_CHECK_LAUNCH("timestep_norm_bwd (one launch)");
    hipLaunchKernelGGL(tsn_bwd_param_kernel, dim3((unsigned)ceil_div(2 * (int64_t)P.H, 32)), dim3(256), 0, s, P);
    MEGA_CHECK_LAUNCH("timestep_norm_bwd (parameters)");
    return MEGA_OK;
  }
}

template <typename T>
int launch_bwd(const TsnBwdParams& P, int vec, hipStream_t s) {
  constexpr int FULL = 16 / (int)sizeof(T);
  return vec == FULL ? launch_tiles<T, FULL>(P, s) : launch_tiles<T, 1>(P, s);
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" size_t mega_timestep_norm_bwd_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t H, int64_t G) {
  BwdGeom g;
  if (B <= 0 || L <= 0 || H <= 0 || G <= 0 || H % G != 0 || !bwd_geometry(dtype, B, L, H, G, &g)) return 256;
  return bwd_workspace_need(g);
}

extern "C" void mega_test_timestep_norm_bwd_onepass(int on) { g_onepass.store(on ? 1 : 0); }

extern "C" int mega_group_timestep_norm_bwd(const void* y_grad, const float* mean_grad, const float* var_grad,
                                            const void* x, int dtype, const float* prev_mean, const int64_t* count,
                                            const float* group_mean, const float* cummean, const float* cumrstd,
                                            const float* gamma, const uint8_t* mask, int64_t B, int64_t L, int64_t H,
                                            int64_t G, void* x_grad, float* prev_mean_grad, float* prev_var_grad,
                                            float* gamma_grad, float* beta_grad, void* workspace,
                                            size_t workspace_bytes, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "timestep_norm_bwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && L >= 0 && H > 0 && G > 0 && H % G == 0, MEGA_ERR_ARG,
               "timestep_norm_bwd: bad shape B=%ld L=%ld H=%ld G=%ld", (long)B, (long)L, (long)H, (long)G);
  MEGA_REQUIRE(prev_mean_grad && prev_var_grad && gamma_grad && beta_grad, MEGA_ERR_ARG,
               "timestep_norm_bwd: null gradient output");
  hipStream_t s = (hipStream_t)stream;
  if (B == 0 || L == 0) {
    // nothing between the incoming state gradients and the outgoing ones
    if (B > 0) {
      if (mean_grad) hipMemcpyAsync(prev_mean_grad, mean_grad, (size_t)B * G * 4, hipMemcpyDeviceToDevice, s);
      else zero_async(prev_mean_grad, (size_t)B * G * 4, s);
      if (var_grad) hipMemcpyAsync(prev_var_grad, var_grad, (size_t)B * G * 4, hipMemcpyDeviceToDevice, s);
      else zero_async(prev_var_grad, (size_t)B * G * 4, s);
    }
    zero_async(gamma_grad, (size_t)H * 4, s);
    zero_async(beta_grad, (size_t)H * 4, s);
    return MEGA_OK;
  }
  MEGA_REQUIRE(y_grad && x && x_grad && prev_mean && count && cummean && cumrstd && gamma, MEGA_ERR_ARG,
               "timestep_norm_bwd: null pointer argument");
  BwdGeom g;
  MEGA_REQUIRE(bwd_geometry(dtype, B, L, H, G, &g), MEGA_ERR_UNSUPPORTED,
               "timestep_norm_bwd: H=%ld G=%ld outside the supported envelope (H <= 8192, G <= %d)", (long)H, (long)G,
               kMaxTileCells);
  if (g.vec > 1 && ((((uintptr_t)y_grad | (uintptr_t)x | (uintptr_t)x_grad | (uintptr_t)gamma) % 16) != 0))
    g.vec = 1;                             // element-wise tiling when a buffer is not 16-byte aligned
  const size_t need = bwd_workspace_need(g);
  MEGA_REQUIRE(workspace && workspace_bytes >= need && ((uintptr_t)workspace % 16) == 0, MEGA_ERR_WORKSPACE,
               "timestep_norm_bwd: workspace of %zu bytes (16-byte aligned) needed", need);
  char* w = (char*)workspace;
  TsnBwdParams P;
  const bool onepass = g.onepass && g.vec == 8 && g_onepass.load() != 0;
  if (onepass) {
    if (!audit_on())
      if (const int rc = lookback_pending("timestep_norm_bwd")) return rc;
    P.dy = y_grad; P.x = x; P.dx = x_grad; P.mean_grad = mean_grad; P.var_grad = var_grad; P.prev_mean = prev_mean;
    P.count = count; P.group_mean = group_mean; P.cummean = cummean; P.cumrstd = cumrstd; P.gamma = gamma; P.mask = mask;
    P.agg = nullptr; P.state = nullptr;
    P.rec = (unsigned long long*)w; w += g.op_rec_bytes;
    P.brec = (unsigned long long*)w; w += g.op_brec_bytes;
    P.part = (float*)w;
    P.prev_mean_grad = prev_mean_grad; P.prev_var_grad = prev_var_grad; P.gamma_grad = gamma_grad; P.beta_grad = beta_grad;
    P.B = (int)B; P.L = (int)L; P.H = (int)H; P.G = (int)G; P.Dg = (int)(H / G); P.TT = g.op_tt; P.nt = g.op_nt;
    P.nblk = g.op_nblk;
    P.R = make_row_tiling(G, H / G, 8);
    if (audit_on()) {
      // per (row, tile, group) and per (row, block of tiles, group): one map of four tagged words; per (row, tile): the
      // tile's share of the gamma / beta gradients, 2 H floats
      audit_use(P.rec, (size_t)B * g.op_nt * G * 32, "timestep_norm_bwd: tile records");
      if (g.op_nblk) audit_use(P.brec, (size_t)B * g.op_nblk * G * 32, "timestep_norm_bwd: block records");
      else audit_use(P.rec, 32, "timestep_norm_bwd: block records (none)");
      audit_use(P.part, (size_t)B * g.op_nt * 2 * H * 4, "timestep_norm_bwd: parameter-gradient shares");
      audit_use(y_grad, (size_t)B * L * H * 2, "timestep_norm_bwd: y_grad");
      audit_use(x, (size_t)B * L * H * 2, "timestep_norm_bwd: x");
      audit_use(x_grad, (size_t)B * L * H * 2, "timestep_norm_bwd: x_grad");
      audit_use(cummean, (size_t)B * L * G * 4, "timestep_norm_bwd: cummean");
      audit_use(cumrstd, (size_t)B * L * G * 4, "timestep_norm_bwd: cumrstd");
      return MEGA_OK;
    }
    P.lb = lookback_launch(true);
    const int rc = dtype == MEGA_BF16 ? launch_onepass<bf16_t>(P, g.op_rec_bytes + g.op_brec_bytes, s)
                                      : launch_onepass<f16_t>(P, g.op_rec_bytes + g.op_brec_bytes, s);
    return rc != MEGA_OK ? rc : lookback_verify("timestep_norm_bwd", s);
  }
  P.rec = nullptr; P.brec = nullptr; P.nblk = 0; P.lb = LookbackLaunch{nullptr, 0u, 0};
  const size_t es_ = dtype == MEGA_F32 ? 4 : 2;
  if (g.feature && ((((uintptr_t)y_grad | (uintptr_t)x | (uintptr_t)x_grad) % (2 * es_)) == 0) &&
      ((((uintptr_t)cummean | (uintptr_t)cumrstd | (uintptr_t)gamma | (uintptr_t)prev_mean) % 8) == 0)) {
    P.dy = y_grad; P.x = x; P.dx = x_grad; P.mean_grad = mean_grad; P.var_grad = var_grad; P.prev_mean = prev_mean;
    P.count = count; P.group_mean = nullptr; P.cummean = cummean; P.cumrstd = cumrstd; P.gamma = gamma; P.mask = mask;
    P.agg = (float*)w; w += g.fb_agg_bytes;
    P.state = (float*)w; w += g.fb_state_bytes;
    P.part = (float*)w;
    P.prev_mean_grad = prev_mean_grad; P.prev_var_grad = prev_var_grad; P.gamma_grad = gamma_grad; P.beta_grad = beta_grad;
    P.B = (int)B; P.L = (int)L; P.H = (int)H; P.G = (int)G; P.Dg = 1; P.TT = kFbT; P.nt = g.fb_nt;
    P.R = make_row_tiling(G, 1, 1);
    if (audit_on()) {
      // per (row, tile, channel): one map of four floats and one pair of state gradients; per (row, tile): the tile's
      // share of the gamma / beta gradients, 2 H floats
      audit_use(P.agg, (size_t)B * g.fb_nt * H * 16, "timestep_norm_bwd: per-feature tile maps");
      audit_use(P.state, (size_t)B * g.fb_nt * H * 8, "timestep_norm_bwd: per-feature pairs entering the tiles");
      audit_use(P.part, (size_t)B * g.fb_nt * 2 * H * 4, "timestep_norm_bwd: parameter-gradient shares");
      audit_use(y_grad, (size_t)B * L * H * es_, "timestep_norm_bwd: y_grad");
      audit_use(x, (size_t)B * L * H * es_, "timestep_norm_bwd: x");
      audit_use(x_grad, (size_t)B * L * H * es_, "timestep_norm_bwd: x_grad");
      audit_use(cummean, (size_t)B * L * G * 4, "timestep_norm_bwd: cummean");
      audit_use(cumrstd, (size_t)B * L * G * 4, "timestep_norm_bwd: cumrstd");
      return MEGA_OK;
    }
    switch (dtype) {
      case MEGA_F32: return launch_feature<float>(P, s);
      case MEGA_BF16: return launch_feature<bf16_t>(P, s);
      default: return launch_feature<f16_t>(P, s);
    }
  }
  P.dy = y_grad; P.x = x; P.dx = x_grad; P.mean_grad = mean_grad; P.var_grad = var_grad; P.prev_mean = prev_mean;
  P.count = count; P.group_mean = group_mean; P.cummean = cummean; P.cumrstd = cumrstd; P.gamma = gamma; P.mask = mask;
  P.agg = (float*)w; w += g.agg_bytes;
  P.state = (float*)w; w += g.state_bytes;
  P.part = (float*)w;
  P.prev_mean_grad = prev_mean_grad; P.prev_var_grad = prev_var_grad; P.gamma_grad = gamma_grad; P.beta_grad = beta_grad;
  P.B = (int)B; P.L = (int)L; P.H = (int)H; P.G = (int)G; P.Dg = (int)(H / G); P.TT = g.tt; P.nt = g.nt;
  P.R = make_row_tiling(G, H / G, g.vec);
  if (audit_on()) {
    // per (row, tile, group): one map of four floats and one pair of state gradients; per (row, tile): the tile's
    // share of the gamma / beta gradients, 2 H floats
    const size_t es = dtype == MEGA_F32 ? 4 : 2;
    audit_use(P.agg, (size_t)B * g.nt * G * 16, "timestep_norm_bwd: tile maps");
    audit_use(P.state, (size_t)B * g.nt * G * 8, "timestep_norm_bwd: pairs entering the tiles");
    audit_use(P.part, (size_t)B * g.nt * 2 * H * 4, "timestep_norm_bwd: parameter-gradient shares");
    audit_use(y_grad, (size_t)B * L * H * es, "timestep_norm_bwd: y_grad");
    audit_use(x, (size_t)B * L * H * es, "timestep_norm_bwd: x");
    audit_use(x_grad, (size_t)B * L * H * es, "timestep_norm_bwd: x_grad");
    audit_use(cummean, (size_t)B * L * G * 4, "timestep_norm_bwd: cummean");
    audit_use(cumrstd, (size_t)B * L * G * 4, "timestep_norm_bwd: cumrstd");
    return MEGA_OK;
  }
  switch (dtype) {
    case MEGA_F32: return launch_bwd<float>(P, g.vec, s);
    case MEGA_BF16: return launch_bwd<bf16_t>(P, g.vec, s);
    default: return launch_bwd<f16_t>(P, g.vec, s);
  }
}

extern "C" int mega_timestep_norm_bwd(const void* y_grad, const float* mean_grad, const float* var_grad, const void* x,
                                      int dtype, const float* prev_mean, const int64_t* count, const float* cummean,
                                      const float* cumrstd, const float* gamma, const uint8_t* mask, int64_t B,
                                      int64_t L, int64_t H, void* x_grad, float* prev_mean_grad, float* prev_var_grad,
                                      float* gamma_grad, float* beta_grad, void* workspace, size_t workspace_bytes,
                                      void* stream) {
  return mega_group_timestep_norm_bwd(y_grad, mean_grad, var_grad, x, dtype, prev_mean, count, nullptr, cummean,
                                      cumrstd, gamma, mask, B, L, H, H, x_grad, prev_mean_grad, prev_var_grad,
                                      gamma_grad, beta_grad, workspace, workspace_bytes, stream);
}
