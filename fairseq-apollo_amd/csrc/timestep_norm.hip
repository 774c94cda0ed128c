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
//   Tiles map to workgroup ids in time-major order; workgroups are dispatched in id order, so
//   a tile only ever waits for tiles whose workgroups were dispatched before it; the wait is
//   bounded and sets an error word instead of spinning forever.  Published words carry the
//   launch epoch as a tag, so nothing has to be cleared between launches and no single
//   address is hit by one atomic per workgroup on the way in.
#include "tsn_common.h"

// Phase markers: a profiling build defines MEGA_TSN_TR(k) to stamp a clock; no-ops here.
#ifndef MEGA_TSN_TR
#define MEGA_TSN_TR(k)
#endif

namespace mega {

namespace {

constexpr int kThreads = 256;
constexpr int kNV = 16;                       // vectors kept in registers per thread
constexpr int kPartCap = kThreads * kNV;      // vectors per tile
constexpr int kMaxTT = 64;                    // tokens per tile (16 lanes x 4 tokens in the scan)
constexpr int kLbWords = 4352;                // 64-bit words staged in LDS per look-back round
constexpr int kLbBlock = 32;                  // tiles per block record: a tile looks back over the whole blocks before
                                              // it and the earlier tiles of its own block, not over every earlier tile
#ifndef MEGA_TSN_LBDIRECT
#define MEGA_TSN_LBDIRECT 128
#endif
constexpr int kLbDirect = MEGA_TSN_LBDIRECT;  // rows of up to this many tiles look back over the tiles themselves: one
                                              // round of records, and no wait for a block's last tile to add its block up

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
  // [B*ntiles][2G+1] 64-bit words, value in the low half, launch tag in the high half:
  // word 0 = unmasked tokens of the tile, word 1+2g = mean, word 2+2g = variance of group g
  unsigned long long* rec;
  // [B*nblk][2G+1] words of the same form: the aggregate of kLbBlock consecutive tiles, left by the block's last
  // tile once it has seen the others
  unsigned long long* brec;
  int B, L, H, G;
  int TT, ntiles, nblk;
  int TPT;           // vectors per token
  int LPG;           // vectors per group
  float eps;
  LookbackLaunch lb; // status word, poll limit, test hook
};

// LPGT > 0: groups are LPGT adjacent lanes and are reduced with lane shuffles;
// LPGT == 0: any group size, partial sums go through LDS.
template <typename T, int VEC, bool HOIST, int LPGT>
__global__ __launch_bounds__(kThreads) void group_tsn_kernel(const TsnParams P) {
  extern __shared__ float smem[];
  float* s_mean = smem;                            // [TT*G]  group mean, later running mean
  float* s_var = s_mean + (size_t)P.TT * P.G;      // [TT*G]  group var, later running rstd
  uint8_t* s_mask = (uint8_t*)(s_var + (size_t)P.TT * P.G);   // [TT]
  unsigned long long* s_lbw = (unsigned long long*)(s_mask + ((P.TT + 15) / 16) * 16);   // [kLbWords]
  float* part = (float*)(s_lbw + kLbWords);                   // [kPartCap] (LPGT == 0 only)

  __shared__ uint32_t s_gave_up;                   // a wait of this workgroup ran into the poll limit
  const int tid = threadIdx.x;
  if (tid == 0) s_gave_up = 0u;
  const int ticket = (int)blockIdx.x;
  const uint32_t tag = P.hdr->epoch + 1u;
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

  MEGA_TSN_TR(0);
  // ---- everything the tail of the kernel needs from global memory is requested up front, so
  // that no cold miss sits between the look-back and the stores: the prior state of the first
  // 16 groups and the affine parameters of this thread's features
  const int row16 = tid >> 4, l16 = tid & 15;
  const int gfirst = row16 < G ? row16 : G - 1;
  const Moments prior0 = {(float)P.prev_count[b], P.prev_mean[(size_t)b * G + gfirst], P.prev_var[(size_t)b * G + gfirst]};
  // HOIST (kThreads is a multiple of the vectors per token): vector j of a thread belongs to token
  // tok0 + j * tps and always to the same features, so the loops below need no division
  const int tok0 = tid / TPT, vi0 = tid - tok0 * TPT, tps = kThreads / TPT;
  int g0;
  if constexpr (LPGT > 0) g0 = vi0 / LPGT; else g0 = vi0 / LPG;
  float gam[VEC], bet[VEC];
  if (HOIST) {
    const int f0 = vi0 * VEC;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      gam[i] = P.gamma[f0 + i];
      bet[i] = P.beta[f0 + i];
    }
  }
  // ---- load the tile (one contiguous block) and the mask bytes
  V xv[kNV];
#pragma unroll
  for (int j = 0; j < kNV; ++j) {
    // vectors beyond the tile read its last one again and whatever is computed from them is dropped: a branch here
    // makes the compiler carry a vector of 16-bit values as separate registers from the load on
    const int v = min(j * kThreads + tid, nvec - 1);
    xv[j] = xin[v];
  }
  for (int t = tid; t < nt; t += kThreads)
    s_mask[t] = P.mask ? (P.mask[(size_t)b * P.L + t0 + t] != 0) : 0;

  // ---- moments of every (token, group): mean first, then the variance around it
  if (LPGT > 0) {
#pragma unroll
    for (int j = 0; j < kNV; ++j) {
      const int v = j * kThreads + tid;
      float m, gv;
      if constexpr (sizeof(T) == 2 && VEC >= 2) {
        // 16-bit activations: sum and sum of squares by packed dot products.  The difference
        // E[x^2] - mean^2 is taken in fp32, which resolves more than the 8 / 11 significant bits
        // the inputs themselves carry.
        float s = 0.f, q = 0.f;
        const uint32_t* w = (const uint32_t*)&xv[j];
#pragma unroll
        for (int i = 0; i < VEC / 2; ++i) {
          s = dot2_ones<T>(w[i], s);
          q = dot2_self<T>(w[i], q);
        }
        m = group_sum<LPGT>(s) * inv_dg;
        gv = fmaxf(group_sum<LPGT>(q) * inv_dg - m * m, 0.f);
      } else {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < VEC; ++i) s += to_float(xv[j].v[i]);
        m = group_sum<LPGT>(s) * inv_dg;
        float s2 = 0.f;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          const float d = to_float(xv[j].v[i]) - m;
          s2 += d * d;
        }
        gv = group_sum<LPGT>(s2) * inv_dg;
      }
      if ((tid & (LPGT - 1)) == 0 && v < nvec) {
        const int tok = HOIST ? tok0 + j * tps : v / TPT;
        const int g = HOIST ? g0 : (v - tok * TPT) / LPGT;
        s_mean[tok * G + g] = m;
        s_var[tok * G + g] = gv;
      }
    }
    __syncthreads();
  } else if constexpr (sizeof(T) == 2 && VEC >= 2) {
    // groups of any number of vectors, 16-bit activations: every vector's sum and sum of squares (packed dot
    // products, as above) go through LDS once, and a thread per (token, group) adds the group's up
    float2* part2 = (float2*)part;
#pragma unroll
    for (int j = 0; j < kNV; ++j) {
      const int v = j * kThreads + tid;
      if (v < nvec) {
        float s = 0.f, q = 0.f;
        const uint32_t* w = (const uint32_t*)&xv[j];
#pragma unroll
        for (int i = 0; i < VEC / 2; ++i) {
          s = dot2_ones<T>(w[i], s);
          q = dot2_self<T>(w[i], q);
        }
        part2[v] = make_float2(s, q);
      }
    }
    __syncthreads();
    for (int item = tid; item < nt * G; item += kThreads) {
      const int tok = item / G, g = item - tok * G;
      const float2* pp = part2 + tok * TPT + g * LPG;
      float s = 0.f, q = 0.f;
      for (int i = 0; i < LPG; ++i) {
        s += pp[i].x;
        q += pp[i].y;
      }
      const float m = s * inv_dg;
      s_mean[item] = m;
      s_var[item] = fmaxf(q * inv_dg - m * m, 0.f);
    }
    __syncthreads();
  } else {
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
  }

  // ---- running statistics.  A row of 16 lanes owns one group: lane l16 scans its TPL tokens, the
  // row scans across lanes and publishes the tile aggregate.  The aggregates of the earlier tiles of
  // this batch row are then fetched as one contiguous block into LDS (every word says by itself
  // whether it has been published: no fence on either side) and folded into the carry-in.
  MEGA_TSN_TR(1);
  const int TPL = (P.TT + 15) >> 4;                 // tokens per lane (<= 4)
  const size_t trow = (size_t)b * P.ntiles;
  const bool last_tile = tile == P.ntiles - 1;
  const int W = 2 * G + 1;                          // words per tile record
  // the tile's own statistics of a set of 16 groups: every lane's prefixes over its tokens, the row's scan
  auto own_scan = [&](const int gc, const bool active, const int g, const bool first_pass, Moments (&pref)[4]) -> Moments {
    Moments st = {0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int tok = l16 * TPL + u;
      if (u < TPL && tok < nt) {
        const float gm = s_mean[tok * G + gc];
        const float gv = s_var[tok * G + gc];
        if (first_pass && P.group_mean && active) P.group_mean[((size_t)b * P.L + t0 + tok) * G + g] = gm;
        if (!s_mask[tok]) st = merge(st, Moments{1.f, gm, gv});
      }
      pref[u] = st;
    }
    return row_scan(st);
  };
  // With more than 16 groups the aggregates of all of them are published before the first look-back: a tile that
  // waited for the earlier tiles' first 16 groups before publishing its own next 16 would make the row a chain.
  if (G > 16) {
    for (int gbase = 0; gbase < G; gbase += 16) {
      const int g = gbase + row16;
      const bool active = g < G;
      Moments pref[4];
      const Moments inc = own_scan(active ? g : G - 1, active, g, true, pref);
      if (l16 == 15 && active && !(P.lb.withhold_first && tile == 0)) {
        unsigned long long* mine = P.rec + (trow + tile) * W;
        put_rec(mine + 1 + 2 * g, tagged(__float_as_uint(inc.mean), tag));
        put_rec(mine + 2 + 2 * g, tagged(__float_as_uint(inc.var), tag));
        if (g == 0) put_rec(mine, tagged((uint32_t)inc.n, tag));
      }
    }
  }
  for (int gbase = 0; gbase < G; gbase += 16) {
    const int g = gbase + row16;
    const bool active = g < G;
    const int gc = active ? g : G - 1;
    // a look-back fetches the count word and the words of this set of groups only
    const int wlo = 1 + 2 * gbase;                    // first group word of the set
    const int WS = min(32, W - wlo) + 1;              // words per record staged: count + the set's
    const int RT = kLbWords / WS;                     // earlier tiles per look-back round
    Moments pref[4];
    const Moments inc = own_scan(gc, active, g, G <= 16, pref);
    const Moments exc = dpp_m<0x111>(inc);          // exclusive: what the lanes before this one hold
    if (G <= 16 && l16 == 15 && active && !(P.lb.withhold_first && tile == 0)) {
      unsigned long long* mine = P.rec + (trow + tile) * W;
      put_rec(mine + 1 + 2 * g, tagged(__float_as_uint(inc.mean), tag));
      put_rec(mine + 2 + 2 * g, tagged(__float_as_uint(inc.var), tag));
      if (g == 0) put_rec(mine, tagged((uint32_t)inc.n, tag));
    }
    MEGA_TSN_TR(2);
    // what came before: the records of the kblk whole blocks of tiles before this one, then those of the itile
    // earlier tiles of its own block (a row of 1024 tiles costs its last tile 31 + 31 records, not 1023), RT per round
    const int lbb = P.ntiles > kLbDirect ? kLbBlock : P.ntiles;   // tiles per block record (the whole row: none)
    const int kblk = tile / lbb, itile = tile - kblk * lbb;
    const int nprev = kblk + itile;
    const unsigned long long* bsrc = P.brec + (size_t)b * P.nblk * W;
    const unsigned long long* tsrc = P.rec + (trow + (size_t)kblk * lbb) * W;
    const int nrb = kblk;                             // block records come first in the list
    Moments accB = {0.f, 0.f, 0.f}, accT = {0.f, 0.f, 0.f};
    uint32_t prevcnt = 0;
    auto fetch = [&](const int r0, const int r1) {      // records r0 .. r1 - 1 of the list
    for (int p0 = r0; p0 < r1; p0 += RT) {
      const int np = min(RT, r1 - p0);
      __syncthreads();                              // the staging buffers are free again
      {
        // all loads of a batch are issued before the first one is looked at
        constexpr int kBatch = 8;
        const int nw = np * WS;                       // staged words of this pass
        auto word = [&](const int i) -> const unsigned long long* {
          const int r = i / WS, k = i - r * WS;       // record of the pass, word of the staged record
          const int rec = p0 + r;                     // record in the list of all records
          const int wsrc = k == 0 ? 0 : wlo + k - 1;
          return (rec < nrb ? bsrc + (size_t)rec * W : tsrc + (size_t)(rec - nrb) * W) + wsrc;
        };
        for (int i0 = tid; i0 < nw; i0 += kThreads * kBatch) {
          unsigned long long w[kBatch];
#pragma unroll
          for (int u = 0; u < kBatch; ++u) {
            const int i = i0 + u * kThreads;
            w[u] = i < nw ? get_rec(word(i)) : tagged(0u, tag);
          }
          // words that are not there yet are asked for again together, one round trip per round
          uint32_t spins = 0;
          for (;;) {
            bool pending = false;
#pragma unroll
            for (int u = 0; u < kBatch; ++u) pending |= (uint32_t)(w[u] >> 32) != tag;
            if (!pending) break;
            if (++spins > P.lb.spin_limit) {
              s_gave_up = 1u;
              report_give_up(P.hdr, P.lb.status);
              break;
            }
            __builtin_amdgcn_s_sleep(1);
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
              const int i = i0 + u * kThreads;
              if ((uint32_t)(w[u] >> 32) != tag) w[u] = get_rec(word(i));
            }
          }
#pragma unroll
          for (int u = 0; u < kBatch; ++u) {
            const int i = i0 + u * kThreads;
            if (i < nw) s_lbw[i] = w[u];
          }
        }
      }
      __syncthreads();
      for (int i = l16; i < np; i += 16) {
        const unsigned long long* rw = s_lbw + i * WS;
        const uint32_t c = (uint32_t)rw[0];
        Moments a;
        a.n = (float)c;
        a.mean = __uint_as_float((uint32_t)rw[1 + 2 * (gc - gbase)]);
        a.var = __uint_as_float((uint32_t)rw[2 + 2 * (gc - gbase)]);
        if (p0 + i < kblk) accB = merge(accB, a);
        else accT = merge(accT, a);
        prevcnt += c;
      }
    }
    };
    // the last tile of a block first collects the block's own tiles and leaves the block's aggregate for the tiles
    // of the later blocks, then turns to the earlier blocks: a block record never waits for another block record.
    // A tile that gave up leaves nothing, so that the later ones give up as well instead of building on a partial sum
    const bool closes_block = itile == lbb - 1 && P.ntiles > kLbDirect;
    if (closes_block) {
      fetch(kblk, nprev);
      accT = row_reduce(accT);
      if (l16 == 15 && active && s_gave_up == 0u) {
        unsigned long long* mine = P.brec + ((size_t)b * P.nblk + kblk) * W;
        const Moments ba = merge(accT, inc);
        put_rec(mine + 1 + 2 * g, tagged(__float_as_uint(ba.mean), tag));
        put_rec(mine + 2 + 2 * g, tagged(__float_as_uint(ba.var), tag));
        if (g == 0) put_rec(mine, tagged((uint32_t)ba.n, tag));
      }
      fetch(0, kblk);
    } else {
      fetch(0, nprev);
      accT = row_reduce(accT);
    }
    MEGA_TSN_TR(3);
    Moments acc = merge(row_reduce(accB), accT);
    // words that never came: everything this tile derives from the earlier tiles is NaN, not a partial sum
    const bool poison = s_gave_up != 0u;
    if (poison) acc.mean = __builtin_nanf("");
    const uint32_t prevtot = row_sum_u32(prevcnt);    // the lanes hold disjoint sets of earlier tiles
    Moments prior = prior0;
    if (gbase != 0) prior = Moments{(float)P.prev_count[b], P.prev_mean[(size_t)b * G + gc], P.prev_var[(size_t)b * G + gc]};
    const Moments carry = merge(prior, acc);
    const Moments base = merge(carry, exc);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int tok = l16 * TPL + u;
      if (u < TPL && tok < nt && active) {
        const Moments full = merge(base, pref[u]);
        const float rstd = __builtin_amdgcn_rsqf(full.var + P.eps);
        s_mean[tok * G + g] = full.mean;
        s_var[tok * G + g] = rstd;
        const size_t o = ((size_t)b * P.L + t0 + tok) * G + g;
        if (P.cummean) P.cummean[o] = full.mean;
        if (P.cumrstd) P.cumrstd[o] = rstd;
      }
    }
    if (last_tile && l16 == 15 && active) {
      const Moments fin = merge(carry, inc);
      P.mean[(size_t)b * G + g] = fin.mean;
      P.var[(size_t)b * G + g] = fin.var;
      if (g == 0) P.count[b] = poison ? (int64_t)-1 : P.prev_count[b] + (int64_t)prevtot + (int64_t)inc.n;
    }
  }
  __syncthreads();
  MEGA_TSN_TR(4);

  // ---- normalise and store
#pragma unroll
  for (int j = 0; j < kNV; ++j) {
    const int v = j * kThreads + tid;
    if (v < nvec) {
      const int tok = HOIST ? tok0 + j * tps : v / TPT;
      const int vi = HOIST ? vi0 : v - tok * TPT;
      const int g = HOIST ? g0 : vi / LPG;
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
      const float rr = masked ? 0.f : r;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float a = rr * gam[i];
        const float c = masked ? 0.f : bet[i] - m * a;
        out.v[i] = from_float<T>(to_float(xv[j].v[i]) * a + c);
      }
      yout[v] = out;
    }
  }

  MEGA_TSN_TR(5);
  // ---- retire: the last workgroup to finish opens the next epoch (two-level count so that no
  // single address sees one atomic per workgroup)
  if (tid == 0) {
    const uint32_t total = gridDim.x;
    const uint32_t k = blockIdx.x & 31u;
    const uint32_t quota = (total - k + 31u) / 32u;
    if (atomicAdd(&P.hdr->done1[k], 1u) == quota - 1u) {
      publish_u32(&P.hdr->done1[k], 0u);
      const uint32_t classes = total < 32u ? total : 32u;
      if (atomicAdd(&P.hdr->done2, 1u) == classes - 1u) {
        publish_u32(&P.hdr->done2, 0u);
        publish_u32(&P.hdr->epoch, tag == 0xffffffffu ? 0u : tag);
      }
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

// ---- the per-feature variant in parallel over time (fairseq/csrc/ops/timestep_norm_kernel.cu:73-185 scans time
// in parallel as well).  Time is cut into tiles of kFeatTT tokens:
//   feature_tile_moments   one thread per (row, tile, feature): Welford state of the tile from an empty start
//   feature_tile_scan      one thread per (row, feature): the states become "everything before the tile",
//                          prior included (WelfordCombine, fairseq/csrc/utils.h:66-76), in place
//   feature_tile_apply     one thread per (row, tile, feature): the per-element update of the serial kernel from
//                          that start, normalise, store; the last tile writes the final state
// x is read twice and y written once; the states are 12 bytes per feature and tile.
#ifndef MEGA_FEAT_TT
#define MEGA_FEAT_TT 64
#endif
constexpr int kFeatTT = MEGA_FEAT_TT;

struct FeatArgs {
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
  float* cummean;
  float* cumrstd;
  float* agg;            // [B][ntiles][3][H]: count (as float; after the scan: as int bits), mean, variance
  int B, L, H, ntiles;
  float eps;
};

// V features per thread (16-byte loads when the row length allows it)
template <typename T, int V>
__global__ __launch_bounds__(kThreads) void feature_tile_moments(const FeatArgs A) {
  const int h = (blockIdx.x * kThreads + threadIdx.x) * V;
  const int tile = blockIdx.y, b = blockIdx.z;
  if (h >= A.H) return;
  const int t0 = tile * kFeatTT, t1 = min(A.L, t0 + kFeatTT);
  const T* x = (const T*)A.x;
  int m0 = 0;
  float u[V], v[V];
#pragma unroll
  for (int i = 0; i < V; ++i) u[i] = v[i] = 0.f;
  constexpr int kB = 8;                              // tokens requested together (the loads do not wait for each other)
  for (int tb = t0; tb < t1; tb += kB) {
    Vec<T, V> xv[kB];
    bool skip[kB];
#pragma unroll
    for (int k = 0; k < kB; ++k) {
      const int t = min(tb + k, t1 - 1);
      xv[k] = *(const Vec<T, V>*)(x + ((size_t)b * A.L + t) * A.H + h);
      skip[k] = tb + k >= t1 || (A.mask && A.mask[(size_t)b * A.L + t]);
    }
#pragma unroll
    for (int k = 0; k < kB; ++k) {
      if (skip[k]) continue;
      const float coef = 1.0f / (float)(m0 + 1);
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float xf = to_float(xv[k].v[i]);
        const float d1 = xf - u[i];
        const float m1 = u[i] + coef * d1;
        v[i] = v[i] + coef * (d1 * (xf - m1) - v[i]);
        u[i] = m1;
      }
      ++m0;
    }
  }
  float* a = A.agg + (((size_t)b * A.ntiles + tile) * 3) * A.H + h;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    a[i] = (float)m0;
    a[(size_t)A.H + i] = u[i];
    a[2 * (size_t)A.H + i] = v[i];
  }
}

__global__ __launch_bounds__(kThreads) void feature_tile_scan(const FeatArgs A) {
  const int h = blockIdx.x * kThreads + threadIdx.x;
  const int b = blockIdx.y;
  if (h >= A.H) return;
  int64_t cnt = A.prev_count[b];
  Moments run = {(float)cnt, A.prev_mean[(size_t)b * A.H + h], A.prev_var[(size_t)b * A.H + h]};
  constexpr int kB = 8;                                // tiles requested together
  const int64_t c0 = cnt;
  for (int tb = 0; tb < A.ntiles; tb += kB) {
    Moments own[kB];
#pragma unroll
    for (int k = 0; k < kB; ++k) {
      const int tile = min(tb + k, A.ntiles - 1);
      const float* a = A.agg + (((size_t)b * A.ntiles + tile) * 3) * A.H + h;
      own[k] = Moments{a[0], a[(size_t)A.H], a[2 * (size_t)A.H]};
    }
#pragma unroll
    for (int k = 0; k < kB; ++k) {
      const int tile = tb + k;
      if (tile >= A.ntiles) break;
      float* a = A.agg + (((size_t)b * A.ntiles + tile) * 3) * A.H + h;
      a[0] = __int_as_float((int)(cnt - c0));              // tokens of this call before the tile (exact)
      a[(size_t)A.H] = run.mean;
      a[2 * (size_t)A.H] = run.var;
      if (own[k].n > 0.f) run = combine(run, own[k]);      // a fully masked tile leaves the state as it is
      cnt += (int64_t)own[k].n;
    }
  }
}

template <typename T, int V>
__global__ __launch_bounds__(kThreads) void feature_tile_apply(const FeatArgs A) {
  const int h = (blockIdx.x * kThreads + threadIdx.x) * V;
  const int tile = blockIdx.y, b = blockIdx.z;
  if (h >= A.H) return;
  const int t0 = tile * kFeatTT, t1 = min(A.L, t0 + kFeatTT);
  const T* x = (const T*)A.x;
  T* y = (T*)A.y;
  const float* a = A.agg + (((size_t)b * A.ntiles + tile) * 3) * A.H + h;
  int64_t m0 = A.prev_count[b] + (int64_t)__float_as_int(a[0]);
  float u[V], v[V], w[V], bb[V];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    u[i] = a[(size_t)A.H + i];
    v[i] = a[2 * (size_t)A.H + i];
    w[i] = A.gamma[h + i];
    bb[i] = A.beta[h + i];
  }
  constexpr int kB = 8;                              // tokens requested together
  for (int tb = t0; tb < t1; tb += kB) {
    Vec<T, V> xq[kB];
    bool mk[kB];
#pragma unroll
    for (int k = 0; k < kB; ++k) {
      const int t = min(tb + k, t1 - 1);
      xq[k] = *(const Vec<T, V>*)(x + ((size_t)b * A.L + t) * A.H + h);
      mk[k] = A.mask && A.mask[(size_t)b * A.L + t];
    }
#pragma unroll
    for (int k = 0; k < kB; ++k) {
    const int t = tb + k;
    if (t >= t1) break;
    const size_t o = ((size_t)b * A.L + t) * A.H + h;
    const bool masked = mk[k];
    const Vec<T, V> xv = xq[k];
    const float coef = 1.0f / (float)(m0 + 1);
    Vec<T, V> out;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const float xf = to_float(xv.v[i]);
      const float d1 = xf - u[i];
      const float m1 = u[i] + coef * d1;
      const float m2 = v[i] + coef * (d1 * (xf - m1) - v[i]);
      const float rstd = __builtin_amdgcn_rsqf(m2 + A.eps);
      out.v[i] = from_float<T>(masked ? 0.f : (xf - m1) * rstd * w[i] + bb[i]);
      if (!masked) {
        u[i] = m1;
        v[i] = m2;
      }
      if (A.cummean) A.cummean[o + i] = masked ? u[i] : m1;
      if (A.cumrstd) A.cumrstd[o + i] = masked ? __builtin_amdgcn_rsqf(v[i] + A.eps) : rstd;
    }
    *(Vec<T, V>*)(y + o) = out;
    if (!masked) ++m0;
    }
  }
  if (tile == A.ntiles - 1) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      A.mean[(size_t)b * A.H + h + i] = u[i];
      A.var[(size_t)b * A.H + h + i] = v[i];
    }
    if (h == 0) A.count[b] = m0;
  }
}

constexpr int kFeatSerialMax = 2 * kFeatTT;           // rows up to this many tokens take the serial kernel
size_t feature_tsn_workspace_bytes(int64_t B, int64_t L, int64_t H) {
  if (L <= kFeatSerialMax) return 0;
  return (size_t)B * (size_t)ceil_div(L, kFeatTT) * 3 * (size_t)H * 4;
}

struct TsnGeom {
  int vec, tpt, lpg, tt, ntiles, lpgt;
  size_t smem;
};

bool tsn_geometry(int dtype, int64_t B, int64_t L, int64_t H, int64_t G, TsnGeom* g) {
  const int esize = dtype == MEGA_F32 ? 4 : 2;
  const int64_t dg = H / G;
  int vec = 16 / esize;
  while (vec > 1 && dg % vec != 0) vec /= 2;
  const int64_t tpt = H / vec;
  if (tpt > kPartCap || 2 * G + 1 > kLbWords) return false;
  int tt = (int)(kPartCap / tpt);
  if (tt > kMaxTT) tt = kMaxTT;
  while (tt > 8 && B * ceil_div(L, tt) < 512) tt /= 2;
  if (tt > L) tt = (int)L;
  if (tt < 1) tt = 1;
  g->vec = vec;
  g->tpt = (int)tpt;
  g->lpg = (int)(dg / vec);
  g->tt = tt;
  g->ntiles = (int)ceil_div(L, tt);
  const int lpg = g->lpg;
  g->lpgt = (lpg <= 64 && (lpg & (lpg - 1)) == 0) ? lpg : 0;
  size_t bytes = 2 * (size_t)tt * G * 4 + align_up((size_t)tt, 16) + (size_t)kLbWords * 8;
  if (g->lpgt == 0) bytes += (size_t)kPartCap * (esize == 2 && vec >= 2 ? 8 : 4);   // 16-bit: (sum, sum of squares)
  g->smem = bytes;
  return g->smem <= 150 * 1024;
}

template <typename T, int VEC, int LPGT>
int launch_group_tsn2(const TsnParams& P, const TsnGeom& g, hipStream_t stream) {
  const bool hoist = (kThreads % g.tpt) == 0;
  const dim3 grid((unsigned)(P.B * P.ntiles));
  auto kern = hoist ? group_tsn_kernel<T, VEC, true, LPGT> : group_tsn_kernel<T, VEC, false, LPGT>;
  if (g.smem > 64 * 1024) {
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)g.smem);
  }
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), g.smem, stream, P);
  MEGA_CHECK_LAUNCH("group_timestep_norm_fwd");
  return MEGA_OK;
}

template <typename T, int VEC>
int launch_group_tsn(const TsnParams& P, const TsnGeom& g, hipStream_t stream) {
  switch (g.lpgt) {
    case 1: return launch_group_tsn2<T, VEC, 1>(P, g, stream);
    case 2: return launch_group_tsn2<T, VEC, 2>(P, g, stream);
    case 4: return launch_group_tsn2<T, VEC, 4>(P, g, stream);
    case 8: return launch_group_tsn2<T, VEC, 8>(P, g, stream);
    case 16: return launch_group_tsn2<T, VEC, 16>(P, g, stream);
    case 32: return launch_group_tsn2<T, VEC, 32>(P, g, stream);
    case 64: return launch_group_tsn2<T, VEC, 64>(P, g, stream);
    default: return launch_group_tsn2<T, VEC, 0>(P, g, stream);
  }
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

// header, tile records, block records
size_t tsn_workspace_bytes(int64_t B, int64_t G, int ntiles) {
  const size_t n = (size_t)B * ntiles + (size_t)B * ceil_div(ntiles, kLbBlock);
  return align_up(sizeof(TsnHeader), 256) + align_up(n * (2 * (size_t)G + 1) * 8, 256);
}

}  // namespace

}  // namespace mega

using namespace mega;

extern "C" size_t mega_timestep_norm_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t H, int64_t G) {
  // G == H names both the per-feature variant (mega_timestep_norm_fwd) and the group variant with one channel per
  // group (mega_group_timestep_norm_fwd): the size covers whichever entry point the workspace is handed to
  size_t need = 256;
  if (B > 0 && L > 0 && H > 0 && G == H) {
    const size_t f = feature_tsn_workspace_bytes(B, L, H);
    need = f > need ? f : need;
  }
  TsnGeom g;
  if (B > 0 && L > 0 && H > 0 && G > 0 && H % G == 0 && tsn_geometry(dtype, B, L, H, G, &g)) {
    const size_t t = tsn_workspace_bytes(B, G, g.ntiles);
    need = t > need ? t : need;
  }
  return need;
}

static int group_tsn_fwd_impl(const void* x, void* y, int dtype, const int64_t* prev_count,
                              const float* prev_mean, const float* prev_var, const float* gamma,
                              const float* beta, const uint8_t* mask, int64_t B, int64_t L, int64_t H,
                              int64_t G, double eps, int64_t* count, float* mean, float* var,
                              float* group_mean, float* cummean, float* cumrstd, void* workspace,
                              size_t workspace_bytes, bool fixed_scratch, void* stream) {
  if (const int rc = lookback_pending("group_timestep_norm_fwd")) return rc;
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
  // every tile of a row reads the prior state while the row's last tile writes the new one
  MEGA_REQUIRE(!ranges_overlap(prev_count, (size_t)B * 8, count, (size_t)B * 8) &&
                   !ranges_overlap(prev_mean, (size_t)B * G * 4, mean, (size_t)B * G * 4) &&
                   !ranges_overlap(prev_var, (size_t)B * G * 4, var, (size_t)B * G * 4),
               MEGA_ERR_ARG,
               "group_timestep_norm_fwd: count / mean / var must not overlap prev_count / prev_mean / prev_var "
               "(the state is not updated in place)");
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
  if (fixed_scratch) {
    MEGA_REQUIRE(workspace_bytes >= tsn_workspace_bytes(B, G, g.ntiles), MEGA_ERR_UNSUPPORTED,
                 "group_timestep_norm_fwd_noalloc: B=%ld L=%ld G=%ld needs %zu bytes of tile records, the library's "
                 "fixed scratch array holds %zu (B * (T + ceil(T / 32)) * (2 G + 1) * 8 + 256 with T = ceil(L / %d) must fit); use "
                 "mega_group_timestep_norm_fwd with a caller workspace",
                 (long)B, (long)L, (long)G, tsn_workspace_bytes(B, G, g.ntiles), workspace_bytes, g.tt);
  }
  MEGA_REQUIRE(workspace != nullptr && workspace_bytes >= tsn_workspace_bytes(B, G, g.ntiles),
               MEGA_ERR_WORKSPACE, "group_timestep_norm_fwd: workspace of %zu bytes needed",
               tsn_workspace_bytes(B, G, g.ntiles));
  char* w = (char*)workspace;
  TsnParams P;
  P.x = x; P.y = y; P.prev_count = prev_count; P.prev_mean = prev_mean; P.prev_var = prev_var;
  P.gamma = gamma; P.beta = beta; P.mask = mask; P.count = count; P.mean = mean; P.var = var;
  P.group_mean = group_mean; P.cummean = cummean; P.cumrstd = cumrstd;
  P.hdr = (TsnHeader*)w; w += align_up(sizeof(TsnHeader), 256);
  P.rec = (unsigned long long*)w;
  P.brec = P.rec + (size_t)B * g.ntiles * (2 * (size_t)G + 1);
  P.B = (int)B; P.L = (int)L; P.H = (int)H; P.G = (int)G;
  P.TT = g.tt; P.ntiles = g.ntiles; P.nblk = (int)ceil_div(g.ntiles, kLbBlock); P.TPT = g.tpt; P.LPG = g.lpg; P.eps = (float)eps;
  P.lb = lookback_launch(!fixed_scratch);
  int rc;
  switch (dtype) {
    case MEGA_F32: rc = dispatch_vec<float>(P, g, s); break;
    case MEGA_BF16: rc = dispatch_vec<bf16_t>(P, g, s); break;
    default: rc = dispatch_vec<f16_t>(P, g, s); break;
  }
  // the entry point that may not allocate may not wait either (it serves callers under stream capture)
  return rc != MEGA_OK || fixed_scratch ? rc : lookback_verify("group_timestep_norm_fwd", s);
}

extern "C" int mega_group_timestep_norm_fwd(const void* x, void* y, int dtype,
                                            const int64_t* prev_count, const float* prev_mean,
                                            const float* prev_var, const float* gamma,
                                            const float* beta, const uint8_t* mask, int64_t B,
                                            int64_t L, int64_t H, int64_t G, double eps,
                                            int64_t* count, float* mean, float* var,
                                            float* group_mean, float* cummean, float* cumrstd,
                                            void* workspace, size_t workspace_bytes, void* stream) {
  return group_tsn_fwd_impl(x, y, dtype, prev_count, prev_mean, prev_var, gamma, beta, mask, B, L, H, G, eps, count,
                            mean, var, group_mean, cummean, cumrstd, workspace, workspace_bytes, false, stream);
}

// ---------------------------------------------------------------- the same call without a workspace argument
// For callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc): the launch epoch, retire counters and tile records live in a
// file-scope device array instead of a caller workspace.  Every GPU holds its own copy of the array
// at its own address; host code never uses the array's name as an address (it is a host-side
// stand-in), only the pointer hipGetSymbolAddress returns for the current device, looked up once per
// device.  The array starts zero-filled (device globals do), which is the "zero once" the workspace
// protocol asks for; after that every launch leaves the header consistent and the records carry
// launch tags, so nothing is cleared between calls even when the shape changes.  All calls on one
// GPU share the array: calls that can overlap in time (two streams) race.
namespace {
constexpr size_t kStaticScratchBytes = (size_t)1 << 20;
constexpr int kMaxDevices = 64;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* g_scratch_ptr[kMaxDevices];   // per device: the address of that device's copy, 0 = not looked up yet

static int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  MEGA_REQUIRE(e == hipSuccess && dev >= 0 && dev < kMaxDevices, MEGA_ERR_LAUNCH,
               "group_timestep_norm_fwd_noalloc: no current HIP device (%s)", hipGetErrorString(e));
  void* p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    MEGA_REQUIRE(e == hipSuccess && p != nullptr, MEGA_ERR_LAUNCH,
                 "group_timestep_norm_fwd_noalloc: hipGetSymbolAddress failed on device %d: %s", dev,
                 hipGetErrorString(e));
    __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);   // two threads racing here store the same address
  }
  *out = p;
  return MEGA_OK;
}

extern "C" int mega_group_timestep_norm_fwd_noalloc(const void* x, void* y, int dtype,
                                                    const int64_t* prev_count, const float* prev_mean,
                                                    const float* prev_var, const float* gamma,
                                                    const float* beta, const uint8_t* mask, int64_t B,
                                                    int64_t L, int64_t H, int64_t G, double eps,
                                                    int64_t* count, float* mean, float* var,
                                                    float* group_mean, float* cummean, float* cumrstd,
                                                    void* stream) {
  void* ptr = nullptr;
  const int rc = static_scratch(&ptr);
  if (rc != MEGA_OK) return rc;
  // a give-up of a bounded wait is reported through the device's status word, which this entry point may not create
  // (creating it allocates pinned host memory): without it a failure would show only as NaN outputs
  MEGA_REQUIRE(lookback_launch(false).status != nullptr, MEGA_ERR_UNSUPPORTED,
               "group_timestep_norm_fwd_noalloc: call mega_lookback_init() once per device first (outside graph "
               "capture): it creates the status word through which a failed wait is reported");
  return group_tsn_fwd_impl(x, y, dtype, prev_count, prev_mean, prev_var, gamma, beta, mask, B, L, H, G, eps, count,
                            mean, var, group_mean, cummean, cumrstd, ptr, kStaticScratchBytes, true, stream);
}

extern "C" int mega_timestep_norm_fwd(const void* x, void* y, int dtype, const int64_t* prev_count,
                                      const float* prev_mean, const float* prev_var,
                                      const float* gamma, const float* beta, const uint8_t* mask,
                                      int64_t B, int64_t L, int64_t H, double eps, int64_t* count,
                                      float* mean, float* var, float* cummean, float* cumrstd,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "timestep_norm_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && L >= 0 && H > 0, MEGA_ERR_ARG, "timestep_norm_fwd: bad shape");
  MEGA_REQUIRE(B < 65536 && B * L * H < (int64_t)1 << 40, MEGA_ERR_UNSUPPORTED, "timestep_norm_fwd: too large");
  if (B == 0) return MEGA_OK;
  MEGA_REQUIRE(prev_count && prev_mean && prev_var && gamma && beta && count && mean && var, MEGA_ERR_ARG,
               "timestep_norm_fwd: null state / parameter pointer");
  // every block of features of a row reads prev_count while the first one writes count
  MEGA_REQUIRE(!ranges_overlap(prev_count, (size_t)B * 8, count, (size_t)B * 8), MEGA_ERR_ARG,
               "timestep_norm_fwd: count must not overlap prev_count");
  MEGA_REQUIRE(L == 0 || (x && y), MEGA_ERR_ARG, "timestep_norm_fwd: null x / y");
  hipStream_t s = (hipStream_t)stream;
  {
    // with a workspace: three kernels parallel over time tiles; without (or for short sequences): one thread per
    // (row, feature) walks the whole sequence
    const size_t need = feature_tsn_workspace_bytes(B, L, H);
    const int64_t ntiles = ceil_div(L, kFeatTT);
    if (need > 0 && workspace && workspace_bytes >= need && ((uintptr_t)workspace % 4) == 0 && ntiles < 65536) {
      // mean / var may be the prior buffers (the scan has consumed the prior before the last tile writes), count not
      FeatArgs A;
      A.x = x; A.y = y; A.prev_count = prev_count; A.prev_mean = prev_mean; A.prev_var = prev_var; A.gamma = gamma;
      A.beta = beta; A.mask = mask; A.count = count; A.mean = mean; A.var = var; A.cummean = cummean;
      A.cumrstd = cumrstd; A.agg = (float*)workspace; A.B = (int)B; A.L = (int)L; A.H = (int)H; A.ntiles = (int)ntiles;
      A.eps = (float)eps;
      const int es = dtype == MEGA_F32 ? 4 : 2;
      // 8-byte pieces per thread: enough threads to fill the chip at 64 tokens per tile
      const bool wide = H % (8 / es) == 0 && ((uintptr_t)x % 8) == 0 && ((uintptr_t)y % 8) == 0;
      const int64_t hv = wide ? H / (8 / es) : H;                  // threads along the features
      const dim3 gt((unsigned)ceil_div(hv, kThreads), (unsigned)ntiles, (unsigned)B);
      const dim3 gs((unsigned)ceil_div(H, kThreads), (unsigned)B);
#define LAUNCH_FPAR(T, V)                                                                \
  hipLaunchKernelGGL((feature_tile_moments<T, V>), gt, dim3(kThreads), 0, s, A);         \
  hipLaunchKernelGGL(feature_tile_scan, gs, dim3(kThreads), 0, s, A);                    \
  hipLaunchKernelGGL((feature_tile_apply<T, V>), gt, dim3(kThreads), 0, s, A)
      if (wide) {
        switch (dtype) {
          case MEGA_F32: LAUNCH_FPAR(float, 2); break;
          case MEGA_BF16: LAUNCH_FPAR(bf16_t, 4); break;
          default: LAUNCH_FPAR(f16_t, 4); break;
        }
      } else {
        switch (dtype) {
          case MEGA_F32: LAUNCH_FPAR(float, 1); break;
          case MEGA_BF16: LAUNCH_FPAR(bf16_t, 1); break;
          default: LAUNCH_FPAR(f16_t, 1); break;
        }
      }
#undef LAUNCH_FPAR
      MEGA_CHECK_LAUNCH("timestep_norm_fwd (time tiles)");
      return MEGA_OK;
    }
  }
  // one thread per (row, feature) walking the whole sequence: right for short rows, two orders of magnitude slower
  // than the tiled kernels for long ones, so a long row without its workspace is refused rather than served slowly
  MEGA_REQUIRE(L <= kFeatSerialMax, MEGA_ERR_WORKSPACE,
               "timestep_norm_fwd: L = %ld needs a workspace of %zu bytes (mega_timestep_norm_workspace_bytes with "
               "G = H); without one only rows of up to %d tokens are served",
               (long)L, feature_tsn_workspace_bytes(B, L, H), kFeatSerialMax);
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
