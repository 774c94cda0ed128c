// Parameter-gradient sums of the moving-average layer on the matrix cores (16-bit activations,
// no mask, kernel lags from 0: the common training case).  Same result as ema_param_grad_kernel
// (ema_bwd.hip): per batch row and channel
//     sum2[n] = sum_t dy[t] s_n[t],   sum1[n] = sum_t dy[t] g_n[t],   dyx = sum_t dy[t] x[t]
// with s[t] = q s[t-1] + x[t] and g = ds/dq, which are the reference's
//     sum_l dk[l] q^l  and  sum_l dk[l] l q^(l-1)      (fairseq/csrc/ops/ema_parameters.cc:80-97)
// for the kernel gradient dk[l] = sum_t dy[t] x[t-l] of fftconv's backward
// (fairseq/modules/fused_ops/fftconv.py:66-88).
//
// Time is cut into tiles of 32 tokens.  With h_k = s at the last token of tile k, hd_k = dh_k/dq,
// Q = q^32 and Qd = 32 q^31:
//     s[32k+t] = q^(t+1) h_(k-1) + (tile-local part),
//     h_k  = Q h_(k-1) + b_k,                    b_k  = sum_j q^(31-j) x_k[j]
//     hd_k = Q hd_(k-1) + Qd h_(k-1) + bd_k,     bd_k = sum_j (31-j) q^(30-j) x_k[j]
//     sum2 = sum_k a_k h_(k-1) + sum_l q^l C[l],                      a_k  = sum_t q^(t+1) dy_k[t]
//     sum1 = sum_k (ad_k h_(k-1) + a_k hd_(k-1)) + sum_l l q^(l-1) C[l],  ad_k = sum_t (t+1) q^t dy_k[t]
// where C[l] = sum_t M[t][t-l] collects the diagonals of the tile-local correlation matrix
// M[t][j] = sum_k dy_k[t] x_k[j]  (C[0] is dyx).  a, ad, b, bd are products of constant 32 x 32
// tables (powers of q, two bf16 terms each) with 16 tiles at a time, M is a product of the data
// with itself: all of it v_mfma_f32_16x16x32_bf16.  What remains on the vector ALUs is one short
// recurrence per tile instead of one per token.
//
// One workgroup = 8 channels of one batch row, one wave per channel; a step is 512 tokens:
//   park the prefetched x / dy pieces in LDS (one row per channel, time-contiguous)
//   pass 1 (every wave, its channel): the table products; b, bd go to LDS, a, ad stay in registers
//   scan (threads = channel x state): walk the 16 tiles, replace (b, bd) by (h, hd) before the tile
//   pass 2 (every wave): sum2 += a h, sum1 += ad h + a hd in the product's own lane layout.
#include "common.h"

namespace mega {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kTCh = 8;                    // channels (= waves) per workgroup
constexpr int kTThreads = kTCh * 64;
constexpr int kStep = 512;                 // tokens per step: 16 tiles of 32
constexpr int kRowB = kStep * 2 + 16;      // bytes of one channel's row of a step in LDS
constexpr int kTileB = 16 * 16 + 16;       // bytes of one tile's 16 states x (b, bd) in LDS

struct TileGradArgs {
  const uint16_t* dy;
  const uint16_t* x;
  int64_t sgb, sgd, sgl;    // dy strides (elements)
  int64_t sxb, sxd, sxl;    // x strides
  const float* q;           // [D, N, 2]
  float* sums;              // [B, D, N, 4]
  float* dyx;               // [B, D]
  int B, D, N, L;
  int x_chan_fast, g_chan_fast;
};

__device__ __forceinline__ cfloat cpow_small(cfloat q, int e) {     // q^e, 0 <= e < 64
  cfloat r = {1.f, 0.f};
  cfloat b = q;
#pragma unroll
  for (int i = 0; i < 6; ++i) {
    if (e & (1 << i)) r = cmul(r, b);
    b = cmul(b, b);
  }
  return r;
}

// v as two bf16 terms
__device__ __forceinline__ void split2(float v, __bf16& hi, __bf16& lo) {
  hi = (__bf16)v;
  lo = (__bf16)(v - (float)hi);
}

__global__ __launch_bounds__(kTThreads) void ema_param_grad_tile_kernel(const TileGradArgs A) {
  __shared__ __attribute__((aligned(16))) char s_x[kTCh * kRowB];
  __shared__ __attribute__((aligned(16))) char s_g[kTCh * kRowB];
  __shared__ __attribute__((aligned(16))) char s_out[kTCh * 16 * kTileB];
  __shared__ __attribute__((aligned(16))) char s_zero[kStep];     // what the unused k slots of the data product read
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int col = lane & 15, r = lane >> 4;
  // workgroups that share the lines of a channel-contiguous operand get ids on one XCD
  const int total = gridDim.x;
  const int v = (total % 8 == 0) ? (int)(blockIdx.x % 8) * (total / 8) + (int)(blockIdx.x / 8) : (int)blockIdx.x;
  const int ncb = A.D / kTCh;
  const int b = v / ncb;
  const int c0 = (v - b * ncb) * kTCh;
  const int d = c0 + wave;                                  // this wave's channel

  // ---- loads: one 16-byte piece of x and of dy per thread and step
  // channel-contiguous operand: thread <-> token, the piece holds the 8 channels;
  // time-contiguous operand: thread <-> (channel, group of 8 tokens)
  const int lmax = A.L - 1;
  const uint16_t* xb = A.x + (int64_t)b * A.sxb + (A.x_chan_fast ? (int64_t)c0 : (int64_t)(c0 + (tid >> 6)) * A.sxd);
  const uint16_t* gb = A.dy + (int64_t)b * A.sgb + (A.g_chan_fast ? (int64_t)c0 : (int64_t)(c0 + (tid >> 6)) * A.sgd);
  const int xtok = A.x_chan_fast ? tid : 8 * (tid & 63);      // first token of the piece inside a step
  const int gtok = A.g_chan_fast ? tid : 8 * (tid & 63);
  const int xlast = A.x_chan_fast ? lmax : A.L - 8;           // last valid first-token
  const int glast = A.g_chan_fast ? lmax : A.L - 8;
  uint4 px, pg;
  auto fetch = [&](int t0) {
    px = *(const uint4*)(xb + (int64_t)min(t0 + xtok, xlast) * A.sxl);
    pg = *(const uint4*)(gb + (int64_t)min(t0 + gtok, glast) * A.sgl);
  };
  auto park = [&](char* base, const uint4& p, bool chan_fast, int tok, bool valid) {
    const uint4 z = valid ? p : make_uint4(0u, 0u, 0u, 0u);
    if (chan_fast) {
      const uint32_t w[4] = {z.x, z.y, z.z, z.w};
#pragma unroll
      for (int e = 0; e < 8; ++e)
        *(uint16_t*)(base + e * kRowB + tok * 2) = (uint16_t)(w[e >> 1] >> ((e & 1) * 16));
    } else {
      *(uint4*)(base + (tid >> 6) * kRowB + tok * 2) = z;
    }
  };

  fetch(0);                                  // in flight while the tables are built

  // ---- constant operands: rows = (state, re | im), 16 rows per block, columns = token in tile
  bf16x8 Ta[2][2], Tad[2][2], Tb[2][2], Tbd[2][2];          // [term][row block]
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    const int n = 8 * rb + (col >> 1);
    const bool im = col & 1;
    cfloat q1 = {0.f, 0.f};
    if (n < A.N) {
      q1.re = A.q[((size_t)d * A.N + n) * 2];
      q1.im = A.q[((size_t)d * A.N + n) * 2 + 1];
    }
    cfloat up = cpow_small(q1, 8 * r);                       // q^(8r + e)
    cfloat dn = cpow_small(q1, 24 - 8 * r);                  // q^(24 - 8r + m)
    const cfloat below = r < 3 ? cpow_small(q1, 23 - 8 * r) : cfloat{0.f, 0.f};
    float pu[9], pd[9];                                      // pd[m + 1] = q^(24 - 8r + m), pd[0] = q^(23 - 8r)
    pd[0] = im ? below.im : below.re;
#pragma unroll
    for (int e = 0; e < 9; ++e) {
      pu[e] = im ? up.im : up.re;
      up = cmul(up, q1);
      if (e < 8) {
        pd[e + 1] = im ? dn.im : dn.re;
        dn = cmul(dn, q1);
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int k = 8 * r + e;                               // token in tile
      __bf16 h0, l0;
      split2(pu[e + 1], h0, l0);                             // q^(k+1)
      Ta[0][rb][e] = h0; Ta[1][rb][e] = l0;
      split2((float)(k + 1) * pu[e], h0, l0);                // (k+1) q^k
      Tad[0][rb][e] = h0; Tad[1][rb][e] = l0;
      split2(pd[8 - e], h0, l0);                             // q^(31-k) = q^(24 - 8r + 7 - e)
      Tb[0][rb][e] = h0; Tb[1][rb][e] = l0;
      split2((float)(31 - k) * pd[7 - e], h0, l0);           // (31-k) q^(30-k)
      Tbd[0][rb][e] = h0; Tbd[1][rb][e] = l0;
    }
  }

  // ---- scan threads: (channel, state) with Q = q^32, Qd = 32 q^31 and the carried h, hd
  const int sch = tid >> 4, sn = tid & 15;                   // meaningful for tid < 128
  cfloat Q = {0.f, 0.f}, Qd = {0.f, 0.f}, h = {0.f, 0.f}, hd = {0.f, 0.f};
  if (tid < kTCh * 16 && sn < A.N) {
    cfloat q1;
    q1.re = A.q[((size_t)(c0 + sch) * A.N + sn) * 2];
    q1.im = A.q[((size_t)(c0 + sch) * A.N + sn) * 2 + 1];
    const cfloat q31 = cpow_small(q1, 31);
    Q = cmul(q31, q1);
    Qd = {32.f * q31.re, 32.f * q31.im};
  }

  f32x4 S2a[2], S1a[2];                      // per row block: (state 2r: re, im, state 2r+1: re, im) partial sums
  f32x4 M[2][2];                             // tile-local correlation, blocks [dy half][x half]
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    S2a[i] = S1a[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    M[i][0] = M[i][1] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const char* xrow = s_x + wave * kRowB;
  const char* grow = s_g + wave * kRowB;
  char* orow = s_out + wave * 16 * kTileB;

  s_zero[tid] = 0;
  for (int t0 = 0; t0 < A.L; t0 += kStep) {
    park(s_x, px, A.x_chan_fast, xtok, t0 + xtok <= xlast);
    park(s_g, pg, A.g_chan_fast, gtok, t0 + gtok <= glast);
    __syncthreads();
    fetch(t0 + kStep);                       // clamped past the end; in flight under the arithmetic

    // ---- pass 1: columns = the 16 tiles of the step
    const bf16x8 X = *(const bf16x8*)(xrow + (32 * col + 8 * r) * 2);
    const bf16x8 G = *(const bf16x8*)(grow + (32 * col + 8 * r) * 2);
    f32x4 Sa[2], Sad[2], Sb[2], Sbd[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) Sa[rb] = Sad[rb] = Sb[rb] = Sbd[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
    // term by term, so that products into the same accumulator sit eight instructions apart
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        Sb[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Tb[w][rb], X, Sb[rb], 0, 0, 0);
        Sbd[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Tbd[w][rb], X, Sbd[rb], 0, 0, 0);
        Sa[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Ta[w][rb], G, Sa[rb], 0, 0, 0);
        Sad[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Tad[w][rb], G, Sad[rb], 0, 0, 0);
      }
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      // states 8 rb + 2r and + 1 of tile `col`: (b re, b im, bd re, bd im)
      char* o = orow + col * kTileB + (8 * rb + 2 * r) * 16;
      *(float4*)o = make_float4(Sb[rb][0], Sb[rb][1], Sbd[rb][0], Sbd[rb][1]);
      *(float4*)(o + 16) = make_float4(Sb[rb][2], Sb[rb][3], Sbd[rb][2], Sbd[rb][3]);
    }
    // tile-local correlation: contraction over the 16 tiles; the k slots 16..31 (lanes with r >= 2)
    // read a row of zeros
    {
      const char* gsrc = r < 2 ? grow + (32 * 8 * r + col) * 2 : s_zero;
      const char* xsrc = r < 2 ? xrow + (32 * 8 * r + col) * 2 : s_zero;
      bf16x8 Gt[2], Xt[2];
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int off = (32 * e + 16 * hf) * 2;
          Gt[hf][e] = __builtin_bit_cast(__bf16, *(const uint16_t*)(gsrc + off));
          Xt[hf][e] = __builtin_bit_cast(__bf16, *(const uint16_t*)(xsrc + off));
        }
      }
#pragma unroll
      for (int th = 0; th < 2; ++th)
#pragma unroll
        for (int jh = 0; jh < 2; ++jh)
          M[th][jh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Gt[th], Xt[jh], M[th][jh], 0, 0, 0);
    }
    __syncthreads();

    // ---- scan over the 16 tiles: leave the state before each tile where its (b, bd) was
    if (tid < kTCh * 16) {
      char* o = s_out + sch * 16 * kTileB + sn * 16;
      // groups of four tiles: the next group's (b, bd) are on their way while this one is walked
      float4 in[4], nx[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) in[i] = *(const float4*)(o + i * kTileB);
#pragma unroll
      for (int kg = 0; kg < 4; ++kg) {
        if (kg < 3) {
#pragma unroll
          for (int i = 0; i < 4; ++i) nx[i] = *(const float4*)(o + (4 * kg + 4 + i) * kTileB);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          *(float4*)(o + (4 * kg + i) * kTileB) = make_float4(h.re, h.im, hd.re, hd.im);
          const cfloat nhd = {fmaf(Q.re, hd.re, fmaf(-Q.im, hd.im, fmaf(Qd.re, h.re, fmaf(-Qd.im, h.im, in[i].z)))),
                              fmaf(Q.re, hd.im, fmaf(Q.im, hd.re, fmaf(Qd.re, h.im, fmaf(Qd.im, h.re, in[i].w))))};
          const cfloat nh = {fmaf(Q.re, h.re, fmaf(-Q.im, h.im, in[i].x)), fmaf(Q.re, h.im, fmaf(Q.im, h.re, in[i].y))};
          h = nh;
          hd = nhd;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) in[i] = nx[i];
      }
    }
    __syncthreads();

    // ---- pass 2: sum2 += a h, sum1 += ad h + a hd for the lane's four states of tile `col`
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      const char* o = orow + col * kTileB + (8 * rb + 2 * r) * 16;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const float4 st = *(const float4*)(o + 16 * u);       // h re, h im, hd re, hd im
        const float ar = Sa[rb][2 * u], ai = Sa[rb][2 * u + 1];
        const float dr = Sad[rb][2 * u], di = Sad[rb][2 * u + 1];
        S2a[rb][2 * u] = fmaf(ar, st.x, fmaf(-ai, st.y, S2a[rb][2 * u]));
        S2a[rb][2 * u + 1] = fmaf(ar, st.y, fmaf(ai, st.x, S2a[rb][2 * u + 1]));
        S1a[rb][2 * u] = fmaf(dr, st.x, fmaf(-di, st.y, fmaf(ar, st.z, fmaf(-ai, st.w, S1a[rb][2 * u]))));
        S1a[rb][2 * u + 1] = fmaf(dr, st.y, fmaf(di, st.x, fmaf(ar, st.w, fmaf(ai, st.z, S1a[rb][2 * u + 1]))));
      }
    }
    // the next park overwrites s_x / s_g, which every wave finished reading before the scan
    // barrier; this wave's part of s_out is rewritten by this wave only, after its own reads above
  }

  // ---- per wave: fold the tile columns, add the tile-local part, store
  __syncthreads();                            // the last scan's writes are consumed; s_out is free for reuse
#pragma unroll
  for (int rb = 0; rb < 2; ++rb)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float a = S2a[rb][i], c = S1a[rb][i];
#pragma unroll
      for (int m = 1; m < 16; m <<= 1) {
        a += __shfl_xor(a, m);
        c += __shfl_xor(c, m);
      }
      S2a[rb][i] = a;
      S1a[rb][i] = c;
    }
  float* wbuf = (float*)orow;                 // 16 * kTileB = 4352 bytes: M as [32][33] floats = 4224 bytes
#pragma unroll
  for (int th = 0; th < 2; ++th)
#pragma unroll
    for (int jh = 0; jh < 2; ++jh)
#pragma unroll
      for (int i = 0; i < 4; ++i) wbuf[(16 * th + 4 * r + i) * 33 + 16 * jh + col] = M[th][jh][i];
  __builtin_amdgcn_wave_barrier();            // LDS operations of one wave complete in order
  float C = 0.f;                              // lane l < 32: C[l]
  if (lane < 32)
    for (int t = lane; t < 32; ++t) C += wbuf[t * 33 + t - lane];
  // Horner in q: p = sum_l C[l] q^l, dp = sum_l l C[l] q^(l-1), lanes = states
  cfloat qn = {0.f, 0.f};
  if (lane < A.N) {
    qn.re = A.q[((size_t)d * A.N + lane) * 2];
    qn.im = A.q[((size_t)d * A.N + lane) * 2 + 1];
  }
  cfloat p = {0.f, 0.f}, dp = {0.f, 0.f};
  for (int l = 31; l >= 0; --l) {
    const float cl = __shfl(C, l);
    dp = cadd(cmul(dp, qn), p);
    p = cmul(p, qn);
    p.re += cl;
  }
  // after the fold every lane of group r holds the sums of states 2r, 2r+1 (row block 0) and
  // 8+2r, 8+2r+1 (row block 1); lane n < 16 collects those of state n
  float s2r, s2i, s1r, s1i;
  {
    const int n = lane & 15;
    const int src = ((n & 7) >> 1) * 16;
    const bool hi = n >> 3, odd = n & 1;
    float g2[2][4], g1[2][4];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        g2[rb][i] = __shfl(S2a[rb][i], src);
        g1[rb][i] = __shfl(S1a[rb][i], src);
      }
    s2r = hi ? (odd ? g2[1][2] : g2[1][0]) : (odd ? g2[0][2] : g2[0][0]);
    s2i = hi ? (odd ? g2[1][3] : g2[1][1]) : (odd ? g2[0][3] : g2[0][1]);
    s1r = hi ? (odd ? g1[1][2] : g1[1][0]) : (odd ? g1[0][2] : g1[0][0]);
    s1i = hi ? (odd ? g1[1][3] : g1[1][1]) : (odd ? g1[0][3] : g1[0][1]);
  }
  if (lane < A.N) {
    float4* dst = (float4*)A.sums + ((size_t)b * A.D + d) * A.N + lane;
    *dst = make_float4(s2r + p.re, s2i + p.im, s1r + dp.re, s1i + dp.im);
  }
  const float c0v = __shfl(C, 0);
  if (lane == 0) A.dyx[(size_t)b * A.D + d] = c0v;
}

}  // namespace

// The matrix-core form covers 16-bit bf16 operands without a mask and with lags from 0, whole
// groups of 8 channels, and operands whose 16-byte pieces are aligned: channel-contiguous
// (stride 1 over channels; any token stride that is a multiple of 8, negative for reversed time) or
// time-contiguous (token stride +1, length a multiple of 8).
bool ema_param_grad_tile_covers(int dtype, const void* dy, const void* x, int64_t sgb, int64_t sgd, int64_t sgl,
                                int64_t sxb, int64_t sxd, int64_t sxl, const uint8_t* mask, int64_t B, int64_t D,
                                int64_t N, int64_t L, int lag_one) {
  if (dtype != MEGA_BF16 || mask || lag_one || N > 16 || D % kTCh != 0 || L < 8) return false;
  if (B * (D / kTCh) >= (int64_t)1 << 31) return false;
  auto ok = [&](const void* p, int64_t sb, int64_t sd, int64_t sl) {
    if (((uintptr_t)p % 16) || sb % 8) return false;
    if (sd == 1) return sl % 8 == 0;
    return sl == 1 && sd % 8 == 0 && L % 8 == 0;
  };
  return ok(dy, sgb, sgd, sgl) && ok(x, sxb, sxd, sxl);
}

void ema_param_grad_tile_launch(const void* dy, const void* x, int64_t sgb, int64_t sgd, int64_t sgl, int64_t sxb,
                                int64_t sxd, int64_t sxl, const float* q, int64_t B, int64_t D, int64_t N, int64_t L,
                                float* sums, float* dyx, hipStream_t s) {
  TileGradArgs A;
  A.dy = (const uint16_t*)dy; A.x = (const uint16_t*)x;
  A.sgb = sgb; A.sgd = sgd; A.sgl = sgl; A.sxb = sxb; A.sxd = sxd; A.sxl = sxl;
  A.q = q; A.sums = sums; A.dyx = dyx;
  A.B = (int)B; A.D = (int)D; A.N = (int)N; A.L = (int)L;
  A.x_chan_fast = sxd == 1 ? 1 : 0;
  A.g_chan_fast = sgd == 1 ? 1 : 0;
  hipLaunchKernelGGL(ema_param_grad_tile_kernel, dim3((unsigned)(B * (D / kTCh))), dim3(kTThreads), 0, s, A);
}

}  // namespace mega
