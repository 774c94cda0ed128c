// Moving-average layer on the matrix cores for [B, D, L] rows of any activation type, parallel over time:
//   y = k * x + omega x  with the carried state, per channel (fairseq/modules/base_moving_average.py:120-172;
//   the reference's fused convolution serves fp32 / fp16 / bf16 alike, ops/fftconv_kernel.cu:214-269).
// A wave owns one (batch, channel) row and one block of 1024 tokens = 16 segments of 64 tokens = the 16 MFMA
// columns; per 32-token tile  y = K x + C h_start,  h_end = Q h_start + P x  with the K / P / C operand images of
// ema_image_kernel (csrc/ema_mfma.h).  fp32 / fp16 activations run on fp16 operands: x = x_hi + x_lo as two fp16
// terms (22 significant bits; one term for fp16 input), K, P and C as two fp16 terms, the states go into the C
// product as two terms: every product is formed as hi*hi + lo*hi + hi*lo (error ~ 2^-22), accumulation and the
// recurrences are fp32.  bf16 activations run on the bf16 operands of the other kernels (K, P two terms).
// Blocks of a row are independent workgroups.  What a block inherits from the earlier ones comes through
// memory without any waiting: a first kernel (ema_rows_state_kernel) leaves every block's end state from a zero
// start, the second (ema_rows_apply_kernel) adds the earlier blocks' states up with the powers of q^1024,
// starts its segments from the right state and writes y once.  A single block needs the second kernel only.
#include "ema_mfma.h"
#include "tsn_common.h"

namespace mega {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kRW = 4;                    // waves (rows) per workgroup
constexpr int kRBlk = 1024;               // tokens per block
constexpr int kRWaveLds = 4096;           // two bf16 planes of the block, later y as fp32
constexpr int kRecF = 2 * kNS;            // floats per (row, block) record: 16 complex states

struct RowsArgs {
  const void* x;         // [B, D, L] rows: element (b, d, t) at b * sxb + d * sxd + t
  void* y;
  int64_t sxb, sxd, syb, syd;
  const uint8_t* mask;   // [B, L] or null
  const uint4* image;    // [K][kImgSlots][64]
  const float* omega;    // [D]: residual of masked tokens (they do not enter the convolution), or null
  const float* h_in;     // [B, D, N, 2] or null
  float* h_out;          // [B, D, N, 2] or null
  float* rec;            // [R][S][kRecF]: end state of every block from a zero start
  float* acc;            // [B, D, L] fp32 partial sums of the other direction (acc_mode 1: written, 2: added)
  int acc_mode;
  int koff;              // first coefficient row of this direction (0 or D)
  int reverse;           // tokens are walked from the last to the first
  int B, D, N, L, S, R;
  int is_complex;
  int both;              // both directions in this launch: forward as given, backward with rows D .. 2D - 1
  int64_t rec_dir;       // floats from the forward records to the backward ones
};

__device__ __forceinline__ uint4 img_slot(const char* base, int slot, uint32_t lane_off) {
  return *(const uint4*)(base + slot * 1024 + lane_off);
}

__device__ __forceinline__ void load_c4(const char* base, int slot, uint32_t lane_off, float (&re)[4], float (&im)[4]) {
  const uint4 a = img_slot(base, slot, lane_off), b = img_slot(base, slot + 1, lane_off);
  re[0] = __uint_as_float(a.x); im[0] = __uint_as_float(a.y);
  re[1] = __uint_as_float(a.z); im[1] = __uint_as_float(a.w);
  re[2] = __uint_as_float(b.x); im[2] = __uint_as_float(b.y);
  re[3] = __uint_as_float(b.z); im[3] = __uint_as_float(b.w);
}

// the four states (2r, 2r+1, 8+2r, 9+2r) of row block r from table `tab` of the compact slot
__device__ __forceinline__ void load_cmp(const char* base, int tab, uint32_t r_off, float (&re)[4], float (&im)[4]) {
  const uint4 a = *(const uint4*)(base + kSlotCmp * 1024 + tab * 128 + r_off);
  const uint4 b = *(const uint4*)(base + kSlotCmp * 1024 + tab * 128 + 64 + r_off);
  re[0] = __uint_as_float(a.x); im[0] = __uint_as_float(a.y);
  re[1] = __uint_as_float(a.z); im[1] = __uint_as_float(a.w);
  re[2] = __uint_as_float(b.x); im[2] = __uint_as_float(b.y);
  re[3] = __uint_as_float(b.z); im[3] = __uint_as_float(b.w);
}

// one step of the inclusive scan of h_j = R h_{j-1} + e_j across the 16 lanes of a row
template <int CTRL>
__device__ __forceinline__ void scan_step(float (&er)[4], float (&ei)[4], const float (&rr)[4], const float (&ri)[4]) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const float tr = dpp_f<CTRL>(er[u]), ti = dpp_f<CTRL>(ei[u]);
    er[u] = fmaf(tr, rr[u], fmaf(-ti, ri[u], er[u]));
    ei[u] = fmaf(ti, rr[u], fmaf(tr, ri[u], ei[u]));
  }
}

__device__ __forceinline__ void csquare(const float (&ar)[4], const float (&ai)[4], float (&br)[4], float (&bi)[4]) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    br[u] = ar[u] * ar[u] - ai[u] * ai[u];
    bi[u] = 2.f * ar[u] * ai[u];
  }
}

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;

// F16: fp16 operands (fp32 / fp16 activations), else bf16
template <bool F16>
__device__ __forceinline__ f32x4 mfma(uint4 a, uint4 b, f32x4 c) {
  if (F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// v as hi + lo in the operand type (16-bit patterns)
template <bool F16>
__device__ __forceinline__ void split16(float v, uint16_t* hi, uint16_t* lo) {
  if (F16) {
    const _Float16 h = (_Float16)v;
    *hi = __builtin_bit_cast(uint16_t, h);
    *lo = __builtin_bit_cast(uint16_t, (_Float16)(v - (float)h));
  } else {
    const __bf16 h = (__bf16)v;
    *hi = __builtin_bit_cast(uint16_t, h);
    *lo = __builtin_bit_cast(uint16_t, (__bf16)(v - (float)h));
  }
}

// byte offset of token i of the block inside a bf16 plane: segment row of 128 bytes, 16-byte chunks
// XOR-swizzled by the segment so that the B-operand reads of the 16 segments fall on different banks
__device__ __forceinline__ int plane_off(int i) {
  const int j = i >> 6, c8 = (i >> 3) & 7, e = i & 7;
  return j * 128 + ((c8 ^ (j >> 1)) << 4) + e * 2;
}

// STATE: only the block's end state is wanted (first kernel; with A.both the grid holds both directions).  NX: terms
// of x; F16: fp16 operands; VEC: rows, mask and partial sums are aligned for four tokens per access and L is a
// multiple of 4.  BOTH (second kernel, L a multiple of 1024, VEC): a wave forms both directions of its 1024 tokens
// of memory, backward first, and adds them up in LDS, so that y is written once and no partial sums pass
// through memory.
// Workgroups per CU the register budget is set for.  The apply kernel wants about 150 registers per lane: at four
// workgroups (128 registers) it spills inside the block loop, and every reload of a spilled register waits
// (vmcnt(0)) for the row loads in flight as well; at three it keeps everything in registers.
#ifndef MEGA_ROWS_MINB
#define MEGA_ROWS_MINB 3
#endif
template <typename T, int NX, bool F16, bool STATE, bool VEC, bool BOTH>
__global__ __launch_bounds__(64 * kRW, MEGA_ROWS_MINB) void ema_rows_kernel(const RowsArgs A) {
  constexpr int kWaveLds = (BOTH ? 2 : 1) * kRWaveLds;
  __shared__ __attribute__((aligned(16))) char lds[kRW * kWaveLds];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int nrg = (A.R + kRW - 1) / kRW;
  int bid = (int)blockIdx.x, dirsel = 0;
  if (STATE && A.both) {
    const int per = nrg * (A.S - 1);
    dirsel = bid >= per ? 1 : 0;
    bid -= dirsel * per;
  }
  const int sm = bid / nrg;                             // time-major: the early blocks of all rows first
  const int row = (bid - sm * nrg) * kRW + wave;
  if (row >= A.R) return;
  const int b = row / A.D, d = row - b * A.D;
  const int j = lane & 15, r = lane >> 4;
  char* plane = lds + wave * kWaveLds;                  // hi plane at 0, lo plane at 2048
  float* ys = (float*)(plane + (BOTH ? kRWaveLds : 0)); // y as fp32 (over the used-up x unless both directions meet here)
  const T* xr = (const T*)A.x + (size_t)b * A.sxb + (size_t)d * A.sxd;
  const uint32_t loff = (uint32_t)lane * 16, roff = (uint32_t)r * 16;
  constexpr int NL = 8;                                // loads in flight per lane and round (element-wise path)
  const uint8_t* mrow = A.mask ? A.mask + (size_t)b * A.L : nullptr;
  int reverse = 0, i0 = 0;
#pragma unroll 1
  for (int pass = 0; pass < (BOTH ? 2 : 1); ++pass) {
  // this pass's direction: its block in walking order, coefficient rows, records and carried states
  const bool back = BOTH ? pass == 0 : (STATE && dirsel) ? true : A.reverse != 0;
  const bool second = BOTH || (STATE && A.both);         // the launch covers both directions
  reverse = back ? 1 : 0;
  const int s = (BOTH && back) ? A.S - 1 - sm : sm;
  const int koff = second ? (back ? A.D : 0) : A.koff;
  float* rec = A.rec + ((second && back) ? A.rec_dir : 0);
  const float* h_in = (second && back) ? nullptr : A.h_in;
  float* h_out = (second && back) ? nullptr : A.h_out;
  i0 = s * kRBlk;                                       // first token of the block in walking order
  const char* img = (const char*)A.image + (size_t)(koff + d) * kImgRowBytes;

  // ---- the block of x into LDS as two 16-bit planes (masked and out-of-range tokens as zeros); every load of
  // the block is requested before the first one is used
  if (VEC) {
    // four consecutive tokens per lane and access, all requested at once
    Vec<T, 4> xq[4];
    uint32_t mq[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int w = i0 + m * 256 + 4 * lane;
      const int wc = w < A.L ? w : A.L - 4;
      const int t = reverse ? A.L - 4 - wc : wc;         // first of the four in memory
      xq[m] = *(const Vec<T, 4>*)(xr + t);
      mq[m] = mrow ? *(const uint32_t*)(mrow + t) : 0u;
    }
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int i = m * 256 + 4 * lane;
      const bool in = i0 + i < A.L;
      uint16_t hi[4], lo[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int src = reverse ? 3 - e : e;             // memory element of walking token e
        const bool masked = ((mq[m] >> (8 * src)) & 0xffu) != 0u;
        const float v = (in && !masked) ? to_float(xq[m].v[src]) : 0.f;
        split16<F16>(v, &hi[e], &lo[e]);
      }
      const int o = plane_off(i);
      *(uint2*)(plane + o) = make_uint2(hi[0] | ((uint32_t)hi[1] << 16), hi[2] | ((uint32_t)hi[3] << 16));
      if (NX > 1) *(uint2*)(plane + 2048 + o) = make_uint2(lo[0] | ((uint32_t)lo[1] << 16), lo[2] | ((uint32_t)lo[3] << 16));
    }
  } else {
#pragma unroll 1
  for (int k0 = 0; k0 < kRBlk / 64; k0 += NL) {
    float xv[NL];
    uint8_t mk[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const int w = i0 + (k0 + k) * 64 + lane;
      const int wc = w < A.L ? w : A.L - 1;
      const int t = reverse ? A.L - 1 - wc : wc;
      xv[k] = to_float(xr[t]);
      mk[k] = mrow ? mrow[t] : (uint8_t)0;
    }
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const int i = (k0 + k) * 64 + lane;
      const float v = (i0 + i < A.L && !mk[k]) ? xv[k] : 0.f;
      uint16_t hi, lo;
      split16<F16>(v, &hi, &lo);
      const int o = plane_off(i);
      *(uint16_t*)(plane + o) = hi;
      if (NX > 1) *(uint16_t*)(plane + 2048 + o) = lo;
    }
  }
  }
  // operands of the state products
  constexpr int kSP = F16 ? kSlotP16 : kSlotP, kSK = F16 ? kSlotK16 : kSlotK, kSC = F16 ? kSlotC16 : kSlotC;
  constexpr int NC = F16 ? 2 : 1;                       // terms of C and of the state operand
  uint4 P[2][2];
#pragma unroll
  for (int w = 0; w < 2; ++w)
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) P[w][mb] = img_slot(img, kSP + 2 * w + mb, loff);
  // everything else the wave will need from memory is requested here as well, so that the kernel pays one
  // round trip, not one per stage: multipliers, the earlier blocks' states, the operands of the output products
  float Qr[4], Qi[4], RSr[4], RSi[4];
  load_cmp(img, kCmpQ32, roff, Qr, Qi);
  load_cmp(img, kCmpRS, roff, RSr, RSi);
  const uint2 reach = *(const uint2*)(img + kSlotCmp * 1024 + kCmpReach * 128);
  const int nn[4] = {2 * r, 2 * r + 1, 8 + 2 * r, 9 + 2 * r};
  const int nterms = s + (h_in ? 1 : 0);
  float RWJr[4], RWJi[4], RWr[4], RWi[4], RJr[4], RJi[4], tr[4], ti[4];
  uint4 Kw[2][2], Cw[NC][2];
  if (!STATE) {
    load_c4(img, kSlotRWJ, loff, RWJr, RWJi);            // (q^1024)^j of this lane's states
    load_cmp(img, kCmpRW, roff, RWr, RWi);
    load_c4(img, kSlotRJ, loff, RJr, RJi);
    // lane (j, r): the end state of block s - 1 - j (or the caller's state behind block 0)
#pragma unroll
    for (int u = 0; u < 4; ++u) tr[u] = ti[u] = 0.f;
    if (j < s) {
      const float* e = rec + ((size_t)row * A.S + (s - 1 - j)) * kRecF;
      const float4 a = *(const float4*)(e + (2 * r) * 2), c = *(const float4*)(e + (8 + 2 * r) * 2);
      tr[0] = a.x; ti[0] = a.y; tr[1] = a.z; ti[1] = a.w;
      tr[2] = c.x; ti[2] = c.y; tr[3] = c.z; ti[3] = c.w;
    } else if (h_in && j == s) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (nn[u] < A.N) {
          const size_t o = (((size_t)b * A.D + d) * A.N + nn[u]) * 2;
          tr[u] = h_in[o];
          ti[u] = A.is_complex ? h_in[o + 1] : 0.f;
        }
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  const int steps = __builtin_amdgcn_readfirstlane((int)reach.x);
  const int look = __builtin_amdgcn_readfirstlane((int)reach.y);
  __builtin_amdgcn_wave_barrier();                      // the wave's own LDS writes precede its reads

  // ---- end states of the segments from a zero start: F after the first tile, E after the second
  const char* xrow = plane + j * 128;
  float Er[4], Ei[4], Fr[4], Fi[4];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int co = ((4 * t + r) ^ (j >> 1)) << 4;
    const uint4 Xh = *(const uint4*)(xrow + co);
    f32x4 S0 = {0.f, 0.f, 0.f, 0.f}, S1 = {0.f, 0.f, 0.f, 0.f};
    S0 = mfma<F16>(P[0][0], Xh, S0);
    S1 = mfma<F16>(P[0][1], Xh, S1);
    S0 = mfma<F16>(P[1][0], Xh, S0);
    S1 = mfma<F16>(P[1][1], Xh, S1);
    if (NX > 1) {
      const uint4 Xl = *(const uint4*)(xrow + 2048 + co);
      S0 = mfma<F16>(P[0][0], Xl, S0);
      S1 = mfma<F16>(P[0][1], Xl, S1);
    }
    const float sr[4] = {S0[0], S0[2], S1[0], S1[2]};
    const float si[4] = {S0[1], S0[3], S1[1], S1[3]};
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (t == 0) {
        Fr[u] = sr[u];
        Fi[u] = si[u];
      } else {
        Er[u] = fmaf(Qr[u], Fr[u], fmaf(-Qi[u], Fi[u], sr[u]));
        Ei[u] = fmaf(Qr[u], Fi[u], fmaf(Qi[u], Fr[u], si[u]));
      }
    }
  }
  // the operands of the output products travel under the scan and the sums below
  __builtin_amdgcn_sched_barrier(0);
  if (!STATE) {
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) Kw[w][mb] = img_slot(img, kSK + 2 * w + mb, loff);
#pragma unroll
    for (int w = 0; w < NC; ++w)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) Cw[w][mb] = img_slot(img, kSC + 2 * w + mb, loff);
  }
  __builtin_amdgcn_sched_barrier(0);
  // inclusive scan over the 16 segments by doubling; a step over d segments is skipped when |q|^(64 d) < 2^-24
  // for every state of the channel
  if (steps > 0) {
    float Rr[4], Ri[4], R2r[4], R2i[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      Rr[u] = RSr[u];
      Ri[u] = RSi[u];
    }
    scan_step<0x111>(Er, Ei, Rr, Ri);
    if (steps > 1) {
      csquare(Rr, Ri, R2r, R2i);
      scan_step<0x112>(Er, Ei, R2r, R2i);
      if (steps > 2) {
        csquare(R2r, R2i, Rr, Ri);
        scan_step<0x114>(Er, Ei, Rr, Ri);
        if (steps > 3) {
          csquare(Rr, Ri, R2r, R2i);
          scan_step<0x118>(Er, Ei, R2r, R2i);
        }
      }
    }
  }
  if (STATE) {
    // lane 15 of a row holds the block's end state from a zero start
    if (j == 15) {
      float* e = rec + ((size_t)row * A.S + s) * kRecF;
      *(float4*)(e + (2 * r) * 2) = make_float4(Er[0], Ei[0], Er[1], Ei[1]);
      *(float4*)(e + (8 + 2 * r) * 2) = make_float4(Er[2], Ei[2], Er[3], Ei[3]);
    }
    return;
  }

  // ---- what the block inherits: h_start = sum_d (q^1024)^d T_{s-1-d} (+ (q^1024)^s h_in); lane (j, r) holds
  // the term d = j for its four states, the 16 lanes of a row add up
  float Cr[4] = {0.f, 0.f, 0.f, 0.f}, Ci[4] = {0.f, 0.f, 0.f, 0.f};
  if (nterms > 0) {
    const bool have = j < nterms && j < look;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float cr = RWJr[u] * tr[u] - RWJi[u] * ti[u];
      const float ci = RWJr[u] * ti[u] + RWJi[u] * tr[u];
      Cr[u] = group_sum<16>(have ? cr : 0.f);
      Ci[u] = group_sum<16>(have ? ci : 0.f);
    }
  }
  if (h_out && s == A.S - 1 && j == 15) {
    // state after the last token: the block's own end state plus q^1024 times what it inherited
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (nn[u] < A.N) {
        const size_t o = (((size_t)b * A.D + d) * A.N + nn[u]) * 2;
        h_out[o] = fmaf(RWr[u], Cr[u], fmaf(-RWi[u], Ci[u], Er[u]));
        h_out[o + 1] = fmaf(RWr[u], Ci[u], fmaf(RWi[u], Cr[u], Ei[u]));
      }
    }
  }
  // start state of segment j: the inclusive value of segment j - 1 plus (q^64)^j times the inherited state
  float hr[4], hi[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    hr[u] = dpp_f<0x111>(Er[u]);
    hi[u] = dpp_f<0x111>(Ei[u]);
  }
  if (nterms > 0) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      hr[u] = fmaf(RJr[u], Cr[u], fmaf(-RJi[u], Ci[u], hr[u]));
      hi[u] = fmaf(RJr[u], Ci[u], fmaf(RJi[u], Cr[u], hi[u]));
    }
  }

  // ---- y = K x + C h per tile
  f32x4 Y[2][2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int co = ((4 * t + r) ^ (j >> 1)) << 4;
    const uint4 Xh = *(const uint4*)(xrow + co);
    uint16_t hh[8], hl[8];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      split16<F16>(hr[u], &hh[2 * u], &hl[2 * u]);
      split16<F16>(hi[u], &hh[2 * u + 1], &hl[2 * u + 1]);
    }
    const uint4 Hh = make_uint4(hh[0] | ((uint32_t)hh[1] << 16), hh[2] | ((uint32_t)hh[3] << 16),
                                hh[4] | ((uint32_t)hh[5] << 16), hh[6] | ((uint32_t)hh[7] << 16));
    f32x4 Y0 = {0.f, 0.f, 0.f, 0.f}, Y1 = {0.f, 0.f, 0.f, 0.f};
    Y0 = mfma<F16>(Cw[0][0], Hh, Y0);
    Y1 = mfma<F16>(Cw[0][1], Hh, Y1);
    Y0 = mfma<F16>(Kw[0][0], Xh, Y0);
    Y1 = mfma<F16>(Kw[0][1], Xh, Y1);
    Y0 = mfma<F16>(Kw[1][0], Xh, Y0);
    Y1 = mfma<F16>(Kw[1][1], Xh, Y1);
    {
      // the states as two terms in either operand type (one bf16 term leaves 2^-9 of sum |gamma q h| at the first
      // tokens of every tile, which shows where the states cancel in the sum over the states)
      const uint4 Hl = make_uint4(hl[0] | ((uint32_t)hl[1] << 16), hl[2] | ((uint32_t)hl[3] << 16),
                                  hl[4] | ((uint32_t)hl[5] << 16), hl[6] | ((uint32_t)hl[7] << 16));
      if (NC > 1) {
        Y0 = mfma<F16>(Cw[NC - 1][0], Hh, Y0);
        Y1 = mfma<F16>(Cw[NC - 1][1], Hh, Y1);
      }
      Y0 = mfma<F16>(Cw[0][0], Hl, Y0);
      Y1 = mfma<F16>(Cw[0][1], Hl, Y1);
    }
    if (NX > 1) {
      const uint4 Xl = *(const uint4*)(xrow + 2048 + co);
      Y0 = mfma<F16>(Kw[0][0], Xl, Y0);
      Y1 = mfma<F16>(Kw[0][1], Xl, Y1);
    }
    Y[t][0] = Y0;
    Y[t][1] = Y1;
    if (t == 0) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float nr = fmaf(Qr[u], hr[u], fmaf(-Qi[u], hi[u], Fr[u]));
        hi[u] = fmaf(Qr[u], hi[u], fmaf(Qi[u], hr[u], Fi[u]));
        hr[u] = nr;
      }
    }
  }
  // ---- y through LDS (fp32, in walking order; x is used up; the 16-byte pieces of a segment's 256 bytes are
  // XOR-swizzled by the segment so that the 16 segments' stores fall on different banks) and out in whole runs
  // of 64 tokens
  __builtin_amdgcn_wave_barrier();
  if (BOTH && back) {
    // in the order of memory: walking piece (j, c) is piece (15 - j, 15 - c) there, its four tokens reversed
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int jm = 15 - j, cm = 15 - (t * 8 + h * 4 + r);
        *(float4*)(ys + jm * 64 + ((cm ^ jm) & 15) * 4) = make_float4(Y[t][h][3], Y[t][h][2], Y[t][h][1], Y[t][h][0]);
      }
  } else {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        float4* at = (float4*)(ys + j * 64 + (((t * 8 + h * 4 + r) ^ j) & 15) * 4);
        float4 v = make_float4(Y[t][h][0], Y[t][h][1], Y[t][h][2], Y[t][h][3]);
        if (BOTH) {
          const float4 o = *at;
          v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
        }
        *at = v;
      }
  }
  __builtin_amdgcn_wave_barrier();
  }  // pass
  T* yr = (T*)A.y + (size_t)b * A.syb + (size_t)d * A.syd;
  float* ar = A.acc ? A.acc + ((size_t)b * A.D + d) * A.L : nullptr;
  const bool resid = A.omega && A.mask;                  // masked tokens keep their residual omega x
  const float om = resid ? A.omega[d] : 0.f;
  if (VEC) {
    float4 add[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int w = i0 + m * 256 + 4 * lane;
      const int wc = w < A.L ? w : A.L - 4;
      const int t = reverse ? A.L - 4 - wc : wc;
      add[m] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (A.acc_mode == 2) add[m] = *(const float4*)(ar + t);
      if (resid) {
        const Vec<T, 4> xo = *(const Vec<T, 4>*)(xr + t);
        const uint32_t mm = *(const uint32_t*)(mrow + t);
        add[m].x += (mm & 0xffu) ? om * to_float(xo.v[0]) : 0.f;
        add[m].y += (mm & 0xff00u) ? om * to_float(xo.v[1]) : 0.f;
        add[m].z += (mm & 0xff0000u) ? om * to_float(xo.v[2]) : 0.f;
        add[m].w += (mm & 0xff000000u) ? om * to_float(xo.v[3]) : 0.f;
      }
    }
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int i = m * 256 + 4 * lane;
      const int w = i0 + i;
      if (w < A.L) {
        const int t = reverse ? A.L - 4 - w : w;
        const float4 yv = *(const float4*)(ys + (i & ~63) + (((((i & 63) >> 2) ^ (i >> 6)) & 15) << 2));
        // memory order: the four walking tokens reversed when time runs backwards
        float4 v = reverse ? make_float4(yv.w, yv.z, yv.y, yv.x) : yv;
        v.x += add[m].x; v.y += add[m].y; v.z += add[m].z; v.w += add[m].w;
        if (A.acc_mode == 1) {
          *(float4*)(ar + t) = v;
        } else {
          Vec<T, 4> o;
          o.v[0] = from_float<T>(v.x); o.v[1] = from_float<T>(v.y); o.v[2] = from_float<T>(v.z); o.v[3] = from_float<T>(v.w);
          *(Vec<T, 4>*)(yr + t) = o;
        }
      }
    }
    return;
  }
#pragma unroll 1
  for (int k0 = 0; k0 < kRBlk / 64; k0 += NL) {
    float add[NL];
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const int w = i0 + (k0 + k) * 64 + lane;
      const int wc = w < A.L ? w : A.L - 1;
      const int t = reverse ? A.L - 1 - wc : wc;
      add[k] = 0.f;
      if (A.acc_mode == 2) add[k] = ar[t];
      if (resid) {                                       // both loads unconditional: no load waits for another
        const float xo = to_float(xr[t]);
        const uint8_t m = mrow[t];
        add[k] += m ? om * xo : 0.f;
      }
    }
#pragma unroll
    for (int k = 0; k < NL; ++k) {
      const int i = (k0 + k) * 64 + lane;
      const int w = i0 + i;
      if (w < A.L) {
        const int t = reverse ? A.L - 1 - w : w;
        const float v = ys[(i & ~63) + (((((i & 63) >> 2) ^ (i >> 6)) & 15) << 2) + (i & 3)] + add[k];
        if (A.acc_mode == 1) ar[t] = v;
        else yr[t] = from_float<T>(v);
      }
    }
  }
}

template <typename T, int NX, bool F16, bool VEC>
int launch_rows_v(const RowsArgs& A, hipStream_t s) {
  const int nrg = (A.R + kRW - 1) / kRW;
  const unsigned per_state = (unsigned)(nrg * (A.S - 1)), per_apply = (unsigned)(nrg * A.S);
  if (A.S > 1) {
    // end states of the blocks 0 .. S - 2 (nobody inherits from the last one), of both directions when asked
    hipLaunchKernelGGL((ema_rows_kernel<T, NX, F16, true, VEC, false>), dim3(per_state * (A.both ? 2 : 1)), dim3(64 * kRW),
                       0, s, A);
  }
  if (A.both) {
    if constexpr (VEC)
      hipLaunchKernelGGL((ema_rows_kernel<T, NX, F16, false, true, true>), dim3(per_apply), dim3(64 * kRW), 0, s, A);
  } else {
    hipLaunchKernelGGL((ema_rows_kernel<T, NX, F16, false, VEC, false>), dim3(per_apply), dim3(64 * kRW), 0, s, A);
  }
  MEGA_CHECK_LAUNCH("ema_fwd (rows on the matrix cores)");
  return MEGA_OK;
}

// four tokens per access when every row, the mask and the partial sums start on such a boundary
template <typename T>
bool rows_vec_ok(const RowsArgs& A) {
  const size_t al = 4 * sizeof(T);
  return A.L % 4 == 0 && A.L >= 4 && ((uintptr_t)A.x % al) == 0 && ((uintptr_t)A.y % al) == 0 &&
         A.sxb % 4 == 0 && A.sxd % 4 == 0 && A.syb % 4 == 0 && A.syd % 4 == 0 &&
         (!A.mask || ((uintptr_t)A.mask % 4) == 0) && (!A.acc || ((uintptr_t)A.acc % 16) == 0);
}

template <typename T, int NX, bool F16>
int launch_rows(const RowsArgs& A, hipStream_t s) {
  return rows_vec_ok<T>(A) ? launch_rows_v<T, NX, F16, true>(A, s) : launch_rows_v<T, NX, F16, false>(A, s);
}

}  // namespace

size_t ema_rows_record_bytes(int64_t B, int64_t D, int64_t L, int bidirectional) {
  const int64_t S = ceil_div(L, kRBlk);
  if (S <= 1 || S > 16) return 0;
  return (size_t)B * D * S * kRecF * 4 * (bidirectional ? 2 : 1);
}

// [B, D, L] rows on both sides (time contiguous), at most 16 blocks of 1024 tokens, ndim <= 16, no truncation
bool ema_rows_covers(int dtype, int64_t sxb, int64_t sxd, int64_t sxl, int64_t syb, int64_t syd, int64_t syl,
                     int64_t B, int64_t D, int64_t N, int64_t L, int64_t Lk, const float* h_out) {
  if (N > kNS || Lk > 0 || sxl != 1 || syl != 1 || L < 64) return false;
  if (ceil_div(L, kRBlk) > 16) return false;
  if (h_out && L % kRBlk != 0) return false;           // the state after the last token of a partial block
  if (B * D >= (int64_t)1 << 26) return false;          // the grids stay below 2^31 workgroups
  (void)dtype; (void)sxb; (void)sxd; (void)syb; (void)syd;
  return true;
}

int ema_rows_run(const void* x, void* y, int dtype, int64_t sxb, int64_t sxd, int64_t syb, int64_t syd,
                 const void* image, int is_complex, const float* omega, const uint8_t* mask, const float* h_in,
                 float* h_out, int64_t B, int64_t D, int64_t N, int64_t L, int bidirectional, float* acc, float* rec,
                 hipStream_t s) {
  RowsArgs A;
  A.x = x; A.y = y; A.sxb = sxb; A.sxd = sxd; A.syb = syb; A.syd = syd; A.mask = mask;
  A.image = (const uint4*)image; A.B = (int)B; A.D = (int)D; A.N = (int)N; A.L = (int)L;
  A.S = (int)ceil_div(L, kRBlk); A.R = (int)(B * D); A.is_complex = is_complex;
  A.both = 0; A.rec_dir = (int64_t)B * D * A.S * kRecF;
  auto launch = [&](const RowsArgs& a) -> int {
    switch (dtype) {
      case MEGA_F32: return launch_rows<float, 2, true>(a, s);
      case MEGA_F16: return launch_rows<f16_t, 1, true>(a, s);
      default: return launch_rows<bf16_t, 1, false>(a, s);
    }
  };
  A.koff = 0; A.reverse = 0; A.omega = mask ? omega : nullptr; A.h_in = h_in; A.h_out = h_out;
  A.acc = nullptr; A.acc_mode = 0; A.rec = rec;
  if (bidirectional) {
    const bool vec = dtype == MEGA_F32 ? rows_vec_ok<float>(A) : rows_vec_ok<bf16_t>(A);
    if (vec && L % kRBlk == 0) {
      // whole blocks: the two directions of a block of memory meet inside one wave
      A.both = 1;
      return launch(A);
    }
    // the direction back in time first, into the fp32 partial sums
    RowsArgs Bk = A;
    Bk.koff = (int)D; Bk.reverse = 1; Bk.omega = nullptr; Bk.h_in = nullptr; Bk.h_out = nullptr;
    Bk.acc = acc; Bk.acc_mode = 1;
    Bk.rec = rec + A.rec_dir;
    const int rc = launch(Bk);
    if (rc) return rc;
    A.acc = acc; A.acc_mode = 2;
  }
  return launch(A);
}

}  // namespace mega
