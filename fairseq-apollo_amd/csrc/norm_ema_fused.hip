// TimestepNorm -> moving-average layer in one kernel (gfx950, bf16 activations, 64 or 128 channels per
// norm group, ndim <= 16, optional padding mask, rows of any length up to 16 blocks): what MovingAverageGatedAttention.forward does at
// fairseq/modules/moving_average_gated_attention.py:304-315 (x = norm(x); mx = move(x^T)) with
// TimestepNorm per fairseq/csrc/ops/timestep_norm.cc:218-316 and the layer per
// fairseq/modules/base_moving_average.py:120-172.  x is read once, xn (the norm's output, which the
// layer also feeds to v_proj) and y are written once.
//
// A workgroup (16 waves) owns one (batch row, 64 channels of a norm group, block of 1024 tokens): whole 128-byte
// lines of x, xn and -- with [B, D, L] rows -- y.  A group of 128 channels is shared by two workgroups, each of
// which reads the group's whole lines for the moments.  The blocks are aligned to the end of the row: a row that is
// not a whole number of blocks starts inside block 0, behind virtual tokens that count as padding.
//   1. load the block, per-token moments of the group (packed dot products + DPP), Welford scan over
//      the block's tokens (padding weighs nothing), publish the block aggregate, fold the earlier blocks'
//      aggregates of the same (row, group) and the prior state into the carry-in, finish mean / rstd per token;
//   2. normalise from registers, store xn (zeros at padding), and stage xn (bf16, as the layer sees it) into LDS
//      transposed to channel rows;
//   3. per channel (4 per wave), with the operand images of ema_image_kernel:
//        phase A: end states of the 16 segments (64 tokens = 2 tiles each) from a zero start on the
//                 matrix cores, scanned across the 16 lanes of a DPP row; the block's end state from a
//                 zero start is parked in LDS and published;
//      look-back: the earlier blocks' end states (and the caller's carried state) folded into the
//                 block's start state, h_start = sum_d (q^1024)^d E_{s-1-d}, parked over the end states;
//        phase B: the segment scan again, segment start state = what the segment before left + (q^64)^j h_start,
//                 y_tile = K x_tile + C h (h as one bf16 term, two for slow poles and few states), bf16, back into LDS over x, and
//                 out as whole rows.
// Blocks map to workgroup ids time-major and workgroups are dispatched in id order, so a block only
// waits for blocks dispatched before it; every wait is bounded and poisons the block's outputs with
// NaN (and sets the error word of the workspace header) when it gives up.
#include <type_traits>

#include "ema_mfma.h"
#include "tsn_common.h"

// Phase markers: a profiling build defines MEGA_FTR(k) to stamp a clock per workgroup; no-ops here.
#ifndef MEGA_FTR
#define MEGA_FTR(k)
#define MEGA_FTR_END()
#endif
#ifndef MEGA_FTR2
#define MEGA_FTR2(k)
#endif

// Held-back block starts of a one-round launch: ticks of 10 ns per block index (mod 4), and the least share of the
// compute units the launch has to fill (1 / MEGA_FUSED_STAGGER_FILL) for them to be used.
#ifndef MEGA_FUSED_STAGGER
#define MEGA_FUSED_STAGGER 60
#endif
#ifndef MEGA_FUSED_STAGGER_FILL
#define MEGA_FUSED_STAGGER_FILL 4
#endif
#ifndef MEGA_FUSED_STAGGER_BLOCKS
#define MEGA_FUSED_STAGGER_BLOCKS 4
#endif
#ifndef MEGA_FUSED_TWO_TERMS
#define MEGA_FUSED_TWO_TERMS 0
#endif

namespace mega {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kFW = 16;                       // waves per workgroup
constexpr int kFT = kFW * 64;                 // threads
constexpr int kFC = 64;                       // channels per workgroup = per norm group
constexpr int kFSeg = 1024;                   // tokens per block: 16 segments x 2 tiles x 32
constexpr int kFCPW = kFC / kFW;              // channels per wave
constexpr int kFNLD = kFSeg * 8 / kFT;        // 16-byte pieces per thread
constexpr int kFRow = kFSeg * 2;              // bytes of one channel row in LDS
constexpr int kFTile = kFC * kFRow + (kFC / 4) * 16;
constexpr int kFRecW = 4 + kFC * kNS * 2;     // 64-bit words per block record: n, mean, var, pad, end states
constexpr int kFMaxBlocks = 16;               // terms of the look-back sum (earlier blocks + the carried state): one per lane of a row
constexpr int kFTabs = 2;                     // per-state multiplier tables kept in LDS: q^32, q^64
constexpr size_t kFSmem = (size_t)kFTile + 2 * kFSeg * 4 + 64 + (size_t)kFTabs * kFC * 128 + kFC * 8;

static_assert(kSEGT == 2, "the fused kernel uses the q^64 segment multipliers of the image");
static_assert(kFSmem <= 160 * 1024, "LDS of one workgroup");

struct FusedArgs {
  const bf16_t* x;       // [B, L, D]
  bf16_t* xn;            // [B, L, D]
  bf16_t* y;             // strides (syb, syd, syl): [B, D, L] rows (syl == 1) or [B, L, D] (syd == 1)
  int64_t syb, syd, syl;
  const int64_t* prev_count;
  const float* prev_mean;
  const float* prev_var;
  int64_t* count;
  float* mean;
  float* var;
  const float* gamma;    // [D] (weight + 1)
  const float* beta;     // [D]
  const uint8_t* mask;   // [B, L], nonzero = padding: no part in the statistics, xn = 0; or null
  const uint4* image;    // [D][kImgSlots][64]
  const float* h_in;     // [B, D, N, 2] or null
  float* h_out;          // [B, D, N, 2] or null
  float* cummean;        // [B, L, G] running mean / rstd of every token, kept for the norm's backward pass; or null
  float* cumrstd;
  TsnHeader* hdr;
  unsigned long long* rec;   // [B * D / 64][S + 1][kFRecW]; slot S: the caller's carried state, put there by block 0
  int B, L, D, G, N, S;
  int pad;               // S * 1024 - L virtual tokens in front of every row: the block grid ends at the row's last token
  float eps;
  int is_complex;
  int xcd_map;
  int stagger;           // start of block s held back by (s & 3) * stagger ticks of 10 ns (0: all start at once)
  LookbackLaunch lb;     // status word, poll limit, test hook
};

__device__ __forceinline__ int row_base(int c) { return c * kFRow + (c >> 2) * 16; }

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  bf16x2_t v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float lane_bcast(float v, int src_lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src_lane << 2, __builtin_bit_cast(int, v)));
}

// one step of the inclusive scan of h_j = R h_{j-1} + e_j across the 16 lanes of a row: lanes take the
// value SH lanes to the left (zero outside the row) times R^SH
template <int CTRL>
__device__ __forceinline__ void scan_step(float (&er)[4], float (&ei)[4], const float (&rr)[4], const float (&ri)[4]) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const float tr = dpp_f<CTRL>(er[u]), ti = dpp_f<CTRL>(ei[u]);
    const float nri = -ri[u];
    er[u] = fmaf(tr, rr[u], er[u]);
    er[u] = fmaf(ti, nri, er[u]);
    ei[u] = fmaf(ti, rr[u], ei[u]);
    ei[u] = fmaf(tr, ri[u], ei[u]);
  }
}

__device__ __forceinline__ void csquare(const float (&ar)[4], const float (&ai)[4], float (&br)[4], float (&bi)[4]) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    br[u] = ar[u] * ar[u] - ai[u] * ai[u];
    bi[u] = 2.f * ar[u] * ai[u];
  }
}

// activations leave once and are not read again by this kernel: streaming (non-temporal) stores
#ifndef MEGA_FUSED_NT
#define MEGA_FUSED_NT 1
#endif
__device__ __forceinline__ void store_stream(uint4* p, uint4 v) {
#if MEGA_FUSED_NT
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  __builtin_nontemporal_store(__builtin_bit_cast(u32x4, v), (u32x4*)p);
#else
  *p = v;
#endif
}

// slot `slot` of an operand image: uniform base, 32-bit lane offset (scalar-base addressing)
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

// the four states of row block r from table `tab` of the compact slot: two 16-byte pieces that the 16 lanes of
// a row share (one line per table leaves the cache, not a slot)
__device__ __forceinline__ void load_cmp(const char* base, int tab, uint32_t r_off, float (&re)[4], float (&im)[4]) {
  const uint4 a = *(const uint4*)(base + kSlotCmp * 1024 + tab * 128 + r_off);
  const uint4 b = *(const uint4*)(base + kSlotCmp * 1024 + tab * 128 + 64 + r_off);
  re[0] = __uint_as_float(a.x); im[0] = __uint_as_float(a.y);
  re[1] = __uint_as_float(a.z); im[1] = __uint_as_float(a.w);
  re[2] = __uint_as_float(b.x); im[2] = __uint_as_float(b.y);
  re[3] = __uint_as_float(b.z); im[3] = __uint_as_float(b.w);
}

// the same from the copy of tables 0..2 in LDS
__device__ __forceinline__ void lds_cmp(const char* s_tab, int tab, int c, uint32_t r_off, float (&re)[4], float (&im)[4]) {
  const float4 a = *(const float4*)(s_tab + (tab * kFC + c) * 128 + r_off);
  const float4 b = *(const float4*)(s_tab + (tab * kFC + c) * 128 + 64 + r_off);
  re[0] = a.x; im[0] = a.y; re[1] = a.z; im[1] = a.w;
  re[2] = b.x; im[2] = b.y; re[3] = b.z; im[3] = b.w;
}

// LOUT 0: y as [B, D, L] rows; 1: y as [B, L, D].  GC: channels per norm group, 64 or 128.  A group of 128 channels
// is shared by two workgroups: each reads the group's whole lines for the moments (both add in the same order, so
// both arrive at the same statistics to the last bit) and keeps its own 64 channels.
// STAG: the start of block s is held back by s * A.stagger ticks (an instance of its own: the launches that do not
// hold anything back run the code without the wait).
template <int LOUT, int GC, bool STAG>
__global__ __launch_bounds__(kFT) void norm_ema_fused_kernel(const FusedArgs A) {
  constexpr int kParts = GC / kFC;
  static_assert(kParts == 1 || kParts == 2, "one or two workgroups per norm group");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* tile = smem;
  float* s_gm = (float*)(smem + kFTile);      // [kFSeg] group mean of a token, later the running mean
  float* s_gv = s_gm + kFSeg;                 // [kFSeg] group variance, later the running rstd
  float* s_wt = s_gv + kFSeg;                 // [4][4] totals of the four scanning waves
  float* s_end = s_gm;                        // [kFC][kNS][2] block end states from a zero start (after step 2)
  char* s_tab = (char*)(s_wt + 16);           // [kFTabs][kFC][kNS] complex: q^32, q^64 of every channel
  uint2* s_reach = (uint2*)(s_tab + kFTabs * kFC * 128);   // [kFC] reach of every channel's slowest pole

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: channel rows and image addresses stay scalar
  const int G = A.G;
  const int U = G * kParts;                              // workgroups per (batch row, block)
  const int BU = A.B * U;
  const int s = (int)blockIdx.x / BU, local = (int)blockIdx.x - s * BU;
  int b, unit;
  if (A.xcd_map) {
    // consecutive workgroup ids go to the 8 XCDs in turn: keep a group's blocks (and with them the operand
    // images of its channels and the lines its two halves share) on one XCD, U / 8 units per XCD
    const int up = U >> 3, xcd = local & 7, slot = local >> 3;
    unit = xcd * up + slot % up;
    b = slot / up;
  } else {
    b = local / U;
    unit = local - b * U;
  }
  const int g = unit / kParts, part = unit - g * kParts;
  const int cb = g * GC + part * kFC;                    // the workgroup's first channel
  const uint32_t tag = A.hdr->epoch + 1u;
  // The blocks are aligned to the end of the row: block 0 starts `pad` virtual tokens before the first one (they
  // count as padding: no statistics, zeros into the moving average, nothing stored), so the last block ends at the
  // last token and the state handed back is the state after it.
  const int t0 = s * kFSeg - A.pad;
  const bool front = s == 0 && A.pad > 0;                // uniform: this block holds virtual tokens
  const int piece = tid & 7, tokl = tid >> 3;            // 16-byte piece of the 128-byte line, token 0..127
  // addresses of the block's lines: a uniform base per 128-token round plus one 32-bit lane offset
  const int64_t xblk = ((int64_t)b * A.L + t0) * A.D + (int64_t)cb;      // (negative offsets inside a front block are never used)
  const uint32_t toff = (uint32_t)tokl * (uint32_t)A.D + piece * 8;
  const size_t brow = (size_t)b * G + g;                 // statistics of the group
  const size_t rrow = brow * kParts + part;              // records of the workgroup (its own copy of the statistics too)
  unsigned long long* const myrec = A.rec + (rrow * (A.S + 1) + s) * kFRecW;
  bool poison = false;

  MEGA_FTR(0);
  // A launch of a single round has every workgroup of the chip asking for its block at the same moment, and every
  // block after a row's first then waits for the records of the blocks before it.  Blocks 1..3 of every four ask a
  // little later each (constant 100 MHz clock, a bounded wait): the requests spread out, and the later start is time
  // the block would have spent waiting for those records.
  if (STAG && s != 0) {
    const uint64_t t_end = wall_clock64() + (uint64_t)(s * A.stagger);
    while (wall_clock64() < t_end) __builtin_amdgcn_s_sleep(4);
  }
  // ---- everything the norm needs from memory is requested before the block itself
  const Moments prior = {(float)A.prev_count[b], A.prev_mean[brow], A.prev_var[brow]};
  float gam[8], bet[8];
  load_params<8>(A.gamma + cb + piece * 8, gam);
  load_params<8>(A.beta + cb + piece * 8, bet);
  uint4 xv[kFNLD];
  uint4 xo[kParts == 2 ? kFNLD : 1];
  const int64_t oblk = ((int64_t)b * A.L + t0) * A.D + (int64_t)(g * GC + (1 - part) * kFC);
  // padding flags of the thread's eight tokens (bit k: token k * 128 + tokl): the caller's mask and the virtual
  // tokens of a front block
  uint32_t mbits = 0;
  if (!front) {
#pragma unroll
    for (int k = 0; k < kFNLD; ++k) xv[k] = *(const uint4*)(A.x + xblk + (int64_t)k * 128 * A.D + toff);
    // the other half of the group's lines, for the moments only (the workgroup of that half reads the same lines on
    // the same XCD)
    if (kParts == 2) {
#pragma unroll
      for (int k = 0; k < kFNLD; ++k) xo[k] = *(const uint4*)(A.x + oblk + (int64_t)k * 128 * A.D + toff);
    }
    if (A.mask) {
      const uint8_t* mrow = A.mask + (int64_t)b * A.L + t0 + tokl;
#pragma unroll
      for (int k = 0; k < kFNLD; ++k) mbits |= (mrow[k * 128] != 0 ? 1u : 0u) << k;
    }
  } else {
#pragma unroll
    for (int k = 0; k < kFNLD; ++k) {
      const bool real = k * 128 + tokl >= A.pad;
      const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
      xv[k] = real ? *(const uint4*)(A.x + xblk + (int64_t)k * 128 * A.D + toff) : zero;
      if (kParts == 2) xo[k] = real ? *(const uint4*)(A.x + oblk + (int64_t)k * 128 * A.D + toff) : zero;
      const bool padded = !real || (A.mask && A.mask[(int64_t)b * A.L + t0 + k * 128 + tokl] != 0);
      mbits |= (padded ? 1u : 0u) << k;
    }
  }

  // the per-state multipliers of the group's 64 channels (three lines per channel) go to LDS once
  {
    static_assert(kCmpQ32 == 0 && kCmpRS == 1 && kFTabs == 2, "tables 0..1 of the compact slot are staged");
    const char* ibase = (const char*)A.image + (size_t)cb * kImgRowBytes + kSlotCmp * 1024;
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int idx = it * kFT + tid;               // (table, channel, 16-byte piece)
      if (idx < kFTabs * kFC * 8) {
        const int t = idx / (kFC * 8), rem = idx - t * (kFC * 8), c = rem >> 3, pc = rem & 7;
        *(uint4*)(s_tab + (t * kFC + c) * 128 + pc * 16) =
            *(const uint4*)(ibase + (size_t)c * kImgRowBytes + t * 128 + pc * 16);
      }
    }
    // and how far every channel's slowest pole reaches (asked for here, used after the norm: no wave waits for it)
    if (tid < kFC) s_reach[tid] = *(const uint2*)(ibase + (size_t)tid * kImgRowBytes + kCmpReach * 128);
  }

  // ---- the caller's carried state joins the records the later look-ups read: slot S of the row, written by block 0
  if (s == 0 && A.h_in) {
    const int c = tid >> 4, n = tid & 15;
    float2 v = make_float2(0.f, 0.f);
    if (n < A.N) {
      v = *(const float2*)(A.h_in + (((size_t)b * A.D + cb + c) * A.N + n) * 2);
      if (!A.is_complex) v.y = 0.f;
    }
    unsigned long long* e = A.rec + (rrow * (A.S + 1) + A.S) * kFRecW + 4 + ((size_t)c * kNS + n) * 2;
    put_rec(e, tagged(__float_as_uint(v.x), tag));
    put_rec(e + 1, tagged(__float_as_uint(v.y), tag));
  }

  // ---- moments of every token's group (64 channels = the 8 lanes of a line)
#pragma unroll
  for (int k = 0; k < kFNLD; ++k) {
    const uint32_t w[4] = {xv[k].x, xv[k].y, xv[k].z, xv[k].w};
    float sm = 0.f, sq = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sm = dot2_ones<bf16_t>(w[i], sm);
      sq = dot2_self<bf16_t>(w[i], sq);
    }
    if (kParts == 2) {
      const uint32_t wo[4] = {xo[k].x, xo[k].y, xo[k].z, xo[k].w};
      float so = 0.f, qo = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        so = dot2_ones<bf16_t>(wo[i], so);
        qo = dot2_self<bf16_t>(wo[i], qo);
      }
      // lower half first in both workgroups
      sm = part == 0 ? sm + so : so + sm;
      sq = part == 0 ? sq + qo : qo + sq;
    }
    const float m = group_sum<8>(sm) * (1.0f / GC);
    const float v = fmaxf(group_sum<8>(sq) * (1.0f / GC) - m * m, 0.f);
    if (piece == 0) {
      s_gm[k * 128 + tokl] = m;
      s_gv[k * 128 + tokl] = ((mbits >> k) & 1u) ? -1.f : v;        // a negative variance marks padding
    }
  }
  __syncthreads();
  MEGA_FTR(1);

  // ---- running statistics: waves 0..3 scan 256 tokens each (4 per lane), the wave totals meet in LDS
  Moments pref[4], lane_exc = {0.f, 0.f, 0.f};
  if (wave < 4) {
    const float4 m4 = *(const float4*)(s_gm + wave * 256 + lane * 4);
    const float4 v4 = *(const float4*)(s_gv + wave * 256 + lane * 4);
    const float mm[4] = {m4.x, m4.y, m4.z, m4.w}, vv[4] = {v4.x, v4.y, v4.z, v4.w};
    // padding counts for nothing: weight 0 (the merges keep the other side's statistics)
    Moments st = {vv[0] >= 0.f ? 1.f : 0.f, mm[0], fmaxf(vv[0], 0.f)};
    pref[0] = st;
#pragma unroll
    for (int u = 1; u < 4; ++u) {
      st = merge(st, Moments{vv[u] >= 0.f ? 1.f : 0.f, mm[u], fmaxf(vv[u], 0.f)});
      pref[u] = st;
    }
    const Moments inc = row_scan(st);
    const Moments exc = dpp_m<0x111>(inc);
    Moments acc = {0.f, 0.f, 0.f}, rp = {0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const Moments t = {__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, inc.n), 16 * r + 15)),
                         __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, inc.mean), 16 * r + 15)),
                         __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, inc.var), 16 * r + 15))};
      if ((lane >> 4) == r) rp = acc;
      acc = merge(acc, t);
    }
    lane_exc = merge(rp, exc);
    if (lane == 0) {
      s_wt[wave * 4] = acc.n;
      s_wt[wave * 4 + 1] = acc.mean;
      s_wt[wave * 4 + 2] = acc.var;
    }
  }
  __syncthreads();
  if (wave < 4) {
    Moments wpre = {0.f, 0.f, 0.f}, tot = {0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if (w == wave) wpre = tot;
      tot = merge(tot, Moments{s_wt[w * 4], s_wt[w * 4 + 1], s_wt[w * 4 + 2]});
    }
    if (wave == 0 && lane == 0 && !(A.lb.withhold_first && s == 0)) {
      put_rec(myrec, tagged((uint32_t)tot.n, tag));
      put_rec(myrec + 1, tagged(__float_as_uint(tot.mean), tag));
      put_rec(myrec + 2, tagged(__float_as_uint(tot.var), tag));
    }
    MEGA_FTR(2);
    // earlier blocks of this (row, group): lane i fetches block i's aggregate
    Moments accp = {0.f, 0.f, 0.f};
    if (s > 0) {
      const unsigned long long* rp = A.rec + (rrow * (A.S + 1) + (lane < s ? lane : s - 1)) * kFRecW;
      unsigned long long w0, w1, w2;
      uint32_t spins = 0;
      for (;;) {
        w0 = get_rec(rp);
        w1 = get_rec(rp + 1);
        w2 = get_rec(rp + 2);
        const bool ok = (uint32_t)(w0 >> 32) == tag && (uint32_t)(w1 >> 32) == tag && (uint32_t)(w2 >> 32) == tag;
        if (__all(ok)) break;
        if (++spins > A.lb.spin_limit) {
          poison = true;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
      for (int i = 0; i < s; ++i) {
        const Moments t = {(float)(uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)w0, i),
                           __builtin_bit_cast(float, __builtin_amdgcn_readlane((int)(uint32_t)w1, i)),
                           __builtin_bit_cast(float, __builtin_amdgcn_readlane((int)(uint32_t)w2, i))};
        accp = merge(accp, t);
      }
    }
    MEGA_FTR(3);
    Moments carry = merge(prior, accp);
    if (poison) {
      carry.mean = __builtin_nanf("");
      if (lane == 0) report_give_up(A.hdr, A.lb.status);
    }
    const Moments base = merge(carry, merge(wpre, lane_exc));
    Moments full = base;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      full = merge(base, pref[u]);
      const float rstd = __builtin_amdgcn_rsqf(full.var + A.eps);
      s_gm[wave * 256 + lane * 4 + u] = full.mean;
      s_gv[wave * 256 + lane * 4 + u] = rstd;
      // training: the statistics the norm's backward pass reads (a padded token holds the carried ones)
      if (A.cummean && part == 0) {
        const int64_t tok = (int64_t)t0 + wave * 256 + lane * 4 + u;
        if (tok >= 0) {
          const int64_t o = ((int64_t)b * A.L + tok) * A.G + g;
          A.cummean[o] = full.mean;
          A.cumrstd[o] = rstd;
        }
      }
    }
    if (s == A.S - 1 && wave == 3 && lane == 63 && part == 0) {
      A.mean[brow] = full.mean;
      A.var[brow] = full.var;
      // tokens that count: whole numbers below 2^24, exact in the float sums
      if (g == 0) A.count[b] = poison ? (int64_t)-1 : A.prev_count[b] + (int64_t)(accp.n + tot.n);
    }
  }
  __syncthreads();

  // operand loaders of the moving-average phases (one register set: a channel's operands are requested as soon
  // as the previous channel's have been used, and travel under the rest of that channel's work)
  const uint32_t loff0 = (uint32_t)lane * 16;
  const uint32_t koff0 = (uint32_t)(((lane & 15) - 8 * (lane >> 4) + 24) * 16);
  auto load_p = [&](const int c, bf16x8 (&P)[kNWP][2]) {
    const char* img = (const char*)A.image + (size_t)(cb + c) * kImgRowBytes;
    uint32_t loff = loff0;
    asm volatile("" : "+v"(loff));
#pragma unroll
    for (int w = 0; w < kNWP; ++w)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) P[w][mb] = __builtin_bit_cast(bf16x8, img_slot(img, kSlotP + 2 * w + mb, loff));
  };
  auto load_kc = [&](const int c, bf16x8 (&K)[kNWK][2], bf16x8 (&C)[kNWC][2]) {
    const char* img = (const char*)A.image + (size_t)(cb + c) * kImgRowBytes;
    uint32_t loff = loff0;
    asm volatile("" : "+v"(loff));
    // K from the slot that holds each distinct vector once: 7 lines per term leave the cache instead of 16
    uint32_t koff = koff0;
    asm volatile("" : "+v"(koff));
#pragma unroll
    for (int w = 0; w < kNWK; ++w)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
        K[w][mb] = __builtin_bit_cast(bf16x8, *(const uint4*)(img + ((kSlotKT + w) * 1024 + mb * 256) + koff));
#pragma unroll
    for (int w = 0; w < kNWC; ++w)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) C[w][mb] = __builtin_bit_cast(bf16x8, img_slot(img, kSlotC + 2 * w + mb, loff));
  };
  // the P operand of the wave's first channel travels under the normalisation
  bf16x8 Pa[kNWP][2];
  load_p(wave, Pa);

  // ---- normalise from registers and stage xn (bf16, as the layer sees it) transposed: channel rows of 16
  // segments x 128 bytes, 16-byte chunk c of segment j at chunk c ^ (j >> 1) (the 16 lanes of a matrix-core
  // operand load then cover all banks); the lanes of tokens (2m, 2m+1) swap halves so that each writes dwords
  // (even token | odd token << 16) of four channels
  {
    const int odd = tokl & 1;
    const uint32_t sel_lo = odd ? 0x01000504u : 0x05040100u;
    const uint32_t sel_hi = odd ? 0x03020706u : 0x07060302u;
    const int tl = tokl & ~1;
    char* wbase = tile + row_base(piece * 8 + odd * 4) + (tl >> 6) * 128 + ((tl & 7) >> 1) * 4;
    const int c8 = (tl & 63) >> 3;
    // weight + 1 = 1 and bias = 0 for every channel of the group (the module's initial values): the affine step
    // is skipped, one multiply-add per element less (a wave sees all 64 channels, so the branch is uniform)
    bool plain = true;
#pragma unroll
    for (int i = 0; i < 8; ++i) plain = plain && gam[i] == 1.f && bet[i] == 0.f;
    const bool ident = __all(plain);
    auto stage = [&](auto IDENT, auto MASKED, auto FRONT) {
#pragma unroll
    for (int k = 0; k < kFNLD; ++k) {
      const int tok = k * 128 + tokl;
      const float m = s_gm[tok], r = s_gv[tok];
      const float mr = m * r;
      const uint32_t w[4] = {xv[k].x, xv[k].y, xv[k].z, xv[k].w};
      uint32_t o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float lo = fmaf(__uint_as_float(w[i] << 16), r, -mr);
        const float hi = fmaf(__uint_as_float(w[i] & 0xffff0000u), r, -mr);
        o[i] = decltype(IDENT)::value ? pack_bf16(lo, hi)
                                      : pack_bf16(fmaf(lo, gam[2 * i], bet[2 * i]), fmaf(hi, gam[2 * i + 1], bet[2 * i + 1]));
      }
      if (decltype(MASKED)::value) {
        const bool pad = (mbits >> k) & 1u;                 // padding leaves as zeros, whatever x holds there
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = pad ? 0u : o[i];
      }
      if (!decltype(FRONT)::value || k * 128 + tokl >= A.pad)              // virtual tokens have no place in xn
        store_stream((uint4*)(A.xn + xblk + (int64_t)k * 128 * A.D + toff), make_uint4(o[0], o[1], o[2], o[3]));
      const uint32_t s0 = odd ? o[0] : o[2], s1 = odd ? o[1] : o[3];
      const uint32_t r0 = dpp_u<0x128>(s0), r1 = dpp_u<0x128>(s1);       // row_ror:8 = the partner token's lane
      const uint32_t m0 = odd ? o[2] : o[0], m1 = odd ? o[3] : o[1];
      char* wp = wbase + (2 * k) * 128 + ((c8 ^ k) << 4);
      *(uint32_t*)(wp) = __builtin_amdgcn_perm(r0, m0, sel_lo);
      *(uint32_t*)(wp + kFRow) = __builtin_amdgcn_perm(r0, m0, sel_hi);
      *(uint32_t*)(wp + 2 * kFRow) = __builtin_amdgcn_perm(r1, m1, sel_lo);
      *(uint32_t*)(wp + 3 * kFRow) = __builtin_amdgcn_perm(r1, m1, sel_hi);
    }
    };
    if (front) {
      if (ident) {
        stage(std::true_type{}, std::true_type{}, std::true_type{});
      } else {
        stage(std::false_type{}, std::true_type{}, std::true_type{});
      }
    } else if (A.mask) {
      if (ident) {
        stage(std::true_type{}, std::true_type{}, std::false_type{});
      } else {
        stage(std::false_type{}, std::true_type{}, std::false_type{});
      }
    } else if (ident) {
      stage(std::true_type{}, std::false_type{}, std::false_type{});
    } else {
      stage(std::false_type{}, std::false_type{}, std::false_type{});
    }
  }
  __syncthreads();

  MEGA_FTR(4);
  // ---- moving average.  MFMA lane layout: column j = lane & 15 is segment j, r = lane >> 4 holds the
  // states (2r, 2r+1, 8+2r, 9+2r) of the 32-row state products.
  const int j = lane & 15, r = lane >> 4;
  const int nn[4] = {2 * r, 2 * r + 1, 8 + 2 * r, 9 + 2 * r};
  const bool last_block = s == A.S - 1;
  const int nterms = s + (A.h_in ? 1 : 0);
  const uint32_t roff0 = (uint32_t)r * 16;
  // how far the channels' slowest poles reach (figures of the operand image, uniform per wave and channel)
  int nsteps[kFCPW], nlook[kFCPW];
#pragma unroll
  for (int i = 0; i < kFCPW; ++i) {
    const uint2 rw = s_reach[wave + kFW * i];
    nsteps[i] = __builtin_amdgcn_readfirstlane((int)rw.x);
    nlook[i] = __builtin_amdgcn_readfirstlane((int)rw.y);
  }

  // the wave's own row leaves as whole lines ([B, D, L] rows)
  auto store_row = [&](const int c) {
    // LDS operations of one wave are performed in order: the lanes' writes above are visible to the
    // reads below without waiting for anything else (a release fence would also wait for the wave's
    // outstanding global stores)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    const char* rb = tile + row_base(c);
    bf16_t* yr = A.y + (int64_t)b * A.syb + (int64_t)(cb + c) * A.syd + t0;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int q = k * 64 + lane;                 // 16-byte chunk of the row: segment q >> 3, chunk q & 7
      const uint4 v = *(const uint4*)(rb + (q >> 3) * 128 + (((q & 7) ^ (q >> 4)) << 4));
      if (q * 8 >= -t0) store_stream((uint4*)(yr + q * 8), v);      // (a front block: the row begins inside it, at a multiple of 8)
    }
  };

  // End states of channel c's 16 segments from a zero start (P products; F = the state after a segment's first
  // tile), scanned across the row by doubling: E becomes the state after segment j with the block started from
  // zero.  A step over d segments is skipped (uniform branch) when |q|^(64 d) < 2^-24 for every state of the
  // channel: what it would add is below fp32 resolution.
  auto segment_scan = [&](const int c, const int steps, const bf16x8 (&P)[kNWP][2], const bf16x8& X0, const bf16x8& X1,
                          const float (&Qr)[4], const float (&Qi)[4], float (&Er)[4], float (&Ei)[4], float (&Fr)[4],
                          float (&Fi)[4], const uint32_t roff) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      f32x4 S0 = {0.f, 0.f, 0.f, 0.f}, S1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < kNWP; ++w) {
        S0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(P[w][0], t == 0 ? X0 : X1, S0, 0, 0, 0);
        S1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(P[w][1], t == 0 ? X0 : X1, S1, 0, 0, 0);
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
    if (steps > 0) {
      float Rr[4], Ri[4], R2r[4], R2i[4];
      lds_cmp(s_tab, kCmpRS, c, roff, Rr, Ri);
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
  };

  // ---- phase A, what the later blocks wait for: the block's end state from a zero start (lane 15 of every row
  // after the scan), parked in LDS and published
  MEGA_FTR(5);
  // it goes before the other waves' phase B
  __builtin_amdgcn_s_setprio(2);
#pragma unroll
  for (int i = 0; i < kFCPW; ++i) {
    const int c = wave + kFW * i;
    uint32_t roff = roff0;
    asm volatile("" : "+v"(roff));
    float Qr[4], Qi[4];
    lds_cmp(s_tab, kCmpQ32, c, roff, Qr, Qi);
    const char* row = tile + row_base(c) + j * 128;
    const bf16x8 X0 = *(const bf16x8*)(row + (((r) ^ (j >> 1)) << 4));
    const bf16x8 X1 = *(const bf16x8*)(row + (((4 + r) ^ (j >> 1)) << 4));
    float Er[4], Ei[4], Fr[4], Fi[4];
    segment_scan(c, nsteps[i], Pa, X0, X1, Qr, Qi, Er, Ei, Fr, Fi, roff);
    if (j == 15) {
      *(float4*)(s_end + (c * kNS + 2 * r) * 2) = make_float4(Er[0], Ei[0], Er[1], Ei[1]);
      *(float4*)(s_end + (c * kNS + 8 + 2 * r) * 2) = make_float4(Er[2], Ei[2], Er[3], Ei[3]);
    }
    // the next channel's P operand (after the last channel: the first one's again, for phase B)
    __builtin_amdgcn_sched_barrier(0);
    load_p(i + 1 < kFCPW ? wave + kFW * (i + 1) : wave, Pa);
    __builtin_amdgcn_sched_barrier(0);
    MEGA_FTR(6 + i);
  }
  if (!last_block && !(A.lb.withhold_first && s == 0)) {
    // the wave's four channels x 16 states x (re, im) = 128 words: two per lane
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    const int cp = wave + kFW * (lane >> 4);
    const float2 v = *(const float2*)(s_end + (cp * kNS + (lane & 15)) * 2);
    unsigned long long* e = myrec + 4 + ((size_t)cp * kNS + (lane & 15)) * 2;
    put_rec(e, tagged(__float_as_uint(v.x), tag));
    put_rec(e + 1, tagged(__float_as_uint(v.y), tag));
  }
  __builtin_amdgcn_s_setprio(0);

  // the operands of phase B's first channel travel under the wait for the earlier blocks
  bf16x8 Ka[kNWK][2], Ca[kNWC][2];
  load_kc(wave, Ka, Ca);
  float Jr[4] = {0.f, 0.f, 0.f, 0.f}, Ji[4] = {0.f, 0.f, 0.f, 0.f};
  auto load_j = [&](const int c) {
    const char* img = (const char*)A.image + (size_t)(cb + c) * kImgRowBytes;
    uint32_t loff = loff0;
    asm volatile("" : "+v"(loff));
    load_c4(img, kSlotRJ, loff, Jr, Ji);             // (q^64)^j
  };
  load_j(wave);

  // ---- start state of the block: h_start = sum_{d >= 0} (q^1024)^d E_{s-1-d}, E_{-1} being the caller's carried
  // state (slot S of the row's records).  Lane (j, r) works for channel wave + 16 (j >> 2) and takes the terms
  // d = (j & 3) + 4 k; the four lanes of a quad add up.
  float Cr[4] = {0.f, 0.f, 0.f, 0.f}, Ci[4] = {0.f, 0.f, 0.f, 0.f};
  if (nterms > 0) {
    const int cl = wave + kFW * (j >> 2);
    const int chl = cb + cl;
    int look = 0;                                  // blocks back that still reach this lane's channel
#pragma unroll
    for (int i = 0; i < kFCPW; ++i) look = (j >> 2) == i ? nlook[i] : look;
    const char* wimg = (const char*)A.image + (size_t)chl * kImgRowBytes;
    int maxlook = 0;
#pragma unroll
    for (int i = 0; i < kFCPW; ++i) maxlook = nlook[i] > maxlook ? nlook[i] : maxlook;
    const int nrounds = nterms < maxlook ? nterms : maxlook;
    for (int d0 = 0; d0 < nrounds; d0 += 4) {
      const int d = d0 + (j & 3);
      const bool have = d < nterms && d < look;
      const int slot = have ? (d < s ? s - 1 - d : A.S) : 0;
      const unsigned long long* e = A.rec + (rrow * (A.S + 1) + slot) * kFRecW + 4 + (size_t)cl * kNS * 2 + 4 * r;
      float Wr[4], Wi[4];
      load_c4(wimg, kSlotRWJ, (uint32_t)(((r << 4) | (have ? d : 0)) * 16), Wr, Wi);      // (q^1024)^d
      unsigned long long w[8];
      uint32_t spins = 0;
      for (;;) {
        bool ok = true;
#pragma unroll
        for (int u = 0; u < 4; ++u) {              // states (2r, 2r+1) and (8+2r, 9+2r): two runs of four words
          w[u] = have ? get_rec(e + u) : tagged(0u, tag);
          w[4 + u] = have ? get_rec(e + 16 + u) : tagged(0u, tag);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) ok &= (uint32_t)(w[u] >> 32) == tag;
        if (__all(ok)) break;
        if (++spins > A.lb.spin_limit) {
          poison = true;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float er = __uint_as_float((uint32_t)w[2 * u]), ei = __uint_as_float((uint32_t)w[2 * u + 1]);
        Cr[u] = fmaf(Wr[u], er, fmaf(-Wi[u], ei, Cr[u]));
        Ci[u] = fmaf(Wr[u], ei, fmaf(Wi[u], er, Ci[u]));
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      Cr[u] = group_sum<4>(Cr[u]);
      Ci[u] = group_sum<4>(Ci[u]);
    }
    if (poison) {
      Cr[0] = __builtin_nanf("");
      if (lane == 0) report_give_up(A.hdr, A.lb.status);
    }
  }
  // h_start (zero when nothing comes in) is parked over the wave's own end states, which have left; the last block
  // first returns the state after its last token: end state from a zero start + (q^1024) h_start
  asm volatile("" ::: "memory");
  __builtin_amdgcn_wave_barrier();
  if (last_block && A.h_out && (j & 3) == 0) {
    const int cl = wave + kFW * (j >> 2);
    const int ch = cb + cl;
    float Rr[4], Ri[4];
    load_cmp((const char*)A.image + (size_t)ch * kImgRowBytes, kCmpRW, roff0, Rr, Ri);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (nn[u] < A.N) {
        const float er = s_end[(cl * kNS + nn[u]) * 2], ei = s_end[(cl * kNS + nn[u]) * 2 + 1];
        const size_t o = (((size_t)b * A.D + ch) * A.N + nn[u]) * 2;
        A.h_out[o] = fmaf(Rr[u], Cr[u], fmaf(-Ri[u], Ci[u], er));
        A.h_out[o + 1] = fmaf(Rr[u], Ci[u], fmaf(Ri[u], Cr[u], ei));
      }
    }
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_wave_barrier();
  if ((j & 3) == 0) {
    const int cl = wave + kFW * (j >> 2);
    *(float4*)(s_end + (cl * kNS + 2 * r) * 2) = make_float4(Cr[0], Ci[0], Cr[1], Ci[1]);
    *(float4*)(s_end + (cl * kNS + 8 + 2 * r) * 2) = make_float4(Cr[2], Ci[2], Cr[3], Ci[3]);
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_wave_barrier();
  MEGA_FTR(10);

  // ---- phase B per channel: the segment scan again (cheaper than keeping four channels' scans in registers across
  // the wait), start state of segment j = what segment j - 1 left + (q^64)^j h_start, then
  // y_tile = K x_tile + C h (h: the state at the tile's first token, carried into the product as two bf16 terms where
  // one would show; at a segment's second tile h = q^32 h + F), bf16,
  // back into LDS over x, and out as whole rows.
#pragma unroll
  for (int i = 0; i < kFCPW; ++i) {
    const int c = wave + kFW * i;
    // One bf16 term for the states leaves an error of 2^-9 of sum |gamma q h| at the first tokens of every tile.  It
    // shows where the states dwarf y (slow poles: |q|^128 >= 2^-24 for some state of the channel), in layers of few
    // states, whose rounding errors do not average out in the sum over the states, and in real-valued layers, whose
    // input weights alternate in sign along the states so that the states cancel by construction: those take a
    // second term (hi + lo).  MEGA_FUSED_TWO_TERMS=1 gives every channel the second term (+ 0.7 us at the headline
    // shape).
    const bool two_terms = MEGA_FUSED_TWO_TERMS || nsteps[i] >= 2 || A.N <= 8 || !A.is_complex;
    uint32_t roff = roff0;
    asm volatile("" : "+v"(roff));
    char* row = tile + row_base(c) + j * 128;
    const bf16x8 X0 = *(const bf16x8*)(row + (((r) ^ (j >> 1)) << 4));
    const bf16x8 X1 = *(const bf16x8*)(row + (((4 + r) ^ (j >> 1)) << 4));
    float hr[4], hi[4], Fr[4], Fi[4];
    {
      float Qr[4], Qi[4];
      lds_cmp(s_tab, kCmpQ32, c, roff, Qr, Qi);
      segment_scan(c, nsteps[i], Pa, X0, X1, Qr, Qi, hr, hi, Fr, Fi, roff);
    }
    MEGA_FTR2(0);
    __builtin_amdgcn_sched_barrier(0);
    if (i + 1 < kFCPW) load_p(wave + kFW * (i + 1), Pa);
    __builtin_amdgcn_sched_barrier(0);
    {
      const float4 b0 = *(const float4*)(s_end + (c * kNS + 2 * r) * 2);
      const float4 b1 = *(const float4*)(s_end + (c * kNS + 8 + 2 * r) * 2);
      const float br[4] = {b0.x, b0.z, b1.x, b1.z}, bi[4] = {b0.y, b0.w, b1.y, b1.w};
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float sr = dpp_f<0x111>(hr[u]), si = dpp_f<0x111>(hi[u]);
        hr[u] = fmaf(Jr[u], br[u], fmaf(-Ji[u], bi[u], sr));
        hi[u] = fmaf(Jr[u], bi[u], fmaf(Ji[u], br[u], si));
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (i + 1 < kFCPW) load_j(wave + kFW * (i + 1));
    __builtin_amdgcn_sched_barrier(0);
    MEGA_FTR2(1);
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      asm volatile("" ::: "memory");              // x again from LDS: cheaper than eight registers across the scan
      const bf16x8 X = *(const bf16x8*)(row + (((4 * t + r) ^ (j >> 1)) << 4));
      f32x4 Y0 = {0.f, 0.f, 0.f, 0.f}, Y1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < kNWK; ++w) {
        Y0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Ka[w][0], X, Y0, 0, 0, 0);
        Y1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Ka[w][1], X, Y1, 0, 0, 0);
      }
      bf16x8 Hop;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        Hop[2 * u] = (__bf16)hr[u];
        Hop[2 * u + 1] = (__bf16)hi[u];
      }
#pragma unroll
      for (int w = 0; w < kNWC; ++w) {
        Y0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Ca[w][0], Hop, Y0, 0, 0, 0);
        Y1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Ca[w][1], Hop, Y1, 0, 0, 0);
      }
      if (two_terms) {
        bf16x8 Hlo;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          Hlo[2 * u] = (__bf16)(hr[u] - (float)Hop[2 * u]);
          Hlo[2 * u + 1] = (__bf16)(hi[u] - (float)Hop[2 * u + 1]);
        }
#pragma unroll
        for (int w = 0; w < kNWC; ++w) {
          Y0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Ca[w][0], Hlo, Y0, 0, 0, 0);
          Y1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Ca[w][1], Hlo, Y1, 0, 0, 0);
        }
      }
      if (t == 0) {
        float Qr[4], Qi[4];
        lds_cmp(s_tab, kCmpQ32, c, roff, Qr, Qi);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float nr = fmaf(Qr[u], hr[u], fmaf(-Qi[u], hi[u], Fr[u]));
          hi[u] = fmaf(Qr[u], hi[u], fmaf(Qi[u], hr[u], Fi[u]));
          hr[u] = nr;
        }
      }
      // y (bf16) over x: tokens 32 t + 4 r + {0..3} and 32 t + 16 + 4 r + {0..3} of segment j
      *(uint2*)(row + (((4 * t + (r >> 1)) ^ (j >> 1)) << 4) + (r & 1) * 8) =
          make_uint2(pack_bf16(Y0[0], Y0[1]), pack_bf16(Y0[2], Y0[3]));
      *(uint2*)(row + (((4 * t + 2 + (r >> 1)) ^ (j >> 1)) << 4) + (r & 1) * 8) =
          make_uint2(pack_bf16(Y1[0], Y1[1]), pack_bf16(Y1[2], Y1[3]));
      MEGA_FTR2(2 + t);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (i + 1 < kFCPW) load_kc(wave + kFW * (i + 1), Ka, Ca);
    __builtin_amdgcn_sched_barrier(0);
    MEGA_FTR2(4);
    if (LOUT == 0) store_row(c);
    __builtin_amdgcn_sched_barrier(0);
    MEGA_FTR(11 + i);
  }
  if (LOUT == 1) {
    // [B, L, D]: the inverse of the staging step, whole lines of 64 channels per token
    __syncthreads();
    const int odd = tokl & 1;
    const uint32_t sel_keep = odd ? 0x07060302u : 0x05040100u;
    const uint32_t sel_give = odd ? 0x05040100u : 0x07060302u;
    const int tl = tokl & ~1;
    const char* rbase = tile + row_base(piece * 8 + odd * 4) + (tl >> 6) * 128 + ((tl & 7) >> 1) * 4;
    const int c8 = (tl & 63) >> 3;
    bf16_t* yb = A.y + (int64_t)b * A.syb + (int64_t)(cb + piece * 8) * A.syd;
#pragma unroll
    for (int k = 0; k < kFNLD; ++k) {
      const int tok = k * 128 + tokl;
      const char* rp = rbase + (2 * k) * 128 + ((c8 ^ k) << 4);
      uint32_t w[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = *(const uint32_t*)(rp + e * kFRow);
      const uint32_t keep0 = __builtin_amdgcn_perm(w[1], w[0], sel_keep);
      const uint32_t keep1 = __builtin_amdgcn_perm(w[3], w[2], sel_keep);
      const uint32_t got0 = dpp_u<0x128>(__builtin_amdgcn_perm(w[1], w[0], sel_give));
      const uint32_t got1 = dpp_u<0x128>(__builtin_amdgcn_perm(w[3], w[2], sel_give));
      uint4 o;
      o.x = odd ? got0 : keep0;
      o.y = odd ? got1 : keep1;
      o.z = odd ? keep0 : got0;
      o.w = odd ? keep1 : got1;
      if (t0 + tok >= 0) store_stream((uint4*)(yb + (int64_t)(t0 + tok) * A.syl), o);
    }
  }

  MEGA_FTR_END();
  // ---- retire: the last workgroup to finish opens the next epoch
  if (tid == 0) {
    const uint32_t total = gridDim.x;
    const uint32_t k = blockIdx.x & 31u;
    const uint32_t quota = (total - k + 31u) / 32u;
    if (atomicAdd(&A.hdr->done1[k], 1u) == quota - 1u) {
      publish_u32(&A.hdr->done1[k], 0u);
      const uint32_t classes = total < 32u ? total : 32u;
      if (atomicAdd(&A.hdr->done2, 1u) == classes - 1u) {
        publish_u32(&A.hdr->done2, 0u);
        publish_u32(&A.hdr->epoch, tag == 0xffffffffu ? 0u : tag);
      }
    }
  }
}

// R: record rows = workgroups per block = B * D / 64
size_t fused_ws_bytes(int64_t R, int64_t S) {
  return align_up(sizeof(TsnHeader), 256) + align_up((size_t)R * (S + 1) * kFRecW * 8, 256);
}

bool fused_covers(int dtype, int64_t B, int64_t L, int64_t D, int64_t G, int64_t N, const void* x, const void* xn,
                  const void* y, int64_t syb, int64_t syd, int64_t syl, const uint8_t* mask, const float* h_in) {
  (void)mask;
  if (dtype != MEGA_BF16 || G <= 0 || (D != G * kFC && D != G * 2 * kFC) || N > kNS || N <= 0) return false;
  if (L <= 0 || ceil_div(L, kFSeg) + (h_in ? 1 : 0) > kFMaxBlocks) return false;
  // a ragged first block (the block grid is aligned to the end of the row): no carried state in (it would have to
  // enter in the middle of a block), and rows in time must begin at a multiple of 8 inside it
  if (L % kFSeg != 0 && (h_in || (syl == 1 && L % 8 != 0))) return false;
  if (((uintptr_t)x % 16) || ((uintptr_t)xn % 16) || ((uintptr_t)y % 16)) return false;
  const bool rows = syl == 1 && syd % 8 == 0 && syb % 8 == 0;
  const bool lines = syd == 1 && syl % 8 == 0 && syb % 8 == 0;
  if (!rows && !lines) return false;
  if (B * (D / kFC) * ceil_div(L, kFSeg) >= (int64_t)1 << 31) return false;
  return true;
}

}  // namespace
}  // namespace mega

using namespace mega;

// workspace (zero once, then owned by these calls): launch header + the records of whichever route a shape takes
extern "C" size_t mega_norm_ema_fwd_workspace_bytes(int64_t B, int64_t L, int64_t D, int64_t G, int64_t N) {
  (void)N;
  if (B <= 0 || L <= 0 || D <= 0 || G <= 0) return 256;
  const size_t fused = fused_ws_bytes(B * ceil_div(D, kFC), ceil_div(L, kFSeg));
  const size_t tsn = mega_timestep_norm_workspace_bytes(MEGA_BF16, B, L, D, G);
  return fused > tsn ? fused : tsn;
}

// scratch (no initialisation, contents never survive a call): the moving average's own workspace when the two
// operators run one after the other, or room for kernel generation when no image is passed
extern "C" size_t mega_norm_ema_fwd_scratch_bytes(int64_t B, int64_t L, int64_t D, int64_t G, int64_t N) {
  (void)G;
  if (B <= 0 || L <= 0 || D <= 0 || N <= 0) return 256;
  const size_t ema = mega_ema_fwd_workspace_bytes(B, D, N, L, 0, 0);
  const size_t img = mega_ema_image_bytes(D, N, 0);
  return align_up(ema > img ? ema : img, 256);
}

extern "C" int mega_norm_ema_fwd_train(const void* x, void* xn, void* y, int dtype, int64_t syb, int64_t syd,
                                       int64_t syl, const int64_t* prev_count, const float* prev_mean,
                                       const float* prev_var, const float* norm_gamma, const float* norm_beta,
                                       const uint8_t* mask, double eps, int64_t* count, float* mean, float* var,
                                       float* cummean, float* cumrstd, const float* p, const float* q,
                                       const float* gamma, int is_complex, const float* omega, const float* h_in,
                                       float* h_out, int64_t B, int64_t L, int64_t D, int64_t G, int64_t N,
                                       const void* image, void* workspace, size_t workspace_bytes, void* scratch,
                                       size_t scratch_bytes, void* stream) {
  if (const int rc = lookback_pending("norm_ema_fwd")) return rc;
  MEGA_REQUIRE((cummean == nullptr) == (cumrstd == nullptr), MEGA_ERR_ARG,
               "norm_ema_fwd: cummean and cumrstd go together");
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG,
               "norm_ema_fwd: unknown dtype %d", dtype);
  MEGA_REQUIRE(B >= 0 && L >= 0 && D > 0 && G > 0 && N > 0 && D % G == 0, MEGA_ERR_ARG,
               "norm_ema_fwd: bad shape B=%ld L=%ld D=%ld G=%ld N=%ld", (long)B, (long)L, (long)D, (long)G, (long)N);
  if (B == 0) return MEGA_OK;
  const size_t need = mega_norm_ema_fwd_workspace_bytes(B, L > 0 ? L : 1, D, G, N);
  MEGA_REQUIRE(workspace && workspace_bytes >= need, MEGA_ERR_WORKSPACE, "norm_ema_fwd: workspace of %zu bytes needed",
               need);
  hipStream_t s = (hipStream_t)stream;
  const int64_t S = ceil_div(L > 0 ? L : 1, kFSeg);
  char* w = (char*)workspace;
  const bool one_kernel = L > 0 && (image || mega_ema_image_bytes(D, N, 0) > 0) &&
                          fused_covers(dtype, B, L, D, G, N, x, xn, y, syb, syd, syl, mask, h_in);
  if (!one_kernel || !image) {
    const size_t sneed = mega_norm_ema_fwd_scratch_bytes(B, L > 0 ? L : 1, D, G, N);
    MEGA_REQUIRE(scratch && scratch_bytes >= sneed, MEGA_ERR_WORKSPACE, "norm_ema_fwd: scratch of %zu bytes needed",
                 sneed);
  }
  if (one_kernel) {
    MEGA_REQUIRE(x && xn && y && prev_count && prev_mean && prev_var && norm_gamma && norm_beta && count && mean &&
                     var && p && q && gamma && omega,
                 MEGA_ERR_ARG, "norm_ema_fwd: null pointer argument");
    MEGA_REQUIRE(!ranges_overlap(prev_count, (size_t)B * 8, count, (size_t)B * 8) &&
                     !ranges_overlap(prev_mean, (size_t)B * G * 4, mean, (size_t)B * G * 4) &&
                     !ranges_overlap(prev_var, (size_t)B * G * 4, var, (size_t)B * G * 4),
                 MEGA_ERR_ARG, "norm_ema_fwd: count / mean / var must not overlap prev_count / prev_mean / prev_var");
    MEGA_REQUIRE(!h_in || !h_out || !ranges_overlap(h_in, (size_t)B * D * N * 8, h_out, (size_t)B * D * N * 8),
                 MEGA_ERR_ARG, "norm_ema_fwd: h_out must not overlap h_in (every block reads h_in, the last writes h_out)");
    const void* img = image;
    if (!img) {
      // no cached image: kernel generation runs with every call
      const int rc = ema_image_build(p, q, gamma, is_complex, omega, D, N, 0, 1, scratch, s, kImgPC | kImgKT | kImgBlocks);
      if (rc) return rc;
      img = scratch;
    }
    FusedArgs A;
    A.x = (const bf16_t*)x; A.xn = (bf16_t*)xn; A.y = (bf16_t*)y; A.syb = syb; A.syd = syd; A.syl = syl;
    A.prev_count = prev_count; A.prev_mean = prev_mean; A.prev_var = prev_var; A.count = count; A.mean = mean;
    A.var = var; A.gamma = norm_gamma; A.beta = norm_beta; A.mask = mask; A.image = (const uint4*)img; A.h_in = h_in; A.h_out = h_out;
    A.cummean = cummean; A.cumrstd = cumrstd;
    A.hdr = (TsnHeader*)w; A.rec = (unsigned long long*)(w + align_up(sizeof(TsnHeader), 256));
    A.B = (int)B; A.L = (int)L; A.D = (int)D; A.G = (int)G; A.N = (int)N; A.S = (int)S; A.eps = (float)eps;
    A.pad = (int)(S * kFSeg - L);
    A.is_complex = is_complex;
    const int parts = (int)(D / (G * kFC));              // workgroups per norm group
    A.xcd_map = ((G * parts) % 8 == 0) ? 1 : 0;
    A.lb = lookback_launch(true);
    const dim3 grid((unsigned)(B * G * parts * S));
    // held-back starts only where the launch is one round of workgroups (one per compute unit) and fills most of it
    const int cus = device_cu_count();
    A.stagger = (S > 1 && S <= MEGA_FUSED_STAGGER_BLOCKS && (int64_t)grid.x <= cus &&
                 (int64_t)grid.x * MEGA_FUSED_STAGGER_FILL >= cus * (MEGA_FUSED_STAGGER_FILL - 1))
                    ? MEGA_FUSED_STAGGER
                    : 0;
    typedef void (*Kern)(const FusedArgs);
    const int lout = syl == 1 ? 0 : 1;
    const Kern kerns[2][2][2] = {
        {{norm_ema_fused_kernel<0, 64, false>, norm_ema_fused_kernel<0, 64, true>},
         {norm_ema_fused_kernel<1, 64, false>, norm_ema_fused_kernel<1, 64, true>}},
        {{norm_ema_fused_kernel<0, 128, false>, norm_ema_fused_kernel<0, 128, true>},
         {norm_ema_fused_kernel<1, 128, false>, norm_ema_fused_kernel<1, 128, true>}}};
    const int stag = A.stagger > 0 ? 1 : 0;
    const Kern kern = kerns[parts - 1][lout][stag];
    static uint64_t attr_seen[2][2][2] = {{{0, 0}, {0, 0}}, {{0, 0}, {0, 0}}};
    if (first_on_device(&attr_seen[parts - 1][lout][stag])) {
      (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kFSmem);
    }
    hipLaunchKernelGGL(kern, grid, dim3(kFT), kFSmem, s, A);
    MEGA_CHECK_LAUNCH("norm_ema_fwd");
    return lookback_verify("norm_ema_fwd", s);
  }
  // outside the one-kernel envelope: the two operators one after the other
  // (x -> xn by the norm, xn read through its transposed view by the moving average); the norm keeps its
  // launch header and tile records in the same workspace (same header, same protocol)
  int rc = mega_group_timestep_norm_fwd(x, xn, dtype, prev_count, prev_mean, prev_var, norm_gamma, norm_beta, mask, B, L,
                                        D, G, eps, count, mean, var, nullptr, cummean, cumrstd, workspace,
                                        workspace_bytes, stream);
  if (rc) return rc;
  return mega_ema_fwd(xn, y, dtype, L * D, 1, D, syb, syd, syl, p, q, gamma, is_complex, omega, mask, h_in, h_out, B, D,
                      N, L, 0, 0, 1, image, scratch, scratch_bytes, stream);
}

extern "C" int mega_norm_ema_fwd(const void* x, void* xn, void* y, int dtype, int64_t syb, int64_t syd, int64_t syl,
                                 const int64_t* prev_count, const float* prev_mean, const float* prev_var,
                                 const float* norm_gamma, const float* norm_beta, const uint8_t* mask, double eps,
                                 int64_t* count, float* mean, float* var, const float* p, const float* q,
                                 const float* gamma, int is_complex, const float* omega, const float* h_in,
                                 float* h_out, int64_t B, int64_t L, int64_t D, int64_t G, int64_t N,
                                 const void* image, void* workspace, size_t workspace_bytes, void* scratch,
                                 size_t scratch_bytes, void* stream) {
  return mega_norm_ema_fwd_train(x, xn, y, dtype, syb, syd, syl, prev_count, prev_mean, prev_var, norm_gamma, norm_beta,
                                 mask, eps, count, mean, var, nullptr, nullptr, p, q, gamma, is_complex, omega, h_in,
                                 h_out, B, L, D, G, N, image, workspace, workspace_bytes, scratch, scratch_bytes, stream);
}
