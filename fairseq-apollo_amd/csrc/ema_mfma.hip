// Moving-average layer forward on the matrix cores (gfx950 MFMA), ndim <= 16, bf16 activations.
//
// For one channel the layer is y = k * x + omega x with k[l] = Re sum_n p gamma q^l
// (fairseq/modules/complex_exponential_moving_average.py:98-109,
// fairseq/modules/base_moving_average.py:120-172).  Time is cut into tiles of 32 tokens.
// With h the carried state (h' = q h + p x, fairseq/csrc/ops/ema_hidden.cc:31-63) a tile is
//
//     y_tile = K x_tile + C h_start        K[i][i'] = k[i - i'] (lower-triangular Toeplitz)
//     h_end  = Q h_start + P x_tile        C[i][n]  = gamma_n q_n^{i+1},  P[n][i] = p_n q_n^{31-i}
//
// which is the reference's own incremental decomposition (kernel + carried-state bias,
// fairseq/csrc/ops/ema_parameters.cc:37-77) applied per tile.  K, P, C are 32x32 matrices that
// depend on the channel only.
//
// Kernel generation (ema_image_kernel): a workgroup of four waves per coefficient row; every wave builds the
// q-power table in LDS and the waves share out what is formed from it: the MFMA A-operand images of K, P, C
// (bf16, optionally with a second bf16 correction term) plus the per-state multipliers q^32 and q^(32 SEGT).  The image is what the
// reference caches as `_coeffs` / recomputes as the D x L kernel; here it is 9-13 KB per channel
// whatever L is.
//
// Streaming (ema_mfma_kernel): one wave owns one (batch, channel) row for the whole sequence and
// keeps the image in registers; a workgroup is 16 waves = 16 adjacent channels, so a [B, L, D]
// tensor is streamed as 32-byte pieces per token that the workgroup transposes through LDS (the
// four workgroups that share a 128-byte line are placed on the same XCD), and a [B, D, L] tensor
// as contiguous rows.  A super-chunk of 16 segments x SEGT tiles is resident in LDS.  The 16
// MFMA columns are the 16 segments, so the tile-to-tile recurrence stays inside a lane:
//   sweep 1: segment end states from a zero start            (P products only)
//   scan   : 16-step serial scan over the segments per state (lanes 0..15, values in registers)
//   sweep 2: K, P, C products with the true start states; y overwrites x in LDS
#include "ema_mfma.h"

// Phase markers of the streaming kernel: a profiling build defines MEGA_TR(k) to stamp the
// shader clock; here they expand to nothing.
#ifndef MEGA_TR
#define MEGA_TR(k)
#define MEGA_TR_FLUSH()
#endif

// 1: the states enter the output product as two bf16 terms for every channel (one term leaves an error of 2^-9 of
// sum |gamma q h| at the first tokens of every tile); 0: only for slow poles, layers of few states and real-valued
// layers, the rule of the one-kernel block.  The C operand is one bf16 term either way (2^-9 of the same sum)
#ifndef MEGA_TWO_ALWAYS
#define MEGA_TWO_ALWAYS 0
#endif
namespace mega {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kWaves = 16;               // channels per workgroup
constexpr int kThreadsM = kWaves * 64;

// ------------------------------------------------------------------------------------------
// kernel generation
// ------------------------------------------------------------------------------------------
struct ImageArgs {
  const float* p;        // [K, N]
  const float* q;        // [K, N, 2]
  const float* gamma;    // [K, N, 2]
  const float* omega;    // [D] or null
  uint4* image;          // [K][kImgSlots][64]
  int K, D, N;
  int is_complex;
  int lag_back;          // rows >= D exclude the current sample (backward half with shift)
  int parts;             // 1: the bf16 K / P / C operands are wanted, 2: the fp16 ones (the tables always are)
};

__device__ __forceinline__ float bf_split(float v, __bf16* h) {
  *h = (__bf16)v;
  return v - (float)(*h);
}

constexpr int kPrepWaves = 4;
constexpr int kPowB = 33 * kNS * 8;
constexpr int kAuxB = 64 * 4 + kNS * 4 + kNS * 8 + kNS * 16;

// The powers of q are formed in double precision and rounded once: a power q^L formed by fp32 products carries L
// roundings of q, which at L = 15 * 1024 and |q| = 1 - 3e-5 is 4e-4 of a term that still matters (the reference
// takes exp(l log q), complex_exponential_moving_average.py:103-106, whose error does not grow with l either).
struct cdouble {
  double re, im;
};
__device__ __forceinline__ cdouble cmuld(cdouble a, cdouble b) {
  return {a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
}
__device__ __forceinline__ cfloat to_cfloat(cdouble a) { return {(float)a.re, (float)a.im}; }

__global__ __launch_bounds__(kPrepWaves * 64) void ema_image_kernel(const ImageArgs A) {
  __shared__ __attribute__((aligned(16))) char smem[kPrepWaves * (kPowB + kAuxB)];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int kr = blockIdx.x;                        // one coefficient row per workgroup, shared by its four waves
  const int lag = (kr >= A.D && A.lag_back) ? 1 : 0;
  float2* pw = (float2*)(smem + wave * kPowB);
  float* kkt = (float*)(smem + kPrepWaves * kPowB + wave * kAuxB);   // [64]: k[idx] at kkt[32 + idx]
  float* pbuf = kkt + 64;
  float2* gbuf = (float2*)(pbuf + kNS);
  double2* q32d = (double2*)(gbuf + kNS);                             // [kNS]: q^32 before rounding
  const int r = lane >> 4;
  {
    const int n = lane & 15, blk = lane >> 4;
    float qr = 0.f, qi = 0.f, pv = 0.f, gr = 0.f, gi = 0.f;
    if (n < A.N) {
      const size_t o = ((size_t)kr * A.N + n);
      qr = A.q[o * 2];
      qi = A.is_complex ? A.q[o * 2 + 1] : 0.f;
      pv = A.p[o];
      gr = A.gamma[o * 2];
      gi = A.is_complex ? A.gamma[o * 2 + 1] : 0.f;
    }
    const cdouble q1 = {(double)qr, (double)qi};
    const cdouble q2 = cmuld(q1, q1), q4 = cmuld(q2, q2), q8 = cmuld(q4, q4), q16 = cmuld(q8, q8), q24 = cmuld(q16, q8);
    cdouble base = blk == 0 ? cdouble{1.0, 0.0} : blk == 1 ? q8 : blk == 2 ? q16 : q24;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      pw[(8 * blk + t) * kNS + n] = make_float2((float)base.re, (float)base.im);
      base = cmuld(base, q1);
    }
    if (blk == 3) {
      pw[32 * kNS + n] = make_float2((float)base.re, (float)base.im);
      q32d[n] = make_double2(base.re, base.im);
    }
    if (blk == 0) {
      pbuf[n] = pv;
      gbuf[n] = make_float2(gr, gi);
    }
  }
  __syncthreads();
  {
    // k[e] = Re sum_n p gamma q^e; lag 1 shifts it by one tap; omega joins tap 0 of the forward rows
    const int e = lane & 31;
    float s = 0.f;
#pragma unroll
    for (int n = 0; n < kNS; ++n) {
      const float2 w = pw[e * kNS + n];
      const float2 g = gbuf[n];
      s += pbuf[n] * (g.x * w.x - g.y * w.y);
    }
    const int idx = e + lag;
    if (lane < 32) {
      if (idx < 32) kkt[32 + idx] = s;
      kkt[lane] = 0.f;
    }
  }
  __syncthreads();
  if (lane == 0) {
    if (lag) kkt[32] = 0.f;
    if (A.omega && kr < A.D) kkt[32] += A.omega[kr];
  }
  __syncthreads();
  uint4* img = A.image + (size_t)kr * kImgSlots * 64;
  const int m = lane & 15, g = lane >> 4;
  // ---- the K / P / C operands in the matrix-core A layout: bf16 terms (kImgKFull: K, kImgPC: P and C) and fp16 terms
  // (kImgF16); only what the caller's kernel reads is formed and written.  The four waves of the workgroup hold the
  // same tables and share the channel's work: wave 0 the P operand and the per-state tables, wave 1 the C operand,
  // wave 2 the K operand (full and compact), wave 3 the multipliers of the block kernels.
  const bool want_k = A.parts & kImgKFull, want_pc = A.parts & kImgPC, want_16 = A.parts & kImgF16;
  typedef __attribute__((ext_vector_type(8))) _Float16 f16x8v;
  // value of operand `o` (0: K, 1: P, 2: C) at row `row`, k-slot t of block g
  auto value = [&](const int o, const int row, const int t) -> float {
    const int k = 8 * g + t;
    if (o == 0) return kkt[32 + row - k];                  // K: rows = output time, k = input time (Toeplitz)
    if (o == 1) {                                          // P: rows = (state, part), k = input time i: p q^{31-i}
      const int n = row >> 1, part = row & 1;
      const float2 w = pw[(31 - k) * kNS + n];
      return pbuf[n] * (part ? w.y : w.x);
    }
    // C: rows = output time i; k-slot t of block g <-> state 2g + t/2 (t < 4) or 8 + 2g + (t-4)/2, part t & 1:
    // Re(gamma q^{i+1-lag}) multiplies Re h, -Im(...) multiplies Im h
    const int n = (t < 4) ? (2 * g + (t >> 1)) : (8 + 2 * g + ((t - 4) >> 1));
    const float2 w = pw[(row + 1 - lag) * kNS + n];
    const float2 gm = gbuf[n];
    return (t & 1) ? -(gm.x * w.y + gm.y * w.x) : (gm.x * w.x - gm.y * w.y);
  };
  auto build = [&](const int o, const int nw, const int slot, const bool want_bf, const int slot16) {
    if (!want_bf && !want_16) return;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      bf16x8 hi8, lo8;
      f16x8v h0, h1;
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const float v = value(o, 16 * mb + m, t);
        __bf16 h;
        const float rem = bf_split(v, &h);
        hi8[t] = h;
        lo8[t] = (__bf16)rem;
        const _Float16 h16 = (_Float16)v;
        h0[t] = h16;
        h1[t] = (_Float16)(v - (float)h16);
      }
      if (want_bf) {
        img[(slot + mb) * 64 + lane] = __builtin_bit_cast(uint4, hi8);
        if (nw > 1) img[(slot + 2 * (nw - 1) + mb) * 64 + lane] = __builtin_bit_cast(uint4, lo8);
      }
      if (want_16) {
        img[(size_t)(slot16 + mb) * 64 + lane] = __builtin_bit_cast(uint4, h0);
        img[(size_t)(slot16 + 2 + mb) * 64 + lane] = __builtin_bit_cast(uint4, h1);
      }
    }
  };
  static_assert(kNWK <= 2 && kNWP <= 2 && kNWC <= 2, "operands of one or two bf16 terms");
  if (wave == 0) build(1, kNWP, kSlotP, want_pc, kSlotK16 + 4);
  if (wave == 1) build(2, kNWC, kSlotC, want_pc, kSlotK16 + 8);
  if (wave == 2) build(0, kNWK, kSlotK, want_k, kSlotK16);
  if (wave == 0 && (A.parts & kImgStream)) {
    // q^32 of this lane's four states (2r, 2r+1, 8+2r, 9+2r)
    const float2 a = pw[32 * kNS + 2 * r], bq = pw[32 * kNS + 2 * r + 1];
    const float2 c = pw[32 * kNS + 8 + 2 * r], d = pw[32 * kNS + 9 + 2 * r];
    img[kSlotQ32 * 64 + lane] = make_uint4(__float_as_uint(a.x), __float_as_uint(a.y), __float_as_uint(bq.x),
                                           __float_as_uint(bq.y));
    img[(kSlotQ32 + 1) * 64 + lane] = make_uint4(__float_as_uint(c.x), __float_as_uint(c.y), __float_as_uint(d.x),
                                                 __float_as_uint(d.y));
    // scan multiplier q^(32 SEGT) of state `lane >> 2`
    cdouble Rd = {1.0, 0.0};
    const double2 w = q32d[lane >> 2];
    for (int t = 0; t < kSEGT; ++t) Rd = cmuld(Rd, cdouble{w.x, w.y});
    const cfloat R = to_cfloat(Rd);
    img[kSlotScan * 64 + lane] = make_uint4(__float_as_uint(R.re), __float_as_uint(R.im), 0u, 0u);
  }
  if (wave == 3 && (A.parts & kImgBlocks)) {
    // multipliers in the matrix-core lane layout (lane = segment j + 16 r, states 2r, 2r+1, 8+2r, 9+2r), for the
    // kernels that scan 16 segments of 64 tokens across the lanes of a row and look back over blocks of 1024 tokens:
    // (q^64)^j and (q^1024)^j, each power by squaring and multiplying (at most eight products in a row)
    const int nn[4] = {2 * r, 2 * r + 1, 8 + 2 * r, 9 + 2 * r};
    cfloat RJ[4], RWJ[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const double2 w32 = q32d[nn[u]];
      cdouble sq = cmuld(cdouble{w32.x, w32.y}, cdouble{w32.x, w32.y});          // q^64
      cdouble a = {1.0, 0.0};
#pragma unroll
      for (int bit = 0; bit < 4; ++bit) {
        if (m & (1 << bit)) a = cmuld(a, sq);
        sq = cmuld(sq, sq);
      }
      RJ[u] = to_cfloat(a);                                                       // sq = q^1024 now
      cdouble c = {1.0, 0.0};
#pragma unroll
      for (int bit = 0; bit < 4; ++bit) {
        if (m & (1 << bit)) c = cmuld(c, sq);
        sq = cmuld(sq, sq);
      }
      RWJ[u] = to_cfloat(c);
    }
    auto put2 = [&](const int slot, const cfloat (&v)[4]) {
      img[slot * 64 + lane] = make_uint4(__float_as_uint(v[0].re), __float_as_uint(v[0].im),
                                         __float_as_uint(v[1].re), __float_as_uint(v[1].im));
      img[(slot + 1) * 64 + lane] = make_uint4(__float_as_uint(v[2].re), __float_as_uint(v[2].im),
                                               __float_as_uint(v[3].re), __float_as_uint(v[3].im));
    };
    put2(kSlotRJ, RJ);
    put2(kSlotRWJ, RWJ);
  }
  {
    if (wave == 0 && lane < kNS) {
      // the per-state multipliers once per state (a lane of the streaming kernels reads 16 bytes = two states)
      float2* cmp = (float2*)(img + (size_t)kSlotCmp * 64);
      const double2 w32 = q32d[lane];
      cdouble v = {w32.x, w32.y};
      cmp[kCmpQ32 * kNS + lane] = make_float2((float)v.re, (float)v.im);
      v = cmuld(v, v);
      cmp[kCmpRS * kNS + lane] = make_float2((float)v.re, (float)v.im);
      v = cmuld(v, v);
      cmp[kCmpRS2 * kNS + lane] = make_float2((float)v.re, (float)v.im);
      v = cmuld(v, v);
      cmp[kCmpRS4 * kNS + lane] = make_float2((float)v.re, (float)v.im);
      v = cmuld(v, v);
      cmp[kCmpRS8 * kNS + lane] = make_float2((float)v.re, (float)v.im);
      v = cmuld(v, v);
      cmp[kCmpRW * kNS + lane] = make_float2((float)v.re, (float)v.im);
    }
    if (wave == 2 && lane < 56 && (A.parts & kImgKT)) {
      // the K operand once per distinct content: lane (m, g) of row block mb holds k[16 mb + m - 8 g - t], t = 0..7,
      // which depends on delta = 16 mb + m - 8 g (-24..31) only; vector delta + 24 of term w sits at byte
      // 16 (delta + 24) of slot kSlotKT + w (7 lines per term instead of 16)
      const int delta = lane - 24;
#pragma unroll
      for (int w = 0; w < kNWK; ++w) {
        bf16x8 v;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          __bf16 h;
          const float rem = bf_split(kkt[32 + delta - t], &h);
          v[t] = w == 0 ? h : (__bf16)rem;
        }
        img[(size_t)(kSlotKT + w) * 64 + lane] = __builtin_bit_cast(uint4, v);
      }
    }
    {
      // reach of the channel's slowest pole: m = max |q|^64; a contribution over t tokens is dropped by the
      // streaming kernels once |q|^t < 2^-24 (below fp32 resolution of what it is added to)
      const float2 w32 = pw[32 * kNS + (lane & 15)];
      float m = w32.x * w32.x + w32.y * w32.y;             // |q^32|^2 = |q|^64
#pragma unroll
      for (int o = 8; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
      const float lim = 0x1p-24f;
      float md = m;
      int nsteps = 0;
      for (int t = 0; t < 4; ++t) {                         // |q|^(64 d) for d = 1, 2, 4, 8
        if (md >= lim) nsteps = t + 1;
        md *= md;
      }
      // md = |q|^1024 now
      int nlook = 1;
      float w = md;
      while (nlook < 16 && w >= lim) {
        w *= md;
        ++nlook;
      }
      if (wave == 0 && lane == 0) {
        uint32_t* rw = (uint32_t*)(img + (size_t)kSlotCmp * 64) + kCmpReach * kNS * 2;
        rw[0] = (uint32_t)nsteps;
        rw[1] = (uint32_t)nlook;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// streaming
// ------------------------------------------------------------------------------------------
struct MfmaArgs {
  const void* x;
  void* y;
  int64_t sxb, sxd, sxl, syb, syd, syl;
  const uint4* image;    // [K][kImgSlots][64]
  const float* omega;    // [D] or null (null: no residual in this pass)
  const uint8_t* mask;   // [B, L] or null
  const float* h_in;     // [B, D, N, 2] or null
  float* h_tile;         // [B, D, 16, 2]: state after the last whole 32-token tile, or null
  const float* acc_in;   // fp32, strides (sab, sad, sal), or null
  float* acc_out;        // fp32, same strides; when set y is not written
  int64_t sab, sad, sal;
  int B, D, N, L;
  int koff;              // first coefficient row of this direction
  int reverse;           // logical time runs backwards
  int is_complex;
  int xcd_map;           // 1: sibling channel blocks share an XCD
};

struct Geo {
  static constexpr int SEG = kSEGT * 32;           // tokens per segment
  static constexpr int SC = SEG * 16;              // tokens per super-chunk
  static constexpr int SEGB = SEG * 2 + 16;        // bytes per segment in an LDS row (padded)
  static constexpr int ROWB = SEGB * 16 + 16;      // bytes per channel row; (ROWB / 4) % 16 == 4
  static constexpr int XBUF = ROWB * kWaves;
  static constexpr int SCANJ = 20;                 // complex slots per segment in the scan buffer (16 + 4 pad)
  static constexpr int SCANB = 16 * SCANJ * 8;     // segment states per channel
  static constexpr int QTAB = XBUF + kWaves * SCANB;   // q^32 of every wave's channel: [kWaves][4 row blocks][4 states] complex
  static constexpr int TOTAL = QTAB + kWaves * 128;
  static_assert((ROWB / 4) % 16 == 4, "row stride must spread the four rows of a store over the banks");
  __device__ static __forceinline__ int pos(int t) { return (t / SEG) * SEGB + (t % SEG) * 2; }
};

__device__ __forceinline__ uint32_t dpp_swap2(uint32_t v) {      // lane ^ 2 within a quad
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, true);
}

// Layouts (LIN of x, LOUT of y, independent): 0 = [B, D, L] rows contiguous in time, 1 = [B, L, D]
// channels contiguous.  LIN 1 / LOUT 0 reads the transposed view the layer passes and writes the
// rows the reference's convolution returns (rfft / irfft output, fused_ops/fftconv.py:45-61).
// FAST: whole super-chunks and whole channel blocks only, no padding mask, no partial sums:
// every load and store of the streaming loop is unconditional straight-line code, so the
// stores of one super-chunk stay in flight under the next one's staging and sweeps (with a
// branch around them the loop has to drain them before it may consume the prefetched loads).
template <int LIN, int LOUT, int MODE>
__global__ __launch_bounds__(kThreadsM) void ema_mfma_kernel(const MfmaArgs A) {
  using G = Geo;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int j = lane & 15, r = lane >> 4;          // MFMA column / row block

  // ---- which (batch, channel block)
  const int ncb = (A.D + kWaves - 1) / kWaves;
  int b, cb;
  {
    const int g = blockIdx.x;
    if (A.xcd_map) {
      const int xcd = g & 7, slot = g >> 3;
      const int s = slot & 3, gi = (slot >> 2) * 8 + xcd;
      const int per = ncb >> 2;
      b = gi / per;
      cb = (gi - b * per) * 4 + s;
    } else {
      b = g / ncb;
      cb = g - b * ncb;
    }
  }
  const int ch = cb * kWaves + wave;
  // MODE 0: general; 1: FAST; 2: FAST with an even number of super-chunks, two of them in flight
  constexpr bool FAST = MODE != 0;
  const bool ch_ok = FAST || ch < A.D;
  const int chc = ch_ok ? ch : A.D - 1;            // idle waves compute on a valid row, never store
  char* xrow = smem + wave * G::ROWB;
  char* scan = smem + G::XBUF + wave * G::SCANB;

  const int nsc = (A.L + G::SC - 1) / G::SC;
  const int last_tile = A.L / 32 - 1;             // global index of the last whole tile
  constexpr int NLD = G::SC * 2 * kWaves / (kThreadsM * 16);   // 16-byte pieces per thread per super-chunk
  // MODE 2 keeps two super-chunks of loads in flight (one register set each): the 32-byte pieces
  // make a load take longer from issue to arrival than one super-chunk takes to compute.  Its loop
  // has no branch around a load or a store (loads past the end fetch token 0 again and are never
  // used), so every wait inside the loop counts exactly what may stay in flight.
  constexpr int DEPTH = MODE == 2 ? 2 : 1;
  uint4 preA[NLD], preB[NLD];
  const bf16_t* xg = (const bf16_t*)A.x;
  // layout 1: a lane pair (lane, lane ^ 2) covers tokens (2m, 2m+1) x 8 channels (half = lane & 1)
  const int half = tid & 1;
  const int odd = (tid >> 1) & 1;
  // byte selectors of v_perm_b32 (source bytes 0..3 = second operand, 4..7 = first operand):
  // staging packs (even token | odd token << 16) per channel, the store unpacks it again
  const uint32_t sel_lo = odd ? 0x01000504u : 0x05040100u;
  const uint32_t sel_hi = odd ? 0x03020706u : 0x07060302u;
  const uint32_t sel_keep = odd ? 0x07060302u : 0x05040100u;
  const uint32_t sel_give = odd ? 0x05040100u : 0x07060302u;

  auto issue_loads = [&](int sc, uint4 (&pre)[NLD]) {
    const int t0 = sc * G::SC;
#pragma unroll
    for (int k = 0; k < NLD; ++k) {
      pre[k] = make_uint4(0, 0, 0, 0);
      if (LIN == 1) {
        const int tk = k * (kThreadsM / 2) + (tid >> 1);
        const int tau = t0 + tk;
        const int c0 = cb * kWaves + half * 8;
        if (FAST) {
          int t = A.reverse ? A.L - 1 - tau : tau;
          if (MODE == 2) t = sc < nsc ? t : 0;
          pre[k] = *(const uint4*)(xg + b * A.sxb + (int64_t)t * A.sxl + c0);
        } else if (tau < A.L && c0 < A.D) {
          const int t = A.reverse ? A.L - 1 - tau : tau;
          if (!(A.mask && A.mask[(size_t)b * A.L + t]))
            pre[k] = *(const uint4*)(xg + b * A.sxb + (int64_t)t * A.sxl + c0);
        }
      } else {
        const int tk = k * 512 + lane * 8;
        const int tau = t0 + tk;
        if (FAST || tau < A.L) {
          int t = A.reverse ? A.L - 8 - tau : tau;
          if (MODE == 2) t = sc < nsc ? t : 0;
          uint4 v = *(const uint4*)(xg + b * A.sxb + (int64_t)chc * A.sxd + t);
          if (A.reverse) {
            uint4 w;
            w.x = (v.w >> 16) | (v.w << 16);
            w.y = (v.z >> 16) | (v.z << 16);
            w.z = (v.y >> 16) | (v.y << 16);
            w.w = (v.x >> 16) | (v.x << 16);
            v = w;
          }
          if (!FAST && A.mask) {
            const uint2 mk = *(const uint2*)(A.mask + (size_t)b * A.L + t);
            const uint32_t mm[2] = {mk.x, mk.y};
            uint32_t* vv = (uint32_t*)&v;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const int src = A.reverse ? 7 - e : e;           // mask byte of logical element e
              const bool pad = ((mm[src >> 2] >> ((src & 3) * 8)) & 0xffu) != 0;
              if (pad) vv[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
            }
          }
          pre[k] = v;
        }
      }
    }
  };

  MEGA_TR(0);
  issue_loads(0, preA);

  // ---- operand images of this channel: registers for the whole kernel
  bf16x8 Kw[kNWK][2], Pw[kNWP][2], Cw[kNWC][2];
  char* const qtab = smem + G::QTAB + wave * 128;
  // segment scan: lane (n = lane >> 2, c = lane & 3) owns state n over segments 4c .. 4c+3
  float Rr, Ri;                        // q^(32 SEGT) of state n: the scan's multiplier
  float Hcr = 0.f, Hci = 0.f;          // carried state of state n, in the lanes with c == 0 (zero elsewhere)
  bool two_terms = false;              // the states enter the output product as two bf16 terms (wave-uniform)
  {
    const uint4* img = A.image + (size_t)(A.koff + chc) * kImgSlots * 64 + lane;
    int slot = 0;
#pragma unroll
    for (int w = 0; w < kNWK; ++w)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) Kw[w][mb] = __builtin_bit_cast(bf16x8, img[(slot++) * 64]);
#pragma unroll
    for (int w = 0; w < kNWP; ++w)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) Pw[w][mb] = __builtin_bit_cast(bf16x8, img[(slot++) * 64]);
#pragma unroll
    for (int w = 0; w < kNWC; ++w)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) Cw[w][mb] = __builtin_bit_cast(bf16x8, img[(slot++) * 64]);
    const uint4 qa = img[(slot++) * 64], qb = img[(slot++) * 64], rr = img[(slot++) * 64];
    // q^32 of the lane's four states waits in LDS between uses (eight registers less across the streaming loop);
    // only the wave itself reads its table
    if (j == 0) {
      *(uint4*)(qtab + r * 32) = qa;
      *(uint4*)(qtab + r * 32 + 16) = qb;
    }
    Rr = __uint_as_float(rr.x);
    Ri = __uint_as_float(rr.y);
    // the second term where the reach word of the image says |q|^128 >= 2^-24 for some state of the channel, in
    // layers of few states (their rounding errors do not average out in the sum over the states) and in real-valued
    // layers (input weights of alternating sign: the states cancel by construction)
    two_terms = A.N <= 8 || !A.is_complex ||
                __builtin_amdgcn_readfirstlane(
                    (int)*(const uint32_t*)((const char*)(A.image + (size_t)(A.koff + chc) * kImgSlots * 64) +
                                            kSlotCmp * 1024 + kCmpReach * 128)) >= 2;
    if (A.h_in && (lane & 3) == 0 && (lane >> 2) < A.N && ch_ok) {
      const size_t o = (((size_t)b * A.D + ch) * A.N + (lane >> 2)) * 2;
      Hcr = A.h_in[o];
      Hci = A.is_complex ? A.h_in[o + 1] : 0.f;
    }
  }
  MEGA_TR(1);
  if (DEPTH == 2) issue_loads(1, preB);
  // The first super-chunk and the images are consumed here, outside the loop (only the second
  // super-chunk's loads stay pending): a wait for them placed inside the loop would also drain the
  // loads that are meant to stay in flight across iterations.
  {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    auto pin = [](bf16x8& v) {
      u32x4 t = __builtin_bit_cast(u32x4, v);
      asm volatile("" : "+v"(t));
      v = __builtin_bit_cast(bf16x8, t);
    };
#pragma unroll
    for (int w = 0; w < kNWK; ++w) { pin(Kw[w][0]); pin(Kw[w][1]); }
#pragma unroll
    for (int w = 0; w < kNWP; ++w) { pin(Pw[w][0]); pin(Pw[w][1]); }
#pragma unroll
    for (int w = 0; w < kNWC; ++w) { pin(Cw[w][0]); pin(Cw[w][1]); }
    asm volatile("" : "+v"(Rr), "+v"(Ri), "+v"(Hcr), "+v"(Hci));
  }

  MEGA_TR(2);
  auto body = [&](const int sc, uint4 (&pre)[NLD]) {
    const int t0 = sc * G::SC;
    MEGA_TR(3 + sc * 9);
    // ---- stage the prefetched super-chunk into LDS
#pragma unroll
    for (int k = 0; k < NLD; ++k) {
      if (LIN == 1) {
        // pair exchange: the even-token lane ends up with channels 0..3 of both tokens, the
        // odd-token lane with channels 4..7, each as dwords (even token | odd token << 16)
        const int tk = k * (kThreadsM / 2) + (tid >> 1);
        const uint4 v = pre[k];
        const uint32_t s0 = odd ? v.x : v.z, s1 = odd ? v.y : v.w;
        const uint32_t r0 = dpp_swap2(s0), r1 = dpp_swap2(s1);      // the partner's token, my channels
        const uint32_t m0 = odd ? v.z : v.x, m1 = odd ? v.w : v.y;  // my token, my channels
        uint32_t w[4];
        w[0] = __builtin_amdgcn_perm(r0, m0, sel_lo);
        w[1] = __builtin_amdgcn_perm(r0, m0, sel_hi);
        w[2] = __builtin_amdgcn_perm(r1, m1, sel_lo);
        w[3] = __builtin_amdgcn_perm(r1, m1, sel_hi);
        char* base = smem + (half * 8 + odd * 4) * G::ROWB + G::pos(tk & ~1);
#pragma unroll
        for (int e = 0; e < 4; ++e) *(uint32_t*)(base + e * G::ROWB) = w[e];
      } else {
        const int tk = k * 512 + lane * 8;
        *(uint4*)(xrow + G::pos(tk)) = pre[k];
      }
    }
    MEGA_TR(4 + sc * 9);
    __syncthreads();
    MEGA_TR(5 + sc * 9);
    if (MODE == 2 || sc + DEPTH < nsc) issue_loads(sc + DEPTH, pre);      // the staged registers are free again
    MEGA_TR(6 + sc * 9);

    // ---- sweep 1: segment end states from a zero start
    float Qr[4], Qi[4];
    auto load_q = [&]() {
      asm volatile("" ::: "memory");
      const float4 qa = *(const float4*)(qtab + r * 32), qb = *(const float4*)(qtab + r * 32 + 16);
      Qr[0] = qa.x; Qi[0] = qa.y; Qr[1] = qa.z; Qi[1] = qa.w;
      Qr[2] = qb.x; Qi[2] = qb.y; Qr[3] = qb.z; Qi[3] = qb.w;
    };
    load_q();
    float Er[4] = {0.f, 0.f, 0.f, 0.f}, Ei[4] = {0.f, 0.f, 0.f, 0.f};
    const char* xcol = xrow + j * G::SEGB + r * 16;
#pragma unroll
    for (int i = 0; i < kSEGT; ++i) {
      const bf16x8 X = *(const bf16x8*)(xcol + i * 64);
      f32x4 S0 = {0.f, 0.f, 0.f, 0.f}, S1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < kNWP; ++w) {
        S0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Pw[w][0], X, S0, 0, 0, 0);
        S1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Pw[w][1], X, S1, 0, 0, 0);
      }
      const float sr[4] = {S0[0], S0[2], S1[0], S1[2]};
      const float si[4] = {S0[1], S0[3], S1[1], S1[3]};
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float nr = fmaf(Qr[u], Er[u], fmaf(-Qi[u], Ei[u], sr[u]));
        const float ni = fmaf(Qr[u], Ei[u], fmaf(Qi[u], Er[u], si[u]));
        Er[u] = nr;
        Ei[u] = ni;
      }
    }
    MEGA_TR(7 + sc * 9);
    // ---- scan over the 16 segments (per state), carried across super-chunks
    {
      // [16 segments][SCANJ] complex: states (2r, 2r+1) of segment j at float4 [j * SCANJ/2 + r]
      float4* sb = (float4*)scan;
      constexpr int J4 = G::SCANJ / 2;
      sb[j * J4 + r] = make_float4(Er[0], Ei[0], Er[1], Ei[1]);
      sb[j * J4 + 4 + r] = make_float4(Er[2], Ei[2], Er[3], Ei[3]);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_wave_barrier();
      {
        const int n = lane >> 2, c = lane & 3;
        // powers of the multiplier, rebuilt here rather than held in registers across the loop
        // (the opaque copy keeps the compiler from hoisting them back out)
        float Tr = Rr, Ti = Ri;
        asm volatile("" : "+v"(Tr), "+v"(Ti));
        const float R2r = Tr * Tr - Ti * Ti, R2i = 2.f * Tr * Ti;
        const float R3r = R2r * Tr - R2i * Ti, R3i = R2r * Ti + R2i * Tr;
        float R4r = R2r * R2r - R2i * R2i, R4i = 2.f * R2r * R2i;
        float R8r = R4r * R4r - R4i * R4i, R8i = 2.f * R4r * R4i;
        if (c < 1) { R4r = 0.f; R4i = 0.f; }     // quarter 0 has no predecessor
        if (c < 2) { R8r = 0.f; R8i = 0.f; }     // quarters 0, 1 have none two back
        float2* s2 = (float2*)scan + (4 * c) * G::SCANJ + n;
        float2 e[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) e[k] = s2[k * G::SCANJ];
        // quarter-local exclusive scan (the carry enters quarter 0 here)
        float ar = Hcr, ai = Hci, outr[4], outi[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          outr[k] = ar;
          outi[k] = ai;
          const float nr = fmaf(Rr, ar, fmaf(-Ri, ai, e[k].x));
          const float ni = fmaf(Rr, ai, fmaf(Ri, ar, e[k].y));
          ar = nr;
          ai = ni;
        }
        // inclusive scan of the quarter totals across the quad (multipliers q^(4 seg), q^(8 seg))
        {
          const float xr = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ar), 0x90, 0xf, 0xf, false));
          const float xi = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ai), 0x90, 0xf, 0xf, false));
          ar = fmaf(R4r, xr, fmaf(-R4i, xi, ar));
          ai = fmaf(R4r, xi, fmaf(R4i, xr, ai));
        }
        {
          const float xr = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ar), 0x44, 0xf, 0xf, false));
          const float xi = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ai), 0x44, 0xf, 0xf, false));
          ar = fmaf(R8r, xr, fmaf(-R8i, xi, ar));
          ai = fmaf(R8r, xi, fmaf(R8i, xr, ai));
        }
        // carry into this quarter = total up to the previous one (quarter 0 already has its own)
        float cr = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ar), 0x90, 0xf, 0xf, false));
        float ci = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ai), 0x90, 0xf, 0xf, false));
        const float tr = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ar), 0xFF, 0xf, 0xf, false));
        const float ti = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ai), 0xFF, 0xf, 0xf, false));
        cr = c == 0 ? 0.f : cr;
        ci = c == 0 ? 0.f : ci;
        Hcr = c == 0 ? tr : 0.f;
        Hci = c == 0 ? ti : 0.f;
        outr[0] += cr;
        outi[0] += ci;
        outr[1] = fmaf(Rr, cr, fmaf(-Ri, ci, outr[1]));
        outi[1] = fmaf(Rr, ci, fmaf(Ri, cr, outi[1]));
        outr[2] = fmaf(R2r, cr, fmaf(-R2i, ci, outr[2]));
        outi[2] = fmaf(R2r, ci, fmaf(R2i, cr, outi[2]));
        outr[3] = fmaf(R3r, cr, fmaf(-R3i, ci, outr[3]));
        outi[3] = fmaf(R3r, ci, fmaf(R3i, cr, outi[3]));
#pragma unroll
        for (int k = 0; k < 4; ++k) s2[k * G::SCANJ] = make_float2(outr[k], outi[k]);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_wave_barrier();
    }
    float Hr[4], Hi[4];
    {
      const float4* sb = (const float4*)scan;
      constexpr int J4 = G::SCANJ / 2;
      const float4 a = sb[j * J4 + r], c = sb[j * J4 + 4 + r];
      Hr[0] = a.x; Hi[0] = a.y; Hr[1] = a.z; Hi[1] = a.w;
      Hr[2] = c.x; Hi[2] = c.y; Hr[3] = c.z; Hi[3] = c.w;
    }
    MEGA_TR(8 + sc * 9);
    // ---- sweep 2: outputs
    load_q();
    char* ycol = xrow + j * G::SEGB;
#pragma unroll
    for (int i = 0; i < kSEGT; ++i) {
      const bf16x8 X = *(const bf16x8*)(xcol + i * 64);
      f32x4 S0 = {0.f, 0.f, 0.f, 0.f}, S1 = {0.f, 0.f, 0.f, 0.f};
      f32x4 Y0 = {0.f, 0.f, 0.f, 0.f}, Y1 = {0.f, 0.f, 0.f, 0.f};
      bf16x8 Hop;
      {
        const float hv[8] = {Hr[0], Hi[0], Hr[1], Hi[1], Hr[2], Hi[2], Hr[3], Hi[3]};
#pragma unroll
        for (int t = 0; t < 8; ++t) Hop[t] = (__bf16)hv[t];
      }
#pragma unroll
      for (int w = 0; w < kNWP; ++w) {
        S0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Pw[w][0], X, S0, 0, 0, 0);
        S1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Pw[w][1], X, S1, 0, 0, 0);
      }
#pragma unroll
      for (int w = 0; w < kNWC; ++w) {
        Y0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Cw[w][0], Hop, Y0, 0, 0, 0);
        Y1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Cw[w][1], Hop, Y1, 0, 0, 0);
      }
#pragma unroll
      for (int w = 0; w < kNWK; ++w) {
        Y0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Kw[w][0], X, Y0, 0, 0, 0);
        Y1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Kw[w][1], X, Y1, 0, 0, 0);
      }
      if (MEGA_TWO_ALWAYS || two_terms) {
        // the states can dwarf y and cancel in the sum over the states, so what bf16 drops of them is carried into
        // the product as a second term
        {
          const float hv[8] = {Hr[0], Hi[0], Hr[1], Hi[1], Hr[2], Hi[2], Hr[3], Hi[3]};
#pragma unroll
          for (int t = 0; t < 8; ++t) Hop[t] = (__bf16)(hv[t] - (float)Hop[t]);      // in place: no second register set
        }
#pragma unroll
        for (int w = 0; w < kNWC; ++w) {
          Y0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Cw[w][0], Hop, Y0, 0, 0, 0);
          Y1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(Cw[w][1], Hop, Y1, 0, 0, 0);
        }
      }
      const float sr[4] = {S0[0], S0[2], S1[0], S1[2]};
      const float si[4] = {S0[1], S0[3], S1[1], S1[3]};
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float nr = fmaf(Qr[u], Hr[u], fmaf(-Qi[u], Hi[u], sr[u]));
        const float ni = fmaf(Qr[u], Hi[u], fmaf(Qi[u], Hr[u], si[u]));
        Hr[u] = nr;
        Hi[u] = ni;
      }
      if (!FAST && A.h_tile && ch_ok) {
        const int gt = (t0 + j * G::SEG + i * 32) >> 5;
        if (gt == last_tile) {
          float* ho = A.h_tile + (((size_t)b * A.D + ch) * kNS) * 2;
          const int nn[4] = {2 * r, 2 * r + 1, 8 + 2 * r, 9 + 2 * r};
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            ho[nn[u] * 2] = Hr[u];
            ho[nn[u] * 2 + 1] = Hi[u];
          }
        }
      }
      // y (bf16) overwrites x in place: tokens 32 i + 16 mb + 4 r + {0..3} of segment j
      {
        bf16_t o0[4], o1[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          o0[u] = from_float<bf16_t>(Y0[u]);
          o1[u] = from_float<bf16_t>(Y1[u]);
        }
        *(uint2*)(ycol + i * 64 + r * 8) = *(const uint2*)o0;
        *(uint2*)(ycol + i * 64 + 32 + r * 8) = *(const uint2*)o1;
      }
    }
    MEGA_TR(9 + sc * 9);
    if (LOUT == 1) __syncthreads();      // the channel-contiguous store reads every wave's row; a
                                         // time-contiguous one only the wave's own
    MEGA_TR(10 + sc * 9);
    // ---- store the super-chunk
    bf16_t* yg = (bf16_t*)A.y;
#pragma unroll
    for (int k = 0; k < NLD; ++k) {
      if (LOUT == 1) {
        const int tk = k * (kThreadsM / 2) + (tid >> 1);
        const int tau = t0 + tk;
        const int c0 = cb * kWaves + half * 8;
        // four dwords (even token | odd token << 16) of channels half*8 + odd*4 + {0..3}
        const char* base = smem + (half * 8 + odd * 4) * G::ROWB + G::pos(tk & ~1);
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = *(const uint32_t*)(base + e * G::ROWB);
        // my token's halves of my four channels stay, the partner token's halves go to the partner
        const uint32_t keep0 = __builtin_amdgcn_perm(w[1], w[0], sel_keep);
        const uint32_t keep1 = __builtin_amdgcn_perm(w[3], w[2], sel_keep);
        const uint32_t got0 = dpp_swap2(__builtin_amdgcn_perm(w[1], w[0], sel_give));
        const uint32_t got1 = dpp_swap2(__builtin_amdgcn_perm(w[3], w[2], sel_give));
        uint4 o;     // channels c0 .. c0+7 of token tk
        o.x = odd ? got0 : keep0;
        o.y = odd ? got1 : keep1;
        o.z = odd ? keep0 : got0;
        o.w = odd ? keep1 : got1;
        if (FAST) {
          const int t = A.reverse ? A.L - 1 - tau : tau;
          *(uint4*)(yg + b * A.syb + (int64_t)t * A.syl + c0) = o;
        } else if (tau < A.L && c0 < A.D) {
          const int t = A.reverse ? A.L - 1 - tau : tau;
          const bool direct = !A.acc_in && !A.acc_out && !(A.mask && A.omega);
          if (direct) {
            *(uint4*)(yg + b * A.syb + (int64_t)t * A.syl + c0) = o;
          } else {
            float v[8];
            const uint32_t* oo = (const uint32_t*)&o;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = __uint_as_float((e & 1) ? (oo[e >> 1] & 0xffff0000u) : (oo[e >> 1] << 16));
            if (A.acc_in) {
              const float* ai = A.acc_in + b * A.sab + (int64_t)t * A.sal + c0;
#pragma unroll
              for (int e = 0; e < 8; ++e) v[e] += ai[e];
            }
            if (A.mask && A.omega && A.mask[(size_t)b * A.L + t]) {
              // the residual uses the unmasked input (base_moving_average.py:138)
              const bf16_t* xo = xg + b * A.sxb + (int64_t)t * A.sxl + (int64_t)c0 * A.sxd;
#pragma unroll
              for (int e = 0; e < 8; ++e) v[e] += A.omega[c0 + e] * to_float(xo[e * A.sxd]);
            }
            if (A.acc_out) {
              float* ao = A.acc_out + b * A.sab + (int64_t)t * A.sal + c0;
#pragma unroll
              for (int e = 0; e < 8; ++e) ao[e] = v[e];
            } else {
              Vec<bf16_t, 8> ov;
#pragma unroll
              for (int e = 0; e < 8; ++e) ov.v[e] = from_float<bf16_t>(v[e]);
              *(Vec<bf16_t, 8>*)(yg + b * A.syb + (int64_t)t * A.syl + c0) = ov;
            }
          }
        }
      } else {
        const int tk = k * 512 + lane * 8;
        const int tau = t0 + tk;
        if (FAST) {
          const int t = A.reverse ? A.L - 8 - tau : tau;
          uint4 v = *(const uint4*)(xrow + G::pos(tk));
          if (A.reverse) {
            uint4 w;
            w.x = (v.w >> 16) | (v.w << 16);
            w.y = (v.z >> 16) | (v.z << 16);
            w.z = (v.y >> 16) | (v.y << 16);
            w.w = (v.x >> 16) | (v.x << 16);
            v = w;
          }
          *(uint4*)(yg + b * A.syb + (int64_t)ch * A.syd + t) = v;
        } else if (tau < A.L && ch_ok) {
          const int t = A.reverse ? A.L - 8 - tau : tau;       // first physical token of the 8
          Vec<bf16_t, 8> in = *(const Vec<bf16_t, 8>*)(xrow + G::pos(tk));
          float v[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = to_float(in.v[A.reverse ? 7 - e : e]);   // physical order
          if (A.acc_in) {
            const float* ai = A.acc_in + b * A.sab + (int64_t)ch * A.sad + t;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] += ai[e];
          }
          if (A.mask && A.omega) {
            const uint8_t* mk = A.mask + (size_t)b * A.L + t;
            const bf16_t* xo = xg + b * A.sxb + (int64_t)ch * A.sxd + (int64_t)t * A.sxl;
            const float om = A.omega[ch];
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (mk[e]) v[e] += om * to_float(xo[e * A.sxl]);
          }
          if (A.acc_out) {
            float* ao = A.acc_out + b * A.sab + (int64_t)ch * A.sad + t;
#pragma unroll
            for (int e = 0; e < 8; ++e) ao[e] = v[e];
          } else {
            Vec<bf16_t, 8> o;
#pragma unroll
            for (int e = 0; e < 8; ++e) o.v[e] = from_float<bf16_t>(v[e]);
            *(Vec<bf16_t, 8>*)(yg + b * A.syb + (int64_t)ch * A.syd + t) = o;
          }
        }
      }
    }
    MEGA_TR(11 + sc * 9);
    __syncthreads();
  };
  if (DEPTH == 2) {
    for (int sc = 0; sc < nsc; sc += 2) {
      body(sc, preA);
      body(sc + 1, preB);
    }
  } else {
    for (int sc = 0; sc < nsc; ++sc) body(sc, preA);
  }
  MEGA_TR(3 + nsc * 9);
  MEGA_TR_FLUSH();
  if (FAST && A.h_tile && (lane & 3) == 0) {
    // L is a whole number of super-chunks: the carried scan state is the state at time L
    float* ho = A.h_tile + (((size_t)b * A.D + ch) * kNS + (lane >> 2)) * 2;
    ho[0] = Hcr;
    ho[1] = Hci;
  }
}

// Finishes the carried state: from the state after the last whole tile (time Lb = 32 floor(L/32))
// to time L: h = q^r h_tile + sum_{i<r} p q^{r-1-i} x[Lb + i], r = L - Lb < 32.
template <typename T>
__global__ void ema_state_tail_kernel(const T* __restrict__ x, int64_t sxb, int64_t sxd, int64_t sxl,
                                      const uint8_t* __restrict__ mask, const float* __restrict__ p,
                                      const float* __restrict__ q, const float* __restrict__ h_tile,
                                      float* __restrict__ h_out, int B, int D, int N, int L, int is_complex) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (int64_t)B * D * N) return;
  const int n = (int)(gid % N);
  const int d = (int)((gid / N) % D);
  const int b = (int)(gid / ((int64_t)N * D));
  const float qr = q[((size_t)d * N + n) * 2], qi = is_complex ? q[((size_t)d * N + n) * 2 + 1] : 0.f;
  const float pv = p[(size_t)d * N + n];
  const float* ht = h_tile + (((size_t)b * D + d) * kNS + n) * 2;
  float hr = ht[0], hi = ht[1];
  const int Lb = (L / 32) * 32;
  for (int t = Lb; t < L; ++t) {
    float u = 0.f;
    if (!(mask && mask[(size_t)b * L + t])) u = to_float(x[b * sxb + d * sxd + t * sxl]);
    const float nr = qr * hr - qi * hi + pv * u;
    const float ni = qr * hi + qi * hr;
    hr = nr;
    hi = ni;
  }
  float* ho = h_out + (((size_t)b * D + d) * N + n) * 2;
  ho[0] = hr;
  ho[1] = hi;
}

}  // namespace

// Memory layout of one side of the call: 1 = channels contiguous (16-byte pieces of 8 channels),
// 0 = time contiguous (pieces of 8 tokens), -1 = neither (the generic path takes it).
static int side_layout(int64_t sb, int64_t sd, int64_t sl, int64_t D, int64_t L) {
  if (sd == 1 && D % 8 == 0 && sl % 8 == 0 && sb % 8 == 0) return 1;
  if (sl == 1 && L % 8 == 0 && sd % 8 == 0 && sb % 8 == 0) return 0;
  return -1;
}

size_t ema_image_bytes(int64_t D, int64_t N, int bidirectional) {
  if (N > kNS || D <= 0) return 0;
  return (size_t)(bidirectional ? 2 * D : D) * kImgRowBytes;
}

int ema_image_build(const float* p, const float* q, const float* gamma, int is_complex, const float* omega, int64_t D,
                    int64_t N, int bidirectional, int shift, void* image, hipStream_t s, int parts) {
  ImageArgs A;
  A.parts = parts;
  A.p = p; A.q = q; A.gamma = gamma; A.omega = omega; A.image = (uint4*)image;
  A.K = (int)(bidirectional ? 2 * D : D); A.D = (int)D; A.N = (int)N; A.is_complex = is_complex;
  A.lag_back = shift ? 1 : 0;
  hipLaunchKernelGGL(ema_image_kernel, dim3((unsigned)A.K), dim3(kPrepWaves * 64), 0, s, A);
  MEGA_CHECK_LAUNCH("ema kernel generation");
  return MEGA_OK;
}

// Host side: decides whether the matrix-core path covers a request and launches it.
// Returns 1 if handled, 0 if the caller must use the generic path, < 0 on a launch error.
int ema_mfma_try(const void* x, void* y, int dtype, int64_t sxb, int64_t sxd, int64_t sxl, int64_t syb,
                 int64_t syd, int64_t syl, const float* p, const float* q, const void* image, int is_complex,
                 const float* omega, const uint8_t* mask, const float* h_in, float* h_out, int64_t B, int64_t D,
                 int64_t N, int64_t L, int bidirectional, int64_t Lk, float* acc, float* h_tile, hipStream_t s) {
  if (!ema_mfma_covers(dtype, sxb, sxd, sxl, syb, syd, syl, x, y, mask, B, D, N, L, Lk)) return 0;
  const int lin = side_layout(sxb, sxd, sxl, D, L), lout = side_layout(syb, syd, syl, D, L);
  using G = Geo;
  const int ncb = (int)ceil_div(D, kWaves);
  MfmaArgs A;
  A.x = x; A.y = y; A.sxb = sxb; A.sxd = sxd; A.sxl = sxl; A.syb = syb; A.syd = syd; A.syl = syl;
  A.image = (const uint4*)image; A.mask = mask;
  A.B = (int)B; A.D = (int)D; A.N = (int)N; A.L = (int)L; A.is_complex = is_complex;
  A.xcd_map = ((lin == 1 || lout == 1) && ncb % 4 == 0 && ((B * ncb) % 32) == 0) ? 1 : 0;
  // fp32 partial sums between the two directions live in [B, D, L]-shaped storage with y's layout
  A.sab = lout == 1 ? L * D : D * L;
  A.sad = lout == 1 ? 1 : L;
  A.sal = lout == 1 ? D : 1;
  const dim3 grid((unsigned)(B * ncb));
  const bool fast = !bidirectional && !mask && L % G::SC == 0 && D % kWaves == 0;
  auto launch = [&](const MfmaArgs& a) -> int {
    typedef void (*Kern)(const MfmaArgs);
    static const Kern table[12] = {
        ema_mfma_kernel<0, 0, 0>, ema_mfma_kernel<0, 0, 1>, ema_mfma_kernel<0, 0, 2>,
        ema_mfma_kernel<0, 1, 0>, ema_mfma_kernel<0, 1, 1>, ema_mfma_kernel<0, 1, 2>,
        ema_mfma_kernel<1, 0, 0>, ema_mfma_kernel<1, 0, 1>, ema_mfma_kernel<1, 0, 2>,
        ema_mfma_kernel<1, 1, 0>, ema_mfma_kernel<1, 1, 1>, ema_mfma_kernel<1, 1, 2>};
    static uint64_t attr_seen[12] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const int mode = fast ? ((L / G::SC) % 2 == 0 ? 2 : 1) : 0;
    const int ki = (lin * 2 + lout) * 3 + mode;
    const Kern kern = table[ki];
    if (first_on_device(&attr_seen[ki])) {
      (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, G::TOTAL);
    }
    hipLaunchKernelGGL(kern, grid, dim3(kThreadsM), G::TOTAL, s, a);
    MEGA_CHECK_LAUNCH("ema_fwd (matrix-core path)");
    return MEGA_OK;
  };
  if (bidirectional) {
    MfmaArgs Bk = A;
    Bk.koff = (int)D; Bk.reverse = 1;
    Bk.omega = nullptr; Bk.h_in = nullptr; Bk.h_tile = nullptr; Bk.acc_in = nullptr; Bk.acc_out = acc;
    int rc = launch(Bk);
    if (rc) return rc;
  }
  A.koff = 0; A.reverse = 0; A.omega = omega; A.h_in = h_in;
  A.h_tile = h_out ? h_tile : nullptr;
  A.acc_in = bidirectional ? acc : nullptr; A.acc_out = nullptr;
  int rc = launch(A);
  if (rc) return rc;
  if (h_out) {
    const int64_t n = B * D * N;
    hipLaunchKernelGGL(ema_state_tail_kernel<bf16_t>, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s,
                       (const bf16_t*)x, sxb, sxd, sxl, mask, p, q, h_tile, h_out, (int)B, (int)D, (int)N, (int)L,
                       is_complex);
    MEGA_CHECK_LAUNCH("ema_fwd state tail");
  }
  return 1;
}

bool ema_mfma_covers(int dtype, int64_t sxb, int64_t sxd, int64_t sxl, int64_t syb, int64_t syd, int64_t syl,
                     const void* x, const void* y, const uint8_t* mask, int64_t B, int64_t D, int64_t N, int64_t L,
                     int64_t Lk) {
  if (dtype != MEGA_BF16 || N > kNS || Lk > 0 || L < 256) return false;
  const int lin = side_layout(sxb, sxd, sxl, D, L), lout = side_layout(syb, syd, syl, D, L);
  if (lin < 0 || lout < 0) return false;
  if (((uintptr_t)x % 16) || ((uintptr_t)y % 16) || (mask && lin == 0 && ((uintptr_t)mask % 8))) return false;
  if (B * ceil_div(D, kWaves) >= (int64_t)1 << 31) return false;
  return true;
}

}  // namespace mega
