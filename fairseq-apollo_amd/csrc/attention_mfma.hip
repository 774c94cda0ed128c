// Attention on the matrix cores: y = softmax_causal(scale q k^T) v per (batch, head)
// (fairseq/csrc/ops/attention_kernel.cu:40-131), 16-bit activations.
//
//   S = scale q k^T        batched NT GEMM, v_mfma_f32_16x16x32_{bf16,f16}, fp32 out; causal: tiles
//                          above the diagonal are skipped
//   P = softmax_causal(S)  one workgroup per row, fp32 in, 16-bit out (right-aligned mask, a fully
//                          masked row gives zeros: fairseq/csrc/softmax.cuh:90-153)
//   y = P v                the same kernel with v read in place as a K-major operand (its tile goes to LDS as it
//                          lies in memory, the fragments come out of transposing LDS reads); causal: the
//                          reduction stops at the diagonal.  v rows that are not whole 16-byte pieces go
//                          through a transposed copy instead
//
// Backward (fairseq/csrc/ops/attention_kernel.cu:133-255), with the forward's weights w:
//   dW = dy v^T            fp32 out; causal: tiles above the diagonal are skipped
//   dS = scale w (dW - rowsum(w dW))       one wave per row, zeros behind the causal limit
//   dv = w^T dy, dk = dS^T q               both operands K-major (w, dS, dy, q read in place); causal: the
//                                          reduction starts at the diagonal, long row tiles first
//   dq = dS k                              k K-major; causal: the reduction stops at the diagonal
//   (rows of w that are not whole 16-byte pieces: transposed, zero-padded copies of w, dS, dy, q, k instead)
//
// The GEMM: (64 WM) x (64 WN) output tile per workgroup of WM x WN waves (64 x 64 each as 4 x 4 MFMA
// blocks): 128 x 128 for the scores, 256 x 256 for the second product, which carries the flops.
// K step 64, operands staged through LDS as dense 128-byte rows with XOR-swizzled 16-byte pieces (no bank
// conflicts), register prefetch of the next K step, all tiles of one batch entry on one XCD, epilogue through LDS.
#include "common.h"

namespace mega {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int BM = 128, BN = 128, BK = 64;      // BM: block size of the causal bookkeeping and the small tile
#ifndef MEGA_GEMM_SWZ
#define MEGA_GEMM_SWZ 1
#endif
// bytes per LDS row of BK 16-bit elements: dense rows whose 16-byte pieces are XOR-swizzled by the row
// (piece c of row r sits at c ^ ((r >> 1) & 7): the 16 rows a fragment read touches cover every bank once)
constexpr int PITCH = MEGA_GEMM_SWZ ? BK * 2 : BK * 2 + 16;
__device__ __forceinline__ int lds_piece(int row, int piece) { return MEGA_GEMM_SWZ ? (piece ^ ((row >> 1) & 7)) : piece; }
constexpr int KP = BK / 8;                // 16-byte pieces per operand row and K step

struct GemmArgs {
  const void* A;      // [batch][M][K] rows with pitch lda (elements), batch stride sa
  const void* Bm;     // [batch][N][K] rows with pitch ldb, batch stride sb
  void* C;            // [batch][M][N] pitch ldc, batch stride sc
  int64_t lda, ldb, ldc, sa, sb, sc;
  // batch index = bo * nin + bi; per operand the address is base + bo * s?o + bi * s?i
  int64_t sai, sbi, sci;
  int nin;
  int M, N, K;
  float alpha;
  int causal;         // 1: S = q k^T (skip tiles with n0 > m0 + BM - 1); 2: y = P v (K stops at m0 + BM);
                      // 3: y = P^T v (row m of the product is column m of P: K starts at m0)
  int kshift;         // causal offset: row m (of P) sees columns <= m + kshift
  // xcd != 0: one-dimensional grid; every tile of a batch entry runs on one XCD (workgroup ids go
  // round-robin over the 8 XCDs), so both operands of a batch entry are fetched into one L2 only;
  // the long row tiles of a causal product come first
  int xcd, mt, nt;
  // softmax-backward epilogue (EPI = 1): C holds elements of the input type, C[m][n] = alpha E[m][n] (acc - rowdot[m])
  // with zeros behind the causal limit; E has C's batch layout with pitch lde and strides se / sei, rowdot is
  // [batch][M] fp32
  const void* E = nullptr;
  const float* rowdot = nullptr;
  int64_t lde = 0, se = 0, sei = 0;
};

template <typename T>
__device__ __forceinline__ f32x4 mfma16(uint4 a, uint4 b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mfma16<bf16_t>(uint4 a, uint4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mfma16<f16_t>(uint4 a, uint4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// A K-major operand tile in LDS (an operand that enters the product through its columns: BK rows of W 16-bit elements,
// row k = the W values the tile's rows / columns have at reduction index k): dense rows whose 32-byte spans are
// XOR-swizzled by the row, so that the transposing fragment reads (ds_read_b64_tr_b16: four rows, four 8-byte columns
// per group of 16 lanes) fall on different banks.  The XOR touches the low three bits of the span index only.
__device__ __forceinline__ int kmajor_piece(int row, int piece) {
  const int vs = (row & 3) + 4 * ((row >> 3) & 1);
  return (((piece >> 1) ^ vs) << 1) | (piece & 1);
}
// the MFMA operand fragment (16 rows or columns x 32 reduction indices) of a K-major tile: lane (n, g) ends up with
// the eight consecutive reduction indices 8 g .. 8 g + 7 of tile column 16 span + n.  base = tile + the lane's part
// (kmajor_lane), rowbytes = 2 W
__device__ __forceinline__ uint4 kmajor_frag(const char* base, int rowbytes, int span, int vsw) {
  typedef __attribute__((ext_vector_type(4))) short s4v;
  const char* q0 = base + (((span & 7) ^ vsw) * 32) + (span >> 3) * 256;
  const s4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*)(q0));
  const s4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*)(q0 + 4 * rowbytes));
  const uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
  return make_uint4(l2.x, l2.y, h2.x, h2.y);
}

// C = alpha A B^T; TIn 16-bit, TOut float or TIn.  WM x WN waves, each a 64 x 64 block of the
// (64 WM) x (64 WN) output tile.  The operand traffic from L2 per flop falls with the tile edge:
// 2 x 2 waves (128 x 128) need 1/64 byte per flop, 4 x 4 waves (256 x 256) half of that.
// AT / BT: the operand is stored K-major, [K][M] with pitch lda / [K][N] with pitch ldb (C = A^T-stored ... : the
// product reduces over the operand's rows), and is read in place: its tile goes to LDS as it lies in memory and the
// fragments come out of transposing LDS reads.  M (N) must be a multiple of 8 then.
template <typename TIn, typename TOut, int WM, int WN, bool AT = false, bool BT = false, int EPI = 0, int FM = 4,
          int FN = FM>
__global__ __launch_bounds__(64 * WM * WN) void gemm_nt_kernel(const GemmArgs G) {
  static_assert(EPI == 0 || sizeof(TOut) == 4, "the softmax-backward epilogue stages fp32");
  constexpr int WTM = 16 * FM, WTN = 16 * FN;                     // a wave's block of the output tile
  constexpr int TM = WTM * WM, TN = WTN * WN, NT = 64 * WM * WN;
  constexpr int NLA = TM * KP / NT, NLB = TN * KP / NT;          // 16-byte pieces per thread and K step
  static_assert(TM * KP % NT == 0 && TN * KP % NT == 0, "tile rows must divide over the threads");
  extern __shared__ __attribute__((aligned(16))) char lds[];     // 2 x (TM + TN) x PITCH
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int m0, n0, bz;
  if (G.xcd) {
    int rest = (int)blockIdx.x >> 3;
    const int ntile = rest % G.nt;
    rest /= G.nt;
    // the long row tiles first: the late rows of a causal product, the early ones when the reduction starts at
    // the diagonal (mode 3)
    const int mtile = G.causal == 3 ? rest % G.mt : G.mt - 1 - rest % G.mt;
    rest /= G.mt;
    bz = rest * 8 + ((int)blockIdx.x & 7);
    m0 = mtile * TM;
    n0 = ntile * TN;
  } else {
    m0 = blockIdx.y * TM;
    n0 = blockIdx.x * TN;
    bz = blockIdx.z;
  }
  if (G.causal == 1 && n0 > m0 + TM - 1 + G.kshift) return;      // entirely above the diagonal
  const int bo = bz / G.nin, bi = bz - bo * G.nin;
  const TIn* A = (const TIn*)G.A + bo * G.sa + bi * G.sai;
  const TIn* Bm = (const TIn*)G.Bm + bo * G.sb + bi * G.sbi;
  TOut* C = (TOut*)G.C + bo * G.sc + bi * G.sci;     // EPI = 1: unused, the result goes out as TIn (below)
  int Kend = G.K;
  if (G.causal == 2) Kend = min(G.K, m0 + TM + G.kshift);
  if (Kend < 0) Kend = 0;
  const int nk = (Kend + BK - 1) / BK;
  const int kt0 = G.causal == 3 ? max(0, m0 - G.kshift) / BK : 0;      // first K step that can hold a non-zero

  // global -> register staging: a wave-uniform tile pointer plus a 32-bit byte offset per lane and piece
  const int lrow = tid / KP, lcol = (tid % KP) * 8;              // rows 0 .. NT/KP - 1 (+ h * NT/KP)
  uint4 ra[NLA], rb[NLB];
  uint32_t offa[NLA], offb[NLB];
  int kra[NLA], krb[NLB];                                        // K-major: the piece's row of the K step
  bool oka[NLA], okb[NLB];                                       // the piece's row / column lies inside the matrix
#pragma unroll
  for (int h = 0; h < NLA; ++h) {
    if (AT) {
      const int pi = tid + h * NT;
      kra[h] = pi / (TM / 8);
      const int mc = (pi % (TM / 8)) * 8;
      oka[h] = m0 + mc < G.M;
      offa[h] = (uint32_t)(((int64_t)kra[h] * G.lda + mc) * 2);
    } else {
      const int r = lrow + h * (NT / KP);
      kra[h] = 0;
      oka[h] = m0 + r < G.M;
      offa[h] = (uint32_t)(((int64_t)r * G.lda + lcol) * 2);
    }
  }
#pragma unroll
  for (int h = 0; h < NLB; ++h) {
    if (BT) {
      const int pi = tid + h * NT;
      krb[h] = pi / (TN / 8);
      const int nc = (pi % (TN / 8)) * 8;
      okb[h] = n0 + nc < G.N;
      offb[h] = (uint32_t)(((int64_t)krb[h] * G.ldb + nc) * 2);
    } else {
      const int r = lrow + h * (NT / KP);
      krb[h] = 0;
      okb[h] = n0 + r < G.N;
      offb[h] = (uint32_t)(((int64_t)r * G.ldb + lcol) * 2);
    }
  }
  auto gload = [&](int kt) {
    const int k = kt * BK + lcol;
    // tile origin of this K step: row m0 / n0 at column kt BK, or (K-major) row kt BK at column m0 / n0
    const char* Au = (const char*)(AT ? A + (int64_t)kt * BK * G.lda + m0 : A + (int64_t)m0 * G.lda + kt * BK);
    const char* Bu = (const char*)(BT ? Bm + (int64_t)kt * BK * G.ldb + n0 : Bm + (int64_t)n0 * G.ldb + kt * BK);
#pragma unroll
    for (int h = 0; h < NLA; ++h) {
      ra[h] = make_uint4(0, 0, 0, 0);
      if (oka[h] && (AT ? kt * BK + kra[h] < Kend : k < Kend)) ra[h] = *(const uint4*)(Au + offa[h]);
    }
#pragma unroll
    for (int h = 0; h < NLB; ++h) {
      rb[h] = make_uint4(0, 0, 0, 0);
      if (okb[h] && (BT ? kt * BK + krb[h] < Kend : k < Kend)) rb[h] = *(const uint4*)(Bu + offb[h]);
    }
  };
  auto lstore = [&](int buf) {
    char* la = lds + buf * (TM + TN) * PITCH;
    char* lb = la + TM * PITCH;
#pragma unroll
    for (int h = 0; h < NLA; ++h) {
      if (AT) {
        const int pi = tid + h * NT, kr = pi / (TM / 8), mp = pi % (TM / 8);
        *(uint4*)(la + kr * (TM * 2) + kmajor_piece(kr, mp) * 16) = ra[h];
      } else {
        const int r = lrow + h * (NT / KP);
        *(uint4*)(la + r * PITCH + lds_piece(r, tid % KP) * 16) = ra[h];
      }
    }
#pragma unroll
    for (int h = 0; h < NLB; ++h) {
      if (BT) {
        const int pi = tid + h * NT, kr = pi / (TN / 8), np = pi % (TN / 8);
        *(uint4*)(lb + kr * (TN * 2) + kmajor_piece(kr, np) * 16) = rb[h];
      } else {
        const int r = lrow + h * (NT / KP);
        *(uint4*)(lb + r * PITCH + lds_piece(r, tid % KP) * 16) = rb[h];
      }
    }
  };
  f32x4 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int wm = (wave / WN) * WTM, wn = (wave % WN) * WTN;
  const int fr = lane & 15;                                       // fragment row; lane >> 4 is its 16-byte k block
  // the lane's part of a K-major fragment address: row 8 g + (n >> 2) of the 32-row block, 8-byte column n & 3
  const int ksr = fr >> 2, kvsw = ksr + 4 * ((lane >> 4) & 1);
  const int klane_a = (8 * (lane >> 4) + ksr) * (TM * 2) + (fr & 3) * 8;
  const int klane_b = (8 * (lane >> 4) + ksr) * (TN * 2) + (fr & 3) * 8;
  static_assert(!(AT || BT) || PITCH == BK * 2, "a K-major tile takes the room of its row-major form");
  static_assert(!AT || TM == 128 || TM == 256, "a K-major tile row is 256 or 512 bytes");
  static_assert(!BT || TN == 128 || TN == 256, "a K-major tile row is 256 or 512 bytes");

  if (nk > kt0) {
    gload(kt0);
    lstore(0);
  }
  __syncthreads();
  for (int kt = kt0; kt < nk; ++kt) {
    const int buf = (kt - kt0) & 1;
    if (kt + 1 < nk) gload(kt + 1);
    const char* la = lds + buf * (TM + TN) * PITCH;
    const char* lb = la + TM * PITCH;
#pragma unroll
    for (int kk = 0; kk < BK / 32; ++kk) {
      uint4 fa[FM];
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        if (AT)
          fa[i] = kmajor_frag(la + kk * 32 * (TM * 2) + klane_a, TM * 2, (wm >> 4) + i, kvsw);
        else
          fa[i] = *(const uint4*)(la + (wm + i * 16 + fr) * PITCH + lds_piece(wm + i * 16 + fr, kk * 4 + (lane >> 4)) * 16);
      }
      // the B fragments one column block at a time (four at once do not fit the 128 registers of a 16-wave
      // workgroup next to the K-major address arithmetic)
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        uint4 fb;
        if (BT)
          fb = kmajor_frag(lb + kk * 32 * (TN * 2) + klane_b, TN * 2, (wn >> 4) + j, kvsw);
        else
          fb = *(const uint4*)(lb + (wn + j * 16 + fr) * PITCH + lds_piece(wn + j * 16 + fr, kk * 4 + (lane >> 4)) * 16);
#pragma unroll
        for (int i = 0; i < FM; ++i) acc[i][j] = mfma16<TIn>(fa[i], fb, acc[i][j]);
        // K-major forms: keep the compiler from fetching all four B fragments ahead (that spills in the loop)
        if ((AT || BT) && WM * WN == 16 && (j & 1)) __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (kt + 1 < nk) lstore(buf ^ 1);
    __syncthreads();
  }
  // D layout: column = lane & 15, rows 4 (lane >> 4) + {0..3}
  const int cn = lane & 15, cr = (lane >> 4) * 4;
  constexpr int VW = 16 / (int)sizeof(TOut);                     // elements per 16-byte piece
  constexpr int CP = TN + VW;                                    // row pitch of the staged tile in elements
  // the tile leaves through LDS (the operand buffers are free after the last barrier) as 16-byte pieces, TN *
  // sizeof(TOut) contiguous bytes per row: whole, or in NH slices of rows when it is larger than the operand buffers
  constexpr size_t lds_bytes = (size_t)2 * (TM + TN) * PITCH;
  constexpr size_t tile_bytes = (size_t)TM * CP * sizeof(TOut);
  constexpr int NH = tile_bytes <= lds_bytes ? 1 : tile_bytes / 2 <= lds_bytes ? 2 : (tile_bytes / 4 <= lds_bytes && TM >= 256) ? 4 : 0;
  if constexpr (EPI == 1) {
    TIn* D = (TIn*)G.C + bo * G.sc + bi * G.sci;
    const TIn* Ep = (const TIn*)G.E + bo * G.se + bi * G.sei;
    const float* rd = G.rowdot + (int64_t)bz * G.M;
    auto value = [&](float a, float e, float rdv, int m, int n) {
      return (!G.causal || n <= m + G.kshift) ? G.alpha * e * (a - rdv) : 0.f;
    };
    const bool wide4 = NH > 0 && (G.ldc % 4) == 0 && (G.lde % 4) == 0 && ((((uintptr_t)D) | ((uintptr_t)Ep)) % 8) == 0 &&
                       n0 + TN <= G.N;
    if (NH > 0 && wide4) {
      constexpr int HR = TM / (NH > 0 ? NH : 1);
      float* Cs = (float*)lds;
#pragma unroll
      for (int h = 0; h < NH; ++h) {
        if (h > 0) __syncthreads();
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          if ((wm + i * 16) / HR != h) continue;                 // this block of rows belongs to another slice
#pragma unroll
          for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int u = 0; u < 4; ++u) Cs[(wm - h * HR + i * 16 + cr + u) * CP + wn + j * 16 + cn] = acc[i][j][u];
        }
        __syncthreads();
        constexpr int PPR = TN / 4;
#pragma unroll
        for (int u = 0; u < HR * PPR / NT; ++u) {
          const int pi = tid + u * NT;
          const int r = pi / PPR, pc = pi - r * PPR;
          const int m = m0 + h * HR + r, n = n0 + pc * 4;
          if (m < G.M) {
            const float4 a = *(const float4*)(Cs + r * CP + pc * 4);
            const Vec<TIn, 4> e = *(const Vec<TIn, 4>*)(Ep + (int64_t)m * G.lde + n);
            const float rdv = rd[m];
            Vec<TIn, 4> o;
            o.v[0] = from_float<TIn>(value(a.x, to_float(e.v[0]), rdv, m, n));
            o.v[1] = from_float<TIn>(value(a.y, to_float(e.v[1]), rdv, m, n + 1));
            o.v[2] = from_float<TIn>(value(a.z, to_float(e.v[2]), rdv, m, n + 2));
            o.v[3] = from_float<TIn>(value(a.w, to_float(e.v[3]), rdv, m, n + 3));
            *(Vec<TIn, 4>*)(D + (int64_t)m * G.ldc + n) = o;
          }
        }
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int n = n0 + wn + j * 16 + cn;
        if (n >= G.N) continue;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int m = m0 + wm + i * 16 + cr + u;
          if (m < G.M)
            D[(int64_t)m * G.ldc + n] =
                from_float<TIn>(value(acc[i][j][u], to_float(Ep[(int64_t)m * G.lde + n]), rd[m], m, n));
        }
      }
    return;
  }
  const bool wide = NH > 0 && (G.ldc % VW) == 0 && (((uintptr_t)C) % 16) == 0 && n0 + TN <= G.N;
  if (NH > 0 && wide) {
    constexpr int HR = TM / (NH > 0 ? NH : 1);                   // rows per slice (a multiple of 16)
    TOut* Cs = (TOut*)lds;
#pragma unroll
    for (int h = 0; h < NH; ++h) {
      if (h > 0) __syncthreads();                                // the previous slice has left
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        if ((wm + i * 16) / HR != h) continue;                   // this block of rows belongs to another slice
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int u = 0; u < 4; ++u)
            Cs[(wm - h * HR + i * 16 + cr + u) * CP + wn + j * 16 + cn] = from_float<TOut>(acc[i][j][u] * G.alpha);
      }
      __syncthreads();
      constexpr int PPR = TN / VW;                               // pieces per row
#pragma unroll
      for (int u = 0; u < HR * PPR / NT; ++u) {
        const int pi = tid + u * NT;
        const int r = pi / PPR, pc = pi - r * PPR;
        if (m0 + h * HR + r < G.M)
          *(uint4*)(C + (int64_t)(m0 + h * HR + r) * G.ldc + n0 + pc * VW) = *(const uint4*)(Cs + r * CP + pc * VW);
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const int n = n0 + wn + j * 16 + cn;
      if (n >= G.N) continue;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int m = m0 + wm + i * 16 + cr + u;
        if (m < G.M) C[(int64_t)m * G.ldc + n] = from_float<TOut>(acc[i][j][u] * G.alpha);
      }
    }
}

template <typename TIn, typename TOut, int WM, int WN, bool AT = false, bool BT = false, int EPI = 0, int FM = 4,
          int FN = FM>
void launch_gemm(GemmArgs G, int64_t M, int64_t N, int64_t batches, bool xcd, hipStream_t s) {
  constexpr int TM = 16 * FM * WM, TN = 16 * FN * WN;
  constexpr int smem = 2 * (TM + TN) * PITCH;
  auto kern = gemm_nt_kernel<TIn, TOut, WM, WN, AT, BT, EPI, FM, FN>;
  static uint64_t attr_seen = 0;
  if (smem > 64 * 1024 && first_on_device(&attr_seen)) {
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
  }
  if (audit_on()) {
    // the last element each operand is addressed at, from the kernel's own indexing: 16-byte pieces whose first
    // element passes the bounds test, rows below M / N, reduction steps below K; batch bz = bo nin + bi
    const int64_t bo = (batches - 1) / G.nin, bi = batches - 1 < G.nin ? batches - 1 : G.nin - 1;
    auto pieces = [](int64_t n) { return (n - 1) / 8 * 8 + 8; };
    const size_t a_el = AT ? (size_t)((G.K - 1) * G.lda + pieces(G.M)) : (size_t)((G.M - 1) * G.lda + pieces(G.K));
    const size_t b_el = BT ? (size_t)((G.K - 1) * G.ldb + pieces(G.N)) : (size_t)((G.N - 1) * G.ldb + pieces(G.K));
    const size_t c_el = (size_t)((G.M - 1) * G.ldc + G.N);
    audit_use((const TIn*)G.A + bo * G.sa + bi * G.sai, a_el * sizeof(TIn), "gemm operand A");
    audit_use((const TIn*)G.A, 1, "gemm operand A (first batch)");
    audit_use((const TIn*)G.Bm + bo * G.sb + bi * G.sbi, b_el * sizeof(TIn), "gemm operand B");
    audit_use((const TIn*)G.Bm, 1, "gemm operand B (first batch)");
    if (EPI == 1) {
      audit_use((TIn*)G.C + bo * G.sc + bi * G.sci, c_el * sizeof(TIn), "gemm result (softmax-backward epilogue)");
      audit_use((const TIn*)G.E + bo * G.se + bi * G.sei, (size_t)((G.M - 1) * G.lde + G.N) * sizeof(TIn),
                "gemm epilogue operand E");
      audit_use(G.rowdot, (size_t)batches * G.M * 4, "gemm epilogue row sums");
    } else {
      audit_use((TOut*)G.C + bo * G.sc + bi * G.sci, c_el * sizeof(TOut), "gemm result");
    }
    return;
  }
  G.xcd = xcd ? 1 : 0;
  G.mt = (int)ceil_div(M, TM);
  G.nt = (int)ceil_div(N, TN);
  const dim3 grid3((unsigned)G.nt, (unsigned)G.mt, (unsigned)batches);
  const dim3 grid1((unsigned)((int64_t)G.nt * G.mt * batches));
  hipLaunchKernelGGL(kern, xcd ? grid1 : grid3, dim3(64 * WM * WN), smem, s, G);
}

// v [B][L][Nh][H2] -> vt [B][Nh][H2][Lp] (Lp = L rounded up to 8, zero padded).  64 x 64 tiles:
// 16-byte loads along H2, 2-byte gathers from LDS, 16-byte stores along L.  `vec` = H2 % 8 == 0 and
// v 16-byte aligned (otherwise element-wise loads).
template <typename T>
__global__ __launch_bounds__(256) void transpose_v_kernel(const T* __restrict__ v, T* __restrict__ vt, int L, int Nh,
                                                          int H2, int Lp, int vec) {
  constexpr int TP = 66;                                         // LDS row pitch in elements (33 dwords)
  __shared__ T tile[64 * TP];
  const int bn = blockIdx.z;
  const int b = bn / Nh, n = bn - b * Nh;
  const int l0 = blockIdx.x * 64, h0 = blockIdx.y * 64;
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int pi = threadIdx.x + u * 256;
    const int li = pi >> 3, hc = (pi & 7) * 8;
    const int l = l0 + li, h = h0 + hc;
    Vec<T, 8> val;
#pragma unroll
    for (int e = 0; e < 8; ++e) val.v[e] = from_float<T>(0.f);
    if (l < L) {
      const T* src = v + (((int64_t)b * L + l) * Nh + n) * H2 + h;
      if (vec && h + 8 <= H2) {
        val = *(const Vec<T, 8>*)src;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (h + e < H2) val.v[e] = src[e];
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) tile[li * TP + hc + e] = val.v[e];
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int pi = threadIdx.x + u * 256;
    const int hi = pi >> 3, lc = (pi & 7) * 8;
    const int h = h0 + hi, l = l0 + lc;
    if (h < H2 && l < Lp) {
      Vec<T, 8> out;
#pragma unroll
      for (int e = 0; e < 8; ++e) out.v[e] = tile[(lc + e) * TP + hi];
      *(Vec<T, 8>*)(vt + (((int64_t)b * Nh + n) * H2 + h) * Lp + l) = out;     // Lp % 8 == 0: whole pieces
    }
  }
}

// causal softmax of fp32 scores into 16-bit probabilities; rows [outer][inner], pitch in elements
// (multiples of 4).  One wave per row, four rows per workgroup: the row is read once into registers
// (up to 32 values per lane = 2048 columns; longer rows are read three times), reductions stay
// inside the wave.  Columns past the causal limit are written as zeros only up to `zcols`, the end of
// the 256-column block the diagonal falls into (the second product, with row tiles of 128 or 256,
// never reads beyond it), unless the caller wants the whole weight matrix (zero_all).
template <typename TOut>
__global__ __launch_bounds__(256) void softmax_f32_kernel(const float* __restrict__ s, TOut* __restrict__ p, int outer,
                                                          int inner, int64_t spitch, int64_t ppitch, int pcols,
                                                          int causal, int zero_all, int64_t nrows) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= nrows) return;
  const int r = (int)(row % outer);
  int n = causal ? inner - outer + r + 1 : inner;
  if (n < 0) n = 0;
  int zcols = pcols;
  if (causal && !zero_all) zcols = min(pcols, ((n + 255) / 256) * 256);
  const float* sp = s + row * spitch;
  TOut* pp = p + row * ppitch;
  auto wave_max = [](float v) {
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m));
    return v;
  };
  auto wave_sum = [](float v) {
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m);
    return v;
  };
  constexpr int NV = 8;                              // float4 per lane held in registers: 2048 columns
  if (n <= 64 * 4 * NV && sizeof(TOut) == 2) {
    float4 v[NV];
    float m = -INFINITY;
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int j = (u * 64 + lane) * 4;
      v[u] = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
      if (j < n) {
        v[u] = *(const float4*)(sp + j);
        if (j + 1 >= n) v[u].y = -INFINITY;
        if (j + 2 >= n) v[u].z = -INFINITY;
        if (j + 3 >= n) v[u].w = -INFINITY;
      }
      m = fmaxf(m, fmaxf(fmaxf(v[u].x, v[u].y), fmaxf(v[u].z, v[u].w)));
    }
    m = wave_max(m);
    const bool dead = !(m > -INFINITY) || !(m < INFINITY);
    float sum = 0.f;
    if (!dead) {
#pragma unroll
      for (int u = 0; u < NV; ++u) {
        v[u].x = __expf(v[u].x - m); v[u].y = __expf(v[u].y - m);
        v[u].z = __expf(v[u].z - m); v[u].w = __expf(v[u].w - m);
        sum += (v[u].x + v[u].y) + (v[u].z + v[u].w);
      }
    } else {
      // every key masked or dropped: the registers hold -inf, and -inf * 0 would be NaN
#pragma unroll
      for (int u = 0; u < NV; ++u) v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    sum = wave_sum(sum);
    const float c = (dead || sum == 0.f) ? 0.f : 1.0f / sum;
    // live columns from registers (exp(-inf) = 0 covers the tail of a partial quad) ...
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int j = (u * 64 + lane) * 4;
      if (j < zcols && j < n) {
        TOut o0 = from_float<TOut>(v[u].x * c), o1 = from_float<TOut>(v[u].y * c);
        TOut o2 = from_float<TOut>(v[u].z * c), o3 = from_float<TOut>(v[u].w * c);
        uint2 w;
        w.x = (uint32_t)__builtin_bit_cast(uint16_t, o0) | ((uint32_t)__builtin_bit_cast(uint16_t, o1) << 16);
        w.y = (uint32_t)__builtin_bit_cast(uint16_t, o2) | ((uint32_t)__builtin_bit_cast(uint16_t, o3) << 16);
        *(uint2*)(pp + j) = w;
      }
    }
    // ... and zeros from the first whole quad past the limit up to zcols
    for (int j = ((n + 3) / 4 + lane) * 4; j < zcols; j += 256) *(uint2*)(pp + j) = make_uint2(0u, 0u);
    return;
  }
  float m = -INFINITY;
  for (int j = lane; j < n; j += 64) m = fmaxf(m, sp[j]);
  m = wave_max(m);
  const bool dead = !(m > -INFINITY) || !(m < INFINITY);
  float sum = 0.f;
  if (!dead)
    for (int j = lane; j < n; j += 64) sum += __expf(sp[j] - m);
  sum = wave_sum(sum);
  const float c = (dead || sum == 0.f) ? 0.f : 1.0f / sum;
  for (int j = lane; j < zcols; j += 64) {
    const float e = (j < n && !dead) ? __expf(sp[j] - m) * c : 0.f;
    pp[j] = from_float<TOut>(e);
  }
}

// DropKey on the fp32 scores, in place, ahead of the softmax: element (row, j) of the [B*Nh*L, L]
// score matrix becomes -inf when its uniform draw falls below `dropout`.  Launched only when
// dropout > 0, so the inference path does not pay for it.
__global__ __launch_bounds__(256) void dropkey_f32_kernel(float* __restrict__ s, int outer, int inner, int64_t spitch,
                                                          int causal, float dropout, uint64_t seed, int64_t nrows) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= nrows) return;
  const int r = (int)(row % outer);
  int n = causal ? inner - outer + r + 1 : inner;
  if (n > inner) n = inner;
  float* sp = s + row * spitch;
  const uint64_t e0 = (uint64_t)row * (uint64_t)inner;
  for (int j = lane; j < n; j += 64)
    if (hash_uniform(seed, e0 + j) < dropout) sp[j] = -INFINITY;
}

// rowdot[b, n, l] = sum_d dy[b, l, n, d] y[b, l, n, d]: with y = w v this is sum_j w[l, j] (dy v^T)[l, j], the row
// sum the softmax backward subtracts (attention_kernel.cu:195-203), without the L x L weight gradient in memory.
// One wave per (b, l, n) row of H2 elements (H2 % 8 == 0, 16-byte aligned rows), four rows per workgroup.
template <typename T>
__global__ __launch_bounds__(256) void rowdot_kernel(const T* __restrict__ dy, const T* __restrict__ y,
                                                     float* __restrict__ out, int L, int Nh, int H2, int64_t nrows) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= nrows) return;
  const int n = (int)(row % Nh);
  const int64_t bl = row / Nh;
  const int l = (int)(bl % L);
  const int64_t b = bl / L;
  const T* a = dy + row * H2;
  const T* c = y + row * H2;
  float acc = 0.f;
  for (int p = lane * 8; p < H2; p += 512) {
    const Vec<T, 8> x = *(const Vec<T, 8>*)(a + p);
    const Vec<T, 8> z = *(const Vec<T, 8>*)(c + p);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc = fmaf(to_float(x.v[e]), to_float(z.v[e]), acc);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if (lane == 0) out[(b * Nh + n) * L + l] = acc;
}

// Softmax backward on the fp32 weight gradient of the first backward product
// (fairseq/csrc/ops/attention_kernel.cu:195-203, softmax.cuh AttentionSoftmaxBwdKernel):
//   ds[r, c] = scale * w[r, c] * (dw[r, c] - sum_c' w[r, c'] dw[r, c']),
// w rows of `wpitch` elements, dw and ds rows of `pitch` (a multiple of 8, >= inner).  One wave per row, four rows
// per workgroup.  Columns behind the causal limit are not read (the product skips tiles above the diagonal and leaves
// them unwritten) and every column of ds from the limit to the end of the pitch is written as zero: the products
// that follow read whole rows and whole columns of ds.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void softmax_bwd_f32_kernel(const float* __restrict__ dw, const T* __restrict__ w,
                                                              T* __restrict__ ds, int outer, int inner, int64_t wpitch,
                                                              int64_t pitch, int causal, float scale, int64_t nrows) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= nrows) return;
  const int r = (int)(row % outer);
  int limit = causal ? inner - outer + r + 1 : inner;
  if (limit < 0) limit = 0;
  if (limit > inner) limit = inner;
  const float* dwr = dw + row * pitch;
  const T* wr = w + row * wpitch;
  T* dsr = ds + row * pitch;
  float dot = 0.f;
  for (int c = lane * VEC; c < limit; c += 64 * VEC) {
    const Vec<float, VEC> a = *(const Vec<float, VEC>*)(dwr + c);
    const Vec<T, VEC> b = *(const Vec<T, VEC>*)(wr + c);
#pragma unroll
    for (int e = 0; e < VEC; ++e)
      if (c + e < limit) dot = fmaf(a.v[e], to_float(b.v[e]), dot);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) dot += __shfl_xor(dot, o);
  for (int c = lane * VEC; c < (int)pitch; c += 64 * VEC) {
    Vec<T, VEC> o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) o.v[e] = from_float<T>(0.f);
    if (c < limit) {
      const Vec<float, VEC> a = *(const Vec<float, VEC>*)(dwr + c);
      const Vec<T, VEC> b = *(const Vec<T, VEC>*)(wr + c);
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        if (c + e < limit) o.v[e] = from_float<T>(scale * to_float(b.v[e]) * (a.v[e] - dot));
    }
    *(Vec<T, VEC>*)(dsr + c) = o;
  }
}

// ---------------------------------------------------------------------------------------------
// One kernel for the whole op when the weights are not wanted: scores, causal softmax and the
// second product per tile of 64 keys, with running row maxima and sums (no L x L array in memory).
// The products are formed transposed, S^T = k q^T and y^T = v^T P^T, so that a query is a column
// (lane & 15) of every accumulator: the running maximum, the rescaling of y and the row sum are
// per-lane scalars, and the probabilities go from the accumulators of the first product straight
// into the B operand of the second (the keys of a 32-key block are assigned to MFMA rows so that a
// lane ends up with eight consecutive keys).  A workgroup of 8 waves owns 256 queries of one
// (batch, head) and 256 columns of v; a wave owns 32 queries.  k and v tiles go from global memory
// straight into LDS (global_load ... lds), two buffers, the next tile in flight under the current
// tile's products; no staging registers, so the 128 accumulator registers of y leave room for the rest.
// v stays in its own layout (keys x columns): the A operand of the second product, v^T, is formed by the
// transposing LDS reads of gfx950 (ds_read_b64_tr_b16), so no transposed copy of v is made.
// Phase clocks: a profiling build defines these to add up the cycles a wave spends per phase; no-ops here.
#ifndef MEGA_ATR
#define MEGA_ATR_BEGIN()
#define MEGA_ATR_MARK()
#define MEGA_ATR(k)
#define MEGA_ATR_END()
#endif
constexpr int FBN = 64, FNW = 8;        // keys per tile, waves per workgroup

struct FlashArgs {
  const void* q;      // [B, L, Nh, H1]
  const void* k;      // [B, L, Nh, H1]
  const void* v;      // [B, L, Nh, H2]
  void* y;            // [B, L, Nh, H2]
  int L, Nh, H1, H2;
  float scale_log2;   // scale * log2(e)
  int causal;
  int xcd, mt, ns;
};

template <typename T>
__device__ __forceinline__ uint32_t pack2(float a, float b);
template <>
__device__ __forceinline__ uint32_t pack2<bf16_t>(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) __bf16 v2;
  const v2 v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, v);
}
template <>
__device__ __forceinline__ uint32_t pack2<f16_t>(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) _Float16 v2;
  const v2 v = {(_Float16)a, (_Float16)b};
  return __builtin_bit_cast(uint32_t, v);
}

// 16 bytes per lane from global memory straight into LDS (lane i of the wave lands at lds_base + 16 i).  Written as
// assembly on purpose: the compiler cannot tell which LDS reads a tile in flight may alias and would make every
// wave wait for the loads it has just issued (vmcnt(0)) before its first read of the current tile.  Here the
// loads are invisible to that bookkeeping; the kernel waits for them itself (vmcnt(0), then the workgroup barrier)
// before anybody reads the buffer they fill.
// M0 (the LDS base of such a load) is put back afterwards: the compiler does not honour a clobber of it.
__device__ __forceinline__ void lds_dma16(const void* base /* wave-uniform */, uint32_t lane_off, uint32_t lds_base) {
  uint32_t keep;
  asm volatile(
      "s_mov_b32 %[keep], m0\n\t"
      "s_mov_b32 m0, %[lds]\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %[off], %[base]\n\t"
      "s_mov_b32 m0, %[keep]"
      : [keep] "=&s"(keep)
      : [off] "v"(lane_off), [base] "s"(base), [lds] "s"(lds_base)
      : "memory");
}
__device__ __forceinline__ void lds_dma16(const void* addr /* per lane */, uint32_t lds_base) {
  uint32_t keep;
  asm volatile(
      "s_mov_b32 %[keep], m0\n\t"
      "s_mov_b32 m0, %[lds]\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %[addr], off\n\t"
      "s_mov_b32 m0, %[keep]"
      : [keep] "=&s"(keep)
      : [addr] "v"(addr), [lds] "s"(lds_base)
      : "memory");
}
// maximum over the four lanes that hold one query column (lanes n, n + 16, n + 32, n + 48), the same value in all
// four, with the lane-swap instructions of gfx950 instead of two trips through the LDS crossbar:
// v_permlane32_swap exchanges the upper half of its first operand with the lower half of its second,
// v_permlane16_swap the odd rows of 16 lanes of the first with the even rows of the second
__device__ __forceinline__ float quad_max(float t) {
  const uint32_t u = __builtin_bit_cast(uint32_t, t);
  const auto h = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const float m = fmaxf(__builtin_bit_cast(float, h[0]), __builtin_bit_cast(float, h[1]));
  const uint32_t v = __builtin_bit_cast(uint32_t, m);
  const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
  return fmaxf(__builtin_bit_cast(float, r[0]), __builtin_bit_cast(float, r[1]));
}

__device__ __forceinline__ uint32_t lds_addr(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

// KS = H1 / 32 reduction steps of the first product, FQB blocks of 16 queries per wave, FBD columns of v per
// workgroup (FQB * FBD = 512: 128 accumulator registers per lane either way).  Launched as 32 queries x 256 columns
// per wave; 16 queries x 512 columns (half as many workgroups repeat the score product and the softmax of a query
// tile, twice the LDS reads per matrix instruction) measured the same within 3 % from H2 = 512 to 2048
template <typename T, int KS, int FQB, int FBD>
__global__ __launch_bounds__(64 * FNW) void flash_fwd_kernel(const FlashArgs A) {
  constexpr int FBM = 16 * FNW * FQB;       // queries per workgroup
  constexpr int VR = 64 * FNW / (FBD / 8);  // rows of the v tile one load instruction of the workgroup covers
  constexpr int H1 = 32 * KS;
  constexpr int QW = 16 * FQB;              // queries per wave
  constexpr int KROW = H1 * 2;              // bytes per k row in LDS (dense; 16-byte pieces XOR-swizzled by the row)
  constexpr int KPC = H1 / 8;               // pieces per k row (8 or 16)
  constexpr int KB = FBN * KROW, VB = FBD * FBN * 2, BUF = KB + VB;
  constexpr int NKL = FBN * KPC / (64 * FNW);            // 16-byte pieces of a k tile per lane
  constexpr int NVL = FBD * (FBN / 8) / (64 * FNW);      // of a v^T tile
  static_assert(NKL >= 1 && FBN * KPC % (64 * FNW) == 0 && FBD * (FBN / 8) % (64 * FNW) == 0,
                "the tiles must divide over the lanes");
  extern __shared__ __attribute__((aligned(16))) char lds[];     // two k tiles, then two v tiles
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int bz, mtile, slab;
  {
    int rest = A.xcd ? (int)blockIdx.x >> 3 : (int)blockIdx.x;
    slab = rest % A.ns;
    rest /= A.ns;
    mtile = A.mt - 1 - rest % A.mt;                      // the long (late) query tiles of a causal call first
    rest /= A.mt;
    bz = A.xcd ? rest * 8 + ((int)blockIdx.x & 7) : rest;
  }
  const int b = bz / A.Nh, h = bz - b * A.Nh;
  const int m0 = mtile * FBM, d0 = slab * FBD;
  const int qw0 = m0 + wave * QW;
  const int n = lane & 15, g = lane >> 4;
  const T* qb = (const T*)A.q + ((int64_t)b * A.L * A.Nh + h) * H1;
  const T* kb_ = (const T*)A.k + ((int64_t)b * A.L * A.Nh + h) * H1;
  const T* vb = (const T*)A.v + ((int64_t)b * A.L * A.Nh + h) * A.H2 + d0;
  const int64_t vs = (int64_t)A.Nh * A.H2;               // row stride of v in elements
  const int64_t rs = (int64_t)A.Nh * H1;                 // row stride of q and k in elements

  // q^T as B operand: lane (n, g) holds q[query n of the block][32 s + 8 g ..]
  uint4 Qr[FQB][KS];
#pragma unroll
  for (int j = 0; j < FQB; ++j) {
    const int qi = qw0 + 16 * j + n;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      Qr[j][s] = make_uint4(0, 0, 0, 0);
      if (qi < A.L) Qr[j][s] = *(const uint4*)(qb + (int64_t)qi * rs + 32 * s + 8 * g);
    }
  }
  // tiles of keys this workgroup / this wave has to look at
  const int klim_wg = A.causal ? min(A.L, m0 + FBM) : A.L;         // keys < klim
  const int klim_w = A.causal ? min(A.L, qw0 + QW) : A.L;
  const int nkt = (klim_wg + FBN - 1) / FBN;

  // ---- tiles travel from global memory straight into LDS (no staging registers): lane i of a load
  // instruction supplies the 16 bytes that belong at the i-th piece of the wave's 1 KB of the tile image, so
  // every lane fetches the piece its LDS position stands for.  k image: row lrow = 16 (2 a + hb) + 4 gg + t holds
  // key 32 a + 8 gg + 4 hb + t (MFMA row block 2 a + hb then leaves lane (n, g) with keys 32 a + 8 g + 4 hb + {0..3}),
  // piece c at position c ^ (lrow & 15) (128-byte rows: c ^ ((lrow >> 1) & 7)).  v^T image: row r (128 bytes), piece c at position c ^ ((r >> 1) & 7).
  // Rows and columns past the end are fetched from the last valid one: their scores are masked, and a
  // probability of zero meets a finite value.
  // common case (whole tile inside the sequence, whole slab inside v): one per-lane byte offset per operand,
  // everything else is uniform (load u of a lane is 32 u keys / 64 u rows of v^T further on)
  uint32_t koff0, voffu[2];                  // v: loads of even / odd number (they differ in bit 3 of the row when a
  {                                          // load covers 8 rows, and the swizzle looks at that bit)
    const int lrow = tid / KPC, pp = tid % KPC;
    const int a = lrow >> 5, hb = (lrow >> 4) & 1, gg = (lrow >> 2) & 3, t = lrow & 3;
    const int key = 32 * a + 8 * gg + 4 * hb + t;
    const int kc = (pp ^ (KPC == 16 ? (lrow & 15) : ((lrow >> 1) & 7))) * 8;
    koff0 = (uint32_t)((key * (int)rs + kc) * 2);
    // v image: row = key (512 bytes), 16-byte piece p at position (((p >> 1) ^ vswz(row)) << 1) | (p & 1): the
    // 32-byte spans are XOR-swizzled so that the transposing reads of a fragment (four rows, four 8-byte
    // columns per group of 16 lanes) fall on different banks
    const int r = tid / (FBD / 8), vp = tid % (FBD / 8);
#pragma unroll
    for (int par = 0; par < 2; ++par) {
      const int rr = r + VR * par;             // a row of the loads with this parity
      const int p = ((((vp >> 1) ^ ((rr & 3) + 4 * ((rr >> 3) & 1))) << 1) | (vp & 1));
      voffu[par] = (uint32_t)((r * (int)vs + p * 8) * 2);
    }
  }
  static_assert(64 * FNW / KPC == 32 || NKL == 1, "load u of the k tile starts 32 u keys further on");
  static_assert(VR * NVL == FBN, "the loads of the v tile cover its rows in turn");
  const bool whole_slab = d0 + FBD <= A.H2;
  auto issue_tile = [&](int kt) {
    const int k0 = kt * FBN;
    const uint32_t lk = lds_addr(lds) + (kt & 1) * KB + wave * 1024;
    const uint32_t lv = lds_addr(lds) + 2 * KB + (kt & 1) * VB + wave * 1024;
    if (whole_slab && k0 + FBN <= A.L) {
      const char* kbase = (const char*)(kb_ + (int64_t)k0 * rs);
      const char* vbase = (const char*)(vb + (int64_t)k0 * vs);
#pragma unroll
      for (int u = 0; u < NKL; ++u) lds_dma16(kbase + (int64_t)u * 32 * rs * 2, koff0, lk + u * 1024 * FNW);
#pragma unroll
      for (int u = 0; u < NVL; ++u) lds_dma16(vbase + (int64_t)u * VR * vs * 2, voffu[u & 1], lv + u * 1024 * FNW);
      return;
    }
    // the last tile of a sequence / a partial slab: rows and columns past the end come from the last valid one
    asm volatile("" ::: "memory");
#pragma unroll
    for (int u = 0; u < NKL; ++u) {
      const int P = u * 64 * FNW + tid;
      const int lrow = P / KPC, pp = P % KPC;
      const int a = lrow >> 5, hb = (lrow >> 4) & 1, gg = (lrow >> 2) & 3, t = lrow & 3;
      const int key = min(k0 + 32 * a + 8 * gg + 4 * hb + t, A.L - 1);
      const int kc = (pp ^ (KPC == 16 ? (lrow & 15) : ((lrow >> 1) & 7))) * 8;
      lds_dma16(kb_ + (int64_t)key * rs + kc, lk + u * 1024 * FNW);
    }
#pragma unroll
    for (int u = 0; u < NVL; ++u) {
      const int P = u * 64 * FNW + tid;
      const int r = P / (FBD / 8), pp = P % (FBD / 8);
      const int key = min(k0 + r, A.L - 1);
      const int pc = ((((pp >> 1) ^ ((r & 3) + 4 * ((r >> 3) & 1))) << 1) | (pp & 1));
      const int col = min(pc * 8, A.H2 - d0 - 8);
      lds_dma16(vb + (int64_t)key * vs + col, lv + u * 1024 * FNW);
    }
  };

  f32x4 O[FBD / 16][FQB];
#pragma unroll
  for (int i = 0; i < FBD / 16; ++i)
#pragma unroll
    for (int j = 0; j < FQB; ++j) O[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  float mrun[FQB], lrun[FQB], pend[FQB];
#pragma unroll
  for (int j = 0; j < FQB; ++j) {
    mrun[j] = -INFINITY;
    lrun[j] = 0.f;
    pend[j] = 1.0f;
  }

  uint4 Pb[2][FQB];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int j = 0; j < FQB; ++j) Pb[a][j] = make_uint4(0, 0, 0, 0);
  MEGA_ATR_BEGIN();
  // ---- the two phases of a key tile.  scores: S^T = k q^T, mask, running maximum and sum; leaves the probabilities
  // (Pb) and the factor y has to be rescaled by (pend).  second: y^T += v^T P^T.
  auto scores = [&](int kt) {
    const int k0 = kt * FBN;
    if (k0 >= klim_w) return;                            // wave-uniform: no key of the tile is visible
    const char* lk = lds + (kt & 1) * KB;
    f32x4 S[4][FQB];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int j = 0; j < FQB; ++j) S[kb][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    {
      // fragment f = 4 s + kb: row 16 kb + n, piece 4 s + g at position (4 s + g) ^ n; two fragments ahead
      const char* kfrag = lk + n * KROW;
      const int ksw = KPC == 16 ? n : ((n >> 1) & 7);
      auto kaddr = [&](int f) { return kfrag + (f & 3) * 16 * KROW + (((f >> 2) * 4 + g) ^ ksw) * 16; };
      // the order below is kept as written (the fragment reads run DK fragments ahead of the products that
      // use them, so that the LDS latency is covered): no scheduling across the markers
      constexpr int DK = 4;
      uint4 fk[DK + 1];
#pragma unroll
      for (int f = 0; f < DK; ++f) fk[f] = *(const uint4*)kaddr(f);
#pragma unroll
      for (int f = 0; f < 4 * KS; ++f) {
        const int s = f >> 2, kb = f & 3;
        if (f + DK < 4 * KS) fk[(f + DK) % (DK + 1)] = *(const uint4*)kaddr(f + DK);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < FQB; ++j) S[kb][j] = mfma16<T>(fk[f % (DK + 1)], Qr[j][s], S[kb][j]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    MEGA_ATR(0);
    // mask, running maximum and sum; key of S[kb][j][u]: k0 + 32 (kb >> 1) + 8 g + 4 (kb & 1) + u
    const bool edge = (A.causal && k0 + FBN - 1 > qw0) || k0 + FBN > A.L;
#pragma unroll
    for (int j = 0; j < FQB; ++j) {
      const int qi = qw0 + 16 * j + n;
      const int lim = A.causal ? min(qi, A.L - 1) : A.L - 1;      // last visible key
      if (edge) {
        // only the tiles on the diagonal and the last one carry this code (kept a branch: the empty asm
        // statement stops the compiler from turning it into selects executed on every tile)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int kb = 0; kb < 4; ++kb)
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int key = k0 + 32 * (kb >> 1) + 8 * g + 4 * (kb & 1) + u;
            S[kb][j][u] = key <= lim ? S[kb][j][u] : -INFINITY;
          }
      }
      float tmax = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int u = 0; u < 4; ++u) tmax = fmaxf(tmax, S[kb][j][u]);
      tmax = quad_max(tmax);
      tmax *= A.scale_log2;                                        // scale > 0: the maximum commutes with it
      // the running maximum moves only when a tile exceeds it by more than 2^8: probabilities up to 256
      // are as exact as those below 1, and y is rescaled on few tiles
      const float mnew = tmax > mrun[j] + 8.0f ? tmax : mrun[j];
      const float muse = mnew == -INFINITY ? 0.f : mnew;
      const float corr = __builtin_amdgcn_exp2f(mrun[j] - muse);
      mrun[j] = mnew;
      float psum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float pv = __builtin_amdgcn_exp2f(fmaf(S[kb][j][u], A.scale_log2, -muse));
          S[kb][j][u] = pv;
          psum += pv;
        }
      lrun[j] = lrun[j] * corr + psum;
      pend[j] = corr;                                              // y is rescaled where it is next touched
#pragma unroll
      for (int a = 0; a < 2; ++a)
        Pb[a][j] = make_uint4(pack2<T>(S[2 * a][j][0], S[2 * a][j][1]), pack2<T>(S[2 * a][j][2], S[2 * a][j][3]),
                              pack2<T>(S[2 * a + 1][j][0], S[2 * a + 1][j][1]),
                              pack2<T>(S[2 * a + 1][j][2], S[2 * a + 1][j][3]));
    }
    MEGA_ATR(1);
  };
  auto second = [&](int kt) {
    if (kt * FBN >= klim_w) return;
    int vbo = (kt & 1) * VB;
    asm volatile("" : "+s"(vbo));                        // per step: keeps the fragment addresses out of loop-invariant registers
    const char* lv = lds + 2 * KB + vbo;
#pragma unroll
    for (int j = 0; j < FQB; ++j) {
      if (__any(pend[j] != 1.0f)) {
#pragma unroll
        for (int i = 0; i < FBD / 16; ++i)
#pragma unroll
          for (int u = 0; u < 4; ++u) O[i][j][u] *= pend[j];
      }
    }
    // fragment f = 2 i + a: the A operand v^T[d = 16 i + n][keys 32 a + 8 g ..+7] out of the key-major tile by two
    // transposing reads (ds_read_b64_tr_b16: lane s of a group of 16 supplies 8 bytes = 4 columns of one row;
    // lane l receives element l & 3 of the lanes (l >> 2) + 4 x, x = 0..3).  Source lane s points at row
    // 32 a + 8 g + 4 hh + (s >> 2), columns 16 i + 4 (s & 3): the result is 4 consecutive keys of column 16 i + n.
    const int sr = n >> 2, sc = n & 3;
    const char* vsrc = lv + (8 * g + sr) * (FBD * 2) + sc * 8;
    const int vsw = sr + 4 * (g & 1);
    // the swizzle touches the low three bits of the column block only: eight per-lane addresses, the rest of a
    // fragment's position is an immediate offset
    const char* va[8];
#pragma unroll
    for (int il = 0; il < 8; ++il) va[il] = vsrc + ((il ^ vsw) * 32);
    typedef __attribute__((ext_vector_type(4))) short s4v;
    auto vread = [&](int f) {
      const int i = f >> 1, a = f & 1;
      const char* q0 = va[i & 7] + a * 32 * (FBD * 2) + (i >> 3) * 256;
      const s4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*)(q0));
      const s4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*)(q0 + 4 * (FBD * 2)));
      const uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
      return make_uint4(l2.x, l2.y, h2.x, h2.y);
    };
    constexpr int NF = 2 * (FBD / 16);
    constexpr int DV = 6;                            // fragments in flight ahead of the products
    uint4 fv[DV + 1];
#pragma unroll
    for (int f = 0; f < DV; ++f) fv[f] = vread(f);
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      const int i = f >> 1, a = f & 1;
      if (f + DV < NF) fv[(f + DV) % (DV + 1)] = vread(f + DV);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < FQB; ++j) O[i][j] = mfma16<T>(fv[f % (DV + 1)], Pb[a][j], O[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
    MEGA_ATR(2);
  };

  if (nkt > 0) issue_tile(0);
  __builtin_amdgcn_s_waitcnt(0x0F70);                    // vmcnt(0): this wave's pieces have landed
  __syncthreads();
  MEGA_ATR_MARK();
  for (int kt = 0; kt < nkt; ++kt) {
    if (kt + 1 < nkt) issue_tile(kt + 1);                // lands under this tile's products
    MEGA_ATR(5);
    scores(kt);
    second(kt);
    __builtin_amdgcn_s_waitcnt(0x0F70);                  // vmcnt(0): the next tile's pieces of this wave have landed
    MEGA_ATR(3);
    __syncthreads();
    MEGA_ATR(4);
  }
  MEGA_ATR_END();
  // ---- 1 / row sum, then the wave's block of y leaves through LDS as whole 512-byte rows
  constexpr int OP = FBD * 2 + 16;                       // pitch of a staged row
  static_assert(16 * OP <= 2 * BUF / FNW, "a wave stages 16 rows at a time in its share of LDS");
  __syncthreads();                                       // the last products have read their tiles
  char* stage = lds + wave * (2 * BUF / FNW);
  T* yb = (T*)A.y + ((int64_t)b * A.L * A.Nh + h) * A.H2 + d0;
  const int64_t ys = (int64_t)A.Nh * A.H2;
#pragma unroll
  for (int j = 0; j < FQB; ++j) {
    float l = lrun[j];
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    const float inv = l > 0.f ? 1.0f / l : 0.f;          // a row without a visible key gives zeros
#pragma unroll
    for (int i = 0; i < FBD / 16; ++i) {
      const uint2 w = make_uint2(pack2<T>(O[i][j][0] * inv, O[i][j][1] * inv), pack2<T>(O[i][j][2] * inv, O[i][j][3] * inv));
      *(uint2*)(stage + n * OP + (16 * i + 4 * g) * 2) = w;
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int u = 0; u < 16 * (FBD / 8) / 64; ++u) {
      const int pi = lane + u * 64;
      const int r = pi / (FBD / 8), c = pi % (FBD / 8);
      const int qi = qw0 + 16 * j + r;
      if (qi < A.L && d0 + c * 8 < A.H2) *(uint4*)(yb + (int64_t)qi * ys + c * 8) = *(const uint4*)(stage + r * OP + c * 16);
    }
    __builtin_amdgcn_wave_barrier();
  }
}

template <typename T>
bool flash_covers(const void* v, const void* y, int64_t L, int64_t H1, int64_t H2) {
  return (H1 == 64 || H1 == 128) && H2 % 8 == 0 && H2 >= 64 && L >= 64 && ((uintptr_t)y % 16) == 0 &&
         ((uintptr_t)v % 16) == 0;
}

template <typename T>
void launch_flash(const void* q, const void* k, const void* v, void* y, int64_t B, int64_t L, int64_t Nh,
                  int64_t H1, int64_t H2, float scale, int causal, hipStream_t s) {
  constexpr int fqb = 2, fbd = 256, fbm = 16 * FNW * fqb;
  FlashArgs F;
  F.q = q; F.k = k; F.v = v; F.y = y;
  F.L = (int)L; F.Nh = (int)Nh; F.H1 = (int)H1; F.H2 = (int)H2;
  F.scale_log2 = scale * 1.4426950408889634f;
  F.causal = causal ? 1 : 0;
  F.mt = (int)ceil_div(L, fbm);
  F.ns = (int)ceil_div(H2, fbd);
  const int64_t BN_ = B * Nh;
  F.xcd = BN_ % 8 == 0 ? 1 : 0;
  const dim3 grid((unsigned)(BN_ * F.mt * F.ns));
  const int ks = (int)(H1 / 32);
  const size_t smem = 2 * ((size_t)FBN * H1 * 2 + (size_t)fbd * FBN * 2);
#define MEGA_FLASH(KS_)                                                                                       \
  {                                                                                                           \
    auto kern = flash_fwd_kernel<T, KS_, fqb, fbd>;                                                           \
    static uint64_t attr_seen = 0;                                                                            \
    if (first_on_device(&attr_seen)) {                                                                        \
      (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);    \
    }                                                                                                         \
    hipLaunchKernelGGL(kern, grid, dim3(64 * FNW), smem, s, F);                                               \
  }
  if (ks == 2) MEGA_FLASH(2) else MEGA_FLASH(4)
#undef MEGA_FLASH
}

template <typename T>
int run_attention(const void* q, const void* k, const void* v, void* y, void* w, int64_t B, int64_t L, int64_t Nh,
                  int64_t H1, int64_t H2, float scale, int causal, float dropout, uint64_t seed, char* ws,
                  hipStream_t s) {
  const int64_t Lp = (L + 7) / 8 * 8;
  const int64_t BN_ = B * Nh;
  float* S = (float*)ws;
  ws += align_up((size_t)BN_ * L * Lp * 4, 256);
  // probabilities [B*Nh][L][Lp]; when the caller wants the weights and their rows need no padding, they are written
  // where the caller wants them and the second product reads them there
  T* P = (w && Lp == L && ((uintptr_t)w % 16) == 0) ? (T*)w : (T*)ws;
  ws += align_up((size_t)BN_ * L * Lp * sizeof(T), 256);
  T* Vt = (T*)ws;                                  // [B*Nh][H2][Lp]
  if (!w && dropout <= 0.f && scale > 0.f && flash_covers<T>(v, y, L, H1, H2)) {
    launch_flash<T>(q, k, v, y, B, L, Nh, H1, H2, scale, causal, s);
    MEGA_CHECK_LAUNCH("attention_fwd (one-kernel path)");
    return MEGA_OK;
  }
  // v enters the second product through its columns: read in place (K-major form of the kernel) when its rows are
  // whole 16-byte pieces, through a transposed, zero-padded copy otherwise
  const bool v_inplace = H2 % 8 == 0 && ((uintptr_t)v % 16) == 0;
  if (!v_inplace && y) {
    const dim3 grid((unsigned)ceil_div(Lp, 64), (unsigned)ceil_div(H2, 64), (unsigned)BN_);
    hipLaunchKernelGGL(transpose_v_kernel<T>, grid, dim3(256), 0, s, (const T*)v, Vt, (int)L, (int)Nh, (int)H2, (int)Lp,
                       0);
  }
  GemmArgs G;
  // S[b,n] = scale q[b,:,n,:] k[b,:,n,:]^T
  G.A = q; G.Bm = k; G.C = S;
  G.lda = Nh * H1; G.ldb = Nh * H1; G.ldc = Lp;
  G.sa = L * Nh * H1; G.sai = H1; G.sb = L * Nh * H1; G.sbi = H1; G.sc = Nh * L * Lp; G.sci = L * Lp;
  G.nin = (int)Nh; G.M = (int)L; G.N = (int)L; G.K = (int)H1; G.alpha = scale; G.causal = causal ? 1 : 0; G.kshift = 0;
  const bool xcd = BN_ % 8 == 0;
  launch_gemm<T, float, 2, 2>(G, L, L, BN_, xcd, s);
  if (dropout > 0.f)
    hipLaunchKernelGGL(dropkey_f32_kernel, dim3((unsigned)ceil_div(BN_ * L, 4)), dim3(256), 0, s, S, (int)L, (int)L, Lp,
                       causal, dropout, seed, (int64_t)(BN_ * L));
  hipLaunchKernelGGL(softmax_f32_kernel<T>, dim3((unsigned)ceil_div(BN_ * L, 4)), dim3(256), 0, s, S, P, (int)L, (int)L,
                     Lp, Lp, (int)Lp, causal, w ? 1 : 0, (int64_t)(BN_ * L));
  if (w && (void*)P != w) {
    // the weights the reference returns: [B, Nh, L, L]
    hipMemcpy2DAsync(w, (size_t)L * sizeof(T), P, (size_t)Lp * sizeof(T), (size_t)L * sizeof(T), (size_t)(BN_ * L),
                     hipMemcpyDeviceToDevice, s);
  }
  if (!y) {                                        // the weights alone (a backward that forms them again)
    MEGA_CHECK_LAUNCH("attention_fwd (weights)");
    return MEGA_OK;
  }
  // y[b,:,n,:] = P[b,n] v[b,:,n,:]  ==  P (v^T)^T
  G.A = P; G.C = y;
  G.lda = Lp; G.ldc = Nh * H2;
  G.sa = Nh * L * Lp; G.sai = L * Lp; G.sc = L * Nh * H2; G.sci = H2;
  G.M = (int)L; G.N = (int)H2; G.alpha = 1.0f; G.causal = causal ? 2 : 0;
  // the second product carries the flops: 256 x 256 tiles when the problem has that many rows and columns
  if (v_inplace) {
    G.Bm = v; G.ldb = Nh * H2; G.sb = L * Nh * H2; G.sbi = H2; G.K = (int)L;
    if (L >= 256 && H2 >= 256) launch_gemm<T, T, 4, 4, false, true>(G, L, H2, BN_, xcd, s);
    else launch_gemm<T, T, 2, 2, false, true>(G, L, H2, BN_, xcd, s);
  } else {
    G.Bm = Vt; G.ldb = Lp; G.sb = Nh * H2 * Lp; G.sbi = H2 * Lp; G.K = (int)Lp;
    if (L >= 256 && H2 >= 256) launch_gemm<T, T, 4, 4>(G, L, H2, BN_, xcd, s);
    else launch_gemm<T, T, 2, 2>(G, L, H2, BN_, xcd, s);
  }
  MEGA_CHECK_LAUNCH("attention_fwd (matrix-core path)");
  return MEGA_OK;
}

// workspace of the backward, in this order (each part 256-byte aligned)
struct BwdWs {
  size_t dw, ds, wt, dst, dyt, qt, kt, rowdot, total;
};
BwdWs bwd_workspace(size_t es, int64_t B, int64_t L, int64_t Nh, int64_t H1, int64_t H2) {
  const int64_t Lp = (L + 7) / 8 * 8, BN_ = B * Nh;
  BwdWs W;
  size_t o = 0;
  auto take = [&](size_t bytes) {
    const size_t at = o;
    o += align_up(bytes, 256);
    return at;
  };
  W.dw = take((size_t)BN_ * L * Lp * 4);       // fp32 [BN][L][Lp]
  W.ds = take((size_t)BN_ * L * Lp * es);      // [BN][L][Lp]
  W.wt = take((size_t)BN_ * L * Lp * es);      // w^T [BN][L][Lp]
  W.dst = take((size_t)BN_ * Lp * Lp * es);    // dS^T [BN][Lp][Lp] (rows past L are zero)
  W.dyt = take((size_t)BN_ * H2 * Lp * es);    // dy^T [BN][H2][Lp]
  W.qt = take((size_t)BN_ * H1 * Lp * es);     // q^T [BN][H1][Lp]
  W.kt = take((size_t)BN_ * H1 * Lp * es);     // k^T
  W.rowdot = take((size_t)BN_ * L * 4);        // fp32 [BN][L]
  W.total = o;
  return W;
}

template <typename T>
void launch_transpose(const T* src, T* dst, int64_t batches, int64_t rows, int64_t nin, int64_t cols, int64_t Lp,
                      hipStream_t s) {
  // src [batches / nin][rows][nin][cols] -> dst [batches][cols][Lp]
  if (audit_on()) {
    audit_use(src, (size_t)batches * rows * cols * sizeof(T), "transpose source");
    audit_use(dst, (size_t)batches * cols * Lp * sizeof(T), "transpose destination");
    return;
  }
  const dim3 grid((unsigned)ceil_div(Lp, 64), (unsigned)ceil_div(cols, 64), (unsigned)batches);
  const int vec = (cols % 8 == 0 && ((uintptr_t)src % 16) == 0) ? 1 : 0;
  hipLaunchKernelGGL(transpose_v_kernel<T>, grid, dim3(256), 0, s, src, dst, (int)rows, (int)nin, (int)cols, (int)Lp,
                     vec);
}

template <typename T>
int run_attention_bwd(const void* dy, const void* q, const void* k, const void* v, const void* w, const void* y,
                      void* dq, void* dk, void* dv, int64_t B, int64_t L, int64_t Nh, int64_t H1, int64_t H2, float scale,
                      int causal, char* ws, hipStream_t s) {
  const int64_t Lp = (L + 7) / 8 * 8, BN_ = B * Nh;
  const BwdWs W = bwd_workspace(sizeof(T), B, L, Nh, H1, H2);
  float* dW = (float*)(ws + W.dw);
  T* dS = (T*)(ws + W.ds);
  T* Wt = (T*)(ws + W.wt);
  T* dSt = (T*)(ws + W.dst);
  T* dYt = (T*)(ws + W.dyt);
  T* Qt = (T*)(ws + W.qt);
  T* Kt = (T*)(ws + W.kt);
  const bool xcd = BN_ % 8 == 0;
  // operands that enter a product through their columns (w, dS, dy, q, k) are read in place by the K-major form of
  // the kernel when their rows are whole 16-byte pieces; otherwise through transposed, zero-padded copies
  const bool inplace = L % 8 == 0 && ((uintptr_t)w % 16) == 0;
  if (!inplace) {
    launch_transpose<T>((const T*)dy, dYt, BN_, L, Nh, H2, Lp, s);
    launch_transpose<T>((const T*)q, Qt, BN_, L, Nh, H1, Lp, s);
    launch_transpose<T>((const T*)k, Kt, BN_, L, Nh, H1, Lp, s);
    launch_transpose<T>((const T*)w, Wt, BN_, L, 1, L, Lp, s);
  }
  GemmArgs G;
  G.nin = (int)Nh; G.kshift = 0;
  // dW[b,n] = dy[b,:,n,:] v[b,:,n,:]^T (attention_kernel.cu:176-193)
  G.A = dy; G.Bm = v; G.C = dW;
  G.lda = Nh * H2; G.ldb = Nh * H2; G.ldc = Lp;
  G.sa = L * Nh * H2; G.sai = H2; G.sb = L * Nh * H2; G.sbi = H2; G.sc = Nh * L * Lp; G.sci = L * Lp;
  G.M = (int)L; G.N = (int)L; G.K = (int)H2; G.alpha = 1.0f; G.causal = causal ? 1 : 0;
  // with the forward's y at hand the row sum of the softmax backward is dy . y, known before the product, and dS
  // leaves the product's epilogue directly: no fp32 weight gradient in memory, no softmax-backward pass
  const bool fused = inplace && y != nullptr && ((uintptr_t)y % 16) == 0;
  if (fused) {
    float* rd = (float*)(ws + W.rowdot);
    const int64_t nrows = B * L * Nh;
    if (audit_on()) {
      audit_use(dy, (size_t)nrows * H2 * sizeof(T), "row dot: y_grad");
      audit_use(y, (size_t)nrows * H2 * sizeof(T), "row dot: y");
      audit_use(rd, (size_t)nrows * 4, "row dot: sums");
    } else {
      hipLaunchKernelGGL(rowdot_kernel<T>, dim3((unsigned)ceil_div(nrows, 4)), dim3(256), 0, s, (const T*)dy, (const T*)y,
                         rd, (int)L, (int)Nh, (int)H2, nrows);
    }
    G.C = dS; G.E = w; G.rowdot = rd; G.lde = L; G.se = Nh * L * L; G.sei = L * L; G.alpha = scale;
    if (L >= 512) launch_gemm<T, float, 4, 4, false, false, 1>(G, L, L, BN_, xcd, s);
    else launch_gemm<T, float, 2, 2, false, false, 1>(G, L, L, BN_, xcd, s);
  } else if (L >= 512) {
    launch_gemm<T, float, 4, 4>(G, L, L, BN_, xcd, s);
  } else {
    launch_gemm<T, float, 2, 2>(G, L, L, BN_, xcd, s);
  }
  // dS = scale w (dW - rowsum(w dW)) (attention_kernel.cu:195-203)
  if (!fused) {
    const int64_t nrows = BN_ * L;
    const dim3 grid((unsigned)ceil_div(nrows, 4));
    const bool vec = L % 4 == 0 && ((uintptr_t)w % 8) == 0;
    if (audit_on()) {
      // rows of dW / dS have pitch Lp, rows of w pitch L; L columns each
      audit_use(dW, (size_t)((nrows - 1) * Lp + L) * 4, "softmax backward: weight gradient");
      audit_use(w, (size_t)nrows * L * sizeof(T), "softmax backward: weights");
      audit_use(dS, (size_t)nrows * Lp * sizeof(T), "softmax backward: score gradient (whole rows of the pitch)");
    } else if (vec)
      hipLaunchKernelGGL((softmax_bwd_f32_kernel<T, 4>), grid, dim3(256), 0, s, dW, (const T*)w, dS, (int)L, (int)L, L, Lp,
                         causal, scale, nrows);
    else
      hipLaunchKernelGGL((softmax_bwd_f32_kernel<T, 1>), grid, dim3(256), 0, s, dW, (const T*)w, dS, (int)L, (int)L, L, Lp,
                         causal, scale, nrows);
  }
  if (inplace) {
    // dv[b,:,n,:] = w[b,n]^T dy[b,:,n,:] (attention_kernel.cu:155-174): both operands K-major
    G.A = w; G.Bm = dy; G.C = dv;
    G.lda = L; G.ldb = Nh * H2; G.ldc = Nh * H2;
    G.sa = Nh * L * L; G.sai = L * L; G.sb = L * Nh * H2; G.sbi = H2; G.sc = L * Nh * H2; G.sci = H2;
    G.M = (int)L; G.N = (int)H2; G.K = (int)L; G.alpha = 1.0f; G.causal = causal ? 3 : 0;
    if (L >= 256 && H2 >= 256) launch_gemm<T, T, 2, 4, true, true, 0, 8, 4>(G, L, H2, BN_, xcd, s);
    else launch_gemm<T, T, 2, 2, true, true>(G, L, H2, BN_, xcd, s);
    // dq[b,:,n,:] = dS[b,n] k[b,:,n,:] (attention_kernel.cu:205-222): k K-major
    G.A = dS; G.Bm = k; G.C = dq;
    G.lda = Lp; G.ldb = Nh * H1; G.ldc = Nh * H1;
    G.sa = Nh * L * Lp; G.sai = L * Lp; G.sb = L * Nh * H1; G.sbi = H1; G.sc = L * Nh * H1; G.sci = H1;
    G.N = (int)H1; G.causal = causal ? 2 : 0;
    launch_gemm<T, T, 2, 2, false, true, 0, 2, 4>(G, L, H1, BN_, xcd, s);
    // dk[b,:,n,:] = dS[b,n]^T q[b,:,n,:] (attention_kernel.cu:224-241): both operands K-major
    G.Bm = q; G.C = dk;
    G.causal = causal ? 3 : 0;
    launch_gemm<T, T, 2, 2, true, true>(G, L, H1, BN_, xcd, s);
    if (!audit_on()) {
      MEGA_CHECK_LAUNCH("attention_bwd");
    }
    return MEGA_OK;
  }
  // dS [BN][L][Lp] -> dS^T [BN][Lp][Lp]
  launch_transpose<T>(dS, dSt, BN_, L, 1, Lp, Lp, s);
  // dv[b,:,n,:] = w[b,n]^T dy[b,:,n,:] (attention_kernel.cu:155-174): rows of w^T against rows of dy^T
  G.A = Wt; G.Bm = dYt; G.C = dv;
  G.lda = Lp; G.ldb = Lp; G.ldc = Nh * H2;
  G.sa = Nh * L * Lp; G.sai = L * Lp; G.sb = Nh * H2 * Lp; G.sbi = H2 * Lp; G.sc = L * Nh * H2; G.sci = H2;
  G.M = (int)L; G.N = (int)H2; G.K = (int)Lp; G.alpha = 1.0f; G.causal = causal ? 3 : 0;
  if (L >= 256 && H2 >= 256) launch_gemm<T, T, 4, 4>(G, L, H2, BN_, xcd, s);
  else launch_gemm<T, T, 2, 2>(G, L, H2, BN_, xcd, s);
  // dq[b,:,n,:] = dS[b,n] k[b,:,n,:] (attention_kernel.cu:205-222)
  G.A = dS; G.Bm = Kt; G.C = dq;
  G.lda = Lp; G.ldb = Lp; G.ldc = Nh * H1;
  G.sa = Nh * L * Lp; G.sai = L * Lp; G.sb = Nh * H1 * Lp; G.sbi = H1 * Lp; G.sc = L * Nh * H1; G.sci = H1;
  G.M = (int)L; G.N = (int)H1; G.K = (int)Lp; G.causal = causal ? 2 : 0;
  launch_gemm<T, T, 2, 2>(G, L, H1, BN_, xcd, s);
  // dk[b,:,n,:] = dS[b,n]^T q[b,:,n,:] (attention_kernel.cu:224-241)
  G.A = dSt; G.Bm = Qt;  G.C = dk;
  G.sa = Nh * Lp * Lp; G.sai = Lp * Lp;
  G.causal = causal ? 3 : 0;
  launch_gemm<T, T, 2, 2>(G, L, H1, BN_, xcd, s);
  if (!audit_on()) {
    MEGA_CHECK_LAUNCH("attention_bwd");
  }
  return MEGA_OK;
}

}  // namespace

bool attention_mfma_covers(int dtype, const void* q, const void* k, const void* v, int64_t B, int64_t L, int64_t Nh,
                           int64_t H1, int64_t H2) {
  if (dtype == MEGA_F32) return false;
  if (H1 % 8 != 0) return false;                              // 16-byte operand rows of q and k
  if (((uintptr_t)q % 16) || ((uintptr_t)k % 16)) return false;
  if (B * Nh > 65535 || L >= (int64_t)1 << 24) return false;
  (void)v; (void)H2;
  return true;
}

size_t attention_mfma_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t Nh, int64_t H2) {
  const int64_t Lp = (L + 7) / 8 * 8;
  const size_t es = dtype == MEGA_F32 ? 4 : 2;
  return align_up((size_t)B * Nh * L * Lp * 4, 256) + align_up((size_t)B * Nh * L * Lp * es, 256) +
         align_up((size_t)B * Nh * H2 * Lp * es, 256);
}

int attention_mfma_run(const void* q, const void* k, const void* v, void* y, void* w, int dtype, int64_t B, int64_t L,
                       int64_t Nh, int64_t H1, int64_t H2, float scale, int causal, float dropout, uint64_t seed,
                       void* ws, hipStream_t s) {
  if (dtype == MEGA_BF16)
    return run_attention<bf16_t>(q, k, v, y, w, B, L, Nh, H1, H2, scale, causal, dropout, seed, (char*)ws, s);
  return run_attention<f16_t>(q, k, v, y, w, B, L, Nh, H1, H2, scale, causal, dropout, seed, (char*)ws, s);
}

bool attention_mfma_bwd_covers(int dtype, const void* dy, const void* q, const void* k, const void* v, const void* dq,
                               const void* dk, const void* dv, int64_t B, int64_t L, int64_t Nh, int64_t H1,
                               int64_t H2) {
  if (dtype == MEGA_F32) return false;
  if (H1 % 8 != 0 || H2 % 8 != 0) return false;                // 16-byte operand and result rows
  const uintptr_t all = (uintptr_t)dy | (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)dq | (uintptr_t)dk |
                        (uintptr_t)dv;
  if (all % 16) return false;
  if (B * Nh > 65535 || L >= (int64_t)1 << 15) return false;   // L x L x batch index arithmetic in the transposes
  return true;
}

size_t attention_mfma_bwd_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t Nh, int64_t H1, int64_t H2) {
  return bwd_workspace(dtype == MEGA_F32 ? 4 : 2, B, L, Nh, H1, H2).total;
}

int attention_mfma_bwd_run(const void* dy, const void* q, const void* k, const void* v, const void* w, const void* y,
                           void* dq, void* dk, void* dv, int dtype, int64_t B, int64_t L, int64_t Nh, int64_t H1, int64_t H2,
                           float scale, int causal, void* ws, hipStream_t s) {
  if (dtype == MEGA_BF16)
    return run_attention_bwd<bf16_t>(dy, q, k, v, w, y, dq, dk, dv, B, L, Nh, H1, H2, scale, causal, (char*)ws, s);
  return run_attention_bwd<f16_t>(dy, q, k, v, w, y, dq, dk, dv, B, L, Nh, H1, H2, scale, causal, (char*)ws, s);
}

}  // namespace mega
