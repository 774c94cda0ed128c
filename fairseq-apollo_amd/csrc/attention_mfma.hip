// Attention on the matrix cores: y = softmax_causal(scale q k^T) v per (batch, head)
// (fairseq/csrc/ops/attention_kernel.cu:40-131), 16-bit activations.
//
//   S = scale q k^T        batched NT GEMM, v_mfma_f32_16x16x32_{bf16,f16}, fp32 out; causal: tiles
//                          above the diagonal are skipped
//   P = softmax_causal(S)  one workgroup per row, fp32 in, 16-bit out (right-aligned mask, a fully
//                          masked row gives zeros: fairseq/csrc/softmax.cuh:90-153)
//   y = P v                the same NT GEMM against v^T (v is transposed once through LDS); causal:
//                          the reduction stops at the diagonal
//
// The GEMM: 128 x 128 output tile per workgroup (4 waves, 64 x 64 each as 4 x 4 MFMA blocks),
// K step 32, operands staged through LDS with an 80-byte row pitch (conflict-free 16-byte reads),
// register prefetch of the next K step.
#include "common.h"

namespace mega {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int BM = 128, BN = 128, BK = 32;
constexpr int PITCH = 80;                 // bytes per LDS row of 32 16-bit elements (+ 16 pad)

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
  int causal;         // 1: S = q k^T (skip tiles with n0 > m0 + BM - 1); 2: y = P v (K stops at m0 + BM)
  int kshift;         // causal offset: row m sees columns <= m + kshift
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

// C = alpha A B^T; TIn 16-bit, TOut float or TIn
template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void gemm_nt_kernel(const GemmArgs G) {
  __shared__ __attribute__((aligned(16))) char lds[2 * (BM + BN) * PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  if (G.causal == 1 && n0 > m0 + BM - 1 + G.kshift) return;      // entirely above the diagonal
  const int bz = blockIdx.z;
  const int bo = bz / G.nin, bi = bz - bo * G.nin;
  const TIn* A = (const TIn*)G.A + bo * G.sa + bi * G.sai;
  const TIn* Bm = (const TIn*)G.Bm + bo * G.sb + bi * G.sbi;
  TOut* C = (TOut*)G.C + bo * G.sc + bi * G.sci;
  int Kend = G.K;
  if (G.causal == 2) Kend = min(G.K, m0 + BM + G.kshift);
  if (Kend < 0) Kend = 0;
  const int nk = (Kend + BK - 1) / BK;

  // global -> register staging: thread covers 2 x 16 bytes of A and of B per K step
  const int lrow = tid >> 2, lcol = (tid & 3) * 8;               // rows 0..63 (+64), 8 elements each
  uint4 ra[2], rb[2];
  auto gload = [&](int kt) {
    const int k = kt * BK + lcol;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = lrow + h * 64;
      ra[h] = make_uint4(0, 0, 0, 0);
      rb[h] = make_uint4(0, 0, 0, 0);
      if (m0 + r < G.M && k < Kend) ra[h] = *(const uint4*)(A + (int64_t)(m0 + r) * G.lda + k);
      if (n0 + r < G.N && k < Kend) rb[h] = *(const uint4*)(Bm + (int64_t)(n0 + r) * G.ldb + k);
    }
  };
  auto lstore = [&](int buf) {
    char* la = lds + buf * (BM + BN) * PITCH;
    char* lb = la + BM * PITCH;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = lrow + h * 64;
      *(uint4*)(la + r * PITCH + lcol * 2) = ra[h];
      *(uint4*)(lb + r * PITCH + lcol * 2) = rb[h];
    }
  };
  f32x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int fr = lane & 15, fk = (lane >> 4) * 16;                // fragment row, byte offset of the k block

  if (nk > 0) {
    gload(0);
    lstore(0);
  }
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) gload(kt + 1);
    const char* la = lds + buf * (BM + BN) * PITCH;
    const char* lb = la + BM * PITCH;
    uint4 fa[4], fb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) fa[i] = *(const uint4*)(la + (wm + i * 16 + fr) * PITCH + fk);
#pragma unroll
    for (int j = 0; j < 4; ++j) fb[j] = *(const uint4*)(lb + (wn + j * 16 + fr) * PITCH + fk);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = mfma16<TIn>(fa[i], fb[j], acc[i][j]);
    if (kt + 1 < nk) lstore(buf ^ 1);
    __syncthreads();
  }
  // D layout: column = lane & 15, rows 4 (lane >> 4) + {0..3}
  const int cn = lane & 15, cr = (lane >> 4) * 4;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + wn + j * 16 + cn;
      if (n >= G.N) continue;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int m = m0 + wm + i * 16 + cr + u;
        if (m < G.M) C[(int64_t)m * G.ldc + n] = from_float<TOut>(acc[i][j][u] * G.alpha);
      }
    }
}

// v [B][L][Nh][H2] -> vt [B][Nh][H2][Lp] (Lp = L rounded up to 8, zero padded)
template <typename T>
__global__ __launch_bounds__(256) void transpose_v_kernel(const T* __restrict__ v, T* __restrict__ vt, int L, int Nh,
                                                          int H2, int Lp) {
  __shared__ T tile[32][33];
  const int bn = blockIdx.z;
  const int b = bn / Nh, n = bn - b * Nh;
  const int l0 = blockIdx.x * 32, h0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;      // 32 x 8
  for (int i = ty; i < 32; i += 8) {
    const int l = l0 + i, h = h0 + tx;
    T val = from_float<T>(0.f);
    if (l < L && h < H2) val = v[(((int64_t)b * L + l) * Nh + n) * H2 + h];
    tile[i][tx] = val;
  }
  __syncthreads();
  for (int i = ty; i < 32; i += 8) {
    const int h = h0 + i, l = l0 + tx;
    if (h < H2 && l < Lp) vt[(((int64_t)b * Nh + n) * H2 + h) * Lp + l] = tile[tx][i];
  }
}

// causal softmax of fp32 scores into 16-bit probabilities; rows [outer][inner], pitch in elements
template <typename TOut>
__global__ __launch_bounds__(256) void softmax_f32_kernel(const float* __restrict__ s, TOut* __restrict__ p, int outer,
                                                          int inner, int64_t spitch, int64_t ppitch, int pcols,
                                                          int causal) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const int r = (int)(row % outer);
  int n = causal ? inner - outer + r + 1 : inner;
  if (n < 0) n = 0;
  const float* sp = s + row * spitch;
  TOut* pp = p + row * ppitch;
  auto reduce = [&](float v, bool is_max) {
    for (int m = 32; m >= 1; m >>= 1) {
      const float o = __shfl_xor(v, m);
      v = is_max ? fmaxf(v, o) : v + o;
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < 4; ++i) t = is_max ? fmaxf(t, red[i]) : t + red[i];
    return t;
  };
  float m = -INFINITY;
  for (int j = threadIdx.x; j < n; j += 256) m = fmaxf(m, sp[j]);
  m = reduce(m, true);
  const bool dead = !(m > -INFINITY) || !(m < INFINITY);
  float sum = 0.f;
  if (!dead)
    for (int j = threadIdx.x; j < n; j += 256) sum += __expf(sp[j] - m);
  sum = reduce(sum, false);
  const float c = (dead || sum == 0.f) ? 0.f : 1.0f / sum;
  for (int j = threadIdx.x; j < pcols; j += 256) {
    const float e = (j < n && !dead) ? __expf(sp[j] - m) * c : 0.f;
    pp[j] = from_float<TOut>(e);
  }
}

template <typename T>
int run_attention(const void* q, const void* k, const void* v, void* y, void* w, int64_t B, int64_t L, int64_t Nh,
                  int64_t H1, int64_t H2, float scale, int causal, char* ws, hipStream_t s) {
  const int64_t Lp = (L + 7) / 8 * 8;
  const int64_t BN_ = B * Nh;
  float* S = (float*)ws;
  ws += align_up((size_t)BN_ * L * Lp * 4, 256);
  T* P = (T*)ws;                                   // [B*Nh][L][Lp]
  ws += align_up((size_t)BN_ * L * Lp * sizeof(T), 256);
  T* Vt = (T*)ws;                                  // [B*Nh][H2][Lp]
  {
    const dim3 grid((unsigned)ceil_div(Lp, 32), (unsigned)ceil_div(H2, 32), (unsigned)BN_);
    hipLaunchKernelGGL(transpose_v_kernel<T>, grid, dim3(256), 0, s, (const T*)v, Vt, (int)L, (int)Nh, (int)H2, (int)Lp);
  }
  GemmArgs G;
  // S[b,n] = scale q[b,:,n,:] k[b,:,n,:]^T
  G.A = q; G.Bm = k; G.C = S;
  G.lda = Nh * H1; G.ldb = Nh * H1; G.ldc = Lp;
  G.sa = L * Nh * H1; G.sai = H1; G.sb = L * Nh * H1; G.sbi = H1; G.sc = Nh * L * Lp; G.sci = L * Lp;
  G.nin = (int)Nh; G.M = (int)L; G.N = (int)L; G.K = (int)H1; G.alpha = scale; G.causal = causal ? 1 : 0; G.kshift = 0;
  {
    const dim3 grid((unsigned)ceil_div(L, BN), (unsigned)ceil_div(L, BM), (unsigned)BN_);
    hipLaunchKernelGGL((gemm_nt_kernel<T, float>), grid, dim3(256), 0, s, G);
  }
  hipLaunchKernelGGL(softmax_f32_kernel<T>, dim3((unsigned)(BN_ * L)), dim3(256), 0, s, S, P, (int)L, (int)L, Lp, Lp,
                     (int)Lp, causal);
  if (w) {
    // the weights the reference returns: [B, Nh, L, L]
    hipMemcpy2DAsync(w, (size_t)L * sizeof(T), P, (size_t)Lp * sizeof(T), (size_t)L * sizeof(T), (size_t)(BN_ * L),
                     hipMemcpyDeviceToDevice, s);
  }
  // y[b,:,n,:] = P[b,n] v[b,:,n,:]  ==  P (v^T)^T
  G.A = P; G.Bm = Vt; G.C = y;
  G.lda = Lp; G.ldb = Lp; G.ldc = Nh * H2;
  G.sa = Nh * L * Lp; G.sai = L * Lp; G.sb = Nh * H2 * Lp; G.sbi = H2 * Lp; G.sc = L * Nh * H2; G.sci = H2;
  G.M = (int)L; G.N = (int)H2; G.K = (int)Lp; G.alpha = 1.0f; G.causal = causal ? 2 : 0;
  {
    const dim3 grid((unsigned)ceil_div(H2, BN), (unsigned)ceil_div(L, BM), (unsigned)BN_);
    hipLaunchKernelGGL((gemm_nt_kernel<T, T>), grid, dim3(256), 0, s, G);
  }
  MEGA_CHECK_LAUNCH("attention_fwd (matrix-core path)");
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
                       int64_t Nh, int64_t H1, int64_t H2, float scale, int causal, void* ws, hipStream_t s) {
  if (dtype == MEGA_BF16) return run_attention<bf16_t>(q, k, v, y, w, B, L, Nh, H1, H2, scale, causal, (char*)ws, s);
  return run_attention<f16_t>(q, k, v, y, w, B, L, Nh, H1, H2, scale, causal, (char*)ws, s);
}

}  // namespace mega
