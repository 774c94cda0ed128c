/* CPU oracle, plain C.  TEST INFRASTRUCTURE ONLY: loaded by tests/, by
 * __graft_entry__.smoke() and by the cpu_baseline leg of bench.py, never by the
 * product path.
 *
 * Each function restates the loop structure of the reference's CPU
 * implementation (file:line given per function, relative to the reference
 * tree), including where it parallelises (at::parallel_for -> omp parallel for),
 * so that timing it on host cores stands for the reference's CPU path.
 * All of these are checked against mega_oracle.py (numpy fp64), closed forms
 * and, where it is built, oracle/_ref in tests/test_oracle_c.py.
 */
#include <complex.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ */
/* EMA kernel generation: csrc/ops/ema_parameters.cc:37-52            */
/* w[d,l] = sum_n Re(p gamma exp(l log q)); parallel over d           */
/* ------------------------------------------------------------------ */
#define DEF_EMA_KERNEL(NAME, T, CT, CEXP)                                          \
  void NAME(const T* p, const T* logq /* [K,N,2] */, const T* gamma /* [K,N,2] */, \
            int64_t K, int64_t N, int64_t L, T* w) {                               \
    _Pragma("omp parallel for schedule(static)")                                   \
    for (int64_t i = 0; i < K; ++i) {                                              \
      for (int64_t j = 0; j < L; ++j) {                                            \
        T sum = 0;                                                                 \
        for (int64_t k = 0; k < N; ++k) {                                          \
          const int64_t o = (i * N + k) * 2;                                       \
          const CT c = p[i * N + k] * (gamma[o] + gamma[o + 1] * I);               \
          const CT lq = logq[o] + logq[o + 1] * I;                                 \
          const CT qw = CEXP(lq * (T)j);                                           \
          sum += creal(c * qw);                                                    \
        }                                                                          \
        w[i * L + j] = sum;                                                        \
      }                                                                            \
    }                                                                              \
  }
DEF_EMA_KERNEL(ora_ema_kernel_f32, float, float complex, cexpf)
DEF_EMA_KERNEL(ora_ema_kernel_f64, double, double complex, cexp)

/* bias from a carried state: csrc/ops/ema_parameters.cc:54-77        */
#define DEF_EMA_BIAS(NAME, T, CT, CEXP)                                            \
  void NAME(const T* logq, const T* gamma, const T* h /* [B,K,N,2] */, int64_t B,  \
            int64_t K, int64_t N, int64_t L, T* b) {                               \
    _Pragma("omp parallel for schedule(static)")                                   \
    for (int64_t i = 0; i < B * K; ++i) {                                          \
      const int64_t d = i % K;                                                     \
      for (int64_t j = 0; j < L; ++j) {                                            \
        T sum = 0;                                                                 \
        for (int64_t k = 0; k < N; ++k) {                                          \
          const int64_t o = (d * N + k) * 2;                                       \
          const int64_t oh = (i * N + k) * 2;                                      \
          const CT lq = logq[o] + logq[o + 1] * I;                                 \
          const CT g = gamma[o] + gamma[o + 1] * I;                                \
          const CT hh = h[oh] + h[oh + 1] * I;                                     \
          const CT qw = CEXP(lq * (T)(j + 1));                                     \
          sum += creal(qw * g * hh);                                               \
        }                                                                          \
        b[i * L + j] = sum;                                                        \
      }                                                                            \
    }                                                                              \
  }
DEF_EMA_BIAS(ora_ema_bias_f32, float, float complex, cexpf)
DEF_EMA_BIAS(ora_ema_bias_f64, double, double complex, cexp)

/* hidden state: csrc/ops/ema_hidden.cc:31-63                         */
#define DEF_EMA_HIDDEN(NAME, T, CT, CEXP)                                          \
  void NAME(const T* x /* [B,D,L] */, const T* p, const T* logq, const T* h,       \
            int64_t B, int64_t D, int64_t N, int64_t L, T* y /* [B,D,N,2] */) {    \
    _Pragma("omp parallel for schedule(static)")                                   \
    for (int64_t i = 0; i < D * N; ++i) {                                          \
      const int64_t d = i / N;                                                     \
      const CT lq = logq[2 * i] + logq[2 * i + 1] * I;                             \
      for (int64_t b = 0; b < B; ++b) {                                            \
        const T* xp = x + (b * D + d) * L;                                         \
        CT sum = 0;                                                                \
        for (int64_t j = 0; j < L; ++j) {                                          \
          sum += CEXP(lq * (T)(L - j - 1)) * xp[j];                                \
        }                                                                          \
        sum *= p[i];                                                               \
        if (h != NULL) {                                                           \
          const int64_t o = (b * D * N + i) * 2;                                   \
          sum += CEXP(lq * (T)L) * (h[o] + h[o + 1] * I);                          \
        }                                                                          \
        y[(b * D * N + i) * 2] = creal(sum);                                       \
        y[(b * D * N + i) * 2 + 1] = cimag(sum);                                   \
      }                                                                            \
    }                                                                              \
  }
DEF_EMA_HIDDEN(ora_ema_hidden_f32, float, float complex, cexpf)
DEF_EMA_HIDDEN(ora_ema_hidden_f64, double, double complex, cexp)

/* ------------------------------------------------------------------ */
/* direct causal convolution (small sizes; the reference uses FFTs)   */
/* y[b,d,t] = sum_{j<=t, j<Lk} k[d,j] x[b,d,t-j]                      */
/* ------------------------------------------------------------------ */
void ora_causal_conv_direct_f64(const double* x, const double* k, int64_t B, int64_t D,
                                int64_t L, int64_t Lk, double* y) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < B * D; ++r) {
    const int64_t d = r % D;
    for (int64_t t = 0; t < L; ++t) {
      double s = 0;
      const int64_t jm = t + 1 < Lk ? t + 1 : Lk;
      for (int64_t j = 0; j < jm; ++j) s += k[d * Lk + j] * x[r * L + t - j];
      y[r * L + t] = s;
    }
  }
}

/* ------------------------------------------------------------------ */
/* Welford helpers: csrc/utils.h:55-76                                */
/* ------------------------------------------------------------------ */
#define DEF_WELFORD(T, SFX)                                                        \
  static inline void welford_update_##SFX(int64_t m0, T* m1, T* m2, T x) {         \
    const T coef = (T)1 / (T)(m0 + 1);                                             \
    const T d1 = x - *m1;                                                          \
    *m1 += coef * d1;                                                              \
    const T d2 = d1 * (x - *m1) - *m2;                                             \
    *m2 += coef * d2;                                                              \
  }                                                                                \
  static inline void welford_combine_##SFX(int64_t a0, T a1, T a2, int64_t b0,     \
                                           T b1, T b2, T* m1, T* m2) {             \
    const int64_t m0 = a0 + b0;                                                    \
    const T c1 = m0 == 0 ? (T)0 : (T)a0 / (T)m0;                                   \
    const T c2 = m0 == 0 ? (T)0 : (T)b0 / (T)m0;                                   \
    const T delta = b1 - a1;                                                       \
    *m1 = c1 * a1 + c2 * b1;                                                       \
    *m2 = c1 * a2 + c2 * b2 + (c1 * delta) * (c2 * delta);                         \
  }                                                                                \
  /* moments of one row in chunks of 16 with a binary cascade: utils.h:79-118 */   \
  static void rowwise_moments_##SFX(int64_t n, const T* x, T* mean, T* var) {      \
    int64_t num_chunks = (n + 15) / 16;                                            \
    int64_t depth = 1;                                                             \
    while (((int64_t)1 << depth) < num_chunks) ++depth;                            \
    int64_t m0s[64];                                                               \
    T m1s[64], m2s[64];                                                            \
    for (int64_t i = 0; i < depth; ++i) { m0s[i] = 0; m1s[i] = 0; m2s[i] = 0; }    \
    for (int64_t i = 0; i < num_chunks; ++i) {                                     \
      const int64_t l = i * 16, r = l + 16 < n ? l + 16 : n;                       \
      for (int64_t j = l; j < r; ++j) {                                            \
        welford_update_##SFX(m0s[0], &m1s[0], &m2s[0], x[j]);                      \
        m0s[0] += 1;                                                               \
      }                                                                            \
      int64_t cnt = i + 1;                                                         \
      for (int64_t j = 1; j < depth && (cnt & 1) == 0; ++j) {                      \
        T u, v;                                                                    \
        welford_combine_##SFX(m0s[j], m1s[j], m2s[j], m0s[j - 1], m1s[j - 1],      \
                              m2s[j - 1], &u, &v);                                 \
        m0s[j] += m0s[j - 1]; m1s[j] = u; m2s[j] = v;                              \
        m0s[j - 1] = 0; m1s[j - 1] = 0; m2s[j - 1] = 0;                            \
        cnt >>= 1;                                                                 \
      }                                                                            \
    }                                                                              \
    for (int64_t i = 1; i < depth; ++i) {                                          \
      T u, v;                                                                      \
      welford_combine_##SFX(m0s[0], m1s[0], m2s[0], m0s[i], m1s[i], m2s[i], &u, &v); \
      m0s[0] += m0s[i]; m1s[0] = u; m2s[0] = v;                                    \
    }                                                                              \
    *mean = m1s[0];                                                                \
    *var = m2s[0];                                                                 \
  }
DEF_WELFORD(float, f32)
DEF_WELFORD(double, f64)

/* ------------------------------------------------------------------ */
/* group TimestepNorm forward: csrc/ops/timestep_norm.cc:218-316      */
/* stage 1 parallel over (b,l,g); stage 2 parallel over b only        */
/* ------------------------------------------------------------------ */
#define DEF_GROUP_TSN(NAME, T, SFX, SQRT)                                          \
  void NAME(const T* x /* [B,L,H] */, const int64_t* prev_count, const T* prev_mean, \
            const T* prev_var /* [B,G] */, const T* gamma, const T* beta,          \
            const uint8_t* mask /* [B,L] or NULL */, int64_t B, int64_t L,         \
            int64_t H, int64_t G, double eps, T* y, int64_t* count, T* mean,       \
            T* var, T* scratch /* 2*B*L*G */) {                                    \
    const int64_t Dg = H / G;                                                      \
    T* gmean = scratch;                                                            \
    T* gvar = scratch + B * L * G;                                                 \
    _Pragma("omp parallel for schedule(static)")                                   \
    for (int64_t i = 0; i < B * L * G; ++i) {                                      \
      rowwise_moments_##SFX(Dg, x + i * Dg, &gmean[i], &gvar[i]);                  \
    }                                                                              \
    _Pragma("omp parallel for schedule(static)")                                   \
    for (int64_t i = 0; i < B; ++i) {                                              \
      int64_t m0 = prev_count[i];                                                  \
      T* u = mean + i * G;                                                         \
      T* v = var + i * G;                                                          \
      for (int64_t g = 0; g < G; ++g) { u[g] = prev_mean[i * G + g]; v[g] = prev_var[i * G + g]; } \
      for (int64_t j = 0; j < L; ++j) {                                            \
        const int masked = mask != NULL && mask[i * L + j];                        \
        for (int64_t g = 0; g < G; ++g) {                                          \
          T m1, m2;                                                                \
          welford_combine_##SFX(m0, u[g], v[g], 1, gmean[(i * L + j) * G + g],     \
                                gvar[(i * L + j) * G + g], &m1, &m2);              \
          const T rstd = (T)1 / SQRT(m2 + (T)eps);                                 \
          if (!masked) { u[g] = m1; v[g] = m2; }                                   \
          const T* xp = x + (i * L + j) * H + g * Dg;                              \
          T* yp = y + (i * L + j) * H + g * Dg;                                    \
          for (int64_t k = 0; k < Dg; ++k) {                                       \
            yp[k] = masked ? (T)0 : (xp[k] - m1) * rstd * gamma[g * Dg + k] + beta[g * Dg + k]; \
          }                                                                        \
        }                                                                          \
        m0 += masked ? 0 : 1;                                                      \
      }                                                                            \
      count[i] = m0;                                                               \
    }                                                                              \
  }
DEF_GROUP_TSN(ora_group_timestep_norm_f32, float, f32, sqrtf)
DEF_GROUP_TSN(ora_group_timestep_norm_f64, double, f64, sqrt)

/* per-feature TimestepNorm forward: csrc/ops/timestep_norm.cc:23-103 */
#define DEF_TSN(NAME, T, SFX, SQRT)                                                \
  void NAME(const T* x, const int64_t* prev_count, const T* prev_mean,             \
            const T* prev_var /* [B,H] */, const T* gamma, const T* beta,          \
            const uint8_t* mask, int64_t B, int64_t L, int64_t H, double eps,      \
            T* y, int64_t* count, T* mean, T* var) {                               \
    _Pragma("omp parallel for schedule(static)")                                   \
    for (int64_t i = 0; i < B; ++i) {                                              \
      int64_t m0 = prev_count[i];                                                  \
      T* u = mean + i * H;                                                         \
      T* v = var + i * H;                                                          \
      for (int64_t k = 0; k < H; ++k) { u[k] = prev_mean[i * H + k]; v[k] = prev_var[i * H + k]; } \
      for (int64_t j = 0; j < L; ++j) {                                            \
        const int masked = mask != NULL && mask[i * L + j];                        \
        for (int64_t k = 0; k < H; ++k) {                                          \
          const T xv = x[(i * L + j) * H + k];                                     \
          T m1 = u[k], m2 = v[k];                                                  \
          welford_update_##SFX(m0, &m1, &m2, xv);                                  \
          const T rstd = (T)1 / SQRT(m2 + (T)eps);                                 \
          y[(i * L + j) * H + k] = masked ? (T)0 : (xv - m1) * rstd * gamma[k] + beta[k]; \
          if (!masked) { u[k] = m1; v[k] = m2; }                                   \
        }                                                                          \
        m0 += masked ? 0 : 1;                                                      \
      }                                                                            \
      count[i] = m0;                                                               \
    }                                                                              \
  }
DEF_TSN(ora_timestep_norm_f32, float, f32, sqrtf)
DEF_TSN(ora_timestep_norm_f64, double, f64, sqrt)

/* ------------------------------------------------------------------ */
/* attention softmax forward: csrc/softmax.cuh:90-153                 */
/* rows x[outer, inner]; causal keeps inner - outer + r + 1 columns    */
/* ------------------------------------------------------------------ */
void ora_attention_softmax_f64(const double* x, int64_t batch, int64_t outer, int64_t inner,
                               int causal, double* y) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < batch * outer; ++i) {
    const int64_t r = i % outer;
    int64_t n = causal ? inner - outer + r + 1 : inner;
    if (n < 0) n = 0;
    const double* xp = x + i * inner;
    double* yp = y + i * inner;
    double m = -INFINITY;
    for (int64_t j = 0; j < n; ++j) m = xp[j] > m ? xp[j] : m;
    double s = 0;
    for (int64_t j = 0; j < inner; ++j) {
      yp[j] = (j < n && isfinite(m)) ? exp(xp[j] - m) : 0.0;
      s += yp[j];
    }
    const double c = s == 0 ? 0.0 : 1.0 / s;
    for (int64_t j = 0; j < inner; ++j) yp[j] *= c;
  }
}
