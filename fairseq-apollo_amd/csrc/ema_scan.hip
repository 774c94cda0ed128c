// Generic (any N <= 32, real or complex, any stride) EMA path on the vector ALUs:
// the recurrence h' = q h + p x, y = Re sum_n gamma h, evaluated as a chunked scan.
//
//   pass A  chunk_state : S[c] = sum_{i in chunk c} q^{len-1-i} u_i        (zero start)
//   pass B  chunk_scan  : H_in[c] = state at the start of chunk c (serial over the few
//                         chunks), H_out = state after the last chunk
//   pass C  chunk_apply : runs the recurrence inside every chunk from H_in[c] and writes y
//
// This is exactly the decomposition the reference uses for incremental evaluation
// (kernel + carried-state bias + ema_hidden,
// fairseq/modules/base_moving_average.py:144-160, fairseq/csrc/ops/ema_parameters.cc:54-77,
// fairseq/csrc/ops/ema_hidden.cc:31-63), applied per chunk instead of per call; the
// D x L convolution kernel is never formed.
//
// A "pass set" (A, B, C) evaluates one causal filter along one time direction.  The
// layer is a sum of pass sets: forward direction; for bidirectional layers the reversed
// direction with the second half of the coefficient rows
// (fairseq/modules/fused_ops/fftconv.py:85-100); a kernel truncated to Lk taps is
// "full filter minus the same filter delayed by Lk and scaled by q^Lk".
//
// Thread mapping: TPR = ceil(N/4) lanes share one (batch, channel) row, 4 complex
// states each; rows are laid out channel-fastest so that [B,L,D] activations are read
// coalesced.  Activations with a contiguous time axis ([B,D,L]) take the *_rows kernels,
// which stage sub-tiles of time through LDS.  On such rows, a one-sided untruncated layer
// whose rows fit one workgroup's units runs the three passes in one kernel
// (ema_rows_fused_kernel), and a two-sided untruncated layer whose chunks fit one sub-tile
// runs both directions from the same staged samples (bidir_*_rows_kernel, one launch for
// both chunk scans) instead of one pass set per direction.
#include "common.h"
#include "ema_mfma.h"

namespace mega {

namespace {

constexpr int kNPT = 4;          // complex states per thread
constexpr int kBlock = 256;

// coefficient image of one pass set, padded to NP = TPR*4 states per row (zeros beyond N)
struct PassCoef {
  const float* q;   // [Drows, np, 2]
  const float* c;   // [Drows, np, 2]  output coefficient (gamma, or -gamma q^Lk)
  const float* p;   // [Drows, np]     input coefficient
  int np;           // states per row in memory: NP for the padded images, N for the caller's own arrays
};

// element offset of state n of row d, or -1 for a padded state that the arrays do not hold (all of its
// coefficients are zero); the kernels of the two-sided row passes and the chunk scan read through it
__device__ __forceinline__ int64_t coef_at(const PassCoef& cf, int d, int n) {
  return n < cf.np ? (int64_t)d * cf.np + n : -1;
}

struct PassArgs {
  const void* x;
  int64_t sxb, sxd, sxl;
  const uint8_t* mask;     // [B, L] or null
  PassCoef coef;
  const float* h_in;       // [B, D, N, 2] or null (true carried state)
  float* h_out;            // [B, D, N, 2] or null
  float* st;               // [B, nchunks, D, NP, 2] chunk states / chunk-start states
  int B, D, N, L;
  int NP, TPR;
  int Tc, nchunks;
  int reverse;             // logical time runs from the end of the sequence
  int before;              // output uses the state before absorbing the current sample
  int tshift;              // the filter input is delayed by tshift samples
  // output stage
  const float* acc_in;     // fp32 partial sums from earlier pass sets, or null: [B, L, D], or [B, D, L]
  float* acc_out;          // when the passes run on time-contiguous rows; null when this pass set writes y
  void* y;
  int64_t syb, syd, syl;
  const float* omega;      // [D]
};

// sum over the TPR (1, 2, 4 or 8) adjacent lanes of a unit, left in every one of them: lane exchanges
// inside quads, then between the two quads of an 8-lane half (data-parallel primitives, no LDS traffic)
template <int CTRL>
__device__ __forceinline__ float lane_swap(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float unit_sum(float v, int tpr) {
  if (tpr >= 2) v += lane_swap<0xB1>(v);     // quad_perm [1, 0, 3, 2]
  if (tpr >= 4) v += lane_swap<0x4E>(v);     // quad_perm [2, 3, 0, 1]
  if (tpr >= 8) v += lane_swap<0x141>(v);    // mirror inside each half row of 8 lanes
  return v;
}

template <typename T>
__device__ __forceinline__ float load_u(const PassArgs& A, int b, int d, int tau) {
  // logical sample tau of the (delayed, masked) filter input
  const int ts = tau - A.tshift;
  if (ts < 0) return 0.f;
  const int t = A.reverse ? A.L - 1 - ts : ts;
  // both loads are issued before either is looked at: one round trip, not two
  const T v = ((const T*)A.x)[b * A.sxb + d * A.sxd + t * A.sxl];
  const uint8_t pad = A.mask ? A.mask[(size_t)b * A.L + t] : (uint8_t)0;
  return pad ? 0.f : to_float(v);
}

template <typename T, bool CPLX>
__global__ __launch_bounds__(kBlock) void chunk_state_kernel(const PassArgs A) {
  const int64_t gid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t total = (int64_t)A.B * A.nchunks * A.D * A.TPR;
  if (gid >= total) return;
  const int ns = (int)(gid % A.TPR);
  const int d = (int)((gid / A.TPR) % A.D);
  const int c = (int)((gid / ((int64_t)A.TPR * A.D)) % A.nchunks);
  const int b = (int)(gid / ((int64_t)A.TPR * A.D * A.nchunks));
  float qr[kNPT], qi[kNPT], hr[kNPT], hi[kNPT];
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    const size_t o = ((size_t)d * A.NP + ns * kNPT + k) * 2;
    qr[k] = A.coef.q[o];
    qi[k] = CPLX ? A.coef.q[o + 1] : 0.f;
    hr[k] = 0.f;
    hi[k] = 0.f;
  }
  const int t0 = c * A.Tc;
  const int t1 = min(t0 + A.Tc, A.L);
  for (int tau = t0; tau < t1; ++tau) {
    const float u = load_u<T>(A, b, d, tau);
#pragma unroll
    for (int k = 0; k < kNPT; ++k) {
      if (CPLX) {
        const float nr = qr[k] * hr[k] - qi[k] * hi[k] + u;
        const float ni = qr[k] * hi[k] + qi[k] * hr[k];
        hr[k] = nr;
        hi[k] = ni;
      } else {
        hr[k] = qr[k] * hr[k] + u;
      }
    }
  }
  float* sp = A.st + ((((size_t)b * A.nchunks + c) * A.D + d) * A.NP + ns * kNPT) * 2;
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    sp[2 * k] = hr[k];
    sp[2 * k + 1] = hi[k];
  }
}

// Exclusive scan of the chunk states.  A (batch, channel) row is owned by G lane groups of NP
// threads (thread = one state of one group); a group owns a run of consecutive chunks.  Pass 1 folds
// the run into one aggregate (loads in batches, all of a batch in flight), the groups' aggregates
// meet in LDS and every thread folds the earlier groups' into its start state, pass 2 walks the
// run again and leaves the state at the start of every chunk in place of the chunk's own sum.
// G is a power of two (1 when there are few chunks, then a workgroup owns 256 / NP rows).
constexpr int kScanBatch = 8;

template <bool CPLX>
__device__ __forceinline__ void chunk_scan_body(const PassArgs& A, const int G, float* s_agg) {
  const int n = threadIdx.x % A.NP;
  const int grp = (threadIdx.x / A.NP) % G;
  const int rloc = threadIdx.x / (A.NP * G);
  const int rows_per_wg = kBlock / (A.NP * G);
  const int64_t row = (int64_t)blockIdx.x * rows_per_wg + rloc;
  const bool live = row < (int64_t)A.B * A.D;
  const int d = live ? (int)(row % A.D) : 0;
  const int b = live ? (int)(row / A.D) : 0;
  const int64_t oc = coef_at(A.coef, d, n);
  const double qr = oc >= 0 ? A.coef.q[oc * 2] : 0.0, qi = CPLX && oc >= 0 ? A.coef.q[oc * 2 + 1] : 0.0;
  const float p = oc >= 0 ? A.coef.p[oc] : 0.f;
  double Qr, Qi;
  cpow_int(qr, qi, A.Tc, &Qr, &Qi);
  const float fQr = (float)Qr, fQi = (float)Qi;
  const int cpg = (A.nchunks + G - 1) / G;
  const int cb = min(grp * cpg, A.nchunks), ce = live ? min(cb + cpg, A.nchunks) : cb;
  const size_t cstride = (size_t)A.D * A.NP * 2;
  float* base = A.st + (((size_t)b * A.nchunks) * A.D + d) * A.NP * 2 + (size_t)n * 2;
  // pass 1: the run's aggregate from a zero start
  float hr = 0.f, hi = 0.f;
  for (int c = cb; c < ce; c += kScanBatch) {
    float sr[kScanBatch], si[kScanBatch];
#pragma unroll
    for (int k = 0; k < kScanBatch; ++k) {
      const bool ok = c + k < ce;
      const float* sp = base + (size_t)(ok ? c + k : c) * cstride;
      sr[k] = sp[0];
      si[k] = CPLX ? sp[1] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < kScanBatch; ++k)
      if (c + k < ce) {
        const float nr = fQr * hr - fQi * hi + p * sr[k];
        const float ni = fQr * hi + fQi * hr + p * si[k];
        hr = nr;
        hi = ni;
      }
  }
  s_agg[threadIdx.x * 2] = hr;
  s_agg[threadIdx.x * 2 + 1] = hi;
  __syncthreads();
  // start state of the run: the carried state pushed through the earlier runs
  hr = 0.f;
  hi = 0.f;
  if (live && A.h_in && n < A.N) {
    const size_t oh = (((size_t)b * A.D + d) * A.N + n) * 2;
    hr = A.h_in[oh];
    hi = CPLX ? A.h_in[oh + 1] : 0.f;
  }
  if (grp > 0) {
    double Gr, Gi;
    cpow_int(qr, qi, (int64_t)A.Tc * cpg, &Gr, &Gi);
    const float fGr = (float)Gr, fGi = (float)Gi;
    for (int j = 0; j < grp; ++j) {
      const int o = (threadIdx.x - (grp - j) * A.NP) * 2;
      const float nr = fGr * hr - fGi * hi + s_agg[o];
      const float ni = fGr * hi + fGi * hr + s_agg[o + 1];
      hr = nr;
      hi = ni;
    }
  }
  // pass 2: chunk-start states in place; the last chunk of the row may be shorter
  float Lr = fQr, Li = fQi;
  if (ce == A.nchunks && ce > cb) {
    double lr, li;
    cpow_int(qr, qi, A.L - (int64_t)(A.nchunks - 1) * A.Tc, &lr, &li);
    Lr = (float)lr;
    Li = (float)li;
  }
  for (int c = cb; c < ce; c += kScanBatch) {
    float sr[kScanBatch], si[kScanBatch];
#pragma unroll
    for (int k = 0; k < kScanBatch; ++k) {
      const bool ok = c + k < ce;
      const float* sp = base + (size_t)(ok ? c + k : c) * cstride;
      sr[k] = sp[0];
      si[k] = CPLX ? sp[1] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < kScanBatch; ++k)
      if (c + k < ce) {
        float* sp = base + (size_t)(c + k) * cstride;
        sp[0] = hr;
        sp[1] = hi;
        const bool last = c + k == A.nchunks - 1;
        const float Ar = last ? Lr : fQr, Ai = last ? Li : fQi;
        const float nr = Ar * hr - Ai * hi + p * sr[k];
        const float ni = Ar * hi + Ai * hr + p * si[k];
        hr = nr;
        hi = ni;
      }
  }
  if (A.h_out && n < A.N && ce == A.nchunks && ce > cb) {
    const size_t oh = (((size_t)b * A.D + d) * A.N + n) * 2;
    A.h_out[oh] = hr;
    A.h_out[oh + 1] = hi;
  }
}

template <bool CPLX>
__global__ __launch_bounds__(kBlock) void chunk_scan_kernel(const PassArgs A, const int G) {
  __shared__ float s_agg[kBlock * 2];
  chunk_scan_body<CPLX>(A, G, s_agg);
}

// the scans of the two directions of a two-sided layer in one launch (blockIdx.y picks the direction)
template <bool CPLX>
__global__ __launch_bounds__(kBlock) void chunk_scan2_kernel(const PassArgs A, const PassArgs R, const int G) {
  __shared__ float s_agg[kBlock * 2];
  if (blockIdx.y == 0) chunk_scan_body<CPLX>(A, G, s_agg);
  else chunk_scan_body<CPLX>(R, G, s_agg);
}

template <typename T, bool CPLX>
__global__ __launch_bounds__(kBlock) void chunk_apply_kernel(const PassArgs A) {
  const int64_t gid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t total = (int64_t)A.B * A.nchunks * A.D * A.TPR;
  const bool live = gid < total;
  const int64_t g2 = live ? gid : total - 1;     // keep whole lane groups converged for the shuffles
  const int ns = (int)(g2 % A.TPR);
  const int d = (int)((g2 / A.TPR) % A.D);
  const int c = (int)((g2 / ((int64_t)A.TPR * A.D)) % A.nchunks);
  const int b = (int)(g2 / ((int64_t)A.TPR * A.D * A.nchunks));
  float qr[kNPT], qi[kNPT], cr[kNPT], ci[kNPT], pp[kNPT], hr[kNPT], hi[kNPT];
  const float* sp = A.st + ((((size_t)b * A.nchunks + c) * A.D + d) * A.NP + ns * kNPT) * 2;
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    const size_t o = ((size_t)d * A.NP + ns * kNPT + k) * 2;
    qr[k] = A.coef.q[o];
    qi[k] = CPLX ? A.coef.q[o + 1] : 0.f;
    cr[k] = A.coef.c[o];
    ci[k] = CPLX ? A.coef.c[o + 1] : 0.f;
    pp[k] = A.coef.p[o / 2];
    hr[k] = sp[2 * k];
    hi[k] = sp[2 * k + 1];
  }
  const float om = A.omega ? A.omega[d] : 0.f;
  const int t0 = c * A.Tc;
  const int t1 = min(t0 + A.Tc, A.L);
  for (int tau = t0; tau < t1; ++tau) {
    const float u = load_u<T>(A, b, d, tau);
    float acc = 0.f;
    if (A.before) {
#pragma unroll
      for (int k = 0; k < kNPT; ++k) acc += CPLX ? (cr[k] * hr[k] - ci[k] * hi[k]) : cr[k] * hr[k];
    }
#pragma unroll
    for (int k = 0; k < kNPT; ++k) {
      const float pu = pp[k] * u;
      if (CPLX) {
        const float nr = qr[k] * hr[k] - qi[k] * hi[k] + pu;
        const float ni = qr[k] * hi[k] + qi[k] * hr[k];
        hr[k] = nr;
        hi[k] = ni;
      } else {
        hr[k] = qr[k] * hr[k] + pu;
      }
    }
    if (!A.before) {
#pragma unroll
      for (int k = 0; k < kNPT; ++k) acc += CPLX ? (cr[k] * hr[k] - ci[k] * hi[k]) : cr[k] * hr[k];
    }
    acc = unit_sum(acc, A.TPR);
    if (ns == 0 && live) {
      const int t = A.reverse ? A.L - 1 - tau : tau;
      const size_t oa = ((size_t)b * A.L + t) * A.D + d;
      if (A.acc_in) acc += A.acc_in[oa];
      if (A.acc_out) {
        A.acc_out[oa] = acc;
      } else {
        float xr = 0.f;
        if (A.omega) xr = to_float(((const T*)A.x)[b * A.sxb + d * A.sxd + t * A.sxl]);
        ((T*)A.y)[b * A.syb + d * A.syd + t * A.syl] = from_float<T>(acc + om * xr);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// The same two passes for activations whose time axis is contiguous ([B, D, L] rows): the units of
// a workgroup (unit = one chunk of one row, TPR lanes) are consecutive (row, chunk) pairs, their
// samples are staged through LDS one sub-tile of steps at a time with loads and stores that run along
// time, and the partial sums of earlier pass sets are kept as [B, D, L] as well.
// A sub-tile is 64 steps (32 when the chunks are no longer than that, or when a unit is a single
// lane and a workgroup holds 256 units).
constexpr int kUnitWords = 7;      // 32-bit words of the unit map per unit
__host__ __device__ inline int rows_ts_log2(int tpr, int tc) { return tpr >= 2 && tc > 32 ? 6 : 5; }
__host__ __device__ inline size_t rows_lds_bytes(int tpr, int tc) {
  const int U = kBlock / tpr;
  return (size_t)U * ((1 << rows_ts_log2(tpr, tc)) + 1 + kUnitWords) * 4;
}

struct UnitMap {
  float* tile;     // [U][pitch], pitch = ts + 1: the units of a wave fall into different banks
  int64_t* uxo;    // offset of the unit's row in x (time stride 1), and in y
  int64_t* uyo;
  int* ub;
  int* ud;
  int* ut0;
  int U, tsl, ts, pitch;
};

__device__ __forceinline__ UnitMap unit_map(const PassArgs& A, float* lds, int lanes, int tsl) {
  UnitMap m;
  m.U = kBlock / lanes;
  m.tsl = tsl;
  m.ts = 1 << m.tsl;
  m.pitch = m.ts + 1;
  m.tile = lds;
  m.uxo = (int64_t*)(lds + (size_t)m.U * m.pitch);       // U is a multiple of 32: 8-byte aligned
  m.uyo = m.uxo + m.U;
  m.ub = (int*)(m.uyo + m.U);
  m.ud = m.ub + m.U;
  m.ut0 = m.ud + m.U;
  const int64_t units = (int64_t)A.B * A.D * A.nchunks;
  for (int u = threadIdx.x; u < m.U; u += kBlock) {
    const int64_t g = (int64_t)blockIdx.x * m.U + u;
    int b = 0, d = 0, t0 = -1;
    if (g < units) {
      const int64_t row = g / A.nchunks;
      b = (int)(row / A.D);
      d = (int)(row % A.D);
      t0 = (int)(g % A.nchunks) * A.Tc;
    }
    m.ub[u] = b;
    m.ud[u] = d;
    m.ut0[u] = t0;
    m.uxo[u] = b * A.sxb + d * A.sxd;
    m.uyo[u] = b * A.syb + d * A.syd;
  }
  return m;
}

// logical sample tau of the (delayed, masked) filter input of a time-contiguous row at offset xo
template <typename T>
__device__ __forceinline__ float load_row_u(const PassArgs& A, int64_t xo, int b, int tau) {
  const int ts = tau - A.tshift;
  if (ts < 0) return 0.f;
  const int t = A.reverse ? A.L - 1 - ts : ts;
  const T v = ((const T*)A.x)[xo + t];
  const uint8_t pad = A.mask ? A.mask[(size_t)b * A.L + t] : (uint8_t)0;
  return pad ? 0.f : to_float(v);
}

// logical steps of the unit that fall into the sub-tile starting s0 steps into the chunk
__device__ __forceinline__ int unit_steps(const PassArgs& A, const UnitMap& m, int t0, int s0) {
  if (t0 < 0) return 0;
  const int n = min(A.Tc - s0, A.L - (t0 + s0));
  return n < 0 ? 0 : (n > m.ts ? m.ts : n);
}

// values that are the same in every lane of a wave, moved to scalar registers
__device__ __forceinline__ int uniform_i32(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int64_t uniform_i64(int64_t v) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}
constexpr int kWaves = kBlock / 64;
constexpr int kUnitBatch = 8;        // units per wave whose loads are in flight together (U / kWaves is a multiple)

// y = sums + omega x for 64-step sub-tiles: the store phase of the single-sub-tile kernels, one unit
// per wave and pass (wave-uniform unit entries as in stage_inputs)
template <typename T>
__device__ __forceinline__ void store_outputs64(const PassArgs& A, const UnitMap& m, const float* sums) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int ub = 0; ub < m.U / kWaves; ub += kUnitBatch) {
    float acc[kUnitBatch], xr[kUnitBatch], om[kUnitBatch];
#pragma unroll
    for (int j = 0; j < kUnitBatch; ++j) {
      const int u = (ub + j) * kWaves + wave;
      const int t0 = uniform_i32(m.ut0[u]);
      acc[j] = sums[u * m.pitch + lane];
      xr[j] = 0.f;
      om[j] = 0.f;
      if (lane < unit_steps(A, m, t0, 0)) {
        om[j] = A.omega[uniform_i32(m.ud[u])];
        xr[j] = to_float(((const T*)A.x)[uniform_i64(m.uxo[u]) + t0 + lane]);
      }
    }
#pragma unroll
    for (int j = 0; j < kUnitBatch; ++j) {
      const int u = (ub + j) * kWaves + wave;
      const int t0 = uniform_i32(m.ut0[u]);
      if (lane < unit_steps(A, m, t0, 0))
        ((T*)A.y)[uniform_i64(m.uyo[u]) + t0 + lane] = from_float<T>(acc[j] + om[j] * xr[j]);
    }
  }
}

// samples beyond a unit's steps are staged as zeros; a thread's elements go in batches whose loads
// are all issued before the first of them is used
constexpr int kStageBatch = 8;       // elements per thread and batch of the store phases
constexpr int kLoadBatch = 16;       // of the staging loads

template <typename T>
__device__ __forceinline__ void stage_inputs(const PassArgs& A, const UnitMap& m, int s0) {
  if (m.tsl == 6) {
    // a wave covers one unit per pass: the unit's entries of the map are wave-uniform (scalar
    // registers), a lane only adds its own step to the addresses
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int ub = 0; ub < m.U / kWaves; ub += kUnitBatch) {
      float v[kUnitBatch];
#pragma unroll
      for (int j = 0; j < kUnitBatch; ++j) {
        const int u = (ub + j) * kWaves + wave;
        const int t0 = uniform_i32(m.ut0[u]);
        v[j] = 0.f;
        if (lane < unit_steps(A, m, t0, s0))
          v[j] = load_row_u<T>(A, uniform_i64(m.uxo[u]), uniform_i32(m.ub[u]), t0 + s0 + lane);
      }
#pragma unroll
      for (int j = 0; j < kUnitBatch; ++j) m.tile[((ub + j) * kWaves + wave) * m.pitch + lane] = v[j];
    }
    return;
  }
  const int per_thread = (m.U << m.tsl) / kBlock;          // ts / TPR: 4 or a multiple of the batch
  for (int e0 = 0; e0 < per_thread; e0 += kLoadBatch) {
    float v[kLoadBatch];
#pragma unroll
    for (int j = 0; j < kLoadBatch; ++j) {
      const int i = (e0 + j) * kBlock + threadIdx.x;
      const int u = i >> m.tsl, off = i & (m.ts - 1);
      const int t0 = e0 + j < per_thread ? m.ut0[u] : -1;
      v[j] = 0.f;
      if (e0 + j < per_thread && off < unit_steps(A, m, t0, s0))
        v[j] = load_row_u<T>(A, m.uxo[u], m.ub[u], t0 + s0 + off);
    }
#pragma unroll
    for (int j = 0; j < kLoadBatch; ++j) {
      const int i = (e0 + j) * kBlock + threadIdx.x;
      if (e0 + j < per_thread) m.tile[(i >> m.tsl) * m.pitch + (i & (m.ts - 1))] = v[j];
    }
  }
}

constexpr int kStepBlock = 8;      // steps whose samples are fetched from LDS together

template <typename T, bool CPLX>
__global__ __launch_bounds__(kBlock) void chunk_state_rows_kernel(const PassArgs A) {
  extern __shared__ float lds[];
  const UnitMap m = unit_map(A, lds, A.TPR, rows_ts_log2(A.TPR, A.Tc));
  __syncthreads();
  const int u = threadIdx.x / A.TPR, ns = threadIdx.x % A.TPR;
  const int t0 = m.ut0[u], d = m.ud[u], b = m.ub[u];
  float qr[kNPT], qi[kNPT], hr[kNPT], hi[kNPT];
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    const size_t o = ((size_t)d * A.NP + ns * kNPT + k) * 2;
    qr[k] = A.coef.q[o];
    qi[k] = CPLX ? A.coef.q[o + 1] : 0.f;
    hr[k] = 0.f;
    hi[k] = 0.f;
  }
  for (int s0 = 0; s0 < A.Tc; s0 += m.ts) {
    stage_inputs<T>(A, m, s0);
    __syncthreads();
    const int steps = unit_steps(A, m, t0, s0);
    const float* row = m.tile + u * m.pitch;
    for (int i0 = 0; i0 < steps; i0 += kStepBlock) {
      float xs[kStepBlock];
#pragma unroll
      for (int j = 0; j < kStepBlock; ++j) xs[j] = row[i0 + j];      // inside the row: ts is a multiple of the block
#pragma unroll
      for (int j = 0; j < kStepBlock; ++j) {
        if (i0 + j < steps) {                                        // the state must not run past the last step
#pragma unroll
          for (int k = 0; k < kNPT; ++k) {
            if (CPLX) {
              const float nr = qr[k] * hr[k] - qi[k] * hi[k] + xs[j];
              const float ni = qr[k] * hi[k] + qi[k] * hr[k];
              hr[k] = nr;
              hi[k] = ni;
            } else {
              hr[k] = qr[k] * hr[k] + xs[j];
            }
          }
        }
      }
    }
    __syncthreads();
  }
  if (t0 < 0) return;
  const int c = t0 / A.Tc;
  float* sp = A.st + ((((size_t)b * A.nchunks + c) * A.D + d) * A.NP + ns * kNPT) * 2;
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    sp[2 * k] = hr[k];
    sp[2 * k + 1] = hi[k];
  }
}

template <typename T, bool CPLX>
__global__ __launch_bounds__(kBlock) void chunk_apply_rows_kernel(const PassArgs A) {
  extern __shared__ float lds[];
  const UnitMap m = unit_map(A, lds, A.TPR, rows_ts_log2(A.TPR, A.Tc));
  __syncthreads();
  const int u = threadIdx.x / A.TPR, ns = threadIdx.x % A.TPR;
  const int t0 = m.ut0[u], d = m.ud[u], b = m.ub[u];
  float qr[kNPT], qi[kNPT], cr[kNPT], ci[kNPT], pp[kNPT], hr[kNPT], hi[kNPT];
  const int c = t0 < 0 ? 0 : t0 / A.Tc;
  const float* sp = A.st + ((((size_t)b * A.nchunks + c) * A.D + d) * A.NP + ns * kNPT) * 2;
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    const size_t o = ((size_t)d * A.NP + ns * kNPT + k) * 2;
    qr[k] = A.coef.q[o];
    qi[k] = CPLX ? A.coef.q[o + 1] : 0.f;
    cr[k] = A.coef.c[o];
    ci[k] = CPLX ? A.coef.c[o + 1] : 0.f;
    pp[k] = A.coef.p[o / 2];
    hr[k] = sp[2 * k];
    hi[k] = sp[2 * k + 1];
  }
  for (int s0 = 0; s0 < A.Tc; s0 += m.ts) {
    stage_inputs<T>(A, m, s0);
    __syncthreads();
    const int steps = unit_steps(A, m, t0, s0);
    float* row = m.tile + u * m.pitch;
    // whole blocks of steps: the zeros staged past the last step only touch a state that is not
    // used again (a short sub-tile is the unit's last) and outputs that the store below skips
    for (int i0 = 0; i0 < steps; i0 += kStepBlock) {
      float xs[kStepBlock];
#pragma unroll
      for (int j = 0; j < kStepBlock; ++j) xs[j] = row[i0 + j];
#pragma unroll
      for (int j = 0; j < kStepBlock; ++j) {
        float acc = 0.f;
        if (A.before) {
#pragma unroll
          for (int k = 0; k < kNPT; ++k) acc += CPLX ? (cr[k] * hr[k] - ci[k] * hi[k]) : cr[k] * hr[k];
        }
#pragma unroll
        for (int k = 0; k < kNPT; ++k) {
          const float pu = pp[k] * xs[j];
          if (CPLX) {
            const float nr = qr[k] * hr[k] - qi[k] * hi[k] + pu;
            const float ni = qr[k] * hi[k] + qi[k] * hr[k];
            hr[k] = nr;
            hi[k] = ni;
          } else {
            hr[k] = qr[k] * hr[k] + pu;
          }
        }
        if (!A.before) {
#pragma unroll
          for (int k = 0; k < kNPT; ++k) acc += CPLX ? (cr[k] * hr[k] - ci[k] * hi[k]) : cr[k] * hr[k];
        }
        xs[j] = unit_sum(acc, A.TPR);
      }
      if (ns == 0) {                      // the samples of these steps have been consumed by every lane of the unit
#pragma unroll
        for (int j = 0; j < kStepBlock; ++j) row[i0 + j] = xs[j];
      }
    }
    __syncthreads();
    const int per_thread = (m.U << m.tsl) / kBlock;
    for (int e0 = 0; e0 < per_thread; e0 += kStageBatch) {
      float acc[kStageBatch], xr[kStageBatch], om[kStageBatch];
      int64_t oy[kStageBatch];
      size_t oa[kStageBatch];
      bool on[kStageBatch];
#pragma unroll
      for (int j = 0; j < kStageBatch; ++j) {
        const int i = (e0 + j) * kBlock + threadIdx.x;
        const int uu = i >> m.tsl, off = i & (m.ts - 1);
        const bool mine = e0 + j < per_thread;
        const int tt0 = mine ? m.ut0[uu] : -1;
        on[j] = mine && off < unit_steps(A, m, tt0, s0);
        const int tau = tt0 + s0 + off;
        const int t = A.reverse ? A.L - 1 - tau : tau;
        const int bb = mine ? m.ub[uu] : 0, dd = mine ? m.ud[uu] : 0;
        acc[j] = mine ? m.tile[uu * m.pitch + off] : 0.f;
        oa[j] = ((size_t)bb * A.D + dd) * A.L + t;
        oy[j] = (mine ? m.uyo[uu] : 0) + t;
        xr[j] = 0.f;
        om[j] = 0.f;
        if (on[j]) {
          if (A.acc_in) acc[j] += A.acc_in[oa[j]];
          if (!A.acc_out && A.omega) {
            om[j] = A.omega[dd];
            xr[j] = to_float(((const T*)A.x)[m.uxo[uu] + t]);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < kStageBatch; ++j) {
        if (!on[j]) continue;
        if (A.acc_out) A.acc_out[oa[j]] = acc[j];
        else ((T*)A.y)[oy[j]] = from_float<T>(acc[j] + om[j] * xr[j]);
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------------
// Two-sided layers on time-contiguous rows whose chunks fit one sub-tile: both directions share the
// staged samples.  The direction that runs back in time uses the same chunk boundaries as the forward
// one (its chunk j is the forward chunk nchunks - 1 - j, walked from its last sample to its first);
// the only chunk that can be short is then the first it meets, where the state is still zero, so the
// scan's uniform factor q^Tc holds for it as well.  `rc`, `st_r`: coefficients and chunk states of
// that direction; `before`: its output at a sample excludes the sample itself (fftconv.py:85-100
// with shift).
__host__ __device__ inline size_t bidir_lds_bytes(int tpr, int tc) {
  const int U = kBlock / tpr;
  return (size_t)U * (2 * ((1 << rows_ts_log2(tpr, tc)) + 1) + kUnitWords) * 4;
}

// h <- q h + x (the imaginary parts are untouched for real coefficients)
template <bool CPLX>
__device__ __forceinline__ void state_step(float qr, float qi, float& hr, float& hi, float x) {
  if (CPLX) {
    const float nr = qr * hr - qi * hi + x;
    hi = qr * hi + qi * hr;
    hr = nr;
  } else {
    hr = fmaf(qr, hr, x);
  }
}

template <typename T, bool CPLX>
__global__ __launch_bounds__(kBlock) void bidir_state_rows_kernel(const PassArgs A, const PassCoef rc,
                                                                  float* __restrict__ st_r) {
  extern __shared__ float lds[];
  const UnitMap m = unit_map(A, lds, A.TPR, rows_ts_log2(A.TPR, A.Tc));
  __syncthreads();
  const int u = threadIdx.x / A.TPR, ns = threadIdx.x % A.TPR;
  const int t0 = m.ut0[u], d = m.ud[u], b = m.ub[u];
  float fr[kNPT], fi[kNPT], br[kNPT], bi[kNPT], hr[kNPT], hi[kNPT], gr[kNPT], gi[kNPT];
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    const int64_t o = coef_at(A.coef, d, ns * kNPT + k);
    fr[k] = o >= 0 ? A.coef.q[o * 2] : 0.f;
    fi[k] = CPLX && o >= 0 ? A.coef.q[o * 2 + 1] : 0.f;
    br[k] = o >= 0 ? rc.q[o * 2] : 0.f;
    bi[k] = CPLX && o >= 0 ? rc.q[o * 2 + 1] : 0.f;
    hr[k] = hi[k] = gr[k] = gi[k] = 0.f;
  }
  stage_inputs<T>(A, m, 0);
  __syncthreads();
  const int steps = unit_steps(A, m, t0, 0);
  const float* row = m.tile + u * m.pitch;
  // whole blocks of steps run unguarded; the block that holds the last step checks every step
  const int whole = steps / kStepBlock * kStepBlock;
  for (int i0 = 0; i0 < steps; i0 += kStepBlock) {
    float xs[kStepBlock];
#pragma unroll
    for (int j = 0; j < kStepBlock; ++j) xs[j] = row[i0 + j];
    if (i0 < whole) {
#pragma unroll
      for (int j = 0; j < kStepBlock; ++j)
#pragma unroll
        for (int k = 0; k < kNPT; ++k) state_step<CPLX>(fr[k], fi[k], hr[k], hi[k], xs[j]);
    } else {
#pragma unroll
      for (int j = 0; j < kStepBlock; ++j)
        if (i0 + j < steps) {
#pragma unroll
          for (int k = 0; k < kNPT; ++k) state_step<CPLX>(fr[k], fi[k], hr[k], hi[k], xs[j]);
        }
    }
  }
  for (int i0 = ((steps - 1) / kStepBlock) * kStepBlock; i0 >= 0 && steps > 0; i0 -= kStepBlock) {
    float xs[kStepBlock];
#pragma unroll
    for (int j = 0; j < kStepBlock; ++j) xs[j] = row[i0 + j];
    if (i0 < whole) {
#pragma unroll
      for (int j = kStepBlock - 1; j >= 0; --j)
#pragma unroll
        for (int k = 0; k < kNPT; ++k) state_step<CPLX>(br[k], bi[k], gr[k], gi[k], xs[j]);
    } else {
#pragma unroll
      for (int j = kStepBlock - 1; j >= 0; --j)
        if (i0 + j < steps) {
#pragma unroll
          for (int k = 0; k < kNPT; ++k) state_step<CPLX>(br[k], bi[k], gr[k], gi[k], xs[j]);
        }
    }
  }
  if (t0 < 0) return;
  const int c = t0 / A.Tc;
  float* sf = A.st + ((((size_t)b * A.nchunks + c) * A.D + d) * A.NP + ns * kNPT) * 2;
  float* sr = st_r + ((((size_t)b * A.nchunks + (A.nchunks - 1 - c)) * A.D + d) * A.NP + ns * kNPT) * 2;
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    sf[2 * k] = hr[k];
    sf[2 * k + 1] = hi[k];
    sr[2 * k] = gr[k];
    sr[2 * k + 1] = gi[k];
  }
}

// One direction of the apply pass over the unit's staged samples (ASC: forward in time, its outputs
// are stored to out[]; otherwise from the last sample to the first, added to out[]).  The state is
// carried as h / p, so a step is h <- q h + x and the output coefficient is c p: one multiply per
// state and step less (padded states have p = c = 0 and stay zero).
template <bool CPLX, bool ASC, bool BEFORE>
__device__ __forceinline__ void bidir_sweep(const PassCoef& cf, const float* st, int d, int NP, int ns, int tpr,
                                            const float* row, float* out, int steps) {
  float qr[kNPT], qi[kNPT], cr[kNPT], ci[kNPT], hr[kNPT], hi[kNPT];
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    const int64_t o = coef_at(cf, d, ns * kNPT + k);
    qr[k] = o >= 0 ? cf.q[o * 2] : 0.f;
    qi[k] = CPLX && o >= 0 ? cf.q[o * 2 + 1] : 0.f;
    const float p = o >= 0 ? cf.p[o] : 0.f;
    const float ip = p != 0.f ? 1.0f / p : 0.f;
    cr[k] = o >= 0 ? cf.c[o * 2] * p : 0.f;
    ci[k] = CPLX && o >= 0 ? cf.c[o * 2 + 1] * p : 0.f;
    hr[k] = st[2 * k] * ip;
    hi[k] = CPLX ? st[2 * k + 1] * ip : 0.f;
  }
  if (steps <= 0) return;
  const int last = ((steps - 1) / kStepBlock) * kStepBlock;
  for (int i0 = ASC ? 0 : last; ASC ? i0 <= last : i0 >= 0; i0 += ASC ? kStepBlock : -kStepBlock) {
    float xs[kStepBlock];
#pragma unroll
    for (int j = 0; j < kStepBlock; ++j) xs[j] = row[i0 + j];
    // walking back, the zeros staged past the last step come first: they must leave the state alone
    const bool tail = !ASC && i0 == last;
#pragma unroll
    for (int jj = 0; jj < kStepBlock; ++jj) {
      const int j = ASC ? jj : kStepBlock - 1 - jj;
      float acc = 0.f;
      if (BEFORE) {
#pragma unroll
        for (int k = 0; k < kNPT; ++k) acc += CPLX ? (cr[k] * hr[k] - ci[k] * hi[k]) : cr[k] * hr[k];
      }
      if (!tail || i0 + j < steps) {
#pragma unroll
        for (int k = 0; k < kNPT; ++k) state_step<CPLX>(qr[k], qi[k], hr[k], hi[k], xs[j]);
      }
      if (!BEFORE) {
#pragma unroll
        for (int k = 0; k < kNPT; ++k) acc += CPLX ? (cr[k] * hr[k] - ci[k] * hi[k]) : cr[k] * hr[k];
      }
      xs[j] = unit_sum(acc, tpr);
    }
    if (ns == 0) {
#pragma unroll
      for (int j = 0; j < kStepBlock; ++j) {
        if (ASC) out[i0 + j] = xs[j];
        else out[i0 + j] += xs[j];
      }
    }
  }
}

template <typename T, bool CPLX>
__global__ __launch_bounds__(kBlock) void bidir_apply_rows_kernel(const PassArgs A, const PassCoef rc,
                                                                  const float* __restrict__ st_r, const int before) {
  extern __shared__ float lds[];
  UnitMap m = unit_map(A, lds + (size_t)(kBlock / A.TPR) * ((1 << rows_ts_log2(A.TPR, A.Tc)) + 1), A.TPR,
                       rows_ts_log2(A.TPR, A.Tc));
  float* outs = lds;                      // [U][pitch] sums of both directions (every step that is read back
  __syncthreads();                        // is first stored by the forward sweep); the samples follow it
  const int u = threadIdx.x / A.TPR, ns = threadIdx.x % A.TPR;
  const int t0 = m.ut0[u], d = m.ud[u], b = m.ub[u];
  const int c = t0 < 0 ? 0 : t0 / A.Tc;
  stage_inputs<T>(A, m, 0);
  __syncthreads();
  const int steps = unit_steps(A, m, t0, 0);
  const float* row = m.tile + u * m.pitch;
  float* out = outs + u * m.pitch;
  const size_t so = (((size_t)b * A.nchunks) * A.D + d) * A.NP + ns * kNPT;
  const size_t cs = (size_t)A.D * A.NP;
  bidir_sweep<CPLX, true, false>(A.coef, A.st + (so + (size_t)c * cs) * 2, d, A.NP, ns, A.TPR, row, out, steps);
  const float* sr = st_r + (so + (size_t)(A.nchunks - 1 - c) * cs) * 2;
  if (before) bidir_sweep<CPLX, false, true>(rc, sr, d, A.NP, ns, A.TPR, row, out, steps);
  else bidir_sweep<CPLX, false, false>(rc, sr, d, A.NP, ns, A.TPR, row, out, steps);
  __syncthreads();
  if (m.tsl == 6) {
    store_outputs64<T>(A, m, outs);
    return;
  }
  const int per_thread = (m.U << m.tsl) / kBlock;
  for (int e0 = 0; e0 < per_thread; e0 += kStageBatch) {
    float acc[kStageBatch], xr[kStageBatch], om[kStageBatch];
    int64_t oy[kStageBatch];
    bool on[kStageBatch];
#pragma unroll
    for (int j = 0; j < kStageBatch; ++j) {
      const int i = (e0 + j) * kBlock + threadIdx.x;
      const int uu = i >> m.tsl, off = i & (m.ts - 1);
      const bool mine = e0 + j < per_thread;
      const int tt0 = mine ? m.ut0[uu] : -1;
      on[j] = mine && off < unit_steps(A, m, tt0, 0);
      const int t = tt0 + off;
      const int dd = mine ? m.ud[uu] : 0;
      acc[j] = mine ? outs[uu * m.pitch + off] : 0.f;
      oy[j] = (mine ? m.uyo[uu] : 0) + t;
      xr[j] = 0.f;
      om[j] = 0.f;
      if (on[j]) {
        om[j] = A.omega[dd];
        xr[j] = to_float(((const T*)A.x)[m.uxo[uu] + t]);
      }
    }
#pragma unroll
    for (int j = 0; j < kStageBatch; ++j)
      if (on[j]) ((T*)A.y)[oy[j]] = from_float<T>(acc[j] + om[j] * xr[j]);
  }
}

// ---------------------------------------------------------------------------------------------
// One-sided layers on time-contiguous rows short enough that all chunks of a row are units of one
// workgroup (L <= 64 * U): the three passes in one kernel.  Chunk sums meet in LDS, every unit folds
// the sums of the row's earlier chunks into its start state (all of them whole chunks), then runs the
// recurrence over the samples that are still staged.  A.Tc is the sub-tile length and A.nchunks a
// power of two that divides the units of a workgroup, so a workgroup holds whole rows.
__host__ __device__ inline size_t fused_lds_bytes(int tpr, int tsl) {
  const int U = kBlock / tpr;
  return ((size_t)U * ((1 << tsl) + 1 + kUnitWords) + (size_t)kBlock * kNPT * 2) * 4;
}

// The coefficients come straight from the caller's arrays (p [D, N], q and gamma [D, N, 2]); states
// beyond N are zero.
template <typename T, bool CPLX>
__global__ __launch_bounds__(kBlock) void ema_rows_fused_kernel(const PassArgs A, const int tsl,
                                                                const float* __restrict__ p_raw,
                                                                const float* __restrict__ q_raw,
                                                                const float* __restrict__ g_raw) {
  extern __shared__ float lds[];
  const UnitMap m = unit_map(A, lds, A.TPR, tsl);
  float* agg = (float*)(m.ut0 + m.U);                 // [kBlock][kNPT][2] chunk sums
  __syncthreads();
  const int u = threadIdx.x / A.TPR, ns = threadIdx.x % A.TPR;
  const int t0 = m.ut0[u], d = m.ud[u], b = m.ub[u];
  float qr[kNPT], qi[kNPT], cr[kNPT], ci[kNPT], pp[kNPT], hr[kNPT], hi[kNPT];
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    const int n = ns * kNPT + k;
    const bool real_state = n < A.N;
    const size_t o = ((size_t)d * A.N + (real_state ? n : 0)) * 2;
    qr[k] = real_state ? q_raw[o] : 0.f;
    qi[k] = CPLX && real_state ? q_raw[o + 1] : 0.f;
    cr[k] = real_state ? g_raw[o] : 0.f;
    ci[k] = CPLX && real_state ? g_raw[o + 1] : 0.f;
    pp[k] = real_state ? p_raw[o / 2] : 0.f;
    hr[k] = 0.f;
    hi[k] = 0.f;
  }
  stage_inputs<T>(A, m, 0);
  __syncthreads();
  const int steps = unit_steps(A, m, t0, 0);
  const int whole = steps / kStepBlock * kStepBlock;
  float* row = m.tile + u * m.pitch;
  // chunk sums from a zero start
  for (int i0 = 0; i0 < steps; i0 += kStepBlock) {
    float xs[kStepBlock];
#pragma unroll
    for (int j = 0; j < kStepBlock; ++j) xs[j] = row[i0 + j];
#pragma unroll
    for (int j = 0; j < kStepBlock; ++j)
      if (i0 < whole || i0 + j < steps) {
#pragma unroll
        for (int k = 0; k < kNPT; ++k) state_step<CPLX>(qr[k], qi[k], hr[k], hi[k], xs[j]);
      }
  }
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    agg[(threadIdx.x * kNPT + k) * 2] = hr[k];
    agg[(threadIdx.x * kNPT + k) * 2 + 1] = hi[k];
  }
  __syncthreads();
  // start state: the carried state pushed through the row's earlier chunks
  const int cidx = u & (A.nchunks - 1);
#pragma unroll
  for (int k = 0; k < kNPT; ++k) {
    const int n = ns * kNPT + k;
    float sr = 0.f, si = 0.f;
    if (A.h_in && n < A.N && t0 >= 0) {
      const size_t oh = (((size_t)b * A.D + d) * A.N + n) * 2;
      sr = A.h_in[oh];
      si = CPLX ? A.h_in[oh + 1] : 0.f;
    }
    double Qr, Qi;
    cpow_int((double)qr[k], (double)qi[k], A.Tc, &Qr, &Qi);
    const float fQr = (float)Qr, fQi = (float)Qi;
    for (int j = 0; j < cidx; ++j) {
      const float* a = agg + ((size_t)(threadIdx.x - (cidx - j) * A.TPR) * kNPT + k) * 2;
      const float nr = fQr * sr - fQi * si + pp[k] * a[0];
      const float ni = fQr * si + fQi * sr + pp[k] * a[1];
      sr = nr;
      si = ni;
    }
    hr[k] = sr;
    hi[k] = si;
  }
  // outputs; the state must be exact after the last step (it may be the carried state that is returned)
  for (int i0 = 0; i0 < steps; i0 += kStepBlock) {
    float xs[kStepBlock];
#pragma unroll
    for (int j = 0; j < kStepBlock; ++j) xs[j] = row[i0 + j];
#pragma unroll
    for (int j = 0; j < kStepBlock; ++j) {
      if (i0 < whole || i0 + j < steps) {
#pragma unroll
        for (int k = 0; k < kNPT; ++k) state_step<CPLX>(qr[k], qi[k], hr[k], hi[k], pp[k] * xs[j]);
      }
      float acc = 0.f;
#pragma unroll
      for (int k = 0; k < kNPT; ++k) acc += CPLX ? (cr[k] * hr[k] - ci[k] * hi[k]) : cr[k] * hr[k];
      xs[j] = unit_sum(acc, A.TPR);
    }
    if (ns == 0) {
#pragma unroll
      for (int j = 0; j < kStepBlock; ++j) row[i0 + j] = xs[j];
    }
  }
  if (A.h_out && t0 >= 0 && t0 < A.L && t0 + A.Tc >= A.L) {
#pragma unroll
    for (int k = 0; k < kNPT; ++k) {
      const int n = ns * kNPT + k;
      if (n < A.N) {
        const size_t oh = (((size_t)b * A.D + d) * A.N + n) * 2;
        A.h_out[oh] = hr[k];
        A.h_out[oh + 1] = hi[k];
      }
    }
  }
  __syncthreads();
  if (m.tsl == 6) {
    store_outputs64<T>(A, m, m.tile);
    return;
  }
  const int per_thread = (m.U << m.tsl) / kBlock;
  for (int e0 = 0; e0 < per_thread; e0 += kStageBatch) {
    float acc[kStageBatch], xr[kStageBatch], om[kStageBatch];
    int64_t oy[kStageBatch];
    bool on[kStageBatch];
#pragma unroll
    for (int j = 0; j < kStageBatch; ++j) {
      const int i = (e0 + j) * kBlock + threadIdx.x;
      const int uu = i >> m.tsl, off = i & (m.ts - 1);
      const bool mine = e0 + j < per_thread;
      const int tt0 = mine ? m.ut0[uu] : -1;
      on[j] = mine && off < unit_steps(A, m, tt0, 0);
      const int t = tt0 + off;
      acc[j] = mine ? m.tile[uu * m.pitch + off] : 0.f;
      oy[j] = (mine ? m.uyo[uu] : 0) + t;
      xr[j] = 0.f;
      om[j] = 0.f;
      if (on[j]) {
        om[j] = A.omega[m.ud[uu]];
        xr[j] = to_float(((const T*)A.x)[m.uxo[uu] + t]);
      }
    }
#pragma unroll
    for (int j = 0; j < kStageBatch; ++j)
      if (on[j]) ((T*)A.y)[oy[j]] = from_float<T>(acc[j] + om[j] * xr[j]);
  }
}

// builds the padded coefficient images of up to 4 pass sets:
//   set 0: forward rows [0,D)            set 1: forward tail  (c = -gamma q^Lk)
//   set 2: backward rows [D,2D)          set 3: backward tail
// `from_log`: q_or_logq holds log q (operator-level entry points) instead of q
__global__ void coef_prep_kernel(const float* __restrict__ p, const float* __restrict__ q_or_logq,
                                 const float* __restrict__ gamma, int from_log, int cplx, int D, int N,
                                 int NP, int nsets_dir, int64_t Lk, float* out) {
  // out layout per set: q [D,NP,2], c [D,NP,2], p [D,NP]
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t per = (int64_t)D * NP;
  if (gid >= per * nsets_dir) return;
  const int dir = (int)(gid / per);
  const int d = (int)((gid % per) / NP);
  const int n = (int)(gid % NP);
  const size_t setsz = (size_t)per * 5;
  float* o_full = out + (size_t)(2 * dir) * setsz;
  float* o_tail = out + (size_t)(2 * dir + 1) * setsz;
  const size_t oi = (size_t)d * NP + n;
  double qr = 0, qi = 0, gr = 0, gi = 0, pv = 0;
  if (n < N) {
    const size_t src = ((size_t)(dir * D + d) * N + n);
    const double a = q_or_logq[src * 2], bb = cplx ? q_or_logq[src * 2 + 1] : 0.0;
    if (from_log) {
      const double m = exp(a);
      qr = m * cos(bb);
      qi = m * sin(bb);
    } else {
      qr = a;
      qi = bb;
    }
    gr = gamma[src * 2];
    gi = cplx ? gamma[src * 2 + 1] : 0.0;
    pv = p ? p[src] : 1.0;
  }
  o_full[oi * 2] = (float)qr;
  o_full[oi * 2 + 1] = (float)qi;
  o_full[per * 2 + oi * 2] = (float)gr;
  o_full[per * 2 + oi * 2 + 1] = (float)gi;
  o_full[per * 4 + oi] = (float)pv;
  if (Lk > 0) {
    double tr, ti;
    cpow_int(qr, qi, Lk, &tr, &ti);
    o_tail[oi * 2] = (float)qr;
    o_tail[oi * 2 + 1] = (float)qi;
    o_tail[per * 2 + oi * 2] = (float)(-(gr * tr - gi * ti));
    o_tail[per * 2 + oi * 2 + 1] = (float)(-(gr * ti + gi * tr));
    o_tail[per * 4 + oi] = (float)pv;
  }
}

struct Plan {
  int NP, TPR, Tc, nchunks;
  size_t coef_bytes, st_bytes, acc_bytes, tile_bytes, image_bytes, rows_bytes, total;
};

Plan make_plan(int64_t B, int64_t D, int64_t N, int64_t L, int nsets, bool need_acc, bool bidirectional = false) {
  Plan pl;
  int tpr = 1;
  while (tpr * kNPT < N) tpr <<= 1;
  pl.TPR = tpr;
  pl.NP = tpr * kNPT;
  const int64_t rows = B * D * tpr;
  int64_t want = ceil_div(262144, rows > 0 ? rows : 1);
  int64_t maxc = ceil_div(L, 32);
  int64_t nch = want < 1 ? 1 : want;
  if (nch > maxc) nch = maxc;
  if (nch < 1) nch = 1;
  int64_t tc = ceil_div(L, nch);
  tc = ceil_div(tc, 8) * 8;
  if (tc < 1) tc = 1;
  pl.Tc = (int)tc;
  pl.nchunks = (int)ceil_div(L, tc);
  if (pl.nchunks < 1) pl.nchunks = 1;
  pl.coef_bytes = align_up((size_t)D * pl.NP * 5 * 4 * 4, 256);   // 4 sets
  // chunk states; a two-sided layer may keep both directions' at once
  pl.st_bytes = align_up((size_t)B * pl.nchunks * D * pl.NP * 2 * 4, 256) * (bidirectional ? 2 : 1);
  pl.acc_bytes = need_acc ? align_up((size_t)B * L * D * 4, 256) : 0;
  (void)nsets;
  pl.tile_bytes = align_up((size_t)B * D * 16 * 2 * 4, 256);      // state after the last whole tile
  pl.image_bytes = align_up(ema_image_bytes(D, N, bidirectional ? 1 : 0), 256);   // when the caller brings none
  pl.rows_bytes = align_up(ema_rows_record_bytes(B, D, L, bidirectional ? 1 : 0), 256);   // block end states of the rows path
  pl.total = pl.coef_bytes + pl.st_bytes + pl.acc_bytes + pl.tile_bytes + pl.image_bytes + pl.rows_bytes;
  return pl;
}

// lane groups per row of the chunk scan: enough that a group's run is a few load batches
inline int scan_groups(int NP, int nchunks) {
  int g = 1;
  while (g * NP < kBlock && g * 2 * kScanBatch <= nchunks) g <<= 1;
  return g;
}

template <typename T, bool CPLX>
int run_pass_set_t(PassArgs& A, bool state_only, hipStream_t s) {
  const int64_t tA = (int64_t)A.B * A.nchunks * A.D * A.TPR;
  // time-contiguous activations take the LDS-staged passes
  const bool rows = A.sxl == 1 && A.L > 1 && (state_only || A.syl == 1);
  const size_t lds = rows_lds_bytes(A.TPR, A.Tc);
  const dim3 gridA((unsigned)ceil_div(tA, kBlock));
  if (rows)
    hipLaunchKernelGGL((chunk_state_rows_kernel<T, CPLX>), gridA, dim3(kBlock), lds, s, A);
  else
    hipLaunchKernelGGL((chunk_state_kernel<T, CPLX>), gridA, dim3(kBlock), 0, s, A);
  const int G = scan_groups(A.NP, A.nchunks);
  const int rows_per_wg = kBlock / (A.NP * G);
  hipLaunchKernelGGL((chunk_scan_kernel<CPLX>), dim3((unsigned)ceil_div((int64_t)A.B * A.D, rows_per_wg)),
                     dim3(kBlock), 0, s, A, G);
  if (!state_only) {
    if (rows)
      hipLaunchKernelGGL((chunk_apply_rows_kernel<T, CPLX>), gridA, dim3(kBlock), lds, s, A);
    else
      hipLaunchKernelGGL((chunk_apply_kernel<T, CPLX>), gridA, dim3(kBlock), 0, s, A);
  }
  MEGA_CHECK_LAUNCH("ema pass");
  return MEGA_OK;
}

template <typename T>
int run_pass_set(PassArgs& A, bool cplx, bool state_only, hipStream_t s) {
  return cplx ? run_pass_set_t<T, true>(A, state_only, s) : run_pass_set_t<T, false>(A, state_only, s);
}

// one-sided, untruncated layers on short time-contiguous rows: one kernel (see ema_rows_fused_kernel)
inline bool fused_rows_plan(const PassArgs& A, int* tsl, int* nch) {
  if (!(A.sxl == 1 && A.syl == 1 && A.L > 1)) return false;
  const int U = kBlock / A.TPR;
  int l2 = 5;
  if ((int64_t)A.L > (int64_t)U << l2) l2 = A.TPR >= 2 ? 6 : 5;
  if ((int64_t)A.L > (int64_t)U << l2) return false;
  int n = 1;
  while (((int64_t)n << l2) < A.L) n <<= 1;
  *tsl = l2;
  *nch = n;
  return true;
}

template <typename T>
int run_fused_rows(PassArgs& A, bool cplx, int tsl, int nch, const float* p, const float* q, const float* gamma,
                   hipStream_t s) {
  A.Tc = 1 << tsl;
  A.nchunks = nch;
  const int U = kBlock / A.TPR;
  const dim3 grid((unsigned)ceil_div((int64_t)A.B * A.D * nch, U));
  const size_t lds = fused_lds_bytes(A.TPR, tsl);
  if (cplx) hipLaunchKernelGGL((ema_rows_fused_kernel<T, true>), grid, dim3(kBlock), lds, s, A, tsl, p, q, gamma);
  else hipLaunchKernelGGL((ema_rows_fused_kernel<T, false>), grid, dim3(kBlock), lds, s, A, tsl, p, q, gamma);
  MEGA_CHECK_LAUNCH("ema fused row pass");
  return MEGA_OK;
}

// both directions of a two-sided layer in three launches (state, scans, apply); see the kernels
inline bool bidir_rows_ok(const PassArgs& A) {
  return A.sxl == 1 && A.syl == 1 && A.L > 1 && A.Tc <= (1 << rows_ts_log2(A.TPR, A.Tc));
}

template <typename T, bool CPLX>
int run_bidir_rows_t(PassArgs& A, const PassCoef& rc, float* st_r, int before, hipStream_t s) {
  const int64_t tA = (int64_t)A.B * A.nchunks * A.D * A.TPR;
  const dim3 gridA((unsigned)ceil_div(tA, kBlock));
  hipLaunchKernelGGL((bidir_state_rows_kernel<T, CPLX>), gridA, dim3(kBlock), rows_lds_bytes(A.TPR, A.Tc), s, A, rc,
                     st_r);
  const int G = scan_groups(A.NP, A.nchunks);
  const int rows_per_wg = kBlock / (A.NP * G);
  const dim3 gridB((unsigned)ceil_div((int64_t)A.B * A.D, rows_per_wg), 2);
  PassArgs R = A;
  R.coef = rc;
  R.st = st_r;
  R.h_in = nullptr;
  R.h_out = nullptr;
  hipLaunchKernelGGL((chunk_scan2_kernel<CPLX>), gridB, dim3(kBlock), 0, s, A, R, G);
  hipLaunchKernelGGL((bidir_apply_rows_kernel<T, CPLX>), gridA, dim3(kBlock), bidir_lds_bytes(A.TPR, A.Tc), s, A, rc,
                     (const float*)st_r, before);
  MEGA_CHECK_LAUNCH("ema two-sided passes");
  return MEGA_OK;
}

int run_bidir_rows(int dtype, PassArgs& A, const PassCoef& rc, float* st_r, int before, bool cplx, hipStream_t s) {
#define MEGA_BIDIR(T) \
  return cplx ? run_bidir_rows_t<T, true>(A, rc, st_r, before, s) : run_bidir_rows_t<T, false>(A, rc, st_r, before, s)
  switch (dtype) {
    case MEGA_F32: MEGA_BIDIR(float);
    case MEGA_BF16: MEGA_BIDIR(bf16_t);
    default: MEGA_BIDIR(f16_t);
  }
#undef MEGA_BIDIR
}

int run_pass_set_dtype(int dtype, PassArgs& A, bool cplx, bool state_only, hipStream_t s) {
  switch (dtype) {
    case MEGA_F32: return run_pass_set<float>(A, cplx, state_only, s);
    case MEGA_BF16: return run_pass_set<bf16_t>(A, cplx, state_only, s);
    default: return run_pass_set<f16_t>(A, cplx, state_only, s);
  }
}

PassCoef coef_of(float* base, int set, int64_t D, int NP) {
  const size_t per = (size_t)D * NP;
  float* o = base + (size_t)set * per * 5;
  return PassCoef{o, o + per * 2, o + per * 4, NP};
}

// ---------------------------------------------------------------- single decode step
template <typename T, bool CPLX>
__global__ __launch_bounds__(kBlock) void ema_step_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                          const float* __restrict__ p,
                                                          const float* __restrict__ q,
                                                          const float* __restrict__ gamma,
                                                          const float* __restrict__ omega,
                                                          const float* h_in, float* h_out, int B, int D,
                                                          int N) {
  const int64_t gid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (gid >= (int64_t)B * D) return;
  const int d = (int)(gid % D);
  const float xv = to_float(x[gid]);
  float acc = 0.f;
  const size_t ho = (size_t)gid * N * 2;
  const size_t co = (size_t)d * N;
  for (int n = 0; n < N; ++n) {
    const float qr = q[(co + n) * 2], qi = CPLX ? q[(co + n) * 2 + 1] : 0.f;
    const float gr = gamma[(co + n) * 2], gi = CPLX ? gamma[(co + n) * 2 + 1] : 0.f;
    float hr = 0.f, hi = 0.f;
    if (h_in) {
      hr = h_in[ho + 2 * n];
      hi = CPLX ? h_in[ho + 2 * n + 1] : 0.f;
    }
    const float nr = qr * hr - qi * hi + p[co + n] * xv;
    const float ni = qr * hi + qi * hr;
    h_out[ho + 2 * n] = nr;
    h_out[ho + 2 * n + 1] = ni;
    acc += gr * nr - gi * ni;
  }
  y[gid] = from_float<T>(acc + omega[d] * xv);
}

// ---------------------------------------------------------------- materialised kernel / bias
// w[d,l] = Re sum_n p gamma exp(l log q); b[b,d,l] = Re sum_n gamma h exp((l+1) log q)
// (fairseq/csrc/ops/ema_parameters.cc:37-77).  One thread per (row, block of 16 lags): the
// block base power is taken from exp / sincos with the phase reduced in double, the 15
// following powers by multiplication.
constexpr int kLagBlock = 16;
__global__ __launch_bounds__(kBlock) void ema_kernel_bias_kernel(const float* __restrict__ p,
                                                                 const float* __restrict__ log_q,
                                                                 const float* __restrict__ gamma,
                                                                 const float* __restrict__ h, int B, int K,
                                                                 int N, int L, float* w, float* bias) {
  // rows: first K kernel rows, then B*K bias rows
  const int nblk = (L + kLagBlock - 1) / kLagBlock;
  const int64_t gid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t rows = (int64_t)K + (h ? (int64_t)B * K : 0);
  if (gid >= rows * nblk) return;
  const int blk = (int)(gid % nblk);
  const int64_t row = gid / nblk;
  const bool is_bias = row >= K;
  const int d = is_bias ? (int)((row - K) % K) : (int)row;
  const int64_t bd = is_bias ? row - K : 0;
  const int l0 = blk * kLagBlock;
  const int e0 = is_bias ? l0 + 1 : l0;
  float acc[kLagBlock];
#pragma unroll
  for (int i = 0; i < kLagBlock; ++i) acc[i] = 0.f;
  for (int n = 0; n < N; ++n) {
    const size_t o = ((size_t)d * N + n) * 2;
    const double lr = log_q[o], li = log_q[o + 1];
    double cr, ci;
    if (is_bias) {
      const size_t oh = ((size_t)bd * N + n) * 2;
      const double gr = gamma[o], gi = gamma[o + 1], hr = h[oh], hi = h[oh + 1];
      cr = gr * hr - gi * hi;
      ci = gr * hi + gi * hr;
    } else {
      cr = (double)p[o / 2] * gamma[o];
      ci = (double)p[o / 2] * gamma[o + 1];
    }
    const double mag = exp(lr * e0);
    double ang = li * e0;
    ang -= 6.283185307179586476925 * rint(ang * 0.15915494309189533577);
    double sn, cs;
    sincos(ang, &sn, &cs);
    // v = c q^{e0}
    float vr = (float)(mag * (cr * cs - ci * sn));
    float vi = (float)(mag * (cr * sn + ci * cs));
    const double m1 = exp(lr);
    double s1, c1;
    sincos(li, &s1, &c1);
    const float qr = (float)(m1 * c1), qi = (float)(m1 * s1);
#pragma unroll
    for (int i = 0; i < kLagBlock; ++i) {
      acc[i] += vr;
      const float t = vr * qr - vi * qi;
      vi = vr * qi + vi * qr;
      vr = t;
    }
  }
  float* out = is_bias ? bias + (size_t)bd * L : w + (size_t)d * L;
#pragma unroll
  for (int i = 0; i < kLagBlock; ++i)
    if (l0 + i < L) out[l0 + i] = acc[i];
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" size_t mega_ema_fwd_workspace_bytes(int64_t B, int64_t D, int64_t N, int64_t L,
                                               int bidirectional, int64_t truncation) {
  if (B <= 0 || D <= 0 || N <= 0 || L <= 0) return 256;
  const bool trunc = truncation > 0 && truncation < L;
  const bool need_acc = bidirectional || trunc;
  return make_plan(B, D, N, L, 4, need_acc, bidirectional != 0).total;
}

extern "C" size_t mega_ema_image_bytes(int64_t D, int64_t N, int bidirectional) {
  return ema_image_bytes(D, N, bidirectional);
}

extern "C" int mega_ema_prepare(const float* p, const float* q, const float* gamma, int is_complex,
                                const float* omega, int64_t D, int64_t N, int bidirectional, int shift,
                                void* image, size_t image_bytes, void* stream) {
  MEGA_REQUIRE(D > 0 && N > 0, MEGA_ERR_ARG, "ema_prepare: bad shape D=%ld N=%ld", (long)D, (long)N);
  const size_t need = ema_image_bytes(D, N, bidirectional);
  MEGA_REQUIRE(need > 0, MEGA_ERR_UNSUPPORTED, "ema_prepare: ndim=%ld has no operand image (ndim <= 16 only)", (long)N);
  MEGA_REQUIRE(p && q && gamma && omega && image, MEGA_ERR_ARG, "ema_prepare: null pointer argument");
  MEGA_REQUIRE(image_bytes >= need && ((uintptr_t)image % 16) == 0, MEGA_ERR_WORKSPACE,
               "ema_prepare: image of %zu bytes (16-byte aligned) needed", need);
  return ema_image_build(p, q, gamma, is_complex, omega, D, N, bidirectional, shift, image, (hipStream_t)stream);
}

extern "C" size_t mega_ema_hidden_workspace_bytes(int64_t B, int64_t D, int64_t N, int64_t L) {
  if (B <= 0 || D <= 0 || N <= 0 || L <= 0) return 256;
  return make_plan(B, D, N, L, 1, false).total;
}

static int check_common(const char* who, int dtype, int64_t B, int64_t D, int64_t N, int64_t L) {
  MEGA_REQUIRE(dtype == MEGA_F32 || dtype == MEGA_BF16 || dtype == MEGA_F16, MEGA_ERR_ARG, "%s: unknown dtype %d",
               who, dtype);
  MEGA_REQUIRE(B >= 0 && D > 0 && N > 0 && L >= 0, MEGA_ERR_ARG, "%s: bad shape B=%ld D=%ld N=%ld L=%ld", who,
               (long)B, (long)D, (long)N, (long)L);
  MEGA_REQUIRE(N <= 32, MEGA_ERR_UNSUPPORTED, "%s: ndim=%ld > 32 is not supported", who, (long)N);
  MEGA_REQUIRE(B * D * 8 < (int64_t)1 << 31 && L < (int64_t)1 << 30, MEGA_ERR_UNSUPPORTED, "%s: shape too large",
               who);
  return MEGA_OK;
}

extern "C" int mega_ema_fwd(const void* x, void* y, int dtype, int64_t sxb, int64_t sxd, int64_t sxl,
                            int64_t syb, int64_t syd, int64_t syl, const float* p, const float* q,
                            const float* gamma, int is_complex, const float* omega, const uint8_t* mask,
                            const float* h_in, float* h_out, int64_t B, int64_t D, int64_t N, int64_t L,
                            int bidirectional, int64_t truncation, int shift, const void* image,
                            void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_common("ema_fwd", dtype, B, D, N, L);
  if (rc) return rc;
  MEGA_REQUIRE(!(bidirectional && (h_in || h_out)), MEGA_ERR_ARG,
               "ema_fwd: bidirectional EMA does not support incremental state");
  if (B == 0 || L == 0) return MEGA_OK;
  MEGA_REQUIRE(x && y && p && q && gamma && omega, MEGA_ERR_ARG, "ema_fwd: null pointer argument");
  const int64_t Lk = (truncation > 0 && truncation < L) ? truncation : 0;
  MEGA_REQUIRE(!(Lk > 0 && (h_in || h_out)), MEGA_ERR_UNSUPPORTED,
               "ema_fwd: truncation together with incremental state is not supported");
  const bool need_acc = bidirectional || Lk > 0;
  const Plan pl = make_plan(B, D, N, L, 4, need_acc, bidirectional != 0);
  MEGA_REQUIRE(workspace && workspace_bytes >= pl.total, MEGA_ERR_WORKSPACE,
               "ema_fwd: workspace of %zu bytes needed", pl.total);
  hipStream_t s = (hipStream_t)stream;
  char* w = (char*)workspace;
  float* coef = (float*)w;
  float* st = (float*)(w + pl.coef_bytes);
  float* acc = need_acc ? (float*)(w + pl.coef_bytes + pl.st_bytes) : nullptr;
  float* h_tile = (float*)(w + pl.coef_bytes + pl.st_bytes + pl.acc_bytes);
  // [B, D, L] rows: fp32 / fp16 always, bf16 when the streaming kernel (one workgroup per 16 channels, the whole
  // sequence) would leave most of the chip idle
  const bool stream_ok = ema_mfma_covers(dtype, sxb, sxd, sxl, syb, syd, syl, x, y, mask, B, D, N, L, Lk);
  if (ema_rows_covers(dtype, sxb, sxd, sxl, syb, syd, syl, B, D, N, L, Lk, h_out) &&
      (!stream_ok || B * ceil_div(D, 16) < 128)) {
    const void* img = image;
    char* wimg = w + pl.coef_bytes + pl.st_bytes + pl.acc_bytes + pl.tile_bytes;
    if (!img) {
      rc = ema_image_build(p, q, gamma, is_complex, omega, D, N, bidirectional, shift, wimg, s,
                           (dtype == MEGA_BF16 ? kImgBf16 : kImgF16) | kImgBlocks);
      if (rc) return rc;
      img = wimg;
    }
    return ema_rows_run(x, y, dtype, sxb, sxd, syb, syd, img, is_complex, omega, mask, h_in, h_out, B, D, N, L,
                        bidirectional, acc, (float*)(wimg + pl.image_bytes), s);
  }
  // rows too long for the rows kernel (more than 16 blocks of 1024 tokens) with fewer than 16 channel blocks: the
  // streaming kernel would run on that many workgroups, the time-parallel vector-ALU passes below are quicker
  // (B1 x D64 x L65536 in bf16: 155 -> 77 us one-sided, 427 -> 102 us two-sided; from 16 channel blocks on they lose)
  const bool few_rows = sxl == 1 && syl == 1 && B * ceil_div(D, 16) < 16;
  if (stream_ok && !few_rows) {
    const void* img = image;
    if (!img) {
      // no cached image: kernel generation runs with every call
      void* wimg = w + pl.coef_bytes + pl.st_bytes + pl.acc_bytes + pl.tile_bytes;
      rc = ema_image_build(p, q, gamma, is_complex, omega, D, N, bidirectional, shift, wimg, s, kImgBf16 | kImgStream);
      if (rc) return rc;
      img = wimg;
    }
    rc = ema_mfma_try(x, y, dtype, sxb, sxd, sxl, syb, syd, syl, p, q, img, is_complex, omega, mask, h_in, h_out, B,
                      D, N, L, bidirectional, Lk, acc, h_tile, s);
    if (rc != 0) return rc < 0 ? rc : MEGA_OK;
  }
  if (!bidirectional && Lk == 0) {
    PassArgs A;
    A.x = x; A.sxb = sxb; A.sxd = sxd; A.sxl = sxl; A.mask = mask;
    A.coef = coef_of(coef, 0, D, pl.NP);
    A.h_in = h_in; A.h_out = h_out; A.st = st;
    A.B = (int)B; A.D = (int)D; A.N = (int)N; A.L = (int)L;
    A.NP = pl.NP; A.TPR = pl.TPR; A.Tc = pl.Tc; A.nchunks = pl.nchunks;
    A.reverse = 0; A.before = 0; A.tshift = 0;
    A.acc_in = nullptr; A.acc_out = nullptr;
    A.y = y; A.syb = syb; A.syd = syd; A.syl = syl;
    A.omega = omega;
    int tsl = 0, nch = 0;
    if (fused_rows_plan(A, &tsl, &nch)) {
      switch (dtype) {
        case MEGA_F32: return run_fused_rows<float>(A, is_complex != 0, tsl, nch, p, q, gamma, s);
        case MEGA_BF16: return run_fused_rows<bf16_t>(A, is_complex != 0, tsl, nch, p, q, gamma, s);
        default: return run_fused_rows<f16_t>(A, is_complex != 0, tsl, nch, p, q, gamma, s);
      }
    }
  }
  if (bidirectional && Lk == 0) {
    PassArgs A;
    A.x = x; A.sxb = sxb; A.sxd = sxd; A.sxl = sxl; A.mask = mask;
    // both directions read the caller's arrays: rows [0, D) run forward, rows [D, 2D) back in time
    A.coef = PassCoef{q, gamma, p, (int)N};
    A.h_in = nullptr; A.h_out = nullptr; A.st = st;
    A.B = (int)B; A.D = (int)D; A.N = (int)N; A.L = (int)L;
    A.NP = pl.NP; A.TPR = pl.TPR; A.Tc = pl.Tc; A.nchunks = pl.nchunks;
    A.reverse = 0; A.before = 0; A.tshift = 0;
    A.acc_in = nullptr; A.acc_out = nullptr;
    A.y = y; A.syb = syb; A.syd = syd; A.syl = syl;
    A.omega = omega;
    if (bidir_rows_ok(A))
      return run_bidir_rows(dtype, A, PassCoef{q + D * N * 2, gamma + D * N * 2, p + D * N, (int)N},
                            (float*)((char*)st + pl.st_bytes / 2), shift ? 1 : 0,
                            is_complex != 0, s);
  }
  const int ndir = bidirectional ? 2 : 1;
  {
    const int64_t n = (int64_t)D * pl.NP * ndir;
    hipLaunchKernelGGL(coef_prep_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s, p, q, gamma, 0,
                       is_complex ? 1 : 0, (int)D, (int)N, pl.NP, ndir, Lk, coef);
    MEGA_CHECK_LAUNCH("ema_fwd coefficient prep");
  }
  // list of pass sets; the last one writes y
  struct SetDesc { int set, reverse, before, tshift; };
  SetDesc sets[4];
  int ns = 0;
  if (bidirectional) {
    sets[ns++] = {2, 1, shift ? 1 : 0, 0};
    if (Lk > 0) sets[ns++] = {3, 1, shift ? 1 : 0, (int)Lk};
  }
  if (Lk > 0) sets[ns++] = {1, 0, 0, (int)Lk};
  sets[ns++] = {0, 0, 0, 0};
  for (int i = 0; i < ns; ++i) {
    PassArgs A;
    A.x = x; A.sxb = sxb; A.sxd = sxd; A.sxl = sxl; A.mask = mask;
    A.coef = coef_of(coef, sets[i].set, D, pl.NP);
    const bool main_set = sets[i].set == 0;
    A.h_in = main_set ? h_in : nullptr;
    A.h_out = main_set ? h_out : nullptr;
    A.st = st;
    A.B = (int)B; A.D = (int)D; A.N = (int)N; A.L = (int)L;
    A.NP = pl.NP; A.TPR = pl.TPR; A.Tc = pl.Tc; A.nchunks = pl.nchunks;
    A.reverse = sets[i].reverse; A.before = sets[i].before; A.tshift = sets[i].tshift;
    A.acc_in = i > 0 ? acc : nullptr;
    A.acc_out = i < ns - 1 ? acc : nullptr;
    A.y = y; A.syb = syb; A.syd = syd; A.syl = syl;
    A.omega = omega;
    rc = run_pass_set_dtype(dtype, A, is_complex != 0, false, s);
    if (rc) return rc;
  }
  return MEGA_OK;
}

extern "C" int mega_ema_hidden_fwd(const void* x, int dtype, int64_t sxb, int64_t sxd, int64_t sxl,
                                   const float* p, const float* log_q, const float* h, int64_t B, int64_t D,
                                   int64_t N, int64_t L, float* h_out, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  int rc = check_common("ema_hidden_fwd", dtype, B, D, N, L);
  if (rc) return rc;
  if (B == 0) return MEGA_OK;
  MEGA_REQUIRE(p && log_q && h_out && (L == 0 || x), MEGA_ERR_ARG, "ema_hidden_fwd: null pointer argument");
  hipStream_t s = (hipStream_t)stream;
  if (L == 0) {
    if (h) hipMemcpyAsync(h_out, h, (size_t)B * D * N * 8, hipMemcpyDeviceToDevice, s);
    else zero_async(h_out, (size_t)B * D * N * 8, s);
    return MEGA_OK;
  }
  const Plan pl = make_plan(B, D, N, L, 1, false);
  MEGA_REQUIRE(workspace && workspace_bytes >= pl.total, MEGA_ERR_WORKSPACE,
               "ema_hidden_fwd: workspace of %zu bytes needed", pl.total);
  char* w = (char*)workspace;
  float* coef = (float*)w;
  float* st = (float*)(w + pl.coef_bytes);
  const int64_t n = (int64_t)D * pl.NP;
  // gamma is not needed for the state; pass log_q as a stand-in that is never read as gamma
  hipLaunchKernelGGL(coef_prep_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, s, p, log_q, log_q, 1, 1,
                     (int)D, (int)N, pl.NP, 1, (int64_t)0, coef);
  MEGA_CHECK_LAUNCH("ema_hidden_fwd coefficient prep");
  PassArgs A;
  A.x = x; A.sxb = sxb; A.sxd = sxd; A.sxl = sxl; A.mask = nullptr;
  A.coef = coef_of(coef, 0, D, pl.NP);
  A.h_in = h; A.h_out = h_out; A.st = st;
  A.B = (int)B; A.D = (int)D; A.N = (int)N; A.L = (int)L;
  A.NP = pl.NP; A.TPR = pl.TPR; A.Tc = pl.Tc; A.nchunks = pl.nchunks;
  A.reverse = 0; A.before = 0; A.tshift = 0;
  A.acc_in = nullptr; A.acc_out = nullptr; A.y = nullptr; A.syb = A.syd = A.syl = 0; A.omega = nullptr;
  return run_pass_set_dtype(dtype, A, true, true, s);
}

extern "C" int mega_ema_step(const void* x, void* y, int dtype, const float* p, const float* q,
                             const float* gamma, int is_complex, const float* omega, const float* h_in,
                             float* h_out, int64_t B, int64_t D, int64_t N, void* stream) {
  int rc = check_common("ema_step", dtype, B, D, N, 1);
  if (rc) return rc;
  if (B == 0) return MEGA_OK;
  MEGA_REQUIRE(x && y && p && q && gamma && omega && h_out, MEGA_ERR_ARG, "ema_step: null pointer argument");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)ceil_div(B * D, kBlock));
#define LAUNCH_STEP(T, C)                                                                             \
  hipLaunchKernelGGL((ema_step_kernel<T, C>), grid, dim3(kBlock), 0, s, (const T*)x, (T*)y, p, q, gamma, \
                     omega, h_in, h_out, (int)B, (int)D, (int)N)
  if (is_complex) {
    if (dtype == MEGA_F32) LAUNCH_STEP(float, true);
    else if (dtype == MEGA_BF16) LAUNCH_STEP(bf16_t, true);
    else LAUNCH_STEP(f16_t, true);
  } else {
    if (dtype == MEGA_F32) LAUNCH_STEP(float, false);
    else if (dtype == MEGA_BF16) LAUNCH_STEP(bf16_t, false);
    else LAUNCH_STEP(f16_t, false);
  }
#undef LAUNCH_STEP
  MEGA_CHECK_LAUNCH("ema_step");
  return MEGA_OK;
}

extern "C" int mega_ema_parameters_fwd(const float* p, const float* log_q, const float* gamma, const float* h,
                                       int64_t B, int64_t K, int64_t N, int64_t L, float* w, float* b,
                                       void* stream) {
  MEGA_REQUIRE(K > 0 && N > 0 && L >= 0 && B >= 0, MEGA_ERR_ARG, "ema_parameters_fwd: bad shape");
  MEGA_REQUIRE(N <= 32, MEGA_ERR_UNSUPPORTED, "ema_parameters_fwd: ndim=%ld > 32 is not supported", (long)N);
  MEGA_REQUIRE(p && log_q && gamma && w, MEGA_ERR_ARG, "ema_parameters_fwd: null pointer argument");
  MEGA_REQUIRE(!h || b, MEGA_ERR_ARG, "ema_parameters_fwd: carried state given without a bias output");
  if (L == 0) return MEGA_OK;
  const int64_t rows = K + (h ? B * K : 0);
  const int64_t nblk = ceil_div(L, kLagBlock);
  MEGA_REQUIRE(rows * nblk < (int64_t)1 << 40, MEGA_ERR_UNSUPPORTED, "ema_parameters_fwd: shape too large");
  hipLaunchKernelGGL(ema_kernel_bias_kernel, dim3((unsigned)ceil_div(rows * nblk, kBlock)), dim3(kBlock), 0,
                     (hipStream_t)stream, p, log_q, gamma, h, (int)B, (int)K, (int)N, (int)L, w, b);
  MEGA_CHECK_LAUNCH("ema_parameters_fwd");
  return MEGA_OK;
}
