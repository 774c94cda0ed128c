// Matrix-core EMA path: entry points shared between ema_mfma.hip and the C ABI in ema_scan.hip.
#pragma once
#include "common.h"

namespace mega {

// bytes of the per-channel operand images for a layer (0: the layer is outside the fast path)
size_t ema_image_bytes(int64_t D, int64_t N, int bidirectional);

// kernel generation: coefficients -> operand images
int ema_image_build(const float* p, const float* q, const float* gamma, int is_complex, const float* omega, int64_t D,
                    int64_t N, int bidirectional, int shift, void* image, hipStream_t s);

// true when the streaming kernel handles this request (dtype, layout, alignment, sizes)
bool ema_mfma_covers(int dtype, int64_t sxb, int64_t sxd, int64_t sxl, int64_t syb, int64_t syd, int64_t syl,
                     const void* x, const void* y, const uint8_t* mask, int64_t B, int64_t D, int64_t N, int64_t L,
                     int64_t Lk);

// 1 = handled, 0 = not covered, < 0 = launch error
int ema_mfma_try(const void* x, void* y, int dtype, int64_t sxb, int64_t sxd, int64_t sxl, int64_t syb,
                 int64_t syd, int64_t syl, const float* p, const float* q, const void* image, int is_complex,
                 const float* omega, const uint8_t* mask, const float* h_in, float* h_out, int64_t B, int64_t D,
                 int64_t N, int64_t L, int bidirectional, int64_t Lk, float* acc, float* h_tile, hipStream_t s);

}  // namespace mega
