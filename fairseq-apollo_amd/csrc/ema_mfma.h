// Matrix-core EMA path: entry points shared between ema_mfma.hip and the C ABI in ema_scan.hip.
#pragma once
#include "common.h"

namespace mega {

// ---- layout of the per-channel operand image (written by ema_image_kernel): kImgSlots slots of
// 64 lanes x 16 bytes.  Slots [0, kNOPS): the MFMA A operands K (Toeplitz of k[0..31]), P (p q^(31-i)),
// C (gamma q^(i+1)), each as kNW* bf16 terms x 2 row blocks.  Then, per lane (j = lane & 15, r = lane >> 4)
// for the four states (2r, 2r+1, 8+2r, 9+2r) as (re, im) pairs, two slots each:
//   kSlotQ32  q^32      kSlotRS  q^64      kSlotRJ  (q^64)^j      kSlotRW  q^1024      kSlotRWJ  (q^1024)^j
// and one slot in the layout of the 64-lane segment scan (kSlotScan: q^(32 kSEGT) of state lane >> 2).
// kSlotKT (kNWK slots): the K operand once per distinct content, 56 vectors of 16 bytes per term; lane (m, g) of
// row block mb finds its vector at byte 16 (16 mb + m - 8 g + 24).
// kSlotK16 / kSlotP16 / kSlotC16 (4 slots each: term w, row block mb at 2 w + mb): the same three operands as two
// fp16 terms (22 significant bits), for the kernel that serves fp32 / fp16 activations.
constexpr int kNS = 16;                  // complex states per channel (zero padded)
#ifndef MEGA_SEGT
#define MEGA_SEGT 2
#endif
constexpr int kSEGT = MEGA_SEGT;         // tiles per segment: super-chunk = 16 * kSEGT * 32 tokens
#ifndef MEGA_NWK
#define MEGA_NWK 2
#endif
#ifndef MEGA_NWP
#define MEGA_NWP 2
#endif
#ifndef MEGA_NWC
#define MEGA_NWC 1
#endif
constexpr int kNWK = MEGA_NWK;           // bf16 terms of the Toeplitz operand K
constexpr int kNWP = MEGA_NWP;           // bf16 terms of the state-input operand P
constexpr int kNWC = MEGA_NWC;           // bf16 terms of the state-output operand C
constexpr int kNOPS = 2 * (kNWK + kNWP + kNWC);
constexpr int kSlotK = 0, kSlotP = 2 * kNWK, kSlotC = 2 * (kNWK + kNWP);
constexpr int kSlotQ32 = kNOPS, kSlotScan = kNOPS + 2, kSlotRS = kNOPS + 3, kSlotRJ = kNOPS + 5, kSlotRW = kNOPS + 7,
              kSlotRWJ = kNOPS + 9, kSlotCmp = kNOPS + 11, kSlotKT = kNOPS + 12, kSlotK16 = kNOPS + 12 + kNWK,
              kSlotP16 = kSlotK16 + 4, kSlotC16 = kSlotP16 + 4;
constexpr int kImgSlots = kSlotC16 + 4;
// kSlotCmp: per-state multipliers once each, six tables of 16 complex values (128 bytes = one line):
// and one line of reach figures (how far the slowest pole of the channel carries before |q|^t < 2^-24):
//   word 0: how many of the doubling steps 64, 128, 256, 512 tokens still matter (0..4)
//   word 1: how many blocks of 1024 tokens back a block has to look (1..16)
enum { kCmpQ32 = 0, kCmpRS = 1, kCmpRS2 = 2, kCmpRS4 = 3, kCmpRS8 = 4, kCmpRW = 5, kCmpReach = 6 };
constexpr size_t kImgRowBytes = (size_t)kImgSlots * 64 * 16;

// bytes of the per-channel operand images for a layer (0: the layer is outside the fast path)
size_t ema_image_bytes(int64_t D, int64_t N, int bidirectional);

// kernel generation: coefficients -> operand images.  `parts` says which slots are formed and written (the compact
// per-state tables and the reach line always are): an image that is kept serves any kernel (kImgAll); a call that
// generates the image for itself asks for what its own kernel reads
constexpr int kImgKFull = 1;     // the bf16 K operand, one vector per lane (streaming and row kernels)
constexpr int kImgF16 = 2;       // K, P, C as two fp16 terms (row kernel on fp32 / fp16 activations)
constexpr int kImgPC = 4;        // the bf16 P and C operands
constexpr int kImgStream = 8;    // q^32 and the scan multiplier in the streaming kernel's lane layouts
constexpr int kImgBlocks = 16;   // (q^64)^j and (q^1024)^j (kernels that work on blocks of 1024 tokens)
constexpr int kImgKT = 32;       // the bf16 K operand once per distinct vector (one-kernel norm -> moving average)
constexpr int kImgBf16 = kImgKFull | kImgPC;
constexpr int kImgAll = 63;
int ema_image_build(const float* p, const float* q, const float* gamma, int is_complex, const float* omega, int64_t D,
                    int64_t N, int bidirectional, int shift, void* image, hipStream_t s, int parts = kImgAll);

// true when the streaming kernel handles this request (dtype, layout, alignment, sizes)
bool ema_mfma_covers(int dtype, int64_t sxb, int64_t sxd, int64_t sxl, int64_t syb, int64_t syd, int64_t syl,
                     const void* x, const void* y, const uint8_t* mask, int64_t B, int64_t D, int64_t N, int64_t L,
                     int64_t Lk);

// 1 = handled, 0 = not covered, < 0 = launch error
int ema_mfma_try(const void* x, void* y, int dtype, int64_t sxb, int64_t sxd, int64_t sxl, int64_t syb,
                 int64_t syd, int64_t syl, const float* p, const float* q, const void* image, int is_complex,
                 const float* omega, const uint8_t* mask, const float* h_in, float* h_out, int64_t B, int64_t D,
                 int64_t N, int64_t L, int bidirectional, int64_t Lk, float* acc, float* h_tile, hipStream_t s);

// ---- [B, D, L] rows of any activation type, parallel over blocks of 1024 tokens (csrc/ema_rows.hip)
size_t ema_rows_record_bytes(int64_t B, int64_t D, int64_t L, int bidirectional);
bool ema_rows_covers(int dtype, int64_t sxb, int64_t sxd, int64_t sxl, int64_t syb, int64_t syd, int64_t syl,
                     int64_t B, int64_t D, int64_t N, int64_t L, int64_t Lk, const float* h_out);
int ema_rows_run(const void* x, void* y, int dtype, int64_t sxb, int64_t sxd, int64_t syb, int64_t syd,
                 const void* image, int is_complex, const float* omega, const uint8_t* mask, const float* h_in,
                 float* h_out, int64_t B, int64_t D, int64_t N, int64_t L, int bidirectional, float* acc, float* rec,
                 hipStream_t s);

}  // namespace mega
