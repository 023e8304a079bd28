// Kernel argument blocks shared by the CASTLE HIP kernels and the C-ABI layer.
#pragma once
#include <stdint.h>

namespace castle {

// A (B, H, L, d) view with unit stride along d; strides are in elements.
struct View4 {
  void* ptr;
  int64_t sb, sh, sl;
};

struct CoreShape {
  int B, H, L, d;
  int Lp;     // L rounded up to 128
  int nblk;   // Lp / kNB
  float scale;
  int rotary;   // 1: qc, kc, qu, ku, vu are rotated by their row position (RoPE) inside the kernels
  int cus;      // compute units of the device (0: unknown), for prio_by_band
};

// Header of the forward workspace (its first 256 bytes), written on the device by the forward pass.
// The kernels work on vu_s = vu * vu_scale (a power of two <= 1 chosen from max|vu| so that no
// lookahead state can leave the fp16 range: L * max|vu_s| <= 2^15); the scores use
// Su = su_mul * Su_s with su_mul = 1 / vu_scale.  For fp32 tensors both are 1.
struct WsHeader {
  int status;       // bit 0: an input element was clamped to the fp16 range; bit 1: a T' element was
  float vu_scale;
  float su_mul;
};
constexpr int kAmaxBlocks = 256;   // partial maxima written by amax_kernel
// the same for the backward pass: the kernels work on dO * grad_scale (a power of two that puts
// max|dO| into [16, 32)) and multiply the gradients by grad_unscale = 1 / grad_scale when storing
struct BwdHeader {
  float grad_scale;
  float grad_unscale;
};

// Workspace written by the forward pass and read again by the backward pass.
struct FwdWorkspace {
  WsHeader* hdr;
  float* amax_part;   // [kAmaxBlocks] partial maxima of |vu|
  void* t_blk;    // [B*H][Lp][kNB]  T[i][j_local]  = tril(Qc_I Vu_I^T), unscaled
  void* tt_blk;   // [B*H][Lp][kNB]  T^T per block: [j][i_local]
  void* ttx_blk;  // [B*H][Lp][kNB]  rows j of even blocks I: (Qc'_{I+1} Vu_I^T)^T [j][i_local of block I+1]; odd blocks unused
  void* usnap;    // [B*H][snap_rows(nblk)][d]  forward state at block starts
  float* lse;     // [B*H][Lp] natural-log softmax normaliser
  // The six operands in the compute type, each [B*H][Lp][d] contiguous, rows >= L zero
  // (written by the prep kernel; every other kernel reads these instead of the caller's tensors).
  // qc_p is pre-multiplied by scale * log2(e).
  void *qc_p, *kc_p, *vc_p, *qu_p, *ku_p, *vu_p;
};

struct FwdArgs {
  CoreShape s;
  View4 qc, kc, vc, qu, ku, vu;
  View4 out;      // written as (B, H, L, d) through arbitrary strides
  View4 U;        // ptr == nullptr when the final lookahead keys are not wanted
  FwdWorkspace ws;
  int with_t = 1; // the scan launch also fills the T' blocks (0 when only the snapshots are recomputed for a backward pass)
  int u_half = 0; // U is written in the half-precision cache format (see kUHalfScale) instead of the tensor type
};

struct BwdArgs {
  CoreShape s;
  View4 qc, kc, vc, qu, ku, vu, out, dout;
  View4 dqc, dkc, dvc, dqu, dku, dvu;
  FwdWorkspace ws;
  BwdHeader* bhdr;
  float* amax_part;   // [kAmaxBlocks] partial maxima of |dO|
  void* gsnap;    // [B*H][snap_rows(nblk)][d]  reverse state at block ends
  float* delta;   // [B*H][Lp]  rowsum(dO * O)
  // Score-gradient tiles handed from the key-stationary to the query-stationary kernel (16-bit
  // operands, d <= 64 only, else nullptr): per head (Lp/32)^2 tiles of 32 keys x 32 queries,
  // tile (kt, it) at ((kt * (Lp/32) + it) * 1024 elements; only tiles with kt <= it are written.
  // Inside a tile, element (key k, query i) sits at (i / 16) * 512 + k * 16 + i % 16.
  void* dout_p;   // [B*H][Lp][d]  dO in the compute type, rows >= L zero (written by the delta kernel)
  void* ds_mat;   // dS
  void* dsu_mat;  // dSu
};

// Half-precision cache format of the lookahead keys, for bf16 caches: the U buffer holds IEEE fp16
// values of U * kUHalfScale, saturated at +-65504, in the same 2 bytes per element.  The cached step
// rounds every U row once per write-back; bf16 keeps 8 significant bits, fp16 keeps 11, so the
// rounding noise a long decode accumulates is 8 times smaller.  The power-of-two factor moves the
// fp16 window to |U| in [2^-18, 4.2e6]: below it the absolute error (4e-6) is far under what a bf16
// value of any score-relevant size carries; above it the keys saturate instead of becoming infinite
// (lookahead scores of that size are beyond what any 16-bit cache resolves).
constexpr float kUHalfScale = 0.015625f;   // 2^-6
constexpr float kUHalfUnscale = 64.f;

// size of the per-GPU partial-result array behind castle_decode_step_static
constexpr int64_t kDecodeStaticScratchBytes = (int64_t)4 << 20;

// Deferred write-back of the lookahead keys: U is written every kDecodeDefer-th step only; in
// between, the vu rows of the tokens not yet folded into the stored U ("pending") sit in a small
// ring buffer, the gates they got from every cached row in a per-row fp32 side array, and every step
// adds gate * vu of the pending tokens on the fly in fp32.
constexpr int kDecodeDefer = 4;

struct DecodeArgs {
  int B, H, d;
  int t;            // rows already in the cache (used when t_dev is NULL)
  const int* t_dev; // optional: the row count lives in device memory and is read by the kernels
  int capacity;     // rows the cache buffers can hold; with t_dev a step at t >= capacity writes nothing
  int splits;       // partitions of the t rows per (b, h)
  float scale;
  int rotary;       // 1: the new token's qc, kc, qu, ku, vu are rotated by position t
  int u_half;       // 1: the U buffer is in the half-precision cache format (kUHalfScale)
  View4 U, qu_cache, kc_cache, vc_cache;   // capacity buffers, row t is appended
  View4 qc, kc, vc, qu, ku, vu;            // new token, L == 1
  View4 out;                               // (B, H, 1, d)
  float* part;      // [B*H][splits][d + 2]  partial (acc, m, l)
  // deferred write-back (pend_ku.ptr == nullptr: U is written every step)
  View4 pend_vu;            // (B, H, kDecodeDefer, d): row j % kDecodeDefer holds vu of token j (rotated when rotary)
  View4 pend_gate;          // (B, H, capacity, kDecodeDefer) fp32: [k][j % kDecodeDefer] = gate of row k for pending token j
  int base0;                // rows of U are complete up to source base0 - 1 at least (e.g. the prefill length)
  const int* base0_dev;     // the same from device memory (graph replay): base0_dev[0]
};
// first source not yet folded into the stored lookahead keys when the cache holds t rows
__host__ __device__ inline int decode_base(int base0, int t) {
  const int b = t - t % kDecodeDefer;
  return b > base0 ? b : base0;
}

}  // namespace castle
