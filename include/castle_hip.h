/* C ABI of libcastle_hip.so: the CASTLE (causal attention with lookahead keys) hot path
 * for AMD MI355X (gfx950).  Plain pointers and sizes only; every tensor pointer is DEVICE
 * memory, every call enqueues work on the HIP stream handed in (a hipStream_t passed as
 * void*; NULL = the default stream) and returns without synchronising.
 *
 * Return value of the int entry points: 0 on success, negative on error
 * (castle_error_string() gives the text).  Inputs are never modified.
 *
 * Reference interfaces replaced (paths inside lucidrains/lookahead-keys-attention):
 *   castle_fwd          lookahead_keys_attention_triton.py:417-506  CastleAttentionFunction.forward
 *                       (= castle_attention_triton, :605, called at lookahead_keys_attention.py:122);
 *                       math of lookahead_keys_attention.py:132-164
 *   castle_bwd          lookahead_keys_attention_triton.py:508-602  CastleAttentionFunction.backward
 *   castle_decode_step  lookahead_keys_attention.py:166-203         the seq_len == 1 branch of Castle.forward
 *   castle_decode_step_device_count   the same step, row count in device memory (graph replay)
 */
#ifndef CASTLE_HIP_H_
#define CASTLE_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CASTLE_ABI_VERSION 5

/* element types of the tensors (accumulation is always fp32) */
#define CASTLE_F32 0
#define CASTLE_BF16 1
#define CASTLE_F16 2

/* flags of castle_fwd / castle_bwd.  By default bf16 tensors are converted to fp16 when they are
 * loaded (exact for |x| < 65504) and every operand the kernels produce internally is fp16:
 * same MFMA rate, 3 more mantissa bits, which keeps the gradients of long sequences inside the
 * bf16 tolerance.  CASTLE_FLAG_BF16_OPERANDS keeps bf16 MFMA operands instead (full bf16 range).
 * castle_bwd must get the same flags as the castle_fwd call whose workspace it reads.
 * CASTLE_FLAG_ROTARY: the kernels rotate qc, kc, qu, ku, vu (not vc) by their row position
 * (rotary position embedding over interleaved pairs, base 10000: what Castle(rotary_emb=True) does
 * before its core, lookahead_keys_attention.py:106-112); castle_bwd then returns the gradients with
 * respect to the un-rotated operands; castle_decode_step rotates the new token by position t and
 * appends the rotated qu, kc rows.  The final lookahead keys U are those of the rotated operands. */
#define CASTLE_FLAG_BF16_OPERANDS 1
#define CASTLE_FLAG_ROTARY 2
/* castle_bwd / castle_bwd_workspace_bytes only: do not hand dS / dSu tiles from the first backward
 * kernel to the second (2 * B * H * Lp * Lp elements of workspace); the second kernel recomputes
 * the score chain instead.  Slower, for callers short of memory. */
#define CASTLE_FLAG_RECOMPUTE_SCORES 4
/* castle_bwd / castle_bwd_workspace_bytes only: the forward state buffer was not kept; castle_bwd
 * runs the forward scan again (from the operand copies in the forward workspace) into its own
 * workspace before anything else.  What a forward call must keep for its backward is then O(L d). */
#define CASTLE_FLAG_RECOMPUTE_STATE 8

/* castle_fwd (its U output), castle_decode_step*, castle_decode_flush; bf16 tensors only (else
 * CASTLE_ERR_DTYPE); castle_bwd ignores it.  The lookahead-key buffer U is held in a half-precision
 * cache format instead of bf16: each 2-byte element is the IEEE fp16 value of U * 2^-6, saturated at
 * +-65504 (so |U| up to 4.2e6 is held, with 11 significant bits down to |U| = 2^-8 and an absolute
 * step of 4e-6 below).  The reference's step re-rounds the whole of U to the module type at every
 * token (lookahead_keys_attention.py:183); in bf16 those roundings add up to a few per cent over some
 * hundred steps, in this format to an eighth of that, for the same bytes.  Every entry point that
 * touches one U buffer must get the same setting; a reader converts with  U = 64 * (fp16 bits). */
#define CASTLE_FLAG_U_HALF 16

/* error codes */
#define CASTLE_OK 0
#define CASTLE_ERR_DTYPE (-1)      /* unknown element type */
#define CASTLE_ERR_SHAPE (-2)      /* unsupported head dim / size, or (dtype, d) does not fit the LDS */
#define CASTLE_ERR_LAUNCH (-3)     /* HIP reported a launch / configuration error */
#define CASTLE_ERR_WORKSPACE (-4)  /* workspace NULL, misaligned or too small */
#define CASTLE_ERR_ARG (-5)        /* NULL pointer, misaligned pointer or stride */
#define CASTLE_ERR_SCRATCH (-6)    /* castle_decode_step_static: partial results exceed the static scratch */

/* A (B, H, L, d) tensor view: element strides for b, h and l; the d axis has stride 1.
 * ptr must be 16-byte aligned and every stride a multiple of 16 bytes / sizeof(element). */
typedef struct castle_view4 {
  void* ptr;
  int64_t stride_b;
  int64_t stride_h;
  int64_t stride_l;
} castle_view4;

/* Deferred write-back of the lookahead keys in the cached step (optional argument of the three
 * castle_decode_step* entry points; NULL = U is written by every step, as the reference's step does,
 * lookahead_keys_attention.py:183).  With it the U rows are written on every 4th step only (the steps
 * whose row count t has (t + 1) % 4 == 0).  In between, the vu rows of the up to 3 tokens not yet
 * folded into the stored U ("pending") sit in `vu_ring`, a (B, H, 4, d) buffer in the element type
 * (token j in row j % 4, written by the step that appends j), and the gate each cached row k got from
 * pending token j in `gates`, a (B, H, capacity, 4) fp32 array ([k][j % 4]; stride_l is not used, the
 * rows are 4 floats apart).  Every step adds gate * vu of the pending tokens in fp32: a tenth less
 * HBM traffic per step and a quarter of the roundings of a 16-bit U.  `base`: every U row already
 * holds all sources below `base` (the prefill length, or the row count at the last castle_decode_flush);
 * the sources pending at row count t are max(base, t - t % 4) .. t - 1.  `base_device`, if not NULL,
 * is read by the kernels instead (graph replay).  The stored U is complete whenever nothing is
 * pending; castle_decode_flush makes it so at any other time. */
typedef struct castle_deferred {
  castle_view4 vu_ring;
  castle_view4 gates;
  int32_t base;
  const int32_t* base_device;
} castle_deferred;

int castle_abi_version(void);
const char* castle_error_string(int code);

/* Bytes of the two device buffers castle_fwd needs.  `workspace` (castle_fwd_workspace_bytes,
 * grows like L d): the forward pass leaves there what the backward pass reads again (a header with
 * the range-control scalars and a status word, operand copies in the compute type, per-block T
 * tiles, log-sum-exp); keep it alive and unmodified until castle_bwd has run.  `state`
 * (castle_fwd_state_bytes, grows like L^2 d / 128): the snapshots of the lookahead state, scratch
 * for a forward pass alone; castle_bwd reads them too, unless it is told to recompute them
 * (CASTLE_FLAG_RECOMPUTE_STATE), in which case the buffer can be dropped right after castle_fwd.
 * < 0 on error.  After the stream has finished castle_fwd, the int32 at workspace + 0 is a status
 * word: bit 0 = an input element beyond the fp16 range was clamped (bf16 tensors, fp16 operands),
 * bit 1 = an entry of T' = s qc.vu was. */
int64_t castle_fwd_workspace_bytes(int B, int H, int L, int d, int dtype);
int64_t castle_fwd_state_bytes(int B, int H, int L, int d, int dtype);

/* Parallel forward.  qc,kc,vc,qu,ku,vu: (B,H,L,d), unscaled, as handed to
 * castle_attention_triton (lookahead_keys_attention.py:122).  out: (B,H,L,d) view that is
 * written (any strides, e.g. those of a (B,L,H,d) buffer).  U: optional (NULL, or a view
 * with ptr == NULL, to skip) final lookahead keys for the decode cache
 * (lookahead_keys_attention.py:161-164).  d in {16,32,64,128}; fp32 needs d <= 64.
 * flags: any of CASTLE_FLAG_BF16_OPERANDS, CASTLE_FLAG_ROTARY, CASTLE_FLAG_U_HALF (format of U). */
int castle_fwd(const castle_view4* qc, const castle_view4* kc, const castle_view4* vc,
               const castle_view4* qu, const castle_view4* ku, const castle_view4* vu,
               int B, int H, int L, int d, int dtype, float scale, int flags,
               const castle_view4* out, const castle_view4* U,
               void* workspace, int64_t workspace_bytes, void* state, int64_t state_bytes, void* stream);

/* Bytes of extra device workspace castle_bwd needs: reverse state snapshots, delta, a copy of dout in
 * the compute type and, for the 16-bit element types, the dS / dSu score-gradient tiles its first
 * kernel hands to its second (2 * B * H * Lp * Lp elements, Lp = L rounded up to 128; left out, and
 * the score chain recomputed instead, under CASTLE_FLAG_RECOMPUTE_SCORES or when they would exceed
 * 40 GiB, or the byte count found in the environment variable CASTLE_MAX_SCORE_TILE_BYTES when
 * the library first needed it).  `flags`: those the castle_bwd call will get. */
int64_t castle_bwd_workspace_bytes(int B, int H, int L, int d, int dtype, int flags);

/* Parallel backward.  Same operands as castle_fwd plus the forward output `out`, the
 * upstream gradient `dout`, the forward workspace as castle_fwd left it and its state buffer
 * (NULL with CASTLE_FLAG_RECOMPUTE_STATE).  Writes the six
 * gradients (all (B,H,L,d) views; every element is written, nothing is accumulated).
 * U carries no gradient (lookahead_keys_attention_triton.py:513-515).  d in {16,32,64}, and 128 for
 * the 16-bit element types (there every kernel runs twice, each pass keeping half of the outputs). */
int castle_bwd(const castle_view4* qc, const castle_view4* kc, const castle_view4* vc,
               const castle_view4* qu, const castle_view4* ku, const castle_view4* vu,
               const castle_view4* out, const castle_view4* dout,
               int B, int H, int L, int d, int dtype, float scale, int flags,
               const castle_view4* dqc, const castle_view4* dkc, const castle_view4* dvc,
               const castle_view4* dqu, const castle_view4* dku, const castle_view4* dvu,
               const void* fwd_workspace, int64_t fwd_workspace_bytes,
               const void* fwd_state, int64_t fwd_state_bytes,
               void* bwd_workspace, int64_t bwd_workspace_bytes, void* stream);

/* Bytes of device workspace castle_decode_step needs for a cache of up to t_max rows. */
int64_t castle_decode_workspace_bytes(int B, int H, int d, int t_max);

/* One cached decode step (lookahead_keys_attention.py:166-203), in place.
 * U, qu_cache, kc_cache, vc_cache: (B,H,capacity,d) buffers holding t valid rows;
 * t >= capacity is rejected (CASTLE_ERR_SHAPE) because row t is written.  The call updates U rows 0..t-1 in place (U_k += sigmoid(s qu_k.ku) vu),
 * writes row t of all four (U_t = 0, qu, kc, vc of the new token) and writes
 * out (B,H,1,d) = softmax_k(s qc.kc_k - silu(s qc.U_k)) vc_k over k = 0..t.
 * qc..vu: the new token's (B,H,1,d) operands (stride_l unused).  After the call the cache
 * holds t+1 rows.  d in {16,32,64,128}.  flags: any of CASTLE_FLAG_ROTARY, CASTLE_FLAG_U_HALF. */
int castle_decode_step(const castle_view4* U, const castle_view4* qu_cache,
                       const castle_view4* kc_cache, const castle_view4* vc_cache, int t, int capacity,
                       const castle_view4* qc, const castle_view4* kc, const castle_view4* vc,
                       const castle_view4* qu, const castle_view4* ku, const castle_view4* vu,
                       int B, int H, int d, int dtype, float scale, int flags,
                       const castle_view4* out, const castle_deferred* deferred,
                       void* workspace, int64_t workspace_bytes, void* stream);

/* Folds the pending sources into the stored lookahead keys (see castle_deferred): afterwards the U
 * rows 0 .. t-1 are what a step-by-step update would have left.  POSTCONDITION the caller must
 * establish before the next step or flush on this cache: `base` (and *base_device, when the steps read
 * the base from device memory) = t.  The call does not write either; a second flush, or a step, with
 * the old base adds the same gate * vu terms again.  `gates` must hold `capacity` rows of 4 floats
 * (not checked).  flags: 0 or CASTLE_FLAG_U_HALF. */
int castle_decode_flush(const castle_view4* U, const castle_view4* qu_cache, int t, const castle_deferred* deferred,
                        int B, int H, int d, int dtype, float scale, int flags, void* stream);

/* The same step with the row count t read by the kernels from device memory (*t_device, an int32
 * the caller keeps and advances), so that the enqueued work does not depend on t: one captured HIP
 * graph of a whole model step can be replayed for every token.  `capacity` = rows of the cache
 * buffers; the work split is sized for it, and a step found at *t_device >= capacity (or < 0)
 * writes nothing.  No counterpart in the reference (its step takes t from the tensor shapes,
 * lookahead_keys_attention.py:166-203); meant for callers that replay a captured step.  The call
 * itself records only kernel launches on `stream` (no memset, no allocation, no synchronisation). */
int castle_decode_step_device_count(const castle_view4* U, const castle_view4* qu_cache,
                                    const castle_view4* kc_cache, const castle_view4* vc_cache,
                                    const int32_t* t_device, int capacity,
                                    const castle_view4* qc, const castle_view4* kc, const castle_view4* vc,
                                    const castle_view4* qu, const castle_view4* ku, const castle_view4* vu,
                                    int B, int H, int d, int dtype, float scale, int flags,
                                    const castle_view4* out, const castle_deferred* deferred,
                                    void* workspace, int64_t workspace_bytes, void* stream);

/* The cached step for callers that cannot allocate or bring a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same kernels and results as castle_decode_step (t_device == NULL: row count t from
 * the host) or castle_decode_step_device_count (t_device != NULL: t is ignored), but the partial
 * results of the split pass live in a 4 MiB array that is part of the library's device code, one
 * copy per GPU, held until the process ends.  The call allocates nothing and clears nothing (every
 * partial that is read was written by the same call).  B * H * splits * (d + 2) * 4 bytes must fit
 * the array (splits <= 64, about 640 / (B*H) for small batches: e.g. B*H up to 8065 heads at
 * d = 128), else CASTLE_ERR_SCRATCH.  All calls on one GPU share that GPU's array: calls that
 * overlap on one GPU (different streams, or graph replays running side by side) race.  The first
 * call on a device looks the array's address up (hipGetSymbolAddress); make that call outside
 * stream capture. */
int castle_decode_step_static(const castle_view4* U, const castle_view4* qu_cache,
                              const castle_view4* kc_cache, const castle_view4* vc_cache,
                              int t, const int32_t* t_device, int capacity,
                              const castle_view4* qc, const castle_view4* kc, const castle_view4* vc,
                              const castle_view4* qu, const castle_view4* ku, const castle_view4* vu,
                              int B, int H, int d, int dtype, float scale, int flags,
                              const castle_view4* out, const castle_deferred* deferred, void* stream);

/* Rotary position embedding of one tensor, out of place: out[b,h,l,:] = R(first_position + l) x[b,h,l,:]
 * (the rotation CASTLE_FLAG_ROTARY applies inside the kernels; lookahead_keys_attention.py:112).  Used to
 * fill the qu / kc rows of a decode cache after a rotary prefill. */
int castle_rope(const castle_view4* x, const castle_view4* out, int B, int H, int L, int d, int dtype,
                int first_position, void* stream);

/* y[M, N] = x[M, K] w[N, K]^T, all three row-major in the 16-bit element type `dtype` (leading
 * dimensions ldx, ldw, ldy in elements; fp32 accumulation), for the few rows of a decode step: the
 * fused projection and the output projection around the cached step, which the reference runs as
 * nn.Linear on a (B, 1, dim) tensor (lookahead_keys_attention.py:99 and :209 with seq_len == 1).
 * Meant for M up to a few dozen rows (one workgroup per 32 x 32 output tile, K split over its
 * waves); any M works.  K % 8 == 0, N % 2 == 0, x / w 16-byte aligned with ldx, ldw % 8 == 0. */
int castle_small_linear(const void* x, const void* w, void* y, int M, int N, int K,
                        int64_t ldx, int64_t ldw, int64_t ldy, int dtype, void* stream);

/* The same product with the per-row work of a transformer block's token step folded in (each saves a
 * launch and a pass over the activations; no counterpart in the reference, whose callers run these as
 * separate modules: train_triton.py:102-107, 161-165 around lookahead_keys_attention.py:95, 99, 209):
 *   norm_weight != NULL: RMS normalisation of the x rows in front, y = ((x / sqrt(mean(x^2) + eps)) * norm_weight) w^T
 *                        (nn.RMSNorm; K elements, 16-byte aligned);
 *   activation:          CASTLE_ACT_GELU applies the erf form of GELU to the product;
 *   residual != NULL:    a (M, N) tensor with leading dimension ldr added last (may alias y).
 * Order: normalise, multiply, activate, add. */
#define CASTLE_ACT_NONE 0
#define CASTLE_ACT_GELU 1
int castle_small_linear_fused(const void* x, const void* w, void* y, int M, int N, int K,
                              int64_t ldx, int64_t ldw, int64_t ldy, int dtype,
                              const void* norm_weight, float eps, int activation,
                              const void* residual, int64_t ldr, void* stream);

/* Per-kernel timing (no counterpart in the reference; for benchmarks).  While enabled, every
 * kernel launched by the entry points above is bracketed by a HIP event pair on its stream.
 * castle_profile_enable(on) also discards pending records.  castle_profile_read waits for the
 * recorded kernels, writes up to max_records (slot, milliseconds) pairs in launch order, clears
 * the records and returns their number (< 0 on error).  Slots: 0 operand copies (with the pass for max|vu|), 1 forward scan (with the T' blocks),
 * 2 forward attention, 3 delta, 4 backward key-stationary, 5 backward query-stationary,
 * 6 decode stream, 7 decode finish. */
int castle_profile_enable(int on);
int castle_profile_read(int* slots, float* ms, int max_records);

#ifdef __cplusplus
}
#endif
#endif /* CASTLE_HIP_H_ */
