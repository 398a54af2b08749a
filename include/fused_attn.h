/*
 * C ABI of the gfx950 fused multi-head attention forward library
 * (libfused_attn_gfx950.so).  Plain pointers and sizes only: no torch types, no HIP
 * types in the signatures, so the same entry points can be bound from C++, ctypes or
 * any FFI.
 *
 * All tensors are IEEE fp16 in device memory.  q, k, v and out share one addressing
 * rule, given in ELEMENTS:
 *     element(b, h, l, d) = base + b*stride_b + h*stride_h + l*stride_l + d      (d < H)
 * The reference layout [B, L, R*H] (reference src/fused_attn_extention.cu:24-27,50-52;
 * head h = columns [h*H, (h+1)*H), reference include/fused_attn.cuh:683-690) is
 *     stride_b = L*R*H, stride_h = H, stride_l = R*H,
 * and a [B, R, L, H] tensor is stride_b = R*L*H, stride_h = L*H, stride_l = H.
 * Strides must be multiples of 8 elements and the base pointers 16-byte aligned.
 *
 * Return value of every int function: 0 = success, < 0 = invalid argument (FA_ERR_*),
 * > 0 = a hipError_t raised by the runtime.  Nothing here ever calls exit().
 */
#ifndef FUSED_ATTN_H_
#define FUSED_ATTN_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FA_OK 0
#define FA_ERR_NULL_POINTER (-1)
#define FA_ERR_BAD_HEAD_DIM (-2)
#define FA_ERR_BAD_SHAPE (-3)
#define FA_ERR_BAD_STRIDE (-4)
#define FA_ERR_MISALIGNED (-5)
#define FA_ERR_TOO_LARGE (-6)
#define FA_ERR_BAD_FLAGS (-7)
#define FA_ERR_BAD_SCALE (-8)

#define FA_FLAG_CAUSAL 1
#define FA_FLAG_BF16 2

/*
 * out = softmax(q k^T * scale [+ mask]) v for every (batch, head), non-causal.
 *
 * Replaces launch_attention_kernel<head_dim, chunk_size>(batch_size, seq_len,
 * num_features, queries, keys, values, mask, output, syncronize)
 * (reference include/fused_attn.cuh:860-894) together with the kernel it launches
 * (reference include/fused_attn.cuh:605-858).  Differences a caller can see:
 *   - head_dim is a run-time argument (16, 32, 64 or 128), there is no chunk_size:
 *     the key tile is an internal choice and L need not be a multiple of anything;
 *   - the launch goes to `stream` (a hipStream_t, NULL = the null stream) and the
 *     call returns without synchronising;
 *   - `mask` (nullable) is an additive fp16 [B, L, L] tensor shared by all heads and is
 *     applied to every key, not only to the first chunk.  Rows whose keys are all -inf
 *     produce zeros.
 * `scale` is finite and > 0 (FA_ERR_BAD_SCALE otherwise); the reference fixes it at
 * 1/sqrt(head_dim) (reference include/fused_attn.cuh:727).
 * B, R, L >= 1.  L*stride_l, R*stride_h and B*stride_b must stay below 2^62 elements and
 * stride_l must not exceed 2^24 elements (FA_ERR_TOO_LARGE otherwise).
 * Accuracy: scores, softmax state and both products are accumulated in float32; the softmax
 * weights are rounded to fp16 before they multiply the values, scaled by a power of two chosen
 * from L so that a row of L keys loses at most 2^-13 (1.2e-4) of its weight to the bottom of the
 * fp16 range: a key more than 13 + ceil(log2 L) log2 units below the largest score of its row
 * contributes nothing (25 units, 17 natural-log units, at L = 4096).  The reference accumulates
 * everything in fp16 (reference include/fused_attn.cuh:174,257,650-653).
 */
int fa_fwd(const void* q, const void* k, const void* v, const void* mask, void* out,
           int64_t B, int64_t R, int64_t L, int64_t H,
           int64_t stride_b, int64_t stride_h, int64_t stride_l,
           float scale, void* stream);

/*
 * fa_fwd with two extensions the reference lists as not done yet (reference README.md:135-142,
 * "backward pass", and its GPT/LLaMA use case, README.md:8):
 *   flags & FA_FLAG_CAUSAL : query i attends to keys j <= i only; key tiles above the diagonal
 *                            are skipped.  Not combinable with `mask`.
 *   flags & FA_FLAG_BF16   : q, k, v, out (and mask) hold bfloat16 instead of fp16 (reference
 *                            README.md:137 lists other input types as not done).  Same kernels,
 *                            bf16 matrix instructions, probabilities rounded to bf16.
 *   lse (nullable)         : float32 [B, R, L] in device memory, receives
 *                            log(sum_j exp(score_ij)) per query row (-inf for a row whose keys
 *                            are all masked): what a backward pass needs to recompute the
 *                            probabilities.
 * Everything else as fa_fwd, which is fa_fwd_ex with lse = NULL and flags = 0.  There is no
 * counterpart in the reference (its kernel is non-causal and keeps no row statistics).
 */
int fa_fwd_ex(const void* q, const void* k, const void* v, const void* mask, void* out, void* lse,
              int64_t B, int64_t R, int64_t L, int64_t H,
              int64_t stride_b, int64_t stride_h, int64_t stride_l,
              float scale, int flags, void* stream);

/*
 * fa_fwd_ex with strides of its own for `out`: q, k and v share (stride_b, stride_h, stride_l),
 * out is addressed with (out_stride_b, out_stride_h, out_stride_l), under the same rules
 * (multiples of 8 elements, last dimension contiguous; the 2^24 limit applies to stride_l only).
 * This is what lets q, k and v be three views into one packed projection output (say
 * [B, L, 3, R, H], the layout a fused QKV projection writes: reference README.md:137 lists that
 * front end as not done) while out is an ordinary contiguous tensor, with no copy on either side.
 * The reference has no counterpart: its launcher takes contiguous [B, L, R*H] tensors only
 * (reference src/fused_attn_extention.cu:34-44).
 */
int fa_fwd_strided(const void* q, const void* k, const void* v, const void* mask, void* out, void* lse,
                   int64_t B, int64_t R, int64_t L, int64_t H,
                   int64_t stride_b, int64_t stride_h, int64_t stride_l,
                   int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_l,
                   float scale, int flags, void* stream);

/*
 * The launch the library would make for a problem, without making it (no GPU is touched): for
 * tests of the launcher and for tuning.  has_mask != 0 stands for an additive mask with 16-byte
 * aligned rows.  Fills plan[0..6] with: wave64s per workgroup; query rows per wave; workgroups
 * launched; workgroups that do work (the rest exit at once); workgroups per (batch, head), or
 * pairs of query tiles per head for a causal launch of the eight-wave kernel and for those masked
 * launches of it that pairs cost no round of the chip; 0, or, when the
 * query tiles of a causal launch are dealt out to a resident grid, the heads per XCD; the edge of
 * the matrix instruction's tile, 32, or 16 at head_dim 64 and 128 for plain launches of the eight-wave
 * kernel whose workgroups fill whole rounds of the chip (the last round at least seven eighths full)
 * and for its causal launches from seven eighths of a round on.
 * The reference has no counterpart (its grid is fixed at (B, L / chunk_size, R),
 * reference include/fused_attn.cuh:872-883).
 */
int fa_fwd_plan(int64_t B, int64_t R, int64_t L, int64_t H, int flags, int has_mask, int* plan);

/*
 * 1 if fa_fwd accepts this head_dim, else 0.  Counterpart of the compile-time
 * (head_dim, chunk_size) dispatch table (reference src/fused_attn_extention.cu:72-111).
 */
int fa_fwd_query(int64_t H);

/*
 * The power of two (as a base-2 exponent) the softmax weights of a row of L keys are divided by
 * before they are rounded to 16 bits for the second product: a key at the running maximum of its
 * row gets the weight 2^-bias.  11 - ceil(log2 L), kept inside [-8, 6]: see "Accuracy" under fa_fwd.
 * Exported so that callers and tests can state the accuracy limit of a launch; no counterpart in the
 * reference, which keeps every intermediate in fp16 (reference include/fused_attn.cuh:174,257,650-653).
 */
float fa_fwd_reference_bias(int64_t L);

/*
 * Human-readable text for a status returned by fa_fwd.  Replaces the print-and-exit
 * macros CHECK_CUDA_ERROR / CHECK_LAST_CUDA_ERROR (reference include/fused_attn.cuh:17-42).
 * The returned pointer is static storage.
 */
const char* fa_strerror(int status);

/*
 * Timed replay for benchmarks: launches fa_fwd `iters` times back to back on `stream`,
 * bracketed by HIP events recorded on that same stream, waits, and writes the average
 * milliseconds per launch to *ms_per_launch.  Counterpart of the timing loop in
 * reference tests/benchmark_fused_attn.py:36-42 (wall clock around 128 launches).
 */
int fa_fwd_timed(const void* q, const void* k, const void* v, const void* mask, void* out,
                 int64_t B, int64_t R, int64_t L, int64_t H,
                 int64_t stride_b, int64_t stride_h, int64_t stride_l,
                 float scale, void* stream, int iters, float* ms_per_launch);

/*
 * fa_fwd_timed for every form of the launch: the arguments of fa_fwd_strided (flags, lse, strides
 * of `out`) followed by those of the timing loop.  The same counterpart in the reference
 * (tests/benchmark_fused_attn.py:36-42); fa_fwd_timed is this with lse = NULL, flags = 0 and the
 * strides of q for out.
 */
int fa_fwd_timed_ex(const void* q, const void* k, const void* v, const void* mask, void* out, void* lse,
                    int64_t B, int64_t R, int64_t L, int64_t H,
                    int64_t stride_b, int64_t stride_h, int64_t stride_l,
                    int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_l,
                    float scale, int flags, void* stream, int iters, float* ms_per_launch);

/*
 * Fused QKV projection, the front end the reference lists as not done (reference README.md:137;
 * its kernel takes queries, keys and values as three separate tensors, reference
 * src/fused_attn_extention.cu:15-22):
 *     qkv[b, l, s, :] = x[b, l, :] w[:, s F : (s + 1) F] (+ bias[s F : (s + 1) F]),   s = 0, 1, 2,  F = R H
 * x is [B, L, F_in], w is [F_in, 3 F] (input features along the rows), bias (nullable) is [3 F], qkv
 * is the packed [B, L, 3, F] tensor, all contiguous, fp16 (bfloat16 with FA_FLAG_BF16), f32
 * accumulation, one rounding.  The three slices qkv[:, :, s, :] are what fa_fwd_strided takes as q,
 * k and v (stride_b = 3 L F, stride_h = H, stride_l = 3 F) without a copy.
 * rope_cos / rope_sin (both or neither; nullable): float32 [L, H / 2] tables of a rotary position
 * encoding in the rotate-half form, applied to every head of the q and k slices before the rounding:
 *     out[i] = y[i] cos[l, i] - y[i + H/2] sin[l, i],  out[i + H/2] = y[i + H/2] cos[l, i] + y[i] sin[l, i]
 * for i < H / 2, y the projected head vector.
 * F_in and F must be multiples of 64 (FA_ERR_BAD_SHAPE otherwise); x, w, qkv and the tables 16-byte
 * aligned, bias 8-byte aligned.  Launches on `stream` and returns without synchronising.
 */
int fa_qkv_proj(const void* x, const void* w, const void* bias, void* qkv,
                int64_t B, int64_t L, int64_t F_in, int64_t R, int64_t H,
                const float* rope_cos, const float* rope_sin, int flags, void* stream);

/*
 * The launch fa_qkv_proj would make for a problem, without making it (no GPU is touched): for
 * tests of the launcher.  Fills plan[0..3] with: workgroups launched; workgroups that do work (a
 * resident grid: workgroup w of them takes the tiles w, w + working, ...); output tiles of 256 x 256
 * (row tiles times feature tiles); feature tiles.  No counterpart in the reference (see fa_qkv_proj).
 */
int fa_qkv_proj_plan(int64_t B, int64_t L, int64_t F_in, int64_t R, int64_t H, int* plan);

#ifdef __cplusplus
}
#endif

#endif /* FUSED_ATTN_H_ */
