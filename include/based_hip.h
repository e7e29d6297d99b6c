/*
 * based_hip.h — C ABI of libbased_hip.so, the MI355X (gfx950) kernels behind the Based
 * sequence mixers.
 *
 * Every entry point takes raw device pointers, element strides and sizes, and a HIP
 * stream (passed as void*; NULL = the default stream).  Launches are asynchronous on that
 * stream; pointers are borrowed until the work on the stream has finished.  Nothing here
 * allocates, synchronises or reads device memory from the host, so every call can be
 * captured into a HIP graph.
 *
 * Return value: BASED_OK (0) on success, otherwise one of the BASED_ERR_* codes; a
 * human-readable reason is then available from based_hip_last_error() (thread-local).
 * Unsupported shapes are rejected before anything is launched.
 *
 * Citations name the reference (HazyResearch/based) code each entry point stands in for.
 */
#ifndef BASED_HIP_H
#define BASED_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BASED_API __attribute__((visibility("default")))

enum {
  BASED_OK = 0,
  BASED_ERR_SHAPE = 1,  /* unsupported size (feature dim, head dim, window ...) */
  BASED_ERR_DTYPE = 2,  /* unsupported element type */
  BASED_ERR_ALIGN = 3,  /* pointer or stride not aligned as the kernel requires */
  BASED_ERR_ARG = 4,    /* null pointer / negative size */
  BASED_ERR_LAUNCH = 5  /* the HIP runtime refused the launch */
};

/* element types of q / k / v / y tensors */
enum { BASED_BF16 = 0, BASED_F32 = 1 };

/* feature dimension of the TaylorExp map this library is built for, and its expansion
 * 1 + d + d*d (based/models/mixers/linear_attention.py:255-256). */
#define BASED_FEATURE_DIM 16
#define BASED_EXPANDED_DIM 273

BASED_API int based_hip_version(void);
BASED_API const char* based_hip_last_error(void);

/*
 * Recurrent decode step of Taylor linear attention, feature map fused.
 * Replaces TaylorExp.forward on q,k + LinearAttention.recurrent_forward up to (not
 * including) out_proj: based/models/mixers/linear_attention.py:136-140,230-249.
 *
 *   kv_state[b,h,e,f] += v[b,h,e] * phi(k[b,h])[f]          (in place, fp32)
 *   k_state [b,h,f]   += phi(k[b,h])[f]                     (in place, fp32)
 *   y[b,h,e] = sum_f phi(q)[f] kv_state[b,h,e,f] / (sum_f phi(q)[f] k_state[b,h,f] + eps)
 *
 * q, k : raw 16-dim vectors, element (b,h,i) at  q[b*q_sb + h*q_sh + i]
 * v, y : dv-dim vectors,     element (b,h,e) at  v[b*v_sb + h*v_sh + e]
 * kv_state : contiguous fp32 (B, H, 1, dv, 273); k_state : contiguous fp32 (B, H, 1, 1, 273)
 *            (layout of LinearAttention.allocate_inference_cache, linear_attention.py:258-269)
 * dv must be a multiple of 16, 16 <= dv <= 256.  kv_state must be 16-byte aligned.
 * io_dtype is the element type of q, k, v and y.
 */
BASED_API int based_linear_attn_step(const void* q, const void* k, const void* v,
                           float* kv_state, float* k_state, void* y,
                           int64_t B, int64_t H, int64_t dv,
                           int64_t q_sb, int64_t q_sh, int64_t k_sb, int64_t k_sh,
                           int64_t v_sb, int64_t v_sh, int64_t y_sb, int64_t y_sh,
                           float eps, int io_dtype, void* stream);

/*
 * The same step with the write-back of the state deferred (no counterpart in the reference, whose
 * recurrent_forward rewrites kv_state on every token, based/models/mixers/linear_attention.py:
 * 230-252; y is the same up to fp32 summation order).  Writing the state is half of the step's
 * memory traffic and the output does not need it: with S the state as last written and
 * (k_j, v_j) the tokens since,
 *   phi(q) . (S + sum_j phi(k_j) v_j^T) = phi(q) . S + sum_j (1 + s_j + s_j^2 / 2) v_j,  s_j = q . k_j / 4.
 * A call reads kv_state, updates k_state, and keeps the raw k and v of the token in a ring per
 * (batch, head); the call that finds period - 1 tokens there applies them and its own token to
 * kv_state in one read-modify-write pass and empties the ring.  period = 1 is
 * based_linear_attn_step.  Between those calls kv_state lacks the ring's tokens:
 * based_linear_attn_flush_deferred applies them (for a reader of kv_state other than this call).
 *
 *   pend_k : (B, H, BASED_DEFERRED_MAX_STEPS, 16) fp32, contiguous
 *   pend_v : (B, H, BASED_DEFERRED_MAX_STEPS, dv) fp32, contiguous
 *   pend_n : (B, H) int32, tokens in the ring; zero it when the state is (re)initialised
 *   period : 1 .. BASED_DEFERRED_MAX_STEPS; other arguments as based_linear_attn_step
 */
#define BASED_DEFERRED_MAX_STEPS 8
BASED_API int based_linear_attn_step_deferred(
    const void* q, const void* k, const void* v, float* kv_state, float* k_state, float* pend_k, float* pend_v,
    int32_t* pend_n, void* y, int64_t B, int64_t H, int64_t dv, int64_t q_sb, int64_t q_sh, int64_t k_sb,
    int64_t k_sh, int64_t v_sb, int64_t v_sh, int64_t y_sb, int64_t y_sh, float eps, int period, int io_dtype,
    void* stream);
BASED_API int based_linear_attn_flush_deferred(float* kv_state, const float* pend_k, const float* pend_v,
                                               int32_t* pend_n, int64_t B, int64_t H, int64_t dv, void* stream);

/*
 * Causal Taylor linear attention over a whole sequence (prefill), feature map,
 * normaliser and decode-state construction fused.
 * Replaces LinearAttention.parallel_forward up to (not including) out_proj, and the
 * state einsums that follow it: based/models/mixers/linear_attention.py:169-183,220-222
 * (same arithmetic as the O(L) causal product in
 * train/csrc/causal_dot_prod/causal_attention.cpp:82-124 plus its normaliser).
 *
 *   y[b,h,i,:] = sum_{j<=i} (phi(q_i).phi(k_j)) v_j / (phi(q_i).sum_{j<=i} phi(k_j) + eps)
 *   kv_state[b,h,e,f] = sum_n v[n,e] phi(k_n)[f],  k_state[b,h,f] = sum_n phi(k_n)[f]
 *
 * q, k : element (b,h,l,i) at q[b*q_sb + h*q_sh + l*q_sl + i]   (i < 16 contiguous)
 * v, y : element (b,h,l,e) at v[b*v_sb + h*v_sh + l*v_sl + e]   (e < dv contiguous)
 * kv_state / k_state: as above; either both NULL (training-style forward, no state
 * written) or both non-NULL (overwritten, not accumulated).
 * dv in {64, 128}; any L >= 1.  Row starts of q, k (32 B for bf16) and v, y must be
 * 16-byte aligned.
 */
BASED_API int based_linear_attn_prefill(const void* q, const void* k, const void* v, void* y,
                              float* kv_state, float* k_state,
                              int64_t B, int64_t H, int64_t L, int64_t dv,
                              int64_t q_sb, int64_t q_sh, int64_t q_sl,
                              int64_t k_sb, int64_t k_sh, int64_t k_sl,
                              int64_t v_sb, int64_t v_sh, int64_t v_sl,
                              int64_t y_sb, int64_t y_sh, int64_t y_sl,
                              float eps, int io_dtype, void* stream);

/*
 * Same computation as based_linear_attn_prefill for SMALL batches: each sequence is cut into
 * n_seg segments of whole 64-token chunks that are scanned concurrently (every segment first
 * accumulates its own contribution to the state, an exclusive prefix over segments follows,
 * then every segment is read out from its prefix), so that B*H chains of a short batch can
 * still fill the GPU.  Same reference lines as based_linear_attn_prefill; results agree with
 * it to accumulation order.
 *
 * based_linear_attn_prefill_plan reports the segment count this library would use for a shape
 * (1 = do not split) and the bytes of device workspace that count needs
 * (B*H*(dv/64) * n_seg * BASED_PREFILL_SEGMENT_STATE_BYTES); the caller allocates
 * the workspace (16-byte aligned; contents need no initialisation and are scratch afterwards)
 * and passes both to based_linear_attn_prefill_split.  n_seg <= 1 forwards to the unsplit
 * entry point.  bf16, dv in {64, 128} only.
 */
#define BASED_PREFILL_SEGMENT_STATE_BYTES 43008 /* one (chain, segment) state in the workspace */
BASED_API int based_linear_attn_prefill_plan(int64_t B, int64_t H, int64_t L, int64_t dv, int io_dtype,
                                             int64_t* n_seg, int64_t* workspace_bytes);
BASED_API int based_linear_attn_prefill_split(const void* q, const void* k, const void* v, void* y,
                              float* kv_state, float* k_state,
                              int64_t B, int64_t H, int64_t L, int64_t dv,
                              int64_t q_sb, int64_t q_sh, int64_t q_sl,
                              int64_t k_sb, int64_t k_sh, int64_t k_sl,
                              int64_t v_sb, int64_t v_sh, int64_t v_sl,
                              int64_t y_sb, int64_t y_sh, int64_t y_sl,
                              float eps, int io_dtype,
                              int64_t n_seg, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * based_linear_attn_prefill_split without a workspace argument and without any allocation.
 * No counterpart in the reference: it exists for callers that cannot allocate device memory
 * (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  The
 * per-segment states go to a static device array that is part of the library's code object:
 * BASED_STATIC_SCRATCH_BYTES (64 MiB) per GPU the library runs on, held until the process
 * ends.  B*H*(dv/64) * n_seg * BASED_PREFILL_SEGMENT_STATE_BYTES must fit (every segment count that
 * based_linear_attn_prefill_plan returns does); larger requests return BASED_ERR_SHAPE and
 * launch nothing.  The first call on a device looks the array's address up (make it outside
 * a capture).  All calls on one GPU share the array: calls that overlap in time on one GPU
 * (different streams, different threads) race; calls ordered on one stream do not.  The array
 * keeps the previous call's contents; the kernels overwrite every entry they read.
 * Arguments and results are those of based_linear_attn_prefill_split; n_seg <= 1 forwards to
 * based_linear_attn_prefill, which uses no scratch.
 */
#define BASED_STATIC_SCRATCH_BYTES (64ll << 20)
BASED_API int based_linear_attn_prefill_split_static(const void* q, const void* k, const void* v, void* y,
                              float* kv_state, float* k_state,
                              int64_t B, int64_t H, int64_t L, int64_t dv,
                              int64_t q_sb, int64_t q_sh, int64_t q_sl,
                              int64_t k_sb, int64_t k_sh, int64_t k_sl,
                              int64_t v_sb, int64_t v_sh, int64_t v_sl,
                              int64_t y_sb, int64_t y_sh, int64_t y_sl,
                              float eps, int io_dtype, int64_t n_seg, void* stream);

/*
 * Sliding-window causal softmax attention over a whole sequence.
 * Replaces the flash-attn call behind FlashSelfAttention / FlashCrossAttention with
 * causal=True, window_size=(w_left, 0): based/models/mixers/slide_attention.py:100-106,
 * 206-213.  Query i attends keys j in [i - w_left, i].
 *
 * q, k, v, o : element (b,l,h,c) at p[b*sb + l*sl + h*sh + c], c < 64 contiguous.
 * head dim is 64; 0 <= w_left <= 128 (pass window_size // 2 of the module; the released
 * checkpoints use 128).  bf16 only.
 *
 * rope_cos, rope_sin : NULL, or fp32 tables (rope_len, 32) of cos / sin(position * inv_freq[i]):
 *   q and k are rotated inside the kernel (non-interleaved rotary over the whole head:
 *   channel c pairs with c + 32), the job of the rotary layer the reference applies to qkv
 *   before the attention (slide_attention.py:346-355, 553-556).  Positions start at 0;
 *   rope_len >= L.
 * kcache_out, vcache_out : NULL, or a KV cache (element (b,t,h,c) at p[b*c_sb + t*c_st +
 *   h*c_sh + c], max_seqlen >= L rows) that receives the (rotated) k rows and the v rows of
 *   tokens 0..L-1: the copy _update_kv_cache makes at prefill (slide_attention.py:255-281).
 */
BASED_API int based_swa_prefill(const void* q, const void* k, const void* v, void* o,
                      int64_t B, int64_t H, int64_t L,
                      int64_t q_sb, int64_t q_sl, int64_t q_sh,
                      int64_t k_sb, int64_t k_sl, int64_t k_sh,
                      int64_t v_sb, int64_t v_sl, int64_t v_sh,
                      int64_t o_sb, int64_t o_sl, int64_t o_sh,
                      int w_left, float scale,
                      const float* rope_cos, const float* rope_sin, int64_t rope_len,
                      void* kcache_out, void* vcache_out,
                      int64_t c_sb, int64_t c_st, int64_t c_sh, int64_t max_seqlen,
                      int io_dtype, void* stream);

/*
 * Sliding-window decode step against a linear KV cache.
 * Replaces flash_attn_with_kvcache(q, k_cache, v_cache, k_new, v_new, cache_seqlens,
 * causal=True, window_size=(w_left,0)): based/models/mixers/slide_attention.py:471-481
 * (and the cache write of _update_kv_cache, :255-281).
 *
 * Writes k_new/v_new (B,1,H,64) into row `pos` of the caches, then attends rows
 * [pos - w_left, pos].  pos is cache_seqlens[b] when cache_seqlens (device int32, B
 * entries) is non-NULL — nothing is read on the host, so the call is graph-capturable —
 * else pos_host for every b.  A host position outside [0, max_seqlen) (or beyond the rotary
 * table) is refused with BASED_ERR_ARG; a DEVICE-side position outside that range cannot be
 * refused by the host, so the kernel leaves the cache row unwritten and fills o[b, :, :] of that
 * batch entry with NaN.
 *
 * kcache, vcache : element (b,t,h,c) at p[b*c_sb + t*c_st + h*c_sh + c]; the reference's
 *   packed (B, max_seqlen, 2, H, 64) cache is passed as two pointers 1 plane apart.
 * q, k_new, v_new, o : element (b,h,c) at p[b*sb + h*sh + c].
 * rope_cos, rope_sin : NULL, or the tables described at based_swa_prefill: q and k_new are
 *   rotated at position pos before use (and the rotated k_new is what enters the cache), as
 *   flash_attn_with_kvcache does with its rotary_cos / rotary_sin arguments
 *   (slide_attention.py:400-427).  The position comes from the same place as the cache row,
 *   so a captured graph needs no host-side position.
 */
BASED_API int based_swa_step(const void* q, const void* k_new, const void* v_new,
                   void* kcache, void* vcache, void* o,
                   const int32_t* cache_seqlens, int64_t pos_host,
                   int64_t B, int64_t H, int64_t max_seqlen,
                   int64_t q_sb, int64_t q_sh, int64_t kn_sb, int64_t kn_sh,
                   int64_t vn_sb, int64_t vn_sh, int64_t o_sb, int64_t o_sh,
                   int64_t c_sb, int64_t c_st, int64_t c_sh,
                   int w_left, float scale,
                   const float* rope_cos, const float* rope_sin, int64_t rope_len,
                   int io_dtype, void* stream);

/*
 * Gated short convolution of the Based stack (the mixer of 17 of the 27 layers of the 360m
 * configuration), prefill form.  Replaces, in based/models/mixers/convolution.py, the body of
 * BaseConv.forward between the two projections (:201-208: split, ShortConvolution.forward
 * :47-86 = depthwise causal nn.Conv1d with padding K-1 truncated to L, SiLU, gate) and the state
 * initialisation of ShortConvolution.forward (:62-68).
 *
 *   u      : (B, L, 2D): u1 = u[..., :D] is convolved, u2 = u[..., D:] gates; element (b,l,c) at
 *            u[b*u_sb + l*u_sl + c]
 *   weight : (D, 1, K) contiguous, same dtype as u (the nn.Conv1d weight); K in 2..4
 *   bias   : (D) or NULL (the conv bias)
 *   y      : (B, L, D), y = silu(conv(u1) + bias) * u2; element (b,l,c) at y[b*y_sb + l*y_sl + c]
 *   state  : NULL, or (B, D, K) contiguous of dtype state_dtype, overwritten with the last K
 *            inputs u1 of every channel, oldest first, zero-filled on the left when L < K
 * D must be a multiple of 8 (bf16) / 4 (fp32); strides likewise; u, y 16-byte aligned.
 */
BASED_API int based_gated_conv_prefill(const void* u, const void* weight, const void* bias, void* y,
                             void* state, int64_t B, int64_t L, int64_t D, int K,
                             int64_t u_sb, int64_t u_sl, int64_t y_sb, int64_t y_sl,
                             int io_dtype, int state_dtype, void* stream);

/*
 * Single-token form on the rolling state.  Replaces ShortConvolution.step
 * (convolution.py:104-108: roll the (B, D, K) state left by one, append the input, contract with
 * the conv weight) together with BaseConv.forward's SiLU and gate (:204-207).
 *
 *   u     : (B, 2D) rows at u[b*u_sb + c]     y : (B, D) rows at y[b*y_sb + c]
 *   state : (B, D, K) contiguous, updated in place
 *   bias  : (D) or NULL
 * D must be a multiple of 8; all tensors 16-byte aligned.
 */
BASED_API int based_gated_conv_step(const void* u, void* state, const void* weight, const void* bias,
                          void* y, int64_t B, int64_t D, int K, int64_t u_sb, int64_t y_sb,
                          int io_dtype, int state_dtype, void* stream);

/*
 * The short convolution on its own, y = conv(u) (+ bias), no activation, no gate: the
 * ShortConvolution module used as a mixer by itself (based/models/mixers/convolution.py:47-109,
 * the path without the fused CUDA kernel; the reference's "conv" test model,
 * based/tests/test_generation.py:37-45).  Arguments as based_gated_conv_prefill / _step, except
 * that u has D channels (rows u[b*u_sb + l*u_sl + c], c < D).
 */
BASED_API int based_short_conv_prefill(const void* u, const void* weight, const void* bias, void* y,
                             void* state, int64_t B, int64_t L, int64_t D, int K,
                             int64_t u_sb, int64_t u_sl, int64_t y_sb, int64_t y_sl,
                             int io_dtype, int state_dtype, void* stream);
BASED_API int based_short_conv_step(const void* u, void* state, const void* weight, const void* bias,
                          void* y, int64_t B, int64_t D, int K, int64_t u_sb, int64_t y_sb,
                          int io_dtype, int state_dtype, void* stream);

/*
 * Residual add + RMSNorm of the prenorm block, one pass.  Replaces, in based/models/block.py,
 * `residual = dropped + residual; hidden = norm(residual.to(dtype=norm.weight.dtype));
 * residual = residual.to(torch.float32)` (:134-139 and :151-155, dropout-free) with the RMSNorm
 * of based/ops/triton/layer_norm.py:117-118,926-953 (no bias), and the closing
 * add + ln_f of the model (gpt.py:667-674).
 *
 *   x            : (rows, D), row r at x[r*x_sr]; dtype x_dtype (also the dtype of weight and y)
 *   residual_in  : NULL (first block: r = x) or (rows, D) of residual_dtype
 *   weight       : (D) contiguous
 *   y            : (rows, D) = rms_norm(cast(x + residual_in)) * weight, the cast being to x_dtype
 *   residual_out : NULL or (rows, D) of residual_dtype, receives x + residual_in (fp32 sum)
 * D multiple of 8, at most 4096; strides multiples of 8 elements; 16-byte aligned tensors.
 */
BASED_API int based_add_rms_norm(const void* x, const void* residual_in, const void* weight, void* y,
                       void* residual_out, int64_t rows, int64_t D, int64_t x_sr, int64_t ri_sr,
                       int64_t y_sr, int64_t ro_sr, float eps, int x_dtype, int residual_dtype,
                       void* stream);

/*
 * SwiGLU gate of the MLP: out[r, c] = u[r, c] * silu(u[r, F + c]), the element-wise part of
 * GatedMlp.forward between fc1 and fc2 (based/models/mlp.py:147-151: y, gate = fc1(x).chunk(2);
 * y * silu(gate)).  u: (rows, 2F) rows at u[r*u_sr]; out: (rows, F) rows at out[r*o_sr].
 * F multiple of 8 (bf16) / 4 (fp32); strides likewise; 16-byte aligned tensors.
 */
BASED_API int based_swiglu(const void* u, void* out, int64_t rows, int64_t F, int64_t u_sr, int64_t o_sr,
                 int io_dtype, void* stream);

/*
 * A projection of a single-token step, with the element-wise operation in front of it:
 *
 *     y[m, n] = sum_k pro(x)[m, k] * weight[n, k]  (+ bias[n])       m < M <= 32, bf16, fp32 sums
 *
 * Stands in for the `nn.Linear` calls of a decoding step, where the batch is the only row
 * dimension: proj_q / proj_k / proj_v and out_proj (based/models/mixers/linear_attention.py:
 * 105-108,126-128,251-252), Wqkv and out_proj (slide_attention.py:332-336,541,599), in_proj and
 * out_proj of BaseConv (convolution.py:195-210), fc1 and fc2 (based/models/mlp.py:141-157) and
 * the LM head (gpt.py:794-827); and, through `prologue`, for what the reference runs between them:
 *
 *   BASED_PROLOGUE_NONE          pro(x) = x, (M, K)
 *   BASED_PROLOGUE_ADD_RMS_NORM  r = x + residual_in (r = x if residual_in is NULL), fp32;
 *                                pro(x) = rms_norm(bf16(r)) * norm_weight, rounded to bf16;
 *                                residual_out (if not NULL, and never residual_in itself) <- r.
 *                                The arithmetic of based_add_rms_norm (block.py:134-139,151-155;
 *                                based/ops/triton/layer_norm.py:117-118).
 *   BASED_PROLOGUE_SWIGLU        x is (M, 2K); pro(x)[m, k] = x[m, k] * silu(x[m, K + k]), the
 *                                arithmetic of based_swiglu (mlp.py:147-151).
 *
 * and, through `epilogue`, for what consumes the output of a projection in (value, gate) pairs;
 * weight then has N = 2F rows, value rows first, and y is (M, F):
 *
 *   BASED_EPILOGUE_NONE             y = the projection
 *   BASED_EPILOGUE_SWIGLU           y[m, f] = p[m, f] * silu(p[m, F + f]) with p the projection
 *                                   rounded to bf16: fc1 and the gate (mlp.py:147-151)
 *   BASED_EPILOGUE_GATED_CONV_STEP  one step of BaseConv's gated short convolution on p: the
 *                                   arithmetic of based_gated_conv_step (convolution.py:78-109,
 *                                   195-210); conv_state (M, F, conv_k) of conv_state_dtype is
 *                                   rolled and updated in place, conv_weight (F, conv_k) and
 *                                   conv_bias (F, or NULL) are bf16, conv_k 2 to 4.
 *   Paired epilogues take K up to 2048 and not the SwiGLU prologue.
 *
 *   x            : rows at x[m * x_row_stride]; with x_row_index (M int64 values on the device)
 *                  row m is x[x_row_index[m] * x_row_stride] instead: the embedding lookup of the
 *                  first block (gpt.py:622-631).  An index outside [0, x_index_rows) gives that
 *                  row of y NaN; nothing is read out of bounds.
 *   weight       : (N, K) rows at weight[n * w_row_stride]; bias NULL or (N) contiguous
 *   y            : (M, N) or (M, F), rows at y[m * y_row_stride]
 *   residual_in / residual_out : fp32 (M, K), rows at the given strides (norm prologue only)
 * K multiple of 8, at most 4096; row strides of x and weight multiples of 8 elements, of the
 * residuals multiples of 4; x, weight, norm_weight and the residuals 16-byte aligned.
 */
enum { BASED_PROLOGUE_NONE = 0, BASED_PROLOGUE_ADD_RMS_NORM = 1, BASED_PROLOGUE_SWIGLU = 2 };
enum { BASED_EPILOGUE_NONE = 0, BASED_EPILOGUE_SWIGLU = 1, BASED_EPILOGUE_GATED_CONV_STEP = 2 };
#define BASED_DECODE_LINEAR_MAX_ROWS 32
BASED_API int based_decode_linear(const void* x, int64_t x_row_stride, const int64_t* x_row_index,
                        int64_t x_index_rows, const void* weight, int64_t w_row_stride,
                        const void* bias, void* y, int64_t y_row_stride, int64_t M, int64_t N,
                        int64_t K, int prologue, const float* residual_in, int64_t ri_row_stride,
                        float* residual_out, int64_t ro_row_stride, const void* norm_weight,
                        float eps, int epilogue, void* conv_state, int conv_state_dtype,
                        const void* conv_weight, const void* conv_bias, int conv_k, void* stream);

/*
 * Sliding-window attention for head dimensions other than 64 and for every rotary shape of the
 * reference's constructor, on the MFMA path: any head dim that is a multiple of 8 up to 128 (112
 * and 128 are the released 1B / 1.3B models: n_embd 1792 / 2048 over 16 heads,
 * train/configs/experiment/reference/based-1b.yaml:94-99), rotary over the first `rotary_dim`
 * channels (a multiple of 16, at most D; slide_attention.py:346-355: RotaryEmbedding(rotary_emb_dim,
 * interleaved=rotary_emb_interleaved)), half-split pairs (c, c + rotary_dim/2) or, with
 * rotary_interleaved != 0, pairs (2i, 2i+1).  Replaces the same reference calls as
 * based_swa_prefill / based_swa_step (flash_attn_qkvpacked_func / flash_attn_kvpacked_func after
 * _update_kv_cache, slide_attention.py:59-106,150-213,255-281; flash_attn_with_kvcache with its
 * rotary arguments, slide_attention.py:384-481) with the same argument meaning, plus:
 *   D                      : head dim; rows of q, k, v, o and the cache hold D contiguous elements
 *   rope_cos / rope_sin    : fp32 (rope_len, rotary_dim / 2), NULL for no rotary
 *   rotary_dim, rotary_interleaved : as above (ignored without tables)
 * All element strides multiples of 8, all tensors 16-byte aligned, 0 <= w_left <= 128, bf16.
 * A device-side position outside the cache or the rotary table leaves the cache untouched and
 * writes NaN to that (batch, head) output row.
 */
BASED_API int based_swa_prefill_wide(const void* q, const void* k, const void* v, void* o, int64_t B,
                           int64_t H, int64_t L, int64_t D,
                           int64_t q_sb, int64_t q_sl, int64_t q_sh,
                           int64_t k_sb, int64_t k_sl, int64_t k_sh,
                           int64_t v_sb, int64_t v_sl, int64_t v_sh,
                           int64_t o_sb, int64_t o_sl, int64_t o_sh,
                           int w_left, float scale,
                           const float* rope_cos, const float* rope_sin, int64_t rope_len,
                           int64_t rotary_dim, int rotary_interleaved,
                           void* kcache_out, void* vcache_out,
                           int64_t c_sb, int64_t c_st, int64_t c_sh, int64_t max_seqlen,
                           int io_dtype, void* stream);
BASED_API int based_swa_step_wide(const void* q, const void* k_new, const void* v_new,
                        void* kcache, void* vcache, void* o,
                        const int32_t* cache_seqlens, int64_t pos_host,
                        int64_t B, int64_t H, int64_t D, int64_t max_seqlen,
                        int64_t q_sb, int64_t q_sh, int64_t kn_sb, int64_t kn_sh,
                        int64_t vn_sb, int64_t vn_sh, int64_t o_sb, int64_t o_sh,
                        int64_t c_sb, int64_t c_st, int64_t c_sh,
                        int w_left, float scale,
                        const float* rope_cos, const float* rope_sin, int64_t rope_len,
                        int64_t rotary_dim, int rotary_interleaved,
                        int io_dtype, void* stream);

/*
 * The same sliding-window attention for head dimensions other than 64 (any multiple of 8 up to
 * 128), bf16, fp32 arithmetic, one wavefront per query: not a performance path; a plain second
 * statement of the same attention (the reference's own test models have 16-dim heads,
 * based/tests/test_generation.py:7-34,69-80) that the tests hold the MFMA kernels against.  Same reference lines
 * and argument meaning as based_swa_prefill / based_swa_step, plus the head dimension D; no
 * in-kernel rotary (the caller rotates q and k first).
 */
BASED_API int based_swa_prefill_anydim(const void* q, const void* k, const void* v, void* o,
                             int64_t B, int64_t H, int64_t L, int64_t D,
                             int64_t q_sb, int64_t q_sl, int64_t q_sh,
                             int64_t k_sb, int64_t k_sl, int64_t k_sh,
                             int64_t v_sb, int64_t v_sl, int64_t v_sh,
                             int64_t o_sb, int64_t o_sl, int64_t o_sh,
                             int w_left, float scale,
                             void* kcache_out, void* vcache_out,
                             int64_t c_sb, int64_t c_st, int64_t c_sh, int64_t max_seqlen,
                             int io_dtype, void* stream);
BASED_API int based_swa_step_anydim(const void* q, const void* k_new, const void* v_new,
                          void* kcache, void* vcache, void* o,
                          const int32_t* cache_seqlens, int64_t pos_host,
                          int64_t B, int64_t H, int64_t D, int64_t max_seqlen,
                          int64_t q_sb, int64_t q_sh, int64_t kn_sb, int64_t kn_sh,
                          int64_t vn_sb, int64_t vn_sh, int64_t o_sb, int64_t o_sh,
                          int64_t c_sb, int64_t c_st, int64_t c_sh,
                          int w_left, float scale, int io_dtype, void* stream);

/*
 * Greedy sampling of one decoding step and the bookkeeping of the loop around it, in one launch
 * that can be recorded in the same graph as the step: replaces sample(logits, top_k=1) =
 * logits.argmax(dim=-1) (based/generation.py:64-70), the append of the token to the sequences
 * and the advance of seqlen_offset (generation.py:190-204), and the copies of the next input ids,
 * position ids and lengths_per_sample into the recorded graph's static tensors
 * (generation.py:725-735).  Per batch row b:
 *   tok = first index of the largest of logits[b, 0..V) (NaN counts as the largest, as torch.argmax)
 *   p = lengths[b]                       position of the token the step just processed
 *   next_ids[b * ids_stride] = tok       the next step's input
 *   sequences[b * seq_stride + p + 1] = tok   (skipped when sequences is NULL or p + 1 >= seq_len)
 *   lengths[b] = p + 1;  position_ids[b * pos_stride] = p + 1 (position_ids may be NULL)
 * logits: bf16 or fp32, row stride logits_stride elements (>= V); ids and positions int64,
 * lengths int32.
 */
BASED_API int based_greedy_step(const void* logits, int64_t B, int64_t V, int64_t logits_stride,
                                int64_t* next_ids, int64_t ids_stride, int64_t* sequences,
                                int64_t seq_stride, int64_t seq_len, int32_t* lengths,
                                int64_t* position_ids, int64_t pos_stride, int io_dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BASED_HIP_H */
