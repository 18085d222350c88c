/*
 * maltos_hip.h -- C ABI of libmaltos_hip.so, the MI355X (gfx950) kernels for the per-GPU
 * training-step hot path of MALTOS: causal / document-masked attention forward and backward,
 * ring block attention with log-sum-exp merge, RMSNorm, interleaved RoPE, SwiGLU, causal
 * cross-entropy, global-norm clipping and fused AdamW over flat fp32 buffers.
 *
 * The reference (xing7code/maltos) is pure Python and has no FFI; each entry point below names
 * the reference call site (file:line under the reference tree) whose native work it replaces.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer unless stated otherwise.  Nothing here allocates or frees
 *    device memory: outputs and workspaces are caller-allocated.
 *  - `stream` is a hipStream_t passed as void*; NULL is the default stream.  All work is enqueued
 *    asynchronously on it; no entry point synchronises the host.
 *  - Return value: MLTS_OK (0) or an MLTS_ERR_* code; mlts_last_error() gives the message of the
 *    last failure on the calling thread.  Argument checks happen on the host before any launch.
 *  - dtype codes: MLTS_F32 = 0, MLTS_BF16 = 1.
 *  - Tensors are described by element strides where noted; the innermost (head_dim / hidden)
 *    dimension is always contiguous.
 */
#ifndef MALTOS_HIP_H
#define MALTOS_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLTS_OK 0
#define MLTS_ERR_INVALID 1     /* bad shape / pointer / alignment / dtype */
#define MLTS_ERR_UNSUPPORTED 2 /* valid request this build has no kernel for (see mlts_attn_supports) */
#define MLTS_ERR_LAUNCH 3      /* HIP runtime reported an error at launch */

#define MLTS_F32 0
#define MLTS_BF16 1

/* attention mask modes */
#define MLTS_MASK_NONE 0   /* every key visible (ring off-diagonal blocks) */
#define MLTS_MASK_CAUSAL 1 /* key j visible to query i iff j <= i + (Sk - Sq) */
#define MLTS_MASK_DOC 2    /* visible iff k_pos[j] <= q_pos[i] && q_seq[i] == k_seq[j] && q_seq[i] >= 0 */

typedef void* mlts_stream_t;

int mlts_abi_version(void);
const char* mlts_last_error(void);

/* Measurement aid with no counterpart in the reference (it times whole steps with a device
 * synchronise, tools/profile_train_perf.py:900-919): when enabled, the main kernel of each entry
 * point is bracketed by HIP events on its launch stream.  Names: "attn_fwd", "attn_bwd_dkdv",
 * "attn_bwd_dq", "attn_delta", "attn_doc_prepass", "attn_merge", "adamw", "ce", "rmsnorm_fwd",
 * "rmsnorm_bwd", "rope", "swiglu_fwd", "swiglu_bwd", "grad_to_f32", "grad_sum_slices".
 * mlts_kernel_timing_read synchronises on the recorded events and returns the summed kernel time
 * and the number of launches since timing was enabled.  Enabling or disabling clears the records. */
void mlts_kernel_timing_enable(int enable);
int mlts_kernel_timing_read(const char* name, double* total_ms, int64_t* launches);

/* ------------------------------------------------------------------------------------------ */
/* Attention                                                                                  */
/* ------------------------------------------------------------------------------------------ */

/* Layout of one attention call.  q/o/do/dq are [B, Hq, Sq, D]; k/v/dk/dv are [B, Hkv, Sk, D];
 * strides are in elements for (batch, head, seq); D is contiguous.  Query head h reads KV head
 * h / (Hq / Hkv) (the reference's repeat_interleave, models/llama.py:97-100). */
typedef struct mlts_attn_shape {
  int32_t B, Hq, Hkv, Sq, Sk, D;
  int32_t dtype;     /* MLTS_BF16 (MFMA path) or MLTS_F32 */
  int32_t mask_mode; /* MLTS_MASK_* */
  float scale;       /* softmax scale, the reference uses D^-0.5 (utils/attention_backend.py:128) */
  int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3];
  /* MLTS_MASK_DOC only: int32 [B, Sq] / [B, Sk] contiguous position and sequence ids
   * (runtime/layers/attn_masking_utils.py:54-87).  seq id < 0 marks padding
   * (utils/constants.py:4); padded queries produce zeros and lse = -inf. */
  const int32_t* q_pos;
  const int32_t* k_pos;
  const int32_t* q_seq;
  const int32_t* k_seq;
  /* MLTS_MASK_DOC only, optional: a plan built by mlts_attn_doc_plan for the same B, Hq, Hkv, Sq, Sk and the same
   * contents of the four id arrays.  NULL: the call builds its own at the front of its workspace. */
  const void* doc_plan;
} mlts_attn_shape;

/* NULL if (dtype, D, mask_mode, strides) is served by a kernel, else a static reason string.
 * Mirrors flash_attn_fallback_reason / flash_attn_dense_block_fallback_reason
 * (runtime/layers/flash_utils.py:105-135). */
const char* mlts_attn_supports(const mlts_attn_shape* s);

/* Bytes of device workspace mlts_attn_fwd / mlts_attn_bwd need for this shape: the per-row statistics the kernels
 * share (delta, LSE in base 2): O(B * Hq * Sq), the workspace class of the flash backward the reference calls
 * (runtime/layers/flash_utils.py:239-258).  With MLTS_MASK_DOC also the per-tile position / sequence-id ranges and
 * the visibility bits of the (64 queries, 64 keys) pairs that a document boundary or the causal diagonal cuts, which a
 * pre-pass forms once per call for all heads: B * Sq * Sk / 8 bytes (forward), twice that (backward). */
int64_t mlts_attn_fwd_workspace_bytes(const mlts_attn_shape* s);
int64_t mlts_attn_bwd_workspace_bytes(const mlts_attn_shape* s, int accumulate_f32);

/* Document-mask plan: what mlts_attn_fwd and mlts_attn_bwd derive from the ids in front of their kernels (tile
 * statistics, visibility bits of the tile pairs a document boundary or the diagonal cuts, the order in which the
 * kernels walk their blocks).  It depends on B, Hq / Hkv, Sq, Sk and the ids only, not on q, k, v: every layer of a
 * model, forward and backward, attends under the same mask, so a caller can build the plan once per batch into a
 * buffer of mlts_attn_doc_plan_bytes (16-byte aligned, B * Sq * Sk / 4 bytes and a little) and pass it in
 * mlts_attn_shape::doc_plan; the calls then skip their pre-pass (three small launches, 28 us at B=2, S=8192) and
 * mlts_attn_*_workspace_bytes no longer include it.  The plan must not be rewritten while a call that uses it is in
 * flight.  No counterpart in the reference, whose callers rebuild the varlen metadata per call
 * (runtime/layers/flash_utils.py:566-640).  Returns 0 bytes / does nothing for shapes the generic kernels serve. */
int64_t mlts_attn_doc_plan_bytes(const mlts_attn_shape* s);
int mlts_attn_doc_plan(const mlts_attn_shape* s, void* plan, int64_t plan_bytes, mlts_stream_t stream);

/* O = softmax(scale * Q K^T + mask) V and LSE = logsumexp (natural log, fp32, [B, Hq, Sq]).
 * Replaces F.scaled_dot_product_attention (utils/attention_backend.py:60-64,109-116),
 * flash_attn_dense / flash_attn_dense_with_lse / flash_attn_varlen
 * (runtime/layers/flash_utils.py:180-215,266-276,493-520). */
int mlts_attn_fwd(const mlts_attn_shape* s, const void* q, const void* k, const void* v, void* o,
                  float* lse, void* workspace, int64_t workspace_bytes, mlts_stream_t stream);

/* dQ, dK, dV by recompute from (Q, K, V, O, LSE, dO); O and LSE may be the GLOBAL ones of a ring
 * schedule, which is what makes per-block calls compose.  Replaces flash_attn_dense_backward
 * (runtime/layers/flash_utils.py:218-263) and the autograd of SDPA.
 * accumulate_f32 (strides dq_stride etc are in elements of the respective type):
 *   MLTS_BWD_OVERWRITE (0)     dq/dk/dv have the input dtype and are overwritten.
 *   MLTS_BWD_ACCUMULATE (1)    dq/dk/dv are fp32 and are ADDED to (the `dq += block_dq.float()` form of
 *                              runtime/layers/functional.py:1121-1146).
 *   MLTS_BWD_DQ_ACCUMULATE (2) dq is fp32 and added to; dk/dv have the input dtype and are overwritten: a block of a
 *                              ring step on the rank that owns the queries, where a K/V chunk meets the local queries
 *                              exactly once (functional.py:1104-1146: one `dk += ...` per chunk and rank).
 *   MLTS_BWD_DQ_STORE (3)      as 2, but dq (fp32) is overwritten: the first block of such an accumulation, which
 *                              saves clearing the fp32 buffer beforehand. */
#define MLTS_BWD_OVERWRITE 0
#define MLTS_BWD_ACCUMULATE 1
#define MLTS_BWD_DQ_ACCUMULATE 2
#define MLTS_BWD_DQ_STORE 3
int mlts_attn_bwd(const mlts_attn_shape* s, const void* dout, const int64_t do_stride[3], const void* q,
                  const void* k, const void* v, const void* o, const float* lse, void* dq,
                  const int64_t dq_stride[3], void* dk, const int64_t dk_stride[3], void* dv,
                  const int64_t dv_stride[3], int accumulate_f32, void* workspace, int64_t workspace_bytes,
                  mlts_stream_t stream);

/* mlts_attn_bwd for callers that cannot allocate device memory or bring a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and
 * results as mlts_attn_bwd with a workspace of exactly mlts_attn_bwd_workspace_bytes (the recomputing backward); the
 * workspace is a buffer of MLTS_ATTN_BWD_NOALLOC_MAX_WORKSPACE bytes inside the library image, one copy per GPU, held
 * until the process ends.  Shapes whose workspace is larger (about B * Hq * Sq > 1 M query rows; with MLTS_MASK_DOC
 * also B * Sq * Sk / 4 bytes of visibility bits, e.g. B * S * S beyond about 28 M) are rejected with MLTS_ERR_INVALID.  No hipMalloc / hipFree is made.  All calls on one GPU share that buffer.  Calls on
 * different streams of one GPU are made to take turns (each waits for an event recorded behind the last), except calls
 * recorded into a HIP graph: graphs that hold this call and may run at the same time on one GPU race on the buffer and
 * must be ordered by the caller, or use mlts_attn_bwd with one workspace per graph. */
#define MLTS_ATTN_BWD_NOALLOC_MAX_WORKSPACE (8 << 20)
int mlts_attn_bwd_noalloc(const mlts_attn_shape* s, const void* dout, const int64_t do_stride[3], const void* q,
                          const void* k, const void* v, const void* o, const float* lse, void* dq,
                          const int64_t dq_stride[3], void* dk, const int64_t dk_stride[3], void* dv,
                          const int64_t dv_stride[3], int accumulate_f32, mlts_stream_t stream);

/* Log-sum-exp merge of one block into the running fp32 state, rows [q_off, q_off + q_len):
 *   lse' = logaddexp(lse, lse_b); out' = out * exp(lse - lse') + out_b * exp(lse_b - lse'),
 * with exp(-inf - x) := 0 (a row where both are -inf becomes 0 with lse -inf).  Replaces
 * _merge_attention_blocks / _exp_delta_or_zero (runtime/layers/functional.py:717-748).
 * out_acc fp32 [B, H, S, D] contiguous; lse_acc fp32 [B, H, S]; o_blk [B, H, q_len, D] of
 * blk_dtype with strides; lse_blk fp32 [B, H, q_len] contiguous. */
int mlts_attn_merge(float* out_acc, float* lse_acc, const void* o_blk, const int64_t o_blk_stride[3],
                    int32_t blk_dtype, const float* lse_blk, int32_t B, int32_t H, int32_t S, int32_t D,
                    int32_t q_off, int32_t q_len, mlts_stream_t stream);

/* ------------------------------------------------------------------------------------------ */
/* Layer kernels                                                                              */
/* ------------------------------------------------------------------------------------------ */

/* y = w * round(x * rsqrt(mean(x^2) + eps)) with fp32 statistics and the reference's two
 * roundings (models/llama.py:55-57).  x, y [rows, hidden] contiguous; rstd_out fp32 [rows]. */
int mlts_rmsnorm_fwd(const void* x, const void* w, void* y, float* rstd_out, int64_t rows, int32_t hidden,
                     float eps, int32_t dtype, mlts_stream_t stream);
/* dx [rows, hidden]; dw [hidden] (same dtype).  dw_partial: fp32 workspace of
 * mlts_rmsnorm_bwd_workspace_bytes(rows, hidden) bytes. */
int64_t mlts_rmsnorm_bwd_workspace_bytes(int64_t rows, int32_t hidden);
int mlts_rmsnorm_bwd(const void* dy, const void* x, const void* w, const float* rstd, void* dx, void* dw,
                     void* workspace, int64_t workspace_bytes, int64_t rows, int32_t hidden, int32_t dtype,
                     mlts_stream_t stream);
/* The residual add in front of a norm fused into it (models/llama.py:224-230 `x = x + sublayer(...)` followed by the
 * next RMSNorm, :55-57): sum_out = round(x + res), y = RMSNorm(sum_out) with the roundings of the two separate ops.
 * sum_out and y are different buffers; sum_out may alias x or res. */
int mlts_add_rmsnorm_fwd(const void* x, const void* res, void* sum_out, const void* w, void* y, float* rstd_out,
                         int64_t rows, int32_t hidden, float eps, int32_t dtype, mlts_stream_t stream);
/* Backward of the pair: x is the summed row (sum_out above), dres the gradient reaching it by the residual path;
 * dx = round(dx of the norm) + dres, the gradient of both addends.  Other arguments as mlts_rmsnorm_bwd. */
int mlts_add_rmsnorm_bwd(const void* dy, const void* x, const void* w, const float* rstd, const void* dres, void* dx,
                         void* dw, void* workspace, int64_t workspace_bytes, int64_t rows, int32_t hidden, int32_t dtype,
                         mlts_stream_t stream);


/* Interleaved-pair rotary embedding (models/llama.py:89-94,134-144):
 *   (x[2i], x[2i+1]) -> (x[2i] c - x[2i+1] s, x[2i] s + x[2i+1] c), c/s = cos/sin[pos, i],
 * every product and the sum rounded to `dtype` as the reference's eager ops do.
 * x, y: [B, H, S, D] with element strides (batch, head, seq); cos/sin: [max_pos, D/2] of `dtype`.
 * positions: int32 [B, S] or NULL (then pos = position_offset + s).  inverse != 0 rotates by
 * -theta, which is the backward pass.  y may be x with the same strides (rotation in place); any other overlap of the
 * two is undefined. */
int mlts_rope(const void* x, const int64_t x_stride[3], void* y, const int64_t y_stride[3], const void* cos_tab,
              const void* sin_tab, int32_t max_pos, const int32_t* positions, int32_t position_offset,
              int32_t B, int32_t H, int32_t S, int32_t D, int32_t dtype, int32_t inverse,
              mlts_stream_t stream);

/* The two rotations of one attention layer, q = rotary(q) and k = rotary(k) (models/llama.py:143-144), in one launch:
 * operand a is [B, Ha, S, D], operand b [B, Hb, S, D]; everything else as mlts_rope, whose results it equals bit for
 * bit.  Each operand must hold fewer than 2^31 16-byte vectors. */
int mlts_rope_pair(const void* xa, const int64_t xa_stride[3], void* ya, const int64_t ya_stride[3], int32_t Ha,
                   const void* xb, const int64_t xb_stride[3], void* yb, const int64_t yb_stride[3], int32_t Hb,
                   const void* cos_tab, const void* sin_tab, int32_t max_pos, const int32_t* positions,
                   int32_t position_offset, int32_t B, int32_t S, int32_t D, int32_t dtype, int32_t inverse,
                   mlts_stream_t stream);

/* h = round(silu(gate)) * up (models/llama.py:205-206); n = number of elements, contiguous. */
int mlts_swiglu_fwd(const void* gate, const void* up, void* h, int64_t n, int32_t dtype, mlts_stream_t stream);
int mlts_swiglu_bwd(const void* dh, const void* gate, const void* up, void* dgate, void* dup, int64_t n,
                    int32_t dtype, mlts_stream_t stream);

/* The same over [rows, cols] matrices with row strides in elements (multiples of 16 bytes): gate and up are the two
 * column halves of ONE projection output (gate_proj and up_proj of models/llama.py:196-206 run as one GEMM over their
 * adjacent weights), dgate and dup the halves of one gradient buffer, so that the next GEMM reads them without a copy. */
int mlts_swiglu_fwd_rows(const void* gate, const void* up, int64_t ld_in, void* h, int64_t ld_h, int64_t rows, int64_t cols,
                         int32_t dtype, mlts_stream_t stream);
int mlts_swiglu_bwd_rows(const void* dh, int64_t ld_dh, const void* gate, const void* up, int64_t ld_in, void* dgate, void* dup,
                         int64_t ld_out, int64_t rows, int64_t cols, int32_t dtype, mlts_stream_t stream);

/* Causal cross-entropy, forward and gradient in one pass over the logits (utils/losses.py:9-15):
 *   loss = sum_{t: label_t != ignore_index} (logsumexp(z_t) - z_t[label_t]) / max(1, #targets)
 *   dlogits_t = (softmax(z_t) - onehot(label_t)) / max(1, #targets) for supervised rows, else 0.
 * logits, dlogits: [rows, vocab] contiguous of `dtype` (dlogits may alias logits); labels int64
 * [rows]; loss_out fp32 [1]; count_out int32 [1]; workspace: fp32 [rows] + 64 bytes. */
int64_t mlts_ce_workspace_bytes(int64_t rows);
int mlts_ce_fwd_bwd(const void* logits, const int64_t* labels, void* dlogits, float* loss_out,
                    int32_t* count_out, void* workspace, int64_t workspace_bytes, int64_t rows, int32_t vocab,
                    int64_t ignore_index, int32_t dtype, mlts_stream_t stream);
/* x *= *scale (device fp32 scalar) unless *scale == 1: applies the upstream d(loss) to the
 * gradient that mlts_ce_fwd_bwd stored. */
int mlts_scale_by_device_scalar(void* x, const float* scale, int64_t n, int32_t dtype, mlts_stream_t stream);

/* ------------------------------------------------------------------------------------------ */
/* Optimizer step over flat buffers                                                           */
/* ------------------------------------------------------------------------------------------ */

#define MLTS_SQNORM_WS_BYTES 16384

/* dst_f32[i] (=|+=) float(src[i]); optional fused sum of squares of the RESULT in fp64.
 * Replaces the per-parameter grad upcast of MasterWeightsOptimizer.copy_master_params
 * (runtime/optim.py:43-56).  sq_out (fp64 [1]) and workspace (MLTS_SQNORM_WS_BYTES) may be NULL. */
int mlts_grad_to_f32(float* dst, const void* src, int32_t src_dtype, int64_t n, int accumulate, double* sq_out,
                     void* workspace, mlts_stream_t stream);

/* out[i] = (accumulate ? out[i] : 0) + sum over s < slices of parts[s * n + i], added in fp32 and rounded once to
 * `dtype` (bf16 or fp32; out and parts share it).  Finishes a weight gradient dW = dY^T X of nn.Linear
 * (models/llama.py:69-75,196-198) that was computed as `slices` row-slice products, and with accumulate != 0 adds it
 * onto the gradient already held in a view of the flat gradient buffer (runtime/plugins/zero1.py:117-121), which is
 * what autograd's `param.grad += dW` does there in a second pass. */
int mlts_grad_sum_slices(void* out, const void* parts, int32_t dtype, int32_t slices, int64_t n, int accumulate,
                         mlts_stream_t stream);

/* *sq_out = sum x[i]^2 accumulated in fp64 (runtime/plugins/grad_clip.py:62-77,
 * runtime/plugins/zero_common.py:324-329).  workspace: MLTS_SQNORM_WS_BYTES. */
int mlts_sq_norm(const float* x, int64_t n, double* sq_out, void* workspace, mlts_stream_t stream);

/* x *= scale (runtime/plugins/grad_clip.py:55-58). */
int mlts_scale(float* x, float scale, int64_t n, mlts_stream_t stream);

/* Decoupled-weight-decay Adam on flat fp32 p/g/m/v (torch.optim.AdamW as built by
 * train/cli.py:432-441, stepped inside runtime/optim.py:65-71):
 *   g' = g * c;  p *= 1 - lr*wd;  m = lerp(m, g', 1-b1);  v = b2 v + (1-b2) g'^2;
 *   p -= (lr / (1-b1^t)) * m / (sqrt(v)/sqrt(1-b2^t) + eps)
 * c = grad_scale, further multiplied by the clip coefficient max_norm / (sqrt(*sq_norm) + 1e-6)
 * when sq_norm != NULL and that coefficient is < 1 (runtime/plugins/grad_clip.py:54-58).
 * p_lowp, if not NULL, receives bf16(p) in the same pass (the write-back of
 * runtime/optim.py:68-70).  step is the 1-based step count t. */
int mlts_adamw_step(float* p, const float* g, float* m, float* v, void* p_lowp, int64_t n, float lr, float beta1,
                    float beta2, float eps, float weight_decay, int64_t step, float grad_scale,
                    const double* sq_norm, float max_norm, mlts_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MALTOS_HIP_H */
