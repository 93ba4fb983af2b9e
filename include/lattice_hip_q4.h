/*
 * lattice_hip_q4.h — C ABI of liblattice_hip_q4.so: lattice's Q4 block-quantized
 * matmul path (decode GEMV, prefill GEMM, single-LoRA epilogue, grouped MoE expert
 * GEMV) on AMD MI355X (gfx950).
 *
 * Conventions shared with the reference backend this replaces
 * (crates/inference/src/forward/metal_qwen35/inner/dispatch.rs):
 *   - row-major everywhere; a weight matrix is W[N,K] (out x in) and the op is
 *     Y[M,N] = X[M,K] . W^T;
 *   - weights are lattice's native 20-byte Q4 blocks, byte for byte
 *     ([f16 scale][f16 bias][16 bytes, low nibble = even index], 32 weights per
 *     block, row stride (K/32)*20 bytes; crates/inference/src/weights/q4_weights.rs:65-92);
 *   - offsets are BYTES; M == 0 or N == 0 is a silent no-op; K == 0 or K % 32 != 0
 *     is an error (the reference asserts, dispatch.rs:185-188);
 *   - every output element of rows < N is overwritten (no accumulate) except where a
 *     function says it accumulates.
 * Pointers named *_dev are device addresses on the context's GPU.  `stream` is a
 * hipStream_t passed as void* (NULL = the default stream); launches are asynchronous.
 * Every function returns LQ4_OK (0) or a negative LQ4_E_* code and never throws or
 * aborts; lq4_last_error() gives the message for the calling thread's last failure.
 */
#ifndef LATTICE_HIP_Q4_H
#define LATTICE_HIP_Q4_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LQ4_BLOCK_BYTES 20   /* q4_weights.rs:84  Q4_BLOCK_BYTES   */
#define LQ4_BLOCK_WEIGHTS 32 /* q4_weights.rs:92  Q4_BLOCK_WEIGHTS */

enum {
    LQ4_OK = 0,
    LQ4_E_INVALID = -1,  /* bad argument (null pointer, K % 32 != 0, out-of-range view) */
    LQ4_E_HIP = -2,      /* a HIP runtime call failed; message carries hipGetErrorString */
    LQ4_E_BLOCK = -3,    /* a block's scale/bias failed the ingress rule               */
    LQ4_E_NOMEM = -4,
    LQ4_E_UNSUPPORTED = -5 /* e.g. LoRA rank above LQ4_MAX_LORA_RANK                   */
};

enum { LQ4_F32 = 0, LQ4_F16 = 1 }; /* element type of activations / LoRA factors */

#define LQ4_MAX_LORA_RANK 64   /* the reference's kernels assume rank <= 64 (qwen35.metal:2302) */
#define LQ4_MAX_TOP_K 256      /* MAX_TOP_K of the reference's GPU top-k (shaders/qwen35.metal:1686) */
#define LQ4_MAX_GEMV_BATCH 16  /* lq4_gemv handles 1..16 rows; use lq4_gemm above that          */

typedef struct lq4_ctx lq4_ctx;       /* one per GPU; owns small scratch buffers          */
typedef struct lq4_weight lq4_weight; /* replaces Q4WeightBuf (forward/metal_qwen35.rs:599-636) */
typedef struct lq4_lora lq4_lora;     /* replaces one LoraLayerData projection (metal_qwen35.rs:1701-1716) */

const char* lq4_last_error(void);
const char* lq4_version(void);

/* ---- context ------------------------------------------------------------------ */
/* A context owns scratch buffers, the LoRA t = A.x buffer and a few hand-over words that its calls
 * share.  A call that uses them on another stream than the previous such call makes its stream wait
 * (hipStreamWaitEvent) for everything queued on that previous stream so far, so calls alternating
 * between streams are ordered instead of racing, without a host stall; when one of the two streams is
 * being captured the dependency becomes part of the capture, like any other cross-stream edge.  What
 * this cannot order: replays of graphs captured on different streams, and calls from several host
 * threads at once.  Those need a context each. */
int lq4_ctx_create(int device_ordinal, lq4_ctx** out);
int lq4_ctx_destroy(lq4_ctx* ctx);
/* hipStreamSynchronize(stream); the counterpart of commit()+wait_until_completed()
 * (forward/metal_qwen35.rs:6447). */
int lq4_sync(lq4_ctx* ctx, void* stream);

/* ---- weights: upload and residency ------------------------------------------- */
/* Host-side per-block ingress rule = validate_q4_block_metadata_scan
 * (q4_weights.rs:907-918; rule in weights/ingress.rs:542-559): every block's scale
 * finite and > 0, bias finite.  On failure returns LQ4_E_BLOCK and stores the first
 * offending block index and reason (1 = scale, 2 = bias). */
int lq4_validate_blocks(const uint8_t* host_payload, size_t nbytes, int64_t* bad_block,
                        int* reason);

/* Replaces mmap_q4_weight + new_buffer_with_bytes_no_copy (metal_qwen35.rs:660-702):
 * copies `nbytes` of host memory VERBATIM into a resident device allocation (no
 * repacking).  `payload_offset` is where the block payload starts inside that buffer
 * (36 for a whole 2-D .q4 file, 0 for raw blocks), as in Q4WeightBuf.  `validate` != 0
 * runs lq4_validate_blocks over the payload first (Q4BlockCheck::Now,
 * q4_weights.rs:926-947) and publishes nothing to the GPU if it fails. */
int lq4_weight_upload(lq4_ctx* ctx, const uint8_t* host_bytes, size_t nbytes,
                      uint64_t payload_offset, int validate, lq4_weight** out);
/* Wraps bytes that already live on the device (caller keeps ownership and must keep
 * them alive); used for buffers assembled on the GPU, e.g. fused gate||up
 * (metal_qwen35.rs:12137-12152). */
int lq4_weight_wrap(lq4_ctx* ctx, const void* blocks_dev, size_t nbytes, uint64_t payload_offset,
                    lq4_weight** out);
int lq4_weight_free(lq4_weight* w);
/* Device address of byte 0 of the buffer (payload_offset not applied) and its size. */
int lq4_weight_info(const lq4_weight* w, const void** base_dev, size_t* nbytes,
                    uint64_t* payload_offset);

/* ---- LoRA --------------------------------------------------------------------- */
/* Replaces the per-projection upload in load_lora_adapter (metal_qwen35.rs:3806-3986):
 * A is [rank, d_in], B is [d_out, rank], row-major, host memory, f32 (as the
 * reference stores them) or f16.  rank <= LQ4_MAX_LORA_RANK. */
int lq4_lora_upload(lq4_ctx* ctx, const void* a_host, const void* b_host, int dtype,
                    uint32_t rank, uint32_t d_in, uint32_t d_out, lq4_lora** out);
int lq4_lora_free(lq4_lora* l);

/* Stand-alone form of dispatch_lora_if_active (layers/mod.rs:15-51), for callers that
 * keep the base projection and the adapter as separate steps:
 *   y[r, 0..d_out) += lora_scale * B . (A . x[r, 0..d_in))      for r < rows.
 * ACCUMULATES into y.  A NULL `lora` (no adapter for this layer/module) is a no-op.
 * x_dev: f32 or f16 [rows, d_in]; y_dev: f32 [rows, d_out]. */
int lq4_lora_apply(lq4_ctx* ctx, const lq4_lora* lora, float lora_scale, const void* x_dev,
                   int x_dtype, uint32_t rows, float* y_dev, void* stream);

/* ---- decode GEMV ---------------------------------------------------------------
 * Replaces dispatch_matmul / dispatch_matmul_q4 (dispatch.rs:148-168, 231-245) and
 * the m == 1 arm of dispatch_gemm_q4 (dispatch.rs:190-200), extended to small
 * batches so the weights stream from HBM once for all rows:
 *   y[b, 0..N) = W . x[b, 0..K)            for b < batch (1..LQ4_MAX_GEMV_BATCH)
 * and, when `lora` is non-NULL, the delta of dispatch_lora_if_active
 * (layers/mod.rs:15-51) fused into the same store:
 *   y[b, n] += lora_scale * sum_j B[n, j] * (sum_k A[j, k] * x[b, k]).
 * x_dev: f32 [batch, K]; y_dev: f32 [batch, N]; W starts at
 * payload_offset + w_extra_offset bytes into the weight buffer (qw_extra_offset of
 * dispatch_gemm_at, dispatch.rs:935-980).
 * At batch 1 with a LoRA adapter the launch computes A . x itself and keeps a few words of
 * hand-over state in the context: such calls must not overlap on two streams of one context.  The
 * same holds at 2..8 rows where the integer matrix-core kernel serves the call and its tiles leave
 * `rank` CUs idle, and (without any state) from 9 rows on for ranks up to 16, where the few-token
 * kernel computes A . X for its own token tile: no launch for A . x precedes any of these.
 * Activation range: at batch 1 any finite f32 value (activations are staged as 23-bit fixed point
 * scaled by a power of two per 32-element block and multiplied exactly, so the result tracks an f32
 * GEMV as the reference's gemv_q4_decode does, shaders/qwen35.metal:794-866; an infinite or NaN
 * activation makes every output NaN); at batch 2..16 activations are split into unscaled f16 pairs
 * (two rows) or rounded to f16 (more), and |x| >= 65504 becomes infinity -- except where the integer
 * matrix-core kernel serves the call (3..8 rows of a matrix of at most 4096 x 2048 unless the context
 * was created under LQ4_GEMV_I8=0): it keeps 24 bits (up to four rows: an f32 GEMV, as the
 * reference's gemm_q4 is) or 16 bits (five to eight) of every activation below its 32-element block's
 * largest magnitude and takes any finite f32 value; a row that holds an infinity or a NaN comes back
 * NaN.  The guaranteed contract is the weaker one. */
int lq4_gemv(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
             const float* x_dev, uint32_t batch, float* y_dev, const lq4_lora* lora,
             float lora_scale, void* stream);

/* Several projections of the same activations in one call: y_i[b, 0..n_i) = W_i . x[b, 0..K) for i < count, each
 * with its own optional LoRA epilogue as in lq4_gemv.  Replaces the runs of dispatch_matmul calls on one input
 * buffer -- q, k and v of an attention layer (inner/layers/gqa.rs:72-98 with their LoRA deltas behind them,
 * gqa.rs:100-127), qkv and z of a GDN layer, for which the reference had to write a merged weight file to save a
 * dispatch (inner/layers/gdn.rs:68-73, weights/q4_weights.rs:1553-1643) -- without asking the caller to store the
 * matrices together: the views may lie anywhere.
 * At batch 1 the projections are ONE launch: the GEMV kernel walks the rows of the matrices stacked one under the
 * other (launch, staging of x and start of the stream paid once), and the A . x of every adapter among them is
 * computed by a few workgroups of that same launch, as lq4_gemv does for one adapter (ranks summing to more than 64:
 * one more launch in front instead).  Needs K * 4.5 bytes <= 128 KB of LDS (K <= 29120) and, for K of 512 or 1024 (rows
 * side by side in a wave), every n_i a multiple of 4 or 2.  At batch 2..8 projections whose n_i are multiples of 16,
 * with K <= 2048 and at most 4096 rows in all, are one launch of the integer matrix-core kernel over the stacked rows
 * (the A . X of all adapters in producer workgroups of that launch where CUs are idle for them, else in one
 * launch in front).  Other shapes and batches up to 16 go projection by projection
 * through lq4_gemv's own routing (still one A . X launch for all adapters that need one).  At batch 17..128 every
 * projection takes lq4_gemm's routing for f32 activations, and those the few-token kernel serves share one packed
 * image of x (one pack launch for q, k and v instead of three; adapters of rank <= 16 up to 64 rows have their
 * A . X computed inside that kernel, no launch for it).  Above 128 rows: LQ4_E_INVALID, use lq4_gemm.
 * A projection with n == 0 is skipped.  Results are those of `count` lq4_gemv calls to the contract's tolerance
 * (bit-identical without LoRA at batch 1: same kernel, same order of summation).  The A . x values live in the
 * context: calls with adapters must not overlap on two streams of one context.  Every projection is checked
 * before anything is launched. */
#define LQ4_MAX_PROJECTIONS 8
typedef struct lq4_projection {
    const lq4_weight* w;
    uint64_t w_extra_offset;
    uint32_t n;
    float* y_dev;            /* f32 [batch, n] */
    const lq4_lora* lora;    /* NULL = none */
    float lora_scale;
} lq4_projection;
int lq4_gemv_multi(lq4_ctx* ctx, const lq4_projection* proj, uint32_t count, uint32_t k, const float* x_dev,
                   uint32_t batch, void* stream);

/* ---- prefill GEMM --------------------------------------------------------------
 * Replaces dispatch_gemm / dispatch_gemm_at -> dispatch_gemm_q4[_at]
 * (dispatch.rs:170-229, 507-525, 935-1097): Y[M,N] = X[M,K] . W^T, X f32 or f16
 * (the reference's tiled kernel rounds f32 X to half in-tile,
 * shaders/gemm_q4_tiled.metal:45-48), f32 accumulate, Y f32.  m <= LQ4_MAX_GEMV_BATCH
 * with f32 X routes to the GEMV kernel, as m == 1 does in the reference.  Optional
 * LoRA delta as in lq4_gemv, applied per row (apply_lora_rows,
 * crates/inference/src/lora_hook.rs). */
int lq4_gemm(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
             const void* x_dev, int x_dtype, uint32_t m, float* y_dev, const lq4_lora* lora,
             float lora_scale, void* stream);

/* ---- MoE ----------------------------------------------------------------------
 * Device restatement of compute_router_probs (from the logits on) + select_top_k +
 * renormalize_selected (crates/inference/src/model/qwen35/moe.rs:39-125; GPU twin
 * layers/mod.rs:226-289): softmax over all E, top-k by strict '>' (ties keep the lower
 * id), selected weights renormalised to sum 1.  logits_dev f32 [tokens, E];
 * ids_dev i32 [tokens, top_k] (-1 = unfilled slot); weights_dev f32 [tokens, top_k]. */
int lq4_moe_route(lq4_ctx* ctx, const float* logits_dev, uint32_t tokens, uint32_t num_experts,
                  uint32_t top_k, int32_t* ids_dev, float* weights_dev, void* stream);

/* Replaces accumulate_routed_experts (moe.rs:127-190) / the expert part of
 * encode_moe_ffn (layers/mod.rs:542-660), reading the experts' Q4 blocks directly
 * instead of a CPU-dequantised f16 copy:
 *   y[t,:] = sum_s weights[t,s] * W_down[e] . ( silu(W_gate[e] . x[t]) * (W_up[e] . x[t]) ),
 *   e = ids[t,s]; slots with e outside [0, E) are skipped.
 * gate_up: [E, 2*inter, hidden] (gate rows then up rows per expert); down:
 * [E, hidden, inter]; both expert-major native blocks.  Tokens routed to the same
 * expert share one pass over that expert's weights.  x_dev f32 [tokens, hidden];
 * y_dev f32 [tokens, hidden] (overwritten).  tokens*top_k <= 4096.  Up to 8 tokens (hidden <= 8192,
 * top_k * inter <= 8192) every pair is served as a one-token GEMV and the weighted sum over a
 * token's slots is formed inside the down pass; larger steps group the pairs by expert. */
int lq4_moe_grouped_gemv(lq4_ctx* ctx, const lq4_weight* gate_up, const lq4_weight* down,
                         uint32_t num_experts, uint32_t inter, uint32_t hidden,
                         const float* x_dev, uint32_t tokens, const int32_t* ids_dev,
                         const float* weights_dev, uint32_t top_k, float* y_dev, void* stream);

/* Replaces apply_shared_expert (crates/inference/src/model/qwen35/moe.rs:194-250) / step 2 of
 * encode_moe_ffn (forward/metal_qwen35/inner/layers/mod.rs:313-413) with its closing
 * moe_shared_gate_add (shaders/qwen35.metal:2379-2392), the always-active expert of the MoE FFN:
 *   g[t]    = 1 / (1 + exp(-dot(x[t], shared_gate)))
 *   y[t,:] += g[t] * W_down . ( silu(W_gate . x[t]) * (W_up . x[t]) )
 * y_dev is ACCUMULATED into: call it after lq4_moe_grouped_gemv on the same y (the reference adds the
 * shared expert onto the routed experts' sum), or on a zeroed y for the shared part alone.
 * gate_up: [2*shared_inter, hidden], gate_proj rows then up_proj rows (the fused gate||up layout of
 * the dense MLP); down: [hidden, shared_inter]; shared_gate_dev f32 [hidden]; x_dev f32
 * [tokens, hidden], 16-byte aligned; y_dev f32 [tokens, hidden].  The intermediate results live in a
 * library buffer that grows on first use (not during stream capture; run the shape once before). */
int lq4_moe_shared_expert(lq4_ctx* ctx, const lq4_weight* gate_up, const lq4_weight* down,
                          const float* shared_gate_dev, uint32_t shared_inter, uint32_t hidden,
                          const float* x_dev, uint32_t tokens, float* y_dev, void* stream);

/* The whole MoE FFN of one layer: moe_ffn_step (crates/inference/src/model/qwen35/moe.rs:8-36) /
 * encode_moe_ffn (forward/metal_qwen35/inner/layers/mod.rs:226-660) from the router logits on:
 * lq4_moe_route, lq4_moe_grouped_gemv and lq4_moe_shared_expert behind one call, with the routing
 * tables in library scratch.  y_dev f32 [tokens, hidden] is overwritten.  Everything runs on
 * `stream` in order (the shared expert beside the routed experts on a second stream was measured
 * slower on MI355X).  Argument meaning and limits as in the three calls it replaces, and the same
 * results bit for bit, except where a shared expert as wide as the routed ones (shared_inter ==
 * inter) rides along with them, whose sums are formed in a different order: equal to the three calls
 * to f32 rounding (1e-5 relative).  That is the case
 *   - up to 8 tokens with hidden <= 8192 and (top_k + 1) * inter <= 8192: two launches (every
 *     (token, slot) pair as a one-token GEMV, the shared expert as one more slot, the router and the
 *     shared expert's gate inside the first launch when num_experts <= 256);
 *   - from 9 to 384 tokens (num_experts < 1024): the shared expert is one more expert of the grouped
 *     kernels, chosen by every token with sigmoid(x . shared_gate) as its routing weight, which the
 *     router launch computes: four launches (five above 512 (token, slot) pairs, where a grouping
 *     launch runs first), none of the shared expert's own. */
int lq4_moe_ffn(lq4_ctx* ctx, const float* router_logits_dev, const lq4_weight* gate_up, const lq4_weight* down,
                uint32_t num_experts, uint32_t top_k, uint32_t inter, const lq4_weight* shared_gate_up,
                const lq4_weight* shared_down, const float* shared_gate_dev, uint32_t shared_inter,
                uint32_t hidden, const float* x_dev, uint32_t tokens, float* y_dev, void* stream);

/* ---- lm_head top-k ------------------------------------------------------------
 * Exact top-k over `n` f32 logits in the reference's candidate order (higher logit first,
 * ties to the lower token id, NaN last as the (-inf, 0xFFFFFFFF) sentinel): the result of
 * logits_topk_first_pass + logits_topk_merge_pass (shaders/qwen35.metal:1683-1778, driven by
 * dispatch_topk_enc, inner/dispatch.rs:1425-1500).  out_logits_dev / out_ids_dev receive top_k
 * entries in rank order; slots beyond the number of non-NaN logits hold sentinels.
 * top_k <= LQ4_MAX_TOP_K. */
int lq4_topk(lq4_ctx* ctx, const float* logits_dev, uint32_t n, uint32_t top_k, float* out_logits_dev,
             uint32_t* out_ids_dev, void* stream);

/* Replaces the two-stage lm_head path: lm_head_block_topk_q4 (shaders/qwen35.metal:1935-1985,
 * dispatch_lm_head_block_stage1_enc, inner/dispatch.rs:1317-1373) followed by
 * dispatch_block_topk_merge_enc (inner/dispatch.rs:1378-1421).  logits = W[vocab, K] . x (batch-1
 * GEMV, f32-faithful) are kept in library scratch and never handed to the caller; the top_k
 * best (logit, token id) pairs come back in rank order.  Both stages are exact, so the result
 * equals lq4_gemv followed by lq4_topk.
 * The GEMV and the selection are two launches.  (A form that selected inside the GEMV's own launch, as
 * lm_head_block_topk_q4 computes its block candidates inside the GEMV kernel, existed and was removed: making the
 * logits visible to the selecting workgroup inside the launch - write-through stores, their acknowledgement, the
 * maximum's exchange and a ticket, one after the other at the end of every workgroup - cost more than the second
 * launch's pass over 1 MB of logits: 248 320 x 2048, top 50: 82.9 us against 76.7.) */
int lq4_lm_head_topk(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t vocab, uint32_t k,
                     const float* x_dev, uint32_t top_k, float* out_logits_dev, uint32_t* out_ids_dev,
                     void* stream);

/* lq4_lm_head_topk for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it).  No counterpart in the reference.  Same
 * arguments, same result bit for bit; the logits and the candidate buffers live in a fixed
 * LQ4_STATIC_SCRATCH_BYTES array inside the library's device code instead of the context's growable
 * scratch, so the call makes no hipMalloc / hipFree and calls no allocating routine.  Shapes whose
 * scratch (vocab * 4 bytes, rounded up to 256, plus the selection's candidate buffers) does not fit
 * return LQ4_E_UNSUPPORTED: vocabularies up to 262 144 with top_k <= 256 fit.  Every context on one
 * GPU shares that GPU's array: calls of one context on alternating streams are ordered like its other
 * calls (see lq4_ctx_create), calls of two contexts that overlap on one GPU race. */
#define LQ4_STATIC_SCRATCH_BYTES (2u << 20)
int lq4_lm_head_topk_static(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t vocab, uint32_t k,
                            const float* x_dev, uint32_t top_k, float* out_logits_dev, uint32_t* out_ids_dev,
                            void* stream);

/* ---- elementwise steps either side of the decode GEMVs ---------------------------
 * Shifted RMSNorm of Qwen3.5 with the residual add in front of it: v = base + delta (delta may be
 * NULL: plain norm), residual_out = v (skipped if NULL), normed_out = v * rsqrt(mean(v^2) + eps) *
 * (1 + gamma).  Replaces dispatch_fused_residual_add_norm / _batch (inner/dispatch.rs:1171-1266,
 * shaders/qwen35.metal:739-767, 2219-2249) and dispatch_rms_norm (inner/dispatch.rs:525; CPU form
 * qwen35_rms_norm, model/qwen35/norm.rs:6-23).  `rows` rows of `hidden` floats. */
int lq4_residual_add_rmsnorm(lq4_ctx* ctx, const float* base_dev, const float* delta_dev, const float* gamma_dev,
                             uint32_t hidden, uint32_t rows, float eps, float* residual_out_dev,
                             float* normed_out_dev, void* stream);

/* out[r, i] = silu(gate_up[r, i]) * gate_up[r, count + i] for rows of [gate(count) | up(count)];
 * out rows are out_stride floats apart (out == gate_up with out_stride == 2 * count is the
 * in-place form of silu_mul_fused, shaders/qwen35.metal:712-722, dispatch_silu_mul_fused
 * inner/dispatch.rs:916-930). */
int lq4_silu_mul(lq4_ctx* ctx, const float* gate_up_dev, uint32_t count, uint32_t rows, float* out_dev,
                 uint32_t out_stride, void* stream);

/* residual += src; dst = residual (dst may be NULL).  Replaces dispatch_add_and_copy
 * (inner/dispatch.rs:1268-1290, shaders/qwen35.metal:2255-2266). */
int lq4_add_and_copy(lq4_ctx* ctx, const float* src_dev, float* residual_dev, float* dst_dev, size_t count,
                     void* stream);

/* The same steps fused into the batch-1 GEMV, so that a decode MLP is two launches
 * (norm + gate||up GEMV, then silu*up + down GEMV + residual add) instead of five. */
#define LQ4_PRO_NONE 0        /* activations = x_dev[K] */
#define LQ4_PRO_ADD_RMSNORM 1 /* activations = shifted RMSNorm(base + delta); x_dev is ignored */
#define LQ4_PRO_SILU_MUL 2    /* activations = silu(x_dev[0..K)) * x_dev[K..2K) */
#define LQ4_EPI_NONE 0        /* y_dev[N] = W . activations (+ LoRA) */
#define LQ4_EPI_ADD_RESIDUAL 1 /* also residual[N] += that; copy_dst[N] = residual (if not NULL);
                                  y_dev may then be NULL */
/* LQ4_EPI_SILU_MUL_PAIRS (2, defined with the chain below): W = [N/2 gate rows | N/2 up rows] and
 * y_dev[N/2] receives silu(W_i . activations) * (W_(N/2+i) . activations), the dispatch_silu_mul_fused
 * that follows the gate||up GEMV (inner/dispatch.rs:916-930): a wave takes the two rows of a pair, so
 * the [gate | up] vector never reaches memory.  One row only (lq4_gemv_fused, lq4_gemv_chain). */
typedef struct lq4_gemv_fusion {
    int prologue;
    const float* base;   /* ADD_RMSNORM: [K] */
    const float* delta;  /* ADD_RMSNORM: [K] or NULL */
    const float* gamma;  /* ADD_RMSNORM: [K] */
    float eps;
    float* residual_out; /* ADD_RMSNORM: [K] or NULL; must not overlap base or delta */
    int epilogue;
    float* residual;     /* ADD_RESIDUAL: [N], updated in place */
    float* copy_dst;     /* ADD_RESIDUAL: [N] or NULL */
} lq4_gemv_fusion;

/* lq4_gemv at batch 1 with the elementwise steps above applied while the activations are staged
 * and while the result is stored.  Equals the unfused sequence lq4_residual_add_rmsnorm /
 * lq4_silu_mul -> lq4_gemv -> lq4_add_and_copy to f32 rounding (the sum of squares is formed in a
 * different order).  Shapes or options the fused kernel does not take (K too long for LDS, a LoRA
 * adapter together with a prologue, LQ4_EPI_SILU_MUL_PAIRS with K of 512 or 1024 or with an
 * adapter) run as exactly that sequence through library scratch. */
int lq4_gemv_fused(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                   const float* x_dev, float* y_dev, const lq4_gemv_fusion* fusion, const lq4_lora* lora,
                   float lora_scale, void* stream);

/* lq4_gemv_fused for `batch` activation rows (1 <= batch <= LQ4_MAX_GEMV_BATCH), the decode
 * steps of several sequences at once; the batched elementwise shaders it folds in are
 * fused_residual_add_norm_batch (shaders/qwen35.metal:2219-2249, dispatch_fused_residual_add_norm_batch,
 * inner/dispatch.rs:1171-1266) and silu_mul_fused over rows (shaders/qwen35.metal:712-722).  Every
 * per-row array is dense: fusion->base, delta and residual_out are [batch, K]; gamma is [K] and shared;
 * x_dev is [batch, K] (LQ4_PRO_NONE) or [batch, 2K] rows of [gate | up] (LQ4_PRO_SILU_MUL); y_dev,
 * fusion->residual and copy_dst are [batch, N].  batch == 1 is lq4_gemv_fused.  For 2..8 rows the
 * epilogue runs inside the small-batch GEMV's launch, and so does the prologue while its input is
 * at most 64 KB (each workgroup forms 1/rms of every row, one wave per row, before it stages the
 * rows; every workgroup repeats that work, so beyond a few rows one stand-alone launch is cheaper
 * and the library runs that instead).  More than 8 rows, K too long for LDS, or a LoRA adapter run
 * as the unfused sequence through library scratch.  Same results as that sequence to f32 rounding. */
int lq4_gemv_fused_batch(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                         const float* x_dev, uint32_t batch, float* y_dev, const lq4_gemv_fusion* fusion,
                         const lq4_lora* lora, float lora_scale, void* stream);

/* ---- a chain of one-token GEMVs behind one call ------------------------------------------------
 * The reference encodes a whole token into one command buffer (forward_step,
 * forward/metal_qwen35.rs:6943, committed once at :6447): o -> residual add + RMSNorm -> gate||up ->
 * silu * up -> down -> residual add + next layer's RMSNorm -> qkv follow each other without the host
 * in between (encode_mlp_block, inner/layers/mod.rs; the elementwise dispatches at
 * inner/dispatch.rs:916-930, 1171-1290).  lq4_gemv_chain is that unit here: up to
 * LQ4_CHAIN_MAX_STEPS batch-1 GEMVs, each fed by an external vector or by an earlier step's result,
 * behind one call.  Every step is one fused launch (lq4_gemv_fused: the elementwise work rides in the
 * GEMV's prologue and epilogue; only a step that ends in silu * up on rows too short for the fused form
 * runs the stand-alone silu * up kernel).  Results that no step's y_dev asks for live in library scratch.
 *
 * Step j computes r_j = epilogue(W_j . prologue(...)):
 *   prologue   LQ4_PRO_NONE         activations = x_dev [K], or r_(j-1) when from_previous != 0
 *              LQ4_PRO_ADD_RMSNORM  v = base + delta as in lq4_gemv_fusion (base or delta may be NULL),
 *                                   with r_(j-1) in the place of delta when from_previous != 0;
 *                                   activations = v * rsqrt(mean(v^2) + eps) * (1 + gamma);
 *                                   residual_out (if not NULL, no overlap with base/delta) = v
 *                                   (dispatch_fused_residual_add_norm, inner/dispatch.rs:1171-1266)
 *              LQ4_PRO_SILU_MUL     activations = silu(x_dev[0..K)) * x_dev[K..2K), external only
 *   epilogue   LQ4_EPI_NONE           r = W . x                          [N]
 *              LQ4_EPI_ADD_RESIDUAL   r = residual + W . x, residual = r [N]  (dispatch_add_and_copy)
 *              LQ4_EPI_SILU_MUL_PAIRS r[i] = silu(y[i]) * y[i + N/2]     [N/2] for W = [gate rows | up
 *                                     rows], the fused buffer of metal_qwen35.rs:12137-12152
 *                                     (dispatch_silu_mul_fused)
 *   y_dev      receives r_j when not NULL (the last step needs y_dev or a residual).
 * With from_previous the step's K must equal the length of r_(j-1).  Any input vector (x_dev, base,
 * delta) may also be the y_dev or residual_out of an earlier step of the same chain.  Vectors of
 * different steps must be identical or disjoint.  The call keeps intermediate results in the context:
 * chains must not overlap on two streams of one context. */
#define LQ4_CHAIN_MAX_STEPS 16
#define LQ4_EPI_SILU_MUL_PAIRS 2
typedef struct lq4_chain_step {
    const lq4_weight* w;
    uint64_t w_extra_offset;
    uint32_t n, k;
    int from_previous;
    const float* x_dev;
    int prologue;
    const float* base;
    const float* delta;
    const float* gamma;
    float eps;
    float* residual_out;
    int epilogue;
    float* residual;
    float* y_dev;
} lq4_chain_step;
int lq4_gemv_chain(lq4_ctx* ctx, const lq4_chain_step* steps, uint32_t n_steps, void* stream);

/* Grows every scratch buffer of the context (partial tiles of K-sliced GEMMs, packed few-token operands,
 * MoE and shared-expert intermediates, lm_head logits, the results a chain keeps between its steps) to at
 * least `bytes` ahead of time.  The library grows them on demand
 * otherwise, which allocates: a call that would have to grow it while its stream is being captured
 * into a HIP graph returns LQ4_E_UNSUPPORTED instead.  Outgrown buffers stay allocated until
 * lq4_ctx_destroy, so launches already queued or captured keep valid addresses.  No counterpart in
 * the reference. */
int lq4_ctx_reserve_scratch(lq4_ctx* ctx, size_t bytes);

/* ---- Q8_0 sibling format -----------------------------------------------------------
 * 34-byte blocks [u16 f16 scale d][32 x i8], w = q * d, rows of K/32 blocks, 2-byte aligned
 * (forward/metal_qwen35.rs:2310-2346).  Weight handles are format-agnostic byte buffers: upload
 * Q8_0 blocks with lq4_weight_upload(..., validate = 0) or wrap them with lq4_weight_wrap.
 * lq4_gemv_q8 replaces dispatch_matmul_q8 (inner/dispatch.rs:61-84; batch 1 is the decode GEMV,
 * batch <= 16 rows take the tile kernel), lq4_gemm_q8 replaces dispatch_gemm_q8
 * (inner/dispatch.rs:86-146): same conventions as lq4_gemv / lq4_gemm, no LoRA argument (apply
 * lq4_lora_apply afterwards). */
int lq4_gemv_q8(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                const float* x_dev, uint32_t batch, float* y_dev, void* stream);
int lq4_gemm_q8(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                const void* x_dev, int x_dtype, uint32_t m, float* y_dev, void* stream);

/* ---- Q3 sibling format --------------------------------------------------------------
 * 16-byte blocks [u16 f16 scale][u16 f16 bias][8 bytes low-2-bit plane][4 bytes high-1-bit
 * plane], w = (low2 | hi << 2) * scale + bias, rows of K/32 blocks, 4-byte aligned
 * (weights/q3_weights.rs:13-52).  Upload with lq4_weight_upload(..., validate = 0) or wrap.
 * lq4_gemv_q3 / lq4_gemm_q3 replace dispatch_matmul_q3 / dispatch_gemm_q3
 * (inner/dispatch.rs:269-325): same conventions as the Q8_0 pair above. */
int lq4_gemv_q3(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                const float* x_dev, uint32_t batch, float* y_dev, void* stream);
int lq4_gemm_q3(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                const void* x_dev, int x_dtype, uint32_t m, float* y_dev, void* stream);

/* ---- probes --------------------------------------------------------------------
 * Writes f32(nibble)*scale + bias for every weight of W[N,K] to out_dev (f32 [N,K]):
 * the bit-exactness probe for nibble unpack and scale/bias indexing against
 * dequantize_row_q4_0 (q4_weights.rs:340-353). */
int lq4_dequant(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n,
                uint32_t k, float* out_dev, void* stream);

/* Calibration: one launch that only streams `nbytes` (16-byte aligned buffer) through the
 * vector memory path.  Timing it gives the read-bandwidth ceiling of this GPU at that
 * launch size, the figure the GEMV kernels are held against.  No counterpart in the
 * reference. */
int lq4_probe_read(lq4_ctx* ctx, const void* p_dev, size_t nbytes, void* stream);
/* The same with the launch spelled out, for sweeps: `workgroups` of 256 threads (0: the library's
 * choice), 64 / 128 / 256 bytes in flight per thread, workgroups interleaved at 4 KB x (bytes / 16)
 * granularity (`strided`) or one contiguous chunk each, plain or non-temporal loads.  lq4_probe_read
 * is (0, 128, strided, non-temporal), the fastest of the sweep from 8 MB to 1 GB. */
int lq4_probe_read_config(lq4_ctx* ctx, const void* p_dev, size_t nbytes, uint32_t workgroups, uint32_t bytes_in_flight,
                          int strided, int nontemporal, void* stream);

/* Which kernel serves y = W . x for one token without LoRA (lq4_gemv at batch 1, the GEMV of
 * lq4_lm_head_topk in two launches, a one-row step of lq4_gemv_chain without LoRA).  Per context; a new
 * context starts from the environment variable LQ4_GEMV_KERNEL, else AUTO.
 *   AUTO        by shape: the LDS-ring kernel where it is measured faster (rows of at least 2048 weights and
 *               20 MB of weights in at least 3072 rows, 6 MB when K is not a multiple of 2048, 12 MB at
 *               K = 4096), else the lane-owns-block kernel
 *   LANE_BLOCKS always the kernel in which each lane loads its own blocks into registers
 *   LDS_RING    the kernel that streams whole 1280-byte slabs into a per-wave ring of LDS slots wherever the
 *               shape fits it (K <= 24576), else the other one
 * Both accumulate a row's blocks in the same order inside a slab; results agree to the contract's tolerance
 * and are bit-identical for rows of one slab (K <= 2048).  No counterpart in the reference. */
enum { LQ4_GEMV_KERNEL_AUTO = 0, LQ4_GEMV_KERNEL_LANE_BLOCKS = 1, LQ4_GEMV_KERNEL_LDS_RING = 2 };
int lq4_set_gemv_kernel(lq4_ctx* ctx, int which);

/* Tuning/test hook, per context (a new context starts from the environment variable LQ4_GEMM_KERNEL,
 * else 0): 0 = lq4_gemm picks its kernel by shape (default), 1 = always
 * the LDS-staged tile kernel, 2 = always the weights-in-registers kernel, 3 = always the
 * few-token kernel, 4 = always the weights-in-registers kernel at two workgroups per CU (Q4 without
 * LoRA; packs the activations into scratch first).  Results are identical in contract either way.
 * No counterpart in the reference. */
int lq4_set_gemm_kernel(lq4_ctx* ctx, int which);

/* Calibration: plain device copy of `nbytes` (both buffers 16-byte aligned, nbytes a multiple
 * of 16).  It reads and writes exactly nbytes, which scales the memory-traffic counters of a
 * profiler run.  No counterpart in the reference. */
int lq4_probe_copy(lq4_ctx* ctx, const void* src_dev, void* dst_dev, size_t nbytes, void* stream);

/* Launch counters per kernel family since context creation (the role of
 * PathProofCounters, metal_qwen35.rs:2144-2190): proves which path served a call. */
typedef struct lq4_path_counters {
    uint64_t gemv, gemm, lora_a, moe_route, moe_gate_up, moe_down, dequant, topk, gemv_fused, elementwise;
    uint64_t gemv_chain;       /* lq4_gemv_chain calls (each of their steps also counts under gemv_fused) */
    uint64_t lora_t_fallback;  /* waves of one-token LoRA launches that computed A.x themselves because
                                  the producers' hand-over did not arrive in time (read from the device:
                                  this call waits for the GPU) */
    uint64_t gemv_multi;       /* lq4_gemv_multi calls served by one stacked launch */
} lq4_path_counters;
int lq4_get_path_counters(const lq4_ctx* ctx, lq4_path_counters* out);

/* ---- plain device-memory helpers for callers without a HIP binding ------------ */
int lq4_malloc(lq4_ctx* ctx, size_t nbytes, void** out_dev);
int lq4_free(lq4_ctx* ctx, void* p_dev);
int lq4_memcpy_h2d(lq4_ctx* ctx, void* dst_dev, const void* src_host, size_t nbytes);
int lq4_memcpy_d2h(lq4_ctx* ctx, void* dst_host, const void* src_dev, size_t nbytes);

#ifdef __cplusplus
}
#endif
#endif /* LATTICE_HIP_Q4_H */
