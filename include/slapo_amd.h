/*
 * slapo_amd.h -- C ABI of libslapo_amd.so: the gfx950 (MI355X / CDNA4) kernels behind
 * Slapo's fused-op hot path (slapo.op attention + FusedMLP epilogues + dropout RNG).
 *
 * The reference (awslabs/slapo) is pure Python and has no FFI of its own: the points where it
 * leaves Python for a fused kernel are third-party calls.  Every entry point below names the
 * reference call site whose callee it replaces.  All entry points
 *   - take plain device pointers, sizes, strides and a hipStream_t passed as void*;
 *   - never allocate or free memory (workspaces are caller-provided, except for
 *     slapo_amd_attn_bwd_static_scratch, whose workspace is an array inside the library);
 *   - are stateless and re-entrant; they enqueue work on `stream` and return without
 *     synchronising;
 *   - return 0 on success or a negative SLAPO_ERR_* code (see slapo_amd_status_string).
 *
 * Tensors: q/k/v/o/do/dq/dk/dv are logically [batch, seqlen, heads, head_dim] with head_dim
 * contiguous; the three outer strides are given in elements, so the fused-QKV GEMM output
 * ([B,S,H,3D] view, reference slapo/op/attention.py:469-481) can be consumed without copies.
 */
#ifndef SLAPO_AMD_H
#define SLAPO_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SLAPO_AMD_ABI_VERSION 3

/* status codes */
#define SLAPO_OK 0
#define SLAPO_ERR_DTYPE (-1)     /* unsupported element type                               */
#define SLAPO_ERR_SHAPE (-2)     /* unsupported / inconsistent sizes (e.g. head_dim > 128) */
#define SLAPO_ERR_ALIGN (-3)     /* pointer or stride not aligned as the kernel requires   */
#define SLAPO_ERR_ARG (-4)       /* null pointer / out-of-range scalar argument            */
#define SLAPO_ERR_LAUNCH (-5)    /* hipLaunch / hipGetLastError reported a failure         */
#define SLAPO_ERR_DEVICE (-6)    /* no usable gfx950 device                                */
#define SLAPO_ERR_WORKSPACE (-7) /* caller workspace missing or too small                  */

/* element types */
#define SLAPO_F32 0
#define SLAPO_F16 1
#define SLAPO_BF16 2

int slapo_amd_abi_version(void);
const char* slapo_amd_status_string(int status);

/* ------------------------------------------------------------------------------------------
 * Dropout RNG (Philox4x32-10 with ATen's element <-> (subsequence, counter, lane) mapping).
 *
 * Replaces: the ATen native_dropout launch reached from torch.nn.functional.dropout at
 * slapo/op/fused_bias.py:74 (bias_dropout) and slapo/op/attention.py:179-180 (xformers_ref).
 * The mask is a pure function of (seed, offset, plan), so it can be regenerated in backward
 * and under activation-checkpoint recompute (slapo/checkpoint.py:79-92).
 *
 * (seed, offset) normally travel by value with the call.  A caller whose launches are replayed
 * (a captured HIP graph) sets plan.rng_state to 16 bytes of device memory holding {seed, offset}
 * as two uint64 instead: every kernel of the call then reads the pair from there when it runs,
 * the by-value seed / offset of the call are ignored, and what writes those 16 bytes (ordered
 * before the call on its stream, e.g. a random-number kernel captured into the same graph)
 * decides the mask of each replay.  slapo_amd_dropout_plan[_for] leave the field NULL; the host
 * mirror slapo_amd_dropout_mask_host refuses a plan that has it set (SLAPO_ERR_ARG).  This is
 * what stands in for the device-side (seed, offset) that ATen's generator hands a captured
 * launch (the reference's F.dropout calls capture; slapo/op/fused_bias.py:74).
 * ---------------------------------------------------------------------------------------- */
typedef struct slapo_dropout_plan {
    int64_t numel;            /* elements of the tensor the mask is drawn for                  */
    int64_t total_threads;    /* T = 256 * grid: Philox subsequences in use                     */
    int32_t vec;              /* elements handled per subsequence per loop trip: 1,2,4,8,16     */
    int32_t calls_per_iter;   /* Philox calls per loop trip = ceil(vec/4) (1 when vec == 1)     */
    int64_t offset_increment; /* amount the generator's offset must be advanced after the draw */
    const void* rng_state;    /* NULL, or a device address of two uint64 {seed, offset}: see above */
} slapo_dropout_plan;

/* Host Philox4x32-10 block function (10 rounds).  Pure host code; usable without a GPU. */
void slapo_amd_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);

/* Launch geometry ATen would choose for a dense tensor of `numel` elements of `elem_bytes`
 * bytes whose data pointer is aligned to `ptr_align` bytes, on a device with `num_cus`
 * compute units and `max_threads_per_cu` resident threads per CU.  Pure host code. */
int slapo_amd_dropout_plan_for(int64_t numel, int elem_bytes, int64_t ptr_align, int num_cus,
                               int max_threads_per_cu, slapo_dropout_plan* plan);

/* Same, reading num_cus / max_threads_per_cu from HIP device `device`. */
int slapo_amd_dropout_plan(int64_t numel, int elem_bytes, int64_t ptr_align, int device,
                           slapo_dropout_plan* plan);

/* Largest 32-bit Philox output that is KEPT for drop probability p (keep iff
 * 2^-32 + float(v) * 2^-32 < (float)(1.0 - p)); *keep_all is set when every output is kept and
 * *keep_none when none is.  Pure host code. */
uint32_t slapo_amd_dropout_threshold(double p, int* keep_all, int* keep_none);

/* Host mirror: mask[i] = 1 if element i is kept.  Pure host code (test / debugging aid). */
int slapo_amd_dropout_mask_host(uint8_t* mask, const slapo_dropout_plan* plan, double p,
                                uint64_t seed, uint64_t offset);

/* Device version of the same (mask is a device pointer to numel bytes). */
int slapo_amd_dropout_mask(uint8_t* mask, const slapo_dropout_plan* plan, double p,
                           uint64_t seed, uint64_t offset, void* stream);

/* ------------------------------------------------------------------------------------------
 * FusedMLP epilogues.  x / y / out / grads are [rows, cols] row-major with row stride == cols;
 * bias is [cols].  dtype is one of SLAPO_F32 / SLAPO_F16 / SLAPO_BF16 for all tensors of a call.
 * ---------------------------------------------------------------------------------------- */

/* out = gelu_tanh(y + bias).
 * Replaces: BiasGeLUFunction.bias_gelu (slapo/op/fused_bias.py:18-21) reached from
 * LinearWithAct.forward (slapo/op/linear.py:184-188); also bias_new_gelu (fused_bias.py:63-64). */
int slapo_amd_bias_gelu_fwd(const void* y, const void* bias, void* out, int64_t rows,
                            int64_t cols, int dtype, void* stream);

/* Bytes of fp32 workspace the two backward epilogues need for the column (bias) reduction. */
size_t slapo_amd_colsum_workspace_bytes(int64_t rows, int64_t cols);

/* dx = dgelu_tanh(y + bias) * grad;  dbias[c] = sum_r dx[r, c]  (dbias may be NULL).
 * Replaces: BiasGeLUFunction.bias_gelu_back + autograd's broadcast reduction of the bias
 * gradient (slapo/op/fused_bias.py:26-34, 42-46). */
int slapo_amd_bias_gelu_bwd(const void* grad, const void* y, const void* bias, void* dx,
                            void* dbias, void* workspace, size_t workspace_bytes, int64_t rows,
                            int64_t cols, int dtype, void* stream);

/* out = dropout(x + bias, p) [+ residual]   (residual may be NULL; p == 0 disables dropout).
 * The mask is the one torch.nn.functional.dropout would draw for the [rows, cols] tensor under
 * generator state (seed, offset) and launch plan `plan` (ignored when p == 0).
 * Replaces: bias_dropout (slapo/op/fused_bias.py:67-74) reached from LinearWithDropout.forward
 * (slapo/op/linear.py:252-258); with residual, the fusion pattern of tests/test_fusion.py:179-180. */
int slapo_amd_bias_dropout_residual_fwd(const void* x, const void* bias, const void* residual,
                                        void* out, int64_t rows, int64_t cols, int dtype,
                                        double p, uint64_t seed, uint64_t offset,
                                        const slapo_dropout_plan* plan, void* stream);

/* dx = grad * mask / (1 - p);  dbias[c] = sum_r dx[r, c] (dbias may be NULL).  The residual
 * gradient is `grad` itself and needs no kernel.  Replaces: autograd of the same pattern. */
int slapo_amd_bias_dropout_residual_bwd(const void* grad, void* dx, void* dbias,
                                        void* workspace, size_t workspace_bytes, int64_t rows,
                                        int64_t cols, int dtype, double p, uint64_t seed,
                                        uint64_t offset, const slapo_dropout_plan* plan,
                                        void* stream);

/* y = layer_norm(z) * gamma + beta with z = dropout(x + bias, p) + residual over rows of `cols`
 * elements (biased variance, rstd = 1 / sqrt(var + eps), as torch.nn.LayerNorm); the mask is the
 * one torch.nn.functional.dropout would draw for the [rows, cols] tensor.  bias and residual may
 * be NULL.  z is rounded to the tensor type before the statistics are taken, as the unfused
 * modules do.  Optional outputs for the backward: z [rows, cols], mean and rstd [rows] fp32
 * (each may be NULL).  Needs cols % (16 / element size) == 0, 16-byte aligned pointers
 * (SLAPO_ERR_ALIGN) and cols <= 8192 for the 16-bit types, 4096 for fp32 (SLAPO_ERR_SHAPE).
 * Replaces: the fused module that `.fuse()` builds for the pattern
 * F.layer_norm(F.dropout(x + bias) + residual) in tests/test_fusion.py:157-204 and
 * docs/source/scripts/attention-single-gpu.py:333-346. */
int slapo_amd_bias_dropout_residual_ln_fwd(const void* x, const void* bias, const void* residual,
                                           const void* gamma, const void* beta, void* z, void* y,
                                           float* mean, float* rstd, int64_t rows, int64_t cols,
                                           int dtype, double eps, double p, uint64_t seed,
                                           uint64_t offset, const slapo_dropout_plan* plan,
                                           void* stream);

/* Bytes of fp32 workspace the backward below needs when any of dgamma / dbeta / dbias is asked
 * for: one partial row triple per 16 rows. */
size_t slapo_amd_ln_bwd_workspace_bytes(int64_t rows, int64_t cols);

/* Backward of slapo_amd_bias_dropout_residual_ln_fwd from grad_y and the saved z, mean, rstd:
 * dresidual = dz, dx = dz * mask / (1 - p), dgamma / dbeta / dbias = column sums (two-stage, no
 * atomics).  Every output may be NULL (at least one must not be).  Replaces: autograd of the same
 * pattern. */
int slapo_amd_bias_dropout_residual_ln_bwd(const void* grad_y, const void* z, const float* mean,
                                           const float* rstd, const void* gamma, void* dx,
                                           void* dresidual, void* dgamma, void* dbeta,
                                           void* dbias, void* workspace, size_t workspace_bytes,
                                           int64_t rows, int64_t cols, int dtype, double p,
                                           uint64_t seed, uint64_t offset,
                                           const slapo_dropout_plan* plan, void* stream);

/* ------------------------------------------------------------------------------------------
 * Vocab-parallel cross entropy, the part computed on one shard [rows, vocab] of the logits
 * (vocabulary ids vocab_start .. vocab_start + vocab - 1).  Replaces the tensor passes of
 * _VocabParallelCrossEntropy.forward / .backward (slapo/op/cross_entropy.py:21-124).
 *
 * Forward, one read of the logits: per row the local maximum row_max, sum_exp = sum exp(x -
 * row_max), predicted = logit of target[row] if it lies in this shard (else 0) and sum_logits =
 * sum x (for label smoothing); all fp32 [rows].  The tensor-parallel group combines them as
 * M = max row_max, S = sum sum_exp * exp(row_max - M), P = sum predicted (the reference's three
 * all-reduces, :25, :56, :62), loss = log S + M - P.
 * Backward, one read and one write: grad_logits = grad_loss * (exp(x - row_max) * inv_sum_exp
 * - [v == target] * (1 - s) - s / vocab) with the COMBINED row_max = M and inv_sum_exp = 1 / S and
 * s = label_smoothing * vocab / (vocab - 1) (:112-122).  target is int64; any dtype of SLAPO_*;
 * rows need no alignment beyond that of an element. */
int slapo_amd_vocab_ce_fwd(const void* logits, const int64_t* target, float* row_max,
                           float* sum_exp, float* predicted, float* sum_logits, int64_t rows,
                           int64_t vocab, int64_t vocab_start, int dtype, void* stream);
int slapo_amd_vocab_ce_bwd(const void* logits, const int64_t* target, const float* row_max,
                           const float* inv_sum_exp, const float* grad_loss, void* grad_logits,
                           int64_t rows, int64_t vocab, int64_t vocab_start,
                           double label_smoothing, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Attention:  O = dropout(softmax(Q K^T * scale + bias + mask)) V, forward and backward.
 *
 * Replaces: the attn_fn callees of FlashAttentionOp.forward -- xformers
 * memory_efficient_attention (slapo/op/attention.py:315), flash-attn Triton flash_attn_func
 * (:328-336) and flash_attn_unpadded_func (:353-364); semantics pinned by the native
 * restatements xformers_ref (:134-196) and flash_attn_ref (:39-131).
 * ---------------------------------------------------------------------------------------- */
typedef struct slapo_attn_params {
    int32_t dtype;    /* SLAPO_F16 / SLAPO_BF16 (MFMA kernels) or SLAPO_F32 (fp32 FMA kernels)  */
    int32_t batch;
    int32_t heads;
    int32_t seqlen_q;
    int32_t seqlen_k;
    int32_t head_dim; /* <= 128 and a multiple of 8 for 16-bit types; <= 128 for fp32           */
    int32_t causal;   /* key j visible to query i only if j <= i                                */
    int32_t window;   /* > 0: additionally i - j < window (local causal attention); 0 = off     */
    float scale;      /* softmax scale (reference default head_dim^-0.5)                        */
    float p_drop;     /* dropout probability on the attention matrix; 0 disables                */
    uint64_t seed;    /* Philox seed (generator seed)                                           */
    uint64_t offset;  /* Philox offset (generator offset at entry of forward)                   */
    /* element strides of [batch, seqlen, heads] for each tensor; head_dim stride is 1.  For the
     * 16-bit types: multiples of 8, and the seqlen stride in [0, 2^24) (SLAPO_ERR_ALIGN /
     * SLAPO_ERR_SHAPE otherwise) */
    int64_t q_strides[3];
    int64_t k_strides[3];
    int64_t v_strides[3];
    int64_t o_strides[3];
    /* additive fp32 bias addressed as bias[b*s0 + h*s1 + i*s2 + j*s3]; stride 0 broadcasts
     * (the reference's "b11k" layout is {Sk, 0, 0, 1}, "bhqk" is {H*Sq*Sk, Sq*Sk, Sk, 1}).
     * With s2 == 0 (the bias depends on the key only) the kernels stage the bias of a key tile
     * through LDS instead of reading it per score: pass a padding mask in that form. */
    int64_t bias_strides[4];
    /* launch plan of the dropout mask over the dense [batch*heads, seqlen_q, seqlen_k] fp32
     * probability tensor (only read when p_drop > 0).  With plan.rng_state set the kernels read
     * {seed, offset} from that device address and ignore the two fields above; a backward call
     * must then find the values its forward found there. */
    slapo_dropout_plan plan;
    /* Optional (may be NULL), 16-bit types with p_drop > 0 only: device buffer of
     * slapo_amd_attn_keep_mask_bytes(prm) bytes.  The forward call stores the dropout keep bits
     * in it (one bit per score; with window > 0 a kernel launched ahead of the forward kernel on
     * the same stream draws them and the forward kernel reads them), and a backward that is given
     * the same buffer reads them instead of drawing every Philox block again in both of its
     * kernels.  The results are bitwise the same with and without it.  Words whose keys no query
     * of the row's 32-query group can see under the causal mask are not written; with a window,
     * only the words that hold a key the row itself can see are (the rest is never applied to a
     * non-zero probability).  Layout: uint32 words [batch*heads][ceil(seqlen_k/32)][pitch],
     * pitch = seqlen_q rounded up to 4; bit j of word (bh, w, i) = keep(query i, key 32 w + j). */
    void* keep_mask;
} slapo_attn_params;

/* Size in bytes of the keep_mask buffer (0 when p_drop == 0 or the type is SLAPO_F32). */
size_t slapo_amd_attn_keep_mask_bytes(const slapo_attn_params* prm);

/* lse: [batch, heads, seqlen_q] fp32, natural-log sum-exp of the masked, scaled scores.  Bias
 * values at or below -5e8 (other than -inf) are one masking value; a query row that sees nothing
 * but keys masked with it attends to them uniformly, as in the reference's arithmetic, and its
 * lse slot holds n * 2^100 (n = number of those keys) for the backward, which gives such rows the
 * gradients of that uniform softmax.  The backward must therefore be given the same bias as the
 * forward: only its bias builds decode that value (the host cannot inspect lse, so a backward
 * called without the bias returns zero gradients for such rows without an error). */
int slapo_amd_attn_fwd(const slapo_attn_params* prm, const void* q, const void* k, const void* v,
                       const float* bias, void* o, float* lse, void* stream);

/* Workspace (bytes) the backward needs: fp32 delta = rowsum(dO * O), one value per query row. */
size_t slapo_amd_attn_bwd_workspace_bytes(const slapo_attn_params* prm);

/* dq/dk/dv use q_strides/k_strides/v_strides of a DENSE [B,S,H,D] layout given in
 * dq_strides/dk_strides/dv_strides; `dout` uses o_strides. */
int slapo_amd_attn_bwd(const slapo_attn_params* prm, const void* q, const void* k, const void* v,
                       const float* bias, const void* o, const void* dout, const float* lse,
                       void* dq, void* dk, void* dv, const int64_t dq_strides[3],
                       const int64_t dk_strides[3], const int64_t dv_strides[3], void* workspace,
                       size_t workspace_bytes, void* stream);

/* The backward runs as stages on `stream`, in this order:
 *   PREPARE  SLAPO_F32 only: delta = rowsum(dO * O) into the workspace (a no-op for 16-bit types);
 *   DQ       workgroups own query rows and write dq; for 16-bit types this stage also computes
 *            delta for its rows and stores it in the workspace;
 *   DKDV     workgroups own key rows and write dk, dv; reads delta from the workspace.
 * DQ and DKDV both recompute the probabilities from lse and write disjoint outputs: no atomics,
 * no zero-initialised accumulator, bitwise reproducible.  slapo_amd_attn_bwd runs all stages;
 * this entry point runs the stages named in `stages` (a bit-or of the constants below, executed
 * in the order above) so that a caller can time one of them.  Arguments are those of
 * slapo_amd_attn_bwd and must be the same across the calls of one backward pass.  For SLAPO_F32
 * both gradient stages are served by the FMA kernels (DKDV runs them all, DQ is a no-op). */
#define SLAPO_BWD_PREPARE 1
#define SLAPO_BWD_DKDV 2
#define SLAPO_BWD_DQ 4
#define SLAPO_BWD_ALL 7
int slapo_amd_attn_bwd_stages(const slapo_attn_params* prm, const void* q, const void* k,
                              const void* v, const float* bias, const void* o, const void* dout,
                              const float* lse, void* dq, void* dk, void* dv,
                              const int64_t dq_strides[3], const int64_t dk_strides[3],
                              const int64_t dv_strides[3], void* workspace,
                              size_t workspace_bytes, int stages, void* stream);

/* slapo_amd_attn_bwd without the workspace arguments.  No counterpart in the reference: it is
 * for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  delta is kept in a 4 MiB array inside the library, one copy per device,
 * held until the process ends; the call itself allocates and frees nothing.  Limit:
 * batch * heads * seqlen_q <= 1 048 576, else SLAPO_ERR_WORKSPACE.  All calls on one device share
 * the array (every call overwrites the part it reads, so nothing has to be cleared): calls that
 * overlap in time on one device, on any streams, race.  Results are bitwise those of
 * slapo_amd_attn_bwd. */
int slapo_amd_attn_bwd_static_scratch(const slapo_attn_params* prm, const void* q, const void* k,
                                      const void* v, const float* bias, const void* o,
                                      const void* dout, const float* lse, void* dq, void* dk,
                                      void* dv, const int64_t dq_strides[3],
                                      const int64_t dk_strides[3], const int64_t dv_strides[3],
                                      void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SLAPO_AMD_H */
