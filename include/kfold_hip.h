/*
 * kfold_hip.h — C ABI of libkfold_hip.so: the MI355X (gfx950) backend for K-Fold's
 * Pairformer pair-update path (triangle multiplication, triangle attention, pair-bias
 * attention, transitions, block composition).
 *
 * The library is what a `kernel_backend="hip"` branch of the reference's modules binds
 * to; each entry point names the reference interface it replaces (paths relative to the
 * reference's src/kfold).  All pointers are device pointers unless stated otherwise.
 *
 * Conventions
 *   - every function returns 0 on success or a negative KFH_E* code; kfh_last_error()
 *     returns a thread-local message for the last failure on the calling thread;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); every call
 *     only enqueues work on it and never synchronises;
 *   - `io_dtype` / `w_dtype` select the element type of activations / source weights:
 *     KFH_BF16 (0) or KFH_F32 (1).  Arithmetic is bf16 MFMA with fp32 accumulation and fp32
 *     LayerNorm / softmax statistics (what the reference computes under its bf16 autocast,
 *     inference/runner.py:565-571); the pair-bias attention entry points also take
 *     `arith` = KFH_ARITH_F32 for the fp32 arithmetic the reference's diffusion stack runs in
 *     (model/model.py:419, fp32_dot_precision="ieee" in
 *     kernels/triton/attention_pair_bias/dispatch.py:439,453): every product is then carried
 *     to fp32 accuracy on the bf16 matrix cores by splitting each fp32 operand into three
 *     bf16 parts (six part products per k-step);
 *   - masks are one byte per element, non-zero = valid;
 *   - inputs are only read; `out` must not overlap an input unless the entry point says
 *     so (the `residual` arguments may alias `out`);
 *   - packed weights ("blobs") and workspaces are caller-owned device buffers of the
 *     sizes the *_bytes() queries return, 256-byte aligned; a blob is written once by the
 *     *_pack() call and is read-only afterwards, so it may be shared by concurrent calls;
 *     a workspace must not be shared by calls that may overlap in time.
 */
#ifndef KFOLD_HIP_H
#define KFOLD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KFH_BF16 0
#define KFH_F32 1

/* arithmetic of the pair-bias attention entry points; blobs, bias tiles and workspaces of one
 * arithmetic cannot be used with the other */
#define KFH_ARITH_BF16 0 /* bf16 operands, fp32 accumulation (bf16 autocast of the reference)   */
#define KFH_ARITH_F32 1  /* fp32-accurate products ("ieee"), for fp32 activations and weights   */

#define KFH_OK 0
#define KFH_EINVAL (-1)      /* bad argument (shape, dtype, null pointer, small workspace) */
#define KFH_EUNSUPPORTED (-2) /* valid request the kernels are not built for (e.g. C != 128) */
#define KFH_EHIP (-3)         /* a HIP runtime call failed; message holds hipGetErrorString */

#define KFH_OUTGOING 0
#define KFH_INCOMING 1

/* stage selectors of the *_forward_stages() entry points */
#define KFH_STAGE_IN 1   /* LayerNorm + input projections                      */
#define KFH_STAGE_CORE 2 /* the contraction (tri-mul) / the attention (tri-attn) */
#define KFH_STAGE_OUT 4  /* output projection, gate, residual                   */
#define KFH_STAGE_ALL 7

int kfh_version(void);
const char* kfh_last_error(void);

/* ---------------------------------------------------------------------------------------
 * Triangle multiplication (Algorithms 12/13).
 * Replaces kernels/triton/triangle_multiplication/ops.py:22 `precompute` and :49 `forward`
 * as called from model/primitives/triangle_multiplication.py:94-145
 * (`triton_triangluar_mult`); math of the torch path at :212-229 and :296-313.
 * ------------------------------------------------------------------------------------- */

/* Size of the packed-weight blob for channel count C (= hidden D). */
size_t kfh_trimul_packed_bytes(int C);

/* Pack one module's weights.  ln_* are [C]; p_in_w, g_in_w are [2C, C]; p_out_w, g_out_w are
 * [C, C]; all row-major [out, in] as in the reference's Linear (primitives/linear.py:35). */
int kfh_trimul_pack(const void* ln_in_w, const void* ln_in_b, const void* p_in_w,
                    const void* g_in_w, const void* ln_out_w, const void* ln_out_b,
                    const void* p_out_w, const void* g_out_w, int w_dtype, int C, void* blob,
                    void* stream);

/* Workspace for one call with N tokens: enough for one batch element, batch elements are then
 * processed in turn.  The *_batched size (>= the former) lets a call take all B elements through
 * every kernel at once where the path supports it (the widths assembled from the token-track
 * kernels, e.g. the C = 64 template stack, model/modules/apo_module.py:376-384 flattens templates
 * into the batch); kfh_trimul_forward picks that mode when workspace_bytes suffices for it. */
size_t kfh_trimul_workspace_bytes(int N, int C);
size_t kfh_trimul_workspace_bytes_batched(int B, int N, int C);

/* out[b,i,j,:] = (residual ? residual[b,i,j,:] : 0) + TriangleMultiplication(z, mask)[b,i,j,:]
 * z, out, residual: [B, N, N, C] contiguous, io_dtype.  mask: [B, N, N] bytes.
 * `residual` may be NULL and may alias `out`; `out` may alias `z` only if residual == z
 * (the in-place `z += update` of modules/apo_module.py:153-160). */
int kfh_trimul_forward(const void* z, const uint8_t* mask, const void* blob, const void* residual,
                       void* out, void* workspace, size_t workspace_bytes, int B, int N, int C,
                       int direction, float eps, int io_dtype, void* stream);

/* Same as kfh_trimul_forward but runs only the kernels selected by `stages` (an OR of
 * KFH_STAGE_*).  Later stages read what earlier ones left in `workspace` AND, for
 * KFH_STAGE_OUT, `z` again (the output gate sigmoid(W_go LN_in(z)) is recomputed from it):
 * every stage of one op must be given the same, unmodified z (a split around a write to z,
 * e.g. IN|CORE, then other work, then OUT with out == z, is the intended use — OUT reads a row
 * of z before it writes it).  For profiling, benchmarks of the individual kernels and callers
 * that order the write to `out` against other streams; no counterpart in the reference. */
int kfh_trimul_forward_stages(const void* z, const uint8_t* mask, const void* blob,
                              const void* residual, void* out, void* workspace,
                              size_t workspace_bytes, int B, int N, int C, int direction, float eps,
                              int io_dtype, int stages, void* stream);
/* The stages over a range of result rows: KFH_STAGE_CORE and KFH_STAGE_OUT take rows
 * [row0, row0 + nrows) of the result (out[b, i, :, :] for i in the range, both directions);
 * KFH_STAGE_IN always makes all rows and is called once, with row0 = 0, nrows = N.  For a caller
 * that overlaps the phases of one op: the contraction of one range on one stream beside the output
 * phase (LayerNorm, gate, projection, residual: memory-bound) of the range before on another,
 * ordered by the caller's events (the reference has no counterpart: its op is one call,
 * model/primitives/triangle_multiplication.py:212-229).  The ranges run the kernels of the whole op
 * on offset pointers: results have the bits of kfh_trimul_forward.  B = 1, C = 128 or 256; row0 a
 * multiple of kfh_trimul_row_granule(N, C) (the contraction's tile rows), nrows as well unless the
 * range ends at N. */
int kfh_trimul_row_granule(int N, int C);
int kfh_trimul_forward_rows(const void* z, const uint8_t* mask, const void* blob,
                            const void* residual, void* out, void* workspace,
                            size_t workspace_bytes, int B, int N, int C, int direction, float eps,
                            int io_dtype, int stages, int row0, int nrows, void* stream);

/* ---------------------------------------------------------------------------------------
 * Triangle attention around the starting / ending node (Algorithms 14/15).
 * Replaces kernels/triton/triangle_attention/ops.py:24 `precompute` and :56 `forward` as
 * called from model/primitives/triangle_attention.py:63-129 (`triton_triangular_attn`);
 * math of the torch path at :375-434, :246-335, :132-152.
 * ------------------------------------------------------------------------------------- */
size_t kfh_triattn_packed_bytes(int C, int H);

/* ln_* [C]; q_w, k_w, v_w, g_w [H*Dh, C] (mha.linear_{q,k,v,g}); bias_w [H, C] (`linear`);
 * o_w [C, H*Dh] (mha.linear_o).  The 1/sqrt(Dh) query scale is folded in here. */
int kfh_triattn_pack(const void* ln_w, const void* ln_b, const void* q_w, const void* k_w,
                     const void* v_w, const void* g_w, const void* bias_w, const void* o_w,
                     int w_dtype, int C, int H, void* blob, void* stream);

size_t kfh_triattn_workspace_bytes(int N, int C, int H);
/* as kfh_trimul_workspace_bytes_batched: all B elements through the projection kernels at once
 * (the attention core stays one launch per element: its pair bias is the element's) */
size_t kfh_triattn_workspace_bytes_batched(int B, int N, int C, int H);

/* out = (residual or 0) + TriangleAttention{Starting,Ending}Node(x, mask).
 * x, out, residual: [B, N, N, C]; mask: [B, N, N] bytes (mask[b,i,k] gates key k of row i;
 * for `ending` != 0 the op runs on the (i,j)-transposed x and mask and transposes the
 * result back, without materialising any transpose).  Masked keys get probability exactly
 * 0; a row whose keys are all masked attends uniformly over its N keys (the reference's
 * finite -1e9 semantics, triangle_attention.py:328).  Aliasing rules as for
 * kfh_trimul_forward. */
int kfh_triattn_forward(const void* x, const uint8_t* mask, const void* blob, const void* residual,
                        void* out, void* workspace, size_t workspace_bytes, int B, int N, int C,
                        int H, int ending, float eps, int io_dtype, void* stream);

/* Stage-selective variant, see kfh_trimul_forward_stages: KFH_STAGE_OUT of the C = 128, 4-head
 * path reads `x` again for the gate sigmoid(W_g LN(x)) (other widths keep their gate in the
 * workspace); give every stage the same, unmodified x. */
int kfh_triattn_forward_stages(const void* x, const uint8_t* mask, const void* blob,
                               const void* residual, void* out, void* workspace,
                               size_t workspace_bytes, int B, int N, int C, int H, int ending,
                               float eps, int io_dtype, int stages, void* stream);
/* As kfh_trimul_forward_rows: attention (KFH_STAGE_CORE) and output phase (KFH_STAGE_OUT) over the
 * attention rows [row0, row0 + nrows) — x[b, i] for the starting node, x[b, :, i] for the ending node
 * (model/primitives/triangle_attention.py:400-402) —, KFH_STAGE_IN over all rows.  B = 1, C = 128,
 * H = 4; a range has 48 rows at least when N >= 48 (the attention kernel of the whole op must take
 * the range as well, so that the bits are those of kfh_triattn_forward). */
int kfh_triattn_forward_rows(const void* x, const uint8_t* mask, const void* blob,
                             const void* residual, void* out, void* workspace,
                             size_t workspace_bytes, int B, int N, int C, int H, int ending,
                             float eps, int io_dtype, int stages, int row0, int nrows, void* stream);

/* ---------------------------------------------------------------------------------------
 * Transition (Algorithm 11, SwiGLU).  Replaces the torch modules
 * model/layers/folding/transition.py:48-68 + model/primitives/activation.py:27-29, which the
 * reference runs unfused on every backend.  C = 128 and C = 256 with expansion 2 or 4 (the
 * pair track of the Pairformer block and of the trunk's TriangularBlock,
 * model/modules/tri_stack.py:119-125) run as one fused kernel and need no workspace; other
 * channel counts (multiples of 32 up to 2048: the token track, the C = 64 template stack) run
 * as LayerNorm + two MFMA linears through the workspace.
 * ------------------------------------------------------------------------------------- */
size_t kfh_transition_packed_bytes(int C, int expansion);

/* ln_* [C]; swiglu_w [2*C*expansion, C] (`swiglu.linear`); out_w [C, C*expansion] (`linear_out`). */
int kfh_transition_pack(const void* ln_w, const void* ln_b, const void* swiglu_w, const void* out_w,
                        int w_dtype, int C, int expansion, void* blob, void* stream);

size_t kfh_transition_workspace_bytes(long long rows, int C, int expansion);

/* out[r,:] = ((residual ? residual[r,:] : 0) + Transition(x[r,:])) * (mask ? mask[r] != 0 : 1)
 * for r < rows; x, out, residual: [rows, C].  `out` may alias `x` and `residual`.  `mask`
 * (one byte per row, or NULL) is the final `z * pair_mask` of modules/apo_module.py:172. */
int kfh_transition_forward(const void* x, const void* blob, const void* residual, const uint8_t* mask,
                           void* out, void* workspace, size_t workspace_bytes, long long rows, int C,
                           int expansion, float eps, int io_dtype, void* stream);

/* The same computation for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  The library-internal scratch that kfh_transition_forward takes as `workspace`
 * (LayerNorm-ed rows and SwiGLU hidden activations, kfh_transition_workspace_bytes()) lives
 * in a static device array of kfh_transition_static_scratch_bytes() = 8 MiB per GPU, held until
 * the process ends; the call allocates and frees nothing.  Requests that need more scratch
 * fail with KFH_EINVAL (e.g. C = 384, expansion 4: up to 2184 rows).  All calls on one GPU
 * share the array: calls that may overlap in time on one GPU (different streams or threads)
 * race; calls on one stream are ordered.  Results are bit-identical to
 * kfh_transition_forward.
 * Set-up: kfh_transition_static_scratch_bytes() also resolves and keeps the array's address on
 * the CURRENT device; call it once per device (with that device current) before the first
 * kfh_transition_forward_static there if that first call must do no lookup (graph capture).
 * kfh_transition_forward_static uses the array of the current device: `stream` must belong to
 * the device that is current at the call. */
size_t kfh_transition_static_scratch_bytes(void);
int kfh_transition_forward_static(const void* x, const void* blob, const void* residual,
                                  const uint8_t* mask, void* out, long long rows, int C, int expansion,
                                  float eps, int io_dtype, void* stream);

/* ---------------------------------------------------------------------------------------
 * Pair bias of the token-track attention, as "bias tiles": the layout the attention
 * kernel reads, [batch][head][query block of 32][key block of 32][tile], values
 * pre-multiplied by log2(e); a tile is 2 KiB of bf16 (KFH_ARITH_BF16) or 4 KiB of fp32
 * (KFH_ARITH_F32); inside a tile the 1024 values are in the register order of the
 * kernel's transposed score accumulator (an opaque layout: produce tiles only with the
 * calls below).
 * ------------------------------------------------------------------------------------- */
size_t kfh_bias_tiles_bytes(int nbatch, int H, int L, int arith);

/* tiles <- dense pair bias [nbatch, H, L, L] (io_dtype), the `pair_bias` argument of
 * model/primitives/attention.py:28-37. */
int kfh_bias_tiles_from_dense(const void* dense, int io_dtype, void* tiles, int nbatch, int H, int L,
                              int arith, void* stream);

/* tiles <- linear_pair_bias(layernorm_z(z)) moved to [B, H, N, N]
 * (model/modules/confidence_head.py:162-163) in one pass over z [B, N, N, C]; w is [H, C].
 * bf16 tiles (KFH_ARITH_BF16): the confidence head and trunk run under autocast. */
size_t kfh_pair_bias_packed_bytes(int C, int H);
int kfh_pair_bias_pack(const void* ln_w, const void* ln_b, const void* w, int w_dtype, int C, int H,
                       void* blob, void* stream);
int kfh_pair_bias_project(const void* z, const void* blob, void* tiles, int B, int N, int C, int H,
                          float eps, int io_dtype, void* stream);

/* ---------------------------------------------------------------------------------------
 * Self attention with pair bias (Algorithm 24).  Replaces
 * kernels/triton/attention_pair_bias/dispatch.py:370 `triton_attention_pair_bias` as called
 * from model/primitives/attention.py:62-66, and with apply_norm != 0 the whole
 * `SelfAttentionPairBias.forward` (model/layers/folding/attention_pair_bias.py:114-158);
 * math of the torch path at attention.py:75-94, :239-271, :122-168.
 * C = channel_a, H heads of C/H (<= 64) channels, Cs = conditioning channels (0 = none).
 * ------------------------------------------------------------------------------------- */
size_t kfh_apb_packed_bytes(int C, int H, int Cs, int arith);

/* q_w,k_w,v_w,g_w,o_w [C, C]; q_b [C] or NULL (`linear_q.bias`); unconditioned: ln_w, ln_b [C]
 * (`layernorm_a`); conditioned (Cs > 0): adaln_s_w [Cs] (`adaln_a.layernorm_s.weight`),
 * adaln_g_w [C, Cs] + adaln_g_b [C] (`adaln_a.linear_g`), adaln_bias_w [C, Cs]
 * (`adaln_a.linear_bias`), ada_out_w [C, Cs] + ada_out_b [C] (`linear_ada_out`). */
int kfh_apb_pack(const void* ln_w, const void* ln_b, const void* q_w, const void* q_b, const void* k_w,
                 const void* v_w, const void* g_w, const void* o_w, const void* adaln_s_w,
                 const void* adaln_g_w, const void* adaln_g_b, const void* adaln_bias_w,
                 const void* ada_out_w, const void* ada_out_b, int w_dtype, int C, int H, int Cs,
                 int arith, void* blob, void* stream);

size_t kfh_apb_workspace_bytes(int S, int L, int C, int H, int Cs, int arith);

/* a, out, residual: [S, L, C]; s_cond: [S or 1, L, Cs]; bias_tiles: [S or 1] batches of tiles;
 * mask: [S or 1, L] bytes (valid keys); the *_per_sample flags say which of the two.
 * apply_norm = 0: `a` is already normalised (the functional entry, attention.py:28) and no
 * conditioning gate is applied; apply_norm != 0: LayerNorm (Cs = 0) or AdaLN + the
 * sigmoid(linear_ada_out(s)) output gate (Cs > 0) are applied as the module does.
 * out = (residual or 0) + result; `residual` may alias `out`, `out` must not alias `a`
 * unless residual == a.  Fully masked key sets give uniform attention (finite -1e9).
 * `arith` must be the one the blob, the bias tiles and the workspace size were made for. */
int kfh_apb_forward(const void* a, const void* s_cond, const void* bias_tiles, const uint8_t* mask,
                    const void* blob, const void* residual, void* out, void* workspace,
                    size_t workspace_bytes, int S, int L, int C, int H, int Cs, int apply_norm,
                    int bias_per_sample, int mask_per_sample, int s_per_sample, float eps,
                    int io_dtype, int arith, void* stream);

/* ---------------------------------------------------------------------------------------
 * Cross attention with pair bias over local windows: the whole
 * `CrossAttentionPairBias.forward` (model/layers/folding/attention_pair_bias.py:161-260; math of
 * model/primitives/attention.py:75-94, :239-271) of the atom transformer: W windows, each with
 * Lq queries (32) attending to Lk keys (128) under its own bias [H, Lq, Lk] and key mask [Lk].
 * C = channel_a (a multiple of 32), H heads of C/H <= 64 channels, Cs = conditioning channels
 * (0 = none, else a multiple of 16).  `arith` as for kfh_apb_*: KFH_ARITH_F32 is the fp32
 * ("ieee") arithmetic the reference selects for its diffusion stack (model/model.py:419).
 * ------------------------------------------------------------------------------------- */
size_t kfh_cross_apb_packed_bytes(int C, int H, int Cs, int arith);

/* unconditioned: lnq_*, lnk_* [C] (`layernorm_a_q`, `layernorm_a_k`); conditioned: adaq_* / adak_*
 * are `adaln_a_q` / `adaln_a_k` (`layernorm_s.weight` [Cs], `linear_g` [C, Cs] + bias [C],
 * `linear_bias` [C, Cs]) and ada_out_* is `linear_ada_out`.  q_w .. o_w [C, C], q_b [C] or NULL. */
int kfh_cross_apb_pack(const void* lnq_w, const void* lnq_b, const void* lnk_w, const void* lnk_b,
                       const void* q_w, const void* q_b, const void* k_w, const void* v_w, const void* g_w,
                       const void* o_w, const void* adaq_s_w, const void* adaq_g_w, const void* adaq_g_b,
                       const void* adaq_bias_w, const void* adak_s_w, const void* adak_g_w,
                       const void* adak_g_b, const void* adak_bias_w, const void* ada_out_w,
                       const void* ada_out_b, int w_dtype, int C, int H, int Cs, int arith, void* blob,
                       void* stream);

size_t kfh_cross_apb_workspace_bytes(int W, int Lq, int Lk, int C, int H, int Cs, int arith);

/* a_q, out, residual: [W, Lq, C]; a_k: [W, Lk, C]; s_q: [W, Lq, Cs], s_k: [W, Lk, Cs] (Cs > 0);
 * pair_bias: dense [W, H, Lq, Lk] of bias_dtype; mask: [W, Lk] bytes.
 * apply_norm != 0: the whole module (LayerNorm or AdaLN of both sides, attention, and with
 * Cs > 0 the sigmoid(linear_ada_out(s_q)) output gate); apply_norm = 0: a_q / a_k are already
 * normalised and s_q / s_k are ignored — the functional entry `attention_pair_bias(module, x_q,
 * x_k, ...)` of model/primitives/attention.py:28-94 with x_q != x_k, as
 * CrossAttentionPairBias.forward calls it (attention_pair_bias.py:250-258).
 * out = (residual or 0) + result; `residual` may alias `out`.  A window whose keys are all
 * masked attends uniformly over its Lk keys (finite -1e9). */
int kfh_cross_apb_forward(const void* a_q, const void* a_k, const void* s_q, const void* s_k,
                          const void* pair_bias, int bias_dtype, const uint8_t* mask, const void* blob,
                          const void* residual, void* out, void* workspace, size_t workspace_bytes, int W,
                          int Lq, int Lk, int C, int H, int Cs, int apply_norm, float eps, int io_dtype,
                          int arith, void* stream);

/* ---------------------------------------------------------------------------------------
 * Parcae recurrence step of the trunk: replaces the torch line
 *   z = a * z + F.linear(self.layernorm_z(u_t), b)             (model/model.py:528)
 * with a, b from `_parcae_discretized_dynamics` (model/model.py:272-277):
 *   delta = softplus(parcae_log_delta), a = exp(-delta * exp(parcae_log_a)),
 *   b = delta[:, None] * parcae_b_cont.
 * C = 128 or 256 (the shipping pair width).  One fused pass, no workspace.
 * ------------------------------------------------------------------------------------- */
size_t kfh_parcae_packed_bytes(int C);

/* ln_* [C] (`layernorm_z`); log_a, log_delta [C]; b_cont [C, C] ([out, in]).  The dynamics are
 * evaluated here, once per weight update, as the reference does once per `run_trunk` call. */
int kfh_parcae_pack(const void* ln_w, const void* ln_b, const void* log_a, const void* log_delta,
                    const void* b_cont, int w_dtype, int C, void* blob, void* stream);

/* out[r,:] = a * z[r,:] + b LN(u[r,:] + u_add[r,:]) for r < rows; z, u, u_add, out: [rows, C]
 * (io_dtype).  `u_add` may be NULL; with it the sum `u_t = z_inputs + lm_stack(...)` of
 * model/model.py:526 never goes through memory.  `out` may alias `z` (the in-place update of
 * the pair state); it must not alias `u` or `u_add`. */
int kfh_parcae_step(const void* z, const void* u, const void* u_add, const void* blob, void* out,
                    long long rows, int C, float eps, int io_dtype, void* stream);

/* ---------------------------------------------------------------------------------------
 * The pair track of one Pairformer block in one call (modules/apo_module.py:145-172, eval mode):
 *   z += TriMulOut(z, m); z += TriMulIn(z, m); z += TriAttStart(z, m); z += TriAttEnd(z, m);
 *   z  = (z + Transition(z)) * m
 * in place on z [B, N, N, C] with pair_mask [B, N, N] (bytes), the five blobs from kfh_trimul_pack
 * (outgoing, incoming), kfh_triattn_pack (starting, ending node) and kfh_transition_pack, and one
 * workspace of kfh_pair_block_workspace_bytes() bytes shared by the five ops (they run one after the
 * other on `stream`).  Same kernels and bits as the five calls made separately; supported shapes are
 * those all three ops support (C = 128 with 4 heads fused; other multiples of 32 up to 256 through
 * the assembled paths).
 * ------------------------------------------------------------------------------------- */
size_t kfh_pair_block_workspace_bytes(int B, int N, int C, int H, int expansion);
int kfh_pair_block_forward(void* z, const uint8_t* pair_mask, const void* trimul_out_blob,
                           const void* trimul_in_blob, const void* triattn_start_blob,
                           const void* triattn_end_blob, const void* transition_blob, void* workspace,
                           size_t workspace_bytes, int B, int N, int C, int H, int expansion, float eps,
                           int io_dtype, void* stream);

/* ---------------------------------------------------------------------------------------
 * The single track that follows the pair track (modules/confidence_head.py:161-175, eval mode):
 *   bias = linear_pair_bias(LN(z));  s += SelfAttentionPairBias(s, None, bias, mask);  s += Transition(s)
 * in place on s [B, N, Cs]; z [B, N, N, Cz] is only read; token_mask [B, N] (bytes).  Blobs from
 * kfh_pair_bias_pack, kfh_apb_pack (unconditioned, bf16 arithmetic) and kfh_transition_pack.  The
 * workspace also holds the bias tiles.  Same kernels and bits as the three calls made separately.
 * ------------------------------------------------------------------------------------- */
size_t kfh_single_track_workspace_bytes(int B, int N, int Cz, int Cs, int H, int expansion);
int kfh_single_track_forward(const void* z, void* s, const uint8_t* token_mask, const void* pair_bias_blob,
                             const void* apb_blob, const void* transition_blob, void* workspace,
                             size_t workspace_bytes, int B, int N, int Cz, int Cs, int H, int expansion,
                             float eps, int io_dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KFOLD_HIP_H */
