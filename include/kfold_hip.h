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
 *     KFH_BF16 (0) or KFH_F32 (1).  Arithmetic is always bf16 MFMA with fp32
 *     accumulation and fp32 LayerNorm / softmax statistics;
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

#define KFH_OK 0
#define KFH_EINVAL (-1)      /* bad argument (shape, dtype, null pointer, small workspace) */
#define KFH_EUNSUPPORTED (-2) /* valid request the kernels are not built for (e.g. C != 128) */
#define KFH_EHIP (-3)         /* a HIP runtime call failed; message holds hipGetErrorString */

#define KFH_OUTGOING 0
#define KFH_INCOMING 1

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

/* Workspace for one call with N tokens (per batch element; batches are processed in turn). */
size_t kfh_trimul_workspace_bytes(int N, int C);

/* out[b,i,j,:] = (residual ? residual[b,i,j,:] : 0) + TriangleMultiplication(z, mask)[b,i,j,:]
 * z, out, residual: [B, N, N, C] contiguous, io_dtype.  mask: [B, N, N] bytes.
 * `residual` may be NULL and may alias `out`; `out` may alias `z` only if residual == z
 * (the in-place `z += update` of modules/apo_module.py:153-160). */
int kfh_trimul_forward(const void* z, const uint8_t* mask, const void* blob, const void* residual,
                       void* out, void* workspace, size_t workspace_bytes, int B, int N, int C,
                       int direction, float eps, int io_dtype, void* stream);

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

#ifdef __cplusplus
}
#endif
#endif /* KFOLD_HIP_H */
