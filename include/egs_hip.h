/*
 * egs_hip.h -- C ABI of the MI355X (gfx950) fused expert gather / scatter-with-linear library.
 *
 * The reference reaches its device code through four Python callables bound in module
 * globals (reference egs/triton_kernels.py:26-29, bound at :569-578) which launch three
 * Triton kernels (:49-143 gather, :156-247 scatter, :261-356 dW).  This header is what a
 * binding of that surface sees instead: plain device pointers, sizes and enums.
 *
 * Conventions for every entry point
 *   - returns EGS_OK (0) or a negative egs_status; never throws, never synchronises;
 *   - thread-safe and re-entrant: the library keeps no mutable state except once-per-device
 *     set-up flags (and the built-in buffer of egs_dw_builtin_scratch, see there); it launches on
 *     the calling thread's current device;
 *   - all tensor pointers are device pointers, borrowed until the enqueued work completes;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*, NULL = default stream);
 *   - arguments are validated before any HIP call, so bad arguments are reported even on a
 *     host without a GPU;
 *   - no device memory is allocated: scratch is a caller-provided workspace whose size comes
 *     from egs_workspace_bytes();
 *   - tensors are dense row-major ([B,T,I] sources may carry explicit batch/token strides,
 *     inner stride 1);  Ind is [B,E,K] of int16/int32/int64/uint8 and is never written;
 *   - Ind is read through aligned 8-byte windows: the 8-byte aligned words that contain its first
 *     and its last element must lie inside the allocation.  Any buffer that starts at an address
 *     hipMalloc (or an allocator that rounds to 8 bytes or more, such as torch's) returned, or at
 *     an element offset into one, satisfies this;
 *   - a pick whose index is outside [0,T) contributes nothing (gather writes a zero row,
 *     scatter and dW skip it); egs_validate_indices() reports such picks.
 */
#ifndef EGS_HIP_H
#define EGS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EGS_ABI_VERSION 1

typedef enum egs_status {
    EGS_OK = 0,
    EGS_ERR_NULL_POINTER = -1,
    EGS_ERR_BAD_SHAPE = -2,
    EGS_ERR_BAD_DTYPE = -3,     /* counterpart of ValueError("Unknown dtype"), reference egs/triton_kernels.py:23 */
    EGS_ERR_BAD_LAYOUT = -4,
    EGS_ERR_BAD_MODE = -5,
    EGS_ERR_WORKSPACE = -6,     /* workspace missing, or smaller than the kernels selected for these operands need */
    EGS_ERR_ALIGNMENT = -7,
    EGS_ERR_HIP = -8,           /* a HIP runtime call failed; see egs_last_hip_error() */
    EGS_ERR_UNSUPPORTED = -9,
    EGS_ERR_BAD_STRIDE = -10,
    EGS_ERR_SCRATCH_LIMIT = -11 /* egs_dw_builtin_scratch: the sizes need more than EGS_BUILTIN_SCRATCH_BYTES */
} egs_status;

/* element types; 0..2 are the reference's dtype ids (egs/triton_kernels.py:15-23) */
typedef enum egs_dtype {
    EGS_F32 = 0,
    EGS_F16 = 1,
    EGS_BF16 = 2,
    EGS_FP8_E4M3 = 3            /* OCP e4m3fn, weights of the gather only */
} egs_dtype;

typedef enum egs_index_dtype {
    EGS_IND_I16 = 0,
    EGS_IND_I32 = 1,
    EGS_IND_I64 = 2,
    EGS_IND_U8 = 3
} egs_index_dtype;

/* how the weight (or weight gradient) is stored.  The reference passes swapped strides
 * instead (egs/triton_kernels.py:468, :504, :521). */
typedef enum egs_w_layout {
    EGS_W_EIJ = 0,              /* [E, I, J]  gather-side weight  */
    EGS_W_EJI = 1               /* [E, J, I]  scatter-side weight */
} egs_w_layout;

typedef enum egs_scatter_mode {
    EGS_SCATTER_DETERMINISTIC = 0,  /* fixed summation order, bitwise reproducible, no atomics   */
    EGS_SCATTER_ATOMIC = 1,         /* fp32 atomic accumulation, order of additions unspecified  */
    EGS_SCATTER_COMPACT = 2         /* DETERMINISTIC without a workspace: where the sizes allow (16-bit types, reduction
                                     * 32 / 64 / 128, output columns a multiple of 32, T <= 1024, more than 1024 picks per
                                     * batch element) the product rows stay on the compute unit, the picks are sorted there
                                     * too, and egs_workspace_bytes returns 0 - the reference's kernel
                                     * (egs/triton_kernels.py:156-247) has no intermediate either, and its README
                                     * (README.md:36) sells the path on memory; DETERMINISTIC spends B*E*K*I*4 bytes of
                                     * workspace on fp32 product rows and is faster at large shapes with even routing;
                                     * same tolerances, its own (fixed) order of additions */
} egs_scatter_mode;

typedef enum egs_op {
    EGS_OP_GATHER_GEMM = 0,
    EGS_OP_GEMM_SCATTER = 1,
    EGS_OP_DW = 2,
    EGS_OP_GATHER_BACKWARD = 3,     /* GEMM_SCATTER + DW sharing one workspace */
    EGS_OP_SCATTER_BACKWARD = 4     /* GATHER_GEMM + DW */
} egs_op;

/* problem sizes shared by every entry point:
 *   B batches, T tokens per batch, E experts, K picks per (batch, expert),
 *   I = width of the [B,T,I] side, J = width of the [B,E,K,J] side. */
typedef struct egs_dims {
    int32_t B, T, E, K, I, J;
} egs_dims;

int egs_abi_version(void);
const char *egs_status_string(int status);
/* text of the last HIP error seen by the calling thread ("" if none) */
const char *egs_last_hip_error(void);

/* bytes of scratch the op needs for these sizes (0 is a valid answer: small experts run on
 * kernels that keep every intermediate on the CU).  `mode` is an egs_scatter_mode and only matters for ops
 * that scatter.  The answer holds for dense operands that start on a 16-byte boundary (what hipMalloc and
 * torch return); every entry point derives the requirement again from the operands it is given, and an
 * operand off that grid can select a general kernel that needs more: the call then returns
 * EGS_ERR_WORKSPACE and launches nothing; copy such operands to aligned storage first. */
size_t egs_workspace_bytes(int op, int mode, const egs_dims *d, int act_dtype);

/* ---------------------------------------------------------------------------------------
 * Kernel-level entry points (one per reference kernel)
 * ------------------------------------------------------------------------------------- */

/* Y[b,e,k,j] = sum_i X[b, Ind[b,e,k], i] * W(e,i,j)
 * Replaces expert_gather_kernel (reference egs/triton_kernels.py:49-143).
 *   X    [B,T,I] act_dtype, strides (ldx_b, ldx_t, 1) in elements
 *   W    [E,I,J] (EGS_W_EIJ: gather forward) or [E,J,I] (EGS_W_EJI: dY of the scatter), w_dtype
 *   w_scale  NULL, or for w_dtype == EGS_FP8_E4M3 a float [E,J] per-output-column scale
 *   Y    [B,E,K,J] act_dtype, dense */
int egs_gather_gemm(const void *X, const void *W, const void *Ind, void *Y, const float *w_scale,
                    const egs_dims *d, int64_t ldx_b, int64_t ldx_t,
                    int act_dtype, int w_dtype, int ind_dtype, int w_layout, void *stream);

/* Out[b,t,i] = sum_{e,k : Ind[b,e,k]=t} sum_j Y[b,e,k,j] * W(e,i,j); rows nobody picks are 0.
 * Replaces expert_scatter_kernel (reference egs/triton_kernels.py:156-247).
 *   Y    [B,E,K,J] act_dtype, dense
 *   W    [E,J,I] (EGS_W_EJI: scatter forward) or [E,I,J] (EGS_W_EIJ: dX of the gather), act_dtype
 *   Out  [B,T,I] act_dtype, dense; fully overwritten */
int egs_gemm_scatter(const void *Y, const void *W, const void *Ind, void *Out,
                     void *workspace, size_t workspace_bytes, const egs_dims *d,
                     int act_dtype, int ind_dtype, int w_layout, int mode, void *stream);

/* dW(e,i,j) = sum_{b,k} Xsrc[b, Ind[b,e,k], i] * Ysrc[b,e,k,j], fp32 accumulation in a fixed
 * order (split over the batch, then a second fixed-order pass).
 * Replaces expert_gather_scatter_dW_kernel (reference egs/triton_kernels.py:261-356).
 *   Xsrc [B,T,I] strides (ldx_b, ldx_t, 1);  Ysrc [B,E,K,J] dense;  both act_dtype
 *   dW   [E,I,J] (EGS_W_EIJ) or [E,J,I] (EGS_W_EJI) in out_dtype; fully overwritten */
int egs_dw(const void *Xsrc, const void *Ysrc, const void *Ind, void *dW,
           void *workspace, size_t workspace_bytes, const egs_dims *d,
           int64_t ldx_b, int64_t ldx_t,
           int act_dtype, int out_dtype, int ind_dtype, int dw_layout, void *stream);

/* egs_dw for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  No counterpart in the reference, whose launchers allocate
 * with torch on every call (egs/triton_kernels.py:408-409, :491-492).
 * Same arguments, kernels and results (bit for bit) as egs_dw, minus the workspace: the fp32 partial
 * sums of the split reduction live in a buffer of EGS_BUILTIN_SCRATCH_BYTES that is part of the
 * library's device image (every GPU the library runs on holds one until the process ends).  The call
 * allocates and frees nothing; the buffer's device address is looked up the first time the entry point
 * runs on a device, so make that first call outside graph capture.
 * Sizes whose partial sums (egs_workspace_bytes(EGS_OP_DW, ...)) exceed the buffer are rejected with
 * EGS_ERR_SCRATCH_LIMIT before anything is enqueued.
 * All calls on one GPU share that GPU's buffer: calls that may overlap in time (different streams,
 * different threads) race on it; serialise them, or use egs_dw with workspaces of their own. */
#define EGS_BUILTIN_SCRATCH_BYTES (16u << 20)
int egs_dw_builtin_scratch(const void *Xsrc, const void *Ysrc, const void *Ind, void *dW, const egs_dims *d,
                           int64_t ldx_b, int64_t ldx_t,
                           int act_dtype, int out_dtype, int ind_dtype, int dw_layout, void *stream);

/* Inference variant of the gather with fp8 weights AND fp8 activations, on the fp8 matrix instruction:
 *   Y[b,e,k,j] = xs[b,t] * w_scale[e,j] * sum_i Xq[b,t,i] * Wq(e,i,j),   t = Ind[b,e,k],
 * where every source row X[b,t,:] is first quantised to e4m3 (round to nearest even) with its own scale
 * xs[b,t] = max|X[b,t,:]| / 448 (1 for an all-zero row).  Both steps run on `stream`; the quantised rows and
 * their scales live in the workspace (egs_gather_gemm_fp8act_workspace_bytes(), 256-byte aligned).
 * No counterpart in the reference, whose expert_gather_kernel (egs/triton_kernels.py:49-143) takes
 * fp32/fp16/bf16 only (:15-23); a different numerical contract from egs_gather_gemm with fp8 weights, which
 * keeps the activations in bf16.
 *   X    [B,T,I] bf16, strides (ldx_b, ldx_t, 1) in elements, multiples of 8;  I % 128 == 0
 *   Wq   [E,I,J] e4m3fn;  w_scale float [E,J];  J % 16 == 0
 *   Y    [B,E,K,J] bf16, dense
 * Shapes outside these limits return EGS_ERR_UNSUPPORTED. */
size_t egs_gather_gemm_fp8act_workspace_bytes(const egs_dims *d);
int egs_gather_gemm_fp8act(const void *X, const void *Wq, const float *w_scale, const void *Ind, void *Y,
                           void *workspace, size_t workspace_bytes, const egs_dims *d,
                           int64_t ldx_b, int64_t ldx_t, int ind_dtype, void *stream);

/* ---------------------------------------------------------------------------------------
 * Routing table in caller-owned memory (new; the reference has nothing of the kind: its scatter kernel adds with
 * atomics, egs/triton_kernels.py:247).  The one-kernel scatter of small experts sorts the picks of a batch element by
 * token before it can add product rows in a fixed order; Ind decides that order alone, so it can be computed once per
 * Ind and reused by every scatter over the same Ind: the scatter forward, and the scatter inside the gather's backward.
 *   - egs_routing_table_bytes(): size of the table for these sizes, 0 if no kernel would read one (then pass no table).
 *   - egs_expert_gather_forward_table(): egs_expert_gather_forward, and fills `table` from Ind in the same launch
 *     (a launch of its own when the operands do not select the small-expert gather).
 *   - egs_expert_scatter_forward_table(), egs_expert_gather_backward_table(): the plain entry points with a table that
 *     was filled from the SAME Ind contents and the same sizes; results are bit-identical to the plain entry points.
 *     The table is only read.  A table built from other indices gives wrong sums without any error: the caller owns
 *     that invariant.  (Its entries are clamped to the ranges a table of these sizes can hold, so even memory that was
 *     never filled cannot make a kernel run on or touch anything but its own rows.)
 * `table` NULL makes each of these the plain entry point.  A table argument for sizes that have no use for one returns
 * EGS_ERR_UNSUPPORTED; `table` must be 256-byte aligned (EGS_ERR_ALIGNMENT) and at least egs_routing_table_bytes() long
 * (EGS_ERR_WORKSPACE).
 * ------------------------------------------------------------------------------------- */
size_t egs_routing_table_bytes(const egs_dims *d, int dtype);

int egs_expert_gather_forward_table(const void *X, const void *W, const void *Ind, void *Y,
                                    void *table, size_t table_bytes,
                                    const egs_dims *d, int64_t ldx_b, int64_t ldx_t,
                                    int dtype, int ind_dtype, void *stream);

int egs_expert_scatter_forward_table(const void *Y, const void *W, const void *Ind,
                                     const void *table, size_t table_bytes, void *Out,
                                     void *workspace, size_t workspace_bytes, const egs_dims *d,
                                     int dtype, int ind_dtype, int mode, void *stream);

int egs_expert_gather_backward_table(const void *X, const void *W, const void *Ind,
                                     const void *table, size_t table_bytes,
                                     const void *grad_Y, void *grad_X, void *grad_W,
                                     void *workspace, size_t workspace_bytes, const egs_dims *d,
                                     int64_t ldx_b, int64_t ldx_t,
                                     int dtype, int ind_dtype, int mode, void *stream);

/* Which capture, if any, `stream` is recording into a HIP graph right now: *id = 0 when it is not capturing, else the
 * runtime's identifier of that capture (unique per capture in the process).  For bindings that keep a routing table next to
 * Ind: a table filled by a captured launch holds nothing until the graph is replayed, so it may only serve launches
 * of the same capture.  No counterpart in the reference.  Returns EGS_ERR_NULL_POINTER / EGS_ERR_HIP. */
int egs_stream_capture_id(void *stream, unsigned long long *id);

/* ---------------------------------------------------------------------------------------
 * Inference block (new; no single kernel of the reference corresponds to it): the reference's call pattern
 *   out = scatter(act(gather(x, Ind)), Ind, T)          (test_speed.ipynb:73-75)
 * in ONE kernel for small experts; the rows Y[B,E,K,J] between the two products stay in registers:
 *   Out[b,t,:] = sum over picks (e,k) of t, in pick order, of  act(X[b,Ind[b,e,k],:] . Wg[e]) . Ws[e]
 * Wg is [E,I,J], Ws is [E,J,I], Out [B,T,I] is written completely (tokens nobody picked become zero); the
 * activation is applied to the fp32 product and the result rounded to the element type, as a stored Y would
 * be.  Bitwise reproducible, no workspace.  Taken for 16-bit types, I in {32, 64, 128}, J in {32, 64} and at most 1024
 * picks per batch element (egs_expert_mlp_supported); anything else returns EGS_ERR_UNSUPPORTED and the caller composes
 * egs_expert_gather_forward, its own activation and egs_expert_scatter_forward.
 * ------------------------------------------------------------------------------------- */
typedef enum egs_activation {
    EGS_ACT_NONE = 0,
    EGS_ACT_RELU = 1,
    EGS_ACT_GELU = 2,           /* erf form (torch.nn.functional.gelu default) */
    EGS_ACT_SILU = 3,
    EGS_ACT_GELU_TANH = 4       /* tanh approximation */
} egs_activation;

/* 1 if egs_expert_mlp_forward takes these sizes (with dense operands that start on a 16-byte boundary), else 0 */
int egs_expert_mlp_supported(const egs_dims *d, int dtype);

int egs_expert_mlp_forward(const void *X, const void *Wg, const void *Ws, const void *Ind, void *Out,
                           const egs_dims *d, int64_t ldx_b, int64_t ldx_t,
                           int dtype, int ind_dtype, int activation, void *stream);

/* ---------------------------------------------------------------------------------------
 * Launcher-level entry points (one per reference callable)
 * ------------------------------------------------------------------------------------- */

/* expert_gather_forward_call(X, W[E,I,J], Ind) -> Y          reference egs/triton_kernels.py:367-392 */
int egs_expert_gather_forward(const void *X, const void *W, const void *Ind, void *Y,
                              const egs_dims *d, int64_t ldx_b, int64_t ldx_t,
                              int dtype, int ind_dtype, void *stream);

/* expert_gather_backward_call(X, W[E,I,J], Ind, grad_Y) -> (grad_X, grad_W)   reference :400-441 */
int egs_expert_gather_backward(const void *X, const void *W, const void *Ind, const void *grad_Y,
                               void *grad_X, void *grad_W,
                               void *workspace, size_t workspace_bytes, const egs_dims *d,
                               int64_t ldx_b, int64_t ldx_t,
                               int dtype, int ind_dtype, int mode, void *stream);

/* expert_scatter_forward_call(Y, W[E,J,I], Ind, T) -> Out     reference :449-474 */
int egs_expert_scatter_forward(const void *Y, const void *W, const void *Ind, void *Out,
                               void *workspace, size_t workspace_bytes, const egs_dims *d,
                               int dtype, int ind_dtype, int mode, void *stream);

/* expert_scatter_backward_call(Y, W[E,J,I], Ind, grad_Out) -> (grad_Y, grad_W)   reference :483-525 */
int egs_expert_scatter_backward(const void *Y, const void *W, const void *Ind, const void *grad_Out,
                                void *grad_Y, void *grad_W,
                                void *workspace, size_t workspace_bytes, const egs_dims *d,
                                int64_t ldg_b, int64_t ldg_t,
                                int dtype, int ind_dtype, void *stream);

/* ---------------------------------------------------------------------------------------
 * Debug helper (no counterpart in the reference, which never checks Ind)
 * ------------------------------------------------------------------------------------- */

/* adds to *d_bad_count (device int32, caller-zeroed) the number of entries outside [0,T) */
int egs_validate_indices(const void *Ind, int ind_dtype, int64_t n, int32_t T,
                         int32_t *d_bad_count, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* EGS_HIP_H */
