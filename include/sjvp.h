/*
 * sjvp.h - C ABI of the MI355X (gfx950) fused attention-JVP kernels.
 *
 * The library is the drop-in for the three kernel-level entry points of olsdavis/semicat's
 * semicat/jvp_utils (paths below are relative to that repository):
 *
 *   sjvp_fwd   replaces flash_attention_jvp_multihead_triton_kernel_wrapper
 *              (semicat/jvp_utils/ryu_triton.py:295-422, kernel :73-291)
 *   sjvp_bwd   replaces, in ONE call, both
 *              flash_jvp_backward._flash_attn_backward   (cotangent on the tangent output,
 *              semicat/jvp_utils/flash_jvp_backward.py:2293-2714) and
 *              flash_attn_triton._flash_attn_backward    (cotangent on the primal output,
 *              semicat/jvp_utils/flash_attn_triton.py:974-1093)
 *
 * Conventions
 *   - Tensors are [B,H,L,D] views described by a base pointer and three element strides
 *     (batch, head, sequence); the last dimension has unit stride (the reference asserts the same,
 *     flash_jvp_backward.py:2321-2322).  q, tq, o, to, dO, dTO, dq, dtq have L = Lq; the k/v side has
 *     L = Lk.  Any [B,S,H,D] caller layout is expressed through the strides.
 *   - dtype: SJVP_BF16 or SJVP_FP16 for every tensor (MFMA kernels; accumulation and softmax are
 *     fp32), or SJVP_FP32: the correctness mode, fp32 tensors and fp32 arithmetic throughout on the
 *     vector ALUs (the reference's fp32 math path, ryu_triton.py:426-454; not tuned for speed), or
 *     SJVP_FP32_BF16: fp32 tensors whose elements are rounded to bf16 as they are loaded, bf16 MFMA
 *     arithmetic, results stored as fp32, i.e. the casts that functional.py:318-322,330-331 put
 *     around the op for fp32 callers, folded into it (sjvp_fwd, sjvp_bwd*; not sjvp_rope).  Strides
 *     are always in elements of the tensors' own storage type.
 *   - Row statistics lse / mu / li are fp32 [B,H,Lr] contiguous with Lr = ceil(Lq/128)*128
 *     (ryu_triton.py:351-358); rows >= Lq receive log(Lk), 0, Lk.
 *   - scale == 0 selects the default 1/sqrt(D) (ryu_triton.py:324-325); a negative or non-finite
 *     scale is an error.
 *   - The caller owns every buffer, including the workspace; the library allocates no device
 *     memory, keeps no pointer after returning, has no mutable global state (except the per-device
 *     address of sjvp_bwd_noalloc()'s static scratch and the mode of sjvp_set_row_sum_repair()), enqueues on the given hipStream_t (passed as
 *     void*) of the CURRENT device and returns without synchronising.
 *   - Every function returns SJVP_OK (0) or a negative error code; nothing aborts or throws.
 *     Argument errors are detected before anything is launched.
 *   - Results are deterministic: no atomics are used.
 */
#ifndef SJVP_H
#define SJVP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SJVP_VERSION 1

enum sjvp_dtype { SJVP_BF16 = 0, SJVP_FP16 = 1, SJVP_FP32 = 2, SJVP_FP32_BF16 = 3 };

enum sjvp_status {
    SJVP_OK = 0,
    SJVP_ERR_NULL = -1,      /* a required pointer is NULL                                   */
    SJVP_ERR_SHAPE = -2,     /* B, H, Lq or Lk < 1, or sizes beyond the 32-bit index range   */
    SJVP_ERR_HEAD_DIM = -3,  /* D < 16 (ryu_triton.py:319-322) or D > 128 (flash_jvp_backward.py:2318) */
    SJVP_ERR_DTYPE = -4,     /* dtype is not a member of sjvp_dtype                          */
    SJVP_ERR_WORKSPACE = -5, /* workspace NULL or smaller than sjvp_bwd_workspace_bytes()    */
    SJVP_ERR_LAUNCH = -6,    /* the HIP runtime refused a launch (status of hipLaunchKernel) */
    SJVP_ERR_COTANGENT = -7, /* sjvp_bwd called with both dO and dTO NULL                    */
    SJVP_ERR_PARTS = -8,     /* sjvp_bwd_parts: parts is not a combination of sjvp_bwd_part  */
    SJVP_ERR_ROTARY = -9,    /* sjvp_rope: n outside 1..4, rot_dim odd, < 0 or > D, or dtypes that mix bf16 and fp16;
                                sjvp_fwd_rotary / sjvp_bwd_rotary: a shape, dtype or table they do not serve */
    SJVP_ERR_SCALE = -10,    /* scale negative, infinite or NaN (0 selects the default)      */
    SJVP_ERR_SCRATCH = -11   /* sjvp_bwd_noalloc: problem beyond SJVP_NOALLOC_MAX_ROWS, or no static scratch on this device */
};

/* Indices into the stride tables: strides[3*i + {0,1,2}] = (batch, head, sequence) strides in
 * elements of tensor i. */
enum sjvp_fwd_tensor { SJVP_F_Q = 0, SJVP_F_K, SJVP_F_V, SJVP_F_TQ, SJVP_F_TK, SJVP_F_TV, SJVP_F_O,
                       SJVP_F_TO, SJVP_F_COUNT };
enum sjvp_bwd_tensor { SJVP_B_Q = 0, SJVP_B_K, SJVP_B_V, SJVP_B_TQ, SJVP_B_TK, SJVP_B_TV, SJVP_B_O,
                       SJVP_B_TO, SJVP_B_DO, SJVP_B_DTO, SJVP_B_DQ, SJVP_B_DK, SJVP_B_DV, SJVP_B_DTQ,
                       SJVP_B_DTK, SJVP_B_DTV, SJVP_B_COUNT };

/*
 * Fused forward: O = softmax(Q K^T scale) V and its forward-mode tangent
 *   TO = (P * (S_dot - mu)) V + P V_dot,   S_dot = scale (Q_dot K^T + Q K_dot^T),  mu = rowsum(P * S_dot)
 * in one online-softmax pass, plus lse (the reference's M), mu (MU) and, if li != NULL, the
 * exp-sum relative to the row maximum (LI).   Replaces ryu_triton.py:295-422.
 * Primal-only mode: tq = tk = tv = to = mu = NULL computes O and lse only.
 */
int sjvp_fwd(const void* q, const void* k, const void* v, const void* tq, const void* tk,
             const void* tv, void* o, void* to, float* lse, float* mu, float* li, int B, int H,
             int Lq, int Lk, int D, const int64_t* strides /* [SJVP_F_COUNT*3] */, float scale,
             int dtype, void* stream);

/*
 * Fused backward for cotangents dO (on O) and dTO (on TO); either may be NULL (treated as zero,
 * its contractions are skipped), not both.  Fills dq, dk, dv and, when dTO != NULL, dtq, dtk, dtv.
 * With dTO == NULL (the primal node of autograd, functional.py:261-268) tq, tk, tv, to, mu and the
 * three tangent gradients may be NULL.  o, to, lse, mu are the forward's outputs.
 * Replaces flash_jvp_backward.py:2293-2714 and flash_attn_triton.py:974-1093.
 */
int sjvp_bwd(const void* q, const void* k, const void* v, const void* tq, const void* tk,
             const void* tv, const void* o, const void* to, const void* dO, const void* dTO,
             const float* lse, const float* mu, void* dq, void* dk, void* dv, void* dtq, void* dtk,
             void* dtv, void* workspace, size_t workspace_bytes, int B, int H, int Lq, int Lk, int D,
             const int64_t* strides /* [SJVP_B_COUNT*3] */, float scale, int dtype, void* stream);

/*
 * sjvp_bwd() picks its launches by shape: for Lk <= 128 and D <= 64 (rows 16-byte aligned) one
 * launch produces all six gradients and leaves the workspace untouched; otherwise the backward is
 * a row-owned launch (dq, dtq, and the row sums it leaves in the workspace) followed by a
 * column-owned one (dk, dv, dtk, dtv), which consumes that workspace.
 * sjvp_bwd_parts() runs the selected launches of that pair with sjvp_bwd()'s arguments;
 * sjvp_bwd_parts(SJVP_BWD_ALL, ...) is sjvp_bwd().  It has no counterpart in the reference: it exists
 * so that a profiler or benchmark can time the two launches separately.  SJVP_BWD_COL alone is only
 * valid on a workspace that an earlier SJVP_BWD_ROW launch with the same arguments has filled.  (The second
 * pass of the row-owned kernel, see sjvp_set_row_sum_repair, belongs to SJVP_BWD_ROW; with SJVP_BWD_ALL its
 * workgroups are appended to the column-owned launch, since it depends on the first row-owned launch only.)
 */
enum sjvp_bwd_part { SJVP_BWD_ROW = 1, SJVP_BWD_COL = 2, SJVP_BWD_ALL = 3 };
int sjvp_bwd_parts(int parts, const void* q, const void* k, const void* v, const void* tq,
                   const void* tk, const void* tv, const void* o, const void* to, const void* dO,
                   const void* dTO, const float* lse, const float* mu, void* dq, void* dk, void* dv,
                   void* dtq, void* dtk, void* dtv, void* workspace, size_t workspace_bytes, int B,
                   int H, int Lq, int Lk, int D, const int64_t* strides /* [SJVP_B_COUNT*3] */,
                   float scale, int dtype, void* stream);

/*
 * sjvp_fwd() / sjvp_bwd() with the rotary position embedding of semicat/net/duo.py:45-55 folded in:
 * q, k (and tq, tk) are given UNROTATED; the kernels rotate them as they load them (position = row
 * index, column j < 32 paired with j + 32, the rotation of sjvp_rope() with rot_dim = D = 64), and the
 * backward returns the gradients with respect to the unrotated tensors (dq, dk, dtq, dtk pass through
 * the inverse rotation on their way out).  This removes the separate rotary launches and the rotated
 * copies of q, k in front of the op.  Served shapes: D = 64, Lk <= 128 (one workgroup walks a head's
 * keys once), SJVP_BF16 / SJVP_FP16 tensors with 16-byte aligned rows; cos, sin: fp32
 * [table_rows][32] with row stride cs_stride (multiple of 4), 16-byte aligned, table_rows >=
 * max(Lq, Lk).  Anything else returns SJVP_ERR_ROTARY before a launch (use sjvp_rope() + sjvp_fwd()).
 * sjvp_bwd_rotary() needs no workspace.  No counterpart in the reference, which rotates with separate
 * fp32 PyTorch operations.
 */
int sjvp_fwd_rotary(const void* q, const void* k, const void* v, const void* tq, const void* tk,
                    const void* tv, void* o, void* to, float* lse, float* mu, float* li, int B, int H,
                    int Lq, int Lk, int D, const int64_t* strides /* [SJVP_F_COUNT*3] */, float scale,
                    int dtype, const float* cos, const float* sin, int64_t cs_stride, int table_rows,
                    void* stream);
int sjvp_bwd_rotary(const void* q, const void* k, const void* v, const void* tq, const void* tk,
                    const void* tv, const void* o, const void* to, const void* dO, const void* dTO,
                    const float* lse, const float* mu, void* dq, void* dk, void* dv, void* dtq, void* dtk,
                    void* dtv, int B, int H, int Lq, int Lk, int D,
                    const int64_t* strides /* [SJVP_B_COUNT*3] */, float scale, int dtype, const float* cos,
                    const float* sin, int64_t cs_stride, int table_rows, void* stream);

/*
 * sjvp_bwd() with the workspace taken from a static device array inside the library instead of a
 * caller buffer.  It has no counterpart in the reference; it is for callers that cannot allocate
 * device memory around the call: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  The call allocates and frees nothing (neither does the rest of this library).
 *   - Limit: B * H * ceil(Lq/128)*128 <= SJVP_NOALLOC_MAX_ROWS (1 Mi statistic rows, 12.1 MiB of
 *     device memory that every GPU the library runs on holds until the process ends); larger
 *     problems return SJVP_ERR_SCRATCH and must use sjvp_bwd().
 *   - Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (two streams,
 *     two threads) race on it.  Calls on one stream are ordered and safe; nothing has to be cleared
 *     between calls (each launch pair writes every row it later reads).
 *   - The array's address is looked up on the first call on each device (no allocation); make that
 *     first call outside a graph capture.
 * Same results as sjvp_bwd(), bit for bit.
 */
#define SJVP_NOALLOC_MAX_ROWS (1 << 20)
int sjvp_bwd_noalloc(const void* q, const void* k, const void* v, const void* tq, const void* tk,
                     const void* tv, const void* o, const void* to, const void* dO, const void* dTO,
                     const float* lse, const float* mu, void* dq, void* dk, void* dv, void* dtq,
                     void* dtk, void* dtv, int B, int H, int Lq, int Lk, int D,
                     const int64_t* strides /* [SJVP_B_COUNT*3] */, float scale, int dtype, void* stream);

/*
 * Row sums of the backward.  The reference forms sum_4 and sum_7 (the row sums of the cotangent on the
 * tangent output) from the probabilities in a preprocess pass over the keys
 * (flash_jvp_backward.py:2012-2290) and delta from the 16-bit output (flash_attn_triton.py:526-617).
 * This library takes all of them from the 16-bit outputs o, to, which costs no pass, and the
 * row-owned launch then measures what the rounding of o, to left in them (the sums over the keys of
 * dS_dot and of dS, zero in exact arithmetic): it hands the column-owned launch the corrected sums
 * (= the reference's sums), and a second pass of the row-owned kernel (a launch of its own, or workgroups
 * appended to the column-owned launch) recomputes dq, dtq with them for the workgroups that ask for it.
 *   SJVP_REPAIR_OFF     no second pass (dk, dtk still get the corrected sums)
 *   SJVP_REPAIR_AUTO    (default) the second pass runs the workgroups in which a row's residue exceeds
 *                       the rounding of the tiles it is spread over (sharp attention rows, gradients
 *                       formed by cancellation); the others leave at once
 *   SJVP_REPAIR_ALWAYS  the first launch only measures, the second computes every row with the
 *                       corrected sums (the reference's preprocess + backward structure), and the row +
 *                       column pair is taken also for the shapes that would take the single launch,
 *                       whose row sums stay those of the 16-bit outputs (not with sjvp_bwd_rotary):
 *                       every gradient is formed as the reference forms it
 * Process-wide; returns the previous mode, or SJVP_ERR_PARTS for an unknown one.  Calls already
 * enqueued are not affected.
 */
enum sjvp_repair { SJVP_REPAIR_OFF = 0, SJVP_REPAIR_AUTO = 1, SJVP_REPAIR_ALWAYS = 2 };
int sjvp_set_row_sum_repair(int mode);

/* Bytes of caller-provided device scratch sjvp_bwd needs: lse in log2 units and the row sums sum_4
 * and sum_7 + delta (the reference allocates sum_4, sum_7 and delta itself,
 * flash_jvp_backward.py:2355-2356 and flash_attn_triton.py:990), 12 bytes per statistic row, and one
 * 4-byte flag per 64 rows (which row-owned workgroups take the second pass of the repair below). */
size_t sjvp_bwd_workspace_bytes(int B, int H, int Lq, int Lk, int D, int dtype);

/*
 * Rotary position embedding of n (1..4) tensors of one shape in one launch, with the cast to
 * out_dtype and any change of layout folded in.  For position l, i < rot_dim/2 and h = rot_dim/2:
 *   y[b,h,l,i]     = x[b,h,l,i]   cos[l,i] - sign x[b,h,l,i+h] sin[l,i]
 *   y[b,h,l,i+h]   = x[b,h,l,i+h] cos[l,i] + sign x[b,h,l,i]   sin[l,i]
 * with sign = +1, or -1 when `inverse` is non-zero; columns from rot_dim on are copied.  This is the
 * non-interleaved rotation that semicat/net/duo.py:45-55 applies to q and k before the attention op
 * through flash_attn.layers.rotary.apply_rotary_emb_torch (flash_attn 2.8.3, not vendored by the
 * reference), there as separate fp32 PyTorch operations.  The map is linear in x: the same call
 * rotates forward-mode tangents, and the inverse rotation back-propagates cotangents.
 *   x[i], y[i]   [B,H,L,D] views, unit last stride; strides[6*i + {0,1,2}] = (batch, head, sequence)
 *                element strides of x[i], strides[6*i + {3,4,5}] those of y[i]; y[i] may alias x[i]
 *                only if both have the same dtype and strides
 *   cos, sin     fp32 [L][rot_dim/2] with row stride cs_stride (elements); rot_dim = 0 makes the call a
 *                plain cast / layout change of up to four tensors in one launch (cos, sin may be NULL):
 *                the casts that functional.py:318-322,330-331 put around the op for float32 callers
 *   in_dtype, out_dtype   SJVP_BF16, SJVP_FP16 or SJVP_FP32 (not bf16 on one side and fp16 on the other)
 */
int sjvp_rope(int n, const void* const* x, void* const* y, const int64_t* strides /* [n*6] */,
              const float* cos, const float* sin, int64_t cs_stride, int B, int H, int L, int D,
              int rot_dim, int in_dtype, int out_dtype, int inverse, void* stream);

/* Static, NUL-terminated description of a status code. */
const char* sjvp_strerror(int status);

/* SJVP_VERSION the library was built with. */
int sjvp_version(void);

/* "SJVP_BUILD_ID=<hash>": identifies the sources this binary was built from, so that a host layer
 * can refuse a stale library.  No counterpart in the reference. */
const char* sjvp_build_id(void);

#ifdef __cplusplus
}
#endif
#endif /* SJVP_H */
