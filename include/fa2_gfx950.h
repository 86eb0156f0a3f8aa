/*
 * fa2_gfx950.h - C ABI of libfa2_gfx950.so: causal FlashAttention-2 forward and backward
 * as hand-written HIP kernels for AMD MI355X (gfx950, CDNA4).
 *
 * The library replaces the device side of egaoharu-kensei/flash-attention-triton.  Every entry
 * point cites the reference interface it stands in for (paths relative to the reference
 * repository root).  Conventions shared by all entry points:
 *
 *  - Tensors are (batch, nheads, seqlen, headdim) with element stride 1 on headdim; batch, head
 *    and sequence strides are passed in ELEMENTS (the reference kernels take the same three
 *    strides and assume stride 1 on headdim: src/flash_attention_triton/_triton_kernels_v2.py:88-105).
 *  - Causal masking keeps key column j for query row i when j <= i, anchored at the top-left
 *    corner also when seqlen_q != seqlen_k (_triton_kernels_v2.py:139-147).
 *  - The library never allocates, frees or retains device memory: the caller owns every buffer
 *    (as the reference's Python launchers do, flash_attention_2.py:93-100, 195-196, 365-367).
 *  - Calls only enqueue work on `stream` (a hipStream_t passed as void*; NULL = the null
 *    stream) and never synchronise.
 *  - Every function returns an fa2_status (0 = success).  Nothing throws or aborts; a textual
 *    description of the last failure on the calling thread is available from
 *    fa2_last_error_string().
 *  - lse and delta are fp32 arrays of shape (batch, nheads, seqlen_q_rounded) where
 *    seqlen_q_rounded >= seqlen_q is chosen by the caller (the reference pads the row length to
 *    a multiple of max_headdim, flash_attention_2.py:98-99).  Rows [seqlen_q, seqlen_q_rounded)
 *    are written with zeros.
 */
#ifndef FA2_GFX950_H
#define FA2_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FA2_ABI_VERSION 5

/* Largest head dimension the kernels accept (the table's `max_headdim`). */
#define FA2_MAX_HEADDIM 256

typedef enum fa2_status {
  FA2_OK = 0,
  FA2_ERR_NULL_POINTER = 1,     /* a required device pointer is NULL */
  FA2_ERR_BAD_SHAPE = 2,        /* non-positive size, or seqlen_q_rounded < seqlen_q */
  FA2_ERR_BAD_DTYPE = 3,        /* dtype is neither FA2_DTYPE_F16 nor FA2_DTYPE_BF16 */
  FA2_ERR_HEADDIM = 4,          /* headdim > FA2_MAX_HEADDIM */
  FA2_ERR_BAD_STRIDE = 5,       /* negative stride */
  FA2_ERR_BAD_CONFIG = 6,       /* config id outside the table, or not valid for this problem */
  FA2_ERR_WORKSPACE = 7,        /* a workspace is required but NULL */
  FA2_ERR_LAUNCH = 8,           /* hipLaunchKernel reported an error */
  FA2_ERR_TOO_LARGE = 9         /* a size or offset exceeds what the kernels index */
} fa2_status;

typedef enum fa2_dtype {
  FA2_DTYPE_F16 = 0, /* IEEE half: the reference's only compute type (flash_attention_2.py:90) */
  FA2_DTYPE_BF16 = 1 /* bfloat16 on bf16 MFMA; the reference down-casts bf16 to fp16 instead */
} fa2_dtype;

/* Rows (batch * nheads * seqlen_q_rounded) fa2_bwd_fused_noalloc has built-in scratch for: 16 MiB. */
#define FA2_NOALLOC_MAX_ROWS (4u << 20)

/* Ask the table to choose (pass as config_id). */
#define FA2_CONFIG_AUTO (-1)

/*
 * One row of the gfx950 tile/wave table.  Replaces the reference's per-architecture
 * KernelsConfigV2 constants and their selector (flash_attention_2.py:387-642).
 */
typedef struct fa2_config_info {
  int id;
  int headdim_padded; /* head dimension the kernels are instantiated for (>= headdim) */
  int fwd_block_q;    /* query rows per workgroup, forward */
  int fwd_block_kv;   /* key rows per inner step, forward */
  int fwd_waves;      /* wavefronts (64 lanes) per workgroup, forward */
  int bwd_block_q;    /* query rows per inner step, dK/dV kernel */
  int bwd_block_kv;   /* key rows per workgroup, dK/dV kernel */
  int bwd_waves;
  int dq_block_q;     /* query rows per workgroup, dQ kernel */
  int dq_block_kv;
  int dq_waves;
  int lds_direct;     /* the row's LDS-direct kernels (global_load_lds into swizzled tiles): 0 none, 1 forward and
                         backward, 2 forward and dQ only (one wave per SIMD, all 160 KiB of LDS; generic dK/dV) */
  int fwd_wg_per_cu;  /* workgroups that share a CU (what registers and LDS leave room for) */
  int dq_wg_per_cu;
  int dkdv_wg_per_cu;
  int lds_stages;     /* LDS stages of the streamed operand in the kernels of this row */
  int dkdv_passes;    /* passes of the dK/dV kernel over the query tiles (2: half the columns each) */
  int head_group;     /* (batch, head) pairs dispatched together; head_group / 8 share one XCD's L2 */
  int dq_atomic;      /* 1: sequence-parallel row - one backward kernel, dQ accumulated with fp32 global atomics
                         in a workspace (never picked by FA2_CONFIG_AUTO; selected by id) */
  int fwd_exp_folded; /* 1: forward-only row.  The LDS-direct forward multiplies its Q fragments by
                         softmax_scale * log2(e) and rounds them to the input type once, so that the score
                         MFMAs deliver the base-2 exponents themselves (one vector instruction less per
                         score; the reference scales the fp32 scores, _triton_kernels_v2.py:137-152).  O and
                         lse are those of inputs whose Q is perturbed by at most half a unit in the last
                         place.  Never picked by FA2_CONFIG_AUTO and refused by the backward entry points,
                         which recompute the probabilities from Q itself; see fa2_pick_config_forward_only */
} fa2_config_info;

/* One (batch, nheads, seqlen, headdim) tensor: device pointer and strides in elements. */
typedef struct fa2_tensor {
  const void *ptr;
  int64_t stride_batch, stride_head, stride_seq;
} fa2_tensor;

/*
 * Arguments of fa2_fwd as one record (same meaning, field for field).  A caller that launches
 * the same shapes repeatedly keeps the record and only swaps the pointers; a 27-argument call
 * through a foreign-function interface costs more host time than the kernel launch it makes.
 */
typedef struct fa2_fwd_args {
  fa2_tensor q, k, v, o; /* o is written */
  float *lse;
  int batch, nheads, seqlen_q, seqlen_k, headdim, seqlen_q_rounded;
  float softmax_scale;
  int dtype;
  int config_id;
} fa2_fwd_args;

/*
 * Arguments of the backward as one record.  o.ptr == NULL: `delta` is an input, as for fa2_bwd.
 * o.ptr != NULL: `delta` is an output formed on the way, as for fa2_bwd_fused.  dq, dk and dv are
 * written; dq.ptr == NULL or dk.ptr == dv.ptr == NULL skips that kernel (fa2_bwd's rule).
 */
typedef struct fa2_bwd_args {
  fa2_tensor q, k, v, o, d_o, dq, dk, dv;
  const float *lse;
  float *delta;
  void *workspace;
  int batch, nheads, seqlen_q, seqlen_k, headdim, seqlen_q_rounded;
  float softmax_scale;
  int dtype;
  int deterministic;
  int config_id;
} fa2_bwd_args;

/* ABI version of the loaded library; equals FA2_ABI_VERSION of the header it was built from. */
int fa2_abi_version(void);

/* Description of the most recent failure on the calling thread ("" if none). */
const char *fa2_last_error_string(void);

/* Static name of a status code. */
const char *fa2_status_string(int status);

/* Number of rows in the gfx950 table. */
int fa2_config_count(void);

/* Copy table row `config_id` to *out. */
int fa2_config_get(int config_id, fa2_config_info *out);

/*
 * Table lookup: replaces _select_optimal_gpu_architecture (flash_attention_2.py:617-642).
 * Returns the row id (>= 0) that FA2_CONFIG_AUTO stands for, or a negative fa2_status on error.
 * The row depends on the head dimension (the padded dimension the kernels are instantiated for).
 * dtype, seqlen_q, seqlen_k and deterministic are validated and do not change the row: every row
 * runs 128-row workgroups over 64-row streamed tiles in both types, and both backward modes run
 * the same atomic-free kernels.
 */
int fa2_pick_config(int dtype, int headdim, int seqlen_q, int seqlen_k, int deterministic);

/*
 * The row for a forward whose log-sum-exp no backward will read (inference, evaluation under
 * no_grad): for bf16 up to 128 columns the row with fwd_exp_folded = 1, whose extra rounding of Q
 * is of the size of the rounding bf16 inputs already carry; otherwise the row fa2_pick_config
 * returns.  No counterpart in the reference, whose forward is the same in both situations
 * (flash_attention_2.py:283-339).
 */
int fa2_pick_config_forward_only(int dtype, int headdim, int seqlen_q, int seqlen_k);

/*
 * Forward: O = softmax(scale * Q K^T + causal mask) V and the row log-sum-exp.
 * Replaces _flash_attention_forward + _forward_kernel
 * (flash_attention_2.py:61-144, _triton_kernels_v2.py:11-189).
 * q, o: (batch, nheads, seqlen_q, headdim); k, v: (batch, nheads, seqlen_k, headdim);
 * lse: fp32 (batch, nheads, seqlen_q_rounded), natural-log units.
 */
int fa2_fwd(const void *q, const void *k, const void *v, void *o, float *lse,
            int batch, int nheads, int seqlen_q, int seqlen_k, int headdim, int seqlen_q_rounded,
            int64_t q_stride_batch, int64_t q_stride_head, int64_t q_stride_seq,
            int64_t k_stride_batch, int64_t k_stride_head, int64_t k_stride_seq,
            int64_t v_stride_batch, int64_t v_stride_head, int64_t v_stride_seq,
            int64_t o_stride_batch, int64_t o_stride_head, int64_t o_stride_seq,
            float softmax_scale, int dtype, int config_id, void *stream);

/*
 * fa2_fwd with its arguments in one record.  Same reference interface as fa2_fwd
 * (flash_attention_2.py:61-144, _triton_kernels_v2.py:11-189).
 */
int fa2_fwd_packed(const fa2_fwd_args *args, void *stream);

/*
 * Backward preprocess: delta[b,h,i] = sum_d O[b,h,i,d] * dO[b,h,i,d] in fp32.
 * Replaces _backward_preprocess_do_o_dot (_triton_kernels_v2.py:532-608; launched at
 * flash_attention_2.py:218-234).
 */
int fa2_bwd_preprocess(const void *o, const void *d_o, float *delta,
                       int batch, int nheads, int seqlen_q, int headdim, int seqlen_q_rounded,
                       int64_t o_stride_batch, int64_t o_stride_head, int64_t o_stride_seq,
                       int64_t do_stride_batch, int64_t do_stride_head, int64_t do_stride_seq,
                       int dtype, void *stream);

/*
 * Bytes of workspace the backward needs.  Stands in for the reference's dq_accum allocation
 * (flash_attention_2.py:196).  0 for FA2_CONFIG_AUTO and every row it can pick (dQ is written
 * directly); for a sequence-parallel row (dq_atomic) the fp32 dQ accumulator:
 * batch * nheads * ceil(seqlen_q / 64) * 64 * headdim * 4 bytes, 16-byte aligned, which the
 * library clears itself on every call.
 */
size_t fa2_bwd_workspace_bytes(int batch, int nheads, int seqlen_q, int seqlen_k, int headdim,
                               int deterministic, int config_id);

/*
 * Backward main: fills dq, dk, dv (same dtype as q) in place.
 * Replaces _flash_attention_backward's main launch, the dQ zero-fill pre-hook and the final
 * dq.copy_(dq_accum) (flash_attention_2.py:235-277, _configurators_v2.py:81-93,
 * _triton_kernels_v2.py:192-529).
 * With FA2_CONFIG_AUTO both values of `deterministic` run the same two kernels: a key-tile-parallel
 * kernel for dK and dV and a query-tile-parallel kernel that accumulates dQ in registers in a fixed
 * order and writes it once.  There are no atomics, so results are bit-identical from run to run in
 * both modes (the reference's sequence-parallel mode, _triton_kernels_v2.py:336-339, allows
 * run-to-run differences but does not require them); fa2_bwd_workspace_bytes is 0 and `workspace`
 * may be NULL.
 * The reference's sequence-parallel formulation itself - one kernel per key tile that also adds its
 * dQ contributions into an fp32 accumulator with global atomics (_triton_kernels_v2.py:336-339,
 * 466-494), then dq = accumulator (flash_attention_2.py:277) - is the set of table rows with
 * dq_atomic = 1, selected by passing their id as config_id with deterministic = 0 and a workspace
 * of fa2_bwd_workspace_bytes() bytes.  It exists for head dimensions 32, 64 and 128 on 16-byte
 * aligned tensors (FA2_ERR_BAD_CONFIG otherwise), needs dq, dk and dv together, and its dq may
 * differ in the last bits from run to run.  The table never picks it: on MI355X the L2 retires
 * about 1.35 TB/s of fp32 atomic adds whatever their locality, so it is 2-3 times slower than the
 * two-kernel backward.
 * dK/dV and dQ are computed by two kernels launched back to back on `stream`.  A caller that
 * needs only part of the gradient (or wants to time one kernel) may pass dq == NULL to skip the
 * dQ kernel, or dk == dv == NULL to skip the dK/dV kernel; dk and dv are given or omitted
 * together, and at least one of the two groups must be present.
 */
int fa2_bwd(const void *q, const void *k, const void *v, const void *d_o,
            const float *lse, const float *delta, void *workspace,
            void *dq, void *dk, void *dv,
            int batch, int nheads, int seqlen_q, int seqlen_k, int headdim, int seqlen_q_rounded,
            int64_t q_stride_batch, int64_t q_stride_head, int64_t q_stride_seq,
            int64_t k_stride_batch, int64_t k_stride_head, int64_t k_stride_seq,
            int64_t v_stride_batch, int64_t v_stride_head, int64_t v_stride_seq,
            int64_t do_stride_batch, int64_t do_stride_head, int64_t do_stride_seq,
            int64_t dq_stride_batch, int64_t dq_stride_head, int64_t dq_stride_seq,
            int64_t dk_stride_batch, int64_t dk_stride_head, int64_t dk_stride_seq,
            int64_t dv_stride_batch, int64_t dv_stride_head, int64_t dv_stride_seq,
            float softmax_scale, int dtype, int deterministic, int config_id, void *stream);

/*
 * Whole backward in one call: replaces both launches of _flash_attention_backward
 * (flash_attention_2.py:218-277), i.e. fa2_bwd_preprocess followed by fa2_bwd, and gives the same
 * dq, dk, dv (delta may differ in its last bits: the row sums are taken in another order).
 * `delta` is an output here: fp32 (batch, nheads, seqlen_q_rounded) scratch supplied by the caller,
 * filled like fa2_bwd_preprocess fills it.  When the fast dQ kernel applies, that kernel forms
 * delta from the O and dO rows it already holds and the dK/dV kernel runs after it, which saves
 * one launch and one pass over O and dO; otherwise the three kernels run as in the two-call path.
 * dq, dk and dv must all be given.
 */
int fa2_bwd_fused(const void *q, const void *k, const void *v, const void *o, const void *d_o,
                  const float *lse, float *delta, void *workspace,
                  void *dq, void *dk, void *dv,
                  int batch, int nheads, int seqlen_q, int seqlen_k, int headdim, int seqlen_q_rounded,
                  int64_t q_stride_batch, int64_t q_stride_head, int64_t q_stride_seq,
                  int64_t k_stride_batch, int64_t k_stride_head, int64_t k_stride_seq,
                  int64_t v_stride_batch, int64_t v_stride_head, int64_t v_stride_seq,
                  int64_t o_stride_batch, int64_t o_stride_head, int64_t o_stride_seq,
                  int64_t do_stride_batch, int64_t do_stride_head, int64_t do_stride_seq,
                  int64_t dq_stride_batch, int64_t dq_stride_head, int64_t dq_stride_seq,
                  int64_t dk_stride_batch, int64_t dk_stride_head, int64_t dk_stride_seq,
                  int64_t dv_stride_batch, int64_t dv_stride_head, int64_t dv_stride_seq,
                  float softmax_scale, int dtype, int deterministic, int config_id, void *stream);

/*
 * fa2_bwd_fused for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc): same arguments without `delta` and
 * `workspace`, same dq, dk, dv bit for bit.  It has no counterpart in the reference, whose launcher
 * allocates delta itself (flash_attention_2.py:195).  The delta scratch lives in a device array
 * inside the library, FA2_NOALLOC_MAX_ROWS floats (16 MiB) on every GPU the library runs on, held
 * until the process ends; the call allocates and frees nothing and never synchronises.
 * batch * nheads * seqlen_q_rounded above FA2_NOALLOC_MAX_ROWS is refused with
 * FA2_ERR_TOO_LARGE.  All calls on one GPU share that array: two calls that may overlap there
 * (different streams, different threads) race on it - keep them on one stream or use
 * fa2_bwd_fused with separate buffers.  Nothing left in the array by an earlier call is read: each
 * call writes every row of delta before it reads it.  The first call on a device looks up the
 * array's address (hipGetSymbolAddress); make that call outside stream capture.
 */
int fa2_bwd_fused_noalloc(const void *q, const void *k, const void *v, const void *o, const void *d_o,
                          const float *lse, void *dq, void *dk, void *dv,
                          int batch, int nheads, int seqlen_q, int seqlen_k, int headdim, int seqlen_q_rounded,
                          int64_t q_stride_batch, int64_t q_stride_head, int64_t q_stride_seq,
                          int64_t k_stride_batch, int64_t k_stride_head, int64_t k_stride_seq,
                          int64_t v_stride_batch, int64_t v_stride_head, int64_t v_stride_seq,
                          int64_t o_stride_batch, int64_t o_stride_head, int64_t o_stride_seq,
                          int64_t do_stride_batch, int64_t do_stride_head, int64_t do_stride_seq,
                          int64_t dq_stride_batch, int64_t dq_stride_head, int64_t dq_stride_seq,
                          int64_t dk_stride_batch, int64_t dk_stride_head, int64_t dk_stride_seq,
                          int64_t dv_stride_batch, int64_t dv_stride_head, int64_t dv_stride_seq,
                          float softmax_scale, int dtype, int deterministic, int config_id, void *stream);

/*
 * The backward with its arguments in one record: fa2_bwd when args->o.ptr is NULL, fa2_bwd_fused
 * otherwise.  Same reference interface (flash_attention_2.py:147-277).
 */
int fa2_bwd_packed(const fa2_bwd_args *args, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* FA2_GFX950_H */
