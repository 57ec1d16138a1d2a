/*
 * ltr_attn.h - C ABI of the MI355X (gfx950) ring / block attention library.
 *
 * The reference (lwj2015/lightron) is pure Python and has no FFI; each entry point
 * below names the reference code whose arithmetic it replaces.  A binder needs only
 * this header: plain pointers, sizes, no C++ or torch types.  All pointers are DEVICE
 * pointers unless noted.  Every call enqueues work on `stream` (a hipStream_t passed
 * as void*; NULL = the default stream) of the CURRENT device and returns without
 * synchronising.  The library never allocates, frees or keeps a pointer after the
 * call returns; all buffers, including fp32 gradient accumulators, belong to the
 * caller (one exception, stated there: ltr_attn_bwd_noalloc keeps its DELTA workspace in
 * a fixed array of its own).  Return value: 0 on success, a negative LTR_E* code otherwise
 * (nothing is enqueued on error).  Re-entrant and safe to call from several host threads:
 * the only mutable global state is a small per-device record of facts found out on the
 * first call on each device (architecture check, large-LDS opt-in, address of the fixed
 * scratch array), kept in atomics and read-only afterwards.
 *
 * Tensor layout: element strides (in elements, not bytes) are given for the batch,
 * sequence and head dimensions; the head dimension D is contiguous.  This serves
 * [B,S,H,D] (the layout at every reference boundary, ring_attention.py:13),
 * [B,H,S,D] (the layout at the SDPA call sites) and the Ulysses head-slice view
 * (parallel_cp.py:206-208) without copies.  LSE and DELTA are fp32 [B, Hq, Sq]
 * contiguous.
 *
 * Positions: query row i of the local chunk has global position
 *     i <  q_split : q_pos0[0] + i
 *     i >= q_split : q_pos0[1] + (i - q_split)
 * (q_split = Sq for one contiguous chunk; the two-segment form is the zig-zag
 * assignment).  Key row j of KV chunk c has global position chunk[c].pos0 + j.
 * With LTR_CAUSAL a key is visible iff key_pos <= query_pos.  Rows with no visible
 * key get O = 0 and LSE = -inf.
 */
#ifndef LTR_ATTN_H
#define LTR_ATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LTR_ABI_VERSION 8
#define LTR_MAX_CHUNKS 32

/* element types */
#define LTR_BF16 0
#define LTR_F32 1

/* flags */
#define LTR_CAUSAL 1u /* mask by global position */
#define LTR_MERGE 2u  /* forward: o/lse hold an earlier partial result; merge into it */
#define LTR_NO_DQ 4u    /* backward: skip the dQ kernel (dq may be NULL) */
#define LTR_NO_DKDV 8u  /* backward: skip the dK/dV kernel (chunk[].dk/dv may be NULL) */
#define LTR_DQ_BF16 16u /* backward: dq is a bf16 tensor that RECEIVES dQ of this call (no accumulation) */
#define LTR_DELTA_FROM_O 32u /* backward: delta is computed from o by the dQ kernel (and written to delta) */
#define LTR_DKDV_BF16 64u /* backward: chunk[c].dk / dv are bf16 tensors that RECEIVE dK / dV of this call (no accumulation) */
#define LTR_ROPE_Q 128u   /* forward: q is un-rotated; RoPE is applied to it in the kernel's prologue (rope_freqs) */
#define LTR_ROPE_DQ 256u  /* backward: dQ leaves the dQ kernel rotated by the conjugate angles (gradient of LTR_ROPE_Q) */
#define LTR_DKDV_KEYS_128 512u  /* backward, tuning hint: the dK/dV kernel's blocks own 128 keys (the default choice is the library's) */
#define LTR_DKDV_KEYS_256 1024u /* backward, tuning hint: they own 256 keys (bf16, head dim 64 only: LTR_EUNSUP otherwise); results
                                   do not depend on the hint beyond the order of fp32 additions inside a block */
#define LTR_DQ_ROWS_256 2048u /* backward, tuning hint: the dQ kernel's blocks own 256 query rows (the default choice is the library's) */
#define LTR_DQ_ROWS_512 4096u /* backward, tuning hint: they own 512 rows (bf16, head dim 64 only: LTR_EUNSUP otherwise); same results */
#define LTR_FWD_ROWS_256 8192u  /* forward, tuning hint: the kernel's blocks own 256 query rows (the default choice is the library's) */
#define LTR_FWD_ROWS_512 16384u /* forward, tuning hint: they own 512 rows (bf16, head dim 64 only: LTR_EUNSUP otherwise); results differ
                                   only through the tile size (64 instead of 128 keys: the order of fp32 additions) */

#define LTR_FWD_F32_SCALAR 32768u /* forward, fp32 only: run the scalar fp32 kernel instead of the matrix-pipe one (same results to
                                    rounding; the fallback and cross-check of fwd_f32_mfma_kernel) */
#define LTR_BWD_F32_SCALAR 65536u /* backward, fp32 only: the scalar fp32 kernels instead of the matrix-pipe ones (fallback and
                                    cross-check) */

/* error codes */
#define LTR_OK 0
#define LTR_EINVAL (-1)   /* null pointer, bad size, bad flag */
#define LTR_EUNSUP (-2)   /* unsupported head dim / dtype combination */
#define LTR_EALIGN (-3)   /* pointer or stride not 16-byte aligned */
#define LTR_ELAUNCH (-4)  /* HIP reported a launch error */
#define LTR_EDEVICE (-5)  /* current device is not gfx950 */
#define LTR_ETOOBIG (-6)  /* ltr_attn_bwd_noalloc: more rows than the fixed scratch holds */

typedef struct ltr_kv_chunk {
    const void *k; /* [B, sk, Hkv, D] by kv strides */
    const void *v;
    void *dk;      /* fp32 accumulators (bf16 results with LTR_DKDV_BF16), same logical shape, by dk/dv strides (backward only) */
    void *dv;
    int64_t sk;    /* keys in this chunk */
    int64_t pos0;  /* global position of its first key */
} ltr_kv_chunk;

/*
 * ltr_attn_fwd - one rank's local Q chunk attended against n_chunks KV chunks resident
 * in HBM, online softmax across chunks kept in registers, O normalised and LSE written
 * once.  Replaces the whole `for step in range(world_size)` body of
 * ring_attention_kernel (parallel/communication/ring_attention.py:46-118: score GEMM
 * :71, online-softmax update :79-95/:107, PV GEMM and rescale :101-104, normalise :118)
 * and the SDPA calls at parallel/parallel_cp.py:224-229 and model/model.py:193-198.
 * GQA: q head h reads kv head h / (Hq/Hkv)  (model/model.py:11-34, repeat_kv).
 * With LTR_MERGE the epilogue combines the new partial (O', LSE') with the (O, LSE)
 * already in the output buffers by the same rule
 *     LSE = logaddexp(LSE, LSE'),  O = O*exp(LSE_old-LSE) + O'*exp(LSE'-LSE)
 * so a caller that receives KV chunks one at a time (one launch per ring step, as at
 * ring_attention.py:46) needs no separate merge pass.
 */
typedef struct ltr_attn_fwd_args {
    const void *q;      /* [B, Sq, Hq, D] by q strides; dtype io_dtype */
    void *o;            /* same logical shape by o strides; dtype o_dtype */
    float *lse;         /* [B, Hq, Sq] */
    int32_t B, Hq, Hkv, D; /* D in {64, 128} */
    int64_t Sq;
    int64_t q_stride[3];  /* batch, seq, head */
    int64_t o_stride[3];
    int64_t k_stride[3];
    int64_t v_stride[3];
    int64_t q_pos0[2];
    int64_t q_split;
    float scale;          /* 1/sqrt(D) at every reference call site (ring_attention.py:20) */
    uint32_t flags;       /* LTR_CAUSAL | LTR_MERGE | LTR_ROPE_Q | LTR_FWD_ROWS_256 | LTR_FWD_ROWS_512 | LTR_FWD_F32_SCALAR */
    int32_t io_dtype;     /* LTR_BF16 or LTR_F32, of q/k/v */
    int32_t o_dtype;      /* LTR_BF16 or LTR_F32 */
    int32_t n_chunks;     /* 1..LTR_MAX_CHUNKS */
    ltr_kv_chunk chunk[LTR_MAX_CHUNKS];
    /* LTR_ROPE_Q (bf16 only), the fused prologue of apply_rotary_emb (layers/layers.py:44-70, applied to q at
     * parallel/parallel_cp.py:219 and model/model.py:183): every q row is rotated, in the registers that hold it as the
     * MFMA operand, by the angles of its GLOBAL position; no separate pass over q.  rope_freqs: the table of
     * precompute_freqs_cis as interleaved fp32 (cos, sin), [rope_len][D/2][2], row 0 = position rope_pos0; it must
     * cover every position of the local rows.  The rotated row has the bits ltr_rope_apply would have written.
     * q_rot (optional, bf16, own strides): receives the rotated q, which is what ltr_attn_bwd takes as q.
     * K is NOT rotated here: a K row is read by every q block that sees it, so its rotation belongs before the
     * attention (one ltr_rope_apply per K tensor), not inside it. */
    const float *rope_freqs;
    int64_t rope_pos0;
    int64_t rope_len;
    void *q_rot;
    int64_t q_rot_stride[3];
} ltr_attn_fwd_args;

int ltr_attn_fwd(const ltr_attn_fwd_args *args, void *stream);

/*
 * ltr_attn_bwd_delta - DELTA[b,h,i] = sum_d dO[b,i,h,d] * O[b,i,h,d], the row term of
 * the softmax Jacobian.  The reference has no hand-written backward (autograd through
 * ring_attention.py:66-118 / SDPA); this is the first stage of the recompute backward.
 */
typedef struct ltr_attn_delta_args {
    const void *o;
    const void *d_o;
    float *delta;       /* [B, Hq, Sq] */
    int32_t B, Hq, D;
    int64_t Sq;
    int64_t o_stride[3];
    int64_t do_stride[3];
    int32_t o_dtype;    /* dtype of o */
    int32_t do_dtype;   /* dtype of dO */
} ltr_attn_delta_args;

int ltr_attn_bwd_delta(const ltr_attn_delta_args *args, void *stream);

/*
 * ltr_attn_bwd - recompute backward of ltr_attn_fwd for the same Q chunk / KV chunk
 * table: P = exp(S*scale - LSE), dV += P^T dO, dP = dO V^T, dS = P*(dP - DELTA),
 * dQ += dS K * scale, dK += dS^T Q * scale.  Replaces torch autograd through the ring
 * body / SDPA (trainer.py:54 -> parallel_cp.py:224-229).  dq, chunk[c].dk and
 * chunk[c].dv are fp32 ACCUMULATORS: the caller zero-fills them before the first
 * launch that contributes, launches on one stream accumulate (that is how dK/dV sum
 * over the Q chunks of several ranks), and ltr_cast_f32_to_bf16 makes the final cast.
 * dK/dV of a GQA group sum over its Hq/Hkv query heads.  Two kernels are enqueued, one
 * for dK/dV and one for dQ (no atomics: results are bitwise reproducible); LTR_NO_DQ /
 * LTR_NO_DKDV enqueue only one of them, e.g. for a ring step where dK/dV travel with the
 * KV chunk, or to time the kernels separately.  LTR_DQ_BF16: when the chunk table of this
 * call holds every KV chunk the queries can see, dQ is complete after the call, and dq
 * may then be the bf16 result itself (written, not accumulated; dq_stride in bf16
 * elements): no fp32 accumulator, no zero-fill, no final cast.  LTR_DELTA_FROM_O: delta is
 * an OUTPUT workspace; the dQ kernel computes DELTA = rowsum(dO * O) of its rows from o
 * (bf16, o_stride) and stores it, and the dK/dV kernel, enqueued after it, reads it: no
 * separate ltr_attn_bwd_delta launch.  Not combinable with LTR_NO_DQ.  LTR_DKDV_BF16: when q holds
 * every query row that sees the keys of this call's chunks (one rank's own backward, not a ring step whose dK/dV
 * go on to other ranks), dK / dV of those chunks are complete after the call: chunk[c].dk / dv may then be the
 * bf16 results themselves (written for every key, zeros where no query sees it; dk/dv strides in bf16 elements):
 * no fp32 accumulators, no zero-fill, no final cast.  bf16 only.
 */
typedef struct ltr_attn_bwd_args {
    const void *q;
    const void *d_o;      /* same dtype as q */
    const float *lse;     /* [B, Hq, Sq], of the COMPLETE softmax (all chunks) */
    float *delta;         /* [B, Hq, Sq] fp32: input, or workspace written with LTR_DELTA_FROM_O */
    void *dq;             /* fp32 accumulator by dq strides, or the bf16 result with LTR_DQ_BF16 */
    int32_t B, Hq, Hkv, D;
    int64_t Sq;
    int64_t q_stride[3];
    int64_t do_stride[3];
    int64_t dq_stride[3];
    int64_t k_stride[3];
    int64_t v_stride[3];
    int64_t dk_stride[3];
    int64_t dv_stride[3];
    int64_t q_pos0[2];
    int64_t q_split;
    float scale;
    uint32_t flags;       /* LTR_CAUSAL | LTR_NO_DQ | LTR_NO_DKDV | LTR_DQ_BF16 | LTR_DELTA_FROM_O | LTR_DKDV_BF16 | LTR_ROPE_DQ |
                             LTR_DKDV_KEYS_128 | LTR_DKDV_KEYS_256 | LTR_DQ_ROWS_256 | LTR_DQ_ROWS_512 | LTR_BWD_F32_SCALAR */
    int32_t io_dtype;     /* LTR_BF16 or LTR_F32, of q/k/v/dO (LTR_F32: fp32 kernels on v_mfma_f32_32x32x2_f32 for the 1e-4 cases;
                             LTR_DQ_BF16, LTR_DELTA_FROM_O and LTR_DKDV_BF16 are bf16 only and return LTR_EUNSUP with it) */
    int32_t n_chunks;
    ltr_kv_chunk chunk[LTR_MAX_CHUNKS];
    const void *o;        /* forward output, bf16, only read with LTR_DELTA_FROM_O */
    int64_t o_stride[3];
    /* LTR_ROPE_DQ (bf16 only): q is the ROTATED q (q_rot of a forward with LTR_ROPE_Q); the dQ kernel's epilogue rotates
     * dQ by the conjugate angles of each row's global position before it is stored or accumulated, so dq is the
     * gradient of the un-rotated q (torch autograd through the complex multiply at layers/layers.py:67-70).  Table as
     * in ltr_attn_fwd_args.  dK is the gradient of the K that was passed in (rotated beforehand: its gradient goes
     * through ltr_rope_apply with LTR_ROPE_CONJ). */
    const float *rope_freqs;
    int64_t rope_pos0;
    int64_t rope_len;
} ltr_attn_bwd_args;

int ltr_attn_bwd(const ltr_attn_bwd_args *args, void *stream);

/*
 * ltr_attn_bwd_noalloc - ltr_attn_bwd for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  Same arguments and results as ltr_attn_bwd with
 * LTR_DELTA_FROM_O (which it implies: bf16 only, args->o required, LTR_NO_DQ refused), except
 * that args->delta is IGNORED (may be NULL): the DELTA workspace is a fixed array of
 * LTR_NOALLOC_MAX_ROWS floats (4 MiB) in device memory that belongs to the library; each
 * GPU the library runs on holds its own copy until the process ends.  B * Hq * Sq must not
 * exceed LTR_NOALLOC_MAX_ROWS (LTR_ETOOBIG otherwise).  The call allocates and frees
 * nothing and calls no allocating routine.  All calls on one GPU share that GPU's array:
 * two calls whose kernels may overlap on one GPU (different streams, different threads)
 * race on it; calls on one stream are safe.  Every DELTA row a call's dK/dV kernel reads
 * is written by its dQ kernel first, so nothing has to be cleared between calls.
 */
#define LTR_NOALLOC_MAX_ROWS (1 << 20)

int ltr_attn_bwd_noalloc(const ltr_attn_bwd_args *args, void *stream);

/* dst[i] = bf16(src[i]) (round to nearest even), i < n; both contiguous. */
int ltr_cast_f32_to_bf16(const float *src, void *dst, int64_t n, void *stream);

/*
 * ltr_rope_apply - rotary position embedding of one tensor, the arithmetic of
 * apply_rotary_emb (layers/layers.py:44-70): x viewed as complex numbers over ADJACENT
 * pairs (x[2i], x[2i+1]), converted to fp32, multiplied by freqs[s][i] = (cos, sin) of
 * angle s * theta_i, converted back to the input dtype.  The reference applies it to q
 * and k before attention (model/model.py:183, parallel/parallel_cp.py:219); one call
 * per tensor here.  freqs is the table of precompute_freqs_cis (layers/layers.py:18-24)
 * as interleaved fp32 (re, im) pairs, [S][D/2][2] contiguous, row s for sequence index s
 * of x (the caller slices the table for a chunk that starts at a global position).
 * LTR_ROPE_CONJ multiplies by the conjugate instead: that is the gradient of the
 * rotation (torch autograd through the complex multiply in the reference).
 * x and out may be the same buffer.  Element strides as in ltr_attn_fwd_args.
 */
#define LTR_ROPE_CONJ 1u

typedef struct ltr_rope_args {
    const void *x;        /* [B, S, H, D] by strides, D contiguous */
    void *out;            /* same shape, own strides */
    const float *freqs;   /* [S, D/2, 2] fp32 (cos, sin) */
    int32_t B, H, D;      /* D a multiple of 8 */
    int64_t S;
    int64_t x_stride[3], out_stride[3];   /* elements, for B, S, H */
    uint32_t flags;       /* LTR_ROPE_CONJ */
    int32_t io_dtype;     /* LTR_BF16 or LTR_F32, x and out */
} ltr_rope_args;

int ltr_rope_apply(const ltr_rope_args *args, void *stream);

/*
 * ltr_attn_plan - which kernels, with which block sizes, ltr_attn_fwd and ltr_attn_bwd would launch for this problem
 * on the CURRENT device (host call: nothing is enqueued and no pointer in args is read; without a device the answer is
 * for 256 compute units).  It has no counterpart in the reference (which leaves the choice of kernel to the library
 * behind F.scaled_dot_product_attention, model/model.py:193); it is for benchmarks and profiles that must name the kernel
 * they measured, and for tests of the size hints.  The sizes, strides' owner shapes, positions, chunk lengths, dtype and
 * flags of args are read; flags may also carry the forward's hints (LTR_FWD_ROWS_256 / LTR_FWD_ROWS_512 / LTR_FWD_F32_SCALAR).  The library's
 * launches and this answer come from one function, so they cannot drift apart.  Kernel names are those a profiler shows.
 */
typedef struct ltr_attn_plan_t {
    int32_t compute_units;   /* CUs the choices were made for */
    int32_t fwd_rows;        /* query rows per block of the forward kernel */
    int32_t fwd_paired;      /* 1: a block takes a late q tile and its early counterpart (causal balance) */
    int32_t dq_rows;         /* query rows per block of the dQ kernel */
    int32_t dq_paired;
    int32_t dkdv_keys;       /* keys per block of the dK/dV kernel */
    int64_t fwd_blocks, dq_blocks, dkdv_blocks;
    char fwd_kernel[48], dq_kernel[48], dkdv_kernel[48];
} ltr_attn_plan_t;

int ltr_attn_plan(const ltr_attn_bwd_args *args, ltr_attn_plan_t *out);

int ltr_abi_version(void);
const char *ltr_strerror(int code);

#ifdef __cplusplus
}
#endif
#endif /* LTR_ATTN_H */
