/*
 * canon_conv1d.h -- C ABI of the MI355X (gfx950) Canon causal depthwise conv1d.
 *
 * Two operators, the two calls Viby's CanonLayer makes into an accelerated
 * backend (reference = JohanLi233/Viby-Model), plus the backward of the first:
 *
 *   canon_conv1d_fwd     replaces  causal_conv1d_fn      (prefill)
 *   canon_conv1d_update  replaces  causal_conv1d_update  (one decode token)
 *   canon_conv1d_bwd     gradient of canon_conv1d_fwd    (training)
 *   canon_conv1d_update_bwd  gradient of canon_conv1d_update
 *
 * Plain pointers, sizes and element strides only; no framework types.  Every
 * pointer is a DEVICE pointer owned by the caller.  Kernels are enqueued on
 * the given HIP stream and the call returns without synchronising.  Nothing
 * here allocates device memory.
 *
 * Status codes are returned as int; canon_conv1d_last_error() gives the
 * message of the last failing call made by the calling thread.
 */
#ifndef CANON_CONV1D_H
#define CANON_CONV1D_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CANON_CONV1D_ABI_VERSION 9
#define CANON_CONV1D_MIN_WIDTH 2
#define CANON_CONV1D_MAX_WIDTH 4

/* storage type of x / out / states, and (independently) of weight / bias */
enum { CANON_DTYPE_F32 = 0, CANON_DTYPE_BF16 = 1, CANON_DTYPE_F16 = 2 };

/* element type of a padding mask (any value is multiplied in, 0/1 is usual) */
enum {
    CANON_MASK_U8 = 0,  /* also bool */
    CANON_MASK_I32 = 1,
    CANON_MASK_I64 = 2,
    CANON_MASK_F32 = 3,
    CANON_MASK_BF16 = 4,
    CANON_MASK_F16 = 5
};

enum { CANON_ACT_NONE = 0, CANON_ACT_SILU = 1 };

/* residual term added to the activated conv output */
enum {
    CANON_RESIDUAL_NONE = 0,
    CANON_RESIDUAL_MASKED = 1,   /* out += x * mask  (eager CanonLayer, model/model.py:595,675) */
    CANON_RESIDUAL_UNMASKED = 2  /* out += x         (fused branches,  model/model.py:491)     */
};

/*
 * CANON_ROUND_FUSED: fp32 accumulate, SiLU and residual in fp32, one rounding
 *                    to the storage type at the store.
 * CANON_ROUND_EAGER: additionally rounds to the storage type after the conv,
 *                    after SiLU and after the residual add -- the rounding
 *                    points of the reference's eager module, so 16-bit
 *                    results equal it bit for bit.  The update call in this
 *                    mode follows model/model.py:385-396 (each product
 *                    rounded, then the sum, then bias, then SiLU).
 */
enum { CANON_ROUND_FUSED = 0, CANON_ROUND_EAGER = 1 };

enum {
    CANON_OK = 0,
    CANON_ERR_INVALID_ARGUMENT = 1,  /* caller error: shapes, strides, null pointers */
    CANON_ERR_UNSUPPORTED = 2,       /* valid upstream feature this build does not implement */
    CANON_ERR_LAUNCH = 3             /* HIP reported an error at launch */
};

/*
 * Prefill.  Replaces causal_conv1d_fn(x, weight, bias, seq_idx, initial_states,
 * return_final_states, final_states_out, activation) as called at
 * model/model.py:460-466, and fuses what CanonLayer does around that call:
 * the padding-mask multiply (model/model.py:454-457), the residual add (:491)
 * and the conv-state capture (:470-489).
 *
 *   xm[b,c,t]  = mask ? round(x[b,c,t] * mask[b,t]) : x[b,c,t]
 *   y[b,c,t]   = act(bias[c] + sum_{k<W} weight[c,k] * xm[b,c,t-(W-1)+k])
 *   out        = y (+ xm | + x)
 * with xm == 0 for t < 0, or the last W-1 entries of initial_state when given
 * (with seq_idx: also 0 for every position of another packed sequence).
 * final_state (optional) receives the last final_len entries of
 * initial_state ++ xm, zero filled on the left.
 *
 * x / out are logical [batch, channels, seqlen] with element strides; both
 * the time-contiguous ([B,C,L]) and the channel-contiguous ([B,L,C] viewed
 * as [B,C,L], which is what model/model.py:459 passes) layouts have a
 * vectorised kernel, anything else takes a strided scalar kernel.
 * out must not alias x.
 */
typedef struct canon_conv1d_fwd_params {
    uint32_t struct_size;           /* sizeof(canon_conv1d_fwd_params) */
    int32_t x_dtype;                /* CANON_DTYPE_*: x, out, initial_state, final_state */
    int32_t w_dtype;                /* CANON_DTYPE_*: weight and bias (rounded to x_dtype on load) */
    int32_t mask_dtype;             /* CANON_MASK_*, ignored when mask == NULL.  Every (batch, channel) row re-reads its
                                       batch row of the mask through the caches: a mask no wider than x's elements
                                       costs 10-20 % at large sizes and an int64 mask 25-35 % in the time-contiguous
                                       layout (channel-contiguous: under 5 % and under 10 %) */
    int32_t width;                  /* W, 2..4 */
    int32_t activation;             /* CANON_ACT_* */
    int32_t residual_mode;          /* CANON_RESIDUAL_* */
    int32_t round_mode;             /* CANON_ROUND_* */
    int64_t batch, channels, seqlen;
    const void *x;
    int64_t x_stride_b, x_stride_c, x_stride_l;          /* in elements */
    void *out;
    int64_t out_stride_b, out_stride_c, out_stride_l;
    const void *weight;             /* [channels, width] */
    int64_t w_stride_c, w_stride_k;
    const void *bias;               /* [channels] contiguous, or NULL */
    const void *mask;               /* [batch, seqlen], or NULL */
    int64_t mask_stride_b, mask_stride_l;
    const void *initial_state;      /* [batch, channels, initial_len], or NULL */
    int64_t init_stride_b, init_stride_c, init_stride_s;
    int32_t initial_len;            /* >= W-1 when initial_state != NULL */
    int32_t final_len;              /* >= 1 when final_state != NULL */
    void *final_state;              /* [batch, channels, final_len], or NULL */
    int64_t final_stride_b, final_stride_c, final_stride_s;
    const int32_t *seq_idx;         /* [batch, seqlen] or NULL: the `seq_idx` argument of causal_conv1d_fn
                                       (model/model.py:465 passes None).  Positions of one batch row that
                                       carry different values belong to different packed sequences: an input
                                       contributes only to outputs with its own value.  Excludes
                                       initial_state / final_state. */
    int64_t seq_stride_b, seq_stride_l;
} canon_conv1d_fwd_params;

/*
 * Decode update.  Replaces causal_conv1d_update(x, conv_state, weight, bias,
 * activation) as called at model/model.py:305-311 (eager restatement:
 * model/model.py:372-398).
 *
 *   xt[b,c]  = token_mask ? round(x[b,c] * token_mask[b]) : x[b,c]     (model/model.py:277-282)
 *   y[b,c]   = act(bias[c] + sum_{k<W-1} weight[c,k] * state[b,c,S-(W-1)+k] + weight[c,W-1] * xt[b,c])
 *   out      = y (+ xt | + x)
 *   state   <- state shifted left by one, xt appended      (in place, pure copies)
 *
 * state_len S >= W-1.  A contiguous [B,C,S] state with S in {3,4,8} and
 * channel-contiguous x/out takes the vectorised kernel.
 */
typedef struct canon_conv1d_update_params {
    uint32_t struct_size;           /* sizeof(canon_conv1d_update_params) */
    int32_t x_dtype, w_dtype, mask_dtype;
    int32_t width;
    int32_t activation;
    int32_t residual_mode;
    int32_t round_mode;
    int32_t state_len;
    int32_t state_rows;             /* with conv_state_indices: rows of the conv_state pool, or 0 (not stated) */
    int64_t batch, channels;
    const void *x;
    int64_t x_stride_b, x_stride_c;
    void *out;
    int64_t out_stride_b, out_stride_c;
    void *conv_state;               /* [batch, channels, state_len], updated in place */
    int64_t state_stride_b, state_stride_c, state_stride_s;
    const void *weight;
    int64_t w_stride_c, w_stride_k;
    const void *bias;
    const void *token_mask;         /* [batch], or NULL */
    int64_t mask_stride_b;
    const int32_t *cache_seqlens;        /* [batch] or NULL.  Upstream's circular-buffer mode: conv_state is not
                                            shifted; the token is written to slot cache_seqlens[b] % state_len and
                                            the W-1 slots before it (cyclically) are the history.  Strided kernel. */
    const int32_t *conv_state_indices;   /* [batch] or NULL.  Upstream's batch indirection: batch entry b uses row
                                            conv_state_indices[b] of conv_state (a state pool of state_rows rows; the
                                            caller guarantees that the indices are distinct).  An entry whose index is
                                            negative, or not below state_rows when that is stated, is skipped: neither
                                            its state row nor its row of out is read or written (upstream's padding
                                            slots). */
} canon_conv1d_update_params;

/*
 * Backward of canon_conv1d_fwd: the gradient a
 * training step needs so that the fused forward can stay on the accelerated
 * path (trainer/base_trainer.py:274 calls backward through every Canon
 * layer).  Same role as the reference's own backward kernels
 * (causal_conv1d_mps/autograd.py:116-151 and :305-338,
 * causal_conv1d.metal:803-958, 1354-1735), which return dx, dweight, dbias.
 *
 * With z = bias + conv(xm), xm = x * mask, out = act(z) (+ xm | + x):
 *   dz[t]  = dout[t] * act'(z[t])                         (z is recomputed from x)
 *   dxm[t] = sum_k weight[k] * dz[t + (W-1) - k]  (+ dout[t] for RESIDUAL_MASKED)
 *   dx[t]  = dxm[t] * mask[t]                     (+ dout[t] for RESIDUAL_UNMASKED)
 *   dweight[c,k] = sum_{b,t} dz[b,c,t] * xm[b,c,t-(W-1)+k],   dbias[c] = sum_{b,t} dz[b,c,t]
 * With seq_idx, the terms that pair an output step with a tap step of another
 * sequence index (the ones the forward left out) are left out of z, dxm and
 * dweight alike.
 * All arithmetic in fp32; dx is rounded once to the storage type.  dweight and
 * dbias are fp32, OVERWRITTEN (not accumulated into), and reduced in a fixed
 * order in two stages through `workspace` (no float atomics: results are
 * reproducible run to run).
 */
typedef struct canon_conv1d_bwd_params {
    uint32_t struct_size;           /* sizeof(canon_conv1d_bwd_params) */
    int32_t x_dtype;                /* x, dout, dx */
    int32_t w_dtype;                /* weight and bias as used by the forward */
    int32_t mask_dtype;
    int32_t width;
    int32_t activation;
    int32_t residual_mode;
    int32_t reserved0;
    int64_t batch, channels, seqlen;
    const void *x;
    int64_t x_stride_b, x_stride_c, x_stride_l;
    const void *dout;
    int64_t dout_stride_b, dout_stride_c, dout_stride_l;
    void *dx;                       /* must not alias x or dout */
    int64_t dx_stride_b, dx_stride_c, dx_stride_l;
    const void *weight;
    int64_t w_stride_c, w_stride_k;
    const void *bias;               /* or NULL */
    const void *mask;               /* or NULL */
    int64_t mask_stride_b, mask_stride_l;
    float *dweight;                 /* [channels, width] contiguous fp32 */
    float *dbias;                   /* [channels] fp32, or NULL */
    void *workspace;                /* canon_conv1d_bwd_workspace_bytes() bytes, 16-byte aligned */
    int64_t workspace_bytes;
    const int32_t *seq_idx;         /* [batch, seqlen] or NULL: the forward's packed-sequence indices */
    int64_t seq_stride_b, seq_stride_l;
    const void *initial_state;      /* [batch, channels, initial_len] or NULL: the forward's initial_state (the chunked
                                       continuation of model/model.py:647-659 as one differentiable call); its last
                                       W-1 entries enter z as the inputs before t = 0 and dweight with them.  Not with
                                       seq_idx.  Channel-contiguous tensors keep their vector kernel with it;
                                       time-contiguous ones take the strided kernel. */
    int64_t init_stride_b, init_stride_c, init_stride_s;
    int32_t initial_len;            /* >= W-1 when initial_state != NULL */
    int32_t reserved1;
    void *dinitial_state;           /* [batch, channels, initial_len] in x_dtype, or NULL: receives the gradient w.r.t.
                                       initial_state (zero for entries older than W-1); needs initial_state */
    int64_t dinit_stride_b, dinit_stride_c, dinit_stride_s;
    const void *dfinal_state;       /* [batch, channels, final_len] in x_dtype, or NULL: the gradient that arrives through
                                       the forward's final_state (the last final_len entries of initial_state ++ xm):
                                       added to dxm of the last steps and, where the state reaches back before t = 0,
                                       to dinitial_state.  Kernel choice as for initial_state. */
    int64_t dfinal_stride_b, dfinal_stride_c, dfinal_stride_s;
    int32_t final_len;              /* >= 1 when dfinal_state != NULL */
    int32_t reserved2;
} canon_conv1d_bwd_params;

/*
 * Backward of canon_conv1d_update.  Same role as the
 * reference's short_conv_update_bwd (causal_conv1d_mps/autograd.py:465-498,
 * causal_conv1d.metal:1738-1850): dx, dconv_state, dweight, dbias from the
 * token, the state AS IT WAS BEFORE the forward call (the caller keeps a
 * copy, as causal_conv1d_mps/autograd.py:452 does: the forward overwrites
 * it) and dout.  Unlike the reference it also takes the gradient that
 * arrives through the UPDATED state, so that a chain of decode steps can be
 * differentiated end to end.
 *
 * With xt = x * token_mask, z = bias + sum_{k<W-1} weight[k] * state[S-(W-1)+k] + weight[W-1] * xt,
 * out = act(z) (+ xt | + x), state' = state[1:] ++ xt:
 *   dz        = dout * act'(z)
 *   dxt       = weight[W-1] * dz (+ dout for RESIDUAL_MASKED) + dstate_out[S-1]
 *   dx        = dxt * token_mask (+ dout for RESIDUAL_UNMASKED)
 *   dstate[j] = dstate_out[j-1]  (0 for j = 0)  + weight[j-(S-(W-1))] * dz  for j >= S-(W-1)
 *   dweight[c,k] = sum_b dz[b,c] * (k < W-1 ? state[b,c,S-(W-1)+k] : xt[b,c]),   dbias[c] = sum_b dz[b,c]
 * All arithmetic in fp32, dx and dstate rounded once to the storage type;
 * dweight / dbias fp32, overwritten, summed over the batch in a fixed order in
 * two stages through `workspace` (no float atomics).
 */
typedef struct canon_conv1d_update_bwd_params {
    uint32_t struct_size;           /* sizeof(canon_conv1d_update_bwd_params) */
    int32_t x_dtype;                /* x, conv_state, dout, dstate_out, dx, dstate */
    int32_t w_dtype;                /* weight and bias as used by the forward */
    int32_t mask_dtype;
    int32_t width;
    int32_t activation;
    int32_t residual_mode;
    int32_t state_len;
    int64_t batch, channels;
    const void *x;                  /* [batch, channels]: the token of the forward call */
    int64_t x_stride_b, x_stride_c;
    const void *conv_state;         /* [batch, channels, state_len]: the state BEFORE the forward call */
    int64_t state_stride_b, state_stride_c, state_stride_s;
    const void *weight;
    int64_t w_stride_c, w_stride_k;
    const void *bias;               /* or NULL */
    const void *token_mask;         /* [batch], or NULL */
    int64_t mask_stride_b;
    const void *dout;               /* [batch, channels] */
    int64_t dout_stride_b, dout_stride_c;
    const void *dstate_out;         /* [batch, channels, state_len]: gradient w.r.t. the updated state, or NULL (zero) */
    int64_t dstate_out_stride_b, dstate_out_stride_c, dstate_out_stride_s;
    void *dx;                       /* [batch, channels] */
    int64_t dx_stride_b, dx_stride_c;
    void *dstate;                   /* [batch, channels, state_len]: gradient w.r.t. the state before, or NULL (not wanted);
                                       must not alias dstate_out */
    int64_t dstate_stride_b, dstate_stride_c, dstate_stride_s;
    float *dweight;                 /* [channels, width] contiguous fp32, or NULL (no parameter gradients) */
    float *dbias;                   /* [channels] fp32, or NULL; needs dweight */
    void *workspace;                /* canon_conv1d_update_bwd_workspace_bytes() bytes, 16-byte aligned (unused when dweight == NULL) */
    int64_t workspace_bytes;
    /* The decode modes of canon_conv1d_update other than the shift register (both NULL: shift register).
     * cache_seqlens: the forward wrote the token to slot p = cache_seqlens[b] mod state_len and read the width-1
     *   slots before it cyclically (the reference's update kernel, causal_conv1d.metal:755-775, and its backward,
     *   :1738-1850); the formulas above hold with entry j of the state before the step in slot (p + j) mod state_len
     *   and entry j of the updated state in slot (p + 1 + j) mod state_len.
     * conv_state_indices: batch entry b used row conv_state_indices[b] of conv_state, so conv_state, dstate_out and
     *   dstate have state_rows rows.  An entry whose index lies outside the pool was skipped by the forward: its dx
     *   row is zero and it contributes nothing.  Only the rows that entries name are written: fill dstate with
     *   dstate_out (or zeros) before the call, so that rows no entry used pass their gradient on unchanged.  Two
     *   entries naming one row are as undefined here as in the forward. */
    const int32_t *cache_seqlens;        /* [batch] int32, or NULL */
    const int32_t *conv_state_indices;   /* [batch] int32, or NULL */
    int64_t state_rows;                  /* rows of the pool; 0: not stated (indices are only checked for a negative value) */
} canon_conv1d_update_bwd_params;

/*
 * One channel range of a logical [batch, channels, seqlen] input that lives in
 * a tensor of its own.  Canon-B convolves cat(q, k, v) and Canon-D
 * cat(gate, up) along the channels (model/model.py:772-789, 962-971): with
 * parts, the projections are read where they are and the results written to
 * separate tensors, so neither the cat nor a split copy is made.  Part i covers
 * channels [sum of channels of parts < i, + channels) of weight, bias and the
 * states.  For the decode update only the _b and _c strides are read.
 */
#define CANON_CONV1D_MAX_PARTS 4
typedef struct canon_conv1d_part {
    const void *x;
    int64_t x_stride_b, x_stride_c, x_stride_l;
    void *out;
    int64_t out_stride_b, out_stride_c, out_stride_l;
    int64_t channels;
} canon_conv1d_part;

int canon_conv1d_abi_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char *canon_conv1d_last_error(void);

/*
 * Optional set-up of the CURRENT device, once per GPU and process: loads the library's code objects onto it and
 * looks up the address of that GPU's copy of the static scratch buffer (see canon_conv1d_bwd_static), which is
 * where the runtime does its one-time allocations.  Without it the first launch of each kernel family on a device
 * does the same work by itself.  Call it (or make one warm-up call of every entry point you use) BEFORE capturing
 * launches into a HIP graph and before a section of the program that must not allocate.  Has no counterpart in
 * the reference (its Metal library is built and cached on first use, causal_conv1d_mps.mm:35-104).
 */
int canon_conv1d_init(void);

/* Enqueue on `stream` (a hipStream_t; NULL = the default stream). */
int canon_conv1d_fwd(const canon_conv1d_fwd_params *p, void *stream);
int canon_conv1d_update(const canon_conv1d_update_params *p, void *stream);
int canon_conv1d_bwd(const canon_conv1d_bwd_params *p, void *stream);
int canon_conv1d_update_bwd(const canon_conv1d_update_bwd_params *p, void *stream);

/*
 * The same operators with x / out given as 1..CANON_CONV1D_MAX_PARTS channel
 * ranges (p->x, p->out and their strides are ignored; p->channels must equal
 * the sum over the parts; weight, bias, mask and the states are those of the
 * whole problem).  Channel-contiguous parts of width 4 run as ONE launch;
 * other layouts are launched part by part.  Results equal the single-tensor
 * call on the concatenated input bit for bit.
 */
int canon_conv1d_fwd_parts(const canon_conv1d_fwd_params *p, const canon_conv1d_part *parts, int32_t nparts, void *stream);
int canon_conv1d_update_parts(const canon_conv1d_update_params *p, const canon_conv1d_part *parts, int32_t nparts,
                              void *stream);

/*
 * canon_conv1d_bwd for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops and harnesses that forbid hipMalloc).  It
 * has no counterpart in the reference.  Same arguments and results as
 * canon_conv1d_bwd, except that p->workspace / p->workspace_bytes are ignored:
 * the partial sums of dweight / dbias go to a buffer of
 * CANON_CONV1D_STATIC_SCRATCH_BYTES that is part of the library's device image
 * (every GPU the library runs on holds its own copy until the process ends).
 * Nothing is allocated or freed, by the library or by the runtime on its
 * behalf, once the device is set up (canon_conv1d_init, or one earlier call
 * of this function on the GPU: the first one makes the runtime load the
 * library's code object, which allocates).  A problem whose scratch exceeds
 * the buffer is rejected with
 * CANON_ERR_UNSUPPORTED (the metric shape, bf16 [8, 3456, 1024], needs 2.2 MB).
 * All calls on one GPU share that GPU's buffer: calls that overlap in time on
 * one GPU (different streams, different threads) race and must be serialised
 * by the caller; calls that follow each other on one stream are safe.
 */
#define CANON_CONV1D_STATIC_SCRATCH_BYTES (8 << 20)
int canon_conv1d_bwd_static(const canon_conv1d_bwd_params *p, void *stream);

/* Scratch bytes canon_conv1d_bwd needs for these sizes, strides and pointer
 * alignments; with x, dout or dx missing (NULL) the figure also covers the
 * kernel a misaligned pointer would select.  Negative if the arguments are
 * rejected. */
int64_t canon_conv1d_bwd_workspace_bytes(const canon_conv1d_bwd_params *p);
int64_t canon_conv1d_update_bwd_workspace_bytes(const canon_conv1d_update_bwd_params *p);

/*
 * Name of the kernel family the call above would launch for these arguments
 * ("bcl_vec", "bcl_vec_short", "blc_vec", "blc_vec_seq", "generic", "update_vec", "update_generic"), or NULL
 * if the arguments are rejected.  Launches nothing.  Lets a caller or a test
 * assert that a layout takes the fast path.
 */
const char *canon_conv1d_fwd_plan(const canon_conv1d_fwd_params *p);
/* Waves per block of that launch (time-contiguous rows: 8 in unmasked launches of at least 16384 waves, 1 with a
 * mask, else 4; 4 for the other vector kernels and the strided one), 0 for an empty problem, -1 if rejected. */
int canon_conv1d_fwd_plan_waves(const canon_conv1d_fwd_params *p);
const char *canon_conv1d_update_plan(const canon_conv1d_update_params *p);
const char *canon_conv1d_bwd_plan(const canon_conv1d_bwd_params *p);   /* "bwd_blc_vec" | "bwd_bcl_vec" | "bwd_generic" */
/* "blc_vec_pair" (two dense tensors of one shape: one launch of the single-tensor code), "blc_vec_parts" /
 * "update_vec_parts" (one launch over a table of parts) or "per_part" (one launch per part) */
const char *canon_conv1d_fwd_parts_plan(const canon_conv1d_fwd_params *p, const canon_conv1d_part *parts, int32_t nparts);
const char *canon_conv1d_update_parts_plan(const canon_conv1d_update_params *p, const canon_conv1d_part *parts,
                                           int32_t nparts);

#ifdef __cplusplus
}
#endif
#endif /* CANON_CONV1D_H */
