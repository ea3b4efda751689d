/*
 * cc1d.h — C ABI of the MI355X (gfx950) causal depthwise conv1d kernel library.
 *
 * This is the drop-in boundary for the device side of Dao-AILab/causal-conv1d: every
 * entry point below names the reference host function (file:line under the reference
 * tree) whose job it takes over.  The ABI is plain C: raw device pointers, element
 * strides as int64_t, sizes as int32_t, an opaque stream handle.  Nothing here
 * allocates, frees, synchronises the host or throws; every function returns a
 * cc1d_status (0 = success, negative = error, text via cc1d_strerror()).
 *
 * The operator (fp32 accumulation for every I/O type):
 *
 *   out[b,c,t] = act( bias[c] + sum_{w=0..W-1} weight[c,w] * xpad[b,c,t-(W-1-w)] )
 *   xpad[b,c,p] = x[b,c,p]                    (p >= 0)
 *               = initial_states[b,c,p+W-1]   (-(W-1) <= p < 0, if given; else 0)
 *   act(z) = z  or  z / (1 + exp(-z))
 *
 * With seq_idx, a tap contributes only when seq_idx[b,tap] == seq_idx[b,t]; positions
 * with seq_idx[b,t] < 0 produce exactly 0.
 */
#ifndef CC1D_H_
#define CC1D_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CC1D_ABI_VERSION 1

/* Element types.  x-like tensors (x, out, states, dout, dx) share `x_dtype`;
 * weight and bias share `w_dtype`.  All nine combinations are accepted, as in the
 * reference's instantiation list (csrc/causal_conv1d_fwd.cu:383-401). */
typedef enum cc1d_dtype {
    CC1D_F32 = 0,
    CC1D_F16 = 1,
    CC1D_BF16 = 2
} cc1d_dtype;

typedef enum cc1d_status {
    CC1D_OK = 0,
    CC1D_ERR_NULL_POINTER = -1,      /* a required pointer is NULL */
    CC1D_ERR_DTYPE = -2,             /* dtype enum out of range */
    CC1D_ERR_WIDTH = -3,             /* width outside [2, 4] (causal_conv1d.cpp:182) */
    CC1D_ERR_SHAPE = -4,             /* a size is negative or inconsistent */
    CC1D_ERR_X_LAYOUT = -5,          /* x needs stride 1 along dim or seqlen (causal_conv1d.cpp:175) */
    CC1D_ERR_CHANNEL_MULT8 = -6,     /* channel-last needs dim % 8 == 0 (causal_conv1d.cpp:179) */
    CC1D_ERR_CL_STRIDE_MULT8 = -7,   /* channel-last needs batch/seqlen strides % 8 == 0 (causal_conv1d.cpp:180) */
    CC1D_ERR_ALIGNMENT = -8,         /* a channel-last base pointer is not 16-byte aligned */
    CC1D_ERR_SEQ_IDX_LAYOUT = -9,    /* seq_idx needs channel-last x (causal_conv1d.cpp:193) */
    CC1D_ERR_OUT_LAYOUT = -10,       /* an output tensor does not have x's layout */
    CC1D_ERR_STATE_LAYOUT = -11,     /* states tensor layout not usable (causal_conv1d.cpp:218,233,379) */
    CC1D_ERR_STATE_LEN = -12,        /* conv_state_len < width - 1 (causal_conv1d.cpp:491) */
    CC1D_ERR_WORKSPACE = -13,        /* workspace NULL, misaligned or too small */
    CC1D_ERR_BIAS_MISMATCH = -14,    /* bias given without dbias or the reverse (causal_conv1d.cpp:281) */
    CC1D_ERR_SEQ_IDX_STATES = -15,   /* seq_idx combined with initial/final states */
    CC1D_ERR_TOO_LARGE = -16,        /* one batch entry alone exceeds what a grid can express */
    CC1D_ERR_LAUNCH = -17,           /* the HIP runtime refused the launch */
    CC1D_ERR_UNKNOWN_TUNABLE = -18,
    CC1D_ERR_WORKSPACE_LIMIT = -19,  /* cc1d_bwd_noalloc: the problem needs more than the built-in workspace */
    CC1D_ERR_IN_PLACE = -20          /* out shares elements with x, or dx with x or dout: no kernel works in place */
} cc1d_status;

/* Opaque stream handle: pass a hipStream_t (NULL = the default stream). */
typedef void *cc1d_stream_t;

/* ------------------------------------------------------------------------------------
 * Forward.  Replaces causal_conv1d_fwd (csrc/causal_conv1d.cpp:149-258), the parameter
 * block ConvParamsBase (csrc/causal_conv1d.h:9-54) and both launchers
 * causal_conv1d_fwd_cuda / causal_conv1d_channellast_fwd_cuda
 * (csrc/causal_conv1d_fwd.cu:139-170, 350-381).
 *
 * Layout is inferred exactly as the reference does: channel-last iff
 * x_stride_c == 1 && x_stride_l > 1 (causal_conv1d.cpp:176), otherwise channel-first
 * (x_stride_l must be 1).  Unlike the reference, initial_states / final_states are
 * accepted for both layouts.
 * ---------------------------------------------------------------------------------- */
typedef struct cc1d_fwd_params {
    int32_t batch, dim, seqlen, width;
    int32_t x_dtype;                 /* cc1d_dtype of x, out, initial_states, final_states */
    int32_t w_dtype;                 /* cc1d_dtype of weight, bias */
    int32_t silu;                    /* 0 = identity, 1 = SiLU */
    int32_t reserved0;

    const void *x;                   /* (batch, dim, seqlen) */
    int64_t x_stride_b, x_stride_c, x_stride_l;
    const void *weight;              /* (dim, width) */
    int64_t w_stride_c, w_stride_w;
    const void *bias;                /* (dim,) unit stride, or NULL */
    void *out;                       /* (batch, dim, seqlen), same layout family as x */
    int64_t out_stride_b, out_stride_c, out_stride_l;

    const int32_t *seq_idx;          /* contiguous (batch, seqlen) or NULL; channel-last only */

    const void *initial_states;      /* (batch, dim, width-1) or NULL */
    int64_t init_stride_b, init_stride_c, init_stride_l;
    void *final_states;              /* (batch, dim, width-1) or NULL */
    int64_t final_stride_b, final_stride_c, final_stride_l;
} cc1d_fwd_params;

/* Host-only checks (no GPU needed); the same checks run inside cc1d_fwd. */
int cc1d_validate_fwd(const cc1d_fwd_params *p);
int cc1d_fwd(const cc1d_fwd_params *p, cc1d_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Backward.  Replaces causal_conv1d_bwd (csrc/causal_conv1d.cpp:260-463), ConvParamsBwd
 * (csrc/causal_conv1d.h:56-88) and causal_conv1d_bwd_cuda /
 * causal_conv1d_channellast_bwd_cuda (csrc/causal_conv1d_bwd.cu:261-293, 591-632).
 *
 * dweight (fp32, (dim, width)) and dbias (fp32, (dim,)) are ACCUMULATED INTO, like the
 * reference (atomicAdd at bwd.cu:243,255 / add_ at causal_conv1d.cpp:452-459): the
 * caller zeroes them first.  With overwrite_dweight = 1 they are plain outputs instead and
 * need no zeroing (two fill launches fewer per backward call).  The reduction is always a
 * fixed-order two-stage sum (partials in the workspace, then one ordered pass), so results are
 * bit-reproducible run to run; the reference's `deterministic` switch
 * (causal_conv1d.cpp:21-28, 388-437) has nothing left to select.
 *
 * The workspace is caller-owned device memory, 16-byte aligned, of at least
 * cc1d_bwd_workspace_bytes() bytes (the reference allocates its own with at::zeros,
 * causal_conv1d.cpp:396-429).  It needs no initialisation.  A problem too large for one grid is
 * launched as slices of the batch, one after the other on the stream, each adding into
 * dweight / dbias: the sums then follow the slice order (still the same bits run to run).
 * ---------------------------------------------------------------------------------- */
typedef struct cc1d_bwd_params {
    int32_t batch, dim, seqlen, width;
    int32_t x_dtype;                 /* of x, dout, dx, initial_states, dfinal_states, dinitial_states */
    int32_t w_dtype;                 /* of weight, bias */
    int32_t silu;
    int32_t overwrite_dweight;       /* 0: add into dweight / dbias; 1: store the sums, ignore what was there */

    const void *x;
    int64_t x_stride_b, x_stride_c, x_stride_l;
    const void *weight;
    int64_t w_stride_c, w_stride_w;
    const void *bias;                /* or NULL (then dbias must be NULL) */
    const void *dout;                /* same layout family as x */
    int64_t dout_stride_b, dout_stride_c, dout_stride_l;
    const int32_t *seq_idx;          /* or NULL; channel-last only */
    const void *initial_states;      /* or NULL */
    int64_t init_stride_b, init_stride_c, init_stride_l;
    const void *dfinal_states;       /* or NULL; any strides */
    int64_t dfinal_stride_b, dfinal_stride_c, dfinal_stride_l;

    void *dx;                        /* same layout family as x */
    int64_t dx_stride_b, dx_stride_c, dx_stride_l;
    float *dweight;                  /* fp32 (dim, width), accumulated into (or overwritten) */
    int64_t dw_stride_c, dw_stride_w;
    float *dbias;                    /* fp32 (dim,) unit stride, like dweight, or NULL */
    void *dinitial_states;           /* or NULL */
    int64_t dinit_stride_b, dinit_stride_c, dinit_stride_l;
} cc1d_bwd_params;

int cc1d_validate_bwd(const cc1d_bwd_params *p);
int cc1d_bwd_workspace_bytes(const cc1d_bwd_params *p, size_t *bytes);
int cc1d_bwd(const cc1d_bwd_params *p, void *workspace, size_t workspace_bytes,
             cc1d_stream_t stream);

/* The backward for callers that cannot allocate device memory: tight serving loops, harnesses
 * that forbid hipMalloc, code that is to be captured into a HIP graph (capture itself has not been
 * verified with this library; what this entry point guarantees is that it allocates nothing).  No counterpart in the reference, whose
 * backward allocates its workspaces itself with at::zeros (csrc/causal_conv1d.cpp:396-429).
 * Same kernels, same order of additions and same results as cc1d_bwd; the partial-sum workspace
 * is a fixed array of CC1D_BWD_NOALLOC_MAX_WORKSPACE_BYTES inside this library's device image
 * (one copy per GPU, held from the first use of the library on that GPU until the process ends).
 * A problem whose cc1d_bwd_workspace_bytes() exceeds that size is refused with
 * CC1D_ERR_WORKSPACE_LIMIT before anything is launched (16 MiB covers, for instance, the bf16
 * prefill shape (8, 5376, 2048) channel-last at 13.8 MB; a channel-first problem needs
 * batch x ceil(row vectors / 256) x (width + 1) x dim floats once its rows are longer than 64
 * sixteen-byte vectors -- 1.3 MB for fp16 (4, 4096, 8192) -- and none for shorter rows at
 * dim >= 4096).  Calls no hipMalloc / hipFree and nothing that allocates.  The device that owns
 * `stream` must be the current device.  All calls on one GPU share that GPU's array: calls that
 * overlap in time on one GPU (different streams, no ordering between them) race; calls on one
 * stream never do.  The array needs no clearing between calls (every plane that is read was
 * written by the same call).  The first call on a device looks the array's address up
 * (hipGetSymbolAddress): make that call before any stream of the device is being captured. */
#define CC1D_BWD_NOALLOC_MAX_WORKSPACE_BYTES (16u * 1024u * 1024u)
int cc1d_bwd_noalloc(const cc1d_bwd_params *p, cc1d_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Decode-step update.  Replaces causal_conv1d_update (csrc/causal_conv1d.cpp:465-557)
 * and causal_conv1d_update_cuda (csrc/causal_conv1d_update.cu:116-136).
 * conv_state is advanced in place: linear shift when cache_seqlens == NULL
 * (update.cu:72-84,95-98), circular buffer indexed by cache_seqlens[b] % state_len
 * otherwise (update.cu:63-65,86-90,99-103).  conv_state_indices[b] picks the state
 * row; a negative index writes zeros to out[b] and leaves every state row untouched
 * (update.cu:43-54).
 * ---------------------------------------------------------------------------------- */
typedef struct cc1d_update_params {
    int32_t batch, dim, seqlen, width;
    int32_t state_len;               /* conv_state.size(2), >= width - 1 */
    int32_t state_batch;             /* conv_state.size(0); == batch unless indices are given */
    int32_t x_dtype;                 /* of x, out, conv_state */
    int32_t w_dtype;
    int32_t silu;
    int32_t reserved0;

    const void *x;                   /* (batch, dim, seqlen), any strides */
    int64_t x_stride_b, x_stride_c, x_stride_l;
    void *conv_state;                /* (state_batch, dim, state_len), any strides */
    int64_t state_stride_b, state_stride_c, state_stride_l;
    const void *weight;
    int64_t w_stride_c, w_stride_w;
    const void *bias;                /* or NULL */
    void *out;                       /* (batch, dim, seqlen), any strides */
    int64_t out_stride_b, out_stride_c, out_stride_l;
    const int32_t *cache_seqlens;    /* (batch,) unit stride, or NULL */
    const int32_t *conv_state_indices; /* (batch,) unit stride, or NULL */
} cc1d_update_params;

int cc1d_validate_update(const cc1d_update_params *p);
int cc1d_update(const cc1d_update_params *p, cc1d_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Varlen final-state gather.  Replaces the Triton kernel _causal_conv1d_varlen_states
 * and its launch (causal_conv1d/causal_conv1d_varlen.py:8-64):
 *   states[b, :, state_len-k .. state_len) = x[end_b-k .. end_b, :],
 *   k = min(state_len, end_b - start_b); the leading state_len-k columns are zero.
 * ---------------------------------------------------------------------------------- */
typedef struct cc1d_varlen_params {
    int32_t batch;                   /* number of sequences = len(cu_seqlens) - 1 */
    int32_t dim;
    int32_t state_len;
    int32_t x_dtype;                 /* of x and states (a pure copy: any 2- or 4-byte type) */
    int32_t cu_seqlens_is_int64;     /* 0: int32 entries, 1: int64 entries */
    int32_t reserved0;
    int64_t total_tokens;            /* x.size(0) */

    const void *x;                   /* (total_tokens, dim) */
    int64_t x_stride_t, x_stride_c;
    const void *cu_seqlens;          /* (batch + 1,) contiguous, sorted */
    void *states;                    /* (batch, dim, state_len) */
    int64_t states_stride_b, states_stride_c, states_stride_l;
} cc1d_varlen_params;

int cc1d_validate_varlen_states(const cc1d_varlen_params *p);
int cc1d_varlen_states(const cc1d_varlen_params *p, cc1d_stream_t stream);

/* Forward and gather together: what a varlen prefill -> decode hand-off issues back to back,
 * causal_conv1d_fn over the packed batch (causal_conv1d/causal_conv1d_interface.py:99-129) and
 * causal_conv1d_varlen_states on the same tokens (causal_conv1d/causal_conv1d_varlen.py:35-64);
 * the reference has no single call for the pair.  Results are those of cc1d_fwd followed by
 * cc1d_varlen_states.  The gather reads only its own x, so it does not wait for the forward:
 * with a channel-last forward and a gather whose x and states have unit stride along dim
 * (16-byte aligned rows, same element size as the forward's x) both run in ONE kernel launch,
 * the gather in extra workgroups at the end of the forward's grid; any other combination is
 * two launches on `stream`.  `gather->states` must not overlap anything the forward writes. */
int cc1d_fwd_varlen_states(const cc1d_fwd_params *fwd, const cc1d_varlen_params *gather,
                           cc1d_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Misc.
 * ---------------------------------------------------------------------------------- */
const char *cc1d_strerror(int status);
int cc1d_abi_version(void);

/* Diagnostic, host-only: writes the file name of the HIP runtime library this library's launches
 * go through (the shared object that defines hipLaunchKernel for it) into path[0..size), always
 * NUL-terminated.  A process must hold exactly one HIP runtime: a host that also uses PyTorch
 * loads PyTorch (or PyTorch's own libamdhip64.so) BEFORE this library, so that this library's
 * NEEDED entry binds to that copy, and can check here that it did.  No counterpart in the
 * reference, whose kernels are linked into the PyTorch extension itself.  Returns CC1D_OK,
 * CC1D_ERR_NULL_POINTER, or CC1D_ERR_SHAPE when the name does not fit. */
int cc1d_hip_runtime_path(char *path, size_t size);

/* Benchmarking and test hooks: override a launch heuristic (0 restores the built-in choice).
 * Process-global; each knob is an atomic integer read once per launch, so setting one while
 * another thread launches is safe, and no knob changes what a launch computes (only how the
 * work is cut into workgroups and launches).  Known names:
 *   "fwd_cl_rows"   rows of seqlen walked by one lane of the channel-last forward
 *   "fwd_cl_half_vec" -1 = the channel-last forward reads its taps with the general loader even
 *                   when they are packed
 *   "fwd_cl_chunk_runs" workgroup order of the channel-last forward: n > 0 = an XCD takes chunks of n
 *                   consecutive runs, the 8 XCDs side by side on 8 neighbouring chunks; -1 = one
 *                   contiguous slice of the launch per XCD; -n, n > 1 = chunks of n-1 workgroups
 *                   (-2: single workgroups, the hardware's own round-robin order)
 *   "bwd_cl_rows"   same for the channel-last backward
 *   "bwd_cl_chunk_runs" the same for the channel-last backward, whose workgroups take 4 runs each:
 *                   n >= 4 = chunks of n / 4 workgroup rows; -1 = one contiguous slice per XCD
 *   "bwd_cl_lane_bytes" bytes of a row per lane in the channel-last backward on 16-bit data: 4 or 8
 *                   (0: 8 where the rows of dx do not start on 64-byte boundaries, else 4)
 *   "fwd_cf_vecs"   16-byte vectors per wave segment in the channel-first forward
 *   "bwd_cf_parts"  partitions of (batch x seqlen) per channel in the channel-first backward
 *   "launch_limit_shift" n: one launch holds at most 2^(31-n) threads instead of 2^31 (n <= 24), so
 *                   that small tensors exercise the batch slicing below
 *
 * A problem with more work items than one grid holds (2^31 threads) is cut along the batch into
 * slices that fit, launched back to back on the stream; forward, backward and update accept any
 * batch.  CC1D_ERR_TOO_LARGE is left for a single batch entry that does not fit one launch.
 */
int cc1d_set_tunable(const char *name, int32_t value);
int cc1d_get_tunable(const char *name, int32_t *value);

#ifdef __cplusplus
}
#endif
#endif /* CC1D_H_ */
