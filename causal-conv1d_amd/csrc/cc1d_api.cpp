// C-ABI front of the library: argument validation, layout selection and dispatch to
// the kernel launchers.  The checks restate, as status codes, the TORCH_CHECKs of the
// reference's host binding (csrc/causal_conv1d.cpp:158-199, 273-327, 475-542); layout
// selection follows csrc/causal_conv1d.cpp:176,296.  Nothing here allocates or
// synchronises; validation never touches the GPU, so it can run on a GPU-less host.
#include <cstring>

#include "cc1d.h"
#include "cc1d_internal.hpp"

namespace cc1d {

Tunables &tunables() {
    static Tunables t;
    return t;
}

namespace {

bool dtype_ok(int d) { return d == CC1D_F32 || d == CC1D_F16 || d == CC1D_BF16; }

// Checks shared by forward and backward for an x-shaped operand that must follow x's
// layout family (out, dout, dx).
int check_same_family(bool channel_last, int x_dtype, int batch, int seqlen, const void *ptr,
                      int64_t sb, int64_t sc, int64_t sl) {
    if (channel_last) {
        if (sc != 1) return CC1D_ERR_OUT_LAYOUT;
        if ((seqlen > 1 && sl % 8 != 0) || (batch > 1 && sb % 8 != 0)) return CC1D_ERR_CL_STRIDE_MULT8;
        if (!aligned16(ptr)) return CC1D_ERR_ALIGNMENT;
    } else {
        if (sl != 1 && seqlen > 1) return CC1D_ERR_OUT_LAYOUT;
    }
    (void)x_dtype;
    return CC1D_OK;
}

int check_x(int batch, int dim, int seqlen, const void *x, int64_t sb, int64_t sc, int64_t sl,
            bool *channel_last) {
    if (sl != 1 && sc != 1) return CC1D_ERR_X_LAYOUT;
    *channel_last = is_channel_last(sc, sl);
    if (*channel_last) {
        if (dim % 8 != 0) return CC1D_ERR_CHANNEL_MULT8;
        if ((seqlen > 1 && sl % 8 != 0) || (batch > 1 && sb % 8 != 0)) return CC1D_ERR_CL_STRIDE_MULT8;
        if (!aligned16(x)) return CC1D_ERR_ALIGNMENT;
    }
    return CC1D_OK;
}

template <typename P>
int check_common(const P *p) {
    if (p == nullptr) return CC1D_ERR_NULL_POINTER;
    if (!dtype_ok(p->x_dtype) || !dtype_ok(p->w_dtype)) return CC1D_ERR_DTYPE;
    if (p->width < 2 || p->width > 4) return CC1D_ERR_WIDTH;
    if (p->batch < 0 || p->dim < 0 || p->seqlen < 0) return CC1D_ERR_SHAPE;
    return CC1D_OK;
}

template <typename P>
bool is_empty(const P *p) {
    return p->batch == 0 || p->dim == 0 || p->seqlen == 0;
}

}  // namespace
}  // namespace cc1d

using namespace cc1d;

extern "C" {

int cc1d_abi_version(void) { return CC1D_ABI_VERSION; }

const char *cc1d_strerror(int status) {
    switch (status) {
        case CC1D_OK: return "success";
        case CC1D_ERR_NULL_POINTER: return "a required pointer is NULL";
        case CC1D_ERR_DTYPE: return "unsupported dtype (need float32, float16 or bfloat16)";
        case CC1D_ERR_WIDTH: return "causal_conv1d only supports width between 2 and 4";
        case CC1D_ERR_SHAPE: return "inconsistent or negative tensor sizes";
        case CC1D_ERR_X_LAYOUT: return "x must have stride 1 along dim or along seqlen";
        case CC1D_ERR_CHANNEL_MULT8: return "causal_conv1d only supports channel dimension divisible by 8 for now";
        case CC1D_ERR_CL_STRIDE_MULT8: return "causal_conv1d with channel last layout requires strides (stride(0) and stride(2)) to be multiples of 8";
        case CC1D_ERR_ALIGNMENT: return "channel last tensors must start on a 16-byte boundary";
        case CC1D_ERR_SEQ_IDX_LAYOUT: return "seq_idx is only supported for channel last layout";
        case CC1D_ERR_OUT_LAYOUT: return "output tensors must have the same memory layout family as x";
        case CC1D_ERR_STATE_LAYOUT: return "states tensor layout is not supported";
        case CC1D_ERR_STATE_LEN: return "conv_state length must be at least width - 1";
        case CC1D_ERR_WORKSPACE: return "backward workspace is NULL, misaligned or too small";
        case CC1D_ERR_BIAS_MISMATCH: return "bias and dbias must be given together";
        case CC1D_ERR_SEQ_IDX_STATES: return "seq_idx cannot be combined with initial/final states in backward";
        case CC1D_ERR_TOO_LARGE: return "problem too large for one launch";
        case CC1D_ERR_LAUNCH: return "HIP kernel launch failed";
        case CC1D_ERR_UNKNOWN_TUNABLE: return "unknown tunable name";
        default: return "unknown cc1d status";
    }
}

int cc1d_set_tunable(const char *name, int32_t value) {
    if (name == nullptr) return CC1D_ERR_NULL_POINTER;
    Tunables &t = tunables();
    if (!std::strcmp(name, "fwd_cl_rows")) t.fwd_cl_rows = value;
    else if (!std::strcmp(name, "fwd_cl_half_vec")) t.fwd_cl_half_vec = value;
    else if (!std::strcmp(name, "fwd_cl_chunk_runs")) t.fwd_cl_chunk_runs = value;
    else if (!std::strcmp(name, "bwd_cl_rows")) t.bwd_cl_rows = value;
    else if (!std::strcmp(name, "bwd_cl_chunk_runs")) t.bwd_cl_chunk_runs = value;
    else if (!std::strcmp(name, "fwd_cf_vecs")) t.fwd_cf_vecs = value;
    else if (!std::strcmp(name, "bwd_cf_parts")) t.bwd_cf_parts = value;
    else return CC1D_ERR_UNKNOWN_TUNABLE;
    return CC1D_OK;
}

int cc1d_get_tunable(const char *name, int32_t *value) {
    if (name == nullptr || value == nullptr) return CC1D_ERR_NULL_POINTER;
    const Tunables &t = tunables();
    if (!std::strcmp(name, "fwd_cl_rows")) *value = t.fwd_cl_rows;
    else if (!std::strcmp(name, "fwd_cl_half_vec")) *value = t.fwd_cl_half_vec;
    else if (!std::strcmp(name, "fwd_cl_chunk_runs")) *value = t.fwd_cl_chunk_runs;
    else if (!std::strcmp(name, "bwd_cl_rows")) *value = t.bwd_cl_rows;
    else if (!std::strcmp(name, "bwd_cl_chunk_runs")) *value = t.bwd_cl_chunk_runs;
    else if (!std::strcmp(name, "fwd_cf_vecs")) *value = t.fwd_cf_vecs;
    else if (!std::strcmp(name, "bwd_cf_parts")) *value = t.bwd_cf_parts;
    else return CC1D_ERR_UNKNOWN_TUNABLE;
    return CC1D_OK;
}

// ------------------------------------------------------------------------- forward
int cc1d_validate_fwd(const cc1d_fwd_params *p) {
    int st = check_common(p);
    if (st != CC1D_OK) return st;
    if (is_empty(p)) return CC1D_OK;
    if (p->x == nullptr || p->weight == nullptr || p->out == nullptr) return CC1D_ERR_NULL_POINTER;
    bool cl = false;
    st = check_x(p->batch, p->dim, p->seqlen, p->x, p->x_stride_b, p->x_stride_c, p->x_stride_l, &cl);
    if (st != CC1D_OK) return st;
    st = check_same_family(cl, p->x_dtype, p->batch, p->seqlen, p->out, p->out_stride_b,
                           p->out_stride_c, p->out_stride_l);
    if (st != CC1D_OK) return st;
    if (p->seq_idx != nullptr && !cl) return CC1D_ERR_SEQ_IDX_LAYOUT;
    return CC1D_OK;
}

int cc1d_fwd(const cc1d_fwd_params *p, cc1d_stream_t stream) {
    const int st = cc1d_validate_fwd(p);
    if (st != CC1D_OK) return st;
    if (is_empty(p)) return CC1D_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return is_channel_last(p->x_stride_c, p->x_stride_l) ? launch_fwd_channellast(*p, nullptr, s)
                                                         : launch_fwd_channelfirst(*p, s);
}

int cc1d_fwd_varlen_states(const cc1d_fwd_params *fwd, const cc1d_varlen_params *gather, cc1d_stream_t stream) {
    int st = cc1d_validate_fwd(fwd);
    if (st != CC1D_OK) return st;
    st = cc1d_validate_varlen_states(gather);
    if (st != CC1D_OK) return st;
    const bool no_gather = gather->batch == 0 || gather->dim == 0 || gather->state_len == 0;
    if (is_empty(fwd) || no_gather) {
        st = cc1d_fwd(fwd, stream);
        return st != CC1D_OK ? st : cc1d_varlen_states(gather, stream);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    // One launch when the forward is channel-last and the gather moves whole 16-byte vectors
    // of elements as wide as the forward's; two launches otherwise.
    if (is_channel_last(fwd->x_stride_c, fwd->x_stride_l) && varlen_fits_fwd_launch(*fwd, *gather))
        return launch_fwd_channellast(*fwd, gather, s);
    st = cc1d_fwd(fwd, stream);
    return st != CC1D_OK ? st : launch_varlen_states(*gather, s);
}

// ------------------------------------------------------------------------ backward
int cc1d_validate_bwd(const cc1d_bwd_params *p) {
    int st = check_common(p);
    if (st != CC1D_OK) return st;
    if ((p->bias != nullptr) != (p->dbias != nullptr)) return CC1D_ERR_BIAS_MISMATCH;
    if (is_empty(p)) return CC1D_OK;
    if (p->x == nullptr || p->weight == nullptr || p->dout == nullptr || p->dx == nullptr ||
        p->dweight == nullptr)
        return CC1D_ERR_NULL_POINTER;
    bool cl = false;
    st = check_x(p->batch, p->dim, p->seqlen, p->x, p->x_stride_b, p->x_stride_c, p->x_stride_l, &cl);
    if (st != CC1D_OK) return st;
    st = check_same_family(cl, p->x_dtype, p->batch, p->seqlen, p->dout, p->dout_stride_b,
                           p->dout_stride_c, p->dout_stride_l);
    if (st != CC1D_OK) return st;
    st = check_same_family(cl, p->x_dtype, p->batch, p->seqlen, p->dx, p->dx_stride_b,
                           p->dx_stride_c, p->dx_stride_l);
    if (st != CC1D_OK) return st;
    if (p->seq_idx != nullptr) {
        if (!cl) return CC1D_ERR_SEQ_IDX_LAYOUT;
        if (p->initial_states != nullptr || p->dfinal_states != nullptr || p->dinitial_states != nullptr)
            return CC1D_ERR_SEQ_IDX_STATES;
    }
    return CC1D_OK;
}

int cc1d_bwd_workspace_bytes(const cc1d_bwd_params *p, size_t *bytes) {
    if (bytes == nullptr) return CC1D_ERR_NULL_POINTER;
    *bytes = 0;
    const int st = cc1d_validate_bwd(p);
    if (st != CC1D_OK) return st;
    if (is_empty(p)) return CC1D_OK;
    *bytes = is_channel_last(p->x_stride_c, p->x_stride_l) ? bwd_channellast_workspace_bytes(*p)
                                                            : bwd_channelfirst_workspace_bytes(*p);
    return CC1D_OK;
}

int cc1d_bwd(const cc1d_bwd_params *p, void *workspace, size_t workspace_bytes, cc1d_stream_t stream) {
    size_t need = 0;
    const int st = cc1d_bwd_workspace_bytes(p, &need);
    if (st != CC1D_OK) return st;
    if (is_empty(p)) {
        // Nothing to sum: with overwrite_dweight the outputs still have to become zeros.
        if (p->overwrite_dweight != 0 && p->dim > 0 && p->dweight != nullptr)
            return launch_bwd_finalize(nullptr, 0, *p, static_cast<hipStream_t>(stream));
        return CC1D_OK;
    }
    if (need > 0 && (workspace == nullptr || !aligned16(workspace) || workspace_bytes < need))
        return CC1D_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return is_channel_last(p->x_stride_c, p->x_stride_l) ? launch_bwd_channellast(*p, workspace, s)
                                                         : launch_bwd_channelfirst(*p, workspace, s);
}

// -------------------------------------------------------------------------- update
int cc1d_validate_update(const cc1d_update_params *p) {
    int st = check_common(p);
    if (st != CC1D_OK) return st;
    if (p->state_len < p->width - 1) return CC1D_ERR_STATE_LEN;
    if (p->state_batch < 0) return CC1D_ERR_SHAPE;
    if (p->conv_state_indices == nullptr && p->state_batch != p->batch) return CC1D_ERR_SHAPE;
    if (is_empty(p)) return CC1D_OK;
    if (p->x == nullptr || p->weight == nullptr || p->out == nullptr || p->conv_state == nullptr)
        return CC1D_ERR_NULL_POINTER;
    return CC1D_OK;
}

int cc1d_update(const cc1d_update_params *p, cc1d_stream_t stream) {
    const int st = cc1d_validate_update(p);
    if (st != CC1D_OK) return st;
    if (is_empty(p)) return CC1D_OK;
    return launch_update(*p, static_cast<hipStream_t>(stream));
}

// ------------------------------------------------------------------- varlen states
int cc1d_validate_varlen_states(const cc1d_varlen_params *p) {
    if (p == nullptr) return CC1D_ERR_NULL_POINTER;
    if (!dtype_ok(p->x_dtype)) return CC1D_ERR_DTYPE;
    if (p->batch < 0 || p->dim < 0 || p->state_len < 0 || p->total_tokens < 0) return CC1D_ERR_SHAPE;
    if (p->batch == 0 || p->dim == 0 || p->state_len == 0) return CC1D_OK;
    if (p->cu_seqlens == nullptr || p->states == nullptr) return CC1D_ERR_NULL_POINTER;
    if (p->x == nullptr && p->total_tokens > 0) return CC1D_ERR_NULL_POINTER;
    return CC1D_OK;
}

int cc1d_varlen_states(const cc1d_varlen_params *p, cc1d_stream_t stream) {
    const int st = cc1d_validate_varlen_states(p);
    if (st != CC1D_OK) return st;
    if (p->batch == 0 || p->dim == 0 || p->state_len == 0) return CC1D_OK;
    return launch_varlen_states(*p, static_cast<hipStream_t>(stream));
}

}  // extern "C"
