// C-ABI front of the library: argument validation, layout selection and dispatch to
// the kernel launchers.  The checks restate, as status codes, the TORCH_CHECKs of the
// reference's host binding (csrc/causal_conv1d.cpp:158-199, 273-327, 475-542); layout
// selection follows csrc/causal_conv1d.cpp:176,296.  Nothing here allocates or
// synchronises; validation never touches the GPU, so it can run on a GPU-less host.
#include <dlfcn.h>

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

// Byte range [lo, hi) a (batch, dim, width-1) states tensor with non-negative strides covers.
void states_extent(const void *base, int64_t sb, int64_t sc, int64_t sl, const cc1d_fwd_params &p,
                   uintptr_t *lo, uintptr_t *hi) {
    auto span = [](int64_t n, int64_t stride) { return n > 1 ? (uint64_t)(n - 1) * (uint64_t)(stride < 0 ? -stride : stride) : 0u; };
    const uint64_t last = span(p.batch, sb) + span(p.dim, sc) + span(p.width - 1, sl);
    *lo = reinterpret_cast<uintptr_t>(base);
    *hi = *lo + (uintptr_t)((last + 1) * (uint64_t)elem_bytes(p.x_dtype));
}

// Do initial_states and final_states share an element?  Disjoint byte ranges: no.  Otherwise, for two
// views with the same strides (two slices of one buffer), exactly: they share an element iff the
// distance between their bases is db*sb + dc*sc + dl*sl for index differences inside the shape.
// Views with different strides whose byte ranges intersect count as overlapping.
bool states_overlap(const cc1d_fwd_params &p) {
    uintptr_t a0, a1, b0, b1;
    states_extent(p.initial_states, p.init_stride_b, p.init_stride_c, p.init_stride_l, p, &a0, &a1);
    states_extent(p.final_states, p.final_stride_b, p.final_stride_c, p.final_stride_l, p, &b0, &b1);
    if (!(a0 < b1 && b0 < a1)) return false;
    const int64_t sb = p.init_stride_b, sc = p.init_stride_c, sl = p.init_stride_l;
    const bool same_strides = (p.batch <= 1 || sb == p.final_stride_b) && (p.dim <= 1 || sc == p.final_stride_c) &&
                              (p.width <= 2 || sl == p.final_stride_l);
    const int64_t eb = elem_bytes(p.x_dtype);
    const int64_t bytes = (int64_t)b0 - (int64_t)a0;
    if (!same_strides || bytes % eb != 0) return true;
    const int64_t delta = bytes / eb;
    for (int64_t dl = -(p.width - 2); dl <= p.width - 2; ++dl) {
        for (int64_t db = -((int64_t)p.batch - 1); db <= (int64_t)p.batch - 1; ++db) {
            const int64_t rest = delta - (p.width > 2 ? dl * sl : 0) - (p.batch > 1 ? db * sb : 0);
            if (p.dim <= 1 || sc == 0) {
                if (rest == 0) return true;
            } else if (rest % sc == 0 && rest / sc > -(int64_t)p.dim && rest / sc < (int64_t)p.dim) {
                return true;
            }
        }
    }
    return false;
}

// Do an input and an output of shape (batch, dim, seqlen) provably share an element?  No kernel
// here works in place: a row's halo is read by another wavefront than the one that writes the
// positions in front of it.  Decided only where it can be decided exactly -- the same strides for
// both views, nested (each stride larger than everything the smaller ones span): the views then
// share an element iff the distance between their bases is a sum of in-range index differences,
// and with nested strides each difference has two candidates at most.  Anything else (different
// strides, byte ranges that merely interleave, as two column slices of one wider buffer do) is
// let through, as the reference lets everything through.
bool views_share_an_element(int batch, int dim, int seqlen, int eb, const void *a, const void *b, int64_t sb,
                            int64_t sc, int64_t sl, int64_t sb2, int64_t sc2, int64_t sl2) {
    if (a == nullptr || b == nullptr) return false;
    int64_t n[3] = {batch, dim, seqlen}, st[3] = {sb, sc, sl}, st2[3] = {sb2, sc2, sl2};
    for (int i = 0; i < 3; ++i)
        if (n[i] > 1 && (st[i] != st2[i] || st[i] <= 0)) return false;
    const int64_t bytes = (int64_t)(reinterpret_cast<uintptr_t>(b) - reinterpret_cast<uintptr_t>(a));
    if (bytes % eb != 0) return false;
    // dimensions that matter, by falling stride
    int order[3], m = 0;
    for (int i = 0; i < 3; ++i)
        if (n[i] > 1) order[m++] = i;
    for (int i = 0; i < m; ++i)
        for (int j = i + 1; j < m; ++j)
            if (st[order[j]] > st[order[i]]) { const int t = order[i]; order[i] = order[j]; order[j] = t; }
    int64_t inner[3];                                  // what the dimensions behind i span
    for (int i = m - 1; i >= 0; --i) {
        inner[i] = i == m - 1 ? 0 : inner[i + 1] + (n[order[i + 1]] - 1) * st[order[i + 1]];
        if (st[order[i]] <= inner[i]) return false;   // not nested: undecided
    }
    // depth-first over the candidates: |rest - d * stride| must not exceed what is left behind
    struct Walk {
        const int64_t *n, *st, *inner; const int *order; int m;
        bool operator()(int i, int64_t rest) const {
            if (i == m) return rest == 0;
            const int64_t s = st[order[i]];
            int64_t d = rest / s;
            if (rest % s != 0 && rest < 0) --d;        // floor
            for (int64_t c = d; c <= d + 1; ++c) {
                const int64_t r = rest - c * s;
                if (c > -n[order[i]] && c < n[order[i]] && r >= -inner[i] && r <= inner[i] && (*this)(i + 1, r)) return true;
            }
            return false;
        }
    };
    return Walk{n, st, inner, order, m}(0, bytes / eb);
}

// ---- batch slicing ---------------------------------------------------------------------------
// A launcher refuses, before launching anything, a problem that needs more work items than one
// grid holds (CC1D_ERR_TOO_LARGE).  Every batch entry is independent, so the front then halves
// the batch until the pieces fit and launches them one after the other on the same stream: the
// reference's grid(batch, dim) launch has no such ceiling, and neither has this library.
const void *advance(const void *base, int64_t elems, int bytes_per_elem) {
    return base == nullptr ? nullptr : static_cast<const char *>(base) + elems * bytes_per_elem;
}
void *advance(void *base, int64_t elems, int bytes_per_elem) {
    return base == nullptr ? nullptr : static_cast<char *>(base) + elems * bytes_per_elem;
}

cc1d_fwd_params batch_slice(const cc1d_fwd_params &p, int b0, int n) {
    cc1d_fwd_params q = p;
    const int eb = elem_bytes(p.x_dtype);
    q.batch = n;
    q.x = advance(p.x, b0 * p.x_stride_b, eb);
    q.out = advance(p.out, b0 * p.out_stride_b, eb);
    q.seq_idx = static_cast<const int32_t *>(advance(p.seq_idx, (int64_t)b0 * p.seqlen, 4));
    q.initial_states = advance(p.initial_states, b0 * p.init_stride_b, eb);
    q.final_states = advance(p.final_states, b0 * p.final_stride_b, eb);
    return q;
}

cc1d_bwd_params batch_slice(const cc1d_bwd_params &p, int b0, int n) {
    cc1d_bwd_params q = p;
    const int eb = elem_bytes(p.x_dtype);
    q.batch = n;
    q.x = advance(p.x, b0 * p.x_stride_b, eb);
    q.dout = advance(p.dout, b0 * p.dout_stride_b, eb);
    q.dx = advance(p.dx, b0 * p.dx_stride_b, eb);
    q.seq_idx = static_cast<const int32_t *>(advance(p.seq_idx, (int64_t)b0 * p.seqlen, 4));
    q.initial_states = advance(p.initial_states, b0 * p.init_stride_b, eb);
    q.dfinal_states = advance(p.dfinal_states, b0 * p.dfinal_stride_b, eb);
    q.dinitial_states = advance(p.dinitial_states, b0 * p.dinit_stride_b, eb);
    if (b0 > 0) q.overwrite_dweight = 0;              // later slices add to what the first one stored
    return q;
}

cc1d_update_params batch_slice(const cc1d_update_params &p, int b0, int n) {
    cc1d_update_params q = p;
    const int eb = elem_bytes(p.x_dtype);
    q.batch = n;
    q.x = advance(p.x, b0 * p.x_stride_b, eb);
    q.out = advance(p.out, b0 * p.out_stride_b, eb);
    q.cache_seqlens = static_cast<const int32_t *>(advance(p.cache_seqlens, b0, 4));
    if (p.conv_state_indices != nullptr) {
        q.conv_state_indices = static_cast<const int32_t *>(advance(p.conv_state_indices, b0, 4));
    } else {
        q.conv_state = advance(p.conv_state, b0 * p.state_stride_b, eb);
        q.state_batch = n;
    }
    return q;
}

// launch(params) for halves of the batch (recursively) while it answers CC1D_ERR_TOO_LARGE.
// Slices run in batch order.
template <typename P, typename F>
int launch_halves(const P &p, F &&launch) {
    const int st = launch(p);
    if (st != CC1D_ERR_TOO_LARGE || p.batch < 2) return st;
    const int head = p.batch / 2;
    const int first = launch_halves(batch_slice(p, 0, head), launch);
    if (first != CC1D_OK) return first;
    return launch_halves(batch_slice(p, head, p.batch - head), launch);
}

// launch(params) for the whole batch or, when that answers CC1D_ERR_TOO_LARGE, in slices.  Whether
// slicing can succeed is settled before the first slice runs: a launcher is asked, in probe mode,
// about a single batch entry (the smallest slice the halving can end in; a problem whose launch
// size does not shrink with the batch fails here), so an error leaves every output untouched
// instead of partly written.
template <typename P, typename F>
int launch_in_batch_slices(const P &p, F &&launch) {
    const int st = launch(p);
    if (st != CC1D_ERR_TOO_LARGE || p.batch < 2) return st;
    {
        ProbeScope probe;
        const int one = launch(batch_slice(p, 0, 1));
        if (one != CC1D_OK) return one;
    }
    return launch_halves(p, launch);
}

size_t bwd_workspace_one_launch(const cc1d_bwd_params &p) {
    return is_channel_last(p.x_stride_c, p.x_stride_l) ? bwd_channellast_workspace_bytes(p)
                                                       : bwd_channelfirst_workspace_bytes(p);
}
bool bwd_fits_one_launch(const cc1d_bwd_params &p) {
    return is_channel_last(p.x_stride_c, p.x_stride_l) ? bwd_channellast_fits(p) : bwd_channelfirst_fits(p);
}
// The workspace the largest slice needs: slices run one after the other and share it.
size_t bwd_workspace_sliced(const cc1d_bwd_params &p) {
    if (bwd_fits_one_launch(p) || p.batch < 2) return bwd_workspace_one_launch(p);
    const int head = p.batch / 2;
    const size_t a = bwd_workspace_sliced(batch_slice(p, 0, head));
    const size_t b = bwd_workspace_sliced(batch_slice(p, head, p.batch - head));
    return a > b ? a : b;
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
        case CC1D_ERR_WORKSPACE_LIMIT: return "backward needs more workspace than the library's built-in array holds; use cc1d_bwd with a caller-owned workspace";
        case CC1D_ERR_IN_PLACE: return "an output shares elements with an input (out with x, dx with x or dout): the kernels do not work in place";
        default: return "unknown cc1d status";
    }
}

int cc1d_hip_runtime_path(char *path, size_t size) {
    if (path == nullptr || size == 0) return CC1D_ERR_NULL_POINTER;
    path[0] = '\0';
    Dl_info info;
    if (dladdr(reinterpret_cast<const void *>(&hipLaunchKernel), &info) == 0 || info.dli_fname == nullptr)
        return CC1D_ERR_LAUNCH;
    const size_t n = std::strlen(info.dli_fname);
    if (n + 1 > size) return CC1D_ERR_SHAPE;
    std::memcpy(path, info.dli_fname, n + 1);
    return CC1D_OK;
}

namespace {
Knob *find_knob(const char *name) {
    Tunables &t = tunables();
    static const struct { const char *name; Knob Tunables::*knob; } table[] = {
        {"fwd_cl_rows", &Tunables::fwd_cl_rows},
        {"fwd_cl_half_vec", &Tunables::fwd_cl_half_vec},
        {"fwd_cl_chunk_runs", &Tunables::fwd_cl_chunk_runs},
        {"bwd_cl_rows", &Tunables::bwd_cl_rows},
        {"bwd_cl_chunk_runs", &Tunables::bwd_cl_chunk_runs},
        {"bwd_cl_lane_bytes", &Tunables::bwd_cl_lane_bytes},
        {"fwd_cf_vecs", &Tunables::fwd_cf_vecs},
        {"bwd_cf_parts", &Tunables::bwd_cf_parts},
        {"launch_limit_shift", &Tunables::launch_limit_shift},
    };
    for (const auto &e : table)
        if (!std::strcmp(name, e.name)) return &(t.*(e.knob));
    return nullptr;
}
}  // namespace

int cc1d_set_tunable(const char *name, int32_t value) {
    if (name == nullptr) return CC1D_ERR_NULL_POINTER;
    Knob *k = find_knob(name);
    if (k == nullptr) return CC1D_ERR_UNKNOWN_TUNABLE;
    k->set(value);
    return CC1D_OK;
}

int cc1d_get_tunable(const char *name, int32_t *value) {
    if (name == nullptr || value == nullptr) return CC1D_ERR_NULL_POINTER;
    const Knob *k = find_knob(name);
    if (k == nullptr) return CC1D_ERR_UNKNOWN_TUNABLE;
    *value = *k;
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
    if (views_share_an_element(p->batch, p->dim, p->seqlen, elem_bytes(p->x_dtype), p->x, p->out, p->x_stride_b,
                               p->x_stride_c, p->x_stride_l, p->out_stride_b, p->out_stride_c, p->out_stride_l))
        return CC1D_ERR_IN_PLACE;
    // initial_states and final_states may be one and the same tensor (csrc/causal_conv1d.h:44 of the
    // reference: a chunked prefill that keeps a single state buffer): same address, same strides.
    // Every kernel reads a row's initial_states and writes its final_states from one wavefront, reads
    // first.  Two different views that share memory have no such guarantee and are refused.
    if (p->initial_states != nullptr && p->final_states != nullptr && p->width > 1) {
        const bool same = p->initial_states == p->final_states && p->init_stride_b == p->final_stride_b &&
                          p->init_stride_c == p->final_stride_c &&
                          (p->width == 2 || p->init_stride_l == p->final_stride_l);
        if (!same && states_overlap(*p)) return CC1D_ERR_STATE_LAYOUT;
    }
    return CC1D_OK;
}

int cc1d_fwd(const cc1d_fwd_params *p, cc1d_stream_t stream) {
    const int st = cc1d_validate_fwd(p);
    if (st != CC1D_OK) return st;
    if (is_empty(p)) return CC1D_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return launch_in_batch_slices(*p, [s](const cc1d_fwd_params &q) {
        return is_channel_last(q.x_stride_c, q.x_stride_l) ? launch_fwd_channellast(q, nullptr, s)
                                                           : launch_fwd_channelfirst(q, s);
    });
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
    if (is_channel_last(fwd->x_stride_c, fwd->x_stride_l) && varlen_fits_fwd_launch(*fwd, *gather)) {
        st = launch_fwd_channellast(*fwd, gather, s);
        if (st != CC1D_ERR_TOO_LARGE) return st;      // too large for one grid: two calls, the forward in slices
    }
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
    const int eb = elem_bytes(p->x_dtype);
    if (views_share_an_element(p->batch, p->dim, p->seqlen, eb, p->x, p->dx, p->x_stride_b, p->x_stride_c, p->x_stride_l,
                               p->dx_stride_b, p->dx_stride_c, p->dx_stride_l) ||
        views_share_an_element(p->batch, p->dim, p->seqlen, eb, p->dout, p->dx, p->dout_stride_b, p->dout_stride_c,
                               p->dout_stride_l, p->dx_stride_b, p->dx_stride_c, p->dx_stride_l))
        return CC1D_ERR_IN_PLACE;
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
    *bytes = bwd_workspace_sliced(*p);
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
    return launch_in_batch_slices(*p, [s, workspace](const cc1d_bwd_params &q) {
        return is_channel_last(q.x_stride_c, q.x_stride_l) ? launch_bwd_channellast(q, workspace, s)
                                                           : launch_bwd_channelfirst(q, workspace, s);
    });
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
    hipStream_t s = static_cast<hipStream_t>(stream);
    return launch_in_batch_slices(*p, [s](const cc1d_update_params &q) { return launch_update(q, s); });
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
