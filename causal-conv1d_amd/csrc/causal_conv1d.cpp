// PyTorch-ROCm binding: the extension module `causal_conv1d_cuda` with the three entry
// points of the reference (csrc/causal_conv1d.cpp:149-157, 260-272, 465-474, 559-563 —
// same names, same positional signatures, same ownership: the caller allocates every
// output) plus `causal_conv1d_varlen_states`, which replaces the Triton launch of
// causal_conv1d/causal_conv1d_varlen.py:35-64.
//
// This file is host-only C++ (built with g++, no device code, no source translation):
// it checks tensors, fills the C-ABI parameter blocks of include/cc1d.h, takes the
// current HIP stream from c10 and calls the kernel library.  The only memory it
// allocates is the backward workspace, through the caching allocator.
#include <torch/extension.h>
#include <torch/library.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <cstdint>
#include <optional>

#include "cc1d.h"

namespace {

#define CHECK_SHAPE(x, ...) \
    TORCH_CHECK(x.sizes() == torch::IntArrayRef({__VA_ARGS__}), #x " must have shape (" #__VA_ARGS__ ")")

int to_cc1d_dtype(at::ScalarType t, const char *what) {
    switch (t) {
        case at::ScalarType::Float: return CC1D_F32;
        case at::ScalarType::Half: return CC1D_F16;
        case at::ScalarType::BFloat16: return CC1D_BF16;
        default: TORCH_CHECK(false, what, " must be float32, float16 or bfloat16, got ", toString(t));
    }
    return -1;
}

// Sizes travel as int32 in the C ABI; strides and offsets are 64-bit.
int32_t size32(int64_t v, const char *what) {
    TORCH_CHECK(v >= 0 && v <= INT32_MAX, what, " = ", v, " does not fit the 32-bit sizes of the kernel library");
    return static_cast<int32_t>(v);
}

void check_status(int st, const char *op) {
    TORCH_CHECK(st == CC1D_OK, op, ": ", cc1d_strerror(st));
}

// The stream the launches go to: torch's current one.  A stream that is being captured into a
// HIP graph is refused.  Nothing on the launch path allocates, clears memory or synchronises the
// host, so capture ought to work, but it is not verified: the two capture runs of these operators
// (a decode loop, and a forward + backward, under torch.cuda.graph on a side stream) ended in a
// segmentation fault on the host whose cause was never established, and an error that says so
// is better than a crash in a serving process.
cc1d_stream_t current_stream() {
    hipStream_t stream = c10::hip::getCurrentHIPStream().stream();
    if (stream != nullptr) {
        hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
        const hipError_t err = hipStreamIsCapturing(stream, &status);
        TORCH_CHECK(err == hipSuccess && status == hipStreamCaptureStatusNone,
                    "causal_conv1d: the current stream is being captured into a HIP graph; graph capture of "
                    "these operators is not verified in this build and is refused");
    }
    return static_cast<cc1d_stream_t>(stream);
}

void check_bias(const std::optional<at::Tensor> &bias_, at::ScalarType weight_type, int64_t dim) {
    if (!bias_.has_value()) return;
    const auto &bias = bias_.value();
    TORCH_CHECK(bias.scalar_type() == weight_type, "bias must have the dtype of weight");
    TORCH_CHECK(bias.is_cuda(), "bias must be on the GPU");
    TORCH_CHECK(bias.stride(-1) == 1, "bias must be contiguous");
    CHECK_SHAPE(bias, dim);
}

cc1d_fwd_params fwd_params(const at::Tensor &x, const at::Tensor &weight,
                       const std::optional<at::Tensor> &bias_,
                       const std::optional<at::Tensor> &seq_idx_,
                       const std::optional<at::Tensor> &initial_states_, at::Tensor &out,
                       std::optional<at::Tensor> &final_states_out_, bool silu_activation) {
    TORCH_CHECK(x.is_cuda() && weight.is_cuda() && out.is_cuda(), "tensors must be on the GPU");
    TORCH_CHECK(x.dim() == 3, "x must be (batch, dim, seqlen)");
    const int64_t batch = x.size(0), dim = x.size(1), seqlen = x.size(2);
    const int64_t width = weight.size(-1);
    CHECK_SHAPE(weight, dim, width);
    CHECK_SHAPE(out, batch, dim, seqlen);
    TORCH_CHECK(out.scalar_type() == x.scalar_type(), "out must have the dtype of x");
    check_bias(bias_, weight.scalar_type(), dim);

    cc1d_fwd_params p = {};
    p.batch = size32(batch, "batch"); p.dim = size32(dim, "dim"); p.seqlen = size32(seqlen, "seqlen");
    p.width = size32(width, "width");
    p.x_dtype = to_cc1d_dtype(x.scalar_type(), "x");
    p.w_dtype = to_cc1d_dtype(weight.scalar_type(), "weight");
    p.silu = silu_activation ? 1 : 0;
    p.x = x.data_ptr();
    p.x_stride_b = x.stride(0); p.x_stride_c = x.stride(1); p.x_stride_l = x.stride(2);
    p.weight = weight.data_ptr();
    p.w_stride_c = weight.stride(0); p.w_stride_w = weight.stride(1);
    p.bias = bias_.has_value() ? bias_.value().data_ptr() : nullptr;
    p.out = out.data_ptr();
    p.out_stride_b = out.stride(0); p.out_stride_c = out.stride(1); p.out_stride_l = out.stride(2);

    if (seq_idx_.has_value()) {
        const auto &seq_idx = seq_idx_.value();
        TORCH_CHECK(seq_idx.scalar_type() == torch::kInt32, "seq_idx must be int32");
        TORCH_CHECK(seq_idx.is_cuda(), "seq_idx must be on the GPU");
        TORCH_CHECK(seq_idx.is_contiguous(), "seq_idx must be contiguous");
        CHECK_SHAPE(seq_idx, batch, seqlen);
        p.seq_idx = seq_idx.data_ptr<int32_t>();
    }
    if (initial_states_.has_value()) {
        const auto &s = initial_states_.value();
        TORCH_CHECK(s.scalar_type() == x.scalar_type(), "initial_states must have the dtype of x");
        TORCH_CHECK(s.is_cuda(), "initial_states must be on the GPU");
        CHECK_SHAPE(s, batch, dim, width - 1);
        p.initial_states = s.data_ptr();
        p.init_stride_b = s.stride(0); p.init_stride_c = s.stride(1); p.init_stride_l = s.stride(2);
    }
    if (final_states_out_.has_value()) {
        auto &s = final_states_out_.value();
        TORCH_CHECK(s.scalar_type() == x.scalar_type(), "final_states must have the dtype of x");
        TORCH_CHECK(s.is_cuda(), "final_states must be on the GPU");
        CHECK_SHAPE(s, batch, dim, width - 1);
        p.final_states = s.data_ptr();
        p.final_stride_b = s.stride(0); p.final_stride_c = s.stride(1); p.final_stride_l = s.stride(2);
    }

    return p;
}

void causal_conv1d_fwd(const at::Tensor &x, const at::Tensor &weight,
                       const std::optional<at::Tensor> &bias_,
                       const std::optional<at::Tensor> &seq_idx_,
                       const std::optional<at::Tensor> &initial_states_, at::Tensor &out,
                       std::optional<at::Tensor> &final_states_out_, bool silu_activation) {
    const cc1d_fwd_params p = fwd_params(x, weight, bias_, seq_idx_, initial_states_, out, final_states_out_,
                                         silu_activation);
    c10::DeviceGuard device_guard(x.device());   // otherwise the launch lands on device 0
    check_status(cc1d_fwd(&p, current_stream()), "causal_conv1d_fwd");
}

// overwrite = false: dweight / dbias are added into, as in the reference; true: they are plain
// outputs and may come in uninitialised.
void bwd_impl(const at::Tensor &x, const at::Tensor &weight,
              const std::optional<at::Tensor> &bias_, at::Tensor &dout,
              const std::optional<at::Tensor> &seq_idx_,
              const std::optional<at::Tensor> &initial_states_,
              const std::optional<at::Tensor> &dfinal_states_, at::Tensor &dx,
              at::Tensor &dweight, std::optional<at::Tensor> &dbias_,
              std::optional<at::Tensor> &dinitial_states_, bool silu_activation, bool overwrite) {
    TORCH_CHECK(x.is_cuda() && weight.is_cuda() && dout.is_cuda() && dx.is_cuda() && dweight.is_cuda(),
                "tensors must be on the GPU");
    TORCH_CHECK(bias_.has_value() == dbias_.has_value(), "bias and dbias must be given together");
    TORCH_CHECK(x.dim() == 3, "x must be (batch, dim, seqlen)");
    const int64_t batch = x.size(0), dim = x.size(1), seqlen = x.size(2);
    const int64_t width = weight.size(-1);
    CHECK_SHAPE(weight, dim, width);
    CHECK_SHAPE(dout, batch, dim, seqlen);
    CHECK_SHAPE(dx, batch, dim, seqlen);
    CHECK_SHAPE(dweight, dim, width);
    TORCH_CHECK(dout.scalar_type() == x.scalar_type(), "dout must have the dtype of x");
    TORCH_CHECK(dx.scalar_type() == x.scalar_type(), "dx must have the dtype of x");
    TORCH_CHECK(dweight.scalar_type() == at::ScalarType::Float, "dweight must be float32");
    check_bias(bias_, weight.scalar_type(), dim);

    // dout follows x's layout family; re-lay it out when autograd hands over another one
    // (the reference does the same, csrc/causal_conv1d.cpp:297-298).
    TORCH_CHECK(x.stride(2) == 1 || x.stride(1) == 1, "x must have stride 1 along dim or along seqlen");
    const bool channel_last = x.stride(1) == 1 && x.stride(2) > 1;
    if (!channel_last && dout.stride(2) != 1) dout = dout.contiguous();
    if (channel_last && dout.stride(1) != 1) dout = dout.transpose(-1, -2).contiguous().transpose(-1, -2);

    cc1d_bwd_params p = {};
    p.batch = size32(batch, "batch"); p.dim = size32(dim, "dim"); p.seqlen = size32(seqlen, "seqlen");
    p.width = size32(width, "width");
    p.x_dtype = to_cc1d_dtype(x.scalar_type(), "x");
    p.w_dtype = to_cc1d_dtype(weight.scalar_type(), "weight");
    p.silu = silu_activation ? 1 : 0;
    p.overwrite_dweight = overwrite ? 1 : 0;
    p.x = x.data_ptr();
    p.x_stride_b = x.stride(0); p.x_stride_c = x.stride(1); p.x_stride_l = x.stride(2);
    p.weight = weight.data_ptr();
    p.w_stride_c = weight.stride(0); p.w_stride_w = weight.stride(1);
    p.bias = bias_.has_value() ? bias_.value().data_ptr() : nullptr;
    p.dout = dout.data_ptr();
    p.dout_stride_b = dout.stride(0); p.dout_stride_c = dout.stride(1); p.dout_stride_l = dout.stride(2);
    p.dx = dx.data_ptr();
    p.dx_stride_b = dx.stride(0); p.dx_stride_c = dx.stride(1); p.dx_stride_l = dx.stride(2);
    p.dweight = dweight.data_ptr<float>();
    p.dw_stride_c = dweight.stride(0); p.dw_stride_w = dweight.stride(1);
    if (dbias_.has_value()) {
        auto &dbias = dbias_.value();
        TORCH_CHECK(dbias.scalar_type() == at::ScalarType::Float, "dbias must be float32");
        TORCH_CHECK(dbias.is_cuda() && dbias.stride(-1) == 1, "dbias must be a contiguous GPU tensor");
        CHECK_SHAPE(dbias, dim);
        p.dbias = dbias.data_ptr<float>();
    }
    if (seq_idx_.has_value()) {
        const auto &seq_idx = seq_idx_.value();
        TORCH_CHECK(seq_idx.scalar_type() == torch::kInt32, "seq_idx must be int32");
        TORCH_CHECK(seq_idx.is_cuda(), "seq_idx must be on the GPU");
        TORCH_CHECK(seq_idx.is_contiguous(), "seq_idx must be contiguous");
        CHECK_SHAPE(seq_idx, batch, seqlen);
        p.seq_idx = seq_idx.data_ptr<int32_t>();
    }
    if (initial_states_.has_value()) {
        const auto &s = initial_states_.value();
        TORCH_CHECK(s.scalar_type() == x.scalar_type(), "initial_states must have the dtype of x");
        TORCH_CHECK(s.is_cuda(), "initial_states must be on the GPU");
        CHECK_SHAPE(s, batch, dim, width - 1);
        p.initial_states = s.data_ptr();
        p.init_stride_b = s.stride(0); p.init_stride_c = s.stride(1); p.init_stride_l = s.stride(2);
    }
    if (dfinal_states_.has_value()) {
        const auto &s = dfinal_states_.value();
        TORCH_CHECK(s.scalar_type() == x.scalar_type(), "dfinal_states must have the dtype of x");
        TORCH_CHECK(s.is_cuda(), "dfinal_states must be on the GPU");
        CHECK_SHAPE(s, batch, dim, width - 1);
        p.dfinal_states = s.data_ptr();
        p.dfinal_stride_b = s.stride(0); p.dfinal_stride_c = s.stride(1); p.dfinal_stride_l = s.stride(2);
    }
    if (dinitial_states_.has_value()) {
        auto &s = dinitial_states_.value();
        TORCH_CHECK(s.scalar_type() == x.scalar_type(), "dinitial_states must have the dtype of x");
        TORCH_CHECK(s.is_cuda(), "dinitial_states must be on the GPU");
        CHECK_SHAPE(s, batch, dim, width - 1);
        p.dinitial_states = s.data_ptr();
        p.dinit_stride_b = s.stride(0); p.dinit_stride_c = s.stride(1); p.dinit_stride_l = s.stride(2);
    }

    c10::DeviceGuard device_guard(x.device());
    size_t ws_bytes = 0;
    check_status(cc1d_bwd_workspace_bytes(&p, &ws_bytes), "causal_conv1d_bwd");
    at::Tensor workspace;
    void *ws_ptr = nullptr;
    if (ws_bytes > 0) {
        workspace = at::empty({(int64_t)ws_bytes}, at::TensorOptions().dtype(at::kByte).device(x.device()));
        ws_ptr = workspace.data_ptr();
    }
    check_status(cc1d_bwd(&p, ws_ptr, ws_bytes, current_stream()), "causal_conv1d_bwd");
}

void causal_conv1d_bwd(const at::Tensor &x, const at::Tensor &weight,
                       const std::optional<at::Tensor> &bias_, at::Tensor &dout,
                       const std::optional<at::Tensor> &seq_idx_,
                       const std::optional<at::Tensor> &initial_states_,
                       const std::optional<at::Tensor> &dfinal_states_, at::Tensor &dx,
                       at::Tensor &dweight, std::optional<at::Tensor> &dbias_,
                       std::optional<at::Tensor> &dinitial_states_, bool silu_activation) {
    bwd_impl(x, weight, bias_, dout, seq_idx_, initial_states_, dfinal_states_, dx, dweight, dbias_,
             dinitial_states_, silu_activation, false);
}

void causal_conv1d_update(const at::Tensor &x, const at::Tensor &conv_state, const at::Tensor &weight,
                          const std::optional<at::Tensor> &bias_, at::Tensor &out,
                          bool silu_activation, const std::optional<at::Tensor> &cache_seqlens_,
                          const std::optional<at::Tensor> &conv_state_indices_) {
    TORCH_CHECK(x.is_cuda() && conv_state.is_cuda() && weight.is_cuda() && out.is_cuda(),
                "tensors must be on the GPU");
    TORCH_CHECK(conv_state.scalar_type() == x.scalar_type(), "conv_state must have the dtype of x");
    TORCH_CHECK(out.scalar_type() == x.scalar_type(), "out must have the dtype of x");
    // x and out may also be (batch, dim): one token, no seqlen axis.
    const bool flat = x.dim() == 2;
    TORCH_CHECK(flat || x.dim() == 3, "x must be (batch, dim, seqlen)");
    TORCH_CHECK(conv_state.dim() == 3, "conv_state must be (batch, dim, state_len)");
    const int64_t batch = x.size(0), dim = x.size(1), seqlen = flat ? 1 : x.size(2);
    const int64_t width = weight.size(-1);
    const int64_t state_len = conv_state.size(2);
    TORCH_CHECK(state_len >= width - 1, "conv_state length must be at least width - 1");
    CHECK_SHAPE(weight, dim, width);
    if (flat) {
        CHECK_SHAPE(out, batch, dim);
    } else {
        CHECK_SHAPE(out, batch, dim, seqlen);
    }
    check_bias(bias_, weight.scalar_type(), dim);

    cc1d_update_params p = {};
    p.batch = size32(batch, "batch"); p.dim = size32(dim, "dim"); p.seqlen = size32(seqlen, "seqlen");
    p.width = size32(width, "width");
    p.state_len = size32(state_len, "state_len");
    p.state_batch = size32(conv_state.size(0), "conv_state batch");
    p.x_dtype = to_cc1d_dtype(x.scalar_type(), "x");
    p.w_dtype = to_cc1d_dtype(weight.scalar_type(), "weight");
    p.silu = silu_activation ? 1 : 0;
    p.x = x.data_ptr();
    p.x_stride_b = x.stride(0); p.x_stride_c = x.stride(1); p.x_stride_l = flat ? dim : x.stride(2);
    p.conv_state = conv_state.data_ptr();
    p.state_stride_b = conv_state.stride(0); p.state_stride_c = conv_state.stride(1);
    p.state_stride_l = conv_state.stride(2);
    p.weight = weight.data_ptr();
    p.w_stride_c = weight.stride(0); p.w_stride_w = weight.stride(1);
    p.bias = bias_.has_value() ? bias_.value().data_ptr() : nullptr;
    p.out = out.data_ptr();
    p.out_stride_b = out.stride(0); p.out_stride_c = out.stride(1); p.out_stride_l = flat ? dim : out.stride(2);

    if (conv_state_indices_.has_value()) {
        const auto &idx = conv_state_indices_.value();
        TORCH_CHECK(idx.scalar_type() == torch::kInt32, "conv_state_indices must be int32");
        TORCH_CHECK(idx.is_cuda(), "conv_state_indices must be on the GPU");
        TORCH_CHECK(idx.stride(0) == 1, "conv_state_indices must be contiguous");
        CHECK_SHAPE(idx, batch);
        CHECK_SHAPE(conv_state, conv_state.size(0), dim, state_len);
        p.conv_state_indices = idx.data_ptr<int32_t>();
    } else {
        CHECK_SHAPE(conv_state, batch, dim, state_len);
    }
    if (cache_seqlens_.has_value()) {
        const auto &cs = cache_seqlens_.value();
        TORCH_CHECK(cs.scalar_type() == torch::kInt32, "cache_seqlens must be int32");
        TORCH_CHECK(cs.is_cuda(), "cache_seqlens must be on the GPU");
        TORCH_CHECK(cs.stride(-1) == 1, "cache_seqlens must be contiguous");
        CHECK_SHAPE(cs, batch);
        p.cache_seqlens = cs.data_ptr<int32_t>();
    }

    c10::DeviceGuard device_guard(x.device());
    check_status(cc1d_update(&p, current_stream()), "causal_conv1d_update");
}

cc1d_varlen_params varlen_params(const at::Tensor &x, const at::Tensor &cu_seqlens, at::Tensor &states,
                                 int64_t state_len) {
    TORCH_CHECK(x.is_cuda() && cu_seqlens.is_cuda() && states.is_cuda(), "tensors must be on the GPU");
    TORCH_CHECK(x.dim() == 2, "x must be (total_tokens, dim)");
    TORCH_CHECK(cu_seqlens.dim() == 1 && cu_seqlens.size(0) >= 1, "cu_seqlens must be (batch + 1,)");
    TORCH_CHECK(cu_seqlens.is_contiguous(), "cu_seqlens must be contiguous");
    TORCH_CHECK(cu_seqlens.scalar_type() == torch::kInt32 || cu_seqlens.scalar_type() == torch::kInt64,
                "cu_seqlens must be int32 or int64");
    TORCH_CHECK(states.scalar_type() == x.scalar_type(), "states must have the dtype of x");
    const int64_t dim = x.size(1), batch = cu_seqlens.size(0) - 1;
    CHECK_SHAPE(states, batch, dim, state_len);

    cc1d_varlen_params p = {};
    p.batch = size32(batch, "batch"); p.dim = size32(dim, "dim"); p.state_len = size32(state_len, "state_len");
    p.x_dtype = to_cc1d_dtype(x.scalar_type(), "x");
    p.cu_seqlens_is_int64 = cu_seqlens.scalar_type() == torch::kInt64 ? 1 : 0;
    p.total_tokens = x.size(0);
    p.x = x.data_ptr();
    p.x_stride_t = x.stride(0); p.x_stride_c = x.stride(1);
    p.cu_seqlens = cu_seqlens.data_ptr();
    p.states = states.data_ptr();
    p.states_stride_b = states.stride(0); p.states_stride_c = states.stride(1);
    p.states_stride_l = states.stride(2);

    return p;
}

void causal_conv1d_varlen_states(const at::Tensor &x, const at::Tensor &cu_seqlens, at::Tensor &states,
                                 int64_t state_len) {
    const cc1d_varlen_params p = varlen_params(x, cu_seqlens, states, state_len);
    c10::DeviceGuard device_guard(x.device());
    check_status(cc1d_varlen_states(&p, current_stream()), "causal_conv1d_varlen_states");
}

// Forward over a packed batch and the gather of every sequence's last state_len tokens from
// `tokens` (total_tokens, dim), normally a view of x: one call, and one kernel launch when x is
// channel-last.  What causal_conv1d_fwd followed by causal_conv1d_varlen_states would give.
void causal_conv1d_fwd_varlen_states(const at::Tensor &x, const at::Tensor &weight,
                                     const std::optional<at::Tensor> &bias_,
                                     const std::optional<at::Tensor> &seq_idx_, at::Tensor &out,
                                     const at::Tensor &tokens, const at::Tensor &cu_seqlens,
                                     at::Tensor &states, int64_t state_len, bool silu_activation) {
    std::optional<at::Tensor> none;
    const cc1d_fwd_params f = fwd_params(x, weight, bias_, seq_idx_, none, out, none, silu_activation);
    const cc1d_varlen_params v = varlen_params(tokens, cu_seqlens, states, state_len);
    TORCH_CHECK(tokens.device() == x.device(), "tokens must be on the device of x");
    c10::DeviceGuard device_guard(x.device());
    check_status(cc1d_fwd_varlen_states(&f, &v, current_stream()), "causal_conv1d_fwd_varlen_states");
}

// ---- dispatcher entry points -------------------------------------------------------
// The same three operators as torch.library ops, registered from C++ so that a call from
// Python goes dispatcher -> kernel without a Python trampoline in between (a Python-defined
// custom op costs about 8 us of host time per call, more than the decode kernel itself).
// Names, argument order and the set of written arguments are those of
// causal_conv1d/cpp_functions.py:11-91 of the reference.

void fwd_op(const at::Tensor &x, const at::Tensor &weight, const std::optional<at::Tensor> &bias,
            const std::optional<at::Tensor> &seq_idx, const std::optional<at::Tensor> &initial_states,
            at::Tensor &out, const std::optional<at::Tensor> &final_states_out, bool silu_activation) {
    std::optional<at::Tensor> fin = final_states_out;
    causal_conv1d_fwd(x, weight, bias, seq_idx, initial_states, out, fin, silu_activation);
}

// The forward with its result allocated here, in x's layout: one dispatcher hop and no
// empty_like in Python (about a microsecond of host time, which is what a short prefill is
// bound by).  Not an op of the reference.
at::Tensor fwd_out_op(const at::Tensor &x, const at::Tensor &weight, const std::optional<at::Tensor> &bias,
                      const std::optional<at::Tensor> &seq_idx, const std::optional<at::Tensor> &initial_states,
                      const std::optional<at::Tensor> &final_states_out, bool silu_activation) {
    at::Tensor out = at::empty_like(x);
    std::optional<at::Tensor> fin = final_states_out;
    causal_conv1d_fwd(x, weight, bias, seq_idx, initial_states, out, fin, silu_activation);
    return out;
}
at::Tensor fwd_out_meta(const at::Tensor &x, const at::Tensor &, const std::optional<at::Tensor> &,
                        const std::optional<at::Tensor> &, const std::optional<at::Tensor> &,
                        const std::optional<at::Tensor> &, bool) {
    return at::empty_like(x);
}

void bwd_op(const at::Tensor &x, const at::Tensor &weight, const std::optional<at::Tensor> &bias,
            const at::Tensor &dout, const std::optional<at::Tensor> &seq_idx,
            const std::optional<at::Tensor> &initial_states, const std::optional<at::Tensor> &dfinal_states,
            at::Tensor &dx, at::Tensor &dweight, const std::optional<at::Tensor> &dbias,
            const std::optional<at::Tensor> &dinitial_states, bool silu_activation) {
    at::Tensor dout_ = dout;
    std::optional<at::Tensor> db = dbias, dinit = dinitial_states;
    causal_conv1d_bwd(x, weight, bias, dout_, seq_idx, initial_states, dfinal_states, dx, dweight, db, dinit,
                      silu_activation);
}

// The backward with dweight / dbias as plain outputs (no zero-fill before the call): what the
// autograd function of this package uses.  Not an op of the reference.
void bwd_overwrite_op(const at::Tensor &x, const at::Tensor &weight, const std::optional<at::Tensor> &bias,
                      const at::Tensor &dout, const std::optional<at::Tensor> &seq_idx,
                      const std::optional<at::Tensor> &initial_states,
                      const std::optional<at::Tensor> &dfinal_states, at::Tensor &dx, at::Tensor &dweight,
                      const std::optional<at::Tensor> &dbias, const std::optional<at::Tensor> &dinitial_states,
                      bool silu_activation) {
    at::Tensor dout_ = dout;
    std::optional<at::Tensor> db = dbias, dinit = dinitial_states;
    bwd_impl(x, weight, bias, dout_, seq_idx, initial_states, dfinal_states, dx, dweight, db, dinit,
             silu_activation, true);
}

void update_op(const at::Tensor &x, at::Tensor &conv_state, const at::Tensor &weight,
               const std::optional<at::Tensor> &bias, at::Tensor &out, bool silu_activation,
               const std::optional<at::Tensor> &cache_seqlens, const std::optional<at::Tensor> &conv_state_indices) {
    causal_conv1d_update(x, conv_state, weight, bias, out, silu_activation, cache_seqlens, conv_state_indices);
}

// The decode step as the user-facing function needs it: x (batch, dim) or (batch, dim, seqlen),
// the result allocated here and shaped like x.  One dispatcher hop instead of the wrapper's
// unsqueeze / empty_like / op / squeeze in Python, which cost more host time than the kernel
// runs.  Not an op of the reference.
at::Tensor update_out_op(const at::Tensor &x, at::Tensor &conv_state, const at::Tensor &weight,
                         const std::optional<at::Tensor> &bias, bool silu_activation,
                         const std::optional<at::Tensor> &cache_seqlens,
                         const std::optional<at::Tensor> &conv_state_indices) {
    TORCH_CHECK(x.dim() == 2 || x.dim() == 3, "x must be (batch, dim) or (batch, dim, seqlen)");
    at::Tensor out = at::empty_like(x);
    causal_conv1d_update(x, conv_state, weight, bias, out, silu_activation, cache_seqlens, conv_state_indices);
    return out;
}
at::Tensor update_out_meta(const at::Tensor &x, at::Tensor &, const at::Tensor &, const std::optional<at::Tensor> &,
                           bool, const std::optional<at::Tensor> &, const std::optional<at::Tensor> &) {
    return at::empty_like(x);
}

// Shape propagation has nothing to do: every output is an argument.
void fwd_meta(const at::Tensor &, const at::Tensor &, const std::optional<at::Tensor> &,
              const std::optional<at::Tensor> &, const std::optional<at::Tensor> &, at::Tensor &,
              const std::optional<at::Tensor> &, bool) {}
void bwd_meta(const at::Tensor &, const at::Tensor &, const std::optional<at::Tensor> &, const at::Tensor &,
              const std::optional<at::Tensor> &, const std::optional<at::Tensor> &,
              const std::optional<at::Tensor> &, at::Tensor &, at::Tensor &, const std::optional<at::Tensor> &,
              const std::optional<at::Tensor> &, bool) {}
void update_meta(const at::Tensor &, at::Tensor &, const at::Tensor &, const std::optional<at::Tensor> &,
                 at::Tensor &, bool, const std::optional<at::Tensor> &, const std::optional<at::Tensor> &) {}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("causal_conv1d_fwd", &causal_conv1d_fwd, "Causal conv1d forward");
    m.def("causal_conv1d_bwd", &causal_conv1d_bwd, "Causal conv1d backward");
    m.def("causal_conv1d_update", &causal_conv1d_update, "Causal conv1d update");
    m.def("causal_conv1d_varlen_states", &causal_conv1d_varlen_states, "Varlen final-state gather");
    m.def("causal_conv1d_fwd_varlen_states", &causal_conv1d_fwd_varlen_states,
          "Causal conv1d forward and varlen final-state gather in one call");
}

TORCH_LIBRARY_FRAGMENT(DaoAILab, m) {
    m.def("_causal_conv1d_fwd_cpp(Tensor x, Tensor weight, Tensor? bias, Tensor? seq_idx, "
          "Tensor? initial_states, Tensor(a!) out, Tensor(b!)? final_states_out, bool silu_activation) -> ()",
          {at::Tag::pt2_compliant_tag});
    m.def("_causal_conv1d_fwd_out_cpp(Tensor x, Tensor weight, Tensor? bias, Tensor? seq_idx, "
          "Tensor? initial_states, Tensor(a!)? final_states_out, bool silu_activation) -> Tensor",
          {at::Tag::pt2_compliant_tag});
    m.def("_causal_conv1d_bwd_cpp(Tensor x, Tensor weight, Tensor? bias, Tensor dout, Tensor? seq_idx, "
          "Tensor? initial_states, Tensor(a!)? dfinal_states, Tensor(b!) dx, Tensor(c!) dweight, "
          "Tensor(d!)? dbias, Tensor(e!)? dinitial_states, bool silu_activation) -> ()",
          {at::Tag::pt2_compliant_tag});
    m.def("_causal_conv1d_bwd_overwrite_cpp(Tensor x, Tensor weight, Tensor? bias, Tensor dout, Tensor? seq_idx, "
          "Tensor? initial_states, Tensor(a!)? dfinal_states, Tensor(b!) dx, Tensor(c!) dweight, "
          "Tensor(d!)? dbias, Tensor(e!)? dinitial_states, bool silu_activation) -> ()",
          {at::Tag::pt2_compliant_tag});
    m.def("_causal_conv1d_update_out_cpp(Tensor x, Tensor(a!) conv_state, Tensor weight, Tensor? bias, "
          "bool silu_activation, Tensor? cache_seqlens, Tensor? conv_state_indices) -> Tensor",
          {at::Tag::pt2_compliant_tag});
    m.def("_causal_conv1d_update_cpp(Tensor x, Tensor(a!) conv_state, Tensor weight, Tensor? bias, "
          "Tensor(b!) out, bool silu_activation, Tensor? cache_seqlens, Tensor? conv_state_indices) -> ()",
          {at::Tag::pt2_compliant_tag});
}

// One kernel for every real backend: on anything but the GPU it raises (there is no host path).
TORCH_LIBRARY_IMPL(DaoAILab, CompositeExplicitAutograd, m) {
    m.impl("_causal_conv1d_fwd_cpp", &fwd_op);
    m.impl("_causal_conv1d_fwd_out_cpp", &fwd_out_op);
    m.impl("_causal_conv1d_bwd_cpp", &bwd_op);
    m.impl("_causal_conv1d_bwd_overwrite_cpp", &bwd_overwrite_op);
    m.impl("_causal_conv1d_update_cpp", &update_op);
    m.impl("_causal_conv1d_update_out_cpp", &update_out_op);
}

TORCH_LIBRARY_IMPL(DaoAILab, Meta, m) {
    m.impl("_causal_conv1d_fwd_cpp", &fwd_meta);
    m.impl("_causal_conv1d_fwd_out_cpp", &fwd_out_meta);
    m.impl("_causal_conv1d_bwd_cpp", &bwd_meta);
    m.impl("_causal_conv1d_bwd_overwrite_cpp", &bwd_meta);
    m.impl("_causal_conv1d_update_cpp", &update_meta);
    m.impl("_causal_conv1d_update_out_cpp", &update_out_meta);
}
