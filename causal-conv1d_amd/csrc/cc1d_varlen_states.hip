// Varlen final-state gather for gfx950, in plain HIP.  Takes over the Triton kernel
// _causal_conv1d_varlen_states and its launch
// (causal_conv1d/causal_conv1d_varlen.py:8-64 of the reference).
//
//   states[b, :, S-k .. S) = x[end_b - k .. end_b, :],  k = min(S, end_b - start_b),
//   states[b, :, 0 .. S-k) = 0.
//
// A pure copy: it moves raw bit patterns and is bit-exact.  Lanes own one 16-byte vector
// of channels of one (sequence, state column) when x and states have unit stride along
// dim; any other strides take the element kernel.  Rows that cu_seqlens would place
// outside [0, total_tokens) are written as zeros instead of being read.
#include "cc1d_varlen_gather.hpp"

namespace cc1d {
namespace {

template <int DT>
__global__ void __launch_bounds__(kBlock)
varlen_states_vec_kernel(const cc1d_varlen_params p, const uint32_t n_colgroups,
                         const uint32_t total) {
    varlen_gather_vec<DT>(p, n_colgroups, total, blockIdx.x * (uint32_t)kBlock + threadIdx.x);
}

template <int DT>
__global__ void __launch_bounds__(kBlock)
varlen_states_elem_kernel(const cc1d_varlen_params p, const uint32_t total) {
    using T = typename Elem<DT>::type;
    const uint32_t gid = blockIdx.x * (uint32_t)kBlock + threadIdx.x;
    if (gid >= total) return;
    const int c = (int)(gid % (uint32_t)p.dim);
    const uint32_t bs = gid / (uint32_t)p.dim;
    const int s = (int)(bs % (uint32_t)p.state_len);
    const int b = (int)(bs / (uint32_t)p.state_len);
    const int64_t row = source_row(p, b, s);
    T v = T(0.f);
    if (row >= 0) v = ld_raw<DT>(p.x, row * p.x_stride_t + (int64_t)c * p.x_stride_c);
    st_raw<DT>(p.states, (int64_t)b * p.states_stride_b + (int64_t)c * p.states_stride_c +
                             (int64_t)s * p.states_stride_l, v);
}

template <int DT>
int launch_dtype(const cc1d_varlen_params &p, bool vec, hipStream_t stream) {
    if (vec) {
        const uint32_t ncg = (uint32_t)(p.dim / Elem<DT>::kVec);
        const int64_t total = (int64_t)p.batch * p.state_len * ncg;
        if (total >= ((int64_t)1 << 31)) return CC1D_ERR_TOO_LARGE;
        CC1D_LAUNCH((varlen_states_vec_kernel<DT>), dim3((uint32_t)((total + kBlock - 1) / kBlock)),
                           dim3(kBlock), 0, stream, p, ncg, (uint32_t)total);
    } else {
        const int64_t total = (int64_t)p.batch * p.state_len * p.dim;
        if (total >= ((int64_t)1 << 31)) return CC1D_ERR_TOO_LARGE;
        CC1D_LAUNCH((varlen_states_elem_kernel<DT>), dim3((uint32_t)((total + kBlock - 1) / kBlock)),
                           dim3(kBlock), 0, stream, p, (uint32_t)total);
    }
    return launch_status();
}

}  // namespace

int launch_varlen_states(const cc1d_varlen_params &p, hipStream_t stream) {
    const bool vec = varlen_vec_ok(p);
    // 2-byte types only differ in how bits are interpreted; the copy treats them alike.
    return p.x_dtype == CC1D_F32 ? launch_dtype<CC1D_F32>(p, vec, stream)
                                 : launch_dtype<CC1D_F16>(p, vec, stream);
}

}  // namespace cc1d
