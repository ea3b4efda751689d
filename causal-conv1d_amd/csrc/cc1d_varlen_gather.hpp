// Device side of the varlen final-state gather, shared by the stand-alone kernel and by the
// channel-last forward, which can run the gather in extra workgroups of its own grid.
//
//   states[b, :, S-k .. S) = x[end_b - k .. end_b, :],  k = min(S, end_b - start_b),
//   states[b, :, 0 .. S-k) = 0      (causal_conv1d/causal_conv1d_varlen.py:8-32 of the reference)
#pragma once
#include "cc1d_device.hpp"
#include "cc1d_internal.hpp"

namespace cc1d {

__device__ __forceinline__ int64_t cu_at(const void *cu, bool is64, int i) {
    return is64 ? reinterpret_cast<const int64_t *>(cu)[i]
                : (int64_t) reinterpret_cast<const int32_t *>(cu)[i];
}

// Source row of state column s of sequence b, or -1 for a zero column.
__device__ __forceinline__ int64_t source_row(const cc1d_varlen_params &p, int b, int s) {
    const bool is64 = p.cu_seqlens_is_int64 != 0;
    const int64_t end = cu_at(p.cu_seqlens, is64, b + 1);
    int64_t start = cu_at(p.cu_seqlens, is64, b);
    if (start < end - p.state_len) start = end - p.state_len;
    const int64_t row = end - (p.state_len - s);
    return (row >= start && row >= 0 && row < p.total_tokens) ? row : -1;
}

// One 16-byte vector of channels of one (sequence, state column) per thread.  DT only sets
// the element size: the copy moves bit patterns.
template <int DT>
__device__ __forceinline__ void varlen_gather_vec(const cc1d_varlen_params &p, uint32_t n_colgroups,
                                                  uint32_t total, uint32_t gid) {
    constexpr int VEC = Elem<DT>::kVec;
    if (gid >= total) return;
    const int c0 = (int)(gid % n_colgroups) * VEC;
    const uint32_t bs = gid / n_colgroups;
    const int s = (int)(bs % (uint32_t)p.state_len);
    const int b = (int)(bs / (uint32_t)p.state_len);
    const int64_t row = source_row(p, b, s);
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row >= 0) v = ld_vec<DT>(p.x, row * p.x_stride_t + c0);
    st_vec<DT>(p.states, (int64_t)b * p.states_stride_b + (int64_t)s * p.states_stride_l + c0, v);
}

// The gather as a tail of another kernel's grid: workgroups first_block, first_block+1, ...
// of that grid run it.  total == 0: no tail.
struct VarlenTail {
    cc1d_varlen_params p;
    uint32_t n_colgroups;
    uint32_t total;           // threads of the gather
    uint32_t first_block;
};

}  // namespace cc1d
