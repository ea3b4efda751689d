// Host-side contracts between the C-ABI front (cc1d_api.cpp) and the kernel launchers
// (one .hip file per kernel family).  A launcher is only called with parameters that
// passed the matching cc1d_validate_*; it picks the template instance, sizes the grid
// and returns a cc1d_status.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>

#include "cc1d.h"

namespace cc1d {

inline int elem_bytes(int dtype) { return dtype == CC1D_F32 ? 4 : 2; }
inline int vec_elems(int dtype) { return 16 / elem_bytes(dtype); }

// x is channel-last iff stride 1 along dim and stride > 1 along seqlen
// (csrc/causal_conv1d.cpp:176 of the reference).
inline bool is_channel_last(int64_t stride_c, int64_t stride_l) {
    return stride_c == 1 && stride_l > 1;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// weight is fp32, densely packed (dim, width) and 16-byte aligned: lanes may fetch
// their channels' taps as whole vectors.
inline bool weights_contiguous_f32(const void *w, int w_dtype, int64_t sc, int64_t sw, int width) {
    return w_dtype == CC1D_F32 && sw == 1 && sc == width && aligned16(w);
}

// How the fast kernels may read the taps: 1 = packed (dim, width) fp32, 2 = packed in x's own
// 16-bit type (weight and bias 16-byte aligned, whole vectors per lane, PackedTaps on the
// device); 0 = anything else (general loader).
inline int weights_mode(const void *w, const void *bias, int w_dtype, int x_dtype, int64_t sc, int64_t sw, int width) {
    if (!(sw == 1 && sc == width && aligned16(w) && aligned16(bias))) return 0;
    if (w_dtype == CC1D_F32) return 1;
    return w_dtype == x_dtype ? 2 : 0;
}

// Varlen gather: x and states have unit stride along dim and every vector is 16-byte aligned.
inline bool varlen_vec_ok(const cc1d_varlen_params &p) {
    const int v = vec_elems(p.x_dtype);
    return p.dim % v == 0 && p.x_stride_c == 1 && p.x_stride_t % v == 0 && aligned16(p.x) &&
           p.states_stride_c == 1 && p.states_stride_b % v == 0 &&
           (p.state_len <= 1 || p.states_stride_l % v == 0) && aligned16(p.states);
}

// The gather can ride in the channel-last forward's launch: vector copies of elements as
// wide as the forward's.
inline bool varlen_fits_fwd_launch(const cc1d_fwd_params &f, const cc1d_varlen_params &v) {
    return varlen_vec_ok(v) && elem_bytes(v.x_dtype) == elem_bytes(f.x_dtype);
}

// Launch-heuristic overrides for sweeps and for the tests that prove results do not depend on
// launch geometry.  0 = the built-in choice.  Each knob is an independent relaxed atomic: a
// launch reads it once, a concurrent cc1d_set_tunable from another thread is a data-race-free
// store, and no knob changes what a launch computes, only how it is cut into workgroups.
struct Knob {
    std::atomic<int32_t> v{0};
    operator int32_t() const { return v.load(std::memory_order_relaxed); }
    void set(int32_t x) { v.store(x, std::memory_order_relaxed); }
};
struct Tunables {
    Knob fwd_cl_rows, fwd_cl_half_vec, fwd_cl_chunk_runs, bwd_cl_rows, bwd_cl_chunk_runs, bwd_cl_lane_bytes,
        fwd_cf_vecs, bwd_cf_parts, launch_limit_shift;
};
Tunables &tunables();

// The kernels number their work items with 32 bits, so one launch holds fewer than 2^31 threads
// (2^25 wavefronts).  A launcher whose problem needs more returns CC1D_ERR_TOO_LARGE before it
// launches anything, and the C-ABI front then cuts the batch into slices that fit.  The knob
// lowers the limit (by that many bits) so that tests reach the slicing with small tensors.
inline int64_t thread_limit() {
    const int32_t shift = tunables().launch_limit_shift;
    return ((int64_t)1 << 31) >> (shift > 0 && shift <= 24 ? shift : 0);
}
inline int64_t wave_limit() { return thread_limit() / 64; }

// Probe mode, per host thread: a launcher called in it does everything it does before a launch
// (layout choice, geometry, the checks that answer CC1D_ERR_TOO_LARGE) and launches nothing.  The
// C-ABI front uses it to learn whether the smallest batch slice of a problem fits one grid before
// the first slice is launched.
inline thread_local bool g_probe_only = false;
inline bool probe_only() { return g_probe_only; }
struct ProbeScope {
    ProbeScope() { g_probe_only = true; }
    ~ProbeScope() { g_probe_only = false; }
};
#define CC1D_LAUNCH(...)                                            \
    do {                                                            \
        if (!::cc1d::probe_only()) hipLaunchKernelGGL(__VA_ARGS__); \
    } while (0)

inline int launch_status() {
    if (probe_only()) return CC1D_OK;
    return hipGetLastError() == hipSuccess ? CC1D_OK : CC1D_ERR_LAUNCH;
}

int launch_fwd_channellast(const cc1d_fwd_params &p, const cc1d_varlen_params *gather, hipStream_t stream);
int launch_fwd_channelfirst(const cc1d_fwd_params &p, hipStream_t stream);
// Channel-first rows of whole vectors on the 16-byte grid: the tile kernel (cc1d_fwd_channelfirst_tile.hip).
bool fwd_channelfirst_tile_applies(const cc1d_fwd_params &p);
int launch_fwd_channelfirst_tile(const cc1d_fwd_params &p, hipStream_t stream);

size_t bwd_channellast_workspace_bytes(const cc1d_bwd_params &p);
size_t bwd_channelfirst_workspace_bytes(const cc1d_bwd_params &p);
// false: the launcher would answer CC1D_ERR_TOO_LARGE (and launch nothing).
bool bwd_channellast_fits(const cc1d_bwd_params &p);
bool bwd_channelfirst_fits(const cc1d_bwd_params &p);
// Channel-first rows of more than 64 vectors: the tile kernel (cc1d_bwd_channelfirst_tile.hip);
// its workspace is `parts` planes of (width + 1) x dim floats.
bool bwd_channelfirst_tile_applies(const cc1d_bwd_params &p);
bool bwd_channelfirst_tile_fits(const cc1d_bwd_params &p);
int bwd_channelfirst_tile_parts(const cc1d_bwd_params &p);
int launch_bwd_channelfirst_tile(const cc1d_bwd_params &p, float *ws, hipStream_t stream);
int launch_bwd_channellast(const cc1d_bwd_params &p, void *ws, hipStream_t stream);
int launch_bwd_channelfirst(const cc1d_bwd_params &p, void *ws, hipStream_t stream);
// Second stage of both backward layouts: ordered sum of the workspace planes into dweight/dbias.
int launch_bwd_finalize(const float *ws, int n_parts, const cc1d_bwd_params &p, hipStream_t stream);

int launch_update(const cc1d_update_params &p, hipStream_t stream);
int launch_varlen_states(const cc1d_varlen_params &p, hipStream_t stream);

}  // namespace cc1d
