// Decode-step update for gfx950.  Takes over causal_conv1d_update_kernel and its
// launcher (csrc/causal_conv1d_update.cu:23-136 of the reference).
//
// Two kernels:
//  * update_vec_kernel — x, out and conv_state all have unit stride along dim (the
//    layout Mamba-style decoders allocate: (batch, state_len, dim) in memory).  A lane
//    owns one 16-byte vector of channels; every state row, x row and out row moves as
//    one coalesced 16-byte access (the reference moves 2 bytes per lane per access).
//  * update_generic_kernel — any strides, one lane per (batch, channel), element access.
//
// State movement is done on the raw bit patterns, so conv_state is bit-exact.
//
// Linear variant (cache_seqlens == NULL), state_len S, step count L, window W-1:
//   new_state = concat(state, x)[-S:]; the last W-1 entries of that are exactly the
//   sliding window after L steps, the S-(W-1) entries before them are a forward shift
//   (reads always run ahead of writes, so the shift is safe in place).
// Circular variant: window = state[(cs-(W-1)+i) mod S], x[i] is written at (cs+i) mod S,
//   cs = cache_seqlens[b] mod S.
#include "cc1d_device.hpp"
#include "cc1d_internal.hpp"

namespace cc1d {
namespace {

__device__ __forceinline__ int wrap(int v, int n) {   // v in (-n, 2n) -> [0, n)
    v = v < 0 ? v + n : v;
    return v >= n ? v - n : v;
}
__device__ __forceinline__ int positive_mod(int v, int n) {
    const int r = v % n;
    return r < 0 ? r + n : r;
}

template <int DT, int W, bool CIRC>
__global__ void __launch_bounds__(kBlock)
update_vec_kernel(const cc1d_update_params p, const uint32_t n_colgroups, const uint32_t total,
                  const int w_fast) {
    using E = Elem<DT>;
    constexpr int VEC = E::kVec;
    constexpr bool PRECISE = E::kPreciseAct;

    const uint32_t gid = blockIdx.x * (uint32_t)kBlock + threadIdx.x;
    if (gid >= total) return;
    const int c0 = (int)(gid % n_colgroups) * VEC;
    const int b = (int)(gid / n_colgroups);
    const int L = p.seqlen;
    const int S = p.state_len;
    const bool silu_on = p.silu != 0;

    const int64_t xoff = (int64_t)b * p.x_stride_b + c0;
    const int64_t ooff = (int64_t)b * p.out_stride_b + c0;

    const int sb = p.conv_state_indices == nullptr ? b : p.conv_state_indices[b];
    if (sb < 0) {                                     // padding slot: zeros out, state untouched
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int i = 0; i < L; ++i) st_vec<DT>(p.out, ooff + (int64_t)i * p.out_stride_l, z);
        return;
    }
    const int64_t soff = (int64_t)sb * p.state_stride_b + c0;

    // Issue every independent load up front: window rows, first x row, then weights.
    u32x4 rw[W - 1];
    int cs = 0;
    if (CIRC) cs = positive_mod(p.cache_seqlens[b], S);
#pragma unroll
    for (int i = 0; i < W - 1; ++i) {
        const int l = CIRC ? wrap(cs - (W - 1) + i, S) : S - (W - 1) + i;
        rw[i] = ld_vec<DT>(p.conv_state, soff + (int64_t)l * p.state_stride_l);
    }
    u32x4 xr = ld_vec<DT>(p.x, xoff);                 // row 0 (L >= 1)

    float wv[VEC][W], bv[VEC];
    load_weights<W, VEC>(p.weight, p.bias, p.w_dtype, p.w_stride_c, p.w_stride_w, w_fast != 0, c0,
                         wv, bv);

    if (!CIRC) {
        // Entries in front of the window: new_state[j] = concat(state, x)[L + j].
        for (int j = 0; j < S - (W - 1); ++j) {
            const int src = L + j;
            const u32x4 v = src < S
                ? ld_vec<DT>(p.conv_state, soff + (int64_t)src * p.state_stride_l)
                : ld_vec<DT>(p.x, xoff + (int64_t)(src - S) * p.x_stride_l);
            st_vec<DT>(p.conv_state, soff + (int64_t)j * p.state_stride_l, v);
        }
    }

    float xw[W - 1][VEC];
#pragma unroll
    for (int i = 0; i < W - 1; ++i) E::unpack(rw[i], xw[i]);

    int wpos = cs;                                    // circular write position
    for (int i = 0; i < L; ++i) {
        if (i > 0) xr = ld_vec<DT>(p.x, xoff + (int64_t)i * p.x_stride_l);
        if (CIRC) {
            st_vec<DT>(p.conv_state, soff + (int64_t)wpos * p.state_stride_l, xr);
            wpos = wpos + 1 == S ? 0 : wpos + 1;
        }
        float xv[VEC], acc[VEC];
        E::unpack(xr, xv);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            float a = bv[j];
#pragma unroll
            for (int k = 0; k < W - 1; ++k) a = fmaf(wv[j][k], xw[k][j], a);
            a = fmaf(wv[j][W - 1], xv[j], a);
            acc[j] = silu_on ? silu<PRECISE>(a) : a;
        }
        st_vec<DT>(p.out, ooff + (int64_t)i * p.out_stride_l, E::pack(acc));
#pragma unroll
        for (int k = 0; k < W - 2; ++k) {
            rw[k] = rw[k + 1];
#pragma unroll
            for (int j = 0; j < VEC; ++j) xw[k][j] = xw[k + 1][j];
        }
        rw[W - 2] = xr;
#pragma unroll
        for (int j = 0; j < VEC; ++j) xw[W - 2][j] = xv[j];
    }

    if (!CIRC) {
#pragma unroll
        for (int k = 0; k < W - 1; ++k)
            st_vec<DT>(p.conv_state, soff + (int64_t)(S - (W - 1) + k) * p.state_stride_l, rw[k]);
    }
}

template <int DT, int W, bool CIRC>
__global__ void __launch_bounds__(kBlock)
update_generic_kernel(const cc1d_update_params p, const uint32_t total) {
    using E = Elem<DT>;
    using T = typename E::type;
    constexpr bool PRECISE = E::kPreciseAct;

    const uint32_t gid = blockIdx.x * (uint32_t)kBlock + threadIdx.x;
    if (gid >= total) return;
    const int c = (int)(gid % (uint32_t)p.dim);
    const int b = (int)(gid / (uint32_t)p.dim);
    const int L = p.seqlen;
    const int S = p.state_len;
    const bool silu_on = p.silu != 0;

    const int64_t xoff = (int64_t)b * p.x_stride_b + (int64_t)c * p.x_stride_c;
    const int64_t ooff = (int64_t)b * p.out_stride_b + (int64_t)c * p.out_stride_c;
    const int sb = p.conv_state_indices == nullptr ? b : p.conv_state_indices[b];
    if (sb < 0) {
        for (int i = 0; i < L; ++i) st_raw<DT>(p.out, ooff + (int64_t)i * p.out_stride_l, T(0.f));
        return;
    }
    const int64_t soff = (int64_t)sb * p.state_stride_b + (int64_t)c * p.state_stride_c;

    T rw[W - 1];
    int cs = 0;
    if (CIRC) cs = positive_mod(p.cache_seqlens[b], S);
#pragma unroll
    for (int i = 0; i < W - 1; ++i) {
        const int l = CIRC ? wrap(cs - (W - 1) + i, S) : S - (W - 1) + i;
        rw[i] = ld_raw<DT>(p.conv_state, soff + (int64_t)l * p.state_stride_l);
    }
    float wv[W];
#pragma unroll
    for (int w = 0; w < W; ++w)
        wv[w] = ld_weight(p.weight, p.w_dtype, (int64_t)c * p.w_stride_c + w * p.w_stride_w);
    const float bias_v = p.bias == nullptr ? 0.f : ld_weight(p.bias, p.w_dtype, c);

    if (!CIRC) {
        for (int j = 0; j < S - (W - 1); ++j) {
            const int src = L + j;
            const T v = src < S ? ld_raw<DT>(p.conv_state, soff + (int64_t)src * p.state_stride_l)
                                : ld_raw<DT>(p.x, xoff + (int64_t)(src - S) * p.x_stride_l);
            st_raw<DT>(p.conv_state, soff + (int64_t)j * p.state_stride_l, v);
        }
    }
    int wpos = cs;                                    // circular write position
    for (int i = 0; i < L; ++i) {
        const T xr = ld_raw<DT>(p.x, xoff + (int64_t)i * p.x_stride_l);
        if (CIRC) {
            st_raw<DT>(p.conv_state, soff + (int64_t)wpos * p.state_stride_l, xr);
            wpos = wpos + 1 == S ? 0 : wpos + 1;
        }
        float a = bias_v;
#pragma unroll
        for (int k = 0; k < W - 1; ++k) a = fmaf(wv[k], E::to_float(rw[k]), a);
        a = fmaf(wv[W - 1], E::to_float(xr), a);
        st_elem<DT>(p.out, ooff + (int64_t)i * p.out_stride_l, silu_on ? silu<PRECISE>(a) : a);
#pragma unroll
        for (int k = 0; k < W - 2; ++k) rw[k] = rw[k + 1];
        rw[W - 2] = xr;
    }
    if (!CIRC) {
#pragma unroll
        for (int k = 0; k < W - 1; ++k)
            st_raw<DT>(p.conv_state, soff + (int64_t)(S - (W - 1) + k) * p.state_stride_l, rw[k]);
    }
}

// (rows x dim)-shaped operand usable as 16-byte vectors along dim.
bool rows_vec_ok(const void *ptr, int dtype, int64_t sb, int64_t sc, int64_t sl, int n_rows) {
    const int v = vec_elems(dtype);
    return sc == 1 && sb % v == 0 && (n_rows <= 1 || sl % v == 0) && aligned16(ptr);
}

template <int DT, int W>
int launch_w(const cc1d_update_params &p, bool vec, hipStream_t stream) {
    const bool circ = p.cache_seqlens != nullptr;
    if (vec) {
        const uint32_t ncg = (uint32_t)(p.dim / Elem<DT>::kVec);
        const int64_t total = (int64_t)p.batch * ncg;
        if (total >= ((int64_t)1 << 31)) return CC1D_ERR_TOO_LARGE;
        const uint32_t blocks = (uint32_t)((total + kBlock - 1) / kBlock);
        const int w_fast = weights_contiguous_f32(p.weight, p.w_dtype, p.w_stride_c, p.w_stride_w, p.width);
        if (circ) hipLaunchKernelGGL((update_vec_kernel<DT, W, true>), dim3(blocks), dim3(kBlock), 0, stream, p, ncg, (uint32_t)total, w_fast);
        else hipLaunchKernelGGL((update_vec_kernel<DT, W, false>), dim3(blocks), dim3(kBlock), 0, stream, p, ncg, (uint32_t)total, w_fast);
    } else {
        const int64_t total = (int64_t)p.batch * p.dim;
        if (total >= ((int64_t)1 << 31)) return CC1D_ERR_TOO_LARGE;
        const uint32_t blocks = (uint32_t)((total + kBlock - 1) / kBlock);
        if (circ) hipLaunchKernelGGL((update_generic_kernel<DT, W, true>), dim3(blocks), dim3(kBlock), 0, stream, p, (uint32_t)total);
        else hipLaunchKernelGGL((update_generic_kernel<DT, W, false>), dim3(blocks), dim3(kBlock), 0, stream, p, (uint32_t)total);
    }
    return launch_status();
}

template <int DT>
int launch_dtype(const cc1d_update_params &p, bool vec, hipStream_t stream) {
    switch (p.width) {
        case 2: return launch_w<DT, 2>(p, vec, stream);
        case 3: return launch_w<DT, 3>(p, vec, stream);
        default: return launch_w<DT, 4>(p, vec, stream);
    }
}

}  // namespace

int launch_update(const cc1d_update_params &p, hipStream_t stream) {
    const int v = vec_elems(p.x_dtype);
    const bool vec = p.dim % v == 0 &&
        rows_vec_ok(p.x, p.x_dtype, p.x_stride_b, p.x_stride_c, p.x_stride_l, p.seqlen) &&
        rows_vec_ok(p.out, p.x_dtype, p.out_stride_b, p.out_stride_c, p.out_stride_l, p.seqlen) &&
        rows_vec_ok(p.conv_state, p.x_dtype, p.state_stride_b, p.state_stride_c, p.state_stride_l, p.state_len);
    switch (p.x_dtype) {
        case CC1D_F32: return launch_dtype<CC1D_F32>(p, vec, stream);
        case CC1D_F16: return launch_dtype<CC1D_F16>(p, vec, stream);
        default: return launch_dtype<CC1D_BF16>(p, vec, stream);
    }
}

}  // namespace cc1d
