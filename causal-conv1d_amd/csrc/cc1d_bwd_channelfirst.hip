// Channel-first backward for gfx950.  Takes over causal_conv1d_bwd_kernel and its
// launcher (csrc/causal_conv1d_bwd.cu:53-293 of the reference).  Formulas as in the
// channel-last backward; initial_states / dfinal_states / dinitial_states are supported
// for this layout too (the reference refuses them, csrc/causal_conv1d.cpp:349,364).
//
// Design.  A wavefront owns one channel and a contiguous slice of that channel's
// (batch x segment) items, so its dweight/dbias partial sums live in registers across
// all of them and are reduced over the 64 lanes once, at the very end.  With one slice
// per channel (the usual case, dim >= 4096) the sums go straight to dweight/dbias and no
// workspace exists; otherwise each slice stores W+1 floats and the shared second-stage
// kernel adds the slices in a fixed order.  Either way the result is bit-reproducible.
//
// Inside an item the wave walks DOWN the row, 64 sixteen-byte vectors per step:
//  * the x halo on the left comes from the previous lane (DPP shift); lane 0 takes it
//    from lane 63 of the already prefetched next (lower) step;
//  * g = dout * act'(z) is needed W-1 positions to the right for dx: from the next lane
//    (DPP shift), lane 63 takes it from lane 0 of the previous (higher) step.
// Only an item's first and last step fall back to a few wave-uniform element loads.
// Rows of x, dout and dx may sit on different 16-byte grids; lanes follow x's grid and
// the other tensors use vectors when they share it, elements otherwise.
//
// Three kernels share this design.  The streaming kernel takes every launch in which the rows of
// dout and dx lie on the 16-byte grid of the same rows of x (same shape and strides): whole
// 64-vector steps run without bounds checks in two register sets in ping-pong, and lane 0's x
// halo is a separate small load of its own, so the sets do not depend on each other and the
// loads of the next two steps stay in flight while a step is computed; an odd step and the
// partly filled last step of a row are done first, one checked step at a time, and the few
// positions of a row in front of its first whole vector or behind its last one are done one
// per lane, straight from memory.  The general kernel takes tensors on different grids and
// rows longer than 64 vectors.  The short-row kernel takes rows of at most 64 vectors (whole
// vectors on one grid, or element by element), several batch entries of a channel to a
// wavefront and no walk.
//
// Rows longer than 64 vectors normally do not reach these walking kernels: the tile kernel of
// cc1d_bwd_channelfirst_tile.hip takes them (a wavefront per tile of up to 256 vectors of one
// row, fetched straight into LDS; one workspace plane per tile and the shared second stage), at
// any length and alignment.  The launch tunable bwd_cf_parts = -1 brings the walking kernels
// back for the same tensors; dx and dinitial_states are bit-identical either way.
#include <type_traits>

#include "cc1d_device.hpp"
#include "cc1d_internal.hpp"

namespace cc1d {
namespace {

// dweight / dbias are added into unless the caller asked for plain stores.
__device__ __forceinline__ void accumulate(float *dst, float v, int overwrite) {
    *dst = overwrite ? v : *dst + v;
}

struct BwdCfGeom {
    int32_t streaming;        // 0: general kernel; streaming kernel with rows 1: on the 16-byte grid, 2: anywhere on it;
                              // 3: short-row kernel (an item is then a group of batch entries, n_segs 1),
                              // 4: the same with element accesses
    int32_t vecs_per_seg;     // multiple of 64
    int32_t n_segs;           // segments per row
    int32_t n_items;          // batch * n_segs
    int32_t n_parts;          // slices of the item list per channel
    int32_t items_per_part;
    int32_t lanes_log2;       // short-row kernel (streaming 3, 4): log2 of the lanes one row takes
};

template <int DT>
struct alignas(16) RawT {
    typename Elem<DT>::type v[Elem<DT>::kVec];
};

template <int DT, int W>
struct RowCtx {
    const cc1d_bwd_params &p;
    int b, c;
    int64_t xrow, drow;
    float wv[W];
    float bias_v;
    float wvs[W], bias_s;         // taps and bias times -log2(e), for the activation's derivative
    bool silu_on;

    __device__ __forceinline__ void scale_taps() {
#pragma unroll
        for (int w = 0; w < W; ++w) wvs[w] = wv[w] * kSiluPrescale;
        bias_s = bias_v * kSiluPrescale;
    }
    // act'(z) at the position whose window is xwin[0 .. W)
    __device__ __forceinline__ float act_grad(const float *xwin) const {
        return silu_grad_of_window<W, Elem<DT>::kPreciseAct>(wv, bias_v, wvs, bias_s, xwin);
    }

    // xpad[t] for t < L, raw bits
    __device__ __forceinline__ typename Elem<DT>::type x_raw_at(int t) const {
        using T = typename Elem<DT>::type;
        if (t >= 0) return ld_raw<DT>(p.x, xrow + t);
        if (p.initial_states != nullptr && t >= -(W - 1))
            return ld_raw<DT>(p.initial_states, (int64_t)b * p.init_stride_b +
                                                    (int64_t)c * p.init_stride_c +
                                                    (int64_t)(t + W - 1) * p.init_stride_l);
        return T(0.f);
    }
    // xpad[t] for t < L (fp32)
    __device__ __forceinline__ float x_at(int t) const {
        if (t >= 0) return ld_elem<DT>(p.x, xrow + t);
        if (p.initial_states != nullptr && t >= -(W - 1))
            return ld_elem<DT>(p.initial_states, (int64_t)b * p.init_stride_b +
                                                     (int64_t)c * p.init_stride_c +
                                                     (int64_t)(t + W - 1) * p.init_stride_l);
        return 0.f;
    }
    // g[t0 .. t0+N) and the padded x in front of and under them, xp[i] = xpad[t0-(W-1)+i], with
    // every row access issued unconditionally at a clamped index (one memory round trip for
    // the whole span, no branch between the loads); positions outside [0, L) give g = 0.
    template <int N>
    __device__ __forceinline__ void g_span(int t0, float (&gv)[N], float (&xp)[N + W - 1]) const {
        using T = typename Elem<DT>::type;
        const int L = p.seqlen;
        T xraw[N + W - 1], draw[N];
#pragma unroll
        for (int i = 0; i < N + W - 1; ++i) {
            const int q = t0 - (W - 1) + i;
            xraw[i] = ld_raw<DT>(p.x, xrow + (q < 0 ? 0 : q >= L ? L - 1 : q));
        }
#pragma unroll
        for (int k = 0; k < N; ++k) {
            const int q = t0 + k;
            draw[k] = ld_raw<DT>(p.dout, drow + (q < 0 ? 0 : q >= L ? L - 1 : q));
        }
#pragma unroll
        for (int i = 0; i < N + W - 1; ++i) {
            const int q = t0 - (W - 1) + i;
            xp[i] = q >= 0 && q < L ? Elem<DT>::to_float(xraw[i]) : 0.f;
        }
        if (p.initial_states != nullptr && t0 < W - 1) {          // only at a row's start
#pragma unroll
            for (int i = 0; i < N + W - 1; ++i) {
                const int q = t0 - (W - 1) + i;
                if (q < 0 && q >= -(W - 1)) xp[i] = x_at(q);
            }
        }
#pragma unroll
        for (int k = 0; k < N; ++k) {
            const int q = t0 + k;
            float gk = q >= 0 && q < L ? Elem<DT>::to_float(draw[k]) : 0.f;
            if (silu_on) gk *= act_grad(&xp[k]);
            gv[k] = gk;
        }
    }
    // g[t] recomputed from memory with the same operation order as the vector path.
    __device__ __forceinline__ float g_at(int t) const {
        if (t < 0 || t >= p.seqlen) return 0.f;
        float gv = ld_elem<DT>(p.dout, drow + t);
        if (silu_on) {
            float xwin[W];
#pragma unroll
            for (int w = 0; w < W; ++w) xwin[w] = x_at(t - (W - 1) + w);
            gv *= act_grad(xwin);
        }
        return gv;
    }
};

template <int DT, int W>
__global__ void __launch_bounds__(kBlock)
bwd_channelfirst_kernel(const cc1d_bwd_params p, const BwdCfGeom g, float *__restrict__ ws) {
    using E = Elem<DT>;
    using T = typename E::type;
    constexpr int VEC = E::kVec;
    constexpr bool PRECISE = E::kPreciseAct;

    const uint32_t wid = (blockIdx.x * (uint32_t)kBlock + threadIdx.x) / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    if (wid >= (uint32_t)p.dim * (uint32_t)g.n_parts) return;     // whole wave leaves together
    const int part = (int)(wid % (uint32_t)g.n_parts);
    const int c = (int)(wid / (uint32_t)g.n_parts);
    const int L = p.seqlen;

    RowCtx<DT, W> rc{p};
    rc.c = c;
    rc.silu_on = p.silu != 0;
#pragma unroll
    for (int w = 0; w < W; ++w)
        rc.wv[w] = ld_weight(p.weight, p.w_dtype, (int64_t)c * p.w_stride_c + w * p.w_stride_w);
    rc.bias_v = p.bias == nullptr ? 0.f : ld_weight(p.bias, p.w_dtype, c);
    rc.scale_taps();

    float dW[W], dB = 0.f;
#pragma unroll
    for (int w = 0; w < W; ++w) dW[w] = 0.f;

    const int item_begin = part * g.items_per_part;
    int item_end = item_begin + g.items_per_part;
    if (item_end > g.n_items) item_end = g.n_items;

    for (int item = item_begin; item < item_end; ++item) {
        const int seg = item % g.n_segs;
        const int b = item / g.n_segs;
        rc.b = b;
        rc.xrow = (int64_t)b * p.x_stride_b + (int64_t)c * p.x_stride_c;
        rc.drow = (int64_t)b * p.dout_stride_b + (int64_t)c * p.dout_stride_c;
        const int64_t dxrow = (int64_t)b * p.dx_stride_b + (int64_t)c * p.dx_stride_c;
        const int mis = (int)((reinterpret_cast<uintptr_t>(reinterpret_cast<const T *>(p.x) + rc.xrow) / sizeof(T)) % VEC);
        const int mis_d = (int)((reinterpret_cast<uintptr_t>(reinterpret_cast<const T *>(p.dout) + rc.drow) / sizeof(T)) % VEC);
        const int mis_dx = (int)((reinterpret_cast<uintptr_t>(reinterpret_cast<T *>(p.dx) + dxrow) / sizeof(T)) % VEC);
        const bool dout_same = mis_d == mis, dx_same = mis_dx == mis;

        const int n_vecs = (L + mis + VEC - 1) / VEC;
        const int j_begin = seg * g.vecs_per_seg;
        int j_end = j_begin + g.vecs_per_seg;
        if (j_end > n_vecs) j_end = n_vecs;

        if (j_begin < j_end) {
            // Raw 16-byte vectors on x's grid; positions outside [0, L) read as zero
            // (or initial_states for x), element by element where a vector does not fit.
            auto load_x = [&](int j) -> u32x4 {
                const int tf = j * VEC - mis;
                if (tf >= 0 && tf + VEC <= L) return ld_vec_nt<DT>(p.x, rc.xrow + tf);
                RawT<DT> r;
#pragma unroll
                for (int e = 0; e < VEC; ++e) r.v[e] = (tf + e < L) ? rc.x_raw_at(tf + e) : T(0.f);
                return bitcast<u32x4>(r);
            };
            auto load_d = [&](int j) -> u32x4 {
                const int tf = j * VEC - mis;
                if (dout_same && tf >= 0 && tf + VEC <= L) return ld_vec_nt<DT>(p.dout, rc.drow + tf);
                RawT<DT> r;
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    r.v[e] = (tf + e >= 0 && tf + e < L) ? ld_raw<DT>(p.dout, rc.drow + tf + e) : T(0.f);
                return bitcast<u32x4>(r);
            };

            // g just right of the item (positions of the following segment, or beyond L).
            float carry_g[W - 1];
#pragma unroll
            for (int i = 0; i < W - 1; ++i) carry_g[i] = rc.g_at(j_end * VEC - mis + i);

            // Two steps of loads stay in flight: r1 is the next (lower) step, r2 the one after.
            const int n_steps = (j_end - j_begin + kWave - 1) / kWave;
            const u32x4 zero4 = {0u, 0u, 0u, 0u};
            u32x4 r1x = load_x(j_begin + (n_steps - 1) * kWave + lane);
            u32x4 r1d = load_d(j_begin + (n_steps - 1) * kWave + lane);
            u32x4 r2x = zero4, r2d = zero4;
            if (n_steps > 1) {
                r2x = load_x(j_begin + (n_steps - 2) * kWave + lane);
                r2d = load_d(j_begin + (n_steps - 2) * kWave + lane);
            }

            for (int s = n_steps - 1; s >= 0; --s) {
                const int j0 = j_begin + s * kWave;
                float xf[VEC], gf[VEC];
                E::unpack(r1x, xf);
                E::unpack(r1d, gf);
                r1x = r2x; r1d = r2d;
                if (s >= 2) {
                    r2x = load_x(j0 - 2 * kWave + lane);
                    r2d = load_d(j0 - 2 * kWave + lane);
                }

                // x just left of this step: lane 63 of the next (lower) step, which was
                // requested a whole step ago; memory only at the item's lowest step.
                float carry_x[W - 1];
                if (s > 0) {
                    float lower[VEC];
                    E::unpack(r1x, lower);
#pragma unroll
                    for (int i = 0; i < W - 1; ++i) carry_x[i] = read_lane(lower[VEC - (W - 1) + i], kWave - 1);
                } else {
#pragma unroll
                    for (int i = 0; i < W - 1; ++i) carry_x[i] = rc.x_at(j0 * VEC - mis - (W - 1) + i);
                }

                // xx[i] = xpad at position tf-(W-1)+i
                float xx[VEC + W - 1];
#pragma unroll
                for (int i = 0; i < W - 1; ++i) xx[i] = from_prev_lane(xf[VEC - (W - 1) + i], carry_x[i]);
#pragma unroll
                for (int e = 0; e < VEC; ++e) xx[W - 1 + e] = xf[e];

                if (rc.silu_on) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        gf[e] *= rc.act_grad(&xx[e]);
                    }
                }

                // gg[i] = g at position tf+i, i in [0, VEC+W-1)
                float gg[VEC + W - 1];
#pragma unroll
                for (int e = 0; e < VEC; ++e) gg[e] = gf[e];
#pragma unroll
                for (int i = 0; i < W - 1; ++i) {
                    gg[VEC + i] = from_next_lane(gf[i], carry_g[i]);
                    carry_g[i] = read_lane(gf[i], 0);
                }

                const int j = j0 + lane;
                const int tf = j * VEC - mis;
                float dxv[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float a = 0.f;
#pragma unroll
                    for (int k = 0; k < W; ++k) a = fmaf(rc.wv[W - 1 - k], gg[e + k], a);
                    dxv[e] = a;
                }
                if (p.dfinal_states != nullptr && tf + VEC > L - (W - 1)) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const int t = tf + e;
                        if (t >= 0 && t >= L - (W - 1) && t < L)
                            dxv[e] += ld_elem<DT>(p.dfinal_states, (int64_t)b * p.dfinal_stride_b +
                                                                      (int64_t)c * p.dfinal_stride_c +
                                                                      (int64_t)(t - (L - (W - 1))) * p.dfinal_stride_l);
                    }
                }
                if (j < j_end) {
                    if (dx_same && tf >= 0 && tf + VEC <= L) {
                        st_vec_nt<DT>(p.dx, dxrow + tf, E::pack(dxv));
                    } else {
#pragma unroll
                        for (int e = 0; e < VEC; ++e)
                            if (tf + e >= 0 && tf + e < L) st_elem<DT>(p.dx, dxrow + tf + e, dxv[e]);
                    }
                }

                // Partial sums.  Lanes past j_end and positions outside [0, L) hold g == 0.
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    dB += gf[e];
#pragma unroll
                    for (int w = 0; w < W; ++w) dW[w] = fmaf(gf[e], xx[e + w], dW[w]);
                }
            }
        }

        // dinitial_states[b, c, i], i = lane < W-1, by the wave that owns the row's start.
        if (p.dinitial_states != nullptr && seg == 0 && lane < W - 1) {
            const int pp = lane - (W - 1);
            float a = 0.f;
#pragma unroll
            for (int k = 0; k < W; ++k) a = fmaf(rc.wv[W - 1 - k], rc.g_at(pp + k), a);
            if (p.dfinal_states != nullptr && lane >= L)
                a += ld_elem<DT>(p.dfinal_states, (int64_t)b * p.dfinal_stride_b +
                                                     (int64_t)c * p.dfinal_stride_c +
                                                     (int64_t)(lane - L) * p.dfinal_stride_l);
            st_elem<DT>(p.dinitial_states, (int64_t)b * p.dinit_stride_b + (int64_t)c * p.dinit_stride_c +
                                               (int64_t)lane * p.dinit_stride_l, a);
        }
    }

    // One fixed-order reduction over the wave, then a single writer.
#pragma unroll
    for (int w = 0; w < W; ++w) dW[w] = wave_sum(dW[w]);
    dB = wave_sum(dB);
    if (lane == 0) {
        if (g.n_parts == 1) {
#pragma unroll
            for (int w = 0; w < W; ++w)
                accumulate(p.dweight + (int64_t)c * p.dw_stride_c + (int64_t)w * p.dw_stride_w, dW[w], p.overwrite_dweight);
            if (p.dbias != nullptr) accumulate(p.dbias + c, dB, p.overwrite_dweight);
        } else {
            float *dst = ws + (int64_t)part * (W + 1) * p.dim + c;
#pragma unroll
            for (int w = 0; w < W; ++w) dst[(int64_t)w * p.dim] = dW[w];
            dst[(int64_t)W * p.dim] = dB;
        }
    }
}

// GRID: rows may start anywhere on their 16-byte grid and have any length; false: every row
// starts on the grid and is a whole number of vectors long (no edge positions exist, and the
// code for them is compiled out).
template <int DT, int W, bool GRID>
__global__ void __launch_bounds__(kBlock)
bwd_channelfirst_stream_kernel(const cc1d_bwd_params p, const BwdCfGeom g, float *__restrict__ ws) {
    using E = Elem<DT>;
    using T = typename E::type;
    constexpr int VEC = E::kVec;
    constexpr bool PRECISE = E::kPreciseAct;
    // The four elements in front of a step, as one aligned load: 8 bytes of 16-bit data or
    // 16 bytes of fp32; the last W-1 of them are lane 0's halo.
    constexpr int HALO = 4;
    using halo_t = typename RawBytes<HALO * E::kBytes>::type;
    using HP = Pack<DT, HALO>;

    const uint32_t wid = (blockIdx.x * (uint32_t)kBlock + threadIdx.x) / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    if (wid >= (uint32_t)p.dim * (uint32_t)g.n_parts) return;     // whole wave leaves together
    const int part = (int)(wid % (uint32_t)g.n_parts);
    const int c = (int)(wid / (uint32_t)g.n_parts);
    const int L = p.seqlen;

    RowCtx<DT, W> rc{p};
    rc.c = c;
    rc.silu_on = p.silu != 0;
#pragma unroll
    for (int w = 0; w < W; ++w)
        rc.wv[w] = ld_weight(p.weight, p.w_dtype, (int64_t)c * p.w_stride_c + w * p.w_stride_w);
    rc.bias_v = p.bias == nullptr ? 0.f : ld_weight(p.bias, p.w_dtype, c);
    rc.scale_taps();

    float dW[W], dB = 0.f;
#pragma unroll
    for (int w = 0; w < W; ++w) dW[w] = 0.f;

    const int item_begin = part * g.items_per_part;
    int item_end = item_begin + g.items_per_part;
    if (item_end > g.n_items) item_end = g.n_items;
    using No = std::integral_constant<bool, false>;
    using Yes = std::integral_constant<bool, true>;

    for (int item = item_begin; item < item_end; ++item) {
        const int seg = item % g.n_segs;
        const int b = item / g.n_segs;
        rc.b = b;
        rc.xrow = (int64_t)b * p.x_stride_b + (int64_t)c * p.x_stride_c;
        rc.drow = (int64_t)b * p.dout_stride_b + (int64_t)c * p.dout_stride_c;
        const T *xr = reinterpret_cast<const T *>(p.x) + rc.xrow;
        const T *dr = reinterpret_cast<const T *>(p.dout) + rc.drow;
        T *dxr = reinterpret_cast<T *>(p.dx) + (int64_t)b * p.dx_stride_b + (int64_t)c * p.dx_stride_c;

        // The row on its own 16-byte grid (x, dout and dx share it): vector j holds positions
        // j*VEC - mis .. j*VEC - mis + VEC.  Vectors jf0 .. jf1 lie inside the row and are walked
        // below; the up to VEC-1 positions in front of them and behind them are edge positions,
        // each done by one lane straight from memory.
        const int mis = GRID ? (int)((reinterpret_cast<uintptr_t>(xr) / sizeof(T)) % VEC) : 0;
        const int jf0 = mis > 0 ? 1 : 0;
        const int jf1 = (L + mis) / VEC;                // >= jf0: the launcher sends rows shorter than 2 VEC elsewhere
        int j_begin = seg * g.vecs_per_seg;
        int j_end = j_begin + g.vecs_per_seg;
        const bool owns_back = j_begin <= jf1 && jf1 < j_end;
        if (j_begin < jf0) j_begin = jf0;
        if (j_end > jf1) j_end = jf1;

        // The item's lowest full steps, an even number of them, go through the ping-pong
        // pipeline; what is above them (an odd full step, a partly filled last step) is done
        // first, one checked step at a time.
        const bool has_vecs = j_begin < j_end;
        const int n_steps = has_vecs ? (j_end - j_begin) / (2 * kWave) * 2 : 0;
        const int j_pipe_end = j_begin + n_steps * kWave;
        const bool row_top = j_end == jf1, row_bottom = j_begin == jf0;
        const T *xg = xr - mis, *dg = dr - mis;         // grid origins
        T *dxg = dxr - mis;

        // Step k counts down the pipeline's range: k = 0 is its highest 64 vectors.
        auto load_step = [&](int k, u32x4 &rx, u32x4 &rd, halo_t &rh) {
            const int e0 = (j_begin + (n_steps - 1 - k) * kWave) * VEC;   // the step's first element on the grid
            rx = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(xg + e0 + lane * VEC));
            rd = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(dg + e0 + lane * VEC));
            // The HALO elements in front of the step, or (lowest step of the row, where they
            // may lie in front of the row and are replaced below) the step's own first ones.
            const int h0 = e0 - mis >= HALO ? e0 - HALO : e0;
            rh = *reinterpret_cast<const halo_t *>(xg + h0);
        };
        // With rows off the grid the pipeline's first two steps are requested before the edge
        // work, so that its memory round trip and theirs overlap.
        u32x4 ax, ad, bx, bd;
        halo_t ah, bh;
        if (GRID && n_steps > 0) {
            load_step(0, ax, ad, ah);
            load_step(1, bx, bd, bh);
        }

        float edge_g = 0.f;                               // g at this lane's edge position
        const int back = jf1 * VEC - mis;                 // edge positions [back, L)
        {
            const int front = mis == 0 ? 0 : VEC - mis;   // and [0, front)
            int t = -1;
            if (seg == 0 && lane < front) t = lane;
            if (owns_back && lane >= VEC && lane - VEC < L - back) t = back + lane - VEC;
            if (GRID && t >= 0) {
                float gt[W], xp[2 * W - 1];
                rc.template g_span<W>(t, gt, xp);
                float a = 0.f;
#pragma unroll
                for (int k = 0; k < W; ++k) a = fmaf(rc.wv[W - 1 - k], gt[k], a);
                if (p.dfinal_states != nullptr && t >= L - (W - 1))
                    a += ld_elem<DT>(p.dfinal_states, (int64_t)b * p.dfinal_stride_b + (int64_t)c * p.dfinal_stride_c +
                                                          (int64_t)(t - (L - (W - 1))) * p.dfinal_stride_l);
                dxr[t] = E::from_float(a);
                edge_g = gt[0];
                dB += gt[0];
#pragma unroll
                for (int w = 0; w < W; ++w) dW[w] = fmaf(gt[0], xp[w], dW[w]);
            }
            // dinitial_states[i] = dx at position i-(W-1) < 0, by the wave that owns the row's
            // start when the first positions are edge positions (else the walk's lowest step
            // does it from registers).
            if (GRID && mis > 0 && p.dinitial_states != nullptr && seg == 0 && lane >= 2 * VEC && lane < 2 * VEC + W - 1) {
                const int i = lane - 2 * VEC;
                float gi[W], xp[2 * W - 1];
                rc.template g_span<W>(i - (W - 1), gi, xp);
                float a = 0.f;
#pragma unroll
                for (int k = 0; k < W; ++k) a = fmaf(rc.wv[W - 1 - k], gi[k], a);
                st_elem<DT>(p.dinitial_states, (int64_t)b * p.dinit_stride_b + (int64_t)c * p.dinit_stride_c +
                                                   (int64_t)i * p.dinit_stride_l, a);
            }
        }
        if (!has_vecs) continue;
        // g just right of the item: the row's back edge (the lanes above have just computed it),
        // or the next segment's first positions recomputed from memory; zero past the row's end.
        float carry_g[W - 1];
        if (GRID && row_top && owns_back) {
#pragma unroll
            for (int i = 0; i < W - 1; ++i) carry_g[i] = back + i < L ? read_lane(edge_g, VEC + i) : 0.f;
        } else if (j_end * VEC - mis < L) {
            float xp[2 * (W - 1)];
            rc.template g_span<W - 1>(j_end * VEC - mis, carry_g, xp);
        } else {
#pragma unroll
            for (int i = 0; i < W - 1; ++i) carry_g[i] = 0.f;
        }

        // top / bottom: compiled in for the steps that can be the item's highest / lowest;
        // top_rt / bottom_rt say whether this one is, and is the row's end as well.
        auto compute_at = [&](auto top, auto bottom, auto checked, bool top_rt, bool bottom_rt, int e0, int nvalid,
                              const u32x4 &rx, const u32x4 &rd, const halo_t &rh) {
            float xf[VEC], gf[VEC], hf[HALO], carry_x[W - 1];
            E::unpack(rx, xf);
            E::unpack(rd, gf);
            HP::unpack(rh, hf);
#pragma unroll
            for (int i = 0; i < W - 1; ++i) carry_x[i] = hf[HALO - (W - 1) + i];
            if (decltype(bottom)::value) {
                if (bottom_rt) {
#pragma unroll
                    for (int i = 0; i < W - 1; ++i) carry_x[i] = rc.x_at(e0 - mis - (W - 1) + i);
                }
            }
            // xx[i] = xpad at position tf-(W-1)+i
            float xx[VEC + W - 1];
#pragma unroll
            for (int i = 0; i < W - 1; ++i) xx[i] = from_prev_lane(xf[VEC - (W - 1) + i], carry_x[i]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) xx[W - 1 + e] = xf[e];
            if (rc.silu_on) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    gf[e] *= rc.act_grad(&xx[e]);
                }
            }
            // gg[i] = g at position tf+i, i in [0, VEC+W-1)
            float gg[VEC + W - 1];
#pragma unroll
            for (int e = 0; e < VEC; ++e) gg[e] = gf[e];
#pragma unroll
            for (int i = 0; i < W - 1; ++i) {
                gg[VEC + i] = from_next_lane(gf[i], carry_g[i]);
                // A partly filled step: its last vector's right neighbour is what follows the
                // item, not the idle lane behind it.
                if (decltype(checked)::value) gg[VEC + i] = lane == nvalid - 1 ? carry_g[i] : gg[VEC + i];
                carry_g[i] = read_lane(gf[i], 0);
            }
            float dxv[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float a = 0.f;
#pragma unroll
                for (int k2 = 0; k2 < W; ++k2) a = fmaf(rc.wv[W - 1 - k2], gg[e + k2], a);
                dxv[e] = a;
            }
            if (decltype(top)::value) {
                // dfinal_states[i] belongs to position L-(W-1)+i: those of them that lie in the
                // row's last whole vector (the rest are back-edge positions).
                if (top_rt && p.dfinal_states != nullptr && lane == nvalid - 1) {
                    const int first = L - (W - 1) - (e0 - mis + lane * VEC);   // element of this vector at i = 0
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const int i = e - first;
                        if (i >= 0 && i < W - 1)
                            dxv[e] += ld_elem<DT>(p.dfinal_states, (int64_t)b * p.dfinal_stride_b +
                                                                      (int64_t)c * p.dfinal_stride_c +
                                                                      (int64_t)i * p.dfinal_stride_l);
                    }
                }
            }
            if (!decltype(checked)::value || lane < nvalid)
                __builtin_nontemporal_store(E::pack(dxv), reinterpret_cast<u32x4 *>(dxg + e0 + lane * VEC));
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                dB += gf[e];
#pragma unroll
                for (int w = 0; w < W; ++w) dW[w] = fmaf(gf[e], xx[e + w], dW[w]);
            }
            if (decltype(bottom)::value) {
                // dinitial_states[i] = dx at position i-(W-1) < 0: only g[0 .. i] reach it.
                if (bottom_rt && mis == 0 && p.dinitial_states != nullptr && lane == 0) {
#pragma unroll
                    for (int i = 0; i < W - 1; ++i) {
                        float a = 0.f;
#pragma unroll
                        for (int q = 0; q <= i; ++q) a = fmaf(rc.wv[i - q], gf[q], a);
                        st_elem<DT>(p.dinitial_states, (int64_t)b * p.dinit_stride_b + (int64_t)c * p.dinit_stride_c +
                                                           (int64_t)i * p.dinit_stride_l, a);
                    }
                }
            }
        };

        // Checked steps above the pipeline's range, highest first.  Lanes past the item's end
        // read zeros (so their g is zero) and store nothing.
        for (int js = j_begin + (j_end - j_begin - 1) / kWave * kWave; js >= j_pipe_end; js -= kWave) {
            const int nvalid = j_end - js < kWave ? j_end - js : kWave;
            const int e0 = js * VEC;
            u32x4 rx = {0u, 0u, 0u, 0u}, rd = {0u, 0u, 0u, 0u};
            if (lane < nvalid) {
                rx = *reinterpret_cast<const u32x4 *>(xg + e0 + lane * VEC);
                rd = *reinterpret_cast<const u32x4 *>(dg + e0 + lane * VEC);
            }
            const halo_t rh = *reinterpret_cast<const halo_t *>(xg + (e0 - mis >= HALO ? e0 - HALO : e0));
            compute_at(Yes{}, Yes{}, Yes{}, row_top && js + nvalid == j_end, row_bottom && js == j_begin, e0, nvalid,
                       rx, rd, rh);
        }
        if (n_steps == 0) continue;
        const bool pipe_top = row_top && j_pipe_end == j_end;      // nothing was done above it
        auto compute_step = [&](auto top, auto bottom, int k, const u32x4 &rx, const u32x4 &rd, const halo_t &rh) {
            compute_at(top, bottom, No{}, pipe_top, row_bottom, (j_begin + (n_steps - 1 - k) * kWave) * VEC, kWave,
                       rx, rd, rh);
        };

        // Two register sets in ping-pong; the first and last pair of steps are peeled so the
        // loop is entered in the state its back edge leaves and the wait counts stay exact.
        if (!GRID) {
            load_step(0, ax, ad, ah);
            load_step(1, bx, bd, bh);
        }
        if (n_steps == 2) {
            compute_step(Yes{}, No{}, 0, ax, ad, ah);
            compute_step(No{}, Yes{}, 1, bx, bd, bh);
        } else {
            compute_step(Yes{}, No{}, 0, ax, ad, ah);
            load_step(2, ax, ad, ah);
            compute_step(No{}, No{}, 1, bx, bd, bh);
            load_step(3, bx, bd, bh);
            int k = 2;
#pragma clang loop unroll(disable)
            for (; k + 2 < n_steps; k += 2) {
                compute_step(No{}, No{}, k, ax, ad, ah);
                load_step(k + 2, ax, ad, ah);
                compute_step(No{}, No{}, k + 1, bx, bd, bh);
                load_step(k + 3, bx, bd, bh);
            }
            compute_step(No{}, No{}, k, ax, ad, ah);
            compute_step(No{}, Yes{}, k + 1, bx, bd, bh);
        }
    }

    // One fixed-order reduction over the wave, then a single writer.
#pragma unroll
    for (int w = 0; w < W; ++w) dW[w] = wave_sum(dW[w]);
    dB = wave_sum(dB);
    if (lane == 0) {
        if (g.n_parts == 1) {
#pragma unroll
            for (int w = 0; w < W; ++w)
                accumulate(p.dweight + (int64_t)c * p.dw_stride_c + (int64_t)w * p.dw_stride_w, dW[w], p.overwrite_dweight);
            if (p.dbias != nullptr) accumulate(p.dbias + c, dB, p.overwrite_dweight);
        } else {
            float *dst = ws + (int64_t)part * (W + 1) * p.dim + c;
#pragma unroll
            for (int w = 0; w < W; ++w) dst[(int64_t)w * p.dim] = dW[w];
            dst[(int64_t)W * p.dim] = dB;
        }
    }
}

// Rows of at most 64 vectors.  One wavefront per row would leave most lanes idle and walk the
// batch one short row at a time, so a wavefront takes 64 / G batch entries of its channel at once,
// G = 1, 2, 4 ... 64 lanes each: lane (r, v) owns vector v of entry r, x's halo comes from the
// previous lane (vector 0: zeros or initial_states), g's from the next lane (last vector: zeros),
// and an item is one load of x, one of dout and one store of dx per lane.  Formulas, operation
// order and the reduction at the end are those of the kernels above.
// ALIGNED: rows of whole vectors, every tensor on one 16-byte grid.  ALIGNED = false: rows of any
// length (down to 1) anywhere in memory, the same lanes, with a lane's up to VEC positions read
// and written element by element (positions past the row's end read as zero).
template <int DT, int W, bool ALIGNED>
__global__ void __launch_bounds__(kBlock)
bwd_channelfirst_short_kernel(const cc1d_bwd_params p, const BwdCfGeom g, float *__restrict__ ws) {
    using E = Elem<DT>;
    constexpr int VEC = E::kVec;
    constexpr bool PRECISE = E::kPreciseAct;

    const uint32_t wid = (blockIdx.x * (uint32_t)kBlock + threadIdx.x) / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    if (wid >= (uint32_t)p.dim * (uint32_t)g.n_parts) return;     // whole wave leaves together
    const int part = (int)(wid % (uint32_t)g.n_parts);
    const int c = (int)(wid / (uint32_t)g.n_parts);
    const int L = p.seqlen;
    const int n_vecs = (L + VEC - 1) / VEC;
    const int v = lane & ((1 << g.lanes_log2) - 1);
    const int r = lane >> g.lanes_log2;
    const int rows_per_item = kWave >> g.lanes_log2;
    const bool silu_on = p.silu != 0;

    float wv[W], bias_v;
#pragma unroll
    for (int w = 0; w < W; ++w)
        wv[w] = ld_weight(p.weight, p.w_dtype, (int64_t)c * p.w_stride_c + w * p.w_stride_w);
    bias_v = p.bias == nullptr ? 0.f : ld_weight(p.bias, p.w_dtype, c);
    float wvs[W];
#pragma unroll
    for (int w = 0; w < W; ++w) wvs[w] = wv[w] * kSiluPrescale;
    const float bias_s = bias_v * kSiluPrescale;

    float dW[W], dB = 0.f;
#pragma unroll
    for (int w = 0; w < W; ++w) dW[w] = 0.f;

    const int item_begin = part * g.items_per_part;
    int item_end = item_begin + g.items_per_part;
    if (item_end > g.n_items) item_end = g.n_items;

    for (int item = item_begin; item < item_end; ++item) {
        // Lanes without a vector of their own stay in step (the lane shifts need every lane) on
        // entry 0's addresses; they load zeros, add zeros to the sums and store nothing.
        const int b_here = item * rows_per_item + r;
        const bool mine = b_here < p.batch && v < n_vecs;
        const int b = mine ? b_here : 0;
        const int64_t xrow = (int64_t)b * p.x_stride_b + (int64_t)c * p.x_stride_c;
        const int64_t drow = (int64_t)b * p.dout_stride_b + (int64_t)c * p.dout_stride_c;
        const int64_t dxrow = (int64_t)b * p.dx_stride_b + (int64_t)c * p.dx_stride_c;

        float xf[VEC], gf[VEC];
        if (ALIGNED) {
            u32x4 rx = u32x4{0u, 0u, 0u, 0u}, rd = u32x4{0u, 0u, 0u, 0u};
            if (mine) {
                rx = ld_vec_nt<DT>(p.x, xrow + (int64_t)v * VEC);
                rd = ld_vec_nt<DT>(p.dout, drow + (int64_t)v * VEC);
            }
            E::unpack(rx, xf);
            E::unpack(rd, gf);
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) xf[e] = gf[e] = 0.f;
            if (mine) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    if (v * VEC + e < L) {
                        xf[e] = ld_elem<DT>(p.x, xrow + v * VEC + e);
                        gf[e] = ld_elem<DT>(p.dout, drow + v * VEC + e);
                    }
                }
            }
        }
        float halo[W - 1];
#pragma unroll
        for (int i = 0; i < W - 1; ++i) halo[i] = 0.f;
        if (mine && v == 0 && p.initial_states != nullptr) {
#pragma unroll
            for (int i = 0; i < W - 1; ++i)
                halo[i] = ld_elem<DT>(p.initial_states, (int64_t)b * p.init_stride_b + (int64_t)c * p.init_stride_c +
                                                            (int64_t)i * p.init_stride_l);
        }

        // xx[i] = xpad at position v*VEC-(W-1)+i
        float xx[VEC + W - 1];
#pragma unroll
        for (int i = 0; i < W - 1; ++i) {
            const float prev = from_prev_lane(xf[VEC - (W - 1) + i], 0.f);
            xx[i] = v == 0 ? halo[i] : prev;
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) xx[W - 1 + e] = xf[e];

        if (silu_on) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                gf[e] *= silu_grad_of_window<W, PRECISE>(wv, bias_v, wvs, bias_s, &xx[e]);
            }
        }

        // gg[i] = g at position v*VEC+i; nothing follows a row's last vector
        float gg[VEC + W - 1];
#pragma unroll
        for (int e = 0; e < VEC; ++e) gg[e] = gf[e];
#pragma unroll
        for (int i = 0; i < W - 1; ++i) {
            const float next = from_next_lane(gf[i], 0.f);
            gg[VEC + i] = v == n_vecs - 1 ? 0.f : next;
        }

        float dxv[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float a = 0.f;
#pragma unroll
            for (int k = 0; k < W; ++k) a = fmaf(wv[W - 1 - k], gg[e + k], a);
            dxv[e] = a;
        }
        // The row's last W-1 positions take dfinal_states (whole vectors: all in the last one).
        if (ALIGNED) {
            if (p.dfinal_states != nullptr && mine && v == n_vecs - 1) {
#pragma unroll
                for (int i = 0; i < W - 1; ++i)
                    dxv[VEC - (W - 1) + i] += ld_elem<DT>(p.dfinal_states, (int64_t)b * p.dfinal_stride_b +
                                                                               (int64_t)c * p.dfinal_stride_c +
                                                                               (int64_t)i * p.dfinal_stride_l);
            }
            if (mine) st_vec_nt<DT>(p.dx, dxrow + (int64_t)v * VEC, E::pack(dxv));
        } else if (mine) {
            if (p.dfinal_states != nullptr && (v + 1) * VEC > L - (W - 1)) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const int t = v * VEC + e;
                    if (t >= L - (W - 1) && t < L)
                        dxv[e] += ld_elem<DT>(p.dfinal_states, (int64_t)b * p.dfinal_stride_b +
                                                                   (int64_t)c * p.dfinal_stride_c +
                                                                   (int64_t)(t - (L - (W - 1))) * p.dfinal_stride_l);
                }
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                if (v * VEC + e < L) st_elem<DT>(p.dx, dxrow + v * VEC + e, dxv[e]);
        }

#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            dB += gf[e];
#pragma unroll
            for (int w = 0; w < W; ++w) dW[w] = fmaf(gf[e], xx[e + w], dW[w]);
        }

        // dinitial_states[b, c, i]: the expression of dx at position i-(W-1) < 0, by the lane that
        // owns vector 0; where the row is shorter than W-1, final_states[i-L] was a copy of
        // initial_states[i], so its gradient lands here.
        if (p.dinitial_states != nullptr && mine && v == 0) {
#pragma unroll
            for (int i = 0; i < W - 1; ++i) {
                float a = 0.f;
#pragma unroll
                for (int k = 0; k < W; ++k) {
                    const int t = i - (W - 1) + k;
                    a = fmaf(wv[W - 1 - k], t >= 0 ? gf[t] : 0.f, a);
                }
                if (!ALIGNED && p.dfinal_states != nullptr && i >= L)
                    a += ld_elem<DT>(p.dfinal_states, (int64_t)b * p.dfinal_stride_b + (int64_t)c * p.dfinal_stride_c +
                                                          (int64_t)(i - L) * p.dfinal_stride_l);
                st_elem<DT>(p.dinitial_states, (int64_t)b * p.dinit_stride_b + (int64_t)c * p.dinit_stride_c +
                                                   (int64_t)i * p.dinit_stride_l, a);
            }
        }
    }

    // One fixed-order reduction over the wave, then a single writer.
#pragma unroll
    for (int w = 0; w < W; ++w) dW[w] = wave_sum(dW[w]);
    dB = wave_sum(dB);
    if (lane == 0) {
        if (g.n_parts == 1) {
#pragma unroll
            for (int w = 0; w < W; ++w)
                accumulate(p.dweight + (int64_t)c * p.dw_stride_c + (int64_t)w * p.dw_stride_w, dW[w], p.overwrite_dweight);
            if (p.dbias != nullptr) accumulate(p.dbias + c, dB, p.overwrite_dweight);
        } else {
            float *dst = ws + (int64_t)part * (W + 1) * p.dim + c;
#pragma unroll
            for (int w = 0; w < W; ++w) dst[(int64_t)w * p.dim] = dW[w];
            dst[(int64_t)W * p.dim] = dB;
        }
    }
}

// Every row of tensor b lies on the 16-byte grid of the same row of tensor a.
bool rows_share_grid(const void *a, int64_t a_stride_b, int64_t a_stride_c, const void *b, int64_t b_stride_b,
                     int64_t b_stride_c, int vec) {
    return (reinterpret_cast<uintptr_t>(a) - reinterpret_cast<uintptr_t>(b)) % 16 == 0 &&
           (a_stride_b - b_stride_b) % vec == 0 && (a_stride_c - b_stride_c) % vec == 0;
}

BwdCfGeom make_geom(const cc1d_bwd_params &p) {
    const int vec = vec_elems(p.x_dtype);
    // The streaming kernel walks x, dout and dx on one grid per row, and wants a row to hold
    // at least one whole vector wherever it starts on that grid.
    const bool streaming = p.seqlen >= 2 * vec && reinterpret_cast<uintptr_t>(p.x) % elem_bytes(p.x_dtype) == 0 &&
                           rows_share_grid(p.x, p.x_stride_b, p.x_stride_c, p.dout, p.dout_stride_b, p.dout_stride_c, vec) &&
                           rows_share_grid(p.x, p.x_stride_b, p.x_stride_c, p.dx, p.dx_stride_b, p.dx_stride_c, vec);
    // Worst case over row alignments: a row may start up to vec-1 elements into its grid.
    const int64_t max_vecs = ((int64_t)p.seqlen + vec - 1 + vec - 1) / vec;
    const int64_t max_steps = (max_vecs + kWave - 1) / kWave;     // 64-vector steps per row
    // About 16 waves on each of 256 CUs when the problem allows it.
    const int32_t forced_parts = tunables().bwd_cf_parts;
    int64_t parts = forced_parts > 0 ? forced_parts : (4096 + p.dim - 1) / p.dim;
    const int64_t max_parts = (int64_t)p.batch * max_steps;
    if (parts > max_parts) parts = max_parts;
    if (parts < 1) parts = 1;
    BwdCfGeom g;
    const bool on_grid = aligned16(p.x) && p.x_stride_b % vec == 0 && p.x_stride_c % vec == 0 && p.seqlen % vec == 0;
    g.lanes_log2 = 0;
    // Short rows of whole vectors with every tensor on one grid: several batch entries to a
    // wavefront, an item is a group of them.  (16, 5376, 128) bf16 57.2 -> 16.0 us, fp32 43.0 -> 25.0 us;
    // (4, 5376, 256) bf16 18.2 -> 10.3 us.
    // Rows that are not whole vectors on one grid take the same lanes with element accesses:
    // (16, 5376, 100) bf16 107 -> 39 us, (64, 2048, 60) 165 -> 36 us, (256, 5376, 4) 1514 -> 73 us.
    const int64_t n_vecs = ((int64_t)p.seqlen + vec - 1) / vec;
    if (n_vecs <= kWave) {
        const bool aligned = on_grid &&
            rows_share_grid(p.x, p.x_stride_b, p.x_stride_c, p.dout, p.dout_stride_b, p.dout_stride_c, vec) &&
            rows_share_grid(p.x, p.x_stride_b, p.x_stride_c, p.dx, p.dx_stride_b, p.dx_stride_c, vec);
        while ((1 << g.lanes_log2) < n_vecs) ++g.lanes_log2;
        const int64_t per_item = kWave >> g.lanes_log2;
        g.streaming = aligned ? 3 : 4;
        g.vecs_per_seg = kWave;
        g.n_segs = 1;
        g.n_items = (int32_t)((p.batch + per_item - 1) / per_item);
        if (parts > g.n_items) parts = g.n_items;
        g.items_per_part = (int32_t)((g.n_items + parts - 1) / parts);
        g.n_parts = (g.n_items + g.items_per_part - 1) / g.items_per_part;
        return g;
    }
    // The chip holds about 4096 of these wavefronts at once.  A launch of 1 to 1.5 times that many
    // long-lived ones ends with the chip mostly idle while the last few finish, so it is cut finer
    // instead, down to eight steps of work per wavefront: (32, 1536, 2048) bf16 126 -> 107 us,
    // (64, 768, 1024) 69 -> 65 us, (8, 5376, 2048) fp32 205 -> 175 us, (1, 5376, 131072) bf16 875 -> 690 us;
    // other wave counts measured best as they are.
    if (forced_parts <= 0 && p.dim * parts > 4096 && 2 * p.dim * parts < 3 * 4096) {
        int64_t finer = p.batch * max_steps / 8;
        if (finer > 64) finer = 64;
        if (finer > parts) parts = finer;
    }
    // Split rows into segments only if there are fewer rows per channel than slices.
    int64_t n_segs = (parts + p.batch - 1) / p.batch;
    int64_t steps_per_seg = (max_steps + n_segs - 1) / n_segs;
    if (streaming) steps_per_seg = (steps_per_seg + 1) / 2 * 2;    // whole step pairs
    int64_t vps = steps_per_seg * kWave;
    n_segs = (max_vecs + vps - 1) / vps;
    g.streaming = !streaming ? 0 : on_grid ? 1 : 2;
    g.vecs_per_seg = (int32_t)vps;
    g.n_segs = (int32_t)n_segs;
    g.n_items = (int32_t)(p.batch * n_segs);
    g.items_per_part = (int32_t)((g.n_items + parts - 1) / parts);
    g.n_parts = (g.n_items + g.items_per_part - 1) / g.items_per_part;
    return g;
}

template <int DT>
int launch_dtype(const cc1d_bwd_params &p, const BwdCfGeom &g, float *ws, hipStream_t stream) {
    const int64_t waves = (int64_t)p.dim * g.n_parts;
    if (waves >= wave_limit()) return CC1D_ERR_TOO_LARGE;
    const uint32_t blocks = (uint32_t)((waves + (kBlock / kWave) - 1) / (kBlock / kWave));
    if (g.streaming == 3) {                           // short rows, several batch entries to a wavefront
        switch (p.width) {
            case 2: CC1D_LAUNCH((bwd_channelfirst_short_kernel<DT, 2, true>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
            case 3: CC1D_LAUNCH((bwd_channelfirst_short_kernel<DT, 3, true>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
            default: CC1D_LAUNCH((bwd_channelfirst_short_kernel<DT, 4, true>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
        }
        return launch_status();
    }
    if (g.streaming == 4) {                           // the same, rows of any length anywhere in memory
        switch (p.width) {
            case 2: CC1D_LAUNCH((bwd_channelfirst_short_kernel<DT, 2, false>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
            case 3: CC1D_LAUNCH((bwd_channelfirst_short_kernel<DT, 3, false>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
            default: CC1D_LAUNCH((bwd_channelfirst_short_kernel<DT, 4, false>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
        }
        return launch_status();
    }
    if (g.streaming == 1) {                           // rows on the grid, whole vectors
        switch (p.width) {
            case 2: CC1D_LAUNCH((bwd_channelfirst_stream_kernel<DT, 2, false>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
            case 3: CC1D_LAUNCH((bwd_channelfirst_stream_kernel<DT, 3, false>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
            default: CC1D_LAUNCH((bwd_channelfirst_stream_kernel<DT, 4, false>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
        }
        return launch_status();
    }
    if (g.streaming == 2) {                           // rows anywhere on the grid
        switch (p.width) {
            case 2: CC1D_LAUNCH((bwd_channelfirst_stream_kernel<DT, 2, true>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
            case 3: CC1D_LAUNCH((bwd_channelfirst_stream_kernel<DT, 3, true>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
            default: CC1D_LAUNCH((bwd_channelfirst_stream_kernel<DT, 4, true>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
        }
        return launch_status();
    }
    switch (p.width) {
        case 2: CC1D_LAUNCH((bwd_channelfirst_kernel<DT, 2>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
        case 3: CC1D_LAUNCH((bwd_channelfirst_kernel<DT, 3>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
        default: CC1D_LAUNCH((bwd_channelfirst_kernel<DT, 4>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws); break;
    }
    return launch_status();
}

}  // namespace

// Rows of more than 64 vectors take the tile kernel (a forced number of parts keeps them on the
// walking kernels above).
static bool takes_tiles(const cc1d_bwd_params &p) {
    return tunables().bwd_cf_parts == 0 && bwd_channelfirst_tile_applies(p);
}

size_t bwd_channelfirst_workspace_bytes(const cc1d_bwd_params &p) {
    if (takes_tiles(p)) return (size_t)bwd_channelfirst_tile_parts(p) * (p.width + 1) * (size_t)p.dim * sizeof(float);
    const BwdCfGeom g = make_geom(p);
    if (g.n_parts == 1) return 0;
    return (size_t)g.n_parts * (p.width + 1) * (size_t)p.dim * sizeof(float);
}

bool bwd_channelfirst_fits(const cc1d_bwd_params &p) {
    if (takes_tiles(p)) return bwd_channelfirst_tile_fits(p);
    return (int64_t)p.dim * make_geom(p).n_parts < wave_limit();
}

int launch_bwd_channelfirst(const cc1d_bwd_params &p, void *workspace, hipStream_t stream) {
    float *ws = static_cast<float *>(workspace);
    if (takes_tiles(p)) {
        const int st = launch_bwd_channelfirst_tile(p, ws, stream);
        if (st != CC1D_OK) return st;
        return launch_bwd_finalize(ws, bwd_channelfirst_tile_parts(p), p, stream);
    }
    const BwdCfGeom g = make_geom(p);
    int st;
    switch (p.x_dtype) {
        case CC1D_F32: st = launch_dtype<CC1D_F32>(p, g, ws, stream); break;
        case CC1D_F16: st = launch_dtype<CC1D_F16>(p, g, ws, stream); break;
        default: st = launch_dtype<CC1D_BF16>(p, g, ws, stream); break;
    }
    if (st != CC1D_OK || g.n_parts == 1) return st;
    return launch_bwd_finalize(ws, g.n_parts, p, stream);
}

}  // namespace cc1d
