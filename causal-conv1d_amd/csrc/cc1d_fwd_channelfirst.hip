// Channel-first forward for gfx950: x is (batch, dim, seqlen) with unit stride along
// seqlen.  Takes over causal_conv1d_fwd_kernel and its launcher
// (csrc/causal_conv1d_fwd.cu:46-170 of the reference).
//
// Design.  One wavefront owns one segment of one (batch, channel) row and walks it in
// steps of 64 sixteen-byte vectors (1 KiB).  A lane's W-1 left neighbours come from the
// previous lane through a DPP wave shift; lane 0 takes them from lane 63 of the wave's
// previous step (v_readlane), so only a segment's very first step touches memory for
// its halo.  There is no LDS and no barrier, and rows are spread over
// (row x segment) waves instead of one serial loop per row.
//
// Rows need not be 16-byte aligned or a multiple of the vector length: lanes are laid
// out on the row's own 16-byte grid (`mis` = elements between that grid and the row
// start), vectors that stick out of [0, seqlen) are accessed element by element, and
// the same holds for `out` when its rows sit on a different grid than x's.
// initial_states / final_states are supported (the reference refuses them for this
// layout, csrc/causal_conv1d.cpp:213,228).
//
// Four kernels share this design.  The streaming kernel takes every launch in which the rows
// of out lie on the same 16-byte grid as the rows of x (same shape and strides, as
// empty_like gives): whole 64-vector steps run without bounds checks in two register sets in
// ping-pong, which keep the loads of the next two groups in flight while a group is computed
// and stored; what is left over at the end of a segment (fewer than a pair of groups, a partly
// filled step) is two more groups in the same ping-pong with every lane checked; rows of more than
// three steps start their steps on 128-byte lines of out, with a partly filled first step; and
// the few positions of a row in front of its first whole vector or behind its last one are
// produced one per lane, straight from memory.  The general kernel takes out tensors on a different grid.  The short-row
// kernel takes rows of at most 64 vectors, several rows to a wavefront and no walk; the flat
// kernel takes such rows of a contiguous tensor as whole vectors of one flat array.  Rows of
// more than 64 vectors that start on 128-byte lines (tensors of up to 512 MiB) or hold at most
// 128 vectors, and rows off the 16-byte grid of up to 512 vectors (192 of fp32), go to the tile
// kernel of cc1d_fwd_channelfirst_tile.hip (rows fetched straight into LDS; 1-25 % faster on
// lines, 10-40 % off the grid); the launch tunable fwd_cf_vecs = -1 keeps them here.
#include <type_traits>

#include "cc1d_device.hpp"
#include "cc1d_internal.hpp"

// Rows of more than three steps start their steps on 128-byte lines of out (one more, partly
// filled step per row); shorter rows start them at the row's first vector.  (8, 5376, L) bf16, steps
// at the first vector / on lines: L = 1000 32.7 / 38.3 us, 1500 54.7 / 57.3, 2000 62.6 / 57.0, 2400 72.2 / 66.0,
// 3000 101.7 / 84.3, 4080 151 / 133, 6000 200 / 177; fp32 L = 1000 64.7 / 56.6, 1500 103.3 / 83.8 us.
#ifndef CC1D_FWD_CF_ALIGN_MIN_VECS
#define CC1D_FWD_CF_ALIGN_MIN_VECS 193
#endif
#ifndef CC1D_FWD_CF_U2_STEPS
#define CC1D_FWD_CF_U2_STEPS 8
#endif

namespace cc1d {
namespace {

struct FwdCfGeom {
    int32_t streaming;        // steps per register set of the streaming kernel (1 or 2); 0: general kernel
    int32_t vecs_per_seg;     // multiple of 64
    int32_t n_segs;           // segments per row
    uint32_t total_waves;     // batch * dim * n_segs
    int32_t lead_vecs;        // streaming kernel: 7 = a row's steps start on 128-byte lines of out, 0 = at the row's first vector
};

// Row number of the launch -> (batch entry, channel).  Channels run fastest for tensors whose rows
// lie in (batch, dim) order in memory.  BATCH_INNER: for a (dim, batch, seqlen) tensor seen as
// (batch, dim, seqlen) -- Mamba's in_proj output, rearranged "d (b l) -> b d l" -- the batch
// entries of a channel are the neighbours in memory and run fastest instead, so that wavefronts
// that start together work side by side in memory: (32, 1536, 2048) bf16 84.2 -> 65.8 us,
// (8, 5120, 2048) bf16 62.5 -> 55.3 us, fp32 133.4 -> 109.0 us, (16, 5376, 128) bf16 12.1 -> 10.5 us.
// (A template parameter and not a flag: the flag cost two registers in every kernel, which took
// several of them over an occupancy step.)
template <bool BATCH_INNER>
__device__ __forceinline__ void row_to_batch_and_channel(const cc1d_fwd_params &p, uint32_t row, int &b, int &c) {
    if (BATCH_INNER) {
        b = (int)(row % (uint32_t)p.batch);
        c = (int)(row / (uint32_t)p.batch);
    } else {
        c = (int)(row % (uint32_t)p.dim);
        b = (int)(row / (uint32_t)p.dim);
    }
}

// Element t of the zero/initial-state padded row (fp32), for any t < L.
template <int DT, int W>
__device__ __forceinline__ float padded_elem(const cc1d_fwd_params &p, int64_t xrow, int b, int c,
                                             int t) {
    if (t >= 0) return ld_elem<DT>(p.x, xrow + t);
    if (p.initial_states != nullptr && t >= -(W - 1))
        return ld_elem<DT>(p.initial_states, (int64_t)b * p.init_stride_b +
                                                 (int64_t)c * p.init_stride_c +
                                                 (int64_t)(t + W - 1) * p.init_stride_l);
    return 0.f;
}

template <int DT, int W, bool BI>
__global__ void __launch_bounds__(kBlock)
fwd_channelfirst_kernel(const cc1d_fwd_params p, const FwdCfGeom g) {
    using E = Elem<DT>;
    constexpr int VEC = E::kVec;
    constexpr bool PRECISE = E::kPreciseAct;

    const uint32_t wid = (blockIdx.x * (uint32_t)kBlock + threadIdx.x) / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    if (wid >= g.total_waves) return;                 // whole wave leaves together
    const int seg = (int)(wid % (uint32_t)g.n_segs);
    const uint32_t row = wid / (uint32_t)g.n_segs;
    int b, c;
    row_to_batch_and_channel<BI>(p, row, b, c);
    const int L = p.seqlen;
    const bool silu_on = p.silu != 0;

    const int64_t xrow = (int64_t)b * p.x_stride_b + (int64_t)c * p.x_stride_c;
    const int64_t orow = (int64_t)b * p.out_stride_b + (int64_t)c * p.out_stride_c;
    using T = typename E::type;
    const int mis = (int)((reinterpret_cast<uintptr_t>(reinterpret_cast<const T *>(p.x) + xrow) /
                           sizeof(T)) % VEC);
    const int mis_o = (int)((reinterpret_cast<uintptr_t>(reinterpret_cast<T *>(p.out) + orow) /
                             sizeof(T)) % VEC);
    const bool out_same_grid = mis_o == mis;

    const int n_vecs = (L + mis + VEC - 1) / VEC;     // vectors of this row on its grid
    const int j_begin = seg * g.vecs_per_seg;
    int j_end = j_begin + g.vecs_per_seg;
    if (j_end > n_vecs) j_end = n_vecs;

    if (j_begin < j_end) {
        float wv[W], bias_v;
#pragma unroll
        for (int w = 0; w < W; ++w)
            wv[w] = ld_weight(p.weight, p.w_dtype, (int64_t)c * p.w_stride_c + w * p.w_stride_w);
        bias_v = p.bias == nullptr ? 0.f : ld_weight(p.bias, p.w_dtype, c);
        // The arithmetic of the other kernels, bit for bit: taps and bias carry the factor
        // -log2(e) where the activation takes the sums as its exponent (see silu_from_scaled).
        const bool scaled = silu_on && !PRECISE;
        if (scaled) {
            bias_v *= kSiluPrescale;
#pragma unroll
            for (int w = 0; w < W; ++w) wv[w] *= kSiluPrescale;
        }

        // Halo of the segment's first vector, wave-uniform.
        float carry[W - 1];
#pragma unroll
        for (int i = 0; i < W - 1; ++i)
            carry[i] = padded_elem<DT, W>(p, xrow, b, c, j_begin * VEC - mis - (W - 1) + i);

        auto load_step = [&](int j, float (&xf)[VEC]) {
            const int tf = j * VEC - mis;
            if (tf >= 0 && tf + VEC <= L) {
                E::unpack(ld_vec_nt<DT>(p.x, xrow + tf), xf);
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    xf[e] = (tf + e < L) ? padded_elem<DT, W>(p, xrow, b, c, tf + e) : 0.f;
            }
        };

        float nxt[VEC];
        load_step(j_begin + lane, nxt);
        for (int j0 = j_begin; j0 < j_end; j0 += kWave) {
            float xf[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) xf[e] = nxt[e];
            if (j0 + kWave < j_end) load_step(j0 + kWave + lane, nxt);   // prefetch

            // xx[i] = padded x at position tf - (W-1) + i
            float xx[VEC + W - 1];
#pragma unroll
            for (int i = 0; i < W - 1; ++i) {
                xx[i] = from_prev_lane(xf[VEC - (W - 1) + i], carry[i]);
                carry[i] = read_lane(xf[VEC - (W - 1) + i], kWave - 1);
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) xx[W - 1 + e] = xf[e];

            float acc[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float a = bias_v;
#pragma unroll
                for (int w = 0; w < W; ++w) a = fmaf(wv[w], xx[e + w], a);
                acc[e] = scaled ? silu_from_scaled(a) : silu_on ? silu<PRECISE>(a) : a;
            }

            const int j = j0 + lane;
            const int tf = j * VEC - mis;
            if (j < j_end) {
                if (out_same_grid && tf >= 0 && tf + VEC <= L) {
                    st_vec_nt<DT>(p.out, orow + tf, E::pack(acc));
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        if (tf + e >= 0 && tf + e < L) st_elem<DT>(p.out, orow + tf + e, acc[e]);
                }
            }
        }
    }

    // final_states[b, c, i] = xpad[L-(W-1)+i], bit-exact copies, by the row's first wave.
    if (p.final_states != nullptr && seg == 0 && lane < W - 1) {
        const int t = L - (W - 1) + lane;
        T v = T(0.f);
        if (t >= 0) {
            v = ld_raw<DT>(p.x, xrow + t);
        } else if (p.initial_states != nullptr) {
            v = ld_raw<DT>(p.initial_states, (int64_t)b * p.init_stride_b +
                                                 (int64_t)c * p.init_stride_c +
                                                 (int64_t)(t + W - 1) * p.init_stride_l);
        }
        st_raw<DT>(p.final_states, (int64_t)b * p.final_stride_b + (int64_t)c * p.final_stride_c +
                                       (int64_t)lane * p.final_stride_l, v);
    }
}

template <int DT, int W, bool SILU, int U, bool BI>
__global__ void __launch_bounds__(kBlock)
fwd_channelfirst_stream_kernel(const cc1d_fwd_params p, const FwdCfGeom g) {
    using E = Elem<DT>;
    using T = typename E::type;
    constexpr int VEC = E::kVec;
    constexpr bool PRECISE = E::kPreciseAct;
    // 16-bit outputs with SiLU: taps and bias carry the factor -log2(e), so the sums are
    // already the exponent the activation needs (see silu_from_scaled).
    constexpr bool SCALED = SILU && !PRECISE;

    const uint32_t wid = (blockIdx.x * (uint32_t)kBlock + threadIdx.x) / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    if (wid >= g.total_waves) return;                 // whole wave leaves together
    const int seg = (int)(wid % (uint32_t)g.n_segs);
    const uint32_t row = wid / (uint32_t)g.n_segs;
    int b, c;
    row_to_batch_and_channel<BI>(p, row, b, c);
    const int L = p.seqlen;

    const int64_t xrow = (int64_t)b * p.x_stride_b + (int64_t)c * p.x_stride_c;
    const T *xr = reinterpret_cast<const T *>(p.x) + xrow;
    T *orow = reinterpret_cast<T *>(p.out) + (int64_t)b * p.out_stride_b + (int64_t)c * p.out_stride_c;

    // The row on its own 16-byte grid (x and out share it), with the grid's origin moved back to
    // the 128-byte line of out that holds the row's first vector: vector j holds positions
    // j*VEC - mis .. j*VEC - mis + VEC, and a step of 64 vectors starts on a line.  (Steps that
    // start inside a line share a 64-byte block with the step before and the step after, and
    // blocks written in two parts are what such rows lose their time on: (8, 5376, 2000) bf16
    // 75.6 us against 60.7 us at seqlen 2048, (8, 5376, 4080) 167 against 116 us at 4096.)
    // Vectors jf0 .. jf1 lie inside the row and move as vectors; the up to VEC-1 positions in front
    // of them and behind them are edge positions, each produced by one lane straight from memory.
    const int mis0 = (int)((reinterpret_cast<uintptr_t>(xr) / sizeof(T)) % VEC);
    const int lead = g.lead_vecs == 0 ? 0 : (int)(((reinterpret_cast<uintptr_t>(orow) - (uintptr_t)mis0 * sizeof(T)) / 16) % 8);
    const int mis = mis0 + lead * VEC;                // elements between the grid's origin and the row start
    const int jf0 = (mis + VEC - 1) / VEC;            // 0 .. 8
    const int jf1 = (L + mis) / VEC;
    const int j0 = seg * g.vecs_per_seg;              // the segment's steps start here, on a line
    int j_begin = j0;
    int j_end = j_begin + g.vecs_per_seg;
    const bool owns_tail = j_begin <= jf1 && jf1 < j_end;
    if (j_begin < jf0) j_begin = jf0;
    if (j_end > jf1) j_end = jf1;
    // A first step whose leading lanes lie in front of the row's first whole vector (the row's
    // first segment, when the row does not start on a line) is done on its own, checked.
    const bool head = j_begin > j0 && j_begin < j_end;
    const int s_first = head ? 1 : 0;
    // whole groups of U steps, in pairs
    const int n_full = j_begin < j_end ? (j_end - j0) / kWave - s_first : 0;
    const int n_groups = n_full > 0 ? n_full / (2 * U) * 2 : 0;

    float wv[W], bias_v;
#pragma unroll
    for (int w = 0; w < W; ++w)
        wv[w] = ld_weight(p.weight, p.w_dtype, (int64_t)c * p.w_stride_c + w * p.w_stride_w);
    bias_v = p.bias == nullptr ? 0.f : ld_weight(p.bias, p.w_dtype, c);
    if (SCALED) {
        bias_v *= kSiluPrescale;
#pragma unroll
        for (int w = 0; w < W; ++w) wv[w] *= kSiluPrescale;
    }

    // Edge positions: [0, front) by lanes 0.. of the row's first wave, [back, L) by lanes VEC..
    // of the wave whose range holds vector jf1.  A row shorter than its first vector is all
    // front edge.
    {
        const int front = jf1 < jf0 ? L : jf0 * VEC - mis;
        const int back = jf1 < jf0 ? L : jf1 * VEC - mis;
        int t = -1;
        if (seg == 0 && lane < front) t = lane;
        if (owns_tail && lane >= VEC && lane - VEC < L - back) t = back + lane - VEC;
        if (t >= 0) {
            float a = bias_v;
#pragma unroll
            for (int w = 0; w < W; ++w) a = fmaf(wv[w], padded_elem<DT, W>(p, xrow, b, c, t - (W - 1) + w), a);
            a = SCALED ? silu_from_scaled(a) : SILU ? silu<PRECISE>(a) : a;
            orow[t] = E::from_float(a);
        }
    }

    if (j_begin < j_end) {
        // Halo of the segment's first vector, wave-uniform.
        float carry[W - 1];
#pragma unroll
        for (int i = 0; i < W - 1; ++i)
            carry[i] = padded_elem<DT, W>(p, xrow, b, c, j_begin * VEC - mis - (W - 1) + i);

        const T *xs = xr - mis + (j0 + s_first * kWave + lane) * VEC;    // this lane's vector of the first whole step
        T *os = orow - mis + (j0 + s_first * kWave + lane) * VEC;
        auto load_group = [&](int k, u32x4 (&raw)[U]) {
#pragma unroll
            for (int u = 0; u < U; ++u)
                raw[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(xs + (k * U + u) * (kWave * VEC)));
        };
        auto compute_group = [&](int k, const u32x4 (&raw)[U]) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float xf[VEC];
                E::unpack(raw[u], xf);
                // xx[i] = padded x at position tf - (W-1) + i
                float xx[VEC + W - 1];
#pragma unroll
                for (int i = 0; i < W - 1; ++i) {
                    xx[i] = from_prev_lane(xf[VEC - (W - 1) + i], carry[i]);
                    carry[i] = read_lane(xf[VEC - (W - 1) + i], kWave - 1);
                }
#pragma unroll
                for (int e = 0; e < VEC; ++e) xx[W - 1 + e] = xf[e];
                float acc[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float a = bias_v;
#pragma unroll
                    for (int w = 0; w < W; ++w) a = fmaf(wv[w], xx[e + w], a);
                    acc[e] = SCALED ? silu_from_scaled(a) : SILU ? silu<PRECISE>(a) : a;
                }
                __builtin_nontemporal_store(E::pack(acc), reinterpret_cast<u32x4 *>(os + (k * U + u) * (kWave * VEC)));
            }
        };

        // The checked first step's vector is requested first and the first two groups of whole
        // steps right behind it, so that its arithmetic runs while they are in flight.
        const int first = j_begin - j0;               // head: 1 .. 8
        const bool head_mine = head && lane >= first && j0 + lane < j_end;
        u32x4 head_raw = u32x4{0u, 0u, 0u, 0u};
        if (head_mine) head_raw = *reinterpret_cast<const u32x4 *>(xs - kWave * VEC);
        // Steps the whole pairs do not cover (fewer than 2 U whole ones and possibly a partly filled
        // one) are two more groups, requested and computed in the same ping-pong with every lane
        // checked: lanes past the segment's end read zeros and store nothing.  They use the
        // non-temporal policy of the whole steps: with plain accesses for them, (8, 5376, 2000) bf16
        // took 65.6 us against 58.3 us, (8, 5376, 3000) 100.0 against 84.5 us and fp32 (8, 5376, 1000)
        // 66.5 against 56.7 us.  (The checked first step keeps plain accesses: 58.3 against 60.2 us and
        // 84.5 against 92.2 us.)
        auto load_group_checked = [&](int k, u32x4 (&raw)[U]) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                raw[u] = u32x4{0u, 0u, 0u, 0u};
                if (j0 + (s_first + k * U + u) * kWave + lane < j_end)
                    raw[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(xs + (k * U + u) * (kWave * VEC)));
            }
        };
        auto compute_group_checked = [&](int k, const u32x4 (&raw)[U]) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (j0 + (s_first + k * U + u) * kWave >= j_end) break;       // wave-uniform
                const bool mine = j0 + (s_first + k * U + u) * kWave + lane < j_end;
                float xf[VEC];
                E::unpack(raw[u], xf);
                float xx[VEC + W - 1];
#pragma unroll
                for (int i = 0; i < W - 1; ++i) {
                    xx[i] = from_prev_lane(xf[VEC - (W - 1) + i], carry[i]);
                    carry[i] = read_lane(xf[VEC - (W - 1) + i], kWave - 1);
                }
#pragma unroll
                for (int e = 0; e < VEC; ++e) xx[W - 1 + e] = xf[e];
                float acc[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float a = bias_v;
#pragma unroll
                    for (int w = 0; w < W; ++w) a = fmaf(wv[w], xx[e + w], a);
                    acc[e] = SCALED ? silu_from_scaled(a) : SILU ? silu<PRECISE>(a) : a;
                }
                if (mine) __builtin_nontemporal_store(E::pack(acc), reinterpret_cast<u32x4 *>(os + (k * U + u) * (kWave * VEC)));
            }
        };
        u32x4 ra[U], rb[U];
        if (n_groups >= 2) {
            load_group(0, ra);
            load_group(1, rb);
        } else {
            load_group_checked(0, ra);
            load_group_checked(1, rb);
        }
        if (head) {
            // Lanes in front of the row's first whole vector load and store nothing; the one right
            // in front of it hands the halo on.
            float xf[VEC];
            E::unpack(head_raw, xf);
            float xx[VEC + W - 1];
#pragma unroll
            for (int i = 0; i < W - 1; ++i) {
                const float top = lane == first - 1 ? carry[i] : xf[VEC - (W - 1) + i];
                xx[i] = from_prev_lane(top, 0.f);
                carry[i] = read_lane(xf[VEC - (W - 1) + i], kWave - 1);
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) xx[W - 1 + e] = xf[e];
            float acc[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float a = bias_v;
#pragma unroll
                for (int w = 0; w < W; ++w) a = fmaf(wv[w], xx[e + w], a);
                acc[e] = SCALED ? silu_from_scaled(a) : SILU ? silu<PRECISE>(a) : a;
            }
            if (head_mine) *reinterpret_cast<u32x4 *>(os - kWave * VEC) = E::pack(acc);
        }

        // Two register sets of U steps in ping-pong: while one group is computed and stored the
        // loads of the next two are in flight.  The whole groups (an even number) come first,
        // unchecked; the two checked groups close the walk in the same rhythm.
        int k = 0;
        if (n_groups >= 2) {
#pragma clang loop unroll(disable)
            for (; k + 2 < n_groups; k += 2) {
                compute_group(k, ra);
                load_group(k + 2, ra);
                compute_group(k + 1, rb);
                load_group(k + 3, rb);
            }
            compute_group(k, ra);
            load_group_checked(k + 2, ra);
            compute_group(k + 1, rb);
            load_group_checked(k + 3, rb);
            k += 2;
        }
        compute_group_checked(k, ra);
        compute_group_checked(k + 1, rb);
    }

    // final_states[b, c, i] = xpad[L-(W-1)+i], bit-exact copies, by the row's first wave.
    if (p.final_states != nullptr && seg == 0 && lane < W - 1) {
        const int t = L - (W - 1) + lane;
        T v = T(0.f);
        if (t >= 0) {
            v = ld_raw<DT>(p.x, xrow + t);
        } else if (p.initial_states != nullptr) {
            v = ld_raw<DT>(p.initial_states, (int64_t)b * p.init_stride_b +
                                                 (int64_t)c * p.init_stride_c +
                                                 (int64_t)(t + W - 1) * p.init_stride_l);
        }
        st_raw<DT>(p.final_states, (int64_t)b * p.final_stride_b + (int64_t)c * p.final_stride_c +
                                       (int64_t)lane * p.final_stride_l, v);
    }
}

// Rows of at most 64 vectors.  One wavefront per row would leave most of its lanes idle, so a
// wavefront takes 64 / G rows at once, G = 1, 2, 4 ... 64 lanes each (ALIGNED: whole vectors on the
// 16-byte grid): lane (row, v) owns vector v of its row, takes its left halo from the previous lane through the same
// DPP shift as the walk (vector 0 takes zeros or initial_states instead), and the whole launch is
// one load and one store per lane.  Same arithmetic, in the same order, as the other kernels.
// ALIGNED = false: rows of any length up to 64 vectors, anywhere in memory (a contiguous tensor
// whose seqlen is no multiple of the vector length, down to seqlen 1): the same lanes, with a
// lane's up to VEC positions read and written element by element.
template <int DT, int W, bool SILU, bool ALIGNED, bool BI>
__global__ void __launch_bounds__(kBlock)
fwd_channelfirst_short_kernel(const cc1d_fwd_params p, const int n_vecs, const int lanes_log2, const uint32_t n_rows) {
    using E = Elem<DT>;
    using T = typename E::type;
    constexpr int VEC = E::kVec;
    constexpr bool PRECISE = E::kPreciseAct;
    constexpr bool SCALED = SILU && !PRECISE;

    const uint32_t gid = blockIdx.x * (uint32_t)kBlock + threadIdx.x;
    const uint32_t row_here = gid >> lanes_log2;
    const int v = (int)(gid & ((1u << lanes_log2) - 1u));
    // Lanes without a vector of their own stay in step (the lane shift below needs every lane)
    // on row 0's addresses; they load and store nothing.
    const bool mine = row_here < n_rows && v < n_vecs;
    const uint32_t row = mine ? row_here : 0u;
    int b, c;
    row_to_batch_and_channel<BI>(p, row, b, c);
    const int64_t xrow = (int64_t)b * p.x_stride_b + (int64_t)c * p.x_stride_c;
    const int64_t orow = (int64_t)b * p.out_stride_b + (int64_t)c * p.out_stride_c;

    const int L = p.seqlen;
    u32x4 raw = u32x4{0u, 0u, 0u, 0u};
    if (ALIGNED) {
        if (mine) raw = ld_vec_nt<DT>(p.x, xrow + (int64_t)v * VEC);
    } else {
        T elems[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) elems[e] = T(0.f);
        if (mine) {
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                if (v * VEC + e < L) elems[e] = ld_raw<DT>(p.x, xrow + v * VEC + e);
        }
        __builtin_memcpy(&raw, elems, sizeof raw);
    }
    float wv[W], bias_v;
#pragma unroll
    for (int w = 0; w < W; ++w)
        wv[w] = ld_weight(p.weight, p.w_dtype, (int64_t)c * p.w_stride_c + w * p.w_stride_w);
    bias_v = p.bias == nullptr ? 0.f : ld_weight(p.bias, p.w_dtype, c);
    float halo[W - 1];
#pragma unroll
    for (int i = 0; i < W - 1; ++i) halo[i] = 0.f;
    if (mine && v == 0 && p.initial_states != nullptr) {
#pragma unroll
        for (int i = 0; i < W - 1; ++i) halo[i] = padded_elem<DT, W>(p, xrow, b, c, i - (W - 1));
    }
    if (SCALED) {
        bias_v *= kSiluPrescale;
#pragma unroll
        for (int w = 0; w < W; ++w) wv[w] *= kSiluPrescale;
    }

    float xf[VEC];
    E::unpack(raw, xf);
    float xx[VEC + W - 1];
#pragma unroll
    for (int i = 0; i < W - 1; ++i) {
        const float prev = from_prev_lane(xf[VEC - (W - 1) + i], 0.f);
        xx[i] = v == 0 ? halo[i] : prev;
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) xx[W - 1 + e] = xf[e];
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        float a = bias_v;
#pragma unroll
        for (int w = 0; w < W; ++w) a = fmaf(wv[w], xx[e + w], a);
        acc[e] = SCALED ? silu_from_scaled(a) : SILU ? silu<PRECISE>(a) : a;
    }
    if (ALIGNED) {
        if (mine) st_vec_nt<DT>(p.out, orow + (int64_t)v * VEC, E::pack(acc));
    } else if (mine) {
#pragma unroll
        for (int e = 0; e < VEC; ++e)
            if (v * VEC + e < L) st_elem<DT>(p.out, orow + v * VEC + e, acc[e]);
    }

    // final_states[b, c, i] = xpad[L-(W-1)+i], bit-exact copies (from initial_states or zero where
    // the row is shorter than W-1), by the lane that owns the row's last vector.
    if (p.final_states != nullptr && mine && v == n_vecs - 1) {
#pragma unroll
        for (int i = 0; i < W - 1; ++i) {
            const int t = L - (W - 1) + i;
            T e = T(0.f);
            if (t >= 0) {
                e = ld_raw<DT>(p.x, xrow + t);
            } else if (p.initial_states != nullptr) {
                e = ld_raw<DT>(p.initial_states, (int64_t)b * p.init_stride_b + (int64_t)c * p.init_stride_c +
                                                     (int64_t)(t + W - 1) * p.init_stride_l);
            }
            st_raw<DT>(p.final_states, (int64_t)b * p.final_stride_b + (int64_t)c * p.final_stride_c +
                                           (int64_t)i * p.final_stride_l, e);
        }
    }
}

// The rows of one channel's batch entries lie closer together in memory than those of one batch
// entry's channels.
bool batch_entries_are_neighbours(const cc1d_fwd_params &p) {
    return p.batch > 1 && p.dim > 1 && p.x_stride_b < p.x_stride_c;
}

template <int DT>
int launch_short(const cc1d_fwd_params &p, int n_vecs, bool aligned, hipStream_t stream) {
    int lanes_log2 = 0;
    while ((1 << lanes_log2) < n_vecs) ++lanes_log2;
    const int64_t rows = (int64_t)p.batch * p.dim;
    const int64_t threads = rows << lanes_log2;
    if (threads >= thread_limit()) return CC1D_ERR_TOO_LARGE;
    const dim3 grid((uint32_t)((threads + kBlock - 1) / kBlock)), block(kBlock);
    const uint32_t n_rows = (uint32_t)rows;
    const bool batch_inner = batch_entries_are_neighbours(p);
#define CC1D_SHORT3(WIDTH, SILU_ON, BI_ON)                                                                           \
    if (aligned) CC1D_LAUNCH((fwd_channelfirst_short_kernel<DT, WIDTH, SILU_ON, true, BI_ON>), grid, block, 0, \
                                    stream, p, n_vecs, lanes_log2, n_rows);                                           \
    else CC1D_LAUNCH((fwd_channelfirst_short_kernel<DT, WIDTH, SILU_ON, false, BI_ON>), grid, block, 0,       \
                            stream, p, n_vecs, lanes_log2, n_rows)
#define CC1D_SHORT2(WIDTH, SILU_ON)                                                                                  \
    if (batch_inner) { CC1D_SHORT3(WIDTH, SILU_ON, true); } else { CC1D_SHORT3(WIDTH, SILU_ON, false); }
#define CC1D_SHORT(WIDTH)                                                                                             \
    if (p.silu) { CC1D_SHORT2(WIDTH, true); } else { CC1D_SHORT2(WIDTH, false); }
    switch (p.width) {
        case 2: CC1D_SHORT(2); break;
        case 3: CC1D_SHORT(3); break;
        default: CC1D_SHORT(4); break;
    }
#undef CC1D_SHORT
#undef CC1D_SHORT2
#undef CC1D_SHORT3
    return launch_status();
}

// Short rows of a contiguous tensor whose seqlen is no multiple of the vector length (at least
// one vector, at most 64): rows then start anywhere on the 16-byte grid, but batch * dim * seqlen
// elements lie back to back, so a lane owns one whole vector of that flat array: one 16-byte load
// and one 16-byte store, as in the short-row kernel, where element accesses would take VEC of each.
// A vector spans at most two rows; the lane holds the taps of both, takes its left neighbours from
// the previous lane (lane 0 of a wavefront from memory) and masks the taps that reach in front of
// a row's start (or takes initial_states there).  Same arithmetic, in the same order, as the
// other kernels.
template <int DT, int W, bool SILU, bool PACKED_W>
__global__ void __launch_bounds__(kBlock)
fwd_channelfirst_flat_kernel(const cc1d_fwd_params p, const uint32_t n_elems) {
    using E = Elem<DT>;
    using T = typename E::type;
    constexpr int VEC = E::kVec;
    constexpr bool PRECISE = E::kPreciseAct;
    constexpr bool SCALED = SILU && !PRECISE;

    const uint32_t gid = blockIdx.x * (uint32_t)kBlock + threadIdx.x;
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t L = (uint32_t)p.seqlen, D = (uint32_t)p.dim;
    // Lanes past the end stay in step (the lane shift needs every lane) on vector 0.
    const bool mine = (uint64_t)gid * VEC < n_elems;
    const uint32_t f0 = mine ? gid * VEC : 0u;
    const bool whole = f0 + VEC <= n_elems;           // only the array's last vector can be partial

    u32x4 raw = u32x4{0u, 0u, 0u, 0u};
    if (mine) {
        if (whole) {
            raw = ld_vec_nt<DT>(p.x, f0);
        } else {
            T elems[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) elems[e] = f0 + e < n_elems ? ld_raw<DT>(p.x, f0 + e) : T(0.f);
            __builtin_memcpy(&raw, elems, sizeof raw);
        }
    }
    const uint32_t row0 = f0 / L;
    const uint32_t t0 = f0 - row0 * L;
    const uint32_t split = L - t0;                    // elements [split, VEC) belong to the next row
    const uint32_t c0 = row0 % D, b0 = row0 / D;
    const bool wrap = c0 + 1 == D;
    const uint32_t c1 = wrap ? 0u : c0 + 1, b1 = wrap ? b0 + 1 : b0;

    // Taps of the row the vector starts in, and of the next one only where the vector reaches it
    // (one lane in seqlen / VEC).  Packed fp32 taps (a host-checked promise: strides (W, 1), base
    // 16-byte aligned) of even width come in one load.
    float w0[W], w1[W], bias0, bias1 = 0.f;
    auto taps = [&](uint32_t c, float (&wv)[W]) {
        if (PACKED_W && W % 2 == 0) {
            const float *src = static_cast<const float *>(__builtin_assume_aligned(
                reinterpret_cast<const float *>(p.weight) + (int64_t)c * W, W % 2 == 0 ? W * 4 : 4));
#pragma unroll
            for (int w = 0; w < W; ++w) wv[w] = src[w];
        } else {
#pragma unroll
            for (int w = 0; w < W; ++w)
                wv[w] = ld_weight(p.weight, p.w_dtype, (int64_t)c * p.w_stride_c + w * p.w_stride_w);
        }
    };
    taps(c0, w0);
    bias0 = p.bias == nullptr ? 0.f : ld_weight(p.bias, p.w_dtype, c0);
#pragma unroll
    for (int w = 0; w < W; ++w) w1[w] = 0.f;
    if (split < (uint32_t)VEC) {
        taps(c1, w1);
        bias1 = p.bias == nullptr ? 0.f : ld_weight(p.bias, p.w_dtype, c1);
    }
    if (SCALED) {
        bias0 *= kSiluPrescale;
        bias1 *= kSiluPrescale;
#pragma unroll
        for (int w = 0; w < W; ++w) { w0[w] *= kSiluPrescale; w1[w] *= kSiluPrescale; }
    }

    float xf[VEC];
    E::unpack(raw, xf);
    // xx[i] = flat element f0-(W-1)+i
    float xx[VEC + W - 1];
    float first[W - 1];
#pragma unroll
    for (int i = 0; i < W - 1; ++i) first[i] = 0.f;
    if (lane == 0 && f0 >= (uint32_t)(W - 1)) {
#pragma unroll
        for (int i = 0; i < W - 1; ++i) first[i] = ld_elem<DT>(p.x, (int64_t)f0 - (W - 1) + i);
    }
#pragma unroll
    for (int i = 0; i < W - 1; ++i) xx[i] = from_prev_lane(xf[VEC - (W - 1) + i], first[i]);
#pragma unroll
    for (int e = 0; e < VEC; ++e) xx[W - 1 + e] = xf[e];

    const bool has_init = p.initial_states != nullptr;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        const bool next = (uint32_t)e >= split;
        const uint32_t t = next ? (uint32_t)e - split : t0 + (uint32_t)e;
        float a = next ? bias1 : bias0;
#pragma unroll
        for (int w = 0; w < W; ++w) {
            // tap w reads position t-(W-1-w) of the row
            float xv = xx[e + w];
            if (w < W - 1 && t + (uint32_t)w < (uint32_t)(W - 1)) {
                xv = 0.f;
                if (has_init && f0 + e < n_elems)     // (positions past the array's end belong to no row)
                    xv = ld_elem<DT>(p.initial_states, (int64_t)(next ? b1 : b0) * p.init_stride_b +
                                                           (int64_t)(next ? c1 : c0) * p.init_stride_c +
                                                           (int64_t)(t + w) * p.init_stride_l);
            }
            a = fmaf(next ? w1[w] : w0[w], xv, a);
        }
        acc[e] = SCALED ? silu_from_scaled(a) : SILU ? silu<PRECISE>(a) : a;
    }
    if (mine) {
        if (whole) {
            st_vec_nt<DT>(p.out, f0, E::pack(acc));
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                if (f0 + e < n_elems) st_elem<DT>(p.out, f0 + e, acc[e]);
        }
    }

    // final_states[b, c, i] = x[L-(W-1)+i] (a row is never shorter than a vector, so never
    // shorter than W-1), bit-exact copies, by the lane whose vector holds the row's last element.
    if (p.final_states != nullptr && mine && split <= (uint32_t)VEC && f0 + split <= n_elems) {
#pragma unroll
        for (int i = 0; i < W - 1; ++i) {
            const T e = ld_raw<DT>(p.x, (int64_t)f0 + split - (W - 1) + i);
            st_raw<DT>(p.final_states, (int64_t)b0 * p.final_stride_b + (int64_t)c0 * p.final_stride_c +
                                           (int64_t)i * p.final_stride_l, e);
        }
    }
}

template <int DT>
int launch_flat(const cc1d_fwd_params &p, hipStream_t stream) {
    constexpr int VEC = Elem<DT>::kVec;
    const uint32_t n_elems = (uint32_t)((int64_t)p.batch * p.dim * p.seqlen);
    const uint32_t n_vecs = (n_elems + VEC - 1) / VEC;
    const dim3 grid((n_vecs + kBlock - 1) / kBlock), block(kBlock);
    const bool packed = weights_contiguous_f32(p.weight, p.w_dtype, p.w_stride_c, p.w_stride_w, p.width);
#define CC1D_FLAT2(WIDTH, SILU_ON)                                                                                    \
    if (packed) CC1D_LAUNCH((fwd_channelfirst_flat_kernel<DT, WIDTH, SILU_ON, true>), grid, block, 0, stream,  \
                                   p, n_elems);                                                                       \
    else CC1D_LAUNCH((fwd_channelfirst_flat_kernel<DT, WIDTH, SILU_ON, false>), grid, block, 0, stream, p,     \
                            n_elems)
#define CC1D_FLAT(WIDTH)                                                                                              \
    if (p.silu) { CC1D_FLAT2(WIDTH, true); } else { CC1D_FLAT2(WIDTH, false); }
    switch (p.width) {
        case 2: CC1D_FLAT(2); break;
        case 3: CC1D_FLAT(3); break;
        default: CC1D_FLAT(4); break;
    }
#undef CC1D_FLAT
#undef CC1D_FLAT2
    return launch_status();
}

template <int DT, bool SILU, int U, bool BI>
int launch_stream(const cc1d_fwd_params &p, const FwdCfGeom &g, hipStream_t stream) {
    const uint32_t blocks = (g.total_waves + (kBlock / kWave) - 1) / (kBlock / kWave);
    switch (p.width) {
        case 2: CC1D_LAUNCH((fwd_channelfirst_stream_kernel<DT, 2, SILU, U, BI>), dim3(blocks), dim3(kBlock), 0, stream, p, g); break;
        case 3: CC1D_LAUNCH((fwd_channelfirst_stream_kernel<DT, 3, SILU, U, BI>), dim3(blocks), dim3(kBlock), 0, stream, p, g); break;
        default: CC1D_LAUNCH((fwd_channelfirst_stream_kernel<DT, 4, SILU, U, BI>), dim3(blocks), dim3(kBlock), 0, stream, p, g); break;
    }
    return launch_status();
}

template <int DT, bool BI>
int launch_order(const cc1d_fwd_params &p, const FwdCfGeom &g, hipStream_t stream) {
    if (g.streaming == 2) return p.silu ? launch_stream<DT, true, 2, BI>(p, g, stream) : launch_stream<DT, false, 2, BI>(p, g, stream);
    if (g.streaming == 1) return p.silu ? launch_stream<DT, true, 1, BI>(p, g, stream) : launch_stream<DT, false, 1, BI>(p, g, stream);
    const uint32_t blocks = (g.total_waves + (kBlock / kWave) - 1) / (kBlock / kWave);
    switch (p.width) {
        case 2: CC1D_LAUNCH((fwd_channelfirst_kernel<DT, 2, BI>), dim3(blocks), dim3(kBlock), 0, stream, p, g); break;
        case 3: CC1D_LAUNCH((fwd_channelfirst_kernel<DT, 3, BI>), dim3(blocks), dim3(kBlock), 0, stream, p, g); break;
        default: CC1D_LAUNCH((fwd_channelfirst_kernel<DT, 4, BI>), dim3(blocks), dim3(kBlock), 0, stream, p, g); break;
    }
    return launch_status();
}

template <int DT>
int launch_dtype(const cc1d_fwd_params &p, const FwdCfGeom &g, hipStream_t stream) {
    return batch_entries_are_neighbours(p) ? launch_order<DT, true>(p, g, stream) : launch_order<DT, false>(p, g, stream);
}

}  // namespace

int launch_fwd_channelfirst(const cc1d_fwd_params &p, hipStream_t stream) {
    // Rows a little longer than the short-row kernel takes, and longer rows off the 16-byte grid:
    // tile wavefronts (a forced segment length keeps such tensors on the walking kernels below).
    if (tunables().fwd_cf_vecs == 0 && fwd_channelfirst_tile_applies(p)) return launch_fwd_channelfirst_tile(p, stream);
    const int vec = vec_elems(p.x_dtype);
    // The streaming kernel needs every row of out on the 16-byte grid of the same row of x;
    // steps per register set: two once a row has at least eight steps.
    const int eb = elem_bytes(p.x_dtype);
    const bool same_grid = (reinterpret_cast<uintptr_t>(p.x) - reinterpret_cast<uintptr_t>(p.out)) % 16 == 0 &&
                           reinterpret_cast<uintptr_t>(p.x) % eb == 0 &&
                           (p.x_stride_b - p.out_stride_b) % vec == 0 && (p.x_stride_c - p.out_stride_c) % vec == 0;
    const int streaming = !same_grid ? 0 : p.seqlen >= CC1D_FWD_CF_U2_STEPS * kWave * vec ? 2 : 1;
    // Vectors a row can span on its grid: exact when every row starts on the grid, else the
    // worst case (a row may start up to vec-1 elements into its first vector).
    const bool on_grid = aligned16(p.x) && p.x_stride_b % vec == 0 && p.x_stride_c % vec == 0;
    // The streaming kernel moves a row's grid back to the 128-byte line of out its first vector
    // lies in: up to seven more vectors, unless every row of out starts on a line.
    const bool rows_on_lines = on_grid && reinterpret_cast<uintptr_t>(p.out) % 128 == 0 &&
                               (p.out_stride_b * eb) % 128 == 0 && (p.out_stride_c * eb) % 128 == 0;
    const bool align_steps = streaming && !rows_on_lines && ((int64_t)p.seqlen + vec - 1) / vec >= CC1D_FWD_CF_ALIGN_MIN_VECS;
    const int64_t lead_max = align_steps ? 7 * vec : 0;
    const int64_t max_vecs = ((int64_t)p.seqlen + vec - 1 + lead_max + (on_grid && streaming ? 0 : vec - 1)) / vec;
    const int64_t rows = (int64_t)p.batch * p.dim;
    // Short rows of whole vectors, up to eight to a wavefront, no walk: (4, 5376, 256) bf16 11.2 -> 6.0 us,
    // (8, 1024, 512) bf16 6.7 -> 4.8 us, (4, 5376, 256) fp32 10.9 -> 8.5 us, (1, 5376, 64) bf16 4.8 -> 3.3 us.
    // Rows that are not whole vectors on one grid take the same lanes with element accesses:
    // (16, 5376, 100) bf16 45.9 -> 25.4 us, (64, 2048, 60) 63.7 -> 16.4 us, (256, 5376, 4) 360 -> 11.9 us.
    const int64_t short_vecs = ((int64_t)p.seqlen + vec - 1) / vec;
    const int32_t forced_vecs = tunables().fwd_cf_vecs;
    if (short_vecs <= 64 && forced_vecs <= 0) {
        const bool aligned = same_grid && on_grid && p.seqlen % vec == 0;
        // A contiguous tensor of rows that are not whole vectors, but at least one: whole vectors of
        // the flat array, (16, 5376, 100) bf16 25.4 -> 13.5 us, (16, 5376, 130) 28.5 -> 16.2 us, (64, 2048, 60) 16.4 -> 11.6 us.
        const int64_t n_elems = rows * p.seqlen;
        // (Not when final_states may be the buffer initial_states come from: in the flat walk the
        // lane that reads a row's initial_states and the lane that writes its final_states can sit in
        // different wavefronts.)
        const bool states_in_and_out = p.initial_states != nullptr && p.final_states != nullptr;
        const bool flat = !aligned && !states_in_and_out && p.seqlen >= vec && n_elems < thread_limit() &&
                          aligned16(p.x) && aligned16(p.out) &&
                          (p.dim == 1 || (p.x_stride_c == p.seqlen && p.out_stride_c == p.seqlen)) &&
                          (p.batch == 1 || (p.x_stride_b == (int64_t)p.dim * p.seqlen &&
                                            p.out_stride_b == (int64_t)p.dim * p.seqlen));
        if (flat) {
            switch (p.x_dtype) {
                case CC1D_F32: return launch_flat<CC1D_F32>(p, stream);
                case CC1D_F16: return launch_flat<CC1D_F16>(p, stream);
                default: return launch_flat<CC1D_BF16>(p, stream);
            }
        }
        switch (p.x_dtype) {
            case CC1D_F32: return launch_short<CC1D_F32>(p, (int)short_vecs, aligned, stream);
            case CC1D_F16: return launch_short<CC1D_F16>(p, (int)short_vecs, aligned, stream);
            default: return launch_short<CC1D_BF16>(p, (int)short_vecs, aligned, stream);
        }
    }
    int64_t vps;
    if (forced_vecs > 0) {
        vps = forced_vecs;
    } else {
        // Enough waves to cover 256 CUs about 16 deep; otherwise one wave per row, except that
        // long rows (1024 vectors and up) are cut into segments of 256 vectors: many short-lived
        // waves spread more evenly over the CUs than few that live as long as the launch
        // (47.8 -> 43.8 us for fp32 (4, 2048, 4096), 51.2 -> 44.7 us for bf16 (2, 2048, 16384);
        // rows of 512 vectors and less measured better in one piece).
        int64_t want_segs = rows >= 4096 ? 1 : (4096 + rows - 1) / rows;
        if (max_vecs >= 1024 && want_segs < max_vecs / 256) want_segs = max_vecs / 256;
        vps = (max_vecs + want_segs - 1) / want_segs;
    }
    const int64_t quantum = streaming ? 2 * streaming * kWave : kWave;   // whole steps / group pairs
    vps = (vps + quantum - 1) / quantum * quantum;
    if (vps < quantum) vps = quantum;
    FwdCfGeom g;
    g.streaming = streaming;
    g.lead_vecs = align_steps ? 7 : 0;
    g.vecs_per_seg = (int32_t)vps;
    g.n_segs = (int32_t)((max_vecs + vps - 1) / vps);
    const int64_t total = rows * g.n_segs;
    if (total >= wave_limit()) return CC1D_ERR_TOO_LARGE;   // total*64 threads must fit 2^31
    g.total_waves = (uint32_t)total;
    switch (p.x_dtype) {
        case CC1D_F32: return launch_dtype<CC1D_F32>(p, g, stream);
        case CC1D_F16: return launch_dtype<CC1D_F16>(p, g, stream);
        default: return launch_dtype<CC1D_BF16>(p, g, stream);
    }
}

}  // namespace cc1d
