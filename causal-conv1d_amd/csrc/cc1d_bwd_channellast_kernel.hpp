// Kernel of the channel-last backward and its launch templates, shared by the translation units
// that instantiate it: cc1d_bwd_channellast.hip (fp32, geometry, second stage),
// cc1d_bwd_channellast_lanes4.hip and cc1d_bwd_channellast_lanes8.hip (16-bit data with 4- and
// 8-byte lanes).  One source file for all of them took the compiler as long as the rest of the
// library together.
//
// Channel-last backward for gfx950.  Takes over causal_conv1d_channellast_bwd_kernel and
// its launcher (csrc/causal_conv1d_bwd.cu:329-632 of the reference) and the host-side
// deterministic finish (csrc/causal_conv1d.cpp:450-462).
//
//   z[t]  = bias + sum_w weight[w] * xpad[t-(W-1-w)]          (recomputed, never stored)
//   g[t]  = dout[t] * act'(z[t])                              (0 where seq_idx[t] < 0)
//   dx[p] = sum_k weight[W-1-k] * g[p+k]  (+ dfinal_states[p-(L-(W-1))] for p >= L-(W-1))
//   dinitial_states[i] = the same expression at p = i-(W-1) < 0
//   dweight[w] += sum_{b,t} g[t] * xpad[t-(W-1-w)],   dbias += sum_{b,t} g[t]
// with every tap additionally masked by seq_idx equality when seq_idx is given.
//
// Design.  Same geometry as the channel-last forward: a lane owns CH adjacent channels
// (one 4- or 8-byte vector) and walks a run of T rows in ascending order, holding (W-1)-row
// sliding windows of x and g in registers.  The run owns g[t] (hence the dweight/dbias
// terms) for its rows t in [t0, t1) and emits dx one window late: row t completes
// dx[t-(W-1)], so the run writes dx[t0-(W-1) .. t1-(W-1)).  Everything a run needs from
// its neighbour is therefore in front of it (2(W-1) rows of x, W-1 rows of dout, loaded
// once before the walk and found in L2, see the forward kernel), and the walk itself is
// uniform: two loads, one store and the same arithmetic for every row, no branch.  The last
// run of a sequence adds the W-1 closing rows, run 0 routes rows in front of the sequence
// to dinitial_states.  A lane's dweight/dbias partial sums stay in registers for the whole
// run (no cross-lane reduction, no atomics).  The four wavefronts of a workgroup take four
// consecutive runs of the same columns; their partial sums are added through LDS in the order
// of the runs and stored as one workspace plane, and a second kernel adds the planes up in a
// fixed order: results are bit-reproducible.
#pragma once
#include <type_traits>

#include "cc1d_device.hpp"
#include "cc1d_internal.hpp"

// Rows per register set; two sets are in flight per lane.
#ifndef CC1D_BWD_CL_UNROLL
#define CC1D_BWD_CL_UNROLL 4
#endif
#ifndef CC1D_BWD_CL_OCC8
#define CC1D_BWD_CL_OCC8 2
#endif
#ifndef CC1D_BWD_CL_STREAM_STORES
#define CC1D_BWD_CL_STREAM_STORES 1
#endif
// Workgroups per CU the register budget must allow.
#ifndef CC1D_BWD_CL_OCC
#define CC1D_BWD_CL_OCC 4
#endif

namespace cc1d {

struct BwdClGeom {
    int32_t rows_per_run;     // T, a multiple of twice the unroll factor
    int32_t n_runs;           // ceil(seqlen / T)
    int32_t n_quads;          // ceil(n_runs / 4): workgroups along one sequence
    int32_t n_colgroups;      // dim / CH
    uint32_t waves_per_row;   // ceil(n_colgroups / 64): workgroups side by side on one row
    uint32_t total;           // batch * n_quads * waves_per_row workgroups
    uint32_t blocks_per_xcd;  // grid size / 8
    uint32_t blocks_per_chunk; // workgroups an XCD takes in a row before the next XCD's (0: its whole slice)
    int32_t w_mode;           // weights_mode: 0 general loader, 1 / 2 packed taps
    int32_t channels_per_lane;
};

// Channels per lane for 16-bit tensors: 2, i.e. 4-byte lanes.  A lane's windows, taps and
// partial sums then fit 128 registers and four workgroups share a CU, which is worth more to
// this VALU-heavy kernel than wider accesses: 92 us against 102 us with 8-byte lanes and two
// workgroups per CU at (8, 5376, 2048) bf16.  fp32 keeps 2 channels (8 bytes).
#ifndef CC1D_BWD_CL_CH16
#define CC1D_BWD_CL_CH16 2
#endif

// The 16-bit instantiations, one translation unit each: 2 channels (4 bytes) per lane, and 4
// channels (8 bytes) per lane.
int launch_bwd_channellast_16bit_lanes4(const cc1d_bwd_params &p, const BwdClGeom &g, float *ws, hipStream_t stream);
int launch_bwd_channellast_16bit_lanes8(const cc1d_bwd_params &p, const BwdClGeom &g, float *ws, hipStream_t stream);

namespace {

constexpr int kXcds = 8;

constexpr int kRunsPerBlock = kBlock / kWave;   // the wavefronts of a workgroup take consecutive runs

// One wavefront's walk over run `run` of sequence b, columns col*CH .. col*CH+CH per lane: writes
// dx (and dinitial_states) and returns the lane's dweight / dbias terms in dW / dB.
template <int DT, int CH, int W, bool HAS_SEQ, bool SILU, int U, int WM>
__device__ __forceinline__ void
bwd_channellast_run(const cc1d_bwd_params &p, const BwdClGeom &g, const int32_t *__restrict__ seq_idx,
                    const int b, const int run, const uint32_t col, float (&dW)[CH][W], float (&dB)[CH]) {
    using E = Elem<DT>;
    using T_ = typename E::type;
    using P = Pack<DT, CH>;
    using raw_t = typename P::raw_t;
    constexpr bool PRECISE = E::kPreciseAct;
    constexpr bool SCALED = SILU && !PRECISE;         // taps, bias and g carry the factor of the SiLU exponent

    const int c0 = (int)col * CH;
    const int L = p.seqlen;
    const int T = g.rows_per_run;
    const int t0 = run * T;                           // < L by construction of n_runs
    const bool full = t0 + T <= L;                    // the run lies inside the sequence
    const int last = full ? T - 1 : L - 1 - t0;       // last row of this run, run-relative

    // Packed taps are only requested here and turned into fp32 by fill_windows(), after the
    // halo rows and the first row groups have been requested as well.
    float wv[CH][W], bv[CH];
    PackedTaps<W, CH, (WM == 1 ? CC1D_F32 : DT)> taps;
    StridedTaps<W, CH> any_taps;
    if (WM != 0) taps.request(p.weight, p.bias, c0);
    else any_taps.request(p.weight, p.bias, p.w_dtype, p.w_stride_c, p.w_stride_w, c0);

    // Row pointers of this run; offsets inside a run fit 32 bits (checked by the launcher).
    const char *xrun = reinterpret_cast<const char *>(reinterpret_cast<const T_ *>(p.x) + (int64_t)b * p.x_stride_b + c0 + (int64_t)t0 * p.x_stride_l);
    const char *drun = reinterpret_cast<const char *>(reinterpret_cast<const T_ *>(p.dout) + (int64_t)b * p.dout_stride_b + c0 + (int64_t)t0 * p.dout_stride_l);
    // Row i of the walk stores dx row i-(W-1): the pointer is moved back once instead.
    char *dxrun = reinterpret_cast<char *>(reinterpret_cast<T_ *>(p.dx) + (int64_t)b * p.dx_stride_b + c0) +
                  ((int64_t)t0 - (W - 1)) * p.dx_stride_l * (int64_t)sizeof(T_);
    const uint32_t xs = (uint32_t)p.x_stride_l * (uint32_t)sizeof(T_);
    const uint32_t ds = (uint32_t)p.dout_stride_l * (uint32_t)sizeof(T_);
    const uint32_t dxs = (uint32_t)p.dx_stride_l * (uint32_t)sizeof(T_);
    // seq_idx is a kernel argument of its own, marked as not aliasing anything the kernel
    // writes: its loads, at wave-uniform addresses, go through the scalar cache.
    const int32_t *seq = HAS_SEQ ? seq_idx + (int64_t)b * L + t0 : nullptr;

    using No = std::integral_constant<bool, false>;
    using Yes = std::integral_constant<bool, true>;

    // g[t] = dout[t] * act'(z[t]) from the x window in front of row t; taps that cross a
    // sub-sequence boundary are masked, padding rows (id < 0) have no gradient.
    // MASKED = false is for rows whose window holds one non-negative id throughout.
    auto grad_row = [&](auto masked, const float (&xwin)[W - 1][CH], const int (&idwin)[W - 1],
                        const float (&xv)[CH], int cur, float (&gv)[CH]) __attribute__((always_inline)) {
        constexpr bool MASKED = HAS_SEQ && decltype(masked)::value;
        if (SILU) {
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                float z = bv[j];
#pragma unroll
                for (int k = 0; k < W - 1; ++k)
                    z = fmaf((!MASKED || idwin[k] == cur) ? xwin[k][j] : 0.f, wv[j][k], z);
                z = fmaf(wv[j][W - 1], xv[j], z);
                gv[j] *= SCALED ? silu_grad_from_scaled_over_c(z) : silu_grad<PRECISE>(z);
            }
        }
        if (MASKED) {
#pragma unroll
            for (int j = 0; j < CH; ++j) gv[j] = cur < 0 ? 0.f : gv[j];
        }
    };
    // dx[pp] = sum_k weight[W-1-k] * g[pp+k]; gwin holds g[pp .. pp+W-2], gv is g[pp+W-1].
    auto dx_row = [&](auto masked, const float (&gwin)[W - 1][CH], const int (&idwin)[W - 1],
                      const float (&gv)[CH], int cur, float (&dxv)[CH]) __attribute__((always_inline)) {
        constexpr bool MASKED = HAS_SEQ && decltype(masked)::value;
        const int sp = idwin[0];
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            float a = wv[j][W - 1] * gwin[0][j];
#pragma unroll
            for (int k = 1; k < W - 1; ++k)
                a = fmaf((!MASKED || idwin[k] == sp) ? gwin[k][j] : 0.f, wv[j][W - 1 - k], a);
            a = fmaf((!MASKED || cur == sp) ? gv[j] : 0.f, wv[j][0], a);
            dxv[j] = a;
        }
    };

    // Windows at row t: xw[k] = x[t-(W-1)+k], gw[k] = g[t-(W-1)+k], sqw[k] the ids.
    // Filling gw needs the x rows and ids another W-1 steps back.  The rows are requested
    // here; fill_windows() turns them into the windows once the walk's first row groups have
    // been requested as well.
    float xw[W - 1][CH], gw[W - 1][CH];
    int sqw[W - 1];
    raw_t xh_raw[2 * (W - 1)], dh_raw[W - 1];
    int sh[2 * (W - 1)];
#pragma unroll
    for (int q = 0; q < 2 * (W - 1); ++q) {
        const int t = t0 - 2 * (W - 1) + q;
        xh_raw[q] = P::zero();
        if (t >= 0) {
            xh_raw[q] = *reinterpret_cast<const raw_t *>(xrun - (int64_t)(2 * (W - 1) - q) * xs);
        } else if (p.initial_states != nullptr && t >= -(W - 1)) {
            xh_raw[q] = load_state_row<DT, CH>(p.initial_states, p.init_stride_b, p.init_stride_c,
                                               p.init_stride_l, b, c0, t + (W - 1));
        }
        sh[q] = (HAS_SEQ && t >= 0) ? seq[q - 2 * (W - 1)] : -1;
    }
#pragma unroll
    for (int k = 0; k < W - 1; ++k) {
        const int t = t0 - (W - 1) + k;
        dh_raw[k] = P::zero();
        if (t >= 0) dh_raw[k] = *reinterpret_cast<const raw_t *>(drun - (int64_t)(W - 1 - k) * ds);
    }
    auto fill_windows = [&]() __attribute__((always_inline)) {
        if (WM != 0) taps.finish(p.bias != nullptr, wv, bv);
        else any_taps.finish(p.w_dtype, p.bias != nullptr, wv, bv);
        // With SiLU the lane keeps only c w and c bias, c = -log2(e): the sums over the taps are
        // then the exponent the activation's derivative needs, g is carried as g / c, dx comes out
        // unscaled (c w times g / c), and the kernel multiplies its dweight / dbias sums by c once.
        if (SCALED) {
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                bv[j] *= kSiluPrescale;
#pragma unroll
                for (int k = 0; k < W; ++k) wv[j][k] *= kSiluPrescale;
            }
        }
        float xh[2 * (W - 1)][CH];
#pragma unroll
        for (int q = 0; q < 2 * (W - 1); ++q) P::unpack(xh_raw[q], xh[q]);
#pragma unroll
        for (int k = 0; k < W - 1; ++k) {
            float xwin[W - 1][CH];
            int idwin[W - 1];
#pragma unroll
            for (int i = 0; i < W - 1; ++i) {
                idwin[i] = sh[k + i];
#pragma unroll
                for (int j = 0; j < CH; ++j) xwin[i][j] = xh[k + i][j];
            }
            P::unpack(dh_raw[k], gw[k]);              // zero in front of the sequence
            grad_row(Yes{}, xwin, idwin, xh[k + W - 1], sh[k + W - 1], gw[k]);
#pragma unroll
            for (int j = 0; j < CH; ++j) xw[k][j] = xh[k + W - 1][j];
            sqw[k] = sh[k + W - 1];
        }
    };

    // With seq_idx, a run whose rows and halo all carry one non-negative id needs no masks
    // at all; the ids are scalars, so finding that out costs the vector unit nothing, and the
    // run then takes the same arithmetic as a run without seq_idx.
    bool mixed = false;
    if (HAS_SEQ) {
        const int i_lo = t0 >= 2 * (W - 1) ? -2 * (W - 1) : -t0;
        uint32_t lo = (uint32_t)seq[i_lo], hi = lo;
        // Consecutive ids arrive through wide scalar loads; 64 at a time so that the loads
        // of a trip overlap, and the ragged end re-reads the last 16.
        auto scan = [&](auto n, int i) __attribute__((always_inline)) {
#pragma unroll
            for (int k = 0; k < decltype(n)::value; ++k) {
                const uint32_t v = (uint32_t)seq[i + k];
                lo = min(lo, v);
                hi = max(hi, v);
            }
        };
        int i = i_lo;
        for (; i + 63 <= last; i += 64) scan(std::integral_constant<int, 64>{}, i);
        for (; i + 15 <= last; i += 16) scan(std::integral_constant<int, 16>{}, i);
        if (i <= last) {
            if (last - 15 >= i_lo) {
                scan(std::integral_constant<int, 16>{}, last - 15);
            } else {
                for (; i <= last; ++i) scan(std::integral_constant<int, 1>{}, i);
            }
        }
        mixed = lo != hi || (int)hi < 0;
    }

    // CHECKED = false: loads and stores are unconditional (the wait counts the compiler
    // derives are then exact and loads stay in flight across stores).  CHECKED = true: the
    // first rows of run 0 (positions in front of the sequence go to dinitial_states) and
    // ragged or short runs (rows past the end re-read the last valid row and are inert).
    // STREAM: non-temporal loads; the last rows of a run are read with the normal policy
    // because the following run needs them again as its halo.
    auto load_group = [&](auto checked, auto stream, int i0, raw_t (&rx)[U], raw_t (&rd)[U], int (&sq)[U]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = (!decltype(checked)::value || (i0 + u) < last) ? (i0 + u) : last;
            const raw_t *sx = reinterpret_cast<const raw_t *>(xrun + (uint32_t)i * xs);
            const raw_t *sd = reinterpret_cast<const raw_t *>(drun + (uint32_t)i * ds);
            rx[u] = decltype(stream)::value ? __builtin_nontemporal_load(sx) : *sx;
            rd[u] = decltype(stream)::value ? __builtin_nontemporal_load(sd) : *sd;
            sq[u] = HAS_SEQ ? seq[i] : 0;
        }
    };
    auto compute_group = [&](auto checked, auto masked, int i0, const raw_t (&rx)[U], const raw_t (&rd)[U],
                            const int (&sq)[U]) __attribute__((always_inline)) {
        constexpr bool MASKED = HAS_SEQ && decltype(masked)::value;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (decltype(checked)::value && i0 + u > last) continue;   // past the end: inert
            const int cur = sq[u];
            float xv[CH], gv[CH], dxv[CH];
            P::unpack(rx[u], xv);
            P::unpack(rd[u], gv);
            grad_row(masked, xw, sqw, xv, cur, gv);
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                dB[j] += gv[j];
#pragma unroll
                // a padding row (id < 0) has g = 0; its inputs may hold anything, Inf and NaN
                // included, and take a zero here so that 0 * x stays 0
                for (int k = 0; k < W - 1; ++k)
                    dW[j][k] = fmaf(gv[j], (!MASKED || (sqw[k] == cur && cur >= 0)) ? xw[k][j] : 0.f, dW[j][k]);
                dW[j][W - 1] = fmaf(gv[j], (!MASKED || cur >= 0) ? xv[j] : 0.f, dW[j][W - 1]);
            }
            dx_row(masked, gw, sqw, gv, cur, dxv);
            if (!decltype(checked)::value) {
                if (CC1D_BWD_CL_STREAM_STORES) __builtin_nontemporal_store(P::pack(dxv), reinterpret_cast<raw_t *>(dxrun + (uint32_t)(i0 + u) * dxs));
                else *reinterpret_cast<raw_t *>(dxrun + (uint32_t)(i0 + u) * dxs) = P::pack(dxv);
            } else {
                // Row t < L completes position pp = t-(W-1) < L-(W-1): no dfinal term yet.
                const int pp = t0 + i0 + u - (W - 1);
                if (pp >= 0) {
                    *reinterpret_cast<raw_t *>(dxrun + (int64_t)(i0 + u) * dxs) = P::pack(dxv);
                } else if (p.dinitial_states != nullptr) {
                    store_state_row<DT, CH>(p.dinitial_states, p.dinit_stride_b, p.dinit_stride_c,
                                            p.dinit_stride_l, b, c0, pp + (W - 1), P::pack(dxv));
                }
            }
#pragma unroll
            for (int k = 0; k < W - 2; ++k) {
#pragma unroll
                for (int j = 0; j < CH; ++j) { xw[k][j] = xw[k + 1][j]; gw[k][j] = gw[k + 1][j]; }
                sqw[k] = sqw[k + 1];
            }
#pragma unroll
            for (int j = 0; j < CH; ++j) { xw[W - 2][j] = xv[j]; gw[W - 2][j] = gv[j]; }
            sqw[W - 2] = cur;
        }
    };
    // Run 0 routes positions in front of the sequence through the checked form of its first
    // group only, so that group must hold all W-1 of them.
    static_assert(U >= W - 1, "the first group must cover the window");
    raw_t xa[U], da[U], xb[U], db[U];
    int sa[U], sb[U];
    auto walk = [&](auto masked) __attribute__((always_inline)) {
        if (full && T >= 6 * U) {
            // Two register sets in ping-pong: while one group of U rows is computed and stored,
            // the loads of the next two groups are in flight, and nothing is copied at the loop
            // edge.  The first and the last pair of groups are peeled, so the loop is entered
            // in exactly the state its back edge leaves and the wait counts stay exact.
            load_group(No{}, Yes{}, 0, xa, da, sa);
            load_group(No{}, Yes{}, U, xb, db, sb);
            fill_windows();
            if (run > 0) compute_group(No{}, masked, 0, xa, da, sa);
            else compute_group(Yes{}, masked, 0, xa, da, sa);   // positions in front of the sequence
            load_group(No{}, Yes{}, 2 * U, xa, da, sa);
            compute_group(No{}, masked, U, xb, db, sb);
            load_group(No{}, Yes{}, 3 * U, xb, db, sb);
            int i = 2 * U;
#pragma clang loop unroll(disable)
            for (; i + 4 * U < T; i += 2 * U) {
                compute_group(No{}, masked, i, xa, da, sa);
                load_group(No{}, Yes{}, i + 2 * U, xa, da, sa);
                compute_group(No{}, masked, i + U, xb, db, sb);
                load_group(No{}, Yes{}, i + 3 * U, xb, db, sb);
            }
            // i + 4U == T: the run's last 2U rows stay cached for the next run's halo.
            compute_group(No{}, masked, i, xa, da, sa);
            load_group(No{}, No{}, i + 2 * U, xa, da, sa);
            compute_group(No{}, masked, i + U, xb, db, sb);
            load_group(No{}, No{}, i + 3 * U, xb, db, sb);
            compute_group(No{}, masked, i + 2 * U, xa, da, sa);
            compute_group(No{}, masked, i + 3 * U, xb, db, sb);
        } else {
            fill_windows();
            for (int i = 0; i <= last; i += U) {
                load_group(Yes{}, No{}, i, xa, da, sa);
                compute_group(Yes{}, masked, i, xa, da, sa);
            }
        }
    };
    if (HAS_SEQ && mixed) walk(Yes{});
    else walk(No{});

    // The sequence's last run closes it: dx[L-(W-1) .. L) see no further g (zero past the
    // end) and take dfinal_states; with seqlen < W-1 part of that lands in dinitial_states
    // (csrc/causal_conv1d_bwd.cu:535-541, 555-559).
    if (run == g.n_runs - 1) {
        float zero[CH];
#pragma unroll
        for (int j = 0; j < CH; ++j) zero[j] = 0.f;
#pragma unroll
        for (int k = 0; k < W - 1; ++k) {
            const int pp = L - (W - 1) + k;
            float dxv[CH];
            dx_row(Yes{}, gw, sqw, zero, -1, dxv);
            if (p.dfinal_states != nullptr) {
                const raw_t fr = load_state_row<DT, CH>(p.dfinal_states, p.dfinal_stride_b, p.dfinal_stride_c,
                                                        p.dfinal_stride_l, b, c0, k);
                float fv[CH];
                P::unpack(fr, fv);
#pragma unroll
                for (int j = 0; j < CH; ++j) dxv[j] += fv[j];
            }
            if (pp >= 0) {
                *reinterpret_cast<raw_t *>(reinterpret_cast<T_ *>(p.dx) + (int64_t)b * p.dx_stride_b + c0 +
                                           (int64_t)pp * p.dx_stride_l) = P::pack(dxv);
            } else if (p.dinitial_states != nullptr) {
                store_state_row<DT, CH>(p.dinitial_states, p.dinit_stride_b, p.dinit_stride_c,
                                        p.dinit_stride_l, b, c0, pp + (W - 1), P::pack(dxv));
            }
#pragma unroll
            for (int q = 0; q < W - 2; ++q) {
#pragma unroll
                for (int j = 0; j < CH; ++j) gw[q][j] = gw[q + 1][j];
                sqw[q] = sqw[q + 1];
            }
#pragma unroll
            for (int j = 0; j < CH; ++j) gw[W - 2][j] = 0.f;
            sqw[W - 2] = -1;
        }
    }

}

// WM: how the taps are read.  1: packed (dim, W) fp32, 2: packed in x's own 16-bit type (both
// through PackedTaps), 0: any layout and type (general loader).
template <int DT, int CH, int W, bool HAS_SEQ, bool SILU, int U, int WM>
__global__ void __launch_bounds__(kBlock, (CH * Elem<DT>::kBytes == 4 ? CC1D_BWD_CL_OCC : CC1D_BWD_CL_OCC8))
bwd_channellast_kernel(const cc1d_bwd_params p, const BwdClGeom g, float *__restrict__ ws,
                       const int32_t *__restrict__ seq_idx) {
    // Partial sums of wavefronts 1..3, one float per lane and term.
    __shared__ float partial[kRunsPerBlock - 1][(W + 1) * CH][kWave];

    // XCD x executes workgroups x, x+8, x+16, ...; give it chunks of consecutive runs, the 8 XCDs
    // side by side on 8 neighbouring chunks (or, blocks_per_chunk == 0, the x-th contiguous slice).
    const uint32_t xcd = blockIdx.x % kXcds, nth = blockIdx.x / kXcds;
    const uint32_t block = g.blocks_per_chunk == 0
                               ? xcd * g.blocks_per_xcd + nth
                               : ((nth / g.blocks_per_chunk) * kXcds + xcd) * g.blocks_per_chunk + nth % g.blocks_per_chunk;
    // A workgroup takes 64 adjacent vector-columns of four consecutive runs of one sequence,
    // one run per wavefront: a wavefront's row range and the sub-sequence ids it reads are
    // scalars.  Neighbouring workgroups take neighbouring columns of the same rows.
    const int wv_in_block = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const int lane = (int)(threadIdx.x & (kWave - 1));
    const uint32_t col = (block % g.waves_per_row) * (uint32_t)kWave + (uint32_t)lane;
    const uint32_t bq = block / g.waves_per_row;
    const int quad = (int)(bq % (uint32_t)g.n_quads);
    const int b = (int)(bq / (uint32_t)g.n_quads);
    const int run = quad * kRunsPerBlock + wv_in_block;

    float dW[CH][W], dB[CH];
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        dB[j] = 0.f;
#pragma unroll
        for (int w = 0; w < W; ++w) dW[j][w] = 0.f;
    }
    // Workgroups past the end of the grid's last XCD slice, runs past the end of the sequence
    // and lanes past the last column have nothing to walk; they still meet the barrier below.
    const bool active = block < g.total && run < g.n_runs && col < (uint32_t)g.n_colgroups;
    if (active) bwd_channellast_run<DT, CH, W, HAS_SEQ, SILU, U, WM>(p, g, seq_idx, b, run, col, dW, dB);

    // The workgroup's four partial sums are added in the order of the runs and stored once:
    // plane w of part (b, quad), channels c0 .. c0+CH.
    if (wv_in_block > 0) {
#pragma unroll
        for (int w = 0; w <= W; ++w)
#pragma unroll
            for (int j = 0; j < CH; ++j) partial[wv_in_block - 1][w * CH + j][lane] = w < W ? dW[j][w] : dB[j];
    }
    __syncthreads();
    if (wv_in_block == 0 && block < g.total && col < (uint32_t)g.n_colgroups) {
        const int64_t part = (int64_t)b * g.n_quads + quad;
        float *dst = ws + part * (int64_t)(W + 1) * p.dim + (int64_t)col * CH;
#pragma unroll
        for (int w = 0; w <= W; ++w) {
            typename RawBytes<CH * 4>::type o;
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                float v = w < W ? dW[j][w] : dB[j];
#pragma unroll
                for (int r = 0; r < kRunsPerBlock - 1; ++r) v += partial[r][w * CH + j][lane];
                if (SILU && !Elem<DT>::kPreciseAct) v *= kSiluPrescale;     // the runs summed g / c
                o[j] = bitcast<uint32_t>(v);
            }
            *reinterpret_cast<typename RawBytes<CH * 4>::type *>(dst + (int64_t)w * p.dim) = o;
        }
    }
}


template <int DT, int CH, int W, bool HAS_SEQ, int WM>
int launch_instance(const cc1d_bwd_params &p, const BwdClGeom &g, float *ws, hipStream_t stream) {
    constexpr int U = CC1D_BWD_CL_UNROLL;
    const uint32_t blocks = g.blocks_per_xcd * kXcds;
    if (p.silu)
        CC1D_LAUNCH((bwd_channellast_kernel<DT, CH, W, HAS_SEQ, true, U, WM>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws, p.seq_idx);
    else
        CC1D_LAUNCH((bwd_channellast_kernel<DT, CH, W, HAS_SEQ, false, U, WM>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws, p.seq_idx);
    return launch_status();
}

template <int DT, int CH, int WM>
int launch_width(const cc1d_bwd_params &p, const BwdClGeom &g, float *ws, hipStream_t stream) {
    const bool seq = p.seq_idx != nullptr;
    switch (p.width) {
        case 2: return seq ? launch_instance<DT, CH, 2, true, WM>(p, g, ws, stream) : launch_instance<DT, CH, 2, false, WM>(p, g, ws, stream);
        case 3: return seq ? launch_instance<DT, CH, 3, true, WM>(p, g, ws, stream) : launch_instance<DT, CH, 3, false, WM>(p, g, ws, stream);
        default: return seq ? launch_instance<DT, CH, 4, true, WM>(p, g, ws, stream) : launch_instance<DT, CH, 4, false, WM>(p, g, ws, stream);
    }
}

template <int DT, int CH>
int launch_dtype(const cc1d_bwd_params &p, const BwdClGeom &g, float *ws, hipStream_t stream) {
    if (g.w_mode == 1) return launch_width<DT, CH, 1>(p, g, ws, stream);
    if constexpr (DT != CC1D_F32) {
        if (g.w_mode == 2) return launch_width<DT, CH, 2>(p, g, ws, stream);
    }
    return launch_width<DT, CH, 0>(p, g, ws, stream);
}


}  // namespace
}  // namespace cc1d
