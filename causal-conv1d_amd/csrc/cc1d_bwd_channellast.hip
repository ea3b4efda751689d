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
#include <type_traits>

#include "cc1d_device.hpp"
#include "cc1d_internal.hpp"

// Rows per register set; two sets are in flight per lane.
#ifndef CC1D_BWD_CL_UNROLL
#define CC1D_BWD_CL_UNROLL 4
#endif
// Workgroups per CU the register budget must allow.
#ifndef CC1D_BWD_CL_OCC
#define CC1D_BWD_CL_OCC 4
#endif

namespace cc1d {
namespace {

constexpr int kXcds = 8;

constexpr int kRunsPerBlock = kBlock / kWave;   // the wavefronts of a workgroup take consecutive runs

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
};

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
                for (int k = 0; k < W - 1; ++k)
                    dW[j][k] = fmaf(gv[j], (!MASKED || sqw[k] == cur) ? xw[k][j] : 0.f, dW[j][k]);
                dW[j][W - 1] = fmaf(gv[j], xv[j], dW[j][W - 1]);
            }
            dx_row(masked, gw, sqw, gv, cur, dxv);
            if (!decltype(checked)::value) {
                __builtin_nontemporal_store(P::pack(dxv), reinterpret_cast<raw_t *>(dxrun + (uint32_t)(i0 + u) * dxs));
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
__global__ void __launch_bounds__(kBlock, (CH * Elem<DT>::kBytes == 4 ? CC1D_BWD_CL_OCC : 2))
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

}  // namespace

// Second stage shared by both backward layouts: dweight[c, w] += (or =) sum over parts of
// ws[part][w][c]; plane W holds dbias.  A workgroup owns 64 channels of one plane; its 16
// wavefronts each add up every 16th part (four independent chains, so the loads overlap),
// and wavefront 0 combines the 16 slice sums through LDS.  The order of the additions is a
// function of n_parts alone, so results are bit-reproducible.
constexpr int kFinSlices = 16;
constexpr int kFinChannels = 64;

__global__ void __launch_bounds__(kFinSlices * kFinChannels)
bwd_finalize_kernel(const float *__restrict__ ws, int n_parts, int dim, int width,
                    float *__restrict__ dweight, int64_t dw_stride_c, int64_t dw_stride_w,
                    float *__restrict__ dbias, int overwrite) {
    __shared__ float slice_sum[kFinSlices][kFinChannels];
    const int lane = (int)threadIdx.x % kFinChannels;
    const int slice = (int)threadIdx.x / kFinChannels;
    const int cblocks = (dim + kFinChannels - 1) / kFinChannels;
    const int w = (int)blockIdx.x / cblocks;
    const int c = ((int)blockIdx.x % cblocks) * kFinChannels + lane;
    const int64_t part_stride = (int64_t)(width + 1) * dim;
    float s = 0.f;
    if (c < dim) {
        const float *src = ws + (int64_t)w * dim + c;
        float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
        int q = slice;
        for (; q + 3 * kFinSlices < n_parts; q += 4 * kFinSlices) {
            s0 += src[(int64_t)q * part_stride];
            s1 += src[(int64_t)(q + kFinSlices) * part_stride];
            s2 += src[(int64_t)(q + 2 * kFinSlices) * part_stride];
            s3 += src[(int64_t)(q + 3 * kFinSlices) * part_stride];
        }
        for (; q < n_parts; q += kFinSlices) s0 += src[(int64_t)q * part_stride];
        s = (s0 + s1) + (s2 + s3);
    }
    slice_sum[slice][lane] = s;
    __syncthreads();
    if (slice == 0 && c < dim) {
        float total = 0.f;
#pragma unroll
        for (int i = 0; i < kFinSlices; ++i) total += slice_sum[i][lane];
        float *dst = w < width ? dweight + (int64_t)c * dw_stride_c + (int64_t)w * dw_stride_w : dbias + c;
        *dst = overwrite ? total : *dst + total;
    }
}

int launch_bwd_finalize(const float *ws, int n_parts, const cc1d_bwd_params &p, hipStream_t stream) {
    const uint32_t planes = (uint32_t)p.width + (p.dbias != nullptr ? 1u : 0u);
    const uint32_t cblocks = ((uint32_t)p.dim + kFinChannels - 1) / kFinChannels;
    hipLaunchKernelGGL(bwd_finalize_kernel, dim3(planes * cblocks), dim3(kFinSlices * kFinChannels), 0, stream,
                       ws, n_parts, p.dim, p.width, p.dweight, p.dw_stride_c, p.dw_stride_w, p.dbias,
                       p.overwrite_dweight);
    return launch_status();
}

namespace {

// Channels per lane for 16-bit tensors: 2, i.e. 4-byte lanes.  A lane's windows, taps and
// partial sums then fit 128 registers and four workgroups share a CU, which is worth more to
// this VALU-heavy kernel than wider accesses: 92 us against 102 us with 8-byte lanes and two
// workgroups per CU at (8, 5376, 2048) bf16.  fp32 keeps 2 channels (8 bytes).
#ifndef CC1D_BWD_CL_CH16
#define CC1D_BWD_CL_CH16 2
#endif
int channels_per_lane(int x_dtype) { return x_dtype == CC1D_F32 ? 2 : CC1D_BWD_CL_CH16; }

// Returns false when a run cannot be addressed with 32-bit byte offsets.
bool make_geom(const cc1d_bwd_params &p, BwdClGeom &g) {
    constexpr int U2 = 2 * CC1D_BWD_CL_UNROLL;        // the walk is unrolled over two groups
    g.n_colgroups = p.dim / channels_per_lane(p.x_dtype);
    int T = tunables().bwd_cl_rows;
    // Runs of 32 rows, four of them per workgroup: the halo in front of a run costs 9 % more row
    // requests (found in cache: the run in front belongs to the same workgroup or the one
    // before), a workgroup's partial sums are one plane per 128 rows, and the prefill shape
    // launches 10752 wavefronts.  Measured there against 16, 24, 48, 64 and 128 rows, with and
    // without seq_idx.
    // A launch that fills the chip's wavefront slots less than 0.1 times over with 32-row runs is
    // bound by the length of one wavefront's chain and takes 8-row runs: (1, 5376, 64) bf16 8.1
    // against 10.0 us, (1, 2560, 256) fp32 8.2 against 10.5 us, second stage included; from 0.16
    // fills upwards 32 rows are as good or better.
    if (T <= 0) {
        T = 32;
        const int64_t waves32 = (int64_t)p.batch * ((p.seqlen + 31) / 32) * ((g.n_colgroups + kWave - 1) / kWave);
        const int64_t slots = (int64_t)256 * 4 * (p.x_dtype == CC1D_F32 ? 2 : CC1D_BWD_CL_OCC);
        if (10 * waves32 <= slots) T = 8;
    }
    const int cap = (p.seqlen + U2 - 1) / U2 * U2;     // never longer than the sequence
    if (T > cap) T = cap;
    T = (T + U2 - 1) / U2 * U2;
    if (T < U2) T = U2;
    int64_t row_stride = p.x_stride_l > p.dout_stride_l ? p.x_stride_l : p.dout_stride_l;
    if (p.dx_stride_l > row_stride) row_stride = p.dx_stride_l;
    const int64_t row_bytes = row_stride * elem_bytes(p.x_dtype);
    while (T > U2 && (int64_t)(T + U2) * row_bytes >= ((int64_t)1 << 31)) T = (T / 2 + U2 - 1) / U2 * U2;
    if ((int64_t)(T + U2) * row_bytes >= ((int64_t)1 << 31)) return false;
    g.rows_per_run = T;
    g.n_runs = (p.seqlen + T - 1) / T;
    g.n_quads = (g.n_runs + kRunsPerBlock - 1) / kRunsPerBlock;
    g.waves_per_row = (uint32_t)((g.n_colgroups + kWave - 1) / kWave);
    const int64_t total = (int64_t)p.batch * g.n_quads * g.waves_per_row;    // workgroups
    if (total * kBlock >= thread_limit() - kXcds * kBlock) return false;
    g.total = (uint32_t)total;
    g.blocks_per_xcd = (uint32_t)((total + kXcds - 1) / kXcds);
    // Workgroup order, as in the forward: chunks of 4 runs (one workgroup row; 8 runs measured 1-2 %
    // behind), or one contiguous slice per XCD where the launch has fewer than eight chunks per XCD.
    // Slices -> chunks: (8, 5376, 2048) bf16 91.5 -> 90.0 us, (4, 4096, 4096) 77.0 -> 72.6 us,
    // (16, 2048, 2048) 79.0 -> 73.4 us, (8, 10240, 2048) 177.8 -> 173.4 us.
    int chunk_runs = tunables().bwd_cl_chunk_runs;
    // fp32 rows of at most 16 wavefronts measured best in chunks of 16 runs, from four chunks per XCD
    // on: (4, 2048, 4096) 79.1 us in slices, 75.1 in chunks of 4, 70.5 in chunks of 16; (16, 2048, 2048)
    // 148.2 / 138.9 / 133.7 us; wider fp32 rows in chunks of 4 ((8, 5376, 2048) 174.1 -> 173.0 us).
    if (chunk_runs == 0) {
        chunk_runs = 4;
        if (p.x_dtype == CC1D_F32 && g.waves_per_row <= 16 &&
            total >= (int64_t)4 * kXcds * (16 / kRunsPerBlock) * g.waves_per_row) chunk_runs = 16;
        if (chunk_runs == 4 && total < (int64_t)8 * kXcds * g.waves_per_row) chunk_runs = -1;
    }
    g.blocks_per_chunk = chunk_runs <= 0 ? 0u
                                         : (uint32_t)(chunk_runs / kRunsPerBlock > 0 ? chunk_runs / kRunsPerBlock : 1) * g.waves_per_row;
    if (g.blocks_per_chunk != 0)
        g.blocks_per_xcd = (g.blocks_per_xcd + g.blocks_per_chunk - 1) / g.blocks_per_chunk * g.blocks_per_chunk;
    if ((int64_t)g.blocks_per_xcd * kXcds * kBlock >= thread_limit()) return false;
    g.w_mode = weights_mode(p.weight, p.bias, p.w_dtype, p.x_dtype, p.w_stride_c, p.w_stride_w, p.width);
    return true;
}

template <int DT, int CH, int W, bool HAS_SEQ, int WM>
int launch_instance(const cc1d_bwd_params &p, const BwdClGeom &g, float *ws, hipStream_t stream) {
    constexpr int U = CC1D_BWD_CL_UNROLL;
    const uint32_t blocks = g.blocks_per_xcd * kXcds;
    if (p.silu)
        hipLaunchKernelGGL((bwd_channellast_kernel<DT, CH, W, HAS_SEQ, true, U, WM>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws, p.seq_idx);
    else
        hipLaunchKernelGGL((bwd_channellast_kernel<DT, CH, W, HAS_SEQ, false, U, WM>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws, p.seq_idx);
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

size_t bwd_channellast_workspace_bytes(const cc1d_bwd_params &p) {
    BwdClGeom g;
    if (!make_geom(p, g)) return 0;
    return (size_t)p.batch * g.n_quads * (p.width + 1) * (size_t)p.dim * sizeof(float);
}

bool bwd_channellast_fits(const cc1d_bwd_params &p) {
    BwdClGeom g;
    return make_geom(p, g);
}

int launch_bwd_channellast(const cc1d_bwd_params &p, void *workspace, hipStream_t stream) {
    BwdClGeom g;
    if (!make_geom(p, g)) return CC1D_ERR_TOO_LARGE;
    float *ws = static_cast<float *>(workspace);
    int st;
    switch (p.x_dtype) {
        case CC1D_F32: st = launch_dtype<CC1D_F32, 2>(p, g, ws, stream); break;
        case CC1D_F16: st = launch_dtype<CC1D_F16, CC1D_BWD_CL_CH16>(p, g, ws, stream); break;
        default: st = launch_dtype<CC1D_BF16, CC1D_BWD_CL_CH16>(p, g, ws, stream); break;
    }
    if (st != CC1D_OK) return st;
    return launch_bwd_finalize(ws, p.batch * g.n_quads, p, stream);
}

}  // namespace cc1d
