// Channel-last forward for gfx950: x is (batch, seqlen, dim) in memory (unit stride
// along dim).  Takes over causal_conv1d_channellast_fwd_kernel and its launcher
// (csrc/causal_conv1d_fwd.cu:205-381 of the reference).
//
// Design.  The stencil runs along seqlen, which is the strided axis, so nothing has to
// be transposed: a lane owns CH adjacent channels (one 4- or 8-byte vector), keeps their
// W taps and bias in registers and walks down a run of consecutive rows with a
// (W-1)-row sliding window held in registers as fp32.  Per row that is one vector load
// and one vector store per lane, both fully coalesced along dim, no LDS and no barrier.
// The only re-read is the (W-1)-row halo in front of each run.
//
// A wavefront takes 64 adjacent vector-columns of one (batch, run), so the run's row
// range and its seq_idx values are scalars; the columns of a row are covered by
// ceil(dim / (64 CH)) wavefronts, the last one partly idle when dim is not a multiple of
// 64 CH.  Wavefronts are numbered (batch, run, column block) with the column block
// fastest, and workgroups are renumbered so that each of the 8 XCDs (hardware hands
// workgroups to XCDs round-robin) walks chunks of consecutive runs of that order (8 runs, the
// XCDs side by side on 8 neighbouring chunks): the run that follows another along seqlen then
// executes on the same XCD, close in time, and its halo rows are found in that XCD's L2
// instead of being fetched from HBM twice.  For the same reason the halo rows and the last rows of a run are accessed
// with the normal cache policy while everything else streams through (non-temporal).
#include <type_traits>

#include "cc1d_varlen_gather.hpp"

// 1: rows that no later run needs are loaded non-temporally; 0: every load takes the normal policy.
#ifndef CC1D_FWD_CL_STREAM_LOADS
#define CC1D_FWD_CL_STREAM_LOADS 1
#endif
// Rows per register set; two sets are in flight per lane.
#ifndef CC1D_FWD_CL_UNROLL
#define CC1D_FWD_CL_UNROLL 8
#endif
// Channels per lane for 16-bit tensors: 2, i.e. 4-byte lanes, compiled for five workgroups
// per CU (<= 96 registers; CC1D_FWD_CL_OCC4), against three for the 8-byte lanes of fp32 data.  More wavefronts per CU overlap the kernel's
// VALU time with its memory time better than wider accesses do: 56.1 us against 60.1 us with
// 8-byte lanes and three workgroups per CU at the prefill shape.  fp32 keeps 2 channels (8 bytes).
#ifndef CC1D_FWD_CL_CH16
#define CC1D_FWD_CL_CH16 2
#endif
#ifndef CC1D_FWD_CL_OCC4
#define CC1D_FWD_CL_OCC4 5
#endif
#ifndef CC1D_FWD_CL_OCC8
#define CC1D_FWD_CL_OCC8 3
#endif

namespace cc1d {
namespace {

#ifndef CC1D_FWD_CL_STREAM_STORES
#define CC1D_FWD_CL_STREAM_STORES 1
#endif
template <typename V>
__device__ __forceinline__ void store_row(const V &v, V *dst) {
    if (CC1D_FWD_CL_STREAM_STORES) __builtin_nontemporal_store(v, dst);
    else *dst = v;
}

#ifndef CC1D_FWD_CL_XCDS
#define CC1D_FWD_CL_XCDS 8
#endif
constexpr int kXcds = CC1D_FWD_CL_XCDS;

struct FwdClGeom {
    int32_t rows_per_run;     // T, a multiple of twice the unroll factor
    int32_t n_runs;           // ceil(seqlen / T)
    int32_t n_colgroups;      // dim / CH
    uint32_t waves_per_row;   // ceil(n_colgroups / 64): wavefronts side by side on one row
    uint32_t total;           // batch * n_runs * waves_per_row wavefronts
    uint32_t blocks_per_xcd;  // grid size / 8
    uint32_t blocks_per_chunk; // workgroups an XCD takes in a row before the next XCD's (0: its whole slice)
};

// WM: how the taps are read.  1: packed (dim, W) fp32, 2: packed in x's own 16-bit type (both
// through PackedTaps), 0: any layout and type (general loader).
template <int DT, int CH, int W, bool HAS_SEQ, bool SILU, int U, int WM>
__global__ void __launch_bounds__(kBlock, (CH * Elem<DT>::kBytes == 4 ? CC1D_FWD_CL_OCC4 : CC1D_FWD_CL_OCC8))
fwd_channellast_kernel(const cc1d_fwd_params p, const FwdClGeom g, const int32_t *__restrict__ seq_idx,
                       const VarlenTail tail) {
    using E = Elem<DT>;
    using T_ = typename E::type;
    using P = Pack<DT, CH>;
    using raw_t = typename P::raw_t;
    constexpr bool PRECISE = E::kPreciseAct;

    // Workgroups past the forward's own are there for the varlen final-state gather, which
    // reads x only and so needs no ordering against the rows being produced.
    if (blockIdx.x >= tail.first_block) {
        varlen_gather_vec<DT>(tail.p, tail.n_colgroups, tail.total,
                              (blockIdx.x - tail.first_block) * (uint32_t)kBlock + threadIdx.x);
        return;
    }
    // XCD x executes workgroups x, x+8, x+16, ...; give it the x-th contiguous slice.
    const uint32_t xcd = blockIdx.x % kXcds, nth = blockIdx.x / kXcds;
    const uint32_t block = g.blocks_per_chunk == 0
                               ? xcd * g.blocks_per_xcd + nth
                               : ((nth / g.blocks_per_chunk) * kXcds + xcd) * g.blocks_per_chunk + nth % g.blocks_per_chunk;
    // A wavefront never straddles two runs: its batch index, run and row range are scalars,
    // and so are the sub-sequence ids it reads.
    const uint32_t wave = block * (uint32_t)(kBlock / kWave) +
                          (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    if (wave >= g.total) return;
    const uint32_t col = (wave % g.waves_per_row) * (uint32_t)kWave + (threadIdx.x & (kWave - 1));
    const uint32_t rb = wave / g.waves_per_row;
    const int run = (int)(rb % (uint32_t)g.n_runs);
    const int b = (int)(rb / (uint32_t)g.n_runs);
    const int L = p.seqlen;
    const int T = g.rows_per_run;                     // multiple of 2*U
    const int t0 = run * T;                           // < L by construction of n_runs
    const int last = L - 1 - t0;                      // last valid row of this run, run-relative

    // Lanes past the last column group (a row that is no whole number of wavefronts) shadow column
    // group 0 until the wavefront's cross-lane work is done: every address they form is valid, and
    // they leave before the first store.
    const bool col_ok = col < (uint32_t)g.n_colgroups;
    const int c0 = col_ok ? (int)col * CH : 0;

    // With seq_idx, the ids of the run's first rows (a row per lane, see below) are the first thing
    // requested: the look at them then waits for this one load, which finds its line in L2, and
    // not for the halo rows behind it, which may come from HBM.
    int first_ids = 0;
    if (HAS_SEQ) {
        const int t_lane = t0 + (int)(threadIdx.x & (kWave - 1)) - (W - 1);
        const int t = t_lane > L - 1 ? L - 1 : t_lane;
        first_ids = seq_idx[(int64_t)b * L + (t > 0 ? t : 0)];
    }
    // Packed taps are only requested here: everything the run starts with is in flight before
    // the first value is touched (prepare() finishes them).
    constexpr bool WFAST = WM != 0;
    constexpr bool SCALED = SILU && !PRECISE;
    float wv[CH][W], bv[CH];
    PackedTaps<W, CH, (WM == 1 ? CC1D_F32 : DT)> taps;
    StridedTaps<W, CH> any_taps;
    if (WFAST) taps.request(p.weight, p.bias, c0);
    else any_taps.request(p.weight, p.bias, p.w_dtype, p.w_stride_c, p.w_stride_w, c0);
    // 16-bit outputs with SiLU: taps and bias carry the factor -log2(e), so the sums below
    // are already the exponent the activation needs (see silu_from_scaled).  Applied by
    // prepare(), after the first row groups have been requested.
    auto scale_taps = [&]() {
        if (WFAST) taps.finish(p.bias != nullptr, wv, bv);
        else any_taps.finish(p.w_dtype, p.bias != nullptr, wv, bv);
        if (SCALED) {
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                bv[j] *= kSiluPrescale;
#pragma unroll
                for (int k = 0; k < W; ++k) wv[j][k] *= kSiluPrescale;
            }
        }
    };

    const int64_t xoff = (int64_t)b * p.x_stride_b + c0;
    const int64_t ooff = (int64_t)b * p.out_stride_b + c0;
    // Row pointers of this run; offsets inside a run fit 32 bits (checked by the launcher).
    const char *xrun = reinterpret_cast<const char *>(reinterpret_cast<const T_ *>(p.x) + xoff + (int64_t)t0 * p.x_stride_l);
    char *orun = reinterpret_cast<char *>(reinterpret_cast<T_ *>(p.out) + ooff + (int64_t)t0 * p.out_stride_l);
    const uint32_t xs = (uint32_t)p.x_stride_l * (uint32_t)sizeof(T_);
    const uint32_t os = (uint32_t)p.out_stride_l * (uint32_t)sizeof(T_);
    const int32_t *seq = HAS_SEQ ? seq_idx + (int64_t)b * L + t0 : nullptr;

    // Sliding window: xw[i] holds row t-(W-1)+i while row t is being produced.  The halo
    // rows are requested here and unpacked by prepare().
    float xw[W - 1][CH];
    raw_t halo[W - 1];
#pragma unroll
    for (int i = 0; i < W - 1; ++i) {
        const int t = t0 - (W - 1) + i;
        halo[i] = P::zero();
        if (t >= 0) {
            halo[i] = *reinterpret_cast<const raw_t *>(xrun - (int64_t)(W - 1 - i) * xs);
        } else if (p.initial_states != nullptr) {
            halo[i] = load_state_row<DT, CH>(p.initial_states, p.init_stride_b, p.init_stride_c,
                                             p.init_stride_l, b, c0, t + (W - 1));
        }
    }
    auto prepare = [&]() {
        scale_taps();

#pragma unroll
        for (int i = 0; i < W - 1; ++i) P::unpack(halo[i], xw[i]);
    };

    // CHECKED = false: the whole run lies inside the sequence, so loads and stores are
    // unconditional (the wait counts the compiler derives are then exact and loads stay
    // in flight across stores).  CHECKED = true: the ragged last run of a sequence; rows
    // past its end re-read the last valid row and their stores are suppressed.
    // STREAM: non-temporal loads; the last rows of a run are read with the normal policy
    // because the following run needs them again as its halo.
    auto load_group = [&](auto checked, auto stream, int i0, raw_t (&raw)[U]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = (!decltype(checked)::value || (i0 + u) < last) ? (i0 + u) : last;
            const raw_t *src = reinterpret_cast<const raw_t *>(xrun + (uint32_t)i * xs);
            raw[u] = (decltype(stream)::value && CC1D_FWD_CL_STREAM_LOADS) ? __builtin_nontemporal_load(src) : *src;
        }
    };

    // store = false: a group the masked pass produces; only the window moves on.
    auto compute_group = [&](auto checked, auto store, int i0, const raw_t (&raw)[U]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float xv[CH], acc[CH];
            P::unpack(raw[u], xv);
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                float a = bv[j];
#pragma unroll
                for (int k = 0; k < W - 1; ++k) a = fmaf(wv[j][k], xw[k][j], a);
                a = fmaf(wv[j][W - 1], xv[j], a);
                acc[j] = SCALED ? silu_from_scaled(a) : SILU ? silu<PRECISE>(a) : a;
            }
            if (decltype(store)::value && (!decltype(checked)::value || i0 + u <= last))
                store_row(P::pack(acc), reinterpret_cast<raw_t *>(orun + (uint32_t)(i0 + u) * os));
#pragma unroll
            for (int k = 0; k < W - 2; ++k)
#pragma unroll
                for (int j = 0; j < CH; ++j) xw[k][j] = xw[k + 1][j];
#pragma unroll
            for (int j = 0; j < CH; ++j) xw[W - 2][j] = xv[j];
        }
    };

    using No = std::integral_constant<bool, false>;
    using Yes = std::integral_constant<bool, true>;
    static_assert(U >= W - 1, "a group must cover the window");
    raw_t ra[U], rb_[U];
    // With seq_idx the walk computes every row as if no sub-sequence boundary were near (no
    // branch, no ids in the hot loop); the groups of U rows whose rows or window are not all of
    // one non-negative id are redone with masked taps after the walk.  Which groups those are is
    // found here, with all 64 lanes, a row per lane: lane i holds row i-(W-1) of a stretch of
    // whole groups and flags it when its id differs from the row before or is negative (rows in
    // front of the sequence count as id -1 when initial_states are given, as zeros, which no
    // mask changes, otherwise); group k is redone when a flag falls into its rows or the W-2
    // rows before them.  Where more than half of the groups are (sub-sequences of a few tokens),
    // the walk is skipped and the masked pass takes the whole run.
    const bool full = last >= T - 1;
    uint32_t redo = 0;
    bool dense = false;
    auto look_at_ids = [&]() __attribute__((always_inline)) {
    if (HAS_SEQ) {
        const int n_groups = T / U;
        if (n_groups > 32) {
            dense = true;
        } else {
            constexpr int kStretch = (kWave - (W - 1)) / U;            // groups per look
            const int32_t *ids = seq_idx + (int64_t)b * L;
            const int lane = threadIdx.x & (kWave - 1);
            const bool init = p.initial_states != nullptr;
            for (int k0 = 0; k0 < n_groups; k0 += kStretch) {
                const int t_lane = t0 + k0 * U + lane - (W - 1);       // row of this lane
                const int t = t_lane > L - 1 ? L - 1 : t_lane;
                const int id = k0 == 0 ? first_ids : ids[t > 0 ? t : 0];
                // The id of the row before is the previous lane's (a lane shift, no second load);
                // lane 0 gets its own id, and its flag belongs to no group's window.
                const int id_prev = __builtin_amdgcn_update_dpp(id, id, 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
                const bool flag = t_lane > L - 1 ? false
                                : t >= 0 ? (id < 0 || (t > 0 ? id != id_prev : init)) : init;
                const uint64_t flags = __ballot(flag);
                for (int k = 0; k < kStretch && k0 + k < n_groups; ++k)
                    if ((flags >> (k * U + 1)) & ((1ull << (U + W - 2)) - 1)) redo |= 1u << (k0 + k);
            }
            int live = last / U + 1;                                   // groups with rows inside the sequence
            live = live > n_groups ? n_groups : live;
            redo &= live >= 32 ? ~0u : (1u << live) - 1u;
            dense = 2 * __builtin_popcount(redo) > live;
        }
    }
    };
    // The look comes before the run's first rows are requested.  Requesting the rows first and
    // looking at the ids while they are in flight (the ids, requested before everything else, are
    // back long before them) takes the look out of the wavefront's critical path, and measured
    // 3.4 us slower on warm buffers (56.1 against 52.7 us) for 1.3 us gained on cold ones.
    look_at_ids();
    // The masked pass over one group of U rows: taps masked row by row
    // (csrc/causal_conv1d_fwd.cu:316-329), padding tokens exactly zero.  masked_request() asks for
    // the U+W-1 rows and ids the group needs, straight from memory and with no branch between the
    // loads; masked_finish() computes and stores the group's rows.
    constexpr int kSpan = U + W - 1;
    auto masked_request = [&](int i0, raw_t (&rows)[kSpan], int (&sr)[kSpan]) {
#pragma unroll
        for (int q = 0; q < kSpan; ++q) {
            int i = i0 - (W - 1) + q;                  // run-relative row of slot q
            const bool before = t0 + i < 0;           // in front of the sequence: no data
            i = i > last ? last : i;
            i = before ? 0 : i;
            rows[q] = *reinterpret_cast<const raw_t *>(xrun + (int64_t)i * xs);
            const int id = seq[i];
            sr[q] = before ? -1 : id;
        }
    };
    auto masked_finish = [&](int i0, const raw_t (&rows)[kSpan], const int (&sr)[kSpan]) {
        float xr[kSpan][CH];
#pragma unroll
        for (int q = 0; q < kSpan; ++q) P::unpack(rows[q], xr[q]);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int cur = sr[W - 1 + u];
            float acc[CH];
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                float a = bv[j];
#pragma unroll
                for (int k = 0; k < W - 1; ++k)
                    a = fmaf(sr[u + k] == cur ? wv[j][k] : 0.f, xr[u + k][j], a);
                a = fmaf(wv[j][W - 1], xr[u + W - 1][j], a);
                if (SILU) a = SCALED ? silu_from_scaled(a) : silu<PRECISE>(a);
                acc[j] = cur < 0 ? 0.f : a;
            }
            if (i0 + u <= last)
                store_row(P::pack(acc), reinterpret_cast<raw_t *>(orun + (uint32_t)(i0 + u) * os));
        }
    };
    auto marked = [&](int i0) { return HAS_SEQ && ((redo >> (i0 / U)) & 1u) != 0; };
    // A full run does the masked pass of its first marked group up front: the group's rows are
    // requested here, ahead of the walk's own first rows, so that they cost no memory round trip
    // of their own (at the end of the walk they would, with nothing left to overlap it), and are
    // computed and stored while the walk's rows are still in flight.  The walk stores none of the
    // marked groups; those behind the first are done after it.
    raw_t early_rows[kSpan];
    int early_ids[kSpan];
    const int early = (HAS_SEQ && full && !dense && redo != 0) ? __builtin_ctz(redo) : -1;
    if (HAS_SEQ) {
        if (early >= 0) masked_request(early * U, early_rows, early_ids);
    }
    // Rows of a group that will be redone are read with the normal cache policy, so that the
    // second read finds them in L2; everything else streams through.
    if (full && !dense) {
        if (marked(0)) load_group(No{}, No{}, 0, ra); else load_group(No{}, Yes{}, 0, ra);
        if (T > 2 * U && !marked(U)) load_group(No{}, Yes{}, U, rb_);
        else load_group(No{}, No{}, U, rb_);          // the run's last rows: keep them cached
    }
    if (!col_ok) return;                              // no cross-lane traffic below
    auto load_maybe_marked = [&](int i0, raw_t (&raw)[U]) {
        if (marked(i0)) load_group(No{}, No{}, i0, raw);
        else load_group(No{}, Yes{}, i0, raw);
    };
    auto walk_group = [&](int i0, const raw_t (&raw)[U]) {
        if (marked(i0)) compute_group(No{}, No{}, i0, raw);
        else compute_group(No{}, Yes{}, i0, raw);
    };
    auto early_masked = [&]() {
        if (HAS_SEQ) {
            if (early >= 0) masked_finish(early * U, early_rows, early_ids);
        }
    };
    if (dense) {
        // Most groups would be redone: skip the walk, the masked pass below takes the whole run.
        prepare();
    } else if (full) {
        // Two register sets in ping-pong: while one group of U rows is computed and stored,
        // the next two groups' loads are in flight, and nothing is copied at the loop edge
        // (a copy would make the compiler wait for every outstanding access).  The first
        // and the last pair of groups are peeled: the loop is then entered in exactly the
        // state its back edge leaves (stores A, loads A, stores B, loads B pending), which
        // keeps the compiler's wait counts exact, and no load sits behind an exit test.
        if (T > 2 * U) {
            prepare();
            early_masked();
            walk_group(0, ra);
            int i = 2 * U;
            if (T > 4 * U) {
                load_maybe_marked(2 * U, ra);
                walk_group(U, rb_);
                load_maybe_marked(3 * U, rb_);
#pragma clang loop unroll(disable)
                for (; i + 4 * U < T; i += 2 * U) {
                    walk_group(i, ra);
                    load_maybe_marked(i + 2 * U, ra);
                    walk_group(i + U, rb_);
                    load_maybe_marked(i + 3 * U, rb_);
                }
                walk_group(i, ra);
                load_maybe_marked(i + 2 * U, ra);
                walk_group(i + U, rb_);
                i += 2 * U;
            } else {
                load_maybe_marked(2 * U, ra);
                walk_group(U, rb_);
            }
            load_group(No{}, No{}, i + U, rb_);   // the run's last rows: keep them cached
            walk_group(i, ra);
            walk_group(i + U, rb_);
        } else {
            prepare();
            early_masked();
            walk_group(0, ra);
            walk_group(U, rb_);
        }
    } else {
        prepare();
        for (int i = 0; i <= last; i += U) {
            load_group(Yes{}, No{}, i, ra);
            if (marked(i)) compute_group(Yes{}, No{}, i, ra);
            else compute_group(Yes{}, Yes{}, i, ra);
        }
    }

    if (HAS_SEQ) {
        // The marked groups the walk left out (all of the run's groups when the walk was skipped),
        // one group per trip.
        const int live_rows = last + 1 < T ? last + 1 : T;
#pragma clang loop unroll(disable)
        for (int i0 = 0; i0 < live_rows; i0 += U) {
            if (!dense && (!marked(i0) || i0 == early * U)) continue;
            raw_t rows[kSpan];
            int sr[kSpan];
            masked_request(i0, rows, sr);
            masked_finish(i0, rows, sr);
        }
    }

    // final_states[b, c, i] = xpad[L-(W-1)+i], copied from x (or initial_states where L < W-1)
    // by the wavefront of the FIRST run, the one that read initial_states as its halo: the two
    // may be one buffer, and inside one wavefront the reads are complete before the stores.
    if (p.final_states != nullptr && run == 0) {
        wait_for_loads();
        raw_t fin[W - 1];
#pragma unroll
        for (int i = 0; i < W - 1; ++i) {
            const int t = L - (W - 1) + i;
            raw_t r = P::zero();
            if (t >= 0) {
                r = *reinterpret_cast<const raw_t *>(reinterpret_cast<const T_ *>(p.x) + xoff + (int64_t)t * p.x_stride_l);
            } else if (p.initial_states != nullptr) {
                r = load_state_row<DT, CH>(p.initial_states, p.init_stride_b, p.init_stride_c,
                                           p.init_stride_l, b, c0, t + (W - 1));
            }
            fin[i] = r;
        }
        wait_for_loads();                             // rows shorter than W-1 re-read initial_states above
#pragma unroll
        for (int i = 0; i < W - 1; ++i)
            store_state_row<DT, CH>(p.final_states, p.final_stride_b, p.final_stride_c,
                                    p.final_stride_l, b, c0, i, fin[i]);
    }
}

template <int DT, int CH, int W, bool HAS_SEQ, int WM>
int launch_instance(const cc1d_fwd_params &p, const FwdClGeom &g, const VarlenTail &tail, hipStream_t stream) {
    constexpr int U = CC1D_FWD_CL_UNROLL;
    const uint32_t blocks = tail.first_block + (tail.total + kBlock - 1) / kBlock;
    if (p.silu)
        CC1D_LAUNCH((fwd_channellast_kernel<DT, CH, W, HAS_SEQ, true, U, WM>),
                           dim3(blocks), dim3(kBlock), 0, stream, p, g, p.seq_idx, tail);
    else
        CC1D_LAUNCH((fwd_channellast_kernel<DT, CH, W, HAS_SEQ, false, U, WM>),
                           dim3(blocks), dim3(kBlock), 0, stream, p, g, p.seq_idx, tail);
    return launch_status();
}

template <int DT, int CH, int WM>
int launch_width(const cc1d_fwd_params &p, const FwdClGeom &g, const VarlenTail &tail, hipStream_t stream) {
    const bool seq = p.seq_idx != nullptr;
    switch (p.width) {
        case 2: return seq ? launch_instance<DT, CH, 2, true, WM>(p, g, tail, stream) : launch_instance<DT, CH, 2, false, WM>(p, g, tail, stream);
        case 3: return seq ? launch_instance<DT, CH, 3, true, WM>(p, g, tail, stream) : launch_instance<DT, CH, 3, false, WM>(p, g, tail, stream);
        default: return seq ? launch_instance<DT, CH, 4, true, WM>(p, g, tail, stream) : launch_instance<DT, CH, 4, false, WM>(p, g, tail, stream);
    }
}

// 2 channels per lane (4 bytes of 16-bit data, 8 bytes of fp32); taps through PackedTaps when
// they are packed (mode 1 or 2), else through the general loader.
template <int DT>
int launch_lanes(const cc1d_fwd_params &p, const FwdClGeom &g, const VarlenTail &tail, int mode, hipStream_t stream) {
    constexpr int FULL = Elem<DT>::kVec;
    constexpr int HALF = DT == CC1D_F32 ? FULL / 2 : CC1D_FWD_CL_CH16;
    if (mode == 1) return launch_width<DT, HALF, 1>(p, g, tail, stream);
    if constexpr (DT != CC1D_F32) {
        if (mode == 2) return launch_width<DT, HALF, 2>(p, g, tail, stream);
    }
    return launch_width<DT, HALF, 0>(p, g, tail, stream);
}

}  // namespace

// Rows walked by one lane.  Longer runs amortise the per-run start-up (taps, halo); shorter
// runs put more wavefronts in flight, which is what keeps HBM busy while other waves
// compute, and spread the work more evenly over the CUs, and on buffers no cache holds they
// keep the chip's accesses closer together in memory.  32 rows measured best on warm buffers at
// the prefill shape (8 x 2048 rows x 5376 channels) without seq_idx; short sequences take what they have.
// A launch that fills the chip's wavefront slots (256 CUs x 4 SIMDs x `waves_per_simd`) less than
// 0.6 times over with 32-row runs is bound by the length of a wavefront's own chain of loads,
// not by bandwidth, and takes 16-row runs: 3.7 against 4.6 us at (1, 5376, 64) bf16, 5.5 against
// 6.2 us at (1, 5376, 1024), 8.6 against 9.5 us at (1, 5376, 1024) fp32; from about one fill
// upwards 32 rows are as good or better for 16-bit data.
// fp32 rows (8-byte lanes, three wavefronts per SIMD) take 16-row runs at every size: warm / on
// rotating buffer sets, 16 against 32 rows, (4, 2048, 4096) 42.2 / 46.9 against 43.4 / 48.8 us,
// (16, 2048, 2048) 78.9 / 89.1 against 79.6 / 94.4, (8, 5376, 2048) 103.5 / 117.9 against 103.1 / 121.6,
// the same with seq_idx 115.8 / 118.0 against 120.9 / 125.0, (64, 768, 1024) 61.1 / 69.3 against
// 62.2 / 72.6; (4, 8192, 2048) is the one shape of fourteen that lost on rotating sets (90.5 against 88.0).
// bf16 / fp16 with seq_idx take 16-row runs as well: (8, 5376, 2048) 52.5 / 61.4 against 52.5 / 63.3 us,
// (8, 4096, 2048) 40.0 / 47.5 against 40.9 / 50.2, (16, 2048, 2048) 40.4 / 47.3 against 41.2 / 50.2,
// (2, 10240, 4096) 51.6 / 58.9 against 50.7 / 61.2, (8, 6144, 2048) 59.6 / 69.4 against 59.5 / 73.8.
// Without seq_idx 16-row runs gain 0.3 to 1.7 us on rotating sets and lose 1 to 2.5 us on warm ones
// ((8, 5376, 2048) 55.2 / 59.2 against 53.6 / 60.9): they keep 32 rows.
// (A copy kernel that walks the prefill tensor the same way, no arithmetic, takes 59.1 us on
// rotating sets in 32-row runs and 56.0 us in 16-row runs, a plain linear copy 55.6 us.)
static int choose_rows_per_run(int seqlen, int64_t row_bytes, int64_t waves_per_row_of_runs, int waves_per_simd,
                               bool short_runs) {
    constexpr int U = 2 * CC1D_FWD_CL_UNROLL;         // the walk is unrolled over two groups
    int T = tunables().fwd_cl_rows;
    if (T <= 0) {
        T = short_runs ? 16 : 32;
        const int64_t waves32 = waves_per_row_of_runs * ((seqlen + 31) / 32);
        if (10 * waves32 <= 6 * (int64_t)(256 * 4) * waves_per_simd) T = 16;
    }
    const int cap = (seqlen + U - 1) / U * U;          // never longer than the sequence
    if (T > cap) T = cap;
    T = (T + U - 1) / U * U;
    if (T < U) T = U;
    // Byte offsets inside a run are 32-bit in the kernel.
    while (T > U && (int64_t)T * row_bytes >= ((int64_t)1 << 31)) T = (T / 2 + U - 1) / U * U;
    return (int64_t)T * row_bytes >= ((int64_t)1 << 31) ? 0 : T;
}

// gather: a varlen final-state gather to run in the same launch (NULL: none).  It must be one
// the vector gather takes (varlen_vec_ok) on elements as wide as x's.
int launch_fwd_channellast(const cc1d_fwd_params &p, const cc1d_varlen_params *gather, hipStream_t stream) {
    // Channels per lane: 2 (4 bytes of 16-bit data, 8 bytes of fp32).  A fraction of the registers
    // of a 16-byte lane, so more waves per SIMD to overlap compute with memory; measured 9 %
    // (8-byte lanes) and another 7 % (4-byte lanes) faster at the prefill shape.
    // fwd_cl_half_vec = -1 forces the general tap loader.
    const int full = vec_elems(p.x_dtype);
    int mode = weights_mode(p.weight, p.bias, p.w_dtype, p.x_dtype, p.w_stride_c, p.w_stride_w, p.width);
    if (tunables().fwd_cl_half_vec < 0) mode = 0;
    const int ch = p.x_dtype == CC1D_F32 ? full / 2 : CC1D_FWD_CL_CH16;
    FwdClGeom g;
    g.n_colgroups = p.dim / ch;
    const int64_t row_stride = p.x_stride_l > p.out_stride_l ? p.x_stride_l : p.out_stride_l;
    g.waves_per_row = (uint32_t)((g.n_colgroups + kWave - 1) / kWave);
    g.rows_per_run = choose_rows_per_run(p.seqlen, row_stride * elem_bytes(p.x_dtype), (int64_t)p.batch * g.waves_per_row,
                                         p.x_dtype == CC1D_F32 ? CC1D_FWD_CL_OCC8 : CC1D_FWD_CL_OCC4,
                                         p.x_dtype == CC1D_F32 || p.seq_idx != nullptr);
    if (g.rows_per_run == 0) return CC1D_ERR_TOO_LARGE;
    g.n_runs = (p.seqlen + g.rows_per_run - 1) / g.rows_per_run;
    const int64_t total = (int64_t)p.batch * g.n_runs * g.waves_per_row;
    if (total * kWave >= thread_limit() - kXcds * kBlock) return CC1D_ERR_TOO_LARGE;
    g.total = (uint32_t)total;
    const uint32_t blocks = (uint32_t)((total + kBlock / kWave - 1) / (kBlock / kWave));
    // Workgroup order: an XCD takes chunks of `chunk_runs` consecutive runs (all their column
    // blocks), the 8 XCDs take 8 neighbouring chunks at a time.  Inside a chunk a run finds the halo
    // rows it shares with the run above in its own XCD's L2; across XCDs the chip walks through
    // memory as one front instead of eight far-apart streams, which is what counts on buffers that
    // are not already in the caches and translation caches (every layer of a model).  Chunk sizes
    // are measured, warm / on rotating buffer sets of 2 GB, bf16, in us:
    //   row of 42 wavefronts (8, 5376, 2048): slices 54.2 / 62.6, chunks of 2 runs 54.4 / 60.8, 4 runs
    //     53.6 / 60.9, 8 runs 53.2 / 61.5, 16 runs 54.5 / 63.8, hardware order 55.7 / 60.3; the same
    //     picture at (16, 5376, 1024), (32, 5376, 512), (1, 5376, 16384), in fp16 and in fp32
    //   80 wavefronts (2, 10240, 4096): slices 52.9 / 61.2, 2 runs 52.0 / 59.0, 4 runs 53.8 / 61.3
    //   64 wavefronts (4, 8192, 2048): slices 41.8 / 48.0, 4 runs 43.7 / 49.9, 16 runs 42.0 / 47.7
    //   32 wavefronts (8, 4096, 2048): slices 42.4 / 50.8, 8 runs 42.7 / 50.6, 16 runs 41.8 / 48.3
    //   16 wavefronts (16, 2048, 2048): slices 44.5 / 54.8, 8 runs 42.0 / 47.7, 16 runs 42.0 / 48.1
    // (row strides that are large powers of two want the XCDs further apart).  Launches of fewer
    // than eight chunks per XCD take smaller chunks, or else contiguous slices ((2, 8192, 2048):
    // 22.9 us in slices, 25.9 us in 32 chunks).
    int chunk_runs = tunables().fwd_cl_chunk_runs;
    if (chunk_runs == 0) {
        const int64_t wpr = g.waves_per_row;
        if (p.x_dtype == CC1D_F32 && wpr <= 32) {
            // fp32 rows (twice the bytes, fewer wavefronts per CU) measured best in chunks of 16 runs,
            // from four chunks per XCD on: (4, 2048, 4096) 42.5 us in slices, 46.6 in chunks of 8, 41.8 in
            // chunks of 16 (cold 48.1 / 55.5 / 48.3); (16, 2048, 2048) 79.6 / 81.5 / 78.0 us (cold 98 / 102 / 92.6).
            chunk_runs = 16;
            if ((int64_t)blocks < 4 * kXcds * (chunk_runs / 4) * wpr) chunk_runs = -1;
        } else {
            // chunks per XCD the launch gives at a chunk size
            auto chunks_per_xcd = [&](int runs) { return (int64_t)blocks * 4 / ((int64_t)kXcds * runs * wpr); };
            if (wpr > 64) chunk_runs = chunks_per_xcd(2) >= 8 ? 2 : -1;
            else if (wpr > 48) chunk_runs = chunks_per_xcd(16) >= 4 ? 16 : -1;
            else if (wpr > 32) chunk_runs = chunks_per_xcd(4) >= 8 ? 4 : -1;
            else {
                chunk_runs = wpr > 16 && chunks_per_xcd(16) >= 4 ? 16 : 8;
                if (chunk_runs == 8 && chunks_per_xcd(8) < 8) chunk_runs = 4;
                if (chunk_runs == 4 && chunks_per_xcd(4) < 8) chunk_runs = -1;
            }
        }
    }
    // chunk_runs > 0: chunks of that many runs (a run is waves_per_row wavefronts, a workgroup four of
    // them); < -1: chunks of -chunk_runs - 1 workgroups (-2: one workgroup, which is the hardware's own
    // round-robin order); -1: one contiguous slice per XCD.
    g.blocks_per_chunk = chunk_runs > 0 ? (uint32_t)(((int64_t)chunk_runs * g.waves_per_row + 3) / 4)
                         : chunk_runs < -1 ? (uint32_t)(-chunk_runs - 1) : 0u;
    g.blocks_per_xcd = (blocks + kXcds - 1) / kXcds;
    if (g.blocks_per_chunk != 0)
        g.blocks_per_xcd = (g.blocks_per_xcd + g.blocks_per_chunk - 1) / g.blocks_per_chunk * g.blocks_per_chunk;
    if ((int64_t)g.blocks_per_xcd * kXcds * kBlock >= thread_limit()) return CC1D_ERR_TOO_LARGE;
    VarlenTail tail = {};
    tail.first_block = g.blocks_per_xcd * kXcds;
    if (gather != nullptr) {
        tail.p = *gather;
        tail.n_colgroups = (uint32_t)(gather->dim / vec_elems(gather->x_dtype));
        const int64_t threads = (int64_t)gather->batch * gather->state_len * tail.n_colgroups;
        if (threads + (int64_t)tail.first_block * kBlock >= thread_limit()) return CC1D_ERR_TOO_LARGE;
        tail.total = (uint32_t)threads;
    }
    switch (p.x_dtype) {
        case CC1D_F32: return launch_lanes<CC1D_F32>(p, g, tail, mode, stream);
        case CC1D_F16: return launch_lanes<CC1D_F16>(p, g, tail, mode, stream);
        default: return launch_lanes<CC1D_BF16>(p, g, tail, mode, stream);
    }
}

}  // namespace cc1d
