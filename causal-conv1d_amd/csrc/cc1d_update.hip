// Decode-step update for gfx950.  Takes over causal_conv1d_update_kernel and its
// launcher (csrc/causal_conv1d_update.cu:23-136 of the reference).
//
// Four kernels:
//  * update_step_kernel — the decode step proper: one new token (seqlen 1) and x, out,
//    conv_state with unit stride along dim.  A lane owns one 8-byte vector of channels of
//    two consecutive batch entries; all of its loads (window rows, x) are issued before
//    anything is consumed, the taps come through LDS once per workgroup, and the grid is
//    (column blocks, batch blocks), so no index division sits in front of the first load.
//    This shape moves about 22 MB; its
//    run time is within a microsecond of a plain copy of the same footprint, which itself
//    only costs about 1.6 us more than an empty launch.
//  * update_tokens_kernel — 2 to 8 new tokens a call (speculative decoding), same layout and
//    lane width: one batch entry per lane, every x row and the window requested up front,
//    taps through LDS, the tokens then produced in order from registers.
//  * update_vec_kernel — any seqlen, same unit-stride layout (the
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
#include <type_traits>

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

// Arguments of the decode-step kernel, trimmed to what it reads (one scalar load burst).
struct StepArgs {
    const void *x;
    void *out;
    void *conv_state;
    const void *weight;           // packed (dim, W): fp32 or x's own type (template WM)
    const void *bias;             // same type, or NULL
    const int32_t *cache_seqlens;
    const int32_t *conv_state_indices;
    int64_t x_stride_b, out_stride_b, state_stride_b, state_stride_l;
    int32_t batch, state_len;
    uint32_t n_colgroups;
};

// Taps and bias of a workgroup's 64 adjacent column groups (one per lane), fetched once by the
// whole workgroup and handed to the lanes through LDS.  They are the same for every wavefront
// of the workgroup and make up more bytes per lane than a decode step's data, so this takes a
// quarter of the vector-memory instructions that per-lane loads of them would.  Column group g
// owns kTapUnits consecutive 8-byte units in memory; request() has every thread fetch one
// 16-byte pair of units per trip (one unit when a column group has an odd number of them) and
// one unit of the bias, publish() parks them as staged[unit][lane] (read back without bank
// conflicts; see CC1D_TAPS_PAD for the writes), and after a barrier collect() gives a lane its own.  Callers issue request()
// first and their data loads right behind it, so the LDS round trip happens while the data is
// in flight.
constexpr int kStepWaves = kBlock / kWave;
// Extra 8-byte entries per row of the staging array.  collect() reads a row lane by lane and
// never conflicts; publish() writes a thread's units into rows 1 KiB apart, a 4-way bank
// conflict: SQ_LDS_BANK_CONFLICT counts 69,888 cycles per decode launch over the whole chip
// (273 per CU) out of 204,288 LDS-active cycles.  A pad of 2 entries spreads the rows over the
// 32 banks (5,376 conflict cycles left, from the bias rows) but the row stride is then no power
// of two, and the launch measured 0.05 us slower (4.66 against 4.61 us) five times out of five:
// the conflicts are not on the critical path, the address arithmetic is.  Hence 0.
#ifndef CC1D_TAPS_PAD
#define CC1D_TAPS_PAD 0
#endif
constexpr int kTapRow = kWave + CC1D_TAPS_PAD;

template <class Taps, int CH, int W>
struct WorkgroupTaps {
    static constexpr int kTapUnits = Taps::kWords / 2, kBiasUnits = Taps::kBiasWords / 2;
    static constexpr int kUnits = kTapUnits + kBiasUnits;          // rows of the LDS array
    static constexpr int kElem = Taps::k32 ? 4 : 2;
    static constexpr bool kPairs = kTapUnits % 2 == 0;
    static constexpr int kPieces = kPairs ? kWave * kTapUnits / 2 : kWave * kTapUnits;   // per workgroup
    static constexpr int kTrips = (kPieces + kBlock - 1) / kBlock;
    static_assert(Taps::kWords % 2 == 0 && Taps::kBiasWords % 2 == 0, "staged in 8-byte units");
    static_assert(kWave * kBiasUnits <= kBlock, "one trip for the bias");
    u32x4 piece[kTrips];
    u32x2 bias_unit;

    // col0: the workgroup's first column group; cols_here: how many of its 64 exist.
    __device__ __forceinline__ void request(const void *weight, const void *bias, uint32_t col0, uint32_t cols_here) {
        const char *wsrc = reinterpret_cast<const char *>(weight) + (int64_t)col0 * (CH * W * kElem);
        const char *bsrc = reinterpret_cast<const char *>(bias) + (int64_t)col0 * (CH * kElem);
#pragma unroll
        for (int q = 0; q < kTrips; ++q) {
            const uint32_t pi = (uint32_t)q * kBlock + threadIdx.x;
            piece[q] = u32x4{0u, 0u, 0u, 0u};
            if (pi < cols_here * (uint32_t)(kPieces / kWave)) {
                if constexpr (kPairs) {
                    piece[q] = reinterpret_cast<const u32x4 *>(wsrc)[pi];
                } else {
                    const u32x2 v = reinterpret_cast<const u32x2 *>(wsrc)[pi];
                    piece[q].x = v.x;
                    piece[q].y = v.y;
                }
            }
        }
        bias_unit = u32x2{0u, 0u};
        if (bias != nullptr && threadIdx.x < cols_here * (uint32_t)kBiasUnits)
            bias_unit = reinterpret_cast<const u32x2 *>(bsrc)[threadIdx.x];
    }
    __device__ __forceinline__ void publish(u32x2 (&staged)[kUnits][kTapRow]) const {
#pragma unroll
        for (int q = 0; q < kTrips; ++q) {
            const uint32_t pi = (uint32_t)q * kBlock + threadIdx.x;
            if (pi < (uint32_t)kPieces) {
                const uint32_t unit = kPairs ? 2 * pi : pi;
                const uint32_t g = unit / kTapUnits, u = unit % kTapUnits;
                staged[u][g] = u32x2{piece[q].x, piece[q].y};
                if constexpr (kPairs) staged[u + 1][g] = u32x2{piece[q].z, piece[q].w};
            }
        }
        if (threadIdx.x < (uint32_t)(kWave * kBiasUnits))
            staged[kTapUnits + threadIdx.x % kBiasUnits][threadIdx.x / kBiasUnits] = bias_unit;
    }
    static __device__ __forceinline__ void collect(const u32x2 (&staged)[kUnits][kTapRow], uint32_t lane, Taps &taps) {
#pragma unroll
        for (int u = 0; u < kTapUnits; ++u) {
            const u32x2 v = staged[u][lane];
            taps.wraw[2 * u] = v.x;
            taps.wraw[2 * u + 1] = v.y;
        }
#pragma unroll
        for (int u = 0; u < kBiasUnits; ++u) {
            const u32x2 v = staged[kTapUnits + u][lane];
            taps.braw[2 * u] = v.x;
            taps.braw[2 * u + 1] = v.y;
        }
    }
};

// conv_state rows are read and written with the non-temporal policy: a step touches every state
// row of its layer exactly once, and by the time the same layer's next step comes round a model's
// other layers have been through the caches.  At (256, 5376) bf16, width 4, plain / non-temporal,
// us per launch: state (.., 3) shifted in place 4.59 / 4.17-4.37 on one set of buffers and 6.80 / 5.58
// over 40 rotating sets; ring buffer (.., 8) 4.13 / 4.22 and 5.89 / 4.99.  (Loads alone: 4.60 / 5.98 and
// 4.17 / 5.37; stores alone: 4.52 / 6.76 and 3.96 / 5.58.)  x and out keep the plain policy: the
// non-temporal one measured 0.1 us slower for them.  So do the rows in front of the window that a
// state longer than the window shifts along in place: (.., 8) shifted, 7.5 us on one set with the
// plain policy for them against 10.8 us with the non-temporal one.
template <typename V>
__device__ __forceinline__ V ld_state(const V *p) { return __builtin_nontemporal_load(p); }
template <typename V>
__device__ __forceinline__ void st_state(V *p, const V &v) { __builtin_nontemporal_store(v, p); }

// Decode step, one token.  A workgroup takes 64 adjacent column groups (one per lane) of
// 4 x R batch entries (R per wavefront): grid x = blocks of 64 column groups, y = batch / (4 R).
// The taps come through WorkgroupTaps.
template <int DT, int CH, int W, bool CIRC, bool SILU, int R, int WM>
__global__ void __launch_bounds__(kBlock)
update_step_kernel(const StepArgs a) {
    using E = Elem<DT>;
    using T = typename E::type;
    using P = Pack<DT, CH>;
    using raw_t = typename P::raw_t;
    using Taps = PackedTaps<W, CH, (WM == 1 ? CC1D_F32 : DT)>;
    constexpr bool PRECISE = E::kPreciseAct;
    using Staging = WorkgroupTaps<Taps, CH, W>;
    __shared__ u32x2 staged[Staging::kUnits][kTapRow];

    const uint32_t lc = threadIdx.x & (kWave - 1);
    const int wave_row = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const uint32_t col0 = blockIdx.x * (uint32_t)kWave;            // < n_colgroups by the grid's size
    const uint32_t cols_here = a.n_colgroups - col0 < (uint32_t)kWave ? a.n_colgroups - col0 : (uint32_t)kWave;
    // Lanes past the last column group shadow the block's first one: every address they form
    // is valid, and they store nothing.
    const bool col_ok = lc < cols_here;
    const int c0 = (int)(col0 + (col_ok ? lc : 0u)) * CH;
    const int S = a.state_len;
    const T *xb = reinterpret_cast<const T *>(a.x);
    T *ob = reinterpret_cast<T *>(a.out);
    T *sbase = reinterpret_cast<T *>(a.conv_state);

    Staging staging;
    staging.request(a.weight, a.bias, col0, cols_here);

    // Everything this lane reads is requested up front.
    raw_t rw[R][W - 1], xr[R];
    int64_t soff[R];
    int wpos[R];
    bool live[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int b = ((int)blockIdx.y * kStepWaves + wave_row) * R + r;
        live[r] = b < a.batch;
        const int bb = live[r] ? b : 0;
        const int srow = a.conv_state_indices == nullptr ? bb : a.conv_state_indices[bb];
        live[r] = live[r] && srow >= 0;
        soff[r] = (int64_t)(srow < 0 ? 0 : srow) * a.state_stride_b + c0;
        int cs = 0;
        if (CIRC) cs = positive_mod(a.cache_seqlens[bb], S);
        wpos[r] = cs;
#pragma unroll
        for (int i = 0; i < W - 1; ++i) {
            const int l = CIRC ? wrap(cs - (W - 1) + i, S) : S - (W - 1) + i;
            rw[r][i] = ld_state(reinterpret_cast<const raw_t *>(sbase + soff[r] + (int64_t)l * a.state_stride_l));
        }
        xr[r] = *reinterpret_cast<const raw_t *>(xb + (int64_t)bb * a.x_stride_b + c0);
    }

    staging.publish(staged);
    __syncthreads();
    Taps taps;
    Staging::collect(staged, lc, taps);
    float wv[CH][W], bv[CH];
    taps.finish(a.bias != nullptr, wv, bv);
    if (!col_ok) return;

#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int b = ((int)blockIdx.y * kStepWaves + wave_row) * R + r;
        if (b >= a.batch) continue;
        raw_t *orow = reinterpret_cast<raw_t *>(ob + (int64_t)b * a.out_stride_b + c0);
        if (!live[r]) {                               // padding slot: zeros out, state untouched
            *orow = P::zero();
            continue;
        }
        T *st = sbase + soff[r];
        if (CIRC) {
            st_state(reinterpret_cast<raw_t *>(st + (int64_t)wpos[r] * a.state_stride_l), xr[r]);
        } else {
            // new_state = concat(state, x)[-S:]: rows in front of the window move up by one
            // (reads run ahead of writes), the window rows come straight from registers.
            const int head = S - (W - 1);             // rows in front of the window
            for (int j = 0; j + 1 < head; ++j)
                *reinterpret_cast<raw_t *>(st + (int64_t)j * a.state_stride_l) =
                    *reinterpret_cast<const raw_t *>(st + (int64_t)(j + 1) * a.state_stride_l);
            if (head > 0) st_state(reinterpret_cast<raw_t *>(st + (int64_t)(head - 1) * a.state_stride_l), rw[r][0]);
#pragma unroll
            for (int k = 0; k < W - 2; ++k)
                st_state(reinterpret_cast<raw_t *>(st + (int64_t)(head + k) * a.state_stride_l), rw[r][k + 1]);
            st_state(reinterpret_cast<raw_t *>(st + (int64_t)(S - 1) * a.state_stride_l), xr[r]);
        }
        float xv[CH], acc[CH], f[W - 1][CH];
#pragma unroll
        for (int k = 0; k < W - 1; ++k) P::unpack(rw[r][k], f[k]);
        P::unpack(xr[r], xv);
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            float s = bv[j];
#pragma unroll
            for (int k = 0; k < W - 1; ++k) s = fmaf(wv[j][k], f[k][j], s);
            s = fmaf(wv[j][W - 1], xv[j], s);
            acc[j] = SILU ? silu<PRECISE>(s) : s;
        }
        *orow = P::pack(acc);
    }
}

// A few tokens per call (2 .. kMaxTokens, speculative decoding): one batch row per lane, every
// x row and the window requested up front under wave-uniform predicates, then the tokens are
// produced in order from registers.  A workgroup takes 64 adjacent column groups of 4 batch
// entries (one per wavefront): grid x = blocks of 64 column groups, y = batch / 4.  The taps
// come through WorkgroupTaps.
constexpr int kMaxTokens = 8;

struct TokensArgs {
    StepArgs s;
    int64_t x_stride_l, out_stride_l;
    int32_t seqlen;
};

template <int DT, int CH, int W, bool CIRC, bool SILU, int WM>
__global__ void __launch_bounds__(kBlock)
update_tokens_kernel(const TokensArgs ta) {
    using E = Elem<DT>;
    using T = typename E::type;
    using P = Pack<DT, CH>;
    using raw_t = typename P::raw_t;
    constexpr bool PRECISE = E::kPreciseAct;
    using Taps = PackedTaps<W, CH, (WM == 1 ? CC1D_F32 : DT)>;
    using Staging = WorkgroupTaps<Taps, CH, W>;
    __shared__ u32x2 staged[Staging::kUnits][kTapRow];
    const StepArgs &a = ta.s;

    const uint32_t lc = threadIdx.x & (kWave - 1);
    const uint32_t col0 = blockIdx.x * (uint32_t)kWave;            // < n_colgroups by the grid's size
    const uint32_t cols_here = a.n_colgroups - col0 < (uint32_t)kWave ? a.n_colgroups - col0 : (uint32_t)kWave;
    // Lanes past the last column group and wavefronts past the last batch entry shadow valid
    // ones (every address they form is valid) up to the barrier and store nothing.
    const bool col_ok = lc < cols_here;
    const int c0 = (int)(col0 + (col_ok ? lc : 0u)) * CH;
    const int b_raw = (int)blockIdx.y * kStepWaves + __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const bool b_ok = b_raw < a.batch;
    const int b = b_ok ? b_raw : 0;
    const int S = a.state_len;
    const int L = ta.seqlen;                          // 2 .. kMaxTokens
    const T *xrow = reinterpret_cast<const T *>(a.x) + (int64_t)b * a.x_stride_b + c0;
    T *orow = reinterpret_cast<T *>(a.out) + (int64_t)b * a.out_stride_b + c0;

    Staging staging;
    staging.request(a.weight, a.bias, col0, cols_here);

    const int srow = a.conv_state_indices == nullptr ? b : a.conv_state_indices[b];
    T *st = reinterpret_cast<T *>(a.conv_state) + (int64_t)(srow < 0 ? 0 : srow) * a.state_stride_b + c0;
    int cs = 0;
    if (CIRC) cs = positive_mod(a.cache_seqlens[b], S);

    raw_t rw[W - 1], xr[kMaxTokens];
#pragma unroll
    for (int i = 0; i < W - 1; ++i) {
        const int l = CIRC ? wrap(cs - (W - 1) + i, S) : S - (W - 1) + i;
        rw[i] = ld_state(reinterpret_cast<const raw_t *>(st + (int64_t)l * a.state_stride_l));
    }
#pragma unroll
    for (int i = 0; i < kMaxTokens; ++i) {
        xr[i] = P::zero();
        if (i < L) xr[i] = *reinterpret_cast<const raw_t *>(xrow + (int64_t)i * ta.x_stride_l);
    }

    staging.publish(staged);
    __syncthreads();
    Taps taps;
    Staging::collect(staged, lc, taps);
    if (!col_ok || !b_ok) return;
    if (srow < 0) {                                   // padding slot: zeros out, state untouched
        for (int i = 0; i < L; ++i) *reinterpret_cast<raw_t *>(orow + (int64_t)i * ta.out_stride_l) = P::zero();
        return;
    }

    if (CIRC) {
        int wpos = cs;
#pragma unroll
        for (int i = 0; i < kMaxTokens; ++i) {
            if (i < L) {
                st_state(reinterpret_cast<raw_t *>(st + (int64_t)wpos * a.state_stride_l), xr[i]);
                wpos = wpos + 1 == S ? 0 : wpos + 1;
            }
        }
    } else {
        // new_state[j] = concat(state, x)[L + j].  Rows in front of the window come from
        // memory (reads run ahead of writes), window rows and x rows from registers.
        const int head = S - (W - 1);
        for (int j = 0; j + L < head; ++j)
            *reinterpret_cast<raw_t *>(st + (int64_t)j * a.state_stride_l) =
                *reinterpret_cast<const raw_t *>(st + (int64_t)(j + L) * a.state_stride_l);
#pragma unroll
        for (int k = 0; k < W - 1; ++k) {
            const int j = head + k - L;
            if (j >= 0) st_state(reinterpret_cast<raw_t *>(st + (int64_t)j * a.state_stride_l), rw[k]);
        }
#pragma unroll
        for (int i = 0; i < kMaxTokens; ++i) {
            const int j = S - L + i;
            if (i < L && j >= 0) st_state(reinterpret_cast<raw_t *>(st + (int64_t)j * a.state_stride_l), xr[i]);
        }
    }

    float wv[CH][W], bv[CH];
    taps.finish(a.bias != nullptr, wv, bv);
    float f[W - 1][CH];
#pragma unroll
    for (int k = 0; k < W - 1; ++k) P::unpack(rw[k], f[k]);
#pragma unroll
    for (int i = 0; i < kMaxTokens; ++i) {
        if (i < L) {
            float xv[CH], acc[CH];
            P::unpack(xr[i], xv);
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                float z = bv[j];
#pragma unroll
                for (int k = 0; k < W - 1; ++k) z = fmaf(wv[j][k], f[k][j], z);
                z = fmaf(wv[j][W - 1], xv[j], z);
                acc[j] = SILU ? silu<PRECISE>(z) : z;
            }
            *reinterpret_cast<raw_t *>(orow + (int64_t)i * ta.out_stride_l) = P::pack(acc);
#pragma unroll
            for (int k = 0; k < W - 2; ++k)
#pragma unroll
                for (int j = 0; j < CH; ++j) f[k][j] = f[k + 1][j];
#pragma unroll
            for (int j = 0; j < CH; ++j) f[W - 2][j] = xv[j];
        }
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

// Decode step, one token, for conv_state with unit stride along state_len: the (batch, dim,
// state_len) contiguous cache that mamba_ssm's Mamba block allocates (state_len = d_conv) and the
// (slots, dim, width - 1) cache of paged servers, where a channel's whole state is state_len
// consecutive elements.  A lane owns CH adjacent channels, the fewest whose states fill whole
// accesses of VB bytes (two channels of four bf16 states: one 16-byte vector; two channels of three
// bf16 states: three words ...): it loads them once, shifts every state by one position in
// registers (new_state = concat(state, x)[-state_len:], csrc/causal_conv1d_update.cu:72-84,95-98)
// and stores them once; x and out of those channels are one access each.  A workgroup takes 64
// adjacent channel groups (one per lane) of 4 batch entries (one per wavefront): grid x = channel
// groups / 64, y = batch / 4, and its taps are fetched once where their layout allows it.  Same
// arithmetic, in the same order, as the other update kernels; the state moves as raw bits.
// (256, 5120) bf16, on the same buffers every call / on 40 sets of buffers in turn: state_len 4
// 4.1-4.4 / 6.1-6.3 us (12.4 / 14.6 us with one element access per state position; 4.7 / 6.1 us for
// the cache with unit stride along dim), state_len 3 4.5-4.7 / 5.8-5.9 us (4.3 / 5.5), state_len 8
// 6.1-6.5 / 9.6-9.7 us (7.0 / 13.3).  Two batch entries per lane measured the same or slower.
// TAPS: how a lane gets its taps.  1 / 2: packed fp32 / packed in the tensors' own 16-bit type and
// staged once per workgroup through WorkgroupTaps (CH must give whole 8-byte units); 3: packed
// 16-bit, read per lane in whole words; 0: any layout and type, per lane.
// Bytes per access to the state: 16 where a state divides 16 bytes or is a multiple of them; 4 for
// the others (states of 6 or 12 bytes: three elements), where more and narrower lanes measured
// faster: (256, 5120), state_len 3, 16- / 8- / 4-byte accesses: bf16 6.2 / 5.1 / 4.7 us, fp32 9.0 / 8.5 / 7.3 us.
#ifndef CC1D_RS_VB
#define CC1D_RS_VB(state_bytes) ((16 % (state_bytes) == 0 || (state_bytes) % 16 == 0) ? 16 : 4)
#endif
template <bool ON, int W, int CH, int WDT> struct RowStateTaps { using type = PackedTaps<W, CH, WDT>; };
template <int W, int CH, int WDT> struct RowStateTaps<false, W, CH, WDT> { struct type {}; };
template <bool ON, class Taps, int CH, int W> struct RowStateStaging { using type = WorkgroupTaps<Taps, CH, W>; };
template <class Taps, int CH, int W> struct RowStateStaging<false, Taps, CH, W> {
    struct type { static constexpr int kUnits = 1; };
};

template <int DT, int W, int S, int CH, int VB, int TAPS>
__global__ void __launch_bounds__(kBlock)
update_rowstate_kernel(const cc1d_update_params p, const uint32_t n_groups, const int w_contiguous_f32) {
    using E = Elem<DT>;
    using T = typename E::type;
    using vec_t = typename RawBytes<VB>::type;        // one access to the state
    constexpr bool PRECISE = E::kPreciseAct;
    constexpr int NV = CH * S * E::kBytes / VB;       // vectors of state per lane
    constexpr int XB = CH * E::kBytes;                // bytes of x (and of out) per lane
    static_assert(NV * VB == CH * S * E::kBytes && S >= W - 1, "CH whole states fill whole vectors");
    constexpr bool STAGED = TAPS == 1 || TAPS == 2;
    using Taps = typename RowStateTaps<TAPS != 0, W, CH, (TAPS == 1 ? CC1D_F32 : DT)>::type;
    using Staging = typename RowStateStaging<STAGED, Taps, CH, W>::type;
    __shared__ u32x2 staged[Staging::kUnits][kTapRow];

    const uint32_t lc = threadIdx.x & (kWave - 1);
    const uint32_t col0 = blockIdx.x * (uint32_t)kWave;            // < n_groups by the grid's size
    const uint32_t cols_here = n_groups - col0 < (uint32_t)kWave ? n_groups - col0 : (uint32_t)kWave;
    // Lanes past the last channel group shadow the block's first one: every address they form is
    // valid, and they store nothing.
    const bool col_ok = lc < cols_here;
    const int c0 = (int)(col0 + (col_ok ? lc : 0u)) * CH;
    const int b = (int)blockIdx.y * kStepWaves + __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const bool silu_on = p.silu != 0;

    Staging staging;
    Taps taps;
    if constexpr (STAGED) staging.request(p.weight, p.bias, col0, cols_here);
    if constexpr (TAPS == 3) taps.request(p.weight, p.bias, c0);

    // Wavefronts past the last batch entry and those of a padding slot load nothing.
    int srow = -1;
    if (b < p.batch) srow = p.conv_state_indices == nullptr ? b : p.conv_state_indices[b];
    const bool live = srow >= 0;
    vec_t *sp = reinterpret_cast<vec_t *>(reinterpret_cast<T *>(p.conv_state) + (int64_t)(live ? srow : 0) * p.state_stride_b +
                                          (int64_t)c0 * S);
    vec_t raw[NV];
    T xe[CH];
    if (live) {
#pragma unroll
        for (int v = 0; v < NV; ++v) raw[v] = ld_state(sp + v);
        const T *xrow = reinterpret_cast<const T *>(p.x) + (int64_t)b * p.x_stride_b + c0;
        if constexpr (XB >= 4) {                      // one access: the host checked its alignment
            using raw_t = typename RawBytes<XB>::type;
            const raw_t xr = *reinterpret_cast<const raw_t *>(xrow);
            __builtin_memcpy(xe, &xr, sizeof xr);
        } else {
            xe[0] = xrow[0];
        }
    }
    float wv[CH][W], bv[CH];
    if constexpr (STAGED) {
        staging.publish(staged);
        __syncthreads();
        Staging::collect(staged, lc, taps);
    }
    if constexpr (TAPS != 0) {
        taps.finish(p.bias != nullptr, wv, bv);
    } else {
        load_weights<W, CH>(p.weight, p.bias, p.w_dtype, p.w_stride_c, p.w_stride_w, w_contiguous_f32 != 0, c0, wv, bv);
    }
    if (!col_ok || b >= p.batch) return;

    T oe[CH];
    if (live) {
        T se[CH * S], ne[CH * S];
        __builtin_memcpy(se, raw, sizeof raw);
#pragma unroll
        for (int j = 0; j < CH; ++j) {
#pragma unroll
            for (int q = 0; q + 1 < S; ++q) ne[j * S + q] = se[j * S + q + 1];
            ne[j * S + S - 1] = xe[j];
        }
        vec_t next[NV];
        __builtin_memcpy(next, ne, sizeof next);
#pragma unroll
        for (int v = 0; v < NV; ++v) st_state(sp + v, next[v]);
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            float a = bv[j];
#pragma unroll
            for (int k = 0; k < W - 1; ++k) a = fmaf(wv[j][k], E::to_float(se[j * S + S - (W - 1) + k]), a);
            a = fmaf(wv[j][W - 1], E::to_float(xe[j]), a);
            oe[j] = E::from_float(silu_on ? silu<PRECISE>(a) : a);
        }
    } else {                                          // padding slot: zeros out, state untouched
#pragma unroll
        for (int j = 0; j < CH; ++j) oe[j] = T(0.f);
    }
    T *orow = reinterpret_cast<T *>(p.out) + (int64_t)b * p.out_stride_b + c0;
    if constexpr (XB >= 4) {
        using raw_t = typename RawBytes<XB>::type;
        raw_t o;
        __builtin_memcpy(&o, oe, sizeof o);
        *reinterpret_cast<raw_t *>(orow) = o;
    } else {
        orow[0] = oe[0];
    }
}

// (rows x dim)-shaped operand usable as 16-byte vectors along dim.
bool rows_vec_ok(const void *ptr, int dtype, int64_t sb, int64_t sc, int64_t sl, int n_rows) {
    const int v = vec_elems(dtype);
    return sc == 1 && sb % v == 0 && (n_rows <= 1 || sl % v == 0) && aligned16(ptr);
}

// (rows x dim)-shaped operand usable as `lane_bytes`-wide vectors along dim.
bool rows_lane_ok(const void *ptr, int dtype, int lane_bytes, int64_t sb, int64_t sc, int64_t sl, int n_rows) {
    const int v = lane_bytes / elem_bytes(dtype);
    return sc == 1 && sb % v == 0 && (n_rows <= 1 || sl % v == 0) &&
           (reinterpret_cast<uintptr_t>(ptr) % lane_bytes) == 0;
}

constexpr int kStepLaneBytes = 8;
#ifndef CC1D_UPDATE_STEP_ROWS
#define CC1D_UPDATE_STEP_ROWS 2
#endif
constexpr int kStepRows = CC1D_UPDATE_STEP_ROWS;   // batch rows per lane

template <int DT, int W>
int launch_w(const cc1d_update_params &p, bool vec, hipStream_t stream) {
    const bool circ = p.cache_seqlens != nullptr;
    constexpr int CH = kStepLaneBytes / Elem<DT>::kBytes;
    // Taps packed (dim, W) in fp32 or in x's own type, as callers in practice pass them;
    // anything else takes the general kernels below.
    const int mode = weights_mode(p.weight, p.bias, p.w_dtype, DT, p.w_stride_c, p.w_stride_w, p.width);
    const bool step = p.seqlen == 1 && p.dim % CH == 0 && p.batch <= 65535 * kStepRows && mode != 0 &&
        rows_lane_ok(p.x, DT, kStepLaneBytes, p.x_stride_b, p.x_stride_c, p.x_stride_l, 1) &&
        rows_lane_ok(p.out, DT, kStepLaneBytes, p.out_stride_b, p.out_stride_c, p.out_stride_l, 1) &&
        rows_lane_ok(p.conv_state, DT, kStepLaneBytes, p.state_stride_b, p.state_stride_c, p.state_stride_l, p.state_len);
    if (step) {
        StepArgs a;
        a.x = p.x; a.out = p.out; a.conv_state = p.conv_state;
        a.weight = p.weight;
        a.bias = p.bias;
        a.cache_seqlens = p.cache_seqlens; a.conv_state_indices = p.conv_state_indices;
        a.x_stride_b = p.x_stride_b; a.out_stride_b = p.out_stride_b;
        a.state_stride_b = p.state_stride_b; a.state_stride_l = p.state_stride_l;
        a.batch = p.batch; a.state_len = p.state_len;
        a.n_colgroups = (uint32_t)(p.dim / CH);
        const dim3 grid((a.n_colgroups + kWave - 1) / kWave,
                        (uint32_t)((p.batch + kStepWaves * kStepRows - 1) / (kStepWaves * kStepRows)));
        if ((int64_t)grid.x * grid.y * kBlock >= thread_limit()) return CC1D_ERR_TOO_LARGE;
        auto launch = [&](auto wm) {
            constexpr int WM = decltype(wm)::value;
            if (circ) {
                if (p.silu) CC1D_LAUNCH((update_step_kernel<DT, CH, W, true, true, kStepRows, WM>), grid, dim3(kBlock), 0, stream, a);
                else CC1D_LAUNCH((update_step_kernel<DT, CH, W, true, false, kStepRows, WM>), grid, dim3(kBlock), 0, stream, a);
            } else {
                if (p.silu) CC1D_LAUNCH((update_step_kernel<DT, CH, W, false, true, kStepRows, WM>), grid, dim3(kBlock), 0, stream, a);
                else CC1D_LAUNCH((update_step_kernel<DT, CH, W, false, false, kStepRows, WM>), grid, dim3(kBlock), 0, stream, a);
            }
        };
        if (mode == 1) launch(std::integral_constant<int, 1>{});
        else if constexpr (DT != CC1D_F32) launch(std::integral_constant<int, 2>{});
        return launch_status();
    }
    const bool tokens = p.seqlen >= 2 && p.seqlen <= kMaxTokens && p.dim % CH == 0 && p.batch <= 65535 && mode != 0 &&
        rows_lane_ok(p.x, DT, kStepLaneBytes, p.x_stride_b, p.x_stride_c, p.x_stride_l, p.seqlen) &&
        rows_lane_ok(p.out, DT, kStepLaneBytes, p.out_stride_b, p.out_stride_c, p.out_stride_l, p.seqlen) &&
        rows_lane_ok(p.conv_state, DT, kStepLaneBytes, p.state_stride_b, p.state_stride_c, p.state_stride_l, p.state_len);
    if (tokens) {
        TokensArgs ta;
        StepArgs &a = ta.s;
        a.x = p.x; a.out = p.out; a.conv_state = p.conv_state;
        a.weight = p.weight;
        a.bias = p.bias;
        a.cache_seqlens = p.cache_seqlens; a.conv_state_indices = p.conv_state_indices;
        a.x_stride_b = p.x_stride_b; a.out_stride_b = p.out_stride_b;
        a.state_stride_b = p.state_stride_b; a.state_stride_l = p.state_stride_l;
        a.batch = p.batch; a.state_len = p.state_len;
        a.n_colgroups = (uint32_t)(p.dim / CH);
        ta.x_stride_l = p.x_stride_l; ta.out_stride_l = p.out_stride_l; ta.seqlen = p.seqlen;
        const dim3 grid((a.n_colgroups + kWave - 1) / kWave, (uint32_t)((p.batch + kStepWaves - 1) / kStepWaves));
        if ((int64_t)grid.x * grid.y * kBlock >= thread_limit()) return CC1D_ERR_TOO_LARGE;
        auto launch = [&](auto wm) {
            constexpr int WM = decltype(wm)::value;
            if (circ) {
                if (p.silu) CC1D_LAUNCH((update_tokens_kernel<DT, CH, W, true, true, WM>), grid, dim3(kBlock), 0, stream, ta);
                else CC1D_LAUNCH((update_tokens_kernel<DT, CH, W, true, false, WM>), grid, dim3(kBlock), 0, stream, ta);
            } else {
                if (p.silu) CC1D_LAUNCH((update_tokens_kernel<DT, CH, W, false, true, WM>), grid, dim3(kBlock), 0, stream, ta);
                else CC1D_LAUNCH((update_tokens_kernel<DT, CH, W, false, false, WM>), grid, dim3(kBlock), 0, stream, ta);
            }
        };
        if (mode == 1) launch(std::integral_constant<int, 1>{});
        else if constexpr (DT != CC1D_F32) launch(std::integral_constant<int, 2>{});
        return launch_status();
    }
    // conv_state (batch, dim, state_len) with unit stride along state_len: the row-state kernel, for the
    // state lengths in use (2, 3, 4, 8) when dim is a whole number of lanes' channel groups and a
    // lane's accesses to the state, x and out are aligned.
    if (p.seqlen == 1 && !circ && p.state_stride_l == 1 && p.state_stride_c == p.state_len && p.x_stride_c == 1 &&
        p.out_stride_c == 1 && p.state_len >= W - 1 && p.batch <= 65535 * kStepWaves) {
        bool launched = false, too_large = false;
        auto run = [&](auto sc) {
            constexpr int SC = decltype(sc)::value;
            if constexpr (SC >= W - 1) {
                constexpr int kStateBytes = SC * Elem<DT>::kBytes;
                // A lane takes the fewest channels whose states fill whole accesses of VB bytes:
                // VB / gcd(VB, state bytes).
                constexpr int VB = CC1D_RS_VB(kStateBytes);
                constexpr int kGcd = kStateBytes % VB == 0 ? VB : kStateBytes % 8 == 0 && VB >= 8 ? 8 : kStateBytes % 4 == 0 ? 4 : 2;
                constexpr int CHC = VB / kGcd;
                constexpr int kLaneBytes = CHC * Elem<DT>::kBytes;
                if (p.dim % CHC != 0 || reinterpret_cast<uintptr_t>(p.conv_state) % VB != 0 ||
                    (p.state_stride_b * (int64_t)Elem<DT>::kBytes) % VB != 0) return;
                if (kLaneBytes >= 4 &&
                    (!rows_lane_ok(p.x, DT, kLaneBytes, p.x_stride_b, 1, 0, 1) ||
                     !rows_lane_ok(p.out, DT, kLaneBytes, p.out_stride_b, 1, 0, 1))) return;
                const uint32_t n_groups = (uint32_t)(p.dim / CHC);
                const dim3 grid((n_groups + kWave - 1) / kWave, (uint32_t)((p.batch + kStepWaves - 1) / kStepWaves));
                if ((int64_t)grid.x * grid.y * kBlock >= thread_limit()) { too_large = true; return; }
                const int w_fast = weights_contiguous_f32(p.weight, p.w_dtype, p.w_stride_c, p.w_stride_w, p.width);
                constexpr bool kStage32 = CHC % 2 == 0;
                constexpr bool kStage16 = DT != CC1D_F32 && CHC % 4 == 0;
                constexpr bool kLane16 = DT != CC1D_F32 && CHC % 2 == 0 && !kStage16;
                if (mode == 1 && kStage32) {
                    if constexpr (kStage32)
                        CC1D_LAUNCH((update_rowstate_kernel<DT, W, SC, CHC, VB, 1>), grid, dim3(kBlock), 0, stream, p, n_groups, w_fast);
                } else if (mode == 2 && kStage16) {
                    if constexpr (kStage16)
                        CC1D_LAUNCH((update_rowstate_kernel<DT, W, SC, CHC, VB, 2>), grid, dim3(kBlock), 0, stream, p, n_groups, w_fast);
                } else if (mode == 2 && kLane16) {
                    if constexpr (kLane16)
                        CC1D_LAUNCH((update_rowstate_kernel<DT, W, SC, CHC, VB, 3>), grid, dim3(kBlock), 0, stream, p, n_groups, w_fast);
                } else {
                    CC1D_LAUNCH((update_rowstate_kernel<DT, W, SC, CHC, VB, 0>), grid, dim3(kBlock), 0, stream, p, n_groups, w_fast);
                }
                launched = true;
            }
        };
        switch (p.state_len) {
            case 2: run(std::integral_constant<int, 2>{}); break;
            case 3: run(std::integral_constant<int, 3>{}); break;
            case 4: run(std::integral_constant<int, 4>{}); break;
            case 8: run(std::integral_constant<int, 8>{}); break;
            default: break;
        }
        if (too_large) return CC1D_ERR_TOO_LARGE;
        if (launched) return launch_status();
    }
    if (vec) {
        const uint32_t ncg = (uint32_t)(p.dim / Elem<DT>::kVec);
        const int64_t total = (int64_t)p.batch * ncg;
        if (total >= thread_limit()) return CC1D_ERR_TOO_LARGE;
        const uint32_t blocks = (uint32_t)((total + kBlock - 1) / kBlock);
        const int w_fast = weights_contiguous_f32(p.weight, p.w_dtype, p.w_stride_c, p.w_stride_w, p.width);
        if (circ) CC1D_LAUNCH((update_vec_kernel<DT, W, true>), dim3(blocks), dim3(kBlock), 0, stream, p, ncg, (uint32_t)total, w_fast);
        else CC1D_LAUNCH((update_vec_kernel<DT, W, false>), dim3(blocks), dim3(kBlock), 0, stream, p, ncg, (uint32_t)total, w_fast);
    } else {
        const int64_t total = (int64_t)p.batch * p.dim;
        if (total >= thread_limit()) return CC1D_ERR_TOO_LARGE;
        const uint32_t blocks = (uint32_t)((total + kBlock - 1) / kBlock);
        if (circ) CC1D_LAUNCH((update_generic_kernel<DT, W, true>), dim3(blocks), dim3(kBlock), 0, stream, p, (uint32_t)total);
        else CC1D_LAUNCH((update_generic_kernel<DT, W, false>), dim3(blocks), dim3(kBlock), 0, stream, p, (uint32_t)total);
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
