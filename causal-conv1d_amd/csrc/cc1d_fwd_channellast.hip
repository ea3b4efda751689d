// Channel-last forward for gfx950: x is (batch, seqlen, dim) in memory (unit stride
// along dim).  Takes over causal_conv1d_channellast_fwd_kernel and its launcher
// (csrc/causal_conv1d_fwd.cu:205-381 of the reference).
//
// Design.  The stencil runs along seqlen, which is the strided axis, so nothing has to
// be transposed: a lane owns one 4-byte column (two 16-bit channels or one fp32 channel), a
// wavefront 64 adjacent columns of one run of T consecutive rows (T = 16).  The wavefront
// asks for all T + W-1 rows of its run at once, and the data goes from memory straight into
// LDS (buffer_load ... lds: no VGPRs are held while a row is in flight, so the rows in flight
// per CU are bounded by the 160 KB of LDS, not by registers, and eight wavefronts fit a SIMD).
// Every access names its row by a scalar offset into a buffer resource and its column by one
// lane offset that never changes: no vector instruction is spent on addresses.  When the rows
// have landed the lane walks down its column out of LDS with a (W-1)-row window in registers
// as fp32: per row one LDS read, W multiply-adds per channel, the activation, one store.
// No barrier: a wavefront reads only what it fetched itself.  The only rows read twice are
// the W-1 halo rows in front of each run.
//
// Wavefronts are numbered (batch, run, column block) with the column block fastest, four of
// them to a workgroup, and workgroups are renumbered so that each of the 8 XCDs (hardware
// hands workgroups to XCDs round-robin) walks chunks of consecutive runs of that order, the
// XCDs side by side on 8 neighbouring chunks: the run that follows another along seqlen then
// executes on the same XCD, close in time, and finds its halo rows in that XCD's L2, while
// the chip as a whole moves through memory as one front.  For the same reason the halo rows
// and the last W-1 rows of a run are fetched with the normal cache policy and every other row,
// which no other wavefront needs, streams through (non-temporal), as do all stores.
#include <type_traits>

#include "cc1d_varlen_gather.hpp"

#ifndef CC1D_FWD_CL_XCDS
#define CC1D_FWD_CL_XCDS 8
#endif
// Cache policy of the rows no other run reads, and of the stores (buffer instruction aux bits:
// 0 normal, 2 non-temporal).  Measured at the prefill shape (8, 5376, 2048) bf16, the same
// buffers every launch / six rotating sets of buffers: everything normal 50.3 / 58.9 us,
// streaming rows 56.1 / 55.9 us, streaming rows but a normal halo or normal last rows only
// 57.8 / 57.4 and 58.3 / 58.1 us, normal stores 53.7 / 63.5 us.  The first column measures a
// tensor that the previous launch left in the 256 MB last-level cache, which a model's next layer
// does not find; the second is what every layer of a model sees.
#ifndef CC1D_FWD_CL_AUX_STREAM
#define CC1D_FWD_CL_AUX_STREAM 2
#endif
#ifndef CC1D_FWD_CL_AUX_STORE
#define CC1D_FWD_CL_AUX_STORE 2
#endif

namespace cc1d {
namespace {

constexpr int kXcds = CC1D_FWD_CL_XCDS;
constexpr int kGroup = 8;                 // rows computed between two looks at the loop counter
constexpr int kMaxRows = 56;              // 4 wavefronts x (56 + 3) rows x 256 bytes < 64 KB of LDS
constexpr int kRsrcRaw = 0x00020000;      // buffer resource word 3: raw buffer, 32-bit data format

typedef void __attribute__((address_space(3))) *lds_ptr_t;

// What every wavefront reads, in the order it reads it: one block of kernel arguments that a few
// wide scalar loads bring in at once (a wavefront's first vector load waits for them).
struct FwdClArgs {
    uint32_t blocks_per_xcd;   // grid size / 8
    uint32_t blocks_per_chunk; // workgroups an XCD takes in a row before the next XCD's (0: its whole slice)
    uint32_t first_tail_block; // workgroups from here on run the varlen gather
    uint32_t total;            // batch * n_runs * waves_per_row wavefronts
    uint32_t waves_per_row;    // ceil(n_cols / 64): wavefronts side by side on one row
    int32_t n_runs;            // ceil(seqlen / T)
    int32_t rows_per_run;      // T, a multiple of kGroup
    int32_t seqlen;
    int32_t n_cols;            // dim / CH: 4-byte columns of a row
    uint32_t x_row_bytes, out_row_bytes;
    int32_t states;            // bit 0: initial_states given, bit 1: final_states wanted
    const void *x;
    void *out;
    const void *weight;
    const void *bias;
    const int32_t *seq_idx;
    int64_t x_stride_b, out_stride_b;   // elements
};
// What only some wavefronts read (a sequence's first run, the general tap loader, the gather).
struct FwdClRare {
    const void *initial_states;
    void *final_states;
    int64_t init_stride_b, init_stride_c, init_stride_l;
    int64_t final_stride_b, final_stride_c, final_stride_l;
    int64_t w_stride_c, w_stride_w;
    int32_t w_dtype;
    uint32_t tail_n_colgroups, tail_total;
    cc1d_varlen_params tail;
};

// WM: how the taps are read.  1: packed (dim, W) fp32, 2: packed in x's own 16-bit type (both
// through PackedTaps), 0: any layout and type (general loader).
// TS: rows per run as a compile-time constant (the default run length: the loops over a run's rows
// unroll, 0.4 us at the prefill shape), or 0 for the run length in the arguments.
template <int DT, int W, bool HAS_SEQ, bool SILU, int WM, int TS>
__global__ void __launch_bounds__(kBlock, 4)
fwd_channellast_kernel(const FwdClArgs a, const FwdClRare q) {
    using E = Elem<DT>;
    using T_ = typename E::type;
    constexpr int CH = 4 / E::kBytes;
    using P = Pack<DT, CH>;
    using raw_t = typename P::raw_t;
    constexpr bool PRECISE = E::kPreciseAct;
    extern __shared__ uint32_t lds[];                 // [4 wavefronts][T + W-1 rows][64 lanes]

    // Workgroups past the forward's own are there for the varlen final-state gather, which
    // reads x only and so needs no ordering against the rows being produced.
    if (blockIdx.x >= a.first_tail_block) {
        varlen_gather_vec<DT>(q.tail, q.tail_n_colgroups, q.tail_total,
                              (blockIdx.x - a.first_tail_block) * (uint32_t)kBlock + threadIdx.x);
        return;
    }
    // XCD x executes workgroups x, x+8, x+16, ...
    const uint32_t xcd = blockIdx.x % kXcds, nth = blockIdx.x / kXcds;
    const uint32_t block = a.blocks_per_chunk == 0
                               ? xcd * a.blocks_per_xcd + nth
                               : ((nth / a.blocks_per_chunk) * kXcds + xcd) * a.blocks_per_chunk + nth % a.blocks_per_chunk;
    // A wavefront never straddles two runs: its batch index, run and row range are scalars,
    // and so are the sub-sequence ids it reads.
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const int lane = (int)(threadIdx.x & (kWave - 1));
    const uint32_t wave = block * (uint32_t)(kBlock / kWave) + (uint32_t)wv;
    if (wave >= a.total) return;
    const uint32_t col = (wave % a.waves_per_row) * (uint32_t)kWave + (uint32_t)lane;
    const uint32_t rb = wave / a.waves_per_row;
    const int run = (int)(rb % (uint32_t)a.n_runs);
    const int b = (int)(rb / (uint32_t)a.n_runs);
    const int L = a.seqlen;
    const bool has_init = (a.states & 1) != 0;
    const int T = TS != 0 ? TS : a.rows_per_run;
    const int R = T + W - 1;                          // rows of the run in LDS, halo included
    const int t0 = run * T;                           // < L by construction of n_runs
    const int last = L - 1 - t0;                      // last valid row of this run, run-relative

    // Lanes past the last column (a row that is no whole number of wavefronts) shadow column 0:
    // every address they form is valid, and they store nothing.
    const bool col_ok = col < (uint32_t)a.n_cols;
    const int c0 = col_ok ? (int)col * CH : 0;
    const int lane_off = c0 * (int)sizeof(T_);        // byte offset of the lane's column in a row

    // With seq_idx, lane i looks at the id of row t0 - (W-1) + i of the run (the first thing
    // requested, see below).
    int my_id = 0;
    if (HAS_SEQ) {
        const int t_lane = t0 + lane - (W - 1);
        const int t = t_lane > L - 1 ? L - 1 : t_lane;
        my_id = a.seq_idx[(int64_t)b * L + (t > 0 ? t : 0)];
    }
    // Taps are only requested here: everything the run starts with is in flight before the
    // first value is touched.
    constexpr bool WFAST = WM != 0;
    constexpr bool SCALED = SILU && !PRECISE;
    float wv_[CH][W], bv[CH];
    PackedTaps<W, CH, (WM == 1 ? CC1D_F32 : DT)> taps;
    StridedTaps<W, CH> any_taps;
    if (WFAST) taps.request(a.weight, a.bias, c0);
    else any_taps.request(a.weight, a.bias, q.w_dtype, q.w_stride_c, q.w_stride_w, c0);

    // Buffer resources.  x: base = the run's first halo row (W-1 rows in front of the run; where
    // that lies in front of the tensor those rows are never fetched); out: the run's first row.
    // The lane's column is the vector offset, the row a scalar offset (checked by the launcher
    // to fit 31 bits).
    const uint32_t xs = a.x_row_bytes;
    const uint32_t os = a.out_row_bytes;
    const T_ *xbase = reinterpret_cast<const T_ *>(a.x) + (int64_t)b * a.x_stride_b;
    const char *xrun = reinterpret_cast<const char *>(xbase) + ((int64_t)t0 - (W - 1)) * xs;
    char *orun = reinterpret_cast<char *>(reinterpret_cast<T_ *>(a.out) + (int64_t)b * a.out_stride_b) + (int64_t)t0 * os;
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(xrun), 0, -1, kRsrcRaw);
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(orun, 0, -1, kRsrcRaw);
    uint32_t *mine = lds + wv * R * kWave;            // this wavefront's rows
    auto fetch = [&](auto stream, int r) {
        constexpr int aux = decltype(stream)::value ? CC1D_FWD_CL_AUX_STREAM : 0;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)(mine + r * kWave), 4, lane_off, r * (int)xs, 0, aux);
    };
    using No = std::integral_constant<bool, false>;
    using Yes = std::integral_constant<bool, true>;
    // A run inside the sequence fetches its rows with no test per row: the halo and the last
    // W-1 rows (the halo of the run below) with the normal policy, the rest streaming.
    const bool interior = t0 >= W - 1 && last >= T - 1;
    if (interior) {
#pragma unroll
        for (int r = 0; r < W - 1; ++r) fetch(No{}, r);
        for (int r = W - 1; r < T; ++r) fetch(Yes{}, r);
#pragma unroll
        for (int r = 0; r < W - 1; ++r) fetch(No{}, T + r);
    } else {
        // The first run of a sequence (rows in front of it come from initial_states, or are
        // zero) and its ragged last run (rows behind its end are not fetched: what LDS holds
        // there only reaches outputs that are not stored).
        for (int r = 0; r < R; ++r) {
            const int t = t0 - (W - 1) + r;
            if (t >= 0) {
                if (t < L) fetch(No{}, r);
            } else {
                raw_t v = P::zero();
                if (has_init)
                    v = load_state_row<DT, CH>(q.initial_states, q.init_stride_b, q.init_stride_c,
                                               q.init_stride_l, b, c0, t + (W - 1));
                mine[r * kWave + lane] = v[0];
            }
        }
    }

    // With seq_idx the run is computed as if no sub-sequence boundary were near unless one is:
    // lane i flags row t0 - (W-1) + i when its id differs from the row before (the previous
    // lane's, a lane shift) or is negative; rows in front of the sequence count as id -1 when
    // initial_states are given and as zeros, which no mask changes, otherwise.  A run with a
    // flag takes the masked walk for all of its rows.
    bool masked = false;
    if (HAS_SEQ) {
        const int t_lane = t0 + lane - (W - 1);
        const int id_prev = __builtin_amdgcn_update_dpp(my_id, my_id, 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
        const bool in = lane < R && t_lane <= L - 1;
        const bool flag = in && (t_lane >= 0 ? (my_id < 0 || (t_lane > 0 ? (lane > 0 && my_id != id_prev) : has_init)) : has_init);
        masked = __ballot(flag) != 0;
    }
    // 16-bit outputs with SiLU: taps and bias carry the factor -log2(e), so the sums below
    // are already the exponent the activation needs (see silu_from_scaled).
    if (WFAST) taps.finish(a.bias != nullptr, wv_, bv);
    else any_taps.finish(q.w_dtype, a.bias != nullptr, wv_, bv);
    if (SCALED) {
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            bv[j] *= kSiluPrescale;
#pragma unroll
            for (int k = 0; k < W; ++k) wv_[j][k] *= kSiluPrescale;
        }
    }
    // Every row of the run is in LDS behind this wait (a row fetched into LDS counts as a load
    // until it has been written there).
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    if (col_ok) {
        // Sliding window: xw[k] holds row i - (W-1) + k while row i is being produced.
        float xw[W - 1][CH];
#pragma unroll
        for (int k = 0; k < W - 1; ++k) {
            raw_t r;
            r[0] = mine[k * kWave + lane];
            P::unpack(r, xw[k]);
        }
        // CHECKED: the ragged last run of a sequence, stores past its end are suppressed.
        // MASKED: taps masked row by row (csrc/causal_conv1d_fwd.cu:316-329), padding tokens
        // exactly zero; the id of row q of the run is lane q's.
        auto walk = [&](auto checked, auto with_mask) {
            constexpr bool CHECKED = decltype(checked)::value, MASKED = decltype(with_mask)::value;
            for (int i0 = 0; i0 < T; i0 += kGroup) {
                if (CHECKED && i0 > last) break;
                const uint32_t *rows = mine + (i0 + W - 1) * kWave + lane;
                int ids[kGroup + W - 1];
                if (MASKED) {
#pragma unroll
                    for (int q = 0; q < kGroup + W - 1; ++q) {
                        const int id = __builtin_amdgcn_readlane(my_id, i0 + q);
                        ids[q] = t0 + i0 + q - (W - 1) < 0 ? -1 : id;
                    }
                }
#pragma unroll
                for (int u = 0; u < kGroup; ++u) {
                    raw_t r;
                    r[0] = rows[u * kWave];
                    float xv[CH], acc[CH];
                    P::unpack(r, xv);
                    const int cur = MASKED ? ids[u + W - 1] : 0;
#pragma unroll
                    for (int j = 0; j < CH; ++j) {
                        float a = bv[j];
#pragma unroll
                        // a masked tap takes a zero for its input, not for its weight: what another
                        // sub-sequence or a padding token holds there (it may be Inf or NaN) must not
                        // reach this row, as with the reference's conditional add
                        for (int k = 0; k < W - 1; ++k)
                            a = fmaf(wv_[j][k], MASKED && ids[u + k] != cur ? 0.f : xw[k][j], a);
                        a = fmaf(wv_[j][W - 1], xv[j], a);
                        a = SCALED ? silu_from_scaled(a) : SILU ? silu<PRECISE>(a) : a;
                        acc[j] = MASKED && cur < 0 ? 0.f : a;
                    }
                    if (!CHECKED || i0 + u <= last)
                        __builtin_amdgcn_raw_buffer_store_b32(P::pack(acc)[0], ro, lane_off, (i0 + u) * (int)os,
                                                              CC1D_FWD_CL_AUX_STORE);
#pragma unroll
                    for (int k = 0; k < W - 2; ++k)
#pragma unroll
                        for (int j = 0; j < CH; ++j) xw[k][j] = xw[k + 1][j];
#pragma unroll
                    for (int j = 0; j < CH; ++j) xw[W - 2][j] = xv[j];
                }
            }
        };
        const bool full = last >= T - 1;
        if (HAS_SEQ && masked) {
            if (full) walk(No{}, Yes{});
            else walk(Yes{}, Yes{});
        } else {
            if (full) walk(No{}, No{});
            else walk(Yes{}, No{});
        }
    }

    // final_states[b, c, i] = xpad[L-(W-1)+i], copied from x (or initial_states where L < W-1)
    // by the wavefront of the FIRST run, the one that read initial_states as its halo: the two
    // may be one buffer, and inside one wavefront the reads are complete before the stores.
    if ((a.states & 2) != 0 && run == 0 && col_ok) {
        wait_for_loads();
        raw_t fin[W - 1];
#pragma unroll
        for (int i = 0; i < W - 1; ++i) {
            const int t = L - (W - 1) + i;
            raw_t r = P::zero();
            if (t >= 0) {
                r = *reinterpret_cast<const raw_t *>(reinterpret_cast<const char *>(xbase + c0) + (int64_t)t * xs);
            } else if (has_init) {
                r = load_state_row<DT, CH>(q.initial_states, q.init_stride_b, q.init_stride_c,
                                           q.init_stride_l, b, c0, t + (W - 1));
            }
            fin[i] = r;
        }
        wait_for_loads();                             // rows shorter than W-1 re-read initial_states above
#pragma unroll
        for (int i = 0; i < W - 1; ++i)
            store_state_row<DT, CH>(q.final_states, q.final_stride_b, q.final_stride_c,
                                    q.final_stride_l, b, c0, i, fin[i]);
    }
}

constexpr int kDefaultRows = 16;
constexpr size_t kLdsFloorBytes = 160 * 1024 / 6 / 256 * 256;   // LDS a launch asks for at least: six workgroups to a CU

template <int DT, int W, bool HAS_SEQ, int WM>
int launch_instance(const FwdClArgs &a, const FwdClRare &q, bool silu, hipStream_t stream) {
    const uint32_t blocks = a.first_tail_block + (q.tail_total + kBlock - 1) / kBlock;
    // What the four wavefronts' rows take, and no less than a sixth of a CU's LDS: six workgroups a CU
    // (24 wavefronts, about 110 KB of rows in flight) instead of the eight that would fit measured
    // 1-3 % faster at every size -- prefill shape 56.9 -> 56.0 us, (16, 5376, 2048) bf16 110.1 -> 107.1,
    // (1, 5376, 2048) 11.1 -> 10.8; five: 57.1 us at the prefill shape.
    size_t lds_bytes = (size_t)(kBlock / kWave) * (a.rows_per_run + W - 1) * kWave * sizeof(uint32_t);
    if (lds_bytes < kLdsFloorBytes) lds_bytes = kLdsFloorBytes;
    auto launch = [&](auto act, auto ts) {
        CC1D_LAUNCH((fwd_channellast_kernel<DT, W, HAS_SEQ, decltype(act)::value, WM, decltype(ts)::value>),
                    dim3(blocks), dim3(kBlock), lds_bytes, stream, a, q);
    };
    using Fixed = std::integral_constant<int, kDefaultRows>;
    using Any = std::integral_constant<int, 0>;
    if (a.rows_per_run == kDefaultRows) {
        if (silu) launch(std::true_type{}, Fixed{}); else launch(std::false_type{}, Fixed{});
    } else {
        if (silu) launch(std::true_type{}, Any{}); else launch(std::false_type{}, Any{});
    }
    return launch_status();
}

template <int DT, int WM>
int launch_width(const FwdClArgs &a, const FwdClRare &q, int width, bool silu, hipStream_t stream) {
    const bool seq = a.seq_idx != nullptr;
    switch (width) {
        case 2: return seq ? launch_instance<DT, 2, true, WM>(a, q, silu, stream) : launch_instance<DT, 2, false, WM>(a, q, silu, stream);
        case 3: return seq ? launch_instance<DT, 3, true, WM>(a, q, silu, stream) : launch_instance<DT, 3, false, WM>(a, q, silu, stream);
        default: return seq ? launch_instance<DT, 4, true, WM>(a, q, silu, stream) : launch_instance<DT, 4, false, WM>(a, q, silu, stream);
    }
}

// Taps through PackedTaps when they are packed (mode 1 or 2), else through the general loader.
template <int DT>
int launch_taps(const FwdClArgs &a, const FwdClRare &q, int width, bool silu, int mode, hipStream_t stream) {
    if (mode == 1) return launch_width<DT, 1>(a, q, width, silu, stream);
    if constexpr (DT != CC1D_F32) {
        if (mode == 2) return launch_width<DT, 2>(a, q, width, silu, stream);
    }
    return launch_width<DT, 0>(a, q, width, silu, stream);
}

}  // namespace

// Rows per run.  Longer runs amortise the per-run start-up (taps, halo rows); shorter runs keep
// the chip's accesses closer together in memory, which is what counts on buffers no cache
// holds, and hold less LDS, so more of them are in flight.  Measured at the prefill shape
// (8, 5376, 2048) bf16, the same buffers every launch / six rotating sets: 8 rows 64.7 / 62.7 us,
// 16 rows 56.1 / 55.9, 24 rows 57.8 / 57.5, 32 rows 58.5 / 58.3.
// Launches of at most 1536 wavefronts (a fifth of what the chip holds: a prompt of a few dozen
// tokens, a short chunk of a prefill) are bound by one wavefront's chain of fetch, walk and store
// and take runs of 8 rows: (1, 5376, 64) bf16 4.65 -> 4.05 us, (4, 5376, 128) 5.19 -> 4.70,
// (1, 5376, 512) 5.16 -> 4.65; at 2048 wavefronts and more 16 rows are as fast or faster.
static int choose_rows_per_run(int seqlen, int64_t row_bytes, int width, int64_t waves_at_default) {
    int T = tunables().fwd_cl_rows;
    if (T <= 0) T = waves_at_default <= 1536 ? kGroup : kDefaultRows;
    const int cap = (seqlen + kGroup - 1) / kGroup * kGroup;      // never longer than the sequence
    if (T > cap) T = cap;
    T = (T + kGroup - 1) / kGroup * kGroup;
    if (T > kMaxRows) T = kMaxRows;
    // Row offsets inside a run (halo included) are 31-bit scalars in the kernel.
    while (T > kGroup && (int64_t)(T + width - 1) * row_bytes >= ((int64_t)1 << 31)) T -= kGroup;
    return (int64_t)(T + width - 1) * row_bytes >= ((int64_t)1 << 31) ? 0 : T;
}

// gather: a varlen final-state gather to run in the same launch (NULL: none).  It must be one
// the vector gather takes (varlen_vec_ok) on elements as wide as x's.
int launch_fwd_channellast(const cc1d_fwd_params &p, const cc1d_varlen_params *gather, hipStream_t stream) {
    // fwd_cl_half_vec = -1 forces the general tap loader.
    int mode = weights_mode(p.weight, p.bias, p.w_dtype, p.x_dtype, p.w_stride_c, p.w_stride_w, p.width);
    if (tunables().fwd_cl_half_vec < 0) mode = 0;
    const int eb = elem_bytes(p.x_dtype);
    const int ch = 4 / eb;                            // a lane's column is 4 bytes wide
    FwdClArgs a = {};
    a.n_cols = p.dim / ch;
    const int64_t row_stride = p.x_stride_l > p.out_stride_l ? p.x_stride_l : p.out_stride_l;
    a.waves_per_row = (uint32_t)((a.n_cols + kWave - 1) / kWave);
    a.rows_per_run = choose_rows_per_run(p.seqlen, row_stride * eb, p.width,
                                         (int64_t)p.batch * ((p.seqlen + kDefaultRows - 1) / kDefaultRows) * a.waves_per_row);
    if (a.rows_per_run == 0) return CC1D_ERR_TOO_LARGE;
    a.n_runs = (p.seqlen + a.rows_per_run - 1) / a.rows_per_run;
    const int64_t total = (int64_t)p.batch * a.n_runs * a.waves_per_row;
    if (total * kWave >= thread_limit() - kXcds * kBlock) return CC1D_ERR_TOO_LARGE;
    a.total = (uint32_t)total;
    const uint32_t blocks = (uint32_t)((total + kBlock / kWave - 1) / (kBlock / kWave));
    // Workgroup order: an XCD takes chunks of `chunk_runs` consecutive runs (all their column
    // blocks), the 8 XCDs take 8 neighbouring chunks at a time.  Inside a chunk a run finds the halo
    // rows it shares with the run above in its own XCD's L2; across XCDs the chip walks through
    // memory as one front instead of eight far-apart streams, which is what counts on buffers that
    // are not already in the caches and translation caches (every layer of a model).  At the
    // prefill shape, the same buffers every launch / six rotating sets, in us: single workgroups in
    // hardware order 58.6 / 58.3, chunks of 2 runs 56.6 / 56.0, 4 runs 56.5 / 55.9, 8 runs 56.8 / 56.2,
    // 16 runs 57.4 / 57.1, one contiguous slice per XCD 58.8 / 58.7.  Launches of fewer than eight
    // chunks per XCD take smaller chunks, or else contiguous slices.
    int chunk_runs = tunables().fwd_cl_chunk_runs;
    if (chunk_runs == 0) {
        const int64_t wpr = a.waves_per_row;
        auto chunks_per_xcd = [&](int runs) { return (int64_t)blocks * 4 / ((int64_t)kXcds * runs * wpr); };
        chunk_runs = 4;
        if (chunks_per_xcd(4) < 8) chunk_runs = chunks_per_xcd(2) >= 8 ? 2 : -1;
    }
    // chunk_runs > 0: chunks of that many runs (a run is waves_per_row wavefronts, a workgroup four of
    // them); < -1: chunks of -chunk_runs - 1 workgroups (-2: one workgroup, which is the hardware's own
    // round-robin order); -1: one contiguous slice per XCD.
    a.blocks_per_chunk = chunk_runs > 0 ? (uint32_t)(((int64_t)chunk_runs * a.waves_per_row + 3) / 4)
                         : chunk_runs < -1 ? (uint32_t)(-chunk_runs - 1) : 0u;
    a.blocks_per_xcd = (blocks + kXcds - 1) / kXcds;
    if (a.blocks_per_chunk != 0)
        a.blocks_per_xcd = (a.blocks_per_xcd + a.blocks_per_chunk - 1) / a.blocks_per_chunk * a.blocks_per_chunk;
    if ((int64_t)a.blocks_per_xcd * kXcds * kBlock >= thread_limit()) return CC1D_ERR_TOO_LARGE;
    a.first_tail_block = a.blocks_per_xcd * kXcds;
    a.seqlen = p.seqlen;
    a.x_row_bytes = (uint32_t)(p.x_stride_l * eb);
    a.out_row_bytes = (uint32_t)(p.out_stride_l * eb);
    a.states = (p.initial_states != nullptr ? 1 : 0) | (p.final_states != nullptr ? 2 : 0);
    a.x = p.x; a.out = p.out; a.weight = p.weight; a.bias = p.bias; a.seq_idx = p.seq_idx;
    a.x_stride_b = p.x_stride_b; a.out_stride_b = p.out_stride_b;
    FwdClRare q = {};
    q.initial_states = p.initial_states; q.final_states = p.final_states;
    q.init_stride_b = p.init_stride_b; q.init_stride_c = p.init_stride_c; q.init_stride_l = p.init_stride_l;
    q.final_stride_b = p.final_stride_b; q.final_stride_c = p.final_stride_c; q.final_stride_l = p.final_stride_l;
    q.w_stride_c = p.w_stride_c; q.w_stride_w = p.w_stride_w; q.w_dtype = p.w_dtype;
    if (gather != nullptr) {
        q.tail = *gather;
        q.tail_n_colgroups = (uint32_t)(gather->dim / vec_elems(gather->x_dtype));
        const int64_t threads = (int64_t)gather->batch * gather->state_len * q.tail_n_colgroups;
        if (threads + (int64_t)a.first_tail_block * kBlock >= thread_limit()) return CC1D_ERR_TOO_LARGE;
        q.tail_total = (uint32_t)threads;
    }
    const bool silu = p.silu != 0;
    switch (p.x_dtype) {
        case CC1D_F32: return launch_taps<CC1D_F32>(a, q, p.width, silu, mode, stream);
        case CC1D_F16: return launch_taps<CC1D_F16>(a, q, p.width, silu, mode, stream);
        default: return launch_taps<CC1D_BF16>(a, q, p.width, silu, mode, stream);
    }
}

}  // namespace cc1d
