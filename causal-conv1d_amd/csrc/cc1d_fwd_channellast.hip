// Channel-last forward for gfx950: x is (batch, seqlen, dim) in memory (unit stride
// along dim).  Takes over causal_conv1d_channellast_fwd_kernel and its launcher
// (csrc/causal_conv1d_fwd.cu:205-381 of the reference).
//
// Design.  The stencil runs along seqlen, which is the strided axis, so nothing has to
// be transposed: a lane owns one 16-byte vector of channels (8 x 16-bit or 4 x fp32),
// keeps that vector's W taps and bias in registers and walks down a run of consecutive
// rows with a (W-1)-row sliding window held in registers as fp32.  Per row that is one
// 16-byte load and one 16-byte store per lane, both fully coalesced along dim, no LDS
// and no barrier.  The only re-read is the (W-1)-row halo in front of each run.
//
// Work items (batch, run, vector-column) are laid out flat over the grid, so every lane
// is busy for any dim that is a multiple of the vector width; lanes of one wave may sit
// in different runs, which is why seq_idx is tracked per lane.
#include "cc1d_device.hpp"
#include "cc1d_internal.hpp"

#ifndef CC1D_FWD_CL_UNROLL
#define CC1D_FWD_CL_UNROLL 4      // rows in flight per lane (and prefetched one group ahead)
#endif
#ifndef CC1D_FWD_CL_NT
#define CC1D_FWD_CL_NT 1          // streaming (non-temporal) row loads and stores
#endif

namespace cc1d {
namespace {

struct FwdClGeom {
    int32_t rows_per_run;     // T, a multiple of the unroll factor
    int32_t n_runs;           // ceil(seqlen / T)
    int32_t n_colgroups;      // dim / kVec
    uint32_t total;           // batch * n_runs * n_colgroups work items
    int32_t w_fast;           // weights_contiguous_f32
    int32_t init_vec;         // states_vec_ok(initial_states)
    int32_t final_vec;        // states_vec_ok(final_states)
};

template <int DT>
struct alignas(16) RawVec {
    typename Elem<DT>::type v[Elem<DT>::kVec];
};

// One (batch, l) row of a (batch, dim, k) states tensor, channels c0 .. c0+kVec.
template <int DT>
__device__ __forceinline__ u32x4 load_state_row(const void *base, int64_t sb, int64_t sc,
                                                int64_t sl, int b, int c0, int l, bool vec) {
    if (vec) return ld_vec<DT>(base, (int64_t)b * sb + (int64_t)l * sl + c0);
    RawVec<DT> r;
#pragma unroll
    for (int j = 0; j < Elem<DT>::kVec; ++j)
        r.v[j] = ld_raw<DT>(base, (int64_t)b * sb + (int64_t)(c0 + j) * sc + (int64_t)l * sl);
    return bitcast<u32x4>(r);
}
template <int DT>
__device__ __forceinline__ void store_state_row(void *base, int64_t sb, int64_t sc, int64_t sl,
                                                int b, int c0, int l, bool vec, const u32x4 &v) {
    if (vec) {
        st_vec<DT>(base, (int64_t)b * sb + (int64_t)l * sl + c0, v);
        return;
    }
    RawVec<DT> r = bitcast<RawVec<DT>>(v);
#pragma unroll
    for (int j = 0; j < Elem<DT>::kVec; ++j)
        st_raw<DT>(base, (int64_t)b * sb + (int64_t)(c0 + j) * sc + (int64_t)l * sl, r.v[j]);
}

template <int DT, int W, bool HAS_SEQ, int U, bool NT>
__global__ void __launch_bounds__(kBlock)
fwd_channellast_kernel(const cc1d_fwd_params p, const FwdClGeom g) {
    using E = Elem<DT>;
    constexpr int VEC = E::kVec;
    constexpr bool PRECISE = E::kPreciseAct;

    const uint32_t gid = blockIdx.x * (uint32_t)kBlock + threadIdx.x;
    if (gid >= g.total) return;                       // no cross-lane traffic below
    const uint32_t col = gid % (uint32_t)g.n_colgroups;
    const uint32_t rb = gid / (uint32_t)g.n_colgroups;
    const int run = (int)(rb % (uint32_t)g.n_runs);
    const int b = (int)(rb / (uint32_t)g.n_runs);
    const int c0 = (int)col * VEC;
    const int L = p.seqlen;
    const int T = g.rows_per_run;
    const int t0 = run * T;                           // < L by construction of n_runs
    const bool silu_on = p.silu != 0;

    float wv[VEC][W], bv[VEC];
    load_weights<W, VEC>(p.weight, p.bias, p.w_dtype, p.w_stride_c, p.w_stride_w,
                         g.w_fast != 0, c0, wv, bv);

    const int64_t xoff = (int64_t)b * p.x_stride_b + c0;
    const int64_t ooff = (int64_t)b * p.out_stride_b + c0;
    const int32_t *seq = HAS_SEQ ? p.seq_idx + (int64_t)b * L : nullptr;

    // Sliding window: xw[i] holds row t-(W-1)+i while row t is being produced.
    float xw[W - 1][VEC];
    int sqw[W - 1];
#pragma unroll
    for (int i = 0; i < W - 1; ++i) {
        const int t = t0 - (W - 1) + i;
        u32x4 r = {0u, 0u, 0u, 0u};
        if (t >= 0) {
            r = ld_vec<DT>(p.x, xoff + (int64_t)t * p.x_stride_l);
        } else if (p.initial_states != nullptr) {
            r = load_state_row<DT>(p.initial_states, p.init_stride_b, p.init_stride_c,
                                   p.init_stride_l, b, c0, t + (W - 1), g.init_vec != 0);
        }
        E::unpack(r, xw[i]);
        sqw[i] = (HAS_SEQ && t >= 0) ? seq[t] : -1;
    }

    u32x4 nraw[U];
    int nseq[U];
    auto load_group = [&](int t) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int tt = t + u;
            u32x4 r = {0u, 0u, 0u, 0u};
            int s = -1;
            if (tt < L) {
                r = NT ? ld_vec_nt<DT>(p.x, xoff + (int64_t)tt * p.x_stride_l)
                       : ld_vec<DT>(p.x, xoff + (int64_t)tt * p.x_stride_l);
                if (HAS_SEQ) s = seq[tt];
            }
            nraw[u] = r;
            nseq[u] = s;
        }
    };
    load_group(t0);

    for (int i = 0; i < T; i += U) {
        u32x4 raw[U];
        int sq[U];
#pragma unroll
        for (int u = 0; u < U; ++u) { raw[u] = nraw[u]; sq[u] = nseq[u]; }
        if (i + U < T) load_group(t0 + i + U);        // prefetch the next group of rows

#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int t = t0 + i + u;
            float xv[VEC], acc[VEC];
            E::unpack(raw[u], xv);

            bool plain = true;
            if (HAS_SEQ) {
                const int cur = sq[u];
                plain = cur >= 0;
#pragma unroll
                for (int k = 0; k < W - 1; ++k) plain = plain && (sqw[k] == cur);
            }
            if (plain) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    float a = bv[j];
#pragma unroll
                    for (int k = 0; k < W - 1; ++k) a = fmaf(wv[j][k], xw[k][j], a);
                    acc[j] = fmaf(wv[j][W - 1], xv[j], a);
                }
            } else {
                // A sub-sequence boundary (or padding) inside the window: rare, so the
                // masked form lives on its own branch.
                const int cur = sq[u];
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    float a = bv[j];
#pragma unroll
                    for (int k = 0; k < W - 1; ++k)
                        a = fmaf(sqw[k] == cur ? wv[j][k] : 0.f, xw[k][j], a);
                    acc[j] = fmaf(wv[j][W - 1], xv[j], a);
                }
            }
            if (silu_on) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[j] = silu<PRECISE>(acc[j]);
            }
            if (HAS_SEQ) {
                if (sq[u] < 0) {                      // padding token: exact zero
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
                }
            }
            if (t < L) {
                const u32x4 o = E::pack(acc);
                if (NT) st_vec_nt<DT>(p.out, ooff + (int64_t)t * p.out_stride_l, o);
                else st_vec<DT>(p.out, ooff + (int64_t)t * p.out_stride_l, o);
            }
#pragma unroll
            for (int k = 0; k < W - 2; ++k) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) xw[k][j] = xw[k + 1][j];
                sqw[k] = sqw[k + 1];
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) xw[W - 2][j] = xv[j];
            sqw[W - 2] = sq[u];
        }
    }

    // final_states[b, c, i] = xpad[L-(W-1)+i]: the last run re-reads those few rows
    // (just streamed, still in cache) instead of tracking them through the loop.
    if (p.final_states != nullptr && run == g.n_runs - 1) {
#pragma unroll
        for (int i = 0; i < W - 1; ++i) {
            const int t = L - (W - 1) + i;
            u32x4 r = {0u, 0u, 0u, 0u};
            if (t >= 0) {
                r = ld_vec<DT>(p.x, xoff + (int64_t)t * p.x_stride_l);
            } else if (p.initial_states != nullptr) {
                r = load_state_row<DT>(p.initial_states, p.init_stride_b, p.init_stride_c,
                                       p.init_stride_l, b, c0, t + (W - 1), g.init_vec != 0);
            }
            store_state_row<DT>(p.final_states, p.final_stride_b, p.final_stride_c,
                                p.final_stride_l, b, c0, i, g.final_vec != 0, r);
        }
    }
}

template <int DT, int W, bool HAS_SEQ>
int launch_instance(const cc1d_fwd_params &p, const FwdClGeom &g, hipStream_t stream) {
    const uint32_t blocks = (g.total + kBlock - 1) / kBlock;
    hipLaunchKernelGGL((fwd_channellast_kernel<DT, W, HAS_SEQ, CC1D_FWD_CL_UNROLL, CC1D_FWD_CL_NT != 0>),
                       dim3(blocks), dim3(kBlock), 0, stream, p, g);
    return launch_status();
}

template <int DT>
int launch_dtype(const cc1d_fwd_params &p, const FwdClGeom &g, hipStream_t stream) {
    const bool seq = p.seq_idx != nullptr;
    switch (p.width) {
        case 2: return seq ? launch_instance<DT, 2, true>(p, g, stream) : launch_instance<DT, 2, false>(p, g, stream);
        case 3: return seq ? launch_instance<DT, 3, true>(p, g, stream) : launch_instance<DT, 3, false>(p, g, stream);
        default: return seq ? launch_instance<DT, 4, true>(p, g, stream) : launch_instance<DT, 4, false>(p, g, stream);
    }
}

}  // namespace

// Rows walked by one lane.  Longer runs amortise the (W-1)-row halo re-read; shorter
// runs put more wavefronts in flight.  The target is about 24 waves per CU on 256 CUs
// while keeping the halo overhead at or below (W-1)/32.
static int choose_rows_per_run(int64_t batch, int64_t n_colgroups, int seqlen) {
    constexpr int U = CC1D_FWD_CL_UNROLL;
    int forced = tunables().fwd_cl_rows;
    int T;
    if (forced > 0) {
        T = forced;
    } else {
        const int64_t target_lanes = (int64_t)256 * 24 * kWave;
        T = 128;
        while (T > 32 && batch * n_colgroups * ((seqlen + T - 1) / T) < target_lanes) T >>= 1;
    }
    const int cap = (seqlen + U - 1) / U * U;          // never longer than the sequence
    if (T > cap) T = cap;
    T = (T + U - 1) / U * U;
    return T < U ? U : T;
}

int launch_fwd_channellast(const cc1d_fwd_params &p, hipStream_t stream) {
    const int vec = vec_elems(p.x_dtype);
    FwdClGeom g;
    g.n_colgroups = p.dim / vec;
    g.rows_per_run = choose_rows_per_run(p.batch, g.n_colgroups, p.seqlen);
    g.n_runs = (p.seqlen + g.rows_per_run - 1) / g.rows_per_run;
    const int64_t total = (int64_t)p.batch * g.n_runs * g.n_colgroups;
    if (total >= ((int64_t)1 << 31)) return CC1D_ERR_TOO_LARGE;
    g.total = (uint32_t)total;
    g.w_fast = weights_contiguous_f32(p.weight, p.w_dtype, p.w_stride_c, p.w_stride_w, p.width);
    g.init_vec = states_vec_ok(p.initial_states, p.x_dtype, p.init_stride_b, p.init_stride_c, p.init_stride_l);
    g.final_vec = states_vec_ok(p.final_states, p.x_dtype, p.final_stride_b, p.final_stride_c, p.final_stride_l);
    switch (p.x_dtype) {
        case CC1D_F32: return launch_dtype<CC1D_F32>(p, g, stream);
        case CC1D_F16: return launch_dtype<CC1D_F16>(p, g, stream);
        default: return launch_dtype<CC1D_BF16>(p, g, stream);
    }
}

}  // namespace cc1d
