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
// Design.  Same geometry as the channel-last forward: a lane owns one 16-byte vector of
// channels and walks a run of rows in ascending order, holding (W-1)-row sliding windows
// of x and g in registers.  dx[p] is emitted W-1 steps late, when g[p+W-1] has arrived,
// so one ascending pass yields dx, and the lane's dweight/dbias partial sums stay in
// registers for the whole run (no cross-lane reduction, no atomics).  Each run then
// stores its partials to a workspace plane and a second kernel adds them up in a fixed
// order: results are bit-reproducible.  Halo cost per run: W-1 rows of x in front,
// W-1 rows of x and dout behind.
#include "cc1d_device.hpp"
#include "cc1d_internal.hpp"

#ifndef CC1D_BWD_CL_UNROLL
#define CC1D_BWD_CL_UNROLL 2
#endif

namespace cc1d {
namespace {

struct BwdClGeom {
    int32_t rows_per_run;
    int32_t n_runs;
    int32_t n_colgroups;
    uint32_t total;
    int32_t w_fast;
    int32_t init_vec;
    int32_t dinit_vec;
};

template <int DT>
struct alignas(16) RawVecB {
    typename Elem<DT>::type v[Elem<DT>::kVec];
};

template <int DT, int W, bool HAS_SEQ, bool SILU, int U>
__global__ void __launch_bounds__(kBlock)
bwd_channellast_kernel(const cc1d_bwd_params p, const BwdClGeom g, float *__restrict__ ws) {
    using E = Elem<DT>;
    constexpr int VEC = E::kVec;
    constexpr bool PRECISE = E::kPreciseAct;

    const uint32_t gid = blockIdx.x * (uint32_t)kBlock + threadIdx.x;
    if (gid >= g.total) return;
    const uint32_t col = gid % (uint32_t)g.n_colgroups;
    const uint32_t rb = gid / (uint32_t)g.n_colgroups;
    const int run = (int)(rb % (uint32_t)g.n_runs);
    const int b = (int)(rb / (uint32_t)g.n_runs);
    const int c0 = (int)col * VEC;
    const int L = p.seqlen;
    const int T = g.rows_per_run;
    const int t0 = run * T;
    const int t1 = t0 + T < L ? t0 + T : L;           // rows [t0, t1) are this lane's own
    const int t_last = t1 + (W - 1);                  // exclusive end of the walk

    float wv[VEC][W], bv[VEC];
    load_weights<W, VEC>(p.weight, p.bias, p.w_dtype, p.w_stride_c, p.w_stride_w,
                         g.w_fast != 0, c0, wv, bv);

    const int64_t xoff = (int64_t)b * p.x_stride_b + c0;
    const int64_t doff = (int64_t)b * p.dout_stride_b + c0;
    const int64_t dxoff = (int64_t)b * p.dx_stride_b + c0;
    const int32_t *seq = HAS_SEQ ? p.seq_idx + (int64_t)b * L : nullptr;

    // Windows: xw[k] = x[t-(W-1)+k], gw[k] = g[t-(W-1)+k], sqw[k] likewise, at step t.
    float xw[W - 1][VEC], gw[W - 1][VEC];
    int sqw[W - 1];
#pragma unroll
    for (int k = 0; k < W - 1; ++k) {
        const int t = t0 - (W - 1) + k;
        u32x4 r = {0u, 0u, 0u, 0u};
        if (t >= 0) {
            r = ld_vec<DT>(p.x, xoff + (int64_t)t * p.x_stride_l);
        } else if (p.initial_states != nullptr) {
            if (g.init_vec) {
                r = ld_vec<DT>(p.initial_states, (int64_t)b * p.init_stride_b +
                                                     (int64_t)(t + W - 1) * p.init_stride_l + c0);
            } else {
                RawVecB<DT> rv;
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    rv.v[j] = ld_raw<DT>(p.initial_states, (int64_t)b * p.init_stride_b +
                                                               (int64_t)(c0 + j) * p.init_stride_c +
                                                               (int64_t)(t + W - 1) * p.init_stride_l);
                r = bitcast<u32x4>(rv);
            }
        }
        E::unpack(r, xw[k]);
#pragma unroll
        for (int j = 0; j < VEC; ++j) gw[k][j] = 0.f;
        sqw[k] = (HAS_SEQ && t >= 0) ? seq[t] : -1;
    }

    float dW[VEC][W], dB[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        dB[j] = 0.f;
#pragma unroll
        for (int w = 0; w < W; ++w) dW[j][w] = 0.f;
    }

    u32x4 nx[U], nd[U];
    int nseq[U];
    auto load_group = [&](int t) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int tt = t + u;
            u32x4 rx = {0u, 0u, 0u, 0u}, rd = {0u, 0u, 0u, 0u};
            int s = -1;
            if (tt < L && tt < t_last) {
                rx = ld_vec_nt<DT>(p.x, xoff + (int64_t)tt * p.x_stride_l);
                rd = ld_vec_nt<DT>(p.dout, doff + (int64_t)tt * p.dout_stride_l);
                if (HAS_SEQ) s = seq[tt];
            }
            nx[u] = rx; nd[u] = rd; nseq[u] = s;
        }
    };
    load_group(t0);

    const int n_steps = T + (W - 1);                  // uniform trip count; extra steps are inert
    for (int i = 0; i < n_steps; i += U) {
        u32x4 rx[U], rd[U];
        int sq[U];
#pragma unroll
        for (int u = 0; u < U; ++u) { rx[u] = nx[u]; rd[u] = nd[u]; sq[u] = nseq[u]; }
        if (i + U < n_steps) load_group(t0 + i + U);

#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int t = t0 + i + u;
            const int cur = sq[u];
            float xv[VEC], gv[VEC];
            E::unpack(rx[u], xv);
            E::unpack(rd[u], gv);                     // dout[t]; zero for t >= L

            bool tapm[W - 1];                         // tap k (row t-(W-1)+k) feeds row t
#pragma unroll
            for (int k = 0; k < W - 1; ++k) tapm[k] = !HAS_SEQ || sqw[k] == cur;

            if (SILU) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    float z = bv[j];
#pragma unroll
                    for (int k = 0; k < W - 1; ++k) z = fmaf(tapm[k] ? wv[j][k] : 0.f, xw[k][j], z);
                    z = fmaf(wv[j][W - 1], xv[j], z);
                    gv[j] *= silu_grad<PRECISE>(z);
                }
            }
            if (HAS_SEQ) {
                if (cur < 0) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) gv[j] = 0.f;
                }
            }

            if (t < t1) {                             // own row: dweight / dbias partials
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    dB[j] += gv[j];
#pragma unroll
                    for (int k = 0; k < W - 1; ++k)
                        dW[j][k] = fmaf(gv[j], tapm[k] ? xw[k][j] : 0.f, dW[j][k]);
                    dW[j][W - 1] = fmaf(gv[j], xv[j], dW[j][W - 1]);
                }
            }

            // Emit position pp = t-(W-1): g[pp .. pp+W-2] = gw[0..W-2], g[pp+W-1] = gv.
            const int pp = t - (W - 1);
            const bool emit_dx = pp >= t0 && pp < t1;
            const bool emit_dinit = pp < 0 && t0 == 0 && p.dinitial_states != nullptr && t < W - 1;
            if (emit_dx || emit_dinit) {
                const int sp = sqw[0];
                float dxv[VEC];
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    float a = wv[j][W - 1] * gw[0][j];
#pragma unroll
                    for (int k = 1; k < W - 1; ++k)
                        a = fmaf((!HAS_SEQ || sqw[k] == sp) ? wv[j][W - 1 - k] : 0.f, gw[k][j], a);
                    a = fmaf((!HAS_SEQ || cur == sp) ? wv[j][0] : 0.f, gv[j], a);
                    dxv[j] = a;
                }
                if (p.dfinal_states != nullptr && pp >= L - (W - 1)) {
                    const int fl = pp - (L - (W - 1));
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        dxv[j] += ld_elem<DT>(p.dfinal_states, (int64_t)b * p.dfinal_stride_b +
                                                                   (int64_t)(c0 + j) * p.dfinal_stride_c +
                                                                   (int64_t)fl * p.dfinal_stride_l);
                }
                if (emit_dx) {
                    st_vec_nt<DT>(p.dx, dxoff + (int64_t)pp * p.dx_stride_l, E::pack(dxv));
                } else {
                    const int il = pp + (W - 1);
                    if (g.dinit_vec) {
                        st_vec<DT>(p.dinitial_states, (int64_t)b * p.dinit_stride_b +
                                                          (int64_t)il * p.dinit_stride_l + c0, E::pack(dxv));
                    } else {
#pragma unroll
                        for (int j = 0; j < VEC; ++j)
                            st_elem<DT>(p.dinitial_states, (int64_t)b * p.dinit_stride_b +
                                                               (int64_t)(c0 + j) * p.dinit_stride_c +
                                                               (int64_t)il * p.dinit_stride_l, dxv[j]);
                    }
                }
            }

#pragma unroll
            for (int k = 0; k < W - 2; ++k) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) { xw[k][j] = xw[k + 1][j]; gw[k][j] = gw[k + 1][j]; }
                sqw[k] = sqw[k + 1];
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) { xw[W - 2][j] = xv[j]; gw[W - 2][j] = gv[j]; }
            sqw[W - 2] = cur;
        }
    }

    // Partials of this run: plane w of part (b, run), channels c0 .. c0+VEC.
    const int64_t part = (int64_t)b * g.n_runs + run;
    float *dst = ws + part * (int64_t)(W + 1) * p.dim + c0;
#pragma unroll
    for (int w = 0; w <= W; ++w) {
#pragma unroll
        for (int q = 0; q < VEC / 4; ++q) {
            u32x4 o;
            if (w < W) {
                o.x = bitcast<uint32_t>(dW[4 * q][w]); o.y = bitcast<uint32_t>(dW[4 * q + 1][w]);
                o.z = bitcast<uint32_t>(dW[4 * q + 2][w]); o.w = bitcast<uint32_t>(dW[4 * q + 3][w]);
            } else {
                o.x = bitcast<uint32_t>(dB[4 * q]); o.y = bitcast<uint32_t>(dB[4 * q + 1]);
                o.z = bitcast<uint32_t>(dB[4 * q + 2]); o.w = bitcast<uint32_t>(dB[4 * q + 3]);
            }
            *reinterpret_cast<u32x4 *>(dst + (int64_t)w * p.dim + 4 * q) = o;
        }
    }
}

}  // namespace

// Second stage shared by both backward layouts: dweight[c, w] += sum over parts, in
// ascending part order, of ws[part][w][c]; plane W holds dbias.  One lane per (w, c).
__global__ void __launch_bounds__(kBlock)
bwd_finalize_kernel(const float *__restrict__ ws, int n_parts, int dim, int width,
                    float *__restrict__ dweight, int64_t dw_stride_c, int64_t dw_stride_w,
                    float *__restrict__ dbias) {
    const uint32_t gid = blockIdx.x * (uint32_t)kBlock + threadIdx.x;
    const uint32_t planes = (uint32_t)width + (dbias != nullptr ? 1u : 0u);
    if (gid >= planes * (uint32_t)dim) return;
    const int c = (int)(gid % (uint32_t)dim);
    const int w = (int)(gid / (uint32_t)dim);
    const int64_t part_stride = (int64_t)(width + 1) * dim;
    const float *src = ws + (int64_t)w * dim + c;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;    // four interleaved chains, fixed order
    int q = 0;
    for (; q + 4 <= n_parts; q += 4) {
        s0 += src[(int64_t)q * part_stride];
        s1 += src[(int64_t)(q + 1) * part_stride];
        s2 += src[(int64_t)(q + 2) * part_stride];
        s3 += src[(int64_t)(q + 3) * part_stride];
    }
    for (; q < n_parts; ++q) s0 += src[(int64_t)q * part_stride];
    const float total = (s0 + s1) + (s2 + s3);
    if (w < width) dweight[(int64_t)c * dw_stride_c + (int64_t)w * dw_stride_w] += total;
    else dbias[c] += total;
}

int launch_bwd_finalize(const float *ws, int n_parts, const cc1d_bwd_params &p, hipStream_t stream) {
    const uint32_t planes = (uint32_t)p.width + (p.dbias != nullptr ? 1u : 0u);
    const uint32_t total = planes * (uint32_t)p.dim;
    hipLaunchKernelGGL(bwd_finalize_kernel, dim3((total + kBlock - 1) / kBlock), dim3(kBlock), 0, stream,
                       ws, n_parts, p.dim, p.width, p.dweight, p.dw_stride_c, p.dw_stride_w, p.dbias);
    return launch_status();
}

namespace {

BwdClGeom make_geom(const cc1d_bwd_params &p) {
    constexpr int U = CC1D_BWD_CL_UNROLL;
    const int vec = vec_elems(p.x_dtype);
    BwdClGeom g;
    g.n_colgroups = p.dim / vec;
    int T = tunables().bwd_cl_rows;
    if (T <= 0) {
        // Runs of 128 rows keep the partial-sum planes at about 2.6% of the tensor traffic;
        // go shorter only when that is needed to put about 8 waves on each of 256 CUs.
        const int64_t target_lanes = (int64_t)256 * 8 * kWave;
        T = 128;
        while (T > 32 && (int64_t)p.batch * g.n_colgroups * ((p.seqlen + T - 1) / T) < target_lanes) T >>= 1;
    }
    const int cap = (p.seqlen + U - 1) / U * U;
    if (T > cap) T = cap;
    T = (T + U - 1) / U * U;
    if (T < U) T = U;
    g.rows_per_run = T;
    g.n_runs = (p.seqlen + T - 1) / T;
    g.total = 0;
    g.w_fast = weights_contiguous_f32(p.weight, p.w_dtype, p.w_stride_c, p.w_stride_w, p.width);
    g.init_vec = states_vec_ok(p.initial_states, p.x_dtype, p.init_stride_b, p.init_stride_c, p.init_stride_l);
    g.dinit_vec = states_vec_ok(p.dinitial_states, p.x_dtype, p.dinit_stride_b, p.dinit_stride_c, p.dinit_stride_l);
    return g;
}

template <int DT, int W, bool HAS_SEQ>
int launch_instance(const cc1d_bwd_params &p, const BwdClGeom &g, float *ws, hipStream_t stream) {
    const uint32_t blocks = (g.total + kBlock - 1) / kBlock;
    if (p.silu)
        hipLaunchKernelGGL((bwd_channellast_kernel<DT, W, HAS_SEQ, true, CC1D_BWD_CL_UNROLL>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws);
    else
        hipLaunchKernelGGL((bwd_channellast_kernel<DT, W, HAS_SEQ, false, CC1D_BWD_CL_UNROLL>), dim3(blocks), dim3(kBlock), 0, stream, p, g, ws);
    return launch_status();
}

template <int DT>
int launch_dtype(const cc1d_bwd_params &p, const BwdClGeom &g, float *ws, hipStream_t stream) {
    const bool seq = p.seq_idx != nullptr;
    switch (p.width) {
        case 2: return seq ? launch_instance<DT, 2, true>(p, g, ws, stream) : launch_instance<DT, 2, false>(p, g, ws, stream);
        case 3: return seq ? launch_instance<DT, 3, true>(p, g, ws, stream) : launch_instance<DT, 3, false>(p, g, ws, stream);
        default: return seq ? launch_instance<DT, 4, true>(p, g, ws, stream) : launch_instance<DT, 4, false>(p, g, ws, stream);
    }
}

}  // namespace

size_t bwd_channellast_workspace_bytes(const cc1d_bwd_params &p) {
    const BwdClGeom g = make_geom(p);
    return (size_t)p.batch * g.n_runs * (p.width + 1) * (size_t)p.dim * sizeof(float);
}

int launch_bwd_channellast(const cc1d_bwd_params &p, void *workspace, hipStream_t stream) {
    BwdClGeom g = make_geom(p);
    const int64_t total = (int64_t)p.batch * g.n_runs * g.n_colgroups;
    if (total >= ((int64_t)1 << 31)) return CC1D_ERR_TOO_LARGE;
    g.total = (uint32_t)total;
    float *ws = static_cast<float *>(workspace);
    int st;
    switch (p.x_dtype) {
        case CC1D_F32: st = launch_dtype<CC1D_F32>(p, g, ws, stream); break;
        case CC1D_F16: st = launch_dtype<CC1D_F16>(p, g, ws, stream); break;
        default: st = launch_dtype<CC1D_BF16>(p, g, ws, stream); break;
    }
    if (st != CC1D_OK) return st;
    return launch_bwd_finalize(ws, p.batch * g.n_runs, p, stream);
}

}  // namespace cc1d
