// Channel-last backward: launch geometry, the fp32 instantiations and the second stage that adds
// the partial sums of dweight / dbias.  The kernel itself is in cc1d_bwd_channellast_kernel.hpp.
#include "cc1d_bwd_channellast_kernel.hpp"

namespace cc1d {


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
    CC1D_LAUNCH(bwd_finalize_kernel, dim3(planes * cblocks), dim3(kFinSlices * kFinChannels), 0, stream,
                       ws, n_parts, p.dim, p.width, p.dweight, p.dw_stride_c, p.dw_stride_w, p.dbias,
                       p.overwrite_dweight);
    return launch_status();
}

namespace {

// Channels per lane: 2 (4 bytes of 16-bit data, 8 bytes of fp32).  16-bit data whose dx rows do not
// all start on 64-byte boundaries (a column slice of a wider tensor: mamba_ssm hands over dx as a
// view of its d_in_proj-wide gradient buffer, rows of 21152 bytes at 2.7B) takes 4: a wavefront's
// store of a row then covers 512 bytes instead of 256, and the 64-byte blocks it shares with the
// neighbouring wavefronts, written in two parts, are half as many per byte.  (8, 5376, 2048) bf16
// with row strides of 10752 / 10768 / 10784 / 10816 bytes for dx: 93 / 128 / 118 / 96 us with 4-byte
// lanes (loads are not sensitive: x as such a view costs 1-4 %); 8-byte lanes: 100 us on aligned
// rows, 109-111 us at 21152 bytes (119 us with 4-byte lanes), (16, 1792, 2048) at 6704 bytes 76
// against 88 us.  Launches that do not fill the chip keep 4-byte lanes.
int channels_per_lane(const cc1d_bwd_params &p) {
    if (p.x_dtype == CC1D_F32) return 2;
    const int32_t forced = tunables().bwd_cl_lane_bytes;
    if (forced == 4 || forced == 8) return forced / 2;
    const int64_t eb = 2;
    const bool rows_on_64 = reinterpret_cast<uintptr_t>(p.dx) % 64 == 0 &&
                            (p.seqlen <= 1 || (p.dx_stride_l * eb) % 64 == 0) &&
                            (p.batch <= 1 || (p.dx_stride_b * eb) % 64 == 0);
    if (rows_on_64) return CC1D_BWD_CL_CH16;
    const int64_t waves32 = (int64_t)p.batch * ((p.seqlen + 31) / 32) * ((p.dim / CC1D_BWD_CL_CH16 + kWave - 1) / kWave);
    return waves32 >= 2 * 4096 ? 4 : CC1D_BWD_CL_CH16;
}

// Returns false when a run cannot be addressed with 32-bit byte offsets.
bool make_geom(const cc1d_bwd_params &p, BwdClGeom &g) {
    constexpr int U2 = 2 * CC1D_BWD_CL_UNROLL;        // the walk is unrolled over two groups
    g.channels_per_lane = channels_per_lane(p);
    g.n_colgroups = p.dim / g.channels_per_lane;
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
        const int64_t slots = (int64_t)256 * 4 * (g.channels_per_lane * elem_bytes(p.x_dtype) == 4 ? CC1D_BWD_CL_OCC : CC1D_BWD_CL_OCC8);
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
        default:
            st = g.channels_per_lane == 4 ? launch_bwd_channellast_16bit_lanes8(p, g, ws, stream)
                                          : launch_bwd_channellast_16bit_lanes4(p, g, ws, stream);
            break;
    }
    if (st != CC1D_OK) return st;
    return launch_bwd_finalize(ws, p.batch * g.n_quads, p, stream);
}

}  // namespace cc1d