// Channel-first backward for gfx950, rows longer than 64 vectors: short-lived tile wavefronts.
// Takes over causal_conv1d_bwd_kernel (csrc/causal_conv1d_bwd.cu:53-259 of the reference) for
// these rows; formulas as in cc1d_bwd_channelfirst.hip, whose kernels keep the short rows.
//
//   z[t]  = bias + sum_w weight[w] * xpad[t-(W-1-w)]
//   g[t]  = dout[t] * act'(z[t])
//   dx[p] = sum_k weight[W-1-k] * g[p+k]   (+ dfinal_states[p-(L-(W-1))] for p >= L-(W-1))
//   dinitial_states[i] = the same expression at p = i-(W-1) < 0
//   dweight[w] += sum_{b,t} g[t] * xpad[t-(W-1-w)],   dbias += sum_{b,t} g[t]
//
// Design.  A wavefront takes a tile of up to four 64-vector steps of one (batch, channel) row
// and asks for all of its x and dout at once.  x goes from memory straight into LDS
// (buffer_load_dwordx4 ... lds), where a lane finds its neighbours' elements, together with the
// vector in front of the tile (the x halo) and the vectors behind it (the W-1 positions whose g
// the tile's last lane needs); dout, which only the lane that owns it reads, goes to registers
// (four per step: with LDS for one tensor instead of two, seven wavefronts share a SIMD instead
// of four: 1-3 % at most shapes, (2, 2048, 16384) bf16 71.1 -> 69.2 us).  The launch is thousands of wavefronts
// that live for one memory round trip and a few hundred instructions each and sweep through
// memory as one compact front in the order of the rows -- where one long-lived wavefront per
// channel walks 4096 far-apart streams at once, which is what bounds that design at the
// backward's benchmark shape (fp16 (4, 4096, 8192): 141 us for its memory pattern alone,
// 122 us for this one).  Each of the three tensors is a buffer resource per row, based at the
// row's first element wherever that lies (the vector accesses need no alignment, so rows of any
// length anywhere in memory take the same path: (16, 4096, 1001) bf16 costs 4 % more than 1000
// where the walking kernel took 2.2 times as long), and what lies outside a row needs no test:
// the vector in front of the first tile and everything behind the row's end is out of range,
// reads as zero and is not stored.  A 16-bit row of odd length ends in half a dword, which the
// range check would drop: that one element is fetched and stored on its own.  A row whose last
// 64-vector step would hold at most 64 positions ends in a tail instead: the row's last tile
// fetches those vectors as well and takes their positions one per lane, ahead of its steps
// ((16, 4096, 1025) bf16 103 -> 87 us, 2049: 194 -> 149 us; 1024 / 2048: 77 / 134 us).
// The steps of a tile are computed top down.  A lane's x halo is the upper half of the previous
// vector in LDS; the g values to the right of its vector come from the next lane (DPP shift),
// for the last lane from the step above (carried), for the top step from the vectors behind the
// tile.  The lane's dweight / dbias terms stay in registers across the tile, are reduced over
// the 64 lanes in a fixed order (DPP) and stored as one workspace plane per (batch entry, tile);
// the second-stage kernel shared with the other backward kernels adds the planes in a fixed
// order: no atomics, bit-reproducible.
#include <type_traits>

#include "cc1d_device.hpp"
#include "cc1d_internal.hpp"

namespace cc1d {
namespace {

// Most 64-vector steps a tile has (256 vectors, 4 KiB per tensor).  Fewer cost more wavefronts, each
// with its taps, its g values behind the tile and its reduction (fp16 (4, 4096, 8192): three steps
// 145 us, two 150 us against 140 us); six and eight measured no better than four.
constexpr int kTileSteps = 4;
constexpr int kTailVecs = kWave / 4;              // most vectors 64 positions can span (fp32)
constexpr int kRsrcRaw = 0x00020000;              // buffer resource word 3: raw buffer, 32-bit data format

typedef void __attribute__((address_space(3))) *lds_ptr_t;

struct BwdCfTileArgs {
    uint32_t total;               // rows * tiles_per_row wavefronts
    uint32_t tiles_per_row;
    int32_t steps_per_tile;       // 64-vector steps of every tile but a row's last, which may have fewer (1 .. 4)
    int32_t seqlen;
    int32_t body_vecs;            // vectors of a row that are walked as vectors (all of them, or a whole number of steps)
    int32_t tail_vecs;            // vectors behind them, done one position per lane (0: none)
    int32_t batch, dim;
    int32_t batch_inner;          // rows numbered with the batch entry fastest
    int32_t w_dtype;
    const void *x;
    const void *dout;
    void *dx;
    const void *weight;
    const void *bias;
    float *ws;                    // [batch * tiles_per_row][W + 1][dim]
    int64_t x_stride_b, x_stride_c, dout_stride_b, dout_stride_c, dx_stride_b, dx_stride_c;   // elements
    int64_t w_stride_c, w_stride_w;
    const void *initial_states;
    const void *dfinal_states;
    void *dinitial_states;
    int64_t init_stride_b, init_stride_c, init_stride_l;
    int64_t dfinal_stride_b, dfinal_stride_c, dfinal_stride_l;
    int64_t dinit_stride_b, dinit_stride_c, dinit_stride_l;
};

// Sum over the 64 lanes in a fixed order, result in lane 63: prefix sums inside each row of 16
// lanes (row_shr 1, 2, 4, 8), then the rows' totals across (row_bcast 15, 31).
__device__ __forceinline__ float wave_total_in_lane63(float v) {
    v += bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), 0x111, 0xf, 0xf, true));
    v += bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), 0x112, 0xf, 0xf, true));
    v += bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), 0x114, 0xf, 0xf, true));
    v += bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), 0x118, 0xf, 0xf, true));
    v += bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), 0x142, 0xa, 0xf, true));   // row_bcast:15 into rows 1, 3
    v += bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), 0x143, 0xc, 0xf, true));   // row_bcast:31 into rows 2, 3
    return v;
}

template <int DT, int W, bool SILU>
__global__ void __launch_bounds__(kBlock, 4)
bwd_channelfirst_tile_kernel(const BwdCfTileArgs a) {
    using E = Elem<DT>;
    using T = typename E::type;
    constexpr int VEC = E::kVec;
    constexpr int EB = E::kBytes;
    constexpr bool PRECISE = E::kPreciseAct;
    extern __shared__ u32x4 lds[];                    // [wavefront][x vectors]
    const int tile_vecs = a.steps_per_tile * kWave;
    const int XV = tile_vecs + 2 + kTailVecs;         // vectors of x a tile holds

    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const int lane = (int)(threadIdx.x & (kWave - 1));
    const uint32_t wid = blockIdx.x * (uint32_t)(kBlock / kWave) + (uint32_t)wv;
    if (wid >= a.total) return;
    const int tile = (int)(wid % a.tiles_per_row);
    const uint32_t row = wid / a.tiles_per_row;
    int b, c;
    if (a.batch_inner) { b = (int)(row % (uint32_t)a.batch); c = (int)(row / (uint32_t)a.batch); }
    else { c = (int)(row % (uint32_t)a.dim); b = (int)(row / (uint32_t)a.dim); }
    const int L = a.seqlen;

    const T *xrow = reinterpret_cast<const T *>(a.x) + (int64_t)b * a.x_stride_b + (int64_t)c * a.x_stride_c;
    const T *drow = reinterpret_cast<const T *>(a.dout) + (int64_t)b * a.dout_stride_b + (int64_t)c * a.dout_stride_c;
    T *dxrow = reinterpret_cast<T *>(a.dx) + (int64_t)b * a.dx_stride_b + (int64_t)c * a.dx_stride_c;
    // The range check works on whole dwords: a 16-bit row of odd length ends in half a dword,
    // which stays outside the resources; its element is moved separately below.
    const int row_bytes = (L * EB) & ~3;
    const bool odd_tail = ((L * EB) & 2) != 0;
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(xrow), 0, row_bytes, kRsrcRaw);
    const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(drow), 0, row_bytes, kRsrcRaw);
    const __amdgpu_buffer_rsrc_t rdx = __builtin_amdgcn_make_buffer_rsrc(dxrow, 0, row_bytes, kRsrcRaw);
    const int v0 = tile * tile_vecs;                  // the tile's first vector
    int steps = (a.body_vecs - v0 + kWave - 1) / kWave;   // steps of the tile that reach into the row
    steps = steps > a.steps_per_tile ? a.steps_per_tile : steps;
    // A row whose last step would hold at most 64 positions ends in a tail instead: its last tile
    // fetches those vectors too and takes their positions one per lane (an eighth of a step's
    // instructions instead of a whole step for a handful of lanes).
    const int tail_vecs = tile == (int)a.tiles_per_row - 1 ? a.tail_vecs : 0;
    // x goes to LDS, where a lane finds its neighbours' elements: vector i of the wavefront's LDS
    // holds row vector v0 - 1 + i (for the row's first tile the offset below wraps around: out of
    // range, zeros).  dout is needed by the lane that owns it only and goes to registers: LDS for
    // one tensor instead of two lets twice as many wavefronts share a CU.
    u32x4 *xl = lds + wv * XV;
    const int vx = (lane + v0 - 1) * 16, vd = (lane + v0) * 16;
    u32x4 dreg[kTileSteps];
#pragma unroll
    for (int s = 0; s < kTileSteps; ++s) dreg[s] = u32x4{0u, 0u, 0u, 0u};
    // Step s: the lane's offset in the vector register, s KiB as the instruction's immediate
    // offset, which the hardware adds to the LDS address as well, so the LDS pointer stays put.
    // (A scalar offset would do for the address but is left out of the range check, which the
    // row's ends rely on.)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)xl, 16, vx, 0, 0, 2);
    dreg[0] = __builtin_amdgcn_raw_buffer_load_b128(rd, vd, 0, 2);
    if (steps > 1) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)xl, 16, vx, 0, 1024, 2);
        dreg[1] = __builtin_amdgcn_raw_buffer_load_b128(rd, vd + 1024, 0, 2);
    }
    if (steps > 2) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)xl, 16, vx, 0, 2048, 2);
        dreg[2] = __builtin_amdgcn_raw_buffer_load_b128(rd, vd + 2048, 0, 2);
    }
    if (steps > 3) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)xl, 16, vx, 0, 3072, 2);
        dreg[3] = __builtin_amdgcn_raw_buffer_load_b128(rd, vd + 3072, 0, 2);
    }
    // behind the tile: two more vectors of x and the row's tail; the one vector of dout behind the
    // tile (what the top step's last lane needs) is the same for every lane
    if (lane < 2 + tail_vecs) __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)(xl + steps * kWave), 16, vx + steps * 1024, 0, 0, 0);
    const u32x4 dbehind = __builtin_amdgcn_raw_buffer_load_b128(rd, (v0 + steps * kWave) * 16, 0, 0);
    // the tail's dout, one position per lane
    const int p_tail = (v0 + steps * kWave) * VEC + lane;
    T tail_d = T(0.f);
    if (tail_vecs > 0 && p_tail < L) tail_d = ld_raw<DT>(drow, p_tail);

    // Taps and bias of the channel (wave-uniform); with the fast activation also times -log2(e),
    // so that the sum over the window is the exponent the derivative needs.
    float wv_[W], wvs[W], bias_v, bias_s;
#pragma unroll
    for (int w = 0; w < W; ++w)
        wv_[w] = ld_weight(a.weight, a.w_dtype, (int64_t)c * a.w_stride_c + w * a.w_stride_w);
    bias_v = a.bias == nullptr ? 0.f : ld_weight(a.bias, a.w_dtype, c);
#pragma unroll
    for (int w = 0; w < W; ++w) wvs[w] = wv_[w] * kSiluPrescale;
    bias_s = bias_v * kSiluPrescale;

    // What the resources leave out, fetched by single lanes: the odd last element of a 16-bit row
    // (by the tile that holds it) and initial_states in front of the row (by its first tile).
    const int tile_first = v0 * VEC, tile_end = (v0 + steps * kWave + tail_vecs) * VEC;   // positions [tile_first, tile_end)
    const bool holds_last = odd_tail && L - 1 >= tile_first - VEC && L - 1 < tile_end + VEC;
    T last_x = T(0.f), last_d = T(0.f);
    if (holds_last) {
        if (lane == 0) last_x = ld_raw<DT>(xrow, L - 1);
        last_d = ld_raw<DT>(drow, L - 1);             // every lane: the lane that owns the position patches its vector
    }
    T init_raw[W - 1];
    const bool has_init = a.initial_states != nullptr && tile == 0;
    if (has_init && lane == 0) {
#pragma unroll
        for (int i = 0; i < W - 1; ++i)
            init_raw[i] = ld_raw<DT>(a.initial_states, (int64_t)b * a.init_stride_b + (int64_t)c * a.init_stride_c +
                                                           (int64_t)i * a.init_stride_l);
    }
    // dfinal_states is added to the row's last W-1 positions: the tile that holds any of them
    // fetches the values (wave-uniform), and only the steps that hold them look.
    const bool has_dfinal = a.dfinal_states != nullptr && L - 1 >= tile_first && L - (W - 1) < tile_end;
    float dfin[W - 1];
#pragma unroll
    for (int i = 0; i < W - 1; ++i) dfin[i] = 0.f;
    if (has_dfinal) {
#pragma unroll
        for (int i = 0; i < W - 1; ++i)
            dfin[i] = ld_elem<DT>(a.dfinal_states, (int64_t)b * a.dfinal_stride_b + (int64_t)c * a.dfinal_stride_c +
                                                       (int64_t)i * a.dfinal_stride_l);
    }
    // Every vector of the tile is in LDS behind this wait (a vector fetched into LDS counts as a
    // load until it has been written there).
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (holds_last && lane == 0) {
        // LDS element index of row position p: p + VEC - tile_first
        const int ix = L - 1 + VEC - tile_first;
        if (ix >= 0 && ix < XV * VEC) reinterpret_cast<T *>(xl)[ix] = last_x;
    }
    if (has_init && lane == 0) {
#pragma unroll
        for (int i = 0; i < W - 1; ++i) reinterpret_cast<T *>(xl)[VEC - (W - 1) + i] = init_raw[i];
    }
    asm volatile("" ::: "memory");                    // the elements written above are read below as parts of vectors

    auto act_grad = [&](const float *xwin) { return silu_grad_of_window<W, PRECISE>(wv_, bias_v, wvs, bias_s, xwin); };
    float dW[W], dB = 0.f;
#pragma unroll
    for (int w = 0; w < W; ++w) dW[w] = 0.f;
    // g at the W-1 positions behind the tile's steps, in every lane (the values are wave-uniform)
    float carry[W - 1];
    if (tail_vecs > 0) {
        // The row's tail, one position per lane; lanes behind the row's end hold zeros.  Every lane
        // takes part in the lane shifts.
        const int p = (v0 + steps * kWave) * VEC + lane;
        const bool in_row = p < L;
        const T *xe = reinterpret_cast<const T *>(xl) + (p + VEC - tile_first) - (W - 1);
        float xw[W];
#pragma unroll
        for (int k = 0; k < W; ++k) xw[k] = in_row ? E::to_float(xe[k]) : 0.f;
        const float dv = in_row ? E::to_float(tail_d) : 0.f;
        float g[W];
        g[0] = SILU ? __builtin_fmaf(dv, act_grad(xw), 0.f) : dv;
#pragma unroll
        for (int k = 1; k < W; ++k) g[k] = from_next_lane(g[k - 1], 0.f);
        float acc = wv_[W - 1] * g[0];
#pragma unroll
        for (int k = 1; k < W; ++k) acc = fmaf(wv_[W - 1 - k], g[k], acc);
        if (has_dfinal) {
#pragma unroll
            for (int i = 0; i < W - 1; ++i)
                if (p == L - (W - 1) + i) acc += dfin[i];
        }
        if (in_row) st_elem<DT>(dxrow, p, acc);
        dB += g[0];
#pragma unroll
        for (int k = 0; k < W; ++k) dW[k] = fmaf(g[0], xw[k], dW[k]);
#pragma unroll
        for (int e = 0; e < W - 1; ++e) carry[e] = read_lane(g[0], e);
    } else {
        float xa[VEC], xb[VEC], dv[VEC];
        E::unpack(xl[steps * kWave], xa);
        E::unpack(xl[steps * kWave + 1], xb);
        E::unpack(dbehind, dv);
        float xwin[2 * (W - 1)];
#pragma unroll
        for (int i = 0; i < W - 1; ++i) { xwin[i] = xa[VEC - (W - 1) + i]; xwin[W - 1 + i] = xb[i]; }
#pragma unroll
        for (int e = 0; e < W - 1; ++e) carry[e] = SILU ? __builtin_fmaf(dv[e], act_grad(&xwin[e]), 0.f) : dv[e];
    }

#pragma unroll
    for (int s = kTileSteps - 1; s >= 0; --s) {
        if (s >= steps) continue;
        float xp[VEC], xc[VEC], dv[VEC];
        E::unpack(xl[s * kWave + lane], xp);
        E::unpack(xl[s * kWave + lane + 1], xc);
        E::unpack(dreg[s], dv);
        const int p0 = (v0 + s * kWave + lane) * VEC;      // first position of the lane's vector
        const int step_first = (v0 + s * kWave) * VEC;
        if (holds_last && L - 1 >= step_first && L - 1 < step_first + kWave * VEC) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) dv[e] = p0 + e == L - 1 ? E::to_float(last_d) : dv[e];
        }
        // xw[i] = padded x at position (first position of the lane's vector) - (W-1) + i
        float xw[VEC + W - 1], g[VEC + W - 1];
#pragma unroll
        for (int i = 0; i < W - 1; ++i) xw[i] = xp[VEC - (W - 1) + i];
#pragma unroll
        for (int e = 0; e < VEC; ++e) xw[W - 1 + e] = xc[e];
#pragma unroll
        for (int e = 0; e < VEC; ++e) g[e] = SILU ? __builtin_fmaf(dv[e], act_grad(&xw[e]), 0.f) : dv[e];
#pragma unroll
        for (int e = 0; e < W - 1; ++e) g[VEC + e] = from_next_lane(g[e], carry[e]);
#pragma unroll
        for (int e = 0; e < W - 1; ++e) carry[e] = read_lane(g[e], 0);
        float dxv[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float acc = wv_[W - 1] * g[e];
#pragma unroll
            for (int k = 1; k < W; ++k) acc = fmaf(wv_[W - 1 - k], g[e + k], acc);
            dxv[e] = acc;
            dB += g[e];
#pragma unroll
            for (int k = 0; k < W; ++k) dW[k] = fmaf(g[e], xw[e + k], dW[k]);
        }
        if (has_dfinal && L - 1 >= step_first && L - (W - 1) < step_first + kWave * VEC) {
#pragma unroll
            for (int e = 0; e < VEC; ++e)
#pragma unroll
                for (int i = 0; i < W - 1; ++i)
                    if (p0 + e == L - (W - 1) + i) dxv[e] += dfin[i];
        }
        const u32x4 packed = E::pack(dxv);
        // dwords behind the row's end are out of range: not stored
        __builtin_amdgcn_raw_buffer_store_b128(packed, rdx, vd + s * 1024, 0, 2);
        if (odd_tail && L - 1 >= p0 && L - 1 < p0 + VEC) {
            T out[VEC];
            __builtin_memcpy(out, &packed, sizeof(packed));
            st_raw<DT>(dxrow, L - 1, out[(L - 1) - p0]);
        }
        // dinitial_states[i] is dx at position i - (W-1) in front of the row: the row's first lane
        // has the g values it takes (csrc/causal_conv1d_bwd.cu:544-561)
        if (a.dinitial_states != nullptr && tile == 0 && s == 0 && lane == 0) {
#pragma unroll
            for (int i = 0; i < W - 1; ++i) {
                float acc = 0.f;
#pragma unroll
                for (int k = W - 1 - i; k < W; ++k) acc = fmaf(wv_[W - 1 - k], g[i - (W - 1) + k], acc);
                st_elem<DT>(a.dinitial_states, (int64_t)b * a.dinit_stride_b + (int64_t)c * a.dinit_stride_c +
                                                   (int64_t)i * a.dinit_stride_l, acc);
            }
        }
    }

    // The tile's sums over its lanes, in a fixed order, to plane (batch entry, tile) of the workspace.
#pragma unroll
    for (int w = 0; w < W; ++w) dW[w] = wave_total_in_lane63(dW[w]);
    dB = wave_total_in_lane63(dB);
    if (lane == kWave - 1) {
        float *dst = a.ws + ((int64_t)b * a.tiles_per_row + tile) * (int64_t)(W + 1) * a.dim + c;
#pragma unroll
        for (int w = 0; w < W; ++w) dst[(int64_t)w * a.dim] = dW[w];
        dst[(int64_t)W * a.dim] = dB;
    }
}

template <int DT, int W>
int launch_tile_act(const cc1d_bwd_params &p, const BwdCfTileArgs &a, hipStream_t stream) {
    const uint32_t blocks = (a.total + (kBlock / kWave) - 1) / (kBlock / kWave);
    // per wavefront: steps_per_tile steps of x, the vectors around them, room for a tail
    const size_t lds = (size_t)(kBlock / kWave) * (a.steps_per_tile * kWave + 2 + kTailVecs) * sizeof(u32x4);
    if (p.silu) CC1D_LAUNCH((bwd_channelfirst_tile_kernel<DT, W, true>), dim3(blocks), dim3(kBlock), lds, stream, a);
    else CC1D_LAUNCH((bwd_channelfirst_tile_kernel<DT, W, false>), dim3(blocks), dim3(kBlock), lds, stream, a);
    return launch_status();
}

template <int DT>
int launch_tile_width(const cc1d_bwd_params &p, const BwdCfTileArgs &a, hipStream_t stream) {
    switch (p.width) {
        case 2: return launch_tile_act<DT, 2>(p, a, stream);
        case 3: return launch_tile_act<DT, 3>(p, a, stream);
        default: return launch_tile_act<DT, 4>(p, a, stream);
    }
}

// The vectors of a row's last, partly filled step when they hold at most 64 positions.
int tail_vecs_of_row(const cc1d_bwd_params &p) {
    const int vec = vec_elems(p.x_dtype);
    const int rem = (int)((((int64_t)p.seqlen + vec - 1) / vec) % kWave);
    return rem > 0 && rem * vec <= kWave ? rem : 0;
}

// A row's steps are dealt to as few tiles of at most four steps as hold them, evenly (five steps:
// 3 + 2, not 4 + 1): a tile's LDS is sized for steps_per_tile, and the fewer it holds the more
// wavefronts fit a CU -- (16, 4096, 1024) bf16, two steps a row: 80.4 -> 75.7 us with LDS for two
// steps instead of four.
int64_t steps_of_row(const cc1d_bwd_params &p) {
    const int vec = vec_elems(p.x_dtype);
    const int64_t body_vecs = ((int64_t)p.seqlen + vec - 1) / vec - tail_vecs_of_row(p);
    return (body_vecs + kWave - 1) / kWave;
}
int64_t tiles_per_row(const cc1d_bwd_params &p) { return (steps_of_row(p) + kTileSteps - 1) / kTileSteps; }
int steps_per_tile(const cc1d_bwd_params &p) {
    const int64_t tiles = tiles_per_row(p);
    return (int)((steps_of_row(p) + tiles - 1) / tiles);
}

}  // namespace

// Rows of more than 64 vectors (shorter ones share wavefronts in the short-row kernel), shorter
// than 2 GiB; any alignment, any strides between rows.
bool bwd_channelfirst_tile_applies(const cc1d_bwd_params &p) {
    const int vec = vec_elems(p.x_dtype);
    return ((int64_t)p.seqlen + vec - 1) / vec > kWave && (int64_t)p.seqlen * elem_bytes(p.x_dtype) < ((int64_t)1 << 31) - 64;
}

int bwd_channelfirst_tile_parts(const cc1d_bwd_params &p) { return (int)(p.batch * tiles_per_row(p)); }

bool bwd_channelfirst_tile_fits(const cc1d_bwd_params &p) {
    return (int64_t)p.batch * p.dim * tiles_per_row(p) < wave_limit() && (int64_t)p.batch * tiles_per_row(p) < ((int64_t)1 << 30);
}

int launch_bwd_channelfirst_tile(const cc1d_bwd_params &p, float *ws, hipStream_t stream) {
    if (!bwd_channelfirst_tile_fits(p)) return CC1D_ERR_TOO_LARGE;
    BwdCfTileArgs a = {};
    a.tiles_per_row = (uint32_t)tiles_per_row(p);
    a.steps_per_tile = steps_per_tile(p);
    a.total = (uint32_t)((int64_t)p.batch * p.dim * a.tiles_per_row);
    a.seqlen = p.seqlen; a.batch = p.batch; a.dim = p.dim;
    a.tail_vecs = tail_vecs_of_row(p);
    a.body_vecs = (int32_t)(((int64_t)p.seqlen + vec_elems(p.x_dtype) - 1) / vec_elems(p.x_dtype)) - a.tail_vecs;
    a.batch_inner = p.batch > 1 && p.dim > 1 && p.x_stride_b < p.x_stride_c ? 1 : 0;
    a.w_dtype = p.w_dtype;
    a.x = p.x; a.dout = p.dout; a.dx = p.dx; a.weight = p.weight; a.bias = p.bias; a.ws = ws;
    a.x_stride_b = p.x_stride_b; a.x_stride_c = p.x_stride_c;
    a.dout_stride_b = p.dout_stride_b; a.dout_stride_c = p.dout_stride_c;
    a.dx_stride_b = p.dx_stride_b; a.dx_stride_c = p.dx_stride_c;
    a.w_stride_c = p.w_stride_c; a.w_stride_w = p.w_stride_w;
    a.initial_states = p.initial_states; a.dfinal_states = p.dfinal_states; a.dinitial_states = p.dinitial_states;
    a.init_stride_b = p.init_stride_b; a.init_stride_c = p.init_stride_c; a.init_stride_l = p.init_stride_l;
    a.dfinal_stride_b = p.dfinal_stride_b; a.dfinal_stride_c = p.dfinal_stride_c; a.dfinal_stride_l = p.dfinal_stride_l;
    a.dinit_stride_b = p.dinit_stride_b; a.dinit_stride_c = p.dinit_stride_c; a.dinit_stride_l = p.dinit_stride_l;
    switch (p.x_dtype) {
        case CC1D_F32: return launch_tile_width<CC1D_F32>(p, a, stream);
        case CC1D_F16: return launch_tile_width<CC1D_F16>(p, a, stream);
        default: return launch_tile_width<CC1D_BF16>(p, a, stream);
    }
}

}  // namespace cc1d
