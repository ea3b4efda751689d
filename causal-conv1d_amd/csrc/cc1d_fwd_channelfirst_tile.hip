// Channel-first forward for gfx950: short-lived tile wavefronts.  Takes over
// causal_conv1d_fwd_kernel (csrc/causal_conv1d_fwd.cu:46-170 of the reference) for rows of more
// than 64 sixteen-byte vectors: rows of whole vectors on the 16-byte grid that start on 128-byte
// lines (tensors of up to 512 MiB) or hold at most 128 vectors, and rows off that grid -- a length
// that is no whole number of vectors, a view that starts inside a vector, out on another grid
// than x -- of up to 512 vectors of 16-bit data, 192 of fp32.  Everything else stays with the
// kernels of cc1d_fwd_channelfirst.hip (see fwd_channelfirst_tile_applies below for the
// measurements behind the limits).
//
// Design.  A wavefront takes a tile of up to four 64-vector steps (4 KiB) of one (batch, channel)
// row and asks for all of it at once: the data goes from memory straight into LDS
// (buffer_load_dwordx4 ... lds), together with the vector in front of the tile, whose last W-1
// elements are the tile's halo.  No registers are held while the tile is in flight, a tile needs
// 4.4 KB of LDS, and eight wavefronts fit a SIMD; they live for one memory round trip and a few
// hundred instructions, so the launch moves through memory as one compact front in the order of
// the rows instead of as thousands of long-lived streams.  The row is a buffer resource of its
// own: the lane's vector is the vector offset, the step the instruction's immediate offset (which
// the hardware adds to the LDS address as well), and what lies outside the row needs no test --
// the vector in front of the first tile and the steps behind the row's end are out of range, read
// as zeros and are not stored.  A lane's left neighbours come out of LDS (the upper half of the
// previous vector), so there is no cross-lane traffic and no barrier.  The resource is based at
// the row's first element wherever that lies (vector accesses need no alignment), so rows of any
// length anywhere in memory take the same path; a 16-bit row of odd length ends in half a dword,
// which the range check would drop: that one element is fetched and stored on its own.  A row
// whose last 64-vector step would hold at most 64 positions ends in a tail instead: the last
// tile fetches those vectors as well and produces their positions one per lane.
#include <type_traits>

#include "cc1d_device.hpp"
#include "cc1d_internal.hpp"

namespace cc1d {
namespace {

constexpr int kTileSteps = 4;                     // 64-vector steps per tile
constexpr int kTileVecs = kTileSteps * kWave;     // 256 vectors, 4 KiB
constexpr int kTailVecs = kWave / 4;              // most vectors 64 positions can span (fp32)
constexpr int kLdsVecs = kTileVecs + 1 + kTailVecs; // LDS vectors of one wavefront
constexpr int kRsrcRaw = 0x00020000;              // buffer resource word 3: raw buffer, 32-bit data format

typedef void __attribute__((address_space(3))) *lds_ptr_t;

struct FwdCfTileArgs {
    uint32_t total;               // rows * tiles_per_row wavefronts
    uint32_t tiles_per_row;
    int32_t seqlen;
    int32_t body_vecs;            // vectors of a row that are walked as vectors (all of them, or a whole number of steps)
    int32_t tail_vecs;            // vectors behind them, done one position per lane (0: none)
    int32_t batch, dim;
    int32_t batch_inner;          // rows numbered with the batch entry fastest
    int32_t w_dtype;
    int32_t states;               // bit 0: initial_states given, bit 1: final_states wanted
    const void *x;
    void *out;
    const void *weight;
    const void *bias;
    int64_t x_stride_b, x_stride_c, out_stride_b, out_stride_c;     // elements
    int64_t w_stride_c, w_stride_w;
    const void *initial_states;
    void *final_states;
    int64_t init_stride_b, init_stride_c, init_stride_l;
    int64_t final_stride_b, final_stride_c, final_stride_l;
};

template <int DT, int W, bool SILU>
__global__ void __launch_bounds__(kBlock, 4)
fwd_channelfirst_tile_kernel(const FwdCfTileArgs a) {
    using E = Elem<DT>;
    using T = typename E::type;
    constexpr int VEC = E::kVec;
    constexpr int EB = E::kBytes;
    constexpr bool PRECISE = E::kPreciseAct;
    constexpr bool SCALED = SILU && !PRECISE;         // taps and bias carry the factor of the SiLU exponent
    extern __shared__ u32x4 lds[];                    // [wavefront][halo vector + tile + tail]

    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const int lane = (int)(threadIdx.x & (kWave - 1));
    const uint32_t wid = blockIdx.x * (uint32_t)(kBlock / kWave) + (uint32_t)wv;
    if (wid >= a.total) return;
    const int tile = (int)(wid % a.tiles_per_row);
    const uint32_t row = wid / a.tiles_per_row;
    // Channels run fastest for tensors whose rows lie in (batch, dim) order in memory; for a
    // (dim, batch, seqlen) tensor seen as (batch, dim, seqlen) the batch entries of a channel are
    // the neighbours in memory and run fastest instead.
    int b, c;
    if (a.batch_inner) { b = (int)(row % (uint32_t)a.batch); c = (int)(row / (uint32_t)a.batch); }
    else { c = (int)(row % (uint32_t)a.dim); b = (int)(row / (uint32_t)a.dim); }

    const T *xrow = reinterpret_cast<const T *>(a.x) + (int64_t)b * a.x_stride_b + (int64_t)c * a.x_stride_c;
    T *orow = reinterpret_cast<T *>(a.out) + (int64_t)b * a.out_stride_b + (int64_t)c * a.out_stride_c;
    const int L = a.seqlen;
    // The range check works on whole dwords: a 16-bit row of odd length ends in half a dword,
    // which stays outside the resources; its element is moved separately below.
    const int row_bytes = (L * EB) & ~3;
    const bool odd_tail = ((L * EB) & 2) != 0;
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(xrow), 0, row_bytes, kRsrcRaw);
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(orow, 0, row_bytes, kRsrcRaw);
    const int v0 = tile * kTileVecs;                  // the tile's first vector
    int steps = (a.body_vecs - v0 + kWave - 1) / kWave;   // steps of the tile that reach into the row
    steps = steps > kTileSteps ? kTileSteps : steps;
    const bool last_tile = tile == (int)a.tiles_per_row - 1;
    // A row whose last step would hold at most 64 positions ends in a tail instead: its last tile
    // fetches those vectors too and produces their positions one per lane (an eighth of a step's
    // instructions instead of a whole step for a handful of lanes).
    const int tail_vecs = last_tile ? a.tail_vecs : 0;
    // LDS vector i of the wavefront holds row vector v0 - 1 + i.  For the row's first tile the
    // offset below wraps around: out of range, LDS gets zeros (the row's zero padding).
    const int vx = (lane + v0 - 1) * 16;
    u32x4 *mine = lds + wv * kLdsVecs;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)mine, 16, vx, 0, 0, 2);
    if (steps > 1) __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)mine, 16, vx, 0, 1024, 2);
    if (steps > 2) __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)mine, 16, vx, 0, 2048, 2);
    if (steps > 3) __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)mine, 16, vx, 0, 3072, 2);
    if (lane < 1 + tail_vecs) __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)(mine + steps * kWave), 16, vx + steps * 1024, 0, 0, 2);

    float wv_[W], bias_v;
#pragma unroll
    for (int w = 0; w < W; ++w)
        wv_[w] = ld_weight(a.weight, a.w_dtype, (int64_t)c * a.w_stride_c + w * a.w_stride_w);
    bias_v = a.bias == nullptr ? 0.f : ld_weight(a.bias, a.w_dtype, c);
    if (SCALED) {
        bias_v *= kSiluPrescale;
#pragma unroll
        for (int w = 0; w < W; ++w) wv_[w] *= kSiluPrescale;
    }
    // The row's first tile takes initial_states as its halo: its first lane fetches the W-1 values.
    float init[W - 1];
#pragma unroll
    for (int i = 0; i < W - 1; ++i) init[i] = 0.f;
    const bool first_lane_of_row = tile == 0 && lane == 0;
    if ((a.states & 1) != 0 && first_lane_of_row) {
#pragma unroll
        for (int i = 0; i < W - 1; ++i)
            init[i] = ld_elem<DT>(a.initial_states, (int64_t)b * a.init_stride_b + (int64_t)c * a.init_stride_c +
                                                        (int64_t)i * a.init_stride_l);
    }
    // The odd last element of a 16-bit row, by the first lane of the tile that holds it.
    const int tile_first = v0 * VEC;                  // the tile's positions start here
    const bool holds_last = odd_tail && last_tile;
    T last_x = T(0.f);
    if (holds_last && lane == 0) last_x = ld_raw<DT>(xrow, L - 1);
    // Every vector of the tile is in LDS behind this wait (a vector fetched into LDS counts as a
    // load until it has been written there).
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (holds_last && lane == 0) reinterpret_cast<T *>(mine)[L - 1 + VEC - tile_first] = last_x;
    asm volatile("" ::: "memory");                    // the element written above is read below as part of a vector

    for (int s = 0; s < steps; ++s) {
        float xp[VEC], xc[VEC];
        E::unpack(mine[s * kWave + lane], xp);
        E::unpack(mine[s * kWave + lane + 1], xc);
        // xx[i] = padded x at position (first position of the lane's vector) - (W-1) + i
        float xx[VEC + W - 1];
#pragma unroll
        for (int i = 0; i < W - 1; ++i) xx[i] = xp[VEC - (W - 1) + i];
        if (s == 0 && first_lane_of_row) {
#pragma unroll
            for (int i = 0; i < W - 1; ++i) xx[i] = init[i];
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) xx[W - 1 + e] = xc[e];
        float acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float s_ = bias_v;
#pragma unroll
            for (int w = 0; w < W; ++w) s_ = fmaf(wv_[w], xx[e + w], s_);
            acc[e] = SCALED ? silu_from_scaled(s_) : SILU ? silu<PRECISE>(s_) : s_;
        }
        // dwords behind the row's end are out of range: not stored
        const u32x4 packed = E::pack(acc);
        __builtin_amdgcn_raw_buffer_store_b128(packed, ro, (lane + v0) * 16 + s * 1024, 0, 2);
        const int p0 = (v0 + s * kWave + lane) * VEC;  // first position of the lane's vector
        if (odd_tail && L - 1 >= p0 && L - 1 < p0 + VEC) {
            T o[VEC];
            __builtin_memcpy(o, &packed, sizeof(packed));
            st_raw<DT>(orow, L - 1, o[(L - 1) - p0]);
        }
    }

    if (tail_vecs > 0) {
        const int p = (v0 + steps * kWave) * VEC + lane;   // one position per lane
        if (p < L) {
            const T *win = reinterpret_cast<const T *>(mine) + (p + VEC - tile_first) - (W - 1);
            float s_ = bias_v;
#pragma unroll
            for (int w = 0; w < W; ++w) s_ = fmaf(wv_[w], E::to_float(win[w]), s_);
            st_elem<DT>(orow, p, SCALED ? silu_from_scaled(s_) : SILU ? silu<PRECISE>(s_) : s_);
        }
    }

    // final_states[b, c, i] = x[L-(W-1)+i], copied by the wavefront of the row's FIRST tile, the
    // one that read initial_states: the two may be one buffer, and inside one wavefront the
    // reads are complete (the wait above) before the stores.  Rows here hold more than 64
    // vectors, so the values all come from x.
    if ((a.states & 2) != 0 && tile == 0 && lane < W - 1) {
        const T v = ld_raw<DT>(xrow, L - (W - 1) + lane);
        st_raw<DT>(a.final_states, (int64_t)b * a.final_stride_b + (int64_t)c * a.final_stride_c +
                                       (int64_t)lane * a.final_stride_l, v);
    }
}

template <int DT, int W>
int launch_tile_act(const cc1d_fwd_params &p, const FwdCfTileArgs &a, hipStream_t stream) {
    const uint32_t blocks = (a.total + (kBlock / kWave) - 1) / (kBlock / kWave);
    // What the four wavefronts' tiles take (eight workgroups fit a CU), and for rows of three steps
    // and more a fifth of a CU's LDS: wavefronts that fetch 3-4 KiB each run 2-4 % faster five
    // workgroups to a CU than eight -- (8, 5376, 2048) bf16 57.9 -> 56.6 us, (4, 4096, 8192) fp16
    // 87.6 -> 83.8, (8, 5376, 4095) 123.5 -> 120.9 -- while rows of two steps lose ((16, 4096, 1001)
    // 48.6 -> 56.0 us) and keep all eight.
    size_t lds = (size_t)(kBlock / kWave) * kLdsVecs * sizeof(u32x4);
    if (a.body_vecs > 2 * kWave && lds < 160 * 1024 / 5) lds = 160 * 1024 / 5;
    if (p.silu) CC1D_LAUNCH((fwd_channelfirst_tile_kernel<DT, W, true>), dim3(blocks), dim3(kBlock), lds, stream, a);
    else CC1D_LAUNCH((fwd_channelfirst_tile_kernel<DT, W, false>), dim3(blocks), dim3(kBlock), lds, stream, a);
    return launch_status();
}

template <int DT>
int launch_tile_width(const cc1d_fwd_params &p, const FwdCfTileArgs &a, hipStream_t stream) {
    switch (p.width) {
        case 2: return launch_tile_act<DT, 2>(p, a, stream);
        case 3: return launch_tile_act<DT, 3>(p, a, stream);
        default: return launch_tile_act<DT, 4>(p, a, stream);
    }
}

}  // namespace

// Which launches take tiles (rows of at most 64 vectors share wavefronts in the short-row kernel).
// Over rotating buffer sets, tiles against the walking kernel, us:
//  * rows of whole vectors on the 16-byte grid, up to twice 64 vectors: a walking wavefront has one
//    or two steps and nothing to overlap its own latency with; (4, 5376, 520) bf16 13.1 / 15.2,
//    (16, 5376, 1024) 55.8 / 60.7, (64, 2048, 1024) fp16 with states 89.5 / 105.7;
//  * longer rows when every row of x and of out starts on a 128-byte line and a tensor holds at
//    most 512 MiB: (4, 2048, 4096) bf16 24.2 / 25.1, fp32 43.2 / 44.1, (8, 5376, 2048) bf16 56.8 / 58.2,
//    (1, 5376, 2048) 10.0 / 11.2, (2, 1024, 2048) 5.3 / 7.0.  Beyond that size the walk, whose
//    wavefronts are fewer and longer-lived, is ahead ((64, 5376, 2048) bf16 459.8 / 448.0), and so it is
//    for rows on the grid that do not start on lines, where it moves the steps of a row onto the
//    lines of out and a tile cannot ((8, 5376, 3000) bf16 90.6 / 83.7, (8, 5376, 1500) fp32 88.6 / 83.6);
//  * rows off the grid (a length that is no whole number of vectors, a view that starts inside a
//    vector, out on another grid than x), up to 512 vectors of 16-bit data and 192 of fp32: the
//    walking kernels do the positions outside whole vectors one per lane in front of every row's
//    walk, which costs a row of one or two steps more than the row itself; (16, 4096, 1001) bf16
//    49.1 / 79.7, 1501: 69.9 / 88.9, (4, 4096, 4095) 48.2 / 54.5, 8191: 101.7 / 92.5; fp32 (8, 4096, 513)
//    28.3 / 31.2, 1001: 54.3 / 52.4, 2047: 108.2 / 94.7.
bool fwd_channelfirst_tile_applies(const cc1d_fwd_params &p) {
    const int vec = vec_elems(p.x_dtype), eb = elem_bytes(p.x_dtype);
    const int64_t n_vecs = ((int64_t)p.seqlen + vec - 1) / vec;
    if (n_vecs <= kWave || (int64_t)p.seqlen * eb >= ((int64_t)1 << 31) - 64) return false;
    const bool on_grid = p.seqlen % vec == 0 &&
                         aligned16(p.x) && p.x_stride_b % vec == 0 && p.x_stride_c % vec == 0 &&
                         aligned16(p.out) && p.out_stride_b % vec == 0 && p.out_stride_c % vec == 0;
    if (!on_grid) return n_vecs <= (p.x_dtype == CC1D_F32 ? 3 * kWave : 8 * kWave);
    if (n_vecs <= 2 * kWave) return true;
    auto on_lines = [eb](const void *base, int64_t stride_b, int64_t stride_c) {
        return reinterpret_cast<uintptr_t>(base) % 128 == 0 && stride_b * eb % 128 == 0 && stride_c * eb % 128 == 0;
    };
    return on_lines(p.x, p.x_stride_b, p.x_stride_c) && on_lines(p.out, p.out_stride_b, p.out_stride_c) &&
           (int64_t)p.batch * p.dim * p.seqlen * eb <= ((int64_t)1 << 29);
}

int launch_fwd_channelfirst_tile(const cc1d_fwd_params &p, hipStream_t stream) {
    const int vec = vec_elems(p.x_dtype);
    FwdCfTileArgs a = {};
    a.seqlen = p.seqlen;
    const int n_vecs = (int)(((int64_t)p.seqlen + vec - 1) / vec);
    const int rem = n_vecs % kWave;
    a.tail_vecs = rem > 0 && rem * vec <= kWave ? rem : 0;
    a.body_vecs = n_vecs - a.tail_vecs;
    a.tiles_per_row = (uint32_t)((a.body_vecs + kTileVecs - 1) / kTileVecs);
    const int64_t total = (int64_t)p.batch * p.dim * a.tiles_per_row;
    if (total >= wave_limit()) return CC1D_ERR_TOO_LARGE;
    a.total = (uint32_t)total;
    a.batch = p.batch; a.dim = p.dim;
    a.batch_inner = p.batch > 1 && p.dim > 1 && p.x_stride_b < p.x_stride_c ? 1 : 0;
    a.w_dtype = p.w_dtype;
    a.states = (p.initial_states != nullptr ? 1 : 0) | (p.final_states != nullptr ? 2 : 0);
    a.x = p.x; a.out = p.out; a.weight = p.weight; a.bias = p.bias;
    a.x_stride_b = p.x_stride_b; a.x_stride_c = p.x_stride_c;
    a.out_stride_b = p.out_stride_b; a.out_stride_c = p.out_stride_c;
    a.w_stride_c = p.w_stride_c; a.w_stride_w = p.w_stride_w;
    a.initial_states = p.initial_states; a.final_states = p.final_states;
    a.init_stride_b = p.init_stride_b; a.init_stride_c = p.init_stride_c; a.init_stride_l = p.init_stride_l;
    a.final_stride_b = p.final_stride_b; a.final_stride_c = p.final_stride_c; a.final_stride_l = p.final_stride_l;
    switch (p.x_dtype) {
        case CC1D_F32: return launch_tile_width<CC1D_F32>(p, a, stream);
        case CC1D_F16: return launch_tile_width<CC1D_F16>(p, a, stream);
        default: return launch_tile_width<CC1D_BF16>(p, a, stream);
    }
}

}  // namespace cc1d
