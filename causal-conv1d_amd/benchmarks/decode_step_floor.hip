// What a launch of the decode step's size costs on this part, and how close the step kernel is to it.
// A standalone program (HIP runtime only, no PyTorch): the library's own launch_update at the decode
// shape (bf16, batch 256, dim 5376, width 4, SiLU; conv_state (256, 5376, 3) shifted in place, then
// (256, 5376, 8) as a ring buffer), next to an empty kernel of the same grid, to copy kernels that move
// the linear step's exact footprint (per lane and batch row: three state rows and x in, three state rows
// and out back) with 4-, 8- and 16-byte lanes and 1, 2 or 4 rows per lane, and to the step kernel
// itself at other lane widths and rows per lane.  HIP events around N back-to-back launches on one set
// of buffers (warm) and over 40 rotating sets (more than the 256 MB Infinity Cache).
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         -Iinclude -Icausal-conv1d_amd/csrc causal-conv1d_amd/benchmarks/decode_step_floor.hip -o /tmp/decode_step_floor
//   /tmp/decode_step_floor 2000
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include <algorithm>
#include "../csrc/cc1d_update.hip"

namespace cc1d { Tunables &tunables() { static Tunables t; return t; } }
using namespace cc1d;

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); exit(1);} } while (0)

__global__ void __launch_bounds__(256) empty_kernel(const StepArgs a) { if (a.batch < 0) *(int *)a.out = 0; }

// Same footprint as the linear step, no arithmetic: per (row, colgroup) read 4 x 8 bytes, write 4 x 8 bytes.
// NT: the state rows with the non-temporal policy, as the step kernel reads and writes them.
template <bool NT>
__global__ void __launch_bounds__(256) copy_kernel(const StepArgs a) {
    using raw_t = u32x2;
    const uint32_t lane = threadIdx.x & 63;
    const int c0 = (int)(blockIdx.x * 64 + lane) * 4;
    const int b0 = ((int)blockIdx.y * 4 + (int)(threadIdx.x / 64)) * 2;
    const __bf16 *xb = reinterpret_cast<const __bf16 *>(a.x);
    __bf16 *ob = reinterpret_cast<__bf16 *>(a.out);
    __bf16 *sb = reinterpret_cast<__bf16 *>(a.conv_state);
    raw_t v[2][4];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const raw_t *src = reinterpret_cast<const raw_t *>(sb + (int64_t)(b0 + r) * a.state_stride_b + c0 + (int64_t)i * a.state_stride_l);
            v[r][i] = NT ? __builtin_nontemporal_load(src) : *src;
        }
        v[r][3] = *reinterpret_cast<const raw_t *>(xb + (int64_t)(b0 + r) * a.x_stride_b + c0);
    }
#pragma unroll
    for (int r = 0; r < 2; ++r) {
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            raw_t *dst = reinterpret_cast<raw_t *>(sb + (int64_t)(b0 + r) * a.state_stride_b + c0 + (int64_t)i * a.state_stride_l);
            if (NT) __builtin_nontemporal_store(v[r][(i + 1) & 3], dst);
            else *dst = v[r][(i + 1) & 3];
        }
        *reinterpret_cast<raw_t *>(ob + (int64_t)(b0 + r) * a.out_stride_b + c0) = v[r][0];
    }
}

template <int CHB, int R>   // CHB channels (2 bytes each) per lane, R rows per lane, 4 waves per block
__global__ void __launch_bounds__(256) copy_kernel_t(const StepArgs a) {
    using raw_t = typename RawBytes<CHB * 2>::type;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t ncg = (uint32_t)(a.n_colgroups * 4 / CHB);
    const uint32_t cg = blockIdx.x * 64 + lane;
    if (cg >= ncg) return;
    const int c0 = (int)cg * CHB;
    const int b0 = ((int)blockIdx.y * 4 + (int)(threadIdx.x / 64)) * R;
    const __bf16 *xb = reinterpret_cast<const __bf16 *>(a.x);
    __bf16 *ob = reinterpret_cast<__bf16 *>(a.out);
    __bf16 *sb = reinterpret_cast<__bf16 *>(a.conv_state);
    raw_t v[R][4];
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int i = 0; i < 3; ++i) v[r][i] = *reinterpret_cast<const raw_t *>(sb + (int64_t)(b0 + r) * a.state_stride_b + c0 + (int64_t)i * a.state_stride_l);
        v[r][3] = *reinterpret_cast<const raw_t *>(xb + (int64_t)(b0 + r) * a.x_stride_b + c0);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int i = 0; i < 3; ++i) *reinterpret_cast<raw_t *>(sb + (int64_t)(b0 + r) * a.state_stride_b + c0 + (int64_t)i * a.state_stride_l) = v[r][(i + 1) & 3];
        *reinterpret_cast<raw_t *>(ob + (int64_t)(b0 + r) * a.out_stride_b + c0) = v[r][0];
    }
}

struct Set { void *x, *out, *state; };

int main(int argc, char **argv) {
    const int B = 256, D = 5376, W = 4;
    const int iters = argc > 1 ? atoi(argv[1]) : 2000;
    hipStream_t stream; CK(hipStreamCreate(&stream));
    std::vector<uint16_t> hx((size_t)B * D), hst((size_t)B * 8 * D);
    srand(1);
    auto rnd_bf16 = [] { float f = (rand() / (float)RAND_MAX - 0.5f) * 4.f; uint32_t u; memcpy(&u, &f, 4); return (uint16_t)(u >> 16); };
    for (auto &v : hx) v = rnd_bf16();
    for (auto &v : hst) v = rnd_bf16();
    std::vector<float> hw((size_t)D * W), hb(D);
    for (auto &v : hw) v = rand() / (float)RAND_MAX - 0.5f;
    for (auto &v : hb) v = rand() / (float)RAND_MAX - 0.5f;
    std::vector<int32_t> hcs(B);
    for (auto &v : hcs) v = rand() % 1000;
    float *dw, *db; int32_t *dcs;
    CK(hipMalloc(&dw, hw.size() * 4)); CK(hipMalloc(&db, hb.size() * 4)); CK(hipMalloc(&dcs, B * 4));
    CK(hipMemcpy(dw, hw.data(), hw.size() * 4, hipMemcpyHostToDevice));
    CK(hipMemcpy(db, hb.data(), hb.size() * 4, hipMemcpyHostToDevice));
    CK(hipMemcpy(dcs, hcs.data(), B * 4, hipMemcpyHostToDevice));
    const int NSETS = 40;
    for (int circ = 0; circ < 2; ++circ) {
        const int S = circ ? 8 : 3;
        std::vector<Set> sets(NSETS);
        for (auto &s : sets) {
            CK(hipMalloc(&s.x, (size_t)B * D * 2)); CK(hipMalloc(&s.out, (size_t)B * D * 2)); CK(hipMalloc(&s.state, (size_t)B * S * D * 2));
            CK(hipMemcpy(s.x, hx.data(), (size_t)B * D * 2, hipMemcpyHostToDevice));
            CK(hipMemcpy(s.state, hst.data(), (size_t)B * S * D * 2, hipMemcpyHostToDevice));
        }
        auto params = [&](const Set &s) {
            cc1d_update_params p = {};
            p.batch = B; p.dim = D; p.seqlen = 1; p.width = W; p.state_len = S; p.state_batch = B;
            p.x_dtype = CC1D_BF16; p.w_dtype = CC1D_F32; p.silu = 1;
            p.x = s.x; p.x_stride_b = D; p.x_stride_c = 1; p.x_stride_l = D;
            p.conv_state = s.state; p.state_stride_b = (int64_t)S * D; p.state_stride_c = 1; p.state_stride_l = D;
            p.weight = dw; p.w_stride_c = W; p.w_stride_w = 1; p.bias = db;
            p.out = s.out; p.out_stride_b = D; p.out_stride_c = 1; p.out_stride_l = D;
            p.cache_seqlens = circ ? dcs : nullptr;
            return p;
        };
        auto args = [&](const Set &s) {
            StepArgs a; a.x = s.x; a.out = s.out; a.conv_state = s.state; a.weight = dw; a.bias = db;
            a.cache_seqlens = circ ? dcs : nullptr; a.conv_state_indices = nullptr;
            a.x_stride_b = D; a.out_stride_b = D; a.state_stride_b = (int64_t)S * D; a.state_stride_l = D;
            a.batch = B; a.state_len = S; a.n_colgroups = D / 4; return a;
        };
        struct Variant { const char *name; void (*launch)(const StepArgs &, const cc1d_update_params &, hipStream_t, int); };
        const int c = circ;
        std::vector<Variant> vs;
        vs.push_back({"library launch_update", [](const StepArgs &, const cc1d_update_params &p, hipStream_t s, int) { launch_update(p, s); }});
        vs.push_back({"empty kernel, same grid", [](const StepArgs &a, const cc1d_update_params &, hipStream_t s, int) { hipLaunchKernelGGL(empty_kernel, dim3(21, 32), dim3(256), 0, s, a); }});
        vs.push_back({"copy kernel, linear footprint", [](const StepArgs &a, const cc1d_update_params &, hipStream_t s, int) { hipLaunchKernelGGL(copy_kernel<false>, dim3(21, 32), dim3(256), 0, s, a); }});
        vs.push_back({"copy kernel, state rows non-temporal", [](const StepArgs &a, const cc1d_update_params &, hipStream_t s, int) { hipLaunchKernelGGL(copy_kernel<true>, dim3(21, 32), dim3(256), 0, s, a); }});
#define COPYT(CHB, R) vs.push_back({"copy " #CHB " ch/lane R=" #R, [](const StepArgs &a, const cc1d_update_params &, hipStream_t s, int) { \
            const uint32_t ncg = a.n_colgroups * 4 / CHB; \
            hipLaunchKernelGGL((copy_kernel_t<CHB, R>), dim3((ncg + 63) / 64, a.batch / (4 * R)), dim3(256), 0, s, a); }})
        COPYT(4, 1); COPYT(4, 2); COPYT(4, 4); COPYT(8, 1); COPYT(8, 2); COPYT(8, 4); COPYT(2, 2); COPYT(2, 4);
#define LIBK(CH, R) vs.push_back({"step kernel CH=" #CH " R=" #R, [](const StepArgs &a0, const cc1d_update_params &, hipStream_t s, int circ) { \
            StepArgs a = a0; a.n_colgroups = a0.n_colgroups * 4 / CH; \
            const dim3 grid((a.n_colgroups + 63) / 64, (a.batch + 4 * R - 1) / (4 * R)); \
            if (circ) hipLaunchKernelGGL((update_step_kernel<CC1D_BF16, CH, 4, true, true, R, 1>), grid, dim3(256), 0, s, a); \
            else hipLaunchKernelGGL((update_step_kernel<CC1D_BF16, CH, 4, false, true, R, 1>), grid, dim3(256), 0, s, a); }})
        LIBK(4, 1); LIBK(4, 2); LIBK(4, 4); LIBK(8, 1); LIBK(8, 2); LIBK(2, 2); LIBK(2, 4);
        // correctness of every variant against the library on fresh copies
        std::vector<uint16_t> ref_out((size_t)B * D), ref_st((size_t)B * S * D), got_out((size_t)B * D), got_st((size_t)B * S * D);
        for (size_t v = 0; v < vs.size(); ++v) {
            if (strstr(vs[v].name, "empty") || strstr(vs[v].name, "copy")) continue;
            CK(hipMemcpy(sets[0].state, hst.data(), (size_t)B * S * D * 2, hipMemcpyHostToDevice));
            CK(hipMemset(sets[0].out, 0, (size_t)B * D * 2));
            vs[v].launch(args(sets[0]), params(sets[0]), stream, c);
            CK(hipStreamSynchronize(stream));
            auto &o = v == 0 ? ref_out : got_out; auto &st = v == 0 ? ref_st : got_st;
            CK(hipMemcpy(o.data(), sets[0].out, o.size() * 2, hipMemcpyDeviceToHost));
            CK(hipMemcpy(st.data(), sets[0].state, st.size() * 2, hipMemcpyDeviceToHost));
            if (v > 0 && (memcmp(ref_out.data(), got_out.data(), o.size() * 2) || memcmp(ref_st.data(), got_st.data(), st.size() * 2)))
                printf("MISMATCH %s\n", vs[v].name);
        }
        hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
        auto time_it = [&](const Variant &v, bool rotate) {
            for (int i = 0; i < 200; ++i) v.launch(args(sets[rotate ? i % NSETS : 0]), params(sets[rotate ? i % NSETS : 0]), stream, c);
            CK(hipStreamSynchronize(stream));
            CK(hipEventRecord(e0, stream));
            for (int i = 0; i < iters; ++i) v.launch(args(sets[rotate ? i % NSETS : 0]), params(sets[rotate ? i % NSETS : 0]), stream, c);
            CK(hipEventRecord(e1, stream)); CK(hipEventSynchronize(e1));
            float ms; CK(hipEventElapsedTime(&ms, e0, e1));
            return ms * 1e3f / iters;
        };
        printf("== %s (S=%d), %d launches per figure, us per launch: warm (3 rounds) | rotated over %d sets (2 rounds)\n", circ ? "circular" : "linear", S, iters, NSETS);
        std::vector<std::vector<float>> warm(vs.size()), rot(vs.size());
        for (int round = 0; round < 3; ++round)
            for (size_t v = 0; v < vs.size(); ++v) warm[v].push_back(time_it(vs[v], false));
        for (int round = 0; round < 2; ++round)
            for (size_t v = 0; v < vs.size(); ++v) rot[v].push_back(time_it(vs[v], true));
        for (size_t v = 0; v < vs.size(); ++v)
            printf("%-34s warm %.3f %.3f %.3f | rotated %.3f %.3f\n", vs[v].name, warm[v][0], warm[v][1], warm[v][2], rot[v][0], rot[v][1]);
        fflush(stdout);
        for (auto &s : sets) { CK(hipFree(s.x)); CK(hipFree(s.out)); CK(hipFree(s.state)); }
    }
    return 0;
}
