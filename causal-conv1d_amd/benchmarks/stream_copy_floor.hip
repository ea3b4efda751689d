// What HBM gives a kernel that reads a tensor once and writes one of the same size, on buffers no
// cache holds, and how much of it the channel-last kernels' way of walking a tensor keeps.
// A standalone program (HIP runtime only, no PyTorch), no arithmetic in any kernel:
//   linear copies   one 16-byte vector per thread, workgroups in hardware order, with plain or
//                   non-temporal loads and stores; the read half and the write half alone;
//   row-walk copies the access pattern of fwd_channellast_kernel: the tensor is (rows x row_bytes),
//                   a wavefront owns 64 lanes x LB bytes of a row and walks T consecutive rows, U rows
//                   requested at a time in two register sets (ping-pong) or one, workgroups in
//                   hardware order or in chunks of `chunk` runs per XCD as the library orders them.
//   row-stream copies the access pattern of the channel-first kernels: the tensor is (batch, channels,
//                   row_bytes), a wavefront owns `segs`-th parts of the rows of one channel and streams
//                   them 1 KB (64 lanes x 16 bytes) at a time, `depth` steps requested ahead, either
//                   walking the batch itself or one batch entry per wavefront; with a second input
//                   tensor (the backward's x and dout) or one (the forward).
// Default tensor: 16384 rows of 10752 bytes, the prefill forward's x (8 x 2048 rows of 5376 bf16);
// the row-stream copies run at the shapes of the forward sweep, (4, 2048, 4096) 16-bit, and of the
// backward configuration, (4, 4096, 8192) 16-bit.
// Every figure is the median of five bursts of launches over rotating sets of buffers (more than
// the 256 MB last-level cache), HIP events around each burst.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         causal-conv1d_amd/benchmarks/stream_copy_floor.hip -o /tmp/stream_copy_floor
//   /tmp/stream_copy_floor [rows row_bytes]
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); exit(1); } } while (0)

typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
template <int LB> struct Lane;
template <> struct Lane<4> { typedef unsigned int type; };
template <> struct Lane<8> { typedef u32x2 type; };
template <> struct Lane<16> { typedef u32x4 type; };

template <bool NT_LOAD, bool NT_STORE>
__global__ void __launch_bounds__(256) linear_copy(const u32x4 *src, u32x4 *dst, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const u32x4 v = NT_LOAD ? __builtin_nontemporal_load(src + i) : src[i];
    if (NT_STORE) __builtin_nontemporal_store(v, dst + i);
    else dst[i] = v;
}
__global__ void __launch_bounds__(256) linear_read(const u32x4 *src, u32x4 *dst, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const u32x4 v = __builtin_nontemporal_load(src + i);
    if (v.x == 0x12345678u && v.y == 0x9abcdef0u && v.z == v.w) dst[i] = v;     // never with these inputs
}
__global__ void __launch_bounds__(256) linear_write(u32x4 *dst, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) __builtin_nontemporal_store(u32x4{1u, 2u, 3u, (unsigned)i}, dst + i);
}

// chunk_blocks: workgroups an XCD takes in a row before the next XCD's (0: hardware order).
template <int LB, int U, bool PING>
__global__ void __launch_bounds__(256) row_walk_copy(const char *src, char *dst, int rows, int row_bytes, int T,
                                                     int waves_per_row, unsigned total_waves, unsigned chunk_blocks) {
    typedef typename Lane<LB>::type V;
    unsigned block = blockIdx.x;
    if (chunk_blocks) {
        const unsigned xcd = blockIdx.x % 8, nth = blockIdx.x / 8;
        block = ((nth / chunk_blocks) * 8 + xcd) * chunk_blocks + nth % chunk_blocks;
    }
    const unsigned wave = block * 4 + threadIdx.x / 64, lane = threadIdx.x % 64;
    if (wave >= total_waves) return;
    const unsigned col = (wave % waves_per_row) * 64 + lane, run = wave / waves_per_row;
    if ((int)(col * LB) >= row_bytes) return;
    const size_t off = (size_t)run * T * row_bytes + (size_t)col * LB;
    const char *s = src + off;
    char *d = dst + off;
    int n = rows - (int)run * T;                      // a multiple of 2 U by the choice of sizes below
    if (n > T) n = T;
    auto row_in = [&](int r) { return __builtin_nontemporal_load(reinterpret_cast<const V *>(s + (size_t)r * row_bytes)); };
    auto row_out = [&](int r, V v) { __builtin_nontemporal_store(v, reinterpret_cast<V *>(d + (size_t)r * row_bytes)); };
    if (!PING) {
        for (int r = 0; r < n; r += U) {
            V v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = row_in(r + u);
#pragma unroll
            for (int u = 0; u < U; ++u) row_out(r + u, v[u]);
        }
    } else {
        V a[U], b[U];
#pragma unroll
        for (int u = 0; u < U; ++u) a[u] = row_in(u);
        for (int r = 0; r < n; r += 2 * U) {
#pragma unroll
            for (int u = 0; u < U; ++u) b[u] = row_in(r + U + u);
#pragma unroll
            for (int u = 0; u < U; ++u) row_out(r + u, a[u]);
            if (r + 2 * U < n) {
#pragma unroll
                for (int u = 0; u < U; ++u) a[u] = row_in(r + 2 * U + u);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) row_out(r + U + u, b[u]);
        }
    }
}

// Every access below is guarded by its step index; the host checks that a segment is a whole
// number of 1 KB steps, so the last step of the last row ends exactly at the tensor's end.
template <int DEPTH, bool DESCENDING, bool TWO_INPUTS>
__global__ void __launch_bounds__(256) row_stream_copy(const char *in0, const char *in1, char *out, int batch, int channels,
                                                       int row_bytes, int segs, int wave_per_batch_entry) {
    const unsigned wid = blockIdx.x * 4 + threadIdx.x / 64, lane = threadIdx.x % 64;
    const unsigned per_entry = (unsigned)(channels * segs);
    if (wid >= per_entry * (wave_per_batch_entry ? (unsigned)batch : 1u)) return;
    const unsigned c = (wid / segs) % channels, seg = wid % segs;
    const int seg_bytes = row_bytes / segs, steps = seg_bytes / 1024;
    const int b_lo = wave_per_batch_entry ? (int)(wid / per_entry) : 0, b_hi = wave_per_batch_entry ? b_lo + 1 : batch;
    for (int b = b_lo; b < b_hi; ++b) {
        const size_t row = ((size_t)b * channels + c) * row_bytes + (size_t)seg * seg_bytes + lane * 16;
        auto at = [&](int k) { return row + (size_t)(DESCENDING ? steps - 1 - k : k) * 1024; };
        u32x4 v0[DEPTH + 1], v1[DEPTH + 1];
#pragma unroll
        for (int q = 0; q < DEPTH + 1; ++q) { v0[q] = u32x4{0u, 0u, 0u, 0u}; v1[q] = u32x4{0u, 0u, 0u, 0u}; }
#pragma unroll
        for (int q = 0; q < DEPTH; ++q) {
            if (q < steps) {
                v0[q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(in0 + at(q)));
                if (TWO_INPUTS) v1[q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(in1 + at(q)));
            }
        }
        for (int k = 0; k < steps; k += DEPTH + 1) {
#pragma unroll
            for (int j = 0; j < DEPTH + 1; ++j) {
                const int slot = (j + DEPTH) % (DEPTH + 1);      // step k+j+DEPTH goes where step k+j-1 was
                if (k + j + DEPTH < steps) {
                    v0[slot] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(in0 + at(k + j + DEPTH)));
                    if (TWO_INPUTS) v1[slot] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(in1 + at(k + j + DEPTH)));
                }
                if (k + j < steps) __builtin_nontemporal_store(v0[j] ^ v1[j], reinterpret_cast<u32x4 *>(out + at(k + j)));
            }
        }
    }
}

// The channel-first shapes: the forward sweep's (two streams) and the backward configuration's (three).
static void row_stream_section(bool backward) {
    const int batch = 4, channels = backward ? 4096 : 2048, row_bytes = (backward ? 8192 : 4096) * 2;
    const size_t bytes = (size_t)batch * channels * row_bytes;
    const int sets = backward ? 2 : 6, reps = backward ? 10 : 30;
    const double streams = backward ? 3.0 : 2.0;
    std::vector<char *> in0(sets), in1(sets), out(sets);
    for (int s = 0; s < sets; ++s) {
        CK(hipMalloc(&in0[s], bytes));
        CK(hipMalloc(&in1[s], bytes));
        CK(hipMalloc(&out[s], bytes));
        CK(hipMemset(in0[s], 1, bytes));
        CK(hipMemset(in1[s], 2, bytes));
        CK(hipMemset(out[s], 0, bytes));
    }
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    printf("row-stream copies, (%d, %d, %d) 2-byte elements, %s: %d tensors of %.1f MB per launch, %d rotating sets\n", batch, channels,
           row_bytes / 2, backward ? "two inputs and one output" : "one input and one output", (int)streams, bytes / 1e6, sets);
    auto bench = [&](const std::string &name, auto launch) {
        std::vector<float> t;
        for (int round = 0; round < 5; ++round) {
            for (int i = 0; i < sets; ++i) launch(i);
            CK(hipDeviceSynchronize());
            CK(hipEventRecord(e0));
            for (int i = 0; i < reps; ++i) launch(i % sets);
            CK(hipEventRecord(e1));
            CK(hipEventSynchronize(e1));
            float ms;
            CK(hipEventElapsedTime(&ms, e0, e1));
            t.push_back(ms * 1e3f / reps);
        }
        std::sort(t.begin(), t.end());
        printf("%-62s median %7.2f us  min %7.2f  %.3f of 8 TB/s\n", name.c_str(), t[2], t[0], streams * bytes / t[2] * 1e-6 / 8.0);
        fflush(stdout);
    };
#define STREAM(DEPTH, DESC, TWO, SEGS, PER_ENTRY)                                                                     \
    {                                                                                                                 \
        if (row_bytes % (SEGS * 1024) != 0) { printf("segment is no whole number of steps\n"); exit(1); }            \
        const unsigned waves = (unsigned)(channels * SEGS) * (PER_ENTRY ? (unsigned)batch : 1u);                      \
        bench(std::string("rows in " #SEGS " part(s), " #DEPTH " step(s) ahead") +                                    \
                  (PER_ENTRY ? ", a wavefront per batch entry" : ", a wavefront walks the batch"),                    \
              [&](int s) {                                                                                            \
                  hipLaunchKernelGGL((row_stream_copy<DEPTH, DESC, TWO>), dim3((waves + 3) / 4), dim3(256), 0, 0, in0[s], \
                                     in1[s], out[s], batch, channels, row_bytes, SEGS, PER_ENTRY ? 1 : 0);           \
              });                                                                                                     \
    }
    if (backward) {
        STREAM(1, true, true, 1, false)
        STREAM(3, true, true, 1, false)
        STREAM(1, true, true, 2, false)
        STREAM(1, true, true, 4, false)
        STREAM(1, true, true, 16, false)
        STREAM(1, true, true, 1, true)
        STREAM(1, true, true, 4, true)
    } else {
        STREAM(1, false, false, 1, true)
        STREAM(3, false, false, 1, true)
        STREAM(1, false, false, 2, true)
        STREAM(3, false, false, 2, true)
        STREAM(1, false, false, 8, true)
    }
#undef STREAM
    for (int s = 0; s < sets; ++s) {
        CK(hipFree(in0[s]));
        CK(hipFree(in1[s]));
        CK(hipFree(out[s]));
    }
}

int main(int argc, char **argv) {
    const int rows = argc > 2 ? atoi(argv[1]) : 8 * 2048;
    const int row_bytes = argc > 2 ? atoi(argv[2]) : 5376 * 2;
    if (rows % 64 != 0 || row_bytes % 16 != 0) { printf("rows must be a multiple of 64, row_bytes of 16\n"); return 1; }
    const int sets = 6, reps = 30;
    const size_t bytes = (size_t)rows * row_bytes, n16 = bytes / 16;
    std::vector<char *> src(sets), dst(sets);
    for (int s = 0; s < sets; ++s) {
        CK(hipMalloc(&src[s], bytes));
        CK(hipMalloc(&dst[s], bytes));
        CK(hipMemset(src[s], s + 1, bytes));
        CK(hipMemset(dst[s], 0, bytes));
    }
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    auto bench = [&](const std::string &name, double moved, auto launch) {
        std::vector<float> t;
        for (int round = 0; round < 5; ++round) {
            for (int i = 0; i < sets; ++i) launch(i);
            CK(hipDeviceSynchronize());
            CK(hipEventRecord(e0));
            for (int i = 0; i < reps; ++i) launch(i % sets);
            CK(hipEventRecord(e1));
            CK(hipEventSynchronize(e1));
            float ms;
            CK(hipEventElapsedTime(&ms, e0, e1));
            t.push_back(ms * 1e3f / reps);
        }
        std::sort(t.begin(), t.end());
        printf("%-62s median %7.2f us  min %7.2f  %.3f of 8 TB/s\n", name.c_str(), t[2], t[0], moved / t[2] * 1e-6 / 8.0);
        fflush(stdout);
    };
    printf("tensor: %d rows x %d bytes = %.1f MB, read once and written once per launch; %d rotating pairs of buffers\n",
           rows, row_bytes, bytes / 1e6, sets);
    const dim3 lin((unsigned)((n16 + 255) / 256));
    auto S = [&](int s) { return reinterpret_cast<const u32x4 *>(src[s]); };
    auto D = [&](int s) { return reinterpret_cast<u32x4 *>(dst[s]); };
    bench("linear copy, plain loads and stores", 2.0 * bytes, [&](int s) { hipLaunchKernelGGL((linear_copy<false, false>), lin, dim3(256), 0, 0, S(s), D(s), n16); });
    bench("linear copy, non-temporal loads", 2.0 * bytes, [&](int s) { hipLaunchKernelGGL((linear_copy<true, false>), lin, dim3(256), 0, 0, S(s), D(s), n16); });
    bench("linear copy, non-temporal stores", 2.0 * bytes, [&](int s) { hipLaunchKernelGGL((linear_copy<false, true>), lin, dim3(256), 0, 0, S(s), D(s), n16); });
    bench("linear copy, non-temporal loads and stores", 2.0 * bytes, [&](int s) { hipLaunchKernelGGL((linear_copy<true, true>), lin, dim3(256), 0, 0, S(s), D(s), n16); });
    bench("linear read only (non-temporal)", 1.0 * bytes, [&](int s) { hipLaunchKernelGGL(linear_read, lin, dim3(256), 0, 0, S(s), D(s), n16); });
    bench("linear write only (non-temporal)", 1.0 * bytes, [&](int s) { hipLaunchKernelGGL(linear_write, lin, dim3(256), 0, 0, D(s), n16); });
    bench("hipMemcpyAsync device to device", 2.0 * bytes, [&](int s) { CK(hipMemcpyAsync(dst[s], src[s], bytes, hipMemcpyDeviceToDevice, 0)); });
#define WALK(LB, U, PING, T, CHUNK_RUNS)                                                                              \
    {                                                                                                                 \
        const int wpr = (row_bytes / LB + 63) / 64, runs = (rows + T - 1) / T;                                        \
        const unsigned total = (unsigned)(wpr * runs);                                                                \
        const unsigned blocks = ((total + 3) / 4 + 7) / 8 * 8;                                                        \
        const unsigned chunk = CHUNK_RUNS > 0 ? (unsigned)((CHUNK_RUNS * wpr + 3) / 4) : 0u;                          \
        bench(std::string("row walk, " #LB "-byte lanes, " #T "-row runs, " #U " rows per set") +                     \
                  (PING ? ", two sets" : ", one set") + (CHUNK_RUNS > 0 ? ", chunks of " #CHUNK_RUNS " runs" : ", hardware order"), \
              2.0 * bytes, [&](int s) {                                                                               \
                  hipLaunchKernelGGL((row_walk_copy<LB, U, PING>), dim3(blocks), dim3(256), 0, 0, src[s], dst[s], rows, \
                                     row_bytes, T, wpr, total, chunk);                                                \
              });                                                                                                     \
    }
    WALK(4, 8, true, 64, 4)
    WALK(4, 8, true, 32, 4)
    WALK(4, 8, true, 32, 0)
    WALK(4, 8, true, 16, 4)
    WALK(4, 8, true, 16, 0)
    WALK(4, 8, false, 8, 4)
    WALK(4, 4, true, 32, 4)
    WALK(4, 16, false, 32, 4)
    WALK(8, 8, true, 32, 4)
    WALK(8, 8, true, 16, 4)
    WALK(16, 8, true, 32, 4)
    WALK(16, 8, true, 16, 4)
    WALK(16, 1, false, 1, 0)
    for (int s = 0; s < sets; ++s) {
        CK(hipFree(src[s]));
        CK(hipFree(dst[s]));
    }
    row_stream_section(false);
    row_stream_section(true);
    return 0;
}
