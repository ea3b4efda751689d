// Host-only exercise of the C-ABI front (validation, batch slicing, status texts, tunables) and
// of the plain-C oracle, meant to run under AddressSanitizer and UndefinedBehaviorSanitizer.
#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "cc1d.h"
#include "stub_log.hpp"

extern "C" {
void cc1d_oracle_fwd(const float *x, const float *w, const float *bias, const int32_t *seq, const float *init,
                     int B, int D, int L, int W, int silu, double *out, double *final_states);
}

#define CHECK(cond) do { if (!(cond)) { std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); return 1; } } while (0)

static char arena[1 << 20];
static void *at(size_t off) { return arena + off; }

static cc1d_fwd_params fwd(int B, int D, int L, bool channel_last) {
    cc1d_fwd_params p;
    std::memset(&p, 0, sizeof p);
    p.batch = B; p.dim = D; p.seqlen = L; p.width = 4; p.x_dtype = CC1D_BF16; p.w_dtype = CC1D_F32; p.silu = 1;
    p.x = at(0); p.out = at(1 << 18); p.weight = at(1 << 19); p.bias = at((1 << 19) + 4096);
    if (channel_last) { p.x_stride_b = (int64_t)L * D; p.x_stride_c = 1; p.x_stride_l = D; }
    else { p.x_stride_b = (int64_t)D * L; p.x_stride_c = L; p.x_stride_l = 1; }
    p.out_stride_b = p.x_stride_b; p.out_stride_c = p.x_stride_c; p.out_stride_l = p.x_stride_l;
    p.w_stride_c = 4; p.w_stride_w = 1;
    return p;
}

static int test_fwd_slices() {
    for (int channel_last = 0; channel_last < 2; ++channel_last) {
        for (int cap : {1000, 7, 3, 1}) {
            g_calls.clear(); g_capacity = cap;
            cc1d_fwd_params p = fwd(13, 16, 24, channel_last);
            int32_t seq[13 * 24] = {0};
            if (channel_last) p.seq_idx = seq;
            CHECK(cc1d_fwd(&p, nullptr) == CC1D_OK);
            int covered = 0;
            for (const StubCall &c : g_calls) {                  // slices tile the batch in order, pointers advanced
                CHECK(c.batch <= cap && c.batch >= 1);
                CHECK(c.a == (const char *)p.x + (int64_t)covered * p.x_stride_b * 2);
                CHECK(c.b == (const char *)p.out + (int64_t)covered * p.out_stride_b * 2);
                if (channel_last) CHECK(c.c == seq + (int64_t)covered * 24);
                covered += c.batch;
            }
            CHECK(covered == 13);
            CHECK(cap >= 13 ? g_calls.size() == 1 : g_calls.size() > 1);
        }
    }
    g_capacity = 0;                                              // not even one batch entry fits
    g_calls.clear();
    cc1d_fwd_params p = fwd(4, 16, 24, false);
    CHECK(cc1d_fwd(&p, nullptr) == CC1D_ERR_TOO_LARGE && g_calls.empty());
    g_capacity = 1 << 30;
    return 0;
}

static int test_bwd_slices() {
    cc1d_bwd_params p;
    std::memset(&p, 0, sizeof p);
    p.batch = 9; p.dim = 16; p.seqlen = 24; p.width = 4; p.x_dtype = CC1D_F16; p.w_dtype = CC1D_F32; p.silu = 1;
    p.overwrite_dweight = 1;
    p.x = at(0); p.dout = at(1 << 16); p.dx = at(1 << 17); p.weight = at(1 << 19);
    p.dweight = (float *)at((1 << 19) + 8192);
    p.x_stride_b = 16 * 24; p.x_stride_c = 24; p.x_stride_l = 1;
    p.dout_stride_b = p.dx_stride_b = 16 * 24; p.dout_stride_c = p.dx_stride_c = 24; p.dout_stride_l = p.dx_stride_l = 1;
    p.w_stride_c = 4; p.w_stride_w = 1; p.dw_stride_c = 4; p.dw_stride_w = 1;
    for (int cap : {100, 4, 1}) {
        g_calls.clear(); g_capacity = cap;
        size_t need = 0;
        CHECK(cc1d_bwd_workspace_bytes(&p, &need) == CC1D_OK);
        const int largest = cap >= 9 ? 9 : cap == 4 ? 4 : 1;    // capacity 4: 9 -> 4 + 5 -> 4 + (2 + 3)
        CHECK(need == (size_t)largest * 32);
        alignas(16) static char ws[4096];
        CHECK(cc1d_bwd(&p, ws, need, nullptr) == CC1D_OK);
        int covered = 0;
        for (size_t i = 0; i < g_calls.size(); ++i) {
            CHECK(g_calls[i].batch <= cap);
            CHECK(g_calls[i].a == (const char *)p.x + (int64_t)covered * p.x_stride_b * 2);
            CHECK(g_calls[i].c == ws);                           // one workspace, shared by the slices
            CHECK(g_calls[i].flag == (i == 0 ? 1 : 0));          // only the first slice overwrites dweight
            covered += g_calls[i].batch;
        }
        CHECK(covered == 9);
        CHECK(cc1d_bwd(&p, ws, need ? need - 1 : 0, nullptr) == (need ? CC1D_ERR_WORKSPACE : CC1D_OK));
    }
    g_capacity = 1 << 30;
    return 0;
}

static int test_update_slices() {
    cc1d_update_params p;
    std::memset(&p, 0, sizeof p);
    p.batch = 10; p.dim = 8; p.seqlen = 1; p.width = 4; p.state_len = 3; p.state_batch = 10;
    p.x_dtype = CC1D_BF16; p.w_dtype = CC1D_F32;
    p.x = at(0); p.out = at(4096); p.conv_state = at(8192); p.weight = at(1 << 19);
    p.x_stride_b = 8; p.x_stride_c = 1; p.x_stride_l = 8;
    p.out_stride_b = 8; p.out_stride_c = 1; p.out_stride_l = 8;
    p.state_stride_b = 24; p.state_stride_c = 1; p.state_stride_l = 8;
    p.w_stride_c = 4; p.w_stride_w = 1;
    int32_t idx[10] = {3, 1, -1, 0, 9, 8, 7, 6, 5, 4};
    for (int with_idx = 0; with_idx < 2; ++with_idx) {
        p.conv_state_indices = with_idx ? idx : nullptr;
        p.state_batch = with_idx ? 12 : 10;
        g_calls.clear(); g_capacity = 3;
        CHECK(cc1d_update(&p, nullptr) == CC1D_OK);
        int covered = 0;
        for (const StubCall &c : g_calls) {
            CHECK(c.a == (const char *)p.x + (int64_t)covered * 8 * 2);
            if (with_idx) {                                      // the state table is not sliced, the index list is
                CHECK(c.b == p.conv_state && c.c == idx + covered && c.flag == 12);
            } else {
                CHECK(c.b == (const char *)p.conv_state + (int64_t)covered * 24 * 2 && c.flag == c.batch);
            }
            covered += c.batch;
        }
        CHECK(covered == 10 && g_calls.size() >= 4);
    }
    g_capacity = 1 << 30;
    return 0;
}

static int test_validation_and_texts() {
    CHECK(cc1d_validate_fwd(nullptr) == CC1D_ERR_NULL_POINTER);
    cc1d_fwd_params p = fwd(2, 16, 24, true);
    CHECK(cc1d_validate_fwd(&p) == CC1D_OK);
    p.width = 5; CHECK(cc1d_validate_fwd(&p) == CC1D_ERR_WIDTH); p.width = 4;
    p.dim = 12; CHECK(cc1d_validate_fwd(&p) == CC1D_ERR_CHANNEL_MULT8); p.dim = 16;
    // states: one buffer, two windows of one cache, two overlapping windows
    p.initial_states = at(2 << 18); p.final_states = at(2 << 18);
    p.init_stride_b = p.final_stride_b = 16 * 8; p.init_stride_c = p.final_stride_c = 1; p.init_stride_l = p.final_stride_l = 16;
    CHECK(cc1d_validate_fwd(&p) == CC1D_OK);
    p.final_states = (char *)at(2 << 18) + 3 * 16 * 2;
    CHECK(cc1d_validate_fwd(&p) == CC1D_OK);
    p.final_states = (char *)at(2 << 18) + 2 * 16 * 2;
    CHECK(cc1d_validate_fwd(&p) == CC1D_ERR_STATE_LAYOUT);
    for (int st = 0; st >= -25; --st) {
        const char *text = cc1d_strerror(st);
        CHECK(text != nullptr && std::strlen(text) > 0);
    }
    int32_t v = -1;
    CHECK(cc1d_set_tunable("fwd_cl_rows", 64) == CC1D_OK && cc1d_get_tunable("fwd_cl_rows", &v) == CC1D_OK && v == 64);
    CHECK(cc1d_set_tunable("fwd_cl_rows", 0) == CC1D_OK);
    CHECK(cc1d_set_tunable("nope", 1) == CC1D_ERR_UNKNOWN_TUNABLE && cc1d_set_tunable(nullptr, 1) == CC1D_ERR_NULL_POINTER);
    char small[4], path[4096];
    CHECK(cc1d_hip_runtime_path(nullptr, 0) == CC1D_ERR_NULL_POINTER);
    const int st = cc1d_hip_runtime_path(path, sizeof path);
    CHECK(st == CC1D_OK || st == CC1D_ERR_LAUNCH);
    if (st == CC1D_OK && std::strlen(path) >= sizeof small) CHECK(cc1d_hip_runtime_path(small, sizeof small) == CC1D_ERR_SHAPE);
    return 0;
}

static int test_oracle_c() {
    const int B = 2, D = 3, L = 9, W = 4;
    std::vector<float> x(B * D * L), w(D * W), bias(D), init(B * D * (W - 1));
    for (size_t i = 0; i < x.size(); ++i) x[i] = std::sin(0.7f * (float)i);
    for (size_t i = 0; i < w.size(); ++i) w[i] = 0.25f * std::cos(1.3f * (float)i);
    for (size_t i = 0; i < bias.size(); ++i) bias[i] = 0.1f * (float)i;
    for (size_t i = 0; i < init.size(); ++i) init[i] = 0.5f - 0.01f * (float)i;
    std::vector<int32_t> seq(B * L, 0);
    for (int t = 5; t < L; ++t) seq[t] = 1;
    seq[B * L - 1] = -1;
    std::vector<double> out(B * D * L), fin(B * D * (W - 1));
    cc1d_oracle_fwd(x.data(), w.data(), bias.data(), nullptr, init.data(), B, D, L, W, 1, out.data(), fin.data());
    for (double v : out) CHECK(std::isfinite(v));
    CHECK(fin[0] == (double)x[L - 3]);
    cc1d_oracle_fwd(x.data(), w.data(), bias.data(), seq.data(), nullptr, B, D, L, W, 1, out.data(), nullptr);
    CHECK(out[(size_t)(B * D - 1) * L + L - 1] == 0.0);          // padding position
    // first row of the second sub-sequence sees only its own tap
    const double z = (double)bias[0] + (double)w[3] * (double)x[5];
    CHECK(std::fabs(out[5] - z / (1.0 + std::exp(-z))) < 1e-12);
    return 0;
}

int main() {
    int rc = 0;
    rc |= test_fwd_slices();
    rc |= test_bwd_slices();
    rc |= test_update_slices();
    rc |= test_validation_and_texts();
    rc |= test_oracle_c();
    std::printf(rc == 0 ? "host sanitizer run ok\n" : "host sanitizer run FAILED\n");
    return rc;
}
