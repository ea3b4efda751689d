// Stand-ins for the kernel launchers, for a host-only build of the C-ABI front (cc1d_api.cpp)
// under AddressSanitizer / UndefinedBehaviorSanitizer: no GPU, no HIP runtime.  A launcher here
// records what it was asked to launch and answers CC1D_ERR_TOO_LARGE when the problem holds more
// than `g_capacity` batch entries, which is how the front's batch slicing is driven on the CPU.
#include <vector>

#include "cc1d_internal.hpp"
#include "stub_log.hpp"

std::vector<StubCall> g_calls;
int g_capacity = 1 << 30;

extern "C" hipError_t hipLaunchKernel(const void *, dim3, dim3, void **, size_t, hipStream_t) { return hipSuccess; }
extern "C" hipError_t hipGetLastError(void) { return hipSuccess; }

namespace cc1d {

static int record(const char *what, int batch, const void *x, const void *out, const void *aux, int flag) {
    if (batch > g_capacity) return CC1D_ERR_TOO_LARGE;
    if (probe_only()) return CC1D_OK;                 // the front asking whether a slice would fit: nothing runs
    g_calls.push_back({what, batch, x, out, aux, flag});
    return CC1D_OK;
}

int launch_fwd_channellast(const cc1d_fwd_params &p, const cc1d_varlen_params *gather, hipStream_t) {
    return record(gather ? "fwd_cl+gather" : "fwd_cl", p.batch, p.x, p.out, p.seq_idx, 0);
}
int launch_fwd_channelfirst(const cc1d_fwd_params &p, hipStream_t) {
    return record("fwd_cf", p.batch, p.x, p.out, p.final_states, 0);
}
size_t bwd_channellast_workspace_bytes(const cc1d_bwd_params &p) { return p.batch > g_capacity ? 0 : (size_t)p.batch * 64; }
size_t bwd_channelfirst_workspace_bytes(const cc1d_bwd_params &p) { return p.batch > g_capacity ? 0 : (size_t)p.batch * 32; }
bool bwd_channellast_fits(const cc1d_bwd_params &p) { return p.batch <= g_capacity; }
bool bwd_channelfirst_fits(const cc1d_bwd_params &p) { return p.batch <= g_capacity; }
int launch_bwd_channellast(const cc1d_bwd_params &p, void *ws, hipStream_t) {
    return record("bwd_cl", p.batch, p.x, p.dx, ws, p.overwrite_dweight);
}
int launch_bwd_channelfirst(const cc1d_bwd_params &p, void *ws, hipStream_t) {
    return record("bwd_cf", p.batch, p.x, p.dx, ws, p.overwrite_dweight);
}
int launch_bwd_finalize(const float *, int, const cc1d_bwd_params &p, hipStream_t) {
    return record("bwd_finalize", p.batch, p.x, p.dx, nullptr, p.overwrite_dweight);
}
int launch_update(const cc1d_update_params &p, hipStream_t) {
    return record("update", p.batch, p.x, p.conv_state, p.conv_state_indices, p.state_batch);
}
int launch_varlen_states(const cc1d_varlen_params &p, hipStream_t) {
    return record("varlen", p.batch, p.x, p.states, p.cu_seqlens, 0);
}

}  // namespace cc1d
