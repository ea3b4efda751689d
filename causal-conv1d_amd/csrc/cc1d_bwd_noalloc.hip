// cc1d_bwd_noalloc: the backward for callers that cannot allocate device memory (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It is cc1d_bwd with
// the partial-sum workspace taken from a fixed array in this library's own device image instead
// of from the caller: same kernels, same order of additions, same bits.
//
// The array lives once per GPU, from the moment the code object is loaded there until the
// process ends.  Its device address is looked up once per device (hipGetSymbolAddress with that
// device current) and only that address is ever handed to a kernel: in host code the array's
// name is a host-side stand-in, not a device pointer.
//
// Every call on a GPU uses that GPU's one array: two such calls may not overlap in time (calls on
// one stream never do; calls on different streams of one GPU must be ordered by the caller).
// The kernels write every workspace plane they later read, so nothing has to be cleared and a
// call does not depend on what the previous one left behind.
#include <atomic>
#include <mutex>

#include "cc1d_internal.hpp"

namespace {

static __device__ __align__(256) unsigned char scratch[CC1D_BWD_NOALLOC_MAX_WORKSPACE_BYTES];

constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];
std::mutex g_lookup_mutex;

// Device address of `scratch` on the current device, looked up on the first call there.
int scratch_on_current_device(void **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return CC1D_ERR_LAUNCH;
    void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        std::lock_guard<std::mutex> lock(g_lookup_mutex);
        ptr = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (ptr == nullptr) {
            void *found = nullptr;
            if (hipGetSymbolAddress(&found, HIP_SYMBOL(scratch)) != hipSuccess || found == nullptr) {
                (void)hipGetLastError();
                return CC1D_ERR_LAUNCH;
            }
            g_scratch_ptr[dev].store(found, std::memory_order_release);
            ptr = found;
        }
    }
    *out = ptr;
    return CC1D_OK;
}

}  // namespace

extern "C" int cc1d_bwd_noalloc(const cc1d_bwd_params *p, cc1d_stream_t stream) {
    size_t need = 0;
    const int st = cc1d_bwd_workspace_bytes(p, &need);      // validates p; host only
    if (st != CC1D_OK) return st;
    if (need > (size_t)CC1D_BWD_NOALLOC_MAX_WORKSPACE_BYTES) return CC1D_ERR_WORKSPACE_LIMIT;
    void *ws = nullptr;
    if (need > 0) {
        const int found = scratch_on_current_device(&ws);
        if (found != CC1D_OK) return found;
    }
    return cc1d_bwd(p, ws, need, stream);
}
