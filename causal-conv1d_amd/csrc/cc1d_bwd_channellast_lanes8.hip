// Channel-last backward on 16-bit data with 4 channels (8 bytes) per lane: the instantiations only.
#include "cc1d_bwd_channellast_kernel.hpp"

namespace cc1d {

int launch_bwd_channellast_16bit_lanes8(const cc1d_bwd_params &p, const BwdClGeom &g, float *ws, hipStream_t stream) {
    if (p.x_dtype == CC1D_F16) return launch_dtype<CC1D_F16, 4>(p, g, ws, stream);
    return launch_dtype<CC1D_BF16, 4>(p, g, ws, stream);
}

}  // namespace cc1d
