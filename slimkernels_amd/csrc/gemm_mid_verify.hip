// Verification instantiations of the kernel for 33..256 token rows: the same body with the int32 group sums written
// out as the matrix core left them.  One translation unit per group size (gemm_mid_verify_gs*.hip), so that the
// production object carries none of it and the three build side by side.
#include "w2a8_launch.h"

namespace w2a8 {

hipError_t launch_mid_verify_gs1(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream);
hipError_t launch_mid_verify_gs2(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream);
hipError_t launch_mid_verify_gs4(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream);

hipError_t launch_mid_verify(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    if (gs == 1) return launch_mid_verify_gs1(p, asym, out_bf16, stream);
    if (gs == 2) return launch_mid_verify_gs2(p, asym, out_bf16, stream);
    return launch_mid_verify_gs4(p, asym, out_bf16, stream);
}

}  // namespace w2a8
