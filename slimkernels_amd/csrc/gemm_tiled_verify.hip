// Verification instantiations of the fast tiled kernels: the same bodies with the int32 group sums written out as the
// matrix core left them (a translation unit of their own, so that the production objects carry none of it).
#include "tiled_bodies.h"

namespace w2a8 {

hipError_t launch_tiled_verify(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    return launch_tiled_impl<true>(p, gs, asym, out_bf16, stream);
}

hipError_t launch_tiled_w4_verify(const GemmParams& p, int gs, bool out_bf16, hipStream_t stream) {
    return launch_tiled_w4_impl<true>(p, gs, out_bf16, stream);
}

}  // namespace w2a8
