// Verification instantiations of the kernel for 33..128 token rows: the same body with the int32 group sums written
// out as the matrix core left them (a translation unit of their own, so that the production object carries none of it).
#include "mid_bodies.h"

namespace w2a8 {

hipError_t launch_mid_verify(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    return launch_mid_impl<true>(p, gs, asym, out_bf16, stream);
}

}  // namespace w2a8
