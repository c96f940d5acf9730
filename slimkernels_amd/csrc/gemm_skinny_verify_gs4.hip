// Verification instantiations of the one-problem skinny kernel for groups of 256 (4 steps of 64 per group).
#include "skinny_bodies.h"

namespace w2a8 {

hipError_t launch_skinny_verify_gs4(const GemmParams& p, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    launch_nw<4, true>(p, waves, asym, out_bf16, stream);
    return hipGetLastError();
}

}  // namespace w2a8
