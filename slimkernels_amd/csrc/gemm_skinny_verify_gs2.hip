// Verification instantiations of the one-problem skinny kernel for groups of 128 (2 steps of 64 per group).
#include "skinny_bodies.h"

namespace w2a8 {

hipError_t launch_skinny_verify_gs2(const GemmParams& p, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    launch_nw<2, true>(p, waves, asym, out_bf16, stream);
    return hipGetLastError();
}

}  // namespace w2a8
