// Verification instantiations of the one-problem skinny kernel for groups of 64 (1 step of 64 per group).
#include "skinny_bodies.h"

namespace w2a8 {

hipError_t launch_skinny_verify_gs1(const GemmParams& p, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    launch_nw<1, true>(p, waves, asym, out_bf16, stream);
    return hipGetLastError();
}

}  // namespace w2a8
