// Verification instantiations of the grouped skinny kernel (see gemm_skinny_verify.hip).
#include "skinny_bodies.h"

namespace w2a8 {

hipError_t launch_skinny_grouped_verify(const GroupedParams& gp, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    return launch_skinny_grouped_impl<true>(gp, gs, asym, out_bf16, stream);
}

}  // namespace w2a8
