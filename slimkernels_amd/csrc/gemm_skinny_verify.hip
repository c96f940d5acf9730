// Verification instantiations of the skinny-M kernels: the production bodies (skinny_bodies.h) with the int32 dump
// switched on.  A verification launch takes the same instantiation choices as the production launch of the same
// problem; its outputs are bit-identical with the production launch's.  The one-problem kernel's instantiations are
// spread over three more translation units, one per group size (gemm_skinny_verify_gs*.hip), and the grouped kernel's
// sit in gemm_skinny_grouped_verify.hip, to build in parallel.
#include "skinny_bodies.h"

namespace w2a8 {

hipError_t launch_skinny_verify_gs1(const GemmParams& p, int waves, bool asym, bool out_bf16, hipStream_t stream);
hipError_t launch_skinny_verify_gs2(const GemmParams& p, int waves, bool asym, bool out_bf16, hipStream_t stream);
hipError_t launch_skinny_verify_gs4(const GemmParams& p, int waves, bool asym, bool out_bf16, hipStream_t stream);

hipError_t launch_skinny_verify(const GemmParams& p, int gs, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    if (gs == 1) return launch_skinny_verify_gs1(p, waves, asym, out_bf16, stream);
    if (gs == 2) return launch_skinny_verify_gs2(p, waves, asym, out_bf16, stream);
    return launch_skinny_verify_gs4(p, waves, asym, out_bf16, stream);
}

hipError_t launch_skinny_shared_verify(const GemmParams& p, int gs, int kparts, bool asym, bool out_bf16, hipStream_t stream) {
    return launch_skinny_shared_impl<true>(p, gs, kparts, asym, out_bf16, stream);
}

}  // namespace w2a8
