// Verification instantiations of the kernel for 33..256 token rows, groups of 64 (see gemm_mid_verify.hip).
#include "mid_bodies.h"

namespace w2a8 {

hipError_t launch_mid_verify_gs1(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream) {
    return launch_mid_verify_one<1>(p, asym, out_bf16, stream);
}

}  // namespace w2a8
