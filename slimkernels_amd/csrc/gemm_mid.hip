// Production instantiations of the kernel for 33..128 token rows (mid_bodies.h): one workgroup takes a strip of 64
// channels with every token row.
#include "mid_bodies.h"

namespace w2a8 {

hipError_t launch_mid(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    return launch_mid_impl<false>(p, gs, asym, out_bf16, stream);
}

}  // namespace w2a8
