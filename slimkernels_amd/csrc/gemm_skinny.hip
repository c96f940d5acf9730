// Production instantiations of the skinny-M kernels (bodies and launch templates: skinny_bodies.h).
#include "skinny_bodies.h"

namespace w2a8 {

template <int J, int GS, int NW>
static void launch_fused_jgn(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream) {
    const dim3 grid(p.strips, p.split), block(NW * 64);
    if (asym) {
        if (out_bf16) skinny_fused_kernel<J, GS, NW, true, OutBF16><<<grid, block, 0, stream>>>(p);
        else skinny_fused_kernel<J, GS, NW, true, OutF16><<<grid, block, 0, stream>>>(p);
    } else {
        if (out_bf16) skinny_fused_kernel<J, GS, NW, false, OutBF16><<<grid, block, 0, stream>>>(p);
        else skinny_fused_kernel<J, GS, NW, false, OutF16><<<grid, block, 0, stream>>>(p);
    }
}

template <int GS>
static void launch_fused_gs(const GemmParams& p, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    if (p.M == 1) {
        if (waves >= 16) launch_fused_jgn<1, GS, 16>(p, asym, out_bf16, stream);
        else if (waves >= 8) launch_fused_jgn<1, GS, 8>(p, asym, out_bf16, stream);
        else launch_fused_jgn<1, GS, 4>(p, asym, out_bf16, stream);
    } else {
        if (waves >= 16) launch_fused_jgn<4, GS, 16>(p, asym, out_bf16, stream);
        else if (waves >= 8) launch_fused_jgn<4, GS, 8>(p, asym, out_bf16, stream);
        else launch_fused_jgn<4, GS, 4>(p, asym, out_bf16, stream);
    }
}

hipError_t launch_skinny_fused(const GemmParams& p, int gs, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    if (gs == 1) launch_fused_gs<1>(p, waves, asym, out_bf16, stream);
    else if (gs == 2) launch_fused_gs<2>(p, waves, asym, out_bf16, stream);
    else launch_fused_gs<4>(p, waves, asym, out_bf16, stream);
    return hipGetLastError();
}


hipError_t launch_skinny(const GemmParams& p, int gs, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    return launch_skinny_impl<false>(p, gs, waves, asym, out_bf16, stream);
}

hipError_t launch_skinny_shared(const GemmParams& p, int gs, int kparts, bool asym, bool out_bf16, hipStream_t stream) {
    return launch_skinny_shared_impl<false>(p, gs, kparts, asym, out_bf16, stream);
}

hipError_t launch_skinny_grouped(const GroupedParams& gp, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    return launch_skinny_grouped_impl<false>(gp, gs, asym, out_bf16, stream);
}

}  // namespace w2a8
