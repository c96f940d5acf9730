// The skinny kernel with the token rows quantised inside the launch by the grid's first workgroups (bodies in
// skinny_bodies.h): production instantiations for 16-row blocks; four, eight or sixteen waves per workgroup, as the same shape gets
// them with rows quantised beforehand (so that the two roads add up in the same order).
#include "skinny_bodies.h"

namespace w2a8 {

namespace {

template <int GS, int NW, bool ASYM, bool NT, bool WIDE>
void rows_out(const GemmParams& p, bool out_bf16, int spin_limit, hipStream_t stream) {
    const dim3 grid(p.strips, p.split, (p.M + 15) / 16), block(NW * 64);
    if (out_bf16) skinny_rows_kernel<GS, NW, ASYM, NT, WIDE, OutBF16><<<grid, block, 0, stream>>>(p, spin_limit);
    else skinny_rows_kernel<GS, NW, ASYM, NT, WIDE, OutF16><<<grid, block, 0, stream>>>(p, spin_limit);
}

// cache policy and activation fetch as launch_rows picks them for already quantised rows
template <int GS, int NW, bool ASYM>
void rows_shape(const GemmParams& p, bool out_bf16, int spin_limit, hipStream_t stream) {
    const bool wide = p.M >= kWideRows && p.K >= kWideK && p.strips * max(p.split, 1) * NW * ((p.M + 15) / 16) >= kWideWaves;
    const bool once = p.M <= 16;  // one row block: every weight byte is used once
    if (once && !wide) rows_out<GS, NW, ASYM, true, false>(p, out_bf16, spin_limit, stream);
    else if (once) rows_out<GS, NW, ASYM, true, true>(p, out_bf16, spin_limit, stream);
    else if (!wide) rows_out<GS, NW, ASYM, false, false>(p, out_bf16, spin_limit, stream);
    else rows_out<GS, NW, ASYM, false, true>(p, out_bf16, spin_limit, stream);
}

template <int GS>
void rows_gs(const GemmParams& p, int waves, bool asym, bool out_bf16, int spin_limit, hipStream_t stream) {
    if (waves >= 16) {
        if (asym) rows_shape<GS, 16, true>(p, out_bf16, spin_limit, stream);
        else rows_shape<GS, 16, false>(p, out_bf16, spin_limit, stream);
    } else if (waves >= 8) {
        if (asym) rows_shape<GS, 8, true>(p, out_bf16, spin_limit, stream);
        else rows_shape<GS, 8, false>(p, out_bf16, spin_limit, stream);
    } else {
        if (asym) rows_shape<GS, 4, true>(p, out_bf16, spin_limit, stream);
        else rows_shape<GS, 4, false>(p, out_bf16, spin_limit, stream);
    }
}

}  // namespace

hipError_t launch_skinny_rows(const GemmParams& p, int gs, int waves, bool asym, bool out_bf16, int spin_limit, hipStream_t stream) {
    if (gs == 1) rows_gs<1>(p, waves, asym, out_bf16, spin_limit, stream);
    else if (gs == 2) rows_gs<2>(p, waves, asym, out_bf16, spin_limit, stream);
    else rows_gs<4>(p, waves, asym, out_bf16, spin_limit, stream);
    return hipGetLastError();
}

}  // namespace w2a8
