// Skinny-M (M <= 32) split-K W2A8 GEMM for gfx950: the HBM-bound decode regime.
//
// Grid (strips, split).  A workgroup of four wavefronts owns one 64-channel strip
// and a contiguous range of scale groups; its waves take contiguous sub-ranges, so
// each wave streams one contiguous run of 1 KiB weight units straight from global
// memory into VGPRs (one global_load_dwordx4 per lane and unit, no LDS staging:
// nothing in a unit is shared between waves).  The activation operand of a step is
// loaded once per wave and reused by the strip's four 16-channel sub-blocks.
// Per group the int32 accumulators are drained into fp32 running sums with the
// group's scale; the four waves' sums meet in LDS, and for split > 1 the
// workgroups' partial tiles meet in the workspace, summed in a fixed order by the
// last workgroup to arrive (deterministic, no float atomics).
#include "w2a8_launch.h"

namespace w2a8 {

template <int MB, int GS, bool ASYM, bool DUMP, typename OutT>
__global__ __launch_bounds__(256) void skinny_kernel(const GemmParams p) {
    __shared__ float red[4][MB * 16][kStripN + 1];
    __shared__ int s_last;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int strip = blockIdx.x;
    const int split = blockIdx.y;

    // contiguous group range of this workgroup, then of this wave
    const int wg_g0 = min(split * p.groups_per_split, p.G);
    const int wg_g1 = min(wg_g0 + p.groups_per_split, p.G);
    const int per_wave = (wg_g1 - wg_g0 + 3) >> 2;
    const int g0 = min(wg_g0 + wave * per_wave, wg_g1);
    const int g1 = min(g0 + per_wave, wg_g1);

    float t[MB][4][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int pp = 0; pp < 4; ++pp)
#pragma unroll
            for (int j = 0; j < 4; ++j) t[mb][pp][j] = 0.0f;

    const uint32_t* wbase = p.w_r + (size_t)strip * p.steps * kUnitDwords + lane * 4;
    const size_t sg_base = (size_t)strip * p.G;

    // activation operand rows of this lane (row = mb*16 + col), clamped pointer + validity
    const int8_t* arow[MB];
    bool avalid[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = mb * 16 + col;
        avalid[mb] = m < p.M;
        arow[mb] = p.q + (size_t)(avalid[mb] ? m : 0) * p.ldq + quad * 16;
    }

    for (int g = g0; g < g1; ++g) {
        // scales of the lane's four sub-block columns, with the 4^-p operand scaling folded in
        const uint2 sraw = *reinterpret_cast<const uint2*>(p.s_r + ((sg_base + g) * 16 + col) * 4);
        float sc[4];
        sc[0] = half_bits_to_float((uint16_t)(sraw.x & 0xffffu));
        sc[1] = half_bits_to_float((uint16_t)(sraw.x >> 16)) * 0.25f;
        sc[2] = half_bits_to_float((uint16_t)(sraw.y & 0xffffu)) * 0.0625f;
        sc[3] = half_bits_to_float((uint16_t)(sraw.y >> 16)) * 0.015625f;
        // effective zero-points in operand units: zp * 4^p, and (zp - 2) * 64 for the sign-bit field
        int zpe[4];
        if (ASYM) {
            const uint32_t zraw = *reinterpret_cast<const uint32_t*>(p.zp_r + ((sg_base + g) * 16 + col) * 4);
            zpe[0] = (int)(zraw & 0xffu);
            zpe[1] = (int)((zraw >> 8) & 0xffu) * 4;
            zpe[2] = (int)((zraw >> 16) & 0xffu) * 16;
            zpe[3] = ((int)(zraw >> 24) - 2) * 64;
        } else {
            zpe[0] = p.zp_const;
            zpe[1] = p.zp_const * 4;
            zpe[2] = p.zp_const * 16;
            zpe[3] = (p.zp_const - 2) * 64;
        }

        // accumulators start at -zp * rowsum so that they end as the true group sums (x 4^p)
        v4i acc[MB][4];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int m0 = mb * 16 + quad * 4;  // D rows of this lane: m0 .. m0+3
            v4i rs = {0, 0, 0, 0};
            if (m0 < p.M) rs = *reinterpret_cast<const v4i*>(p.rowsum + (size_t)g * p.ldr + m0);
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) acc[mb][pp] = rs * (-zpe[pp]);
        }

#pragma unroll
        for (int s = 0; s < GS; ++s) {
            const int step = g * GS + s;
            const v4i w = *reinterpret_cast<const v4i*>(wbase + (size_t)step * kUnitDwords);
            v4i a[MB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                a[mb] = v4i{0, 0, 0, 0};
                if (avalid[mb]) a[mb] = *reinterpret_cast<const v4i*>(arow[mb] + (size_t)step * kStepK);
            }
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                const v4i b = w & (int)(0x03030303u << (2 * pp));
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) acc[mb][pp] = mfma_i8_16x16x64(a[mb], b, acc[mb][pp]);
            }
        }

#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    t[mb][pp][j] = __builtin_fmaf((float)acc[mb][pp][j], sc[pp], t[mb][pp][j]);
                    if (DUMP) {
                        const int m = mb * 16 + quad * 4 + j;
                        const int n = strip * kStripN + pp * 16 + col;
                        if (m < p.M && n < p.N) {
                            const int v = acc[mb][pp][j] >> (2 * pp);  // exact: a multiple of 4^p
                            if (p.dump_mode == 1)
                                p.acc_dump[((size_t)m * p.N + n) * p.G + g] = v;
                            else
                                atomicAdd(p.acc_dump + (size_t)m * p.N + n, v);
                        }
                    }
                }
    }

    // ---- meet the four waves in LDS
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int pp = 0; pp < 4; ++pp)
#pragma unroll
            for (int j = 0; j < 4; ++j) red[wave][mb * 16 + quad * 4 + j][pp * 16 + col] = t[mb][pp][j];
    __syncthreads();

    constexpr int kTile = MB * 16 * kStripN;  // elements of the workgroup's output tile
    uint16_t* out = reinterpret_cast<uint16_t*>(p.out);
    if (p.split == 1) {
        for (int e = tid; e < kTile; e += 256) {
            const int m = e >> 6, nl = e & 63;
            const int n = strip * kStripN + nl;
            if (m < p.M && n < p.N) {
                const float v = ((red[0][m][nl] + red[1][m][nl]) + red[2][m][nl]) + red[3][m][nl];
                out[(size_t)m * p.ldo + n] = OutT::cast(v * p.s_a[m]);
            }
        }
        return;
    }

    // ---- split-K: publish this workgroup's partial tile, last arrival reduces all of them
    float* mine = p.ws_partial + ((size_t)split * p.strips + strip) * kTile;
    for (int e = tid; e < kTile; e += 256) {
        const int m = e >> 6, nl = e & 63;
        mine[e] = ((red[0][m][nl] + red[1][m][nl]) + red[2][m][nl]) + red[3][m][nl];
    }
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const unsigned prev = atomicAdd(p.ws_counter + strip, 1u);
        s_last = (prev == (unsigned)(p.split - 1));
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    for (int e = tid; e < kTile; e += 256) {
        const int m = e >> 6, nl = e & 63;
        const int n = strip * kStripN + nl;
        float v = 0.0f;
        for (int sp = 0; sp < p.split; ++sp)
            v += __builtin_nontemporal_load(p.ws_partial + ((size_t)sp * p.strips + strip) * kTile + e);
        if (m < p.M && n < p.N) out[(size_t)m * p.ldo + n] = OutT::cast(v * p.s_a[m]);
    }
    if (tid == 0) p.ws_counter[strip] = 0u;  // leave the workspace ready for the next call
}

template <int MB, int GS, bool ASYM, bool DUMP>
static void launch_out(const GemmParams& p, bool out_bf16, hipStream_t stream) {
    const dim3 grid(p.strips, p.split), block(256);
    if (out_bf16)
        skinny_kernel<MB, GS, ASYM, DUMP, OutBF16><<<grid, block, 0, stream>>>(p);
    else
        skinny_kernel<MB, GS, ASYM, DUMP, OutF16><<<grid, block, 0, stream>>>(p);
}

template <int MB, int GS>
static void launch_flags(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream) {
    const bool dump = p.acc_dump != nullptr && p.dump_mode != 0;
    if (asym) {
        if (dump) launch_out<MB, GS, true, true>(p, out_bf16, stream);
        else launch_out<MB, GS, true, false>(p, out_bf16, stream);
    } else {
        if (dump) launch_out<MB, GS, false, true>(p, out_bf16, stream);
        else launch_out<MB, GS, false, false>(p, out_bf16, stream);
    }
}

template <int MB>
static void launch_gs(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    if (gs == 1) launch_flags<MB, 1>(p, asym, out_bf16, stream);
    else if (gs == 2) launch_flags<MB, 2>(p, asym, out_bf16, stream);
    else launch_flags<MB, 4>(p, asym, out_bf16, stream);
}

hipError_t launch_skinny(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    if (p.M <= 16) launch_gs<1>(p, gs, asym, out_bf16, stream);
    else launch_gs<2>(p, gs, asym, out_bf16, stream);
    return hipGetLastError();
}

}  // namespace w2a8
