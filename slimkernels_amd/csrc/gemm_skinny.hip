// Skinny-M (M <= 32) split-K W2A8 GEMM for gfx950: the HBM-bound decode regime.
//
// Grid (strips, split).  A workgroup of NW (4, 8 or 16) wavefronts owns one 64-channel strip
// and a contiguous range of scale groups; its waves take contiguous sub-ranges, so
// each wave streams a run of 1 KiB weight units (step-major layout) straight from global
// memory into VGPRs (one global_load_dwordx4 per lane and unit, no LDS staging:
// nothing in a unit is shared between waves).  The activation operand of a step is
// loaded once per wave and reused by the strip's four 16-channel sub-blocks.
//
// The kernel is a latency problem before it is a bandwidth problem (a whole decode
// GEMM is a few microseconds), so every load is issued as early as possible:
//  * weights and activations run through a register ring kDepth steps deep (the
//    load for step s + kDepth is issued when step s is consumed);
//  * the per-group metadata (scales, zero-points, activation row sums) of the next
//    16 steps is fetched into registers one chunk ahead and parked in a wave-private
//    LDS area, from which each group reads it with short ds_read latency;
//  * the token scales s_a needed by the epilogue are fetched at kernel entry.
// Per group the int32 accumulators are drained into fp32 running sums with the
// group's scale; the workgroup's waves' sums meet in LDS, and for split > 1 the
// workgroups' partial tiles meet in the workspace, summed in a fixed order by the
// last workgroup to arrive (deterministic, no float atomics).
#include "w2a8_launch.h"

namespace w2a8 {

// NW = wavefronts per workgroup (the split of K inside a workgroup).
// D = ring depth in steps = steps per metadata chunk = granule of the K partition (4 or 8).
template <int MB, int NW, int D>
struct SkinnySmem {
    union {
        struct {
            uint16_t scale[NW][D][16][4];  // [wave][group in chunk][col][sub-block]
            uint8_t zp[NW][D][16][4];
            int32_t rowsum[NW][D][MB * 16];
        } meta;
        float red[NW][MB * 16][kStripN + 1];
    };
    int last;
};

// J = live rows per lane of a D fragment: 4 in general, 1 when M == 1 (only row 0 of the 16x16
// block is a real token, so three quarters of the drain arithmetic can be dropped).
// ZM = zero-point mode: 0 uniform zero-point 2 (the symmetric levels; folded with shifts),
// 1 any other uniform zero-point, 2 per-(group, channel) zero-points read from zp_r.
template <int MB, int J, int GS, int NW, int ZM, bool DUMP, typename OutT, int kDepth>
__device__ __forceinline__ void skinny_body(const GemmParams& p, const int strip, const int split,
                                            SkinnySmem<MB, NW, kDepth>& sm) {
    constexpr bool ASYM = ZM == 2;
    constexpr bool SYM2 = ZM == 0;
    constexpr int kThreads = NW * 64;
    constexpr int kGroupsPerChunk = kDepth / GS;
    constexpr int kTile = MB * 16 * kStripN;  // elements of the workgroup's output tile
    constexpr int kOutPerThread = (kTile + kThreads - 1) / kThreads;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps ranges and bases in SGPRs
    const int col = lane & 15, quad = lane >> 4;

    // token scales for the epilogue (element e = tid + kThreads*i -> row e >> 6), fetched first
    float sa[kOutPerThread];
#pragma unroll
    for (int i = 0; i < kOutPerThread; ++i) sa[i] = p.s_a[min((tid + kThreads * i) >> 6, p.M - 1)];

    // Step range of this workgroup (groups_per_split is a multiple of a 4-step chunk's groups), then
    // of this wave, in whole chunks of kDepth steps; only a range's last chunk can be ragged.
    const int wg_s0 = min(split * p.groups_per_split, p.G) * GS;
    const int wg_s1 = min((split + 1) * p.groups_per_split, p.G) * GS;
    const int wg_chunks = (wg_s1 - wg_s0 + kDepth - 1) / kDepth;
    const int per_wave = (wg_chunks + NW - 1) / NW;
    const int s0 = min(wg_s0 + wave * per_wave * kDepth, wg_s1);
    const int s1 = min(s0 + per_wave * kDepth, wg_s1);
    const int g1 = s1 / GS;
    const int s_last = s1 - 1;

    // Addressing: wave-uniform 64-bit bases (SGPRs) plus 32-bit per-lane offsets.  No load is
    // predicated or sits under a branch: out-of-range rows, groups and steps are clamped onto valid
    // addresses instead, so the number of loads in flight is the same on every path and the
    // s_waitcnt the compiler places before each use waits for exactly that load (a token row >= M
    // only ever feeds output rows >= M, which are not stored; a clamped step or group is never used).
    const char* wb = reinterpret_cast<const char*>(p.w_r) + (size_t)strip * (kUnitDwords * 4);
    const size_t wstride = (size_t)p.strips * (kUnitDwords * 4);  // bytes between consecutive steps of a strip
    const uint32_t wlane = lane * 16;
    const char* qb = reinterpret_cast<const char*>(p.q);
    uint32_t aoff[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) aoff[mb] = (uint32_t)min(mb * 16 + col, p.M - 1) * (uint32_t)p.ldq + quad * 16;

    // ---- metadata prefetch registers: one chunk (kGroupsPerChunk groups) ahead
    v4i m_scale;     // scales: 4 groups x 128 B = 512 B per wave: lanes 0..31, 16 B each
    v4i m_zp;        // zero-points: 4 groups x 64 B: lanes 0..15
    v4i m_rs[MB];    // row sums: lane -> (group lane >> 2, rows 4*(lane & 3) ..): lanes 0..15
    auto fetch_meta = [&](int gfirst) {  // groups gfirst .. gfirst + kGroupsPerChunk - 1, clamped to g1 - 1
        const size_t sgi = (size_t)min(gfirst + (lane >> 3), g1 - 1) * p.strips + strip;
        m_scale = *reinterpret_cast<const v4i*>(reinterpret_cast<const char*>(p.s_r) + sgi * 128 + (lane & 7) * 16);
        const int gq = min(gfirst + (lane >> 2), g1 - 1);
        if (ASYM)
            m_zp = *reinterpret_cast<const v4i*>(reinterpret_cast<const char*>(p.zp_r) +
                                                 ((size_t)gq * p.strips + strip) * 64 + (lane & 3) * 16);
        const int32_t* rp = p.rowsum + (size_t)gq * p.ldr;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            m_rs[mb] = *reinterpret_cast<const v4i*>(rp + min(mb * 16 + (lane & 3) * 4, p.ldr - 4));
    };
    auto park_meta = [&]() {
        if (lane < kDepth * 8)
            *reinterpret_cast<v4i*>(reinterpret_cast<char*>(&sm.meta.scale[wave][0][0][0]) + lane * 16) = m_scale;
        if (lane < kDepth * 4) {
            if (ASYM) *reinterpret_cast<v4i*>(reinterpret_cast<char*>(&sm.meta.zp[wave][0][0][0]) + lane * 16) = m_zp;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                *reinterpret_cast<v4i*>(&sm.meta.rowsum[wave][lane >> 2][mb * 16 + (lane & 3) * 4]) = m_rs[mb];
        }
    };

    // ---- weight / activation register ring
    v4i wring[kDepth];
    v4i aring[kDepth][MB];
    auto issue = [&](int slot, int step) {  // step is wave-uniform
        wring[slot] = *reinterpret_cast<const v4i*>(wb + (size_t)step * wstride + wlane);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            aring[slot][mb] = *reinterpret_cast<const v4i*>(qb + (size_t)step * kStepK + aoff[mb]);
    };

    float t[MB][4][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int pp = 0; pp < 4; ++pp)
#pragma unroll
            for (int j = 0; j < 4; ++j) t[mb][pp][j] = 0.0f;

    if (s0 < s1) {
        // Same issue order as inside the loop (metadata first, then the ring), fenced, so that the
        // wait counts the compiler derives for the loop head hold on the entry path as well.
        fetch_meta(s0 / GS);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < kDepth; ++i) issue(i, min(s0 + i, s_last));
        __builtin_amdgcn_sched_barrier(0);

        v4i acc[MB][4];
        v4i nrs[MB];
        int zps[4];
        float sc[4];

        for (int cbase = s0; cbase < s1; cbase += kDepth) {
            const int gchunk = cbase / GS;
            park_meta();                              // this chunk's metadata: registers -> LDS
            fetch_meta(gchunk + kGroupsPerChunk);     // next chunk's metadata: global -> registers
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < kDepth; ++i) {
                const int step = cbase + i;
                const int gi = i / GS;  // group within the chunk
                if (i % GS == 0) {
                    // a group past the end of K (ragged last chunk) is neutralised by a zero scale
                    const float live = (gchunk + gi < g1) ? 1.0f : 0.0f;
                    const uint2 sraw = *reinterpret_cast<const uint2*>(&sm.meta.scale[wave][gi][col][0]);
                    sc[0] = half_bits_to_float((uint16_t)(sraw.x & 0xffffu)) * live;
                    sc[1] = half_bits_to_float((uint16_t)(sraw.x >> 16)) * (0.25f * live);
                    sc[2] = half_bits_to_float((uint16_t)(sraw.y & 0xffffu)) * (0.0625f * live);
                    sc[3] = half_bits_to_float((uint16_t)(sraw.y >> 16)) * (0.015625f * live);
                    // effective zero-points in operand units: zp * 4^p, (zp - 2) * 64 for the sign-bit field
                    if (ASYM) {
                        const uint32_t zraw = *reinterpret_cast<const uint32_t*>(&sm.meta.zp[wave][gi][col][0]);
                        zps[0] = (int)(zraw & 0xffu);
                        zps[1] = (int)((zraw >> 8) & 0xffu) * 4;
                        zps[2] = (int)((zraw >> 16) & 0xffu) * 16;
                        zps[3] = ((int)(zraw >> 24) - 2) * 64;
                    } else {
                        zps[0] = p.zp_const;
                        zps[1] = p.zp_const * 4;
                        zps[2] = p.zp_const * 16;
                        zps[3] = (p.zp_const - 2) * 64;
                    }
                    // -rowsum of the lane's D rows: the zero-point term -zp * rowsum is folded in at the drain
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        nrs[mb] = -*reinterpret_cast<const v4i*>(&sm.meta.rowsum[wave][gi][mb * 16 + quad * 4]);
                }

#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    const v4i b = wring[i] & (int)(0x03030303u << (2 * pp));
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)  // the first step of a group starts from C = 0 (inline constant)
                        acc[mb][pp] = mfma_i8_16x16x64(aring[i][mb], b, (i % GS == 0) ? v4i{0, 0, 0, 0} : acc[mb][pp]);
                }
                // Refill the slot only now that its old contents are dead, so the load can land in the
                // same registers (no copies at the loop back-edge, and the wait before the next use is
                // for exactly this load).  The fences stop the scheduler from sinking the four steps'
                // loads to the end of the chunk, which would serialise load and compute.
                __builtin_amdgcn_sched_barrier(0);
                issue(i, min(step + kDepth, s_last));
                __builtin_amdgcn_sched_barrier(0);

                if (i % GS == GS - 1) {
                    const int g = gchunk + gi;
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                            for (int j = 0; j < J; ++j) {
                                // true group sum (x 4^p) = raw - zp_eff * rowsum
                                if (SYM2) {  // zero-point 2 everywhere: 2 * 4^p = 1 << (2p + 1); field 3 needs nothing
                                    if (pp < 3) acc[mb][pp][j] += nrs[mb][j] << (2 * pp + 1);
                                } else {
                                    acc[mb][pp][j] += __mul24(nrs[mb][j], zps[pp]);
                                }
                                t[mb][pp][j] = __builtin_fmaf((float)acc[mb][pp][j], sc[pp], t[mb][pp][j]);
                                if (DUMP) {
                                    const int m = mb * 16 + quad * 4 + j;
                                    const int n = strip * kStripN + pp * 16 + col;
                                    if (g < g1 && m < p.M && n < p.N) {
                                        const int v = acc[mb][pp][j] >> (2 * pp);  // exact: a multiple of 4^p
                                        if (p.dump_mode == 1)
                                            p.acc_dump[((size_t)m * p.N + n) * p.G + g] = v;
                                        else
                                            atomicAdd(p.acc_dump + (size_t)m * p.N + n, v);
                                    }
                                }
                            }
                }
            }
        }
    }

    // ---- meet the workgroup's waves in LDS (the metadata area is dead once every wave is here)
    __syncthreads();

#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int pp = 0; pp < 4; ++pp)
#pragma unroll
            for (int j = 0; j < 4; ++j) sm.red[wave][mb * 16 + quad * 4 + j][pp * 16 + col] = t[mb][pp][j];
    __syncthreads();

    uint16_t* out = reinterpret_cast<uint16_t*>(p.out);
    if (p.split == 1) {
#pragma unroll
        for (int i = 0; i < kOutPerThread; ++i) {
            const int e = tid + kThreads * i;
            const int m = e >> 6, nl = e & 63;
            const int n = strip * kStripN + nl;
            if (e < kTile && m < p.M && n < p.N) {
                float v = sm.red[0][m][nl];
#pragma unroll
                for (int w = 1; w < NW; ++w) v += sm.red[w][m][nl];
                out[(size_t)m * p.ldo + n] = OutT::cast(v * sa[i]);
            }
        }
        return;
    }

    // ---- split-K: publish this workgroup's partial tile, last arrival reduces all of them.
    // The partials are written and read with agent-scope relaxed atomics (write-through stores,
    // cache-bypassing loads on gfx950), so no L2 write-back / invalidate fence is needed: a fence
    // here costs about a microsecond per workgroup and serialises on each XCD's L2.
    // s_waitcnt vmcnt(0) makes every lane's stores complete before the arrival counter moves.
    float* mine = p.ws_partial + ((size_t)split * p.strips + strip) * kTile;
#pragma unroll
    for (int i = 0; i < kOutPerThread; ++i) {
        const int e = tid + kThreads * i;
        if (e < kTile) {
            const int m = e >> 6, nl = e & 63;
            float v = sm.red[0][m][nl];
#pragma unroll
            for (int w = 1; w < NW; ++w) v += sm.red[w][m][nl];
            __hip_atomic_store(mine + e, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned prev = __hip_atomic_fetch_add(p.ws_counter + strip, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sm.last = (prev == (unsigned)(p.split - 1));
    }
    __syncthreads();
    if (!sm.last) return;
#pragma unroll
    for (int i = 0; i < kOutPerThread; ++i) {
        const int e = tid + kThreads * i;
        if (e >= kTile) break;
        const int m = e >> 6, nl = e & 63;
        const int n = strip * kStripN + nl;
        float v = 0.0f;
        for (int sp = 0; sp < p.split; ++sp)
            v += __hip_atomic_load(p.ws_partial + ((size_t)sp * p.strips + strip) * kTile + e, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        if (m < p.M && n < p.N) out[(size_t)m * p.ldo + n] = OutT::cast(v * sa[i]);
    }
    if (tid == 0) __hip_atomic_store(p.ws_counter + strip, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int MB, int J, int GS, int NW, int ZM, bool DUMP, typename OutT>
__global__ __launch_bounds__(NW * 64) void skinny_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) SkinnySmem<MB, NW, 4> sm;
    skinny_body<MB, J, GS, NW, ZM, DUMP, OutT, 4>(p, blockIdx.x, blockIdx.y, sm);
}

// Several independent skinny GEMMs in one launch: workgroup ids are cut into runs, one run per
// problem (one workgroup per strip, no split-K: together the problems fill the chip), and each
// workgroup runs the single-problem body on its problem.  All problems share the group size,
// the zero-point mode and the output type; M may differ (the three row-count variants live side
// by side in the kernel).  The problem table travels in the kernel arguments.
#ifndef SLIMK_GROUPED_WAVES_PER_SIMD
#define SLIMK_GROUPED_WAVES_PER_SIMD 2
#endif
template <int GS, int ZM, typename OutT>
__global__ __launch_bounds__(256, SLIMK_GROUPED_WAVES_PER_SIMD) void skinny_grouped_kernel(const GroupedParams gp) {
    __shared__ __attribute__((aligned(16))) union {
        SkinnySmem<1, 4, 4> one;
        SkinnySmem<2, 4, 4> two;
    } sm;
    const int wg = blockIdx.x;
    int i = 0;
    while (i + 1 < gp.count && wg >= gp.wg_begin[i + 1]) ++i;
    const GemmParams& p = gp.prob[i];
    const int strip = wg - gp.wg_begin[i];
    if (p.M == 1) skinny_body<1, 1, GS, 4, ZM, false, OutT, 4>(p, strip, 0, sm.one);
    else if (p.M <= 16) skinny_body<1, 4, GS, 4, ZM, false, OutT, 4>(p, strip, 0, sm.one);
    else skinny_body<2, 4, GS, 4, ZM, false, OutT, 4>(p, strip, 0, sm.two);
}

template <int MB, int J, int GS, int NW, int ZM, bool DUMP>
static void launch_out(const GemmParams& p, bool out_bf16, hipStream_t stream) {
    const dim3 grid(p.strips, p.split), block(NW * 64);
    if (out_bf16)
        skinny_kernel<MB, J, GS, NW, ZM, DUMP, OutBF16><<<grid, block, 0, stream>>>(p);
    else
        skinny_kernel<MB, J, GS, NW, ZM, DUMP, OutF16><<<grid, block, 0, stream>>>(p);
}

template <int MB, int J, int GS, int NW, bool DUMP>
static void launch_zm(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream) {
    if (asym) launch_out<MB, J, GS, NW, 2, DUMP>(p, out_bf16, stream);
    else if (p.zp_const == 2) launch_out<MB, J, GS, NW, 0, DUMP>(p, out_bf16, stream);
    else launch_out<MB, J, GS, NW, 1, DUMP>(p, out_bf16, stream);
}

template <int MB, int GS, int NW>
static void launch_flags(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream) {
    const bool dump = p.acc_dump != nullptr && p.dump_mode != 0;
    if (dump) launch_zm<MB, 4, GS, 4, true>(p, asym, out_bf16, stream);  // verification: 4 waves, all rows
    else if (MB == 1 && p.M == 1) launch_zm<MB, (MB == 1 ? 1 : 4), GS, NW, false>(p, asym, out_bf16, stream);
    else launch_zm<MB, 4, GS, NW, false>(p, asym, out_bf16, stream);
}

template <int MB, int GS>
static void launch_nw(const GemmParams& p, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    if (MB == 1) {
        if (waves >= 16) launch_flags<MB, GS, (MB == 1 ? 16 : 8)>(p, asym, out_bf16, stream);
        else launch_flags<MB, GS, 4>(p, asym, out_bf16, stream);
    } else {
        if (waves >= 8) launch_flags<MB, GS, 8>(p, asym, out_bf16, stream);
        else launch_flags<MB, GS, 4>(p, asym, out_bf16, stream);
    }
}

template <int MB>
static void launch_gs(const GemmParams& p, int gs, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    if (gs == 1) launch_nw<MB, 1>(p, waves, asym, out_bf16, stream);
    else if (gs == 2) launch_nw<MB, 2>(p, waves, asym, out_bf16, stream);
    else launch_nw<MB, 4>(p, waves, asym, out_bf16, stream);
}

template <int GS, int ZM>
static void launch_grouped_out(const GroupedParams& gp, int total_wgs, bool out_bf16, hipStream_t stream) {
    if (out_bf16) skinny_grouped_kernel<GS, ZM, OutBF16><<<dim3(total_wgs), dim3(256), 0, stream>>>(gp);
    else skinny_grouped_kernel<GS, ZM, OutF16><<<dim3(total_wgs), dim3(256), 0, stream>>>(gp);
}

template <int GS>
static void launch_grouped_zm(const GroupedParams& gp, int total_wgs, int zm, bool out_bf16, hipStream_t stream) {
    if (zm == 0) launch_grouped_out<GS, 0>(gp, total_wgs, out_bf16, stream);
    else if (zm == 1) launch_grouped_out<GS, 1>(gp, total_wgs, out_bf16, stream);
    else launch_grouped_out<GS, 2>(gp, total_wgs, out_bf16, stream);
}

hipError_t launch_skinny_grouped(const GroupedParams& gp, int gs, int zm, bool out_bf16, hipStream_t stream) {
    const int total_wgs = gp.wg_begin[gp.count];
    if (gs == 1) launch_grouped_zm<1>(gp, total_wgs, zm, out_bf16, stream);
    else if (gs == 2) launch_grouped_zm<2>(gp, total_wgs, zm, out_bf16, stream);
    else launch_grouped_zm<4>(gp, total_wgs, zm, out_bf16, stream);
    return hipGetLastError();
}

hipError_t launch_skinny(const GemmParams& p, int gs, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    if (p.M <= 16) launch_gs<1>(p, gs, waves, asym, out_bf16, stream);
    else launch_gs<2>(p, gs, waves, asym, out_bf16, stream);
    return hipGetLastError();
}

}  // namespace w2a8
