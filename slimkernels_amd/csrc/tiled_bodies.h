// Bodies, kernels and launch templates of the fast tiled W2A8 GEMM for gfx950 (included by gemm_tiled.hip, which
// instantiates the production kernels, and by gemm_tiled_verify.hip, which instantiates the verification ones): the int8-MFMA-bound prefill regime; group size 64, 128 or 256, any K the group
// size divides (a group of 256 spans two stages and keeps its int32 sums in registers between them, 64-row tiles
// only; an odd number of 64-element steps ends in a half-empty stage whose second step reads as zero).
//
// Workgroup = 4 wavefronts side by side along the channels; workgroup tile 128 (or 64) tokens x 256
// channels (four weight strips); wave tile 128 x 64 = 8 x 4 blocks of v_mfma_i32_16x16x64_i8.
// A wide-in-N tile is the cheap one here: per reduction element a tile fetches BM bytes of
// activations but only BN/4 bytes of 2-bit weights.
//
// What bounds the kernel is the vector ALU next to the matrix core, not the matrix core: every
// accumulator must be drained into an fp32 running sum once per scale group (v_cvt_f32_i32 +
// v_fma_f32 per element per group -- at group 128 that is as many VALU cycles as MFMA cycles).
// Measured on one CU: a SIMD spends max(16, 8 + 4 V) cycles per v_mfma_i32_16x16x64_i8 that has V
// vector instructions beside it (the MFMA holds the issue port for 8 cycles, a vector instruction
// for 4); the main loop below has V = 5.3, so 0.55 of the matrix core is its ceiling.
// Everything else is arranged to add as little VALU work as possible:
//  * the high bit of every 2-bit field is flipped (one v_xor per dword) and the field moved to
//    the top of its byte (v_lshlrev + v_and), so each operand byte reads as 64 * (code - 2):
//    the zero-point is gone before the MFMA and no row-sum term is needed; the factor 64 is
//    divided out of the fp32 scale;
//  * the unpacked weight operand of a wave (one strip) is reused by its eight token blocks;
//  * activations sit in LDS in MFMA-operand order (1 KiB per 16-row x 64-k block, lane-major),
//    so every fragment read is one conflict-free ds_read_b128 and the global->LDS transfer is a
//    16-byte-per-lane LDS-direct copy that holds no registers while in flight;
//  * a wave's weights are its own strip and nobody else's; they take the same LDS-direct road into a
//    wave-private corner of the stage buffer;
//  * three stage buffers: the loads of stage s+2 are in flight while stage s is consumed, one
//    barrier per 128-element stage (with one workgroup on a CU there is no other wave to hide a
//    stage's load latency behind).
#pragma once
#include <type_traits>

#include "w2a8_launch.h"

namespace w2a8 {

namespace fast {
constexpr int kBN = 256;
constexpr int kStageSteps = 2;
constexpr int kStrips = kBN / kStripN;                     // 4 strips per workgroup, one per wave
constexpr int kAQueue = 4;                                 // activation fragments kept in flight from LDS
}  // namespace fast

// BM = token rows of the workgroup tile: 128, or 64 when 128-row tiles would leave CUs idle
// (fewer tiles than CUs, or a single workgroup per CU with nothing to hide its latencies behind).
// W4: 4-bit weights held as two 2-bit planes (hi digits in steps 0 .. steps-1 of w_r, lo digits in steps
// steps .. 2*steps-1; s_r rows 0 .. G-1 = 4 * scale) with the uniform zero-point 8.  Both digits of a step are fetched
// and put together before the MFMA: the operand byte 64 * (hi - 2) | 16 * lo is 16 * (code - 8), and the hi plane's
// scale times the 1/64 of the 2-bit path is scale / 16: one pass over K instead of two over 2K.
// DUMP: verification instantiation of the same body: every per-group int32 accumulator is also written out (exactly,
// as the MFMA left it, before its conversion to fp32); nothing else changes, so the output bits are the production
// instantiation's.
template <int BM, int GS, bool SPLIT, bool ZP, typename OutT, bool W4 = false, bool DUMP = false>
__device__ __forceinline__ void tiled_body(const GemmParams& p) {
    using namespace fast;
    constexpr int kBM = BM;
    constexpr int kMB = kBM / 16;                  // token blocks per wave (8 or 4)
    constexpr int kABlocks = kMB * kStageSteps;    // activation blocks per stage (16 or 8)
    constexpr int kStageDwords = kABlocks * 256;   // 16 or 8 KiB of activations per stage
    constexpr int kALoads = kABlocks / 4;          // LDS-direct activation block loads per wave and stage
    constexpr int kWPlanes = W4 ? 2 : 1;
    constexpr int kWDwords = kStrips * kStageSteps * 256 * kWPlanes;  // the four waves' weight units of a stage: 8 KiB a plane
    constexpr int kBufDwords = kStageDwords + kWDwords;
    constexpr int kBufs = 3;                       // stage s+2 is in flight while stage s is consumed
    __shared__ __attribute__((aligned(16))) uint32_t lds[kBufs][kBufDwords];
    // GS = 64-element steps per scale group: 1, 2, or 4.  With 4 a group spans two stages: every token block keeps
    // its own int32 accumulators from the first stage of a group to the second (kLong), the drain happens in the
    // second stages only, and the stage loop runs over pairs of stages.
    constexpr bool kLong = GS == 4;
    static_assert(!kLong || (BM == 64 && !W4), "a group of 256 runs on 64-row W2 tiles only");
    constexpr int GSE = kLong ? kStageSteps : GS;       // steps of a group inside one stage
    constexpr int kGroupsPerStage = kStageSteps / GSE;  // 2 (group 64) or 1 (group 128, 256)

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15, quad = lane >> 4;

    // Tile order: consecutive workgroup ids land on different XCDs (id % 8), each with its own
    // L2.  When the channel tiles divide by eight, every XCD owns one band of channel tiles for all
    // token tiles: its share of the weights then stays in its L2 for the whole kernel and only the
    // activations stream through (token tile major, so concurrent tiles share activation rows).
    // Otherwise, with two to four token tiles, the token tiles of a channel tile stay on one XCD and the channel tiles
    // are dealt out evenly (xcd_place: 11008 x 14336 at 80..128 rows 44.8..48.8 -> 40.8..43.1 us); with one token tile or
    // more than four, every XCD gets one contiguous run of tiles, channel tile fastest (one token tile dealt out by
    // xcd_place, neighbouring channel tiles on different XCDs, measured 17 % slower on that matrix: 29.9 -> 34.9 us).
    const int tiles_n = (p.strips + kStrips - 1) / kStrips;
    const int tiles_m = (p.M + kBM - 1) / kBM;
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int xcd = (int)(blockIdx.x & 7), local = (int)(blockIdx.x >> 3);
    int tile;
    if (tiles_n % 8 == 0) {
        const int band = tiles_n / 8;
        tile = (local / band) * tiles_n + xcd * band + local % band;
    } else if (tiles_m >= 2 && tiles_m <= 4) {
        int n_tile, m_tile_i;
        if (!xcd_place((int)blockIdx.x, tiles_n, tiles_m, n_tile, m_tile_i)) return;
        tile = m_tile_i * tiles_n + n_tile;
    } else {
        tile = xcd * per_xcd + local;
    }
    if (local >= per_xcd || tile >= total) return;
    const int m_tile = (tile / tiles_n) * kBM;
    const int strip0 = (tile % tiles_n) * kStrips;
    const int strip = min(strip0 + wave, p.strips - 1);  // clamped: a surplus wave recomputes the last strip, stores nothing
    const bool strip_ok = strip0 + wave < p.strips;
    // this workgroup's share of K in stages (all of it unless K is split over blockIdx.y)
    // (an odd step count ends in a stage whose second step lies past the weights and the scales: both read as zero
    // through the range-checked buffer loads, so that step's group adds nothing)
    const int all_stages = (p.steps + kStageSteps - 1) / kStageSteps;
    const int stages_per_split = SPLIT ? p.groups_per_split * GS / kStageSteps : all_stages;
    const int stage0 = SPLIT ? (int)blockIdx.y * stages_per_split : 0;
    const int n_stages = min(stages_per_split, all_stages - stage0);

    // ---- loads, one stage ahead, all through buffer instructions: a wave-uniform descriptor plus a
    // scalar offset that advances per stage, so no vector ALU work goes into addresses, and rows
    // past M read as zero (out-of-range buffer reads return 0).
    //  * activations: wave w copies blocks w, w+4, w+8, w+12 (block = step_in_stage * 8 + token block)
    //    straight from global memory into LDS (buffer_load_dwordx4 ... lds: lane l lands at 16*l);
    //  * weights: the two units of the wave's own strip (one per step) go to registers;
    //  * scales: the lane's four sub-block scales of each group of the stage.
    const __amdgpu_buffer_rsrc_t q_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t*>(p.q), 0, (int)min((size_t)p.M * p.ldq, (size_t)0x7fffffff), 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(p.w_r), 0, (int)min(weight_bytes(p.strips, p.steps * kWPlanes), (size_t)0x7fffffff), 0x00020000);
    const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.s_r), 0, (int)min((size_t)p.strips * p.G * 128, (size_t)0x7fffffff), 0x00020000);
    uint32_t a_off[kALoads];
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
        const int blk = wave + 4 * i;  // block = step_in_stage * kMB + token block
        a_off[i] = (uint32_t)(m_tile + (blk % kMB) * 16 + col) * (uint32_t)p.ldq + (blk / kMB) * kStepK + quad * 16;
    }
    const uint32_t b_run_pitch = (uint32_t)p.strips * (kRunSteps * kUnitBytes);  // bytes between runs of four steps of a strip
    const uint32_t b_strip_off = (uint32_t)strip * (kRunSteps * kUnitBytes);
    auto unit_off = [&](int step) { return (uint32_t)(step / kRunSteps) * b_run_pitch + (uint32_t)(step % kRunSteps) * kUnitBytes + b_strip_off; };
    const uint32_t s_lane_off = (uint32_t)(strip * 16 + col) * 8;
    const uint32_t s_group_stride = (uint32_t)p.strips * 128;               // bytes between groups of a strip
    typedef unsigned v2u __attribute__((ext_vector_type(2)));
    typedef unsigned v4u_t __attribute__((ext_vector_type(4)));
    v2u sraw[kGroupsPerStage];
    // Activations and this wave's weight units go straight from global memory into LDS (no registers
    // held while in flight), two stages ahead; the scales, a few bytes, go to registers one stage ahead.
    constexpr int kLdsLoads = kALoads + kStageSteps * kWPlanes;  // LDS-direct loads a wave issues per stage
    auto fetch = [&](int stage, int buf) {
#pragma unroll
        for (int i = 0; i < kALoads; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                q_rsrc, (__attribute__((address_space(3))) void*)&lds[buf][(wave + 4 * i) * 256], 16, a_off[i],
                (stage0 + stage) * (kStageSteps * kStepK), 0, 0);
#pragma unroll
        for (int s = 0; s < kStageSteps; ++s)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                w_rsrc, (__attribute__((address_space(3))) void*)&lds[buf][kStageDwords + (wave * kStageSteps + s) * 256], 16,
                lane * 16, unit_off((stage0 + stage) * kStageSteps + s), 0, 0);
        if constexpr (W4) {
#pragma unroll
            for (int s = 0; s < kStageSteps; ++s)   // the lo digits of the same steps: p.steps units further on
                __builtin_amdgcn_raw_ptr_buffer_load_lds(
                    w_rsrc, (__attribute__((address_space(3))) void*)&lds[buf][kStageDwords + kWDwords / 2 + (wave * kStageSteps + s) * 256], 16,
                    lane * 16, unit_off((stage0 + stage) * kStageSteps + s + p.steps), 0, 0);
        }
    };
    auto fetch_scales = [&](int stage) {
#pragma unroll
        for (int gi = 0; gi < kGroupsPerStage; ++gi)
            sraw[gi] = __builtin_amdgcn_raw_buffer_load_b64(
                s_rsrc, s_lane_off, ((stage0 + stage) * kStageSteps / GS + gi) * s_group_stride, 0);
    };
    // All but the newest stage's LDS-direct loads of this wave have arrived (loads complete in issue
    // order; the newest kLdsLoads may still be in flight), then meet the other waves.
    // (A bare s_barrier: __syncthreads() would add a fence that waits for every outstanding LDS-direct
    // load.  LDS is only written by those loads and only read with ds_read here, and a wave's reads of
    // a stage have all returned before it gets here, so nothing else needs ordering.)
    auto land = [&]() {
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kLdsLoads) : "memory");
    };

    float t[kMB][4][4];
#pragma unroll
    for (int mb = 0; mb < kMB; ++mb)
#pragma unroll
        for (int pp = 0; pp < 4; ++pp)
#pragma unroll
            for (int j = 0; j < 4; ++j) t[mb][pp][j] = 0.0f;

    fetch_scales(0);
    fetch(0, 0);
    fetch(min(1, n_stages - 1), 1);

    if (ZP) {
        // Zero-points other than the 2 the operand bytes are centred on: the missing term
        // -(zp - 2) * scale * rowsum of this workgroup's groups goes into the running sums first, as a
        // small matrix product over the groups through v_mfma_f32_16x16x4_f32 (lane (col, quad) supplies
        // token col / channel col of group 4b + quad; same D layout as the int8 MFMA), four blocks of
        // four groups per round so that a round's loads are in flight together.
        typedef float v4f __attribute__((ext_vector_type(4)));
        typedef _Float16 v4h __attribute__((ext_vector_type(4)));
        constexpr int kRound = 4;
        const int g_lo = stage0 * kStageSteps / GS, g_cnt = min(n_stages * kStageSteps / GS, p.G - g_lo);
        const uint32_t* zp32 = reinterpret_cast<const uint32_t*>(p.zp_r);
        int rrow[kMB];
#pragma unroll
        for (int mb = 0; mb < kMB; ++mb) rrow[mb] = min(m_tile + mb * 16 + col, p.M - 1);
        for (int gb = 0; gb < g_cnt; gb += 4 * kRound) {
            v2u zs[kRound];
            uint32_t zz[kRound];
            uint32_t zl[W4 ? kRound : 1];  // W4: the zero-points of the lo plane (rows G .. 2G-1)
            int rs[kRound][kMB];
#pragma unroll
            for (int b = 0; b < kRound; ++b) {
                const int g = g_lo + min(gb + 4 * b + quad, g_cnt - 1);  // clamped; masked below
                zs[b] = __builtin_amdgcn_raw_buffer_load_b64(s_rsrc, s_lane_off, g * s_group_stride, 0);
                zz[b] = p.zp_r ? zp32[((size_t)g * p.strips + strip) * 16 + col] : (uint32_t)p.zp_const * 0x01010101u;
                if constexpr (W4) zl[b] = zp32[((size_t)(g + p.G) * p.strips + strip) * 16 + col];
#pragma unroll
                for (int mb = 0; mb < kMB; ++mb) rs[b][mb] = p.rowsum[(size_t)g * p.ldr + rrow[mb]];
            }
#pragma unroll
            for (int b = 0; b < kRound; ++b) {
                const bool on = gb + 4 * b + quad < g_cnt;
                const v4h sh = __builtin_bit_cast(v4h, zs[b]);
                float zb[4];
#pragma unroll
                for (int pp = 0; pp < 4; ++pp)
                    // W4: sh is 4 * scale and the operand bytes are centred on 8 = 4 * 2 + 0: what is missing is
                    // (8 - 4 * zp_hi - zp_lo) * scale = (2 - zp_hi - zp_lo / 4) * sh
                    if constexpr (W4)
                        zb[pp] = on ? (2.0f - (float)((zz[b] >> (8 * pp)) & 0xffu) - 0.25f * (float)((zl[b] >> (8 * pp)) & 0xffu)) * (float)sh[pp] : 0.0f;
                    else
                        zb[pp] = on ? (2.0f - (float)((zz[b] >> (8 * pp)) & 0xffu)) * (float)sh[pp] : 0.0f;
#pragma unroll
                for (int mb = 0; mb < kMB; ++mb) {
                    const float rsf = (float)rs[b][mb];
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp) {
                        v4f c = {t[mb][pp][0], t[mb][pp][1], t[mb][pp][2], t[mb][pp][3]};
                        c = __builtin_amdgcn_mfma_f32_16x16x4f32(rsf, zb[pp], c, 0, 0, 0);
#pragma unroll
                        for (int j = 0; j < 4; ++j) t[mb][pp][j] = c[j];
                    }
                }
            }
        }
    }
    land();

    // accumulator sets (two, alternating; with a group of 256 one per token block, alive from the first stage of
    // a group to the second) and the scale of the unit carried over a stage boundary; zero to start with, so the
    // first carried drain adds nothing
    constexpr int kAccSets = kLong ? kMB : 2;
    v4i acc[kAccSets][4];
    float sc_prev[4];
#pragma unroll
    for (int pp = 0; pp < 4; ++pp) {
#pragma unroll
        for (int a = 0; a < kAccSets; ++a) acc[a][pp] = v4i{0, 0, 0, 0};
        sc_prev[pp] = 0.0f;
    }

    int buf = 0;
    // one stage; kHalf (group of 256 only): 0 = first stage of a group, 1 = second
    auto run_stage = [&](const int stage, auto half_tag) {
        constexpr int kHalf = decltype(half_tag)::value;
        const uint32_t* la = &lds[buf][lane * 4];
        auto lds_a = [&](int r) {  // r-th fragment in consumption order: token block r / 2, step r % 2
            return *reinterpret_cast<const v4i*>(la + ((r % kStageSteps) * kMB + r / kStageSteps) * 256);
        };
        v4i aq[kAQueue];
#pragma unroll
        for (int r = 0; r < kAQueue; ++r) aq[r] = lds_a(r);

        float sc[kGroupsPerStage][4];
#pragma unroll
        for (int gi = 0; gi < kGroupsPerStage; ++gi) {
            // operand bytes are 64 * (code - 2): fold 1/64 into the scale (exact)
            sc[gi][0] = half_bits_to_float((uint16_t)(sraw[gi].x & 0xffffu)) * 0.015625f;
            sc[gi][1] = half_bits_to_float((uint16_t)(sraw[gi].x >> 16)) * 0.015625f;
            sc[gi][2] = half_bits_to_float((uint16_t)(sraw[gi].y & 0xffffu)) * 0.015625f;
            sc[gi][3] = half_bits_to_float((uint16_t)(sraw[gi].y >> 16)) * 0.015625f;
        }

        // unpack this wave's strip for both steps of the stage (loaded during the previous stage)
        v4i b[kStageSteps][4];
#pragma unroll
        for (int s = 0; s < kStageSteps; ++s) {
            const v4i w = *reinterpret_cast<const v4i*>(la + kStageDwords + (wave * kStageSteps + s) * 256);
            const v4i wf = w ^ (int)0x2a2a2a2au;  // flip the high bit of fields 0..2: code -> two's complement of code - 2
#pragma unroll
            for (int pp = 0; pp < 3; ++pp) b[s][pp] = (wf << (6 - 2 * pp)) & (int)0xc0c0c0c0u;
            b[s][3] = w & (int)0xc0c0c0c0u;  // field 3 is stored already flipped
            if constexpr (W4) {
                typedef unsigned v4w __attribute__((ext_vector_type(4)));
                const v4w wl = __builtin_bit_cast(v4w, *reinterpret_cast<const v4i*>(la + kStageDwords + kWDwords / 2 + (wave * kStageSteps + s) * 256));
                b[s][0] |= __builtin_bit_cast(v4i, (wl << 4) & 0x30303030u);
                b[s][1] |= __builtin_bit_cast(v4i, (wl << 2) & 0x30303030u);
                b[s][2] |= __builtin_bit_cast(v4i, wl & 0x30303030u);
                b[s][3] |= __builtin_bit_cast(v4i, ((wl ^ 0x80808080u) >> 2) & 0x30303030u);  // stored flipped: back to the code
            }
        }

        // the scales of the next stage first, then the stage after next into the buffer that stage - 1 used
        // (every wave is past the barrier that ended stage - 1); the last iterations re-read the last
        // stage into an idle buffer: harmless, and the number of loads in flight stays the same
        fetch_scales(min(stage + 1, n_stages - 1));
        fetch(min(stage + 2, n_stages - 1), buf == 0 ? 2 : buf - 1);

        // Work units in order: (token block, group of the stage).  The MFMAs of unit u go into
        // accumulator set u & 1 and are written before the drain of unit u - 1, so the matrix core
        // works on one unit while the vector ALU folds the previous one; the last unit of a stage
        // is drained at the top of the next stage (or after the loop).
        constexpr int kUnits = kMB * kGroupsPerStage;
#pragma unroll
        for (int u = 0; u < kUnits; ++u) {
            const int mb = u / kGroupsPerStage, gi = u % kGroupsPerStage;
            // The drain of the previous unit (for u == 0: the last unit of the previous stage, scale
            // sc_prev) is dealt out evenly between this unit's MFMAs, with fences so that the
            // scheduler keeps the weave: the matrix core then always has the next MFMA queued behind
            // a few vector instructions instead of behind a whole drain.
            const int pu = (u + kUnits - 1) % kUnits;
            const int pmb = pu / kGroupsPerStage, pgi = pu % kGroupsPerStage;
            constexpr int kDrainPerMfma = 16 / (GSE * 4);  // elements of the previous unit per MFMA of this one
            // which accumulator set this unit's MFMAs write and which one is drained beside them; a group of 256
            // drains in its second stage (the block before this one) and, for the last block, at the top of the
            // next group's first stage
            const int cur = kLong ? mb : (u & 1), prev = kLong ? pmb : ((u & 1) ^ 1);
            const bool drains = !kLong || (kHalf == 1 ? u > 0 : u == 0);
            const bool from_zero = !kLong || kHalf == 0;
#pragma unroll
            for (int s = 0; s < GSE; ++s) {
                const int r = mb * kStageSteps + gi * GSE + s;  // fragment index in consumption order
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    acc[cur][pp] = mfma_i8_16x16x64(aq[r % kAQueue], b[gi * GSE + s][pp],
                                                    s == 0 && from_zero ? v4i{0, 0, 0, 0} : acc[cur][pp]);
                    if (drains) {
#pragma unroll
                        for (int d = 0; d < kDrainPerMfma; ++d) {
                            const int e = (s * 4 + pp) * kDrainPerMfma + d;  // 0..15: sub-block e / 4, row e % 4
                            t[pmb][e / 4][e % 4] = __builtin_fmaf((float)acc[prev][e / 4][e % 4],
                                                                  u == 0 ? sc_prev[e / 4] : sc[pgi][e / 4], t[pmb][e / 4][e % 4]);
                            if constexpr (DUMP) {  // the previous unit's group: for u == 0 the last group before this stage
                                const int g_here = (stage0 + stage) * kStageSteps / GS;
                                const int g_dump = kLong ? (u == 0 ? g_here - 1 : g_here) : g_here + (u == 0 ? -1 : pgi);
                                if ((u > 0 || stage > 0) && strip_ok && g_dump < p.G)
                                    dump_group_sum<W4>(p, m_tile + pmb * 16 + quad * 4 + e % 4, strip * kStripN + (e / 4) * 16 + col,
                                                       g_dump, acc[prev][e / 4][e % 4] >> (W4 ? 4 : 6), W4 ? 8 : 2);
                            }
                        }
                    }
                    if (pp == 3 && r + kAQueue < kABlocks) aq[r % kAQueue] = lds_a(r + kAQueue);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
#pragma unroll
        for (int pp = 0; pp < 4; ++pp) sc_prev[pp] = sc[kGroupsPerStage - 1][pp];

        land();
        buf = buf == kBufs - 1 ? 0 : buf + 1;
    };
    if constexpr (kLong) {
        for (int stage = 0; stage < n_stages; stage += 2) {  // whole groups: an even number of stages
            run_stage(stage, std::integral_constant<int, 0>{});
            run_stage(stage + 1, std::integral_constant<int, 1>{});
        }
    } else {
        for (int stage = 0; stage < n_stages; ++stage) run_stage(stage, std::integral_constant<int, 1>{});
    }
    // the last unit of the last stage
    constexpr int kLastSet = kLong ? kMB - 1 : 1;
#pragma unroll
    for (int pp = 0; pp < 4; ++pp)
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            t[kMB - 1][pp][j] = __builtin_fmaf((float)acc[kLastSet][pp][j], sc_prev[pp], t[kMB - 1][pp][j]);
            if constexpr (DUMP) {
                const int g_dump = (stage0 + n_stages) * kStageSteps / GS - 1;
                if (strip_ok && g_dump < p.G)
                    dump_group_sum<W4>(p, m_tile + (kMB - 1) * 16 + quad * 4 + j, strip * kStripN + pp * 16 + col,
                                       g_dump, acc[kLastSet][pp][j] >> (W4 ? 4 : 6), W4 ? 8 : 2);
            }
        }

    uint16_t* out = reinterpret_cast<uint16_t*>(p.out);
    if (SPLIT) {
        // ---- split-K: every workgroup of the tile publishes its fp32 partial sums (fragment order:
        // the wave that reduces them has the same lane layout, so no transposition), the last to
        // arrive adds them up in split order (deterministic) and finishes.  Agent-scope relaxed
        // atomics: write-through stores and cache-bypassing loads, no L2 fence needed.
        // Partials move as 16-byte buffer stores / loads at system-coherent cache policy (write-through,
        // read around the L2 of whichever XCD the reducing workgroup runs on): plain memory
        // instructions, so the reduction's loads are all in flight together.
        constexpr int kTileBytes = kBM * kBN * 4;
        constexpr int kCoherent = 17;  // sc0 | sc1
        typedef float v4f __attribute__((ext_vector_type(4)));
        const int n_split = (int)gridDim.y;
        const __amdgpu_buffer_rsrc_t ws_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            p.ws_partial, 0, (int)((size_t)n_split * total * kTileBytes), 0x00020000);
        const uint32_t ws_lane = (uint32_t)wave * (kMB * 16 * 64 * 4) + lane * 16;   // this wave's fragments, this lane's 16 bytes
        const uint32_t ws_tile = (uint32_t)tile * kTileBytes;
        const uint32_t ws_split_pitch = (uint32_t)total * kTileBytes;
        // A 16-byte-per-lane buffer store reads its data registers some time after it issues (longer when the memory
        // pipeline is backed up, as it is for the workgroups of a launch that start last).  With a register in the
        // scalar-offset field the compiler knows of no hazard there, and a vector instruction scheduled behind such a
        // store once reused the store's first data register for the address of the next stores: the partial sums of
        // four lanes in sixteen went to memory as that address (130 x 4096 x 1024 in eight splits, bf16 out: 48..150
        // outputs short of one split's share on every run).  Three independent measures against it: the split's and the tile's base go into the per-lane offset, so the scalar offset is the constant
        // zero, the form whose wait states the compiler inserts itself; every address is made before the first store
        // and each store is followed by two idle cycles written here (the wait the hardware needs, whatever the
        // scheduler and the register allocator do); and fences keep everything else out of the run of stores.
        const uint32_t ws_base = blockIdx.y * ws_split_pitch + ws_tile;
        uint32_t ws_off[kMB];
#pragma unroll
        for (int mb = 0; mb < kMB; ++mb) {
            ws_off[mb] = ws_lane + mb * 4096 + ws_base;
            asm volatile("" : "+v"(ws_off[mb]));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mb = 0; mb < kMB; ++mb)
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                const v4f v = {t[mb][pp][0], t[mb][pp][1], t[mb][pp][2], t[mb][pp][3]};
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u_t, v), ws_rsrc, ws_off[mb] + pp * 1024, 0, kCoherent);
                asm volatile("s_nop 1" ::: "memory");
            }
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        if (tid == 0) {
            const unsigned prev = __hip_atomic_fetch_add(p.ws_counter + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            lds[0][0] = (prev == (unsigned)(n_split - 1));
        }
        __syncthreads();
        if (lds[0][0] == 0) return;
        // one split at a time, four token blocks' fragments in flight together (one memory latency per split and
        // half tile; all eight blocks at once would not fit the registers next to the running sums)
        constexpr int kChunk = 4;
#pragma unroll
        for (int mb0 = 0; mb0 < kMB; mb0 += kChunk) {
#pragma unroll
            for (int mb = 0; mb < kChunk; ++mb)
#pragma unroll
                for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                    for (int j = 0; j < 4; ++j) t[mb0 + mb][pp][j] = 0.0f;
            for (int sp = 0; sp < n_split; ++sp) {
                v4f v[kChunk][4];
#pragma unroll
                for (int mb = 0; mb < kChunk; ++mb)
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp)
                        v[mb][pp] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(
                            ws_rsrc, ws_lane + ((mb0 + mb) * 4 + pp) * 1024, sp * ws_split_pitch + ws_tile, kCoherent));
#pragma unroll
                for (int mb = 0; mb < kChunk; ++mb)
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                        for (int j = 0; j < 4; ++j) t[mb0 + mb][pp][j] += v[mb][pp][j];
            }
        }
        if (tid == 0) __hip_atomic_store(p.ws_counter + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- epilogue: out = cast(t * s_a[m])
    // the token scales first, all loads in flight together (a load inside the store loop would not
    // move above the stores before it and would cost one memory latency per row)
    float sa_row[kMB][4];
#pragma unroll
    for (int mb = 0; mb < kMB; ++mb)
#pragma unroll
        for (int j = 0; j < 4; ++j) sa_row[mb][j] = p.s_a[min(m_tile + mb * 16 + quad * 4 + j, p.M - 1)];

    if ((p.N & 7) == 0 && (p.ldo & 7) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0) {
        // Rows of 8 channels x 2 bytes = one 16-byte store per lane, eight lanes per 128-byte line of an
        // output row.  The accumulator layout has a lane's values in different rows, so they turn
        // through LDS: each wave owns a corner of the (now idle) stage buffers, writes 32 token rows
        // x 64 channels of scaled fp32 sums (row pitch 68 floats: the four row groups of a write fall
        // into different banks), and reads them back as 8 consecutive channels per lane.
        // Every wave's LDS-direct loads must have landed and every wave must be out of the main
        // loop before the buffers change their use.
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
        if (!strip_ok) return;
        constexpr int kPitch = 68;
        static_assert(32 * kPitch * 4 * kStrips <= (int)sizeof(lds), "output staging exceeds the stage buffers");
        float* stage_out = reinterpret_cast<float*>(&lds[0][0]) + wave * (32 * kPitch);
        typedef float v4f_t __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int rd = 0; rd < kMB / 2; ++rd) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        stage_out[(h * 16 + quad * 4 + j) * kPitch + pp * 16 + col] = t[rd * 2 + h][pp][j] * sa_row[rd * 2 + h][j];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = i * 8 + (lane >> 3), cg = lane & 7;
                const v4f_t lo = *reinterpret_cast<const v4f_t*>(stage_out + row * kPitch + cg * 8);
                const v4f_t hi = *reinterpret_cast<const v4f_t*>(stage_out + row * kPitch + cg * 8 + 4);
                v4u_t v;
                v.x = (uint32_t)OutT::cast(lo.x) | ((uint32_t)OutT::cast(lo.y) << 16);
                v.y = (uint32_t)OutT::cast(lo.z) | ((uint32_t)OutT::cast(lo.w) << 16);
                v.z = (uint32_t)OutT::cast(hi.x) | ((uint32_t)OutT::cast(hi.y) << 16);
                v.w = (uint32_t)OutT::cast(hi.z) | ((uint32_t)OutT::cast(hi.w) << 16);
                const int m = m_tile + rd * 32 + row, n = strip * kStripN + cg * 8;
                if (m < p.M && n < p.N) *reinterpret_cast<v4u_t*>(out + (size_t)m * p.ldo + n) = v;
            }
        }
        return;
    }

    // any N, row pitch and alignment of out: one 2-byte store per value
    if (!strip_ok) return;
#pragma unroll
    for (int mb = 0; mb < kMB; ++mb)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m_tile + mb * 16 + quad * 4 + j;
            if (m >= p.M) continue;
            const float sa = sa_row[mb][j];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                const int n = strip * kStripN + pp * 16 + col;
                if (n < p.N) out[(size_t)m * p.ldo + n] = OutT::cast(t[mb][pp][j] * sa);
            }
        }
}

// 128-row tiles: two workgroups (eight waves) per CU; 64-row tiles need fewer registers: three (two with a group of
// 256, whose token blocks each keep a set of int32 accumulators).
template <int GS, bool SPLIT, bool ZP, typename OutT, bool DUMP = false>
__global__ __launch_bounds__(256, 2) void tiled_kernel(const GemmParams p) {
    tiled_body<128, GS, SPLIT, ZP, OutT, false, DUMP>(p);
}
template <int GS, bool SPLIT, bool ZP, typename OutT, bool DUMP = false>
__global__ __launch_bounds__(256, DUMP || GS == 4 ? 2 : 3) void tiled_kernel_bm64(const GemmParams p) {
    tiled_body<64, GS, SPLIT, ZP, OutT, false, DUMP>(p);
}

// 4-bit weights, one pass (64-row tiles: three stage buffers of 24 KiB leave room for two workgroups on a CU)
template <int GS, bool SPLIT, bool ZP, typename OutT, bool DUMP = false>
__global__ __launch_bounds__(256, 2) void tiled_kernel_w4(const GemmParams p) {
    tiled_body<64, GS, SPLIT, ZP, OutT, true, DUMP>(p);
}

template <bool DUMP>
static hipError_t launch_tiled_w4_impl(const GemmParams& p, int gs, bool out_bf16, hipStream_t stream) {
    const int tiles = (int)tiled_w4_tiles(p.M, p.strips);
    const dim3 grid((tiles + 7) / 8 * 8, p.split > 1 ? p.split : 1), block(256);
#define SLIMK_W4_LAUNCH(GSV, ZPV)                                                                         \
    do {                                                                                                  \
        if (p.split > 1) {                                                                                \
            if (out_bf16) tiled_kernel_w4<GSV, true, ZPV, OutBF16, DUMP><<<grid, block, 0, stream>>>(p);  \
            else tiled_kernel_w4<GSV, true, ZPV, OutF16, DUMP><<<grid, block, 0, stream>>>(p);            \
        } else {                                                                                          \
            if (out_bf16) tiled_kernel_w4<GSV, false, ZPV, OutBF16, DUMP><<<grid, block, 0, stream>>>(p); \
            else tiled_kernel_w4<GSV, false, ZPV, OutF16, DUMP><<<grid, block, 0, stream>>>(p);           \
        }                                                                                                 \
    } while (0)
    const bool zp = p.zp_r != nullptr;   // per-group zero-points: the planes' (rows 0..G-1 hi, G..2G-1 lo) and p.rowsum
    if (gs == 1) {
        if (zp) SLIMK_W4_LAUNCH(1, true);
        else SLIMK_W4_LAUNCH(1, false);
    } else {
        if (zp) SLIMK_W4_LAUNCH(2, true);
        else SLIMK_W4_LAUNCH(2, false);
    }
#undef SLIMK_W4_LAUNCH
    return hipGetLastError();
}

// Tile height and tile count of the fast kernel for a problem: two workgroups fit a CU, so below
// about two 128-row tiles per CU, 64-row tiles fill the chip better.  A group of 256 (gs = 4) has 64-row tiles only.
inline void tiled_fast_tiles(int M, int strips, int gs, int* bm, int* tiles) {
    const int tiles_n = (strips + fast::kStrips - 1) / fast::kStrips;
    const int tiles128 = tiles_n * ((M + 127) / 128);
    const bool small = tiles128 < 2 * 256 || gs == 4;
    *bm = small ? 64 : 128;
    *tiles = small ? tiles_n * ((M + 63) / 64) : tiles128;
}

// A verification call (DUMP) runs the same body with the dump switched on: same tile height, same split.
template <bool DUMP>
static hipError_t launch_tiled_impl(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    if (!tiled_fast_supported(p, gs, asym)) return hipErrorInvalidValue;  // (group sizes the library does not offer)
    int bm, tiles;
    tiled_fast_tiles(p.M, p.strips, gs, &bm, &tiles);
    const dim3 grid((tiles + 7) / 8 * 8, p.split > 1 ? p.split : 1), block(256);
    const bool zp = asym || p.zp_const != 2;
    const bool split = p.split > 1;
#define SLIMK_TILED_LAUNCH_BM64(GSV, ZPV)                                                                     \
    do {                                                                                                      \
        if (split) {                                                                                          \
            if (out_bf16) tiled_kernel_bm64<GSV, true, ZPV, OutBF16, DUMP><<<grid, block, 0, stream>>>(p);    \
            else tiled_kernel_bm64<GSV, true, ZPV, OutF16, DUMP><<<grid, block, 0, stream>>>(p);              \
        } else {                                                                                              \
            if (out_bf16) tiled_kernel_bm64<GSV, false, ZPV, OutBF16, DUMP><<<grid, block, 0, stream>>>(p);   \
            else tiled_kernel_bm64<GSV, false, ZPV, OutF16, DUMP><<<grid, block, 0, stream>>>(p);             \
        }                                                                                                     \
    } while (0)
#define SLIMK_TILED_LAUNCH(GSV, ZPV)                                                                          \
    do {                                                                                                      \
        if (bm == 128 && split) {                                                                             \
            if (out_bf16) tiled_kernel<GSV, true, ZPV, OutBF16, DUMP><<<grid, block, 0, stream>>>(p);         \
            else tiled_kernel<GSV, true, ZPV, OutF16, DUMP><<<grid, block, 0, stream>>>(p);                   \
        } else if (bm == 128) {                                                                               \
            if (out_bf16) tiled_kernel<GSV, false, ZPV, OutBF16, DUMP><<<grid, block, 0, stream>>>(p);        \
            else tiled_kernel<GSV, false, ZPV, OutF16, DUMP><<<grid, block, 0, stream>>>(p);                  \
        } else {                                                                                              \
            SLIMK_TILED_LAUNCH_BM64(GSV, ZPV);                                                                \
        }                                                                                                     \
    } while (0)
    if (gs == 1) {
        if (zp) SLIMK_TILED_LAUNCH(1, true);
        else SLIMK_TILED_LAUNCH(1, false);
    } else if (gs == 2) {
        if (zp) SLIMK_TILED_LAUNCH(2, true);
        else SLIMK_TILED_LAUNCH(2, false);
    } else {
        if (zp) SLIMK_TILED_LAUNCH_BM64(4, true);
        else SLIMK_TILED_LAUNCH_BM64(4, false);
    }
#undef SLIMK_TILED_LAUNCH
#undef SLIMK_TILED_LAUNCH_BM64
    return hipGetLastError();
}

}  // namespace w2a8
