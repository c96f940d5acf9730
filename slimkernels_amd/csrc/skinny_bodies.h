// Skinny-M (M <= 32) W2A8 GEMMs for gfx950: the HBM-bound decode regime.  Two kernels.
//
// skinny_kernel: one GEMM per launch.  Grid (strips, split, 16-row token blocks).  A workgroup of
// NW (4, 8 or 16) wavefronts owns one 64-channel strip and a contiguous range of scale groups; its
// waves take contiguous sub-ranges, so each wave streams a run of 1 KiB weight units (four consecutive
// steps of a strip are 4 KiB in one piece) straight from global memory into VGPRs (one buffer_load_dwordx4 per lane and unit:
// nothing in a unit is shared between waves).  A single decode GEMM is a latency problem before
// it is a bandwidth problem (the whole thing is a few microseconds), so every load is issued as
// early as possible:
//  * weights and activations run through a register ring kDepth steps deep (the load for step
//    s + kDepth is issued when step s is consumed), addressed through buffer descriptors with a
//    per-lane offset fixed for the kernel and a scalar offset per step;
//  * the per-group metadata (scales, zero-points, activation row sums) is fetched into registers
//    one chunk ahead and parked in a wave-private LDS area;
//  * the token scales s_a needed by the epilogue are fetched at kernel entry.
// Per group the int32 accumulators are drained into fp32 running sums with the group's fp16 scale
// (cvt + fma_mix); the workgroup's waves' sums meet in LDS, and for split > 1 the workgroups'
// partial tiles meet in the workspace, summed in a fixed order by the last workgroup to arrive
// (deterministic, no float atomics).
//
// skinny_grouped_kernel: several GEMMs per launch, built for throughput; see shared_body below.
#pragma once
#include "w2a8_launch.h"

namespace w2a8 {

// cache policy of the weight loads when every byte is used exactly once (the nt bit of the buffer
// instruction); with two 16-row blocks the second block's read is meant to hit in L2 instead
constexpr int kStreamOnce = 2;
constexpr int kDepth = 4;  // ring depth in steps = steps per metadata chunk = granule of the K partition

typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

// NWP = wavefronts per workgroup.  Each wave owns a private metadata area; the reduction tile
// reuses the same memory once every wave has left its loop.
struct SkinnyMeta {
    uint16_t scale[kDepth][16][4];  // [group in chunk][col][sub-block]
    uint8_t zp[kDepth][16][4];
    int32_t rowsum[kDepth][16];
};

// FUSED: the workgroup quantises the (at most four) token rows itself before it needs them.
struct FusedRows {
    int8_t q[kFusedMaxBytes];                  // [row][K]
    v4i rowsum[kFusedMaxBytes / kStepK];       // [group]: the rows' sums of q over the group (rows past M: 0)
    float s_a[kFusedMaxRows];
    float amax[16][kFusedMaxRows];             // per wave, then reduced
};
struct NoFusedRows {};

template <int NWP, bool WIDE, bool FUSED = false>
struct SkinnySmem {
    union {
        SkinnyMeta meta[NWP];
        float red[NWP][16][kStripN + 1];
    };
    v4u atile[WIDE ? NWP : 1][kDepth][64];  // WIDE: a wave's activation fragments of one chunk, in MFMA operand order
    int last;
    typename std::conditional<FUSED, FusedRows, NoFusedRows>::type fused;
};

// ---------------------------------------------------------------------------------------------
// Activation rows quantised inside the GEMM launch by the grid's own first workgroups (skinny_rows_kernel: 5..32 token
// rows, or fewer rows too long for the in-workgroup form above).  Workgroup i < M of the grid (in dispatch order)
// quantises row i (and i + the grid's size, ..., should the grid be smaller than M) of the fp16 / bf16 activations p.x into the caller's workspace, where p.q / p.s_a / p.rowsum point
// -- the numbers of act_quant_kernel: per-token scale absmax / 127, IEEE binary32 division, round-half-even, clip to
// +-127, the per-group sums of q -- and then raises the first of two counters at the end of the workspace's counter
// block; every workgroup, the quantising ones included, goes on to its GEMM share, starts its weight stream and only
// then waits for the counter to reach M.  The second counter counts the workgroups that are past the wait; the last
// of them puts both back to zero, so the workspace is ready for the next call when the kernel ends.
template <int THREADS>
__device__ __forceinline__ void rows_quantise_row(const GemmParams& p, const int m, float* scratch) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint16_t* xr = p.x + (size_t)m * p.ldx;
    const int nvec = p.K / 8;
    const bool bf16 = p.x_bf16 != 0;
    auto load8 = [&](const uint16_t* src, float (&f)[8]) {
        const uint4 raw = *reinterpret_cast<const uint4*>(src);
        const uint32_t wds[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (bf16) {
                f[2 * i] = __uint_as_float(wds[i] << 16);
                f[2 * i + 1] = __uint_as_float(wds[i] & 0xffff0000u);
            } else {
                f[2 * i] = half_bits_to_float((uint16_t)(wds[i] & 0xffffu));
                f[2 * i + 1] = half_bits_to_float((uint16_t)(wds[i] >> 16));
            }
        }
    };
    float amax = 0.0f;
    for (int v = tid; v < nvec; v += THREADS) {
        float f[8];
        load8(xr + (size_t)v * 8, f);
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(f[i]));
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if (lane == 0) scratch[wave] = amax;
    __syncthreads();
    float a = scratch[0];
#pragma unroll
    for (int w = 1; w < THREADS / 64; ++w) a = fmaxf(a, scratch[w]);
    __syncthreads();  // scratch is free again
    const float s = fmaxf(a, 1e-9f) / 127.0f;
    const float inv_s = 1.0f / s;
    if (tid == 0) const_cast<float*>(p.s_a)[m] = s;
    int8_t* qr = const_cast<int8_t*>(p.q) + (size_t)m * p.ldq;
    int32_t* rs = const_cast<int32_t*>(p.rowsum);
    const int tpg = p.K / p.G / 8;  // threads per scale group (8 elements each): 8, 16 or 32, whole groups per wave
    for (int v0 = 0; v0 < nvec; v0 += THREADS) {  // (every thread makes every trip: the shuffles need whole waves)
        const int v = v0 + tid;
        int sum = 0;
        if (v < nvec) {
            float f[8];
            load8(xr + (size_t)v * 8, f);  // second read of the row: from the cache
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float r = rne_quotient(f[i], s, inv_s);  // = rintf(f[i] / s), bit for bit
                r = fminf(fmaxf(r, -127.0f), 127.0f);
                const int qi = (int)r;
                sum += qi;
                if (i < 4) lo |= (uint32_t)(qi & 0xff) << (8 * i);
                else hi |= (uint32_t)(qi & 0xff) << (8 * (i - 4));
            }
            *reinterpret_cast<uint2*>(qr + (size_t)v * 8) = make_uint2(lo, hi);
        }
        for (int off = 1; off < tpg; off <<= 1) sum += __shfl_xor(sum, off, 64);
        if (v < nvec && v % tpg == 0) rs[(size_t)(v / tpg) * p.ldr + m] = sum;
    }
}

template <int THREADS>
__device__ __forceinline__ void rows_quantise_and_signal(const GemmParams& p, float* scratch) {
    const int wg = (int)(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z));  // dispatch order
    if (wg >= p.M) return;  // (the same for the whole workgroup)
    const int total = (int)(gridDim.x * gridDim.y * gridDim.z);
    unsigned done = 0;
    for (int m = wg; m < p.M; m += total, ++done) rows_quantise_row<THREADS>(p, m, scratch);  // (a grid smaller than M: several rows)
    // Every thread's stores have reached this XCD's L2 (s_waitcnt), then ONE thread writes that L2 back to where the
    // other XCDs see it and raises the counter: the write-back is an operation on the whole L2 and serialises there,
    // one per workgroup is what is needed and a fence in every wave is 4..16 times that.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        __hip_atomic_fetch_add(p.ws_counter + kRowFlagSlot, done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// The bounded wait for the rows.  flag: one int of LDS.  A workgroup whose polls run out quantises every row itself:
// the same bytes to the same places as the workgroups it gave up on, so whoever reads them reads the same thing.
template <int THREADS>
__device__ __forceinline__ void rows_wait(const GemmParams& p, float* scratch, int* flag, const int spin_limit) {
    unsigned* const flags = p.ws_counter + kRowFlagSlot;
    if (threadIdx.x == 0) {
        int ok = 0;
        for (int i = 0; i < spin_limit; ++i) {
            if (__hip_atomic_load(flags, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= (unsigned)p.M) {
                ok = 1;
                break;
            }
            __builtin_amdgcn_s_sleep(2);
        }
        *flag = ok;
        // one invalidate per workgroup (this CU's L1 and the XCD's L2 drop what they hold of memory other XCDs write),
        // before the barrier that lets the other waves read the rows: an invalidate in every wave serialises on the L2
        if (ok) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    }
    __syncthreads();
    if (*flag == 0) {
        for (int m = 0; m < p.M; ++m) rows_quantise_row<THREADS>(p, m, scratch);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0) __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "agent");
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const unsigned total = gridDim.x * gridDim.y * gridDim.z;
        const unsigned prev = __hip_atomic_fetch_add(flags + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev == total - 1) {  // every workgroup is past its wait: ready for the next call
            __hip_atomic_store(flags, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(flags + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// One wave's share of one strip and one block of 16 token rows (a problem with 17..32 rows is
// run as two row blocks by two sets of waves: the second read of the weights comes from L2, and
// the small register footprint of a single block is what lets four waves share a SIMD).
//   J     live rows per lane of a D fragment: 4 in general, 1 when M == 1 (only row 0 of the 16x16
//         block is a real token, so three quarters of the drain arithmetic are dropped)
//   GS    steps per scale group
//   NWK   waves that split the workgroup's K range among them (1: the wave owns all of it and
//         stores its results itself; NWP: all the workgroup's waves, meeting in LDS)
//   ASYM  per-(group, channel) zero-points from zp_r instead of the uniform zp_const
//   DUMP  verification instantiation: the exact int32 group sums are also written out, as the MFMAs left them and
//         before their conversion to fp32; nothing else changes, so the output bits are the production instantiation's
//   FUSED the activations arrive as fp16 / bf16 rows (at most four, rows x K <= 32 KiB) and every
//         workgroup quantises them itself into LDS while its first weights are on the way: the numbers
//         of act_quant_kernel (per-token scale, int8 values, per-group sums), no separate launch
//   WIDE  activations are fetched two steps wide (whole 128-byte lines of the row-major tokens: half
//         the cache lines of a step-by-step fetch once there are eight rows or more) and turned into
//         MFMA operand order through a wave-private LDS tile; no barrier, the wave only meets itself
//
// Zero-points.  The MFMA operand of field p is code * 4^p (p < 3) or 64 * (code - 2) (p = 3), so
// a group's true sum is raw - zpe * rowsum with zpe = zp * 4^p resp. (zp - 2) * 64.  The timed
// kernels never form that integer: the term -zpe * scale * rowsum is itself a small matrix
// product over the groups (16 tokens x 16 channels x up to 4 groups of a chunk) and goes through
// one v_mfma_f32_16x16x4_f32 per chunk and sub-block, accumulating straight into the fp32 running
// sums (same D layout as the int8 MFMA).
template <int J, int GS, int NWK, int NWP, bool ASYM, bool DUMP, bool NT, bool WIDE, bool FUSED, typename OutT, bool ROWS = false>
__device__ __forceinline__ void skinny_body(const GemmParams& p, const int strip, const int split, const int mblk,
                                            const int kwave, const int pwave, SkinnySmem<NWP, WIDE, FUSED>& sm,
                                            const int spin_limit = 0) {
    static_assert(!FUSED || (!WIDE && !DUMP && NWK == NWP), "fused activation quantisation: the plain production body");
    static_assert(!ROWS || (!FUSED && !DUMP && NWK == NWP), "rows quantised by the grid's first workgroups: a production body");
    // 16-row blocks a wave works on per weight unit: one.  (The loops below are written over MB: two blocks per wave,
    // which halve the passes over the weights of a problem with more than 16 rows, were measured and are slower on
    // small matrices and under 10 % faster on large ones.)
    constexpr int MB = 1;
    static_assert(NWK == 1 || NWK == NWP, "K is split over one wave or over the whole workgroup");
    constexpr int kThreads = NWP * 64;
    constexpr int kGroupsPerChunk = kDepth / GS;
    constexpr int kTile = MB * 16 * kStripN;                 // elements of a strip's output tile (workspace pitch)
    constexpr int kLive = (J == 1 ? 1 : MB * 16) * kStripN;  // elements of it that can hold real tokens
    constexpr int kOutPerThread = (kLive + kThreads - 1) / kThreads;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int col = lane & 15, quad = lane >> 4;
    SkinnyMeta& meta = sm.meta[pwave];

    // this row block's view of the per-token operands
    const int m0 = mblk * 16;
    const int M = min(16, p.M - m0);
    const int8_t* const qp = p.q + (size_t)m0 * p.ldq;
    const float* const sap = p.s_a + m0;
    const int32_t* const rsp = p.rowsum + m0;
    const int ldr = p.ldr - m0;
    uint16_t* const out = reinterpret_cast<uint16_t*>(p.out) + (size_t)m0 * p.ldo;
    const int mblocks = (p.M + 15) >> 4;
    const int tile_id = strip * mblocks + mblk;  // index of this (strip, row block) in the split-K workspace

    // token scales for the epilogue, fetched first
    float sa[NWK == 1 ? MB * J : kOutPerThread];
    auto load_sa = [&]() {
        if (NWK == 1) {  // this wave stores D fragments itself: rows mb*16 + quad*4 + j
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int j = 0; j < J; ++j) sa[mb * J + j] = sap[min(mb * 16 + quad * 4 + j, M - 1)];
        } else {  // element e = tid + kThreads*i of the reduced tile -> row e >> 6
#pragma unroll
            for (int i = 0; i < kOutPerThread; ++i) sa[i] = sap[min((tid + kThreads * i) >> 6, M - 1)];
        }
    };
    if (!FUSED && !ROWS) load_sa();  // (FUSED, ROWS: once the rows are quantised)

    // Step range of this workgroup (groups_per_split is a multiple of a chunk's groups), then of this
    // wave, in whole chunks of kDepth steps; only a range's last chunk can be ragged.
    const int wg_s0 = min(split * p.groups_per_split, p.G) * GS;
    const int wg_s1 = min((split + 1) * p.groups_per_split, p.G) * GS;
    const int wg_chunks = (wg_s1 - wg_s0 + kDepth - 1) / kDepth;
    const int per_wave = (wg_chunks + NWK - 1) / NWK;
    const int s0 = min(wg_s0 + kwave * per_wave * kDepth, wg_s1);
    const int s1 = min(s0 + per_wave * kDepth, wg_s1);
    const int g1 = s1 / GS;
    const int len = s1 - s0;
    auto stepof = [&](int it) { return s0 + min(it, len - 1); };  // iterations past the end repeat the last step

    // Addressing: buffer descriptors with a per-lane offset fixed for the whole kernel and a scalar
    // offset per step, so no vector ALU work goes into addresses.  No load is predicated or sits
    // under a branch: out-of-range rows, groups and steps are clamped onto valid ones instead, so the
    // number of loads in flight is the same on every path and the s_waitcnt the compiler places
    // before each use waits for exactly that load (a token row >= M only ever feeds output rows >= M,
    // which are not stored; a clamped step or group is never used).
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(p.w_r), 0, (int)weight_bytes(p.strips, p.steps), 0x00020000);
    const __amdgpu_buffer_rsrc_t q_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t*>(qp), 0, (int)((size_t)(M - 1) * p.ldq + p.K), 0x00020000);
    const uint32_t wstride = (uint32_t)p.strips * (kRunSteps * kUnitBytes);  // bytes between consecutive runs of a strip
    const uint32_t wbase = (uint32_t)strip * (kRunSteps * kUnitBytes);
    const uint32_t wlane = lane * 16;
    uint32_t aoff[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) aoff[mb] = (uint32_t)min(mb * 16 + col, M - 1) * (uint32_t)p.ldq + quad * 16;

    // ---- metadata prefetch registers: one chunk (kGroupsPerChunk groups) ahead
    v4i m_scale;     // scales: up to 4 groups x 128 B = 512 B per wave: lanes 0..31, 16 B each
    v4i m_zp;        // zero-points: up to 4 groups x 64 B: lanes 0..15
    v4i m_rs[MB];    // row sums: lane -> (group lane >> 2, rows 4*(lane & 3) ..): lanes 0..15
    auto fused_rowsum = [&](int g) -> v4i {
        if constexpr (FUSED) return sm.fused.rowsum[g];
        else return v4i{0, 0, 0, 0};
    };
    // (FUSED: the row sums come from LDS once the rows are quantised; the entry path fetches the
    // global part before that and the row sums after it)
    auto fetch_meta = [&](int gfirst, bool global_part = true, bool rowsum_part = true) {  // groups gfirst .. gfirst + kGroupsPerChunk - 1, clamped to g1 - 1
        const int gq = min(gfirst + (lane >> 2), g1 - 1);
        if (global_part) {
            const size_t sgi = (size_t)min(gfirst + (lane >> 3), g1 - 1) * p.strips + strip;
            m_scale = *reinterpret_cast<const v4i*>(reinterpret_cast<const char*>(p.s_r) + sgi * 128 + (lane & 7) * 16);
            if (ASYM)
                m_zp = *reinterpret_cast<const v4i*>(reinterpret_cast<const char*>(p.zp_r) +
                                                     ((size_t)gq * p.strips + strip) * 64 + (lane & 3) * 16);
        }
        if (FUSED) {
            if (rowsum_part) m_rs[0] = (lane & 3) == 0 ? fused_rowsum(gq) : v4i{0, 0, 0, 0};  // rows 0..3 only
        } else if (rowsum_part) {
            const int32_t* rp = rsp + (size_t)gq * p.ldr;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                m_rs[mb] = *reinterpret_cast<const v4i*>(rp + min(mb * 16 + (lane & 3) * 4, ldr - 4));
        }
    };
    auto park_meta = [&](int gfirst) {  // the registers hold groups gfirst ..
        // a group past the end of the range (ragged last chunk) gets zero scales: it then adds nothing
        // (decided here, where the loaded registers are first needed anyway, not at the load)
        if (gfirst + (lane >> 3) >= g1) m_scale = v4i{0, 0, 0, 0};
        if (lane < kDepth * 8) *reinterpret_cast<v4i*>(reinterpret_cast<char*>(&meta.scale[0][0][0]) + lane * 16) = m_scale;
        if (lane < kDepth * 4) {
            if (ASYM) *reinterpret_cast<v4i*>(reinterpret_cast<char*>(&meta.zp[0][0][0]) + lane * 16) = m_zp;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                *reinterpret_cast<v4i*>(&meta.rowsum[lane >> 2][mb * 16 + (lane & 3) * 4]) = m_rs[mb];
        }
    };

    // ---- weight / activation register ring
    v4u wring[kDepth];
    v4u aring[kDepth][MB];
    auto issue_a = [&](int slot, int step) {
        if (!WIDE && !FUSED) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                aring[slot][mb] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, aoff[mb], step * kStepK, 0);
        }
    };
    auto issue = [&](int slot, int step, bool with_a = true) {  // step is wave-uniform
        wring[slot] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wlane, (step / kRunSteps) * wstride + (step % kRunSteps) * kUnitBytes + wbase,
                                                            NT ? kStreamOnce : 0);
        if (with_a) issue_a(slot, step);
    };
    // WIDE: fragment (pair q, row half h) of a chunk: lane l reads row 8h + l/8, 16-byte piece l%8 of the
    // 128 bytes the pair's two steps cover, and parks it at step 2q + piece/4, lane (piece%4)*16 + row.
    // (A pair that starts on the range's last step reads 64 bytes past it: the bytes of the next
    // step or, past K, zeros or the next row; that step carries a zero scale.)
    v4u awide[kDepth];
    const uint32_t wpiece = lane & 7;
    const int wrow[2] = {lane >> 3, 8 + (lane >> 3)};
    auto fetch_wide = [&](int it) {
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                awide[2 * q + h] = __builtin_amdgcn_raw_buffer_load_b128(
                    q_rsrc, (uint32_t)min(wrow[h], M - 1) * (uint32_t)p.ldq + wpiece * 16, stepof(it + 2 * q) * kStepK, 0);
    };
    auto park_wide = [&]() {
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int h = 0; h < 2; ++h) sm.atile[WIDE ? pwave : 0][2 * q + (wpiece >> 2)][(wpiece & 3) * 16 + wrow[h]] = awide[2 * q + h];
    };

    // running sums, in units of 4^p (sub-block p < 3) resp. 64 (p = 3) times the result
    v4f t[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int pp = 0; pp < 4; ++pp) t[mb][pp] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    // uniform zero-point in operand units, negated
    const float czu[4] = {-(float)p.zp_const, -(float)(p.zp_const * 4), -(float)(p.zp_const * 16),
                          -(float)((p.zp_const - 2) * 64)};

    if (s0 < s1) {
        // Same issue order as inside the loop (metadata first, then the ring), fenced, so that the
        // wait counts the compiler derives for the loop head hold on the entry path as well.
        fetch_meta(stepof(0) / GS, true, !FUSED && !ROWS);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < kDepth; ++i) issue(i, stepof(i), !ROWS);
        if (WIDE && !ROWS) fetch_wide(0);
        __builtin_amdgcn_sched_barrier(0);
    }

    if constexpr (ROWS) {
        // ---- the token rows are being quantised by the first p.M workgroups of this grid (rows_quantise_and_signal,
        // called by the kernel before this body): with the first weights on their way, wait until all rows are in
        // memory, then fetch what depends on them.  The wait is bounded: a workgroup that does not see the rows arrive
        // within spin_limit polls quantises them itself (same arithmetic, same bytes to the same places), so every wave
        // reaches the end of the kernel whatever happens to the others.
        rows_wait<kThreads>(p, &sm.red[0][0][0], &sm.last, spin_limit);
        load_sa();
        if (s0 < s1) {
#pragma unroll
            for (int i = 0; i < kDepth; ++i) issue_a(i, stepof(i));
            if (WIDE) fetch_wide(0);
        }
    }

    if constexpr (FUSED) {
        // ---- the workgroup quantises the token rows (every wave takes part, also one without steps),
        // while the loads above are on the way.  Pass 1: per-row absmax.  Pass 2: q = clip(rne(x / s)),
        // the per-group sums of q; IEEE binary32 division, as act_quant_kernel.
        FusedRows& fr = sm.fused;
        constexpr int tpg = GS * 8;  // threads per scale group (8 elements each)
        const int nvec = p.K / 8;
        const bool bf16 = p.x_bf16 != 0;
        auto load8 = [&](const uint16_t* src, float (&f)[8]) {
            const uint4 raw = *reinterpret_cast<const uint4*>(src);
            const uint32_t wds[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (bf16) {
                    f[2 * i] = __uint_as_float(wds[i] << 16);
                    f[2 * i + 1] = __uint_as_float(wds[i] & 0xffff0000u);
                } else {
                    f[2 * i] = half_bits_to_float((uint16_t)(wds[i] & 0xffffu));
                    f[2 * i + 1] = half_bits_to_float((uint16_t)(wds[i] >> 16));
                }
            }
        };
        auto quantise8 = [&](const float (&f)[8], float s, uint32_t& lo, uint32_t& hi) -> int {
            int sum = 0;
            lo = 0; hi = 0;
            const float inv_s = 1.0f / s;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float r = rne_quotient(f[i], s, inv_s);  // = rintf(f[i] / s), bit for bit
                r = fminf(fmaxf(r, -127.0f), 127.0f);
                const int qi = (int)r;
                sum += qi;
                if (i < 4) lo |= (uint32_t)(qi & 0xff) << (8 * i);
                else hi |= (uint32_t)(qi & 0xff) << (8 * (i - 4));
            }
            return sum;
        };
        constexpr int kKeep = 4;  // 8-element vectors of the row a thread keeps in registers between the passes
        if (J == 1 && nvec <= kKeep * kThreads) {
            // one token row (the decode case): the row is read once and stays in registers
            float f[kKeep][8];
            float amax = 0.0f;
#pragma unroll
            for (int it = 0; it < kKeep; ++it) {
                const int v = tid + it * kThreads;
                if (v < nvec) {
                    load8(p.x + (size_t)v * 8, f[it]);
#pragma unroll
                    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(f[it][i]));
                }
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
            if (lane == 0) fr.amax[pwave][0] = amax;
            __syncthreads();
            float a = fr.amax[0][0];
            for (int w = 1; w < NWP; ++w) a = fmaxf(a, fr.amax[w][0]);
            const float s = fmaxf(a, 1e-9f) / 127.0f;
            if (tid < kFusedMaxRows) fr.s_a[tid] = s;
#pragma unroll
            for (int it = 0; it < kKeep; ++it) {
                const int v = tid + it * kThreads;
                if (v < nvec) {  // whole groups of threads are in or out
                    uint32_t lo, hi;
                    int sum = quantise8(f[it], s, lo, hi);
                    *reinterpret_cast<uint2*>(&fr.q[(size_t)v * 8]) = make_uint2(lo, hi);
                    for (int off = 1; off < tpg; off <<= 1) sum += __shfl_xor(sum, off, 64);
                    if (v % tpg == 0) fr.rowsum[v / tpg] = v4i{sum, 0, 0, 0};
                }
            }
        } else {
            float amax[kFusedMaxRows] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (int v = tid; v < nvec; v += kThreads) {
#pragma unroll
                for (int m = 0; m < kFusedMaxRows; ++m) {
                    if (m < p.M) {
                        float f[8];
                        load8(p.x + (size_t)m * p.ldx + (size_t)v * 8, f);
#pragma unroll
                        for (int i = 0; i < 8; ++i) amax[m] = fmaxf(amax[m], fabsf(f[i]));
                    }
                }
            }
#pragma unroll
            for (int m = 0; m < kFusedMaxRows; ++m) {
#pragma unroll
                for (int off = 32; off >= 1; off >>= 1) amax[m] = fmaxf(amax[m], __shfl_xor(amax[m], off, 64));
                if (lane == 0) fr.amax[pwave][m] = amax[m];
            }
            __syncthreads();
            float srow[kFusedMaxRows];
#pragma unroll
            for (int m = 0; m < kFusedMaxRows; ++m) {
                float a = fr.amax[0][m];
                for (int w = 1; w < NWP; ++w) a = fmaxf(a, fr.amax[w][m]);
                srow[m] = fmaxf(a, 1e-9f) / 127.0f;
            }
            if (tid < kFusedMaxRows) fr.s_a[tid] = srow[tid];
            for (int v = tid; v < nvec; v += kThreads) {
                int sums[kFusedMaxRows] = {0, 0, 0, 0};
#pragma unroll
                for (int m = 0; m < kFusedMaxRows; ++m) {
                    if (m < p.M) {
                        float f[8];
                        load8(p.x + (size_t)m * p.ldx + (size_t)v * 8, f);
                        uint32_t lo, hi;
                        sums[m] = quantise8(f, srow[m], lo, hi);
                        *reinterpret_cast<uint2*>(&fr.q[(size_t)m * p.K + (size_t)v * 8]) = make_uint2(lo, hi);
                    }
                }
#pragma unroll
                for (int m = 0; m < kFusedMaxRows; ++m)
                    for (int off = 1; off < tpg; off <<= 1) sums[m] += __shfl_xor(sums[m], off, 64);
                if (v % tpg == 0) fr.rowsum[v / tpg] = v4i{sums[0], sums[1], sums[2], sums[3]};
            }
        }
        __syncthreads();
        if (NWK == 1) {
#pragma unroll
            for (int j = 0; j < J; ++j) sa[j] = fr.s_a[min(quad * 4 + j, kFusedMaxRows - 1)];
        } else {
#pragma unroll
            for (int i = 0; i < kOutPerThread; ++i) sa[i] = fr.s_a[min((tid + kThreads * i) >> 6, kFusedMaxRows - 1)];
        }
    }

    if (s0 < s1) {
        if (FUSED || ROWS) fetch_meta(stepof(0) / GS, false, true);  // the row sums of the first chunk, now that they exist

        v4i acc[MB][4];
        v4h sc;          // the group's four sub-block scales, kept in fp16: the drain's fma reads them as such

        for (int it = 0; it < len; it += kDepth) {
            const int gchunk = stepof(it) / GS;
            park_meta(gchunk);                        // this chunk's metadata: registers -> LDS
            fetch_meta(stepof(it + kDepth) / GS);     // next chunk's metadata: global -> registers
            __builtin_amdgcn_sched_barrier(0);

            {
                // zero-point term of the whole chunk: lane (col, quad) supplies token col / channel col of
                // group `quad` of the chunk; lanes whose quad is past the chunk's groups supply zero
                const int gi = quad % kGroupsPerChunk;
                const bool on = quad < kGroupsPerChunk;
                const v4h zs = *reinterpret_cast<const v4h*>(&meta.scale[gi][col][0]);
                float zb[4];
                if (ASYM) {
                    const uint32_t zraw = *reinterpret_cast<const uint32_t*>(&meta.zp[gi][col][0]);
                    zb[0] = -(float)(zraw & 0xffu) * (float)zs[0];
                    zb[1] = -4.0f * (float)((zraw >> 8) & 0xffu) * (float)zs[1];
                    zb[2] = -16.0f * (float)((zraw >> 16) & 0xffu) * (float)zs[2];
                    zb[3] = (128.0f - 64.0f * (float)(zraw >> 24)) * (float)zs[3];
                } else {
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp) zb[pp] = czu[pp] * (float)zs[pp];
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const int rsi = meta.rowsum[gi][mb * 16 + col];
                    const float rsf = on ? (float)rsi : 0.0f;
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp)
                        if (ASYM || pp < 3 || p.zp_const != 2)  // uniform zero-point 2: field 3 is already centred
                            t[mb][pp] = __builtin_amdgcn_mfma_f32_16x16x4f32(rsf, zb[pp], t[mb][pp], 0, 0, 0);
                }
            }

            if constexpr (FUSED) {
                const int8_t* qrow = &sm.fused.q[(size_t)min(col, M - 1) * p.K + quad * 16];
#pragma unroll
                for (int i = 0; i < kDepth; ++i)
                    aring[i][0] = *reinterpret_cast<const v4u*>(qrow + (size_t)stepof(it + i) * kStepK);
            }
            if (WIDE) {
                park_wide();                  // this chunk's fragments: registers -> LDS tile
                fetch_wide(it + kDepth);      // next chunk's: global -> registers
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < kDepth; ++i) aring[i][0] = sm.atile[WIDE ? pwave : 0][i][lane];
            }

#pragma unroll
            for (int i = 0; i < kDepth; ++i) {
                const int gi = i / GS;  // group within the chunk
                if (i % GS == 0) {
                    sc = *reinterpret_cast<const v4h*>(&meta.scale[gi][col][0]);
                }

#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    const v4i b = __builtin_bit_cast(v4i, wring[i] & (0x03030303u << (2 * pp)));
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)  // the first step of a group starts from C = 0 (inline constant)
                        acc[mb][pp] = mfma_i8_16x16x64(__builtin_bit_cast(v4i, aring[i][mb]), b,
                                                       (i % GS == 0) ? v4i{0, 0, 0, 0} : acc[mb][pp]);
                }
                // Refill the slot only now that its old contents are dead, so the load can land in the
                // same registers (no copies at the loop back-edge, and the wait before the next use is
                // for exactly this load).  The fences stop the scheduler from sinking the four steps'
                // loads to the end of the chunk, which would serialise load and compute.
                __builtin_amdgcn_sched_barrier(0);
                issue(i, stepof(it + i + kDepth));
                __builtin_amdgcn_sched_barrier(0);

                if (i % GS == GS - 1) {
                    const int g = gchunk + gi;
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                            for (int j = 0; j < J; ++j) {
                                t[mb][pp][j] = __builtin_fmaf((float)acc[mb][pp][j], (float)sc[pp], t[mb][pp][j]);
                                if constexpr (DUMP) {  // operand of field p: code * 4^p, or 64 * (code - 2) for p = 3
                                    if (g < g1)
                                        dump_group_sum(p, m0 + mb * 16 + quad * 4 + j, strip * kStripN + pp * 16 + col, g,
                                                       acc[mb][pp][j] >> (2 * pp), pp == 3 ? 2 : 0);
                                }
                            }
                }
            }
        }
    }

    constexpr float kUnscale[4] = {1.0f, 0.25f, 0.0625f, 0.015625f};  // 4^-p, exact

    if (NWK == 1) {  // the wave owns the strip's whole K range: store the D fragments directly
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    const int m = mb * 16 + quad * 4 + j;
                    const int n = strip * kStripN + pp * 16 + col;
                    if (m < M && n < p.N)
                        out[(size_t)m * p.ldo + n] = OutT::cast((t[mb][pp][j] * kUnscale[pp]) * sa[mb * J + j]);
                }
        return;
    }

    // ---- meet the workgroup's waves in LDS (the metadata area is dead once every wave is here)
    __syncthreads();
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int pp = 0; pp < 4; ++pp)
#pragma unroll
            for (int j = 0; j < J; ++j)
                if (J > 1 || quad == 0) sm.red[pwave][mb * 16 + quad * 4 + j][pp * 16 + col] = t[mb][pp][j] * kUnscale[pp];
    __syncthreads();

    if (p.split == 1) {
#pragma unroll
        for (int i = 0; i < kOutPerThread; ++i) {
            const int e = tid + kThreads * i;
            const int m = e >> 6, nl = e & 63;
            const int n = strip * kStripN + nl;
            if (e < kLive && m < M && n < p.N) {
                float v = sm.red[0][m][nl];
#pragma unroll
                for (int w = 1; w < NWP; ++w) v += sm.red[w][m][nl];
                out[(size_t)m * p.ldo + n] = OutT::cast(v * sa[i]);
            }
        }
        return;
    }

    // ---- split-K: publish this workgroup's partial tile, last arrival reduces all of them.
    // The partials move at system-coherent cache policy (write-through stores, loads around the
    // reader's L2), so no L2 write-back / invalidate fence is needed: a fence here costs about a
    // microsecond per workgroup and serialises on each XCD's L2.  They are plain memory instructions,
    // so the reduction keeps four splits' loads in flight at a time (one memory latency per four
    // splits instead of one per split).  s_waitcnt vmcnt(0) makes every lane's stores complete
    // before the arrival counter moves.
    constexpr int kCoherent = 17;  // sc0 | sc1
    const size_t tiles = (size_t)p.strips * mblocks;
    const __amdgpu_buffer_rsrc_t ws_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        p.ws_partial, 0, (int)min((size_t)p.split * tiles * kTile * 4, (size_t)0x7fffffff), 0x00020000);
    const uint32_t split_pitch = (uint32_t)(tiles * kTile * 4);
    const uint32_t tile_off = (uint32_t)tile_id * (kTile * 4);
#pragma unroll
    for (int i = 0; i < kOutPerThread; ++i) {
        const int e = tid + kThreads * i;
        if (e < kLive) {
            const int m = e >> 6, nl = e & 63;
            float v = sm.red[0][m][nl];
#pragma unroll
            for (int w = 1; w < NWP; ++w) v += sm.red[w][m][nl];
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), ws_rsrc, tile_off + e * 4, split * split_pitch, kCoherent);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned prev = __hip_atomic_fetch_add(p.ws_counter + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sm.last = (prev == (unsigned)(p.split - 1));
    }
    __syncthreads();
    if (!sm.last) return;
#pragma unroll
    for (int i = 0; i < kOutPerThread; ++i) {
        const int e = tid + kThreads * i;
        if (e >= kLive) break;
        const int m = e >> 6, nl = e & 63;
        const int n = strip * kStripN + nl;
        float v = 0.0f;
        for (int sp0 = 0; sp0 < p.split; sp0 += 4) {
            float part[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)  // past the last split: the last one again, not added
                part[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                              ws_rsrc, tile_off + e * 4, min(sp0 + u, p.split - 1) * split_pitch, kCoherent));
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (sp0 + u < p.split) v += part[u];
        }
        if (m < M && n < p.N) out[(size_t)m * p.ldo + n] = OutT::cast(v * sa[i]);
    }
    if (tid == 0) __hip_atomic_store(p.ws_counter + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int J, int GS, int NW, bool ASYM, bool DUMP, bool NT, bool WIDE, typename OutT>
__global__ __launch_bounds__(NW * 64) void skinny_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) SkinnySmem<NW, WIDE> sm;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: keeps ranges and bases in SGPRs
    skinny_body<J, GS, NW, NW, ASYM, DUMP, NT, WIDE, false, OutT>(p, blockIdx.x, blockIdx.y, blockIdx.z, wave, wave, sm);
}

// The same with the activation quantisation inside (at most four token rows, given as fp16 / bf16).
template <int J, int GS, int NW, bool ASYM, typename OutT>
__global__ __launch_bounds__(NW * 64) void skinny_fused_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) SkinnySmem<NW, false, true> sm;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    skinny_body<J, GS, NW, NW, ASYM, false, true, false, true, OutT>(p, blockIdx.x, blockIdx.y, 0, wave, wave, sm);
}

// The same with the token rows quantised by the grid's first workgroups (see rows_quantise_row): fp16 / bf16 rows in.
template <int GS, int NW, bool ASYM, bool NT, bool WIDE, typename OutT>
__global__ __launch_bounds__(NW * 64) void skinny_rows_kernel(const GemmParams p, const int spin_limit) {
    __shared__ __attribute__((aligned(16))) SkinnySmem<NW, WIDE> sm;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    rows_quantise_and_signal<NW * 64>(p, &sm.red[0][0][0]);
    skinny_body<4, GS, NW, NW, ASYM, false, NT, WIDE, false, OutT, true>(p, blockIdx.x, blockIdx.y, blockIdx.z, wave, wave, sm,
                                                                          spin_limit);
}

// ---------------------------------------------------------------------------------------------
// Grouped launch: several independent skinny GEMMs in one kernel.
//
// What bounds a decode GEMM on this chip is the per-CU vector memory path: every wave-wide load,
// hit or miss, takes a slot in it, and the slots not taken by weight lines coming from HBM are
// lost bandwidth.  With one activation load per weight load (the single-launch body above) half
// the slots carry activations.  Here the eight waves of a workgroup work on neighbouring strips
// of one problem over the same range of K and share its activations through LDS: per chunk of four
// steps the chunk's four 1 KiB A fragments are fetched once per sharing set, one step per wave,
// parked in a double-buffered LDS area, and read back by every wave of the set with ds_read_b128
// (lane l of a fragment sits at 16*l: conflict-free).  One barrier per chunk keeps the set in step.
//
// Workgroup = NK k-parts x NS strips (NK * NS = 8 waves).  Short reductions use NK = 1 (nothing to
// reduce, each wave stores its own D fragments); long ones split K over 2 or 4 parts that meet in
// LDS, so that every wave of the launch streams a run of comparable length (48..96 steps) and its
// start-up and wind-down cost is spread over enough steps.
constexpr int kGroupedWaves = kGroupedWavesPerWg;  // w2a8_common.h: the host sizes the grid with it
constexpr int kShareRows = 8;  // token rows from which activations are shared through LDS

// Per-group metadata is handled in blocks of kBlockGroups groups: one block's scales, zero-points
// and activation row sums are fetched with three or four wave-wide loads (instead of a few small
// loads every chunk), parked in a wave-private LDS area, and the block's whole zero-point term goes
// through four fp32 MFMAs per sub-block at the block's start.
constexpr int kBlockGroups = 16;

struct GroupedMeta {
    uint16_t scale[kBlockGroups][16][4];  // [group of the block][col][sub-block]   2 KiB
    int32_t rowsum[kBlockGroups][16];     //                                        1 KiB
    uint8_t zp[kBlockGroups][16][4];      //                                        1 KiB
};

struct GroupedSmem {
    union {
        GroupedMeta meta[kGroupedWaves];
        float red[kGroupedWaves][16][kStripN + 1];
    };
    v4u abuf[4][2][kDepth][64];  // [k-part][parity][step of the chunk][lane]
    int last;                    // split-K: this workgroup was the last of its unit to arrive
};

// SPLIT: the workgroup owns only the steps of K-split `split` (one-problem launches: grid.y splits,
// partial tiles meet in the caller's workspace, the last workgroup of a unit to arrive adds them
// up in split order and stores).
// DUMP: verification instantiation, as in skinny_body: the int32 group sums are also written out, nothing else changes.
template <int J, int GS, int NK, bool SHARE, bool ASYM, bool NT, bool SPLIT, typename OutT, bool DUMP = false>
__device__ __forceinline__ void shared_body(const GemmParams& p, const int unit, const int mblk, const int wave,
                                            GroupedSmem& sm, const int split = 0) {
    constexpr int NS = kGroupedWaves / NK;               // waves (strips) sharing one activation stream
    constexpr int NL = NS >= kDepth ? 1 : kDepth / NS;   // A fragments a loading wave fetches per chunk
    constexpr int kThreads = kGroupedWaves * 64;
    constexpr int kGroupsPerChunk = kDepth / GS;         // GS = 4 is one group per chunk
    constexpr int kChunksPerBlock = kBlockGroups / kGroupsPerChunk;
    constexpr int kLive = (J == 1 ? 1 : 16) * kStripN;   // elements of a strip's tile that can hold real tokens
    constexpr int kOutPerThread = (NS * kLive + kThreads - 1) / kThreads;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int col = lane & 15, quad = lane >> 4;
    const int kpart = wave / NS, swave = wave % NS;
    const int strip_raw = unit * NS + swave;
    const bool active = strip_raw < p.strips;       // a padding wave streams a valid strip but stores nothing
    const int strip = min(strip_raw, p.strips - 1);
    GroupedMeta& meta = sm.meta[wave];

    // this row block's view of the per-token operands
    const int m0 = mblk * 16;
    const int M = min(16, p.M - m0);
    const int8_t* const qp = p.q + (size_t)m0 * p.ldq;
    const float* const sap = p.s_a + m0;
    const int32_t* const rsp = p.rowsum + m0;
    const int ldr = p.ldr - m0;
    uint16_t* const out = reinterpret_cast<uint16_t*>(p.out) + (size_t)m0 * p.ldo;

    // token scales for the epilogue, fetched first
    float sa[NK == 1 && !SPLIT ? J : kOutPerThread];
    if (NK == 1 && !SPLIT) {
#pragma unroll
        for (int j = 0; j < J; ++j) sa[j] = sap[min(quad * 4 + j, M - 1)];
    } else {
#pragma unroll
        for (int i = 0; i < kOutPerThread; ++i) sa[i] = sap[min(((tid + kThreads * i) % kLive) >> 6, M - 1)];
    }

    // K range of this k-part in whole chunks; every part runs the same number of chunk iterations
    // (the barrier count must agree), a shorter last part idles through the extra ones with zero scales.
    const int wg_s0 = SPLIT ? min(split * p.groups_per_split, p.G) * GS : 0;
    const int wg_s1 = SPLIT ? min((split + 1) * p.groups_per_split, p.G) * GS : p.steps;
    const int chunks = (wg_s1 - wg_s0 + kDepth - 1) / kDepth;
    const int per_part = (chunks + NK - 1) / NK;
    const int s0 = min(wg_s0 + kpart * per_part * kDepth, wg_s1);
    const int s1 = min(s0 + per_part * kDepth, wg_s1);
    const int g0 = s0 / GS, g1 = s1 / GS;
    const int len = s1 - s0;
    auto stepof = [&](int it) { return s0 + max(min(it, len - 1), 0); };

    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(p.w_r), 0, (int)weight_bytes(p.strips, p.steps), 0x00020000);
    const __amdgpu_buffer_rsrc_t q_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t*>(qp), 0, (int)((size_t)(M - 1) * p.ldq + p.K), 0x00020000);
    const uint32_t wstride = (uint32_t)p.strips * (kRunSteps * kUnitBytes);  // bytes between consecutive runs of a strip
    const uint32_t wbase = (uint32_t)strip * (kRunSteps * kUnitBytes);
    const uint32_t wlane = lane * 16;
    const uint32_t aoff = (uint32_t)min(col, M - 1) * (uint32_t)p.ldq + quad * 16;

    // ---- metadata of one block of groups: global -> registers (a block ahead) -> LDS.
    // Groups past the part's end are clamped onto its last group for the loads and get zero scales
    // when parked, so they add nothing.
    v4i m_scale[2], m_zp, m_rs;
    auto fetch_meta = [&](int gfirst) {
#pragma unroll
        for (int n = 0; n < 2; ++n) {  // scales: 16 groups x 128 B: lane -> group 8n + lane/8
            const size_t sgi = (size_t)max(min(gfirst + n * 8 + (lane >> 3), g1 - 1), 0) * p.strips + strip;
            const v4i* sp = reinterpret_cast<const v4i*>(reinterpret_cast<const char*>(p.s_r) + sgi * 128 + (lane & 7) * 16);
            m_scale[n] = NT ? __builtin_nontemporal_load(sp) : *sp;
        }
        const int gq = max(min(gfirst + (lane >> 2), g1 - 1), 0);  // row sums / zero-points: lane -> group lane/4
        if (ASYM)
            m_zp = *reinterpret_cast<const v4i*>(reinterpret_cast<const char*>(p.zp_r) +
                                                 ((size_t)gq * p.strips + strip) * 64 + (lane & 3) * 16);
        m_rs = *reinterpret_cast<const v4i*>(rsp + (size_t)gq * p.ldr + min((lane & 3) * 4, ldr - 4));
    };
    auto park_meta = [&](int gfirst) {
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            if (gfirst + n * 8 + (lane >> 3) >= g1) m_scale[n] = v4i{0, 0, 0, 0};
            *reinterpret_cast<v4i*>(reinterpret_cast<char*>(&meta.scale[0][0][0]) + n * 1024 + lane * 16) = m_scale[n];
        }
        if (ASYM) *reinterpret_cast<v4i*>(reinterpret_cast<char*>(&meta.zp[0][0][0]) + lane * 16) = m_zp;
        *reinterpret_cast<v4i*>(&meta.rowsum[lane >> 2][(lane & 3) * 4]) = m_rs;
    };

    // ---- weights: register ring.  Activations: with few token rows a fragment is only a line or two
    // and each wave keeps its own register ring of them (SHARE = false: no LDS hand-over, no
    // barrier); otherwise they are fetched once per sharing set and handed round through LDS.
    v4u wring[kDepth];
    auto issue_w = [&](int slot, int step) {
        wring[slot] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wlane, (step / kRunSteps) * wstride + (step % kRunSteps) * kUnitBytes + wbase,
                                                            NT ? kStreamOnce : 0);
    };
    v4u aring[kDepth];
    auto issue_a = [&](int slot, int step) {
        if (!SHARE) aring[slot] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, aoff, step * kStepK, 0);
    };
    // Shared fragments are fetched two steps wide so that every load touches whole 128-byte lines of
    // the row-major activations: fragment f of a chunk = (step pair f / 2, row half f % 2); lane l
    // reads row 8 * half + l / 8, 16-byte piece l % 8 of the pair's 128 bytes, and parks it where the
    // MFMA operand order wants it (step 2 * pair + piece / 4, lane (piece % 4) * 16 + row).
    const bool loader = SHARE && swave < kDepth;  // wave-uniform
    v4u areg[NL];
    const int frow[2] = {lane >> 3, 8 + (lane >> 3)};
    const uint32_t fpiece = lane & 7;
    auto fetch_a = [&](int it) {  // this wave's share of the chunk that starts at iteration `it`
        if (loader) {
#pragma unroll
            for (int n = 0; n < NL; ++n) {
                const int f = swave + n * NS;
                areg[n] = __builtin_amdgcn_raw_buffer_load_b128(
                    q_rsrc, (uint32_t)min(frow[f & 1], M - 1) * (uint32_t)p.ldq + fpiece * 16, stepof(it + 2 * (f >> 1)) * kStepK, 0);
            }
        }
    };
    auto park_a = [&](int parity) {
        if (loader) {
#pragma unroll
            for (int n = 0; n < NL; ++n) {
                const int f = swave + n * NS;
                sm.abuf[kpart][parity][2 * (f >> 1) + (fpiece >> 2)][(fpiece & 3) * 16 + frow[f & 1]] = areg[n];
            }
        }
    };

    // running sums, in units of 4^p (sub-block p < 3) resp. 64 (p = 3) times the result
    v4f t[4];
#pragma unroll
    for (int pp = 0; pp < 4; ++pp) t[pp] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    const float czu[4] = {-(float)p.zp_const, -(float)(p.zp_const * 4), -(float)(p.zp_const * 16),
                          -(float)((p.zp_const - 2) * 64)};

    fetch_meta(g0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < kDepth; ++i) {
        issue_w(i, stepof(i));
        issue_a(i, stepof(i));
    }
    if (SHARE) {
        fetch_a(0);
        __builtin_amdgcn_sched_barrier(0);
        park_a(0);
        fetch_a(kDepth);
    }
    __builtin_amdgcn_sched_barrier(0);

    v4i acc[4];
    v4h sc;
    const int blocks = (per_part + kChunksPerBlock - 1) / kChunksPerBlock;
    for (int blk = 0; blk < blocks; ++blk) {
        const int gblock = g0 + blk * kBlockGroups;
        park_meta(gblock);                       // this block's metadata: registers -> LDS
        fetch_meta(gblock + kBlockGroups);       // next block's: global -> registers
        __builtin_amdgcn_sched_barrier(0);

        // zero-point term of the whole block: lane (col, quad) supplies token col / channel col of
        // group 4b + quad; -zpe * scale * rowsum summed over four groups per fp32 MFMA
#pragma unroll
        for (int b = 0; b < kBlockGroups / 4; ++b) {
            const int gi = 4 * b + quad;
            const v4h zs = *reinterpret_cast<const v4h*>(&meta.scale[gi][col][0]);
            float zb[4];
            if (ASYM) {
                const uint32_t zraw = *reinterpret_cast<const uint32_t*>(&meta.zp[gi][col][0]);
                zb[0] = -(float)(zraw & 0xffu) * (float)zs[0];
                zb[1] = -4.0f * (float)((zraw >> 8) & 0xffu) * (float)zs[1];
                zb[2] = -16.0f * (float)((zraw >> 16) & 0xffu) * (float)zs[2];
                zb[3] = (128.0f - 64.0f * (float)(zraw >> 24)) * (float)zs[3];
            } else {
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) zb[pp] = czu[pp] * (float)zs[pp];
            }
            const float rsf = (float)meta.rowsum[gi][col];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp)
                if (ASYM || pp < 3 || p.zp_const != 2)  // uniform zero-point 2: field 3 is already centred
                    t[pp] = __builtin_amdgcn_mfma_f32_16x16x4f32(rsf, zb[pp], t[pp], 0, 0, 0);
        }

        const int c_end = min(per_part - blk * kChunksPerBlock, kChunksPerBlock);
        for (int cc = 0; cc < c_end; ++cc) {
            const int c = blk * kChunksPerBlock + cc;
            const int it = c * kDepth;
            if (SHARE) {
                __syncthreads();             // chunk c's fragments are in place; chunk c-1's are no longer read
                park_a((c + 1) & 1);         // chunk c+1's fragments: registers -> LDS
                fetch_a(it + 2 * kDepth);    // chunk c+2's: global -> registers
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < kDepth; ++i) aring[i] = sm.abuf[kpart][c & 1][i][lane];
            }
            const uint16_t* const scp = &meta.scale[cc * kGroupsPerChunk][col][0];  // this chunk's groups
#pragma unroll
            for (int i = 0; i < kDepth; ++i) {
                if (i % GS == 0) sc = *reinterpret_cast<const v4h*>(scp + (i / GS) * 64);
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    const v4i b = __builtin_bit_cast(v4i, wring[i] & (0x03030303u << (2 * pp)));
                    acc[pp] = mfma_i8_16x16x64(__builtin_bit_cast(v4i, aring[i]), b, (i % GS == 0) ? v4i{0, 0, 0, 0} : acc[pp]);
                }
                // refill the slot only now that its old contents are dead (see skinny_body)
                __builtin_amdgcn_sched_barrier(0);
                issue_w(i, stepof(it + i + kDepth));
                issue_a(i, stepof(it + i + kDepth));
                __builtin_amdgcn_sched_barrier(0);
                if (i % GS == GS - 1) {
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                        for (int j = 0; j < J; ++j) {
                            t[pp][j] = __builtin_fmaf((float)acc[pp][j], (float)sc[pp], t[pp][j]);
                            if constexpr (DUMP) {
                                const int g = stepof(it + i) / GS;
                                if (active && it + i < len)
                                    dump_group_sum(p, m0 + quad * 4 + j, strip * kStripN + pp * 16 + col, g,
                                                   acc[pp][j] >> (2 * pp), pp == 3 ? 2 : 0);
                            }
                        }
                }
            }
        }
    }

    constexpr float kUnscale[4] = {1.0f, 0.25f, 0.0625f, 0.015625f};  // 4^-p, exact
    if (NK == 1 && !SPLIT) {
        if (active) {
#pragma unroll
            for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    const int m = quad * 4 + j;
                    const int n = strip * kStripN + pp * 16 + col;
                    if (m < M && n < p.N) out[(size_t)m * p.ldo + n] = OutT::cast((t[pp][j] * kUnscale[pp]) * sa[j]);
                }
        }
        return;
    }

    // ---- the k-parts of each strip meet in LDS (the metadata area is dead once every wave is here)
    __syncthreads();
#pragma unroll
    for (int pp = 0; pp < 4; ++pp)
#pragma unroll
        for (int j = 0; j < J; ++j)
            if (J > 1 || quad == 0) sm.red[wave][quad * 4 + j][pp * 16 + col] = t[pp][j] * kUnscale[pp];
    __syncthreads();
    if (!SPLIT) {
#pragma unroll
        for (int i = 0; i < kOutPerThread; ++i) {
            const int e = tid + kThreads * i;
            const int sidx = e / kLive, w = e % kLive;
            const int m = w >> 6, nl = w & 63;
            const int so = unit * NS + sidx;
            const int n = so * kStripN + nl;
            if (sidx < NS && so < p.strips && m < M && n < p.N) {
                float v = sm.red[sidx][m][nl];
#pragma unroll
                for (int kp = 1; kp < NK; ++kp) v += sm.red[kp * NS + sidx][m][nl];
                out[(size_t)m * p.ldo + n] = OutT::cast(v * sa[i]);
            }
        }
        return;
    }

    // ---- split-K: publish this workgroup's partial tiles (one 16 x 64 fp32 tile per strip and row
    // block, the one-problem kernel's workspace layout), count arrivals per unit, the last one reduces
    // in split order.  Partials move at system-coherent cache policy (write-through stores, loads
    // around the reader's L2), a split's loads all in flight together.
    constexpr int kCoherent = 17;  // sc0 | sc1
    constexpr int kTile = 16 * kStripN;
    const int mblocks = (p.M + 15) >> 4;
    const int n_split = p.split;
    const size_t tiles = (size_t)p.strips * mblocks;
    const __amdgpu_buffer_rsrc_t ws_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        p.ws_partial, 0, (int)min((size_t)n_split * tiles * kTile * 4, (size_t)0x7fffffff), 0x00020000);
    const uint32_t split_pitch = (uint32_t)(tiles * kTile * 4);
    uint32_t eoff[kOutPerThread];
    bool eon[kOutPerThread];
#pragma unroll
    for (int i = 0; i < kOutPerThread; ++i) {
        const int e = tid + kThreads * i;
        const int sidx = e / kLive, w = e % kLive;
        const int so = unit * NS + sidx;
        eon[i] = sidx < NS && so < p.strips;
        eoff[i] = (uint32_t)(((size_t)min(so, p.strips - 1) * mblocks + mblk) * kTile + w) * 4;
    }
#pragma unroll
    for (int i = 0; i < kOutPerThread; ++i) {
        const int e = tid + kThreads * i;
        const int sidx = min(e / kLive, NS - 1), w = e % kLive;
        float v = sm.red[sidx][w >> 6][w & 63];
#pragma unroll
        for (int kp = 1; kp < NK; ++kp) v += sm.red[kp * NS + sidx][w >> 6][w & 63];
        if (eon[i]) __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), ws_rsrc, eoff[i], split * split_pitch, kCoherent);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int counter_id = (unit * NS) * mblocks + mblk;  // the unit's first strip stands for the unit
    if (tid == 0) {
        const unsigned prev = __hip_atomic_fetch_add(p.ws_counter + counter_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sm.last = (prev == (unsigned)(n_split - 1));
    }
    __syncthreads();
    if (!sm.last) return;
    float v[kOutPerThread];
#pragma unroll
    for (int i = 0; i < kOutPerThread; ++i) v[i] = 0.0f;
    for (int sp = 0; sp < n_split; ++sp) {
        float part[kOutPerThread];
#pragma unroll
        for (int i = 0; i < kOutPerThread; ++i)
            part[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ws_rsrc, eoff[i], sp * split_pitch, kCoherent));
#pragma unroll
        for (int i = 0; i < kOutPerThread; ++i) v[i] += part[i];
    }
#pragma unroll
    for (int i = 0; i < kOutPerThread; ++i) {
        const int e = tid + kThreads * i;
        const int sidx = e / kLive, w = e % kLive;
        const int m = w >> 6, nl = w & 63;
        const int n = (unit * NS + sidx) * kStripN + nl;
        if (eon[i] && m < M && n < p.N) out[(size_t)m * p.ldo + n] = OutT::cast(v[i] * sa[i]);
    }
    if (tid == 0) __hip_atomic_store(p.ws_counter + counter_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Workgroup ids are cut into runs, one run per problem.  Within a problem, workgroups come in sets
// of eight per 16-row token block: consecutive workgroup ids go to different XCDs, so the two row
// blocks of a set of strips, eight ids apart, share an XCD and its L2 (the second read of the
// weights hits there).  Which unit of a set an XCD takes is the host's choice per problem
// (xcd_slots): the last, partial set of every problem leaves some XCDs without work, and the host
// deals those gaps out evenly, because an XCD's 32 CUs can only stream so much.  All problems share the group size, the zero-point mode and the output
// type.  The problem table travels in the kernel arguments.
template <int GS, bool ASYM, typename OutT, bool DUMP = false>
__global__ __launch_bounds__(kGroupedWaves * 64, 4) void skinny_grouped_kernel(const GroupedParams gp) {
    __shared__ __attribute__((aligned(16))) GroupedSmem sm;
    const int wg = blockIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // problem index = number of run boundaries at or below this workgroup id: one lane per boundary,
    // one ballot (a serial walk of the table costs a scalar load latency per problem)
    const int bl = min((int)(threadIdx.x & 63), kMaxGroup - 1);
    const bool past = bl + 1 < gp.count && wg >= gp.wg_begin[bl + 1];
    const int i = __builtin_amdgcn_readfirstlane(__builtin_popcountll(__ballot(past)));
    const GemmParams& p = gp.prob[i];
    const int local = wg - gp.wg_begin[i];
    const int mblocks = (p.M + 15) >> 4;
    const int mblk = (local >> 3) % mblocks;
    const int unit = (local / (8 * mblocks)) * 8 + (int)((gp.xcd_slots[i] >> (3 * (local & 7))) & 7u);  // set of strips
    const int nk = gp.kparts[i];
    if (unit * (kGroupedWaves / nk) >= p.strips) return;  // padding workgroup (uniform)
    // activations go through LDS once a fragment spans enough cache lines to be worth a barrier
    const int mrows = min(16, p.M - mblk * 16);
    if (nk == 1) {
        if (p.M == 1) shared_body<1, GS, 1, false, ASYM, true, false, OutT, DUMP>(p, unit, mblk, wave, sm);
        else if (mrows < kShareRows) shared_body<4, GS, 1, false, ASYM, true, false, OutT, DUMP>(p, unit, mblk, wave, sm);
        else if (mblocks == 1) shared_body<4, GS, 1, true, ASYM, true, false, OutT, DUMP>(p, unit, mblk, wave, sm);
        else shared_body<4, GS, 1, true, ASYM, false, false, OutT, DUMP>(p, unit, mblk, wave, sm);
    } else if (nk == 2) {
        if (p.M == 1) shared_body<1, GS, 2, false, ASYM, true, false, OutT, DUMP>(p, unit, mblk, wave, sm);
        else if (mrows < kShareRows) shared_body<4, GS, 2, false, ASYM, true, false, OutT, DUMP>(p, unit, mblk, wave, sm);
        else if (mblocks == 1) shared_body<4, GS, 2, true, ASYM, true, false, OutT, DUMP>(p, unit, mblk, wave, sm);
        else shared_body<4, GS, 2, true, ASYM, false, false, OutT, DUMP>(p, unit, mblk, wave, sm);
    } else if (nk == 4) {
        if (p.M == 1) shared_body<1, GS, 4, false, ASYM, true, false, OutT, DUMP>(p, unit, mblk, wave, sm);
        else if (mrows < kShareRows) shared_body<4, GS, 4, false, ASYM, true, false, OutT, DUMP>(p, unit, mblk, wave, sm);
        else if (mblocks == 1) shared_body<4, GS, 4, true, ASYM, true, false, OutT, DUMP>(p, unit, mblk, wave, sm);
        else shared_body<4, GS, 4, true, ASYM, false, false, OutT, DUMP>(p, unit, mblk, wave, sm);
    } else {  // eight k-parts of one strip (small launches of long reductions): nobody to share activations with
        if (p.M == 1) shared_body<1, GS, 8, false, ASYM, true, false, OutT, DUMP>(p, unit, mblk, wave, sm);
        else if (mblocks == 1) shared_body<4, GS, 8, false, ASYM, true, false, OutT, DUMP>(p, unit, mblk, wave, sm);
        else shared_body<4, GS, 8, false, ASYM, false, false, OutT, DUMP>(p, unit, mblk, wave, sm);
    }
}

// One problem through the shared-activation body.  For 17..32 token rows on matrices big
// enough to be bound by bandwidth (measured 8..27 % faster than one strip per workgroup there), for the problems of
// 33..256 rows the host predicts it fastest for, and with four k-parts x two strips for 12..16 rows on very wide
// matrices (more strips than the CUs take as one-strip workgroups at a time).
// The grid is one-dimensional and placed by xcd_place: a set is a (unit, K split) pair, its members are its row
// blocks.  (Dealing whole units out instead, K splits in blockIdx.y, left 5120 channels = 20 units at 96 rows in two
// splits with 36 workgroups on four XCDs of 32 CUs and 24 on the others: 30.6 us, now 22.3 us.)
template <int GS, int NK, bool ASYM, typename OutT, bool DUMP = false>
__global__ __launch_bounds__(kGroupedWaves * 64, 4) void skinny_shared_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) GroupedSmem sm;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int mblocks = (p.M + 15) >> 4;
    constexpr int kPerUnit = kGroupedWaves / NK;
    const int units = (p.strips + kPerUnit - 1) / kPerUnit;
    struct { int unit, mblk, split; } at;
    int pair;
    if (!xcd_place(blockIdx.x, units * (p.split > 1 ? p.split : 1), mblocks, pair, at.mblk)) return;  // (uniform)
    at.unit = pair % units;
    at.split = pair / units;
    if (mblocks == 1) {  // one row block: every weight byte is used once (loads marked stream-once)
        if (p.split > 1) shared_body<4, GS, NK, true, ASYM, true, true, OutT, DUMP>(p, at.unit, at.mblk, wave, sm, at.split);
        else shared_body<4, GS, NK, true, ASYM, true, false, OutT, DUMP>(p, at.unit, at.mblk, wave, sm);
        return;
    }
    // several row blocks: all but the first read of the weights come from L2
    if (p.split > 1) shared_body<4, GS, NK, true, ASYM, false, true, OutT, DUMP>(p, at.unit, at.mblk, wave, sm, at.split);
    else shared_body<4, GS, NK, true, ASYM, false, false, OutT, DUMP>(p, at.unit, at.mblk, wave, sm);
}

template <int GS, int NK, bool DUMP>
static void launch_shared_nk(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream) {
    const int per_unit = kGroupedWaves / NK;
    const int units = (p.strips + per_unit - 1) / per_unit;
    const dim3 grid(xcd_grid(units * (p.split > 1 ? p.split : 1), (p.M + 15) / 16)), block(kGroupedWaves * 64);
    if (asym) {
        if (out_bf16) skinny_shared_kernel<GS, NK, true, OutBF16, DUMP><<<grid, block, 0, stream>>>(p);
        else skinny_shared_kernel<GS, NK, true, OutF16, DUMP><<<grid, block, 0, stream>>>(p);
    } else {
        if (out_bf16) skinny_shared_kernel<GS, NK, false, OutBF16, DUMP><<<grid, block, 0, stream>>>(p);
        else skinny_shared_kernel<GS, NK, false, OutF16, DUMP><<<grid, block, 0, stream>>>(p);
    }
}

// kparts: k-parts per workgroup, kSharedParts (four strips share an activation stream) or twice that (two strips)
template <bool DUMP>
static hipError_t launch_skinny_shared_impl(const GemmParams& p, int gs, int kparts, bool asym, bool out_bf16, hipStream_t stream) {
    if (kparts == kSharedParts) {
        if (gs == 1) launch_shared_nk<1, kSharedParts, DUMP>(p, asym, out_bf16, stream);
        else if (gs == 2) launch_shared_nk<2, kSharedParts, DUMP>(p, asym, out_bf16, stream);
        else launch_shared_nk<4, kSharedParts, DUMP>(p, asym, out_bf16, stream);
    } else {
        if (gs == 1) launch_shared_nk<1, 2 * kSharedParts, DUMP>(p, asym, out_bf16, stream);
        else if (gs == 2) launch_shared_nk<2, 2 * kSharedParts, DUMP>(p, asym, out_bf16, stream);
        else launch_shared_nk<4, 2 * kSharedParts, DUMP>(p, asym, out_bf16, stream);
    }
    return hipGetLastError();
}

template <int J, int GS, int NW, bool ASYM, bool DUMP, bool NT, bool WIDE>
static void launch_out(const GemmParams& p, bool out_bf16, hipStream_t stream) {
    const dim3 grid(p.strips, p.split, (p.M + 15) / 16), block(NW * 64);
    if (out_bf16)
        skinny_kernel<J, GS, NW, ASYM, DUMP, NT, WIDE, OutBF16><<<grid, block, 0, stream>>>(p);
    else
        skinny_kernel<J, GS, NW, ASYM, DUMP, NT, WIDE, OutF16><<<grid, block, 0, stream>>>(p);
}

template <int J, int GS, int NW, bool DUMP, bool NT, bool WIDE>
static void launch_zm(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream) {
    if (asym) launch_out<J, GS, NW, true, DUMP, NT, WIDE>(p, out_bf16, stream);
    else launch_out<J, GS, NW, false, DUMP, NT, WIDE>(p, out_bf16, stream);
}

// Two-steps-wide activation fetch pays from 16 token rows on when the reduction is long (measured:
// 4..15 % faster at K >= 8192, M = 16..32; the LDS turn costs a short problem more than the saved
// cache-line slots bring) and the launch puts enough waves on a CU to hide that turn: with four waves or fewer per
// CU (224 or 256 strips, unsplit, four waves each) it is 17..19 % slower (14336 x 8192 at 16 rows: 12.4 against
// 10.1 us; 16384 x 16384: 21.9 against 18.1 us), with seven or more 4..5 % faster.
constexpr int kWideRows = 16, kWideK = 8192, kWideWaves = 1536;

template <int GS, int NW, bool DUMP>
static void launch_rows(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream) {
    const bool wide = p.M >= kWideRows && p.K >= kWideK && p.strips * max(p.split, 1) * NW * ((p.M + 15) / 16) >= kWideWaves;
    if (p.M == 1) launch_zm<1, GS, NW, DUMP, true, false>(p, asym, out_bf16, stream);
    else if (p.M <= 16 && !wide) launch_zm<4, GS, NW, DUMP, true, false>(p, asym, out_bf16, stream);
    else if (p.M <= 16) launch_zm<4, GS, NW, DUMP, true, true>(p, asym, out_bf16, stream);
    // two row blocks share the weights in L2
    else if (!wide) launch_zm<4, GS, NW, DUMP, false, false>(p, asym, out_bf16, stream);
    else launch_zm<4, GS, NW, DUMP, false, true>(p, asym, out_bf16, stream);
}

// A verification call (DUMP) picks exactly the instantiation the production call would: same rows per lane, waves per
// workgroup, cache policy and activation fetch.
template <int GS, bool DUMP>
static void launch_nw(const GemmParams& p, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    if (waves >= 16) launch_rows<GS, 16, DUMP>(p, asym, out_bf16, stream);
    else if (waves >= 8) launch_rows<GS, 8, DUMP>(p, asym, out_bf16, stream);
    else launch_rows<GS, 4, DUMP>(p, asym, out_bf16, stream);
}

template <int GS, bool ASYM, bool DUMP>
static void launch_grouped_out(const GroupedParams& gp, int total_wgs, bool out_bf16, hipStream_t stream) {
    if (out_bf16) skinny_grouped_kernel<GS, ASYM, OutBF16, DUMP><<<dim3(total_wgs), dim3(kGroupedWaves * 64), 0, stream>>>(gp);
    else skinny_grouped_kernel<GS, ASYM, OutF16, DUMP><<<dim3(total_wgs), dim3(kGroupedWaves * 64), 0, stream>>>(gp);
}

template <int GS, bool DUMP>
static void launch_grouped_zm(const GroupedParams& gp, int total_wgs, bool asym, bool out_bf16, hipStream_t stream) {
    if (asym) launch_grouped_out<GS, true, DUMP>(gp, total_wgs, out_bf16, stream);
    else launch_grouped_out<GS, false, DUMP>(gp, total_wgs, out_bf16, stream);
}

template <bool DUMP>
static hipError_t launch_skinny_grouped_impl(const GroupedParams& gp, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    const int total_wgs = gp.wg_begin[gp.count];
    if (gs == 1) launch_grouped_zm<1, DUMP>(gp, total_wgs, asym, out_bf16, stream);
    else if (gs == 2) launch_grouped_zm<2, DUMP>(gp, total_wgs, asym, out_bf16, stream);
    else launch_grouped_zm<4, DUMP>(gp, total_wgs, asym, out_bf16, stream);
    return hipGetLastError();
}

template <bool DUMP>
static hipError_t launch_skinny_impl(const GemmParams& p, int gs, int waves, bool asym, bool out_bf16, hipStream_t stream) {
    if (gs == 1) launch_nw<1, DUMP>(p, waves, asym, out_bf16, stream);
    else if (gs == 2) launch_nw<2, DUMP>(p, waves, asym, out_bf16, stream);
    else launch_nw<4, DUMP>(p, waves, asym, out_bf16, stream);
    return hipGetLastError();
}


}  // namespace w2a8
