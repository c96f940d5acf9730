// The W2A8 GEMM for 33..256 token rows on gfx950: between the weight-streaming kernels for a few rows (which pass over
// the weights once per block of 16 rows) and the tiled kernel (whose 64 x 256 tiles are too few, or need K split over
// many workgroups, while the rows are this few).
//
// Workgroup = four strips of 64 channels (one per wave) x up to six blocks of 16 token rows (MB; more than 96 rows run
// as two or three row parts of equal height, blockIdx.z) x a range of K (blockIdx.y).
//  * Weights: a wave streams the 1 KiB units of its own strip straight into a register ring (buffer loads, scalar
//    offsets), unpacks a unit ONCE - high bit of every field flipped, field moved to the top of its byte: bytes
//    64 * (code - 2), no row-sum term for the symmetric levels - and uses the operand for all MB row blocks.
//  * Activations are shared by the four waves: the fragments (16 rows x 64 k, 1 KiB, MFMA operand order) of a piece
//    of P = min(2, steps per group) steps go from global memory straight into a ring of four slots in LDS (LDS-direct
//    loads: no registers held while in flight), every wave fetching a quarter of them, three pieces ahead; one
//    barrier per piece says that a piece has landed and that the slot read before it is free again.  A fragment is
//    read back with one conflict-free ds_read_b128 right before its MFMAs, the next one while those run.
//  * A piece's accumulators (one set of 4 x 4 per row block, two sets alternating) are drained into fp32 running sums
//    with the group's scale while the next row block's MFMAs run.  A group of 256 is two pieces with the same scale.
//  * Zero-points other than 2 (per-group, or the upstream quantiser's 1) add (2 - zp) * scale * rowsum per group
//    through fp32 MFMAs before the main loop, as in the tiled kernel.
//  * split > 1: the workgroups of a strip set publish their running sums in the workspace (one fp32 tile of 16 x 64
//    per strip and row block, as many as the one-strip kernel uses; a lane's four rows of a 16-channel block are
//    16 consecutive bytes) and the last one to arrive adds them up in split order.
// The LDS-direct loads are waited for with counts written here (the compiler's own waits cover the register loads; it
// counts the LDS-direct loads as memory operations but leaves the LDS reads behind them alone), so the order in which
// a wave issues its memory operations is fixed by scheduling fences and the prologue issues them in the order of
// the steady state.
#pragma once
#include <type_traits>

#include "w2a8_launch.h"

namespace w2a8 {

// ZP: some zero-point differs from 2 (per-group zero-points, or a uniform one other than 2)
// DUMP: verification instantiation: the exact int32 group sums are also written out; nothing else changes.
template <int MB, int GS, bool ZP, typename OutT, bool DUMP>
__device__ __forceinline__ void mid_body(const GemmParams& p) {
    constexpr int P = mid::piece_steps(GS);          // steps per piece
    constexpr int NW = mid::kWaves;
    constexpr int kSlots = mid::kSlots;              // activation ring: pieces in LDS
    constexpr int kRound = mid::kPiecesPerRound;
    constexpr int kWSteps = kRound * P;              // weight ring: steps in flight per wave (one round ahead)
    constexpr int kFrags = MB * P;                   // activation fragments (1 KiB) per piece
    constexpr int kFw = mid::frags_per_wave(MB, GS); // ... of which a wave fetches this many
    constexpr int kPiecesPerGroup = GS / P;          // 1, or 2 for a group of 256
    constexpr int kGroupsPerRound = kRound / kPiecesPerGroup;  // scale fetches per round: 4 or 2
    static_assert(kRound == kSlots, "a piece's ring slot is its place in the unrolled round");
    typedef float v4f __attribute__((ext_vector_type(4)));
    typedef _Float16 v4h __attribute__((ext_vector_type(4)));
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    typedef unsigned v2u __attribute__((ext_vector_type(2)));

    // activation ring [slot][fragment][256 dwords] and one more fragment that surplus fetches land in; once the loop is
    // over the same memory holds a 16 x 64 fp32 tile per wave (rows padded to 68: lanes (col, quad) write four rows
    // each without bank conflicts, rows are read back as 16-byte pieces), and its last dword the split-K verdict
    constexpr int kSpare = kSlots * kFrags * 256;
    constexpr int kStagePitch = 68, kStageDwords = 16 * kStagePitch;
    constexpr int kLdsDwords = ((kSpare + 256) > NW * kStageDwords ? (kSpare + 256) : NW * kStageDwords) + 4;
    __shared__ __attribute__((aligned(16))) uint32_t lds[kLdsDwords + MB * 16];   // (+ the token scales of the row part)
    constexpr int kVerdict = kLdsDwords - 1;
    float* const sa_lds = reinterpret_cast<float*>(&lds[kLdsDwords]);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15, quad = lane >> 4;
    const int split = blockIdx.y;
    const int strip_raw = blockIdx.x * NW + wave;
    const bool strip_ok = strip_raw < p.strips;      // (a wave past the last strip computes the last one again and stores nothing)
    const int strip = min(strip_raw, p.strips - 1);
    const int mblocks_all = (p.M + 15) >> 4;
    const int mb0 = blockIdx.z * MB;                 // first row block of this row part
    const int mblocks = min(MB, mblocks_all - mb0);  // (surplus blocks compute zeros and store nothing)
    const int row0 = mb0 * 16;

    // K range of this workgroup (whole groups: groups_per_split), in pieces
    const int s0 = min(split * p.groups_per_split, p.G) * GS;
    const int s1 = min((split + 1) * p.groups_per_split, p.G) * GS;
    const int pieces = (s1 - s0) / P;
    const int rounds = (pieces + kRound - 1) / kRound;
    auto first_step = [&](int piece) { return s0 + max(min(piece, pieces - 1), 0) * P; };  // pieces past the end repeat the last

    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(p.w_r), 0, (int)weight_bytes(p.strips, p.steps), 0x00020000);
    const __amdgpu_buffer_rsrc_t q_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t*>(p.q), 0, (int)min((size_t)p.M * p.ldq, (size_t)0x7fffffff), 0x00020000);  // rows past M read as zero
    const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.s_r), 0, (int)min((size_t)p.strips * p.G * 128, (size_t)0x7fffffff), 0x00020000);
    const uint32_t wstride = (uint32_t)p.strips * (kRunSteps * kUnitBytes);
    const uint32_t wbase = (uint32_t)strip * (kRunSteps * kUnitBytes);
    const uint32_t wlane = lane * 16;
    const uint32_t s_lane_off = (uint32_t)(strip * 16 + col) * 8;
    const uint32_t s_group_stride = (uint32_t)p.strips * 128;
    // the fragments this wave fetches of every piece: wave, wave + NW, ... (fragment f = row block f / P, step f % P);
    // a surplus one reads past the end of the buffer (zeros, no memory traffic) into the spare fragment
    uint32_t a_off[kFw];
    int a_dst[kFw];
#pragma unroll
    for (int j = 0; j < kFw; ++j) {
        const int f = wave + NW * j;
        const bool on = f < kFrags;
        a_off[j] = on ? (uint32_t)(row0 + (f / P) * 16 + col) * (uint32_t)p.ldq + quad * 16 + (f % P) * kStepK : 0x80000000u;
        a_dst[j] = on ? f * 256 : -1;
    }

    // the token scales of the row part: asked for first, parked in LDS for the end once the pipeline's first loads are
    // out (parking them here would hold those loads back by a trip to memory)
    const float sa_mine = p.s_a[min(row0 + min(tid, MB * 16 - 1), p.M - 1)];

    float t[MB][4][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int pp = 0; pp < 4; ++pp)
#pragma unroll
            for (int j = 0; j < 4; ++j) t[mb][pp][j] = 0.0f;

    if (ZP && pieces > 0) {
        // the term (2 - zp) * scale * rowsum of this workgroup's groups, four groups per fp32 MFMA (lane (col, quad)
        // supplies token col / channel col of group 4b + quad)
        const int g_lo = s0 / GS, g_cnt = (s1 - s0) / GS;
        const uint32_t* zp32 = reinterpret_cast<const uint32_t*>(p.zp_r);
        int rrow[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) rrow[mb] = min(row0 + mb * 16 + col, p.M - 1);
        // (sixteen groups' loads are asked for together: a turn of four groups is a dozen MFMAs, far less than a trip to memory)
        constexpr int kTurns = 4;
        for (int gb0 = 0; gb0 < g_cnt; gb0 += 4 * kTurns) {
            v2u zs[kTurns];
            uint32_t zz[kTurns];
            int rs[kTurns][MB];
#pragma unroll
            for (int i = 0; i < kTurns; ++i) {
                const int g = g_lo + min(gb0 + 4 * i + quad, g_cnt - 1);  // clamped; masked below
                zs[i] = __builtin_amdgcn_raw_buffer_load_b64(s_rsrc, s_lane_off, g * s_group_stride, 0);
                zz[i] = p.zp_r ? zp32[((size_t)g * p.strips + strip) * 16 + col] : (uint32_t)p.zp_const * 0x01010101u;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) rs[i][mb] = p.rowsum[(size_t)g * p.ldr + rrow[mb]];
            }
#pragma unroll
            for (int i = 0; i < kTurns; ++i) {
                const int gb = gb0 + 4 * i;
                if (gb < g_cnt) {   // (uniform)
                    const bool on = gb + quad < g_cnt;
                    const v4h sh = __builtin_bit_cast(v4h, zs[i]);
                    float zb[4];
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp) zb[pp] = on ? (2.0f - (float)((zz[i] >> (8 * pp)) & 0xffu)) * (float)sh[pp] : 0.0f;
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        const float rsf = (float)rs[i][mb];
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
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // nothing of this phase is in flight when the pipeline starts
    }

    // ---- the pipeline.  Memory operations of a wave, in issue order, per piece i:
    //        [scales of the next round, when i is a round's first piece: kGroupsPerRound loads]
    //        weights of piece i + kRound (P loads, into the ring slots piece i has just been unpacked from)
    //        ... wait for this wave's share of the activations of piece i, barrier ...
    //        its share of the activations of piece i + kSlots - 1 (kFw LDS-direct loads, into the slot piece i - 1
    //        was read from: every wave is past those reads once it has reached the barrier)
    //        ... MFMAs of piece i ...
    //      so between the issue of a piece's activations and the wait for them lie (kSlots - 2) x (P + kFw) + P
    //      operations, plus a round's scale loads when a round started in between (always, but for a round's last
    //      piece); the prologue issues its loads in the same interleaving.
    v4u wring[kWSteps];
    v2u sreg[kGroupsPerRound], snext[kGroupsPerRound];
    auto issue_w = [&](int slot, int piece, int s) {
        const int step = first_step(piece) + s;
        wring[slot] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wlane, (step / kRunSteps) * wstride + (step % kRunSteps) * kUnitBytes + wbase, 0);
    };
    auto issue_a = [&](int slot, int piece) {
        const uint32_t k_off = (uint32_t)first_step(piece) * kStepK;
#pragma unroll
        for (int j = 0; j < kFw; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                q_rsrc, (__attribute__((address_space(3))) void*)&lds[a_dst[j] >= 0 ? slot * (kFrags * 256) + a_dst[j] : kSpare], 16,
                a_off[j], k_off, 0, 0);
    };
    auto fetch_scales = [&](int round, v2u (&dst)[kGroupsPerRound]) {   // the groups of a round's pieces (clamped to the range)
#pragma unroll
        for (int gi = 0; gi < kGroupsPerRound; ++gi)
            dst[gi] = __builtin_amdgcn_raw_buffer_load_b64(
                s_rsrc, s_lane_off, (first_step(round * kRound + gi * kPiecesPerGroup) / GS) * s_group_stride, 0);
    };

    if (pieces > 0) {
        __builtin_amdgcn_sched_barrier(0);
        fetch_scales(0, snext);
        // weights of the first round, the activations of the first kSlots - 1 pieces between the last of them
        constexpr int kFirst = kWSteps - (kSlots - 2) * P;
#pragma unroll
        for (int i = 0; i < kFirst; ++i) issue_w(i, i / P, i % P);
#pragma unroll
        for (int sl = 0; sl < kSlots - 1; ++sl) {
            if (sl > 0) {
#pragma unroll
                for (int i = 0; i < P; ++i) issue_w(kFirst + (sl - 1) * P + i, (kFirst + (sl - 1) * P + i) / P, i);
            }
            __builtin_amdgcn_sched_barrier(0);
            issue_a(sl, sl);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    if (tid < MB * 16) sa_lds[tid] = sa_mine;   // (the barrier after the loop lies between this write and its readers)

    v4i acc[2][4];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int pp = 0; pp < 4; ++pp) acc[a][pp] = v4i{0, 0, 0, 0};

    for (int r = 0; r < rounds; ++r) {
#pragma unroll
        for (int gi = 0; gi < kGroupsPerRound; ++gi) sreg[gi] = snext[gi];
#pragma unroll
        for (int u = 0; u < kRound; ++u) {
            const int piece = r * kRound + u;
            const bool live = piece < pieces;                   // (uniform) a piece past the end adds nothing: zero scale
            __builtin_amdgcn_sched_barrier(0);
            if (u == 0) fetch_scales(r + 1, snext);
            __builtin_amdgcn_sched_barrier(0);
            // unpack the piece's weight units, then refill their ring slots with the units of the same piece one round on
            v4i b[P][4];
#pragma unroll
            for (int s = 0; s < P; ++s) {
                const v4i w = __builtin_bit_cast(v4i, wring[u * P + s]);
                const v4i wf = w ^ (int)0x2a2a2a2au;            // flip the high bit of fields 0..2: two's complement of code - 2
#pragma unroll
                for (int pp = 0; pp < 3; ++pp) b[s][pp] = (wf << (6 - 2 * pp)) & (int)0xc0c0c0c0u;
                b[s][3] = w & (int)0xc0c0c0c0u;                 // field 3 is stored already flipped
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < P; ++s) issue_w(u * P + s, piece + kRound, s);
            __builtin_amdgcn_sched_barrier(0);
            // the piece's scales: operand bytes are 64 * (code - 2), so 1/64 goes into the scale (exact)
            const v2u sr = sreg[u / kPiecesPerGroup];
            const float unit = live ? 0.015625f : 0.0f;        // (one scalar select: no branch cuts the unrolled piece in blocks)
            float sc[4];
            sc[0] = half_bits_to_float((uint16_t)(sr.x & 0xffffu)) * unit;
            sc[1] = half_bits_to_float((uint16_t)(sr.x >> 16)) * unit;
            sc[2] = half_bits_to_float((uint16_t)(sr.y & 0xffffu)) * unit;
            sc[3] = half_bits_to_float((uint16_t)(sr.y >> 16)) * unit;
            // this wave's share of the piece's activations has landed: all but the operations issued after it; behind
            // the barrier so has every wave's, and the slot of the piece before is free
            constexpr int kBehind = (kSlots - 2) * (P + kFw) + P;
            if (u < kRound - 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kBehind + kGroupsPerRound) : "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kBehind) : "memory");
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            issue_a((u + kSlots - 1) % kSlots, piece + kSlots - 1);
            __builtin_amdgcn_sched_barrier(0);
            const uint32_t* const slot = &lds[u * (kFrags * 256) + lane * 4];
            const int g = first_step(piece) / GS;
            // row blocks: MFMAs of block mb into accumulator set mb & 1, the drain of block mb - 1 woven in between; the
            // two fragments after the one in use are on their way from LDS while the MFMAs of the one in use run
            v4i a_nxt = *reinterpret_cast<const v4i*>(slot);
            v4i a_nxt2 = kFrags > 1 ? *reinterpret_cast<const v4i*>(slot + 256) : v4i{0, 0, 0, 0};
#pragma unroll
            for (int mb = 0; mb <= MB; ++mb) {
                const int cur = mb & 1, prev = cur ^ 1;
#pragma unroll
                for (int s = 0; s < P; ++s) {
                    const v4i a = a_nxt;
                    a_nxt = a_nxt2;
                    if (mb * P + s + 2 < kFrags) a_nxt2 = *reinterpret_cast<const v4i*>(slot + (mb * P + s + 2) * 256);
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp) {
                        if (mb < MB) acc[cur][pp] = mfma_i8_16x16x64(a, b[s][pp], s == 0 ? v4i{0, 0, 0, 0} : acc[cur][pp]);
                        if (mb > 0) {
                            constexpr int kPer = 16 / (4 * P);   // drained elements per MFMA of the next block
#pragma unroll
                            for (int d = 0; d < kPer; ++d) {
                                const int e = (s * 4 + pp) * kPer + d;   // 0..15: sub-block e / 4, row e % 4
                                t[mb - 1][e / 4][e % 4] = __builtin_fmaf((float)acc[prev][e / 4][e % 4], sc[e / 4], t[mb - 1][e / 4][e % 4]);
                                if constexpr (DUMP) {
                                    if (live && strip_ok) {   // a group of 256: its second piece adds to what its first one wrote
                                        const int m = row0 + (mb - 1) * 16 + quad * 4 + e % 4, n = strip * kStripN + (e / 4) * 16 + col;
                                        const int v = acc[prev][e / 4][e % 4] >> 6;
                                        const bool first = first_step(piece) % GS == 0;
                                        if (first) dump_group_sum(p, m, n, g, v, 2);
                                        else if (m < p.M && n < p.N) {
                                            if (p.dump_mode == 1) p.acc_dump[((size_t)m * p.N + n) * p.G + g] += v;
                                            else atomicAdd(p.acc_dump + (size_t)m * p.N + n, v);
                                        }
                                    }
                                }
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            // every fragment of the slot has been read (the MFMAs took them) before this wave reaches the next barrier
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // (the last fetches, repeats of the last piece, have landed)

    __syncthreads();   // every wave is out of the loop: the ring is free for the output tiles
    uint16_t* const out = reinterpret_cast<uint16_t*>(p.out);
    float* const stage = reinterpret_cast<float*>(lds) + wave * kStageDwords;
    const bool wide = ((reinterpret_cast<uintptr_t>(p.out) | (uintptr_t)(2 * (size_t)p.ldo)) & 7) == 0;   // rows of 8-byte pieces
    const auto store_out = [&]() {   // out = running sum x token scale, a block of 16 rows at a time through the wave's tile
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            if (mb < mblocks) {   // (uniform)
#pragma unroll
                for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                    for (int j = 0; j < 4; ++j) stage[(quad * 4 + j) * kStagePitch + pp * 16 + col] = t[mb][pp][j];
#pragma unroll
                for (int i = 0; i < 4; ++i) {   // lane (col, quad): row i x 4 + quad, channels col x 4 .. + 3
                    const v4f v = *reinterpret_cast<const v4f*>(&stage[(i * 4 + quad) * kStagePitch + col * 4]);
                    const int m = row0 + mb * 16 + i * 4 + quad, n = strip * kStripN + col * 4;
                    const float sa = sa_lds[mb * 16 + i * 4 + quad];
                    uint16_t h[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) h[c] = OutT::cast(v[c] * sa);
                    if (strip_ok && m < p.M) {
                        uint16_t* const dst = out + (size_t)m * p.ldo + n;
                        if (wide && n + 3 < p.N) {
                            *reinterpret_cast<v2u*>(dst) = v2u{(unsigned)h[0] | ((unsigned)h[1] << 16), (unsigned)h[2] | ((unsigned)h[3] << 16)};
                        } else {
#pragma unroll
                            for (int c = 0; c < 4; ++c)
                                if (n + c < p.N) dst[c] = h[c];
                        }
                    }
                }
            }
        }
    };
    if (p.split <= 1) {
        store_out();
        return;
    }

    // ---- split-K: publish the running sums; the last workgroup of the strip set and row part to arrive adds them up in
    // split order.  Tile (strip, row block) of split s lies at ((s x strips + strip) x row blocks + block) x 4 KiB; a
    // lane's element (pp, j) at ((pp x 64 + lane) x 4 + j) x 4 bytes within it.
    constexpr int kCoherent = 17;  // sc0 | sc1
    constexpr int kTileBytes = 16 * kStripN * 4;
    const size_t tiles = (size_t)p.strips * mblocks_all;
    const __amdgpu_buffer_rsrc_t ws_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        p.ws_partial, 0, (int)min((size_t)p.split * tiles * kTileBytes, (size_t)0x7fffffff), 0x00020000);
    const uint32_t split_pitch = (uint32_t)(tiles * kTileBytes);
    const uint32_t lane_off = (uint32_t)(strip * mblocks_all + mb0) * kTileBytes + lane * 16;
    if (strip_ok) {
        uint32_t off[MB * 4];   // (addresses first: nothing but the stores and their waits between the stores)
#pragma unroll
        for (int i = 0; i < MB * 4; ++i) off[i] = lane_off + (i / 4) * kTileBytes + (i % 4) * 1024 + split * split_pitch;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                if (mb < mblocks) {   // (uniform)
                    const v4u v = {__builtin_bit_cast(uint32_t, t[mb][pp][0]), __builtin_bit_cast(uint32_t, t[mb][pp][1]),
                                   __builtin_bit_cast(uint32_t, t[mb][pp][2]), __builtin_bit_cast(uint32_t, t[mb][pp][3])};
                    __builtin_amdgcn_raw_buffer_store_b128(v, ws_rsrc, off[mb * 4 + pp], 0, kCoherent);
                    asm volatile("s_nop 1" ::: "memory");
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int counter_id = (blockIdx.x * NW) * mblocks_all + mb0;   // the set's first tile stands for the set
    if (tid == 0) {
        const unsigned prev = __hip_atomic_fetch_add(p.ws_counter + counter_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        lds[kVerdict] = (prev == (unsigned)(p.split - 1));
    }
    __syncthreads();
    if (lds[kVerdict] == 0) return;
    // the partial tiles come from memory, not from this XCD's L2: a row block's loads (four channel blocks x up to four
    // splits) are in flight together, and with up to four row blocks the next block's as well
    const auto fetch = [&](int mb, int sp0, v4u (&dst)[16]) {
#pragma unroll
        for (int pp = 0; pp < 4; ++pp)
#pragma unroll
            for (int u = 0; u < 4; ++u)   // past the last split: the last one again, not added
                dst[pp * 4 + u] = __builtin_amdgcn_raw_buffer_load_b128(
                    ws_rsrc, lane_off + mb * kTileBytes + pp * 1024 + min(sp0 + u, p.split - 1) * split_pitch, 0, kCoherent);
    };
    constexpr bool kTwoDeep = MB <= 4;   // (registers for two row blocks' loads in flight next to the sums)
    v4u part[kTwoDeep ? 2 : 1][16];
    if (kTwoDeep) fetch(0, 0, part[0]);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        v4u (&mine)[16] = part[kTwoDeep ? mb & 1 : 0];
        if (kTwoDeep && mb + 1 < MB) {
            if (mb + 1 < mblocks) fetch(mb + 1, 0, part[kTwoDeep ? (mb + 1) & 1 : 0]);   // (uniform)
        }
        if (mb < mblocks) {   // (uniform)
            v4f sum[4];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) sum[pp] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            for (int sp0 = 0; sp0 < p.split; sp0 += 4) {
                if (!kTwoDeep || sp0 > 0) fetch(mb, sp0, mine);
#pragma unroll
                for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        if (sp0 + u < p.split) sum[pp] += __builtin_bit_cast(v4f, mine[pp * 4 + u]);
            }
#pragma unroll
            for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                for (int j = 0; j < 4; ++j) t[mb][pp][j] = sum[pp][j];
        }
    }
    store_out();
    if (tid == 0) __hip_atomic_store(p.ws_counter + counter_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int MB, int GS, bool ZP, typename OutT, bool DUMP>
__global__ __launch_bounds__(mid::kWaves * 64, 2) void mid_kernel(const GemmParams p) {
    mid_body<MB, GS, ZP, OutT, DUMP>(p);
}

template <int MB, int GS, bool DUMP>
static void launch_mid_mb(const GemmParams& p, bool zp, bool out_bf16, hipStream_t stream) {
    const dim3 grid((p.strips + mid::kWaves - 1) / mid::kWaves, p.split > 1 ? p.split : 1, mid_row_parts(p.M)), block(mid::kWaves * 64);
    if (zp) {
        if (out_bf16) mid_kernel<MB, GS, true, OutBF16, DUMP><<<grid, block, 0, stream>>>(p);
        else mid_kernel<MB, GS, true, OutF16, DUMP><<<grid, block, 0, stream>>>(p);
    } else {
        if (out_bf16) mid_kernel<MB, GS, false, OutBF16, DUMP><<<grid, block, 0, stream>>>(p);
        else mid_kernel<MB, GS, false, OutF16, DUMP><<<grid, block, 0, stream>>>(p);
    }
}

template <int GS, bool DUMP>
static void launch_mid_gs(const GemmParams& p, bool zp, bool out_bf16, hipStream_t stream) {
    switch (mid_row_blocks(p.M)) {
        case 3: launch_mid_mb<3, GS, DUMP>(p, zp, out_bf16, stream); break;
        case 4: launch_mid_mb<4, GS, DUMP>(p, zp, out_bf16, stream); break;
        case 5: launch_mid_mb<5, GS, DUMP>(p, zp, out_bf16, stream); break;
        default: launch_mid_mb<6, GS, DUMP>(p, zp, out_bf16, stream); break;
    }
}

template <bool DUMP>
static hipError_t launch_mid_impl(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    const bool zp = asym || p.zp_const != 2;
    if (gs == 1) launch_mid_gs<1, DUMP>(p, zp, out_bf16, stream);
    else if (gs == 2) launch_mid_gs<2, DUMP>(p, zp, out_bf16, stream);
    else launch_mid_gs<4, DUMP>(p, zp, out_bf16, stream);
    return hipGetLastError();
}

// one group size of the verification instantiations (a translation unit each: they build side by side)
template <int GS>
static hipError_t launch_mid_verify_one(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream) {
    launch_mid_gs<GS, true>(p, asym || p.zp_const != 2, out_bf16, stream);
    return hipGetLastError();
}

}  // namespace w2a8
