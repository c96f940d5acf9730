// Generic tiled W2A8 GEMM for gfx950: every zero-point mode, every group size, ragged K, and
// the int32 verification dumps.  The fast path for the common case (uniform zero-point 2, group
// 64 or 128) lives in gemm_tiled.hip; this kernel is the reference form of the same scheme.
//
// Workgroup = 4 wavefronts as 2 (tokens) x 2 (channels); workgroup tile 128 tokens x
// 128 channels (two weight strips); wave tile 64 x 64 = 4 x 4 MFMA blocks of
// v_mfma_i32_16x16x64_i8.  The reduction runs in stages of two 64-element steps.
// Both operands are staged in LDS in MFMA-operand order: every 16-row x 64-k
// activation block and every weight unit is 1 KiB laid out lane-major, so each
// fragment read is one ds_read_b128 per lane at offset 16*lane (conflict-free by
// construction) and every global->LDS transfer is a 16-byte-per-lane copy.  Two LDS
// buffers: the next stage is fetched into registers while the current one is
// multiplied, then written to the other buffer; one barrier per stage.
// At each scale-group boundary the int32 accumulators are folded into fp32 running
// sums (v_cvt_f32_i32 + v_fma_f32 per element) and restarted at -zp * rowsum.
#include "w2a8_launch.h"

namespace w2a8 {

constexpr int kBM = 128, kBN = 128;
constexpr int kStageSteps = 2;
constexpr int kABlocks = (kBM / 16) * kStageSteps;        // 16 activation blocks per stage
constexpr int kBUnits = (kBN / kStripN) * kStageSteps;    // 4 weight units per stage
constexpr int kStageDwords = (kABlocks + kBUnits) * 256;  // 20 KiB per stage

template <int GS, bool ASYM, bool DUMP, typename OutT>
__global__ __launch_bounds__(256) void tiled_generic_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) uint32_t lds[2][kStageDwords];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;  // wave position inside the workgroup tile
    const int m_tile = blockIdx.y * kBM;
    const int strip0 = blockIdx.x * (kBN / kStripN);
    const int strip = strip0 + wn;                 // strip of this wave
    const bool strip_ok = strip < p.strips;
    const int n_stages = (p.steps + kStageSteps - 1) / kStageSteps;

    // ---- global -> register staging assignment
    // activation blocks: wave w fetches blocks w, w+4, w+8, w+12 (block = step_in_stage*8 + mb)
    // weight units:      wave w fetches unit w (unit = step_in_stage*2 + strip_in_tile)
    v4i ga[4], gb;
    const int8_t* a_src[4];
    bool a_ok[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int blk = wave + 4 * i;
        const int mb = blk & 7;
        const int m = m_tile + mb * 16 + col;
        a_ok[i] = m < p.M;
        a_src[i] = p.q + (size_t)(a_ok[i] ? m : 0) * p.ldq + (blk >> 3) * kStepK + quad * 16;
    }
    const int b_strip = strip0 + (wave & 1);
    const bool b_ok = b_strip < p.strips;
    const uint32_t* b_src = p.w_r + ((size_t)(wave >> 1) * p.strips + (b_ok ? b_strip : 0)) * kUnitDwords + lane * 4;
    const size_t b_step_stride = (size_t)p.strips * kUnitDwords;  // dwords between consecutive steps of a strip

    auto fetch = [&](int stage) {
        const int step0 = stage * kStageSteps;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int step = step0 + ((wave + 4 * i) >> 3);
            ga[i] = v4i{0, 0, 0, 0};
            if (a_ok[i] && step < p.steps) ga[i] = *reinterpret_cast<const v4i*>(a_src[i] + (size_t)step0 * kStepK);
        }
        const int bstep = step0 + (wave >> 1);
        gb = v4i{0, 0, 0, 0};
        if (b_ok && bstep < p.steps) gb = *reinterpret_cast<const v4i*>(b_src + (size_t)step0 * b_step_stride);
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            *reinterpret_cast<v4i*>(&lds[buf][(wave + 4 * i) * 256 + lane * 4]) = ga[i];
        *reinterpret_cast<v4i*>(&lds[buf][(kABlocks + wave) * 256 + lane * 4]) = gb;
    };

    float t[4][4][4];
    v4i acc[4][4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int pp = 0; pp < 4; ++pp) {
            acc[mb][pp] = v4i{0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 4; ++j) t[mb][pp][j] = 0.0f;
        }

    const size_t sg_strip = (size_t)(strip_ok ? strip : 0);
    const int m_wave = m_tile + wm * 64;  // first token row of this wave

    auto group_begin = [&](int g) {
        int zpe[4];
        if (ASYM) {
            const uint32_t zraw = *reinterpret_cast<const uint32_t*>(p.zp_r + (((size_t)g * p.strips + sg_strip) * 16 + col) * 4);
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
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
            const int m0 = m_wave + mb * 16 + quad * 4;
            v4i rs = {0, 0, 0, 0};
            if (m0 < p.M) rs = *reinterpret_cast<const v4i*>(p.rowsum + (size_t)g * p.ldr + m0);
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) acc[mb][pp] = rs * (-zpe[pp]);
        }
    };
    auto group_end = [&](int g) {
        const uint2 sraw = *reinterpret_cast<const uint2*>(p.s_r + (((size_t)g * p.strips + sg_strip) * 16 + col) * 4);
        float sc[4];
        sc[0] = half_bits_to_float((uint16_t)(sraw.x & 0xffffu));
        sc[1] = half_bits_to_float((uint16_t)(sraw.x >> 16)) * 0.25f;
        sc[2] = half_bits_to_float((uint16_t)(sraw.y & 0xffffu)) * 0.0625f;
        sc[3] = half_bits_to_float((uint16_t)(sraw.y >> 16)) * 0.015625f;
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int pp = 0; pp < 4; ++pp)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    t[mb][pp][j] = __builtin_fmaf((float)acc[mb][pp][j], sc[pp], t[mb][pp][j]);
                    if (DUMP) {
                        const int m = m_wave + mb * 16 + quad * 4 + j;
                        const int n = strip * kStripN + pp * 16 + col;
                        if (strip_ok && m < p.M && n < p.N) {
                            const int v = acc[mb][pp][j] >> (2 * pp);
                            if (p.dump_mode == 1)
                                p.acc_dump[((size_t)m * p.N + n) * p.G + g] = v;
                            else
                                p.acc_dump[(size_t)m * p.N + n] += v;  // one wave owns (m, n): no race
                        }
                    }
                }
    };

    fetch(0);
    stash(0);
    __syncthreads();

    for (int stage = 0; stage < n_stages; ++stage) {
        const int buf = stage & 1;
        if (stage + 1 < n_stages) fetch(stage + 1);
#pragma unroll
        for (int s = 0; s < kStageSteps; ++s) {
            const int step = stage * kStageSteps + s;
            if (step < p.steps) {
                if (step % GS == 0) group_begin(step / GS);
                const v4i w = *reinterpret_cast<const v4i*>(&lds[buf][(kABlocks + s * 2 + wn) * 256 + lane * 4]);
                v4i b[4];
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) b[pp] = w & (int)(0x03030303u << (2 * pp));
#pragma unroll
                for (int mb = 0; mb < 4; ++mb) {
                    const v4i a = *reinterpret_cast<const v4i*>(&lds[buf][(s * 8 + wm * 4 + mb) * 256 + lane * 4]);
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp) acc[mb][pp] = mfma_i8_16x16x64(a, b[pp], acc[mb][pp]);
                }
                if (step % GS == GS - 1) group_end(step / GS);
            }
        }
        if (stage + 1 < n_stages) stash(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: out = cast(t * s_a[m])
    if (!strip_ok) return;
    uint16_t* out = reinterpret_cast<uint16_t*>(p.out);
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m_wave + mb * 16 + quad * 4 + j;
            if (m >= p.M) continue;
            const float sa = p.s_a[m];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                const int n = strip * kStripN + pp * 16 + col;
                if (n < p.N) out[(size_t)m * p.ldo + n] = OutT::cast(t[mb][pp][j] * sa);
            }
        }
}

template <int GS, bool ASYM, bool DUMP>
static void launch_out(const GemmParams& p, bool out_bf16, hipStream_t stream) {
    const dim3 grid((p.strips + 1) / 2, (p.M + kBM - 1) / kBM), block(256);
    if (out_bf16)
        tiled_generic_kernel<GS, ASYM, DUMP, OutBF16><<<grid, block, 0, stream>>>(p);
    else
        tiled_generic_kernel<GS, ASYM, DUMP, OutF16><<<grid, block, 0, stream>>>(p);
}

template <int GS>
static void launch_flags(const GemmParams& p, bool asym, bool out_bf16, hipStream_t stream) {
    const bool dump = p.acc_dump != nullptr && p.dump_mode != 0;
    if (asym) {
        if (dump) launch_out<GS, true, true>(p, out_bf16, stream);
        else launch_out<GS, true, false>(p, out_bf16, stream);
    } else {
        if (dump) launch_out<GS, false, true>(p, out_bf16, stream);
        else launch_out<GS, false, false>(p, out_bf16, stream);
    }
}

hipError_t launch_tiled_generic(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    if (gs == 1) launch_flags<1>(p, asym, out_bf16, stream);
    else if (gs == 2) launch_flags<2>(p, asym, out_bf16, stream);
    else launch_flags<4>(p, asym, out_bf16, stream);
    return hipGetLastError();
}

}  // namespace w2a8
