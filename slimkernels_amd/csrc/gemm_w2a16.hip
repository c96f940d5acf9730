// Weight-only W2 GEMM for gfx950: fp16 activations times 2-bit weights on the fp16 matrix cores
// (v_mfma_f32_16x16x32_f16), fp32 accumulation, the few-token-rows regime where the weight stream
// bounds the time.  Upstream's sketch of this form is the notebook kernel `w2matmul`
// (slimkernels/triton/gemm_splitk.ipynb cell 1: 2-bit fields widened to fp16 in front of tl.dot).
//
//   out[m][n] = sum_g scale[g][n] * sum_{k in group g} x[m][k] * (code[n][k] - zp[g][n])
//
// The weights are the repacked units of the W2A8 kernels (w2a8_common.h), read once.  A unit's dword i
// holds, in 2-bit field p of byte b, the code of channel p*16 + col at k = quad*16 + 4*i + b.  Widening
// without shifts: dword & (0x00030003 << 2p), read as an fp16 pair, is the pair of subnormals
// 4^p * code * 2^-24 of bytes 0 and 2, the same on (dword >> 8) the pair of bytes 1 and 3; one packed fp16
// fma, x * 2^15 - 4^p * zp * 2^-9, leaves 4^p * 2^-9 * (code - zp), exact, and 2^9 * 4^-p goes into the
// fp32 scale (fp16 subnormals are operands like any other here).  The lane's eight
// k-values of one MFMA therefore come in the order 0,2,1,3,4,6,5,7; the activation operand is put in
// the same order with two v_perm_b32 per register pair.
//
// Work split: a workgroup is 4, 8 or 16 wavefronts that take as many K-parts of ONE strip of 64 channels and
// 16 token rows and add their sums up through LDS; blockIdx.y splits K further across workgroups when the
// strips alone would leave CUs idle (fp32 partial sums to a workspace, summed in split order by a second
// kernel: deterministic).  Activations are read straight from global memory (they stay in L2; rows past M
// are out of range of the buffer descriptor and read as zero without a memory access).  Every wave keeps
// three chunks of 128 reduction elements of weights in flight while it works on a fourth.
//
// bf16 activations (XBF) go to v_mfma_f32_16x16x32_bf16.  The vector ALU has no bf16 arithmetic, so the codes are not
// centred in front of the matrix core: a field shifted to mantissa bits 6:5 and OR-ed onto 0x3f80 is the bf16 number
// 1 + code / 4 (one shift and one v_and_or_b32 per register), a fifth MFMA per 32 reduction elements against ones sums
// the activations of the group, and at the group's end
//   sum_k x * (code - zp) = 4 * sum_k x * (1 + code / 4) - (4 + zp) * sum_k x
// is put together in fp32 (every product is exact; the two sums are a few times larger than their difference, which
// costs an fp32 accumulation a few of its 24 bits).
#include <algorithm>

#include "w2a8_launch.h"

namespace w2a8 {

namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

constexpr int kChunkSteps = 2;   // steps (of 64) per loop iteration

// GS = steps per scale group (1, 2 or 4); kWaves = K-parts per workgroup (4, 8 or 16); ZP = per-group
// zero-points; PARTIAL = write fp32 partial sums instead of the output
typedef __bf16 v8b __attribute__((ext_vector_type(8)));

// (The bf16 form is held to 128 registers, two eight-wave workgroups per CU: left alone it takes 162 and one
// workgroup, 35.7 instead of 22.0 us at 28672 x 8192, one row; groups of 256 would spill 252 bytes at that limit and
// keep the compiler's own choice, as every fp16 instantiation does.)
// unit, split_idx, mblk: the workgroup's set of strips, its K split (PARTIAL) and its block of 16 token rows.
// lp: log2 of the K-parts per strip inside the workgroup, P; the workgroup holds kWaves / P strips (unit * kWaves / P
// onwards), wave w works on strip w / P, part w % P.  One launch of one problem runs P = kWaves (one strip).
template <int GS, int kWaves, bool ZP, bool PARTIAL, typename OutT, bool XBF>
__device__ __forceinline__ void w2a16_body(const W2A16Params& p, const int unit, const int split_idx, const int mblk,
                                           const int lp, float (&red)[kWaves][16][64]) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15, quad = lane >> 4;
    const int m0 = mblk * 16;
    const int P = 1 << lp, sidx = wave >> lp, kp = wave & (P - 1);
    const int strip_raw = unit * (kWaves >> lp) + sidx;
    const bool strip_ok = strip_raw < p.strips;     // a surplus wave streams the last strip and stores nothing
    const int strip = min(strip_raw, p.strips - 1);

    // K-parts in granules of max(GS, 2) steps, dealt out evenly over split * kWaves parts (a part may be empty)
    constexpr int kGranule = GS > kChunkSteps ? GS : kChunkSteps;
    const int n_gran = p.steps / kGranule;
    const int parts = p.split * P;
    const int part = split_idx * P + kp;
    const int gr0 = (int)((long long)part * n_gran / parts), gr1 = (int)((long long)(part + 1) * n_gran / parts);
    const int step0 = gr0 * kGranule;
    const int n_chunks = (gr1 - gr0) * (kGranule / kChunkSteps);

    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.x), 0, (int)min((size_t)p.M * p.ldx * 2, (size_t)0x7fffffff), 0x00020000);
    const uint32_t x_lane = ((uint32_t)(m0 + col) * (uint32_t)p.ldx + quad * 16) * 2;   // bytes
    const uint32_t* w_lane = p.w_r + ((size_t)strip * kRunSteps * 64 + lane) * 4;       // the strip's first run of four steps
    const size_t w_run = (size_t)p.strips * kRunSteps * kUnitDwords;                    // dwords between runs
    const uint16_t* s_lane = p.s_r + ((size_t)strip * 16 + col) * 4;
    const uint8_t* z_lane = ZP ? p.zp_r + ((size_t)strip * 16 + col) * 4 : nullptr;
    const size_t sz_group = (size_t)p.strips * 64;                                      // elements between groups

    constexpr int kGPC = GS == 1 ? 2 : 1;  // scale groups that start or continue in one chunk
    struct WChunk {
        v4i w[kChunkSteps];
    };
    struct AChunk {
        v4u a[kChunkSteps][2];
        uint2 s[kGPC];
        uint32_t z[kGPC];
    };
    auto load_w = [&](int c) {
        WChunk ch;
        const int st = step0 + c * kChunkSteps;
#pragma unroll
        for (int s = 0; s < kChunkSteps; ++s) ch.w[s] = *reinterpret_cast<const v4i*>(w_lane + (size_t)((st + s) / kRunSteps) * w_run + (size_t)((st + s) % kRunSteps) * kUnitDwords);
        return ch;
    };
    auto load_a = [&](int c) {
        AChunk ch;
        const int st = step0 + c * kChunkSteps;
#pragma unroll
        for (int s = 0; s < kChunkSteps; ++s)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                ch.a[s][h] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, x_lane + (uint32_t)((st + s) * kStepK * 2 + h * 16), 0, 0);
#pragma unroll
        for (int gi = 0; gi < kGPC; ++gi) {
            const int g = (st + gi) / GS;   // GS == 1: groups st, st + 1; otherwise the group of step st
            ch.s[gi] = *reinterpret_cast<const uint2*>(s_lane + (size_t)g * sz_group);
            ch.z[gi] = ZP ? *reinterpret_cast<const uint32_t*>(z_lane + (size_t)g * sz_group) : 0u;
        }
        return ch;
    };

    float t[4][4];
    v4f acc[4];
    v4f acc_x = {0.f, 0.f, 0.f, 0.f};   // XBF: the group's activation sums per token row
#pragma unroll
    for (int pp = 0; pp < 4; ++pp) {
        acc[pp] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) t[pp][j] = 0.f;
    }

    auto compute = [&](const WChunk& cw, const AChunk& cur, int c) {
#pragma unroll
        for (int s = 0; s < kChunkSteps; ++s) {
            const int gi = GS == 1 ? s : 0;
            // -zp * 4^p * 2^-9 as an fp16 pair, per sub-block
            v2h zneg[4];
#pragma unroll
            for (int pp = 0; pp < 4; ++pp) {
                const uint32_t z = ZP ? (cur.z[gi] >> (8 * pp)) & 0xffu : (uint32_t)p.zp_const;
                const _Float16 zh = (_Float16)(-(float)(z << (2 * pp)) * (1.0f / 512.0f));
                zneg[pp] = v2h{zh, zh};
            }
            const v4i wf = cw.w[s] ^ (int)0x80808080u;      // field 3 is stored with its high bit flipped
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const v4u d = cur.a[s][h];
                const v4u ap = {__builtin_amdgcn_perm(d[1], d[0], 0x05040100u), __builtin_amdgcn_perm(d[1], d[0], 0x07060302u),
                                __builtin_amdgcn_perm(d[3], d[2], 0x05040100u), __builtin_amdgcn_perm(d[3], d[2], 0x07060302u)};
                const uint32_t e0 = (uint32_t)wf[2 * h], e1 = (uint32_t)wf[2 * h + 1];
                if constexpr (XBF) {
                    constexpr uint32_t kOne = 0x3f803f80u, kField = 0x00600060u;
                    const v4u ones = {kOne, kOne, kOne, kOne};
                    acc_x = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8b, ap), __builtin_bit_cast(v8b, ones), acc_x, 0, 0, 0);
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp) {
                        // field p of a half-word's low byte (even bytes) resp. high byte (odd bytes) -> mantissa bits 6:5
                        const int up = 5 - 2 * pp;   // 5, 3, 1, -1
                        const auto even = [&](uint32_t v) { return pp < 3 ? v << (up & 31) : v >> 1; };
                        const v4u b = {(even(e0) & kField) | kOne, ((e0 >> (8 - up)) & kField) | kOne,
                                       (even(e1) & kField) | kOne, ((e1 >> (8 - up)) & kField) | kOne};
                        acc[pp] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8b, ap), __builtin_bit_cast(v8b, b), acc[pp], 0, 0, 0);
                    }
                    continue;
                }
                const uint32_t o0 = e0 >> 8, o1 = e1 >> 8;
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    const uint32_t mask = 0x00030003u << (2 * pp);
                    // a masked field alone is an fp16 subnormal, 4^p * code * 2^-24: one packed fma per
                    // register pair scales it by 2^15 and takes the zero-point off (exact)
                    const v2h up = {(_Float16)32768.0f, (_Float16)32768.0f};
                    const v2h b0 = __builtin_elementwise_fma(__builtin_bit_cast(v2h, e0 & mask), up, zneg[pp]);
                    const v2h b1 = __builtin_elementwise_fma(__builtin_bit_cast(v2h, o0 & mask), up, zneg[pp]);
                    const v2h b2 = __builtin_elementwise_fma(__builtin_bit_cast(v2h, e1 & mask), up, zneg[pp]);
                    const v2h b3 = __builtin_elementwise_fma(__builtin_bit_cast(v2h, o1 & mask), up, zneg[pp]);
                    const v8h b = {b0[0], b0[1], b1[0], b1[1], b2[0], b2[1], b3[0], b3[1]};
                    acc[pp] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, ap), b, acc[pp], 0, 0, 0);
                }
            }
            // end of a scale group: fold the group's sums into the running sums
            const bool group_ends = GS <= kChunkSteps ? ((s + 1) % GS == 0)
                                                      : (((step0 + c * kChunkSteps + s + 1) % GS) == 0);
            if (group_ends && XBF) {
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    const uint32_t raw = pp < 2 ? cur.s[gi].x : cur.s[gi].y;
                    const float sc4 = half_bits_to_float((uint16_t)((pp & 1) ? raw >> 16 : raw & 0xffffu)) * 4.0f;
                    const uint32_t z = ZP ? (cur.z[gi] >> (8 * pp)) & 0xffu : (uint32_t)p.zp_const;
                    const float off = -(4.0f + (float)z) * 0.25f;
#pragma unroll
                    for (int j = 0; j < 4; ++j) t[pp][j] = __builtin_fmaf(__builtin_fmaf(off, acc_x[j], acc[pp][j]), sc4, t[pp][j]);
                    acc[pp] = v4f{0.f, 0.f, 0.f, 0.f};
                }
                acc_x = v4f{0.f, 0.f, 0.f, 0.f};
            } else if (group_ends) {
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    const uint32_t raw = pp < 2 ? cur.s[gi].x : cur.s[gi].y;
                    const float sc = half_bits_to_float((uint16_t)((pp & 1) ? raw >> 16 : raw & 0xffffu)) *
                                     (512.0f / (float)(1 << (2 * pp)));
#pragma unroll
                    for (int j = 0; j < 4; ++j) t[pp][j] = __builtin_fmaf(acc[pp][j], sc, t[pp][j]);
                    acc[pp] = v4f{0.f, 0.f, 0.f, 0.f};
                }
            }
        }
    };
    // The weights, which come from HBM, are fetched three (two) chunks ahead through a ring of buffers; the
    // activations and scales, which come from L2, one chunk ahead (two buffers).  Past the end the fetches
    // re-read the last chunk and nobody uses them.
    constexpr int kAhead = kWaves == 16 ? 1 : 3;   // sixteen waves leave each 128 registers: a shorter ring
    constexpr int kRing = kAhead + 1;              // 4 or 2: even, so the two activation buffers alternate with it
    if (n_chunks > 0) {
        const int last = n_chunks - 1;
        WChunk wq[kRing];
        AChunk aq[2];
        aq[0] = load_a(0);
#pragma unroll
        for (int i = 0; i < kAhead; ++i) wq[i] = load_w(min(i, last));
        // whole trips of kRing chunks without a branch inside (a branch makes the compiler wait for every
        // load in flight where the paths meet); the prefetches past the end re-read the last chunk
        int c = 0;
        for (; c + kRing <= n_chunks; c += kRing) {
#pragma unroll
            for (int i = 0; i < kRing; ++i) {
                // activations first: loads complete in issue order, so waiting for these next time
                // leaves the younger weight fetches in flight
                aq[(i + 1) & 1] = load_a(min(c + i + 1, last));
                wq[(i + kAhead) % kRing] = load_w(min(c + i + kAhead, last));
                compute(wq[i], aq[i & 1], c + i);
            }
        }
        // the last chunks (fewer than kRing): their weights are already on the way
#pragma unroll
        for (int i = 0; i < kRing - 1; ++i) {
            if (c + i < n_chunks) {
                if (c + i + 1 < n_chunks) aq[(i + 1) & 1] = load_a(c + i + 1);
                compute(wq[i], aq[i & 1], c + i);
            }
        }
    }

    // the K-parts of the workgroup meet in LDS; wave w finishes 16 / kWaves of the 16 accumulator rows
#pragma unroll
    for (int pp = 0; pp < 4; ++pp)
#pragma unroll
        for (int j = 0; j < 4; ++j) red[wave][pp * 4 + j][lane] = t[pp][j];
    __syncthreads();
    // wave (strip s, part k) finishes rows k * 16 / P onwards of strip s: the parts' sums in part order
    const int rows = 16 >> lp;
    for (int i = 0; i < rows; ++i) {
        const int r = kp * rows + i, pp = r >> 2, j = r & 3;
        float v = red[sidx << lp][r][lane];
        for (int w = 1; w < P; ++w) v += red[(sidx << lp) + w][r][lane];
        const int m = m0 + quad * 4 + j;
        const int n = strip * kStripN + pp * 16 + col;
        if (strip_ok && m < p.M && n < p.N) {
            if (PARTIAL) p.ws[((size_t)split_idx * p.M + m) * p.N + n] = v;
            else reinterpret_cast<uint16_t*>(p.out)[(size_t)m * p.ldo + n] = OutT::cast(v);
        }
    }
}

template <int GS, int kWaves, bool ZP, bool PARTIAL, typename OutT, bool XBF = false>
__global__ __launch_bounds__(kWaves * 64, XBF && GS < 4 ? 4 : 1) void w2a16_kernel(const W2A16Params p) {
    __shared__ float red[kWaves][16][64];
    constexpr int kLogWaves = kWaves == 16 ? 4 : kWaves == 8 ? 3 : 2;
    w2a16_body<GS, kWaves, ZP, PARTIAL, OutT, XBF>(p, (int)blockIdx.x, (int)blockIdx.y, (int)blockIdx.z, kLogWaves, red);
}

// Several problems in one launch (no K splits across workgroups): workgroup ids are cut into runs, one per problem,
// set of strips fastest within a run; every problem has its own number of K-parts per strip (a long reduction all the
// waves of a workgroup on one strip, a short one several strips side by side); the problem table travels in the kernel
// arguments.
template <int GS, int kWaves, bool ZP, typename OutT, bool XBF>
__global__ __launch_bounds__(kWaves * 64, XBF && GS < 4 ? 4 : 1) void w2a16_grouped_kernel(const W2A16Group gp) {
    __shared__ float red[kWaves][16][64];
    const int wg = (int)blockIdx.x;
    // problem index = number of run boundaries at or below this workgroup id: one lane per boundary, one ballot
    const int bl = min((int)(threadIdx.x & 63), kMaxGroup - 1);
    const bool past = bl + 1 < gp.count && wg >= gp.wg_begin[bl + 1];
    const int i = __builtin_amdgcn_readfirstlane(__builtin_popcountll(__ballot(past)));
    const W2A16Params& p = gp.prob[i];
    const int local = wg - gp.wg_begin[i];
    const int lp = gp.log_parts[i];
    const int per = kWaves >> lp, units = (p.strips + per - 1) / per;
    w2a16_body<GS, kWaves, ZP, false, OutT, XBF>(p, local % units, 0, local / units, lp, red);
}

template <typename OutT>
__global__ __launch_bounds__(256) void w2a16_reduce_kernel(const float* __restrict__ ws, int split, int M, int N,
                                                           uint16_t* __restrict__ out, int ldo) {
    const size_t total = (size_t)M * N;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        float v = ws[i];
        for (int s = 1; s < split; ++s) v += ws[(size_t)s * total + i];
        out[(i / N) * ldo + i % N] = OutT::cast(v);
    }
}

template <int GS, int W, bool ZP, bool PARTIAL>
void launch_one(const W2A16Params& p, bool out_bf16, dim3 grid, hipStream_t stream) {
    if (p.x_bf16) {
        if (out_bf16) w2a16_kernel<GS, W, ZP, PARTIAL, OutBF16, true><<<grid, dim3(W * 64), 0, stream>>>(p);
        else w2a16_kernel<GS, W, ZP, PARTIAL, OutF16, true><<<grid, dim3(W * 64), 0, stream>>>(p);
        return;
    }
    if (out_bf16) w2a16_kernel<GS, W, ZP, PARTIAL, OutBF16><<<grid, dim3(W * 64), 0, stream>>>(p);
    else w2a16_kernel<GS, W, ZP, PARTIAL, OutF16><<<grid, dim3(W * 64), 0, stream>>>(p);
}

template <int GS, int W>
void launch_w(const W2A16Params& p, bool out_bf16, dim3 grid, hipStream_t stream) {
    const bool zp = p.zp_r != nullptr, partial = p.split > 1;
    if (zp) {
        if (partial) launch_one<GS, W, true, true>(p, out_bf16, grid, stream);
        else launch_one<GS, W, true, false>(p, out_bf16, grid, stream);
    } else {
        if (partial) launch_one<GS, W, false, true>(p, out_bf16, grid, stream);
        else launch_one<GS, W, false, false>(p, out_bf16, grid, stream);
    }
}

template <int GS>
void launch_gs(const W2A16Params& p, int waves, bool out_bf16, dim3 grid, hipStream_t stream) {
    if (waves == 16) launch_w<GS, 16>(p, out_bf16, grid, stream);
    else if (waves == 8) launch_w<GS, 8>(p, out_bf16, grid, stream);
    else launch_w<GS, 4>(p, out_bf16, grid, stream);
}

}  // namespace

// K splits across workgroups: one unless the strips (x blocks of 16 token rows) alone leave most CUs idle;
// then enough for about one workgroup per CU, every K-part at least two granules (256 reduction elements at
// group size <= 128) long.
int w2a16_auto_split(int M, int strips, int steps, int gs) {
    const int granule = gs > kChunkSteps ? gs : kChunkSteps;
    const int n_gran = steps / granule;
    const long long base = (long long)strips * ((M + 15) / 16);
    if (base >= 192) return 1;
    long long split = (256 + base - 1) / base;
    const int cap = n_gran / (2 * 4);
    if (split > cap) split = cap;
    if (split > 64) split = 64;
    return split < 1 ? 1 : (int)split;
}

// K-parts inside a workgroup (4, 8 or 16 wavefronts): towards 16 wavefronts per CU over the whole launch,
// every part at least four chunks (one trip of the main loop) long where K allows.
static int w2a16_waves(int M, int strips, int steps, int gs, int split) {
    const int chunks = steps / kChunkSteps;
    const long long wgs = (long long)strips * ((M + 15) / 16) * split;
    const long long wanted = 4096 / (wgs < 1 ? 1 : wgs);
    int waves = wanted >= 12 ? 16 : wanted >= 6 ? 8 : 4;
    while (waves > 4 && (long long)waves * split * 4 > chunks) waves /= 2;
    return waves;
}

namespace {
template <int GS, int W>
void launch_group_w(const W2A16Group& gp, bool zp, bool out_bf16, bool x_bf16, dim3 grid, hipStream_t stream) {
#define SLIMK_W2A16_GROUP(ZPV, OUT, XB) w2a16_grouped_kernel<GS, W, ZPV, OUT, XB><<<grid, dim3(W * 64), 0, stream>>>(gp)
    if (zp) {
        if (x_bf16) { if (out_bf16) SLIMK_W2A16_GROUP(true, OutBF16, true); else SLIMK_W2A16_GROUP(true, OutF16, true); }
        else { if (out_bf16) SLIMK_W2A16_GROUP(true, OutBF16, false); else SLIMK_W2A16_GROUP(true, OutF16, false); }
    } else {
        if (x_bf16) { if (out_bf16) SLIMK_W2A16_GROUP(false, OutBF16, true); else SLIMK_W2A16_GROUP(false, OutF16, true); }
        else { if (out_bf16) SLIMK_W2A16_GROUP(false, OutBF16, false); else SLIMK_W2A16_GROUP(false, OutF16, false); }
    }
#undef SLIMK_W2A16_GROUP
}
template <int GS>
void launch_group_gs(const W2A16Group& gp, int waves, bool zp, bool out_bf16, bool x_bf16, dim3 grid, hipStream_t stream) {
    if (waves == 16) launch_group_w<GS, 16>(gp, zp, out_bf16, x_bf16, grid, stream);
    else if (waves == 8) launch_group_w<GS, 8>(gp, zp, out_bf16, x_bf16, grid, stream);
    else launch_group_w<GS, 4>(gp, zp, out_bf16, x_bf16, grid, stream);
}
}  // namespace

// gp.waves wavefronts per workgroup (4, 8 or 16), gp.log_parts[i] the K-parts per strip of problem i
hipError_t launch_w2a16_grouped(const W2A16Group& gp, int gs, bool zp, bool out_bf16, bool x_bf16, hipStream_t stream) {
    const dim3 grid((unsigned)gp.wg_begin[gp.count]);
    if (gs == 1) launch_group_gs<1>(gp, gp.waves, zp, out_bf16, x_bf16, grid, stream);
    else if (gs == 2) launch_group_gs<2>(gp, gp.waves, zp, out_bf16, x_bf16, grid, stream);
    else launch_group_gs<4>(gp, gp.waves, zp, out_bf16, x_bf16, grid, stream);
    return hipGetLastError();
}

hipError_t launch_w2a16(const W2A16Params& p, int gs, bool out_bf16, hipStream_t stream) {
    const dim3 grid((unsigned)p.strips, (unsigned)p.split, (unsigned)((p.M + 15) / 16));
    const int waves = w2a16_waves(p.M, p.strips, p.steps, gs, p.split);
    if (gs == 1) launch_gs<1>(p, waves, out_bf16, grid, stream);
    else if (gs == 2) launch_gs<2>(p, waves, out_bf16, grid, stream);
    else launch_gs<4>(p, waves, out_bf16, grid, stream);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    if (p.split > 1) {
        const size_t total = (size_t)p.M * p.N;
        const unsigned blocks = (unsigned)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
        if (out_bf16)
            w2a16_reduce_kernel<OutBF16><<<dim3(blocks), dim3(256), 0, stream>>>(p.ws, p.split, p.M, p.N, (uint16_t*)p.out, p.ldo);
        else
            w2a16_reduce_kernel<OutF16><<<dim3(blocks), dim3(256), 0, stream>>>(p.ws, p.split, p.M, p.N, (uint16_t*)p.out, p.ldo);
    }
    return hipGetLastError();
}

}  // namespace w2a8
