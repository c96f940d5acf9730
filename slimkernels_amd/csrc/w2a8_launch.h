// Internal host-side launch entry points, one per kernel family.  Each validates
// nothing (the C ABI layer did) and only enqueues on the given stream.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "w2a8_common.h"

namespace w2a8 {

hipError_t launch_repack(const uint8_t* w_packed, int ldw, const uint16_t* scales, const uint8_t* zp,
                         int N, int K, int group_size, uint32_t* w_r, uint16_t* s_r, uint8_t* zp_r,
                         hipStream_t stream);

hipError_t launch_act_quant(const void* x, int ldx, bool x_bf16, int M, int K, int group_size,
                            int8_t* q, int ldq, float* s_a, int32_t* rowsum, int ldr, int copies, hipStream_t stream);

// mode: 0 upstream quantizer (zero-point 1), 1 symmetric levels (zero-point 2), 2 per-group zero-points
hipError_t launch_quantize_weight(const void* w, int ldw, bool w_bf16, int N, int K, int group_size, int mode,
                                  uint8_t* packed, int ldp, uint16_t* scales, uint8_t* zp, hipStream_t stream);

// 4-bit codes written as the two 2-bit planes over 2K that the W2 kernels take (packed [N][ldp >= 2K/4],
// scales and zp [2G][N]); asym false: levels -8..7, true: per-group zero-points
hipError_t launch_quantize_weight4(const void* w, int ldw, bool w_bf16, int N, int K, int group_size, bool asym,
                                   uint8_t* packed, int ldp, uint16_t* scales, uint8_t* zp, hipStream_t stream);

hipError_t launch_fill_zero(void* p, size_t bytes, hipStream_t stream);

hipError_t launch_read_probe(const void* src, size_t bytes, uint32_t* sink, hipStream_t stream);

// gs = 64-element steps per scale group (1, 2 or 4); waves = wavefronts per workgroup (4, 8 or 16)
hipError_t launch_skinny(const GemmParams& p, int gs, int waves, bool asym, bool out_bf16, hipStream_t stream);

// the same kernel with the activation quantisation inside: p.x / p.ldx / p.x_bf16 instead of p.q, p.s_a, p.rowsum;
// at most kFusedMaxRows token rows with rows x K <= kFusedMaxBytes
hipError_t launch_skinny_fused(const GemmParams& p, int gs, int waves, bool asym, bool out_bf16, hipStream_t stream);
// The same for up to 32 rows, quantised by the grid's first workgroups into the workspace (p.q / p.s_a / p.rowsum point
// there, p.ws_counter at the workspace's counter block); spin_limit bounds the wait for the rows.
hipError_t launch_skinny_rows(const GemmParams& p, int gs, int waves, bool asym, bool out_bf16, int spin_limit, hipStream_t stream);

// one problem through the shared-activation workgroups (kparts k-parts x 8 / kparts strips per workgroup, kparts =
// kSharedParts or twice that; p.split K splits across workgroups)
hipError_t launch_skinny_shared(const GemmParams& p, int gs, int kparts, bool asym, bool out_bf16, hipStream_t stream);

// asym: every problem carries per-group zero-points (zp_r); otherwise each uses its uniform zp_const
hipError_t launch_skinny_grouped(const GroupedParams& gp, int gs, bool asym, bool out_bf16, hipStream_t stream);

// Verification instantiations of the three launches above (gemm_skinny_verify.hip): the same bodies with the int32
// dump switched on (p.acc_dump / p.dump_mode, per problem in a grouped launch), same instantiation choices.
hipError_t launch_skinny_verify(const GemmParams& p, int gs, int waves, bool asym, bool out_bf16, hipStream_t stream);
hipError_t launch_skinny_shared_verify(const GemmParams& p, int gs, int kparts, bool asym, bool out_bf16, hipStream_t stream);
hipError_t launch_skinny_grouped_verify(const GroupedParams& gp, int gs, bool asym, bool out_bf16, hipStream_t stream);

// 33..256 token rows: one workgroup per set of four strips (a wave each) and row part (three to six blocks of 16 rows;
// more than 96 rows run as two or three parts of equal height), K split over blockIdx.y in whole groups
// (p.groups_per_split); the split workspace holds one fp32 tile of 16 x 64 per strip, row block and split and one
// arrival counter per strip and row block, as the one-strip kernel's does.  launch_mid_verify: the instantiations with
// the int32 dump.
constexpr int kMidMaxRows = 256;
namespace mid {
constexpr int kWaves = 4;           // strips per workgroup
constexpr int kSlots = 4;           // pieces of activations in LDS
constexpr int kPiecesPerRound = 4;  // pieces per unrolled round of the main loop (a piece's ring slot is compile-time)
__host__ __device__ constexpr int piece_steps(int GS) { return GS >= 2 ? 2 : 1; }   // 64-element steps per piece
__host__ __device__ constexpr int frags_per_wave(int MB, int GS) { return (MB * piece_steps(GS) + kWaves - 1) / kWaves; }
}  // namespace mid
// the row parts a launch runs as and the row blocks per part it is instantiated for (3..6)
inline int mid_row_parts(int M) { return ((M + 15) / 16 + 5) / 6; }
inline int mid_row_blocks(int M) {
    const int blocks = (M + 15) / 16, parts = mid_row_parts(M);
    const int mb = (blocks + parts - 1) / parts;
    return mb < 3 ? 3 : mb;
}

hipError_t launch_mid(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream);
hipError_t launch_mid_verify(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream);

// 4-bit weights as two planes (w_r over 2 * p.steps steps, s_r over 2 * p.G groups), uniform zero-point 8, one pass
// over K: p.K / p.steps / p.G describe K, not 2K; gs 1 or 2; p.steps even
// p.split > 1: K split over blockIdx.y in whole 128-element stages (p.groups_per_split), workspace = one arrival
// counter and p.split fp32 tiles of 64 x 256 per tile (tiled_w4_tiles)
hipError_t launch_tiled_w4(const GemmParams& p, int gs, bool out_bf16, hipStream_t stream);
hipError_t launch_tiled_w4_verify(const GemmParams& p, int gs, bool out_bf16, hipStream_t stream);
size_t tiled_w4_tiles(int M, int strips);
int tiled_w4_auto_split(int M, int strips, int steps);

// The tiled kernel (group 64 / 128 / 256); with p.acc_dump launch_tiled hands over to the verification
// instantiations (launch_tiled_verify, a translation unit of their own).
hipError_t launch_tiled(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream);
hipError_t launch_tiled_verify(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream);
// Split-K of the fast tiled kernel (gs = 64-element steps per group): the factor it would choose, the largest it
// accepts, what a requested factor comes to (whole stages per split; *groups_per_split = a split's length in groups),
// and the number of tiles a split workspace must hold (64 x 256 fp32 each, per split).
bool tiled_fast_supported(const GemmParams& p, int gs, bool asym);
int tiled_fast_auto_split(int M, int strips, int steps, int gs);
int tiled_fast_max_split(int M, int strips, int steps, int gs);
int tiled_fast_effective_split(int steps, int gs, int split, int* groups_per_split);
size_t tiled_fast_workspace_tiles(int M, int strips, int gs);
// Weight-only form (fp16 activations on the fp16 matrix cores, gemm_w2a16.hip).
struct W2A16Params {
    const uint16_t* x;      // [M][ldx] fp16 bits (bf16 bits with x_bf16)
    const uint32_t* w_r;    // repacked codes
    const uint16_t* s_r;    // [G][strips][16][4] fp16 bits
    const uint8_t* zp_r;    // [G][strips][16][4] or nullptr
    void* out;              // [M][ldo] fp16 / bf16 bits
    float* ws;              // [split][M][N] partial sums when split > 1
    int ldx, ldo;
    int M, N, K;
    int G, steps, strips;
    int zp_const;
    int split;              // K splits across workgroups (grid.y)
    bool x_bf16;            // bf16 activations: the bf16 matrix cores
};
int w2a16_auto_split(int M, int strips, int steps, int gs);
hipError_t launch_w2a16(const W2A16Params& p, int gs, bool out_bf16, hipStream_t stream);
// Several weight-only problems in one launch (each unsplit; the activation type, zero-point mode and output type are
// the launch's): problem i owns workgroups wg_begin[i] .. wg_begin[i+1]-1, sets of strips x blocks of 16 token rows;
// a workgroup of `waves` wavefronts holds waves >> log_parts[i] strips of problem i, each in 1 << log_parts[i] K-parts.
struct W2A16Group {
    W2A16Params prob[kMaxGroup];
    int wg_begin[kMaxGroup + 1];
    int log_parts[kMaxGroup];
    int count;
    int waves;
};
hipError_t launch_w2a16_grouped(const W2A16Group& gp, int gs, bool zp, bool out_bf16, bool x_bf16, hipStream_t stream);

}  // namespace w2a8
