// Fast tiled W2A8 GEMM for gfx950, production instantiations and the launch heuristics (the kernels themselves are in
// tiled_bodies.h; the verification instantiations, which also write out the int32 group sums, in
// gemm_tiled_verify.hip).
#include "tiled_bodies.h"

namespace w2a8 {

size_t tiled_w4_tiles(int M, int strips) {
    return (size_t)((strips + fast::kStrips - 1) / fast::kStrips) * (size_t)((M + 63) / 64);
}

// K splits of the one-pass W4 kernel: the rule of the 64-row W2 tiles (about two workgroups per CU, every split at
// least eight stages long; two halves for a long reduction with one workgroup on most CUs)
int tiled_w4_auto_split(int M, int strips, int steps) {
    const int tiles = (int)tiled_w4_tiles(M, strips);
    const int stages = steps / fast::kStageSteps;
    if (tiles > 128) return tiles <= 256 && stages >= 64 ? 2 : 1;
    int split = 512 / tiles;
    if (split > 8) split = 8;
    if (split > stages / 8) split = stages / 8;
    if (split < 1) split = 1;
    const int sps = (stages + split - 1) / split;
    return (stages + sps - 1) / sps;
}

hipError_t launch_tiled_w4(const GemmParams& p, int gs, bool out_bf16, hipStream_t stream) {
    if (p.acc_dump != nullptr && p.dump_mode != 0) return launch_tiled_w4_verify(p, gs, out_bf16, stream);
    return launch_tiled_w4_impl<false>(p, gs, out_bf16, stream);
}

bool tiled_fast_supported(const GemmParams& p, int gs, bool asym) {
    (void)asym;
    return (gs == 1 || gs == 2 || gs == 4) && p.steps % gs == 0;
}

// a split owns whole groups: stages for groups of 64 and 128, pairs of stages for groups of 256
int tiled_fast_max_split(int M, int strips, int steps, int gs) {
    (void)M; (void)strips;
    return gs == 4 ? steps / 4 : (steps + fast::kStageSteps - 1) / fast::kStageSteps;
}

// With at most half as many 64-row tiles as CUs, K is split over several workgroups per tile so that
// about two workgroups per CU exist.  Measured: a workgroup alone on a CU spends about 0.7 us per
// 128-element stage and two on a CU about 1.25 us for both; a split costs the reducing workgroup
// about a microsecond plus 0.8 us per partial tile it reads.  Hence up to eight splits, each at
// least eight stages (K >= 1024 per split) long; with more tiles than that a split gains nothing
// unless the reduction is long.
int tiled_fast_auto_split(int M, int strips, int steps, int gs) {
    int bm, tiles;
    tiled_fast_tiles(M, strips, gs, &bm, &tiles);
    const int stages = (steps + fast::kStageSteps - 1) / fast::kStageSteps;
    // one workgroup per CU on most CUs and a long reduction: two halves (measured at 128 x 28672 x 8192,
    // 224 tiles of 64 stages: 67.5 -> 61.2 us; at 32 stages per tile the halves are slower: 28.1 -> 31.6 us)
    if (tiles > 128) return tiles <= 256 && stages >= 64 ? 2 : 1;
    int split = 512 / tiles;
    if (split > 8) split = 8;
    if (split > stages / 8) split = stages / 8;
    if (split < 1) split = 1;
    return tiled_fast_effective_split(steps, gs, split, nullptr);
}

// What a requested split comes to: whole stages per split (an even number of them with a group of 256), the last
// split possibly shorter, empty splits dropped.  *groups_per_split, when asked for, is a split's length in groups.
int tiled_fast_effective_split(int steps, int gs, int split, int* groups_per_split) {
    const int stages = (steps + fast::kStageSteps - 1) / fast::kStageSteps;
    if (split < 1) split = 1;
    int sps = (stages + split - 1) / split;
    if (gs == 4) sps = (sps + 1) / 2 * 2;
    if (groups_per_split) *groups_per_split = sps * fast::kStageSteps / gs;
    return (stages + sps - 1) / sps;
}

// in units of 64 x 256 tiles (a 128-row tile counts twice)
size_t tiled_fast_workspace_tiles(int M, int strips, int gs) {
    int bm, tiles;
    tiled_fast_tiles(M, strips, gs, &bm, &tiles);
    return (size_t)tiles * (bm / 64);
}

hipError_t launch_tiled(const GemmParams& p, int gs, bool asym, bool out_bf16, hipStream_t stream) {
    if (p.acc_dump != nullptr && p.dump_mode != 0) return launch_tiled_verify(p, gs, asym, out_bf16, stream);
    return launch_tiled_impl<false>(p, gs, asym, out_bf16, stream);
}

}  // namespace w2a8
