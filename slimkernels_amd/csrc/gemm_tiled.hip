// Fast tiled W2A8 GEMM for gfx950, production instantiations and the launch heuristics (the kernels themselves are in
// tiled_bodies.h; the verification instantiations, which also write out the int32 group sums, in
// gemm_tiled_verify.hip).
#include "tiled_bodies.h"

namespace w2a8 {

size_t tiled_w4_tiles(int M, int strips) {
    return (size_t)((strips + fast::kStrips - 1) / fast::kStrips) * (size_t)((M + 63) / 64);
}

// The split a score of three factors picks among 1, 2, 3, 4, 6 and 8 for `tiles` 64-row tiles of `stages` stages:
//  * how evenly the workgroups fill the CUs: with n = ceil(workgroups / 256) on the fullest CU, workgroups / (256 n);
//  * how well a CU runs with n workgroups on it, relative to a full house: `alone` for one, `paired` for two
//    (nothing hides a lone workgroup's latencies);
//  * what a workgroup spends outside its stages (prologue, epilogue, publishing or adding up partial tiles): about
//    ten stages' worth, so a split of `per` stages is per / (per + 10) efficient.
static int scored_split(int tiles, int stages, double alone, double paired) {
    static const int kCandidates[] = {1, 2, 3, 4, 6, 8};
    int best_split = 1;
    double best_score = -1.0;
    for (int split : kCandidates) {
        const int per = (stages + split - 1) / split;         // stages per split
        if (split > 1 && per < 8) break;                      // (shorter splits were never the best measured)
        const long long wgs = (long long)tiles * ((stages + per - 1) / per);
        const long long n = (wgs + 255) / 256;
        const double fill = (double)wgs / (256.0 * (double)n);
        const double together = n == 1 ? alone : (n == 2 ? paired : 1.0);
        const double score = fill * together * (double)per / ((double)per + 10.0);
        if (score > best_score * 1.0001) {
            best_score = score;
            best_split = split;
        }
    }
    return best_split;
}

// K splits of the one-pass W4 kernel (two workgroups fit a CU): the rule of the 64-row W2 tiles below with the
// factors its own measurements give (thirty shapes, six split values each: within 0.3 % of the best on average, 4 %
// at worst; the rule by tile count it replaces lost up to 26 %).  More than 400 tiles are not split.
int tiled_w4_auto_split(int M, int strips, int steps) {
    const int tiles = (int)tiled_w4_tiles(M, strips);
    const int stages = steps / fast::kStageSteps;
    if (tiles > 400) return 1;
    const int split = scored_split(tiles, stages, 0.8, 1.0);
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

// K splits of the 64-row tiles: scored_split() above with the factors fitted to measurements of 1, 2, 3, 4, 6 and 8
// splits on thirty shapes (64..512 token rows on the Llama-8B and 70B-class linears, groups of 64 and 128): one
// workgroup alone on a CU reaches about 0.7 of what three reach together, two 0.9.  The rule picks within 1 % of the
// best measured split on average, 9 % at worst, where the rule by tile count it replaces lost up to 32 %.
// 128-row tiles (a chip-filling problem) are not split, nor are more than 400 64-row tiles: measured slower (the
// partial tiles of a thousand workgroups are 130 MB of traffic: 2048 x 4096 x 14336 in two halves 151 against 134 us).
// Groups of 256 (two workgroups per CU, not three) keep the rule by tile count they were measured with.
int tiled_fast_auto_split(int M, int strips, int steps, int gs) {
    int bm, tiles;
    tiled_fast_tiles(M, strips, gs, &bm, &tiles);
    if (bm != 64 || tiles > 400) return 1;
    const int stages = (steps + fast::kStageSteps - 1) / fast::kStageSteps;
    if (gs == 4) {
        if (tiles > 128) return tiled_fast_effective_split(steps, gs, tiles <= 256 && stages >= 64 ? 2 : 1, nullptr);
        int split = 512 / tiles;
        if (split > 8) split = 8;
        if (split > stages / 8) split = stages / 8;
        return tiled_fast_effective_split(steps, gs, split < 1 ? 1 : split, nullptr);
    }
    const int best_split = scored_split(tiles, stages, 0.7, 0.9);
    return tiled_fast_effective_split(steps, gs, best_split, nullptr);
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
