// C ABI of the W2A8 path (declared in include/slimk_w2a8.h): argument validation on
// the host, kernel selection, launches.  No allocation, no synchronisation.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <string>

#include "../../include/slimk_w2a8.h"
#include "w2a8_launch.h"

// The library-owned split-K workspace of slimk_w2a8_gemm_static (see static_workspace() below).
static __device__ __align__(256) unsigned char scratch[SLIMK_W2A8_STATIC_WORKSPACE_BYTES];

namespace {

thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

int hip_result(hipError_t e, const char* what) {
    if (e == hipSuccess) return SLIMK_OK;
    return fail(SLIMK_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// common K / group checks; returns 0 or an error code (message set)
int check_kg(int K, int group_size) {
    if (K <= 0 || K % w2a8::kStepK != 0)
        return fail(SLIMK_ERR_BAD_SHAPE, "K=%d must be a positive multiple of 64", K);
    if (group_size != 64 && group_size != 128 && group_size != 256)
        return fail(SLIMK_ERR_BAD_SHAPE, "group_size=%d must be 64, 128 or 256", group_size);
    if (K % group_size != 0)
        return fail(SLIMK_ERR_BAD_SHAPE, "K=%d is not a multiple of group_size=%d", K, group_size);
    return SLIMK_OK;
}

// The kernels address weights and activations through 32-bit buffer offsets.
int check_extent(int M, int N, int K, int ldq) {
    const size_t wbytes = w2a8::weight_bytes((N + w2a8::kStripN - 1) / w2a8::kStripN, K / w2a8::kStepK);
    const size_t qbytes = (size_t)M * (size_t)ldq;
    if (wbytes > 0x7fffffffu || qbytes > 0x7fffffffu)
        return fail(SLIMK_ERR_UNSUPPORTED, "repacked weights (%zu bytes) or activations (%zu bytes) exceed 2 GiB", wbytes, qbytes);
    return SLIMK_OK;
}

bool shape_ok(int K, int group_size) {
    return K > 0 && K % 64 == 0 && (group_size == 64 || group_size == 128 || group_size == 256) &&
           K % group_size == 0;
}

int strips_of(int N) { return (N + w2a8::kStripN - 1) / w2a8::kStripN; }

// A split-K workspace starts with a block of arrival counters of FIXED size, whatever the problem, followed by the
// fp32 partial tiles.  Every kernel leaves the counters it used at zero, and because the block does not move
// with the shape, a workspace zeroed once stays valid for any sequence of problems (a counter block sized by the
// problem would let a later, larger block overlap an earlier call's partial sums).
constexpr size_t kCounterBlockBytes = w2a8::kCounterBlockBytes;
static_assert(kCounterBlockBytes == SLIMK_W2A8_COUNTER_BLOCK_BYTES, "the header names the counter block's size");
constexpr int kMaxCounters = w2a8::kMaxSplitCounters;  // (the block's last two slots belong to the row-quantising kernels)

constexpr int kSkinnyMaxRows = 256;

// The skinny kernel partitions K in chunks of four 64-element steps; a split owns whole chunks.
int chunk_groups(int group_size) { return group_size >= 256 ? 1 : 256 / group_size; }

// Groups per split for a requested split factor, rounded up to whole chunks; the effective split
// (number of non-empty splits) is ceil(G / groups_per_split) <= requested.
int groups_per_split(int G, int group_size, int split) {
    const int cg = chunk_groups(group_size);
    int gps = (G + split - 1) / split;
    return (gps + cg - 1) / cg * cg;
}

// The shared-activation workgroups (eight waves = two k-parts x four strips whose waves fetch the activations once)
// as a launch of one problem: K is split across workgroups until about 256 exist, as long as a wave keeps at least
// six chunks of four steps.
constexpr size_t kSharedMinWeightBytes = (size_t)24 << 20;
constexpr int kSharedParts = w2a8::kSharedParts;
// 12..16 rows on 384 strips and more take the form with four k-parts x two strips: one strip per workgroup leaves
// 448 four-wave workgroups on 256 CUs, a quarter of the CUs with half the load, and every strip fetches the
// activations for itself (28672 x 8192 at 14 / 16 rows: 18.9 / 18.8 -> 17.3 / 17.4 us, 28672 x 4096: 10.7 / 11.1 ->
// 10.0 us, 32768 x 8192 at 12 rows: 18.2 -> 16.5 us; at 10 rows and below, and on 256 strips and fewer, the one-strip
// kernel is ahead or level).
constexpr int kWideSharedStrips = 384, kWideSharedRows = 12;
int skinny_shared_parts(int M, int N) { return M <= 16 && strips_of(N) >= kWideSharedStrips ? 2 * kSharedParts : kSharedParts; }
int skinny_shared_split(int M, int N, int K, int group_size) {
    const int parts = skinny_shared_parts(M, N);
    const int per_unit = w2a8::kGroupedWavesPerWg / parts;
    const int units = (strips_of(N) + per_unit - 1) / per_unit * ((M + 15) / 16);
    const int chunks = (K / 64 + 3) / 4;
    int split = (256 + units / 2) / units;
    if (split > chunks / (parts * 6)) split = chunks / (parts * 6);
    // never a few workgroups more than CUs: they would run as a second round (12288 x 12288 at 17..32 rows, 96 units:
    // 22.6 us at three splits, 20.1 us at two)
    while (split > 1 && units * split > 256) --split;
    if (split < 1) split = 1;
    const int G = K / group_size;
    const int gps = groups_per_split(G, group_size, split);
    return (G + gps - 1) / gps;
}

// K splits of the one-strip skinny kernel, from a sweep of waves x splits on eleven shapes at 1, 4 and 16 token rows:
// a split costs its workgroups a round trip through the workspace (about 0.8 us), so it pays only for long reductions
// (128 steps and more); never more workgroups than CUs, and every wave of a part keeps a chunk of four steps.
int skinny_plain_split(int N, int K, int group_size) {
    const int strips = strips_of(N);
    const int G = K / group_size;
    const int steps = K / 64;
    int split = 1;
    if (strips <= 128 && steps >= 128) split = std::min(256 / strips, steps / 32);
    if (split > 32) split = 32;
    const int gps = groups_per_split(G, group_size, split);
    return (G + gps - 1) / gps;
}

// 33..256 token rows: four kernels can take the problem.
//   plain  - the one-strip skinny kernel, 16 rows at a time, the passes side by side as workgroups of their own (each
//            re-reading weights and activations, all but the first out of L2): the fastest while the workgroups are
//            few (4096 x 4096: 5.6 us at 33 rows, tiled 17.3).
//   shared - the shared-activation workgroups (four strips x two k-parts fetch a row block's activations once): a
//            quarter of the plain kernel's workgroups at a higher cost each (11008 x 4096 at 80 rows: 13.5 us, plain
//            16.0, tiled 20.8; 4096 x 28672 at 33..80 rows: 24.3..33.1 us, tiled 39.5..40.7).
//   tiled  - 64 x 256 tiles through LDS: the cheapest per row once the rows fill its tiles and the reduction is long
//            enough to amortise its start-up.
//   strips - SLIMK_KERNEL_MID, four strips x every row of a row part per workgroup: ahead where 64-row tiles would run
//            mostly empty on a large matrix (28672 x 8192, groups of 64: 36.7 -> 32.3 us at 33 rows, 57.6 -> 46.4 at 80;
//            16384 x 16384: 51.4 -> 42.4 at 80, 68.4 -> 60.2 at 130).
// The choice is the smallest of four predicted times.  Each prediction is a start-up cost, a cost of splitting K
// across workgroups, and rounds of workgroups (256: one per CU; the strips form runs two per CU side by side) times a
// cost per round that grows with the steps a workgroup (plain, tiled, strips) or a wave (shared) runs through; plain and
// shared also pay for the weights' first trip from HBM, groups of 64 cost every form more per step.  The coefficients
// are a least-squares fit (on the logarithm of predicted / measured) to 615 timed cases: all four kernels on 32
// matrices (1024..28672 channels, K = 3072..28672, 1..64 MiB) at 33, 48, 64, 80, 96, 128, 160 and 256 rows in groups of
// 128, eight of them also in groups of 64 and of 256, and further row counts (40..240) on twelve, weights streamed from
// HBM: picking by the prediction costs 0.5 % over the best kernel of each case on average (worst case 15 %; fitted
// on two thirds of the matrices and judged on the rest: 0.4..1.0 %; a three-way prediction with size rules for the
// strips form, which this replaces: 2.2 %, up to 47 %).
// Reductions of up to 2048 elements keep the rule they were measured with (plain while its passes over the weights
// stay under 100 MiB).
enum MidRoute { kMidPlain, kMidShared, kMidTiled, kMidStrips };
int mid_split(int M, int N, int K, int group_size);
// skinny_only: the faster of the two skinny forms (what an explicit request for the skinny kernel runs)
MidRoute mid_route(int M, int N, int K, int group_size, bool skinny_only = false) {
    if (M > kSkinnyMaxRows) return skinny_only ? kMidPlain : kMidTiled;
    const int strips = strips_of(N), steps = K / w2a8::kStepK, blocks = (M + 15) / 16;
    const size_t weight_bytes = (size_t)strips * 64 * (K / 4);
    if (K <= 2048) return skinny_only || (size_t)blocks * weight_bytes <= ((size_t)100 << 20) ? kMidPlain : kMidTiled;
    const float weight_mib = (float)weight_bytes / 1048576.0f;
    // a step costs more in groups of 64 and less in groups of 256 and more than in groups of 128: factors per form
    const auto by_group = [&](float of64, float of256) { return group_size == 64 ? of64 : (group_size >= 256 ? of256 : 1.0f); };
    const auto rounds = [](long long wgs, float smooth) {  // between whole rounds and the plain ratio
        const float whole = (float)((wgs + 255) / 256), ratio = std::max(1.0f, (float)wgs / 256.0f);
        return smooth * ratio + (1.0f - smooth) * whole;
    };
    const int plain_split = skinny_plain_split(N, K, group_size);
    const float plain_cost = 2.569f + (plain_split > 1 ? 3.476f : 0.0f) + 0.1133f * weight_mib +
                             rounds((long long)strips * plain_split * blocks, 0.473f) *
                                 (0.961f + 0.0356f * (float)steps / (float)plain_split) * by_group(1.086f, 0.939f);
    const int shared_split = skinny_shared_split(M, N, K, group_size);
    const int units = (strips + 3) / 4 * blocks;
    const float shared_cost = 6.125f + (shared_split > 1 ? 2.584f : 0.0f) + 0.0599f * weight_mib +
                              rounds((long long)units * shared_split, 0.318f) *
                                  (-0.321f + 0.2239f * (float)steps / (2.0f * (float)shared_split)) * by_group(1.337f, 0.805f);
    if (skinny_only) return plain_cost <= shared_cost ? kMidPlain : kMidShared;
    float tiled_cost = 1e30f, strips_cost = 1e30f;
    if (group_size <= 256) {
        const int gs = group_size / w2a8::kStepK;
        const int tiled_split = w2a8::tiled_fast_auto_split(M, strips, steps, gs);
        const int tiles = (int)w2a8::tiled_fast_workspace_tiles(M, strips, gs);
        const int stages = (steps + 1) / 2;
        const int per = (stages + tiled_split - 1) / tiled_split;
        const int n = (tiles * tiled_split + 255) / 256;  // workgroups per CU: up to three run side by side
        const float together = n == 1 ? 1.0f : (n == 2 ? 1.515f : (n == 3 ? 2.136f : 0.695f * (float)n));
        tiled_cost = -0.846f + (tiled_split > 1 ? 7.117f : 0.0f) +
                     ((float)per + 8.09f) * 0.7121f * together * by_group(1.245f, 0.915f);
        // (a split launch of the strips form needs an arrival counter per strip and row block)
        if (M <= w2a8::kMidMaxRows && (size_t)strips * blocks <= (size_t)kMaxCounters) {
            const int split = mid_split(M, N, K, group_size);
            const int mb = w2a8::mid_row_blocks(M), piece_steps = w2a8::mid::piece_steps(gs);
            const long long wgs = (long long)((strips + w2a8::mid::kWaves - 1) / w2a8::mid::kWaves) * w2a8::mid_row_parts(M) * split;
            const float turns = (float)(((wgs + 255) / 256 + 1) / 2);   // two workgroups of a CU run side by side ...
            const float pair = wgs > 256 ? 1.730f : 1.0f;                // ... each slower than one alone
            const float pieces = (float)((steps / piece_steps + split - 1) / split);
            const float piece = (0.3812f + 0.0786f * (float)mb) * by_group(0.675f, 1.014f);   // (a piece of groups of 64 is one step)
            strips_cost = 5.845f + (split > 1 ? 3.211f * (float)mb - 3.363f : 0.0f) + turns * pair * pieces * piece;
        }
    }
    const float skinny_cost = std::min(plain_cost, shared_cost), other_cost = std::min(tiled_cost, strips_cost);
    if (skinny_cost <= other_cost) return plain_cost <= shared_cost ? kMidPlain : kMidShared;
    return tiled_cost <= strips_cost ? kMidTiled : kMidStrips;
}


// The kernel for 33..256 rows (a workgroup = four strips x the rows of a row part): K splits across workgroups in
// rounds of four pieces (a piece = two 64-element steps, one with groups of 64).  Two workgroups on a CU run side by
// side in about the time of one, a third waits for a place: the split is the largest power of two (up to 8) that keeps
// the launch within 512 workgroups and every workgroup at two rounds or more (28672 x 8192 at 33 rows, 112 strip sets:
// 59.7 / 38.1 / 39.4 / 32.3 / 39.2 / 36.6 us at 1 / 2 / 3 / 4 / 6 / 8 splits; splits that are no power of two measured
// behind their neighbours on every shape).
int mid_groups_per_split(int G, int group_size, int split) {
    const int gs = group_size / w2a8::kStepK;
    const int round_groups = std::max(1, w2a8::mid::kPiecesPerRound * w2a8::mid::piece_steps(gs) / gs);  // groups per round
    const int gps = (G + split - 1) / split;
    return (gps + round_groups - 1) / round_groups * round_groups;
}
int mid_split(int M, int N, int K, int group_size) {
    const int units = (strips_of(N) + w2a8::mid::kWaves - 1) / w2a8::mid::kWaves * w2a8::mid_row_parts(M);
    const int G = K / group_size, gs = group_size / w2a8::kStepK;
    const int pieces = K / w2a8::kStepK / w2a8::mid::piece_steps(gs);
    int split = 1;
    while (split < 8 && units * split * 2 <= 512 && pieces / (split * 2) >= 2 * w2a8::mid::kPiecesPerRound) split *= 2;
    const int gps = mid_groups_per_split(G, group_size, split);
    return (G + gps - 1) / gps;
}

int resolve_kernel(int M, int N, int K, int group_size, int kernel) {
    if (kernel == SLIMK_KERNEL_AUTO) {
        if (M <= 32) return SLIMK_KERNEL_SKINNY;
        const MidRoute r = mid_route(M, N, K, group_size);
        return r == kMidTiled ? SLIMK_KERNEL_TILED : (r == kMidStrips ? SLIMK_KERNEL_MID : SLIMK_KERNEL_SKINNY);
    }
    return kernel;
}

// One problem with 17..32 token rows on a matrix big enough to be bound by bandwidth goes through the shared-activation
// workgroups: 8..27 % faster there than one strip per workgroup (at 16 rows and below the one-strip kernel is as fast
// or faster); with more rows, where it is predicted the faster of the two skinny forms (which is also what an explicit
// request for the skinny kernel runs on a shape that SLIMK_KERNEL_AUTO gives to another kernel).
bool skinny_shared_applies(int M, int N, int K, int group_size) {
    if (M >= kWideSharedRows && M <= 16) return strips_of(N) >= kWideSharedStrips;
    if (M <= 16 || M > kSkinnyMaxRows) return false;
    if (M <= 32) return (size_t)strips_of(N) * 64 * (K / 4) >= kSharedMinWeightBytes;
    return mid_route(M, N, K, group_size, true) == kMidShared;
}

int auto_split(int M, int N, int K, int group_size, int kernel) {
    if (kernel == SLIMK_KERNEL_MID) return mid_split(M, N, K, group_size);
    if (kernel != SLIMK_KERNEL_SKINNY) {
        // the fast tiled kernel splits K when its tiles would leave CUs idle (groups of up to 256)
        if (group_size > 256) return 1;
        return w2a8::tiled_fast_auto_split(M, strips_of(N), K / w2a8::kStepK, group_size / w2a8::kStepK);
    }
    if (skinny_shared_applies(M, N, K, group_size)) return skinny_shared_split(M, N, K, group_size);
    return skinny_plain_split(N, K, group_size);
}

// Wavefronts per workgroup of the skinny kernel (the in-workgroup split of K).  Split runs: eight (sixteen measured
// 3..9 % slower on every split shape of the sweep).  Unsplit with at most four token rows and at most one workgroup
// per CU (256 strips): eight waves per strip instead of four shorten each wave's run and put more loads in flight on
// a CU (4096 x 4096, M = 1: 5.09 -> 4.72 us; 11008 x 8192: 8.3 -> 7.2 us; 12288 x 12288: 11.5 -> 9.8 us); with
// more strips than CUs (28672 x 8192: 12.9 -> 14.4 us) and with more rows they lose.
// slimk_w2a8_gemm_fused: up to four rows of at most 32 KiB of int8 values together are quantised by every workgroup for
// itself into LDS; more rows (up to 32) or longer ones by the grid's first workgroups into the workspace.
bool fused_in_workgroup(int M, int K) { return M <= w2a8::kFusedMaxRows && (size_t)M * K <= (size_t)w2a8::kFusedMaxBytes; }
size_t fused_rows_q_bytes(int K) { return ((size_t)w2a8::kRowsMax * K + 255) / 256 * 256; }
size_t fused_rows_area_bytes(int K, int G) {  // int8 rows, 32 token scales, group sums [G][32]
    return fused_rows_q_bytes(K) + 256 + ((size_t)G * w2a8::kRowsMax * 4 + 255) / 256 * 256;
}
// polls of the row-quantising kernels' wait before a workgroup quantises the rows itself (a poll is about a microsecond)
std::atomic<int> g_rows_spin_limit{20000};

int skinny_waves(int M, int N, int K, int split) {
    if (split > 1) return 8;
    return M <= 4 && strips_of(N) <= 256 && K >= 2048 ? 8 : 4;
}

}  // namespace

extern "C" {

int slimk_w2a8_version(void) { return SLIMK_W2A8_VERSION; }
const char* slimk_w2a8_arch(void) { return "gfx950"; }
const char* slimk_w2a8_last_error(void) { return g_last_error.c_str(); }

size_t slimk_w2a8_repacked_weight_bytes(int N, int K) {
    if (N <= 0 || K <= 0 || K % 64 != 0) return 0;
    return w2a8::weight_bytes(strips_of(N), K / 64);
}

size_t slimk_w2a8_repacked_scale_bytes(int N, int K, int group_size) {
    if (N <= 0 || !shape_ok(K, group_size)) return 0;
    return (size_t)strips_of(N) * (K / group_size) * 64 * 2;
}

size_t slimk_w2a8_repacked_zp_bytes(int N, int K, int group_size) {
    if (N <= 0 || !shape_ok(K, group_size)) return 0;
    return (size_t)strips_of(N) * (K / group_size) * 64;
}

int slimk_w2a8_gemm_auto_split_k(int M, int N, int K, int group_size, int kernel) {
    if (M <= 0 || N <= 0 || !shape_ok(K, group_size)) return 0;
    return auto_split(M, N, K, group_size, resolve_kernel(M, N, K, group_size, kernel));
}

int slimk_w2a8_gemm_auto_route(int M, int N, int K, int group_size) {
    if (M <= 0 || N <= 0 || !shape_ok(K, group_size)) return 0;
    const int kern = resolve_kernel(M, N, K, group_size, SLIMK_KERNEL_AUTO);
    if (kern == SLIMK_KERNEL_TILED) return 2;
    if (kern == SLIMK_KERNEL_MID) return 4;
    return skinny_shared_applies(M, N, K, group_size) ? 3 : 1;
}

size_t slimk_w2a8_gemm_workspace_bytes(int M, int N, int K, int group_size, int kernel, int split_k) {
    if (M <= 0 || N <= 0 || !shape_ok(K, group_size)) return 0;
    const int kern = resolve_kernel(M, N, K, group_size, kernel);
    if (split_k <= 0) split_k = auto_split(M, N, K, group_size, kern);
    if (split_k <= 1) return 0;
    const int strips = strips_of(N);
    if (kern == SLIMK_KERNEL_TILED) {  // one arrival counter and `split_k` fp32 tiles of 64 x 256 per 64-row tile
        const size_t tiles = w2a8::tiled_fast_workspace_tiles(M, strips, group_size / w2a8::kStepK);
        return kCounterBlockBytes + (size_t)split_k * tiles * 64 * 256 * sizeof(float);
    }
    const int mblocks = (M + 15) / 16;  // one tile and one arrival counter per (strip, block of 16 rows)
    const size_t tile = (size_t)16 * w2a8::kStripN;
    return kCounterBlockBytes + (size_t)split_k * strips * mblocks * tile * sizeof(float);
}

int slimk_w2a8_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
    if (workspace_bytes == 0) return SLIMK_OK;
    if (!workspace) return fail(SLIMK_ERR_NULL_POINTER, "workspace is NULL");
    if (!aligned16(workspace) || workspace_bytes % 4 != 0)
        return fail(SLIMK_ERR_MISALIGNED, "workspace must be 16-byte aligned and a multiple of 4 bytes");
    return hip_result(w2a8::launch_fill_zero(workspace, workspace_bytes, (hipStream_t)stream), "workspace_init");
}

int slimk_w2a8_repack(const uint8_t* w_packed, int ldw, const uint16_t* scales, const uint8_t* zp,
                      int N, int K, int group_size,
                      uint32_t* w_r, uint16_t* s_r, uint8_t* zp_r, void* stream) {
    if (!w_packed || !scales || !w_r || !s_r) return fail(SLIMK_ERR_NULL_POINTER, "repack: NULL buffer");
    if (zp && !zp_r) return fail(SLIMK_ERR_NULL_POINTER, "repack: zp given but zp_r is NULL");
    if (N <= 0) return fail(SLIMK_ERR_BAD_SHAPE, "N=%d must be positive", N);
    if (int rc = check_kg(K, group_size)) return rc;
    if (ldw < K / 4) return fail(SLIMK_ERR_BAD_SHAPE, "ldw=%d is smaller than K/4=%d", ldw, K / 4);
    if (!aligned16(w_r) || !aligned16(s_r) || (zp_r && !aligned16(zp_r)))
        return fail(SLIMK_ERR_MISALIGNED, "repack: outputs must be 16-byte aligned");
    return hip_result(w2a8::launch_repack(w_packed, ldw, scales, zp, N, K, group_size, w_r, s_r, zp_r,
                                          (hipStream_t)stream),
                      "repack");
}

int slimk_w2a8_quantize_weight(const void* w, int ldw, int w_dtype, int N, int K, int group_size, int mode,
                               uint8_t* packed, int ldp, uint16_t* scales, uint8_t* zp, void* stream) {
    if (!w || !packed || !scales) return fail(SLIMK_ERR_NULL_POINTER, "quantize_weight: NULL buffer");
    if (N <= 0) return fail(SLIMK_ERR_BAD_SHAPE, "N=%d must be positive", N);
    if (int rc = check_kg(K, group_size)) return rc;
    if (w_dtype != SLIMK_F16 && w_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "w_dtype=%d", w_dtype);
    if (mode < SLIMK_QUANT_REF || mode > SLIMK_QUANT_ASYM) return fail(SLIMK_ERR_BAD_ENUM, "mode=%d", mode);
    if (mode == SLIMK_QUANT_ASYM && !zp) return fail(SLIMK_ERR_NULL_POINTER, "quantize_weight: per-group zero-points need zp");
    if (ldw < K || ldp < K / 4) return fail(SLIMK_ERR_BAD_SHAPE, "ldw=%d / ldp=%d too small for K=%d", ldw, ldp, K);
    if (K / 8 > 65535 * 256) return fail(SLIMK_ERR_UNSUPPORTED, "K=%d too long", K);
    if (!aligned16(w) || ldw % 8 != 0 || (reinterpret_cast<uintptr_t>(packed) & 1u) || ldp % 2 != 0 ||
        (reinterpret_cast<uintptr_t>(scales) & 1u))
        return fail(SLIMK_ERR_MISALIGNED, "quantize_weight: w 16-byte aligned, ldw %% 8 == 0, packed / ldp / scales 2-byte aligned");
    return hip_result(w2a8::launch_quantize_weight(w, ldw, w_dtype == SLIMK_BF16, N, K, group_size, mode, packed, ldp,
                                                   scales, zp, (hipStream_t)stream),
                      "quantize_weight");
}

int slimk_w2a8_quantize_weight4(const void* w, int ldw, int w_dtype, int N, int K, int group_size, int mode,
                                uint8_t* planes, int ldp, uint16_t* scales2, uint8_t* zp2, void* stream) {
    if (!w || !planes || !scales2 || !zp2) return fail(SLIMK_ERR_NULL_POINTER, "quantize_weight4: NULL buffer");
    if (N <= 0) return fail(SLIMK_ERR_BAD_SHAPE, "N=%d must be positive", N);
    if (int rc = check_kg(K, group_size)) return rc;
    if (w_dtype != SLIMK_F16 && w_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "w_dtype=%d", w_dtype);
    if (mode != SLIMK_QUANT_SYM && mode != SLIMK_QUANT_ASYM) return fail(SLIMK_ERR_BAD_ENUM, "mode=%d (SYM or ASYM)", mode);
    if (ldw < K || ldp < K / 2) return fail(SLIMK_ERR_BAD_SHAPE, "ldw=%d / ldp=%d too small for K=%d", ldw, ldp, K);
    if (!aligned16(w) || ldw % 8 != 0 || (reinterpret_cast<uintptr_t>(planes) & 1u) || ldp % 2 != 0 ||
        (reinterpret_cast<uintptr_t>(scales2) & 1u))
        return fail(SLIMK_ERR_MISALIGNED, "quantize_weight4: w 16-byte aligned, ldw %% 8 == 0, planes / ldp / scales2 2-byte aligned");
    return hip_result(w2a8::launch_quantize_weight4(w, ldw, w_dtype == SLIMK_BF16, N, K, group_size, mode == SLIMK_QUANT_ASYM,
                                                    planes, ldp, scales2, zp2, (hipStream_t)stream),
                      "quantize_weight4");
}

int slimk_w2a8_act_quant_rep(const void* x, int ldx, int x_dtype, int M, int K, int group_size, int copies,
                             int8_t* q, int ldq, float* s_a, int32_t* rowsum, int ldr, void* stream) {
    if (!x || !q || !s_a) return fail(SLIMK_ERR_NULL_POINTER, "act_quant: NULL buffer");
    if (M <= 0) return fail(SLIMK_ERR_BAD_SHAPE, "M=%d must be positive", M);
    if (copies < 1 || copies > 4) return fail(SLIMK_ERR_BAD_SHAPE, "copies=%d must be 1..4", copies);
    if (int rc = check_kg(K, group_size)) return rc;
    if (x_dtype != SLIMK_F16 && x_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "x_dtype=%d", x_dtype);
    if (ldx < K || (long long)ldq < (long long)copies * K)
        return fail(SLIMK_ERR_BAD_SHAPE, "ldx=%d smaller than K=%d or ldq=%d smaller than copies * K", ldx, K, ldq);
    if (rowsum && ldr < M) return fail(SLIMK_ERR_BAD_SHAPE, "ldr=%d smaller than M=%d", ldr, M);
    if (!aligned16(x) || !aligned16(q) || ldx % 8 != 0 || ldq % 16 != 0)
        return fail(SLIMK_ERR_MISALIGNED, "act_quant: x, q must be 16-byte aligned, ldx %% 8 == 0, ldq %% 16 == 0");
    if (rowsum && (!aligned16(rowsum) || ldr % 4 != 0))
        return fail(SLIMK_ERR_MISALIGNED, "act_quant: rowsum must be 16-byte aligned and ldr %% 4 == 0");
    return hip_result(w2a8::launch_act_quant(x, ldx, x_dtype == SLIMK_BF16, M, K, group_size, q, ldq, s_a,
                                             rowsum, ldr, copies, (hipStream_t)stream),
                      "act_quant");
}

int slimk_w2a8_act_quant(const void* x, int ldx, int x_dtype, int M, int K, int group_size,
                         int8_t* q, int ldq, float* s_a, int32_t* rowsum, int ldr, void* stream) {
    return slimk_w2a8_act_quant_rep(x, ldx, x_dtype, M, K, group_size, 1, q, ldq, s_a, rowsum, ldr, stream);
}

}  // extern "C"

namespace {

int static_workspace(void** ptr, hipStream_t stream);

// fit_split: the call is slimk_w2a8_gemm_static's: `workspace` is NULL and workspace_bytes the size of the library-owned
// array; a split factor chosen here (split_k <= 0) is lowered until its workspace fits that size (a caller's explicit
// split never is), and the array itself is looked up only once every argument has passed validation and the launch
// turns out to split K.
int gemm_impl(const int8_t* q, int ldq, const float* s_a, const int32_t* rowsum, int ldr,
              const uint32_t* w_r, const uint16_t* s_r, const uint8_t* zp_r, int zp_const,
              int M, int N, int K, int group_size,
              void* out, int ldo, int out_dtype,
              int32_t* acc_dump, int dump_mode,
              void* workspace, size_t workspace_bytes,
              int kernel, int split_k, void* stream, bool fit_split) {
    if (!q || !s_a || !w_r || !s_r || !out) return fail(SLIMK_ERR_NULL_POINTER, "gemm: NULL buffer");
    if (M <= 0 || N <= 0) return fail(SLIMK_ERR_BAD_SHAPE, "M=%d, N=%d must be positive", M, N);
    if (int rc = check_kg(K, group_size)) return rc;
    // the row sums fold zero-points; the fast tiled kernel centres its operand bytes on 2 and reads none for that value
    const int kern_for_rowsum = resolve_kernel(M, N, K, group_size, kernel);
    const bool rowsum_unused = !zp_r && zp_const == 2 && group_size <= 256 &&
                               (kern_for_rowsum == SLIMK_KERNEL_TILED || kern_for_rowsum == SLIMK_KERNEL_MID);
    if (!rowsum && !rowsum_unused)
        return fail(SLIMK_ERR_NULL_POINTER, "gemm: rowsum is NULL (only the tiled kernel and SLIMK_KERNEL_MID, with the uniform zero-point 2 and a group size of at most 256, do without)");
    if (!rowsum) ldr = (M + 3) / 4 * 4;
    if (out_dtype != SLIMK_F16 && out_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "out_dtype=%d", out_dtype);
    if (kernel < SLIMK_KERNEL_AUTO || kernel > SLIMK_KERNEL_MID) return fail(SLIMK_ERR_BAD_ENUM, "kernel=%d", kernel);
    if (dump_mode < SLIMK_DUMP_NONE || dump_mode > SLIMK_DUMP_SUM) return fail(SLIMK_ERR_BAD_ENUM, "dump_mode=%d", dump_mode);
    if (dump_mode != SLIMK_DUMP_NONE && !acc_dump) return fail(SLIMK_ERR_NULL_POINTER, "gemm: dump_mode set but acc_dump is NULL");
    if (ldq < K || ldo < N || ldr < M) return fail(SLIMK_ERR_BAD_SHAPE, "gemm: ldq=%d, ldo=%d or ldr=%d too small", ldq, ldo, ldr);
    if (zp_const < 0 || zp_const > 3) return fail(SLIMK_ERR_BAD_SHAPE, "zp_const=%d must be 0..3", zp_const);
    if (int rc = check_extent(M, N, K, ldq)) return rc;
    if (!aligned16(q) || ldq % 16 != 0 || (rowsum && (!aligned16(rowsum) || ldr % 4 != 0)) || !aligned16(w_r) ||
        !aligned16(s_r) || (zp_r && !aligned16(zp_r)))
        return fail(SLIMK_ERR_MISALIGNED, "gemm: q, rowsum, w_r, s_r, zp_r must be 16-byte aligned; ldq %% 16 == 0; ldr %% 4 == 0");
    if ((reinterpret_cast<uintptr_t>(out) & 1u) != 0) return fail(SLIMK_ERR_MISALIGNED, "gemm: out must be 2-byte aligned");

    const int kern = resolve_kernel(M, N, K, group_size, kernel);
    if (kern == SLIMK_KERNEL_SKINNY && M > kSkinnyMaxRows)
        return fail(SLIMK_ERR_UNSUPPORTED, "the skinny kernel handles M <= %d (M=%d)", kSkinnyMaxRows, M);
    if (kern == SLIMK_KERNEL_MID && (M > w2a8::kMidMaxRows || group_size > 256))
        return fail(SLIMK_ERR_UNSUPPORTED, "SLIMK_KERNEL_MID handles M <= %d and groups of up to 256 (M=%d, group_size=%d)",
                    w2a8::kMidMaxRows, M, group_size);
    const int G = K / group_size;
    const bool split_chosen_here = split_k <= 0;
    if (split_k <= 0) {
        split_k = auto_split(M, N, K, group_size, kern);
        if (fit_split)
            while (split_k > 1 && slimk_w2a8_gemm_workspace_bytes(M, N, K, group_size, kern, split_k) > workspace_bytes) --split_k;
    }
    if (split_k > G) return fail(SLIMK_ERR_BAD_SHAPE, "split_k=%d exceeds the number of groups %d", split_k, G);
    int gps;
    if (kern == SLIMK_KERNEL_TILED) {
        // only the fast kernel (groups of up to 256) splits K
        w2a8::GemmParams probe{};
        probe.acc_dump = dump_mode != SLIMK_DUMP_NONE ? acc_dump : nullptr; probe.dump_mode = dump_mode;
        probe.zp_const = zp_const; probe.steps = K / w2a8::kStepK;
        const int gs_t = group_size / w2a8::kStepK;
        const bool can = w2a8::tiled_fast_supported(probe, gs_t, zp_r != nullptr) &&
                         w2a8::tiled_fast_max_split(M, strips_of(N), K / w2a8::kStepK, gs_t) > 1 &&
                         (size_t)split_k * w2a8::tiled_fast_workspace_tiles(M, strips_of(N), gs_t) * 64 * 256 * 4 < 0x7fffffffu;
        if (split_k > 1 && !can) {
            if (!split_chosen_here)
                return fail(SLIMK_ERR_UNSUPPORTED, "this tiled GEMM cannot split K (split_k=%d)", split_k);
            split_k = 1;
        }
        gps = G;
        if (split_k > 1)  // effective split: whole 128-element stages (256 with that group size) per split
            split_k = w2a8::tiled_fast_effective_split(K / w2a8::kStepK, gs_t, split_k, &gps);
        if (split_k <= 1) gps = G;
    } else {
        gps = kern == SLIMK_KERNEL_MID ? mid_groups_per_split(G, group_size, split_k) : groups_per_split(G, group_size, split_k);
        split_k = (G + gps - 1) / gps;  // effective split: the request is an upper bound (whole chunks / rounds per split)
    }

    w2a8::GemmParams p{};
    p.q = q; p.s_a = s_a; p.rowsum = rowsum; p.w_r = w_r; p.s_r = s_r; p.zp_r = zp_r;
    p.out = out; p.acc_dump = dump_mode != SLIMK_DUMP_NONE ? acc_dump : nullptr;
    p.ldq = ldq; p.ldr = ldr; p.ldo = ldo;
    p.M = M; p.N = N; p.K = K; p.G = G; p.steps = K / w2a8::kStepK; p.strips = strips_of(N);
    p.zp_const = zp_const; p.dump_mode = dump_mode;
    p.split = split_k; p.groups_per_split = gps;

    if (split_k > 1) {
        const size_t need = slimk_w2a8_gemm_workspace_bytes(M, N, K, group_size, kern, split_k);
        if (fit_split && workspace_bytes < need)
            return fail(SLIMK_ERR_WORKSPACE, "gemm_static: split_k=%d needs %zu bytes of workspace, the library-owned one holds %zu "
                        "(pass a smaller split_k, 0 to let the library choose one that fits, or use slimk_w2a8_gemm)",
                        split_k, need, workspace_bytes);
        if (fit_split)
            if (int rc = static_workspace(&workspace, (hipStream_t)stream)) return rc;
        if (need - kCounterBlockBytes >= 0x7fffffffu)
            return fail(SLIMK_ERR_UNSUPPORTED, "split_k=%d: %zu bytes of partial sums, 2 GiB or more", split_k, need - kCounterBlockBytes);
        if (!workspace) return fail(SLIMK_ERR_WORKSPACE, "split_k=%d needs a workspace of %zu bytes", split_k, need);
        if (workspace_bytes < need)
            return fail(SLIMK_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes, need);
        if (!aligned16(workspace)) return fail(SLIMK_ERR_MISALIGNED, "workspace must be 16-byte aligned");
        p.ws_counter = reinterpret_cast<unsigned*>(workspace);
        const int counters = kern != SLIMK_KERNEL_TILED ? p.strips * ((M + 15) / 16)
                                                         : (int)w2a8::tiled_fast_workspace_tiles(M, p.strips, group_size / w2a8::kStepK);
        if (counters > kMaxCounters)
            return fail(SLIMK_ERR_UNSUPPORTED, "split_k over %d output tiles (at most %d arrival counters)", counters, kMaxCounters);
        p.ws_partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kCounterBlockBytes);
    }

    hipStream_t st = (hipStream_t)stream;
    if (dump_mode == SLIMK_DUMP_SUM) {
        if (int rc = hip_result(w2a8::launch_fill_zero(acc_dump, (size_t)M * N * sizeof(int32_t), st), "dump clear")) return rc;
    }
    const int gs = group_size / w2a8::kStepK;
    const bool asym = zp_r != nullptr;
    const bool out_bf16 = out_dtype == SLIMK_BF16;
    // a call with a dump runs the verification instantiation of the kernel the same call without one would run
    const bool dump = p.acc_dump != nullptr;
    if (kern == SLIMK_KERNEL_MID)
        return hip_result(dump ? w2a8::launch_mid_verify(p, gs, asym, out_bf16, st) : w2a8::launch_mid(p, gs, asym, out_bf16, st), "mid gemm");
    if (kern == SLIMK_KERNEL_SKINNY && skinny_shared_applies(M, N, K, group_size))
        return hip_result(dump ? w2a8::launch_skinny_shared_verify(p, gs, skinny_shared_parts(M, N), asym, out_bf16, st)
                               : w2a8::launch_skinny_shared(p, gs, skinny_shared_parts(M, N), asym, out_bf16, st), "shared skinny gemm");
    if (kern == SLIMK_KERNEL_SKINNY)
        return hip_result(dump ? w2a8::launch_skinny_verify(p, gs, skinny_waves(M, N, K, split_k), asym, out_bf16, st)
                               : w2a8::launch_skinny(p, gs, skinny_waves(M, N, K, split_k), asym, out_bf16, st), "skinny gemm");
    return hip_result(w2a8::launch_tiled(p, gs, asym, out_bf16, st), "tiled gemm");
}

// ---- the library-owned split-K workspace of slimk_w2a8_gemm_static: a device array of fixed size, one copy per GPU
// the library runs on, held until the process ends.  Its name is a host-side stand-in, not a device address:
// the address on the current device comes from hipGetSymbolAddress, once per device, and only that pointer is
// ever handed to a kernel.
constexpr size_t kStaticWorkspaceBytes = SLIMK_W2A8_STATIC_WORKSPACE_BYTES;
static_assert(kStaticWorkspaceBytes > kCounterBlockBytes && kStaticWorkspaceBytes % 256 == 0, "static workspace size");

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices];   // per device: where that device's copy of `scratch` lives (nullptr: not asked yet)

// The current device's copy of the array; on the first call on a device its counter block is cleared on `stream`
// (the array starts as zeros and every GEMM leaves its counters at zero, so this only guards the very first use).
// That first use must not fall inside a stream capture: the clear would be recorded into the caller's graph.
int static_workspace(void** ptr, hipStream_t stream) {
    int dev = -1;
    if (hipError_t e = hipGetDevice(&dev)) return hip_result(e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(SLIMK_ERR_UNSUPPORTED, "device ordinal %d (at most %d devices)", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipError_t e = hipStreamIsCapturing(stream, &cap)) return hip_result(e, "hipStreamIsCapturing");
        if (cap != hipStreamCaptureStatusNone)
            return fail(SLIMK_ERR_UNSUPPORTED, "gemm_static: the first split-K call on a device sets the library-owned workspace up "
                        "and must be made outside stream capture");
        void* p = nullptr;
        if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch))) return hip_result(e, "hipGetSymbolAddress(scratch)");
        if (!p || !aligned16(p)) return fail(SLIMK_ERR_HIP, "hipGetSymbolAddress(scratch) returned %p", p);
        if (int rc = hip_result(w2a8::launch_fill_zero(p, kCounterBlockBytes, stream), "static workspace clear")) return rc;
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return SLIMK_OK;
}

}  // namespace

extern "C" {

int slimk_w2a8_gemm(const int8_t* q, int ldq, const float* s_a, const int32_t* rowsum, int ldr,
                    const uint32_t* w_r, const uint16_t* s_r, const uint8_t* zp_r, int zp_const,
                    int M, int N, int K, int group_size,
                    void* out, int ldo, int out_dtype,
                    int32_t* acc_dump, int dump_mode,
                    void* workspace, size_t workspace_bytes,
                    int kernel, int split_k, void* stream) {
    return gemm_impl(q, ldq, s_a, rowsum, ldr, w_r, s_r, zp_r, zp_const, M, N, K, group_size, out, ldo, out_dtype,
                     acc_dump, dump_mode, workspace, workspace_bytes, kernel, split_k, stream, false);
}

size_t slimk_w2a8_static_workspace_bytes(void) { return kStaticWorkspaceBytes; }

int slimk_w2a8_gemm_static(const int8_t* q, int ldq, const float* s_a, const int32_t* rowsum, int ldr,
                           const uint32_t* w_r, const uint16_t* s_r, const uint8_t* zp_r, int zp_const,
                           int M, int N, int K, int group_size,
                           void* out, int ldo, int out_dtype,
                           int kernel, int split_k, void* stream) {
    // every argument is validated before anything touches the GPU; the library-owned array is looked up (and, on a
    // device's first split-K call, its counters cleared) only when the launch splits K
    return gemm_impl(q, ldq, s_a, rowsum, ldr, w_r, s_r, zp_r, zp_const, M, N, K, group_size, out, ldo, out_dtype,
                     nullptr, SLIMK_DUMP_NONE, nullptr, kStaticWorkspaceBytes, kernel, split_k, stream, true);
}

int slimk_w2a8_gemm_fused(const void* x, int ldx, int x_dtype,
                          const uint32_t* w_r, const uint16_t* s_r, const uint8_t* zp_r, int zp_const,
                          int M, int N, int K, int group_size,
                          void* out, int ldo, int out_dtype,
                          void* workspace, size_t workspace_bytes, int split_k, void* stream) {
    if (!x || !w_r || !s_r || !out) return fail(SLIMK_ERR_NULL_POINTER, "gemm_fused: NULL buffer");
    if (M <= 0 || N <= 0) return fail(SLIMK_ERR_BAD_SHAPE, "M=%d, N=%d must be positive", M, N);
    if (int rc = check_kg(K, group_size)) return rc;
    if (x_dtype != SLIMK_F16 && x_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "x_dtype=%d", x_dtype);
    if (out_dtype != SLIMK_F16 && out_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "out_dtype=%d", out_dtype);
    if (zp_const < 0 || zp_const > 3) return fail(SLIMK_ERR_BAD_SHAPE, "zp_const=%d must be 0..3", zp_const);
    if (ldx < K || ldo < N) return fail(SLIMK_ERR_BAD_SHAPE, "ldx=%d / ldo=%d too small for K=%d / N=%d", ldx, ldo, K, N);
    if (M > w2a8::kRowsMax) return fail(SLIMK_ERR_UNSUPPORTED, "gemm_fused handles M <= %d (M=%d)", w2a8::kRowsMax, M);
    if (int rc = check_extent(M, N, K, K)) return rc;
    if (!aligned16(x) || ldx % 8 != 0 || !aligned16(w_r) || !aligned16(s_r) || (zp_r && !aligned16(zp_r)) ||
        (reinterpret_cast<uintptr_t>(out) & 1u))
        return fail(SLIMK_ERR_MISALIGNED, "gemm_fused: x, w_r, s_r, zp_r must be 16-byte aligned; ldx %% 8 == 0; out 2-byte aligned");
    const int G = K / group_size;
    const bool in_workgroup = fused_in_workgroup(M, K);
    if (split_k <= 0) split_k = in_workgroup ? auto_split(M, N, K, group_size, SLIMK_KERNEL_SKINNY) : skinny_plain_split(N, K, group_size);
    if (split_k > G) return fail(SLIMK_ERR_BAD_SHAPE, "split_k=%d exceeds the number of groups %d", split_k, G);
    const int gps = groups_per_split(G, group_size, split_k);
    split_k = (G + gps - 1) / gps;

    w2a8::GemmParams p{};
    p.x = reinterpret_cast<const uint16_t*>(x); p.ldx = ldx; p.x_bf16 = x_dtype == SLIMK_BF16 ? 1 : 0;
    p.w_r = w_r; p.s_r = s_r; p.zp_r = zp_r; p.out = out; p.ldo = ldo;
    p.M = M; p.N = N; p.K = K; p.G = G; p.steps = K / w2a8::kStepK; p.strips = strips_of(N);
    p.zp_const = zp_const; p.split = split_k; p.groups_per_split = gps;
    if (!in_workgroup) {
        // The rows are quantised by the grid's first workgroups into the workspace: counter block, the int8 rows, their
        // scales and group sums, then the split-K partial tiles.
        const size_t need = slimk_w2a8_gemm_fused_workspace_bytes(M, N, K, group_size, split_k);
        if (!workspace) return fail(SLIMK_ERR_WORKSPACE, "gemm_fused with M=%d, K=%d needs a workspace of %zu bytes", M, K, need);
        if (workspace_bytes < need)
            return fail(SLIMK_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes, need);
        if (!aligned16(workspace)) return fail(SLIMK_ERR_MISALIGNED, "workspace must be 16-byte aligned");
        const int counters = p.strips * ((M + 15) / 16);
        if (split_k > 1 && counters > kMaxCounters)
            return fail(SLIMK_ERR_UNSUPPORTED, "split_k over %d output tiles (at most %d arrival counters)", counters, kMaxCounters);
        char* base = reinterpret_cast<char*>(workspace);
        char* rows = base + kCounterBlockBytes;
        p.ws_counter = reinterpret_cast<unsigned*>(base);
        p.q = reinterpret_cast<const int8_t*>(rows); p.ldq = K;
        p.s_a = reinterpret_cast<const float*>(rows + fused_rows_q_bytes(K));
        p.rowsum = reinterpret_cast<const int32_t*>(rows + fused_rows_q_bytes(K) + 256); p.ldr = w2a8::kRowsMax;
        p.ws_partial = reinterpret_cast<float*>(rows + fused_rows_area_bytes(K, G));
        return hip_result(w2a8::launch_skinny_rows(p, group_size / w2a8::kStepK, skinny_waves(M, N, K, split_k), zp_r != nullptr,
                                                   out_dtype == SLIMK_BF16, g_rows_spin_limit.load(), (hipStream_t)stream),
                          "row-quantising skinny gemm");
    }
    if (split_k > 1) {
        const size_t need = slimk_w2a8_gemm_workspace_bytes(M, N, K, group_size, SLIMK_KERNEL_SKINNY, split_k);
        if (!workspace) return fail(SLIMK_ERR_WORKSPACE, "split_k=%d needs a workspace of %zu bytes", split_k, need);
        if (workspace_bytes < need)
            return fail(SLIMK_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes, need);
        if (!aligned16(workspace)) return fail(SLIMK_ERR_MISALIGNED, "workspace must be 16-byte aligned");
        p.ws_counter = reinterpret_cast<unsigned*>(workspace);
        if (p.strips > kMaxCounters)
            return fail(SLIMK_ERR_UNSUPPORTED, "split_k over %d output tiles (at most %d arrival counters)", p.strips, kMaxCounters);
        p.ws_partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kCounterBlockBytes);
    }
    return hip_result(w2a8::launch_skinny_fused(p, group_size / w2a8::kStepK, skinny_waves(M, N, K, split_k), zp_r != nullptr,
                                                out_dtype == SLIMK_BF16, (hipStream_t)stream),
                      "fused skinny gemm");
}

size_t slimk_w2a8_gemm_fused_workspace_bytes(int M, int N, int K, int group_size, int split_k) {
    if (M <= 0 || M > w2a8::kRowsMax || N <= 0 || !shape_ok(K, group_size)) return 0;
    if (fused_in_workgroup(M, K)) return slimk_w2a8_gemm_workspace_bytes(M, N, K, group_size, SLIMK_KERNEL_SKINNY, split_k);
    const int G = K / group_size;
    if (split_k <= 0) split_k = skinny_plain_split(N, K, group_size);
    const int gps = groups_per_split(G, group_size, split_k);
    split_k = (G + gps - 1) / gps;
    size_t bytes = kCounterBlockBytes + fused_rows_area_bytes(K, G);
    if (split_k > 1) bytes += (size_t)split_k * strips_of(N) * ((M + 15) / 16) * 16 * w2a8::kStripN * sizeof(float);
    return bytes;
}

int slimk_w2a8_set_fused_spin_limit(int polls) {
    if (polls < 0) polls = 0;
    return g_rows_spin_limit.exchange(polls);
}

}  // extern "C"

namespace {

int gemm_grouped_impl(const slimk_w2a8_problem* problems, int count, int group_size, int out_dtype,
                      int32_t* const* acc_dumps, int dump_mode, void* stream) {
    if (!problems) return fail(SLIMK_ERR_NULL_POINTER, "gemm_grouped: problems is NULL");
    if (dump_mode != SLIMK_DUMP_NONE) {
        if (dump_mode != SLIMK_DUMP_GROUPS && dump_mode != SLIMK_DUMP_SUM) return fail(SLIMK_ERR_BAD_ENUM, "dump_mode=%d", dump_mode);
        if (!acc_dumps) return fail(SLIMK_ERR_NULL_POINTER, "gemm_grouped: dump_mode set but acc_dumps is NULL");
        for (int i = 0; i < count && i < SLIMK_W2A8_MAX_GROUP; ++i)
            if (!acc_dumps[i]) return fail(SLIMK_ERR_NULL_POINTER, "gemm_grouped: acc_dumps[%d] is NULL", i);
    }
    if (count < 1 || count > SLIMK_W2A8_MAX_GROUP)
        return fail(SLIMK_ERR_BAD_SHAPE, "gemm_grouped: count=%d must be 1..%d", count, SLIMK_W2A8_MAX_GROUP);
    if (out_dtype != SLIMK_F16 && out_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "out_dtype=%d", out_dtype);
    if (group_size != 64 && group_size != 128 && group_size != 256)
        return fail(SLIMK_ERR_BAD_SHAPE, "group_size=%d must be 64, 128 or 256", group_size);
    // longest-running workgroups first, so that they do not start last: longest reductions first and, among
    // equal reductions, most token rows first (more activation traffic and matrix work per weight byte;
    // measured on the Llama-8B decode sweep: 46.5 -> 43.7 us against rising M)
    int order[SLIMK_W2A8_MAX_GROUP];
    for (int i = 0; i < count; ++i) order[i] = i;
    const auto before_in_launch = [&](int a, int b) {
        return problems[a].K != problems[b].K ? problems[a].K > problems[b].K : problems[a].M > problems[b].M;
    };
    for (int i = 1; i < count; ++i)
        for (int j = i; j > 0 && before_in_launch(order[j], order[j - 1]); --j) {
            const int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t;
        }
    static_assert(SLIMK_W2A8_MAX_GROUP == w2a8::kMaxGroup, "group limit");
    w2a8::GroupedParams gp{};
    gp.count = count;
    int zm = -1, wgs = 0;
    long long xcd_load[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    // A workgroup of eight waves covers 8 strips x all of K, 4 strips x 2 halves or 2 strips x 4 quarters
    // (measured on the Llama-8B decode shapes: runs of 32..64 steps per wave stream best).
    const auto kparts_of = [](int steps) { return steps > 192 ? 4 : (steps > 32 ? 2 : 1); };
    // K-parts per problem.  A launch that would not even put one workgroup on every CU is bound by
    // latency, not bandwidth: there the problem whose waves run longest is split further (down to runs
    // of four chunks) until the CUs are covered.
    int kparts[SLIMK_W2A8_MAX_GROUP];
    {
        const auto wgs_of = [&](int i, int parts) {
            const int per_unit = w2a8::kGroupedWavesPerWg / parts;
            return (strips_of(problems[i].N) + per_unit - 1) / per_unit * ((problems[i].M + 15) / 16);
        };
        int total = 0;
        for (int i = 0; i < count; ++i) {
            kparts[i] = problems[i].K >= 64 ? kparts_of(problems[i].K / w2a8::kStepK) : 1;
            total += problems[i].N > 0 && problems[i].M > 0 ? wgs_of(i, kparts[i]) : 0;
        }
        while (total < 256) {
            int pick = -1, run = 0;
            for (int i = 0; i < count; ++i) {
                const int r = (problems[i].K / w2a8::kStepK + 3) / 4 / kparts[i];  // chunks per part
                if (kparts[i] < 8 && r >= 8 && r > run && problems[i].N > 0 && problems[i].M > 0) { pick = i; run = r; }
            }
            if (pick < 0) break;
            total += wgs_of(pick, kparts[pick] * 2) - wgs_of(pick, kparts[pick]);
            kparts[pick] *= 2;
        }
        // 512 workgroups run at once (two per CU); those beyond start as the first ones end, into a
        // chip that is emptying.  The problems that start there (in launch order) get twice the
        // k-parts: a second round of about twice the workgroups, each half as long.
        int before = 0;
        for (int oi = 0; oi < count; ++oi) {
            const int i = order[oi];
            if (problems[i].N <= 0 || problems[i].M <= 0) continue;
            const int r = (problems[i].K / w2a8::kStepK + 3) / 4 / kparts[i];
            if (before >= 512 && kparts[i] < 4 && r >= 8) kparts[i] *= 2;
            before += wgs_of(i, kparts[i]);
        }
    }
    for (int i = 0; i < count; ++i) {
        const slimk_w2a8_problem& pr = problems[order[i]];
        if (!pr.q || !pr.s_a || !pr.rowsum || !pr.w_r || !pr.s_r || !pr.out)
            return fail(SLIMK_ERR_NULL_POINTER, "gemm_grouped: problem %d has a NULL buffer", order[i]);
        if (pr.M <= 0 || pr.N <= 0) return fail(SLIMK_ERR_BAD_SHAPE, "gemm_grouped: problem %d: M=%d, N=%d", order[i], pr.M, pr.N);
        if (pr.M > 32) return fail(SLIMK_ERR_UNSUPPORTED, "gemm_grouped: problem %d has M=%d > 32", order[i], pr.M);
        if (int rc = check_kg(pr.K, group_size)) return rc;
        if (pr.ldq < pr.K || pr.ldo < pr.N || pr.ldr < pr.M)
            return fail(SLIMK_ERR_BAD_SHAPE, "gemm_grouped: problem %d: a leading dimension is too small", order[i]);
        if (pr.zp_const < 0 || pr.zp_const > 3) return fail(SLIMK_ERR_BAD_SHAPE, "gemm_grouped: problem %d: zp_const=%d", order[i], pr.zp_const);
        if (int rc = check_extent(pr.M, pr.N, pr.K, pr.ldq)) return rc;
        if (!aligned16(pr.q) || pr.ldq % 16 != 0 || !aligned16(pr.rowsum) || pr.ldr % 4 != 0 || !aligned16(pr.w_r) ||
            !aligned16(pr.s_r) || (pr.zp_r && !aligned16(pr.zp_r)) || (reinterpret_cast<uintptr_t>(pr.out) & 1u))
            return fail(SLIMK_ERR_MISALIGNED, "gemm_grouped: problem %d breaks an alignment rule of slimk_w2a8_gemm", order[i]);
        const int this_zm = pr.zp_r ? 1 : 0;
        if (zm >= 0 && this_zm != zm)
            return fail(SLIMK_ERR_UNSUPPORTED, "gemm_grouped: problems mix uniform and per-group zero-points");
        zm = this_zm;
        w2a8::GemmParams& g = gp.prob[i];
        g.q = pr.q; g.s_a = pr.s_a; g.rowsum = pr.rowsum; g.w_r = pr.w_r; g.s_r = pr.s_r; g.zp_r = pr.zp_r;
        g.out = pr.out; g.ldq = pr.ldq; g.ldr = pr.ldr; g.ldo = pr.ldo;
        g.M = pr.M; g.N = pr.N; g.K = pr.K; g.G = pr.K / group_size; g.steps = pr.K / w2a8::kStepK;
        g.strips = strips_of(pr.N); g.zp_const = pr.zp_const;
        g.split = 1; g.groups_per_split = groups_per_split(g.G, group_size, 1);
        if (dump_mode != SLIMK_DUMP_NONE) { g.acc_dump = acc_dumps[order[i]]; g.dump_mode = dump_mode; }
        gp.wg_begin[i] = wgs;
        gp.kparts[i] = kparts[order[i]];
        // units (sets of 8, 4 or 2 strips) in whole sets of eight, times the row blocks of 16 tokens
        const int per_unit = w2a8::kGroupedWavesPerWg / gp.kparts[i];
        const int units = (g.strips + per_unit - 1) / per_unit;
        const int mblocks = (pr.M + 15) / 16;
        wgs += (units + 7) / 8 * 8 * mblocks;
        // The workgroup with id % 8 == x runs on XCD x.  The units of the last, partial set go to the
        // XCDs that have the least work so far (work = steps a workgroup streams).
        int by_load[8];
        for (int x = 0; x < 8; ++x) by_load[x] = x;
        for (int a = 1; a < 8; ++a)
            for (int b = a; b > 0 && xcd_load[by_load[b]] < xcd_load[by_load[b - 1]]; --b) {
                const int t = by_load[b]; by_load[b] = by_load[b - 1]; by_load[b - 1] = t;
            }
        uint32_t slots = 0;
        const long long unit_work = (long long)mblocks * (g.steps / gp.kparts[i] + 16);
        for (int slot = 0; slot < 8; ++slot) {
            slots |= (uint32_t)slot << (3 * by_load[slot]);
            if (slot < units % 8) xcd_load[by_load[slot]] += unit_work;
        }
        gp.xcd_slots[i] = slots;
    }
    gp.wg_begin[count] = wgs;
    // A single problem that the one-problem kernel runs unsplit is faster there (measured 5 us
    // against 7.6 us at 4096 x 4096, M = 1: one strip per workgroup puts more waves on the chip).
    if (count == 1 && auto_split(problems[0].M, problems[0].N, problems[0].K, group_size, SLIMK_KERNEL_SKINNY) == 1) {
        const slimk_w2a8_problem& pr = problems[0];
        return slimk_w2a8_gemm(pr.q, pr.ldq, pr.s_a, pr.rowsum, pr.ldr, pr.w_r, pr.s_r, pr.zp_r, pr.zp_const, pr.M, pr.N, pr.K,
                               group_size, pr.out, pr.ldo, out_dtype, dump_mode != SLIMK_DUMP_NONE ? acc_dumps[0] : nullptr, dump_mode,
                               nullptr, 0, SLIMK_KERNEL_SKINNY, 1, stream);
    }
    hipStream_t st = (hipStream_t)stream;
    if (dump_mode == SLIMK_DUMP_SUM)
        for (int i = 0; i < count; ++i)
            if (int rc = hip_result(w2a8::launch_fill_zero(acc_dumps[i], (size_t)problems[i].M * problems[i].N * sizeof(int32_t), st), "dump clear"))
                return rc;
    const int gs = group_size / w2a8::kStepK;
    return hip_result(dump_mode != SLIMK_DUMP_NONE ? w2a8::launch_skinny_grouped_verify(gp, gs, zm == 1, out_dtype == SLIMK_BF16, st)
                                                   : w2a8::launch_skinny_grouped(gp, gs, zm == 1, out_dtype == SLIMK_BF16, st),
                      "grouped skinny gemm");
}

}  // namespace

extern "C" {

int slimk_w2a8_gemm_grouped(const slimk_w2a8_problem* problems, int count, int group_size, int out_dtype,
                            void* stream) {
    return gemm_grouped_impl(problems, count, group_size, out_dtype, nullptr, SLIMK_DUMP_NONE, stream);
}

int slimk_w2a8_gemm_grouped_verify(const slimk_w2a8_problem* problems, int count, int group_size, int out_dtype,
                                   int32_t* const* acc_dumps, int dump_mode, void* stream) {
    if (dump_mode == SLIMK_DUMP_NONE) return fail(SLIMK_ERR_BAD_ENUM, "gemm_grouped_verify: dump_mode must be GROUPS or SUM");
    return gemm_grouped_impl(problems, count, group_size, out_dtype, acc_dumps, dump_mode, stream);
}

int slimk_w4a8_gemm_auto_split_k(int M, int N, int K, int group_size) {
    if (M <= 0 || N <= 0 || !shape_ok(K, group_size) || K % 128 != 0 || group_size > 128) return 0;
    return w2a8::tiled_w4_auto_split(M, strips_of(N), K / w2a8::kStepK);
}

size_t slimk_w4a8_gemm_workspace_bytes(int M, int N, int K, int group_size, int split_k) {
    if (split_k <= 0) split_k = slimk_w4a8_gemm_auto_split_k(M, N, K, group_size);
    if (split_k <= 1 || M <= 0 || N <= 0) return 0;
    const size_t tiles = w2a8::tiled_w4_tiles(M, strips_of(N));
    return kCounterBlockBytes + (size_t)split_k * tiles * 64 * 256 * sizeof(float);
}

int slimk_w4a8_gemm(const int8_t* q, int ldq, const float* s_a, const int32_t* rowsum, int ldr,
                    const uint32_t* w_r, const uint16_t* s_r, const uint8_t* zp_r,
                    int M, int N, int K, int group_size,
                    void* out, int ldo, int out_dtype,
                    void* workspace, size_t workspace_bytes, int split_k, void* stream) {
    if (!q || !s_a || !w_r || !s_r || !out) return fail(SLIMK_ERR_NULL_POINTER, "w4a8_gemm: NULL buffer");
    if (zp_r && !rowsum) return fail(SLIMK_ERR_NULL_POINTER, "w4a8_gemm: per-group zero-points need the row sums");
    if (M <= 0 || N <= 0) return fail(SLIMK_ERR_BAD_SHAPE, "M=%d, N=%d must be positive", M, N);
    if (int rc = check_kg(K, group_size)) return rc;
    if (zp_r && ldr < M) return fail(SLIMK_ERR_BAD_SHAPE, "ldr=%d smaller than M=%d", ldr, M);
    if (zp_r && (!aligned16(zp_r) || !aligned16(rowsum) || ldr % 4 != 0))
        return fail(SLIMK_ERR_MISALIGNED, "w4a8_gemm: zp_r and rowsum must be 16-byte aligned and ldr %% 4 == 0");
    if (K % 128 != 0 || group_size > 128)
        return fail(SLIMK_ERR_UNSUPPORTED, "w4a8_gemm: K=%d must be a multiple of 128 and group_size=%d 64 or 128", K, group_size);
    if (out_dtype != SLIMK_F16 && out_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "out_dtype=%d", out_dtype);
    if (ldq < K || ldo < N) return fail(SLIMK_ERR_BAD_SHAPE, "ldq=%d / ldo=%d too small for K=%d / N=%d", ldq, ldo, K, N);
    if (2LL * K > 0x7fffffff) return fail(SLIMK_ERR_UNSUPPORTED, "K=%d too long", K);
    if (int rc = check_extent(M, N, 2 * K, ldq)) return rc;
    if (!aligned16(q) || ldq % 16 != 0 || !aligned16(w_r) || !aligned16(s_r) || (reinterpret_cast<uintptr_t>(out) & 1u))
        return fail(SLIMK_ERR_MISALIGNED, "w4a8_gemm: q, w_r, s_r must be 16-byte aligned; ldq %% 16 == 0; out 2-byte aligned");
    const int stages = K / (2 * w2a8::kStepK);
    if (split_k <= 0) split_k = w2a8::tiled_w4_auto_split(M, strips_of(N), K / w2a8::kStepK);
    if (split_k > stages) return fail(SLIMK_ERR_BAD_SHAPE, "split_k=%d exceeds the %d stages of 128 reduction elements", split_k, stages);
    const size_t tiles = w2a8::tiled_w4_tiles(M, strips_of(N));
    if (split_k > 1 && (size_t)split_k * tiles * 64 * 256 * 4 >= 0x7fffffffu)
        return fail(SLIMK_ERR_UNSUPPORTED, "w4a8_gemm: split_k=%d over %zu tiles needs more than 2 GiB of partial sums", split_k, tiles);
    const int sps = split_k > 1 ? (stages + split_k - 1) / split_k : stages;
    if (split_k > 1) split_k = (stages + sps - 1) / sps;   // effective split: whole stages per split

    w2a8::GemmParams p{};
    p.q = q; p.s_a = s_a; p.w_r = w_r; p.s_r = s_r; p.out = out; p.ldq = ldq; p.ldo = ldo;
    p.zp_r = zp_r; p.rowsum = zp_r ? rowsum : nullptr; p.ldr = ldr;
    p.M = M; p.N = N; p.K = K; p.G = K / group_size; p.steps = K / w2a8::kStepK; p.strips = strips_of(N);
    p.zp_const = 2; p.split = split_k; p.groups_per_split = split_k > 1 ? sps * (128 / group_size) : p.G;
    if (split_k > 1) {
        const size_t need = kCounterBlockBytes + (size_t)split_k * tiles * 64 * 256 * sizeof(float);
        if (!workspace) return fail(SLIMK_ERR_WORKSPACE, "split_k=%d needs a workspace of %zu bytes", split_k, need);
        if (workspace_bytes < need)
            return fail(SLIMK_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes, need);
        if (!aligned16(workspace)) return fail(SLIMK_ERR_MISALIGNED, "workspace must be 16-byte aligned");
        p.ws_counter = reinterpret_cast<unsigned*>(workspace);
        p.ws_partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kCounterBlockBytes);
    }
    return hip_result(w2a8::launch_tiled_w4(p, group_size / w2a8::kStepK, out_dtype == SLIMK_BF16, (hipStream_t)stream), "w4a8_gemm");
}

int slimk_w2a16_gemm_auto_split_k(int M, int N, int K, int group_size) {
    if (M <= 0 || N <= 0 || !shape_ok(K, group_size) || K % 128 != 0) return 0;
    return w2a8::w2a16_auto_split(M, strips_of(N), K / w2a8::kStepK, group_size / w2a8::kStepK);
}

size_t slimk_w2a16_gemm_workspace_bytes(int M, int N, int K, int group_size, int split_k) {
    if (split_k <= 0) split_k = slimk_w2a16_gemm_auto_split_k(M, N, K, group_size);
    if (split_k <= 1 || M <= 0 || N <= 0) return 0;
    return (size_t)split_k * (size_t)M * (size_t)N * sizeof(float);
}

int slimk_w2a16_gemm(const void* x, int ldx, int x_dtype,
                     const uint32_t* w_r, const uint16_t* s_r, const uint8_t* zp_r, int zp_const,
                     int M, int N, int K, int group_size,
                     void* out, int ldo, int out_dtype,
                     void* workspace, size_t workspace_bytes, int split_k, void* stream) {
    if (!x || !w_r || !s_r || !out) return fail(SLIMK_ERR_NULL_POINTER, "w2a16_gemm: NULL buffer");
    if (M <= 0 || N <= 0) return fail(SLIMK_ERR_BAD_SHAPE, "M=%d, N=%d must be positive", M, N);
    if (int rc = check_kg(K, group_size)) return rc;
    if (K % 128 != 0) return fail(SLIMK_ERR_UNSUPPORTED, "w2a16_gemm: K=%d must be a multiple of 128", K);
    if (x_dtype != SLIMK_F16 && x_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "x_dtype=%d", x_dtype);
    if (out_dtype != SLIMK_F16 && out_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "out_dtype=%d", out_dtype);
    if (zp_const < 0 || zp_const > 3) return fail(SLIMK_ERR_BAD_SHAPE, "zp_const=%d must be 0..3", zp_const);
    if (ldx < K || ldo < N) return fail(SLIMK_ERR_BAD_SHAPE, "ldx=%d / ldo=%d too small for K=%d / N=%d", ldx, ldo, K, N);
    if (int rc = check_extent(M, N, K, 2 * ldx)) return rc;
    if (!aligned16(x) || ldx % 8 != 0 || !aligned16(w_r) || !aligned16(s_r) || (zp_r && !aligned16(zp_r)) ||
        (reinterpret_cast<uintptr_t>(out) & 1u))
        return fail(SLIMK_ERR_MISALIGNED, "w2a16_gemm: x, w_r, s_r, zp_r must be 16-byte aligned; ldx %% 8 == 0; out 2-byte aligned");
    const int gs = group_size / w2a8::kStepK, steps = K / w2a8::kStepK;
    const int granules = steps / (gs > 2 ? gs : 2);
    if (split_k <= 0) split_k = w2a8::w2a16_auto_split(M, strips_of(N), steps, gs);
    if (split_k > 64 || (split_k > 1 && split_k * 4 > granules))
        return fail(SLIMK_ERR_BAD_SHAPE, "split_k=%d: at most 64 and at most a quarter of the %d K granules", split_k, granules);

    w2a8::W2A16Params p{};
    p.x = reinterpret_cast<const uint16_t*>(x); p.ldx = ldx;
    p.w_r = w_r; p.s_r = s_r; p.zp_r = zp_r; p.out = out; p.ldo = ldo;
    p.M = M; p.N = N; p.K = K; p.G = K / group_size; p.steps = steps; p.strips = strips_of(N);
    p.zp_const = zp_const; p.split = split_k; p.x_bf16 = x_dtype == SLIMK_BF16;
    if (split_k > 1) {
        const size_t need = (size_t)split_k * (size_t)M * (size_t)N * sizeof(float);
        if (!workspace) return fail(SLIMK_ERR_WORKSPACE, "split_k=%d needs a workspace of %zu bytes", split_k, need);
        if (workspace_bytes < need)
            return fail(SLIMK_ERR_WORKSPACE, "workspace of %zu bytes is smaller than the %zu needed", workspace_bytes, need);
        if (!aligned16(workspace)) return fail(SLIMK_ERR_MISALIGNED, "workspace must be 16-byte aligned");
        p.ws = reinterpret_cast<float*>(workspace);
    }
    return hip_result(w2a8::launch_w2a16(p, gs, out_dtype == SLIMK_BF16, (hipStream_t)stream), "w2a16_gemm");
}

int slimk_w2a16_gemm_grouped(const slimk_w2a16_problem* problems, int count, int group_size, int x_dtype, int out_dtype,
                             void* stream) {
    if (!problems) return fail(SLIMK_ERR_NULL_POINTER, "w2a16_gemm_grouped: problems is NULL");
    if (count < 1 || count > SLIMK_W2A8_MAX_GROUP)
        return fail(SLIMK_ERR_BAD_SHAPE, "w2a16_gemm_grouped: count=%d must be 1..%d", count, SLIMK_W2A8_MAX_GROUP);
    if (x_dtype != SLIMK_F16 && x_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "x_dtype=%d", x_dtype);
    if (out_dtype != SLIMK_F16 && out_dtype != SLIMK_BF16) return fail(SLIMK_ERR_BAD_ENUM, "out_dtype=%d", out_dtype);
    if (group_size != 64 && group_size != 128 && group_size != 256)
        return fail(SLIMK_ERR_BAD_SHAPE, "group_size=%d must be 64, 128 or 256", group_size);
    // longest reductions first, so that the workgroups that run longest do not start last
    int order[SLIMK_W2A8_MAX_GROUP];
    for (int i = 0; i < count; ++i) order[i] = i;
    for (int i = 1; i < count; ++i)
        for (int j = i; j > 0 && problems[order[j]].K > problems[order[j - 1]].K; --j) {
            const int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t;
        }
    w2a8::W2A16Group gp{};
    gp.count = count;
    // Sixteen waves per workgroup when a reduction of the launch is long enough to occupy them (128 steps and more),
    // eight otherwise; a problem's strips take as many K-parts as leave a part eight steps (four chunks, one trip of
    // the kernel's main loop), the rest of the workgroup's waves go to neighbouring strips.
    int max_steps = 0;
    for (int i = 0; i < count; ++i) max_steps = std::max(max_steps, problems[i].K / w2a8::kStepK);
    gp.waves = max_steps >= 128 ? 16 : 8;
    int zm = -1;
    long long wgs = 0;
    for (int i = 0; i < count; ++i) {
        const slimk_w2a16_problem& pr = problems[order[i]];
        if (!pr.x || !pr.w_r || !pr.s_r || !pr.out)
            return fail(SLIMK_ERR_NULL_POINTER, "w2a16_gemm_grouped: problem %d has a NULL buffer", order[i]);
        if (pr.M <= 0 || pr.N <= 0) return fail(SLIMK_ERR_BAD_SHAPE, "w2a16_gemm_grouped: problem %d: M=%d, N=%d", order[i], pr.M, pr.N);
        if (int rc = check_kg(pr.K, group_size)) return rc;
        if (pr.K % 128 != 0) return fail(SLIMK_ERR_UNSUPPORTED, "w2a16_gemm_grouped: problem %d: K=%d must be a multiple of 128", order[i], pr.K);
        if (pr.zp_const < 0 || pr.zp_const > 3) return fail(SLIMK_ERR_BAD_SHAPE, "w2a16_gemm_grouped: problem %d: zp_const=%d", order[i], pr.zp_const);
        if (pr.ldx < pr.K || pr.ldo < pr.N)
            return fail(SLIMK_ERR_BAD_SHAPE, "w2a16_gemm_grouped: problem %d: a leading dimension is too small", order[i]);
        if (int rc = check_extent(pr.M, pr.N, pr.K, 2 * pr.ldx)) return rc;
        if (!aligned16(pr.x) || pr.ldx % 8 != 0 || !aligned16(pr.w_r) || !aligned16(pr.s_r) || (pr.zp_r && !aligned16(pr.zp_r)) ||
            (reinterpret_cast<uintptr_t>(pr.out) & 1u))
            return fail(SLIMK_ERR_MISALIGNED, "w2a16_gemm_grouped: problem %d breaks an alignment rule of slimk_w2a16_gemm", order[i]);
        const int this_zm = pr.zp_r ? 1 : 0;
        if (zm >= 0 && this_zm != zm)
            return fail(SLIMK_ERR_UNSUPPORTED, "w2a16_gemm_grouped: problems mix uniform and per-group zero-points");
        zm = this_zm;
        w2a8::W2A16Params& g = gp.prob[i];
        g.x = reinterpret_cast<const uint16_t*>(pr.x); g.ldx = pr.ldx;
        g.w_r = pr.w_r; g.s_r = pr.s_r; g.zp_r = pr.zp_r; g.out = pr.out; g.ldo = pr.ldo;
        g.M = pr.M; g.N = pr.N; g.K = pr.K; g.G = pr.K / group_size; g.steps = pr.K / w2a8::kStepK; g.strips = strips_of(pr.N);
        g.zp_const = pr.zp_const; g.split = 1; g.x_bf16 = x_dtype == SLIMK_BF16;
        int lp = 0;
        while ((2 << lp) <= gp.waves && g.steps / (2 << lp) >= 8) ++lp;
        gp.log_parts[i] = lp;
        const int per = gp.waves >> lp;
        gp.wg_begin[i] = (int)wgs;
        wgs += (long long)((g.strips + per - 1) / per) * ((pr.M + 15) / 16);
        if (wgs > (1 << 24)) return fail(SLIMK_ERR_UNSUPPORTED, "w2a16_gemm_grouped: more than 2^24 workgroups");
    }
    gp.wg_begin[count] = (int)wgs;
    return hip_result(w2a8::launch_w2a16_grouped(gp, group_size / w2a8::kStepK, zm == 1, out_dtype == SLIMK_BF16,
                                                 x_dtype == SLIMK_BF16, (hipStream_t)stream), "w2a16 grouped gemm");
}

int slimk_w2a8_read_probe(const void* src, size_t bytes, uint32_t* sink, void* stream) {
    if (!src || !sink) return fail(SLIMK_ERR_NULL_POINTER, "read_probe: NULL buffer");
    if (bytes == 0 || bytes % 16 != 0 || !aligned16(src))
        return fail(SLIMK_ERR_MISALIGNED, "read_probe: bytes must be a positive multiple of 16 and src 16-byte aligned");
    return hip_result(w2a8::launch_read_probe(src, bytes, sink, (hipStream_t)stream), "read_probe");
}

}  // extern "C"
