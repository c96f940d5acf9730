/*
 * slimk_w2a8.h — C ABI of the MI355X (gfx950) W2A8 GEMM path.
 *
 * W2A8 = 2-bit weight codes, four per byte in the upstream matrix_packer.py
 * layout, multiplied by per-token int8 activations on v_mfma_i32_16x16x64_i8,
 * accumulated in int32 per scale group, and dequantised in a fused epilogue:
 *
 *   acc[m,n,g] = sum_{k in group g} q[m,k] * (code[n,k] - zp[g,n])          (int32)
 *   out[m,n]   = cast( s_a[m] * sum_g float(acc[m,n,g]) * float(scale[g,n]) )
 *
 * Upstream interface this replaces: the host launcher
 *   gemm_tn(m, n, a_k, b_k, alpha, A, ldA, B, ldB, beta, C, ldC, stream)
 *   slimkernels/cute/gemm/wgmma_sm90_W2A8.cu:428-437
 * (raw device pointers, explicit leading dimensions, caller-owned buffers, a
 * stream argument) and the notebook entry wint2_gemm(activation, weight, scale)
 * (triton.ipynb cell 1).  Upstream names the 2-bit operand "A" with m = output
 * channels; here M = tokens, N = output channels, K = reduction length.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer unless said otherwise.  The caller owns
 *    all buffers; nothing here allocates or frees device memory.
 *  - Every call only enqueues work on `stream` (a hipStream_t passed as void*;
 *    NULL = the default stream) and returns; nothing synchronises.
 *  - Return value: SLIMK_OK or a SLIMK_ERR_* code.  Arguments are validated on
 *    the host before anything is launched, so a bad call never reaches the GPU.
 *    slimk_w2a8_last_error() returns a thread-local description of the most
 *    recent failure on the calling thread.  Nothing throws or aborts.
 *  - Re-entrant: concurrent calls from several host threads on different streams
 *    are fine as long as they do not share a split-K workspace.  The only state
 *    the library keeps is the device array behind slimk_w2a8_gemm_static (one per
 *    GPU, shared by the calls of that entry point) and the poll limit set by the
 *    test hook slimk_w2a8_set_fused_spin_limit.
 *
 * Shape limits: K % 64 == 0, group_size in {64, 128, 256}, K % group_size == 0.
 * M, N >= 1 are otherwise arbitrary (ragged tiles are handled inside).
 *
 * 4-bit weights (upstream: the notebook kernel w4matmul_splitk,
 * slimkernels/triton/gemm_splitk.ipynb cell 0) need no entry point of their own:
 * a code c = 4 * hi + lo is two 2-bit digits, and a W4 GEMM over K with G groups
 * is these calls over K' = 2K with 2G groups -- columns 0..K-1 the hi digits with
 * scales 4 * s and zero-points zp >> 2, columns K..2K-1 the lo digits with scales
 * s and zero-points zp & 3 -- against q and its row sums laid down twice
 * (slimk_w2a8_act_quant_rep writes them so; slimk_w2a8_quantize_weight4 quantises
 * a weight straight into the two planes).
 *
 * The weight-only form (fp16 activations as they are, upstream's notebook kernel
 * w2matmul) is slimk_w2a16_gemm at the end of this file; it takes the same
 * repacked weights.
 */
#ifndef SLIMK_W2A8_H
#define SLIMK_W2A8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SLIMK_W2A8_VERSION 100 /* major*10000 + minor*100 + patch */

enum slimk_status {
    SLIMK_OK = 0,
    SLIMK_ERR_NULL_POINTER = 1,
    SLIMK_ERR_BAD_SHAPE = 2,      /* non-positive size, K/group divisibility, leading dim too small */
    SLIMK_ERR_MISALIGNED = 3,     /* a pointer or leading dimension breaks a 16-byte rule */
    SLIMK_ERR_BAD_ENUM = 4,       /* dtype / kernel / dump selector out of range */
    SLIMK_ERR_WORKSPACE = 5,      /* split-K requested but workspace missing or too small */
    SLIMK_ERR_HIP = 6,            /* a HIP runtime call failed (see last_error) */
    SLIMK_ERR_UNSUPPORTED = 7     /* valid but not implemented combination */
};

enum slimk_dtype { SLIMK_F16 = 0, SLIMK_BF16 = 1 };

/* which GEMM kernel slimk_w2a8_gemm runs */
enum slimk_kernel {
    SLIMK_KERNEL_AUTO = 0,   /* skinny for M <= 32; for 33..256 rows whichever of the two skinny forms, the tiled kernel
                                and SLIMK_KERNEL_MID is predicted the fastest (slimk_w2a8_gemm_auto_route tells which);
                                tiled beyond */
    SLIMK_KERNEL_SKINNY = 1, /* weight-streaming split-K kernel, M <= 256 (16 rows per pass over the weights) */
    SLIMK_KERNEL_TILED = 2,  /* LDS-pipelined MFMA tile kernel, any M */
    SLIMK_KERNEL_MID = 3     /* workgroups of four 64-channel strips x up to 96 token rows (more rows: two or three row
                                parts), activations shared through LDS, weights streamed once per row part straight to
                                registers, K split across workgroups: M <= 256, groups of up to 256; split workspace
                                sized as for SLIMK_KERNEL_SKINNY.  SLIMK_KERNEL_AUTO takes it where it is predicted the
                                fastest of the four forms: row counts that leave 64-row tiles partly empty (33..48,
                                65..96, 129..160) on large matrices (3..30 % faster than the tiled kernel there) */
};

/* what the optional int32 verification buffer receives */
enum slimk_dump {
    SLIMK_DUMP_NONE = 0,
    SLIMK_DUMP_GROUPS = 1, /* acc_dump[M][N][G]: every per-group accumulator */
    SLIMK_DUMP_SUM = 2     /* acc_dump[M][N]:    sum over groups of the accumulators */
};

/* ---- queries (host only, never touch the GPU) ------------------------------------------- */

/* Library version (SLIMK_W2A8_VERSION) and the one ISA the code objects were built for. */
int slimk_w2a8_version(void);
const char* slimk_w2a8_arch(void);
/* Thread-local text of the last error on this thread ("" if none). */
const char* slimk_w2a8_last_error(void);

/* Byte sizes of the gfx950-private buffers slimk_w2a8_repack fills.  0 on a bad shape. */
size_t slimk_w2a8_repacked_weight_bytes(int N, int K);
size_t slimk_w2a8_repacked_scale_bytes(int N, int K, int group_size);
size_t slimk_w2a8_repacked_zp_bytes(int N, int K, int group_size);

/* Split-K factor slimk_w2a8_gemm would choose for this problem (1 = no workspace needed),
 * and the workspace bytes a given split needs (0 when split_k <= 1).  Both kernels can split K:
 * the skinny one when few strips leave CUs idle (and for 17..32 token rows on matrices of 24 MiB
 * or more, where workgroups of four strips share the activations), the tiled one when its 64-row tiles
 * alone would leave CUs idle or unevenly loaded (up to eight splits of at least 1024 elements of K each).
 * Split results are deterministic (partials are added in split order)
 * but their fp32 summation order differs from the unsplit one.
 * No upstream counterpart: upstream has no split-K launcher (the idea appears only in
 * slimkernels/triton/gemm_splitk.ipynb cell 0). */
int slimk_w2a8_gemm_auto_split_k(int M, int N, int K, int group_size, int kernel);
size_t slimk_w2a8_gemm_workspace_bytes(int M, int N, int K, int group_size, int kernel, int split_k);

/* Which kernel form SLIMK_KERNEL_AUTO takes for this problem: 1 = skinny, one 64-channel strip per workgroup;
 * 2 = tiled; 3 = skinny, workgroups of several strips that share the activations (12..16 token rows on 384 strips
 * and more, 17..32 rows on matrices of 24 MiB or more, and the problems of 33..256 rows for which it is predicted
 * the fastest of the four); 4 = SLIMK_KERNEL_MID (the problems of 33..256 rows for which it is predicted the fastest:
 * row counts that leave 64-row tiles partly empty, on large matrices).  For 33..256 rows the prediction is a cost
 * formula per form, fitted to timings of all four on 32 matrices; it picks within 0.5 % of the best form on average.
 * 0 for a shape the library does not take.  A query for tests and tuning; no upstream counterpart (upstream's
 * launcher has one kernel with one fixed tiling, slimkernels/cute/gemm/wgmma_sm90_W2A8.cu:448-450). */
int slimk_w2a8_gemm_auto_route(int M, int N, int K, int group_size);

/* ---- device work ------------------------------------------------------------------------ */

/* Zero a split-K workspace once after allocating it (a fill kernel, safe under graph capture).
 * A workspace is a block of arrival counters of fixed size (64 KiB, whatever the problem) followed by the fp32
 * partial tiles.  Every GEMM leaves the counters it used at zero again when it finishes, and the counter block
 * never moves, so one initialisation serves any number of later calls of any shapes and kernels (2-bit, 4-bit
 * one-pass, fused) that use the workspace one at a time; calls that overlap in time (different streams) need
 * a workspace each.  Only the counter block has to start at zero (the partial tiles are written before they are
 * read): passing min(workspace_bytes, SLIMK_W2A8_COUNTER_BLOCK_BYTES) here is enough and spares the fill of a
 * large workspace. */
#define SLIMK_W2A8_COUNTER_BLOCK_BYTES (64u << 10)
int slimk_w2a8_workspace_init(void* workspace, size_t workspace_bytes, void* stream);

/* Re-lay the interchange format into the gfx950 streaming layout.
 *   w_packed [N][ldw] uint8 : matrix_packer.py:33-34 layout, ldw >= K/4 bytes per row
 *   scales   [G][N]   fp16  : quantization.py:53 layout (G = K / group_size)
 *   zp       [G][N]   uint8 : zero-points 0..3, or NULL for a uniform zero-point
 *   w_r / s_r / zp_r        : outputs, sizes from the slimk_w2a8_repacked_*_bytes queries;
 *                             zp_r may be NULL exactly when zp is NULL
 * Replaces what upstream gets from TMA + the 128-byte shared-memory swizzle
 * (wgmma_sm90_W2A8.cu:455-456,465-466): the bank-conflict-free operand order is
 * baked into the stored weights instead. */
int slimk_w2a8_repack(const uint8_t* w_packed, int ldw, const uint16_t* scales, const uint8_t* zp,
                      int N, int K, int group_size,
                      uint32_t* w_r, uint16_t* s_r, uint8_t* zp_r, void* stream);

/* which level set slimk_w2a8_quantize_weight produces */
enum slimk_quant_mode {
    SLIMK_QUANT_REF = 0,  /* upstream quantize_to_uint2: zero-point 1, scale = absmax / 1.5 (quantization.py:29-46) */
    SLIMK_QUANT_SYM = 1,  /* levels -2..1: zero-point 2, scale = absmax / 2 */
    SLIMK_QUANT_ASYM = 2  /* scale = (max - min) / 3, zero-point = clip(rne(-min / scale), 0, 3) per group */
};

/* Group-wise 2-bit weight quantisation on the GPU: the work of upstream quantize_to_uint2
 * (quantization.py:17-53) followed by pack_matrix (matrix_packer.py:14-34), for a weight in the
 * nn.Linear orientation, with the same numbers as the host-side functions of this package
 * (binary32 arithmetic, IEEE division, round-half-even, the scale rounded to fp16 once).
 *   w      [N][ldw] fp16 or bf16 (w_dtype), groups of group_size consecutive elements along K
 *   packed [N][ldp] uint8 : four codes per byte along K, first code in bits 7:6; ldp >= K/4
 *   scales [G][N]   fp16
 *   zp     [G][N]   uint8 : written when non-NULL (constant 1 / 2 for REF / SYM); required for ASYM
 * The outputs are the inputs of slimk_w2a8_repack.  w 16-byte aligned, ldw % 8 == 0, packed and
 * ldp 2-byte aligned. */
int slimk_w2a8_quantize_weight(const void* w, int ldw, int w_dtype, int N, int K, int group_size, int mode,
                               uint8_t* packed, int ldp, uint16_t* scales, uint8_t* zp, void* stream);

/* Group-wise 4-bit weight quantisation on the GPU, written as the W2 operand over a reduction of 2K that the
 * GEMM entry points take for 4-bit weights (see the top of this file): code = 4 * hi + lo,
 *   planes  [N][ldp] uint8 : hi digits (code >> 2) in bytes 0 .. K/4-1 of a row, lo digits (code & 3) in bytes
 *                            K/4 .. 2K/4-1, four digits per byte along K, first in bits 7:6; ldp >= K/2
 *   scales2 [2G][N] fp16   : rows 0..G-1 = 4 * s, rows G..2G-1 = s
 *   zp2     [2G][N] uint8  : rows 0..G-1 = zp >> 2, rows G..2G-1 = zp & 3
 * mode SLIMK_QUANT_SYM: levels -8..7, s = max(absmax, 1e-9) / 8, zp = 8; SLIMK_QUANT_ASYM: s = max(max - min, 1e-9) / 15,
 * zp = clip(rne(-min / s), 0, 15); binary32 arithmetic, IEEE division, round-half-even, s rounded to fp16 once: the
 * numbers of this package's host functions (slimkernels_amd/w4.py: prepare_w4 + split_planes).  The outputs go to
 * slimk_w2a8_repack with K' = 2K.  Alignment as for slimk_w2a8_quantize_weight.
 * Upstream has no 4-bit quantiser (its W4 kernel runs on random codes, gemm_splitk.ipynb cell 2). */
int slimk_w2a8_quantize_weight4(const void* w, int ldw, int w_dtype, int N, int K, int group_size, int mode,
                                uint8_t* planes, int ldp, uint16_t* scales2, uint8_t* zp2, void* stream);

/* Per-token activation quantisation (no upstream counterpart; upstream feeds FP8,
 * wgmma_sm90_W2A8.cu:533-536).
 *   x [M][ldx] fp16 or bf16 (x_dtype)
 *   q [M][ldq] int8     = clip(rne(x / s_a[m]), -127, 127)
 *   s_a [M]    float32  = max(absmax_k |x[m,k]|, 1e-9) / 127
 *   rowsum [G][ldr] int32 = sum of q over each group (needed by the GEMM to fold
 *                           zero-points); ldr >= M, ldr % 4 == 0.  NULL: the sums are not formed (a quarter
 *                           faster on prefill-sized inputs); slimk_w2a8_gemm takes such an activation where it
 *                           reads no row sums: the tiled kernel with zp_r NULL and zp_const 2
 *                           (slimk_w2a8_gemm_auto_route(M, N, K, group_size) == 2 says when AUTO goes there)
 * ldx, ldq in elements; x, q, rowsum 16-byte aligned; ldx % 8 == 0, ldq % 16 == 0. */
int slimk_w2a8_act_quant(const void* x, int ldx, int x_dtype, int M, int K, int group_size,
                         int8_t* q, int ldq, float* s_a, int32_t* rowsum, int ldr, void* stream);

/* The same with the quantised row and its group sums laid down `copies` (1..4) times: q [M][ldq] holds the row
 * at columns c * K .. c * K + K - 1 for c < copies (ldq >= copies * K), rowsum is [copies * G][ldr] with group g
 * of copy c in row c * G + g.  This is the activation operand of a reduction over copies * K whose weight is
 * several digit planes of one matrix (4-bit weights as two 2-bit planes: copies = 2, see the top of this file).
 * No upstream counterpart. */
int slimk_w2a8_act_quant_rep(const void* x, int ldx, int x_dtype, int M, int K, int group_size, int copies,
                             int8_t* q, int ldq, float* s_a, int32_t* rowsum, int ldr, void* stream);

/* The GEMM.  Counterpart of gemm_tn (wgmma_sm90_W2A8.cu:428-437); alpha/beta, unused
 * upstream (:408), are dropped.
 *   q, ldq, s_a, rowsum, ldr : outputs of slimk_w2a8_act_quant
 *   w_r, s_r, zp_r           : outputs of slimk_w2a8_repack; zp_r NULL -> every zero-point
 *                              equals zp_const (2 for the symmetric levels {-2..1},
 *                              1 for the upstream quantizer)
 *   out [M][ldo]             : fp16 or bf16 (out_dtype), ldo in elements
 *   acc_dump, dump_mode      : optional int32 verification output (see slimk_dump); NULL/0
 *                              in production.  A call with a dump runs the verification instantiation of
 *                              the very kernel body the same call without one runs (same kernel choice,
 *                              tile shape, split and wave count; the accumulators are written out as the
 *                              matrix core left them, before their conversion to fp32), so the production
 *                              instantiations carry no extra code and the two calls' outputs are
 *                              bit-identical.  The fast tiled kernel takes every supported group size and K
 *                              (a group of 256 on 64-row tiles only).
 *   rowsum                   : may be NULL for the tiled kernel with zp_r NULL and zp_const 2 (it is not
 *                              read there)
 *   workspace                : required when the effective split_k > 1
 *                              (slimk_w2a8_gemm_workspace_bytes), else may be NULL
 *   kernel, split_k          : SLIMK_KERNEL_* and the split-K factor; 0 = choose.  split_k is an upper
 *                              bound: a split owns whole 256-element chunks of K, so fewer may be used
 * Repacked weights and activations are addressed with 32-bit offsets: more than 2 GiB of either
 * is SLIMK_ERR_UNSUPPORTED. */
int slimk_w2a8_gemm(const int8_t* q, int ldq, const float* s_a, const int32_t* rowsum, int ldr,
                    const uint32_t* w_r, const uint16_t* s_r, const uint8_t* zp_r, int zp_const,
                    int M, int N, int K, int group_size,
                    void* out, int ldo, int out_dtype,
                    int32_t* acc_dump, int dump_mode,
                    void* workspace, size_t workspace_bytes,
                    int kernel, int split_k, void* stream);

/* slimk_w2a8_gemm for callers that cannot allocate device memory and so cannot supply a split-K workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart upstream (its
 * launcher never splits K).  Same arguments and results as slimk_w2a8_gemm without acc_dump / dump_mode /
 * workspace / workspace_bytes: the arrival counters and partial sums of a split-K launch live in a device array
 * inside the library, SLIMK_W2A8_STATIC_WORKSPACE_BYTES per GPU the library is used on, held until the process
 * ends.  The call allocates and frees nothing, on the device or through any library.
 *  - split_k = 0: the library's choice, lowered until its workspace fits the array (bit-identical with
 *    slimk_w2a8_gemm given the same effective split); an explicit split_k whose workspace
 *    (slimk_w2a8_gemm_workspace_bytes) exceeds the array is refused with SLIMK_ERR_WORKSPACE before any launch.
 *  - Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (different streams,
 *    concurrent graph launches) race on it; calls ordered on one stream, of any shapes, are fine (each leaves
 *    the counters at zero, the partial sums need no clearing).
 *  - Arguments are validated first, as in slimk_w2a8_gemm: a rejected call touches neither the array nor the GPU.
 *    The first call on each GPU that splits K looks the array's address up and clears its counter block with a
 *    small kernel on `stream`; make that call outside stream capture (inside one it is refused with
 *    SLIMK_ERR_UNSUPPORTED rather than recorded into the caller's graph). */
#define SLIMK_W2A8_STATIC_WORKSPACE_BYTES ((16u << 20) + (64u << 10))
size_t slimk_w2a8_static_workspace_bytes(void);
int slimk_w2a8_gemm_static(const int8_t* q, int ldq, const float* s_a, const int32_t* rowsum, int ldr,
                           const uint32_t* w_r, const uint16_t* s_r, const uint8_t* zp_r, int zp_const,
                           int M, int N, int K, int group_size,
                           void* out, int ldo, int out_dtype,
                           int kernel, int split_k, void* stream);

/* The GEMM for up to 32 token rows with the activation quantisation inside: x [M][ldx] fp16 or bf16 (x_dtype)
 * takes the place of q, s_a and rowsum - one launch instead of two on the latency-bound decode path, the numbers of
 * slimk_w2a8_act_quant, the result bit-identical with slimk_w2a8_act_quant followed by slimk_w2a8_gemm (skinny
 * kernel, one strip per workgroup, same split_k).  Two forms, chosen by shape:
 *  - M <= 4 and M * K <= 32768: every workgroup quantises the rows itself into LDS while its first weights are on
 *    the way.  Workspace and split_k as for slimk_w2a8_gemm with SLIMK_KERNEL_SKINNY (none unless K is split).
 *  - otherwise (M <= 32): the first M workgroups of the grid quantise one row each into the workspace and raise a
 *    counter there; every workgroup starts its weight stream and then waits for the rows (a bounded wait: a workgroup
 *    that does not see them arrive in time quantises them itself, so the kernel ends whatever happens).  This form
 *    ALWAYS needs a workspace of slimk_w2a8_gemm_fused_workspace_bytes(...) bytes, zeroed once with
 *    slimk_w2a8_workspace_init (the kernel leaves its counters at zero; calls that share a workspace must not overlap
 *    in time).  A workspace of that size also serves slimk_w2a8_gemm calls of the same shape.
 * M > 32: SLIMK_ERR_UNSUPPORTED.  x 16-byte aligned, ldx % 8 == 0.
 * No upstream counterpart (upstream feeds already quantised FP8, wgmma_sm90_W2A8.cu:533-536; the model-level caller
 * is llama.py:15-19). */
size_t slimk_w2a8_gemm_fused_workspace_bytes(int M, int N, int K, int group_size, int split_k);
int slimk_w2a8_gemm_fused(const void* x, int ldx, int x_dtype,
                          const uint32_t* w_r, const uint16_t* s_r, const uint8_t* zp_r, int zp_const,
                          int M, int N, int K, int group_size,
                          void* out, int ldo, int out_dtype,
                          void* workspace, size_t workspace_bytes, int split_k, void* stream);
/* Test hook, no upstream counterpart: the number of polls (about a microsecond each) the second form above waits for
 * the rows before a workgroup quantises them itself; returns the previous value (default 20000).  0 makes every
 * workgroup take that road, which is how the tests reach it; results do not depend on the value. */
int slimk_w2a8_set_fused_spin_limit(int polls);

/* One problem of a grouped launch: the arguments of slimk_w2a8_gemm that describe data. */
typedef struct slimk_w2a8_problem {
    const int8_t* q;
    const float* s_a;
    const int32_t* rowsum;
    const uint32_t* w_r;
    const uint16_t* s_r;
    const uint8_t* zp_r; /* NULL: uniform zero-point zp_const */
    void* out;
    int ldq, ldr, ldo;
    int M, N, K;
    int zp_const;
} slimk_w2a8_problem;

#define SLIMK_W2A8_MAX_GROUP 24

/* Several independent skinny (M <= 32) GEMMs in ONE kernel launch.  A decode step issues many
 * small GEMMs whose individual run time is a few microseconds of mostly launch and memory
 * latency; run together they fill the chip and stream from HBM at several times the rate
 * (the throughput-oriented kernel: eight-wave workgroups, activations shared through LDS).
 * `problems` is a HOST array of `count` (1..SLIMK_W2A8_MAX_GROUP) entries, copied into the
 * kernel arguments (so the call is graph-capturable and the array may be reused at once).
 * All problems share group_size and out_dtype, and either all carry per-group zero-points
 * (zp_r non-NULL) or none does (each then uses its own zp_const); M, N, K may differ.
 * The order of the entries is the caller's to choose: inside the launch the problems run longest
 * reduction first and, among equal reductions, most token rows first.
 * No split-K, no workspace.  A launch too small to cover the chip splits its longest reductions
 * further inside the workgroups; a lone problem that slimk_w2a8_gemm would run unsplit is handed
 * to that kernel (faster for one problem).
 * No upstream counterpart. */
int slimk_w2a8_gemm_grouped(const slimk_w2a8_problem* problems, int count, int group_size, int out_dtype,
                            void* stream);

/* slimk_w2a8_gemm_grouped with the int32 verification output of slimk_w2a8_gemm: acc_dumps is a HOST array of
 * `count` device pointers, acc_dumps[i] receiving problem i's accumulators ([M][N][G] for SLIMK_DUMP_GROUPS,
 * [M][N] for SLIMK_DUMP_SUM).  Runs the verification instantiation of the grouped kernel (same bodies, same
 * placement of the problems); the outputs are bit-identical with slimk_w2a8_gemm_grouped's.
 * No upstream counterpart (test infrastructure of this library). */
int slimk_w2a8_gemm_grouped_verify(const slimk_w2a8_problem* problems, int count, int group_size, int out_dtype,
                                   int32_t* const* acc_dumps, int dump_mode, void* stream);

/* 4-bit weights in ONE pass over K, for more than 32 token rows: the tiled kernel fetches the hi and the lo digit of
 * every weight and puts them together in front of the matrix core (the int8 operand is 16 * (code - 8)), instead of
 * running the two planes as a reduction over 2K.
 *   q [M][ldq], s_a [M]   : slimk_w2a8_act_quant over K (laid down once)
 *   rowsum [G][ldr]       : its per-group row sums; read only with zp_r
 *   w_r, s_r              : slimk_w2a8_repack of the two planes with K' = 2K (hi digits first) and their scales
 *                           [2G][N] (4 * s, then s), e.g. the outputs of slimk_w2a8_quantize_weight4
 *   zp_r                  : NULL: every zero-point is 8 (the planes' are 2 and 0; mode SYM); else the planes'
 *                           repacked zero-points (rows 0..G-1 zp >> 2, rows G..2G-1 zp & 3): the difference from 8
 *                           enters through the row sums, (8 - zp) * scale * rowsum per group
 *   M, N, K, group_size   : K is the reduction length of the 4-bit matrix (not 2K); K % 128 == 0, group_size 64 or 128
 * int32 sums per group are exact; the result differs from the two-plane route only in fp32 summation order.  Any M works (64-row tiles); up to 32 token rows are better served by slimk_w2a8_gemm over the
 * planes (the few-rows kernels).
 *   workspace, split_k    : as for slimk_w2a8_gemm with the tiled kernel (K split over several workgroups per tile when
 *                           the tiles alone leave CUs idle; 0 = choose): slimk_w4a8_gemm_workspace_bytes(...) bytes,
 *                           zero-initialised once with slimk_w2a8_workspace_init, left zero by every call; may be
 *                           the workspace of the slimk_w2a8_gemm calls on the same stream
 * Replaces upstream's w4matmul_splitk (slimkernels/triton/gemm_splitk.ipynb cell 0: SPLIT_K = 4 with atomic adds; here
 * the partial tiles meet in the workspace and are summed in split order, so results do not depend on timing). */
int slimk_w4a8_gemm_auto_split_k(int M, int N, int K, int group_size);
size_t slimk_w4a8_gemm_workspace_bytes(int M, int N, int K, int group_size, int split_k);
int slimk_w4a8_gemm(const int8_t* q, int ldq, const float* s_a, const int32_t* rowsum, int ldr,
                    const uint32_t* w_r, const uint16_t* s_r, const uint8_t* zp_r,
                    int M, int N, int K, int group_size,
                    void* out, int ldo, int out_dtype,
                    void* workspace, size_t workspace_bytes, int split_k, void* stream);

/* Weight-only form: x [M][ldx] fp16 or bf16 activations are NOT quantised; the 2-bit codes are widened to the
 * activations' type in front of the fp16 resp. bf16 matrix cores and every scale group's fp32 sum is scaled into the
 * fp32 result:
 *   out[m][n] = cast( sum_g scales[g][n] * sum_{k in g} x[m][k] * (code[n][k] - zp[g][n]) ).
 * Same repacked weight operands as slimk_w2a8_gemm (w_r, s_r, zp_r / zp_const).  Built for few token rows
 * (the weight stream bounds the time); any M works, 16 rows at a time, each re-reading the weights.
 * K % 128 == 0; x_dtype SLIMK_F16 or SLIMK_BF16 (bf16: the codes enter the matrix core as 1 + code / 4 and the
 * group's activation sum, a fifth MFMA, takes the offset and the zero-point off in fp32); x 16-byte aligned,
 * ldx % 8 == 0.  split_k: K splits across workgroups, 0 = choose; with more than one the caller supplies
 * slimk_w2a16_gemm_workspace_bytes(...) bytes of workspace (fp32 partial sums, summed in split order by a
 * second kernel: results do not depend on timing).  The workspace needs no initialisation.
 * Replaces the upstream notebook kernel w2matmul(a, b, c) (slimkernels/triton/gemm_splitk.ipynb cell 1:
 * `b = ((b >> 4) & 0b11).to(tl.float16); accumulator = tl.dot(a, b, accumulator)`), which has no scales,
 * no zero-point and reads one field per word. */
int slimk_w2a16_gemm_auto_split_k(int M, int N, int K, int group_size);
size_t slimk_w2a16_gemm_workspace_bytes(int M, int N, int K, int group_size, int split_k);
int slimk_w2a16_gemm(const void* x, int ldx, int x_dtype,
                     const uint32_t* w_r, const uint16_t* s_r, const uint8_t* zp_r, int zp_const,
                     int M, int N, int K, int group_size,
                     void* out, int ldo, int out_dtype,
                     void* workspace, size_t workspace_bytes, int split_k, void* stream);

/* One problem of a grouped weight-only launch: the arguments of slimk_w2a16_gemm that describe data. */
typedef struct slimk_w2a16_problem {
    const void* x;       /* [M][ldx] fp16 or bf16 (the launch's x_dtype) */
    const uint32_t* w_r;
    const uint16_t* s_r;
    const uint8_t* zp_r; /* NULL: uniform zero-point zp_const */
    void* out;
    int ldx, ldo;
    int M, N, K;
    int zp_const;
} slimk_w2a16_problem;

/* Several independent weight-only GEMMs in ONE kernel launch (the linears of a decode step that do not depend on one
 * another): `problems` is a HOST array of `count` (1..SLIMK_W2A8_MAX_GROUP) entries, copied into the kernel arguments
 * (graph-capturable, the array may be reused at once).  All problems share group_size, x_dtype and out_dtype, and
 * either all carry per-group zero-points or none does; M, N, K may differ (K % 128 == 0 each).  No K splits across
 * workgroups and no workspace: a workgroup holds one or several strips of a problem, each in as many K-parts as its
 * reduction length suggests (so the fp32 summation order can differ from a single launch's).
 * Inside the launch the problems run longest reduction first.
 * No upstream counterpart (the notebook kernel w2matmul is one GEMM per launch). */
int slimk_w2a16_gemm_grouped(const slimk_w2a16_problem* problems, int count, int group_size, int x_dtype, int out_dtype,
                             void* stream);

/* Streaming-read calibration kernel: sums `bytes` (multiple of 16) of device memory into
 * sink[0..] so that a profiler can relate its FETCH_SIZE counter to a known byte count and
 * the benchmark can quote the achievable HBM read rate next to the GEMM's. */
int slimk_w2a8_read_probe(const void* src, size_t bytes, uint32_t* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SLIMK_W2A8_H */
