// Weight repack, activation quantisation, fill and read-probe kernels (gfx950).
#include "w2a8_launch.h"

namespace w2a8 {

// ------------------------------------------------------------------ weight repack
// One thread builds one dword of the streaming layout from four bytes of the
// interchange layout (matrix_packer.py:33-34: byte j of row n holds k = 4j..4j+3,
// k = 4j in bits 7:6).  See w2a8_common.h for the target layout.
__global__ __launch_bounds__(256) void repack_codes_kernel(const uint8_t* __restrict__ w_packed, int ldw,
                                                           int N, int strips, int steps, size_t total_dwords,
                                                           uint32_t* __restrict__ w_r) {
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total_dwords) return;
    const int i = (int)(idx & 3);
    const int lane = (int)((idx >> 2) & 63);
    const size_t unit = idx >> 8;                       // units in memory order: run, strip, step of the run
    const size_t rs = unit / kRunSteps;
    const int strip = (int)(rs % (size_t)strips);
    const int step = (int)(rs / (size_t)strips) * kRunSteps + (int)(unit % kRunSteps);
    if (step >= steps) {                                // padding of the last run
        w_r[idx] = 0u;
        return;
    }
    const int col = lane & 15, quad = lane >> 4;
    const int src_byte = step * 16 + quad * 4 + i;  // (step*64 + quad*16 + 4*i) / 4
    uint32_t out = 0;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int n = strip * kStripN + p * 16 + col;
        uint32_t byte = (n < N) ? (uint32_t)w_packed[(size_t)n * ldw + src_byte] : 0u;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            uint32_t code = (byte >> (6 - 2 * b)) & 3u;
            if (p == 3) code ^= 2u;
            out |= code << (8 * b + 2 * p);
        }
    }
    w_r[idx] = out;
}

// scales [G][N] fp16 -> s_r [G][strips][16][4]; zero-points likewise (one byte each).
__global__ __launch_bounds__(256) void repack_scales_kernel(const uint16_t* __restrict__ scales,
                                                            const uint8_t* __restrict__ zp, int N, int strips,
                                                            size_t total, uint16_t* __restrict__ s_r,
                                                            uint8_t* __restrict__ zp_r) {
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int p = (int)(idx & 3);
    const int col = (int)((idx >> 2) & 15);
    const size_t sg = idx >> 6;
    const int strip = (int)(sg % (size_t)strips);
    const int g = (int)(sg / (size_t)strips);
    const int n = strip * kStripN + p * 16 + col;
    s_r[idx] = (n < N) ? scales[(size_t)g * N + n] : (uint16_t)0;
    if (zp_r) zp_r[idx] = (n < N) ? zp[(size_t)g * N + n] : (uint8_t)0;
}

hipError_t launch_repack(const uint8_t* w_packed, int ldw, const uint16_t* scales, const uint8_t* zp,
                         int N, int K, int group_size, uint32_t* w_r, uint16_t* s_r, uint8_t* zp_r,
                         hipStream_t stream) {
    const int steps = K / kStepK;
    const int strips = (N + kStripN - 1) / kStripN;
    const int G = K / group_size;
    const size_t total = weight_bytes(strips, steps) / 4;
    repack_codes_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream>>>(
        w_packed, ldw, N, strips, steps, total, w_r);
    const size_t stotal = (size_t)strips * G * 64;
    repack_scales_kernel<<<dim3((unsigned)((stotal + 255) / 256)), dim3(256), 0, stream>>>(
        scales, zp, N, strips, stotal, s_r, zp ? zp_r : nullptr);
    return hipGetLastError();
}

// ------------------------------------------------------------------ activation quantisation
// One workgroup per token row.  Pass 1: absmax.  Pass 2: q = clip(rne(x / s)), the
// per-group sums of q, all with IEEE binary32 division (this file is compiled
// without fast-math).  Each thread handles 8 consecutive elements (one 16-byte load).
template <bool BF16>
__device__ __forceinline__ void widen8(const uint4& raw, float (&v)[8]) {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (BF16) {
            v[2 * i] = __uint_as_float(w[i] << 16);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        } else {
            v[2 * i] = half_bits_to_float((uint16_t)(w[i] & 0xffffu));
            v[2 * i + 1] = half_bits_to_float((uint16_t)(w[i] >> 16));
        }
    }
}

template <bool BF16>
__device__ __forceinline__ void load8(const uint16_t* p, float (&v)[8]) {
    const uint4 raw = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (BF16) {
            v[2 * i] = __uint_as_float(w[i] << 16);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        } else {
            v[2 * i] = half_bits_to_float((uint16_t)(w[i] & 0xffffu));
            v[2 * i + 1] = half_bits_to_float((uint16_t)(w[i] >> 16));
        }
    }
}

// Row of a workgroup.  rowsum is [group][row]: a row's sums are 4 bytes each, a cache line of 128 bytes holds those
// of 32 consecutive rows.  Workgroup ids go round the eight XCDs, each with an L2 of its own, so with row = id the 32
// writers of a line sit on all eight L2s and the line goes to memory in pieces (a fifth of the kernel's time at
// 4096 x 14336: 8 of 43.6 us).  With blocks of 32 consecutive rows dealt to the XCDs instead, a line is put together
// in one L2.  The grid is rounded up to whole sets of 256 rows; ids whose row is past the end do nothing.
__device__ __forceinline__ int act_quant_row(int id, bool by_xcd) {
    if (!by_xcd) return id;
    const int xcd = id & 7, k = id >> 3;
    return (((k >> 5) << 3) + xcd) * 32 + (k & 31);
}
constexpr int kRowsByXcd = 256;  // from this many rows on
static int act_quant_grid(int M) { return M >= kRowsByXcd ? (M + 255) / 256 * 256 : M; }

template <bool BF16>
__global__ __launch_bounds__(256) void act_quant_kernel(const uint16_t* __restrict__ x, int ldx, int M, int K,
                                                        int group_size, int8_t* __restrict__ q, int ldq,
                                                        float* __restrict__ s_a,
                                                        int32_t* __restrict__ rowsum, int ldr, int copies) {
    __shared__ float red[4];
    const int m = act_quant_row(blockIdx.x, M >= kRowsByXcd);
    if (m >= M) return;  // (uniform: the grid is rounded up to whole sets of rows)
    const int tid = threadIdx.x;
    const uint16_t* xr = x + (size_t)m * ldx;
    const int nvec = K / 8;
    const int iters = (nvec + 255) / 256;

    float amax = 0.0f;
    for (int it = 0; it < iters; ++it) {
        const int v = it * 256 + tid;
        if (v < nvec) {
            float f[8];
            load8<BF16>(xr + (size_t)v * 8, f);
#pragma unroll
            for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(f[i]));
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float s = fmaxf(amax, 1e-9f) / 127.0f;
    if (tid == 0) s_a[m] = s;
    const float inv_s = 1.0f / s;

    const int tpg = group_size / 8;  // threads per scale group: 8, 16 or 32
    int8_t* qr = q + (size_t)m * ldq;
    for (int it = 0; it < iters; ++it) {
        const int v = it * 256 + tid;
        int sum = 0;
        if (v < nvec) {
            float f[8];
            load8<BF16>(xr + (size_t)v * 8, f);
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
            for (int cp = 0; cp < copies; ++cp)   // copies > 1: the row laid down again K further on
                *reinterpret_cast<uint2*>(qr + (size_t)cp * K + (size_t)v * 8) = make_uint2(lo, hi);
        }
        // nvec is a multiple of tpg, so a group's threads are all valid or all idle
        for (int off = 1; off < tpg; off <<= 1) sum += __shfl_xor(sum, off, 64);
        if (rowsum && v < nvec && (v % tpg) == 0)
            for (int cp = 0; cp < copies; ++cp) rowsum[((size_t)cp * (nvec / tpg) + v / tpg) * ldr + m] = sum;
    }
}

// The same with the row read once: a thread keeps its KEEP 16-byte vectors (K <= 2048 * KEEP) in registers
// between the absmax pass and the quantising pass, all of its loads in flight together.  With many rows the
// two-pass kernel moves every row twice (the second time from L2) in phases that the workgroups of a round
// go through together; this one moves it once.  Same arithmetic per element: bit-identical results.
// THREADS: 256 in general (many rows: several workgroups per CU); 512 or 1024 for a few rows, where one row per
// workgroup leaves most of the chip idle and a row's time is what its one CU needs for the arithmetic.  The IEEE
// divisions (a dozen instructions each) were most of that arithmetic: rne_quotient() (w2a8_common.h) avoids nearly
// all of them (32 rows x 28672: 8.2 -> 7.2 us; 4096 x 4096: 17.6 -> 15.2 us).
// SUMS false: no per-group sums of q (rowsum is not touched): what a caller asks for whose GEMM folds no zero-point
// through them (the tiled kernel with the symmetric levels): the sums' adds, shuffles and scattered 4-byte stores are
// a sixth of the kernel's time at 4096 x 14336.
template <bool BF16, int KEEP, int THREADS = 256, bool SUMS = true>
__global__ __launch_bounds__(THREADS) void act_quant_keep_kernel(const uint16_t* __restrict__ x, int ldx, int M, int K,
                                                             int group_size, int8_t* __restrict__ q, int ldq,
                                                             float* __restrict__ s_a,
                                                             int32_t* __restrict__ rowsum, int ldr, int copies) {
    __shared__ float red[THREADS / 64];
    const int m = act_quant_row(blockIdx.x, M >= kRowsByXcd);
    if (m >= M) return;  // (uniform: the grid is rounded up to whole sets of rows)
    const int tid = threadIdx.x;
    const uint16_t* xr = x + (size_t)m * ldx;
    const int nvec = K / 8;
    uint4 raw[KEEP];
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
        const int v = it * THREADS + tid;
        raw[it] = v < nvec ? *reinterpret_cast<const uint4*>(xr + (size_t)v * 8) : make_uint4(0, 0, 0, 0);
    }
    float amax = 0.0f;
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
        float f[8];
        widen8<BF16>(raw[it], f);
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(f[i]));
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = red[0];
#pragma unroll
    for (int w = 1; w < THREADS / 64; ++w) amax = fmaxf(amax, red[w]);
    const float s = fmaxf(amax, 1e-9f) / 127.0f;
    if (tid == 0) s_a[m] = s;
    const float inv_s = 1.0f / s;

    const int tpg = group_size / 8;  // threads per scale group: 8, 16 or 32
    int8_t* qr = q + (size_t)m * ldq;
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
        const int v = it * THREADS + tid;
        int sum = 0;
        if (v < nvec) {
            float f[8];
            widen8<BF16>(raw[it], f);
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float r = rne_quotient(f[i], s, inv_s);  // = rintf(f[i] / s), bit for bit
                r = fminf(fmaxf(r, -127.0f), 127.0f);
                const int qi = (int)r;
                if (SUMS) sum += qi;
                if (i < 4) lo |= (uint32_t)(qi & 0xff) << (8 * i);
                else hi |= (uint32_t)(qi & 0xff) << (8 * (i - 4));
            }
            for (int cp = 0; cp < copies; ++cp)   // copies > 1: the row laid down again K further on
                *reinterpret_cast<uint2*>(qr + (size_t)cp * K + (size_t)v * 8) = make_uint2(lo, hi);
        }
        if constexpr (SUMS) {
            for (int off = 1; off < tpg; off <<= 1) sum += __shfl_xor(sum, off, 64);
            if (v < nvec && (v % tpg) == 0)
                for (int cp = 0; cp < copies; ++cp) rowsum[((size_t)cp * (nvec / tpg) + v / tpg) * ldr + m] = sum;
        }
    }
}

constexpr int kFewRows = 64;  // up to this many rows a long row gets 1024 threads

template <bool BF16, bool SUMS>
static void launch_act_quant_keep(const void* x, int ldx, int M, int K, int group_size, int8_t* q, int ldq, float* s_a,
                                  int32_t* rowsum, int ldr, int copies, hipStream_t stream) {
    const dim3 grid((unsigned)act_quant_grid(M)), block(256);
    if (M <= kFewRows && K > 2048 && K <= 4096) {  // a few rows: 512 threads a row, one vector each
        act_quant_keep_kernel<BF16, 1, 512, SUMS><<<grid, dim3(512), 0, stream>>>((const uint16_t*)x, ldx, M, K, group_size, q, ldq, s_a, rowsum, ldr, copies);
        return;
    }
    if (M <= kFewRows && K > 4096) {  // a few long rows: 1024 threads a row
        const dim3 wide(1024);
        if (K <= 8192)
            act_quant_keep_kernel<BF16, 1, 1024, SUMS><<<grid, wide, 0, stream>>>((const uint16_t*)x, ldx, M, K, group_size, q, ldq, s_a, rowsum, ldr, copies);
        else if (K <= 16384)
            act_quant_keep_kernel<BF16, 2, 1024, SUMS><<<grid, wide, 0, stream>>>((const uint16_t*)x, ldx, M, K, group_size, q, ldq, s_a, rowsum, ldr, copies);
        else
            act_quant_keep_kernel<BF16, 4, 1024, SUMS><<<grid, wide, 0, stream>>>((const uint16_t*)x, ldx, M, K, group_size, q, ldq, s_a, rowsum, ldr, copies);
        return;
    }
    if (K <= 4096)
        act_quant_keep_kernel<BF16, 2, 256, SUMS><<<grid, block, 0, stream>>>((const uint16_t*)x, ldx, M, K, group_size, q, ldq, s_a, rowsum, ldr, copies);
    else if (K <= 8192)
        act_quant_keep_kernel<BF16, 4, 256, SUMS><<<grid, block, 0, stream>>>((const uint16_t*)x, ldx, M, K, group_size, q, ldq, s_a, rowsum, ldr, copies);
    else
        act_quant_keep_kernel<BF16, 8, 256, SUMS><<<grid, block, 0, stream>>>((const uint16_t*)x, ldx, M, K, group_size, q, ldq, s_a, rowsum, ldr, copies);
}

hipError_t launch_act_quant(const void* x, int ldx, bool x_bf16, int M, int K, int group_size,
                            int8_t* q, int ldq, float* s_a, int32_t* rowsum, int ldr, int copies, hipStream_t stream) {
    if (K <= 16384 || (M <= kFewRows && K <= 32768)) {
        if (rowsum) {
            if (x_bf16) launch_act_quant_keep<true, true>(x, ldx, M, K, group_size, q, ldq, s_a, rowsum, ldr, copies, stream);
            else launch_act_quant_keep<false, true>(x, ldx, M, K, group_size, q, ldq, s_a, rowsum, ldr, copies, stream);
        } else {
            if (x_bf16) launch_act_quant_keep<true, false>(x, ldx, M, K, group_size, q, ldq, s_a, rowsum, ldr, copies, stream);
            else launch_act_quant_keep<false, false>(x, ldx, M, K, group_size, q, ldq, s_a, rowsum, ldr, copies, stream);
        }
        return hipGetLastError();
    }
    if (x_bf16)
        act_quant_kernel<true><<<dim3(act_quant_grid(M)), dim3(256), 0, stream>>>((const uint16_t*)x, ldx, M, K, group_size, q,
                                                                 ldq, s_a, rowsum, ldr, copies);
    else
        act_quant_kernel<false><<<dim3(act_quant_grid(M)), dim3(256), 0, stream>>>((const uint16_t*)x, ldx, M, K, group_size, q,
                                                                  ldq, s_a, rowsum, ldr, copies);
    return hipGetLastError();
}

// ------------------------------------------------------------------ weight quantisation
// fp16 / bf16 weights [N][ldw] -> the interchange format: packed 2-bit codes [N][ldp] (four codes per
// byte along K, first code in bits 7:6: matrix_packer.py:33-34 upstream), group scales [G][N] fp16
// and zero-points [G][N] (quantization.py:29-53 upstream for mode 0; the symmetric and asymmetric
// level sets otherwise).  All arithmetic in binary32 with IEEE division and round-half-even, the
// scale rounded to fp16 once for storage after the codes are made with the fp32 one.
// Each thread handles 8 consecutive elements of one row (one 16-byte load); the group_size / 8
// threads of a group sit in one wave and meet through shuffles.
//   mode 0: zero-point 1, scale = absmax / 1.5      (upstream quantizer)
//   mode 1: zero-point 2, scale = absmax / 2        (levels -2..1)
//   mode 2: scale = (max - min) / 3, zero-point = clip(rne(-min / scale), 0, 3) per group
template <bool BF16>
__global__ __launch_bounds__(256) void quantize_weight_kernel(const uint16_t* __restrict__ w, int ldw, int N, int K,
                                                              int group_size, int mode, uint8_t* __restrict__ packed,
                                                              int ldp, uint16_t* __restrict__ scales,
                                                              uint8_t* __restrict__ zp) {
    const int n = blockIdx.x;                      // rows on grid.x: no 65535 limit on N
    const int v = blockIdx.y * 256 + threadIdx.x;  // 8-element vector of the row
    const bool on = v < K / 8;                      // K / 8 is a multiple of a group's threads: whole groups on or off
    float f[8];
    if (on) {
        load8<BF16>(w + (size_t)n * ldw + (size_t)v * 8, f);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = 0.0f;
    }
    float hi = f[0], lo = f[0], amax = fabsf(f[0]);
#pragma unroll
    for (int i = 1; i < 8; ++i) {
        hi = fmaxf(hi, f[i]);
        lo = fminf(lo, f[i]);
        amax = fmaxf(amax, fabsf(f[i]));
    }
    const int tpg = group_size / 8;
    for (int off = 1; off < tpg; off <<= 1) {
        hi = fmaxf(hi, __shfl_xor(hi, off, 64));
        lo = fminf(lo, __shfl_xor(lo, off, 64));
        amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    }
    const float tiny = 1e-9f;
    float s, zero;
    if (mode == 0) {
        s = fmaxf(amax, tiny) / 1.5f;
        zero = 1.0f;
    } else if (mode == 1) {
        s = fmaxf(amax, tiny) / 2.0f;
        zero = 2.0f;
    } else {
        s = fmaxf(hi - lo, tiny) / 3.0f;
        zero = fminf(fmaxf(rintf(-lo / s), 0.0f), 3.0f);
    }
    if (!on) return;
    uint32_t bytes = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float level = fminf(fmaxf(rintf(f[i] / s) + zero, 0.0f), 3.0f);
        const uint32_t code = (uint32_t)(int)level;
        bytes |= code << ((i >> 2) * 8 + 6 - 2 * (i & 3));  // byte i / 4, first code of a byte in bits 7:6
    }
    *reinterpret_cast<uint16_t*>(packed + (size_t)n * ldp + (size_t)v * 2) = (uint16_t)bytes;
    if (v % tpg == 0) {
        const size_t g = (size_t)(v / tpg);
        scales[g * N + n] = __builtin_bit_cast(uint16_t, (_Float16)s);
        if (zp) zp[g * N + n] = (uint8_t)(int)zero;
    }
}

hipError_t launch_quantize_weight(const void* w, int ldw, bool w_bf16, int N, int K, int group_size, int mode,
                                  uint8_t* packed, int ldp, uint16_t* scales, uint8_t* zp, hipStream_t stream) {
    const dim3 grid((unsigned)N, (unsigned)((K / 8 + 255) / 256)), block(256);
    if (w_bf16)
        quantize_weight_kernel<true><<<grid, block, 0, stream>>>((const uint16_t*)w, ldw, N, K, group_size, mode, packed,
                                                                ldp, scales, zp);
    else
        quantize_weight_kernel<false><<<grid, block, 0, stream>>>((const uint16_t*)w, ldw, N, K, group_size, mode, packed,
                                                                 ldp, scales, zp);
    return hipGetLastError();
}

// 4-bit weights as two 2-bit planes over 2K (the operand the W2 kernels take for W4): thread = 8 elements of a
// row as above; codes 0..15 with s = max(absmax, 1e-9) / 8, zero 8 (asym false) or s = max(max - min, 1e-9) / 15,
// zero = clip(rne(-min / s), 0, 15) (asym true).  The hi digits (code >> 2) go to bytes 0 .. K/4-1 of the row
// with scales fp16(4 * fp16(s)) and zero-points zero >> 2 in rows 0 .. G-1; the lo digits (code & 3) to bytes
// K/4 .. 2K/4-1 with scales fp16(s) and zero-points zero & 3 in rows G .. 2G-1.
template <bool BF16>
__global__ __launch_bounds__(256) void quantize_weight4_kernel(const uint16_t* __restrict__ w, int ldw, int N, int K,
                                                               int group_size, int asym, uint8_t* __restrict__ packed,
                                                               int ldp, uint16_t* __restrict__ scales,
                                                               uint8_t* __restrict__ zp) {
    const int n = blockIdx.x;
    const int v = blockIdx.y * 256 + threadIdx.x;
    const bool on = v < K / 8;
    float f[8];
    if (on) {
        load8<BF16>(w + (size_t)n * ldw + (size_t)v * 8, f);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = 0.0f;
    }
    float hi = f[0], lo = f[0], amax = fabsf(f[0]);
#pragma unroll
    for (int i = 1; i < 8; ++i) {
        hi = fmaxf(hi, f[i]);
        lo = fminf(lo, f[i]);
        amax = fmaxf(amax, fabsf(f[i]));
    }
    const int tpg = group_size / 8;
    for (int off = 1; off < tpg; off <<= 1) {
        hi = fmaxf(hi, __shfl_xor(hi, off, 64));
        lo = fminf(lo, __shfl_xor(lo, off, 64));
        amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    }
    const float tiny = 1e-9f;
    float s, zero;
    if (!asym) {
        s = fmaxf(amax, tiny) / 8.0f;
        zero = 8.0f;
    } else {
        s = fmaxf(hi - lo, tiny) / 15.0f;
        zero = fminf(fmaxf(rintf(-lo / s), 0.0f), 15.0f);
    }
    if (!on) return;
    uint32_t hi_bytes = 0, lo_bytes = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float level = fminf(fmaxf(rintf(f[i] / s) + zero, 0.0f), 15.0f);
        const uint32_t code = (uint32_t)(int)level;
        const int at = (i >> 2) * 8 + 6 - 2 * (i & 3);  // byte i / 4, first code of a byte in bits 7:6
        hi_bytes |= (code >> 2) << at;
        lo_bytes |= (code & 3u) << at;
    }
    uint8_t* row = packed + (size_t)n * ldp;
    *reinterpret_cast<uint16_t*>(row + (size_t)v * 2) = (uint16_t)hi_bytes;
    *reinterpret_cast<uint16_t*>(row + (size_t)(K / 4) + (size_t)v * 2) = (uint16_t)lo_bytes;
    if (v % tpg == 0) {
        const size_t g = (size_t)(v / tpg), G = (size_t)(K / group_size);
        const _Float16 s16 = (_Float16)s;
        scales[g * N + n] = __builtin_bit_cast(uint16_t, (_Float16)((float)s16 * 4.0f));
        scales[(G + g) * N + n] = __builtin_bit_cast(uint16_t, s16);
        const uint32_t z = (uint32_t)(int)zero;
        zp[g * N + n] = (uint8_t)(z >> 2);
        zp[(G + g) * N + n] = (uint8_t)(z & 3u);
    }
}

hipError_t launch_quantize_weight4(const void* w, int ldw, bool w_bf16, int N, int K, int group_size, bool asym,
                                   uint8_t* packed, int ldp, uint16_t* scales, uint8_t* zp, hipStream_t stream) {
    const dim3 grid((unsigned)N, (unsigned)((K / 8 + 255) / 256)), block(256);
    if (w_bf16)
        quantize_weight4_kernel<true><<<grid, block, 0, stream>>>((const uint16_t*)w, ldw, N, K, group_size, asym ? 1 : 0,
                                                                 packed, ldp, scales, zp);
    else
        quantize_weight4_kernel<false><<<grid, block, 0, stream>>>((const uint16_t*)w, ldw, N, K, group_size, asym ? 1 : 0,
                                                                  packed, ldp, scales, zp);
    return hipGetLastError();
}

// ------------------------------------------------------------------ fill / probe
__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t* p, size_t n_dwords) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n_dwords; i += (size_t)gridDim.x * 256) p[i] = 0u;
}

hipError_t launch_fill_zero(void* p, size_t bytes, hipStream_t stream) {
    const size_t n = bytes / 4;
    if (n == 0) return hipSuccess;
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (blocks > 4096) blocks = 4096;
    fill_zero_kernel<<<dim3(blocks), dim3(256), 0, stream>>>((uint32_t*)p, n);
    return hipGetLastError();
}

// Grid-stride 16-byte reads, xor-folded so the loads cannot be dropped.
__global__ __launch_bounds__(256) void read_probe_kernel(const v4i* __restrict__ src, size_t n_vec,
                                                         uint32_t* __restrict__ sink) {
    uint32_t acc = 0;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n_vec; i += (size_t)gridDim.x * 256) {
        const v4i v = __builtin_nontemporal_load(src + i);
        acc ^= (uint32_t)(v.x ^ v.y ^ v.z ^ v.w);
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;  // practically never true: keeps the loads alive
}

hipError_t launch_read_probe(const void* src, size_t bytes, uint32_t* sink, hipStream_t stream) {
    const size_t n = bytes / 16;
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (blocks > 256 * 16) blocks = 256 * 16;
    if (blocks == 0) blocks = 1;
    read_probe_kernel<<<dim3(blocks), dim3(256), 0, stream>>>((const v4i*)src, n, sink);
    return hipGetLastError();
}

}  // namespace w2a8
