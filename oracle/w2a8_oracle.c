/*
 * CPU oracle for the W2A8 GEMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain scalar C, the arithmetic the GPU kernels must
 * reproduce.  It is the checker used by tests/, by __graft_entry__.smoke() and
 * by the cpu_baseline leg of bench.py; nothing in the product package links,
 * imports or calls it.
 *
 * Reference anchors (paths relative to the upstream SlimKernels tree):
 *   w2o_pack / w2o_unpack        matrix_packer.py:29-34, :57-64
 *   w2o_quantize_w2 (mode REF)   quantization.py:26-46
 *   w2o_dequantize_w2            quantization.py:83-93
 *   operand orientation          slimkernels/cute/gemm/wgmma_sm90_W2A8.cu:528-531,563
 *                                (weights [N, K/4] bytes K-major, activations [M, K])
 *   MSB-first field order        slimkernels/cute/atom/mma_sm90_gmma.hpp:52-73
 * The int8 activation quantizer, the int32 accumulation and the dequant
 * epilogue have no upstream counterpart (the upstream kernel multiplies FP8
 * activations and stores nothing, wgmma_sm90_W2A8.cu:408); they are defined
 * here and pinned by closed forms, brute force and exact-arithmetic
 * invariants in tests/test_oracle.py.
 *
 * Pinning status of each function (what fails if it is wrong):
 *   w2o_pack, w2o_unpack     upstream known-answer vectors
 *                            (test_matrix_packer.py:7-22,45-58) + exhaustive bytes
 *   w2o_quantize_w2 REF      upstream known-answer vector (test_quantization.py:110-139),
 *                            zero matrix (:40-48), extreme values (:58-75)
 *   w2o_quantize_w2 SYM/ASYM closed-form level tables, tie vectors, reconstruction bound
 *   w2o_act_quant            closed form on hand-computed rows, tie vectors, invariants
 *   w2o_gemm_acc             brute-force python loops on tiny shapes, exact fp64/fp32
 *                            BLAS identity, zero-point folding identity
 *   w2o_epilogue             all-ones-scales special case, fp64 evaluation bound
 *
 * Build: see oracle/Makefile (gcc -O3 -ffp-contract=off; no fast-math, so the
 * float divisions and roundings are IEEE-754 binary32 exactly as written).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { W2O_MODE_REF = 0, W2O_MODE_SYM = 1, W2O_MODE_ASYM = 2 };

/* ---- fp16 / bf16 conversion (round to nearest even), no compiler extensions ---- */

static float half_bits_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: value = man * 2^-24 */
            float v = (float)man * 5.9604644775390625e-08f;
            memcpy(&bits, &v, 4);
            bits |= sign;
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static uint16_t float_to_half_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0u));
    }
    if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax < 0x33000001u) { /* < 2^-25 (or == 2^-25, ties to even -> 0) */
        return (uint16_t)sign;
    }
    int e = (int)(ax >> 23) - 127; /* unbiased exponent */
    uint32_t m = (ax & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift; /* number of low bits dropped */
    uint32_t base;
    if (e < -14) { /* subnormal half: value = q * 2^-24 */
        shift = -e - 1; /* m * 2^(e-23) / 2^-24 = m * 2^(e+1) */
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x7fffffu;
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q += 1; /* carry may bump the exponent: fine */
    return (uint16_t)(sign | (base + q));
}

static uint16_t float_to_bf16_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7fffu + lsb;
    return (uint16_t)(x >> 16);
}

static float bf16_bits_to_float(uint16_t b) {
    uint32_t x = (uint32_t)b << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

float w2o_half_to_float(uint16_t h) { return half_bits_to_float(h); }
uint16_t w2o_float_to_half(float f) { return float_to_half_bits(f); }
float w2o_bf16_to_float(uint16_t h) { return bf16_bits_to_float(h); }
uint16_t w2o_float_to_bf16(float f) { return float_to_bf16_bits(f); }

/* ---- 2-bit packer: matrix_packer.py:29-34 (pack), :57-64 (unpack) ----
 * codes [rows, cols] uint8 in 0..3  ->  out [rows, cols/4]; the first of each
 * four codes lands in bits 7:6, the last in bits 1:0.
 * returns 0, or 2 (cols % 4), 3 (value > 3) mirroring the upstream checks
 * at matrix_packer.py:16-21. */
int w2o_pack(const uint8_t* codes, long rows, long cols, uint8_t* out) {
    if (cols % 4 != 0) return 2;
    for (long i = 0; i < rows * cols; ++i)
        if (codes[i] > 3) return 3;
    long pc = cols / 4;
    for (long r = 0; r < rows; ++r)
        for (long j = 0; j < pc; ++j) {
            const uint8_t* c = codes + r * cols + 4 * j;
            out[r * pc + j] = (uint8_t)((c[0] << 6) | (c[1] << 4) | (c[2] << 2) | c[3]);
        }
    return 0;
}

int w2o_unpack(const uint8_t* packed, long rows, long pcols, uint8_t* codes) {
    for (long r = 0; r < rows; ++r)
        for (long j = 0; j < pcols; ++j) {
            uint8_t b = packed[r * pcols + j];
            uint8_t* c = codes + (r * pcols + j) * 4;
            c[0] = (b >> 6) & 3;
            c[1] = (b >> 4) & 3;
            c[2] = (b >> 2) & 3;
            c[3] = b & 3;
        }
    return 0;
}

/* ---- 2-bit group quantizer ----
 * w is [K, N] row-major (K rows are grouped, one scale per (group, column)),
 * exactly the orientation of quantization.py:26.  All arithmetic in binary32.
 *   REF  (quantization.py:29-46): s = max(absmax,1e-9)/1.5 ; code = clip(rne(w/s)+1, 0, 3)
 *   SYM  : s = max(absmax,1e-9)/2   ; code = clip(rne(w/s), -2, 1) + 2      (zero-point 2)
 *   ASYM : s = max(max-min,1e-9)/3  ; zp = clip(rne(-min/s), 0, 3) ; code = clip(rne(w/s)+zp, 0, 3)
 * rne = round half to even (numpy np.round, quantization.py:46; C rintf in the default mode).
 * scales [G, N] binary32; zp [G, N] uint8 (REF writes 1, SYM writes 2). */
int w2o_quantize_w2(const float* w, long K, long N, long g, int mode,
                    uint8_t* codes, float* scales, uint8_t* zp) {
    if (g <= 0 || K % g != 0) return 2;
    long G = K / g;
    for (long gi = 0; gi < G; ++gi)
        for (long n = 0; n < N; ++n) {
            float amax = 0.0f, vmax = -INFINITY, vmin = INFINITY;
            for (long r = 0; r < g; ++r) {
                float v = w[(gi * g + r) * N + n];
                float a = fabsf(v);
                if (a > amax) amax = a;
                if (v > vmax) vmax = v;
                if (v < vmin) vmin = v;
            }
            float s;
            int z;
            if (mode == W2O_MODE_REF) {
                s = fmaxf(amax, 1e-9f) / 1.5f;
                z = 1;
            } else if (mode == W2O_MODE_SYM) {
                s = fmaxf(amax, 1e-9f) / 2.0f;
                z = 2;
            } else {
                s = fmaxf(vmax - vmin, 1e-9f) / 3.0f;
                float zf = rintf(-vmin / s);
                z = (int)fminf(fmaxf(zf, 0.0f), 3.0f);
            }
            scales[gi * N + n] = s;
            zp[gi * N + n] = (uint8_t)z;
            for (long r = 0; r < g; ++r) {
                float v = w[(gi * g + r) * N + n];
                float q = rintf(v / s) + (float)z;
                q = fminf(fmaxf(q, 0.0f), 3.0f);
                codes[(gi * g + r) * N + n] = (uint8_t)q;
            }
        }
    return 0;
}

/* quantization.py:83-93 generalised to a per-(group, column) zero-point:
 * out[k, n] = fp16( (float(code) - zp) * scale ).  Upstream is zp == 1. */
int w2o_dequantize_w2(const uint8_t* codes, const float* scales, const uint8_t* zp,
                      long K, long N, long g, uint16_t* out_half) {
    if (g <= 0 || K % g != 0) return 2;
    for (long k = 0; k < K; ++k)
        for (long n = 0; n < N; ++n) {
            long gi = k / g;
            float v = ((float)codes[k * N + n] - (float)zp[gi * N + n]) * scales[gi * N + n];
            out_half[k * N + n] = float_to_half_bits(v);
        }
    return 0;
}

/* ---- per-token int8 activation quantizer (no upstream counterpart) ----
 * x [M, K] fp16 (x_is_bf16 = 0) or bf16 bits.
 *   s_a[m]  = max(absmax_k |x[m,k]|, 1e-9) / 127        (binary32 divide)
 *   q[m,k]  = clip(rne(x[m,k] / s_a[m]), -127, 127)      (binary32 divide)
 *   rowsum[gi, m] = sum_{k in group gi} q[m,k]          (int32, layout [G, ldr])
 */
int w2o_act_quant(const uint16_t* x, int x_is_bf16, long M, long K, long g,
                  int8_t* q, float* s_a, int32_t* rowsum, long ldr) {
    if (g <= 0 || K % g != 0) return 2;
    for (long m = 0; m < M; ++m) {
        float amax = 0.0f;
        for (long k = 0; k < K; ++k) {
            float v = x_is_bf16 ? bf16_bits_to_float(x[m * K + k]) : half_bits_to_float(x[m * K + k]);
            float a = fabsf(v);
            if (a > amax) amax = a;
        }
        float s = fmaxf(amax, 1e-9f) / 127.0f;
        s_a[m] = s;
        for (long gi = 0; gi < K / g; ++gi) {
            int32_t rs = 0;
            for (long k = gi * g; k < (gi + 1) * g; ++k) {
                float v = x_is_bf16 ? bf16_bits_to_float(x[m * K + k]) : half_bits_to_float(x[m * K + k]);
                float r = rintf(v / s);
                r = fminf(fmaxf(r, -127.0f), 127.0f);
                q[m * K + k] = (int8_t)r;
                rs += (int32_t)r;
            }
            if (rowsum) rowsum[gi * ldr + m] = rs;
        }
    }
    return 0;
}

/* ---- int32 per-group accumulators ----
 * acc[m, n, gi] = sum_{k in group gi} q[m,k] * (code[n,k] - zp[gi,n])
 * q [M, K] int8; packed [N, K/4] in the matrix_packer.py layout; zp [G, N]. */
int w2o_gemm_acc(const int8_t* q, const uint8_t* packed, const uint8_t* zp,
                 long M, long N, long K, long g, int32_t* acc) {
    if (g <= 0 || K % g != 0 || K % 4 != 0) return 2;
    long G = K / g;
    int8_t* wrow = (int8_t*)malloc((size_t)K);
    if (!wrow) return 9;
    for (long n = 0; n < N; ++n) {
        for (long j = 0; j < K / 4; ++j) {
            uint8_t b = packed[n * (K / 4) + j];
            wrow[4 * j + 0] = (int8_t)((b >> 6) & 3);
            wrow[4 * j + 1] = (int8_t)((b >> 4) & 3);
            wrow[4 * j + 2] = (int8_t)((b >> 2) & 3);
            wrow[4 * j + 3] = (int8_t)(b & 3);
        }
        for (long gi = 0; gi < G; ++gi) {
            int z = zp[gi * N + n];
            for (long k = gi * g; k < (gi + 1) * g; ++k) wrow[k] = (int8_t)(wrow[k] - z);
        }
        for (long m = 0; m < M; ++m) {
            const int8_t* a = q + m * K;
            for (long gi = 0; gi < G; ++gi) {
                int32_t s = 0;
                for (long k = gi * g; k < (gi + 1) * g; ++k) s += (int32_t)a[k] * (int32_t)wrow[k];
                acc[(m * N + n) * G + gi] = s;
            }
        }
    }
    free(wrow);
    return 0;
}

/* ---- dequant epilogue ----
 * t = 0; for gi ascending: t = fmaf(float(acc[m,n,gi]), float(scale_half[gi,n]), t)
 * out[m,n] = cast( t * s_a[m] )          cast = fp16 (out_is_bf16 = 0) or bf16, RNE.
 * scales are the fp16-stored values [G, N]. */
int w2o_epilogue(const int32_t* acc, const uint16_t* scale_half, const float* s_a,
                 long M, long N, long G, int out_is_bf16, uint16_t* out, float* out_f32) {
    for (long m = 0; m < M; ++m)
        for (long n = 0; n < N; ++n) {
            float t = 0.0f;
            for (long gi = 0; gi < G; ++gi)
                t = fmaf((float)acc[(m * N + n) * G + gi], half_bits_to_float(scale_half[gi * N + n]), t);
            float v = t * s_a[m];
            if (out_f32) out_f32[m * N + n] = v;
            if (out) out[m * N + n] = out_is_bf16 ? float_to_bf16_bits(v) : float_to_half_bits(v);
        }
    return 0;
}

/* Fused form used for timing the whole CPU path and for large shapes: never
 * materialises acc[M,N,G].  acc_sum (optional) receives sum_gi acc[m,n,gi]. */
int w2o_gemm_fused(const int8_t* q, const float* s_a, const uint8_t* packed,
                   const uint16_t* scale_half, const uint8_t* zp,
                   long M, long N, long K, long g, int out_is_bf16,
                   uint16_t* out, int32_t* acc_sum) {
    if (g <= 0 || K % g != 0 || K % 4 != 0) return 2;
    long G = K / g;
    int8_t* wrow = (int8_t*)malloc((size_t)K);
    if (!wrow) return 9;
    for (long n = 0; n < N; ++n) {
        for (long j = 0; j < K / 4; ++j) {
            uint8_t b = packed[n * (K / 4) + j];
            wrow[4 * j + 0] = (int8_t)((b >> 6) & 3);
            wrow[4 * j + 1] = (int8_t)((b >> 4) & 3);
            wrow[4 * j + 2] = (int8_t)((b >> 2) & 3);
            wrow[4 * j + 3] = (int8_t)(b & 3);
        }
        for (long gi = 0; gi < G; ++gi) {
            int z = zp[gi * N + n];
            for (long k = gi * g; k < (gi + 1) * g; ++k) wrow[k] = (int8_t)(wrow[k] - z);
        }
        for (long m = 0; m < M; ++m) {
            const int8_t* a = q + m * K;
            float t = 0.0f;
            int32_t tot = 0;
            for (long gi = 0; gi < G; ++gi) {
                int32_t s = 0;
                for (long k = gi * g; k < (gi + 1) * g; ++k) s += (int32_t)a[k] * (int32_t)wrow[k];
                tot += s;
                t = fmaf((float)s, half_bits_to_float(scale_half[gi * N + n]), t);
            }
            float v = t * s_a[m];
            if (out) out[m * N + n] = out_is_bf16 ? float_to_bf16_bits(v) : float_to_half_bits(v);
            if (acc_sum) acc_sum[m * N + n] = tot;
        }
    }
    free(wrow);
    return 0;
}
