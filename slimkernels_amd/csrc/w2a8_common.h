// Shared definitions of the gfx950 W2A8 kernels: the streaming weight layout, the
// kernel parameter block and a few device helpers.
//
// Streaming weight layout ("repacked", private to this library)
// -------------------------------------------------------------
// The N x K code matrix is cut into units of 64 output channels (a "strip") by
// 64 reduction elements (a "step").  One unit is 1 KiB: 64 lanes x 4 dwords, stored
// so that lane l of a wavefront reads its 16 bytes at offset 16*l (one coalesced
// global_load_dwordx4 / one conflict-free ds_read_b128 per wave and unit).
//
//   unit address   = w_r + ((((step / 4) * strips + strip) * 4 + step % 4) * 64 + lane) * 4     [dwords]
//   (four consecutive steps of a strip form one run of 4 KiB, the runs of all strips for the same four steps follow
//    each other: what a wave streams back to back is contiguous, and what all strips need at the same moment is one
//    sequential band - a whole strip in one piece would be `strips` power-of-two-strided streams that pile onto a few
//    HBM channels, single 1 KiB units per step measured 3..9 % slower than the 4 KiB runs; a step count that is no
//    multiple of four is padded with zero units)
//   lane l         : col = l & 15, quad = l >> 4
//   dword i, byte b, 2-bit field p of that byte (bits 2p+1:2p) holds the code of
//       n = strip*64 + p*16 + col          k = step*64 + quad*16 + 4*i + b
//
// so `dword_i & (0x03030303 << 2p)` for i = 0..3 IS the 16-byte B operand of
// v_mfma_i32_16x16x64_i8 for the 16 channels of sub-block p, scaled by 4^p, with no
// shifts: one v_and per operand dword.  Field p = 3 sits in the sign bits of its
// byte, so the repack stores it as (code xor 2) = two's complement of (code - 2);
// the byte then reads as 64 * (code - 2).  The 4^p factor is divided out of the
// fp32 scale (exact, a power of two) and the "-2" moves into the zero-point.
//
// Scales and zero-points are stored per (group, strip) as [16 cols][4 sub-blocks]
// (index (group * strips + strip) * 64 + col * 4 + p) so that a lane fetches the four
// values it needs with one 8-byte (4-byte) load.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace w2a8 {

constexpr int kStripN = 64;      // output channels per strip
constexpr int kStepK = 64;       // reduction elements per MFMA step
constexpr int kUnitDwords = 256; // dwords per (strip, step) unit
// Order of the units in memory: kRunSteps consecutive steps of a strip lie together (a run of 4 KiB: what one wave
// streams back to back), the runs of all strips for the same steps follow each other, then the next kRunSteps steps.
// A step count that is no multiple of kRunSteps is padded with zero units.
constexpr int kRunSteps = 4;
constexpr int kUnitBytes = kUnitDwords * 4;
__host__ __device__ constexpr int weight_runs(int steps) { return (steps + kRunSteps - 1) / kRunSteps; }
__host__ __device__ constexpr size_t weight_bytes(int strips, int steps) {
    return (size_t)weight_runs(steps) * (size_t)strips * kRunSteps * kUnitBytes;
}
// byte offset of unit (step, strip): a kernel keeps run_pitch = strips * kRunSteps * kUnitBytes and
// strip_base = strip * kRunSteps * kUnitBytes and adds (step / kRunSteps) * run_pitch + (step % kRunSteps) * kUnitBytes
__host__ __device__ constexpr uint32_t weight_unit_offset(int step, int strip, int strips) {
    return (uint32_t)((((step / kRunSteps) * strips + strip) * kRunSteps + step % kRunSteps) * kUnitBytes);
}

typedef int v4i __attribute__((ext_vector_type(4)));

struct GemmParams {
    const int8_t* q;        // [M][ldq]
    const uint16_t* x;      // fused activation quantisation only: [M][ldx] fp16 / bf16 bits
    const float* s_a;       // [M]
    const int32_t* rowsum;  // [G][ldr]
    const uint32_t* w_r;    // repacked codes
    const uint16_t* s_r;    // [G][strips][16][4] fp16 bits
    const uint8_t* zp_r;    // [G][strips][16][4] or nullptr
    void* out;              // [M][ldo] fp16 / bf16 bits
    int32_t* acc_dump;      // verification output or nullptr
    float* ws_partial;      // split-K partial tiles
    unsigned* ws_counter;   // split-K arrival counters (zero between calls)
    int ldq, ldr, ldo;
    int ldx, x_bf16;        // fused activation quantisation only
    int M, N, K;
    int G;                  // number of scale groups = K / group_size
    int steps;              // K / 64
    int strips;             // ceil(N / 64)
    int zp_const;
    int dump_mode;
    int split;              // split-K factor (grid.y)
    int groups_per_split;   // ceil(G / split)
};

// A split-K workspace starts with a block of arrival counters of fixed size (64 KiB), whatever the problem; the
// kernels that quantise the token rows themselves keep their two counters (rows ready, workgroups past the wait) in
// its last two slots.
constexpr int kCounterBlockBytes = 64 << 10;
constexpr int kRowFlagSlot = kCounterBlockBytes / 4 - 2;
constexpr int kMaxSplitCounters = kRowFlagSlot;  // arrival counters a split-K launch may use
constexpr int kRowsMax = 32;                     // token rows of a launch that quantises them itself

// Problem table of a grouped skinny launch; passed by value in the kernel arguments (< 4 KiB).
constexpr int kGroupedWavesPerWg = 8;  // wavefronts per workgroup of the grouped skinny kernel
constexpr int kFusedMaxRows = 4;       // fused activation quantisation: at most this many token rows ...
constexpr int kFusedMaxBytes = 32768;  // ... and rows x K int8 values (held in LDS)
constexpr int kSharedParts = 2;  // k-parts per workgroup when one problem runs through the shared-activation workgroups
constexpr int kMaxGroup = 24;
struct GroupedParams {
    GemmParams prob[kMaxGroup];
    int wg_begin[kMaxGroup + 1];  // problem i owns workgroups wg_begin[i] .. wg_begin[i+1]-1
    int kparts[kMaxGroup];  // 1, 2, 4 or 8: parts K is split into inside a workgroup of eight waves (8, 4, 2 or 1 strips)
    uint32_t xcd_slots[kMaxGroup];  // 3 bits per XCD x: which unit of a set of eight the workgroup with id % 8 == x takes
    int count;
};

__device__ __forceinline__ v4i mfma_i8_16x16x64(v4i a, v4i b, v4i c) {
    // D[i][j] += sum_k A[i][k] * B[k][j]; lane l supplies row/col (l & 15) and the
    // 16 k-values of quarter (l >> 4); D lane l, element j = row 4*(l>>4)+j, col l&15.
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
}

// rintf(x / s) for |x / s| <= 127, with 1 / s at hand.  t = x * (1 / s) lies within 1.5 * 2^-23 * 127 = 2.3e-5 of the
// quotient the IEEE division returns, so the two round to the same integer unless t is that close to a tie; t - rintf(t)
// is exact, and within 2^-14 of a tie the division decides.  Bit-identical with rintf(x / s) for finite x.
__device__ __forceinline__ float rne_quotient(float x, float s, float inv_s) {
    const float t = x * inv_s;
    const float r = rintf(t);
    if (fabsf(fabsf(t - r) - 0.5f) < 6.1035156e-5f) return rintf(x / s);
    return r;
}

__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

// Verification instantiations only: record the exact int32 sum of one (token m, channel n, scale group g).
// `value` is sum_k q * (code - c0) as the kernel's operand encoding yields it (c0 = 0 for the plain fields,
// 2 for the bytes centred on the symmetric levels, 8 for the joined 4-bit digits); the true sum
// sum_k q * (code - zp) follows in integers from the group's row sum.  W4: the zero-point is 4 * hi + lo of the two
// planes (rows g and g + G of zp_r), 8 without zp_r.
template <bool W4 = false>
__device__ __forceinline__ void dump_group_sum(const GemmParams& p, int m, int n, int g, int value, int c0) {
    if (m >= p.M || n >= p.N || g >= p.G) return;
    const size_t zi = (size_t)(n >> 6) * 64 + (n & 15) * 4 + ((n >> 4) & 3);
    int zp;
    if (W4) zp = p.zp_r ? 4 * (int)p.zp_r[(size_t)g * p.strips * 64 + zi] + (int)p.zp_r[(size_t)(g + p.G) * p.strips * 64 + zi] : 8;
    else zp = p.zp_r ? (int)p.zp_r[(size_t)g * p.strips * 64 + zi] : p.zp_const;
    int v = value;
    if (zp != c0) v += (c0 - zp) * p.rowsum[(size_t)g * p.ldr + m];
    if (p.dump_mode == 1) p.acc_dump[((size_t)m * p.N + n) * p.G + g] = v;
    else atomicAdd(p.acc_dump + (size_t)m * p.N + n, v);
}

// The output is defined as cast(fp32 product): the empty asm keeps the compiler from folding the
// caller's fp32 multiply into a v_fma_mixlo_f16, which would round the exact product once.
struct OutF16 {
    static __device__ __forceinline__ uint16_t cast(float v) {
        asm volatile("" : "+v"(v));
        return __builtin_bit_cast(uint16_t, (_Float16)v);
    }
};
struct OutBF16 {
    static __device__ __forceinline__ uint16_t cast(float v) {
        uint32_t x = __float_as_uint(v);
        if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
        x += 0x7fffu + ((x >> 16) & 1u);
        return (uint16_t)(x >> 16);
    }
};

// Placement of a one-dimensional grid on the eight XCDs.  Workgroups go to the XCDs in turn, so blockIdx.x & 7 names
// the XCD and blockIdx.x >> 3 the workgroup's place in that XCD's queue.  The work is `sets` sets of `members`
// workgroups each, the members of a set reading the same weights: they take consecutive places in one XCD's queue
// (all but the first read come from its L2), and the sets are dealt out to the XCDs evenly; what is left when their
// number is no multiple of eight goes round the XCDs member by member, so no XCD gets more than one workgroup more than
// another.  The grid is xcd_grid(sets, members) workgroups; false: a padding workgroup.
__host__ __device__ __forceinline__ bool xcd_place(const int local, const int sets, const int members, int& set, int& member) {
    const int even = sets >> 3, rest = sets & 7;
    const int xcd = local & 7, slot = local >> 3;
    if (slot < even * members) {
        set = (slot / members) * 8 + xcd;
        member = slot % members;
        return true;
    }
    const int t = (slot - even * members) * 8 + xcd;
    if (t >= rest * members) return false;
    set = even * 8 + t % rest;
    member = t / rest;
    return true;
}
inline int xcd_grid(const int sets, const int members) { return (sets * members + 7) / 8 * 8; }

}  // namespace w2a8
