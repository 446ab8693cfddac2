// Device-side core of the 4-bit activation quantizers, shared by the stand-alone quantize kernel and
// by the GEMM epilogue that quantizes for the next layer.  Arithmetic contract (IEEE fp32,
// round-to-nearest-even, no contraction), following src/kernels/zgemm/gemm_w4a4.cuh:429-523 (INT4) and
// :85-187 (NVFP4):
//   amax = max |y| over the group (y are bf16 values held as fp32)
//   INT4 : s = amax * fl32(1/7) (signed) or fl32(1/15) (unsigned); stored scale bf16(s);
//          code = clamp(rne(y * fl32(1/s)), lo, hi); a zero group gives codes 0 and scale 0
//   NVFP4: s = min(amax * fl32(1/6), 448); stored scale e4m3(s); code = e2m1(y * fl32(1/s))
#pragma once

#include "svdq_common.h"

namespace svdq {

constexpr float RECIP_7 = 1.0f / 7.0f;
constexpr float RECIP_15 = 1.0f / 15.0f;
constexpr float RECIP_6 = 1.0f / 6.0f;
constexpr float RNE_MAGIC = 12582912.0f;  // 1.5 * 2^23: adding it rounds to an integer (RNE)

__device__ inline float smooth_quotient(float x, float rcp) {
    // bf16(x / smooth) as fp32, see the header comment
    return bf16_bits_to_f32(f32_to_bf16_bits(__fmul_rn(x, rcp)));
}

// fp32 (finite, >= 0, <= 448) -> e4m3 bit pattern, round to nearest even
__device__ inline uint32_t f32_to_e4m3(float s) {
    if (s < 0.0009765625f) return 0;  // below half of the smallest subnormal (2^-10) rounds to 0
    if (s < 0.015625f) {              // subnormal range: multiples of 2^-9
        float t = __fadd_rn(__fmul_rn(s, 512.0f), RNE_MAGIC);
        return f32_bits(t) & 0xFF;    // 0..8 (8 == smallest normal, pattern 0x08)
    }
    uint32_t b = f32_bits(s);
    b += 0x7FFFFu + ((b >> 20) & 1u);  // round mantissa to 3 bits, ties to even
    const int ex = (int)(b >> 23) - 127 + 7;
    return (uint32_t)(ex << 3) | ((b >> 20) & 7u);
}

// fp32 -> 4-bit e2m1 pattern, round to nearest even, saturating at 6: the rule the hardware conversion
// below implements (grid 0 .5 1 1.5 2 3 4 6; ties go to the pattern with an even low bit; the sign bit
// is kept, also for zero).  Kept as the statement of the rule and for host-side checks.
__host__ __device__ inline uint32_t f32_to_e2m1(float v) {
    const float a = v < 0.f ? -v : v;
    uint32_t c;
    if (a <= 0.25f) c = 0;
    else if (a < 0.75f) c = 1;
    else if (a <= 1.25f) c = 2;
    else if (a < 1.75f) c = 3;
    else if (a <= 2.5f) c = 4;
    else if (a < 3.5f) c = 5;
    else if (a <= 5.0f) c = 6;
    else c = 7;
    return c | ((f32_bits(v) >> 28) & 8u);
}

// 8 fp32 -> one word of e2m1 patterns (element j in bits [4j, 4j+4)) with the hardware conversion
// v_cvt_scalef32_pk_fp4_f32 at scale 1: two values per instruction.  It agrees with f32_to_e2m1 on
// every non-NaN fp32 bit pattern (checked exhaustively on gfx950).
__device__ inline uint32_t pack8_e2m1(const float (&t)[8]) {
    uint32_t w = 0;
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, t[0], t[1], 1.0f, 0);
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, t[2], t[3], 1.0f, 1);
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, t[4], t[5], 1.0f, 2);
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, t[6], t[7], 1.0f, 3);
    return w;
}


// INT4: one lane holds 32 consecutive elements of a row = half of a 64-group; the other half lives in
// the lane `partner_xor` away.  The 32 codes of the lane leave as the E2M3
// patterns of code / 8, 6 bits each, code j in bits [6 j, 6 j + 6) of a 192-bit string (`lo` = bits
// [0, 128), `hi` = the rest).  The hardware conversion takes the even and the odd elements as two
// sources and interleaves them, divides by its scale operand (8: an exponent change) and rounds to the
// nearest E2M3 value, ties to even: below 2 the format's values are the multiples of 1 / 8, so this is the
// rounding of y * r to the nearest integer code (rne_to_int of the reference) and no separate rounding
// instruction is needed.
template <bool UNSIGNED>
__device__ inline void quantize_int4_half_group_e2m3(const float (&y)[32], int partner_xor, u32x4_t &lo, u32x2_t &hi, float &scale) {
    typedef uint32_t u32x6_t __attribute__((ext_vector_type(6)));
    float amax = 0.f;
#pragma unroll
    for (int e = 0; e < 32; e += 2) amax = __builtin_fmaxf(__builtin_fmaxf(amax, __builtin_fabsf(y[e])), __builtin_fabsf(y[e + 1]));  // one three-way maximum per pair
    amax = fmaxf(amax, __shfl_xor(amax, partner_xor));
    const float s = __fmul_rn(amax, UNSIGNED ? RECIP_15 : RECIP_7);
    const float rcp = s > 0.f ? __fdiv_rn(1.0f, s) : 0.f;
    float16_t ev, od;
#pragma unroll
    for (int e = 0; e < 16; e++) {
        if (UNSIGNED) {
            ev[e] = __builtin_amdgcn_fmed3f(__fmul_rn(y[2 * e], rcp), 0.0f, 15.0f);
            od[e] = __builtin_amdgcn_fmed3f(__fmul_rn(y[2 * e + 1], rcp), 0.0f, 15.0f);
        } else {
            // signed codes need no clamp: |y| <= amax and rcp = fl(1 / fl(amax / 7)) give |y * rcp| <= 7 (1 + 2^-21),
            // which rounds to 7 at most (the reference clamps to [-8, 7], which these values never leave)
            ev[e] = __fmul_rn(y[2 * e], rcp);
            od[e] = __fmul_rn(y[2 * e + 1], rcp);
        }
    }
    // The instruction works through its 32 inputs in several passes and writes result words while later inputs are
    // still to be read: a destination that overlaps the sources anywhere but at the first registers of the first
    // source comes out wrong in its last words (seen: the last two words when the register allocator placed the
    // destination across the end of the first source).  The compiler's definition of the instruction does not
    // say so; the early-clobber constraint below keeps the destination off both sources.
    u32x6_t w;
    asm("v_cvt_scalef32_2xpk16_fp6_f32 %0, %1, %2, %3" : "=&v"(w) : "v"(ev), "v"(od), "s"(8.0f));
    lo = u32x4_t{w[0], w[1], w[2], w[3]};
    hi = u32x2_t{w[4], w[5]};
    scale = s;
}

// One lane holds two whole 16-groups.  Produces 16 bytes of E2M1 patterns and the two E4M3 scales.
__device__ inline void quantize_nvfp4_two_groups(const float (&y)[32], u32x4_t &words, uint32_t (&sc)[2]) {
#pragma unroll
    for (int h = 0; h < 2; h++) {
        float amax = 0.f;
#pragma unroll
        for (int e = 0; e < 16; e++) amax = fmaxf(amax, fabsf(y[16 * h + e]));
        const float s = fminf(__fmul_rn(amax, RECIP_6), 448.0f);
        const float rcp = s > 0.f ? __fdiv_rn(1.0f, s) : 0.f;
        sc[h] = f32_to_e4m3(s);
#pragma unroll
        for (int wi = 0; wi < 2; wi++) {
            float t[8];
#pragma unroll
            for (int j = 0; j < 8; j++) t[j] = __fmul_rn(y[16 * h + 8 * wi + j], rcp);
            // (a zero group gives codes 0 whatever the signs of its zeros)
            words[2 * h + wi] = s > 0.f ? pack8_e2m1(t) : 0u;
        }
    }
}

}  // namespace svdq
