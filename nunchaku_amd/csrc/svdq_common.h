// Shared host/device helpers of the gfx950 SVDQuant W4A4 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/svdq_amd.h"

namespace svdq {

// ---- error reporting (thread local, no allocation) ---------------------------------------------
inline char *err_buf() {
    static thread_local char buf[512] = {0};
    return buf;
}
inline int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(err_buf(), 512, fmt, ap);
    va_end(ap);
    return code;
}
// A launch is reported by what hipGetLastError() says right after it.  That call returns the last error of the
// thread, whoever caused it, so an error left behind by an earlier call (this library's or anybody else's) is
// discarded first: what check_launch reports then belongs to the launch it follows.
#define SVDQ_LAUNCH(...)                 \
    do {                                 \
        (void)hipGetLastError();         \
        hipLaunchKernelGGL(__VA_ARGS__); \
    } while (0)
inline int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SVDQ_ELAUNCH, "%s: %s (%s)", what, hipGetErrorString(e), hipGetErrorName(e));
    return SVDQ_OK;
}
// number of compute units of a device, asked once (0: the query failed)
inline int compute_units(int dev) {
    static int cached[64] = {0};
    if (dev < 0 || dev >= 64) return 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            return 0;
        }
        cached[dev] = n;
    }
    return cached[dev];
}
#define SVDQ_REQUIRE(cond, ...) \
    do {                        \
        if (!(cond)) return svdq::fail(SVDQ_EINVAL, __VA_ARGS__); \
    } while (0)

// ---- vector types -------------------------------------------------------------------------------
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// ---- bf16 <-> fp32 bit helpers ------------------------------------------------------------------
__host__ __device__ inline float bf16_bits_to_f32(uint32_t b) {
    union { uint32_t u; float f; } v;
    v.u = b << 16;
    return v.f;
}
__host__ __device__ inline uint32_t f32_bits(float f) {
    union { uint32_t u; float f; } v;
    v.f = f;
    return v.u;
}
__host__ __device__ inline float bits_f32(uint32_t u) {
    union { uint32_t u; float f; } v;
    v.u = u;
    return v.f;
}
// round-to-nearest-even fp32 -> bf16 bit pattern (finite inputs); on the device this is the hardware
// conversion (v_cvt_pk_bf16_f32), on the host the usual integer rounding
__host__ __device__ inline uint32_t f32_to_bf16_bits(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
#else
    uint32_t u = f32_bits(f);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return u >> 16;
#endif
}

// two fp32 -> packed bf16 pair (lo in bits [15:0]), round-to-nearest-even: one v_cvt_pk_bf16_f32
__device__ inline uint32_t pack_bf16x2(float lo, float hi) {
    typedef float float2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2_t{lo, hi}, bf16x2_t));
}

// Native tile geometry of NVFP4 operands (activations and weights alike):
//   [rows/32][K/64][32 rows][8 words]; word w of a (row, 64-group) holds elements 8w .. 8w+7, element e
//   of a word in bits [4e, 4e+4) (plain E2M1 nibbles).
constexpr int TILE_ROWS = 32;
constexpr int GROUP_K = 64;
constexpr int TILE_BYTES = TILE_ROWS * GROUP_K / 2;  // 1024

__host__ __device__ inline uint32_t rotl32(uint32_t x, int r) { return (x << r) | (x >> (32 - r)); }

// INT4 operands of the GEMM (activations and weights alike) are stored as E2M3 (fp6) patterns of
// code / 8, which is exact for every code in [-15, 15]: the fp6 matrix instruction then multiplies the
// bare codes at twice the INT8 rate and returns fp32.  (Divided by 8 the codes fill the format's
// subnormals and its first binade, where the spacing is uniform: the pattern is the sign and the 4-bit
// magnitude as they are, and the hardware's round-to-nearest-even conversion of a real number to the
// format IS the rounding to the nearest integer code.)  A "fragment" is one operand of
// v_mfma_f32_32x32x64_f8f6f4: 32 rows x 64 codes (one k-group) = 1536 bytes.  Slot s = row + 32 * half
// (half = which 32 of the 64 codes) owns the 192-bit string with code j of its half in bits
// [6 j, 6 j + 6); the first 16 bytes of the string are stored at 16 s, the last 8 at 1024 + 8 s, so that
// a wave fetches a fragment with one 16-byte and one 8-byte LDS read per lane, both conflict-free.
// Fragments are grouped per workgroup tile: activations [M_pad/128][K/64][4 fragments], weights
// [ceil(N/256)][K/64][8 fragments] (columns beyond N hold zero codes): a workgroup's operands of one
// k-group are one contiguous run of 6 KB and one of 12 KB.
constexpr int FRAG_BYTES = 1536;
constexpr int ACT_BLOCK_ROWS = 128, WGT_BLOCK_COLS = 256;

// E2M3 pattern of code / 8 for an integer code in [-15, 15] (bias 1, subnormals, no inf / nan):
// magnitudes 0..7 are the subnormals x / 8, 8..15 the first binade 1 + (x - 8) / 8, so the five low bits
// are x itself; the sign is bit 5.
__host__ __device__ inline uint32_t int4_code_to_e2m3(int code) {
    const uint32_t x = code < 0 ? -code : code;
    const uint32_t m = x;
    return m | (code < 0 ? 32u : 0u);
}

}  // namespace svdq
