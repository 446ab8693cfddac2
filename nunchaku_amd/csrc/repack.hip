// Load-time conversion of reference-format checkpoint tensors into the layouts the gfx950 kernels
// read.  Every kernel is a plain gather: one thread computes where its output element lives in the
// reference storage (the 32-lane fragment order written by NunchakuWeightPacker,
// nunchaku/lora/flux/packer.py:187-398) and copies it.  These run once per tensor, so they are
// written for clarity, not speed.
#include "svdq_common.h"

using namespace svdq;

namespace {

// ---- qweight ------------------------------------------------------------------------------------
// Reference storage (packer.py:210-239, loader gemm_base.cuh:278-294): u32 words
// [N/128][K/64][j:8][lane:32][c:4]; word c of lane (g = lane/4, t = lane%4) in 16-row tile j holds
// row 16j + g + 8*(c>=2), columns 32*(c odd) + 8t + [0..8), element e in bits [4e, 4e+4).
// Native form of NVFP4 weights: [N/32][K/64][32 rows][8 words], word w of a row holds columns
// 8w + [0..8), plain nibbles.  (INT4 weights take the other kernel below.)
__global__ void repack_qweight_kernel(const uint32_t *__restrict__ src, uint32_t *__restrict__ dst, int64_t N, int64_t K) {
    const int64_t total = N * K / 8;
    const int64_t kgroups = K / 64;
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int w = i % 8;
        const int r = (i / 8) % 32;
        const int64_t g = (i / 256) % kgroups;
        const int64_t nt = i / (256 * kgroups);
        const int64_t n = nt * 32 + r;
        const int64_t bn = n / 128;
        const int nn = n % 128;
        const int j = nn / 16, gl = nn % 8, chi = (nn % 16) / 8;
        const int codd = w / 4, t = w % 4;
        const int lane = gl * 4 + t, c = chi * 2 + codd;
        const int64_t s = (((bn * kgroups + g) * 8 + j) * 32 + lane) * 4 + c;
        dst[i] = src[s];
    }
}

// INT4 weights for the fp6 matrix instruction: E2M3 fragments [ceil(N/256)][K/64][8 fragments]
// (svdq_common.h).  One thread per fragment slot = (row, half of the k-group): it gathers the four
// reference words that hold the row's 32 codes of that half and writes the 192-bit string.
__global__ void repack_qweight_e2m3_kernel(const uint32_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t N, int64_t K) {
    const int64_t kgroups = K / 64;
    const int64_t nblocks = (N + WGT_BLOCK_COLS - 1) / WGT_BLOCK_COLS;
    const int64_t total = nblocks * kgroups * 8 * 64;
    const int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int slot = (int)(i % 64);
    const int frag = (int)((i / 64) % 8);
    const int64_t g = (i / 512) % kgroups;
    const int64_t nblk = i / (512 * kgroups);
    const int64_t n = nblk * WGT_BLOCK_COLS + frag * 32 + slot % 32;
    const int half = slot / 32;
    unsigned long long bits[3] = {0, 0, 0};
    if (n < N) {
        const int64_t bn = n / 128;
        const int nn = (int)(n % 128);
        const int j16 = nn / 16, gl = nn % 8, chi = (nn % 16) / 8;
        const int c = chi * 2 + half;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint32_t word = src[(((bn * kgroups + g) * 8 + j16) * 32 + (gl * 4 + t)) * 4 + c];
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int nib = (word >> (4 * e)) & 0xF;
                const unsigned long long pat = int4_code_to_e2m3(nib >= 8 ? nib - 16 : nib);
                const int bit = 6 * (8 * t + e);
                bits[bit / 64] |= pat << (bit % 64);
                if (bit % 64 > 58) bits[bit / 64 + 1] |= pat >> (64 - bit % 64);
            }
        }
    }
    uint8_t *f = dst + ((nblk * kgroups + g) * 8 + frag) * FRAG_BYTES;
    *(unsigned long long *)(f + slot * 16) = bits[0];
    *(unsigned long long *)(f + slot * 16 + 8) = bits[1];
    *(unsigned long long *)(f + 1024 + slot * 8) = bits[2];
}

// ---- 16-bit per-channel values in the reference "wscale" order ----------------------------------
// Reference storage (packer.py:286-301, loader gemm_base.cuh:474-489): [N/128][G][lane:32][v:4];
// lane holds channels 16*(lane/4) + 2*(lane%4) + {0, 1, 8, 9}.
__device__ inline int64_t wscale_src_index(int64_t g, int64_t n, int64_t G) {
    const int64_t bn = n / 128;
    const int nn = n % 128;
    const int a = nn / 16, b = (nn % 16) / 8, c = (nn % 8) / 2, d = nn % 2;
    return ((bn * G + g) * 32 + (4 * a + c)) * 4 + (2 * b + d);
}

// INT4 weight scales as the operand of the GEMM's factor MFMA: [ceil(N/256)][K/64][256 columns] x
// {bf16(64 s), 0, 0, 0} (the 64 undoes the division by 8 of both operands' codes; exact, a power of two).
// Columns beyond N hold zero.
__global__ void repack_wscales_kernel(const uint16_t *__restrict__ src, unsigned long long *__restrict__ dst, int64_t N, int64_t G) {
    const int64_t nblocks = (N + WGT_BLOCK_COLS - 1) / WGT_BLOCK_COLS;
    const int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (i >= nblocks * G * WGT_BLOCK_COLS) return;
    const int64_t n = (i / (G * WGT_BLOCK_COLS)) * WGT_BLOCK_COLS + i % WGT_BLOCK_COLS;
    const int64_t g = (i / WGT_BLOCK_COLS) % G;
    unsigned long long v = 0;
    if (n < N) v = f32_to_bf16_bits(64.0f * bf16_bits_to_f32(src[wscale_src_index(g, n, G)]));
    dst[i] = v;
}

// exponent shift that puts the largest NVFP4 scale of a column into [2^10, 2^11): the fp16 products
// of the NVFP4 GEMM then stay below the fp16 maximum
constexpr int NORM_TARGET_EXP = 10;

// ---- NVFP4 micro scales --------------------------------------------------------------------------
// Reference storage (packer.py:346-360, loader gemm_w4a4.cuh:75-83): bytes
// [N/128][K/64][lane:32][p:4][byte:4]; word p of lane L is channel 32p + 8*(L%4) + L/4, its bytes
// the four 16-wide groups of the 64-wide k tile.
__device__ inline float e4m3_to_f32(uint32_t b) {
    const uint32_t ex = (b >> 3) & 0xF, m = b & 7;
    float v = ex == 0 ? ldexpf((float)m, -9) : ldexpf((float)(8 + m), (int)ex - 10);
    return (b & 0x80) ? -v : v;
}

__global__ void repack_wmscales_kernel(const uint8_t *__restrict__ src, _Float16 *__restrict__ dst,
                                       float *__restrict__ colnorm, int64_t N, int64_t G) {
    const int64_t n = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (n >= N) return;
    const int64_t bn = n / 128;
    const int nn = n % 128;
    const int p = nn / 32, q = (nn % 32) / 8, w = nn % 8;
    const int lane = 4 * w + q;
    const int64_t ktiles = G / 4;
    float amax = 0.f;
    for (int64_t g = 0; g < G; g++) {
        const int64_t s = (((bn * ktiles + g / 4) * 32 + lane) * 4 + p) * 4 + (g % 4);
        amax = fmaxf(amax, fabsf(e4m3_to_f32(src[s])));
    }
    int e = 0;
    if (amax > 0.f) {
        int ex;
        frexpf(amax, &ex);
        e = NORM_TARGET_EXP - (ex - 1);
    }
    for (int64_t g = 0; g < G; g++) {
        const int64_t s = (((bn * ktiles + g / 4) * 32 + lane) * 4 + p) * 4 + (g % 4);
        dst[((g / 4) * N + n) * 4 + (g % 4)] = (_Float16)ldexpf(e4m3_to_f32(src[s]), e);  // [K/64][N][4]
    }
    colnorm[n] = ldexpf(1.0f, -e);
}

__global__ void repack_vector_kernel(const uint16_t *__restrict__ src, uint16_t *__restrict__ dst, int64_t N) {
    const int64_t n = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (n < N) dst[n] = src[wscale_src_index(0, n, 1)];
}

__global__ void repack_smooth_kernel(const uint16_t *__restrict__ src, float *__restrict__ dst, int64_t K) {
    const int64_t k = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (k < K) dst[k] = __fdiv_rn(1.0f, bf16_bits_to_f32(src[wscale_src_index(0, k, 1)]));
}

// ---- low-rank weights ----------------------------------------------------------------------------
// Reference storage (packer.py:362-398, loader lora.cuh:43-59): 16-bit values
// [C/16][R/16][lane:32][d:4][h:2] with g = lane/4, t = lane%4:
//   down: channel = 16c + 2t + h + 8*(d odd), rank = 16r + g + 8*(d>=2)
//   up:   channel = 16c + g + 8*(d>=2),       rank = 16r + 2t + h + 8*(d odd)
__device__ inline int64_t lora_src_index(int64_t ch, int64_t rk, int64_t R, bool down) {
    const int64_t c = ch / 16, r = rk / 16;
    const int cc = ch % 16, rr = rk % 16;
    int g, t, h, d;
    if (down) {
        t = (cc % 8) / 2; h = cc % 2; g = rr % 8;
        d = 2 * (rr / 8) + cc / 8;
    } else {
        g = cc % 8; t = (rr % 8) / 2; h = rr % 2;
        d = 2 * (cc / 8) + rr / 8;
    }
    return (((c * (R / 16) + r) * 32 + (4 * g + t)) * 4 + d) * 2 + h;
}

// Native proj_down: [K/128][step:4][R/16][lane:64][8]; lane (rank = lane%16, q = lane/16) of MFMA
// step i holds proj_down[128c + 32q + 8i + j][16*rt + rank], j = 0..7.
__global__ void repack_lora_down_kernel(const uint16_t *__restrict__ src, uint16_t *__restrict__ dst, int64_t K, int64_t R) {
    const int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (i >= K * R) return;
    const int j = i % 8;
    const int lane = (i / 8) % 64;
    const int64_t rt = (i / 512) % (R / 16);
    const int step = (i / (512 * (R / 16))) % 4;
    const int64_t c = i / (2048 * (R / 16));
    const int64_t k = 128 * c + 32 * (lane / 16) + 8 * step + j;
    const int64_t rk = 16 * rt + lane % 16;
    dst[i] = src[lora_src_index(k, rk, R, true)];
}

__global__ void repack_lora_up_kernel(const uint16_t *__restrict__ src, uint16_t *__restrict__ dst, int64_t N, int64_t R) {
    const int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (i >= N * R) return;
    dst[i] = src[lora_src_index(i / R, i % R, R, false)];
}

// Rotary table: one thread per float of the native order [rows/32][16 slots][64 lanes][4].  Source: the
// order written by pack_rotemb (nunchaku/models/embeddings.py:88-120) = float4 [rows/16][16 tiles j][32
// lanes], lane 4 g + t holding floats 8 j + 2 t + {0, 1} of rows g (.xy) and g + 8 (.zw)
// (loader: src/kernels/zgemm/epilogues.cuh:282-305).
__global__ void repack_rotemb_kernel(const float *__restrict__ src, float *__restrict__ dst, int64_t rows) {
    const int64_t o = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
    if (o >= rows * 128) return;
    const int e = (int)(o & 3), l = (int)((o >> 2) & 63), s = (int)((o >> 8) & 15);
    const int64_t b = o >> 12;
    const int64_t row = 32 * b + (l & 31);
    const int d = 32 * (s >> 2) + 8 * (s & 3) + 4 * (l >> 5) + e;  // float of the row: sin of pair d/2 (even d) or cos (odd d)
    const int rr = (int)(row & 15), g = rr & 7, half = rr >> 3;
    const int j = d >> 3, t = (d & 7) >> 1;
    dst[o] = src[((((row >> 4) * 16 + j) * 8 + g) * 4 + t) * 4 + half * 2 + (d & 1)];
}

inline unsigned blocks_for(int64_t n, int bs = 256) { return (unsigned)((n + bs - 1) / bs); }

}  // namespace

extern "C" {

int svdq_abi_version(void) { return SVDQ_ABI_VERSION; }
const char *svdq_last_error(void) { return svdq::err_buf(); }

int svdq_repack_qweight(const void *src, void *dst, int64_t N, int64_t K, int fp4, void *stream) {
    SVDQ_REQUIRE(src && dst, "repack_qweight: null pointer");
    SVDQ_REQUIRE(src != dst, "repack_qweight: in-place repack is not supported");
    SVDQ_REQUIRE(N > 0 && K > 0 && N % 128 == 0 && K % 128 == 0, "repack_qweight: N (%lld) and K (%lld) must be multiples of 128",
                 (long long)N, (long long)K);
    if (!fp4) {
        const int64_t slots = ((N + WGT_BLOCK_COLS - 1) / WGT_BLOCK_COLS) * (K / 64) * 8 * 64;
        SVDQ_REQUIRE((uintptr_t)dst % 16 == 0, "repack_qweight: dst must be 16-byte aligned");
        SVDQ_LAUNCH(repack_qweight_e2m3_kernel, dim3(blocks_for(slots)), dim3(256), 0, (hipStream_t)stream, (const uint32_t *)src,
                           (uint8_t *)dst, N, K);
        return check_launch("repack_qweight");
    }
    const int64_t total = N * K / 8;
    unsigned grid = blocks_for(total);
    if (grid > 65536u) grid = 65536u;
    SVDQ_LAUNCH(repack_qweight_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const uint32_t *)src,
                       (uint32_t *)dst, N, K);
    return check_launch("repack_qweight");
}

int svdq_repack_wscales(const void *src, void *dst_scales, int64_t N, int64_t K, void *stream) {
    SVDQ_REQUIRE(src && dst_scales, "repack_wscales: null pointer");
    SVDQ_REQUIRE(N > 0 && K > 0 && N % 128 == 0 && K % 64 == 0, "repack_wscales: N %% 128 and K %% 64 must be 0");
    SVDQ_REQUIRE((uintptr_t)dst_scales % 16 == 0, "repack_wscales: dst must be 16-byte aligned");
    const int64_t total = ((N + WGT_BLOCK_COLS - 1) / WGT_BLOCK_COLS) * (K / 64) * WGT_BLOCK_COLS;
    SVDQ_LAUNCH(repack_wscales_kernel, dim3(blocks_for(total)), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)src,
                       (unsigned long long *)dst_scales, N, K / 64);
    return check_launch("repack_wscales");
}

int svdq_repack_wmscales(const void *src, void *dst_scales, void *dst_colnorm, int64_t N, int64_t K, void *stream) {
    SVDQ_REQUIRE(src && dst_scales && dst_colnorm, "repack_wmscales: null pointer");
    SVDQ_REQUIRE(N > 0 && K > 0 && N % 128 == 0 && K % 64 == 0, "repack_wmscales: N %% 128 and K %% 64 must be 0");
    SVDQ_LAUNCH(repack_wmscales_kernel, dim3(blocks_for(N)), dim3(256), 0, (hipStream_t)stream, (const uint8_t *)src,
                       (_Float16 *)dst_scales, (float *)dst_colnorm, N, K / 16);
    return check_launch("repack_wmscales");
}

int svdq_repack_vector(const void *src, void *dst, int64_t N, void *stream) {
    SVDQ_REQUIRE(src && dst && src != dst, "repack_vector: null or aliased pointer");
    SVDQ_REQUIRE(N > 0 && N % 128 == 0, "repack_vector: N (%lld) must be a multiple of 128", (long long)N);
    SVDQ_LAUNCH(repack_vector_kernel, dim3(blocks_for(N)), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)src,
                       (uint16_t *)dst, N);
    return check_launch("repack_vector");
}

int svdq_repack_smooth(const void *src, void *dst_rcp, int64_t K, void *stream) {
    SVDQ_REQUIRE(src && dst_rcp, "repack_smooth: null pointer");
    SVDQ_REQUIRE(K > 0 && K % 128 == 0, "repack_smooth: K (%lld) must be a multiple of 128", (long long)K);
    SVDQ_LAUNCH(repack_smooth_kernel, dim3(blocks_for(K)), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)src,
                       (float *)dst_rcp, K);
    return check_launch("repack_smooth");
}

int svdq_repack_lora_down(const void *src, void *dst, int64_t K, int64_t R, void *stream) {
    SVDQ_REQUIRE(src && dst && src != dst, "repack_lora_down: null or aliased pointer");
    SVDQ_REQUIRE(K > 0 && K % 128 == 0 && R > 0 && R % 16 == 0, "repack_lora_down: K %% 128 and R %% 16 must be 0");
    SVDQ_LAUNCH(repack_lora_down_kernel, dim3(blocks_for(K * R)), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t *)src, (uint16_t *)dst, K, R);
    return check_launch("repack_lora_down");
}

int svdq_repack_lora_up(const void *src, void *dst, int64_t N, int64_t R, void *stream) {
    SVDQ_REQUIRE(src && dst && src != dst, "repack_lora_up: null or aliased pointer");
    SVDQ_REQUIRE(N > 0 && N % 16 == 0 && R > 0 && R % 16 == 0, "repack_lora_up: N %% 16 and R %% 16 must be 0");
    SVDQ_LAUNCH(repack_lora_up_kernel, dim3(blocks_for(N * R)), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t *)src, (uint16_t *)dst, N, R);
    return check_launch("repack_lora_up");
}

int svdq_repack_rotemb(const void *src, void *dst, int64_t rows, void *stream) {
    SVDQ_REQUIRE(src && dst && src != dst, "repack_rotemb: null or aliased pointer");
    SVDQ_REQUIRE(rows > 0 && rows % 32 == 0, "repack_rotemb: rows (%lld) must be a positive multiple of 32", (long long)rows);
    SVDQ_LAUNCH(repack_rotemb_kernel, dim3(blocks_for(rows * 128)), dim3(256), 0, (hipStream_t)stream, (const float *)src,
                       (float *)dst, rows);
    return check_launch("repack_rotemb");
}

}  // extern "C"
