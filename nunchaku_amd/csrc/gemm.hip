// Operator 2: W4A4 GEMM with fused epilogue for gfx950.  Counterpart of gemm_w4a4_kernel /
// gemm_w4a4_fp4_kernel (src/kernels/zgemm/gemm_w4a4.cuh:1046-1095, :358-405) and of the epilogue
// chain composed in gemm_w4a4_launch_impl.cuh:172-309.
//
// How the contraction is mapped to the matrix cores
// -------------------------------------------------
// Every 64-wide (16-wide for NVFP4) k-group carries its own activation scale (per row) and weight
// scale (per column).  Applying them after an integer MFMA costs three VALU instructions per
// accumulator per group, which caps an int8-MFMA kernel far below the matrix-core rate.  Instead
// both operands are dequantized *in registers* to fp16 -- (code) * (scale) is exact in fp16 because
// a 4-bit code has at most 3 significant bits and a bf16 / e4m3 scale at most 8 -- and fed to
// v_mfma_f32_32x32x16_f16 with fp32 accumulation.  The result equals the fp32 dequantize-then-matmul
// definition up to fp32 summation order; no per-group post-scaling exists.
//
// Range: activation scales are renormalised per row and weight scales per column by powers of two
// (largest scale of a row / column moved into [2^11, 2^12)), so the fp16 products never overflow and
// only contributions 2^-25 below the largest of their row / column can underflow.  The shifts are
// undone exactly in the epilogue.
//
// Dequantization of one 32-bit word (8 codes, element e in bits [4e, 4e+4)):
//   (w & 0x000F000F) | 0x64006400 -> two fp16 values 1024 + u          (elements 0 and 4)
//   (w & 0x00F000F0) | 0x64006400 -> two fp16 values 1024 + 16 u       (elements 1 and 5)
//   same on w >> 8                                                     (elements 2, 6 and 3, 7)
// followed by a packed fp16 subtract of the bias (1032 / 1152 for offset-binary signed codes,
// 1024 for unsigned ones) and a packed multiply by the scale (or scale / 16).  Both operands use
// the same element-to-slot order, so the contraction pairs equal k.
//
// Tiling: workgroup = 4 waves (2 x 2), block tile 256 x 256, wave tile 128 x 128 = 4 x 4 MFMA tiles,
// 256 fp32 accumulators per lane.  Operand tiles are staged through a 3-deep LDS ring, one k-group
// per stage; global loads for group g+3 are issued before the math of group g.
#include "svdq_common.h"

using namespace svdq;

namespace {

constexpr int BM = 256, BN = 256;
constexpr int STAGES = 3;
constexpr int STAGE_A = 0, STAGE_B = 8192, STAGE_AS = 16384, STAGE_BS = 16384 + 2048;
constexpr int STAGE_BYTES = 16384 + 4096;  // 8 KB A codes, 8 KB B codes, 2 KB + 2 KB packed scales
constexpr int OUT_LD = 136;                // bf16 elements per row of the store-staging slab (128 + pad)
constexpr int ROWNORM_OFF = STAGES * STAGE_BYTES;  // fp32 [256] row de-normalisation factors
constexpr int ROWMAX_OFF = ROWNORM_OFF + 1024;     // u32 [256] scratch for the row maximum
constexpr int LDS_BYTES = ROWMAX_OFF + 1024;
constexpr int NORM_TARGET_EXP = 11;

struct GemmParams {
    const uint8_t *act;
    const uint16_t *ascales;
    const uint8_t *wgt;
    const _Float16 *wscales;
    const float *colnorm;
    const uint16_t *bias;
    const uint16_t *wcscales;
    const float *lora_act;
    const uint16_t *lora_up;
    uint16_t *out;
    int M_pad, N, K, M_out, N_out, R_up;
    float alpha;
    float lora_scales[8];
    int gelu;
};

__device__ inline half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ inline uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }

// (a & mask) | magic in one VALU instruction (the compiler otherwise emits an AND and an OR because
// VOP3 cannot carry 32-bit literals; here the constants live in registers)
__device__ inline uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) {
    uint32_t d;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(mask), "v"(magic));
    return d;
}

// 8 codes of one word -> 8 fp16 values (code - bias) * scale in slot order [0,4,1,5,2,6,3,7]
template <bool UNSIGNED>
__device__ inline half8_t dequant_word(uint32_t w, half2_t s, half2_t s16, uint32_t magic) {
    const half2_t off1 = UNSIGNED ? half2_t{(_Float16)1024.f, (_Float16)1024.f} : half2_t{(_Float16)1032.f, (_Float16)1032.f};
    const half2_t off16 = UNSIGNED ? half2_t{(_Float16)1024.f, (_Float16)1024.f} : half2_t{(_Float16)1152.f, (_Float16)1152.f};
    const uint32_t w8 = w >> 8;
    const half2_t t0 = as_half2(and_or(w, 0x000F000Fu, magic));
    const half2_t t1 = as_half2(and_or(w, 0x00F000F0u, magic));
    const half2_t t2 = as_half2(and_or(w8, 0x000F000Fu, magic));
    const half2_t t3 = as_half2(and_or(w8, 0x00F000F0u, magic));
    const half2_t a0 = (t0 - off1) * s;
    const half2_t a1 = (t1 - off16) * s16;
    const half2_t a2 = (t2 - off1) * s;
    const half2_t a3 = (t3 - off16) * s16;
    return half8_t{a0[0], a0[1], a1[0], a1[1], a2[0], a2[1], a3[0], a3[1]};
}

__device__ inline float gelu_tanh(float x) {
    // x * (0.5 + 0.5 * tanh(0.79788456 * (x + 0.044715 x^3)))   (epilogues.cuh:22-44)
    const float u = 0.79788456f * (x + 0.044715f * x * x * x);
    // tanh(u) = 1 - 2 / (exp(2u) + 1); exact enough in fp32 and safe for large |u|
    const float e = __expf(2.0f * u);
    const float t = 1.0f - 2.0f / (e + 1.0f);
    return x * (0.5f + 0.5f * t);
}

template <bool ACT_UNSIGNED>
__global__ void __launch_bounds__(256, 1) gemm_w4a4_int4_kernel(GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int r32 = lane & 31, h = lane >> 5;

    // ---- block coordinates: consecutive ids of one XCD (id % 8) walk down M inside a band of N
    const int mblocks = p.M_pad / BM, nblocks = (p.N + BN - 1) / BN;
    const int nwg = mblocks * nblocks;
    int id = blockIdx.x;
    {
        const int per_xcd = (nwg + 7) / 8;
        const int xcd = id % 8, slot = id / 8;
        const int lin = xcd * per_xcd + slot;
        // when nwg is not a multiple of 8 some (xcd, slot) pairs fall outside: fall back to identity
        id = (nwg % 8 == 0) ? lin : id;
    }
    const int bm = id % mblocks, bn = id / mblocks;
    const int m0 = bm * BM, n0 = bn * BN;
    const int kgroups = p.K / 64;
    const int ntiles_total = p.N / 32;

    float *rownorm = (float *)(lds + ROWNORM_OFF);
    uint32_t *rowmax = (uint32_t *)(lds + ROWMAX_OFF);

    // ---- prologue: largest activation scale of each of my 256 rows -> power-of-two renormalisation
    rowmax[tid] = 0;
    __syncthreads();
    {
        const int oct = tid & 31, gs = tid >> 5;
        uint32_t mx[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int g = gs; g < kgroups; g += 8) {
            const u32x4_t v = *(const u32x4_t *)(p.ascales + (size_t)g * p.M_pad + m0 + 8 * oct);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                mx[2 * j] = max(mx[2 * j], v[j] & 0x7FFFu);
                mx[2 * j + 1] = max(mx[2 * j + 1], (v[j] >> 16) & 0x7FFFu);
            }
        }
#pragma unroll
        for (int j = 0; j < 8; j++) atomicMax(&rowmax[8 * oct + j], mx[j]);
    }
    __syncthreads();
    int my_shift;  // thread tid owns row tid of the block when staging scales
    {
        const int ex = (int)(rowmax[tid] >> 7);  // biased bf16 exponent of the row maximum
        my_shift = ex == 0 ? 0 : NORM_TARGET_EXP - (ex - 127);
        rownorm[tid] = ldexpf(1.0f, -my_shift);
    }
    const bool col_ok = n0 + tid < p.N;

    // ---- staging helpers
    u32x4_t ld_a[2], ld_b[2];
    uint16_t ld_as;
    _Float16 ld_bs;
    const int ca = tid >> 6;
    const int mt0 = m0 / 32, nt0 = n0 / 32;
    auto issue_loads = [&](int g) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int t = ca + 4 * j;
            ld_a[j] = *(const u32x4_t *)(p.act + ((size_t)(mt0 + t) * kgroups + g) * TILE_BYTES + lane * 16);
            ld_b[j] = (nt0 + t < ntiles_total)
                          ? *(const u32x4_t *)(p.wgt + ((size_t)(nt0 + t) * kgroups + g) * TILE_BYTES + lane * 16)
                          : u32x4_t{0x88888888u, 0x88888888u, 0x88888888u, 0x88888888u};
        }
        ld_as = p.ascales[(size_t)g * p.M_pad + m0 + tid];
        ld_bs = col_ok ? p.wscales[(size_t)g * p.N + n0 + tid] : (_Float16)0.f;
    };
    auto store_stage = [&](int st) {
        uint8_t *base = lds + st * STAGE_BYTES;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int t = ca + 4 * j;
            *(u32x4_t *)(base + STAGE_A + t * TILE_BYTES + lane * 16) = ld_a[j];
            *(u32x4_t *)(base + STAGE_B + t * TILE_BYTES + lane * 16) = ld_b[j];
        }
        const _Float16 sa = (_Float16)ldexpf(bf16_bits_to_f32(ld_as), my_shift);
        const _Float16 sa16 = sa * (_Float16)0.0625f;
        const _Float16 sb16 = ld_bs * (_Float16)0.0625f;
        *(u32x2_t *)(base + STAGE_AS + tid * 8) = u32x2_t{as_u32(half2_t{sa, sa}), as_u32(half2_t{sa16, sa16})};
        *(u32x2_t *)(base + STAGE_BS + tid * 8) = u32x2_t{as_u32(half2_t{ld_bs, ld_bs}), as_u32(half2_t{sb16, sb16})};
    };

    float16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    // prologue: the first STAGES groups; all loads are issued before the first LDS store
    {
        u32x4_t pa[STAGES][2], pb[STAGES][2];
        uint16_t pas[STAGES];
        _Float16 pbs[STAGES];
#pragma unroll
        for (int s = 0; s < STAGES; s++) {
            if (s < kgroups) {
                issue_loads(s);
                pa[s][0] = ld_a[0]; pa[s][1] = ld_a[1]; pb[s][0] = ld_b[0]; pb[s][1] = ld_b[1];
                pas[s] = ld_as; pbs[s] = ld_bs;
            }
        }
#pragma unroll
        for (int s = 0; s < STAGES; s++) {
            if (s < kgroups) {
                ld_a[0] = pa[s][0]; ld_a[1] = pa[s][1]; ld_b[0] = pb[s][0]; ld_b[1] = pb[s][1];
                ld_as = pas[s]; ld_bs = pbs[s];
                store_stage(s);
            }
        }
    }
    __syncthreads();

    uint32_t magic = 0x64006400u;
    asm volatile("" : "+v"(magic));  // keep the constant in a vector register
    for (int g = 0; g < kgroups; g++) {
        const int st = g % STAGES;
        const bool more = g + STAGES < kgroups;
        if (more) issue_loads(g + STAGES);

        const uint8_t *base = lds + st * STAGE_BYTES;
        u32x4_t araw[4], braw[4];
        u32x2_t asc[4], bsc[4];
#pragma unroll
        for (int t = 0; t < 4; t++) {
            araw[t] = *(const u32x4_t *)(base + STAGE_A + (wm * 4 + t) * TILE_BYTES + r32 * 32 + h * 16);
            braw[t] = *(const u32x4_t *)(base + STAGE_B + (wn * 4 + t) * TILE_BYTES + r32 * 32 + h * 16);
            asc[t] = *(const u32x2_t *)(base + STAGE_AS + (wm * 128 + t * 32 + r32) * 8);
            bsc[t] = *(const u32x2_t *)(base + STAGE_BS + (wn * 128 + t * 32 + r32) * 8);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            half8_t a[4], b[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                a[t] = dequant_word<ACT_UNSIGNED>(araw[t][i], as_half2(asc[t][0]), as_half2(asc[t][1]), magic);
                b[t] = dequant_word<false>(braw[t][i], as_half2(bsc[t][0]), as_half2(bsc[t][1]), magic);
            }
#pragma unroll
            for (int mt = 0; mt < 4; mt++)
#pragma unroll
                for (int nt = 0; nt < 4; nt++)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mt], b[nt], acc[mt][nt], 0, 0, 0);
        }
        __syncthreads();
        if (more) store_stage(st);
    }
    __syncthreads();

    // ---- epilogue, one 32-row slab (mt) of the wave tile at a time ------------------------------
    // accumulator element e of tile (mt, nt): row 8*(e/4) + 4*h + e%4, column r32 of the tile
    const int wrow0 = m0 + wm * 128, wcol0 = n0 + wn * 128;
    float colf[4], biasf[4];
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
        const int n = wcol0 + nt * 32 + r32;
        const bool ok = n < p.N;
        float cf = ok ? p.colnorm[n] * p.alpha : 0.f;
        if (ok && p.wcscales) cf *= bf16_bits_to_f32(p.wcscales[n]);
        colf[nt] = cf;
        biasf[nt] = (ok && p.bias) ? bf16_bits_to_f32(p.bias[n]) : 0.f;
    }
    uint16_t *slab = (uint16_t *)(lds + wave * (32 * OUT_LD * 2));
    const int nsteps = p.R_up / 16;
#pragma unroll
    for (int mt = 0; mt < 4; mt++) {
        // undo the power-of-two normalisation; per-channel scale and bias (EpilogueBias, gemm_base.cuh:710-781)
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const float rn = rownorm[wm * 128 + mt * 32 + 8 * (e / 4) + 4 * h + (e % 4)];
#pragma unroll
            for (int nt = 0; nt < 4; nt++) acc[mt][nt][e] = acc[mt][nt][e] * rn * colf[nt] + biasf[nt];
        }
        // low-rank up projection: acc += bf16(lora_act * scale) @ up^T   (lora.cuh:110-241)
        for (int s = 0; s < nsteps; s++) {
            const float ls = p.lora_scales[s < 8 ? s : 7];
            const float4_t *ap = (const float4_t *)(p.lora_act + (size_t)(wrow0 + mt * 32 + r32) * p.R_up + 16 * s + 8 * h);
            const float4_t v0 = ap[0], v1 = ap[1];
            u32x4_t w;
            w[0] = f32_to_bf16_bits(v0[0] * ls) | (f32_to_bf16_bits(v0[1] * ls) << 16);
            w[1] = f32_to_bf16_bits(v0[2] * ls) | (f32_to_bf16_bits(v0[3] * ls) << 16);
            w[2] = f32_to_bf16_bits(v1[0] * ls) | (f32_to_bf16_bits(v1[1] * ls) << 16);
            w[3] = f32_to_bf16_bits(v1[2] * ls) | (f32_to_bf16_bits(v1[3] * ls) << 16);
            const bf16x8_t la = __builtin_bit_cast(bf16x8_t, w);
#pragma unroll
            for (int nt = 0; nt < 4; nt++) {
                const int n = wcol0 + nt * 32 + r32;
                const u32x4_t bw = n < p.N ? *(const u32x4_t *)(p.lora_up + (size_t)n * p.R_up + 16 * s + 8 * h) : u32x4_t{0, 0, 0, 0};
                acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(la, __builtin_bit_cast(bf16x8_t, bw), acc[mt][nt], 0, 0, 0);
            }
        }
        if (p.gelu) {
#pragma unroll
            for (int nt = 0; nt < 4; nt++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[mt][nt][e] = gelu_tanh(acc[mt][nt][e]);
        }
        // bf16 tile -> per-wave LDS slab (32 rows x 128 columns) -> 16-byte row-contiguous global stores
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
#pragma unroll
            for (int e = 0; e < 16; e++)
                slab[(8 * (e / 4) + 4 * h + (e % 4)) * OUT_LD + nt * 32 + r32] = (uint16_t)f32_to_bf16_bits(acc[mt][nt][e]);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (p.out) {
#pragma unroll
            for (int pass = 0; pass < 8; pass++) {
                const int rr = pass * 4 + (lane >> 4), cc = (lane & 15) * 8;
                const int m = wrow0 + mt * 32 + rr, n = wcol0 + cc;
                if (m < p.M_out && n < p.N_out) *(u32x4_t *)(p.out + (size_t)m * p.N_out + n) = *(const u32x4_t *)(slab + rr * OUT_LD + cc);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}

}  // namespace

extern "C" int svdq_gemm_w4a4(const svdq_gemm_args *a, void *stream) {
    SVDQ_REQUIRE(a, "gemm: null args");
    SVDQ_REQUIRE(a->act && a->ascales && a->wgt && a->wscales && a->colnorm, "gemm: act/ascales/wgt/wscales/colnorm must not be null");
    SVDQ_REQUIRE(a->M_pad > 0 && a->M_pad % 256 == 0, "gemm: M_pad (%lld) must be a positive multiple of 256", (long long)a->M_pad);
    SVDQ_REQUIRE(a->N > 0 && a->N % 128 == 0, "gemm: N (%lld) must be a positive multiple of 128", (long long)a->N);
    SVDQ_REQUIRE(a->K > 0 && a->K % 128 == 0, "gemm: K (%lld) must be a positive multiple of 128", (long long)a->K);
    SVDQ_REQUIRE(a->out || a->qout, "gemm: one of out / qout must be given");
    SVDQ_REQUIRE((a->lora_up != nullptr) == (a->lora_act_in != nullptr), "gemm: lora_up and lora_act_in go together");
    SVDQ_REQUIRE(a->R_up >= 0 && a->R_up % 16 == 0 && a->R_up <= 128, "gemm: R_up (%lld) must be a multiple of 16, at most 128", (long long)a->R_up);
    SVDQ_REQUIRE((a->R_up > 0) == (a->lora_up != nullptr), "gemm: R_up and lora_up disagree");
    if (a->out) {
        SVDQ_REQUIRE(a->M_out > 0 && a->M_out <= a->M_pad && a->M_pad - a->M_out < 256, "gemm: M_out (%lld) does not fit M_pad (%lld)",
                     (long long)a->M_out, (long long)a->M_pad);
        SVDQ_REQUIRE(a->N_out > 0 && a->N_out <= a->N && a->N - a->N_out < 128 && a->N_out % 8 == 0,
                     "gemm: N_out (%lld) must be a multiple of 8 within 128 of N (%lld)", (long long)a->N_out, (long long)a->N);
    }
    SVDQ_REQUIRE(((uintptr_t)a->act | (uintptr_t)a->wgt | (uintptr_t)a->ascales | (uintptr_t)a->out | (uintptr_t)a->lora_act_in |
                  (uintptr_t)a->lora_up) % 16 == 0, "gemm: pointers must be 16-byte aligned");
    SVDQ_REQUIRE(a->M_pad * a->N < (1ll << 40) && a->K < (1 << 24), "gemm: shape too large");
    if (a->fuse_silu) return fail(SVDQ_EUNSUPPORTED, "gemm: fuse_silu is not implemented");
    if (a->fp4) return fail(SVDQ_EUNSUPPORTED, "gemm: NVFP4 operands are not implemented yet");
    if (a->qout) return fail(SVDQ_EUNSUPPORTED, "gemm: next-layer quantization epilogue is not implemented yet");

    GemmParams p;
    p.act = (const uint8_t *)a->act;
    p.ascales = (const uint16_t *)a->ascales;
    p.wgt = (const uint8_t *)a->wgt;
    p.wscales = (const _Float16 *)a->wscales;
    p.colnorm = a->colnorm;
    p.bias = (const uint16_t *)a->bias;
    p.wcscales = (const uint16_t *)a->wcscales;
    p.lora_act = a->lora_act_in;
    p.lora_up = (const uint16_t *)a->lora_up;
    p.out = (uint16_t *)a->out;
    p.M_pad = (int)a->M_pad; p.N = (int)a->N; p.K = (int)a->K;
    p.M_out = (int)a->M_out; p.N_out = (int)a->N_out; p.R_up = (int)a->R_up;
    p.alpha = a->alpha;
    for (int i = 0; i < 8; i++) p.lora_scales[i] = (a->lora_scales && i < (a->R_up + 15) / 16) ? a->lora_scales[i] : 1.0f;
    p.gelu = 0;

    const int nwg = (int)(a->M_pad / BM) * (int)((a->N + BN - 1) / BN);
    auto kern = a->act_unsigned ? gemm_w4a4_int4_kernel<true> : gemm_w4a4_int4_kernel<false>;
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if (e != hipSuccess) return fail(SVDQ_ELAUNCH, "gemm: cannot reserve %d bytes of LDS: %s", LDS_BYTES, hipGetErrorString(e));
    hipLaunchKernelGGL(kern, dim3(nwg), dim3(256), LDS_BYTES, (hipStream_t)stream, p);
    return check_launch("gemm_w4a4");
}
