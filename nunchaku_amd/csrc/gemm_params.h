// Kernel argument block and tile constants of the W4A4 GEMM, shared by the host entry point
// (gemm.hip) and the per-variant kernel translation units (gemm_variant.hip).
#pragma once

#include "svdq_common.h"

namespace svdq {


constexpr int BM = 256, BN = 256;
constexpr int STAGES = 4;
// per stage: 8 KB A codes, 8 KB B codes, then 16 bytes of packed fp16 scale pairs per row / column:
// INT4 {16s,16s} {-24s,-24s} (8 bytes used; -16s for unsigned codes); NVFP4 one {s,s} pair for each
// of the four 16-groups
constexpr int STAGE_A = 0, STAGE_B = 8192, STAGE_AS = 16384, STAGE_BS = 16384 + 4096;
constexpr int STAGE_BYTES = 16384 + 8192;
constexpr int OUT_LD = 136;                // bf16 elements per row of the store-staging slab (128 + pad)
constexpr int MAX_BATCH = 8;                       // tiles whose row shifts are tabulated at once
constexpr int SLAB_OFF = STAGES * STAGE_BYTES;     // 4 waves x (32 rows x OUT_LD bf16): epilogue staging
constexpr int SHIFT_OFF = SLAB_OFF + 4 * 32 * OUT_LD * 2;  // int [MAX_BATCH][256] row renormalisation shifts
constexpr int TAB_OFF = SHIFT_OFF + MAX_BATCH * 256 * 4;   // 4 waves x float [2][128]: column factors and biases
constexpr int FLAG_OFF = TAB_OFF + 4 * 1024;               // one word: a thread's reading of an arrival counter, for all
constexpr int NORMW_OFF = FLAG_OFF + 16;                   // 4 waves x float [128]: RMS-norm weights of the wave's head
constexpr int LDS_BYTES = NORMW_OFF + 4 * 512;
constexpr int NORM_TARGET_EXP = 10;


struct GemmParams {
    long long *stamps;  // debug builds only: per-workgroup phase timestamps
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
    // next-layer fusion
    uint8_t *qout;               // native activation tiles [M_pad, N/2]
    void *oscales;               // bf16 [N/64, M_pad] or fp8 [N/16, M_pad]
    const float *next_smooth_rcp;  // fp32 [N]
    const bf16x8_t *next_down;   // native proj_down of the next layer ([N, R_down])
    float *next_lora_out;        // fp32 [M_pad, R_down], zeroed before the launch, accumulated atomically
    // tiles shared by two workgroups: parked partial sums (fp32 [2 * workgroups][256 threads][64] x 4)
    // and one arrival counter per tile (zero between launches)
    float *partials;
    int *counters;
    int M_pad, N, K, M_out, N_out, R_up, R_down;
    float alpha;
    float lora_scales[8];
    int gelu;
    int silu;  // x * sigmoid(x) before the store (next-layer variants only)
    // RMS norm + rotary embedding on the q and k heads of a fused QKV projection (next-layer variants only)
    const uint16_t *norm_q, *norm_k;  // bf16 [128]
    const float *rotary;              // fp32 [rot_rows/32][16][64 lanes][4], see svdq_gemm_args; null: no such epilogue
    int rot_rows, rope_cols;          // rope_cols = 2 N / 3: the columns of q and k
    float norm_eps;
};


}  // namespace svdq
