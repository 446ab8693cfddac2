// Kernel argument block and tile constants of the W4A4 GEMM, shared by the host entry point
// (gemm.hip) and the per-variant kernel translation units (gemm_variant.hip).
#pragma once

#include "svdq_common.h"

namespace svdq {


// ranks of the low-rank branch: multiples of 16 up to this (the reference: MAX_RANK = 1024, lora.cuh:22)
constexpr int MAX_RANK = 1024;

constexpr int BM = 256, BN = 256;
// NVFP4 kernel: the operands of one k-group (64 wide) as fp16, dequantized once per workgroup: per operand
// [8 tiles of 32 rows][4 steps of 16 k][2 halves of 8 k][32 rows] x 16 bytes = 32 KB (a wave's fetch of one matrix
// instruction's operand is 1 KB contiguous), activations then weights; two such buffers alternate.
constexpr int OP_BYTES = 8 * 4 * 2 * 32 * 16;    // one operand of one k-group
constexpr int OPBUF_BYTES = 2 * OP_BYTES;          // activations + weights
constexpr int OUT_LD = 136;                // bf16 elements per row of the store-staging slab (128 + pad)
constexpr int MAX_BATCH = 8;                       // tiles whose row shifts are tabulated at once
constexpr int SLAB_OFF = 0;                        // 4 waves x (32 rows x OUT_LD bf16): epilogue staging, in the operand buffers' place
static_assert(4 * 32 * OUT_LD * 2 <= 2 * OPBUF_BYTES, "the epilogue's slabs reuse the operand buffers");
constexpr int SHIFT_OFF = 2 * OPBUF_BYTES;                 // int [MAX_BATCH][256] row renormalisation shifts
constexpr int TAB_OFF = SHIFT_OFF + MAX_BATCH * 256 * 4;   // 4 waves x float [2][128]: column factors and biases
constexpr int FLAG_OFF = TAB_OFF + 4 * 1024;               // one word: a thread's reading of an arrival counter, for all
constexpr int NORMW_OFF = FLAG_OFF + 16;                   // 4 waves x float [128]: RMS-norm weights of the wave's head
constexpr int LDS_BYTES = NORMW_OFF + 4 * 512;
static_assert(LDS_BYTES <= 160 * 1024, "one workgroup per compute unit");
constexpr int NORM_TARGET_EXP = 10;


// Separate q / k / v outputs of a fused QKV projection (EpiloguePackQKV, epilogues.cuh:427-550): fp16
// [heads][rows][128] each, head h at h * head_stride elements.  Rows [attn_tokens, rows) are written with
// the mask value of the tensor: 0 for q and v, NaN for k.
struct QkvOut {
    uint16_t *q, *k, *v;      // null: the epilogue is not composed
    long long stride_q, stride_k, stride_v;
    int attn_tokens, rows;
};

// One wave writes a 32-row x 128-column bf16 slab (one head of q, k or v; rows `ld` elements apart in LDS)
// to the tensor its columns belong to.  Values go bf16 -> fp32 -> fp16 as the reference's convert_half2
// does (epilogues.cuh:446-453); 16 bytes per lane and pass, rows contiguous within a head.
__device__ inline void store_qkv_slab(const QkvOut &o, const uint16_t *slab, int ld, int lane, int row0, int col0, int third) {
    const int which = col0 / third, head = (col0 - which * third) >> 7;
    uint16_t *base = which == 0 ? o.q : (which == 1 ? o.k : o.v);
    const long long stride = which == 0 ? o.stride_q : (which == 1 ? o.stride_k : o.stride_v);
    const uint32_t maskw = which == 1 ? 0x7FFF7FFFu : 0u;  // fp16 NaN pairs for k (epilogues.cuh:543), zeros for q and v
    base += (size_t)head * stride;
#pragma unroll
    for (int pass = 0; pass < 8; pass++) {
        const int rr = pass * 4 + (lane >> 4), cc = (lane & 15) * 8, m = row0 + rr;
        const u32x4_t w = *(const u32x4_t *)(slab + rr * ld + cc);
        u32x4_t d;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const _Float16 lo = (_Float16)bits_f32(w[j] << 16), hi = (_Float16)bits_f32(w[j] & 0xFFFF0000u);
            d[j] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
            if (m >= o.attn_tokens) d[j] = maskw;
        }
        if (m < o.rows) __builtin_nontemporal_store(d, (u32x4_t *)(base + (size_t)m * 128 + cc));
    }
}

// Linear attention (EpilogueLiteLA::apply_litela, epilogues.cuh:572-655).  A wave's 128 output columns are two heads
// of [k 32 | v 32].  vk[i][j] = sum over rows of v[row][i] * relu(k[row][j]) on the matrix cores (the rows are the
// contraction index: both operands are read down the columns of the 32-row bf16 slab in LDS, rows `ld` elements
// apart), row 32 = sum of relu(k[row][j]).  In the INT4 kernel a wave keeps the sums of its slabs in registers
// (VkSums), the two waves of a column half meet in LDS, and the workgroup's row block goes to its own slot of the
// workspace ([row block][head] x 1056 floats, the 32 x 32 part in the lanes' order: a wave's store is 1 KB contiguous);
// the NVFP4 kernel parks every 32-row slab.  A small kernel behind the GEMM adds the row blocks of a batch entry in
// ascending order (reduce_vk_kernel in gemm.hip).
// The reference adds with atomics in the order of arrival (epilogues.cuh:649); atomics here, 2.4 M of them at 4096
// rows and 72 heads, doubled the kernel's time.
constexpr int VK_HEAD_FLOATS = 33 * 32;
struct VkSums {
    float16_t d[2];  // per head: vk[i][j], element e of lane l is i = 8 (e / 4) + 4 (l / 32) + e % 4, j = l % 32
    float ks[2];     // per head: this lane's part of the column sum of relu(k) for j = l % 32
};
__device__ inline void litela_clear(VkSums &s) {
#pragma unroll
    for (int hd = 0; hd < 2; hd++) {
#pragma unroll
        for (int e = 0; e < 16; e++) s.d[hd][e] = 0.f;
        s.ks[hd] = 0.f;
    }
}
__device__ inline void litela_add_slab(VkSums &s, const uint16_t *slab, int ld, int lane) {
    const int j = lane & 31, kb = lane >> 5;
#pragma unroll
    for (int hd = 0; hd < 2; hd++) {
#pragma unroll
        for (int st = 0; st < 2; st++) {
            u32x4_t kw, vw;
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                uint32_t kk[2], vv[2];
#pragma unroll
                for (int f = 0; f < 2; f++) {
                    const uint16_t *rowp = slab + (16 * st + 8 * kb + e + f) * ld + hd * 64 + j;
                    kk[f] = rowp[0];
                    vv[f] = rowp[32];
                    if (kk[f] & 0x8000u) kk[f] = 0;  // ReLU on the bf16 value
                    s.ks[hd] += bits_f32(kk[f] << 16);
                }
                kw[e / 2] = kk[0] | (kk[1] << 16);
                vw[e / 2] = vv[0] | (vv[1] << 16);
            }
            s.d[hd] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vw), __builtin_bit_cast(bf16x8_t, kw), s.d[hd], 0, 0, 0);
        }
    }
}
// Writes the wave's two heads to dst (2 x 1056 floats, LDS or the workspace).
template <bool STREAM>
__device__ inline void litela_park(const VkSums &s, float *dst, int lane) {
    const int j = lane & 31, kb = lane >> 5;
#pragma unroll
    for (int hd = 0; hd < 2; hd++) {
        const float ks = s.ks[hd] + __shfl_xor(s.ks[hd], 32);
        float *d = dst + hd * VK_HEAD_FLOATS;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const float4_t v = float4_t{s.d[hd][4 * g], s.d[hd][4 * g + 1], s.d[hd][4 * g + 2], s.d[hd][4 * g + 3]};
            if (STREAM) __builtin_nontemporal_store(v, (float4_t *)(d + (g * 64 + lane) * 4));
            else *(float4_t *)(d + (g * 64 + lane) * 4) = v;
        }
        if (kb == 0) d[1024 + j] = ks;
    }
}
// s = s + what another wave parked at src (the rows of s come first).
__device__ inline void litela_add_parked(VkSums &s, const float *src, int lane) {
    const int j = lane & 31, kb = lane >> 5;
#pragma unroll
    for (int hd = 0; hd < 2; hd++) {
        const float ks = s.ks[hd] + __shfl_xor(s.ks[hd], 32);
        const float *d = src + hd * VK_HEAD_FLOATS;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const float4_t v = *(const float4_t *)(d + (g * 64 + lane) * 4);
#pragma unroll
            for (int i = 0; i < 4; i++) s.d[hd][4 * g + i] += v[i];
        }
        s.ks[hd] = kb == 0 ? ks + d[1024 + j] : 0.f;
    }
}
// After the last slab of a tile, called by all four waves (2 x 2, wave = 2 wm + wn) when the tile holds k | v columns
// (a condition uniform over the workgroup): the lower waves hand their sums to the upper ones through their own slab
// areas, which they no longer need, and the upper ones store the row block's share.  `kv`: this wave's columns are k | v.
__device__ inline void litela_finish(VkSums &s, bool kv, int wm, int wn, unsigned char *slabs, int slab_bytes, float *share, int lane) {
    if (kv && wm == 1) litela_park<false>(s, (float *)(slabs + (2 + wn) * slab_bytes), lane);
    __syncthreads();
    if (kv && wm == 0) {
        litela_add_parked(s, (const float *)(slabs + (2 + wn) * slab_bytes), lane);
        litela_park<true>(s, share, lane);
    }
}

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
    // next-layer fusion
    uint8_t *qout;               // native activation tiles [M_pad, N/2]
    void *oscales;               // bf16 [N/64, M_pad] or fp8 [N/16, M_pad]
    const float *next_smooth_rcp;  // fp32 [N]
    const bf16x8_t *next_down;   // native proj_down of the next layer ([N, R_down])
    float *next_lora_out;        // fp32 [M_pad, R_down], written by the kernel that adds the shares behind the GEMM
    // tiles shared by two workgroups: parked partial sums (fp32 [2 * workgroups][256 threads][64] x 4)
    // and one arrival counter per tile (zero between launches)
    float *partials;
    int *counters;
    int M_pad, N, K, M_out, N_out, R_up, R_down;
    float alpha;
    float lora_scales[MAX_RANK / 16];
    int gelu;
    int silu;  // x * sigmoid(x) before the store (next-layer variants only)
    // RMS norm + rotary embedding on the q and k heads of a fused QKV projection (next-layer variants only)
    const uint16_t *norm_q, *norm_k;  // bf16 [128]
    const float *rotary;              // fp32 [rot_rows/32][16][64 lanes][4], see svdq_gemm_args; null: no such epilogue
    int rot_rows, rope_cols;          // rope_cols = 2 N / 3: the columns of q and k
    float norm_eps;
    QkvOut qkv;
    // linear attention (see g6::Params) and the parked shares of the next layer's low-rank projection
    float *vk, *vk_part;
    int vk_rows;
    int whole_band;              // 0, or (whole tiles only) the band height of the tile numbering in row blocks
    float *next_lora_part;  // [N/128 column chunks][M_pad/32 slabs][R_down/16][2][64 lanes] x float4
};


// ---- INT4 GEMM on the fp6 matrix instruction (gemm6_kernel.h) -------------------------------------
namespace g6 {
constexpr int BM = 128, BN = 256;  // workgroup tile; 4 waves as 2 x 2, wave tile 64 x 128
// One stage of the LDS ring holds one k-group of the workgroup's operands:
//   4 activation fragments | 8 weight fragments | weight scales 256 x {64 s, 0, 0, 0} bf16 |
//   activation scales 128 x bf16 | zeros (what the upper half-wave reads as its activation scale)
constexpr int ST_A = 0, ST_W = 4 * FRAG_BYTES, ST_WS = ST_W + 8 * FRAG_BYTES, ST_AS = ST_WS + 256 * 8, ST_Z = ST_AS + 256;
constexpr int STAGE_BYTES = ST_Z + 128;
constexpr int STAGES = 3;
constexpr int COPIES_PER_WAVE = 6;  // asynchronous copies every wave issues per k-group
// epilogue (reuses the ring): per wave one 32-row slab of bf16, then the column tables
constexpr int OUT_LD = 136;
constexpr int SLAB_BYTES = 32 * OUT_LD * 2;
constexpr int EP_TAB = 4 * SLAB_BYTES;     // float cf[256], bias[256]
constexpr int EP_NORMW = EP_TAB + 2048;    // 4 waves x float [128]: RMS-norm weights of the wave's head
constexpr int EP_FLAG = EP_NORMW + 2048;   // one word handed from thread 0 to the workgroup
constexpr int EP_RED = EP_FLAG + 16;       // [2 rank tiles][2 row halves][2][64 lanes] x float4: the two column halves' low-rank sums meet here
constexpr int EP_RED_BYTES = 2 * 2 * 2 * 64 * 16;  // two rank tiles at a time
constexpr int EP_DOWN = EP_RED + EP_RED_BYTES;  // the next layer's proj_down for the tile's 256 columns, up to 2 rank tiles
constexpr int EP_END = EP_DOWN + 16384;
constexpr int LDS_BYTES = STAGES * STAGE_BYTES > EP_END ? STAGES * STAGE_BYTES : EP_END;
static_assert(2 * LDS_BYTES <= 160 * 1024, "two workgroups share a compute unit's LDS");

struct Params {
    const uint8_t *act;        // fragments [M_pad/128][K/64][4]
    const uint16_t *ascales;   // bf16 [K/64][M_pad]
    const uint8_t *wgt;        // fragments [ceil(N/256)][K/64][8]
    const uint8_t *wscales;    // [ceil(N/256)][K/64][256] x {bf16 64 * scale, 0, 0, 0}
    const uint16_t *bias;      // bf16 [N] or null
    const uint16_t *wcscales;  // bf16 [N] or null
    const float *lora_act;     // fp32 [M_pad][R_up]
    const uint16_t *lora_up;   // bf16 [N][R_up]
    uint16_t *out;             // bf16 [M_out][N_out] or null
    // next-layer fusion
    uint8_t *qout;                 // fragments [M_pad/128][N/64][4] of the next layer's activations
    uint16_t *oscales;             // bf16 [N/64][M_pad]
    const float *next_smooth_rcp;  // fp32 [N]
    const bf16x8_t *next_down;     // native proj_down of the next layer
    float *next_lora_out;          // fp32 [M_pad][R_down]
    float *next_lora_part;         // [N/256 column blocks][M_pad/128][128 x R_down] partial projections, in the lanes' order
    // tiles split along K: parked partial sums and one arrival counter per tile (zero between launches)
    float *partials;
    int *counters;
    int band;          // row blocks per band of the tile numbering
    int kparts;
    int M_pad, N, K, M_out, N_out, R_up, R_down;
    float alpha;
    float lora_scales[MAX_RANK / 16];
    int gelu, silu;
    const uint16_t *norm_q, *norm_k;
    const float *rotary;
    int rot_rows, rope_cols;
    float norm_eps;
    QkvOut qkv;
    // linear attention (EpilogueLiteLA, epilogues.cuh:552-681; next-layer variant only): columns [0, N/3) are q,
    // stored through `out` after a ReLU; the rest is [head][k 32 | v 32]; vk[batch][head][i][j] += sum over the
    // tile's rows of v[i] relu(k[j]) (i < 32) and of relu(k[j]) (i = 32)
    float *vk;           // fp32 [batch][2 N / 3 / 64][33][32]; null: no such epilogue
    float *vk_part;      // workspace: [M_pad / 128 row blocks][heads] x 1056 floats, every row block's sums
    int vk_rows;         // rows per batch entry, a multiple of 256
};
}  // namespace g6

}  // namespace svdq
