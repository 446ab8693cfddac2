// Second half of the linear attention the W4A4 GEMM's EpilogueLiteLA feeds: every token's relu(q) of a head times
// the head's [33][32] sums, normalised by the last row.  Counterpart of EpilogueLiteLA::vk_mul_q_kernel
// (src/kernels/zgemm/epilogues.cuh:683-744), launched by linearattn_vk_mul_q
// (gemm_w4a4_launch_impl.cuh:427-448).
//
// out[token][i] = sum_k vk[i][k] q[token][k] is a [32 x 32] x [32 x tokens] product per head, which the reference
// computes in fp32 (:719-729).  Here: v_mfma_f32_32x32x16_bf16 with tokens as columns.  q is bf16 already; every fp32
// element of vk is split into three bf16 terms that add up to it exactly (8 + 8 + 8 significant bits, by truncation),
// so the three products per element are exact and only the fp32 accumulation rounds, as it does in the reference.  The
// split operands stay in registers for all the tokens a wave sees.  Which k a lane contracts and which output a row of
// the left operand stands for are free choices: lane half h takes k = 16 h ... 16 h + 15, and row r = 8 g + 4 h' + e
// stands for output 16 h' + 4 g + e, so that a lane's two 16-byte requests for its token's q are the right operands as
// they come, and it ends up with 16 contiguous outputs (two 16-byte stores).  The denominator, row 32 of the sums, is
// 16 multiply-adds per lane and one exchange between the lane halves.  A workgroup is four consecutive heads (one per
// wave) over the same tokens: together the waves use whole lines of q.  Bound by the q traffic, 128 bytes per
// (token, head).
#include "svdq_common.h"

using namespace svdq;

namespace {

constexpr int HEAD_DIM = 32;
constexpr int TOKENS_PER_WG = 64, BLOCKS = TOKENS_PER_WG / 32;

__global__ void __launch_bounds__(256) vk_mul_q_kernel(uint16_t *q, const float *vk, float eps, int num_tokens, int tokens_pad, int heads) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int head = blockIdx.y * 4 + wave, batch = blockIdx.z;
    if (head >= heads) return;  // (no barrier in this kernel)
    const int col = lane & 31, h = lane >> 5;
    const int t0 = blockIdx.x * TOKENS_PER_WG;
    // all of the wave's q first: one round of memory latency
    u32x4_t w[BLOCKS][2];
    uint16_t *rowp[BLOCKS];
#pragma unroll
    for (int blk = 0; blk < BLOCKS; blk++) {
        int token = t0 + blk * 32 + col;
        token = token < tokens_pad ? token : tokens_pad - 1;  // (results of such lanes are not stored)
        rowp[blk] = q + (((size_t)batch * tokens_pad + token) * heads + head) * HEAD_DIM + 16 * h;
#pragma unroll
        for (int i = 0; i < 2; i++) w[blk][i] = *(const u32x4_t *)(rowp[blk] + 8 * i);
    }
    const float *hvk = vk + ((size_t)batch * heads + head) * (HEAD_DIM + 1) * HEAD_DIM;
    // left operand: vk[output of row lane % 32][k = 16 h + 8 t ... + 7] for t = 0, 1, in three bf16 terms; the same k
    // of row 32 for the denominator
    const int out_row = 16 * ((col >> 2) & 1) + 4 * (col >> 3) + (col & 3);
    float dn[16];
    bf16x8_t a[3][2];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float4_t av = *(const float4_t *)(hvk + out_row * HEAD_DIM + 16 * h + 4 * i);
        const float4_t dv = *(const float4_t *)(hvk + HEAD_DIM * HEAD_DIM + 16 * h + 4 * i);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            dn[4 * i + j] = dv[j];
            const float x = av[j];
            const uint32_t hi = f32_bits(x) & 0xFFFF0000u;
            const float r1 = x - bits_f32(hi);  // exact: at most 16 significant bits are left
            const uint32_t mid = f32_bits(r1) & 0xFFFF0000u;
            const float r2 = r1 - bits_f32(mid);  // exact: at most 8 significant bits, a bf16 value
            const int t = i >> 1, e = 4 * (i & 1) + j;
            a[0][t][e] = __builtin_bit_cast(__bf16, (uint16_t)(hi >> 16));
            a[1][t][e] = __builtin_bit_cast(__bf16, (uint16_t)(mid >> 16));
            a[2][t][e] = __builtin_bit_cast(__bf16, (uint16_t)(f32_bits(r2) >> 16));
        }
    }
#pragma unroll
    for (int blk = 0; blk < BLOCKS; blk++) {
        if (t0 + blk * 32 >= num_tokens) break;
        float16_t d;
#pragma unroll
        for (int e = 0; e < 16; e++) d[e] = 0.f;
        float den = 0.f;
#pragma unroll
        for (int s = 0; s < 16; s++) {
            const uint32_t word = w[blk][s >> 3][(s >> 1) & 3];
            den = __builtin_fmaf(bits_f32((s & 1) ? word & 0xFFFF0000u : word << 16), dn[s], den);
        }
        // the smallest terms first
#pragma unroll
        for (int term = 2; term >= 0; term--)
#pragma unroll
            for (int t = 0; t < 2; t++) d = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[term][t], __builtin_bit_cast(bf16x8_t, w[blk][t]), d, 0, 0, 0);
        den += __shfl_xor(den, 32);
        const float rden = 1.0f / (den + eps);
        if (t0 + blk * 32 + col < num_tokens) {
            // element 4 g + e of the result is row 8 g + 4 h + e of the product: output 16 h + 4 g + e of this lane's token
#pragma unroll
            for (int i = 0; i < 2; i++) {
                u32x4_t o;
#pragma unroll
                for (int j = 0; j < 4; j++) o[j] = pack_bf16x2(d[8 * i + 2 * j] * rden, d[8 * i + 2 * j + 1] * rden);
                *(u32x4_t *)(rowp[blk] + 8 * i) = o;
            }
        }
    }
}

}  // namespace

extern "C" int svdq_linearattn_vk_mul_q(void *q, const float *vk, int64_t batch, int64_t num_tokens, int64_t tokens_pad, int64_t heads,
                                        float eps, void *stream) {
    SVDQ_REQUIRE(q && vk, "vk_mul_q: q and vk must not be null");
    SVDQ_REQUIRE(batch > 0 && batch < 65536 && heads > 0 && heads < 65536, "vk_mul_q: batch (%lld) and heads (%lld) must be in 1..65535",
                 (long long)batch, (long long)heads);
    SVDQ_REQUIRE(num_tokens > 0 && num_tokens <= tokens_pad && tokens_pad < (1ll << 31), "vk_mul_q: num_tokens (%lld) must be in 1..tokens_pad (%lld)",
                 (long long)num_tokens, (long long)tokens_pad);
    SVDQ_REQUIRE((uintptr_t)q % 16 == 0 && (uintptr_t)vk % 16 == 0, "vk_mul_q: pointers must be 16-byte aligned");
    SVDQ_LAUNCH(vk_mul_q_kernel, dim3((unsigned)((num_tokens + TOKENS_PER_WG - 1) / TOKENS_PER_WG), (unsigned)((heads + 3) / 4), (unsigned)batch), dim3(256), 0, (hipStream_t)stream,
                       (uint16_t *)q, vk, eps, (int)num_tokens, (int)tokens_pad, (int)heads);
    return check_launch("linearattn_vk_mul_q");
}
