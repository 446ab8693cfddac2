// Second half of the linear attention the W4A4 GEMM's EpilogueLiteLA feeds: every token's relu(q) of a head times
// the head's [33][32] sums, normalised by the last row.  Counterpart of EpilogueLiteLA::vk_mul_q_kernel
// (src/kernels/zgemm/epilogues.cuh:683-744), launched by linearattn_vk_mul_q
// (gemm_w4a4_launch_impl.cuh:427-448).
//
// One thread per (token, head): 64 bytes of q in, 64 bytes out, in place; the head's sums are read by all
// threads of the workgroup at the same addresses (scalar-like broadcast reads from LDS).  Bound by the q
// traffic: 128 bytes per (token, head).
#include "svdq_common.h"

using namespace svdq;

namespace {

constexpr int HEAD_DIM = 32;

__global__ void __launch_bounds__(256) vk_mul_q_kernel(uint16_t *q, const float *vk, float eps, int num_tokens, int tokens_pad, int heads) {
    __shared__ float svk[(HEAD_DIM + 1) * HEAD_DIM];
    const int head = blockIdx.y, batch = blockIdx.z;
    const float *hvk = vk + ((size_t)batch * heads + head) * (HEAD_DIM + 1) * HEAD_DIM;
    for (int i = threadIdx.x; i < (HEAD_DIM + 1) * HEAD_DIM; i += 256) svk[i] = hvk[i];
    __syncthreads();
    const int token = blockIdx.x * 256 + threadIdx.x;
    if (token >= num_tokens) return;
    uint16_t *qp = q + (((size_t)batch * tokens_pad + token) * heads + head) * HEAD_DIM;
    float qf[HEAD_DIM];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const u32x4_t w = *(const u32x4_t *)(qp + 8 * i);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            qf[8 * i + 2 * j] = bits_f32(w[j] << 16);
            qf[8 * i + 2 * j + 1] = bits_f32(w[j] & 0xFFFF0000u);
        }
    }
    // out[j] = sum_i q[i] * vk[j][i], i ascending in fp32 as in the reference (:719-729)
    float den = 0.f;
#pragma unroll
    for (int i = 0; i < HEAD_DIM; i++) den = __builtin_fmaf(qf[i], svk[HEAD_DIM * HEAD_DIM + i], den);
    const float rden = 1.0f / (den + eps);
#pragma unroll
    for (int j0 = 0; j0 < HEAD_DIM; j0 += 8) {
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < HEAD_DIM; i++) s = __builtin_fmaf(qf[i], svk[(j0 + j) * HEAD_DIM + i], s);
            o[j] = s * rden;
        }
        u32x4_t w;
#pragma unroll
        for (int j = 0; j < 4; j++) w[j] = pack_bf16x2(o[2 * j], o[2 * j + 1]);
        *(u32x4_t *)(qp + j0) = w;
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
    hipLaunchKernelGGL(vk_mul_q_kernel, dim3((unsigned)((num_tokens + 255) / 256), (unsigned)heads, (unsigned)batch), dim3(256), 0, (hipStream_t)stream,
                       (uint16_t *)q, vk, eps, (int)num_tokens, (int)tokens_pad, (int)heads);
    return check_launch("linearattn_vk_mul_q");
}
