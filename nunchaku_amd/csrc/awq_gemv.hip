// AWQ W4A16 GEMV: out[m, n] = sum_k bf16(code[n, k] * scale[k/64, n] + zero[k/64, n]) * x[m, k] for m <= 8 rows.
// Counterpart of gemv_kernel (src/kernels/awq/gemv_awq.cu:84-215) behind ops.gemv_awq
// (nunchaku/csrc/pybind.cpp, nunchaku/ops/gemv.py), used by AWQW4A16Linear (nunchaku/models/linear.py:138-208).
//
// HBM-bound: every weight byte is read once.  The kernel reads the reference's storage as it is (no
// repack): per 4 output rows and 64 input channels a block of 128 bytes, 32 bytes per row
// (nunchaku/models/text_encoders/tinychat_utils.py:76-106).  Word i2 of a row's 16 bytes of a 32-channel half,
// nibble p + 4 b, is channel 8 p + 2 i2 + b: the nibbles p and p + 4 are a pair of neighbouring channels, which
// after dequantization is one packed bf16 pair, and the four pairs of one p are eight consecutive channels.
#include "svdq_common.h"

using namespace svdq;

namespace {

struct AwqParams {
    const uint16_t *x;       // bf16 [M, K]
    const uint8_t *qweight;  // reference storage, [N/4][K/64][4 rows][32 bytes]
    const uint16_t *scales;  // bf16 [K/64, N]
    const uint16_t *zeros;   // bf16 [K/64, N]
    const uint16_t *bias;    // bf16 [N] or null
    uint16_t *out;           // bf16 [M, N]
    int M, N, K;
};


// The products go to the matrix cores (with v_dot2_f32_bf16 per row of x and pair instead, one row took 11.9 us
// against 11.3 at K = 3072, N = 18432, four rows 17.4 against 12.0, eight 28.0 against 14.7).
// A workgroup owns 16 output channels; its four waves take the 128-channel steps of K in turn and meet in LDS at the
// end.  Lane l holds output channel l % 16 and the 32 input channels 128 it + 32 (l / 16) + [0, 32) of a step: the four
// packed pairs of nibble position p (channels 8 p ... 8 p + 7 of the 32) are the second operand of the p-th
// v_mfma_f32_16x16x32_bf16 of the step as they come, the first is x[m = l % 16][the same 8 channels] (zero for rows
// beyond M).  The result tile has channel l % 16 and rows 4 (l / 16) + [0, 4) in lane l.
template <bool XLDS>
__global__ void __launch_bounds__(256) awq_gemv_mfma_kernel(AwqParams p) {
    extern __shared__ u32x4_t xlds[];  // XLDS (x fits: up to 64 KB): [M][K] bf16; then, always, 4 waves x 64 lanes x float4
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const size_t xquads = XLDS ? (size_t)p.M * p.K / 8 : 0;
    if (XLDS) {
        for (int i = threadIdx.x; i < (int)xquads; i += 256) xlds[i] = ((const u32x4_t *)p.x)[i];
        __syncthreads();
    }
    int wg = blockIdx.x;
    if (gridDim.x % 8 == 0) wg = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;  // neighbours in N on one XCD: they share lines of scales
    const int n = lane & 15, kb = lane >> 4;
    const int row_raw = wg * 16 + n;
    const int row = row_raw < p.N ? row_raw : p.N - 1;  // a channel beyond N repeats the last one and is not stored
    const int kblocks = p.K / 64;
    const int steps = (p.K + 127) / 128;
    const uint8_t *wrow = p.qweight + ((size_t)(row >> 2) * kblocks * 4 + (row & 3)) * 32 + (kb & 1) * 16;  // + 128 per 64-channel block
    const bool xrow = n < p.M;  // this lane supplies row n of x to the first operand

    constexpr int DEPTH = 3;
    u32x4_t wq[DEPTH + 1];
    uint16_t sq[DEPTH + 1], zq[DEPTH + 1];
    auto block_of = [&](int it) {  // the lane's 64-channel block in step it, clamped to the last valid one
        const int cb = it * 2 + (kb >> 1);
        return cb < kblocks ? cb : kblocks - 1;
    };
    auto load_w = [&](int it, int slot) {
        const int cb = block_of(it);
        wq[slot] = __builtin_nontemporal_load((const u32x4_t *)(wrow + (size_t)cb * 128));
        sq[slot] = p.scales[(size_t)cb * p.N + row];
        zq[slot] = p.zeros[(size_t)cb * p.N + row];
    };
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    auto step = [&](int it, int slot) {
        const bool ok = it * 2 + (kb >> 1) < kblocks;
        const u32x4_t w = wq[slot];
        const float s = ok ? bf16_bits_to_f32(sq[slot]) : 0.f, z = ok ? bf16_bits_to_f32(zq[slot]) : 0.f;
        load_w(it + 4 * DEPTH, slot == 0 ? DEPTH : slot - 1);
        const int k0 = block_of(it) * 64 + 32 * (kb & 1);
        u32x4_t xa[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            xa[j] = u32x4_t{0, 0, 0, 0};
            if (xrow) {
                const size_t xoff = (size_t)n * p.K + k0 + 8 * j;
                xa[j] = XLDS ? xlds[xoff / 8] : *(const u32x4_t *)(p.x + xoff);
            }
        }
        const uint32_t lo[4] = {w[0] & 0x0F0F0F0Fu, w[1] & 0x0F0F0F0Fu, w[2] & 0x0F0F0F0Fu, w[3] & 0x0F0F0F0Fu};
        const uint32_t hi[4] = {(w[0] >> 4) & 0x0F0F0F0Fu, (w[1] >> 4) & 0x0F0F0F0Fu, (w[2] >> 4) & 0x0F0F0F0Fu, (w[3] >> 4) & 0x0F0F0F0Fu};
#pragma unroll
        for (int pq = 0; pq < 4; pq++) {
            // nibbles pq and pq + 4 of word i2 are channels 8 pq + 2 i2 and 8 pq + 2 i2 + 1
            u32x4_t wb;
#pragma unroll
            for (int i2 = 0; i2 < 4; i2++) {
                const uint32_t src = (pq & 1) ? hi[i2] : lo[i2];
                const int byte = pq >> 1;
                const float q0 = (float)((src >> (8 * byte)) & 0xFFu), q1 = (float)((src >> (8 * byte + 16)) & 0xFFu);
                wb[i2] = pack_bf16x2(__builtin_fmaf(q0, s, z), __builtin_fmaf(q1, s, z));  // bf16(code * scale + zero), see above
            }
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, xa[pq]), __builtin_bit_cast(bf16x8_t, wb), acc, 0, 0, 0);
        }
    };
    // wave w takes the steps w, w + 4, ...; the ring of DEPTH + 1 register sets is indexed statically
#pragma unroll
    for (int d = 0; d < DEPTH; d++) load_w(wave + 4 * d, d);
    for (int it0 = wave; it0 < steps; it0 += 4 * (DEPTH + 1)) {
#pragma unroll
        for (int sl = 0; sl <= DEPTH; sl++) {
            if (it0 + 4 * sl >= steps) goto done;
            step(it0 + 4 * sl, sl);
        }
    }
done:
    float4_t *red = (float4_t *)(xlds + xquads);
    red[wave * 64 + lane] = acc;
    __syncthreads();
    if (wave == 0) {
        const float4_t a1 = red[64 + lane], a2 = red[128 + lane], a3 = red[192 + lane];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int m = 4 * kb + i;
            if (m < p.M && row_raw < p.N) {
                // the reference stores bf16 and adds the bias to that (linear.py:183-185): two roundings
                float o = bf16_bits_to_f32(f32_to_bf16_bits(((acc[i] + a1[i]) + a2[i]) + a3[i]));
                if (p.bias) o = bf16_bits_to_f32(f32_to_bf16_bits(o + bf16_bits_to_f32(p.bias[row])));
                p.out[(size_t)m * p.N + row] = (uint16_t)f32_to_bf16_bits(o);
            }
        }
    }
}

int launch_mfma(const AwqParams &p, hipStream_t stream) {
    const size_t xbytes = (size_t)p.M * p.K * 2, red = 4 * 64 * 16;
    const dim3 grid((p.N + 15) / 16);
    if (xbytes <= 64 * 1024) {
        auto kern = awq_gemv_mfma_kernel<true>;
        if (xbytes + red > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(xbytes + red));
            if (e != hipSuccess) return fail(SVDQ_ELAUNCH, "awq_gemv: cannot reserve %zu bytes of LDS: %s", xbytes + red, hipGetErrorString(e));
        }
        SVDQ_LAUNCH(kern, grid, dim3(256), xbytes + red, stream, p);
    } else {
        SVDQ_LAUNCH((awq_gemv_mfma_kernel<false>), grid, dim3(256), red, stream, p);
    }
    return check_launch("awq_gemv_w4a16");
}

}  // namespace

extern "C" int svdq_awq_gemv_w4a16(const svdq_awq_gemv_args *a, void *stream) {
    SVDQ_REQUIRE(a, "awq_gemv: null args");
    SVDQ_REQUIRE(a->x && a->qweight && a->scales && a->zeros && a->out, "awq_gemv: x/qweight/scales/zeros/out must not be null");
    SVDQ_REQUIRE(a->M > 0 && a->M <= 8, "awq_gemv: M (%lld) must be in 1..8", (long long)a->M);  // gemv_awq.cu:262
    SVDQ_REQUIRE(a->N > 0 && a->N % 4 == 0, "awq_gemv: N (%lld) must be a positive multiple of 4", (long long)a->N);
    SVDQ_REQUIRE(a->K > 0 && a->K % 64 == 0 && a->K < (1 << 24), "awq_gemv: K (%lld) must be a positive multiple of 64", (long long)a->K);
    SVDQ_REQUIRE(a->N < (1ll << 28), "awq_gemv: shape too large");
    if (a->group_size != 64) return fail(SVDQ_EUNSUPPORTED, "awq_gemv: group_size %d (only 64 is supported, as in the reference)", a->group_size);  // gemv_awq.cu:263
    SVDQ_REQUIRE(((uintptr_t)a->x | (uintptr_t)a->qweight) % 16 == 0, "awq_gemv: x and qweight must be 16-byte aligned");
    AwqParams p{(const uint16_t *)a->x, (const uint8_t *)a->qweight, (const uint16_t *)a->scales, (const uint16_t *)a->zeros,
                (const uint16_t *)a->bias, (uint16_t *)a->out, (int)a->M, (int)a->N, (int)a->K};
    hipStream_t st = (hipStream_t)stream;
    return launch_mfma(p, st);
}
