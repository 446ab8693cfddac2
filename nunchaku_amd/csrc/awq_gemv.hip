// AWQ W4A16 GEMV: out[m, n] = sum_k bf16(code[n, k] * scale[k/64, n] + zero[k/64, n]) * x[m, k] for m <= 8 rows.
// Counterpart of gemv_kernel (src/kernels/awq/gemv_awq.cu:84-215) behind ops.gemv_awq
// (nunchaku/csrc/pybind.cpp, nunchaku/ops/gemv.py), used by AWQW4A16Linear (nunchaku/models/linear.py:138-208).
//
// HBM-bound: every weight byte is read once.  The kernel reads the reference's storage as it is (no
// repack): per 4 output rows and 64 input channels a block of 128 bytes, 32 bytes per row
// (nunchaku/models/text_encoders/tinychat_utils.py:76-106), so a 4-row group is contiguous along K and a
// wave-wide 16-byte load covers 4 rows x 512 channels in 1 KB.  One wave owns one 4-row group for the
// whole K extent; lane l holds row (l % 8) / 2 and the 32 channels 512 it + 64 (l / 8) + 32 (l % 2) + [0, 32).
// Word i2 of its 16 bytes, nibble p + 4 b, is channel 8 p + 2 i2 + b: the nibbles p and p + 4 are a pair
// of neighbouring channels, which after dequantization is one packed bf16 pair for v_dot2_f32_bf16 against
// the pair of activations as loaded.
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

typedef __bf16 bf16x2_v __attribute__((ext_vector_type(2)));

// XLDS: the rows of x are copied to LDS once per workgroup (every wave needs all of x; from global memory
// the activation loads, 64 bytes per lane, row of x and step, outweigh the weight stream from 2 rows on).
template <int MT, bool XLDS>
__global__ void __launch_bounds__(256) awq_gemv_kernel(AwqParams p) {
    extern __shared__ u32x4_t xlds[];  // [M][K] bf16
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (XLDS) {
        const int n16 = p.M * p.K / 8;
        for (int i = threadIdx.x; i < n16; i += 256) xlds[i] = ((const u32x4_t *)p.x)[i];
        __syncthreads();
    }
    // Workgroups are dealt to the 8 XCDs in turn (blockIdx % 8), each with its own L2.  A 128-byte line of
    // scales or zeros serves 64 output rows = 16 row groups = 4 workgroups: consecutive workgroups of the
    // row order are therefore given to the same XCD, so that the line is fetched from memory once, not 8 times.
    int wg = blockIdx.x;
    if (gridDim.x % 8 == 0) wg = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
    const int rg = wg * 4 + wave;  // 4-row group
    if (rg * 4 >= p.N) return;
    const int u = lane & 7, blk = lane >> 3;
    const int row = rg * 4 + (u >> 1);
    const int kblocks = p.K / 64;
    const int iters = (kblocks + 7) / 8;
    const u32x4_t *wp = (const u32x4_t *)(p.qweight + (size_t)rg * p.K * 2) + lane;

    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m] = 0.f;

    // Weights, scales and zeros are requested DEPTH steps ahead (a ring of DEPTH + 1 register sets, indexed
    // statically).  Every request is unconditional: a step or channel block past the end re-reads the last
    // valid one and gets scale and zero 0, so that it contributes nothing; a request behind a branch would make
    // the compiler's wait counting assume the worst and wait for the requests made ahead.
    constexpr int DEPTH = 3;
    u32x4_t wq[DEPTH + 1];
    uint16_t sq[DEPTH + 1], zq[DEPTH + 1];
    auto load_w = [&](int it, int slot) {
        int kb = it * 8 + blk;
        kb = kb < kblocks ? kb : kblocks - 1;
        wq[slot] = __builtin_nontemporal_load((const u32x4_t *)(p.qweight + ((size_t)rg * kblocks + kb) * 128) + u);
        sq[slot] = p.scales[(size_t)kb * p.N + row];
        zq[slot] = p.zeros[(size_t)kb * p.N + row];
    };
    auto step = [&](int it, int slot) {
        const bool ok = it * 8 + blk < kblocks;
        const u32x4_t w = wq[slot];
        const float s = ok ? bf16_bits_to_f32(sq[slot]) : 0.f, z = ok ? bf16_bits_to_f32(zq[slot]) : 0.f;
        load_w(it + DEPTH, slot == 0 ? DEPTH : slot - 1);  // the set freed by the previous step ... see the ring below
        // activations of this lane's 32 channels for every row of x (a channel block past the end is
        // clamped to the last one: its weights are zero)
        int kb = it * 8 + blk;
        kb = kb < kblocks ? kb : kblocks - 1;
        const int k0 = kb * 64 + 32 * (u & 1);
        uint32_t xv[MT][16];
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const size_t xoff = (size_t)(m < p.M ? m : p.M - 1) * p.K + k0;
            const u32x4_t *xp = XLDS ? xlds + xoff / 8 : (const u32x4_t *)(p.x + xoff);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u32x4_t v = xp[i];
                xv[m][4 * i] = v[0]; xv[m][4 * i + 1] = v[1]; xv[m][4 * i + 2] = v[2]; xv[m][4 * i + 3] = v[3];
            }
        }
#pragma unroll
        for (int i2 = 0; i2 < 4; i2++) {
            const uint32_t lo = w[i2] & 0x0F0F0F0Fu, hi = (w[i2] >> 4) & 0x0F0F0F0Fu;  // nibbles 0 2 4 6 / 1 3 5 7, one per byte
#pragma unroll
            for (int pq = 0; pq < 4; pq++) {
                const uint32_t src = (pq & 1) ? hi : lo;
                const int byte = pq >> 1;  // nibble pq is byte pq / 2 of its word, nibble pq + 4 two bytes higher
                const float q0 = (float)((src >> (8 * byte)) & 0xFFu), q1 = (float)((src >> (8 * byte + 16)) & 0xFFu);
                // bf16(code * scale + zero): the sum of a 12-bit product and an 8-bit number, rounded once to fp32
                // and then to bf16 (the reference rounds once, to bf16; the two differ only on exact ties of the
                // second rounding)
                const uint32_t pair = pack_bf16x2(__builtin_fmaf(q0, s, z), __builtin_fmaf(q1, s, z));
                const int xw = i2 + 4 * pq;  // channels 8 pq + 2 i2 + {0, 1} = word 4 pq + i2 of the lane's 16
#pragma unroll
                for (int m = 0; m < MT; m++)
                    acc[m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_v, pair), __builtin_bit_cast(bf16x2_v, xv[m][xw]), acc[m], false);
            }
        }
    };
#pragma unroll
    for (int d = 0; d < DEPTH; d++) load_w(d, d);
    // step it uses set it % (DEPTH + 1) and refills the set of step it - 1, which is (it + DEPTH) % (DEPTH + 1)
    for (int it0 = 0; it0 < iters; it0 += DEPTH + 1) {
#pragma unroll
        for (int sl = 0; sl <= DEPTH; sl++) {
            if (it0 + sl >= iters) goto done;
            step(it0 + sl, sl);
        }
    }
done:
    // lanes with the same (l % 8) / 2 hold parts of the same row
#pragma unroll
    for (int m = 0; m < MT; m++) {
        float a = acc[m];
        a += __shfl_xor(a, 1);
        a += __shfl_xor(a, 8);
        a += __shfl_xor(a, 16);
        a += __shfl_xor(a, 32);
        if (lane < 8 && (lane & 1) == 0 && m < p.M) {
            // the reference stores bf16 and adds the bias to that (linear.py:183-185): two roundings
            float o = bf16_bits_to_f32(f32_to_bf16_bits(a));
            if (p.bias) o = bf16_bits_to_f32(f32_to_bf16_bits(o + bf16_bits_to_f32(p.bias[row])));
            p.out[(size_t)m * p.N + row] = (uint16_t)f32_to_bf16_bits(o);
        }
    }
}

template <int MT>
int launch(const AwqParams &p, hipStream_t stream) {
    const size_t xbytes = (size_t)p.M * p.K * 2;
    const dim3 grid((p.N / 4 + 3) / 4);
    if (xbytes <= 64 * 1024) {
        auto kern = awq_gemv_kernel<MT, true>;
        if (xbytes > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)xbytes);
            if (e != hipSuccess) return fail(SVDQ_ELAUNCH, "awq_gemv: cannot reserve %zu bytes of LDS: %s", xbytes, hipGetErrorString(e));
        }
        hipLaunchKernelGGL(kern, grid, dim3(256), xbytes, stream, p);
    } else {
        hipLaunchKernelGGL((awq_gemv_kernel<MT, false>), grid, dim3(256), 0, stream, p);
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
    if (a->M == 1) return launch<1>(p, st);
    if (a->M == 2) return launch<2>(p, st);
    if (a->M <= 4) return launch<4>(p, st);
    return launch<8>(p, st);
}
