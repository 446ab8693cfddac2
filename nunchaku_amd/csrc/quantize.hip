// Operator 1: activation smoothing + 4-bit quantization + low-rank down projection in one pass
// over x.  Counterpart of quantize_w4a4_fuse_lora_kernel (src/kernels/zgemm/gemm_w4a4.cuh:1097-1184).
//
// Work split: one workgroup (NW = 8 waves) owns 16*MT consecutive rows for the whole K extent, so the
// low-rank projection needs no atomics and no pre-zeroed output.  Wave w walks the 128-column
// chunks c = w, w+NW, ... and requests the activations of its next chunk before it works on the
// current one: the kernel is bound by memory latency unless enough bytes are in flight per compute
// unit.  Inside a chunk lane (r = lane%16, q = lane/16) holds, for each 16-row
// tile, the 32 consecutive columns 128c + 32q + [0, 32) of row r: half of a 64-group (INT4) or two
// whole 16-groups (NVFP4).  The same registers feed the bf16 MFMA of the low-rank projection
// (operand slot (q, j) of step i = column 128c + 32q + 8i + j; proj_down is stored in that order).
//
// Arithmetic (bit-exact contract; IEEE, round-to-nearest-even):
//   y    = bf16(x / smooth)        computed as bf16(x * fl32(1/smooth)).  For bf16 operands this
//                                  equals bf16(fl32(x / smooth)) bit for bit: the quotient of two
//                                  8-bit significands is never a bf16 rounding midpoint and is
//                                  otherwise at least 2^-16 (relative) away from one, while the two
//                                  fp32 roundings of the product move it by less than 2^-22.
//   amax = max |y| over the group; s = f32(amax) * fl32(1/7); stored scale bf16(s); r = fl32(1/s)
//   code = clamp(rne(y * r), -8, 7)               (gemm_w4a4.cuh:429-523)
//   NVFP4: s = min(f32(amax) * fl32(1/6), 448), stored e4m3(s), code = e2m1(y * fl32(1/s))
//                                                  (gemm_w4a4.cuh:85-187)
#include "svdq_quant.h"

using namespace svdq;

namespace {

struct QuantParams {
    const uint16_t *x;       // bf16 [M, K]
    uint8_t *act;            // native tiles
    void *oscales;           // bf16 [K/64, M_pad] or fp8 [K/16, M_pad]
    const bf16x8_t *down;    // native proj_down
    float *lora_out;         // [M_pad, R]
    const float *smooth_rcp; // [K] or null
    int M, M_pad, K, R;
};

constexpr int NW = 8;  // waves per workgroup

template <int MT, int RT_MAX, bool FP4>
__global__ void __launch_bounds__(64 * NW) quantize_fuse_lora_kernel(QuantParams p) {
    extern __shared__ float red[];  // [NW waves][MT][RT][64][4]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int row0 = blockIdx.x * (16 * MT);
    const int kgroups = p.K / 64;
    const int RT = p.R / 16;

    float4_t acc[MT][RT_MAX];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int rt = 0; rt < RT_MAX; rt++) acc[mt][rt] = float4_t{0.f, 0.f, 0.f, 0.f};

    // x of one chunk: MT tiles x 4 steps x 8 bf16 per lane
    auto load_x = [&](int c, u32x4_t (&xv)[MT][4]) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            const int row = row0 + 16 * mt + r;
            const u32x4_t *src = (const u32x4_t *)(p.x + (size_t)row * p.K + 128 * c + 32 * q);
#pragma unroll
            for (int i = 0; i < 4; i++) xv[mt][i] = row < p.M ? src[i] : u32x4_t{0, 0, 0, 0};
        }
    };
    const int nchunks = p.K / 128;
    u32x4_t xv_next[MT][4];
    if (wave < nchunks) load_x(wave, xv_next);
    for (int c = wave; c < nchunks; c += NW) {
        const int kbase = 128 * c + 32 * q;
        u32x4_t xv[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int i = 0; i < 4; i++) xv[mt][i] = xv_next[mt][i];
        if (c + NW < nchunks) load_x(c + NW, xv_next);
        // ---- reciprocal smoothing factors of my 32 columns
        float rs[32];
        if (p.smooth_rcp) {
            const float4_t *sp = (const float4_t *)(p.smooth_rcp + kbase);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float4_t v = sp[i];
                rs[4 * i] = v[0]; rs[4 * i + 1] = v[1]; rs[4 * i + 2] = v[2]; rs[4 * i + 3] = v[3];
            }
        }
        // ---- low-rank down projection on the raw activations
        if (RT > 0) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
#pragma unroll
                for (int rt = 0; rt < RT_MAX; rt++) {
                    if (rt < RT) {
                        const bf16x8_t b = p.down[((size_t)(c * 4 + i) * RT + rt) * 64 + lane];
#pragma unroll
                        for (int mt = 0; mt < MT; mt++) {
                            bf16x8_t a = __builtin_bit_cast(bf16x8_t, xv[mt][i]);
                            acc[mt][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt][rt], 0, 0, 0);
                        }
                    }
                }
            }
        }
        // ---- smooth, quantize, store
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            const int row = row0 + 16 * mt + r;
            float y[32];
#pragma unroll
            for (int i = 0; i < 4; i++) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t w = xv[mt][i][j];
                    const float lo = bits_f32(w << 16), hi = bits_f32(w & 0xFFFF0000u);
                    const int e = 8 * i + 2 * j;
                    y[e] = p.smooth_rcp ? smooth_quotient(lo, rs[e]) : lo;
                    y[e + 1] = p.smooth_rcp ? smooth_quotient(hi, rs[e + 1]) : hi;
                }
            }
            const size_t tile = (size_t)(row / 32) * kgroups + (2 * c + (q >> 1));
            uint8_t *dst = p.act + tile * TILE_BYTES + (row % 32) * 32 + 16 * (q & 1);
            u32x4_t words;
            if (!FP4) {
                float s;
                quantize_int4_half_group<false>(y, 16, words, s);
                if ((q & 1) == 0)
                    ((uint16_t *)p.oscales)[(size_t)(2 * c + (q >> 1)) * p.M_pad + row] = (uint16_t)f32_to_bf16_bits(s);
            } else {
                uint32_t sc[2];
                quantize_nvfp4_two_groups(y, words, sc);
                // NVFP4 scales: [K/64][M_pad][4] -- the four 16-groups of a 64-group side by side
                uint16_t *os = (uint16_t *)p.oscales;
                os[((size_t)(2 * c + (q >> 1)) * p.M_pad + row) * 2 + (q & 1)] = (uint16_t)(sc[0] | (sc[1] << 8));
            }
            *(u32x4_t *)dst = words;
        }
    }

    // ---- reduce the waves' partial projections and write lora_act[row][rank]
    if (RT > 0) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int rt = 0; rt < RT_MAX; rt++)
                if (rt < RT) *(float4_t *)&red[(((wave * MT + mt) * RT + rt) * 64 + lane) * 4] = acc[mt][rt];
        __syncthreads();
        const int total = 16 * MT * p.R;
        for (int idx = threadIdx.x; idx < total; idx += 64 * NW) {
            const int row = idx / p.R, rank = idx % p.R;
            const int mt = row / 16, rr = row % 16, rt = rank / 16, rc = rank % 16;
            const int src_lane = 16 * (rr / 4) + rc, i = rr % 4;  // 16x16 MFMA result layout
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < NW; w++) sum += red[(((w * MT + mt) * RT + rt) * 64 + src_lane) * 4 + i];
            p.lora_out[(size_t)(row0 + row) * p.R + rank] = sum;
        }
    }
}

template <int MT, int RT_MAX, bool FP4>
int launch(const QuantParams &p, hipStream_t stream) {
    const size_t smem = (size_t)NW * MT * (p.R / 16) * 64 * 4 * sizeof(float);
    auto kern = quantize_fuse_lora_kernel<MT, RT_MAX, FP4>;
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return fail(SVDQ_ELAUNCH, "quantize: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kern, dim3(p.M_pad / (16 * MT)), dim3(64 * NW), smem, stream, p);
    return check_launch("quantize_w4a4_act_fuse_lora");
}

template <bool FP4>
int dispatch(const QuantParams &p, hipStream_t stream) {
    // rows per workgroup: enough workgroups to cover the chip, but amortise proj_down reads at high rank
    const int RT = p.R / 16;
    if (RT <= 2) return p.M_pad >= 8192 ? launch<2, 2, FP4>(p, stream) : launch<1, 2, FP4>(p, stream);
    if (RT <= 4) return launch<2, 4, FP4>(p, stream);
    if (RT <= 8) return launch<2, 8, FP4>(p, stream);
    return fail(SVDQ_EUNSUPPORTED, "quantize: rank %d > 128 is not supported", p.R);
}

}  // namespace

extern "C" int svdq_quantize_w4a4_act_fuse_lora(const svdq_quantize_args *a, void *stream) {
    SVDQ_REQUIRE(a, "quantize: null args");
    SVDQ_REQUIRE(a->input && a->output && a->oscales, "quantize: input/output/oscales must not be null");
    SVDQ_REQUIRE(a->M > 0 && a->M_pad >= a->M && a->M_pad % 256 == 0, "quantize: M_pad (%lld) must be a multiple of 256 and >= M (%lld)",
                 (long long)a->M_pad, (long long)a->M);
    SVDQ_REQUIRE(a->K > 0 && a->K % 128 == 0, "quantize: K (%lld) must be a multiple of 128", (long long)a->K);
    SVDQ_REQUIRE(a->R >= 0 && a->R % 16 == 0, "quantize: rank (%lld) must be a multiple of 16", (long long)a->R);
    SVDQ_REQUIRE(a->R == 0 || (a->lora_down && a->lora_act_out), "quantize: lora_down/lora_act_out must be given when R > 0");
    SVDQ_REQUIRE(a->M_pad < (1ll << 31) / 4 && a->K < (1 << 24), "quantize: shape too large");
    SVDQ_REQUIRE(((uintptr_t)a->input % 16 == 0) && ((uintptr_t)a->output % 16 == 0) && ((uintptr_t)a->lora_down % 16 == 0) &&
                     ((uintptr_t)a->smooth_rcp % 16 == 0),
                 "quantize: pointers must be 16-byte aligned");
    if (a->fuse_glu) return fail(SVDQ_EUNSUPPORTED, "quantize: fuse_glu is not implemented");
    QuantParams p;
    p.x = (const uint16_t *)a->input;
    p.act = (uint8_t *)a->output;
    p.oscales = a->oscales;
    p.down = (const bf16x8_t *)a->lora_down;
    p.lora_out = a->lora_act_out;
    p.smooth_rcp = a->smooth_rcp;
    p.M = (int)a->M; p.M_pad = (int)a->M_pad; p.K = (int)a->K; p.R = (int)a->R;
    return a->fp4 ? dispatch<true>(p, (hipStream_t)stream) : dispatch<false>(p, (hipStream_t)stream);
}
