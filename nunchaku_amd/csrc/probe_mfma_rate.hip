// Measurement aid for bench.py (not part of the operator ABI): the rate at which this GPU sustains
// v_mfma_f32_32x32x16_f16, the instruction the W4A4 GEMM issues, with nothing else going on.  One workgroup
// of 4 waves per compute unit; every wave runs a stream of independent MFMAs on 16 accumulator tiles, the
// GEMM's own shape.  With constant operands the clock stays near its maximum; with random operand bits the
// power management lowers it, and that lower rate is what a GEMM on real data can at best reach.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

__global__ void __launch_bounds__(256, 1) mfma_stream_kernel(float *out, int iters, const half8_t *src) {
    float16_t acc[16];
    for (int i = 0; i < 16; i++)
        for (int e = 0; e < 16; e++) acc[i][e] = 0.f;
    half8_t a[4], b[4];
    for (int t = 0; t < 4; t++) {
        a[t] = src[(threadIdx.x * 8 + t) % 4096];
        b[t] = src[(threadIdx.x * 8 + 4 + t + blockIdx.x) % 4096];
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 16; i++) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i % 4], b[i / 4], acc[i], 0, 0, 0);
    }
    float s = 0.f;
    for (int i = 0; i < 16; i++)
        for (int e = 0; e < 16; e++) s += acc[i][e];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace

// random_operands: 0 = every operand register holds the same constant, 1 = random signs and mantissas
// (magnitudes 0.25 .. 0.5, so the sums stay finite).  Returns 0 and the rate in TFLOP/s, or -1.
extern "C" int svdq_probe_mfma_rate(int random_operands, int iters, int launches, double *tflops) {
    int dev = 0, ncu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -1;
    float *out = nullptr;
    half8_t *src = nullptr;
    if (hipMalloc((void **)&out, (size_t)ncu * 256 * 4) != hipSuccess || hipMalloc((void **)&src, 4096 * 16) != hipSuccess) return -1;
    uint16_t *h = (uint16_t *)malloc(4096 * 16);
    uint32_t x = 12345u;
    for (int i = 0; i < 4096 * 8; i++) {
        x = x * 1664525u + 1013904223u;
        h[i] = random_operands ? (uint16_t)(((x >> 16) & 0x83FFu) | 0x3400u) : (uint16_t)0x3400u;
    }
    hipMemcpy(src, h, 4096 * 16, hipMemcpyHostToDevice);
    free(h);
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    hipLaunchKernelGGL(mfma_stream_kernel, dim3(ncu), dim3(256), 0, 0, out, iters, src);  // warm-up
    hipEventRecord(e0, 0);
    for (int l = 0; l < launches; l++) hipLaunchKernelGGL(mfma_stream_kernel, dim3(ncu), dim3(256), 0, 0, out, iters, src);
    hipEventRecord(e1, 0);
    const hipError_t err = hipEventSynchronize(e1);
    float ms = 0.f;
    hipEventElapsedTime(&ms, e0, e1);
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    hipFree(out);
    hipFree(src);
    if (err != hipSuccess || ms <= 0.f) return -1;
    *tflops = (double)launches * ncu * 4 * (double)iters * 16 * 2.0 * 32 * 32 * 16 / (ms * 1e9);
    return 0;
}
