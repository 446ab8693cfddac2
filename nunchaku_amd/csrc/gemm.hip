// Host entry point of operator 2 (argument validation, kernel variant selection).  The device code
// lives in gemm_kernel.h and is instantiated per variant in gemm_variant.hip.
#include "gemm_params.h"

using namespace svdq;

namespace svdq {
int launch_gemm_int4_v0(const GemmParams &p, int nwg, hipStream_t stream);
int launch_gemm_int4_v1(const GemmParams &p, int nwg, hipStream_t stream);
int launch_gemm_int4u_v2(const GemmParams &p, int nwg, hipStream_t stream);
int launch_gemm_int4u_v3(const GemmParams &p, int nwg, hipStream_t stream);
int launch_gemm_fp4_v4(const GemmParams &p, int nwg, hipStream_t stream);
int launch_gemm_fp4_v5(const GemmParams &p, int nwg, hipStream_t stream);
}  // namespace svdq

#include <mutex>
#include <stdlib.h>

namespace {
// Workspace for tiles shared between two workgroups, one per (device, stream): launches on one stream
// run one after the other and can share it, launches on different streams may overlap and must not.
// It is allocated the first time a launch needs it and kept until the process ends.
struct Workspace {
    int dev;
    hipStream_t stream;
    uint8_t *ptr;
    size_t counters_bytes, partials_bytes;
};
constexpr int MAX_WORKSPACES = 16;
Workspace g_ws[MAX_WORKSPACES];
int g_ws_count = 0;
std::mutex g_ws_mutex;

__global__ void zero_f32_kernel(float *p, int64_t n);

// returns nullptr (and sets the error text) on failure
Workspace *get_workspace(int dev, hipStream_t stream, size_t counters_bytes, size_t partials_bytes) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace *w = nullptr;
    for (int i = 0; i < g_ws_count; i++)
        if (g_ws[i].dev == dev && g_ws[i].stream == stream) w = &g_ws[i];
    if (w && w->counters_bytes >= counters_bytes && w->partials_bytes >= partials_bytes) return w;
    if (!w) {
        if (g_ws_count == MAX_WORKSPACES) {
            fail(SVDQ_ELAUNCH, "gemm: more than %d (device, stream) pairs need a shared-tile workspace", MAX_WORKSPACES);
            return nullptr;
        }
        w = &g_ws[g_ws_count];
        *w = Workspace{dev, stream, nullptr, 0, 0};
    } else {
        (void)hipFree(w->ptr);  // waits for the device: no launch is still using it
        w->ptr = nullptr;
    }
    if (counters_bytes < (1u << 18)) counters_bytes = 1u << 18;
    counters_bytes = (counters_bytes + 255) & ~(size_t)255;
    uint8_t *ptr = nullptr;
    hipError_t e = hipMalloc((void **)&ptr, counters_bytes + partials_bytes);
    if (e != hipSuccess) {
        fail(SVDQ_ELAUNCH, "gemm: cannot allocate %zu bytes of shared-tile workspace: %s", counters_bytes + partials_bytes, hipGetErrorString(e));
        w->counters_bytes = w->partials_bytes = 0;
        return nullptr;
    }
    // the arrival counters start at zero (and every launch leaves them at zero); cleared by a kernel on
    // the caller's stream so that the clearing is ordered before the launch that follows
    const int64_t n = (int64_t)(counters_bytes / 4);
    hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, stream, (float *)ptr, n);
    w->ptr = ptr;
    w->counters_bytes = counters_bytes;
    w->partials_bytes = partials_bytes;
    if (w == &g_ws[g_ws_count]) g_ws_count++;
    return w;
}

__global__ void zero_f32_kernel(float *p, int64_t n) {
    const int64_t i = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) * 4;
    if (i + 3 < n) *(float4_t *)(p + i) = float4_t{0.f, 0.f, 0.f, 0.f};
    else for (int64_t j = i; j < n; j++) p[j] = 0.f;
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
    // scale tables are addressed with 32-bit lane offsets
    SVDQ_REQUIRE((a->K / 64) * a->M_pad * 4 < (1ll << 31) && (a->K / 64) * a->N * 8 < (1ll << 31), "gemm: scale tables too large");
    // SiLU goes with the plain store only (gemm_w4a4_launch_impl.cuh:404-417)
    if (a->fuse_silu && (a->qout || a->rotary_emb || !a->out)) return fail(SVDQ_EUNSUPPORTED, "gemm: fuse_silu goes with `out` alone (no qout, no rotary_emb)");
    if (a->fp4 && a->act_unsigned) return fail(SVDQ_EINVAL, "gemm: NVFP4 activations are never unsigned");
    // INT4 adds the low-rank projection before scaling, which is exact only for power-of-two column factors
    // (the reference asserts alpha == 1 for INT4, gemm_w4a4_launch_impl.cuh:107, and only NVFP4 layers carry wcscales)
    if (!a->fp4 && (a->alpha != 1.0f || a->wcscales)) return fail(SVDQ_EUNSUPPORTED, "gemm: alpha != 1 and wcscales are NVFP4-only");
    if (a->qout) {
        SVDQ_REQUIRE(a->oscales && a->next_smooth_rcp, "gemm: qout needs oscales and next_smooth_rcp");
        SVDQ_REQUIRE(((uintptr_t)a->qout | (uintptr_t)a->next_smooth_rcp) % 16 == 0, "gemm: qout pointers must be 16-byte aligned");
    }
#ifndef SVDQ_GEMM_TIMING
    SVDQ_REQUIRE((a->next_lora_down != nullptr) == (a->next_lora_act_out != nullptr) && (a->next_lora_down != nullptr) == (a->R_down > 0),
                 "gemm: next_lora_down, next_lora_act_out and R_down go together");
#endif
    SVDQ_REQUIRE(a->R_down >= 0 && a->R_down % 16 == 0 && a->R_down <= 128, "gemm: R_down (%lld) must be a multiple of 16, at most 128", (long long)a->R_down);

    if (a->rotary_emb) {
        SVDQ_REQUIRE(a->norm_q && a->norm_k, "gemm: rotary_emb needs norm_q and norm_k");
        SVDQ_REQUIRE(a->N % 384 == 0, "gemm: rotary_emb needs N (%lld) to be three equal parts of 128-wide heads", (long long)a->N);
        SVDQ_REQUIRE(a->out && !a->qout && a->N_out == a->N, "gemm: rotary_emb goes with a full-width `out` and no qout");
        SVDQ_REQUIRE(a->rot_rows >= a->M_out && a->rot_rows <= a->M_pad && a->rot_rows % 32 == 0,
                     "gemm: rotary_emb has %lld rows for %lld output rows (must cover them, in whole blocks of 32)", (long long)a->rot_rows, (long long)a->M_out);
        SVDQ_REQUIRE(((uintptr_t)a->rotary_emb % 16 == 0) && ((uintptr_t)a->norm_q % 8 == 0) && ((uintptr_t)a->norm_k % 8 == 0),
                     "gemm: rotary_emb / norm pointers are not aligned");
    } else {
        SVDQ_REQUIRE(!a->norm_q && !a->norm_k, "gemm: norm_q / norm_k need rotary_emb");
    }

    GemmParams p;
#ifdef SVDQ_GEMM_TIMING
    p.stamps = (long long *)a->next_lora_act_out;  // debug builds borrow this slot for the stamp buffer
#else
    p.stamps = nullptr;
#endif
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
    p.qout = (uint8_t *)a->qout;
    p.oscales = a->oscales;
    p.next_smooth_rcp = a->next_smooth_rcp;
    p.next_down = (const bf16x8_t *)a->next_lora_down;
    p.next_lora_out = a->next_lora_act_out;
    p.R_down = (int)a->R_down;
    p.M_pad = (int)a->M_pad; p.N = (int)a->N; p.K = (int)a->K;
    p.M_out = (int)a->M_out; p.N_out = (int)a->N_out; p.R_up = (int)a->R_up;
    p.alpha = a->alpha;
    for (int i = 0; i < 8; i++) p.lora_scales[i] = (a->lora_scales && i < (a->R_up + 15) / 16) ? a->lora_scales[i] : 1.0f;
    p.norm_q = (const uint16_t *)a->norm_q;
    p.norm_k = (const uint16_t *)a->norm_k;
    p.rotary = a->rotary_emb;
    p.rot_rows = (int)a->rot_rows;
    p.rope_cols = (int)(a->N / 3 * 2);
    p.norm_eps = a->norm_eps;
    p.silu = a->fuse_silu != 0;
    p.gelu = a->qout != nullptr;  // the GELU is composed exactly when the next layer's input is produced (launch_impl.cuh:282-309)
#ifdef SVDQ_GEMM_TIMING
    p.next_down = nullptr; p.next_lora_out = nullptr; p.R_down = 0;
#endif

    // persistent workgroups: one per compute unit, each walking over its share of the output tiles
    const int ntiles = (int)(a->M_pad / BM) * (int)((a->N + BN - 1) / BN);
    int dev = 0, ncu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || ncu <= 0)
        return fail(SVDQ_ELAUNCH, "gemm: cannot query the number of compute units");
    int nwg = ntiles < ncu ? ntiles : ncu;
    if (getenv("SVDQ_GEMM_NO_SHARED_TILES")) {  // whole tiles only: the largest workgroup count that divides the tile count
        while (ntiles % nwg != 0) nwg--;
    } else if (ntiles < ncu) {
        // fewer tiles than compute units: several workgroups per tile, each with at least 12 units (24
        // k-groups) of work.  The fixed cost of a workgroup and of adding up the parked parts (one round
        // trip to memory per part and 32-row slab) outweighs a finer split: M=256, K=N=3072 takes 119 us
        // with 4 units per workgroup, 79 with 8, 71 with 12, 75 unsplit.  SVDQ_GEMM_MIN_UNITS overrides
        // the number (the tests use it to reach splits among many workgroups).
        const long long units = (long long)ntiles * (a->K / 128);
        const char *mu = getenv("SVDQ_GEMM_MIN_UNITS");
        const int min_units = mu && atoi(mu) > 0 ? atoi(mu) : 12;
        long long w = units / min_units;
        if (w > ncu) w = ncu;
        if (w > nwg) nwg = (int)w;
    }
    // the work is split evenly in units of two k-groups; unless the tile count is a multiple of the
    // workgroup count, some tiles are then shared by two or more workgroups and need the workspace
    p.partials = nullptr;
    p.counters = nullptr;
    if (nwg > ntiles || ntiles % nwg != 0) {
        Workspace *w = get_workspace(dev, (hipStream_t)stream, (size_t)ntiles * 4, (size_t)2 * nwg * 256 * 64 * 16);
        if (!w) return SVDQ_ELAUNCH;
        p.counters = (int *)w->ptr;
        p.partials = (float *)(w->ptr + w->counters_bytes);
    }
    // (the kernels with the next-layer epilogue also carry the norm + rotary epilogue)
    const bool next = a->qout != nullptr || a->next_lora_down != nullptr || a->rotary_emb != nullptr || a->fuse_silu;
    if (p.next_lora_out) {  // the low-rank projection for the next layer is accumulated across column blocks
        const int64_t n = a->M_pad * a->R_down;
        hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, (hipStream_t)stream, p.next_lora_out, n);
    }
    hipStream_t st = (hipStream_t)stream;
    if (a->fp4) return next ? launch_gemm_fp4_v5(p, nwg, st) : launch_gemm_fp4_v4(p, nwg, st);
    if (a->act_unsigned) return next ? launch_gemm_int4u_v3(p, nwg, st) : launch_gemm_int4u_v2(p, nwg, st);
    return next ? launch_gemm_int4_v1(p, nwg, st) : launch_gemm_int4_v0(p, nwg, st);
}
