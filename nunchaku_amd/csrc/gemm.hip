// Host entry point of operator 2 (argument validation, kernel variant selection).  The device code
// lives in gemm_kernel.h and is instantiated per variant in gemm_variant.hip.
#include "gemm_params.h"

using namespace svdq;

namespace svdq {
int launch_gemm_fp4_v4(const GemmParams &p, int nwg, hipStream_t stream);
int launch_gemm_fp4_v5(const GemmParams &p, int nwg, hipStream_t stream);
namespace g6 {
int launch_plain(const Params &p, int nwg, hipStream_t stream);
int launch_next(const Params &p, int nwg, hipStream_t stream);
}  // namespace g6
}  // namespace svdq

#include <mutex>
#include <stdlib.h>
#include <vector>

namespace {
// Workspace of one (device, stream) pair: launches on one stream run one after the other and can share
// it, launches on different streams may overlap and must not.  It is allocated the first time a launch
// needs one.  A block that has been handed to a launch is never freed behind the caller's back: a HIP graph
// captured through this entry point holds the block's address for as long as the graph lives.  A pair
// that needs more than it has gets a new, larger block (at least half as large again, so that all the
// blocks a pair ever outgrew stay below twice its present one) and the old one is retired, still
// allocated; svdq_release_workspaces is the only place that frees.  The first `zero_bytes` hold arrival
// counters: zero when allocated, and every launch that completes leaves them at zero again.  The rest is
// scratch (parked partial sums, low-rank shares).
struct Workspace {
    int dev;
    hipStream_t stream;
    uint8_t *ptr;
    size_t zero_bytes, scratch_bytes;
    bool dirty;  // a launch failed: the zero region is cleared again before the next use
};
struct Retired {
    int dev;
    void *ptr;
};
std::vector<Workspace> g_ws;
std::vector<Retired> g_retired;
std::mutex g_ws_mutex;  // held from the look-up until the launch that uses the workspace has been enqueued

__global__ void zero_f32_kernel(float *p, int64_t n) {
    const int64_t i = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) * 4;
    if (i + 3 < n) *(float4_t *)(p + i) = float4_t{0.f, 0.f, 0.f, 0.f};
    else for (int64_t j = i; j < n; j++) p[j] = 0.f;
}

// Sums the shares that the column blocks (INT4 kernel: 256 columns each) or chunks (NVFP4 kernel: 128 columns) of a
// GEMM launch left for the next layer's low-rank projection, in ascending order, and writes lora_act [M_pad][R]
// row-major.  A share is [M_pad / 32 slabs][R / 16 rank tiles][2 halves of 16 rows][64 lanes] x float4, lane l holding
// rows 4 (l / 16) + [0, 4), rank l % 16 of a 16 x 16 tile (the result registers of the matrix instruction).
__global__ void __launch_bounds__(256) reduce_shares_kernel(const float4_t *part, float *out, int nshares, int M_pad, int R) {
    const int RT = R / 16, quads = M_pad * R / 4;
    const int item = blockIdx.x * 256 + threadIdx.x;
    if (item >= quads) return;
    float4_t sum = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int b0 = 0; b0 < nshares; b0 += 8) {  // eight requests in flight
        float4_t v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = part[(size_t)(b0 + u < nshares ? b0 + u : nshares - 1) * quads + item];
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (b0 + u < nshares) {
#pragma unroll
                for (int e = 0; e < 4; e++) sum[e] += v[u][e];
            }
    }
    const int ln = item & 63, m2 = (item >> 6) & 1, rest = item >> 7;  // rest = slab * RT + rank tile
    const int rt = rest % RT, slab32 = rest / RT;
    const int row = slab32 * 32 + 16 * m2 + 4 * (ln >> 4), rank = 16 * rt + (ln & 15);
#pragma unroll
    for (int e = 0; e < 4; e++) out[(size_t)(row + e) * R + rank] = sum[e];
}

// Sums the linear-attention shares of the row blocks of a GEMM launch (gemm_params.h; per row block and head 1056 floats:
// the 32 x 32 part [i][j] in the order of the matrix instruction's result registers, element e of lane l at
// ((e / 4) * 64 + l) * 4 + e % 4 with i = 8 (e / 4) + 4 (l / 32) + e % 4, j = l % 32; then the 32 column sums) into
// out_vk [batch][head][33][32].
__global__ void __launch_bounds__(256) reduce_vk_kernel(const float *part, float *out, int batch, int blocks_per_batch, int heads) {
    // 64 outputs per workgroup; the row blocks of an output are split over four threads (more requests in flight),
    // whose sums are added in ascending order
    __shared__ float quarter[4][64];
    const int idx = blockIdx.x * 64 + (threadIdx.x & 63), qt = threadIdx.x >> 6;
    const bool live = idx < batch * heads * VK_HEAD_FLOATS;
    float sum = 0.f;
    if (live) {
        const int pos = idx % VK_HEAD_FLOATS, head = (idx / VK_HEAD_FLOATS) % heads, b = idx / (VK_HEAD_FLOATS * heads);
        int src = pos;  // row 32: stored as it is
        if (pos < 1024) {
            const int i = pos >> 5, j = pos & 31;
            const int g = i >> 3, kb = (i >> 2) & 1, e3 = i & 3;
            src = (g * 64 + kb * 32 + j) * 4 + e3;
        }
        const float *p0 = part + ((size_t)b * blocks_per_batch * heads + head) * VK_HEAD_FLOATS + src;
        const size_t stride = (size_t)heads * VK_HEAD_FLOATS;
        const int per = (blocks_per_batch + 3) / 4, first = qt * per, last = first + per < blocks_per_batch ? first + per : blocks_per_batch;
        for (int s0 = first; s0 < last; s0 += 8) {  // eight requests in flight
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = p0[(size_t)(s0 + u < last ? s0 + u : last - 1) * stride];
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (s0 + u < last) sum += v[u];
        }
    }
    quarter[qt][threadIdx.x & 63] = sum;
    __syncthreads();
    if (live && qt == 0) out[idx] = ((quarter[0][threadIdx.x] + quarter[1][threadIdx.x]) + quarter[2][threadIdx.x]) + quarter[3][threadIdx.x];
}

void clear_zero_region(Workspace *w) {
    const int64_t n = (int64_t)(w->zero_bytes / 4);
    if (n > 0) SVDQ_LAUNCH(zero_f32_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, w->stream, (float *)w->ptr, n);
    w->dirty = false;
}

// (the caller holds g_ws_mutex) returns nullptr, with the error text set, on failure
Workspace *get_workspace(int dev, hipStream_t stream, size_t zero_bytes, size_t scratch_bytes) {
    Workspace *w = nullptr;
    for (Workspace &cand : g_ws)
        if (cand.dev == dev && cand.stream == stream) w = &cand;
    if (w && w->zero_bytes >= zero_bytes && w->scratch_bytes >= scratch_bytes) {
        if (w->dirty) clear_zero_region(w);
        return w;
    }
    // A new block is needed.  Not while the stream is being captured: the allocation is not a stream
    // operation, and the runtime refuses it in a capture of the global mode.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone) {
        fail(SVDQ_EUNSUPPORTED, "gemm: this call needs %zu bytes of workspace that the stream's pair does not have yet, and the stream is being "
             "captured: make the call once before the capture, or use svdq_gemm_w4a4_noalloc", zero_bytes + scratch_bytes);
        return nullptr;
    }
    if (w) {
        if (zero_bytes < w->zero_bytes) zero_bytes = w->zero_bytes;
        if (scratch_bytes < w->scratch_bytes + w->scratch_bytes / 2) scratch_bytes = w->scratch_bytes + w->scratch_bytes / 2;
    }
    zero_bytes = (zero_bytes + (1u << 20) - 1) & ~(size_t)((1u << 20) - 1);  // in steps of 1 MB: few regrows
    uint8_t *ptr = nullptr;
    hipError_t e = hipMalloc((void **)&ptr, zero_bytes + scratch_bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        fail(SVDQ_ELAUNCH, "gemm: cannot allocate %zu bytes of workspace: %s", zero_bytes + scratch_bytes, hipGetErrorString(e));
        return nullptr;
    }
    if (w) {
        // launches already enqueued on this stream (and graphs that captured this block) go on using the old block
        g_retired.push_back(Retired{dev, w->ptr});
    } else {
        g_ws.push_back(Workspace{dev, stream, nullptr, 0, 0, false});
        w = &g_ws.back();
    }
    w->ptr = ptr;
    w->zero_bytes = zero_bytes;
    w->scratch_bytes = scratch_bytes;
    clear_zero_region(w);  // on the caller's stream: ordered before the launch that follows
    return w;
}

// ---- the scratch of svdq_gemm_w4a4_noalloc --------------------------------------------------------
// A fixed array in device memory, one copy per GPU, held until the process ends: first the region that
// must be zero when a launch starts (arrival counters), then parked partial sums and low-rank shares.
constexpr size_t NOALLOC_ZERO_BYTES = 1u << 20, NOALLOC_SCRATCH_BYTES = 80u << 20;
static __device__ __align__(256) unsigned char scratch[NOALLOC_ZERO_BYTES + NOALLOC_SCRATCH_BYTES];
uint8_t *g_scratch_ptr[64] = {nullptr};  // the array's device address on each GPU, asked once per GPU
std::mutex g_scratch_mutex;

// the array's address on device `dev` (which is the current device), or nullptr with the error text set
uint8_t *scratch_address(int dev) {
    if (dev < 0 || dev >= 64) {
        fail(SVDQ_ELAUNCH, "gemm: device index %d out of range", dev);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            fail(SVDQ_ELAUNCH, "gemm: cannot locate the scratch array on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = (uint8_t *)ptr;
    }
    return g_scratch_ptr[dev];
}

// Where a launch gets its workspace from: the per-(device, stream) allocation of svdq_gemm_w4a4, or the
// fixed scratch array of svdq_gemm_w4a4_noalloc.
struct WorkspaceView {
    uint8_t *zero;     // zero_bytes that are zero when the launch starts
    uint8_t *scratch;  // scratch_bytes of anything
    Workspace *owner;  // the allocation behind it (nullptr for the fixed array)
};

// (the caller holds g_ws_mutex when `noalloc` is false) false, with the error text set, on failure
bool acquire_workspace(bool noalloc, int dev, hipStream_t st, size_t zero_bytes, size_t scratch_bytes, WorkspaceView *v) {
    if (!noalloc) {
        Workspace *w = get_workspace(dev, st, zero_bytes, scratch_bytes);
        if (!w) return false;
        *v = WorkspaceView{w->ptr, w->ptr + w->zero_bytes, w};
        return true;
    }
    if (zero_bytes > NOALLOC_ZERO_BYTES || scratch_bytes > NOALLOC_SCRATCH_BYTES) {
        fail(SVDQ_EUNSUPPORTED, "gemm (noalloc): this call needs %zu + %zu bytes of workspace, the fixed scratch holds %zu + %zu; use svdq_gemm_w4a4",
             zero_bytes, scratch_bytes, NOALLOC_ZERO_BYTES, NOALLOC_SCRATCH_BYTES);
        return false;
    }
    uint8_t *base = scratch_address(dev);
    if (!base) return false;
    // The array keeps the last call's contents.  A launch that completes leaves its counters and sums at
    // zero, one that failed or was aborted does not: what this launch needs to be zero is cleared (by a
    // fill kernel, which a caller's graph capture can record).
    const int64_t n = (int64_t)((zero_bytes + 15) / 16 * 4);
    if (n > 0) SVDQ_LAUNCH(zero_f32_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, st, (float *)base, n);
    *v = WorkspaceView{base, base + NOALLOC_ZERO_BYTES, nullptr};
    return true;
}

// Into how many parts along K the tiles of an INT4 launch are split when the caller leaves that to the library.
// Launches with more tiles than compute units are not split: every part parks 128 KB of sums and the last one fetches
// them all, which only pays while compute units would otherwise stand idle.  Below that, a model of the time in us,
// fitted to launches of 24 ... 216 tiles at K = 3072 and 12288 on 256 compute units: a k-group takes a workgroup 0.55 us
// while it has its compute unit to itself and 0.95 us when two share one; prologue and epilogue 4.4; a split costs
// 5.3 + 2.6 per part beyond the first (four parts, whose last one keeps its own sums in registers: 11.5), half as much
// again when compute units are shared.  Measured, whole / best split: 24 tiles at K = 3072 31.2 / 22.5 (4 parts; 3
// parts 24.2), 72 tiles 31.3 / 27.3 (3), 96 tiles 31.8 / 31.0 (2; not split), 144 tiles 32.1 / 38.1 (not split);
// K = 12288: 24 tiles 105.9 / 39.6 (6), 72 tiles 105.6 / 51.7 (3), 144 tiles 106.2 / 78.4 (3).
int choose_kparts(int ntiles, int kgroups, int ncu) {
    if (ntiles > ncu) return 1;
    int best = 1;
    double best_t = 0.55 * kgroups + 4.4;
    for (int k : {2, 3, 4, 6, 8}) {
        const int units = ntiles * k, g = (kgroups + k - 1) / k;
        if (g < 12 || units > 2 * ncu) break;
        const bool shared = units > ncu;
        const double t = g * (shared ? 0.95 : 0.55) + 4.4 + (k == 4 ? 11.5 : 5.3 + 2.6 * (k - 1)) * (shared ? 1.5 : 1.0);
        if (t < (best == 1 ? 0.90 : 0.95) * best_t) {  // a split has to pay clearly; more parts likewise
            best = k;
            best_t = t;
        }
    }
    return best;
}

// ---- INT4: fp6 matrix instruction on the bare codes (gemm6_kernel.h) --------------------------------
int gemm_int4(const svdq_gemm_args *a, hipStream_t st, int dev, int ncu, bool noalloc) {
    g6::Params p;
    p.act = (const uint8_t *)a->act;
    p.ascales = (const uint16_t *)a->ascales;
    p.wgt = (const uint8_t *)a->wgt;
    p.wscales = (const uint8_t *)a->wscales;
    p.bias = (const uint16_t *)a->bias;
    p.wcscales = (const uint16_t *)a->wcscales;
    p.lora_act = a->lora_act_in;
    p.lora_up = (const uint16_t *)a->lora_up;
    p.out = (uint16_t *)a->out;
    p.qout = (uint8_t *)a->qout;
    p.oscales = (uint16_t *)a->oscales;
    p.next_smooth_rcp = a->next_smooth_rcp;
    p.next_down = (const bf16x8_t *)a->next_lora_down;
    p.next_lora_out = a->next_lora_act_out;
    p.next_lora_part = nullptr;
    p.partials = nullptr;
    p.counters = nullptr;
    p.M_pad = (int)a->M_pad; p.N = (int)a->N; p.K = (int)a->K;
    p.M_out = (int)a->M_out; p.N_out = (int)a->N_out; p.R_up = (int)a->R_up; p.R_down = (int)a->R_down;
    p.alpha = a->alpha;
    for (int i = 0; i < MAX_RANK / 16; i++) p.lora_scales[i] = (a->lora_scales && i < (a->R_up + 15) / 16) ? a->lora_scales[i] : 1.0f;
    p.norm_q = (const uint16_t *)a->norm_q;
    p.norm_k = (const uint16_t *)a->norm_k;
    p.rotary = a->rotary_emb;
    p.rot_rows = (int)a->rot_rows;
    p.rope_cols = (int)(a->N / 3 * 2);
    p.norm_eps = a->norm_eps;
    p.qkv.q = (uint16_t *)a->out_q; p.qkv.k = (uint16_t *)a->out_k; p.qkv.v = (uint16_t *)a->out_v;
    p.qkv.stride_q = a->qkv_head_stride[0]; p.qkv.stride_k = a->qkv_head_stride[1]; p.qkv.stride_v = a->qkv_head_stride[2];
    p.qkv.attn_tokens = (int)a->attn_tokens; p.qkv.rows = (int)a->qkv_rows;
    p.vk = a->out_vk;
    p.vk_rows = (int)a->vk_rows;
    p.silu = a->fuse_silu != 0;
    p.gelu = a->qout != nullptr;  // the GELU is composed exactly when the next layer's input is produced (launch_impl.cuh:282-309)

    // One workgroup per 128 x 256 output tile (or per part of one split along K), two resident per compute unit.
    const int mblocks = p.M_pad / g6::BM, nblocks = (p.N + g6::BN - 1) / g6::BN;
    const int ntiles = mblocks * nblocks, kgroups = p.K / 64;
    const int kparts = a->k_split > 0 ? (int)(a->k_split < kgroups ? a->k_split : kgroups) : choose_kparts(ntiles, kgroups, ncu);
    p.kparts = kparts;
    // bands of about ten row blocks, all of the same height where the count allows it
    p.band = (mblocks + (mblocks + 9) / 10 - 1) / ((mblocks + 9) / 10);
    const bool next = a->qout != nullptr || a->next_lora_down != nullptr || a->rotary_emb != nullptr || a->fuse_silu || a->out_vk != nullptr;
    const size_t cnt_bytes = (size_t)ntiles * 4;
    const size_t part_bytes = kparts > 1 ? (size_t)ntiles * kparts * g6::BM * g6::BN * 4 : 0;
    const size_t share_bytes = p.next_down ? (size_t)nblocks * p.M_pad * p.R_down * 4 : 0;  // every column block's share of the next projection
    const size_t vk_bytes = p.vk ? (size_t)(p.M_pad / g6::BM) * (p.N / 96) * VK_HEAD_FLOATS * 4 : 0;  // every row block's linear-attention sums
    if (kparts == 1 && !p.next_down && !p.vk) return next ? g6::launch_next(p, ntiles, st) : g6::launch_plain(p, ntiles, st);
    std::unique_lock<std::mutex> lock(g_ws_mutex, std::defer_lock);
    if (!noalloc) lock.lock();
    const size_t cnt_pad = kparts > 1 ? (cnt_bytes + 255) & ~(size_t)255 : 0;
    WorkspaceView w;
    const size_t scratch_bytes = part_bytes + share_bytes + vk_bytes;
    if (!acquire_workspace(noalloc, dev, st, cnt_pad, scratch_bytes, &w)) return noalloc && (cnt_pad > NOALLOC_ZERO_BYTES || scratch_bytes > NOALLOC_SCRATCH_BYTES) ? SVDQ_EUNSUPPORTED : SVDQ_ELAUNCH;
    p.counters = (int *)w.zero;
    p.partials = (float *)w.scratch;
    p.next_lora_part = (float *)(w.scratch + part_bytes);
    p.vk_part = (float *)(w.scratch + part_bytes + share_bytes);
    int rc = next ? g6::launch_next(p, ntiles * kparts, st) : g6::launch_plain(p, ntiles * kparts, st);
    if (rc == SVDQ_OK && p.next_down) {
        // the column blocks' shares of the next layer's low-rank projection, added in ascending order
        const int quads = p.M_pad * p.R_down / 4;
        SVDQ_LAUNCH(reduce_shares_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, st, (const float4_t *)p.next_lora_part,
                           p.next_lora_out, nblocks, p.M_pad, p.R_down);
        rc = check_launch("gemm_w4a4 (low-rank shares)");
    }
    if (rc == SVDQ_OK && p.vk) {
        // the row blocks' linear-attention sums, added per batch entry in ascending order of the rows
        const int heads = p.N / 96, n = (p.M_pad / p.vk_rows) * heads * VK_HEAD_FLOATS;
        SVDQ_LAUNCH(reduce_vk_kernel, dim3((unsigned)((n + 63) / 64)), dim3(256), 0, st, (const float *)p.vk_part, p.vk, p.M_pad / p.vk_rows,
                           p.vk_rows / g6::BM, heads);
        rc = check_launch("gemm_w4a4 (linear-attention sums)");
    }
    if (rc != SVDQ_OK && w.owner) w.owner->dirty = true;
    return rc;
}

// ---- NVFP4: fp16 matrix instruction on dequantized operands (gemm_kernel.h) -------------------------
int gemm_fp4(const svdq_gemm_args *a, hipStream_t st, int dev, int ncu, bool noalloc) {
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
    p.qout = (uint8_t *)a->qout;
    p.oscales = a->oscales;
    p.next_smooth_rcp = a->next_smooth_rcp;
    p.next_down = (const bf16x8_t *)a->next_lora_down;
    p.next_lora_out = a->next_lora_act_out;
    p.R_down = (int)a->R_down;
    p.M_pad = (int)a->M_pad; p.N = (int)a->N; p.K = (int)a->K;
    p.M_out = (int)a->M_out; p.N_out = (int)a->N_out; p.R_up = (int)a->R_up;
    p.alpha = a->alpha;
    for (int i = 0; i < MAX_RANK / 16; i++) p.lora_scales[i] = (a->lora_scales && i < (a->R_up + 15) / 16) ? a->lora_scales[i] : 1.0f;
    p.norm_q = (const uint16_t *)a->norm_q;
    p.norm_k = (const uint16_t *)a->norm_k;
    p.rotary = a->rotary_emb;
    p.rot_rows = (int)a->rot_rows;
    p.rope_cols = (int)(a->N / 3 * 2);
    p.norm_eps = a->norm_eps;
    p.qkv.q = (uint16_t *)a->out_q; p.qkv.k = (uint16_t *)a->out_k; p.qkv.v = (uint16_t *)a->out_v;
    p.qkv.stride_q = a->qkv_head_stride[0]; p.qkv.stride_k = a->qkv_head_stride[1]; p.qkv.stride_v = a->qkv_head_stride[2];
    p.qkv.attn_tokens = (int)a->attn_tokens; p.qkv.rows = (int)a->qkv_rows;
    p.silu = a->fuse_silu != 0;
    p.gelu = a->qout != nullptr;

    // persistent workgroups: one per compute unit, each walking over its share of the output tiles
    const int ntiles = (int)(a->M_pad / BM) * (int)((a->N + BN - 1) / BN);
    int nwg = ntiles < ncu ? ntiles : ncu;
    int divisor = nwg;  // the largest workgroup count that divides the tile count
    while (ntiles % divisor != 0) divisor--;
    if (a->k_split == 1 || (a->k_split == 0 && ntiles >= ncu && divisor * 100 >= ncu * 84)) {
        // Whole tiles only: asked for, or at least 84 % of the compute units get a whole number of tiles (M = 4608,
        // N = 9216: 216 workgroups x 3 tiles 257 us, 256 even shares 256).  Then the
        // workgroups that share a block of weight columns walk K in step and find it in their L2, and no sums
        // travel through the workspace (M = 4608, N = 21504: 252 workgroups x 6 tiles 549 us, 256 even shares 560).
        nwg = divisor;
    } else if (ntiles < ncu) {
        // Fewer tiles than compute units.  A workgroup alone on its compute unit takes 1.3 us per k-group plus 12 us; the
        // parties of a tile meet through the workspace, which costs about 6 us + 13.5 us per party (measured, 12 tiles:
        // K = 3072 whole 74.6 us, two / three / four parties 63.0 / 64.0 / 69.8; K = 12288 whole 256.8, two / three /
        // four / six / eight parties 158.1 / 130.2 / 122.4 / 126.2 / 139.0).  So: whole tiles unless a split into equal
        // parts pays by that count, or the caller asks for k_split parts.
        const int kg = (int)(a->K / 64);
        int parties = 1;
        if (a->k_split > 1) {
            parties = (int)a->k_split;
        } else {
            double best = 1.3 * kg + 12.0;
            for (int cand : {2, 3, 4, 6, 8}) {
                if (ntiles * cand > ncu || kg / cand < 12) break;
                const double t = 1.3 * kg / cand + 6.0 + 13.5 * cand;
                if (t < (parties == 1 ? 0.90 : 0.95) * best) {  // a split has to pay clearly; more parts likewise
                    best = t;
                    parties = cand;
                }
            }
        }
        const long long units = (long long)ntiles * (a->K / 128);
        long long w = (long long)ntiles * parties;
        if (w > units) w = units;
        if (w > ncu) w = ncu;
        if (w > nwg) nwg = (int)w;
    }
    // the work is split evenly in units of two k-groups; unless the tile count is a multiple of the
    // workgroup count, some tiles are then shared by two or more workgroups and need the workspace
    p.partials = nullptr;
    p.counters = nullptr;
    // (the kernels with the next-layer epilogue also carry the norm + rotary epilogue)
    p.vk = a->out_vk;
    p.vk_rows = (int)a->vk_rows;
    p.vk_part = nullptr;
    p.next_lora_part = nullptr;
    const bool next = a->qout != nullptr || a->next_lora_down != nullptr || a->rotary_emb != nullptr || a->fuse_silu || a->out_vk != nullptr;
    const bool shared_tiles = !(nwg <= ntiles && ntiles % nwg == 0);
    p.whole_band = 0;
    if (!shared_tiles) {
        // bands about as high as the window of an XCD's workgroups (an eighth of them) is wide, all of the same height
        // where the count allows it
        const int mblocks = p.M_pad / BM;
        int h = 1;
        while (h * h * 8 < nwg) h++;
        const int nbands = (mblocks + h - 1) / h;
        p.whole_band = (mblocks + nbands - 1) / nbands;
    }
    // every 128-column chunk's share of the next layer's low-rank projection, every row block's linear-attention sums
    const size_t share_bytes = p.next_down ? (size_t)(p.N / 128) * p.M_pad * p.R_down * 4 : 0;
    const size_t vk_bytes = p.vk ? (size_t)(p.M_pad / 32) * (p.N / 96) * VK_HEAD_FLOATS * 4 : 0;  // (this kernel: per 32-row slab)
    if (!shared_tiles && !share_bytes && !vk_bytes) return next ? launch_gemm_fp4_v5(p, nwg, st) : launch_gemm_fp4_v4(p, nwg, st);
    std::unique_lock<std::mutex> lock(g_ws_mutex, std::defer_lock);
    if (!noalloc) lock.lock();
    const size_t zero_bytes = shared_tiles ? (size_t)ntiles * 4 : 0, part_bytes = shared_tiles ? (size_t)2 * nwg * 256 * 64 * 16 : 0;
    const size_t scratch_bytes = part_bytes + share_bytes + vk_bytes;
    WorkspaceView w;
    if (!acquire_workspace(noalloc, dev, st, zero_bytes, scratch_bytes, &w)) return noalloc && (zero_bytes > NOALLOC_ZERO_BYTES || scratch_bytes > NOALLOC_SCRATCH_BYTES) ? SVDQ_EUNSUPPORTED : SVDQ_ELAUNCH;
    if (shared_tiles) {
        p.counters = (int *)w.zero;
        p.partials = (float *)w.scratch;
    }
    p.next_lora_part = (float *)(w.scratch + part_bytes);
    p.vk_part = (float *)(w.scratch + part_bytes + share_bytes);
    int rc = next ? launch_gemm_fp4_v5(p, nwg, st) : launch_gemm_fp4_v4(p, nwg, st);
    if (rc == SVDQ_OK && p.next_down) {
        const int quads = p.M_pad * p.R_down / 4;
        SVDQ_LAUNCH(reduce_shares_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, st, (const float4_t *)p.next_lora_part,
                           p.next_lora_out, p.N / 128, p.M_pad, p.R_down);
        rc = check_launch("gemm_w4a4 (low-rank shares)");
    }
    if (rc == SVDQ_OK && p.vk) {
        const int heads = p.N / 96, n = (p.M_pad / p.vk_rows) * heads * VK_HEAD_FLOATS;
        SVDQ_LAUNCH(reduce_vk_kernel, dim3((unsigned)((n + 63) / 64)), dim3(256), 0, st, (const float *)p.vk_part, p.vk, p.M_pad / p.vk_rows,
                           p.vk_rows / 32, heads);
        rc = check_launch("gemm_w4a4 (linear-attention sums)");
    }
    if (rc != SVDQ_OK && w.owner) w.owner->dirty = true;
    return rc;
}
}  // namespace

namespace {
int gemm_entry(const svdq_gemm_args *a, void *stream, bool noalloc) {
    SVDQ_REQUIRE(a, "gemm: null args");
    SVDQ_REQUIRE(a->act && a->ascales && a->wgt && a->wscales, "gemm: act/ascales/wgt/wscales must not be null");
    SVDQ_REQUIRE(!a->fp4 || a->colnorm, "gemm: NVFP4 needs colnorm");
    SVDQ_REQUIRE(a->M_pad > 0 && a->M_pad % 256 == 0, "gemm: M_pad (%lld) must be a positive multiple of 256", (long long)a->M_pad);
    SVDQ_REQUIRE(a->N > 0 && a->N % 128 == 0, "gemm: N (%lld) must be a positive multiple of 128", (long long)a->N);
    SVDQ_REQUIRE(a->K > 0 && a->K % 128 == 0, "gemm: K (%lld) must be a positive multiple of 128", (long long)a->K);
    SVDQ_REQUIRE(a->out || a->qout || a->out_q, "gemm: one of out / qout / out_q must be given");
    SVDQ_REQUIRE((a->lora_up != nullptr) == (a->lora_act_in != nullptr), "gemm: lora_up and lora_act_in go together");
    SVDQ_REQUIRE(a->R_up >= 0 && a->R_up % 16 == 0 && a->R_up <= MAX_RANK, "gemm: R_up (%lld) must be a multiple of 16, at most %d", (long long)a->R_up, MAX_RANK);
    SVDQ_REQUIRE((a->R_up > 0) == (a->lora_up != nullptr), "gemm: R_up and lora_up disagree");
    SVDQ_REQUIRE(a->k_split >= 0, "gemm: k_split must not be negative");
    if (a->out) {
        SVDQ_REQUIRE(a->M_out > 0 && a->M_out <= a->M_pad && a->M_pad - a->M_out < 256, "gemm: M_out (%lld) does not fit M_pad (%lld)",
                     (long long)a->M_out, (long long)a->M_pad);
        if (a->out_vk) {
            SVDQ_REQUIRE(a->N_out * 3 == a->N && a->M_out == a->M_pad, "gemm: with out_vk, `out` is the q third of all rows: [M_pad, N/3]");
        } else {
            SVDQ_REQUIRE(a->N_out > 0 && a->N_out <= a->N && a->N - a->N_out < 128 && a->N_out % 8 == 0,
                         "gemm: N_out (%lld) must be a multiple of 8 within 128 of N (%lld)", (long long)a->N_out, (long long)a->N);
        }
    }
    if (a->out_vk) {
        // EpilogueLiteLA (gemm_w4a4_launch_impl.cuh:311-345)
        SVDQ_REQUIRE(a->out && !a->qout && !a->rotary_emb && !a->next_lora_down && !a->fuse_silu, "gemm: out_vk goes with `out` (the q third) alone");
        SVDQ_REQUIRE(a->N % 384 == 0, "gemm: out_vk needs N (%lld) to be three equal parts of whole 128-column blocks", (long long)a->N);
        SVDQ_REQUIRE(a->vk_rows > 0 && a->vk_rows % 256 == 0 && a->M_pad % a->vk_rows == 0,
                     "gemm: vk_rows (%lld) must be a multiple of 256 that divides M_pad (%lld)", (long long)a->vk_rows, (long long)a->M_pad);
        SVDQ_REQUIRE((uintptr_t)a->out_vk % 16 == 0, "gemm: out_vk must be 16-byte aligned");
    }
    SVDQ_REQUIRE(((uintptr_t)a->act | (uintptr_t)a->wgt | (uintptr_t)a->ascales | (uintptr_t)a->wscales | (uintptr_t)a->out |
                  (uintptr_t)a->lora_act_in | (uintptr_t)a->lora_up) % 16 == 0, "gemm: pointers must be 16-byte aligned");
    SVDQ_REQUIRE(a->M_pad * a->N < (1ll << 40) && a->K < (1 << 24), "gemm: shape too large");
    // scale tables are addressed with 32-bit lane offsets
    SVDQ_REQUIRE((a->K / 64) * a->M_pad * 4 < (1ll << 31) && (a->K / 64) * a->N * 8 < (1ll << 31), "gemm: scale tables too large");
    // SiLU goes with the plain store only (gemm_w4a4_launch_impl.cuh:404-417)
    if (a->fuse_silu && (a->qout || a->rotary_emb || !a->out)) return fail(SVDQ_EUNSUPPORTED, "gemm: fuse_silu goes with `out` alone (no qout, no rotary_emb)");
    if (a->fp4 && a->act_unsigned) return fail(SVDQ_EINVAL, "gemm: NVFP4 activations are never unsigned");
    if (a->qout) {
        SVDQ_REQUIRE(a->oscales && a->next_smooth_rcp, "gemm: qout needs oscales and next_smooth_rcp");
        SVDQ_REQUIRE(((uintptr_t)a->qout | (uintptr_t)a->next_smooth_rcp) % 16 == 0, "gemm: qout pointers must be 16-byte aligned");
    }
    SVDQ_REQUIRE((a->next_lora_down != nullptr) == (a->next_lora_act_out != nullptr) && (a->next_lora_down != nullptr) == (a->R_down > 0),
                 "gemm: next_lora_down, next_lora_act_out and R_down go together");
    SVDQ_REQUIRE(a->R_down >= 0 && a->R_down % 16 == 0 && a->R_down <= MAX_RANK, "gemm: R_down (%lld) must be a multiple of 16, at most %d", (long long)a->R_down, MAX_RANK);

    if (a->rotary_emb) {
        SVDQ_REQUIRE(a->norm_q && a->norm_k, "gemm: rotary_emb needs norm_q and norm_k");
        SVDQ_REQUIRE(a->N % 384 == 0, "gemm: rotary_emb needs N (%lld) to be three equal parts of 128-wide heads", (long long)a->N);
        SVDQ_REQUIRE(!a->qout, "gemm: rotary_emb goes without qout");
        const long long covered = a->out_q ? a->attn_tokens : a->M_out;
        if (a->out_q) {
            // EpiloguePackQKV in place of the plain store (gemm_w4a4_launch_impl.cuh:380-397)
            SVDQ_REQUIRE(!a->out && a->out_k && a->out_v, "gemm: out_q, out_k and out_v go together, without `out`");
            SVDQ_REQUIRE(a->qkv_rows > 0 && a->qkv_rows <= a->M_pad && a->attn_tokens >= 0 && a->attn_tokens <= a->qkv_rows,
                         "gemm: attn_tokens (%lld) <= qkv_rows (%lld) <= M_pad (%lld) does not hold", (long long)a->attn_tokens,
                         (long long)a->qkv_rows, (long long)a->M_pad);
            SVDQ_REQUIRE(a->qkv_head_stride[0] >= a->qkv_rows * 128 && a->qkv_head_stride[1] >= a->qkv_rows * 128 && a->qkv_head_stride[2] >= a->qkv_rows * 128,
                         "gemm: a head of out_q / out_k / out_v holds qkv_rows x 128 values, the head strides are smaller");
            SVDQ_REQUIRE(a->qkv_head_stride[0] % 8 == 0 && a->qkv_head_stride[1] % 8 == 0 && a->qkv_head_stride[2] % 8 == 0 &&
                             ((uintptr_t)a->out_q | (uintptr_t)a->out_k | (uintptr_t)a->out_v) % 16 == 0,
                         "gemm: out_q / out_k / out_v and their head strides must be 16-byte aligned");
        } else {
            SVDQ_REQUIRE(a->out && a->N_out == a->N, "gemm: rotary_emb goes with a full-width `out` (or with out_q, out_k, out_v)");
        }
        SVDQ_REQUIRE(a->rot_rows >= covered && a->rot_rows <= a->M_pad && a->rot_rows % 32 == 0,
                     "gemm: rotary_emb has %lld rows for %lld output rows (must cover them, in whole blocks of 32)", (long long)a->rot_rows, covered);
        SVDQ_REQUIRE(((uintptr_t)a->rotary_emb % 16 == 0) && ((uintptr_t)a->norm_q % 8 == 0) && ((uintptr_t)a->norm_k % 8 == 0),
                     "gemm: rotary_emb / norm pointers are not aligned");
    } else {
        SVDQ_REQUIRE(!a->norm_q && !a->norm_k, "gemm: norm_q / norm_k need rotary_emb");
        SVDQ_REQUIRE(!a->out_q && !a->out_k && !a->out_v, "gemm: out_q / out_k / out_v need rotary_emb (the reference composes them only there)");
    }

    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fail(SVDQ_ELAUNCH, "gemm: cannot identify the current device");
    const int ncu = compute_units(dev);
    if (ncu <= 0) return fail(SVDQ_ELAUNCH, "gemm: cannot query the number of compute units");
    return a->fp4 ? gemm_fp4(a, (hipStream_t)stream, dev, ncu, noalloc) : gemm_int4(a, (hipStream_t)stream, dev, ncu, noalloc);
}
}  // namespace

extern "C" int svdq_gemm_w4a4(const svdq_gemm_args *a, void *stream) { return gemm_entry(a, stream, false); }

extern "C" int svdq_gemm_w4a4_noalloc(const svdq_gemm_args *a, void *stream) { return gemm_entry(a, stream, true); }

extern "C" int svdq_release_workspaces(void) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    int prev = 0;
    if (hipGetDevice(&prev) != hipSuccess) return fail(SVDQ_ELAUNCH, "release_workspaces: cannot identify the current device");
    int rc = SVDQ_OK;
    auto release = [&](int dev, void *ptr) {
        if (!ptr) return;
        // everything enqueued on the block's device has finished before the block goes
        if (hipSetDevice(dev) != hipSuccess || hipDeviceSynchronize() != hipSuccess || hipFree(ptr) != hipSuccess) {
            (void)hipGetLastError();
            rc = fail(SVDQ_ELAUNCH, "release_workspaces: cannot free a block on device %d", dev);
        }
    };
    for (Workspace &w : g_ws) release(w.dev, w.ptr);
    for (Retired &r : g_retired) release(r.dev, r.ptr);
    g_ws.clear();
    g_retired.clear();
    (void)hipSetDevice(prev);
    return rc;
}
