// Operator 1: activation smoothing + 4-bit quantization + low-rank down projection in one pass
// over x.  Counterpart of quantize_w4a4_fuse_lora_kernel (src/kernels/zgemm/gemm_w4a4.cuh:1097-1184).
//
// Work split: one workgroup (NW waves) owns 16*MT consecutive rows for the whole K extent, so the
// low-rank projection needs no atomics and no pre-zeroed output.  Wave w walks the 128-column
// chunks c = w, w+NW, ... and keeps the activations of its next DEPTH chunks requested while it works
// on the current one: the kernel is bound by memory latency unless enough bytes are in flight per
// compute unit.  The reciprocal smoothing factors are copied to LDS once per workgroup, and the
// low-rank operands of a chunk are requested before its quantization and used after it.  Inside a
// chunk lane (r = lane%16, q = lane/16) holds, for each 16-row
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
    const uint16_t *x;       // bf16 [M, K], or [M, 2K] (value, gate) pairs when the kernel applies the gated unit
    uint8_t *act;            // INT4: E2M3 fragments [M_pad/128][K/64][4]; NVFP4: nibble tiles [M_pad/32][K/64][32][32 B]
    void *oscales;           // bf16 [K/64, M_pad] or fp8 [K/16, M_pad]
    const bf16x8_t *down;    // native proj_down
    float *lora_out;         // [M_pad, R]
    const float *smooth_rcp; // [K] or null
    int M, M_pad, K, R;
    int rt_base;             // first 16-rank tile of the projection this launch computes (ranks above 128 take several launches)
};

constexpr uint32_t RSRC_WORD3 = 0x00020000;  // raw buffer, 32-bit data format

// SMOOTH: 0 = no smoothing factors, 1 = the K reciprocal factors are copied to LDS once per workgroup,
// 2 = read from global memory per chunk (K too large for LDS).
//
// GLU: the input row holds 2K columns, pairs (value, gate); the K columns that are smoothed, quantized
// and projected are bf16(value * bf16(gate * sigmoid(gate))) (load_act_to_fpsum<fuse_glu>,
// gemm_base.cuh:612-623; silu, gemm_utils.cuh:322-327).  A lane then reads 64 consecutive input columns
// for its 32, and everything after the product is as without GLU.
//
// ROWS (high ranks): the waves of a workgroup split its rows instead of its chunks: wave w owns the 16 MT rows
// after row 16 MT (NW b + w) and all waves walk every chunk together.  The chunk of proj_down they all need (4 KB
// per rank tile: 32 KB at rank 128, more than the activations of the chunk) is then fetched once per workgroup and
// chunk, one chunk ahead, into an LDS double buffer; with chunks split among the waves every wave fetched its own
// chunks' operands from the L2, one dependent request after the other.  No sums cross waves, so there is no
// reduction at the end either.
//
// Ranks above 16 RT_MAX: a launch projects onto the rank tiles [rt_base, rt_base + RT_MAX) only (its accumulators
// live in registers), so the operator launches the kernel once per window of 128 ranks; the launches after the
// first (QUANT false) read x again, which the caches still hold, and neither quantize nor store codes.
template <int NW, int MT, int RT_MAX, int DEPTH, bool FP4, int SMOOTH, bool GLU, bool ROWS, bool QUANT = true>
__global__ void __launch_bounds__(64 * NW) quantize_fuse_lora_kernel(QuantParams p) {
    // smoothing factors [K] during the walk; then, chunks split: [NW waves][MT][RT][64][4] partial projections;
    // rows split: behind the factors two buffers of [4 steps][RT][64 lanes] x 16 bytes of proj_down
    extern __shared__ __attribute__((aligned(16))) float lds[];  // (the alignment lets the factors be read 16 bytes at a time)
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, q = lane >> 4;
    const int row0 = ROWS ? (blockIdx.x * NW + wave) * (16 * MT) : blockIdx.x * (16 * MT);
    const int row_end = row0 + 16 * MT;  // the rows this workgroup (ROWS: wave) writes are [row0, row_end)
    const int kgroups = p.K / 64;
    const int RT_all = p.R / 16;                                                         // rank tiles of proj_down and lora_out
    const int RT = RT_all - p.rt_base < RT_MAX ? RT_all - p.rt_base : RT_MAX;            // rank tiles of this launch
    const int nchunks = p.K / 128;

    float4_t acc[MT][RT_MAX];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int rt = 0; rt < RT_MAX; rt++) acc[mt][rt] = float4_t{0.f, 0.f, 0.f, 0.f};

    // The workgroup's rows as a buffer whose size ends with the last valid row: rows beyond M read as zero
    // without a branch.
    int rows_valid = (p.M < row_end ? p.M : row_end) - row0;
    rows_valid = rows_valid < 0 ? 0 : rows_valid;
    // (descriptor words made scalar explicitly: a descriptor the compiler takes for lane-dependent is
    // looped over lane by lane)
    constexpr int XW = GLU ? 2 : 1;  // input columns per quantized column
    constexpr int XL = 4 * XW;       // 16-byte loads per lane, tile and chunk
    const int ld = XW * p.K;         // input row length
    const uint64_t xbase = (uint64_t)(p.x + (size_t)row0 * ld);
    const uint64_t xbase_s = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(xbase >> 32)) << 32) |
                             (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)xbase);
    const __amdgpu_buffer_rsrc_t xrsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)xbase_s, 0, __builtin_amdgcn_readfirstlane(rows_valid * ld * 2), RSRC_WORD3);
    // A load instruction fetches whole 256-byte (512 with GLU) runs of consecutive rows, 16 bytes per lane: rows
    // RPI * i + lane / PPR, 16-byte piece lane % PPR.  (Every cache line is then touched by one instruction only;
    // fetching the matrix-core operand layout directly, 16 rows x 64 scattered bytes per instruction, was 15 % slower
    // on the whole kernel.)  The pieces are brought into that layout through a per-wave LDS area, see below.
    constexpr int PPR = 16 * XW, RPI = 64 / PPR;  // pieces per row, rows per instruction
    const uint32_t x_voff = (uint32_t)((lane / PPR) * ld * 2 + (lane % PPR) * 16);
    __shared__ __attribute__((aligned(16))) uint8_t transpose_area[NW][16 * PPR * 16];
    uint8_t *tr = transpose_area[wave];

    // x of one chunk: MT tiles x 4 steps x 8 bf16 per lane (twice that with GLU)
    // Requests are unconditional (a request behind a branch makes the compiler's wait counting assume the
    // worst on every path and wait for the chunks requested ahead): a chunk index past the end gets a lane
    // offset beyond the buffer size instead, which reads zeros and touches no memory.  (The hardware checks
    // the lane offset against the size, not the scalar offset that carries the chunk.)
    auto load_x = [&](int c, u32x4_t (&xv)[MT][XL]) {
        const uint32_t beyond = c < nchunks ? 0u : 0x80000000u;
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int i = 0; i < XL; i++)
                xv[mt][i] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, (x_voff | beyond) + (uint32_t)((16 * mt + RPI * i) * ld) * 2, c * 256 * XW, 0);
    };
    // proj_down as a buffer too: empty when there is no low-rank branch, so that its requests need no branch
    const __amdgpu_buffer_rsrc_t drsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.down, 0, RT > 0 ? p.K * p.R * 2 : 0, RSRC_WORD3);
    auto load_down = [&](int c, int i, int rt) {
        return __builtin_bit_cast(bf16x8_t, __builtin_amdgcn_raw_buffer_load_b128(drsrc, lane * 16, (((c * 4 + i) * RT_all + p.rt_base + (rt < RT ? rt : 0)) * 64) * 16, 0));
    };

    // DEPTH chunks are requested ahead of the one being worked on
    u32x4_t xv[DEPTH + 1][MT][XL];
    constexpr int CSTEP = ROWS ? 1 : NW;  // distance between the chunks a wave works on
    const int cfirst = ROWS ? 0 : wave;
#pragma unroll
    for (int s = 0; s < DEPTH; s++) load_x(cfirst + s * CSTEP, xv[s]);

    if (QUANT && SMOOTH == 1) {
        for (int k = threadIdx.x * 4; k < p.K; k += 64 * NW * 4) *(float4_t *)&lds[k] = *(const float4_t *)(p.smooth_rcp + k);
        __syncthreads();
    }

    // rows split: wave w fetches the 1 KB pieces w, w + NW, ... of a chunk's 4 RT KB of proj_down
    uint8_t *down_lds = (uint8_t *)lds + (SMOOTH == 1 ? (size_t)p.K * 4 : 0);
    const int down_chunk_bytes = 4 * RT * 1024;
    constexpr int DPW = ROWS ? (4 * RT_MAX + NW - 1) / NW : 1;  // pieces per wave
    u32x4_t dstage[DPW];
    auto fetch_down = [&](int c) {
        const uint32_t beyond = c < nchunks ? 0u : 0x80000000u;
#pragma unroll
        for (int j = 0; j < DPW; j++) {
            const int piece = wave + j * NW;
            dstage[j] = __builtin_amdgcn_raw_buffer_load_b128(drsrc, (uint32_t)(lane * 16) | beyond | (piece < 4 * RT ? 0u : 0x80000000u),
                                                              c * down_chunk_bytes + (piece < 4 * RT ? piece : 0) * 1024, 0);
        }
    };
    auto park_down = [&](int buf) {
#pragma unroll
        for (int j = 0; j < DPW; j++) {
            const int piece = wave + j * NW;
            if (piece < 4 * RT) *(u32x4_t *)(down_lds + buf * down_chunk_bytes + piece * 1024 + lane * 16) = dstage[j];
        }
    };
    if (ROWS && RT > 0) {
        fetch_down(0);
        park_down(0);
        __syncthreads();
    }

    auto process = [&](int c, u32x4_t (&xin)[MT][XL], u32x4_t (&x_ahead)[MT][XL]) {
        const int kbase = 128 * c + 32 * q;
        // ---- from the load layout to the operand layout: lane (r, q) gets the XL pieces XL * q + i of row r.
        // Row-major in LDS with the pieces of row r rotated by rot(r).  A 16-byte write is served eight consecutive
        // lanes at a time (one row, consecutive pieces: any rotation will do).  A 16-byte read is served 16 lanes at
        // a time, and not consecutive ones: lanes 0-3, 12-15 and 20-27 together, then 4-11, 16-19 and 28-31 (measured
        // pair by pair; the same in the upper half-wave), that is rows {0-3, 12-15} of one q with rows {4-11} of
        // the next.  Their pieces are XL apart, so the rotation must send both row sets to one set of eight 16-byte
        // bank groups that, moved by XL, gives the other eight: r with bit 2 cleared for XL = 4, and for XL = 8 the
        // low two bits of r with bits 2 and 3 both set to bit 3 (with rot(r) = r every such read took two turns).
        // The area is private to the wave, whose LDS operations complete in order.
        auto rot = [](int row) { return XL == 4 ? (row & 11) : ((row & 3) | ((row & 8) ? 12 : 0)); };
        u32x4_t xraw[MT][XL];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
#pragma unroll
            for (int i = 0; i < XL; i++) {
                const int row = RPI * i + lane / PPR, piece = lane % PPR;
                *(u32x4_t *)(tr + row * (PPR * 16) + ((piece + rot(row)) % PPR) * 16) = xin[mt][i];
            }
#pragma unroll
            for (int i = 0; i < XL; i++) xraw[mt][i] = *(const u32x4_t *)(tr + r * (PPR * 16) + ((XL * q + i + rot(r)) % PPR) * 16);
        }
        // ---- requests first: the low-rank operands of this chunk (all four steps when they fit the
        // registers), then the activations DEPTH chunks ahead.  In this order a wait for the operands
        // does not wait for the activations.
        constexpr bool DOWN_UPFRONT = !ROWS && RT_MAX <= 2;
        bf16x8_t dn[DOWN_UPFRONT ? 4 : 1][RT_MAX];
        if (ROWS) fetch_down(c + 1);
        if (DOWN_UPFRONT) {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int rt = 0; rt < RT_MAX; rt++) dn[i][rt] = load_down(c, i, rt);
        }
        load_x(c + DEPTH * CSTEP, x_ahead);
        __builtin_amdgcn_sched_barrier(0);

        // ---- the gated unit: 16 (value, gate) pairs of two loads become the 8 bf16 of one step
        u32x4_t xglu[GLU ? MT : 1][4];
        if (GLU) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        float v[2];
#pragma unroll
                        for (int h = 0; h < 2; h++) {
                            const uint32_t w = xraw[mt][2 * i + (2 * j + h) / 4][(2 * j + h) % 4];
                            const float val = bits_f32(w << 16), gate = bits_f32(w & 0xFFFF0000u);
                            const float sg = gate * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * gate));
                            v[h] = val * bits_f32(f32_to_bf16_bits(sg) << 16);
                        }
                        xglu[mt][i][j] = pack_bf16x2(v[0], v[1]);
                    }
        }
        auto xs = [&](int mt, int i) -> u32x4_t {
            if constexpr (GLU) return xglu[mt][i];
            else return xraw[mt][i];
        };

        // ---- smooth, quantize, store
#pragma unroll
        for (int mt = 0; mt < (QUANT ? MT : 0); mt++) {
            const int row = row0 + 16 * mt + r;
            float y[32];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float4_t rs0, rs1;
                if (SMOOTH == 1) {
                    rs0 = *(const float4_t *)&lds[kbase + 8 * i];
                    rs1 = *(const float4_t *)&lds[kbase + 8 * i + 4];
                } else if (SMOOTH == 2) {
                    rs0 = *(const float4_t *)(p.smooth_rcp + kbase + 8 * i);
                    rs1 = *(const float4_t *)(p.smooth_rcp + kbase + 8 * i + 4);
                }
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t w = xs(mt, i)[j];
                    float lo = bits_f32(w << 16), hi = bits_f32(w & 0xFFFF0000u);
                    if (FP4) {
                        // the reference adds its shift (zero here) before the division, which turns -0 into
                        // +0 (gemm_w4a4.cuh:986); only the E2M1 sign bit can tell the difference
                        lo += 0.0f;
                        hi += 0.0f;
                    }
                    const int e = 8 * i + 2 * j;
                    if (SMOOTH) {
                        // bf16(x / smooth) for the pair: two products, one packed hardware rounding
                        const float r0 = j < 2 ? rs0[2 * j] : rs1[2 * j - 4], r1 = j < 2 ? rs0[2 * j + 1] : rs1[2 * j - 3];
                        const uint32_t pr = pack_bf16x2(__fmul_rn(lo, r0), __fmul_rn(hi, r1));
                        y[e] = bits_f32(pr << 16);
                        y[e + 1] = bits_f32(pr & 0xFFFF0000u);
                    } else {
                        y[e] = lo;
                        y[e + 1] = hi;
                    }
                }
            }
            if (!FP4) {
                // E2M3 fragments [M_pad/128][K/64][4]: this lane's 32 codes are one fragment slot
                u32x4_t lo;
                u32x2_t hi;
                float s;
                quantize_int4_half_group_e2m3<false>(y, 16, lo, hi, s);
                // (both lanes of a group hold the same scale and store it: no branch)
                ((uint16_t *)p.oscales)[(size_t)(2 * c + (q >> 1)) * p.M_pad + row] = (uint16_t)f32_to_bf16_bits(s);
                uint8_t *frag = p.act + (((size_t)(row / ACT_BLOCK_ROWS) * kgroups + (2 * c + (q >> 1))) * 4 + (row % ACT_BLOCK_ROWS) / 32) * FRAG_BYTES;
                const int slot = (row % 32) + 32 * (q & 1);
                *(u32x4_t *)(frag + slot * 16) = lo;
                *(u32x2_t *)(frag + 1024 + slot * 8) = hi;
            } else {
                const size_t tile = (size_t)(row / 32) * kgroups + (2 * c + (q >> 1));
                uint8_t *dst = p.act + tile * TILE_BYTES + (row % 32) * 32 + 16 * (q & 1);
                u32x4_t words;
                uint32_t sc[2];
                quantize_nvfp4_two_groups(y, words, sc);
                // NVFP4 scales: [K/64][M_pad][4] -- the four 16-groups of a 64-group side by side
                uint16_t *os = (uint16_t *)p.oscales;
                os[((size_t)(2 * c + (q >> 1)) * p.M_pad + row) * 2 + (q & 1)] = (uint16_t)(sc[0] | (sc[1] << 8));
                *(u32x4_t *)dst = words;
            }
        }

        // ---- low-rank down projection on the raw activations (rank tiles beyond R repeat tile 0 into
        // accumulators that are never stored: cheaper than a branch per tile)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int rt = 0; rt < RT_MAX; rt++) {
                bf16x8_t b;
                if (ROWS) b = *(const bf16x8_t *)(down_lds + (c & 1) * down_chunk_bytes + ((i * RT + (rt < RT ? rt : 0)) * 64 + lane) * 16);
                else b = DOWN_UPFRONT ? dn[i][rt] : load_down(c, i, rt);
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
                    acc[mt][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, xs(mt, i)), b, acc[mt][rt], 0, 0, 0);
            }
        if (ROWS && RT > 0) {
            // the next chunk's operands go to the other buffer, which everybody finished reading before the
            // previous barrier
            park_down((c + 1) & 1);
            __syncthreads();
        }
    };

    // wave w walks the chunks w, w + NW, ...; the ring of DEPTH + 1 register buffers is indexed statically
    for (int c0 = cfirst;; c0 += (DEPTH + 1) * CSTEP) {
#pragma unroll
        for (int s = 0; s <= DEPTH; s++) {
            const int c = c0 + s * CSTEP;
            if (c >= nchunks) goto walked;
            process(c, xv[s], xv[(s + DEPTH) % (DEPTH + 1)]);
        }
    }
walked:

    if (ROWS) {
        // every wave holds the finished sums of its own rows: lane l has rows 4 (l / 16) + [0, 4), rank l % 16 of a tile
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int rt = 0; rt < RT_MAX; rt++)
                if (rt < RT) {
#pragma unroll
                    for (int i = 0; i < 4; i++) p.lora_out[(size_t)(row0 + 16 * mt + 4 * q + i) * p.R + 16 * (p.rt_base + rt) + r] = acc[mt][rt][i];
                }
        return;
    }
    // ---- reduce the waves' partial projections and write lora_act[row][rank]
    if (RT > 0) {
        if (QUANT && SMOOTH == 1) __syncthreads();  // the factors in LDS are not needed any more
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int rt = 0; rt < RT_MAX; rt++)
                if (rt < RT) *(float4_t *)&lds[(((wave * MT + mt) * RT + rt) * 64 + lane) * 4] = acc[mt][rt];
        __syncthreads();
        const int RW = 16 * RT;  // ranks of this launch
        const int total = 16 * MT * RW;
        for (int idx = threadIdx.x; idx < total; idx += 64 * NW) {
            const int row = idx / RW, rank = idx % RW;
            const int mt = row / 16, rr = row % 16, rt = rank / 16, rc = rank % 16;
            const int src_lane = 16 * (rr / 4) + rc, i = rr % 4;  // 16x16 MFMA result layout
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < NW; w++) sum += lds[(((w * MT + mt) * RT + rt) * 64 + src_lane) * 4 + i];
            p.lora_out[(size_t)(row0 + row) * p.R + 16 * p.rt_base + rank] = sum;
        }
    }
}

constexpr size_t SMOOTH_LDS_MAX = 64 * 1024;  // two workgroups of a compute unit must fit side by side

template <int NW, int MT, int RT_MAX, int DEPTH, bool FP4, int SMOOTH, bool GLU, bool ROWS = false, bool QUANT = true>
int launch_as(const QuantParams &p, hipStream_t stream) {
    const int rt_launch = p.R / 16 - p.rt_base < RT_MAX ? p.R / 16 - p.rt_base : RT_MAX;
    size_t smem = (size_t)NW * MT * rt_launch * 64 * 4 * sizeof(float);
    if (SMOOTH == 1 && (size_t)p.K * 4 > smem) smem = (size_t)p.K * 4;
    if (ROWS) smem = (SMOOTH == 1 ? (size_t)p.K * 4 : 0) + 2 * (size_t)(p.R / 16) * 4096;
    auto kern = quantize_fuse_lora_kernel<NW, MT, RT_MAX, DEPTH, FP4, SMOOTH, GLU, ROWS, QUANT>;
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return fail(SVDQ_ELAUNCH, "quantize: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
    }
    const int rows_per_wg = 16 * MT * (ROWS ? NW : 1);
    SVDQ_LAUNCH(kern, dim3((p.M_pad + rows_per_wg - 1) / rows_per_wg), dim3(64 * NW), smem, stream, p);
    return check_launch("quantize_w4a4_act_fuse_lora");
}

template <int NW, int MT, int RT_MAX, int DEPTH, bool FP4, bool GLU, bool ROWS = false>
int launch(const QuantParams &p, hipStream_t stream) {
    if (!p.smooth_rcp) return launch_as<NW, MT, RT_MAX, DEPTH, FP4, 0, GLU, ROWS, true>(p, stream);
    if ((size_t)p.K * 4 <= SMOOTH_LDS_MAX) return launch_as<NW, MT, RT_MAX, DEPTH, FP4, 1, GLU, ROWS, true>(p, stream);
    return launch_as<NW, MT, RT_MAX, DEPTH, FP4, 2, GLU, ROWS, true>(p, stream);
}

// the rank tiles from 8 on, 8 per launch: projection only (no smoothing factors, no codes, either precision)
template <int NW, int MT, int DEPTH, bool GLU>
int project_further(const QuantParams &p0, hipStream_t stream) {
    QuantParams p = p0;
    for (p.rt_base = 8; p.rt_base < p.R / 16; p.rt_base += 8) {
        const int rc = launch_as<NW, MT, 8, DEPTH, false, 0, GLU, false, false>(p, stream);
        if (rc != SVDQ_OK) return rc;
    }
    return SVDQ_OK;
}

template <bool FP4, bool GLU>
int dispatch(const QuantParams &p, hipStream_t stream) {
    // Rows and waves per workgroup by shape and rank, from measurements (below).
    const int RT = p.R / 16;
    // (with GLU a chunk in flight is twice the registers: one chunk ahead, 16 rows)
    if (GLU) {
        if (RT <= 2) return launch<4, 1, 2, 1, FP4, true>(p, stream);
        if (RT <= 4) return launch<4, 1, 4, 1, FP4, true>(p, stream);
        if (RT <= 8) return launch<4, 1, 8, 1, FP4, true>(p, stream);
        const int rc = launch<4, 1, 8, 1, FP4, true>(p, stream);
        return rc != SVDQ_OK ? rc : project_further<4, 1, 1, true>(p, stream);
    } else {
        int dev = 0;
        const int ncu = hipGetDevice(&dev) == hipSuccess && compute_units(dev) > 0 ? compute_units(dev) : 256;
        // High ranks with many rows: the waves split the rows (eight waves, 128 rows per workgroup) and share each chunk
        // of proj_down through LDS.  Ranks 80 ... 128, K = 3072: M = 18432 52.4 us (four waves on 32 rows each: 61.8; the
        // chunk-split forms 87 and more), M = 12288 51.3 against 58.3; below 32 rows per compute unit the chunk-split
        // form wins (M = 8192: 33.2 against 51.0).  Ranks 48 ... 64: M = 18432 41.0 against 50.7.
        if (RT > 4 && RT <= 8 && (FP4 ? p.M_pad >= 128 * 128 : p.M_pad > 32 * ncu)) return launch<8, 1, 8, 1, FP4, false, true>(p, stream);
        if (RT > 2 && RT <= 4 && p.M_pad >= 256 * 64) return launch<8, 1, 4, 1, FP4, false, true>(p, stream);
        // Up to one 16-row workgroup per compute unit (256 of them) the walk over K is what takes the time: eight waves
        // split it (M = 256 ... 4096 at K = 3072: 7.9 ... 10.1 us against 9.0 ... 11.3 with four; K = 12288, M = 256:
        // 19.6 against 25.5).
        // (two chunks requested ahead: the same at K = 3072, M = 256 and K = 12288: 16.5 us against 20.1)
        if (RT <= 2 && p.M_pad <= 16 * ncu) return launch<8, 1, 2, 2, FP4, false>(p, stream);
        // Beyond that, at ranks up to 32 (measured at K = 3072 unless noted, on 256 compute units):
        //   up to two 16-row blocks per compute unit, and long rows at any M: eight waves on 32 rows, fewer workgroups
        //   than compute units included (M = 4608: 11.5 us against 12.6 for one workgroup per compute unit with equal
        //   shares of the rows, whose partly filled second block costs its full arithmetic, and 13.3 for 288 workgroups of
        //   16 rows; K = 12288: 31.9 against 33.5 and 40.0);
        //   more rows than that with short rows: many small workgroups, four waves on 16 rows with two chunks requested
        //   ahead (M = 12288: 22.0 us against 25.3; K = 4096: 31.4 against 40.8; M = 18432: 31.5 against 35.6; equal from
        //   M = 36864 on and at K = 6144 from M = 18432 on).
        //   (NVFP4, whose quantizer is the heavier one, is better off with the small workgroups from 16 rows per compute
        //   unit on while the rows are short: M = 4608: 12.5 us against 13.4, M = 8192: 15.6 against 16.4)
        if (RT <= 2 && (p.K > 6144 || p.M_pad >= 128 * ncu || (!FP4 && p.M_pad <= 32 * ncu))) return launch<8, 2, 2, 1, FP4, false>(p, stream);
        if (RT <= 2) return launch<4, 1, 2, 2, FP4, false>(p, stream);
        // Ranks 48 ... 128 below the row counts of the rows-split form: eight waves on 32 rows (M = 4608, K = 3072: rank
        // 128 28.8 us, rank 64 16.0; four waves on the same rows 44.8 and 22.5; K = 12288, rank 128: 97 against 167);
        // with few rows (up to 8 per compute unit) many small workgroups with two chunks ahead (M = 2048, rank 128: 18.9
        // against 25.6; M = 256: 18.2 against 18.6).
        const bool few_rows = p.M_pad <= 8 * ncu;
        if (RT <= 4) return few_rows ? launch<4, 1, 4, 2, FP4, false>(p, stream) : launch<8, 2, 4, 1, FP4, false>(p, stream);
        // (NVFP4 at ranks 80 ... 128: the small workgroups at any row count, M = 4608: 29.7 us against 36.0, M = 12288: 57.7
        // against 71.1, K = 6144: 55.2 against 63.3; at rank 64 the large ones as for INT4, 16.5 against 25.1)
        if (RT <= 8) return few_rows || FP4 ? launch<4, 1, 8, 2, FP4, false>(p, stream) : launch<8, 2, 8, 1, FP4, false>(p, stream);
        // ranks above 128: the first 128 with the codes, the rest in further launches over the same rows
        if (few_rows) {
            const int rc = launch<4, 1, 8, 2, FP4, false>(p, stream);
            return rc != SVDQ_OK ? rc : project_further<4, 1, 2, false>(p, stream);
        }
        const int rc = launch<8, 2, 8, 1, FP4, false>(p, stream);
        return rc != SVDQ_OK ? rc : project_further<8, 2, 1, false>(p, stream);
    }
}

}  // namespace

extern "C" int svdq_quantize_w4a4_act_fuse_lora(const svdq_quantize_args *a, void *stream) {
    SVDQ_REQUIRE(a, "quantize: null args");
    SVDQ_REQUIRE(a->input && a->output && a->oscales, "quantize: input/output/oscales must not be null");
    SVDQ_REQUIRE(a->M > 0 && a->M_pad >= a->M && a->M_pad % 256 == 0, "quantize: M_pad (%lld) must be a multiple of 256 and >= M (%lld)",
                 (long long)a->M_pad, (long long)a->M);
    SVDQ_REQUIRE(a->K > 0 && a->K % 128 == 0, "quantize: K (%lld) must be a multiple of 128", (long long)a->K);
    SVDQ_REQUIRE(a->R >= 0 && a->R % 16 == 0 && a->R <= 1024, "quantize: rank (%lld) must be a multiple of 16, at most 1024 (lora.cuh:22)", (long long)a->R);
    SVDQ_REQUIRE(a->R == 0 || (a->lora_down && a->lora_act_out), "quantize: lora_down/lora_act_out must be given when R > 0");
    SVDQ_REQUIRE(a->M_pad < (1ll << 31) / 4 && a->K < (1 << 24) && a->K * a->R < (1ll << 30), "quantize: shape too large");
    SVDQ_REQUIRE(((uintptr_t)a->input % 16 == 0) && ((uintptr_t)a->output % 16 == 0) && ((uintptr_t)a->lora_down % 16 == 0) &&
                     ((uintptr_t)a->smooth_rcp % 16 == 0),
                 "quantize: pointers must be 16-byte aligned");
    QuantParams p;
    p.x = (const uint16_t *)a->input;
    p.act = (uint8_t *)a->output;
    p.oscales = a->oscales;
    p.down = (const bf16x8_t *)a->lora_down;
    p.lora_out = a->lora_act_out;
    p.smooth_rcp = a->smooth_rcp;
    p.M = (int)a->M; p.M_pad = (int)a->M_pad; p.K = (int)a->K; p.R = (int)a->R;
    p.rt_base = 0;
    hipStream_t s = (hipStream_t)stream;
    if (a->fuse_glu) return a->fp4 ? dispatch<true, true>(p, s) : dispatch<false, true>(p, s);
    return a->fp4 ? dispatch<true, false>(p, s) : dispatch<false, false>(p, s);
}
