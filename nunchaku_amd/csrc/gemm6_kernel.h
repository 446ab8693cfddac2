// Operator 2, INT4 operands: W4A4 GEMM with fused epilogue on the fp6 matrix instruction of gfx950.
// Counterpart of gemm_w4a4_kernel (src/kernels/zgemm/gemm_w4a4.cuh:1046-1095, main loop :831-928,
// scale application gemm_base.cuh:367-409) and of the epilogue chain composed in
// gemm_w4a4_launch_impl.cuh:172-309.
//
// How the contraction is mapped to the matrix cores
// -------------------------------------------------
//   out[m, n] = sum_g as[m, g] ws[g, n] * sum_{k in g} a[m, k] w[k, n]        (g: 64-wide k-groups)
// The inner sums are integer products of 4-bit codes.  Both operands are stored as E2M3 patterns of
// code / 8 (exact for codes -15 .. 15), so that ONE v_mfma_f32_32x32x64_f8f6f4 gives the inner sum of a
// 32 x 32 tile for one group, exactly, in fp32, at twice the rate of the INT8 matrix instruction and
// with no conversion afterwards.  The rank-1 factor as[m, g] * (64 ws[g, n]) of the same tile comes from
// a second, small matrix instruction (v_mfma_f32_32x32x8bf16_1k with a single non-zero k slot: the
// product of two bf16 numbers is exact in fp32), and one v_fmac_f32 per accumulator and group adds
// product * factor to the fp32 accumulator.  Every term is therefore the exactly dequantized product
// rounded once by the fp32 accumulation: the fp32 dequantize-then-matmul definition, in group order.
// Measured alternatives (fixed instruction streams, all compute units busy): the INT8 matrix
// instruction with conversion and scaling of its i32 result is VALU-bound at 25-33 % of the INT8
// peak; this scheme reaches 52-57 % in the bare loop, where the clock granted by the power management,
// not the issue rate, is the limit.
//
// Tiling: workgroup = 4 waves (2 x 2), block tile 128 x 256, wave tile 64 x 128 = 2 x 4 MFMA tiles;
// 128 fp32 accumulators per lane in ordinary vector registers (the fma reads them); two workgroups
// per compute unit, one tile (or one k-part of a tile) per workgroup, so that one workgroup's
// prologue / epilogue overlaps the other's main loop.  The weight fragment is the first MFMA operand:
// a lane holds one output ROW (lane % 32) and result register e is column 8 (e / 4) + 4 (lane / 32) +
// e % 4 of the 32-column tile.
//
// Staging: per k-group a workgroup needs 6 KB of activation fragments, 12 KB of weight fragments,
// 2 KB of weight scales (stored as {64 s, 0, 0, 0} bf16, the MFMA operand of the factor) and 256 bytes
// of activation scales; all are contiguous runs in memory and go global -> LDS with asynchronous
// copies (no registers, no ds_write), three stages deep.  One workgroup barrier per k-group, placed
// after the last LDS read of the group: behind it the copies of group l + 3 overwrite the stage of
// group l, and the first operands of group l + 1 are fetched, so the MFMA stream never drains at a
// group boundary.  A copy has two group times to land.
#pragma once

#include <type_traits>

#include "gemm_params.h"
#include "svdq_quant.h"

namespace svdq {
namespace g6 {

typedef int v8i_t __attribute__((ext_vector_type(8)));
typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef int v2i_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));

struct Frag {
    u32x4_t lo;  // bits [0, 128) of the lane's 192-bit code string
    u32x2_t hi;  // bits [128, 192)
};

// inner sums of one 32 x 32 tile over one k-group (elements 6 and 7 of the operand vectors are not
// read by the fp6 form of the instruction)
__device__ inline float16_t mfma_codes(const Frag &w, const Frag &x) {
    const v8i_t a = __builtin_shufflevector(__builtin_shufflevector(__builtin_bit_cast(v4i_t, w.lo), __builtin_bit_cast(v4i_t, w.lo), 0, 1, 2, 3, -1, -1, -1, -1),
                                            __builtin_shufflevector(__builtin_bit_cast(v2i_t, w.hi), __builtin_bit_cast(v2i_t, w.hi), 0, 1, -1, -1, -1, -1, -1, -1),
                                            0, 1, 2, 3, 8, 9, -1, -1);
    const v8i_t b = __builtin_shufflevector(__builtin_shufflevector(__builtin_bit_cast(v4i_t, x.lo), __builtin_bit_cast(v4i_t, x.lo), 0, 1, 2, 3, -1, -1, -1, -1),
                                            __builtin_shufflevector(__builtin_bit_cast(v2i_t, x.hi), __builtin_bit_cast(v2i_t, x.hi), 0, 1, -1, -1, -1, -1, -1, -1),
                                            0, 1, 2, 3, 8, 9, -1, -1);
    const float16_t z = {};
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, z, 2, 2, 0, 0, 0, 0);  // E2M3 x E2M3, no block scales
}

// factor tile 64 ws[n] * as[m]: the weight operand is {64 s, 0, 0, 0} in both half-waves (k slots 0-3 and
// 4-7), the activation operand carries its scale in k slot 0 and zero in k slot 4, anything finite
// elsewhere
__device__ inline float16_t mfma_factor(u32x2_t ws, uint32_t as) {
    const float16_t z = {};
    return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(bf16x4_t, ws), __builtin_bit_cast(bf16x4_t, u32x2_t{as, 0u}), z, 0, 0, 0);
}

__device__ inline float gelu_tanh(float x) {
    // x * (0.5 + 0.5 * tanh(u)), u = 0.79788456 * (x + 0.044715 x^3)   (epilogues.cuh:22-44)
    // With tanh(u) = 1 - 2 / (exp(2u) + 1) this is x - x / (exp(2u) + 1): one hardware exp2 and one hardware
    // reciprocal (1 ulp each), safe at both ends (exp2 -> inf gives x, exp2 -> 0 gives 0).
    constexpr float C1 = 2.0f * 0.79788456f * 1.4426950408889634f, C2 = C1 * 0.044715f;  // 2u * log2(e) = x (C1 + C2 x^2)
    const float w = x * __builtin_fmaf(C2, x * x, C1);
    const float r = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(w) + 1.0f);
    return __builtin_fmaf(-x, r, x);
}

// Partial sums of a tile split along K travel through memory with system-scope accesses (sc0 sc1): they
// bypass the caches that are not coherent between the XCDs, so no cache write-back or invalidation is
// needed around them, only completion (vmcnt) before the arrival counter is touched.  Layout of a slot:
// [32 quads][256 threads] x float4 (a wave's access covers 1 KB).
constexpr int PARTIAL_SC0_SC1 = 0x11;
constexpr int PARTIAL_SLOT_FLOATS = 32 * 256 * 4;
__device__ inline __amdgpu_buffer_rsrc_t partial_rsrc(const float *slot) {
    return __builtin_amdgcn_make_buffer_rsrc((void *)slot, 0, PARTIAL_SLOT_FLOATS * 4, 0x00020000);
}

template <bool NEXT>
__global__ void __launch_bounds__(256, 2) gemm6_kernel(Params p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int r32 = lane & 31, h = lane >> 5;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;

    // ---- which tile, which part of its k-groups ------------------------------------------------
    // Workgroups go to the XCDs round robin (blockIdx % 8); the remap gives each XCD one contiguous run
    // of tile numbers, and the tiles are numbered in bands of p.band row blocks (about ten), down the band
    // first: the 64 workgroups resident on an XCD at one time then cover about 10 row blocks x 6 column
    // blocks, whose operands (6 KB per row block and k-group, 14 KB per column block) they share in that
    // XCD's L2.  Measured at 36 x 48 tiles, bytes fetched from beyond the L2 per launch: bands of 6 / 9 / 12 /
    // 16 / 18 / 36 row blocks 317 / 296 / 308 / 355 / 396 / 604 MB (the time does not change: 169-171 us).
    const int mblocks = p.M_pad / BM, nblocks = (p.N + BN - 1) / BN;
    const int kgroups = p.K / 64;
    const int total = (int)gridDim.x;
    int v = (int)blockIdx.x;
    if (total % 8 == 0) v = (v % 8) * (total / 8) + v / 8;
    const int tile = v / p.kparts, part = v - tile * p.kparts;
    const int BAND = p.band;
    const int band = tile / (BAND * nblocks), in_band = tile - band * (BAND * nblocks);
    const int band_rows = mblocks - band * BAND < BAND ? mblocks - band * BAND : BAND;
    const int mb = band * BAND + in_band % band_rows, nb = in_band / band_rows;
    const int gb = (int)((long long)kgroups * part / p.kparts);
    const int ng = (int)((long long)kgroups * (part + 1) / p.kparts) - gb;
    const int m0 = mb * BM, n0 = nb * BN;

    // ---- staging ---------------------------------------------------------------------------------
    // Every wave issues COPIES_PER_WAVE copies per k-group: three consecutive 1 KB chunks of the weight
    // fragments (one base, the instruction's offset field advances both the memory and the LDS address),
    // one chunk of the activation fragments, one more of those (waves 0, 1) or of the weight scales
    // (waves 2, 3), and the 256 bytes of activation scales (all four waves write the same bytes: the
    // counts stay equal, which keeps the wait below a constant).  The four source pointers are
    // wave-uniform and advance by a constant per k-group.
    const uint32_t copy_voff = lane * 16;
    const bool low = wave < 2;
    const uint8_t *src_w = p.wgt + ((size_t)nb * kgroups + gb) * (8 * FRAG_BYTES) + wave * 3072;
    const uint8_t *src_a = p.act + ((size_t)mb * kgroups + gb) * (4 * FRAG_BYTES) + wave * 1024;
    const uint8_t *src_x = low ? p.act + ((size_t)mb * kgroups + gb) * (4 * FRAG_BYTES) + (4 + wave) * 1024
                               : p.wscales + ((size_t)nb * kgroups + gb) * 2048 + (wave - 2) * 1024;
    const uint8_t *src_q = (const uint8_t *)(p.ascales + (size_t)gb * p.M_pad + m0);
    const uint32_t stride_x = low ? 4 * FRAG_BYTES : 2048, stride_q = (uint32_t)p.M_pad * 2;
    const uint32_t dst_w = lds_base + ST_W + wave * 3072, dst_a = lds_base + ST_A + wave * 1024;
    const uint32_t dst_x = lds_base + (low ? ST_A + (4 + wave) * 1024 : ST_WS + (wave - 2) * 1024), dst_q = lds_base + ST_AS;
    // The requests of a k-group are issued one at a time, spread over the steps of the main loop: a wave
    // that issues its six requests back to back stands still until the memory pipeline has taken them,
    // about 30 cycles each.  First the three weight chunks (W), later the other three (R).
    auto copy_w = [&](uint32_t stage_off, int i) {  // weight chunk i of the next k-group whose weights are not requested yet
        if (i == 0) asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3" :: "s"(dst_w), "s"(stage_off), "v"(copy_voff), "s"(src_w) : "memory", "m0", "scc");
        if (i == 1) asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3 offset:1024" :: "s"(dst_w), "s"(stage_off), "v"(copy_voff), "s"(src_w) : "memory", "m0", "scc");
        if (i == 2) {
            asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3 offset:2048" :: "s"(dst_w), "s"(stage_off), "v"(copy_voff), "s"(src_w) : "memory", "m0", "scc");
            src_w += 8 * FRAG_BYTES;
        }
    };
    auto copy_r = [&](uint32_t stage_off, int i) {  // the rest: activation chunk, activation / weight-scale chunk, activation scales
        if (i == 0) asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3" :: "s"(dst_a), "s"(stage_off), "v"(copy_voff), "s"(src_a) : "memory", "m0", "scc");
        if (i == 1) asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3" :: "s"(dst_x), "s"(stage_off), "v"(copy_voff), "s"(src_x) : "memory", "m0", "scc");
        if (i == 2) {
            uint32_t voff4;
            asm volatile("v_lshrrev_b32 %0, 2, %1" : "=v"(voff4) : "v"(copy_voff));
            asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %2, %3" :: "s"(dst_q), "s"(stage_off), "v"(voff4), "s"(src_q) : "memory", "m0", "scc");
            src_a += 4 * FRAG_BYTES;
            src_x += stride_x;
            src_q += stride_q;
        }
    };

    // what the upper half-wave reads as its activation scale
    if (tid < STAGES * 32) *(uint32_t *)(lds + (tid >> 5) * STAGE_BYTES + ST_Z + (tid & 31) * 4) = 0u;

    // groups 0 and 1 entirely, the weights of group 2
    for (int i = 0; i < 3; i++) copy_w(0, i);
    for (int i = 0; i < 3; i++) copy_r(0, i);
    if (ng > 1) {
        for (int i = 0; i < 3; i++) copy_w(STAGE_BYTES, i);
        for (int i = 0; i < 3; i++) copy_r(STAGE_BYTES, i);
    }
    if (ng > 2)
        for (int i = 0; i < 3; i++) copy_w(2 * STAGE_BYTES, i);

    // per-lane read offsets inside a stage
    const uint32_t off16 = lane * 16, off8 = 1024 + lane * 8;
    const uint32_t off_ws = ST_WS + (128 * wn + r32) * 8;
    const uint32_t off_as = h ? ST_Z : ST_AS + (64 * wm + r32) * 2;
    auto read_x = [&](uint32_t sb, int mt, Frag &f, uint32_t &as) {
        const uint8_t *base = lds + sb + ST_A + (2 * wm + mt) * FRAG_BYTES;
        f.lo = *(const u32x4_t *)(base + off16);
        f.hi = *(const u32x2_t *)(base + off8);
        as = *(const uint16_t *)(lds + sb + off_as + mt * 64);
    };
    auto read_w = [&](uint32_t sb, int nt, Frag &f, u32x2_t &ws) {
        const uint8_t *base = lds + sb + ST_W + (4 * wn + nt) * FRAG_BYTES;
        f.lo = *(const u32x4_t *)(base + off16);
        f.hi = *(const u32x2_t *)(base + off8);
        ws = *(const u32x2_t *)(lds + sb + off_ws + nt * 256);
    };

    float16_t acc[8];  // tile t = 2 nt + mt
#pragma unroll
    for (int t = 0; t < 8; t++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[t][e] = 0.f;

    // group 0 has landed
    if (ng > 2) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
    else if (ng > 1) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    Frag X[2], W[2];
    u32x2_t wsop[2];
    uint32_t asop[2];
    float16_t P[2], F[2];
    read_x(0, 0, X[0], asop[0]);
    read_x(0, 1, X[1], asop[1]);
    read_w(0, 0, W[0], wsop[0]);
    P[0] = mfma_codes(W[0], X[0]);
    F[0] = mfma_factor(wsop[0], asop[0]);

#define SVDQ_FMA(T, B)                                                                                   \
    _Pragma("unroll") for (int e = 0; e < 16; e++) acc[T][e] = __builtin_fmaf(P[B][e], F[B][e], acc[T][e]);
    // One step: the two matrix instructions of the NEXT tile (into buffer BN) are issued, the LDS reads
    // that refill dead operand registers follow, and the previous tile (buffer BC) is accumulated with
    // its 16 fma interleaved between the matrix instructions.  The scheduling fences pin that order: left
    // alone, the scheduler gathers the matrix instructions of several steps, which keeps all their
    // result tiles alive and spills.
#define SVDQ_STEP(T, BC, BN, WF, XF, WSO, ASO, NREADS, READS)                                            \
    P[BN] = mfma_codes(WF, XF);                                                                          \
    F[BN] = mfma_factor(WSO, ASO);                                                                       \
    READS;                                                                                               \
    SVDQ_FMA(T, BC)                                                                                      \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                                   \
    if (NREADS) __builtin_amdgcn_sched_group_barrier(0x100, NREADS, 0);                                  \
    __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);                                                   \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                                   \
    __builtin_amdgcn_sched_group_barrier(0x002, 9, 0);                                                   \
    __builtin_amdgcn_sched_barrier(0);

    uint32_t sb = 0;  // byte offset of the stage of group l
    // The loop body is one basic block (a branch inside it lets the compiler sink the fma of all steps
    // below the branch, with all their operands alive).  Requests of iteration l: in steps 0-2 the rest of
    // group l + 2 (its stage, that of group l - 1, was free since the previous barrier and already
    // received the weights), in steps 5-7, behind the barrier, the weights of group l + 3 into the stage
    // of group l.  At the barrier group l + 1 must have landed; the six requests of group l + 2 are the
    // only ones issued after it.  MODE 2: both (l + 3 < ng), 1: only the rest of group l + 2 (l = ng - 3),
    // 0: nothing left to request.
    auto group_body = [&](auto MODE_T) {
        constexpr int MODE = decltype(MODE_T)::value;
        const uint32_t sb_next = sb == (STAGES - 1) * STAGE_BYTES ? 0 : sb + STAGE_BYTES;
        const uint32_t sb_prev = sb == 0 ? (STAGES - 1) * STAGE_BYTES : sb - STAGE_BYTES;
        // step t issues the matrix instructions of tile t + 1 (tile = 2 nt + mt) and accumulates tile t
        if (MODE >= 1) copy_r(sb_prev, 0);
        SVDQ_STEP(0, 0, 1, W[0], X[1], wsop[0], asop[1], 3, read_w(sb, 1, W[1], wsop[1]))
        if (MODE >= 1) copy_r(sb_prev, 1);
        SVDQ_STEP(1, 1, 0, W[1], X[0], wsop[1], asop[0], 0, )
        if (MODE >= 1) copy_r(sb_prev, 2);
        SVDQ_STEP(2, 0, 1, W[1], X[1], wsop[1], asop[1], 3, read_w(sb, 2, W[0], wsop[0]))
        SVDQ_STEP(3, 1, 0, W[0], X[0], wsop[0], asop[0], 0, )
        SVDQ_STEP(4, 0, 1, W[0], X[1], wsop[0], asop[1], 3, read_w(sb, 3, W[1], wsop[1]))
        P[0] = mfma_codes(W[1], X[0]);
        F[0] = mfma_factor(wsop[1], asop[0]);
        __builtin_amdgcn_sched_barrier(0);
        // Every LDS read of this group has been issued, and the last one has arrived (the instruction
        // above needed it).  Behind the barrier the stage may be overwritten, and the next group's
        // stage, whose copies every wave has waited for, may be read.
        if (MODE >= 1) asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (MODE == 2) copy_w(sb, 0);
        read_x(sb_next, 0, X[0], asop[0]);
        read_w(sb_next, 0, W[0], wsop[0]);
        SVDQ_FMA(5, 1)
        __builtin_amdgcn_sched_barrier(0);
        if (MODE == 2) copy_w(sb, 1);
        SVDQ_STEP(6, 0, 1, W[1], X[1], wsop[1], asop[1], 3, read_x(sb_next, 1, X[1], asop[1]))
        if (MODE == 2) copy_w(sb, 2);
        // (tile 0 of the next group; of nothing after the last group)
        SVDQ_STEP(7, 1, 0, W[0], X[0], wsop[0], asop[0], 0, )
        sb = sb_next;
    };
    int l = 0;
    for (; l + 3 < ng; l++) group_body(std::integral_constant<int, 2>{});
    if (l + 2 < ng) {
        group_body(std::integral_constant<int, 1>{});
        l++;
    }
    for (; l < ng; l++) group_body(std::integral_constant<int, 0>{});
#undef SVDQ_STEP
#undef SVDQ_FMA
    __syncthreads();  // the ring is free: the epilogue reuses it

    // ---- a tile split along K --------------------------------------------------------------------
    // Every part parks its sums in its slot of the workspace; whoever arrives last adds all parts in
    // ascending order, so the result does not depend on who that is, and runs the epilogue.  Nobody waits for
    // anybody.
    if (p.kparts > 1) {
        float *slot = p.partials + ((size_t)tile * p.kparts + part) * PARTIAL_SLOT_FLOATS;
        const __amdgpu_buffer_rsrc_t mine = partial_rsrc(slot);
#pragma unroll
        for (int t = 0; t < 8; t++)
#pragma unroll
            for (int q = 0; q < 4; q++)
                __builtin_amdgcn_raw_buffer_store_b128(
                    __builtin_bit_cast(u32x4_t, float4_t{acc[t][4 * q], acc[t][4 * q + 1], acc[t][4 * q + 2], acc[t][4 * q + 3]}), mine,
                    ((t * 4 + q) * 256 + tid) * 16, 0, PARTIAL_SC0_SC1);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the parked sums are in memory before the counter says so
        __syncthreads();
        int *flag = (int *)(lds + EP_FLAG);
        if (tid == 0) *flag = __hip_atomic_fetch_add(p.counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        const bool last = *flag == p.kparts - 1;
        if (!last) return;
        if (tid == 0) __hip_atomic_store(p.counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
        // Four parts (what the launcher chooses for the fewest tiles): the last one keeps its own sums in its registers
        // and fetches only the others'.  The sum (((0 + s0) + s1) + s2) + s3 is evaluated in exactly that order whoever
        // is last: the parts before its own are added up first (from zero), then its own joins (a single addition gives
        // the same result with its operands exchanged), then the parts after it.  Written without branches: a part on
        // the wrong side of the own contributes +0, which changes nothing because no sum here is ever -0.  (One form
        // only: with a form per number of parts the compiler carries the 128 accumulators through the alternatives by
        // way of scratch memory; with two or three parts the general form below is as fast.)
        if (p.kparts == 4) {
            constexpr int NOTH = 3;  // the other parts, j-th of them in ascending order: part j + (j >= own)
            __amdgpu_buffer_rsrc_t r[NOTH];
#pragma unroll
            for (int j = 0; j < NOTH; j++) r[j] = partial_rsrc(p.partials + ((size_t)tile * 4 + j + (j >= part ? 1 : 0)) * PARTIAL_SLOT_FLOATS);
            // (items of half a 32 x 32 block: 8 accumulators per lane and part; a ring of three, two in flight)
            float4_t o[3][NOTH][2];
            auto request = [&](int i) {
#pragma unroll
                for (int j = 0; j < NOTH; j++)
#pragma unroll
                    for (int q = 0; q < 2; q++)
                        o[i % 3][j][q] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(r[j], ((i * 2 + q) * 256 + tid) * 16, 0, PARTIAL_SC0_SC1));
            };
            request(0);
            request(1);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                if (i + 2 < 16) request(i + 2);
                const int t = i >> 1, e0 = (i & 1) * 8;
                float before[8];
#pragma unroll
                for (int e = 0; e < 8; e++) before[e] = 0.f;
#pragma unroll
                for (int j = 0; j < NOTH; j++)
#pragma unroll
                    for (int e = 0; e < 8; e++) before[e] += j < part ? o[i % 3][j][e / 4][e % 4] : 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) acc[t][e0 + e] = before[e] + acc[t][e0 + e];
#pragma unroll
                for (int j = 0; j < NOTH; j++)
#pragma unroll
                    for (int e = 0; e < 8; e++) acc[t][e0 + e] += j >= part ? o[i % 3][j][e / 4][e % 4] : 0.f;
            }
        } else {
            // any other number of parts: all of them from memory, the own included (a running sum of the parts before
            // the own would need a second set of accumulators beyond four parts), two parts at a time, the requests of the next eighth of the tile in
            // flight while one is added; every element still adds its parts in ascending order
#pragma unroll
            for (int t = 0; t < 8; t++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[t][e] = 0.f;
            for (int pt0 = 0; pt0 < p.kparts; pt0 += 2) {
                const bool two = pt0 + 1 < p.kparts;
                const __amdgpu_buffer_rsrc_t r0 = partial_rsrc(p.partials + ((size_t)tile * p.kparts + pt0) * PARTIAL_SLOT_FLOATS);
                const __amdgpu_buffer_rsrc_t r1 = partial_rsrc(p.partials + ((size_t)tile * p.kparts + (two ? pt0 + 1 : pt0)) * PARTIAL_SLOT_FLOATS);
                float4_t o[2][2][4];
                auto request = [&](int t, int b) {
#pragma unroll
                    for (int q = 0; q < 4; q++) o[b][0][q] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(r0, ((t * 4 + q) * 256 + tid) * 16, 0, PARTIAL_SC0_SC1));
                    if (two) {
#pragma unroll
                        for (int q = 0; q < 4; q++) o[b][1][q] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(r1, ((t * 4 + q) * 256 + tid) * 16, 0, PARTIAL_SC0_SC1));
                    }
                };
                request(0, 0);
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    if (t + 1 < 8) request(t + 1, (t + 1) & 1);
#pragma unroll
                    for (int e = 0; e < 16; e++) acc[t][e] += o[t & 1][0][e / 4][e % 4];
                    if (two) {
#pragma unroll
                        for (int e = 0; e < 16; e++) acc[t][e] += o[t & 1][1][e / 4][e % 4];
                    }
                }
            }
        }
    }

    // ---- epilogue --------------------------------------------------------------------------------
    const int wrow0 = m0 + wm * 64, wcol0 = n0 + wn * 128;
    // per-column factor (alpha and wcscales; EpilogueBias, gemm_base.cuh:710-781) and bias of the
    // workgroup's 256 columns
    float *coltab = (float *)(lds + EP_TAB);
    const bool has_cf = p.alpha != 1.0f || p.wcscales != nullptr;
    {
        const int n = n0 + tid;
        const bool ok = n < p.N;
        float cf = p.alpha;
        if (ok && p.wcscales) cf *= bf16_bits_to_f32(p.wcscales[n]);
        coltab[tid] = cf;
        coltab[256 + tid] = (ok && p.bias) ? bf16_bits_to_f32(p.bias[n]) : 0.f;
        if (NEXT && p.next_down && p.R_down <= 32) {
            // the next layer's proj_down for the tile's 256 columns (two 128-chunks, 4 KB per rank tile each,
            // contiguous in memory) goes to LDS once: both row halves and both slabs read it from there
            const int npieces = 8 * (p.R_down / 16);
            for (int pc = wave; pc < npieces; pc += 4) {
                if (n0 + (pc / (npieces / 2)) * 128 < p.N)
                    *(u32x4_t *)(lds + EP_DOWN + pc * 1024 + lane * 16) =
                        *(const u32x4_t *)((const uint8_t *)p.next_down + ((size_t)(n0 / 128) * (npieces / 2) + pc) * 1024 + lane * 16);
            }
        }
        if (NEXT && p.rotary && tid < 128) {
            // RMS-norm weights of the heads the two column halves are (q below N/3, k below 2N/3)
            ((float *)(lds + EP_NORMW))[tid] = bf16_bits_to_f32((n0 < p.rope_cols / 2 ? p.norm_q : p.norm_k)[tid]);
            ((float *)(lds + EP_NORMW))[128 + tid] = bf16_bits_to_f32((n0 + 128 < p.rope_cols / 2 ? p.norm_q : p.norm_k)[tid]);
        }
    }
    __syncthreads();
    const float *cfw = coltab + wn * 128, *bsw = coltab + 256 + wn * 128;
    if (has_cf) {  // the main term alone carries alpha and the per-channel scales (the low-rank term does not)
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4_t cf = *(const float4_t *)(cfw + nt * 32 + 8 * q + 4 * h);
#pragma unroll
                for (int mt = 0; mt < 2; mt++)
#pragma unroll
                    for (int i = 0; i < 4; i++) acc[2 * nt + mt][4 * q + i] *= cf[i];
            }
    }
    // Low-rank up projection (lora.cuh:110-241): out += bf16(lora_act * scale) @ up^T on the matrix
    // cores, straight into the accumulators.  Two 16-rank steps per round; every request of a round is
    // issued before any of its data is touched, so a round costs one memory latency.
    const int nsteps = p.R_up / 16;
    for (int s0 = 0; s0 < nsteps; s0 += 2) {
        const bool two = s0 + 1 < nsteps;
        const int s1 = two ? s0 + 1 : s0;
        float4_t ra[2][2][2];
        u32x4_t rb[4][2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const float4_t *ap = (const float4_t *)(p.lora_act + (size_t)(wrow0 + t * 32 + r32) * p.R_up + 8 * h);
            ra[t][0][0] = ap[4 * s0]; ra[t][0][1] = ap[4 * s0 + 1];
            ra[t][1][0] = ap[4 * s1]; ra[t][1][1] = ap[4 * s1 + 1];
        }
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int n = wcol0 + t * 32 + r32;
            const u32x4_t *bp = (const u32x4_t *)(p.lora_up + (size_t)(n < p.N ? n : 0) * p.R_up + 8 * h);
            rb[t][0] = bp[2 * s0];
            rb[t][1] = bp[2 * s1];
            if (n >= p.N) rb[t][0] = rb[t][1] = u32x4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int k = 0; k < 2; k++) {
            if (k == 1 && !two) break;
            const float ls = p.lora_scales[s0 + k];
            bf16x8_t la[2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const float4_t v0 = ra[t][k][0], v1 = ra[t][k][1];
                u32x4_t w;
                w[0] = pack_bf16x2(v0[0] * ls, v0[1] * ls);
                w[1] = pack_bf16x2(v0[2] * ls, v0[3] * ls);
                w[2] = pack_bf16x2(v1[0] * ls, v1[1] * ls);
                w[3] = pack_bf16x2(v1[2] * ls, v1[3] * ls);
                la[t] = __builtin_bit_cast(bf16x8_t, w);
            }
#pragma unroll
            for (int nt = 0; nt < 4; nt++)
#pragma unroll
                for (int mt = 0; mt < 2; mt++)
                    acc[2 * nt + mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, rb[nt][k]), la[mt], acc[2 * nt + mt], 0, 0, 0);
        }
    }

    // reciprocal smoothing factors of the next layer for the 32 columns this lane quantizes
    // (work item of the quantizing pass: row = item / 4, 32-column quarter = item % 4 = lane % 4)
    float nrs[32];
    if (NEXT && p.qout) {
        const float4_t *sp = (const float4_t *)(p.next_smooth_rcp + (wcol0 < p.N ? wcol0 : 0) + (lane & 3) * 32);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float4_t v4 = sp[i];
            nrs[4 * i] = v4[0]; nrs[4 * i + 1] = v4[1]; nrs[4 * i + 2] = v4[2]; nrs[4 * i + 3] = v4[3];
        }
    }
    const bool down_in_lds = NEXT && p.next_down && p.R_down <= 32;
    const bool interior = m0 + BM <= p.M_out && n0 + BN <= p.N_out;  // the whole tile lies inside the output
    uint16_t *slab = (uint16_t *)(lds + wave * SLAB_BYTES);
    const int ngroups_out = p.N / 64;
    VkSums vks;  // linear attention: the sums of the wave's two slabs
    if (NEXT && p.vk) litela_clear(vks);
    // next layer's low-rank projection at ranks up to 32: [slab][rank tile][16-row half] sums of the wave's 128 columns,
    // kept until both slabs are done so that the column halves meet once per tile
    float4_t down_sums[2][2][2];
    const bool down_once = NEXT && p.next_down && p.R_down <= 32;
    // one 32-row slab of the wave tile, instantiated twice with a compile-time slab index
    auto slab_epilogue = [&](auto MT) {
        constexpr int mt = decltype(MT)::value;
        float16_t v[4];
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4_t bs = *(const float4_t *)(bsw + nt * 32 + 8 * q + 4 * h);
#pragma unroll
                for (int i = 0; i < 4; i++) v[nt][4 * q + i] = acc[2 * nt + mt][4 * q + i] + bs[i];
            }
        if (NEXT && p.rotary && wcol0 < p.rope_cols) {
            // EpilogueRMSNormRope (epilogues.cuh:269-425): the wave's 128 columns are one head of q or k.
            // The lane holds 64 values of its row, lane ^ 32 the other 64.  The (sin, cos) table is stored in
            // this loop's order ([32-row block][nt][q][lane] x float4: a wave-wide request is 1 KB
            // contiguous), requested two column tiles ahead.
            int blk = (wrow0 + mt * 32) >> 5;
            blk = blk < (p.rot_rows >> 5) ? blk : (p.rot_rows >> 5) - 1;  // (rows beyond the output are never stored)
            const float4_t *rp = (const float4_t *)p.rotary + (size_t)blk * (16 * 64) + lane;
            const float *normw = (const float *)(lds + EP_NORMW) + wn * 128;
            float4_t sc[2][4];
#pragma unroll
            for (int nt = 0; nt < 2; nt++)
#pragma unroll
                for (int q = 0; q < 4; q++) sc[nt][q] = rp[(nt * 4 + q) * 64];
            float ss = 0.f;
#pragma unroll
            for (int nt = 0; nt < 4; nt++)
#pragma unroll
                for (int e = 0; e < 16; e++) ss += v[nt][e] * v[nt][e];
            ss += __shfl_xor(ss, 32);
            const float coef = __builtin_amdgcn_rsqf(ss * (1.0f / 128.0f) + p.norm_eps);
#pragma unroll
            for (int nt = 0; nt < 4; nt++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float4_t w4 = *(const float4_t *)(normw + nt * 32 + 8 * q + 4 * h);
                    const float4_t s4 = sc[nt & 1][q];  // sin, cos of the two pairs
#pragma unroll
                    for (int pr = 0; pr < 2; pr++) {
                        const float x = v[nt][4 * q + 2 * pr] * (coef * w4[2 * pr]);
                        const float y = v[nt][4 * q + 2 * pr + 1] * (coef * w4[2 * pr + 1]);
                        const float sn = s4[2 * pr], cs = s4[2 * pr + 1];
                        v[nt][4 * q + 2 * pr] = x * cs - y * sn;
                        v[nt][4 * q + 2 * pr + 1] = x * sn + y * cs;
                    }
                }
                if (nt < 2) {
#pragma unroll
                    for (int q = 0; q < 4; q++) sc[nt & 1][q] = rp[((nt + 2) * 4 + q) * 64];
                }
            }
        }
        if (NEXT && p.silu) {
            // EpilogueSilu (gemm_base.cuh:783-792, gemm_utils.cuh:322-327): x * sigmoid(x) = x / (1 + exp(-x))
#pragma unroll
            for (int nt = 0; nt < 4; nt++)
#pragma unroll
                for (int e = 0; e < 16; e++)
                    v[nt][e] = v[nt][e] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v[nt][e]));
        }
        if (NEXT && p.gelu) {
#pragma unroll
            for (int nt = 0; nt < 4; nt++)
#pragma unroll
                for (int e = 0; e < 16; e++) v[nt][e] = gelu_tanh(v[nt][e]);
        }
        if (NEXT && p.vk && wcol0 < p.N / 3) {
            // the q third of a linear-attention projection is stored after a ReLU (epilogues.cuh:662-674)
#pragma unroll
            for (int nt = 0; nt < 4; nt++)
#pragma unroll
                for (int e = 0; e < 16; e++) v[nt][e] = __builtin_fmaxf(v[nt][e], 0.f);
        }
        // bf16 tile -> per-wave LDS slab (32 rows x 128 columns), four columns per write: every later
        // consumer reads whole rows
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                u32x2_t w;
                w[0] = pack_bf16x2(v[nt][4 * q], v[nt][4 * q + 1]);
                w[1] = pack_bf16x2(v[nt][4 * q + 2], v[nt][4 * q + 3]);
                *(u32x2_t *)(slab + r32 * OUT_LD + nt * 32 + 8 * q + 4 * h) = w;
            }
        // the slab is private to this wave: LDS operations of one wave complete in order, so only the
        // compiler has to be kept from reordering across this point
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        // EpilogueDefault (gemm_base.cuh:667-698): 16-byte row-contiguous stores.  Streaming stores: the
        // tile is not read again by this kernel.
        if (NEXT && p.vk && wcol0 >= p.N / 3 && wcol0 < p.N) litela_add_slab(vks, slab, OUT_LD, lane);
        if (NEXT && p.qkv.q && wcol0 < p.N) store_qkv_slab(p.qkv, slab, OUT_LD, lane, wrow0 + mt * 32, wcol0, p.N / 3);
        if (p.out && interior) {  // no bounds to check: all slab reads first, then all stores
            u32x4_t d[8];
#pragma unroll
            for (int pass = 0; pass < 8; pass++) d[pass] = *(const u32x4_t *)(slab + (pass * 4 + (lane >> 4)) * OUT_LD + (lane & 15) * 8);
            uint16_t *gp = p.out + (size_t)(wrow0 + mt * 32 + (lane >> 4)) * p.N_out + wcol0 + (lane & 15) * 8;
#pragma unroll
            for (int pass = 0; pass < 8; pass++) __builtin_nontemporal_store(d[pass], (u32x4_t *)(gp + (size_t)(pass * 4) * p.N_out));
        } else if (p.out) {
#pragma unroll
            for (int pass = 0; pass < 8; pass++) {
                const int rr = pass * 4 + (lane >> 4), cc = (lane & 15) * 8;
                const int m = wrow0 + mt * 32 + rr, n = wcol0 + cc;
                if (m < p.M_out && n < p.N_out)
                    __builtin_nontemporal_store(*(const u32x4_t *)(slab + rr * OUT_LD + cc), (u32x4_t *)(p.out + (size_t)m * p.N_out + n));
            }
        }
        if (NEXT && p.next_down) {
            // Low-rank down projection of the next layer on the bf16 tile (EpilogueLoraDown,
            // lora.cuh:243-353): this wave's 128 columns are one 128-chunk of the next layer's K.  The two
            // column halves of the workgroup meet in LDS (leaving that out and storing a share per half bought
            // nothing); the sum goes to the workgroup's slot of the
            // workspace, in the lanes' own order (a wave's store is 1 KB contiguous), and a small kernel launched
            // behind this one adds the slots of all column blocks in ascending order (reduce_shares_kernel in
            // gemm.hip): the same result from run to run, and this kernel never waits for its own stores.  (The
            // reference adds with fp32 atomics in the order of arrival, lora.cuh:82-94.  Adding up inside this
            // kernel, by whoever brings a row block's last share, needs every workgroup to wait until all its
            // stores, the 64 KB of output included, have been acknowledged before it can say so: that wait cost
            // 28 us at M = 4608, N = 12288, with atomics and with parked shares alike.)
            const int RT = p.R_down / 16;
            const int r16 = lane & 15, q = lane >> 4;
            float *red = (float *)(lds + EP_RED);  // [rank tile of the pair][row half][m2][64 lanes] x float4
            const __amdgpu_buffer_rsrc_t slot = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(p.next_lora_part + ((size_t)nb * (p.M_pad / BM) + mb) * (size_t)(BM * p.R_down)), 0, BM * p.R_down * 4, 0x00020000);
            for (int rt0 = 0; rt0 < RT; rt0 += 2) {
                float4_t d[2][2];
#pragma unroll
                for (int g = 0; g < 2; g++) {
                    d[g][0] = d[g][1] = float4_t{0.f, 0.f, 0.f, 0.f};
                    const int rt = rt0 + g;
                    if (rt < RT && wcol0 < p.N) {
                        bf16x8_t b[4];
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            if (down_in_lds) b[i] = *(const bf16x8_t *)(lds + EP_DOWN + (((wn * 4 + i) * RT + rt) * 64 + lane) * 16);
                            else b[i] = p.next_down[((size_t)((wcol0 / 128) * 4 + i) * RT + rt) * 64 + lane];
                        }
#pragma unroll
                        for (int i = 0; i < 4; i++) {
#pragma unroll
                            for (int m2 = 0; m2 < 2; m2++) {
                                const bf16x8_t a = *(const bf16x8_t *)(slab + (16 * m2 + r16) * OUT_LD + 32 * q + 8 * i);
                                d[g][m2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[i], d[g][m2], 0, 0, 0);
                            }
                        }
                    }
                }
                if (down_once) {  // (one pair of rank tiles at most)
#pragma unroll
                    for (int g = 0; g < 2; g++)
#pragma unroll
                        for (int m2 = 0; m2 < 2; m2++) down_sums[mt][g][m2] = d[g][m2];
                    break;
                }
                if (wn == 1) {
#pragma unroll
                    for (int g = 0; g < 2; g++)
#pragma unroll
                        for (int m2 = 0; m2 < 2; m2++) *(float4_t *)(red + (((g * 2 + wm) * 2 + m2) * 64 + lane) * 4) = d[g][m2];
                }
                __syncthreads();
                if (wn == 0) {
#pragma unroll
                    for (int g = 0; g < 2; g++)
#pragma unroll
                        for (int m2 = 0; m2 < 2; m2++) {
                            if (rt0 + g >= RT) continue;
                            const float4_t o = *(const float4_t *)(red + (((g * 2 + wm) * 2 + m2) * 64 + lane) * 4);
                            const float4_t sum = float4_t{d[g][m2][0] + o[0], d[g][m2][1] + o[1], d[g][m2][2] + o[2], d[g][m2][3] + o[3]};
                            // share layout [32-row slab][rank tile][m2][64 lanes] x float4; this workgroup's slabs are 4 mb + 2 wm + mt
                            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, sum), slot,
                                                                   (((((wm * 2 + mt) * RT + rt0 + g) * 2 + m2) * 64) + lane) * 16, 0, 0);
                        }
                }
                __syncthreads();
            }
        }
        if (NEXT && p.qout && wcol0 < p.N) {
            // EpilogueQuantize (gemm_w4a4.cuh:930-1043): shift, smooth, quantize for the next layer
            // (unsigned codes after a +0.171875 shift, launch_impl.cuh:286-294)
#pragma unroll
            for (int pass = 0; pass < 2; pass++) {
                const int item = pass * 64 + lane;
                const int rr = item >> 2, qc = item & 3;
                const u32x4_t *sp = (const u32x4_t *)(slab + rr * OUT_LD + qc * 32);
                float y[32];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const u32x4_t v4 = sp[i];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        float lo = bits_f32(v4[j] << 16), hi = bits_f32(v4[j] & 0xFFFF0000u);
                        lo = bf16_bits_to_f32(f32_to_bf16_bits(__fadd_rn(lo, 0.171875f)));
                        hi = bf16_bits_to_f32(f32_to_bf16_bits(__fadd_rn(hi, 0.171875f)));
                        y[8 * i + 2 * j] = smooth_quotient(lo, nrs[8 * i + 2 * j]);
                        y[8 * i + 2 * j + 1] = smooth_quotient(hi, nrs[8 * i + 2 * j + 1]);
                    }
                }
                const int m = wrow0 + mt * 32 + rr;
                const int gidx = (wcol0 + qc * 32) / 64;
                u32x4_t lo4;
                u32x2_t hi2;
                float sc;
                quantize_int4_half_group_e2m3<true>(y, 1, lo4, hi2, sc);
                if ((qc & 1) == 0) p.oscales[(size_t)gidx * p.M_pad + m] = (uint16_t)f32_to_bf16_bits(sc);
                uint8_t *frag = p.qout + (((size_t)(m / ACT_BLOCK_ROWS) * ngroups_out + gidx) * 4 + (m % ACT_BLOCK_ROWS) / 32) * FRAG_BYTES;
                const int slot = (m % 32) + 32 * (qc & 1);
                *(u32x4_t *)(frag + slot * 16) = lo4;
                *(u32x2_t *)(frag + 1024 + slot * 8) = hi2;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_sched_barrier(0);  // keep the slabs apart: hoisting the next slab's work multiplies live registers
    };
    __builtin_amdgcn_sched_barrier(0);
    slab_epilogue(std::integral_constant<int, 0>{});
    slab_epilogue(std::integral_constant<int, 1>{});
    if (down_once) {
        // the right column half hands its sums over through its own slab area, which it no longer needs; the left
        // one adds and stores the workgroup's share: [32-row slab 2 wm + mt][rank tile][16-row half][64 lanes] x float4
        static_assert(SLAB_BYTES >= 2 * 2 * 2 * 64 * 16, "a wave's sums pass through its slab area");
        const int RT = p.R_down / 16;
        float4_t *xchg = (float4_t *)(lds + (2 * wm + 1) * SLAB_BYTES);
        if (wn == 1) {
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int g = 0; g < 2; g++)
#pragma unroll
                    for (int m2 = 0; m2 < 2; m2++) xchg[((mt * 2 + g) * 2 + m2) * 64 + lane] = down_sums[mt][g][m2];
        }
        __syncthreads();
        if (wn == 0) {
            const __amdgpu_buffer_rsrc_t slot = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(p.next_lora_part + ((size_t)nb * (p.M_pad / BM) + mb) * (size_t)(BM * p.R_down)), 0, BM * p.R_down * 4, 0x00020000);
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int g = 0; g < 2; g++) {
                    if (g >= RT) continue;
#pragma unroll
                    for (int m2 = 0; m2 < 2; m2++) {
                        const float4_t o = xchg[((mt * 2 + g) * 2 + m2) * 64 + lane], d = down_sums[mt][g][m2];
                        const float4_t sum = float4_t{d[0] + o[0], d[1] + o[1], d[2] + o[2], d[3] + o[3]};
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, sum), slot,
                                                               (((((wm * 2 + mt) * RT + g) * 2 + m2) * 64) + lane) * 16, 0, 0);
                    }
                }
        }
    }
    if (NEXT && p.vk && n0 + BN > p.N / 3) {
        static_assert(SLAB_BYTES >= 2 * VK_HEAD_FLOATS * 4, "a wave's two heads pass through its slab area");
        const int third = p.N / 3;
        litela_finish(vks, wcol0 >= third && wcol0 < p.N, wm, wn, lds, SLAB_BYTES,
                      p.vk_part + ((size_t)mb * (2 * third / 64) + (wcol0 - third) / 64) * VK_HEAD_FLOATS, lane);
    }
}

template <bool NEXT>
int launch_gemm6(const Params &p, int nwg, hipStream_t stream) {
    auto kern = gemm6_kernel<NEXT>;
    // the attribute is set once per device (racing first calls both set it, which is harmless)
    static bool lds_reserved[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(SVDQ_ELAUNCH, "gemm: cannot identify the current device");
    if (!lds_reserved[dev]) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        if (e != hipSuccess) return fail(SVDQ_ELAUNCH, "gemm: cannot reserve %d bytes of LDS: %s", LDS_BYTES, hipGetErrorString(e));
        lds_reserved[dev] = true;
    }
    SVDQ_LAUNCH(kern, dim3(nwg), dim3(256), LDS_BYTES, stream, p);
    return check_launch("gemm_w4a4");
}

}  // namespace g6
}  // namespace svdq
