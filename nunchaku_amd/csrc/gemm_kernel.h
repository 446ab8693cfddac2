// Operator 2, NVFP4 operands: W4A4 GEMM with fused epilogue for gfx950.  Counterpart of
// gemm_w4a4_fp4_kernel (src/kernels/zgemm/gemm_w4a4.cuh:273-405) and of the epilogue chain composed in
// gemm_w4a4_launch_impl.cuh:172-309.  (INT4 operands take gemm6_kernel.h.)
//
// How the contraction is mapped to the matrix cores
// -------------------------------------------------
// Every 16-wide k-group carries its own activation scale (per row, E4M3) and weight scale (per column,
// E4M3).  The block-scaled fp4 matrix instruction takes power-of-two scales per 32 elements only, so
// both operands are dequantized to fp16 -- (code) * (scale) is exact in fp16: an E2M1 code has 2
// significant bits and an E4M3 scale 4 -- and fed to v_mfma_f32_32x32x16_f16 with fp32 accumulation.
// The result equals the fp32 dequantize-then-matmul definition up to fp32 summation order; no
// per-group post-scaling exists.
//
// Every element is dequantized ONCE per workgroup: thread t owns row m0 + t of the tile's activations
// and column n0 + t of its weights, fetches their codes and scales of a k-group into registers, converts
// them (the hardware E2M1 -> fp16 conversion and one packed multiply per pair: 8 instructions per 8
// codes) and writes the fp16 operands to LDS in the order the matrix instruction reads them; all four
// waves then take their operands from there.  (The first kernel converted in every wave that used an
// element, twice per workgroup, and the conversions, not the matrix instructions, set its pace.)
//
// Range: activation scales are renormalised per row and weight scales per column by powers of two
// (largest scale of a row / column moved into [2^10, 2^11)), so the fp16 products never overflow and
// only contributions 2^-25 below the largest of their row / column can underflow.  The shifts are
// undone exactly in the epilogue.
//
// Tiling: workgroup = 4 waves (2 x 2), block tile 256 x 256, wave tile 128 x 128 = 4 x 4 MFMA tiles,
// 256 fp32 accumulators per lane.  Two LDS buffers of fp16 operands alternate, one k-group each, one
// workgroup barrier per k-group: while the matrix instructions of group g run from one buffer, the
// codes of group g + 1 (requested a group earlier) are converted into the other and those of group
// g + 2 are requested.
#pragma once

#include <type_traits>

#include "gemm_params.h"
#include "svdq_quant.h"

namespace svdq {


__device__ inline half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ inline uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }

// 8 E2M1 patterns of one word -> 8 fp16 values pattern_value * scale, slot order [0..7].  The
// hardware conversion yields the exact E2M1 value (its scale operand only contributes an exponent).
__device__ inline half8_t dequant_word_fp4(uint32_t w, half2_t s) {
    const half2_t t0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 0) * s;
    const half2_t t1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 1) * s;
    const half2_t t2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 2) * s;
    const half2_t t3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 3) * s;
    return half8_t{t0[0], t0[1], t1[0], t1[1], t2[0], t2[1], t3[0], t3[1]};
}

__device__ inline float e4m3_to_f32(uint32_t b) {
    const uint32_t ex = (b >> 3) & 0xF, m = b & 7;
    return ex == 0 ? ldexpf((float)m, -9) : ldexpf((float)(8 + m), (int)ex - 10);
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

// Partial sums of a tile shared by two workgroups travel through memory with system-scope accesses
// (sc0 sc1): they bypass the caches that are not coherent between the XCDs, so no cache write-back or
// invalidation is needed around them, only completion (vmcnt) before the arrival counter is touched.
// Raw buffer intrinsics carry the cache policy and are ordinary compiler-visible memory operations: the
// compiler places the waits for the loaded registers itself (a register that an asm load is still going to
// write is not safe from compiler-made copies).  `slot` is the wave-uniform start of a workspace slot (the
// descriptor lives in scalar registers); layout of a slot [64 quads][256 threads] x float4.
constexpr int PARTIAL_SC0_SC1 = 0x11;  // aux bits of the buffer intrinsics on gfx940+: sc0 = 1, sc1 = 16
__device__ inline __amdgpu_buffer_rsrc_t partial_rsrc(const float4_t *slot) {
    return __builtin_amdgcn_make_buffer_rsrc((void *)slot, 0, 64 * 256 * 16, 0x00020000);
}
__device__ inline void store_partial(__amdgpu_buffer_rsrc_t r, int tid, int quad, float4_t v) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, v), r, (quad * 256 + tid) * 16, 0, PARTIAL_SC0_SC1);
}
__device__ inline float4_t load_partial(__amdgpu_buffer_rsrc_t r, int tid, int quad) {
    return __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(r, (quad * 256 + tid) * 16, 0, PARTIAL_SC0_SC1));
}

// NEXT: the epilogue also prepares the next layer's input (GELU, quantize, low-rank down); the plain
// variant carries none of that code or of its registers.
template <bool NEXT>
__global__ void __launch_bounds__(256, 1) gemm_w4a4_kernel(GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // Thread coordinates.  They are re-derived from an opaque copy of the thread index at the top of every
    // tile (and again for the epilogue): otherwise everything computed from them anywhere in the kernel
    // is hoisted to the kernel entry and kept in registers, or spilled, across all loops.
    int tid = threadIdx.x;
    int lane = tid & 63, wave = tid >> 6;
    int wm = wave >> 1, wn = wave & 1;
    int r32 = lane & 31, h = lane >> 5;
    auto refresh_thread_coordinates = [&]() {
        int t = threadIdx.x;
        asm volatile("" : "+v"(t));
        tid = t; lane = t & 63; wave = t >> 6;
        wm = wave >> 1; wn = wave & 1; r32 = lane & 31; h = lane >> 5;
    };

    // ---- persistent workgroups, work split in units of two k-groups ----------------------------
    // The tiles are numbered down M first (consecutive tiles share their weight columns) and every
    // tile is a run of K/128 units.  Workgroup v (of W) takes the units [U v / W, U (v+1) / W) of the
    // concatenated run: every workgroup gets the same amount of work whatever the tile count, at the
    // price that a tile may be shared by two workgroups (never more: the host launches at most as many
    // workgroups as there are tiles, so a share is at least one tile long).  A shared tile's two
    // partial sums are combined by whichever workgroup finishes second (see below).
    // v is blockIdx remapped so that the 8 XCDs (blockIdx % 8) each own one contiguous band of tiles.
    const int mblocks = p.M_pad / BM, nblocks = (p.N + BN - 1) / BN;
    const int ntiles = mblocks * nblocks;
    const int kgroups = p.K / 64, kunits = kgroups / 2;
    const int ntiles32 = p.N / 32;
    const int nwg = gridDim.x;
    const int xcd = (int)blockIdx.x % 8, extra = nwg % 8;  // XCD x holds nwg / 8 workgroups, one more if x < nwg % 8
    const int vwg = xcd * (nwg / 8) + (xcd < extra ? xcd : extra) + (int)blockIdx.x / 8;
    const long long units = (long long)ntiles * kunits;
    const long long u_begin = units * vwg / nwg, u_end = units * (vwg + 1) / nwg;
    const int first_tile = (int)(u_begin / kunits);
    const int nseg = u_end > u_begin ? (int)((u_end - 1) / kunits) - first_tile + 1 : 0;
    // segment s of this workgroup: tile first_tile + s, k-groups [gb, ge)
    // Whole tiles only (p.whole_band != 0, the workgroup count divides the tile count): in its step s workgroup v takes
    // tile s W + v of a numbering in bands of p.whole_band row blocks, down the band first.  All workgroups walk K in
    // step, so the 32 of an XCD, which hold consecutive numbers, cover a compact window of the output at any time and
    // share its rows of activations and columns of weights in their L2.
    auto segment = [&](int sidx, int &tile, int &gb, int &ge) {
        if (p.whole_band) {
            tile = sidx * nwg + vwg;
            gb = 0;
            ge = kgroups;
            return;
        }
        tile = first_tile + sidx;
        const long long t0 = (long long)tile * kunits;
        gb = sidx == 0 ? 2 * (int)(u_begin - t0) : 0;
        ge = u_end - t0 < kunits ? 2 * (int)(u_end - t0) : kgroups;
    };
    auto tile_coords = [&](int tile, int &m0, int &n0) {
        if (p.whole_band) {
            const int per_band = p.whole_band * nblocks;
            const int band = tile / per_band, in_band = tile - band * per_band;
            const int rows = mblocks - band * p.whole_band < p.whole_band ? mblocks - band * p.whole_band : p.whole_band;
            m0 = (band * p.whole_band + in_band % rows) * BM;
            n0 = (in_band / rows) * BN;
            return;
        }
        m0 = (tile % mblocks) * BM;
        n0 = (tile / mblocks) * BN;
    };

    // the workgroups [lo, hi] whose shares reach into a tile (units [t0, t0 + kunits)); more than two only
    // when there are fewer tiles than workgroups
    auto tile_parties = [&](int tile, int &lo, int &hi) {
        const long long t0 = (long long)tile * kunits, t1 = t0 + kunits;
        lo = (int)(((t0 + 1) * nwg + units - 1) / units) - 1;  // first v with units (v + 1) / nwg > t0
        hi = (int)((t1 * nwg - 1) / units);                    // last v with units v / nwg < t1
    };
    int *rowshift = (int *)(lds + SHIFT_OFF);  // [MAX_BATCH][256] power-of-two renormalisation of the rows
    constexpr uint32_t AS_ELT = 4, BS_ELT = 8;  // bytes of scales per (64-group, row / column)
    const uint32_t as_stride = (uint32_t)p.M_pad * AS_ELT, bs_stride = (uint32_t)p.N * BS_ELT;

    // Everything thread t needs to stage its row of activations and its column of weights of one tile: the
    // addresses of their first k-group (codes: 32 bytes per row and k-group in tiles of 32 rows, 1 KB per tile
    // and k-group; scales: one word of four e4m3 per row, four fp16 per column and k-group).
    struct TileCtx {
        int tile, gb, ge;  // k-groups [gb, ge) of the tile
        int m0, n0, shift;
        int col_ok;
        const uint8_t *a_ptr, *b_ptr, *as_ptr, *bs_ptr;
    };
    // follow: the segment after the one given by prev_* (the next tile, from its first k-group), without divisions
    auto make_ctx = [&](int sidx, int slot, int tid, bool follow, int prev_tile, int prev_m0, int prev_n0) {
        TileCtx c;
        if (follow && !p.whole_band) {
            c.tile = prev_tile + 1;
            c.gb = 0;
            const long long left = u_end - (long long)c.tile * kunits;
            c.ge = left < kunits ? 2 * (int)left : kgroups;
            c.m0 = prev_m0 + BM;
            c.n0 = prev_n0;
            if (c.m0 == p.M_pad) {
                c.m0 = 0;
                c.n0 += BN;
            }
        } else {
            segment(sidx, c.tile, c.gb, c.ge);
            tile_coords(c.tile, c.m0, c.n0);
        }
        c.shift = rowshift[slot * 256 + tid];  // thread tid stages row tid
        // (N is a multiple of 128: the columns of a 32-column tile are inside or outside together; a thread beyond N
        // fetches the last tile's codes instead and converts them with scale zero)
        c.col_ok = c.n0 + tid < p.N;
        const int tb = c.n0 / 32 + (tid >> 5) < ntiles32 ? c.n0 / 32 + (tid >> 5) : ntiles32 - 1;
        c.a_ptr = p.act + (size_t)(c.m0 / 32 + (tid >> 5)) * kgroups * TILE_BYTES + (tid & 31) * 32;
        c.b_ptr = p.wgt + (size_t)tb * kgroups * TILE_BYTES + (tid & 31) * 32;
        c.as_ptr = (const uint8_t *)p.ascales + (size_t)(c.m0 + tid) * AS_ELT;
        c.bs_ptr = (const uint8_t *)p.wscales + (size_t)(c.col_ok ? c.n0 + tid : p.N - 1) * BS_ELT;
        return c;
    };

    // ---- staging -----------------------------------------------------------------------------
    // One k-group of a thread's row and column on their way from memory to LDS: 64 + 64 codes and their scales.
    // Ordinary loads: the compiler tracks the registers they write and places the waits itself.
    struct Raw {
        u32x4_t a[2], b[2];
        uint32_t as;
        u32x2_t bs;
    };
    // (l counts the k-groups of the segment; requests past the end of K repeat the last group and are never used)
    auto load_raw = [&](const TileCtx &c, int l, Raw &r) {
        const uint32_t gc = (uint32_t)(c.gb + l < kgroups ? c.gb + l : kgroups - 1);
        const u32x4_t *ap = (const u32x4_t *)(c.a_ptr + gc * TILE_BYTES), *bp = (const u32x4_t *)(c.b_ptr + gc * TILE_BYTES);
        r.a[0] = ap[0];
        r.a[1] = ap[1];
        r.b[0] = bp[0];
        r.b[1] = bp[1];
        r.as = *(const uint32_t *)(c.as_ptr + gc * as_stride);
        r.bs = *(const u32x2_t *)(c.bs_ptr + gc * bs_stride);
    };
    // Words 2 ks and 2 ks + 1 of the thread's row and of its column (16-group ks of the k-group) -> fp16 -> the
    // operand buffer: word w holds the codes of k = 8 w .. 8 w + 7, which are one lane's operand of the matrix
    // instruction (step w / 2, half w % 2); a wave's 64 threads write 64 consecutive 16-byte slots per word.
    // `which`: 0, 1 the two words of the row, 2, 3 those of the column.
    auto group_scales = [&](const TileCtx &c, const Raw &r, int ks, half2_t &sa2, half2_t &sb2) {
        // e4m3 -> fp16 with the row's shift, without branches (a branch would end the scheduling region in which the
        // conversions are interleaved with the matrix instructions)
        const uint32_t e8 = (r.as >> (8 * ks)) & 0x7Fu, ex = e8 >> 3;
        const _Float16 sa = (_Float16)ldexpf((float)((e8 & 7u) | (ex ? 8u : 0u)), (int)(ex ? ex : 1u) - 10 + c.shift);
        const uint32_t hb = c.col_ok ? (r.bs[ks >> 1] >> (16 * (ks & 1))) & 0xFFFFu : 0u;
        sa2 = half2_t{sa, sa};
        sb2 = as_half2(hb | (hb << 16));
    };
    auto convert_word = [&](const Raw &r, uint32_t buf, int ks, int which, half2_t sa2, half2_t sb2, int tid) {
        uint8_t *base = lds + buf * OPBUF_BYTES + (tid >> 5) * (4 * 2 * 32 * 16) + (tid & 31) * 16 + (ks * 2 + (which & 1)) * 512;
        const int w = 2 * ks + (which & 1);
        if (which < 2) *(half8_t *)base = dequant_word_fp4(r.a[w >> 2][w & 3], sa2);
        else *(half8_t *)(base + OP_BYTES) = dequant_word_fp4(r.b[w >> 2][w & 3], sb2);
    };
    auto convert_store = [&](const TileCtx &c, const Raw &r, uint32_t buf, int ks, int tid) {
        half2_t sa2, sb2;
        group_scales(c, r, ks, sa2, sb2);
#pragma unroll
        for (int which = 0; which < 4; which++) convert_word(r, buf, ks, which, sa2, sb2, tid);
    };

    float16_t acc[4][4];
    int coltab_n0 = -1;  // first column of the tile whose column tables are in LDS (wave-uniform)
    Raw rawa, rawb, rawc, rawd;  // codes on their way: `rawc`, `rawd` are converted next, the other two are requests in flight

    // The arithmetic of one k-group: four steps of 16 matrix instructions on the operands in buffer `buf`; the
    // operands of a step are fetched during the step before; between the matrix instructions the group `rc` is
    // converted into the other buffer, one 16-group per step.
    half8_t opa[2][4], opb[2][4];
    auto read_a = [&](uint32_t buf, int ks, int t, half8_t &a) {
        a = *(const half8_t *)(lds + buf * OPBUF_BYTES + (ks * 2 + h) * 512 + r32 * 16 + (wm * 4 + t) * (4 * 2 * 32 * 16));
    };
    auto read_b = [&](uint32_t buf, int ks, int t, half8_t &b) {
        b = *(const half8_t *)(lds + buf * OPBUF_BYTES + OP_BYTES + (ks * 2 + h) * 512 + r32 * 16 + (wn * 4 + t) * (4 * 2 * 32 * 16));
    };
    // One piece (of six) of a k-group's requests: a thread's two 16-byte halves of its row's codes, the same of its
    // column's, the row's scales, the column's scales.
    auto load_piece = [&](const TileCtx &c, int l, Raw &r, int piece) {
        const uint32_t gc = (uint32_t)(c.gb + l < kgroups ? c.gb + l : kgroups - 1);
        if (piece == 0) r.a[0] = *(const u32x4_t *)(c.a_ptr + gc * TILE_BYTES);
        if (piece == 1) r.a[1] = *(const u32x4_t *)(c.a_ptr + gc * TILE_BYTES + 16);
        if (piece == 2) r.b[0] = *(const u32x4_t *)(c.b_ptr + gc * TILE_BYTES);
        if (piece == 3) r.b[1] = *(const u32x4_t *)(c.b_ptr + gc * TILE_BYTES + 16);
        if (piece == 4) r.as = *(const uint32_t *)(c.as_ptr + gc * as_stride);
        if (piece == 5) r.bs = *(const u32x2_t *)(c.bs_ptr + gc * bs_stride);
    };
    // A k-group is four steps of 16 k; a step is four quarters, each in this order and fenced from the next (left
    // alone, the scheduler gathers the matrix instructions in long runs and the conversions in others, and the two
    // pipes take turns instead of working side by side): two operand tiles of the next step are requested, one word
    // of `rc` is converted and stored, four matrix instructions are issued with the conversion between them.  A wave
    // is alone on its SIMD, so whatever stands in front of a matrix instruction is lost time; therefore also:
    //   - the scales of a step's 16-group are prepared during the step before (those of the next group's first step
    //     during this group's last, from `rc_next`);
    //   - the requests for later groups (LOADS: both groups the iteration asks for) are issued one per quarter;
    //   - a second barrier in the middle of the group publishes the first half of the other buffer, so that the
    //     operands of the next group's first step can be fetched during this group's last step instead of behind
    //     the barrier that ends the group; neither barrier waits for the LDS queue to drain (see below).
    // (the group behind the last one of a segment is converted too, into the buffer nobody reads any more: a
    // condition would split the body into basic blocks)
    half2_t sa2, sb2;  // scales of the 16-group converted next
    auto group = [&](auto LOADS_T, const TileCtx &c, uint32_t buf, const Raw &rc, const Raw &rc_next, int l_load, Raw &ld0, Raw &ld1) {
        constexpr bool LOADS = decltype(LOADS_T)::value;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int nq = ks * 4 + q;  // quarter of the group
                half2_t sa2n = sa2, sb2n = sb2;
                if (q == 3) group_scales(c, ks < 3 ? rc : rc_next, (ks + 1) & 3, sa2n, sb2n);
                if (LOADS && nq < 12) load_piece(c, l_load + nq / 6, nq < 6 ? ld0 : ld1, nq % 6);
                // (the next step's first quarter needs all four weight tiles and the first activation tile: the
                // weight tiles are requested first, every operand at least two quarters before its use)
                const uint32_t rbuf = ks < 3 ? buf : buf ^ 1;
                if (q < 2) {
                    read_b(rbuf, (ks + 1) & 3, 2 * q, opb[(ks + 1) & 1][2 * q]);
                    read_b(rbuf, (ks + 1) & 3, 2 * q + 1, opb[(ks + 1) & 1][2 * q + 1]);
                } else {
                    read_a(rbuf, (ks + 1) & 3, 2 * q - 4, opa[(ks + 1) & 1][2 * q - 4]);
                    read_a(rbuf, (ks + 1) & 3, 2 * q - 3, opa[(ks + 1) & 1][2 * q - 3]);
                }
                convert_word(rc, buf ^ 1, ks, q, sa2, sb2, tid);
#pragma unroll
                for (int nt = 0; nt < 4; nt++)
                    acc[q][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(opb[ks & 1][nt], opa[ks & 1][q], acc[q][nt], 0, 0, 0);
                if (LOADS && nq < 12) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                if (q == 3) {  // (with the preparation of the next step's scales)
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                } else {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                sa2 = sa2n;
                sb2 = sb2n;
                // The two barriers of a group stand one quarter BEHIND the stores they publish (the end of the previous
                // group, the end of step 1): a wave's LDS operations complete in order, so waiting until only this
                // quarter's three (two fetches, one store) are outstanding proves the earlier stores complete without
                // draining the queue of fetches that keeps the matrix instructions fed.  What this quarter stores
                // belongs to the half that the next barrier publishes; nobody fetches what a wave one quarter ahead
                // overwrites (that region was last fetched a whole group earlier).
                if (q == 0 && (ks == 0 || ks == 2)) asm volatile("s_waitcnt lgkmcnt(3)\n\ts_barrier" ::: "memory");
            }
        }
    };

  for (int batch0 = 0; batch0 < nseg; batch0 += MAX_BATCH) {
    const int nbatch = nseg - batch0 < MAX_BATCH ? nseg - batch0 : MAX_BATCH;
    {
    int tid_p = threadIdx.x;  // opaque copy: nothing derived from it is kept in registers beyond this block
    asm volatile("" : "+v"(tid_p));
    const int tid = tid_p;
    // ---- largest activation scale of every row of the batch's tiles -> power-of-two shift that
    //      moves it into [2^10, 2^11)
    __syncthreads();  // the previous batch is done with the table
    {
        // four e4m3 scales per (row, 64-group) packed in one word; e4m3 patterns of
        // non-negative values order like unsigned bytes
        for (int t = 0; t < nbatch; t++) {
            int m0, n0;
            int tile_t, gb_t, ge_t;
            segment(batch0 + t, tile_t, gb_t, ge_t);
            tile_coords(tile_t, m0, n0);
            const uint32_t *sp = (const uint32_t *)p.ascales + m0 + tid;
            uint32_t mx = 0;
            for (int g0 = 0; g0 < kgroups; g0 += 8) {  // eight requests in flight (a maximum does not mind seeing the last group again)
                uint32_t v[8];
#pragma unroll
                for (int u = 0; u < 8; u++) v[u] = sp[(size_t)(g0 + u < kgroups ? g0 + u : kgroups - 1) * p.M_pad];
#pragma unroll
                for (int u = 0; u < 8; u++)
                    mx = max(max(mx, v[u] & 0x7Fu), max((v[u] >> 8) & 0x7Fu, max((v[u] >> 16) & 0x7Fu, (v[u] >> 24) & 0x7Fu)));
            }
            int ex = 0;
            if (mx) frexpf(e4m3_to_f32(mx), &ex);  // value in [2^(ex-1), 2^ex)
            rowshift[t * 256 + tid] = mx == 0 ? 0 : NORM_TARGET_EXP - (ex - 1);
        }
    }
    }
    __syncthreads();

    TileCtx cur = make_ctx(batch0, 0, threadIdx.x, false, 0, 0, 0);

   for (int ti = 0; ti < nbatch; ti++) {
    const bool have_next = ti + 1 < nbatch;
    refresh_thread_coordinates();
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    // Groups 0 to 2 of the segment are requested, group 0 converted into buffer 0 (the previous tile's epilogue is
    // done with the LDS it shares with the buffers: every tile ends with a barrier).  An iteration multiplies groups
    // l and l + 1 (buffers 0 and 1) and converts groups l + 1 and l + 2 from `rawc` and `rawd`; groups l + 3 and
    // l + 4 are requested during its first group into `rawa` and `rawb` and handed over at its end.  Segments are an
    // even number of groups long.
    load_raw(cur, 0, rawa);
    load_raw(cur, 1, rawc);
    load_raw(cur, 2, rawd);
#pragma unroll
    for (int ks = 0; ks < 4; ks++) convert_store(cur, rawa, 0, ks, tid);
    group_scales(cur, rawc, 0, sa2, sb2);
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 4; t++) {
        read_b(0, 0, t, opb[0][t]);
        read_a(0, 0, t, opa[0][t]);
    }
    const int seg_len = cur.ge - cur.gb;
    for (int l = 0; l < seg_len; l += 2) {
        group(std::true_type{}, cur, 0, rawc, rawd, l + 3, rawa, rawb);   // group l; group l + 1 -> buffer 1
        group(std::false_type{}, cur, 1, rawd, rawa, 0, rawa, rawb);      // group l + 1; group l + 2 -> buffer 0
        rawc = rawa;
        rawd = rawb;
    }
    // pin the accumulators in the accumulation registers across the loop exit: without this the
    // register allocator may place the 256 copies into ordinary registers inside the loop body
    asm volatile("" : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[0][2]), "+a"(acc[0][3]), "+a"(acc[1][0]), "+a"(acc[1][1]),
                      "+a"(acc[1][2]), "+a"(acc[1][3]), "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[2][2]), "+a"(acc[2][3]),
                      "+a"(acc[3][0]), "+a"(acc[3][1]), "+a"(acc[3][2]), "+a"(acc[3][3]));
    __syncthreads();
    // Thread coordinates for the epilogue, re-derived from an opaque copy of the thread index: nothing
    // computed from them can be hoisted above the main loop and occupy registers there.
    int tid_e = threadIdx.x;
    asm volatile("" : "+v"(tid_e));
    const int tid = tid_e, lane = tid_e & 63, wave = __builtin_amdgcn_readfirstlane(tid_e >> 6);
    const int wm = wave >> 1, wn = wave & 1, r32 = lane & 31, h = lane >> 5;
    const int m0 = cur.m0, n0 = cur.n0, tile_e = cur.tile;
    const int *tile_shift = rowshift + ti * 256;

    // ---- a tile shared with other workgroups ---------------------------------------------------
    // Every party holds the sum over its part of K.  Whoever finishes last adds all parties' sums in ascending order
    // of the workgroups, its own (from its registers) in their place: the result does not depend on who that is, so
    // the output is the same from launch to launch.  Nobody waits: the others park their accumulators in their slot
    // of the workspace (workgroup v parks the tile its share begins in at 2 v, the one it ends in at 2 v + 1; layout of
    // a slot [64 quads][256 threads] x float4, a wave's access covers 1 KB) and go on.  (Starting the accumulators
    // from a neighbour's parked sums where they happen to be there already saves the parking, but changes the order
    // of the additions with the timing: outputs then differed in their last bit from launch to launch.)
    bool run_epilogue = true, combine = false;
    int party_lo = 0, party_hi = -1;  // (worked out here, not ahead of the main loop, where they would occupy registers)
    if (cur.gb != 0 || cur.ge != kgroups) {
        tile_parties(tile_e, party_lo, party_hi);
        const bool is_head = cur.gb != 0;  // the share begins inside this tile
        const int others = party_hi - party_lo;
        float4_t *mine = (float4_t *)p.partials + (size_t)(2 * vwg + (is_head ? 0 : 1)) * (64 * 256);
        int *counter = p.counters + cur.tile;
        int *flag = (int *)(lds + FLAG_OFF);
        // (a look at the counter first saves the parking when everybody else is already done; not worth a
        // round trip where that is unlikely: a share begins with its shared tile and ends with the other)
        bool last = false;
        if (!is_head) {
            if (tid == 0) *flag = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            last = *flag == others;
            __syncthreads();
        }
        if (!last) {
            const __amdgpu_buffer_rsrc_t mine_rsrc = partial_rsrc(mine);
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++)
                        store_partial(mine_rsrc, tid, (i * 4 + j) * 4 + q,
                                      float4_t{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]});
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the parked sums are in memory before the counter says so
            __syncthreads();
            if (tid == 0) *flag = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            last = *flag == others;
            __syncthreads();
        }
        run_epilogue = last;
        combine = last;
        if (last && tid == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
    }
    // ---- epilogue -----------------------------------------------------------------------------
    // The MFMAs were issued with the weight tile as the first operand, so a lane holds one output ROW
    // (r32 of the 32-row tile) and accumulator element e is COLUMN 8*(e/4) + 4*h + e%4 of the 32-column
    // tile: four consecutive elements are four consecutive output columns.
    const int wrow0 = m0 + wm * 128, wcol0 = n0 + wn * 128;
    // per-column factor (undoes the column normalisation, applies alpha and wcscales) and bias of the
    // wave's 128 columns, tabulated in LDS (EpilogueBias, gemm_base.cuh:710-781)
    // (kept across tiles: consecutive tiles of a workgroup mostly lie in the same 256 columns)
    float *coltab = (float *)(lds + TAB_OFF + wave * 1024);  // [128] factors, then [128] biases
    if (run_epilogue && n0 != coltab_n0) {
        coltab_n0 = n0;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int n = wcol0 + 2 * lane + j;
            const bool ok = n < p.N;
            float cf = ok ? p.colnorm[n] * p.alpha : 0.f;
            if (ok && p.wcscales) cf *= bf16_bits_to_f32(p.wcscales[n]);
            coltab[2 * lane + j] = cf;
            coltab[128 + 2 * lane + j] = (ok && p.bias) ? bf16_bits_to_f32(p.bias[n]) : 0.f;
            if (NEXT && p.rotary)  // RMS-norm weights of the head these 128 columns are (q below N/3, k below 2N/3)
                ((float *)(lds + NORMW_OFF + wave * 512))[2 * lane + j] = bf16_bits_to_f32((wcol0 < p.rope_cols / 2 ? p.norm_q : p.norm_k)[2 * lane + j]);
        }
    }
    // Low-rank up projection (lora.cuh:110-241): out += bf16(lora_act * scale) @ up^T on the matrix cores.
    // The projection is added to the accumulators BEFORE they are scaled.  The accumulators are in
    // normalised units (out = acc * rn[row] * cf[col] + bias), so the operands are divided by rn and cf
    // first; the matrix cores then update the accumulators in place and the operands are dead before the
    // output pass starts.  rn is a power of two (the division only changes exponents); cf
    // (column normalisation x alpha x wcscales) is an arbitrary number, so up / cf is passed as the sum of
    // two bf16 numbers (the rounded quotient and the rounded remainder: relative error 2^-17, below the
    // rounding noise of the main loop) in two matrix-core steps; wcscales must not be zero.
    const int nsteps = p.R_up / 16;
    if (run_epilogue && nsteps > 0) {
        {
            // two 16-rank steps per round; every request of a round is issued before any of its data is
            // touched, so a round costs one memory latency
            for (int s0 = 0; s0 < nsteps; s0 += 2) {
                const bool two = s0 + 1 < nsteps;
                const int s1 = two ? s0 + 1 : s0;
                float4_t ra[4][2][2];
                u32x4_t rb[4][2];
                float rcf[4], lsr[4];
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const float4_t *ap = (const float4_t *)(p.lora_act + (size_t)(wrow0 + t * 32 + r32) * p.R_up + 8 * h);
                    ra[t][0][0] = ap[4 * s0]; ra[t][0][1] = ap[4 * s0 + 1];
                    ra[t][1][0] = ap[4 * s1]; ra[t][1][1] = ap[4 * s1 + 1];
                    const int n = wcol0 + t * 32 + r32;
                    const bool ok = n < p.N;
                    const u32x4_t *bp = (const u32x4_t *)(p.lora_up + (size_t)(ok ? n : 0) * p.R_up + 8 * h);
                    rb[t][0] = bp[2 * s0];
                    rb[t][1] = bp[2 * s1];
                    float cf = ok ? p.colnorm[n] * p.alpha : 1.f;
                    if (ok && p.wcscales) cf *= bf16_bits_to_f32(p.wcscales[n]);
                    rcf[t] = ok ? __fdiv_rn(1.0f, cf) : 0.f;
                    lsr[t] = ldexpf(1.0f, tile_shift[wm * 128 + t * 32 + r32]);
                }
#pragma unroll
                for (int k = 0; k < 2; k++) {
                    if (k == 1 && !two) break;
                    const float ls = p.lora_scales[s0 + k];
                    bf16x8_t la[4], lb[4], lb_rem[4];
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        const float f = ls * lsr[t];
                        const float4_t v0 = ra[t][k][0], v1 = ra[t][k][1];
                        u32x4_t w;
                        w[0] = pack_bf16x2(v0[0] * f, v0[1] * f);
                        w[1] = pack_bf16x2(v0[2] * f, v0[3] * f);
                        w[2] = pack_bf16x2(v1[0] * f, v1[1] * f);
                        w[3] = pack_bf16x2(v1[2] * f, v1[3] * f);
                        la[t] = __builtin_bit_cast(bf16x8_t, w);
                        u32x4_t bw = rb[t][k], br = u32x4_t{0, 0, 0, 0};
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const float q0 = bits_f32(bw[i] << 16) * rcf[t], q1 = bits_f32(bw[i] & 0xFFFF0000u) * rcf[t];
                            bw[i] = pack_bf16x2(q0, q1);
                            br[i] = pack_bf16x2(q0 - bits_f32(bw[i] << 16), q1 - bits_f32(bw[i] & 0xFFFF0000u));
                        }
                        lb[t] = __builtin_bit_cast(bf16x8_t, bw);
                        lb_rem[t] = __builtin_bit_cast(bf16x8_t, br);
                    }
#pragma unroll
                    for (int mt = 0; mt < 4; mt++)
#pragma unroll
                        for (int nt = 0; nt < 4; nt++)
                            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lb[nt], la[mt], acc[mt][nt], 0, 0, 0);
#pragma unroll
                    for (int mt = 0; mt < 4; mt++)
#pragma unroll
                        for (int nt = 0; nt < 4; nt++)
                            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lb_rem[nt], la[mt], acc[mt][nt], 0, 0, 0);
                }
            }
        }
    }
    // reciprocal smoothing factors of the next layer for the 32 columns this lane quantizes
    // (work item of the quantizing pass: row = item / 4, 32-column quarter = item % 4 = lane % 4)
    float nrs[32];
    if (NEXT && p.qout && run_epilogue) {
        const float4_t *sp = (const float4_t *)(p.next_smooth_rcp + (wcol0 < p.N ? wcol0 : 0) + (lane & 3) * 32);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float4_t v = sp[i];
            nrs[4 * i] = v[0]; nrs[4 * i + 1] = v[1]; nrs[4 * i + 2] = v[2]; nrs[4 * i + 3] = v[3];
        }
    }
    const bool interior = m0 + BM <= p.M_out && n0 + BN <= p.N_out;  // the whole tile lies inside the output
    uint16_t *slab = (uint16_t *)(lds + SLAB_OFF + wave * (32 * OUT_LD * 2));
    const int ngroups_out = p.N / 64;
    // one 32-row slab of the wave tile; instantiated four times with a compile-time slab index (a
    // pragma-unrolled loop of this size is refused by the unroller, which would push the
    // accumulators into scratch memory)
    auto slab_epilogue = [&](auto MT, auto COMBINE_T) {
        constexpr int mt = decltype(MT)::value;
        constexpr bool COMBINE = decltype(COMBINE_T)::value;  // a tile shared with a neighbour: add its partial sums
        // undo the power-of-two normalisation of the lane's row
        const float rn = ldexpf(1.0f, -tile_shift[wm * 128 + mt * 32 + r32]);
        // (the accumulators are only read from here on: updating them in place makes the register
        // allocator copy and spill whole tuples)
        float4_t other[16];  // COMBINE: the parties' sums of this slab, added in ascending order of the workgroups
        if (COMBINE) {
#pragma unroll
            for (int k = 0; k < 16; k++) other[k] = float4_t{0.f, 0.f, 0.f, 0.f};
            for (int v = party_lo; v <= party_hi; v++) {
                if (v == vwg) {
#pragma unroll
                    for (int k = 0; k < 16; k++)
#pragma unroll
                        for (int i = 0; i < 4; i++) other[k][i] += acc[mt][k >> 2][4 * (k & 3) + i];
                    continue;
                }
                // a workgroup parks the tile its share begins inside at slot 2 v, otherwise at 2 v + 1
                const bool begins_inside = units * v / nwg > (long long)tile_e * kunits;
                const __amdgpu_buffer_rsrc_t r = partial_rsrc((const float4_t *)p.partials + (size_t)(2 * v + (begins_inside ? 0 : 1)) * (64 * 256));
#pragma unroll
                for (int k = 0; k < 16; k++) other[k] += load_partial(r, tid, mt * 16 + k);
            }
        }
        // the column factors and biases of a 32-column tile are requested one tile ahead of their use:
        // fetched right where they are needed, every group of four would pay the full LDS latency
        float16_t v[4];
        float4_t cfv[2][4], bsv[2][4];
        auto load_cols = [&](int nt, float4_t (&cf)[4], float4_t (&bs)[4]) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                cf[q] = *(const float4_t *)(coltab + nt * 32 + 8 * q + 4 * h);
                bs[q] = *(const float4_t *)(coltab + 128 + nt * 32 + 8 * q + 4 * h);
            }
        };
        load_cols(0, cfv[0], bsv[0]);
#pragma unroll
        for (int nt = 0; nt < 4; nt++) {
            if (nt < 3) load_cols(nt + 1, cfv[(nt + 1) & 1], bsv[(nt + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4_t cf = cfv[nt & 1][q], bs = bsv[nt & 1][q];
                if (COMBINE) {
                    const float4_t o = other[nt * 4 + q];
#pragma unroll
                    for (int i = 0; i < 4; i++) v[nt][4 * q + i] = __builtin_fmaf(o[i] * rn, cf[i], bs[i]);
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) v[nt][4 * q + i] = __builtin_fmaf(acc[mt][nt][4 * q + i] * rn, cf[i], bs[i]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (NEXT && p.rotary && wcol0 < p.rope_cols) {
            // EpilogueRMSNormRope (epilogues.cuh:269-425): the wave's 128 columns are one head of q or k.
            // The lane holds 64 values of its row, lane ^ 32 the other 64.  The (sin, cos) table is stored in
            // this loop's order ([32-row block][nt][q][lane] x float4: a wave-wide request is 1 KB
            // contiguous), requested two column tiles ahead.
            int blk = (wrow0 + mt * 32) >> 5;
            blk = blk < (p.rot_rows >> 5) ? blk : (p.rot_rows >> 5) - 1;  // (rows beyond the output are never stored)
            const float4_t *rp = (const float4_t *)p.rotary + (size_t)blk * (16 * 64) + lane;
            const float *normw = (const float *)(lds + NORMW_OFF + wave * 512);
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
        // compiler has to be kept from reordering across this point (a fence would also wait for the
        // global stores in flight)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        // EpilogueDefault (gemm_base.cuh:667-698): 16-byte row-contiguous stores.  Streaming stores: the
        // tile is not read again by this kernel.
        if (NEXT && p.vk && wcol0 >= p.N / 3 && wcol0 < p.N) {
            // every 32-row slab parks its own sums (this kernel has no registers to carry them from slab to slab)
            VkSums vks;
            litela_clear(vks);
            litela_add_slab(vks, slab, OUT_LD, lane);
            const int third = p.N / 3;
            litela_park<true>(vks, p.vk_part + ((size_t)((wrow0 + mt * 32) >> 5) * (2 * third / 64) + (wcol0 - third) / 64) * VK_HEAD_FLOATS, lane);
        }
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
        if (NEXT && p.next_down && wcol0 < p.N) {
            // low-rank down projection of the next layer on the bf16 tile (EpilogueLoraDown,
            // lora.cuh:243-353): this wave's 128 columns are one 128-chunk of the next layer's K
            const int RT = p.R_down / 16;
            const int r16 = lane & 15, q = lane >> 4;
            // (the operands of rank tile rt + 1 are requested before rank tile rt is worked on: one exposed
            // memory latency per slab instead of one per rank tile)
            bf16x8_t nb[4];
#pragma unroll
            for (int i = 0; i < 4; i++) nb[i] = p.next_down[((size_t)((wcol0 / 128) * 4 + i) * RT) * 64 + lane];
            for (int rt = 0; rt < RT; rt++) {
                float4_t d[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
                bf16x8_t b[4];
#pragma unroll
                for (int i = 0; i < 4; i++) b[i] = nb[i];
                const int rt_next = rt + 1 < RT ? rt + 1 : rt;
#pragma unroll
                for (int i = 0; i < 4; i++) nb[i] = p.next_down[((size_t)((wcol0 / 128) * 4 + i) * RT + rt_next) * 64 + lane];
#pragma unroll
                for (int i = 0; i < 4; i++) {
#pragma unroll
                    for (int m2 = 0; m2 < 2; m2++) {
                        const bf16x8_t a = *(const bf16x8_t *)(slab + (16 * m2 + r16) * OUT_LD + 32 * q + 8 * i);
                        d[m2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[i], d[m2], 0, 0, 0);
                    }
                }
                // This chunk's share of the sums over N goes to the workspace, in the lanes' own order; a small kernel
                // behind this one adds the chunks' shares in ascending order (reduce_shares_kernel in gemm.hip): the
                // same result from run to run (the reference adds with atomics in the order of arrival, lora.cuh:82-94).
#pragma unroll
                for (int m2 = 0; m2 < 2; m2++)
                    __builtin_nontemporal_store(d[m2], (float4_t *)(p.next_lora_part + (size_t)(wcol0 / 128) * p.M_pad * p.R_down) +
                                                           ((size_t)(((wrow0 + mt * 32) >> 5) * RT + rt) * 2 + m2) * 64 + lane);
            }
        }
        if (NEXT && p.qout && wcol0 < p.N) {
            // EpilogueQuantize (gemm_w4a4.cuh:930-1043): shift, smooth, quantize for the next layer
#pragma unroll
            for (int pass = 0; pass < 2; pass++) {
                const int item = pass * 64 + lane;
                const int rr = item >> 2, qc = item & 3;
                const u32x4_t *sp = (const u32x4_t *)(slab + rr * OUT_LD + qc * 32);
                float y[32];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const u32x4_t v = sp[i];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        float lo = bits_f32(v[j] << 16), hi = bits_f32(v[j] & 0xFFFF0000u);
                        y[8 * i + 2 * j] = smooth_quotient(lo, nrs[8 * i + 2 * j]);
                        y[8 * i + 2 * j + 1] = smooth_quotient(hi, nrs[8 * i + 2 * j + 1]);
                    }
                }
                const int m = wrow0 + mt * 32 + rr;
                const int gidx = (wcol0 + qc * 32) / 64;
                u32x4_t words;
                uint32_t sc[2];
                quantize_nvfp4_two_groups(y, words, sc);
                uint16_t *os = (uint16_t *)p.oscales;  // [N/64][M_pad][4]
                os[((size_t)gidx * p.M_pad + m) * 2 + (qc & 1)] = (uint16_t)(sc[0] | (sc[1] << 8));
                *(u32x4_t *)(p.qout + ((size_t)(m / 32) * ngroups_out + gidx) * TILE_BYTES + (m % 32) * 32 + 16 * (qc & 1)) = words;
            }
        }
        // the slab is private to this wave: LDS operations of one wave complete in order, so only the
        // compiler has to be kept from reordering across this point (a fence would also wait for the
        // global stores in flight)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_sched_barrier(0);  // keep the four slabs apart: hoisting the next slab's work multiplies live registers
    };
    __builtin_amdgcn_sched_barrier(0);
    if (run_epilogue && !combine) {
        slab_epilogue(std::integral_constant<int, 0>{}, std::false_type{});
        slab_epilogue(std::integral_constant<int, 1>{}, std::false_type{});
        slab_epilogue(std::integral_constant<int, 2>{}, std::false_type{});
        slab_epilogue(std::integral_constant<int, 3>{}, std::false_type{});
    } else if (run_epilogue) {
        slab_epilogue(std::integral_constant<int, 0>{}, std::true_type{});
        slab_epilogue(std::integral_constant<int, 1>{}, std::true_type{});
        slab_epilogue(std::integral_constant<int, 2>{}, std::true_type{});
        slab_epilogue(std::integral_constant<int, 3>{}, std::true_type{});
    }
    // (the next tile's context is worked out here, behind the epilogue: its four addresses would otherwise sit in
    // scratch memory while the epilogue needs the registers)
    if (have_next) cur = make_ctx(batch0 + ti + 1, ti + 1, threadIdx.x, true, tile_e, m0, n0);
    __syncthreads();
   }  // tiles of the batch
  }    // batches
}


template <bool NEXT>
int launch_gemm_variant(const GemmParams &p, int nwg, hipStream_t stream) {
    auto kern = gemm_w4a4_kernel<NEXT>;
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

}  // namespace svdq
