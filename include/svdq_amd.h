/*
 * svdq_amd.h -- C ABI of the MI355X (gfx950) SVDQuant W4A4 + low-rank linear path.
 *
 * This is the drop-in boundary for the two operators that nunchaku exposes from its native
 * module as `_C.ops.quantize_w4a4_act_fuse_lora` and `_C.ops.gemm_w4a4`
 * (reference: nunchaku/csrc/pybind.cpp:108-110, nunchaku/csrc/ops.h:10-110), plus the one-time
 * load-time conversion of reference-format checkpoint tensors into the layouts these kernels read.
 *
 * Conventions
 *   - plain pointers to DEVICE memory, sizes as int64_t, no framework types;
 *   - every function only enqueues work on `stream` (a hipStream_t passed as void*) and returns;
 *     no synchronisation; safe to call from several threads.  One exception to "no allocation, no
 *     global state": some calls of svdq_gemm_w4a4 keep a workspace per (device, stream) pair, see there;
 *   - return value 0 on success, a negative SVDQ_E* code otherwise; arguments are validated before
 *     anything is launched, so a failed call has no side effect;
 *   - `svdq_last_error()` returns a thread-local human-readable message for the last failure.
 *
 * Notation: M tokens, M_pad = M rounded up to 256, K in-features, N out-features, R low-rank rank,
 * G group size (64 for INT4, 16 for NVFP4).
 *
 * INT4 operands (activations and weights alike) are held as E2M3 (fp6) patterns of code / 8 -- exact
 * for every code in [-15, 15]; the pattern is the sign bit and the 4-bit magnitude -- in "fragments": one operand of the fp6 matrix instruction, 32 rows x
 * one 64-wide k-group = 1536 bytes.  Slot s = row + 32 * half (half: which 32 of the 64 codes) owns a
 * 192-bit string, code j of its half in bits [6 j, 6 j + 6); the first 16 bytes of the string lie at
 * byte 16 s of the fragment, the last 8 at 1024 + 8 s.  Activations: [M_pad/128][K/64][4 fragments]
 * (0.75 byte per element); weights: [ceil(N/256)][K/64][8 fragments], columns beyond N zero.
 */
#ifndef SVDQ_AMD_H
#define SVDQ_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SVDQ_OK 0
#define SVDQ_EINVAL -1       /* null pointer, bad shape, bad alignment */
#define SVDQ_EUNSUPPORTED -2 /* valid request that this build does not implement */
#define SVDQ_ELAUNCH -3      /* the HIP runtime refused the launch */

#define SVDQ_ABI_VERSION 5

int svdq_abi_version(void);
const char *svdq_last_error(void);

/* ------------------------------------------------------------------------------------------
 * Load-time repack: reference storage layout -> native layout.  Each runs once per tensor.
 * The reference layouts are the ones NunchakuWeightPacker writes
 * (nunchaku/lora/flux/packer.py:187-398) and the CUDA loaders read
 * (src/kernels/zgemm/gemm_base.cuh:265-340,474-489, lora.cuh:43-59, gemm_w4a4.cuh:46-83).
 * ------------------------------------------------------------------------------------------ */

/* qweight int8 [N, K/2] (reference lane order, two's complement nibbles)
 *   INT4 (fp4 == 0) -> E2M3 fragments [ceil(N/256)][K/64][8], ceil(N/256) * 256 * K * 3 / 4 bytes;
 *   NVFP4 (fp4 != 0) -> int8 [N, K/2]: tiles [N/32][K/64][32 rows][32 bytes], byte b of a (row, group)
 *      holds elements 2b (low nibble) and 2b+1 (high nibble), patterns unchanged.
 * Replaces the implicit layout contract of packed_wgt_t loads, gemm_base.cuh:278-294. */
int svdq_repack_qweight(const void *src, void *dst, int64_t N, int64_t K, int fp4, void *stream);

/* INT4 wscales bf16 [K/64, N] (reference lane order) -> native [ceil(N/256)][K/64][256 columns] x 8 bytes
 * {bf16(64 * scale), 0, 0, 0}: the operand of the matrix instruction that forms the per-group factor
 * (the 64 undoes the division by 8 of both operands' codes; columns beyond N hold zero).
 * ceil(N/256) * 256 * (K/64) * 8 bytes.  Replaces packed_wscale_t loads, gemm_base.cuh:474-489. */
int svdq_repack_wscales(const void *src, void *dst_scales, int64_t N, int64_t K, void *stream);

/* NVFP4 micro scales fp8-e4m3 [K/16, N] (reference lane order) -> native fp16 [K/64][N][4] (the four
 * 16-groups of a 64-wide k tile side by side) and fp32 colnorm [N], normalised as above.
 * Replaces packed_wmscale_t loads, gemm_w4a4.cuh:75-83. */
int svdq_repack_wmscales(const void *src, void *dst_scales, void *dst_colnorm, int64_t N, int64_t K, void *stream);

/* bias / smooth_factor / wcscales bf16 [N] (reference lane order) -> bf16 [N] in channel order.
 * Replaces the packed_wscale_t view of these vectors, gemm_w4a4_launch_impl.cuh:186-187,294. */
int svdq_repack_vector(const void *src, void *dst, int64_t N, void *stream);

/* smooth_factor bf16 [K] (reference lane order) -> fp32 [K] holding the correctly rounded
 * reciprocal 1/smooth[k] in channel order (what the quantizer multiplies by). */
int svdq_repack_smooth(const void *src, void *dst_rcp, int64_t K, void *stream);

/* proj_down bf16 [K, R] (reference lane order) -> native bf16 [K/128][4][R/16][64][8]: operand
 * order of the 16x16x32 bf16 MFMA used by the quantize kernel.  Replaces lora.cuh:43-59. */
int svdq_repack_lora_down(const void *src, void *dst, int64_t K, int64_t R, void *stream);

/* proj_up bf16 [N, R] (reference lane order) -> bf16 [N, R] row-major in channel/rank order. */
int svdq_repack_lora_up(const void *src, void *dst, int64_t N, int64_t R, void *stream);

/* Rotary table fp32 [rows, 128] in the order written by pack_rotemb (nunchaku/models/embeddings.py:88-120:
 * per 16 rows and 8 floats the fp32 accumulator fragment of an m16n8 MMA; loaded by
 * EpilogueRMSNormRope::load_rotemb, src/kernels/zgemm/epilogues.cuh:282-305) -> the order the GEMM
 * epilogue reads, [rows/32][16][64][4] (see svdq_gemm_args.rotary_emb).  rows: a multiple of 32. */
int svdq_repack_rotemb(const void *src, void *dst, int64_t rows, void *stream);

/* ------------------------------------------------------------------------------------------
 * Operator 1: smooth + quantize activations + low-rank down projection, one pass over x.
 * Replaces ops.quantize_w4a4_act_fuse_lora (nunchaku/csrc/ops.h:82-110 ->
 * src/kernels/zgemm/gemm_w4a4_launch_impl.cuh:450-521, kernel gemm_w4a4.cuh:1097-1184).
 * ------------------------------------------------------------------------------------------ */
typedef struct svdq_quantize_args {
    const void *input;      /* bf16 [M, K] row-major */
    void *output;           /* INT4: E2M3 fragments [M_pad/128][K/64][4], M_pad * K * 3 / 4 bytes;
                               NVFP4: u8 [M_pad, K/2] tiles [M_pad/32][K/64][32 rows][32 B]         */
    void *oscales;          /* INT4: bf16 [K/64][M_pad]; NVFP4: fp8-e4m3, K/16 * M_pad values stored as
                               [K/64][M_pad][4] (four 16-groups of a 64-group side by side)      */
    const void *lora_down;  /* native proj_down (svdq_repack_lora_down) or NULL when R == 0       */
    float *lora_act_out;    /* fp32 [M_pad, R] row-major; fully written (no pre-zero needed)       */
    const float *smooth_rcp;/* fp32 [K] from svdq_repack_smooth, or NULL for no smoothing          */
    int64_t M, M_pad, K, R; /* R: a multiple of 16 up to 1024; above 128 the projection takes one more
                               launch over x per 128 ranks                                          */
    int32_t fp4;            /* 0: INT4 group 64 (signed); 1: NVFP4 group 16                        */
    int32_t fuse_glu;       /* 1: input is bf16 [M, 2K], pairs (value, gate); the K columns that are
                               quantized and projected are bf16(value * bf16(gate * sigmoid(gate)))
                               (load_act_to_fpsum<fuse_glu>, gemm_base.cuh:612-623)                */
} svdq_quantize_args;

int svdq_quantize_w4a4_act_fuse_lora(const svdq_quantize_args *args, void *stream);

/* ------------------------------------------------------------------------------------------
 * Operator 2: W4A4 GEMM with fused epilogue.
 * Replaces ops.gemm_w4a4 (nunchaku/csrc/ops.h:10-80 -> gemm_w4a4_launch_impl.cuh:7-424, kernels
 * gemm_w4a4.cuh:1046-1095 and :358-405).  Epilogue order (launch_impl.cuh:172-280):
 *   acc * alpha * wcscales + bias -> + low-rank up -> GELU/SiLU -> [low-rank down of the next
 *   layer] -> store bf16 `out` and/or shift + smooth + quantize for the next layer (`qout`).
 * The GELU is applied exactly when `qout` is given (launch_impl.cuh:282-309).
 *
 * INT4 runs on the fp6 matrix instruction (one workgroup per 128 x 256 output tile); NVFP4 runs on the
 * fp16 matrix instruction with dequantized operands (persistent workgroups, 256 x 256 tiles).
 *
 * Workspace.  Most INT4 calls need none and touch no global state.  Four kinds of call keep a
 * workspace per (device, stream) pair, allocated with hipMalloc the first time the pair needs it:
 *   - INT4 with so few output tiles that they are split along K (no more tiles than compute units and a long
 *     enough K, or k_split > 1): 128 KB of fp32 partial sums per tile and part, at most 64 MB by the library's
 *     own choice;
 *   - next_lora_down: 4 bytes per element of next_lora_act_out and 256-column block of N (128 for NVFP4) (every
 *     block leaves its share there and a small kernel launched behind the GEMM adds the shares in ascending
 *     order, so the result does not depend on the order in which the blocks finish);
 *   - out_vk: 4224 bytes per head and 128 rows (NVFP4: 32 rows);
 *   - NVFP4 whenever the number of 256 x 256 tiles is not a multiple of the number of compute units:
 *     512 KB per compute unit.
 * A block that a launch has used is never freed or moved by a later call: a HIP graph that captured a call keeps
 * the block's address.  A pair that comes to need more gets a new block at least half as large again and the old
 * one stays allocated (all the blocks a pair has outgrown are smaller than twice its present one); nothing
 * synchronises.  svdq_release_workspaces frees them all.  A call that would have to allocate while its stream is
 * being captured returns SVDQ_EUNSUPPORTED: make the call once before the capture (the block is then there), or
 * use svdq_gemm_w4a4_noalloc, the variant for callers that cannot allocate.
 * Calls on one stream run in order and share the workspace safely; the same stream must not be used
 * from two threads at once.
 *
 * Ranks: R_up and R_down are multiples of 16 up to 1024 (the reference's MAX_RANK, lora.cuh:22).
 * ------------------------------------------------------------------------------------------ */
typedef struct svdq_gemm_args {
    const void *act;        /* as written by operator 1 (INT4: E2M3 fragments; NVFP4: nibble tiles)     */
    const void *ascales;    /* as written by operator 1: bf16 [K/64][M_pad] or fp8 [K/64][M_pad][4] */
    const void *wgt;        /* native qweight (svdq_repack_qweight)                                 */
    const void *wscales;    /* native scales (svdq_repack_wscales / _wmscales)                      */
    const float *colnorm;   /* NVFP4: fp32 [N] from svdq_repack_wmscales; INT4: ignored, may be NULL */
    const void *bias;       /* bf16 [N] channel order, or NULL                                      */
    const void *wcscales;   /* bf16 [N] channel order, or NULL; NVFP4 with a low-rank branch: no element may
                               be zero (the low-rank term is added in units of the column factor); the
                               Python wrappers check it once per tensor, a caller of the C ABI must     */
    const float *lora_act_in; /* fp32 [M_pad, R_up] row-major, or NULL                              */
    const void *lora_up;    /* bf16 [N, R_up] (svdq_repack_lora_up), or NULL                        */
    const float *lora_scales; /* HOST pointer, ceil(R_up/16) floats, or NULL for all ones           */
    void *out;              /* bf16 [M_out, N_out] row-major, or NULL                               */
    /* next-layer fusion (all NULL unless qout is given) */
    void *qout;             /* the next layer's activations, in operator 1's output format           */
    void *oscales;          /* bf16 [N/64][M_pad] (INT4 unsigned) or fp8 [N/64][M_pad][4] (NVFP4)   */
    const float *next_smooth_rcp; /* fp32 [N] from svdq_repack_smooth of the next layer             */
    const void *next_lora_down;   /* native proj_down of the next layer ([N, R_down]) or NULL       */
    float *next_lora_act_out;     /* fp32 [M_pad, R_down]; fully written by the call                */
    int64_t M_pad, N, K;
    int64_t M_out, N_out;   /* shape of `out` (M_out <= M_pad, N_out <= N)                          */
    int64_t R_up, R_down;
    float alpha;            /* per-tensor scale (NVFP4 wtscale; the reference asserts 1 for INT4,
                               launch_impl.cuh:107, this library applies whatever is given)          */
    int32_t act_unsigned;   /* INT4 activations are unsigned codes 0..15                            */
    int32_t fuse_silu;      /* x * sigmoid(x) before the store (EpilogueSilu, gemm_base.cuh:783-792);
                               only with `out` alone, as in launch_impl.cuh:404-417                  */
    int32_t fp4;            /* operands are NVFP4                                                   */
    /* RMS norm + rotary embedding of the q and k thirds of a fused QKV projection (all NULL / 0
     * otherwise).  Replaces EpilogueRMSNormRope, src/kernels/zgemm/epilogues.cuh:269-425, composed as in
     * gemm_w4a4_launch_impl.cuh:347-402 (after bias and low-rank up, before the store).  Columns
     * [0, N/3) are q, [N/3, 2N/3) are k, the rest (v) passes through; heads are 128 columns wide;
     * N must be a multiple of 384.  Per row and head: x *= rsqrt(mean(x^2) + norm_eps) * weight, then
     * every pair (x[2i], x[2i+1]) is rotated by (sin, cos) = rotary_emb[row][2i], [2i+1].          */
    const void *norm_q;     /* bf16 [128]                                                           */
    const void *norm_k;     /* bf16 [128]                                                           */
    const float *rotary_emb;/* fp32, rot_rows * 128 values in the order [rot_rows/32][16][64][4]: block b,
                               slot s = 4 nt + q, lane l = r + 32 h hold floats 32 nt + 8 q + 4 h + [0, 4)
                               of row 32 b + r, where float 2i of a row is sin and 2i + 1 cos of pair i
                               (svdq_repack_rotemb writes it from the reference's pack_rotemb order)  */
    int64_t rot_rows;       /* rows of rotary_emb: M_out <= rot_rows <= M_pad, a multiple of 32      */
    float norm_eps;         /* the reference uses 1e-6 (launch_impl.cuh:374)                        */
    int32_t k_split;        /* 0: the library decides.  n > 0: split every output tile along K into n parts
                               whose partial sums meet in the workspace (1: never split); a tuning and
                               testing knob with no counterpart in the reference                      */
    /* Separate q / k / v outputs of a fused QKV projection, in place of `out` (all NULL / 0 otherwise; needs
     * rotary_emb).  Replaces EpiloguePackQKV, src/kernels/zgemm/epilogues.cuh:427-550, composed after the norm
     * and rotation as in gemm_w4a4_launch_impl.cuh:380-397.  Each tensor is fp16 [heads = N/384][qkv_rows][128],
     * head h at h * qkv_head_stride[i] elements (i = 0, 1, 2 for q, k, v: the tensors may be row ranges of larger
     * ones, as in nunchaku/models/attention_processors/flux.py:139-160); values are fp16(bf16(x)) as in the
     * reference (epilogues.cuh:446-453).  Rows [attn_tokens, qkv_rows) are written with the reference's mask
     * values: 0 in q and v, NaN in k (epilogues.cuh:539-545).  Within a head the reference orders the values for
     * its own attention kernel's matrix fragments; here they are plain [row][128], the order attention kernels
     * on this hardware read.                                                                             */
    void *out_q, *out_k, *out_v;
    int64_t qkv_head_stride[3];
    int64_t attn_tokens;    /* rows that hold tokens (the reference's actualM of this epilogue)              */
    int64_t qkv_rows;       /* rows written per head, attn_tokens <= qkv_rows <= M_pad                       */
    /* Linear attention (NULL / 0 otherwise).  Replaces EpilogueLiteLA,
     * src/kernels/zgemm/epilogues.cuh:552-681, selected as in gemm_w4a4_launch_impl.cuh:311-345 (with `out` alone,
     * after bias and low-rank up).  N = 3 * heads * 32.  Columns [0, N/3) are q: `out` = bf16 [M_pad, N/3] receives
     * relu(q) (the reference's out_linearattn).  The other columns hold, per head, 32 of k then 32 of v, and
     *   out_vk[b][head][i][j] = sum over the vk_rows rows of batch entry b of v[row][i] * relu(k[row][j]),  i < 32,
     *   out_vk[b][head][32][j] = sum of relu(k[row][j]),
     * on the bf16-rounded values, accumulated in fp32.  Every row of the GEMM counts, padding rows included, as in
     * the reference.  out_vk is fully written (the reference clears it first and adds with atomics in the order of
     * arrival, :335, :649): every row block of a workgroup leaves its sums in the workspace and a small kernel launched behind the
     * GEMM adds them in ascending order, so the result is the same from run to run.                             */
    float *out_vk;          /* fp32 [M_pad / vk_rows][2 N / 3 / 64][33][32]                                   */
    int64_t vk_rows;        /* rows per batch entry: a multiple of 256 that divides M_pad                     */
} svdq_gemm_args;

int svdq_gemm_w4a4(const svdq_gemm_args *args, void *stream);

/* The same operator for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  It runs the
 * same kernels as svdq_gemm_w4a4 and gives the same results bit for bit, but calls that need a workspace
 * (see above) take it from a fixed array in device memory (81 MB on every GPU the library runs on, held
 * until the process ends: 1 MB for arrival counters, 80 MB for partial sums and low-rank shares) instead
 * of allocating one: no hipMalloc, hipFree or other allocating call is made.  A call whose need exceeds
 * the array returns SVDQ_EUNSUPPORTED with a message that says how much it wanted (examples that fit:
 * INT4 M_pad = 256, K = N = 3072 split six ways (k_split = 6), 18.9 MB of partial sums; next_lora_down at
 * M_pad = 4608, N = 12288, R_down = 32, 28.3 MB of shares).  All calls on one GPU share the array, whatever their stream: calls that overlap
 * in time on one GPU race with each other.  What a launch needs to be zero at its start is cleared by a
 * fill kernel on `stream` first. */
int svdq_gemm_w4a4_noalloc(const svdq_gemm_args *args, void *stream);

/* Frees every workspace block svdq_gemm_w4a4 has allocated, on all devices, after waiting for the work
 * enqueued on them (hipDeviceSynchronize).  No counterpart in the reference (which allocates per call
 * through its tensor type).  The caller promises that no other thread is inside svdq_gemm_w4a4 and that no
 * HIP graph that captured a call of it will be replayed afterwards.  Later calls allocate again. */
int svdq_release_workspaces(void);

/* ------------------------------------------------------------------------------------------
 * Linear attention, second half: q[b][t][h][:] <- (vk[b][h][:32] q) / (vk[b][h][32] . q + eps), in place.
 * Replaces kernels::linearattn_vk_mul_q (src/kernels/zgemm/zgemm.h:37 ->
 * gemm_w4a4_launch_impl.cuh:427-448, kernel epilogues.cuh:683-744; the reference passes eps = 1e-6).
 * q: bf16 [batch][tokens_pad][heads][32], the `out` of svdq_gemm_w4a4 with out_vk; vk: its out_vk.
 * Rows num_tokens .. tokens_pad of every batch entry are left as they are.
 * ------------------------------------------------------------------------------------------ */
int svdq_linearattn_vk_mul_q(void *q, const float *vk, int64_t batch, int64_t num_tokens, int64_t tokens_pad, int64_t heads,
                             float eps, void *stream);

/* ------------------------------------------------------------------------------------------
 * AWQ W4A16 GEMV (the other quantized linear of the reference's models: modulation layers, text
 * encoder), for 1..8 rows of x.  Replaces ops.gemv_awq (nunchaku/ops/gemv.py ->
 * src/kernels/awq/gemv_awq.cu:84-294) and the bias add of AWQW4A16Linear.forward
 * (nunchaku/models/linear.py:172-186).  out[m, n] = sum_k bf16(code[n, k] * scales[k/64, n] +
 * zeros[k/64, n]) * x[m, k], fp32 accumulation, bf16 result (+ bias, added to the bf16 result).
 * qweight is read in the reference's own storage (no repack).
 * ------------------------------------------------------------------------------------------ */
typedef struct svdq_awq_gemv_args {
    const void *x;        /* bf16 [M, K] row-major                                                   */
    const void *qweight;  /* int32 [N/4, K/2] as stored by the reference (tinychat_utils.py:76-106)  */
    const void *scales;   /* bf16 [K/64, N]                                                          */
    const void *zeros;    /* bf16 [K/64, N]: minus the scaled zero point                             */
    const void *bias;     /* bf16 [N] or NULL                                                        */
    void *out;            /* bf16 [M, N] row-major                                                   */
    int64_t M, N, K;      /* 1 <= M <= 8 (gemv_awq.cu:262), N % 4 == 0, K % 64 == 0                  */
    int32_t group_size;   /* must be 64 (gemv_awq.cu:263)                                            */
} svdq_awq_gemv_args;

int svdq_awq_gemv_w4a16(const svdq_awq_gemv_args *args, void *stream);




#ifdef __cplusplus
}
#endif
#endif /* SVDQ_AMD_H */
