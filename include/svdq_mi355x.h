/*
 * svdq_mi355x.h -- C ABI of the MI355X (gfx950) SVDQuant kernel library (libsvdq_mi355x.so).
 *
 * Plain pointers and sizes only; every pointer is a device pointer unless stated otherwise, every
 * buffer is owned by the caller, and the library allocates nothing.  All launches are asynchronous on the
 * given stream (a hipStream_t passed as void*; NULL = the default stream).  Functions return 0 on success or a
 * negative SVDQ_E_* code; svdq_last_error() gives the message for the calling thread.
 *
 * "T" below is bfloat16 (dtype code SVDQ_BF16) or float16 (SVDQ_FP16); one T per call.
 *
 * Each entry point replaces one binding of the reference (paths relative to the reference checkout):
 *   svdq_quantize_act        nunchaku/ops/quantize.py:82-87      (_C.ops.quantize_w4a4_act_fuse_lora /
 *                                                                 ops/triton/gemm_w4a4.py:1521 quantize_w4a4_act_fuse_lora)
 *   svdq_gemm_w4a4           nunchaku/ops/gemm.py:151-207        (_C.ops.gemm_w4a4 / ops/triton/gemm_w4a4.py:1003 gemm_w4a4),
 *                            kernel-argument structs modelled on ops/triton/native/w4a4.py:80-124
 *   svdq_awq_gemv_w4a16      nunchaku/ops/dispatch.py:19-34      (_C.ops.gemv_awq / ops/triton/awq.py:186 awq_gemv_w4a16)
 *   svdq_awq_dequantize      nunchaku/ops/dispatch.py:37-49      (_C.ops.gemm_awq / ops/triton/awq.py:83 awq_dequantize + torch.matmul)
 *   svdq_attention_fp16      nunchaku/ops/dispatch.py:67-99      (_C.ops.attention_fp16 / ops/triton/attention.py:111 attention_fp16)
 *   svdq_row_stats           nunchaku/models/normalization.py:97 (the LayerNorm statistics; applied inside svdq_quantize_act)
 *   svdq_gated_residual      nunchaku/models/transformers/transformer_flux_v2.py:233-243, :326-330 (gate * y + residual)
 *   svdq_unpack_mma_*        nunchaku/ops/triton/layout.py:36-292 (checkpoint layout -> natural layout)
 *   svdq_transpose_lora_down no counterpart: one-time re-layout of a LoRA-down weight, see below
 *   svdq_group_acc_i32       no counterpart: debug read-out of the exact int32 group accumulators
 */
#ifndef SVDQ_MI355X_H
#define SVDQ_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SVDQ_ABI_VERSION 9

enum { SVDQ_BF16 = 0, SVDQ_FP16 = 1 };
enum { SVDQ_PRE_NONE = 0, SVDQ_PRE_GLU = 1, SVDQ_PRE_GELU = 2 }; /* svdq_quantize_args.prologue */

enum {
    SVDQ_OK = 0,
    SVDQ_E_INVALID = -1,     /* bad shape / alignment / combination of arguments */
    SVDQ_E_UNSUPPORTED = -2, /* valid in the reference, not implemented here      */
    SVDQ_E_LAUNCH = -3       /* HIP reported an error for the launch              */
};

/* Epilogue of svdq_gemm_w4a4 (reference: ops/triton/gemm_w4a4.py:1151-1205 dispatch). */
enum {
    SVDQ_EPI_PLAIN = 0,        /* bias + LoRA-up, store T                                             */
    SVDQ_EPI_QK_NORM_ROPE = 1, /* + per-head RMSNorm and RoPE on the Q and K thirds (gemm_w4a4.py:499) */
    SVDQ_EPI_GELU_QUANT = 2,   /* + GELU, next layer's LoRA-down, +shift, unsigned int4 requantization  */
    SVDQ_EPI_SWIGLU_QUANT = 3  /* + silu(gate)*up on 16-interleaved columns, signed int4 requantization */
};

/*
 * Activation quantizer: per-channel smooth divide, per-group-64 absmax int4 quantization, fused LoRA-down.
 * Reference arithmetic: ops/triton/gemm_w4a4.py:1397-1455 (int4 branches).  Rows >= M of out/scales/lora_act
 * are never written.
 */
typedef struct {
    const void *x;           /* (M, K) T, row stride ld_x elements                                          */
    const void *smooth;      /* (K,) T or NULL                                                              */
    const void *lora_down_t; /* (R, K) T: the (K, R) LoRA-down weight transposed, row stride K; NULL iff R=0 */
    void *out;               /* (>= M, K/2) uint8, low nibble = even k, row stride ld_out bytes             */
    void *scales;            /* (K/64, >= M) T, element [g, m] at g*ld_scales + m                           */
    float *lora_act;         /* (>= M, R) fp32, row stride ld_lora_act elements; NULL iff R=0               */
    int32_t M, K, R;         /* K % 64 == 0, R % 16 == 0                                                    */
    int32_t ld_x, ld_out, ld_scales, ld_lora_act;
    int32_t dtype;           /* SVDQ_BF16 / SVDQ_FP16                                                       */
    int32_t is_unsigned;     /* 0: codes in [-8, 7], absmax / 7;  1: codes in [0, 15], max / 15             */
    int32_t prologue;        /* SVDQ_PRE_NONE; SVDQ_PRE_GLU: x is (M, 2K) and the quantized value is
                              * x[:, :K] * silu(x[:, K:]) (fuse_glu); SVDQ_PRE_GELU: tanh-GELU of x (fuse_gelu,
                              * ops/triton/gemm_w4a4.py:1403-1408): the LoRA-down sees the result rounded to T */
    float shift;             /* added before smoothing (0.171875 after GELU, else 0)                        */
    /* Optional norm prologue (NULL norm_stats = off; only with SVDQ_PRE_NONE): the quantized and LoRA-projected value is
     * T(T(T((x - mean[m]) * rstd[m]) * norm_scale[k]) + norm_shift[k]), i.e. LayerNorm without affine followed by the
     * adaLN modulate, each step rounded to T as separate elementwise kernels would
     * (nunchaku/models/normalization.py:97-104, models/transformers/transformer_flux_v2.py:236-237). */
    const float *norm_stats;       /* (M, 2) fp32 rows of (mean, rstd), from svdq_row_stats                  */
    const void *norm_scale;        /* (batches, K) T: element (b, k) at b * norm_ld + k * norm_stride        */
    const void *norm_shift;        /* (batches, K) T, same strides                                           */
    int32_t norm_rows_per_batch;   /* rows m sharing one scale / shift vector (multiple of 16); 0 = all rows */
    int32_t norm_ld, norm_stride;  /* in elements (the adaLN projection interleaves its six vectors: stride 6) */
    /* How `out` is written (no counterpart in the reference; 1 and 2 need `out` 16-byte aligned and holding            */
    /* ceil(M / 32) * 32 rows' worth, ld_out is then not used):                                                         */
    /*   0  the (M, K / 2) matrix of packed int4 codes;                                                                 */
    /*   1  the same bytes in the lane order of the GEMM's fp8 main loop: the 32 packed bytes of (row m, group g) go to  */
    /*      out + ((m / 32) * (K / 64) + g) * 1024 + (32 * h + m % 32) * 16, h = 0 / 1 for bytes 0-15 / 16-31; the GEMM  */
    /*      takes it with svdq_gemm_args.act_blocked = 1 and reads 1 KB per load instruction instead of 16-byte pieces   */
    /*      of 32 rows (about 3 % of a launch);                                                                          */
    /*   2  the same integers as fp6 (e2m3) codes, sign << 5 | magnitude, in that lane order: 48 bytes per row and group. */
    /*      Of (row m, group g), lane 32 h + m % 32 owns the values k = 2 p + h (p = 0 .. 31), code p in bits 6 p .. 6 p + 5 */
    /*      of 24 bytes; their first 16 lie at out + ((m / 32) * (K / 64) + g) * 1536 + 16 * lane, their last 8 at          */
    /*      ... + 1024 + 8 * lane.  The GEMM takes it with act_blocked = 2: the matrix instruction reads the codes as they  */
    /*      are (fp6 x fp6, no nibble unpack, no offset term for signed activations; about 8 % of a launch).               */
    int32_t out_blocked;
    /* non-zero: `scales` is written for the GEMM's svdq_gemm_args.ascales_blocked: the eight scales of groups 8 j .. 8 j + 7 */
    /* of a row side by side, element ((m / 32) * (K / 512) + g / 8) * 256 + (m % 32) * 8 + g % 8 (K must be a multiple of  */
    /* 512; the buffer holds ceil(M / 32) * 32 * (K / 64) elements, 16-byte aligned; ld_scales is not used).  No          */
    /* counterpart in the reference.                                                                                      */
    int32_t scales_blocked;
} svdq_quantize_args;

int svdq_quantize_act(const svdq_quantize_args *args, void *stream);

/* Per-row mean and 1 / sqrt(biased variance + eps) of x (M, K) T in fp32: stats[m] = (mean, rstd).  The statistics
 * LayerNorm needs (nunchaku/models/normalization.py:97), for the quantizer's norm prologue. */
int svdq_row_stats(const void *x, float *stats, int32_t M, int32_t K, int32_t ld_x, int32_t dtype, float eps,
                   void *stream);

/* Gated residual update of a transformer block, one pass: out[m, k] = T(x[m, k] + T(gate[b, k] * t[m, k])) with
 * t = y, or T(y + y2) when y2 is given (the three elementwise torch kernels of
 * nunchaku/models/transformers/transformer_flux_v2.py:233-234, :241-243 and :326-330, each step rounded to T), and,
 * when stats is not NULL, the (mean, rstd) row statistics of out for the next layer's norm prologue.  gate element
 * (b, k) is at b * gate_ld + k * gate_stride with b = m / rows_per_batch (rows_per_batch 0 = one vector).
 * clip > 0: out is limited to [-clip, clip] before it is stored and before the statistics (the model's
 * `hidden_states.clip(-65504, 65504)` of fp16 runs, transformer_flux_v2.py:255-256, :340-341); 0 = off.
 * K % 8 == 0, K <= 8192; x, y, y2, out rows 16-byte aligned with the row strides ld_* in elements; out may be x. */
int svdq_gated_residual(const void *x, const void *gate, const void *y, const void *y2, void *out, float *stats,
                        int32_t M, int32_t K, int32_t ld_x, int32_t ld_y, int32_t ld_out, int32_t rows_per_batch,
                        int32_t gate_ld, int32_t gate_stride, int32_t dtype, float eps, float clip, void *stream);

/* (K, R) row-major T  ->  (R, K) row-major T.  Done once per weight; the quantizer and the fused
 * requantizing epilogues read the transposed form so their MFMA operands are K-contiguous. */
int svdq_transpose_lora_down(const void *lora_down, void *lora_down_t, int32_t K, int32_t R, int32_t ld_in,
                             void *stream);

/*
 * W4A4 GEMM: out[m, n] = sum_g as[g, m] * ws[g, n] * (sum_{k in g} a[m, k] w[n, k])  (exact integer per group: int8 MFMA
 *                        on packed weights, fp8 x fp6 MFMA on int4-valued codes with pre-split weights)
 *                        + T(lora_act[m, :]) . lora_up[n, :] + bias[n],  then the epilogue.
 * Reference arithmetic: ops/triton/gemm_w4a4.py:447-488 (main loop), 156-209 (epilogue), 499-521 (QK), 730-778
 * (GELU + requantization), 998-1000 (SwiGLU semantics).
 */
typedef struct {
    const void *act;        /* (M, K/2) packed int4, row stride ld_act bytes (multiple of 16, base 16-B aligned) */
    const void *wgt;        /* (N, K/2) packed signed int4, row stride ld_wgt bytes (same alignment); not read,  */
                            /* and may be NULL, when wgt_planes is given                                         */
    const void *wgt_planes; /* optional: the same weights and `wscales` re-laid-out by svdq_split_weight_planes  */
                            /* (then `wgt` is not read, fp8 main loop); NULL = unpack `wgt` inside the GEMM      */
                            /* (int8 main loop)                                                                  */
    const void *ascales;    /* (K/64, >= M) T, group stride ld_ascales elements                                 */
    const void *wscales;    /* (K/64, >= N) T, group stride ld_wscales elements                                 */
    const void *bias;       /* (N,) T or NULL                                                                   */
    const float *lora_act;  /* (>= M, R) fp32, row stride ld_lora_act; NULL iff R = 0                           */
    const void *lora_up;    /* (N, R) T, row stride ld_lora_up; NULL iff R = 0                                  */
    void *out;              /* (actual_m, N) T, row stride ld_out (rows 16-byte aligned: base and ld_out % 8);   */
                            /* may be NULL for the requantizing epilogues                                       */
    int32_t M, N, K, R;     /* K % 64 == 0, N % 8 == 0, R % 16 == 0                                             */
    int32_t actual_m;       /* rows of out that exist (<= M); rows beyond are computed but never written       */
    int32_t ld_act, ld_wgt, ld_ascales, ld_wscales, ld_lora_act, ld_lora_up, ld_out;
    int32_t dtype;
    int32_t act_unsigned;   /* activation nibbles are [0, 15] instead of two's complement                       */
    int32_t epilogue;       /* SVDQ_EPI_*                                                                       */
    /* SVDQ_EPI_QK_NORM_ROPE: N = 3 * heads * 128 */
    const void *norm_q;     /* (128,) T  */
    const void *norm_k;     /* (128,) T  */
    const float *rotary;    /* (actual_m, 128) fp32 rows of (sin, cos) pairs, row stride ld_rotary elements     */
    int32_t ld_rotary;
    float eps;
    /* SVDQ_EPI_GELU_QUANT / SVDQ_EPI_SWIGLU_QUANT: NQ = N (GELU) or N/2 (SwiGLU) quantized columns */
    void *qout;               /* (>= M, NQ/2) uint8, row stride ld_qout bytes                                   */
    void *oscales;            /* (NQ/64, >= M) T, group stride ld_oscales                                       */
    const void *smooth_next;  /* (NQ,) T or NULL                                                                */
    const void *lora_down_t;  /* (R2, NQ) T, the next layer's (NQ, R2) LoRA-down transposed; NULL iff R2 = 0    */
    float *lora_act_out;      /* (>= M, R2) fp32, row stride ld_lora_act_out                                    */
    float *scratch;           /* svdq_gemm_w4a4_scratch_bytes() bytes of fp32 LoRA-down partial sums, or NULL    */
    int32_t R2, ld_qout, ld_oscales, ld_lora_act_out;
    float shift;              /* 0.171875 for GELU (ops/triton/gemm_w4a4.py:918), 0 for SwiGLU                  */
    /* SVDQ_EPI_QK_NORM_ROPE, optional: the same table as `rotary`, re-laid-out by svdq_block_rotary (the fp8 main    */
    /* loop's epilogue then reads 1 KB per load instruction instead of 32-byte pieces of 32 rows); NULL = not given  */
    const float *rotary_blocked;
    /* SVDQ_EPI_GELU_QUANT, optional: `lora_down_t` re-laid-out by svdq_block_lora_down (the epilogue then reads each of */
    /* its LoRA-down operands as 1 KB in a row instead of 8-byte pieces of 32 rows); NULL = not given                   */
    const void *lora_down_blocked;
    /* 1 / 2: `act` is not the (M, K / 2) matrix but what the quantizer writes with out_blocked = 1 / 2 (its bytes, or   */
    /* fp6 codes, in the fp8 main loop's lane order; pre-split weights only; with 2 act_unsigned is not looked at)      */
    int32_t act_blocked;    /* (`act` must then hold ceil(M / 32) * 32 rows' worth, 16-byte aligned; ld_act unused) */
    /* 1 / 2: the requantizing epilogues write `qout` that way, for the GEMM that consumes it (ld_qout unused; `qout`   */
    /* must hold ceil(M / 32) * 32 rows' worth: NQ / 2 bytes a row, 3 NQ / 4 with 2)                                    */
    int32_t qout_blocked;
    /* non-zero (act_blocked = 2 only, K a multiple of 512): `ascales` in the layout of svdq_quantize_args.scales_blocked -- */
    /* one 16-byte load per lane brings the activation scales of four stages instead of two 2-byte loads per stage        */
    /* (ld_ascales unused)                                                                                                */
    int32_t ascales_blocked;
    /* non-zero: the requantizing epilogues write `oscales` in that layout (NQ a multiple of 512; ld_oscales unused)      */
    int32_t oscales_blocked;
} svdq_gemm_args;

int svdq_gemm_w4a4(const svdq_gemm_args *args, void *stream);

/*
 * One-time re-layout of a rotary table for the Q/K RMSNorm + RoPE epilogue: (rows, 128) fp32 rows of (sin, cos) pairs,
 * row stride ld_rotary elements -> ceil(rows / 32) blocks of 32 rows, each as sixteen 1 KB pieces in the order the
 * epilogue's lanes read them: piece (column block bn, j) holds, for lane (row r = lane % 32, h = lane / 32), the four
 * floats of columns 32 bn + 8 j + 4 h .. + 3 of row r (rows past the end repeat row 0, as the epilogue does for rows it
 * never stores).  `blocked` needs svdq_rotary_blocked_bytes(rows) = ceil(rows / 32) * 16 KB, 16-byte aligned.  The
 * table of a diffusion transformer is the same for every block and step, so callers make this once per table.  No
 * counterpart in the reference.
 */
int svdq_block_rotary(const float *rotary, float *blocked, int32_t rows, int32_t ld_rotary, void *stream);
size_t svdq_rotary_blocked_bytes(int32_t rows);

/*
 * One-time re-layout of the next layer's transposed LoRA-down weight (R2, N) T for the GELU + requantization epilogue:
 * per (128-column tile, chunk of 32 ranks) eight 1 KB pieces, one per matrix instruction of the tile's partial product
 * (column block bn, half s of it), in lane order: lane (rank r = lane % 32, h = lane / 32) finds the eight values
 * lora_down_t[32 c + r][128 t + 32 bn + 16 s + 4 h + {0..3, 8..11}] as 16 contiguous bytes (ranks past R2: zeros).
 * `blocked` needs svdq_lora_down_blocked_bytes(N, R2) = (N / 128) * ceil(R2 / 32) * 8 KB, 16-byte aligned; N % 128 == 0.
 * Made once per weight like the transposed copy itself.  No counterpart in the reference.
 */
int svdq_block_lora_down(const void *lora_down_t, void *blocked, int32_t N, int32_t R2, int32_t dtype, void *stream);
size_t svdq_lora_down_blocked_bytes(int32_t N, int32_t R2);

/* The fp8 main loop exists in two builds: three workgroups per CU (fills a loaded CU best) and two per CU with
 * software-pipelined steps (a workgroup on its own runs faster); svdq_gemm_w4a4 picks by the number of 128x128 tiles and
 * CUs.  This overrides the choice for the whole process: -1 = by tile count (default), 0 = three per CU, 1 = two per CU.
 * For tuning and tests; results of the two are bit-identical.  No counterpart in the reference. */
int svdq_gemm_w4a4_set_variant(int32_t variant);

/*
 * One-time re-layout of a weight for the GEMM.  Every (32-row block, pair of scale groups = one stage of the main
 * loop) becomes three 1 KB blocks of fp6 (e2m3) codes in the order the MFMA lanes read them: a signed int4 value v is
 * stored as the six bits sign | |v|, which the matrix instruction reads as v / 8 exactly; a lane's 32 weights of a
 * group are six registers (blocks 0 and 1: registers 0-3 of the pair's first and second group, block 2: registers 4-5
 * of both; a missing second group is zeros).  v_mfma_scale_f32_32x32x64_f8f6f4 takes them next to fp8 activation codes
 * at the int8 rate, a whole 64-deep group per instruction, and returns the integer dot product as fp32, which saves
 * the GEMM one of its two scaling multiplies per output and group.  Behind the codes sit, per (32-row block, stage),
 * 32 rows of six T values: the two pieces (hi + lo) of D = -ws[g, n] * (8 * sum of the group's even-k weights
 * - 7 * sum of its odd-k weights) for the stage's two groups, then the two weight scales themselves; each block of
 * rows has one more (zero) stage than the loop runs.  The GEMM carries a signed activation a as a + 8 for even k and
 * a - 7 for odd k (sign | magnitude fp8 codes, one bit operation per plane) and adds as[g, m] * D[g, n] back with a
 * 16-bit matrix instruction; with the two signs the offset term has no systematic part whatever the mean of the
 * weights.  The last 16 bytes are a status word: non-zero when a D piece or a scale is not finite in T (fp16 weight
 * scales above about 17: |8 We - 7 Wo| reaches 3840); such a copy must not be used (the Python cache then keeps the packed weight and the int8 loop).
 * `planes` needs svdq_weight_planes_bytes(N, K) bytes = ceil(N/32) * (ceil(K/128) * 3072 + (ceil(K/128) + 1) * 384)
 * + 16: 0.84 bytes per weight.  The copy depends on `wgt` AND `wscales` (dtype = their type); once it exists the
 * GEMM reads neither (`wgt` may then be NULL, and a caller may free the packed weight).  No counterpart in the
 * reference (its SwiGLU path re-orders weight rows at load in the same spirit, ops/fused.py:83-105).
 */
int svdq_split_weight_planes(const void *wgt, const void *wscales, void *planes, int32_t N, int32_t K, int32_t ld_wgt,
                             int32_t ld_wscales, int32_t dtype, void *stream);
size_t svdq_weight_planes_bytes(int32_t N, int32_t K);

/* Bytes of `scratch` needed by a requantizing epilogue with LoRA-down (0 when R2 == 0). */
size_t svdq_gemm_w4a4_scratch_bytes(int32_t M, int32_t N, int32_t R2, int32_t epilogue);

/*
 * svdq_gemm_w4a4 for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  `args->scratch` is ignored: the LoRA-down partial
 * sums go to a buffer of SVDQ_STATIC_SCRATCH_BYTES built into the library (one per GPU, held until the process
 * ends).  Returns SVDQ_E_UNSUPPORTED when svdq_gemm_w4a4_scratch_bytes(M, N, R2, epilogue) exceeds it.  Calls no
 * hipMalloc / hipFree.  All calls on one GPU share the buffer: calls that overlap in time on one GPU (two streams) race;
 * calls on one stream are ordered.  Results are bit-identical to svdq_gemm_w4a4's.
 */
#define SVDQ_STATIC_SCRATCH_BYTES (16u << 20)
int svdq_gemm_w4a4_static_scratch(const svdq_gemm_args *args, void *stream);
size_t svdq_gemm_w4a4_static_scratch_capacity(void);
/* Looks up the buffer's address on the current device now instead of in the first svdq_gemm_w4a4_static_scratch call
 * there: call it once per device before capturing that entry point into a HIP graph (the look-up is not a stream
 * operation).  16 MiB hold M * ceil(N / 128) * R2 * 4 bytes: at R2 = 32, M * N up to 16.8 M (M = 4608: N <= 3584); the
 * FLUX.1 fc1 shape (M = 4608, N = 12288: 56.6 MB) needs svdq_gemm_w4a4 with a caller's buffer. */
int svdq_gemm_w4a4_static_scratch_prepare(void);

/*
 * Debug: exact int32 accumulators of one scale group, p[m, n] = sum_{k in group g} a[m, k] * w[n, k], computed by
 * the instruction sequence of one of the GEMM's two main loops: path 0 = nibble unpack + v_mfma_i32_32x32x32_i8 (packed
 * weights), path 1 = fp8 / fp6 codes + v_mfma_scale_f32_32x32x64_f8f6f4 with the +8 offset of signed activations taken out
 * (pre-split weights).  out (M, N) int32 row-major.
 */
int svdq_group_acc_i32(const void *act, const void *wgt, int32_t *out, int32_t M, int32_t N, int32_t K,
                       int32_t ld_act, int32_t ld_wgt, int32_t group, int32_t act_unsigned, int32_t path, void *stream);

/*
 * AWQ W4A16 GEMV, group 64, TinyChat packing (models/text_encoders/tinychat_utils.py:76-106):
 * out[m, n] = sum_c s[c, n] * sum_{k in c} x[m, k] q[n, k] + z[c, n] * sum_{k in c} x[m, k]   (ops/triton/awq.py:160-182)
 */
typedef struct {
    const void *x;       /* (M, K) T, row stride ld_x                               */
    const void *qweight; /* (N/4, K) int16 (= (N/4, K/2) int32), row stride K int16 */
    const void *scales;  /* (K/64, N) T, group stride ld_scales                     */
    const void *zeros;   /* (K/64, N) T, same stride                                */
    void *out;           /* (M, N) T, row stride ld_out                             */
    int32_t M, N, K;     /* M <= 32, N % 32 == 0, K % 64 == 0                       */
    int32_t ld_x, ld_scales, ld_out;
    int32_t dtype;
} svdq_awq_gemv_args;

int svdq_awq_gemv_w4a16(const svdq_awq_gemv_args *args, void *stream);

/*
 * The same GEMV for `count` weights of one shape in a single launch (M <= 8).  The adaLN projections of a diffusion
 * transformer all take the same vector (models/normalization.py: silu(temb)) and do not depend on the blocks before them,
 * so they can run together; one 32 MB weight is too short a read to reach the HBM rate (launch ramp and tail), many
 * behind each other stream like one long read.  `first` (host memory) is problem 0: M, N, K, the leading dimensions and
 * the dtype hold for all problems.  `problems` is a DEVICE array of `count` svdq_awq_gemv_args (8-byte aligned), of which
 * only the five pointers x, qweight, scales, zeros, out are read; entry 0 must equal `first`'s.  Every problem's tensors
 * must meet the alignment rules of svdq_awq_gemv_w4a16: only problem 0 can be checked here, the others are the caller's to
 * check.  Results are bit-identical to count single calls.  No counterpart in the reference.
 */
int svdq_awq_gemv_w4a16_batched(const svdq_awq_gemv_args *first, const svdq_awq_gemv_args *problems, int32_t count,
                                void *stream);

/*
 * Dense decode of a TinyChat-packed AWQ weight (nunchaku/ops/triton/awq.py:48-118 awq_dequantize, the first half of
 * awq_gemm_w4a16 :232-251 and of the group_size != 64 branch of awq_gemv_w4a16 :226-228; the matmul that follows is
 * the caller's): out[n, k] = T(q[n, k] * s[k / group_size, n] + z[k / group_size, n]) in fp32.
 * qweight (N/4, K) int16 as above; scales / zeros (K / group_size, N) T with group stride ld_scales; out (N, K) T with
 * row stride ld_out.  N % 4 == 0, K % 64 == 0, group_size a multiple of 32 that divides K.
 */
int svdq_awq_dequantize(const void *qweight, const void *scales, const void *zeros, void *out, int32_t N, int32_t K,
                        int32_t group_size, int32_t ld_scales, int32_t ld_out, int32_t dtype, void *stream);

/*
 * Unmasked scaled-dot-product attention, head dimension D = 128 or 64 (nunchaku/ops/dispatch.py:67-99 attention_fp16 /
 * ops/triton/attention.py:111-169): o[b, t, h*D + d] = softmax_k(scale * q[b,h,t,:] . k[b,h,k,:]) . v[b,h,k,d], fp32
 * softmax and accumulation, P rounded to T.  Strides are in elements; the last dimension of q, k, v, o is contiguous.
 * No workspace: v is read in place (the kernel transposes its tiles on the way out of LDS).
 */
typedef struct {
    const void *q;  /* (B, H, Tq, D) T  */
    const void *k;  /* (B, H, Tkv, D) T */
    const void *v;  /* (B, H, Tkv, D) T */
    void *o;        /* (B, Tq, H * D) T */
    int64_t sqb, sqh, sqm, skb, skh, skn, svb, svh, svn, sob, som;
    int32_t B, H, Tq, Tkv, D;
    int32_t dtype;
    float scale;    /* normally D ** -0.5 */
} svdq_attention_args;

int svdq_attention_fp16(const svdq_attention_args *args, void *stream);

/*
 * Checkpoint ingestion.  The published SVDQuant int4 checkpoints hold every tensor of a quantized linear pre-shuffled
 * for the register fragments of the CUDA kernels (nunchaku/lora/flux/packer.py:173-226 pack_weight, :228-262
 * pack_scale, :300-338 pack_lowrank_weight); these undo that in one pass on the device, as the reference does at load
 * time (nunchaku/ops/triton/layout.py:36-120 unpack_weight[_packed_nibbles], :155-184 unpack_scale, :226-292
 * convert_svdq_linear_to_natural_layout).  Source and destination must not overlap.
 *
 *   weight   packed (N, K / 2) bytes            -> natural (N, K / 2) bytes, low nibble = even k; N, K multiples of 128;
 *                                                  ld_natural in bytes
 *   scale    packed groups * N 16-bit values    -> natural (groups, N); N a multiple of 128.  groups = K / 64 for
 *                                                  wscales, 1 for bias / smooth_factor / wcscales; ld_natural in elements
 *   lowrank  packed (C, R) 16-bit values        -> natural (C, R): down = 0 for proj_up (C = out features), down = 1
 *                                                  for proj_down (C = in features); C, R multiples of 16
 */
int svdq_unpack_mma_weight(const void *packed, void *natural, int32_t N, int32_t K, int32_t ld_natural, void *stream);
int svdq_unpack_mma_scale(const void *packed, void *natural, int32_t N, int32_t groups, int32_t ld_natural, void *stream);
int svdq_unpack_mma_lowrank(const void *packed, void *natural, int32_t C, int32_t R, int32_t down, int32_t ld_natural,
                            void *stream);

/* Message for the last non-zero return on the calling thread ("" if none). */
const char *svdq_last_error(void);

/* SVDQ_ABI_VERSION the library was built with. */
int svdq_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* SVDQ_MI355X_H */
