// Activation quantizer for gfx950: smooth divide, per-group-64 absmax int4 quantization and the fused LoRA-down
// projection in one pass over the activations.
//
// Arithmetic follows the reference's _quantize_tile_kernel (nunchaku/ops/triton/gemm_w4a4.py:1397-1455): fp32
// throughout, reciprocal-then-multiply for the smooth factor and for the group scale (both IEEE divides), the stored
// scale rounded to the 16-bit type while the codes use the unrounded one, round-half-to-even through the 1.5*2^23
// add, clamp, low nibble first.  The LoRA-down product consumes the raw 16-bit activations (before shift and
// smoothing) on the 16x16x32 MFMA with fp32 accumulation.
//
// Work split: one workgroup = 16 (or 32) rows x all of K, eight wavefronts taking scale groups round-robin with two
// groups in flight each; on the grid's second axis, one workgroup row per chunk of 32 LoRA ranks and, where CUs are
// left over, up to three rows that only quantize a slice of the groups each.  A group's operands (16 rows x 128 bytes of activations, 32 ranks x 128 bytes of the transposed
// LoRA-down weight (R, K)) are fetched straight into LDS (global_load_lds_dwordx4) by loads whose 64 lanes cover eight
// full 128-byte rows -- read lane-per-row from global memory, the same bytes cost the memory pipeline four times as
// many cycles -- and land in a tile whose 16-byte chunks are XOR-swizzled by the row so that the transposed read-back
// is conflict free.  Lane (m = lane % 16, q = lane / 16) then owns the 16 consecutive channels [64 g + 16 q, +16)
// of row m: a group's absmax needs two cross-lane steps, and the lane's two 16-byte halves are exactly the B operands
// of two 16x16x32 MFMAs whose A operands come from the LoRA-down tile.
//
// Output: the reference's (M, K / 2) matrix of packed nibbles and (K / 64, M) scales, or -- for the GEMM of this library --
// the same bytes in its lanes' order, or the same integers as fp6 codes in that order (from the hardware's float -> fp6
// conversion), with the scales in that order as well.
#include <algorithm>

#include "svdq_common.h"

// the codes and scales are a bit-exact contract: no multiply-add contraction anywhere in this file
#pragma clang fp contract(off)

namespace svdq {

constexpr int Q_ROWS = 16;         // rows of one MFMA pass; a workgroup takes QR = 16 or 32 rows (one or two passes)
constexpr int Q_WAVES = 8;
constexpr int Q_ROW_BYTES = 128;  // one scale group of one row (64 x 16 bit)
constexpr int Q_RCHUNK = 32;  // LoRA ranks per pass over the row block
constexpr int Q32_ABOVE = 256, Q32_UPTO = 512;  // number of 16-row workgroups for which 32-row workgroups are used instead

// sum_j (0x4B400000 << 4 j) mod 2^32: what eight magic-biased codes add up to besides their nibbles
constexpr uint32_t pack_bias() {
    uint32_t c = 0;
    for (int j = 0; j < 8; j++) c += (uint32_t)RNE_MAGIC_BITS << (4 * j);
    return c;
}

// per-group vectors a lane fetches for the group's 64 channels (one channel per lane), shared through LDS later
struct QVecs {
    uint16_t sm, ns, nh;  // smooth factor, norm scale, norm shift
};

template <typename T, bool UNSIGNED, int PRE, bool HAS_LORA, bool HAS_SMOOTH, bool NORM, int QR>
__global__ __launch_bounds__(Q_WAVES * 64, QR == 32 ? 1 : (NORM ? 4 : 2)) void quantize_act_kernel(svdq_quantize_args a) {
    constexpr bool GLU = PRE == SVDQ_PRE_GLU, GELU = PRE == SVDQ_PRE_GELU;
    constexpr int NH = QR / Q_ROWS;  // 16-row halves of the row block: each LoRA-down tile read serves all of them
    // per wavefront: two activation stages (16 rows, + the gate tile with GLU) and one LoRA-down tile (32 ranks), 128
    // bytes a row.  The LoRA-down tile is an L2 hit and the first thing a group consumes: one group ahead is enough.
    constexpr int XS_BYTES = (GLU ? 2 : 1) * QR * Q_ROW_BYTES, G_OFF = QR * Q_ROW_BYTES;
    constexpr int L_OFF = 2 * XS_BYTES;
    constexpr int WAVE_BYTES = L_OFF + (HAS_LORA ? Q_RCHUNK * Q_ROW_BYTES : 0);
    // the cross-wave sum after the loop keeps each wavefront's partial products in that wavefront's own (then idle) stages
    static_assert(!HAS_LORA || Q_RCHUNK * (QR + 1) * 4 <= WAVE_BYTES, "partial products do not fit the wavefront's stages");
    __shared__ __align__(16) uint8_t smem[Q_WAVES * WAVE_BYTES];
    __shared__ float lds_rs[Q_WAVES][64];
    __shared__ float lds_ns[NORM ? Q_WAVES : 1][64], lds_nh[NORM ? Q_WAVES : 1][64];
    auto lds_acc = [&](int w) { return (float (*)[QR + 1])(smem + w * WAVE_BYTES); };  // [Q_RCHUNK][QR + 1] of wavefront w

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: keep it in an SGPR
    const int ml = lane & 15;
    const int kq = lane >> 4;
    const int m0 = blockIdx.x * QR;
    const int ngroups = a.K / GROUP;
    // The grid's second axis: nq >= 0 workgroup rows that only quantize, each its own slice of the groups (a shorter chain
    // of group steps per wavefront where CUs would otherwise idle), then one row per chunk of 32 ranks.
    const int rchunks = (a.R + Q_RCHUNK - 1) / Q_RCHUNK;
    const int nq = HAS_LORA ? max((int)gridDim.y - rchunks, 0) : 0;
    const bool qonly = (int)blockIdx.y < nq;
    const int g_lo = qonly ? (ngroups * (int)blockIdx.y) / nq : 0, g_hi = qonly ? (ngroups * ((int)blockIdx.y + 1)) / nq : ngroups;
    const int gw = g_lo + wave;  // this wavefront's groups: gw + Q_WAVES * i < g_hi
    const int nmy = max((g_hi - gw + Q_WAVES - 1) / Q_WAVES, 0);
    // Block loads: lane l of load i fetches chunk (l % 8) ^ (l / 8) of tile row 8 i + l / 8 into LDS slot l of that
    // load's 1 KB, i.e. tile[row][chunk ^ (row & 7)].  Rows >= M re-read row M - 1 and ranks >= R rank R - 1 (valid
    // memory; nothing is stored for them).  Addresses = uniform base + 32-bit lane offset (+ uniform group step).
    const int drow = lane >> 3, dchunk = (lane & 7) ^ drow;
    const uint8_t *__restrict__ xbase = (const uint8_t *)a.x + (size_t)m0 * a.ld_x * 2;
    uint32_t xdma[2 * NH];
#pragma unroll
    for (int i = 0; i < 2 * NH; i++) xdma[i] = (uint32_t)(min(m0 + 8 * i + drow, a.M - 1) - m0) * a.ld_x * 2 + dchunk * 16;
    // read-back: lane (m, q) takes chunks 2 q and 2 q + 1 of tile row m (and of row m + 16 of the LoRA-down tile)
    const int rd_lo = ml * Q_ROW_BYTES + (((2 * kq) ^ (ml & 7)) * 16), rd_hi = ml * Q_ROW_BYTES + (((2 * kq + 1) ^ (ml & 7)) * 16);
    uint8_t *const wbase = smem + wave * WAVE_BYTES;
    const uint16_t *__restrict__ smooth = (const uint16_t *)a.smooth;
    uint8_t *__restrict__ outbase = (uint8_t *)a.out + (size_t)m0 * a.ld_out + gw * (GROUP / 2);
    const uint32_t outoff = (uint32_t)ml * a.ld_out + kq * 8;
    uint16_t *__restrict__ scales = (uint16_t *)a.scales + (size_t)gw * a.ld_scales + m0;
    // scales_blocked: the eight scales of groups 8 j .. 8 j + 7 of a row side by side (16 bytes), 32 rows to a 512-byte block:
    // group gw + 8 i of row m at ((m / 32) * (ngroups / 8) + gw / 8 + i) * 256 + (m % 32) * 8 + gw % 8
    uint16_t *__restrict__ const scalesb = (uint16_t *)a.scales + ((size_t)(m0 >> 5) * (ngroups >> 3) + (gw >> 3)) * 256 + (gw & 7);
    // out_blocked: the 32 packed bytes of (row, group) go where the GEMM's lane (row % 32, half) of that 32-row block and
    // group finds them, [32-row block][group][64 lanes x 16 bytes]: this lane's 8 bytes are half kq / 2, offset 8 (kq % 2)
    uint8_t *__restrict__ bout[NH];
#pragma unroll
    for (int h = 0; h < NH; h++) {
        const int m = m0 + Q_ROWS * h + ml;
        bout[h] = (uint8_t *)a.out + (size_t)(m >> 5) * ngroups * 1024 + (((kq >> 1) * 32 + (m & 31)) * 16 + (kq & 1) * 8);
    }
    // out_blocked == 2: fp6 codes (sign << 5 | magnitude) where the GEMM's lane 32 kh + row % 32 of the row block and
    // group finds its 32 values k = 2 p + kh as 24 bytes, code p at bits 6 p: the first 16 bytes at 16 lane, the last 8 at
    // 1024 + 8 lane of the (row block, group)'s 1536.  This lane's even channels are codes 8 kq .. 8 kq + 7 of kh = 0, its odd
    // ones the same codes of kh = 1: two 48-bit pieces at byte 6 kq of those 24, each stored as an aligned dword and a
    // 16-bit half (low dword + high half for even kq, low half + high dword for odd kq).
    const bool f6 = a.out_blocked == 2;
    typedef float v8f __attribute__((ext_vector_type(8)));
    typedef float v16f __attribute__((ext_vector_type(16)));
    typedef unsigned v6u __attribute__((ext_vector_type(6)));
    uint8_t *__restrict__ const f6base = (uint8_t *)a.out + (size_t)(m0 >> 5) * ngroups * 1536;
    uint32_t f6o32[NH], f6o16[NH];
#pragma unroll
    for (int h = 0; h < NH; h++) {
        const uint32_t r = (uint32_t)(m0 + Q_ROWS * h + ml) & 31u;
        f6o32[h] = kq == 0 ? 16u * r : kq == 1 ? 16u * r + 8u : kq == 2 ? 16u * r + 12u : 1024u + 8u * r + 4u;
        f6o16[h] = kq == 0 ? 16u * r + 4u : kq == 1 ? 16u * r + 6u : kq == 2 ? 1024u + 8u * r : 1024u + 8u * r + 2u;
    }
    const uint32_t f6d32 = kq < 3 ? 512u : 256u, f6d16 = kq < 2 ? 512u : 256u;  // from kh = 0 to kh = 1
    constexpr int GSTEP = Q_WAVES * GROUP;  // elements between consecutive groups of one wavefront
    const float qmax = UNSIGNED ? 15.0f : 7.0f;
    const float rmagic = UNSIGNED ? RNE_MAGIC : RNE_MAGIC + 8.0f;  // signed codes are packed as c + 8, then ^ 8
    const bool has_shift = a.shift != 0.0f;
    // norm prologue: this lane's row statistics, and the workgroup's scale / shift vectors (one batch per workgroup)
    float n_mean[NH], n_rstd[NH];
    const uint16_t *__restrict__ nscale = nullptr, *__restrict__ nshift = nullptr;
    if (NORM) {
#pragma unroll
        for (int h = 0; h < NH; h++) {
            const int mr = min(m0 + Q_ROWS * h + ml, a.M - 1);
            n_mean[h] = a.norm_stats[2 * mr];
            n_rstd[h] = a.norm_stats[2 * mr + 1];
        }
        const size_t voff = a.norm_rows_per_batch > 0 ? (size_t)(m0 / a.norm_rows_per_batch) * a.norm_ld : 0;
        nscale = (const uint16_t *)a.norm_scale + voff;
        nshift = (const uint16_t *)a.norm_shift + voff;
    }

    // Ranks beyond Q_RCHUNK: the grid's second axis.  Workgroup (row block, rc) projects onto ranks [32 rc, 32 rc + 32);
    // only rc = 0 quantizes.  (The further workgroups read the activations again, from the memory-side cache, and
    // run next to the others on CUs the row blocks alone leave idle.)
    // With one more workgroup row than rank chunks, row 0 only quantizes and rows 1 .. project (the two kinds of work
    // then run side by side on different CUs instead of one after the other in every wavefront).
    {
        const bool split = nq > 0;
        const int rc = max((int)blockIdx.y - nq, 0);
        const bool do_lora = HAS_LORA && !qonly;
        v4f acc0[NH], acc1[NH];
#pragma unroll
        for (int h = 0; h < NH; h++) acc0[h] = acc1[h] = (v4f){0.f, 0.f, 0.f, 0.f};
        // ranks >= R re-read rank R - 1; their accumulator rows are never stored
        const uint8_t *__restrict__ lbase = (const uint8_t *)a.lora_down_t;
        uint32_t ldma[4] = {0, 0, 0, 0};
        if (HAS_LORA) {
#pragma unroll
            for (int i = 0; i < 4; i++)
                ldma[i] = (uint32_t)min(rc * Q_RCHUNK + 8 * i + drow, a.R - 1) * a.K * 2 + dchunk * 16;
        }
        const bool do_quant = split ? qonly : rc == 0;

        constexpr int NX = (GLU ? 4 : 2) * NH;  // block loads of one activation stage
        auto group_off = [&](int i) {  // byte offset of group wave + Q_WAVES * i in a row; past the end: the last group
            return (uint32_t)min(gw + Q_WAVES * i, ngroups - 1) * (GROUP * 2);
        };
        auto issue_x = [&](int i, QVecs &qv) {
            const uint32_t k0 = group_off(i);
            uint8_t *dst = wbase + (i & 1) * XS_BYTES;
            // the per-channel vectors of the lane's channel first: older than the block loads, their wait does not
            // cover them
            if (HAS_SMOOTH && do_quant) qv.sm = smooth[(k0 >> 1) + lane];
            if (NORM) {
                qv.ns = nscale[((k0 >> 1) + lane) * a.norm_stride];
                qv.nh = nshift[((k0 >> 1) + lane) * a.norm_stride];
            }
#pragma unroll
            for (int j = 0; j < 2 * NH; j++)
                __builtin_amdgcn_global_load_lds((const SVDQ_AS1 void *)(xbase + (xdma[j] + k0)),
                                                 (SVDQ_AS3 void *)(dst + j * 1024), 16, 0, 0);
            if (GLU) {
#pragma unroll
                for (int j = 0; j < 2 * NH; j++)
                    __builtin_amdgcn_global_load_lds((const SVDQ_AS1 void *)(xbase + (size_t)a.K * 2 + (xdma[j] + k0)),
                                                     (SVDQ_AS3 void *)(dst + G_OFF + j * 1024), 16, 0, 0);
            }
        };
        auto issue_l = [&](int i) {
            if (!do_lora) return;
            const uint32_t k0 = group_off(i);
#pragma unroll
            for (int j = 0; j < 4; j++)
                __builtin_amdgcn_global_load_lds((const SVDQ_AS1 void *)(lbase + (ldma[j] + k0)),
                                                 (SVDQ_AS3 void *)(wbase + L_OFF + j * 1024), 16, 0, 0);
        };

        struct Ops {
            v4i xlo[NH], xhi[NH], glo[NH], ghi[NH], l0lo, l0hi, l1lo, l1hi;
        };
        auto fetch = [&](int i, Ops &o) {  // LDS -> registers, in the MFMA operand layout
            const uint8_t *src = wbase + (i & 1) * XS_BYTES;
#pragma unroll
            for (int h = 0; h < NH; h++) {
                o.xlo[h] = *(const v4i *)(src + h * Q_ROWS * Q_ROW_BYTES + rd_lo);
                o.xhi[h] = *(const v4i *)(src + h * Q_ROWS * Q_ROW_BYTES + rd_hi);
                if (GLU) {
                    o.glo[h] = *(const v4i *)(src + G_OFF + h * Q_ROWS * Q_ROW_BYTES + rd_lo);
                    o.ghi[h] = *(const v4i *)(src + G_OFF + h * Q_ROWS * Q_ROW_BYTES + rd_hi);
                }
            }
            if (do_lora) {
                o.l0lo = *(const v4i *)(wbase + L_OFF + rd_lo);
                o.l0hi = *(const v4i *)(wbase + L_OFF + rd_hi);
                o.l1lo = *(const v4i *)(wbase + L_OFF + 16 * Q_ROW_BYTES + rd_lo);
                o.l1hi = *(const v4i *)(wbase + L_OFF + 16 * Q_ROW_BYTES + rd_hi);
            }
        };

        auto process = [&](int i, const Ops &o, const QVecs qv) {
            const uint16_t smv = qv.sm;
            const v4i l0lo = o.l0lo, l0hi = o.l0hi, l1lo = o.l1lo, l1hi = o.l1hi;
            // per-channel vectors of the group, once for all halves: 1/smooth (one IEEE divide per lane) and the norm
            // prologue's scale / shift, shared through LDS
            if (NORM) {
                lds_ns[wave][lane] = T::to_f32(qv.ns);
                lds_nh[wave][lane] = T::to_f32(qv.nh);
            }
            if (HAS_SMOOTH && do_quant) lds_rs[wave][lane] = 1.0f / T::to_f32(smv);
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int h = 0; h < NH; h++) {
            const int m = m0 + Q_ROWS * h + ml;
            const bool row_ok = m < a.M;
            v4i cxlo = o.xlo[h], cxhi = o.xhi[h];
            const v4i glo = o.glo[h], ghi = o.ghi[h];
            float v[16];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v[2 * j] = T::lo_f32((uint32_t)cxlo[j]);
                v[2 * j + 1] = T::hi_f32((uint32_t)cxlo[j]);
                v[8 + 2 * j] = T::lo_f32((uint32_t)cxhi[j]);
                v[8 + 2 * j + 1] = T::hi_f32((uint32_t)cxhi[j]);
            }
            if (GLU) {
                // x[:, k] * silu(x[:, K + k]); the LoRA-down then sees the product rounded to T
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float g0 = T::lo_f32((uint32_t)glo[j]), g1 = T::hi_f32((uint32_t)glo[j]);
                    const float g2 = T::lo_f32((uint32_t)ghi[j]), g3 = T::hi_f32((uint32_t)ghi[j]);
                    v[2 * j] = v[2 * j] * (g0 / (1.0f + __expf(-g0)));
                    v[2 * j + 1] = v[2 * j + 1] * (g1 / (1.0f + __expf(-g1)));
                    v[8 + 2 * j] = v[8 + 2 * j] * (g2 / (1.0f + __expf(-g2)));
                    v[8 + 2 * j + 1] = v[8 + 2 * j + 1] * (g3 / (1.0f + __expf(-g3)));
                }
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    cxlo[j] = (int)pack2<T>(v[2 * j], v[2 * j + 1]);
                    cxhi[j] = (int)pack2<T>(v[8 + 2 * j], v[8 + 2 * j + 1]);
                }
            }
            if (GELU) {
                // tanh-GELU of the input (the unfused form of the GEMM's GELU epilogue); the LoRA-down sees it rounded to T
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = gelu_tanh(v[j]);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    cxlo[j] = (int)pack2<T>(v[2 * j], v[2 * j + 1]);
                    cxhi[j] = (int)pack2<T>(v[8 + 2 * j], v[8 + 2 * j + 1]);
                }
            }
            if (NORM) {
                // LayerNorm, scale, shift, each rounded to T; the LoRA-down sees the result
                // (two values per rounding instruction; the last packed pair is the LoRA-down operand itself)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const v4f sc = *(const v4f *)&lds_ns[wave][kq * 16 + 4 * j];
                    const v4f sh = *(const v4f *)&lds_nh[wave][kq * 16 + 4 * j];
#pragma unroll
                    for (int e = 0; e < 4; e += 2) {
                        const int i = 4 * j + e;
                        uint32_t w = pack2<T>((v[i] - n_mean[h]) * n_rstd[h], (v[i + 1] - n_mean[h]) * n_rstd[h]);
                        w = pack2<T>(T::lo_f32(w) * sc[e], T::hi_f32(w) * sc[e + 1]);
                        w = pack2<T>(T::lo_f32(w) + sh[e], T::hi_f32(w) + sh[e + 1]);
                        v[i] = T::lo_f32(w);
                        v[i + 1] = T::hi_f32(w);
                        if (i < 8) cxlo[i / 2] = (int)w; else cxhi[(i - 8) / 2] = (int)w;
                    }
                }
            }
            if (do_lora) {
                acc0[h] = mfma16_16bit<T>(l0lo, cxlo, acc0[h]);
                acc0[h] = mfma16_16bit<T>(l0hi, cxhi, acc0[h]);
                acc1[h] = mfma16_16bit<T>(l1lo, cxlo, acc1[h]);
                acc1[h] = mfma16_16bit<T>(l1hi, cxhi, acc1[h]);
            }
            if (!do_quant) continue;
            if (has_shift) {
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = v[j] + a.shift;
            }
            if (HAS_SMOOTH) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const v4f rs = *(const v4f *)&lds_rs[wave][kq * 16 + 4 * j];
#pragma unroll
                    for (int e = 0; e < 4; e++) v[4 * j + e] = v[4 * j + e] * rs[e];
                }
            }
            float gmax = 0.0f;
#pragma unroll
            for (int j = 0; j < 16; j += 2)
                gmax = UNSIGNED ? __builtin_fmaxf(__builtin_fmaxf(v[j], v[j + 1]), gmax)
                                : __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v[j]), __builtin_fabsf(v[j + 1])), gmax);
            gmax = max_with_lane_xor32(max_with_lane_xor16(gmax));
            const float scale = gmax / qmax;
            const float safe = (scale == 0.0f) ? 1.0f : scale;
            const float rq = 1.0f / safe;
            // The magic add rounds to nearest-even and leaves code (+ 8 when signed) in the low mantissa bits; shifted
            // adds pack eight of them per dword (the constant upper bits add up to pack_bias()).  Signed codes need
            // no clamp: |x| <= gmax gives |x * (1 / (gmax / 7))| <= 7 (1 + 3 * 2^-24), which rounds to <= 7; unsigned codes
            // only need the lower clamp (negative values), the upper bound holds the same way.
            if (f6) {
                // the same products, rounded to the same integers by the hardware's float -> fp6 conversion: e2m3 codes
                // are sign | magnitude with steps of 1 / 8 up to 15 / 8, so q / 8 (the instruction's scale operand) rounds to
                // nearest-even exactly as q does.  It converts 2 x 16 values, result code 2 i from the first source's
                // element i and code 2 i + 1 from the second's: codes 0 .. 7 get the even channels, 8 .. 15 the odd ones
                // (elements 8 .. 15 of the sources are not used and left undefined).
                v8f c0, c1;
#pragma unroll
                for (int j = 0; j < 16; j++) {
                    float q = v[j] * rq;
                    if (UNSIGNED) q = __builtin_fmaxf(q, 0.0f);
                    const int c = j >> 1, o = (j & 1) * 4 + (c >> 1);
                    if (c & 1)
                        c1[o] = q;
                    else
                        c0[o] = q;
                }
                const v16f cv0 = __builtin_shufflevector(c0, c0, 0, 1, 2, 3, 4, 5, 6, 7, -1, -1, -1, -1, -1, -1, -1, -1);
                const v16f cv1 = __builtin_shufflevector(c1, c1, 0, 1, 2, 3, 4, 5, 6, 7, -1, -1, -1, -1, -1, -1, -1, -1);
                const v6u d = __builtin_amdgcn_cvt_scalef32_2xpk16_fp6_f32(cv0, cv1, 8.0f);
                const uint32_t plo[2] = {d[0], __builtin_amdgcn_alignbit(d[2], d[1], 16)};  // [0]: even channels, [1]: odd
                const uint32_t phi[2] = {d[1], d[2] >> 16};                                 // (only their low 16 bits are used)
                if (row_ok) {
                    if (kq == 0) {
                        if (a.scales_blocked)
                            scalesb[(size_t)i * 256 + ((m0 + Q_ROWS * h + ml) & 31) * 8] = T::from_f32(scale);
                        else
                            (scales + (size_t)i * Q_WAVES * a.ld_scales)[Q_ROWS * h + ml] = T::from_f32(scale);
                    }
                    uint8_t *blk = f6base + (size_t)(gw + Q_WAVES * i) * 1536;
#pragma unroll
                    for (int e = 0; e < 2; e++) {
                        const uint32_t d32 = (kq & 1) ? __builtin_amdgcn_alignbit(phi[e], plo[e], 16) : plo[e];
                        const uint32_t d16 = (kq & 1) ? plo[e] : phi[e];
                        *(uint32_t *)(blk + f6o32[h] + (e ? f6d32 : 0u)) = d32;
                        *(uint16_t *)(blk + f6o16[h] + (e ? f6d16 : 0u)) = (uint16_t)d16;
                    }
                }
                continue;
            }
            uint32_t w0 = 0u - pack_bias(), w1 = 0u - pack_bias();
#pragma unroll
            for (int j = 0; j < 8; j++) {
                float q0 = v[j] * rq, q1 = v[8 + j] * rq;
                if (UNSIGNED) {
                    q0 = __builtin_fmaxf(q0, 0.0f);
                    q1 = __builtin_fmaxf(q1, 0.0f);
                }
                const uint32_t b0 = __float_as_uint(q0 + rmagic), b1 = __float_as_uint(q1 + rmagic);
                asm("v_lshl_add_u32 %0, %1, %2, %0" : "+v"(w0) : "v"(b0), "n"(4 * j));
                asm("v_lshl_add_u32 %0, %1, %2, %0" : "+v"(w1) : "v"(b1), "n"(4 * j));
            }
            if (!UNSIGNED) {
                w0 ^= 0x88888888u;
                w1 ^= 0x88888888u;
            }
            if (row_ok) {
                if (kq == 0) {
                    if (a.scales_blocked)
                        scalesb[(size_t)i * 256 + ((m0 + Q_ROWS * h + ml) & 31) * 8] = T::from_f32(scale);
                    else
                        (scales + (size_t)i * Q_WAVES * a.ld_scales)[Q_ROWS * h + ml] = T::from_f32(scale);
                }
                uint8_t *dst = a.out_blocked ? bout[h] + (size_t)(gw + Q_WAVES * i) * 1024
                                             : outbase + (size_t)i * (GSTEP / 2) + (uint32_t)(Q_ROWS * h) * a.ld_out + outoff;
                *(uint2 *)dst = make_uint2(w0, w1);
            }
            }  // halves
            __builtin_amdgcn_wave_barrier();  // the shared vectors are rewritten by the next group
        };

        // Two groups of activations and one LoRA-down tile in flight per wavefront; each wavefront owns its LDS, so no
        // barrier in the loop.  Per group: wait for its tiles, pull them into registers, refill the freed LDS (next
        // group's LoRA-down tile, the activations two groups on), then compute from the registers.
        QVecs sm_a = {0, 0, 0}, sm_b = {0, 0, 0};
        Ops ops;
        issue_x(0, sm_a);
        issue_l(0);
        issue_x(1, sm_b);
        auto step = [&](int i, QVecs &sm) {
            // group i's activations and LoRA-down tile have landed: the loads issued after them are at least the NX
            // block loads of group i + 1's activations
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(NX, 15));
            fetch(i, ops);
            const QVecs smv = sm;
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));  // the LDS reads have returned
            issue_l(i + 1);
            issue_x(i + 2, sm);
            process(i, ops, smv);
        };
        for (int i = 0; i < nmy; i += 2) {
            step(i, sm_a);
            if (i + 1 < nmy) step(i + 1, sm_b);
        }
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));

        if (do_lora) {
            // fixed-order sum of the wavefronts' partial products (this wavefront is done with its own stages)
            float (*mine)[QR + 1] = lds_acc(wave);
#pragma unroll
            for (int h = 0; h < NH; h++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    mine[4 * kq + i][Q_ROWS * h + ml] = acc0[h][i];
                    mine[16 + 4 * kq + i][Q_ROWS * h + ml] = acc1[h][i];
                }
            __syncthreads();
            for (int o = threadIdx.x; o < QR * Q_RCHUNK; o += Q_WAVES * 64) {
                const int mm = o / Q_RCHUNK, r = o % Q_RCHUNK;
                float s = lds_acc(0)[r][mm];
#pragma unroll
                for (int w = 1; w < Q_WAVES; w++) s += lds_acc(w)[r][mm];
                if (m0 + mm < a.M && rc * Q_RCHUNK + r < a.R)
                    a.lora_act[(size_t)(m0 + mm) * a.ld_lora_act + rc * Q_RCHUNK + r] = s;
            }
        }
    }
}

template <int CTRL>
__device__ inline float q_dpp(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}
// Sum over the wavefront, the same value in every lane, fixed order: pairs, quads, octets, rows of sixteen lanes (data
// parallel primitives, no LDS round trips), then the four rows in order.
__device__ inline float wave_sum(float s) {
    s += q_dpp<0xB1>(s);   // quad_perm [1, 0, 3, 2]
    s += q_dpp<0x4E>(s);   // quad_perm [2, 3, 0, 1]
    s += q_dpp<0x141>(s);  // row_half_mirror
    s += q_dpp<0x140>(s);  // row_mirror
    const int b = __builtin_bit_cast(int, s);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)), r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)), r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return ((r0 + r1) + r2) + r3;
}

// one wavefront per row: mean, then the centred sum of squares, fixed reduction order.  Rows of up to 8192 values are
// read once and kept in registers, their loads issued eight at a time without branches (offsets past the end of the
// row are clamped and those chunks not used), so that a wavefront has 8 KB in flight instead of 1; longer rows are read
// twice, the second time from cache.
template <typename T>
__global__ __launch_bounds__(256) void row_stats_kernel(const uint16_t *x, float *stats, int M, int K, long ld_x, float eps) {
    constexpr int MAXC = 16, BATCH = 8;  // 16-byte chunks per lane kept in registers; loads in flight
    const int lane = threadIdx.x & 63, m = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (m >= M) return;
    const uint16_t *row = x + (long)m * ld_x;
    float s = 0.0f, q = 0.0f, mean;
    if (K <= 512 * MAXC) {
        v4i r[MAXC];
#pragma unroll
        for (int c0 = 0; c0 < MAXC; c0 += BATCH)
            if (512 * c0 < K) {
#pragma unroll
                for (int u = 0; u < BATCH; u++) r[c0 + u] = *(const v4i *)(row + min(8 * lane + 512 * (c0 + u), K - 8));
            }
#pragma unroll
        for (int c = 0; c < MAXC; c++)
            if (8 * lane + 512 * c < K) {
#pragma unroll
                for (int e = 0; e < 4; e++) s += T::lo_f32((uint32_t)r[c][e]) + T::hi_f32((uint32_t)r[c][e]);
            }
        mean = wave_sum(s) / (float)K;
#pragma unroll
        for (int c = 0; c < MAXC; c++)
            if (8 * lane + 512 * c < K) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float d0 = T::lo_f32((uint32_t)r[c][e]) - mean, d1 = T::hi_f32((uint32_t)r[c][e]) - mean;
                    q += d0 * d0 + d1 * d1;
                }
            }
    } else {
        for (int k = 8 * lane; k < K; k += 512) {
            const v4i w = *(const v4i *)(row + k);
#pragma unroll
            for (int e = 0; e < 4; e++) s += T::lo_f32((uint32_t)w[e]) + T::hi_f32((uint32_t)w[e]);
        }
        mean = wave_sum(s) / (float)K;
        for (int k = 8 * lane; k < K; k += 512) {
            const v4i w = *(const v4i *)(row + k);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float d0 = T::lo_f32((uint32_t)w[e]) - mean, d1 = T::hi_f32((uint32_t)w[e]) - mean;
                q += d0 * d0 + d1 * d1;
            }
        }
    }
    const float var = wave_sum(q) / (float)K;
    if (lane == 0) {
        stats[2 * m] = mean;
        stats[2 * m + 1] = 1.0f / sqrtf(var + eps);
    }
}

// one wavefront per row; the rounded results stay in registers (packed) for the statistics, so the row is read once
template <typename T, bool SUM2, bool STATS>
__global__ __launch_bounds__(256) void gated_residual_kernel(const uint16_t *x, const uint16_t *gate, const uint16_t *y,
                                                             const uint16_t *y2, uint16_t *out, float *stats, int M, int K,
                                                             long ld_x, long ld_y, long ld_out, int rows_per_batch,
                                                             long gate_ld, int gate_stride, float eps, float clip) {
    constexpr int MAXC = 16;  // 16-byte chunks per lane: K <= 64 * 8 * 16
    const int lane = threadIdx.x & 63, m = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (m >= M) return;
    const uint16_t *xr = x + (long)m * ld_x, *yr = y + (long)m * ld_y, *y2r = SUM2 ? y2 + (long)m * ld_y : nullptr;
    const uint16_t *gr = gate + (rows_per_batch > 0 ? (long)(m / rows_per_batch) * gate_ld : 0);
    uint16_t *orow = out + (long)m * ld_out;
    v4i res[MAXC];
    float s = 0.0f;
    constexpr int BATCH = 2;  // chunks whose loads (x, y, y2, gate: up to eight) are issued together, without branches
#pragma unroll
    for (int c0 = 0; c0 < MAXC; c0 += BATCH) {
        if (512 * c0 >= K) break;
        v4i xb[BATCH], yb[BATCH], zb[BATCH], gb[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; u++) {
            const int kk = min(8 * lane + 512 * (c0 + u), K - 8);  // past the end: the row's last chunk again, not used
            xb[u] = *(const v4i *)(xr + kk);
            yb[u] = *(const v4i *)(yr + kk);
            zb[u] = SUM2 ? *(const v4i *)(y2r + kk) : (v4i){0, 0, 0, 0};
            gb[u] = gate_stride == 1 ? *(const v4i *)(gr + kk) : (v4i){0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < BATCH; u++) {
            const int c = c0 + u, k = 8 * lane + 512 * c;
            if (k < K) {
                const v4i xv = xb[u], yv = yb[u], zv = zb[u];
                float g[8];
                if (gate_stride == 1) {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        g[2 * e] = T::lo_f32((uint32_t)gb[u][e]);
                        g[2 * e + 1] = T::hi_f32((uint32_t)gb[u][e]);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) g[e] = T::to_f32(gr[(long)(k + e) * gate_stride]);
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {  // every step rounded to T, two values per rounding instruction
                    uint32_t w = (uint32_t)yv[e];
                    if (SUM2) w = pack2<T>(T::lo_f32(w) + T::lo_f32((uint32_t)zv[e]), T::hi_f32(w) + T::hi_f32((uint32_t)zv[e]));
                    w = pack2<T>(g[2 * e] * T::lo_f32(w), g[2 * e + 1] * T::hi_f32(w));
                    w = pack2<T>(T::lo_f32((uint32_t)xv[e]) + T::lo_f32(w), T::hi_f32((uint32_t)xv[e]) + T::hi_f32(w));
                    float o0 = T::lo_f32(w), o1 = T::hi_f32(w);
                    if (clip > 0.0f) {  // x.clip(-clip, clip): infinities become the limit, NaN stays
                        o0 = o0 > clip ? clip : (o0 < -clip ? -clip : o0);
                        o1 = o1 > clip ? clip : (o1 < -clip ? -clip : o1);
                        w = pack2<T>(o0, o1);
                    }
                    s += o0 + o1;
                    res[c][e] = (int)w;
                }
                *(v4i *)(orow + k) = res[c];
            }
        }
    }
    if (!STATS) return;
    const float mean = wave_sum(s) / (float)K;
    float q = 0.0f;
#pragma unroll
    for (int c = 0; c < MAXC; c++) {
        if (8 * lane + 512 * c < K) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float d0 = T::lo_f32((uint32_t)res[c][e]) - mean, d1 = T::hi_f32((uint32_t)res[c][e]) - mean;
                q += d0 * d0 + d1 * d1;
            }
        }
    }
    const float var = wave_sum(q) / (float)K;
    if (lane == 0) {
        stats[2 * m] = mean;
        stats[2 * m + 1] = 1.0f / sqrtf(var + eps);
    }
}

__global__ void transpose_kr_kernel(const uint16_t *in, uint16_t *out, int K, int R, int ld_in) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= K * R) return;
    const int r = idx / K, k = idx % K;
    out[idx] = in[(size_t)k * ld_in + r];
}

// Rows per workgroup.  A workgroup streams 4 KB of LoRA-down weight per group whatever its number of rows, and the
// vector memory pipe of a CU is what that traffic is bound by: with 16-row workgroups, M = 4608 puts two of them on 32 of
// the 256 CUs and the launch waits for those.  32-row workgroups (one LoRA-down tile read for two MFMA passes; a longer
// chain per wavefront, 12 us even for one workgroup per CU) are faster where the 16-row grid needs between one and two
// workgroups per CU: 13.4 against 14.2 us at M = 4608, 14.6 against 15.5 at 6144, 16.2 against 16.7 at 8192 (K = 3072,
// R = 32); below and above that range the 16-row kernel wins.
static int quantize_rows_per_workgroup(const svdq_quantize_args &a) {
    if (a.R == 0 || a.prologue != SVDQ_PRE_NONE) return Q_ROWS;
    if (a.norm_stats) return Q_ROWS;  // twice the arithmetic per value: 19.0 against 19.9 us at M = 4608, 20.6 against 21.7 at 8192
    const int wg16 = (a.M + 15) / 16;
    return (wg16 > Q32_ABOVE && wg16 <= Q32_UPTO) ? 32 : Q_ROWS;
}

static int device_cus() {
    static int cus = 0;
    if (!cus) {
        int dev = 0, n = 0;
        cus = hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0 ? n : 256;
    }
    return cus;
}

// Second grid axis: one workgroup row per chunk of 32 ranks, plus rows that only quantize where that still leaves about
// one workgroup per CU: quantizing and projecting then run side by side on different CUs (K = 3072, R = 32: 6.4
// against 7.9 us at M = 512, 7.1 against 8.5 at 2048, 12.3 against 13.4 at 4608 with 32-row workgroups; slower once the
// CUs are taken: 9.9 against 9.5 us at M = 4096, 17.2 against 14.5 at 6144).  While CUs are left over, up to three such
// rows share the groups between them: a wavefront's chain of group steps gets shorter (M = 1024: 7.8 -> 5.1 us with
// three, M = 512: 7.6 -> 4.9; slower again beyond one workgroup per CU: M = 1024 with four 6.4 us, M = 4608 with two
// 14.2 against 12.8).
static int quantize_grid_y(const svdq_quantize_args &a, int row_blocks, int rows) {
    if (a.R == 0) return 1;
    const int chunks = (a.R + Q_RCHUNK - 1) / Q_RCHUNK, cus = device_cus();
    // (with a prologue the workgroups that only project compute it a second time: only where half the CUs would idle
    // anyway; norm prologue, M = 512: 10.4 against 11.8 us, M = 4608: 25.5 against 20.7)
    const bool prologue = a.norm_stats || a.prologue != SVDQ_PRE_NONE;
    const int limit = prologue ? cus / 2 : cus + (rows == 32 ? cus / 8 : 0);
    if (row_blocks * (chunks + 1) > limit) return chunks;
    const int nq = std::min({3, limit / row_blocks - chunks, a.K / GROUP});
    return chunks + std::max(nq, 1);
}

template <typename T, bool U, int G, bool NORM>
static void launch_quantize3(const svdq_quantize_args &a, hipStream_t s) {
    const dim3 block(Q_WAVES * 64);
    const bool lora = a.R > 0, sm = a.smooth != nullptr;
    if constexpr (G == SVDQ_PRE_NONE) {
        if (quantize_rows_per_workgroup(a) == 32) {
            const dim3 grid((a.M + 31) / 32, quantize_grid_y(a, (a.M + 31) / 32, 32));
            if (sm)
                hipLaunchKernelGGL((quantize_act_kernel<T, U, G, true, true, NORM, 32>), grid, block, 0, s, a);
            else
                hipLaunchKernelGGL((quantize_act_kernel<T, U, G, true, false, NORM, 32>), grid, block, 0, s, a);
            return;
        }
    }
    const dim3 grid((a.M + Q_ROWS - 1) / Q_ROWS, quantize_grid_y(a, (a.M + Q_ROWS - 1) / Q_ROWS, Q_ROWS));
    if (lora && sm)
        hipLaunchKernelGGL((quantize_act_kernel<T, U, G, true, true, NORM, 16>), grid, block, 0, s, a);
    else if (lora)
        hipLaunchKernelGGL((quantize_act_kernel<T, U, G, true, false, NORM, 16>), grid, block, 0, s, a);
    else if (sm)
        hipLaunchKernelGGL((quantize_act_kernel<T, U, G, false, true, NORM, 16>), grid, block, 0, s, a);
    else
        hipLaunchKernelGGL((quantize_act_kernel<T, U, G, false, false, NORM, 16>), grid, block, 0, s, a);
}

template <typename T, bool U, int G>
static void launch_quantize2(const svdq_quantize_args &a, hipStream_t s) {
    if constexpr (G == SVDQ_PRE_NONE) {
        if (a.norm_stats) {
            launch_quantize3<T, U, SVDQ_PRE_NONE, true>(a, s);
            return;
        }
    }
    launch_quantize3<T, U, G, false>(a, s);
}

template <typename T>
static void launch_quantize(const svdq_quantize_args &a, hipStream_t s) {
    if (a.prologue == SVDQ_PRE_GLU) {
        if (a.is_unsigned)
            launch_quantize2<T, true, SVDQ_PRE_GLU>(a, s);
        else
            launch_quantize2<T, false, SVDQ_PRE_GLU>(a, s);
    } else if (a.prologue == SVDQ_PRE_GELU) {
        if (a.is_unsigned)
            launch_quantize2<T, true, SVDQ_PRE_GELU>(a, s);
        else
            launch_quantize2<T, false, SVDQ_PRE_GELU>(a, s);
    } else {
        if (a.is_unsigned)
            launch_quantize2<T, true, SVDQ_PRE_NONE>(a, s);
        else
            launch_quantize2<T, false, SVDQ_PRE_NONE>(a, s);
    }
}

}  // namespace svdq

using namespace svdq;

extern "C" int svdq_quantize_act(const svdq_quantize_args *args, void *stream) {
    if (!args) {
        set_error("svdq_quantize_act: null args");
        return SVDQ_E_INVALID;
    }
    const svdq_quantize_args &a = *args;
    if (a.M < 0 || a.K <= 0 || a.K % GROUP) {
        set_error("svdq_quantize_act: K=%d must be a positive multiple of 64 (M=%d)", a.K, a.M);
        return SVDQ_E_INVALID;
    }
    if (a.R < 0 || a.R % 16 || (a.R > 0 && (!a.lora_down_t || !a.lora_act))) {
        set_error("svdq_quantize_act: R=%d must be a multiple of 16 with lora_down_t and lora_act given", a.R);
        return SVDQ_E_INVALID;
    }
    if (!a.x || !a.out || !a.scales) {
        set_error("svdq_quantize_act: x, out and scales are required");
        return SVDQ_E_INVALID;
    }
    if (a.ld_x % 8 || ((uintptr_t)a.x & 15) || (a.R > 0 && ((uintptr_t)a.lora_down_t & 15))) {
        set_error("svdq_quantize_act: x rows and lora_down_t must be 16-byte aligned (ld_x=%d)", a.ld_x);
        return SVDQ_E_INVALID;
    }
    if (a.out_blocked < 0 || a.out_blocked > 2) {
        set_error("svdq_quantize_act: out_blocked=%d (0: the (M, K / 2) matrix, 1: its bytes in lane order, 2: fp6 codes in lane order)",
                  a.out_blocked);
        return SVDQ_E_INVALID;
    }
    if ((!a.out_blocked && a.ld_out % 8) || ((uintptr_t)a.out & (a.out_blocked ? 15 : 7))) {
        set_error("svdq_quantize_act: out rows must be 8-byte aligned (ld_out=%d)", a.ld_out);
        return SVDQ_E_INVALID;
    }
    if (a.prologue < SVDQ_PRE_NONE || a.prologue > SVDQ_PRE_GELU) {
        set_error("svdq_quantize_act: unknown prologue %d", a.prologue);
        return SVDQ_E_INVALID;
    }
    if (a.scales_blocked && (a.K % 512 || ((uintptr_t)a.scales & 15))) {
        set_error("svdq_quantize_act: scales_blocked needs K %% 512 == 0 (K=%d) and 16-byte aligned scales", a.K);
        return SVDQ_E_INVALID;
    }
    if (a.ld_x < (a.prologue == SVDQ_PRE_GLU ? 2 : 1) * a.K || (!a.out_blocked && a.ld_out < a.K / 2) || (!a.scales_blocked && a.ld_scales < a.M) ||
        (a.R > 0 && a.ld_lora_act < a.R)) {
        set_error("svdq_quantize_act: a leading dimension is smaller than its row");
        return SVDQ_E_INVALID;
    }
    if (a.dtype != SVDQ_BF16 && a.dtype != SVDQ_FP16) {
        set_error("svdq_quantize_act: dtype %d", a.dtype);
        return SVDQ_E_INVALID;
    }
    if (a.norm_stats) {
        if (a.prologue != SVDQ_PRE_NONE) {
            set_error("svdq_quantize_act: the norm prologue cannot be combined with the GLU / GELU prologue");
            return SVDQ_E_UNSUPPORTED;
        }
        if (!a.norm_scale || !a.norm_shift || a.norm_rows_per_batch < 0 || a.norm_rows_per_batch % Q_ROWS ||
            a.norm_stride < 1 || a.norm_ld < 0) {
            set_error("svdq_quantize_act: the norm prologue needs norm_scale and norm_shift, norm_stride >= 1 and "
                      "norm_rows_per_batch=%d a multiple of 16", a.norm_rows_per_batch);
            return SVDQ_E_INVALID;
        }
    }
    if (a.M == 0) return SVDQ_OK;
    if (a.dtype == SVDQ_BF16)
        launch_quantize<BF16>(a, (hipStream_t)stream);
    else
        launch_quantize<FP16>(a, (hipStream_t)stream);
    return check_launch("svdq_quantize_act");
}

extern "C" int svdq_row_stats(const void *x, float *stats, int32_t M, int32_t K, int32_t ld_x, int32_t dtype, float eps,
                              void *stream) {
    if (!x || !stats || M < 0 || K <= 0 || K % 8 || ld_x < K || ld_x % 8 || ((uintptr_t)x & 15)) {
        set_error("svdq_row_stats: bad arguments (M=%d K=%d ld_x=%d; K and ld_x multiples of 8, x 16-byte aligned)", M, K, ld_x);
        return SVDQ_E_INVALID;
    }
    if (dtype != SVDQ_BF16 && dtype != SVDQ_FP16) {
        set_error("svdq_row_stats: dtype %d", dtype);
        return SVDQ_E_INVALID;
    }
    if (M == 0) return SVDQ_OK;
    const dim3 grid((M + 3) / 4), block(256);
    if (dtype == SVDQ_BF16)
        hipLaunchKernelGGL(row_stats_kernel<BF16>, grid, block, 0, (hipStream_t)stream, (const uint16_t *)x, stats, M, K, (long)ld_x, eps);
    else
        hipLaunchKernelGGL(row_stats_kernel<FP16>, grid, block, 0, (hipStream_t)stream, (const uint16_t *)x, stats, M, K, (long)ld_x, eps);
    return check_launch("svdq_row_stats");
}

template <typename T>
static void launch_gated_residual(const void *x, const void *gate, const void *y, const void *y2, void *out, float *stats,
                                  int M, int K, long ld_x, long ld_y, long ld_out, int rpb, long gate_ld, int gate_stride,
                                  float eps, float clip, hipStream_t s) {
    const dim3 grid((M + 3) / 4), block(256);
#define SVDQ_GR(S2, ST)                                                                                                   \
    hipLaunchKernelGGL((gated_residual_kernel<T, S2, ST>), grid, block, 0, s, (const uint16_t *)x, (const uint16_t *)gate, \
                       (const uint16_t *)y, (const uint16_t *)y2, (uint16_t *)out, stats, M, K, ld_x, ld_y, ld_out, rpb,   \
                       gate_ld, gate_stride, eps, clip)
    if (y2 && stats)
        SVDQ_GR(true, true);
    else if (y2)
        SVDQ_GR(true, false);
    else if (stats)
        SVDQ_GR(false, true);
    else
        SVDQ_GR(false, false);
#undef SVDQ_GR
}

extern "C" int svdq_gated_residual(const void *x, const void *gate, const void *y, const void *y2, void *out, float *stats,
                                   int32_t M, int32_t K, int32_t ld_x, int32_t ld_y, int32_t ld_out, int32_t rows_per_batch,
                                   int32_t gate_ld, int32_t gate_stride, int32_t dtype, float eps, float clip, void *stream) {
    if (!x || !gate || !y || !out || M < 0 || K <= 0 || K % 8) {
        set_error("svdq_gated_residual: x, gate, y and out are required and K=%d must be a positive multiple of 8 (M=%d)", K, M);
        return SVDQ_E_INVALID;
    }
    if (K > 8192) {
        set_error("svdq_gated_residual: K=%d exceeds 8192 (a row is held in one wavefront's registers)", K);
        return SVDQ_E_UNSUPPORTED;
    }
    auto al = [](const void *p) { return ((uintptr_t)p & 15) == 0; };
    if (ld_x < K || ld_y < K || ld_out < K || ld_x % 8 || ld_y % 8 || ld_out % 8 || !al(x) || !al(y) || !al(out) ||
        (y2 && !al(y2)) || rows_per_batch < 0 || gate_stride < 1 || (gate_stride == 1 && (!al(gate) || gate_ld % 8))) {
        set_error("svdq_gated_residual: rows of x, y, y2, out (and of a contiguous gate) must be 16-byte aligned and hold K elements");
        return SVDQ_E_INVALID;
    }
    if (dtype != SVDQ_BF16 && dtype != SVDQ_FP16) {
        set_error("svdq_gated_residual: dtype %d", dtype);
        return SVDQ_E_INVALID;
    }
    if (!(clip >= 0.0f)) {
        set_error("svdq_gated_residual: clip must be 0 (off) or a positive limit");
        return SVDQ_E_INVALID;
    }
    if (M == 0) return SVDQ_OK;
    if (dtype == SVDQ_BF16)
        launch_gated_residual<BF16>(x, gate, y, y2, out, stats, M, K, ld_x, ld_y, ld_out, rows_per_batch, gate_ld, gate_stride, eps, clip, (hipStream_t)stream);
    else
        launch_gated_residual<FP16>(x, gate, y, y2, out, stats, M, K, ld_x, ld_y, ld_out, rows_per_batch, gate_ld, gate_stride, eps, clip, (hipStream_t)stream);
    return check_launch("svdq_gated_residual");
}

extern "C" int svdq_transpose_lora_down(const void *lora_down, void *lora_down_t, int32_t K, int32_t R,
                                         int32_t ld_in, void *stream) {
    if (!lora_down || !lora_down_t || K <= 0 || R <= 0 || ld_in < R) {
        set_error("svdq_transpose_lora_down: bad arguments (K=%d R=%d ld_in=%d)", K, R, ld_in);
        return SVDQ_E_INVALID;
    }
    const int n = K * R;
    hipLaunchKernelGGL(transpose_kr_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t *)lora_down, (uint16_t *)lora_down_t, K, R, ld_in);
    return check_launch("svdq_transpose_lora_down");
}
