// AWQ W4A16 GEMV (group 64, TinyChat-packed weights) for gfx950, small M (<= 32 rows).
//
// Arithmetic (reference: nunchaku/ops/triton/awq.py:160-182):
//   out[m, n] = sum_c  s[c, n] * sum_{k in c} x[m, k] q[n, k]  +  z[c, n] * sum_{k in c} x[m, k]      (fp32)
//
// N*K/2 bytes of weights are read exactly once, for all M rows together (the reference launches one pass over the
// weights per row).
//
// Storage order is the access order.  Packed row a = n / 4 holds, for scale group c, 128 contiguous bytes =
// 4 channels (b = n % 4) x 2 halves (h) x 16 bytes; the 16 bytes of (n, c, h) are eight int16 whose nibble j' holds
// k = 64 c + 32 h + 8 j' + j (j = position of the int16).  A lane loads exactly one such piece per group, eight lanes
// one contiguous 128-byte piece of a packed row, one load instruction 8 packed rows x 128 bytes.  Nibble plane j' of the
// loaded dwords, OR-ed with the bit pattern of 128.0 (bf16) / 1024.0 (fp16), is directly an MFMA B operand (exact:
// 128 + q and 1024 + q are representable); the A operand is the matching piece of x.  The constant offset is folded
// into the zero-point term:
//   s * (D - OFF * xs) + z * xs = s * D + (z - OFF * s) * xs,   xs = sum_{k in c} x[m, k]  (in LDS).
//
// One workgroup = 32 channels x all of K; its eight wavefronts take groups round-robin with up to six weight loads per
// lane in flight (all of a wavefront's groups at K = 3072); partial sums are added through LDS in a fixed order.
// A batched launch with five to eight rows gives a workgroup 64 channels where that leaves two workgroups per CU.
#include <type_traits>

#include "svdq_common.h"

namespace svdq {

constexpr int AWQ_WAVES = 8;  // wavefronts per workgroup (4 and 16 measured slower)
constexpr int AWQ_NB = 32;    // channels per workgroup
constexpr int AWQ_PF = 6;     // weight loads in flight per lane (all of a wavefront's groups at K = 3072)
constexpr size_t AWQ_LDS_MAX = 65536;  // dynamic LDS a launch may ask for

template <typename T>
struct AwqMagic;
template <>
struct AwqMagic<BF16> {
    static constexpr uint32_t bits = 0x43004300u;  // two bf16 128.0
    static constexpr float off = 128.0f;
};
template <>
struct AwqMagic<FP16> {
    static constexpr uint32_t bits = 0x64006400u;  // two fp16 1024.0
    static constexpr float off = 1024.0f;
};

// ((w >> sh) & mask) | magic with the mask held in a register so that the and/or pair is one v_and_or_b32
__device__ inline int nibble_plane(int w, int sh, uint32_t mask, uint32_t magic) {
    return (int)((((uint32_t)w >> sh) & mask) | magic);
}

__device__ inline v4i awq_wload(const v4i *p) {
    return __builtin_nontemporal_load(p);  // streamed once: do not keep in cache
}


// 4x4x4 MFMA in 16 independent blocks (block = lane / 4): D[block][row][col = lane % 4] += sum over 4 k of
// A[block][row = lane % 4][k] * B[block][k][col]; four 16-bit values per lane, passed as raw bits
template <typename T>
__device__ inline v4f mfma4_16bit(v2i a, v2i b, v4f c);
template <>
__device__ inline v4f mfma4_16bit<BF16>(v2i a, v2i b, v4f c) {
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(v4s, a), __builtin_bit_cast(v4s, b), c, 0, 0, 0);
}
template <>
__device__ inline v4f mfma4_16bit<FP16>(v2i a, v2i b, v4f c) {
    return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(v4h, a), __builtin_bit_cast(v4h, b), c, 0, 0, 0);
}

template <int CTRL>
__device__ inline float dpp_f32(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}

// M <= 8, RP = M rounded up to 1, 2, 4 or 8.
//
// The kernel is bound by instruction issue as much as by HBM (a wavefront has about 440 issue slots in the time its
// share of the weights streams in), so every wavefront works alone until the final sum and with as few instructions as
// possible: one global_load_lds for the activations of all its groups (RP = 1; one per 64 pieces otherwise), one for
// their scales and zeros, then the weight pieces into registers, all issued back to back in straight-line code so
// that each wait counts exactly the loads that must have returned; no workgroup barrier before the final sum.
//
// RP <= 4 uses the 4x4x4 MFMA (16 blocks of 4 channels x 4 rows, 8 cycles) in place of the 32x32x16 one (32 cycles for
// the same number of weights): block 2 q + h holds channels 4 q .. 4 q + 3 over half h of the group, so that the eight
// lanes of a channel quad still load one contiguous 128-byte piece of a packed row; the two halves are added in the
// final sum.  RP = 8 keeps the 32x32x16 MFMA with lane = (channel, half).
//
// LDS of wavefront w:  x tiles of its AWQ_PF groups (RP rows x 128 bytes each; the 16-byte piece pc of row r sits in
// slot pc ^ r, rows 128 bytes apart would otherwise meet in the same banks) | s of the groups (64 bytes each) | z;
// after the tables of all wavefronts: xs[w][group][8] fp32 = sums of the activations per (half, row) (RP <= 4) or per
// row (RP = 8).  The partial sums of the final reduction reuse the wavefront's own x tiles.
template <int RP, int CB = 1>
constexpr int awq_wave_bytes() { return AWQ_PF * RP * 128 + 2 * AWQ_PF * 64 * CB; }

//
// BATCH: one launch serves `count` weights of one shape (the adaLN projections of a model all take the same vector and
// differ only in their tensors): workgroup b works on problem b / (N / 32), whose five pointers it reads from `table`;
// everything else comes from `a`.  A 32 MB weight by itself is read at 60 % of the HBM peak at best (launch ramp and
// tail of a 6 us kernel); several in one launch stream like one long read.
//
// CB = 2 (RP = 8 only): the workgroup takes 64 channels, every wavefront both 32-channel blocks of its groups, so that
// the activation tiles, their sums and the MFMA A operand reads are paid once per 64 channels (at eight rows they are
// as many bytes out of L2 as the weights are out of HBM).  Half as many workgroups: for launches with enough of them.
template <typename T, int RP, bool BATCH, int CB = 1>
__global__ __launch_bounds__(AWQ_WAVES * 64) __attribute__((amdgpu_waves_per_eu(RP <= 4 ? 6 : 4))) void awq_gemv_rows_kernel(svdq_awq_gemv_args a, const svdq_awq_gemv_args *table) {
    static_assert(CB == 1 || (CB == 2 && RP == 8), "two channel blocks per wavefront only with eight rows");
    constexpr int NBW = AWQ_NB * CB;  // channels per workgroup
    extern __shared__ __align__(16) uint8_t lds8[];
    int blk = blockIdx.x;
    if constexpr (BATCH) {
        const int nblk = a.N / NBW, pi = blk / nblk;  // uniform: scalar loads
        blk -= pi * nblk;
        a.x = table[pi].x;
        a.qweight = table[pi].qweight;
        a.scales = table[pi].scales;
        a.zeros = table[pi].zeros;
        a.out = table[pi].out;
    }
    constexpr bool SMALL = RP <= 4;
    constexpr int WB = awq_wave_bytes<RP, CB>(), XPIECES = AWQ_PF * 8 * RP, XPASSES = (XPIECES + 63) / 64;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ngroups = a.K / GROUP;
    const int nb0 = blk * NBW;
    uint8_t *xw = lds8 + wave * WB, *szw = xw + AWQ_PF * RP * 128;
    float *xsw = (float *)(lds8 + AWQ_WAVES * WB) + wave * (AWQ_PF * 8);

    // channel and half of the group this lane multiplies
    const int ch = SMALL ? ((lane >> 3) << 2) | (lane & 3) : lane & 31;
    const int half = SMALL ? (lane >> 2) & 1 : lane >> 5;
    // weight piece: packed row n / 4, int16 column 64 c + 16 (n % 4) + 8 h  (byte offsets from the tensor, 32 bits)
    const uint32_t woff = ((uint32_t)((nb0 + ch) >> 2) * (uint32_t)a.K + 16 * (ch & 3) + 8 * half) * 2;
    // MFMA A operand: row min(lane % 4 or lane % 32, M - 1) (rows >= M land in accumulator rows nobody reads)
    const int arow = min(SMALL ? lane & 3 : lane & 31, a.M - 1);
    const uint8_t *aop = xw + arow * 128;
    int aslot[4];
#pragma unroll
    for (int pl = 0; pl < 4; pl++) aslot[pl] = 16 * ((4 * half + pl) ^ arow);

    uint32_t mask = 0x000F000Fu;
    asm volatile("" : "+v"(mask));  // keep the mask in a VGPR: v_and_or_b32 takes only one literal
    float acc[SMALL ? RP : 4 * CB];
#pragma unroll
    for (int i = 0; i < (SMALL ? RP : 4 * CB); i++) acc[i] = 0.0f;

    // One batch: NV groups c = base + 8 u of this wavefront (NV < AWQ_PF only in the last batch of a ragged K)
    auto batch = [&](auto nv_tag, int base) {
        constexpr int NV = decltype(nv_tag)::value;
        // activations: piece q = lane + 64 i is (group u = q / (8 RP), row r = (q / 8) % RP, slot q % 8)
#pragma unroll
        for (int i = 0; i < XPASSES; i++) {
            const int q = lane + 64 * i, u = q / (8 * RP), r = (q >> 3) & (RP - 1), slot = q & 7;
            const int c = min(base + AWQ_WAVES * u, ngroups - 1);
            const uint32_t off = ((uint32_t)min(r, a.M - 1) * (uint32_t)a.ld_x + c * GROUP + 8 * (slot ^ r)) * 2;
            if (XPIECES % 64 == 0 || i + 1 < XPASSES || q < XPIECES)
                __builtin_amdgcn_global_load_lds((const SVDQ_AS1 void *)((const uint8_t *)a.x + off), (SVDQ_AS3 void *)(xw + 1024 * i), 16, 0, 0);
        }
        if constexpr (CB == 2) {  // lanes 0 .. 8 PF - 1 = (group, 16-byte piece of its 64 channels), scales then zeros
            const int c = min(base + AWQ_WAVES * (lane >> 3), ngroups - 1);
            const uint32_t off = ((uint32_t)c * (uint32_t)a.ld_scales + nb0 + 8 * (lane & 7)) * 2;
            if (lane < 8 * AWQ_PF) {
                __builtin_amdgcn_global_load_lds((const SVDQ_AS1 void *)((const uint8_t *)a.scales + off), (SVDQ_AS3 void *)szw, 16, 0, 0);
                __builtin_amdgcn_global_load_lds((const SVDQ_AS1 void *)((const uint8_t *)a.zeros + off), (SVDQ_AS3 void *)(szw + AWQ_PF * 128), 16, 0, 0);
            }
        } else {   // scales: lanes 0 .. 4 PF - 1 = (group, 16-byte piece of its 32 channels); zeros: the next 4 PF lanes
            const bool z = lane >= 4 * AWQ_PF;
            const int t = lane - (z ? 4 * AWQ_PF : 0), c = min(base + AWQ_WAVES * (t >> 2), ngroups - 1);
            const uint32_t off = ((uint32_t)c * (uint32_t)a.ld_scales + nb0 + 8 * (t & 3)) * 2;
            if (lane < 8 * AWQ_PF)
                __builtin_amdgcn_global_load_lds((const SVDQ_AS1 void *)((const uint8_t *)(z ? a.zeros : a.scales) + off), (SVDQ_AS3 void *)szw, 16, 0, 0);
        }
        v4i wreg[NV * CB];  // channel block cb of group u in wreg[CB u + cb] (eight packed rows = 16 K bytes further on)
#pragma unroll
        for (int u = 0; u < NV; u++)
#pragma unroll
            for (int cb = 0; cb < CB; cb++)
                wreg[CB * u + cb] = awq_wload((const v4i *)((const uint8_t *)a.qweight + (woff + (uint32_t)cb * 16u * (uint32_t)a.K +
                                                                                          (uint32_t)(base + AWQ_WAVES * u) * (GROUP * 2))));
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(NV * CB, 15));  // activations, scales and zeros have landed
        // sums of the activations: every lane adds up its own piece, then the lanes of a (half) row are added
#pragma unroll
        for (int i = 0; i < XPASSES; i++) {
            const int q = min(lane + 64 * i, XPIECES - 1), u = q / (8 * RP), r = (q >> 3) & (RP - 1), slot = q & 7;
            const v4i v = *(const v4i *)(xw + 16 * q);
            float s = 0.0f;  // one dot-product instruction per pair of values (against (1, 1)) instead of two unpacks and two adds
#pragma unroll
            for (int e = 0; e < 4; e++) s = T::sum2((uint32_t)v[e], s);
            s += dpp_f32<0xB1>(s);  // quad_perm [1, 0, 3, 2]
            s += dpp_f32<0x4E>(s);  // quad_perm [2, 3, 0, 1]
            if (SMALL) {            // slots 4 h .. 4 h + 3 hold the pieces of half h (r < 4 permutes within them)
                if ((slot & 3) == 0) xsw[u * 8 + (slot >> 2) * 4 + r] = s;
            } else {
                s += dpp_f32<0x141>(s);  // row_half_mirror: lane i <-> 7 - i of the octet
                if (slot == 0) xsw[u * 8 + r] = s;
            }
        }
#pragma unroll
        for (int u = 0; u < NV; u++) {
            const v4i w = wreg[CB * u];
            const float s = T::to_f32(((const uint16_t *)szw)[u * NBW + ch]);
            const float zz = T::to_f32(((const uint16_t *)szw)[(AWQ_PF + u) * NBW + ch]) - AwqMagic<T>::off * s;
            const uint8_t *at = aop + u * (RP * 128);
            if constexpr (CB == 2) {
                v4i xa[4];
#pragma unroll
                for (int pl = 0; pl < 4; pl++) xa[pl] = *(const v4i *)(at + aslot[pl]);
                const v4f xv = *(const v4f *)(xsw + u * 8 + 4 * half);
#pragma unroll
                for (int cb = 0; cb < CB; cb++) {
                    const v4i wc = wreg[CB * u + cb];
                    const float sc = T::to_f32(((const uint16_t *)szw)[u * NBW + 32 * cb + ch]);
                    const float zc = T::to_f32(((const uint16_t *)szw)[(AWQ_PF + u) * NBW + 32 * cb + ch]) - AwqMagic<T>::off * sc;
                    v16f d;
#pragma unroll
                    for (int i = 0; i < 16; i++) d[i] = 0.0f;
#pragma unroll
                    for (int pl = 0; pl < 4; pl++) {
                        v4i wb;
#pragma unroll
                        for (int e = 0; e < 4; e++) wb[e] = nibble_plane(wc[e], 4 * pl, mask, AwqMagic<T>::bits);
                        d = mfma32_16bit<T>(xa[pl], wb, d);
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        acc[4 * cb + e] = __builtin_fmaf(sc, d[e], acc[4 * cb + e]);
                        acc[4 * cb + e] = __builtin_fmaf(zc, xv[e], acc[4 * cb + e]);
                    }
                }
            } else if constexpr (SMALL) {
                v4f d0 = {0.0f, 0.0f, 0.0f, 0.0f}, d1 = d0;
#pragma unroll
                for (int pl = 0; pl < 4; pl++) {
                    v4i wb;
#pragma unroll
                    for (int e = 0; e < 4; e++) wb[e] = nibble_plane(w[e], 4 * pl, mask, AwqMagic<T>::bits);
                    const v4i xa = *(const v4i *)(at + aslot[pl]);
                    d0 = mfma4_16bit<T>(v2i{xa[0], xa[1]}, v2i{wb[0], wb[1]}, d0);
                    d1 = mfma4_16bit<T>(v2i{xa[2], xa[3]}, v2i{wb[2], wb[3]}, d1);
                }
                const v4f xv = *(const v4f *)(xsw + u * 8 + 4 * half);
#pragma unroll
                for (int r = 0; r < RP; r++) {
                    acc[r] = __builtin_fmaf(s, d0[r] + d1[r], acc[r]);
                    acc[r] = __builtin_fmaf(zz, xv[r], acc[r]);
                }
            } else {
                v16f d;
#pragma unroll
                for (int i = 0; i < 16; i++) d[i] = 0.0f;
#pragma unroll
                for (int pl = 0; pl < 4; pl++) {
                    v4i wb;
#pragma unroll
                    for (int e = 0; e < 4; e++) wb[e] = nibble_plane(w[e], 4 * pl, mask, AwqMagic<T>::bits);
                    const v4i xa = *(const v4i *)(at + aslot[pl]);
                    d = mfma32_16bit<T>(xa, wb, d);
                }
                const v4f xv = *(const v4f *)(xsw + u * 8 + 4 * half);
#pragma unroll
                for (int e = 0; e < 4; e++) {  // accumulator register e = row 4 h + e (rows 0 .. 7)
                    acc[e] = __builtin_fmaf(s, d[e], acc[e]);
                    acc[e] = __builtin_fmaf(zz, xv[e], acc[e]);
                }
            }
        }
    };
    for (int base = wave; base < ngroups; base += AWQ_PF * AWQ_WAVES) {
        const int nv = (ngroups - base + AWQ_WAVES - 1) / AWQ_WAVES;  // wave-uniform
        if (nv >= AWQ_PF) batch(std::integral_constant<int, AWQ_PF>{}, base);
        else if (nv == 5) batch(std::integral_constant<int, 5>{}, base);
        else if (nv == 4) batch(std::integral_constant<int, 4>{}, base);
        else if (nv == 3) batch(std::integral_constant<int, 3>{}, base);
        else if (nv == 2) batch(std::integral_constant<int, 2>{}, base);
        else batch(std::integral_constant<int, 1>{}, base);
    }

    // fixed-order sum over the wavefronts (and halves): partial sums [half][row][channel] (RP <= 4) or [row][channel]
    // in the wavefront's own, now unused, x tiles; then store T
    float *red = (float *)xw;
    if constexpr (SMALL) {
#pragma unroll
        for (int r = 0; r < RP; r++) red[(half * RP + r) * AWQ_NB + ch] = acc[r];
    } else {
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
#pragma unroll
            for (int e = 0; e < 4; e++) red[(4 * half + e) * NBW + 32 * cb + ch] = acc[4 * cb + e];
    }
    __syncthreads();
    if (tid < a.M * NBW) {
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < AWQ_WAVES; w++) {
            const float *rw = (const float *)(lds8 + w * WB);
            if constexpr (SMALL)
                s += rw[tid] + rw[RP * AWQ_NB + tid];
            else
                s += rw[tid];
        }
        ((uint16_t *)a.out)[(size_t)(tid / NBW) * a.ld_out + nb0 + tid % NBW] = T::from_f32(s);
    }
}

// 8 < M <= 32, MQ = ceil(M / 8) accumulator register quads hold real rows.  One workgroup = 32 channels x all of K; its
// wavefronts take groups round-robin; the scales and zeros of the channels and the group sums of the activations are
// staged in LDS, the MFMA A operand is read from global memory (L2: every workgroup reads the same rows).
template <typename T, int MQ>
__global__ __launch_bounds__(AWQ_WAVES * 64) void awq_gemv_kernel(svdq_awq_gemv_args a) {
    // xs[K/64][8*MQ] fp32 | red[AWQ_WAVES][8*MQ][32] fp32 | sz[K/64][2][32] 16-bit
    extern __shared__ __align__(16) float lds[];
    constexpr int MR = 8 * MQ;
    const int ngroups = a.K / GROUP;
    float *xs = lds;
    float *red = lds + (size_t)ngroups * MR;
    uint16_t *sz = (uint16_t *)(red + AWQ_WAVES * MR * AWQ_NB);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keep it in an SGPR
    const int l32 = lane & 31, half = lane >> 5;
    const int nb0 = blockIdx.x * AWQ_NB;
    const int n = nb0 + l32;
    const uint16_t *__restrict__ x = (const uint16_t *)a.x;

    // scales / zeros of the 32 channels: group c, 64 bytes each -> thread (c = p / 4, piece = p % 4)
    for (int p = tid; p < ngroups * 4; p += AWQ_WAVES * 64) {
        *(v4i *)(sz + ((p >> 2) * 2 + 0) * AWQ_NB + 8 * (p & 3)) =
            *(const v4i *)((const uint16_t *)a.scales + (size_t)(p >> 2) * a.ld_scales + nb0 + 8 * (p & 3));
        *(v4i *)(sz + ((p >> 2) * 2 + 1) * AWQ_NB + 8 * (p & 3)) =
            *(const v4i *)((const uint16_t *)a.zeros + (size_t)(p >> 2) * a.ld_scales + nb0 + 8 * (p & 3));
    }
    // xs[c][m] = sum of the group's 64 activations (fp32)
    for (int p = tid; p < ngroups * MR; p += AWQ_WAVES * 64) {
        const int c = p / MR, m = p % MR;
        float s = 0.0f;
        if (m < a.M) {
            const v4i *xp = (const v4i *)(x + (size_t)m * a.ld_x + c * GROUP);
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const v4i v = xp[q];
#pragma unroll
                for (int e = 0; e < 4; e++) s += T::lo_f32((uint32_t)v[e]) + T::hi_f32((uint32_t)v[e]);
            }
        }
        xs[p] = s;
    }
    __syncthreads();

    float acc[4 * MQ];
#pragma unroll
    for (int i = 0; i < 4 * MQ; i++) acc[i] = 0.0f;

    // this lane's weight stream: packed row n / 4, int16 column 64 c + 16 (n % 4) + 8 h, groups c = wave + 8 i
    const uint16_t *__restrict__ wq = (const uint16_t *)a.qweight + (size_t)(n >> 2) * a.K + 16 * (n & 3) + 8 * half;
    // A operand row of this lane; rows >= M repeat row M - 1 (their products land in accumulator rows nobody reads)
    const uint16_t *xrow = x + (size_t)min(l32, a.M - 1) * a.ld_x + 32 * half;
    uint32_t mask = 0x000F000Fu;
    asm volatile("" : "+v"(mask));  // keep the mask in a VGPR: v_and_or_b32 takes only one literal
    v16f zero16;
#pragma unroll
    for (int i = 0; i < 16; i++) zero16[i] = 0.0f;

    for (int base = wave; base < ngroups; base += AWQ_PF * AWQ_WAVES) {
        // AWQ_PF weight loads in flight, issued without branches (past the end the last group is fetched again) so
        // that every wait counts exactly the loads that must have returned
        v4i wreg[AWQ_PF];
#pragma unroll
        for (int u = 0; u < AWQ_PF; u++)
            wreg[u] = awq_wload((const v4i *)(wq + (size_t)min(base + AWQ_WAVES * u, ngroups - 1) * GROUP));
#pragma unroll
        for (int u = 0; u < AWQ_PF; u++) {
            const int c = base + AWQ_WAVES * u;
            if (c < ngroups) {
                const v4i w = wreg[u];
                const float s = T::to_f32(sz[(c * 2 + 0) * AWQ_NB + l32]);
                const float zz = T::to_f32(sz[(c * 2 + 1) * AWQ_NB + l32]) - AwqMagic<T>::off * s;
                const uint16_t *xg = xrow + c * GROUP;
                v16f d;
#pragma unroll
                for (int pl = 0; pl < 4; pl++) {
                    v4i wb;
#pragma unroll
                    for (int e = 0; e < 4; e++) wb[e] = nibble_plane(w[e], 4 * pl, mask, AwqMagic<T>::bits);
                    const v4i xa = *(const v4i *)(xg + 8 * pl);
                    d = mfma32_16bit<T>(xa, wb, pl == 0 ? zero16 : d);
                }
#pragma unroll
                for (int q = 0; q < MQ; q++) {
                    const v4f xv = *(const v4f *)(xs + c * MR + 8 * q + 4 * half);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        acc[4 * q + e] = __builtin_fmaf(s, d[4 * q + e], acc[4 * q + e]);
                        acc[4 * q + e] = __builtin_fmaf(zz, xv[e], acc[4 * q + e]);
                    }
                }
            }
        }
    }

    // fixed-order sum over the wavefronts, then store T
#pragma unroll
    for (int q = 0; q < MQ; q++)
#pragma unroll
        for (int e = 0; e < 4; e++) red[(wave * MR + 8 * q + 4 * half + e) * AWQ_NB + l32] = acc[4 * q + e];
    __syncthreads();
    for (int o = tid; o < a.M * AWQ_NB; o += AWQ_WAVES * 64) {
        const int m = o / AWQ_NB, nn = o % AWQ_NB;
        float s = red[(0 * MR + m) * AWQ_NB + nn];
#pragma unroll
        for (int w = 1; w < AWQ_WAVES; w++) s += red[(w * MR + m) * AWQ_NB + nn];
        ((uint16_t *)a.out)[(size_t)m * a.ld_out + nb0 + nn] = T::from_f32(s);
    }
}

// Dense decode of a TinyChat-packed weight: out[n, k] = T(q[n, k] * s[k / group, n] + z[k / group, n]), fp32 arithmetic
// (reference: nunchaku/ops/triton/awq.py:48-79; q * s is exact in fp32, so there is one rounding before the one to T).
// Thread idx walks the packed tensor in storage order, 16 bytes each: piece (a = n / 4, c = k / 64, b = n % 4,
// h = (k / 32) % 2) holds eight int16 whose nibble j' is k = 64 c + 32 h + 8 j' + j (j = position of the int16), i.e.
// the 32 consecutive outputs out[n, 64 c + 32 h ... + 32): reads are contiguous, stores are 64-byte row pieces.
template <typename T>
__global__ __launch_bounds__(256) void awq_dequant_kernel(const v4i *__restrict__ qweight, const uint16_t *__restrict__ scales,
                                                          const uint16_t *__restrict__ zeros, uint16_t *__restrict__ out,
                                                          int N, int K, int group, int ld_scales, int ld_out) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int g64 = K / GROUP;
    if (idx >= (size_t)(N / 4) * g64 * 8) return;
    const int h = idx & 1, b = (idx >> 1) & 3;
    const int c = (int)((idx >> 3) % g64), a = (int)((idx >> 3) / g64);
    const int n = 4 * a + b, k0 = GROUP * c + 32 * h;
    const v4i w = awq_wload(qweight + idx);
    const float s = T::to_f32(scales[(size_t)(k0 / group) * ld_scales + n]);
    const float z = T::to_f32(zeros[(size_t)(k0 / group) * ld_scales + n]);
    uint16_t *o = out + (size_t)n * ld_out + k0;
#pragma unroll
    for (int jp = 0; jp < 4; jp++) {  // nibble jp of the eight int16 = eight consecutive k
        v4i r;
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t word = (uint32_t)w[d];  // int16 2 d (low half) and 2 d + 1
            const float lo = (float)((word >> (4 * jp)) & 15u), hi = (float)((word >> (16 + 4 * jp)) & 15u);
            r[d] = (int)pack2<T>(__builtin_fmaf(lo, s, z), __builtin_fmaf(hi, s, z));
        }
        *(v4i *)(o + 8 * jp) = r;
    }
}

// LDS of a launch with more than eight rows (the kernels for up to eight rows need a fixed amount)
static size_t awq_lds_bytes(int K, int M) {
    if (M <= 8) return 0;
    const int MQ = (M + 7) / 8;
    size_t b = ((size_t)(K / GROUP) * 8 * MQ + (size_t)AWQ_WAVES * 8 * MQ * AWQ_NB) * sizeof(float);
    b += (size_t)(K / GROUP) * 2 * AWQ_NB * 2;
    return b;
}

template <typename T, bool BATCH>
static void launch_awq_rows(const svdq_awq_gemv_args &a, const svdq_awq_gemv_args *table, int count, hipStream_t s) {
    const dim3 grid((unsigned)(a.N / AWQ_NB) * (unsigned)count), block(AWQ_WAVES * 64);
    constexpr size_t XS_BYTES = (size_t)AWQ_WAVES * AWQ_PF * 8 * sizeof(float);
    // 64-channel workgroups once the launch still has two and more of them for each of the 256 CUs
    if constexpr (BATCH) if (a.M > 4 && a.N % (2 * AWQ_NB) == 0 && (size_t)(a.N / (2 * AWQ_NB)) * (size_t)count >= 512) {
        constexpr size_t LDS2 = (size_t)AWQ_WAVES * awq_wave_bytes<8, 2>() + XS_BYTES;
        hipLaunchKernelGGL((awq_gemv_rows_kernel<T, 8, BATCH, 2>), dim3(grid.x / 2), block, LDS2, s, a, table);
        return;
    }
    if (a.M <= 1)
        hipLaunchKernelGGL((awq_gemv_rows_kernel<T, 1, BATCH>), grid, block, AWQ_WAVES * awq_wave_bytes<1>() + XS_BYTES, s, a, table);
    else if (a.M <= 2)
        hipLaunchKernelGGL((awq_gemv_rows_kernel<T, 2, BATCH>), grid, block, AWQ_WAVES * awq_wave_bytes<2>() + XS_BYTES, s, a, table);
    else if (a.M <= 4)
        hipLaunchKernelGGL((awq_gemv_rows_kernel<T, 4, BATCH>), grid, block, AWQ_WAVES * awq_wave_bytes<4>() + XS_BYTES, s, a, table);
    else
        hipLaunchKernelGGL((awq_gemv_rows_kernel<T, 8, BATCH>), grid, block, AWQ_WAVES * awq_wave_bytes<8>() + XS_BYTES, s, a, table);
}

template <typename T>
static void launch_awq(const svdq_awq_gemv_args &a, hipStream_t s) {
    if (a.M <= 8) {
        launch_awq_rows<T, false>(a, nullptr, 1, s);
        return;
    }
    const dim3 grid(a.N / AWQ_NB), block(AWQ_WAVES * 64);
    const size_t sh = awq_lds_bytes(a.K, a.M);
    if (a.M <= 16)
        hipLaunchKernelGGL((awq_gemv_kernel<T, 2>), grid, block, sh, s, a);
    else if (a.M <= 24)
        hipLaunchKernelGGL((awq_gemv_kernel<T, 3>), grid, block, sh, s, a);
    else
        hipLaunchKernelGGL((awq_gemv_kernel<T, 4>), grid, block, sh, s, a);
}

}  // namespace svdq

using namespace svdq;

// shape and the tensors of one problem; `what` names the entry point in messages
static int awq_check(const svdq_awq_gemv_args &a, const char *what, int max_rows) {
    if (a.dtype != SVDQ_BF16 && a.dtype != SVDQ_FP16) {
        set_error("%s: dtype %d", what, a.dtype);
        return SVDQ_E_INVALID;
    }
    if (a.M < 0 || a.M > max_rows || a.N <= 0 || a.N % AWQ_NB || a.K <= 0 || a.K % GROUP) {
        set_error("%s: M=%d N=%d K=%d needs M <= %d, N %% 32 == 0, K %% 64 == 0", what, a.M, a.N, a.K, max_rows);
        return SVDQ_E_INVALID;
    }
    if (!a.x || !a.qweight || !a.scales || !a.zeros || !a.out) {
        set_error("%s: null tensor", what);
        return SVDQ_E_INVALID;
    }
    if (((uintptr_t)a.x & 15) || a.ld_x % 8 || a.ld_x < a.K || ((uintptr_t)a.qweight & 15) || a.ld_scales < a.N ||
        a.ld_out < a.N || ((uintptr_t)a.scales & 15) || ((uintptr_t)a.zeros & 15) || a.ld_scales % 8) {
        set_error("%s: x rows, qweight and scale / zero rows must be 16-byte aligned; leading dimensions >= row length", what);
        return SVDQ_E_INVALID;
    }
    if (awq_lds_bytes(a.K, a.M) > AWQ_LDS_MAX) {  // K = 12288 with M > 16, K > 16384 with M > 8
        set_error("%s: K=%d with M=%d needs %zu bytes of LDS tables (limit %zu)", what, a.K, a.M, awq_lds_bytes(a.K, a.M), AWQ_LDS_MAX);
        return SVDQ_E_UNSUPPORTED;
    }
    if (a.M <= 8 && ((size_t)a.N * a.K / 2 >= ((size_t)1 << 32) || (size_t)(a.K / GROUP) * a.ld_scales * 2 >= ((size_t)1 << 32) ||
                     (size_t)a.M * a.ld_x * 2 >= ((size_t)1 << 32))) {  // the kernel for up to eight rows addresses with 32-bit byte offsets
        set_error("%s: N=%d K=%d ld_scales=%d ld_x=%d: a tensor of 4 GiB or more", what, a.N, a.K, a.ld_scales, a.ld_x);
        return SVDQ_E_UNSUPPORTED;
    }
    return SVDQ_OK;
}

extern "C" int svdq_awq_gemv_w4a16(const svdq_awq_gemv_args *args, void *stream) {
    if (!args) {
        set_error("svdq_awq_gemv_w4a16: null args");
        return SVDQ_E_INVALID;
    }
    const svdq_awq_gemv_args &a = *args;
    const int rc = awq_check(a, "svdq_awq_gemv_w4a16", 32);
    if (rc) return rc;
    if (a.M == 0) return SVDQ_OK;
    if (a.dtype == SVDQ_BF16)
        launch_awq<BF16>(a, (hipStream_t)stream);
    else
        launch_awq<FP16>(a, (hipStream_t)stream);
    return check_launch("svdq_awq_gemv_w4a16");
}

extern "C" int svdq_awq_gemv_w4a16_batched(const svdq_awq_gemv_args *first, const svdq_awq_gemv_args *problems, int32_t count,
                                           void *stream) {
    if (!first || !problems || count <= 0 || ((uintptr_t)problems & 7)) {
        set_error("svdq_awq_gemv_w4a16_batched: needs the first problem (host), the table of all problems (device) and count > 0");
        return SVDQ_E_INVALID;
    }
    const svdq_awq_gemv_args &a = *first;
    const int rc = awq_check(a, "svdq_awq_gemv_w4a16_batched", 8);
    if (rc) return rc;
    if ((size_t)(a.N / AWQ_NB) * (size_t)count >= ((size_t)1 << 31)) {
        set_error("svdq_awq_gemv_w4a16_batched: %d problems of N=%d are too many workgroups for one launch", count, a.N);
        return SVDQ_E_UNSUPPORTED;
    }
    if (a.M == 0) return SVDQ_OK;
    if (a.dtype == SVDQ_BF16)
        launch_awq_rows<BF16, true>(a, problems, count, (hipStream_t)stream);
    else
        launch_awq_rows<FP16, true>(a, problems, count, (hipStream_t)stream);
    return check_launch("svdq_awq_gemv_w4a16_batched");
}

extern "C" int svdq_awq_dequantize(const void *qweight, const void *scales, const void *zeros, void *out, int32_t N,
                                   int32_t K, int32_t group_size, int32_t ld_scales, int32_t ld_out, int32_t dtype,
                                   void *stream) {
    if (dtype != SVDQ_BF16 && dtype != SVDQ_FP16) {
        set_error("svdq_awq_dequantize: dtype %d", dtype);
        return SVDQ_E_INVALID;
    }
    if (N <= 0 || N % 4 || K <= 0 || K % GROUP || group_size <= 0 || group_size % 32 || K % group_size) {
        set_error("svdq_awq_dequantize: N=%d K=%d group_size=%d needs N %% 4 == 0, K %% 64 == 0, group_size %% 32 == 0 dividing K",
                  N, K, group_size);
        return SVDQ_E_INVALID;
    }
    if (!qweight || !scales || !zeros || !out || ((uintptr_t)qweight & 15) || ((uintptr_t)out & 15) || ld_out % 8 ||
        ld_out < K || ld_scales < N) {
        set_error("svdq_awq_dequantize: qweight and out rows must be 16-byte aligned; ld_out >= K, ld_scales >= N");
        return SVDQ_E_INVALID;
    }
    const size_t pieces = (size_t)(N / 4) * (K / GROUP) * 8;
    const dim3 grid((unsigned)((pieces + 255) / 256)), block(256);
    if (dtype == SVDQ_BF16)
        hipLaunchKernelGGL(awq_dequant_kernel<BF16>, grid, block, 0, (hipStream_t)stream, (const v4i *)qweight,
                           (const uint16_t *)scales, (const uint16_t *)zeros, (uint16_t *)out, N, K, group_size, ld_scales, ld_out);
    else
        hipLaunchKernelGGL(awq_dequant_kernel<FP16>, grid, block, 0, (hipStream_t)stream, (const v4i *)qweight,
                           (const uint16_t *)scales, (const uint16_t *)zeros, (uint16_t *)out, N, K, group_size, ld_scales, ld_out);
    return check_launch("svdq_awq_dequantize");
}
