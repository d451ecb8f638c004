// AWQ W4A16 GEMV (group 64, TinyChat-packed weights) for gfx950, small M (<= 32 rows).
//
// Arithmetic (reference: nunchaku/ops/triton/awq.py:160-182):
//   out[m, n] = sum_c  s[c, n] * sum_{k in c} x[m, k] q[n, k]  +  z[c, n] * sum_{k in c} x[m, k]      (fp32)
//
// The kernel is HBM-bound: N*K/2 bytes of weights are read exactly once, for all M rows together (the reference
// launches one pass over the weights per row).
//
// Storage order is the access order.  Packed row a = n / 4 holds, for scale group c, 128 contiguous bytes =
// 4 channels (b = n % 4) x 2 halves (h) x 16 bytes; the 16 bytes of (n, c, h) are eight int16 whose nibble j' holds
// k = 64 c + 32 h + 8 j' + j (j = position of the int16).  Lane (n = lane % 32, h = lane / 32) of a wavefront loads
// exactly that 16-byte piece, so one load instruction reads 8 packed rows x 128 contiguous bytes.  Nibble plane j' of
// the loaded dwords, OR-ed with the bit pattern of 128.0 (bf16) / 1024.0 (fp16), is directly the B operand of one
// 32x32x16 MFMA (exact: 128 + q and 1024 + q are representable); the A operand is the matching 16 bytes of x.  Four
// MFMAs cover the group; the constant offset is folded into the zero-point term:
//   s * (D - OFF * xs) + z * xs = s * D + (z - OFF * s) * xs,   xs = sum_{k in c} x[m, k]  (precomputed in LDS).
// Only accumulator registers whose rows are < M are post-processed (rows m = 8 (i / 4) + 4 h + i % 4).
//
// One workgroup = 32 channels x all of K; its eight wavefronts take groups round-robin.  The small loads (activations,
// the channels' scales and zeros) are issued first and staged in LDS while up to six weight loads per lane (all of a
// wavefront's groups at K = 3072) are in flight; partial sums are added through LDS in a fixed order.  Up to eight rows
// of activations are staged in LDS as well when they fit next to the tables (M = 8 up to K = 3072, M = 2 up to
// K = 12288); otherwise the MFMA operand is read from global memory.
#include "svdq_common.h"

namespace svdq {

constexpr int AWQ_WAVES = 8;  // wavefronts per workgroup (4 and 16 measured slower)
constexpr int AWQ_NB = 32;    // channels per workgroup
constexpr int AWQ_PF = 6;     // weight loads in flight per lane (all of a wavefront's groups at K = 3072)
constexpr int AWQ_XPAD = 8;   // 16-bit elements of padding per staged activation row
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

// MQ = ceil(M / 8): accumulator register quads that hold real rows; X_IN_LDS: the activations are staged in LDS
template <typename T, int MQ, bool X_IN_LDS>
__global__ __launch_bounds__(AWQ_WAVES * 64, 6) void awq_gemv_kernel(svdq_awq_gemv_args a) {
    // xs[K/64][8*MQ] fp32 | red[AWQ_WAVES][8*MQ][32] fp32 | sz[K/64][2][32] 16-bit | (X_IN_LDS) x[M][K + pad] 16-bit
    extern __shared__ __align__(16) float lds[];
    constexpr int MR = 8 * MQ;
    const int ngroups = a.K / GROUP;
    float *xs = lds;
    float *red = lds + (size_t)ngroups * MR;
    uint16_t *sz = (uint16_t *)(red + AWQ_WAVES * MR * AWQ_NB);
    uint16_t *xl = sz + (size_t)ngroups * 2 * AWQ_NB;
    const int xld = a.K + AWQ_XPAD;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keep it in an SGPR
    const int l32 = lane & 31, half = lane >> 5;
    const int nb0 = blockIdx.x * AWQ_NB;
    const int n = nb0 + l32;
    const uint16_t *__restrict__ x = (const uint16_t *)a.x;

    // 1. the small loads first (activations, scales, zeros), so that waiting for them does not wait for the weights
    v4i xst[3];  // up to 3 x 16-byte pieces of activations per thread (M * K / 8 <= 3 * 256 covers M = 2 at K = 3072)
    const int per_row = a.K / 8, xpieces = X_IN_LDS ? a.M * per_row : 0;
    if (X_IN_LDS) {
#pragma unroll
        for (int u = 0; u < 3; u++) {
            const int p = tid + u * AWQ_WAVES * 64;
            if (p < xpieces) xst[u] = *(const v4i *)(x + (size_t)(p / per_row) * a.ld_x + 8 * (p % per_row));
        }
    }
    // scales / zeros of the 32 channels: group c, 64 bytes each -> thread (c = p / 4, piece = p % 4)
    v4i sst[2], zst[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int p = tid + u * AWQ_WAVES * 64;
        if (p < ngroups * 4) {
            sst[u] = *(const v4i *)((const uint16_t *)a.scales + (size_t)(p >> 2) * a.ld_scales + nb0 + 8 * (p & 3));
            zst[u] = *(const v4i *)((const uint16_t *)a.zeros + (size_t)(p >> 2) * a.ld_scales + nb0 + 8 * (p & 3));
        }
    }

    // 2. this lane's weight stream: packed row n / 4, int16 column 64 c + 16 (n % 4) + 8 h, groups c = wave + 4 i
    const uint16_t *__restrict__ wq =
        (const uint16_t *)a.qweight + (size_t)(n >> 2) * a.K + 16 * (n & 3) + 8 * half + (size_t)wave * GROUP;
    const int wstep = AWQ_WAVES * GROUP;
    const int nmy = (ngroups - wave + AWQ_WAVES - 1) / AWQ_WAVES;
    v4i wreg[AWQ_PF];
#pragma unroll
    for (int u = 0; u < AWQ_PF; u++)
        if (u < nmy) wreg[u] = awq_wload((const v4i *)(wq + (size_t)u * wstep));

    // 3. stage the small data in LDS
    if (X_IN_LDS) {
#pragma unroll
        for (int u = 0; u < 3; u++) {
            const int p = tid + u * AWQ_WAVES * 64;
            if (p < xpieces) *(v4i *)(xl + (p / per_row) * xld + 8 * (p % per_row)) = xst[u];
        }
        for (int p = tid + 3 * AWQ_WAVES * 64; p < xpieces; p += AWQ_WAVES * 64)  // more rows: plain copy loop
            *(v4i *)(xl + (p / per_row) * xld + 8 * (p % per_row)) = *(const v4i *)(x + (size_t)(p / per_row) * a.ld_x + 8 * (p % per_row));
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int p = tid + u * AWQ_WAVES * 64;
        if (p < ngroups * 4) {
            *(v4i *)(sz + ((p >> 2) * 2 + 0) * AWQ_NB + 8 * (p & 3)) = sst[u];
            *(v4i *)(sz + ((p >> 2) * 2 + 1) * AWQ_NB + 8 * (p & 3)) = zst[u];
        }
    }
    for (int p = tid + 2 * AWQ_WAVES * 64; p < ngroups * 4; p += AWQ_WAVES * 64) {  // K > 8192
        *(v4i *)(sz + ((p >> 2) * 2 + 0) * AWQ_NB + 8 * (p & 3)) =
            *(const v4i *)((const uint16_t *)a.scales + (size_t)(p >> 2) * a.ld_scales + nb0 + 8 * (p & 3));
        *(v4i *)(sz + ((p >> 2) * 2 + 1) * AWQ_NB + 8 * (p & 3)) =
            *(const v4i *)((const uint16_t *)a.zeros + (size_t)(p >> 2) * a.ld_scales + nb0 + 8 * (p & 3));
    }
    __syncthreads();
    // xs[c][m] = sum of the group's 64 activations (fp32)
    for (int p = tid; p < ngroups * MR; p += AWQ_WAVES * 64) {
        const int c = p / MR, m = p % MR;
        float s = 0.0f;
        if (m < a.M) {
            const v4i *xp = X_IN_LDS ? (const v4i *)(xl + m * xld + c * GROUP) : (const v4i *)(x + (size_t)m * a.ld_x + c * GROUP);
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

    // A operand row of this lane; rows >= M repeat row M - 1 (their products land in accumulator rows nobody reads)
    const int arow = min(l32, a.M - 1);
    const uint16_t *xrow = (X_IN_LDS ? xl + arow * xld : x + (size_t)arow * a.ld_x) + 32 * half + wave * GROUP;
    const float *xsp = xs + wave * MR + 4 * half;
    const uint16_t *szp = sz + wave * 2 * AWQ_NB + l32;
    uint32_t mask = 0x000F000Fu;
    asm volatile("" : "+v"(mask));  // keep the mask in a VGPR: v_and_or_b32 takes only one literal
    v16f zero16;
#pragma unroll
    for (int i = 0; i < 16; i++) zero16[i] = 0.0f;

    for (int base = 0;;) {
#pragma unroll
        for (int u = 0; u < AWQ_PF; u++) {
            const int idx = base + u;
            if (idx < nmy) {
                const v4i w = wreg[u];
                const float s = T::to_f32(szp[idx * (AWQ_WAVES * 2 * AWQ_NB)]);
                const float zz = T::to_f32(szp[idx * (AWQ_WAVES * 2 * AWQ_NB) + AWQ_NB]) - AwqMagic<T>::off * s;
                const uint16_t *xg = xrow + idx * wstep;
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
                    const v4f xv = *(const v4f *)(xsp + idx * (AWQ_WAVES * MR) + 8 * q);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        acc[4 * q + e] = __builtin_fmaf(s, d[4 * q + e], acc[4 * q + e]);
                        acc[4 * q + e] = __builtin_fmaf(zz, xv[e], acc[4 * q + e]);
                    }
                }
            }
        }
        base += AWQ_PF;
        if (base >= nmy) break;
#pragma unroll
        for (int u = 0; u < AWQ_PF; u++)  // K > 3072: next batch of this wavefront's groups
            if (base + u < nmy) wreg[u] = awq_wload((const v4i *)(wq + (size_t)(base + u) * wstep));
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

// LDS of a launch without the staged activations, and the bytes those would add
static size_t awq_lds_bytes(int K, int M) {
    const int MQ = (M + 7) / 8;
    size_t b = ((size_t)(K / GROUP) * 8 * MQ + (size_t)AWQ_WAVES * 8 * MQ * AWQ_NB) * sizeof(float);
    b += (size_t)(K / GROUP) * 2 * AWQ_NB * 2;
    return b;
}
static size_t awq_x_lds_bytes(int K, int M) { return (size_t)M * (K + AWQ_XPAD) * 2; }
static bool awq_stage_x(int K, int M) {
    // wherever they fit: read from global memory instead, the eight rows of M = 8 cost 17.6 us against 12.6 us at the
    // FLUX adaLN shape (four 16-byte activation loads per lane and group next to one weight load)
    return M <= 8 && awq_lds_bytes(K, M) + awq_x_lds_bytes(K, M) <= AWQ_LDS_MAX;
}

template <typename T>
static void launch_awq(const svdq_awq_gemv_args &a, hipStream_t s) {
    const int MQ = (a.M + 7) / 8;
    const dim3 grid(a.N / AWQ_NB), block(AWQ_WAVES * 64);
    const bool xl = awq_stage_x(a.K, a.M);
    const size_t sh = awq_lds_bytes(a.K, a.M) + (xl ? awq_x_lds_bytes(a.K, a.M) : 0);
    switch (MQ) {
        case 1:
            if (xl)
                hipLaunchKernelGGL((awq_gemv_kernel<T, 1, true>), grid, block, sh, s, a);
            else
                hipLaunchKernelGGL((awq_gemv_kernel<T, 1, false>), grid, block, sh, s, a);
            break;
        case 2: hipLaunchKernelGGL((awq_gemv_kernel<T, 2, false>), grid, block, sh, s, a); break;
        case 3: hipLaunchKernelGGL((awq_gemv_kernel<T, 3, false>), grid, block, sh, s, a); break;
        default: hipLaunchKernelGGL((awq_gemv_kernel<T, 4, false>), grid, block, sh, s, a); break;
    }
}

}  // namespace svdq

using namespace svdq;

extern "C" int svdq_awq_gemv_w4a16(const svdq_awq_gemv_args *args, void *stream) {
    if (!args) {
        set_error("svdq_awq_gemv_w4a16: null args");
        return SVDQ_E_INVALID;
    }
    const svdq_awq_gemv_args &a = *args;
    if (a.dtype != SVDQ_BF16 && a.dtype != SVDQ_FP16) {
        set_error("svdq_awq_gemv_w4a16: dtype %d", a.dtype);
        return SVDQ_E_INVALID;
    }
    if (a.M < 0 || a.M > 32 || a.N <= 0 || a.N % AWQ_NB || a.K <= 0 || a.K % GROUP) {
        set_error("svdq_awq_gemv_w4a16: M=%d N=%d K=%d needs M <= 32, N %% 32 == 0, K %% 64 == 0", a.M, a.N, a.K);
        return SVDQ_E_INVALID;
    }
    if (!a.x || !a.qweight || !a.scales || !a.zeros || !a.out) {
        set_error("svdq_awq_gemv_w4a16: null tensor");
        return SVDQ_E_INVALID;
    }
    if (((uintptr_t)a.x & 15) || a.ld_x % 8 || a.ld_x < a.K || ((uintptr_t)a.qweight & 15) || a.ld_scales < a.N ||
        a.ld_out < a.N || ((uintptr_t)a.scales & 15) || ((uintptr_t)a.zeros & 15) || a.ld_scales % 8) {
        set_error("svdq_awq_gemv_w4a16: x rows, qweight and scale / zero rows must be 16-byte aligned; leading dimensions >= row length");
        return SVDQ_E_INVALID;
    }
    if (awq_lds_bytes(a.K, a.M) > AWQ_LDS_MAX) {  // K = 12288 with M > 16, K > 16384 with M > 8
        set_error("svdq_awq_gemv_w4a16: K=%d with M=%d needs %zu bytes of LDS tables (limit %zu)", a.K, a.M,
                  awq_lds_bytes(a.K, a.M), AWQ_LDS_MAX);
        return SVDQ_E_UNSUPPORTED;
    }
    if (a.M == 0) return SVDQ_OK;
    if (a.dtype == SVDQ_BF16)
        launch_awq<BF16>(a, (hipStream_t)stream);
    else
        launch_awq<FP16>(a, (hipStream_t)stream);
    return check_launch("svdq_awq_gemv_w4a16");
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
