// Checkpoint ingestion: tensors as the published SVDQuant int4 checkpoints hold them -> the natural layouts the
// kernels here read.  The checkpoints store every tensor of a quantized linear pre-shuffled for the register
// fragments of NVIDIA's mma.m16n8k32 (reference: nunchaku/lora/flux/packer.py:173-226 pack_weight, :228-262
// pack_scale, :300-338 pack_lowrank_weight; the inverse the reference applies at load time is
// nunchaku/ops/triton/layout.py:36-120, :155-184, :226-292).  All three are pure permutations, done here in one pass
// on the device, one element group per thread, reads gathered and writes coalesced.
//
// Index algebra (n = output row, k = input column, "lane" = the CUDA lane that owned the element):
//  * weight: a 32-bit word holds 8 consecutive k of one row, nibble j = k + j, which is also the natural byte order
//    (low nibble = even k), so words move whole.  With n = 128 nt + 16 np + 8 ns + nl and k = 64 kt + 32 ks + 8 kl,
//    the checkpoint keeps the word at index (((((nt KT + kt) 8 + np) 8 + nl) 4 + kl) 2 + ns) 2 + ks.
//  * scale (16-bit; per group or one vector): n = 128 ng + 16 a + 8 b + 2 c + d is kept at
//    (ng G + g) 128 + 16 a + 4 c + 2 b + d; the natural tensor is (G, N).
//  * low-rank factors (16-bit), 16 x 16 blocks [cp][rp]: inside a block the "n-like" index i = 8 ns + nl and the
//    "k-like" index j = 8 ks + 2 kl + e are kept at (((nl 4 + kl) 2 + ns) 2 + ks) 2 + e.  For the up factor (N, R) the
//    n-like index runs along N (cp blocks) and the k-like along R; for the down factor, kept as (K, R) on disk, the
//    n-like index runs along R (rp blocks) and the k-like along K (cp blocks).
#include "svdq_common.h"

namespace svdq {

__global__ __launch_bounds__(256) void unpack_mma_weight_kernel(const uint32_t *packed, uint8_t *natural, int N, int KW,
                                                                long ld_natural) {
    // one thread per natural word: (n, kw), kw = k / 8
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long)N * KW) return;
    const int n = (int)(idx / KW), kw = (int)(idx % KW);
    const int nt = n >> 7, np = (n >> 4) & 7, ns = (n >> 3) & 1, nl = n & 7;
    const int kt = kw >> 3, ks = (kw >> 2) & 1, kl = kw & 3;
    const long w = ((((((long)nt * (KW >> 3) + kt) * 8 + np) * 8 + nl) * 4 + kl) * 2 + ns) * 2 + ks;
    *(uint32_t *)(natural + (long)n * ld_natural + 4 * kw) = packed[w];
}

__global__ __launch_bounds__(256) void unpack_mma_scale_kernel(const uint16_t *packed, uint16_t *natural, int N, int G,
                                                               long ld_natural) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;  // natural (g, n)
    if (idx >= (long)G * N) return;
    const int g = (int)(idx / N), n = (int)(idx % N);
    const int ng = n >> 7, a = (n >> 4) & 7, b = (n >> 3) & 1, c = (n >> 1) & 3, d = n & 1;
    natural[(long)g * ld_natural + n] = packed[((long)ng * G + g) * 128 + 16 * a + 4 * c + 2 * b + d];
}

__global__ __launch_bounds__(256) void unpack_mma_lowrank_kernel(const uint16_t *packed, uint16_t *natural, int C, int R,
                                                                 int down, long ld_natural) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;  // natural (c, r)
    if (idx >= (long)C * R) return;
    const int c = (int)(idx / R), r = (int)(idx % R);
    const int i = down ? (r & 15) : (c & 15);  // n-like index inside the block
    const int j = down ? (c & 15) : (r & 15);  // k-like index inside the block
    const int ns = i >> 3, nl = i & 7, ks = j >> 3, kl = (j >> 1) & 3, e = j & 1;
    const long blk = (long)(c >> 4) * (R >> 4) + (r >> 4);
    natural[(long)c * ld_natural + r] = packed[blk * 256 + ((((nl * 4 + kl) * 2 + ns) * 2 + ks) * 2 + e)];
}

}  // namespace svdq

using namespace svdq;

extern "C" int svdq_unpack_mma_weight(const void *packed, void *natural, int32_t N, int32_t K, int32_t ld_natural,
                                      void *stream) {
    if (!packed || !natural || N <= 0 || K <= 0) {
        set_error("svdq_unpack_mma_weight: null tensor or empty shape N=%d K=%d", N, K);
        return SVDQ_E_INVALID;
    }
    if (N % 128 || K % 128) {
        set_error("svdq_unpack_mma_weight: N=%d and K=%d must be multiples of 128 (the checkpoint's padded tile)", N, K);
        return SVDQ_E_INVALID;
    }
    if (ld_natural < K / 2 || ld_natural % 4 || ((uintptr_t)packed & 3) || ((uintptr_t)natural & 3)) {
        set_error("svdq_unpack_mma_weight: rows of the natural tensor must hold K / 2 bytes and be 4-byte aligned");
        return SVDQ_E_INVALID;
    }
    const long words = (long)N * (K / 8);
    hipLaunchKernelGGL(unpack_mma_weight_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint32_t *)packed, (uint8_t *)natural, N, K / 8, (long)ld_natural);
    return check_launch("svdq_unpack_mma_weight");
}

extern "C" int svdq_unpack_mma_scale(const void *packed, void *natural, int32_t N, int32_t groups, int32_t ld_natural,
                                     void *stream) {
    if (!packed || !natural || N <= 0 || groups <= 0) {
        set_error("svdq_unpack_mma_scale: null tensor or empty shape N=%d groups=%d", N, groups);
        return SVDQ_E_INVALID;
    }
    if (N % 128 || ld_natural < N) {
        set_error("svdq_unpack_mma_scale: N=%d must be a multiple of 128 and fit the row stride %d", N, ld_natural);
        return SVDQ_E_INVALID;
    }
    const long n = (long)N * groups;
    hipLaunchKernelGGL(unpack_mma_scale_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t *)packed, (uint16_t *)natural, N, groups, (long)ld_natural);
    return check_launch("svdq_unpack_mma_scale");
}

extern "C" int svdq_unpack_mma_lowrank(const void *packed, void *natural, int32_t C, int32_t R, int32_t down,
                                       int32_t ld_natural, void *stream) {
    if (!packed || !natural || C <= 0 || R <= 0) {
        set_error("svdq_unpack_mma_lowrank: null tensor or empty shape C=%d R=%d", C, R);
        return SVDQ_E_INVALID;
    }
    if (C % 16 || R % 16 || ld_natural < R) {
        set_error("svdq_unpack_mma_lowrank: C=%d and R=%d must be multiples of 16 and fit the row stride %d", C, R, ld_natural);
        return SVDQ_E_INVALID;
    }
    const long n = (long)C * R;
    hipLaunchKernelGGL(unpack_mma_lowrank_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t *)packed, (uint16_t *)natural, C, R, down ? 1 : 0, (long)ld_natural);
    return check_launch("svdq_unpack_mma_lowrank");
}
