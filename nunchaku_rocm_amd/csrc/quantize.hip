// Activation quantizer for gfx950: smooth divide, per-group-64 absmax int4 quantization and the fused LoRA-down
// projection in one pass over the activations.
//
// Arithmetic follows the reference's _quantize_tile_kernel (nunchaku/ops/triton/gemm_w4a4.py:1397-1455): fp32
// throughout, reciprocal-then-multiply for the smooth factor and for the group scale (both IEEE divides), the stored
// scale rounded to the 16-bit type while the codes use the unrounded one, round-half-to-even through the 1.5*2^23
// add, clamp, low nibble first.  The LoRA-down product consumes the raw 16-bit activations (before shift and
// smoothing) on the 16x16x32 MFMA with fp32 accumulation.
//
// Work split: one workgroup = 16 rows x all of K, four wavefronts taking scale groups round-robin.  Lane
// (m = lane % 16, q = lane / 16) owns 16 consecutive channels [64 g + 16 q, +16) of row m, so a wavefront reads
// 16 rows x 128 contiguous bytes per group, a group's absmax needs two cross-lane steps, and the lane's two
// 16-byte halves are exactly the B operands of two MFMAs whose A operands come from the transposed LoRA-down
// weight (R, K).
#include "svdq_common.h"

// the codes and scales are a bit-exact contract: no multiply-add contraction anywhere in this file
#pragma clang fp contract(off)

namespace svdq {

constexpr int Q_ROWS = 16;
constexpr int Q_WAVES = 4;
constexpr int Q_RCHUNK = 32;  // LoRA ranks per pass over the row block

template <typename T, bool UNSIGNED, bool GLU>
__global__ __launch_bounds__(Q_WAVES * 64) void quantize_act_kernel(svdq_quantize_args a) {
    __shared__ float lds_rs[Q_WAVES][64];
    __shared__ float lds_acc[Q_WAVES][Q_RCHUNK][Q_ROWS + 1];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int ml = lane & 15;
    const int kq = lane >> 4;
    const int m0 = blockIdx.x * Q_ROWS;
    const int m = m0 + ml;
    const bool row_ok = m < a.M;
    const int ngroups = a.K / GROUP;
    const uint16_t *xrow = (const uint16_t *)a.x + (size_t)(row_ok ? m : 0) * a.ld_x;
    const uint16_t *smooth = (const uint16_t *)a.smooth;
    const uint16_t *ldt = (const uint16_t *)a.lora_down_t;
    const float qmax = UNSIGNED ? 15.0f : 7.0f;
    const float qlo = UNSIGNED ? 0.0f : -8.0f;
    const float qhi = UNSIGNED ? 15.0f : 7.0f;

    const int nchunks = a.R > 0 ? (a.R + Q_RCHUNK - 1) / Q_RCHUNK : 1;
    for (int rc = 0; rc < nchunks; rc++) {
        v4f acc[2];
        acc[0] = (v4f){0.f, 0.f, 0.f, 0.f};
        acc[1] = (v4f){0.f, 0.f, 0.f, 0.f};
        const int r0 = rc * Q_RCHUNK + ml;  // LoRA row of this lane's A operand (block 0), block 1 = +16
        const bool r_ok0 = r0 < a.R, r_ok1 = r0 + 16 < a.R;

        for (int g = wave; g < ngroups; g += Q_WAVES) {
            const int k0 = g * GROUP + kq * 16;
            v4i xlo = (v4i){0, 0, 0, 0}, xhi = (v4i){0, 0, 0, 0};
            if (row_ok) {
                xlo = *(const v4i *)(xrow + k0);
                xhi = *(const v4i *)(xrow + k0 + 8);
            }
            float v[16];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v[2 * j] = T::lo_f32((uint32_t)xlo[j]);
                v[2 * j + 1] = T::hi_f32((uint32_t)xlo[j]);
                v[8 + 2 * j] = T::lo_f32((uint32_t)xhi[j]);
                v[8 + 2 * j + 1] = T::hi_f32((uint32_t)xhi[j]);
            }
            if (GLU) {
                // x[:, k] * silu(x[:, K + k]); the LoRA-down then sees the product rounded to T
                v4i glo = (v4i){0, 0, 0, 0}, ghi = (v4i){0, 0, 0, 0};
                if (row_ok) {
                    glo = *(const v4i *)(xrow + a.K + k0);
                    ghi = *(const v4i *)(xrow + a.K + k0 + 8);
                }
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    float g0 = T::lo_f32((uint32_t)glo[j]), g1 = T::hi_f32((uint32_t)glo[j]);
                    float g2 = T::lo_f32((uint32_t)ghi[j]), g3 = T::hi_f32((uint32_t)ghi[j]);
                    v[2 * j] = v[2 * j] * (g0 / (1.0f + __expf(-g0)));
                    v[2 * j + 1] = v[2 * j + 1] * (g1 / (1.0f + __expf(-g1)));
                    v[8 + 2 * j] = v[8 + 2 * j] * (g2 / (1.0f + __expf(-g2)));
                    v[8 + 2 * j + 1] = v[8 + 2 * j + 1] * (g3 / (1.0f + __expf(-g3)));
                }
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    xlo[j] = (int)pack2<T>(v[2 * j], v[2 * j + 1]);
                    xhi[j] = (int)pack2<T>(v[8 + 2 * j], v[8 + 2 * j + 1]);
                }
            }

            if (a.R > 0) {
                v4i z = (v4i){0, 0, 0, 0};
                const uint16_t *lp = ldt + (size_t)r0 * a.K + k0;
                v4i a0lo = r_ok0 ? *(const v4i *)(lp) : z;
                v4i a0hi = r_ok0 ? *(const v4i *)(lp + 8) : z;
                v4i a1lo = r_ok1 ? *(const v4i *)(lp + (size_t)16 * a.K) : z;
                v4i a1hi = r_ok1 ? *(const v4i *)(lp + (size_t)16 * a.K + 8) : z;
                acc[0] = mfma16_16bit<T>(a0lo, xlo, acc[0]);
                acc[0] = mfma16_16bit<T>(a0hi, xhi, acc[0]);
                acc[1] = mfma16_16bit<T>(a1lo, xlo, acc[1]);
                acc[1] = mfma16_16bit<T>(a1hi, xhi, acc[1]);
            }

            if (rc == 0) {
                if (a.smooth != nullptr) {
                    // 1/smooth for the group's 64 channels: one IEEE divide per lane, shared through LDS
                    lds_rs[wave][lane] = 1.0f / T::to_f32(smooth[g * GROUP + lane]);
                    __builtin_amdgcn_wave_barrier();
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        v4f rs = *(const v4f *)&lds_rs[wave][kq * 16 + 4 * j];
#pragma unroll
                        for (int e = 0; e < 4; e++) v[4 * j + e] = (v[4 * j + e] + a.shift) * rs[e];
                    }
                    __builtin_amdgcn_wave_barrier();
                } else {
#pragma unroll
                    for (int j = 0; j < 16; j++) v[j] = v[j] + a.shift;
                }
                float gmax = 0.0f;
#pragma unroll
                for (int j = 0; j < 16; j++) gmax = fmaxf(gmax, UNSIGNED ? v[j] : fabsf(v[j]));
                gmax = fmaxf(gmax, __shfl_xor(gmax, 16));
                gmax = fmaxf(gmax, __shfl_xor(gmax, 32));
                const float scale = gmax / qmax;
                const float safe = (scale == 0.0f) ? 1.0f : scale;
                if (row_ok && kq == 0) ((uint16_t *)a.scales)[(size_t)g * a.ld_scales + m] = T::from_f32(scale);
                const float rq = 1.0f / safe;
                uint32_t w0 = 0, w1 = 0;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    // clamp, then the magic add leaves the two's-complement nibble in the low mantissa bits
                    float q0 = __builtin_amdgcn_fmed3f(v[j] * rq, qlo, qhi) + RNE_MAGIC;
                    float q1 = __builtin_amdgcn_fmed3f(v[8 + j] * rq, qlo, qhi) + RNE_MAGIC;
                    w0 |= (__float_as_uint(q0) & 0xFu) << (4 * j);
                    w1 |= (__float_as_uint(q1) & 0xFu) << (4 * j);
                }
                if (row_ok) {
                    uint2 pk = make_uint2(w0, w1);
                    *(uint2 *)((uint8_t *)a.out + (size_t)m * a.ld_out + g * (GROUP / 2) + kq * 8) = pk;
                }
            }
        }

        if (a.R > 0) {
            // fixed-order sum of the four wavefronts' partial products
#pragma unroll
            for (int i = 0; i < 4; i++) {
                lds_acc[wave][4 * kq + i][ml] = acc[0][i];
                lds_acc[wave][16 + 4 * kq + i][ml] = acc[1][i];
            }
            __syncthreads();
            for (int o = threadIdx.x; o < Q_ROWS * Q_RCHUNK; o += Q_WAVES * 64) {
                const int mm = o / Q_RCHUNK, r = o % Q_RCHUNK;
                float s = lds_acc[0][r][mm];
#pragma unroll
                for (int w = 1; w < Q_WAVES; w++) s += lds_acc[w][r][mm];
                if (m0 + mm < a.M && rc * Q_RCHUNK + r < a.R)
                    a.lora_act[(size_t)(m0 + mm) * a.ld_lora_act + rc * Q_RCHUNK + r] = s;
            }
            __syncthreads();
        }
    }
}

__global__ void transpose_kr_kernel(const uint16_t *in, uint16_t *out, int K, int R, int ld_in) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= K * R) return;
    const int r = idx / K, k = idx % K;
    out[idx] = in[(size_t)k * ld_in + r];
}

template <typename T>
static void launch_quantize(const svdq_quantize_args &a, hipStream_t s) {
    dim3 grid((a.M + Q_ROWS - 1) / Q_ROWS), block(Q_WAVES * 64);
    if (a.fuse_glu) {
        if (a.is_unsigned)
            hipLaunchKernelGGL((quantize_act_kernel<T, true, true>), grid, block, 0, s, a);
        else
            hipLaunchKernelGGL((quantize_act_kernel<T, false, true>), grid, block, 0, s, a);
    } else {
        if (a.is_unsigned)
            hipLaunchKernelGGL((quantize_act_kernel<T, true, false>), grid, block, 0, s, a);
        else
            hipLaunchKernelGGL((quantize_act_kernel<T, false, false>), grid, block, 0, s, a);
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
    if (a.ld_out % 8 || ((uintptr_t)a.out & 7)) {
        set_error("svdq_quantize_act: out rows must be 8-byte aligned (ld_out=%d)", a.ld_out);
        return SVDQ_E_INVALID;
    }
    if (a.ld_x < (a.fuse_glu ? 2 : 1) * a.K || a.ld_out < a.K / 2 || a.ld_scales < a.M ||
        (a.R > 0 && a.ld_lora_act < a.R)) {
        set_error("svdq_quantize_act: a leading dimension is smaller than its row");
        return SVDQ_E_INVALID;
    }
    if (a.dtype != SVDQ_BF16 && a.dtype != SVDQ_FP16) {
        set_error("svdq_quantize_act: dtype %d", a.dtype);
        return SVDQ_E_INVALID;
    }
    if (a.M == 0) return SVDQ_OK;
    if (a.dtype == SVDQ_BF16)
        launch_quantize<BF16>(a, (hipStream_t)stream);
    else
        launch_quantize<FP16>(a, (hipStream_t)stream);
    return check_launch("svdq_quantize_act");
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
