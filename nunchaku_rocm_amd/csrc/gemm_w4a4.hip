// W4A4 GEMM for gfx950 with per-group-64 scales on both operands, LoRA-up, bias and fused epilogues.
//
// Arithmetic contract (reference: nunchaku/ops/triton/gemm_w4a4.py:447-488, 156-209, 499-521, 730-778):
//   out[m, n] = sum_g as[g, m] * ws[g, n] * p_g[m, n]  +  T(lora_act[m, :]) . lora_up[n, :]  +  bias[n]
// with p_g the exact int32 dot product of the group's 64 int4 pairs.
//
// Two kernels share one epilogue.  In both, 256 threads = four wavefronts, each 32 activation rows x all 128 weight rows
// of a 128x128 tile.  The fp8 kernel passes the weight tile as the MFMA's first operand and the activation tile as its
// second, so a lane of the result owns one activation row m and its registers walk the block's weight rows: the
// orientation every row-wise epilogue wants; the int8 kernel has them the other way round (its scale FMAs want the weight
// scale per lane) and turns its results through LDS after the loop.  K is staged through LDS 128 at
// a time (two scale groups), two stages; operands that several wavefronts read go global -> LDS directly
// (buffer_load ... lds in the fp8 kernel, global_load_lds in the int8 kernel; no registers), one stage ahead, into a
// lane-linear layout (LDS slot l of a 1 KB block = the 16 bytes MFMA lane l needs), so the operand reads are bank-conflict
// free by construction; one raw s_barrier per stage with explicit s_waitcnt.
//
//  * gemm_w4a4_f8_kernel (pre-split weights, svdq_split_weight_planes; the default for module weights): an activation
//    is carried as the fp8 (e4m3) code of value * 2^-9, a weight as the fp6 (e2m3) code of value / 8, 24 bytes per lane
//    and group.  One v_mfma_scale_f32_32x32x64_f8f6f4 with block scales 2^9 and 2^3 gives the exact p_g of a whole
//    group as fp32; as[g, m] * ws[g, n] of the block comes from a 16-bit matrix instruction on the scales themselves
//    (exact: one non-zero product); one FMA per output and group is left for the VALU.  Signed activations become
//    sign | magnitude codes by one bit operation per plane: even k carry a + 8, odd k carry a - 7, so that the offset
//    term 8 * (sum of even weights) - 7 * (sum of odd weights) has no systematic part whatever the mean of the
//    weight codes; it is taken out again every four stages with a 16-bit matrix instruction on (as, -ws * offset),
//    whose operands travel with the weights.  Only the weights go through LDS (with their scales and offset terms);
//    a wavefront's own 32 activation rows and activation scales go to registers, one stage ahead.  The kernel is held
//    to 168 vector registers and 48.5 KB of LDS so that three workgroups share a CU (three wavefronts per SIMD): a
//    wavefront issues scale product, group product and the sixteen FMAs of a step in program order (single result
//    buffers) and the other two wavefronts of the SIMD fill the matrix pipe and the vector ALU meanwhile.
//    Fed by this library's own quantizer or requantizing epilogues (act_blocked = 2) the activations arrive as fp6 codes
//    sign | magnitude in the loop's lane order and go into the matrix instruction as loaded: fp6 x fp6 (half the matrix
//    time per group), no unpack, no offset, one instantiation for signed and unsigned activations; their scales can come
//    in the loop's order too (ascales_blocked: one 16-byte load per lane every four stages).
//  * gemm_w4a4_i8_kernel (packed weights): a 16-byte LDS read holds 32 nibbles; the even and the odd nibbles are split
//    into two int8 planes with shift/mask only (signed values land in the high nibble of each byte, i.e. times 16;
//    unsigned activations in the low nibble, times 1).  Both operands use the same split, so the K order inside a group
//    is a shared permutation and the dot product is unchanged; the power-of-two factor is folded exactly into the weight
//    scale.  p_g comes from two v_mfma_i32_32x32x32_i8 whose accumulator starts at the bit pattern of 1.5*2^23, so the
//    int32 result read as fp32 is (1.5*2^23 + p) exactly and  fma(bits, ws', -1.5*2^23*ws')  gives p*ws' with one
//    rounding and no int->float convert; a second fma applies as[g, m] and accumulates: two VALU ops per output and
//    group.  Needs no copy of the weight.
//
//  * The bias and the first 32 ranks of lora_up of the tile are fetched into LDS together with stage 0, in MFMA lane
//    order, so that the LoRA-up section does not wait for them.
//  * With "lane = activation row" (the fp8 kernel's native orientation; the int8 kernel turns its four 32x32 blocks
//    through a private LDS tile after LoRA-up and bias) row-wise epilogue work (RMSNorm sum of squares, RoPE pairs,
//    group absmax, nibble packing, the next layer's LoRA-down operand) is in-lane plus one exchange with lane ^ 32.
//  * The 16-bit output leaves through a wavefront-private, XOR-swizzled LDS tile as 256-byte row segments, stored
//    non-temporally.  Everything after the main loop is private to a wavefront: one barrier follows the loop, none
//    after it.
//  * Workgroup ids are first regrouped so that each XCD (ids are dealt round-robin over 8 XCDs) works on a
//    contiguous range of tiles, then swizzled in bands of m-tiles for L2 reuse of the weight tile.
#include <algorithm>
#include <atomic>
#include <type_traits>

#include "svdq_common.h"

namespace svdq {

constexpr int BM = 128, BN = 128;     // workgroup tile (activation rows x weight rows)
constexpr int KSTAGE = 128;           // K per LDS stage = two scale groups
constexpr int BLK_BYTES = 64 * 16;    // one MFMA operand block (32 rows x 16 bytes per lane) of one group, lane-linear
constexpr int NWAVES = 4, NTHREADS = NWAVES * 64;  // one wavefront per 32 activation rows
constexpr int NBN = BN / 32;                        // 32-row weight blocks per wavefront: it owns 32 x 128 outputs
// the first 32 ranks of the tile's lora_up, fetched next to stage 0: [2 c][4 blocks] 1 KB blocks in MFMA lane order,
// then the tile's 128 bias values, then the 128 RMSNorm weights of the tile's head (Q/K norm + RoPE epilogue)
constexpr int LORA_UP_BYTES = 8 * BLK_BYTES;
constexpr int EPI_NORM_OFF = LORA_UP_BYTES + BN * 2;
constexpr int EPI_LDS_BYTES = EPI_NORM_OFF + 128 * 2;
constexpr int TP_PITCH = 36;                        // floats per row of the accumulator transposition tile
constexpr int PRIV_BYTES = 32 * BN * 2;             // a wavefront's private epilogue memory: its 32 output rows of 256 bytes
static_assert(32 * TP_PITCH * 4 <= PRIV_BYTES, "the transposition tile of one block does not fit");
constexpr int GROUP_M_TILES = 8;      // m-tiles per raster band
constexpr int NUM_XCD = 8;

// ---- int8 kernel: stage layout: activation blocks [4 blocks of 32 rows][2 groups] packed (1 KB each), weight blocks
// [4 blocks][2 groups], then the scales
constexpr int I8_W_OFF = 4 * 2 * BLK_BYTES;                  // 8192
constexpr int I8_AS_OFF = I8_W_OFF + 4 * 2 * BLK_BYTES;      // 16384: float as[2][BM]
constexpr int I8_WS_OFF = I8_AS_OFF + 2 * BM * 4;            // 17408: float2 (ws', -magic * ws')[2][BN]
constexpr int I8_BUF_BYTES = I8_WS_OFF + 2 * BN * 8;         // 19456
static_assert(2 * PRIV_BYTES <= I8_BUF_BYTES, "two wavefronts' private epilogue memory must fit one staging buffer");

// ---- fp8 kernel
constexpr int F8_SCALE = (int)0x88888888;  // e8m0 block scale 2^9 in every byte: an fp8 code c (value c * 2^-9) counts as c
constexpr int F6_SCALE = (int)0x82828282;  // e8m0 block scale 2^3: an fp6 (e2m3) code c <= 15 (value c / 8) counts as c
// Pre-split weights, per (block of 32 rows, stage of two groups): three 1 KB blocks in MFMA lane order.  A lane's 32
// weights of a group are 32 six-bit codes = six registers: blocks 0 and 1 hold registers 0-3 of the stage's first and
// second group (16 bytes per lane), block 2 registers 4-5 of both (8 + 8 bytes per lane).
constexpr int WPL_BLOCKS = 3;
constexpr int F8_STAGE_BYTES = NBN * WPL_BLOCKS * BLK_BYTES;  // 12288
// ... and, per (block of 32 rows, stage), 32 rows of six 16-bit values: the two pieces (hi + lo) of
// D = -ws * (8 * sum of the group's even weights - 7 * sum of its odd weights) for the stage's two groups, then the two
// weight scales.  A 12-byte-per-lane global -> LDS load puts lane l's bytes at 16 l, so in LDS a row takes 16 bytes; they
// sit in a ring of eight stages per block; one load brings a stage and the one after it (64 lanes = two stages' rows)
// into an even slot and its neighbour.
constexpr int AUX_ROW = 12;                                  // bytes per row and stage in memory
constexpr int AUX_BLK = 32 * AUX_ROW;                        // 384
constexpr int AUX_LROW = 16;                                 // ... and in LDS
constexpr int AUX_LBLK = 32 * AUX_LROW;                      // 512
constexpr int AUX_SLOTS = 8;
constexpr int AUX_NBLK_BYTES = AUX_SLOTS * AUX_LBLK;         // 4096
constexpr int F8_RING_BYTES = NBN * AUX_NBLK_BYTES;          // 16384: after the loop two wavefronts' private memory
static_assert(2 * PRIV_BYTES <= F8_RING_BYTES, "two wavefronts' private epilogue memory must fit the ring");
static_assert(PRIV_BYTES <= F8_STAGE_BYTES, "a wavefront's private epilogue memory must fit a staging buffer");
constexpr int PLANES_STATUS_BYTES = 16;  // trailing status word of a pre-split weight

__host__ __device__ inline size_t planes_code_bytes(int N, int K) {
    return (size_t)((N + 31) / 32) * (size_t)((K / GROUP + 1) / 2) * (WPL_BLOCKS * BLK_BYTES);
}
__host__ __device__ inline size_t planes_aux_bytes(int N, int K) {  // one stage of padding per block of rows
    return (size_t)((N + 31) / 32) * (size_t)((K / GROUP + 1) / 2 + 1) * AUX_BLK;
}

__device__ inline void unpack_signed(v4i p, v4i &even, v4i &odd) {
    even = (p << 4) & (int)0xF0F0F0F0;  // 16 * value in each byte
    odd = p & (int)0xF0F0F0F0;
}
__device__ inline void unpack_unsigned(v4i p, v4i &even, v4i &odd) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    v4u u = __builtin_bit_cast(v4u, p);
    even = __builtin_bit_cast(v4i, u & 0x0F0F0F0Fu);
    odd = __builtin_bit_cast(v4i, (u >> 4) & 0x0F0F0F0Fu);
}

// fp6 (e2m3) code of a signed int4 value: sign bit | magnitude in the low four bits; a code c <= 15 stands for c / 8.
__device__ inline uint32_t f6_code(int v) { return (uint32_t)((v < 0 ? 0x20 : 0) | (v < 0 ? -v : v)); }
// The six registers of a lane's fp6 operand: 32 six-bit codes, code p in bits 6 p .. 6 p + 5.  The matrix instruction
// numbers K differently per format: an fp8 lane of half h holds K 16 h .. 16 h + 15 and 32 + 16 h .. 47 + 16 h (the even,
// then the odd nibbles of the lane's 16 packed activation bytes), an fp6 lane of half h holds K 32 h .. 32 h + 31.  So
// the weight lanes of half 0 carry the even nibbles of all 32 packed bytes of the row's group, those of half 1 the odd.
__device__ inline void f6_pack(const v4i lo16, const v4i hi16, int odd, uint32_t (&d)[6]) {
#pragma unroll
    for (int i = 0; i < 6; i++) d[i] = 0;
#pragma unroll
    for (int p = 0; p < 32; p++) {
        const int by = ((p < 16 ? lo16 : hi16)[(p & 15) >> 2] >> (8 * (p & 3))) & 0xFF;
        const uint32_t c = f6_code((((odd ? by >> 4 : by) & 0xF) ^ 8) - 8);
        const int bit = 6 * p;
        d[bit >> 5] |= c << (bit & 31);
        if ((bit & 31) > 26) d[(bit >> 5) + 1] |= c >> (32 - (bit & 31));
    }
}
// 8 * (sum of the even-k weights) - 7 * (sum of the odd-k weights) of one group (32 packed bytes): what the fp8 path's
// offset activation codes (a + 8 for even k, a - 7 for odd k) add to the group's dot product.
__device__ inline int group_offset_term(const v4i lo16, const v4i hi16) {
    int we = 0, wo = 0;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const v4i p = h ? hi16 : lo16;
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int j = 0; j < 8; j += 2) {
                we += (((p[e] >> (4 * j)) & 0xF) ^ 8) - 8;
                wo += (((p[e] >> (4 * j + 4)) & 0xF) ^ 8) - 8;
            }
    }
    return 8 * we - 7 * wo;
}

// Register loads of the fp8 loop go through raw buffers: address = descriptor base + scalar offset (the group or stage)
// + 32-bit lane offset, so no vector instruction computes an address.  The range covers everything (offsets are clamped
// where rows or columns run out).
__device__ inline __amdgpu_buffer_rsrc_t g_buffer(const void *base) {
    return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)0xFFFFFFFFu, 0x00020000);  // raw buffer, 32-bit data format
}
__device__ inline uint16_t g_load16(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t uniform_off) {
    return __builtin_amdgcn_raw_buffer_load_b16(r, (int)lane_off, (int)uniform_off, 0);
}
__device__ inline v4i g_load128(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t uniform_off) {
    return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(r, (int)lane_off, (int)uniform_off, 0));
}

__device__ inline v2i g_load64(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t uniform_off) {
    return __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(r, (int)lane_off, (int)uniform_off, 0));
}

// Block loads global -> LDS through a raw buffer: the 64 lanes' 16 (or 12) bytes at base + lane offset + scalar offset land at
// lds + 16 * lane; base and scalar offset live in SGPRs, so the loop's block loads need no vector address arithmetic.
__device__ inline void g_load16_lds(__amdgpu_buffer_rsrc_t r, uint8_t *lds, uint32_t lane_off, uint32_t uniform_off) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (SVDQ_AS3 void *)lds, 16, (int)lane_off, (int)uniform_off, 0, 0);
}
__device__ inline void g_load12_lds(__amdgpu_buffer_rsrc_t r, uint8_t *lds, uint32_t lane_off, uint32_t uniform_off) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (SVDQ_AS3 void *)lds, 12, (int)lane_off, (int)uniform_off, 0, 0);
}

__device__ inline v16i magic_acc() {
    v16i c;
#pragma unroll
    for (int i = 0; i < 16; i++) c[i] = RNE_MAGIC_BITS;
    return c;
}

// (pid_m, pid_n) of this workgroup: XCD-contiguous renumbering, then m-banded raster.
__device__ inline void tile_ids(int tiles_m, int tiles_n, int &pid_m, int &pid_n) {
    const int nb = gridDim.x;
    const int bid = blockIdx.x;
    const int xcd = bid % NUM_XCD, loc = bid / NUM_XCD;
    const int per = (nb + NUM_XCD - 1) / NUM_XCD, rem = nb % NUM_XCD;
    const int start = (rem == 0 || xcd < rem) ? xcd * per : rem * per + (xcd - rem) * (per - 1);
    const int id = start + loc;
    const int band = GROUP_M_TILES * tiles_n;
    const int first_m = (id / band) * GROUP_M_TILES;
    const int gm = min(tiles_m - first_m, GROUP_M_TILES);
    pid_m = first_m + (id % band) % gm;
    pid_n = (id % band) / gm;
}

// Epilogue operands every wavefront of the tile needs, fetched global -> LDS next to stage 0: the tile's 128 bias
// values, the first 32 ranks of lora_up and (Q/K norm + RoPE epilogue, Q and K tiles) the head's 128 norm weights.
template <int EPI>
__device__ inline void fetch_epilogue_operands(const svdq_gemm_args &a, uint8_t *sepi, int n0, int wm, int lane) {
    const int l32 = lane & 31, half = lane >> 5;
    if constexpr (EPI == SVDQ_EPI_QK_NORM_ROPE) {
        const int part = n0 / (a.N / 3);
        if (part < 2 && wm == 2) {  // 64 lanes x 4 bytes
            const uint8_t *src = (const uint8_t *)(part == 0 ? a.norm_q : a.norm_k) + 4 * lane;
            __builtin_amdgcn_global_load_lds((const SVDQ_AS1 void *)src, (SVDQ_AS3 void *)(sepi + EPI_NORM_OFF), 4, 0, 0);
        }
    }
    if (a.bias != nullptr && wm == 3) {  // 64 lanes x 4 bytes = the tile's 128 bias values
        const uint8_t *src = (const uint8_t *)a.bias + (size_t)min(n0 + 2 * lane, a.N - 2) * 2;
        __builtin_amdgcn_global_load_lds((const SVDQ_AS1 void *)src, (SVDQ_AS3 void *)(sepi + LORA_UP_BYTES), 4, 0, 0);
    }
    if (a.R > 0) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int q = wm * 2 + i, c = q >> 2, blk = q & 3;  // wave-uniform
            const uint8_t *src = (const uint8_t *)a.lora_up + ((size_t)min(n0 + blk * 32 + l32, a.N - 1) * a.ld_lora_up + 16 * c + 8 * half) * 2;
            if (16 * c < a.R)
                __builtin_amdgcn_global_load_lds((const SVDQ_AS1 void *)src, (SVDQ_AS3 void *)(sepi + q * BLK_BYTES), 16, 0, 0);
        }
    }
}

// Requantized activations as fp6 codes in the consuming GEMM's lane order (qout_blocked == 2).  A lane of the epilogue
// owns, of its row's group of 64 values, the runs k = 8 t + 4 half .. + 3 (t = 0 .. 7): codes p = 4 t + 2 half, + 1 of the
// consuming lane of K half 0 (its even k) and the same codes of the lane of K half 1 (its odd k), i.e. one 12-bit piece
// per t and consuming lane, at bit 24 t + 12 half of that lane's 192.  f6_pack_unit places four pieces (96 bits);
// f6_swap_unit trades the two half-filled units with lane ^ 32 (all lanes of the wavefront must be active) -- every lane
// ends up with all of one consuming lane's 24 bytes -- and f6_store writes their first 16 at 16 l and their last 8 at
// 1024 + 8 l of the (row block, group)'s 1536, l = 32 half + row % 32.
__device__ inline void f6_pack_unit(uint32_t p0, uint32_t p1, uint32_t p2, uint32_t p3, uint32_t sh, uint32_t (&d)[3]) {
    const uint64_t lo = ((uint64_t)p0 | ((uint64_t)p1 << 24)) << sh, hi = ((uint64_t)p2 | ((uint64_t)p3 << 24)) << sh;
    d[0] = (uint32_t)lo;
    d[1] = (uint32_t)(lo >> 32) | ((uint32_t)hi << 16);
    d[2] = (uint32_t)(hi >> 16);
}
__device__ inline void f6_swap_unit(const uint32_t (&v0)[3], const uint32_t (&v1)[3], uint32_t *r) {
#pragma unroll
    for (int i = 0; i < 3; i++) {
        const auto sw = __builtin_amdgcn_permlane32_swap(v0[i], v1[i], false, false);
        r[i] = sw[0] | sw[1];
    }
}
__device__ inline void f6_store(const uint32_t (&r)[6], uint8_t *blk, int lane, bool ok) {
    if (ok) {
        *(v4i *)(blk + 16 * lane) = (v4i){(int)r[0], (int)r[1], (int)r[2], (int)r[3]};
        *(v2i *)(blk + 1024 + 8 * lane) = (v2i){(int)r[4], (int)r[5]};
    }
}

// Everything after the main loop, for one wavefront: acc[bn][i] holds out[m = mw0 + 8 (i >> 2) + 4 half + (i & 3)]
// [n = n0 + 32 bn + lane % 32] without LoRA-up and bias -- or, with ROWS_IN_LANES (a main loop that passes the weights as
// the matrix instruction's first operand), out[m = mw0 + lane % 32][n = n0 + 32 bn + 8 (i >> 2) + 4 half + (i & 3)],
// which is the orientation every row-wise epilogue wants: the turn through LDS below is then not needed.  `priv` is PRIV_BYTES of LDS nobody else touches from here on;
// `sepi` holds what fetch_epilogue_operands brought.  No workgroup barrier inside.
template <typename T, int EPI, bool ROWS_IN_LANES = false>
__device__ __forceinline__ void tile_epilogue(const svdq_gemm_args &a, v16f (&acc)[NBN], uint8_t *priv, const uint8_t *sepi,
                                              int m0, int n0, int pid_n, int wm, int lane) {
    const int l32 = lane & 31, half = lane >> 5;
    const int mw0 = m0 + wm * 32;

    // Q/K RMSNorm + RoPE: the lane's rotary entries of a 32-column block are fetched two blocks ahead of their use, the
    // first two blocks' before the transposition (issued one load at a time next to the arithmetic, as the compiler orders
    // them under this register pressure, the sixteen dependent L2 round trips took 6 % of the launch); the head's norm
    // weights came into LDS next to stage 0.
    const int qk_part = EPI == SVDQ_EPI_QK_NORM_ROPE ? n0 / (a.N / 3) : 2;  // 0 = Q, 1 = K, 2 = V or no such epilogue
    v4f qk_sc[2][4];
    auto qk_fetch = [&](int bn, int buf) {
        if (a.rotary_blocked != nullptr) {
            // re-laid-out table: the 64 lanes of a load read 1 KB in a row.  (From the (rows, 128) table a load fetches
            // 32-byte pieces of 32 different rows; at the QKV shape that was 8 of the epilogue's 11 us.)
            const int rb = min(mw0 >> 5, (a.actual_m + 31) / 32 - 1);
            const v4f *p = (const v4f *)a.rotary_blocked + ((size_t)rb * 16 + bn * 4) * 64 + lane;
#pragma unroll
            for (int j = 0; j < 4; j++) qk_sc[buf][j] = p[j * 64];
            return;
        }
        const int m = mw0 + l32;
        const float *rot = a.rotary + (size_t)(m < a.actual_m ? m : 0) * a.ld_rotary;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int d = bn * 32 + 8 * j + 4 * half;  // channel within the head
            qk_sc[buf][j] = *(const v4f *)(rot + d);  // (sin, cos, sin, cos)
        }
    };


    // ---- LoRA-up and bias, still in the main loop's orientation (lane = weight row, registers = activation rows) ----
    // The bias and the first 32 ranks of lora_up were fetched into LDS next to stage 0 and arrived long ago; the
    // wavefront's own rows of lora_act and ranks beyond 32 come from global memory, all loads of a 32-rank pass issued
    // before their first use.  Rows past N / M hold copies of the last row: they only reach outputs that are never stored.
    if (a.R > 0) {
        const uint16_t *lu = (const uint16_t *)a.lora_up;
        const float *la = a.lora_act + (size_t)min(mw0 + l32, a.M - 1) * a.ld_lora_act + half * 8;
        for (int r0 = 0; r0 < a.R; r0 += 32) {
            const bool two = r0 + 16 < a.R;  // uniform: the second 16 ranks of this pass exist
            v4i ua[2][NBN];
            v4f uf[2][2];
#pragma unroll
            for (int c = 0; c < 2; c++) {
                if (c == 1 && !two) break;
                uf[c][0] = *(const v4f *)(la + r0 + 16 * c);
                uf[c][1] = *(const v4f *)(la + r0 + 16 * c + 4);
#pragma unroll
                for (int blk = 0; blk < NBN; blk++) {
                    if (r0 == 0)
                        ua[c][blk] = *(const v4i *)(sepi + (c * 4 + blk) * BLK_BYTES + lane * 16);
                    else
                        ua[c][blk] = *(const v4i *)(lu + (size_t)min(n0 + blk * 32 + l32, a.N - 1) * a.ld_lora_up + r0 + 16 * c + half * 8);
                }
            }
#pragma unroll
            for (int c = 0; c < 2; c++) {
                if (c == 1 && !two) break;
                const v4f f0 = uf[c][0], f1 = uf[c][1];
                v4i ub;
                ub[0] = (int)pack2<T>(f0[0], f0[1]);
                ub[1] = (int)pack2<T>(f0[2], f0[3]);
                ub[2] = (int)pack2<T>(f1[0], f1[1]);
                ub[3] = (int)pack2<T>(f1[2], f1[3]);
#pragma unroll
                for (int bn = 0; bn < NBN; bn++)
                    acc[bn] = ROWS_IN_LANES ? mfma32_16bit<T>(ua[c][bn], ub, acc[bn]) : mfma32_16bit<T>(ub, ua[c][bn], acc[bn]);
            }
        }
    }
    if (a.bias != nullptr) {
#pragma unroll
        for (int bn = 0; bn < NBN; bn++) {
            if constexpr (ROWS_IN_LANES) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint2 b4 = *(const uint2 *)(sepi + LORA_UP_BYTES + (bn * 32 + 8 * j + 4 * half) * 2);
                    acc[bn][4 * j + 0] += T::lo_f32(b4.x);
                    acc[bn][4 * j + 1] += T::hi_f32(b4.x);
                    acc[bn][4 * j + 2] += T::lo_f32(b4.y);
                    acc[bn][4 * j + 3] += T::hi_f32(b4.y);
                }
            } else {
                const float b = T::to_f32(*(const uint16_t *)(sepi + LORA_UP_BYTES + (bn * 32 + l32) * 2));
#pragma unroll
                for (int i = 0; i < 16; i++) acc[bn][i] += b;
            }
        }
    }

    if constexpr (EPI == SVDQ_EPI_QK_NORM_ROPE) {
        if (qk_part < 2) {  // measured: issued ahead of LoRA-up as well, the launch takes 0.6 % longer
            qk_fetch(0, 0);
            qk_fetch(1, 1);
        }
    }

    // ---- transposition: lane = weight row -> lane = activation row ---------------------------------------------
    // One 32x32 block at a time through the private tile (the LDS operations of one wavefront complete in order).
    // Afterwards lane (m = lane % 32, half) holds columns 32 bn + 8 j + 4 half + e of row m in acc[bn][4 j + e]: row-wise
    // epilogue work is in-lane plus one exchange with lane ^ 32, and no epilogue needs another wavefront's data.
    if constexpr (!ROWS_IN_LANES) {
        float *tp = (float *)priv;
#pragma unroll
        for (int bn = 0; bn < NBN; bn++) {
#pragma unroll
            for (int i = 0; i < 16; i++) tp[(8 * (i >> 2) + 4 * half + (i & 3)) * TP_PITCH + l32] = acc[bn][i];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v4f v = *(const v4f *)(tp + l32 * TP_PITCH + 8 * j + 4 * half);
                acc[bn][4 * j + 0] = v[0];
                acc[bn][4 * j + 1] = v[1];
                acc[bn][4 * j + 2] = v[2];
                acc[bn][4 * j + 3] = v[3];
            }
        }
    }

    // Output rows go out through LDS: in registers a lane holds 4 consecutive columns of one row, which stored directly
    // is an 8-byte piece per row and lane; staged as the wavefront's [32 rows][256 bytes] tile, each store instruction
    // writes four contiguous 256-byte row segments instead.  16-byte chunk c of row r sits at chunk c ^ (r & 15), its two
    // 8-byte halves swapped for rows 16-31: writes and reads are free of bank conflicts.
    auto store_out = [&]() {
#pragma unroll
        for (int bn = 0; bn < NBN; bn++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                uint2 v;
                v.x = pack2<T>(acc[bn][4 * j], acc[bn][4 * j + 1]);
                v.y = pack2<T>(acc[bn][4 * j + 2], acc[bn][4 * j + 3]);
                *(uint2 *)(priv + l32 * (BN * 2) + (((4 * bn + j) ^ (l32 & 15)) << 4) + 8 * (half ^ (l32 >> 4))) = v;
            }
        uint16_t *out = (uint16_t *)a.out;
        const int c = lane & 15, n = n0 + c * 8;
#pragma unroll
        for (int pass = 0; pass < 8; pass++) {
            const int r = 4 * pass + (lane >> 4), m = mw0 + r;  // rows 16-31 are passes 4-7
            v4i q = *(const v4i *)(priv + r * (BN * 2) + ((c ^ (r & 15)) << 4));
            if (pass >= 4) q = (v4i){q[2], q[3], q[0], q[1]};
            if (m < a.actual_m && n < a.N)
                // streamed: the 85 MB of a QKV output do not fit any cache level of the CU, and lines left dirty in L2 have
                // to be written back before the next kernel on the stream starts (measured: 1 % of the launch)
                __builtin_nontemporal_store(q, (v4i *)(out + (size_t)m * a.ld_out + n));
        }
    };

    if (EPI == SVDQ_EPI_PLAIN) {
        store_out();
        return;
    }

    if (EPI == SVDQ_EPI_QK_NORM_ROPE) {
        // the 128-wide tile is one head, all of it in this wavefront; part 0 = Q, 1 = K, 2 = V (untouched)
        if (qk_part < 2) {
            float ss = 0.0f;
#pragma unroll
            for (int bn = 0; bn < NBN; bn++)
#pragma unroll
                for (int i = 0; i < 16; i++) ss += acc[bn][i] * acc[bn][i];
            ss += __shfl_xor(ss, 32);
            const float rstd = 1.0f / sqrtf(ss / 128.0f + a.eps);
#pragma unroll
            for (int bn = 0; bn < NBN; bn++) {
                const int buf = bn & 1;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint2 wb = *(const uint2 *)(sepi + EPI_NORM_OFF + (bn * 32 + 8 * j + 4 * half) * 2);
                    const v4f sc = qk_sc[buf][j];
                    const float x0 = acc[bn][4 * j + 0] * rstd * T::lo_f32(wb.x);
                    const float x1 = acc[bn][4 * j + 1] * rstd * T::hi_f32(wb.x);
                    const float x2 = acc[bn][4 * j + 2] * rstd * T::lo_f32(wb.y);
                    const float x3 = acc[bn][4 * j + 3] * rstd * T::hi_f32(wb.y);
                    acc[bn][4 * j + 0] = x0 * sc[1] - x1 * sc[0];
                    acc[bn][4 * j + 1] = x0 * sc[0] + x1 * sc[1];
                    acc[bn][4 * j + 2] = x2 * sc[3] - x3 * sc[2];
                    acc[bn][4 * j + 3] = x2 * sc[2] + x3 * sc[3];
                }
                if (bn + 2 < NBN) qk_fetch(bn + 2, buf);  // behind the block's last use of this buffer
            }
        }
        store_out();
        return;
    }

    if (EPI == SVDQ_EPI_GELU_QUANT) {
        const uint16_t *ldt = (const uint16_t *)a.lora_down_t;
        // needed further down, issued before the GELU arithmetic: the next layer's smoothing factors of columns lane and
        // 64 + lane
        uint16_t smv[2] = {0, 0};
        const bool has_sm = a.smooth_next != nullptr;
        if (has_sm) {
#pragma unroll
            for (int t = 0; t < 2; t++) smv[t] = ((const uint16_t *)a.smooth_next)[min(n0 + 64 * t + lane, a.N - 1)];
        }
        if (a.out != nullptr) store_out();  // pre-GELU output, when asked for
#pragma unroll
        for (int bn = 0; bn < NBN; bn++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[bn][i] = gelu_tanh(acc[bn][i]);

        // next layer's LoRA-down on the un-shifted, un-smoothed GELU output rounded to T:
        // D[r][m] = sum_n ldT[r][n] * x[n][m] over the tile's 128 columns; registers [8 s, 8 s + 8) of a block are one
        // MFMA's B operand.  One partial per n-tile, summed in tile order by lora_part_reduce_kernel.
        for (int rc = 0; rc < a.R2; rc += 32) {
            v16f d;
#pragma unroll
            for (int i = 0; i < 16; i++) d[i] = 0.0f;
            const int r = rc + l32;
#pragma unroll
            for (int bn = 0; bn < NBN; bn++) {
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    // (fetched ahead of the GELU arithmetic, all at once or two column blocks ahead, these loads spill
                    // registers and the launch is no faster: the other workgroups of the CU cover their latency)
                    v4i la = (v4i){0, 0, 0, 0};
                    if (a.lora_down_blocked != nullptr) {
                        // re-laid-out copy: the operand of this instruction is 1 KB in lane order (from the (R2, N) copy a
                        // lane fetches two 8-byte pieces of its rank's row, 32 rows to a load instruction)
                        la = ((const v4i *)a.lora_down_blocked)[(((size_t)pid_n * ((a.R2 + 31) / 32) + rc / 32) * 8 + bn * 2 + s) * 64 + lane];
                    } else if (r < a.R2) {
                        const uint16_t *lp = ldt + (size_t)r * a.N + n0 + bn * 32 + 16 * s + 4 * half;
                        const uint2 q0 = *(const uint2 *)lp, q1 = *(const uint2 *)(lp + 8);
                        la = (v4i){(int)q0.x, (int)q0.y, (int)q1.x, (int)q1.y};
                    }
                    v4i xb;
#pragma unroll
                    for (int e = 0; e < 4; e++) xb[e] = (int)pack2<T>(acc[bn][8 * s + 2 * e], acc[bn][8 * s + 2 * e + 1]);
                    d = mfma32_16bit<T>(la, xb, d);
                }
            }
            const int m = mw0 + l32;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int rr = rc + 8 * j + 4 * half;
                if (m < a.M && rr < a.R2)
                    *(v4f *)(a.scratch + ((size_t)pid_n * a.M + m) * a.R2 + rr) = (v4f){d[4 * j], d[4 * j + 1], d[4 * j + 2], d[4 * j + 3]};
            }
        }

        // +shift, * 1/smooth, unsigned per-64 quantization: the wavefront's 128 columns are two groups
        float *lds_rs = (float *)priv;  // [BN], this wavefront's own copy
#pragma unroll
        for (int t = 0; t < 2; t++) lds_rs[64 * t + lane] = has_sm ? 1.0f / T::to_f32(smv[t]) : 1.0f;
        const int m = mw0 + l32;
#pragma unroll
        for (int gi = 0; gi < 2; gi++) {
            const int g = (n0 + 64 * gi) / GROUP;
            float gmax = 0.0f;
#pragma unroll
            for (int b2 = 0; b2 < 2; b2++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int bn = 2 * gi + b2;
                    const v4f rs = *(const v4f *)(lds_rs + bn * 32 + 8 * j + 4 * half);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float v = (acc[bn][4 * j + e] + a.shift) * rs[e];
                        acc[bn][4 * j + e] = v;
                        gmax = fmaxf(gmax, v);
                    }
                }
            gmax = max_with_lane_xor32(gmax);
            const float scale = gmax / 15.0f;
            const float safe = (scale == 0.0f) ? 1.0f : scale;
            const float rq = 1.0f / safe;
            if (half == 0 && m < a.M && n0 + 64 * gi < a.N)  // (oscales_blocked: the consuming GEMM's ascales_blocked layout)
                ((uint16_t *)a.oscales)[a.oscales_blocked ? ((size_t)(m >> 5) * (a.N / (8 * GROUP)) + (g >> 3)) * 256 + (m & 31) * 8 + (g & 7)
                                                          : (size_t)g * a.ld_oscales + m] = T::from_f32(scale);
            if (a.qout_blocked == 2) {
                uint32_t vec[6];
#pragma unroll
                for (int b2 = 0; b2 < 2; b2++) {
                    const int bn = 2 * gi + b2;
                    uint32_t pc[2][4];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        uint32_t c[4];
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            c[e] = __float_as_uint(__builtin_amdgcn_fmed3f(acc[bn][4 * j + e] * rq, 0.0f, 15.0f) + RNE_MAGIC) & 0xFu;
                        pc[0][j] = c[0] | (c[2] << 6);
                        pc[1][j] = c[1] | (c[3] << 6);
                    }
                    uint32_t d0[3], d1[3];
                    f6_pack_unit(pc[0][0], pc[0][1], pc[0][2], pc[0][3], 12u * half, d0);
                    f6_pack_unit(pc[1][0], pc[1][1], pc[1][2], pc[1][3], 12u * half, d1);
                    f6_swap_unit(d0, d1, vec + 3 * b2);
                }
                f6_store(vec, (uint8_t *)a.qout + ((size_t)(m >> 5) * (a.N / GROUP) + g) * 1536, 32 * half + (m & 31), m < a.M);
                continue;
            }
#pragma unroll
            for (int b2 = 0; b2 < 2; b2++) {
                const int bn = 2 * gi + b2;
                uint32_t mine[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    uint32_t w = 0;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float q = __builtin_amdgcn_fmed3f(acc[bn][4 * j + e] * rq, 0.0f, 15.0f) + RNE_MAGIC;
                        w |= (__float_as_uint(q) & 0xFu) << (4 * e);
                    }
                    mine[j] = w;  // 16 bits: columns 8 j + 4 half + 0..3
                }
                // lane and lane ^ 32 hold alternating 16-bit pieces of one 16-byte run (dword j = piece of half 0 in
                // the low 16 bits, piece of half 1 in the high 16 bits); trade so half 0 stores dwords 0-1 and half 1
                // stores dwords 2-3
                uint32_t dw[2];
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const uint32_t keep = half ? mine[2 + t] : mine[t];
                    const uint32_t send = half ? mine[t] : mine[2 + t];
                    const uint32_t theirs = __shfl_xor(send, 32);
                    dw[t] = half ? (theirs | (keep << 16)) : (keep | (theirs << 16));
                }
                if (m < a.M) {
                    // (qout_blocked: where lane (m % 32, bn % 2) of the consuming GEMM's row block and group reads its 16 bytes)
                    uint8_t *dst = a.qout_blocked
                                       ? (uint8_t *)a.qout + ((size_t)(m >> 5) * (a.N / GROUP) + g) * 1024 + (((bn & 1) * 32 + (m & 31)) * 16 + 8 * half)
                                       : (uint8_t *)a.qout + (size_t)m * a.ld_qout + (n0 + bn * 32) / 2 + 8 * half;
                    *(uint2 *)dst = make_uint2(dw[0], dw[1]);
                }
            }
        }
        return;
    }

    if (EPI == SVDQ_EPI_SWIGLU_QUANT) {
        // Output columns come in 16-blocks [gate | up]: registers j = 0, 1 of a 32-column block are gate values and
        // j = 2, 3 the matching up values, so y = silu(gate) * up is formed in-lane.  The tile's 128 columns give 64
        // y columns = one quantization group, all of it in this wavefront.
        const int H = a.N / 2;
        const uint16_t *ldt = (const uint16_t *)a.lora_down_t;
        const int yt0 = n0 / 2;  // first y column of the tile
        uint16_t smv = 0;
        const bool has_sm = a.smooth_next != nullptr;
        if (has_sm) smv = ((const uint16_t *)a.smooth_next)[min(yt0 + lane, H - 1)];
        float y[NBN][8];  // [bn][4 j + e]: y column 16 bn + 8 j + 4 half + e of the tile's 64
#pragma unroll
        for (int bn = 0; bn < NBN; bn++)
#pragma unroll
            for (int i = 0; i < 8; i++) y[bn][i] = silu(acc[bn][i]) * acc[bn][8 + i];
        const int m = mw0 + l32;
        for (int rc = 0; rc < a.R2; rc += 32) {
            v16f d;
#pragma unroll
            for (int i = 0; i < 16; i++) d[i] = 0.0f;
            const int r = rc + l32;
#pragma unroll
            for (int s = 0; s < NBN; s++) {
                v4i la = (v4i){0, 0, 0, 0};
                if (r < a.R2) {
                    const uint16_t *lp = ldt + (size_t)r * H + yt0 + 16 * s + 4 * half;
                    const uint2 q0 = *(const uint2 *)lp, q1 = *(const uint2 *)(lp + 8);
                    la = (v4i){(int)q0.x, (int)q0.y, (int)q1.x, (int)q1.y};
                }
                v4i xb;
#pragma unroll
                for (int e = 0; e < 4; e++) xb[e] = (int)pack2<T>(y[s][2 * e], y[s][2 * e + 1]);
                d = mfma32_16bit<T>(la, xb, d);
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int rr = rc + 8 * j + 4 * half;
                if (m < a.M && rr < a.R2)
                    *(v4f *)(a.scratch + ((size_t)pid_n * a.M + m) * a.R2 + rr) = (v4f){d[4 * j], d[4 * j + 1], d[4 * j + 2], d[4 * j + 3]};
            }
        }

        // * 1/smooth, signed per-64 quantization over the tile's 64 y columns
        float *lds_rs = (float *)priv;  // [64], this wavefront's own copy
        lds_rs[lane] = has_sm ? 1.0f / T::to_f32(smv) : 1.0f;
        float gmax = 0.0f;
#pragma unroll
        for (int bn = 0; bn < NBN; bn++)
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const v4f rs = *(const v4f *)(lds_rs + 16 * bn + 8 * j + 4 * half);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float v = (y[bn][4 * j + e] + a.shift) * rs[e];
                    y[bn][4 * j + e] = v;
                    gmax = fmaxf(gmax, fabsf(v));
                }
            }
        gmax = max_with_lane_xor32(gmax);
        const float scale = gmax / 7.0f;
        const float safe = (scale == 0.0f) ? 1.0f : scale;
        const float rq = 1.0f / safe;
        if (half == 0 && m < a.M) {
            const int g = yt0 / GROUP;
            ((uint16_t *)a.oscales)[a.oscales_blocked ? ((size_t)(m >> 5) * (H / (8 * GROUP)) + (g >> 3)) * 256 + (m & 31) * 8 + (g & 7)
                                                      : (size_t)g * a.ld_oscales + m] = T::from_f32(scale);
        }
        if (a.qout_blocked == 2) {
            // sign | magnitude: the magnitude rounds as the value does; the magic constant gets 32 more for a negative one
            uint32_t vec[6];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                uint32_t pc[2][4];
#pragma unroll
                for (int t = 0; t < 4; t++) {  // piece 4 u + t: block bn = 2 u + t / 2, register run j = t % 2
                    uint32_t c[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float q = __builtin_amdgcn_fmed3f(y[2 * u + (t >> 1)][4 * (t & 1) + e] * rq, -8.0f, 7.0f);
                        const uint32_t mg = ((uint32_t)((int)__float_as_uint(q) >> 31) & 32u) | (uint32_t)RNE_MAGIC_BITS;
                        c[e] = __float_as_uint(__builtin_fabsf(q) + __uint_as_float(mg)) & 0x3Fu;
                    }
                    pc[0][t] = c[0] | (c[2] << 6);
                    pc[1][t] = c[1] | (c[3] << 6);
                }
                uint32_t d0[3], d1[3];
                f6_pack_unit(pc[0][0], pc[0][1], pc[0][2], pc[0][3], 12u * half, d0);
                f6_pack_unit(pc[1][0], pc[1][1], pc[1][2], pc[1][3], 12u * half, d1);
                f6_swap_unit(d0, d1, vec + 3 * u);
            }
            f6_store(vec, (uint8_t *)a.qout + ((size_t)(m >> 5) * (H / GROUP) + yt0 / GROUP) * 1536, 32 * half + (m & 31), m < a.M);
            return;
        }
#pragma unroll
        for (int bn = 0; bn < NBN; bn++) {
            uint32_t mine[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                uint32_t w = 0;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float q = __builtin_amdgcn_fmed3f(y[bn][4 * j + e] * rq, -8.0f, 7.0f) + RNE_MAGIC;
                    w |= (__float_as_uint(q) & 0xFu) << (4 * e);
                }
                mine[j] = w;  // 16 bits: y columns 16 bn + 8 j + 4 half + 0..3
            }
            // dword j of the block's 8-byte run = piece of half 0 (low 16 bits) | piece of half 1 (high 16 bits);
            // half h keeps dword h
            const uint32_t keep = half ? mine[1] : mine[0];
            const uint32_t send = half ? mine[0] : mine[1];
            const uint32_t theirs = __shfl_xor(send, 32);
            const uint32_t dw = half ? (theirs | (keep << 16)) : (keep | (theirs << 16));
            if (m < a.M) {
                // (qout_blocked: the tile's 64 y columns are one group of the consuming GEMM; byte 8 bn + 4 half of its 32)
                uint8_t *dst = a.qout_blocked
                                   ? (uint8_t *)a.qout + ((size_t)(m >> 5) * (H / GROUP) + yt0 / GROUP) * 1024 + (((bn >> 1) * 32 + (m & 31)) * 16 + 8 * (bn & 1) + 4 * half)
                                   : (uint8_t *)a.qout + (size_t)m * a.ld_qout + (yt0 + 16 * bn) / 2 + 4 * half;
                *(uint32_t *)dst = dw;
            }
        }
        return;
    }
}

// ---- packed weights: int8 main loop -------------------------------------------------------------------------------------
template <typename T, bool ACT_UNSIGNED, int EPI, bool ODDG>  // ODDG: K / 64 is odd
__global__ __launch_bounds__(NTHREADS, 2) void gemm_w4a4_i8_kernel(svdq_gemm_args a) {
    // Three separate LDS objects: the compiler then knows that a block load into one staging buffer cannot touch what
    // is being read from the other (one object would make every LDS read wait for the loads in flight).
    __shared__ __align__(16) uint8_t sbuf0[I8_BUF_BYTES];
    __shared__ __align__(16) uint8_t sbuf1[I8_BUF_BYTES];
    __shared__ __align__(16) uint8_t sepi[EPI_LDS_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wm = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: the wavefront's 32-row block of the tile
    const int l32 = lane & 31, half = lane >> 5;

    int pid_m, pid_n;
    tile_ids((a.M + BM - 1) / BM, (a.N + BN - 1) / BN, pid_m, pid_n);
    const int m0 = pid_m * BM, n0 = pid_n * BN;

    // ---- operand staging: global -> LDS directly (global_load_lds_dwordx4), one stage ahead ----------------------
    // A stage holds 1 KB operand blocks (operand, 32-row block, group).  Lane l of a block load fetches the 16 bytes MFMA
    // lane l will read and the hardware writes them to LDS slot l of the block: lane l = (row l % 32, half l / 32) of a
    // row-major tile.  The 8 activation + 8 weight block loads of a stage are dealt in runs to the four wavefronts.
    constexpr int NLOADS = 16, PER_WAVE = NLOADS / NWAVES, NABLK = 8;
    // each load's address = wave-uniform base (SGPRs) + a 32-bit offset (lane part + stage * step; operands < 4 GiB)
    const uint8_t *gbase[PER_WAVE];
    uint32_t goff[PER_WAVE];
    int ldst[PER_WAVE];
    uint32_t gcap[PER_WAVE];
    const int G = a.K / GROUP;
    // K / 64 odd: the last stage has one group only.  The loads of its second group stop one stage earlier (they re-read
    // valid memory) and its scales are staged as zero, so it adds nothing.  A load's stage offset is min(s * step, cap).
    auto cap_of = [&](int gg, const uint8_t *&base) -> uint32_t {
        if (gg == 0) return (uint32_t)(G / 2) * (uint32_t)(KSTAGE / 2);  // G is odd: stages 0 .. G / 2
        if (G == 1) {  // no earlier stage: read the first group's bytes instead
            base -= 32;
            return 0u;
        }
        return (uint32_t)(G / 2 - 1) * (uint32_t)(KSTAGE / 2);
    };
#pragma unroll
    for (int i = 0; i < PER_WAVE; i++) {
        const int q = wm * PER_WAVE + i;  // wave-uniform
        if (q < NABLK) {                  // activation block q: (blk = q / 2, group q % 2)
            const int blk = q >> 1, gg = q & 1;
            gbase[i] = (const uint8_t *)a.act + (size_t)m0 * a.ld_act + gg * 32;
            goff[i] = (uint32_t)(min(m0 + blk * 32 + l32, a.M - 1) - m0) * (uint32_t)a.ld_act + half * 16;
            ldst[i] = (blk * 2 + gg) * BLK_BYTES;
            if constexpr (ODDG) gcap[i] = cap_of(gg, gbase[i]);
        } else {                          // packed weight block j: (blk = j / 2, group j % 2)
            const int j = q - NABLK, blk = j >> 1, gg = j & 1;
            gbase[i] = (const uint8_t *)a.wgt + (size_t)n0 * a.ld_wgt + gg * 32;
            goff[i] = (uint32_t)(min(n0 + blk * 32 + l32, a.N - 1) - n0) * (uint32_t)a.ld_wgt + half * 16;
            ldst[i] = I8_W_OFF + (blk * 2 + gg) * BLK_BYTES;
            if constexpr (ODDG) gcap[i] = cap_of(gg, gbase[i]);
        }
    }
    auto dma_one = [&](int s, uint8_t *dstbuf, int i) {  // block load i of stage s into a staging buffer
        const uint8_t *src;
        if constexpr (ODDG)
            src = gbase[i] + (goff[i] + min((uint32_t)s * (uint32_t)(KSTAGE / 2), gcap[i]));  // stage part wave-uniform
        else
            src = gbase[i] + (goff[i] + (uint32_t)s * (uint32_t)(KSTAGE / 2));
        __builtin_amdgcn_global_load_lds((const SVDQ_AS1 void *)src, (SVDQ_AS3 void *)(dstbuf + ldst[i]), 16, 0, 0);
    };
    // Scales go through registers (converted to fp32 and pre-multiplied on the way), one stage ahead: thread
    // (group sg of the stage, row sr of the tile) fetches one activation scale and one weight scale.
    const int sg = tid >> 7, sr = tid & 127;
    const int sgu = __builtin_amdgcn_readfirstlane(sg);
    const uint16_t *gAS = (const uint16_t *)a.ascales + (size_t)sgu * a.ld_ascales + m0;  // wave-uniform
    const uint16_t *gWS = (const uint16_t *)a.wscales + (size_t)sgu * a.ld_wscales + n0;
    const uint32_t as_off = 2 * (uint32_t)(min(m0 + sr, a.M - 1) - m0), ws_off = 2 * (uint32_t)(min(n0 + sr, a.N - 1) - n0);
    const uint32_t as_step = 4 * (uint32_t)a.ld_ascales, ws_step = 4 * (uint32_t)a.ld_wscales;  // bytes per stage
    const float fold = ACT_UNSIGNED ? (1.0f / 16.0f) : (1.0f / 256.0f);
    uint16_t ras, rws;
    uint32_t as_cap = 0, ws_cap = 0;
    if constexpr (ODDG) {
        as_cap = (uint32_t)(G / 2) * as_step;
        ws_cap = (uint32_t)(G / 2) * ws_step;
        if (sgu == 1) {  // this wavefront's group of the last stage does not exist
            if (G == 1) {
                gAS -= a.ld_ascales;
                gWS -= a.ld_wscales;
            }
            as_cap = G == 1 ? 0u : (uint32_t)(G / 2 - 1) * as_step;
            ws_cap = G == 1 ? 0u : (uint32_t)(G / 2 - 1) * ws_step;
        }
    }
    auto load_scales = [&](int s) {
        if (ODDG) {
            const uint16_t va = *(const uint16_t *)((const uint8_t *)gAS + (as_off + min((uint32_t)s * as_step, as_cap)));
            const uint16_t vw = *(const uint16_t *)((const uint8_t *)gWS + (ws_off + min((uint32_t)s * ws_step, ws_cap)));
            const bool off = s == G / 2 && sgu == 1;
            ras = off ? (uint16_t)0 : va;  // +0 in both 16-bit types
            rws = off ? (uint16_t)0 : vw;
        } else {
            ras = *(const uint16_t *)((const uint8_t *)gAS + (as_off + (uint32_t)s * as_step));
            rws = *(const uint16_t *)((const uint8_t *)gWS + (ws_off + (uint32_t)s * ws_step));
        }
    };
    auto store_scales = [&](uint8_t *base) {
        ((float *)(base + I8_AS_OFF))[sg * BM + sr] = T::to_f32(ras);
        const float w = T::to_f32(rws) * fold;
        ((float2 *)(base + I8_WS_OFF))[sg * BN + sr] = make_float2(w, -RNE_MAGIC * w);
    };

    // Main-loop accumulators: MFMA A operand = activations, B operand = weights, so a lane owns one weight row n and its
    // registers walk the wavefront's 32 activation rows: the weight scale is a per-lane scalar and the 16 activation
    // scales a lane needs per group are shared by the wavefront's four weight blocks.
    v16f acc[NBN];
#pragma unroll
    for (int bn = 0; bn < NBN; bn++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[bn][i] = 0.0f;

    const v16i cmagic = magic_acc();
    const int nstages = ODDG ? a.K / KSTAGE + 1 : a.K / KSTAGE;
    const int offW = I8_W_OFF + lane * 16;
    const int offA = wm * 2 * BLK_BYTES + lane * 16;

    load_scales(0);
#pragma unroll
    for (int i = 0; i < PER_WAVE; i++) dma_one(0, sbuf0, i);
    fetch_epilogue_operands<EPI>(a, sepi, n0, wm, lane);
    // One stage = eight (group, weight block) steps, software-pipelined inside the wavefront: the MFMAs of step b + 1
    // are issued before the dequantisation FMAs of step b, and the operands of step b + 2 are read from LDS behind
    // them, so the VALU work of a step runs while the matrix pipe works on the next one.
    auto stage = [&](auto par_tag, int s) {
        constexpr int P = decltype(par_tag)::value;
        uint8_t *base = P ? sbuf1 : sbuf0;   // this stage's operands
        uint8_t *other = P ? sbuf0 : sbuf1;  // being refilled for the next stage
        // everything issued for stage s (scale registers, then operand blocks) has landed
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
        store_scales(base);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));  // scale writes visible before the barrier
        __builtin_amdgcn_s_barrier();
        // The other buffer was last read in the previous stage, before the barrier: refill it during this stage.  The last
        // stage re-fetches itself into the idle buffer (harmless, and keeps the stage one basic block).
        const int sn = min(s + 1, nstages - 1);
        load_scales(sn);
        auto read_w = [&](int b, v4i &we, v4i &wo, float2 &wsp) {
            const int gg = b >> 2, bn = b & 3;
            const v4i wp = *(const v4i *)(base + offW + (bn * 2 + gg) * BLK_BYTES);
            unpack_signed(wp, we, wo);
            wsp = ((const float2 *)(base + I8_WS_OFF))[gg * BN + bn * 32 + l32];
        };
        auto read_a = [&](int gg, v4i &ae, v4i &ao) {
            const v4i ap = *(const v4i *)(base + offA + gg * BLK_BYTES);
            if (ACT_UNSIGNED)
                unpack_unsigned(ap, ae, ao);
            else
                unpack_signed(ap, ae, ao);
        };
        auto read_as = [&](int gg, v4f (&asv)[4]) {
#pragma unroll
            for (int j = 0; j < 4; j++)
                asv[j] = *(const v4f *)((const float *)(base + I8_AS_OFF) + gg * BM + wm * 32 + 8 * j + 4 * half);
        };
        v4i ae[2], ao[2], we[2], wo[2];
        float2 wsp[2];
        v4f asv[2][4];
        v16i t[2];
        read_a(0, ae[0], ao[0]);
        read_w(0, we[0], wo[0], wsp[0]);
        read_as(0, asv[0]);
        read_w(1, we[1], wo[1], wsp[1]);
        t[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ae[0], we[0], cmagic, 0, 0, 0);
        t[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ao[0], wo[0], t[0], 0, 0, 0);
        read_a(1, ae[1], ao[1]);
        read_as(1, asv[1]);
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const int cur = b & 1, nxt = cur ^ 1;
            float2 wcur = wsp[cur];
            if (b + 1 < 8) {
                const int g1 = (b + 1) >> 2;
                t[nxt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ae[g1], we[nxt], cmagic, 0, 0, 0);
                t[nxt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ao[g1], wo[nxt], t[nxt], 0, 0, 0);
            }
            if (b + 2 < 8) read_w(b + 2, we[cur], wo[cur], wsp[cur]);
            if (b < PER_WAVE) dma_one(sn, other, b);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float u = __builtin_fmaf(__int_as_float(t[cur][i]), wcur.x, wcur.y);
                acc[b & 3][i] = __builtin_fmaf(u, asv[b >> 2][i >> 2][i & 3], acc[b & 3][i]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    {
        int s = 0;
        for (; s + 1 < nstages; s += 2) {
            stage(std::integral_constant<int, 0>{}, s);
            stage(std::integral_constant<int, 1>{}, s + 1);
        }
        if (s < nstages) stage(std::integral_constant<int, 0>{}, s);
    }
    // The last stage's (redundant) block loads of this wavefront have landed; then every wavefront has left the main loop:
    // the staging memory becomes the wavefronts' private epilogue memory.
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    __syncthreads();
    tile_epilogue<T, EPI>(a, acc, (wm < 2 ? sbuf0 : sbuf1) + (wm & 1) * PRIV_BYTES, sepi, m0, n0, pid_n, wm, lane);
}

// ---- pre-split weights: fp8 x fp6 main loop --------------------------------------------------------------------------------
// PIPE = false: held to 168 registers, three workgroups per CU, a step's matrix instructions and FMAs in program order.
// PIPE = true: two workgroups per CU, the matrix instructions of step b + 1 issued ahead of the FMAs of step b (two sets
// of result registers): a workgroup on its own runs faster, which pays when few, long tiles leave CUs half empty.
// F6ACT (act_blocked == 2; instantiated with ACT_UNSIGNED, i.e. without the offset correction): the activations arrive
// as fp6 codes (sign | magnitude, what the matrix instruction wants of a signed value too) in lane order -- per 32 rows
// and group 1 KB of the lanes' first 16 bytes and 512 bytes of their last 8 -- and go into the matrix instruction as
// they are loaded: fp6 x fp6 (half the matrix-pipe time of fp8 x fp6), no nibble unpack, no offset to take out.
// SB (ascales_blocked, with F6ACT; K / 64 a multiple of 8): the activation scales of the eight groups of four stages lie
// side by side per row: one 16-byte load per lane every four stages instead of two 2-byte loads per stage.
template <typename T, bool ACT_UNSIGNED, int EPI, bool PIPE, bool F6ACT = false, bool SB = false>
__global__ __launch_bounds__(NTHREADS, PIPE ? 2 : 3) void gemm_w4a4_f8_kernel(svdq_gemm_args a) {
    static_assert(!F6ACT || ACT_UNSIGNED, "fp6 activation codes carry their sign: there is no offset to correct");
    static_assert(!SB || F6ACT, "blocked activation scales come with fp6 activation codes");
    // Separate LDS objects: the compiler then knows that a block load into one staging buffer cannot touch what is being
    // read from the other (one object would make every LDS read wait for the loads in flight).
    __shared__ __align__(16) uint8_t sbuf0[F8_STAGE_BYTES];
    __shared__ __align__(16) uint8_t sbuf1[F8_STAGE_BYTES];
    __shared__ __align__(16) uint8_t sring[F8_RING_BYTES];
    __shared__ __align__(16) uint8_t sepi[EPI_LDS_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wm = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: the wavefront's 32-row block of the tile
    const int l32 = lane & 31, half = lane >> 5;

    int pid_m, pid_n;
    tile_ids((a.M + BM - 1) / BM, (a.N + BN - 1) / BN, pid_m, pid_n);
    const int m0 = pid_m * BM, n0 = pid_n * BN;
    const int G = a.K / GROUP, nstages = (G + 1) / 2;

    // ---- what a wavefront fetches per stage, one stage ahead ------------------------------------------------------
    // global -> LDS: the three 1 KB code blocks of weight block wm of the tile and its 12-byte rows of scales and offset
    // terms (address = wave-uniform base in SGPRs + a 32-bit offset: lane part + stage * step).  A block of rows past N
    // re-reads the last block (its outputs are never stored).
    const int nblk = min(n0 / 32 + wm, (a.N + 31) / 32 - 1);
    const uint8_t *wbase = (const uint8_t *)a.wgt_planes + (size_t)nblk * nstages * (WPL_BLOCKS * BLK_BYTES);
    const uint8_t *xbase = (const uint8_t *)a.wgt_planes + planes_code_bytes(a.N, a.K) + (size_t)nblk * (nstages + 1) * AUX_BLK;
    const __amdgpu_buffer_rsrc_t rW = g_buffer(wbase), rX = g_buffer(xbase);
    auto dma = [&](int s, uint8_t *dstbuf, int slot, int i) {  // i = 0, 1, 2: code blocks of stage s; i = 3: its scales and offset terms
        if (i < WPL_BLOCKS) {
            g_load16_lds(rW, dstbuf + (wm * WPL_BLOCKS + i) * BLK_BYTES, (uint32_t)lane * 16u,
                         (uint32_t)s * (uint32_t)(WPL_BLOCKS * BLK_BYTES) + (uint32_t)(i * BLK_BYTES));
        } else {
            // 64 lanes x 12 bytes = the rows of stage s and of stage s + 1 (the copy has one stage of padding), into the given
            // ring slot and the one after it: issued before the loop for stages 0 and 1 and then by every odd stage for the two
            // stages after it (an even slot and its neighbour)
            g_load12_lds(rX, sring + wm * AUX_NBLK_BYTES + slot * AUX_LBLK, (uint32_t)lane * (uint32_t)AUX_ROW, (uint32_t)s * (uint32_t)AUX_BLK);
        }
    };
    // registers: the 16 packed bytes of the lane's activation row (row wm * 32 + l32, K half lane / 32) of both groups,
    // exactly what the lane holds as MFMA operand after the unpack, and the row's two activation scales.  A group past
    // the end (K / 64 odd) re-reads the last one: its weight codes, scale and offset term are stored as zero.
    v4i araw[2];
    v8i a6[2][2];  // F6ACT: [stage parity][group], loaded one stage ahead into the set the running stage does not read
    uint16_t qa[2];
    const int mrow = min(m0 + wm * 32 + l32, a.M - 1);
    // Activations either as the (M, K / 2) matrix (a lane fetches the 16 bytes of its own row: 32 rows to a load
    // instruction) or in lane order (act_blocked: per 32 rows and group 1 KB = lane l's 16 bytes at 16 l, groups in a
    // row): the same two loads per stage, base + lane offset + group * step, with other constants.
    const bool ablk = F6ACT || a.act_blocked != 0;
    const uint32_t sAct = F6ACT ? 1536u : ablk ? 1024u : 32u;
    // a tile's row blocks past the last one that exists (M no multiple of 128) re-read the last: their rows are never stored
    const int rblk = min((m0 >> 5) + wm, ((a.M + 31) >> 5) - 1);
    const __amdgpu_buffer_rsrc_t rAct = g_buffer((const uint8_t *)a.act + (ablk ? (size_t)rblk * G * sAct : (size_t)m0 * a.ld_act));
    const __amdgpu_buffer_rsrc_t rAS = g_buffer(a.ascales);
    const uint32_t oAct = ablk ? (uint32_t)lane * 16u : (uint32_t)(mrow - m0) * (uint32_t)a.ld_act + half * 16;
    const uint32_t oExt = 1024u + (uint32_t)lane * 8u;
    const uint32_t oA = 2u * (uint32_t)mrow;
    // SB: dword ST of sc_cur = the row's scales of the two groups of stage ST of the current four stages; sc_nxt is loaded
    // during their first stage (512 bytes per 32 rows and four stages)
    v4i sc_cur = {0, 0, 0, 0}, sc_nxt = {0, 0, 0, 0};
    const __amdgpu_buffer_rsrc_t rASb = g_buffer((const uint8_t *)a.ascales + (SB ? (size_t)rblk * (G >> 3) * 512 : 0));
    const uint32_t oAb = (uint32_t)l32 * 16u;
    if constexpr (SB) sc_cur = g_load128(rASb, oAb, 0);
    auto load_regs = [&](int s, auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
#pragma unroll
        for (int gg = 0; gg < 2; gg++) {
            const int gi = min(2 * s + gg, G - 1);
            if constexpr (!SB) qa[gg] = g_load16(rAS, oA, (uint32_t)gi * (uint32_t)a.ld_ascales * 2u);
            if constexpr (F6ACT) {
                const v4i lo = g_load128(rAct, oAct, (uint32_t)gi * sAct);
                const v2i hi = g_load64(rAct, oExt, (uint32_t)gi * sAct);
                a6[SET][gg] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], 0, 0};
            } else {
                araw[gg] = g_load128(rAct, oAct, (uint32_t)gi * sAct);
            }
        }
    };

    v16f acc[NBN];
#pragma unroll
    for (int bn = 0; bn < NBN; bn++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[bn][i] = 0.0f;

    // ---- the offset of signed activations, taken out every four stages ------------------------------------------------
    // The fp8 operand holds a + 8 for even k and a - 7 for odd k, so a group's product comes out
    // as p_g + (8 We - 7 Wo) with We / Wo the sums of the group's even / odd weights.  D[g, n] = -ws[g, n] (8 We - 7 Wo)
    // travels with the weights as two 16-bit pieces; acc += sum_g as[g, m] * D[g, n] over the eight groups of four stages is
    // one 32x32x16 matrix instruction per weight block: K slot 4 * (stage of the four) + 2 * (group of the stage) + piece.
    // The activation-side operand collects the activation scales stage by stage (lanes of half h own stages 2 h and
    // 2 h + 1); the weight-side operand is read from the ring.  It is applied at the start of the following stage, when none
    // of this wavefront's loads is in flight.
    int ub[4] = {0, 0, 0, 0};
    auto corr = [&](uint32_t off0, uint32_t off1) {  // byte offsets in a block's ring of the lane's two stages
        const v4i ubv = {ub[0], ub[1], ub[2], ub[3]};
#pragma unroll
        for (int bn = 0; bn < NBN; bn++) {
            const uint32_t *p0 = (const uint32_t *)(sring + bn * AUX_NBLK_BYTES + off0);
            const uint32_t *p1 = (const uint32_t *)(sring + bn * AUX_NBLK_BYTES + off1);
            acc[bn] = mfma32_16bit<T>((v4i){(int)p0[0], (int)p0[1], (int)p1[0], (int)p1[1]}, ubv, acc[bn]);
        }
    };
    int par = 0;                                         // parity of the group of four stages: ring slots 0-3 or 4-7
    uint32_t rcur = (uint32_t)l32 * AUX_LROW;            // this lane's row in slot 0 / 4 of the current four stages
    uint32_t rprev = rcur + (uint32_t)(4 + 2 * half) * AUX_LBLK;  // ... in its first stage of the previous four
    if constexpr (!ACT_UNSIGNED) {
        // the first stage applies a correction for four stages that never ran: its weight-side operand must be finite
        v4i *z = (v4i *)(sring + wm * AUX_NBLK_BYTES + 4 * AUX_LBLK) + lane;
        z[0] = z[64] = (v4i){0, 0, 0, 0};
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
    }

    load_regs(0, std::integral_constant<int, 0>{});
#pragma unroll
    for (int i = 0; i < 4; i++) dma(0, sbuf0, 0, i);
    fetch_epilogue_operands<EPI>(a, sepi, n0, wm, lane);

    // One stage = eight (group, weight block) steps: scale product, group product, sixteen FMAs.  The operands of the next
    // step (the step after next when PIPE) are read from LDS behind the matrix instructions.
    auto stage = [&](auto st_tag, int s) {
        constexpr int ST = decltype(st_tag)::value;   // stage within its group of four
        uint8_t *base = (ST & 1) ? sbuf1 : sbuf0;     // this stage's operands
        uint8_t *other = (ST & 1) ? sbuf0 : sbuf1;    // being refilled for the next stage
        // everything this wavefront issued for stage s (registers, then blocks) has landed
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
        // two's complement nibble -> a + 8 is a flip of the nibble's top bit; -> a - 7 = -(7 - a) is a flip of the other
        // three plus the fp8 sign bit: written per plane so that mask and flip are one three-input bit operation
        v8i a8[2];
        if constexpr (F6ACT) {
            a8[0] = a6[ST & 1][0];
            a8[1] = a6[ST & 1][1];
        } else {
#pragma unroll
            for (int gg = 0; gg < 2; gg++) {
                typedef unsigned v4u __attribute__((ext_vector_type(4)));
                const v4u u = __builtin_bit_cast(v4u, araw[gg]);
                const unsigned fe = ACT_UNSIGNED ? 0u : 0x08080808u, fo = ACT_UNSIGNED ? 0u : 0x87878787u;
                const v4u e = (u & 0x0F0F0F0Fu) ^ fe, o = ((u >> 4) & 0x0F0F0F0Fu) ^ fo;
                a8[gg] = (v8i){(int)e[0], (int)e[1], (int)e[2], (int)e[3], (int)o[0], (int)o[1], (int)o[2], (int)o[3]};
            }
        }
        // Operands of the scale products as[m] * ws[n] for a 32x32x8 matrix instruction on 16-bit values: lanes 0-31 hold K
        // slots 0-3, two to a register.  The weight side is the dword (ws of the first group, ws of the second group) as it
        // lies in the ring; the activation side carries as of the step's group in that group's slot and zero elsewhere
        // (also in lanes 32-63, whose weight-side values therefore do not matter).
        int qa0, qa1;
        if constexpr (SB) {
            qa0 = sc_cur[ST] & 0xFFFF;
            qa1 = sc_cur[ST] & (int)0xFFFF0000;
            if constexpr (ST == 0) sc_nxt = g_load128(rASb, oAb, (uint32_t)min((s >> 2) + 1, (nstages >> 2) - 1) * 512u);
        } else {
            qa0 = (int)qa[0];
            qa1 = (int)((uint32_t)qa[1] << 16);
        }
        const v2i sa[2] = {(v2i){half ? 0 : qa0, 0}, (v2i){half ? 0 : qa1, 0}};
        __builtin_amdgcn_s_barrier();
        if constexpr (!ACT_UNSIGNED) {
            if constexpr (ST == 0) {
                corr(rprev, rprev + AUX_LBLK);
#pragma unroll
                for (int e = 0; e < 4; e++) ub[e] = 0;
            }
            const bool mine = half == (ST >> 1);
            ub[2 * (ST & 1)] = mine ? (qa0 | (qa0 << 16)) : ub[2 * (ST & 1)];
            ub[2 * (ST & 1) + 1] = mine ? (qa1 | (int)((uint32_t)qa1 >> 16)) : ub[2 * (ST & 1) + 1];
        }
        uint32_t wsd[NBN];
#pragma unroll
        for (int bn = 0; bn < NBN; bn++) wsd[bn] = *(const uint32_t *)(sring + bn * AUX_NBLK_BYTES + ST * AUX_LBLK + 8 + rcur);
        // The other buffer was last read in the previous stage, before the barrier: refill it during this stage.  The last
        // stage re-fetches itself (harmless, and keeps the stage one basic block); its rows go to the next ring slot all
        // the same, which nobody reads.
        const int sn = min(s + 1, nstages - 1), slotn = (s + 1) & (AUX_SLOTS - 1);
        load_regs(sn, std::integral_constant<int, (ST + 1) & 1>{});
        auto read_w8 = [&](int b) -> v8i {  // six registers of fp6 codes (the matrix instruction ignores the last two)
            const int gg = b >> 2, bn = b & 3;
            const v4i lo = *(const v4i *)(base + lane * 16 + (bn * WPL_BLOCKS + gg) * BLK_BYTES);
            const v2i hi = *(const v2i *)(base + lane * 16 + (bn * WPL_BLOCKS + 2) * BLK_BYTES + gg * 8);
            return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], 0, 0};
        };
        const v16f z16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        // as[m] * ws[n] of a step, exact (two 16-bit values, one non-zero product): a 16-bit matrix instruction, which runs
        // beside the vector FMAs; the fp32 rank-1 matrix instruction shares the vector ALUs and does not
        auto scales = [&](int b) -> v16f { return mfma32_16bit_k8<T>((v2i){(int)wsd[b & 3], 0}, sa[b >> 2], z16); };
        auto group = [&](int b, const v8i &w) -> v16f {
            if constexpr (F6ACT)
                return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, a8[b >> 2], z16, 2, 2, 0, F6_SCALE, 0, F6_SCALE);
            else
                return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, a8[b >> 2], z16, 2, 0, 0, F6_SCALE, 0, F8_SCALE);
        };
        if constexpr (!PIPE) {
            v8i w8[2];
            w8[0] = read_w8(0);
#pragma unroll
            for (int b = 0; b < 8; b++) {
                const v16f S = scales(b);
                const v16f P = group(b, w8[b & 1]);
                __builtin_amdgcn_sched_barrier(0);
                if (b + 1 < 8) w8[(b + 1) & 1] = read_w8(b + 1);
                if (b < WPL_BLOCKS || (b == WPL_BLOCKS && (ST & 1))) dma(sn, other, slotn, b);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < 16; i++) acc[b & 3][i] = __builtin_fmaf(P[i], S[i], acc[b & 3][i]);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            v8i w8[3];
            v16f S[2], P[2];
            w8[0] = read_w8(0);
            w8[1] = read_w8(1);
            S[0] = scales(0);
            P[0] = group(0, w8[0]);
#pragma unroll
            for (int b = 0; b < 8; b++) {
                const int cur = b & 1, nxt = cur ^ 1;
                if (b + 1 < 8) {
                    S[nxt] = scales(b + 1);
                    P[nxt] = group(b + 1, w8[(b + 1) % 3]);
                }
                // the operand reads of step b + 2 stay behind the matrix instructions: hoisted above them, the wait for step
                // b + 1's operands would also wait for these
                __builtin_amdgcn_sched_barrier(0);
                if (b + 2 < 8) w8[(b + 2) % 3] = read_w8(b + 2);
                if (b < WPL_BLOCKS || (b == WPL_BLOCKS && (ST & 1))) dma(sn, other, slotn, b);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < 16; i++) acc[b & 3][i] = __builtin_fmaf(P[cur][i], S[cur][i], acc[b & 3][i]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    int s = 0;
    for (; s + 4 <= nstages; s += 4) {
        stage(std::integral_constant<int, 0>{}, s);
        stage(std::integral_constant<int, 1>{}, s + 1);
        stage(std::integral_constant<int, 2>{}, s + 2);
        stage(std::integral_constant<int, 3>{}, s + 3);
        if constexpr (SB) sc_cur = sc_nxt;
        par ^= 1;
        rcur = (uint32_t)l32 * AUX_LROW + (uint32_t)(4 * par) * AUX_LBLK;
        rprev = (uint32_t)l32 * AUX_LROW + (uint32_t)(4 * (par ^ 1) + 2 * half) * AUX_LBLK;
    }
    const int rem = nstages - s;  // 0 .. 3 stages of a last, partial group of four
    if (rem >= 1) stage(std::integral_constant<int, 0>{}, s);
    if (rem >= 2) stage(std::integral_constant<int, 1>{}, s + 1);
    if (rem >= 3) stage(std::integral_constant<int, 2>{}, s + 2);
    // The last stage's (redundant) loads of this wavefront have landed.
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    if constexpr (!ACT_UNSIGNED) {
        if (rem == 0) {
            corr(rprev, rprev + AUX_LBLK);
        } else {
            // a stage past the end reads the rows of the last real one: its activation-side entries are zero
            const uint32_t r0 = (uint32_t)l32 * AUX_LROW + (uint32_t)(4 * par) * AUX_LBLK;
            corr(r0 + (uint32_t)min(2 * half, rem - 1) * AUX_LBLK, r0 + (uint32_t)min(2 * half + 1, rem - 1) * AUX_LBLK);
        }
    }
    // Every wavefront has left the main loop: the staging memory becomes the wavefronts' private epilogue memory.
    __syncthreads();
    uint8_t *priv = wm == 0 ? sbuf0 : wm == 1 ? sbuf1 : sring + (wm - 2) * PRIV_BYTES;
    tile_epilogue<T, EPI, true>(a, acc, priv, sepi, m0, n0, pid_n, wm, lane);
}

// lora_act_out[m, r] = sum over n-tiles of the partial LoRA-down products, in tile order (deterministic)
__global__ __launch_bounds__(64) void lora_part_reduce_kernel(const float *part, float *out, int tiles, int M, int R2,
                                                              int ld_out) {
    const int idx = (blockIdx.x * 64 + threadIdx.x) * 4;  // four consecutive r of one row (R2 % 16 == 0)
    if (idx >= M * R2) return;
    const size_t stride = (size_t)M * R2;
    v4f s = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 8
    for (int t = 0; t < tiles; t++) s += *(const v4f *)(part + t * stride + idx);
    *(v4f *)(out + (size_t)(idx / R2) * ld_out + idx % R2) = s;
}

// Debug read-out of one group's exact int32 accumulators: one wavefront per 32x32 block, operands straight from
// global memory, same unpack + MFMA sequence as the GEMM main loop.
template <bool ACT_UNSIGNED>
__global__ __launch_bounds__(64) void group_acc_kernel(const uint8_t *act, const uint8_t *wgt, int32_t *out, int M,
                                                       int N, int ld_act, int ld_wgt, int group) {
    const int lane = threadIdx.x, l32 = lane & 31, half = lane >> 5;
    const int nb = blockIdx.x * 32, mb = blockIdx.y * 32;
    const v4i wp = *(const v4i *)(wgt + (size_t)min(nb + l32, N - 1) * ld_wgt + group * 32 + half * 16);
    const v4i ap = *(const v4i *)(act + (size_t)min(mb + l32, M - 1) * ld_act + group * 32 + half * 16);
    v4i we, wo, ae, ao;
    unpack_signed(wp, we, wo);
    if (ACT_UNSIGNED)
        unpack_unsigned(ap, ae, ao);
    else
        unpack_signed(ap, ae, ao);
    v16i t = __builtin_amdgcn_mfma_i32_32x32x32_i8(we, ae, magic_acc(), 0, 0, 0);
    t = __builtin_amdgcn_mfma_i32_32x32x32_i8(wo, ao, t, 0, 0, 0);
    const int m = mb + l32;
    if (m >= M) return;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int n = nb + 8 * (i >> 2) + 4 * half + (i & 3);
        if (n < N) out[(size_t)m * N + n] = (t[i] - RNE_MAGIC_BITS) >> (ACT_UNSIGNED ? 4 : 8);
    }
}

// The same read-out through the instructions of the pre-split (fp8) path (operands in the other order): activation nibbles as fp8 codes
// (signed ones as a + 8 for even k and a - 7 for odd k), weights as fp6 codes,
// v_mfma_scale_f32_32x32x64_f8f6f4 with block scales 2^9 and 2^3, offset term 8 We - 7 Wo taken out.  Every value involved
// is an integer below 2^24, so the fp32 result is exact.
template <bool ACT_UNSIGNED>
__global__ __launch_bounds__(64) void group_acc_f8_kernel(const uint8_t *act, const uint8_t *wgt, int32_t *out, int M,
                                                          int N, int ld_act, int ld_wgt, int group) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    const int lane = threadIdx.x, l32 = lane & 31, half = lane >> 5;
    const int nb = blockIdx.x * 32, mb = blockIdx.y * 32;
    const v4u u = __builtin_bit_cast(v4u, *(const v4i *)(act + (size_t)min(mb + l32, M - 1) * ld_act + group * 32 + half * 16));
    const unsigned fe = ACT_UNSIGNED ? 0u : 0x08080808u, fo = ACT_UNSIGNED ? 0u : 0x87878787u;
    const v4u e = (u & 0x0F0F0F0Fu) ^ fe, o = ((u >> 4) & 0x0F0F0F0Fu) ^ fo;
    const v8i a8 = {(int)e[0], (int)e[1], (int)e[2], (int)e[3], (int)o[0], (int)o[1], (int)o[2], (int)o[3]};
    uint32_t w6[6];
    const uint8_t *wrow = wgt + (size_t)min(nb + l32, N - 1) * ld_wgt + group * 32;
    f6_pack(*(const v4i *)wrow, *(const v4i *)(wrow + 16), half, w6);
    const v8i w8 = {(int)w6[0], (int)w6[1], (int)w6[2], (int)w6[3], (int)w6[4], (int)w6[5], 0, 0};
    const int offs = ACT_UNSIGNED ? 0 : group_offset_term(*(const v4i *)wrow, *(const v4i *)(wrow + 16));
    const v16f z16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    v16f t = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, w8, z16, 0, 2, 0, F8_SCALE, 0, F6_SCALE);
    // The matrix instruction reads the operands of all 64 lanes: pin it here, ahead of the lane-dependent stores below
    // (moved behind a divergent branch, it ran with some lanes' operands never loaded).
    asm volatile("" : "+v"(t));
    const int n = nb + l32;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int m = mb + 8 * (i >> 2) + 4 * half + (i & 3);
        if (m < M && n < N) out[(size_t)m * N + n] = (int)t[i] - offs;
    }
}


// transposed LoRA-down weight -> the order the GELU epilogue's lanes read it (svdq_block_lora_down): one thread per lane
// and matrix-instruction operand
__global__ __launch_bounds__(256) void block_lora_down_kernel(const uint16_t *ldt, v4i *out, int N, int R2, int pieces) {
    const int o = blockIdx.x * 256 + threadIdx.x;
    if (o >= pieces) return;
    const int lane = o & 63, blk = (o >> 6) & 7, nrc = (R2 + 31) / 32, chunk = (o >> 9) % nrc, tile = (o >> 9) / nrc;
    const int r = chunk * 32 + (lane & 31), col = tile * 128 + (blk >> 1) * 32 + 16 * (blk & 1) + 4 * (lane >> 5);
    v4i v = {0, 0, 0, 0};
    if (r < R2) {
        const uint2 q0 = *(const uint2 *)(ldt + (size_t)r * N + col), q1 = *(const uint2 *)(ldt + (size_t)r * N + col + 8);
        v = (v4i){(int)q0.x, (int)q0.y, (int)q1.x, (int)q1.y};
    }
    out[o] = v;
}

// rotary table -> the order the Q/K epilogue's lanes read it (svdq_block_rotary): one thread per 16-byte piece
__global__ __launch_bounds__(256) void block_rotary_kernel(const float *rot, v4f *out, int rows, int ld, int pieces) {
    const int o = blockIdx.x * 256 + threadIdx.x;
    if (o >= pieces) return;
    const int lane = o & 63, j = (o >> 6) & 3, bn = (o >> 8) & 3, rb = o >> 10;
    const int row = rb * 32 + (lane & 31), d = bn * 32 + 8 * j + 4 * (lane >> 5);
    out[o] = *(const v4f *)(rot + (size_t)(row < rows ? row : 0) * ld + d);
}

template <typename T, bool U, bool ODDG>
static void launch_gemm_i8(const svdq_gemm_args &a, hipStream_t s) {
    const dim3 grid(((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN)), block(NTHREADS);
    switch (a.epilogue) {
        case SVDQ_EPI_PLAIN:
            hipLaunchKernelGGL((gemm_w4a4_i8_kernel<T, U, SVDQ_EPI_PLAIN, ODDG>), grid, block, 0, s, a);
            break;
        case SVDQ_EPI_QK_NORM_ROPE:
            hipLaunchKernelGGL((gemm_w4a4_i8_kernel<T, U, SVDQ_EPI_QK_NORM_ROPE, ODDG>), grid, block, 0, s, a);
            break;
        case SVDQ_EPI_GELU_QUANT:
            hipLaunchKernelGGL((gemm_w4a4_i8_kernel<T, U, SVDQ_EPI_GELU_QUANT, ODDG>), grid, block, 0, s, a);
            break;
        case SVDQ_EPI_SWIGLU_QUANT:
            hipLaunchKernelGGL((gemm_w4a4_i8_kernel<T, U, SVDQ_EPI_SWIGLU_QUANT, ODDG>), grid, block, 0, s, a);
            break;
    }
}

// Workgroups per CU for the fp8 kernel.  Three (PIPE = false) keep a full CU about 8 % busier than two (PIPE = true), but a
// workgroup of the two-per-CU kernel runs faster, which decides when the last round of tiles leaves most CUs with one or
// two workgroups.  Cost model, in units of a tile's share of a fully loaded three-per-CU CU: whole rounds cost 3 (three per
// CU) or 2 * 1.08 (two per CU); a last round whose fullest CU holds k tiles costs 1.75 / 2.15 / 3 (k = 1 / 2 / 3) or
// 1.4 / 2 (k = 1 / 2).  The constants are measured (K = 3072, N = 9216: M = 512 -> 288 tiles, M = 1024 -> 576, M = 4608 -> 2592;
// K = 12288, N = 3072, M = 4608 -> 864), and the model picks as the measurements do: 2592, 3456, 4608 and 576 tiles -> three per
// CU; 864 and 288 tiles -> two.
static int cu_count() {
    static std::atomic<int> cached{0};
    int n = cached.load(std::memory_order_relaxed);
    if (n > 0) return n;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
        n = 256;
    cached.store(n, std::memory_order_relaxed);
    return n;
}
static std::atomic<int> g_f8_variant{-1};  // svdq_gemm_w4a4_set_variant
static bool two_workgroups_per_cu(long tiles) {
    const int forced = g_f8_variant.load(std::memory_order_relaxed);
    if (forced >= 0) return forced == 1;
    const long cus = cu_count();
    auto cost = [&](long occ, double round, const double (&last)[3]) {
        const long full = tiles / (cus * occ), rem = tiles - full * cus * occ;
        return (double)full * round + (rem == 0 ? 0.0 : last[(rem + cus - 1) / cus - 1]);
    };
    const double last3[3] = {1.75, 2.15, 3.0}, last2[3] = {1.4, 2.0, 2.0};
    return cost(2, 2.16, last2) < cost(3, 3.0, last3);
}

template <typename T, bool U, bool PIPE, bool F6ACT, bool SB = false>
static void launch_gemm_f8p(const svdq_gemm_args &a, hipStream_t s) {
    const dim3 grid(((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN)), block(NTHREADS);
    switch (a.epilogue) {
        case SVDQ_EPI_PLAIN:
            hipLaunchKernelGGL((gemm_w4a4_f8_kernel<T, U, SVDQ_EPI_PLAIN, PIPE, F6ACT, SB>), grid, block, 0, s, a);
            break;
        case SVDQ_EPI_QK_NORM_ROPE:
            hipLaunchKernelGGL((gemm_w4a4_f8_kernel<T, U, SVDQ_EPI_QK_NORM_ROPE, PIPE, F6ACT, SB>), grid, block, 0, s, a);
            break;
        case SVDQ_EPI_GELU_QUANT:
            hipLaunchKernelGGL((gemm_w4a4_f8_kernel<T, U, SVDQ_EPI_GELU_QUANT, PIPE, F6ACT, SB>), grid, block, 0, s, a);
            break;
        case SVDQ_EPI_SWIGLU_QUANT:
            hipLaunchKernelGGL((gemm_w4a4_f8_kernel<T, U, SVDQ_EPI_SWIGLU_QUANT, PIPE, F6ACT, SB>), grid, block, 0, s, a);
            break;
    }
}

template <typename T, bool U>
static void launch_gemm_f8(const svdq_gemm_args &a, hipStream_t s) {
    const bool two = two_workgroups_per_cu((long)((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN));
    if (a.act_blocked == 2) {  // fp6 codes carry their sign: one instantiation for signed and unsigned activations
        if (a.ascales_blocked) {
            if (two)
                launch_gemm_f8p<T, true, true, true, true>(a, s);
            else
                launch_gemm_f8p<T, true, false, true, true>(a, s);
        } else if (two) {
            launch_gemm_f8p<T, true, true, true>(a, s);
        } else {
            launch_gemm_f8p<T, true, false, true>(a, s);
        }
    } else if (two) {
        launch_gemm_f8p<T, U, true, false>(a, s);
    } else {
        launch_gemm_f8p<T, U, false, false>(a, s);
    }
}

template <typename T, bool U>
static void launch_gemm_epi(const svdq_gemm_args &a, hipStream_t s) {
    if (a.wgt_planes != nullptr)
        launch_gemm_f8<T, U>(a, s);
    else if ((a.K / GROUP) & 1)
        launch_gemm_i8<T, U, true>(a, s);
    else
        launch_gemm_i8<T, U, false>(a, s);
}

// Weight re-layout, codes: thread (block of 32 rows, stage of two groups, lane) turns the nibbles of its parity of each
// group's 32 packed bytes into six registers of fp6 codes; a group past the end (K / 64 odd) is stored as zeros.  Thread 0 clears the status word.
__global__ void split_weight_planes_kernel(const uint8_t *wgt, uint8_t *planes, int32_t *status, int N, int G, int ld_wgt) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx == 0) *status = 0;  // the kernel that may raise it runs after this one
    const int lane = idx & 63;
    const size_t bs = idx >> 6;  // nblk * nst + s
    const int nst = (G + 1) / 2;
    const int s = (int)(bs % nst), nblk = (int)(bs / nst);
    if (nblk >= (N + 31) / 32) return;
    const int row = min(nblk * 32 + (lane & 31), N - 1);
    uint8_t *dst = planes + bs * (WPL_BLOCKS * BLK_BYTES) + lane * 16;
#pragma unroll
    for (int gg = 0; gg < 2; gg++) {
        const int g = 2 * s + gg;
        uint32_t d[6] = {0, 0, 0, 0, 0, 0};
        if (g < G) {
            const uint8_t *src = wgt + (size_t)row * ld_wgt + g * 32;
            f6_pack(*(const v4i *)src, *(const v4i *)(src + 16), lane >> 5, d);
        }
        *(v4i *)(dst + gg * BLK_BYTES) = (v4i){(int)d[0], (int)d[1], (int)d[2], (int)d[3]};
        *(v2i *)(dst + 2 * BLK_BYTES + gg * 8) = (v2i){(int)d[4], (int)d[5]};
    }
}

// Weight re-layout, scales and offset terms: thread (block of 32 rows, stage, row of the block) writes the row's six
// 16-bit values of the stage: for each of the two groups the pieces hi, lo of
// D = -ws * (8 * sum of the even-k weights - 7 * sum of the odd-k weights)  (the product is exact in fp32; hi + lo carry it
// to 16 significant bits in bf16, 22 in fp16), then the two weight scales.  Rows past N repeat row N - 1; a group past the
// end and the stage of padding behind each block's last stage are zeros.  `status` is set to 1 when a piece is not finite
// (fp16 scales of about 17 and more), in which case the copy must not be used.
template <typename T>
__global__ void weight_aux_kernel(const uint8_t *wgt, const uint16_t *wscales, uint16_t *aux, int32_t *status, int N, int G,
                                  int ld_wgt, int ld_wscales) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int r = idx & 31;
    const size_t bs = idx >> 5;  // nblk * (nst + 1) + s
    const int nst = (G + 1) / 2;
    const int s = (int)(bs % (nst + 1)), nblk = (int)(bs / (nst + 1));
    if (nblk >= (N + 31) / 32) return;
    const int row = min(nblk * 32 + r, N - 1);
    uint16_t v[6] = {0, 0, 0, 0, 0, 0};
    bool bad = false;
#pragma unroll
    for (int gg = 0; gg < 2; gg++) {
        const int g = 2 * s + gg;
        if (s < nst && g < G) {
            const uint8_t *src = wgt + (size_t)row * ld_wgt + g * 32;
            const uint16_t ws = wscales[(size_t)g * ld_wscales + row];
            float d = -(T::to_f32(ws) * (float)group_offset_term(*(const v4i *)src, *(const v4i *)(src + 16)));
            const uint16_t hi = T::from_f32(d);
            d -= T::to_f32(hi);
            const uint16_t lo = T::from_f32(d);
            bad = bad || !isfinite(T::to_f32(hi)) || !isfinite(T::to_f32(lo)) || !isfinite(T::to_f32(ws));
            v[2 * gg] = hi;
            v[2 * gg + 1] = lo;
            v[4 + gg] = ws;
        }
    }
    uint32_t *dst = (uint32_t *)(aux + idx * 6);
    dst[0] = (uint32_t)v[0] | ((uint32_t)v[1] << 16);
    dst[1] = (uint32_t)v[2] | ((uint32_t)v[3] << 16);
    dst[2] = (uint32_t)v[4] | ((uint32_t)v[5] << 16);
    if (bad) *status = 1;
}

}  // namespace svdq

using namespace svdq;

static bool al16(const void *p) { return ((uintptr_t)p & 15) == 0; }

extern "C" size_t svdq_weight_planes_bytes(int32_t N, int32_t K) {
    if (N <= 0 || K <= 0) return 0;
    return planes_code_bytes(N, K) + planes_aux_bytes(N, K) + PLANES_STATUS_BYTES;  // fp6 codes, scales and offset terms, status word
}

extern "C" int svdq_split_weight_planes(const void *wgt, const void *wscales, void *planes, int32_t N, int32_t K,
                                        int32_t ld_wgt, int32_t ld_wscales, int32_t dtype, void *stream) {
    if (!wgt || !wscales || !planes || N <= 0 || K <= 0 || K % GROUP || ld_wgt % 16 || ld_wgt < K / 2 || ld_wscales < N ||
        ((uintptr_t)wgt & 15) || ((uintptr_t)planes & 15) || (dtype != SVDQ_BF16 && dtype != SVDQ_FP16)) {
        set_error("svdq_split_weight_planes: bad arguments (N=%d K=%d ld_wgt=%d ld_wscales=%d dtype=%d; rows must be 16-byte aligned)",
                  N, K, ld_wgt, ld_wscales, dtype);
        return SVDQ_E_INVALID;
    }
    const int G = K / GROUP, nblk = (N + 31) / 32, nst = (G + 1) / 2;
    hipStream_t st = (hipStream_t)stream;
    uint8_t *aux = (uint8_t *)planes + planes_code_bytes(N, K);
    int32_t *status = (int32_t *)(aux + planes_aux_bytes(N, K));
    const size_t n = (size_t)nblk * nst * 64;
    hipLaunchKernelGGL(split_weight_planes_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                       (const uint8_t *)wgt, (uint8_t *)planes, status, N, G, ld_wgt);
    int rc = check_launch("svdq_split_weight_planes");
    if (rc) return rc;
    const size_t nd = (size_t)nblk * (nst + 1) * 32;
    if (dtype == SVDQ_BF16)
        hipLaunchKernelGGL(weight_aux_kernel<BF16>, dim3((unsigned)((nd + 255) / 256)), dim3(256), 0, st,
                           (const uint8_t *)wgt, (const uint16_t *)wscales, (uint16_t *)aux, status, N, G, ld_wgt, ld_wscales);
    else
        hipLaunchKernelGGL(weight_aux_kernel<FP16>, dim3((unsigned)((nd + 255) / 256)), dim3(256), 0, st,
                           (const uint8_t *)wgt, (const uint16_t *)wscales, (uint16_t *)aux, status, N, G, ld_wgt, ld_wscales);
    return check_launch("svdq_split_weight_planes (scales and offset terms)");
}

extern "C" size_t svdq_gemm_w4a4_scratch_bytes(int32_t M, int32_t N, int32_t R2, int32_t epilogue) {
    if (R2 <= 0 || (epilogue != SVDQ_EPI_GELU_QUANT && epilogue != SVDQ_EPI_SWIGLU_QUANT)) return 0;
    return (size_t)((N + BN - 1) / BN) * (size_t)M * (size_t)R2 * sizeof(float);
}

static int gemm_w4a4_checked(const svdq_gemm_args &a, void *stream) {
    if (a.dtype != SVDQ_BF16 && a.dtype != SVDQ_FP16) {
        set_error("svdq_gemm_w4a4: dtype %d", a.dtype);
        return SVDQ_E_INVALID;
    }
    if (a.M < 0 || a.N <= 0 || a.K <= 0 || a.K % GROUP || a.N % 8) {
        set_error("svdq_gemm_w4a4: M=%d N=%d K=%d needs K %% 64 == 0 and N %% 8 == 0", a.M, a.N, a.K);
        return SVDQ_E_INVALID;
    }
    if (!a.act || (!a.wgt && !a.wgt_planes) || !a.ascales || !a.wscales) {
        set_error("svdq_gemm_w4a4: act, wgt (or wgt_planes), ascales and wscales are required");
        return SVDQ_E_INVALID;
    }
    if (a.wgt_planes && !al16(a.wgt_planes)) {
        set_error("svdq_gemm_w4a4: wgt_planes must be 16-byte aligned");
        return SVDQ_E_INVALID;
    }
    if (a.act_blocked < 0 || a.act_blocked > 2) {
        set_error("svdq_gemm_w4a4: act_blocked=%d (0: the (M, K / 2) matrix, 1: its bytes in lane order, 2: fp6 codes in lane order)",
                  a.act_blocked);
        return SVDQ_E_INVALID;
    }
    if (a.act_blocked && !a.wgt_planes) {
        set_error("svdq_gemm_w4a4: act_blocked needs wgt_planes (the int8 main loop reads the (M, K / 2) matrix only)");
        return SVDQ_E_UNSUPPORTED;
    }
    if (!al16(a.act) || (!a.act_blocked && (a.ld_act % 16 || a.ld_act < a.K / 2)) ||
        (!a.wgt_planes && (!al16(a.wgt) || a.ld_wgt % 16 || a.ld_wgt < a.K / 2))) {  // wgt is not read next to wgt_planes
        set_error("svdq_gemm_w4a4: act/wgt rows must be 16-byte aligned and at least K/2 bytes (ld_act=%d ld_wgt=%d)",
                  a.ld_act, a.ld_wgt);
        return SVDQ_E_INVALID;
    }
    if (a.ascales_blocked && (a.act_blocked != 2 || a.K % 512 || !al16(a.ascales))) {
        set_error("svdq_gemm_w4a4: ascales_blocked needs act_blocked = 2, K %% 512 == 0 (K=%d) and 16-byte aligned ascales", a.K);
        return a.act_blocked != 2 ? SVDQ_E_UNSUPPORTED : SVDQ_E_INVALID;
    }
    if ((!a.ascales_blocked && a.ld_ascales < a.M) || a.ld_wscales < a.N) {
        set_error("svdq_gemm_w4a4: scale rows shorter than M / N");
        return SVDQ_E_INVALID;
    }
    {   // the kernel addresses operands with 32-bit offsets from a tile's base
        const size_t lim = (size_t)1 << 32, G = (size_t)(a.K / GROUP);
        if (G * a.ld_ascales * 2 >= lim || G * a.ld_wscales * 2 >= lim || (size_t)(BM + 1) * a.ld_act >= lim ||
            (!a.wgt_planes && (size_t)(BN + 1) * a.ld_wgt >= lim) ||
            (a.wgt_planes && (size_t)(G / 2 + 2) * (WPL_BLOCKS * BLK_BYTES) >= lim)) {
            set_error("svdq_gemm_w4a4: K=%d with row strides %d / %d / %d / %d: operands too large for 32-bit offsets", a.K,
                      a.ld_act, a.ld_wgt, a.ld_ascales, a.ld_wscales);
            return SVDQ_E_UNSUPPORTED;
        }
    }
    if (a.R < 0 || a.R % 16 || (a.R > 0 && (!a.lora_act || !a.lora_up))) {
        set_error("svdq_gemm_w4a4: R=%d must be a multiple of 16 with lora_act and lora_up given", a.R);
        return SVDQ_E_INVALID;
    }
    if (a.R > 0 && (!al16(a.lora_act) || !al16(a.lora_up) || a.ld_lora_act % 4 || a.ld_lora_up % 8 ||
                    a.ld_lora_act < a.R || a.ld_lora_up < a.R)) {
        set_error("svdq_gemm_w4a4: LoRA rows must be 16-byte aligned");
        return SVDQ_E_INVALID;
    }
    if (a.bias && ((uintptr_t)a.bias & 7)) {
        set_error("svdq_gemm_w4a4: bias must be 8-byte aligned");
        return SVDQ_E_INVALID;
    }
    if (a.actual_m < 0 || a.actual_m > a.M) {
        set_error("svdq_gemm_w4a4: actual_m=%d outside [0, M=%d]", a.actual_m, a.M);
        return SVDQ_E_INVALID;
    }
    const bool quant = a.epilogue == SVDQ_EPI_GELU_QUANT || a.epilogue == SVDQ_EPI_SWIGLU_QUANT;
    if (!quant && !a.out) {
        set_error("svdq_gemm_w4a4: out is required for this epilogue");
        return SVDQ_E_INVALID;
    }
    if (a.out && (!al16(a.out) || a.ld_out % 8 || a.ld_out < a.N)) {
        set_error("svdq_gemm_w4a4: out rows must be 16-byte aligned and at least N long (ld_out=%d)", a.ld_out);
        return SVDQ_E_INVALID;
    }
    if (a.epilogue == SVDQ_EPI_QK_NORM_ROPE) {
        if (a.N % 3 || (a.N / 3) % 128) {
            set_error("svdq_gemm_w4a4: N=%d is not three whole sets of 128-wide heads", a.N);
            return SVDQ_E_INVALID;
        }
        if (!a.norm_q || !a.norm_k || !a.rotary || ((uintptr_t)a.norm_q & 7) || ((uintptr_t)a.norm_k & 7) ||
            !al16(a.rotary) || a.ld_rotary % 4 || a.ld_rotary < 128) {
            set_error("svdq_gemm_w4a4: norm_q, norm_k (128,) and rotary (actual_m, 128) fp32 16-byte aligned rows are required");
            return SVDQ_E_INVALID;
        }
        if (a.rotary_blocked && !al16(a.rotary_blocked)) {
            set_error("svdq_gemm_w4a4: rotary_blocked must be 16-byte aligned");
            return SVDQ_E_INVALID;
        }
    } else if (quant) {
        const int NQ = a.epilogue == SVDQ_EPI_SWIGLU_QUANT ? a.N / 2 : a.N;
        if (a.N % 128 || a.M % 16) {
            set_error("svdq_gemm_w4a4: the requantizing epilogues need N %% 128 == 0 and M %% 16 == 0 (M=%d N=%d)", a.M, a.N);
            return SVDQ_E_INVALID;
        }
        if (a.epilogue == SVDQ_EPI_SWIGLU_QUANT && a.out) {
            set_error("svdq_gemm_w4a4: the SwiGLU epilogue writes qout/oscales only; out must be NULL");
            return SVDQ_E_INVALID;
        }
        if (a.qout_blocked < 0 || a.qout_blocked > 2) {
            set_error("svdq_gemm_w4a4: qout_blocked=%d (0: the (M, N / 2) matrix, 1: its bytes in lane order, 2: fp6 codes in lane order)",
                      a.qout_blocked);
            return SVDQ_E_INVALID;
        }
        if (!a.qout || !a.oscales || ((uintptr_t)a.qout & (a.qout_blocked ? 15 : 7)) ||
            (!a.qout_blocked && (a.ld_qout % 8 || a.ld_qout < NQ / 2)) || (!a.oscales_blocked && a.ld_oscales < a.M)) {
            set_error("svdq_gemm_w4a4: qout (8-byte aligned rows) and oscales are required");
            return SVDQ_E_INVALID;
        }
        if (a.oscales_blocked && (NQ % 512 || !al16(a.oscales))) {
            set_error("svdq_gemm_w4a4: oscales_blocked needs %d requantized columns to be a multiple of 512 and 16-byte aligned oscales", NQ);
            return SVDQ_E_INVALID;
        }
        if (a.R2 < 0 || a.R2 % 16 ||
            (a.R2 > 0 && (!a.lora_down_t || !a.lora_act_out || !a.scratch || ((uintptr_t)a.lora_down_t & 7) ||
                          !al16(a.scratch) || !al16(a.lora_act_out) || a.ld_lora_act_out % 4 || a.ld_lora_act_out < a.R2))) {
            set_error("svdq_gemm_w4a4: R2=%d must be a multiple of 16 with lora_down_t, lora_act_out (16-byte aligned rows) and scratch given", a.R2);
            return SVDQ_E_INVALID;
        }
    } else if (a.epilogue != SVDQ_EPI_PLAIN) {
        set_error("svdq_gemm_w4a4: unknown epilogue %d", a.epilogue);
        return SVDQ_E_INVALID;
    }
    if (a.M == 0 || (a.actual_m == 0 && !quant)) return SVDQ_OK;  // nothing to write
    hipStream_t s = (hipStream_t)stream;
    if (a.dtype == SVDQ_BF16) {
        if (a.act_unsigned)
            launch_gemm_epi<BF16, true>(a, s);
        else
            launch_gemm_epi<BF16, false>(a, s);
    } else {
        if (a.act_unsigned)
            launch_gemm_epi<FP16, true>(a, s);
        else
            launch_gemm_epi<FP16, false>(a, s);
    }
    int rc = check_launch("svdq_gemm_w4a4");
    if (rc) return rc;
    if (quant && a.R2 > 0) {
        const int n = a.M * a.R2;
        hipLaunchKernelGGL(lora_part_reduce_kernel, dim3((n / 4 + 63) / 64), dim3(64), 0, s, a.scratch, a.lora_act_out,
                           (a.N + BN - 1) / BN, a.M, a.R2, a.ld_lora_act_out);
        rc = check_launch("svdq_gemm_w4a4 (LoRA-down partial sum)");
    }
    return rc;
}

extern "C" size_t svdq_lora_down_blocked_bytes(int32_t N, int32_t R2) {
    return N <= 0 || R2 <= 0 ? 0 : (size_t)(N / 128) * ((R2 + 31) / 32) * 8 * 1024;
}

extern "C" int svdq_block_lora_down(const void *lora_down_t, void *blocked, int32_t N, int32_t R2, int32_t dtype, void *stream) {
    if (!lora_down_t || !blocked || N <= 0 || N % 128 || R2 <= 0 || R2 % 16 || ((uintptr_t)lora_down_t & 7) || ((uintptr_t)blocked & 15) ||
        (dtype != SVDQ_BF16 && dtype != SVDQ_FP16)) {
        set_error("svdq_block_lora_down: N=%d R2=%d dtype=%d; needs N %% 128 == 0, R2 %% 16 == 0, aligned tensors", N, R2, dtype);
        return SVDQ_E_INVALID;
    }
    const int pieces = (N / 128) * ((R2 + 31) / 32) * 512;
    hipLaunchKernelGGL(block_lora_down_kernel, dim3((pieces + 255) / 256), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)lora_down_t,
                       (v4i *)blocked, N, R2, pieces);
    return check_launch("svdq_block_lora_down");
}

extern "C" size_t svdq_rotary_blocked_bytes(int32_t rows) { return rows <= 0 ? 0 : (size_t)((rows + 31) / 32) * 16 * 1024; }

extern "C" int svdq_block_rotary(const float *rotary, float *blocked, int32_t rows, int32_t ld_rotary, void *stream) {
    if (!rotary || !blocked || rows <= 0 || ld_rotary < 128 || ld_rotary % 4 || ((uintptr_t)rotary & 15) || ((uintptr_t)blocked & 15)) {
        set_error("svdq_block_rotary: rows=%d ld_rotary=%d; needs rows > 0, rows of 128 fp32 with ld_rotary %% 4 == 0, 16-byte aligned tensors", rows, ld_rotary);
        return SVDQ_E_INVALID;
    }
    const int pieces = (rows + 31) / 32 * 1024;
    hipLaunchKernelGGL(block_rotary_kernel, dim3((pieces + 255) / 256), dim3(256), 0, (hipStream_t)stream, rotary, (v4f *)blocked, rows, ld_rotary, pieces);
    return check_launch("svdq_block_rotary");
}

extern "C" int svdq_gemm_w4a4_set_variant(int32_t variant) {
    if (variant < -1 || variant > 1) {
        set_error("svdq_gemm_w4a4_set_variant: %d is not -1 (by tile count), 0 (three workgroups per CU) or 1 (two)", variant);
        return SVDQ_E_INVALID;
    }
    g_f8_variant.store(variant, std::memory_order_relaxed);
    return SVDQ_OK;
}

extern "C" int svdq_gemm_w4a4(const svdq_gemm_args *args, void *stream) {
    if (!args) {
        set_error("svdq_gemm_w4a4: null args");
        return SVDQ_E_INVALID;
    }
    return gemm_w4a4_checked(*args, stream);
}

// ---- the same GEMM for callers that cannot allocate --------------------------------------------------------------
// The LoRA-down partial sums of the requantizing epilogues live in a file-scope device array instead of a buffer the
// caller brings.  In host code the array's name is only a stand-in; its device address is looked up once per device,
// with that device current, and that pointer is what the kernels get.
constexpr size_t STATIC_SCRATCH_BYTES = SVDQ_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
static std::atomic<void *> g_scratch_ptr[MAX_DEVICES];

extern "C" size_t svdq_gemm_w4a4_static_scratch_capacity(void) { return STATIC_SCRATCH_BYTES; }

// Device address of the array on the current device, looked up on first use there (every device holds its own copy).
static int static_scratch_ptr(void **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        set_error("svdq_gemm_w4a4_static_scratch: no current device (or device index above %d)", MAX_DEVICES - 1);
        return SVDQ_E_LAUNCH;
    }
    void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            set_error("svdq_gemm_w4a4_static_scratch: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return SVDQ_E_LAUNCH;
        }
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return SVDQ_OK;
}

extern "C" int svdq_gemm_w4a4_static_scratch_prepare(void) {
    void *ptr = nullptr;
    return static_scratch_ptr(&ptr);
}

extern "C" int svdq_gemm_w4a4_static_scratch(const svdq_gemm_args *args, void *stream) {
    if (!args) {
        set_error("svdq_gemm_w4a4_static_scratch: null args");
        return SVDQ_E_INVALID;
    }
    svdq_gemm_args a = *args;
    const size_t need = svdq_gemm_w4a4_scratch_bytes(a.M, a.N, a.R2, a.epilogue);
    if (need > STATIC_SCRATCH_BYTES) {
        set_error("svdq_gemm_w4a4_static_scratch: M=%d N=%d R2=%d needs %zu bytes of LoRA-down partial sums, the built-in "
                  "buffer holds %zu; use svdq_gemm_w4a4 with a caller-provided scratch", a.M, a.N, a.R2, need,
                  STATIC_SCRATCH_BYTES);
        return SVDQ_E_UNSUPPORTED;
    }
    a.scratch = nullptr;
    if (need > 0) {
        void *ptr = nullptr;
        const int rc = static_scratch_ptr(&ptr);
        if (rc) return rc;
        a.scratch = (float *)ptr;  // every (tile, row, rank) entry the reduction reads is written first: nothing to clear
    }
    return gemm_w4a4_checked(a, stream);
}

extern "C" int svdq_group_acc_i32(const void *act, const void *wgt, int32_t *out, int32_t M, int32_t N, int32_t K,
                                  int32_t ld_act, int32_t ld_wgt, int32_t group, int32_t act_unsigned, int32_t path,
                                  void *stream) {
    if (!act || !wgt || !out || M <= 0 || N <= 0 || K <= 0 || K % GROUP || group < 0 || group >= K / GROUP ||
        !al16(act) || !al16(wgt) || ld_act % 16 || ld_wgt % 16 || path < 0 || path > 1) {
        set_error("svdq_group_acc_i32: bad arguments (M=%d N=%d K=%d group=%d)", M, N, K, group);
        return SVDQ_E_INVALID;
    }
    const dim3 grid((N + 31) / 32, (M + 31) / 32), block(64);
    if (path == 1) {
        if (act_unsigned)
            hipLaunchKernelGGL(group_acc_f8_kernel<true>, grid, block, 0, (hipStream_t)stream, (const uint8_t *)act,
                               (const uint8_t *)wgt, out, M, N, ld_act, ld_wgt, group);
        else
            hipLaunchKernelGGL(group_acc_f8_kernel<false>, grid, block, 0, (hipStream_t)stream, (const uint8_t *)act,
                               (const uint8_t *)wgt, out, M, N, ld_act, ld_wgt, group);
        return check_launch("svdq_group_acc_i32");
    }
    if (act_unsigned)
        hipLaunchKernelGGL(group_acc_kernel<true>, grid, block, 0, (hipStream_t)stream, (const uint8_t *)act,
                           (const uint8_t *)wgt, out, M, N, ld_act, ld_wgt, group);
    else
        hipLaunchKernelGGL(group_acc_kernel<false>, grid, block, 0, (hipStream_t)stream, (const uint8_t *)act,
                           (const uint8_t *)wgt, out, M, N, ld_act, ld_wgt, group);
    return check_launch("svdq_group_acc_i32");
}
