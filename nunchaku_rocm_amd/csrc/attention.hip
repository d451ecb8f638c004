// Unmasked scaled-dot-product attention (flash-attention forward) for gfx950, head dimension 128 or 64.
//
// Arithmetic (reference: nunchaku/ops/triton/attention.py:37-169): q is multiplied by scale * log2(e) and rounded to
// the 16-bit type; per block of keys S = q k^T in fp32, online softmax with exp2 (a row reference m and row sum l),
// P rounded to the 16-bit type, O = O * 2^(m_old - m_new) + P v in fp32; at the end O / l, stored as
// (B, Tq, H * 128).  Two choices the mathematics leaves open differ from the reference: the reference m is only moved
// when a row maximum exceeds it by more than 8 (P then lies in (0, 2^8] instead of (0, 1]: the same O / l, since P, O
// and l all carry the same power of two), and l sums the rounded P the matrix instruction sees, not the unrounded one.
//
// How it maps to CDNA4:
//  * Everything is computed transposed.  S^T = K Q^T puts the keys in the MFMA's A operand and the queries in its B
//    operand, so in the 32x32 accumulator a lane owns ONE query (column) and its registers walk the keys: the row
//    maximum and row sum of the softmax are in-lane reductions plus one exchange with lane ^ 32
//    (v_permlane32_swap), and the rescaling of the output accumulator is a per-lane scalar.  O^T = V^T P^T then
//    takes P^T as its B operand straight from those accumulator registers (eight values of a lane are the eight
//    k-slots the operand wants: keys 4 h .. 4 h + 3 and 8 + 4 h .. 8 + 4 h + 3 of a 16-key chunk for the lanes of
//    half h), with no trip through LDS.
//  * The S^T accumulator starts at minus the row reference, so the scores leave the matrix instruction ready for
//    exp2: no subtraction per score.
//  * V is never transposed in memory: K and V tiles (64 keys x 2 D bytes each) stream buffer -> LDS directly
//    (buffer_load_dwordx4 ... lds, whole rows per load, per-lane offsets fixed and the tile chosen by the scalar
//    buffer base, 16-byte chunks XOR-swizzled so that the operand reads are conflict free), two tiles in flight, one
//    barrier per 64 keys; the V^T operand comes out of the V tile through the transposing LDS read of gfx950
//    (ds_read_b64_tr_b16: sixteen lanes pass the addresses of four rows x 16 columns and lane l receives column l
//    of the four rows), two reads per operand.
//  * 256 threads = 4 wavefronts of 32 queries, two workgroups per CU; Q stays in registers (pre-scaled), the output
//    accumulator is D / 2 registers.  A tile is processed as two 32-key halves so that the softmax instructions of one
//    half sit between the matrix instructions of the other (see the pipeline comment in the kernel).
//  * Workgroups of one head run on one XCD (when the head count is a multiple of 8), so K and V of a head are
//    fetched into one L2 only.
#include <type_traits>

#include "svdq_common.h"

namespace svdq {

constexpr int AT_BQ = 128, AT_BK = 64;     // queries per workgroup, keys per tile

// Geometry for head dimension D (128 or 64).  K and V tiles are [key][2 D bytes]; every block load moves 1 KB
// (64 lanes x 16 bytes) = whole rows; 16-byte chunks are XOR-swizzled by the row so that the operand reads touch every
// bank once.  K (32 rows x one chunk per half-wave): rows of 256 bytes by row & 15, rows of 128 bytes (two rows span
// the 64 banks) by row / 2 & 7.  V (a transposing read = 4 rows x 32 bytes per 16 lanes, two such groups with
// neighbouring 32-byte column slots per half-wave): the eight (row, slot) pairs of a half-wave must land in eight
// different 32-byte slots of the 256 bytes the banks span, so the 64-byte quarter of a row is swizzled by row & 3
// (256-byte rows) or the 64-byte half by row / 2 & 1 (128-byte rows, where rows r and r + 1 already differ by half
// the banks).
template <int D>
struct AtGeo {
    static constexpr int NC = D / 16;               // 16-wide k chunks of q k^T = matrix instructions per 32-key half
    static constexpr int NDT = D / 32;              // 32-row d tiles of O^T
    static constexpr int KROW = 2 * D;              // bytes per key row
    static constexpr int KCH = KROW / 16;           // chunks per key row (16 or 8)
    static constexpr int KT_BYTES = AT_BK * KROW;   // K tile
    static constexpr int VT_BYTES = KT_BYTES;       // V tile
    static constexpr int STAGE = KT_BYTES + VT_BYTES;
    static constexpr int LOADS = KT_BYTES / 1024 / 4;  // block loads per wavefront and tile, of K and of V alike
    static constexpr int OPITCH = 2 * D + 16;       // staged output row
    __host__ __device__ static constexpr int kswz(int row) { return KROW == 256 ? (row & 15) : ((row >> 1) & 7); }
    __host__ __device__ static constexpr int vswz(int row) { return KROW == 256 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); }
};

constexpr uint32_t AT_RSRC_FLAGS = 0x00020000;  // raw buffer, 32-bit data format (gfx9 family)

// 16 bytes per lane from a raw buffer (`bytes` long from `base`; reads past it return zero) straight into LDS at
// lds + 16 * lane.  Plain functions, so that the kernel template below calls no target builtin with dependent operands.
__device__ inline __amdgpu_buffer_rsrc_t at_buffer(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)bytes, AT_RSRC_FLAGS);
}
__device__ inline void at_load16_lds(__amdgpu_buffer_rsrc_t r, uint8_t *lds, uint32_t lane_off, uint32_t wave_off) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (SVDQ_AS3 void *)lds, 16, lane_off, wave_off, 0, 0);
}
// four rows x one column of a [row][col] 16-bit matrix in LDS: the sixteen lanes of a group pass the addresses of
// (row r = lane % 16 / 4, columns 4 (lane % 4) .. + 3) and lane l of the group receives column l of rows 0 .. 3
typedef short v4s16 __attribute__((ext_vector_type(4)));
typedef int v2i32 __attribute__((ext_vector_type(2)));
__device__ inline v2i32 at_read_tr(const uint8_t *p) {
    return __builtin_bit_cast(v2i32, __builtin_amdgcn_ds_read_tr16_b64_v4i16((SVDQ_AS3 v4s16 *)p));
}
constexpr float AT_LAZY = 8.0f;                 // the accumulator is rescaled when a row maximum grew by more than this

template <typename T, int D>
__global__ __launch_bounds__(256, 2) void attention_kernel(svdq_attention_args a, int ntile, int xcd_heads) {
    using G = AtGeo<D>;
    constexpr int NC = G::NC, NDT = G::NDT, LOADS = G::LOADS;
    // Two separate LDS objects, one per stage, and a main loop unrolled over them: the compiler then knows that a tile
    // load into one stage cannot touch what is being read from the other.  With one object and a run-time stage offset
    // it made every LDS read wait for all loads in flight, i.e. for the tile that was requested just before.
    static_assert(AT_BQ == 128 && 64 * G::OPITCH <= G::STAGE, "the output tile is staged as two halves of 64 rows, one per stage");
    __shared__ __align__(16) uint8_t smem0[G::STAGE];
    __shared__ __align__(16) uint8_t smem1[G::STAGE];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;
    // workgroup -> (batch * head, query tile).  Workgroups are dealt to the eight XCDs round-robin; when the head count
    // allows it, a head's query tiles all land on one XCD so that its K and V stay in that XCD's L2.
    int bh, qt;
    if (xcd_heads) {
        const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
        bh = (j / ntile) * 8 + xcd;
        qt = j % ntile;
    } else {
        bh = blockIdx.x / ntile;
        qt = blockIdx.x % ntile;
    }
    const int b = bh / a.H, h = bh % a.H;
    const int q0 = qt * AT_BQ;

    // ---- Q^T operand: lane (q, half) holds q[16 c + 8 half, +8) for c < NC, scaled and rounded to T ---------------
    const int qrow = min(q0 + wave * 32 + l32, a.Tq - 1);
    const uint16_t *qp = (const uint16_t *)a.q + (long)b * a.sqb + (long)h * a.sqh + (long)qrow * a.sqm + 8 * half;
    const float qscale = a.scale * 1.4426950408889634f;
    v4i qop[NC];
#pragma unroll
    for (int c = 0; c < NC; c++) {
        const v4i raw = *(const v4i *)(qp + 16 * c);
#pragma unroll
        for (int e = 0; e < 4; e++)
            qop[c][e] = (int)pack2<T>(T::lo_f32((uint32_t)raw[e]) * qscale, T::hi_f32((uint32_t)raw[e]) * qscale);
    }

    // ---- tile loads (buffer -> LDS, 16 bytes per lane): lane l of load i fetches one chunk of key row
    // (64 / KCH) i + l / KCH of K and of V alike.  LOADS K and LOADS V loads per wavefront and tile.  The per-lane
    // offsets never change; the tile is selected by the (scalar) buffer base, and key rows past the end lie outside
    // the buffers' ranges and arrive as zeros.
    const uint8_t *kbase = (const uint8_t *)a.k + ((long)b * a.skb + (long)h * a.skh) * 2;
    const uint8_t *vbase = (const uint8_t *)a.v + ((long)b * a.svb + (long)h * a.svh) * 2;
    const uint32_t kbytes = (uint32_t)(((long)(a.Tkv - 1) * a.skn + D) * 2);
    const uint32_t vbytes = (uint32_t)(((long)(a.Tkv - 1) * a.svn + D) * 2);
    const uint32_t ktile = (uint32_t)(AT_BK * a.skn * 2), vtile = (uint32_t)(AT_BK * a.svn * 2);
    uint32_t kvo[LOADS], vvo[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; j++) {
        const int i = wave * LOADS + j;
        const int row = (64 / G::KCH) * i + lane / G::KCH;
        kvo[j] = (uint32_t)row * (uint32_t)(a.skn * 2) + (uint32_t)(((lane % G::KCH) ^ G::kswz(row)) * 16);
        vvo[j] = (uint32_t)row * (uint32_t)(a.svn * 2) + (uint32_t)(((lane % G::KCH) ^ G::vswz(row)) * 16);
    }
    auto issue_k = [&](int blk, uint8_t *stage, int j) {
        const uint32_t off = (uint32_t)blk * ktile;
        at_load16_lds(at_buffer(kbase + off, kbytes - off), stage + (wave * G::LOADS + j) * 1024, kvo[j], 0);
    };
    auto issue_v = [&](int blk, uint8_t *stage, int j) {
        const uint32_t off = (uint32_t)blk * vtile;
        at_load16_lds(at_buffer(vbase + off, vbytes - off), stage + G::KT_BYTES + (wave * G::LOADS + j) * 1024, vvo[j], 0);
    };

    // operand read offsets.  K rows 32 t + l32 (chunk 2 c + half).  V^T operand of d tile dt and 16-key chunk c: lane
    // (half, dq = lane / 16 % 2, r = lane % 16 / 4, c4 = lane % 4) passes the address of V[16 c + 4 half + r (+ 8 for
    // the second read)][32 dt + 16 dq + 4 c4] and receives d = 32 dt + lane % 32, keys 4 half .. + 3 (8 + 4 half .. + 3)
    int koff[NC], vtoff[NDT];
#pragma unroll
    for (int c = 0; c < NC; c++) koff[c] = l32 * G::KROW + (((2 * c + half) ^ G::kswz(l32)) * 16);
    {
        const int dq = (lane >> 4) & 1, r = (lane & 15) >> 2, c4 = lane & 3, key = 4 * half + r;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
            vtoff[dt] = G::KT_BYTES + key * G::KROW + (((4 * dt + 2 * dq + (c4 >> 1)) ^ G::vswz(key)) * 16) + 8 * (c4 & 1);
    }
    // (keys 16 c + 8 + key have the same swizzle as key: both leave key % 4 and, for 128-byte rows, key / 2 % 2 alone)
    auto read_v = [&](const uint8_t *st, int dt, int c) {
        const v2i32 lo = at_read_tr(st + vtoff[dt] + c * (16 * G::KROW));
        const v2i32 hi = at_read_tr(st + vtoff[dt] + c * (16 * G::KROW) + 8 * G::KROW);
        return v4i{lo[0], lo[1], hi[0], hi[1]};
    };

    v16f acc_o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc_o[dt][i] = 0.0f;
    // Scores come out of the matrix instructions already relative to the row's reference: the accumulator of S^T starts
    // at -bias (cinit), so p = 2^s' with s' = s - bias needs no subtraction.  bias trails the true row maximum by at
    // most AT_LAZY (it only moves when a maximum exceeds it by more than that), which keeps p <= 2^AT_LAZY.
    // The bias itself only lives in cinit; gap = reference - bias: 0 once a reference exists, -inf before the first keys.
    float gap = -INFINITY, l_run = 0.0f;
    v16f cinit;
#pragma unroll
    for (int i = 0; i < 16; i++) cinit[i] = 0.0f;

    const int nblk = (a.Tkv + AT_BK - 1) / AT_BK;
    // Software pipeline.  Tile t lives in stage t & 1 and is handled as two halves of 32 keys, each a complete online-
    // softmax step, so that the softmax arithmetic of one half is issued between the matrix instructions of the other:
    //   (A) S0 = K[0:32] Q^T                            + V^T operand reads (keys 0..31)
    //   (B) S1 = K[32:64] Q^T         ||  softmax(S0)   + V^T operand reads (keys 32..63)
    //   (C) O^T += V^T[:, 0:32] P0^T  ||  softmax(S1)
    //       barrier: tile t + 1 has landed for everybody, nobody reads tile t any more
    //   (D) O^T += V^T[:, 32:64] P1^T                   + K operand reads of tile t + 1, loads of tile t + 2 into
    //                                                     the stage tile t has left
    // The compiler is kept from regrouping the slots (one matrix instruction plus its share of the rest).
#pragma unroll
    for (int j = 0; j < LOADS; j++) issue_k(0, smem0, j);
#pragma unroll
    for (int j = 0; j < LOADS; j++) issue_v(0, smem0, j);
    {
        const int t1 = min(1, nblk - 1);
#pragma unroll
        for (int j = 0; j < LOADS; j++) issue_k(t1, smem1, j);
#pragma unroll
        for (int j = 0; j < LOADS; j++) issue_v(t1, smem1, j);
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * LOADS, 15));  // tile 0 (the older half of the loads)
    __builtin_amdgcn_s_barrier();
    v4i rk[2 * NC], rv[4 * NDT];  // rk[NC t + c]: K rows 32 t.., chunk c;  rv[4 dt + c]: V^T rows 32 dt.., 16-key chunk c
#pragma unroll
    for (int c = 0; c < NC; c++) {
        rk[c] = *(const v4i *)(smem0 + koff[c]);
        rk[NC + c] = *(const v4i *)(smem0 + 32 * G::KROW + koff[c]);
    }

    float shift, alpha, rs;  // rs: this half's row sum, at the new reference
    auto max3 = [](float x, float y, float z) {
        float r;
        asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(y), "v"(z));
        return r;
    };
    // row maximum of one half (16 scores of this lane, 16 of lane ^ 32) relative to the bias; when it exceeds the
    // allowance: shift = how far the reference moves, alpha = the factor that moves the accumulator there (0 before the
    // first keys).  Returns whether any lane of the wavefront moved.
    auto row_max = [&](const v16f &sv) -> bool {
        float mx = max3(sv[0], sv[1], sv[2]);
#pragma unroll
        for (int i = 3; i < 15; i += 2) mx = max3(mx, sv[i], sv[i + 1]);
        mx = max3(mx, sv[15], sv[15]);
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
        mx = max3(__uint_as_float(sw[0]), __uint_as_float(sw[1]), __uint_as_float(sw[1]));
        const bool need = mx > gap + AT_LAZY;
        shift = need ? mx : 0.0f;
        alpha = __builtin_amdgcn_exp2f(need ? gap - mx : 0.0f);
        gap = need ? 0.0f : gap;
        return __builtin_amdgcn_ballot_w64(need) != 0;
    };
    auto shift16 = [&](v16f &sv) {
#pragma unroll
        for (int i = 0; i < 16; i++) sv[i] -= shift;
    };
    // four scores -> two packed P values; the row sum adds what the matrix instruction will see (the rounded P)
    auto exp4 = [&](const v16f &sv, int i0, v4i &pw, int e0) {
        float p[4];
#pragma unroll
        for (int e = 0; e < 4; e++) p[e] = __builtin_amdgcn_exp2f(sv[i0 + e]);
        pw[e0] = (int)pack2<T>(p[0], p[1]);
        pw[e0 + 1] = (int)pack2<T>(p[2], p[3]);
        rs = T::sum2((uint32_t)pw[e0], rs);
        rs = T::sum2((uint32_t)pw[e0 + 1], rs);
    };
    // the reference moved: accumulator and row sum to the new reference, later scores start from the new bias
    auto rescale = [&]() {
        l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < G::NDT; dt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc_o[dt][i] *= alpha;
        shift16(cinit);
    };

    auto tile = [&](auto par_tag, int blk) {  // tile blk, which lives in stage par_tag
        constexpr int PAR = decltype(par_tag)::value;
        uint8_t *st = PAR ? smem1 : smem0;
        const uint8_t *sn = PAR ? smem0 : smem1;
        const int nxt = min(blk + 2, nblk - 1);  // past the end: the last tile again, into a stage nobody reads
        const bool ragged = blk == nblk - 1 && (a.Tkv & (AT_BK - 1));
        v16f s0, s1;
        v4i pop[4];  // P^T operand: chunk cc of half t = accumulator quads 2 cc, 2 cc + 1 of S_t

        // ---- (A) ---------------------------------------------------------------------------------------------------------
#pragma unroll
        for (int c = 0; c < NC; c++) {
            s0 = mfma32_16bit<T>(rk[c], qop[c], c == 0 ? cinit : s0);
            rv[4 * (c % NDT) + c / NDT] = read_v(st, c % NDT, c / NDT);  // chunks 0, 1: keys 0..31
            __builtin_amdgcn_sched_barrier(0);
        }
        if (ragged) {  // keys past the end count as -inf
#pragma unroll
            for (int i = 0; i < 16; i++)
                if (blk * AT_BK + 8 * (i >> 2) + 4 * half + (i & 3) >= a.Tkv) s0[i] = -INFINITY;
        }

        // ---- (B) ---------------------------------------------------------------------------------------------------------
        bool moved = false;
#pragma unroll
        for (int c = 0; c < NC; c++) {
            s1 = mfma32_16bit<T>(rk[NC + c], qop[c], c == 0 ? cinit : s1);
            rv[4 * (c % NDT) + 2 + c / NDT] = read_v(st, c % NDT, 2 + c / NDT);  // keys 32..63
            if (c == 0) {
                moved = row_max(s0);
                rs = 0.0f;
                if (moved) shift16(s0);
            }
#pragma unroll
            for (int j = 0; j < 4; j++)  // the four exp slices go with slots 1 .. 4 (the last slot takes what is left)
                if (c == (1 + j < NC - 1 ? 1 + j : NC - 1)) exp4(s0, 4 * j, pop[j >> 1], 2 * (j & 1));
            __builtin_amdgcn_sched_barrier(0);
        }
        if (moved) {
            shift16(s1);  // computed from the old bias
            rescale();
        }
        l_run += rs;
        if (ragged) {
#pragma unroll
            for (int i = 0; i < 16; i++)
                if (blk * AT_BK + 32 + 8 * (i >> 2) + 4 * half + (i & 3) >= a.Tkv) s1[i] = -INFINITY;
        }
        __builtin_amdgcn_sched_barrier(0);

        // ---- (C) ---------------------------------------------------------------------------------------------------------
#pragma unroll
        for (int c = 0; c < NC; c++) {
            acc_o[c % NDT] = mfma32_16bit<T>(rv[4 * (c % NDT) + c / NDT], pop[c / NDT], acc_o[c % NDT]);
            if (c == 0) {
                moved = row_max(s1);
                rs = 0.0f;
                if (moved) shift16(s1);
            }
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (c == (1 + j < NC - 1 ? 1 + j : NC - 1)) exp4(s1, 4 * j, pop[2 + (j >> 1)], 2 * (j & 1));
            __builtin_amdgcn_sched_barrier(0);
        }
        if (moved) rescale();
        l_run += rs;
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));  // my loads of tile blk + 1 have landed, my reads of tile blk are done
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);

        // ---- (D) ---------------------------------------------------------------------------------------------------------
#pragma unroll
        for (int c = 0; c < NC; c++) {
            acc_o[c % NDT] = mfma32_16bit<T>(rv[4 * (c % NDT) + 2 + c / NDT], pop[2 + c / NDT], acc_o[c % NDT]);
            rk[2 * c] = *(const v4i *)(sn + ((2 * c) / NC) * (32 * G::KROW) + koff[(2 * c) % NC]);
            rk[2 * c + 1] = *(const v4i *)(sn + ((2 * c + 1) / NC) * (32 * G::KROW) + koff[(2 * c + 1) % NC]);
            if (c & 1) issue_k(nxt, st, c >> 1); else issue_v(nxt, st, c >> 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    {
        int blk = 0;
        for (; blk + 1 < nblk; blk += 2) {
            tile(std::integral_constant<int, 0>{}, blk);
            tile(std::integral_constant<int, 1>{}, blk + 1);
        }
        if (blk < nblk) tile(std::integral_constant<int, 0>{}, blk);
    }

    // ---- O = O^T / l, staged through LDS so that rows leave as 256-byte segments -------------------------------------
    l_run += __shfl_xor(l_run, 32);
    const float inv = 1.0f / (l_run == 0.0f ? 1.0f : l_run);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));  // the redundant last tile load has landed
    __syncthreads();
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint2 w;
            w.x = pack2<T>(acc_o[dt][4 * j] * inv, acc_o[dt][4 * j + 1] * inv);
            w.y = pack2<T>(acc_o[dt][4 * j + 2] * inv, acc_o[dt][4 * j + 3] * inv);
            *(uint2 *)((wave < 2 ? smem0 : smem1) + ((wave & 1) * 32 + l32) * G::OPITCH + (32 * dt + 8 * j + 4 * half) * 2) = w;
        }
    __syncthreads();
    uint16_t *op = (uint16_t *)a.o + (long)b * a.sob + (long)h * D;
    constexpr int OCH = D / 8, OROWS = 256 / OCH;  // 16-byte chunks per output row, rows per pass
    const int c = tid % OCH;
#pragma unroll
    for (int pass = 0; pass < AT_BQ / OROWS; pass++) {
        const int row = pass * OROWS + tid / OCH, q = q0 + row;
        if (q < a.Tq) *(v4i *)(op + (long)q * a.som + 8 * c) = *(const v4i *)((row < 64 ? smem0 : smem1) + (row & 63) * G::OPITCH + c * 16);
    }
}

template <typename T, int D>
static void launch_attention(const svdq_attention_args &a, hipStream_t s) {
    const int ntile = (a.Tq + AT_BQ - 1) / AT_BQ;
    const int xcd_heads = (a.B * a.H) % 8 == 0;
    hipLaunchKernelGGL((attention_kernel<T, D>), dim3((unsigned)(ntile * a.H * a.B)), dim3(256), 0, s, a, ntile, xcd_heads);
}

}  // namespace svdq

using namespace svdq;

extern "C" int svdq_attention_fp16(const svdq_attention_args *args, void *stream) {
    if (!args) {
        set_error("svdq_attention_fp16: null args");
        return SVDQ_E_INVALID;
    }
    const svdq_attention_args &a = *args;
    if (a.dtype != SVDQ_BF16 && a.dtype != SVDQ_FP16) {
        set_error("svdq_attention_fp16: dtype %d", a.dtype);
        return SVDQ_E_INVALID;
    }
    if (a.D != 128 && a.D != 64) {
        set_error("svdq_attention_fp16: head dimension %d is not supported (128 and 64 only)", a.D);
        return SVDQ_E_UNSUPPORTED;
    }
    if (a.B <= 0 || a.H <= 0 || a.Tq < 0 || a.Tkv <= 0 || a.B > 65535 || a.H > 65535) {
        set_error("svdq_attention_fp16: bad shape B=%d H=%d Tq=%d Tkv=%d", a.B, a.H, a.Tq, a.Tkv);
        return SVDQ_E_INVALID;
    }
    if (!a.q || !a.k || !a.v || !a.o) {
        set_error("svdq_attention_fp16: null tensor");
        return SVDQ_E_INVALID;
    }
    auto al = [](const void *p) { return ((uintptr_t)p & 15) == 0; };
    if (!al(a.q) || !al(a.k) || !al(a.v) || !al(a.o) || a.sqm % 8 || a.sqh % 8 || a.sqb % 8 || a.skn % 8 ||
        a.skh % 8 || a.skb % 8 || a.svn % 8 || a.svh % 8 || a.svb % 8 || a.som % 8 || a.sob % 8) {
        set_error("svdq_attention_fp16: tensors and their row / head / batch strides must be 16-byte aligned");
        return SVDQ_E_INVALID;
    }
    if (a.Tq == 0) return SVDQ_OK;
    const int Tpad = (a.Tkv + AT_BK - 1) / AT_BK * AT_BK;
    if (((size_t)Tpad * a.svn + a.D) * 2 >= ((size_t)1 << 31) || ((size_t)Tpad * a.skn + a.D) * 2 >= ((size_t)1 << 31) ||
        (size_t)a.B * a.H * ((a.Tq + AT_BQ - 1) / AT_BQ) >= ((size_t)1 << 31)) {
        set_error("svdq_attention_fp16: Tq=%d Tkv=%d key / value stride %lld / %lld: too large for 32-bit tile offsets", a.Tq, a.Tkv,
                  (long long)a.skn, (long long)a.svn);
        return SVDQ_E_UNSUPPORTED;
    }
    if (a.skn < a.D || a.svn < a.D) {
        set_error("svdq_attention_fp16: key or value rows overlap (stride %lld / %lld < head dimension)", (long long)a.skn, (long long)a.svn);
        return SVDQ_E_INVALID;
    }
    hipStream_t s = (hipStream_t)stream;
    if (a.D == 128) {
        if (a.dtype == SVDQ_BF16)
            launch_attention<BF16, 128>(a, s);
        else
            launch_attention<FP16, 128>(a, s);
    } else {
        if (a.dtype == SVDQ_BF16)
            launch_attention<BF16, 64>(a, s);
        else
            launch_attention<FP16, 64>(a, s);
    }
    return check_launch("svdq_attention_fp16");
}
