// Matrix x matrix for passes over many tokens (prompts): the same dots as the GEMV, but with every
// weight tile reused for 128 tokens, on the matrix cores.
//
//  * gemm_q8act_kernel: Q4_0 / Q8_0 weight rows x Q8_0 activation rows.  Replaces the
//    Dot<Q4_0,Q8_0> / Dot<Q8_0,Q8_0> loops of OperatorMatMulImpl::execute for ne11 > 1
//    (backend/host/operator/mat.cpp:130-143, backend/host/include/simd/vec_dot.h:42-115 in the Spy
//    tree).  One v_mfma_i32_32x32x32_i8 contracts exactly one 32-element quantization block for a
//    32 x 32 output tile, so the int32 block dots are exact; each is then scaled by
//    h2f(d_w) * h2f(d_x) and accumulated in fp32 like the reference's fma (vec_dot.h:76-79).  The scale
//    products of a tile come from an fp16 MFMA (outer product of the two scale vectors, exact in fp32):
//    matrix and vector instructions of a SIMD were measured to add up rather than overlap here, and the
//    MFMA costs half the cycles of the 16 multiplications it replaces.
//    Nibbles are unpacked to int8 (n - 8) on the way into LDS.
//  * gemm_f16_kernel: fp16 rows x fp16 rows with fp32 accumulation (Dot<FP16,FP16>,
//    vec_dot.h:117-146) for the attention products of a prompt pass: strided left operand (the K cache
//    view, the transposed V cache view), right operand converted to fp16 by the caller.
//
// Both: 256 threads = 2 x 2 waves, 128 x 128 output tile per workgroup, each wave 2 x 2 MFMA tiles
// of 32 x 32; operands double-buffered in LDS with a row stride of 80 bytes (conflict-free for the
// 128-bit fragment reads of 32 consecutive rows).
#include "common.cuh"
#include <stdlib.h>
#include <string.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));

#define GEMM_TILE 128
#define GEMM_SKINNY_MAX_TILES 160 // the 32-row kernel is used up to 64 activation rows and wherever the 128 x 128 tiling would give at most this many workgroups (measured crossover)
#define GEMM_KQ_SMALL_MAX_TILES 768 // Q4_K / Q6_K: the 64 x 64 tiling is used where it gives at most this many workgroups (3 per CU: all resident at once)
#define GEMM_ROWB 80             // bytes per LDS row: 64 payload + 16 pad
#ifndef GEMM_WGS
#define GEMM_WGS 3                // workgroups per CU the tile kernel is compiled for (register budget 512 / GEMM_WGS per lane)
#endif
#ifndef GEMM_PF_Q4_0
#define GEMM_PF_Q4_0 1           // stages of global loads in flight for Q4_0; two (+2-5 % for M >= 11008) no longer fit the register budget of three workgroups per CU next to the 16 registers of the accumulator bias
#endif

// 32-bit word of 4 packed nibbles (already masked to 0..15 per byte) -> 4 int8 of (n - 8)
static __device__ __forceinline__ uint32_t nib_m8(uint32_t lo) { return (lo + 0x78787878u) ^ 0x80808080u; }

// Workgroups of the XCD-aware one-dimensional grid of gemm_q8act_kernel for gx x gy tiles: 8 XCDs x ceil(gx / 4) x ceil(gy / 2), or
// 8 x ceil(gx / 8) x gy for an odd gy
// (the workgroups whose tile falls outside return at once).
static inline int64_t gemm_xcd_grid(int64_t gx, int64_t gy) { const int64_t xt = (gy & 1) ? 1 : 2, xm = 8 / xt; return 8 * ((gx + xm - 1) / xm) * ((gy + xt - 1) / xt); }
// 1 where an XCD's quarter of the gx weight tiles (128 rows of K / 32 blocks each) does not fit its L2 with room to spare
static inline int gemm_t_inner(int64_t gx, int64_t K, int wtype) {      // (sized for the 4 x 2 arrangement)
    return ((gx + 3) / 4) * GEMM_TILE * (K / 32) * (wtype == SPY_HIP_Q4_0 ? 18 : 34) > (3ll << 20);
}

template <int WT>
__global__ __launch_bounds__(256, GEMM_WGS) void gemm_q8act_kernel(const uint8_t *__restrict__ W1, const uint8_t *__restrict__ xq, float *__restrict__ dst1,
                                                            int M, int K, int T, int64_t dst_stride, const uint8_t *__restrict__ W2, float *__restrict__ dst2, int t_inner) {
    // Optionally two weight matrices of the same shape against the same activations in one grid (gate and up): the
    // workgroups of the second follow those of the first, which halves the share of the grid's tail.
    // Workgroup L of the one-dimensional grid runs on XCD L % 8, each with its own L2.  The eight XCDs form a 4 x 2
    // arrangement over (weight tiles, activation tiles) (8 x 1 for an odd number of activation tiles): XCD (mj, ti) takes the
    // weight tiles = mj (mod 4) against the activation tiles = ti (mod 2), so that a weight tile is fetched by two L2s and an activation tile by four (a
    // row-major grid has every L2 fetch all the activations).  Where the XCD's share of the weight matrix is larger than
    // its 4 MB L2 (t_inner), the activation tiles of one weight tile follow each other: the hundred or so workgroups an
    // XCD runs at a time then share a dozen weight tiles and its activation tiles, where the other order streams all its
    // weight tiles through the L2 once per activation tile (measured: 14 times the algorithmic bytes for gate|up, and
    // 5-9 % slower).  Where the share fits (4096 x 4096), weight tiles follow each other (that order is 9 % faster there).
    const int tiles1 = (M + GEMM_TILE - 1) / GEMM_TILE, gx = W2 ? 2 * tiles1 : tiles1, gy = (T + GEMM_TILE - 1) / GEMM_TILE;
    int gbx, gby;
    {
        // an odd number of activation tiles (one, for up to 128 tokens) would leave half of the XCDs short of work: 8 x 1 then
        const int xt = (gy & 1) ? 1 : 2, xm = 8 / xt;
        const int xcd = (int)blockIdx.x & 7, slot = (int)blockIdx.x >> 3, nt = (gy + xt - 1) / xt, nm = (gx + xm - 1) / xm;
        const int sm = t_inner ? slot / nt : slot % nm, stt = t_inner ? slot % nt : slot / nm;
        gbx = sm * xm + (xcd % xm);
        gby = stt * xt + (xcd / xm);
        if (gbx >= gx || gby >= gy) return;
    }
    const bool second = W2 != nullptr && gbx >= tiles1;
    const uint8_t *W = second ? W2 : W1;
    float *dst = second ? dst2 : dst1;
    const int bx = second ? gbx - tiles1 : gbx;
    constexpr int PF = (WT == SPY_HIP_Q4_0) ? GEMM_PF_Q4_0 : 1; // stages of global loads in flight per thread
    constexpr int PAIR_DW = (WT == SPY_HIP_Q4_0) ? 9 : 17;       // dwords per pair of weight blocks
    constexpr int HALF_DW = (WT == SPY_HIP_Q4_0) ? 5 : 9;        // dwords that cover one block of the pair
    __shared__ __attribute__((aligned(16))) uint8_t sA[2][GEMM_TILE * GEMM_ROWB];
    __shared__ __attribute__((aligned(16))) uint8_t sB[2][GEMM_TILE * GEMM_ROWB];
    __shared__ uint16_t sAd[2][2][GEMM_TILE];                                // fp16 block scales [buffer][block of the pair][row]
    __shared__ uint16_t sBd[2][2][GEMM_TILE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const int m0 = bx * GEMM_TILE, t0 = gby * GEMM_TILE;
    const int nstage = K / 64;
    const size_t RBw = (size_t)(K / 32) * (WT == SPY_HIP_Q4_0 ? 18 : 34), RBx = (size_t)(K / 32) * 34;

    // Every thread moves one weight block and one activation block per stage: row tid & 127, block
    // tid >> 7 of the 4-byte aligned block pair (block 0 starts at byte 0, block 1 in the middle of a
    // dword: the dwords that cover it are loaded and the scale / quants picked out with byte selectors that
    // are the same for a whole wave).  Rows beyond the matrix re-read its last row (their outputs are never stored).
    const int lrow = tid & 127, half = __builtin_amdgcn_readfirstlane(tid >> 7);
    const uint32_t qsel = half ? 0x07060504u : 0x05040302u;  // v_perm_b32 selector over {raw[i+1], raw[i]}: quants dword-aligned / starting mid-dword
    const uint32_t dshift = half ? 16 : 0;                    // the fp16 scale sits in the upper / lower half of raw[0]
    const uint32_t *gA = (const uint32_t *)(W + (size_t)min(m0 + lrow, M - 1) * RBw) + half * (HALF_DW - 1);
    const uint32_t *gB = (const uint32_t *)(xq + (size_t)min(t0 + lrow, T - 1) * RBx) + half * 8;
    // Global loads run PF stages ahead of the stage being multiplied (a ring of raw registers): with one
    // stage ahead a workgroup advances one stage per memory round trip, whatever the matrix cores could do.
    uint32_t rawA[PF][HALF_DW], rawB[PF][9];
    auto gload = [&](int slot, int s) {                      // 4-byte aligned: 128-bit loads + one dword
        __builtin_memcpy(rawA[slot], __builtin_assume_aligned(gA + (size_t)s * PAIR_DW, 4), HALF_DW * 4);
        __builtin_memcpy(rawB[slot], __builtin_assume_aligned(gB + (size_t)s * 17, 4), 36);
    };
    auto unpack = [&](int b, int slot) {
        uint32_t q[8];
        if constexpr (WT == SPY_HIP_Q4_0) {
            // {d, qs[16]}: element j = low nibble of qs[j], element j+16 = high nibble (quant.h:25-28); stored as n - 8
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t n = __builtin_amdgcn_perm(rawA[slot][i + 1], rawA[slot][i], qsel);
                q[i] = nib_m8(n & 0x0F0F0F0Fu);
                q[4 + i] = nib_m8((n >> 4) & 0x0F0F0F0Fu);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) q[i] = __builtin_amdgcn_perm(rawA[slot][i + 1], rawA[slot][i], qsel);
        }
        uint4 *ra = (uint4 *)(sA[b] + lrow * GEMM_ROWB + half * 32);
        ra[0] = make_uint4(q[0], q[1], q[2], q[3]); ra[1] = make_uint4(q[4], q[5], q[6], q[7]);
        sAd[b][half][lrow] = (uint16_t)(rawA[slot][0] >> dshift);
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = __builtin_amdgcn_perm(rawB[slot][i + 1], rawB[slot][i], qsel);   // {d, qs[32]} (quant.h:139-142)
        uint4 *rb = (uint4 *)(sB[b] + lrow * GEMM_ROWB + half * 32);
        rb[0] = make_uint4(q[0], q[1], q[2], q[3]); rb[1] = make_uint4(q[4], q[5], q[6], q[7]);
        sBd[b][half][lrow] = (uint16_t)(rawB[slot][0] >> dshift);
    };

    float acc[2][2][16];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // Per block and 32 x 32 tile: the int32 block dots from one int8 MFMA, and the scale products
    // h2f(d_w) * h2f(d_x) of the same tile from one fp16 MFMA whose operands hold the scales at k = 0 and zeros
    // elsewhere (an outer product; fp16 x fp16 is exact in fp32, so these are the bits of the scalar product).
    // That leaves a subtraction (below) and an fma per output on the vector units, which bound this kernel.
    // The block dots are accumulated onto the integer 0x4B400000: as a float that is 12582912 + dot exactly (|dot| <= 32 * 127 * 127
    // < 2^22), and subtracting 12582912 gives float(dot) with a full-rate instruction where a conversion runs at half rate.
    const int k0mask = lane < 32 ? 0xFFFF : 0;
    // (Q4_0 only: the Q8_0 kernel has no 16 registers to spare at three workgroups per CU -- it spilled and ran 15-30 % slower)
    constexpr bool BIAS = WT == SPY_HIP_Q4_0;
    v16i bias;
#pragma unroll
    for (int r = 0; r < 16; r++) bias[r] = BIAS ? 0x4B400000 : 0;
    auto multiply = [&](int b) {
#pragma unroll 1
        for (int blk = 0; blk < 2; blk++) {
            v4i fa[2], fb[2];
            v4h ha[2], hb[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                fa[i] = *(const v4i *)(sA[b] + (wm * 64 + i * 32 + (lane & 31)) * GEMM_ROWB + blk * 32 + (lane >> 5) * 16);
                fb[i] = *(const v4i *)(sB[b] + (wn * 64 + i * 32 + (lane & 31)) * GEMM_ROWB + blk * 32 + (lane >> 5) * 16);
                const int da = sAd[b][blk][wm * 64 + i * 32 + (lane & 31)];
                const int dx = sBd[b][blk][wn * 64 + i * 32 + (lane & 31)] & k0mask;             // lanes 32..63 carry k = 4..7: zero
                ha[i] = __builtin_bit_cast(v4h, v2i{da, 0});
                hb[i] = __builtin_bit_cast(v4h, v2i{dx, 0});
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    v16f zf = {0};
                    const v16i I = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], bias, 0, 0, 0);
                    const v16f S = __builtin_amdgcn_mfma_f32_32x32x8f16(ha[i], hb[j], zf, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[i][j][r] = fmaf(S[r], BIAS ? __int_as_float(I[r]) - 12582912.0f : (float)I[r], acc[i][j][r]);
                }
        }
    };

#pragma unroll
    for (int j = 0; j < PF; j++) gload(j, min(j, nstage - 1));
    unpack(0, 0);
    __syncthreads();
    for (int s0 = 0; s0 < nstage; s0 += PF) {
#pragma unroll
        for (int j = 0; j < PF; j++) {
            const int s = s0 + j;                              // stage in LDS buffer s & 1; its raw registers (slot j) are free
            if (s < nstage) {
                gload(j, min(s + PF, nstage - 1));      // unconditional: the last stages re-read the last one
                multiply(s & 1);
                if (s + 1 < nstage) unpack((s & 1) ^ 1, (j + 1) % PF);
                __syncthreads();
            }
        }
    }
    // C layout of the 32x32 MFMA: lane -> column (token) lane & 31; register r -> row (r / 4) * 8 + (lane >> 5) * 4 + (r & 3)
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int t = t0 + wn * 64 + j * 32 + (lane & 31);
            if (t < T) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int m = m0 + wm * 64 + i * 32 + g * 8 + (lane >> 5) * 4;
                    float *o = dst + (size_t)t * dst_stride + m;
                    if (m + 3 < M && (((uintptr_t)o) & 15) == 0) *(float4 *)o = make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
                    else {
#pragma unroll
                        for (int e = 0; e < 4; e++) if (m + e < M) o[e] = acc[i][j][4 * g + e];
                    }
                }
            }
        }
}

// ---- few activation rows (16 .. 128 tokens) ----------------------------------------------------------
// The 128 x 128 tile leaves most of the part idle when T is small (M / 128 workgroups, most of each tile
// padding).  Here a workgroup owns 32 weight rows and its 4 waves work independently of each other: wave =
// (token sub-tile of 32) x (contiguous slice of K), NTW x KS = 4.  A wave copies a chunk of 8 blocks of its
// 32 weight rows and 32 activation rows into its own LDS area with 16-byte loads that run along the rows
// (9 or 17 consecutive lanes per row: a row-per-lane pattern would touch 64 cache lines per instruction),
// one chunk ahead in registers; lane (row = lane & 31, half = lane >> 5) then picks its MFMA fragment out of
// the raw blocks (4-byte aligned LDS reads + a 16-bit funnel shift where a block starts mid-dword).  The weight
// scales of the 32 rows go through a wave-private LDS line so that a lane can read those of its 16
// accumulator rows.  No workgroup barrier until the K slices are summed (through LDS, in a fixed order).
#define GSK_CH 8                  // blocks per chunk (K % 256 == 0)
template <int WT> struct gsk_traits {
    static constexpr int WBLK = (WT == SPY_HIP_Q4_0) ? 18 : 34;
    static constexpr int WP = GSK_CH * WBLK / 16;                        // 16-byte pieces per weight row and chunk: 9 / 17
    static constexpr int WS = (WT == SPY_HIP_Q4_0) ? 176 : 272;          // LDS row strides: 16-byte aligned, 2-way bank conflicts at worst
    static constexpr int XP = 17, XS = 272;
    static constexpr int NWI = (32 * WP + 63) / 64, NXI = (32 * XP + 63) / 64;
    static constexpr int WAVE_LDS = 32 * WS + 32 * XS + GSK_CH * 128;   // weights, activations, weight scales [block][row]
};
// 16 int8 of half `kh` of Q8_0 block bb (34 bytes each, chunk-relative) of an LDS row, and the block's scale
static __device__ __forceinline__ void gsk_frag_q8(const uint8_t *row, int bb, int kh, v4i &q, float &d) {
    if ((bb & 1) == 0) {                                   // block at 34 bb = 0 mod 4: quants start mid-dword
        const uint32_t *p = (const uint32_t *)(row + 34 * bb + 16 * kh);
        const uint32_t w0 = p[0], w1 = p[1], w2 = p[2], w3 = p[3], w4 = p[4];
        q = v4i{(int)__builtin_amdgcn_alignbit(w1, w0, 16), (int)__builtin_amdgcn_alignbit(w2, w1, 16),
                (int)__builtin_amdgcn_alignbit(w3, w2, 16), (int)__builtin_amdgcn_alignbit(w4, w3, 16)};
        d = h2f((uint16_t)(*(const uint32_t *)(row + 34 * bb) & 0xFFFFu));
    } else {                                               // block at 34 bb = 2 mod 4: quants dword-aligned
        const uint32_t *p = (const uint32_t *)(row + 34 * bb + 2 + 16 * kh);
        q = v4i{(int)p[0], (int)p[1], (int)p[2], (int)p[3]};
        d = h2f((uint16_t)(*(const uint32_t *)(row + 34 * bb - 2) >> 16));
    }
}
template <int WT, int NTW>
__global__ __launch_bounds__(256, 2) void gemm_skinny_kernel(const uint8_t *__restrict__ W, const uint8_t *__restrict__ xq, float *__restrict__ dst,
                                                          int M, int K, int T, int64_t dst_stride) {
    using TR = gsk_traits<WT>;
    constexpr int KS = 4 / NTW;
    extern __shared__ __attribute__((aligned(16))) uint8_t gsk_smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), tw = wave % NTW, ks = wave / NTW;
    const int row = lane & 31, kh = lane >> 5;
    const int m0 = blockIdx.x * 32, t0 = blockIdx.y * (32 * NTW) + tw * 32;
    const int nblk = K / 32, nchunk = nblk / GSK_CH;
    const int c_begin = ks * nchunk / KS, c_end = (ks + 1) * nchunk / KS;
    uint8_t *sw = gsk_smem + (size_t)wave * TR::WAVE_LDS, *sx = sw + 32 * TR::WS;
    float *s_dw = (float *)(sx + 32 * TR::XS);
    const size_t RBw = (size_t)nblk * TR::WBLK, RBx = (size_t)nblk * 34;

    // piece p = lane + 64 i of the chunk: row p / WP, 16 bytes at column p % WP (clamped: the last lanes repeat the last piece)
    uint4 rw[TR::NWI], rx[TR::NXI];
    int wofs[TR::NWI], xofs[TR::NXI];
    uint32_t wgo[TR::NWI], xgo[TR::NXI];                    // byte offsets into W / xq (the launcher checks that they fit)
#pragma unroll
    for (int i = 0; i < TR::NWI; i++) {
        const int p = min(lane + 64 * i, 32 * TR::WP - 1), r = p / TR::WP, c = p - r * TR::WP;
        wofs[i] = r * TR::WS + c * 16;
        wgo[i] = (uint32_t)((size_t)min(m0 + r, M - 1) * RBw + c * 16);
    }
#pragma unroll
    for (int i = 0; i < TR::NXI; i++) {
        const int p = min(lane + 64 * i, 32 * TR::XP - 1), r = p / TR::XP, c = p - r * TR::XP;
        xofs[i] = r * TR::XS + c * 16;
        xgo[i] = (uint32_t)((size_t)min(t0 + r, T - 1) * RBx + c * 16);
    }
    auto gload = [&](int c) {
        const uint8_t *wb = W + (size_t)c * (GSK_CH * TR::WBLK), *xb = xq + (size_t)c * (GSK_CH * 34);
#pragma unroll
        for (int i = 0; i < TR::NWI; i++) { uint4 v; __builtin_memcpy(&v, __builtin_assume_aligned(wb + wgo[i], 2), 16); rw[i] = v; }
#pragma unroll
        for (int i = 0; i < TR::NXI; i++) { uint4 v; __builtin_memcpy(&v, __builtin_assume_aligned(xb + xgo[i], 2), 16); rx[i] = v; }
    };
    float acc[16];
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;
    if (c_begin < c_end) gload(c_begin);
    for (int c = c_begin; c < c_end; c++) {
#pragma unroll
        for (int i = 0; i < TR::NWI; i++) *(uint4 *)(sw + wofs[i]) = rw[i];
#pragma unroll
        for (int i = 0; i < TR::NXI; i++) *(uint4 *)(sx + xofs[i]) = rx[i];
        gload(min(c + 1, c_end - 1));                        // unconditional: the last chunk re-reads itself
        // weight scales of the chunk as floats [block][row], written once per chunk (half kh takes blocks 4 kh .. 4 kh + 3)
#pragma unroll
        for (int j = 0; j < GSK_CH / 2; j++) {
            const int bb = kh * (GSK_CH / 2) + j;
            const uint32_t dd = *(const uint32_t *)(sw + row * TR::WS + bb * TR::WBLK - ((j & 1) ? 2 : 0));
            s_dw[bb * 32 + row] = h2f((uint16_t)((j & 1) ? dd >> 16 : dd & 0xFFFFu));
        }
#pragma unroll 1
        for (int bp = 0; bp < GSK_CH / 2; bp++) {             // block pairs: the even block starts dword-aligned, the odd one mid-dword
            const uint8_t *wr = sw + row * TR::WS + bp * (2 * TR::WBLK), *xr = sx + row * TR::XS + bp * 68;
#pragma unroll
            for (int bb = 0; bb < 2; bb++) {
                v4i fa, fb;
                float dwf = 0.0f, dxf;
                gsk_frag_q8(xr, bb, kh, fb, dxf);
                if constexpr (WT == SPY_HIP_Q4_0) {
                    // {d, qs[16]}: element j = low nibble of qs[j], element j + 16 = high nibble (quant.h:25-28)
                    uint32_t n0, n1, n2, n3;
                    if (bb == 0) {
                        const uint32_t *p = (const uint32_t *)wr;
                        const uint32_t w0 = p[0], w1 = p[1], w2 = p[2], w3 = p[3], w4 = p[4];
                        n0 = __builtin_amdgcn_alignbit(w1, w0, 16); n1 = __builtin_amdgcn_alignbit(w2, w1, 16);
                        n2 = __builtin_amdgcn_alignbit(w3, w2, 16); n3 = __builtin_amdgcn_alignbit(w4, w3, 16);
                    } else {
                        const uint32_t *p = (const uint32_t *)(wr + 16);
                        n0 = p[1]; n1 = p[2]; n2 = p[3]; n3 = p[4];
                    }
                    const int sh = kh * 4;
                    fa = v4i{(int)nib_m8((n0 >> sh) & 0x0F0F0F0Fu), (int)nib_m8((n1 >> sh) & 0x0F0F0F0Fu),
                             (int)nib_m8((n2 >> sh) & 0x0F0F0F0Fu), (int)nib_m8((n3 >> sh) & 0x0F0F0F0Fu)};
                } else gsk_frag_q8(wr, bb, kh, fa, dwf);
                (void)dwf;
                v16i z = {0};
                const v16i I = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, z, 0, 0, 0);
                float dw[16];
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const float4 v = *(const float4 *)&s_dw[(2 * bp + bb) * 32 + g * 8 + kh * 4];
                    dw[4 * g] = v.x; dw[4 * g + 1] = v.y; dw[4 * g + 2] = v.z; dw[4 * g + 3] = v.w;
                }
#pragma unroll
                for (int r = 0; r < 16; r++) acc[r] = fmaf(dw[r] * dxf, (float)I[r], acc[r]);
            }
        }
    }
    if constexpr (KS > 1) {
        // the slices of K meet in the waves with ks == 0: the others park their sums in their own (now idle) LDS area
        float *park = (float *)sw;
        if (ks > 0) {
#pragma unroll
            for (int r = 0; r < 16; r++) park[r * 64 + lane] = acc[r];
        }
        __syncthreads();
        if (ks > 0) return;
#pragma unroll
        for (int k = 1; k < KS; k++) {
            const float *other = (const float *)(gsk_smem + (size_t)(k * NTW + tw) * TR::WAVE_LDS);
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r] += other[r * 64 + lane];
        }
    }
    // C layout of the 32x32 MFMA: lane -> column (token) lane & 31; register r -> row (r / 4) * 8 + (lane >> 5) * 4 + (r & 3)
    const int t = t0 + row;
    if (t < T) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int m = m0 + g * 8 + kh * 4;
            float *o = dst + (size_t)t * dst_stride + m;
            if (m + 3 < M && (((uintptr_t)o) & 15) == 0) *(float4 *)o = make_float4(acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]);
            else {
#pragma unroll
                for (int e = 0; e < 4; e++) if (m + e < M) o[e] = acc[4 * g + e];
            }
        }
    }
}

template <int WT, int NTW>
static int launch_gemm_skinny_ntw(hipStream_t st, const void *w, const void *xq, float *dst, int64_t M, int64_t K, int64_t T, int64_t dst_stride) {
    auto kern = gemm_skinny_kernel<WT, NTW>;
    constexpr size_t lds = 4 * (size_t)gsk_traits<WT>::WAVE_LDS;
    { const int rc_ = spy_raise_lds_limit((const void *)kern, lds); if (rc_) return rc_; }
    kern<<<dim3((unsigned)((M + 31) / 32), (unsigned)((T + 32 * NTW - 1) / (32 * NTW))), dim3(256), lds, st>>>(
        (const uint8_t *)w, (const uint8_t *)xq, dst, (int)M, (int)K, (int)T, dst_stride);
    return SPY_LAUNCH_RC();
}
template <int WT>
static int launch_gemm_skinny(hipStream_t st, const void *w, const void *xq, float *dst, int64_t M, int64_t K, int64_t T, int64_t dst_stride) {
    // Token sub-tiles per workgroup (the other waves split K): as many as still leave two workgroups per compute unit.  A wave
    // advances one chunk of K per memory round trip, so with few workgroups (4096 rows x 128 tokens: 128) the launch is a chain
    // of K / 256 round trips on half of the compute units; splitting K four ways instead gives 512 workgroups a quarter as long.
    const int64_t rows = (M + 31) / 32, want = 512;
    if (T <= 32) return launch_gemm_skinny_ntw<WT, 1>(st, w, xq, dst, M, K, T, dst_stride);
    if (T > 64 && rows * ((T + 127) / 128) >= want) return launch_gemm_skinny_ntw<WT, 4>(st, w, xq, dst, M, K, T, dst_stride);
    if (T <= 64 || rows * ((T + 63) / 64) >= want) return launch_gemm_skinny_ntw<WT, 2>(st, w, xq, dst, M, K, T, dst_stride);
    return launch_gemm_skinny_ntw<WT, 1>(st, w, xq, dst, M, K, T, dst_stride);
}

// ---- K-quant weights ---------------------------------------------------------------------------------
// Same tiling.  A stage is a quarter super-block (64 elements), a thread unpacks one 32-element half of it:
//   Q4_K: sub-block a = 2j + half of the super-block: nibbles 0..15 as int8, scale d*sc and minimum dmin*m;
//         value = d*sc*q - dmin*m, so the tile gets  dx * (d*sc * I - dmin*m * sum(q_x))  per block, with
//         dx * sum(q_x) prepared once per activation block.  The minimum terms are an outer product over the
//         block index: one fp32 MFMA per tile and stage adds those of both blocks (k = block of the pair).
//   Q6_K: 32 elements l + 32 m (m = 2 (j & 1) + half) of half n = j >> 1: (q - 32) as int8; they span TWO
//         16-element scale groups, which the 32x32x32 MFMA keeps apart when the right operand is zeroed in
//         one lane half (lanes 0..31 carry k = 0..15, lanes 32..63 k = 16..31): two MFMAs, I_lo and I_hi,
//         combined as integers sc_lo * I_lo + sc_hi * I_hi, then scaled by dx * d.
static __device__ __forceinline__ void q4k_sc_m(const uint32_t h1, const uint32_t h2, const uint32_t h3, int a, int &sc, int &mn) {
    auto byte = [&](int k) -> uint32_t { const uint32_t w = k < 4 ? h1 : (k < 8 ? h2 : h3); return (w >> (8 * (k & 3))) & 0xFFu; };
    if (a < 4) { sc = byte(a) & 63; mn = byte(a + 4) & 63; }
    else { sc = (byte(a + 4) & 0x0F) | ((byte(a - 4) >> 6) << 4); mn = (byte(a + 4) >> 4) | ((byte(a) >> 6) << 4); }
}

template <bool Q4K> struct kq_scale { typedef float type; };
template <> struct kq_scale<false> { typedef uint16_t type; };
// NI x NI MFMA tiles of 32 x 32 per wave: 2 = the 128 x 128 workgroup tile; 1 = a 64 x 64 tile for shapes that would give the
// large tile too few workgroups to fill the part (waves 0-1 then move the weights, waves 2-3 the activations).
template <int WT, int NI>
__global__ __launch_bounds__(256, NI == 2 ? 2 : 3) void gemm_kq_kernel(const uint8_t *__restrict__ W, const uint8_t *__restrict__ xq, float *__restrict__ dst,
                                                         int M, int K, int T, int64_t dst_stride) {
    constexpr bool Q4K = (WT == SPY_HIP_Q4_K);
    constexpr int RAW = Q4K ? 12 : 18;
    constexpr int TILE = 64 * NI, WT32 = 32 * NI;        // rows of the workgroup tile / of a wave's part of it
    __shared__ __attribute__((aligned(16))) uint8_t sA[2][TILE * GEMM_ROWB];
    __shared__ __attribute__((aligned(16))) uint8_t sB[2][TILE * GEMM_ROWB];
    using scale_t = typename kq_scale<Q4K>::type;
    __shared__ __attribute__((aligned(16))) scale_t sAd[2][2][TILE];    // Q4_K: d*sc (float)  Q6_K: d (fp16 bits)
    __shared__ __attribute__((aligned(16))) int sAm[2][2][TILE];        // Q4_K: bits of dmin*m Q6_K: sc_lo | sc_hi << 16
    __shared__ __attribute__((aligned(16))) scale_t sBd[2][2][TILE];    // dx (Q4_K: float, Q6_K: fp16 bits)
    __shared__ __attribute__((aligned(16))) float sBs[2][2][TILE];      // dx * sum(q_x)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.x * TILE, t0 = blockIdx.y * TILE;
    const int nstage = K / 64;
    const size_t RBw = (size_t)spy_row_size(WT, K), RBx = (size_t)(K / 32) * 34;
    const int lrow = tid & (TILE - 1), half = NI == 2 ? tid >> 7 : (tid >> 6) & 1;
    const bool doA = NI == 2 || tid < 128, doB = NI == 2 || tid >= 128;   // wave-uniform
    const uint8_t *gA = W + (size_t)min(m0 + lrow, M - 1) * RBw;
    const uint32_t *gB = (const uint32_t *)(xq + (size_t)min(t0 + lrow, T - 1) * RBx) + half * 8;
    uint32_t rawA[RAW], rawB[9];
    auto gload = [&](int s) {
        const int sbi = s >> 2, j = s & 3;
        if (!doA) {
        } else if constexpr (Q4K) {
            const uint8_t *sb = gA + (size_t)sbi * 144;
            const uint4 hdr = *(const uint4 *)sb, q0 = *(const uint4 *)(sb + 16 + 32 * j), q1 = *(const uint4 *)(sb + 32 + 32 * j);
            rawA[0] = hdr.x; rawA[1] = hdr.y; rawA[2] = hdr.z; rawA[3] = hdr.w;
            rawA[4] = q0.x; rawA[5] = q0.y; rawA[6] = q0.z; rawA[7] = q0.w; rawA[8] = q1.x; rawA[9] = q1.y; rawA[10] = q1.z; rawA[11] = q1.w;
        } else {
            const int n = j >> 1, m = 2 * (j & 1) + half;
            const uint8_t *sb = gA + (size_t)sbi * 210;
            uint4 l0, l1, h0, h1;
            __builtin_memcpy(&l0, __builtin_assume_aligned(sb + 64 * n + 32 * (m & 1), 2), 16);
            __builtin_memcpy(&l1, __builtin_assume_aligned(sb + 64 * n + 32 * (m & 1) + 16, 2), 16);
            __builtin_memcpy(&h0, __builtin_assume_aligned(sb + 128 + 32 * n, 2), 16);
            __builtin_memcpy(&h1, __builtin_assume_aligned(sb + 128 + 32 * n + 16, 2), 16);
            rawA[0] = l0.x; rawA[1] = l0.y; rawA[2] = l0.z; rawA[3] = l0.w; rawA[4] = l1.x; rawA[5] = l1.y; rawA[6] = l1.z; rawA[7] = l1.w;
            rawA[8] = h0.x; rawA[9] = h0.y; rawA[10] = h0.z; rawA[11] = h0.w; rawA[12] = h1.x; rawA[13] = h1.y; rawA[14] = h1.z; rawA[15] = h1.w;
            rawA[16] = *(const uint16_t *)(sb + 192 + 8 * n + 2 * m);
            rawA[17] = *(const uint16_t *)(sb + 208);
        }
        if (doB) {
#pragma unroll
            for (int i = 0; i < 9; i++) rawB[i] = gB[(size_t)s * 17 + i];
        }
    };
    auto unpack = [&](int b, int s) {
        const int j = s & 3;
        uint32_t q[8];
        if (!doA) {
        } else if constexpr (Q4K) {
            int sc, mn;
            q4k_sc_m(rawA[1], rawA[2], rawA[3], 2 * j + half, sc, mn);
#pragma unroll
            for (int i = 0; i < 8; i++) q[i] = half ? (rawA[4 + i] >> 4) & 0x0F0F0F0Fu : rawA[4 + i] & 0x0F0F0F0Fu;
            sAd[b][half][lrow] = h2f((uint16_t)(rawA[0] & 0xFFFFu)) * (float)sc;
            sAm[b][half][lrow] = __float_as_int(h2f((uint16_t)(rawA[0] >> 16)) * (float)mn);
        } else {
            const int m = 2 * (j & 1) + half;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const uint32_t lo = (m & 2) ? (rawA[i] >> 4) & 0x0F0F0F0Fu : rawA[i] & 0x0F0F0F0Fu;
                const uint32_t hi = (rawA[8 + i] >> (2 * m)) & 0x03030303u;
                q[i] = (lo | (hi << 4)) + 0x60606060u ^ 0x80808080u;
            }
            sAd[b][half][lrow] = (uint16_t)(rawA[17] & 0xFFFFu);
            sAm[b][half][lrow] = (int)(uint16_t)(int16_t)(int8_t)(rawA[16] & 0xFFu) | ((int)(int8_t)((rawA[16] >> 8) & 0xFFu) << 16);
        }
        if (doA) {
            uint4 *ra = (uint4 *)(sA[b] + lrow * GEMM_ROWB + half * 32);
            ra[0] = make_uint4(q[0], q[1], q[2], q[3]); ra[1] = make_uint4(q[4], q[5], q[6], q[7]);
        }
        if (!doB) return;
        // activations: {d, qs[32]} (quant.h:139-142)
        const uint16_t dxh = (uint16_t)(half ? rawB[0] >> 16 : rawB[0] & 0xFFFFu);
        const float dx = h2f(dxh);
        int bsum = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) { q[i] = half ? rawB[i + 1] : __builtin_amdgcn_alignbit(rawB[i + 1], rawB[i], 16); bsum = __builtin_amdgcn_sdot4((int)q[i], 0x01010101, bsum, false); }
        uint4 *rb = (uint4 *)(sB[b] + lrow * GEMM_ROWB + half * 32);
        rb[0] = make_uint4(q[0], q[1], q[2], q[3]); rb[1] = make_uint4(q[4], q[5], q[6], q[7]);
        if constexpr (Q4K) { sBd[b][half][lrow] = dx; sBs[b][half][lrow] = dx * (float)bsum; }
        else sBd[b][half][lrow] = dxh;
    };

    float acc[NI][NI][16];
#pragma unroll
    for (int i = 0; i < NI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    const int k0mask = lane < 32 ? 0xFFFF : 0;
    gload(0);
    unpack(0, 0);
    __syncthreads();
    for (int s = 0; s < nstage; s++) {
        const int b = s & 1;
        gload(min(s + 1, nstage - 1));
#pragma unroll 1
        for (int blk = 0; blk < 2; blk++) {
            v4i fa[NI], fb[NI];
#pragma unroll
            for (int i = 0; i < NI; i++) {
                fa[i] = *(const v4i *)(sA[b] + (wm * WT32 + i * 32 + (lane & 31)) * GEMM_ROWB + blk * 32 + (lane >> 5) * 16);
                fb[i] = *(const v4i *)(sB[b] + (wn * WT32 + i * 32 + (lane & 31)) * GEMM_ROWB + blk * 32 + (lane >> 5) * 16);
            }
#pragma unroll
            for (int i = 0; i < NI; i++) {
                int am[16];
                if constexpr (!Q4K) {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const int4 u = *(const int4 *)&sAm[b][blk][wm * WT32 + i * 32 + g * 8 + (lane >> 5) * 4];
                        am[4 * g] = u.x; am[4 * g + 1] = u.y; am[4 * g + 2] = u.z; am[4 * g + 3] = u.w;
                    }
                }
                if constexpr (Q4K) {
                    float dw[16];
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const float4 v = *(const float4 *)&sAd[b][blk][wm * WT32 + i * 32 + g * 8 + (lane >> 5) * 4];
                        dw[4 * g] = v.x; dw[4 * g + 1] = v.y; dw[4 * g + 2] = v.z; dw[4 * g + 3] = v.w;
                    }
#pragma unroll
                    for (int j = 0; j < NI; j++) {
                        const float dx = sBd[b][blk][wn * WT32 + j * 32 + (lane & 31)];
                        v16i z = {0};
                        const v16i I = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], z, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++) acc[i][j][r] = fmaf(dw[r] * dx, (float)I[r], acc[i][j][r]);
                    }
                } else {
                    // d (fp16) x dx (fp16) for the whole tile from one fp16 MFMA: scales at k = 0, zeros elsewhere (exact in fp32)
                    const v4h ha = __builtin_bit_cast(v4h, v2i{(int)sAd[b][blk][wm * WT32 + i * 32 + (lane & 31)], 0});
#pragma unroll
                    for (int j = 0; j < NI; j++) {
                        const v4h hb = __builtin_bit_cast(v4h, v2i{(int)sBd[b][blk][wn * WT32 + j * 32 + (lane & 31)] & k0mask, 0});
                        v16i z = {0};
                        v16f zf = {0};
                        const v4i zero4 = {0, 0, 0, 0};
                        const v4i blo = lane < 32 ? fb[j] : zero4, bhi = lane < 32 ? zero4 : fb[j];
                        const v16i Ilo = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], blo, z, 0, 0, 0);
                        const v16i Ihi = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], bhi, z, 0, 0, 0);
                        const v16f S = __builtin_amdgcn_mfma_f32_32x32x8f16(ha, hb, zf, 0, 0, 0);
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            // 24-bit multiplies (full rate): |I| <= 16 * 31 * 127 and the scales are int8
                            const int sv = __mul24((int)(int16_t)(am[r] & 0xFFFF), Ilo[r]) + __mul24(am[r] >> 16, Ihi[r]);
                            acc[i][j][r] = fmaf(S[r], (float)sv, acc[i][j][r]);
                        }
                        __builtin_amdgcn_sched_barrier(0);       // one tile's three MFMA results at a time: two would not fit the register file
                    }
                }
            }
        }
        if constexpr (Q4K) {
            // the minimum terms of the stage's two blocks, -(dmin * m)[row][blk] * (dx * sum q_x)[token][blk], are an outer
            // product over the block index: one fp32 MFMA per tile (k = block of the pair, carried by the lane half)
            // adds both to the accumulators instead of 32 fmas per lane
#pragma unroll
            for (int i = 0; i < NI; i++) {
                const float a2 = -__int_as_float(sAm[b][lane >> 5][wm * WT32 + i * 32 + (lane & 31)]);
#pragma unroll
                for (int j = 0; j < NI; j++) {
                    const float b2 = sBs[b][lane >> 5][wn * WT32 + j * 32 + (lane & 31)];
                    v16f c;
#pragma unroll
                    for (int r = 0; r < 16; r++) c[r] = acc[i][j][r];
                    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a2, b2, c, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[i][j][r] = c[r];
                }
            }
        }
        if (s + 1 < nstage) unpack(b ^ 1, s + 1);
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < NI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++) {
            const int t = t0 + wn * WT32 + j * 32 + (lane & 31);
            if (t < T) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int m = m0 + wm * WT32 + i * 32 + g * 8 + (lane >> 5) * 4;
                    float *o = dst + (size_t)t * dst_stride + m;
                    if (m + 3 < M && (((uintptr_t)o) & 15) == 0) *(float4 *)o = make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
                    else {
#pragma unroll
                        for (int e = 0; e < 4; e++) if (m + e < M) o[e] = acc[i][j][4 * g + e];
                    }
                }
            }
        }
}

extern "C" int spy_hip_gemm_q8_0act(void *stream, int wtype, const void *w_dev, const void *xq_dev, float *dst_dev,
                                    int64_t M, int64_t K, int64_t T, int64_t dst_stride) {
    SPY_CHECK_ARG(w_dev && xq_dev && dst_dev && M > 0 && K > 0 && T > 0 && dst_stride >= M);
    SPY_CHECK_ARG(K % 64 == 0 && ((wtype != SPY_HIP_Q4_K && wtype != SPY_HIP_Q6_K) || K % 256 == 0));
    SPY_CHECK_ARG((M + GEMM_TILE - 1) / GEMM_TILE <= 0x7fffffff && (T + GEMM_TILE - 1) / GEMM_TILE <= 65535);
    const dim3 grid((unsigned)((M + GEMM_TILE - 1) / GEMM_TILE), (unsigned)((T + GEMM_TILE - 1) / GEMM_TILE));
    hipStream_t st = (hipStream_t)stream;
    const char *force = getenv("SPY_HIP_GEMM");           // "tile" / "skinny" / "tile64": measurement switch
    const bool skinny = K % 256 == 0 && M * (K / 32) * 34 < (int64_t)1 << 31 && T * (K / 32) * 34 < (int64_t)1 << 31 && (force ? !strcmp(force, "skinny") : (T <= 64 || (int64_t)grid.x * grid.y <= GEMM_SKINNY_MAX_TILES));
    if (skinny && wtype == SPY_HIP_Q4_0) return launch_gemm_skinny<SPY_HIP_Q4_0>(st, w_dev, xq_dev, dst_dev, M, K, T, dst_stride);
    if (skinny && wtype == SPY_HIP_Q8_0) return launch_gemm_skinny<SPY_HIP_Q8_0>(st, w_dev, xq_dev, dst_dev, M, K, T, dst_stride);
    // K-quant weights against few activation rows: the one-row-per-wave kernels (4 activation rows per pass over the
    // weights) beat the 128 x 128 tile, which leaves most of the part idle there (T = 16: 32 us against 130-230 us)
    if ((wtype == SPY_HIP_Q4_K || wtype == SPY_HIP_Q6_K) && T <= 32 && K <= 12288 && !force)
        return spy_hip_gemv_q8_0act(stream, wtype, w_dev, xq_dev, dst_dev, nullptr, M, K, T, dst_stride);
    const int64_t xgrid = gemm_xcd_grid(grid.x, grid.y);
    SPY_CHECK_ARG((wtype != SPY_HIP_Q4_0 && wtype != SPY_HIP_Q8_0) || xgrid <= 0x7fffffff);
    const int t_inner = gemm_t_inner(grid.x, K, wtype);
    if (wtype == SPY_HIP_Q4_0) gemm_q8act_kernel<SPY_HIP_Q4_0><<<dim3((unsigned)xgrid), dim3(256), 0, st>>>((const uint8_t *)w_dev, (const uint8_t *)xq_dev, dst_dev, (int)M, (int)K, (int)T, dst_stride, nullptr, nullptr, t_inner);
    else if (wtype == SPY_HIP_Q8_0) gemm_q8act_kernel<SPY_HIP_Q8_0><<<dim3((unsigned)xgrid), dim3(256), 0, st>>>((const uint8_t *)w_dev, (const uint8_t *)xq_dev, dst_dev, (int)M, (int)K, (int)T, dst_stride, nullptr, nullptr, t_inner);
    else if (wtype == SPY_HIP_Q4_K || wtype == SPY_HIP_Q6_K) {
        // 64 x 64 tiles where the 128 x 128 tiling gives too few workgroups to fill the part: 1.8-2.9 x faster up to 512 activation
        // rows of the 7B shapes, equal where its own workgroups stop being resident all at once, 30 % slower beyond
        const dim3 grid64((unsigned)((M + 63) / 64), (unsigned)((T + 63) / 64));
        const bool small = force ? !strcmp(force, "tile64") : (int64_t)grid64.x * grid64.y <= GEMM_KQ_SMALL_MAX_TILES;
        SPY_CHECK_ARG(!small || (T + 63) / 64 <= 65535);
        if (wtype == SPY_HIP_Q4_K) {
            if (small) gemm_kq_kernel<SPY_HIP_Q4_K, 1><<<grid64, dim3(256), 0, st>>>((const uint8_t *)w_dev, (const uint8_t *)xq_dev, dst_dev, (int)M, (int)K, (int)T, dst_stride);
            else gemm_kq_kernel<SPY_HIP_Q4_K, 2><<<grid, dim3(256), 0, st>>>((const uint8_t *)w_dev, (const uint8_t *)xq_dev, dst_dev, (int)M, (int)K, (int)T, dst_stride);
        } else {
            if (small) gemm_kq_kernel<SPY_HIP_Q6_K, 1><<<grid64, dim3(256), 0, st>>>((const uint8_t *)w_dev, (const uint8_t *)xq_dev, dst_dev, (int)M, (int)K, (int)T, dst_stride);
            else gemm_kq_kernel<SPY_HIP_Q6_K, 2><<<grid, dim3(256), 0, st>>>((const uint8_t *)w_dev, (const uint8_t *)xq_dev, dst_dev, (int)M, (int)K, (int)T, dst_stride);
        }
    } else return SPY_HIP_EUNSUPPORTED;
    return SPY_LAUNCH_RC();
}

// Two weight matrices of the same type and shape against the same activations (gate and up of a layer): one grid
// where the 128 x 128 tile kernel applies, else two launches.  Same results as two calls of spy_hip_gemm_q8_0act.
int spy_gemm_q8act_pair(hipStream_t st, int wtype, const void *w1, const void *w2, const void *xq, float *dst1, float *dst2,
                        int64_t M, int64_t K, int64_t T, int64_t dst_stride) {
    SPY_CHECK_ARG(w1 && w2 && xq && dst1 && dst2 && M > 0 && K > 0 && T > 0 && dst_stride >= M);
    const int64_t tiles = (M + GEMM_TILE - 1) / GEMM_TILE, ttiles = (T + GEMM_TILE - 1) / GEMM_TILE;
    const bool tile_kernel = (wtype == SPY_HIP_Q4_0 || wtype == SPY_HIP_Q8_0) && K % 64 == 0 && T > 64 && tiles * ttiles > GEMM_SKINNY_MAX_TILES &&
                             2 * tiles <= 0x7fffffff && ttiles <= 65535 && !getenv("SPY_HIP_GEMM");
    if (!tile_kernel) {
        int rc = spy_hip_gemm_q8_0act(st, wtype, w1, xq, dst1, M, K, T, dst_stride);
        return rc ? rc : spy_hip_gemm_q8_0act(st, wtype, w2, xq, dst2, M, K, T, dst_stride);
    }
    const int64_t xgrid = gemm_xcd_grid(2 * tiles, ttiles);
    SPY_CHECK_ARG(xgrid <= 0x7fffffff);
    const int t_inner = gemm_t_inner(2 * tiles, K, wtype);
    if (wtype == SPY_HIP_Q4_0) gemm_q8act_kernel<SPY_HIP_Q4_0><<<dim3((unsigned)xgrid), dim3(256), 0, st>>>((const uint8_t *)w1, (const uint8_t *)xq, dst1, (int)M, (int)K, (int)T, dst_stride, (const uint8_t *)w2, dst2, t_inner);
    else gemm_q8act_kernel<SPY_HIP_Q8_0><<<dim3((unsigned)xgrid), dim3(256), 0, st>>>((const uint8_t *)w1, (const uint8_t *)xq, dst1, (int)M, (int)K, (int)T, dst_stride, (const uint8_t *)w2, dst2, t_inner);
    return SPY_LAUNCH_RC();
}

// ---- fp16 x fp16 -> fp32 ----------------------------------------------------------------------------
// dst[batch][n][m] = sum_k A[batch][m][k] * B[batch][n][k];  A: fp16, k contiguous, row stride a_nb1 and
// batch stride a_nb2 in bytes (16-byte aligned rows); B: fp16 [batch][N][K] contiguous (K % 8 == 0);
// dst: f32, m contiguous, d_nb1 / d_nb2 in bytes.
struct gemm_f16_args {
    const uint8_t *A; const uint16_t *B; uint8_t *dst;
    int M, N, K;
    int64_t a_nb1, a_nb2, d_nb1, d_nb2;
    // causal structure of the attention products of a pass that starts at position `past` (column n = token past + n,
    // which sees positions 0 .. past + n); -1 = none.
    //  skip_past:  rows m are cache positions (scores): tiles whose rows are all beyond what their columns see are not
    //              computed (the softmax that follows never reads them)
    //  klimit_past: the contraction runs over cache positions (probabilities x V^T): it stops where the tile's
    //              probabilities are all zero (adding the zero products would not change a bit)
    int skip_past, klimit_past;
};

__global__ __launch_bounds__(256) void gemm_f16_kernel(gemm_f16_args a) {
    __shared__ __attribute__((aligned(16))) uint8_t sA[2][GEMM_TILE * GEMM_ROWB];     // 128 rows x 32 halfs (+ pad)
    __shared__ __attribute__((aligned(16))) uint8_t sB[2][GEMM_TILE * GEMM_ROWB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.x * GEMM_TILE, n0 = blockIdx.y * GEMM_TILE, bz = blockIdx.z;
    const int K = a.K, n_last = min(n0 + GEMM_TILE - 1, a.N - 1);
    if (a.skip_past >= 0 && m0 > a.skip_past + n_last) return;
    const int nstage = ((a.klimit_past >= 0 ? min(K, a.klimit_past + n_last + 1) : K) + 31) / 32;
    const uint8_t *Ab = a.A + (size_t)bz * a.a_nb2;
    const uint16_t *Bb = a.B + (size_t)bz * a.N * K;
    // each thread moves two 16-byte chunks of A and two of B per stage: chunk c = tid + i*256 -> row c / 4, k-chunk c % 4
    uint4 ra[2], rb[2];
    auto gload = [&](int s) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int c = tid + i * 256, row = c >> 2, kc = c & 3, k = s * 32 + kc * 8;
            const int kk = min(k, K - 8);                                           // unconditional loads; chunks past K are zeroed
            ra[i] = *(const uint4 *)(Ab + (size_t)min(m0 + row, a.M - 1) * a.a_nb1 + (size_t)kk * 2);
            rb[i] = *(const uint4 *)(Bb + (size_t)min(n0 + row, a.N - 1) * K + kk);
            if (k >= K) { ra[i] = make_uint4(0, 0, 0, 0); rb[i] = make_uint4(0, 0, 0, 0); }
        }
    };
    auto stash = [&](int b) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int c = tid + i * 256, row = c >> 2, kc = c & 3;
            *(uint4 *)(sA[b] + row * GEMM_ROWB + kc * 16) = ra[i];
            *(uint4 *)(sB[b] + row * GEMM_ROWB + kc * 16) = rb[i];
        }
    };
    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
    gload(0);
    stash(0);
    __syncthreads();
    for (int s = 0; s < nstage; s++) {
        const int b = s & 1;
        gload(min(s + 1, nstage - 1));
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            v8h fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                fa[i] = *(const v8h *)(sA[b] + (wm * 64 + i * 32 + (lane & 31)) * GEMM_ROWB + ks * 32 + (lane >> 5) * 16);
                fb[i] = *(const v8h *)(sB[b] + (wn * 64 + i * 32 + (lane & 31)) * GEMM_ROWB + ks * 32 + (lane >> 5) * 16);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (s + 1 < nstage) stash(b ^ 1);
        __syncthreads();
    }
    uint8_t *Db = a.dst + (size_t)bz * a.d_nb2;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int n = n0 + wn * 64 + j * 32 + (lane & 31);
            if (n < a.N) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int m = m0 + wm * 64 + i * 32 + g * 8 + (lane >> 5) * 4;
                    float *o = (float *)(Db + (size_t)n * a.d_nb1) + m;
                    if (m + 3 < a.M && (((uintptr_t)o) & 15) == 0) *(float4 *)o = make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
                    else {
#pragma unroll
                        for (int e = 0; e < 4; e++) if (m + e < a.M) o[e] = acc[i][j][4 * g + e];
                    }
                }
            }
        }
}

// used by the MatMul operator for (F16, F16) operands with many right-hand rows
int spy_gemm_f16_launch(hipStream_t st, const void *A, int64_t a_nb1, int64_t a_nb2, const uint16_t *B, void *dst, int64_t d_nb1, int64_t d_nb2,
                        int64_t M, int64_t N, int64_t K, int64_t nbatch, int skip_past, int klimit_past) {
    SPY_CHECK_ARG(A && B && dst && M > 0 && N > 0 && K >= 8 && nbatch > 0 && K % 8 == 0);
    SPY_CHECK_ARG(a_nb1 % 16 == 0 && a_nb2 % 16 == 0 && ((uintptr_t)A & 15) == 0 && ((uintptr_t)B & 15) == 0);
    SPY_CHECK_ARG((N + GEMM_TILE - 1) / GEMM_TILE <= 65535 && nbatch <= 65535);
    gemm_f16_args a;
    a.A = (const uint8_t *)A; a.B = B; a.dst = (uint8_t *)dst; a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.a_nb1 = a_nb1; a.a_nb2 = a_nb2; a.d_nb1 = d_nb1; a.d_nb2 = d_nb2; a.skip_past = skip_past; a.klimit_past = klimit_past;
    gemm_f16_kernel<<<dim3((unsigned)((M + GEMM_TILE - 1) / GEMM_TILE), (unsigned)((N + GEMM_TILE - 1) / GEMM_TILE), (unsigned)nbatch), dim3(256), 0, st>>>(a);
    return SPY_LAUNCH_RC();
}
