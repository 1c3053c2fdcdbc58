// Attention of a prompt pass in the host backend's summation order: the three operators
//   KQ = MatMul(K cache, Q)   Dot<FP16,FP16> over the 128 elements of a head   (vec_dot.h:117-146)
//   P  = Softmax(KQ, mask)    table exp, sum in groups of four                  (non-linear.cpp:86-180)
//   O  = MatMul(V^T cache, P) Dot<FP16,FP16> over the cached positions
// as three kernels that leave out what the causal mask removes and keep every float operation that is left in
// the host's order, so the outputs equal those of the operator-by-operator exact path (exact_order.hip) bit for bit:
//   * a masked score is never read, a masked probability is +0: an fma with a +0 factor leaves a finite accumulator
//     unchanged, and (a + 0) in the softmax sum is a;
//   * what still depends on the length n of the whole row is passed in (n_total, the cached positions after the whole
//     call): the host's fp16 dot runs its 32 accumulators over whole chunks of 32 elements while i + 32 < n and adds
//     the last 1..32 elements one by one, and the softmax sum adds the last n % 4 terms one by one.  A call may therefore
//     be cut into chunks of query rows without moving a rounding.
// Values that cannot occur are not looked after: the fp16 caches are written by this library's float -> half
// conversion, which never produces the pattern 0xFFFF that the host's conversion table maps to 0 (conversion.h:39-41).
#include "common.cuh"

namespace {

typedef _Float16 xp_half2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ xp_half2 xp_pack(float a, float b) {
    xp_half2 r;
    r.x = __builtin_bit_cast(_Float16, f2h(a));
    r.y = __builtin_bit_cast(_Float16, f2h(b));
    return r;
}

// ---------------------------------------------------------------- scores
// One workgroup per (head, 128 query rows); a lane takes query rows t0 + lane and t0 + 64 + lane, their 2 x 128 q values
// as packed fp16 pairs in registers.  A tile of 64 key rows is brought into LDS by the whole workgroup; every lane of a
// wave reads the same key row -- LDS delivers that as a broadcast, but
// at the cost of a full read, which is why a key row read serves two query rows per lane: with one, the kernel ran at the
// LDS read rate (16 ds_read_b128 per 160 vector instructions).  A wave takes 16 of the 64 cached positions of a tile; the
// scores go through LDS as well so that the rows of S are written in whole segments.
#define XP_QT 128
#define XP_KSEG 512
// fma(float(lower halves), c) and fma(float(upper halves), c) of two packed fp16 pairs, written out as instructions: left to
// itself the compiler folds only one fp16 source into v_fma_mix_f32 and converts the loop-invariant q values to fp32 (once, which
// doubles the registers they occupy, or inside the loop, which doubles the instructions)
__device__ __forceinline__ float xp_fma_lo(uint32_t a, uint32_t b, float c) {
    float r;
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[1,1,0]" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float xp_fma_hi(uint32_t a, uint32_t b, float c) {
    float r;
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,1,0] op_sel_hi:[1,1,0]" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// One key row (in LDS, 16 x 16 bytes) against the two query rows of a lane; the row is taken in its four chunks of 32 elements
// so that only one chunk of it is in registers at a time.  A: the first query row takes part (else its score is not needed).
template <bool A>
__device__ __forceinline__ void xp_dot128_pair(const uint32_t (&qa)[64], const uint32_t (&qb)[64], const uint4 *kr, float &sa, float &sb) {
    float sum_a[32], sum_b[32];
    // chunks of 32 elements while i + 32 < 128: accumulator l takes elements l, 32 + l, 64 + l
#pragma unroll
    for (int c = 0; c < 3; c++) {
        uint4 k4[4];
#pragma unroll
        for (int v = 0; v < 4; v++) k4[v] = kr[4 * c + v];
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const uint32_t kw[4] = {k4[v].x, k4[v].y, k4[v].z, k4[v].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int l = 8 * v + 2 * i, qi = 16 * c + 4 * v + i;
                if (A) {
                    sum_a[l] = xp_fma_lo(kw[i], qa[qi], c == 0 ? 0.0f : sum_a[l]);
                    sum_a[l + 1] = xp_fma_hi(kw[i], qa[qi], c == 0 ? 0.0f : sum_a[l + 1]);
                }
                sum_b[l] = xp_fma_lo(kw[i], qb[qi], c == 0 ? 0.0f : sum_b[l]);
                sum_b[l + 1] = xp_fma_hi(kw[i], qb[qi], c == 0 ? 0.0f : sum_b[l + 1]);
            }
        }
    }
    // the last 32 elements one by one (their products are exact in fp32, so each step is one fma)
    float tail_a = 0.0f, tail_b = 0.0f;
    {
        uint4 k4[4];
#pragma unroll
        for (int v = 0; v < 4; v++) k4[v] = kr[12 + v];
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const uint32_t kw[4] = {k4[v].x, k4[v].y, k4[v].z, k4[v].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int qi = 48 + 4 * v + i;
                if (A) { tail_a = xp_fma_lo(kw[i], qa[qi], tail_a); tail_a = xp_fma_hi(kw[i], qa[qi], tail_a); }
                tail_b = xp_fma_lo(kw[i], qb[qi], tail_b);
                tail_b = xp_fma_hi(kw[i], qb[qi], tail_b);
            }
        }
    }
    // FP16::block_reduce (vec_util.h:61-71), then result = tail + that sum
    auto reduce = [](float (&sum)[32]) {
#pragma unroll
        for (int l = 0; l < 8; l++) { sum[l] += sum[16 + l]; sum[8 + l] += sum[24 + l]; }
#pragma unroll
        for (int l = 0; l < 8; l++) sum[l] += sum[8 + l];
        const float u0 = sum[0] + sum[4], u1 = sum[1] + sum[5], u2 = sum[2] + sum[6], u3 = sum[3] + sum[7];
        return (u0 + u1) + (u2 + u3);
    };
    if (A) sa = tail_a + reduce(sum_a);
    sb = tail_b + reduce(sum_b);
}

__global__ __launch_bounds__(256, 2) void xp_scores_kernel(const float *__restrict__ q, const uint16_t *__restrict__ kc, float *__restrict__ S,
                                                           int T, int H, int P, int64_t s_row) {
    __shared__ float s_tile[XP_QT][65];
    __shared__ __align__(16) uint4 s_k[64][16];                  // 64 key rows of 256 bytes
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // The head is the fastest-running index of the grid: consecutive workgroups go to the eight XCDs in turn, and with the query tile
    // there an XCD would get tiles k and k + 8 of 16 only -- under the causal mask 24 to 10 units of work (68 % of the compute units
    // busy over the launch).  With the head there every XCD gets the same mix of tiles, and the key rows of its heads stay in its L2.
    const int t0 = ((int)gridDim.y - 1 - (int)blockIdx.y) * XP_QT, h = blockIdx.x;      // the longest rows first
    const int64_t d = (int64_t)H * 128;
    // the cached positions are dealt out in segments of XP_KSEG over blockIdx.z, so that the workgroups are of similar length
    // (one workgroup per 128 query rows would make the longest rows the critical path of the launch)
    const int kv_end = min(P + min(t0 + XP_QT - 1, T - 1) + 1, ((int)blockIdx.z + 1) * XP_KSEG);       // cached positions that some row of the tile may see, within this segment
    if ((int)blockIdx.z * XP_KSEG >= kv_end) return;
    uint32_t qa[64], qb[64];
    {
        const float4 *qp = (const float4 *)(q + (int64_t)min(t0 + lane, T - 1) * d + (int64_t)h * 128);
        const float4 *qp2 = (const float4 *)(q + (int64_t)min(t0 + 64 + lane, T - 1) * d + (int64_t)h * 128);
#pragma unroll
        for (int i = 0; i < 32; i++) {
            const float4 f = qp[i], f2 = qp2[i];
            qa[2 * i] = __builtin_bit_cast(uint32_t, xp_pack(f.x, f.y));
            qa[2 * i + 1] = __builtin_bit_cast(uint32_t, xp_pack(f.z, f.w));
            qb[2 * i] = __builtin_bit_cast(uint32_t, xp_pack(f2.x, f2.y));
            qb[2 * i + 1] = __builtin_bit_cast(uint32_t, xp_pack(f2.z, f2.w));
        }
    }
    const int kv_end_a = P + min(t0 + 63, T - 1) + 1;            // cached positions that some row of the tile's first half may see
    // staging: thread -> key row tid / 4 of the tile, 64 of its 256 bytes
    const int st_row = threadIdx.x >> 2, st_q = (threadIdx.x & 3) * 4;
    uint4 kst0, kst1, kst2, kst3;
#define XP_FETCH_K(kv_first) do { \
        const uint4 *src_ = (const uint4 *)(kc + (int64_t)min((kv_first) + st_row, kv_end - 1) * d + (int64_t)h * 128) + st_q; \
        kst0 = src_[0]; kst1 = src_[1]; kst2 = src_[2]; kst3 = src_[3]; } while (0)
    for (int kv0 = (int)blockIdx.z * XP_KSEG; kv0 < kv_end; kv0 += 64) {
        // (no key tile travelling in registers during the dots: with 2 x 64 registers of q values and 2 x 32 accumulators there is
        // no room for it; the second workgroup of the compute unit covers the wait)
        XP_FETCH_K(kv0);
        s_k[st_row][st_q] = kst0; s_k[st_row][st_q + 1] = kst1; s_k[st_row][st_q + 2] = kst2; s_k[st_row][st_q + 3] = kst3;
        __syncthreads();
        const bool first_half = kv0 < kv_end_a;                   // else the whole key tile lies behind the mask of query rows t0 .. t0 + 63
#pragma unroll 1
        for (int j = 0; j < 16; j++) {
            const int kvl = wave * 16 + j;
            float sa = 0.0f, sb = 0.0f;
            if (kv0 + kvl < kv_end) {
                if (first_half) xp_dot128_pair<true>(qa, qb, s_k[kvl], sa, sb);
                else xp_dot128_pair<false>(qa, qb, s_k[kvl], sa, sb);
            }
            s_tile[lane][kvl] = sa;
            s_tile[64 + lane][kvl] = sb;
        }
        __syncthreads();
        {
            const int row = threadIdx.x >> 1, seg = threadIdx.x & 1;
            if (t0 + row < T && (row >= 64 || first_half)) {
                float4 *out = (float4 *)(S + ((int64_t)h * T + t0 + row) * s_row + kv0 + seg * 32);
#pragma unroll
                for (int i = 0; i < 8; i++)
                    out[i] = make_float4(s_tile[row][seg * 32 + 4 * i], s_tile[row][seg * 32 + 4 * i + 1], s_tile[row][seg * 32 + 4 * i + 2],
                                         s_tile[row][seg * 32 + 4 * i + 3]);
            }
        }
        // the next tile's key rows go into s_k at the top of the loop: every wave is past its reads of s_k once it has passed the
        // barrier above, and the barrier after the writes orders them against the next reads
    }
#undef XP_FETCH_K
}

// ---------------------------------------------------------------- softmax
// One workgroup per (head, query row); L = the positions the row may see.  A thread keeps its share of the row in registers
// (groups of four consecutive elements, the unit of the host's sum), so the row is read once and written once.  The
// probabilities leave as fp16 (the first step of the KQV MatMul, mat.cpp:37), followed by zeros up to the end of the 32-row
// tile's last chunk, which the product kernel reads.
#define XP_SM_R 8          // groups per thread: rows of up to 8192 positions
__global__ __launch_bounds__(256) void xp_softmax_kernel(const float *__restrict__ S, uint16_t *__restrict__ P16, const float *__restrict__ lut, int T, int P,
                                                         int64_t s_row, int n_total, float scale) {
    __shared__ __align__(16) float s_grp[256 * XP_SM_R];
    __shared__ float s_part[4], s_rem[4];
    __shared__ float s_out;
    const int t = blockIdx.x, h = blockIdx.y;
    const float4 *s4 = (const float4 *)(S + ((int64_t)h * T + t) * s_row);
    uint16_t *p = P16 + ((int64_t)h * T + t) * s_row;
    const int L = P + t + 1, ng_row = (L + 3) / 4;       // groups that hold an element of the row
    float v[XP_SM_R][4];
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < XP_SM_R; r++) {
        const int g = threadIdx.x + 256 * r;
        if (g < ng_row) {
            const float4 f = s4[g];
            const float e[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float x = e[k] + 0.0f;                   // + the mask value of an allowed position
                x = x * scale;
                v[r][k] = x;
                if (4 * g + k < L) mx = fmaxf(mx, x);
            }
        }
    }
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(s_part[0], s_part[1]), fmaxf(s_part[2], s_part[3]));
    // std::reduce in libstdc++: groups of four as init + ((a0 + a1) + (a2 + a3)) over the first n_total / 4 * 4 elements, the rest one
    // by one; groups and elements past L are zeros and leave the sum as it is
    const int ng_sum = min(n_total / 4, ng_row);
#pragma unroll
    for (int r = 0; r < XP_SM_R; r++) {
        const int g = threadIdx.x + 256 * r;
        if (g < ng_row) {
#pragma unroll
            for (int k = 0; k < 4; k++) v[r][k] = 4 * g + k < L ? lut[f2h(v[r][k] - mx)] : 0.0f;
            const float v1 = v[r][0] + v[r][1], v2 = v[r][2] + v[r][3];
            if (g < ng_sum) s_grp[g] = v1 + v2;
            else {                                       // the group that n_total cuts short: its elements are added one by one
#pragma unroll
                for (int k = 0; k < 4; k++) s_rem[k] = v[r][k];
            }
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float init = 0.0f;
        int g = 0;
        for (; g + 4 <= ng_sum; g += 4) {
            const float4 a = *(const float4 *)&s_grp[g];
            init = init + a.x; init = init + a.y; init = init + a.z; init = init + a.w;
        }
        for (; g < ng_sum; g++) init = init + s_grp[g];
        for (int i = n_total / 4 * 4; i < min(n_total, L); i++) init = init + s_rem[i & 3];
        s_out = init;
    }
    __syncthreads();
    const float inv = 1.0f / s_out;
    const int zend = (int)min((int64_t)((P + (t | 31) + 1 + 31) & ~31), s_row);       // a multiple of 32
    uint2 *p4 = (uint2 *)p;
#pragma unroll
    for (int r = 0; r < XP_SM_R; r++) {
        const int g = threadIdx.x + 256 * r;
        if (g < ng_row) {
            uint16_t o[4];
#pragma unroll
            for (int k = 0; k < 4; k++) o[k] = 4 * g + k < L ? f2h(v[r][k] * inv) : (uint16_t)0;
            p4[g] = make_uint2((uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16));
        }
    }
    for (int g = ng_row + threadIdx.x; g < zend / 4; g += 256) p4[g] = make_uint2(0, 0);
}

// ---------------------------------------------------------------- product with V^T
// One workgroup per (head, 32 query rows, 32 of the 128 output elements); eight groups of 32 lanes, a group takes four
// output elements.  Lane l of a group keeps accumulator l (cached positions 32c + l) of its 4 x 32 outputs, so a V value is
// loaded once for 32 query rows; the probabilities of a chunk come through LDS, transposed to [position][row].
// After the chunks the 32 accumulators of every output are added in the tree of FP16::block_reduce, spread over the lanes so
// that lane l ends with the outputs of query row l, and the scalar tail of the host loop follows.
#define XP_PT 32
#define XP_SC 4            // chunks of 32 positions per stage
__global__ __launch_bounds__(256, 2) void xp_pv_kernel(const uint16_t *__restrict__ P16, const uint16_t *__restrict__ vt, float *__restrict__ out,
                                                       int T, int H, int P, int64_t p_row, int64_t C, int n_total) {
    __shared__ __align__(16) uint16_t s_p[2][32 * XP_SC][40];  // [buffer][position in the stage][query row], rows of 80 bytes
    const int g = threadIdx.x >> 5, l = threadIdx.x & 31;
    const int t0 = ((int)gridDim.z - 1 - (int)blockIdx.z) * XP_PT, h = blockIdx.x;      // head fastest: see xp_scores_kernel
    const int dd0 = blockIdx.y * 32 + g * 4;
    const int Lmax = P + min(t0 + XP_PT - 1, T - 1) + 1;
    const int tail_start = (n_total - 1) / 32 * 32;
    const int nchunk = min(tail_start, (Lmax + 31) & ~31) / 32;
    const int nstage = (nchunk + XP_SC - 1) / XP_SC;
    const uint16_t *vrow[4];
#pragma unroll
    for (int j = 0; j < 4; j++) vrow[j] = vt + ((int64_t)h * 128 + dd0 + j) * C + l;
    // staging of the probabilities: thread -> query row tid % 32, sixteen positions; neighbouring lanes write neighbouring
    // query rows of one position, i.e. neighbouring LDS words (the other way round, 64 lanes would meet in four banks)
    const int st_t = threadIdx.x & 31, st_k = (threadIdx.x >> 5) * 16;
    const uint16_t *prow = P16 + ((int64_t)h * T + min(t0 + st_t, T - 1)) * p_row + st_k;
    float acc[4][32];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int i = 0; i < 32; i++) acc[j][i] = 0.0f;
    uint4 pst[2];
    uint16_t vn[XP_SC][4];
    auto fetch = [&](int s) {
        pst[0] = *(const uint4 *)(prow + 32 * XP_SC * s);
        pst[1] = *(const uint4 *)(prow + 32 * XP_SC * s + 8);
#pragma unroll
        for (int c = 0; c < XP_SC; c++) {
            const int pos = 32 * (XP_SC * s + c);
#pragma unroll
            for (int j = 0; j < 4; j++) vn[c][j] = pos + l < Lmax ? vrow[j][pos] : (uint16_t)0;      // past Lmax every probability is 0; the cache may hold anything there
        }
    };
    auto put = [&](int buf) {
#pragma unroll
        for (int v = 0; v < 2; v++) {
            const uint32_t w[4] = {pst[v].x, pst[v].y, pst[v].z, pst[v].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                s_p[buf][st_k + 8 * v + 2 * i][st_t] = (uint16_t)(w[i] & 0xFFFFu);
                s_p[buf][st_k + 8 * v + 2 * i + 1][st_t] = (uint16_t)(w[i] >> 16);
            }
        }
    };
    if (nstage > 0) {
        fetch(0);
        put(0);
    }
    __syncthreads();
    for (int s = 0; s < nstage; s++) {
        const int buf = s & 1;
        _Float16 vc[XP_SC][4];
#pragma unroll
        for (int c = 0; c < XP_SC; c++)
#pragma unroll
            for (int j = 0; j < 4; j++) vc[c][j] = __builtin_bit_cast(_Float16, vn[c][j]);
        if (s + 1 < nstage) fetch(s + 1);
#pragma unroll
        for (int c = 0; c < XP_SC; c++) {
            if (XP_SC * s + c < nchunk) {
                const uint4 *pp = (const uint4 *)&s_p[buf][32 * c + l][0];
#pragma unroll
                for (int qd = 0; qd < 4; qd++) {
                    const uint4 w4 = pp[qd];
                    const uint32_t w[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const xp_half2 p2 = __builtin_bit_cast(xp_half2, w[i]);
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            acc[j][8 * qd + 2 * i] = fmaf((float)vc[c][j], (float)p2.x, acc[j][8 * qd + 2 * i]);
                            acc[j][8 * qd + 2 * i + 1] = fmaf((float)vc[c][j], (float)p2.y, acc[j][8 * qd + 2 * i + 1]);
                        }
                    }
                }
            }
        }
        if (s + 1 < nstage) put(buf ^ 1);
        __syncthreads();
    }
    // The tree: sum[l] += sum[l + 16], sum[l] += sum[l + 8], t_l = sum[l] + sum[l + 4], (t0 + t1) + (t2 + t3), where l is the lane.
    // At each step a lane keeps the half of its query rows that matches its own lane bit and hands the other half to its
    // partner, so 16 + 8 + 4 + 2 + 1 exchanges per output element leave lane l with the sum of query row l.
    float res[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float a16[16], a8[8], a4[4], a2[2];
        const bool b4 = l & 16, b3 = l & 8, b2 = l & 4, b0 = l & 1, b1 = l & 2;
#pragma unroll
        for (int k = 0; k < 16; k++) {
            const float keep = b4 ? acc[j][k + 16] : acc[j][k], send = b4 ? acc[j][k] : acc[j][k + 16];
            a16[k] = keep + __shfl_xor(send, 16, SPY_WAVE);
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float keep = b3 ? a16[k + 8] : a16[k], send = b3 ? a16[k] : a16[k + 8];
            a8[k] = keep + __shfl_xor(send, 8, SPY_WAVE);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const float keep = b2 ? a8[k + 4] : a8[k], send = b2 ? a8[k] : a8[k + 4];
            a4[k] = keep + __shfl_xor(send, 4, SPY_WAVE);
        }
        // query rows left: 4 per lane, their index = (l & 28) + k; the tree goes on with lane bit 0, then bit 1
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const float keep = b0 ? a4[2 * k + 1] : a4[2 * k], send = b0 ? a4[2 * k] : a4[2 * k + 1];
            a2[k] = keep + __shfl_xor(send, 1, SPY_WAVE);
        }
        {
            const float keep = b1 ? a2[1] : a2[0], send = b1 ? a2[0] : a2[1];
            res[j] = keep + __shfl_xor(send, 2, SPY_WAVE);
        }
    }
    // lane l now holds query row t0 + l: rows were halved by lane bits 4, 3, 2 (index bits 4, 3, 2), then bit 0 chose index bit 0 and
    // bit 1 index bit 1
    const int t = t0 + l;
    if (t >= T) return;
    const int Lt = P + t + 1;                                      // positions row t sees
    const int tail_end = min(n_total, Lt);
    const uint16_t *pr = P16 + ((int64_t)h * T + t) * p_row;
    float o4[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float tail = 0.0f;
        const uint16_t *vr = vt + ((int64_t)h * 128 + dd0 + j) * C;
        for (int i = tail_start; i < tail_end; i++) {
            const float pr_ = h2f(vr[i]) * h2f(pr[i]);
            tail += pr_;
        }
        o4[j] = tail + res[j];
    }
    *(float4 *)(out + (int64_t)t * H * 128 + (int64_t)h * 128 + dd0) = make_float4(o4[0], o4[1], o4[2], o4[3]);
}

}   // namespace

// q: fp32 [T][H][128] after Rope; kc: fp16 [position][H][128]; vt: fp16 [H * 128][C]; out: fp32 [T][H][128];
// S: H * T * s_row floats and P16: H * T * s_row halves of scratch, s_row = spy_exact_prompt_attn_row(P + T)
int64_t spy_exact_prompt_attn_row(int64_t n_kv) { return (n_kv + 127) & ~(int64_t)127; }

int spy_exact_prompt_attn(hipStream_t st, const float *q, const uint16_t *kc, const uint16_t *vt, float *S, uint16_t *P16, float *out, const float *lut,
                          int T, int H, int P, int64_t C, int n_total, float scale) {
    if (T <= 0 || H <= 0 || H > 65535 || P < 0 || (int64_t)P + T > C || n_total < P + T || n_total > C || C % 32) return SPY_HIP_EINVAL;
    if ((int64_t)P + T > 1024 * XP_SM_R) return SPY_HIP_EUNSUPPORTED;      // the softmax kernel keeps a row in the registers of 256 threads
    if (((uintptr_t)q & 15) || ((uintptr_t)kc & 15) || ((uintptr_t)S & 15) || ((uintptr_t)P16 & 7) || ((uintptr_t)out & 15)) return SPY_HIP_EINVAL;
    const int64_t s_row = spy_exact_prompt_attn_row((int64_t)P + T);
    xp_scores_kernel<<<dim3((unsigned)H, (unsigned)((T + XP_QT - 1) / XP_QT), (unsigned)((P + T + XP_KSEG - 1) / XP_KSEG)), dim3(256), 0, st>>>(q, kc, S, T, H, P, s_row);
    if (hipGetLastError() != hipSuccess) return SPY_HIP_EINVAL;
    xp_softmax_kernel<<<dim3((unsigned)T, (unsigned)H), dim3(256), 0, st>>>(S, P16, lut, T, P, s_row, n_total, scale);
    if (hipGetLastError() != hipSuccess) return SPY_HIP_EINVAL;
    xp_pv_kernel<<<dim3((unsigned)H, 4, (unsigned)((T + XP_PT - 1) / XP_PT)), dim3(256), 0, st>>>(P16, vt, out, T, H, P, s_row, C, n_total);
    return SPY_LAUNCH_RC();
}

int spy_exact_luts(const float **lut);           // exact_order.hip

extern "C" size_t spy_hip_prompt_attention_exact_scratch_size(int32_t T, int32_t H, int32_t past) {
    if (T <= 0 || H <= 0 || past < 0) return 0;
    return (size_t)spy_exact_prompt_attn_row((int64_t)past + T) * (size_t)T * (size_t)H * 6;       // fp32 scores, then fp16 probabilities
}

extern "C" int spy_hip_prompt_attention_exact(void *stream, const float *q, const void *k_cache, const void *v_cache, float *out, int32_t T, int32_t H,
                                              int32_t hd, int32_t past, int64_t n_ctx, int32_t n_total, float scale, void *scratch, size_t scratch_bytes) {
    SPY_CHECK_ARG(q && k_cache && v_cache && out && scratch);
    if (hd != 128 || n_ctx % 32) return SPY_HIP_EUNSUPPORTED;
    const size_t need = spy_hip_prompt_attention_exact_scratch_size(T, H, past);
    if (!need) return SPY_HIP_EINVAL;
    if (scratch_bytes < need || ((uintptr_t)scratch & 255)) return SPY_HIP_ENOSPACE;
    const float *lut = nullptr;
    const int rc = spy_exact_luts(&lut);
    if (rc) return rc;
    float *S = (float *)scratch;
    uint16_t *P16 = (uint16_t *)((uint8_t *)scratch + need / 6 * 4);
    return spy_exact_prompt_attn((hipStream_t)stream, q, (const uint16_t *)k_cache, (const uint16_t *)v_cache, S, P16, out, lut, T, H, past, n_ctx, n_total, scale);
}
