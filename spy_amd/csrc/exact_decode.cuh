// Kernels of the fused single-token pass in the HOST BACKEND'S SUMMATION ORDER: the same launches as
// decode_kernels.cuh (weights streamed once, activations quantized in LDS, epilogues fused), but every fp32 sum is
// added in the order of Spy's CPU loops, so that each output equals the CPU backend's bit for bit:
//   * quantized dots (vec_dot.h:42-115): eight accumulators per output element, lane l takes four products of every
//     block, acc[l] = fma(d_w * d_x, float(part[l]), acc[l]) block after block, then hsum_float_8 (vec_util.h:75-81);
//     K-quant rows: the project's order, one accumulator, one term per 32-element block;
//   * fp16 dots (vec_dot.h:117-146): 4 x 8 accumulators over chunks of 32 while i + 32 < n, the reduction tree, then
//     the scalar tail;
//   * NormRMS and Softmax sums (non-linear.cpp:129-223): libstdc++'s groups of four added to ONE running sum;
//   * exp and silu from the two fp16-indexed tables filled by the host's libm, the RoPE angles from a host table.
//
// How a serial sum is made fast.  The integer block dots stay where they are (64 lanes x v_dot4, one block pair per
// lane, weights read once, coalesced).  What changes is what follows them: instead of scaling and adding its blocks in
// lane order, a lane writes the eight partial sums of each of its blocks (as floats) and the block's scale product into
// LDS, transposed, and after a workgroup barrier ONE lane per accumulator walks its row of LDS block after block:
// 8 lanes per output element, 64 lanes = 8 output elements per wave, fed by 128-bit LDS reads.  The walk is a chain of
// dependent fmas (about 4 ns each on this part, whatever else the compute unit does), so a 4096-wide row costs about
// 0.6 us of latency per batch of rows; batches are as large as LDS allows (32 rows of 128 blocks).
#pragma once

#include "decode_kernels.cuh"

#define XG_THREADS 1024
#define XG_WAVES 16
#define XG_NBS 128                         // blocks per K slab (= 64 lanes x one block pair)
#ifndef XG_PSUM
#define XG_PSUM 1                          // gate|up: the running sum of the norm through xg_exact_sum (0: one chain, as in the other kernels)
#endif
#ifndef XG_DEPTH
#define XG_DEPTH 3                         // rows per wave requested ahead of their use
#endif

template <int WT> struct xg_traits { static constexpr int NCH = (WT == SPY_HIP_Q4_0 || WT == SPY_HIP_Q8_0) ? 8 : 1; };
// floats of LDS per row slot: NCH rows of partials (+4: bank skew between the rows) and the row of scale products (+4: skew between slots)
static __host__ __device__ constexpr int xg_slot_floats(int nch) { return nch * (XG_NBS + 4) + XG_NBS + 4; }

struct xg_args {
    const uint8_t *W0, *W1, *W2;
    int M, K;                              // output elements (RESID / STORE: rows of W0; GATEUP: rows of W0 = rows of W1; QKV: n_embd), contraction length
    const float *x_in, *normw; float eps;
    const float *resid; float *out;
    const dev_state *st; const float *rope_tab; uint16_t *q16, *kc, *vc;   // rope_tab: [n_ctx][hd] cos, sin per pair, from the host's libm
    const float *lut;                      // exp table [65536], then silu table [65536] (lookup_table_impl/non-linear.h:39-47,131-139)
    int n_ctx, d, hd;
    uint8_t *q8_dump;                      // tests: workgroup 0 writes its staged activations here as native Q8_0 blocks
    int pos_imm, rope_row0;                // st == nullptr: the position as a number; first position of rope_tab
    long long *dbg;                        // measurement builds (-DXDBG_STAMPS): wall-clock stamps of workgroup 0
};
#ifdef XDBG_STAMPS
#define XSTAMP(dbg, i) do { if ((dbg) && blockIdx.x == 0 && threadIdx.x == 0) (dbg)[i] = wall_clock64(); } while (0)
#else
#define XSTAMP(dbg, i) do { } while (0)
#endif

// libstdc++'s std::reduce over the n values at s (LDS, 16-byte aligned; up to 40 floats beyond n may be read, never added): ONE
// running sum, value after value.  Every lane of the calling wave walks the same chain (same addresses: LDS broadcasts them), so
// the result is wave-uniform.  The additions are a chain of dependent operations (about 4 ns each); the 128-bit LDS reads of the
// next sixteen values are requested before the current sixteen additions (two register sets), so their latency hides behind the chain.
static __device__ __forceinline__ float xg_serial_sum(const float *s, int n, float init) {
    float4 a[2], b[2], c[2];
    auto ld = [&](float4 (&r)[2], int i) {
#pragma unroll
        for (int u = 0; u < 2; u++) r[u] = *(const float4 *)(s + i + 4 * u);
    };
    auto run = [&](const float4 (&r)[2]) {
#pragma unroll
        for (int u = 0; u < 2; u++) { init = init + r[u].x; init = init + r[u].y; init = init + r[u].z; init = init + r[u].w; }
    };
    // groups of 8 values, each requested two groups (sixteen dependent additions) ahead of its use: three register sets in rotation
    const int n24 = n - n % 24;
    int i = 0;
    if (n24) {
        ld(a, 0);
        ld(b, 8);
        for (; i < n24; i += 24) {
            ld(c, i + 16);
            __builtin_amdgcn_sched_barrier(0);
            run(a);
            __builtin_amdgcn_sched_barrier(0);
            ld(a, i + 24);                               // up to 28 floats beyond n: read, never added
            __builtin_amdgcn_sched_barrier(0);
            run(b);
            __builtin_amdgcn_sched_barrier(0);
            ld(b, i + 32);
            __builtin_amdgcn_sched_barrier(0);
            run(c);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    for (; i < n; i++) init = init + s[i];
    return init;
}

// ---- the same running sum, for NON-NEGATIVE terms, mostly in parallel and still bit for bit -----------------------------
// While the running sum s stays inside one binade [2^e, 2^(e+1)) it is an integer multiple S of ulp = 2^(e-23), and adding a term
// g >= 0 with round-to-nearest-even is integer arithmetic: with f = g / ulp (exact: a power-of-two scaling),
//     RNE(S + f) = S + floor(f) + r,   r = 1 if frac(f) > 1/2, 0 if < 1/2, and for frac(f) = 1/2 the parity of S + floor(f).
// So a term is a map from the parity of the incoming S to an increment, (inc_even, inc_odd), maps compose associatively
// (C[p] = A[p] + B[(p + A[p]) & 1]), and 64 consecutive terms reduce to one pair in four DPP steps and three scalar ones.  The
// sum is non-decreasing, so if the chunk's first and last value lie in binade e, every value between does.  Wave c reduces
// chunk c (terms 64 c .. 64 c + 63) against the binade that an approximate prefix sum predicts; then one wave walks the chunks:
// where the exact running sum has the predicted exponent and bits(s) + increment keeps it (the integer addition on the float's
// bits IS s + increment * ulp), the chunk is one addition; otherwise (the sum crosses a power of two inside the chunk, the first
// chunk, a wrong prediction) the chunk's 64 terms are added one by one as above.  Nothing is approximated in what is kept: the
// prediction only selects which chunks take the short way.
struct xg_psum_lds { float cs[32]; int t0[32], t1[32], eb[32]; };
// g[j]: term 1024 j + tid of the n <= 1024 NG terms (0 beyond n), all of them also at s_g in LDS (written before the call,
// 16-byte aligned, readable 40 floats beyond n).  Every thread of the 1024 calls; the sum is returned by wave 0 only (wave-uniform).
// `others` runs in the other waves once their part is done, i.e. while wave 0 walks.
template <int NG, class Others>
static __device__ __forceinline__ float xg_exact_sum(const float (&g)[NG], int n, const float *s_g, xg_psum_lds *L, float init, Others others, long long *dbg = nullptr) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nchunk = (n + 63) >> 6;
    // sum over the wave through DPP only (no LDS permutes), read from lane 63; the order of these additions does not matter:
    // they only predict binades
    auto total = [](float v) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wave_total_lane63(v)), 63)); };
#pragma unroll
    for (int j = 0; j < NG; j++) {
        const float cs = total(g[j]);
        if (lane == 0) L->cs[wave + 16 * j] = cs;
    }
    XSTAMP(dbg, 8);
    __syncthreads();                                     // chunk sums and (by the caller) the terms are in LDS
    XSTAMP(dbg, 9);
#pragma unroll
    for (int j = 0; j < NG; j++) {
        const int c = wave + 16 * j;
        if (c < nchunk) {
            const float before = total(lane < c ? L->cs[lane & 31] : 0.0f) + init, after = before + L->cs[c];
            const int eb = (__float_as_int(before) >> 23) & 0xFF;
            const float f = ldexpf(g[j], 150 - eb);      // g / ulp
            const bool fits = f < 16777216.0f;           // false for a NaN too
            const int fl = fits ? (int)f : 0;
            const float frac = f - (float)fl;
            const int up = frac > 0.5f ? 1 : 0, tie = frac == 0.5f ? 1 : 0;
            int a0 = fl + (up | (tie & fl & 1)), a1 = fl + (up | (tie & ~fl & 1));    // incoming S even / odd: a tie rounds to the even neighbour
            // within each row of 16 lanes: lane l takes over the terms of lane l + d (row_shl), earlier terms first; lanes
            // that reach beyond their row compute values nobody uses
#define XG_PS_STEP(CTRL) { const int b0 = __builtin_amdgcn_update_dpp(0, a0, CTRL, 0xF, 0xF, true), b1 = __builtin_amdgcn_update_dpp(0, a1, CTRL, 0xF, 0xF, true); \
                           a0 = a0 + ((a0 & 1) ? b1 : b0); a1 = a1 + ((a1 & 1) ? b0 : b1); }   /* incoming odd: the parity after the first part is (1 + a1) & 1 */
            XG_PS_STEP(0x101) XG_PS_STEP(0x102) XG_PS_STEP(0x104) XG_PS_STEP(0x108)
#undef XG_PS_STEP
            // the four rows in order, as scalars
            int t0 = __builtin_amdgcn_readlane(a0, 0), t1 = __builtin_amdgcn_readlane(a1, 0);
#pragma unroll
            for (int r = 1; r < 4; r++) {
                const int b0 = __builtin_amdgcn_readlane(a0, 16 * r), b1 = __builtin_amdgcn_readlane(a1, 16 * r);
                t0 = t0 + ((t0 & 1) ? b1 : b0);
                t1 = t1 + ((t1 & 1) ? b0 : b1);
            }
            const bool ok = __all(fits) && c > 0 && eb >= 1 && eb < 254 && ((__float_as_int(after) >> 23) & 0xFF) == eb;
            if (lane == 0) { L->t0[c] = t0; L->t1[c] = t1; L->eb[c] = ok ? eb : -1; }
        }
    }
    XSTAMP(dbg, 10);
    __syncthreads();
    XSTAMP(dbg, 11);
    float s = init;
    if (wave == 0) {
        const int vt0 = L->t0[lane & 31], vt1 = L->t1[lane & 31], veb = L->eb[lane & 31];
        // the terms of the chunks predicted to need the long way are requested ahead: the first such chunk now, the next one
        // when the current one is taken up (a chunk that fails without having been predicted pays the LDS latency)
        const unsigned long long slowmask = __ballot(lane < nchunk && veb < 0);
        auto next_slow = [&](int from) -> int { const unsigned long long m = from < 64 ? (slowmask >> from) << from : 0ull; return m ? __builtin_ctzll(m) : -1; };
        // (its first 32 terms; the other 32 are requested when the chunk is taken up and arrive behind the first 32 additions)
        float4 v[8], w[8];
        auto request = [&](int c) {
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = *(const float4 *)(s_g + 64 * c + 4 * u);
        };
        int pre = next_slow(0);
        if (pre >= 0) request(pre);
        int bits = __builtin_amdgcn_readfirstlane(__float_as_int(s));             // the running sum as a scalar
        [[maybe_unused]] int nfall = 0;
        for (int c = 0; c < nchunk; c++) {
            const int eb = __builtin_amdgcn_readlane(veb, c), t = (bits & 1) ? __builtin_amdgcn_readlane(vt1, c) : __builtin_amdgcn_readlane(vt0, c);
            const int nb = bits + t;
            if (eb == (bits >> 23) && (nb >> 23) == eb && t >= 0) { bits = nb; continue; }
            s = __int_as_float(bits);
            nfall++;
            if (n - 64 * c >= 64) {                      // a whole chunk one by one
                if (c != pre) request(c);
#pragma unroll
                for (int u = 0; u < 8; u++) w[u] = *(const float4 *)(s_g + 64 * c + 32 + 4 * u);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < 8; u++) { s = s + v[u].x; s = s + v[u].y; s = s + v[u].z; s = s + v[u].w; }
                __builtin_amdgcn_sched_barrier(0);
                if (c == pre) { pre = next_slow(c + 1); if (pre >= 0) request(pre); }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < 8; u++) { s = s + w[u].x; s = s + w[u].y; s = s + w[u].z; s = s + w[u].w; }
            } else s = xg_serial_sum(s_g + 64 * c, n - 64 * c, s);
            bits = __builtin_amdgcn_readfirstlane(__float_as_int(s));
        }
        s = __int_as_float(bits);
        XSTAMP(dbg, 12);
#ifdef XDBG_STAMPS
        if (dbg && blockIdx.x == 0 && threadIdx.x == 0) dbg[13] = nfall;
#endif
    } else others();
    return s;
}

// ---- activations: f32 vector -> (RMSNorm * weight ->) Q8_0 in LDS, sums in the host order --------------------------
// NormRMS (non-linear.cpp:194-223): sum = std::transform_reduce(x, x) = groups of four ((x0^2 + x1^2) + (x2^2 + x3^2))
// added to one running sum in order; scale = 1 / sqrt(sum / n + eps); y = x * scale; then the Mul node: y * w.
// The 1024 threads form the group sums (one float4 each per 4096 elements), lane 0 of wave 0 adds them.
template <int NITK, bool NORM, bool PSUM = false, class Issue>
static __device__ __forceinline__ void xg_stage(const float4 (&xv)[NITK], const float4 (&wv)[NORM ? NITK : 1], int K, float eps,
                                                int8_t *s_q, int2 *s_meta, float *s_grp, float *s_sum, Issue issue_rows) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float scale = 1.0f;
    if constexpr (NORM) {
        float grp[NITK];
#pragma unroll
        for (int j = 0; j < NITK; j++) {
            const int i = tid + j * XG_THREADS;
            grp[j] = 0.0f;
            if (i < K / 4) {
                const float4 v = xv[j];
                const float a0 = v.x * v.x, a1 = v.y * v.y, a2 = v.z * v.z, a3 = v.w * v.w;
                const float v1 = a0 + a1, v2 = a2 + a3;
                grp[j] = v1 + v2;
                s_grp[i] = grp[j];
            }
        }
        // The weight rows are requested only after the group sums (and the scan of the sum): a wave that asks for several rows sits
        // in the issue stage until the memory queue has room, and a request made earlier would hold up the barriers for every wave.
        // Wave 0 walks the sum first.
        if constexpr (NITK <= 2 && PSUM) {
            xg_psum_lds *L = (xg_psum_lds *)(s_grp + ((K / 4 + 3) & ~3) + 64);
            const float tot = xg_exact_sum<NITK>(grp, K / 4, s_grp, L, 0.0f, issue_rows);
            if (wave == 0) { if (lane == 0) *s_sum = tot; issue_rows(); }
        } else {
            __syncthreads();
            if (wave == 0) {
                const float init = xg_serial_sum(s_grp, K / 4, 0.0f);
                if (lane == 0) *s_sum = init;
            }
            issue_rows();
        }
        __syncthreads();
        const float mean = *s_sum / (float)K;
        scale = 1.0f / sqrtf(mean + eps);
    } else issue_rows();
#pragma unroll
    for (int j = 0; j < NITK; j++) {
        const int i = tid + j * XG_THREADS;
        if (i < K / 4) {
            float4 v = xv[j];
            if constexpr (NORM) {
                const float4 w = wv[j];
                v.x = (v.x * scale) * w.x; v.y = (v.y * scale) * w.y; v.z = (v.z * scale) * w.z; v.w = (v.w * scale) * w.w;
            }
            int2 meta;
            const uint32_t q = quantize_oct(v, meta);
            ((uint32_t *)s_q)[act_dw(i, K >> 6)] = q;
            if ((tid & 7) == 0) s_meta[i >> 3] = meta;
        }
    }
    __syncthreads();
}

// the staged activations of a workgroup as native Q8_0 blocks (tests compare them with Quantizator<FP32,Q8_0>)
static __device__ __forceinline__ void xg_dump_q8(const int8_t *s_q, const int2 *s_meta, int K, uint8_t *out) {
    for (int b = threadIdx.x; b < K / 32; b += XG_THREADS) {
        uint16_t *dst = (uint16_t *)(out + (size_t)b * 34);
        dst[0] = f2h(__int_as_float(s_meta[b].x));
        for (int i = 0; i < 8; i++) {
            const uint32_t q = ((const uint32_t *)s_q)[act_dw(b * 8 + i, K >> 6)];
            dst[1 + 2 * i] = (uint16_t)(q & 0xFFFFu); dst[2 + 2 * i] = (uint16_t)(q >> 16);
        }
    }
}

// ---- phase 1: a lane's block pair of one weight row -> partial sums and scale products in LDS -------------------------
// x[0..3]: the 64 int8 activations of the pair (16 bytes each), mm / mm2: their {scale bits, sum q} (see load_act_frag),
// n8[i] = -8 * (sum of the four bytes of activation dword i): folds the -8 of the Q4_0 nibbles into the accumulator
// input of v_dot4, so that each partial sum is sum (n - 8) * q exactly as sub_epi8 / maddubs / madd form it.
// slot: this row's LDS record; pl: the pair's index within the slab (= lane).
template <int WT>
static __device__ __forceinline__ void xg_phase1(const uint32_t *w, const act_frag<1> &f, const int (&n8)[16], int p, int pl, float *slot) {
    constexpr int NCH = xg_traits<WT>::NCH;
    float *P = slot, *D = slot + NCH * (XG_NBS + 4);
    const int4 x0 = f.x[0][0], x1 = f.x[0][1], x2 = f.x[0][2], x3 = f.x[0][3], mm = f.mm[0], mm2 = f.mm2[0];
    if constexpr (WT == SPY_HIP_Q4_0 || WT == SPY_HIP_Q8_0) {
        int pa[8], pb[8];
        float sA, sB;
        if constexpr (WT == SPY_HIP_Q4_0) {
            sA = h2f((uint16_t)(w[0] & 0xFFFFu)) * __int_as_float(mm.x); sB = h2f((uint16_t)(w[4] >> 16)) * __int_as_float(mm.z);
            const uint32_t a[4] = {__builtin_amdgcn_alignbit(w[1], w[0], 16), __builtin_amdgcn_alignbit(w[2], w[1], 16),
                                   __builtin_amdgcn_alignbit(w[3], w[2], 16), __builtin_amdgcn_alignbit(w[4], w[3], 16)};
            const int xa[4] = {x0.x, x0.y, x0.z, x0.w}, xb[4] = {x1.x, x1.y, x1.z, x1.w}, xc[4] = {x2.x, x2.y, x2.z, x2.w}, xd[4] = {x3.x, x3.y, x3.z, x3.w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                // accumulators 4..7: low nibbles against elements 0..15; 0..3: high nibbles against 16..31 (vec_dot.h:62-78)
                pa[4 + k] = __builtin_amdgcn_sdot4((int)(a[k] & 0x0F0F0F0Fu), xa[k], n8[k], false);
                pa[k]     = __builtin_amdgcn_sdot4((int)((a[k] >> 4) & 0x0F0F0F0Fu), xb[k], n8[4 + k], false);
                pb[4 + k] = __builtin_amdgcn_sdot4((int)(w[5 + k] & 0x0F0F0F0Fu), xc[k], n8[8 + k], false);
                pb[k]     = __builtin_amdgcn_sdot4((int)((w[5 + k] >> 4) & 0x0F0F0F0Fu), xd[k], n8[12 + k], false);
            }
        } else {
            sA = h2f((uint16_t)(w[0] & 0xFFFFu)) * __int_as_float(mm.x); sB = h2f((uint16_t)(w[8] >> 16)) * __int_as_float(mm.z);
            const int xa[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w}, xb[8] = {x2.x, x2.y, x2.z, x2.w, x3.x, x3.y, x3.z, x3.w};
#pragma unroll
            for (int l = 0; l < 8; l++) {               // accumulator l: elements 4l..4l+3 (vec_util.h:126-132)
                pa[l] = __builtin_amdgcn_sdot4((int)__builtin_amdgcn_alignbit(w[l + 1], w[l], 16), xa[l], 0, false);
                pb[l] = __builtin_amdgcn_sdot4((int)w[9 + l], xb[l], 0, false);
            }
        }
#pragma unroll
        for (int l = 0; l < 8; l++) *(float2 *)(P + l * (XG_NBS + 4) + 2 * pl) = make_float2((float)pa[l], (float)pb[l]);
        *(float2 *)(D + 2 * pl) = make_float2(sA, sB);
    } else if constexpr (WT == SPY_HIP_Q4_K) {
        // the two sub-blocks of the lane: term = d * float(sc * isum) - dmin * float(m * sum q), scale = d_x (one accumulator per row)
        const int j = p & 3, a = 2 * j;
        const float d = h2f((uint16_t)(w[0] & 0xFFFFu)), dmin = h2f((uint16_t)(w[0] >> 16));
        int scA, mA, scB, mB;
        if (j < 2) {
            scA = byte_of3(w[1], w[2], w[3], a) & 63;     mA = byte_of3(w[1], w[2], w[3], a + 4) & 63;
            scB = byte_of3(w[1], w[2], w[3], a + 1) & 63; mB = byte_of3(w[1], w[2], w[3], a + 5) & 63;
        } else {
            const uint32_t hA = byte_of3(w[1], w[2], w[3], a + 4), hB = byte_of3(w[1], w[2], w[3], a + 5);
            scA = (hA & 0x0F) | ((byte_of3(w[1], w[2], w[3], a - 4) >> 6) << 4); mA = (hA >> 4) | ((byte_of3(w[1], w[2], w[3], a) >> 6) << 4);
            scB = (hB & 0x0F) | ((byte_of3(w[1], w[2], w[3], a - 3) >> 6) << 4); mB = (hB >> 4) | ((byte_of3(w[1], w[2], w[3], a + 1) >> 6) << 4);
        }
        int iA = 0, iB = 0;
        const int xa[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w}, xb[8] = {x2.x, x2.y, x2.z, x2.w, x3.x, x3.y, x3.z, x3.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            iA = __builtin_amdgcn_sdot4((int)(w[4 + i] & 0x0F0F0F0Fu), xa[i], iA, false);
            iB = __builtin_amdgcn_sdot4((int)((w[4 + i] >> 4) & 0x0F0F0F0Fu), xb[i], iB, false);
        }
        const float posA = d * (float)__mul24(scA, iA), negA = dmin * (float)__mul24(mA, mm.y);
        const float posB = d * (float)__mul24(scB, iB), negB = dmin * (float)__mul24(mB, mm.w);
        *(float2 *)(P + 2 * pl) = make_float2(posA - negA, posB - negB);
        *(float2 *)(D + 2 * pl) = make_float2(__int_as_float(mm.x), __int_as_float(mm.z));
    } else {
        // Q6_K: lane (n, e) holds the 16-element halves e of the four Q8_0 blocks 4n .. 4n+3 of its super-block; the other
        // halves are in the neighbouring lane.  term of block t = float(sc[2t] * isum(t, 0) + sc[2t+1] * isum(t, 1)), scale = d_x * d
        const uint32_t *qa = w, *qb = w + 4, *qh = w + 8;
        const uint32_t s0 = w[12], s1 = w[13];
        const int e = p & 1;
        const float d = h2f((uint16_t)(w[14] & 0xFFFFu));
        int isum[4] = {0, 0, 0, 0};
        const int xm[4][4] = {{x0.x, x0.y, x0.z, x0.w}, {x1.x, x1.y, x1.z, x1.w}, {x2.x, x2.y, x2.z, x2.w}, {x3.x, x3.y, x3.z, x3.w}};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t h = qh[i];
            isum[0] = __builtin_amdgcn_sdot4((int)q6_m32((qa[i] & 0x0F0F0F0Fu) | ((h & 0x03030303u) << 4)), xm[0][i], isum[0], false);
            isum[1] = __builtin_amdgcn_sdot4((int)q6_m32((qb[i] & 0x0F0F0F0Fu) | ((h & 0x0C0C0C0Cu) << 2)), xm[1][i], isum[1], false);
            isum[2] = __builtin_amdgcn_sdot4((int)q6_m32(((qa[i] >> 4) & 0x0F0F0F0Fu) | (h & 0x30303030u)), xm[2][i], isum[2], false);
            isum[3] = __builtin_amdgcn_sdot4((int)q6_m32(((qb[i] >> 4) & 0x0F0F0F0Fu) | ((h >> 2) & 0x30303030u)), xm[3][i], isum[3], false);
        }
        int sv[4];
#pragma unroll
        for (int m = 0; m < 4; m++) {
            const int k = e + 2 * m;
            const int sc = (int)(int8_t)(((k < 4 ? s0 : s1) >> (8 * (k & 3))) & 0xFFu);
            const int v = __mul24(sc, isum[m]);
            sv[m] = v + __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);          // + the neighbour lane's half (quad_perm [1,0,3,2]); integer, order-free
        }
        const float dx[4] = {__int_as_float(mm.x), __int_as_float(mm.z), __int_as_float(mm2.x), __int_as_float(mm2.z)};
        // lane e writes blocks m = 2e, 2e+1 of the four: global block 2p, 2p+1
        const float t0 = (float)(e ? sv[2] : sv[0]), t1 = (float)(e ? sv[3] : sv[1]);
        const float c0 = (e ? dx[2] : dx[0]) * d, c1 = (e ? dx[3] : dx[1]) * d;
        *(float2 *)(P + 2 * pl) = make_float2(t0, t1);
        *(float2 *)(D + 2 * pl) = make_float2(c0, c1);
    }
}

// ---- phase 2: one lane walks one accumulator over the blocks of a slab ------------------------------------------------
template <int NCH>
static __device__ __forceinline__ float xg_chain(const float *P, const float *D, int nblk, float acc) {
    // nblk % 4 == 0.  Eight blocks per group; the 128-bit reads of a group are requested two groups (sixteen dependent fmas,
    // about the latency of an LDS read under load) before its fmas: three register sets in rotation, no copies.  Reads beyond
    // nblk stay inside the row's 128 + 4 floats and are not used.
    // (Taking the scale products, which the eight lanes of a row share, from one lane per quad through DPP broadcasts cut the LDS
    // traffic but measured slower: 1.25 instead of 0.8 us per 128 blocks.)
    float4 p0[2], p1[2], p2[2], d0[2], d1[2], d2[2];
    auto ld = [&](float4 (&p)[2], float4 (&d)[2], int b) {
#pragma unroll
        for (int u = 0; u < 2; u++) { p[u] = *(const float4 *)(P + min(b + 4 * u, XG_NBS - 4)); d[u] = *(const float4 *)(D + min(b + 4 * u, XG_NBS - 4)); }
    };
    auto run = [&](const float4 (&p)[2], const float4 (&d)[2], int b) {
#pragma unroll
        for (int u = 0; u < 2; u++)
            if (b + 4 * u < nblk) { acc = fmaf(d[u].x, p[u].x, acc); acc = fmaf(d[u].y, p[u].y, acc); acc = fmaf(d[u].z, p[u].z, acc); acc = fmaf(d[u].w, p[u].w, acc); }
    };
    ld(p0, d0, 0);
    ld(p1, d1, 8);
    for (int b = 0; b < nblk; b += 24) {
        ld(p2, d2, b + 16);
        __builtin_amdgcn_sched_barrier(0);
        run(p0, d0, b);
        __builtin_amdgcn_sched_barrier(0);
        ld(p0, d0, b + 24);
        __builtin_amdgcn_sched_barrier(0);
        run(p1, d1, b + 8);
        __builtin_amdgcn_sched_barrier(0);
        ld(p1, d1, b + 32);
        __builtin_amdgcn_sched_barrier(0);
        run(p2, d2, b + 16);
        __builtin_amdgcn_sched_barrier(0);
    }
    return acc;
}

// hsum_float_8 over the eight lanes of an output element: (a0+a4)+(a2+a6) + (a1+a5)+(a3+a7); the operands of each
// addition commute, so the three exchanges leave the same bits in all eight lanes (vec_util.h:75-81)
static __device__ __forceinline__ float xg_hsum8(float acc) {
    acc += __shfl_xor(acc, 4, SPY_WAVE);
    acc += __shfl_xor(acc, 2, SPY_WAVE);
    acc += __shfl_xor(acc, 1, SPY_WAVE);
    return acc;
}

// ---- the kernel --------------------------------------------------------------------------------------------------------
// 1024 threads; wave w of the grid (gw) owns, per step, RPS rows:
//   EPI_RESID / EPI_STORE : rows gw * RPS + j + k * NW * RPS                              (NSTEP steps)
//   EPI_GATEUP            : RPS = 2: row i = gw + k * NW of W0 (gate) and of W1 (up)      (NSTEP steps)
//   EPI_QKV               : step 0: rows 2 gw, 2 gw + 1 of [W0; W1] (a RoPE pair), step 1: row gw of W2
// A step's rows of all 16 waves form one batch: phase 1 (all waves) -> barrier -> phase 2 (the first lanes, one per
// accumulator) -> barrier, per slab of 4096 elements of K; the accumulators stay in their lanes from slab to slab.
template <int WT, int NITK, int RPS, int NSTEP, int EPI, int WTV = WT>
__global__ __launch_bounds__(XG_THREADS) void xgemv_kernel(xg_args a) {
    constexpr bool NORM = (EPI != EPI_RESID);
    constexpr int NCH = xg_traits<WT>::NCH, NCHV = xg_traits<WTV>::NCH;
    constexpr int NROW = EPI == EPI_QKV ? 3 : RPS * NSTEP;                  // rows per wave
    constexpr int SLOTF = xg_slot_floats(NCH > NCHV ? NCH : NCHV);
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_sum;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int NW = (int)gridDim.x * XG_WAVES, gw = (int)blockIdx.x * XG_WAVES + wave;
    const int K = a.K, npair = K / 64;
    const size_t RB = (size_t)spy_row_size(WT, K);

    // row index (within its matrix) and base of the wave's row r (0 .. NROW-1); rows beyond the matrix re-read a valid row and are dropped in the epilogue
    auto row_of = [&](int r, bool &valid) -> int {
        if constexpr (EPI == EPI_QKV) { valid = gw < a.d; const int j = gw % a.d; return r == 2 ? j : ((2 * j) % a.d) + r; }
        else if constexpr (EPI == EPI_GATEUP) { const int u = gw + (r >> 1) * NW; valid = u < a.M; return valid ? u : gw % a.M; }
        else { const int u = (gw + (r / RPS) * NW) * RPS + (r % RPS); valid = u < a.M; return valid ? u : u % a.M; }
    };
    auto row_ptr = [&](int r) -> const uint8_t * {
        bool v; int i = row_of(r, v);
#ifdef XDBG_SMALLROWS
        i &= 255;                                   // measurement build: every workgroup re-reads the same cached rows
#endif
        if constexpr (EPI == EPI_QKV) {
            if (r == 2) return a.W2 + (size_t)i * spy_row_size(WTV, K);
            return (2 * (gw % a.d) < a.d ? a.W0 : a.W1) + (size_t)i * RB;
        } else if constexpr (EPI == EPI_GATEUP) return ((r & 1) ? a.W1 : a.W0) + (size_t)i * RB;
        else return a.W0 + (size_t)i * RB;
    };

    // 1. the activation vector, 2. the first rows (issue_first): all unconditional, in this order (the compute unit serves its requests in order)
    float4 xv[NITK], wv[NORM ? NITK : 1];
#pragma unroll
    for (int j = 0; j < NITK; j++) {
        const int i = min(tid + j * XG_THREADS, K / 4 - 1);
        xv[j] = ((const float4 *)a.x_in)[i];
        if constexpr (NORM) wv[j] = ((const float4 *)a.normw)[i];
    }
    // rows requested ahead of their use: all of the wave's rows where their registers allow (Q4_0 rows, up to 6), so
    // that the weights stream in while the serial sum of the norm is walked; XG_DEPTH otherwise
    // The sum of the norm in chunks (xg_exact_sum) pays where the wait that follows it is short: gate|up with three rows requested
    // ahead (17.1 against 18.5 us; with all six requested the waves sit in the issue stage for longer than the serial walk takes, and
    // the chunked sum gains nothing: 19.6).  It lost in the other kernels with a norm (qkv 13.2 against 12.7 at any depth, head 22.0
    // against 20.6).
    constexpr bool PSUM = XG_PSUM && EPI == EPI_GATEUP;
    constexpr int DEPTH = (!PSUM && NROW <= 6 && wt_traits<WT>::PAIR_DW * NITK <= 9) ? NROW : (XG_DEPTH < NROW ? XG_DEPTH : NROW);
    constexpr int RING = NROW < DEPTH + 1 ? NROW : DEPTH + 1;
    wtile<WT, NITK> t[RING];
    wtile<WTV, NITK> tv;
    auto issue = [&](int r) {
        if (EPI == EPI_QKV && r == 2) load_tile<WTV, 64, NITK>(tv, row_ptr(r), npair, lane);
        else load_tile<WT, 64, NITK>(t[r % RING], row_ptr(r), npair, lane);
    };
    auto issue_first = [&]() {
        if constexpr (!NORM) __builtin_amdgcn_s_barrier();      // x of every wave ahead of every wave's rows in the compute unit's memory queue
#pragma unroll
        for (int r = 0; r < NROW; r++) if (r < DEPTH) issue(r);
    };

    // 3. stage the activations (the first rows are requested inside: after the group sums of the norm, or at once)
    int8_t *s_q = (int8_t *)smem;
    int2 *s_meta = (int2 *)(smem + staged_q_bytes(K));
    float *s_part = (float *)(smem + ((staged_bytes(K) + 15) & ~(size_t)15));      // row slots; the group sums of the norm use the same bytes before
    XSTAMP(a.dbg, 16);
    xg_stage<NITK, NORM, PSUM>(xv, wv, K, a.eps, s_q, s_meta, s_part, &s_sum, issue_first);
    XSTAMP(a.dbg, 17);
    if (a.q8_dump && blockIdx.x == 0) xg_dump_q8(s_q, s_meta, K, a.q8_dump);
    staged_act act; act.q = s_q; act.meta = s_meta;

    constexpr int NSTEPS = EPI == EPI_QKV ? 2 : NSTEP;
    static_assert(NITK == 1 || NROW == 1, "rows longer than one slab are walked one row per wave");
    act_frag<1> af, av;
    int n8[16];
#pragma unroll
    for (int step = 0; step < NSTEPS; step++) {
        const int r0 = EPI == EPI_QKV ? 2 * step : step * RPS;                  // first row of the step
        const int rows = EPI == EPI_QKV ? 2 - step : RPS;
        const bool vstep = EPI == EPI_QKV && step == 1;
        const int nch = vstep ? NCHV : NCH;
        const int chains = XG_WAVES * rows * nch;
        float acc = 0.0f;
#pragma unroll
        for (int it = 0; it < NITK; it++) {
            const int nblk = min(XG_NBS, K / 32 - it * XG_NBS);                // blocks of this slab
            if (nblk > 0) {
                const int p = it * 64 + lane;
                // this lane's activations of the slab (the same for every row) and the -8 * sum q per dword: read once where the
                // rows are one slab long (every step uses the same ones), per slab otherwise
                if (NITK > 1 || step == 0) {
                    if (p < npair) {
                        load_act_frag<WT, 1>(af, act, npair, p);
                        if constexpr (WT == SPY_HIP_Q4_0) {
                            const int xs[16] = {af.x[0][0].x, af.x[0][0].y, af.x[0][0].z, af.x[0][0].w, af.x[0][1].x, af.x[0][1].y, af.x[0][1].z, af.x[0][1].w,
                                                af.x[0][2].x, af.x[0][2].y, af.x[0][2].z, af.x[0][2].w, af.x[0][3].x, af.x[0][3].y, af.x[0][3].z, af.x[0][3].w};
#pragma unroll
                            for (int i = 0; i < 16; i++) n8[i] = -8 * __builtin_amdgcn_sdot4(xs[i], 0x01010101, 0, false);
                        }
                    }
                }
                if constexpr (WTV != WT) { if (vstep && p < npair) load_act_frag<WTV, 1>(av, act, npair, p); }
#pragma unroll
                for (int j = 0; j < rows; j++) {
                    const int r = r0 + j;
                    if (it == 0 && r + DEPTH < NROW) issue(r + DEPTH);            // its ring slot held row r - 1, multiplied in the previous step
                    float *slot = s_part + (size_t)(wave * rows + j) * SLOTF;
                    if (p < npair) {
                        if (vstep) { if constexpr (WTV != WT) xg_phase1<WTV>(tv.w[it], av, n8, p, lane, slot); else xg_phase1<WTV>(tv.w[it], af, n8, p, lane, slot); }
                        else xg_phase1<WT>(t[r % RING].w[it], af, n8, p, lane, slot);
                    }
                }
                XSTAMP(a.dbg, 18 + 3 * (step * NITK + it));
                __syncthreads();
                XSTAMP(a.dbg, 19 + 3 * (step * NITK + it));
                if (tid < chains) {
                    const int slot_i = tid / nch, l = tid % nch;
                    const float *slot = s_part + (size_t)slot_i * SLOTF;
                    if (nch == 8) acc = xg_chain<8>(slot + l * (XG_NBS + 4), slot + nch * (XG_NBS + 4), nblk, acc);
                    else acc = xg_chain<1>(slot + l * (XG_NBS + 4), slot + nch * (XG_NBS + 4), nblk, acc);
                }
                XSTAMP(a.dbg, 20 + 3 * (step * NITK + it));
                __syncthreads();
            }
        }
        // epilogue of the step: the lanes that walked accumulator 0 of a row hold its total after the tree
        if (nch == 8) acc = xg_hsum8(acc);
        const bool owner = tid < chains && (tid % nch) == 0;
        const int slot_i = tid / nch;                                         // = wave_of_row * rows + j
        const int ow = slot_i / rows, oj = slot_i % rows;                      // the wave that owned the row and its index in the step
        const int ogw = (int)blockIdx.x * XG_WAVES + ow;
        if constexpr (EPI == EPI_RESID || EPI == EPI_STORE) {
            const int u = (ogw + step * NW) * RPS + oj;
            if (owner && u < a.M) a.out[u] = (EPI == EPI_RESID && a.resid) ? acc + a.resid[u] : acc;       // Add(KQV_linear, x) / Add(ffn_out, ffn_input); no resid: the MatMul alone
        } else if constexpr (EPI == EPI_GATEUP) {
            const float up = __shfl_xor(acc, nch, SPY_WAVE);                   // the row after (up_i) sits nch lanes further
            const int i = ogw + step * NW;
            if (owner && oj == 0 && i < a.M) a.out[i] = up * a.lut[65536 + f2h(acc)];             // Mul(ffn_up, Silu(ffn_gate)) (ffn.cpp:24-35, non-linear.cpp:11-14)
        } else {
            const int pos = a.st ? a.st->pos : a.pos_imm;
            const float *rt = a.rope_tab + (size_t)(pos - a.rope_row0) * a.hd;
            if (step == 0) {
                const float x1 = __shfl_xor(acc, nch, SPY_WAVE);
                if (owner && oj == 0 && ogw < a.d) {
                    const int row = (2 * ogw) % a.d, k2 = row % a.hd;
                    const float c = rt[k2], sn = rt[k2 + 1];
                    // (x0, x1) -> (x0*c - x1*s, x0*s + x1*c), every product rounded (non-linear.cpp:349-364)
                    const float pa_ = acc * c, pb_ = x1 * sn, pc_ = acc * sn, pd_ = x1 * c;
                    const uint32_t pr = (uint32_t)f2h(pa_ - pb_) | ((uint32_t)f2h(pc_ + pd_) << 16);
                    if (2 * ogw < a.d) ((uint32_t *)a.q16)[ogw] = pr;                                  // attn_score rounds Q to fp16 (mat.cpp:37)
                    else ((uint32_t *)(a.kc + (size_t)pos * a.d))[ogw - a.d / 2] = pr;                 // KCache_cpy: [token][head][hd]
                }
            } else {
                if (owner && ogw < a.d) a.vc[(size_t)ogw * a.n_ctx + pos] = f2h(acc);                 // VCache_cpy: [d][C] column pos
            }
        }
    }
}

// ---- attention scores in the order of Dot<FP16,FP16> -------------------------------------------------------------------
// The cached tokens are dealt out evenly over the workgroups (one per compute unit): workgroup b takes tokens
// b * tpw .. (b + 1) * tpw - 1, tpw = ceil(n_kv / workgroups), all heads, in rounds of XS_TOK tokens.  The keys of a round
// (8 KiB per token, [head][128] fp16) are read coalesced, XS_NLD 16-byte pieces per thread all requested at once and a
// round ahead of their use, and laid into LDS; then ONE thread per (token, head) key walks the dot exactly as vec_dot.h:124-145 does for n = 128:
// accumulators sum[j][l] over the chunks i = 0, 32, 64 (i + 32 < n), the reduction tree of FP16::block_reduce, then the
// scalar tail over elements 96..127 (a product of two fp16 values is exact in fp32, so `tail += a * b` is the fma it is
// written as here), result = tail + simd.  Stored: t = dot * scale (mask 0, then * scale: non-linear.cpp:141-150).
#define XS_THREADS 1024
#define XS_TOK 18
#define XS_NLD 9                                        // pieces per thread requested together: 1024 x 9 x 16 bytes = 18 tokens of 32 heads
static inline size_t xattn_scores_lds(int n_head) { return (size_t)(XS_TOK + 1) * n_head * 16 * 16; }
// kc is not a restrict pointer on purpose: the loads of the next round must stay where they are written, ahead of the
// barrier and the dots of the current round, so that they are in flight meanwhile.
template <int DUMMY>
__global__ __launch_bounds__(XS_THREADS) void xattn_scores_kernel(const dev_state *st, int pos_imm, const uint16_t *__restrict__ q16, const uint16_t *kc,
                                                                  float *__restrict__ scores, int n_head, int n_ctx, float scale) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int n_kv = (st ? st->pos : pos_imm) + 1;
    const int tpw = (n_kv + (int)gridDim.x - 1) / (int)gridDim.x;
    const int t_begin = blockIdx.x * tpw, t_end = min(n_kv, t_begin + tpw);
    if (t_begin >= t_end) return;
    const int d = n_head * 128, tid = threadIdx.x;
    uint4 *s_k = (uint4 *)smem;                         // [XS_TOK][n_head][16 chunks of 16 bytes], chunk index rotated per key against bank conflicts
    uint4 *s_qh = s_k + XS_TOK * n_head * 16;           // [n_head][16]
    const int per_tok = n_head * 16;                    // 16-byte pieces per token
    // the pieces in flight: named registers (an indexed array that lives across the rounds ends up in scratch memory)
    uint4 k0, k1, k2, k3, k4, k5, k6, k7, k8;
    static_assert(XS_NLD == 9, "nine named registers");
#define XS_EACH(X) X(0, k0) X(1, k1) X(2, k2) X(3, k3) X(4, k4) X(5, k5) X(6, k6) X(7, k7) X(8, k8)
    auto request = [&](int t0, int npiece, int c0) {
#define XS_REQ(u, r) { const int c = min(c0 + u * XS_THREADS + tid, npiece - 1); const int tt = c / per_tok, rem = c - tt * per_tok; \
                       r = *(const uint4 *)(kc + (size_t)(t0 + tt) * d + rem * 8); }
        XS_EACH(XS_REQ)
#undef XS_REQ
    };
    auto lay = [&](int npiece, int c0) {
#define XS_LAY(u, r) { const int c = c0 + u * XS_THREADS + tid; \
                       if (c < npiece) { const int tt = c / per_tok, rem = c - tt * per_tok, hh = rem >> 4, ch = rem & 15; \
                                         s_k[(tt * n_head + hh) * 16 + ((ch + tt + 8 * (hh & 1)) & 15)] = r; } }
        XS_EACH(XS_LAY)
#undef XS_LAY
    };
#undef XS_EACH
    request(t_begin, min(XS_TOK, t_end - t_begin) * per_tok, 0);
    for (int c = tid; c < per_tok; c += XS_THREADS) s_qh[c] = *(const uint4 *)(q16 + c * 8);
    for (int t0 = t_begin; t0 < t_end; t0 += XS_TOK) {
        const int nt = min(XS_TOK, t_end - t0), npiece = nt * per_tok;
        if (t0 != t_begin) __syncthreads();             // the previous round's keys have been read
        lay(npiece, 0);                                 // the first batch of the round was requested a round ahead
        for (int c0 = XS_NLD * XS_THREADS; c0 < npiece; c0 += XS_NLD * XS_THREADS) { request(t0, npiece, c0); lay(npiece, c0); }
        if (t0 + XS_TOK < t_end) request(t0 + XS_TOK, min(XS_TOK, t_end - t0 - XS_TOK) * per_tok, 0);
        __syncthreads();
        for (int key = tid; key < nt * n_head; key += XS_THREADS) {
            const int hh = key / nt, tt = key - hh * nt;
            const uint4 *kp = s_k + (tt * n_head + hh) * 16, *qp = s_qh + hh * 16;
            const int rot = tt + 8 * (hh & 1);
            float sum[4][8];
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int l = 0; l < 8; l++) sum[j][l] = 0.0f;
#pragma unroll
            for (int i = 0; i < 3; i++) {                // chunks of 32 elements = 4 x 16 bytes
                __builtin_amdgcn_sched_barrier(0);      // one chunk's LDS reads at a time: the next round's keys occupy registers meanwhile
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint4 kv = kp[(4 * i + j + rot) & 15], qv = qp[4 * i + j];
                    const uint32_t kw[4] = {kv.x, kv.y, kv.z, kv.w}, qw[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        sum[j][2 * e] = fmaf(h2f((uint16_t)(kw[e] & 0xFFFFu)), h2f((uint16_t)(qw[e] & 0xFFFFu)), sum[j][2 * e]);
                        sum[j][2 * e + 1] = fmaf(h2f((uint16_t)(kw[e] >> 16)), h2f((uint16_t)(qw[e] >> 16)), sum[j][2 * e + 1]);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int l = 0; l < 8; l++) { sum[0][l] += sum[2][l]; sum[1][l] += sum[3][l]; }
#pragma unroll
            for (int l = 0; l < 8; l++) sum[0][l] += sum[1][l];
            const float u0 = sum[0][0] + sum[0][4], u1 = sum[0][1] + sum[0][5], u2 = sum[0][2] + sum[0][6], u3 = sum[0][3] + sum[0][7];
            const float v0 = u0 + u1, v1 = u2 + u3;
            const float simd = v0 + v1;
            float tail = 0.0f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint4 kv = kp[(12 + j + rot) & 15], qv = qp[12 + j];
                const uint32_t kw[4] = {kv.x, kv.y, kv.z, kv.w}, qw[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    tail = fmaf(h2f((uint16_t)(kw[e] & 0xFFFFu)), h2f((uint16_t)(qw[e] & 0xFFFFu)), tail);
                    tail = fmaf(h2f((uint16_t)(kw[e] >> 16)), h2f((uint16_t)(qw[e] >> 16)), tail);
                }
            }
            scores[(size_t)hh * n_ctx + t0 + tt] = (tail + simd) * scale;
        }
    }
}

// ---- softmax + P.V^T in the host order ---------------------------------------------------------------------------------
// One 1024-thread workgroup per (head, 16 rows of V^T); wave w streams row w into registers (16-byte pieces, all requested
// before the softmax's serial sum so that the row arrives while that sum is walked).
// Softmax (non-linear.cpp:129-180): m = max t; e = exp_table[fp16(t - m)]; sum = std::reduce(e) = groups of four added to
// one running sum, then the last n % 4 elements; p = e * (1 / sum), rounded to fp16 for the product (mat.cpp:37).
// P.V^T (vec_dot.h:124-145 with n = n_kv): output row r has 4 x 8 accumulators, accumulator (j, l) adds elements
// 32 i + 8 j + l for every chunk with 32 i + 32 < n_kv.  The 16 waves lay their rows into LDS; then 32 lanes hold the
// accumulators of one row (two rows per wave, the 16 rows in waves 0..7) and read V^T and P from LDS; tree; scalar tail (the
// last 1..32 elements, by the lane of accumulator 0).
#define XP_THREADS 1024
#define XP_NP 10                           // 16-byte pieces per lane of a V^T row: n_ctx <= 5120
#ifndef XP_PSUM
#define XP_PSUM 0                          // the softmax sum through xg_exact_sum: 4.1 instead of 4.9 us for the sum, but the V^T rows are then requested later and the kernel takes 15.2 instead of 14.0 us
#endif
#define XP_NS 5                            // scores per thread: n_ctx <= 5120
static inline int xattn_pv_vstride(int n_ctx) { return ((n_ctx + 63) / 64) * 64 + 32; }        // halfs between rows in LDS: = 64 bytes mod 128, the two rows of a wave on different banks
static inline size_t xattn_pv_lds(int n_ctx) {
    const size_t p_bytes = (size_t)((n_ctx + 32 + 7) & ~7) * 2, v_bytes = (size_t)16 * xattn_pv_vstride(n_ctx) * 2 + 1024;      // + the walk's read-ahead
    const size_t soft = (size_t)n_ctx * 4 + (size_t)((n_ctx / 4 + 3) & ~3) * 4;                  // t / e and the group sums live where the rows go later
    return p_bytes + (v_bytes > soft ? v_bytes : soft);
}
template <int DUMMY>
__global__ __launch_bounds__(XP_THREADS) void xattn_pv_kernel(const dev_state *st, int pos_imm, const float *__restrict__ scores, const uint16_t *vc,
                                                              float *attn_out, const float *__restrict__ lut, int n_ctx, long long *dbg) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[16];
    __shared__ float s_sum;
    XSTAMP(dbg, 0);
    const int n_kv = (st ? st->pos : pos_imm) + 1;
    const int hd_ = blockIdx.x >> 3, dgrp = blockIdx.x & 7;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int VS = ((n_ctx + 63) / 64) * 64 + 32;
    uint16_t *s_p = (uint16_t *)smem;                                 // n_ctx + 32 halfs: the probabilities as fp16
    uint8_t *region = smem + (size_t)((n_ctx + 32 + 7) & ~7) * 2;
    float *s_e = (float *)region;                                     // n_ctx floats: e (softmax phase)
    float *s_grp = s_e + n_ctx;                                       // n_ctx / 4 group sums
    uint16_t *s_v = (uint16_t *)region;                               // 16 rows x VS halfs (product phase)
    const float *srow = scores + (size_t)hd_ * n_ctx;
    const uint16_t *vrow = vc + (size_t)(hd_ * 128 + dgrp * 16 + wave) * n_ctx;
    // ---- softmax: scores -> registers, maximum ----
    float sreg[XP_NS];
#pragma unroll
    for (int u = 0; u < XP_NS; u++) sreg[u] = srow[min(tid + u * XP_THREADS, n_ctx - 1)];
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < XP_NS; u++) if (tid + u * XP_THREADS < n_kv) mx = fmaxf(mx, sreg[u]);
    mx = wave_max(mx);
    if (lane == 0) s_red[wave] = mx;
    __syncthreads();
    mx = s_red[0];
#pragma unroll
    for (int w = 1; w < 16; w++) mx = fmaxf(mx, s_red[w]);
    XSTAMP(dbg, 1);
    // exponentials from the table
#pragma unroll
    for (int u = 0; u < XP_NS; u++) sreg[u] = lut[f2h(sreg[u] - mx)];
#pragma unroll
    for (int u = 0; u < XP_NS; u++) { const int j = tid + u * XP_THREADS; if (j < n_kv) s_e[j] = sreg[u]; }
    __syncthreads();
    XSTAMP(dbg, 2);
    const int ngrp = n_kv / 4;
    float grp[2];
    static_assert(XP_NS * XP_THREADS / 4 <= 2 * XP_THREADS, "two group sums per thread");
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int g = tid + u * XP_THREADS;
        grp[u] = 0.0f;
        if (g < ngrp) {
            const float4 v = *(const float4 *)(s_e + 4 * g);
            const float v1 = v.x + v.y, v2 = v.z + v.w;
            grp[u] = v1 + v2;
            s_grp[g] = grp[u];
        }
    }
    if (!XP_PSUM) __syncthreads();
    XSTAMP(dbg, 3);
    // The V^T rows are requested now, by every wave but the one that walks the sum (a wave that asks for its whole row sits in the
    // issue stage until the memory queue has room, i.e. for most of the row's transfer time): the rows arrive while the sum is walked.
    // vc is not a restrict pointer on purpose: the loads must stay between the two barriers around them.
    uint4 vb0, vb1, vb2, vb3, vb4, vb5, vb6, vb7, vb8, vb9;
    const int last_piece = (n_kv - 1) >> 3;
    auto load_row = [&]() {
        const uint16_t *vp = vrow;
        vb0 = *(const uint4 *)(vp + (size_t)min(0 * 64 + lane, last_piece) * 8); vb1 = *(const uint4 *)(vp + (size_t)min(1 * 64 + lane, last_piece) * 8);
        vb2 = *(const uint4 *)(vp + (size_t)min(2 * 64 + lane, last_piece) * 8); vb3 = *(const uint4 *)(vp + (size_t)min(3 * 64 + lane, last_piece) * 8);
        vb4 = *(const uint4 *)(vp + (size_t)min(4 * 64 + lane, last_piece) * 8); vb5 = *(const uint4 *)(vp + (size_t)min(5 * 64 + lane, last_piece) * 8);
        vb6 = *(const uint4 *)(vp + (size_t)min(6 * 64 + lane, last_piece) * 8); vb7 = *(const uint4 *)(vp + (size_t)min(7 * 64 + lane, last_piece) * 8);
        vb8 = *(const uint4 *)(vp + (size_t)min(8 * 64 + lane, last_piece) * 8); vb9 = *(const uint4 *)(vp + (size_t)min(9 * 64 + lane, last_piece) * 8);
    };
    if (XP_PSUM) {
        xg_psum_lds *L = (xg_psum_lds *)(s_grp + ((n_ctx / 4 + 3) & ~3) + 64);
        float init = xg_exact_sum<2>(grp, ngrp, s_grp, L, 0.0f, load_row, dbg);
        if (wave == 0) {
            for (int j = ngrp * 4; j < n_kv; j++) init = init + s_e[j];
            if (lane == 0) s_sum = init;
            load_row();
        }
    } else if (wave != 0) load_row();
    else {
        float init = xg_serial_sum(s_grp, ngrp, 0.0f);
        for (int j = ngrp * 4; j < n_kv; j++) init = init + s_e[j];
        if (lane == 0) s_sum = init;
        load_row();
    }
    __syncthreads();
    XSTAMP(dbg, 4);
    const float inv = 1.0f / s_sum;
#pragma unroll
    for (int u = 0; u < XP_NS; u++) { const int j = tid + u * XP_THREADS; if (j < n_kv) s_p[j] = f2h(sreg[u] * inv); }
    // ---- the rows into LDS (s_e / s_grp are dead: every thread passed the barrier after the sum) ----
    {
        uint16_t *dst = s_v + (size_t)wave * VS + lane * 8;
        if (0 * 64 + lane <= last_piece) *(uint4 *)(dst + 0 * 512) = vb0;
        if (1 * 64 + lane <= last_piece) *(uint4 *)(dst + 1 * 512) = vb1;
        if (2 * 64 + lane <= last_piece) *(uint4 *)(dst + 2 * 512) = vb2;
        if (3 * 64 + lane <= last_piece) *(uint4 *)(dst + 3 * 512) = vb3;
        if (4 * 64 + lane <= last_piece) *(uint4 *)(dst + 4 * 512) = vb4;
        if (5 * 64 + lane <= last_piece) *(uint4 *)(dst + 5 * 512) = vb5;
        if (6 * 64 + lane <= last_piece) *(uint4 *)(dst + 6 * 512) = vb6;
        if (7 * 64 + lane <= last_piece) *(uint4 *)(dst + 7 * 512) = vb7;
        if (8 * 64 + lane <= last_piece) *(uint4 *)(dst + 8 * 512) = vb8;
        if (9 * 64 + lane <= last_piece) *(uint4 *)(dst + 9 * 512) = vb9;
    }
    __syncthreads();
    XSTAMP(dbg, 5);
    // ---- P . V^T ----
    // One lane per accumulator: each step is two 16-bit LDS reads and one fma that takes the fp16 operands as they are; a
    // wave issues an instruction every 2.6 ns or so whatever the other waves do, so the walk is spread over eight waves.
    if (wave < 8) {
        const int nfull = (n_kv - 1) / 32;                            // chunks with 32 i + 32 < n_kv
        const int r16 = wave * 2 + (lane >> 5), cl = lane & 31;       // row of the 16 and accumulator 8 j + l
        const _Float16 *vr = (const _Float16 *)s_v + (size_t)r16 * VS + cl, *pr = (const _Float16 *)s_p + cl;
        float acc = 0.0f;
        const int ntail = n_kv - 32 * nfull;                          // 1 .. 32
        const float tprod = cl < ntail ? (float)vr[32 * nfull] * (float)pr[32 * nfull] : 0.0f;
        _Float16 va[8], pa[8], vb[8], pb[8];
        auto ld = [&](_Float16 (&v)[8], _Float16 (&q)[8], int i) {   // up to 16 chunks beyond nfull are read and not used: the next row, or the slack after the last
#pragma unroll
            for (int u = 0; u < 8; u++) { v[u] = vr[32 * (i + u)]; q[u] = pr[32 * (i + u)]; }
        };
        auto run = [&](const _Float16 (&v)[8], const _Float16 (&q)[8]) {
#pragma unroll
            for (int u = 0; u < 8; u++) acc = fmaf((float)v[u], (float)q[u], acc);
        };
        int i = 0;
        const int n16 = nfull - nfull % 16;
        if (n16) {
            ld(va, pa, 0);
            for (; i < n16; i += 16) {
                ld(vb, pb, i + 8);
                __builtin_amdgcn_sched_barrier(0);
                run(va, pa);
                __builtin_amdgcn_sched_barrier(0);
                ld(va, pa, i + 16);
                __builtin_amdgcn_sched_barrier(0);
                run(vb, pb);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        for (; i < nfull; i++) acc = fmaf((float)vr[32 * i], (float)pr[32 * i], acc);
        XSTAMP(dbg, 6);
        acc += __shfl_xor(acc, 16, SPY_WAVE);         // sum[0] += sum[2], sum[1] += sum[3]
        acc += __shfl_xor(acc, 8, SPY_WAVE);          // sum[0] += sum[1]
        acc += __shfl_xor(acc, 4, SPY_WAVE);          // t_l = sum[0][l] + sum[0][l + 4]
        acc += __shfl_xor(acc, 1, SPY_WAVE);          // t_0 + t_1, t_2 + t_3
        acc += __shfl_xor(acc, 2, SPY_WAVE);          // (t_0 + t_1) + (t_2 + t_3)
        // the scalar tail: elements 32 nfull .. n_kv - 1, one after the other.  A product of two fp16 values is exact in fp32, so
        // `tail = fma(v, p, tail)` is `tail + v * p` with the product formed beforehand: lane cl forms the product of element
        // 32 nfull + cl (operands read before the walk above), the 32 products are fetched with wave permutes that do not depend
        // on each other, and what remains serial is one addition per element.
        float tp[32];
#pragma unroll
        for (int e = 0; e < 32; e++) tp[e] = __shfl(tprod, (lane & 32) + e, SPY_WAVE);
        float tail = 0.0f;
#pragma unroll
        for (int e = 0; e < 32; e++) if (e < ntail) tail = tail + tp[e];
        if (cl == 0) attn_out[hd_ * 128 + dgrp * 16 + r16] = tail + acc;
        XSTAMP(dbg, 7);
    }
}
