// The whole single-token pass as ONE persistent kernel: one 1024-thread workgroup per compute unit,
// the six phases of a layer (qkv, scores, softmax+PV, wo, gate|up, down) separated by grid barriers,
// and the weight / KV-cache rows of the NEXT phase requested before each barrier so that HBM keeps
// streaming while the barrier and the activation staging of the next phase run.
//
// Arithmetic is the same as in the per-phase kernels of decode_kernels.cuh (same rounding points of
// the operator graph, same reduction trees), so both paths give the same results.
//
// Work split (NW = 16 * gridDim.x waves): one weight row per wave and step, 64 lanes x one block
// pair (36 / 68 bytes) each:
//   qkv     : wave j -> rows 2j, 2j+1 of [wq; wk] (a RoPE pair) and row j of wv
//   scores  : unit u = (token, group of 4 heads) = 1 KiB of the K cache; wave takes u = gw + k*NW
//   pv      : wave r -> V^T row r (one head dim, contiguous over tokens); a workgroup = 16 rows of one head
//   wo/down : wave r -> row r;   gate|up: wave i -> rows gate_i, up_i (i = gw + k*NW);   head: r = gw + k*NW
//
// Memory visibility between workgroups (different XCDs do not share an L2): everything one phase
// hands to the next is written with agent-scope atomic stores by wave 0 of the workgroup, which
// waits for their completion before it arrives at the barrier, and read with agent-scope atomic
// loads after it.  Waves 0..3 ("late" waves) never have a prefetch outstanding at a barrier: vector
// loads return in order, so only a wave without older loads in flight can poll the barrier flag or
// fetch the new activations quickly; they stage the activations for everybody and request their own
// rows right after.
#pragma once

#include "decode_kernels.cuh"

#define MEGA_THREADS 1024
#define MEGA_WAVES 16
#define MEGA_LATE 4                 // waves that stage activations (256 threads)
#define MEGA_FAN 16                 // workgroups per leaf counter of the barrier
#define MEGA_MAX_LEAF 64
#define MEGA_RS 10                  // K-cache units per wave in the scores phase
#define MEGA_RV 10                  // 128-bit pieces per lane of a V^T row (64 lanes x 8 tokens each)
#define MEGA_DEPTH 3                // gate|up row buffers requested ahead of their use
#define MEGA_SLOTS 40               // results per wave and phase handed to wave 0 through LDS

struct mega_sync {                  // zero-initialised once; every counter on its own 128-byte line
    uint32_t leaf[MEGA_MAX_LEAF][32];
    uint32_t top[32];
    uint32_t flag[32];
    uint32_t epoch[32];             // barriers completed by earlier launches
};

struct mega_layer {
    const uint8_t *wq, *wk, *wv, *wo, *w_gate, *w_up, *w_down;
    const float *attn_norm, *ffn_norm;
    uint16_t *kc, *vc;
};

struct mega_args {
    const mega_layer *layers;
    int n_layer, d, F, H, hd, n_ctx, n_vocab;
    float eps, theta_scale, att_scale;
    const uint8_t *tok_embd; int embd_q8;
    const float *out_norm; const uint8_t *w_out;
    dev_state *st; mega_sync *sync;
    float *x, *x1, *attn_out, *hbuf, *scores, *logits;
    uint16_t *q16;
    uint32_t spin_limit;
    long long *dbg;                 // optional: wall-clock stamps (10 ns units) of layer 1's phases from two workgroups
};

template <int WT> struct mega_traits {
    static constexpr int RH = 4;                                  // head rows per wave and batch
    static constexpr int RG = (WT == SPY_HIP_Q4_0) ? 3 : 2;     // gate|up row pairs per wave
};

static __host__ __device__ inline size_t mega_lds_bytes(int d, int F, int hd, int n_ctx) {
    const int kmax = d > F ? d : F;
    size_t n = staged_bytes(kmax);                       // staged activations
    n += (size_t)hd * 4;                                 // RoPE cos|sin
    n += (size_t)MEGA_WAVES * MEGA_SLOTS * 4;            // results for wave 0
    n += (size_t)n_ctx * 4 + (size_t)n_ctx * 2 + 16;     // softmax: t (f32), p (f16)
    n += (size_t)d * 2;                                  // q (f16)
    return (n + 15) & ~(size_t)15;
}

// Grid barrier number b (1-based, counts up over the life of the sync block, wraps).  Called by
// thread 0 of every workgroup after its stores have completed.  Arrivals go to MEGA_FAN-way leaf
// counters, the last arrival of a leaf to the top counter, the last of those publishes b in the
// flag everybody polls.  The poll is bounded: on expiry the error flag is raised and every
// workgroup leaves the kernel.
static __device__ __forceinline__ bool mega_arrive_and_wait(mega_sync *s, dev_state *st, uint32_t b, uint32_t G, uint32_t spin_limit) {
    const uint32_t nleaf = (G + MEGA_FAN - 1) / MEGA_FAN, leaf = blockIdx.x / MEGA_FAN;
    const uint32_t members = (leaf == nleaf - 1) ? G - leaf * MEGA_FAN : MEGA_FAN;
    const uint32_t v = __hip_atomic_fetch_add(&s->leaf[leaf][0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (v + 1u == members * b) {
        const uint32_t t = __hip_atomic_fetch_add(&s->top[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (t + 1u == nleaf * b) __hip_atomic_store(&s->flag[0], b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    uint32_t spins = 0;
    while ((int32_t)(__hip_atomic_load(&s->flag[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - b) < 0) {
        if (++spins > spin_limit) { __hip_atomic_store(&st->err, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); return false; }
        __builtin_amdgcn_s_sleep(2);
    }
    return true;
}

template <int WT, int NITF>
__global__ __launch_bounds__(MEGA_THREADS) void mega_decode_kernel(mega_args a) {
    constexpr int RH = mega_traits<WT>::RH, RG = mega_traits<WT>::RG;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ float s_red[MEGA_WAVES];
    __shared__ int s_ok;

    const int d = a.d, F = a.F, hd = a.hd, H = a.H, n_ctx = a.n_ctx, V = a.n_vocab;
    const int kmax = d > F ? d : F;
    int8_t *s_q = (int8_t *)smem;
    int2 *s_meta = (int2 *)(smem + staged_q_bytes(kmax));
    float *s_rope = (float *)(smem + staged_bytes(kmax));
    float *s_out = s_rope + hd;                                   // [MEGA_WAVES][MEGA_SLOTS]
    float *s_t = s_out + MEGA_WAVES * MEGA_SLOTS;                 // n_ctx
    uint16_t *s_p = (uint16_t *)(s_t + n_ctx);                    // n_ctx (+8)
    uint16_t *s_q16 = s_p + n_ctx + 8;                            // d
    staged_act act; act.q = s_q; act.meta = s_meta;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t G = gridDim.x;
    const int NW = (int)G * MEGA_WAVES, gw = (int)blockIdx.x * MEGA_WAVES + wave;
    const bool late = wave < MEGA_LATE;
    const int pos = a.st->pos, n_kv = pos + 1;
    int tok = a.st->token;
    if (tok < 0 || tok >= V) { if (blockIdx.x == 0 && tid == 0) a.st->err = 1; tok = 0; }
    uint32_t bar = ldc(&a.sync->epoch[0]);                        // barriers done before this launch

    const int npd = d / 64, npf = F / 64;
    const size_t RBd = (size_t)(d / 32) * wt_traits<WT>::BLK, RBf = (size_t)(F / 32) * wt_traits<WT>::BLK;
    const int HG = H / 4;

    // RoPE table of this position: theta_0 = pos, theta_{k+1} = theta_k * theta_scale in fp32
    // (non-linear.cpp:304-309 in the Spy tree), cosf / sinf of it
    if (tid < hd / 2) {
        float theta = (float)pos;
        for (int j = 0; j < tid; j++) theta *= a.theta_scale;
        s_rope[2 * tid] = cosf(theta);
        s_rope[2 * tid + 1] = sinf(theta);
    }

    int dbg_n = 0, dbg_layer = -1;
    auto stamp = [&]() {
        if (a.dbg && dbg_layer == 1 && tid == 0 && (blockIdx.x == 0 || blockIdx.x == 100) && dbg_n < 64)
            a.dbg[(blockIdx.x == 0 ? 0 : 64) + dbg_n] = wall_clock64();
        ++dbg_n;
    };
    // ---- helpers ---------------------------------------------------------------------------------
    // wave 0 writes the workgroup's results, waits for the stores, thread 0 goes through the barrier
    auto publish_and_sync = [&](auto writer) -> bool {
        stamp();
        ++bar;
        __syncthreads();                                  // every wave's results are in s_out
        if (wave == 0) {
            writer();
            __builtin_amdgcn_s_waitcnt(0);                // the stores above have completed
            if (lane == 0) s_ok = mega_arrive_and_wait(a.sync, a.st, bar, G, a.spin_limit) ? 1 : 0;
        }
        __syncthreads();
        stamp();
        return s_ok != 0;
    };
    // RMSNorm * weight -> Q8_0 in LDS by the late waves (d <= 4096: four float4 per thread);
    // NormRMS as non-linear.cpp:216-219, the weight Mul as its own rounding step
    auto stage_norm = [&](const float4 (&xv)[4], const float *normw) {
        float4 wv[4];
        float acc = 0.0f;
        if (late) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int i = min(tid + j * 256, d / 4 - 1);
                wv[j] = ((const float4 *)normw)[i];
                if (tid + j * 256 < d / 4) { const float4 v = xv[j]; acc = fmaf(v.x, v.x, acc); acc = fmaf(v.y, v.y, acc); acc = fmaf(v.z, v.z, acc); acc = fmaf(v.w, v.w, acc); }
            }
            acc = group_sum<64>(acc);
            if (lane == 0) s_red[wave] = acc;
        }
        __syncthreads();
        if (late) {
            const float sum = (s_red[0] + s_red[1]) + (s_red[2] + s_red[3]);
            const float scale = 1.0f / sqrtf(sum / (float)d + a.eps);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int i = tid + j * 256;
                if (i < d / 4) {
                    float4 v = xv[j];
                    const float4 w = wv[j];
                    v.x = (v.x * scale) * w.x; v.y = (v.y * scale) * w.y; v.z = (v.z * scale) * w.z; v.w = (v.w * scale) * w.w;
                    int2 meta;
                    const uint32_t q = quantize_oct(v, meta);
                    ((uint32_t *)s_q)[act_dw(i, d >> 6)] = q;
                    if ((tid & 7) == 0) s_meta[i >> 3] = meta;
                }
            }
        }
        __syncthreads();
    };
    // plain f32 vector (already in registers, NV float4 per late thread) -> Q8_0 in LDS
    auto stage_plain = [&](auto &pv, int K) {
        constexpr int NV = sizeof(pv) / sizeof(float4);
        if (late) {
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const int i = tid + j * 256;
                if (i < K / 4) {
                    int2 meta;
                    const uint32_t q = quantize_oct(pv[j], meta);
                    ((uint32_t *)s_q)[act_dw(i, K >> 6)] = q;
                    if ((tid & 7) == 0) s_meta[i >> 3] = meta;
                }
            }
        }
        __syncthreads();
    };
    auto load_x4 = [&](float4 (&xv)[4], const float *src) {          // late waves: d floats, coherent
#pragma unroll
        for (int j = 0; j < 4; j++) xv[j] = ldc4(src + 4 * min(tid + j * 256, d / 4 - 1));
    };
    auto row_dot_d = [&](const wtile<WT, 1> &t) -> float {
        float acc[1] = {0.0f};
        dot_tile<WT, 64, 1, 1>(t, &act, npd, lane, acc, nullptr);
        return group_sum<64>(acc[0]);
    };

    // Every buffer below is written at two program points: before a barrier by the early waves and
    // after it by the late ones.  At the first point the late waves clear it instead, so that the
    // compiler sees a definition on every path and does not keep the registers reserved before it.
    auto clear_tile = [&](auto &t) {
        uint32_t *p = (uint32_t *)&t;
#pragma unroll
        for (int i = 0; i < (int)(sizeof(t) / 4); i++) p[i] = 0u;
    };

    // ---- buffers that live across barriers (the prefetched rows of the next phase) -----------------
    wtile<WT, 1> wq0, wq1, wq2;                 // qkv: rows 2j, 2j+1, v row j
    uint4 kb[MEGA_RS];                          // scores: K-cache units
    uint4 vb[MEGA_RV];                          // pv: V^T row pieces
    wtile<WT, 1> wo0;                           // wo row
    wtile<WT, 1> wg[2 * RG];                    // gate|up rows
    wtile<WT, NITF> wd0;                        // down row
    wtile<WT, 1> wh[RH];                        // head rows

    auto fetch_qkv = [&](const mega_layer &L) {
        const int j = gw % d;                   // waves beyond the matrix re-read other rows (unused)
        const bool isq = 2 * j < d;
        const uint8_t *p0 = isq ? L.wq + (size_t)(2 * j) * RBd : L.wk + (size_t)(2 * j - d) * RBd;
        load_tile<WT, 64, 1>(wq0, p0, npd, lane);
        load_tile<WT, 64, 1>(wq1, p0 + RBd, npd, lane);
        load_tile<WT, 64, 1>(wq2, L.wv + (size_t)j * RBd, npd, lane);
    };
    auto fetch_scores = [&](const mega_layer &L) {
        const int nunit = n_kv * HG;
#pragma unroll
        for (int k = 0; k < MEGA_RS; k++) {
            const int u = (gw + k * NW) % nunit;
            const int token = u / HG, hg = u - token * HG;
            kb[k] = *(const uint4 *)(L.kc + (size_t)token * d + hg * 512 + lane * 8);
        }
    };
    auto fetch_v = [&](const mega_layer &L) {
        const uint16_t *vrow = L.vc + (size_t)(gw % d) * n_ctx;
#pragma unroll
        for (int i = 0; i < MEGA_RV; i++) vb[i] = *(const uint4 *)(vrow + (size_t)min(i * 64 + lane, n_ctx / 8 - 1) * 8);
    };
    auto fetch_wo = [&](const mega_layer &L) { load_tile<WT, 64, 1>(wo0, L.wo + (size_t)(gw % d) * RBd, npd, lane); };
    // buffers [b0, b1) of a gate|up batch: buffer 2k = gate row, 2k+1 = up row of pair k0 + k.  Only
    // MEGA_DEPTH buffers are requested ahead of their use (the vector-memory queue of a compute unit
    // is finite; whatever waits behind a deep prefetch -- barrier polls, activation loads -- waits long).
    auto fetch_gateup = [&](const mega_layer &L, int k0, int b0, int b1) {
#pragma unroll
        for (int b = 0; b < 2 * RG; b++) {
            if (b >= b0 && b < b1) {
                const int u = gw + (k0 + (b >> 1)) * NW, i = u < F ? u : gw % F;
                load_tile<WT, 64, 1>(wg[b], ((b & 1) ? L.w_up : L.w_gate) + (size_t)i * RBd, npd, lane);
            }
        }
    };
    auto fetch_down = [&](const mega_layer &L) { load_tile<WT, 64, NITF>(wd0, L.w_down + (size_t)(gw % d) * RBf, npf, lane); };
    auto fetch_head = [&](int k0) {
#pragma unroll
        for (int k = 0; k < RH; k++) { const int u = gw + (k0 + k) * NW; load_tile<WT, 64, 1>(wh[k], a.w_out + (size_t)(u < V ? u : gw % V) * RBd, npd, lane); }
    };

    // ---- layer 0 input: the embedding row (GetRow, view.cpp:33-81: F32 copy or Q8_0 dequant) -----
    float4 xv[4];
    clear_tile(xv);
    if (late) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = min(tid + j * 256, d / 4 - 1);
            if (!a.embd_q8) xv[j] = ((const float4 *)((const float *)a.tok_embd + (size_t)tok * d))[i];
            else {
                const blk_q8_0 *row = (const blk_q8_0 *)(a.tok_embd + (size_t)tok * (d / 32) * 34) + (i >> 3);
                const float dd = h2f(row->d);
                const int8_t *q = row->qs + 4 * (i & 7);
                xv[j] = make_float4((float)q[0] * dd, (float)q[1] * dd, (float)q[2] * dd, (float)q[3] * dd);
            }
        }
        if (blockIdx.x == 0 && wave == 0) {                 // the residual stream of layer 0, for the wo phase
            for (int i = lane; i < d; i += 64) {
                float v;
                if (!a.embd_q8) v = ((const float *)a.tok_embd)[(size_t)tok * d + i];
                else { const blk_q8_0 *row = (const blk_q8_0 *)(a.tok_embd + (size_t)tok * (d / 32) * 34) + (i >> 5); v = (float)row->qs[i & 31] * h2f(row->d); }
                stc(a.x + i, v);
            }
        }
    }
    fetch_qkv(a.layers[0]);

    for (int il = 0; il < a.n_layer; il++) {
        const mega_layer &L = a.layers[il];
        dbg_layer = il; dbg_n = 0;
        // ================= qkv: attn_norm, Q/K/V_project, rope, KV-cache copies =====================
        stage_norm(xv, L.attn_norm);
        stamp();
        {
            const float s0 = row_dot_d(wq0), s1 = row_dot_d(wq1), s2 = row_dot_d(wq2);
            if (!late) fetch_scores(L); else clear_tile(kb);
            if (lane == 0 && gw < d) {
                const int row = (2 * gw) % d, k = (row % hd) >> 1;
                const float c = s_rope[2 * k], sn = s_rope[2 * k + 1];
                // (x0, x1) -> (x0*c - x1*s, x0*s + x1*c) on adjacent rows (non-linear.cpp:359-363)
                const float v0 = s0 * c - s1 * sn, v1 = s0 * sn + s1 * c;
                s_out[wave * MEGA_SLOTS + 0] = __uint_as_float((uint32_t)f2h(v0) | ((uint32_t)f2h(v1) << 16));
                s_out[wave * MEGA_SLOTS + 1] = __uint_as_float((uint32_t)f2h(s2));
            }
        }
        if (!publish_and_sync([&]() {
                if (lane < MEGA_WAVES) {
                    const int j = (int)blockIdx.x * MEGA_WAVES + lane;
                    if (j < d) {
                        const uint32_t pr = __float_as_uint(s_out[lane * MEGA_SLOTS + 0]);
                        if (2 * j < d) stc((uint32_t *)a.q16 + j, pr);                                   // attn_score rounds Q to fp16 (mat.cpp:37)
                        else stc((uint32_t *)(L.kc + (size_t)pos * d) + (j - d / 2), pr);                // KCache_cpy: [token][head][hd]
                        stc(L.vc + (size_t)j * n_ctx + pos, (uint16_t)__float_as_uint(s_out[lane * MEGA_SLOTS + 1]));   // VCache_cpy: [d][C] column pos
                    }
                }
            })) return;

        // ================= scores: t = (K.q) * scale ================================================
        if (late) {
            for (int i = tid; i < d / 2; i += 256) ((uint32_t *)s_q16)[i] = ldc((const uint32_t *)a.q16 + i);
            fetch_scores(L);
        }
        __syncthreads();
        stamp();
        {
            const int nunit = n_kv * HG;
#pragma unroll
            for (int k = 0; k < MEGA_RS; k++) {
                const int u = gw + k * NW;
                const bool valid = u < nunit;
                const int uc = u % nunit, token = uc / HG, hg = uc - token * HG;
                uint4 kv = kb[k];
                if (token == pos) {                       // written in the phase before: read it coherently
                    const uint32_t *p = (const uint32_t *)(L.kc + (size_t)token * d + hg * 512 + lane * 8);
                    kv = make_uint4(ldc(p), ldc(p + 1), ldc(p + 2), ldc(p + 3));
                }
                const int head = hg * 4 + (lane >> 4);
                const uint4 qv = *(const uint4 *)(s_q16 + head * 128 + (lane & 15) * 8);
                const uint32_t kw[4] = {kv.x, kv.y, kv.z, kv.w}, qw[4] = {qv.x, qv.y, qv.z, qv.w};
                float s = 0.0f;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    s = fmaf(h2f((uint16_t)(kw[j] & 0xFFFFu)), h2f((uint16_t)(qw[j] & 0xFFFFu)), s);
                    s = fmaf(h2f((uint16_t)(kw[j] >> 16)), h2f((uint16_t)(qw[j] >> 16)), s);
                }
                s = group_sum<16>(s);
                if ((lane & 15) == 0 && valid) s_out[wave * MEGA_SLOTS + k * 4 + (lane >> 4)] = s * a.att_scale;
            }
            if (!late) fetch_v(L); else clear_tile(vb);
        }
        if (!publish_and_sync([&]() {
                const int nunit = n_kv * HG;
                for (int idx = lane; idx < MEGA_WAVES * MEGA_RS * 4; idx += 64) {
                    const int w = idx / (MEGA_RS * 4), r = idx - w * (MEGA_RS * 4), k = r >> 2, hq = r & 3;
                    const int u = ((int)blockIdx.x * MEGA_WAVES + w) + k * NW;
                    if (u < nunit) {
                        const int token = u / HG, hg = u - token * HG;
                        stc(a.scores + (size_t)(hg * 4 + hq) * n_ctx + token, s_out[w * MEGA_SLOTS + r]);
                    }
                }
            })) return;

        // ================= softmax + KQV ==============================================================
        // m = max t; e = expf(float(fp16(t - m))); p = e * (1/sum e) (non-linear.cpp:158-176); P is
        // rounded to fp16 for the KQV product (mat.cpp:37, vec_dot.h:117-146)
        {
            const int head = min((int)blockIdx.x * MEGA_WAVES, d - 1) / hd;
            const float *srow = a.scores + (size_t)head * n_ctx;
            const int n_pad = (n_kv + 7) & ~7;
            float mx = -INFINITY;
            if (late) {
                for (int j = tid; j < n_kv; j += 256) { const float t = ldc(srow + j); s_t[j] = t; mx = fmaxf(mx, t); }
                fetch_v(L);
                mx = wave_max(mx);
                if (lane == 0) s_red[wave] = mx;
            }
            __syncthreads();
            float sum = 0.0f;
            if (late) {
                mx = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
                for (int j = tid; j < n_kv; j += 256) { const float e = expf(h2f(f2h(s_t[j] - mx))); s_t[j] = e; sum += e; }
                sum = group_sum<64>(sum);
            }
            __syncthreads();
            if (late && lane == 0) s_red[wave] = sum;
            __syncthreads();
            if (late) {
                const float inv = 1.0f / ((s_red[0] + s_red[1]) + (s_red[2] + s_red[3]));
                for (int j = tid; j < n_pad; j += 256) s_p[j] = j < n_kv ? f2h(s_t[j] * inv) : (uint16_t)0;
            }
            __syncthreads();
            stamp();
            float acc = 0.0f;
#pragma unroll
            for (int i = 0; i < MEGA_RV; i++) {
                const int pc = i * 64 + lane;
                if (pc * 8 < n_kv) {
                    const uint4 pp = *(const uint4 *)(s_p + pc * 8);
                    const uint32_t vw[4] = {vb[i].x, vb[i].y, vb[i].z, vb[i].w}, pw[4] = {pp.x, pp.y, pp.z, pp.w};
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        // cache slots past n_kv hold whatever was there before: never multiply them in
                        if (pc * 8 + 2 * j < n_kv) acc = fmaf(h2f((uint16_t)(vw[j] & 0xFFFFu)), h2f((uint16_t)(pw[j] & 0xFFFFu)), acc);
                        if (pc * 8 + 2 * j + 1 < n_kv) acc = fmaf(h2f((uint16_t)(vw[j] >> 16)), h2f((uint16_t)(pw[j] >> 16)), acc);
                    }
                }
            }
            acc = group_sum<64>(acc);
            if (!late) fetch_wo(L); else clear_tile(wo0);
            if (lane == 0) s_out[wave * MEGA_SLOTS] = acc;
        }
        if (!publish_and_sync([&]() {
                const int r = (int)blockIdx.x * MEGA_WAVES + lane;
                if (lane < MEGA_WAVES && r < d) stc(a.attn_out + r, s_out[lane * MEGA_SLOTS]);
            })) return;

        // ================= wo: KQV_linear + ffn_input ================================================
        if (late) { load_x4(xv, a.attn_out); fetch_wo(L); } else clear_tile(xv);
        stage_plain(xv, d);
        stamp();
        {
            const float s = row_dot_d(wo0);
            if (!late) fetch_gateup(L, 0, 0, MEGA_DEPTH); else clear_tile(wg);
            if (lane == 0) s_out[wave * MEGA_SLOTS] = s;
        }
        if (!publish_and_sync([&]() {
                const int r = (int)blockIdx.x * MEGA_WAVES + lane;
                if (lane < MEGA_WAVES && r < d) stc(a.x1 + r, s_out[lane * MEGA_SLOTS] + ldc(a.x + r));
            })) return;

        // ================= gate|up: ffn_norm, ffn_up, ffn_gate, silu, ffn_par ========================
        if (late) { load_x4(xv, a.x1); fetch_gateup(L, 0, 0, MEGA_DEPTH); } else clear_tile(xv);
        stage_norm(xv, L.ffn_norm);
        stamp();
        const int ground = (F + NW - 1) / NW;                                  // row pairs per wave (<= MEGA_SLOTS)
        for (int k0 = 0; k0 < ground; k0 += RG) {
            if (k0 > 0) fetch_gateup(L, k0, 0, MEGA_DEPTH);                     // the first batch was requested before the barrier
#pragma unroll
            for (int k = 0; k < RG; k++) {
                fetch_gateup(L, k0, 2 * k + MEGA_DEPTH, 2 * k + 2 + MEGA_DEPTH);
                const float g = row_dot_d(wg[2 * k]), u = row_dot_d(wg[2 * k + 1]);
                if (lane == 0 && k0 + k < ground) s_out[wave * MEGA_SLOTS + k0 + k] = u * silu_lut(g);   // Mul(ffn_up, silu(ffn_gate)) (ffn.cpp:24-35)
            }
        }
        if (!late) fetch_down(L); else clear_tile(wd0);
        if (!publish_and_sync([&]() {
                for (int idx = lane; idx < MEGA_WAVES * ground; idx += 64) {
                    const int w = idx / ground, k = idx - w * ground;
                    const int i = ((int)blockIdx.x * MEGA_WAVES + w) + k * NW;
                    if (i < F) stc(a.hbuf + i, s_out[w * MEGA_SLOTS + k]);
                }
            })) return;

        // ================= down: ffn_down + logit_output =============================================
        {
            float4 hv[4 * NITF];
            if (late) {
#pragma unroll
                for (int j = 0; j < 4 * NITF; j++) hv[j] = ldc4(a.hbuf + 4 * min(tid + j * 256, F / 4 - 1));
                fetch_down(L);
            } else clear_tile(hv);
            stage_plain(hv, F);
        }
        stamp();
        {
            float acc[1] = {0.0f};
            dot_tile<WT, 64, NITF, 1>(wd0, &act, npf, lane, acc, nullptr);
            const float s = group_sum<64>(acc[0]);
            if (!late && il + 1 < a.n_layer) fetch_qkv(a.layers[il + 1]); else { clear_tile(wq0); clear_tile(wq1); clear_tile(wq2); }
            if (lane == 0) s_out[wave * MEGA_SLOTS] = s;
        }
        if (!publish_and_sync([&]() {
                const int r = (int)blockIdx.x * MEGA_WAVES + lane;
                if (lane < MEGA_WAVES && r < d) stc(a.x + r, s_out[lane * MEGA_SLOTS] + ldc(a.x1 + r));
            })) return;
        if (late) { load_x4(xv, a.x); if (il + 1 < a.n_layer) fetch_qkv(a.layers[il + 1]); } else clear_tile(xv);
    }

    // ================= result_norm, result_linear, output ===========================================
    stage_norm(xv, a.out_norm);
    for (int k0 = 0; k0 * NW < V; k0 += RH) {
        fetch_head(k0);
#pragma unroll
        for (int k = 0; k < RH; k++) {
            const float s = row_dot_d(wh[k]);
            const int r = gw + (k0 + k) * NW;
            if (lane == 0 && r < V) a.logits[r] = s;          // read by the next kernel (sampling): plain store
        }
    }
    __syncthreads();
    if (blockIdx.x == 0 && tid == 0) a.sync->epoch[0] = bar;  // every workgroup has passed barrier `bar`
}
