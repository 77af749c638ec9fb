// Gated delta rule with one decay per key channel, over the rows of a step.
//
// Per head, with S [D, V] in 32-bit carried from token to token for each request:
//     S <- diag(g_t) S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t
// (the read-out sees the token's own write). Around it, all in 32-bit:
//     q_t, k_t: unit vectors per head, x / sqrt(sum x^2 + 1e-6), q times D^-1/2
//     beta_t = sigmoid(b_t)
//     g_t[i] = exp(-exp(A_log[h]) * softplus(a_t[h,i] + dt_bias[h,i]))
//     out_t[j] = o_t[j] / sqrt(mean_j o_t[j]^2 + eps) * norm_w[j] * sigmoid(c_t[h,j])
// Inputs: qkv, the rows after the short convolution and its activation, [q heads | k heads | v heads]
// (G heads of D for q and k, H heads of V for v; head h reads q/k head h / (H/G)); b, one column per
// head of some wider rows; ag, rows [a: H*D | c: H*V], the decay's and the output gate's projections.
//
// The recurrence (in two forms, see below) and the output. The recurrence: a workgroup takes (head, VB columns of S, request) and walks the
// request's rows in chunks of up to DR_TC_MAX; for a chunk everything that does not depend on S (decays, unit
// vectors, beta) is prepared in LDS by all threads, then the recurrence runs over the chunk without a
// barrier and writes the read-outs o in 32-bit. A column j of S belongs to RS neighbouring lanes, each
// with DPT rows in registers; the two sums over rows are finished by data-parallel moves. Columns of
// one head are independent, so a head is spread over V / VB workgroups: the walk over the tokens is the
// long pole, and it is as long for 16 columns as for 128. The output kernel norms a head's read-out
// over all its columns, weighs and gates it: a wave per (row, head). Steps whose longest request has eight
// rows or more take the recurrence kernel with feeder waves (below); single tokens and short portions the plain
// one, which needs half the threads, few registers and little LDS, so that many workgroups share a CU.
//
// A second rule runs on the same kernels (rule 1, "outer"): the gated outer-product memory of a linear attention,
//     S <- diag(alpha_t) S + k_t v_t^T;   o_t = S^T q_t,    alpha_t[i] = sigmoid(a_t[h,i] + bias[h,i])^rate
// with q times D^-1/2 and k as they come (no unit vectors), no beta and no correction term (u = v), and the output
// gate silu(c) in place of sigmoid(c). The decay is formed as exp(-rate softplus(-(a + bias))).
//
// A third rule (rule 2, "scalar"): the memory of a state-space layer whose decay is one number per head and token,
//     delta_t = softplus(d_t[h] + bias[h]);   S <- exp(-exp(A_log[h]) delta_t) S + k_t (delta_t v_t)^T;   o_t = S^T q_t
// with q and k as they come, shared by the heads of a group as in the delta rule. delta and the decay are formed once
// per row by the exact routines (delta multiplies what is written, so its relative error counts where it is tiny);
// delta takes beta's place, the decay fills the row's decays. The read-out goes to a kernel of its own, which adds
// skip[h] v_t, gates and norms in equal parts of the row.
#include "common.h"

#define DR_TC_MAX 32      // rows of a chunk; fewer where a head's rows would not fit the LDS
#define DR_PAD 4

__device__ __forceinline__ float dr_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float dr_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }
// (single precision: beyond 30, log1p(e^x) and x are the same number)
__device__ __forceinline__ float dr_softplus_exact(float x) { return x > 30.f ? x : log1pf(expf(x)); }
// The decay exp(-A softplus(x)) by the hardware's exponential and logarithm (relative error about 1e-6; where
// e^x is tiny, log(1 + e^x) is off by at most one rounding of 1, 6e-8, and so is the decay): this runs once per
// token and key channel inside the walk over the tokens, where the exact routines' hundred instructions count.
__device__ __forceinline__ float dr_decay(float neg_a, float x) {
    const float sp = x > 20.f ? x : __logf(1.f + __expf(x));
    return __expf(neg_a * sp);
}

// Sum over the RS (1, 2, 4 or 8) neighbouring lanes that share a column, in every one of them, by
// data-parallel moves inside a row of 16 lanes: partner lane ^ 1, then lane ^ 2, then the other quad
// of the eight (mirrored: after the first two steps a quad's lanes all hold the quad's sum).
__device__ __forceinline__ float dr_group_sum(float v, int RS) {
    if (RS >= 2)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    if (RS >= 4)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    if (RS >= 8)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    return v;
}

// (one or two waves a SIMD: the walk is a chain of dependent steps, and registers for the next token's operands
// serve it better than more waves would)
template <typename T, int DPT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 2))) void delta_rule_kernel(
    const T* __restrict__ qkv, long long ld_qkv, const T* __restrict__ b, long long ld_b, const T* __restrict__ ag,
    long long ld_ag, const float* __restrict__ A_log, const float* __restrict__ dt_bias, float* __restrict__ S,
    const int* __restrict__ cu_q, const int* __restrict__ slot_ids, float* __restrict__ o_raw, int H, int G, int D, int V,
    int RS, int VB, int TC, int rule, float rate) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int tid = threadIdx.x, NT = blockDim.x, lane = tid & 63, wave = tid >> 6, n_waves = NT >> 6;
    const int col_blocks = (V + VB - 1) / VB;
    const int h = blockIdx.x / col_blocks, j0 = (blockIdx.x - h * col_blocks) * VB;
    const int s = blockIdx.y, kvh = h / (H / G);
    const int base = cu_q[s], q_len = cu_q[s + 1] - base;
    if (q_len <= 0) return;
    const int PS = DPT + DR_PAD;                    // a lane group's rows in LDS, padded against bank conflicts
    const int DP = RS * PS;
    float* k_s = smem;                              // [TC][DP]
    float* q_s = k_s + TC * DP;                     // [TC][DP]
    float* g_s = q_s + TC * DP;                     // [TC][DP]
    float* v_s = g_s + TC * DP;                     // [TC][VB]
    float* beta_s = v_s + TC * VB;                  // [TC]

    const int jl = tid / RS, rp = tid % RS, j = j0 + jl;
    const bool live = jl < VB && j < V;
    // the state is kept column by column, [slot][head][V][D]: a lane's rows of its column are one run of memory,
    // and the lanes of a wave read neighbouring runs
    float* Sc = S + (((size_t)slot_ids[s] * H + h) * V + (live ? j : 0)) * D;
    const bool vec = (D & 3) == 0;
    float st[DPT];
#pragma unroll
    for (int ii = 0; ii < DPT; ii += 4) {
        const int i = rp * DPT + ii;
        float4 v4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) {
            if (vec) {
                if (i < D) v4 = *reinterpret_cast<const float4*>(Sc + i);
            } else {
                if (i < D) v4.x = Sc[i];
                if (i + 1 < D) v4.y = Sc[i + 1];
                if (i + 2 < D) v4.z = Sc[i + 2];
                if (i + 3 < D) v4.w = Sc[i + 3];
            }
        }
        st[ii] = v4.x; st[ii + 1] = v4.y; st[ii + 2] = v4.z; st[ii + 3] = v4.w;
    }
    const float neg_a = rule == 1 ? -rate : -expf(A_log[h]);
    const float a_sign = rule == 1 ? -1.f : 1.f;
    const float q_scale = rule == 2 ? 1.f : 1.0f / sqrtf((float)D);
    const int Dfull = RS * DPT;

    for (int c0 = 0; c0 < q_len; c0 += TC) {
        const int nt = min(TC, q_len - c0);
        // ---- what the chunk's rows bring, into LDS
        // (rule 2: the row's step before its softplus, which the wave that takes the row turns into delta)
        if (tid < nt)
            beta_s[tid] = rule == 2 ? to_f(ag[(size_t)(base + c0 + tid) * ld_ag + h]) + dt_bias[h]
                          : rule ? 1.f : dr_sigmoid(to_f(b[(size_t)(base + c0 + tid) * ld_b + h]));
        for (int idx = tid; idx < nt * VB; idx += NT) {
            const int tt = idx / VB, jj = idx - tt * VB;
            v_s[idx] = j0 + jj < V ? to_f(qkv[(size_t)(base + c0 + tt) * ld_qkv + 2 * G * D + h * V + j0 + jj]) : 0.f;
        }
        // (four elements a thread at a time: their loads are on their way together)
        for (int idx0 = tid; idx0 < nt * Dfull; idx0 += 4 * NT) {
            float kk[4], qq[4], aa[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int idx = idx0 + x * NT;
                const int tt = idx / Dfull, i = idx - tt * Dfull;
                kk[x] = qq[x] = 0.f;
                aa[x] = 0.f;
                if (idx < nt * Dfull && i < D) {
                    const T* row = qkv + (size_t)(base + c0 + tt) * ld_qkv;
                    qq[x] = to_f(row[kvh * D + i]);
                    kk[x] = to_f(row[G * D + kvh * D + i]);
                    if (rule != 2)
                        aa[x] = a_sign * (to_f(ag[(size_t)(base + c0 + tt) * ld_ag + h * D + i]) + dt_bias[h * D + i]);
                }
            }
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int idx = idx0 + x * NT;
                if (idx >= nt * Dfull) break;
                const int tt = idx / Dfull, i = idx - tt * Dfull;
                const int at = tt * DP + (i / DPT) * PS + (i % DPT);
                k_s[at] = kk[x];
                q_s[at] = qq[x];
                g_s[at] = (i < D && rule != 2) ? dr_decay(neg_a, aa[x]) : 1.f;
            }
        }
        __syncthreads();
        for (int tt = wave; tt < nt; tt += n_waves) {          // unit vectors: a wave per row
            if (rule == 2) {
                // one step and one decay for the whole row
                const float delta = dr_softplus_exact(beta_s[tt]);
                const float dec = expf(neg_a * delta);
                __builtin_amdgcn_wave_barrier();
                if (lane == 0) beta_s[tt] = delta;
                for (int i = lane; i < D; i += 64) g_s[tt * DP + (i / DPT) * PS + (i % DPT)] = dec;
                continue;
            }
            float sk = 0.f, sq = 0.f;
            for (int i = lane; i < D; i += 64) {
                const int at = tt * DP + (i / DPT) * PS + (i % DPT);
                sk = fmaf(k_s[at], k_s[at], sk);
                sq = fmaf(q_s[at], q_s[at], sq);
            }
            sk = rule ? 1.f : 1.0f / sqrtf(wave_sum(sk) + 1e-6f);
            sq = rule ? q_scale : q_scale / sqrtf(wave_sum(sq) + 1e-6f);
            for (int i = lane; i < D; i += 64) {
                const int at = tt * DP + (i / DPT) * PS + (i % DPT);
                k_s[at] *= sk;
                q_s[at] *= sq;
            }
        }
        __syncthreads();
        // ---- the recurrence over the chunk
        // (a token's k, g and q are read from LDS while the token before it is worked on)
        float kreg[DPT], greg[DPT], qreg[DPT];
#pragma unroll
        for (int ii = 0; ii < DPT; ii += 4) {
            *reinterpret_cast<float4*>(kreg + ii) = *reinterpret_cast<const float4*>(k_s + rp * PS + ii);
            *reinterpret_cast<float4*>(greg + ii) = *reinterpret_cast<const float4*>(g_s + rp * PS + ii);
            *reinterpret_cast<float4*>(qreg + ii) = *reinterpret_cast<const float4*>(q_s + rp * PS + ii);
        }
        for (int tt = 0; tt < nt; ++tt) {
            const int nx = min(tt + 1, nt - 1);
            const float* kr = k_s + nx * DP + rp * PS;
            const float* qr = q_s + nx * DP + rp * PS;
            const float* gr = g_s + nx * DP + rp * PS;
            float kn[DPT], gn[DPT], qn[DPT];
#pragma unroll
            for (int ii = 0; ii < DPT; ii += 4) {
                *reinterpret_cast<float4*>(kn + ii) = *reinterpret_cast<const float4*>(kr + ii);
                *reinterpret_cast<float4*>(gn + ii) = *reinterpret_cast<const float4*>(gr + ii);
                *reinterpret_cast<float4*>(qn + ii) = *reinterpret_cast<const float4*>(qr + ii);
            }
            const float beta = beta_s[tt], vv = v_s[tt * VB + (live ? jl : 0)];
            float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;         // four chains, so that no sum waits for the one before
#pragma unroll
            for (int ii = 0; ii < DPT; ii += 4) {
                st[ii] *= greg[ii]; st[ii + 1] *= greg[ii + 1]; st[ii + 2] *= greg[ii + 2]; st[ii + 3] *= greg[ii + 3];
                a0 = fmaf(st[ii], kreg[ii], a0);
                a1 = fmaf(st[ii + 1], kreg[ii + 1], a1);
                a2 = fmaf(st[ii + 2], kreg[ii + 2], a2);
                a3 = fmaf(st[ii + 3], kreg[ii + 3], a3);
            }
            // (the outer-product rule has no correction term: what is written is the value itself)
            const float acc = rule ? 0.f : dr_group_sum((a0 + a1) + (a2 + a3), RS);
            const float u = beta * (vv - acc);
            float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
            for (int ii = 0; ii < DPT; ii += 4) {
                st[ii] = fmaf(kreg[ii], u, st[ii]);
                st[ii + 1] = fmaf(kreg[ii + 1], u, st[ii + 1]);
                st[ii + 2] = fmaf(kreg[ii + 2], u, st[ii + 2]);
                st[ii + 3] = fmaf(kreg[ii + 3], u, st[ii + 3]);
                o0 = fmaf(st[ii], qreg[ii], o0);
                o1 = fmaf(st[ii + 1], qreg[ii + 1], o1);
                o2 = fmaf(st[ii + 2], qreg[ii + 2], o2);
                o3 = fmaf(st[ii + 3], qreg[ii + 3], o3);
            }
            const float o = dr_group_sum((o0 + o1) + (o2 + o3), RS);
            if (live && rp == 0) o_raw[(size_t)(base + c0 + tt) * H * V + h * V + j] = o;
#pragma unroll
            for (int ii = 0; ii < DPT; ++ii) {
                kreg[ii] = kn[ii];
                greg[ii] = gn[ii];
                qreg[ii] = qn[ii];
            }
        }
        __syncthreads();                                       // before the next chunk overwrites LDS
    }
#pragma unroll
    for (int ii = 0; ii < DPT; ii += 4) {
        const int i = rp * DPT + ii;
        if (!live) continue;
        if (vec) {
            if (i < D) *reinterpret_cast<float4*>(Sc + i) = make_float4(st[ii], st[ii + 1], st[ii + 2], st[ii + 3]);
        } else {
            if (i < D) Sc[i] = st[ii];
            if (i + 1 < D) Sc[i + 1] = st[ii + 1];
            if (i + 2 < D) Sc[i + 2] = st[ii + 2];
            if (i + 3 < D) Sc[i + 3] = st[ii + 3];
        }
    }
}

// Sum over a wave's 64 lanes, in every lane, without LDS: inside each row of 16 lanes by data-parallel moves
// (lane ^ 1, lane ^ 2, the other quad of eight, the other half of the row), then over the four rows by lane swaps.
__device__ __forceinline__ float dr_wave_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    return rows_sum(v);
}

// Waves of two kinds. The first DR_WALKERS / 64 waves walk the tokens: column j of S belongs to RS neighbouring
// lanes, each with DPT rows in registers. The other DR_FEEDERS / 64 waves prepare the next chunk meanwhile, into
// the other of two LDS buffers: a feeder wave takes every other row of the chunk, asks for all its rows' q, k
// and decay projections at once, forms the unit vectors with sums over its own lanes (no trip through LDS) and the
// decays, and writes them where the walkers will read them. A workgroup is alone on its CU, and a chunk's loads
// would otherwise each cost the walk a trip to memory; this way the walk never waits for memory.
#define DR_WALKERS 128
#define DR_FEEDERS 128
#define DR_BATCH 32          // elements of q, k and decay projection that a feeder lane asks for at once
template <typename T, int DPT>
__global__ __launch_bounds__(DR_WALKERS + DR_FEEDERS) __attribute__((amdgpu_waves_per_eu(1, 2))) void delta_rule_fed_kernel(
    const T* __restrict__ qkv, long long ld_qkv, const T* __restrict__ b, long long ld_b, const T* __restrict__ ag,
    long long ld_ag, const float* __restrict__ A_log, const float* __restrict__ dt_bias, float* __restrict__ S,
    const int* __restrict__ cu_q, const int* __restrict__ slot_ids, float* __restrict__ o_raw, int H, int G, int D, int V,
    int RS, int VB, int TC, int rule, float rate) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int col_blocks = (V + VB - 1) / VB;
    const int h = blockIdx.x / col_blocks, j0 = (blockIdx.x - h * col_blocks) * VB;
    const int s = blockIdx.y, kvh = h / (H / G);
    const int base = cu_q[s], q_len = cu_q[s + 1] - base;
    if (q_len <= 0) return;
    const int PS = DPT + DR_PAD;                    // a lane group's rows in LDS, padded against bank conflicts
    const int DP = RS * PS;
    const int BUF = (TC * (3 * DP + VB) + TC + 3) & ~3;        // floats of one buffer: k, q, g [TC][DP], v [TC][VB], beta [TC]
    const int Dfull = RS * DPT;
    const bool feeder = tid >= DR_WALKERS;
    const float neg_a = rule == 1 ? -rate : -expf(A_log[h]);
    const float a_sign = rule == 1 ? -1.f : 1.f;
    const float q_scale = rule == 2 ? 1.f : 1.0f / sqrtf((float)D);

    // ---- a feeder's work for the chunk that starts at row c0, into buffer `to`
    auto feed = [&](int c0, int to) {
        float* k_s = smem + (size_t)to * BUF;
        float* q_s = k_s + TC * DP;
        float* g_s = q_s + TC * DP;
        float* v_s = g_s + TC * DP;
        float* beta_s = v_s + TC * VB;
        const int ft = tid - DR_WALKERS, fw = ft >> 6;
        const int nt = min(TC, q_len - c0);
        // the chunk's values and betas (every feeder thread has a share, whether or not its wave has rows)
        auto feed_values = [&]() {
            float bv = (ft < nt && !rule) ? to_f(b[(size_t)(base + c0 + ft) * ld_b + h]) : 0.f;
            if (ft < nt && rule == 2) bv = to_f(ag[(size_t)(base + c0 + ft) * ld_ag + h]) + dt_bias[h];
            for (int idx0 = ft; idx0 < nt * VB; idx0 += 4 * DR_FEEDERS) {
                float vv[4];
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const int idx = idx0 + x * DR_FEEDERS;
                    const int tt = idx / VB, jj = idx - tt * VB;
                    vv[x] = (idx < nt * VB && j0 + jj < V)
                                ? to_f(qkv[(size_t)(base + c0 + tt) * ld_qkv + 2 * G * D + h * V + j0 + jj]) : 0.f;
                }
#pragma unroll
                for (int x = 0; x < 4; ++x)
                    if (idx0 + x * DR_FEEDERS < nt * VB) v_s[idx0 + x * DR_FEEDERS] = vv[x];
            }
            if (ft < nt) beta_s[ft] = rule == 2 ? dr_softplus_exact(bv) : rule ? 1.f : dr_sigmoid(bv);
        };
        bool values_done = false;
        constexpr int EPL = (8 * DPT + 63) / 64;            // elements of a row per lane (RS <= 8)
        constexpr int ROWS = DR_BATCH / EPL;                // rows a wave asks for at once
        for (int t0 = fw; t0 < nt; t0 += (DR_FEEDERS / 64) * ROWS) {
            float fq[ROWS][EPL], fk[ROWS][EPL], fa[ROWS][EPL];
#pragma unroll
            for (int m = 0; m < ROWS; ++m) {
                const int tt = t0 + m * (DR_FEEDERS / 64);
#pragma unroll
                for (int e = 0; e < EPL; ++e) {
                    const int i = lane + 64 * e;
                    fq[m][e] = fk[m][e] = fa[m][e] = 0.f;
                    if (tt < nt && i < D) {
                        const T* row = qkv + (size_t)(base + c0 + tt) * ld_qkv;
                        fq[m][e] = to_f(row[kvh * D + i]);
                        fk[m][e] = to_f(row[G * D + kvh * D + i]);
                        fa[m][e] = rule == 2 ? to_f(ag[(size_t)(base + c0 + tt) * ld_ag + h]) + dt_bias[h]
                                   : a_sign * (to_f(ag[(size_t)(base + c0 + tt) * ld_ag + h * D + i]) + dt_bias[h * D + i]);
                    }
                }
            }
            if (!values_done) {
                feed_values();                               // behind the first batch's loads: all on their way together
                values_done = true;
            }
#pragma unroll
            for (int m = 0; m < ROWS; ++m) {
                const int tt = t0 + m * (DR_FEEDERS / 64);
                if (tt >= nt) break;
                float sk = 0.f, sq = 0.f;
#pragma unroll
                for (int e = 0; e < EPL; ++e) {
                    sk = fmaf(fk[m][e], fk[m][e], sk);
                    sq = fmaf(fq[m][e], fq[m][e], sq);
                }
                sk = rule ? 1.f : 1.0f / sqrtf(dr_wave_sum(sk) + 1e-6f);
                sq = rule ? q_scale : q_scale / sqrtf(dr_wave_sum(sq) + 1e-6f);
                // (rule 2: one decay for the whole row; lanes with an element of the row hold its step in fa[m][0])
                const float row_decay = (rule == 2 && lane < D) ? expf(neg_a * dr_softplus_exact(fa[m][0])) : 1.f;
#pragma unroll
                for (int e = 0; e < EPL; ++e) {
                    const int i = lane + 64 * e;
                    if (i < Dfull) {
                        const int at = tt * DP + (i / DPT) * PS + (i % DPT);
                        k_s[at] = fk[m][e] * sk;
                        q_s[at] = fq[m][e] * sq;
                        g_s[at] = i >= D ? 1.f : rule == 2 ? row_decay : dr_decay(neg_a, fa[m][e]);
                    }
                }
            }
        }
        if (!values_done) feed_values();
    };

    // ---- a walker's state: its rows of its column, kept column by column in memory
    const int jl = tid / RS, rp = tid % RS, j = j0 + jl;
    const bool live = !feeder && jl < VB && j < V;
    // the state is kept column by column, [slot][head][V][D]: a lane's rows of its column are one run of memory,
    // and the lanes of a wave read neighbouring runs
    float* Sc = S + (((size_t)slot_ids[s] * H + h) * V + (live ? j : 0)) * D;
    const bool vec = (D & 3) == 0;
    float st[DPT];
#pragma unroll
    for (int ii = 0; ii < DPT; ii += 4) {
        const int i = rp * DPT + ii;
        float4 v4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) {
            if (vec) {
                if (i < D) v4 = *reinterpret_cast<const float4*>(Sc + i);
            } else {
                if (i < D) v4.x = Sc[i];
                if (i + 1 < D) v4.y = Sc[i + 1];
                if (i + 2 < D) v4.z = Sc[i + 2];
                if (i + 3 < D) v4.w = Sc[i + 3];
            }
        }
        st[ii] = v4.x; st[ii + 1] = v4.y; st[ii + 2] = v4.z; st[ii + 3] = v4.w;
    }

    if (feeder) feed(0, 0);
    __syncthreads();
    int it = 0;
    for (int c0 = 0; c0 < q_len; c0 += TC, ++it) {
        const int nt = min(TC, q_len - c0);
        const int cur = it & 1;
        if (feeder) {
            if (c0 + TC < q_len) feed(c0 + TC, cur ^ 1);
        } else {
            const float* k_s = smem + (size_t)cur * BUF;
            const float* q_s = k_s + TC * DP;
            const float* g_s = q_s + TC * DP;
            const float* v_s = g_s + TC * DP;
            const float* beta_s = v_s + TC * VB;
            // ---- the recurrence over the chunk
            for (int tt = 0; tt < nt; ++tt) {
                const float* kr = k_s + tt * DP + rp * PS;
                const float* qr = q_s + tt * DP + rp * PS;
                const float* gr = g_s + tt * DP + rp * PS;
                float kreg[DPT];
                float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;     // four chains, so that no sum waits for the one before
#pragma unroll
                for (int ii = 0; ii < DPT; ii += 4) {
                    const float4 k4 = *reinterpret_cast<const float4*>(kr + ii);
                    const float4 g4 = *reinterpret_cast<const float4*>(gr + ii);
                    kreg[ii] = k4.x; kreg[ii + 1] = k4.y; kreg[ii + 2] = k4.z; kreg[ii + 3] = k4.w;
                    st[ii] *= g4.x; st[ii + 1] *= g4.y; st[ii + 2] *= g4.z; st[ii + 3] *= g4.w;
                    a0 = fmaf(st[ii], k4.x, a0);
                    a1 = fmaf(st[ii + 1], k4.y, a1);
                    a2 = fmaf(st[ii + 2], k4.z, a2);
                    a3 = fmaf(st[ii + 3], k4.w, a3);
                }
                const float acc = rule ? 0.f : dr_group_sum((a0 + a1) + (a2 + a3), RS);
                const float u = beta_s[tt] * (v_s[tt * VB + (live ? jl : 0)] - acc);
                float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
                for (int ii = 0; ii < DPT; ii += 4) {
                    const float4 q4 = *reinterpret_cast<const float4*>(qr + ii);
                    st[ii] = fmaf(kreg[ii], u, st[ii]);
                    st[ii + 1] = fmaf(kreg[ii + 1], u, st[ii + 1]);
                    st[ii + 2] = fmaf(kreg[ii + 2], u, st[ii + 2]);
                    st[ii + 3] = fmaf(kreg[ii + 3], u, st[ii + 3]);
                    o0 = fmaf(st[ii], q4.x, o0);
                    o1 = fmaf(st[ii + 1], q4.y, o1);
                    o2 = fmaf(st[ii + 2], q4.z, o2);
                    o3 = fmaf(st[ii + 3], q4.w, o3);
                }
                const float o = dr_group_sum((o0 + o1) + (o2 + o3), RS);
                if (live && rp == 0) o_raw[(size_t)(base + c0 + tt) * H * V + h * V + j] = o;
            }
        }
        __syncthreads();                                       // the next chunk is complete; this one may be overwritten
    }
#pragma unroll
    for (int ii = 0; ii < DPT; ii += 4) {
        const int i = rp * DPT + ii;
        if (!live) continue;
        if (vec) {
            if (i < D) *reinterpret_cast<float4*>(Sc + i) = make_float4(st[ii], st[ii + 1], st[ii + 2], st[ii + 3]);
        } else {
            if (i < D) Sc[i] = st[ii];
            if (i + 1 < D) Sc[i + 1] = st[ii + 1];
            if (i + 2 < D) Sc[i + 2] = st[ii + 2];
            if (i + 3 < D) Sc[i + 3] = st[ii + 3];
        }
    }
}

// out[t, h, :] = o[t, h, :] / sqrt(mean(o^2) + eps) * norm_w * sigmoid(c[t, h, :]): a wave per (row, head)
template <typename T>
__global__ __launch_bounds__(256) void delta_out_kernel(const float* __restrict__ o_raw, const T* __restrict__ gate,
                                                        long long ld_gate, const float* __restrict__ norm_w, float eps,
                                                        T* __restrict__ out, long long n_rows, int H, int V, int silu_gate) {
    const long long row = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int lane = threadIdx.x & 63;
    const long long t = row / H;
    const int h = (int)(row - t * H);
    const float* o = o_raw + (size_t)row * V;
    float ss = 0.f;
    for (int jj = lane; jj < V; jj += 64) ss = fmaf(o[jj], o[jj], ss);
    const float rstd = 1.0f / sqrtf(wave_sum(ss) / (float)V + eps);
    for (int jj = lane; jj < V; jj += 64) {
        const float c = to_f(gate[(size_t)t * ld_gate + (size_t)h * V + jj]);
        out[(size_t)row * V + jj] = from_f<T>(o[jj] * rstd * norm_w[jj] * (silu_gate ? c * dr_sigmoid(c) : dr_sigmoid(c)));
    }
}

// How a head's state is spread: RS lanes (a power of two) of DPT rows each to a column, VB columns a workgroup.
static bool delta_rule_plan(int D, int V, int* RS_out, int* DPT_out, int* VB_out) {
    if (D < 1 || V < 1 || D > 512 || V > 4096) return false;
    int RS = 8;
    while (RS > 1 && (D + RS - 1) / RS < 8) RS >>= 1;
    const int need = (D + RS - 1) / RS;
    int DPT = 4;
    while (DPT < need) DPT <<= 1;
    if (DPT > 64) return false;
    int VB = 128 / RS;                              // two waves a workgroup
    if (VB > V) VB = V;
    *RS_out = RS;
    *DPT_out = DPT;
    *VB_out = VB;
    return true;
}

static size_t delta_rule_lds(int DPT, int RS, int VB, int TC) {
    return sizeof(float) * ((size_t)TC * (3 * RS * (DPT + DR_PAD) + VB) + TC);
}
// rows of a chunk: as many as fit, a power of two from 4 to DR_TC_MAX (0: not even four)
static int delta_rule_chunk(int DPT, int RS, int VB) {
    for (int tc = DR_TC_MAX; tc >= 4; tc >>= 1)
        if (delta_rule_lds(DPT, RS, VB, tc) <= 150 * 1024) return tc;
    return 0;
}

// The same for the kernel with feeder waves: two buffers
static size_t delta_rule_fed_lds(int DPT, int RS, int VB, int TC) {
    return 2 * sizeof(float) * (((size_t)TC * (3 * RS * (DPT + DR_PAD) + VB) + TC + 3) & ~(size_t)3);
}
static int delta_rule_fed_chunk(int DPT, int RS, int VB) {
    for (int tc = DR_TC_MAX; tc >= 8; tc >>= 1)
        if (delta_rule_fed_lds(DPT, RS, VB, tc) <= 150 * 1024) return tc;
    return 0;
}

extern "C" int ra_delta_rule_fits(int D, int V) {
    int RS, DPT, VB;
    if (!delta_rule_plan(D, V, &RS, &DPT, &VB)) return 0;
    return delta_rule_chunk(DPT, RS, VB) > 0 ? 1 : 0;
}

template <typename T>
static int delta_rule_fed_launch(hipStream_t st, int DPT, dim3 grid, size_t lds, const void* qkv, long long ld_qkv,
                                 const void* b, long long ld_b, const void* ag, long long ld_ag, const float* A_log,
                                 const float* dt_bias, float* S, const int* cu_q, const int* slot_ids, float* o_raw, int H,
                                 int G, int D, int V, int RS, int VB, int TC, int rule, float rate) {
#define DR_FED(DPT_)                                                                                                  \
    do {                                                                                                              \
        if (lds > 64 * 1024 &&                                                                                        \
            hipFuncSetAttribute((const void*)delta_rule_fed_kernel<T, DPT_>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                (int)lds) != hipSuccess)                                                              \
            return RA_ERR_LAUNCH;                                                                                     \
        hipLaunchKernelGGL((delta_rule_fed_kernel<T, DPT_>), grid, dim3(DR_WALKERS + DR_FEEDERS), lds, st, (const T*)qkv, \
                           ld_qkv, (const T*)b, ld_b, (const T*)ag, ld_ag, A_log, dt_bias, S, cu_q, slot_ids, o_raw, H, G, \
                           D, V, RS, VB, TC, rule, rate);                                                                       \
    } while (0)
    switch (DPT) {
        case 4: DR_FED(4); break;
        case 8: DR_FED(8); break;
        case 16: DR_FED(16); break;
        case 32: DR_FED(32); break;
        case 64: DR_FED(64); break;
        default: return RA_ERR_ARG;
    }
#undef DR_FED
    return ra_launch_status();
}

template <typename T>
static int delta_rule_launch(hipStream_t st, int DPT, dim3 grid, dim3 block, size_t lds, const void* qkv, long long ld_qkv,
                             const void* b, long long ld_b, const void* ag, long long ld_ag, const float* A_log,
                             const float* dt_bias, float* S, const int* cu_q, const int* slot_ids, float* o_raw, int H, int G,
                             int D, int V, int RS, int VB, int TC, int rule, float rate) {
#define DR_GO(DPT_)                                                                                               \
    do {                                                                                                          \
        if (lds > 64 * 1024 &&                                                                                    \
            hipFuncSetAttribute((const void*)delta_rule_kernel<T, DPT_>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                (int)lds) != hipSuccess)                                                          \
            return RA_ERR_LAUNCH;                                                                                 \
        hipLaunchKernelGGL((delta_rule_kernel<T, DPT_>), grid, block, lds, st, (const T*)qkv, ld_qkv, (const T*)b, ld_b, \
                           (const T*)ag, ld_ag, A_log, dt_bias, S, cu_q, slot_ids, o_raw, H, G, D, V, RS, VB, TC, rule, rate); \
    } while (0)
    switch (DPT) {
        case 4: DR_GO(4); break;
        case 8: DR_GO(8); break;
        case 16: DR_GO(16); break;
        case 32: DR_GO(32); break;
        case 64: DR_GO(64); break;
        default: return RA_ERR_ARG;
    }
#undef DR_GO
    return ra_launch_status();
}

// qkv [T, 2 G D + H V] rows; b: rows whose first H columns are the heads' beta (before the sigmoid); ag [T, H D + H V];
// S fp32 [slots, H, V, D] (column by column); o_raw fp32 [T, H V] scratch; out [T, H V]; max_q_len: the longest request's rows.
// (ag: the decay's projection, H D columns of rows ld_ag apart; gate: the output gate's, H V columns of rows ld_gate
// apart; rule 0: the delta rule, 1: the outer-product rule with decay exponent `rate`, for which b and A_log are null)
static int delta_rule_run(const void* qkv, long long ld_qkv, const void* b, long long ld_b, const void* ag,
                          long long ld_ag, const void* gate, long long ld_gate, const float* A_log, const float* dt_bias,
                          const float* norm_w, float eps, float* S, const int* cu_q, const int* slot_ids, float* o_raw,
                          void* out, int n_seqs, int T_tokens, int max_q_len, int H, int G, int D, int V, int rule,
                          float rate, int dtype, void* stream) {
    if (n_seqs <= 0 || T_tokens <= 0) return RA_OK;
    int RS, DPT, VB;
    if (!delta_rule_plan(D, V, &RS, &DPT, &VB) || H < 1 || G < 1 || H % G || n_seqs > 65535) return RA_ERR_ARG;
    if (ld_qkv < (long long)2 * G * D + (long long)H * V || (rule == 0 && ld_b < H) ||
        ld_ag < (rule == 2 ? (long long)H : (long long)H * D) || ld_gate < (long long)H * V)
        return RA_ERR_ARG;
    if (dtype != RA_DTYPE_F32 && dtype != RA_DTYPE_BF16) return RA_ERR_ARG;
    int TC = delta_rule_chunk(DPT, RS, VB);
    if (TC <= 0 || max_q_len < 1) return RA_ERR_ARG;
    // no chunk longer than the step's longest request: a step of single tokens takes an eighth of the LDS, and
    // eight times the workgroups share a CU while each waits for its state
    while (TC > 4 && (TC >> 1) >= max_q_len) TC >>= 1;
    const size_t lds = delta_rule_lds(DPT, RS, VB, TC);
    const int col_blocks = (V + VB - 1) / VB;
    if ((long long)H * col_blocks > 0x7fffffffLL) return RA_ERR_ARG;
    dim3 grid(H * col_blocks, n_seqs), block(((VB * RS + 63) / 64) * 64);
    hipStream_t st = (hipStream_t)stream;
    int rc;
    // requests of eight rows and more: the kernel whose feeder waves prepare the next chunk while this one is walked
    // (while the workgroups are few: from about one and a half per CU on, the CUs' other workgroups fill the waits, and
    // the plain kernel's smaller footprint wins: measured, 32 heads of 128 x 128, four requests of 512 rows 1.48 against
    // 1.77 ms, one of 2,048 rows 2.75 against 1.76 ms)
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    const bool few = (long long)grid.x * grid.y <= (long long)cus * 3 / 2;
    const int TCF = (max_q_len >= 8 && few) ? delta_rule_fed_chunk(DPT, RS, VB) : 0;
    if (TCF > 0 && VB * RS <= DR_WALKERS) {
        int tcf = TCF;
        while (tcf > 8 && (tcf >> 1) >= max_q_len) tcf >>= 1;
        const size_t flds = delta_rule_fed_lds(DPT, RS, VB, tcf);
        if (dtype == RA_DTYPE_F32)
            rc = delta_rule_fed_launch<float>(st, DPT, grid, flds, qkv, ld_qkv, b, ld_b, ag, ld_ag, A_log, dt_bias, S, cu_q,
                                              slot_ids, o_raw, H, G, D, V, RS, VB, tcf, rule, rate);
        else
            rc = delta_rule_fed_launch<bf16>(st, DPT, grid, flds, qkv, ld_qkv, b, ld_b, ag, ld_ag, A_log, dt_bias, S, cu_q,
                                             slot_ids, o_raw, H, G, D, V, RS, VB, tcf, rule, rate);
    } else if (dtype == RA_DTYPE_F32)
        rc = delta_rule_launch<float>(st, DPT, grid, block, lds, qkv, ld_qkv, b, ld_b, ag, ld_ag, A_log, dt_bias, S, cu_q,
                                      slot_ids, o_raw, H, G, D, V, RS, VB, TC, rule, rate);
    else
        rc = delta_rule_launch<bf16>(st, DPT, grid, block, lds, qkv, ld_qkv, b, ld_b, ag, ld_ag, A_log, dt_bias, S, cu_q,
                                     slot_ids, o_raw, H, G, D, V, RS, VB, TC, rule, rate);
    if (rc != RA_OK) return rc;
    if (rule == 2) return RA_OK;                      // (the caller's own kernel takes the read-outs)
    const long long n_rows = (long long)T_tokens * H;
    dim3 ogrid((unsigned)((n_rows + 3) / 4)), oblock(256);
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(delta_out_kernel<float>, ogrid, oblock, 0, st, o_raw, (const float*)gate, ld_gate, norm_w,
                           eps, (float*)out, n_rows, H, V, rule);
    else
        hipLaunchKernelGGL(delta_out_kernel<bf16>, ogrid, oblock, 0, st, o_raw, (const bf16*)gate, ld_gate, norm_w,
                           eps, (bf16*)out, n_rows, H, V, rule);
    return ra_launch_status();
}

extern "C" int ra_delta_rule(const void* qkv, long long ld_qkv, const void* b, long long ld_b, const void* ag,
                             long long ld_ag, const float* A_log, const float* dt_bias, const float* norm_w, float eps,
                             float* S, const int* cu_q, const int* slot_ids, float* o_raw, void* out, int n_seqs,
                             int T_tokens, int max_q_len, int H, int G, int D, int V, int dtype, void* stream) {
    if (ld_ag < (long long)H * D + (long long)H * V) return RA_ERR_ARG;
    const size_t el = dtype == RA_DTYPE_F32 ? 4 : 2;
    const void* gate = (const char*)ag + (size_t)H * D * el;
    return delta_rule_run(qkv, ld_qkv, b, ld_b, ag, ld_ag, gate, ld_ag, A_log, dt_bias, norm_w, eps, S, cu_q, slot_ids,
                          o_raw, out, n_seqs, T_tokens, max_q_len, H, G, D, V, 0, 0.f, dtype, stream);
}

// The outer-product rule: qkv rows [q: H D | k: H D | v: H V]; a [T, H D] the decay's logits before their bias;
// gate [T, H V]; decay = sigmoid(a + bias)^rate; out = rmsnorm_V(o) norm_w silu(gate).
extern "C" int ra_outer_rule(const void* qkv, long long ld_qkv, const void* a, long long ld_a, const void* gate,
                             long long ld_gate, const float* bias, float rate, const float* norm_w, float eps, float* S,
                             const int* cu_q, const int* slot_ids, float* o_raw, void* out, int n_seqs, int T_tokens,
                             int max_q_len, int H, int D, int V, int dtype, void* stream) {
    if (!(rate > 0.f) || bias == nullptr) return RA_ERR_ARG;
    return delta_rule_run(qkv, ld_qkv, nullptr, 0, a, ld_a, gate, ld_gate, nullptr, bias, norm_w, eps, S, cu_q, slot_ids,
                          o_raw, out, n_seqs, T_tokens, max_q_len, H, H, D, V, 1, rate, dtype, stream);
}

// out[t, part] = y / sqrt(mean over the part of y^2 + eps) * norm_w with y = (o[t, c] + skip[head of c] v[t, c]) * silu(z[t, c]),
// the row of H V channels cut into n_parts equal parts: a wave per (row, part). A part's elements stay in registers
// between the sum and the result (up to 16 a lane; longer parts are formed again).
#define SO_KEEP 16
template <typename T>
__global__ __launch_bounds__(256) void scalar_out_kernel(const float* __restrict__ o_raw, const T* __restrict__ v,
                                                         long long ld_v, const T* __restrict__ gate, long long ld_gate,
                                                         const float* __restrict__ skip, const float* __restrict__ norm_w,
                                                         float eps, T* __restrict__ out, long long n_units, int n_parts,
                                                         int L, int V) {
    const long long unit = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (unit >= n_units) return;
    const int lane = threadIdx.x & 63;
    const long long t = unit / n_parts;
    const int c0 = (int)(unit - t * n_parts) * L;
    const size_t inner = (size_t)n_parts * L;
    auto value = [&](int c) {
        const float z = to_f(gate[(size_t)t * ld_gate + c]);
        const float y = fmaf(skip[c / V], to_f(v[(size_t)t * ld_v + c]), o_raw[(size_t)t * inner + c]);
        return y * (z / (1.0f + expf(-z)));
    };
    float ss = 0.f;
    if (L <= 64 * SO_KEEP) {
        float y[SO_KEEP];
#pragma unroll
        for (int i = 0; i < SO_KEEP; ++i) {
            const int e = lane + 64 * i;
            y[i] = e < L ? value(c0 + e) : 0.f;
            ss = fmaf(y[i], y[i], ss);
        }
        const float rstd = 1.0f / sqrtf(wave_sum(ss) / (float)L + eps);
#pragma unroll
        for (int i = 0; i < SO_KEEP; ++i) {
            const int e = lane + 64 * i;
            if (e < L) out[(size_t)t * inner + c0 + e] = from_f<T>(y[i] * rstd * norm_w[c0 + e]);
        }
        return;
    }
    for (int e = lane; e < L; e += 64) {
        const float y = value(c0 + e);
        ss = fmaf(y, y, ss);
    }
    const float rstd = 1.0f / sqrtf(wave_sum(ss) / (float)L + eps);
    for (int e = lane; e < L; e += 64) out[(size_t)t * inner + c0 + e] = from_f<T>(value(c0 + e) * rstd * norm_w[c0 + e]);
}

// The scalar rule: qkv rows [q: G D | k: G D | v: H V]; d [T, H] the step before its bias and softplus; gate [T, H V];
// S fp32 [slots, H, V, D]; out = groupnorm_{n_parts}((o + skip v) silu(gate)) norm_w, norm_w [H V], skip [H].
extern "C" int ra_scalar_rule(const void* qkv, long long ld_qkv, const void* d, long long ld_d, const void* gate,
                              long long ld_gate, const float* A_log, const float* d_bias, const float* skip,
                              const float* norm_w, int n_parts, float eps, float* S, const int* cu_q, const int* slot_ids,
                              float* o_raw, void* out, int n_seqs, int T_tokens, int max_q_len, int H, int G, int D, int V,
                              int dtype, void* stream) {
    if (n_seqs <= 0 || T_tokens <= 0) return RA_OK;
    if (A_log == nullptr || d_bias == nullptr || skip == nullptr || norm_w == nullptr || n_parts < 1 ||
        ((long long)H * V) % n_parts)
        return RA_ERR_ARG;
    const int rc = delta_rule_run(qkv, ld_qkv, nullptr, 0, d, ld_d, gate, ld_gate, A_log, d_bias, norm_w, eps, S, cu_q,
                                  slot_ids, o_raw, out, n_seqs, T_tokens, max_q_len, H, G, D, V, 2, 0.f, dtype, stream);
    if (rc != RA_OK) return rc;
    const int L = (int)((long long)H * V / n_parts);
    const long long n_units = (long long)T_tokens * n_parts;
    const size_t el = dtype == RA_DTYPE_F32 ? 4 : 2;
    const void* v = (const char*)qkv + (size_t)2 * G * D * el;
    dim3 ogrid((unsigned)((n_units + 3) / 4)), oblock(256);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(scalar_out_kernel<float>, ogrid, oblock, 0, st, o_raw, (const float*)v, ld_qkv, (const float*)gate,
                           ld_gate, skip, norm_w, eps, (float*)out, n_units, n_parts, L, V);
    else
        hipLaunchKernelGGL(scalar_out_kernel<bf16>, ogrid, oblock, 0, st, o_raw, (const bf16*)v, ld_qkv, (const bf16*)gate,
                           ld_gate, skip, norm_w, eps, (bf16*)out, n_units, n_parts, L, V);
    return ra_launch_status();
}
