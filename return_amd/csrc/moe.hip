// Routed feed-forward (mixture of experts): the router's choice, the grouping of (token, choice) pairs by
// expert, the experts' products over those groups, and the weighted sum.
//
//   route     z [T][E] 32-bit router logits -> ids [T][top], weights [T][top]
//             s = sigmoid(z) (or softmax-free: only sigmoid is built); choice score c = s + bias (bias may be
//             null). Experts form n_groups equal groups of neighbours; a group's score is the sum of its two
//             largest choice scores (its largest, for groups of one); only the keep best groups stay eligible.
//             The top eligible experts by choice score are taken, largest first (ties: the lower number); the
//             weights are their s, divided by their sum + norm_eps. Law 2: s = softmax(z) over all experts, the
//             choice is made on s, a group's score is its largest s, the weights are the chosen s as they are.
//   plan      pairs p = t * top + k grouped by expert: order[] lists the pairs expert by expert, and tiles[]
//             lists (expert, first place in order[], places) for runs of at most `rows` places of one expert.
//             One workgroup (a counting sort). A pair's result does not depend on its place in a tile.
//   product   for every tile: y[p] = W_e x[row(p)] with row(p) = p / top (the token's row) or p itself;
//             gated: W_e = [gate rows; up rows], y = silu(gate) * up. An FMA form for every size and both
//             storage types, and two matrix-core forms for bfloat16 with K % 8 == 0: operands straight from
//             memory for tiles of 16 or 64 rows (few rows an expert: the weights are read once, the time is
//             the reading), tiles of 128 rows staged in LDS where an expert has many rows.
//   combine   out[t] = sum_k weights[t][k] * y[t * top + k], k in order, 32-bit sums; optionally one more term,
//             extra[t] * sigmoid(logit[t]) (an expert that every token uses, behind a gate of one number a token).
#include "common.h"

#define MOE_MAX_EXPERTS 1024

// What a gated product makes of its two halves: kind 0, silu(g) * u; kind 1 ("clamped"), with g <- min(g, limit)
// and u <- clamp(u, -limit, limit): g * sigmoid(slope * g) * (u + 1).
struct MoeAct {
    int kind;
    float limit, slope;
};
__device__ __forceinline__ float moe_gate(float g, float u, const MoeAct act) {
    if (act.kind == 1) {
        g = fminf(g, act.limit);
        u = fminf(fmaxf(u, -act.limit), act.limit);
        return g / (1.0f + expf(-act.slope * g)) * (u + 1.0f);
    }
    return g / (1.0f + expf(-g)) * u;
}

// ------------------------------------------------------------------ route: one wave per token
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ z, const float* __restrict__ bias,
                                                        int T, int E, int top, int n_groups, int keep, float norm_eps,
                                                        int* __restrict__ ids, float* __restrict__ weights, int law) {
    extern __shared__ float sm[];                          // per wave: s[E], c[E], group score [n_groups]
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + wave;
    if (t >= T) return;                                    // (no block-wide barrier below)
    float* s = sm + (size_t)wave * (2 * E + n_groups);
    float* c = s + E;
    float* gs = c + E;
    const int per = E / n_groups;
    // law 2: s = softmax(z) over all experts; the choice is made on s, a group scores its largest s, and the weights
    // are the chosen s as they are
    float z_top = -INFINITY, z_den = 1.f;
    if (law == 2) {
        for (int e = lane; e < E; e += 64) z_top = fmaxf(z_top, z[(size_t)t * E + e]);
        z_top = wave_max(z_top);
        float part = 0.f;
        for (int e = lane; e < E; e += 64) part += expf(z[(size_t)t * E + e] - z_top);
        z_den = wave_sum(part);
    }
    for (int e = lane; e < E; e += 64) {
        // law 1: the choice is made on the logits plus their bias, and the weights are the softmax over the chosen
        // ones alone (s holds the logit, turned into exp(logit - largest) as it is taken)
        const float zv = z[(size_t)t * E + e];
        const float v = law == 2 ? expf(zv - z_top) / z_den
                                 : law == 1 ? zv + (bias ? bias[e] : 0.f) : 1.0f / (1.0f + expf(-zv));
        s[e] = v;
        c[e] = law != 0 ? v : v + (bias ? bias[e] : 0.f);
    }
    __builtin_amdgcn_wave_barrier();
    if (n_groups > 1 && keep < n_groups) {
        for (int g = lane; g < n_groups; g += 64) {
            float a = -INFINITY, b = -INFINITY;            // the two largest of the group
            for (int e = g * per; e < (g + 1) * per; ++e) {
                const float v = c[e];
                if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
            }
            gs[g] = (per > 1 && law != 2) ? a + b : a;
        }
        __builtin_amdgcn_wave_barrier();
        // a group stays when fewer than `keep` groups beat it (a tie goes to the lower number)
        for (int g = lane; g < n_groups; g += 64) {
            int better = 0;
            for (int o = 0; o < n_groups; ++o) better += (gs[o] > gs[g]) || (gs[o] == gs[g] && o < g);
            if (better >= keep)
                for (int e = g * per; e < (g + 1) * per; ++e) c[e] = -INFINITY;
        }
        __builtin_amdgcn_wave_barrier();
    }
    float sum = 0.f, my_w = 0.f, largest = 0.f;
    int my_id = 0;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int at = 0x7fffffff;
        for (int e = lane; e < E; e += 64) {
            const float v = c[e];
            if (v > best) { best = v; at = e; }            // (rising e: the lower number wins a tie)
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oa = __shfl_xor(at, o, 64);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
        if (at >= E) at = 0;                               // (fewer eligible experts than top: refused on the host)
        if (k == 0) largest = s[at];
        const float w = law == 1 ? expf(s[at] - largest) : s[at];
        sum += w;
        if (lane == k) { my_id = at; my_w = w; }
        __builtin_amdgcn_wave_barrier();
        if (lane == 0) c[at] = -INFINITY;                  // taken
        __builtin_amdgcn_wave_barrier();
    }
    if (lane < top) {
        ids[(size_t)t * top + lane] = my_id;
        weights[(size_t)t * top + lane] = law == 2 ? my_w : my_w / (sum + norm_eps);
    }
}

extern "C" int ra_moe_route_law(const float* z, const float* bias, int T, int E, int top, int n_groups, int keep,
                                float norm_eps, int* ids, float* weights, int law, void* stream) {
    if (T <= 0) return RA_OK;
    if (law < 0 || law > 2 || (law == 1 && n_groups != 1)) return RA_ERR_ARG;
    if (E < 1 || E > MOE_MAX_EXPERTS || top < 1 || top > E || top > 64 || n_groups < 1 || E % n_groups || keep < 1 ||
        keep > n_groups || (long long)keep * (E / n_groups) < top)
        return RA_ERR_ARG;
    const size_t lds = (size_t)4 * (2 * E + n_groups) * sizeof(float);
    hipLaunchKernelGGL(moe_route_kernel, dim3((T + 3) / 4), dim3(256), lds, (hipStream_t)stream, z, bias, T, E, top,
                       n_groups, keep, norm_eps, ids, weights, law);
    return ra_launch_status();
}

extern "C" int ra_moe_route(const float* z, const float* bias, int T, int E, int top, int n_groups, int keep,
                            float norm_eps, int* ids, float* weights, void* stream) {
    return ra_moe_route_law(z, bias, T, E, top, n_groups, keep, norm_eps, ids, weights, 0, stream);
}

// ------------------------------------------------------------------ plan: one workgroup
// meta[0] = number of tiles. order [n_pairs], tiles [max_tiles][3].
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ ids, int n_pairs, int E, int rows,
                                                        int* __restrict__ order, int* __restrict__ tiles,
                                                        int* __restrict__ meta) {
    __shared__ int count[MOE_MAX_EXPERTS];
    __shared__ int first[MOE_MAX_EXPERTS + 1];
    __shared__ int tile_first[MOE_MAX_EXPERTS + 1];
    const int tid = threadIdx.x, n_thr = blockDim.x;
    for (int e = tid; e < E; e += n_thr) count[e] = 0;
    __syncthreads();
    for (int p = tid; p < n_pairs; p += n_thr) atomicAdd(&count[ids[p]], 1);
    __syncthreads();
    if (tid == 0) {
        int at = 0, tl = 0;
        for (int e = 0; e < E; ++e) {
            first[e] = at;
            tile_first[e] = tl;
            at += count[e];
            tl += (count[e] + rows - 1) / rows;
        }
        first[E] = at;
        tile_first[E] = tl;
        meta[0] = tl;
    }
    __syncthreads();
    // a pair's place among its expert's pairs is whatever the atomic gives: a row's result does not depend
    // on its place in a tile
    __shared__ int running[MOE_MAX_EXPERTS];
    for (int e = tid; e < E; e += n_thr) running[e] = 0;
    __syncthreads();
    for (int p = tid; p < n_pairs; p += n_thr) {
        const int e = ids[p];
        order[first[e] + atomicAdd(&running[e], 1)] = p;
    }
    for (int e = tid; e < E; e += n_thr) {
        const int n = count[e];
        for (int i = 0, tl = tile_first[e]; i < n; i += rows, ++tl) {
            tiles[3 * tl] = e;
            tiles[3 * tl + 1] = first[e] + i;
            tiles[3 * tl + 2] = min(rows, n - i);
        }
    }
}

extern "C" int ra_moe_plan(const int* ids, int n_pairs, int E, int rows, int* order, int* tiles, int* meta,
                           void* stream) {
    if (n_pairs <= 0) return RA_OK;
    if (E < 1 || E > MOE_MAX_EXPERTS || rows < 1) return RA_ERR_ARG;
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, ids, n_pairs, E, rows, order,
                       tiles, meta);
    return ra_launch_status();
}

// ------------------------------------------------------------------ product, FMA form
// Workgroup (tile, 64 result columns): 16 rows of one expert at most. Thread (c = tid % 64, rq = tid / 64)
// forms rows rq*4..rq*4+3 of column c; x through LDS in pieces of 32 of K.
#define MOE_FMA_ROWS 16
template <typename T, bool GATED>
__global__ __launch_bounds__(256) void moe_product_fma_kernel(
    const T* __restrict__ x, const T* __restrict__ w, T* __restrict__ y, const int* __restrict__ order,
    const int* __restrict__ tiles, const int* __restrict__ meta, int N, int K, int top_div, const MoeAct act) {
    if ((int)blockIdx.x >= meta[0]) return;
    __shared__ float xs[MOE_FMA_ROWS][33];
    __shared__ int pair_s[MOE_FMA_ROWS];
    const int e = tiles[3 * blockIdx.x], at = tiles[3 * blockIdx.x + 1], n = tiles[3 * blockIdx.x + 2];
    const int tid = threadIdx.x, c = tid & 63, rq = tid >> 6;
    if (tid < MOE_FMA_ROWS) pair_s[tid] = tid < n ? order[at + tid] : -1;
    __syncthreads();
    const int col = blockIdx.y * 64 + c;
    const size_t w_rows = GATED ? 2 * (size_t)N : (size_t)N;
    const T* wg = w + ((size_t)e * w_rows + min(col, N - 1)) * K;
    const T* wu = GATED ? wg + (size_t)N * K : wg;
    float ag[4] = {0.f, 0.f, 0.f, 0.f}, au[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += 32) {
        for (int i = tid; i < MOE_FMA_ROWS * 32; i += 256) {
            const int r = i >> 5, kk = i & 31;
            const int p = pair_s[r];
            xs[r][kk] = (p >= 0 && k0 + kk < K) ? to_f(x[(size_t)(p / top_div) * K + k0 + kk]) : 0.f;
        }
        __syncthreads();
        const int kn = min(32, K - k0);
        for (int kk = 0; kk < kn; ++kk) {
            const float g = to_f(wg[k0 + kk]);
            const float u = GATED ? to_f(wu[k0 + kk]) : 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float xv = xs[rq * 4 + i][kk];
                ag[i] = fmaf(xv, g, ag[i]);
                if (GATED) au[i] = fmaf(xv, u, au[i]);
            }
        }
        __syncthreads();
    }
    if (col >= N) return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int p = pair_s[rq * 4 + i];
        if (p < 0) continue;
        float v = ag[i];
        if (GATED) {
            // the two products are stored values of type T before the activation, as a product kernel and an
            // activation kernel apart would have them
            const float g = round_to<T>(ag[i]), u = round_to<T>(au[i]);
            v = moe_gate(g, u, act);
        }
        y[(size_t)p * N + col] = from_f<T>(v);
    }
}

// ------------------------------------------------------------------ product, matrix-core form (bfloat16)
// Workgroup of four waves per (tile of up to 16*RT rows of one expert, 64*CT result columns): wave w forms
// columns (4 blockIdx.y + w) * 16 CT ... by MFMA 16x16x32: A = 16 weight rows (one per lane n, 8 of K per
// lane group g), B = 16 rows of x, so lane (n, g) ends up with row n, columns 4g..4g+3 of each tile of 16.
// Operands come straight from memory (a weight row is read by one tile's waves only; x rows by the four
// waves, from L2).
typedef __bf16 moe_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float moe_float4_t __attribute__((ext_vector_type(4)));

template <bool GATED, int RT, int CT>
__global__ __launch_bounds__(256) void moe_product_mfma_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ w, bf16* __restrict__ y, const int* __restrict__ order,
    const int* __restrict__ tiles, const int* __restrict__ meta, int N, int K, int top_div, const MoeAct act) {
    if ((int)blockIdx.x >= meta[0]) return;
    const int e = tiles[3 * blockIdx.x], at = tiles[3 * blockIdx.x + 1], n_rows = tiles[3 * blockIdx.x + 2];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int col0 = (blockIdx.y * 4 + wave) * 16 * CT;
    if (col0 >= N) return;
    int pair[RT];
    const bf16* xr[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        pair[r] = (16 * r + n) < n_rows ? order[at + 16 * r + n] : -1;
        xr[r] = x + (size_t)(pair[r] >= 0 ? pair[r] / top_div : 0) * K;
    }
    const size_t w_rows = GATED ? 2 * (size_t)N : (size_t)N;
    const bf16* wr[CT];
#pragma unroll
    for (int c = 0; c < CT; ++c) wr[c] = w + ((size_t)e * w_rows + min(col0 + 16 * c + n, N - 1)) * K;
    moe_float4_t ag[RT][CT], au[RT][CT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            ag[r][c] = moe_float4_t{0.f, 0.f, 0.f, 0.f};
            au[r][c] = moe_float4_t{0.f, 0.f, 0.f, 0.f};
        }
    const moe_bf16x8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};
    // several k-steps of 32 at a time (eight with tiles of 16 rows, four with 64), all their loads asked for before
    // the first product: with one or two rows an expert the kernel only reads W, and a lane then has 128 (gated: 256)
    // bytes of it on their way instead of 16
    constexpr int KU = RT == 1 ? 8 : 4;
    for (int k0 = 0; k0 < K; k0 += 32 * KU) {
        moe_bf16x8_t b[KU][RT], a[KU][CT], a2[KU][CT];
#pragma unroll
        for (int u = 0; u < KU; ++u) {
            const int k = k0 + 32 * u + 8 * g;
            const bool in = k < K;                         // (K % 8 == 0: a group of 8 lies inside or outside)
#pragma unroll
            for (int c = 0; c < CT; ++c) {
                a[u][c] = in ? *reinterpret_cast<const moe_bf16x8_t*>(wr[c] + k) : z8;
                if (GATED) a2[u][c] = in ? *reinterpret_cast<const moe_bf16x8_t*>(wr[c] + (size_t)N * K + k) : z8;
            }
#pragma unroll
            for (int r = 0; r < RT; ++r)
                b[u][r] = (in && pair[r] >= 0) ? *reinterpret_cast<const moe_bf16x8_t*>(xr[r] + k) : z8;
        }
#pragma unroll
        for (int u = 0; u < KU; ++u)
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int c = 0; c < CT; ++c) {
                    ag[r][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][c], b[u][r], ag[r][c], 0, 0, 0);
                    if (GATED) au[r][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[u][c], b[u][r], au[r][c], 0, 0, 0);
                }
    }
    MFMA_SETTLE();
    // ag[r][c][i] = result[row n of group r][column col0 + 16c + 4g + i]
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        if (pair[r] < 0) continue;
        bf16* yr = y + (size_t)pair[r] * N;
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            const int col = col0 + 16 * c + 4 * g;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[i] = ag[r][c][i];
                if (GATED) {
                    const float gg = round_to<bf16>(ag[r][c][i]), uu = round_to<bf16>(au[r][c][i]);
                    v[i] = moe_gate(gg, uu, act);
                }
            }
            if (col + 3 < N && (N & 3) == 0) {
                uint2 pk;
                pk.x = (uint32_t)f2bf_bits(v[0]) | ((uint32_t)f2bf_bits(v[1]) << 16);
                pk.y = (uint32_t)f2bf_bits(v[2]) | ((uint32_t)f2bf_bits(v[3]) << 16);
                *reinterpret_cast<uint2*>(yr + col) = pk;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (col + i < N) yr[col + i] = from_f<bf16>(v[i]);
            }
        }
    }
}

// ------------------------------------------------------------------ product, matrix-core form with tiles in LDS
// For many rows per expert: a workgroup per (tile of up to 128 rows of one expert, 128 result columns, or 64
// gated ones with their gate and up rows), k-steps of 32, four waves as 2 x 2, each 64 x 64 as 4 x 4 MFMA tiles;
// both operands staged in LDS with padded rows, two buffers, the next k-step travelling through registers (the
// scheme of the tiled product for many rows, with the rows of x gathered by pair and W taken from the expert).
// Gated: of a wave's four tiles of W rows the first two are gate rows and the last two the up rows of the same
// columns, so a lane holds both halves of a result and forms silu(gate) * up itself.
#define MT_BM 128
#define MT_BK 32
#define MT_LD (MT_BK + 8)
typedef uint32_t moe_uint4_t __attribute__((ext_vector_type(4)));

template <bool GATED>
__global__ __launch_bounds__(256) void moe_product_tile_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ w, bf16* __restrict__ y, const int* __restrict__ order,
    const int* __restrict__ tiles, const int* __restrict__ meta, int N, int K, int top_div, const MoeAct act) {
    // (The tiles of columns of one tile of rows follow one another in the grid: they share the rows of x, which then
    // come from L2. With the tiles of rows first, every workgroup in flight read other rows and another expert's W:
    // 1.2 times slower at 8,192 pairs over 32 experts. Eight tiles of columns at a time through all tiles of rows, so
    // that an expert's W is shared too, was measured and is no faster.)
    if ((int)blockIdx.y >= meta[0]) return;
    __shared__ __attribute__((aligned(16))) uint16_t a_s[2][MT_BM * MT_LD];
    __shared__ __attribute__((aligned(16))) uint16_t w_s[2][128 * MT_LD];
    constexpr int CN = GATED ? 64 : 128;                       // result columns per workgroup
    const int e = tiles[3 * blockIdx.y], at = tiles[3 * blockIdx.y + 1], n_rows = tiles[3 * blockIdx.y + 2];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    const int n0 = blockIdx.x * CN;

    // staging: 128 rows x 4 pieces of 16 bytes per operand; a thread moves 2 pieces of each
    const int ld_row = tid >> 1, ld_p = (tid & 1) * 2;
    const int a_pair = order[at + min(ld_row, n_rows - 1)];
    const bf16* a_src = x + (size_t)(a_pair / top_div) * K + ld_p * 8;
    size_t w_row;
    if (GATED) {
        const int t4 = (ld_row >> 4) & 3;                      // which of the wave's four tiles of W rows
        const int col = n0 + (ld_row >> 6) * 32 + (t4 & 1) * 16 + (ld_row & 15);
        w_row = (size_t)e * 2 * N + (size_t)(t4 >> 1) * N + min(col, N - 1);
    } else {
        w_row = (size_t)e * N + min(n0 + ld_row, N - 1);
    }
    const bf16* w_src = w + w_row * K + ld_p * 8;
    const moe_uint4_t zero = {0u, 0u, 0u, 0u};
    moe_uint4_t ar[2], wr[2];
    moe_float4_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = moe_float4_t{0.f, 0.f, 0.f, 0.f};
#define MT_FETCH(k0_)                                                                        \
    _Pragma("unroll") for (int p = 0; p < 2; ++p) {                                          \
        const bool in_ = (k0_) + (ld_p + p) * 8 < K;                                         \
        ar[p] = in_ ? *reinterpret_cast<const moe_uint4_t*>(a_src + (k0_) + p * 8) : zero;   \
        wr[p] = in_ ? *reinterpret_cast<const moe_uint4_t*>(w_src + (k0_) + p * 8) : zero;   \
    }
#define MT_STAGE(buf_)                                                                       \
    _Pragma("unroll") for (int p = 0; p < 2; ++p) {                                          \
        *reinterpret_cast<moe_uint4_t*>(&a_s[buf_][ld_row * MT_LD + (ld_p + p) * 8]) = ar[p]; \
        *reinterpret_cast<moe_uint4_t*>(&w_s[buf_][ld_row * MT_LD + (ld_p + p) * 8]) = wr[p]; \
    }
    MT_FETCH(0)
    MT_STAGE(0)
    if (MT_BK < K) { MT_FETCH(MT_BK) }
    __syncthreads();
    const bool rows_here = wm * 64 < n_rows;                  // (a wave whose rows all lie beyond the tile's only moves data)
    int it = 0;
    for (int k0 = 0; k0 < K; k0 += MT_BK, ++it) {
        const int cur = it & 1;
        if (k0 + MT_BK < K) {
            MT_STAGE(cur ^ 1)
            if (k0 + 2 * MT_BK < K) { MT_FETCH(k0 + 2 * MT_BK) }
        }
        if (rows_here) {
            moe_bf16x8_t af[4], wf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                af[i] = *reinterpret_cast<const moe_bf16x8_t*>(&a_s[cur][(wm * 64 + i * 16 + n) * MT_LD + 8 * g]);
                wf[i] = *reinterpret_cast<const moe_bf16x8_t*>(&w_s[cur][(wn * 64 + i * 16 + n) * MT_LD + 8 * g]);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (wm * 64 + j * 16 >= n_rows) break;         // (the same in every lane: groups of rows beyond the tile's)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i], af[j], acc[i][j], 0, 0, 0);
            }
        }
        __syncthreads();
    }
#undef MT_FETCH
#undef MT_STAGE
    MFMA_SETTLE();
    // acc[i][j][e]: row wm*64 + j*16 + n of the tile, W row (wn*64 + i*16 + 4g + e) of the workgroup's 128
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int m = wm * 64 + j * 16 + n;
        if (m >= n_rows) continue;
        bf16* yr = y + (size_t)order[at + m] * N;
#pragma unroll
        for (int i = 0; i < (GATED ? 2 : 4); ++i) {
            const int col = GATED ? n0 + wn * 32 + i * 16 + 4 * g : n0 + wn * 64 + i * 16 + 4 * g;
            float v[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                v[c] = acc[i][j][c];
                if (GATED) {
                    const float gg = round_to<bf16>(acc[i][j][c]), uu = round_to<bf16>(acc[i + 2][j][c]);
                    v[c] = moe_gate(gg, uu, act);
                }
            }
            if (col + 3 < N && (N & 3) == 0) {
                uint2 pk;
                pk.x = (uint32_t)f2bf_bits(v[0]) | ((uint32_t)f2bf_bits(v[1]) << 16);
                pk.y = (uint32_t)f2bf_bits(v[2]) | ((uint32_t)f2bf_bits(v[3]) << 16);
                *reinterpret_cast<uint2*>(yr + col) = pk;
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    if (col + c < N) yr[col + c] = from_f<bf16>(v[c]);
            }
        }
    }
}

// rows of a tile that the product kernel behind these arguments takes (what ra_moe_plan is to be called with)
extern "C" int ra_moe_tile_rows(int n_pairs, int E, int K, int dtype) {
    if (dtype == RA_DTYPE_BF16 && K % 8 == 0) return n_pairs >= 64 * E ? 128 : (n_pairs >= 24 * E ? 64 : 16);
    return MOE_FMA_ROWS;
}

// x [rows][K]; w [E][N or 2N][K]; y [n_pairs][N]; the row of pair p in x is p / top_div (top_div = top: the
// token's row; 1: the pair's own row). max_tiles: the grid's first dimension, at least the number of tiles
// the plan can have (n_pairs / rows + E); workgroups beyond meta[0] leave at once.
// (act_kind, limit, slope: what a gated product makes of its halves, see MoeAct)
extern "C" int ra_moe_product_act(const void* x, const void* w, void* y, const int* order, const int* tiles,
                                  const int* meta, int max_tiles, int tile_rows, int N, int K, int top_div, int gated,
                                  int act_kind, float limit, float slope, int dtype, void* stream) {
    if (max_tiles <= 0) return RA_OK;
    if (N < 1 || K < 1 || top_div < 1 || act_kind < 0 || act_kind > 1) return RA_ERR_ARG;
    const MoeAct act = {act_kind, limit, slope};
    hipStream_t st = (hipStream_t)stream;
    if (dtype == RA_DTYPE_BF16 && K % 8 == 0 && tile_rows == MT_BM) {
        const int cn = gated ? 64 : 128;
        dim3 grid((N + cn - 1) / cn, max_tiles);
        if (grid.y > 65535) return RA_ERR_ARG;
        if (gated)
            hipLaunchKernelGGL(moe_product_tile_kernel<true>, grid, dim3(256), 0, st, (const bf16*)x, (const bf16*)w,
                               (bf16*)y, order, tiles, meta, N, K, top_div, act);
        else
            hipLaunchKernelGGL(moe_product_tile_kernel<false>, grid, dim3(256), 0, st, (const bf16*)x, (const bf16*)w,
                               (bf16*)y, order, tiles, meta, N, K, top_div, act);
        return ra_launch_status();
    }
    if (dtype == RA_DTYPE_BF16 && K % 8 == 0 && (tile_rows == 16 || tile_rows == 64)) {
        const bf16 *xb = (const bf16*)x, *wb = (const bf16*)w;
        bf16* yb = (bf16*)y;
#define MOE_GO(G_, RT_, CT_)                                                                                    \
    hipLaunchKernelGGL((moe_product_mfma_kernel<G_, RT_, CT_>), dim3(max_tiles, (N + 64 * CT_ - 1) / (64 * CT_)), \
                       dim3(256), 0, st, xb, wb, yb, order, tiles, meta, N, K, top_div, act)
        if (tile_rows == 64) { if (gated) MOE_GO(true, 4, 1); else MOE_GO(false, 4, 2); }
        else { if (gated) MOE_GO(true, 1, 1); else MOE_GO(false, 1, 1); }
#undef MOE_GO
        return ra_launch_status();
    }
    if (tile_rows != MOE_FMA_ROWS) return RA_ERR_ARG;
    dim3 grid(max_tiles, (N + 63) / 64), block(256);
#define MOE_FMA(T_, G_)                                                                                         \
    hipLaunchKernelGGL((moe_product_fma_kernel<T_, G_>), grid, block, 0, st, (const T_*)x, (const T_*)w, (T_*)y,  \
                       order, tiles, meta, N, K, top_div, act)
    if (dtype == RA_DTYPE_F32) { if (gated) MOE_FMA(float, true); else MOE_FMA(float, false); }
    else if (dtype == RA_DTYPE_BF16) { if (gated) MOE_FMA(bf16, true); else MOE_FMA(bf16, false); }
    else return RA_ERR_ARG;
#undef MOE_FMA
    return ra_launch_status();
}

extern "C" int ra_moe_product(const void* x, const void* w, void* y, const int* order, const int* tiles,
                              const int* meta, int max_tiles, int tile_rows, int N, int K, int top_div, int gated,
                              int dtype, void* stream) {
    return ra_moe_product_act(x, w, y, order, tiles, meta, max_tiles, tile_rows, N, K, top_div, gated, 0, 0.f, 0.f, dtype,
                              stream);
}

// ------------------------------------------------------------------ combine
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ y, const float* __restrict__ weights, T* __restrict__ out,
                                   int top, int N, long long total, const T* __restrict__ extra,
                                   const T* __restrict__ logit, long long ld_logit) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / N;
    const int c = (int)(i - t * N);
    float acc = 0.f;
    for (int k = 0; k < top; ++k) acc = fmaf(weights[t * top + k], to_f(y[((size_t)t * top + k) * N + c]), acc);
    // one more term that every token has: extra[t] times sigmoid(logit[t]), added last
    if (extra != nullptr) acc = fmaf(to_f(extra[i]), 1.0f / (1.0f + expf(-to_f(logit[t * ld_logit]))), acc);
    out[i] = from_f<T>(acc);
}

// extra [T, N] and logit (one number a token, rows ld_logit elements apart) may be null: no further term
extern "C" int ra_moe_combine_extra(const void* y, const float* weights, void* out, int T, int top, int N,
                                    const void* extra, const void* logit, long long ld_logit, int dtype, void* stream) {
    const long long total = (long long)T * N;
    if (total <= 0) return RA_OK;
    if ((extra == nullptr) != (logit == nullptr) || (extra != nullptr && ld_logit < 1)) return RA_ERR_ARG;
    dim3 block(256), grid((unsigned)((total + 255) / 256));
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(moe_combine_kernel<float>, grid, block, 0, (hipStream_t)stream, (const float*)y, weights,
                           (float*)out, top, N, total, (const float*)extra, (const float*)logit, ld_logit);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(moe_combine_kernel<bf16>, grid, block, 0, (hipStream_t)stream, (const bf16*)y, weights,
                           (bf16*)out, top, N, total, (const bf16*)extra, (const bf16*)logit, ld_logit);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}

extern "C" int ra_moe_combine(const void* y, const float* weights, void* out, int T, int top, int N, int dtype,
                              void* stream) {
    return ra_moe_combine_extra(y, weights, out, T, top, N, nullptr, nullptr, 0, dtype, stream);
}
