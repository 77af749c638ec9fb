// Attention over a latent row per token: what is prepared for it, and the plain (32-bit FMA) kernel.
//
// The cache holds, for every token, c [C] (a normed latent, in the value pool) and kr [R] (a rotated key part
// shared by all heads, in the key pool); both pools have one "kv head". Every query head h brings a query of
// C + R elements, qq = [W_uk,h^T q_flat | rot(q_rot)], and its score with the key at position j is
//     s_j = (qq[:C] . c_j + qq[C:] . kr_j) * scale,   j <= the query's position,
// the weights are exp(s_j - m) / (sum_j exp(s_j - m) + exp(sink_h - m)) (the sink is one more term of the
// denominator that has no value; sink null: none), and the output is sum_j p_j c_j, a row of C elements that
// the caller multiplies by W_uv,h. Scores, weights and sums are 32-bit. With a window w > 0 the query at position i
// reads the keys j with 0 <= i - j < w only. R may be 0: then there is no rotated part, the key pool's rows are empty
// and nothing of it is read or written.
//
//   latent_kv_prepare   per token, from the rows z = [a: Q | b: C | r: R | ...] of the first product:
//                       cq = a / sqrt(mean(a^2) + eps) * wq  (the query's latent, to cq_out),
//                       c = b / sqrt(mean(b^2) + eps) * wc   (to the value pool's row of the token's slot),
//                       kr = r with its first `rot` elements turned by the token's position, element i with
//                       i + rot/2 (to the key pool's row).
//   latent_q_prepare    qq[t][h] = [q_lat[h][t] | turned q[t][h][D:]]  (q rows are heads of [D | R]).
//   attention_latent_plain   a workgroup per (token, QR heads): the heads of a token read the same rows, so a
//                       row that is loaded serves QR scores. The waves take the blocks of 64 keys in turn (block b,
//                       counted from position 0, is wave b % WAVES's), so a row's sums are formed in an order that
//                       depends on nothing but its position; the waves are merged through LDS in wave order.
//                       Four lanes share a key for the scores; for the sums over c the lanes run along its elements.
// Tables as in the other attention kernels: page_table[cu_pages[s] + i] is the i-th listed page of request s,
// whose first row holds position kv_start[s]; the new tokens of s are rows cu_q[s] .. cu_q[s+1]-1 and sit at
// positions q_start[s], q_start[s] + 1, ...
#include "common.h"

// ------------------------------------------------------------------ preparation
template <typename T>
__global__ __launch_bounds__(256) void latent_kv_prepare_kernel(
    const T* __restrict__ z, long long ld_z, int Q, int C, int R, const float* __restrict__ wq,
    const float* __restrict__ wc, float eps, const int* __restrict__ positions, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int rot, T* __restrict__ cq_out, T* __restrict__ k_pool, T* __restrict__ v_pool,
    const int* __restrict__ slot_mapping, int P) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const T* zr = z + (size_t)t * ld_z;
    float ss = 0.f;
    for (int i = tid; i < Q; i += 256) {
        const float a = to_f(zr[i]);
        ss = fmaf(a, a, ss);
    }
    const float rq = 1.0f / sqrtf(block_sum(ss, scratch) / (float)Q + eps);
    for (int i = tid; i < Q; i += 256) cq_out[(size_t)t * Q + i] = from_f<T>(to_f(zr[i]) * rq * wq[i]);
    if (v_pool == nullptr) return;
    ss = 0.f;
    for (int i = tid; i < C; i += 256) {
        const float a = to_f(zr[Q + i]);
        ss = fmaf(a, a, ss);
    }
    const float rc = 1.0f / sqrtf(block_sum(ss, scratch) / (float)C + eps);
    const int slot = slot_mapping[t];
    if (slot < 0) return;
    T* vr = v_pool + ra_cache_offset(slot, 0, 1, P, C);
    for (int i = tid; i < C; i += 256) vr[i] = from_f<T>(to_f(zr[Q + i]) * rc * wc[i]);
    T* kr = k_pool + ra_cache_offset(slot, 0, 1, P, R);
    const int half = rot >> 1, pos = positions[t];
    for (int i = tid; i < R; i += 256) {
        float v = to_f(zr[Q + C + i]);
        if (i < rot) {
            const int f = i < half ? i : i - half;
            const float cs = cos_t[(size_t)pos * half + f], sn = sin_t[(size_t)pos * half + f];
            const float other = to_f(zr[Q + C + (i < half ? i + half : i - half)]);
            v = i < half ? v * cs - other * sn : v * cs + other * sn;
        }
        kr[i] = from_f<T>(v);
    }
}

extern "C" int ra_latent_kv_prepare(const void* z, long long ld_z, int T_tokens, int Q, int C, int R, const float* wq,
                                    const float* wc, float eps, const int* positions, const float* cos_t,
                                    const float* sin_t, int rot, void* cq_out, void* k_pool, void* v_pool,
                                    const int* slot_mapping, int P, int dtype, void* stream) {
    if (T_tokens <= 0) return RA_OK;
    if (Q < 1 || C < 1 || R < 0 || rot < 0 || rot > R || (rot & 1) || ld_z < (long long)Q + C + R || P < 1 ||
        (rot > 0 && (cos_t == nullptr || sin_t == nullptr)) || (v_pool != nullptr && slot_mapping == nullptr) ||
        (v_pool != nullptr && R > 0 && k_pool == nullptr))
        return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(latent_kv_prepare_kernel<float>, dim3(T_tokens), dim3(256), 0, st, (const float*)z, ld_z, Q, C, R,
                           wq, wc, eps, positions, cos_t, sin_t, rot, (float*)cq_out, (float*)k_pool, (float*)v_pool,
                           slot_mapping, P);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(latent_kv_prepare_kernel<bf16>, dim3(T_tokens), dim3(256), 0, st, (const bf16*)z, ld_z, Q, C, R,
                           wq, wc, eps, positions, cos_t, sin_t, rot, (bf16*)cq_out, (bf16*)k_pool, (bf16*)v_pool,
                           slot_mapping, P);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}

template <typename T>
__global__ __launch_bounds__(256) void latent_q_prepare_kernel(
    const T* __restrict__ q, const T* __restrict__ q_lat, int T_tokens, int Hn, int D, int R, int C,
    const int* __restrict__ positions, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot,
    T* __restrict__ qq) {
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    T* dst = qq + ((size_t)t * Hn + h) * (C + R);
    const T* lat = q_lat + ((size_t)h * T_tokens + t) * C;
    for (int i = tid; i < C; i += 256) dst[i] = lat[i];
    const T* qr = q + ((size_t)t * Hn + h) * (D + R) + D;
    const int half = rot >> 1, pos = positions[t];
    for (int i = tid; i < R; i += 256) {
        float v = to_f(qr[i]);
        if (i < rot) {
            const int f = i < half ? i : i - half;
            const float cs = cos_t[(size_t)pos * half + f], sn = sin_t[(size_t)pos * half + f];
            const float other = to_f(qr[i < half ? i + half : i - half]);
            v = i < half ? v * cs - other * sn : v * cs + other * sn;
        }
        dst[C + i] = from_f<T>(v);
    }
}

extern "C" int ra_latent_q_prepare(const void* q, const void* q_lat, int T_tokens, int Hn, int D, int R, int C,
                                   const int* positions, const float* cos_t, const float* sin_t, int rot, void* qq,
                                   int dtype, void* stream) {
    if (T_tokens <= 0) return RA_OK;
    if (Hn < 1 || Hn > 65535 || D < 0 || R < 0 || C < 1 || rot < 0 || rot > R || (rot & 1) ||
        (rot > 0 && (cos_t == nullptr || sin_t == nullptr)))
        return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(T_tokens, Hn);
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(latent_q_prepare_kernel<float>, grid, dim3(256), 0, st, (const float*)q, (const float*)q_lat,
                           T_tokens, Hn, D, R, C, positions, cos_t, sin_t, rot, (float*)qq);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(latent_q_prepare_kernel<bf16>, grid, dim3(256), 0, st, (const bf16*)q, (const bf16*)q_lat,
                           T_tokens, Hn, D, R, C, positions, cos_t, sin_t, rot, (bf16*)qq);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}

// ------------------------------------------------------------------ the plain kernel
#define LAT_MAX_ACC 8       // C <= 64 * 8
#define LAT_BLOCK 64

__device__ __forceinline__ void lat_load4(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void lat_load4(const bf16* p, float (&v)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}

template <typename T, int QR, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void attn_latent_plain_kernel(
    const T* __restrict__ qq, T* __restrict__ out, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int* __restrict__ page_table, const int* __restrict__ cu_pages, const int* __restrict__ kv_start,
    const int* __restrict__ cu_q, const int* __restrict__ q_start, const int* __restrict__ tok_ids, int n_seqs,
    int T_rows, int T_tokens, int Hn, int C, int R, int P, float scale, const float* __restrict__ sink, int window) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int Dk = C + R;
    float* q_s = smem;                                   // [QR][Dk]
    float* p_s = q_s + QR * Dk;                          // [WAVES][QR][64]
    int* row_s = (int*)(p_s + WAVES * QR * 64);          // [WAVES][64]
    float* ml_s = (float*)(row_s + WAVES * 64);          // [WAVES][QR][2]
    float* acc_s = ml_s + WAVES * QR * 2;                // [WAVES][QR][C]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, part = lane & 3, sub = lane >> 2;
    const int t = tok_ids ? tok_ids[blockIdx.x] : (int)blockIdx.x;
    const int h0 = blockIdx.y * QR;
    int s = 0;
    {
        int lo = 0, hi = n_seqs - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
        }
        s = lo;
    }
    const int pos = q_start[s] + (t - cu_q[s]);
    const int start = kv_start[s];
    const int first_key = window > 0 ? max(start, pos - window + 1) : start;      // the earliest key this row reads
    const int* pt = page_table + cu_pages[s];
    const int n_listed = cu_pages[s + 1] - cu_pages[s];
    const bool vec = ((C | R) & 3) == 0;

    for (int idx = tid; idx < QR * Dk; idx += WAVES * 64) {
        const int r = idx / Dk, e = idx - r * Dk;
        q_s[idx] = h0 + r < Hn ? to_f(qq[((size_t)t * Hn + h0 + r) * Dk + e]) : 0.f;
    }
    __syncthreads();

    float m[QR], l[QR], acc[QR][LAT_MAX_ACC];
#pragma unroll
    for (int r = 0; r < QR; ++r) {
        m[r] = -INFINITY;
        l[r] = 0.f;
#pragma unroll
        for (int i = 0; i < LAT_MAX_ACC; ++i) acc[r][i] = 0.f;
    }
    float* my_p = p_s + wave * QR * 64;
    int* my_row = row_s + wave * 64;

    const int b_first = first_key / LAT_BLOCK;
    int b = b_first + ((wave - b_first) % WAVES + WAVES) % WAVES;          // first block >= b_first of this wave
    for (; b * LAT_BLOCK <= pos; b += WAVES) {
        const int base = b * LAT_BLOCK;
        // ---- scores: 16 keys at once, four lanes to a key
        float sc[4][QR];
#pragma unroll
        for (int sp = 0; sp < 4; ++sp) {
            const int kk = 16 * sp + sub;
            const int p = base + kk;
            const int idx = p - start;
            const int pi = idx >= 0 ? idx / P : 0;
            const bool there = p <= pos && p >= first_key && idx >= 0 && pi < n_listed;
            const int row = there ? pt[pi] * P + (idx - pi * P) : -1;             // [page][row in page], one kv head
            float dot[QR];
#pragma unroll
            for (int r = 0; r < QR; ++r) dot[r] = 0.f;
            if (there) {
                const T* cr = v_pool + (size_t)row * C;
                const T* kr = k_pool + (size_t)row * R;
                if (vec) {
                    for (int j = part; 4 * j < C; j += 4) {
                        float kv[4];
                        lat_load4(cr + 4 * j, kv);
#pragma unroll
                        for (int r = 0; r < QR; ++r) {
                            const float4 qv = *reinterpret_cast<const float4*>(q_s + r * Dk + 4 * j);
                            dot[r] = fmaf(qv.x, kv[0], dot[r]);
                            dot[r] = fmaf(qv.y, kv[1], dot[r]);
                            dot[r] = fmaf(qv.z, kv[2], dot[r]);
                            dot[r] = fmaf(qv.w, kv[3], dot[r]);
                        }
                    }
                    for (int j = part; 4 * j < R; j += 4) {
                        float kv[4];
                        lat_load4(kr + 4 * j, kv);
#pragma unroll
                        for (int r = 0; r < QR; ++r) {
                            const float4 qv = *reinterpret_cast<const float4*>(q_s + r * Dk + C + 4 * j);
                            dot[r] = fmaf(qv.x, kv[0], dot[r]);
                            dot[r] = fmaf(qv.y, kv[1], dot[r]);
                            dot[r] = fmaf(qv.z, kv[2], dot[r]);
                            dot[r] = fmaf(qv.w, kv[3], dot[r]);
                        }
                    }
                } else {
                    for (int e = part; e < C; e += 4) {
                        const float kv = to_f(cr[e]);
#pragma unroll
                        for (int r = 0; r < QR; ++r) dot[r] = fmaf(q_s[r * Dk + e], kv, dot[r]);
                    }
                    for (int e = part; e < R; e += 4) {
                        const float kv = to_f(kr[e]);
#pragma unroll
                        for (int r = 0; r < QR; ++r) dot[r] = fmaf(q_s[r * Dk + C + e], kv, dot[r]);
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < QR; ++r) {
                float d = dot[r];
                d += __shfl_xor(d, 1, 64);
                d += __shfl_xor(d, 2, 64);
                sc[sp][r] = there ? d * scale : -INFINITY;
            }
            if (part == 0) my_row[kk] = row;
        }
        // ---- running maximum and sum of every row; the block's weights into LDS
#pragma unroll
        for (int r = 0; r < QR; ++r) {
            const float mx = wave_max(fmaxf(fmaxf(sc[0][r], sc[1][r]), fmaxf(sc[2][r], sc[3][r])));
            const float m_new = fmaxf(m[r], mx);
            const float alpha = (m[r] == -INFINITY) ? 0.f : expf(m[r] - m_new);
            float mine = 0.f;
#pragma unroll
            for (int sp = 0; sp < 4; ++sp) {
                const float pr = (sc[sp][r] == -INFINITY) ? 0.f : expf(sc[sp][r] - m_new);
                if (part == 0) {
                    my_p[r * 64 + 16 * sp + sub] = pr;
                    mine += pr;
                }
            }
            l[r] = l[r] * alpha + wave_sum(mine);
            m[r] = m_new;
#pragma unroll
            for (int i = 0; i < LAT_MAX_ACC; ++i) acc[r][i] *= alpha;
        }
        __builtin_amdgcn_wave_barrier();                 // LDS serves a wave's accesses in order
        // ---- sums over c: the lanes run along its elements
        const int nk = min(LAT_BLOCK, pos - base + 1);
#pragma unroll 4
        for (int kk = 0; kk < nk; ++kk) {
            const int row = max(my_row[kk], 0);          // a key that is not there has weight 0
            const T* cr = v_pool + (size_t)row * C;
            float pv[QR];
#pragma unroll
            for (int r = 0; r < QR; ++r) pv[r] = my_p[r * 64 + kk];
#pragma unroll
            for (int i = 0; i < LAT_MAX_ACC; ++i) {
                const int e = lane + 64 * i;
                if (e < C) {
                    const float v = to_f(cr[e]);
#pragma unroll
                    for (int r = 0; r < QR; ++r) acc[r][i] = fmaf(pv[r], v, acc[r][i]);
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }

    // ---- merge of the waves, in wave order
#pragma unroll
    for (int r = 0; r < QR; ++r) {
        if (lane == 0) {
            ml_s[(wave * QR + r) * 2] = m[r];
            ml_s[(wave * QR + r) * 2 + 1] = l[r];
        }
#pragma unroll
        for (int i = 0; i < LAT_MAX_ACC; ++i) {
            const int e = lane + 64 * i;
            if (e < C) acc_s[(wave * QR + r) * C + e] = acc[r][i];
        }
    }
    __syncthreads();
    for (int idx = tid; idx < QR * C; idx += WAVES * 64) {
        const int r = idx / C, e = idx - r * C;
        if (h0 + r >= Hn) continue;
        float mm = sink ? sink[h0 + r] : -INFINITY;      // the sink takes part in the maximum, so nothing overflows
        for (int w = 0; w < WAVES; ++w) mm = fmaxf(mm, ml_s[(w * QR + r) * 2]);
        float num = 0.f, den = 0.f;
        for (int w = 0; w < WAVES; ++w) {
            const float mw = ml_s[(w * QR + r) * 2];
            const float ew = (mw == -INFINITY) ? 0.f : expf(mw - mm);
            num = fmaf(acc_s[(w * QR + r) * C + e], ew, num);
            den = fmaf(ml_s[(w * QR + r) * 2 + 1], ew, den);
        }
        if (sink) den += expf(sink[h0 + r] - mm);
        out[((size_t)(h0 + r) * T_rows + t) * C + e] = from_f<T>(den > 0.f ? num / den : 0.f);
    }
}

static size_t latent_plain_lds(int QR, int WAVES, int C, int R) {
    return sizeof(float) * ((size_t)QR * (C + R) + (size_t)WAVES * QR * 64 + WAVES * 64 + WAVES * QR * 2 +
                            (size_t)WAVES * QR * C);
}

template <typename T, int QR, int WAVES>
static int latent_plain_launch(hipStream_t st, const void* qq, void* out, const void* k_pool, const void* v_pool,
                               const int* page_table, const int* cu_pages, const int* kv_start, const int* cu_q,
                               const int* q_start, const int* tok_ids, int n_seqs, int T_rows, int T_tokens, int Hn, int C,
                               int R, int P, float scale, const float* sink, int window) {
    const size_t lds = latent_plain_lds(QR, WAVES, C, R);
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute((const void*)attn_latent_plain_kernel<T, QR, WAVES>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
        return RA_ERR_LAUNCH;
    dim3 grid(T_tokens, (Hn + QR - 1) / QR), block(WAVES * 64);
    hipLaunchKernelGGL((attn_latent_plain_kernel<T, QR, WAVES>), grid, block, lds, st, (const T*)qq, (T*)out,
                       (const T*)k_pool, (const T*)v_pool, page_table, cu_pages, kv_start, cu_q, q_start, tok_ids, n_seqs,
                       T_rows, T_tokens, Hn, C, R, P, scale, sink, window);
    return ra_launch_status();
}

extern "C" int ra_attention_latent_plain_fits(int C, int R) {
    return (C >= 1 && C <= 64 * LAT_MAX_ACC && R >= 0 && R <= 512 &&
            latent_plain_lds(4, 8, C, R) <= 150 * 1024) ? 1 : 0;
}

extern "C" int ra_attention_latent_plain_window(const void* qq, void* out, const void* k_pool, const void* v_pool,
                                                const int* page_table, const int* cu_pages, const int* kv_start,
                                                const int* cu_q, const int* q_start, const int* tok_ids, int n_seqs,
                                                int T_rows, int T_tokens, int Hn, int C, int R, int P, float scale,
                                                const float* sink, int single, int window, int dtype, void* stream);

// qq [T_rows][Hn][C + R]; out [Hn][T_rows][C]; tok_ids (or null: all rows) lists the T_tokens rows to work on
extern "C" int ra_attention_latent_plain(const void* qq, void* out, const void* k_pool, const void* v_pool,
                                         const int* page_table, const int* cu_pages, const int* kv_start,
                                         const int* cu_q, const int* q_start, const int* tok_ids, int n_seqs,
                                         int T_rows, int T_tokens, int Hn, int C, int R, int P, float scale,
                                         const float* sink, int single, int dtype, void* stream) {
    return ra_attention_latent_plain_window(qq, out, k_pool, v_pool, page_table, cu_pages, kv_start, cu_q, q_start, tok_ids,
                                            n_seqs, T_rows, T_tokens, Hn, C, R, P, scale, sink, single, 0, dtype, stream);
}

// the same with a window (0: none)
extern "C" int ra_attention_latent_plain_window(const void* qq, void* out, const void* k_pool, const void* v_pool,
                                                const int* page_table, const int* cu_pages, const int* kv_start,
                                                const int* cu_q, const int* q_start, const int* tok_ids, int n_seqs,
                                                int T_rows, int T_tokens, int Hn, int C, int R, int P, float scale,
                                                const float* sink, int single, int window, int dtype, void* stream) {
    if (T_tokens <= 0 || n_seqs <= 0) return RA_OK;
    if (window < 0) return RA_ERR_ARG;
    if (!ra_attention_latent_plain_fits(C, R) || Hn < 1 || Hn > 65535 * 4 || P < 1 || T_tokens > T_rows) return RA_ERR_ARG;
    if (dtype != RA_DTYPE_F32 && dtype != RA_DTYPE_BF16) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
#define LAT_GO(T_, QR_, W_)                                                                                   \
    return latent_plain_launch<T_, QR_, W_>(st, qq, out, k_pool, v_pool, page_table, cu_pages, kv_start, cu_q, \
                                            q_start, tok_ids, n_seqs, T_rows, T_tokens, Hn, C, R, P, scale, sink, window)
    // rows of requests that bring one token: eight waves over the keys; else four
    if (dtype == RA_DTYPE_F32) {
        if (single) LAT_GO(float, 4, 8); else LAT_GO(float, 4, 4);
    } else {
        if (single) LAT_GO(bf16, 4, 8); else LAT_GO(bf16, 4, 4);
    }
#undef LAT_GO
}
