// Attention over a latent row per token on the matrix cores, bfloat16: the new tokens of a request, a portion
// of a prompt or a single token, over what the paged cache holds for it. The formulas and the tables are those of
// attention_latent.hip; sizes: a latent of C = 32, 64, 96, 128, 160, 192, 256, 384 or 512 elements, a rotated key
// part of R = 0 (none), 16, 32 or 64, at most 64 heads. With a window w > 0 a query at position i reads the keys j
// with 0 <= i - j < w: a tile's walk begins at the key block of its first row's earliest key.
//
// BUILD-VARIANTS: LAT_C32=1 LAT_C32=2 LAT_C32=3 LAT_C32=4 LAT_C32=5 LAT_C32=6 LAT_C32=8 LAT_C32=12 LAT_C32=16 LAT_API=1
//
// Every head of a token reads the same rows [c | kr], so the rows of a q tile are (token, head) pairs: a tile is
// TT = 64 / heads tokens (at least one) with all their heads, row r = token r / heads, head r % heads, and a row
// of keys that is brought into LDS serves up to 64 of them. One workgroup of four waves per tile; wave w owns
// rows 16w .. 16w+15. Per pass a tile of BN keys sits in LDS, each row [c (C) | kr (R)] with padding, and serves
// both products: as the keys of the scores, and its first C columns as the values. The next tile's rows are on
// their way from the cache into registers while this one is used.
//  scores  S^T = K Q^T by MFMA 16x16x32 bf16: A = 16 key rows from LDS, B = the wave's 16 query rows held in
//          registers. Lane (n, g) gets query n, keys 4g..4g+3 of each 16-key tile.
//  softmax one running maximum and sum per row, the scale folded into the exponent; 32-bit.
//  P.V     O^T += V^T P^T, P as the sum of two bfloat16 halves (two MFMAs), so that the weights keep 16 bits of
//          mantissa; the contraction runs over the keys in the order the lanes hold them, V^T comes from the
//          row-major tile through the transposing LDS read (ds_read_b64_tr_b16).
//  end     the sink's term joins the denominator (with the common maximum moved to the larger of the two, so that
//          nothing overflows); o = a / l.
// Requests that bring one token: their tile has `heads` rows; n_splits workgroups share the keys of a tile and
// leave maximum, sum and unnormed row to the merge kernel, which also adds the sink's term.
#include "common.h"

typedef __bf16 lbf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 lbf16x2_t __attribute__((ext_vector_type(2)));
typedef short lshort4_t __attribute__((ext_vector_type(4)));
typedef short lshort8_t __attribute__((ext_vector_type(8)));
typedef float lfloat4_t __attribute__((ext_vector_type(4)));
typedef float lfloat2_t __attribute__((ext_vector_type(2)));
typedef uint32_t luint4_t __attribute__((ext_vector_type(4)));
typedef lshort4_t __attribute__((address_space(3))) * llds_short4_ptr;

#define LAT_LOG2E 1.44269504088896340736f

#ifdef LAT_C32

__device__ __forceinline__ uint32_t lpack2(float a, float b) {
    const lfloat2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, lbf16x2_t));
}

template <int C32, int R16, int BN>
__global__ __launch_bounds__(256) void attn_latent_mfma_kernel(
    const bf16* __restrict__ qq, bf16* __restrict__ out, const bf16* __restrict__ k_pool,
    const bf16* __restrict__ v_pool, const int* __restrict__ page_table, const int* __restrict__ cu_pages,
    const int* __restrict__ kv_start, const int* __restrict__ cu_q, const int* __restrict__ q_start,
    const int* __restrict__ tiles,       // [n_tiles][2]: request number, first token of the tile within its new tokens
    int n_tiles, int T_rows, int Hn, int TT, int P, float scale, const float* __restrict__ sink, int n_splits,
    float* __restrict__ part, int window) {
    constexpr int C = 32 * C32, R = 16 * R16, CR = C + R, C16 = 2 * C32;
    constexpr int RF = R / 32;                          // whole 32-element steps of the rotated part
    constexpr bool TAIL16 = (R % 32) != 0;
    constexpr int NQ = C32 + RF;                        // whole 32-element steps of a score
    constexpr int KS = CR + (80 - CR % 64) % 64;        // row stride (elements): rows shift by 8 banks
    constexpr int LPR = CR / 8, LPC = C / 8;            // 16-byte pieces in one row, and in its latent part
    constexpr int NT = 256;
    constexpr int NK = (BN * LPR + NT - 1) / NT;        // pieces per thread per tile
    extern __shared__ __attribute__((aligned(16))) uint16_t k_s[];     // [BN][KS]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int tile = blockIdx.x;
    const int seg = tiles[2 * tile], q_off = tiles[2 * tile + 1];
    const int q_len = cu_q[seg + 1] - cu_q[seg];
    const int pos0 = q_start[seg];
    const int start = kv_start[seg];
    const int* pt = page_table + cu_pages[seg];

    // this lane's query row (for the B operands and for the mask): row n of the wave's 16
    const int row = wave * 16 + n;
    const int t_in = row / Hn, head = row - t_in * Hn;
    const int q_local = q_off + t_in;
    const bool q_ok = t_in < TT && q_local < q_len;
    const int pos_q = pos0 + q_local;
    const lbf16x8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};
    lbf16x8_t bq[NQ], bq_tail = z8;
    {
        const bf16* qp = qq + ((size_t)(cu_q[seg] + (q_ok ? q_local : 0)) * Hn + (q_ok ? head : 0)) * CR;
#pragma unroll
        for (int j = 0; j < NQ; ++j) {
            const lbf16x8_t v = *reinterpret_cast<const lbf16x8_t*>(qp + 32 * j + 8 * g);
            bq[j] = q_ok ? v : z8;
        }
        if constexpr (TAIL16) {
            if (q_ok && g < 2) bq_tail = *reinterpret_cast<const lbf16x8_t*>(qp + 32 * NQ + 8 * g);
        }
    }

    const int n_tok = min(TT, q_len - q_off);            // tokens of this tile
    const int tile_first_pos = pos0 + q_off;
    const int tile_last_pos = tile_first_pos + n_tok - 1;
    const int u_first = ((window > 0 ? max(start, tile_first_pos - window + 1) : start) / BN) * BN;
    // the wave's rows: the positions of its first and last token
    const int wave_first_pos = tile_first_pos + (wave * 16) / Hn;
    const int wave_last_pos = min(tile_first_pos + (wave * 16 + 15) / Hn, tile_last_pos);
    const bool wave_has_rows = (wave * 16) / Hn < n_tok;

    const float scale2 = scale * LAT_LOG2E;
    float m_run = -INFINITY, l_run = 0.f;
    lfloat4_t acc[C16];
#pragma unroll
    for (int dt = 0; dt < C16; ++dt) acc[dt] = lfloat4_t{0.f, 0.f, 0.f, 0.f};

    luint4_t kreg[NK];
    const int p_shift = (P & (P - 1)) == 0 ? __builtin_ctz(P) : -1;
    // cache row of key position kp (clamped into what this tile may read, so every address is valid)
    auto row_of = [&](int kp) {
        const int idx = min(max(kp, start), tile_last_pos) - start;
        const int pi = p_shift >= 0 ? (idx >> p_shift) : (idx / P);
        return pt[pi] * P + (idx - pi * P);
    };
    // The cache rows of a tile's pieces are looked up one pass before the pieces are asked for, so that a fetch
    // does not wait for the page table first.
    int rk[NK];
#define LAT_ROWS(u_)                                                                      \
    {                                                                                     \
        _Pragma("unroll") for (int i = 0; i < NK; ++i) {                                  \
            const int pc = tid + NT * i;                                                  \
            rk[i] = pc < BN * LPR ? row_of((u_) + pc / LPR) : 0;                          \
        }                                                                                 \
    }
#define LAT_FETCH()                                                                       \
    {                                                                                     \
        _Pragma("unroll") for (int i = 0; i < NK; ++i) {                                  \
            const int pc = tid + NT * i;                                                  \
            if (pc < BN * LPR) {                                                          \
                const int c_ = pc % LPR;                                                  \
                kreg[i] = c_ < LPC                                                        \
                    ? *reinterpret_cast<const luint4_t*>(v_pool + (size_t)rk[i] * C + 8 * c_)             \
                    : *reinterpret_cast<const luint4_t*>(k_pool + (size_t)rk[i] * R + 8 * (c_ - LPC));    \
            }                                                                             \
        }                                                                                 \
    }
#define LAT_STAGE()                                                                       \
    {                                                                                     \
        _Pragma("unroll") for (int i = 0; i < NK; ++i) {                                  \
            const int pc = tid + NT * i;                                                  \
            if (pc < BN * LPR) {                                                          \
                const int r_ = pc / LPR, c_ = pc - r_ * LPR;                              \
                *reinterpret_cast<luint4_t*>(k_s + r_ * KS + 8 * c_) = kreg[i];           \
            }                                                                             \
        }                                                                                 \
    }

    // With n_splits > 1 the workgroups blockIdx.y = 0, 1, ... share the tile's key blocks evenly and leave their
    // sums to the merge kernel.
    int u_lo = u_first, u_hi = tile_last_pos;            // first key block, and the last key, of this workgroup
    if (n_splits > 1) {
        const int blocks = (tile_last_pos - u_first) / BN + 1;
        const int per = (blocks + n_splits - 1) / n_splits;
        u_lo = u_first + (int)blockIdx.y * per * BN;
        u_hi = min(tile_last_pos, u_lo + per * BN - 1);
    }
    if (u_lo <= u_hi) {
        LAT_ROWS(u_lo)
        LAT_FETCH()
        LAT_ROWS(u_lo + BN)                              // (beyond the last key the rows are clamped to valid ones)
    }
    for (int u = u_lo; u <= u_hi; u += BN) {
        __syncthreads();                                 // every wave is done with the tile before
        LAT_STAGE()
        __syncthreads();
        if (u + BN <= u_hi) {                            // the next tile, on its way while this one is used
            LAT_FETCH()
            LAT_ROWS(u + 2 * BN)
        }

        // a tile that lies wholly above every row of the wave has nothing for it; nor has any tile for a wave
        // whose rows all lie beyond the tile's tokens (such waves only help to move the tiles)
        if (wave_has_rows && u <= wave_last_pos && (window <= 0 || u + BN - 1 > wave_first_pos - window)) {
            lfloat4_t cs[BN / 16];
#pragma unroll
            for (int st = 0; st < BN / 16; ++st) {
                const uint16_t* kr = &k_s[(st * 16 + n) * KS];
                cs[st] = lfloat4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < NQ; ++j) {
                    const lbf16x8_t a = *reinterpret_cast<const lbf16x8_t*>(kr + 32 * j + 8 * g);
                    cs[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bq[j], cs[st], 0, 0, 0);
                }
                if constexpr (TAIL16) {
                    lbf16x8_t a = z8;
                    if (g < 2) a = *reinterpret_cast<const lbf16x8_t*>(kr + 32 * NQ + 8 * g);
                    cs[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bq_tail, cs[st], 0, 0, 0);
                }
            }
            MFMA_SETTLE();
            // a tile that every row of the wave reads whole needs no mask
            const bool need_mask = (u + BN - 1 > wave_first_pos) || (u < start) || (window > 0 && u <= wave_last_pos - window);
            luint4_t pw[BN / 32], pl[BN / 32];           // the weights' upper and lower halves, in the order the B operand wants
            float s[BN / 16][4];
            float mx = -INFINITY;
            if (need_mask) {
#pragma unroll
                for (int st = 0; st < BN / 16; ++st)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int kpos = u + st * 16 + 4 * g + i;
                        const bool ok = kpos >= start && kpos <= pos_q && (window <= 0 || kpos > pos_q - window);
                        s[st][i] = ok ? cs[st][i] : -INFINITY;
                        mx = fmaxf(mx, s[st][i]);
                    }
            } else {
#pragma unroll
                for (int st = 0; st < BN / 16; ++st)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s[st][i] = cs[st][i];
                        mx = fmaxf(mx, s[st][i]);
                    }
            }
            mx = rows_max(mx);
            const float m_new = fmaxf(m_run, mx);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;      // a row that sees no key yet keeps m = -inf
            const float off = -m_use * scale2;
            float lsum = 0.f;
#pragma unroll
            for (int st = 0; st < BN / 16; ++st)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s[st][i] = __builtin_amdgcn_exp2f(fmaf(s[st][i], scale2, off));      // 2^(-inf) = 0 for masked keys
                    lsum += s[st][i];
                }
            lsum = rows_sum(lsum);
            const float alpha = (m_run == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_run - m_use) * scale2);
            l_run = l_run * alpha + lsum;
            if (__any(m_new != m_run)) {
#pragma unroll
                for (int dt = 0; dt < C16; ++dt) {
                    acc[dt][0] *= alpha;
                    acc[dt][1] *= alpha;
                    acc[dt][2] *= alpha;
                    acc[dt][3] *= alpha;
                }
            }
            m_run = m_new;
            // the weights go into the product as two bfloat16 numbers each, p = hi + lo (16 bits of mantissa between
            // them): the product's operands are 16-bit, the weights are not rounded to that
#pragma unroll
            for (int b = 0; b < BN / 32; ++b) {
                const luint4_t hi = luint4_t{lpack2(s[2 * b][0], s[2 * b][1]), lpack2(s[2 * b][2], s[2 * b][3]),
                                             lpack2(s[2 * b + 1][0], s[2 * b + 1][1]), lpack2(s[2 * b + 1][2], s[2 * b + 1][3])};
                pw[b] = hi;
                float r[8];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    r[2 * e] = s[2 * b + e / 2][2 * (e & 1)] - __uint_as_float(hi[e] << 16);
                    r[2 * e + 1] = s[2 * b + e / 2][2 * (e & 1) + 1] - __uint_as_float(hi[e] & 0xffff0000u);
                }
                pl[b] = luint4_t{lpack2(r[0], r[1]), lpack2(r[2], r[3]), lpack2(r[4], r[5]), lpack2(r[6], r[7])};
            }
            // ---- O^T += V^T P^T, 32 keys per MFMA; V^T through the transposing LDS read
#pragma unroll
            for (int b = 0; b < BN / 32; ++b) {
                // this lane's address as lane l' = n of its group: key 32b + 4g + n/4, columns 4(n%4)..+3
                const uint16_t* vr = &k_s[(32 * b + 4 * g + (n >> 2)) * KS + 4 * (n & 3)];
#pragma unroll
                for (int dt = 0; dt < C16; ++dt) {
                    const lshort4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((llds_short4_ptr)(vr + dt * 16));
                    const lshort4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((llds_short4_ptr)(vr + 16 * KS + dt * 16));
                    const lshort8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(lbf16x8_t, both), __builtin_bit_cast(lbf16x8_t, pl[b]), acc[dt], 0, 0, 0);
                    acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(lbf16x8_t, both), __builtin_bit_cast(lbf16x8_t, pw[b]), acc[dt], 0, 0, 0);
                }
            }
        }
    }
#undef LAT_FETCH
#undef LAT_ROWS
#undef LAT_STAGE
    MFMA_SETTLE();
    // ---- acc[dt][i] = O^T[d = 16dt + 4g + i][query n]
    if (!q_ok) return;
    if (n_splits > 1) {
        // per row and split: the running maximum (a raw score), the sum and the unnormed row
        float* pm = part + (((size_t)tile * Hn + head) * n_splits + blockIdx.y) * (C + 2);
        if (g == 0) {
            pm[0] = m_run;
            pm[1] = l_run;
        }
#pragma unroll
        for (int dt = 0; dt < C16; ++dt) {
            float* d = pm + 2 + dt * 16 + 4 * g;
            d[0] = acc[dt][0];
            d[1] = acc[dt][1];
            d[2] = acc[dt][2];
            d[3] = acc[dt][3];
        }
        return;
    }
    // the sink: one more term exp(sink - M) in the denominator, M the maximum of the scaled scores; with the
    // common maximum moved to max(M, sink)
    float f;
    {
        const float M2 = (m_run == -INFINITY) ? -INFINITY : m_run * scale2;      // in powers of two
        float keep = 1.f, den = l_run;
        if (sink != nullptr) {
            const float s2 = sink[head] * LAT_LOG2E;
            const float top = fmaxf(M2, s2);
            keep = (M2 == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(M2 - top);
            den = l_run * keep + __builtin_amdgcn_exp2f(s2 - top);
        }
        f = den > 0.f ? keep / den : 0.f;
    }
    bf16* op = out + ((size_t)head * T_rows + cu_q[seg] + q_local) * C;
#pragma unroll
    for (int dt = 0; dt < C16; ++dt) {
        uint2 w;
        w.x = lpack2(acc[dt][0] * f, acc[dt][1] * f);
        w.y = lpack2(acc[dt][2] * f, acc[dt][3] * f);
        *reinterpret_cast<uint2*>(op + dt * 16 + 4 * g) = w;
    }
}

#define LAT_CAT2(a, b) a##b
#define LAT_CAT(a, b) LAT_CAT2(a, b)
#define LAT_PART_ARGS int R16, dim3 grid, hipStream_t st, const bf16* qq, bf16* out, const bf16* kp, const bf16* vp,   \
    const int* pt, const int* cup, const int* kvs, const int* cuq, const int* qs, const int* tiles, int n_tiles,       \
    int T_rows, int Hn, int TT, int P, float scale, const float* sink, int n_splits, float* part, int window

template <int RR>
static int lat_part_launch(LAT_PART_ARGS) {
    constexpr int CR = 32 * LAT_C32 + 16 * RR;
    constexpr int KS = CR + (80 - CR % 64) % 64;
    // 64 keys a pass while a row of keys and rotated parts stays short, else 32 (the tile on its way sits in registers)
    constexpr int BN = CR >= 320 ? 32 : 64;
    constexpr int LDS = BN * KS * 2;
    if (LDS > 64 * 1024 &&
        hipFuncSetAttribute((const void*)attn_latent_mfma_kernel<LAT_C32, RR, BN>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS) != hipSuccess)
        return RA_ERR_LAUNCH;
    hipLaunchKernelGGL((attn_latent_mfma_kernel<LAT_C32, RR, BN>), grid, dim3(256), LDS, st, qq, out, kp, vp, pt, cup, kvs,
                       cuq, qs, tiles, n_tiles, T_rows, Hn, TT, P, scale, sink, n_splits, part, window);
    return RA_OK;
}

extern "C" int LAT_CAT(ra_latent_part_, LAT_C32)(LAT_PART_ARGS) {
    switch (R16) {
        case 0: return lat_part_launch<0>(R16, grid, st, qq, out, kp, vp, pt, cup, kvs, cuq, qs, tiles, n_tiles, T_rows, Hn,
                                          TT, P, scale, sink, n_splits, part, window);
        case 1: return lat_part_launch<1>(R16, grid, st, qq, out, kp, vp, pt, cup, kvs, cuq, qs, tiles, n_tiles, T_rows, Hn,
                                          TT, P, scale, sink, n_splits, part, window);
        case 2: return lat_part_launch<2>(R16, grid, st, qq, out, kp, vp, pt, cup, kvs, cuq, qs, tiles, n_tiles, T_rows, Hn,
                                          TT, P, scale, sink, n_splits, part, window);
        case 4: return lat_part_launch<4>(R16, grid, st, qq, out, kp, vp, pt, cup, kvs, cuq, qs, tiles, n_tiles, T_rows, Hn,
                                          TT, P, scale, sink, n_splits, part, window);
        default: return RA_ERR_ARG;
    }
}
#endif  // LAT_C32

#ifdef LAT_API
#define LAT_PART_ARGS int R16, dim3 grid, hipStream_t st, const bf16* qq, bf16* out, const bf16* kp, const bf16* vp,   \
    const int* pt, const int* cup, const int* kvs, const int* cuq, const int* qs, const int* tiles, int n_tiles,       \
    int T_rows, int Hn, int TT, int P, float scale, const float* sink, int n_splits, float* part, int window
extern "C" int ra_latent_part_1(LAT_PART_ARGS);
extern "C" int ra_latent_part_2(LAT_PART_ARGS);
extern "C" int ra_latent_part_3(LAT_PART_ARGS);
extern "C" int ra_latent_part_4(LAT_PART_ARGS);
extern "C" int ra_latent_part_5(LAT_PART_ARGS);
extern "C" int ra_latent_part_6(LAT_PART_ARGS);
extern "C" int ra_latent_part_8(LAT_PART_ARGS);
extern "C" int ra_latent_part_12(LAT_PART_ARGS);
extern "C" int ra_latent_part_16(LAT_PART_ARGS);

// Whether the matrix-core kernel takes a latent of C, a rotated part of R and Hn heads.
extern "C" int ra_attention_latent_mfma_fits(int C, int R, int Hn) {
    if (C % 32 || Hn < 1 || Hn > 64) return 0;
    const int c32 = C / 32;
    const bool c_ok = (c32 >= 1 && c32 <= 6) || c32 == 8 || c32 == 12 || c32 == 16;
    return c_ok && (R == 0 || R == 16 || R == 32 || R == 64);
}

// Tokens per q tile for Hn heads: the lists of tiles a step brings are cut to this many rows.
extern "C" int ra_attention_latent_mfma_tile_tokens(int Hn) {
    return Hn >= 1 && Hn <= 64 ? 64 / Hn : 0;
}

// The sums of a tile's splits into its output rows: the splits' maxima, sums and unnormed rows are merged in split
// order, the sink's term joins the denominator. One wave per (tile, head); the tile's one token is row cu_q[request].
__global__ __launch_bounds__(64) void attn_latent_merge_kernel(const float* __restrict__ part, bf16* __restrict__ out,
                                                               const int* __restrict__ tiles, const int* __restrict__ cu_q,
                                                               int T_rows, int Hn, int C, int n_splits, float scale,
                                                               const float* __restrict__ sink) {
    const int tile = blockIdx.x / Hn, head = blockIdx.x % Hn, lane = threadIdx.x;
    const float scale2 = scale * LAT_LOG2E;
    const float* pp = part + (size_t)blockIdx.x * n_splits * (C + 2);
    const int token_row = cu_q[tiles[2 * tile]] + tiles[2 * tile + 1];
    // lane sp reads split sp's maximum and sum (n_splits <= 64), all at once
    const float* mine = pp + (size_t)min(lane, n_splits - 1) * (C + 2);
    const float my_m = lane < n_splits ? mine[0] : -INFINITY;
    const float my_l = lane < n_splits ? mine[1] : 0.f;
    const float m_all = wave_max(my_m);
    const float M2 = (m_all == -INFINITY) ? -INFINITY : m_all * scale2;
    const float s2 = sink != nullptr ? sink[head] * LAT_LOG2E : -INFINITY;
    const float top = fmaxf(M2, s2);
    // weight of split sp's sums under the common maximum `top`
    const float my_w = (my_m == -INFINITY || top == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(my_m * scale2 - top);
    float l = 0.f, a[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};       // elements lane, lane + 64, ... (C <= 512)
    for (int s0 = 0; s0 < n_splits; s0 += 4) {           // four splits' rows asked for at once, added in split order
        float raw[4][8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float* pm = pp + (size_t)min(s0 + j, n_splits - 1) * (C + 2) + 2;
#pragma unroll
            for (int i = 0; i < 8; ++i) raw[j][i] = lane + 64 * i < C ? pm[lane + 64 * i] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (s0 + j >= n_splits) break;
            const float wgt = __shfl(my_w, s0 + j, 64);
            l = fmaf(__shfl(my_l, s0 + j, 64), wgt, l);
#pragma unroll
            for (int i = 0; i < 8; ++i) a[i] = fmaf(raw[j][i], wgt, a[i]);
        }
    }
    if (sink != nullptr && top != -INFINITY) l += __builtin_amdgcn_exp2f(s2 - top);
    const float f = l > 0.f ? 1.0f / l : 0.f;
    bf16* op = out + ((size_t)head * T_rows + token_row) * C;
#pragma unroll
    for (int i = 0; i < 8; ++i)
        if (lane + 64 * i < C) op[lane + 64 * i] = from_f<bf16>(a[i] * f);
}

// floats of the buffer that n_splits > 1 needs for n_tiles one-token tiles
extern "C" long long ra_attention_latent_mfma_part_floats(int n_tiles, int Hn, int C, int n_splits) {
    return (long long)n_tiles * Hn * n_splits * (C + 2);
}

extern "C" int ra_attention_latent_mfma_window_bf16(const void* qq, void* out, const void* k_pool, const void* v_pool,
                                                    const int* page_table, const int* cu_pages, const int* kv_start,
                                                    const int* cu_q, const int* q_start, const int* tiles, int n_tiles,
                                                    int T_rows, int Hn, int C, int R, int P, float scale,
                                                    const float* sink, int n_splits, float* part, int window,
                                                    void* stream);

// qq [T_rows][Hn][C + R]; out [Hn][T_rows][C]. tiles: int32 [n_tiles][2] = (request number, first token of the tile
// within the request's new tokens), tiles of TT = 64 / Hn tokens over the requests to work on (a request that brings
// one token is one tile). n_splits > 1: every tile has ONE token, its keys are shared among n_splits workgroups
// whose sums go through part (ra_attention_latent_mfma_part_floats floats) and the merge kernel.
extern "C" int ra_attention_latent_mfma_bf16(const void* qq, void* out, const void* k_pool, const void* v_pool,
                                             const int* page_table, const int* cu_pages, const int* kv_start,
                                             const int* cu_q, const int* q_start, const int* tiles, int n_tiles,
                                             int T_rows, int Hn, int C, int R, int P, float scale, const float* sink,
                                             int n_splits, float* part, void* stream) {
    return ra_attention_latent_mfma_window_bf16(qq, out, k_pool, v_pool, page_table, cu_pages, kv_start, cu_q, q_start,
                                                tiles, n_tiles, T_rows, Hn, C, R, P, scale, sink, n_splits, part, 0, stream);
}

// the same with a window (0: none)
extern "C" int ra_attention_latent_mfma_window_bf16(const void* qq, void* out, const void* k_pool, const void* v_pool,
                                                    const int* page_table, const int* cu_pages, const int* kv_start,
                                                    const int* cu_q, const int* q_start, const int* tiles, int n_tiles,
                                                    int T_rows, int Hn, int C, int R, int P, float scale,
                                                    const float* sink, int n_splits, float* part, int window,
                                                    void* stream) {
    if (n_tiles <= 0) return RA_OK;
    if (window < 0) return RA_ERR_ARG;
    if (!ra_attention_latent_mfma_fits(C, R, Hn) || P <= 0 || n_splits < 1 || n_splits > 64 || !(scale > 0.f) ||
        (n_splits > 1 && part == nullptr) || (long long)n_tiles * Hn > 0x7fffffffLL)
        return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int TT = ra_attention_latent_mfma_tile_tokens(Hn);
    dim3 grid(n_tiles, n_splits);
    int rc;
#define LAT_GO(k)                                                                                             \
    rc = ra_latent_part_##k(R / 16, grid, st, (const bf16*)qq, (bf16*)out, (const bf16*)k_pool, (const bf16*)v_pool, \
                            page_table, cu_pages, kv_start, cu_q, q_start, tiles, n_tiles, T_rows, Hn, TT, P, scale, \
                            sink, n_splits, part, window)
    switch (C / 32) {
        case 1: LAT_GO(1); break;
        case 2: LAT_GO(2); break;
        case 3: LAT_GO(3); break;
        case 4: LAT_GO(4); break;
        case 5: LAT_GO(5); break;
        case 6: LAT_GO(6); break;
        case 8: LAT_GO(8); break;
        case 12: LAT_GO(12); break;
        case 16: LAT_GO(16); break;
        default: return RA_ERR_ARG;
    }
#undef LAT_GO
    if (rc != RA_OK) return rc;
    if (n_splits > 1)
        hipLaunchKernelGGL(attn_latent_merge_kernel, dim3(n_tiles * Hn), dim3(64), 0, st, part, (bf16*)out, tiles, cu_q,
                           T_rows, Hn, C, n_splits, scale, sink);
    return ra_launch_status();
}
#endif  // LAT_API
