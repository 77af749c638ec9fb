// Row kernels of a layer whose sublayers run side by side, of an attention with biases and blended values, and of
// an expert that every token uses.
//
//   add_rmsnorm_pair   h += a + b (the 32-bit stream; a and b, in the storage type, may each be null), then two RMS
//                      norms of the same row with weights of their own: x1 = h / sqrt(mean(h^2) + eps1) * w1,
//                      x2 = h / sqrt(mean(h^2) + eps2) * w2. One workgroup per row, one pass over the row: its
//                      elements stay in registers between the sum of squares and the two results.
//   qkv_blend_prepare  one wave per (token, head) over the projection row [q heads | k heads | v heads], all heads
//                      of D elements: a 32-bit bias per column is added; the first R elements of a q or k head turn by
//                      the token's position, element j with j + R/2; q goes to q_out [T, Hq, D], k to its row of the
//                      key pool. v: mode 1 writes the first Dv elements of the biased v into `first` (32-bit,
//                      [T, Hkv, Dv]: a head's true width, which layers of other row widths share) and v into the
//                      value pool; mode 2 stores (1 - lambda) v + lambda first[t]; mode 0 stores v.
//   clamped_mul        out[t][i] = g sigmoid(slope g) (u + 1) with g = min(gu[t][i], limit),
//                      u = clamp(gu[t][I + i], -limit, limit); gu rows are ld_gu elements apart.
#include "common.h"
#include <algorithm>

#define PR_THREADS 256
#define PR_KEEP 16

template <typename T>
__global__ __launch_bounds__(PR_THREADS) void add_rmsnorm_pair_kernel(
    float* __restrict__ h, const T* __restrict__ a, const T* __restrict__ b, const float* __restrict__ w1, float eps1,
    T* __restrict__ x1, const float* __restrict__ w2, float eps2, T* __restrict__ x2, int H) {
    __shared__ float scratch[16];
    const size_t r = blockIdx.x;
    float* hr = h + r * H;
    const bool fits = H <= PR_THREADS * PR_KEEP;
    float ss = 0.f;
    if (fits) {
        // every read of the row is asked for before the first sum
        float v[PR_KEEP], av[PR_KEEP], bv[PR_KEEP], w1v[PR_KEEP], w2v[PR_KEEP];
#pragma unroll
        for (int i = 0; i < PR_KEEP; ++i) {
            const int c = threadIdx.x + i * PR_THREADS;
            const bool in = c < H;
            v[i] = in ? hr[c] : 0.f;
            av[i] = (in && a != nullptr) ? to_f(a[r * H + c]) : 0.f;
            bv[i] = (in && b != nullptr) ? to_f(b[r * H + c]) : 0.f;
            w1v[i] = in ? w1[c] : 0.f;
            w2v[i] = in ? w2[c] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < PR_KEEP; ++i) {
            v[i] = (v[i] + av[i]) + bv[i];
            ss = fmaf(v[i], v[i], ss);
        }
        const float ms = block_sum(ss, scratch) / (float)H;
        const float r1 = 1.0f / sqrtf(ms + eps1), r2 = 1.0f / sqrtf(ms + eps2);
#pragma unroll
        for (int i = 0; i < PR_KEEP; ++i) {
            const int c = threadIdx.x + i * PR_THREADS;
            if (c < H) {
                if (a != nullptr || b != nullptr) hr[c] = v[i];
                x1[r * H + c] = from_f<T>(v[i] * r1 * w1v[i]);
                x2[r * H + c] = from_f<T>(v[i] * r2 * w2v[i]);
            }
        }
        return;
    }
    for (int c = threadIdx.x; c < H; c += PR_THREADS) {
        float v = hr[c];
        if (a != nullptr) v += to_f(a[r * H + c]);
        if (b != nullptr) v += to_f(b[r * H + c]);
        if (a != nullptr || b != nullptr) hr[c] = v;
        ss = fmaf(v, v, ss);
    }
    const float ms = block_sum(ss, scratch) / (float)H;
    const float r1 = 1.0f / sqrtf(ms + eps1), r2 = 1.0f / sqrtf(ms + eps2);
    for (int c = threadIdx.x; c < H; c += PR_THREADS) {
        const float v = hr[c];                               // (the thread's own store, or the stream as it was)
        x1[r * H + c] = from_f<T>(v * r1 * w1[c]);
        x2[r * H + c] = from_f<T>(v * r2 * w2[c]);
    }
}

// The same for rows of H = 4 n elements up to 4,096: a thread takes four neighbours at a time (16-byte reads of the
// stream and the weights, 8- or 16-byte reads of the deltas), all asked for before the first sum.
__device__ __forceinline__ float4 pr_load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 pr_load4(const bf16* p) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(t.x << 16), __uint_as_float(t.x & 0xffff0000u), __uint_as_float(t.y << 16),
                       __uint_as_float(t.y & 0xffff0000u));
}
__device__ __forceinline__ void pr_store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void pr_store4(bf16* p, float4 v) {
    uint2 t;
    t.x = (uint32_t)f2bf_bits(v.x) | ((uint32_t)f2bf_bits(v.y) << 16);
    t.y = (uint32_t)f2bf_bits(v.z) | ((uint32_t)f2bf_bits(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = t;
}

#define PR_VEC 4          // groups of four a thread: rows up to 4 * 4 * 256
template <typename T>
__global__ __launch_bounds__(PR_THREADS) void add_rmsnorm_pair_vec_kernel(
    float* __restrict__ h, const T* __restrict__ a, const T* __restrict__ b, const float* __restrict__ w1, float eps1,
    T* __restrict__ x1, const float* __restrict__ w2, float eps2, T* __restrict__ x2, int H) {
    __shared__ float scratch[16];
    const size_t r = blockIdx.x;
    float* hr = h + r * H;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 v[PR_VEC], av[PR_VEC], bv[PR_VEC], w1v[PR_VEC], w2v[PR_VEC];
#pragma unroll
    for (int i = 0; i < PR_VEC; ++i) {
        const int c = 4 * (threadIdx.x + i * PR_THREADS);
        const bool in = c < H;
        v[i] = in ? pr_load4(hr + c) : zero;
        av[i] = (in && a != nullptr) ? pr_load4(a + r * H + c) : zero;
        bv[i] = (in && b != nullptr) ? pr_load4(b + r * H + c) : zero;
        w1v[i] = in ? pr_load4(w1 + c) : zero;
        w2v[i] = in ? pr_load4(w2 + c) : zero;
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PR_VEC; ++i) {
        v[i].x = (v[i].x + av[i].x) + bv[i].x;
        v[i].y = (v[i].y + av[i].y) + bv[i].y;
        v[i].z = (v[i].z + av[i].z) + bv[i].z;
        v[i].w = (v[i].w + av[i].w) + bv[i].w;
        ss = fmaf(v[i].x, v[i].x, ss);
        ss = fmaf(v[i].y, v[i].y, ss);
        ss = fmaf(v[i].z, v[i].z, ss);
        ss = fmaf(v[i].w, v[i].w, ss);
    }
    const float ms = block_sum(ss, scratch) / (float)H;
    const float r1 = 1.0f / sqrtf(ms + eps1), r2 = 1.0f / sqrtf(ms + eps2);
#pragma unroll
    for (int i = 0; i < PR_VEC; ++i) {
        const int c = 4 * (threadIdx.x + i * PR_THREADS);
        if (c < H) {
            if (a != nullptr || b != nullptr) pr_store4(hr + c, v[i]);
            pr_store4(x1 + r * H + c, make_float4(v[i].x * r1 * w1v[i].x, v[i].y * r1 * w1v[i].y, v[i].z * r1 * w1v[i].z,
                                                  v[i].w * r1 * w1v[i].w));
            pr_store4(x2 + r * H + c, make_float4(v[i].x * r2 * w2v[i].x, v[i].y * r2 * w2v[i].y, v[i].z * r2 * w2v[i].z,
                                                  v[i].w * r2 * w2v[i].w));
        }
    }
}

extern "C" int ra_add_rmsnorm_pair(float* h, const void* a, const void* b, const float* w1, float eps1, void* x1,
                                   const float* w2, float eps2, void* x2, int rows, int H, int dtype, void* stream) {
    if (rows <= 0) return RA_OK;
    if (H < 1 || h == nullptr || w1 == nullptr || w2 == nullptr || x1 == nullptr || x2 == nullptr) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (dtype != RA_DTYPE_F32 && dtype != RA_DTYPE_BF16) return RA_ERR_ARG;
    const auto aligned = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    if (H % 4 == 0 && H <= 4 * PR_VEC * PR_THREADS && aligned(h) && aligned(a) && aligned(b) && aligned(w1) && aligned(w2) &&
        aligned(x1) && aligned(x2) && (dtype == RA_DTYPE_F32 || H % 8 == 0)) {
        if (dtype == RA_DTYPE_F32)
            hipLaunchKernelGGL(add_rmsnorm_pair_vec_kernel<float>, dim3(rows), dim3(PR_THREADS), 0, st, h, (const float*)a,
                               (const float*)b, w1, eps1, (float*)x1, w2, eps2, (float*)x2, H);
        else
            hipLaunchKernelGGL(add_rmsnorm_pair_vec_kernel<bf16>, dim3(rows), dim3(PR_THREADS), 0, st, h, (const bf16*)a,
                               (const bf16*)b, w1, eps1, (bf16*)x1, w2, eps2, (bf16*)x2, H);
        return ra_launch_status();
    }
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(add_rmsnorm_pair_kernel<float>, dim3(rows), dim3(PR_THREADS), 0, st, h, (const float*)a,
                           (const float*)b, w1, eps1, (float*)x1, w2, eps2, (float*)x2, H);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(add_rmsnorm_pair_kernel<bf16>, dim3(rows), dim3(PR_THREADS), 0, st, h, (const bf16*)a,
                           (const bf16*)b, w1, eps1, (bf16*)x1, w2, eps2, (bf16*)x2, H);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}

// ------------------------------------------------------------------ q/k/v preparation with biases and blended values
template <typename T>
__global__ void qkv_blend_prepare_kernel(const T* __restrict__ qkv, int Hq, int Hkv, int D, const float* __restrict__ bias,
                                         const int* __restrict__ positions, const float* __restrict__ cos_t,
                                         const float* __restrict__ sin_t, int R, T* __restrict__ q_out,
                                         T* __restrict__ k_pool, T* __restrict__ v_pool, const int* __restrict__ slots,
                                         int P, long long pool_rows, float* __restrict__ first, int Dv, int mode,
                                         float lambda, long long n_rows) {
    const long long row = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int lane = threadIdx.x & 63;
    const int heads = Hq + 2 * Hkv;
    const int t = (int)(row / heads);
    const int head = (int)(row % heads);
    const T* src = qkv + row * D;
    const float* b = bias + (size_t)head * D;
    if (head >= Hq + Hkv) {
        // a value head: bias, the first layer's values out or blended in, the cache row
        const int kvh = head - Hq - Hkv;
        float* fr = first != nullptr ? first + ((size_t)t * Hkv + kvh) * Dv : nullptr;
        T* dst = nullptr;
        if (v_pool != nullptr) {
            const long long s = slots[t];
            if (s >= 0 && s < pool_rows) dst = v_pool + ra_cache_offset(s, kvh, Hkv, P, D);
        }
        for (int c = lane; c < D; c += 64) {
            float v = to_f(src[c]) + b[c];
            if (mode == 1 && c < Dv) fr[c] = v;
            else if (mode == 2) v = (1.0f - lambda) * v + (c < Dv ? lambda * fr[c] : 0.f);
            if (dst != nullptr) dst[c] = from_f<T>(v);
        }
        return;
    }
    T* dst;
    if (head < Hq) {
        dst = q_out + ((size_t)t * Hq + head) * D;
    } else {
        if (k_pool == nullptr) return;
        const long long s = slots[t];
        if (s < 0 || s >= pool_rows) return;
        dst = k_pool + ra_cache_offset(s, head - Hq, Hkv, P, D);
    }
    const int half = R >> 1;
    const int pos = positions[t];
    for (int j = lane; j < half; j += 64) {
        const float x1 = to_f(src[j]) + b[j], x2 = to_f(src[j + half]) + b[j + half];
        const float cs = cos_t[(size_t)pos * half + j], sn = sin_t[(size_t)pos * half + j];
        dst[j] = from_f<T>(x1 * cs - x2 * sn);
        dst[j + half] = from_f<T>(x2 * cs + x1 * sn);
    }
    for (int c = R + lane; c < D; c += 64) dst[c] = from_f<T>(to_f(src[c]) + b[c]);
}

extern "C" int ra_qkv_blend_prepare(const void* qkv, int T_tokens, int Hq, int Hkv, int D, const float* bias,
                                    const int* positions, const float* cos_t, const float* sin_t, int R, void* q_out,
                                    void* k_pool, void* v_pool, const int* slots, int P, long long pool_rows,
                                    float* first, int Dv, int mode, float lambda, int dtype, void* stream) {
    if (T_tokens <= 0) return RA_OK;
    if ((k_pool == nullptr) != (v_pool == nullptr) || (k_pool != nullptr && (P <= 0 || slots == nullptr))) return RA_ERR_ARG;
    if (D < 1 || Hq < 1 || Hkv < 1 || R < 0 || R > D || (R & 1) || bias == nullptr || q_out == nullptr ||
        (R > 0 && (cos_t == nullptr || sin_t == nullptr)) || mode < 0 || mode > 2 ||
        (mode != 0 && (first == nullptr || Dv < 1 || Dv > D)))
        return RA_ERR_ARG;
    const long long n_rows = (long long)T_tokens * (Hq + 2 * Hkv);
    dim3 block(256), grid((unsigned)((n_rows + 3) / 4));
    hipStream_t st = (hipStream_t)stream;
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(qkv_blend_prepare_kernel<float>, grid, block, 0, st, (const float*)qkv, Hq, Hkv, D, bias,
                           positions, cos_t, sin_t, R, (float*)q_out, (float*)k_pool, (float*)v_pool, slots, P, pool_rows,
                           first, Dv, mode, lambda, n_rows);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(qkv_blend_prepare_kernel<bf16>, grid, block, 0, st, (const bf16*)qkv, Hq, Hkv, D, bias,
                           positions, cos_t, sin_t, R, (bf16*)q_out, (bf16*)k_pool, (bf16*)v_pool, slots, P, pool_rows,
                           first, Dv, mode, lambda, n_rows);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}

// ------------------------------------------------------------------ the shared expert's activation
template <typename T>
__global__ void clamped_mul_kernel(const T* __restrict__ gu, long long ld_gu, T* __restrict__ out, int I, float limit,
                                   float slope, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t t = i / I;
        const int c = (int)(i - t * I);
        const float g = fminf(to_f(gu[t * ld_gu + c]), limit);
        const float u = fminf(fmaxf(to_f(gu[t * ld_gu + I + c]), -limit), limit);
        out[i] = from_f<T>(g / (1.0f + expf(-slope * g)) * (u + 1.0f));
    }
}

extern "C" int ra_clamped_mul(const void* gu, long long ld_gu, void* out, int T_tokens, int I, float limit, float slope,
                              int dtype, void* stream) {
    if (T_tokens <= 0) return RA_OK;
    if (I < 1 || ld_gu < 2LL * I || !(limit > 0.f)) return RA_ERR_ARG;
    const size_t total = (size_t)T_tokens * I;
    const unsigned blocks = (unsigned)std::min<size_t>((total + 255) / 256, 65535u * 16u);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(clamped_mul_kernel<float>, dim3(blocks), dim3(256), 0, st, (const float*)gu, ld_gu, (float*)out,
                           I, limit, slope, total);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(clamped_mul_kernel<bf16>, dim3(blocks), dim3(256), 0, st, (const bf16*)gu, ld_gu, (bf16*)out, I,
                           limit, slope, total);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}
