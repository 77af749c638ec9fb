// Row-wise kernels around the residual stream of layers that have a norm behind each sublayer as well as in
// front of it, and whose stream is a weighted sum of all layers' results:
//   post_norm_add   h[r] += y[r] / sqrt(mean(y[r]^2) + eps) * w; optionally x[r] = h[r] / sqrt(mean(h[r]^2) + eps2) * w2,
//                   the norm in front of the next sublayer, in the same kernel. The normed y never leaves 32-bit.
//   depth_mix       out[r] = sum_{j < count} a[j] * results[j][r], terms in order, 32-bit; optionally the next
//                   layer's first norm of out as well.
//   post_norm_mix   both in one pass over a row, for a layer whose last sublayer's norm is followed at once by the
//                   weighted sum: results[count-1][r] += rmsnorm(y[r]) w, then out[r] as depth_mix forms it (the terms
//                   in the same order, so the same bits as the two kernels one after the other).
//   heads_gate      out[t][h * Dv + d] = o[h][t][d] * sigmoid(gate[t][h]): the result of a product batched over
//                   heads, laid out token by token again, each head times its gate.
//   silu_mul_bias   out[t][i] = silu(gu[t][i] + b[i]) * (gu[t][I + i] + b[I + i])
// One workgroup per row; a row's elements stay in registers between the passes (up to 16 a thread, beyond that
// they are read again).
#include "common.h"
#include <algorithm>

#define SR_THREADS 256
#define SR_KEEP 16
#define DM_MAX_TERMS 256

template <typename T>
__global__ __launch_bounds__(SR_THREADS) void post_norm_add_kernel(float* __restrict__ h, const T* __restrict__ y,
                                                                   const float* __restrict__ w, float eps,
                                                                   const float* __restrict__ w2, float eps2,
                                                                   T* __restrict__ x, int H) {
    __shared__ float scratch[16];
    const size_t r = blockIdx.x;
    const T* yr = y + r * H;
    float* hr = h + r * H;
    const bool fits = H <= SR_THREADS * SR_KEEP;
    float v[SR_KEEP];
    float ss = 0.f;
    if (fits) {
        // everything the row needs is asked for at once: y, the stream and both weights (a read that waits for a
        // sum that waits for a read is what a short step's time goes to)
        float hv[SR_KEEP], wv[SR_KEEP], w2v[SR_KEEP];
#pragma unroll
        for (int i = 0; i < SR_KEEP; ++i) {
            const int c = threadIdx.x + i * SR_THREADS;
            const bool in = c < H;
            v[i] = in ? to_f(yr[c]) : 0.f;
            hv[i] = in ? hr[c] : 0.f;
            wv[i] = in ? w[c] : 0.f;
            w2v[i] = (in && w2 != nullptr) ? w2[c] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < SR_KEEP; ++i) ss = fmaf(v[i], v[i], ss);
        const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)H + eps);
        float ss2 = 0.f;
#pragma unroll
        for (int i = 0; i < SR_KEEP; ++i) {
            const int c = threadIdx.x + i * SR_THREADS;
            if (c < H) {
                v[i] = hv[i] + v[i] * rstd * wv[i];
                hr[c] = v[i];
                ss2 = fmaf(v[i], v[i], ss2);
            }
        }
        if (w2 == nullptr) return;                     // (the same for every thread of the workgroup)
        const float rstd2 = 1.0f / sqrtf(block_sum(ss2, scratch) / (float)H + eps2);
        T* xr = x + r * H;
#pragma unroll
        for (int i = 0; i < SR_KEEP; ++i) {
            const int c = threadIdx.x + i * SR_THREADS;
            if (c < H) xr[c] = from_f<T>(v[i] * rstd2 * w2v[i]);
        }
        return;
    }
    for (int c = threadIdx.x; c < H; c += SR_THREADS) {
        const float a = to_f(yr[c]);
        ss = fmaf(a, a, ss);
    }
    const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)H + eps);
    float ss2 = 0.f;
    for (int c = threadIdx.x; c < H; c += SR_THREADS) {
        const float a = hr[c] + to_f(yr[c]) * rstd * w[c];
        hr[c] = a;
        ss2 = fmaf(a, a, ss2);
    }
    if (w2 == nullptr) return;
    const float rstd2 = 1.0f / sqrtf(block_sum(ss2, scratch) / (float)H + eps2);
    T* xr = x + r * H;
    for (int c = threadIdx.x; c < H; c += SR_THREADS) xr[c] = from_f<T>(hr[c] * rstd2 * w2[c]);
}

// ---- rows of a multiple of four elements, at most SR_THREADS * 16: a thread holds SR_G groups of four neighbours
#define SR_G 4
__device__ __forceinline__ void sr_load4(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void sr_load4(const bf16* p, float (&v)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ __forceinline__ void sr_store4(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void sr_store4(bf16* p, const float (&v)[4]) {
    uint2 t;
    t.x = (uint32_t)from_f<bf16>(v[0]).x | ((uint32_t)from_f<bf16>(v[1]).x << 16);
    t.y = (uint32_t)from_f<bf16>(v[2]).x | ((uint32_t)from_f<bf16>(v[3]).x << 16);
    *reinterpret_cast<uint2*>(p) = t;
}

// post_norm_add and, with MIX, the weighted sum behind it (results, count, a, out as in post_norm_mix; h is then
// results[count - 1]). Every read of the row is asked for before the first sum.
template <typename T, bool MIX>
__global__ __launch_bounds__(SR_THREADS) void post_norm_vec_kernel(float* __restrict__ h, const T* __restrict__ y,
                                                                   const float* __restrict__ w, float eps,
                                                                   const float* __restrict__ w2, float eps2,
                                                                   T* __restrict__ x, int H, const float* __restrict__ results,
                                                                   long long stride, int count, const float* __restrict__ a,
                                                                   float* __restrict__ out) {
    __shared__ float scratch[16];
    __shared__ float a_s[DM_MAX_TERMS];
    if (MIX)
        for (int j = threadIdx.x; j < count; j += SR_THREADS) a_s[j] = a[j];
    const size_t r = blockIdx.x;
    const T* yr = y + r * H;
    float* hr = h + r * H;
    float v[SR_G][4], hv[SR_G][4], wv[SR_G][4], w2v[SR_G][4];
    float ss = 0.f;
#pragma unroll
    for (int g = 0; g < SR_G; ++g) {
        const int c = (threadIdx.x + g * SR_THREADS) * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[g][e] = hv[g][e] = wv[g][e] = w2v[g][e] = 0.f;
        if (c < H) {
            sr_load4(yr + c, v[g]);
            sr_load4(hr + c, hv[g]);
            sr_load4(w + c, wv[g]);
            if (w2 != nullptr) sr_load4(w2 + c, w2v[g]);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) ss = fmaf(v[g][e], v[g][e], ss);
    }
    float acc[SR_G][4];
    if (MIX) {
        __syncthreads();                               // a_s is there
        const float* src = results + r * H;
        // the older terms of the sum, in order (they do not wait for the norm)
#pragma unroll
        for (int g = 0; g < SR_G; ++g) {
            const int c = (threadIdx.x + g * SR_THREADS) * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[g][e] = 0.f;
            if (c < H) {
                for (int j = 0; j < count - 1; j += 4) {
                    float t[4][4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) sr_load4(src + (size_t)min(j + k, count - 2) * stride + c, t[k]);
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        if (j + k < count - 1) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[g][e] = fmaf(a_s[j + k], t[k][e], acc[g][e]);
                        }
                }
            }
        }
    }
    const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)H + eps);
    const float a_last = MIX ? a_s[count - 1] : 0.f;
    float ss2 = 0.f;
#pragma unroll
    for (int g = 0; g < SR_G; ++g) {
        const int c = (threadIdx.x + g * SR_THREADS) * 4;
        if (c < H) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[g][e] = hv[g][e] + v[g][e] * rstd * wv[g][e];
            sr_store4(hr + c, v[g]);
            if (MIX) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[g][e] = fmaf(a_last, v[g][e], acc[g][e]);
                sr_store4(out + r * H + c, v[g]);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) ss2 = fmaf(v[g][e], v[g][e], ss2);
        }
    }
    if (w2 == nullptr) return;                         // (the same for every thread of the workgroup)
    const float rstd2 = 1.0f / sqrtf(block_sum(ss2, scratch) / (float)H + eps2);
    T* xr = x + r * H;
#pragma unroll
    for (int g = 0; g < SR_G; ++g) {
        const int c = (threadIdx.x + g * SR_THREADS) * 4;
        if (c < H) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[g][e] = v[g][e] * rstd2 * w2v[g][e];
            sr_store4(xr + c, v[g]);
        }
    }
}

static bool sr_vec_ok(int H, const void* p0, const void* p1, const void* p2, const void* p3) {
    auto al = [](const void* p) { return p == nullptr || ((uintptr_t)p & 15) == 0; };
    return H % 4 == 0 && H <= SR_THREADS * 4 * SR_G && al(p0) && al(p1) && al(p2) && al(p3);
}

extern "C" int ra_post_norm_add(float* h, const void* y, const float* w, float eps, const float* w2, float eps2,
                                void* x, int rows, int H, int dtype, void* stream) {
    if (rows <= 0) return RA_OK;
    if (H < 1 || (w2 != nullptr && x == nullptr)) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (sr_vec_ok(H, h, y, w, w2) && sr_vec_ok(H, x, nullptr, nullptr, nullptr) && (dtype == RA_DTYPE_F32 || dtype == RA_DTYPE_BF16)) {
        if (dtype == RA_DTYPE_F32)
            hipLaunchKernelGGL((post_norm_vec_kernel<float, false>), dim3(rows), dim3(SR_THREADS), 0, st, h, (const float*)y, w,
                               eps, w2, eps2, (float*)x, H, nullptr, 0, 0, nullptr, nullptr);
        else
            hipLaunchKernelGGL((post_norm_vec_kernel<bf16, false>), dim3(rows), dim3(SR_THREADS), 0, st, h, (const bf16*)y, w,
                               eps, w2, eps2, (bf16*)x, H, nullptr, 0, 0, nullptr, nullptr);
        return ra_launch_status();
    }
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(post_norm_add_kernel<float>, dim3(rows), dim3(SR_THREADS), 0, st, h, (const float*)y, w, eps, w2,
                           eps2, (float*)x, H);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(post_norm_add_kernel<bf16>, dim3(rows), dim3(SR_THREADS), 0, st, h, (const bf16*)y, w, eps, w2,
                           eps2, (bf16*)x, H);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}

template <typename T>
__global__ __launch_bounds__(SR_THREADS) void depth_mix_kernel(const float* __restrict__ results, long long stride,
                                                               int count, const float* __restrict__ a,
                                                               float* __restrict__ out, const float* __restrict__ w2,
                                                               float eps2, T* __restrict__ x, int H) {
    __shared__ float scratch[16];
    __shared__ float a_s[DM_MAX_TERMS];
    for (int j = threadIdx.x; j < count; j += SR_THREADS) a_s[j] = a[j];
    __syncthreads();
    const size_t r = blockIdx.x;
    const float* src = results + r * H;
    float* dst = out + r * H;
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += SR_THREADS) {
        float acc = 0.f;
        int j = 0;
        for (; j + 8 <= count; j += 8) {               // eight terms asked for at once, added in order
            float t[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] = src[(size_t)(j + e) * stride + c];
#pragma unroll
            for (int e = 0; e < 8; ++e) acc = fmaf(a_s[j + e], t[e], acc);
        }
        {
            float t[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] = j + e < count ? src[(size_t)(j + e) * stride + c] : 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (j + e < count) acc = fmaf(a_s[j + e], t[e], acc);
        }
        dst[c] = acc;
        ss = fmaf(acc, acc, ss);
    }
    if (w2 == nullptr) return;
    const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)H + eps2);
    T* xr = x + r * H;
    for (int c = threadIdx.x; c < H; c += SR_THREADS) xr[c] = from_f<T>(dst[c] * rstd * w2[c]);   // (a thread reads what it wrote)
}

// results: fp32 [n][rows][H] with `stride` elements from one result to the next; out may be one of the later results
extern "C" int ra_depth_mix(const float* results, long long stride, int count, const float* a, float* out,
                            const float* w2, float eps2, void* x, int rows, int H, int dtype, void* stream) {
    if (rows <= 0) return RA_OK;
    if (H < 1 || count < 1 || count > DM_MAX_TERMS || (w2 != nullptr && x == nullptr)) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(depth_mix_kernel<float>, dim3(rows), dim3(SR_THREADS), 0, st, results, stride, count, a, out, w2,
                           eps2, (float*)x, H);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(depth_mix_kernel<bf16>, dim3(rows), dim3(SR_THREADS), 0, st, results, stride, count, a, out, w2,
                           eps2, (bf16*)x, H);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}

// rows of at most SR_THREADS * SR_KEEP elements
template <typename T>
__global__ __launch_bounds__(SR_THREADS) void post_norm_mix_kernel(float* __restrict__ results, long long stride, int count,
                                                                   const float* __restrict__ a, const T* __restrict__ y,
                                                                   const float* __restrict__ w, float eps,
                                                                   float* __restrict__ out, const float* __restrict__ w2,
                                                                   float eps2, T* __restrict__ x, int H) {
    __shared__ float scratch[16];
    __shared__ float a_s[DM_MAX_TERMS];
    for (int j = threadIdx.x; j < count; j += SR_THREADS) a_s[j] = a[j];
    const size_t r = blockIdx.x;
    const T* yr = y + r * H;
    float* hr = results + (size_t)(count - 1) * stride + r * H;     // the layer's result so far
    const float* src = results + r * H;
    // everything the row needs is asked for before the first sum: y, the result so far, the weights
    float v[SR_KEEP], hv[SR_KEEP], wv[SR_KEEP], w2v[SR_KEEP];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < SR_KEEP; ++i) {
        const int c = threadIdx.x + i * SR_THREADS;
        const bool in = c < H;
        v[i] = in ? to_f(yr[c]) : 0.f;
        hv[i] = in ? hr[c] : 0.f;
        wv[i] = in ? w[c] : 0.f;
        w2v[i] = (in && w2 != nullptr) ? w2[c] : 0.f;
        ss = fmaf(v[i], v[i], ss);
    }
    __syncthreads();                                   // a_s is there
    // the older terms of the sum, in order (they do not wait for the norm)
    float acc[SR_KEEP];
#pragma unroll
    for (int i = 0; i < SR_KEEP; ++i) {
        const int c = threadIdx.x + i * SR_THREADS;
        acc[i] = 0.f;
        if (c < H) {
            int j = 0;
            for (; j + 8 <= count - 1; j += 8) {
                float t[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) t[e] = src[(size_t)(j + e) * stride + c];
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[i] = fmaf(a_s[j + e], t[e], acc[i]);
            }
            float t[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] = j + e < count - 1 ? src[(size_t)(j + e) * stride + c] : 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (j + e < count - 1) acc[i] = fmaf(a_s[j + e], t[e], acc[i]);
        }
    }
    const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)H + eps);
    const float a_last = a_s[count - 1];
    float* dst = out + r * H;
    float ss2 = 0.f;
#pragma unroll
    for (int i = 0; i < SR_KEEP; ++i) {
        const int c = threadIdx.x + i * SR_THREADS;
        if (c < H) {
            const float hn = hv[i] + v[i] * rstd * wv[i];
            hr[c] = hn;
            acc[i] = fmaf(a_last, hn, acc[i]);
            dst[c] = acc[i];
            ss2 = fmaf(acc[i], acc[i], ss2);
        }
    }
    if (w2 == nullptr) return;
    const float rstd2 = 1.0f / sqrtf(block_sum(ss2, scratch) / (float)H + eps2);
    T* xr = x + r * H;
#pragma unroll
    for (int i = 0; i < SR_KEEP; ++i) {
        const int c = threadIdx.x + i * SR_THREADS;
        if (c < H) xr[c] = from_f<T>(acc[i] * rstd2 * w2v[i]);
    }
}

// results: fp32 [n][rows][H]; row count - 1 takes the post norm of y, out (a later row) the sum over the first count
extern "C" int ra_post_norm_mix(float* results, long long stride, int count, const float* a, const void* y, const float* w,
                                float eps, float* out, const float* w2, float eps2, void* x, int rows, int H, int dtype,
                                void* stream) {
    if (rows <= 0) return RA_OK;
    if (H < 1 || H > SR_THREADS * SR_KEEP || count < 1 || count > DM_MAX_TERMS || (w2 != nullptr && x == nullptr))
        return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (stride % 4 == 0 && sr_vec_ok(H, results, y, w, w2) && sr_vec_ok(H, x, out, nullptr, nullptr) &&
        (dtype == RA_DTYPE_F32 || dtype == RA_DTYPE_BF16)) {
        float* hh = results + (size_t)(count - 1) * stride;
        if (dtype == RA_DTYPE_F32)
            hipLaunchKernelGGL((post_norm_vec_kernel<float, true>), dim3(rows), dim3(SR_THREADS), 0, st, hh, (const float*)y, w,
                               eps, w2, eps2, (float*)x, H, results, stride, count, a, out);
        else
            hipLaunchKernelGGL((post_norm_vec_kernel<bf16, true>), dim3(rows), dim3(SR_THREADS), 0, st, hh, (const bf16*)y, w,
                               eps, w2, eps2, (bf16*)x, H, results, stride, count, a, out);
        return ra_launch_status();
    }
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(post_norm_mix_kernel<float>, dim3(rows), dim3(SR_THREADS), 0, st, results, stride, count, a,
                           (const float*)y, w, eps, out, w2, eps2, (float*)x, H);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(post_norm_mix_kernel<bf16>, dim3(rows), dim3(SR_THREADS), 0, st, results, stride, count, a,
                           (const bf16*)y, w, eps, out, w2, eps2, (bf16*)x, H);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}

template <typename T>
__global__ void heads_gate_kernel(const T* __restrict__ o, const T* __restrict__ gate, long long ld_gate,
                                  T* __restrict__ out, int T_tokens, int Hn, int Dv) {
    const size_t n = (size_t)T_tokens * Hn * Dv;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const size_t t = i / ((size_t)Hn * Dv);
        const int rem = (int)(i - t * Hn * Dv), hh = rem / Dv, d = rem - hh * Dv;
        float v = to_f(o[((size_t)hh * T_tokens + t) * Dv + d]);
        if (gate != nullptr) v *= 1.0f / (1.0f + expf(-to_f(gate[t * ld_gate + hh])));
        out[i] = from_f<T>(v);
    }
}

extern "C" int ra_heads_gate(const void* o, const void* gate, long long ld_gate, void* out, int T_tokens, int Hn, int Dv,
                             int dtype, void* stream) {
    if (T_tokens <= 0) return RA_OK;
    if (Hn < 1 || Dv < 1 || (gate != nullptr && ld_gate < Hn)) return RA_ERR_ARG;
    const size_t n = (size_t)T_tokens * Hn * Dv;
    const unsigned blocks = (unsigned)std::min<size_t>((n + 255) / 256, 65535u * 16u);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(heads_gate_kernel<float>, dim3(blocks), dim3(256), 0, st, (const float*)o, (const float*)gate,
                           ld_gate, (float*)out, T_tokens, Hn, Dv);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(heads_gate_kernel<bf16>, dim3(blocks), dim3(256), 0, st, (const bf16*)o, (const bf16*)gate,
                           ld_gate, (bf16*)out, T_tokens, Hn, Dv);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}

template <typename T>
__global__ void silu_mul_bias_kernel(const T* __restrict__ gu, const float* __restrict__ b, T* __restrict__ out, int I,
                                     size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t t = i / I;
        const int c = (int)(i - t * I);
        const float g = to_f(gu[t * 2 * I + c]) + b[c], u = to_f(gu[t * 2 * I + I + c]) + b[I + c];
        out[i] = from_f<T>(g / (1.0f + expf(-g)) * u);
    }
}

extern "C" int ra_silu_mul_bias(const void* gu, const float* b, void* out, int T_tokens, int I, int dtype, void* stream) {
    if (T_tokens <= 0) return RA_OK;
    if (I < 1 || b == nullptr) return RA_ERR_ARG;
    const size_t total = (size_t)T_tokens * I;
    const unsigned blocks = (unsigned)std::min<size_t>((total + 255) / 256, 65535u * 16u);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(silu_mul_bias_kernel<float>, dim3(blocks), dim3(256), 0, st, (const float*)gu, b, (float*)out, I,
                           total);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(silu_mul_bias_kernel<bf16>, dim3(blocks), dim3(256), 0, st, (const bf16*)gu, b, (bf16*)out, I,
                           total);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}
