// Row-wise kernels around the residual stream of layers that have a norm behind each sublayer as well as in
// front of it, and whose stream is a weighted sum of all layers' results:
//   post_norm_add   h[r] += y[r] / sqrt(mean(y[r]^2) + eps) * w; optionally x[r] = h[r] / sqrt(mean(h[r]^2) + eps2) * w2,
//                   the norm in front of the next sublayer, in the same kernel. The normed y never leaves 32-bit.
//   depth_mix       out[r] = sum_{j < count} a[j] * results[j][r], terms in order, 32-bit; optionally the next
//                   layer's first norm of out as well.
//   heads_gate      out[t][h * Dv + d] = o[h][t][d] * sigmoid(gate[t][h]): the result of a product batched over
//                   heads, laid out token by token again, each head times its gate.
//   silu_mul_bias   out[t][i] = silu(gu[t][i] + b[i]) * (gu[t][I + i] + b[I + i])
// One workgroup per row; a row's elements stay in registers between the passes (up to 16 a thread, beyond that
// they are read again).
#include "common.h"
#include <algorithm>

#define SR_THREADS 256
#define SR_KEEP 16

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

extern "C" int ra_post_norm_add(float* h, const void* y, const float* w, float eps, const float* w2, float eps2,
                                void* x, int rows, int H, int dtype, void* stream) {
    if (rows <= 0) return RA_OK;
    if (H < 1 || (w2 != nullptr && x == nullptr)) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
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

#define DM_MAX_TERMS 256
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
