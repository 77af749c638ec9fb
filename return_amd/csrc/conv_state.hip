// Causal convolution over time on each channel, for requests that arrive in pieces: the last
// taps-1 inputs of every request are kept between steps in a tail [slots + 1, taps-1, C], so a
// row's result does not depend on how the request was cut into steps.
//
//   y_t[c] = sum_j w[c][j] * x_(t - taps + 1 + j)[c] + b[c]    (w's last column is the current row's; zeros
//                                                          before the request's first row; b null: no bias)
//   out_t  = act(y_t)  or  act(x_t + y_t)                 (flags: 1 adds the input, 2 applies SiLU)
//
// x: rows of ld_x elements of which C are read (a column slice of a wider projection is fine),
// out: rows of ld_out elements. Request s brings rows cu_q[s]..cu_q[s+1]-1 and owns tail row
// slot_ids[s]. All sums in 32-bit; the result and the tail are rounded to the storage type.
//
// Grid (segments of CONV_SEG rows, requests, chunks of 256 channels); a thread owns one channel
// and walks its segment's rows with the last taps-1 inputs in registers. Only a request's first
// segment reads the tail (CONV_SEG >= taps-1), and the same thread writes the new tail for its
// channel when it is done, so no other thread ever sees a tail half way.
#include "common.h"

#define CONV_SEG 16
#define CONV_MAX_TAPS 8

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(
    const T* __restrict__ x, long long ld_x, const float* __restrict__ w, T* __restrict__ tail,
    const int* __restrict__ cu_q, const int* __restrict__ slot_ids, T* __restrict__ out, long long ld_out,
    int C, int taps, int flags, const float* __restrict__ bias) {
    const int s = blockIdx.y;
    const int base = cu_q[s];
    const int q_len = cu_q[s + 1] - base;
    const int first = blockIdx.x * CONV_SEG;
    if (first >= q_len) return;
    const int c = blockIdx.z * 256 + threadIdx.x;
    if (c >= C) return;
    const int last = min(first + CONV_SEG, q_len);
    const int back = taps - 1;
    T* my_tail = tail + ((size_t)slot_ids[s] * back) * C + c;

    const float b0 = bias != nullptr ? bias[c] : 0.f;
    float wt[CONV_MAX_TAPS], win[CONV_MAX_TAPS], old[CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
        wt[j] = j < taps ? w[(size_t)c * taps + j] : 0.f;
        win[j] = old[j] = 0.f;
        if (j < back) {
            const int li = first - back + j;                 // the input that far back, among this step's rows or before
            win[j] = li >= 0 ? to_f(x[(size_t)(base + li) * ld_x + c]) : to_f(my_tail[(size_t)(back + li) * C]);
            old[j] = win[j];
        }
    }
    for (int li = first; li < last; ++li) {
        const float cur = to_f(x[(size_t)(base + li) * ld_x + c]);
        float y = b0;
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS - 1; ++j)
            if (j < back) y = fmaf(wt[j], win[j], y);
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS; ++j)
            if (j == back) y = fmaf(wt[j], cur, y);
        if (flags & 1) y += cur;
        if (flags & 2) y = y / (1.f + expf(-y));
        out[(size_t)(base + li) * ld_out + c] = from_f<T>(y);
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS - 1; ++j)
            if (j + 1 < back) win[j] = win[j + 1];
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS; ++j)
            if (j == back - 1) win[j] = cur;
    }
    if (first == 0) {
        // the new tail: the last taps-1 inputs of (old tail, this step's rows)
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS - 1; ++j) {
            if (j < back) {
                const int li = q_len - back + j;
                float v = 0.f;
                if (li >= 0) v = to_f(x[(size_t)(base + li) * ld_x + c]);
                else {
#pragma unroll
                    for (int k = 0; k < CONV_MAX_TAPS - 1; ++k)
                        if (k == back + li) v = old[k];
                }
                my_tail[(size_t)j * C] = from_f<T>(v);
            }
        }
    }
}

// x [T rows], w fp32 [C, taps], tail [slots, taps-1, C], out [T rows]; max_q_len: the longest request of the step.
static int causal_conv_run(const void* x, long long ld_x, const float* w, const float* bias, void* tail, const int* cu_q,
                           const int* slot_ids, void* out, long long ld_out, int n_seqs, int max_q_len,
                           int C, int taps, int flags, int dtype, void* stream) {
    if (n_seqs <= 0 || max_q_len <= 0) return RA_OK;
    if (taps < 1 || taps > CONV_MAX_TAPS || taps - 1 > CONV_SEG || C <= 0 || ld_x < C || ld_out < C) return RA_ERR_ARG;
    if (n_seqs > 65535 || (C + 255) / 256 > 65535) return RA_ERR_ARG;
    if (dtype != RA_DTYPE_F32 && dtype != RA_DTYPE_BF16) return RA_ERR_ARG;
    dim3 grid((max_q_len + CONV_SEG - 1) / CONV_SEG, n_seqs, (C + 255) / 256), block(256);
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(causal_conv_kernel<float>, grid, block, 0, (hipStream_t)stream, (const float*)x, ld_x, w,
                           (float*)tail, cu_q, slot_ids, (float*)out, ld_out, C, taps, flags, bias);
    else
        hipLaunchKernelGGL(causal_conv_kernel<bf16>, grid, block, 0, (hipStream_t)stream, (const bf16*)x, ld_x, w,
                           (bf16*)tail, cu_q, slot_ids, (bf16*)out, ld_out, C, taps, flags, bias);
    return ra_launch_status();
}

extern "C" int ra_causal_conv(const void* x, long long ld_x, const float* w, void* tail, const int* cu_q,
                              const int* slot_ids, void* out, long long ld_out, int n_seqs, int max_q_len,
                              int C, int taps, int flags, int dtype, void* stream) {
    return causal_conv_run(x, ld_x, w, nullptr, tail, cu_q, slot_ids, out, ld_out, n_seqs, max_q_len, C, taps, flags,
                           dtype, stream);
}

// the same with a bias per channel (fp32 [C]) added to the filter's sum before the activation
extern "C" int ra_causal_conv_bias(const void* x, long long ld_x, const float* w, const float* bias, void* tail,
                                   const int* cu_q, const int* slot_ids, void* out, long long ld_out, int n_seqs,
                                   int max_q_len, int C, int taps, int flags, int dtype, void* stream) {
    return causal_conv_run(x, ld_x, w, bias, tail, cu_q, slot_ids, out, ld_out, n_seqs, max_q_len, C, taps, flags,
                           dtype, stream);
}
