// Diagonal matrices directly in front of and behind a butterfly product, folded into its factors:
//   diag(out_scale) B diag(in_scale) = the product of the same factors with the columns of the
//   first applied factor scaled by in_scale and the rows of the last applied one by out_scale.
// A few thousand multiplications on the factors instead of two elementwise passes over the
// activations (and, backward, four more plus two column sums).  in_scale has up to n entries
// (every stack reads the same input), out_scale up to stacks * n (the stacks' outputs side by
// side); entries past their lengths count as 1.
//
// Gradients follow PyTorch's convention for complex values (the gradient of a product with
// respect to one operand carries the conjugate of the other); every sum runs in a fixed order.
#pragma once

#include "common.hpp"

namespace bf {

constexpr int kScaleThreads = 256;

struct ScaleArgs {
    const void *tw;         // (S, NS, n/2, 2, 2) dense, stages in order of application
    const void *in_scale;   // in_len entries, or null
    const void *out_scale;  // out_len entries, or null
    const void *grad;       // backward: gradient with respect to the scaled factors
    void *out;              // forward: the scaled factors; backward: d_tw
    void *d_in;             // backward: in_len entries
    void *d_out;            // backward: out_len entries
    int64_t in_len, out_len;
    int nstacks, nstages, log_n;
    int first_log_stride;   // log2 of the stride of the first / last applied stage
    int last_log_stride;
};

// element that sits at position pos (0 / 1) of pair p of a stage of stride 2^sl, and back
__device__ __forceinline__ int pair_element(int p, int pos, int sl)
{
    return ((p >> sl) << (sl + 1)) | (pos << sl) | (p & ((1 << sl) - 1));
}
__device__ __forceinline__ int element_pair(int e, int sl) { return ((e >> (sl + 1)) << sl) | (e & ((1 << sl) - 1)); }

template <typename T>
__device__ __forceinline__ T one_of();
template <>
__device__ __forceinline__ float one_of<float>() { return 1.0f; }
template <>
__device__ __forceinline__ float2 one_of<float2>() { return make_float2(1.0f, 0.0f); }

// factor that entry (stack s, stage t, pair p, row r, column c) of the product takes
template <typename T>
__device__ __forceinline__ T scale_in_factor(const ScaleArgs &a, int t, int p, int c)
{
    if (t != 0 || a.in_scale == nullptr) return one_of<T>();
    const int e = pair_element(p, c, a.first_log_stride);
    return e < a.in_len ? reinterpret_cast<const T *>(a.in_scale)[e] : one_of<T>();
}
template <typename T>
__device__ __forceinline__ T scale_out_factor(const ScaleArgs &a, int s, int t, int p, int r)
{
    if (t != a.nstages - 1 || a.out_scale == nullptr) return one_of<T>();
    const int64_t e = ((int64_t)s << a.log_n) + pair_element(p, r, a.last_log_stride);
    return e < a.out_len ? reinterpret_cast<const T *>(a.out_scale)[e] : one_of<T>();
}

// grid: ceil(S * NS * 2n / kScaleThreads); one factor entry per thread
template <typename T, bool BACKWARD>
__global__ __launch_bounds__(kScaleThreads) void scale_twiddle_kernel(ScaleArgs a)
{
    const int64_t idx = (int64_t)blockIdx.x * kScaleThreads + threadIdx.x;
    const int half_log = a.log_n - 1;
    const int64_t total = ((int64_t)a.nstacks * a.nstages) << (half_log + 2);
    if (idx >= total) return;
    const int c = (int)(idx & 1), r = (int)((idx >> 1) & 1);
    const int p = (int)((idx >> 2) & ((1 << half_log) - 1));
    const int64_t st = idx >> (half_log + 2);
    const int t = (int)(st % a.nstages), s = (int)(st / a.nstages);
    const T f = mul(scale_in_factor<T>(a, t, p, c), scale_out_factor<T>(a, s, t, p, r));
    if constexpr (BACKWARD)
        reinterpret_cast<T *>(a.out)[idx] = mul(reinterpret_cast<const T *>(a.grad)[idx], conj_of(f));
    else
        reinterpret_cast<T *>(a.out)[idx] = mul(reinterpret_cast<const T *>(a.tw)[idx], f);
}

// grid: ceil((in_len + out_len) / kScaleThreads); one diagonal entry per thread:
//   d_in[e]  = sum over stacks s and rows r of grad[s][0][p][r][c] conj(tw[s][0][p][r][c] * out factor)
//   d_out[j] = sum over columns c of grad[s][last][p][r][c] conj(tw[s][last][p][r][c] * in factor)
template <typename T>
__global__ __launch_bounds__(kScaleThreads) void scale_twiddle_grad_kernel(ScaleArgs a)
{
    const int64_t idx = (int64_t)blockIdx.x * kScaleThreads + threadIdx.x;
    const int half_log = a.log_n - 1;
    const T *tw = reinterpret_cast<const T *>(a.tw);
    const T *g = reinterpret_cast<const T *>(a.grad);
    const int64_t n_in = a.in_scale != nullptr ? a.in_len : 0;
    const int64_t n_out = a.out_scale != nullptr ? a.out_len : 0;
    if (idx < n_in) {
        const int e = (int)idx;
        const int c = (e >> a.first_log_stride) & 1, p = element_pair(e, a.first_log_stride);
        T sum = zero_of(T());
        for (int s = 0; s < a.nstacks; ++s) {
            for (int r = 0; r < 2; ++r) {
                const int64_t at = ((((int64_t)s * a.nstages) << half_log) + p) * 4 + r * 2 + c;
                sum = macc(sum, mul(tw[at], scale_out_factor<T>(a, s, 0, p, r)), g[at]);
            }
        }
        reinterpret_cast<T *>(a.d_in)[e] = sum;
    } else if (idx < n_in + n_out) {
        const int64_t j = idx - n_in;
        const int s = (int)(j >> a.log_n), e = (int)(j & ((1 << a.log_n) - 1));
        const int t = a.nstages - 1;
        const int r = (e >> a.last_log_stride) & 1, p = element_pair(e, a.last_log_stride);
        T sum = zero_of(T());
        for (int c = 0; c < 2; ++c) {
            const int64_t at = (((((int64_t)s * a.nstages + t)) << half_log) + p) * 4 + r * 2 + c;
            sum = macc(sum, mul(tw[at], scale_in_factor<T>(a, t, p, c)), g[at]);
        }
        reinterpret_cast<T *>(a.d_out)[j] = sum;
    }
}

}  // namespace bf
