// Bias of a butterfly layer: output = multiply(...) + bias, and d_bias = sum of grad over the batch.
//
// The forward kernels that write the final output add the bias themselves (one register per
// element a thread owns, loaded once); bias_add_kernel is the fallback for schedules whose
// last pass runs in a kernel without that hook.  The bias gradient is a column sum of the
// output gradient: row partitions first (each thread adds its rows in ascending order), then
// the partitions in ascending order -- no atomics, so it is bitwise reproducible.
#pragma once

#include "common.hpp"

namespace bf {

constexpr int kBiasThreads = 256;

struct BiasArgs {
    const void *bias;      // (S, width) dense
    void *out;             // forward fallback: output, updated in place
    const void *grad;      // gradient: (B, S, width) through `view`
    void *partial;         // (nparts, S, width)
    void *d_bias;          // (S, width) dense
    View view;
    int64_t batch;
    int64_t width;         // columns that exist (output_size)
    int64_t rows_per_part;
    int64_t nparts;
};

// grid: (ceil(width / kBiasThreads), S, row partitions)
template <typename T>
__global__ __launch_bounds__(kBiasThreads) void bias_add_kernel(BiasArgs a)
{
    const int64_t col = (int64_t)blockIdx.x * kBiasThreads + threadIdx.x;
    const int stack = blockIdx.y;
    if (col >= a.width) return;
    const int64_t vc = view_col(a.view, col);
    if (vc < 0) return;
    const T b = reinterpret_cast<const T *>(a.bias)[stack * a.width + col];
    T *out = reinterpret_cast<T *>(a.out) + stack * a.view.ss + vc * a.view.se;
    const int64_t r0 = (int64_t)blockIdx.z * a.rows_per_part;
    const int64_t r1 = r0 + a.rows_per_part < a.batch ? r0 + a.rows_per_part : a.batch;
    for (int64_t r = r0; r < r1; ++r) out[r * a.view.sb] = add(out[r * a.view.sb], b);
}

template <typename T>
__global__ __launch_bounds__(kBiasThreads) void bias_grad_partial_kernel(BiasArgs a)
{
    const int64_t col = (int64_t)blockIdx.x * kBiasThreads + threadIdx.x;
    const int stack = blockIdx.y;
    if (col >= a.width) return;
    const int64_t vc = view_col(a.view, col);
    const T *g = reinterpret_cast<const T *>(a.grad) + stack * a.view.ss + (vc < 0 ? 0 : vc) * a.view.se;
    const int64_t r0 = (int64_t)blockIdx.z * a.rows_per_part;
    const int64_t r1 = vc < 0 ? r0 : (r0 + a.rows_per_part < a.batch ? r0 + a.rows_per_part : a.batch);
    // four running sums keep four loads in flight; they are combined in a fixed order
    T s0 = zero_of(T()), s1 = s0, s2 = s0, s3 = s0;
    int64_t r = r0;
    for (; r + 4 <= r1; r += 4) {
        s0 = add(s0, g[r * a.view.sb]);
        s1 = add(s1, g[(r + 1) * a.view.sb]);
        s2 = add(s2, g[(r + 2) * a.view.sb]);
        s3 = add(s3, g[(r + 3) * a.view.sb]);
    }
    for (; r < r1; ++r) s0 = add(s0, g[r * a.view.sb]);
    reinterpret_cast<T *>(a.partial)[((int64_t)blockIdx.z * gridDim.y + stack) * a.width + col] =
        add(add(s0, s1), add(s2, s3));
}

// grid: (ceil(width / kBiasThreads), S)
template <typename T>
__global__ __launch_bounds__(kBiasThreads) void bias_grad_final_kernel(BiasArgs a)
{
    const int64_t col = (int64_t)blockIdx.x * kBiasThreads + threadIdx.x;
    const int stack = blockIdx.y;
    if (col >= a.width) return;
    const T *part = reinterpret_cast<const T *>(a.partial) + stack * a.width + col;
    T s = zero_of(T());
    for (int64_t k = 0; k < a.nparts; ++k) s = add(s, part[k * gridDim.y * a.width]);
    reinterpret_cast<T *>(a.d_bias)[stack * a.width + col] = s;
}

}  // namespace bf
