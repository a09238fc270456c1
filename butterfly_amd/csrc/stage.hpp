// One stage of a base-4 product per launch, for the stages of long rows that couple elements
// further apart than a register-resident chunk reaches (rows beyond 1024 in float, beyond 256 in
// complex64): a radix-4 stage on the bit pair (b, b + 1), or the 2x2 stage that ends a block of
// odd log_n, at any stride.
//
// Twiddle-stationary like the other kernels: thread q of a workgroup owns group q of the stage
// (a quad or a pair of elements `stride` apart), keeps that group's factor (and, backward, its
// d_twiddle sums) in registers for the whole launch, and walks the rows of its workgroup.  Rows
// are read once and written once; consecutive threads own consecutive groups, so accesses are
// coalesced over runs of `stride` elements.  The d_twiddle sums leave as one partial slice per
// workgroup, in the layout of the twiddle tensor, for the fixed-order reduce.
#pragma once

#include "common.hpp"

namespace bf {

constexpr int kStageThreads = 256;
constexpr int kStageRows = 2;   // rows a thread has in flight

struct StageArgs {
    const void *tw;            // this stage's factors, stack 0: (n / RADIX, RADIX, RADIX)
    int64_t tw_stack_stride;   // scalars
    int log_stride;
    int64_t n;
    const void *x_in;
    View x_view;
    void *x_out;               // forward
    View xo_view;
    const void *g_out;         // backward
    View g_view;
    void *g_in;
    View gi_view;
    void *partial;             // (gridDim.x, S, slot) scalars
    int64_t slot;
    int64_t batch;
    int64_t rows_per_wg;
};

// columns of the RADIX elements of group q
template <int RADIX>
__device__ __forceinline__ void stage_columns(int64_t q, int log_stride, int64_t (&col)[RADIX])
{
    const int64_t st = (int64_t)1 << log_stride;
    const int64_t low = q & (st - 1);
    const int64_t pos = RADIX * (q - low) + low;
#pragma unroll
    for (int c = 0; c < RADIX; ++c) col[c] = pos + c * st;
}

template <typename T, int RADIX>
__global__ __launch_bounds__(kStageThreads) void stage_fw_kernel(StageArgs a)
{
    const int64_t q = (int64_t)blockIdx.z * kStageThreads + threadIdx.x;
    if (q >= a.n / RADIX) return;
    const int stack = blockIdx.y;
    const T *F = reinterpret_cast<const T *>(a.tw) + stack * a.tw_stack_stride + q * (RADIX * RADIX);
    T f[RADIX][RADIX];
#pragma unroll
    for (int r = 0; r < RADIX; ++r)
#pragma unroll
        for (int c = 0; c < RADIX; ++c) f[r][c] = F[r * RADIX + c];
    int64_t col[RADIX], in_off[RADIX], out_off[RADIX];
    stage_columns<RADIX>(q, a.log_stride, col);
#pragma unroll
    for (int c = 0; c < RADIX; ++c) {
        const int64_t ic = view_col(a.x_view, col[c]), oc = view_col(a.xo_view, col[c]);
        in_off[c] = ic >= 0 ? ic * a.x_view.se : -1;
        out_off[c] = oc >= 0 ? oc * a.xo_view.se : -1;
    }
    const T *xin = reinterpret_cast<const T *>(a.x_in) + stack * a.x_view.ss;
    T *xout = reinterpret_cast<T *>(a.x_out) + stack * a.xo_view.ss;
    const int64_t b0 = (int64_t)blockIdx.x * a.rows_per_wg;
    const int64_t b1 = b0 + a.rows_per_wg < a.batch ? b0 + a.rows_per_wg : a.batch;
    for (int64_t b = b0; b < b1; b += kStageRows) {
        T x[kStageRows][RADIX];
#pragma unroll
        for (int k = 0; k < kStageRows; ++k)
#pragma unroll
            for (int c = 0; c < RADIX; ++c)
                x[k][c] = (b + k < b1 && in_off[c] >= 0) ? xin[(b + k) * a.x_view.sb + in_off[c]] : zero_of(T());
#pragma unroll
        for (int k = 0; k < kStageRows; ++k) {
            if (b + k >= b1) break;
#pragma unroll
            for (int r = 0; r < RADIX; ++r) {
                T y = mul(f[r][0], x[k][0]);
#pragma unroll
                for (int c = 1; c < RADIX; ++c) y = mac(y, f[r][c], x[k][c]);
                if (out_off[r] >= 0) xout[(b + k) * a.xo_view.sb + out_off[r]] = y;
            }
        }
    }
}

template <typename T, int RADIX>
__global__ __launch_bounds__(kStageThreads) void stage_bw_kernel(StageArgs a)
{
    const int64_t q = (int64_t)blockIdx.z * kStageThreads + threadIdx.x;
    if (q >= a.n / RADIX) return;
    const int stack = blockIdx.y;
    const T *F = reinterpret_cast<const T *>(a.tw) + stack * a.tw_stack_stride + q * (RADIX * RADIX);
    T f[RADIX][RADIX], acc[RADIX][RADIX];
#pragma unroll
    for (int r = 0; r < RADIX; ++r)
#pragma unroll
        for (int c = 0; c < RADIX; ++c) {
            f[r][c] = F[r * RADIX + c];
            acc[r][c] = zero_of(T());
        }
    int64_t col[RADIX], x_off[RADIX], g_off[RADIX], gi_off[RADIX];
    stage_columns<RADIX>(q, a.log_stride, col);
#pragma unroll
    for (int c = 0; c < RADIX; ++c) {
        const int64_t xc = view_col(a.x_view, col[c]), gc = view_col(a.g_view, col[c]), ic = view_col(a.gi_view, col[c]);
        x_off[c] = xc >= 0 ? xc * a.x_view.se : -1;
        g_off[c] = gc >= 0 ? gc * a.g_view.se : -1;
        gi_off[c] = ic >= 0 ? ic * a.gi_view.se : -1;
    }
    const T *xin = reinterpret_cast<const T *>(a.x_in) + stack * a.x_view.ss;
    const T *gout = reinterpret_cast<const T *>(a.g_out) + stack * a.g_view.ss;
    T *gin = reinterpret_cast<T *>(a.g_in) + stack * a.gi_view.ss;
    const int64_t b0 = (int64_t)blockIdx.x * a.rows_per_wg;
    const int64_t b1 = b0 + a.rows_per_wg < a.batch ? b0 + a.rows_per_wg : a.batch;
    // rows in ascending order: the sums of a workgroup are reproducible
    for (int64_t b = b0; b < b1; b += kStageRows) {
        T x[kStageRows][RADIX], g[kStageRows][RADIX];
#pragma unroll
        for (int k = 0; k < kStageRows; ++k)
#pragma unroll
            for (int c = 0; c < RADIX; ++c) {
                const bool row = b + k < b1;
                x[k][c] = (row && x_off[c] >= 0) ? xin[(b + k) * a.x_view.sb + x_off[c]] : zero_of(T());
                g[k][c] = (row && g_off[c] >= 0) ? gout[(b + k) * a.g_view.sb + g_off[c]] : zero_of(T());
            }
#pragma unroll
        for (int k = 0; k < kStageRows; ++k) {
            if (b + k >= b1) break;
#pragma unroll
            for (int r = 0; r < RADIX; ++r)
#pragma unroll
                for (int c = 0; c < RADIX; ++c) acc[r][c] = macc(acc[r][c], x[k][c], g[k][r]);   // g_r conj(x_c)
#pragma unroll
            for (int c = 0; c < RADIX; ++c) {
                T d = mul(conj_of(f[0][c]), g[k][0]);
#pragma unroll
                for (int r = 1; r < RADIX; ++r) d = macc(d, f[r][c], g[k][r]);
                if (gi_off[c] >= 0) gin[(b + k) * a.gi_view.sb + gi_off[c]] = d;
            }
        }
    }
    T *part = reinterpret_cast<T *>(a.partial) + ((int64_t)blockIdx.x * gridDim.y + stack) * a.slot + q * (RADIX * RADIX);
#pragma unroll
    for (int r = 0; r < RADIX; ++r)
#pragma unroll
        for (int c = 0; c < RADIX; ++c) part[r * RADIX + c] = acc[r][c];
}

}  // namespace bf
