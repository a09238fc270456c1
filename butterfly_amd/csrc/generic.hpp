// General-shape kernels: any log_n whose rows fit in LDS, any nblocks, base-2 and base-4,
// float and complex64, arbitrary operand strides.  One workgroup keeps whole rows in LDS
// and walks a range [t0, t1) of the flat stage list, so a long schedule can be cut into
// several launches when the backward pass cannot hold every stage input at once.
#pragma once

#include "common.hpp"

namespace bf {

constexpr int kGenericThreads = 256;

struct GenericFwArgs {
    Schedule sc;
    int t0, t1;           // stage range
    int rows_per_wg;      // rows staged in LDS together
    int64_t batch;
    const void *tw2;      // 2x2 factors
    const void *tw4;      // 4x4 factors (base-4 only)
    const void *in;
    View in_view;
    void *out;
    View out_view;
};

// One 2x2 stage on R rows held in LDS at buf[r * n + j].
template <typename T>
__device__ __forceinline__ void lds_stage2(T *buf, const T *tw, int log_n, int log_stride,
                                           int rows, int tid)
{
    const int half = 1 << (log_n - 1);
    const int st = 1 << log_stride;
    const int items = rows << (log_n - 1);
    for (int it = tid; it < items; it += kGenericThreads) {
        const int r = it >> (log_n - 1);
        const int p = it & (half - 1);
        const int low = p & (st - 1);
        const int pos = ((p - low) << 1) + low;
        const T t00 = tw[4 * p + 0], t01 = tw[4 * p + 1], t10 = tw[4 * p + 2], t11 = tw[4 * p + 3];
        T *row = buf + ((int64_t)r << log_n);
        const T x0 = row[pos], x1 = row[pos + st];
        row[pos] = mac(mul(t00, x0), t01, x1);
        row[pos + st] = mac(mul(t10, x0), t11, x1);
    }
}

// One 4x4 stage on R rows held in LDS.
template <typename T>
__device__ __forceinline__ void lds_stage4(T *buf, const T *tw, int log_n, int log_stride,
                                           int rows, int tid)
{
    const int quarter = 1 << (log_n - 2);
    const int st = 1 << log_stride;
    const int items = rows << (log_n - 2);
    for (int it = tid; it < items; it += kGenericThreads) {
        const int r = it >> (log_n - 2);
        const int q = it & (quarter - 1);
        const int low = q & (st - 1);
        const int pos = ((q - low) << 2) + low;
        T *row = buf + ((int64_t)r << log_n);
        T x[4], y[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) x[c] = row[pos + c * st];
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            T acc = mul(tw[16 * q + 4 * rr], x[0]);
#pragma unroll
            for (int c = 1; c < 4; ++c) acc = mac(acc, tw[16 * q + 4 * rr + c], x[c]);
            y[rr] = acc;
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) row[pos + c * st] = y[c];
    }
}

template <typename T>
__global__ __launch_bounds__(kGenericThreads) void generic_fw_kernel(GenericFwArgs a)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *buf = reinterpret_cast<T *>(smem_raw);
    const int tid = threadIdx.x;
    const int s = blockIdx.y;
    const int log_n = a.sc.log_n;
    const int n = 1 << log_n;
    const int64_t b0 = (int64_t)blockIdx.x * a.rows_per_wg;
    int rows = a.rows_per_wg;
    if (b0 + rows > a.batch) rows = (int)(a.batch - b0);

    const T *in = reinterpret_cast<const T *>(a.in);
    for (int it = tid; it < (rows << log_n); it += kGenericThreads) {
        const int r = it >> log_n, j = it & (n - 1);
        T v = zero_of(T());
        const int64_t jc = view_col(a.in_view, j);
        if (jc >= 0) v = in[(b0 + r) * a.in_view.sb + s * a.in_view.ss + jc * a.in_view.se];
        buf[it] = v;
    }
    for (int t = a.t0; t < a.t1; ++t) {
        __syncthreads();
        const StageInfo si = stage_info(a.sc, t);
        if (si.radix4) {
            const T *tw = reinterpret_cast<const T *>(a.tw4) + s * a.sc.tw4_stack_stride + si.tw_off;
            lds_stage4<T>(buf, tw, log_n, si.log_stride, rows, tid);
        } else {
            const T *tw = reinterpret_cast<const T *>(a.tw2) + s * a.sc.tw2_stack_stride + si.tw_off;
            lds_stage2<T>(buf, tw, log_n, si.log_stride, rows, tid);
        }
    }
    __syncthreads();
    T *out = reinterpret_cast<T *>(a.out);
    for (int it = tid; it < (rows << log_n); it += kGenericThreads) {
        const int r = it >> log_n, j = it & (n - 1);
        const int64_t jc = view_col(a.out_view, j);
        if (jc >= 0) out[(b0 + r) * a.out_view.sb + s * a.out_view.ss + jc * a.out_view.se] = buf[it];
    }
}

struct GenericBwArgs {
    Schedule sc;
    int t0, t1;            // stage range of this launch
    int64_t batch;
    const void *tw2;
    const void *tw4;
    const void *x_in;      // input of stage t0
    View x_view;
    const void *g_out;     // gradient w.r.t. the output of stage t1 - 1
    View g_view;
    void *g_in;            // gradient w.r.t. the input of stage t0
    View gi_view;          // columns in [n, width) are zero-filled
    void *partial;         // (gridDim.x, S, t1 - t0, slot) per-workgroup d_twiddle sums
    int64_t slot;          // scalars reserved per stage in `partial`
};

// Persistent workgroups: workgroup w handles rows w, w + G, ...; the d_twiddle sum of
// those rows lives in a private slice of `partial`, each entry touched by one fixed
// thread, in ascending row order -- no atomics, reproducible.
template <typename T>
__global__ __launch_bounds__(kGenericThreads) void generic_bw_kernel(GenericBwArgs a)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int tid = threadIdx.x;
    const int s = blockIdx.y;
    const int log_n = a.sc.log_n;
    const int n = 1 << log_n;
    const int nst = a.t1 - a.t0;
    T *xs = reinterpret_cast<T *>(smem_raw);  // nst planes of n: input of each stage
    T *g = xs + ((int64_t)nst << log_n);      // running gradient
    const T *x_in = reinterpret_cast<const T *>(a.x_in);
    const T *g_out = reinterpret_cast<const T *>(a.g_out);
    T *g_in = reinterpret_cast<T *>(a.g_in);
    T *part = reinterpret_cast<T *>(a.partial) +
              ((int64_t)blockIdx.x * gridDim.y + s) * nst * a.slot;

    bool first_row = true;
    for (int64_t b = blockIdx.x; b < a.batch; b += gridDim.x) {
        for (int j = tid; j < n; j += kGenericThreads) {
            T v = zero_of(T()), gv = zero_of(T());
            const int64_t xc = view_col(a.x_view, j), gc = view_col(a.g_view, j);
            if (xc >= 0) v = x_in[b * a.x_view.sb + s * a.x_view.ss + xc * a.x_view.se];
            if (gc >= 0) gv = g_out[b * a.g_view.sb + s * a.g_view.ss + gc * a.g_view.se];
            xs[j] = v;
            g[j] = gv;
        }
        // forward replay: plane k + 1 = stage (t0 + k) applied to plane k
        for (int k = 0; k + 1 < nst; ++k) {
            __syncthreads();
            const StageInfo si = stage_info(a.sc, a.t0 + k);
            const T *src = xs + ((int64_t)k << log_n);
            T *dst = xs + ((int64_t)(k + 1) << log_n);
            const int st = 1 << si.log_stride;
            if (si.radix4) {
                const T *tw = reinterpret_cast<const T *>(a.tw4) + s * a.sc.tw4_stack_stride + si.tw_off;
                for (int q = tid; q < (n >> 2); q += kGenericThreads) {
                    const int low = q & (st - 1);
                    const int pos = ((q - low) << 2) + low;
                    T x[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) x[c] = src[pos + c * st];
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) {
                        T acc = mul(tw[16 * q + 4 * rr], x[0]);
#pragma unroll
                        for (int c = 1; c < 4; ++c) acc = mac(acc, tw[16 * q + 4 * rr + c], x[c]);
                        dst[pos + rr * st] = acc;
                    }
                }
            } else {
                const T *tw = reinterpret_cast<const T *>(a.tw2) + s * a.sc.tw2_stack_stride + si.tw_off;
                for (int p = tid; p < (n >> 1); p += kGenericThreads) {
                    const int low = p & (st - 1);
                    const int pos = ((p - low) << 1) + low;
                    const T x0 = src[pos], x1 = src[pos + st];
                    dst[pos] = mac(mul(tw[4 * p + 0], x0), tw[4 * p + 1], x1);
                    dst[pos + st] = mac(mul(tw[4 * p + 2], x0), tw[4 * p + 3], x1);
                }
            }
        }
        // reverse sweep
        for (int k = nst - 1; k >= 0; --k) {
            __syncthreads();
            const StageInfo si = stage_info(a.sc, a.t0 + k);
            const T *x = xs + ((int64_t)k << log_n);
            T *pk = part + (int64_t)k * a.slot;
            const int st = 1 << si.log_stride;
            if (si.radix4) {
                const T *tw = reinterpret_cast<const T *>(a.tw4) + s * a.sc.tw4_stack_stride + si.tw_off;
                for (int q = tid; q < (n >> 2); q += kGenericThreads) {
                    const int low = q & (st - 1);
                    const int pos = ((q - low) << 2) + low;
                    T gv[4], xv[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) { gv[c] = g[pos + c * st]; xv[c] = x[pos + c * st]; }
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        T acc = mul(conj_of(tw[16 * q + c]), gv[0]);
#pragma unroll
                        for (int rr = 1; rr < 4; ++rr) acc = macc(acc, tw[16 * q + 4 * rr + c], gv[rr]);
                        g[pos + c * st] = acc;
                    }
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr)
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            const T old = first_row ? zero_of(T()) : pk[16 * q + 4 * rr + c];
                            pk[16 * q + 4 * rr + c] = macc(old, xv[c], gv[rr]);
                        }
                }
            } else {
                const T *tw = reinterpret_cast<const T *>(a.tw2) + s * a.sc.tw2_stack_stride + si.tw_off;
                for (int p = tid; p < (n >> 1); p += kGenericThreads) {
                    const int low = p & (st - 1);
                    const int pos = ((p - low) << 1) + low;
                    const T g0 = g[pos], g1 = g[pos + st];
                    const T x0 = x[pos], x1 = x[pos + st];
                    g[pos] = macc(mul(conj_of(tw[4 * p + 0]), g0), tw[4 * p + 2], g1);
                    g[pos + st] = macc(mul(conj_of(tw[4 * p + 1]), g0), tw[4 * p + 3], g1);
                    T o0 = zero_of(T()), o1 = o0, o2 = o0, o3 = o0;
                    if (!first_row) { o0 = pk[4 * p + 0]; o1 = pk[4 * p + 1]; o2 = pk[4 * p + 2]; o3 = pk[4 * p + 3]; }
                    pk[4 * p + 0] = macc(o0, x0, g0);
                    pk[4 * p + 1] = macc(o1, x1, g0);
                    pk[4 * p + 2] = macc(o2, x0, g1);
                    pk[4 * p + 3] = macc(o3, x1, g1);
                }
            }
        }
        __syncthreads();
        const int64_t jend = a.gi_view.width > n ? a.gi_view.width : n;
        for (int64_t j = tid; j < jend; j += kGenericThreads) {
            const int64_t jc = j < n ? view_col(a.gi_view, j) : j;
            if (jc >= 0) g_in[b * a.gi_view.sb + s * a.gi_view.ss + jc * a.gi_view.se] = j < n ? g[j] : zero_of(T());
        }
        __syncthreads();
        first_row = false;
    }
}

struct ReduceArgs {
    Schedule sc;
    int t0, t1;
    int nparts;        // number of per-workgroup partial slices
    int elem_floats;   // 1 for float, 2 for complex64
    int64_t nstacks;
    const float *partial;
    int64_t slot;      // scalars reserved per stage in `partial`
    float *d_tw2;
    float *d_tw4;
};

// d_twiddle[s][stage][j] = sum over partial slices.  Works on raw floats (a complex sum is
// two float sums).  A workgroup covers 64 consecutive floats: thread (q, j4) adds the slices
// of group q (a contiguous sixteenth of them, ascending) for the float4 at j4; the sixteen
// group sums are then added in ascending q.  The order is fixed by nparts alone, so results
// are reproducible run to run.
// grid: (ceil(slot * elem_floats / 64), t1 - t0, S), block 256.
__global__ __launch_bounds__(256) void reduce_partials_kernel(ReduceArgs a)
{
    __shared__ float4 sm[16][16];
    const int j4 = threadIdx.x & 15, q = threadIdx.x >> 4;
    const int k = blockIdx.y;
    const int s = blockIdx.z;
    const int nst = a.t1 - a.t0;
    const StageInfo si = stage_info(a.sc, a.t0 + k);
    const int64_t n = (int64_t)1 << a.sc.log_n;
    const int64_t ef = a.elem_floats;
    const int64_t count = (si.radix4 ? 4 * n : 2 * n) * ef;   // floats in this stage
    const int64_t f = (int64_t)blockIdx.x * 64 + j4 * 4;
    const int64_t slot_f = a.slot * ef;
    const int64_t wg_stride = a.nstacks * nst * slot_f;
    const int chunk = (a.nparts + 15) / 16;
    const int w0 = q * chunk;
    const int w1 = w0 + chunk < a.nparts ? w0 + chunk : a.nparts;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (f < count) {
        const float *src = a.partial + ((int64_t)s * nst + k) * slot_f + f;
#pragma unroll 8
        for (int w = w0; w < w1; ++w) {
            const float4 v = *reinterpret_cast<const float4 *>(src + (int64_t)w * wg_stride);
            acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
        }
    }
    sm[q][j4] = acc;
    __syncthreads();
    if (q == 0 && f < count) {
        float4 t = sm[0][j4];
#pragma unroll
        for (int qq = 1; qq < 16; ++qq) {
            const float4 v = sm[qq][j4];
            t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w;
        }
        float *dst = si.radix4 ? a.d_tw4 + (s * a.sc.tw4_stack_stride + si.tw_off) * ef
                               : a.d_tw2 + (s * a.sc.tw2_stack_stride + si.tw_off) * ef;
        *reinterpret_cast<float4 *>(dst + f) = t;
    }
}

}  // namespace bf
