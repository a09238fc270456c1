// Stages that pair element bits >= 10 of rows longer than 1024.
//
// Such a stage couples elements 1024 (or 2048) apart, so a thread takes one low position
// p in [0, 1024) and holds the 2^H elements {p + j * 1024} of a row in registers; all the
// stages of the pass run in registers with their 2x2 factors resident for the whole launch.
// Threads of a workgroup take consecutive p, so every access is a coalesced row segment.
// The pass is purely streaming: one read and one write of the activation (plus one read of
// the gradient in the backward pass).
#pragma once

#include "common.hpp"
#include "fast.hpp"

namespace bf {

constexpr int kHighThreads = 256;
constexpr int kHighLowBits = 10;  // bits below this are handled by the chunked kernels

struct HighArgs {
    const void *tw;            // twiddle tensor, stack 0
    int64_t tw_stack_stride;   // scalars
    int64_t tw_stage_stride;   // scalars between stages: (n / 2) * 4
    int tw_stage[4];           // global stage number of every local stage
    const void *x_in;          // activation entering the pass
    View x_view;
    void *x_out;               // forward: activation leaving the pass
    View xo_view;
    const void *g_out;         // backward: gradient w.r.t. the activation leaving the pass
    View g_view;
    void *g_in;                // backward: gradient w.r.t. the activation entering the pass
    View gi_view;
    void *partial;             // backward: (gridDim.x, S, NST, partial_slot) scalars
    int64_t partial_slot;
    int64_t batch;
    int64_t rows_per_wg;
};

// hb(s): which of the H high bits stage s pairs (bit 10 + hb)
template <int PAT>
__host__ __device__ constexpr int high_bit_of(int s) { return (PAT >> s) & 1; }

template <typename T, int H, int NST, int PAT>
struct HighTwiddle {
    static constexpr int E = 1 << H;
    T t[NST][E / 2][4];

    // pair q of stage s couples registers j0 (bit hb clear) and j0 | (1 << hb)
    __device__ static constexpr int j0_of(int s, int q)
    {
        const int hb = high_bit_of<PAT>(s);
        // insert a zero at bit position hb of q
        return ((q >> hb) << (hb + 1)) | (q & ((1 << hb) - 1));
    }

    __device__ __forceinline__ void load(const HighArgs &a, int stack, int p)
    {
        const T *base = reinterpret_cast<const T *>(a.tw) + stack * a.tw_stack_stride;
        static_for<0, NST>([&](auto S) {
            constexpr int s = S;
            constexpr int hb = high_bit_of<PAT>(s);
            constexpr int b = kHighLowBits + hb;
            static_for<0, E / 2>([&](auto Q) {
                constexpr int q = Q;
                constexpr int j0 = j0_of(s, q);
                const int e = (j0 << kHighLowBits) | p;
                const int i = ((e >> (b + 1)) << b) | (e & ((1 << b) - 1));
                const T *src = base + a.tw_stage[s] * a.tw_stage_stride + (int64_t)i * 4;
#pragma unroll
                for (int k = 0; k < 4; ++k) t[s][q][k] = src[k];
            });
        });
    }
};

template <typename T, int H, int NST, int PAT>
__global__ __launch_bounds__(kHighThreads) void high_fw_kernel(HighArgs a)
{
    using TW = HighTwiddle<T, H, NST, PAT>;
    constexpr int E = 1 << H;
    const int p = blockIdx.z * kHighThreads + threadIdx.x;
    const int stack = blockIdx.y;
    TW tw;
    tw.load(a, stack, p);

    const int64_t r0 = (int64_t)blockIdx.x * a.rows_per_wg;
    const int64_t r1 = r0 + a.rows_per_wg < a.batch ? r0 + a.rows_per_wg : a.batch;
    const T *in = reinterpret_cast<const T *>(a.x_in) + stack * a.x_view.ss;
    T *out = reinterpret_cast<T *>(a.x_out) + stack * a.xo_view.ss;

    auto load_row = [&](int64_t row, T (&v)[E]) {
#pragma unroll
        for (int j = 0; j < E; ++j) {
            const int col = (j << kHighLowBits) | p;
            v[j] = (row < r1 && col < a.x_view.width) ? in[row * a.x_view.sb + col * a.x_view.se] : zero_of(T());
        }
    };
    T nxt[E];
    load_row(r0, nxt);
    for (int64_t row = r0; row < r1; ++row) {
        T v[E];
#pragma unroll
        for (int j = 0; j < E; ++j) v[j] = nxt[j];
        load_row(row + 1, nxt);
        static_for<0, NST>([&](auto S) {
            constexpr int s = S;
            constexpr int hb = high_bit_of<PAT>(s);
            static_for<0, E / 2>([&](auto Q) {
                constexpr int q = Q;
                constexpr int j0 = TW::j0_of(s, q), j1 = j0 | (1 << hb);
                const T x0 = v[j0], x1 = v[j1];
                v[j0] = mac(mul(tw.t[s][q][0], x0), tw.t[s][q][1], x1);
                v[j1] = mac(mul(tw.t[s][q][2], x0), tw.t[s][q][3], x1);
            });
        });
#pragma unroll
        for (int j = 0; j < E; ++j) {
            const int col = (j << kHighLowBits) | p;
            if (col < a.xo_view.width) out[row * a.xo_view.sb + col * a.xo_view.se] = v[j];
        }
    }
}

// Backward of the same pass: replays the stages keeping their inputs, then walks back.
// d_twiddle sums stay in registers across all rows of the workgroup and are written once
// into the partial slice of this row partition (workgroups with different blockIdx.z own
// different pair indices of the same slice).
template <typename T, int H, int NST, int PAT>
__global__ __launch_bounds__(kHighThreads) void high_bw_kernel(HighArgs a)
{
    using TW = HighTwiddle<T, H, NST, PAT>;
    constexpr int E = 1 << H;
    const int p = blockIdx.z * kHighThreads + threadIdx.x;
    const int stack = blockIdx.y;
    TW tw;
    tw.load(a, stack, p);
    T acc[NST][E / 2][4];
    static_for<0, NST>([&](auto S) {
        static_for<0, E / 2>([&](auto Q) {
#pragma unroll
            for (int k = 0; k < 4; ++k) acc[S][Q][k] = zero_of(T());
        });
    });

    const int64_t r0 = (int64_t)blockIdx.x * a.rows_per_wg;
    const int64_t r1 = r0 + a.rows_per_wg < a.batch ? r0 + a.rows_per_wg : a.batch;
    const T *xin = reinterpret_cast<const T *>(a.x_in) + stack * a.x_view.ss;
    const T *gout = reinterpret_cast<const T *>(a.g_out) + stack * a.g_view.ss;
    T *gin = reinterpret_cast<T *>(a.g_in) + stack * a.gi_view.ss;

    auto load_row = [&](int64_t row, T (&x)[E], T (&g)[E]) {
#pragma unroll
        for (int j = 0; j < E; ++j) {
            const int col = (j << kHighLowBits) | p;
            x[j] = (row < r1 && col < a.x_view.width) ? xin[row * a.x_view.sb + col * a.x_view.se] : zero_of(T());
            g[j] = (row < r1 && col < a.g_view.width) ? gout[row * a.g_view.sb + col * a.g_view.se] : zero_of(T());
        }
    };
    T nx[E], ng[E];
    load_row(r0, nx, ng);
    for (int64_t row = r0; row < r1; ++row) {
        T act[NST][E], g[E];
#pragma unroll
        for (int j = 0; j < E; ++j) {
            act[0][j] = nx[j];
            g[j] = ng[j];
        }
        load_row(row + 1, nx, ng);
        static_for<0, NST - 1>([&](auto S) {
            constexpr int s = S;
            constexpr int hb = high_bit_of<PAT>(s);
            static_for<0, E / 2>([&](auto Q) {
                constexpr int q = Q;
                constexpr int j0 = TW::j0_of(s, q), j1 = j0 | (1 << hb);
                const T x0 = act[s][j0], x1 = act[s][j1];
                act[s + 1][j0] = mac(mul(tw.t[s][q][0], x0), tw.t[s][q][1], x1);
                act[s + 1][j1] = mac(mul(tw.t[s][q][2], x0), tw.t[s][q][3], x1);
            });
        });
        static_for<0, NST>([&](auto S) {
            constexpr int s = NST - 1 - S;
            constexpr int hb = high_bit_of<PAT>(s);
            static_for<0, E / 2>([&](auto Q) {
                constexpr int q = Q;
                constexpr int j0 = TW::j0_of(s, q), j1 = j0 | (1 << hb);
                const T g0 = g[j0], g1 = g[j1];
                const T x0 = act[s][j0], x1 = act[s][j1];
                acc[s][q][0] = macc(acc[s][q][0], x0, g0);
                acc[s][q][1] = macc(acc[s][q][1], x1, g0);
                acc[s][q][2] = macc(acc[s][q][2], x0, g1);
                acc[s][q][3] = macc(acc[s][q][3], x1, g1);
                g[j0] = macc(mul(conj_of(tw.t[s][q][0]), g0), tw.t[s][q][2], g1);
                g[j1] = macc(mul(conj_of(tw.t[s][q][1]), g0), tw.t[s][q][3], g1);
            });
        });
#pragma unroll
        for (int j = 0; j < E; ++j) {
            const int col = (j << kHighLowBits) | p;
            if (col < a.gi_view.width) gin[row * a.gi_view.sb + col * a.gi_view.se] = g[j];
        }
    }

    T *part = reinterpret_cast<T *>(a.partial) + ((int64_t)blockIdx.x * gridDim.y + stack) * NST * a.partial_slot;
    static_for<0, NST>([&](auto S) {
        constexpr int s = S;
        constexpr int hb = high_bit_of<PAT>(s);
        constexpr int b = kHighLowBits + hb;
        static_for<0, E / 2>([&](auto Q) {
            constexpr int q = Q;
            constexpr int j0 = TW::j0_of(s, q);
            const int e = (j0 << kHighLowBits) | p;
            const int i = ((e >> (b + 1)) << b) | (e & ((1 << b) - 1));
            T *d = part + (int64_t)s * a.partial_slot + (int64_t)i * 4;
#pragma unroll
            for (int k = 0; k < 4; ++k) d[k] = acc[s][q][k];
        });
    });
}

}  // namespace bf
