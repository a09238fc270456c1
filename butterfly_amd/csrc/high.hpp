// Stages that pair element bits >= 10 of rows longer than 1024.
//
// A pass handles the stages on H adjacent bits [low_bits, low_bits + H), low_bits >= 10.  A
// thread takes one setting p of all the other bits and holds the 2^H elements of a row that
// differ in those H bits in registers; all the stages of the pass run in registers with their
// 2x2 factors resident for the whole launch.  Threads of a workgroup take consecutive p, whose
// low ten bits are the element's low ten bits, so every access is a coalesced row segment.
// The pass is purely streaming: one read and one write of the activation (plus one read of
// the gradient in the backward pass).  Used for rows of 2048 and 4096 (one or two high bits);
// longer rows run their high bits through the kernels of fast.hpp on tiles (SpanPlan).
#pragma once

#include "common.hpp"
#include "fast.hpp"

namespace bf {

constexpr int kHighThreads = 256;
// Element index of register j of thread p: the H bits of j inserted at bit position lb of p.
__device__ __forceinline__ int high_col(int p, int j, int lb, int H)
{
    return ((p >> lb) << (lb + H)) | (j << lb) | (p & ((1 << lb) - 1));
}

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
    int low_bits;              // position of the lowest of the H bits this pass works on (>= 10)
};

// hb(s): which of the H bits stage s pairs (bit low_bits + hb); two bits of PAT per stage
template <int PAT>
__host__ __device__ constexpr int high_bit_of(int s) { return (PAT >> (2 * s)) & 3; }

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
            const int b = a.low_bits + hb;
            static_for<0, E / 2>([&](auto Q) {
                constexpr int q = Q;
                constexpr int j0 = j0_of(s, q);
                const int e = high_col(p, j0, a.low_bits, H);
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

    int x_col[E], xo_col[E];  // tensor columns of the thread's elements (-1: none)
#pragma unroll
    for (int j = 0; j < E; ++j) {
        const int col = high_col(p, j, a.low_bits, H);
        x_col[j] = (int)view_col(a.x_view, col);
        xo_col[j] = (int)view_col(a.xo_view, col);
    }
    auto load_row = [&](int64_t row, T (&v)[E]) {
#pragma unroll
        for (int j = 0; j < E; ++j) {
            v[j] = (row < r1 && x_col[j] >= 0) ? in[row * a.x_view.sb + x_col[j] * a.x_view.se] : zero_of(T());
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
            if (xo_col[j] >= 0) out[row * a.xo_view.sb + xo_col[j] * a.xo_view.se] = v[j];
        }
    }
}

// Backward of the same pass: replays the stages keeping their inputs, then walks back.
// d_twiddle sums stay in registers across all rows of the workgroup and are written once
// into the partial slice of this row partition (workgroups with different blockIdx.z own
// different pair indices of the same slice).
//
// The factors and sums leave room for three wavefronts per SIMD only, too few to keep HBM
// busy with register prefetch, so rows are fetched straight into LDS (load_row_to_lds in
// fast.hpp) kHighAhead rows ahead: a lane reads back exactly the dwords it fetched itself, so
// no barrier is involved, only the wait for the wavefront's own requests.  All operands are
// addressed with 32-bit offsets from the workgroup's first row (the host checks the span).
// THREADS positions per workgroup (gridDim.z = (n >> H) / THREADS): as many as the registers
// allow, so that a workgroup touches long contiguous pieces of every quarter-row.
constexpr int kHighAhead = 3;   // rows requested ahead; kHighAhead + 1 row slots in LDS

template <typename T, int H, int NST, int PAT, int THREADS>
__global__ __launch_bounds__(THREADS) void high_bw_kernel(HighArgs a)
{
    using TW = HighTwiddle<T, H, NST, PAT>;
    constexpr int E = 1 << H;
    constexpr int W = (int)sizeof(T) / 4;  // dwords per scalar: the planes of a complex row are fetched separately
    constexpr int EB = (int)sizeof(T);
    // complex64 rows would have to be fetched as two strided 32-bit planes, which measured
    // slower than plain register prefetch: float only
    constexpr bool DIRECT = W == 1;
    constexpr int SLOT = 2 * E * W * THREADS;  // dwords per row slot: x and g, E elements, W planes
    __shared__ float rows[DIRECT ? (kHighAhead + 1) * SLOT : 1];
    const int p = blockIdx.z * THREADS + threadIdx.x;
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
    const int nr = (int)(r1 - r0);
    const BufDesc x_desc = make_desc(reinterpret_cast<const T *>(a.x_in) + stack * a.x_view.ss + r0 * a.x_view.sb);
    const BufDesc g_desc = make_desc(reinterpret_cast<const T *>(a.g_out) + stack * a.g_view.ss + r0 * a.g_view.sb);
    const __amdgpu_buffer_rsrc_t gi_rs =
        make_rsrc(reinterpret_cast<T *>(a.g_in) + stack * a.gi_view.ss + r0 * a.gi_view.sb);
    const int x_row = (int)(a.x_view.sb * EB), g_row = (int)(a.g_view.sb * EB), gi_row = (int)(a.gi_view.sb * EB);
    int x_off[E], g_off[E], gi_off[E];
#pragma unroll
    for (int j = 0; j < E; ++j) {
        const int col = high_col(p, j, a.low_bits, H);
        const int64_t xc = view_col(a.x_view, col), gc = view_col(a.g_view, col), gic = view_col(a.gi_view, col);
        x_off[j] = xc >= 0 ? (int)(xc * a.x_view.se * EB) : kOob;
        g_off[j] = gc >= 0 ? (int)(gc * a.g_view.se * EB) : kOob;
        gi_off[j] = gic >= 0 ? (int)(gic * a.gi_view.se * EB) : kOob;
    }
    // slot layout, in dwords: [x | g][element j][plane][thread]; a wavefront's 64 lanes are contiguous
    const unsigned wave_addr =
        (unsigned)(unsigned long long)(LdsFloat *)rows + (unsigned)(threadIdx.x & ~63) * 4;
    auto fetch_row = [&](int row) {  // row relative to r0
        const unsigned slot_addr = wave_addr + (unsigned)(row & kHighAhead) * SLOT * 4;
#pragma unroll
        for (int j = 0; j < E; ++j) {
#pragma unroll
            for (int w = 0; w < W; ++w) {
                load_row_to_lds(x_desc, slot_addr + ((0 * E + j) * W + w) * THREADS * 4,
                                row < nr && x_off[j] != kOob ? x_off[j] + 4 * w : kOob, row * x_row);
                load_row_to_lds(g_desc, slot_addr + ((1 * E + j) * W + w) * THREADS * 4,
                                row < nr && g_off[j] != kOob ? g_off[j] + 4 * w : kOob, row * g_row);
            }
        }
    };
    auto read_row = [&](int row, int which, int j) -> T {
        const float *src = rows + (row & kHighAhead) * SLOT + (which * E + j) * W * THREADS + threadIdx.x;
        if constexpr (W == 1) return src[0];
        else return make_float2(src[0], src[THREADS]);
    };
    static_assert((kHighAhead & (kHighAhead + 1)) == 0, "row slots are indexed with a mask");
    // memory operations issued after the requests of a row and before that row is read: the
    // requests of the kHighAhead following rows and the stores of the kHighAhead rows before it
    constexpr int YOUNGER = kHighAhead * (2 * E * W + E);
    static_assert(YOUNGER <= 63, "the wait counter holds 6 bits");

    // register flavour: one row ahead
    const __amdgpu_buffer_rsrc_t x_rs = make_rsrc(reinterpret_cast<const T *>(a.x_in) + stack * a.x_view.ss + r0 * a.x_view.sb);
    const __amdgpu_buffer_rsrc_t g_rs = make_rsrc(reinterpret_cast<const T *>(a.g_out) + stack * a.g_view.ss + r0 * a.g_view.sb);
    auto load_row = [&](int row, T (&x)[E], T (&g)[E]) {
#pragma unroll
        for (int j = 0; j < E; ++j) {
            x[j] = buf_load<T>(x_rs, row < nr ? x_off[j] : kOob, row * x_row);
            g[j] = buf_load<T>(g_rs, row < nr ? g_off[j] : kOob, row * g_row);
        }
    };
    T nx[E], ng[E];
    if constexpr (DIRECT) {
#pragma unroll
        for (int r = 0; r < kHighAhead; ++r) {
            fetch_row(r);
            // stores that the range check discards: every row then sees the same number of
            // younger operations, the first ones included
#pragma unroll
            for (int j = 0; j < E; ++j) buf_store(gi_rs, kOob, 0, zero_of(T()));
        }
    } else {
        load_row(0, nx, ng);
    }
    for (int row = 0; row < nr; ++row) {
        T act[NST][E], g[E];
        if constexpr (DIRECT) {
            fetch_row(row + kHighAhead);
            wait_rows_in_lds<YOUNGER>();
#pragma unroll
            for (int j = 0; j < E; ++j) {
                act[0][j] = read_row(row, 0, j);
                g[j] = read_row(row, 1, j);
            }
        } else {
#pragma unroll
            for (int j = 0; j < E; ++j) {
                act[0][j] = nx[j];
                g[j] = ng[j];
            }
            load_row(row + 1, nx, ng);
        }
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
        for (int j = 0; j < E; ++j) buf_store(gi_rs, gi_off[j], row * gi_row, g[j]);
    }
    if constexpr (DIRECT) wait_rows_in_lds<0>();  // requests past the last row (they fetch nothing)

    T *part = reinterpret_cast<T *>(a.partial) + ((int64_t)blockIdx.x * gridDim.y + stack) * NST * a.partial_slot;
    static_for<0, NST>([&](auto S) {
        constexpr int s = S;
        constexpr int hb = high_bit_of<PAT>(s);
        const int b = a.low_bits + hb;
        static_for<0, E / 2>([&](auto Q) {
            constexpr int q = Q;
            constexpr int j0 = TW::j0_of(s, q);
            const int e = high_col(p, j0, a.low_bits, H);
            const int i = ((e >> (b + 1)) << b) | (e & ((1 << b) - 1));
            T *d = part + (int64_t)s * a.partial_slot + (int64_t)i * 4;
#pragma unroll
            for (int k = 0; k < 4; ++k) d[k] = acc[s][q][k];
        });
    });
}

}  // namespace bf
