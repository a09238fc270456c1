// Twiddle-stationary base-4 kernels for the shapes fast4.hpp does not take: odd log_n (the
// block ends with one 2x2 stage) and complex64, n = 2^L <= 1024; one block per launch.
//
// Same ownership as fast.hpp (1024 threads, one element per thread and row, factors in
// registers for the whole launch, layouts A and B with an LDS transpose between them).  A
// radix-4 stage couples the four elements that differ in two adjacent bits (b, b + 1), which
// need not be aligned to an even bit here (with decreasing stride and odd log_n the pairs are
// (1,2), (3,4), ...).  The three partners are reached by composing the single-bit exchanges of
// fast.hpp: bit b, bit b + 1, and bit b + 1 of the value that came over bit b -- three
// exchanges, as many as an aligned pair needs.  Both bits are always reachable in one layout:
// A serves bits 0..5, B serves the bits from NSWAP up.
//
// Backward: the thread keeps the COLUMN of the factor that belongs to its element,
// colm[m] = T[r ^ m][r].  One set of exchanges (of the gradient) then serves both products:
//   dT[r ^ m][r] += g(partner m) * conj(x)          (x: the thread's own stage input)
//   g            <- sum_m conj(T[r ^ m][r]) * g(partner m)
#pragma once

#include "fast.hpp"

namespace bf {

template <int L, bool INC>
struct Plan4G {
    static_assert(L >= 2 && L <= 10, "one block of a row of at most 1024 elements");
    static constexpr int NS4 = L / 2;
    static constexpr bool ODD = (L & 1) != 0;
    static constexpr int NS = NS4 + (ODD ? 1 : 0);   // stage NS4 is the 2x2 stage when L is odd
    static constexpr int NSWAP = L > 6 ? L - 6 : 0;
    static constexpr int SLOTS = 1024 >> L;
    // lowest bit a stage works on, and how many bits
    static constexpr int lo(int s) { return s < NS4 ? (INC ? 2 * s : L - 2 - 2 * s) : (INC ? L - 1 : 0); }
    static constexpr int width(int s) { return s < NS4 ? 2 : 1; }
    static constexpr int layout(int s)
    {
        int cur = 0;
        for (int j = 0; j <= s; ++j) {
            if (lo(j) + width(j) - 1 >= 6) cur = 1;
            else if (lo(j) < NSWAP) cur = 0;
        }
        return cur;
    }
    static constexpr int layout_before(int s) { return s == 0 ? 0 : layout(s - 1); }
    static constexpr int layout_after(int s) { return s == NS - 1 ? 0 : layout(s + 1); }
    // exchange kind of a single bit (see FastPlan::kind)
    static constexpr int kind(int bit) { return bit >= 6 ? bit - 6 : bit; }
};

// Rows longer than 2^L run these kernels on their 2^L-element chunks (blockIdx.z) for the stages
// that stay inside a chunk: chunk c uses the factor quads (pairs) c * 2^L / 4 (/ 2) onward of
// every stage, and its sums land at the same place in the partial slice.
struct Fast4GArgs {
    const void *tw4;           // radix-4 factors of the first stage run here, stack 0: (stages, n_full/4, 4, 4)
    int64_t tw4_stack_stride;  // scalars
    int64_t tw4_stage_stride;  // scalars between consecutive stages: (n_full / 4) * 16
    const void *tw2;           // the block's 2x2 factors, stack 0: (n_full/2, 2, 2); odd L only
    int64_t tw2_stack_stride;
    int64_t n_full;            // length of the whole row (2^L when the row is one chunk)
    const void *x_in;
    View x_view;
    void *x_out;               // forward output
    View xo_view;
    const void *g_out;         // backward
    View g_view;
    void *g_in;
    View gi_view;
    void *partial;             // (gridDim.x, S, NS, 4 n) scalars
    int64_t batch;
    int64_t ngroups;
    int64_t groups_per_wg;
};

template <typename T, int L, bool INC, bool WITH_COLUMN>
struct Factors4G {
    using P = Plan4G<L, INC>;
    static constexpr int NS4 = P::NS4;
    T row[NS4][4];                         // row[s][m]  = T[r][r ^ m]
    T colm[WITH_COLUMN ? NS4 : 1][4];      // colm[s][m] = T[r ^ m][r]
    T ta, tb, tc;                          // 2x2 stage: T[r][r], T[r][1 - r], T[1 - r][r]

    __device__ __forceinline__ void load(const Fast4GArgs &a, int stack, int chunk, const FastCoords &c)
    {
        constexpr int n = 1 << L;
        const T *tw4 = reinterpret_cast<const T *>(a.tw4) + stack * a.tw4_stack_stride + (int64_t)chunk * (n / 4) * 16;
        static_for<0, NS4>([&](auto S) {
            constexpr int s = S;
            constexpr int b = P::lo(s);
            const int e = P::layout(s) ? c.eB : c.eA;
            const int r = (e >> b) & 3;
            const int q = ((e >> (b + 2)) << b) | (e & ((1 << b) - 1));
            const T *F = tw4 + (int64_t)s * a.tw4_stage_stride + q * 16;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                row[s][m] = F[r * 4 + (r ^ m)];
                if constexpr (WITH_COLUMN) colm[s][m] = F[(r ^ m) * 4 + r];
            }
        });
        ta = tb = tc = zero_of(T());
        if constexpr (P::ODD) {
            constexpr int b = P::lo(NS4);
            const int e = P::layout(NS4) ? c.eB : c.eA;
            const int r = (e >> b) & 1;
            const int i = ((e >> (b + 1)) << b) | (e & ((1 << b) - 1));
            const T *F = reinterpret_cast<const T *>(a.tw2) + stack * a.tw2_stack_stride +
                         ((int64_t)chunk * (n / 2) + i) * 4;
            ta = F[3 * r];
            tb = F[r + 1];
            tc = F[2 - r];
        }
    }
};

// The values of v held by the three partners of a radix-4 stage on bits (B0, B0 + 1).
template <int K0, int K1, typename T>
__device__ __forceinline__ void partners4(T v, int bperm_addr, T &p1, T &p2, T &p3)
{
    p1 = partner<K0>(v, bperm_addr);
    p2 = partner<K1>(v, bperm_addr);
    p3 = partner<K1>(p1, bperm_addr);
}

template <typename T, int L, bool INC, int R>
__global__ __launch_bounds__(kFastThreads) void fast4g_fw_kernel(Fast4GArgs a)
{
    using P = Plan4G<L, INC>;
    constexpr int NS = P::NS, NS4 = P::NS4, SLOTS = P::SLOTS;
    constexpr int EB = (int)sizeof(T);
    __shared__ T lds[P::NSWAP > 0 ? 2 * R * kFastRowWords : 1];
    const int t = threadIdx.x;
    const int stack = blockIdx.y;
    const int chunk = blockIdx.z;
    const FastCoords c = fast_coords<L>(t);
    const int col = (chunk << L) + c.eA;   // column of this thread's element in the whole row

    Factors4G<T, L, INC, false> f;
    f.load(a, stack, chunk, c);

    const int64_t g0 = (int64_t)blockIdx.x * a.groups_per_wg;
    const int64_t g1 = g0 + a.groups_per_wg < a.ngroups ? g0 + a.groups_per_wg : a.ngroups;
    const int ng = (int)(g1 - g0);
    const int64_t row_end = g1 * SLOTS < a.batch ? g1 * SLOTS : a.batch;
    const int rows_valid = (int)(row_end - g0 * SLOTS);
    const __amdgpu_buffer_rsrc_t in_rs =
        make_rsrc(reinterpret_cast<const T *>(a.x_in) + g0 * SLOTS * a.x_view.sb + stack * a.x_view.ss);
    const __amdgpu_buffer_rsrc_t out_rs =
        make_rsrc(reinterpret_cast<T *>(a.x_out) + g0 * SLOTS * a.xo_view.sb + stack * a.xo_view.ss);
    const int in_row = (int)(a.x_view.sb * EB), out_row = (int)(a.xo_view.sb * EB);
    const int64_t in_col = view_col(a.x_view, col), out_col = view_col(a.xo_view, col);
    const int in_thr = in_col >= 0 ? c.slot * in_row + (int)(in_col * a.x_view.se * EB) : kOob;
    const int out_thr = out_col >= 0 ? c.slot * out_row + (int)(out_col * a.xo_view.se * EB) : kOob;

    auto load_rows = [&](int grel, T (&v)[R]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const bool ok = (grel + r) * SLOTS + c.slot < rows_valid;
            v[r] = buf_load<T>(in_rs, ok ? in_thr : kOob, (grel + r) * SLOTS * in_row);
        }
    };
    // Transposes alternate between two buffers, so one barrier each is enough: a wavefront
    // writes a buffer again only after the barrier of the transpose in between, which every
    // wavefront reaches after it has read that buffer.
    int par = 0;
    auto transpose = [&](T (&v)[R], int to_b) {
        const int wr = to_b ? c.fA : c.fB, rd = to_b ? c.fB : c.fA;
        T *buf = lds + par * R * kFastRowWords;
#pragma unroll
        for (int r = 0; r < R; ++r) buf[r * kFastRowWords + wr] = v[r];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r) v[r] = buf[r * kFastRowWords + rd];
        par ^= 1;
    };

    T nxt[R];
    load_rows(0, nxt);
    for (int grel = 0; grel < ng; grel += R) {
        T v[R];
#pragma unroll
        for (int r = 0; r < R; ++r) v[r] = nxt[r];
        load_rows(grel + R, nxt);
        static_for<0, NS>([&](auto S) {
            constexpr int s = S;
            if constexpr (P::layout(s) != P::layout_before(s)) transpose(v, P::layout(s));
            if constexpr (s < NS4) {
                constexpr int K0 = P::kind(P::lo(s)), K1 = P::kind(P::lo(s) + 1);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    T p1, p2, p3;
                    partners4<K0, K1>(v[r], c.bperm_addr, p1, p2, p3);
                    T y = mul(f.row[s][0], v[r]);
                    y = mac(y, f.row[s][1], p1);
                    y = mac(y, f.row[s][2], p2);
                    y = mac(y, f.row[s][3], p3);
                    v[r] = y;
                }
            } else {
                constexpr int K = P::kind(P::lo(s));
#pragma unroll
                for (int r = 0; r < R; ++r) v[r] = fw_product<K>(v[r], f.ta, f.tb, c.bperm_addr);
            }
        });
        if constexpr (P::layout(NS - 1) != 0) transpose(v, 0);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const bool ok = (grel + r) * SLOTS + c.slot < rows_valid;
            buf_store(out_rs, ok ? out_thr : kOob, (grel + r) * SLOTS * out_row, v[r]);
        }
    }
}

// R row groups per iteration: their transposes share the barriers.
template <typename T, int L, bool INC, int R>
__global__ __launch_bounds__(kFastThreads) void fast4g_bw_kernel(Fast4GArgs a)
{
    using P = Plan4G<L, INC>;
    constexpr int n = 1 << L, NS = P::NS, NS4 = P::NS4, SLOTS = P::SLOTS;
    constexpr int EB = (int)sizeof(T);
    // two transpose buffers of R rows; the epilogue's slot reduction reuses the same memory
    constexpr int kRedWords = SLOTS > 1 ? 4 * 1024 : 1;
    constexpr int kRowWords = P::NSWAP > 0 ? 2 * R * kFastRowWords : 1;
    constexpr int kLdsWords = kRedWords > kRowWords ? kRedWords : kRowWords;
    __shared__ T lds[kLdsWords];
    const int t = threadIdx.x;
    const int stack = blockIdx.y;
    const int chunk = blockIdx.z;
    const FastCoords c = fast_coords<L>(t);
    const int col = (chunk << L) + c.eA;   // column of this thread's element in the whole row

    Factors4G<T, L, INC, true> f;
    f.load(a, stack, chunk, c);
    T acc[NS4][4];   // acc[s][m] = dT[r ^ m][r]
    static_for<0, NS4>([&](auto S) {
#pragma unroll
        for (int m = 0; m < 4; ++m) acc[S][m] = zero_of(T());
    });
    T self2 = zero_of(T()), cross2 = zero_of(T());   // 2x2 stage: dT[r][r], dT[1 - r][r]

    const int64_t g0 = (int64_t)blockIdx.x * a.groups_per_wg;
    const int64_t g1 = g0 + a.groups_per_wg < a.ngroups ? g0 + a.groups_per_wg : a.ngroups;
    const int ng = (int)(g1 - g0);
    const int64_t row_end = g1 * SLOTS < a.batch ? g1 * SLOTS : a.batch;
    const int rows_valid = (int)(row_end - g0 * SLOTS);
    const __amdgpu_buffer_rsrc_t x_rs =
        make_rsrc(reinterpret_cast<const T *>(a.x_in) + g0 * SLOTS * a.x_view.sb + stack * a.x_view.ss);
    const __amdgpu_buffer_rsrc_t g_rs =
        make_rsrc(reinterpret_cast<const T *>(a.g_out) + g0 * SLOTS * a.g_view.sb + stack * a.g_view.ss);
    const __amdgpu_buffer_rsrc_t gi_rs =
        make_rsrc(reinterpret_cast<T *>(a.g_in) + g0 * SLOTS * a.gi_view.sb + stack * a.gi_view.ss);
    const int x_row = (int)(a.x_view.sb * EB), g_row = (int)(a.g_view.sb * EB), gi_row = (int)(a.gi_view.sb * EB);
    const int64_t x_col = view_col(a.x_view, col), g_col = view_col(a.g_view, col), gi_col = view_col(a.gi_view, col);
    const int x_thr = x_col >= 0 ? c.slot * x_row + (int)(x_col * a.x_view.se * EB) : kOob;
    const int g_thr = g_col >= 0 ? c.slot * g_row + (int)(g_col * a.g_view.se * EB) : kOob;
    const int gi_thr = gi_col >= 0 ? c.slot * gi_row + (int)(gi_col * a.gi_view.se * EB) : kOob;

    int par = 0;   // see fast4g_fw_kernel
    auto transpose = [&](T (&v)[R], int to_b) {
        const int wr = to_b ? c.fA : c.fB, rd = to_b ? c.fB : c.fA;
        T *buf = lds + par * R * kFastRowWords;
#pragma unroll
        for (int r = 0; r < R; ++r) buf[r * kFastRowWords + wr] = v[r];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r) v[r] = buf[r * kFastRowWords + rd];
        par ^= 1;
    };
    auto row_ok = [&](int grp) { return grp * SLOTS + c.slot < rows_valid; };
    // (`full`: the caller knows that these row groups exist for every row slot of the workgroup)
    auto load_rows = [&](int grel, T (&x)[R], T (&g)[R], bool full = false) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const bool ok = full || row_ok(grel + r);
            x[r] = buf_load<T>(x_rs, ok ? x_thr : kOob, (grel + r) * SLOTS * x_row);
            g[r] = buf_load<T>(g_rs, ok ? g_thr : kOob, (grel + r) * SLOTS * g_row);
        }
    };

    T nx[R], ngr[R];
    load_rows(0, nx, ngr);
    // FULL: the groups this iteration stores and the ones it prefetches exist for every row slot,
    // so no access needs its range mask: all but the last iterations of a workgroup.
    auto iteration = [&](int grel, auto FULL) {
        constexpr bool full = decltype(FULL)::value;
        T v[R], gv[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            v[r] = nx[r];
            gv[r] = ngr[r];
        }
        load_rows(grel + R, nx, ngr, full);
        T act[NS][R];
        static_for<0, NS>([&](auto S) {
            constexpr int s = S;
            if constexpr (P::layout(s) != P::layout_before(s)) transpose(v, P::layout(s));
#pragma unroll
            for (int r = 0; r < R; ++r) {
                act[s][r] = v[r];
                if constexpr (s + 1 < NS) {   // (the 2x2 stage is always last: only radix-4 stages here)
                    constexpr int K0 = P::kind(P::lo(s)), K1 = P::kind(P::lo(s) + 1);
                    T p1, p2, p3;
                    partners4<K0, K1>(v[r], c.bperm_addr, p1, p2, p3);
                    T y = mul(f.row[s][0], v[r]);
                    y = mac(y, f.row[s][1], p1);
                    y = mac(y, f.row[s][2], p2);
                    y = mac(y, f.row[s][3], p3);
                    v[r] = y;
                }
            }
        });
        static_for<0, NS>([&](auto S) {
            constexpr int s = NS - 1 - S;
            if constexpr (P::layout(s) != P::layout_after(s)) transpose(gv, P::layout(s));
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const T xs = act[s][r];
                if constexpr (s < NS4) {
                    constexpr int K0 = P::kind(P::lo(s)), K1 = P::kind(P::lo(s) + 1);
                    T g1v, g2v, g3v;
                    partners4<K0, K1>(gv[r], c.bperm_addr, g1v, g2v, g3v);
                    fmac_pinned(acc[s][0], gv[r], xs);
                    fmac_pinned(acc[s][1], g1v, xs);
                    fmac_pinned(acc[s][2], g2v, xs);
                    fmac_pinned(acc[s][3], g3v, xs);
                    T d = mul(conj_of(f.colm[s][0]), gv[r]);
                    d = macc(d, f.colm[s][1], g1v);
                    d = macc(d, f.colm[s][2], g2v);
                    d = macc(d, f.colm[s][3], g3v);
                    gv[r] = d;
                } else {
                    constexpr int K = P::kind(P::lo(s));
                    bw_products<K>(self2, cross2, gv[r], xs, f.ta, f.tc, c.bperm_addr);
                }
            }
        });
        if constexpr (P::layout(0) != 0) transpose(gv, 0);
#pragma unroll
        for (int r = 0; r < R; ++r)
            buf_store(gi_rs, full || row_ok(grel + r) ? gi_thr : kOob, (grel + r) * SLOTS * gi_row, gv[r]);
    };
    int grel = 0;
    for (; grel < ng && (grel + 2 * R) * SLOTS <= rows_valid; grel += R) iteration(grel, std::true_type{});
    for (; grel < ng; grel += R) iteration(grel, std::false_type{});

    // ---- partial sums of this workgroup, in the layout of the twiddle tensors
    int t2 = t;
    asm volatile("" : "+v"(t2));   // (recompute the coordinates instead of keeping them alive)
    const FastCoords c2 = fast_coords<L>(t2);
    const int64_t slot = 4 * a.n_full;   // scalars per stage in a partial slice
    T *part = reinterpret_cast<T *>(a.partial) + ((int64_t)blockIdx.x * gridDim.y + stack) * NS * slot;
    static_for<0, NS>([&](auto S) {
        constexpr int s = S;
        constexpr int b = P::lo(s);
        const int e = P::layout(s) ? c2.eB : c2.eA;
        T vals[4];
        if constexpr (s < NS4) {
#pragma unroll
            for (int m = 0; m < 4; ++m) vals[m] = acc[s][m];
        } else {
            vals[0] = self2;
            vals[1] = cross2;
            vals[2] = vals[3] = zero_of(T());
        }
        constexpr int M = s < NS4 ? 4 : 2;   // entries a thread holds for this stage
        // where entry m of element eo goes inside the stage's slice
        auto dest = [&](int eo, int m) -> int {
            if constexpr (s < NS4) {
                const int r = (eo >> b) & 3;
                const int q = ((eo >> (b + 2)) << b) | (eo & ((1 << b) - 1));
                return q * 16 + (r ^ m) * 4 + r;
            } else {
                const int r = (eo >> b) & 1;
                const int i = ((eo >> (b + 1)) << b) | (eo & ((1 << b) - 1));
                return i * 4 + (m == 0 ? 3 * r : 2 - r);
            }
        };
        T *d = part + (int64_t)s * slot + (s < NS4 ? (int64_t)chunk * (n / 4) * 16 : (int64_t)chunk * (n / 2) * 4);
        if constexpr (SLOTS == 1) {
#pragma unroll
            for (int m = 0; m < M; ++m) d[dest(e, m)] = vals[m];
        } else {
            // add the row slots of this workgroup in ascending order, then one thread per entry
            __syncthreads();
#pragma unroll
            for (int m = 0; m < M; ++m) lds[(c2.slot * n + e) * M + m] = vals[m];
            __syncthreads();
            for (int o = t2; o < M * n; o += kFastThreads) {
                T sum = lds[o];
#pragma unroll 4
                for (int sl = 1; sl < SLOTS; ++sl) sum = add(sum, lds[sl * M * n + o]);
                d[dest(o / M, o % M)] = sum;
            }
        }
    });
}

}  // namespace bf
