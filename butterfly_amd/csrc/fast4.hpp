// Twiddle-stationary kernels for base-4 float rows, n = 2^L <= 1024 with L even: one block of
// L / 2 radix-4 stages per launch.
//
// Same ownership as fast.hpp: 1024 threads, one element per thread and row, factors in
// registers for the whole launch.  A radix-4 stage couples the four elements that differ in
// an aligned bit pair (2j, 2j+1); the three partners are reached with
//   pair on phi bits (0,1): quad_perm [1,0,3,2] / [2,3,0,1] / [3,2,1,0]
//   pair on phi bits (2,3): row_half_mirror / row_mirror / row_ror:8
//   pair on lane bits (4,5): ds_swizzle xor 16, ds_bpermute xor 32 / xor 48
// and pairs (6,7), (8,9) after the LDS transpose into layout B, where they sit on the phi
// bits.  Each thread keeps its own ROW of the 4x4 factor (forward) and its own COLUMN
// (backward: one set of gradient exchanges serves the d_twiddle column and d_x).
#pragma once

#include "fast.hpp"

namespace bf {

template <int L, bool INC>
struct Plan4 {
    static_assert(L % 2 == 0 && L >= 2 && L <= 10, "base-4 fast path needs an even log_n <= 10");
    static constexpr int NS = L / 2;
    static constexpr int NSWAP = L > 6 ? L - 6 : 0;
    static constexpr int SLOTS = 1024 >> L;
    // low bit of the bit pair coupled by stage s
    static constexpr int bit(int s) { return 2 * (INC ? s : NS - 1 - s); }
    static constexpr int layout(int s)
    {
        int cur = 0;
        for (int j = 0; j <= s; ++j) {
            const int b = bit(j);
            if (b >= 6) cur = 1;
            else if (b < NSWAP) cur = 0;
        }
        return cur;
    }
    static constexpr int layout_before(int s) { return s == 0 ? 0 : layout(s - 1); }
    static constexpr int layout_after(int s) { return s == NS - 1 ? 0 : layout(s + 1); }
    // exchange kind: 0 = phi bits (0,1), 1 = phi bits (2,3), 2 = lane bits (4,5)
    static constexpr int kind(int s)
    {
        const int b = bit(s);
        return (b >= 6 ? b - 6 : b) / 2;
    }
};

// value held by the thread whose element differs by mask M (1, 2, 3) in the stage's bit pair
template <int KQ, int M>
__device__ __forceinline__ float partner4(float v, int lane)
{
    if constexpr (KQ == 0) {
        if constexpr (M == 1) return dpp_move<0xB1>(v);        // quad_perm [1,0,3,2]
        else if constexpr (M == 2) return dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
        else return dpp_move<0x1B>(v);                         // quad_perm [3,2,1,0]
    } else if constexpr (KQ == 1) {
        if constexpr (M == 1) return dpp_move<0x141>(v);       // row_half_mirror: lane ^ 7
        else if constexpr (M == 2) return dpp_move<0x140>(v);  // row_mirror:      lane ^ 15
        else return dpp_move<0x128>(v);                        // row_ror:8:       lane ^ 8
    } else {
        if constexpr (M == 1)
            return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
        else
            return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ (16 * M)) << 2,
                                                                          __builtin_bit_cast(int, v)));
    }
}

// Forward radix-4 stage on DPP lanes for two rows at once: y = sum_m row[m] * (v of partner m),
// the partners read through the DPP operand of the multiply-add.  Two rows per block keep two
// instructions between any write of v0 / v1 (the previous stage's last instructions) and its
// first DPP read, the wait states that read needs.
#define BF_FW4_BLOCK(C1, C2, C3)                                                                     \
    asm volatile("v_mul_f32_e32 %0, %4, %2\n\t"                                                      \
                 "v_mul_f32_e32 %1, %4, %3\n\t"                                                      \
                 "v_fmac_f32_dpp %0, %2, %5 " C1 " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"      \
                 "v_fmac_f32_dpp %1, %3, %5 " C1 " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"      \
                 "v_fmac_f32_dpp %0, %2, %6 " C2 " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"      \
                 "v_fmac_f32_dpp %1, %3, %6 " C2 " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"      \
                 "v_fmac_f32_dpp %0, %2, %7 " C3 " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"      \
                 "v_fmac_f32_dpp %1, %3, %7 " C3 " row_mask:0xf bank_mask:0xf bound_ctrl:1"           \
                 : "=&v"(y0), "=&v"(y1)                                                              \
                 : "v"(v0), "v"(v1), "v"(row[0]), "v"(row[1]), "v"(row[2]), "v"(row[3]))

template <int KQ>
__device__ __forceinline__ void fw4_pair_dpp(float &v0, float &v1, const float (&row)[4])
{
    static_assert(KQ == 0 || KQ == 1, "DPP exchange kinds only");
    float y0, y1;
    if constexpr (KQ == 0) BF_FW4_BLOCK("quad_perm:[1,0,3,2]", "quad_perm:[2,3,0,1]", "quad_perm:[3,2,1,0]");
    else BF_FW4_BLOCK("row_half_mirror", "row_mirror", "row_ror:8");
    v0 = y0;
    v1 = y1;
}
#undef BF_FW4_BLOCK

// Reverse radix-4 stage on DPP lanes, one row: the column sums acc[m] += g(partner m) * x and
// g <- sum_m col[m] * g(partner m), every partner read through a DPP operand; the two plain
// instructions in front are the wait states after the write of g.
#define BF_BW4_BLOCK(C1, C2, C3)                                                                     \
    asm volatile("v_fmac_f32_e32 %0, %5, %6\n\t"                                                     \
                 "v_mul_f32_e32 %4, %7, %5\n\t"                                                      \
                 "v_fmac_f32_dpp %1, %5, %6 " C1 " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"      \
                 "v_fmac_f32_dpp %4, %5, %8 " C1 " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"      \
                 "v_fmac_f32_dpp %2, %5, %6 " C2 " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"      \
                 "v_fmac_f32_dpp %4, %5, %9 " C2 " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"      \
                 "v_fmac_f32_dpp %3, %5, %6 " C3 " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"      \
                 "v_fmac_f32_dpp %4, %5, %10 " C3 " row_mask:0xf bank_mask:0xf bound_ctrl:1"          \
                 : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "=&v"(d)                  \
                 : "v"(g), "v"(x), "v"(col[0]), "v"(col[1]), "v"(col[2]), "v"(col[3]))

template <int KQ>
__device__ __forceinline__ void bw4_dpp(float (&acc)[4], float &g, float x, const float (&col)[4])
{
    static_assert(KQ == 0 || KQ == 1, "DPP exchange kinds only");
    float d;
    if constexpr (KQ == 0) BF_BW4_BLOCK("quad_perm:[1,0,3,2]", "quad_perm:[2,3,0,1]", "quad_perm:[3,2,1,0]");
    else BF_BW4_BLOCK("row_half_mirror", "row_mirror", "row_ror:8");
    g = d;
}
#undef BF_BW4_BLOCK

struct Fast4Args {
    const float *tw4;          // factors of this block, stack 0: (L/2, n/4, 4, 4)
    int64_t tw_stack_stride;
    const float *x_in;
    View x_view;
    float *x_out;              // forward output
    View xo_view;
    const float *g_out;        // backward
    View g_view;
    float *g_in;
    View gi_view;
    float *partial;            // (gridDim.x, S, L/2, 4 n)
    int64_t batch;
    int64_t ngroups;
    int64_t groups_per_wg;
};

template <int L, bool INC, bool WITH_COLUMN>
struct Factors4 {
    static constexpr int NS = L / 2;
    float row[NS][4];  // row[s][m] = T[r][r ^ m]
    float colm[WITH_COLUMN ? NS : 1][4];  // colm[s][m] = T[r ^ m][r]

    // One 16-byte load per stage: the thread's row T[r][0..3] (the four lanes of a quad cover
    // its 64 bytes), put into partner order by two conditional swaps (an xor permutation
    // decomposes by bits).  The column comes from the partners: the thread at r ^ m holds
    // T[r ^ m][(r ^ m) ^ m] = T[r ^ m][r] as its own entry m.  tw: 16-byte aligned.
    __device__ __forceinline__ void load(const float *tw, const FastCoords &c, int lane)
    {
        using P = Plan4<L, INC>;
        constexpr int n = 1 << L;
        static_for<0, NS>([&](auto S) {
            constexpr int s = S;
            constexpr int b = P::bit(s);
            constexpr int lay = P::layout(s);
            const int e = lay ? c.eB : c.eA;
            const int r = (e >> b) & 3;
            const int q = ((e >> (b + 2)) << b) | (e & ((1 << b) - 1));
            const float4 v = *reinterpret_cast<const float4 *>(tw + ((int64_t)s * (n / 4) + q) * 16 + r * 4);
            const bool o1 = (r & 1) != 0, o2 = (r & 2) != 0;
            const float a0 = o1 ? v.y : v.x, a1 = o1 ? v.x : v.y, a2 = o1 ? v.w : v.z, a3 = o1 ? v.z : v.w;
            row[s][0] = o2 ? a2 : a0;
            row[s][1] = o2 ? a3 : a1;
            row[s][2] = o2 ? a0 : a2;
            row[s][3] = o2 ? a1 : a3;
            if constexpr (WITH_COLUMN) {
                constexpr int KQ = P::kind(s);
                colm[s][0] = row[s][0];
                colm[s][1] = partner4<KQ, 1>(row[s][1], lane);
                colm[s][2] = partner4<KQ, 2>(row[s][2], lane);
                colm[s][3] = partner4<KQ, 3>(row[s][3], lane);
            }
        });
    }
};

template <int L, bool INC, int R>
__global__ __launch_bounds__(kFastThreads) void fast4_fw_kernel(Fast4Args a)
{
    using P = Plan4<L, INC>;
    constexpr int NS = P::NS, SLOTS = P::SLOTS;
    __shared__ float lds[P::NSWAP > 0 ? 2 * R * kFastRowWords : 1];
    const int t = threadIdx.x;
    const int lane = t & 63;
    const int stack = blockIdx.y;
    const FastCoords c = fast_coords<L>(t);

    Factors4<L, INC, false> f;
    f.load(a.tw4 + stack * a.tw_stack_stride, c, lane);

    const int64_t g0 = (int64_t)blockIdx.x * a.groups_per_wg;
    const int64_t g1 = g0 + a.groups_per_wg < a.ngroups ? g0 + a.groups_per_wg : a.ngroups;
    const int ng = (int)(g1 - g0);
    const int64_t row_end = g1 * SLOTS < a.batch ? g1 * SLOTS : a.batch;
    const int rows_valid = (int)(row_end - g0 * SLOTS);
    const __amdgpu_buffer_rsrc_t in_rs = make_rsrc(a.x_in + g0 * SLOTS * a.x_view.sb + stack * a.x_view.ss);
    const __amdgpu_buffer_rsrc_t out_rs = make_rsrc(a.x_out + g0 * SLOTS * a.xo_view.sb + stack * a.xo_view.ss);
    const int in_row = (int)(a.x_view.sb * 4), out_row = (int)(a.xo_view.sb * 4);
    const int64_t in_col = view_col(a.x_view, c.eA), out_col = view_col(a.xo_view, c.eA);
    const int in_thr = in_col >= 0 ? c.slot * in_row + (int)(in_col * a.x_view.se * 4) : kOob;
    const int out_thr = out_col >= 0 ? c.slot * out_row + (int)(out_col * a.xo_view.se * 4) : kOob;

    auto load_rows = [&](int grel, float (&v)[R]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const bool ok = (grel + r) * SLOTS + c.slot < rows_valid;
            v[r] = buf_load<float>(in_rs, ok ? in_thr : kOob, (grel + r) * SLOTS * in_row);
        }
    };
    // Transposes alternate between two buffers, so one barrier each is enough: a wavefront
    // writes a buffer again only after the barrier of the transpose in between, which every
    // wavefront reaches after it has read that buffer.
    int par = 0;
    auto transpose = [&](float (&v)[R], int to_b) {
        const int wr = to_b ? c.fA : c.fB, rd = to_b ? c.fB : c.fA;
        float *buf = lds + par * R * kFastRowWords;
#pragma unroll
        for (int r = 0; r < R; ++r) buf[r * kFastRowWords + wr] = v[r];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r) v[r] = buf[r * kFastRowWords + rd];
        par ^= 1;
    };

    float nxt[R];
    load_rows(0, nxt);
    // (this loop keeps its range masks: it is bound by HBM, and a second, unmasked copy of the
    // body measured slower)
    for (int grel = 0; grel < ng; grel += R) {
        float v[R];
#pragma unroll
        for (int r = 0; r < R; ++r) v[r] = nxt[r];
        load_rows(grel + R, nxt);
        static_for<0, NS>([&](auto S) {
            constexpr int s = S;
            constexpr int KQ = P::kind(s);
            if constexpr (P::layout(s) != P::layout_before(s)) transpose(v, P::layout(s));
            if constexpr (KQ < 2 && R % 2 == 0) {
#pragma unroll
                for (int r = 0; r < R; r += 2) fw4_pair_dpp<KQ>(v[r], v[r + 1], f.row[s]);
            } else {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    float y = f.row[s][0] * v[r];
                    y = fmaf(f.row[s][1], partner4<KQ, 1>(v[r], lane), y);
                    y = fmaf(f.row[s][2], partner4<KQ, 2>(v[r], lane), y);
                    y = fmaf(f.row[s][3], partner4<KQ, 3>(v[r], lane), y);
                    v[r] = y;
                }
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
template <int L, bool INC, int R>
__global__ __launch_bounds__(kFastThreads) void fast4_bw_kernel(Fast4Args a)
{
    using P = Plan4<L, INC>;
    constexpr int n = 1 << L, NS = P::NS, SLOTS = P::SLOTS;
    __shared__ float lds[P::NSWAP > 0 ? 2 * R * kFastRowWords : 1];
    const int t = threadIdx.x;
    const int lane = t & 63;
    const int stack = blockIdx.y;
    const FastCoords c = fast_coords<L>(t);

    Factors4<L, INC, true> f;
    f.load(a.tw4 + stack * a.tw_stack_stride, c, lane);
    float acc[NS][4];  // acc[s][m] = sum (g of the partner at mask m) * x = dT[r ^ m][r]
    static_for<0, NS>([&](auto S) {
#pragma unroll
        for (int m = 0; m < 4; ++m) acc[S][m] = 0.0f;
    });

    const int64_t g0 = (int64_t)blockIdx.x * a.groups_per_wg;
    const int64_t g1 = g0 + a.groups_per_wg < a.ngroups ? g0 + a.groups_per_wg : a.ngroups;
    const int ng = (int)(g1 - g0);
    const int64_t row_end = g1 * SLOTS < a.batch ? g1 * SLOTS : a.batch;
    const int rows_valid = (int)(row_end - g0 * SLOTS);
    const __amdgpu_buffer_rsrc_t x_rs = make_rsrc(a.x_in + g0 * SLOTS * a.x_view.sb + stack * a.x_view.ss);
    const __amdgpu_buffer_rsrc_t g_rs = make_rsrc(a.g_out + g0 * SLOTS * a.g_view.sb + stack * a.g_view.ss);
    const __amdgpu_buffer_rsrc_t gi_rs = make_rsrc(a.g_in + g0 * SLOTS * a.gi_view.sb + stack * a.gi_view.ss);
    const int x_row = (int)(a.x_view.sb * 4), g_row = (int)(a.g_view.sb * 4), gi_row = (int)(a.gi_view.sb * 4);
    const int64_t x_col = view_col(a.x_view, c.eA), g_col = view_col(a.g_view, c.eA), gi_col = view_col(a.gi_view, c.eA);
    const int x_thr = x_col >= 0 ? c.slot * x_row + (int)(x_col * a.x_view.se * 4) : kOob;
    const int g_thr = g_col >= 0 ? c.slot * g_row + (int)(g_col * a.g_view.se * 4) : kOob;
    const int gi_thr = gi_col >= 0 ? c.slot * gi_row + (int)(gi_col * a.gi_view.se * 4) : kOob;

    int par = 0;   // see fast4_fw_kernel
    auto transpose = [&](float (&v)[R], int to_b) {
        const int wr = to_b ? c.fA : c.fB, rd = to_b ? c.fB : c.fA;
        float *buf = lds + par * R * kFastRowWords;
#pragma unroll
        for (int r = 0; r < R; ++r) buf[r * kFastRowWords + wr] = v[r];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r) v[r] = buf[r * kFastRowWords + rd];
        par ^= 1;
    };
    auto row_ok = [&](int grp) { return grp * SLOTS + c.slot < rows_valid; };
    auto load_rows = [&](int grel, float (&x)[R], float (&g)[R], bool full = false) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const bool ok = full || row_ok(grel + r);
            x[r] = buf_load<float>(x_rs, ok ? x_thr : kOob, (grel + r) * SLOTS * x_row);
            g[r] = buf_load<float>(g_rs, ok ? g_thr : kOob, (grel + r) * SLOTS * g_row);
        }
    };

    float nx[R], ngr[R];
    load_rows(0, nx, ngr);
    // FULL: the groups this iteration stores and the ones it prefetches exist for every row slot,
    // so no access needs its range mask: all but the last iterations of a workgroup.
    auto iteration = [&](int grel, auto FULL) {
        constexpr bool full = decltype(FULL)::value;
        float v[R], gv[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            v[r] = nx[r];
            gv[r] = ngr[r];
        }
        load_rows(grel + R, nx, ngr, full);
        float act[NS][R];
        static_for<0, NS>([&](auto S) {
            constexpr int s = S;
            constexpr int KQ = P::kind(s);
            if constexpr (P::layout(s) != P::layout_before(s)) transpose(v, P::layout(s));
#pragma unroll
            for (int r = 0; r < R; ++r) act[s][r] = v[r];
            if constexpr (s + 1 < NS) {
                if constexpr (KQ < 2 && R % 2 == 0) {
#pragma unroll
                    for (int r = 0; r < R; r += 2) fw4_pair_dpp<KQ>(v[r], v[r + 1], f.row[s]);
                } else {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        float y = f.row[s][0] * v[r];
                        y = fmaf(f.row[s][1], partner4<KQ, 1>(v[r], lane), y);
                        y = fmaf(f.row[s][2], partner4<KQ, 2>(v[r], lane), y);
                        y = fmaf(f.row[s][3], partner4<KQ, 3>(v[r], lane), y);
                        v[r] = y;
                    }
                }
            }
        });
        static_for<0, NS>([&](auto S) {
            constexpr int s = NS - 1 - S;
            constexpr int KQ = P::kind(s);
            if constexpr (P::layout(s) != P::layout_after(s)) transpose(gv, P::layout(s));
#pragma unroll
            for (int r = 0; r < R; ++r) {
                // one set of exchanges (of the gradient) serves both products: the thread sums
                // the COLUMN of d_twiddle that belongs to its element, dT[r ^ m][r] += g(partner m) * x,
                // and d_x[r] = sum_m T[r ^ m][r] g(partner m)
                const float xs = act[s][r];
                if constexpr (KQ < 2) {
                    bw4_dpp<KQ>(acc[s], gv[r], xs, f.colm[s]);
                } else {
                const float g1 = partner4<KQ, 1>(gv[r], lane);
                const float g2 = partner4<KQ, 2>(gv[r], lane);
                const float g3 = partner4<KQ, 3>(gv[r], lane);
                fmac_pinned(acc[s][0], gv[r], xs);
                fmac_pinned(acc[s][1], g1, xs);
                fmac_pinned(acc[s][2], g2, xs);
                fmac_pinned(acc[s][3], g3, xs);
                float d = f.colm[s][0] * gv[r];
                d = fmaf(f.colm[s][1], g1, d);
                d = fmaf(f.colm[s][2], g2, d);
                d = fmaf(f.colm[s][3], g3, d);
                gv[r] = d;
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

    int t2 = t;
    asm volatile("" : "+v"(t2));
    const FastCoords c2 = fast_coords<L>(t2);
    float *part = a.partial + ((int64_t)blockIdx.x * gridDim.y + stack) * NS * (4 * n);
    __shared__ float red[SLOTS > 1 ? 4 * 1024 : 1];
    static_for<0, NS>([&](auto S) {
        constexpr int s = S;
        constexpr int b = P::bit(s);
        constexpr int lay = P::layout(s);
        const int e = lay ? c2.eB : c2.eA;
        if constexpr (SLOTS == 1) {
            const int r = (e >> b) & 3;
            const int q = ((e >> (b + 2)) << b) | (e & ((1 << b) - 1));
            float *d = part + (int64_t)s * (4 * n) + q * 16 + r;
#pragma unroll
            for (int m = 0; m < 4; ++m) d[(r ^ m) * 4] = acc[s][m];
        } else {
            // add the row slots of this workgroup in ascending order, then one thread per entry
            __syncthreads();
#pragma unroll
            for (int m = 0; m < 4; ++m) red[(c2.slot * n + e) * 4 + m] = acc[s][m];
            __syncthreads();
            for (int o = t2; o < 4 * n; o += kFastThreads) {
                float sum = red[o];
                for (int sl = 1; sl < SLOTS; ++sl) sum += red[sl * 4 * n + o];
                const int eo = o >> 2, m = o & 3;
                const int r = (eo >> b) & 3;
                const int q = ((eo >> (b + 2)) << b) | (eo & ((1 << b) - 1));
                part[(int64_t)s * (4 * n) + q * 16 + (r ^ m) * 4 + r] = sum;
            }
        }
    });
}

}  // namespace bf
