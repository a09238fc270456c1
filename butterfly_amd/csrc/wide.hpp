// Forward kernel for rows of 2048 and 4096 elements: one whole block (log_n stages) per launch.
//
// A workgroup of 1024 threads owns one row at a time.  Thread t holds Q = n / 1024 elements,
// 1024 apart: element bits 10 and 11 live in the register index, the ten low bits are laid out
// over the workgroup exactly as in fast.hpp (layouts A and B, DPP / swizzle exchanges, LDS
// transposes between the layouts, the Q quarter-rows travelling as one 128-bit access).  A
// stage on bit 10 or 11 pairs two registers of the same thread: no exchange at all.  Every
// factor entry the thread needs (2 per stage and element) stays in registers for the whole
// launch, so a row is read once and written once per block instead of once per group of
// stages on the same side of bit 10.
//
// float rows are fetched straight into LDS two rows ahead (see load_row_to_lds in fast.hpp);
// complex64 (n = 2048 only: 4096 would need 192 factor registers) fetches into registers.
#pragma once

#include "fast.hpp"

namespace bf {

template <int L, bool INC>
struct WidePlan {
    static_assert(L == 11 || L == 12, "rows of 2048 or 4096 elements");
    static constexpr int NS = L;
    static constexpr int QB = L - 10, Q = 1 << QB;
    static constexpr int bit(int s) { return INC ? s : L - 1 - s; }
    // layout of the ten low bits while stage s runs: bits 6..9 need B, bits 0..3 need A,
    // anything else (4, 5 and the register bits) stays where the previous stage left the data
    static constexpr int layout(int s)
    {
        int cur = -1;
        for (int j = 0; j <= s; ++j) {
            const int b = bit(j);
            if (b >= 6 && b < 10) cur = 1;
            else if (b < 4) cur = 0;
        }
        if (cur >= 0) return cur;
        // nothing decided yet: take the layout of the first stage that cares
        for (int j = s + 1; j < NS; ++j) {
            const int b = bit(j);
            if (b >= 6 && b < 10) return 1;
            if (b < 4) return 0;
        }
        return 0;
    }
    static constexpr int layout_before(int s, int start) { return s == 0 ? start : layout(s - 1); }
    // 0..3 DPP pattern, 4 swizzle xor 16, 5 bpermute xor 32, 6 / 7 register bit 0 / 1
    static constexpr int kind(int s)
    {
        const int b = bit(s);
        return b >= 10 ? 6 + (b - 10) : (b >= 6 ? b - 6 : b);
    }
    static constexpr int transposes_before(int s, int start)
    {
        int c = 0, cur = start;
        for (int j = 0; j < s; ++j) {
            if (layout(j) != cur) { ++c; cur = layout(j); }
        }
        return c;
    }
    static constexpr int transposes_total(int start)
    {
        return transposes_before(NS, start) + (layout(NS - 1) != 0 ? 1 : 0);
    }
};

// FastFwArgs: ngroups = rows, groups_per_wg = rows per workgroup, tw_stage[s] = global stage
// number of local stage s (only the first entry is used: the stages of a block are consecutive).
template <typename T, int L, bool INC>
__global__ __launch_bounds__(kFastThreads) void wide_fw_kernel(FastFwArgs a)
{
    using P = WidePlan<L, INC>;
    constexpr int NS = P::NS, Q = P::Q;
    constexpr int EB = (int)sizeof(T);
    constexpr bool DIRECT = sizeof(T) == 4;
    constexpr int SF = DIRECT ? P::layout(0) : 0;
    constexpr int TT = P::transposes_total(SF);
    static_assert(TT >= 1, "a block always crosses between the layouts");
    __shared__ __align__(16) T lds[2 * Q * kFastRowWords];
    __shared__ float lds_rows[DIRECT ? 4 * Q * kFastRowWords : 1];  // 4 row slots of Q quarter-rows
    const int t = threadIdx.x;
    const int stack = blockIdx.y;
    const FastCoords c = fast_coords<10>(t);

    // factor entries: T[r][r] and T[r][1 - r] of the thread's output row, per stage and element
    T ta[NS][Q], tb[NS][Q];
    {
        const T *twp = reinterpret_cast<const T *>(a.tw) + stack * a.tw_stack_stride + a.tw_stage[0] * a.tw_stage_stride;
        static_for<0, NS>([&](auto S) {
            constexpr int s = S;
            constexpr int bit = P::bit(s);
            const int e10 = P::layout(s) ? c.eB : c.eA;
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const int e = (q << 10) | e10;
                const int r = (e >> bit) & 1;
                const int i = ((e >> (bit + 1)) << bit) | (e & ((1 << bit) - 1));
                const T *Tm = twp + s * a.tw_stage_stride + i * 4;
                // the row T[r][0], T[r][1] of the block is contiguous: one load (not at n = 4096,
                // where 96 entries nearly fill the registers and two plain loads per entry pair measure faster)
                if constexpr (sizeof(T) == 4 && NS * Q > 32) {
                    ta[s][q] = Tm[3 * r];
                    tb[s][q] = Tm[r + 1];
                } else if constexpr (sizeof(T) == 4) {
                    const float2 v = *reinterpret_cast<const float2 *>(Tm + 2 * r);
                    ta[s][q] = r ? v.y : v.x;
                    tb[s][q] = r ? v.x : v.y;
                    // (pinned: picked late, the loaded pair and the picks would both stay live)
                    asm volatile("" : "+v"(ta[s][q]), "+v"(tb[s][q]));
                } else {
                    const float4 v = *reinterpret_cast<const float4 *>(Tm + 2 * r);
                    ta[s][q] = r ? make_float2(v.z, v.w) : make_float2(v.x, v.y);
                    tb[s][q] = r ? make_float2(v.x, v.y) : make_float2(v.z, v.w);
                }
            }
        });
    }

    const int64_t r0 = (int64_t)blockIdx.x * a.groups_per_wg;
    const int64_t r1 = r0 + a.groups_per_wg < a.batch ? r0 + a.groups_per_wg : a.batch;
    const int nr = (int)(r1 - r0);
    const T *in_base = reinterpret_cast<const T *>(a.in) + r0 * a.in_view.sb + stack * a.in_view.ss;
    const __amdgpu_buffer_rsrc_t in_rs = make_rsrc(in_base);
    const __amdgpu_buffer_rsrc_t out_rs =
        make_rsrc(reinterpret_cast<T *>(a.out) + r0 * a.out_view.sb + stack * a.out_view.ss);
    const int in_row = (int)(a.in_view.sb * EB), out_row = (int)(a.out_view.sb * EB);
    int in_thr[Q], out_thr[Q], in_dma[Q];
    T bias[Q];
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int col = (q << 10) | c.eA;
        bias[q] = (a.bias && col < a.out_view.width)
                      ? reinterpret_cast<const T *>(a.bias)[stack * a.out_view.width + col]
                      : zero_of(T());
        const int64_t in_col = view_col(a.in_view, col), out_col = view_col(a.out_view, col);
        in_thr[q] = in_col >= 0 ? (int)(in_col * a.in_view.se * EB) : kOob;
        out_thr[q] = out_col >= 0 ? (int)(out_col * a.out_view.se * EB) : kOob;
        const int64_t in_col_d = view_col(a.in_view, (q << 10) | t);
        in_dma[q] = in_col_d >= 0 ? (int)(in_col_d * a.in_view.se * EB) : kOob;
    }
    const BufDesc in_desc = make_desc(in_base);
    const unsigned rows_addr = (unsigned)(unsigned long long)(LdsFloat *)lds_rows + (unsigned)(t >> 6) * 65 * 4;
    // row `row` of this workgroup -> slot (row & 3)
    auto fetch_row = [&](int row) {
#pragma unroll
        for (int q = 0; q < Q; ++q)
            load_row_to_lds(in_desc, rows_addr + ((row & 3) * Q + q) * kFastRowWords * 4, row < nr ? in_dma[q] : kOob,
                            row * in_row);
    };
    auto load_row = [&](int row, T (&v)[Q]) {
#pragma unroll
        for (int q = 0; q < Q; ++q) v[q] = buf_load<T>(in_rs, row < nr ? in_thr[q] : kOob, row * in_row);
    };

    T nxt[Q];
    if constexpr (DIRECT) {
        fetch_row(0);
        fetch_row(1);
        wait_rows_in_lds<0>();
        __syncthreads();
    } else {
        load_row(0, nxt);
        // stores that the range check discards: same history of loads and stores in front of the
        // first iteration as in front of every later one (see fast_fw_kernel)
#pragma unroll
        for (int q = 0; q < Q; ++q) buf_store(out_rs, kOob, EB * q, zero_of(T()));
    }
    for (int row = 0; row < nr; ++row) {
        T v[Q];
        // (the two halves of `lds` alternate across iteration boundaries too: see fast_fw_kernel)
        const int flip = (TT & 1) ? row & 1 : 0;
        if constexpr (DIRECT) {
            fetch_row(row + 2);
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const float x = lds_rows[((row & 3) * Q + q) * kFastRowWords + (SF ? c.fB : c.fA)];
                v[q] = x;
            }
        } else {
#pragma unroll
            for (int q = 0; q < Q; ++q) v[q] = nxt[q];
            load_row(row + 1, nxt);
        }
        // Before the last barrier of the iteration each wavefront waits for the quarter-rows it
        // requested one iteration ago (younger: that iteration's Q stores, this one's Q requests).
        static_for<0, NS>([&](auto S) {
            constexpr int s = S;
            constexpr int K = P::kind(s);
            if constexpr (P::layout(s) != P::layout_before(s, SF)) {
                constexpr int nth = P::transposes_before(s, SF);
                constexpr int to_b = P::layout(s);
                T *buf = lds + ((nth + flip) & 1) * Q * kFastRowWords;
                const int wr = to_b ? c.fA : c.fB, rd = to_b ? c.fB : c.fA;
                transpose_rows<T, Q, DIRECT && nth + 1 == TT, 2 * Q>(buf, wr, rd, v);
            }
            if constexpr (K < 6) {
#pragma unroll
                for (int q = 0; q < Q; ++q) v[q] = fw_product<K>(v[q], ta[s][q], tb[s][q], c.bperm_addr);
            } else {
                constexpr int m = 1 << (K - 6);
                T w[Q];
#pragma unroll
                for (int q = 0; q < Q; ++q) w[q] = mac(mul(ta[s][q], v[q]), tb[s][q], v[q ^ m]);
#pragma unroll
                for (int q = 0; q < Q; ++q) v[q] = w[q];
            }
        });
        if constexpr (P::layout(NS - 1) != 0) {
            constexpr int nth = P::transposes_before(NS, SF);
            T *buf = lds + ((nth + flip) & 1) * Q * kFastRowWords;
            transpose_rows<T, Q, DIRECT, 2 * Q>(buf, c.fB, c.fA, v);
        }
#pragma unroll
        for (int q = 0; q < Q; ++q) buf_store(out_rs, row < nr ? out_thr[q] : kOob, row * out_row, add(v[q], bias[q]));
    }
    if constexpr (DIRECT) wait_rows_in_lds<0>();  // requests past the last row (they fetch nothing)
}

}  // namespace bf
