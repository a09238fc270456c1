// Twiddle-stationary kernels for base-2 rows of n <= 1024, float and complex64.
//
// One workgroup of 1024 threads (16 wavefronts) owns a group of 1024 / n rows at a time and
// keeps every 2x2 factor it needs in registers for the whole launch: thread t holds one
// element per row and, per stage, the two factor entries of its own output row.  Rows
// stream through; HBM sees each row once in and once out.
//
// A stage pairs element e with e ^ (1 << bit).  Where the partner lives decides the
// exchange:
//   * lanes of one 16-lane row:   DPP (quad_perm / row_half_mirror / row_mirror), fused
//     into the multiply.  The 16 lanes of a row hold element low bits phi4(lane), a
//     GF(2)-linear relabelling chosen so that XOR by element bit 0, 1, 2, 3 is exactly one
//     of those four DPP patterns.
//   * lane bits 4 and 5:          ds_swizzle (xor 16) and ds_bpermute (xor 32); these use the
//     LDS crossbar, not the vector ALU.
//   * across wavefronts (element bits >= 6): the workgroup transposes through LDS into a
//     second layout ("B") in which those bits sit on the DPP lanes and the low bits sit on
//     the wavefront index; it transposes back ("A") when low bits are needed again.  A
//     10-stage block costs two transposes, not four exchanges.
//
// The backward kernel replays the forward stages keeping every stage input in registers,
// then walks back accumulating d_twiddle in registers across all rows of the workgroup;
// partial sums are written once at the end and reduced by reduce_partials_kernel in a
// fixed order (no atomics).
#pragma once

#include <type_traits>

#include "common.hpp"

namespace bf {

constexpr int kFastThreads = 1024;
constexpr int kFastRowWords = 1024 + 16;  // one LDS row: 1024 words + 1 pad word per 64

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

__host__ __device__ constexpr int phi4(int l)
{
    return ((l & 1) ? 1 : 0) ^ ((l & 2) ? 2 : 0) ^ ((l & 4) ? 7 : 0) ^ ((l & 8) ? 12 : 0);
}

// What the kernels ask of a plan, derived from its stage -> bit map (D::bit, D::NS, D::LOG).
template <typename D>
struct PlanOps {
    // layout (0 = A, 1 = B) in which stage s runs: bits >= 6 need B, bits < NSWAP need A,
    // anything else stays where the previous stage left the data.
    static constexpr int layout(int s)
    {
        int cur = 0;
        for (int j = 0; j <= s; ++j) {
            const int b = D::bit(j);
            if (b >= 6) cur = 1;
            else if (b < D::NSWAP) cur = 0;
        }
        return cur;
    }
    // (`start`: layout the walk is in before its first stage; A when rows arrive in registers)
    static constexpr int layout_before(int s, int start = 0) { return s == 0 ? start : layout(s - 1); }
    // exchange kind: 0..3 DPP pattern for phi bit, 4 swizzle xor 16, 5 bpermute xor 32
    static constexpr int kind(int s)
    {
        const int b = D::bit(s);
        return b >= 6 ? b - 6 : b;
    }
    // LDS transposes performed before stage s of a forward walk (for buffer parity)
    static constexpr int fw_transposes_before(int s, int start = 0)
    {
        int c = 0, cur = start;
        for (int j = 0; j < s; ++j) {
            if (layout(j) != cur) { ++c; cur = layout(j); }
        }
        return c;
    }
    static constexpr int fw_transposes_total(int start = 0)
    {
        int c = fw_transposes_before(D::NS, start);
        return c + (layout(D::NS - 1) != 0 ? 1 : 0);
    }
};

// NB whole blocks of a row (or 1024-element chunk of a row) of 2^L elements.
template <int L, int NB, bool INC>
struct FastPlan : PlanOps<FastPlan<L, NB, INC>> {
    static constexpr int LOG = L;
    static constexpr int NS = L * NB;
    static constexpr int NSWAP = L > 6 ? L - 6 : 0;  // element bits exchanged between layouts
    static constexpr int SLOTS = 1024 >> L;          // rows a workgroup holds at once

    // element bit paired by stage s
    static constexpr int bit(int s)
    {
        const int k = s / L, idx = s % L;
        const bool inc = INC != ((k & 1) != 0);
        return inc ? idx : L - 1 - idx;
    }
    // column of the full row behind element e of chunk `tile`; pair index (in a stage's factor
    // slice) of the pair that element belongs to = pair_base(tile) + pair_index(...)
    __device__ static __forceinline__ int column(int tile, int e, int) { return (tile << L) + e; }
    __device__ static __forceinline__ int64_t pair_base(int tile) { return (int64_t)tile * (1 << (L - 1)); }
    __device__ static __forceinline__ int pair_index(int, int e, int s_bit, int)
    {
        return ((e >> (s_bit + 1)) << s_bit) | (e & ((1 << s_bit) - 1));
    }
};

// The stages on H adjacent high bits [lb, lb + H) of a long row, run by the same kernels: a
// workgroup takes a tile of 1024 elements made of 2^(10 - H) consecutive elements (virtual bits
// 0 .. 9 - H) for each of the 2^H settings of the high bits (virtual bits 10 - H .. 9); the
// tile index enumerates all other bits.  MODE 0: one sweep up (lb, lb + 1, ...), 1: one sweep
// down, 2: up then down (two blocks meeting in the row's top bits).
template <int H, int MODE>
struct SpanPlan : PlanOps<SpanPlan<H, MODE>> {
    static_assert(H >= 1 && H <= 6, "tiles keep at least 16 consecutive elements");
    static constexpr int LOG = 10;
    static constexpr int NS = MODE == 2 ? 2 * H : H;
    static constexpr int NSWAP = 4;
    static constexpr int SLOTS = 1;
    static constexpr int bit(int s)
    {
        const bool up = MODE == 0 || (MODE == 2 && s < H);
        const int idx = s % H;
        return 10 - H + (up ? idx : H - 1 - idx);
    }
    __device__ static __forceinline__ int column(int tile, int e, int lb)
    {
        const int cb = lb - (10 - H);   // tile bits that sit below the span
        const int lo = e & ((1 << (10 - H)) - 1), gp = e >> (10 - H);
        return lo | ((tile & ((1 << cb) - 1)) << (10 - H)) | (gp << lb) | ((tile >> cb) << (lb + H));
    }
    __device__ static __forceinline__ int64_t pair_base(int) { return 0; }
    __device__ static __forceinline__ int pair_index(int tile, int e, int s_bit, int lb)
    {
        const int col = column(tile, e, lb);
        const int pb = lb + s_bit - (10 - H);
        return ((col >> (pb + 1)) << pb) | (col & ((1 << pb) - 1));
    }
};

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL,
                                                                  0xf, 0xf, true));
}

// Value of `v` held by the partner thread of an exchange of kind K.
template <int K>
__device__ __forceinline__ float partner(float v, int bperm_addr)
{
    if constexpr (K == 0) return dpp_move<0xB1>(v);        // quad_perm [1,0,3,2]
    else if constexpr (K == 1) return dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
    else if constexpr (K == 2) return dpp_move<0x141>(v);  // row_half_mirror
    else if constexpr (K == 3) return dpp_move<0x140>(v);  // row_mirror
    else if constexpr (K == 4)
        return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
    else
        return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(bperm_addr, __builtin_bit_cast(int, v)));
}

template <int K>
__device__ __forceinline__ float2 partner(float2 v, int bperm_addr)
{
    return make_float2(partner<K>(v.x, bperm_addr), partner<K>(v.y, bperm_addr));
}

// acc += g * x, pinned where it is written: the accumulators live across the whole row loop
// and the compiler otherwise sinks these to the end of the iteration, which keeps every
// stage's operands alive and overflows the register file.
__device__ __forceinline__ void fmac_pinned(float &acc, float g, float x)
{
    asm volatile("v_fmac_f32_e32 %0, %1, %2" : "+v"(acc) : "v"(g), "v"(x));
}

// acc -= g * x, pinned
__device__ __forceinline__ void fnmac_pinned(float &acc, float g, float x)
{
    asm volatile("v_fma_f32 %0, -%1, %2, %0" : "+v"(acc) : "v"(g), "v"(x));
}

// acc += g * conj(x), pinned
__device__ __forceinline__ void fmac_pinned(float2 &acc, float2 g, float2 x)
{
    fmac_pinned(acc.x, g.x, x.x);
    fmac_pinned(acc.x, g.y, x.y);
    fmac_pinned(acc.y, g.y, x.x);
    fnmac_pinned(acc.y, g.x, x.y);
}

// The three products of a backward stage, for one element and exchange kind K.  With p the
// partner element of the pair and T the 2x2 factor:
//   self  += g * conj(x)                 dT[me][me]
//   cross += g_p * conj(x)               dT[p][me]: the gradient of the partner's output row
//                                        times this thread's own input
//   g     <- conj(T[me][me]) * g + conj(T[p][me]) * g_p
// so one exchange (of g) serves both, and the thread needs the factor column of its element
// (ta = T[me][me], tc = T[p][me]) rather than the row the forward stage uses.
template <int K, typename T>
__device__ __forceinline__ void bw_products(T &self, T &cross, T &g, T x, T ta, T tc, int bperm_addr)
{
    const T gp = partner<K>(g, bperm_addr);
    fmac_pinned(self, g, x);
    fmac_pinned(cross, gp, x);
    g = macc(mul(conj_of(ta), g), tc, gp);
}

// float and a DPP exchange: both uses of the partner's g read it through the DPP operand of the
// multiply-add itself, so no move materialises it.  The two plain instructions in front keep
// the two wait states a DPP read needs after a VALU write of the same register, whatever the
// compiler schedules in front of the block.
#define BF_BW_PRODUCTS_DPP(CTRL)                                                                   \
    asm volatile("v_fmac_f32_e32 %0, %3, %4\n\t"                                                   \
                 "v_mul_f32_e32 %2, %5, %3\n\t"                                                    \
                 "v_fmac_f32_dpp %1, %3, %4 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"  \
                 "v_fmac_f32_dpp %2, %3, %6 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1"       \
                 : "+v"(self), "+v"(cross), "=&v"(m)                                               \
                 : "v"(g), "v"(x), "v"(ta), "v"(tc))

template <int K>
__device__ __forceinline__ void bw_products_dpp(float &self, float &cross, float &g, float x, float ta, float tc)
{
    static_assert(K >= 0 && K < 4, "DPP exchange kinds only");
    float m;
    if constexpr (K == 0) BF_BW_PRODUCTS_DPP("quad_perm:[1,0,3,2]");
    else if constexpr (K == 1) BF_BW_PRODUCTS_DPP("quad_perm:[2,3,0,1]");
    else if constexpr (K == 2) BF_BW_PRODUCTS_DPP("row_half_mirror");
    else BF_BW_PRODUCTS_DPP("row_mirror");
    g = m;
}
#undef BF_BW_PRODUCTS_DPP

template <int K>
__device__ __forceinline__ void bw_products(float &self, float &cross, float &g, float x, float ta, float tc,
                                            int bperm_addr)
{
    if constexpr (K < 4) {
        bw_products_dpp<K>(self, cross, g, x, ta, tc);
    } else {
        const float gp = partner<K>(g, bperm_addr);
        fmac_pinned(self, g, x);
        fmac_pinned(cross, gp, x);
        g = fmaf(tc, gp, ta * g);
    }
}

// The same stage written with the factor row (ta = T[me][me], tb = T[me][p]) that the forward
// replay holds anyway: two exchanges, but no third factor entry to keep.
//   cross += g * conj(x_p)               dT[me][p]
//   g     <- conj(ta) * g + (conj(tb) * g formed by the partner from its own tb)
template <int K, typename T>
__device__ __forceinline__ void bw_products_row(T &self, T &cross, T &g, T x, T ta, T tb, int bperm_addr)
{
    fmac_pinned(self, g, x);
    fmac_pinned(cross, g, partner<K>(x, bperm_addr));
    const T m = mul(conj_of(tb), g);
    g = add(mul(conj_of(ta), g), partner<K>(m, bperm_addr));
}

// Forward stage for one element: ta * v + tb * (v of the partner).
template <int K>
__device__ __forceinline__ float fw_product(float v, float ta, float tb, int bperm_addr)
{
    const float p = tb * partner<K>(v, bperm_addr);
    return fmaf(ta, v, p);
}

// The same product pinned where it is written, for the backward kernel's replay walk: that
// kernel issues the stages of its two walks in a chosen order (BwPipe::order), which only holds
// if the compiler cannot slide one walk's arithmetic past the other's.  DPP kinds only; the
// plain multiply and the s_nop give the two wait states the DPP read of v needs after a write.
#define BF_FW_PRODUCT_DPP(CTRL)                                                                       \
    asm volatile("v_mul_f32_e32 %0, %2, %1\n\t"                                                       \
                 "s_nop 0\n\t"                                                                        \
                 "v_fmac_f32_dpp %0, %1, %3 " CTRL " row_mask:0xf bank_mask:0xf bound_ctrl:1"          \
                 : "=&v"(out)                                                                         \
                 : "v"(v), "v"(ta), "v"(tb))

template <int K>
__device__ __forceinline__ float fw_product_pinned(float v, float ta, float tb)
{
    static_assert(K >= 0 && K < 4, "DPP exchange kinds only");
    float out;
    if constexpr (K == 0) BF_FW_PRODUCT_DPP("quad_perm:[1,0,3,2]");
    else if constexpr (K == 1) BF_FW_PRODUCT_DPP("quad_perm:[2,3,0,1]");
    else if constexpr (K == 2) BF_FW_PRODUCT_DPP("row_half_mirror");
    else BF_FW_PRODUCT_DPP("row_mirror");
    return out;
}
#undef BF_FW_PRODUCT_DPP

template <int K>
__device__ __forceinline__ float2 fw_product(float2 v, float2 ta, float2 tb, int bperm_addr)
{
    return mac(mul(ta, v), tb, partner<K>(v, bperm_addr));
}

// The same stage in two halves, for exchanges that take an LDS round trip: the partner's value is
// requested first and the arithmetic follows once other work has covered the wait.
__device__ __forceinline__ float fw_finish(float v, float ta, float tb, float pv)
{
    float out;
    asm volatile("v_mul_f32_e32 %0, %3, %4\n\t"
                 "v_fmac_f32_e32 %0, %2, %1"
                 : "=&v"(out)
                 : "v"(v), "v"(ta), "v"(tb), "v"(pv));
    return out;
}
__device__ __forceinline__ float2 fw_finish(float2 v, float2 ta, float2 tb, float2 pv) { return mac(mul(ta, v), tb, pv); }

template <typename T>
__device__ __forceinline__ void bw_finish(T &self, T &cross, T &g, T x, T ta, T tc, T gp)
{
    fmac_pinned(self, g, x);
    fmac_pinned(cross, gp, x);
    g = macc(mul(conj_of(ta), g), tc, gp);
}
__device__ __forceinline__ void bw_finish(float &self, float &cross, float &g, float x, float ta, float tc, float gp)
{
    fmac_pinned(self, g, x);
    fmac_pinned(cross, gp, x);
    g = fmaf(tc, gp, ta * g);
}

// row form: the partner's x and the partner's conj(tb) * g are both needed
template <typename T>
__device__ __forceinline__ void bw_finish_row(T &self, T &cross, T &g, T x, T ta, T px, T pm)
{
    fmac_pinned(self, g, x);
    fmac_pinned(cross, g, px);
    g = add(mul(conj_of(ta), g), pm);
}

// Per-thread coordinates in both layouts.
struct FastCoords {
    int eA, eB;    // element index in layout A / B
    int fA, fB;    // padded LDS word offsets of those elements (slot included)
    int slot;      // which of the workgroup's rows this thread works on
    int bperm_addr;
};

template <int L>
__device__ __forceinline__ FastCoords fast_coords(int t)
{
    constexpr int NSWAP = L > 6 ? L - 6 : 0;
    constexpr int m = (1 << NSWAP) - 1;
    const int v4 = phi4(t & 15), h = (t >> 4) & 3, w = t >> 6;
    const int VA = v4 | (h << 4) | (w << 6);
    const int VB = ((v4 & ~m) | (w & m)) | (h << 4) | (((w & ~m) | (v4 & m)) << 6);
    FastCoords c;
    c.eA = VA & ((1 << L) - 1);
    c.eB = VB & ((1 << L) - 1);
    c.fA = VA + (VA >> 6);
    c.fB = VB + (VB >> 6);
    c.slot = VA >> L;
    c.bperm_addr = ((t & 63) ^ 32) << 2;
    return c;
}

// ---- global memory through buffer resources ---------------------------------------------------
// Every operand is addressed as base + 32-bit byte offset through a raw buffer resource whose
// base is the first row this workgroup touches (stack offset folded in).  An access that must
// not happen (row past the batch, column past the operand width) uses the offset kOob, which
// lies outside the resource's range: the hardware returns zero for such a load and drops
// such a store.  No branches, so the row loop is straight-line code and the prefetch of the
// next rows really overlaps the stages of the current ones.  The host guarantees that all
// valid offsets of one workgroup stay below 2 GiB.
constexpr int kOob = (int)0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)0x80000000u, 0x00020000);
}

// voff: per-thread byte offset (range-checked); soff: wave-uniform byte offset added on top.
template <typename T>
__device__ __forceinline__ T buf_load(__amdgpu_buffer_rsrc_t r, int voff, int soff)
{
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
    } else {
        typedef unsigned v2u __attribute__((ext_vector_type(2)));
        // (bit-casting a vector element in place reads element 0 for both: go through scalars)
        const v2u raw = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0);
        const unsigned lo = raw.x, hi = raw.y;
        return make_float2(__uint_as_float(lo), __uint_as_float(hi));
    }
}

__device__ __forceinline__ void buf_store(__amdgpu_buffer_rsrc_t r, int voff, int soff, float v)
{
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, voff, soff, 0);
}

__device__ __forceinline__ void buf_store(__amdgpu_buffer_rsrc_t r, int voff, int soff, float2 v)
{
    typedef unsigned v2u __attribute__((ext_vector_type(2)));
    v2u raw;
    const float fx = v.x, fy = v.y;
    raw.x = __float_as_uint(fx);
    raw.y = __float_as_uint(fy);
    __builtin_amdgcn_raw_buffer_store_b64(raw, r, voff, soff, 0);
}

// ---- rows fetched straight into LDS -----------------------------------------------------------
// A buffer load with the LDS modifier writes the dword each lane fetches to LDS at
// M0 + 4 * lane: no register holds the row while it is in flight, and the thread that later
// needs an element reads it from LDS in whatever layout its first stage wants.  Lanes whose
// offset is out of range write zero.  The compiler does not see these loads (it would wait
// for them at the next LDS access of any kind); the kernel waits for them itself.
typedef int BufDesc __attribute__((ext_vector_type(4)));

__device__ __forceinline__ BufDesc make_desc(const void *base)
{
    const unsigned long long a = (unsigned long long)base;
    BufDesc d;
    d.x = (int)(unsigned)a;
    d.y = (int)((a >> 32) & 0xffff);
    d.z = (int)0x80000000u;
    d.w = 0x00020000;
    return d;
}

// lds_addr: LDS byte address the wavefront's 64 dwords start at (wave-uniform)
__device__ __forceinline__ void load_row_to_lds(BufDesc desc, unsigned lds_addr, int voff, int soff)
{
    int keep_m0;
    asm volatile("s_mov_b32 %0, m0\n\t"
                 "s_mov_b32 m0, %1\n\t"
                 "s_nop 0\n\t"
                 "buffer_load_dword %2, %3, %4 offen lds\n\t"
                 "s_mov_b32 m0, %0"
                 : "=&s"(keep_m0)
                 : "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(desc), "s"(soff)
                 : "memory");
}

// BF_SAFE_WAITS (a build switch, off in the shipped library): every counted wait becomes "wait for
// all of this wavefront's memory operations".  Results must be the same with and without it; a
// difference would mean a count is wrong.  The row pipelines then also wait for their own stores,
// so the kernels run slower.
template <int N>
__device__ __forceinline__ void wait_rows_in_lds()
{
#ifdef BF_SAFE_WAITS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#else
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
#endif
}

typedef __attribute__((address_space(3))) float LdsFloat;

constexpr int kFastMaxStages = 20;

// Rows longer than 1024 are handled as independent 1024-element chunks (blockIdx.z) for the
// stages that pair bits below 10: chunk c of stage s uses the factor slice starting at pair
// c * 512, and its d_twiddle sums land at the same place in the partial slice.
// All element counts and strides below are in scalars of the kernel's type (float or
// complex64).
struct FastFwArgs {
    const void *tw;            // twiddle tensor, stack 0
    int64_t tw_stack_stride;
    int64_t tw_stage_stride;   // scalars between consecutive stages: (n_full / 2) * 4
    int tw_stage[kFastMaxStages];  // global stage number of every local stage
    const void *in;
    View in_view;
    void *out;
    View out_view;
    int64_t batch;
    int64_t ngroups;           // ceil(batch / SLOTS)
    int64_t groups_per_wg;
    const void *bias;          // NULL, or (S, out_view.width) dense: added to every output row
    int low_bits;              // SpanPlan passes: position of the lowest high bit of the span
};

// (lets the float-only branch of load_factors compile for complex64, where it is never taken)
template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) { return v; }
template <>
__device__ __forceinline__ float2 from_float<float2>(float v) { return make_float2(v, 0.0f); }

// Loads the factor entries each thread needs for every stage: its row (ta, tb) and, for the
// backward kernel, the off-diagonal entry of its column (tc).
// `loaded(S)` runs right after stage S has its entries (the backward kernel parks some of them in
// LDS there, which frees their registers before the next blocks arrive).
template <typename T, typename P, typename F>
__device__ __forceinline__ void load_factors(const void *tw, int64_t stack_off, int64_t stage_stride,
                                             const int (&tw_stage)[kFastMaxStages], int chunk, int low_bits,
                                             const FastCoords &c, T (&ta)[P::NS], T (&tb)[P::NS],
                                             T (&tc)[P::NS], bool want_tc, F &&loaded)
{
    const T *twp = reinterpret_cast<const T *>(tw) + stack_off + P::pair_base(chunk) * 4;
    static_for<0, P::NS>([&](auto S) {
        constexpr int s = S;
        constexpr int bit = P::bit(s);
        constexpr int lay = P::layout(s);
        const int e = lay ? c.eB : c.eA;
        const int r = (e >> bit) & 1;
        const int i = P::pair_index(chunk, e, bit, low_bits);
        const T *Tm = twp + tw_stage[s] * stage_stride + i * 4;
        if (sizeof(T) == 4 && want_tc) {
            // float, all three entries: the whole 2x2 block as one 16-byte load (the factor
            // tensor is dense and 16-byte aligned), then a pick by r -- a third of the load
            // instructions, each fully used, instead of three 4-byte loads that each drag a
            // 16-byte-strided set of cache lines through L1.  (Two entries, or complex64 ones,
            // are faster loaded one by one.)
            const float4 b = *reinterpret_cast<const float4 *>(Tm);
            float pa = r ? b.w : b.x;   // T[r][r]
            float pb = r ? b.z : b.y;   // T[r][1 - r]
            float pc = r ? b.y : b.z;   // T[1 - r][r]
            // pin the picks here: left alone, the compiler keeps the whole blocks (twice the
            // registers) and picks at the first use
            asm volatile("" : "+v"(pa), "+v"(pb), "+v"(pc));
            ta[s] = from_float<T>(pa);
            tb[s] = from_float<T>(pb);
            tc[s] = from_float<T>(pc);
        } else {
            // the thread's row of the block, T[r][0] and T[r][1], is contiguous: one load
            if constexpr (sizeof(T) == 4) {
                const float2 v = *reinterpret_cast<const float2 *>(Tm + 2 * r);
                ta[s] = r ? v.y : v.x;   // T[r][r]
                tb[s] = r ? v.x : v.y;   // T[r][1 - r]
            } else {
                const float4 v = *reinterpret_cast<const float4 *>(Tm + 2 * r);
                ta[s] = r ? make_float2(v.z, v.w) : make_float2(v.x, v.y);
                tb[s] = r ? make_float2(v.x, v.y) : make_float2(v.z, v.w);
            }
            if (want_tc) tc[s] = Tm[2 - r];   // T[1 - r][r]
        }
        loaded(S);
        if constexpr (P::NS > 10 && s % 5 == 4) {
            if (sizeof(T) == 4 && want_tc) __builtin_amdgcn_sched_barrier(0);
        }
    });
}

template <typename T, typename P>
__device__ __forceinline__ void load_factors(const void *tw, int64_t stack_off, int64_t stage_stride,
                                             const int (&tw_stage)[kFastMaxStages], int chunk, int low_bits,
                                             const FastCoords &c, T (&ta)[P::NS], T (&tb)[P::NS],
                                             T (&tc)[P::NS], bool want_tc)
{
    load_factors<T, P>(tw, stack_off, stage_stride, tw_stage, chunk, low_bits, c, ta, tb, tc, want_tc, [](auto) {});
}

// float factors, loaded so that every request of a wavefront covers consecutive pairs.  A stage
// that runs in layout B spreads a wavefront's elements 16 apart, so asking for "my element's
// factor row" there touches 32 different cache lines per request, sixteen wavefronts after one
// another (measured: the factor loads of a two-block kernel took 13 thousand cycles).  Instead
// every thread asks, for every stage, for the factor row of its layout-A element -- consecutive
// lanes, consecutive pairs, 512 contiguous bytes per request -- and the rows of the layout-B stages
// then travel through LDS to the threads that hold those elements in layout B (the same
// transposition the rows themselves take; `batch` stages share a barrier).  The third entry the
// backward kernel keeps, T[1 - r][r], is the partner's off-diagonal entry: one register exchange.
// `scratch`: LDS, `batch` buffers of kFastRowWords float2; the caller may alias it with memory
// that `loaded` writes (a barrier separates the two).
template <typename P, typename F>
__device__ __forceinline__ void load_factors_coalesced(const void *tw, int64_t stack_off, int64_t stage_stride,
                                                       const int (&tw_stage)[kFastMaxStages], int chunk, int low_bits,
                                                       const FastCoords &c, float (&ta)[P::NS], float (&tb)[P::NS],
                                                       float (&tc)[P::NS], bool want_tc, float2 *scratch, int batch,
                                                       F &&loaded)
{
    constexpr int NS = P::NS;
    const float *twp = reinterpret_cast<const float *>(tw) + stack_off + P::pair_base(chunk) * 4;
    float2 row[NS];   // (T[r][r], T[r][1 - r]) of the element this thread holds in layout A
    static_for<0, NS>([&](auto S) {
        constexpr int s = S;
        constexpr int bit = P::bit(s);
        const int r = (c.eA >> bit) & 1;
        const int i = P::pair_index(chunk, c.eA, bit, low_bits);
        const float2 v = *reinterpret_cast<const float2 *>(twp + tw_stage[s] * stage_stride + i * 4 + 2 * r);
        row[s] = r ? make_float2(v.y, v.x) : v;
    });
    // stages that run in layout B, in order
    struct Late { int n; int s[NS]; };
    constexpr Late late = [] {
        Late l{};
        for (int s = 0; s < NS; ++s)
            if (P::layout(s) != 0) l.s[l.n++] = s;
        return l;
    }();
    if constexpr (late.n > 0) {
        for (int j0 = 0; j0 < late.n; j0 += batch) {
            if (j0 > 0) __syncthreads();   // the previous batch has been read
            static_for<0, late.n>([&](auto J) {
                if (J >= j0 && J < j0 + batch) scratch[(J - j0) * kFastRowWords + c.fA] = row[late.s[J]];
            });
            __syncthreads();
            static_for<0, late.n>([&](auto J) {
                if (J >= j0 && J < j0 + batch) row[late.s[J]] = scratch[(J - j0) * kFastRowWords + c.fB];
            });
        }
        __syncthreads();   // `loaded` may write where the scratch buffers are
    }
    static_for<0, NS>([&](auto S) {
        constexpr int s = S;
        ta[s] = row[s].x;
        tb[s] = row[s].y;
        if (want_tc) tc[s] = partner<P::kind(s)>(tb[s], c.bperm_addr);
        loaded(S);
    });
}

// Moves the R values a thread holds (one per row in flight) through LDS: written at word
// `wr`, read back at word `rd` after a barrier.  Four float rows travel as one 128-bit access.
// WAIT: the wavefront first waits for the rows it has requested into LDS (all but the YOUNGER
// newest memory operations), so that the barrier also publishes those.
template <typename T, int R, bool WAIT = false, int YOUNGER = 0>
__device__ __forceinline__ void transpose_rows(T *buf, int wr, int rd, T (&v)[R])
{
    if constexpr (sizeof(T) == 4 && R % 4 == 0) {
        float4 *b4 = reinterpret_cast<float4 *>(buf);
#pragma unroll
        for (int r = 0; r < R; r += 4)
            b4[(r / 4) * kFastRowWords + wr] = make_float4(v[r], v[r + 1], v[r + 2], v[r + 3]);
        if constexpr (WAIT) wait_rows_in_lds<YOUNGER>();
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; r += 4) {
            const float4 q = b4[(r / 4) * kFastRowWords + rd];
            v[r] = q.x;
            v[r + 1] = q.y;
            v[r + 2] = q.z;
            v[r + 3] = q.w;
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) buf[r * kFastRowWords + wr] = v[r];
        if constexpr (WAIT) wait_rows_in_lds<YOUNGER>();
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r) v[r] = buf[r * kFastRowWords + rd];
    }
}

// The hand-counted waits, checked against the order in which the kernels issue their own
// vector-memory operations.  Counters complete in issue order, so `s_waitcnt vmcnt(N)` waits for
// everything but the N newest operations; N must be the number of operations issued between the
// requests for the rows awaited and the wait.
//
// Backward kernel: walk from the top of the iteration in which the rows that the next iteration
// reads are requested (AHEAD - 1 iterations before the one that waits) to the wait in front of
// the last barrier of the waiting iteration.
template <typename Q, int R, int AHEAD>
constexpr int bw_operations_behind_awaited_rows()
{
    int younger = 0;
    for (int j = 1 - AHEAD; j <= 0; ++j) {               // iteration, relative to the waiting one
        if (j != 1 - AHEAD) younger += 2 * R;            // top: R requests for x, R for the gradient
        for (int k = 1; k <= Q::K; ++k) {
            if (k == Q::K && j == 0) return younger;     // the wait, in front of barrier K
            if (Q::DEFER && k == 1) younger += R;        // deferred stores, right behind barrier 1
        }
        if (Q::K == 0 && j == 0) return younger;         // no barriers: the wait precedes the stores
        if (!Q::DEFER) younger += R;                     // stores closing the iteration
    }
    return -1;
}

// Forward kernel: the rows of the next iteration are requested during the previous one (request
// r in phase r mod (TT + 1), phase p behind barrier p; TWO_SETS: behind barrier 1 + r mod TT,
// none at the top); behind the last of them come that iteration's R stores and the waiting
// iteration's requests of the phases in front of its last barrier.
template <int R, int TT, bool TWO_SETS>
constexpr int fw_operations_behind_awaited_rows()
{
    int younger = R;                                       // the stores closing the previous iteration
    // the waiting iteration's own requests up to the wait, which stands in front of barrier TT
    // (in front of the stores when there is no barrier)
    for (int phase = 0; phase < (TT == 0 ? 1 : TT); ++phase)
        for (int r = 0; r < R; ++r) {
            const int at = TWO_SETS ? 1 + r % (TT > 0 ? TT : 1) : r % (TT + 1);
            younger += at == phase ? 1 : 0;
        }
    return younger;
}

// P: FastPlan<L, NB, INC> (whole blocks of a row or chunk) or SpanPlan<H, MODE> (a span of high
// bits of a long row; gridDim.z = n / 1024 tiles).
// WAVES: wavefronts per SIMD the kernel is compiled for.  8 keeps it within 64 registers, so that
// two workgroups fit a compute unit (see TWO_SETS for the LDS side); the host asks for that where
// two resident workgroups pay off.
template <typename T, typename P, int R, int WAVES = 4>
__global__ __launch_bounds__(kFastThreads, WAVES) void fast_fw_kernel(FastFwArgs a)
{
    constexpr int L = P::LOG;
    constexpr int n = 1 << L, NS = P::NS, SLOTS = P::SLOTS;
    constexpr int EB = (int)sizeof(T);
    // float rows are fetched straight into LDS, up to two iterations (2 R row groups) ahead, and
    // the walk starts in the layout of its first stage; complex64 rows arrive in registers, layout A
    constexpr bool DIRECT = sizeof(T) == 4;
    constexpr int SF = DIRECT ? P::layout(0) : 0;
    constexpr int TT = P::fw_transposes_total(SF);  // barriers per iteration
    __shared__ __align__(16) T lds[TT > 0 ? 2 * R * kFastRowWords : 1];
    // Row slots in LDS: four sets of R, an iteration's requests starting at its top, two
    // iterations ahead.  The variant compiled for two workgroups per compute unit has room for two
    // sets only (64 KiB with the transpose buffers at R = 4): a set is read at the top of its
    // iteration and nowhere else, so the requests for the iteration after next refill it as soon as
    // the first barrier has passed.  (One workgroup per unit keeps the longer lead: a memory-bound
    // pass over one block is 6 % slower with two sets.)
    constexpr bool TWO_SETS = TT >= 1 && WAVES >= 8;
    constexpr int SETS = TWO_SETS ? 2 : 4;
    __shared__ float lds_rows[DIRECT ? SETS * R * kFastRowWords : 1];
    const int t = threadIdx.x;
    const int stack = blockIdx.y;
    const int chunk = blockIdx.z;
    const FastCoords c = fast_coords<L>(t);
    const int col = P::column(chunk, c.eA, a.low_bits);  // column of this thread's element in the full row

    const int64_t g0 = (int64_t)blockIdx.x * a.groups_per_wg;
    const int64_t g1 = g0 + a.groups_per_wg < a.ngroups ? g0 + a.groups_per_wg : a.ngroups;
    const int ng = (int)(g1 - g0);
    const int64_t row_end = g1 * SLOTS < a.batch ? g1 * SLOTS : a.batch;
    const int rows_valid = (int)(row_end - g0 * SLOTS);
    const T *in_base = reinterpret_cast<const T *>(a.in) + g0 * SLOTS * a.in_view.sb + stack * a.in_view.ss;
    const int in_row = (int)(a.in_view.sb * EB), out_row = (int)(a.out_view.sb * EB);

    // LDS flavour: lane l of wavefront w fetches element 64 w + l of each row group, which lands
    // at the padded word 65 w + l of the group's slot; `set` alternates between iterations
    const BufDesc in_desc = make_desc(in_base);
    const int slot_d = t >> L, col_d = P::column(chunk, t & (n - 1), a.low_bits);
    const int64_t in_col_d = view_col(a.in_view, col_d);
    const int in_dma = in_col_d >= 0 ? slot_d * in_row + (int)(in_col_d * a.in_view.se * EB) : kOob;
    // (wave-uniform: kept in a scalar register, so the per-row slot offsets are scalar additions)
    const unsigned rows_addr = __builtin_amdgcn_readfirstlane(
        (unsigned)(unsigned long long)(LdsFloat *)lds_rows + (unsigned)(t >> 6) * 65 * 4);
    // (`full`: the caller knows that the row group exists for every row slot of the workgroup)
    auto fetch_row = [&](int grel, int set, int r, bool full = false) {
        const bool ok = full || (grel + r) * SLOTS + slot_d < rows_valid;
        load_row_to_lds(in_desc, rows_addr + (set * R + r) * kFastRowWords * 4, ok ? in_dma : kOob,
                        (grel + r) * SLOTS * in_row);
    };
    // The rows of the first two iterations are requested before anything else: they travel from
    // HBM while the factors, which mostly come from L2, are loaded.
    if constexpr (DIRECT) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            fetch_row(0, 0, r);
            fetch_row(R, 1, r);
        }
    }

    T ta[NS], tb[NS], tc_unused[NS];
    if constexpr (DIRECT)
        // (the transpose buffers are idle until the loop starts: R float2 buffers)
        load_factors_coalesced<P>(a.tw, stack * a.tw_stack_stride, a.tw_stage_stride, a.tw_stage, chunk, a.low_bits, c,
                                  ta, tb, tc_unused, false, reinterpret_cast<float2 *>(lds), R, [](auto) {});
    else
        load_factors<T, P>(a.tw, stack * a.tw_stack_stride, a.tw_stage_stride, a.tw_stage, chunk, a.low_bits, c, ta, tb,
                           tc_unused, false);

    const __amdgpu_buffer_rsrc_t in_rs = make_rsrc(in_base);
    const __amdgpu_buffer_rsrc_t out_rs =
        make_rsrc(reinterpret_cast<T *>(a.out) + g0 * SLOTS * a.out_view.sb + stack * a.out_view.ss);
    // thread-constant part of the offsets; the row group adds a wave-uniform part
    const int64_t in_col = view_col(a.in_view, col), out_col = view_col(a.out_view, col);
    const int in_thr = in_col >= 0 ? c.slot * in_row + (int)(in_col * a.in_view.se * EB) : kOob;
    const int out_thr = out_col >= 0 ? c.slot * out_row + (int)(out_col * a.out_view.se * EB) : kOob;
    const T bias = (a.bias && col < a.out_view.width)
                       ? reinterpret_cast<const T *>(a.bias)[stack * a.out_view.width + col]
                       : zero_of(T());

    auto load_rows = [&](int grel, T (&v)[R]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const bool ok = (grel + r) * SLOTS + c.slot < rows_valid;
            v[r] = buf_load<T>(in_rs, ok ? in_thr : kOob, (grel + r) * SLOTS * in_row);
        }
    };
    // The requests of an iteration are spread over its phases (phase 0: the top, phase p: behind
    // barrier p; row r goes out in phase r mod (TT + 1), with TWO_SETS in phase 1 + r mod TT):
    // sixteen wavefronts asking for R rows each at the same moment, right behind the previous
    // iteration's stores, queue up at the memory pipeline.
    constexpr auto phase_of = [](int r) { return TWO_SETS ? 1 + r % (TT > 0 ? TT : 1) : r % (TT + 1); };
    auto fetch_phase = [&](int grel, int set, auto PHASE, bool full) {
        static_for<0, R>([&](auto RR) {
            if constexpr (phase_of(RR) == decltype(PHASE)::value) fetch_row(grel, set, RR, full);
        });
    };
    // requests of an iteration that go out before its last barrier (all of them when there is none)
    constexpr int EARLY = [phase_of] {
        int c = 0;
        for (int r = 0; r < R; ++r) c += (TT == 0 || phase_of(r) < TT) ? 1 : 0;
        return c;
    }();
    // Before the last barrier of an iteration each wavefront waits for the rows of the next
    // iteration, requested during the previous one.  Younger than those: the previous
    // iteration's R stores and this iteration's EARLY requests.
    constexpr int YOUNGER = R + EARLY;
    static_assert(!DIRECT || YOUNGER == fw_operations_behind_awaited_rows<R, TT, TWO_SETS>(), "wait count of the row fetch");

    T nxt[R];
    if constexpr (DIRECT) {
        wait_rows_in_lds<0>();
        __syncthreads();
    } else {
        load_rows(0, nxt);
        // R stores that the range check discards.  They put the same "loads, then stores"
        // history in front of the first iteration as every later iteration has, so the wait for
        // the prefetched rows at the top of the loop is emitted as "all but the newest R
        // operations" and does not also wait for the previous iteration's stores to be
        // acknowledged.
#pragma unroll
        for (int r = 0; r < R; ++r) buf_store(out_rs, kOob, EB * r, zero_of(T()));
    }
    // FULL: the rows this iteration requests (two iterations ahead) and stores exist for every
    // row slot, so neither needs its range mask: all but the last iterations of a workgroup.
    auto iteration = [&](int grel, auto FULL) {
        constexpr bool full = decltype(FULL)::value;
        T v[R];
        // Transposes alternate between the two halves of `lds` across iteration boundaries too
        // (an odd number per iteration flips the start): a wavefront writes a half again only
        // behind the barrier of the transpose in between, which every wavefront reaches after
        // its read of that half.
        const int flip = (TT & 1) ? (grel / R) & 1 : 0;
        if constexpr (DIRECT) {
            const int set = (grel / R) & (SETS - 1);
            fetch_phase(grel + 2 * R, (set + 2) & (SETS - 1), std::integral_constant<int, 0>{}, full);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float x = lds_rows[(set * R + r) * kFastRowWords + (SF ? c.fB : c.fA)];
                v[r] = x;
            }
        } else {
#pragma unroll
            for (int r = 0; r < R; ++r) v[r] = nxt[r];
            load_rows(grel + R, nxt);
        }

        static_for<0, NS>([&](auto S) {
            constexpr int s = S;
            constexpr int K = P::kind(s);
            if constexpr (P::layout(s) != P::layout_before(s, SF)) {
                constexpr int nth = P::fw_transposes_before(s, SF);  // transposes done so far
                constexpr int to_b = P::layout(s);
                T *buf = lds + ((nth + flip) & 1) * R * kFastRowWords;
                const int wr = to_b ? c.fA : c.fB, rd = to_b ? c.fB : c.fA;
                transpose_rows<T, R, DIRECT && nth + 1 == TT, YOUNGER>(buf, wr, rd, v);
                if constexpr (DIRECT)
                    fetch_phase(grel + 2 * R, ((grel / R) + 2) & (SETS - 1), std::integral_constant<int, nth + 1>{}, full);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) v[r] = fw_product<K>(v[r], ta[s], tb[s], c.bperm_addr);
        });
        if constexpr (P::layout(NS - 1) != 0) {
            constexpr int nth = P::fw_transposes_before(NS, SF);
            T *buf = lds + ((nth + flip) & 1) * R * kFastRowWords;
            transpose_rows<T, R, DIRECT, YOUNGER>(buf, c.fB, c.fA, v);
            if constexpr (DIRECT)
                fetch_phase(grel + 2 * R, ((grel / R) + 2) & (SETS - 1), std::integral_constant<int, nth + 1>{}, full);
        }
        if constexpr (DIRECT && TT == 0) wait_rows_in_lds<YOUNGER>();
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const bool ok = full || (grel + r) * SLOTS + c.slot < rows_valid;
            buf_store(out_rs, ok ? out_thr : kOob, (grel + r) * SLOTS * out_row, add(v[r], bias));
        }
    };
    int grel = 0;
    if constexpr (DIRECT) {
        for (; grel < ng && (grel + 3 * R) * SLOTS <= rows_valid; grel += R) iteration(grel, std::true_type{});
    }
    for (; grel < ng; grel += R) iteration(grel, std::false_type{});
    if constexpr (DIRECT) wait_rows_in_lds<0>();  // requests past the last group (they fetch nothing)
}


struct FastBwArgs {
    const void *tw;
    int64_t tw_stack_stride;
    int64_t tw_stage_stride;
    int tw_stage[kFastMaxStages];
    int low_bits;              // SpanPlan passes: position of the lowest high bit of the span
    int64_t partial_slot;      // scalars per stage in a partial slice: 2 * n_full
    const void *x_in;
    View x_view;
    const void *g_out;
    View g_view;
    void *g_in;
    View gi_view;
    void *partial;             // (gridDim.x, S, NS, partial_slot)
    int64_t batch;
    int64_t ngroups;
    int64_t groups_per_wg;
    // float kernels on 1024-element rows or chunks only: when set, the column sums of g_out over
    // this workgroup's rows (a layer's bias gradient) go to (gridDim.x, S, bias_width)
    void *bias_partial;
    int64_t bias_width;
};

// Backward kernel, software-pipelined over rows: iteration i runs the forward replay of
// row i + 1 (producing its stage inputs) together with the reverse sweep of row i (consuming
// the stage inputs produced one iteration earlier).  Both walks change layout at the same
// phase boundaries, so they share every barrier, and where they move in the same direction
// their transposes travel through LDS as one (x, g) pair.  Two independent dependency chains
// per thread also hide the DPP and LDS latencies that a single chain exposes.
//
// DIRECT: the operands arrive in LDS (see fast_bw_kernel) and each walk starts in the layout
// of its first stage; otherwise they arrive in registers in layout A.
template <typename P, bool DIRECT>
struct BwPipe {
    static constexpr int NS = P::NS;
    static constexpr int SF = DIRECT ? P::layout(0) : 0;       // layout the forward walk starts in
    static constexpr int SB = DIRECT ? P::layout(NS - 1) : 0;  // layout the reverse walk starts in
    // phase in which forward stage s / reverse stage s runs = layout changes up to and
    // including the one in front of it
    static constexpr int fphase(int s)
    {
        int c = 0, cur = SF;
        for (int j = 0; j <= s; ++j)
            if (P::layout(j) != cur) { ++c; cur = P::layout(j); }
        return c;
    }
    static constexpr int bphase(int s)
    {
        int c = 0, cur = SB;
        for (int j = NS - 1; j >= s; --j)
            if (P::layout(j) != cur) { ++c; cur = P::layout(j); }
        return c;
    }
    static constexpr int nF = fphase(NS - 1);
    static constexpr int nB = bphase(0) + (P::layout(0) != 0 ? 1 : 0);  // + closing transpose back to A
    // layout of each walk during phase k
    static constexpr int flay(int k) { return SF ^ (k & 1); }
    static constexpr int blay(int k) { return SB ^ (k & 1); }
    // When the reverse walk ends in layout B and the forward walk has no transpose left to
    // share a barrier with, the closing transpose of the reverse walk is carried into the
    // next iteration and rides on that iteration's first barrier.
    static constexpr bool DEFER = P::layout(0) != 0 && nF < nB && nB >= 2;
    static constexpr int K = DEFER ? nB - 1 : (nF > nB ? nF : nB);  // phases 0..K; phase k >= 1 opens with transposes #k
    static constexpr int f_count(int k)
    {
        int c = 0;
        for (int s = 0; s < NS; ++s) c += fphase(s) == k ? 1 : 0;
        return c;
    }
    static constexpr int f_first(int k)
    {
        for (int s = 0; s < NS; ++s)
            if (fphase(s) == k) return s;
        return NS;
    }
    static constexpr int b_count(int k)
    {
        int c = 0;
        for (int s = 0; s < NS; ++s) c += bphase(s) == k ? 1 : 0;
        return c;
    }
    static constexpr int b_first(int k)  // highest stage of the phase: the reverse walk descends
    {
        for (int s = NS - 1; s >= 0; --s)
            if (bphase(s) == k) return s;
        return -1;
    }

    // Order in which the stages of phase k are issued.  The two walks are independent chains, so
    // any interleaving is valid; what matters is where the exchanges over lane bits 4 and 5 sit.
    // Those go through the LDS crossbar (ds_swizzle / ds_bpermute) and take an LDS round trip;
    // a stage that uses one is issued in two halves (exchange, then the arithmetic on what came
    // back) with up to two register-exchange stages of the other walk in between, and the walk
    // that still has such stages ahead keeps enough of the other walk's cheap stages for them.
    // An entry is walk * 4096 + part * 1024 + (stage's position in its walk's list for the phase);
    // part 0: whole stage, 1: exchange only, 2: the rest.
    struct Order {
        int n;
        int step[4 * NS + 4];
    };
    static constexpr bool f_slow(int k, int i) { return P::kind(f_first(k) + i) >= 4; }
    static constexpr bool b_slow(int k, int j) { return P::kind(b_first(k) - j) >= 4; }
    static constexpr Order order(int k)
    {
        Order o{};
        const int nf = f_count(k), nb = b_count(k);
        int i = 0, j = 0;
        auto push = [&](int walk, int part, int pos) { o.step[o.n++] = walk * 4096 + part * 1024 + pos; };
        while (i < nf || j < nb) {
            const bool lf = i < nf && f_slow(k, i), lb = j < nb && b_slow(k, j);
            if (lf && lb) {
                push(0, 1, i); push(1, 1, j); push(0, 2, i); push(1, 2, j);
                ++i; ++j;
            } else if (lf) {
                push(0, 1, i);
                for (int c = 0; c < 2 && j < nb && !b_slow(k, j); ++c) push(1, 0, j++);
                push(0, 2, i);
                ++i;
            } else if (lb) {
                push(1, 1, j);
                for (int c = 0; c < 2 && i < nf && !f_slow(k, i); ++c) push(0, 0, i++);
                push(1, 2, j);
                ++j;
            } else if (j >= nb) {
                push(0, 0, i++);
            } else if (i >= nf) {
                push(1, 0, j++);
            } else {
                int need_b = 0, have_b = 0, need_f = 0, have_f = 0;
                for (int q = i; q < nf; ++q) { need_b += f_slow(k, q) ? 2 : 0; have_f += f_slow(k, q) ? 0 : 1; }
                for (int q = j; q < nb; ++q) { need_f += b_slow(k, q) ? 2 : 0; have_b += b_slow(k, q) ? 0 : 1; }
                const bool keep_b = have_b <= need_b, keep_f = have_f <= need_f;
                if (keep_b && !keep_f) push(0, 0, i++);
                else if (keep_f && !keep_b) push(1, 0, j++);
                else { push(1, 0, j++); push(0, 0, i++); }
            }
        }
        return o;
    }
};

// (x, g) pair that travels through LDS as one access
template <typename T> struct PairOf;
template <> struct PairOf<float> { typedef float2 type; };
template <> struct PairOf<float2> { typedef float4 type; };
__device__ __forceinline__ float2 make_pair(float x, float g) { return make_float2(x, g); }
__device__ __forceinline__ float4 make_pair(float2 x, float2 g) { return make_float4(x.x, x.y, g.x, g.y); }
__device__ __forceinline__ float pair_x(float2 p) { return p.x; }
__device__ __forceinline__ float pair_g(float2 p) { return p.y; }
__device__ __forceinline__ float2 pair_x(float4 p) { return make_float2(p.x, p.y); }
__device__ __forceinline__ float2 pair_g(float4 p) { return make_float2(p.z, p.w); }

// two adjacent entries as one store
__device__ __forceinline__ void store_pair(float *p, float a, float b) { *reinterpret_cast<float2 *>(p) = make_float2(a, b); }
__device__ __forceinline__ void store_pair(float2 *p, float2 a, float2 b)
{
    *reinterpret_cast<float4 *>(p) = make_float4(a.x, a.y, b.x, b.y);
}

__device__ __forceinline__ void load_pair(const float *p, float &a, float &b)
{
    const float2 v = *reinterpret_cast<const float2 *>(p);
    a = v.x;
    b = v.y;
}
__device__ __forceinline__ void load_pair(const float2 *p, float2 &a, float2 &b)
{
    const float4 v = *reinterpret_cast<const float4 *>(p);
    a = make_float2(v.x, v.y);
    b = make_float2(v.z, v.w);
}

// The R values a thread holds for one walk (one per row group in flight) as one LDS access.
template <typename T, int R>
__device__ __forceinline__ void put_rows(T *base, int idx, const T (&v)[R])
{
    if constexpr (R == 1) base[idx] = v[0];
    else reinterpret_cast<float2 *>(base)[idx] = make_float2(v[0], v[1]);
}

template <typename T, int R>
__device__ __forceinline__ void get_rows(const T *base, int idx, T (&v)[R])
{
    if constexpr (R == 1) {
        v[0] = base[idx];
    } else {
        const float2 p = reinterpret_cast<const float2 *>(base)[idx];
        v[0] = p.x;
        v[1] = p.y;
    }
}

// R: row groups in flight per walk.  Two are possible where one block of float factors
// leaves half of the registers free; each barrier and each LDS round trip then serves two
// rows, and every thread runs four independent dependency chains instead of two.
template <typename T, typename P, int R = 1>
__global__ __launch_bounds__(kFastThreads) void fast_bw_kernel(FastBwArgs a)
{
    constexpr int L = P::LOG;
    constexpr int W = (int)sizeof(T) / 4;
    static_assert(R == 1 || (R == 2 && W == 1), "two row groups in flight: float only");
    // float rows are fetched straight into LDS; complex64 has no LDS to spare for that at
    // 9-10 stages and fetches into registers
    constexpr bool DIRECT = W == 1;
    using Q = BwPipe<P, DIRECT>;
    using Pair = typename PairOf<T>::type;
    constexpr int n = 1 << L, NS = P::NS, SLOTS = P::SLOTS;
    constexpr int EB = (int)sizeof(T);
    // Three factor entries per stage (the row for the forward replay, the column for the
    // reverse sweep) do not fit 128 registers next to the sums for long schedules: the
    // off-diagonal row entries, which only the replay reads, then live in LDS, one private
    // slot per thread and stage; complex64 at 9-10 stages also keeps half of the diagonal
    // entries there.
    constexpr bool COL = !(W == 2 && NS >= 9);  // reverse sweep written with the factor column
    constexpr bool TB_LDS = NS * W * R > 10;
    constexpr int NTA = (W == 2 && NS >= 9) ? NS / 2 : 0;
    // transpose buffers: [parity][walk][rowwords][R]; where both walks move the same way and
    // R = 1, the two walks share one access as an (x, g) pair: [parity][rowwords] pairs
    __shared__ __align__(16) T lds[Q::K > 0 ? 4 * R * kFastRowWords : 1];
    // (two buffers, alternating between iterations: with a single barrier per iteration a fast
    // wavefront could otherwise write the next iteration's values while a slow one still reads)
    __shared__ __align__(16) T lds_carry[Q::DEFER ? 2 * R * kFastRowWords : 1];
    __shared__ T lds_tb[TB_LDS ? NS * kFastThreads : 1];
    __shared__ T lds_ta[NTA > 0 ? NTA * kFastThreads : 1];
    // row slots: 4 sets of R for x, then 4 sets of R for the output gradient
    __shared__ float lds_rows[DIRECT ? 8 * R * kFastRowWords : 1];
    __shared__ float lds_bias[(DIRECT && SLOTS == 1) ? kFastThreads : 1];
    const int t = threadIdx.x;
    const int stack = blockIdx.y;
    const int chunk = blockIdx.z;
    const FastCoords c = fast_coords<L>(t);
    const int col = P::column(chunk, c.eA, a.low_bits);  // column of this thread's element in the full row

    T ta[NS], tb[NS], tc[NS], acc_self[NS], acc_cross[NS];
    auto load_all_factors = [&] {
        auto park = [&](auto S) {
            if constexpr (TB_LDS) lds_tb[S * kFastThreads + t] = tb[S];
            if constexpr (S < NTA) lds_ta[S * kFastThreads + t] = ta[S];
        };
        if constexpr (DIRECT) {
            // scratch for the layout-B stages' factors: the parking area of the off-diagonal
            // entries where there is one (it is filled afterwards), else the transpose buffers
            float2 *scratch = reinterpret_cast<float2 *>(TB_LDS ? reinterpret_cast<float *>(lds_tb)
                                                                : reinterpret_cast<float *>(lds));
            constexpr int room = TB_LDS ? NS * kFastThreads / (2 * kFastRowWords) : 2 * R;   // float2 buffers that fit
            constexpr int batch = room < 5 ? room : 5;
            load_factors_coalesced<P>(a.tw, stack * a.tw_stack_stride, a.tw_stage_stride, a.tw_stage, chunk, a.low_bits,
                                      c, ta, tb, tc, COL, scratch, batch, park);
        } else {
            load_factors<T, P>(a.tw, stack * a.tw_stack_stride, a.tw_stage_stride, a.tw_stage, chunk, a.low_bits, c, ta,
                               tb, tc, COL, park);
        }
        static_for<0, NS>([&](auto S) {
            acc_self[S] = zero_of(T());
            acc_cross[S] = zero_of(T());
        });
    };
    // (rows that arrive in registers: factors first, as the fetch needs no head start in LDS)
    if constexpr (!DIRECT) load_all_factors();

    const int64_t g0 = (int64_t)blockIdx.x * a.groups_per_wg;
    const int64_t g1 = g0 + a.groups_per_wg < a.ngroups ? g0 + a.groups_per_wg : a.ngroups;
    const int ng = (int)(g1 - g0);
    const int64_t row_end = g1 * SLOTS < a.batch ? g1 * SLOTS : a.batch;
    const int rows_valid = (int)(row_end - g0 * SLOTS);
    const T *x_base = reinterpret_cast<const T *>(a.x_in) + g0 * SLOTS * a.x_view.sb + stack * a.x_view.ss;
    const T *g_base = reinterpret_cast<const T *>(a.g_out) + g0 * SLOTS * a.g_view.sb + stack * a.g_view.ss;
    const __amdgpu_buffer_rsrc_t gi_rs =
        make_rsrc(reinterpret_cast<T *>(a.g_in) + g0 * SLOTS * a.gi_view.sb + stack * a.gi_view.ss);
    const int x_row = (int)(a.x_view.sb * EB), g_row = (int)(a.g_view.sb * EB), gi_row = (int)(a.gi_view.sb * EB);
    const int64_t gi_col = view_col(a.gi_view, col);
    const int gi_thr = gi_col >= 0 ? c.slot * gi_row + (int)(gi_col * a.gi_view.se * EB) : kOob;
    auto group_ok = [&](int grp) { return grp >= 0 && grp * SLOTS + c.slot < rows_valid; };
    // (`full`: the caller knows that the group exists for every row slot of the workgroup)
    auto store_grad = [&](int grp, T gval, bool full = false) {
        if (full) buf_store(gi_rs, gi_thr, grp * SLOTS * gi_row, gval);
        else buf_store(gi_rs, group_ok(grp) ? gi_thr : kOob, (grp < 0 ? 0 : grp) * SLOTS * gi_row, gval);
    };

    // --- operand fetch, register flavour: thread t holds its layout-A element
    const __amdgpu_buffer_rsrc_t x_rs = make_rsrc(x_base), g_rs = make_rsrc(g_base);
    const int64_t x_col = view_col(a.x_view, col), g_col = view_col(a.g_view, col);
    const int x_thr = x_col >= 0 ? c.slot * x_row + (int)(x_col * a.x_view.se * EB) : kOob;
    const int g_thr = g_col >= 0 ? c.slot * g_row + (int)(g_col * a.g_view.se * EB) : kOob;
    auto load_x = [&](int grp, bool full = false) {
        if (full) return buf_load<T>(x_rs, x_thr, grp * SLOTS * x_row);
        return buf_load<T>(x_rs, group_ok(grp) ? x_thr : kOob, (grp < 0 ? 0 : grp) * SLOTS * x_row);
    };
    auto load_g = [&](int grp, bool full = false) {
        if (full) return buf_load<T>(g_rs, g_thr, grp * SLOTS * g_row);
        return buf_load<T>(g_rs, group_ok(grp) ? g_thr : kOob, (grp < 0 ? 0 : grp) * SLOTS * g_row);
    };
    // --- operand fetch, LDS flavour: lane l of wavefront w fetches element 64 w + l of the row
    // group, which lands at the padded word 65 w + l of the slot
    const BufDesc x_desc = make_desc(x_base), g_desc = make_desc(g_base);
    const int slot_d = t >> L, col_d = P::column(chunk, t & (n - 1), a.low_bits);
    const int64_t x_col_d = view_col(a.x_view, col_d), g_col_d = view_col(a.g_view, col_d);
    const int x_dma = x_col_d >= 0 ? slot_d * x_row + (int)(x_col_d * a.x_view.se * EB) : kOob;
    const int g_dma = g_col_d >= 0 ? slot_d * g_row + (int)(g_col_d * a.g_view.se * EB) : kOob;
    // (wave-uniform: kept in a scalar register, so the per-row slot offsets are scalar additions)
    const unsigned rows_addr = __builtin_amdgcn_readfirstlane(
        (unsigned)(unsigned long long)(LdsFloat *)lds_rows + (unsigned)(t >> 6) * 65 * 4);
    auto group_ok_d = [&](int grp) { return grp >= 0 && grp * SLOTS + slot_d < rows_valid; };
    // Iteration j replays the R groups R j .. R j + R - 1 (they sit in x set j & 3) and sweeps
    // them one iteration later (output-gradient set j & 3).  Rows are requested AHEAD
    // iterations before they are read: one is enough when the wait for them sits late in the
    // iteration (behind two or more barriers), otherwise two.
    constexpr int AHEAD = Q::K >= 2 ? 1 : 2;
    // Column sum of the output gradient (see FastBwArgs::bias_partial): the thread adds the
    // element it reads at the top of every reverse sweep, into a private LDS word (a register
    // held across the row loop is one too many for the two-block schedules).
    constexpr bool BIAS_SUM = DIRECT && SLOTS == 1;
    const bool bias_on = BIAS_SUM && a.bias_partial != nullptr;
    if constexpr (BIAS_SUM) lds_bias[t] = 0.0f;
    auto fetch_x = [&](int j, bool full = false) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int grp = R * j + r;
            if (full)
                load_row_to_lds(x_desc, rows_addr + ((j & 3) * R + r) * kFastRowWords * 4, x_dma, grp * SLOTS * x_row);
            else
                load_row_to_lds(x_desc, rows_addr + ((j & 3) * R + r) * kFastRowWords * 4,
                                group_ok_d(grp) ? x_dma : kOob, (grp < 0 ? 0 : grp) * SLOTS * x_row);
        }
    };
    auto fetch_g = [&](int j, bool full = false) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int grp = R * j + r;
            if (full)
                load_row_to_lds(g_desc, rows_addr + ((4 + (j & 3)) * R + r) * kFastRowWords * 4, g_dma,
                                grp * SLOTS * g_row);
            else
                load_row_to_lds(g_desc, rows_addr + ((4 + (j & 3)) * R + r) * kFastRowWords * 4,
                                group_ok_d(grp) ? g_dma : kOob, (grp < 0 ? 0 : grp) * SLOTS * g_row);
        }
    };

    // The first rows are requested before anything else: they travel from HBM while the factors,
    // which mostly come from L2, are loaded.
    if constexpr (DIRECT) {
        fetch_x(0);
        fetch_g(-1);  // nothing to sweep yet: rows of zeros
        if constexpr (AHEAD == 2) {
            fetch_x(1);
            fetch_g(0);
        }
        load_all_factors();
    }

    auto tb_of = [&](auto S) -> T {
        if constexpr (TB_LDS) return lds_tb[S * kFastThreads + t];
        else return tb[S];
    };
    auto ta_of = [&](auto S) -> T {
        if constexpr (S < NTA) return lds_ta[S * kFastThreads + t];
        else return ta[S];
    };
    // look-ahead ring for the replay walk's off-diagonal entries (float kernels; see the stage loop)
    constexpr int TB_AHEAD = NS - 1 >= 2 ? 2 : 1;
    T tb_ring[TB_AHEAD];
    if constexpr (W == 1 && NS > 1)
        static_for<0, TB_AHEAD>([&](auto S) { tb_ring[S] = tb_of(std::integral_constant<int, S % (NS - 1)>{}); });

    // rows of iteration `j` out of their LDS slots, in the layouts the two walks start in
    auto read_rows = [&](int j, T (&xv)[R], T (&gr)[R]) {
        if constexpr (DIRECT) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                xv[r] = lds_rows[(((j + 1) & 3) * R + r) * kFastRowWords + (Q::SF ? c.fB : c.fA)];
                gr[r] = lds_rows[((4 + (j & 3)) * R + r) * kFastRowWords + (Q::SB ? c.fB : c.fA)];
            }
        }
    };
    // One pipelined iteration: forward replay of the groups of iteration it + 1 into `nxt`,
    // reverse sweep of the groups of iteration it out of `cur`.  Register flavour: vF / gv
    // enter holding the freshly loaded x and g.  LDS flavour: they are read from the row
    // slots, and the rows of a later iteration are requested; the rows of the next iteration
    // must have landed, for every wavefront, before it starts, so each wavefront waits for
    // its own share of them just before the last barrier of this iteration.  `carry` holds
    // the previous iteration's input gradients still in layout B (DEFER only).  FLIP
    // alternates between the two unrolled calls and keeps the LDS buffers alternating when
    // the number of phases is odd.
    // FULL: every group this iteration touches (the rows it requests, the gradient it sweeps, the
    // gradient it stores) exists for every row slot, so no access needs its range mask: true for
    // all but the first two and the last few iterations of a workgroup.
    auto iteration = [&](auto FLIP, auto FULL, int it, T (&vF)[R], T (&gv)[R], T (&carry)[R], T (&cur)[R][NS],
                         T (&nxt)[R][NS]) {
        constexpr int flip = decltype(FLIP)::value;
        constexpr bool full = decltype(FULL)::value;
        // The next iteration's rows are read out of LDS a phase ahead of their use, right behind
        // the barrier that publishes them, where the registers allow (two more live values).
        constexpr bool PREREAD = DIRECT && Q::K >= 1 && NS * R < 20;
        T pre_x[R], pre_g[R];
        T pend_f[R], pend_b[R], pend_b2[R];  // exchanged values on their way (see BwPipe::order)
        // Memory operations issued after the requests the wait is for and before the wait: this
        // iteration's stores when they come first and, if those requests were made one
        // iteration earlier, that iteration's stores and this iteration's requests.
        constexpr int YOUNGER = ((Q::DEFER && Q::K > 1) ? R : 0) + (AHEAD == 2 ? 3 * R : 0);
        static_assert(!DIRECT || (Q::K == 0 ? 3 * R : YOUNGER) == bw_operations_behind_awaited_rows<Q, R, AHEAD>(),
                      "wait count of the row fetch");
        if constexpr (DIRECT) {
            fetch_x(it + 1 + AHEAD, full);
            fetch_g(it + AHEAD, full);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float xv = vF[r];
                float gr = gv[r];
                // A row group past the end of the batch must add nothing to the d_twiddle sums.
                // Its fetch already asked for zeros (out-of-range offsets), but the sums of the
                // whole launch should not hang on what a fetch that reads nothing leaves in LDS:
                // a zero gradient here makes every product of the sweep zero.
                if (!full && !group_ok(R * it + r)) gr = 0.0f;
                vF[r] = xv;
                gv[r] = gr;
                if constexpr (BIAS_SUM) {
                    if (bias_on) lds_bias[t] += gr;
                }
            }
        }
        static_for<0, Q::K + 1>([&](auto KK) {
            constexpr int k = KK;
            if constexpr (k >= 1) {
                constexpr bool hasF = k <= Q::nF, hasB = k <= Q::nB;
                constexpr bool paired = R == 1 && hasF && hasB && Q::flay(k) == Q::blay(k);
                T *half = lds + ((k + flip * Q::K) & 1) * 2 * R * kFastRowWords;
                Pair *buf = reinterpret_cast<Pair *>(half);
                T *bufF = half, *bufB = half + R * kFastRowWords;
                const int wrF = Q::flay(k) ? c.fA : c.fB, rdF = Q::flay(k) ? c.fB : c.fA;
                const int wrB = Q::blay(k) ? c.fA : c.fB, rdB = Q::blay(k) ? c.fB : c.fA;
                if constexpr (paired) {
                    buf[wrF] = make_pair(vF[0], gv[0]);
                } else {
                    if constexpr (hasF) put_rows<T, R>(bufF, wrF, vF);
                    if constexpr (hasB) put_rows<T, R>(bufB, wrB, gv);
                }
                T *carry_buf = lds_carry + (Q::DEFER ? flip * R * kFastRowWords : 0);
                if constexpr (Q::DEFER && k == 1) put_rows<T, R>(carry_buf, c.fB, carry);
                if constexpr (DIRECT && k == Q::K) wait_rows_in_lds<YOUNGER>();
                __syncthreads();
                // the next iteration's rows are in LDS for everybody now: read them here, a
                // phase of arithmetic ahead of their first use
                if constexpr (PREREAD && k == Q::K) read_rows(it + 1, pre_x, pre_g);
                if constexpr (Q::DEFER && k == 1) {
                    T done[R];
                    get_rows<T, R>(carry_buf, c.fA, done);
#pragma unroll
                    for (int r = 0; r < R; ++r) store_grad(R * (it - 1) + r, done[r], full);
                }
                if constexpr (paired) {
                    const Pair v2 = buf[rdF];
                    vF[0] = pair_x(v2);
                    gv[0] = pair_g(v2);
                } else {
                    if constexpr (hasF) get_rows<T, R>(bufF, rdF, vF);
                    if constexpr (hasB) get_rows<T, R>(bufB, rdB, gv);
                }
            }
            constexpr int cf = Q::f_count(k), cb = Q::b_count(k);
            constexpr int f0 = Q::f_first(k), b0 = Q::b_first(k);
            // complex64: one reverse stage, one forward stage in turn (its exchanges move twice
            // the words and its register budget has no room for values on their way)
            if constexpr (W == 2) {
                static_for<0, (cf > cb ? cf : cb)>([&](auto J) {
                    constexpr int j = J;
                    if constexpr (j < cb) {
                        constexpr int s = b0 - j;
                        const auto SS = std::integral_constant<int, s>{};
                        if constexpr (COL)
                            bw_products<P::kind(s)>(acc_self[s], acc_cross[s], gv[0], cur[0][s], ta_of(SS), tc[s], c.bperm_addr);
                        else
                            bw_products_row<P::kind(s)>(acc_self[s], acc_cross[s], gv[0], cur[0][s], ta_of(SS), tb_of(SS),
                                                        c.bperm_addr);
                    }
                    if constexpr (j < cf) {
                        constexpr int s = f0 + j;
                        const auto SS = std::integral_constant<int, s>{};
                        nxt[0][s] = vF[0];
                        if constexpr (s + 1 < NS) vF[0] = fw_product<P::kind(s)>(vF[0], ta_of(SS), tb_of(SS), c.bperm_addr);
                    }
                });
            }
            constexpr auto ord = Q::order(k);
            static_assert(ord.n >= cf + cb, "every stage of the phase is issued");
            static_for<0, (W == 1 ? ord.n : 0)>([&](auto I) {
                constexpr int code = ord.step[I];
                constexpr int walk = code / 4096, part = (code / 1024) % 4, pos = code % 1024;
                if constexpr (walk == 1) {
                    // reverse stage: uses the gradient before it passes through the stage
                    constexpr int s = b0 - pos;
                    constexpr int Kd = P::kind(s);
                    const auto SS = std::integral_constant<int, s>{};
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        if constexpr (part == 0) {
                            if constexpr (COL)
                                bw_products<Kd>(acc_self[s], acc_cross[s], gv[r], cur[r][s], ta_of(SS), tc[s], c.bperm_addr);
                            else
                                bw_products_row<Kd>(acc_self[s], acc_cross[s], gv[r], cur[r][s], ta_of(SS), tb_of(SS),
                                                    c.bperm_addr);
                        } else if constexpr (part == 1) {
                            if constexpr (COL) {
                                pend_b[r] = partner<Kd>(gv[r], c.bperm_addr);
                            } else {
                                pend_b[r] = partner<Kd>(cur[r][s], c.bperm_addr);
                                pend_b2[r] = partner<Kd>(mul(conj_of(tb_of(SS)), gv[r]), c.bperm_addr);
                            }
                            // (the request stays in front of the other walk's stages that cover it)
                            if (r == R - 1) __builtin_amdgcn_sched_barrier(0);
                        } else {
                            if constexpr (COL)
                                bw_finish(acc_self[s], acc_cross[s], gv[r], cur[r][s], ta_of(SS), tc[s], pend_b[r]);
                            else
                                bw_finish_row(acc_self[s], acc_cross[s], gv[r], cur[r][s], ta_of(SS), pend_b[r], pend_b2[r]);
                        }
                    }
                } else {
                    constexpr int s = f0 + pos;
                    constexpr int Kd = P::kind(s);
                    const auto SS = std::integral_constant<int, s>{};
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        if constexpr (part != 2) nxt[r][s] = vF[r];
                        if constexpr (s + 1 < NS) {
                            if constexpr (part == 1) {
                                pend_f[r] = partner<Kd>(vF[r], c.bperm_addr);
                                if (r == R - 1) __builtin_amdgcn_sched_barrier(0);
                            } else {
                                // The off-diagonal entry comes out of the look-ahead ring, whose slot is
                                // refilled at once with the entry TB_AHEAD product stages further on
                                // (wrapping into the next iteration): the pinned stages keep every LDS read
                                // where it is written, so the look-ahead has to be spelled out.
                                // (slot = position in the endless sequence of product stages, modulo
                                // the ring size: the two unrolled iterations differ when NS - 1 is odd)
                                constexpr int slot = (s + flip * (NS - 1)) % TB_AHEAD;
                                const T tbv = tb_ring[slot];
                                if (r == R - 1)
                                    tb_ring[slot] = tb_of(std::integral_constant<int, (s + TB_AHEAD) % (NS - 1)>{});
                                if constexpr (part == 2) vF[r] = fw_finish(vF[r], ta_of(SS), tbv, pend_f[r]);
                                else if constexpr (Kd < 4) vF[r] = fw_product_pinned<Kd>(vF[r], ta_of(SS), tbv);
                                else vF[r] = fw_product<Kd>(vF[r], ta_of(SS), tbv, c.bperm_addr);
                            }
                        }
                    }
                }
            });
        });
        if constexpr (DIRECT && Q::K == 0) wait_rows_in_lds<3 * R>();
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if constexpr (Q::DEFER) carry[r] = gv[r];
            else store_grad(R * it + r, gv[r], full);
        }
        if constexpr (DIRECT) {
            if constexpr (!PREREAD) read_rows(it + 1, vF, gv);
            else {
#pragma unroll
                for (int r = 0; r < R; ++r) { vF[r] = pre_x[r]; gv[r] = pre_g[r]; }
            }
        }
    };

    T actP[R][NS], actQ[R][NS];
#pragma unroll
    for (int r = 0; r < R; ++r) static_for<0, NS>([&](auto S) { actP[r][S] = zero_of(T()); });
    // iteration it replays the groups of iteration it + 1 and sweeps its own; it = -1 .. nit - 1
    T carry[R], vF[R], gv[R];
#pragma unroll
    for (int r = 0; r < R; ++r) carry[r] = vF[r] = gv[r] = zero_of(T());
    const int nit = (ng + R - 1) / R;
    // (rows in registers: with a deferred closing transpose one more, empty, iteration flushes the
    // last groups; the LDS flavour flushes them on its own behind the loop)
    const int it_end = Q::DEFER ? nit + 1 : nit;
    int flush_it = 0;
    if constexpr (DIRECT) {
        wait_rows_in_lds<0>();
        __syncthreads();
        read_rows(-1, vF, gv);
        const std::false_type masked{};
        const std::true_type unmasked{};
        int it = -1;
        iteration(std::integral_constant<int, 0>{}, masked, it, vF, gv, carry, actP, actQ);
        iteration(std::integral_constant<int, 1>{}, masked, it + 1, vF, gv, carry, actQ, actP);
        // iterations it, it + 1 are FULL when the furthest group they request exists in every slot
        // An odd iteration left over at the end runs on its own where the kernel has the registers
        // for a third copy of the body (whole rows of 1024); the others start one more pair, whose
        // second half finds no rows.
        constexpr int ODD_TAIL = SLOTS == 1 ? 1 : 0;
        for (it = 1; it + ODD_TAIL < nit && (R * (it + 2 + AHEAD) + R) * SLOTS <= rows_valid; it += 2) {
            iteration(std::integral_constant<int, 0>{}, unmasked, it, vF, gv, carry, actP, actQ);
            iteration(std::integral_constant<int, 1>{}, unmasked, it + 1, vF, gv, carry, actQ, actP);
        }
        for (; it + ODD_TAIL < nit; it += 2) {
            iteration(std::integral_constant<int, 0>{}, masked, it, vF, gv, carry, actP, actQ);
            iteration(std::integral_constant<int, 1>{}, masked, it + 1, vF, gv, carry, actQ, actP);
        }
        if constexpr (ODD_TAIL != 0) {
            if (it < nit) {
                iteration(std::integral_constant<int, 0>{}, masked, it, vF, gv, carry, actP, actQ);
                ++it;
            }
        }
        wait_rows_in_lds<0>();  // requests past the last group (they fetch nothing)
        flush_it = it - 1;   // the last iteration that ran (it may lie past the last group)
    } else {
        // complex64: an iteration is long enough to cover the fetch, and four more registers
        // held across a whole iteration would not fit
        T x0 = load_x(0), gm = load_g(-1);
        if constexpr (NS >= 9) {
            // (no second copy of the body for the passes that fill the register file)
            for (int it = -1; it < it_end; it += 2) {
                vF[0] = x0;
                gv[0] = gm;
                const T x1 = load_x(it + 2), gp = load_g(it + 1);
                iteration(std::integral_constant<int, 0>{}, std::false_type{}, it, vF, gv, carry, actP, actQ);
                x0 = load_x(it + 3);
                gm = load_g(it + 2);
                vF[0] = x1;
                gv[0] = gp;
                iteration(std::integral_constant<int, 1>{}, std::false_type{}, it + 1, vF, gv, carry, actQ, actP);
            }
        } else {
        // a pair of iterations: FULL when every group it loads (up to it + 3) and stores exists in
        // every row slot
        auto pair = [&](int it, auto FULL) {
            constexpr bool full = decltype(FULL)::value;
            vF[0] = x0;
            gv[0] = gm;
            const T x1 = load_x(it + 2, full), gp = load_g(it + 1, full);
            iteration(std::integral_constant<int, 0>{}, FULL, it, vF, gv, carry, actP, actQ);
            x0 = load_x(it + 3, full);
            gm = load_g(it + 2, full);
            vF[0] = x1;
            gv[0] = gp;
            iteration(std::integral_constant<int, 1>{}, FULL, it + 1, vF, gv, carry, actQ, actP);
        };
        int it = -1;
        pair(it, std::false_type{});
        for (it = 1; it < it_end && (it + 4) * SLOTS <= rows_valid; it += 2) pair(it, std::true_type{});
        for (; it < it_end; it += 2) pair(it, std::false_type{});
        }
    }

    // Recompute the coordinates from a laundered thread id: sharing them with the prologue
    // would keep one address per stage alive across the whole row loop.
    int t2 = t;
    asm volatile("" : "+v"(t2));
    const FastCoords c2 = fast_coords<L>(t2);
    if constexpr (DIRECT && Q::DEFER) {
        // The input gradient of the last iteration is still in layout B in `carry`: the closing
        // transposition on its own, through the half of the carry buffer that the next iteration
        // would have used (last touched two barriers ago).
        T *carry_buf = lds_carry + (flush_it & 1) * R * kFastRowWords;
        put_rows<T, R>(carry_buf, c2.fB, carry);
        __syncthreads();
        T done[R];
        get_rows<T, R>(carry_buf, c2.fA, done);
#pragma unroll
        for (int r = 0; r < R; ++r) store_grad(R * flush_it + r, done[r]);
    }
    if constexpr (BIAS_SUM) {
        if (bias_on) {
            const int64_t bcol = P::column(chunk, Q::SB ? c2.eB : c2.eA, a.low_bits);
            if (bcol < a.bias_width)
                reinterpret_cast<float *>(a.bias_partial)[((int64_t)blockIdx.x * gridDim.y + stack) * a.bias_width +
                                                          bcol] = lds_bias[t2];
        }
    }
    // One partial slice per workgroup.  When the workgroup holds several rows at once
    // (n < 1024) the per-row-slot sums are first added through LDS in ascending slot order.
    T *part = reinterpret_cast<T *>(a.partial) + ((int64_t)blockIdx.x * gridDim.y + stack) * NS * a.partial_slot +
              P::pair_base(chunk) * 4;
    if constexpr (SLOTS == 1) {
        // Per stage the thread ends up with row r of its pair's 2x2 block: dT[r][r] is its own sum,
        // dT[r][1 - r] its own cross sum (row form) or the cross sum of the pair's other thread,
        // which holds dT[1 - (1 - r)][1 - r] (column form: one more exchange).
        static_for<0, NS>([&](auto S) {
            constexpr int s = S;
            if constexpr (COL) acc_cross[s] = partner<P::kind(s)>(acc_cross[s], c2.bperm_addr);
        });
        // The sums of a stage that ran in layout B belong to elements 16 apart within a wavefront,
        // i.e. to 16-byte pieces 256 bytes apart in the slice.  They first travel through LDS (the
        // factor slots or transposition buffers, dead by now) to the thread that holds the element
        // in layout A, so that every wavefront stores 512 consecutive bytes per stage.
        struct Late { int n; int s[NS]; };
        constexpr Late late = [] {
            Late l{};
            for (int s = 0; s < NS; ++s)
                if (P::layout(s) != 0) l.s[l.n++] = s;
            return l;
        }();
        if constexpr (late.n > 0) {
            T *stage = TB_LDS ? lds_tb : lds;
            constexpr int room = (TB_LDS ? NS * kFastThreads : 4 * R * kFastRowWords) / (2 * kFastRowWords);
            static_assert(room >= 1, "staging area for the partial sums");
            constexpr int nbatch = (late.n + room - 1) / room;
            static_for<0, nbatch>([&](auto BB) {
                constexpr int j0 = BB * room;
                constexpr int j1 = j0 + room < late.n ? j0 + room : late.n;
                __syncthreads();   // the area is free: row loop or previous batch done
                static_for<j0, j1>([&](auto J) {
                    constexpr int s = late.s[J];
                    store_pair(stage + ((J - j0) * kFastRowWords + c2.fB) * 2, acc_self[s], acc_cross[s]);
                });
                __syncthreads();
                static_for<j0, j1>([&](auto J) {
                    constexpr int s = late.s[J];
                    load_pair(stage + ((J - j0) * kFastRowWords + c2.fA) * 2, acc_self[s], acc_cross[s]);
                });
            });
        }
        static_for<0, NS>([&](auto S) {
            constexpr int s = S;
            constexpr int bit = P::bit(s);
            const int e = c2.eA;
            const int r = (e >> bit) & 1;
            const int i = P::pair_index(chunk, e, bit, a.low_bits);
            T *d = part + (int64_t)s * a.partial_slot + i * 4;
            store_pair(d + 2 * r, r ? acc_cross[s] : acc_self[s], r ? acc_self[s] : acc_cross[s]);
        });
    } else {
        // (the factor slots in LDS are dead by now and serve as the staging area)
        __shared__ T red_own[TB_LDS ? 1 : 2 * 1024];
        T *red = TB_LDS ? lds_tb : red_own;
        static_for<0, NS>([&](auto S) {
            constexpr int s = S;
            constexpr int bit = P::bit(s);
            constexpr int lay = P::layout(s);
            const int e = lay ? c2.eB : c2.eA;
            __syncthreads();
            red[(c2.slot * n + e) * 2 + 0] = acc_self[s];
            red[(c2.slot * n + e) * 2 + 1] = acc_cross[s];
            __syncthreads();
            if (t2 < 2 * n) {
                const int eo = t2 >> 1, j = t2 & 1;
                T sum = red[t2];
#pragma unroll 4
                for (int sl = 1; sl < SLOTS; ++sl) sum = add(sum, red[sl * 2 * n + t2]);
                const int r = (eo >> bit) & 1;
                const int i = P::pair_index(chunk, eo, bit, a.low_bits);
                // j = 0: dT[r][r], j = 1: dT[1 - r][r] (column form) or dT[r][1 - r]
                part[(int64_t)s * a.partial_slot + i * 4 + (j ? (COL ? 2 - r : r + 1) : 3 * r)] = sum;
            }
        });
    }
}

}  // namespace bf
