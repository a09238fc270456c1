// Shared device-side helpers: scalar algebra for float / complex64 and the rule that
// maps a flat stage number to (radix, stride, twiddle offset).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bf {

// ---- scalar algebra -------------------------------------------------------------------
// complex64 is a float2 (re, im), the memory layout of torch.complex64.

__device__ __forceinline__ float zero_of(float) { return 0.0f; }
__device__ __forceinline__ float2 zero_of(float2) { return make_float2(0.0f, 0.0f); }

__device__ __forceinline__ float conj_of(float a) { return a; }
__device__ __forceinline__ float2 conj_of(float2 a) { return make_float2(a.x, -a.y); }

__device__ __forceinline__ float mul(float a, float b) { return a * b; }
// (the fused multiply-adds are spelled out: left to the compiler, which of the two products of a
// component gets fused depends on the code around the call, and the same stage would round
// differently in different kernels)
__device__ __forceinline__ float2 mul(float2 a, float2 b)
{
    return make_float2(fmaf(a.x, b.x, -(a.y * b.y)), fmaf(a.x, b.y, a.y * b.x));
}

// acc + a * b
__device__ __forceinline__ float mac(float acc, float a, float b) { return fmaf(a, b, acc); }
__device__ __forceinline__ float2 mac(float2 acc, float2 a, float2 b)
{
    float re = fmaf(a.x, b.x, acc.x);
    re = fmaf(-a.y, b.y, re);
    float im = fmaf(a.x, b.y, acc.y);
    im = fmaf(a.y, b.x, im);
    return make_float2(re, im);
}

// acc + conj(a) * b
__device__ __forceinline__ float macc(float acc, float a, float b) { return fmaf(a, b, acc); }
__device__ __forceinline__ float2 macc(float2 acc, float2 a, float2 b)
{
    float re = fmaf(a.x, b.x, acc.x);
    re = fmaf(a.y, b.y, re);
    float im = fmaf(a.x, b.y, acc.y);
    im = fmaf(-a.y, b.x, im);
    return make_float2(re, im);
}

__device__ __forceinline__ float add(float a, float b) { return a + b; }
__device__ __forceinline__ float2 add(float2 a, float2 b) { return make_float2(a.x + b.x, a.y + b.y); }

// ---- stage schedule -------------------------------------------------------------------
// A multiply is a flat list of nblocks * per stages.  Base-2: per = log_n stages of 2x2
// factors.  Base-4: per = log_n / 2 radix-4 stages followed by one 2x2 stage when log_n is
// odd.  Block k runs with increasing stride when increasing_stride XOR (k odd).
struct Schedule {
    int log_n;
    int nblocks;
    int increasing_stride;
    int base4;
    int per;                  // stages per block
    int64_t tw2_stack_stride; // scalars between stacks in the 2x2 twiddle tensor
    int64_t tw4_stack_stride; // same for the 4x4 twiddle tensor (base-4 only)
};

struct StageInfo {
    int radix4;      // 1: 4x4 factors on quads, 0: 2x2 factors on pairs
    int log_stride;  // distance between the elements of a pair / quad is 1 << log_stride
    int64_t tw_off;  // scalar offset of this stage's factors inside one stack
};

__host__ __device__ __forceinline__ StageInfo stage_info(const Schedule &sc, int t)
{
    StageInfo si;
    const int block = t / sc.per;
    const int idx = t - block * sc.per;
    const bool cur_inc = (sc.increasing_stride != 0) != ((block & 1) != 0);
    const int64_t n = (int64_t)1 << sc.log_n;
    if (!sc.base4) {
        si.radix4 = 0;
        si.log_stride = cur_inc ? idx : sc.log_n - 1 - idx;
        si.tw_off = ((int64_t)block * sc.log_n + idx) * (n / 2) * 4;
    } else {
        const int l4 = sc.log_n / 2;
        if (idx < l4) {
            si.radix4 = 1;
            si.log_stride = cur_inc ? 2 * idx : sc.log_n - 2 - 2 * idx;
            si.tw_off = ((int64_t)block * l4 + idx) * (n / 4) * 16;
        } else {
            si.radix4 = 0;
            si.log_stride = cur_inc ? sc.log_n - 1 : 0;
            si.tw_off = (int64_t)block * (n / 2) * 4;
        }
    }
    return si;
}

// Strided view of a (B, S, width) operand; columns >= width read as zero / are not written.
struct View {
    int64_t sb, ss, se;
    int64_t width;
    const int *perm;  // NULL, or n entries: column c of the row as the kernels see it lives in tensor column perm[c]
};

// Tensor column behind column `col` (< n) of a row as the kernels see it, or -1 when that
// column does not exist in the tensor (reads give zero, writes are dropped).  The table is a
// fixed permutation in front of or behind the multiply, folded into the access.
__device__ __forceinline__ int64_t view_col(const View &v, int64_t col)
{
    if (v.perm) col = v.perm[col];
    return col < v.width ? col : -1;
}

}  // namespace bf
