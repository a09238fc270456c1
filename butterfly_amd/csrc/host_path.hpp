// Host (CPU) path of the butterfly multiply for tensors that live in host memory.
//
// The reference operators accept CPU tensors in float, double, complex64 and complex128
// (csrc/butterfly.cpp:44-52, 84-92 dispatch to csrc/cpu/butterfly_cpu.cpp:17-177), and callers
// such as the module tests run on both devices, so the operator boundary keeps that.  Device
// tensors never come here: they go to the HIP library or fail.
//
// Row-stationary, unlike the reference's whole-batch sweep per stage: one (batch, stack) row is
// carried through every stage in a buffer of n elements (backward: the inputs of all stages of
// that row, nstages * n elements), so the working set stays in cache whatever the batch is.
// Single-threaded; d_twiddle sums run over the batch in ascending order.  Plain pointers, sizes
// and element strides: no tensor types.
#pragma once

#include <cstdint>
#include <vector>

namespace bf_host {

// complex scalar with the textbook product (no special handling of infinities)
template <typename R>
struct Cplx {
    R re, im;
};

template <typename R> inline R zero(R) { return R(0); }
template <typename R> inline Cplx<R> zero(Cplx<R>) { return Cplx<R>{R(0), R(0)}; }
inline float conj_of(float v) { return v; }
inline double conj_of(double v) { return v; }
template <typename R> inline Cplx<R> conj_of(Cplx<R> v) { return Cplx<R>{v.re, -v.im}; }
inline float mul(float a, float b) { return a * b; }
inline double mul(double a, double b) { return a * b; }
template <typename R> inline Cplx<R> mul(Cplx<R> a, Cplx<R> b)
{
    return Cplx<R>{a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
}
inline float add(float a, float b) { return a + b; }
inline double add(double a, double b) { return a + b; }
template <typename R> inline Cplx<R> add(Cplx<R> a, Cplx<R> b) { return Cplx<R>{a.re + b.re, a.im + b.im}; }

struct Shape {
    int64_t batch, nstacks, log_n, nblocks, input_size, output_size;
    bool increasing_stride;
};

// log2 of the stride of stage t (block t / log_n, position t % log_n in the block): blocks
// alternate direction, the first one going up when increasing_stride is set
// (csrc/cpu/butterfly_cpu.cpp:34-36)
inline int stage_log_stride(const Shape &sh, int64_t t)
{
    const int64_t block = t / sh.log_n, idx = t % sh.log_n;
    const bool up = sh.increasing_stride != ((block & 1) != 0);
    return (int)(up ? idx : sh.log_n - 1 - idx);
}

// one stage in place on a row of n elements; tw: the stage's (n/2, 2, 2) factors
template <typename T>
inline void apply_stage(T *row, const T *tw, int64_t n, int log_stride)
{
    const int64_t st = (int64_t)1 << log_stride;
    for (int64_t i = 0; i < n / 2; ++i) {
        const int64_t low = i & (st - 1);
        const int64_t pos = 2 * (i - low) + low;
        const T *f = tw + 4 * i;
        const T x0 = row[pos], x1 = row[pos + st];
        row[pos] = add(mul(f[0], x0), mul(f[1], x1));
        row[pos + st] = add(mul(f[2], x0), mul(f[3], x1));
    }
}

// output (B, S, O) = product of all stages applied to the input zero-padded / trimmed to n.
// twiddle dense (S, nb, log_n, n/2, 2, 2); xs / os: element strides of input / output.
template <typename T>
void multiply_fw(const Shape &sh, const T *twiddle, const T *input, const int64_t xs[3], T *output,
                 const int64_t os[3])
{
    const int64_t n = (int64_t)1 << sh.log_n;
    const int64_t nstages = sh.nblocks * sh.log_n;
    const int64_t stage_elems = (n / 2) * 4;
    std::vector<T> row((size_t)n);
    for (int64_t b = 0; b < sh.batch; ++b) {
        for (int64_t s = 0; s < sh.nstacks; ++s) {
            const T *x = input + b * xs[0] + s * xs[1];
            for (int64_t j = 0; j < n; ++j) row[(size_t)j] = j < sh.input_size ? x[j * xs[2]] : zero(T());
            const T *tw = twiddle + s * nstages * stage_elems;
            for (int64_t t = 0; t < nstages; ++t)
                apply_stage(row.data(), tw + t * stage_elems, n, stage_log_stride(sh, t));
            T *y = output + b * os[0] + s * os[1];
            for (int64_t j = 0; j < sh.output_size; ++j) y[j * os[2]] = row[(size_t)j];
        }
    }
}

// d_twiddle (dense, twiddle shape; overwritten) and d_input (B, S, I): columns >= n get zero.
// grad (B, S, O) is zero-padded to n.  PyTorch's convention for complex gradients
// (csrc/cpu/butterfly_cpu.cpp:143-164): d_input = T^H g, d_twiddle[r][c] += g_r conj(x_c).
template <typename T>
void multiply_bw(const Shape &sh, const T *twiddle, const T *input, const int64_t xs[3], const T *grad,
                 const int64_t gs[3], T *d_twiddle, T *d_input, const int64_t ds[3])
{
    const int64_t n = (int64_t)1 << sh.log_n;
    const int64_t nstages = sh.nblocks * sh.log_n;
    const int64_t stage_elems = (n / 2) * 4;
    for (int64_t k = 0; k < sh.nstacks * nstages * stage_elems; ++k) d_twiddle[k] = zero(T());
    // acts[t] = input of stage t for the row in hand; g = running gradient
    std::vector<T> acts((size_t)((nstages > 0 ? nstages : 1) * n)), g((size_t)n);
    for (int64_t b = 0; b < sh.batch; ++b) {
        for (int64_t s = 0; s < sh.nstacks; ++s) {
            const T *x = input + b * xs[0] + s * xs[1];
            const T *tw = twiddle + s * nstages * stage_elems;
            T *dtw = d_twiddle + s * nstages * stage_elems;
            for (int64_t j = 0; j < n; ++j) acts[(size_t)j] = j < sh.input_size ? x[j * xs[2]] : zero(T());
            for (int64_t t = 0; t + 1 < nstages; ++t) {
                T *next = acts.data() + (t + 1) * n;
                const T *cur = acts.data() + t * n;
                for (int64_t j = 0; j < n; ++j) next[j] = cur[j];
                apply_stage(next, tw + t * stage_elems, n, stage_log_stride(sh, t));
            }
            const T *go = grad + b * gs[0] + s * gs[1];
            for (int64_t j = 0; j < n; ++j) g[(size_t)j] = j < sh.output_size ? go[j * gs[2]] : zero(T());
            for (int64_t t = nstages - 1; t >= 0; --t) {
                const T *xin = acts.data() + t * n;
                const T *f = tw + t * stage_elems;
                T *df = dtw + t * stage_elems;
                const int64_t st = (int64_t)1 << stage_log_stride(sh, t);
                for (int64_t i = 0; i < n / 2; ++i) {
                    const int64_t low = i & (st - 1);
                    const int64_t pos = 2 * (i - low) + low;
                    const T g0 = g[(size_t)pos], g1 = g[(size_t)(pos + st)];
                    const T x0 = xin[pos], x1 = xin[pos + st];
                    const T *fi = f + 4 * i;
                    T *di = df + 4 * i;
                    g[(size_t)pos] = add(mul(conj_of(fi[0]), g0), mul(conj_of(fi[2]), g1));
                    g[(size_t)(pos + st)] = add(mul(conj_of(fi[1]), g0), mul(conj_of(fi[3]), g1));
                    di[0] = add(di[0], mul(g0, conj_of(x0)));
                    di[1] = add(di[1], mul(g0, conj_of(x1)));
                    di[2] = add(di[2], mul(g1, conj_of(x0)));
                    di[3] = add(di[3], mul(g1, conj_of(x1)));
                }
            }
            T *dx = d_input + b * ds[0] + s * ds[1];
            for (int64_t j = 0; j < sh.input_size; ++j) dx[j * ds[2]] = j < n ? g[(size_t)j] : zero(T());
        }
    }
}

}  // namespace bf_host
