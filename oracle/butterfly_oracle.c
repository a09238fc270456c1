/*
 * TEST INFRASTRUCTURE ONLY -- not part of the shipped library.
 *
 * Single-threaded CPU restatement of the reference butterfly multiply, used as
 * the parity checker in tests and as the timed CPU baseline in the benchmark.
 * Nothing in the product path may link or call this file.
 *
 * Functions (one per scalar type f32 / f64 / c64 / c128):
 *   oracle_butterfly_fw_*        csrc/cpu/butterfly_cpu.cpp:17-66
 *   oracle_butterfly_bw_*        csrc/cpu/butterfly_cpu.cpp:68-177
 *   oracle_butterfly_base4_fw_*  torch_butterfly/multiply_base4.py:7-41
 *   oracle_butterfly_base4_bw_*  adjoint of the above (what autograd derives)
 *
 * Arithmetic is kept bit-identical to the reference built with its default
 * flags on x86-64 (g++ -O2, no FMA contraction): separate multiplies and adds,
 * complex products by the naive (ac-bd, ad+bc) rule that c10::complex uses.
 * Build with -ffp-contract=off.
 *
 * Pinning status: fw/bw are checked bit-for-bit against the compiled reference
 * C++ (oracle/_ref) and against committed golden vectors written from it, plus
 * closed forms (Hadamard, DFT), dense brute force and adjoint identities.
 * base4 fw/bw have no native reference; they are pinned by dense brute force,
 * by equivalence with the base-2 path after twiddle fusion, and by the adjoint
 * identity / finite differences.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct { float re, im; } cf32;
typedef struct { double re, im; } cf64;

static inline cf32 cf32_mul(cf32 a, cf32 b) { cf32 r = { a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re }; return r; }
static inline cf32 cf32_add(cf32 a, cf32 b) { cf32 r = { a.re + b.re, a.im + b.im }; return r; }
static inline cf32 cf32_conj(cf32 a) { cf32 r = { a.re, -a.im }; return r; }
static inline cf64 cf64_mul(cf64 a, cf64 b) { cf64 r = { a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re }; return r; }
static inline cf64 cf64_add(cf64 a, cf64 b) { cf64 r = { a.re + b.re, a.im + b.im }; return r; }
static inline cf64 cf64_conj(cf64 a) { cf64 r = { a.re, -a.im }; return r; }
static const cf32 cf32_zero = { 0.0f, 0.0f };
static const cf64 cf64_zero = { 0.0, 0.0 };

#define T float
#define SUF f32
#define MUL(a, b) ((a) * (b))
#define ADD(a, b) ((a) + (b))
#define CONJ(a) (a)
#define ZERO 0.0f
#include "butterfly_oracle_impl.inc"
#undef T
#undef SUF
#undef MUL
#undef ADD
#undef CONJ
#undef ZERO

#define T double
#define SUF f64
#define MUL(a, b) ((a) * (b))
#define ADD(a, b) ((a) + (b))
#define CONJ(a) (a)
#define ZERO 0.0
#include "butterfly_oracle_impl.inc"
#undef T
#undef SUF
#undef MUL
#undef ADD
#undef CONJ
#undef ZERO

#define T cf32
#define SUF c64
#define MUL(a, b) cf32_mul((a), (b))
#define ADD(a, b) cf32_add((a), (b))
#define CONJ(a) cf32_conj(a)
#define ZERO cf32_zero
#include "butterfly_oracle_impl.inc"
#undef T
#undef SUF
#undef MUL
#undef ADD
#undef CONJ
#undef ZERO

#define T cf64
#define SUF c128
#define MUL(a, b) cf64_mul((a), (b))
#define ADD(a, b) cf64_add((a), (b))
#define CONJ(a) cf64_conj(a)
#define ZERO cf64_zero
#include "butterfly_oracle_impl.inc"
#undef T
#undef SUF
#undef MUL
#undef ADD
#undef CONJ
#undef ZERO
