/*
 * C ABI of libbutterfly_hip.so -- butterfly matrix multiply on AMD gfx950 (MI355X).
 *
 * Every pointer argument named twiddle*, input, grad, output, d_* and workspace is a
 * DEVICE pointer.  Nothing here allocates or synchronises: the caller supplies the
 * workspace (size from the *_workspace_bytes query) and the HIP stream (hipStream_t
 * passed as void*, NULL = the null stream); kernels are enqueued and the call returns.
 *
 * Element types: BF_F32 = float; BF_C64 = interleaved (re, im) float pairs, the memory
 * layout of torch.complex64.  All strides are in ELEMENTS of that type, may be zero
 * (broadcast stacks) and must be non-negative.  Twiddles are dense row-major.
 *
 * Return value: 0 on success, a negative BF_ERR_* code otherwise; bf_last_error()
 * returns the message for the calling thread.
 */
#ifndef BUTTERFLY_HIP_H
#define BUTTERFLY_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BF_F32 0
#define BF_C64 1

#define BF_OK 0
#define BF_ERR_INVALID (-1)     /* bad shape / stride / argument                      */
#define BF_ERR_UNSUPPORTED (-2) /* valid request the library cannot run (e.g. n too large) */
#define BF_ERR_HIP (-3)         /* a HIP call or kernel launch failed                 */
#define BF_ERR_WORKSPACE (-4)   /* workspace missing or too small                     */

/* What every size query (*_workspace_bytes, *_saved_bytes) answers for a problem that does not
 * pass validation (bf_last_error() says why); 0 means "valid, no such memory needed".       */
#define BF_SIZE_INVALID ((size_t)-1)

/* Problem description shared by all entry points.  Plain data, no ownership. */
typedef struct bf_problem {
    int32_t dtype;             /* BF_F32 or BF_C64                                              */
    int32_t increasing_stride; /* first block multiplies with stride 1,2,..,n/2 (else n/2,..,1) */
    int64_t batch;             /* B                                                             */
    int64_t nstacks;           /* S                                                             */
    int64_t log_n;             /* n = 1 << log_n                                                */
    int64_t nblocks;           /* nb                                                            */
    int64_t input_size;        /* I: input is zero-padded / trimmed to n                        */
    int64_t output_size;       /* O <= n: columns of output (fw) or of grad (bw)                */
    int64_t input_stride[3];   /* of input  (B, S, I)                                           */
    int64_t output_stride[3];  /* fw: of output (B, S, O); bw: of grad (B, S, O)                */
    int64_t d_input_stride[3]; /* bw only: of d_input (B, S, I)                                 */
} bf_problem;

/* Library version (major * 10000 + minor * 100 + patch). */
int bf_version(void);

/* HIP runtime version the library was built against (HIP_VERSION).  Stands where the
 * reference's torch_butterfly::cuda_version reports CUDA_VERSION (csrc/version.cpp:14-23). */
int bf_hip_version(void);

/* Message describing the last error on this thread ("" if none). */
const char *bf_last_error(void);

/* Forward multiply: output = (prod of nb * log_n block-diagonal 2x2 stages) pad(input).
 * Replaces butterfly_multiply_fw_cuda / butterfly_multiply_fw_cpu behind
 * torch_butterfly::butterfly_multiply_fw (csrc/butterfly.cpp:20-53,
 * csrc/cpu/butterfly_cpu.cpp:17-66, csrc/cuda/butterfly_cuda.cu:349-416).
 *   twiddle (S, nb, log_n, n/2, 2, 2) dense and 16-byte aligned (every entry point that
 *   takes factors or writes their gradients requires that of them).                  */
int bf_butterfly_multiply_fw(const bf_problem *p, const void *twiddle, const void *input,
                             void *output, void *workspace, size_t workspace_bytes, void *stream);

/* Workspace the forward call needs, in bytes: zero when the whole schedule runs in one
 * launch (n <= 1024 with at most two blocks), one (B, S, n) activation otherwise.          */
size_t bf_butterfly_multiply_fw_workspace_bytes(const bf_problem *p);

/* Workspace the backward call needs for this problem, in bytes. */
size_t bf_butterfly_multiply_bw_workspace_bytes(const bf_problem *p);

/* Backward multiply: d_twiddle (dense, twiddle shape, fully overwritten) and d_input
 * (B, S, I) with columns >= n zero-filled.  The batch reduction of d_twiddle uses no
 * atomics: per-workgroup partial sums then a fixed-order second pass, so results are
 * bitwise reproducible run to run.
 * Replaces butterfly_multiply_bw_cuda / butterfly_multiply_bw_cpu behind
 * torch_butterfly::butterfly_multiply_bw (csrc/butterfly.cpp:56-93,
 * csrc/cpu/butterfly_cpu.cpp:68-177, csrc/cuda/butterfly_cuda.cu:534-646).            */
int bf_butterfly_multiply_bw(const bf_problem *p, const void *twiddle, const void *input,
                             const void *grad, void *d_twiddle, void *d_input,
                             void *workspace, size_t workspace_bytes, void *stream);

/* Forward multiply with the layer bias folded into the last pass:
 * output[b][s][c] = multiply(...)[b][s][c] + bias[s][c], bias (S, O) dense (NULL = no bias).
 * Stands where Butterfly.post_process adds the bias as a separate elementwise pass over
 * the output (torch_butterfly/butterfly.py:152-169).  Workspace as for
 * bf_butterfly_multiply_fw.                                                            */
int bf_butterfly_multiply_bias_fw(const bf_problem *p, const void *twiddle, const void *input,
                                  const void *bias, void *output, void *workspace,
                                  size_t workspace_bytes, void *stream);

/* Bias gradient of such a layer: d_bias[s][c] = sum over b of grad[b][s][c], d_bias (S, O)
 * dense, fully overwritten; what autograd derives for the `+ bias` of
 * torch_butterfly/butterfly.py:167-168.  Only batch, nstacks, output_size, dtype and
 * output_stride (the strides of grad) of the problem are used.  Fixed summation order:
 * bitwise reproducible.                                                                */
int bf_butterfly_bias_grad(const bf_problem *p, const void *grad, void *d_bias, void *workspace,
                           size_t workspace_bytes, void *stream);

size_t bf_butterfly_bias_grad_workspace_bytes(const bf_problem *p);

/* Backward multiply that also returns the bias gradient of the layer: as
 * bf_butterfly_multiply_bw, plus d_bias (S, O) = sum over b of grad[b][s][c].  Where the
 * kernel that reads grad can do it (float, rows or chunks of 1024) it forms the column sums
 * on the way, so grad is not read a second time; otherwise this is
 * bf_butterfly_multiply_bw followed by bf_butterfly_bias_grad.  No counterpart in the
 * reference's op set (autograd's sum for torch_butterfly/butterfly.py:167-168).          */
int bf_butterfly_multiply_bias_bw(const bf_problem *p, const void *twiddle, const void *input,
                                  const void *grad, void *d_twiddle, void *d_input, void *d_bias,
                                  void *workspace, size_t workspace_bytes, void *stream);

size_t bf_butterfly_multiply_bias_bw_workspace_bytes(const bf_problem *p);

/* Forward multiply between two fixed permutations of the columns, folded into the first read
 * and the last write of the schedule instead of running as gathers of their own:
 *   u[c]                 = pad(input)[in_perm[c]]   (in_perm NULL: u = pad(input))
 *   y                    = multiply(u) + bias       (bias (S, O) dense, indexed by c; NULL: none)
 *   output[out_index[c]] = y[c]                     (out_index NULL: output[c] = y[c];
 *                                                    entries >= output_size are dropped)
 * in_perm, out_index: device tables of n 32-bit entries, each a permutation of 0..n-1;
 * input_size <= n.  A FixedPermutation(q) module behind the layer, out[i] = y[q[i]], is
 * out_index = inverse of q.  Stands where FixedPermutation runs next to Butterfly as a
 * separate pass over the activations (torch_butterfly/permutation.py:55-78, as built by
 * torch_butterfly/special.py:17-66 for the FFT).  Workspace as for bf_butterfly_multiply_fw. */
int bf_butterfly_multiply_perm_fw(const bf_problem *p, const void *twiddle, const void *input,
                                  const int32_t *in_perm, const int32_t *out_index,
                                  const void *bias, void *output, void *workspace,
                                  size_t workspace_bytes, void *stream);

/* Backward of bf_butterfly_multiply_perm_fw: grad is read through out_index, input through
 * in_perm, and d_input[in_perm[c]] receives the gradient of u[c].  d_bias (S, O) may be NULL.
 * Workspace: bf_butterfly_multiply_bias_bw_workspace_bytes when d_bias is given, otherwise
 * bf_butterfly_multiply_bw_workspace_bytes.                                               */
int bf_butterfly_multiply_perm_bw(const bf_problem *p, const void *twiddle, const void *input,
                                  const void *grad, const int32_t *in_perm,
                                  const int32_t *out_index, void *d_twiddle, void *d_input,
                                  void *d_bias, void *workspace, size_t workspace_bytes,
                                  void *stream);

/* Forward and backward of a pair that share their intermediate activations.  A backward call
 * that runs in several passes (rows longer than 1024, more than two blocks) needs the activation
 * entering every pass after the first, and bf_butterfly_multiply_bw recomputes them with forward
 * launches of its own.  bf_butterfly_multiply_fw_saving runs the forward along the backward's
 * pass plan and leaves those activations in `saved` (bf_butterfly_multiply_saved_bytes bytes:
 * one dense (B, S, n) plane per pass after the first; 0 = single pass, nothing to save, use the
 * plain calls); bf_butterfly_multiply_bw_saved reads them instead of recomputing.  `bias` as in
 * bf_butterfly_multiply_bias_fw, in_perm / out_index as in bf_butterfly_multiply_perm_fw / _bw
 * (each may be NULL).  What the reference's autograd Function would
 * keep between its forward and backward (csrc/butterfly.cpp:99-118 saves twiddle and input only
 * and its backward recomputes everything, csrc/cuda/butterfly_cuda.cu:534-646).             */
size_t bf_butterfly_multiply_saved_bytes(const bf_problem *p);
int bf_butterfly_multiply_fw_saving(const bf_problem *p, const void *twiddle, const void *input,
                                    const void *bias, const int32_t *in_perm,
                                    const int32_t *out_index, void *output, void *saved,
                                    size_t saved_capacity, void *stream);
size_t bf_butterfly_multiply_bw_saved_workspace_bytes(const bf_problem *p, int with_bias);
/* d_bias (S, O) may be NULL; when given it receives the column sums of grad as in
 * bf_butterfly_multiply_bias_bw (size the workspace with with_bias != 0).  saved_bytes: size of
 * the area behind `saved`; the call plans from ITS problem (strides of grad and d_input, column
 * tables) which planes it reads and answers BF_ERR_WORKSPACE when the area is smaller than
 * that, BF_ERR_INVALID when that plan reads none (then use bf_butterfly_multiply_bw).        */
int bf_butterfly_multiply_bw_saved(const bf_problem *p, const void *twiddle, const void *input,
                                   const void *grad, const void *saved, size_t saved_bytes,
                                   const int32_t *in_perm, const int32_t *out_index,
                                   void *d_twiddle, void *d_input, void *d_bias, void *workspace,
                                   size_t workspace_bytes, void *stream);

/* Diagnostic, host only (no device call): how the base-2 forward (backward != 0: backward)
 * call for this problem is cut into launches, one text line per pass in order --
 *   "low t=A..B L=.. nb=.. inc=.. chunks=.."   stages A..B-1 on bits 0..9, 1024-element chunks
 *   "wide t=A..B L=.. inc=.."                   one whole block of a 2048 / 4096 row (forward)
 *   "span t=A..B lb=.. bits=.. mode=.. tiles=.." stages on `bits` adjacent bits from bit lb up
 *                                               (mode 0 one sweep up, 1 down, 2 up then down)
 *   "generic"                                   the LDS fallback kernels
 * No counterpart in the reference (its launch plan is butterfly_max5_plan,
 * csrc/cuda/butterfly_cuda.cu:317-345, internal to the operator).                       */
int bf_describe_plan(const bf_problem *p, int backward, char *text, size_t capacity);

/* Diagonal matrices directly in front of and behind a butterfly product, folded into its
 * factors: scaled = the factors of diag(out_scale) B diag(in_scale), i.e. twiddle
 * (S, nblocks, log_n, n/2, 2, 2) with the columns of the first applied factor multiplied by
 * in_scale and the rows of the last applied one by out_scale.  in_scale: in_len <= n entries
 * (every stack reads the same input); out_scale: out_len <= S * n entries (the stacks'
 * outputs side by side); entries past the lengths count as 1, either pointer may be NULL.
 * All tensors dense, of the given dtype; no workspace.  Replaces the elementwise passes of
 * Diagonal modules next to a Butterfly (torch_butterfly/diagonal.py:31-38, as chained by
 * torch_butterfly/special.py:364-391 and :684-711) by work on the factors alone.          */
int bf_butterfly_scale_twiddle(int dtype, int64_t nstacks, int64_t nblocks, int64_t log_n,
                               int increasing_stride, const void *twiddle, const void *in_scale,
                               int64_t in_len, const void *out_scale, int64_t out_len,
                               void *scaled, void *stream);

/* Its backward: from grad, the gradient with respect to `scaled`, d_twiddle (shape of
 * twiddle), d_in_scale (in_len entries) and d_out_scale (out_len entries), all fully
 * overwritten; PyTorch's convention for complex gradients; fixed summation order.        */
int bf_butterfly_scale_twiddle_bw(int dtype, int64_t nstacks, int64_t nblocks, int64_t log_n,
                                  int increasing_stride, const void *twiddle, const void *in_scale,
                                  int64_t in_len, const void *out_scale, int64_t out_len,
                                  const void *grad, void *d_twiddle, void *d_in_scale,
                                  void *d_out_scale, void *stream);

/* Base-4 forward: per block log_n/2 radix-4 stages from twiddle4
 * (S, nb, log_n/2, n/4, 4, 4), then one 2x2 stage from twiddle2 (S, nb, 1, n/2, 2, 2)
 * when log_n is odd (twiddle2 may be NULL when log_n is even).  twiddle4 (and, backward,
 * d_twiddle4 / d_twiddle2) dense and 16-byte aligned.
 * Native counterpart of butterfly_multiply_base4_torch
 * (torch_butterfly/multiply_base4.py:7-41), which the reference runs as PyTorch ops. */
int bf_butterfly_multiply_base4_fw(const bf_problem *p, const void *twiddle4,
                                   const void *twiddle2, const void *input, void *output,
                                   void *workspace, size_t workspace_bytes, void *stream);

size_t bf_butterfly_multiply_base4_fw_workspace_bytes(const bf_problem *p);

size_t bf_butterfly_multiply_base4_bw_workspace_bytes(const bf_problem *p);

/* Base-4 backward: what autograd derives for multiply_base4.py:7-41.
 * d_twiddle2 may be NULL when log_n is even.                                          */
int bf_butterfly_multiply_base4_bw(const bf_problem *p, const void *twiddle4,
                                   const void *twiddle2, const void *input, const void *grad,
                                   void *d_twiddle4, void *d_twiddle2, void *d_input,
                                   void *workspace, size_t workspace_bytes, void *stream);

/* The base-4 pair that shares its intermediate activations, as bf_butterfly_multiply_fw_saving /
 * _bw_saved do for base 2: several blocks (rows up to 1024) or several passes (longer rows) make
 * bf_butterfly_multiply_base4_bw recompute the activation entering each after the first; the
 * saving forward leaves them in `saved` (bf_butterfly_multiply_base4_saved_bytes; 0 = nothing to
 * save, use the plain calls) and the backward reads them.  What autograd keeps for
 * butterfly_multiply_base4_torch (torch_butterfly/multiply_base4.py:7-41) is every stage's
 * expanded temporaries; this keeps one (B, S, n) plane per pass.                             */
size_t bf_butterfly_multiply_base4_saved_bytes(const bf_problem *p);
int bf_butterfly_multiply_base4_fw_saving(const bf_problem *p, const void *twiddle4,
                                          const void *twiddle2, const void *input, void *output,
                                          void *saved, size_t saved_capacity, void *stream);
size_t bf_butterfly_multiply_base4_bw_saved_workspace_bytes(const bf_problem *p);
int bf_butterfly_multiply_base4_bw_saved(const bf_problem *p, const void *twiddle4,
                                         const void *twiddle2, const void *input,
                                         const void *grad, const void *saved, size_t saved_bytes,
                                         void *d_twiddle4, void *d_twiddle2, void *d_input,
                                         void *workspace, size_t workspace_bytes, void *stream);

/* bf_butterfly_multiply_bw for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same operands and results,
 * but the partial sums and intermediate activations live in a fixed area of
 * BF_NOALLOC_SCRATCH_BYTES that is part of the library's device image (one copy per GPU, held
 * until the process ends) instead of a workspace argument.  No counterpart in the reference.
 * The call allocates and frees nothing.  A problem whose backward workspace
 * (bf_butterfly_multiply_bw_workspace_bytes) exceeds the area is refused with
 * BF_ERR_WORKSPACE.  The device that is current must be the one `stream` belongs to.  All
 * calls on one GPU share that GPU's area: calls that overlap in time on one GPU (different
 * streams or threads) race; calls ordered on one stream are fine.  The first call on a device
 * looks the area's address up (a host-side query, no allocation); make that call outside a
 * stream capture.                                                                         */
#define BF_NOALLOC_SCRATCH_BYTES ((size_t)48 << 20)
int bf_butterfly_multiply_bw_noalloc(const bf_problem *p, const void *twiddle, const void *input,
                                     const void *grad, void *d_twiddle, void *d_input,
                                     void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BUTTERFLY_HIP_H */
