// torch-library shim: registers the torch_butterfly operators and forwards them to the
// C ABI of libbutterfly_hip.so.  No kernels live here.
//
// Operator names, argument order and checks follow the reference shim
// (csrc/butterfly.cpp:20-131): twiddle first, then input, the stride flag and the
// optional output size.  The base-4 operators are new; their argument order follows
// butterfly_multiply_base4_torch (torch_butterfly/multiply_base4.py:7-8).
//
// Device tensors go to the HIP library and nowhere else.  Host tensors are accepted by the three
// operators the reference has (butterfly_multiply, _fw, _bw), in float, double, complex64 and
// complex128 as there (csrc/butterfly.cpp:44-52, 84-92), and run on the single-threaded host
// path of host_path.hpp; the operators that are new here take device tensors only.

#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/csrc/autograd/custom_function.h>
#include <torch/library.h>

#include <tuple>

#include "../../include/butterfly_hip.h"
#include "host_path.hpp"

namespace {

using at::Tensor;

#define CHECK_DEVICE(x) \
    TORCH_CHECK(x.device().type() == at::kCPU || x.device().type() == at::kCUDA, #x " must be on CPU or CUDA")
#define CHECK_SAME_DEVICE(x, y) TORCH_CHECK(x.device() == y.device(), #x " and " #y " must be on the same device")
#define CHECK_DIM(x, y) TORCH_CHECK(x.dim() == y, #x " must have dimension " #y)
#define CHECK_SHAPE(x, ...) \
    TORCH_CHECK(x.sizes() == at::IntArrayRef({__VA_ARGS__}), #x " must have shape (" #__VA_ARGS__ ")")

int dtype_code(const Tensor &t, const char *who)
{
    if (t.scalar_type() == at::kFloat) return BF_F32;
    if (t.scalar_type() == at::kComplexFloat) return BF_C64;
    TORCH_CHECK(false, who, ": device kernels support float32 and complex64, got ", t.scalar_type());
    return -1;
}

void require_device(const Tensor &t, const char *who)
{
    TORCH_CHECK(t.is_cuda(), who, ": tensors must live on a HIP device; this operator has no CPU path");
}

// ---- host tensors ---------------------------------------------------------------------------

bf_host::Shape host_shape(int64_t batch, int64_t nstacks, int64_t log_n, int64_t nblocks, int64_t input_size,
                          int64_t output_size, bool increasing_stride)
{
    bf_host::Shape sh;
    sh.batch = batch;
    sh.nstacks = nstacks;
    sh.log_n = log_n;
    sh.nblocks = nblocks;
    sh.input_size = input_size;
    sh.output_size = output_size;
    sh.increasing_stride = increasing_stride;
    return sh;
}

void host_strides(int64_t dst[3], const Tensor &t)
{
    for (int i = 0; i < 3; ++i) dst[i] = t.stride(i);
}

// Calls f(T()) with T the host path's scalar type for the tensor's dtype.
template <typename F>
void host_dispatch(const Tensor &t, const char *who, F &&f)
{
    switch (t.scalar_type()) {
        case at::kFloat: f(float()); break;
        case at::kDouble: f(double()); break;
        case at::kComplexFloat: f(bf_host::Cplx<float>()); break;
        case at::kComplexDouble: f(bf_host::Cplx<double>()); break;
        default: TORCH_CHECK(false, who, " not implemented for '", t.scalar_type(), "'");
    }
}

Tensor host_multiply_fw(const Tensor &twiddle, const Tensor &input, bool increasing_stride, int64_t log_n,
                        int64_t output_size, const char *who)
{
    const Tensor tw = twiddle.resolve_conj().contiguous();
    const Tensor x = input.resolve_conj();
    const int64_t n = (int64_t)1 << log_n;
    Tensor output = at::empty({x.size(0), x.size(1), n}, x.options());
    if (output_size < n) output = output.slice(2, 0, output_size);
    const bf_host::Shape sh = host_shape(x.size(0), x.size(1), log_n, tw.size(1), x.size(2), output_size, increasing_stride);
    int64_t xs[3], os[3];
    host_strides(xs, x);
    host_strides(os, output);
    host_dispatch(x, who, [&](auto tag) {
        using T = decltype(tag);
        bf_host::multiply_fw<T>(sh, static_cast<const T *>(tw.data_ptr()), static_cast<const T *>(x.data_ptr()), xs,
                                static_cast<T *>(output.data_ptr()), os);
    });
    return output;
}

std::tuple<Tensor, Tensor> host_multiply_bw(const Tensor &twiddle, const Tensor &input, const Tensor &grad,
                                            bool increasing_stride, int64_t log_n, const char *who)
{
    const Tensor tw = twiddle.resolve_conj().contiguous();
    const Tensor x = input.resolve_conj();
    const Tensor g = grad.resolve_conj();
    const int64_t n = (int64_t)1 << log_n;
    const int64_t input_size = x.size(2);
    Tensor d_twiddle = at::empty(tw.sizes(), tw.options());
    Tensor d_input = at::empty({x.size(0), x.size(1), std::max(input_size, n)}, x.options());
    if (input_size < n) d_input = d_input.slice(2, 0, input_size);
    const bf_host::Shape sh = host_shape(x.size(0), x.size(1), log_n, tw.size(1), input_size, g.size(2), increasing_stride);
    int64_t xs[3], gs[3], ds[3];
    host_strides(xs, x);
    host_strides(gs, g);
    host_strides(ds, d_input);
    host_dispatch(x, who, [&](auto tag) {
        using T = decltype(tag);
        bf_host::multiply_bw<T>(sh, static_cast<const T *>(tw.data_ptr()), static_cast<const T *>(x.data_ptr()), xs,
                                static_cast<const T *>(g.data_ptr()), gs, static_cast<T *>(d_twiddle.data_ptr()),
                                static_cast<T *>(d_input.data_ptr()), ds);
    });
    return std::make_tuple(d_twiddle, d_input);
}

void set_strides(int64_t dst[3], const Tensor &t)
{
    for (int i = 0; i < 3; ++i) dst[i] = t.size(i) > 1 ? t.stride(i) : 0;
    for (int i = 0; i < 3; ++i) TORCH_CHECK(dst[i] >= 0, "negative strides are not supported");
}

// PyTorch on ROCm presents HIP devices under the "cuda" device type; these are the stream
// and guard types that go with that.
void *current_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

void check_rc(int rc, const char *who) { TORCH_CHECK(rc == BF_OK, who, ": ", bf_last_error()); }

// Answer of one of the library's size queries: BF_SIZE_INVALID means the problem was refused.
size_t valid_size(size_t bytes)
{
    TORCH_CHECK(bytes != BF_SIZE_INVALID, "torch_butterfly: ", bf_last_error());
    return bytes;
}

// Dense copy of a (small) twiddle tensor; also materialises lazy conjugation.
// dense and 16-byte aligned (the kernels read factor blocks with 16-byte loads): a contiguous view
// at an odd offset into its storage is copied
Tensor dense(const Tensor &t)
{
    Tensor d = t.resolve_conj().contiguous();
    if (d.numel() > 0 && (reinterpret_cast<uintptr_t>(d.data_ptr()) & 15) != 0) d = d.clone();
    return d;
}

struct Shapes {
    int64_t batch, nstacks, nblocks, log_n, n, input_size;
};

bf_problem make_problem(const Shapes &s, const Tensor &input, bool increasing_stride, int64_t output_size,
                        const char *who)
{
    bf_problem p = {};
    p.dtype = dtype_code(input, who);
    p.increasing_stride = increasing_stride;
    p.batch = s.batch;
    p.nstacks = s.nstacks;
    p.log_n = s.log_n;
    p.nblocks = s.nblocks;
    p.input_size = s.input_size;
    p.output_size = output_size;
    set_strides(p.input_stride, input);
    return p;
}

// ---- base-2 -----------------------------------------------------------------------------

// A column table of the *_perm operators: int32, n entries, dense, on the device of `like`.
// Its entries are the caller's responsibility (each table a permutation of 0..n-1).
const int32_t *table_ptr(const Tensor &t, Tensor &keep, const Tensor &like, int64_t n, const char *name,
                         const char *who)
{
    if (!t.defined()) return nullptr;
    TORCH_CHECK(t.device() == like.device(), who, ": ", name, " must be on the device of input");
    TORCH_CHECK(t.scalar_type() == at::kInt, who, ": ", name, " must be int32");
    TORCH_CHECK(t.dim() == 1 && t.size(0) == n, who, ": ", name, " must have n entries");
    keep = t.contiguous();
    return keep.data_ptr<int32_t>();
}

// Shared body of the forward operators (`bias`, `in_perm`, `out_index` undefined = none).
// keep (may be NULL): where the call may leave the intermediate activations that a backward in
// several passes would otherwise recompute; defined on return when it did.
Tensor multiply_fw_impl(const Tensor &twiddle, const Tensor &input, const Tensor &bias, bool increasing_stride,
                        c10::optional<int64_t> output_size, const char *who, const Tensor &in_perm = Tensor(),
                        const Tensor &out_index = Tensor(), Tensor *keep = nullptr)
{
    CHECK_DEVICE(twiddle); CHECK_DEVICE(input); CHECK_SAME_DEVICE(twiddle, input);
    CHECK_DIM(twiddle, 6); CHECK_DIM(input, 3);
    Shapes s;
    s.batch = input.size(0);
    s.nstacks = input.size(1);
    s.input_size = input.size(2);
    s.nblocks = twiddle.size(1);
    s.log_n = twiddle.size(2);
    TORCH_CHECK(s.log_n <= 30, who, ": n must be a power of 2");
    s.n = (int64_t)1 << s.log_n;
    CHECK_SHAPE(twiddle, s.nstacks, s.nblocks, s.log_n, s.n / 2, 2, 2);
    const int64_t output_size_val = output_size.has_value() ? output_size.value() : s.n;
    TORCH_CHECK(output_size_val <= s.n, who, ": output_size must be <= n");
    TORCH_CHECK(output_size_val >= 0, who, ": output_size must be >= 0");
    TORCH_CHECK(twiddle.scalar_type() == input.scalar_type(), who, ": twiddle and input must have the same dtype");
    if (input.is_cpu() && !bias.defined() && !in_perm.defined() && !out_index.defined())
        return host_multiply_fw(twiddle, input, increasing_stride, s.log_n, output_size_val, who);
    require_device(input, who);
    Tensor b;
    if (bias.defined()) {
        CHECK_DEVICE(bias); CHECK_SAME_DEVICE(bias, input);
        CHECK_DIM(bias, 2);
        CHECK_SHAPE(bias, s.nstacks, output_size_val);
        TORCH_CHECK(bias.scalar_type() == input.scalar_type(), who, ": bias and input must have the same dtype");
        b = dense(bias);
    }

    const c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    const Tensor tw = dense(twiddle);
    const Tensor x = input.resolve_conj();
    Tensor output = at::empty({s.batch, s.nstacks, s.n}, x.options());
    if (output_size_val < s.n) output = output.slice(2, 0, output_size_val);
    bf_problem p = make_problem(s, x, increasing_stride, output_size_val, who);
    set_strides(p.output_stride, output);
    Tensor keep_in, keep_out;
    const int32_t *ip = table_ptr(in_perm, keep_in, x, s.n, "in_perm", who);
    const int32_t *oi = table_ptr(out_index, keep_out, x, s.n, "out_index", who);
    if (ip || oi) TORCH_CHECK(s.input_size <= s.n, who, ": column tables need input_size <= n");
    if (keep) {
        // (the backward will make d_input dense over max(input_size, n) columns: same plan)
        const int64_t dw = std::max(s.input_size, s.n);
        p.d_input_stride[0] = s.batch > 1 ? s.nstacks * dw : 0;
        p.d_input_stride[1] = s.nstacks > 1 ? dw : 0;
        p.d_input_stride[2] = s.input_size > 1 ? 1 : 0;
        const size_t nsaved = valid_size(bf_butterfly_multiply_saved_bytes(&p));
        if (nsaved > 0) {
            *keep = at::empty({(int64_t)nsaved}, x.options().dtype(at::kByte));
            check_rc(bf_butterfly_multiply_fw_saving(&p, tw.data_ptr(), x.data_ptr(), b.defined() ? b.data_ptr() : nullptr,
                                                     ip, oi, output.data_ptr(), keep->data_ptr(), nsaved,
                                                     current_stream()),
                     who);
            return output;
        }
    }
    const size_t ws_bytes = valid_size(bf_butterfly_multiply_fw_workspace_bytes(&p));
    Tensor ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
    if (ip || oi) {
        check_rc(bf_butterfly_multiply_perm_fw(&p, tw.data_ptr(), x.data_ptr(), ip, oi,
                                               b.defined() ? b.data_ptr() : nullptr, output.data_ptr(),
                                               ws.data_ptr(), ws_bytes, current_stream()),
                 who);
        return output;
    }
    check_rc(bf_butterfly_multiply_bias_fw(&p, tw.data_ptr(), x.data_ptr(), b.defined() ? b.data_ptr() : nullptr,
                                           output.data_ptr(), ws.data_ptr(), ws_bytes, current_stream()),
             who);
    return output;
}

Tensor butterfly_multiply_fw(const Tensor twiddle, const Tensor input, bool increasing_stride,
                             c10::optional<int64_t> output_size)
{
    return multiply_fw_impl(twiddle, input, Tensor(), increasing_stride, output_size, "butterfly_multiply_fw");
}

// New operators (no counterpart in the reference's op set): the layer bias folded into the
// multiply, where Butterfly.post_process runs a separate elementwise pass
// (torch_butterfly/butterfly.py:152-169).  bias: (nstacks, output_size).
Tensor butterfly_multiply_bias_fw(const Tensor twiddle, const Tensor input, const Tensor bias,
                                  bool increasing_stride, c10::optional<int64_t> output_size)
{
    TORCH_CHECK(bias.defined(), "butterfly_multiply_bias_fw: bias is undefined");
    return multiply_fw_impl(twiddle, input, bias, increasing_stride, output_size, "butterfly_multiply_bias_fw");
}

// d_bias (nstacks, output_size) = sum of grad (batch, nstacks, output_size) over the batch.
Tensor butterfly_bias_grad(const Tensor grad)
{
    CHECK_DEVICE(grad);
    CHECK_DIM(grad, 3);
    require_device(grad, "butterfly_bias_grad");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(grad.device());
    const Tensor g = grad.resolve_conj();
    bf_problem p = {};
    p.dtype = dtype_code(g, "butterfly_bias_grad");
    p.batch = g.size(0);
    p.nstacks = g.size(1);
    p.output_size = g.size(2);
    p.input_size = g.size(2);
    p.nblocks = 1;
    p.log_n = 1;
    while (((int64_t)1 << p.log_n) < p.output_size) ++p.log_n;
    set_strides(p.output_stride, g);
    Tensor d_bias = at::empty({p.nstacks, p.output_size}, g.options());
    const size_t ws_bytes = valid_size(bf_butterfly_bias_grad_workspace_bytes(&p));
    Tensor ws = at::empty({(int64_t)ws_bytes}, g.options().dtype(at::kByte));
    check_rc(bf_butterfly_bias_grad(&p, g.data_ptr(), d_bias.data_ptr(), ws.data_ptr(), ws_bytes, current_stream()),
             "butterfly_bias_grad");
    return d_bias;
}

// Shared body of the backward operators.
// kept: what the forward left in its `keep` (undefined: the backward recomputes what it needs)
std::tuple<Tensor, Tensor, Tensor> multiply_bw_impl(const Tensor &twiddle, const Tensor &input, const Tensor &grad,
                                                    bool increasing_stride, bool with_bias, const char *who,
                                                    const Tensor &in_perm = Tensor(),
                                                    const Tensor &out_index = Tensor(), const Tensor &kept = Tensor())
{
    CHECK_DEVICE(twiddle); CHECK_DEVICE(input); CHECK_DEVICE(grad);
    CHECK_SAME_DEVICE(twiddle, input); CHECK_SAME_DEVICE(input, grad);
    CHECK_DIM(twiddle, 6); CHECK_DIM(input, 3); CHECK_DIM(grad, 3);
    Shapes s;
    s.batch = input.size(0);
    s.nstacks = input.size(1);
    s.input_size = input.size(2);
    s.nblocks = twiddle.size(1);
    s.log_n = twiddle.size(2);
    TORCH_CHECK(s.log_n <= 30, who, ": n must be a power of 2");
    s.n = (int64_t)1 << s.log_n;
    const int64_t output_size = grad.size(2);
    CHECK_SHAPE(twiddle, s.nstacks, s.nblocks, s.log_n, s.n / 2, 2, 2);
    CHECK_SHAPE(grad, s.batch, s.nstacks, output_size);
    TORCH_CHECK(output_size <= s.n, who, ": grad must have at most n columns");
    TORCH_CHECK(twiddle.scalar_type() == input.scalar_type() && grad.scalar_type() == input.scalar_type(), who,
                ": twiddle, input and grad must have the same dtype");
    if (input.is_cpu() && !with_bias && !in_perm.defined() && !out_index.defined()) {
        auto r = host_multiply_bw(twiddle, input, grad, increasing_stride, s.log_n, who);
        return std::make_tuple(std::get<0>(r), std::get<1>(r), Tensor());
    }
    require_device(input, who);

    const c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    const Tensor tw = dense(twiddle);
    const Tensor x = input.resolve_conj();
    const Tensor g = grad.resolve_conj();
    Tensor d_twiddle = at::empty(tw.sizes(), tw.options());
    Tensor d_input = at::empty({s.batch, s.nstacks, std::max(s.input_size, s.n)}, x.options());
    if (s.input_size < s.n) d_input = d_input.slice(2, 0, s.input_size);
    bf_problem p = make_problem(s, x, increasing_stride, output_size, who);
    set_strides(p.output_stride, g);
    set_strides(p.d_input_stride, d_input);
    Tensor d_bias;
    Tensor keep_in, keep_out;
    const int32_t *ip = table_ptr(in_perm, keep_in, x, s.n, "in_perm", who);
    const int32_t *oi = table_ptr(out_index, keep_out, x, s.n, "out_index", who);
    // The forward decided what to keep from a plan made with its own strides; the backward plans
    // from the strides of grad and d_input.  Where that plan reads no kept activations, or more
    // than the forward left, the recomputing call serves the request.
    bool use_kept = kept.defined();
    if (use_kept) {
        const size_t reads = valid_size(bf_butterfly_multiply_saved_bytes(&p));
        if (reads == 0 || reads > (size_t)kept.numel()) use_kept = false;
    }
    if (use_kept) {
        if (ip || oi) TORCH_CHECK(s.input_size <= s.n, who, ": column tables need input_size <= n");
        if (with_bias) d_bias = at::empty({s.nstacks, output_size}, g.options());
        const size_t ws_bytes = valid_size(bf_butterfly_multiply_bw_saved_workspace_bytes(&p, with_bias ? 1 : 0));
        Tensor ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
        check_rc(bf_butterfly_multiply_bw_saved(&p, tw.data_ptr(), x.data_ptr(), g.data_ptr(), kept.data_ptr(),
                                                (size_t)kept.numel(), ip, oi,
                                                d_twiddle.data_ptr(), d_input.data_ptr(),
                                                with_bias ? d_bias.data_ptr() : nullptr, ws.data_ptr(), ws_bytes,
                                                current_stream()),
                 who);
    } else if (ip || oi) {
        TORCH_CHECK(s.input_size <= s.n, who, ": column tables need input_size <= n");
        if (with_bias) d_bias = at::empty({s.nstacks, output_size}, g.options());
        const size_t ws_bytes = with_bias ? valid_size(bf_butterfly_multiply_bias_bw_workspace_bytes(&p))
                                          : valid_size(bf_butterfly_multiply_bw_workspace_bytes(&p));
        Tensor ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
        check_rc(bf_butterfly_multiply_perm_bw(&p, tw.data_ptr(), x.data_ptr(), g.data_ptr(), ip, oi,
                                               d_twiddle.data_ptr(), d_input.data_ptr(),
                                               with_bias ? d_bias.data_ptr() : nullptr, ws.data_ptr(), ws_bytes,
                                               current_stream()),
                 who);
    } else if (with_bias) {
        d_bias = at::empty({s.nstacks, output_size}, g.options());
        const size_t ws_bytes = valid_size(bf_butterfly_multiply_bias_bw_workspace_bytes(&p));
        Tensor ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
        check_rc(bf_butterfly_multiply_bias_bw(&p, tw.data_ptr(), x.data_ptr(), g.data_ptr(), d_twiddle.data_ptr(),
                                               d_input.data_ptr(), d_bias.data_ptr(), ws.data_ptr(), ws_bytes,
                                               current_stream()),
                 who);
    } else {
        const size_t ws_bytes = valid_size(bf_butterfly_multiply_bw_workspace_bytes(&p));
        Tensor ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
        check_rc(bf_butterfly_multiply_bw(&p, tw.data_ptr(), x.data_ptr(), g.data_ptr(), d_twiddle.data_ptr(),
                                          d_input.data_ptr(), ws.data_ptr(), ws_bytes, current_stream()),
                 who);
    }
    return std::make_tuple(d_twiddle, d_input, d_bias);
}

std::tuple<Tensor, Tensor> butterfly_multiply_bw(const Tensor twiddle, const Tensor input,
                                                 const Tensor grad, bool increasing_stride)
{
    auto r = multiply_bw_impl(twiddle, input, grad, increasing_stride, false, "butterfly_multiply_bw");
    return std::make_tuple(std::get<0>(r), std::get<1>(r));
}

// (d_twiddle, d_input, d_bias): the backward of butterfly_multiply_bias_fw
std::tuple<Tensor, Tensor, Tensor> butterfly_multiply_bias_bw(const Tensor twiddle, const Tensor input,
                                                              const Tensor grad, bool increasing_stride)
{
    return multiply_bw_impl(twiddle, input, grad, increasing_stride, true, "butterfly_multiply_bias_bw");
}

using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

class ButterflyMultiply : public torch::autograd::Function<ButterflyMultiply> {
public:
    // wants_grad: a gradient will be asked for.  The forward then runs along the backward's pass
    // plan and keeps the activations between the passes (device tensors whose backward takes
    // several passes: rows beyond 1024, more than two blocks), which the reference's Function
    // (csrc/butterfly.cpp:99-118) leaves to its backward to recompute.
    static Tensor forward(AutogradContext *ctx, Tensor twiddle, Tensor input, bool increasing_stride,
                          c10::optional<int64_t> output_size, bool wants_grad)
    {
        ctx->saved_data["increasing_stride"] = increasing_stride;
        Tensor kept;
        Tensor out = multiply_fw_impl(twiddle, input, Tensor(), increasing_stride, output_size, "butterfly_multiply",
                                      Tensor(), Tensor(), wants_grad && input.is_cuda() ? &kept : nullptr);
        ctx->saved_data["kept"] = kept.defined();
        if (kept.defined()) ctx->save_for_backward({twiddle, input, kept});
        else ctx->save_for_backward({twiddle, input});
        return out;
    }

    static variable_list backward(AutogradContext *ctx, variable_list grad_output)
    {
        const auto saved = ctx->get_saved_variables();
        const bool increasing_stride = ctx->saved_data["increasing_stride"].toBool();
        const Tensor kept = ctx->saved_data["kept"].toBool() ? saved[2] : Tensor();
        auto result = multiply_bw_impl(saved[0], saved[1], grad_output[0], increasing_stride, false,
                                       "butterfly_multiply_bw", Tensor(), Tensor(), kept);
        return {std::get<0>(result), std::get<1>(result), Tensor(), Tensor(), Tensor()};
    }
};

bool grad_wanted(std::initializer_list<Tensor> ts)
{
    if (!at::GradMode::is_enabled()) return false;
    for (const Tensor &t : ts)
        if (t.defined() && t.requires_grad()) return true;
    return false;
}

Tensor butterfly_multiply(Tensor twiddle, Tensor input, bool increasing_stride,
                          c10::optional<int64_t> output_size)
{
    return ButterflyMultiply::apply(twiddle, input, increasing_stride, output_size, grad_wanted({twiddle, input}));
}

class ButterflyMultiplyBias : public torch::autograd::Function<ButterflyMultiplyBias> {
public:
    static Tensor forward(AutogradContext *ctx, Tensor twiddle, Tensor input, Tensor bias, bool increasing_stride,
                          c10::optional<int64_t> output_size, bool wants_grad)
    {
        TORCH_CHECK(bias.defined(), "butterfly_multiply_bias: bias is undefined");
        ctx->saved_data["increasing_stride"] = increasing_stride;
        Tensor kept;
        Tensor out = multiply_fw_impl(twiddle, input, bias, increasing_stride, output_size, "butterfly_multiply_bias",
                                      Tensor(), Tensor(), wants_grad && input.is_cuda() ? &kept : nullptr);
        ctx->saved_data["kept"] = kept.defined();
        if (kept.defined()) ctx->save_for_backward({twiddle, input, kept});
        else ctx->save_for_backward({twiddle, input});
        return out;
    }

    static variable_list backward(AutogradContext *ctx, variable_list grad_output)
    {
        const auto saved = ctx->get_saved_variables();
        const bool increasing_stride = ctx->saved_data["increasing_stride"].toBool();
        const Tensor kept = ctx->saved_data["kept"].toBool() ? saved[2] : Tensor();
        auto result = multiply_bw_impl(saved[0], saved[1], grad_output[0], increasing_stride, true,
                                       "butterfly_multiply_bias_bw", Tensor(), Tensor(), kept);
        return {std::get<0>(result), std::get<1>(result), std::get<2>(result), Tensor(), Tensor(), Tensor()};
    }
};

Tensor butterfly_multiply_bias(Tensor twiddle, Tensor input, Tensor bias, bool increasing_stride,
                               c10::optional<int64_t> output_size)
{
    return ButterflyMultiplyBias::apply(twiddle, input, bias, increasing_stride, output_size,
                                        grad_wanted({twiddle, input, bias}));
}

// New operators: the multiply between two fixed column permutations, folded into the first
// read and the last write (in front: u[c] = input[in_perm[c]]; behind: output[out_index[c]] =
// y[c]; bias (nstacks, output_size) indexed by c).  Where the reference chains FixedPermutation
// and Butterfly modules (torch_butterfly/special.py:17-66), each permutation costs a pass of
// its own over the activations.  Tables: int32 (n,), undefined = identity.
Tensor opt(const c10::optional<Tensor> &t) { return t.has_value() ? t.value() : Tensor(); }

Tensor butterfly_multiply_perm_fw(const Tensor twiddle, const Tensor input, c10::optional<Tensor> in_perm,
                                  c10::optional<Tensor> out_index, c10::optional<Tensor> bias,
                                  bool increasing_stride, c10::optional<int64_t> output_size)
{
    return multiply_fw_impl(twiddle, input, opt(bias), increasing_stride, output_size, "butterfly_multiply_perm_fw",
                            opt(in_perm), opt(out_index));
}

// (d_twiddle, d_input, d_bias); d_bias is undefined unless with_bias
std::tuple<Tensor, Tensor, Tensor> butterfly_multiply_perm_bw(const Tensor twiddle, const Tensor input,
                                                              const Tensor grad, c10::optional<Tensor> in_perm,
                                                              c10::optional<Tensor> out_index, bool with_bias,
                                                              bool increasing_stride)
{
    auto r = multiply_bw_impl(twiddle, input, grad, increasing_stride, with_bias, "butterfly_multiply_perm_bw",
                              opt(in_perm), opt(out_index));
    if (!with_bias) std::get<2>(r) = at::empty({0}, grad.options());  // the schema has no optional results
    return r;
}

class ButterflyMultiplyPerm : public torch::autograd::Function<ButterflyMultiplyPerm> {
public:
    static Tensor forward(AutogradContext *ctx, Tensor twiddle, Tensor input, c10::optional<Tensor> in_perm,
                          c10::optional<Tensor> out_index, c10::optional<Tensor> bias, bool increasing_stride,
                          c10::optional<int64_t> output_size, bool wants_grad)
    {
        ctx->saved_data["increasing_stride"] = increasing_stride;
        ctx->saved_data["with_bias"] = bias.has_value();
        ctx->saved_data["has_in"] = in_perm.has_value();
        ctx->saved_data["has_out"] = out_index.has_value();
        Tensor kept;
        Tensor out = multiply_fw_impl(twiddle, input, opt(bias), increasing_stride, output_size,
                                      "butterfly_multiply_perm", opt(in_perm), opt(out_index),
                                      wants_grad && input.is_cuda() ? &kept : nullptr);
        ctx->saved_data["kept"] = kept.defined();
        variable_list saved = {twiddle, input};
        if (in_perm.has_value()) saved.push_back(in_perm.value());
        if (out_index.has_value()) saved.push_back(out_index.value());
        if (kept.defined()) saved.push_back(kept);
        ctx->save_for_backward(saved);
        return out;
    }

    static variable_list backward(AutogradContext *ctx, variable_list grad_output)
    {
        const auto saved = ctx->get_saved_variables();
        const bool has_in = ctx->saved_data["has_in"].toBool(), has_out = ctx->saved_data["has_out"].toBool();
        c10::optional<Tensor> in_perm, out_index;
        size_t next = 2;
        if (has_in) in_perm = saved[next++];
        if (has_out) out_index = saved[next++];
        const Tensor kept = ctx->saved_data["kept"].toBool() ? saved[next++] : Tensor();
        const bool with_bias = ctx->saved_data["with_bias"].toBool();
        auto r = multiply_bw_impl(saved[0], saved[1], grad_output[0], ctx->saved_data["increasing_stride"].toBool(),
                                  with_bias, "butterfly_multiply_perm_bw", opt(in_perm), opt(out_index), kept);
        return {std::get<0>(r), std::get<1>(r), Tensor(), Tensor(), with_bias ? std::get<2>(r) : Tensor(), Tensor(),
                Tensor(), Tensor()};
    }
};

Tensor butterfly_multiply_perm(Tensor twiddle, Tensor input, c10::optional<Tensor> in_perm,
                               c10::optional<Tensor> out_index, c10::optional<Tensor> bias, bool increasing_stride,
                               c10::optional<int64_t> output_size)
{
    return ButterflyMultiplyPerm::apply(twiddle, input, in_perm, out_index, bias, increasing_stride, output_size,
                                        grad_wanted({twiddle, input, opt(bias)}));
}

// ---- diagonals folded into the factors ------------------------------------------------------
//
// twiddle (S, nb, log_n, n/2, 2, 2) -> the factors of diag(out_scale) B diag(in_scale): what a
// Diagonal module in front of / behind a Butterfly (torch_butterfly/diagonal.py:31-38) does to
// the activations, done to the first / last factor instead.  in_scale up to n entries,
// out_scale up to S * n, same dtype as twiddle; undefined = no diagonal on that side.
struct ScaleShapes {
    int64_t nstacks, nblocks, log_n;
};

ScaleShapes scale_shapes(const Tensor &twiddle, const Tensor &in_scale, const Tensor &out_scale, const char *who)
{
    CHECK_DEVICE(twiddle);
    CHECK_DIM(twiddle, 6);
    ScaleShapes s{twiddle.size(0), twiddle.size(1), twiddle.size(2)};
    TORCH_CHECK(s.log_n >= 1 && s.log_n <= 30 && s.nblocks >= 1, who, ": twiddle must have at least one factor");
    const int64_t n = (int64_t)1 << s.log_n;
    CHECK_SHAPE(twiddle, s.nstacks, s.nblocks, s.log_n, n / 2, 2, 2);
    dtype_code(twiddle, who);
    for (const Tensor *v : {&in_scale, &out_scale}) {
        if (!v->defined()) continue;
        TORCH_CHECK(v->device() == twiddle.device(), who, ": diagonals must be on the device of twiddle");
        TORCH_CHECK(v->dim() == 1, who, ": diagonals must be vectors");
        TORCH_CHECK(v->scalar_type() == twiddle.scalar_type(), who, ": diagonals must have the dtype of twiddle");
    }
    TORCH_CHECK(!in_scale.defined() || in_scale.size(0) <= n, who, ": in_scale has more than n entries");
    TORCH_CHECK(!out_scale.defined() || out_scale.size(0) <= s.nstacks * n, who,
                ": out_scale has more than nstacks * n entries");
    return s;
}

Tensor butterfly_scale_twiddle_fw(const Tensor twiddle, c10::optional<Tensor> in_scale,
                                  c10::optional<Tensor> out_scale, bool increasing_stride)
{
    const char *who = "butterfly_scale_twiddle_fw";
    const Tensor din = opt(in_scale), dout = opt(out_scale);
    const ScaleShapes s = scale_shapes(twiddle, din, dout, who);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(twiddle.device());
    const Tensor tw = dense(twiddle);
    const Tensor a = din.defined() ? dense(din) : din, b = dout.defined() ? dense(dout) : dout;
    Tensor out = at::empty_like(tw);
    check_rc(bf_butterfly_scale_twiddle(dtype_code(tw, who), s.nstacks, s.nblocks, s.log_n, increasing_stride,
                                        tw.data_ptr(), a.defined() ? a.data_ptr() : nullptr,
                                        a.defined() ? a.size(0) : 0, b.defined() ? b.data_ptr() : nullptr,
                                        b.defined() ? b.size(0) : 0, out.data_ptr(), current_stream()),
             who);
    return out;
}

// (d_twiddle, d_in_scale, d_out_scale); an empty tensor stands for the gradient of an absent diagonal
std::tuple<Tensor, Tensor, Tensor> butterfly_scale_twiddle_bw(const Tensor twiddle, c10::optional<Tensor> in_scale,
                                                              c10::optional<Tensor> out_scale, const Tensor grad,
                                                              bool increasing_stride)
{
    const char *who = "butterfly_scale_twiddle_bw";
    const Tensor din = opt(in_scale), dout = opt(out_scale);
    const ScaleShapes s = scale_shapes(twiddle, din, dout, who);
    CHECK_DEVICE(grad);
    TORCH_CHECK(grad.sizes() == twiddle.sizes() && grad.scalar_type() == twiddle.scalar_type() &&
                    grad.device() == twiddle.device(),
                who, ": grad must match twiddle in shape, dtype and device");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(twiddle.device());
    const Tensor tw = dense(twiddle), g = dense(grad);
    const Tensor a = din.defined() ? dense(din) : din, b = dout.defined() ? dense(dout) : dout;
    Tensor d_tw = at::empty_like(tw);
    Tensor d_a = at::empty({a.defined() ? a.size(0) : 0}, tw.options());
    Tensor d_b = at::empty({b.defined() ? b.size(0) : 0}, tw.options());
    check_rc(bf_butterfly_scale_twiddle_bw(dtype_code(tw, who), s.nstacks, s.nblocks, s.log_n, increasing_stride,
                                           tw.data_ptr(), a.defined() ? a.data_ptr() : nullptr,
                                           a.defined() ? a.size(0) : 0, b.defined() ? b.data_ptr() : nullptr,
                                           b.defined() ? b.size(0) : 0, g.data_ptr(), d_tw.data_ptr(),
                                           d_a.data_ptr(), d_b.data_ptr(), current_stream()),
             who);
    return {d_tw, d_a, d_b};
}

class ButterflyScaleTwiddle : public torch::autograd::Function<ButterflyScaleTwiddle> {
public:
    static Tensor forward(AutogradContext *ctx, Tensor twiddle, c10::optional<Tensor> in_scale,
                          c10::optional<Tensor> out_scale, bool increasing_stride)
    {
        ctx->saved_data["increasing_stride"] = increasing_stride;
        ctx->saved_data["has_in"] = in_scale.has_value();
        ctx->saved_data["has_out"] = out_scale.has_value();
        variable_list saved = {twiddle};
        if (in_scale.has_value()) saved.push_back(in_scale.value());
        if (out_scale.has_value()) saved.push_back(out_scale.value());
        ctx->save_for_backward(saved);
        return butterfly_scale_twiddle_fw(twiddle, in_scale, out_scale, increasing_stride);
    }

    static variable_list backward(AutogradContext *ctx, variable_list grad_output)
    {
        const auto saved = ctx->get_saved_variables();
        const bool has_in = ctx->saved_data["has_in"].toBool(), has_out = ctx->saved_data["has_out"].toBool();
        c10::optional<Tensor> in_scale, out_scale;
        size_t next = 1;
        if (has_in) in_scale = saved[next++];
        if (has_out) out_scale = saved[next++];
        auto r = butterfly_scale_twiddle_bw(saved[0], in_scale, out_scale, grad_output[0],
                                            ctx->saved_data["increasing_stride"].toBool());
        return {std::get<0>(r), has_in ? std::get<1>(r) : Tensor(), has_out ? std::get<2>(r) : Tensor(), Tensor()};
    }
};

Tensor butterfly_scale_twiddle(Tensor twiddle, c10::optional<Tensor> in_scale, c10::optional<Tensor> out_scale,
                               bool increasing_stride)
{
    return ButterflyScaleTwiddle::apply(twiddle, in_scale, out_scale, increasing_stride);
}

// ---- base-4 -----------------------------------------------------------------------------

Shapes base4_shapes(const Tensor &twiddle4, const Tensor &twiddle2, const Tensor &input, const char *who)
{
    CHECK_DEVICE(twiddle4); CHECK_DEVICE(twiddle2); CHECK_DEVICE(input);
    CHECK_SAME_DEVICE(twiddle4, input); CHECK_SAME_DEVICE(twiddle2, input);
    CHECK_DIM(twiddle4, 6); CHECK_DIM(twiddle2, 6); CHECK_DIM(input, 3);
    Shapes s;
    s.batch = input.size(0);
    s.nstacks = input.size(1);
    s.input_size = input.size(2);
    s.nblocks = twiddle4.size(1);
    s.log_n = twiddle4.size(2) * 2 + twiddle2.size(2);
    TORCH_CHECK(s.log_n <= 30, who, ": n must be a power of 2");
    s.n = (int64_t)1 << s.log_n;
    TORCH_CHECK(twiddle2.size(2) <= 1, "twiddle2 must have shape (nstacks, nblocks, log_n % 2, n / 2, 2, 2)");
    if (s.log_n / 2 > 0) CHECK_SHAPE(twiddle4, s.nstacks, s.nblocks, s.log_n / 2, s.n / 4, 4, 4);
    if (s.log_n % 2 == 1) CHECK_SHAPE(twiddle2, s.nstacks, s.nblocks, 1, s.n / 2, 2, 2);
    require_device(input, who);
    TORCH_CHECK(twiddle4.scalar_type() == input.scalar_type() && twiddle2.scalar_type() == input.scalar_type(),
                who, ": twiddle4, twiddle2 and input must have the same dtype");
    return s;
}

// keep: when given and the backward of this problem runs in several passes, the forward runs
// along the backward's plan and leaves the activations between its passes there
Tensor base4_fw_impl(const Tensor &twiddle4, const Tensor &twiddle2, const Tensor &input, bool increasing_stride,
                     c10::optional<int64_t> output_size, Tensor *keep)
{
    const Shapes s = base4_shapes(twiddle4, twiddle2, input, "butterfly_multiply_base4_fw");
    const int64_t output_size_val = output_size.has_value() ? output_size.value() : s.n;
    TORCH_CHECK(output_size_val <= s.n, "butterfly_multiply_base4_fw: output_size must be <= n");
    TORCH_CHECK(output_size_val >= 0, "butterfly_multiply_base4_fw: output_size must be >= 0");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    const Tensor tw4 = dense(twiddle4), tw2 = dense(twiddle2);
    const Tensor x = input.resolve_conj();
    Tensor output = at::empty({s.batch, s.nstacks, s.n}, x.options());
    if (output_size_val < s.n) output = output.slice(2, 0, output_size_val);
    bf_problem p = make_problem(s, x, increasing_stride, output_size_val, "butterfly_multiply_base4_fw");
    set_strides(p.output_stride, output);
    if (keep) {
        // (the backward will make d_input dense over max(input_size, n) columns: same plan)
        const int64_t dw = std::max(s.input_size, s.n);
        p.d_input_stride[0] = s.batch > 1 ? s.nstacks * dw : 0;
        p.d_input_stride[1] = s.nstacks > 1 ? dw : 0;
        p.d_input_stride[2] = s.input_size > 1 ? 1 : 0;
        const size_t nsaved = valid_size(bf_butterfly_multiply_base4_saved_bytes(&p));
        if (nsaved > 0) {
            *keep = at::empty({(int64_t)nsaved}, x.options().dtype(at::kByte));
            check_rc(bf_butterfly_multiply_base4_fw_saving(&p, tw4.data_ptr(), tw2.data_ptr(), x.data_ptr(),
                                                           output.data_ptr(), keep->data_ptr(), nsaved,
                                                           current_stream()),
                     "butterfly_multiply_base4");
            return output;
        }
    }
    const size_t ws_bytes = valid_size(bf_butterfly_multiply_base4_fw_workspace_bytes(&p));
    Tensor ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
    check_rc(bf_butterfly_multiply_base4_fw(&p, tw4.data_ptr(), tw2.data_ptr(), x.data_ptr(), output.data_ptr(),
                                            ws.data_ptr(), ws_bytes, current_stream()),
             "butterfly_multiply_base4_fw");
    return output;
}

Tensor butterfly_multiply_base4_fw(const Tensor twiddle4, const Tensor twiddle2, const Tensor input,
                                   bool increasing_stride, c10::optional<int64_t> output_size)
{
    return base4_fw_impl(twiddle4, twiddle2, input, increasing_stride, output_size, nullptr);
}

// kept: the activations a forward with `keep` left behind (undefined: recompute them)
std::tuple<Tensor, Tensor, Tensor> base4_bw_impl(const Tensor &twiddle4, const Tensor &twiddle2, const Tensor &input,
                                                 const Tensor &grad, bool increasing_stride, const Tensor &kept)
{
    const Shapes s = base4_shapes(twiddle4, twiddle2, input, "butterfly_multiply_base4_bw");
    CHECK_DEVICE(grad); CHECK_SAME_DEVICE(input, grad); CHECK_DIM(grad, 3);
    const int64_t output_size = grad.size(2);
    CHECK_SHAPE(grad, s.batch, s.nstacks, output_size);
    TORCH_CHECK(output_size <= s.n, "butterfly_multiply_base4_bw: grad must have at most n columns");
    TORCH_CHECK(grad.scalar_type() == input.scalar_type(),
                "butterfly_multiply_base4_bw: grad and input must have the same dtype");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    const Tensor tw4 = dense(twiddle4), tw2 = dense(twiddle2);
    const Tensor x = input.resolve_conj();
    const Tensor g = grad.resolve_conj();
    Tensor d4 = at::empty(tw4.sizes(), tw4.options());
    Tensor d2 = at::empty(tw2.sizes(), tw2.options());
    Tensor d_input = at::empty({s.batch, s.nstacks, std::max(s.input_size, s.n)}, x.options());
    if (s.input_size < s.n) d_input = d_input.slice(2, 0, s.input_size);
    bf_problem p = make_problem(s, x, increasing_stride, output_size, "butterfly_multiply_base4_bw");
    set_strides(p.output_stride, g);
    set_strides(p.d_input_stride, d_input);
    // (as in the base-2 backward: the plan of this call decides whether the kept planes serve it)
    bool use_kept = kept.defined();
    if (use_kept) {
        const size_t reads = valid_size(bf_butterfly_multiply_base4_saved_bytes(&p));
        if (reads == 0 || reads > (size_t)kept.numel()) use_kept = false;
    }
    if (use_kept) {
        const size_t ws_bytes = valid_size(bf_butterfly_multiply_base4_bw_saved_workspace_bytes(&p));
        Tensor ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
        check_rc(bf_butterfly_multiply_base4_bw_saved(&p, tw4.data_ptr(), tw2.data_ptr(), x.data_ptr(), g.data_ptr(),
                                                      kept.data_ptr(), (size_t)kept.numel(), d4.data_ptr(), d2.data_ptr(),
                                                      d_input.data_ptr(),
                                                      ws.data_ptr(), ws_bytes, current_stream()),
                 "butterfly_multiply_base4_bw");
        return std::make_tuple(d4, d2, d_input);
    }
    const size_t ws_bytes = valid_size(bf_butterfly_multiply_base4_bw_workspace_bytes(&p));
    Tensor ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
    check_rc(bf_butterfly_multiply_base4_bw(&p, tw4.data_ptr(), tw2.data_ptr(), x.data_ptr(), g.data_ptr(),
                                            d4.data_ptr(), d2.data_ptr(), d_input.data_ptr(), ws.data_ptr(),
                                            ws_bytes, current_stream()),
             "butterfly_multiply_base4_bw");
    return std::make_tuple(d4, d2, d_input);
}

std::tuple<Tensor, Tensor, Tensor> butterfly_multiply_base4_bw(const Tensor twiddle4, const Tensor twiddle2,
                                                               const Tensor input, const Tensor grad,
                                                               bool increasing_stride)
{
    return base4_bw_impl(twiddle4, twiddle2, input, grad, increasing_stride, Tensor());
}

class ButterflyMultiplyBase4 : public torch::autograd::Function<ButterflyMultiplyBase4> {
public:
    // wants_grad: as in ButterflyMultiply, the forward keeps the activations between the passes of
    // a backward that runs in several (more than one block, or rows beyond one workgroup's reach)
    static Tensor forward(AutogradContext *ctx, Tensor twiddle4, Tensor twiddle2, Tensor input,
                          bool increasing_stride, c10::optional<int64_t> output_size, bool wants_grad)
    {
        ctx->saved_data["increasing_stride"] = increasing_stride;
        Tensor kept;
        Tensor out = base4_fw_impl(twiddle4, twiddle2, input, increasing_stride, output_size,
                                   wants_grad ? &kept : nullptr);
        ctx->saved_data["kept"] = kept.defined();
        if (kept.defined()) ctx->save_for_backward({twiddle4, twiddle2, input, kept});
        else ctx->save_for_backward({twiddle4, twiddle2, input});
        return out;
    }

    static variable_list backward(AutogradContext *ctx, variable_list grad_output)
    {
        const auto saved = ctx->get_saved_variables();
        const bool increasing_stride = ctx->saved_data["increasing_stride"].toBool();
        const Tensor kept = ctx->saved_data["kept"].toBool() ? saved[3] : Tensor();
        auto r = base4_bw_impl(saved[0], saved[1], saved[2], grad_output[0], increasing_stride, kept);
        return {std::get<0>(r), std::get<1>(r), std::get<2>(r), Tensor(), Tensor(), Tensor()};
    }
};

Tensor butterfly_multiply_base4(Tensor twiddle4, Tensor twiddle2, Tensor input, bool increasing_stride,
                                c10::optional<int64_t> output_size)
{
    return ButterflyMultiplyBase4::apply(twiddle4, twiddle2, input, increasing_stride, output_size,
                                         grad_wanted({twiddle4, twiddle2, input}));
}

int64_t hip_version() { return bf_hip_version(); }

}  // namespace

TORCH_LIBRARY(torch_butterfly, m)
{
    m.def("butterfly_multiply_fw", butterfly_multiply_fw);
    m.def("butterfly_multiply_bw", butterfly_multiply_bw);
    m.def("butterfly_multiply", butterfly_multiply);
    m.def("butterfly_multiply_bias_fw", butterfly_multiply_bias_fw);
    m.def("butterfly_bias_grad", butterfly_bias_grad);
    m.def("butterfly_multiply_bias_bw", butterfly_multiply_bias_bw);
    m.def("butterfly_multiply_bias", butterfly_multiply_bias);
    m.def("butterfly_multiply_perm_fw", butterfly_multiply_perm_fw);
    m.def("butterfly_multiply_perm_bw", butterfly_multiply_perm_bw);
    m.def("butterfly_multiply_perm", butterfly_multiply_perm);
    m.def("butterfly_scale_twiddle_fw", butterfly_scale_twiddle_fw);
    m.def("butterfly_scale_twiddle_bw", butterfly_scale_twiddle_bw);
    m.def("butterfly_scale_twiddle", butterfly_scale_twiddle);
    m.def("butterfly_multiply_base4_fw", butterfly_multiply_base4_fw);
    m.def("butterfly_multiply_base4_bw", butterfly_multiply_base4_bw);
    m.def("butterfly_multiply_base4", butterfly_multiply_base4);
    m.def("hip_version", hip_version);
}
