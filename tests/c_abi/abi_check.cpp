// The C ABI of libbutterfly_hip.so driven from plain C++, with no PyTorch in the process:
// device memory from hipMalloc, the null stream, workspace sizes from the library's queries.
// Every result is compared with the CPU restatement in oracle/liboracle.so (test infrastructure)
// to the tolerances the parity tests use: max|err| / max|ref| <= 1e-5 forward, 1e-4 gradients.
// Exit status 0 when every case passes; one line per case on stdout.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "butterfly_hip.h"

extern "C" {
int oracle_butterfly_fw_f32(const float *, const float *, float *, int64_t, int64_t, int64_t, int64_t, int64_t, int);
int oracle_butterfly_bw_f32(const float *, const float *, const float *, float *, float *, float *, int64_t, int64_t,
                            int64_t, int64_t, int64_t, int64_t, int);
int oracle_butterfly_fw_c64(const float *, const float *, float *, int64_t, int64_t, int64_t, int64_t, int64_t, int);
int oracle_butterfly_bw_c64(const float *, const float *, const float *, float *, float *, float *, int64_t, int64_t,
                            int64_t, int64_t, int64_t, int64_t, int);
int oracle_butterfly_base4_fw_f32(const float *, const float *, const float *, float *, int64_t, int64_t, int64_t,
                                  int64_t, int64_t, int);
int oracle_butterfly_base4_bw_f32(const float *, const float *, const float *, const float *, float *, float *, float *,
                                  float *, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int);
}

#define HIP_OK(expr)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (expr);                                                               \
        if (e_ != hipSuccess) {                                                               \
            std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            std::exit(2);                                                                     \
        }                                                                                     \
    } while (0)

namespace {

// splitmix64 -> roughly normal floats (sum of four uniforms), reproducible everywhere
struct Rng {
    uint64_t s;
    uint64_t next()
    {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    float normal()
    {
        double u = 0;
        for (int i = 0; i < 4; ++i) u += (double)(next() >> 11) * (1.0 / 9007199254740992.0);
        return (float)((u - 2.0) * 1.7320508);
    }
};

std::vector<float> randn(Rng &rng, size_t count, float scale)
{
    std::vector<float> v(count);
    for (auto &x : v) x = rng.normal() * scale;
    return v;
}

struct DeviceBuffer {
    void *p = nullptr;
    explicit DeviceBuffer(size_t bytes) { HIP_OK(hipMalloc(&p, bytes ? bytes : 16)); }
    ~DeviceBuffer() { (void)hipFree(p); }
    DeviceBuffer(const DeviceBuffer &) = delete;
    void upload(const std::vector<float> &h) { HIP_OK(hipMemcpy(p, h.data(), h.size() * sizeof(float), hipMemcpyHostToDevice)); }
    std::vector<float> download(size_t count)
    {
        std::vector<float> h(count);
        HIP_OK(hipMemcpy(h.data(), p, count * sizeof(float), hipMemcpyDeviceToHost));
        return h;
    }
};

double rel_err(const std::vector<float> &got, const std::vector<float> &want)
{
    double scale = 0, err = 0;
    for (size_t i = 0; i < want.size(); ++i) {
        scale = std::fmax(scale, std::fabs((double)want[i]));
        err = std::fmax(err, std::fabs((double)got[i] - (double)want[i]));
    }
    return err / (scale > 0 ? scale : 1.0);
}

int failures = 0;

void report(const char *what, int64_t B, int64_t S, int64_t L, int64_t nb, double fw, double dx, double dtw)
{
    const bool ok = fw <= 1e-5 && dx <= 1e-4 && dtw <= 1e-4;
    if (!ok) ++failures;
    std::printf("%s B=%lld S=%lld log_n=%lld nblocks=%lld: forward %.2e d_input %.2e d_twiddle %.2e %s\n", what,
                (long long)B, (long long)S, (long long)L, (long long)nb, fw, dx, dtw, ok ? "ok" : "FAILED");
    std::fflush(stdout);
}

bf_problem problem(int dtype, int inc, int64_t B, int64_t S, int64_t L, int64_t nb, int64_t I, int64_t O)
{
    const int64_t n = (int64_t)1 << L;
    bf_problem p = {};
    p.dtype = dtype;
    p.increasing_stride = inc;
    p.batch = B;
    p.nstacks = S;
    p.log_n = L;
    p.nblocks = nb;
    p.input_size = I;
    p.output_size = O;
    const int64_t W = I > n ? I : n;
    const int64_t in[3] = {S * I, I, 1}, out[3] = {S * O, O, 1}, din[3] = {S * W, W, 1};
    for (int k = 0; k < 3; ++k) {
        p.input_stride[k] = in[k];
        p.output_stride[k] = out[k];
        p.d_input_stride[k] = din[k];
    }
    return p;
}

void check(int rc, const char *call)
{
    if (rc != BF_OK) {
        std::printf("%s failed (%d): %s\n", call, rc, bf_last_error());
        std::exit(3);
    }
}

// base-2, float (e = 1) or complex64 (e = 2 floats per element)
void base2_case(int dtype, int inc, int64_t B, int64_t S, int64_t L, int64_t nb, int64_t I, int64_t O, uint64_t seed)
{
    const int e = dtype == BF_C64 ? 2 : 1;
    const int64_t n = (int64_t)1 << L, W = I > n ? I : n;
    Rng rng{seed};
    const auto tw = randn(rng, (size_t)(S * nb * L * (n / 2) * 4 * e), 0.70710678f);
    const auto x = randn(rng, (size_t)(B * S * I * e), 1.0f);
    const auto g = randn(rng, (size_t)(B * S * O * e), 1.0f);
    const bf_problem p = problem(dtype, inc, B, S, L, nb, I, O);

    DeviceBuffer d_tw(tw.size() * 4), d_x(x.size() * 4), d_g(g.size() * 4), d_y((size_t)(B * S * O * e) * 4),
        d_dtw(tw.size() * 4), d_dx((size_t)(B * S * W * e) * 4);
    d_tw.upload(tw);
    d_x.upload(x);
    d_g.upload(g);
    const size_t fw_ws = bf_butterfly_multiply_fw_workspace_bytes(&p), bw_ws = bf_butterfly_multiply_bw_workspace_bytes(&p);
    DeviceBuffer ws(fw_ws > bw_ws ? fw_ws : bw_ws);
    check(bf_butterfly_multiply_fw(&p, d_tw.p, d_x.p, d_y.p, ws.p, fw_ws, nullptr), "bf_butterfly_multiply_fw");
    check(bf_butterfly_multiply_bw(&p, d_tw.p, d_x.p, d_g.p, d_dtw.p, d_dx.p, ws.p, bw_ws, nullptr), "bf_butterfly_multiply_bw");
    HIP_OK(hipDeviceSynchronize());
    const auto y = d_y.download((size_t)(B * S * O * e)), dtw = d_dtw.download(tw.size()),
               dx = d_dx.download((size_t)(B * S * W * e));

    std::vector<float> y_full((size_t)(B * S * n * e)), y_ref((size_t)(B * S * O * e)), dtw_ref(tw.size()),
        dx_ref((size_t)(B * S * W * e)), scratch((size_t)((nb * L > 0 ? nb * L : 1) * B * S * n * e));
    if (dtype == BF_F32) {
        oracle_butterfly_fw_f32(tw.data(), x.data(), y_full.data(), B, S, nb, L, I, inc);
        oracle_butterfly_bw_f32(tw.data(), x.data(), g.data(), dtw_ref.data(), dx_ref.data(), scratch.data(), B, S, nb, L, I, O, inc);
    } else {
        oracle_butterfly_fw_c64(tw.data(), x.data(), y_full.data(), B, S, nb, L, I, inc);
        oracle_butterfly_bw_c64(tw.data(), x.data(), g.data(), dtw_ref.data(), dx_ref.data(), scratch.data(), B, S, nb, L, I, O, inc);
    }
    for (int64_t r = 0; r < B * S; ++r)
        for (int64_t j = 0; j < O * e; ++j) y_ref[(size_t)(r * O * e + j)] = y_full[(size_t)(r * n * e + j)];
    // d_input: the I columns of every row that the call owns (rows are W apart on both sides;
    // the restatement also fills the padding columns up to n, which the library leaves alone)
    std::vector<float> dx_got((size_t)(B * S * I * e)), dx_want(dx_got.size());
    for (int64_t r = 0; r < B * S; ++r)
        for (int64_t j = 0; j < I * e; ++j) {
            dx_got[(size_t)(r * I * e + j)] = dx[(size_t)(r * W * e + j)];
            dx_want[(size_t)(r * I * e + j)] = dx_ref[(size_t)(r * W * e + j)];
        }
    report(dtype == BF_F32 ? "base-2 float    " : "base-2 complex64", B, S, L, nb, rel_err(y, y_ref), rel_err(dx_got, dx_want),
           rel_err(dtw, dtw_ref));
}

void base4_case(int inc, int64_t B, int64_t S, int64_t L, int64_t nb, uint64_t seed)
{
    const int64_t n = (int64_t)1 << L, L4 = L / 2, odd = L % 2;
    Rng rng{seed};
    const auto tw4 = randn(rng, (size_t)(S * nb * L4 * (n / 4) * 16), 0.5f);
    const auto tw2 = randn(rng, (size_t)(S * nb * odd * (n / 2) * 4), 0.70710678f);
    const auto x = randn(rng, (size_t)(B * S * n), 1.0f);
    const auto g = randn(rng, (size_t)(B * S * n), 1.0f);
    const bf_problem p = problem(BF_F32, inc, B, S, L, nb, n, n);
    DeviceBuffer d_t4(tw4.size() * 4), d_t2(tw2.size() * 4), d_x(x.size() * 4), d_g(g.size() * 4), d_y(x.size() * 4),
        d_d4(tw4.size() * 4), d_d2(tw2.size() * 4), d_dx(x.size() * 4);
    d_t4.upload(tw4);
    d_t2.upload(tw2);
    d_x.upload(x);
    d_g.upload(g);
    const size_t fw_ws = bf_butterfly_multiply_base4_fw_workspace_bytes(&p),
                 bw_ws = bf_butterfly_multiply_base4_bw_workspace_bytes(&p);
    DeviceBuffer ws(fw_ws > bw_ws ? fw_ws : bw_ws);
    check(bf_butterfly_multiply_base4_fw(&p, d_t4.p, d_t2.p, d_x.p, d_y.p, ws.p, fw_ws, nullptr), "bf_butterfly_multiply_base4_fw");
    check(bf_butterfly_multiply_base4_bw(&p, d_t4.p, d_t2.p, d_x.p, d_g.p, d_d4.p, d_d2.p, d_dx.p, ws.p, bw_ws, nullptr),
          "bf_butterfly_multiply_base4_bw");
    HIP_OK(hipDeviceSynchronize());
    const auto y = d_y.download(x.size()), d4 = d_d4.download(tw4.size()), dx = d_dx.download(x.size());
    std::vector<float> y_ref(x.size()), d4_ref(tw4.size()), d2_ref(tw2.size() + 1), dx_ref(x.size()),
        scratch((size_t)(nb * (L4 + odd) * B * S * n));
    oracle_butterfly_base4_fw_f32(tw4.data(), tw2.data(), x.data(), y_ref.data(), B, S, nb, L, n, inc);
    oracle_butterfly_base4_bw_f32(tw4.data(), tw2.data(), x.data(), g.data(), d4_ref.data(), d2_ref.data(), dx_ref.data(),
                                  scratch.data(), B, S, nb, L, n, n, inc);
    double dtw = rel_err(d4, d4_ref);
    if (odd) {
        d2_ref.resize(tw2.size());
        dtw = std::fmax(dtw, rel_err(d_d2.download(tw2.size()), d2_ref));
    }
    report("base-4 float    ", B, S, L, nb, rel_err(y, y_ref), rel_err(dx, dx_ref), dtw);
}

}  // namespace

int main()
{
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count < 1) {
        std::printf("no HIP device\n");
        return 2;
    }
    std::printf("libbutterfly_hip %d, HIP %d\n", bf_version(), bf_hip_version());
    base2_case(BF_F32, 0, 1500, 1, 10, 2, 1024, 1024, 1);   // the headline kernels, ragged row groups
    base2_case(BF_F32, 1, 300, 2, 10, 2, 1000, 900, 2);     // padded input, trimmed output
    base2_case(BF_F32, 0, 40, 1, 12, 2, 4096, 4096, 3);     // rows of 4096: three passes and a workspace
    base2_case(BF_F32, 1, 1000, 3, 5, 3, 32, 32, 4);        // short rows, three blocks
    base2_case(BF_C64, 1, 200, 2, 8, 1, 256, 200, 5);
    base2_case(BF_C64, 0, 30, 1, 12, 1, 4096, 4096, 6);
    base4_case(1, 2000, 4, 8, 1, 7);
    base4_case(0, 300, 1, 9, 2, 8);
    // an invalid problem is refused with a message, not run
    bf_problem bad = problem(BF_F32, 1, 4, 1, 3, 1, 8, 9);
    const int rc = bf_butterfly_multiply_fw(&bad, nullptr, nullptr, nullptr, nullptr, 0, nullptr);
    std::printf("output_size > n: rc %d (%s)\n", rc, bf_last_error());
    if (rc != BF_ERR_INVALID) ++failures;
    // ... and its size queries say "invalid", which is not the same as "no workspace needed"
    const size_t bad_ws = bf_butterfly_multiply_bw_workspace_bytes(&bad);
    const bf_problem small = problem(BF_F32, 1, 4, 1, 3, 1, 8, 8);
    const size_t small_ws = bf_butterfly_multiply_fw_workspace_bytes(&small);
    std::printf("size queries: invalid problem %s, single-launch forward %zu bytes\n",
                bad_ws == BF_SIZE_INVALID ? "BF_SIZE_INVALID" : "a size", small_ws);
    if (bad_ws != BF_SIZE_INVALID || small_ws != 0) ++failures;
    // the activation-keeping pair: the backward checks the size of the area it is handed
    {
        const bf_problem q = problem(BF_F32, 1, 8, 1, 12, 2, 4096, 4096);
        const size_t keep = bf_butterfly_multiply_saved_bytes(&q);
        const size_t ws_bytes = bf_butterfly_multiply_bw_saved_workspace_bytes(&q, 0);
        DeviceBuffer area(keep), ws(ws_bytes), t((size_t)2 * 12 * 2048 * 4 * 4), v((size_t)8 * 4096 * 4);
        const int short_rc = bf_butterfly_multiply_bw_saved(&q, t.p, v.p, v.p, area.p, keep / 2, nullptr, nullptr, t.p, v.p,
                                                            nullptr, ws.p, ws_bytes, nullptr);
        std::printf("saved area too small: rc %d (%s)\n", short_rc, bf_last_error());
        if (keep == 0 || keep == BF_SIZE_INVALID || short_rc != BF_ERR_WORKSPACE) ++failures;
    }
    std::printf(failures ? "%d case(s) FAILED\n" : "all cases ok\n", failures);
    return failures ? 1 : 0;
}
