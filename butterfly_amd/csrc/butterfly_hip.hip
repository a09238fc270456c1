// C ABI of libbutterfly_hip.so: argument checks, launch planning and kernel launches.
// See include/butterfly_hip.h for the contract of every entry point.

#include "../../include/butterfly_hip.h"

#include <hip/hip_runtime.h>
#include <hip/hip_version.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <utility>

#include "common.hpp"
#include "generic.hpp"
#include "scale.hpp"
#include "fast.hpp"
#include "wide.hpp"
#include "fast4.hpp"
#include "fast4g.hpp"
#include "stage.hpp"
#include "bias.hpp"

namespace {

using namespace bf;

thread_local std::string g_last_error;

int fail(int code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

#define BF_HIP_CHECK(expr)                                                              \
    do {                                                                                \
        hipError_t e_ = (expr);                                                         \
        if (e_ != hipSuccess)                                                           \
            return fail(BF_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_));     \
    } while (0)

// (gfx950 has 160 KiB of LDS per compute unit)
constexpr size_t kGenericFwLds = 128 * 1024;    // most a generic forward workgroup stages
constexpr size_t kGenericBwLds = 144 * 1024;    // most a generic backward workgroup stages
constexpr int kMaxGrid = 1 << 30;

size_t elem_bytes(int dtype) { return dtype == BF_C64 ? 8 : 4; }

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// ---- validation -----------------------------------------------------------------------

int check_problem(const bf_problem *p, bool backward)
{
    if (!p) return fail(BF_ERR_INVALID, "problem descriptor is NULL");
    if (p->dtype != BF_F32 && p->dtype != BF_C64)
        return fail(BF_ERR_INVALID, "dtype must be BF_F32 or BF_C64 (device kernels cover float and complex64)");
    if (p->batch < 0 || p->nstacks < 0 || p->nblocks < 0 || p->input_size < 0 || p->output_size < 0)
        return fail(BF_ERR_INVALID, "sizes must be non-negative");
    if (p->log_n < 0 || p->log_n > 30) return fail(BF_ERR_INVALID, "log_n must be in [0, 30]");
    const int64_t n = (int64_t)1 << p->log_n;
    if (p->output_size > n) return fail(BF_ERR_INVALID, "output_size must be <= n");
    for (int i = 0; i < 3; ++i) {
        if (p->input_stride[i] < 0 || p->output_stride[i] < 0 || (backward && p->d_input_stride[i] < 0))
            return fail(BF_ERR_INVALID, "strides must be non-negative");
    }
    if (p->nstacks > 65535) return fail(BF_ERR_UNSUPPORTED, "nstacks above 65535 is not supported");
    if (p->batch > ((int64_t)1 << 40)) return fail(BF_ERR_UNSUPPORTED, "batch too large");
    return BF_OK;
}

Schedule make_schedule(const bf_problem *p, bool base4)
{
    Schedule sc;
    sc.log_n = (int)p->log_n;
    sc.nblocks = (int)p->nblocks;
    sc.increasing_stride = p->increasing_stride != 0;
    sc.base4 = base4;
    const int64_t n = (int64_t)1 << p->log_n;
    if (base4) {
        sc.per = (int)(p->log_n / 2 + p->log_n % 2);
        sc.tw4_stack_stride = p->nblocks * (p->log_n / 2) * (n / 4) * 16;
        sc.tw2_stack_stride = p->nblocks * (p->log_n % 2) * (n / 2) * 4;
    } else {
        sc.per = (int)p->log_n;
        sc.tw4_stack_stride = 0;
        sc.tw2_stack_stride = p->nblocks * p->log_n * (n / 2) * 4;
    }
    return sc;
}

View make_view(const int64_t stride[3], int64_t width, const int *perm = nullptr)
{
    View v;
    v.sb = stride[0];
    v.ss = stride[1];
    v.se = stride[2];
    v.width = width;
    v.perm = perm;
    return v;
}

View dense_view(int64_t nstacks, int64_t n)
{
    View v;
    v.sb = nstacks * n;
    v.ss = n;
    v.se = 1;
    v.width = n;
    v.perm = nullptr;
    return v;
}

// ---- kernel attributes, once per device ---------------------------------------------------
//
// The LDS fallback kernels ask for more dynamic LDS than the default limit; that permission is a
// property of the function on one device, so it is set the first time a call runs on a device.

constexpr int kMaxDevices = 64;
std::mutex g_device_mutex;
bool g_attr_done[kMaxDevices];

int ensure_attributes()
{
    int device = -1;
    BF_HIP_CHECK(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices)
        return fail(BF_ERR_UNSUPPORTED, "device ordinal %d is outside the %d the library keeps state for", device,
                    kMaxDevices);
    std::lock_guard<std::mutex> lock(g_device_mutex);
    if (g_attr_done[device]) return BF_OK;
    const std::pair<const void *, size_t> wanted[] = {
        {reinterpret_cast<const void *>(&generic_fw_kernel<float>), kGenericFwLds},
        {reinterpret_cast<const void *>(&generic_fw_kernel<float2>), kGenericFwLds},
        {reinterpret_cast<const void *>(&generic_bw_kernel<float>), kGenericBwLds},
        {reinterpret_cast<const void *>(&generic_bw_kernel<float2>), kGenericBwLds},
    };
    for (const auto &w : wanted) {
        const hipError_t e = hipFuncSetAttribute(w.first, hipFuncAttributeMaxDynamicSharedMemorySize, (int)w.second);
        if (e != hipSuccess) return fail(BF_ERR_HIP, "hipFuncSetAttribute failed: %s", hipGetErrorString(e));
    }
    g_attr_done[device] = true;
    return BF_OK;
}

// Compute units of the device that is current, asked once per device.  Grids of the persistent
// kernels (one workgroup per compute unit), the partial areas and the measured crossovers are
// sized from it.  Host-only queries on a machine without a device plan for an MI355X (256).
constexpr int kDefaultNumCU = 256;
int g_num_cu[kMaxDevices];

int num_cu()
{
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
        (void)hipGetLastError();
        return kDefaultNumCU;
    }
    std::lock_guard<std::mutex> lock(g_device_mutex);
    if (g_num_cu[device] == 0) {
        int count = 0;
        if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0) {
            (void)hipGetLastError();
            count = kDefaultNumCU;
        }
        g_num_cu[device] = count;
    }
    return g_num_cu[device];
}
#ifndef BF_FAST_FW_ROWS
#define BF_FAST_FW_ROWS 4
#endif
constexpr int kFastFwRows = BF_FAST_FW_ROWS;  // row groups in flight per forward workgroup
// Iterations (of kFastFwRows row groups) a forward workgroup must have left before a float pass
// over two blocks is spread over two workgroups per compute unit (see fw_wg_per_cu).
#ifndef BF_FAST_FW_PAIR_MIN_ITERS
#define BF_FAST_FW_PAIR_MIN_ITERS 6
#endif
constexpr int kFastFwRowsComplex = 2;       // complex64: half as many (LDS and registers double)

// ---- register-resident multi-pass path (float and complex64, base-2, n <= 2^24) -------------------------
//
// The flat stage list is cut into passes, one kernel launch each, all with the
// twiddle-stationary kernels of fast.hpp:
//   * a LOW pass runs up to 20 consecutive stages that pair element bits below 10 (rows longer
//     than 1024 are treated as independent 1024-element chunks);
//   * a SPAN pass runs the stages on up to five adjacent bits from bit 10 up, on tiles of 1024
//     elements that take all settings of those bits (SpanPlan);
//   * the forward call alone replaces the LOW / SPAN passes of one block by a single WIDE pass
//     (wide.hpp) where the factors of a whole block fit the registers and enough rows share
//     them: float at n = 2048 and 4096, complex64 at n = 2048.
// n <= 1024 with one or two blocks is a single LOW pass: each row is read once and written
// once.  Longer schedules pass the activation through the workspace between launches.

// Largest byte offset one workgroup forms into an operand with these strides; the fast
// kernels address through 32-bit offsets and need it below 2 GiB.
bool span_ok(const int64_t stride[3], int64_t rows, int64_t width, size_t elem)
{
    const double bytes = (double)elem * ((double)rows * (double)stride[0] + (double)width * (double)stride[2]);
    return bytes < 2147483000.0;
}

constexpr int kMaxPasses = 96;
// widest span: tiles of 32 consecutive floats (16 consecutive complex64: the same 128 bytes) per
// setting of the span's bits
constexpr int kSpanMaxBits = 5;
constexpr int kSpanMaxBitsComplex = 6;
constexpr int kSpanMaxStagesComplex = 10;  // stages one complex64 span pass can hold (registers + parked factors)
constexpr int kMaxLogN = 24;  // the chunk index of the register-resident kernels travels in blockIdx.z

struct Pass {
    int t0, t1;     // stage range [t0, t1)
    bool wide;      // forward only: one whole block of a 2048- or 4096-element row (wide.hpp)
    int L, NB;      // LOW: FastPlan<L, NB, inc> on chunks of 2^L elements
    bool inc;
    bool span;      // SPAN: SpanPlan<H, mode> on tiles, H adjacent bits from `lb` up (L = 10, NB = 1)
    int H, lb;
    int mode;       // 0: one sweep up, 1: one sweep down, 2: up then down
};

struct PassPlan {
    bool ok = false;
    int npass = 0;
    Pass pass[kMaxPasses];
    int low = 10;        // bits below the spans: LOW passes run on chunks of 2^low elements
};

// independent columns of work per row and stack of a pass: chunks of a LOW pass, tiles of a span
int64_t pass_lanes(const bf_problem *p, const Pass &q)
{
    if (q.wide) return 1;
    const int reach = q.span ? 10 : q.L;
    return (int64_t)1 << (p->log_n > reach ? p->log_n - reach : 0);
}

// Forward workgroups per compute unit.  The kernel fits a CU twice (64 registers, 64 KiB of LDS).
// A float pass over two blocks is bound by its own chain of arithmetic and LDS transpositions,
// not by memory, and two resident workgroups fill each other's gaps (33.3 against 36.2 us at
// 16384 rows of 1024); each of them loads the whole factor set, so it takes rows to pay off
// (2048 rows: 10.0 against 8.6 us for one block).  One-block passes run at the memory rate either way.
// (The 64-register variant of the two-block forward kernel for 512-element rows, decreasing
// stride first, does not fit its registers -- the build refuses kernels that spill -- so that
// plan always runs one workgroup per CU.)
constexpr bool fw_pairable(int L, bool inc) { return !(L == 9 && !inc); }

int fw_wg_per_cu(const bf_problem *p, const Pass &q)
{
    if (q.wide || q.span || q.NB != 2 || p->dtype != BF_F32 || !fw_pairable(q.L, q.inc)) return 1;
    const int64_t slots = 1024 >> q.L;
    const int64_t iters = ((p->batch + slots - 1) / slots + kFastFwRows - 1) / kFastFwRows;
    const int64_t pairs = std::max<int64_t>(1, 2 * (int64_t)num_cu() / (p->nstacks * pass_lanes(p, q)));
    return iters >= pairs * BF_FAST_FW_PAIR_MIN_ITERS ? 2 : 1;
}

int stage_bit(const bf_problem *p, int t)
{
    const int L = (int)p->log_n;
    const int block = t / L, idx = t % L;
    const bool inc = (p->increasing_stride != 0) != ((block & 1) != 0);
    return inc ? idx : L - 1 - idx;
}

// Rows (over all stacks) from which the whole-block forward kernel of wide.hpp beats the
// chunked + span passes: each of its workgroups first loads the factors of a whole block
// (up to 96 registers per thread), which only pays off over enough rows.  Measured crossovers.
int64_t wide_min_rows(const bf_problem *p)
{
    if (p->log_n == 12) return p->nblocks == 1 ? 2048 : 8192;
    if (p->dtype == BF_C64) return p->nblocks == 1 ? 0 : 2048;
    return p->nblocks == 1 ? 0 : 4096;
}

// permuted: the call reads or writes its rows through column tables (see the low width below)
PassPlan build_passes(const bf_problem *p, bool base4, bool forward_only = false, bool permuted = false)
{
    PassPlan pl;
    const int L = (int)p->log_n;
    if (base4 || L < 1 || L > kMaxLogN || p->nblocks < 1 || p->batch <= 0 || p->nstacks <= 0 ||
        p->input_size <= 0 || p->output_size <= 0)
        return pl;
    const int NS = L * (int)p->nblocks;
    // complex64 needs twice the registers per stage: one block per LOW pass
    const int max_nb = p->dtype == BF_C64 ? 1 : 2;
    if (L <= 10) {
        for (int k = 0; k < p->nblocks; k += max_nb) {
            if (pl.npass == kMaxPasses) return pl;
            Pass &q = pl.pass[pl.npass++];
            q = Pass{};
            q.NB = std::min<int>(max_nb, (int)p->nblocks - k);
            q.t0 = k * L;
            q.t1 = (k + q.NB) * L;
            q.L = L;
            q.inc = (p->increasing_stride != 0) != ((k & 1) != 0);
        }
    } else if (L <= 12 && forward_only && (p->dtype == BF_F32 || L == 11) &&
               p->batch * p->nstacks >= wide_min_rows(p)) {
        for (int k = 0; k < p->nblocks; ++k) {
            if (pl.npass == kMaxPasses) return pl;
            Pass &q = pl.pass[pl.npass++];
            q = Pass{};
            q.wide = true;
            q.t0 = k * L;
            q.t1 = (k + 1) * L;
            q.L = L;
            q.inc = (p->increasing_stride != 0) != ((k & 1) != 0);
        }
    } else {
        // bits 0..low-1: the kernels on chunks of 2^low elements; the bits above them: spans of up
        // to kSpanMaxBits adjacent bits, as equal as possible, each one pass of the same kernels
        // over tiles (SpanPlan) -- float n = 4096: [10,11]; n = 2^20: [10..14] [15..19].
        // float: low = 10.  complex64 holds one block per LOW pass and ten complex stages fill the
        // registers (one row in flight, factors parked in LDS), so its low width is the smallest
        // one (not below 6: then a LOW pass needs no transposition) that keeps the number of
        // spans: n = 4096: LOW on bits 0..5, one span [6..11]; n = 8192: bits 0..6, [7..12].
        const bool cplx = p->dtype == BF_C64;
        const int span_max = cplx ? kSpanMaxBitsComplex : kSpanMaxBits;
        const int nspans = (L - 10 + span_max - 1) / span_max;
        // (rows up to 2^16 only: shorter chunks mean more rows per workgroup, and beyond that the
        // rows a workgroup must reach with 32-bit offsets run out)
        // Not through column tables either: a gather or scatter touches one element per 128-byte
        // line and short chunk, where chunks of 1024 still find several (measured on the bit
        // reversal of special.fft: 1.30 ms against 0.92 ms per step).
        const int low = cplx && L <= 16 && !permuted ? std::max(6, L - span_max * nspans) : 10;
        pl.low = low;
        const int hbits = L - low;
        int group_lb[16], group_bits[16], ngroups = 0;
        for (int b = low; b < L; ++ngroups) {
            group_lb[ngroups] = b;
            group_bits[ngroups] = hbits / nspans + (ngroups < hbits % nspans ? 1 : 0);
            b += group_bits[ngroups];
        }
        auto group_of = [&](int bit) {
            if (bit < low) return -1;
            int g = 0;
            while (bit >= group_lb[g] + group_bits[g]) ++g;
            return g;
        };
        int t = 0;
        while (t < NS) {
            if (pl.npass == kMaxPasses) return pl;
            Pass &q = pl.pass[pl.npass++];
            q = Pass{};
            q.t0 = t;
            const int grp = group_of(stage_bit(p, t));
            const bool high = grp >= 0;
            // a group also takes the way back down where two blocks meet in the row's top bits
            const int lb = high ? group_lb[grp] : 0;
            const int H = high ? group_bits[grp] : 0;
            // (a complex64 span takes the way back down only if both sweeps fit one pass)
            const int cap = high ? (cplx && 2 * H > kSpanMaxStagesComplex ? H : 2 * H) : low * max_nb;
            int u = t;
            while (u < NS && group_of(stage_bit(p, u)) == grp && u - t < cap) ++u;
            q.t1 = u;
            if (high) {
                q.span = true;
                q.L = 10;
                q.NB = 1;
                q.lb = lb;
                q.H = H;
                if (u - t != H && u - t != 2 * H) return pl;
                q.mode = u - t == 2 * H ? 2 : (stage_bit(p, t) == lb ? 0 : 1);
                q.inc = q.mode != 1;
            } else {
                q.L = low;
                if ((u - t) != low && (u - t) != 2 * low) return pl;
                q.NB = (u - t) / low;
                q.inc = stage_bit(p, t) == 0;
            }
            t = u;
        }
    }
    pl.ok = true;
    return pl;
}

int fw_rows(const bf_problem *p) { return p->dtype == BF_C64 ? kFastFwRowsComplex : kFastFwRows; }

struct FastGrid {
    int64_t slots, ngroups, nwg, groups_per_wg;
};

constexpr int64_t kNoRowCap = INT64_MAX / 4;
constexpr int kRowMargin = 8;  // rows a kernel may address past its share (prefetch, rows in flight)

// Rows within reach of 32-bit byte offsets from a workgroup's first row, over all operands of
// the call (the kernels address every operand relative to that row).
int64_t row_cap(const bf_problem *p, bool backward)
{
    const int64_t n = (int64_t)1 << p->log_n;
    const double e = (double)elem_bytes(p->dtype);
    const int64_t dense[3] = {p->nstacks * n, n, 1};
    const int64_t *strides[4] = {p->input_stride, p->output_stride, dense, backward ? p->d_input_stride : dense};
    double cap = (double)kNoRowCap;
    for (const int64_t *st : strides) {
        if (st[0] <= 0) continue;
        cap = std::min(cap, (2147483000.0 / e - (double)n * (double)st[2]) / (double)st[0]);
    }
    return cap < 0 ? 0 : (int64_t)cap;
}

// Row-group partition of a LOW pass: `lanes` independent (stack, chunk) columns share the CUs;
// a workgroup walks at most max_rows rows (more workgroups than compute units if need be).
// `slices`: the pass is a base-2 backward pass, whose workgroups each end with a partial slice of
// the d_twiddle sums (written once, read once by the reduce) whatever the number of rows they
// walked.  With few rows that traffic outweighs the row loop: walking one more row group costs a
// workgroup about as much as 27 * 1024 / n of its slices cost the device (measured on the
// two-block 1024-element kernels at 256 ... 4096 rows: 1.1 us per row against 0.04 us per 160 KiB
// slice written and re-read), so the host picks the number of row groups per workgroup that makes
// groups * row + workgroups * slice least.
FastGrid fast_grid(int64_t batch, int Lk, int64_t lanes, int rows_in_flight, int wg_per_cu,
                   int64_t max_rows = kNoRowCap, bool slices = false)
{
    FastGrid g;
    g.slots = 1024 >> Lk;
    g.ngroups = (batch + g.slots - 1) / g.slots;
    int64_t want = std::max<int64_t>(1, (int64_t)num_cu() * wg_per_cu / lanes);
    const int64_t iters = (g.ngroups + rows_in_flight - 1) / rows_in_flight;
    if (slices && iters > 0) {
        const double slice = 1.0 / (27.0 * (double)g.slots);   // in units of one row group's time
        auto cost = [&](int64_t groups) { return (double)groups + (double)((iters + groups - 1) / groups) * slice; };
        int64_t best = (iters + want - 1) / want;
        for (int64_t groups = best + 1; groups <= iters && (double)groups < cost(best); ++groups)
            if (cost(groups) < cost(best)) best = groups;
        want = (iters + best - 1) / best;
    }
    g.nwg = std::min(want, iters);
    g.groups_per_wg = ((iters + g.nwg - 1) / g.nwg) * rows_in_flight;
    const int64_t max_groups = ((max_rows / g.slots - kRowMargin) / rows_in_flight) * rows_in_flight;
    if (max_groups >= rows_in_flight && g.groups_per_wg > max_groups) g.groups_per_wg = max_groups;
    g.nwg = (g.ngroups + g.groups_per_wg - 1) / g.groups_per_wg;
    return g;
}

// Row partition of a WIDE pass: one row at a time per workgroup.
FastGrid wide_grid(int64_t batch, int64_t nstacks)
{
    FastGrid g;
    g.slots = 1;
    g.ngroups = batch;
    const int64_t want = std::max<int64_t>(1, (int64_t)num_cu() / nstacks);
    g.nwg = std::min(want, batch);
    g.groups_per_wg = (batch + g.nwg - 1) / g.nwg;
    g.nwg = (batch + g.groups_per_wg - 1) / g.groups_per_wg;
    return g;
}

// True when every pass can address its operands with 32-bit offsets.
bool passes_addressable(const bf_problem *p, const PassPlan &pl, bool backward)
{
    const int64_t n = (int64_t)1 << p->log_n;
    const int64_t cap = row_cap(p, backward);
    int64_t rows = 0;
    for (int k = 0; k < pl.npass; ++k) {
        const Pass &q = pl.pass[k];
        const FastGrid g = q.wide ? wide_grid(p->batch, p->nstacks)
                                  : fast_grid(p->batch, q.L, p->nstacks * pass_lanes(p, q), backward ? 1 : fw_rows(p),
                                              backward ? 1 : fw_wg_per_cu(p, q), cap, backward);
        rows = std::max(rows, (g.groups_per_wg + kFastFwRows + 2) * g.slots);
    }
    const int64_t dense[3] = {p->nstacks * n, n, 1};
    const size_t e = elem_bytes(p->dtype);
    if (!span_ok(p->input_stride, rows, n, e) || !span_ok(p->output_stride, rows, n, e) || !span_ok(dense, rows, n, e))
        return false;
    if (backward && !span_ok(p->d_input_stride, rows, n, e)) return false;
    return true;
}

// paired: the grid holds two workgroups per compute unit (fw_wg_per_cu)
template <int L, int NB, bool INC>
void launch_fast_fw_t(bool cplx, bool paired, const FastFwArgs &a, dim3 grid, hipStream_t stream)
{
    if constexpr (NB == 1) {
        if (cplx) {
            hipLaunchKernelGGL((fast_fw_kernel<float2, FastPlan<L, NB, INC>, kFastFwRowsComplex>), grid, dim3(kFastThreads), 0,
                               stream, a);
            return;
        }
    } else if constexpr (fw_pairable(L, INC)) {
        if (paired) {
            hipLaunchKernelGGL((fast_fw_kernel<float, FastPlan<L, NB, INC>, kFastFwRows, 8>), grid, dim3(kFastThreads), 0,
                               stream, a);
            return;
        }
    }
    hipLaunchKernelGGL((fast_fw_kernel<float, FastPlan<L, NB, INC>, kFastFwRows>), grid, dim3(kFastThreads), 0, stream, a);
}

template <int L, int NB, bool INC>
void launch_fast_bw_t(bool cplx, bool two_rows, const FastBwArgs &a, dim3 grid, hipStream_t stream)
{
    if constexpr (NB == 1) {
        if (cplx) {
            hipLaunchKernelGGL((fast_bw_kernel<float2, FastPlan<L, NB, INC>>), grid, dim3(kFastThreads), 0, stream, a);
            return;
        }
        if constexpr (L >= 7) {
            if (two_rows) {
                hipLaunchKernelGGL((fast_bw_kernel<float, FastPlan<L, NB, INC>, 2>), grid, dim3(kFastThreads), 0, stream, a);
                return;
            }
        }
    }
    hipLaunchKernelGGL((fast_bw_kernel<float, FastPlan<L, NB, INC>>), grid, dim3(kFastThreads), 0, stream, a);
}

// SpanPlan passes: the LOW kernels on the tiles of a span of q.H high bits.
template <int H, int MODE>
bool launch_span_t(bool cplx, bool backward, bool two_rows, const FastFwArgs *fw, const FastBwArgs *bw, dim3 grid,
                   hipStream_t stream)
{
    using P = SpanPlan<H, MODE>;
    const dim3 block(kFastThreads);
    // which combinations the host plans: float spans of up to kSpanMaxBits bits, complex64 ones of
    // up to kSpanMaxBitsComplex bits and kSpanMaxStagesComplex stages
    constexpr bool for_float = H <= kSpanMaxBits;
    constexpr bool for_complex = H * (MODE == 2 ? 2 : 1) <= kSpanMaxStagesComplex;
    if (cplx) {
        if constexpr (for_complex) {
            if (!backward) hipLaunchKernelGGL((fast_fw_kernel<float2, P, kFastFwRowsComplex>), grid, block, 0, stream, *fw);
            else hipLaunchKernelGGL((fast_bw_kernel<float2, P>), grid, block, 0, stream, *bw);
            return true;
        }
        return false;
    }
    if constexpr (for_float) {
        if (!backward) hipLaunchKernelGGL((fast_fw_kernel<float, P, kFastFwRows>), grid, block, 0, stream, *fw);
        else if (two_rows) hipLaunchKernelGGL((fast_bw_kernel<float, P, 2>), grid, block, 0, stream, *bw);
        else hipLaunchKernelGGL((fast_bw_kernel<float, P>), grid, block, 0, stream, *bw);
        return true;
    }
    return false;
}

int launch_span(bool cplx, const Pass &q, bool backward, bool two_rows, const FastFwArgs *fw, const FastBwArgs *bw,
                dim3 grid, hipStream_t stream)
{
#define BF_SPAN_CASES(HH)                                                                          \
    case HH * 3 + 0: ok = launch_span_t<HH, 0>(cplx, backward, two_rows, fw, bw, grid, stream); break;   \
    case HH * 3 + 1: ok = launch_span_t<HH, 1>(cplx, backward, two_rows, fw, bw, grid, stream); break;   \
    case HH * 3 + 2: ok = launch_span_t<HH, 2>(cplx, backward, two_rows, fw, bw, grid, stream); break;
    bool ok = false;
    switch (q.H * 3 + q.mode) {
#ifndef BF_DEV_SUBSET
        BF_SPAN_CASES(1) BF_SPAN_CASES(2) BF_SPAN_CASES(3) BF_SPAN_CASES(4) BF_SPAN_CASES(5) BF_SPAN_CASES(6)
#endif
        default: break;
    }
#undef BF_SPAN_CASES
    if (!ok) return fail(BF_ERR_UNSUPPORTED, "no kernel for a span of %d bits in mode %d", q.H, q.mode);
    return BF_OK;
}

#define BF_FAST_DISPATCH(FN, Q, ...)                                                     \
    do {                                                                                 \
        const int key_ = (Q).L * 4 + ((Q).NB - 1) * 2 + ((Q).inc ? 1 : 0);               \
        switch (key_) {                                                                  \
            BF_FAST_SHORT_CASES(FN, __VA_ARGS__) BF_FAST_CASES(FN, 10, __VA_ARGS__)      \
            default: return fail(BF_ERR_UNSUPPORTED, "no fast kernel for this shape");   \
        }                                                                                \
    } while (0)
// BF_DEV_SUBSET (development builds only): instantiate nothing but the kernels of 1024-element
// float / complex64 rows, so that a variant of those compiles in a fraction of the time; every
// other shape answers BF_ERR_UNSUPPORTED.  The shipped library is built without it.
#ifdef BF_DEV_SUBSET
#define BF_FAST_SHORT_CASES(FN, ...)
#else
#define BF_FAST_SHORT_CASES(FN, ...)                                                     \
    BF_FAST_CASES(FN, 1, __VA_ARGS__) BF_FAST_CASES(FN, 2, __VA_ARGS__)                  \
    BF_FAST_CASES(FN, 3, __VA_ARGS__) BF_FAST_CASES(FN, 4, __VA_ARGS__)                  \
    BF_FAST_CASES(FN, 5, __VA_ARGS__) BF_FAST_CASES(FN, 6, __VA_ARGS__)                  \
    BF_FAST_CASES(FN, 7, __VA_ARGS__) BF_FAST_CASES(FN, 8, __VA_ARGS__)                  \
    BF_FAST_CASES(FN, 9, __VA_ARGS__)
#endif
#define BF_FAST_CASES(FN, LL, ...)                              \
    case LL * 4 + 0: FN<LL, 1, false>(__VA_ARGS__); break;      \
    case LL * 4 + 1: FN<LL, 1, true>(__VA_ARGS__); break;       \
    case LL * 4 + 2: FN<LL, 2, false>(__VA_ARGS__); break;      \
    case LL * 4 + 3: FN<LL, 2, true>(__VA_ARGS__); break;

void fill_stage_table(int *dst, int cap, const Pass &q)
{
    for (int s = 0; s < cap; ++s) dst[s] = q.t0 + std::min(s, q.t1 - q.t0 - 1);
}

// Forward through the pass plan.  `scratch` holds one dense (B, S, n) activation when there
// is more than one pass (passes run in place on it).
// `bias` (may be NULL) is added by the last pass when that pass runs in a kernel that can do
// it; *bias_done says whether it was.
int multipass_forward(const bf_problem *p, const PassPlan &pl, const void *tw, const void *input, void *output,
                      void *scratch, const View &in_view, const View &out_view, int first, int last,
                      hipStream_t stream, const void *bias = nullptr, bool *bias_done = nullptr)
{
    if (bias_done) *bias_done = false;
    const int64_t n = (int64_t)1 << p->log_n;
    const View dense = dense_view(p->nstacks, n);
    for (int k = first; k < last; ++k) {
        const Pass &q = pl.pass[k];
        const void *src = k == first ? input : scratch;
        void *dst = k == last - 1 ? output : scratch;
        const View sv = k == first ? in_view : dense;
        const View dv = k == last - 1 ? out_view : dense;
        if (q.wide) {
            const FastGrid g = wide_grid(p->batch, p->nstacks);
            FastFwArgs a = {};
            a.tw = tw;
            a.tw_stack_stride = p->nblocks * p->log_n * (n / 2) * 4;
            a.tw_stage_stride = (n / 2) * 4;
            fill_stage_table(a.tw_stage, kFastMaxStages, q);
            a.in = src;
            a.in_view = sv;
            a.out = dst;
            a.out_view = dv;
            a.batch = p->batch;
            a.ngroups = g.ngroups;
            a.groups_per_wg = g.groups_per_wg;
            if (k == last - 1 && bias) {
                a.bias = bias;
                if (bias_done) *bias_done = true;
            }
            const dim3 grid((unsigned)g.nwg, (unsigned)p->nstacks, 1);
            const dim3 block(kFastThreads);
            const bool cplx = p->dtype == BF_C64;
#ifdef BF_DEV_SUBSET
            (void)cplx; (void)grid; (void)block; (void)a;
            return fail(BF_ERR_UNSUPPORTED, "development subset: no whole-block forward kernels");
#else
            if (q.L == 12 && q.inc) hipLaunchKernelGGL((wide_fw_kernel<float, 12, true>), grid, block, 0, stream, a);
            else if (q.L == 12) hipLaunchKernelGGL((wide_fw_kernel<float, 12, false>), grid, block, 0, stream, a);
            else if (cplx && q.inc) hipLaunchKernelGGL((wide_fw_kernel<float2, 11, true>), grid, block, 0, stream, a);
            else if (cplx) hipLaunchKernelGGL((wide_fw_kernel<float2, 11, false>), grid, block, 0, stream, a);
            else if (q.inc) hipLaunchKernelGGL((wide_fw_kernel<float, 11, true>), grid, block, 0, stream, a);
            else hipLaunchKernelGGL((wide_fw_kernel<float, 11, false>), grid, block, 0, stream, a);
#endif
            BF_HIP_CHECK(hipGetLastError());
        } else {
            const int per_cu = fw_wg_per_cu(p, q);
            const FastGrid g = fast_grid(p->batch, q.L, p->nstacks * pass_lanes(p, q), fw_rows(p), per_cu, row_cap(p, false));
            FastFwArgs a = {};
            a.tw = tw;
            a.tw_stack_stride = p->nblocks * p->log_n * (n / 2) * 4;
            a.tw_stage_stride = (n / 2) * 4;
            fill_stage_table(a.tw_stage, kFastMaxStages, q);
            a.in = src;
            a.in_view = sv;
            a.out = dst;
            a.out_view = dv;
            a.batch = p->batch;
            a.ngroups = g.ngroups;
            a.groups_per_wg = g.groups_per_wg;
            if (k == last - 1 && bias) {
                a.bias = bias;
                if (bias_done) *bias_done = true;
            }
            const dim3 grid((unsigned)g.nwg, (unsigned)p->nstacks, (unsigned)pass_lanes(p, q));
            if (q.span) {
                a.low_bits = q.lb;
                const int rc = launch_span(p->dtype == BF_C64, q, false, false, &a, nullptr, grid, stream);
                if (rc) return rc;
            } else {
                BF_FAST_DISPATCH(launch_fast_fw_t, q, p->dtype == BF_C64, per_cu == 2, a, grid, stream);
            }
            BF_HIP_CHECK(hipGetLastError());
        }
    }
    return BF_OK;
}

// ---- base-4 register-resident path (float, even log_n <= 10): one launch per block -----------

constexpr int kFast4FwRows = 4;

constexpr int kFast4GFwRowsComplex = 2;

// base-4 shapes outside fast4.hpp's aligned float kernels
bool fast4_general(const bf_problem *p) { return p->dtype != BF_F32 || (p->log_n & 1) != 0; }

int fast4_fw_rows(const bf_problem *p) { return p->dtype == BF_C64 ? kFast4GFwRowsComplex : kFast4FwRows; }

// Which register-resident base-4 kernels take this problem: 0 none (generic kernels), 1 the
// aligned float kernels of fast4.hpp (even log_n), 2 the general ones of fast4g.hpp (odd
// log_n, complex64 up to n = 256: beyond that the complex factors outgrow the registers).
int fast4_kind(const bf_problem *p, bool base4, bool backward)
{
    if (!base4 || p->log_n < 2 || p->log_n > 10 || p->nblocks < 1 || p->batch <= 0 || p->nstacks <= 0 ||
        p->input_size <= 0 || p->output_size <= 0)
        return 0;
    if (p->dtype == BF_C64 && p->log_n > 8) return 0;
    const int64_t n = (int64_t)1 << p->log_n;
    const size_t e = elem_bytes(p->dtype);
    const FastGrid g = fast_grid(p->batch, (int)p->log_n, p->nstacks, backward ? 1 : fast4_fw_rows(p), 1);
    const int64_t rows = (g.groups_per_wg + kFast4FwRows + 2) * g.slots;
    const int64_t dense[3] = {p->nstacks * n, n, 1};
    if (!span_ok(p->input_stride, rows, n, e) || !span_ok(p->output_stride, rows, n, e) || !span_ok(dense, rows, n, e))
        return 0;
    if (backward && !span_ok(p->d_input_stride, rows, n, e)) return 0;
    return fast4_general(p) ? 2 : 1;
}

bool fast4_ok(const bf_problem *p, bool base4, bool backward) { return fast4_kind(p, base4, backward) != 0; }

template <int L, bool INC>
void launch_fast4_t(bool backward, const Fast4Args &a, dim3 grid, hipStream_t stream)
{
    // row groups per backward iteration: as many as the registers next to the factors allow
    constexpr int RB = L <= 8 ? 4 : 2;
    if (backward) hipLaunchKernelGGL((fast4_bw_kernel<L, INC, RB>), grid, dim3(kFastThreads), 0, stream, a);
    else hipLaunchKernelGGL((fast4_fw_kernel<L, INC, kFast4FwRows>), grid, dim3(kFastThreads), 0, stream, a);
}

int launch_fast4(int L, bool inc, bool backward, const Fast4Args &a, dim3 grid, hipStream_t stream)
{
    switch (L * 2 + (inc ? 1 : 0)) {
#ifndef BF_DEV_SUBSET
        case 2 * 2 + 0: launch_fast4_t<2, false>(backward, a, grid, stream); break;
        case 2 * 2 + 1: launch_fast4_t<2, true>(backward, a, grid, stream); break;
        case 4 * 2 + 0: launch_fast4_t<4, false>(backward, a, grid, stream); break;
        case 4 * 2 + 1: launch_fast4_t<4, true>(backward, a, grid, stream); break;
        case 6 * 2 + 0: launch_fast4_t<6, false>(backward, a, grid, stream); break;
        case 6 * 2 + 1: launch_fast4_t<6, true>(backward, a, grid, stream); break;
        case 8 * 2 + 0: launch_fast4_t<8, false>(backward, a, grid, stream); break;
        case 8 * 2 + 1: launch_fast4_t<8, true>(backward, a, grid, stream); break;
        case 10 * 2 + 0: launch_fast4_t<10, false>(backward, a, grid, stream); break;
        case 10 * 2 + 1: launch_fast4_t<10, true>(backward, a, grid, stream); break;
#endif
        default: return fail(BF_ERR_UNSUPPORTED, "no base-4 kernel for this shape");
    }
    BF_HIP_CHECK(hipGetLastError());
    return BF_OK;
}

template <typename T, int L, bool INC>
void launch_fast4g_t(bool backward, const Fast4GArgs &a, dim3 grid, hipStream_t stream)
{
    constexpr int R = sizeof(T) == 4 ? kFast4FwRows : kFast4GFwRowsComplex;
    // row groups per backward iteration: what the registers next to the factors allow
    constexpr int RB = sizeof(T) == 4 ? (L <= 7 ? 4 : 2) : (L <= 6 ? 2 : 1);
    if (backward) hipLaunchKernelGGL((fast4g_bw_kernel<T, L, INC, RB>), grid, dim3(kFastThreads), 0, stream, a);
    else hipLaunchKernelGGL((fast4g_fw_kernel<T, L, INC, R>), grid, dim3(kFastThreads), 0, stream, a);
}

// (float L = 10 only runs on the 1024-element chunks of longer rows: whole rows of 1024 take fast4.hpp)
int launch_fast4g(bool cplx, int L, bool inc, bool backward, const Fast4GArgs &a, dim3 grid, hipStream_t stream)
{
#define BF_F4G(LL)                                                                              \
    case LL * 2 + 0: launch_fast4g_t<float, LL, false>(backward, a, grid, stream); break;        \
    case LL * 2 + 1: launch_fast4g_t<float, LL, true>(backward, a, grid, stream); break;
#define BF_C4G(LL)                                                                              \
    case LL * 2 + 0: launch_fast4g_t<float2, LL, false>(backward, a, grid, stream); break;       \
    case LL * 2 + 1: launch_fast4g_t<float2, LL, true>(backward, a, grid, stream); break;
    if (cplx) {
        switch (L * 2 + (inc ? 1 : 0)) {
#ifndef BF_DEV_SUBSET
            BF_C4G(2) BF_C4G(3) BF_C4G(4) BF_C4G(5) BF_C4G(6) BF_C4G(7) BF_C4G(8)
#endif
            default: return fail(BF_ERR_UNSUPPORTED, "no base-4 kernel for this shape");
        }
    } else {
        switch (L * 2 + (inc ? 1 : 0)) {
#ifndef BF_DEV_SUBSET
            BF_F4G(3) BF_F4G(5) BF_F4G(7) BF_F4G(9) BF_F4G(10)
#endif
            default: return fail(BF_ERR_UNSUPPORTED, "no base-4 kernel for this shape");
        }
    }
#undef BF_F4G
#undef BF_C4G
    BF_HIP_CHECK(hipGetLastError());
    return BF_OK;
}

// Operands of block k for the general base-4 kernels
Fast4GArgs fast4g_block_args(const bf_problem *p, const void *tw4, const void *tw2, int k)
{
    const int64_t n = (int64_t)1 << p->log_n;
    const int L = (int)p->log_n;
    const size_t e = elem_bytes(p->dtype);
    Fast4GArgs a = {};
    a.tw4 = static_cast<const char *>(tw4) + (size_t)k * (L / 2) * (n / 4) * 16 * e;
    a.tw4_stack_stride = p->nblocks * (L / 2) * (n / 4) * 16;
    a.tw2 = (L & 1) ? static_cast<const char *>(tw2) + (size_t)k * (n / 2) * 4 * e : nullptr;
    a.tw2_stack_stride = p->nblocks * (L & 1) * (n / 2) * 4;
    a.tw4_stage_stride = (n / 4) * 16;
    a.n_full = n;
    a.batch = p->batch;
    return a;
}

// Forward workgroups per compute unit of the aligned float kernels (fast4.hpp).  They fit a CU
// twice as they are (at most 51 registers, 33 KiB of LDS), and where a block crosses between the
// layouts (n >= 256: LDS transposes, barriers) two resident workgroups fill each other's gaps once
// each has a few iterations: 23.0 against 25.9 us at 16384 x 4 rows of 256, 24.3 against 27.5 at
// 16384 rows of 1024; rows of 64 stay within a wavefront and gain nothing.
int fast4_fw_wg_per_cu(const bf_problem *p)
{
    if (fast4_general(p) || p->log_n < 8) return 1;
    const int64_t slots = 1024 >> p->log_n;
    const int64_t iters = ((p->batch + slots - 1) / slots + kFast4FwRows - 1) / kFast4FwRows;
    const int64_t pairs = std::max<int64_t>(1, 2 * (int64_t)num_cu() / p->nstacks);
    return iters >= pairs * BF_FAST_FW_PAIR_MIN_ITERS ? 2 : 1;
}

// forward of blocks [first, last) through the base-4 kernels; `scratch` as in multipass_forward
int fast4_forward(const bf_problem *p, const void *tw4, const void *tw2, const void *input, void *output,
                  void *scratch, const View &in_view, const View &out_view, int first, int last, hipStream_t stream)
{
    const int64_t n = (int64_t)1 << p->log_n;
    const int L = (int)p->log_n;
    const View dense = dense_view(p->nstacks, n);
    const FastGrid g = fast_grid(p->batch, L, p->nstacks, fast4_fw_rows(p), fast4_fw_wg_per_cu(p));
    if (fast4_general(p)) {
        for (int k = first; k < last; ++k) {
            Fast4GArgs a = fast4g_block_args(p, tw4, tw2, k);
            a.x_in = k == first ? input : scratch;
            a.x_view = k == first ? in_view : dense;
            a.x_out = k == last - 1 ? output : scratch;
            a.xo_view = k == last - 1 ? out_view : dense;
            a.ngroups = g.ngroups;
            a.groups_per_wg = g.groups_per_wg;
            const bool inc = (p->increasing_stride != 0) != ((k & 1) != 0);
            const int rc = launch_fast4g(p->dtype == BF_C64, L, inc, false, a,
                                         dim3((unsigned)g.nwg, (unsigned)p->nstacks), stream);
            if (rc) return rc;
        }
        return BF_OK;
    }
    if ((reinterpret_cast<uintptr_t>(tw4) & 15) != 0)
        return fail(BF_ERR_INVALID, "twiddle4 must be 16-byte aligned");
    for (int k = first; k < last; ++k) {
        Fast4Args a = {};
        a.tw4 = static_cast<const float *>(tw4) + (int64_t)k * (L / 2) * (n / 4) * 16;
        a.tw_stack_stride = p->nblocks * (L / 2) * (n / 4) * 16;
        a.x_in = static_cast<const float *>(k == first ? input : scratch);
        a.x_view = k == first ? in_view : dense;
        a.x_out = static_cast<float *>(k == last - 1 ? output : scratch);
        a.xo_view = k == last - 1 ? out_view : dense;
        a.batch = p->batch;
        a.ngroups = g.ngroups;
        a.groups_per_wg = g.groups_per_wg;
        const bool inc = (p->increasing_stride != 0) != ((k & 1) != 0);
        const int rc = launch_fast4(L, inc, false, a, dim3((unsigned)g.nwg, (unsigned)p->nstacks), stream);
        if (rc) return rc;
    }
    return BF_OK;
}

// ---- base-4 rows beyond the reach of one workgroup's registers ------------------------------------
//
// A block of a long base-4 row is cut into passes, one launch each:
//   * a CHUNK pass: the general base-4 kernels (fast4g.hpp) on independent chunks of 2^LC elements
//     for the stages that stay inside a chunk -- with increasing stride the first LC / 2 radix-4
//     stages (LC = 10 float, 8 complex64); with decreasing stride the last ones and, for odd
//     log_n, the closing 2x2 stage on bit 0 (LC = 9 / 7 then, so that the bit pairs line up);
//   * one STAGE pass (stage.hpp) per remaining stage: the radix-4 stages on the bits above the
//     chunk and, with increasing stride and odd log_n, the closing 2x2 stage on the top bit.
struct Pass4 {
    bool chunk;
    int t0, t1;        // global stage range [t0, t1)
    int LC;            // chunk pass: log2 of the chunk length
    bool inc;
    int block, idx0;   // chunk pass: block and index (within the block) of its first radix-4 stage
};

struct Plan4Long {
    bool ok = false;
    int npass = 0;
    Pass4 pass[kMaxPasses];
};

Plan4Long plan4_long(const bf_problem *p, bool base4)
{
    Plan4Long pl;
    {
        // the chunk kernels address their operands with 32-bit offsets from a workgroup's first row
        const int64_t n = (int64_t)1 << p->log_n;
        const size_t e = elem_bytes(p->dtype);
        const int64_t rows = (p->batch + kFast4FwRows + 2) * 8;   // (any workgroup's share, with margin)
        const int64_t dense[3] = {p->nstacks * n, n, 1};
        if (!span_ok(p->input_stride, rows, n, e) || !span_ok(p->output_stride, rows, n, e) ||
            !span_ok(dense, rows, n, e) || !span_ok(p->d_input_stride, rows, n, e))
            return pl;
    }
    const int L = (int)p->log_n;
    const int reach = p->dtype == BF_C64 ? 8 : 10;
    if (!base4 || L <= reach || L > kMaxLogN || p->nblocks < 1 || p->batch <= 0 || p->nstacks <= 0 ||
        p->input_size <= 0 || p->output_size <= 0)
        return pl;
    const int per = L / 2 + (L & 1), l4 = L / 2;
    for (int k = 0; k < p->nblocks; ++k) {
        const bool inc = (p->increasing_stride != 0) != ((k & 1) != 0);
        const int LC = (inc || !(L & 1)) ? reach : reach - 1;
        const int nlow = LC / 2, nhigh = l4 - nlow;
        auto add = [&](bool chunk, int t0, int t1, int idx0) {
            if (pl.npass == kMaxPasses) return false;
            Pass4 &q = pl.pass[pl.npass++];
            q.chunk = chunk;
            q.t0 = t0;
            q.t1 = t1;
            q.LC = LC;
            q.inc = inc;
            q.block = k;
            q.idx0 = idx0;
            return true;
        };
        if (inc) {
            if (!add(true, k * per, k * per + nlow, 0)) return pl;
            for (int j = nlow; j < per; ++j)
                if (!add(false, k * per + j, k * per + j + 1, j)) return pl;
        } else {
            for (int j = 0; j < nhigh; ++j)
                if (!add(false, k * per + j, k * per + j + 1, j)) return pl;
            if (!add(true, k * per + nhigh, k * per + per, nhigh)) return pl;
        }
    }
    pl.ok = true;
    return pl;
}

struct StageGrid {
    int64_t tiles, nparts, rows_per_wg;
};

StageGrid stage_grid(const bf_problem *p, int radix)
{
    const int64_t n = (int64_t)1 << p->log_n;
    StageGrid g;
    g.tiles = (n / radix + kStageThreads - 1) / kStageThreads;
    const int64_t want = std::max<int64_t>(1, (int64_t)num_cu() * 8 / (g.tiles * p->nstacks));
    g.nparts = std::min<int64_t>(std::min<int64_t>(want, p->batch), 65535);
    g.rows_per_wg = (p->batch + g.nparts - 1) / g.nparts;
    g.nparts = (p->batch + g.rows_per_wg - 1) / g.rows_per_wg;
    return g;
}

FastGrid chunk4_grid(const bf_problem *p, const Pass4 &q, bool backward)
{
    const int64_t chunks = (int64_t)1 << (p->log_n - q.LC);
    return fast_grid(p->batch, q.LC, p->nstacks * chunks, backward ? 1 : fast4_fw_rows(p), 1);
}

// partial slices (of 4 n scalars per stage) the backward of this pass writes
int64_t pass4_slices(const bf_problem *p, const Pass4 &q)
{
    if (q.chunk) return chunk4_grid(p, q, true).nwg * (q.t1 - q.t0);
    return stage_grid(p, stage_info(make_schedule(p, true), q.t0).radix4 ? 4 : 2).nparts;
}

// One pass forward (backward == false: x_in -> x_out) or backward (x_in, g_out -> g_in and the
// pass's partial slices; *nparts receives their number per stage).
int run_pass4(const bf_problem *p, const Schedule &sc, const Pass4 &q, bool backward, const void *tw2, const void *tw4,
              const void *x_in, const View &x_view, void *x_out, const View &xo_view, const void *g_out,
              const View &g_view, void *g_in, const View &gi_view, void *partial, int64_t *nparts, hipStream_t stream)
{
    const int64_t n = (int64_t)1 << p->log_n;
    const int L = (int)p->log_n;
    const size_t e = elem_bytes(p->dtype);
    const bool cplx = p->dtype == BF_C64;
    if (q.chunk) {
        const FastGrid g = chunk4_grid(p, q, backward);
        Fast4GArgs a = {};
        a.tw4 = static_cast<const char *>(tw4) + ((size_t)q.block * (L / 2) + q.idx0) * (n / 4) * 16 * e;
        a.tw4_stack_stride = sc.tw4_stack_stride;
        a.tw4_stage_stride = (n / 4) * 16;
        a.tw2 = (L & 1) ? static_cast<const char *>(tw2) + (size_t)q.block * (n / 2) * 4 * e : nullptr;
        a.tw2_stack_stride = sc.tw2_stack_stride;
        a.n_full = n;
        a.x_in = x_in;
        a.x_view = x_view;
        a.x_out = x_out;
        a.xo_view = xo_view;
        a.g_out = g_out;
        a.g_view = g_view;
        a.g_in = g_in;
        a.gi_view = gi_view;
        a.partial = partial;
        a.batch = p->batch;
        a.ngroups = g.ngroups;
        a.groups_per_wg = g.groups_per_wg;
        if (nparts) *nparts = g.nwg;
        return launch_fast4g(cplx, q.LC, q.inc, backward, a,
                             dim3((unsigned)g.nwg, (unsigned)p->nstacks, (unsigned)(n >> q.LC)), stream);
    }
    const StageInfo si = stage_info(sc, q.t0);
    const int radix = si.radix4 ? 4 : 2;
    const StageGrid g = stage_grid(p, radix);
    StageArgs a = {};
    a.tw = static_cast<const char *>(si.radix4 ? tw4 : tw2) + (size_t)si.tw_off * e;
    a.tw_stack_stride = si.radix4 ? sc.tw4_stack_stride : sc.tw2_stack_stride;
    a.log_stride = si.log_stride;
    a.n = n;
    a.x_in = x_in;
    a.x_view = x_view;
    a.x_out = x_out;
    a.xo_view = xo_view;
    a.g_out = g_out;
    a.g_view = g_view;
    a.g_in = g_in;
    a.gi_view = gi_view;
    a.partial = partial;
    a.slot = 4 * n;
    a.batch = p->batch;
    a.rows_per_wg = g.rows_per_wg;
    if (nparts) *nparts = g.nparts;
    const dim3 grid((unsigned)g.nparts, (unsigned)p->nstacks, (unsigned)g.tiles), block(kStageThreads);
    if (!backward) {
        if (cplx && si.radix4) hipLaunchKernelGGL((stage_fw_kernel<float2, 4>), grid, block, 0, stream, a);
        else if (cplx) hipLaunchKernelGGL((stage_fw_kernel<float2, 2>), grid, block, 0, stream, a);
        else if (si.radix4) hipLaunchKernelGGL((stage_fw_kernel<float, 4>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((stage_fw_kernel<float, 2>), grid, block, 0, stream, a);
    } else {
        if (cplx && si.radix4) hipLaunchKernelGGL((stage_bw_kernel<float2, 4>), grid, block, 0, stream, a);
        else if (cplx) hipLaunchKernelGGL((stage_bw_kernel<float2, 2>), grid, block, 0, stream, a);
        else if (si.radix4) hipLaunchKernelGGL((stage_bw_kernel<float, 4>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((stage_bw_kernel<float, 2>), grid, block, 0, stream, a);
    }
    BF_HIP_CHECK(hipGetLastError());
    return BF_OK;
}

// passes [first, last) forward; `scratch` holds the activation between passes (in place)
int long4_forward(const bf_problem *p, const Schedule &sc, const Plan4Long &pl, const void *tw2, const void *tw4,
                  const void *input, void *output, void *scratch, const View &in_view, const View &out_view,
                  int first, int last, hipStream_t stream)
{
    const int64_t n = (int64_t)1 << p->log_n;
    const View dense = dense_view(p->nstacks, n);
    for (int k = first; k < last; ++k) {
        const int rc = run_pass4(p, sc, pl.pass[k], false, tw2, tw4, k == first ? input : scratch,
                                 k == first ? in_view : dense, k == last - 1 ? output : scratch,
                                 k == last - 1 ? out_view : dense, nullptr, dense, nullptr, dense, nullptr, nullptr,
                                 stream);
        if (rc) return rc;
    }
    return BF_OK;
}

// ---- generic forward ----------------------------------------------------------------------

int launch_generic_fw(const bf_problem *p, const Schedule &sc, int t0, int t1, const void *tw2,
                      const void *tw4, const void *in, const View &in_view, void *out,
                      const View &out_view, hipStream_t stream)
{
    const int64_t n = (int64_t)1 << p->log_n;
    const size_t row_bytes = (size_t)n * elem_bytes(p->dtype);
    if (row_bytes > kGenericFwLds)
        return fail(BF_ERR_UNSUPPORTED, "n = %lld does not fit in LDS (row of %zu bytes, limit %zu)",
                    (long long)n, row_bytes, kGenericFwLds);
    if (p->batch == 0 || p->nstacks == 0) return BF_OK;
    int64_t rows = std::max<int64_t>(1, (int64_t)(64 * 1024 / row_bytes));
    rows = std::min<int64_t>(rows, 32);
    while (rows > 1 && ((p->batch + rows - 1) / rows) * p->nstacks < 2048) rows /= 2;
    const int64_t gx = (p->batch + rows - 1) / rows;
    if (gx > kMaxGrid) return fail(BF_ERR_UNSUPPORTED, "batch too large for one launch");
    GenericFwArgs a;
    a.sc = sc;
    a.t0 = t0;
    a.t1 = t1;
    a.rows_per_wg = (int)rows;
    a.batch = p->batch;
    a.tw2 = tw2;
    a.tw4 = tw4;
    a.in = in;
    a.in_view = in_view;
    a.out = out;
    a.out_view = out_view;
    const dim3 grid((unsigned)gx, (unsigned)p->nstacks);
    const size_t lds = (size_t)rows * row_bytes;
    if (p->dtype == BF_F32)
        hipLaunchKernelGGL(generic_fw_kernel<float>, grid, dim3(kGenericThreads), lds, stream, a);
    else
        hipLaunchKernelGGL(generic_fw_kernel<float2>, grid, dim3(kGenericThreads), lds, stream, a);
    BF_HIP_CHECK(hipGetLastError());
    return BF_OK;
}

// Workspace of the forward call: one dense activation when the pass plan has several passes.
size_t forward_workspace(const bf_problem *p, bool base4)
{
    if (fast4_ok(p, base4, false)) {
        const int64_t n4 = (int64_t)1 << p->log_n;
        return p->nblocks > 1 ? align256((size_t)p->batch * p->nstacks * n4 * elem_bytes(p->dtype)) : 0;
    }
    const Plan4Long lp = plan4_long(p, base4);
    if (lp.ok)
        return lp.npass > 1 ? align256(((size_t)p->batch * p->nstacks << p->log_n) * elem_bytes(p->dtype)) : 0;
    const PassPlan mp = build_passes(p, base4, true);
    if (!mp.ok || mp.npass <= 1 || !passes_addressable(p, mp, false)) return 0;
    const int64_t n = (int64_t)1 << p->log_n;
    return align256((size_t)p->batch * p->nstacks * n * elem_bytes(p->dtype));
}

// output += bias over all rows, for schedules whose last pass could not add it itself
template <typename T>
int launch_bias_add(const bf_problem *p, const void *bias, void *output, const View &out_view, hipStream_t stream)
{
    if (p->batch <= 0 || p->nstacks <= 0 || p->output_size <= 0) return BF_OK;
    BiasArgs a = {};
    a.bias = bias;
    a.out = output;
    a.view = out_view;
    a.batch = p->batch;
    a.width = p->output_size;
    const int64_t cols = (p->output_size + kBiasThreads - 1) / kBiasThreads;
    const int64_t want = std::max<int64_t>(1, (int64_t)num_cu() * 8 / (cols * p->nstacks));
    a.nparts = std::min<int64_t>(std::min<int64_t>(want, p->batch), 65535);
    a.rows_per_part = (p->batch + a.nparts - 1) / a.nparts;
    a.nparts = (p->batch + a.rows_per_part - 1) / a.rows_per_part;
    const dim3 grid((unsigned)cols, (unsigned)p->nstacks, (unsigned)a.nparts);
    hipLaunchKernelGGL((bias_add_kernel<T>), grid, dim3(kBiasThreads), 0, stream, a);
    BF_HIP_CHECK(hipGetLastError());
    return BF_OK;
}

// Column tables are only defined over the n columns of the transform and need a stage to ride on.
int check_perms(const bf_problem *p, bool base4, const int *in_perm, const int *out_index)
{
    if (!in_perm && !out_index) return BF_OK;
    const int64_t n = (int64_t)1 << p->log_n;
    if (p->input_size > n) return fail(BF_ERR_INVALID, "column tables need input_size <= n");
    if (make_schedule(p, base4).per * p->nblocks == 0)
        return fail(BF_ERR_UNSUPPORTED, "column tables need at least one stage");
    return BF_OK;
}

int forward(const bf_problem *p, bool base4, const void *tw2, const void *tw4, const void *input,
            void *output, void *workspace, size_t workspace_bytes, void *stream_, const void *bias = nullptr,
            const int *in_perm = nullptr, const int *out_index = nullptr)
{
    int rc = check_problem(p, false);
    if (rc) return rc;
    if ((rc = check_perms(p, base4, in_perm, out_index))) return rc;
    if ((rc = ensure_attributes())) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const Schedule sc = make_schedule(p, base4);
    const int64_t n = (int64_t)1 << p->log_n;
    if (p->batch > 0 && p->nstacks > 0) {
        if (!input && p->input_size > 0) return fail(BF_ERR_INVALID, "input is NULL");
        if (!output && p->output_size > 0) return fail(BF_ERR_INVALID, "output is NULL");
        if (sc.per * sc.nblocks > 0) {
            if (!base4 && !tw2) return fail(BF_ERR_INVALID, "twiddle is NULL");
            if (base4 && p->log_n >= 2 && !tw4) return fail(BF_ERR_INVALID, "twiddle4 is NULL");
            if (base4 && (p->log_n & 1) && !tw2) return fail(BF_ERR_INVALID, "twiddle2 is NULL");
        }
    }
    const View in_view = make_view(p->input_stride, std::min(p->input_size, n), in_perm);
    const View out_view = make_view(p->output_stride, p->output_size, out_index);
    if (fast4_ok(p, base4, false)) {
        const size_t need = forward_workspace(p, base4);
        if (need > 0 && (!workspace || workspace_bytes < need))
            return fail(BF_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
        rc = fast4_forward(p, tw4, tw2, input, output, workspace, in_view, out_view, 0, (int)p->nblocks, stream);
        if (rc || !bias) return rc;
        return p->dtype == BF_C64 ? launch_bias_add<float2>(p, bias, output, out_view, stream)
                                  : launch_bias_add<float>(p, bias, output, out_view, stream);
    }
    const Plan4Long lp = plan4_long(p, base4);
    if (lp.ok) {
        const size_t need = forward_workspace(p, base4);
        if (need > 0 && (!workspace || workspace_bytes < need))
            return fail(BF_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
        rc = long4_forward(p, sc, lp, tw2, tw4, input, output, workspace, in_view, out_view, 0, lp.npass, stream);
        if (rc || !bias) return rc;
        return p->dtype == BF_C64 ? launch_bias_add<float2>(p, bias, output, out_view, stream)
                                  : launch_bias_add<float>(p, bias, output, out_view, stream);
    }
    const PassPlan mp = build_passes(p, base4, true, in_perm || out_index);
    if (mp.ok && passes_addressable(p, mp, false)) {
        const size_t need = forward_workspace(p, base4);
        if (need > 0 && (!workspace || workspace_bytes < need))
            return fail(BF_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
        if ((reinterpret_cast<uintptr_t>(workspace) & 15) != 0)
            return fail(BF_ERR_WORKSPACE, "workspace must be 16-byte aligned");
        if ((reinterpret_cast<uintptr_t>(tw2) & 15) != 0)
            return fail(BF_ERR_INVALID, "twiddle must be 16-byte aligned");
        bool bias_done = false;
        rc = multipass_forward(p, mp, tw2, input, output, workspace, in_view, out_view, 0, mp.npass, stream, bias,
                               &bias_done);
        if (rc || !bias || bias_done) return rc;
        return p->dtype == BF_C64 ? launch_bias_add<float2>(p, bias, output, out_view, stream)
                                  : launch_bias_add<float>(p, bias, output, out_view, stream);
    }
    rc = launch_generic_fw(p, sc, 0, sc.per * sc.nblocks, tw2, tw4, input, in_view, output, out_view, stream);
    if (rc || !bias) return rc;
    return p->dtype == BF_C64 ? launch_bias_add<float2>(p, bias, output, out_view, stream)
                              : launch_bias_add<float>(p, bias, output, out_view, stream);
}

// ---- bias gradient ------------------------------------------------------------------------------

struct BiasGradPlan {
    int64_t cols, nparts, rows_per_part;
    size_t bytes;
};

BiasGradPlan plan_bias_grad(const bf_problem *p)
{
    BiasGradPlan b = {};
    if (p->batch <= 0 || p->nstacks <= 0 || p->output_size <= 0) return b;
    b.cols = (p->output_size + kBiasThreads - 1) / kBiasThreads;
    const int64_t want = std::max<int64_t>(1, (int64_t)num_cu() * 8 / (b.cols * p->nstacks));
    b.nparts = std::min<int64_t>(std::min<int64_t>(want, p->batch), 65535);
    b.rows_per_part = (p->batch + b.nparts - 1) / b.nparts;
    b.nparts = (p->batch + b.rows_per_part - 1) / b.rows_per_part;
    b.bytes = align256((size_t)b.nparts * p->nstacks * p->output_size * elem_bytes(p->dtype));
    return b;
}

template <typename T>
int launch_bias_grad(const bf_problem *p, const BiasGradPlan &b, const void *grad, void *d_bias, void *workspace,
                     hipStream_t stream, const int *out_index)
{
    BiasArgs a = {};
    a.grad = grad;
    a.view = make_view(p->output_stride, p->output_size, out_index);
    a.partial = workspace;
    a.d_bias = d_bias;
    a.batch = p->batch;
    a.width = p->output_size;
    a.rows_per_part = b.rows_per_part;
    a.nparts = b.nparts;
    const dim3 grid1((unsigned)b.cols, (unsigned)p->nstacks, (unsigned)b.nparts);
    hipLaunchKernelGGL((bias_grad_partial_kernel<T>), grid1, dim3(kBiasThreads), 0, stream, a);
    BF_HIP_CHECK(hipGetLastError());
    const dim3 grid2((unsigned)b.cols, (unsigned)p->nstacks, 1);
    hipLaunchKernelGGL((bias_grad_final_kernel<T>), grid2, dim3(kBiasThreads), 0, stream, a);
    BF_HIP_CHECK(hipGetLastError());
    return BF_OK;
}

// ---- generic backward -----------------------------------------------------------------------

struct BwPlan {
    int nstages;
    int chunk;          // stages per launch
    int nchunks;
    int64_t nparts;     // persistent workgroups per stack
    int64_t slot;       // scalars per stage in the partial buffer
    size_t boundary_bytes;  // one (B, S, n) activation plane
    size_t off_boundaries, off_gbuf, off_partials, total;
    bool fits;
    bool fast;          // register-resident pass plan
    bool fast4;         // base-4 register-resident kernels, one launch per block
    bool long4;         // base-4 rows longer than that: chunk and stage passes
};

// saved_boundaries: the activations entering every pass after the first come from the caller
// (left behind by the forward call that saves them) instead of being recomputed into the workspace.
BwPlan plan_bw(const bf_problem *p, bool base4, bool saved_boundaries = false, bool permuted = false)
{
    BwPlan pl = {};
    const int64_t n = (int64_t)1 << p->log_n;
    const size_t e = elem_bytes(p->dtype);
    const size_t row_bytes = (size_t)n * e;
    const Schedule sc = make_schedule(p, base4);
    pl.nstages = sc.per * sc.nblocks;
    if (p->batch == 0 || p->nstacks == 0) {
        // no rows: nothing is launched but the zero fill of d_twiddle, no workspace, any row length
        pl.fits = true;
        return pl;
    }
    if (fast4_ok(p, base4, true)) {
        pl.fits = true;
        pl.fast4 = true;
        pl.nchunks = (int)p->nblocks;
        pl.slot = 4 * n;
        pl.boundary_bytes = align256((size_t)p->batch * p->nstacks * row_bytes);
        pl.nparts = fast_grid(p->batch, (int)p->log_n, p->nstacks, 1, 1).nwg;
        size_t off = 0;
        pl.off_boundaries = off;
        off += p->nblocks > 1 && !saved_boundaries ? (size_t)(p->nblocks - 1) * pl.boundary_bytes : 0;
        pl.off_gbuf = off;
        off += p->nblocks > 1 ? pl.boundary_bytes : 0;
        pl.off_partials = off;
        off += align256((size_t)pl.nparts * p->nstacks * sc.per * pl.slot * e);
        pl.total = off;
        return pl;
    }
    const Plan4Long lp = plan4_long(p, base4);
    if (lp.ok) {
        pl.fits = true;
        pl.long4 = true;
        pl.nchunks = lp.npass;
        pl.slot = 4 * n;
        pl.boundary_bytes = align256((size_t)p->batch * p->nstacks * row_bytes);
        int64_t slices = 1;
        for (int k = 0; k < lp.npass; ++k) slices = std::max(slices, pass4_slices(p, lp.pass[k]));
        size_t off = 0;
        pl.off_boundaries = off;
        off += lp.npass > 1 && !saved_boundaries ? (size_t)(lp.npass - 1) * pl.boundary_bytes : 0;
        pl.off_gbuf = off;
        off += lp.npass > 1 ? pl.boundary_bytes : 0;
        pl.off_partials = off;
        off += align256((size_t)slices * p->nstacks * pl.slot * e);
        pl.total = off;
        return pl;
    }
    const PassPlan mp = build_passes(p, base4, false, permuted);
    if (mp.ok && passes_addressable(p, mp, true)) {
        // boundaries: the activation entering every pass after the first; one gradient plane
        // that the passes update in place; partial slices sized for the widest pass.
        pl.fits = true;
        pl.fast = true;
        pl.nchunks = mp.npass;
        pl.slot = 2 * n;
        pl.boundary_bytes = align256((size_t)p->batch * p->nstacks * row_bytes);
        int64_t nparts = 1, slices = 1;  // slices: partial (stage, 2n) slices of the pass that needs most
        for (int k = 0; k < mp.npass; ++k) {
            const Pass &q = mp.pass[k];
            const int64_t np = fast_grid(p->batch, q.L, p->nstacks * pass_lanes(p, q), 1, 1, row_cap(p, true), true).nwg;
            nparts = std::max(nparts, np);
            slices = std::max(slices, np * (q.t1 - q.t0));
        }
        pl.nparts = nparts;
        size_t off = 0;
        pl.off_boundaries = off;
        off += mp.npass > 1 && !saved_boundaries ? (size_t)(mp.npass - 1) * pl.boundary_bytes : 0;
        pl.off_gbuf = off;
        off += mp.npass > 1 ? pl.boundary_bytes : 0;
        pl.off_partials = off;
        off += align256((size_t)slices * p->nstacks * pl.slot * e);
        pl.total = off;
        return pl;
    }
    pl.fits = 2 * row_bytes <= kGenericBwLds;
    if (!pl.fits) return pl;
    const int cmax = (int)(kGenericBwLds / row_bytes) - 1;
    pl.nchunks = pl.nstages == 0 ? 0 : (pl.nstages + cmax - 1) / cmax;
    pl.chunk = pl.nchunks == 0 ? 0 : (pl.nstages + pl.nchunks - 1) / pl.nchunks;
    pl.nparts = std::min<int64_t>(p->batch, std::max<int64_t>(1, 512 / std::max<int64_t>(1, p->nstacks)));
    pl.slot = base4 ? 4 * n : 2 * n;
    pl.boundary_bytes = align256((size_t)p->batch * p->nstacks * row_bytes);
    size_t off = 0;
    pl.off_boundaries = off;
    off += pl.nchunks > 1 ? (size_t)(pl.nchunks - 1) * pl.boundary_bytes : 0;
    pl.off_gbuf = off;
    off += pl.nchunks > 1 ? pl.boundary_bytes : 0;
    pl.off_partials = off;
    off += align256((size_t)pl.nparts * p->nstacks * pl.chunk * pl.slot * e);
    pl.total = off;
    return pl;
}

template <typename T>
__global__ __launch_bounds__(256) void copy_pad_kernel(const T *in, View iv, T *out, View ov, int64_t batch)
{
    const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int s = blockIdx.y;
    if (j >= ov.width) return;
    for (int64_t b = blockIdx.z; b < batch; b += gridDim.z) {
        T v = zero_of(T());
        if (j < iv.width) v = in[b * iv.sb + s * iv.ss + j * iv.se];
        out[b * ov.sb + s * ov.ss + j * ov.se] = v;
    }
}

int launch_copy_pad(const bf_problem *p, const void *in, const View &iv, void *out, const View &ov,
                    hipStream_t stream)
{
    if (p->batch == 0 || p->nstacks == 0 || ov.width == 0) return BF_OK;
    const dim3 grid((unsigned)((ov.width + 255) / 256), (unsigned)p->nstacks,
                    (unsigned)std::min<int64_t>(p->batch, 1024));
    if (p->dtype == BF_F32)
        hipLaunchKernelGGL(copy_pad_kernel<float>, grid, dim3(256), 0, stream, (const float *)in, iv,
                           (float *)out, ov, p->batch);
    else
        hipLaunchKernelGGL(copy_pad_kernel<float2>, grid, dim3(256), 0, stream, (const float2 *)in, iv,
                           (float2 *)out, ov, p->batch);
    BF_HIP_CHECK(hipGetLastError());
    return BF_OK;
}

int launch_reduce(const bf_problem *p, const Schedule &sc, int t0, int t1, int64_t nparts, const void *partial,
                  int64_t slot, void *d_tw2, void *d_tw4, hipStream_t stream)
{
    if (p->nstacks == 0 || t1 <= t0) return BF_OK;
    if (((reinterpret_cast<uintptr_t>(d_tw2) | reinterpret_cast<uintptr_t>(d_tw4)) & 15) != 0)
        return fail(BF_ERR_INVALID, "d_twiddle pointers must be 16-byte aligned");
    ReduceArgs r;
    r.sc = sc;
    r.t0 = t0;
    r.t1 = t1;
    r.nparts = (int)nparts;
    r.elem_floats = p->dtype == BF_C64 ? 2 : 1;
    r.nstacks = p->nstacks;
    r.partial = static_cast<const float *>(partial);
    r.slot = slot;
    r.d_tw2 = static_cast<float *>(d_tw2);
    r.d_tw4 = static_cast<float *>(d_tw4);
    const dim3 grid((unsigned)((slot * r.elem_floats + 63) / 64), (unsigned)(t1 - t0), (unsigned)p->nstacks);
    hipLaunchKernelGGL(reduce_partials_kernel, grid, dim3(256), 0, stream, r);
    BF_HIP_CHECK(hipGetLastError());
    return BF_OK;
}

// bias_partial / bias_nparts: when given, and when the pass that reads `grad` runs in a kernel
// that can do it, that kernel also leaves the per-workgroup column sums of grad there
// (*bias_nparts slices of (S, output_size)); *bias_nparts stays 0 otherwise.
int backward(const bf_problem *p, bool base4, const void *tw2, const void *tw4, const void *input,
             const void *grad, void *d_tw2, void *d_tw4, void *d_input, void *workspace,
             size_t workspace_bytes, void *stream_, void *bias_partial = nullptr, int64_t *bias_nparts = nullptr,
             const int *in_perm = nullptr, const int *out_index = nullptr, const void *saved = nullptr)
{
    if (bias_nparts) *bias_nparts = 0;
    int rc = check_problem(p, true);
    if (rc) return rc;
    if ((rc = check_perms(p, base4, in_perm, out_index))) return rc;
    if ((rc = ensure_attributes())) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const Schedule sc = make_schedule(p, base4);
    const int64_t n = (int64_t)1 << p->log_n;
    const bool permuted = in_perm || out_index;
    if (p->batch == 0 || p->nstacks == 0) {
        // no rows: d_input is empty and every d_twiddle entry is an empty sum, whatever the row length
        return launch_reduce(p, sc, 0, sc.per * sc.nblocks, 0, nullptr, 4 * n, d_tw2, d_tw4, stream);
    }
    const BwPlan pl = plan_bw(p, base4, saved != nullptr, permuted);
    if (!pl.fits)
        return fail(BF_ERR_UNSUPPORTED, "n = %lld does not fit in LDS for the backward pass", (long long)n);
    if (saved && !(pl.fast || pl.fast4 || pl.long4)) return fail(BF_ERR_INVALID, "this problem has no saved activations");
    const char *saved_planes = static_cast<const char *>(saved);
    if (pl.total > 0 && (!workspace || workspace_bytes < pl.total))
        return fail(BF_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", pl.total, workspace_bytes);
    if ((reinterpret_cast<uintptr_t>(workspace) & 15) != 0)
        return fail(BF_ERR_WORKSPACE, "workspace must be 16-byte aligned");
    if (!base4 && ((reinterpret_cast<uintptr_t>(tw2) | reinterpret_cast<uintptr_t>(d_tw2)) & 15) != 0)
        return fail(BF_ERR_INVALID, "twiddle and d_twiddle must be 16-byte aligned");

    const View x_view = make_view(p->input_stride, std::min(p->input_size, n), in_perm);
    const View g_view = make_view(p->output_stride, std::min(p->output_size, n), out_index);
    const View di_view = make_view(p->d_input_stride, p->input_size, in_perm);
    const View dense = dense_view(p->nstacks, n);
    char *ws = static_cast<char *>(workspace);
    const size_t e_bytes = elem_bytes(p->dtype);

    if (pl.nstages == 0) return launch_copy_pad(p, grad, g_view, d_input, di_view, stream);

    if (pl.fast4) {
        const int L = (int)p->log_n;
        const int P = (int)p->nblocks;
        const int per = sc.per;
        const bool general = fast4_general(p);
        // boundary k = activation entering block k (k >= 1): recomputed here, or kept by the forward
        auto boundary = [&](int k) -> const char * {
            return saved ? saved_planes + (size_t)(k - 1) * pl.boundary_bytes
                         : ws + pl.off_boundaries + (size_t)(k - 1) * pl.boundary_bytes;
        };
        for (int k = 0; k + 1 < P && !saved; ++k) {
            rc = fast4_forward(p, tw4, tw2, k == 0 ? input : boundary(k), const_cast<char *>(boundary(k + 1)), nullptr,
                               k == 0 ? x_view : dense, dense, k, k + 1, stream);
            if (rc) return rc;
        }
        const View dn_view = make_view(p->d_input_stride, std::min(p->input_size, n), in_perm);
        const FastGrid g = fast_grid(p->batch, L, p->nstacks, 1, 1);
        for (int k = P - 1; k >= 0 && general; --k) {
            Fast4GArgs a = fast4g_block_args(p, tw4, tw2, k);
            a.x_in = k == 0 ? input : boundary(k);
            a.x_view = k == 0 ? x_view : dense;
            a.g_out = k == P - 1 ? grad : ws + pl.off_gbuf;
            a.g_view = k == P - 1 ? g_view : dense;
            a.g_in = k == 0 ? d_input : ws + pl.off_gbuf;
            a.gi_view = k == 0 ? dn_view : dense;
            a.partial = ws + pl.off_partials;
            a.ngroups = g.ngroups;
            a.groups_per_wg = g.groups_per_wg;
            const bool inc = (p->increasing_stride != 0) != ((k & 1) != 0);
            rc = launch_fast4g(p->dtype == BF_C64, L, inc, true, a, dim3((unsigned)g.nwg, (unsigned)p->nstacks), stream);
            if (rc) return rc;
            rc = launch_reduce(p, sc, k * per, (k + 1) * per, g.nwg, ws + pl.off_partials, pl.slot, d_tw2, d_tw4,
                               stream);
            if (rc) return rc;
        }
        if (!general && (reinterpret_cast<uintptr_t>(tw4) & 15) != 0)
            return fail(BF_ERR_INVALID, "twiddle4 must be 16-byte aligned");
        for (int k = P - 1; k >= 0 && !general; --k) {
            Fast4Args a = {};
            a.tw4 = static_cast<const float *>(tw4) + (int64_t)k * per * (n / 4) * 16;
            a.tw_stack_stride = sc.tw4_stack_stride;
            a.x_in = static_cast<const float *>(k == 0 ? input : boundary(k));
            a.x_view = k == 0 ? x_view : dense;
            a.g_out = static_cast<const float *>(k == P - 1 ? grad : ws + pl.off_gbuf);
            a.g_view = k == P - 1 ? g_view : dense;
            a.g_in = static_cast<float *>(k == 0 ? d_input : ws + pl.off_gbuf);
            a.gi_view = k == 0 ? dn_view : dense;
            a.partial = reinterpret_cast<float *>(ws + pl.off_partials);
            a.batch = p->batch;
            a.ngroups = g.ngroups;
            a.groups_per_wg = g.groups_per_wg;
            const bool inc = (p->increasing_stride != 0) != ((k & 1) != 0);
            rc = launch_fast4(L, inc, true, a, dim3((unsigned)g.nwg, (unsigned)p->nstacks), stream);
            if (rc) return rc;
            rc = launch_reduce(p, sc, k * per, (k + 1) * per, g.nwg, ws + pl.off_partials, pl.slot, d_tw2, d_tw4,
                               stream);
            if (rc) return rc;
        }
        if (p->input_size > n) {
            View tail = di_view;
            tail.width = p->input_size - n;
            View none = tail;
            none.width = 0;
            char *base = static_cast<char *>(d_input) + (size_t)n * p->d_input_stride[2] * e_bytes;
            rc = launch_copy_pad(p, base, none, base, tail, stream);
            if (rc) return rc;
        }
        return BF_OK;
    }

    if (pl.long4) {
        const Plan4Long lp = plan4_long(p, base4);
        const int P = lp.npass;
        auto boundary = [&](int k) -> const char * {
            return saved ? saved_planes + (size_t)(k - 1) * pl.boundary_bytes
                         : ws + pl.off_boundaries + (size_t)(k - 1) * pl.boundary_bytes;
        };
        // forward replay: boundary k = activation entering pass k (k >= 1), unless the forward kept them
        for (int k = 0; k + 1 < P && !saved; ++k) {
            rc = long4_forward(p, sc, lp, tw2, tw4, k == 0 ? input : boundary(k), const_cast<char *>(boundary(k + 1)),
                               nullptr, k == 0 ? x_view : dense, dense, k, k + 1, stream);
            if (rc) return rc;
        }
        const View dn_view = make_view(p->d_input_stride, std::min(p->input_size, n), in_perm);
        for (int k = P - 1; k >= 0; --k) {
            const Pass4 &q = lp.pass[k];
            int64_t nparts = 0;
            rc = run_pass4(p, sc, q, true, tw2, tw4, k == 0 ? input : boundary(k), k == 0 ? x_view : dense, nullptr,
                           dense, k == P - 1 ? grad : ws + pl.off_gbuf, k == P - 1 ? g_view : dense,
                           k == 0 ? d_input : ws + pl.off_gbuf, k == 0 ? dn_view : dense, ws + pl.off_partials, &nparts,
                           stream);
            if (rc) return rc;
            rc = launch_reduce(p, sc, q.t0, q.t1, nparts, ws + pl.off_partials, pl.slot, d_tw2, d_tw4, stream);
            if (rc) return rc;
        }
        if (p->input_size > n) {
            View tail = di_view;
            tail.width = p->input_size - n;
            View none = tail;
            none.width = 0;
            char *base = static_cast<char *>(d_input) + (size_t)n * p->d_input_stride[2] * e_bytes;
            rc = launch_copy_pad(p, base, none, base, tail, stream);
            if (rc) return rc;
        }
        return BF_OK;
    }

    if (pl.fast) {
        const PassPlan mp = build_passes(p, base4, false, permuted);
        const int P = mp.npass;
        char *bounds = saved ? const_cast<char *>(static_cast<const char *>(saved)) : ws + pl.off_boundaries;
        auto boundary = [&](int k) { return bounds + (size_t)(k - 1) * pl.boundary_bytes; };
        // forward replay: boundary k = activation entering pass k (k >= 1)
        for (int k = 0; k + 1 < P && !saved; ++k) {
            rc = multipass_forward(p, mp, tw2, k == 0 ? input : boundary(k), boundary(k + 1), nullptr,
                                   k == 0 ? x_view : dense, dense, k, k + 1, stream);
            if (rc) return rc;
        }
        const View dn_view = make_view(p->d_input_stride, std::min(p->input_size, n), in_perm);
        for (int k = P - 1; k >= 0; --k) {
            const Pass &q = mp.pass[k];
            const void *xin = k == 0 ? input : boundary(k);
            const View xv = k == 0 ? x_view : dense;
            const void *gout = k == P - 1 ? grad : ws + pl.off_gbuf;
            const View gv = k == P - 1 ? g_view : dense;
            void *gin = k == 0 ? d_input : ws + pl.off_gbuf;
            const View giv = k == 0 ? dn_view : dense;
            int64_t nparts = 0;
            {
                const FastGrid g = fast_grid(p->batch, q.L, p->nstacks * pass_lanes(p, q), 1, 1, row_cap(p, true), true);
                FastBwArgs a = {};
                a.tw = tw2;
                a.tw_stack_stride = sc.tw2_stack_stride;
                a.tw_stage_stride = (n / 2) * 4;
                fill_stage_table(a.tw_stage, kFastMaxStages, q);
                a.partial_slot = pl.slot;
                a.x_in = xin;
                a.x_view = xv;
                a.g_out = gout;
                a.g_view = gv;
                a.g_in = gin;
                a.gi_view = giv;
                a.partial = ws + pl.off_partials;
                a.batch = p->batch;
                a.ngroups = g.ngroups;
                a.groups_per_wg = g.groups_per_wg;
                nparts = g.nwg;
                if (k == P - 1 && bias_partial && bias_nparts && q.L == 10 && p->dtype == BF_F32 && g.nwg <= num_cu()) {
                    a.bias_partial = bias_partial;
                    a.bias_width = p->output_size;
                    *bias_nparts = g.nwg;
                }
                const dim3 grid((unsigned)g.nwg, (unsigned)p->nstacks, (unsigned)pass_lanes(p, q));
                // two row groups in flight once a workgroup has enough of them to fill the pipeline
                if (q.span) {
                    a.low_bits = q.lb;
                    rc = launch_span(p->dtype == BF_C64, q, true, g.groups_per_wg >= 16, nullptr, &a, grid, stream);
                    if (rc) return rc;
                } else {
                    BF_FAST_DISPATCH(launch_fast_bw_t, q, p->dtype == BF_C64, g.groups_per_wg >= 16, a, grid, stream);
                }
                BF_HIP_CHECK(hipGetLastError());
            }
            rc = launch_reduce(p, sc, q.t0, q.t1, nparts, ws + pl.off_partials, pl.slot, d_tw2, d_tw4, stream);
            if (rc) return rc;
        }
        if (p->input_size > n) {
            // input wider than n: those columns get a zero gradient
            View tail = di_view;
            tail.width = p->input_size - n;
            View none = tail;
            none.width = 0;
            char *base = static_cast<char *>(d_input) + (size_t)n * p->d_input_stride[2] * e_bytes;
            rc = launch_copy_pad(p, base, none, base, tail, stream);
            if (rc) return rc;
        }
        return BF_OK;
    }

    const bool have_rows = p->batch > 0 && p->nstacks > 0;
    // forward launches that materialise the input of every chunk after the first
    for (int c = 1; c < pl.nchunks && have_rows; ++c) {
        const void *src = c == 1 ? input : ws + pl.off_boundaries + (size_t)(c - 2) * pl.boundary_bytes;
        void *dst = ws + pl.off_boundaries + (size_t)(c - 1) * pl.boundary_bytes;
        rc = launch_generic_fw(p, sc, (c - 1) * pl.chunk, c * pl.chunk, tw2, tw4, src,
                               c == 1 ? x_view : dense, dst, dense, stream);
        if (rc) return rc;
    }
    const size_t e = elem_bytes(p->dtype);
    for (int c = pl.nchunks - 1; c >= 0; --c) {
        const int t0 = c * pl.chunk;
        const int t1 = std::min(pl.nstages, t0 + pl.chunk);
        if (have_rows) {
            GenericBwArgs a;
            a.sc = sc;
            a.t0 = t0;
            a.t1 = t1;
            a.batch = p->batch;
            a.tw2 = tw2;
            a.tw4 = tw4;
            a.x_in = c == 0 ? input : ws + pl.off_boundaries + (size_t)(c - 1) * pl.boundary_bytes;
            a.x_view = c == 0 ? x_view : dense;
            a.g_out = c == pl.nchunks - 1 ? grad : ws + pl.off_gbuf;
            a.g_view = c == pl.nchunks - 1 ? g_view : dense;
            a.g_in = c == 0 ? d_input : ws + pl.off_gbuf;
            a.gi_view = c == 0 ? di_view : dense;
            a.partial = ws + pl.off_partials;
            a.slot = pl.slot;
            const dim3 grid((unsigned)pl.nparts, (unsigned)p->nstacks);
            const size_t lds = (size_t)(t1 - t0 + 1) * n * e;
            if (p->dtype == BF_F32)
                hipLaunchKernelGGL(generic_bw_kernel<float>, grid, dim3(kGenericThreads), lds, stream, a);
            else
                hipLaunchKernelGGL(generic_bw_kernel<float2>, grid, dim3(kGenericThreads), lds, stream, a);
            BF_HIP_CHECK(hipGetLastError());
        }
        rc = launch_reduce(p, sc, t0, t1, have_rows ? pl.nparts : 0, ws + pl.off_partials, pl.slot, d_tw2, d_tw4,
                           stream);
        if (rc) return rc;
    }
    return BF_OK;
}

// ---- built-in scratch for callers that cannot allocate ----------------------------------------
//
// One fixed array per GPU, held from the moment the library's code is loaded on that GPU until the
// process ends.  In host code `scratch` is only a handle for the symbol: the memory is reached
// through the address hipGetSymbolAddress returns for the device that is current, looked up once
// per device and kept.  Each GPU has its own copy at its own address.
constexpr size_t kScratchBytes = (size_t)48 << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];

int scratch_of_current_device(void **ptr)
{
    int device = -1;
    BF_HIP_CHECK(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices)
        return fail(BF_ERR_UNSUPPORTED, "device ordinal %d is outside the %d the library keeps scratch addresses for",
                    device, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void *address = nullptr;
        BF_HIP_CHECK(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)));
        if (!address) return fail(BF_ERR_HIP, "hipGetSymbolAddress returned no address for the built-in scratch");
        g_scratch_ptr[device] = address;
    }
    *ptr = g_scratch_ptr[device];
    return BF_OK;
}

// Workspace of a base-2 backward call whatever its column tables: the plan may differ with them.
size_t bw_workspace_total(const bf_problem *p, bool saved_boundaries)
{
    return std::max(plan_bw(p, false, saved_boundaries, false).total, plan_bw(p, false, saved_boundaries, true).total);
}

}  // namespace

extern "C" {

int bf_butterfly_multiply_bw_noalloc(const bf_problem *p, const void *twiddle, const void *input, const void *grad,
                                     void *d_twiddle, void *d_input, void *stream)
{
    int rc = check_problem(p, true);
    if (rc) return rc;
    const BwPlan pl = plan_bw(p, false);
    if (!pl.fits)
        return fail(BF_ERR_UNSUPPORTED, "n = %lld does not fit in LDS for the backward pass",
                    (long long)((int64_t)1 << p->log_n));
    if (pl.total > kScratchBytes)
        return fail(BF_ERR_WORKSPACE,
                    "this problem needs %zu bytes of scratch, the built-in area holds %zu: use "
                    "bf_butterfly_multiply_bw with a workspace of the caller's",
                    pl.total, kScratchBytes);
    void *area = nullptr;
    if ((rc = scratch_of_current_device(&area))) return rc;
    // every partial slice and boundary activation in the area is written by this call's own
    // launches before anything reads it, so nothing of an earlier call has to be cleared
    return backward(p, false, twiddle, nullptr, input, grad, d_twiddle, nullptr, d_input, area, kScratchBytes, stream);
}

int bf_version(void) { return 100; }

int bf_hip_version(void) { return HIP_VERSION; }

const char *bf_last_error(void) { return g_last_error.c_str(); }

size_t bf_butterfly_multiply_fw_workspace_bytes(const bf_problem *p)
{
    if (check_problem(p, false)) return BF_SIZE_INVALID;
    return forward_workspace(p, false);
}

int bf_butterfly_multiply_fw(const bf_problem *p, const void *twiddle, const void *input,
                             void *output, void *workspace, size_t workspace_bytes, void *stream)
{
    return forward(p, false, twiddle, nullptr, input, output, workspace, workspace_bytes, stream);
}

size_t bf_butterfly_multiply_bw_workspace_bytes(const bf_problem *p)
{
    if (check_problem(p, true)) return BF_SIZE_INVALID;
    return bw_workspace_total(p, false);
}

int bf_butterfly_multiply_bw(const bf_problem *p, const void *twiddle, const void *input,
                             const void *grad, void *d_twiddle, void *d_input, void *workspace,
                             size_t workspace_bytes, void *stream)
{
    return backward(p, false, twiddle, nullptr, input, grad, d_twiddle, nullptr, d_input, workspace,
                    workspace_bytes, stream);
}

size_t bf_butterfly_multiply_base4_fw_workspace_bytes(const bf_problem *p)
{
    if (check_problem(p, false)) return BF_SIZE_INVALID;
    return forward_workspace(p, true);
}

int bf_butterfly_multiply_bias_fw(const bf_problem *p, const void *twiddle, const void *input, const void *bias,
                                  void *output, void *workspace, size_t workspace_bytes, void *stream)
{
    return forward(p, false, twiddle, nullptr, input, output, workspace, workspace_bytes, stream, bias);
}

size_t bf_butterfly_bias_grad_workspace_bytes(const bf_problem *p)
{
    if (check_problem(p, false)) return BF_SIZE_INVALID;
    return plan_bias_grad(p).bytes;
}

// d_bias[s][c] = sum over the batch of grad[b][s][out_index[c]] (out_index NULL: column c)
static int bias_grad(const bf_problem *p, const void *grad, void *d_bias, void *workspace, size_t workspace_bytes,
                     void *stream, const int *out_index)
{
    int rc = check_problem(p, false);
    if (rc) return rc;
    if (p->nstacks <= 0 || p->output_size <= 0) return BF_OK;
    if (!d_bias) return fail(BF_ERR_INVALID, "d_bias is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (p->batch <= 0) {
        // an empty batch sums to zero: the final kernel over zero partitions writes exactly that
        BiasArgs a = {};
        a.d_bias = d_bias;
        a.width = p->output_size;
        const dim3 grid((unsigned)((p->output_size + kBiasThreads - 1) / kBiasThreads), (unsigned)p->nstacks, 1);
        if (p->dtype == BF_C64) hipLaunchKernelGGL((bias_grad_final_kernel<float2>), grid, dim3(kBiasThreads), 0, s, a);
        else hipLaunchKernelGGL((bias_grad_final_kernel<float>), grid, dim3(kBiasThreads), 0, s, a);
        BF_HIP_CHECK(hipGetLastError());
        return BF_OK;
    }
    if (!grad) return fail(BF_ERR_INVALID, "grad is NULL");
    const BiasGradPlan b = plan_bias_grad(p);
    if (!workspace || workspace_bytes < b.bytes)
        return fail(BF_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", b.bytes, workspace_bytes);
    return p->dtype == BF_C64 ? launch_bias_grad<float2>(p, b, grad, d_bias, workspace, s, out_index)
                              : launch_bias_grad<float>(p, b, grad, d_bias, workspace, s, out_index);
}

int bf_butterfly_bias_grad(const bf_problem *p, const void *grad, void *d_bias, void *workspace,
                           size_t workspace_bytes, void *stream)
{
    return bias_grad(p, grad, d_bias, workspace, workspace_bytes, stream, nullptr);
}

// Bias area behind the backward workspace: room for either the per-workgroup column sums the
// backward kernel leaves (at most one slice per compute unit) or the partitions of the
// stand-alone column sum.
static size_t bias_area_bytes(const bf_problem *p)
{
    const size_t fused = align256((size_t)num_cu() * std::max<int64_t>(p->nstacks, 1) *
                                  std::max<int64_t>(p->output_size, 0) * elem_bytes(p->dtype));
    return std::max(fused, plan_bias_grad(p).bytes);
}

size_t bf_butterfly_multiply_bias_bw_workspace_bytes(const bf_problem *p)
{
    if (check_problem(p, true)) return BF_SIZE_INVALID;
    return align256(bw_workspace_total(p, false)) + bias_area_bytes(p);
}

static int bias_backward(const bf_problem *p, const void *twiddle, const void *input, const void *grad,
                         void *d_twiddle, void *d_input, void *d_bias, void *workspace, size_t workspace_bytes,
                         void *stream, const int *in_perm, const int *out_index, const void *saved = nullptr)
{
    int rc = check_problem(p, true);
    if (rc) return rc;
    const size_t main_bytes = align256(plan_bw(p, false, saved != nullptr, in_perm || out_index).total);
    const size_t need = main_bytes + bias_area_bytes(p);
    if (!workspace || workspace_bytes < need)
        return fail(BF_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    if (!d_bias && p->nstacks > 0 && p->output_size > 0) return fail(BF_ERR_INVALID, "d_bias is NULL");
    char *area = static_cast<char *>(workspace) + main_bytes;
    int64_t nparts = 0;
    rc = backward(p, false, twiddle, nullptr, input, grad, d_twiddle, nullptr, d_input, workspace, main_bytes, stream,
                  area, &nparts, in_perm, out_index, saved);
    if (rc) return rc;
    if (p->nstacks <= 0 || p->output_size <= 0) return BF_OK;
    if (nparts > 0) {
        // the backward kernel left one slice of column sums per workgroup: add them up in order
        BiasArgs a = {};
        a.partial = area;
        a.d_bias = d_bias;
        a.width = p->output_size;
        a.nparts = nparts;
        const dim3 grid((unsigned)((p->output_size + kBiasThreads - 1) / kBiasThreads), (unsigned)p->nstacks, 1);
        hipLaunchKernelGGL((bias_grad_final_kernel<float>), grid, dim3(kBiasThreads), 0,
                           static_cast<hipStream_t>(stream), a);
        BF_HIP_CHECK(hipGetLastError());
        return BF_OK;
    }
    return bias_grad(p, grad, d_bias, area, bias_area_bytes(p), stream, out_index);
}

int bf_butterfly_multiply_bias_bw(const bf_problem *p, const void *twiddle, const void *input, const void *grad,
                                  void *d_twiddle, void *d_input, void *d_bias, void *workspace,
                                  size_t workspace_bytes, void *stream)
{
    return bias_backward(p, twiddle, input, grad, d_twiddle, d_input, d_bias, workspace, workspace_bytes, stream,
                         nullptr, nullptr);
}

int bf_butterfly_multiply_perm_fw(const bf_problem *p, const void *twiddle, const void *input, const int32_t *in_perm,
                                  const int32_t *out_index, const void *bias, void *output, void *workspace,
                                  size_t workspace_bytes, void *stream)
{
    return forward(p, false, twiddle, nullptr, input, output, workspace, workspace_bytes, stream, bias, in_perm,
                   out_index);
}

int bf_butterfly_multiply_perm_bw(const bf_problem *p, const void *twiddle, const void *input, const void *grad,
                                  const int32_t *in_perm, const int32_t *out_index, void *d_twiddle, void *d_input,
                                  void *d_bias, void *workspace, size_t workspace_bytes, void *stream)
{
    if (d_bias)
        return bias_backward(p, twiddle, input, grad, d_twiddle, d_input, d_bias, workspace, workspace_bytes, stream,
                             in_perm, out_index);
    return backward(p, false, twiddle, nullptr, input, grad, d_twiddle, nullptr, d_input, workspace, workspace_bytes,
                    stream, nullptr, nullptr, in_perm, out_index);
}

// Bytes of activations the saving forward leaves for the backward: one dense (B, S, n) plane per
// pass of the backward plan after the first; 0 when the backward is a single pass (or runs on
// kernels that do not use such planes).
static size_t saved_bytes_of_plan(const bf_problem *p, bool permuted)
{
    const BwPlan pl = plan_bw(p, false, true, permuted);
    if (!pl.fits || !pl.fast || pl.nchunks <= 1) return 0;
    return (size_t)(pl.nchunks - 1) * pl.boundary_bytes;
}

// room for the saved activations of a call with or without column tables (the plans may differ)
static size_t saved_bytes(const bf_problem *p)
{
    return std::max(saved_bytes_of_plan(p, false), saved_bytes_of_plan(p, true));
}

size_t bf_butterfly_multiply_saved_bytes(const bf_problem *p)
{
    if (check_problem(p, true)) return BF_SIZE_INVALID;
    return saved_bytes(p);
}

int bf_butterfly_multiply_fw_saving(const bf_problem *p, const void *twiddle, const void *input, const void *bias,
                                    const int32_t *in_perm, const int32_t *out_index, void *output, void *saved,
                                    size_t saved_capacity, void *stream_)
{
    int rc = check_problem(p, false);
    if (rc) return rc;
    if ((rc = check_perms(p, false, in_perm, out_index))) return rc;
    if ((rc = ensure_attributes())) return rc;
    const size_t need = saved_bytes(p);
    if (need == 0) return fail(BF_ERR_INVALID, "this problem has no activations to save: use bf_butterfly_multiply_fw");
    if (!saved || saved_capacity < need)
        return fail(BF_ERR_WORKSPACE, "room for %zu bytes of saved activations needed, %zu given", need, saved_capacity);
    if (!twiddle || !input || !output) return fail(BF_ERR_INVALID, "an operand is NULL");
    if (((reinterpret_cast<uintptr_t>(saved) | reinterpret_cast<uintptr_t>(twiddle)) & 15) != 0)
        return fail(BF_ERR_INVALID, "twiddle and the saved area must be 16-byte aligned");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t n = (int64_t)1 << p->log_n;
    const bool permuted = in_perm || out_index;
    const PassPlan mp = build_passes(p, false, false, permuted);
    const BwPlan pl = plan_bw(p, false, true, permuted);
    if (mp.npass < 2 || !pl.fast) return fail(BF_ERR_INVALID, "this problem has no activations to save");
    const View in_view = make_view(p->input_stride, std::min(p->input_size, n), in_perm);
    const View out_view = make_view(p->output_stride, p->output_size, out_index);
    const View dense = dense_view(p->nstacks, n);
    char *bounds = static_cast<char *>(saved);
    auto boundary = [&](int k) { return bounds + (size_t)(k - 1) * pl.boundary_bytes; };
    const int P = mp.npass;
    // the passes of the backward plan, each into its own plane: plane k = activation entering pass k
    for (int k = 0; k + 1 < P; ++k) {
        rc = multipass_forward(p, mp, twiddle, k == 0 ? input : boundary(k), boundary(k + 1), nullptr,
                               k == 0 ? in_view : dense, dense, k, k + 1, stream);
        if (rc) return rc;
    }
    bool bias_done = false;
    rc = multipass_forward(p, mp, twiddle, boundary(P - 1), output, nullptr, dense, out_view, P - 1, P, stream, bias,
                           &bias_done);
    if (rc || !bias || bias_done) return rc;
    return p->dtype == BF_C64 ? launch_bias_add<float2>(p, bias, output, out_view, stream)
                              : launch_bias_add<float>(p, bias, output, out_view, stream);
}

size_t bf_butterfly_multiply_bw_saved_workspace_bytes(const bf_problem *p, int with_bias)
{
    if (check_problem(p, true)) return BF_SIZE_INVALID;
    const size_t main_bytes = bw_workspace_total(p, true);
    return with_bias ? align256(main_bytes) + bias_area_bytes(p) : main_bytes;
}

int bf_butterfly_multiply_bw_saved(const bf_problem *p, const void *twiddle, const void *input, const void *grad,
                                   const void *saved, size_t saved_bytes_given, const int32_t *in_perm,
                                   const int32_t *out_index, void *d_twiddle, void *d_input, void *d_bias,
                                   void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = check_problem(p, true);
    if (rc) return rc;
    if (!saved || saved_bytes(p) == 0)
        return fail(BF_ERR_INVALID, "this problem has no saved activations: use bf_butterfly_multiply_bw");
    // The planes this call reads follow from its own plan (strides of grad and d_input, column
    // tables): the caller's area must hold them.  A plan of a single pass reads none and runs as
    // the plain call does (its workspace is the same either way).
    const size_t planes = saved_bytes_of_plan(p, in_perm || out_index);
    if (planes == 0) saved = nullptr;
    else if (saved_bytes_given < planes)
        return fail(BF_ERR_WORKSPACE, "the backward reads %zu bytes of saved activations, %zu given", planes,
                    saved_bytes_given);
    if (d_bias)
        return bias_backward(p, twiddle, input, grad, d_twiddle, d_input, d_bias, workspace, workspace_bytes, stream,
                             in_perm, out_index, saved);
    return backward(p, false, twiddle, nullptr, input, grad, d_twiddle, nullptr, d_input, workspace, workspace_bytes,
                    stream, nullptr, nullptr, in_perm, out_index, saved);
}

// One line per launch group of the base-2 schedule, e.g. "low t=0..10 L=10 nb=1 inc=1 chunks=8".
int bf_describe_plan(const bf_problem *p, int backward, char *text, size_t capacity)
{
    int rc = check_problem(p, backward != 0);
    if (rc) return rc;
    if (!text || capacity == 0) return fail(BF_ERR_INVALID, "text buffer is NULL or empty");
    std::string out;
    char line[160];
    const PassPlan mp = build_passes(p, false, backward == 0);
    if (!mp.ok || !passes_addressable(p, mp, backward != 0)) {
        out = "generic\n";
    } else {
        for (int k = 0; k < mp.npass; ++k) {
            const Pass &q = mp.pass[k];
            if (q.wide)
                snprintf(line, sizeof line, "wide t=%d..%d L=%d inc=%d\n", q.t0, q.t1, q.L, (int)q.inc);
            else if (q.span)
                snprintf(line, sizeof line, "span t=%d..%d lb=%d bits=%d mode=%d tiles=%lld\n", q.t0, q.t1, q.lb, q.H,
                         q.mode, (long long)pass_lanes(p, q));
            else
                snprintf(line, sizeof line, "low t=%d..%d L=%d nb=%d inc=%d chunks=%lld\n", q.t0, q.t1, q.L, q.NB,
                         (int)q.inc, (long long)pass_lanes(p, q));
            out += line;
        }
    }
    if (out.size() + 1 > capacity) return fail(BF_ERR_INVALID, "text buffer of %zu bytes is too small", capacity);
    memcpy(text, out.c_str(), out.size() + 1);
    return BF_OK;
}

int bf_butterfly_multiply_base4_fw(const bf_problem *p, const void *twiddle4, const void *twiddle2,
                                   const void *input, void *output, void *workspace, size_t workspace_bytes,
                                   void *stream)
{
    return forward(p, true, twiddle2, twiddle4, input, output, workspace, workspace_bytes, stream);
}

size_t bf_butterfly_multiply_base4_bw_workspace_bytes(const bf_problem *p)
{
    if (check_problem(p, true)) return BF_SIZE_INVALID;
    return plan_bw(p, true).total;
}

int bf_butterfly_multiply_base4_bw(const bf_problem *p, const void *twiddle4, const void *twiddle2,
                                   const void *input, const void *grad, void *d_twiddle4,
                                   void *d_twiddle2, void *d_input, void *workspace,
                                   size_t workspace_bytes, void *stream)
{
    return backward(p, true, twiddle2, twiddle4, input, grad, d_twiddle2, d_twiddle4, d_input,
                    workspace, workspace_bytes, stream);
}

// Base-4 counterpart of the activation-keeping pair: the planes are the activations entering
// every pass of the backward plan after the first (blocks for rows up to 1024, chunk and stage
// passes beyond).
static size_t saved4_bytes(const bf_problem *p)
{
    const BwPlan pl = plan_bw(p, true, true);
    if (!pl.fits || pl.nchunks <= 1) return 0;
    if (!(pl.fast4 && fast4_ok(p, true, false)) && !pl.long4) return 0;
    return (size_t)(pl.nchunks - 1) * pl.boundary_bytes;
}

size_t bf_butterfly_multiply_base4_saved_bytes(const bf_problem *p)
{
    if (check_problem(p, true)) return BF_SIZE_INVALID;
    return saved4_bytes(p);
}

int bf_butterfly_multiply_base4_fw_saving(const bf_problem *p, const void *twiddle4, const void *twiddle2,
                                          const void *input, void *output, void *saved, size_t saved_capacity,
                                          void *stream_)
{
    int rc = check_problem(p, false);
    if (rc) return rc;
    if ((rc = ensure_attributes())) return rc;
    const size_t need = saved4_bytes(p);
    if (need == 0)
        return fail(BF_ERR_INVALID, "this problem has no activations to save: use bf_butterfly_multiply_base4_fw");
    if (!saved || saved_capacity < need)
        return fail(BF_ERR_WORKSPACE, "room for %zu bytes of saved activations needed, %zu given", need, saved_capacity);
    if (!twiddle4 || !input || !output || ((p->log_n & 1) && !twiddle2)) return fail(BF_ERR_INVALID, "an operand is NULL");
    if ((reinterpret_cast<uintptr_t>(saved) & 15) != 0) return fail(BF_ERR_INVALID, "the saved area must be 16-byte aligned");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t n = (int64_t)1 << p->log_n;
    const BwPlan pl = plan_bw(p, true, true);
    const Schedule sc = make_schedule(p, true);
    const View in_view = make_view(p->input_stride, std::min(p->input_size, n), nullptr);
    const View out_view = make_view(p->output_stride, p->output_size, nullptr);
    const View dense = dense_view(p->nstacks, n);
    char *planes = static_cast<char *>(saved);
    auto boundary = [&](int k) { return planes + (size_t)(k - 1) * pl.boundary_bytes; };
    const int P = pl.nchunks;
    const Plan4Long lp = pl.long4 ? plan4_long(p, true) : Plan4Long();
    for (int k = 0; k < P; ++k) {
        const void *in = k == 0 ? input : boundary(k);
        void *out = k == P - 1 ? output : boundary(k + 1);
        const View &iv = k == 0 ? in_view : dense, &ov = k == P - 1 ? out_view : dense;
        rc = pl.long4 ? long4_forward(p, sc, lp, twiddle2, twiddle4, in, out, nullptr, iv, ov, k, k + 1, stream)
                      : fast4_forward(p, twiddle4, twiddle2, in, out, nullptr, iv, ov, k, k + 1, stream);
        if (rc) return rc;
    }
    return BF_OK;
}

size_t bf_butterfly_multiply_base4_bw_saved_workspace_bytes(const bf_problem *p)
{
    if (check_problem(p, true)) return BF_SIZE_INVALID;
    return plan_bw(p, true, true).total;
}

int bf_butterfly_multiply_base4_bw_saved(const bf_problem *p, const void *twiddle4, const void *twiddle2,
                                         const void *input, const void *grad, const void *saved,
                                         size_t saved_bytes_given, void *d_twiddle4, void *d_twiddle2, void *d_input,
                                         void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = check_problem(p, true);
    if (rc) return rc;
    const size_t planes = saved4_bytes(p);
    if (!saved || planes == 0)
        return fail(BF_ERR_INVALID, "this problem has no saved activations: use bf_butterfly_multiply_base4_bw");
    if (saved_bytes_given < planes)
        return fail(BF_ERR_WORKSPACE, "the backward reads %zu bytes of saved activations, %zu given", planes,
                    saved_bytes_given);
    return backward(p, true, twiddle2, twiddle4, input, grad, d_twiddle2, d_twiddle4, d_input, workspace,
                    workspace_bytes, stream, nullptr, nullptr, nullptr, nullptr, saved);
}

static int scale_twiddle(bool bw, int dtype, int64_t nstacks, int64_t nblocks, int64_t log_n, int increasing_stride,
                         const void *twiddle, const void *in_scale, int64_t in_len, const void *out_scale,
                         int64_t out_len, const void *grad, void *out, void *d_in, void *d_out, void *stream)
{
    if (dtype != BF_F32 && dtype != BF_C64) return fail(BF_ERR_INVALID, "dtype must be BF_F32 or BF_C64");
    if (nstacks < 0 || nblocks < 1 || log_n < 1 || log_n > 30)
        return fail(BF_ERR_INVALID, "nstacks >= 0, nblocks >= 1 and log_n in [1, 30] are required");
    const int64_t n = (int64_t)1 << log_n;
    if (nstacks > 65535 || nblocks * log_n > (1 << 20))
        return fail(BF_ERR_UNSUPPORTED, "more than 65535 stacks or 2^20 stages are not supported");
    if (in_scale && (in_len < 0 || in_len > n)) return fail(BF_ERR_INVALID, "in_len must be in [0, n]");
    if (out_scale && (out_len < 0 || out_len > nstacks * n)) return fail(BF_ERR_INVALID, "out_len must be in [0, nstacks * n]");
    if (nstacks == 0) return BF_OK;
    if (!twiddle || !out || (bw && !grad)) return fail(BF_ERR_INVALID, "a factor tensor is NULL");
    if (bw && ((in_scale && in_len > 0 && !d_in) || (out_scale && out_len > 0 && !d_out)))
        return fail(BF_ERR_INVALID, "a diagonal is given without room for its gradient");
    ScaleArgs a{};
    a.tw = twiddle;
    a.in_scale = in_scale;
    a.out_scale = out_scale;
    a.grad = grad;
    a.out = out;
    a.d_in = d_in;
    a.d_out = d_out;
    a.in_len = in_scale ? in_len : 0;
    a.out_len = out_scale ? out_len : 0;
    a.nstacks = (int)nstacks;
    a.nstages = (int)(nblocks * log_n);
    a.log_n = (int)log_n;
    const bool last_increasing = (increasing_stride != 0) != (((nblocks - 1) & 1) != 0);
    a.first_log_stride = increasing_stride ? 0 : (int)log_n - 1;
    a.last_log_stride = last_increasing ? (int)log_n - 1 : 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t entries = nstacks * a.nstages * 2 * n;
    const dim3 grid((unsigned)((entries + kScaleThreads - 1) / kScaleThreads)), block(kScaleThreads);
    if (!bw) {
        if (dtype == BF_F32) hipLaunchKernelGGL((scale_twiddle_kernel<float, false>), grid, block, 0, st, a);
        else hipLaunchKernelGGL((scale_twiddle_kernel<float2, false>), grid, block, 0, st, a);
        BF_HIP_CHECK(hipGetLastError());
        return BF_OK;
    }
    if (dtype == BF_F32) hipLaunchKernelGGL((scale_twiddle_kernel<float, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((scale_twiddle_kernel<float2, true>), grid, block, 0, st, a);
    BF_HIP_CHECK(hipGetLastError());
    const int64_t diag = a.in_len + a.out_len;
    if (diag > 0) {
        const dim3 dgrid((unsigned)((diag + kScaleThreads - 1) / kScaleThreads));
        if (dtype == BF_F32) hipLaunchKernelGGL((scale_twiddle_grad_kernel<float>), dgrid, block, 0, st, a);
        else hipLaunchKernelGGL((scale_twiddle_grad_kernel<float2>), dgrid, block, 0, st, a);
        BF_HIP_CHECK(hipGetLastError());
    }
    return BF_OK;
}

int bf_butterfly_scale_twiddle(int dtype, int64_t nstacks, int64_t nblocks, int64_t log_n, int increasing_stride,
                               const void *twiddle, const void *in_scale, int64_t in_len, const void *out_scale,
                               int64_t out_len, void *scaled, void *stream)
{
    return scale_twiddle(false, dtype, nstacks, nblocks, log_n, increasing_stride, twiddle, in_scale, in_len, out_scale,
                         out_len, nullptr, scaled, nullptr, nullptr, stream);
}

int bf_butterfly_scale_twiddle_bw(int dtype, int64_t nstacks, int64_t nblocks, int64_t log_n, int increasing_stride,
                                  const void *twiddle, const void *in_scale, int64_t in_len, const void *out_scale,
                                  int64_t out_len, const void *grad, void *d_twiddle, void *d_in_scale,
                                  void *d_out_scale, void *stream)
{
    return scale_twiddle(true, dtype, nstacks, nblocks, log_n, increasing_stride, twiddle, in_scale, in_len, out_scale,
                         out_len, grad, d_twiddle, d_in_scale, d_out_scale, stream);
}

}  // extern "C"
