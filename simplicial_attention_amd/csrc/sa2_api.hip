// C ABI of libsa2: argument validation and kernel launches (see include/sa2.h).
#include "sa2.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "sa2_bwd.hpp"
#include "sa2_bwd_kv8.hpp"
#include "sa2_bwd_q.hpp"
#include "sa2_common.hpp"
#include "sa2_lds.hpp"
#include "sa2_qkv_norm.hpp"
#include "sa2_fwd.hpp"
#include "sa2_wide.hpp"
#ifdef SA2_PROFILING
#include "sa2_prof_mix.hpp"
#endif

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_problem(const sa2_problem *p) {
    if (!p) return fail(SA2_ERR_NULL_POINTER, "problem is NULL");
    if (p->batch < 1 || p->seq_len < 1 || p->heads < 1 || p->kv_heads < 1)
        return fail(SA2_ERR_BAD_SHAPE, "batch=%d seq_len=%d heads=%d kv_heads=%d must all be >= 1", p->batch, p->seq_len,
                    p->heads, p->kv_heads);
    if (p->heads % p->kv_heads != 0)
        return fail(SA2_ERR_BAD_SHAPE, "heads=%d is not a multiple of kv_heads=%d", p->heads, p->kv_heads);
    if (p->w1 < 1 || p->w2 < 1) return fail(SA2_ERR_BAD_SHAPE, "windows w1=%d w2=%d must be >= 1", p->w1, p->w2);
    if (p->causal != 1) return fail(SA2_ERR_UNSUPPORTED, "only causal=1 is defined for the sliding windows");
    if (p->dtype != SA2_BF16) return fail(SA2_ERR_UNSUPPORTED, "dtype %d is not supported (bf16 only)", p->dtype);
    if (p->dim_head != 32 && p->dim_head != 64 && p->dim_head != 128 && p->dim_head != 256)
        return fail(SA2_ERR_UNSUPPORTED, "dim_head=%d is not supported (32, 64, 128 or 256)", p->dim_head);
    if (!(p->scale > 0.f) || !std::isfinite(p->scale)) return fail(SA2_ERR_BAD_SHAPE, "scale must be positive and finite");
    if ((int64_t)p->batch * p->heads * ((p->seq_len + 31) / 32) > 0x7fffffffll)
        return fail(SA2_ERR_BAD_SHAPE, "problem too large for a 1-D grid");
    return SA2_OK;
}

int check_tensor(const sa2_tensor *t, const char *name) {
    if (!t || !t->ptr) return fail(SA2_ERR_NULL_POINTER, "tensor %s is NULL", name);
    if ((reinterpret_cast<uintptr_t>(t->ptr) & 15) != 0 || (t->stride_b & 7) != 0 || (t->stride_n & 7) != 0 ||
        (t->stride_h & 7) != 0)
        return fail(SA2_ERR_ALIGNMENT, "tensor %s: base pointer must be 16-byte aligned and strides multiples of 8 elements",
                    name);
    return SA2_OK;
}

sa2::DevTensor dev(const sa2_tensor *t) {
    sa2::DevTensor d;
    d.ptr = static_cast<char *>(t->ptr);
    d.sb = t->stride_b * 2;
    d.sn = t->stride_n * 2;
    d.sh = t->stride_h * 2;
    return d;
}

sa2::KParams base_params(const sa2_problem *p) {
    sa2::KParams k{};
    k.B = p->batch;
    k.N = p->seq_len;
    k.H = p->heads;
    k.HK = p->kv_heads;
    k.G = p->heads / p->kv_heads;
    k.w1 = p->w1;
    k.w2 = p->w2;
    k.scale = p->scale;
    k.scale_log2e = p->scale * sa2::kLog2e;
    return k;
}

int after_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SA2_ERR_LAUNCH, "%s launch failed: %s", what, hipGetErrorString(e));
    return SA2_OK;
}

#define SA2_TRY(expr)                  \
    do {                               \
        int rc_ = (expr);              \
        if (rc_ != SA2_OK) return rc_; \
    } while (0)

// Head dimension 256 runs kernels of its own (sa2_wide.hpp), which keep no forward partials.
constexpr int kWideDimHead = 256;

// Runs the statement with the compile-time constant DH set to the problem's head dimension (validated by
// check_problem): the kernels built for head dimensions 32, 64 and 128 ...
#define SA2_FOR_DIM_HEAD(dim_head, ...)         \
    do {                                        \
        if ((dim_head) == 128) {                \
            constexpr int DH = 128;             \
            __VA_ARGS__;                        \
        } else if ((dim_head) == 64) {          \
            constexpr int DH = 64;              \
            __VA_ARGS__;                        \
        } else {                                \
            constexpr int DH = 32;              \
            __VA_ARGS__;                        \
        }                                       \
    } while (0)

// ... and the kernels that every head dimension shares
#define SA2_FOR_ANY_DIM_HEAD(dim_head, ...)             \
    do {                                                \
        if ((dim_head) == kWideDimHead) {               \
            constexpr int DH = kWideDimHead;            \
            __VA_ARGS__;                                \
        } else {                                        \
            SA2_FOR_DIM_HEAD(dim_head, __VA_ARGS__);    \
        }                                               \
    } while (0)

// Scratch of sa2_bwd_noalloc: delta rows followed by the dK2/dV2 partial rows.  A file-scope device
// array: every GPU the library runs on holds its own copy, at its own address, until the process
// ends.  In host code the array's name is only a handle for hipGetSymbolAddress; kernels and
// runtime calls get the address that call returns for the current device.
constexpr int64_t kNoallocScratchBytes = SA2_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char g_noalloc_scratch[kNoallocScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
unsigned char *g_scratch_ptr[kMaxDevices] = {};

// device address of the scratch array on the current device (looked up once per device)
int noalloc_scratch(unsigned char **out) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return fail(SA2_ERR_LAUNCH, "hipGetDevice failed: %s", hipGetErrorString(e));
    if (device < 0 || device >= kMaxDevices) return fail(SA2_ERR_UNSUPPORTED, "device index %d is not supported (at most %d)", device, kMaxDevices);
    std::lock_guard<std::mutex> guard(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_noalloc_scratch));
        if (e != hipSuccess || !ptr) return fail(SA2_ERR_LAUNCH, "hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
        g_scratch_ptr[device] = static_cast<unsigned char *>(ptr);
    }
    *out = g_scratch_ptr[device];
    return SA2_OK;
}

}  // namespace

extern "C" {

int sa2_version(void) { return SA2_VERSION; }

const char *sa2_last_error(void) { return g_err; }

int sa2_supported(int32_t dim_head, int32_t w1, int32_t w2, int32_t dtype) {
    return (dim_head == 32 || dim_head == 64 || dim_head == 128 || dim_head == kWideDimHead) && w1 >= 1 && w2 >= 1 && dtype == SA2_BF16;
}

static int check_saved(const sa2_problem *prob, const sa2_saved *saved) {
    if (prob->dim_head == kWideDimHead) return fail(SA2_ERR_UNSUPPORTED, "dim_head=%d keeps no forward partials: pass saved = NULL", prob->dim_head);
    if (!saved->t || !saved->m) return fail(SA2_ERR_NULL_POINTER, "saved->t or saved->m is NULL");
    if ((reinterpret_cast<uintptr_t>(saved->t) & 15) != 0) return fail(SA2_ERR_ALIGNMENT, "saved->t must be 16-byte aligned");
    return SA2_OK;
}

int64_t sa2_saved_t_bytes(const sa2_problem *prob) {
    if (check_problem(prob) != SA2_OK) return -1;
    if (prob->dim_head == kWideDimHead) return 0;
    return (int64_t)prob->batch * prob->heads * prob->w2 * ((prob->seq_len + 31) / 32) * 32 * prob->dim_head * 2;
}

int64_t sa2_saved_m_bytes(const sa2_problem *prob) {
    if (check_problem(prob) != SA2_OK) return -1;
    if (prob->dim_head == kWideDimHead) return 0;
    return (int64_t)prob->batch * prob->heads * prob->w2 * prob->seq_len * 4;
}

int sa2_fwd(const sa2_problem *prob, const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
            const sa2_tensor *v1, const sa2_tensor *v2, const sa2_tensor *out, const sa2_tensor *out_residual,
            float *lse, const sa2_saved *saved, void *hip_stream) {
    SA2_TRY(check_problem(prob));
    if (out_residual) SA2_TRY(check_tensor(out_residual, "out_residual"));
    SA2_TRY(check_tensor(q, "q"));
    SA2_TRY(check_tensor(k1, "k1"));
    SA2_TRY(check_tensor(k2, "k2"));
    SA2_TRY(check_tensor(v1, "v1"));
    SA2_TRY(check_tensor(v2, "v2"));
    SA2_TRY(check_tensor(out, "out"));
    if (!lse) return fail(SA2_ERR_NULL_POINTER, "lse is NULL");
    sa2::KParams k = base_params(prob);
    k.q = dev(q);
    k.k1 = dev(k1);
    k.k2 = dev(k2);
    k.v1 = dev(v1);
    k.v2 = dev(v2);
    k.o = dev(out);
    if (out_residual) k.o_lo = dev(out_residual);
    k.lse = lse;
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    if (saved) {
        SA2_TRY(check_saved(prob, saved));
        k.t_save = static_cast<char *>(saved->t);
        k.m_save = saved->m;
    }
    const int grid = prob->batch * prob->heads * ((prob->seq_len + 31) / 32);
    if (prob->dim_head == kWideDimHead) {
        const int wgrid = prob->batch * prob->heads * ((prob->seq_len + 127) / 128);
        hipLaunchKernelGGL(sa2::fwd_wide_kernel<kWideDimHead>, dim3(wgrid), dim3(256), 0, s, k);
    }
    else
        SA2_FOR_DIM_HEAD(prob->dim_head, hipLaunchKernelGGL(sa2::fwd_kernel<DH>, dim3(grid), dim3(512), 0, s, k));
    return after_launch("forward");
}

int sa2_bwd_delta(const sa2_problem *prob, const sa2_tensor *out, const sa2_tensor *out_residual,
                  const sa2_tensor *dout, float *delta, void *hip_stream) {
    SA2_TRY(check_problem(prob));
    if (out_residual) SA2_TRY(check_tensor(out_residual, "out_residual"));
    SA2_TRY(check_tensor(out, "out"));
    SA2_TRY(check_tensor(dout, "dout"));
    if (!delta) return fail(SA2_ERR_NULL_POINTER, "delta is NULL");
    sa2::KParams k = base_params(prob);
    k.o = dev(out);
    if (out_residual) k.o_lo = dev(out_residual);
    k.dout = dev(dout);
    k.delta = delta;
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    int64_t rows = (int64_t)prob->batch * prob->heads * prob->seq_len;
    int lanes_per_row = prob->dim_head / 8;
    int rows_per_block = 256 / lanes_per_row;
    int grid = (int)((rows + rows_per_block - 1) / rows_per_block);
    SA2_FOR_ANY_DIM_HEAD(prob->dim_head, hipLaunchKernelGGL(sa2::delta_kernel<DH>, dim3(grid), dim3(256), 0, s, k));
    return after_launch("delta");
}

static int bwd_common(const sa2_problem *prob, const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
                      const sa2_tensor *v1, const sa2_tensor *v2, const sa2_tensor *dout, const float *lse,
                      const float *delta, sa2::KParams *k) {
    SA2_TRY(check_problem(prob));
    SA2_TRY(check_tensor(q, "q"));
    SA2_TRY(check_tensor(k1, "k1"));
    SA2_TRY(check_tensor(k2, "k2"));
    SA2_TRY(check_tensor(v1, "v1"));
    SA2_TRY(check_tensor(v2, "v2"));
    SA2_TRY(check_tensor(dout, "dout"));
    if (!lse) return fail(SA2_ERR_NULL_POINTER, "lse is NULL");
    if (!delta) return fail(SA2_ERR_NULL_POINTER, "delta is NULL");
    *k = base_params(prob);
    k->q = dev(q);
    k->k1 = dev(k1);
    k->k2 = dev(k2);
    k->v1 = dev(v1);
    k->v2 = dev(v2);
    k->dout = dev(dout);
    k->lse = const_cast<float *>(lse);
    k->delta = const_cast<float *>(delta);
    return SA2_OK;
}

// Profiling builds only (-DSA2_PROFILING, libsa2_prof.so): SA2_BWD_PASS=first launches only the
// MFMA kernel of the dQ/dK2/dV2 entry point, so that it can be timed alone; the results of such a
// call are incomplete.  The product library does not read the environment.
static int bwd_pass_filter() {
#ifdef SA2_PROFILING
    const char *v = std::getenv("SA2_BWD_PASS");
    if (v && std::strcmp(v, "first") == 0) return 1;
#endif
    return 0;
}

// rows below a 32-row query tile that its offsets reach (offsets run in rounds of eight)
static int q_halo(int w2) { return 8 * ((w2 + 7) / 8) - 1; }

// partial rows of dK2 and dV2 (the dV2 half is not needed with saved forward partials)
static int64_t partial_rows_bytes(const sa2_problem *prob) {
    return sa2::qk2_ws_floats(prob->batch, prob->heads, prob->seq_len, prob->dim_head, 32 + q_halo(prob->w2)) * 4;
}

// dK1/dV1 with the key slabs' work split over two workgroups each (fp32 partial results, summed by a second kernel):
// for grids of one to four workgroups per CU on short sequences, where the slabs at the sequence's end (those within
// w1 + 128 rows of it) meet fewer query tiles than the others and whole workgroups of unequal length leave many CUs
// idle at the end.  Measured on the 256 CUs of an MI355X, whole backward: - 3 % and - 8 % at 512 and 896 workgroups of
// N = 2048, D = 64; - 1 to - 2 % at 512 and 768 of D = 128; + 1 to + 2 % at 256 workgroups and at N = 8192, which the rule
// leaves alone.  The rule is a function of the problem alone (the library is built for this one chip), so workspace sizes
// and the kernels that run do not depend on the device or on which thread asked first.
static constexpr int kComputeUnits = 256;
static int cu_count() { return kComputeUnits; }

static bool dkv1_in_parts(const sa2_problem *prob) {
    if (prob->dim_head == kWideDimHead) return false;
    const int ntile = (prob->seq_len + 127) / 128;
    const int64_t grid = (int64_t)prob->batch * prob->kv_heads * ntile;
    const int64_t ragged = (prob->w1 + 127) / 128 + 1;          // slabs per sequence with a shortened range of query tiles
    return grid > cu_count() && grid < 4 * cu_count() && 8 * ragged >= ntile;
}

static int64_t dkv1_parts_bytes(const sa2_problem *prob) {
    if (!dkv1_in_parts(prob)) return 0;
    return 2ll * 2 * prob->batch * prob->kv_heads * prob->seq_len * prob->dim_head * 4;
}

static int64_t max64(int64_t a, int64_t b) { return a > b ? a : b; }

int64_t sa2_bwd_workspace_bytes(const sa2_problem *prob) {
    if (check_problem(prob) != SA2_OK) return -1;
    return max64(partial_rows_bytes(prob), dkv1_parts_bytes(prob));
}

int64_t sa2_bwd_workspace_bytes_with_saved(const sa2_problem *prob) {
    if (check_problem(prob) != SA2_OK) return -1;
    return max64(partial_rows_bytes(prob) / 2, dkv1_parts_bytes(prob));
}

// The launches behind sa2_bwd_dq_dkv2: the MFMA kernel(s) on stream `s`; the kernel that streams the forward's saved
// partials on `s_dv2` (it depends on nothing the backward computes); the reduction of the partial rows on `s_comb`
// (it follows the MFMA kernel: the caller orders the streams).
struct QLaunch {
    sa2::KParams k;
    float *ws;
    int grid, halo;
    bool use_saved;
};

static int prepare_dq_dkv2(const sa2_problem *prob, const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
                           const sa2_tensor *v1, const sa2_tensor *v2, const sa2_tensor *dout, const float *lse,
                           const float *delta, const sa2_saved *saved, const sa2_tensor *dq, const sa2_tensor *dk2,
                           const sa2_tensor *dv2, void *workspace, int64_t workspace_bytes, QLaunch *out) {
    sa2::KParams &k = out->k;
    SA2_TRY(bwd_common(prob, q, k1, k2, v1, v2, dout, lse, delta, &k));
    SA2_TRY(check_tensor(dq, "dq"));
    SA2_TRY(check_tensor(dk2, "dk2"));
    SA2_TRY(check_tensor(dv2, "dv2"));
    if (!workspace) return fail(SA2_ERR_NULL_POINTER, "workspace is NULL");
    if ((reinterpret_cast<uintptr_t>(workspace) & 15) != 0) return fail(SA2_ERR_ALIGNMENT, "workspace must be 16-byte aligned");
    // the dK2 partial rows are the first half of the workspace, the dV2 partial rows the second: with saved
    // forward partials dV2 needs none
    const bool saved_given = saved != nullptr;
    const int64_t need = partial_rows_bytes(prob) / (saved_given ? 2 : 1);
    if (workspace_bytes < need)
        return fail(SA2_ERR_BAD_SHAPE, "workspace of %lld bytes is smaller than the %lld bytes this call needs (sa2_bwd_workspace_bytes%s())",
                    (long long)workspace_bytes, (long long)need, saved_given ? "_with_saved" : "");
    k.dq = dev(dq);
    k.dk2 = dev(dk2);
    k.dv2 = dev(dv2);
    out->ws = static_cast<float *>(workspace);
    out->grid = prob->batch * prob->heads * ((prob->seq_len + 31) / 32);
    out->halo = q_halo(prob->w2);
    // with the forward's saved per-offset T the dv2 pass (a recomputation of S and T) is
    // replaced by a kernel that streams T once
    out->use_saved = saved_given;
    if (saved) {
        SA2_TRY(check_saved(prob, saved));
        k.t_save = static_cast<char *>(saved->t);
        k.m_save = saved->m;
    }
    return SA2_OK;
}

static int launch_q_mfma(const sa2_problem *prob, const QLaunch &L, int pass, hipStream_t s) {
    if (prob->dim_head == kWideDimHead) {
        // one kernel forms dQ and both sets of partial rows
        hipLaunchKernelGGL(sa2::bwd_wide_q_kernel<kWideDimHead>, dim3(L.grid), dim3(256), 0, s, L.k, L.ws, L.halo);
        return after_launch("dq/dk2/dv2");
    }
    SA2_FOR_DIM_HEAD(prob->dim_head, hipLaunchKernelGGL((sa2::bwd_q_kernel<DH, true>), dim3(L.grid), dim3(512), 0, s, L.k, L.ws, L.halo));
    if (pass != 1 && !L.use_saved)
        SA2_FOR_DIM_HEAD(prob->dim_head, hipLaunchKernelGGL((sa2::bwd_q_kernel<DH, false>), dim3(L.grid), dim3(512), 0, s, L.k, L.ws, L.halo));
    return after_launch("dq/dk2/dv2");
}

static int launch_dv2_from_saved(const sa2_problem *prob, const QLaunch &L, hipStream_t s) {
    const int dgrid = prob->batch * prob->kv_heads * ((prob->seq_len + 31) / 32);
    SA2_FOR_DIM_HEAD(prob->dim_head, hipLaunchKernelGGL(sa2::dv2_from_saved_kernel<DH>, dim3(dgrid), dim3(sa2::Dv2Cfg<DH>::THREADS), 0, s, L.k));
    return after_launch("dv2 from saved partials");
}

static int launch_q_combine(const sa2_problem *prob, const QLaunch &L, hipStream_t s) {
    const int64_t rows = (int64_t)prob->batch * prob->kv_heads * prob->seq_len;
    const int rows_per_block = 256 / (prob->dim_head / 8);
    const int cgrid = (int)((rows + rows_per_block - 1) / rows_per_block);
    const int with_dv2 = L.use_saved ? 0 : 1;
    SA2_FOR_ANY_DIM_HEAD(prob->dim_head, hipLaunchKernelGGL(sa2::dk2_dv2_combine_kernel<DH>, dim3(cgrid), dim3(256), 0, s, L.k, L.ws, 32 + L.halo, with_dv2));
    return after_launch("dk2/dv2 combine");
}

int sa2_bwd_dq_dkv2(const sa2_problem *prob, const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
                    const sa2_tensor *v1, const sa2_tensor *v2, const sa2_tensor *dout, const float *lse,
                    const float *delta, const sa2_saved *saved, const sa2_tensor *dq, const sa2_tensor *dk2,
                    const sa2_tensor *dv2, void *workspace, int64_t workspace_bytes, void *hip_stream) {
    QLaunch L;
    SA2_TRY(prepare_dq_dkv2(prob, q, k1, k2, v1, v2, dout, lse, delta, saved, dq, dk2, dv2, workspace, workspace_bytes, &L));
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    const int pass = bwd_pass_filter();
    SA2_TRY(launch_q_mfma(prob, L, pass, s));
    if (pass == 1) return SA2_OK;    // profiling build, one pass: leave the reductions out of its timing
    if (L.use_saved) SA2_TRY(launch_dv2_from_saved(prob, L, s));
    return launch_q_combine(prob, L, s);
}

static int launch_dkv1(const sa2_problem *prob, const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
                       const sa2_tensor *v1, const sa2_tensor *v2, const sa2_tensor *dout, const float *lse,
                       const float *delta, const sa2_tensor *dk1, const sa2_tensor *dv1, float *parts, void *hip_stream) {
    sa2::KParams k;
    SA2_TRY(bwd_common(prob, q, k1, k2, v1, v2, dout, lse, delta, &k));
    SA2_TRY(check_tensor(dk1, "dk1"));
    SA2_TRY(check_tensor(dv1, "dv1"));
    k.dk1 = dev(dk1);
    k.dv1 = dev(dv1);
    k.kv_parts = parts;
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    if (prob->dim_head == kWideDimHead) {
        const int wgrid = prob->batch * prob->kv_heads * ((prob->seq_len + 31) / 32);
        hipLaunchKernelGGL(sa2::bwd_wide_kv_kernel<kWideDimHead>, dim3(wgrid), dim3(256), 0, s, k);
        return after_launch("dk1/dv1");
    }
    const int grid = prob->batch * prob->kv_heads * ((prob->seq_len + 127) / 128);
    // dim_head 128: the two waves of a slab split the contractions; dim_head 64 and 32: each wave forms both outputs
    if (parts) {
        if (prob->dim_head == 128)
            hipLaunchKernelGGL((sa2::bwd_kv8_kernel<128, sa2::kKvSplit, true>), dim3(2 * grid), dim3(512), 0, s, k);
        else if (prob->dim_head == 64)
            hipLaunchKernelGGL((sa2::bwd_kv8_kernel<64, sa2::kKvBoth, true>), dim3(2 * grid), dim3(512), 0, s, k);
        else
            hipLaunchKernelGGL((sa2::bwd_kv8_kernel<32, sa2::kKvBoth, true>), dim3(2 * grid), dim3(512), 0, s, k);
        SA2_TRY(after_launch("dk1/dv1 in parts"));
        const int64_t rows = (int64_t)prob->batch * prob->kv_heads * prob->seq_len;
        const int rows_per_block = 256 / (prob->dim_head / 8);
        const int cgrid = (int)((rows + rows_per_block - 1) / rows_per_block);
        SA2_FOR_DIM_HEAD(prob->dim_head, hipLaunchKernelGGL(sa2::dkv1_parts_combine_kernel<DH>, dim3(cgrid), dim3(256), 0, s, k));
        return after_launch("dk1/dv1 parts combine");
    }
    if (prob->dim_head == 128)
        hipLaunchKernelGGL((sa2::bwd_kv8_kernel<128, sa2::kKvSplit>), dim3(grid), dim3(512), 0, s, k);
    else if (prob->dim_head == 64)
        hipLaunchKernelGGL((sa2::bwd_kv8_kernel<64, sa2::kKvBoth>), dim3(grid), dim3(512), 0, s, k);
    else
        hipLaunchKernelGGL((sa2::bwd_kv8_kernel<32, sa2::kKvBoth>), dim3(grid), dim3(512), 0, s, k);
    return after_launch("dk1/dv1");
}

int sa2_bwd_dkv1(const sa2_problem *prob, const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
                 const sa2_tensor *v1, const sa2_tensor *v2, const sa2_tensor *dout, const float *lse,
                 const float *delta, const sa2_tensor *dk1, const sa2_tensor *dv1, void *hip_stream) {
    return launch_dkv1(prob, q, k1, k2, v1, v2, dout, lse, delta, dk1, dv1, nullptr, hip_stream);
}

int sa2_bwd(const sa2_problem *prob, const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
            const sa2_tensor *v1, const sa2_tensor *v2, const sa2_tensor *out, const sa2_tensor *out_residual,
            const sa2_tensor *dout, const float *lse, const sa2_saved *saved, float *delta_ws, const sa2_tensor *dq,
            const sa2_tensor *dk1, const sa2_tensor *dk2, const sa2_tensor *dv1, const sa2_tensor *dv2, void *workspace,
            int64_t workspace_bytes, void *hip_stream) {
    SA2_TRY(check_problem(prob));
    // every size and pointer is checked before the first launch: a call that fails has written nothing
    const bool parts_wanted = dkv1_in_parts(prob);
    if (parts_wanted && workspace_bytes < dkv1_parts_bytes(prob))
        return fail(SA2_ERR_BAD_SHAPE, "workspace of %lld bytes is smaller than the %lld bytes this problem's dk1/dv1 pass needs (sa2_bwd_workspace_bytes())",
                    (long long)workspace_bytes, (long long)dkv1_parts_bytes(prob));
    if (!delta_ws) return fail(SA2_ERR_NULL_POINTER, "delta is NULL");
    SA2_TRY(check_tensor(out, "out"));
    if (out_residual) SA2_TRY(check_tensor(out_residual, "out_residual"));
    SA2_TRY(check_tensor(dk1, "dk1"));
    SA2_TRY(check_tensor(dv1, "dv1"));
    QLaunch L;
    SA2_TRY(prepare_dq_dkv2(prob, q, k1, k2, v1, v2, dout, lse, delta_ws, saved, dq, dk2, dv2, workspace, workspace_bytes, &L));
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    SA2_TRY(sa2_bwd_delta(prob, out, out_residual, dout, delta_ws, hip_stream));
    SA2_TRY(launch_q_mfma(prob, L, 0, s));
    if (L.use_saved) SA2_TRY(launch_dv2_from_saved(prob, L, s));
    SA2_TRY(launch_q_combine(prob, L, s));
    // the partial rows of dK2/dV2 are spent by now: the partial results of split key slabs reuse the workspace
    float *parts = parts_wanted ? static_cast<float *>(workspace) : nullptr;
    return launch_dkv1(prob, q, k1, k2, v1, v2, dout, lse, delta_ws, dk1, dv1, parts, hip_stream);
}

static int64_t align256(int64_t x) { return (x + 255) & ~int64_t(255); }

int64_t sa2_bwd_noalloc_scratch_bytes(const sa2_problem *prob) {
    const int64_t ws = sa2_bwd_workspace_bytes(prob);
    if (ws < 0) return -1;
    return align256((int64_t)prob->batch * prob->heads * prob->seq_len * 4) + ws;
}

int sa2_bwd_noalloc(const sa2_problem *prob, const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
                    const sa2_tensor *v1, const sa2_tensor *v2, const sa2_tensor *out, const sa2_tensor *out_residual,
                    const sa2_tensor *dout, const float *lse, const sa2_saved *saved, const sa2_tensor *dq,
                    const sa2_tensor *dk1, const sa2_tensor *dk2, const sa2_tensor *dv1, const sa2_tensor *dv2,
                    void *hip_stream) {
    SA2_TRY(check_problem(prob));
    const int64_t need = sa2_bwd_noalloc_scratch_bytes(prob);
    if (need > kNoallocScratchBytes)
        return fail(SA2_ERR_UNSUPPORTED, "this problem needs %lld bytes of scratch, the built-in buffer of sa2_bwd_noalloc holds %lld; "
                    "use sa2_bwd with a caller-owned workspace", (long long)need, (long long)kNoallocScratchBytes);
    unsigned char *scratch = nullptr;
    SA2_TRY(noalloc_scratch(&scratch));
    float *delta = reinterpret_cast<float *>(scratch);
    unsigned char *ws = scratch + align256((int64_t)prob->batch * prob->heads * prob->seq_len * 4);
    // every element of the scratch that a kernel reads was written by an earlier kernel of this same
    // call (delta rows, partial rows), so nothing needs clearing between calls
    return sa2_bwd(prob, q, k1, k2, v1, v2, out, out_residual, dout, lse, saved, delta, dq, dk1, dk2, dv1, dv2, ws,
                   sa2_bwd_workspace_bytes(prob), hip_stream);
}

// ---- fused split + per-head RMSNorm of the qkv projection -------------------------------
static constexpr int kNormMaxBlocks = 2048;

static int norm_groups(const sa2_problem *prob) {
    const int64_t rows = (int64_t)prob->batch * prob->seq_len * (prob->heads + 4 * prob->kv_heads);
    const int rpb = 256 / (prob->dim_head / 8);
    return (int)((rows + rpb - 1) / rpb);
}

static int norm_common(const sa2_problem *prob, const void *qkv, int64_t row_stride, const sa2_tensor *const t[5],
                       const void *const w[5], const float *rstd, sa2::NormParams *np) {
    SA2_TRY(check_problem(prob));
    if (!qkv) return fail(SA2_ERR_NULL_POINTER, "qkv is NULL");
    if (!rstd) return fail(SA2_ERR_NULL_POINTER, "rstd is NULL");
    const int64_t channels = (int64_t)(prob->heads + 4 * prob->kv_heads) * prob->dim_head;
    if (row_stride < channels) return fail(SA2_ERR_BAD_SHAPE, "row_stride %lld is smaller than the %lld channels of a token",
                                           (long long)row_stride, (long long)channels);
    if ((reinterpret_cast<uintptr_t>(qkv) & 15) != 0 || row_stride % 8 != 0)
        return fail(SA2_ERR_ALIGNMENT, "qkv rows must be 16-byte aligned");
    static const char *names[5] = {"q", "k1", "k2", "v1", "v2"};
    *np = sa2::NormParams{};
    for (int x = 0; x < 5; ++x) {
        SA2_TRY(check_tensor(t[x], names[x]));
        np->t[x] = dev(t[x]);
        if (w[x] && (reinterpret_cast<uintptr_t>(w[x]) & 15) != 0) return fail(SA2_ERR_ALIGNMENT, "norm weights must be 16-byte aligned");
        np->w[x] = static_cast<const char *>(w[x]);
    }
    np->qkv = static_cast<const char *>(qkv);
    np->row_stride = row_stride * 2;
    np->rstd = const_cast<float *>(rstd);
    np->B = prob->batch;
    np->N = prob->seq_len;
    np->H = prob->heads;
    np->HK = prob->kv_heads;
    return SA2_OK;
}

int sa2_qkv_norm_fwd(const sa2_problem *prob, const void *qkv, int64_t row_stride, const void *w_q, const void *w_k1,
                     const void *w_k2, const void *w_v1, const void *w_v2, float eps, const sa2_tensor *q,
                     const sa2_tensor *k1, const sa2_tensor *k2, const sa2_tensor *v1, const sa2_tensor *v2, float *rstd,
                     void *hip_stream) {
    const sa2_tensor *const t[5] = {q, k1, k2, v1, v2};
    const void *const w[5] = {w_q, w_k1, w_k2, w_v1, w_v2};
    sa2::NormParams np;
    SA2_TRY(norm_common(prob, qkv, row_stride, t, w, rstd, &np));
    np.eps = eps;
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    const int grid = norm_groups(prob);
    SA2_FOR_ANY_DIM_HEAD(prob->dim_head, hipLaunchKernelGGL(sa2::qkv_norm_fwd_kernel<DH>, dim3(grid), dim3(256), 0, s, np));
    return after_launch("qkv norm forward");
}

int64_t sa2_qkv_norm_bwd_workspace_bytes(const sa2_problem *prob) {
    if (check_problem(prob) != SA2_OK) return -1;
    const int groups = norm_groups(prob);
    const int blocks = groups < kNormMaxBlocks ? groups : kNormMaxBlocks;
    return (int64_t)blocks * 5 * prob->dim_head * 4;
}

int sa2_qkv_norm_bwd(const sa2_problem *prob, const void *qkv, int64_t row_stride, const void *w_q, const void *w_k1,
                     const void *w_k2, const void *w_v1, const void *w_v2, const sa2_tensor *dq, const sa2_tensor *dk1,
                     const sa2_tensor *dk2, const sa2_tensor *dv1, const sa2_tensor *dv2, const float *rstd, void *dqkv,
                     float *dw, void *workspace, int64_t workspace_bytes, void *hip_stream) {
    const sa2_tensor *const t[5] = {dq, dk1, dk2, dv1, dv2};
    const void *const w[5] = {w_q, w_k1, w_k2, w_v1, w_v2};
    sa2::NormParams np;
    SA2_TRY(norm_common(prob, qkv, row_stride, t, w, rstd, &np));
    if (!dqkv || !dw || !workspace) return fail(SA2_ERR_NULL_POINTER, "dqkv, dw or workspace is NULL");
    if ((reinterpret_cast<uintptr_t>(dqkv) & 15) != 0) return fail(SA2_ERR_ALIGNMENT, "dqkv must be 16-byte aligned");
    const int64_t need = sa2_qkv_norm_bwd_workspace_bytes(prob);
    if (workspace_bytes < need)
        return fail(SA2_ERR_BAD_SHAPE, "workspace of %lld bytes is smaller than the %lld bytes sa2_qkv_norm_bwd_workspace_bytes() asks for",
                    (long long)workspace_bytes, (long long)need);
    np.dqkv = static_cast<char *>(dqkv);
    np.dw_part = static_cast<float *>(workspace);
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    const int groups = norm_groups(prob);
    const int blocks = groups < kNormMaxBlocks ? groups : kNormMaxBlocks;
    SA2_FOR_ANY_DIM_HEAD(prob->dim_head, hipLaunchKernelGGL(sa2::qkv_norm_bwd_kernel<DH>, dim3(blocks), dim3(256), 0, s, np, groups));
    SA2_TRY(after_launch("qkv norm backward"));
    const int n = 5 * prob->dim_head;
    hipLaunchKernelGGL(sa2::qkv_norm_dw_kernel, dim3((n + 15) / 16), dim3(256), 0, s, np.dw_part, dw, blocks, n);
    return after_launch("qkv norm weight gradients");
}

#ifdef SA2_PROFILING
// Profiling build only: the instruction-mix loop of sa2_prof_mix.hpp.  `operands`: 64 KiB of bf16 values on the device,
// `out`: workgroups * 512 floats, `clocks`: two 64-bit counters (shader clock, 100 MHz clock) of workgroup 0.  Each SIMD
// executes workgroups / 256 * iters * 32 MFMAs (two waves of 16).  mix: 0 = MFMAs only; 1 = + 4 VALU, 1 exponential and
// 1 LDS fragment read per MFMA; 2 = + 7 VALU, 1 exponential and 2 LDS fragment reads per MFMA.
int sa2_prof_mfma_mix(const void *operands, float *out, unsigned long long *clocks, int mix, int workgroups, int iters, void *hip_stream) {
    if (!operands || !out || !clocks) return fail(SA2_ERR_NULL_POINTER, "operands, out or clocks is NULL");
    if (workgroups < 1 || iters < 1) return fail(SA2_ERR_BAD_SHAPE, "workgroups and iters must be positive");
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    const char *src = static_cast<const char *>(operands);
    if (mix == 0) hipLaunchKernelGGL((sa2::prof_mix_kernel<0, 0, 0>), dim3(workgroups), dim3(512), 0, s, src, out, iters, clocks);
    else if (mix == 1) hipLaunchKernelGGL((sa2::prof_mix_kernel<4, 1, 1>), dim3(workgroups), dim3(512), 0, s, src, out, iters, clocks);
    else if (mix == 2) hipLaunchKernelGGL((sa2::prof_mix_kernel<7, 1, 2>), dim3(workgroups), dim3(512), 0, s, src, out, iters, clocks);
    else return fail(SA2_ERR_UNSUPPORTED, "mix %d is not one of 0, 1, 2", mix);
    return after_launch("instruction-mix loop");
}
#endif

}  // extern "C"
