// C ABI of the library: argument checks of the reference, kernel-family
// choice, workspace carving.  Declarations and contracts: include/d2conv.h.
#include "d2c_common.hpp"
#include "d2c_tiled.hpp"
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <vector>

// Workspace of d2c_conv3d_forward_static: a device array that is part of the library's image, so the call that
// uses it asks the runtime for no memory.  Every GPU the library runs on holds its own copy (at its own
// address) until the process ends.  In host code the name is only a handle for hipGetSymbolAddress; the
// address that kernels and copies get is the one looked up per device below.
static __device__ __align__(256) unsigned char scratch[D2C_STATIC_WORKSPACE_BYTES];

namespace {
thread_local char g_err[512] = "";
std::atomic<uint64_t> g_max_intermediate{1ull << 32};  // dconv3d_gpu.cu:12
std::atomic<int> g_algo_override{D2C_ALGO_AUTO};
std::atomic<int> g_gx_mode{1};
std::atomic<int> g_gw_mode{1};
std::atomic<int> g_bwd_slices{0};

struct ProfState {
    std::mutex mu;
    bool on = false;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> pending[D2C_PROF_COUNT];
    hipEvent_t open_start[D2C_PROF_COUNT] = {};
    double total_ms[D2C_PROF_COUNT] = {};
    int launches[D2C_PROF_COUNT] = {};
    const char *name[D2C_PROF_COUNT] = {};
} g_prof;

struct LdsGrant { const void *fn; int dev, bytes; };
std::mutex g_lds_mu;
std::vector<LdsGrant> g_lds_grants;

__global__ void __launch_bounds__(256) fill_zero_kernel(uint32_t *p, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        p[i] = 0u;
}

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void *g_scratch_ptr[kMaxDevices] = {};

// Address of the current device's copy of `scratch` (looked up once per device, with that device current).
int static_scratch(void **out)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        d2c_set_error("hipGetDevice failed or device index out of range");
        return D2C_ERR_LAUNCH;
    }
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            d2c_set_error("hipGetSymbolAddress(static workspace) on device %d: %s", dev, hipGetErrorString(e));
            return D2C_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return D2C_OK;
}
}  // namespace

int d2c_gx_mode() { return g_gx_mode.load(); }
int d2c_col_weight_mode() { return g_gw_mode.load(); }
int d2c_backward_slices() { return g_bwd_slices.load(); }

void d2c_set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int d2c_check_launch(const char *what)
{
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return D2C_OK;
    d2c_set_error("%s: %s", what, hipGetErrorString(e));
    return D2C_ERR_LAUNCH;
}

int d2c_num_cus()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        d2c_set_error("hipGetDevice failed");
        return 0;
    }
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
        d2c_set_error("hipDeviceGetAttribute(multiprocessor count) failed");
        return 0;
    }
    cached[dev].store(n, std::memory_order_relaxed);
    return n;
}

int d2c_allow_lds(const void *kernel, int bytes, const char *what)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        d2c_set_error("hipGetDevice failed");
        return D2C_ERR_LAUNCH;
    }
    std::lock_guard<std::mutex> lk(g_lds_mu);
    for (const LdsGrant &g : g_lds_grants)
        if (g.fn == kernel && g.dev == dev && g.bytes >= bytes) return D2C_OK;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) {
        d2c_set_error("hipFuncSetAttribute(%s, dynamic LDS %d): %s", what, bytes, hipGetErrorString(e));
        (void)hipGetLastError();
        return D2C_ERR_LAUNCH;
    }
    g_lds_grants.push_back({kernel, dev, bytes});
    return D2C_OK;
}

void d2c_prof_begin(int id, hipStream_t st, const char *name)
{
    if (!g_prof.on) return;
    std::lock_guard<std::mutex> lk(g_prof.mu);
    if (name) g_prof.name[id] = name;
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, st);
    g_prof.open_start[id] = e;
}

void d2c_prof_end(int id, hipStream_t st)
{
    if (!g_prof.on) return;
    std::lock_guard<std::mutex> lk(g_prof.mu);
    if (!g_prof.open_start[id]) return;
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, st);
    g_prof.pending[id].emplace_back(g_prof.open_start[id], e);
    g_prof.open_start[id] = nullptr;
}

void d2c_fill_zero(void *p, size_t bytes, hipStream_t st)
{
    const size_t n = bytes / 4;
    if (n == 0) return;
    size_t g = (n + 255) / 256;
    if (g > 256 * 32) g = 256 * 32;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)g), dim3(256), 0, st, (uint32_t *)p, n);
}

#define D2C_REQUIRE(cond, ...)              \
    do {                                    \
        if (!(cond)) {                      \
            d2c_set_error(__VA_ARGS__);     \
            return D2C_ERR_SHAPE;           \
        }                                   \
    } while (0)

extern "C" {

int32_t d2c_output_size(int32_t in, int32_t k, int32_t stride, int32_t pad, int32_t dil)
{
    return (in + 2 * pad - (dil * (k - 1) + 1)) / stride + 1;
}

const char *d2c_last_error(void) { return g_err; }
int d2c_version(void) { return 2; }
uint64_t d2c_get_max_intermediate_elements(void) { return g_max_intermediate.load(); }
void d2c_set_max_intermediate_elements(uint64_t m) { g_max_intermediate.store(m); }
void d2c_set_algo_override(int algo) { g_algo_override.store(algo); }
void d2c_set_grad_input_mode(int mode) { g_gx_mode.store(mode > 0 ? mode : 0); }
void d2c_set_grad_weight_mode(int mode) { g_gw_mode.store(mode < 0 ? 0 : (mode > 2 ? 2 : mode)); }
void d2c_set_backward_slices(int n) { g_bwd_slices.store(n < 0 ? 0 : n); }

void d2c_profile_enable(int on)
{
    std::lock_guard<std::mutex> lk(g_prof.mu);
    g_prof.on = on != 0;
}

static void prof_drain(int id)
{
    for (auto &pr : g_prof.pending[id]) {
        float ms = 0.f;
        if (hipEventSynchronize(pr.second) == hipSuccess && hipEventElapsedTime(&ms, pr.first, pr.second) == hipSuccess) {
            g_prof.total_ms[id] += ms;
            g_prof.launches[id] += 1;
        }
        (void)hipEventDestroy(pr.first);
        (void)hipEventDestroy(pr.second);
    }
    g_prof.pending[id].clear();
}

void d2c_profile_reset(void)
{
    std::lock_guard<std::mutex> lk(g_prof.mu);
    for (int i = 0; i < D2C_PROF_COUNT; i++) {
        prof_drain(i);
        g_prof.total_ms[i] = 0.0;
        g_prof.launches[i] = 0;
        g_prof.name[i] = nullptr;
    }
}

const char *d2c_profile_kernel_name(int id)
{
    if (id < 0 || id >= D2C_PROF_COUNT) return "";
    std::lock_guard<std::mutex> lk(g_prof.mu);
    return g_prof.name[id] ? g_prof.name[id] : "";
}

int d2c_profile_read(int id, double *total_ms, int *launches)
{
    if (id < 0 || id >= D2C_PROF_COUNT) return D2C_ERR_SHAPE;
    std::lock_guard<std::mutex> lk(g_prof.mu);
    prof_drain(id);
    if (total_ms) *total_ms = g_prof.total_ms[id];
    if (launches) *launches = g_prof.launches[id];
    return D2C_OK;
}

static int check_dtypes(int dtype, int aux)
{
    if (dtype != D2C_F32 && dtype != D2C_F64 && dtype != D2C_BF16) {
        d2c_set_error("unsupported dtype code %d", dtype);
        return D2C_ERR_DTYPE;
    }
    if (!(aux == dtype || (dtype == D2C_BF16 && aux == D2C_F32))) {
        d2c_set_error("aux_dtype %d does not go with dtype %d (offset/mask are of the input's type, or float32 for bfloat16 inputs)", aux, dtype);
        return D2C_ERR_DTYPE;
    }
    return D2C_OK;
}

// Checks of dconv_gpu_common.h:17-24 (groups) and dconv3d_gpu.cu:504-527
// (sizes).  Channel counts of offset / mask are implied by the descriptor; the
// host wrapper compares them with the tensors it holds.
int d2c_conv3d_check(const d2c_conv3d_desc *q)
{
    if (!q) { d2c_set_error("null descriptor"); return D2C_ERR_SHAPE; }
    if (int rc = check_dtypes(q->dtype, q->aux_dtype)) return rc;
    D2C_REQUIRE(q->N > 0 && q->Cin > 0 && q->Cout > 0 && q->D > 0 && q->H > 0 && q->W > 0, "empty input");
    D2C_REQUIRE(q->groups > 0 && q->offset_groups > 0, "group counts must be positive");
    D2C_REQUIRE(q->Cin % q->groups == 0, "weight.size(1) * n_weight_groups == input.size(1) failed");
    D2C_REQUIRE(q->Cout % q->groups == 0, "weight.size(0) %% n_weight_groups == 0 failed");
    D2C_REQUIRE(q->Cout % q->offset_groups == 0, "weight.size(0) %% n_offset_groups == 0 failed");
    D2C_REQUIRE(q->Cin % q->offset_groups == 0, "input.size(1) %% n_offset_groups == 0 failed");
    D2C_REQUIRE(q->kd > 0 && q->kh > 0 && q->kw > 0, "kernel size must be positive");
    D2C_REQUIRE(q->sd > 0 && q->sh > 0 && q->sw > 0, "stride must be positive");
    D2C_REQUIRE(q->pd >= 0 && q->ph >= 0 && q->pw >= 0, "padding must be non-negative");
    D2C_REQUIRE(q->dd > 0 && q->dh > 0 && q->dw > 0, "dilation must be positive");
    const int od = d2c_output_size(q->D, q->kd, q->sd, q->pd, q->dd);
    const int oh = d2c_output_size(q->H, q->kh, q->sh, q->ph, q->dh);
    const int ow = d2c_output_size(q->W, q->kw, q->sw, q->pw, q->dw);
    D2C_REQUIRE(od > 0 && oh > 0 && ow > 0, "computed output size (%d, %d, %d) must be positive", od, oh, ow);
    D2C_REQUIRE(q->Do == od && q->Ho == oh && q->Wo == ow,
                "offset output dims do not match computed dims. Got: (%d, %d, %d) but expected: (%d, %d, %d)",
                q->Do, q->Ho, q->Wo, od, oh, ow);
    const long K = (long)q->kd * q->kh * q->kw, P = (long)od * oh * ow;
    D2C_REQUIRE((long)q->N * q->Cin * q->D * q->H * q->W < (1L << 31) && (long)q->N * q->Cout * P < (1L << 31)
                    && (long)q->N * q->offset_groups * 3 * K * P < (1L << 31)
                    && (long)q->Cout * (q->Cin / q->groups) * K < (1L << 31),
                "tensor with 2^31 or more elements is not supported");
    D2C_REQUIRE(q->offset_axes >= 0 && q->offset_axes <= 7, "offset_axes must be a mask of the axes z, y, x (0 .. 7)");
    D2C_REQUIRE(q->epilogue == D2C_EPILOGUE_NONE || q->epilogue == D2C_EPILOGUE_RELU, "unknown epilogue %d", q->epilogue);
    D2C_REQUIRE((q->backward_flags & ~(D2C_BWD_GW_MASK | D2C_BWD_SLICES(0xff) | D2C_BWD_F32_SPLIT)) == 0, "unknown bits in backward_flags %d",
                q->backward_flags);
    D2C_REQUIRE(q->deform_channels >= 0 && (long)q->N * q->deform_channels * P < (1L << 31),
                "deform_channels must be non-negative and the deformation tensor below 2^31 elements");
    D2C_REQUIRE(q->mask_activation >= D2C_MASK_ACT_NONE && q->mask_activation <= D2C_MASK_ACT_TANH,
                "unknown mask_activation %d", q->mask_activation);
    D2C_REQUIRE(q->epilogue == D2C_EPILOGUE_NONE || (q->epilogue_scale > 0.f && q->epilogue_scale < 3.0e38f),
                "epilogue_scale must be positive and finite");
    return D2C_OK;
}

int d2c_conv1d_check(const d2c_conv1d_desc *q)
{
    if (!q) { d2c_set_error("null descriptor"); return D2C_ERR_SHAPE; }
    if (int rc = check_dtypes(q->dtype, q->aux_dtype)) return rc;
    D2C_REQUIRE(q->N > 0 && q->Cin > 0 && q->Cout > 0 && q->L > 0, "empty input");
    D2C_REQUIRE(q->groups > 0 && q->offset_groups > 0, "group counts must be positive");
    D2C_REQUIRE(q->Cin % q->groups == 0, "weight.size(1) * n_weight_groups == input.size(1) failed");
    D2C_REQUIRE(q->Cout % q->groups == 0, "weight.size(0) %% n_weight_groups == 0 failed");
    D2C_REQUIRE(q->Cout % q->offset_groups == 0, "weight.size(0) %% n_offset_groups == 0 failed");
    D2C_REQUIRE(q->Cin % q->offset_groups == 0, "input.size(1) %% n_offset_groups == 0 failed");
    D2C_REQUIRE(q->k > 0, "kernel size must be positive");
    D2C_REQUIRE(q->s > 0, "stride must be positive");
    D2C_REQUIRE(q->p >= 0, "padding must be non-negative");
    D2C_REQUIRE(q->d > 0, "dilation must be positive");
    const int lo = d2c_output_size(q->L, q->k, q->s, q->p, q->d);
    D2C_REQUIRE(lo > 0, "computed output size %d must be positive", lo);
    D2C_REQUIRE(q->Lo == lo, "offset output dims do not match computed dims. Got: %d but expected: %d", q->Lo, lo);
    D2C_REQUIRE((long)q->N * q->Cin * q->L < (1L << 31) && (long)q->N * q->Cout * lo < (1L << 31)
                    && (long)q->N * q->offset_groups * q->k * lo < (1L << 31)
                    && (long)q->Cout * (q->Cin / q->groups) * q->k < (1L << 31),
                "tensor with 2^31 or more elements is not supported");
    return D2C_OK;
}

static int choose_algo_any_axes(const d2c_conv3d_desc &q, bool quiet);
static int sized_check(const d2c_conv3d_desc *q, const d2c_size_map_desc *z);

// fixed offset axes (the Spatial / Temporal layers) are served by the matrix-core kernels only
static int choose_algo(const d2c_conv3d_desc &q, bool quiet)
{
    const int a = choose_algo_any_axes(q, quiet);
    const bool fixed_axis = (q.offset_axes & 7) != 0 && (q.offset_axes & 7) != 7;
    if (a >= 0 && (q.deform_channels > 0 || q.mask_activation != D2C_MASK_ACT_NONE) &&
        (a != D2C_ALGO_MFMA || !d2c_tiled_packed_supported(q))) {
        if (!quiet)
            d2c_set_error("deform_channels / mask_activation are served by the matrix-core kernels only (split the "
                          "deformation tensor and apply the activation in front of the call instead)");
        return -1;
    }
    if (a >= 0 && fixed_axis && (a != D2C_ALGO_MFMA || !d2c_tiled_axes_supported(q))) {
        if (!quiet)
            d2c_set_error("offset_axes = %d is served by the matrix-core kernels only (in both directions: offset "
                          "groups must lie inside weight groups)", q.offset_axes);
        return -1;
    }
    return a;
}

static int choose_algo_any_axes(const d2c_conv3d_desc &q, bool quiet)
{
    const int forced = g_algo_override.load();
    const bool tiled_ok = d2c_tiled_supported(q);
    if (forced == D2C_ALGO_GENERIC) return D2C_ALGO_GENERIC;
    if (forced == D2C_ALGO_MFMA || forced == D2C_ALGO_DEPTHWISE) {
        const int a = tiled_ok ? d2c_tiled_algo(q) : D2C_ALGO_GENERIC;
        if (a != forced) {
            if (!quiet) d2c_set_error("forced kernel family %d cannot serve this description", forced);
            return -1;
        }
        return a;
    }
    return tiled_ok ? d2c_tiled_algo(q) : D2C_ALGO_GENERIC;
}

int d2c_conv3d_packed_supported(const d2c_conv3d_desc *q, const d2c_size_map_desc *z)
{
    if (!q || (z ? sized_check(q, z) : d2c_conv3d_check(q)) != D2C_OK) return 0;
    return choose_algo(*q, true) == D2C_ALGO_MFMA && d2c_tiled_packed_supported(*q) &&
           (!z || d2c_tiled_sized_supported(*q, true));
}

int d2c_conv3d_algo(const d2c_conv3d_desc *q)
{
    if (d2c_conv3d_check(q) != D2C_OK) return -1;
    return choose_algo(*q, true);
}

size_t d2c_conv3d_forward_workspace_bytes(const d2c_conv3d_desc *q)
{
    if (d2c_conv3d_check(q) != D2C_OK) return 0;
    const int a = choose_algo(*q, true);
    if (a == D2C_ALGO_MFMA || a == D2C_ALGO_DEPTHWISE) return d2c_tiled_forward_ws(*q);
    return 0;
}

size_t d2c_conv3d_backward_workspace_bytes(const d2c_conv3d_desc *q)
{
    if (d2c_conv3d_check(q) != D2C_OK) return 0;
    const int a = choose_algo(*q, true);
    if (a == D2C_ALGO_MFMA || a == D2C_ALGO_DEPTHWISE) return d2c_tiled_backward_ws(*q);
    return d2c_generic_conv3d_backward_ws(*q);
}

static int check_ws(size_t need, void *ws, size_t have)
{
    if (need == 0) return D2C_OK;
    if (!ws || have < need || ((uintptr_t)ws & 255u)) {
        d2c_set_error("workspace of %zu bytes (256-byte aligned) required, got %zu at %p", need, have, ws);
        return D2C_ERR_WORKSPACE;
    }
    return D2C_OK;
}

int d2c_conv3d_forward(const d2c_conv3d_desc *q, const void *x, const void *offset, const void *mask,
                       const void *weight, const void *bias, void *out, void *ws, size_t ws_bytes, void *stream)
{
    if (int rc = d2c_conv3d_check(q)) return rc;
    if (!x || !offset || !weight || !out) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    const int a = choose_algo(*q, false);
    if (a < 0) return D2C_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (a == D2C_ALGO_GENERIC) return d2c_generic_conv3d_forward(*q, x, offset, mask, weight, bias, out, st);
    if (int rc = check_ws(d2c_tiled_forward_ws(*q), ws, ws_bytes)) return rc;
    return d2c_tiled_forward(*q, x, offset, mask, weight, bias, out, ws, st);
}

size_t d2c_conv3d_prepared_bytes(const d2c_conv3d_desc *q)
{
    if (d2c_conv3d_check(q) != D2C_OK) return 0;
    return choose_algo(*q, true) == D2C_ALGO_MFMA ? d2c_tiled_prepared_bytes(*q) : 0;
}

static int check_prepared(const d2c_conv3d_desc &q, void *prepared, size_t prepared_bytes, int reuse, D2cPrepared *out)
{
    out->base = nullptr;
    out->reuse = 0;
    const size_t need = choose_algo(q, true) == D2C_ALGO_MFMA ? d2c_tiled_prepared_bytes(q) : 0;
    if (!prepared || need == 0) return D2C_OK;      // nothing to hold: an ordinary call
    if (prepared_bytes < need || ((uintptr_t)prepared & 255u)) {
        d2c_set_error("prepared region of %zu bytes (256-byte aligned) required, got %zu at %p", need, prepared_bytes, prepared);
        return D2C_ERR_WORKSPACE;
    }
    if (reuse & ~(D2C_REUSE_INPUT | D2C_REUSE_FORWARD_WEIGHTS | D2C_REUSE_BACKWARD_WEIGHTS)) {
        d2c_set_error("unknown bits in reuse flags %d", reuse);
        return D2C_ERR_SHAPE;
    }
    out->base = prepared;
    out->reuse = reuse;
    return D2C_OK;
}

int d2c_conv3d_forward_prepared(const d2c_conv3d_desc *q, const void *x, const void *offset, const void *mask,
                                const void *weight, const void *bias, void *out, void *prepared, size_t prepared_bytes,
                                int32_t reuse, void *ws, size_t ws_bytes, void *stream)
{
    if (int rc = d2c_conv3d_check(q)) return rc;
    if (!x || !offset || !weight || !out) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    const int a = choose_algo(*q, false);
    if (a < 0) return D2C_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (a == D2C_ALGO_GENERIC) return d2c_generic_conv3d_forward(*q, x, offset, mask, weight, bias, out, st);
    D2cPrepared prep;
    if (int rc = check_prepared(*q, prepared, prepared_bytes, reuse, &prep)) return rc;
    if (int rc = check_ws(d2c_tiled_forward_ws(*q), ws, ws_bytes)) return rc;
    return d2c_tiled_forward(*q, x, offset, mask, weight, bias, out, ws, st, nullptr, nullptr, prep.base ? &prep : nullptr);
}

int d2c_conv3d_backward_prepared(const d2c_conv3d_desc *q, const void *gout, const void *x, const void *offset,
                                 const void *mask, const void *weight, void *gx, void *goff, void *gmask, void *gw,
                                 void *gb, void *prepared, size_t prepared_bytes, int32_t reuse, void *ws,
                                 size_t ws_bytes, void *stream)
{
    if (int rc = d2c_conv3d_check(q)) return rc;
    if (!gout || !x || !offset || !weight) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    const int a = choose_algo(*q, false);
    if (a < 0) return D2C_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (a == D2C_ALGO_GENERIC) {
        if (int rc = check_ws(d2c_generic_conv3d_backward_ws(*q), ws, ws_bytes)) return rc;
        return d2c_generic_conv3d_backward(*q, gout, x, offset, mask, weight, gx, goff, gmask, gw, gb, ws, st);
    }
    D2cPrepared prep;
    if (int rc = check_prepared(*q, prepared, prepared_bytes, reuse, &prep)) return rc;
    if (int rc = check_ws(d2c_tiled_backward_ws(*q), ws, ws_bytes)) return rc;
    return d2c_tiled_backward(*q, gout, x, offset, mask, weight, gx, goff, gmask, gw, gb, ws, st, nullptr,
                              prep.base ? &prep : nullptr);
}

size_t d2c_static_workspace_bytes(void) { return (size_t)D2C_STATIC_WORKSPACE_BYTES; }

int d2c_conv3d_forward_static(const d2c_conv3d_desc *q, const void *x, const void *offset, const void *mask,
                              const void *weight, const void *bias, void *out, void *stream)
{
    if (int rc = d2c_conv3d_check(q)) return rc;
    if (!x || !offset || !weight || !out) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    const int a = choose_algo(*q, false);
    if (a < 0) return D2C_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (a == D2C_ALGO_GENERIC) return d2c_generic_conv3d_forward(*q, x, offset, mask, weight, bias, out, st);
    const size_t need = d2c_tiled_forward_ws(*q);
    if (need > (size_t)D2C_STATIC_WORKSPACE_BYTES) {
        d2c_set_error("d2c_conv3d_forward_static: this description needs %zu bytes of workspace, the static one holds "
                      "%zu; use d2c_conv3d_forward with a caller-provided workspace",
                      need, (size_t)D2C_STATIC_WORKSPACE_BYTES);
        return D2C_ERR_WORKSPACE;
    }
    void *ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    return d2c_tiled_forward(*q, x, offset, mask, weight, bias, out, ws, st);
}

int d2c_conv3d_backward(const d2c_conv3d_desc *q, const void *gout, const void *x, const void *offset,
                        const void *mask, const void *weight, void *gx, void *goff, void *gmask, void *gw,
                        void *gb, void *ws, size_t ws_bytes, void *stream)
{
    if (int rc = d2c_conv3d_check(q)) return rc;
    if (!gout || !x || !offset || !weight) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    const int a = choose_algo(*q, false);
    if (a < 0) return D2C_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (a == D2C_ALGO_GENERIC) {
        if (int rc = check_ws(d2c_generic_conv3d_backward_ws(*q), ws, ws_bytes)) return rc;
        return d2c_generic_conv3d_backward(*q, gout, x, offset, mask, weight, gx, goff, gmask, gw, gb, ws, st);
    }
    if (int rc = check_ws(d2c_tiled_backward_ws(*q), ws, ws_bytes)) return rc;
    return d2c_tiled_backward(*q, gout, x, offset, mask, weight, gx, goff, gmask, gw, gb, ws, st);
}

// ---- the operator fed by a size map (dynamic dilation) ----
// Where the matrix-core kernels can form the offsets themselves the map goes straight to them; otherwise it is
// expanded into the front of the workspace by d2c_size_map_offsets_forward and the ordinary call runs behind it
// (and d2c_size_map_offsets_backward folds the offset gradient back).
static int sized_check(const d2c_conv3d_desc *q, const d2c_size_map_desc *z)
{
    if (int rc = d2c_conv3d_check(q)) return rc;
    if (!z) { d2c_set_error("null size-map description"); return D2C_ERR_SHAPE; }
    D2C_REQUIRE(q->offset_groups == 1, "a size map drives one offset group (3K offset channels), got offset_groups = %d",
                q->offset_groups);
    D2C_REQUIRE(z->N == q->N && z->P == q->Do * q->Ho * q->Wo && z->kd == q->kd && z->kh == q->kh && z->kw == q->kw,
                "size-map description does not match the convolution (N, output positions, kernel extents)");
    D2C_REQUIRE(q->kd <= D2C_SIZE_MAX_K && q->kh <= D2C_SIZE_MAX_K && q->kw <= D2C_SIZE_MAX_K,
                "size map: kernel extents at most %d", D2C_SIZE_MAX_K);
    D2C_REQUIRE(z->mode >= D2C_SIZE_XYZ && z->mode <= D2C_SIZE_X && z->activation >= D2C_SIZE_ACT_LINEAR
                    && z->activation <= D2C_SIZE_ACT_RELU_PLUS_ONE, "size map: unknown mode or activation");
    if (q->dtype == D2C_F64 || z->dtype != q->aux_dtype) {
        d2c_set_error("size map: float32 or bfloat16 in the element type of the mask (aux_dtype)");
        return D2C_ERR_DTYPE;
    }
    // a size map inside the layer's deformation tensor, or a modulation activation in the sampler: only where the
    // matrix-core kernels form the offsets themselves (the expansion in front of the other kernels reads a map of its own)
    if ((q->deform_channels > 0 || q->mask_activation != D2C_MASK_ACT_NONE) &&
        !(choose_algo(*q, true) == D2C_ALGO_MFMA && d2c_tiled_sized_supported(*q, true))) {
        d2c_set_error("deform_channels / mask_activation with a size map are served by the matrix-core kernels only");
        return D2C_ERR_UNSUPPORTED;
    }
    return D2C_OK;
}
static size_t expanded_offsets_bytes(const d2c_conv3d_desc &q)
{
    const size_t K = (size_t)q.kd * q.kh * q.kw, P = (size_t)q.Do * q.Ho * q.Wo;
    return d2c_align_up((size_t)q.N * 3 * K * P * d2c_elem_size(q.aux_dtype));
}
static bool sized_fused(const d2c_conv3d_desc &q, bool backward)
{
    const int a = choose_algo(q, true);
    return a == D2C_ALGO_MFMA && d2c_tiled_sized_supported(q, backward);
}

size_t d2c_conv3d_sized_forward_workspace_bytes(const d2c_conv3d_desc *q, const d2c_size_map_desc *z)
{
    if (sized_check(q, z) != D2C_OK) return 0;
    if (sized_fused(*q, false)) return d2c_tiled_forward_ws(*q);
    return expanded_offsets_bytes(*q) + d2c_conv3d_forward_workspace_bytes(q);
}

size_t d2c_conv3d_sized_backward_workspace_bytes(const d2c_conv3d_desc *q, const d2c_size_map_desc *z)
{
    if (sized_check(q, z) != D2C_OK) return 0;
    if (sized_fused(*q, true)) return d2c_tiled_backward_ws(*q, z);
    return 2 * expanded_offsets_bytes(*q) + d2c_conv3d_backward_workspace_bytes(q);
}

int d2c_conv3d_sized_forward(const d2c_conv3d_desc *q, const d2c_size_map_desc *z, const void *x, const void *size_raw,
                             const void *mask, const void *weight, const void *bias, void *out, void *ws,
                             size_t ws_bytes, void *stream)
{
    if (int rc = sized_check(q, z)) return rc;
    if (!x || !size_raw || !weight || !out) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    if (choose_algo(*q, false) < 0) return D2C_ERR_UNSUPPORTED;
    if (int rc = check_ws(d2c_conv3d_sized_forward_workspace_bytes(q, z), ws, ws_bytes)) return rc;
    if (sized_fused(*q, false))
        return d2c_tiled_forward(*q, x, size_raw, mask, weight, bias, out, ws, (hipStream_t)stream, z);
    const size_t ob = expanded_offsets_bytes(*q);
    if (int rc = d2c_size_map_offsets_forward(z, size_raw, ws, stream)) return rc;
    return d2c_conv3d_forward(q, x, ws, mask, weight, bias, out, (char *)ws + ob, ws_bytes - ob, stream);
}

int d2c_conv3d_sized_backward(const d2c_conv3d_desc *q, const d2c_size_map_desc *z, const void *gout, const void *x,
                              const void *size_raw, const void *mask, const void *weight, void *gx, void *gsize,
                              void *gmask, void *gw, void *gb, void *ws, size_t ws_bytes, void *stream)
{
    if (int rc = sized_check(q, z)) return rc;
    if (!gout || !x || !size_raw || !weight) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    if (choose_algo(*q, false) < 0) return D2C_ERR_UNSUPPORTED;
    if (int rc = check_ws(d2c_conv3d_sized_backward_workspace_bytes(q, z), ws, ws_bytes)) return rc;
    if (sized_fused(*q, true))
        return d2c_tiled_backward(*q, gout, x, size_raw, mask, weight, gx, gsize, gmask, gw, gb, ws,
                                  (hipStream_t)stream, z);
    const size_t ob = expanded_offsets_bytes(*q);
    char *off = (char *)ws, *goff = off + ob;
    if (int rc = d2c_size_map_offsets_forward(z, size_raw, off, stream)) return rc;
    if (int rc = d2c_conv3d_backward(q, gout, x, off, mask, weight, gx, gsize ? goff : nullptr, gmask, gw, gb,
                                     goff + ob, ws_bytes - 2 * ob, stream))
        return rc;
    if (gsize) return d2c_size_map_offsets_backward(z, size_raw, goff, gsize, stream);
    return D2C_OK;
}

static bool stats_fused(const d2c_conv3d_desc &q, const d2c_size_map_desc *z)
{
    return choose_algo(q, true) == D2C_ALGO_MFMA && d2c_tiled_forward_fills_stats(q) && (!z || sized_fused(q, false));
}

size_t d2c_conv3d_forward_stats_workspace_bytes(const d2c_conv3d_desc *q, const d2c_size_map_desc *z)
{
    if ((z ? sized_check(q, z) : d2c_conv3d_check(q)) != D2C_OK) return 0;
    if (stats_fused(*q, z)) return d2c_tiled_forward_ws(*q, true);
    return z ? d2c_conv3d_sized_forward_workspace_bytes(q, z) : d2c_conv3d_forward_workspace_bytes(q);
}

int d2c_conv3d_forward_stats(const d2c_conv3d_desc *q, const d2c_size_map_desc *z, const void *x, const void *offset,
                             const void *mask, const void *weight, const void *bias, void *out, float *chan_stats,
                             void *ws, size_t ws_bytes, void *stream)
{
    if (int rc = z ? sized_check(q, z) : d2c_conv3d_check(q)) return rc;
    if (!x || !offset || !weight || !out || !chan_stats) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    if (q->dtype == D2C_F64) { d2c_set_error("output statistics: float32 or bfloat16 only"); return D2C_ERR_DTYPE; }
    const int a = choose_algo(*q, false);
    if (a < 0) return D2C_ERR_UNSUPPORTED;
    // the kernels that add the sums up on their way: matrix-core family, offsets from a tensor or formed in the sampler
    if (stats_fused(*q, z)) {
        if (int rc = check_ws(d2c_tiled_forward_ws(*q, true), ws, ws_bytes)) return rc;
        return d2c_tiled_forward(*q, x, offset, mask, weight, bias, out, ws, (hipStream_t)stream, z, chan_stats);
    }
    if (int rc = z ? d2c_conv3d_sized_forward(q, z, x, offset, mask, weight, bias, out, ws, ws_bytes, stream)
                   : d2c_conv3d_forward(q, x, offset, mask, weight, bias, out, ws, ws_bytes, stream))
        return rc;
    const d2c_group_norm_desc g{q->N, q->Cout, q->Do * q->Ho * q->Wo, 1, q->dtype, 0.f};
    return d2c_channel_stats(&g, out, chan_stats, stream);
}

// ---- the sampled columns of a forward call, kept for the backward call of the same step
static bool columns_served(const d2c_conv3d_desc &q, const d2c_size_map_desc *z)
{
    return choose_algo(q, true) == D2C_ALGO_MFMA && (!z || (sized_fused(q, false) && sized_fused(q, true))) &&
           d2c_tiled_columns_bytes(q, z) > 0;
}

size_t d2c_conv3d_columns_bytes(const d2c_conv3d_desc *q, const d2c_size_map_desc *z)
{
    if ((z ? sized_check(q, z) : d2c_conv3d_check(q)) != D2C_OK) return 0;
    return columns_served(*q, z) ? d2c_tiled_columns_bytes(*q, z) : 0;
}

static int check_columns(const d2c_conv3d_desc &q, const d2c_size_map_desc *z, const void *columns, size_t columns_bytes)
{
    const size_t need = columns_served(q, z) ? d2c_tiled_columns_bytes(q, z) : 0;
    if (need == 0) {
        d2c_set_error("this description keeps no columns (d2c_conv3d_columns_bytes is 0): use the plain calls");
        return D2C_ERR_UNSUPPORTED;
    }
    if (!columns || columns_bytes < need || ((uintptr_t)columns & 255u)) {
        d2c_set_error("column buffer of %zu bytes (256-byte aligned) required, got %zu at %p", need, columns_bytes, columns);
        return D2C_ERR_WORKSPACE;
    }
    return D2C_OK;
}

int d2c_conv3d_forward_columns(const d2c_conv3d_desc *q, const d2c_size_map_desc *z, const void *x, const void *offset,
                               const void *mask, const void *weight, const void *bias, void *out, void *columns,
                               size_t columns_bytes, void *ws, size_t ws_bytes, void *stream)
{
    if (int rc = z ? sized_check(q, z) : d2c_conv3d_check(q)) return rc;
    if (!x || !offset || !weight || !out) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    if (int rc = check_columns(*q, z, columns, columns_bytes)) return rc;
    if (int rc = check_ws(d2c_tiled_forward_ws(*q), ws, ws_bytes)) return rc;
    return d2c_tiled_forward(*q, x, offset, mask, weight, bias, out, ws, (hipStream_t)stream, z, nullptr, nullptr, columns);
}

size_t d2c_conv3d_backward_columns_workspace_bytes(const d2c_conv3d_desc *q, const d2c_size_map_desc *z)
{
    if ((z ? sized_check(q, z) : d2c_conv3d_check(q)) != D2C_OK || !columns_served(*q, z)) return 0;
    return d2c_tiled_backward_ws(*q, z, true);
}

int d2c_conv3d_backward_columns(const d2c_conv3d_desc *q, const d2c_size_map_desc *z, const void *gout, const void *x,
                                const void *offset, const void *mask, const void *weight, const void *columns,
                                size_t columns_bytes, void *gx, void *goff, void *gmask, void *gw, void *gb, void *ws,
                                size_t ws_bytes, void *stream)
{
    if (int rc = z ? sized_check(q, z) : d2c_conv3d_check(q)) return rc;
    if (!gout || !x || !offset || !weight) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    if (int rc = check_columns(*q, z, columns, columns_bytes)) return rc;
    if (int rc = check_ws(d2c_tiled_backward_ws(*q, z, true), ws, ws_bytes)) return rc;
    return d2c_tiled_backward(*q, gout, x, offset, mask, weight, gx, goff, gmask, gw, gb, ws, (hipStream_t)stream, z,
                              nullptr, columns);
}

int d2c_conv3d_corner_index(const d2c_conv3d_desc *q, const void *offset, int32_t *base, uint8_t *flags,
                            void *stream)
{
    if (int rc = d2c_conv3d_check(q)) return rc;
    if (!offset || !base || !flags) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    if (q->deform_channels > 0) { d2c_set_error("corner index: offsets in a tensor of their own only"); return D2C_ERR_UNSUPPORTED; }
    return d2c_generic_conv3d_corners(*q, offset, base, flags, (hipStream_t)stream);
}

int d2c_conv3d_sample(const d2c_conv3d_desc *q, int32_t src_channels, const void *src, const void *offset,
                      void *out, void *stream)
{
    if (int rc = d2c_conv3d_check(q)) return rc;
    if (!src || !offset || !out) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    D2C_REQUIRE(src_channels > 0 && (long)q->N * src_channels * q->D * q->H * q->W < (1L << 31)
                    && (long)q->N * q->offset_groups * q->kd * q->kh * q->kw * src_channels * q->Do * q->Ho * q->Wo < (1L << 31),
                "sample: 1 or more source channels, tensors below 2^31 elements");
    if (q->deform_channels > 0) { d2c_set_error("sample: offsets in a tensor of their own only"); return D2C_ERR_UNSUPPORTED; }
    return d2c_generic_conv3d_sample(*q, src_channels, src, offset, out, (hipStream_t)stream);
}

int d2c_conv3d_offset_histogram(const d2c_conv3d_desc *q, const void *offset, float lo, float hi, int32_t nbins,
                                uint64_t *hist, void *stream)
{
    if (int rc = d2c_conv3d_check(q)) return rc;
    if (!offset || !hist) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    D2C_REQUIRE(lo < hi, "offset histogram: lo < hi");
    if (q->deform_channels > 0) { d2c_set_error("offset histogram: offsets in a tensor of their own only"); return D2C_ERR_UNSUPPORTED; }
    return d2c_generic_conv3d_offset_hist(*q, offset, lo, hi, nbins, reinterpret_cast<unsigned long long *>(hist),
                                          (hipStream_t)stream);
}

static bool use_tiled1d(const d2c_conv1d_desc &q)
{
    return g_algo_override.load() != D2C_ALGO_GENERIC && d2c_tiled1d_supported(q);
}

int d2c_conv1d_algo(const d2c_conv1d_desc *q)
{
    if (d2c_conv1d_check(q) != D2C_OK) return -1;
    return use_tiled1d(*q) ? D2C_ALGO_MFMA : D2C_ALGO_GENERIC;
}

size_t d2c_conv1d_forward_workspace_bytes(const d2c_conv1d_desc *q)
{
    if (d2c_conv1d_check(q) != D2C_OK) return 0;
    return use_tiled1d(*q) ? d2c_tiled1d_forward_ws(*q) : 0;
}

size_t d2c_conv1d_backward_workspace_bytes(const d2c_conv1d_desc *q)
{
    if (d2c_conv1d_check(q) != D2C_OK) return 0;
    return use_tiled1d(*q) ? d2c_tiled1d_backward_ws(*q) : d2c_generic_conv1d_backward_ws(*q);
}

int d2c_conv1d_forward(const d2c_conv1d_desc *q, const void *x, const void *offset, const void *mask,
                       const void *weight, const void *bias, void *out, void *ws, size_t ws_bytes, void *stream)
{
    if (int rc = d2c_conv1d_check(q)) return rc;
    if (!x || !offset || !weight || !out) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    if (use_tiled1d(*q)) {
        if (int rc = check_ws(d2c_tiled1d_forward_ws(*q), ws, ws_bytes)) return rc;
        return d2c_tiled1d_forward(*q, x, offset, mask, weight, bias, out, ws, (hipStream_t)stream);
    }
    return d2c_generic_conv1d_forward(*q, x, offset, mask, weight, bias, out, (hipStream_t)stream);
}

int d2c_conv1d_backward(const d2c_conv1d_desc *q, const void *gout, const void *x, const void *offset,
                        const void *mask, const void *weight, void *gx, void *goff, void *gmask, void *gw,
                        void *gb, void *ws, size_t ws_bytes, void *stream)
{
    if (int rc = d2c_conv1d_check(q)) return rc;
    if (!gout || !x || !offset || !weight) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    if (use_tiled1d(*q)) {
        if (int rc = check_ws(d2c_tiled1d_backward_ws(*q), ws, ws_bytes)) return rc;
        return d2c_tiled1d_backward(*q, gout, x, offset, mask, weight, gx, goff, gmask, gw, gb, ws, (hipStream_t)stream);
    }
    if (int rc = check_ws(d2c_generic_conv1d_backward_ws(*q), ws, ws_bytes)) return rc;
    return d2c_generic_conv1d_backward(*q, gout, x, offset, mask, weight, gx, goff, gmask, gw, gb, ws,
                                       (hipStream_t)stream);
}

}  // extern "C"
