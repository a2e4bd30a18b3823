// Dynamic-dilation front end: predicted size map -> tap offsets, in one kernel
// each way.
//
// The reference builds the offsets of its size-conditioned layers from torch
// operations: the size activation (network/layers.py:171-181), padding of the
// missing axes with ones (utils/grid.py:83-93) and the broadcast product with
// the kernel grid (utils/grid.py:95-98, dconv_native/grid.py:62-80):
//
//     off[n, 3*k + a, p] = base_a(k_a) * (size_a[n, p] - 1),   k = (kz*kh + ky)*kw + kx
//
// with base_a = linspace(-dil_a*(k_a//2), dil_a*(k_a//2), k_a) and size_a the
// activated prediction of the axis (or 1 for an axis the mode does not predict).
// Backward: grad_size_raw[n, c, p] = act'(raw) * sum over the taps and the axes fed
// by channel c of base_a(k_a) * grad_off[n, 3*k + a, p].
#include "d2c_common.hpp"
#include "d2c_mma.hpp"

namespace {

struct SizeMapArgs {
    d2c_size_map_desc q;
    const void *raw;     // [N][channels(mode)][P]
    void *off;           // forward: [N][3K][P] out; backward: grad_off in
    void *graw;          // backward: [N][channels][P] out
};

template <typename T>
__global__ void __launch_bounds__(256) size_map_fwd_kernel(SizeMapArgs a)
{
    const d2c_size_map_desc &q = a.q;
    const int nc = mode_channels(q.mode), K = q.kd * q.kh * q.kw;
    const long total = (long)q.N * q.P;
    const T *raw = reinterpret_cast<const T *>(a.raw);
    T *off = reinterpret_cast<T *>(a.off);
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const long n = i / q.P, p = i - n * q.P;
        float sm1[3];   // size - 1 per axis
#pragma unroll
        for (int ax = 0; ax < 3; ax++) {
            const int c = axis_channel(q.mode, ax);
            sm1[ax] = c < 0 ? 0.f : rnd<T>(size_act<T>(q.activation, elem_to_f32<T>(raw[(n * nc + c) * q.P + p])) - 1.f);
        }
        T *o = off + n * 3 * K * q.P + p;
        for (int k = 0; k < K; k++) {
            const int kx = k % q.kw, ky = (k / q.kw) % q.kh, kz = k / (q.kw * q.kh);
            o[(long)(3 * k + 0) * q.P] = f32_to_elem<T>(rnd<T>(q.base_z[kz]) * sm1[0]);
            o[(long)(3 * k + 1) * q.P] = f32_to_elem<T>(rnd<T>(q.base_y[ky]) * sm1[1]);
            o[(long)(3 * k + 2) * q.P] = f32_to_elem<T>(rnd<T>(q.base_x[kx]) * sm1[2]);
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(256) size_map_bwd_kernel(SizeMapArgs a)
{
    const d2c_size_map_desc &q = a.q;
    const int nc = mode_channels(q.mode), K = q.kd * q.kh * q.kw;
    const long total = (long)q.N * q.P;
    const T *raw = reinterpret_cast<const T *>(a.raw);
    const T *goff = reinterpret_cast<const T *>(a.off);
    T *graw = reinterpret_cast<T *>(a.graw);
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const long n = i / q.P, p = i - n * q.P;
        const T *g = goff + n * 3 * K * q.P + p;
        float acc[3] = {0.f, 0.f, 0.f};
        for (int k = 0; k < K; k++) {
            const int kx = k % q.kw, ky = (k / q.kw) % q.kh, kz = k / (q.kw * q.kh);
            acc[0] = fmaf(q.base_z[kz], elem_to_f32<T>(g[(long)(3 * k + 0) * q.P]), acc[0]);
            acc[1] = fmaf(q.base_y[ky], elem_to_f32<T>(g[(long)(3 * k + 1) * q.P]), acc[1]);
            acc[2] = fmaf(q.base_x[kx], elem_to_f32<T>(g[(long)(3 * k + 2) * q.P]), acc[2]);
        }
        for (int c = 0; c < nc; c++) {
            float s = 0.f;
#pragma unroll
            for (int ax = 0; ax < 3; ax++)
                if (axis_channel(q.mode, ax) == c) s += acc[ax];
            const long ri = (n * nc + c) * q.P + p;
            graw[ri] = f32_to_elem<T>(s * size_act_grad(q.activation, elem_to_f32<T>(raw[ri])));
        }
    }
}

int check(const d2c_size_map_desc *q)
{
    if (!q) {
        d2c_set_error("size map: null description");
        return D2C_ERR_SHAPE;
    }
    if (q->N <= 0 || q->P <= 0 || q->kd <= 0 || q->kh <= 0 || q->kw <= 0 || q->kd > D2C_SIZE_MAX_K
        || q->kh > D2C_SIZE_MAX_K || q->kw > D2C_SIZE_MAX_K) {
        d2c_set_error("size map: N, P and the kernel extents must be positive, kernel extents at most %d",
                      D2C_SIZE_MAX_K);
        return D2C_ERR_SHAPE;
    }
    if (q->mode < D2C_SIZE_XYZ || q->mode > D2C_SIZE_X || q->activation < D2C_SIZE_ACT_LINEAR
        || q->activation > D2C_SIZE_ACT_RELU_PLUS_ONE) {
        d2c_set_error("size map: unknown mode or activation");
        return D2C_ERR_SHAPE;
    }
    if (q->dtype != D2C_F32 && q->dtype != D2C_BF16) {
        d2c_set_error("size map: float32 or bfloat16 only");
        return D2C_ERR_DTYPE;
    }
    return D2C_OK;
}

unsigned grid_for(long n)
{
    long g = (n + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 16384 ? 16384 : g));
}

}  // namespace

extern "C" int d2c_size_map_offsets_forward(const d2c_size_map_desc *q, const void *size_raw, void *offsets, void *stream)
{
    if (int rc = check(q)) return rc;
    SizeMapArgs a{*q, size_raw, offsets, nullptr};
    const dim3 grid(grid_for((long)q->N * q->P));
    hipStream_t st = (hipStream_t)stream;
    if (q->dtype == D2C_BF16) hipLaunchKernelGGL(size_map_fwd_kernel<bf16_t>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(size_map_fwd_kernel<float>, grid, dim3(256), 0, st, a);
    return d2c_check_launch("size_map_fwd_kernel");
}

extern "C" int d2c_size_map_offsets_backward(const d2c_size_map_desc *q, const void *size_raw, const void *grad_offsets,
                                             void *grad_size_raw, void *stream)
{
    if (int rc = check(q)) return rc;
    SizeMapArgs a{*q, size_raw, const_cast<void *>(grad_offsets), grad_size_raw};
    const dim3 grid(grid_for((long)q->N * q->P));
    hipStream_t st = (hipStream_t)stream;
    if (q->dtype == D2C_BF16) hipLaunchKernelGGL(size_map_bwd_kernel<bf16_t>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(size_map_bwd_kernel<float>, grid, dim3(256), 0, st, a);
    return d2c_check_launch("size_map_bwd_kernel");
}
