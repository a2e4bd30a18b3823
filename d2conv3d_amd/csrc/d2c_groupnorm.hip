// Normalisation behind the convolution: the GroupNorm that follows every deformable convolution + activation of the
// reference's refinement modules (network/modules/refinement.py:38-43), from per-channel statistics that the
// forward kernels of the convolution add up while they store the output (FwdArgs::stats, d2c_tiled_fwd.hip), so
// that the statistics pass over the output is not needed.
//
//   chan_stats[n][c] = (sum_p x[n,c,p], sum_p x[n,c,p]^2)                       fp32, per (sample, channel)
//   group g of sample n:  mean = sum / m,  var = sumsq / m - mean^2,  m = (C / groups) * P    (biased, as torch)
//   y = (x - mean) * rstd * gamma[c] + beta[c],   rstd = 1 / sqrt(var + eps)
//   backward, with xh = (x - mean) * rstd and per channel r1 = sum_p gy, r2 = sum_p gy * x:
//     grad_x = rstd * (gamma[c] * gy - A / m - xh * B / m),
//         A = sum_{c' in g} gamma[c'] * r1[c'],  B = sum_{c' in g} gamma[c'] * (r2[c'] - mean * r1[c']) * rstd
//     grad_gamma[c] = sum_n (r2 - mean * r1) * rstd,   grad_beta[c] = sum_n r1
//
// One workgroup per (sample, channel) row of P values; 16-byte accesses where the rows allow them.
#include "d2c_common.hpp"
#include "d2c_mma.hpp"

namespace {

constexpr int kGnThreads = 256;

struct GnArgs {
    d2c_group_norm_desc q;
    const void *x, *gy;          // [N][C][P]
    const float *stats;          // [N][C][2]
    const void *gamma, *beta;    // [C] or NULL (1 / 0)
    void *y;                     // forward: y; backward: grad_x
    float *part;                 // backward: [N][C][2] (r1, r2)
    void *ggamma, *gbeta;
};

D2C_DEV float block_sum(float v, float *red)
{
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < kGnThreads / 64; i++) t += red[i];
    return t;
}

// row of P values as 16-byte vectors where aligned: f(index, value) for every element
template <typename T, typename F> D2C_DEV void for_row(const T *row, int P, F f)
{
    constexpr int VEC = 16 / (int)sizeof(T);
    if (P % VEC == 0 && reinterpret_cast<uintptr_t>(row) % 16 == 0) {
        for (int i = threadIdx.x; i < P / VEC; i += kGnThreads) {
            const uint4 v = reinterpret_cast<const uint4 *>(row)[i];
            const T *e = reinterpret_cast<const T *>(&v);
#pragma unroll
            for (int j = 0; j < VEC; j++) f(i * VEC + j, elem_to_f32<T>(e[j]));
        }
    } else {
        for (int i = threadIdx.x; i < P; i += kGnThreads) f(i, elem_to_f32<T>(row[i]));
    }
}

template <typename T> __global__ void __launch_bounds__(kGnThreads) channel_stats_kernel(GnArgs a)
{
    __shared__ float red[kGnThreads / 64];
    const long rowi = blockIdx.x;
    const T *row = reinterpret_cast<const T *>(a.x) + rowi * a.q.P;
    float s = 0.f, sq = 0.f;
    for_row<T>(row, a.q.P, [&](int, float v) { s += v; sq += v * v; });
    s = block_sum(s, red);
    sq = block_sum(sq, red);
    if (threadIdx.x == 0) {
        const_cast<float *>(a.stats)[rowi * 2] = s;
        const_cast<float *>(a.stats)[rowi * 2 + 1] = sq;
    }
}

// mean and 1 / sqrt(var + eps) of a group from the sums over its (C / groups) * P values.  The per-channel fp32 sums
// are combined, and the variance sum_sq / m - mean^2 is taken, in double: with |mean| far above the standard
// deviation the two terms agree in their leading digits and a float difference would lose the variance.
D2C_DEV void moments_from_sums(double s, double sq, double m, float eps, float &mean, float &rstd)
{
    const double mu = s / m;
    const double var = fmax(sq / m - mu * mu, 0.0);
    mean = (float)mu;
    rstd = (float)(1.0 / sqrt(var + (double)eps));
}

// mean and rstd of the group that channel c of sample n belongs to
D2C_DEV void group_moments(const GnArgs &a, int n, int c, float &mean, float &rstd)
{
    const int cpg = a.q.C / a.q.groups, g = c / cpg;
    const float *st = a.stats + ((long)n * a.q.C + g * cpg) * 2;
    double s = 0.0, sq = 0.0;
    for (int i = 0; i < cpg; i++) { s += (double)st[2 * i]; sq += (double)st[2 * i + 1]; }
    moments_from_sums(s, sq, (double)cpg * (double)a.q.P, a.q.eps, mean, rstd);
}

// the same by all threads of a workgroup together
D2C_DEV void group_moments_block(const GnArgs &a, int n, int c, float &mean, float &rstd, float *)
{
    __shared__ double redd[2][kGnThreads / 64];
    const int cpg = a.q.C / a.q.groups, g = c / cpg;
    const float *st = a.stats + ((long)n * a.q.C + g * cpg) * 2;
    double s = 0.0, sq = 0.0;
    for (int i = threadIdx.x; i < cpg; i += kGnThreads) { s += (double)st[2 * i]; sq += (double)st[2 * i + 1]; }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) { s += __shfl_xor(s, d, 64); sq += __shfl_xor(sq, d, 64); }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) { redd[0][threadIdx.x >> 6] = s; redd[1][threadIdx.x >> 6] = sq; }
    __syncthreads();
    s = sq = 0.0;
#pragma unroll
    for (int i = 0; i < kGnThreads / 64; i++) { s += redd[0][i]; sq += redd[1][i]; }
    moments_from_sums(s, sq, (double)cpg * (double)a.q.P, a.q.eps, mean, rstd);
}

template <typename T> __global__ void __launch_bounds__(kGnThreads) gn_fwd_kernel(GnArgs a)
{
    __shared__ float red[kGnThreads / 64];
    const int n = blockIdx.x / a.q.C, c = blockIdx.x % a.q.C;
    float mean, rstd;
    group_moments_block(a, n, c, mean, rstd, red);
    const float ga = a.gamma ? elem_to_f32<T>(reinterpret_cast<const T *>(a.gamma)[c]) : 1.f;
    const float be = a.beta ? elem_to_f32<T>(reinterpret_cast<const T *>(a.beta)[c]) : 0.f;
    const float sc = rstd * ga, sh = be - mean * sc;
    const T *row = reinterpret_cast<const T *>(a.x) + (long)blockIdx.x * a.q.P;
    T *out = reinterpret_cast<T *>(a.y) + (long)blockIdx.x * a.q.P;
    constexpr int VEC = 16 / (int)sizeof(T);
    if (a.q.P % VEC == 0 && reinterpret_cast<uintptr_t>(row) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
        for (int i = threadIdx.x; i < a.q.P / VEC; i += kGnThreads) {
            const uint4 v = reinterpret_cast<const uint4 *>(row)[i];
            const T *e = reinterpret_cast<const T *>(&v);
            alignas(16) T o[VEC];
#pragma unroll
            for (int j = 0; j < VEC; j++) o[j] = f32_to_elem<T>(fmaf(elem_to_f32<T>(e[j]), sc, sh));
            reinterpret_cast<uint4 *>(out)[i] = *reinterpret_cast<const uint4 *>(o);
        }
    } else {
        for (int i = threadIdx.x; i < a.q.P; i += kGnThreads) out[i] = f32_to_elem<T>(fmaf(elem_to_f32<T>(row[i]), sc, sh));
    }
}

template <typename T> __global__ void __launch_bounds__(kGnThreads) gn_bwd_reduce_kernel(GnArgs a)
{
    __shared__ float red[kGnThreads / 64];
    const long rowi = blockIdx.x;
    const T *xr = reinterpret_cast<const T *>(a.x) + rowi * a.q.P;
    const T *gr = reinterpret_cast<const T *>(a.gy) + rowi * a.q.P;
    float r1 = 0.f, r2 = 0.f;
    constexpr int VEC = 16 / (int)sizeof(T);
    if (a.q.P % VEC == 0 && reinterpret_cast<uintptr_t>(xr) % 16 == 0 && reinterpret_cast<uintptr_t>(gr) % 16 == 0) {
        for (int i = threadIdx.x; i < a.q.P / VEC; i += kGnThreads) {
            const uint4 xv = reinterpret_cast<const uint4 *>(xr)[i], gv = reinterpret_cast<const uint4 *>(gr)[i];
            const T *xe = reinterpret_cast<const T *>(&xv), *ge = reinterpret_cast<const T *>(&gv);
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                const float g = elem_to_f32<T>(ge[j]);
                r1 += g;
                r2 = fmaf(g, elem_to_f32<T>(xe[j]), r2);
            }
        }
    } else {
        for (int i = threadIdx.x; i < a.q.P; i += kGnThreads) {
            const float g = elem_to_f32<T>(gr[i]);
            r1 += g;
            r2 = fmaf(g, elem_to_f32<T>(xr[i]), r2);
        }
    }
    r1 = block_sum(r1, red);
    r2 = block_sum(r2, red);
    if (threadIdx.x == 0) {
        a.part[rowi * 2] = r1;
        a.part[rowi * 2 + 1] = r2;
    }
}

template <typename T> __global__ void __launch_bounds__(kGnThreads) gn_bwd_apply_kernel(GnArgs a)
{
    __shared__ float red[kGnThreads / 64];
    const int n = blockIdx.x / a.q.C, c = blockIdx.x % a.q.C;
    const int cpg = a.q.C / a.q.groups, g = c / cpg;
    float mean, rstd;
    group_moments_block(a, n, c, mean, rstd, red);
    float A = 0.f, B = 0.f;
    for (int i = threadIdx.x; i < cpg; i += kGnThreads) {
        const int cc = g * cpg + i;
        const float gm = a.gamma ? elem_to_f32<T>(reinterpret_cast<const T *>(a.gamma)[cc]) : 1.f;
        const float r1 = a.part[((long)n * a.q.C + cc) * 2], r2 = a.part[((long)n * a.q.C + cc) * 2 + 1];
        A = fmaf(gm, r1, A);
        B = fmaf(gm, (r2 - mean * r1) * rstd, B);
    }
    A = block_sum(A, red);
    B = block_sum(B, red);
    const float m = (float)cpg * (float)a.q.P;
    const float ga = a.gamma ? elem_to_f32<T>(reinterpret_cast<const T *>(a.gamma)[c]) : 1.f;
    // grad_x = rstd * (ga * gy - A / m - xh * B / m) = c1 * gy + c2 * x + c3
    const float c1 = rstd * ga, c2 = -rstd * rstd * B / m, c3 = -rstd * A / m - c2 * mean;
    const T *xr = reinterpret_cast<const T *>(a.x) + (long)blockIdx.x * a.q.P;
    const T *gr = reinterpret_cast<const T *>(a.gy) + (long)blockIdx.x * a.q.P;
    T *out = reinterpret_cast<T *>(a.y) + (long)blockIdx.x * a.q.P;
    constexpr int VEC = 16 / (int)sizeof(T);
    if (a.q.P % VEC == 0 && reinterpret_cast<uintptr_t>(xr) % 16 == 0 && reinterpret_cast<uintptr_t>(gr) % 16 == 0
        && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
        for (int i = threadIdx.x; i < a.q.P / VEC; i += kGnThreads) {
            const uint4 xv = reinterpret_cast<const uint4 *>(xr)[i], gv = reinterpret_cast<const uint4 *>(gr)[i];
            const T *xe = reinterpret_cast<const T *>(&xv), *ge = reinterpret_cast<const T *>(&gv);
            alignas(16) T o[VEC];
#pragma unroll
            for (int j = 0; j < VEC; j++)
                o[j] = f32_to_elem<T>(fmaf(c1, elem_to_f32<T>(ge[j]), fmaf(c2, elem_to_f32<T>(xe[j]), c3)));
            reinterpret_cast<uint4 *>(out)[i] = *reinterpret_cast<const uint4 *>(o);
        }
    } else {
        for (int i = threadIdx.x; i < a.q.P; i += kGnThreads)
            out[i] = f32_to_elem<T>(fmaf(c1, elem_to_f32<T>(gr[i]), fmaf(c2, elem_to_f32<T>(xr[i]), c3)));
    }
}

// grad_gamma / grad_beta: one thread per channel, loop over the samples
template <typename T> __global__ void __launch_bounds__(256) gn_bwd_affine_kernel(GnArgs a)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= a.q.C) return;
    float gg = 0.f, gb = 0.f;
    for (int n = 0; n < a.q.N; n++) {
        float mean, rstd;
        group_moments(a, n, c, mean, rstd);
        const float r1 = a.part[((long)n * a.q.C + c) * 2], r2 = a.part[((long)n * a.q.C + c) * 2 + 1];
        gg += (r2 - mean * r1) * rstd;
        gb += r1;
    }
    if (a.ggamma) reinterpret_cast<T *>(a.ggamma)[c] = f32_to_elem<T>(gg);
    if (a.gbeta) reinterpret_cast<T *>(a.gbeta)[c] = f32_to_elem<T>(gb);
}

int check(const d2c_group_norm_desc *q)
{
    if (!q) { d2c_set_error("group norm: null description"); return D2C_ERR_SHAPE; }
    if (q->N <= 0 || q->C <= 0 || q->P <= 0 || q->groups <= 0 || q->C % q->groups != 0) {
        d2c_set_error("group norm: N, C, P, groups must be positive and groups must divide C");
        return D2C_ERR_SHAPE;
    }
    if ((long)q->N * q->C >= (1L << 31)) { d2c_set_error("group norm: too many rows"); return D2C_ERR_SHAPE; }
    if (q->dtype != D2C_F32 && q->dtype != D2C_BF16) { d2c_set_error("group norm: float32 or bfloat16 only"); return D2C_ERR_DTYPE; }
    if (!(q->eps >= 0.f)) { d2c_set_error("group norm: eps must be non-negative"); return D2C_ERR_SHAPE; }
    return D2C_OK;
}

#define GN_LAUNCH(kernel, grid, block)                                                              \
    do {                                                                                            \
        if (q->dtype == D2C_BF16) hipLaunchKernelGGL(kernel<bf16_t>, grid, block, 0, st, a);        \
        else hipLaunchKernelGGL(kernel<float>, grid, block, 0, st, a);                              \
    } while (0)

}  // namespace

extern "C" int d2c_channel_stats(const d2c_group_norm_desc *q, const void *x, float *chan_stats, void *stream)
{
    if (int rc = check(q)) return rc;
    if (!x || !chan_stats) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    hipStream_t st = (hipStream_t)stream;
    GnArgs a{*q, x, nullptr, chan_stats, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    GN_LAUNCH(channel_stats_kernel, dim3((unsigned)(q->N * q->C)), dim3(kGnThreads));
    return d2c_check_launch("channel_stats_kernel");
}

extern "C" int d2c_group_norm_forward(const d2c_group_norm_desc *q, const void *x, const float *chan_stats,
                                      const void *gamma, const void *beta, void *y, void *stream)
{
    if (int rc = check(q)) return rc;
    if (!x || !chan_stats || !y) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    hipStream_t st = (hipStream_t)stream;
    GnArgs a{*q, x, nullptr, chan_stats, gamma, beta, y, nullptr, nullptr, nullptr};
    GN_LAUNCH(gn_fwd_kernel, dim3((unsigned)(q->N * q->C)), dim3(kGnThreads));
    return d2c_check_launch("gn_fwd_kernel");
}

extern "C" size_t d2c_group_norm_backward_workspace_bytes(const d2c_group_norm_desc *q)
{
    if (check(q) != D2C_OK) return 0;
    return d2c_align_up((size_t)q->N * q->C * 2 * sizeof(float));
}

extern "C" int d2c_group_norm_backward(const d2c_group_norm_desc *q, const void *grad_y, const void *x,
                                       const float *chan_stats, const void *gamma, void *grad_x, void *grad_gamma,
                                       void *grad_beta, void *ws, size_t ws_bytes, void *stream)
{
    if (int rc = check(q)) return rc;
    if (!grad_y || !x || !chan_stats) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    const size_t need = d2c_group_norm_backward_workspace_bytes(q);
    if (!ws || ws_bytes < need || ((uintptr_t)ws & 255u)) {
        d2c_set_error("workspace of %zu bytes (256-byte aligned) required, got %zu at %p", need, ws_bytes, ws);
        return D2C_ERR_WORKSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    GnArgs a{*q, x, grad_y, chan_stats, gamma, nullptr, grad_x, (float *)ws, grad_gamma, grad_beta};
    GN_LAUNCH(gn_bwd_reduce_kernel, dim3((unsigned)(q->N * q->C)), dim3(kGnThreads));
    if (int rc = d2c_check_launch("gn_bwd_reduce_kernel")) return rc;
    if (grad_x) {
        GN_LAUNCH(gn_bwd_apply_kernel, dim3((unsigned)(q->N * q->C)), dim3(kGnThreads));
        if (int rc = d2c_check_launch("gn_bwd_apply_kernel")) return rc;
    }
    if (grad_gamma || grad_beta) {
        GN_LAUNCH(gn_bwd_affine_kernel, dim3((unsigned)((q->C + 255) / 256)), dim3(256));
        if (int rc = d2c_check_launch("gn_bwd_affine_kernel")) return rc;
    }
    return D2C_OK;
}
