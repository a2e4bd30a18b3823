// Direct ("generic") kernels: any shape, f32 / f64 / bf16 storage, no matrix
// cores.  They serve float64 (gradient checks), shapes the tiled kernels do
// not cover, and the 1-D operator.  One thread owns one output element, so no
// intermediate column buffer exists; the price is that samples are recomputed
// by every consumer.  Compute type is float for f32/bf16 storage and double
// for f64 storage.
#include "d2c_common.hpp"

namespace {

constexpr int kBlock = 256;

inline int grid_for(long n, int block = kBlock)
{
    long g = (n + block - 1) / block;
    const long cap = 256L * 64;  // grid-stride beyond 64 blocks per CU
    return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

struct Shape3 {
    int N, Cin, Cout, D, H, W, K, G, groups, Do, Ho, Wo;
    int dt, adt;
    int act;            // forward epilogue: 0 none, 1 act_scale * max(v, 0)
    float act_scale;
    long P, vol;
    TapGeom geo;
};

inline Shape3 shape_of(const d2c_conv3d_desc &q)
{
    Shape3 s;
    s.N = q.N; s.Cin = q.Cin; s.Cout = q.Cout; s.D = q.D; s.H = q.H; s.W = q.W;
    s.K = q.kd * q.kh * q.kw; s.G = q.offset_groups; s.groups = q.groups;
    s.Do = q.Do; s.Ho = q.Ho; s.Wo = q.Wo; s.dt = q.dtype; s.adt = q.aux_dtype;
    s.act = q.epilogue; s.act_scale = q.epilogue_scale;
    s.P = (long)q.Do * q.Ho * q.Wo; s.vol = (long)q.D * q.H * q.W;
    s.geo = make_geom(q);
    return s;
}

// Loads the three offsets and the modulation of (b, g, k, p) and builds the tap.
template <typename CT>
D2C_DEV Tap3<CT> load_tap(const Shape3 &s, const void *off, const void *mask, int b, int g, int k, long p,
                          int oz, int oy, int ox, CT &alpha)
{
    const long ob = (((long)b * s.G + g) * s.K + k) * 3 * s.P + p;
    const CT o0 = ld_as<CT>(off, ob, s.adt);
    const CT o1 = ld_as<CT>(off, ob + s.P, s.adt);
    const CT o2 = ld_as<CT>(off, ob + 2 * s.P, s.adt);
    alpha = mask ? ld_as<CT>(mask, (((long)b * s.G + g) * s.K + k) * s.P + p, s.adt) : (CT)1;
    int bz, by, bx;
    tap_base(s.geo, k, oz, oy, ox, bz, by, bx);
    return make_tap3<CT>(bz, by, bx, o0, o1, o2, s.D, s.H, s.W);
}

// Gathers the 8 corner values of channel plane `xin`, zero where bit c of
// `bits` is clear.
template <typename CT>
D2C_DEV void gather8(const Shape3 &s, const void *x, long plane, const Tap3<CT> &t, unsigned bits, CT *v)
{
#pragma unroll
    for (int c = 0; c < 8; c++) {
        const int zz = t.z0 + ((c >> 2) & 1), yy = t.y0 + ((c >> 1) & 1), xx = t.x0 + (c & 1);
        v[c] = ((bits >> c) & 1u) ? ld_as<CT>(x, plane + ((long)zz * s.H + yy) * s.W + xx, s.dt) : (CT)0;
    }
}

// ------------------------------------------------------------------ forward
// out[b,o,p] = sum_{c in weight group} sum_k W[o,c,k] * alpha * trilinear(x[b,c], pos) + bias[o]
// (dconv3d_gpu.cu:111-203 sampling, :319-353 product, :555-557 bias).
template <typename CT>
__global__ void __launch_bounds__(kBlock)
generic_fwd3d(Shape3 s, const void *x, const void *off, const void *mask, const void *w, const void *bias,
              void *out)
{
    const long total = (long)s.N * s.Cout * s.P;
    const int cg = s.Cin / s.groups, og = s.Cout / s.groups, cpg = s.Cin / s.G;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const long p = idx % s.P;
        const int o = (int)((idx / s.P) % s.Cout);
        const int b = (int)(idx / (s.P * s.Cout));
        const int ox = (int)(p % s.Wo), oy = (int)((p / s.Wo) % s.Ho), oz = (int)(p / ((long)s.Wo * s.Ho));
        const int wg = o / og;
        CT acc = 0;
        for (int k = 0; k < s.K; k++) {
            int c = wg * cg;
            const int cend = c + cg;
            while (c < cend) {
                const int g = c / cpg;
                const int gend = min((g + 1) * cpg, cend);
                CT alpha;
                const Tap3<CT> t = load_tap<CT>(s, off, mask, b, g, k, p, oz, oy, ox, alpha);
                CT a[8];
#pragma unroll
                for (int cc = 0; cc < 8; cc++) a[cc] = tap3_weight(t, cc);
                for (; c < gend; c++) {
                    CT v[8];
                    gather8<CT>(s, x, ((long)b * s.Cin + c) * s.vol, t, t.live, v);
                    CT res = 0;
#pragma unroll
                    for (int cc = 0; cc < 8; cc++) res = d2c_fma<CT>(v[cc], a[cc], res);
                    const CT wv = ld_as<CT>(w, ((long)o * cg + (c - wg * cg)) * s.K + k, s.dt);
                    acc += wv * (alpha * res);
                }
            }
        }
        if (bias) acc += ld_as<CT>(bias, o, s.dt);
        if (s.act) acc = (acc < (CT)0 ? (CT)0 : acc) * (CT)s.act_scale;
        st_as<CT>(out, idx, s.dt, acc);
    }
}

// ---------------------------------------------- backward: input, offset, mask
// One thread per (b, g, k, p) walks the channels of its offset group:
//   gcol   = sum_{o in weight group} W[o,c,k] * gout[b,o,p]      (dconv3d_gpu.cu:976-1000)
//   goff  += alpha * gcol * d(trilinear)/d(z,y,x)               (:708-754, :834-858)
//   gmask += gcol * trilinear                                   (:837-839)
//   gx[corner] += a_corner * alpha * gcol                       (:593-642)
// AT = accumulation type of grad_input (float or double); for bf16 storage the
// caller passes an f32 staging buffer.
template <typename CT, typename AT>
__global__ void __launch_bounds__(kBlock)
generic_bwd3d_data(Shape3 s, const void *gout, const void *x, const void *off, const void *mask, const void *w,
                   AT *gx, void *goff, void *gmask)
{
    const long total = (long)s.N * s.G * s.K * s.P;
    const int cg = s.Cin / s.groups, og = s.Cout / s.groups, cpg = s.Cin / s.G;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const long p = idx % s.P;
        const int k = (int)((idx / s.P) % s.K);
        const int g = (int)((idx / (s.P * s.K)) % s.G);
        const int b = (int)(idx / (s.P * s.K * s.G));
        const int ox = (int)(p % s.Wo), oy = (int)((p / s.Wo) % s.Ho), oz = (int)(p / ((long)s.Wo * s.Ho));
        CT alpha;
        const Tap3<CT> t = load_tap<CT>(s, off, mask, b, g, k, p, oz, oy, ox, alpha);
        CT a[8];
#pragma unroll
        for (int cc = 0; cc < 8; cc++) a[cc] = tap3_weight(t, cc);
        const CT dz = t.hz, dy = t.hy, dx = t.hx;
        CT val0 = 0, val1 = 0, val2 = 0, aval = 0;
        for (int c = g * cpg; c < (g + 1) * cpg; c++) {
            const int wg = c / cg, cl = c - wg * cg;
            CT gcol = 0;
            for (int oo = 0; oo < og; oo++) {
                const int o = wg * og + oo;
                gcol += ld_as<CT>(w, ((long)o * cg + cl) * s.K + k, s.dt)
                      * ld_as<CT>(gout, ((long)b * s.Cout + o) * s.P + p, s.dt);
            }
            const long plane = ((long)b * s.Cin + c) * s.vol;
            if (goff || gmask) {
                CT C[8];
                gather8<CT>(s, x, plane, t, t.inrange, C);
                // C[c] with c = 4*dz+2*dy+dx:  C000=C[0] C001=C[1] C010=C[2] C011=C[3] C100=C[4] ...
                const CT w0 = ((C[4] - C[0]) * (1 - dx) + (C[5] - C[1]) * dx) * (1 - dy)
                            + ((C[6] - C[2]) * (1 - dx) + (C[7] - C[3]) * dx) * dy;
                const CT w1 = ((C[2] - C[0]) * (1 - dz) + (C[6] - C[4]) * dz) * (1 - dx)
                            + ((C[3] - C[1]) * (1 - dz) + (C[7] - C[5]) * dz) * dx;
                const CT w2 = ((C[1] - C[0]) * (1 - dz) + (C[5] - C[4]) * dz) * (1 - dy)
                            + ((C[3] - C[2]) * (1 - dz) + (C[7] - C[6]) * dz) * dy;
                val0 += w0 * gcol; val1 += w1 * gcol; val2 += w2 * gcol;
                if (gmask) {
                    CT res = 0;
#pragma unroll
                    for (int cc = 0; cc < 8; cc++)
                        res = d2c_fma<CT>(((t.live >> cc) & 1u) ? C[cc] : (CT)0, a[cc], res);
                    aval += gcol * res;
                }
            }
            if (gx) {
                const CT base = alpha * gcol;
#pragma unroll
                for (int cc = 0; cc < 8; cc++) {
                    if ((t.live >> cc) & 1u) {
                        const int zz = t.z0 + ((cc >> 2) & 1), yy = t.y0 + ((cc >> 1) & 1), xx = t.x0 + (cc & 1);
                        atomicAdd(&gx[plane + ((long)zz * s.H + yy) * s.W + xx], (AT)(a[cc] * base));
                    }
                }
            }
        }
        if (goff) {
            const long ob = (((long)b * s.G + g) * s.K + k) * 3 * s.P + p;
            st_as<CT>(goff, ob, s.adt, alpha * val0);
            st_as<CT>(goff, ob + s.P, s.adt, alpha * val1);
            st_as<CT>(goff, ob + 2 * s.P, s.adt, alpha * val2);
        }
        if (gmask) st_as<CT>(gmask, (((long)b * s.G + g) * s.K + k) * s.P + p, s.adt, aval);
    }
}

// ------------------------------------------------------- backward: weight
// gW[o,c,k] = sum_b sum_p gout[b,o,p] * alpha * trilinear(x[b,c], pos)   (dconv3d_gpu.cu:1037-1088)
// One wavefront per weight element; lanes stride over (b, p).
template <typename CT>
__global__ void __launch_bounds__(kBlock)
generic_bwd3d_weight(Shape3 s, const void *gout, const void *x, const void *off, const void *mask, void *gw)
{
    const int cg = s.Cin / s.groups, og = s.Cout / s.groups, cpg = s.Cin / s.G;
    const long total = (long)s.Cout * cg * s.K;
    const int lane = threadIdx.x & 63;
    const long wave0 = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const long nwaves = ((long)gridDim.x * blockDim.x) >> 6;
    for (long e = wave0; e < total; e += nwaves) {
        const int k = (int)(e % s.K);
        const int cl = (int)((e / s.K) % cg);
        const int o = (int)(e / ((long)s.K * cg));
        const int c = (o / og) * cg + cl;
        const int g = c / cpg;
        CT acc = 0;
        for (long bp = lane; bp < (long)s.N * s.P; bp += 64) {
            const int b = (int)(bp / s.P);
            const long p = bp % s.P;
            const int ox = (int)(p % s.Wo), oy = (int)((p / s.Wo) % s.Ho), oz = (int)(p / ((long)s.Wo * s.Ho));
            CT alpha;
            const Tap3<CT> t = load_tap<CT>(s, off, mask, b, g, k, p, oz, oy, ox, alpha);
            CT v[8];
            gather8<CT>(s, x, ((long)b * s.Cin + c) * s.vol, t, t.live, v);
            CT res = 0;
#pragma unroll
            for (int cc = 0; cc < 8; cc++) res = d2c_fma<CT>(v[cc], tap3_weight(t, cc), res);
            acc += ld_as<CT>(gout, ((long)b * s.Cout + o) * s.P + p, s.dt) * (alpha * res);
        }
#pragma unroll
        for (int sft = 32; sft > 0; sft >>= 1) acc += __shfl_xor(acc, sft, 64);
        if (lane == 0) st_as<CT>(gw, e, s.dt, acc);
    }
}

// gb[o] = sum_{b,p} gout[b,o,p]   (dconv3d_gpu.cu:1329).  One block per o.
template <typename CT>
__global__ void __launch_bounds__(kBlock)
generic_bias_grad(int N, int Cout, long P, int dt, const void *gout, void *gb)
{
    __shared__ CT part[kBlock / 64];
    const int o = blockIdx.x;
    CT acc = 0;
    for (long bp = threadIdx.x; bp < (long)N * P; bp += blockDim.x) {
        const long b = bp / P, p = bp % P;
        acc += ld_as<CT>(gout, (b * Cout + o) * P + p, dt);
    }
#pragma unroll
    for (int sft = 32; sft > 0; sft >>= 1) acc += __shfl_xor(acc, sft, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        CT t = 0;
        for (int i = 0; i < kBlock / 64; i++) t += part[i];
        st_as<CT>(gb, o, dt, t);
    }
}

// f32 staging buffer -> bf16 tensor of the same layout.
__global__ void __launch_bounds__(kBlock) cvt_f32_to_bf16(const float *src, bf16_t *dst, long n)
{
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        dst[i] = f32_to_bf16(src[i]);
}

template <typename CT>
__global__ void __launch_bounds__(kBlock)
generic_corners3d(Shape3 s, const void *off, int32_t *base, uint8_t *flags)
{
    const long total = (long)s.N * s.G * s.K * s.P;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const long p = idx % s.P;
        const int k = (int)((idx / s.P) % s.K);
        const int g = (int)((idx / (s.P * s.K)) % s.G);
        const int b = (int)(idx / (s.P * s.K * s.G));
        const int ox = (int)(p % s.Wo), oy = (int)((p / s.Wo) % s.Ho), oz = (int)(p / ((long)s.Wo * s.Ho));
        CT alpha;
        const Tap3<CT> t = load_tap<CT>(s, off, nullptr, b, g, k, p, oz, oy, ox, alpha);
        base[idx * 3 + 0] = t.z0;
        base[idx * 3 + 1] = t.y0;
        base[idx * 3 + 2] = t.x0;
        flags[idx] = (uint8_t)t.live;
    }
}

// The sampler alone: a tensor `src` [N, Cs, D, H, W] (a ground-truth mask, say) read at every sampling point of
// the description, out[b, (g*K + k)*Cs + c, p] = trilinear(src[b, c], pos(b, g, k, p)) with the forward pass's rules
// (dconv3d_gpu.cu:48-109: 0 outside (-1, size), corners outside the volume read as 0), no modulation, no weights.
template <typename CT>
__global__ void __launch_bounds__(kBlock)
generic_sample3d(Shape3 s, int Cs, const void *src, const void *off, void *out)
{
    const long total = (long)s.N * s.G * s.K * s.P;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const long p = idx % s.P;
        const int k = (int)((idx / s.P) % s.K);
        const int g = (int)((idx / (s.P * s.K)) % s.G);
        const int b = (int)(idx / (s.P * s.K * s.G));
        const int ox = (int)(p % s.Wo), oy = (int)((p / s.Wo) % s.Ho), oz = (int)(p / ((long)s.Wo * s.Ho));
        CT alpha;
        const Tap3<CT> t = load_tap<CT>(s, off, nullptr, b, g, k, p, oz, oy, ox, alpha);
        CT a[8];
#pragma unroll
        for (int cc = 0; cc < 8; cc++) a[cc] = tap3_weight(t, cc);
        for (int c = 0; c < Cs; c++) {
            CT v[8];
            gather8<CT>(s, src, ((long)b * Cs + c) * s.vol, t, t.live, v);
            CT res = 0;
#pragma unroll
            for (int cc = 0; cc < 8; cc++) res = d2c_fma<CT>(v[cc], a[cc], res);
            st_as<CT>(out, (((long)b * s.G + g) * s.K + k) * Cs * s.P + (long)c * s.P + p, s.dt, res);
        }
    }
}

// Histogram of the offsets per axis: hist[axis][0] counts values below lo, [1 .. nbins] the equal-width bins of
// [lo, hi), [nbins + 1] values at or above hi (and NaN).  Counted in LDS per workgroup, added to `hist` (zeroed by
// the caller of the kernel) with one atomic per non-empty counter.
constexpr int kHistMaxBins = 1024;
template <typename CT>
__global__ void __launch_bounds__(kBlock)
generic_offset_hist3d(Shape3 s, const void *off, float lo, float hi, int nbins, unsigned long long *hist)
{
    extern __shared__ unsigned int s_h[];           // [3][nbins + 2]
    const int nb2 = nbins + 2;
    for (int i = threadIdx.x; i < 3 * nb2; i += blockDim.x) s_h[i] = 0u;
    __syncthreads();
    const long total = (long)s.N * s.G * s.K * 3 * s.P;
    const float scale = (float)nbins / (hi - lo);
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int axis = (int)((idx / s.P) % 3);
        const float v = (float)ld_as<CT>(off, idx, s.adt);
        int bin;
        if (v < lo) bin = 0;
        else if (!(v < hi)) bin = nbins + 1;
        else {
            bin = 1 + (int)((v - lo) * scale);
            if (bin > nbins) bin = nbins;            // (rounding at the upper edge)
        }
        atomicAdd(&s_h[axis * nb2 + bin], 1u);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 3 * nb2; i += blockDim.x)
        if (s_h[i]) atomicAdd(&hist[i], (unsigned long long)s_h[i]);
}

__global__ void __launch_bounds__(256) zero_u64_kernel(unsigned long long *p, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0ull;
}

// =========================================================== 1-D operator
struct Shape1 {
    int N, Cin, Cout, L, K, s, p, d, G, groups, Lo, dt, adt, quirks;
};
inline Shape1 shape_of(const d2c_conv1d_desc &q)
{
    Shape1 s{q.N, q.Cin, q.Cout, q.L, q.k, q.s, q.p, q.d, q.offset_groups, q.groups, q.Lo,
             q.dtype, q.aux_dtype, q.reference_quirks};
    return s;
}

// dconv1d_gpu.cu:12-15
template <typename CT> D2C_DEV CT lerp1(CT v0, CT v1, CT t) { return d2c_fma<CT>(t, v1, d2c_fma<CT>(-t, v0, v0)); }

template <typename CT>
D2C_DEV int floor_to_int_clamped(CT v, int L)
{
    if (!(v == v)) return -4;
    const CT c = v < (CT)-4 ? (CT)-4 : (v > (CT)(L + 4) ? (CT)(L + 4) : v);
    return (int)d2c_floor<CT>(c);
}

// out[b,o,x] = sum_c sum_i W[o,c,i] * alpha * lerp(v0, v1, pos - x0) + bias[o]
// (dconv1d_gpu.cu:17-56, :167-201); both corners gated by range, no early-out.
template <typename CT>
__global__ void __launch_bounds__(kBlock)
generic_fwd1d(Shape1 s, const void *x, const void *off, const void *mask, const void *w, const void *bias,
              void *out)
{
    const long total = (long)s.N * s.Cout * s.Lo;
    const int cg = s.Cin / s.groups, og = s.Cout / s.groups, cpg = s.Cin / s.G;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int ox = (int)(idx % s.Lo);
        const int o = (int)((idx / s.Lo) % s.Cout);
        const int b = (int)(idx / ((long)s.Lo * s.Cout));
        const int wg = o / og;
        CT acc = 0;
        for (int i = 0; i < s.K; i++) {
            int c = wg * cg;
            const int cend = c + cg;
            while (c < cend) {
                const int g = c / cpg;
                const int gend = min((g + 1) * cpg, cend);
                const long ai = ((long)b * s.G * s.K + g * s.K + i) * s.Lo + ox;
                const CT o1 = ld_as<CT>(off, ai, s.adt);
                const CT a = mask ? ld_as<CT>(mask, ai, s.adt) : (CT)1;
                const CT xx = (CT)(ox * s.s - s.p + i * s.d) + o1;
                const int x0 = floor_to_int_clamped<CT>(xx, s.L), x1 = x0 + 1;
                const CT tt = xx - (CT)x0;
                for (; c < gend; c++) {
                    const long row = ((long)b * s.Cin + c) * s.L;
                    const CT v0 = (x0 >= 0 && x0 < s.L) ? ld_as<CT>(x, row + x0, s.dt) : (CT)0;
                    const CT v1 = (x1 >= 0 && x1 < s.L) ? ld_as<CT>(x, row + x1, s.dt) : (CT)0;
                    acc += ld_as<CT>(w, ((long)o * cg + (c - wg * cg)) * s.K + i, s.dt) * (a * lerp1<CT>(v0, v1, tt));
                }
            }
        }
        if (bias) acc += ld_as<CT>(bias, o, s.dt);
        st_as<CT>(out, idx, s.dt, acc);
    }
}

// One thread per (b, g, i, x): grad_offset / grad_mask (dconv1d_gpu.cu:298-353)
// and the scatter into grad_input (:206-251).
template <typename CT, typename AT>
__global__ void __launch_bounds__(kBlock)
generic_bwd1d_data(Shape1 s, const void *gout, const void *x, const void *off, const void *mask, const void *w,
                   AT *gx, void *goff, void *gmask)
{
    const long total = (long)s.N * s.G * s.K * s.Lo;
    const int cg = s.Cin / s.groups, og = s.Cout / s.groups, cpg = s.Cin / s.G;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int ox = (int)(idx % s.Lo);
        const int i = (int)((idx / s.Lo) % s.K);
        const int g = (int)((idx / ((long)s.Lo * s.K)) % s.G);
        const int b = (int)(idx / ((long)s.Lo * s.K * s.G));
        const long ai = ((long)b * s.G * s.K + g * s.K + i) * s.Lo + ox;
        const CT a = mask ? ld_as<CT>(mask, ai, s.adt) : (CT)1;
        const CT xx = (CT)(ox * s.s - s.p + i * s.d) + ld_as<CT>(off, ai, s.adt);
        const int x0 = floor_to_int_clamped<CT>(xx, s.L), x1 = x0 + 1;
        // integer-position rule of the reference: x0 steps down, x1 stays
        int x0q = x0;
        if (s.quirks && (double)(xx - (CT)x0) < 1e-8) x0q -= 1;
        const CT tq = xx - (CT)x0q;
        CT val = 0, aval = 0;
        for (int c = g * cpg; c < (g + 1) * cpg; c++) {
            const int wg = c / cg, cl = c - wg * cg;
            CT gcol = 0;
            for (int oo = 0; oo < og; oo++) {
                const int o = wg * og + oo;
                gcol += ld_as<CT>(w, ((long)o * cg + cl) * s.K + i, s.dt)
                      * ld_as<CT>(gout, ((long)b * s.Cout + o) * s.Lo + ox, s.dt);
            }
            const long row = ((long)b * s.Cin + c) * s.L;
            if (goff || gmask) {
                const CT v0 = (x0q >= 0 && x0q < s.L) ? ld_as<CT>(x, row + x0q, s.dt) : (CT)0;
                const CT v1 = (x1 >= 0 && x1 < s.L) ? ld_as<CT>(x, row + x1, s.dt) : (CT)0;
                aval += gcol * lerp1<CT>(v0, v1, tq);
                val += (v1 - v0) * gcol * a;
            }
            if (gx) {
                const CT grad = a * gcol;
                if (x0 >= 0 && x0 < s.L) atomicAdd(&gx[row + x0], (AT)(((CT)1 - (xx - (CT)x0)) * grad));
                if (x1 >= 0 && x1 < s.L && ((CT)x1 - xx) < (CT)1) atomicAdd(&gx[row + x1], (AT)((xx - (CT)x0) * grad));
            }
        }
        if (goff) st_as<CT>(goff, ai, s.adt, val);
        if (gmask) st_as<CT>(gmask, ai, s.adt, aval);
    }
}

// gW[o,c,i] = sum_{b,x} gout[b,o,x] * alpha * lerp(...)   (dconv1d_gpu.cu:497-537)
template <typename CT>
__global__ void __launch_bounds__(kBlock)
generic_bwd1d_weight(Shape1 s, const void *gout, const void *x, const void *off, const void *mask, void *gw)
{
    const int cg = s.Cin / s.groups, og = s.Cout / s.groups, cpg = s.Cin / s.G;
    const long total = (long)s.Cout * cg * s.K;
    const int lane = threadIdx.x & 63;
    const long wave0 = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const long nwaves = ((long)gridDim.x * blockDim.x) >> 6;
    for (long e = wave0; e < total; e += nwaves) {
        const int i = (int)(e % s.K);
        const int cl = (int)((e / s.K) % cg);
        const int o = (int)(e / ((long)s.K * cg));
        const int c = (o / og) * cg + cl;
        const int g = c / cpg;
        CT acc = 0;
        for (long bp = lane; bp < (long)s.N * s.Lo; bp += 64) {
            const int b = (int)(bp / s.Lo), ox = (int)(bp % s.Lo);
            const long ai = ((long)b * s.G * s.K + g * s.K + i) * s.Lo + ox;
            const CT a = mask ? ld_as<CT>(mask, ai, s.adt) : (CT)1;
            const CT xx = (CT)(ox * s.s - s.p + i * s.d) + ld_as<CT>(off, ai, s.adt);
            const int x0 = floor_to_int_clamped<CT>(xx, s.L), x1 = x0 + 1;
            const long row = ((long)b * s.Cin + c) * s.L;
            const CT v0 = (x0 >= 0 && x0 < s.L) ? ld_as<CT>(x, row + x0, s.dt) : (CT)0;
            const CT v1 = (x1 >= 0 && x1 < s.L) ? ld_as<CT>(x, row + x1, s.dt) : (CT)0;
            acc += ld_as<CT>(gout, ((long)b * s.Cout + o) * s.Lo + ox, s.dt) * (a * lerp1<CT>(v0, v1, xx - (CT)x0));
        }
#pragma unroll
        for (int sft = 32; sft > 0; sft >>= 1) acc += __shfl_xor(acc, sft, 64);
        if (lane == 0) st_as<CT>(gw, e, s.dt, acc);
    }
}

}  // namespace

// ============================================================ host entry
int d2c_generic_conv3d_forward(const d2c_conv3d_desc &q, const void *x, const void *off, const void *mask,
                               const void *w, const void *bias, void *out, hipStream_t st)
{
    const Shape3 s = shape_of(q);
    const long total = (long)s.N * s.Cout * s.P;
    if (q.dtype == D2C_F64)
        hipLaunchKernelGGL(generic_fwd3d<double>, dim3(grid_for(total)), dim3(kBlock), 0, st, s, x, off, mask, w, bias, out);
    else
        hipLaunchKernelGGL(generic_fwd3d<float>, dim3(grid_for(total)), dim3(kBlock), 0, st, s, x, off, mask, w, bias, out);
    return d2c_check_launch("generic_fwd3d");
}

size_t d2c_generic_conv3d_backward_ws(const d2c_conv3d_desc &q)
{
    // bf16 grad_input is accumulated in an f32 staging buffer
    return q.dtype == D2C_BF16 ? d2c_align_up((size_t)q.N * q.Cin * q.D * q.H * q.W * sizeof(float)) : 0;
}

int d2c_generic_conv3d_backward(const d2c_conv3d_desc &q, const void *gout, const void *x, const void *off,
                                const void *mask, const void *w, void *gx, void *goff, void *gmask, void *gw,
                                void *gb, void *ws, hipStream_t st)
{
    const Shape3 s = shape_of(q);
    const long nx = (long)s.N * s.Cin * s.vol;
    if (!mask) gmask = nullptr;
    if (gx || goff || gmask) {
        const long total = (long)s.N * s.G * s.K * s.P;
        if (q.dtype == D2C_F64) {
            if (gx) d2c_fill_zero(gx, nx * sizeof(double), st);
            hipLaunchKernelGGL((generic_bwd3d_data<double, double>), dim3(grid_for(total)), dim3(kBlock), 0, st, s,
                               gout, x, off, mask, w, (double *)gx, goff, gmask);
        } else {
            float *acc = gx ? (q.dtype == D2C_BF16 ? (float *)ws : (float *)gx) : nullptr;
            if (acc) d2c_fill_zero(acc, nx * sizeof(float), st);
            hipLaunchKernelGGL((generic_bwd3d_data<float, float>), dim3(grid_for(total)), dim3(kBlock), 0, st, s,
                               gout, x, off, mask, w, acc, goff, gmask);
            if (acc && q.dtype == D2C_BF16)
                hipLaunchKernelGGL(cvt_f32_to_bf16, dim3(grid_for(nx)), dim3(kBlock), 0, st, acc, (bf16_t *)gx, nx);
        }
        if (int rc = d2c_check_launch("generic_bwd3d_data")) return rc;
    }
    if (gw) {
        const long total = (long)s.Cout * (s.Cin / s.groups) * s.K;
        const int grid = grid_for(total * 64);
        if (q.dtype == D2C_F64)
            hipLaunchKernelGGL(generic_bwd3d_weight<double>, dim3(grid), dim3(kBlock), 0, st, s, gout, x, off, mask, gw);
        else
            hipLaunchKernelGGL(generic_bwd3d_weight<float>, dim3(grid), dim3(kBlock), 0, st, s, gout, x, off, mask, gw);
        if (int rc = d2c_check_launch("generic_bwd3d_weight")) return rc;
    }
    if (gb) {
        if (q.dtype == D2C_F64)
            hipLaunchKernelGGL(generic_bias_grad<double>, dim3(s.Cout), dim3(kBlock), 0, st, s.N, s.Cout, s.P, s.dt, gout, gb);
        else
            hipLaunchKernelGGL(generic_bias_grad<float>, dim3(s.Cout), dim3(kBlock), 0, st, s.N, s.Cout, s.P, s.dt, gout, gb);
        if (int rc = d2c_check_launch("generic_bias_grad")) return rc;
    }
    return D2C_OK;
}

int d2c_generic_conv3d_sample(const d2c_conv3d_desc &q, int Cs, const void *src, const void *off, void *out,
                              hipStream_t st)
{
    const Shape3 s = shape_of(q);
    const long total = (long)s.N * s.G * s.K * s.P;
    if (q.dtype == D2C_F64)
        hipLaunchKernelGGL(generic_sample3d<double>, dim3(grid_for(total)), dim3(kBlock), 0, st, s, Cs, src, off, out);
    else
        hipLaunchKernelGGL(generic_sample3d<float>, dim3(grid_for(total)), dim3(kBlock), 0, st, s, Cs, src, off, out);
    return d2c_check_launch("generic_sample3d");
}

int d2c_generic_conv3d_offset_hist(const d2c_conv3d_desc &q, const void *off, float lo, float hi, int nbins,
                                   unsigned long long *hist, hipStream_t st)
{
    if (nbins < 1 || nbins > kHistMaxBins) {
        d2c_set_error("offset histogram: 1 .. %d bins", kHistMaxBins);
        return D2C_ERR_SHAPE;
    }
    const Shape3 s = shape_of(q);
    const int n = 3 * (nbins + 2);
    hipLaunchKernelGGL(zero_u64_kernel, dim3((n + 255) / 256), dim3(256), 0, st, hist, n);
    const long total = (long)s.N * s.G * s.K * 3 * s.P;
    long g = (total + (long)kBlock * 16 - 1) / ((long)kBlock * 16);     // ~16 values per thread
    if (g < 1) g = 1;
    if (g > 2048) g = 2048;
    const size_t lds = (size_t)n * sizeof(unsigned int);
    if (q.aux_dtype == D2C_F64)
        hipLaunchKernelGGL(generic_offset_hist3d<double>, dim3((unsigned)g), dim3(kBlock), lds, st, s, off, lo, hi, nbins, hist);
    else
        hipLaunchKernelGGL(generic_offset_hist3d<float>, dim3((unsigned)g), dim3(kBlock), lds, st, s, off, lo, hi, nbins, hist);
    return d2c_check_launch("generic_offset_hist3d");
}

int d2c_generic_conv3d_corners(const d2c_conv3d_desc &q, const void *off, int32_t *base, uint8_t *flags,
                               hipStream_t st)
{
    const Shape3 s = shape_of(q);
    const long total = (long)s.N * s.G * s.K * s.P;
    if (q.aux_dtype == D2C_F64)
        hipLaunchKernelGGL(generic_corners3d<double>, dim3(grid_for(total)), dim3(kBlock), 0, st, s, off, base, flags);
    else
        hipLaunchKernelGGL(generic_corners3d<float>, dim3(grid_for(total)), dim3(kBlock), 0, st, s, off, base, flags);
    return d2c_check_launch("generic_corners3d");
}

int d2c_generic_conv1d_forward(const d2c_conv1d_desc &q, const void *x, const void *off, const void *mask,
                               const void *w, const void *bias, void *out, hipStream_t st)
{
    const Shape1 s = shape_of(q);
    const long total = (long)s.N * s.Cout * s.Lo;
    if (q.dtype == D2C_F64)
        hipLaunchKernelGGL(generic_fwd1d<double>, dim3(grid_for(total)), dim3(kBlock), 0, st, s, x, off, mask, w, bias, out);
    else
        hipLaunchKernelGGL(generic_fwd1d<float>, dim3(grid_for(total)), dim3(kBlock), 0, st, s, x, off, mask, w, bias, out);
    return d2c_check_launch("generic_fwd1d");
}

size_t d2c_generic_conv1d_backward_ws(const d2c_conv1d_desc &q)
{
    return q.dtype == D2C_BF16 ? d2c_align_up((size_t)q.N * q.Cin * q.L * sizeof(float)) : 0;
}

int d2c_generic_conv1d_backward(const d2c_conv1d_desc &q, const void *gout, const void *x, const void *off,
                                const void *mask, const void *w, void *gx, void *goff, void *gmask, void *gw,
                                void *gb, void *ws, hipStream_t st)
{
    const Shape1 s = shape_of(q);
    const long nx = (long)s.N * s.Cin * s.L;
    if (gx || goff || gmask) {
        const long total = (long)s.N * s.G * s.K * s.Lo;
        if (q.dtype == D2C_F64) {
            if (gx) d2c_fill_zero(gx, nx * sizeof(double), st);
            hipLaunchKernelGGL((generic_bwd1d_data<double, double>), dim3(grid_for(total)), dim3(kBlock), 0, st, s,
                               gout, x, off, mask, w, (double *)gx, goff, gmask);
        } else {
            float *acc = gx ? (q.dtype == D2C_BF16 ? (float *)ws : (float *)gx) : nullptr;
            if (acc) d2c_fill_zero(acc, nx * sizeof(float), st);
            hipLaunchKernelGGL((generic_bwd1d_data<float, float>), dim3(grid_for(total)), dim3(kBlock), 0, st, s,
                               gout, x, off, mask, w, acc, goff, gmask);
            if (acc && q.dtype == D2C_BF16)
                hipLaunchKernelGGL(cvt_f32_to_bf16, dim3(grid_for(nx)), dim3(kBlock), 0, st, acc, (bf16_t *)gx, nx);
        }
        if (int rc = d2c_check_launch("generic_bwd1d_data")) return rc;
    }
    if (gw) {
        const long total = (long)s.Cout * (s.Cin / s.groups) * s.K;
        const int grid = grid_for(total * 64);
        if (q.dtype == D2C_F64)
            hipLaunchKernelGGL(generic_bwd1d_weight<double>, dim3(grid), dim3(kBlock), 0, st, s, gout, x, off, mask, gw);
        else
            hipLaunchKernelGGL(generic_bwd1d_weight<float>, dim3(grid), dim3(kBlock), 0, st, s, gout, x, off, mask, gw);
        if (int rc = d2c_check_launch("generic_bwd1d_weight")) return rc;
    }
    if (gb) {
        if (q.dtype == D2C_F64)
            hipLaunchKernelGGL(generic_bias_grad<double>, dim3(s.Cout), dim3(kBlock), 0, st, s.N, s.Cout, (long)s.Lo, s.dt, gout, gb);
        else
            hipLaunchKernelGGL(generic_bias_grad<float>, dim3(s.Cout), dim3(kBlock), 0, st, s.N, s.Cout, (long)s.Lo, s.dt, gout, gb);
        if (int rc = d2c_check_launch("generic_bias_grad")) return rc;
    }
    return D2C_OK;
}
