// Channel-separated (depthwise, groups == Cin == Cout) modulated deformable
// conv3d: no GEMM, one multiply per sampled value.  The reference runs this
// case as Cin single-row cuBLAS products over a column buffer
// (dconv3d_gpu.cu:321-353); here one kernel per direction works on the
// channels-last copy of the input; a lane owns 4 consecutive channels, so that
// every corner read of a wavefront is one contiguous 16-byte-per-lane load.
//
//   forward : out[b,c,p]  = bias[c] + sum_k W[c,k] * alpha * trilinear(x[b,c], pos)
//   backward: gcol        = W[c,k] * gout[b,c,p]
//             gx[corner] += a_corner * alpha * gcol                     (sample lists, see d2c_invlist.hip; or atomics)
//             goff, gmask = reductions over the channels of the offset group
//             gW[c,k]    += gout * alpha * trilinear                    (registers, then atomics)
//
// A workgroup owns a tile of 16 output positions.  The corner weights of the
// tile (16 positions x up to 32 taps) are computed once into LDS and shared by
// all channel slices.
#include "d2c_mma.hpp"
#include "d2c_tiled.hpp"

namespace {

constexpr int kDwThreads = 256;
constexpr int kFwdTP = 4;    // positions per tile, forward (small tiles: many workgroups in flight hide the
                             // latency of the dependent gather -> multiply chains)
constexpr int kBwdTP = 16;   // positions per tile, backward (one atomic per tap and channel and tile for grad_weight)
constexpr int kKB = 32;      // taps per batch held in LDS
constexpr int kCV = 4;       // channels per lane

struct DwArgs {
    TiledShape s;
    const void *xcl;           // [N][vol][C]
    const void *off, *mask;
    const void *wt;            // [K][C]  weights, tap-major
    const void *bias;
    void *out;
    // backward
    const void *goutcl;        // [N][P][C]  channels-last copy of grad_out
    float *gxcl;               // [N][vol][C] fp32 accumulator (zeroed) or NULL
    void *goff, *gmask;        // or NULL
    float *gwacc;              // [K][C] fp32 accumulator (zeroed) or NULL
};

template <int TP> constexpr int kNEof = kKB * TP;   // (tap, position) entries per batch

// Workgroups are dealt round-robin to the 8 XCDs; this gives each XCD one contiguous run of tiles, so that
// its L2 sees a compact part of the input.
D2C_DEV int xcd_swizzle(int bid, int n)
{
    const int x = bid & 7, idx = bid >> 3;
    const int q = n >> 3, r = n & 7;
    return x * q + (x < r ? x : r) + idx;
}

// View over dynamic LDS: per entry the live corner weights * alpha, the base
// voxel and live | inrange << 8; for the backward pass also the per-axis
// fractions lz ly lx hz hy hx, alpha, and the 4 offset / mask sums.
template <int TP> struct DwTaps {
    static constexpr int kNE = kNEof<TP>;
    float (*w)[kNE];
    int *idx, *flag;
    float (*frac)[kNE];
    float *alpha;
    float (*aux)[4];
};
template <int TP> D2C_DEV DwTaps<TP> dw_taps(unsigned char *smem, bool bwd)
{
    constexpr int kNE = kNEof<TP>;
    DwTaps<TP> t;
    float *f = reinterpret_cast<float *>(smem);
    t.w = reinterpret_cast<float (*)[kNE]>(f); f += 8 * kNE;
    t.idx = reinterpret_cast<int *>(f); f += kNE;
    t.flag = reinterpret_cast<int *>(f); f += kNE;
    t.frac = nullptr; t.alpha = nullptr; t.aux = nullptr;
    if (bwd) {
        t.frac = reinterpret_cast<float (*)[kNE]>(f); f += 6 * kNE;
        t.alpha = f; f += kNE;
        t.aux = reinterpret_cast<float (*)[4]>(f);
    }
    return t;
}
constexpr size_t kDwLdsFwd = (size_t)10 * kNEof<kFwdTP> * 4;
constexpr size_t kDwLdsBwd = (size_t)21 * kNEof<kBwdTP> * 4;

template <bool BWD, int kTP>
D2C_DEV void dw_coords(const DwArgs &a, const DwTaps<kTP> &t, int m0, int g, int k0, int kn)
{
    const TiledShape &s = a.s;
    for (int task = threadIdx.x; task < kn * kTP; task += kDwThreads) {
        const int pl = task % kTP, kk = task / kTP;
        const int k = k0 + kk, m = m0 + pl;
        float w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        float fr[6] = {0, 0, 0, 0, 0, 0};
        float al = 0.f;
        int idx = 0, flag = 0;
        if (m < s.M) {
            const int b = m / s.P, p = m - b * s.P;
            const int ox = p % s.Wo, oy = (p / s.Wo) % s.Ho, oz = p / (s.Wo * s.Ho);
            const long ob = (((long)b * s.G + g) * s.K + k) * 3 * s.P + p;
            const float o0 = ld_aux(a.off, ob, s.adt);
            const float o1 = ld_aux(a.off, ob + s.P, s.adt);
            const float o2 = ld_aux(a.off, ob + 2 * (long)s.P, s.adt);
            al = a.mask ? ld_aux(a.mask, (((long)b * s.G + g) * s.K + k) * s.P + p, s.adt) : 1.f;
            int bz, by, bx;
            tap_base(s.geo, k, oz, oy, ox, bz, by, bx);
            const Tap3<float> tp = make_tap3<float>(bz, by, bx, o0, o1, o2, s.D, s.H, s.W);
            idx = b * s.vol + (tp.z0 * s.H + tp.y0) * s.W + tp.x0;
            flag = (int)(tp.live | (tp.inrange << 8));
#pragma unroll
            for (int c = 0; c < 8; c++) w[c] = ((tp.live >> c) & 1u) ? tap3_weight(tp, c) * al : 0.f;
            fr[0] = tp.lz; fr[1] = tp.ly; fr[2] = tp.lx; fr[3] = tp.hz; fr[4] = tp.hy; fr[5] = tp.hx;
        }
        const int e = kk * kTP + pl;
#pragma unroll
        for (int c = 0; c < 8; c++) t.w[c][e] = w[c];
        if (BWD) {
#pragma unroll
            for (int c = 0; c < 6; c++) t.frac[c][e] = fr[c];
            t.alpha[e] = al;
        }
        t.idx[e] = idx;
        t.flag[e] = flag;
    }
}

// A lane owns kCV consecutive channels (the channel count of an offset group is a multiple of kCV):
// one vector load per lane, kCV * 64 consecutive channels per wavefront.
template <typename T> D2C_DEV void ld4(const T *p, float *v)
{
    if constexpr (sizeof(T) == 4) {
        const float4 t = *reinterpret_cast<const float4 *>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    } else {
        const uint2 t = *reinterpret_cast<const uint2 *>(p);
        v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
        v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
    }
}
static_assert(kCV == 4, "vector loads of 4 channels");

// ------------------------------------------------------------------ forward
template <typename T>
__global__ void __launch_bounds__(kDwThreads) dw_fwd_kernel(DwArgs a)
{
    constexpr int kTP = kFwdTP;
    extern __shared__ __align__(16) unsigned char smem[];
    const DwTaps<kTP> taps = dw_taps<kTP>(smem, false);
    const TiledShape &s = a.s;
    const int m0 = xcd_swizzle(blockIdx.x, gridDim.x) * kTP;
    const int HW = s.H * s.W;
    const int nslice = (s.cpg + kDwThreads * kCV - 1) / (kDwThreads * kCV);
    const T *xcl = reinterpret_cast<const T *>(a.xcl);
    const T *wt = reinterpret_cast<const T *>(a.wt);
    T *out = reinterpret_cast<T *>(a.out);

    for (int g = 0; g < s.G; g++) {
        for (int k0 = 0; k0 < s.K; k0 += kKB) {   // one batch unless the kernel has more than kKB taps
            const int kn = min(kKB, s.K - k0);
            __syncthreads();
            dw_coords<false, kTP>(a, taps, m0, g, k0, kn);
            __syncthreads();
            for (int sl = 0; sl < nslice; sl++) {
                const int cl = (sl * kDwThreads + threadIdx.x) * kCV;   // first channel (inside the offset group)
                if (cl >= s.cpg) continue;
                const int c = g * s.cpg + cl;
                float bv[kCV] = {0.f, 0.f, 0.f, 0.f};
                if (a.bias && k0 == 0) ld4<T>(reinterpret_cast<const T *>(a.bias) + c, bv);
                for (int p = 0; p < kTP; p++) {
                    const int m = m0 + p;
                    if (m >= s.M) break;
                    float acc[kCV] = {bv[0], bv[1], bv[2], bv[3]};
                    for (int kk = 0; kk < kn; kk++) {
                        const int e = kk * kTP + p;
                        // the table entry is the same for the whole workgroup: keep it in scalar registers
                        const unsigned live = (unsigned)__builtin_amdgcn_readfirstlane(taps.flag[e]) & 0xffu;
                        if (!live) continue;
                        const int idx = __builtin_amdgcn_readfirstlane(taps.idx[e]);
                        float wv[kCV];
                        ld4<T>(wt + (long)(k0 + kk) * s.Cin + c, wv);
                        float xv[8][kCV];
                        // all live corner rows are requested back to back
#pragma unroll
                        for (int cc = 0; cc < 8; cc++) {
                            const int v = idx + ((cc >> 2) & 1) * HW + ((cc >> 1) & 1) * s.W + (cc & 1);
                            if ((live >> cc) & 1u) {
                                ld4<T>(xcl + (long)v * s.Cin + c, xv[cc]);
                            } else {
#pragma unroll
                                for (int j = 0; j < kCV; j++) xv[cc][j] = 0.f;
                            }
                        }
                        float sv[kCV] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int cc = 0; cc < 8; cc++) {
                            const float wc = taps.w[cc][e];
#pragma unroll
                            for (int j = 0; j < kCV; j++) sv[j] = fmaf(wc, xv[cc][j], sv[j]);
                        }
#pragma unroll
                        for (int j = 0; j < kCV; j++) acc[j] = fmaf(wv[j], sv[j], acc[j]);
                    }
                    const int b = m / s.P, pp = m - b * s.P;
#pragma unroll
                    for (int j = 0; j < kCV; j++) {
                        T *o = out + ((long)b * s.Cout + c + j) * s.P + pp;
                        // kernels with more than kKB taps: later batches add to the stored partial sum
                        *o = f32_to_elem<T>(k0 == 0 ? acc[j] : acc[j] + elem_to_f32<T>(*o));
                    }
                }
            }
        }
    }
}

// ----------------------------------------------------------------- backward
// Sum of 4 per-lane values over the 64 lanes: after the exchange steps lane
// group (lane>>4) holds the total of value (lane>>4) in all of its lanes.
D2C_DEV float reduce4_over_wave(float v0, float v1, float v2, float v3, int lane)
{
    // step 1: lanes with bit 5 set keep (v2, v3), others (v0, v1)
    const bool hi5 = lane & 32;
    float k0 = hi5 ? v2 : v0, k1 = hi5 ? v3 : v1;
    float s0 = hi5 ? v0 : v2, s1 = hi5 ? v1 : v3;
    k0 += __shfl_xor(s0, 32, 64);
    k1 += __shfl_xor(s1, 32, 64);
    // step 2: lanes with bit 4 set keep k1, others k0
    const bool hi4 = lane & 16;
    float k = hi4 ? k1 : k0, sd = hi4 ? k0 : k1;
    k += __shfl_xor(sd, 16, 64);
    k += __shfl_xor(k, 8, 64);
    k += __shfl_xor(k, 4, 64);
    k += __shfl_xor(k, 2, 64);
    k += __shfl_xor(k, 1, 64);
    return k;   // value index = (lane >> 5) * 2 + ((lane >> 4) & 1)
}

template <typename T>
__global__ void __launch_bounds__(kDwThreads) dw_bwd_kernel(DwArgs a)
{
    constexpr int kTP = kBwdTP;
    extern __shared__ __align__(16) unsigned char smem[];
    const DwTaps<kTP> taps = dw_taps<kTP>(smem, true);
    float (*s_aux)[4] = taps.aux;   // goff z,y,x and gmask sums over the channels of the group
    const TiledShape &s = a.s;
    const int m0 = xcd_swizzle(blockIdx.x, gridDim.x) * kTP;
    const int HW = s.H * s.W;
    const int lane = threadIdx.x & 63;
    const int nslice = (s.cpg + kDwThreads * kCV - 1) / (kDwThreads * kCV);
    const T *xcl = reinterpret_cast<const T *>(a.xcl);
    const T *wt = reinterpret_cast<const T *>(a.wt);
    const T *goutcl = reinterpret_cast<const T *>(a.goutcl);
    const bool want_aux = a.goff != nullptr || a.gmask != nullptr;

    for (int g = 0; g < s.G; g++) {
        for (int k0 = 0; k0 < s.K; k0 += kKB) {
            const int kn = min(kKB, s.K - k0);
            __syncthreads();
            dw_coords<true, kTP>(a, taps, m0, g, k0, kn);
            for (int e = threadIdx.x; e < kn * kTP; e += kDwThreads)
                s_aux[e][0] = s_aux[e][1] = s_aux[e][2] = s_aux[e][3] = 0.f;
            __syncthreads();
            for (int sl = 0; sl < nslice; sl++) {
                const int cl = (sl * kDwThreads + threadIdx.x) * kCV;
                const bool cok = cl < s.cpg;       // lanes past the group still take part in the reductions
                const int c = g * s.cpg + (cok ? cl : 0);
                for (int kk = 0; kk < kn; kk++) {
                    float wv[kCV] = {0.f, 0.f, 0.f, 0.f};
                    if (cok) ld4<T>(wt + (long)(k0 + kk) * s.Cin + c, wv);
                    float gwv[kCV] = {0.f, 0.f, 0.f, 0.f};
                    for (int p = 0; p < kTP; p++) {
                        const int e = kk * kTP + p;
                        // the table entry is the same for the whole workgroup: keep it in scalar registers
                        const unsigned flag = (unsigned)__builtin_amdgcn_readfirstlane(taps.flag[e]);
                        const unsigned inr = flag >> 8, live = flag & 0xffu;
                        if (!inr) continue;
                        const int idx = __builtin_amdgcn_readfirstlane(taps.idx[e]);
                        const int m = m0 + p;                     // m < M holds where inr != 0
                        float go[kCV] = {0.f, 0.f, 0.f, 0.f};
                        if (cok) ld4<T>(goutcl + (long)m * s.Cout + c, go);
                        float gc[kCV];
#pragma unroll
                        for (int j = 0; j < kCV; j++) gc[j] = wv[j] * go[j];
                        float xv[8][kCV];
#pragma unroll
                        for (int cc = 0; cc < 8; cc++) {
                            const int v = idx + ((cc >> 2) & 1) * HW + ((cc >> 1) & 1) * s.W + (cc & 1);
                            if (((inr >> cc) & 1u) && cok) {
                                ld4<T>(xcl + (long)v * s.Cin + c, xv[cc]);
                            } else {
#pragma unroll
                                for (int j = 0; j < kCV; j++) xv[cc][j] = 0.f;
                            }
                        }
                        float dot[8];
                        float sv[kCV] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int cc = 0; cc < 8; cc++) {
                            float d = 0.f;
#pragma unroll
                            for (int j = 0; j < kCV; j++) d = fmaf(gc[j], xv[cc][j], d);
                            if ((live >> cc) & 1u) {
                                const float wc = taps.w[cc][e];   // a_corner * alpha
#pragma unroll
                                for (int j = 0; j < kCV; j++) sv[j] = fmaf(wc, xv[cc][j], sv[j]);
                                if (a.gxcl && cok) {
                                    const int v = idx + ((cc >> 2) & 1) * HW + ((cc >> 1) & 1) * s.W + (cc & 1);
                                    float *gp = a.gxcl + (long)v * s.Cin + c;
#pragma unroll
                                    for (int j = 0; j < kCV; j++) atomicAdd(gp + j, wc * gc[j]);
                                }
                            }
                            dot[cc] = d;
                        }
#pragma unroll
                        for (int j = 0; j < kCV; j++) gwv[j] = fmaf(go[j], sv[j], gwv[j]);   // sv already holds alpha
                        if (want_aux) {
                            const float lz = taps.frac[0][e], ly = taps.frac[1][e], lx = taps.frac[2][e];
                            const float hz = taps.frac[3][e], hy = taps.frac[4][e], hx = taps.frac[5][e];
                            float gz = 0.f, gy = 0.f, gxx = 0.f, gm = 0.f;
#pragma unroll
                            for (int cc = 0; cc < 8; cc++) {
                                const float wz = (cc & 4) ? hz : lz, wy = (cc & 2) ? hy : ly, wx = (cc & 1) ? hx : lx;
                                const float d = dot[cc];
                                gz += ((cc & 4) ? d : -d) * (wy * wx);
                                gy += ((cc & 2) ? d : -d) * (wz * wx);
                                gxx += ((cc & 1) ? d : -d) * (wz * wy);
                                if ((live >> cc) & 1u) gm += (wz * wy * wx) * d;
                            }
                            const float r = reduce4_over_wave(gz, gy, gxx, gm, lane);
                            if ((lane & 15) == 0) atomicAdd(&s_aux[e][(lane >> 5) * 2 + ((lane >> 4) & 1)], r);
                        }
                    }
                    if (a.gwacc && cok) {
                        float *gw = a.gwacc + (long)(k0 + kk) * s.Cin + c;
#pragma unroll
                        for (int j = 0; j < kCV; j++) atomicAdd(gw + j, gwv[j]);
                    }
                }
            }
            __syncthreads();
            if (want_aux) {
                for (int e = threadIdx.x; e < kn * kTP; e += kDwThreads) {
                    const int p = e % kTP, kk = e / kTP;
                    const int m = m0 + p;
                    if (m >= s.M) continue;
                    const int b = m / s.P, pp = m - b * s.P;
                    const int k = k0 + kk;
                    const float al = taps.alpha[e];
                    if (a.goff) {
                        const long ob = (((long)b * s.G + g) * s.K + k) * 3 * s.P + pp;
                        st_aux(a.goff, ob, s.adt, al * s_aux[e][0]);
                        st_aux(a.goff, ob + s.P, s.adt, al * s_aux[e][1]);
                        st_aux(a.goff, ob + 2 * (long)s.P, s.adt, al * s_aux[e][2]);
                    }
                    if (a.gmask) st_aux(a.gmask, (((long)b * s.G + g) * s.K + k) * s.P + pp, s.adt, s_aux[e][3]);
                }
            }
        }
    }
}

// W[c][0][k] -> wt[k][c]
template <typename T>
__global__ void __launch_bounds__(256) dw_pack_weight_kernel(const T *w, T *wt, int C, int K)
{
    const long n = (long)C * K;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int c = (int)(i % C), k = (int)(i / C);
        wt[i] = w[(long)c * K + k];
    }
}

// gwacc[k][c] (fp32) -> gw[c][0][k]
template <typename T>
__global__ void __launch_bounds__(256) dw_unpack_gw_kernel(const float *gwacc, T *gw, int C, int K)
{
    const long n = (long)C * K;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int k = (int)(i % K), c = (int)(i / K);
        gw[i] = f32_to_elem<T>(gwacc[(long)k * C + c]);
    }
}

inline unsigned g1d(long n)
{
    long g = (n + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 4096 ? 4096 : g));
}

}  // namespace

bool d2c_depthwise_supported(const TiledShape &s)
{
    // a lane's vector of channels must not straddle an offset group
    return s.cg == 1 && s.og == 1 && s.cpg % kCV == 0;
}

template <typename T> int d2c_depthwise_pack_weight(const TiledShape &s, const void *w, void *wt, hipStream_t st)
{
    D2cProfScope prof(D2C_PROF_PACK, st);
    hipLaunchKernelGGL(dw_pack_weight_kernel<T>, dim3(g1d((long)s.Cin * s.K)), dim3(256), 0, st, (const T *)w, (T *)wt,
                       s.Cin, s.K);
    return d2c_check_launch("dw_pack_weight_kernel");
}

template <typename T>
int d2c_depthwise_forward(const TiledShape &s, const void *xcl, const void *off, const void *mask, const void *w,
                          void *wt, const void *bias, void *out, hipStream_t st)
{
    {
        D2cProfScope prof(D2C_PROF_PACK, st);
        hipLaunchKernelGGL(dw_pack_weight_kernel<T>, dim3(g1d((long)s.Cin * s.K)), dim3(256), 0, st, (const T *)w,
                           (T *)wt, s.Cin, s.K);
    }
    DwArgs a{s, xcl, off, mask, wt, bias, out, nullptr, nullptr, nullptr, nullptr, nullptr};
    D2cProfScope prof(D2C_PROF_FWD, st);
    hipLaunchKernelGGL(dw_fwd_kernel<T>, dim3((s.M + kFwdTP - 1) / kFwdTP), dim3(kDwThreads), kDwLdsFwd, st, a);
    return d2c_check_launch("dw_fwd_kernel");
}

// `goutcl` is the channels-last copy of grad_out.  `gxcl` NULL: grad_input is not wanted here (or comes
// from the sample lists afterwards); otherwise it is accumulated with atomics.
template <typename T>
int d2c_depthwise_backward(const TiledShape &s, const void *goutcl, const void *xcl, const void *off, const void *mask,
                           const void *w, void *wt, float *gxcl, void *goff, void *gmask, float *gwacc, void *gw,
                           hipStream_t st)
{
    {
        D2cProfScope prof(D2C_PROF_PACK, st);
        hipLaunchKernelGGL(dw_pack_weight_kernel<T>, dim3(g1d((long)s.Cin * s.K)), dim3(256), 0, st, (const T *)w,
                           (T *)wt, s.Cin, s.K);
        if (gxcl) d2c_fill_zero(gxcl, (size_t)s.N * s.vol * s.Cin * sizeof(float), st);
        if (gwacc) d2c_fill_zero(gwacc, (size_t)s.Cin * s.K * sizeof(float), st);
    }
    DwArgs a{s, xcl, off, mask, wt, nullptr, nullptr, goutcl, gxcl, goff, gmask, gwacc};
    {
        D2cProfScope prof(D2C_PROF_BWD_DATA, st);
        if (hipFuncSetAttribute((const void *)dw_bwd_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)kDwLdsBwd) != hipSuccess)
            return d2c_check_launch("hipFuncSetAttribute(dw_bwd_kernel)");
        hipLaunchKernelGGL(dw_bwd_kernel<T>, dim3((s.M + kBwdTP - 1) / kBwdTP), dim3(kDwThreads), kDwLdsBwd, st, a);
    }
    if (int rc = d2c_check_launch("dw_bwd_kernel")) return rc;
    if (gwacc && gw) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        hipLaunchKernelGGL(dw_unpack_gw_kernel<T>, dim3(g1d((long)s.Cin * s.K)), dim3(256), 0, st, gwacc, (T *)gw,
                           s.Cin, s.K);
        return d2c_check_launch("dw_unpack_gw_kernel");
    }
    return D2C_OK;
}

#define INST(T)                                                                                                      \
    template int d2c_depthwise_pack_weight<T>(const TiledShape &, const void *, void *, hipStream_t);                \
    template int d2c_depthwise_forward<T>(const TiledShape &, const void *, const void *, const void *, const void *, \
                                          void *, const void *, void *, hipStream_t);                                \
    template int d2c_depthwise_backward<T>(const TiledShape &, const void *, const void *, const void *,             \
                                           const void *, const void *, void *, float *, void *, void *, float *,     \
                                           void *, hipStream_t);
INST(bf16_t)
INST(float)
