// Plain depthwise conv3d (one filter per output channel, no sampling): the
// operator of the reference's second extension (ops/fast-depthwise-conv3d,
// csrc/grouped_conv3d.cu), whose kernels take one thread per output element
// and read every input value from memory (:25-92 forward, :97-175 grad_input,
// :178-276 grad_weight with a shared-memory reduction per output channel).
//
// Here the tensors stay NCDHW (W contiguous) and a thread owns kVW consecutive
// elements along W: for 3x3x3 filters with unit stride and dilation along W
// (the backbone's case) an input row segment of kVW + 2 values serves 3 taps of
// kVW outputs, i.e. 13.5 instead of 27 loads per output, all of them coalesced
// along W.  A workgroup works on one (sample, output channel): its 27 weights
// are wavefront-uniform.  Other filter shapes take one element per thread with
// run-time loops.  Sums are float (double for float64 tensors).
//
//   forward     : out[n,co,o]   = bias[co] + sum_k w[co,k] * x[n, co/m, o*s - p + k*d]
//   grad_input  : gx[n,ci,i]    = sum_{co in ci*m..} sum_k w[co,k] * gout[n,co,(i + p - k*d)/s]   (where divisible)
//   grad_weight : gw[co,k]      = sum_{n,o} gout[n,co,o] * x[n, co/m, o*s - p + k*d]   (registers, wavefront and
//                                  workgroup reduction, one atomic per workgroup and tap into a scratch array)
//   grad_bias   : gb[co]        = sum_{n,o} gout[n,co,o]
#include "d2c_common.hpp"

namespace {

constexpr int kVW = 4;         // elements along W per thread (blocked kernels)
constexpr int kThreadsDw = 256;
constexpr int kTX = 16, kTY = 16;   // blocked kernels: a workgroup = kTX groups of kVW elements along W x kTY rows

struct DwcShape {
    d2c_dwconv3d_desc q;
    int mult;       // output channels per input channel
    int K;          // taps
    long P, vol;    // output positions / input voxels per (sample, channel)
};

// storage type -> type of the sums
template <typename ST> struct Acc { typedef float type; };
template <> struct Acc<double> { typedef double type; };
template <typename ST> D2C_DEV typename Acc<ST>::type ldv(const ST *p, long i) { return (typename Acc<ST>::type)p[i]; }
template <> D2C_DEV float ldv<bf16_t>(const bf16_t *p, long i) { return bf16_to_f32(p[i]); }
template <typename ST> D2C_DEV void stv(ST *p, long i, typename Acc<ST>::type v) { p[i] = (ST)v; }
template <> D2C_DEV void stv<bf16_t>(bf16_t *p, long i, float v) { p[i] = f32_to_bf16(v); }

// Tile of a workgroup of the blocked kernels over a volume of `nz` x `ny` rows of `nx4` groups of kVW elements:
// blockIdx.y = (z, tile of rows, tile of groups); the divisions are per workgroup, in scalar registers.
struct Tile2 {
    int z, y, x0;
    bool ok;
};
D2C_DEV Tile2 tile_of(int nz, int ny, int nx4)
{
    const int tx = (nx4 + kTX - 1) / kTX, ty = (ny + kTY - 1) / kTY;
    int b = blockIdx.y;
    const int bx = b % tx; b /= tx;
    const int by = b % ty;
    Tile2 t;
    t.z = b / ty;
    t.y = by * kTY + (int)(threadIdx.x / kTX);
    const int g = bx * kTX + (int)(threadIdx.x % kTX);
    t.x0 = g * kVW;
    t.ok = t.y < ny && g < nx4 && t.z < nz;
    return t;
}
inline unsigned tiles_of(int nz, int ny, int nx4) { return (unsigned)(nz * ((ny + kTY - 1) / kTY) * ((nx4 + kTX - 1) / kTX)); }

// The kVW + 2 values  src[row + first .. row + first + kVW + 1]  of a row of `width` elements, zero outside the row
// or when the row itself is outside the volume (`row_ok` false; `row` is then any row inside the volume).
// VEC: first + 1 is a multiple of kVW, the row is kVW-aligned in memory and `width` a multiple of kVW, so the middle
// kVW values are one vector load (lane-contiguous: a wavefront's request is 1 KiB of whole lines, where scalar
// loads of lanes 16 bytes apart keep the vector-memory path busy four times as long); the two outer values come
// from the neighbouring lanes of the same row (a row of the tile = 16 consecutive lanes = one DPP row), and from
// memory only at the tile's edges.  All lanes of the wavefront must take part.
template <typename ST, bool VEC>
D2C_DEV void row_segment(const ST *src, long row, int first, int width, bool row_ok, typename Acc<ST>::type *v)
{
    typedef typename Acc<ST>::type CT;
    if constexpr (VEC) {
        static_assert(sizeof(CT) == 4 && kVW == 4, "float sums, 4 elements per lane");
        const int x0 = first + 1;
        const bool in = row_ok && x0 < width;       // x0 >= 0 always; whole vector inside when its start is
        float m[4] = {0.f, 0.f, 0.f, 0.f};
        if (in) {
            if constexpr (sizeof(ST) == 4) {
                const float4 t = *reinterpret_cast<const float4 *>(src + row + x0);
                m[0] = t.x; m[1] = t.y; m[2] = t.z; m[3] = t.w;
            } else {
                const uint2 t = *reinterpret_cast<const uint2 *>(src + row + x0);
                m[0] = __uint_as_float(t.x << 16); m[1] = __uint_as_float(t.x & 0xffff0000u);
                m[2] = __uint_as_float(t.y << 16); m[3] = __uint_as_float(t.y & 0xffff0000u);
            }
        }
        // lane i-1's last value / lane i+1's first value; 0 at the ends of the 16-lane row
        float left = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(m[3]), 0x111, 0xF, 0xF, true));   // row_shr 1
        float right = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(m[0]), 0x101, 0xF, 0xF, true));  // row_shl 1
        const int tx = threadIdx.x % kTX;
        if (tx == 0 && in && first >= 0) left = ldv<ST>(src, row + first);
        if (tx == kTX - 1 && row_ok && first + kVW + 1 < width) right = ldv<ST>(src, row + first + kVW + 1);
        v[0] = left; v[1] = m[0]; v[2] = m[1]; v[3] = m[2]; v[4] = m[3]; v[5] = right;
    } else {
#pragma unroll
        for (int i = 0; i < kVW + 2; i++) {
            const int ix = first + i;
            const CT t = ldv<ST>(src, row + min(max(ix, 0), width - 1));
            v[i] = (row_ok && ix >= 0 && ix < width) ? t : (CT)0;
        }
    }
}

// ---------------------------------------------------------------- forward
template <typename ST, int MODE>
__global__ void __launch_bounds__(kThreadsDw) dwc_fwd_kernel(DwcShape s, const ST *x, const ST *w, const ST *bias, ST *out)
{
    typedef typename Acc<ST>::type CT;
    const d2c_dwconv3d_desc &q = s.q;
    const int nc = blockIdx.x, n = nc / q.Cout, co = nc - n * q.Cout, ci = co / s.mult;
    const long xb = ((long)n * q.C + ci) * s.vol, ob = (long)nc * s.P;
    const long wb = (long)co * s.K;
    const CT bv = bias ? ldv<ST>(bias, co) : (CT)0;
    if constexpr (MODE > 0) {
        CT wv[27];
#pragma unroll
        for (int k = 0; k < 27; k++) wv[k] = ldv<ST>(w, wb + k);
        const Tile2 t = tile_of(q.Do, q.Ho, (q.Wo + kVW - 1) / kVW);   // (lanes without an item go along: see row_segment)
        const int oz = t.z, oy = t.y, ox0 = t.x0, ix0 = ox0 - q.pw;
        CT acc[kVW];
#pragma unroll
        for (int i = 0; i < kVW; i++) acc[i] = bv;
        // Every load is made, from an address clamped into the volume, and dropped afterwards if it was outside:
        // without branches around them all 54 loads of a thread are in flight together.
#pragma unroll
        for (int kz = 0; kz < 3; kz++) {
            const int iz = oz * q.sd - q.pd + kz * q.dd;
#pragma unroll
            for (int ky = 0; ky < 3; ky++) {
                const int iy = oy * q.sh - q.ph + ky * q.dh;
                const bool row_ok = t.ok && iz >= 0 && iz < q.D && iy >= 0 && iy < q.H;
                const long rb = xb + ((long)min(max(iz, 0), q.D - 1) * q.H + min(max(iy, 0), q.H - 1)) * q.W;
                CT v[kVW + 2];
                row_segment<ST, MODE == 2>(x, rb, ix0, q.W, row_ok, v);
#pragma unroll
                for (int kx = 0; kx < 3; kx++)
#pragma unroll
                    for (int i = 0; i < kVW; i++) acc[i] = d2c_fma<CT>(wv[(kz * 3 + ky) * 3 + kx], v[i + kx], acc[i]);
            }
        }
        if (!t.ok) return;
        const long o = ob + ((long)oz * q.Ho + oy) * q.Wo + ox0;
#pragma unroll
        for (int i = 0; i < kVW; i++)
            if (ox0 + i < q.Wo) stv<ST>(out, o + i, acc[i]);
    } else {
        for (long it = (long)blockIdx.y * blockDim.x + threadIdx.x; it < s.P; it += (long)gridDim.y * blockDim.x) {
            const int ox = (int)(it % q.Wo), oy = (int)((it / q.Wo) % q.Ho), oz = (int)(it / ((long)q.Wo * q.Ho));
            CT acc = bv;
            for (int kz = 0; kz < q.kd; kz++) {
                const int iz = oz * q.sd - q.pd + kz * q.dd;
                if (iz < 0 || iz >= q.D) continue;
                for (int ky = 0; ky < q.kh; ky++) {
                    const int iy = oy * q.sh - q.ph + ky * q.dh;
                    if (iy < 0 || iy >= q.H) continue;
                    const long rb = xb + ((long)iz * q.H + iy) * q.W;
                    for (int kx = 0; kx < q.kw; kx++) {
                        const int ix = ox * q.sw - q.pw + kx * q.dw;
                        if (ix >= 0 && ix < q.W)
                            acc = d2c_fma<CT>(ldv<ST>(w, wb + (kz * q.kh + ky) * q.kw + kx), ldv<ST>(x, rb + ix), acc);
                    }
                }
            }
            stv<ST>(out, ob + it, acc);
        }
    }
}

// ------------------------------------------------------------- grad_input
// Output position along an axis that tap k of input index i belongs to, or -1.
D2C_DEV int out_index(int i, int p, int k, int d, int s, int n_out)
{
    const int t = i + p - k * d;
    if (t < 0) return -1;
    const int o = t / s;
    return (o * s == t && o < n_out) ? o : -1;
}

template <typename ST, int MODE>
__global__ void __launch_bounds__(kThreadsDw) dwc_bwd_input_kernel(DwcShape s, const ST *gout, const ST *w, ST *gx)
{
    typedef typename Acc<ST>::type CT;
    const d2c_dwconv3d_desc &q = s.q;
    const int nc = blockIdx.x, n = nc / q.C, ci = nc - n * q.C;
    const long xb = (long)nc * s.vol;
    if constexpr (MODE > 0) {
        const Tile2 t = tile_of(q.D, q.H, (q.W + kVW - 1) / kVW);     // (lanes without an item go along: see row_segment)
        const int iz = t.z, iy = t.y, ix0 = t.x0;
        CT acc[kVW];
#pragma unroll
        for (int i = 0; i < kVW; i++) acc[i] = (CT)0;
        for (int m = 0; m < s.mult; m++) {
            const int co = ci * s.mult + m;
            const long gb = ((long)n * q.Cout + co) * s.P, wb = (long)co * 27;
#pragma unroll
            for (int kz = 0; kz < 3; kz++) {
                const int oz = out_index(iz, q.pd, kz, q.dd, q.sd, q.Do);
#pragma unroll
                for (int ky = 0; ky < 3; ky++) {
                    const int oy = out_index(iy, q.ph, ky, q.dh, q.sh, q.Ho);
                    const bool row_ok = t.ok && oz >= 0 && oy >= 0;
                    const long rb = gb + ((long)max(oz, 0) * q.Ho + max(oy, 0)) * q.Wo;
                    // unit stride and dilation along W: ox = ix + pw - kx, so element i of this thread and tap kx
                    // read g[i + 2 - kx] of the segment that starts at ox = ix0 + pw - 2
                    CT g[kVW + 2];
                    row_segment<ST, MODE == 2>(gout, rb, ix0 + q.pw - 2, q.Wo, row_ok, g);
#pragma unroll
                    for (int kx = 0; kx < 3; kx++) {
                        const CT wk = ldv<ST>(w, wb + (kz * 3 + ky) * 3 + kx);
#pragma unroll
                        for (int i = 0; i < kVW; i++) acc[i] = d2c_fma<CT>(wk, g[i + 2 - kx], acc[i]);
                    }
                }
            }
        }
        if (!t.ok) return;
        const long o = xb + ((long)iz * q.H + iy) * q.W + ix0;
#pragma unroll
        for (int i = 0; i < kVW; i++)
            if (ix0 + i < q.W) stv<ST>(gx, o + i, acc[i]);
    } else {
        for (long it = (long)blockIdx.y * blockDim.x + threadIdx.x; it < s.vol; it += (long)gridDim.y * blockDim.x) {
            const int ix = (int)(it % q.W), iy = (int)((it / q.W) % q.H), iz = (int)(it / ((long)q.W * q.H));
            CT acc = (CT)0;
            for (int m = 0; m < s.mult; m++) {
                const int co = ci * s.mult + m;
                const long gb = ((long)n * q.Cout + co) * s.P, wb = (long)co * s.K;
                for (int kz = 0; kz < q.kd; kz++) {
                    const int oz = out_index(iz, q.pd, kz, q.dd, q.sd, q.Do);
                    if (oz < 0) continue;
                    for (int ky = 0; ky < q.kh; ky++) {
                        const int oy = out_index(iy, q.ph, ky, q.dh, q.sh, q.Ho);
                        if (oy < 0) continue;
                        for (int kx = 0; kx < q.kw; kx++) {
                            const int ox = out_index(ix, q.pw, kx, q.dw, q.sw, q.Wo);
                            if (ox >= 0)
                                acc = d2c_fma<CT>(ldv<ST>(w, wb + (kz * q.kh + ky) * q.kw + kx),
                                                  ldv<ST>(gout, gb + ((long)oz * q.Ho + oy) * q.Wo + ox), acc);
                        }
                    }
                }
            }
            stv<ST>(gx, xb + it, acc);
        }
    }
}

// ------------------------------------------------------------ grad_weight
template <typename CT> D2C_DEV CT wave_sum(CT v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// sum of `v` over the workgroup, added to *dst by one thread
template <typename CT> D2C_DEV void block_add(CT v, CT *dst, CT *s_red)
{
    v = wave_sum<CT>(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) s_red[wave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        CT t = (CT)0;
        for (int i = 0; i < kThreadsDw / 64; i++) t += s_red[i];
        atomicAdd(dst, t);
    }
}

// grid = (output channels, shares of the (sample, position) items); gwacc[co][k] and gbacc[co] zeroed beforehand.
// The bias gradient is the sum of the grad_out values that pass through here anyway (gbacc may be NULL).
template <typename ST, int MODE>
__global__ void __launch_bounds__(kThreadsDw) dwc_bwd_weight_kernel(DwcShape s, const ST *gout, const ST *x,
                                                                    typename Acc<ST>::type *gwacc,
                                                                    typename Acc<ST>::type *gbacc)
{
    typedef typename Acc<ST>::type CT;
    __shared__ CT s_red[kThreadsDw / 64];
    const d2c_dwconv3d_desc &q = s.q;
    const int co = blockIdx.x, ci = co / s.mult;
    CT gsum = (CT)0;
    if constexpr (MODE > 0) {
        CT acc[27];
#pragma unroll
        for (int k = 0; k < 27; k++) acc[k] = (CT)0;
        const int wo4 = (q.Wo + kVW - 1) / kVW;
        // items = (sample, z, row); a thread walks the groups of a row, so that no division is in the inner loop
        const int rows = q.N * q.Do * q.Ho;     // < 2^30 (d2c_dwconv3d_check)
        const int tx = threadIdx.x % kTX, ty = threadIdx.x / kTX;
        for (int row = (int)blockIdx.y * kTY + ty; row < rows; row += (int)gridDim.y * kTY) {
            const int oy = row % q.Ho, oz = (row / q.Ho) % q.Do, n = row / (q.Ho * q.Do);
            const long xb = ((long)n * q.C + ci) * s.vol;
            const long grow = ((long)n * q.Cout + co) * s.P + ((long)oz * q.Ho + oy) * q.Wo;
            for (int g0 = 0; g0 < wo4; g0 += kTX) {       // the 16 lanes of a row stay together (see row_segment)
                const int g4 = g0 + tx;
                const int ox0 = g4 * kVW, ix0 = ox0 - q.pw;
                CT g[kVW];
                if constexpr (MODE == 2) {
                    // (Wo is a multiple of kVW here: a group is inside the row or past it as a whole)
                    float m[4] = {0.f, 0.f, 0.f, 0.f};
                    if (ox0 < q.Wo) {
                        if constexpr (sizeof(ST) == 4) {
                            const float4 t = *reinterpret_cast<const float4 *>(gout + grow + ox0);
                            m[0] = t.x; m[1] = t.y; m[2] = t.z; m[3] = t.w;
                        } else {
                            const uint2 t = *reinterpret_cast<const uint2 *>(gout + grow + ox0);
                            m[0] = __uint_as_float(t.x << 16); m[1] = __uint_as_float(t.x & 0xffff0000u);
                            m[2] = __uint_as_float(t.y << 16); m[3] = __uint_as_float(t.y & 0xffff0000u);
                        }
                    }
#pragma unroll
                    for (int i = 0; i < kVW; i++) g[i] = (CT)m[i];
                } else {
#pragma unroll
                    for (int i = 0; i < kVW; i++) g[i] = ox0 + i < q.Wo ? ldv<ST>(gout, grow + ox0 + i) : (CT)0;
                }
#pragma unroll
                for (int i = 0; i < kVW; i++) gsum += g[i];
#pragma unroll
                for (int kz = 0; kz < 3; kz++) {
                    const int iz = oz * q.sd - q.pd + kz * q.dd;
#pragma unroll
                    for (int ky = 0; ky < 3; ky++) {
                        const int iy = oy * q.sh - q.ph + ky * q.dh;
                        const bool row_ok = iz >= 0 && iz < q.D && iy >= 0 && iy < q.H;
                        const long rb = xb + ((long)min(max(iz, 0), q.D - 1) * q.H + min(max(iy, 0), q.H - 1)) * q.W;
                        CT v[kVW + 2];
                        row_segment<ST, MODE == 2>(x, rb, ix0, q.W, row_ok, v);
#pragma unroll
                        for (int kx = 0; kx < 3; kx++)
#pragma unroll
                            for (int i = 0; i < kVW; i++)
                                acc[(kz * 3 + ky) * 3 + kx] = d2c_fma<CT>(g[i], v[i + kx], acc[(kz * 3 + ky) * 3 + kx]);
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < 27; k++) block_add<CT>(acc[k], gwacc + (long)co * 27 + k, s_red);
    } else {
        const long items = s.P * q.N;
        for (int k = 0; k < s.K; k++) {
            const int kx = k % q.kw, ky = (k / q.kw) % q.kh, kz = k / (q.kw * q.kh);
            CT acc = (CT)0;
            for (long it = (long)blockIdx.y * blockDim.x + threadIdx.x; it < items; it += (long)gridDim.y * blockDim.x) {
                const int n = (int)(it / s.P);
                const long r = it - (long)n * s.P;
                const int ox = (int)(r % q.Wo), oy = (int)((r / q.Wo) % q.Ho), oz = (int)(r / ((long)q.Wo * q.Ho));
                const int iz = oz * q.sd - q.pd + kz * q.dd, iy = oy * q.sh - q.ph + ky * q.dh,
                          ix = ox * q.sw - q.pw + kx * q.dw;
                const CT gv = ldv<ST>(gout, ((long)n * q.Cout + co) * s.P + r);
                if (k == 0) gsum += gv;
                if (iz >= 0 && iz < q.D && iy >= 0 && iy < q.H && ix >= 0 && ix < q.W)
                    acc = d2c_fma<CT>(gv, ldv<ST>(x, ((long)n * q.C + ci) * s.vol + ((long)iz * q.H + iy) * q.W + ix), acc);
            }
            block_add<CT>(acc, gwacc + (long)co * s.K + k, s_red);
        }
    }
    if (gbacc) block_add<CT>(gsum, gbacc + co, s_red);
}

template <typename ST>
__global__ void __launch_bounds__(256) dwc_cvt_kernel(const typename Acc<ST>::type *src, ST *dst, long n)
{
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        stv<ST>(dst, i, src[i]);
}

// grad_bias alone (grad_weight not wanted): shares of the positions per output channel, partial sums added to gbacc
template <typename ST>
__global__ void __launch_bounds__(kThreadsDw) dwc_bias_grad_kernel(DwcShape s, const ST *gout,
                                                                   typename Acc<ST>::type *gbacc)
{
    typedef typename Acc<ST>::type CT;
    __shared__ CT s_red[kThreadsDw / 64];
    const d2c_dwconv3d_desc &q = s.q;
    const int co = blockIdx.x;
    CT acc = (CT)0;
    const long items = s.P * q.N;
    for (long it = (long)blockIdx.y * blockDim.x + threadIdx.x; it < items; it += (long)gridDim.y * blockDim.x) {
        const long n = it / s.P, r = it - n * s.P;
        acc += ldv<ST>(gout, (n * q.Cout + co) * s.P + r);
    }
    block_add<CT>(acc, gbacc + co, s_red);
}

DwcShape make_shape(const d2c_dwconv3d_desc &q)
{
    DwcShape s;
    s.q = q;
    s.mult = q.Cout / q.C;
    s.K = q.kd * q.kh * q.kw;
    s.P = (long)q.Do * q.Ho * q.Wo;
    s.vol = (long)q.D * q.H * q.W;
    return s;
}

bool host_blocked(const d2c_dwconv3d_desc &q) { return q.kd == 3 && q.kh == 3 && q.kw == 3 && q.sw == 1 && q.dw == 1; }

unsigned blocks_for(long items, long cap)
{
    long g = (items + kThreadsDw - 1) / kThreadsDw;
    return (unsigned)(g < 1 ? 1 : (g > cap ? cap : g));
}

// vector loads of kVW elements: rows that start kVW-aligned in memory, segments that start one element left of a
// multiple of kVW (padding 1 along W)
template <typename ST> bool vec_ok(const d2c_dwconv3d_desc &q, const void *a, const void *b)
{
    const uintptr_t al = kVW * sizeof(ST);
    return sizeof(ST) <= 4 && q.pw == 1 && q.W % kVW == 0 && q.Wo == q.W && reinterpret_cast<uintptr_t>(a) % al == 0 &&
           (b == nullptr || reinterpret_cast<uintptr_t>(b) % al == 0);
}

template <typename ST>
int forward_t(const d2c_dwconv3d_desc &q, const void *x, const void *w, const void *bias, void *out, hipStream_t st)
{
    const DwcShape s = make_shape(q);
    const unsigned nc = (unsigned)(q.N * q.Cout);
    const dim3 tiles(nc, tiles_of(q.Do, q.Ho, (q.Wo + kVW - 1) / kVW));
    bool done = false;
    if constexpr (sizeof(ST) <= 4) {
        if (host_blocked(q) && vec_ok<ST>(q, x, nullptr)) {
            hipLaunchKernelGGL((dwc_fwd_kernel<ST, 2>), tiles, dim3(kThreadsDw), 0, st, s, (const ST *)x, (const ST *)w,
                               (const ST *)bias, (ST *)out);
            done = true;
        }
    }
    if (!done) {
        if (host_blocked(q))
            hipLaunchKernelGGL((dwc_fwd_kernel<ST, 1>), tiles, dim3(kThreadsDw), 0, st, s, (const ST *)x, (const ST *)w,
                               (const ST *)bias, (ST *)out);
        else
            hipLaunchKernelGGL((dwc_fwd_kernel<ST, 0>), dim3(nc, blocks_for(s.P, 4096)), dim3(kThreadsDw), 0, st, s,
                               (const ST *)x, (const ST *)w, (const ST *)bias, (ST *)out);
    }
    return d2c_check_launch("dwc_fwd_kernel");
}

template <typename ST>
int backward_t(const d2c_dwconv3d_desc &q, const void *gout, const void *x, const void *w, void *gx, void *gw, void *gb,
               void *ws, hipStream_t st)
{
    typedef typename Acc<ST>::type CT;
    const DwcShape s = make_shape(q);
    const bool blocked = host_blocked(q);
    if (gx) {
        const unsigned nc = (unsigned)(q.N * q.C);
        const dim3 tiles(nc, tiles_of(q.D, q.H, (q.W + kVW - 1) / kVW));
        bool done = false;
        if constexpr (sizeof(ST) <= 4) {
            if (blocked && vec_ok<ST>(q, gout, nullptr)) {
                hipLaunchKernelGGL((dwc_bwd_input_kernel<ST, 2>), tiles, dim3(kThreadsDw), 0, st, s, (const ST *)gout,
                                   (const ST *)w, (ST *)gx);
                done = true;
            }
        }
        if (!done) {
            if (blocked)
                hipLaunchKernelGGL((dwc_bwd_input_kernel<ST, 1>), tiles, dim3(kThreadsDw), 0, st, s, (const ST *)gout,
                                   (const ST *)w, (ST *)gx);
            else
                hipLaunchKernelGGL((dwc_bwd_input_kernel<ST, 0>), dim3(nc, blocks_for(s.vol, 4096)), dim3(kThreadsDw), 0,
                                   st, s, (const ST *)gout, (const ST *)w, (ST *)gx);
        }
        if (int rc = d2c_check_launch("dwc_bwd_input_kernel")) return rc;
    }
    if (!gw && !gb) return D2C_OK;
    // scratch: gwacc [Cout][K], then gbacc [Cout]
    const long nw = (long)q.Cout * s.K;
    CT *gwacc = reinterpret_cast<CT *>(ws), *gbacc = gwacc + nw;
    d2c_fill_zero(gwacc, (size_t)(nw + q.Cout) * sizeof(CT), st);
    // shares of the work per output channel: enough workgroups to fill the chip, each with some work
    const long work = blocked ? (long)q.N * q.Do * q.Ho / kTY : (long)q.N * s.P / (4 * kThreadsDw);
    long shares = (2048 + q.Cout - 1) / q.Cout;
    if (shares > work) shares = work;
    if (shares < 1) shares = 1;
    if (shares > 4096) shares = 4096;
    const dim3 grid((unsigned)q.Cout, (unsigned)shares);
    if (gw) {
        bool done = false;
        if constexpr (sizeof(ST) <= 4) {
            if (blocked && vec_ok<ST>(q, x, gout)) {
                hipLaunchKernelGGL((dwc_bwd_weight_kernel<ST, 2>), grid, dim3(kThreadsDw), 0, st, s, (const ST *)gout,
                                   (const ST *)x, gwacc, gb ? gbacc : nullptr);
                done = true;
            }
        }
        if (!done) {
            if (blocked)
                hipLaunchKernelGGL((dwc_bwd_weight_kernel<ST, 1>), grid, dim3(kThreadsDw), 0, st, s, (const ST *)gout,
                                   (const ST *)x, gwacc, gb ? gbacc : nullptr);
            else
                hipLaunchKernelGGL((dwc_bwd_weight_kernel<ST, 0>), grid, dim3(kThreadsDw), 0, st, s, (const ST *)gout,
                                   (const ST *)x, gwacc, gb ? gbacc : nullptr);
        }
        if (int rc = d2c_check_launch("dwc_bwd_weight_kernel")) return rc;
        hipLaunchKernelGGL(dwc_cvt_kernel<ST>, dim3(blocks_for(nw, 1024)), dim3(256), 0, st, gwacc, (ST *)gw, nw);
    } else {
        hipLaunchKernelGGL(dwc_bias_grad_kernel<ST>, grid, dim3(kThreadsDw), 0, st, s, (const ST *)gout, gbacc);
        if (int rc = d2c_check_launch("dwc_bias_grad_kernel")) return rc;
    }
    if (gb) hipLaunchKernelGGL(dwc_cvt_kernel<ST>, dim3(blocks_for(q.Cout, 1024)), dim3(256), 0, st, gbacc, (ST *)gb, (long)q.Cout);
    return d2c_check_launch("dwc_cvt_kernel");
}

template <typename F32, typename F64, typename B16> int by_dtype(int dt, F32 f32, F64 f64, B16 b16)
{
    return dt == D2C_F64 ? f64() : (dt == D2C_F32 ? f32() : b16());
}

}  // namespace

extern "C" {

int d2c_dwconv3d_check(const d2c_dwconv3d_desc *q)
{
    if (!q) { d2c_set_error("null description"); return D2C_ERR_SHAPE; }
    if (q->dtype != D2C_F32 && q->dtype != D2C_F64 && q->dtype != D2C_BF16) {
        d2c_set_error("unsupported dtype %d", q->dtype);
        return D2C_ERR_DTYPE;
    }
    if (q->N < 1 || q->C < 1 || q->Cout < 1 || q->D < 1 || q->H < 1 || q->W < 1) {
        d2c_set_error("tensor sizes must be positive");
        return D2C_ERR_SHAPE;
    }
    if (q->Cout % q->C != 0) {   // grouped_conv3d.cu:306-309
        d2c_set_error("Depthwise out channels should be a multiple of in channels, got %d and %d", q->Cout, q->C);
        return D2C_ERR_SHAPE;
    }
    const int k[3] = {q->kd, q->kh, q->kw}, s[3] = {q->sd, q->sh, q->sw}, p[3] = {q->pd, q->ph, q->pw},
              d[3] = {q->dd, q->dh, q->dw}, in[3] = {q->D, q->H, q->W}, out[3] = {q->Do, q->Ho, q->Wo};
    for (int i = 0; i < 3; i++) {
        if (k[i] < 1) { d2c_set_error("kernel size should be at least 1"); return D2C_ERR_SHAPE; }
        if (s[i] < 1) { d2c_set_error("stride should be at least 1, got %d", s[i]); return D2C_ERR_SHAPE; }          // :314
        if (p[i] < 0) { d2c_set_error("padding should be non-negative, got %d", p[i]); return D2C_ERR_SHAPE; }      // :316
        if (d[i] < 1) { d2c_set_error("dilation should be at least 1, got %d", d[i]); return D2C_ERR_SHAPE; }       // :318
        const int span = in[i] + 2 * p[i] - (d[i] * (k[i] - 1) + 1);
        const int want = span >= 0 ? span / s[i] + 1 : 0;
        if (want < 1) { d2c_set_error("Output size should be positive, got %d at dim %d", want, i + 2); return D2C_ERR_SHAPE; }   // :409
        if (out[i] != want) {
            d2c_set_error("output size %d at dim %d does not match the computed size %d", out[i], i + 2, want);
            return D2C_ERR_SHAPE;
        }
    }
    const long lim = 1L << 31;   // 32-bit indices inside a (sample, channel) volume and over the grid
    if ((long)q->D * q->H * q->W >= lim || (long)q->Do * q->Ho * q->Wo >= lim || (long)q->N * q->Cout >= lim ||
        (long)q->N * q->C >= lim || (long)q->N * q->Do * q->Ho >= lim / 2) {
        d2c_set_error("tensor too large for 32-bit indices");
        return D2C_ERR_UNSUPPORTED;
    }
    // one workgroup per 16 rows x 64 elements of a (sample, channel) volume, counted in the grid's y extent
    const long tiles_in = (long)q->D * ((q->H + 15) / 16) * ((q->W + 63) / 64);
    const long tiles_out = (long)q->Do * ((q->Ho + 15) / 16) * ((q->Wo + 63) / 64);
    if (tiles_in > 65535 || tiles_out > 65535) {
        d2c_set_error("volume too large for the launch grid (%ld tiles per channel)", tiles_in > tiles_out ? tiles_in : tiles_out);
        return D2C_ERR_UNSUPPORTED;
    }
    return D2C_OK;
}

size_t d2c_dwconv3d_backward_workspace_bytes(const d2c_dwconv3d_desc *q)
{
    if (d2c_dwconv3d_check(q) != D2C_OK) return 0;
    return d2c_align_up((size_t)q->Cout * (q->kd * q->kh * q->kw + 1) * (q->dtype == D2C_F64 ? 8 : 4));
}

int d2c_dwconv3d_forward(const d2c_dwconv3d_desc *q, const void *x, const void *weight, const void *bias, void *out,
                         void *stream)
{
    if (int rc = d2c_dwconv3d_check(q)) return rc;
    if (!x || !weight || !out) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    hipStream_t st = (hipStream_t)stream;
    return by_dtype(q->dtype, [&] { return forward_t<float>(*q, x, weight, bias, out, st); },
                    [&] { return forward_t<double>(*q, x, weight, bias, out, st); },
                    [&] { return forward_t<bf16_t>(*q, x, weight, bias, out, st); });
}

int d2c_dwconv3d_backward(const d2c_dwconv3d_desc *q, const void *grad_out, const void *x, const void *weight,
                          void *grad_x, void *grad_weight, void *grad_bias, void *workspace, size_t workspace_bytes,
                          void *stream)
{
    if (int rc = d2c_dwconv3d_check(q)) return rc;
    if (!grad_out || !x || !weight) { d2c_set_error("null tensor pointer"); return D2C_ERR_SHAPE; }
    if (grad_weight || grad_bias) {
        const size_t need = d2c_dwconv3d_backward_workspace_bytes(q);
        if (!workspace || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 256 != 0) {
            d2c_set_error("workspace of %zu bytes (256-byte aligned) needed, got %zu", need, workspace_bytes);
            return D2C_ERR_WORKSPACE;
        }
    }
    hipStream_t st = (hipStream_t)stream;
    return by_dtype(
        q->dtype, [&] { return backward_t<float>(*q, grad_out, x, weight, grad_x, grad_weight, grad_bias, workspace, st); },
        [&] { return backward_t<double>(*q, grad_out, x, weight, grad_x, grad_weight, grad_bias, workspace, st); },
        [&] { return backward_t<bf16_t>(*q, grad_out, x, weight, grad_x, grad_weight, grad_bias, workspace, st); });
}

}  // extern "C"
