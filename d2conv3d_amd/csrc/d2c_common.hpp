// Shared host/device helpers of the D2Conv3D kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/d2conv.h"

#define D2C_DEV __device__ __forceinline__

typedef unsigned short bf16_t;  // raw bfloat16 bits

// ---- bfloat16 <-> float (round to nearest even, NaN kept quiet) -------------
D2C_DEV float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }
D2C_DEV bf16_t f32_to_bf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

// ---- element access with a run-time element type ---------------------------
// The direct ("generic") kernels serve f32, f64 and bf16 storage from one
// instantiation per compute type; the branch is uniform over the grid.
template <typename CT>
D2C_DEV CT ld_as(const void *p, long i, int dt)
{
    if (dt == D2C_F32) return (CT) reinterpret_cast<const float *>(p)[i];
    if (dt == D2C_F64) return (CT) reinterpret_cast<const double *>(p)[i];
    return (CT)bf16_to_f32(reinterpret_cast<const bf16_t *>(p)[i]);
}
template <typename CT>
D2C_DEV void st_as(void *p, long i, int dt, CT v)
{
    if (dt == D2C_F32) reinterpret_cast<float *>(p)[i] = (float)v;
    else if (dt == D2C_F64) reinterpret_cast<double *>(p)[i] = (double)v;
    else reinterpret_cast<bf16_t *>(p)[i] = f32_to_bf16((float)v);
}
static inline size_t d2c_elem_size(int dt) { return dt == D2C_F64 ? 8 : (dt == D2C_F32 ? 4 : 2); }

template <typename CT> D2C_DEV CT d2c_floor(CT v);
template <> D2C_DEV float d2c_floor<float>(float v) { return floorf(v); }
template <> D2C_DEV double d2c_floor<double>(double v) { return floor(v); }
template <typename CT> D2C_DEV CT d2c_fma(CT a, CT b, CT c);
template <> D2C_DEV float d2c_fma<float>(float a, float b, float c) { return fmaf(a, b, c); }
template <> D2C_DEV double d2c_fma<double>(double a, double b, double c) { return fma(a, b, c); }

// ---- one sampling position --------------------------------------------------
// Bookkeeping of trilinear_interpolate (dconv3d_gpu.cu:48-109) and
// get_coordinate_weights (:708-754) for one (tap, output position).
template <typename CT>
struct Tap3 {
    int z0, y0, x0;   // floor of the position
    CT lz, ly, lx;    // weight of the low corner per axis:  (z1 - z)
    CT hz, hy, hx;    // weight of the high corner per axis: (z - z0)
    unsigned live;    // bit c (c = 4*dz+2*dy+dx): corner read by the forward pass
    unsigned inrange; // bit c: corner index inside the volume (no early-out), used by d/d(offset)
};

// Position = float(int base) + offset: the integer part is formed in int and
// converted once, so floor() and the range tests see the same bits as the
// reference (dconv3d_gpu.cu:192-194).
template <typename CT>
D2C_DEV Tap3<CT> make_tap3(int bz, int by, int bx, CT oz, CT oy, CT ox, int D, int H, int W)
{
    Tap3<CT> t;
    const CT z = (CT)bz + oz, y = (CT)by + oy, x = (CT)bx + ox;
    const bool out = (z <= (CT)-1) || ((CT)D <= z) || (y <= (CT)-1) || ((CT)H <= y) || (x <= (CT)-1) || ((CT)W <= x);
    // clamp before the float->int conversion so that huge or non-finite
    // positions give defined integers; such taps have no corner in range.
    const CT zc = z < (CT)-4 ? (CT)-4 : (z > (CT)(D + 4) ? (CT)(D + 4) : z);
    const CT yc = y < (CT)-4 ? (CT)-4 : (y > (CT)(H + 4) ? (CT)(H + 4) : y);
    const CT xc = x < (CT)-4 ? (CT)-4 : (x > (CT)(W + 4) ? (CT)(W + 4) : x);
    const bool finite = (z == z) && (y == y) && (x == x);
    t.z0 = finite ? (int)d2c_floor<CT>(zc) : -4;
    t.y0 = finite ? (int)d2c_floor<CT>(yc) : -4;
    t.x0 = finite ? (int)d2c_floor<CT>(xc) : -4;
    const int z1 = t.z0 + 1, y1 = t.y0 + 1, x1 = t.x0 + 1;
    t.lz = (CT)z1 - z; t.hz = z - (CT)t.z0;
    t.ly = (CT)y1 - y; t.hy = y - (CT)t.y0;
    t.lx = (CT)x1 - x; t.hx = x - (CT)t.x0;
    const unsigned vz0 = (t.z0 >= 0 && t.z0 < D), vz1 = (z1 >= 0 && z1 < D);
    const unsigned vy0 = (t.y0 >= 0 && t.y0 < H), vy1 = (y1 >= 0 && y1 < H);
    const unsigned vx0 = (t.x0 >= 0 && t.x0 < W), vx1 = (x1 >= 0 && x1 < W);
    const unsigned mz = vz0 * 0x0Fu | vz1 * 0xF0u;
    const unsigned my = vy0 * 0x33u | vy1 * 0xCCu;
    const unsigned mx = vx0 * 0x55u | vx1 * 0xAAu;
    t.inrange = finite ? (mz & my & mx) : 0u;
    t.live = out ? 0u : t.inrange;
    return t;
}

// Corner weight a_c of the forward pass, products left to right as in
// dconv3d_gpu.cu:88-95.
template <typename CT>
D2C_DEV CT tap3_weight(const Tap3<CT> &t, int c)
{
    const CT wz = (c & 4) ? t.hz : t.lz;
    const CT wy = (c & 2) ? t.hy : t.ly;
    const CT wx = (c & 1) ? t.hx : t.lx;
    return wz * wy * wx;
}

// Decompose a flat tap index into (i, j, l) and return the integer base
// position of output voxel (oz, oy, ox).
struct TapGeom {
    int kd, kh, kw, sd, sh, sw, pd, ph, pw, dd, dh, dw;
};
D2C_DEV void tap_base(const TapGeom &g, int k, int oz, int oy, int ox, int &bz, int &by, int &bx)
{
    const int l = k % g.kw, j = (k / g.kw) % g.kh, i = k / (g.kw * g.kh);
    bz = oz * g.sd - g.pd + i * g.dd;
    by = oy * g.sh - g.ph + j * g.dh;
    bx = ox * g.sw - g.pw + l * g.dw;
}
static inline TapGeom make_geom(const d2c_conv3d_desc &q)
{
    TapGeom g{q.kd, q.kh, q.kw, q.sd, q.sh, q.sw, q.pd, q.ph, q.pw, q.dd, q.dh, q.dw};
    return g;
}

// ---- host side ---------------------------------------------------------------
void d2c_set_error(const char *fmt, ...);
int d2c_check_launch(const char *what);

// Compute units of the current device (persistent kernels launch one workgroup each); 0 if the query fails,
// with the error text set.
int d2c_num_cus();

// Clears `bytes` (a multiple of 4) with a fill kernel; safe to record into a HIP graph.
void d2c_fill_zero(void *p, size_t bytes, hipStream_t st);

// Event bracket around a kernel launch when instrumentation is on (see d2c_profile_enable).
// `name` (a string literal): the kernel launched inside the bracket, reported by d2c_profile_kernel_name().
void d2c_prof_begin(int id, hipStream_t st, const char *name = nullptr);
void d2c_prof_end(int id, hipStream_t st);
struct D2cProfScope {
    int id; hipStream_t st;
    D2cProfScope(int i, hipStream_t s, const char *name = nullptr) : id(i), st(s) { d2c_prof_begin(id, st, name); }
    ~D2cProfScope() { d2c_prof_end(id, st); }
};

// Raises a kernel's dynamic-LDS limit (hipFuncAttributeMaxDynamicSharedMemorySize); the runtime is asked once
// per (kernel, device), later calls only look the pair up.  Returns D2C_OK or D2C_ERR_LAUNCH with the error text set.
int d2c_allow_lds(const void *kernel, int bytes, const char *what);

static inline size_t d2c_align_up(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }

// Kernel families (defined in their own translation units).
int d2c_generic_conv3d_forward(const d2c_conv3d_desc &q, const void *x, const void *off, const void *mask,
                               const void *w, const void *bias, void *out, hipStream_t st);
size_t d2c_generic_conv3d_backward_ws(const d2c_conv3d_desc &q);
int d2c_generic_conv3d_backward(const d2c_conv3d_desc &q, const void *gout, const void *x, const void *off,
                                const void *mask, const void *w, void *gx, void *goff, void *gmask, void *gw,
                                void *gb, void *ws, hipStream_t st);
int d2c_generic_conv3d_corners(const d2c_conv3d_desc &q, const void *off, int32_t *base, uint8_t *flags,
                               hipStream_t st);
int d2c_generic_conv3d_sample(const d2c_conv3d_desc &q, int Cs, const void *src, const void *off, void *out,
                              hipStream_t st);
int d2c_generic_conv3d_offset_hist(const d2c_conv3d_desc &q, const void *off, float lo, float hi, int nbins,
                                   unsigned long long *hist, hipStream_t st);
int d2c_generic_conv1d_forward(const d2c_conv1d_desc &q, const void *x, const void *off, const void *mask,
                               const void *w, const void *bias, void *out, hipStream_t st);
size_t d2c_generic_conv1d_backward_ws(const d2c_conv1d_desc &q);
int d2c_generic_conv1d_backward(const d2c_conv1d_desc &q, const void *gout, const void *x, const void *off,
                                const void *mask, const void *w, void *gx, void *goff, void *gmask, void *gw,
                                void *gb, void *ws, hipStream_t st);
