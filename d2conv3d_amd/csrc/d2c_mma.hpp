// Matrix-core building blocks shared by the tiled kernels (gfx950, wave64).
//
// All operands move in 16-byte vectors: VEC = 8 bfloat16 or 4 float channels.
// A "k-group" is two such vectors (lane half h = lane / 32 takes vector
// 2*kg + h): 16 bf16 channels = one v_mfma_f32_32x32x16_bf16, or 8 float
// channels = four v_mfma_f32_32x32x2_f32 (element i of both operands' vectors
// feeds MFMA i, so the channel permutation is the same on both sides and the
// sum is unchanged).
//
// Fragment layout of the 32x32 MFMAs (A is M x K, B is K x N, D is M x N):
//   A: lane l holds row  m = l % 32, its k-slice chosen by l / 32
//   B: lane l holds col  n = l % 32, same k-slice
//   D: lane l holds col  n = l % 32, rows m = 8*(r/4) + 4*(l/32) + r%4 for r = 0..15
#pragma once
#include <type_traits>
#include "d2c_common.hpp"

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

template <typename T> struct Elem;
template <> struct Elem<bf16_t> {
    static constexpr int VEC = 8;          // channels per 16-byte vector
    static constexpr int DT = D2C_BF16;
};
template <> struct Elem<float> {
    static constexpr int VEC = 4;
    static constexpr int DT = D2C_F32;
};

// Two floats -> packed bfloat16 pair (round to nearest even), low half first.
D2C_DEV uint32_t pack_bf16x2(float lo, float hi)
{
    f32x2 v = {lo, hi};
    bf16x2_t r = __builtin_convertvector(v, bf16x2_t);
    return __builtin_bit_cast(uint32_t, r);
}

// ---- float problems on the bfloat16 matrix instruction ---------------------------------------------------------
// The float MFMA (v_mfma_f32_32x32x2_f32) runs at 1/16 of the bfloat16 rate.  In the FORWARD kernels a float MFMA
// operand therefore travels as TWO bfloat16 values per element, v ~ hi + lo with hi = bf16(v) and lo = bf16(v - hi)
// (what is left is below 2^-16 |v|), in the 16 bytes that its four floats would take:
// (hi0, hi1) (hi2, hi3) (lo0, lo1) (lo2, lo3).  One k-group (8 channels: 4 per lane half) is then two
// v_mfma_f32_32x32x16_bf16 whose 16-deep reductions hold all four partial products of every element,
// (hi + lo) * (hi' + lo'), summed in float32 by the matrix core: a quarter of the matrix-pipe time of the four float
// instructions.  The producers of the forward operands (weight re-layout, sampled tile) write this form.
// In the BACKWARD pass the grad-column product takes two-term operands as well (TiledShape::f32split == 2, the
// default); the grad-weight kernel that samples again and the 1-D / fallback data kernel keep plain floats and the
// float instruction: the relative error of 4e-6 that two-term operands leave in a long sum is fine for the output
// and for grad_input (values of order 1 against 1e-4 relative / 1e-5 absolute) but not for gradients whose elements
// reach 20 .. 400 and are held to the same absolute 1e-5.  A caller who prefers the speed asks for split operands
// there too (D2C_BWD_F32_SPLIT in the description's backward_flags: f32split == 1, a template parameter of the
// backward kernels).  The grad-weight product over sampled columns is neither: it takes every float apart into THREE
// bfloat16 terms, which represent it exactly, and keeps float32's accuracy on the bfloat16 instruction
// (tiled_bwd_weight_col3_kernel in d2c_tiled_bwd.hip).  -DD2C_F32_NATIVE_MFMA keeps the forward kernels and the
// grad-column product on the float instruction.
#ifdef D2C_F32_NATIVE_MFMA
constexpr bool kF32SplitFwd = false;
#else
constexpr bool kF32SplitFwd = true;
#endif
D2C_DEV float bf16_residual(float v, uint32_t hi_bits)
{
    const float h = __uint_as_float(hi_bits);
    // (an infinite value keeps its infinity in `hi` alone)
    return (__float_as_uint(h) & 0x7fffffffu) == 0x7f800000u ? 0.f : v - h;
}
D2C_DEV uint4 split_f32x4(float v0, float v1, float v2, float v3)
{
    const uint32_t h01 = pack_bf16x2(v0, v1), h23 = pack_bf16x2(v2, v3);
    return make_uint4(h01, h23,
                      pack_bf16x2(bf16_residual(v0, h01 << 16), bf16_residual(v1, h01 & 0xffff0000u)),
                      pack_bf16x2(bf16_residual(v2, h23 << 16), bf16_residual(v3, h23 & 0xffff0000u)));
}
// VEC consecutive reduction elements as the 16-byte operand vector the matrix instructions take
// (SPLIT: float elements as two bfloat16 halves)
template <typename T, bool SPLIT> D2C_DEV uint4 operand_vec(const T *e)
{
    if constexpr (sizeof(T) == 2) {
        return make_uint4(e[0] | ((uint32_t)e[1] << 16), e[2] | ((uint32_t)e[3] << 16), e[4] | ((uint32_t)e[5] << 16),
                          e[6] | ((uint32_t)e[7] << 16));
    } else if constexpr (SPLIT) {
        return split_f32x4(e[0], e[1], e[2], e[3]);
    } else {
        return make_uint4(__float_as_uint(e[0]), __float_as_uint(e[1]), __float_as_uint(e[2]), __float_as_uint(e[3]));
    }
}
// ... of a vector already loaded as 16 bytes of T
template <typename T, bool SPLIT> D2C_DEV uint4 operand_vec16(const uint4 &v)
{
    if constexpr (sizeof(T) == 4 && SPLIT)
        return split_f32x4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
    else return v;
}

// One k-group of the reduction: acc += A (32 rows x 16 / 8 channels) * B (those channels x 32 columns)
template <typename T, bool SPLIT> D2C_DEV void mma_kgroup(f32x16 &acc, const uint4 &a, const uint4 &b)
{
    if constexpr (sizeof(T) == 2) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                      acc, 0, 0, 0);
    } else if constexpr (SPLIT) {
        const uint4 bh = make_uint4(b.x, b.y, b.x, b.y), bl = make_uint4(b.z, b.w, b.z, b.w);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, bh),
                                                      acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, bl),
                                                      acc, 0, 0, 0);
    } else {
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), acc, 0, 0, 0);
    }
}

// acc[i] += w * v[i] over one 16-byte vector of channels (fp32 accumulation).
template <typename T> struct VecAcc;
template <> struct VecAcc<bf16_t> {
    float a[8];
    D2C_DEV void zero() {
#pragma unroll
        for (int i = 0; i < 8; i++) a[i] = 0.f;
    }
    D2C_DEV void fma(float w, const uint4 &v)
    {
        a[0] = fmaf(w, __uint_as_float(v.x << 16), a[0]);
        a[1] = fmaf(w, __uint_as_float(v.x & 0xffff0000u), a[1]);
        a[2] = fmaf(w, __uint_as_float(v.y << 16), a[2]);
        a[3] = fmaf(w, __uint_as_float(v.y & 0xffff0000u), a[3]);
        a[4] = fmaf(w, __uint_as_float(v.z << 16), a[4]);
        a[5] = fmaf(w, __uint_as_float(v.z & 0xffff0000u), a[5]);
        a[6] = fmaf(w, __uint_as_float(v.w << 16), a[6]);
        a[7] = fmaf(w, __uint_as_float(v.w & 0xffff0000u), a[7]);
    }
    D2C_DEV uint4 pack() const
    {
        return make_uint4(pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3]), pack_bf16x2(a[4], a[5]),
                          pack_bf16x2(a[6], a[7]));
    }
};
template <> struct VecAcc<float> {
    float a[4];
    D2C_DEV void zero() { a[0] = a[1] = a[2] = a[3] = 0.f; }
    D2C_DEV void fma(float w, const uint4 &v)
    {
        a[0] = fmaf(w, __uint_as_float(v.x), a[0]);
        a[1] = fmaf(w, __uint_as_float(v.y), a[1]);
        a[2] = fmaf(w, __uint_as_float(v.z), a[2]);
        a[3] = fmaf(w, __uint_as_float(v.w), a[3]);
    }
    // (as an operand of the forward kernels' matrix instructions, see kF32SplitFwd)
    D2C_DEV uint4 pack() const { return operand_vec<float, kF32SplitFwd>(a); }
};

template <typename T> D2C_DEV float elem_to_f32(T v);
template <> D2C_DEV float elem_to_f32<bf16_t>(bf16_t v) { return bf16_to_f32(v); }
template <> D2C_DEV float elem_to_f32<float>(float v) { return v; }
template <typename T> D2C_DEV T f32_to_elem(float v);
template <> D2C_DEV bf16_t f32_to_elem<bf16_t>(float v) { return f32_to_bf16(v); }
template <> D2C_DEV float f32_to_elem<float>(float v) { return v; }

// offset / mask element with the storage type fixed at compile time (no branch in hot loops)
template <bool AUX16> D2C_DEV float ld_auxT(const void *p, long i)
{
    if constexpr (AUX16) return bf16_to_f32(reinterpret_cast<const bf16_t *>(p)[i]);
    else return reinterpret_cast<const float *>(p)[i];
}

// offset / mask element (float32 or bfloat16 storage) as float
D2C_DEV float ld_aux(const void *p, long i, int adt)
{
    return adt == D2C_F32 ? reinterpret_cast<const float *>(p)[i]
                          : bf16_to_f32(reinterpret_cast<const bf16_t *>(p)[i]);
}
D2C_DEV void st_aux(void *p, long i, int adt, float v)
{
    if (adt == D2C_F32) reinterpret_cast<float *>(p)[i] = v;
    else reinterpret_cast<bf16_t *>(p)[i] = f32_to_bf16(v);
}

// ---- tap offsets formed from a predicted size map (the dynamic-dilation layers) --------------------------------
// When SizeSrc::on is set, the `off` argument of the tiled kernels is not the [N, 3K, P] offsets tensor but the raw
// size prediction [N, channels(mode), P], and a tap's offsets are formed where they are needed:
//     off_a = base_a[k_a] * (act(raw_a) - 1)      (network/layers.py:171-181, utils/grid.py:72-98)
// with every intermediate rounded to the storage type, i.e. bit for bit what the expanding kernel of
// d2c_sizemap.hip (and the torch formulation) would have stored.  One offset group only (the reference's
// size-conditioned layers predict 3K offset channels, network/layers.py:184-313).
struct SizeSrc {
    int on;                               // 1: `off` is the raw map; 2: `off` is (size - 1) per axis, float [N][3][P],
                                          //    made from the raw map by one small kernel in front (backward pass)
    int mode, act;                        // D2C_SIZE_*, D2C_SIZE_ACT_*
    float base[3][D2C_SIZE_MAX_K];        // kernel-grid axes z, y, x
};

// channel of the raw map that feeds axis a (0 z, 1 y, 2 x), or -1 for "size 1"
D2C_DEV int axis_channel(int mode, int a)
{
    switch (mode) {
    case D2C_SIZE_XYZ: return a;
    case D2C_SIZE_XXZ: return a == 0 ? 0 : 1;
    case D2C_SIZE_XY: return a == 0 ? -1 : a - 1;
    default: return a == 0 ? -1 : 0;   // D2C_SIZE_X
    }
}
__host__ __device__ inline int mode_channels(int mode) { return mode == D2C_SIZE_XYZ ? 3 : (mode == D2C_SIZE_X ? 1 : 2); }

// value rounded to the storage type, as a tensor between two torch operations would be
template <typename T> D2C_DEV float rnd(float v);
template <> D2C_DEV float rnd<float>(float v) { return v; }
template <> D2C_DEV float rnd<bf16_t>(float v)
{
    // (the hardware conversion, round to nearest even like f32_to_bf16: two instructions)
    typedef float f32x2_ __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_ __attribute__((ext_vector_type(2)));
    const f32x2_ t = {v, 0.f};
    return __uint_as_float(__builtin_bit_cast(uint32_t, __builtin_convertvector(t, bf16x2_)) << 16);
}

// network/layers.py:171-181, operation by operation
template <typename T> D2C_DEV float size_act(int act, float x)
{
    switch (act) {
    case D2C_SIZE_ACT_ELU: return rnd<T>(rnd<T>(x > 0.f ? x : expf(x) - 1.f) + 1.f);
    case D2C_SIZE_ACT_RELU: return fmaxf(rnd<T>(x + 1.f), 0.f);
    case D2C_SIZE_ACT_RELU_PLUS_ONE: return rnd<T>(fmaxf(rnd<T>(x + 1e-3f), 0.f) + 1.f);
    default: return x;
    }
}
D2C_DEV float size_act_grad(int act, float x)
{
    switch (act) {
    case D2C_SIZE_ACT_ELU: return x > 0.f ? 1.f : expf(x);
    case D2C_SIZE_ACT_RELU: return x + 1.f > 0.f ? 1.f : 0.f;
    case D2C_SIZE_ACT_RELU_PLUS_ONE: return x + 1e-3f > 0.f ? 1.f : 0.f;
    default: return 1.f;
    }
}

// Exact n / d for 0 <= n < 2^31 by a multiplication: with l = ceil(log2 d) and m = ceil(2^(31 + l) / d) (which
// fits 32 bits), floor(m * n / 2^(31 + l)) = floor(n / d).  A 32-bit integer division costs ~35 vector
// instructions, a 64-bit one well over a hundred: too much for code that runs once per (tile, tap).
struct FastDiv {
    unsigned m;
    int sh;        // l - 1, or -1 for d == 1
    int d;
};
inline FastDiv make_fastdiv(int d)
{
    FastDiv f{0u, -1, d};
    if (d <= 1) return f;
    int l = 0;
    while ((1ll << l) < d) l++;
    f.m = (unsigned)(((1ull << (31 + l)) + (unsigned long long)d - 1) / (unsigned long long)d);
    f.sh = l - 1;
    return f;
}
D2C_DEV int fdiv(int n, const FastDiv &f) { return f.sh < 0 ? n : (int)(__umulhi((unsigned)n, f.m) >> f.sh); }

// Geometry of the tiled kernels.  Channels are walked in chunks of BKC = 8*VEC
// (64 bf16 / 32 float): one chunk never straddles an offset group or a weight
// group, so all of its channels share the 8 corner positions of a tap.
struct TiledShape {
    int N, Cin, Cout, D, H, W, K, G, groups, Do, Ho, Wo;
    int cg, og, cpg;      // channels per weight group (in / out), per offset group
    int nchunk;           // chunks per weight group = cg / BKC
    int bkc, cpc;         // channels per chunk (BKC); consecutive chunks of a weight group that share an offset group
    int ogp;              // og rounded up to the output tile width
    int adt;
    int P, vol;           // output positions / input voxels per sample
    int M;                // N * P
    int nd;               // 3, or 1 for the 1-D operator mapped onto a 1 x 1 x L volume
    int quirks;           // 1-D only: integer-position rule of dconv1d_gpu.cu:332-336 in grad_offset / grad_mask
    int act;              // forward epilogue: 0 none, 1 act_scale * max(v, 0)
    float act_scale;
    TapGeom geo;
    int axes;             // bit a set: sampling points are displaced along axis a (0 z, 1 y, 2 x); 7 = all
    unsigned keep;        // corners that can have a non-zero weight: with an axis fixed, those on its near plane
    SizeSrc ss;           // offsets formed from a size map instead of read from a tensor
    FastDiv dP, dHW, dW;  // divisions by P, Ho * Wo and Wo
    // Elements between consecutive samples of the offsets tensor (or the size map) and of the mask, and of their
    // gradients: G * K * nd * P and G * K * P for tensors of their own; the channel count of the layer's deformation
    // tensor times P when both pointers point into that one tensor (d2c_conv3d_desc::deform_channels).
    long obs, mbs;
    int mact;             // activation the sampler applies to the mask values it reads (D2C_MASK_ACT_*)
    int f32split;         // float problems: 1 = all backward matrix kernels take two-term bfloat16 operands
                          // (D2C_BWD_F32_SPLIT), 2 = the grad-column product alone (tiled_bwd_col32f_kernel / tiled_bwd_col_kernel), 0 = none
};

// The modulation activation of the self-deforming layers (network/layers.py:107-120, dconv_native/modules.py:71-84),
// applied where a mask value is read; rounded to the storage type AT like the tensor that torch's activation
// would have written.
template <typename AT> D2C_DEV float mask_act(int act, float v)
{
    switch (act) {
    case D2C_MASK_ACT_SIGMOID: return rnd<AT>(1.f / (1.f + expf(-v)));
    case D2C_MASK_ACT_RELU: return fmaxf(v, 0.f);
    case D2C_MASK_ACT_TANH: return rnd<AT>(tanhf(v));
    default: return v;
    }
}
D2C_DEV float mask_act_rt(int act, float v, int adt)
{
    return adt == D2C_BF16 ? mask_act<bf16_t>(act, v) : mask_act<float>(act, v);
}
// d(activated) / d(raw) from the activated value, as torch's backward formulas take it
D2C_DEV float mask_act_grad(int act, float a)
{
    switch (act) {
    case D2C_MASK_ACT_SIGMOID: return a * (1.f - a);
    case D2C_MASK_ACT_RELU: return a > 0.f ? 1.f : 0.f;
    case D2C_MASK_ACT_TANH: return 1.f - a * a;
    default: return 1.f;
    }
}
// element index of mask (b, g, k, p) / of the first offset component of (b, g, k, p)
D2C_DEV long mask_index(const TiledShape &s, int b, int g, int k, int p) { return (long)b * s.mbs + ((long)g * s.K + k) * s.P + p; }
D2C_DEV long offset_index(const TiledShape &s, int b, int g, int k, int p)
{
    return (long)b * s.obs + ((long)g * s.K + k) * (s.nd == 3 ? 3 : 1) * s.P + p;
}

// With offsets fixed along some axes only the corners on the near side of those axes can have weight: 2^(free axes) of
// them.  Slot j of those is the corner whose bits are the bits of j spread over the free axes (corner bit 2 = z,
// 1 = y, 0 = x; `axes` bit 0 = z free, 1 = y, 2 = x).
__host__ __device__ inline int corner_of_slot(int j, int axes)
{
    int c = 0;
    if (axes & 4) { c |= (j & 1); j >>= 1; }          // x
    if (axes & 2) { c |= (j & 1) << 1; j >>= 1; }     // y
    if (axes & 1) { c |= (j & 1) << 2; }              // z
    return c;
}

// make_tap3 for the tiled kernels: corners that a fixed axis leaves with weight zero are not fetched.
D2C_DEV Tap3<float> tiled_tap3(const TiledShape &s, int bz, int by, int bx, float oz, float oy, float ox)
{
    Tap3<float> t = make_tap3<float>(bz, by, bx, oz, oy, ox, s.D, s.H, s.W);
    t.live &= s.keep;
    t.inrange &= s.keep;
    return t;
}

// The three values a sampling point needs, requested early (issue) and turned into offsets late (finish):
// the offsets themselves, or the raw sizes of the position (0 for an axis the mode does not predict).
// (SIZED is a compile-time property of the kernels: the ones that read an offsets tensor carry none of the size-map
// code, which would cost their coordinate wavefronts, the critical ones at small tiles, several per cent)
template <bool AUX16, bool SIZED>
D2C_DEV void tap_offsets_issue(const TiledShape &s, const void *off, int b, int g, int k, int p, float *c)
{
    if constexpr (SIZED) {
        if (s.ss.on == 2) {
            const float *f = reinterpret_cast<const float *>(off) + (long)b * 3 * s.P + p;
            c[0] = f[0]; c[1] = f[s.P]; c[2] = f[2 * (long)s.P];
            return;
        }
#pragma unroll
        for (int ax = 0; ax < 3; ax++) {
            const int ch = axis_channel(s.ss.mode, ax);
            c[ax] = ch < 0 ? 0.f : ld_auxT<AUX16>(off, (long)b * s.obs + (long)ch * s.P + p);
        }
        return;
    }
    const long ab = offset_index(s, b, g, k, p);
    if (s.nd == 3) {
        const long ob = ab;
        // (all three are requested, a fixed axis is dropped by a select: no branches between the loads)
        const float v0 = ld_auxT<AUX16>(off, ob), v1 = ld_auxT<AUX16>(off, ob + s.P);
        const float v2 = ld_auxT<AUX16>(off, ob + 2 * (long)s.P);
        c[0] = (s.axes & 1) ? v0 : 0.f;
        c[1] = (s.axes & 2) ? v1 : 0.f;
        c[2] = (s.axes & 4) ? v2 : 0.f;
    } else {
        c[0] = 0.f; c[1] = 0.f;
        c[2] = ld_auxT<AUX16>(off, ab);
    }
}
// size map: raw sizes of a position -> (size - 1) per axis, the part of a tap's offsets that all taps share
template <bool AUX16> D2C_DEV void size_minus_one(const TiledShape &s, float *c)
{
    typedef typename std::conditional<AUX16, bf16_t, float>::type AT;
#pragma unroll
    for (int ax = 0; ax < 3; ax++)
        c[ax] = axis_channel(s.ss.mode, ax) < 0 ? 0.f : rnd<AT>(size_act<AT>(s.ss.act, c[ax]) - 1.f);
}
// ... and from there the offsets of tap k
template <bool AUX16> D2C_DEV void size_tap_offsets(const TiledShape &s, int k, const float *sm1, float *o)
{
    typedef typename std::conditional<AUX16, bf16_t, float>::type AT;
    const int kz = k / (s.geo.kw * s.geo.kh), ky = (k / s.geo.kw) % s.geo.kh, kx = k % s.geo.kw;
    const float b0 = s.ss.base[0][kz], b1 = s.ss.base[1][ky], b2 = s.ss.base[2][kx];
    const float s0 = sm1[0], s1 = sm1[1], s2 = sm1[2];
    o[0] = rnd<AT>(rnd<AT>(b0) * s0);
    o[1] = rnd<AT>(rnd<AT>(b1) * s1);
    o[2] = rnd<AT>(rnd<AT>(b2) * s2);
}
template <bool AUX16, bool SIZED> D2C_DEV void tap_offsets_finish(const TiledShape &s, int k, float *c)
{
    if constexpr (SIZED) {
        if (s.ss.on == 1) size_minus_one<AUX16>(s, c);
        size_tap_offsets<AUX16>(s, k, c, c);
    }
}

// ---- bias gradient of one output channel by a workgroup of NT threads: gb[o] = sum_{b,p} gout[b,o,p]
// (16-byte loads where the row allows them)
template <typename T, int NT> D2C_DEV void bias_grad_body(const T *gout, T *gb, int N, int Cout, int P, int o)
{
    constexpr int VEC = 16 / (int)sizeof(T);
    __shared__ float part[NT / 64];
    float acc = 0.f;
    for (int b = 0; b < N; b++) {
        const T *row = gout + ((long)b * Cout + o) * P;
        const int head = (int)(((16 - (reinterpret_cast<uintptr_t>(row) & 15)) & 15) / sizeof(T));   // to 16-byte alignment
        const int h = head < P ? head : P;
        const int nvec = (P - h) / VEC;
        if ((int)threadIdx.x < h) acc += elem_to_f32<T>(row[threadIdx.x]);
        const uint4 *rv = reinterpret_cast<const uint4 *>(row + h);
        for (int i = threadIdx.x; i < nvec; i += NT) {
            const uint4 v = rv[i];
            const T *e = reinterpret_cast<const T *>(&v);
#pragma unroll
            for (int j = 0; j < VEC; j++) acc += elem_to_f32<T>(e[j]);
        }
        for (int p = h + nvec * VEC + threadIdx.x; p < P; p += NT) acc += elem_to_f32<T>(row[p]);
    }
#pragma unroll
    for (int sft = 32; sft > 0; sft >>= 1) acc += __shfl_xor(acc, sft, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < NT / 64; i++) t += part[i];
        gb[o] = f32_to_elem<T>(t);
    }
}

// ---- LDS reads of rows that DMA transfers (global_load_lds) filled --------------------------------------------------
// The compiler makes every LDS read wait for all DMA transfers in flight into the same array (it cannot tell the
// half being read from the half being filled), i.e. it drains the requests just issued for a later tile before the
// rows of this one are read.  These reads are hidden from it (inline assembly); the kernels wait for the transfers
// they need themselves (vmcnt) and for the reads with lds_rows_wait(), through which the values must pass before
// they are used.
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
// 16 bytes of a buffer that the kernel reads once, front to back (grad-column rows, sampled columns): a streaming load,
// so that the lines do not push the rows that are gathered again and again out of the L2.
D2C_DEV uint4 ld_stream16(const void *p)
{
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
template <int OFF> D2C_DEV u32x4_t lds_row_read(unsigned lds_addr)
{
    u32x4_t v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(lds_addr), "n"(OFF));
    return v;
}
D2C_DEV void lds_rows_wait(u32x4_t &a, u32x4_t &b, u32x4_t &c, u32x4_t &d)
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
D2C_DEV void lds_rows_wait(u32x4_t &a, u32x4_t &b) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b)); }
D2C_DEV unsigned lds_address(const void *p)
{
    return (unsigned)(size_t)(__attribute__((address_space(3))) const void *)p;
}

// ---- the coordinate wavefront of the DMA-gather kernels ---------------------------------------------------------
// One wavefront per workgroup turns sampling points into table rows (8 corner weights, the element offset of corner
// 000, the corners to fetch); an iteration of the workgroup cannot end before its row is written, so this code is
// written for instruction count: no integer division, no branch, loop constants in vector registers (a scalar
// register that is spilled costs a vector instruction per use), corners dropped through their axis factor.
struct CoordConst {
    float Df, Hf, Wf, Dm1, Hm1, Wm1;      // extents, and extents - 1, as float
    int H, W, Cin;
    unsigned ax0, ax1, ax2;               // all ones where the offsets displace along the axis, else 0
    unsigned keep;
};
// value of lane l (uniform) of a float register
D2C_DEV float lane_value(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }
D2C_DEV void opaque_v(float &v) { asm volatile("" : "+v"(v)); }
D2C_DEV void opaque_v(int &v) { asm volatile("" : "+v"(v)); }
D2C_DEV void opaque_v(unsigned &v) { asm volatile("" : "+v"(v)); }
D2C_DEV CoordConst coord_const(const TiledShape &s)
{
    CoordConst c;
    c.Df = (float)s.D; c.Hf = (float)s.H; c.Wf = (float)s.W;
    c.Dm1 = (float)(s.D - 1); c.Hm1 = (float)(s.H - 1); c.Wm1 = (float)(s.W - 1);
    c.H = s.H; c.W = s.W; c.Cin = s.Cin;
    // (the 1-D operator has one offset component, which the loads deliver in all three slots: x keeps it)
    const int axes = s.nd == 3 ? s.axes : 4;
    c.ax0 = (axes & 1) ? ~0u : 0u; c.ax1 = (axes & 2) ? ~0u : 0u; c.ax2 = (axes & 4) ? ~0u : 0u;
    c.keep = s.keep;
    opaque_v(c.Df); opaque_v(c.Hf); opaque_v(c.Wf); opaque_v(c.Dm1); opaque_v(c.Hm1); opaque_v(c.Wm1);
    opaque_v(c.H); opaque_v(c.W); opaque_v(c.Cin);
    opaque_v(c.ax0); opaque_v(c.ax1); opaque_v(c.ax2); opaque_v(c.keep);
    return c;
}

// Offsets of one sampling point, requested from (uniform address) + (32-bit offset of the lane): the address
// arithmetic stays in scalar registers.  `ub`: first component of the (sample, group, tap) row of the lane with
// offset 0; `cstride`: bytes between components (0 for the one-component offsets of the 1-D operator, whose value is
// then read three times and kept as the x component).
template <bool AUX16> D2C_DEV float ld_aux_at(const char *ub, unsigned lane_bytes)
{
    if constexpr (AUX16) return bf16_to_f32(*reinterpret_cast<const bf16_t *>(ub + lane_bytes));
    else return *reinterpret_cast<const float *>(ub + lane_bytes);
}
template <bool AUX16>
D2C_DEV void coord_offsets_issue(const char *ub, long cstride, unsigned lane_bytes, float *c)
{
    c[0] = ld_aux_at<AUX16>(ub, lane_bytes);
    c[1] = ld_aux_at<AUX16>(ub + cstride, lane_bytes);
    c[2] = ld_aux_at<AUX16>(ub + 2 * cstride, lane_bytes);
}
D2C_DEV void coord_offsets_select(const CoordConst &cc, float *c)
{
    c[0] = __uint_as_float(__float_as_uint(c[0]) & cc.ax0);
    c[1] = __uint_as_float(__float_as_uint(c[1]) & cc.ax1);
    c[2] = __uint_as_float(__float_as_uint(c[2]) & cc.ax2);
}

// Table row of the sampling point (z, y, x) with modulation m; `ok` false (a lane without a position) gives a row
// that fetches nothing.  Bit for bit the weights of make_tap3 / tap3_weight times m for the corners that are live
// there, zero for the others:
//   * a point outside (-1, extent) on any axis, or not a number, has no live corner (make_tap3's `out` / `finite`);
//     inside, floor(z) lies in [-1, D-1], so corner 0 of the axis is in range iff floor(z) >= 0 and corner 1 iff
//     floor(z) < D - 1, and no clamp is needed before the conversion to int;
//   * a corner out of range gets weight zero through its axis factor (the factors of the live corners are untouched,
//     and so are their products, in tap3_weight's order);
//   * m of a point without live corner is dropped (0 * NaN would be NaN; with a live corner all eight products end
//     in the same sum, where a NaN modulation shows up in either formulation).
struct CornerRow {
    float w[8];
    int idx;              // element offset of corner 000 in the channels-last input (only live corners are fetched)
    unsigned live;
};
D2C_DEV CornerRow corner_row(const CoordConst &cc, float z, float y, float x, float m, int vox0, bool ok)
{
    CornerRow r;
    // (bitwise: one chain of compare masks, no branch)
    const bool in = ok & (z > -1.f) & (z < cc.Df) & (y > -1.f) & (y < cc.Hf) & (x > -1.f) & (x < cc.Wf);
    const float zs = in ? z : 0.f, ys = in ? y : 0.f, xs = in ? x : 0.f, ms = in ? m : 0.f;
    const float fz = floorf(zs), fy = floorf(ys), fx = floorf(xs);
    const float hz = zs - fz, hy = ys - fy, hx = xs - fx;
    const float lz = (fz + 1.f) - zs, ly = (fy + 1.f) - ys, lx = (fx + 1.f) - xs;
    // (a corner is fetched where it lies inside the volume AND has a weight: a sampling point that sits on a voxel
    // plane -- zero offsets, i.e. an ordinary convolution, or whole-voxel offsets -- gives the corners on the far side
    // of the plane weight zero, and a modulation of exactly zero, common behind a ReLU, all eight; such corners read
    // the row of zeros like those outside the volume.  For finite inputs the sum is the same.)
    const bool z0 = in & (fz >= 0.f), z1 = in & (fz < cc.Dm1) & (hz > 0.f);
    const bool y0 = in & (fy >= 0.f), y1 = in & (fy < cc.Hm1) & (hy > 0.f);
    const bool x0 = in & (fx >= 0.f), x1 = in & (fx < cc.Wm1) & (hx > 0.f);
    r.live = ((z0 ? 0x0Fu : 0u) | (z1 ? 0xF0u : 0u)) & ((y0 ? 0x33u : 0u) | (y1 ? 0xCCu : 0u))
             & ((x0 ? 0x55u : 0u) | (x1 ? 0xAAu : 0u)) & cc.keep & (ms != 0.f ? 0xFFu : 0u);
    const float az[2] = {z0 ? lz : 0.f, z1 ? hz : 0.f};
    const float ay[2] = {y0 ? ly : 0.f, y1 ? hy : 0.f};
    const float ax[2] = {x0 ? lx : 0.f, x1 ? hx : 0.f};
#pragma unroll
    for (int q = 0; q < 8; q++) r.w[q] = ((az[q >> 2] * ay[(q >> 1) & 1]) * ax[q & 1]) * ms;
    // (24-bit multiplications: the kernels that use this take shapes with D * H and W below 2^23 only; the last
    // product is a full one)
    const int iz = (int)fz, iy = (int)fy, ix = (int)fx;
    r.idx = (vox0 + __mul24(__mul24(iz, cc.H) + iy, cc.W) + ix) * cc.Cin;
    return r;
}

// The forward kernels' last step before a value is stored (NaN stays NaN, as in torch's relu).
__host__ __device__ inline float d2c_epilogue(float v, int act, float scale)
{
    // branch-free: without activation the floor is -inf and the factor 1 (v * 1 is exact)
    const float lo = act ? 0.f : -__builtin_inff(), sc = act ? scale : 1.f;
    return (v < lo ? lo : v) * sc;
}

// Load of a lane's 4 channels from a wavefront-uniform row address plus the lane's byte offset.  The row
// address is pinned to scalar registers, so that the load needs no 64-bit vector arithmetic.
template <typename T> D2C_DEV void ld4_row(const T *row, unsigned lane_bytes, float *v)
{
    typedef const __attribute__((address_space(1))) char *gptr;
    const unsigned long long a = reinterpret_cast<unsigned long long>(row);
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)a);
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(a >> 32));
    gptr p = (gptr)(((unsigned long long)hi << 32) | lo) + lane_bytes;
    typedef float f32x4v __attribute__((ext_vector_type(4)));
    typedef unsigned u32x2v __attribute__((ext_vector_type(2)));
    if constexpr (sizeof(T) == 4) {
        const f32x4v t = *reinterpret_cast<const __attribute__((address_space(1))) f32x4v *>(p);
        v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
    } else {
        const u32x2v t = *reinterpret_cast<const __attribute__((address_space(1))) u32x2v *>(p);
        v[0] = __uint_as_float(t[0] << 16); v[1] = __uint_as_float(t[0] & 0xffff0000u);
        v[2] = __uint_as_float(t[1] << 16); v[3] = __uint_as_float(t[1] & 0xffff0000u);
    }
}

// ---- sample lists: every live sample (b, g, k, p) filed under its base voxel floor(z, y, x) -------------------
struct alignas(16) InvEntry {
    int p, k;              // output position inside the sample, tap
    float hz, hy, hx;      // fractions z - floor(z), ...
    float alpha;           // modulation
    int pad0, pad1;        // pad0: the bin, in entries of the overflow array
};
static_assert(sizeof(InvEntry) == 32, "two 16-byte loads per entry");

// bins cover base voxels -1 .. size-1 per axis
D2C_DEV int bin_of(const TiledShape &s, int b, int g, int z0, int y0, int x0)
{
    return (((b * s.G + g) * (s.D + 1) + (z0 + 1)) * (s.H + 1) + (y0 + 1)) * (s.W + 1) + (x0 + 1);
}

// Mapping of a 1-D grid onto the 8 XCDs, each with an L2 of its own; workgroups are dealt to them round-robin.
// The work is `ncombo` combinations (of batch element, channel slice, ...) of `tpb` tiles each.  It is cut
// into units of (combination, part of its tiles), their number a multiple of 8, and unit u runs on XCD u % 8,
// its tiles in order: the L2 of an XCD then holds the data of one combination at a time.  The grid is
// xcd_unit_grid() workgroups; those with ok == false have no tile.
struct XcdUnit {
    int combo, tile;
    bool ok;
};
__host__ __device__ inline int xcd_unit_parts(int ncombo)
{
    const int low = ncombo & -ncombo;   // largest power of two dividing ncombo
    return low >= 8 ? 1 : 8 / low;
}
D2C_DEV XcdUnit xcd_unit(int bid, int ncombo, int tpb)
{
    const int parts = xcd_unit_parts(ncombo);
    const int tpp = (tpb + parts - 1) / parts;      // tiles of a part
    const int xcd = bid & 7, idx = bid >> 3;
    const int j = idx / tpp, t = idx - j * tpp;
    const int u = j * 8 + xcd;
    XcdUnit r;
    r.combo = u / parts;
    r.tile = (u - r.combo * parts) * tpp + t;
    r.ok = r.tile < tpb;
    return r;
}
inline unsigned xcd_unit_grid(int ncombo, int tpb)
{
    const int parts = xcd_unit_parts(ncombo);
    return (unsigned)(ncombo * parts * ((tpb + parts - 1) / parts));
}

// Lists as buckets of fixed capacity, filled in one pass (a counter per bin; no counting pass, no scan).
// A sample that finds its bucket full goes to one shared overflow array instead, which a separate kernel
// adds into grad_input with atomics: rare for real offset fields (a bucket holds more than twice the mean
// list), and correct however the samples crowd.
struct SampleLists {
    int *counts;         // [nbins] samples filed under the bin (may exceed cap); [nbins]: overflow entries
    InvEntry *entries;   // [nbins][cap]  (of 16-byte packed entries when `compact`)
    InvEntry *ovf;       // [ovf_cap]
    int cap, nbins, ovf_cap;
    int compact;         // bucket entries packed into 16 bytes (bfloat16 problems with P < 2^24 and K < 256)
};
// Packed entry: position | tap << 24, the three fractions as 16-bit fixed point (error < 8e-6, far below what
// bfloat16 gradients resolve), the modulation.  Half the bytes of the scattered stores that file the samples.
D2C_DEV unsigned frac_to_u16(float h)
{
    const unsigned q = (unsigned)(h * 65536.f + 0.5f);
    return q > 65535u ? 65535u : q;
}
D2C_DEV uint4 pack_entry(const InvEntry &e)
{
    return make_uint4((unsigned)e.p | ((unsigned)e.k << 24), frac_to_u16(e.hz) | (frac_to_u16(e.hy) << 16),
                      frac_to_u16(e.hx), __float_as_uint(e.alpha));
}
D2C_DEV InvEntry unpack_entry(const uint4 &q)
{
    InvEntry e;
    e.p = (int)(q.x & 0xffffffu); e.k = (int)(q.x >> 24);
    e.hz = (float)(q.y & 0xffffu) * (1.f / 65536.f); e.hy = (float)(q.y >> 16) * (1.f / 65536.f);
    e.hx = (float)(q.z & 0xffffu) * (1.f / 65536.f);
    e.alpha = __uint_as_float(q.w);
    e.pad0 = 0; e.pad1 = 0;
    return e;
}
// (in two steps, so that a caller can do other work while the counter's old value is on its way)
D2C_DEV int lists_reserve(const SampleLists &L, int bin) { return atomicAdd(&L.counts[bin], 1); }
D2C_DEV void lists_store(const SampleLists &L, int bin, int n, InvEntry e)
{
    if (n < L.cap) {
        if (L.compact) reinterpret_cast<uint4 *>(L.entries)[(long)bin * L.cap + n] = pack_entry(e);
        else L.entries[(long)bin * L.cap + n] = e;
    } else {
        const int m = atomicAdd(&L.counts[L.nbins], 1);
        if (m < L.ovf_cap) {
            e.pad0 = bin;
            L.ovf[m] = e;
        }
    }
}
D2C_DEV void lists_insert(const SampleLists &L, int bin, InvEntry e) { lists_store(L, bin, lists_reserve(L, bin), e); }

// The three offsets (dz, dy, dx) of (b, g, k, p).  The 1-D operator stores one
// offset per tap ([N, G*K, Lo], dconv1d_gpu.cu:40); it displaces along x only.
D2C_DEV void load_offsets(const TiledShape &s, const void *off, int b, int g, int k, int p, float &o0, float &o1,
                          float &o2)
{
    if (s.ss.on) {
        float c[3];
        if (s.adt == D2C_BF16) {
            tap_offsets_issue<true, true>(s, off, b, g, k, p, c);
            tap_offsets_finish<true, true>(s, k, c);
        } else {
            tap_offsets_issue<false, true>(s, off, b, g, k, p, c);
            tap_offsets_finish<false, true>(s, k, c);
        }
        o0 = c[0]; o1 = c[1]; o2 = c[2];
        return;
    }
    if (s.nd == 3) {
        const long ob = offset_index(s, b, g, k, p);
        o0 = (s.axes & 1) ? ld_aux(off, ob, s.adt) : 0.f;
        o1 = (s.axes & 2) ? ld_aux(off, ob + s.P, s.adt) : 0.f;
        o2 = (s.axes & 4) ? ld_aux(off, ob + 2 * (long)s.P, s.adt) : 0.f;
    } else {
        o0 = 0.f; o1 = 0.f;
        o2 = ld_aux(off, offset_index(s, b, g, k, p), s.adt);
    }
}
