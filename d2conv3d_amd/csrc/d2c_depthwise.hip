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
// A workgroup owns a tile of output positions and a slice of 256 channels (one
// 16-byte vector per lane of a wavefront); dw_tile() maps the workgroups so that
// each XCD works on one channel slice of one batch element at a time, which
// then stays in its L2.  The corner weights of the tile are
// computed once into LDS and shared by the four wavefronts.
#include "d2c_mma.hpp"
#include "d2c_tiled.hpp"

namespace {

constexpr int kDwThreads = 256;   // 4 wavefronts
constexpr int kCV = 4;            // consecutive channels per lane
constexpr int kSlice = 64 * kCV;  // channels per workgroup
// forward: 8 consecutive positions per wavefront (one 32-byte output segment per channel)
constexpr int kFwdTP = 32, kFwdKB = 16;
// backward: the taps of a batch are dealt to the wavefronts, each walks all positions of the tile
constexpr int kBwdTP = 16, kBwdKB = 16;

struct DwArgs {
    TiledShape s;
    const void *xcl;           // [N][vol][C]
    const void *off, *mask;
    const void *wt;            // [K][C]  weights, tap-major
    const void *bias;
    void *out;
    // backward
    const void *goutcl;        // [N][P][C]  channels-last copy of grad_out
    float *gxcl;               // [N][vol][C] fp32 accumulator (zeroed) for the atomic scatter, or NULL
    float *auxoff, *auxmask;   // fp32 accumulators (zeroed) laid out like grad_offset / grad_mask, or NULL
    float *gwacc;              // [K][C] fp32 accumulator (zeroed) or NULL
};

// Tile of a workgroup: the combinations of xcd_unit() are (batch element, offset group, channel slice), so
// the L2 of an XCD sees one channel slice of one batch element at a time (3.3 MB of the input for 256 fp32
// channels of 8x15x27 voxels) and not, as with tiles dealt in launch order, all channels of the input.
// Tiles do not straddle batch elements.
struct DwTile {
    int m0, m_end;   // positions [m0, m_end) of the flattened (batch, position) range
    int y;           // offset group * slices + slice
    bool ok;
};
D2C_DEV DwTile dw_tile(const TiledShape &s, int TP, int ny, int bid)
{
    const XcdUnit u = xcd_unit(bid, s.N * ny, (s.P + TP - 1) / TP);
    const int b = u.combo % s.N;
    DwTile r;
    r.y = u.combo / s.N;
    r.ok = u.ok;
    r.m0 = b * s.P + u.tile * TP;
    r.m_end = min(r.m0 + TP, (b + 1) * s.P);
    return r;
}
inline unsigned dw_grid(const TiledShape &s, int TP, int ny) { return xcd_unit_grid(s.N * ny, (s.P + TP - 1) / TP); }

// View over dynamic LDS, one entry per (tap of the batch, position of the tile): the base voxel and
// live | inrange << 8, and
//   forward:  the live corner weights * alpha, corner-major (w[corner][entry]);
//   backward: 16 floats per entry, read as 16-byte vectors: the 8 corner weights * alpha | the per-axis fractions
//             lz ly lx hz | hy hx, alpha, a pad.
template <int TP, int KB> struct DwTaps {
    static constexpr int kNE = KB * TP;
    float (*w)[kNE];
    float4 *pk;
    int *idx, *flag;
};
constexpr int kDwEntryVecs = 4;
template <int TP, int KB> D2C_DEV DwTaps<TP, KB> dw_taps(unsigned char *smem, bool bwd)
{
    constexpr int kNE = KB * TP;
    DwTaps<TP, KB> t;
    float *f = reinterpret_cast<float *>(smem);
    t.w = nullptr; t.pk = nullptr;
    if (bwd) {
        t.pk = reinterpret_cast<float4 *>(f); f += 4 * kDwEntryVecs * kNE;
    } else {
        t.w = reinterpret_cast<float (*)[kNE]>(f); f += 8 * kNE;
    }
    t.idx = reinterpret_cast<int *>(f); f += kNE;
    t.flag = reinterpret_cast<int *>(f); f += kNE;
    return t;
}
constexpr size_t kDwLdsFwd = (size_t)10 * kFwdKB * kFwdTP * 4;
// (+ the grad_out tile of the workgroup: kBwdTP rows of kSlice elements)
constexpr size_t kDwLdsTab = (size_t)(4 * kDwEntryVecs + 2) * kBwdKB * kBwdTP * 4;
constexpr size_t dw_lds_bwd(size_t es) { return kDwLdsTab + (size_t)kBwdTP * kSlice * es; }

template <bool BWD, int TP, int KB>
D2C_DEV void dw_coords(const DwArgs &a, const DwTaps<TP, KB> &t, int m0, int m_end, int g, int k0, int kn)
{
    const TiledShape &s = a.s;
    for (int task = threadIdx.x; task < kn * TP; task += kDwThreads) {
        const int pl = task % TP, kk = task / TP;
        const int k = k0 + kk, m = m0 + pl;
        float w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        float fr[6] = {0, 0, 0, 0, 0, 0};
        float al = 0.f;
        int idx = 0, flag = 0;
        if (m < m_end) {
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
        const int e = kk * TP + pl;
        if (BWD) {
            float4 *q = t.pk + kDwEntryVecs * e;
            q[0] = make_float4(w[0], w[1], w[2], w[3]);
            q[1] = make_float4(w[4], w[5], w[6], w[7]);
            q[2] = make_float4(fr[0], fr[1], fr[2], fr[3]);
            q[3] = make_float4(fr[4], fr[5], al, 0.f);
        } else {
#pragma unroll
            for (int c = 0; c < 8; c++) t.w[c][e] = w[c];
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
template <typename T> D2C_DEV void st4(T *p, const float *v)
{
    if constexpr (sizeof(T) == 4) {
        *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
        *reinterpret_cast<uint2 *>(p) = make_uint2((__float_as_uint(v[0]) >> 16) | (__float_as_uint(v[1]) & 0xffff0000u),
                                                   (__float_as_uint(v[2]) >> 16) | (__float_as_uint(v[3]) & 0xffff0000u));
    }
}
static_assert(kCV == 4, "vector loads of 4 channels");

// ------------------------------------------------------------------ forward
template <typename T>
__global__ void __launch_bounds__(kDwThreads) dw_fwd_kernel(DwArgs a)
{
    constexpr int TP = kFwdTP, KB = kFwdKB, PW = TP / 4;   // PW positions per wavefront
    extern __shared__ __align__(16) unsigned char smem[];
    const DwTaps<TP, KB> taps = dw_taps<TP, KB>(smem, false);
    const TiledShape &s = a.s;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nsl = (s.cpg + kSlice - 1) / kSlice;
    const DwTile tl = dw_tile(s, TP, s.G * nsl, blockIdx.x);
    if (!tl.ok) return;
    const int m0 = tl.m0, m_end = tl.m_end;
    const int HW = s.H * s.W;
    const int g = tl.y / nsl, sl = tl.y - g * nsl;
    const int cl = sl * kSlice + lane * kCV;      // first channel of this lane inside the offset group
    const bool cok = cl < s.cpg;
    const int c = g * s.cpg + (cok ? cl : 0);
    const T *xcl = reinterpret_cast<const T *>(a.xcl);
    const T *wt = reinterpret_cast<const T *>(a.wt);

    float acc[PW][kCV];
#pragma unroll
    for (int i = 0; i < PW; i++)
#pragma unroll
        for (int j = 0; j < kCV; j++) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < s.K; k0 += KB) {
        const int kn = min(KB, s.K - k0);
        __syncthreads();
        dw_coords<false, TP, KB>(a, taps, m0, m_end, g, k0, kn);
        __syncthreads();
        if (!cok) continue;
        for (int kk = 0; kk < kn; kk++) {
            float wv[kCV];
            ld4<T>(wt + (long)(k0 + kk) * s.Cin + c, wv);
#pragma unroll
            for (int i = 0; i < PW; i++) {
                const int e = kk * TP + wave * PW + i;
                // the table entry is the same for the whole wavefront: keep it in scalar registers
                const unsigned live = (unsigned)__builtin_amdgcn_readfirstlane(taps.flag[e]) & 0xffu;
                if (!live) continue;
                const int idx = __builtin_amdgcn_readfirstlane(taps.idx[e]);
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
                for (int j = 0; j < kCV; j++) acc[i][j] = fmaf(wv[j], sv[j], acc[i][j]);
            }
        }
    }
    if (!cok) return;

    // --- bias, convert, store: the PW positions of a wavefront are consecutive in the output row of a channel
    float bv[kCV] = {0.f, 0.f, 0.f, 0.f};
    if (a.bias) ld4<T>(reinterpret_cast<const T *>(a.bias) + c, bv);
    T *out = reinterpret_cast<T *>(a.out);
    const int mf = m0 + wave * PW;
    if (mf >= m_end) return;
    const int bf = mf / s.P, pf = mf - bf * s.P;
    constexpr int EV = 16 / (int)sizeof(T);       // elements per 16-byte store
    const bool fast = mf + PW <= m_end && pf % EV == 0 && s.P % EV == 0;
    if (fast) {
#pragma unroll
        for (int j = 0; j < kCV; j++) {
            T *o = out + ((long)bf * s.Cout + c + j) * s.P + pf;
            alignas(16) T e[PW];
#pragma unroll
            for (int i = 0; i < PW; i++) e[i] = f32_to_elem<T>(d2c_epilogue(acc[i][j] + bv[j], s.act, s.act_scale));
#pragma unroll
            for (int q = 0; q < PW / EV; q++) reinterpret_cast<uint4 *>(o)[q] = reinterpret_cast<const uint4 *>(e)[q];
        }
    } else {
#pragma unroll
        for (int i = 0; i < PW; i++) {
            const int m = mf + i;
            if (m < m_end) {
                const int b = m / s.P, pp = m - b * s.P;
#pragma unroll
                for (int j = 0; j < kCV; j++)
                    out[((long)b * s.Cout + c + j) * s.P + pp] = f32_to_elem<T>(d2c_epilogue(acc[i][j] + bv[j], s.act, s.act_scale));
            }
        }
    }
}

// ----------------------------------------------------------------- backward
// Sum of 4 per-lane values over the 64 lanes: after the exchange steps lane
// group (lane>>4) holds the total of value (lane>>4) in all of its lanes.
template <int CTRL> D2C_DEV float dpp_add(float v)
{
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
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
    // inside the rows of 16 lanes: neighbours of a quad, then rotations of the row by 4 and by 8 lanes
    k = dpp_add<0xB1>(k);    // quad_perm [1, 0, 3, 2]
    k = dpp_add<0x4E>(k);    // quad_perm [2, 3, 0, 1]
    k = dpp_add<0x124>(k);   // row_ror 4
    k = dpp_add<0x128>(k);   // row_ror 8
    return k;   // value index = (lane >> 5) * 2 + ((lane >> 4) & 1)
}

// GXATOM: grad_input scattered with atomics from here (the mode without sample lists).
// `xcl` is followed by one row of zeros (voxel N * vol): corners outside the volume read it, so that their dot
// products vanish without a select and every load of a position is made unconditionally.
template <typename T, bool GXATOM>
__global__ void __launch_bounds__(kDwThreads, 4) dw_bwd_kernel(DwArgs a)   // 4 wavefronts per SIMD: what the LDS allows
{
    constexpr int TP = kBwdTP, KB = kBwdKB;
    extern __shared__ __align__(16) unsigned char smem[];
    const DwTaps<TP, KB> taps = dw_taps<TP, KB>(smem, true);
    const TiledShape &s = a.s;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nsl = (s.cpg + kSlice - 1) / kSlice;
    const DwTile tl = dw_tile(s, TP, s.G * nsl, blockIdx.x);
    if (!tl.ok) return;
    const int m0 = tl.m0, m_end = tl.m_end;
    const int g = tl.y / nsl, sl = tl.y - g * nsl;
    const int cl = sl * kSlice + lane * kCV;
    const bool cok = cl < s.cpg;       // lanes past the group still take part in the reductions
    const int c = g * s.cpg + (cok ? cl : 0);
    const T *wt = reinterpret_cast<const T *>(a.wt);
    const T *xcl = reinterpret_cast<const T *>(a.xcl);
    const int HW = s.H * s.W;
    const int zrow = s.N * s.vol;
    // grad_out of the tile's positions, this slice's channels: every tap needs it, so it is staged in LDS once
    // (rows past the tile and channels past the offset group: zeros)
    T *gotile = reinterpret_cast<T *>(smem + kDwLdsTab);
    {
        const T *goutcl = reinterpret_cast<const T *>(a.goutcl);
        for (int r = wave; r < TP; r += kDwThreads / 64) {
            const int m = m0 + r;
            float v[kCV] = {0.f, 0.f, 0.f, 0.f};
            if (cok && m < m_end) ld4<T>(goutcl + (size_t)m * s.Cout + c, v);
            st4<T>(gotile + r * kSlice + lane * kCV, v);
        }
    }
    const bool want_aux = a.auxoff != nullptr || a.auxmask != nullptr;

    for (int k0 = 0; k0 < s.K; k0 += KB) {
        const int kn = min(KB, s.K - k0);
        __syncthreads();
        dw_coords<true, TP, KB>(a, taps, m0, m_end, g, k0, kn);
        __syncthreads();
        for (int kk = wave; kk < kn; kk += kDwThreads / 64) {
            // (lanes past the offset group hold a zero weight: everything they add to the sums over lanes is zero)
            float wv[kCV] = {0.f, 0.f, 0.f, 0.f};
            if (cok) ld4<T>(wt + (long)(k0 + kk) * s.Cin + c, wv);
            float gwv[kCV] = {0.f, 0.f, 0.f, 0.f};
            // table entries of the tap's positions: lane p holds those of position p; they are the same for the
            // whole wavefront and are read out into scalar registers
            const int vflag = taps.flag[kk * TP + (lane & (TP - 1))];
            const int vidx = taps.idx[kk * TP + (lane & (TP - 1))];
            // The corner rows of a position are requested one position ahead of their use.  Every request is made:
            // a corner out of range reads the row of zeros.  Lanes past the offset group read channel 0 on.
            struct Rows {
                float x[8][kCV];
            };
            unsigned cbytes = (unsigned)c * (unsigned)sizeof(T);
            asm("" : "+v"(cbytes));   // kept a plain 32-bit register: the offset operand of the loads
            auto issue = [&](Rows &r, int p) {
                // (made opaque here, in the block of the loads: the zero-extension of the offset then stays next to
                // them and the loads take the scalar-base + 32-bit-offset form instead of 64-bit vector additions)
                unsigned cb = cbytes;
                asm("" : "+v"(cb));
                const unsigned inr = (unsigned)__builtin_amdgcn_readlane(vflag, p) >> 8;
                const int idx = __builtin_amdgcn_readlane(vidx, p);
#pragma unroll
                for (int cc = 0; cc < 8; cc++) {
                    const int v = ((inr >> cc) & 1u) ? idx + ((cc >> 2) & 1) * HW + ((cc >> 1) & 1) * s.W + (cc & 1) : zrow;
                    ld4_row<T>(xcl + (size_t)v * s.Cin, cb, r.x[cc]);
                }
            };
            float stash = 0.f;
            static_assert(TP == 16, "a row of 16 lanes per result");
            auto compute = [&](const Rows &r, int p) {
                const int e = kk * TP + p;
                const unsigned flag = (unsigned)__builtin_amdgcn_readlane(vflag, p);
                const unsigned inr = flag >> 8, live = flag & 0xffu;   // live is 0 or inr
                if (!inr) return;
                // the entry's 16 floats: the same address in every lane (broadcast reads)
                const float4 q0 = taps.pk[kDwEntryVecs * e], q1 = taps.pk[kDwEntryVecs * e + 1];
                const float wc[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};   // a_corner * alpha, 0 where not live
                float go[kCV], gc[kCV];
                ld4<T>(gotile + p * kSlice + lane * kCV, go);
#pragma unroll
                for (int j = 0; j < kCV; j++) gc[j] = wv[j] * go[j];
                float dot[8];
                float sv[kCV] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int cc = 0; cc < 8; cc++) {
                    float d = gc[0] * r.x[cc][0];
#pragma unroll
                    for (int j = 1; j < kCV; j++) d = fmaf(gc[j], r.x[cc][j], d);
                    dot[cc] = d;
#pragma unroll
                    for (int j = 0; j < kCV; j++) sv[j] = fmaf(wc[cc], r.x[cc][j], sv[j]);
                    if constexpr (GXATOM) {
                        if (((live >> cc) & 1u) && cok) {
                            const int idx = __builtin_amdgcn_readlane(vidx, p);
                            const int v = idx + ((cc >> 2) & 1) * HW + ((cc >> 1) & 1) * s.W + (cc & 1);
                            float *gp = a.gxcl + (long)v * s.Cin + c;
#pragma unroll
                            for (int j = 0; j < kCV; j++) atomicAdd(gp + j, wc[cc] * gc[j]);
                        }
                    }
                }
#pragma unroll
                for (int j = 0; j < kCV; j++) gwv[j] = fmaf(go[j], sv[j], gwv[j]);   // sv already holds alpha
                if (want_aux) {
                    // (read here, where the rows' registers are free again)
                    __builtin_amdgcn_sched_barrier(0);
                    const float4 q2 = taps.pk[kDwEntryVecs * e + 2], q3 = taps.pk[kDwEntryVecs * e + 3];
                    const float lz = q2.x, ly = q2.y, lx = q2.z, hz = q2.w, hy = q3.x, hx = q3.y;
                    // The four results are trilinear forms of the dot products; they are taken axis by axis
                    // (x, then y, then z): interpolated sums and differences.
                    float sx[4], dx[4];   // index = z * 2 + y
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        sx[i] = fmaf(hx, dot[2 * i + 1], lx * dot[2 * i]);
                        dx[i] = dot[2 * i + 1] - dot[2 * i];
                    }
                    float sxy[2], dy[2], sdx[2];   // index = z
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        sxy[i] = fmaf(hy, sx[2 * i + 1], ly * sx[2 * i]);
                        dy[i] = sx[2 * i + 1] - sx[2 * i];
                        sdx[i] = fmaf(hy, dx[2 * i + 1], ly * dx[2 * i]);
                    }
                    const float gz = sxy[1] - sxy[0];
                    const float gy = fmaf(hz, dy[1], lz * dy[0]);
                    const float gxx = fmaf(hz, sdx[1], lz * sdx[0]);
                    // the modulation gradient takes the corners of the forward pass only: all in range, or none
                    const float gm = live ? fmaf(hz, sxy[1], lz * sxy[0]) : 0.f;
                    // sums over the 256 channels of the slice; lane (which * 16 + p) keeps result `which` of
                    // position p until all positions of the tap are done
                    const float rs = reduce4_over_wave(gz, gy, gxx, gm, lane);
                    const float val = lane < 48 ? q3.z * rs : rs;
                    stash = (lane & (TP - 1)) == p ? val : stash;
                }
            };
            static_assert(TP % 2 == 0, "positions are worked on in pairs");
            Rows ra, rb;
            issue(ra, 0);
            for (int p = 0; p < TP; p += 2) {
                issue(rb, p + 1);
                compute(ra, p);
                issue(ra, min(p + 2, TP - 1));   // after the last pair: a repeat, not used
                compute(rb, p + 1);
            }
            if (want_aux) {
                // one atomic instruction per tap: 16 consecutive positions per result; the other channel slices
                // of the offset group add theirs to the same places
                const int which = lane >> 4, m = m0 + (lane & (TP - 1));
                if (m < m_end) {
                    const int b = m / s.P, pp = m - b * s.P;
                    const long ab = (((long)b * s.G + g) * s.K + (k0 + kk)) * s.P + pp;
                    if (which < 3) {
                        if (a.auxoff) atomicAdd(a.auxoff + 3 * ab - 2 * (long)pp + which * (long)s.P, stash);
                    } else if (a.auxmask) {
                        atomicAdd(a.auxmask + ab, stash);
                    }
                }
            }
            if (a.gwacc) {
                // A lane holds 4 consecutive channels; atomics issued that way touch every 64-byte line of the slice's
                // 1 KiB four times.  The values change lanes first (lane l of instruction j takes channel 64 j + l),
                // so that an instruction covers 256 consecutive bytes: a quarter of the memory-side operations.
                static_assert(kCV == 4 && kSlice == 256, "4 x 64 channels per wavefront");
                float *gw = a.gwacc + (long)(k0 + kk) * s.Cin + g * s.cpg + sl * kSlice;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int src = (16 * j + (lane >> 2)) << 2;
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        v[e] = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(gwv[e])));
                    const float val = (lane & 2) ? ((lane & 1) ? v[3] : v[2]) : ((lane & 1) ? v[1] : v[0]);
                    if (sl * kSlice + j * 64 + lane < s.cpg) atomicAdd(gw + j * 64 + lane, val);
                }
            }
        }
    }
}

// What follows the backward kernel, as one launch: the fp32 sums (offset part, then mask part) -> offset / mask gradient
// in their storage type (a NULL destination is skipped), and gwacc[k][c] (fp32) -> gw[c][0][k]
template <typename T>
__global__ void __launch_bounds__(256) dw_finish_kernel(const float *src, void *goff, void *gmask, int adt, long n_off,
                                                        long n_mask, const float *gwacc, T *gw, int C, int K)
{
    const long n_aux = n_off + n_mask, n = n_aux + (gw ? (long)C * K : 0);
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        if (i < n_off) {
            if (goff) st_aux(goff, i, adt, src[i]);
        } else if (i < n_aux) {
            if (gmask) st_aux(gmask, i - n_off, adt, src[i]);
        } else {
            const long q = i - n_aux;
            const int k = (int)(q % K), c = (int)(q / K);
            gw[q] = f32_to_elem<T>(gwacc[(long)k * C + c]);
        }
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

// `wt`: the weights as [K][C] (see dw_prepare_kernel)
template <typename T>
int d2c_depthwise_forward(const TiledShape &s, const void *xcl, const void *off, const void *mask, const void *wt,
                          const void *bias, void *out, hipStream_t st)
{
    DwArgs a{s, xcl, off, mask, wt, bias, out, nullptr, nullptr, nullptr, nullptr, nullptr};
    const int nsl = (s.cpg + kSlice - 1) / kSlice;
    D2cProfScope prof(D2C_PROF_FWD, st, "dw_fwd_kernel");
    hipLaunchKernelGGL(dw_fwd_kernel<T>, dim3(dw_grid(s, kFwdTP, s.G * nsl)), dim3(kDwThreads), kDwLdsFwd, st, a);
    return d2c_check_launch("dw_fwd_kernel");
}

// `goutcl` is the channels-last copy of grad_out, `wt` the weights as [K][C]; `xcl` ends with a row of zeros (voxel
// N * vol).  `gxcl` NULL: grad_input is not wanted
// here (or comes from the sample lists afterwards); otherwise it is accumulated with atomics.  The caller has zeroed
// `gwacc` and `auxacc`.
template <typename T>
int d2c_depthwise_backward(const TiledShape &s, const void *goutcl, const void *xcl, const void *off, const void *mask,
                           const void *wt, float *gxcl, void *goff, void *gmask, float *auxacc, float *gwacc, void *gw,
                           hipStream_t st)
{
    const long n_mask = (long)s.N * s.G * s.K * s.P, n_off = 3 * n_mask;
    float *auxoff = goff ? auxacc : nullptr, *auxmask = gmask ? auxacc + n_off : nullptr;
    if (gxcl) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        d2c_fill_zero(gxcl, (size_t)s.N * s.vol * s.Cin * sizeof(float), st);
    }
    DwArgs a{s, xcl, off, mask, wt, nullptr, nullptr, goutcl, gxcl, auxoff, auxmask, gwacc};
    const int nsl = (s.cpg + kSlice - 1) / kSlice;
    {
        auto kern = gxcl ? &dw_bwd_kernel<T, true> : &dw_bwd_kernel<T, false>;
        const size_t lds = dw_lds_bwd(sizeof(T));
        if (int rc = d2c_allow_lds((const void *)kern, (int)lds, "dw_bwd_kernel")) return rc;
        D2cProfScope prof(D2C_PROF_BWD_DATA, st, "dw_bwd_kernel");
        hipLaunchKernelGGL(kern, dim3(dw_grid(s, kBwdTP, s.G * nsl)), dim3(kDwThreads), lds, st, a);
    }
    if (int rc = d2c_check_launch("dw_bwd_kernel")) return rc;
    const bool want_gw = gwacc && gw;
    if (goff || gmask || want_gw) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        const long n_aux = (goff || gmask) ? n_off + n_mask : 0;
        hipLaunchKernelGGL(dw_finish_kernel<T>, dim3(g1d(n_aux + (want_gw ? (long)s.Cin * s.K : 0))), dim3(256), 0, st,
                           auxacc, goff, gmask, s.adt, (goff || gmask) ? n_off : 0, (goff || gmask) ? n_mask : 0, gwacc,
                           want_gw ? (T *)gw : nullptr, s.Cin, s.K);
        return d2c_check_launch("dw_finish_kernel");
    }
    return D2C_OK;
}

#define INST(T)                                                                                                      \
    template int d2c_depthwise_forward<T>(const TiledShape &, const void *, const void *, const void *, const void *, \
                                          const void *, void *, hipStream_t);                                        \
    template int d2c_depthwise_backward<T>(const TiledShape &, const void *, const void *, const void *,             \
                                           const void *, const void *, float *, void *, void *, float *, float *,    \
                                           void *, hipStream_t);
INST(bf16_t)
INST(float)
