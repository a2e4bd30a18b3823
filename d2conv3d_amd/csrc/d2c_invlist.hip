// grad_input without atomics: inverse sample lists + owner-computes gather.
//
// The reference scatters every sampled value into grad_input with atomicAdd
// (deformable_col2im_gpu_kernel, dconv3d_gpu.cu:562-643).  On this part fp32
// atomics retire at about one element per clock and L2 channel, which makes
// that scatter the slowest piece of the backward pass.  Here the scatter is
// turned around:
//
//   1. every live sample (b, g, k, p) is filed under its base voxel
//      floor(z, y, x) (a bucket of fixed capacity per voxel, filled in one pass;
//      what does not fit goes to an overflow array), with its tap, its three
//      fractions and its modulation;
//   2. the grad-column values gcol[p, (k, chunk), c] are written once by the
//      data kernel (in the element type of the call);
//   3. one 8-lane group per (2 x 2 x 2 voxel cube, channel chunk) walks the
//      lists of the 27 base voxels that can reach the cube, recomputes the
//      corner weights, reads each gcol row segment once and accumulates in
//      registers; every grad_input element is written exactly once.
#include "d2c_mma.hpp"
#include <utility>

#include "d2c_tiled.hpp"

int d2c_gx_mode();

namespace {

template <class F, int... I> D2C_DEV void for_each_const(F &&f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}

D2C_DEV int xcd_swizzle(int bid, int n)
{
    const int x = bid & 7, idx = bid >> 3;
    const int q = n >> 3, r = n & 7;
    return x * q + (x < r ? x : r) + idx;
}

// One pass over the samples that files them in the buckets (the offset / mask gradient kernel does the same
// on its way when it runs, see d2c_aux_grad.hip).
__global__ void __launch_bounds__(256)
lists_pass_kernel(TiledShape s, const void *off, const void *mask, SampleLists L)
{
    const int k = blockIdx.y;
    const int b = blockIdx.z / s.G, g = blockIdx.z - b * s.G;
    for (int p = blockIdx.x * blockDim.x + threadIdx.x; p < s.P; p += gridDim.x * blockDim.x) {
        const int ox = p % s.Wo, oy = (p / s.Wo) % s.Ho, oz = p / (s.Wo * s.Ho);
        float o0, o1, o2;
        load_offsets(s, off, b, g, k, p, o0, o1, o2);
        int bz, by, bx;
        tap_base(s.geo, k, oz, oy, ox, bz, by, bx);
        const Tap3<float> t = tiled_tap3(s, bz, by, bx, o0, o1, o2);
        if (!t.live) continue;
        InvEntry e;
        e.p = p; e.k = k; e.hz = t.hz; e.hy = t.hy; e.hx = t.hx;
        e.alpha = mask ? mask_act_rt(s.mact, ld_aux(mask, mask_index(s, b, g, k, p), s.adt), s.adt) : 1.f;
        e.pad0 = 0; e.pad1 = 0;
        lists_insert(L, bin_of(s, b, g, t.z0, t.y0, t.x0), e);
    }
}

// ---- owner-computes accumulation ------------------------------------------
// gcol layout: [chunk][tap][m = b*P + p][BKC] of T.
// One 8-lane group per 2 x 2 x 2 cube of voxels (and channel chunk): the 27
// base voxels that reach the cube are visited once each, and a grad-column row is read once for all the
// voxels of the cube it contributes to (27 list visits and row reads per 8 voxels instead of 64).
// Per axis, a base voxel at offset r in {0, 1, 2} from the cube's lower neighbour reaches cube voxel
// a in {0, 1} with weight:  r = 0: (h, -),  r = 1: (1 - h, h),  r = 2: (-, 1 - h).
// z and y offsets are compile-time (9 unrolled visits); the 3 base voxels along x are adjacent bins, one
// contiguous range of entries, the x offset of an entry follows from its place in the range.
//
// The bookkeeping of an entry is done ONCE, not by all 8 lanes of its group: a batch is 8
// entries, lane `sub` of the group loads and unpacks entry e0 + sub and works out where its grad-column row lies and
// the (up to 8) weights with which it reaches the cube's voxels; the others read those values with ds_swizzle (a
// broadcast inside the 8 lanes: the LDS crossbar, no LDS memory, no vector-ALU instruction).  Per entry a lane is
// left with the row load, the conversion of its channels and the multiply-adds: about 40 % fewer vector
// instructions than with every lane unpacking every entry, in a kernel that waits for its vector ALU as much as for
// memory (C=512 in 8 groups, 8x30x54: 0.415 -> 0.345 ms; float, C=256: 0.406 -> 0.308 ms).
// RB: rows of a batch requested together (8 for bfloat16, 4 for float: measured).
// SMALL (problems that make fewer than a few hundred of the large workgroups): a workgroup is 8 cubes (1 x 2 x 4)
// and nine wavefronts, one per (z, y) offset of the base voxels; each walks the three x bins of its offset for the 8
// cubes, the nine add their sums in LDS (ds_add_f32), and the workgroup stores the block.  The walk over the 27 base
// voxels of a cube is a chain of dependent loads (list entries, then rows), a ninth as long this way, on nine times
// the wavefronts.
template <int J> D2C_DEV int group8_bcast(int v) { return __builtin_amdgcn_ds_swizzle(v, 0x18 | (J << 5)); }
template <int J> D2C_DEV float group8_bcast(float v) { return __int_as_float(group8_bcast<J>(__float_as_int(v))); }

template <typename T, bool COMPACT, int RB, bool SMALL>
__global__ void __launch_bounds__(SMALL ? 576 : 256, SMALL ? 1 : 4)
gx_owner_cube_kernel(TiledShape s, const T *gcol, SampleLists L, float *gxcl, int c_lo, int c_n)
{
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC;
    constexpr int BY = SMALL ? 2 : 4, BZ = SMALL ? 1 : 2;          // cubes per workgroup: BZ x BY x 4
    const int sub = threadIdx.x & 7, ci = SMALL ? (threadIdx.x & 63) >> 3 : threadIdx.x >> 3;
    const int part = SMALL ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : 0;      // (z, y) offset of this wavefront
    const int ncx = (s.W + 1) / 2, ncy = (s.H + 1) / 2, ncz = (s.D + 1) / 2;
    const int nbx = (ncx + 3) / 4, nby = (ncy + BY - 1) / BY, nbz = (ncz + BZ - 1) / BZ;
    // Workgroups are dealt round-robin to the 8 XCDs.  An XCD takes a contiguous range of the blocks of cubes
    // (neighbours in space share bins and grad-column rows in its L2) and, block by block, the channel chunks one
    // after the other: the chunks of one offset group walk the same lists, which then come from L2.
    // (c_lo, c_n: the channel chunks this launch works on -- a slice of the backward pass, `gcol` then points where
    // chunk 0 WOULD start if the buffer held all chunks)
    const int nblk = s.N * nbz * nby * nbx, nch = c_n;
    const int xcd = blockIdx.x & 7, uidx = blockIdx.x >> 3;
    const int bq = nblk >> 3, br = nblk & 7;
    const int cidx = c_lo + uidx % nch, bi = uidx / nch;
    if (bi >= bq + (xcd < br ? 1 : 0)) return;
    int blk = xcd * bq + (xcd < br ? xcd : br) + bi;
    const int bx = blk % nbx; blk /= nbx;
    const int by = blk % nby; blk /= nby;
    const int bz = blk % nbz;
    const int b = blk / nbz;
    const int cx = bx * 4 + (ci & 3), cy = by * BY + ((ci >> 2) & (BY - 1)), cz = bz * BZ + (ci >> 2) / BY;
    const bool inside = cx < ncx && cy < ncy && cz < ncz;
    if (!SMALL && !inside) return;                        // (whole groups of 8 lanes leave together)
    __shared__ float s_sum[SMALL ? 8 * 8 * BKC : 1];      // [cube][voxel of the cube][channel]
    if constexpr (SMALL) {
        for (int i = threadIdx.x; i < 8 * 8 * BKC; i += 576) s_sum[i] = 0.f;
        __syncthreads();
    }
    const int x0 = cx * 2, y0 = cy * 2, z0 = cz * 2;
    const int g = (cidx * BKC) / s.cpg;
    float acc[2][2][2][VEC];
#pragma unroll
    for (int i = 0; i < 8 * VEC; i++) (&acc[0][0][0][0])[i] = 0.f;
    const T *gbase = gcol + ((long)cidx * s.K * s.M + (long)b * s.P) * BKC + sub * VEC;
    const int nxb = x0 + 1 < s.W ? 3 : 2;

#pragma unroll
    for (int rz = 0; rz < 3; rz++) {
        const int zb = z0 - 1 + rz;
        if (zb > s.D - 1) continue;
        if (SMALL && (rz != part % 3 || !inside)) continue;
#pragma unroll
        for (int ry = 0; ry < 3; ry++) {
            const int yb = y0 - 1 + ry;
            if (yb > s.H - 1) continue;
            if (SMALL && ry != part / 3) continue;
            const int bin1 = bin_of(s, b, g, zb, yb, x0 - 1);
            const int em1 = min(L.counts[bin1], L.cap);
            const int em2 = em1 + min(L.counts[bin1 + 1], L.cap);
            const int e1 = em2 + (nxb == 3 ? min(L.counts[bin1 + 2], L.cap) : 0);
            const uint4 *eb = reinterpret_cast<const uint4 *>(L.entries) + (long)bin1 * L.cap * (COMPACT ? 1 : 2);
            // this lane's entry of a batch (past the last one: the last one again, with weight zero), requested one
            // batch ahead
            uint4 q0n = make_uint4(0, 0, 0, 0), q1n = q0n;
            auto request = [&](int e0) {
                const int ec = max(min(e0 + sub, e1 - 1), 0);
                const int slot = ec < em1 ? ec : (ec < em2 ? ec - em1 + L.cap : ec - em2 + 2 * L.cap);
                if constexpr (COMPACT) {
                    q0n = eb[slot];
                } else {
                    q0n = eb[2 * slot]; q1n = eb[2 * slot + 1];
                }
            };
            if (e1 > 0) request(0);
            for (int e0 = 0; e0 < e1; e0 += 8) {
                const int ei = e0 + sub, ec = min(ei, e1 - 1);
                InvEntry en;
                if constexpr (COMPACT) {
                    en = unpack_entry(q0n);
                } else {
                    en.p = (int)q0n.x; en.k = (int)q0n.y;
                    en.hz = __uint_as_float(q0n.z); en.hy = __uint_as_float(q0n.w);
                    en.hx = __uint_as_float(q1n.x); en.alpha = __uint_as_float(q1n.y);
                }
                request(e0 + 8);
                const int rowi = en.k * s.M + en.p;          // (N * G * K * P is below 2^31: d2c_lists_supported)
                const float al = ei < e1 ? en.alpha : 0.f;
                const float hz = en.hz, hy = en.hy, hx = en.hx;
                // x: offset 0 (base x0-1) reaches voxel c=0 with hx; 1 reaches (1-hx, hx); 2 reaches c=1 with 1-hx
                const bool r0 = ec < em1, r2 = ec >= em2;
                const float wx0 = r0 ? hx : (r2 ? 0.f : 1.f - hx);
                const float wx1 = r0 ? 0.f : (r2 ? 1.f - hx : hx);
                float wq[2][2][2];
#pragma unroll
                for (int az = 0; az < 2; az++) {
                    if ((rz == 0 && az == 1) || (rz == 2 && az == 0)) continue;
                    const float wz = (rz == 0) ? hz : (rz == 2 ? 1.f - hz : (az ? hz : 1.f - hz));
#pragma unroll
                    for (int ay = 0; ay < 2; ay++) {
                        if ((ry == 0 && ay == 1) || (ry == 2 && ay == 0)) continue;
                        const float wy = (ry == 0) ? hy : (ry == 2 ? 1.f - hy : (ay ? hy : 1.f - hy));
                        const float wzy = wz * wy * al;
                        wq[az][ay][0] = wzy * wx0;
                        wq[az][ay][1] = wzy * wx1;
                    }
                }
                // ---- the 8 entries of the batch, RB rows at a time
                for_each_const([&](auto H) {
                    constexpr int h = decltype(H)::value * RB;
                    uint4 row[RB];
                    for_each_const([&](auto I) {
                        constexpr int i = decltype(I)::value;
                        const int rj = group8_bcast<h + i>(rowi);
                        row[i] = *reinterpret_cast<const uint4 *>(gbase + (long)rj * BKC);
                    }, std::make_integer_sequence<int, RB>{});
                    for_each_const([&](auto I) {
                        constexpr int i = decltype(I)::value;
                        const T *re = reinterpret_cast<const T *>(&row[i]);
                        float rv[VEC];
#pragma unroll
                        for (int j = 0; j < VEC; j++) rv[j] = elem_to_f32<T>(re[j]);
#pragma unroll
                        for (int az = 0; az < 2; az++) {
                            if ((rz == 0 && az == 1) || (rz == 2 && az == 0)) continue;
#pragma unroll
                            for (int ay = 0; ay < 2; ay++) {
                                if ((ry == 0 && ay == 1) || (ry == 2 && ay == 0)) continue;
                                const float w0 = group8_bcast<h + i>(wq[az][ay][0]);
                                const float w1 = group8_bcast<h + i>(wq[az][ay][1]);
#pragma unroll
                                for (int j = 0; j < VEC; j++) {
                                    acc[az][ay][0][j] = fmaf(w0, rv[j], acc[az][ay][0][j]);
                                    acc[az][ay][1][j] = fmaf(w1, rv[j], acc[az][ay][1][j]);
                                }
                            }
                        }
                    }, std::make_integer_sequence<int, RB>{});
                }, std::make_integer_sequence<int, 8 / RB>{});
            }
        }
    }
    if constexpr (SMALL) {
        const int prz = part % 3, pry = part / 3;
        if (inside) {
#pragma unroll
            for (int az = 0; az < 2; az++) {
                if ((prz == 0 && az == 1) || (prz == 2 && az == 0)) continue;      // (voxels this offset does not reach)
#pragma unroll
                for (int ay = 0; ay < 2; ay++) {
                    if ((pry == 0 && ay == 1) || (pry == 2 && ay == 0)) continue;
#pragma unroll
                    for (int ax = 0; ax < 2; ax++)
#pragma unroll
                        for (int i = 0; i < VEC; i++)
                            atomicAdd(&s_sum[(ci * 8 + az * 4 + ay * 2 + ax) * BKC + sub * VEC + i], acc[az][ay][ax][i]);
                }
            }
        }
        __syncthreads();
        for (int q = threadIdx.x; q < 8 * 8 * BKC / 4; q += 576) {
            const int c4 = q % (BKC / 4), v = (q / (BKC / 4)) & 7, cube = q / (8 * BKC / 4);
            const int z = (bz * BZ) * 2 + (v >> 2), y = (by * BY + (cube >> 2)) * 2 + ((v >> 1) & 1),
                      x = (bx * 4 + (cube & 3)) * 2 + (v & 1);
            if (z < s.D && y < s.H && x < s.W)
                *reinterpret_cast<float4 *>(gxcl + ((long)b * s.vol + ((long)z * s.H + y) * s.W + x) * s.Cin + cidx * BKC + c4 * 4) =
                    *reinterpret_cast<const float4 *>(&s_sum[q * 4]);
        }
        return;
    }
#pragma unroll
    for (int az = 0; az < 2; az++)
#pragma unroll
        for (int ay = 0; ay < 2; ay++)
#pragma unroll
            for (int ax = 0; ax < 2; ax++) {
                const int z = z0 + az, y = y0 + ay, x = x0 + ax;
                if (z < s.D && y < s.H && x < s.W) {
                    float *o = gxcl + ((long)b * s.vol + ((long)z * s.H + y) * s.W + x) * s.Cin + cidx * BKC + sub * VEC;
#pragma unroll
                    for (int i = 0; i < VEC; i += 4)
                        *reinterpret_cast<float4 *>(o + i) = make_float4(acc[az][ay][ax][i], acc[az][ay][ax][i + 1],
                                                                         acc[az][ay][ax][i + 2], acc[az][ay][ax][i + 3]);
                }
            }
}

// Samples that found their bucket full: added into grad_input with atomics, after the owner kernel has written
// it.  One 8-lane group per (overflow entry, channel chunk of its offset group).
template <typename T>
__global__ void __launch_bounds__(256)
gx_overflow_kernel(TiledShape s, const T *gcol, SampleLists L, float *gxcl, int c_lo, int c_n)
{
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC;
    const int novf = min(L.counts[L.nbins], L.ovf_cap);
    const int sub = threadIdx.x & 7;
    const int cpc = s.cpg / BKC;
    const long ngrp = (long)gridDim.x * 32, total = (long)novf * cpc;
    for (long w = (long)blockIdx.x * 32 + (threadIdx.x >> 3); w < total; w += ngrp) {
        const int i = (int)(w / cpc), jj = (int)(w - (long)i * cpc);
        const InvEntry e = L.ovf[i];
        int bin = e.pad0;
        const int x0 = bin % (s.W + 1) - 1; bin /= s.W + 1;
        const int y0 = bin % (s.H + 1) - 1; bin /= s.H + 1;
        const int z0 = bin % (s.D + 1) - 1; bin /= s.D + 1;
        const int g = bin % s.G, b = bin / s.G;
        const int cidx = (g * s.cpg) / BKC + jj;
        if (cidx < c_lo || cidx >= c_lo + c_n) continue;      // (another slice's sample)
        const uint4 row = *reinterpret_cast<const uint4 *>(gcol + (((long)cidx * s.K + e.k) * s.M + (long)b * s.P + e.p) * BKC
                                                           + sub * VEC);
        const T *re = reinterpret_cast<const T *>(&row);
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const int z = z0 + ((c >> 2) & 1), y = y0 + ((c >> 1) & 1), x = x0 + (c & 1);
            if (z < 0 || z >= s.D || y < 0 || y >= s.H || x < 0 || x >= s.W) continue;
            const float wgt = ((c & 4) ? e.hz : 1.f - e.hz) * ((c & 2) ? e.hy : 1.f - e.hy) * ((c & 1) ? e.hx : 1.f - e.hx)
                              * e.alpha;
            float *o = gxcl + ((long)b * s.vol + ((long)z * s.H + y) * s.W + x) * s.Cin + cidx * BKC + sub * VEC;
#pragma unroll
            for (int j = 0; j < VEC; j++) atomicAdd(o + j, wgt * elem_to_f32<T>(re[j]));
        }
    }
}

// ---- owner-computes accumulation, channel-separated (depthwise) case ---------
// gcol[p, k, c] = W[c, k] * gout[p, c] is one multiply, so no grad-column buffer
// exists: the owner of a voxel reads the channels-last grad_out row of each
// sample that reaches it and the weight row of its tap (staged in LDS).
// A workgroup = kOwnVox 2 x 2 x 2 cubes of voxels consecutive in x, one wavefront
// each, and a slice of kOwnSlice channels; a lane owns kOwnCV consecutive channels
// (one vector load per lane and row).  xcd_unit() gives every XCD one channel slice
// of one batch element at a time, so that the grad_out rows its workgroups gather
// (6.6 MB for 256 fp32 channels of 8x15x27 positions) stay in its L2.
constexpr int kOwnVox = 4, kOwnCV = 4, kOwnSlice = 64 * kOwnCV;

template <typename T> D2C_DEV void ld_vec4(const T *p, float *v)
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

// WLDS: the weights of the channel slice fit LDS (compile-time, so that the wait for a weight row is a wait for LDS
// alone and leaves the grad_out rows in flight).
template <typename T, bool WLDS>
__global__ void __launch_bounds__(64 * kOwnVox)
dw_gx_owner_kernel(TiledShape s, const T *goutcl, const T *wt, SampleLists L, float *gxcl)
{
    constexpr bool w_in_lds = WLDS;
    // One wavefront per 2 x 2 x 2 cube of voxels (kOwnVox cubes consecutive in x per workgroup, sharing the
    // weights of the channel slice in LDS): the lists of the 27 base voxels that reach the cube are walked once
    // each and a grad_out row is read once for all the voxels of the cube it contributes to, like
    // gx_owner_cube_kernel does for the dense case.
    extern __shared__ __align__(16) unsigned char smem[];
    T *s_w = reinterpret_cast<T *>(smem);   // [K][kOwnSlice] weights of the channel slice
    const int t = threadIdx.x & 63;
    // wavefront-uniform quantities, kept in scalar registers
    const int vox = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ncx = (s.W + 1) / 2, ncy = (s.H + 1) / 2, ncz = (s.D + 1) / 2;
    const int nbx = (ncx + kOwnVox - 1) / kOwnVox;
    const int nslice = (s.cpg + kOwnSlice - 1) / kOwnSlice;
    const XcdUnit un = xcd_unit(blockIdx.x, s.N * s.G * nslice, ncz * ncy * nbx);
    if (!un.ok) return;
    const int b = un.combo % s.N;
    const int g = (un.combo / s.N) / nslice, sl = (un.combo / s.N) % nslice;
    int blk = un.tile;
    const int xb = blk % nbx; blk /= nbx;
    const int cy = blk % ncy;
    const int cz = blk / ncy;
    const int cx = xb * kOwnVox + vox;
    const bool valid = cx < ncx;
    const int x0 = cx * 2, y0 = cy * 2, z0 = cz * 2;
    const int nxb = x0 + 1 < s.W ? 3 : 2;          // base voxels x0-1, x0, x0+1 (the last one only if it is a voxel)
    const T *grow = goutcl + (long)b * s.P * s.Cout;

    const int cl = sl * kOwnSlice + t * kOwnCV;   // first channel of this lane inside the offset group
    const bool cok = cl < s.cpg;                  // cpg is a multiple of kOwnCV
    // Lanes past the offset group stay in the walk (every lane holds a list entry for the others to read) on the
    // group's first channels and store nothing.
    const int c = g * s.cpg + (cok ? cl : 0);
    if (w_in_lds) {
        for (int i = threadIdx.x; i < s.K * kOwnSlice; i += 64 * kOwnVox) {
            const int k = i / kOwnSlice, cc = i - k * kOwnSlice;
            const int ch = sl * kOwnSlice + cc;
            s_w[i] = ch < s.cpg ? wt[(long)k * s.Cin + g * s.cpg + ch] : (T)0;
        }
        __syncthreads();
    }
    if (!valid) return;
    float acc[2][2][2][kOwnCV];
#pragma unroll
    for (int i = 0; i < 8 * kOwnCV; i++) (&acc[0][0][0][0])[i] = 0.f;

    // The walk is a software pipeline, because a wavefront has nobody to hide its latencies behind (the launch is
    // one round of 3 - 4 wavefronts per SIMD): the entries of a bucket are loaded by the lanes (lane e holds entry
    // e, two 16-byte loads for up to 64 entries) one bucket ahead and handed out with v_readlane; the grad_out rows
    // of kGE samples are requested while the kGE before them are worked on (C=1024, 8x15x27: 0.172 / 0.136 / 0.142 /
    // 0.158 ms with kGE = 1 / 2 / 4 / 8; a ring of three pairs: 0.139).
    constexpr int kGE = 2;
    unsigned cbytes = (unsigned)c * (unsigned)sizeof(T);
    asm("" : "+v"(cbytes));
    auto bucket = [&](int bi, uint4 &ea, uint4 &eb, int &n, int &bin) {
        const int rz = bi / 9, ry = (bi / 3) % 3, rx = bi % 3;
        const bool ok = z0 - 1 + rz <= s.D - 1 && y0 - 1 + ry <= s.H - 1 && rx < nxb;
        bin = ok ? bin_of(s, b, g, z0 - 1 + rz, y0 - 1 + ry, x0 - 1 + rx) : 0;
        n = ok ? min(L.counts[bin], L.cap) : 0;
        const uint4 *ep = reinterpret_cast<const uint4 *>(L.entries + (long)bin * L.cap + min(t, L.cap - 1));
        ea = ep[0]; eb = ep[1];
    };
    // rows of entries e0 .. e0 + kGE - 1 of the m the lanes hold (past the last one: the last one again)
    auto rows = [&](float (*go)[kOwnCV], const uint4 &ea, int e0, int m) {
        unsigned cb = cbytes;
        // (keeps the loads in the scalar-base + 32-bit-offset form; not volatile: the bucket counts stay scalar loads)
        asm("" : "+v"(cb));
#pragma unroll
        for (int i = 0; i < kGE; i++) {
            const int pp = __builtin_amdgcn_readlane((int)ea.x, min(e0 + i, m - 1));
            ld4_row<T>(grow + (size_t)pp * s.Cout, cb, go[i]);
        }
    };
    uint4 ca, cb4, na = make_uint4(0, 0, 0, 0), nb = na;
    int cn, cbin, nn = 0, nbin = 0;
    bucket(0, ca, cb4, cn, cbin);
    // (one copy of the code per bucket: its place in the 3 x 3 x 3 neighbourhood decides which voxels it reaches)
    for_each_const([&](auto BI) {
        constexpr int bi = decltype(BI)::value;
        constexpr int rz = bi / 9, ry = (bi / 3) % 3, rx = bi % 3;
        // The weights with which a sample reaches its 8 corners, times its modulation: every lane works them out
        // for the entry it holds (64 entries per instruction), the walk below reads them out with v_readlane.
        // Corner (dz, dy, dx) of a sample filed under base voxel r = (rz, ry, rx) is cube voxel a = d + r - 1.
        float cw[8];
        auto corner_weights = [&](const uint4 &ea, const uint4 &eb) {
            const float hz = __uint_as_float(ea.z), hy = __uint_as_float(ea.w), hx = __uint_as_float(eb.x);
            const float al = __uint_as_float(eb.y);
            const float lz = 1.f - hz, ly = 1.f - hy, lx = 1.f - hx;
            const float zy[4] = {lz * ly * al, lz * hy * al, hz * ly * al, hz * hy * al};
#pragma unroll
            for (int q = 0; q < 4; q++) {
                cw[2 * q] = zy[q] * lx;
                cw[2 * q + 1] = zy[q] * hx;
            }
        };
        auto work = [&](const float (*go)[kOwnCV], const uint4 &ea, int e0, int m) {
#pragma unroll
            for (int i = 0; i < kGE; i++) {
                const int e = e0 + i;
                if (e >= m) break;
                const int k = __builtin_amdgcn_readlane((int)ea.y, e);
                float wk[kOwnCV];
                if (w_in_lds) ld_vec4<T>(s_w + k * kOwnSlice + t * kOwnCV, wk);
                else ld_vec4<T>(wt + (long)k * s.Cin + c, wk);
                float v[kOwnCV];
#pragma unroll
                for (int jj = 0; jj < kOwnCV; jj++) v[jj] = wk[jj] * go[i][jj];
#pragma unroll
                for (int az = 0; az < 2; az++) {
                    constexpr int dz0 = 1 - rz;
                    if (az + dz0 < 0 || az + dz0 > 1) continue;
#pragma unroll
                    for (int ay = 0; ay < 2; ay++) {
                        constexpr int dy0 = 1 - ry;
                        if (ay + dy0 < 0 || ay + dy0 > 1) continue;
#pragma unroll
                        for (int ax = 0; ax < 2; ax++) {
                            constexpr int dx0 = 1 - rx;
                            if (ax + dx0 < 0 || ax + dx0 > 1) continue;
                            const int corner = (az + dz0) * 4 + (ay + dy0) * 2 + (ax + dx0);
                            const float w = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cw[corner]), e));
#pragma unroll
                            for (int jj = 0; jj < kOwnCV; jj++) acc[az][ay][ax][jj] = fmaf(w, v[jj], acc[az][ay][ax][jj]);
                        }
                    }
                }
            }
        };
        float goA[kGE][kOwnCV], goB[kGE][kOwnCV];
        if (cn > 0) {
            int m = min(cn, 64);
            rows(goA, ca, 0, m);
            if (bi + 1 < 27) bucket(bi + 1, na, nb, nn, nbin);
            for (int base = 0;;) {
                corner_weights(ca, cb4);
                for (int e0 = 0; e0 < m; e0 += 2 * kGE) {
                    rows(goB, ca, e0 + kGE, m);
                    work(goA, ca, e0, m);
                    rows(goA, ca, e0 + 2 * kGE, m);
                    work(goB, ca, e0 + kGE, m);
                }
                // buckets of more than 64 entries (large kernels): the next 64, not ahead of time
                base += 64;
                if (base >= cn) break;
                m = min(cn - base, 64);
                const uint4 *ep = reinterpret_cast<const uint4 *>(L.entries + (long)cbin * L.cap + min(base + t, L.cap - 1));
                ca = ep[0]; cb4 = ep[1];
                rows(goA, ca, 0, m);
            }
        } else if (bi + 1 < 27) {
            bucket(bi + 1, na, nb, nn, nbin);
        }
        ca = na; cb4 = nb; cn = nn; cbin = nbin;
    }, std::make_integer_sequence<int, 27>{});
#pragma unroll
    for (int az = 0; az < 2; az++)
#pragma unroll
        for (int ay = 0; ay < 2; ay++)
#pragma unroll
            for (int ax = 0; ax < 2; ax++) {
                const int z = z0 + az, y = y0 + ay, x = x0 + ax;
                if (cok && z < s.D && y < s.H && x < s.W) {
                    const long vg = (long)b * s.vol + ((long)z * s.H + y) * s.W + x;
                    *reinterpret_cast<float4 *>(gxcl + vg * s.Cin + c) =
                        make_float4(acc[az][ay][ax][0], acc[az][ay][ax][1], acc[az][ay][ax][2], acc[az][ay][ax][3]);
                }
            }
}

// The samples that found their bucket full (usually none), added with atomics: one 64-lane group per (entry, 256
// channels of its offset group), a lane owns kOwnCV channels.
template <typename T>
__global__ void __launch_bounds__(256)
dw_gx_overflow_kernel(TiledShape s, const T *goutcl, const T *wt, SampleLists L, float *gxcl)
{
    const int novf = min(L.counts[L.nbins], L.ovf_cap);
    const int t = threadIdx.x & 63;
    const int nslice = (s.cpg + kOwnSlice - 1) / kOwnSlice;
    const long ngrp = (long)gridDim.x * 4, total = (long)novf * nslice;
    for (long w = (long)blockIdx.x * 4 + (threadIdx.x >> 6); w < total; w += ngrp) {
        const int i = (int)(w / nslice), sl = (int)(w - (long)i * nslice);
        const InvEntry e = L.ovf[i];
        int bin = e.pad0;
        const int x0 = bin % (s.W + 1) - 1; bin /= s.W + 1;
        const int y0 = bin % (s.H + 1) - 1; bin /= s.H + 1;
        const int z0 = bin % (s.D + 1) - 1; bin /= s.D + 1;
        const int g = bin % s.G, b = bin / s.G;
        const int cl = sl * kOwnSlice + t * kOwnCV;
        if (cl >= s.cpg) continue;
        const int c = g * s.cpg + cl;
        float go[kOwnCV], wk[kOwnCV];
        ld_vec4<T>(goutcl + ((long)b * s.P + e.p) * s.Cout + c, go);
        ld_vec4<T>(wt + (long)e.k * s.Cin + c, wk);
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const int z = z0 + ((q >> 2) & 1), y = y0 + ((q >> 1) & 1), x = x0 + (q & 1);
            if (z < 0 || z >= s.D || y < 0 || y >= s.H || x < 0 || x >= s.W) continue;
            const float wgt = ((q & 4) ? e.hz : 1.f - e.hz) * ((q & 2) ? e.hy : 1.f - e.hy) * ((q & 1) ? e.hx : 1.f - e.hx)
                              * e.alpha;
            float *o = gxcl + ((long)b * s.vol + ((long)z * s.H + y) * s.W + x) * s.Cin + c;
#pragma unroll
            for (int j = 0; j < kOwnCV; j++) atomicAdd(o + j, wgt * (wk[j] * go[j]));
        }
    }
}

inline unsigned g1d(long n, int cap = 16384)
{
    long g = (n + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > cap ? cap : g));
}

}  // namespace

// ------------------------------------------------------------------ host
long d2c_invlist_bins(const TiledShape &s) { return (long)s.N * s.G * (s.D + 1) * (s.H + 1) * (s.W + 1); }

// Bucket capacity: a power of two above 2.2 x the mean list length K * P / vol (8 .. 256), or what
// d2c_set_grad_input_mode() asked for.
int d2c_lists_cap(const TiledShape &s)
{
    const int forced = d2c_gx_mode();
    if (forced >= 2) return forced;
    const double mean = (double)s.K * s.P / s.vol;
    int cap = 8;
    while (cap < 256 && cap < 2.2 * mean) cap *= 2;
    return cap;
}
// 16-byte bucket entries: bfloat16 problems whose position and tap fit 24 + 8 bits
bool d2c_lists_compact(const TiledShape &s, int dtype) { return dtype == D2C_BF16 && s.P < (1 << 24) && s.K < 256; }
void d2c_lists_ws(const TiledShape &s, int dtype, size_t *counts, size_t *entries, size_t *ovf)
{
    const long nb = d2c_invlist_bins(s);
    *counts = d2c_align_up((size_t)(nb + 1) * 4);
    *entries = d2c_align_up((size_t)nb * d2c_lists_cap(s) * (d2c_lists_compact(s, dtype) ? 16 : sizeof(InvEntry)));
    *ovf = d2c_align_up((size_t)s.N * s.G * s.K * s.P * sizeof(InvEntry));
}
// Bins and samples are counted in 32 bits; larger problems take the atomic scatter instead.
bool d2c_lists_supported(const TiledShape &s)
{
    return d2c_invlist_bins(s) < (1L << 31) - 1 && (long)s.N * s.G * s.K * s.P < (1L << 31);
}
// The lists over the three workspace regions sized by d2c_lists_ws; nbins == 0 when the shape is too large.
SampleLists d2c_lists_make(const TiledShape &s, int dtype, void *counts, void *entries, void *ovf)
{
    const long nb = d2c_invlist_bins(s), nsamp = (long)s.N * s.G * s.K * s.P;
    SampleLists L{(int *)counts, (InvEntry *)entries, (InvEntry *)ovf, d2c_lists_cap(s), 0, 0,
                  d2c_lists_compact(s, dtype) ? 1 : 0};
    if (nb < (1L << 31) - 1 && nsamp < (1L << 31)) {
        L.nbins = (int)nb;
        L.ovf_cap = (int)nsamp;
    }
    return L;
}
int d2c_lists_clear(const SampleLists &L, hipStream_t st)
{
    if (L.nbins == 0) {
        d2c_set_error("too many sample bins");
        return D2C_ERR_UNSUPPORTED;
    }
    D2cProfScope prof(D2C_PROF_PACK, st);
    d2c_fill_zero(L.counts, (size_t)(L.nbins + 1) * 4, st);
    return d2c_check_launch("lists_clear");
}
int d2c_lists_fill(const TiledShape &s, const void *off, const void *mask, const SampleLists &L, hipStream_t st);
int d2c_lists_build(const TiledShape &s, const void *off, const void *mask, const SampleLists &L, hipStream_t st)
{
    if (int rc = d2c_lists_clear(L, st)) return rc;
    return d2c_lists_fill(s, off, mask, L, st);
}
// ... the same on counts that the caller has cleared
int d2c_lists_fill(const TiledShape &s, const void *off, const void *mask, const SampleLists &L, hipStream_t st)
{
    if (L.nbins == 0) {
        d2c_set_error("too many sample bins");
        return D2C_ERR_UNSUPPORTED;
    }
    D2cProfScope prof(D2C_PROF_PACK, st);
    const dim3 pgrid(g1d(s.P, 4096), s.K, s.N * s.G);
    hipLaunchKernelGGL(lists_pass_kernel, pgrid, dim3(256), 0, st, s, off, mask, L);
    return d2c_check_launch("lists_pass_kernel");
}

template <typename T>
int d2c_gx_owner_launch(const TiledShape &s, const void *gcol, const SampleLists &L, float *gxcl, hipStream_t st,
                        int c_lo, int c_n)
{
    constexpr int BKC = 8 * Elem<T>::VEC;
    if (c_n <= 0) { c_lo = 0; c_n = s.Cin / BKC; }
    D2cProfScope prof(D2C_PROF_GX_OWNER, st, "gx_owner_cube_kernel");
    const int ncx = (s.W + 1) / 2, ncy = (s.H + 1) / 2, ncz = (s.D + 1) / 2;
    const long nblk = (long)s.N * ((ncz + 1) / 2) * ((ncy + 3) / 4) * ((ncx + 3) / 4);
    constexpr int RB = sizeof(T) == 2 ? 8 : 4;
    // (512 channels on 8x15x27, 128 large workgroups: backward pass 0.41 -> 0.36 ms; 128 channels on 8x30x54, 112:
    // 0.31 -> 0.27; from 224 workgroups on -- 256 channels on 8x30x54 -- the large workgroups are faster)
    if (8 * ((nblk + 7) / 8) * c_n < 160) {
        const long nblk8 = (long)s.N * ncz * ((ncy + 1) / 2) * ((ncx + 3) / 4);
        dim3 grid((unsigned)(8 * ((nblk8 + 7) / 8) * c_n));
        if (L.compact) hipLaunchKernelGGL((gx_owner_cube_kernel<T, true, RB, true>), grid, dim3(576), 0, st, s, (const T *)gcol, L, gxcl, c_lo, c_n);
        else hipLaunchKernelGGL((gx_owner_cube_kernel<T, false, RB, true>), grid, dim3(576), 0, st, s, (const T *)gcol, L, gxcl, c_lo, c_n);
    } else {
        dim3 grid((unsigned)(8 * ((nblk + 7) / 8) * c_n));    // see the kernel's unit mapping
        if (L.compact) hipLaunchKernelGGL((gx_owner_cube_kernel<T, true, RB, false>), grid, dim3(256), 0, st, s, (const T *)gcol, L, gxcl, c_lo, c_n);
        else hipLaunchKernelGGL((gx_owner_cube_kernel<T, false, RB, false>), grid, dim3(256), 0, st, s, (const T *)gcol, L, gxcl, c_lo, c_n);
    }
    if (int rc = d2c_check_launch("gx_owner_kernel")) return rc;
    // the overflow entries, usually none (the kernel reads their number from device memory)
    hipLaunchKernelGGL(gx_overflow_kernel<T>, dim3(512), dim3(256), 0, st, s, (const T *)gcol, L, gxcl, c_lo, c_n);
    return d2c_check_launch("gx_overflow_kernel");
}
template int d2c_gx_owner_launch<bf16_t>(const TiledShape &, const void *, const SampleLists &, float *, hipStream_t, int, int);
template int d2c_gx_owner_launch<float>(const TiledShape &, const void *, const SampleLists &, float *, hipStream_t, int, int);

// Depthwise case: grad_input from the sample lists, the channels-last grad_out and the tap-major weights.
template <typename T>
int d2c_dw_gx_owner_launch(const TiledShape &s, const void *goutcl, const void *wt, const SampleLists &L, float *gxcl,
                           hipStream_t st)
{
    size_t lds = (size_t)s.K * kOwnSlice * sizeof(T);
    const bool w_in_lds = lds <= 144 * 1024;
    if (!w_in_lds) lds = 0;
    auto kern = w_in_lds ? &dw_gx_owner_kernel<T, true> : &dw_gx_owner_kernel<T, false>;
    if (int rc = d2c_allow_lds((const void *)kern, 160 * 1024, "dw_gx_owner_kernel")) return rc;
    D2cProfScope prof(D2C_PROF_GX_OWNER, st, "dw_gx_owner_kernel");
    const int ncx = (s.W + 1) / 2, ncy = (s.H + 1) / 2, ncz = (s.D + 1) / 2;
    const int nslice = (s.cpg + kOwnSlice - 1) / kOwnSlice;
    const unsigned nblk = xcd_unit_grid(s.N * s.G * nslice, ncz * ncy * ((ncx + kOwnVox - 1) / kOwnVox));
    hipLaunchKernelGGL(kern, dim3(nblk), dim3(64 * kOwnVox), lds, st, s, (const T *)goutcl, (const T *)wt, L, gxcl);
    if (int rc = d2c_check_launch("dw_gx_owner_kernel")) return rc;
    // the overflow entries, usually none (the kernel reads their number from device memory)
    hipLaunchKernelGGL(dw_gx_overflow_kernel<T>, dim3(256), dim3(256), 0, st, s, (const T *)goutcl, (const T *)wt, L, gxcl);
    return d2c_check_launch("dw_gx_overflow_kernel");
}
template int d2c_dw_gx_owner_launch<bf16_t>(const TiledShape &, const void *, const void *, const SampleLists &, float *,
                                            hipStream_t);
template int d2c_dw_gx_owner_launch<float>(const TiledShape &, const void *, const void *, const SampleLists &, float *,
                                           hipStream_t);

