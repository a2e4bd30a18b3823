// grad_offset / grad_mask from the grad-column rows (dconv3d_gpu.cu:708-864,
// dconv1d_gpu.cu:318-352), as a kernel of its own.
//
//   dot[corner]  = sum_c gcol[p, k, c] * x[corner(p, k), c]          (c over the channels of the offset group)
//   grad_mask    = sum_corner a_corner * dot[corner]                 (corners of the forward pass)
//   grad_offset  = alpha * sum_corner (d a_corner / d axis) * dot[corner]   (corners gated by range only)
//
// The data kernel writes the grad-column rows [chunk][tap][N*P][BKC] anyway (the
// list-based grad_input reads them).  Doing the dot products here instead of
// inside that kernel frees them from its register budget (its stationary
// operand fills the register file) and from its barriers: here every wavefront
// works alone (no workgroup synchronisation at all), needs few registers, and
// twenty of them per CU hide each other's memory latency.
//
// One wavefront = 64 output positions of one offset group and a share of the
// taps.  Per tap: lane = position computes the corner table of the 64 positions
// (kept in registers, read across lanes with ds_bpermute: no LDS is allocated);
// then, per channel chunk of the group, 8 rounds of
// lane = (position, 16-byte vector): 8 corner vectors + 1 grad-column vector ->
// 8 dot products -> the 4 results (linear in the dots) -> sum over the 8 lanes
// of the position.
#include "d2c_mma.hpp"
#include "d2c_tiled.hpp"

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kMT = 64;                    // positions per wavefront
constexpr int kTab = 9;                    // table words per position: idx, flag, lz ly lx hz hy hx, alpha
constexpr int kRounds = 1;                 // rounds whose loads are in flight together
constexpr int kTapSplit = 27;              // wavefronts per (tile, group), each with its share of the taps: many short
                                           // tasks balance better than few long ones (C=512, 8 groups, 27 taps:
                                           // 0.67 ms at 3 shares, 0.57 at 9, 0.54 at 27; one group of 256 channels
                                           // on 207360 positions: 2.65 / 2.11 / 1.75 ms)

struct AuxArgs {
    TiledShape s;
    const void *xcl;     // [N][vol][Cin]
    const void *off, *mask;
    const void *gcol;    // [chunk][tap][N*P][BKC]
    void *goff, *gmask;  // or NULL
    float *gsize;        // size-map source: fp32 sums [N][3][P] of d(loss)/d(size) per axis (zeroed), instead of goff
    int ntile;           // position tiles
    int nshare;          // tap shares
    SampleLists lists;   // counts != NULL: every live sample is filed in its bucket on the way (for grad_input)
    void *col;           // COL: the sampled columns [chunk][tap][mpad][BKC] (what the forward pass multiplied with W),
    long mpad;           //      rows of all `ntile` position tiles (zeros past the last position); or, in place of the
                         //      grad-column rows (`col` == `gcol`, which nobody reads after this kernel then): N*P rows
    int g_lo, g_n;       // the offset groups [g_lo, g_lo + g_n) this launch works on (a slice of the backward pass;
                         // `gcol` and `col` then point where chunk 0 WOULD start if the buffers held all chunks)
    unsigned xbytes;     // size of `xcl` (below 4 GiB: the matrix kernels address it with 32-bit byte offsets)
};

// Gathers through buffer descriptors.  A load whose offset lies past the descriptor's size returns zeros without
// touching memory: a corner outside the volume, or a position without any corner in range, gets the offset
// kOutside, and neither a branch around the load nor registers cleared beforehand are needed.
constexpr unsigned kOutside = 0xFFFFFFF0u;
typedef unsigned u32x4_b __attribute__((ext_vector_type(4)));
D2C_DEV __amdgpu_buffer_rsrc_t gather_rsrc(const void *p, unsigned bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);   // raw buffer of dwords
}
// `off` when bit `bit` of `keep` is set, kOutside otherwise (kOutside has all the bits of a 16-byte aligned offset)
D2C_DEV unsigned offset_or_outside(unsigned off, unsigned keep, int bit)
{
    const unsigned drop = (unsigned)((int)(~keep << (31 - bit)) >> 31);   // all ones when the bit is clear
    return (drop & kOutside) | off;
}
template <int AUX> D2C_DEV uint4 ld_gather16(__amdgpu_buffer_rsrc_t r, unsigned off)
{
    const u32x4_b v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, AUX);
    return make_uint4(v[0], v[1], v[2], v[3]);
}

// Sum over the 8 lanes of a position without LDS traffic: neighbours of a quad, the other pair of the quad, then
// the other quad of the 8 (row_half_mirror: lane i reads lane 7 - i of its half row; all lanes of a quad hold the
// same value by then).
template <int CTRL> D2C_DEV float dpp_add(float v)
{
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
D2C_DEV float sum_over_8_lanes(float v)
{
    v = dpp_add<0xB1>(v);     // quad_perm [1, 0, 3, 2]
    v = dpp_add<0x4E>(v);     // quad_perm [2, 3, 0, 1]
    return dpp_add<0x141>(v); // row_half_mirror
}

// COL: the kernel also writes the sampled, modulated columns alpha * sum_corner a_corner * x[corner, c] of every
// (position, tap, channel) -- the corner vectors are in its registers anyway -- so that the grad-weight product
// can run as a plain matrix product over them (tiled_bwd_weight_col_kernel) instead of sampling the input again.
template <typename T, bool AUX16, bool SIZED, bool COL>
__global__ void __launch_bounds__(64 * kWavesPerBlock) aux_grad_kernel(AuxArgs a)
{
    constexpr int MT = kMT;
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC;
    const TiledShape &s = a.s;
    const int lane = threadIdx.x & 63;
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // The corner table of the 64 positions of a tap lives in registers (lane = position) and is read by the
    // lanes of the dot-product role with ds_bpermute: the kernel allocates no LDS, so its workgroups fit on a
    // compute unit next to a kernel that fills the LDS.
    float tab[kTab];
    auto tab_of = [&](int i, int pos) {
        return __int_as_float(__builtin_amdgcn_ds_bpermute(pos << 2, __float_as_int(tab[i])));
    };
    // wavefront task = (tile, offset group, tap share).  Workgroups are dealt round-robin to the 8 XCDs, each
    // with an L2 of its own: an XCD works on one part of the positions (tiles that are neighbours in space
    // share its L2).  Its sequence of workgroups: the tap shares of a block of tiles one after the other (their
    // corner rows are the same ones), then the next block of the part, and only then the next offset group, with
    // another part (measured at 8 groups, C=512: 0.65 -> 0.57 ms against tap shares outermost, where the rows of
    // a block were long gone from L2 when its next share came round).  Groups are taken last to first: the
    // grad-column rows of the last groups are the ones the kernel in front wrote last, and what the memory-side
    // cache still holds of them is read first (0.590 -> 0.576 ms).
    const int nblk = (a.ntile + kWavesPerBlock - 1) / kWavesPerBlock, nblk_p = (nblk + 7) / 8;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int share = idx % a.nshare, g = a.g_lo + a.g_n - 1 - idx / (nblk_p * a.nshare);
    const int blk = ((xcd + 3 * g) & 7) * nblk_p + (idx / a.nshare) % nblk_p;
    if (blk >= nblk) return;
    const int tile = blk * kWavesPerBlock + wib;
    if (tile >= a.ntile) return;
    const int k_lo = (int)((long)s.K * share / a.nshare), k_hi = (int)((long)s.K * (share + 1) / a.nshare);
    const int m0 = tile * MT;
    const int cpc = s.cpg / BKC;                   // chunks per offset group
    const int dzc = s.H * s.W * s.Cin, dyc = s.W * s.Cin;

    // lane = position (coordinate role)
    int cb = 0, cp = 0, coz = 0, coy = 0, cox = 0;
    const bool cvalid = m0 + lane < s.M;
    if (cvalid) {
        const int m = m0 + lane;
        cb = m / s.P; cp = m - cb * s.P;
        cox = cp % s.Wo; coy = (cp / s.Wo) % s.Ho; coz = cp / (s.Wo * s.Ho);
    }
    // lane = (position of the round, vector) (dot-product role)
    const int rpos = lane >> 3, ivec = lane & 7;
    const __amdgpu_buffer_rsrc_t xres = gather_rsrc(a.xcl, a.xbytes);
    const char *gcb = reinterpret_cast<const char *>(a.gcol);
    const unsigned grow_bytes = (unsigned)s.M * (unsigned)(BKC * sizeof(T));   // rows of one (chunk, tap): below 4 GiB

    // offsets and modulation of a tap are requested while the previous tap is being worked on
    float craw[4] = {0.f, 0.f, 0.f, 1.f};
    auto coords_issue = [&](int k) {
        if (cvalid) {
            tap_offsets_issue<AUX16, SIZED>(s, a.off, cb, g, k, cp, craw);
            craw[3] = a.mask ? ld_auxT<AUX16>(a.mask, mask_index(s, cb, g, k, cp)) : 1.f;
        }
    };
    if (k_lo < k_hi) coords_issue(k_lo);

    // COL: a column vector is stored one round late, right behind the loads of the next round: those loads are
    // then older than the store, and the wait for them leaves the store in flight for a whole round
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    u32x4 pend_v = {0u, 0u, 0u, 0u};
    u32x4 *pend_p = nullptr;
    for (int k = k_lo; k < k_hi; k++) {
        int lbin = -1, lslot = 0;
        float lhx = 0.f;
        // ---- corner table of the 64 positions for tap k
        {
            float fr[6] = {0, 0, 0, 0, 0, 0};
            float al = 0.f;
            int idx = 0, flag = 0;
            if (cvalid) {
                tap_offsets_finish<AUX16, SIZED>(s, k, craw);
                const float o0 = craw[0], o1 = craw[1], o2 = craw[2];
                typedef typename std::conditional<AUX16, bf16_t, float>::type AT;
                al = (s.mact && a.mask) ? mask_act<AT>(s.mact, craw[3]) : craw[3];
                int bz, by, bx;
                tap_base(s.geo, k, coz, coy, cox, bz, by, bx);
                const Tap3<float> t = tiled_tap3(s, bz, by, bx, o0, o1, o2);
                idx = (cb * s.vol + (t.z0 * s.H + t.y0) * s.W + t.x0) * s.Cin;   // element offset of corner 000
                unsigned inr = t.inrange, auxlive = t.live;
                fr[0] = t.lz; fr[1] = t.ly; fr[2] = t.lx; fr[3] = t.hz; fr[4] = t.hy; fr[5] = t.hx;
                if (a.lists.counts && t.live) {
                    // a place in the sample's bucket is asked for now, the entry is written after the dot
                    // products of this tap, when the answer has long arrived
                    lbin = bin_of(s, cb, g, t.z0, t.y0, t.x0);
                    lslot = lists_reserve(a.lists, lbin);
                    lhx = t.hx;
                }
                if (s.nd == 1) {
                    // 1-D: both corners are gated by range only (dconv1d_gpu.cu:338-339), and at integer
                    // positions the low corner steps down by one while the high corner stays (:332-336);
                    // grad_offset / grad_mask then interpolate with t' = x - (x0 - 1).
                    int x0q = t.x0;
                    if (s.quirks && (double)t.hx < 1e-8) {
                        x0q -= 1;
                        flag |= 1 << 16;
                        const float x = (float)bx + o2;
                        const float tq = x - (float)x0q;
                        fr[2] = 1.f - tq; fr[5] = tq;
                    }
                    const unsigned lo = (x0q >= 0 && x0q < s.W) ? 1u : 0u;
                    const unsigned hi = (t.x0 + 1 >= 0 && t.x0 + 1 < s.W) ? 2u : 0u;
                    inr = lo | hi;
                    auxlive = inr;
                }
                flag |= (int)((inr << 8) | (auxlive << 24));
            }
            tab[0] = __int_as_float(idx);
            tab[1] = __int_as_float(flag);
#pragma unroll
            for (int c = 0; c < 6; c++) tab[2 + c] = fr[c];
            tab[8] = al;
            if (k + 1 < k_hi) coords_issue(k + 1);
        }

        // ---- dot products: 8 rounds of 8 positions x 8 vectors, kRounds at a time; sums over the chunks of the group
#pragma unroll 1
        for (int rp = 0; rp < 8 / kRounds; rp++) {
            float g_acc[kRounds][4];
#pragma unroll
            for (int r = 0; r < kRounds; r++) g_acc[r][0] = g_acc[r][1] = g_acc[r][2] = g_acc[r][3] = 0.f;
#pragma unroll 1
            for (int jj = 0; jj < cpc; jj++) {
                const int c0 = g * s.cpg + jj * BKC;
                // the grad-column rows of this (chunk, tap)
                const __amdgpu_buffer_rsrc_t gres =
                    gather_rsrc(gcb + ((long)(c0 / BKC) * s.K + k) * (long)grow_bytes, grow_bytes);
                uint4 xv[kRounds][8], gq[kRounds];
                // all loads of these rounds are requested before any of them is used
#pragma unroll
                for (int r = 0; r < kRounds; r++) {
                    const int pos = (rp * kRounds + r) * 8 + rpos;
                    const int idx = __float_as_int(tab_of(0, pos));
                    const unsigned flag = (unsigned)__float_as_int(tab_of(1, pos));
                    const unsigned inr = (flag >> 8) & 0xffu;
                    const int qshift = (flag >> 16) & 1;
                    const int ib = idx + c0 + ivec * VEC;
#pragma unroll
                    for (int c = 0; c < 8; c++) {
                        const unsigned o = (unsigned)(ib + ((c >> 2) & 1) * dzc + ((c >> 1) & 1) * dyc
                                                      + ((c & 1) ? s.Cin : -qshift * s.Cin)) * (unsigned)sizeof(T);
                        xv[r][c] = ld_gather16<0>(xres, offset_or_outside(o, inr, c));
                    }
                    // (the grad-column row: read once by this kernel, a streaming load)
                    const unsigned go = (unsigned)((m0 + pos) * BKC + ivec * VEC) * (unsigned)sizeof(T);
                    gq[r] = ld_gather16<2>(gres, inr ? go : kOutside);
                }
                if constexpr (COL) {
                    // (a streaming store: written once, read by another kernel much later; it leaves the rows that
                    // this kernel gathers in the L2)
                    if (pend_p) __builtin_nontemporal_store(pend_v, pend_p);
                }
#pragma unroll
                for (int r = 0; r < kRounds; r++) {
                    const int pos = (rp * kRounds + r) * 8 + rpos;
                    const unsigned live = (unsigned)__float_as_int(tab_of(1, pos)) >> 24;
                    if constexpr (COL) {
                        // corner weights as in the forward pass (dconv3d_gpu.cu:88-95: wz * wy * wx, then the
                        // modulation); a point that is not live contributes nothing, corners out of range read zeros
                        // (the exchange first, with every lane taking part, then the choice)
                        const float al_pos = tab_of(8, pos);
                        const float alv = live ? al_pos : 0.f;
                        const float cz[2] = {tab_of(2, pos) * alv, tab_of(5, pos) * alv}, cy[2] = {tab_of(3, pos), tab_of(6, pos)};
                        const float cx[2] = {tab_of(4, pos), tab_of(7, pos)};
                        // (the modulation goes in first: 14 products for the 8 weights instead of 24)
                        const float czy[4] = {cz[0] * cy[0], cz[0] * cy[1], cz[1] * cy[0], cz[1] * cy[1]};
                        VecAcc<T> va;
                        va.zero();
#pragma unroll
                        for (int c = 0; c < 8; c++) va.fma(czy[c >> 1] * cx[c & 1], xv[r][c]);
                        // (float: the interpolated values themselves, not the two-term operand form of pack())
                        if constexpr (sizeof(T) == 4) {
                            pend_v = u32x4{__float_as_uint(va.a[0]), __float_as_uint(va.a[1]), __float_as_uint(va.a[2]),
                                           __float_as_uint(va.a[3])};
                        } else {
                            const uint4 cv = va.pack();
                            pend_v = u32x4{cv.x, cv.y, cv.z, cv.w};
                        }
                        pend_p = m0 + pos < a.mpad
                                     ? reinterpret_cast<u32x4 *>(reinterpret_cast<char *>(a.col)
                                           + ((((long)(c0 / BKC) * s.K + k) * a.mpad + m0 + pos) * BKC + ivec * VEC) * (long)sizeof(T))
                                     : nullptr;
                    }
                    float dot[8];
                    if constexpr (sizeof(T) == 2) {
                        const bf16x2_t g0 = __builtin_bit_cast(bf16x2_t, gq[r].x), g1 = __builtin_bit_cast(bf16x2_t, gq[r].y);
                        const bf16x2_t g2 = __builtin_bit_cast(bf16x2_t, gq[r].z), g3 = __builtin_bit_cast(bf16x2_t, gq[r].w);
#pragma unroll
                        for (int c = 0; c < 8; c++) {
                            float d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, xv[r][c].x), g0, 0.f, false);
                            d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, xv[r][c].y), g1, d, false);
                            d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, xv[r][c].z), g2, d, false);
                            dot[c] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, xv[r][c].w), g3, d, false);
                        }
                    } else {
#pragma unroll
                        for (int c = 0; c < 8; c++) {
                            float d = __uint_as_float(gq[r].x) * __uint_as_float(xv[r][c].x);
                            d = fmaf(__uint_as_float(gq[r].y), __uint_as_float(xv[r][c].y), d);
                            d = fmaf(__uint_as_float(gq[r].z), __uint_as_float(xv[r][c].z), d);
                            dot[c] = fmaf(__uint_as_float(gq[r].w), __uint_as_float(xv[r][c].w), d);
                        }
                    }
                    // the four results are linear in the 8 dots: combine per lane, then sum over the 8 lanes
                    const float lz = tab_of(2, pos), ly = tab_of(3, pos), lx = tab_of(4, pos);
                    const float hz = tab_of(5, pos), hy = tab_of(6, pos), hx = tab_of(7, pos);
                    // axis by axis (31 operations instead of ~80 for the eight corners one by one): along x the
                    // differences and the interpolated values of the four (z, y) edges, then along y, then z.
                    // (Corners out of range have dot 0.  The modulation gradient counts live corners only, and a
                    // point has either all of its in-range corners live or none: see make_tap3.)
                    float ex[4], sx[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        ex[e] = dot[2 * e + 1] - dot[2 * e];
                        sx[e] = fmaf(hx, dot[2 * e + 1], lx * dot[2 * e]);
                    }
                    float gxx = fmaf(hz, fmaf(hy, ex[3], ly * ex[2]), lz * fmaf(hy, ex[1], ly * ex[0]));
                    const float sy0 = fmaf(hy, sx[1], ly * sx[0]), sy1 = fmaf(hy, sx[3], ly * sx[2]);
                    float gy = fmaf(hz, sx[3] - sx[2], lz * (sx[1] - sx[0]));
                    float gz = sy1 - sy0;
                    float gm = live ? fmaf(hz, sy1, lz * sy0) : 0.f;
                    gz = sum_over_8_lanes(gz);
                    gy = sum_over_8_lanes(gy);
                    gxx = sum_over_8_lanes(gxx);
                    gm = sum_over_8_lanes(gm);
                    g_acc[r][0] += gz; g_acc[r][1] += gy; g_acc[r][2] += gxx; g_acc[r][3] += gm;
                }
            }
            // ---- results of tap k for the positions of these rounds
            // (every lane takes part in the exchange: a lane that is switched off supplies zeros)
            float al_r[kRounds];
#pragma unroll
            for (int r = 0; r < kRounds; r++) al_r[r] = tab_of(8, (rp * kRounds + r) * 8 + rpos);
            if (ivec == 0) {
#pragma unroll
                for (int r = 0; r < kRounds; r++) {
                    const int pos = (rp * kRounds + r) * 8 + rpos;
                    const int m = m0 + pos;
                    if (m < s.M) {
                        const float al = al_r[r];
                        const int b = m / s.P, p = m - b * s.P;
                        if (SIZED && a.gsize) {
                            // size-map source: d(offset_a) / d(size_a) = base_a[k_a]; the taps of a position add up
                            // (fp32 atomics into [N][3][P], finished by size_grad_finish_kernel)
                            const int kq[3] = {k / (s.geo.kw * s.geo.kh), (k / s.geo.kw) % s.geo.kh, k % s.geo.kw};
#pragma unroll
                            for (int ax = 0; ax < 3; ax++)
                                if (axis_channel(s.ss.mode, ax) >= 0)
                                    atomicAdd(a.gsize + ((long)b * 3 + ax) * s.P + p,
                                              s.ss.base[ax][kq[ax]] * (al * g_acc[r][ax]));
                        } else if (a.goff && s.nd == 3) {
                            const long ob = offset_index(s, b, g, k, p);
                            st_aux(a.goff, ob, s.adt, (s.axes & 1) ? al * g_acc[r][0] : 0.f);
                            st_aux(a.goff, ob + s.P, s.adt, (s.axes & 2) ? al * g_acc[r][1] : 0.f);
                            st_aux(a.goff, ob + 2 * (long)s.P, s.adt, (s.axes & 4) ? al * g_acc[r][2] : 0.f);
                        } else if (a.goff) {
                            st_aux(a.goff, offset_index(s, b, g, k, p), s.adt, al * g_acc[r][2]);
                        }
                        // (with a modulation activation in the sampler: the gradient with respect to the raw value)
                        if (a.gmask)
                            st_aux(a.gmask, mask_index(s, b, g, k, p), s.adt,
                                   s.mact ? g_acc[r][3] * mask_act_grad(s.mact, al) : g_acc[r][3]);
                    }
                }
            }
        }
        if (lbin >= 0) {
            InvEntry e;
            e.p = cp; e.k = k; e.hz = tab[5]; e.hy = tab[6]; e.hx = lhx; e.alpha = tab[8];
            e.pad0 = 0; e.pad1 = 0;
            lists_store(a.lists, lbin, lslot, e);
        }
    }
    if constexpr (COL) {
        if (pend_p) __builtin_nontemporal_store(pend_v, pend_p);
    }
}

}  // namespace

// grad_offset / grad_mask of the whole problem from the grad-column rows.  Needs offset groups whose
// channel count is a multiple of the chunk width.
template <typename T>
int d2c_aux_grad_launch(const TiledShape &s, const void *xcl, const void *off, const void *mask, const void *gcol,
                        void *goff, void *gmask, const SampleLists *lists, void *col, bool col_in_place, hipStream_t st,
                        int g_lo, int g_n)
{
    if (g_n <= 0) { g_lo = 0; g_n = s.G; }
    const int ntile = (s.M + kMT - 1) / kMT;
    const int nshare = s.K < kTapSplit ? s.K : kTapSplit;
    // (with the size-map source `goff` is the fp32 accumulator of the size gradient)
    AuxArgs a{s, xcl, off, mask, gcol, s.ss.on ? nullptr : goff, gmask, s.ss.on ? (float *)goff : nullptr, ntile, nshare,
              lists ? *lists : SampleLists{nullptr, nullptr, nullptr, 0, 0, 0}, col, col_in_place ? (long)s.M : (long)ntile * kMT,
              g_lo, g_n, (unsigned)((size_t)s.N * s.vol * s.Cin * sizeof(T))};
    dim3 grid((unsigned)(8 * (((ntile + kWavesPerBlock - 1) / kWavesPerBlock + 7) / 8) * g_n * nshare));
    bool aux16 = false;
    if constexpr (sizeof(T) == 2) aux16 = s.adt == D2C_BF16;
    D2cProfScope prof(D2C_PROF_BWD_AUX, st, "aux_grad_kernel");
    const dim3 blk(64 * kWavesPerBlock);
    if (col && s.nd != 3) {
        d2c_set_error("aux_grad_kernel: sampled columns are written for problems in three dimensions only");
        return D2C_ERR_LAUNCH;
    }
    // (the sampled columns: problems in three dimensions, see d2c_bwd_weight_from_col)
    auto go = [&](auto aux_c, auto sized_c) {
        constexpr bool A16 = decltype(aux_c)::value, SZ = decltype(sized_c)::value;
        if (col) hipLaunchKernelGGL((aux_grad_kernel<T, A16, SZ, true>), grid, blk, 0, st, a);
        else hipLaunchKernelGGL((aux_grad_kernel<T, A16, SZ, false>), grid, blk, 0, st, a);
    };
    if constexpr (sizeof(T) == 2) {
        if (aux16) {
            if (s.ss.on) go(std::true_type{}, std::true_type{});
            else go(std::true_type{}, std::false_type{});
        }
    }
    if (!aux16) {
        if (s.ss.on) go(std::false_type{}, std::true_type{});
        else go(std::false_type{}, std::false_type{});
    }
    return d2c_check_launch("aux_grad_kernel");
}
template int d2c_aux_grad_launch<bf16_t>(const TiledShape &, const void *, const void *, const void *, const void *,
                                         void *, void *, const SampleLists *, void *, bool, hipStream_t, int, int);
template int d2c_aux_grad_launch<float>(const TiledShape &, const void *, const void *, const void *, const void *,
                                        void *, void *, const SampleLists *, void *, bool, hipStream_t, int, int);
