// Backward pass on the matrix cores.
//
// Kernel 1, per workgroup a tile of output positions, per step one (tap, channel chunk):
//     gcol[pos, c]  = sum_o gout[pos, o] * W[o, c, k]                (MFMA; dconv3d_gpu.cu:976-1000)
//   The gout operand of a wavefront (its 32 positions x all output channels of the weight group) stays in registers
//   for the whole kernel; the weight operand of the step is staged in LDS.
//   tiled_bwd_col32_kernel / tiled_bwd_col_kernel (the usual path) write the grad-column rows to a buffer [chunk][tap][position][BKC] in
//   device memory, which two kernels of their own read back: the offset / mask gradient (d2c_aux_grad.hip) and
//   grad_input from per-voxel sample lists (d2c_invlist.hip).  This round trip through memory (N*P*K*Cin elements
//   written once, read twice) is the price of running those two without the barriers and the register budget of
//   the matrix kernel.
//   tiled_bwd_data_kernel (shapes the other path does not take: several passes over the output channels, no sample
//   lists) consumes the rows where they are made:
//     gx[corner, c] += a_corner * alpha * gcol[pos, c]               (atomics; :593-642)
//     dot[corner]    = sum_c gcol[pos, c] * x[corner, c]
//     gmask          = sum_corner a_corner * dot[corner]             (:837-839)
//     goff_axis      = alpha * sum_corner (d a_corner / d axis) * dot[corner]   (:708-754, :848-858)
//
// Kernel 2b (tiled_bwd_weight_col_kernel; bfloat16 problems whose offset / mask gradient kernel runs): grad_weight as
// a plain matrix product over the sampled columns which that kernel writes on its way -- the backward pass samples
// the input once.
//
// Kernel 2 (tiled_bwd_weight_dma_kernel; everything else), per workgroup one (tap, channel chunk)
// and all output channels, looping over position tiles:
//     gW[o, c, k] += sum_pos gout[o, pos] * alpha * trilinear(x[c], pos)       (:1037-1088)
//   The reduction runs over positions, so the MFMA operand wants 8 consecutive
//   positions of one channel per lane: the bfloat16 tile is stored as sampled
//   ([position][channel]) and read with the transposing LDS load
//   (ds_read_b64_tr_b16); the float tile is stored transposed.
#include <algorithm>
#include <functional>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>
#include "d2c_mma.hpp"
#include "d2c_tiled.hpp"

namespace {

constexpr int kThreads = 512;

D2C_DEV int xcd_swizzle(int bid, int n)
{
    const int x = bid & 7, idx = bid >> 3;
    const int q = n >> 3, r = n & 7;
    return x * q + (x < r ? x : r) + idx;
}

// ============================================================ kernel 1
struct BwdDataArgs {
    TiledShape s;
    const void *gout;   // [N][Cout][P]
    const void *xcl;    // [N][vol][Cin]
    const void *off, *mask;
    const void *wt;     // [groups][step][BKC][ogk]   (W transposed per step, zero padded to ogk)
    float *gxcl;        // [N][vol][Cin] fp32 accumulator (zeroed) for the atomic scatter, or NULL
    void *gcolbuf;      // [chunk][tap][N*P][BKC] grad-column values for the list-based grad_input, or NULL
    void *goff, *gmask; // or NULL
    int ogk;            // output channels of this pass rounded up to a whole k-group
    int o0, ogn;        // this pass reduces over output channels [o0, o0 + ogn) of each weight group
    int add_aux;        // later passes add to the offset / mask gradient of earlier ones
    // Few position tiles (small N*P): the steps are dealt to gridDim.z workgroups per tile, and the offset / mask
    // gradient (a sum over the channel chunks of a group) is accumulated with atomics in fp32 scratch arrays
    // laid out like goff / gmask, which a finishing kernel converts.
    float *auxoff, *auxmask;
    // tiled_bwd_col32_kernel: the half-steps [h_lo, h_hi) of the step sequence this launch makes (a slice of the offset
    // groups; h_hi == 0: all of them).  `gcolbuf` then points where chunk 0 WOULD start if the buffer held all chunks.
    int h_lo, h_hi;
};

// NKG = k-groups of the reduction over output channels held in registers.
// SPLIT (float problems): operands as two bfloat16 halves on the bfloat16 matrix instruction (see kF32SplitFwd in
// d2c_mma.hpp), where the caller has asked for it (TiledShape::f32split).
template <typename T, int NKG, bool SPLIT>
__global__ void __launch_bounds__(kThreads) tiled_bwd_data_kernel(BwdDataArgs a)
{
    constexpr int VEC = Elem<T>::VEC;
    constexpr int NV = 8, BKC = NV * VEC;
    constexpr int CB = BKC / 32;           // 32-channel blocks per step (2 for bf16, 1 for float)
    constexpr int PBW = 8 / CB;            // 32-position blocks per workgroup
    constexpr int MT = 32 * PBW;           // positions per workgroup (128 / 256)
    constexpr int GRS = BKC * 4 + 16;      // gcol tile row stride (bytes)
    constexpr int ITEMS = MT * NV / kThreads;

    extern __shared__ __align__(16) unsigned char smem[];
    const TiledShape &s = a.s;
    // Weight tile [BKC][ogk], rows unpadded (a multiple of 128 bytes); the 16-byte pieces of row r are stored
    // at position (piece ^ (r & 7)), which keeps the operand reads of 32 consecutive rows free of bank conflicts.
    const int rowB = a.ogk * (int)sizeof(T);
    unsigned char *s_wt = smem;                          // [BKC][rowB]
    unsigned char *s_gcol = s_wt + BKC * rowB;           // [MT][GRS]
    float *s_w = reinterpret_cast<float *>(s_gcol + MT * GRS);   // [8][MT]  live corner weights * alpha
    float *s_frac = s_w + 8 * MT;                        // [6][MT]  lz ly lx hz hy hx
    float *s_alpha = s_frac + 6 * MT;                    // [MT]
    int *s_idx = reinterpret_cast<int *>(s_alpha + MT);  // [MT]
    int *s_flag = s_idx + MT;                            // [MT]     live | inrange << 8 | 1-D low-corner shift << 16 | mask-gradient corners << 24

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tile = xcd_swizzle(blockIdx.x, gridDim.x);
    const int wg = blockIdx.y;
    const int m0 = tile * MT;
    const int S = s.nchunk * s.K;
    const int dzc = s.H * s.W * s.Cin, dyc = s.W * s.Cin;   // element strides of a step in z / y
    const int cb = wave % CB, pb = wave / CB;
    const int nkg = a.ogk / (2 * VEC);

    // ---- stationary operand: gout[pos, o] of this wavefront's 32 positions
    uint4 ga[NKG];
    {
        const int m = m0 + pb * 32 + (lane & 31);
        const bool ok = m < s.M;
        const int b = ok ? m / s.P : 0, p = ok ? m - b * s.P : 0;
        const T *gp = reinterpret_cast<const T *>(a.gout) + ((long)b * s.Cout + wg * s.og + a.o0) * s.P + p;
#pragma unroll
        for (int kg = 0; kg < NKG; kg++) {
            T e[VEC];
#pragma unroll
            for (int i = 0; i < VEC; i++) {
                const int o = (kg * 2 + (lane >> 5)) * VEC + i;
                e[i] = (ok && kg < nkg && o < a.ogn) ? gp[(long)o * s.P] : (T)0;
            }
            ga[kg] = operand_vec<T, SPLIT>(e);
        }
    }

    // ---- per-position constants of the coordinate threads
    int cbatch = 0, cp = 0, coz = 0, coy = 0, cox = 0;
    bool cvalid = false;
    if (tid < MT) {
        const int m = m0 + tid;
        cvalid = m < s.M;
        if (cvalid) {
            cbatch = m / s.P; cp = m - cbatch * s.P;
            cox = cp % s.Wo; coy = (cp / s.Wo) % s.Ho; coz = cp / (s.Wo * s.Ho);
        }
    }

    // offset / mask gradient accumulators of the positions this thread finalises
    float g_acc[ITEMS][4];
#pragma unroll
    for (int i = 0; i < ITEMS; i++) g_acc[i][0] = g_acc[i][1] = g_acc[i][2] = g_acc[i][3] = 0.f;

    const bool want_aux = a.goff != nullptr || a.gmask != nullptr;

    const int st_lo = (int)((long)S * blockIdx.z / gridDim.z), st_hi = (int)((long)S * (blockIdx.z + 1) / gridDim.z);
    for (int st = st_lo; st < st_hi; st++) {
        // step order: offset group (outer), tap, chunk of the group (inner).  The chunks of a group share
        // the sampling positions of a tap, so its offset / mask gradient accumulates in registers over the
        // inner loop; and a group's channel slice of the input stays in L2 across its taps.
        const int cpc = s.cpg / BKC;                 // chunks per offset group
        const int jj = st % cpc, k = (st / cpc) % s.K, gi = st / (cpc * s.K);
        const int j = gi * cpc + jj;                  // chunk inside the weight group
        const int c0 = wg * s.cg + j * BKC;
        const int g = c0 / s.cpg;
        // last chunk of the group for this tap (or of this workgroup's share) -> flush goff / gmask
        const bool group_end = jj + 1 == cpc || st + 1 == st_hi;

        // (a) weight tile of the step (asynchronous), then its coordinates
        {
            // global -> LDS without passing through registers: one instruction of a wavefront moves 64
            // pieces to 1 KiB of consecutive LDS (lane i's piece lands at base + 16 i), so lane i fetches the
            // piece that the swizzled layout wants there
            const int rp = rowB / 16;                        // 16-byte pieces per weight row (a multiple of 8)
            const uint4 *src = reinterpret_cast<const uint4 *>(a.wt) + ((long)wg * S + st) * BKC * rp;
            const int ninstr = BKC * rp / 64;
            for (int i = wave; i < ninstr; i += kThreads / 64) {
                const int pos = i * 64 + lane;
                const int row = pos / rp, q = pos - row * rp;
                const uint4 *g = src + row * rp + (q ^ (row & 7));
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)g,
                                                 (__attribute__((address_space(3))) void *)(s_wt + i * 1024), 16, 0, 0);
            }
        }
        // (nobody reads the corner table when grad_input comes from the sample lists and the offset / mask
        // gradient from the kernel of d2c_aux_grad.hip)
        if (tid < MT && (a.gxcl != nullptr || want_aux)) {
            float w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            float fr[6] = {0, 0, 0, 0, 0, 0};
            float al = 0.f;
            int idx = 0, flag = 0;
            if (cvalid) {
                float o0, o1, o2;
                load_offsets(s, a.off, cbatch, g, k, cp, o0, o1, o2);
                al = a.mask ? mask_act_rt(s.mact, ld_aux(a.mask, mask_index(s, cbatch, g, k, cp), s.adt), s.adt) : 1.f;
                int bz, by, bx;
                tap_base(s.geo, k, coz, coy, cox, bz, by, bx);
                const Tap3<float> t = tiled_tap3(s, bz, by, bx, o0, o1, o2);
                idx = (cbatch * s.vol + (t.z0 * s.H + t.y0) * s.W + t.x0) * s.Cin;   // element offset of corner 000
                unsigned inr = t.inrange, auxlive = t.live;
                fr[0] = t.lz; fr[1] = t.ly; fr[2] = t.lx; fr[3] = t.hz; fr[4] = t.hy; fr[5] = t.hx;
                if (s.nd == 1) {
                    // 1-D: both corners are gated by range only (dconv1d_gpu.cu:338-339), and at
                    // integer positions the low corner steps down by one while the high corner stays
                    // (:332-336); grad_offset / grad_mask then interpolate with t' = x - (x0 - 1).
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
                flag |= (int)(t.live | (inr << 8) | (auxlive << 24));
#pragma unroll
                for (int c = 0; c < 8; c++) w[c] = ((t.live >> c) & 1u) ? tap3_weight(t, c) * al : 0.f;
            }
#pragma unroll
            for (int c = 0; c < 8; c++) s_w[c * MT + tid] = w[c];
#pragma unroll
            for (int c = 0; c < 6; c++) s_frac[c * MT + tid] = fr[c];
            s_alpha[tid] = al;
            s_idx[tid] = idx;
            s_flag[tid] = flag;
        }
        __builtin_amdgcn_s_waitcnt(0);   // the weight-tile transfers of this wavefront have landed
        __syncthreads();

        // (b) gcol block of this wavefront: rows = positions, columns = channels
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.f;
        {
            const int wrow = cb * 32 + (lane & 31);
            const unsigned char *wb = s_wt + wrow * rowB;
            const int wsw = wrow & 7, wh = lane >> 5;
            if (NKG >= 8 && nkg == NKG && (rowB / 16) % 16 == 0) {
                // The usual case, free of branches.  Fragment kg lies at piece (2 kg + wh) ^ wsw of the row: the pieces
                // of 8 consecutive k-groups share a block of 16 and differ from the next 8 by a constant, so 8 lane
                // addresses + immediate offsets address all of them (32 addresses would not fit the registers
                // next to the stationary operand).
                const unsigned char *wa[8];
#pragma unroll
                for (int i = 0; i < 8; i++) wa[i] = wb + (((i * 2 + wh) ^ wsw) << 4);
#pragma unroll
                for (int kg = 0; kg < NKG; kg++) {
                    const uint4 bf = *reinterpret_cast<const uint4 *>(wa[kg & 7] + (kg >> 3) * 256);
                    mma_kgroup<T, SPLIT>(acc, ga[kg], bf);
                }
            } else {
#pragma unroll
                for (int kg = 0; kg < NKG; kg++) {
                    if (kg < nkg) {
                        const uint4 bf = *reinterpret_cast<const uint4 *>(wb + (((kg * 2 + wh) ^ wsw) << 4));
                        mma_kgroup<T, SPLIT>(acc, ga[kg], bf);
                    }
                }
            }
        }

        // (c) gcol -> LDS (for the dot products), and scatter into grad_input straight from
        //     the accumulators: lanes 0..31 / 32..63 each cover 32 consecutive channels.
        const int ch = cb * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int pl = pb * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            *reinterpret_cast<float *>(s_gcol + pl * GRS + ch * 4) = acc[r];
        }
        if (a.gxcl) {
            float *gbase = a.gxcl + c0 + ch;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int pl = pb * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                const unsigned live = (unsigned)s_flag[pl] & 0xffu;
                if (live) {
                    const int idx = s_idx[pl];
                    const float gv = acc[r];
#pragma unroll
                    for (int c = 0; c < 8; c++) {
                        if ((live >> c) & 1u) {
                            const unsigned o = (unsigned)(idx + ((c >> 2) & 1) * dzc + ((c >> 1) & 1) * dyc + (c & 1) * s.Cin);
                            atomicAdd(gbase + o, s_w[c * MT + pl] * gv);
                        }
                    }
                }
            }
        }
        __syncthreads();

        // (d) grad-column rows out to memory (list-based grad_input)
        if (a.gcolbuf) {
            T *gb = reinterpret_cast<T *>(a.gcolbuf) + ((long)(c0 / BKC) * s.K + k) * s.M * BKC;
#pragma unroll
            for (int i = 0; i < ITEMS; i++) {
                const int item = tid + i * kThreads;
                const int pos = item / NV, vec = item % NV;
                const int m = m0 + pos;
                if (m < s.M) {
                    const float *gp = reinterpret_cast<const float *>(s_gcol + pos * GRS + vec * VEC * 4);
                    uint4 o;
                    if constexpr (sizeof(T) == 2) {
                        o = make_uint4(pack_bf16x2(gp[0], gp[1]), pack_bf16x2(gp[2], gp[3]), pack_bf16x2(gp[4], gp[5]),
                                       pack_bf16x2(gp[6], gp[7]));
                    } else {
                        o = *reinterpret_cast<const uint4 *>(gp);
                    }
                    *reinterpret_cast<uint4 *>(gb + (long)m * BKC + vec * VEC) = o;
                }
            }
        }
        // (e) dot products with the corner vectors, offset / mask gradient
        if (want_aux) {
#pragma unroll
            for (int i = 0; i < ITEMS; i++) {
                const int item = tid + i * kThreads;
                const int pos = item / NV, vec = item % NV;
                const int idx = s_idx[pos];
                const unsigned flag = (unsigned)s_flag[pos];
                const unsigned inr = (flag >> 8) & 0xffu, live = flag >> 24;
                const int qshift = (flag >> 16) & 1;
                float gc[VEC];
                {
                    const float4 *gp4 = reinterpret_cast<const float4 *>(s_gcol + pos * GRS + vec * VEC * 4);
#pragma unroll
                    for (int e = 0; e < VEC / 4; e++) {
                        const float4 t4 = gp4[e];
                        gc[4 * e] = t4.x; gc[4 * e + 1] = t4.y; gc[4 * e + 2] = t4.z; gc[4 * e + 3] = t4.w;
                    }
                }
                const char *xb = reinterpret_cast<const char *>(a.xcl);
                const int ib = idx + c0 + vec * VEC;
                float dot[8];
                uint4 xv[8];
                // all eight (predicated) loads are issued before any of them is used; 32-bit byte offsets
#pragma unroll
                for (int c = 0; c < 8; c++) {
                    const unsigned o = (unsigned)(ib + ((c >> 2) & 1) * dzc + ((c >> 1) & 1) * dyc
                                                  + ((c & 1) ? s.Cin : -qshift * s.Cin)) * (unsigned)sizeof(T);
                    xv[c] = ((inr >> c) & 1u) ? *reinterpret_cast<const uint4 *>(xb + o) : make_uint4(0, 0, 0, 0);
                }
                if constexpr (sizeof(T) == 2) {
                    // the grad-column values in the precision they are stored with (bfloat16 pairs), two
                    // products per instruction, fp32 accumulation
                    bf16x2_t gp[4];
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        gp[e] = __builtin_bit_cast(bf16x2_t, pack_bf16x2(gc[2 * e], gc[2 * e + 1]));
#pragma unroll
                    for (int c = 0; c < 8; c++) {
                        float d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, xv[c].x), gp[0], 0.f, false);
                        d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, xv[c].y), gp[1], d, false);
                        d = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, xv[c].z), gp[2], d, false);
                        dot[c] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, xv[c].w), gp[3], d, false);
                    }
                } else {
#pragma unroll
                    for (int c = 0; c < 8; c++) {
                        const T *xe = reinterpret_cast<const T *>(&xv[c]);
                        float d = 0.f;
#pragma unroll
                        for (int e = 0; e < VEC; e++) d = fmaf(gc[e], elem_to_f32<T>(xe[e]), d);
                        dot[c] = d;
                    }
                }
                // sum over the 8 lanes that share the position
#pragma unroll
                for (int c = 0; c < 8; c++) {
                    dot[c] += __shfl_xor(dot[c], 1, 64);
                    dot[c] += __shfl_xor(dot[c], 2, 64);
                    dot[c] += __shfl_xor(dot[c], 4, 64);
                }
                if (vec == 0) {
                    const float lz = s_frac[0 * MT + pos], ly = s_frac[1 * MT + pos], lx = s_frac[2 * MT + pos];
                    const float hz = s_frac[3 * MT + pos], hy = s_frac[4 * MT + pos], hx = s_frac[5 * MT + pos];
                    float gz = 0.f, gy = 0.f, gxx = 0.f, gm = 0.f;
#pragma unroll
                    for (int c = 0; c < 8; c++) {
                        const float wz = (c & 4) ? hz : lz, wy = (c & 2) ? hy : ly, wx = (c & 1) ? hx : lx;
                        const float d = dot[c];
                        gz += ((c & 4) ? d : -d) * (wy * wx);
                        gy += ((c & 2) ? d : -d) * (wz * wx);
                        gxx += ((c & 1) ? d : -d) * (wz * wy);
                        if ((live >> c) & 1u) gm += (wz * wy * wx) * d;
                    }
                    const float al = s_alpha[pos];
                    g_acc[i][0] += al * gz; g_acc[i][1] += al * gy; g_acc[i][2] += al * gxx; g_acc[i][3] += gm;
                    if (group_end) {
                        const int m = m0 + pos;
                        if (m < s.M) {
                            const int b = m / s.P, p = m - b * s.P;
                            const long ab = (((long)b * s.G + g) * s.K + k) * s.P + p;
                            if (a.auxoff) {
                                if (a.goff && s.nd == 3) {
                                    const long ob = 3 * ab - 2 * (long)p;
#pragma unroll
                                    for (int ax = 0; ax < 3; ax++)
                                        if ((s.axes >> ax) & 1) atomicAdd(a.auxoff + ob + ax * (long)s.P, g_acc[i][ax]);
                                } else if (a.goff) {
                                    atomicAdd(a.auxoff + ab, g_acc[i][2]);
                                }
                                if (a.gmask) atomicAdd(a.auxmask + ab, g_acc[i][3]);
                            } else if (a.goff && s.nd == 3) {
                                const long ob = 3 * ab - 2 * (long)p;   // ((b*G+g)*K+k)*3*P + p
#pragma unroll
                                for (int ax = 0; ax < 3; ax++) {
                                    const long oi = ob + ax * (long)s.P;
                                    st_aux(a.goff, oi, s.adt, ((s.axes >> ax) & 1)
                                               ? g_acc[i][ax] + (a.add_aux ? ld_aux(a.goff, oi, s.adt) : 0.f) : 0.f);
                                }
                            } else if (a.goff) {
                                st_aux(a.goff, ab, s.adt, g_acc[i][2] + (a.add_aux ? ld_aux(a.goff, ab, s.adt) : 0.f));
                            }
                            if (a.gmask && !a.auxoff)
                                st_aux(a.gmask, ab, s.adt, g_acc[i][3] + (a.add_aux ? ld_aux(a.gmask, ab, s.adt) : 0.f));
                        }
                        g_acc[i][0] = g_acc[i][1] = g_acc[i][2] = g_acc[i][3] = 0.f;
                    }
                }
            }
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------
// The grad-column product alone (grad_input comes from the sample lists, the offset / mask gradient from the
// kernel of d2c_aux_grad.hip: the usual case).  tiled_bwd_col_kernel: same tiling and operands as
// tiled_bwd_data_kernel, without its other duties, and with the fragment reads running ahead of the matrix
// instructions.  Where two weight tiles and the float grad-column block fit LDS (DB) the weight tile is
// double-buffered: the DMA transfer of step s+1 is in flight while step s is on the matrix cores.  Two barriers
// per step, both waiting for LDS operations only.  It serves float problems and the bfloat16 reductions that are
// no multiple of 128 channels; the others take tiled_bwd_col32_kernel further down.
D2C_DEV void lds_only_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// at most `n` vector-memory operations of this wavefront still in flight (the counter has six bits: its low four in
// bits 3:0 of the operand, the other two in bits 15:14; counts above 31 wait as for 31)
D2C_DEV void wait_vm_at_most(int n)
{
#define D2C_WAIT_VM_CASE(k) case k: __builtin_amdgcn_s_waitcnt(0x0F70 | ((k) & 15) | (((k) >> 4) << 14)); break;
    switch (n < 0 ? 0 : (n > 31 ? 31 : n)) {
        D2C_WAIT_VM_CASE(0) D2C_WAIT_VM_CASE(1) D2C_WAIT_VM_CASE(2) D2C_WAIT_VM_CASE(3)
        D2C_WAIT_VM_CASE(4) D2C_WAIT_VM_CASE(5) D2C_WAIT_VM_CASE(6) D2C_WAIT_VM_CASE(7)
        D2C_WAIT_VM_CASE(8) D2C_WAIT_VM_CASE(9) D2C_WAIT_VM_CASE(10) D2C_WAIT_VM_CASE(11)
        D2C_WAIT_VM_CASE(12) D2C_WAIT_VM_CASE(13) D2C_WAIT_VM_CASE(14) D2C_WAIT_VM_CASE(15)
        D2C_WAIT_VM_CASE(16) D2C_WAIT_VM_CASE(17) D2C_WAIT_VM_CASE(18) D2C_WAIT_VM_CASE(19)
        D2C_WAIT_VM_CASE(20) D2C_WAIT_VM_CASE(21) D2C_WAIT_VM_CASE(22) D2C_WAIT_VM_CASE(23)
        D2C_WAIT_VM_CASE(24) D2C_WAIT_VM_CASE(25) D2C_WAIT_VM_CASE(26) D2C_WAIT_VM_CASE(27)
        D2C_WAIT_VM_CASE(28) D2C_WAIT_VM_CASE(29) D2C_WAIT_VM_CASE(30) D2C_WAIT_VM_CASE(31)
    }
#undef D2C_WAIT_VM_CASE
}

// (XOR over 8 piece positions.  Spreading the pieces over 16 positions, the 64 banks of this LDS, took the
// bank-conflict cycles of the fragment reads from 50 M to 6 M per launch at C3 and made the kernel 5 % slower.)
D2C_DEV int swizzle_of_row(int row) { return row & 7; }

// Eight k-groups of the matrix step for bfloat16, scheduled by hand: the compiler, short of registers next to a
// 128-register stationary operand, emits read - wait - multiply for every fragment, and it makes LDS reads that it
// sees wait for every DMA transfer in flight into the same array; here the LDS reads run three
// fragments ahead of the matrix instructions (four rotating fragment registers; a register is reloaded after the
// matrix instruction that follows the one which read it).  `w0..w7` are the lane's LDS addresses of the 8 fragments,
// OFF the byte offset of this block of 8.  The fragments from LDS are the first operand, the stationary `g` the
// second: the product comes out transposed (lane = column of `g`, i.e. position).
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
template <int OFF>
D2C_DEV void mma8_bf16_t(f32x16 &acc, const uint4 *g, const unsigned *w)
{
    u32x4 b0, b1, b2, b3;
    const u32x4 g0 = __builtin_bit_cast(u32x4, g[0]), g1 = __builtin_bit_cast(u32x4, g[1]),
                g2 = __builtin_bit_cast(u32x4, g[2]), g3 = __builtin_bit_cast(u32x4, g[3]),
                g4 = __builtin_bit_cast(u32x4, g[4]), g5 = __builtin_bit_cast(u32x4, g[5]),
                g6 = __builtin_bit_cast(u32x4, g[6]), g7 = __builtin_bit_cast(u32x4, g[7]);
    asm volatile(
        "ds_read_b128 %[b0], %[w0] offset:%[off]\n\t"
        "ds_read_b128 %[b1], %[w1] offset:%[off]\n\t"
        "ds_read_b128 %[b2], %[w2] offset:%[off]\n\t"
        "ds_read_b128 %[b3], %[w3] offset:%[off]\n\t"
        "s_waitcnt lgkmcnt(3)\n\t"
        "v_mfma_f32_32x32x16_bf16 %[acc], %[b0], %[g0], %[acc]\n\t"
        "s_waitcnt lgkmcnt(2)\n\t"
        "v_mfma_f32_32x32x16_bf16 %[acc], %[b1], %[g1], %[acc]\n\t"
        "ds_read_b128 %[b0], %[w4] offset:%[off]\n\t"
        "s_waitcnt lgkmcnt(2)\n\t"
        "v_mfma_f32_32x32x16_bf16 %[acc], %[b2], %[g2], %[acc]\n\t"
        "ds_read_b128 %[b1], %[w5] offset:%[off]\n\t"
        "s_waitcnt lgkmcnt(2)\n\t"
        "v_mfma_f32_32x32x16_bf16 %[acc], %[b3], %[g3], %[acc]\n\t"
        "ds_read_b128 %[b2], %[w6] offset:%[off]\n\t"
        "s_waitcnt lgkmcnt(2)\n\t"
        "v_mfma_f32_32x32x16_bf16 %[acc], %[b0], %[g4], %[acc]\n\t"
        "ds_read_b128 %[b3], %[w7] offset:%[off]\n\t"
        "s_waitcnt lgkmcnt(2)\n\t"
        "v_mfma_f32_32x32x16_bf16 %[acc], %[b1], %[g5], %[acc]\n\t"
        "s_waitcnt lgkmcnt(1)\n\t"
        "v_mfma_f32_32x32x16_bf16 %[acc], %[b2], %[g6], %[acc]\n\t"
        "s_waitcnt lgkmcnt(0)\n\t"
        "v_mfma_f32_32x32x16_bf16 %[acc], %[b3], %[g7], %[acc]\n\t"
        : [acc] "+v"(acc), [b0] "=&v"(b0), [b1] "=&v"(b1), [b2] "=&v"(b2), [b3] "=&v"(b3)
        : [g0] "v"(g0), [g1] "v"(g1), [g2] "v"(g2), [g3] "v"(g3), [g4] "v"(g4), [g5] "v"(g5), [g6] "v"(g6), [g7] "v"(g7),
          [w0] "v"(w[0]), [w1] "v"(w[1]), [w2] "v"(w[2]), [w3] "v"(w[3]), [w4] "v"(w[4]), [w5] "v"(w[5]), [w6] "v"(w[6]),
          [w7] "v"(w[7]), [off] "n"(OFF)
        : "memory");
}

// Row stride (bytes) of the float grad-column block in LDS.  bfloat16 problems: unpadded, 128 rows of 256 bytes =
// 32 KiB, which leaves room for two 64 KiB weight tiles (512 reduced channels) in the 160 KiB of a workgroup.
template <typename T> constexpr int col_row_stride() { return 8 * Elem<T>::VEC * 4 + (sizeof(T) == 2 ? 0 : 16); }

template <typename T, int NKG, bool DB, bool SPLIT>
__global__ void __launch_bounds__(kThreads) tiled_bwd_col_kernel(BwdDataArgs a)
{
    constexpr int VEC = Elem<T>::VEC;
    constexpr int NV = 8, BKC = NV * VEC;
    constexpr int CB = BKC / 32;           // 32-channel blocks per step (2 for bf16, 1 for float)
    constexpr int PBW = 8 / CB;            // 32-position blocks per workgroup
    constexpr int MT = 32 * PBW;           // positions per workgroup (128 / 256)
    constexpr int GRS = col_row_stride<T>();   // gcol tile row stride (bytes), float
    constexpr int NW = kThreads / 64;
    constexpr int ITEMS = MT * NV / kThreads;

    extern __shared__ __align__(16) unsigned char smem[];
    const TiledShape &s = a.s;
    const int rowB = a.ogk * (int)sizeof(T);
    const int tileB = BKC * rowB;
    unsigned char *s_wt = smem;                          // [DB ? 2 : 1][BKC][rowB]
    unsigned char *s_gcol = s_wt + (DB ? 2 : 1) * tileB; // [MT][GRS]

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tile = xcd_swizzle(blockIdx.x, gridDim.x);
    const int wg = blockIdx.y;
    const int m0 = tile * MT;
    const int S = s.nchunk * s.K;
    const int cb = wave % CB, pb = wave / CB;
    const int nkg = a.ogk / (2 * VEC);
    const int rp = rowB / 16;                            // 16-byte pieces per weight row (a multiple of 8)
    const int ninstr = BKC * rp / 64;                    // DMA instructions per tile, dealt to the wavefronts
    const int mine = ninstr > wave ? (ninstr - wave + NW - 1) / NW : 0;   // (at most 8: rows of 1 KiB)

    // ---- stationary operand: gout[pos, o] of this wavefront's 32 positions
    uint4 ga[NKG];
    {
        const int m = m0 + pb * 32 + (lane & 31);
        const bool ok = m < s.M;
        const int b = ok ? m / s.P : 0, p = ok ? m - b * s.P : 0;
        const T *gp = reinterpret_cast<const T *>(a.gout) + ((long)b * s.Cout + wg * s.og + a.o0) * s.P + p;
#pragma unroll
        for (int kg = 0; kg < NKG; kg++) {
            T e[VEC];
#pragma unroll
            for (int i = 0; i < VEC; i++) {
                const int o = (kg * 2 + (lane >> 5)) * VEC + i;
                e[i] = (ok && kg < nkg && o < a.ogn) ? gp[(long)o * s.P] : (T)0;
            }
            ga[kg] = operand_vec<T, SPLIT>(e);
        }
    }

    // weight tile of step st: global -> LDS without passing through registers; one instruction of a wavefront
    // moves 64 pieces to 1 KiB of consecutive LDS (lane i's piece lands at base + 16 i), so lane i fetches the
    // piece that the swizzled layout wants there
    auto dma_tile = [&](int st, int buf) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.wt) + ((long)wg * S + st) * BKC * rp;
        for (int i = wave; i < ninstr; i += NW) {
            const int pos = i * 64 + lane;
            const int row = pos / rp, q = pos - row * rp;
            const uint4 *g = src + row * rp + (q ^ swizzle_of_row(row));
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)g,
                                             (__attribute__((address_space(3))) void *)(s_wt + buf * tileB + i * 1024), 16,
                                             0, 0);
        }
    };

    // byte offsets (inside a tile) of this lane's fragments of the first 8 k-groups
    int woff[8];
    {
        const int wrow = cb * 32 + (lane & 31);
        const int wsw = swizzle_of_row(wrow), wh = lane >> 5;
#pragma unroll
        for (int i = 0; i < 8; i++) woff[i] = wrow * rowB + (((i * 2 + wh) ^ wsw) << 4);
    }

    const int st_lo = (int)((long)S * blockIdx.z / gridDim.z), st_hi = (int)((long)S * (blockIdx.z + 1) / gridDim.z);
    if (DB && st_lo < st_hi) dma_tile(st_lo, 0);
    for (int st = st_lo, it = 0; st < st_hi; st++, it++) {
        // step order: offset group (outer), tap, chunk of the group (inner), as in tiled_bwd_data_kernel
        const int cpc = s.cpg / BKC;
        const int jj = st % cpc, k = (st / cpc) % s.K, gi = st / (cpc * s.K);
        const int j = gi * cpc + jj;
        const int c0 = wg * s.cg + j * BKC;
        const bool more = st + 1 < st_hi;
        if constexpr (DB) {
            if (more) dma_tile(st + 1, (it + 1) & 1);
            // this wavefront's pieces of tile st have landed when only its requests for tile st+1 are still in
            // flight (requests complete in order; the grad-column stores of the previous step are older)
            wait_vm_at_most(more ? mine : 0);
        } else {
            // one tile buffer: every wavefront is past the matrix step of st-1 (the barrier behind it).  (Requesting
            // the tile earlier, behind that barrier, so that it comes in while the rows go out, was 3 % slower.)
            dma_tile(st, 0);
            wait_vm_at_most(0);
        }
        lds_only_barrier();

        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.f;
        {
            const unsigned char *wb = s_wt + (DB ? (it & 1) : 0) * tileB;
            if (NKG >= 8 && nkg == NKG && rp % 16 == 0) {
                // The usual case, free of branches.  Fragment kg of this lane lies at piece (2 kg + wh) ^ wsw of its
                // row: the pieces of 8 consecutive k-groups share a block of 16 and differ from the next 8 by a
                // constant, so 8 lane addresses + immediate offsets address all of them; the reads run kPF
                // fragments ahead of the matrix instructions that take them.
                constexpr int kPF = 3;
                uint4 bq[kPF + 1];
#pragma unroll
                for (int i = 0; i < kPF; i++)
                    bq[i] = *reinterpret_cast<const uint4 *>(wb + woff[i & 7] + (i >> 3) * 256);
#pragma unroll
                for (int kg = 0; kg < NKG; kg++) {
                    if (kg + kPF < NKG)
                        bq[(kg + kPF) % (kPF + 1)] =
                            *reinterpret_cast<const uint4 *>(wb + woff[(kg + kPF) & 7] + ((kg + kPF) >> 3) * 256);
                    mma_kgroup<T, SPLIT>(acc, ga[kg], bq[kg % (kPF + 1)]);
                }
            } else {
                const int wrow = cb * 32 + (lane & 31);
                const unsigned char *wr = wb + wrow * rowB;
                const int wsw = swizzle_of_row(wrow), wh = lane >> 5;
#pragma unroll
                for (int kg = 0; kg < NKG; kg++) {
                    if (kg < nkg) {
                        const uint4 bf = *reinterpret_cast<const uint4 *>(wr + (((kg * 2 + wh) ^ wsw) << 4));
                        mma_kgroup<T, SPLIT>(acc, ga[kg], bf);
                    }
                }
            }
        }
        // grad-column block -> LDS: lanes 0..31 / 32..63 each cover 32 consecutive channels
        const int ch = cb * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int pl = pb * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            *reinterpret_cast<float *>(s_gcol + pl * GRS + ch * 4) = acc[r];
        }
        lds_only_barrier();
        // rows out to memory, 16 bytes per thread.  A later pass over the output channels of a wide weight group
        // (a.add_aux) adds to the rows the passes before it left: the sum formed in float, bfloat16 rounded once more
        T *gb = reinterpret_cast<T *>(a.gcolbuf) + ((long)(c0 / BKC) * s.K + k) * s.M * BKC;
#pragma unroll
        for (int i = 0; i < ITEMS; i++) {
            const int item = tid + i * kThreads;
            const int pos = item / NV, vec = item % NV;
            const int m = m0 + pos;
            if (m < s.M) {
                const float *gp = reinterpret_cast<const float *>(s_gcol + pos * GRS + vec * VEC * 4);
                uint4 *dst = reinterpret_cast<uint4 *>(gb + (long)m * BKC + vec * VEC);
                VecAcc<T> va;
#pragma unroll
                for (int e = 0; e < VEC; e++) va.a[e] = gp[e];
                if (a.add_aux) va.fma(1.f, *dst);
                uint4 o;
                if constexpr (sizeof(T) == 2) {
                    o = make_uint4(pack_bf16x2(va.a[0], va.a[1]), pack_bf16x2(va.a[2], va.a[3]),
                                   pack_bf16x2(va.a[4], va.a[5]), pack_bf16x2(va.a[6], va.a[7]));
                } else {
                    o = make_uint4(__float_as_uint(va.a[0]), __float_as_uint(va.a[1]), __float_as_uint(va.a[2]),
                                   __float_as_uint(va.a[3]));
                }
                *dst = o;
            }
        }
    }
}

// The grad-column product for bfloat16 reductions of 128, 256, 384 or 512 channels: one workgroup = 256 positions
// (a wavefront keeps the grad_out rows of 32 of them, its stationary operand), a step = 32 channels of one tap, i.e.
// half a channel chunk; the weight half-tiles ([32 channels][ogk], 32 KiB at 512) go through a ring of kColRing LDS
// buffers and are requested kColAhead steps before their use, one request per wavefront between two blocks of 8
// matrix instructions.  Against the 128-position / 64-channel shape of tiled_bwd_col_kernel: half the weight
// traffic per product, and a transfer has three steps to arrive instead of one (the loaded latency of a tile is
// about a whole step of that kernel, which waited for it at every step).  The product is taken transposed and
// stored from the registers: the lane's weight row is chosen such that its 16 accumulator registers are two runs
// of 8 consecutive channels (see mma8_bf16_t).
constexpr int kColRing = 4, kColAhead = 3;
// ADD (the later passes over a weight group wider than 512 channels): the rows that the passes before it left are
// added, the sum formed in float and rounded to bfloat16 once more.
template <int NB, bool ADD>   // blocks of 8 k-groups: ogk = 128 NB
__global__ void __launch_bounds__(kThreads) tiled_bwd_col32_kernel(BwdDataArgs a)
{
    typedef bf16_t T;
    constexpr int VEC = 8, BKC = 64, HC = 32, MT = 256, NKG = 8 * NB, NW = kThreads / 64;
    constexpr int R = NB;                    // requests per wavefront and half-tile (32 rows x ogk / 8 pieces / 64 / 8)
    static_assert(kColAhead < kColRing && kColRing == 4, "a buffer is refilled a step after its last reader at the earliest");
    extern __shared__ __align__(16) unsigned char smem[];
    const TiledShape &s = a.s;
    const int rowB = a.ogk * (int)sizeof(T), tileB = HC * rowB, rp = rowB / 16;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tile = xcd_swizzle(blockIdx.x, gridDim.x);
    const int wg = blockIdx.y;
    const int m0 = tile * MT;
    const int S = s.nchunk * s.K, S2 = 2 * S;
    const bool full_tile = m0 + MT <= s.M;

    // ---- stationary operand: gout[pos, o] of this wavefront's 32 positions
    uint4 ga[NKG];
    {
        const int m = m0 + wave * 32 + (lane & 31);
        const bool ok = m < s.M;
        const int b = ok ? m / s.P : 0, p = ok ? m - b * s.P : 0;
        const T *gp = reinterpret_cast<const T *>(a.gout) + ((long)b * s.Cout + wg * s.og + a.o0) * s.P + p;
#pragma unroll
        for (int kg = 0; kg < NKG; kg++) {
            T e[VEC];
#pragma unroll
            for (int i = 0; i < VEC; i++) {
                const int o = (kg * 2 + (lane >> 5)) * VEC + i;
                e[i] = (ok && o < a.ogn) ? gp[(long)o * s.P] : (T)0;
            }
            ga[kg] = *reinterpret_cast<uint4 *>(e);
        }
    }

    // request q (0 .. R-1) of this wavefront for half-tile h2 (= 2 * step + half, in the order of the data kernel's
    // steps) into ring buffer `buf`: 64 pieces of 16 bytes to 1 KiB of consecutive LDS, lane i fetching the piece
    // that the swizzled layout wants there
    int psrc[R];      // (which piece of a half-tile the lane fetches does not change from step to step)
#pragma unroll
    for (int q = 0; q < R; q++) {
        const int pos = (wave + q * NW) * 64 + lane;
        const int row = pos / rp, pc = pos - row * rp;
        psrc[q] = row * rp + (pc ^ swizzle_of_row(row));
    }
    auto dma_piece = [&](int h2, int buf, int q) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.wt) + (((long)wg * S + (h2 >> 1)) * BKC + (h2 & 1) * HC) * rp;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + psrc[q]),
                                         (__attribute__((address_space(3))) void *)(smem + buf * tileB + (wave + q * NW) * 1024),
                                         16, 0, 0);
    };

    // LDS addresses of this lane's fragments of the first 8 k-groups in the ring buffer of the current step; the lane's
    // weight row is the one that makes its 16 accumulator registers two runs of 8 consecutive channels
    unsigned woff[8];
    {
        const int ml = lane & 31, i = ml >> 3, hq = (ml >> 2) & 1, j = ml & 3;
        const int wrow = i < 2 ? 8 * hq + 4 * i + j : 16 + 8 * hq + 4 * (i - 2) + j;
        const int wsw = swizzle_of_row(wrow), wh = lane >> 5;
        const unsigned lbase = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)smem;
#pragma unroll
        for (int q = 0; q < 8; q++) woff[q] = lbase + (unsigned)(wrow * rowB + (((q * 2 + wh) ^ wsw) << 4));
    }

    const int hs_lo = a.h_hi ? a.h_lo : 0, hs_n = (a.h_hi ? a.h_hi : S2) - hs_lo;
    const int lo = hs_lo + (int)((long)hs_n * blockIdx.z / gridDim.z), hi = hs_lo + (int)((long)hs_n * (blockIdx.z + 1) / gridDim.z);
    if (lo >= hi) return;
    // (past the end of the range the last half-tile is requested again, into buffers nobody reads: the same number
    // of requests in every step, which the counted waits below rely on)
#pragma unroll
    for (int d = 0; d < kColAhead; d++)
#pragma unroll
        for (int q = 0; q < R; q++) dma_piece(min(lo + d, hi - 1), d, q);

    const int cpc2 = 2 * (s.cpg / BKC);        // half-steps per (offset group, tap)
    // where this lane's 2 x 8 channels of half-step h2 go (step order: offset group (outer), tap, chunk of the group,
    // half (inner))
    const int m_lane = m0 + wave * 32 + (lane & 31);
    auto row_of = [&](int h2) -> T * {
        const int jj2 = h2 % cpc2, k = (h2 / cpc2) % s.K, gi = h2 / (cpc2 * s.K);
        const int j = gi * (cpc2 >> 1) + (jj2 >> 1), half = jj2 & 1;
        const int c0 = wg * s.cg + j * BKC;
        T *gb = reinterpret_cast<T *>(a.gcolbuf) + ((long)(c0 / BKC) * s.K + k) * s.M * BKC;
        return gb + (long)m_lane * BKC + half * HC + 8 * (lane >> 5);
    };
    for (int h2 = lo, it = 0; h2 < hi; h2++, it++) {
        // Half-tile `it` has landed when no more of this wavefront's operations are in flight than it has issued
        // since: the requests of the kColAhead - 1 half-tiles behind it, and the 2 stores of each step since then
        // (only counted when every wavefront of the workgroup stores in every step); ADD: also the 2 loads at the
        // top of the kColAhead - 1 steps since.
        wait_vm_at_most((kColAhead - 1) * R +
                        ((full_tile && it >= kColAhead) ? 2 * kColAhead + (ADD ? 2 * (kColAhead - 1) : 0) : 0));
        lds_only_barrier();
        // (ADD: the rows as the passes before left them, wanted at the end of the step.  Requesting them up to four
        // steps ahead made the pass slower: the counter above completes in order, so a row that is late holds up
        // the weight tiles requested after it.)
        T *row = row_of(h2);
        uint4 pv0 = make_uint4(0, 0, 0, 0), pv1 = pv0;
        if constexpr (ADD) {
            if (m_lane < s.M) {
                pv0 = *reinterpret_cast<const uint4 *>(row);
                pv1 = *reinterpret_cast<const uint4 *>(row + 16);
            }
        }

        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.f;
        const int nx = min(h2 + kColAhead, hi - 1), nbuf = (it + kColAhead) & (kColRing - 1);
        asm volatile("s_nop 4" ::: "memory");
        mma8_bf16_t<0>(acc, ga, woff);
        dma_piece(nx, nbuf, 0);
        if constexpr (NB >= 2) {
            mma8_bf16_t<256>(acc, ga + 8, woff);
            dma_piece(nx, nbuf, 1);
        }
        if constexpr (NB >= 3) {
            mma8_bf16_t<512>(acc, ga + 16, woff);
            dma_piece(nx, nbuf, 2);
        }
        if constexpr (NB >= 4) {
            mma8_bf16_t<768>(acc, ga + 24, woff);
            dma_piece(nx, nbuf, 3);
        }
        asm volatile("s_nop 15\n\ts_nop 7" : "+v"(acc)::"memory");
        // (the fragment addresses move on to the next buffer of the ring)
        const unsigned adv = ((it + 1) & (kColRing - 1)) ? (unsigned)tileB : (unsigned)(-(kColRing - 1) * tileB);
#pragma unroll
        for (int q = 0; q < 8; q++) woff[q] += adv;

        if (m_lane < s.M) {
            if constexpr (ADD) {
                const unsigned pw[8] = {pv0.x, pv0.y, pv0.z, pv0.w, pv1.x, pv1.y, pv1.z, pv1.w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    acc[2 * e] += __uint_as_float(pw[e] << 16);
                    acc[2 * e + 1] += __uint_as_float(pw[e] & 0xffff0000u);
                }
            }
            *reinterpret_cast<uint4 *>(row) =
                make_uint4(pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3]), pack_bf16x2(acc[4], acc[5]),
                           pack_bf16x2(acc[6], acc[7]));
            *reinterpret_cast<uint4 *>(row + 16) =
                make_uint4(pack_bf16x2(acc[8], acc[9]), pack_bf16x2(acc[10], acc[11]), pack_bf16x2(acc[12], acc[13]),
                           pack_bf16x2(acc[14], acc[15]));
        }
    }
    wait_vm_at_most(0);     // (transfers into this workgroup's LDS must not outlive it)
}

// The same kernel for float problems on two-term bfloat16 operands (TiledShape::f32split).  A step = the 32 channels
// of one chunk and tap; its weight tile in LDS is [32 channels][high halves of the 128 NBP reduced channels | their
// low halves] in bfloat16 (pack_weight_bwd_planes_kernel), as large as the bfloat16 kernel's for twice the
// channels; the stationary grad_out rows are kept as a high and a low half too, and the product is
// high x high + low(weight) x high + high(weight) x low, three blocks of matrix instructions per 128 channels instead
// of one (the product of the two low halves, at most 2^-18 of the term, is of the size of the error that the
// rounding of the low halves leaves in the other two and is left out).  The rows leave as floats, two runs of 8
// consecutive channels per lane.  ADD as above.
template <int NBP, bool ADD>   // reduced channels: 128 NBP
__global__ void __launch_bounds__(kThreads) tiled_bwd_col32f_kernel(BwdDataArgs a)
{
    constexpr int BKC = 32, MT = 256, NKG = 8 * NBP, NW = kThreads / 64;
    constexpr int R = 2 * NBP;               // requests per wavefront and tile (32 rows x 512 NBP bytes / 16 / 64 / 8)
    constexpr int ST = 4, LD = ADD ? 4 : 0;  // 16-byte stores / loads of rows per step
    static_assert(kColAhead < kColRing && kColRing == 4, "a buffer is refilled a step after its last reader at the earliest");
    extern __shared__ __align__(16) unsigned char smem[];
    const TiledShape &s = a.s;
    constexpr int rowB = 2 * 128 * NBP * 2, tileB = BKC * rowB, rp = rowB / 16;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tile = xcd_swizzle(blockIdx.x, gridDim.x);
    const int wg = blockIdx.y;
    const int m0 = tile * MT;
    const int S = s.nchunk * s.K;
    const bool full_tile = m0 + MT <= s.M;

    // ---- stationary operand: gout[pos, o] of this wavefront's 32 positions, high and low halves
    uint4 gh[NKG], gm[NKG];
    {
        const int m = m0 + wave * 32 + (lane & 31);
        const bool ok = m < s.M;
        const int b = ok ? m / s.P : 0, p = ok ? m - b * s.P : 0;
        const float *gp = reinterpret_cast<const float *>(a.gout) + ((long)b * s.Cout + wg * s.og + a.o0) * s.P + p;
#pragma unroll
        for (int kg = 0; kg < NKG; kg++) {
            float e[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int o = (kg * 2 + (lane >> 5)) * 8 + i;
                e[i] = (ok && o < a.ogn) ? gp[(long)o * s.P] : 0.f;
            }
            uint32_t h[4], l[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                h[i] = pack_bf16x2(e[2 * i], e[2 * i + 1]);
                l[i] = pack_bf16x2(bf16_residual(e[2 * i], h[i] << 16), bf16_residual(e[2 * i + 1], h[i] & 0xffff0000u));
            }
            gh[kg] = make_uint4(h[0], h[1], h[2], h[3]);
            gm[kg] = make_uint4(l[0], l[1], l[2], l[3]);
        }
    }

    int psrc[R];
#pragma unroll
    for (int q = 0; q < R; q++) {
        const int pos = (wave + q * NW) * 64 + lane;
        const int row = pos / rp, pc = pos - row * rp;
        psrc[q] = row * rp + (pc ^ swizzle_of_row(row));
    }
    auto dma_piece = [&](int st, int buf, int q) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.wt) + ((long)wg * S + st) * BKC * rp;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + psrc[q]),
                                         (__attribute__((address_space(3))) void *)(smem + buf * tileB + (wave + q * NW) * 1024),
                                         16, 0, 0);
    };
    unsigned woff[8];
    {
        const int ml = lane & 31, i = ml >> 3, hq = (ml >> 2) & 1, j = ml & 3;
        const int wrow = i < 2 ? 8 * hq + 4 * i + j : 16 + 8 * hq + 4 * (i - 2) + j;
        const int wsw = swizzle_of_row(wrow), wh = lane >> 5;
        const unsigned lbase = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)smem;
#pragma unroll
        for (int q = 0; q < 8; q++) woff[q] = lbase + (unsigned)(wrow * rowB + (((q * 2 + wh) ^ wsw) << 4));
    }

    const int lo = (int)((long)S * blockIdx.z / gridDim.z), hi = (int)((long)S * (blockIdx.z + 1) / gridDim.z);
    if (lo >= hi) return;
#pragma unroll
    for (int d = 0; d < kColAhead; d++)
#pragma unroll
        for (int q = 0; q < R; q++) dma_piece(min(lo + d, hi - 1), d, q);

    const int cpc = s.cpg / BKC;               // steps per (offset group, tap)
    const int m_lane = m0 + wave * 32 + (lane & 31);
    // where this lane's 2 x 8 channels of a step go (step order: offset group (outer), tap, chunk of the group)
    auto row_of = [&](int st) -> float * {
        const int jj = st % cpc, k = (st / cpc) % s.K, gi = st / (cpc * s.K);
        const int c0 = wg * s.cg + (gi * cpc + jj) * BKC;
        float *gb = reinterpret_cast<float *>(a.gcolbuf) + ((long)(c0 / BKC) * s.K + k) * s.M * BKC;
        return gb + (long)m_lane * BKC + 8 * (lane >> 5);
    };
    for (int st = lo, it = 0; st < hi; st++, it++) {
        // (the counted wait of tiled_bwd_col32_kernel: the requests of the kColAhead - 1 tiles behind this one, and
        // the stores and loads of rows since its own requests)
        wait_vm_at_most((kColAhead - 1) * R +
                        ((full_tile && it >= kColAhead) ? ST * kColAhead + LD * (kColAhead - 1) : 0));
        lds_only_barrier();
        float *row = row_of(st);
        float4 pv[4] = {};
        if constexpr (ADD) {
            if (m_lane < s.M) {
                pv[0] = *reinterpret_cast<const float4 *>(row);
                pv[1] = *reinterpret_cast<const float4 *>(row + 4);
                pv[2] = *reinterpret_cast<const float4 *>(row + 16);
                pv[3] = *reinterpret_cast<const float4 *>(row + 20);
            }
        }

        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.f;
        const int nx = min(st + kColAhead, hi - 1), nbuf = (it + kColAhead) & (kColRing - 1);
        asm volatile("s_nop 4" ::: "memory");
        // high x high, then the weights' low halves x high, then high x the rows' low halves
        mma8_bf16_t<0>(acc, gh, woff);
        dma_piece(nx, nbuf, 0);
        if constexpr (NBP == 2) {
            mma8_bf16_t<256>(acc, gh + 8, woff);
            dma_piece(nx, nbuf, 1);
        }
        mma8_bf16_t<256 * NBP>(acc, gh, woff);
        dma_piece(nx, nbuf, NBP);
        if constexpr (NBP == 2) {
            mma8_bf16_t<768>(acc, gh + 8, woff);
            dma_piece(nx, nbuf, 3);
        }
        mma8_bf16_t<0>(acc, gm, woff);
        if constexpr (NBP == 2) mma8_bf16_t<256>(acc, gm + 8, woff);
        asm volatile("s_nop 15\n\ts_nop 7" : "+v"(acc)::"memory");
        const unsigned adv = ((it + 1) & (kColRing - 1)) ? (unsigned)tileB : (unsigned)(-(kColRing - 1) * tileB);
#pragma unroll
        for (int q = 0; q < 8; q++) woff[q] += adv;

        if (m_lane < s.M) {
            if constexpr (ADD) {
                const float pw[16] = {pv[0].x, pv[0].y, pv[0].z, pv[0].w, pv[1].x, pv[1].y, pv[1].z, pv[1].w,
                                      pv[2].x, pv[2].y, pv[2].z, pv[2].w, pv[3].x, pv[3].y, pv[3].z, pv[3].w};
#pragma unroll
                for (int e = 0; e < 16; e++) acc[e] += pw[e];
            }
            *reinterpret_cast<float4 *>(row) = make_float4(acc[0], acc[1], acc[2], acc[3]);
            *reinterpret_cast<float4 *>(row + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
            *reinterpret_cast<float4 *>(row + 16) = make_float4(acc[8], acc[9], acc[10], acc[11]);
            *reinterpret_cast<float4 *>(row + 20) = make_float4(acc[12], acc[13], acc[14], acc[15]);
        }
    }
    wait_vm_at_most(0);     // (transfers into this workgroup's LDS must not outlive it)
}

template <typename T> size_t bwd_col_lds(int ogk, bool db)
{
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC, CB = BKC / 32, MT = 32 * (8 / CB);
    return (size_t)(db ? 2 : 1) * BKC * ogk * sizeof(T) + (size_t)MT * col_row_stride<T>();
}

template <typename T, int NKG>
int launch_bwd_col(const BwdDataArgs &a, int nsplit, hipStream_t st, bool split)
{
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC, CB = BKC / 32, MT = 32 * (8 / CB);
    const bool db = bwd_col_lds<T>(a.ogk, true) <= 160 * 1024;
    const size_t lds = bwd_col_lds<T>(a.ogk, db);
    dim3 grid((a.s.M + MT - 1) / MT, a.s.groups, nsplit);
    auto go = [&](auto split_c) -> int {
        constexpr bool SP = decltype(split_c)::value;
        const void *fn = db ? (const void *)tiled_bwd_col_kernel<T, NKG, true, SP> : (const void *)tiled_bwd_col_kernel<T, NKG, false, SP>;
        if (int rc = d2c_allow_lds(fn, 160 * 1024, "tiled_bwd_col_kernel")) return rc;
        D2cProfScope prof(D2C_PROF_BWD_DATA, st, "tiled_bwd_col_kernel");
        if (db) hipLaunchKernelGGL((tiled_bwd_col_kernel<T, NKG, true, SP>), grid, dim3(kThreads), lds, st, a);
        else hipLaunchKernelGGL((tiled_bwd_col_kernel<T, NKG, false, SP>), grid, dim3(kThreads), lds, st, a);
        return d2c_check_launch("tiled_bwd_col_kernel");
    };
    if constexpr (sizeof(T) == 4) {
        if (split) return go(std::true_type{});
    }
    return go(std::false_type{});
}

constexpr int kCol32MT = 256;
// float problems on two-term operands: passes of 97 .. 128 or 225 .. 256 reduced channels (the two bfloat16 planes of
// 128 / 256 channels then fill exactly the buffer that holds the pass's float weights)
bool bwd_col32f_ok(int ogn, int dtype, bool split)
{
    return dtype == D2C_F32 && split && ((ogn > 96 && ogn <= 128) || (ogn > 224 && ogn <= 256));
}
int launch_bwd_col32f(const BwdDataArgs &a, int nsplit, hipStream_t st)
{
    const int nbp = a.ogn > 128 ? 2 : 1;
    const size_t lds = (size_t)kColRing * 32 * (2 * 128 * nbp * 2);
    const dim3 grid((a.s.M + kCol32MT - 1) / kCol32MT, a.s.groups, nsplit);
    auto go = [&](auto nb_c, auto add_c) -> int {
        constexpr int NBP = decltype(nb_c)::value;
        constexpr bool ADD = decltype(add_c)::value;
        if (int rc = d2c_allow_lds((const void *)tiled_bwd_col32f_kernel<NBP, ADD>, 160 * 1024, "tiled_bwd_col32f_kernel")) return rc;
        D2cProfScope prof(D2C_PROF_BWD_DATA, st, "tiled_bwd_col32f_kernel");
        hipLaunchKernelGGL((tiled_bwd_col32f_kernel<NBP, ADD>), grid, dim3(kThreads), lds, st, a);
        return d2c_check_launch("tiled_bwd_col32f_kernel");
    };
    if (nbp == 2) return a.add_aux ? go(std::integral_constant<int, 2>{}, std::true_type{}) : go(std::integral_constant<int, 2>{}, std::false_type{});
    return a.add_aux ? go(std::integral_constant<int, 1>{}, std::true_type{}) : go(std::integral_constant<int, 1>{}, std::false_type{});
}
bool bwd_col32_ok(int ogk, int ogn, int dtype) { return dtype == D2C_BF16 && ogk % 128 == 0 && ogk <= 512 && ogn > 0; }
int launch_bwd_col32(const BwdDataArgs &a, int nsplit, hipStream_t st)
{
    const size_t lds = (size_t)kColRing * 32 * a.ogk * 2;
    const dim3 grid((a.s.M + kCol32MT - 1) / kCol32MT, a.s.groups, nsplit);
    auto go = [&](auto nb_c, auto add_c) -> int {
        constexpr int NB = decltype(nb_c)::value;
        constexpr bool ADD = decltype(add_c)::value;
        if (int rc = d2c_allow_lds((const void *)tiled_bwd_col32_kernel<NB, ADD>, 160 * 1024, "tiled_bwd_col32_kernel")) return rc;
        D2cProfScope prof(D2C_PROF_BWD_DATA, st, "tiled_bwd_col32_kernel");
        hipLaunchKernelGGL((tiled_bwd_col32_kernel<NB, ADD>), grid, dim3(kThreads), lds, st, a);
        return d2c_check_launch("tiled_bwd_col32_kernel");
    };
    auto pick = [&](auto add_c) -> int {
        switch (a.ogk / 128) {
        case 1: return go(std::integral_constant<int, 1>{}, add_c);
        case 2: return go(std::integral_constant<int, 2>{}, add_c);
        case 3: return go(std::integral_constant<int, 3>{}, add_c);
        default: return go(std::integral_constant<int, 4>{}, add_c);
        }
    };
    return a.add_aux ? pick(std::true_type{}) : pick(std::false_type{});
}

template <typename T> size_t bwd_data_lds(int ogk)
{
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC, CB = BKC / 32, MT = 32 * (8 / CB);
    return (size_t)BKC * ogk * sizeof(T) + (size_t)MT * (BKC * 4 + 16) + (size_t)MT * (8 + 6 + 1 + 1 + 1) * 4;
}

template <typename T, int NKG>
int launch_bwd_data(const BwdDataArgs &a, int nsplit, hipStream_t st, bool split)
{
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC, CB = BKC / 32, MT = 32 * (8 / CB);
    const size_t lds = bwd_data_lds<T>(a.ogk);
    dim3 grid((a.s.M + MT - 1) / MT, a.s.groups, nsplit);
    auto go = [&](auto split_c) -> int {
        constexpr bool SP = decltype(split_c)::value;
        if (int rc = d2c_allow_lds((const void *)tiled_bwd_data_kernel<T, NKG, SP>, 160 * 1024, "tiled_bwd_data_kernel")) return rc;
        D2cProfScope prof(D2C_PROF_BWD_DATA, st, "tiled_bwd_data_kernel");
        hipLaunchKernelGGL((tiled_bwd_data_kernel<T, NKG, SP>), grid, dim3(kThreads), lds, st, a);
        return d2c_check_launch("tiled_bwd_data_kernel");
    };
    if constexpr (sizeof(T) == 4) {
        if (split) return go(std::true_type{});
    }
    return go(std::false_type{});
}

// ============================================================ kernel 2
struct BwdWeightArgs {
    TiledShape s;
    const void *gout, *xcl, *off, *mask;
    const void *goutp;   // grad_out in MFMA fragment order, see pack_gout_kernel
    float *gwacc;   // [group][chunk*K + tap][og][BKC] fp32 accumulator (zeroed): channel-contiguous rows, so that
                    // the atomics of a wavefront fill whole cache lines
    // The position tiles of an item (weight group, output tile, step) are shared out to nmain + ntail workgroups: the
    // first nmain * main_len tiles are dealt round-robin to the `nmain` main workgroups (those of an item work on
    // neighbouring tiles at any time, which their XCD's L2 likes), the rest likewise to the `ntail` tail workgroups.
    // The main workgroups of all items come first in the grid.  Either ntail == 0 and the main workgroups take all
    // tiles, or the main pieces are as long as the whole launch should take and start at once, and the short tail
    // pieces fill the compute units that are left.
    int otiles, nmain, main_len, ntail, tail_len;
};

constexpr int kWMT = 128;  // positions per tile of the packed grad_out copy

// One workgroup = one (chunk, tap) step, all output channels of the weight group (8 worker wavefronts x 64
// rows), looping over its piece of the 64-position tiles (see BwdWeightArgs).  The corner rows go global -> LDS by DMA loads
// (no gather registers) and the coordinates are computed by a ninth wavefront: while the matrix cores take
// tile `it`, tile it+1 is interpolated from LDS, the rows of tile it+2 are in flight and the table of tile
// it+3 is computed.  Same roles and ring buffers as tiled_fwd_dma_kernel (d2c_tiled_fwd.hip).
constexpr int kWDT = 64;                    // positions per iteration

struct BwdWeightDmaArgs {
    BwdWeightArgs w;
    unsigned zrow;       // byte offset (from xcl) of a 128-byte row of zeros: what dead corners read
};

// NC: corner rows per sampling point, 8, or 4 / 2 when offsets along one / two axes are fixed (see fwd_dma_body).
template <typename T, bool AUX16, bool SIZED, int NC, bool SPLIT>
__global__ void __launch_bounds__(kThreads + 64) tiled_bwd_weight_dma_kernel(BwdWeightDmaArgs aa)
{
    constexpr int RAWPOS = NC * 128;           // raw bytes per position
    constexpr int PPI = 8 / NC;                // positions per DMA instruction
    constexpr int MT = kWDT;
    constexpr int VEC = Elem<T>::VEC;          // positions per 16-byte operand vector
    constexpr int BKC = 8 * VEC;               // channels per step (64 / 32)
    constexpr int CB = BKC / 32;
    constexpr int OB = 2;                      // 32-row blocks of output channels per wavefront
    constexpr int NT = 64 * 8;                 // output channels per workgroup
    constexpr int TRS = MT * (int)sizeof(T) + 16;   // tile row stride: [channel][position]
    constexpr int NKG = MT / (2 * VEC);        // k-groups per iteration (4 / 8)
    constexpr int NKGP = kWMT / (2 * VEC);     // k-groups per tile of the packed grad_out copy
    static_assert(MT * 8 == kThreads, "one (position, vector) item per worker thread");

    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char *s_raw = smem;                                       // [2][MT][8 corners][128 B]
    unsigned char *s_tile = s_raw + 2 * MT * RAWPOS;                   // [2][BKC][TRS]
    float *s_w = reinterpret_cast<float *>(s_tile + 2 * BKC * TRS);    // [3][8][MT]
    int2 *s_if = reinterpret_cast<int2 *>(s_w + 3 * 8 * MT);           // [3][MT] (offset of corner 000, live corners)

    const BwdWeightArgs &a = aa.w;
    const TiledShape &s = a.s;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool worker = wave < 8;
    // step = chunk * K + tap.  Workgroups are dealt round-robin to the 8 XCDs; an XCD takes a contiguous range of
    // the items, i.e. the taps of one or two channel chunks: its L2 then holds the corner rows of those channels only
    // (one eighth of the input at 8 chunks) instead of all of them
    const int ntile = (s.M + MT - 1) / MT;
    const int nstep = s.nchunk * s.K;
    const int nitem = s.groups * a.otiles * nstep;
    int item, t_lo, nmy, t_step;
    if ((int)blockIdx.x < nitem * a.nmain) {
        item = xcd_swizzle(blockIdx.x % nitem, nitem);
        t_lo = blockIdx.x / nitem;
        t_step = a.nmain;
        const int nt = min(ntile, a.nmain * a.main_len);
        nmy = nt > t_lo ? (nt - t_lo + t_step - 1) / t_step : 0;
    } else {
        const int id = blockIdx.x - nitem * a.nmain;
        item = xcd_swizzle(id % nitem, nitem);
        t_lo = a.nmain * a.main_len + id / nitem;
        t_step = a.ntail;
        nmy = ntile > t_lo ? (ntile - t_lo + t_step - 1) / t_step : 0;
    }
    if (nmy <= 0) return;
    const int st = item % nstep, otile = (item / nstep) % a.otiles, wg = item / (nstep * a.otiles);
    const int j = st / s.K, k = st - j * s.K;
    const int c0 = wg * s.cg + j * BKC;
    const int g = c0 / s.cpg;
    const int dzc = s.H * s.W * s.Cin, dyc = s.W * s.Cin;
    const int o_base = otile * NT + wave * 64;
    const bool mma_wave = worker && o_base < s.og;

    f32x16 acc[OB][CB];
#pragma unroll
    for (int ob = 0; ob < OB; ob++)
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[ob][cb][r] = 0.f;

    // --- coordinate wavefront: lane = position of tile i.  The tap is the workgroup's own: its constants are formed
    // once; an iteration takes the position apart (multiplications, no division) and builds the table row.
    const int ctid = tid - kThreads;
    typedef typename std::conditional<AUX16, bf16_t, float>::type AT;
    const CoordConst cc = coord_const(s);
    const int kq[3] = {k / (s.geo.kw * s.geo.kh), (k / s.geo.kw) % s.geo.kh, k % s.geo.kw};
    // where the tap sits relative to (o * stride), as float
    float tapf[3] = {(float)(kq[0] * s.geo.dd - s.geo.pd), (float)(kq[1] * s.geo.dh - s.geo.ph),
                     (float)(kq[2] * s.geo.dw - s.geo.pw)};
    opaque_v(tapf[0]); opaque_v(tapf[1]); opaque_v(tapf[2]);
    float sbase[3] = {0.f, 0.f, 0.f};   // kernel-grid coordinates of the tap (size-map source)
    if constexpr (SIZED) {
#pragma unroll
        for (int ax = 0; ax < 3; ax++) sbase[ax] = rnd<AT>(s.ss.base[ax][kq[ax]]);
    }
    const long cstride = s.nd == 3 ? (long)s.P * (long)sizeof(AT) : 0;
    const long off_tap = (long)(s.nd == 3 ? 3 : 1) * s.P * (long)sizeof(AT);   // bytes per (sample, group, tap)
    const long mask_tap = (long)s.P * (long)sizeof(AT);
    const unsigned off_sample = (unsigned)s.obs * (unsigned)sizeof(AT), mask_sample = (unsigned)s.mbs * (unsigned)sizeof(AT);
    float craw[4] = {0.f, 0.f, 0.f, 1.f};
    int cb_ = 0, cp_ = 0;
    bool cvalid = false;
    auto coords_issue = [&](int i) {
        if (worker) return;
        const int m0 = (t_lo + i * t_step) * MT;                // (m < N * P < 2^31)
        const int m = m0 + ctid;
        cvalid = m < s.M;
        // (a lane without a position reads what the tile's first position reads)
        const int mq = cvalid ? m : m0;
        const int b_lo = fdiv(m0, s.dP);                        // uniform: the tile's first sample
        cb_ = fdiv(mq, s.dP); cp_ = mq - cb_ * s.P;
        if constexpr (SIZED) {
            tap_offsets_issue<AUX16, true>(s, a.off, cb_, g, k, cp_, craw);
        } else {
            const char *ub = reinterpret_cast<const char *>(a.off) + (long)b_lo * s.obs * (long)sizeof(AT) + ((long)g * s.K + k) * off_tap;
            coord_offsets_issue<AUX16>(ub, cstride, (unsigned)(cb_ - b_lo) * off_sample + (unsigned)cp_ * (unsigned)sizeof(AT), craw);
        }
        if (a.mask) {
            const char *um = reinterpret_cast<const char *>(a.mask) + (long)b_lo * s.mbs * (long)sizeof(AT) + ((long)g * s.K + k) * mask_tap;
            craw[3] = ld_aux_at<AUX16>(um, (unsigned)(cb_ - b_lo) * mask_sample + (unsigned)cp_ * (unsigned)sizeof(AT));
        }
    };
    auto coords_finish = [&](int buf) {   // of the tile whose offsets coords_issue requested last
        if (worker) return;
        const int oz = fdiv(cp_, s.dHW), rem = cp_ - oz * (s.Wo * s.Ho);
        const int oy = fdiv(rem, s.dW), ox = rem - oy * s.Wo;
        if constexpr (SIZED) {
            // size-map source: offsets = base_a[k_a] * (size_a - 1); the tap is this workgroup's own
            if (s.ss.on == 1) size_minus_one<AUX16>(s, craw);
#pragma unroll
            for (int ax = 0; ax < 3; ax++) craw[ax] = rnd<AT>(sbase[ax] * craw[ax]);
        }
        coord_offsets_select(cc, craw);
        if (s.mact && a.mask) craw[3] = mask_act<AT>(s.mact, craw[3]);
        const CornerRow r = corner_row(cc, ((float)__mul24(oz, s.geo.sd) + tapf[0]) + craw[0],
                                       ((float)__mul24(oy, s.geo.sh) + tapf[1]) + craw[1],
                                       ((float)__mul24(ox, s.geo.sw) + tapf[2]) + craw[2], craw[3], cb_ * s.vol, cvalid);
#pragma unroll
        for (int c = 0; c < 8; c++) s_w[(buf * 8 + c) * MT + ctid] = r.w[c];
        s_if[buf * MT + ctid] = make_int2(r.idx, (int)r.live);
    };

    // --- corner rows of tile i -> s_raw[rbuf]: worker wavefront w requests positions 8w .. 8w+7
    // (with fewer than 8 corners an instruction covers 8 / NC positions: lane = (position, corner slot, vector))
    const int dslot = (lane >> 3) % NC, dsub = (lane >> 3) / NC, dvec = lane & 7;
    const int dcorner = NC == 8 ? dslot : corner_of_slot(dslot, s.axes);
    const int dcoff = ((dcorner >> 2) & 1) * dzc + ((dcorner >> 1) & 1) * dyc + (dcorner & 1) * s.Cin;
    auto dma_issue = [&](int rbuf, int tbuf) {
        if (!worker) return;
        const char *base = reinterpret_cast<const char *>(a.xcl);
        const int2 vif = s_if[tbuf * MT + wave * (MT / 8) + (lane & 7)];
        const int vidx = vif.x, vflag = vif.y;
#pragma unroll
        for (int i = 0; i < MT / 8 / PPI; i++) {
            const int pos0 = wave * (MT / 8) + i * PPI;
            int idx;
            unsigned live;
            if constexpr (PPI == 1) {
                idx = __builtin_amdgcn_readlane(vidx, i);
                live = (unsigned)__builtin_amdgcn_readlane(vflag, i);
            } else {
                idx = __builtin_amdgcn_ds_bpermute((i * PPI + dsub) << 2, vidx);
                live = (unsigned)__builtin_amdgcn_ds_bpermute((i * PPI + dsub) << 2, vflag);
            }
            const unsigned o = ((live >> dcorner) & 1u)
                                   ? (unsigned)(idx + c0 + dcoff + dvec * VEC) * (unsigned)sizeof(T)
                                   : aa.zrow + (unsigned)dvec * 16u;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(base + o),
                                             (__attribute__((address_space(3))) void *)(s_raw + (rbuf * MT + pos0) * RAWPOS),
                                             16, 0, 0);
        }
    };
    // --- interpolation; thread = (position, 16-byte vector)
    const int ipos = tid >> 3, ivec = tid & 7;
    int wslot[NC];      // row of the weight table that belongs to corner slot c
#pragma unroll
    for (int c = 0; c < NC; c++) wslot[c] = (NC == 8 ? c : corner_of_slot(c, s.axes)) * MT;
    auto interp_store = [&](int rbuf, int tbuf, int dbuf) {
        if (!worker) return;
        // (the rows are read behind the compiler's back, see lds_row_read: the transfers just requested for tile
        // i + 2 stay in flight while tile i + 1 is interpolated)
        const unsigned rp = lds_address(s_raw + (rbuf * MT + ipos) * RAWPOS + ivec * 16);
        VecAcc<T> va;
        va.zero();
        if constexpr (NC == 2) {
            u32x4_t r0 = lds_row_read<0>(rp), r1 = lds_row_read<128>(rp);
            const float w0 = s_w[tbuf * 8 * MT + wslot[0] + ipos], w1 = s_w[tbuf * 8 * MT + wslot[1] + ipos];
            lds_rows_wait(r0, r1);
            va.fma(w0, __builtin_bit_cast(uint4, r0));
            va.fma(w1, __builtin_bit_cast(uint4, r1));
        } else {
#pragma unroll
            for (int h = 0; h < NC / 4; h++) {
                u32x4_t r0 = h ? lds_row_read<512>(rp) : lds_row_read<0>(rp);
                u32x4_t r1 = h ? lds_row_read<640>(rp) : lds_row_read<128>(rp);
                u32x4_t r2 = h ? lds_row_read<768>(rp) : lds_row_read<256>(rp);
                u32x4_t r3 = h ? lds_row_read<896>(rp) : lds_row_read<384>(rp);
                float w[4];
#pragma unroll
                for (int c = 0; c < 4; c++) w[c] = s_w[tbuf * 8 * MT + wslot[h * 4 + c] + ipos];
                lds_rows_wait(r0, r1, r2, r3);
                va.fma(w[0], __builtin_bit_cast(uint4, r0));
                va.fma(w[1], __builtin_bit_cast(uint4, r1));
                va.fma(w[2], __builtin_bit_cast(uint4, r2));
                va.fma(w[3], __builtin_bit_cast(uint4, r3));
            }
        }
        if constexpr (sizeof(T) == 2) {
            // bfloat16: the tile stays [position][channel] (one 16-byte store, rows of TRS bytes: MT == BKC);
            // the matrix wavefronts read it with the transposing LDS load, see mma_tile
            static_assert(sizeof(T) != 2 || MT == BKC, "tile rows of either orientation have the same length");
            *reinterpret_cast<uint4 *>(s_tile + (dbuf * MT + ipos) * TRS + ivec * 16) = va.pack();
        } else {
            // float: stored transposed ([channel][position]), one element per store
            unsigned char *tb = s_tile + dbuf * BKC * TRS + (ivec * VEC) * TRS;
            if constexpr (SPLIT) {
                // (as the two bfloat16 halves of a matrix-instruction operand: the 16 bytes of four consecutive
                // positions hold their four `hi` values, then their four `lo` values)
                unsigned char *tg = tb + (ipos >> 2) * 16 + (ipos & 3) * 2;
#pragma unroll
                for (int e = 0; e < VEC; e++) {
                    const bf16_t hi = f32_to_bf16(va.a[e]);
                    *reinterpret_cast<bf16_t *>(tg + e * TRS) = hi;
                    *reinterpret_cast<bf16_t *>(tg + e * TRS + 8) = f32_to_bf16(bf16_residual(va.a[e], (uint32_t)hi << 16));
                }
            } else {
#pragma unroll
                for (int e = 0; e < VEC; e++) *reinterpret_cast<float *>(tb + e * TRS + ipos * 4) = va.a[e];
            }
        }
    };

    // --- gW block += gout[o, pos] * tile[pos, c]; gout fragments straight from the packed copy
    const int OBT = (s.og + 63) / 64 * 2;
    const int ntp = (s.M + kWMT - 1) / kWMT;     // tiles of the packed copy (kWMT positions each)
    const uint4 *gp4 = reinterpret_cast<const uint4 *>(a.goutp);
    auto gfrag = [&](int i, int kg, int ob) {
        const long t64 = t_lo + (long)i * t_step;
        const long tp = t64 / (kWMT / MT);
        const int kgp = (int)(t64 % (kWMT / MT)) * NKG + kg;
        return gp4[((((long)wg * ntp + tp) * OBT + (o_base >> 5) + ob) * NKGP + kgp) * 64 + lane];
    };
    uint4 ld[8];   // four k-groups in flight; a slot is refilled as soon as the matrix cores have taken it
    auto mma_tile = [&](int i, int dbuf) {
        if (!mma_wave) return;
#pragma unroll
        for (int kg = 0; kg < NKG; kg++) {
            const int kq = kg & 3;
            uint4 bf[CB];
            if constexpr (sizeof(T) == 2) {
                // ds_read_b64_tr_b16: within 16 lanes, lane l element j comes from lane 4j + l/4, element l%4.
                // Source lane (j, q) reads 4 channels of position +j; receiving lane (q, e) then holds channel
                // 4q + e of 4 consecutive positions: two such loads make the 8 positions of an operand vector.
                typedef short v4s __attribute__((ext_vector_type(4)));
                const int l16 = lane & 15, g16 = lane >> 4;
#pragma unroll
                for (int cb = 0; cb < CB; cb++) {
                    const int pos = kg * 16 + (g16 >> 1) * 8 + (l16 >> 2);
                    const int ch = cb * 32 + (g16 & 1) * 16 + (l16 & 3) * 4;
                    const unsigned char *ap = s_tile + (dbuf * MT + pos) * TRS + ch * 2;
                    const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)ap);
                    const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)(ap + 4 * TRS));
                    const uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
                    bf[cb] = make_uint4(lo2.x, lo2.y, hi2.x, hi2.y);
                }
            } else {
#pragma unroll
                for (int cb = 0; cb < CB; cb++) {
                    const int row = cb * 32 + (lane & 31);
                    bf[cb] = *reinterpret_cast<const uint4 *>(s_tile + dbuf * BKC * TRS + row * TRS
                                                              + ((kg * 2 + (lane >> 5)) << 4));
                }
            }
#pragma unroll
            for (int ob = 0; ob < OB; ob++)
#pragma unroll
                for (int cb = 0; cb < CB; cb++) mma_kgroup<T, SPLIT>(acc[ob][cb], ld[kq * 2 + ob], bf[cb]);
            if (kg + 4 < NKG) {
#pragma unroll
                for (int ob = 0; ob < OB; ob++) ld[kq * 2 + ob] = gfrag(i, kg + 4, ob);
            } else if (i + 1 < nmy) {
#pragma unroll
                for (int ob = 0; ob < OB; ob++) ld[kq * 2 + ob] = gfrag(i + 1, kg + 4 - NKG, ob);
            }
        }
    };

    if (nmy > 0) {
        if (mma_wave) {
#pragma unroll
            for (int kq = 0; kq < 4; kq++)
#pragma unroll
                for (int ob = 0; ob < OB; ob++) ld[kq * 2 + ob] = gfrag(0, kq, ob);
        }
        for (int q = 0; q < 3; q++) {
            if (q < nmy) {
                coords_issue(q);
                coords_finish(q % 3);
            }
        }
        __syncthreads();
        dma_issue(0, 0);
        if (1 < nmy) dma_issue(1, 1);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        interp_store(0, 0, 0);
        if (3 < nmy) coords_issue(3);
        if (worker) {
            for (int it = 0; it < nmy; it++) {
                __builtin_amdgcn_s_waitcnt(0);     // the transfers requested in the last iteration have landed
                __syncthreads();
                mma_tile(it, it & 1);
                if (it + 2 < nmy) dma_issue(it & 1, (it + 2) % 3);
                if (it + 1 < nmy) interp_store((it + 1) & 1, (it + 1) % 3, (it + 1) & 1);
            }
        } else {
            // (at default priority: issuing ahead of the two worker wavefronts of its SIMD paid while this code was
            // three times as long; with the short version it costs 5 - 8 %)
            for (int it = 0; it < nmy; it++) {
                // (a barrier that waits for this wavefront's LDS stores only: the offsets it requested stay in
                // flight across it and are waited for where they are used, a whole iteration after the request)
                lds_only_barrier();
                if (it + 3 < nmy) {
                    __builtin_amdgcn_s_waitcnt(0x0F70);    // vmcnt(0)
                    coords_finish(it % 3);
                }
                if (it + 4 < nmy) coords_issue(it + 4);
            }
        }
    }

    if (mma_wave) {
#pragma unroll
        for (int ob = 0; ob < OB; ob++)
#pragma unroll
            for (int cb = 0; cb < CB; cb++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int ol = o_base + ob * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (ol < s.og)
                        atomicAdd(a.gwacc + (((long)wg * s.nchunk * s.K + st) * s.og + ol) * BKC + cb * 32 + (lane & 31),
                                  acc[ob][cb][r]);
                }
    }
}

// ============================================================ kernel 2b
// grad_weight as a plain matrix product over sampled columns held in device memory -- the ones the offset / mask
// gradient kernel left there (aux_grad_kernel<.., COL>; bfloat16 problems), or the ones the forward call of the same
// step kept (tiled_fwd_dma_kernel<.., COLS>; bfloat16 and float):
//     gW[o, (chunk, tap, c)] += sum_pos gout[o, pos] * col[chunk][tap][pos][c]
// One workgroup = one tap and kColChunks channel chunks (128 / 64 columns), all output channels of the weight group (8
// wavefronts x 64 rows), looping over its piece of the 64-position tiles.  No sampling here: the input is not read
// again, there is no coordinate wavefront and no interpolation.  The column tiles (2 x 8 KiB per step) go through
// registers into a double-buffered LDS tile (one 16-byte load per lane and tile, requested a step ahead, and one
// LDS store -- float: four, the tile is kept [channel][position] as the float matrix instruction wants it), the
// grad_out fragments come straight from the fragment-ordered copy, ahead as well.  All loads are ordinary ones, so
// the compiler counts its waits; the barrier waits for LDS operations only.  Twice the columns per grad_out fragment
// of tiled_bwd_weight_dma_kernel: half the fragment traffic per product.
constexpr int kColChunks = 2;

struct BwdWeightColArgs {
    TiledShape s;
    const void *col;     // [chunk][tap][mpad][BKC]
    const void *goutp;   // grad_out in MFMA fragment order, see pack_gout_kernel
    float *gwacc;        // as in BwdWeightArgs
    long mpad;           // rows per (chunk, tap) of `col`: whole 64-position tiles, or N*P when the columns took the place
                         // of the grad-column rows (the last tile then reads into the next block, or the zeroed pad
                         // behind the last one: finite values that meet the zero tail of the grad_out copy)
    int otiles, nmain, main_len, ntail, tail_len;   // as in BwdWeightArgs
    int jp_lo, jp_n;     // the pairs of channel chunks [jp_lo, jp_lo + jp_n) of every weight group this launch works on
                         // (a slice of the backward pass; `col` then points where chunk 0 WOULD start if the buffer
                         // held all chunks)
};

template <typename T>
__global__ void __launch_bounds__(kThreads) tiled_bwd_weight_col_kernel(BwdWeightColArgs a)
{
    constexpr bool F32 = sizeof(T) == 4;
    constexpr int MT = kWDT, VEC = Elem<T>::VEC, BKC = 8 * VEC, NCH = kColChunks, CPB = BKC / 32, CB = NCH * CPB, OB = 2,
                  NT = 64 * 8;
    // bfloat16: tile rows are positions ([position][channel]), 64 bytes more than a row apart, so that the 64-byte
    // segments of four consecutive rows, which 32 lanes of a transposing read fetch together, fall into different
    // quarters of the 64 banks.  float: tile rows are channels ([channel][position]), an odd number of 16-byte units apart
    constexpr int TRS = F32 ? MT * 4 + 16 : MT * 2 + 64;
    constexpr int TROWS = F32 ? BKC : MT;      // rows of one tile
    constexpr int NKG = MT / (2 * VEC);        // k-groups per iteration
    constexpr int NKGP = kWMT / (2 * VEC);     // k-groups per tile of the packed grad_out copy
    // tiles of grad_out fragments in flight (float: 16 fragments per tile and 64 matrix instructions per fragment
    // pair, one tile ahead is a long time)
    constexpr int LA = F32 ? 1 : 2;
    static_assert(MT * 8 == kThreads, "one (position, vector) item per thread and column tile");
    __shared__ __align__(16) unsigned char s_tile[2 * NCH * TROWS * TRS];

    const TiledShape &s = a.s;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ntile = (s.M + MT - 1) / MT;
    const int nstep = a.jp_n * s.K;
    const int nitem = s.groups * a.otiles * nstep;
    int item, t_lo, nmy, t_step;
    if ((int)blockIdx.x < nitem * a.nmain) {
        item = blockIdx.x % nitem;
        t_lo = blockIdx.x / nitem;
        t_step = a.nmain;
        const int nt = min(ntile, a.nmain * a.main_len);
        nmy = nt > t_lo ? (nt - t_lo + t_step - 1) / t_step : 0;
    } else {
        const int id = blockIdx.x - nitem * a.nmain;
        item = id % nitem;
        t_lo = a.nmain * a.main_len + id / nitem;
        t_step = a.ntail;
        nmy = ntile > t_lo ? (ntile - t_lo + t_step - 1) / t_step : 0;
    }
    if (nmy <= 0) return;
    const int st = item % nstep, otile = (item / nstep) % a.otiles, wg = item / (nstep * a.otiles);
    const int jp = a.jp_lo + st / s.K, k = st % s.K;
    const int o_base = otile * NT + wave * 64;
    const bool mma_wave = o_base < s.og;

    f32x16 acc[OB][CB];
#pragma unroll
    for (int ob = 0; ob < OB; ob++)
#pragma unroll
        for (int cb = 0; cb < CB; cb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[ob][cb][r] = 0.f;

    // --- column tiles: thread = (position, 16-byte vector) of each of the two tiles
    static_assert(NCH == 2, "the two tiles of a step are named variables below");
    const int ipos = tid >> 3, ivec = tid & 7;
    const long chunk0 = (long)wg * s.nchunk + jp * NCH;
    const uint4 *const colp0 = reinterpret_cast<const uint4 *>(a.col) + ((chunk0 * s.K + k) * a.mpad + ipos) * (BKC / VEC) + ivec;
    const uint4 *const colp1 = colp0 + (long)s.K * a.mpad * (BKC / VEC);
    // (past the end of the piece the last tile is requested again: the same loads in every iteration, no branches
    // around them, so that the values stay in registers and the compiler's waits count)
    // column tiles in flight: the odd tile (crO) and the even tile (crE) after the one on the matrix cores; a pair of
    // registers is refilled, for the tile three steps on, as soon as it has been written to LDS: two whole steps for
    // a tile to arrive from device memory
    uint4 crO0, crO1, crE0, crE1;
    auto col_row0 = [&](int i) { return (long)(t_lo + min(i, nmy - 1) * t_step) * MT * (BKC / VEC); };
    // this thread's vector of tile `t` (buffer * NCH + chunk of the step) into LDS
    unsigned char *const st_p = F32 ? s_tile + (ivec * VEC) * TRS + ipos * 4 : s_tile + ipos * TRS + ivec * 16;
    auto put = [&](int t, const uint4 &v) {
        if constexpr (F32) {
            *reinterpret_cast<unsigned *>(st_p + (t * TROWS + 0) * TRS) = v.x;
            *reinterpret_cast<unsigned *>(st_p + (t * TROWS + 1) * TRS) = v.y;
            *reinterpret_cast<unsigned *>(st_p + (t * TROWS + 2) * TRS) = v.z;
            *reinterpret_cast<unsigned *>(st_p + (t * TROWS + 3) * TRS) = v.w;
        } else {
            *reinterpret_cast<uint4 *>(st_p + t * TROWS * TRS) = v;
        }
    };

    // --- gW block += gout[o, pos] * tile[pos, c]; gout fragments straight from the packed copy
    const int OBT = (s.og + 63) / 64 * 2;
    const int ntp = (s.M + kWMT - 1) / kWMT;     // tiles of the packed copy (kWMT positions each)
    // (a wavefront without output channels reads the first one's fragments in the prologue, and none after that)
    const uint4 *gp4 = reinterpret_cast<const uint4 *>(a.goutp) + (((long)wg * ntp * OBT + (mma_wave ? o_base >> 5 : 0)) * NKGP) * 64 + lane;
    auto gfrag_p = [&](int i) {     // fragment (k-group 0, row block 0) of tile i of this piece
        const long t64 = t_lo + (long)min(i, nmy - 1) * t_step;
        const long tp = t64 / (kWMT / MT);
        const int kgp = (int)(t64 % (kWMT / MT)) * NKG;
        return gp4 + ((tp * OBT) * NKGP + kgp) * 64;
    };
    // the fragments of LA tiles in flight (two: even / odd iterations); a slot is refilled, for the tile LA steps on,
    // as soon as the matrix cores have taken it
    uint4 ldA[2 * NKG], ldB[LA == 2 ? 2 * NKG : 1];
    typedef short v4s __attribute__((ext_vector_type(4)));
    const int l16 = lane & 15, g16 = lane >> 4;
    // this lane's part of the operand reads.  bfloat16, transposing: position (g16 >> 1) * 8 + (l16 >> 2), channel
    // (g16 & 1) * 16 + (l16 & 3) * 4; float: channel lane % 32, positions 4 * (lane / 32) ..
    const unsigned char *const rd_p = F32 ? s_tile + (lane & 31) * TRS + (lane >> 5) * 16
                                          : s_tile + ((g16 >> 1) * 8 + (l16 >> 2)) * TRS + ((g16 & 1) * 16 + (l16 & 3) * 4) * 2;

    {
        const uint4 *g0 = gfrag_p(0), *g1 = gfrag_p(1);
#pragma unroll
        for (int kg = 0; kg < NKG; kg++)
#pragma unroll
            for (int ob = 0; ob < OB; ob++) ldA[kg * 2 + ob] = g0[(ob * NKGP + kg) * 64];
        if constexpr (LA == 2) {
#pragma unroll
            for (int kg = 0; kg < NKG; kg++)
#pragma unroll
                for (int ob = 0; ob < OB; ob++) ldB[kg * 2 + ob] = g1[(ob * NKGP + kg) * 64];
        }
        const long r0 = col_row0(0), r1 = col_row0(1), r2 = col_row0(2);
        crE0 = ld_stream16(colp0 + r0);
        crE1 = ld_stream16(colp1 + r0);
        crO0 = ld_stream16(colp0 + r1);
        crO1 = ld_stream16(colp1 + r1);
        put(0, crE0);
        put(1, crE1);
        crE0 = ld_stream16(colp0 + r2);
        crE1 = ld_stream16(colp1 + r2);
    }
    lds_only_barrier();
    // Wavefronts without output channels (weight groups of fewer than 512) only move the column tiles.  Each role has
    // a loop of its own: a wait that served both would have to assume the fewer loads in flight.
    auto run = [&](auto mma_c) {
        constexpr bool MMA = decltype(mma_c)::value;
        auto step = [&](int it, uint4(&ld)[2 * NKG], uint4 &cr0, uint4 &cr1) {
            const int dbuf = it & 1;
            if constexpr (MMA) {
                const uint4 *gn = gfrag_p(it + LA);
#pragma unroll
                for (int kg = 0; kg < NKG; kg++) {
                    uint4 bf[CB];
                    if constexpr (F32) {
#pragma unroll
                        for (int cb = 0; cb < CB; cb++)
                            bf[cb] = *reinterpret_cast<const uint4 *>(rd_p + ((dbuf * NCH + cb) * TROWS) * TRS + kg * 32);
                    } else {
                        // ds_read_b64_tr_b16, as in tiled_bwd_weight_dma_kernel: two loads make the 8 positions of an
                        // operand vector
#pragma unroll
                        for (int cb = 0; cb < CB; cb++) {
                            const unsigned char *ap = rd_p + ((dbuf * NCH + (cb >> 1)) * MT + kg * 16) * TRS + (cb & 1) * 64;
                            const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)ap);
                            const v4s hi =
                                __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)(ap + 4 * TRS));
                            const uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
                            bf[cb] = make_uint4(lo2.x, lo2.y, hi2.x, hi2.y);
                        }
                    }
#pragma unroll
                    for (int ob = 0; ob < OB; ob++)
#pragma unroll
                        for (int cb = 0; cb < CB; cb++) mma_kgroup<T, false>(acc[ob][cb], ld[kg * 2 + ob], bf[cb]);
#pragma unroll
                    for (int ob = 0; ob < OB; ob++) ld[kg * 2 + ob] = gn[(ob * NKGP + kg) * 64];
                    // (the requests stay behind the matrix instructions of their k-group)
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // (the other buffer was last read in the iteration before, which every wavefront has left)
            put((dbuf ^ 1) * NCH, cr0);
            put((dbuf ^ 1) * NCH + 1, cr1);
            const long r3 = col_row0(it + 3);
            cr0 = ld_stream16(colp0 + r3);
            cr1 = ld_stream16(colp1 + r3);
            lds_only_barrier();
        };
        // pairs of steps, then the odd one out: no branch inside the loop (see above)
        int it = 0;
        if constexpr (LA == 2) {
            for (; it + 1 < nmy; it += 2) {
                step(it, ldA, crO0, crO1);
                step(it + 1, ldB, crE0, crE1);
            }
        } else {
            for (; it + 1 < nmy; it += 2) {
                step(it, ldA, crO0, crO1);
                step(it + 1, ldA, crE0, crE1);
            }
        }
        if (it < nmy) step(it, ldA, crO0, crO1);
    };
    if (mma_wave) run(std::true_type{});
    else run(std::false_type{});

    if (mma_wave) {
#pragma unroll
        for (int ob = 0; ob < OB; ob++)
#pragma unroll
            for (int cb = 0; cb < CB; cb++) {
                const int stw = (jp * NCH + cb / CPB) * s.K + k;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int ol = o_base + ob * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (ol < s.og)
                        atomicAdd(a.gwacc + (((long)wg * s.nchunk * s.K + stw) * s.og + ol) * BKC + (cb % CPB) * 32 + (lane & 31),
                                  acc[ob][cb][r]);
                }
            }
    }
}

// ============================================================ kernel 2c
// The same product for float problems on the bfloat16 matrix instruction, with float32's accuracy: every float is
// taken apart into THREE bfloat16 terms, v = h + m + l exactly (8 + 8 + 8 significant bits), and of the nine partial
// products of a pair the six largest are summed,
//     h h' + m h'   |   h m' + m m'   |   l h' + h l'
// three v_mfma_f32_32x32x16_bf16 per 8 positions (each 16-deep reduction holds two partial products of 8 pairs)
// against four v_mfma_f32_32x32x2_f32 of twice their length: 3/8 of the matrix-pipe time.  What is dropped
// (m l' + l m' + l l') is below 2^-25 of a product, under float32's own rounding.  The first instruction carries the
// leading term and adds into one accumulator, the two others (terms of at most 2^-8 of it) into a second one, and
// the two are added at the end: the large sum is rounded once per 8 positions instead of four times.
//
// One workgroup = one tap and four channel chunks (128 columns), 256 output channels (8 wavefronts x 32 rows),
// looping over its piece of the 64-position tiles like tiled_bwd_weight_col_kernel.  The float columns are taken
// apart where they are stored to LDS -- three planes [position][32 channels] of bfloat16 per chunk, read with the
// transposing LDS load -- and grad_out comes from a fragment-ordered copy that holds the three terms (pack_gout3_kernel).
constexpr int kCol3Chunks = 4;
constexpr int kCol3Rows = 256;     // output channels per workgroup
constexpr size_t kCol3Lds = (size_t)2 * kCol3Chunks * 3 * kWDT * 64;

// v -> (h, m, l), bfloat16 bits
D2C_DEV void split3(float v, uint32_t &h, uint32_t &m, uint32_t &l)
{
    h = f32_to_bf16(v);
    const float r1 = bf16_residual(v, h << 16);
    m = f32_to_bf16(r1);
    l = f32_to_bf16(r1 - __uint_as_float(m << 16));
}

// grad_out [N][Cout][P] -> fragments of the three terms, indexed like pack_gout_kernel's (float: 16 k-groups of 8
// positions per tile of kWMT): lh[i] = (l0 l1)(l2 l3)(h0 h1)(h2 h3) of the lane's four positions, md[i] = (m0 m1)(m2 m3);
// `md` follows the `total` 16-byte entries of `lh`
__global__ void __launch_bounds__(256) pack_gout3_kernel(const float *gout, uint4 *lh, TiledShape s, int ntile, int OBT,
                                                         long total)
{
    constexpr int VEC = 4, NKGT = kWMT / (2 * VEC);
    uint2 *md = reinterpret_cast<uint2 *>(lh + total);
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int lane = (int)(i & 63);
        long r = i >> 6;
        const int kg = (int)(r % NKGT); r /= NKGT;
        const int ob = (int)(r % OBT); r /= OBT;
        const int tile = (int)(r % ntile);
        const int wg = (int)(r / ntile);
        const int ol = ob * 32 + (lane & 31);
        const long m0 = (long)tile * kWMT + (2 * kg + (lane >> 5)) * VEC;
        uint32_t h[VEC], m[VEC], l[VEC];
#pragma unroll
        for (int q = 0; q < VEC; q++) {
            const long mm = m0 + q;
            float v = 0.f;
            if (ol < s.og && mm < s.M) {
                const int b = (int)(mm / s.P), pp = (int)(mm - (long)b * s.P);
                v = gout[((long)b * s.Cout + wg * s.og + ol) * s.P + pp];
            }
            split3(v, h[q], m[q], l[q]);
        }
        lh[i] = make_uint4(l[0] | (l[1] << 16), l[2] | (l[3] << 16), h[0] | (h[1] << 16), h[2] | (h[3] << 16));
        md[i] = make_uint2(m[0] | (m[1] << 16), m[2] | (m[3] << 16));
    }
}

struct BwdWeightCol3Args {
    TiledShape s;
    const void *col;     // [chunk][tap][mpad][32] float
    const uint4 *lh;     // grad_out fragments, see pack_gout3_kernel
    const uint2 *md;
    float *gwacc;        // as in BwdWeightArgs
    long mpad;           // rows per (chunk, tap) of `col`: whole 64-position tiles
    int otiles, nmain, main_len, ntail, tail_len;   // as in BwdWeightArgs (output tiles of kCol3Rows channels)
};

__global__ void __launch_bounds__(kThreads) tiled_bwd_weight_col3_kernel(BwdWeightCol3Args a)
{
    constexpr int MT = kWDT, NCH = kCol3Chunks, CB = NCH, NT = kCol3Rows;
    constexpr int NKG = MT / 8;                // k-groups (8 positions) per tile
    constexpr int NKGP = kWMT / 8;             // ... per tile of the packed grad_out copy
    constexpr int PLANE = MT * 64;             // bytes of one term of one chunk: [position][32 channels] bfloat16
    constexpr int LAK = 4;                     // k-groups of grad_out fragments in flight
    static_assert(MT * 8 == kThreads, "one (position, vector) item per thread and column tile");
    extern __shared__ __align__(16) unsigned char s_tile[];   // [2 buffers][NCH][3 terms][PLANE]

    const TiledShape &s = a.s;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ntile = (s.M + MT - 1) / MT;
    const int nstep = (s.nchunk / NCH) * s.K;
    const int nitem = s.groups * a.otiles * nstep;
    int item, t_lo, nmy, t_step;
    if ((int)blockIdx.x < nitem * a.nmain) {
        item = blockIdx.x % nitem;
        t_lo = blockIdx.x / nitem;
        t_step = a.nmain;
        const int nt = min(ntile, a.nmain * a.main_len);
        nmy = nt > t_lo ? (nt - t_lo + t_step - 1) / t_step : 0;
    } else {
        const int id = blockIdx.x - nitem * a.nmain;
        item = id % nitem;
        t_lo = a.nmain * a.main_len + id / nitem;
        t_step = a.ntail;
        nmy = ntile > t_lo ? (ntile - t_lo + t_step - 1) / t_step : 0;
    }
    if (nmy <= 0) return;
    const int st = item % nstep, otile = (item / nstep) % a.otiles, wg = item / (nstep * a.otiles);
    const int jq = st / s.K, k = st % s.K;
    const int o_base = otile * NT + wave * 32;
    const bool mma_wave = o_base < s.og;

    f32x16 big[CB], small[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++)
#pragma unroll
        for (int r = 0; r < 16; r++) big[cb][r] = small[cb][r] = 0.f;

    // --- column tiles: thread = (position, 16-byte vector of 4 channels) of each of the four tiles of a step
    const int ipos = tid >> 3, ivec = tid & 7;
    const long chunk0 = (long)wg * s.nchunk + jq * NCH;
    const long cstride = (long)s.K * a.mpad * 8;      // 16-byte vectors from one chunk to the next
    const uint4 *const colp = reinterpret_cast<const uint4 *>(a.col) + ((chunk0 * s.K + k) * a.mpad + ipos) * 8 + ivec;
    // (past the end of the piece the last tile is requested again: the same loads in every iteration)
    auto col_row0 = [&](int i) { return (long)(t_lo + min(i, nmy - 1) * t_step) * MT * 8; };
    uint4 cr[NCH];       // the tile after the one on the matrix cores, requested a whole step before it is stored
    unsigned char *const st_p = s_tile + ipos * 64 + ivec * 8;
    auto put = [&](int buf, int c, const uint4 &v) {
        uint32_t h[4], m[4], l[4];
        split3(__uint_as_float(v.x), h[0], m[0], l[0]);
        split3(__uint_as_float(v.y), h[1], m[1], l[1]);
        split3(__uint_as_float(v.z), h[2], m[2], l[2]);
        split3(__uint_as_float(v.w), h[3], m[3], l[3]);
        unsigned char *d = st_p + ((buf * NCH + c) * 3) * PLANE;
        *reinterpret_cast<uint2 *>(d) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
        *reinterpret_cast<uint2 *>(d + PLANE) = make_uint2(m[0] | (m[1] << 16), m[2] | (m[3] << 16));
        *reinterpret_cast<uint2 *>(d + 2 * PLANE) = make_uint2(l[0] | (l[1] << 16), l[2] | (l[3] << 16));
    };

    // --- grad_out fragments of this wavefront's 32 rows
    const int OBT = (s.og + 63) / 64 * 2;
    const int ntp = (s.M + kWMT - 1) / kWMT;
    const long f0 = (((long)wg * ntp * OBT + (mma_wave ? o_base >> 5 : 0)) * NKGP) * 64 + lane;
    auto frag_at = [&](int i, int kg) {       // index of k-group kg of tile i of this piece
        const long t64 = t_lo + (long)min(i, nmy - 1) * t_step;
        const long tp = t64 / (kWMT / MT);
        const int kgp = (int)(t64 % (kWMT / MT)) * NKG + kg;
        return f0 + ((tp * OBT) * NKGP + kgp) * 64;
    };
    uint4 alh[LAK];
    uint2 amd[LAK];
    typedef short v4s __attribute__((ext_vector_type(4)));
    const int l16 = lane & 15, g16 = lane >> 4;
    // this lane's part of the transposing reads (ds_read_b64_tr_b16: within 16 lanes, lane l element j comes from lane
    // 4j + l/4, element l%4): it reads 4 channels of position 4 * (g16 >> 1) + (l16 >> 2) of a k-group and receives
    // channel (g16 & 1) * 16 + l16 at the four positions 4 * (g16 >> 1) ..
    const unsigned char *const rd_p = s_tile + (4 * (g16 >> 1) + (l16 >> 2)) * 64 + ((g16 & 1) * 16 + (l16 & 3) * 4) * 2;
    auto tr = [&](const unsigned char *p) {
        return __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)p));
    };

    {
#pragma unroll
        for (int q = 0; q < LAK; q++) {
            const long f = frag_at(0, q);
            alh[q] = a.lh[f];
            amd[q] = a.md[f];
        }
        const long r0 = col_row0(0), r1 = col_row0(1);
#pragma unroll
        for (int c = 0; c < NCH; c++) cr[c] = ld_stream16(colp + c * cstride + r0);
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            put(0, c, cr[c]);
            cr[c] = ld_stream16(colp + c * cstride + r1);
        }
    }
    lds_only_barrier();
    auto run = [&](auto mma_c) {
        constexpr bool MMA = decltype(mma_c)::value;
        for (int it = 0; it < nmy; it++) {
            const int dbuf = it & 1;
            if constexpr (MMA) {
#pragma unroll
                for (int kg = 0; kg < NKG; kg++) {
                    const int q = kg % LAK;
                    const uint4 a_lh = alh[q];
                    const uint4 a_hm = make_uint4(alh[q].z, alh[q].w, amd[q].x, amd[q].y);
#pragma unroll
                    for (int cb = 0; cb < CB; cb++) {
                        const unsigned char *bp = rd_p + ((dbuf * NCH + cb) * 3) * PLANE + kg * 8 * 64;
                        const uint2 bh = tr(bp), bm = tr(bp + PLANE), bl = tr(bp + 2 * PLANE);
                        const uint4 b_hh = make_uint4(bh.x, bh.y, bh.x, bh.y), b_mm = make_uint4(bm.x, bm.y, bm.x, bm.y);
                        const uint4 b_hl = make_uint4(bh.x, bh.y, bl.x, bl.y);
                        big[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a_hm),
                                                                          __builtin_bit_cast(bf16x8_t, b_hh), big[cb], 0, 0, 0);
                        small[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a_hm),
                                                                            __builtin_bit_cast(bf16x8_t, b_mm), small[cb], 0, 0, 0);
                        small[cb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a_lh),
                                                                            __builtin_bit_cast(bf16x8_t, b_hl), small[cb], 0, 0, 0);
                    }
                    // the slot is refilled with the fragment LAK k-groups on (of the next tile, past this one's last)
                    const long f = kg + LAK < NKG ? frag_at(it, kg + LAK) : frag_at(it + 1, kg + LAK - NKG);
                    alh[q] = a.lh[f];
                    amd[q] = a.md[f];
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // (the other buffer was last read in the iteration before, which every wavefront has left)
            const long r2 = col_row0(it + 2);
#pragma unroll
            for (int c = 0; c < NCH; c++) {
                put(dbuf ^ 1, c, cr[c]);
                cr[c] = ld_stream16(colp + c * cstride + r2);
            }
            lds_only_barrier();
        }
    };
    if (mma_wave) run(std::true_type{});
    else run(std::false_type{});

    if (mma_wave) {
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            const int stw = (jq * NCH + cb) * s.K + k;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int ol = o_base + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (ol < s.og)
                    atomicAdd(a.gwacc + (((long)wg * s.nchunk * s.K + stw) * s.og + ol) * 32 + (lane & 31),
                              big[cb][r] + small[cb][r]);
            }
        }
    }
}

template <typename T, int NC> constexpr size_t bwd_weight_dma_lds()
{
    constexpr int BKC = 8 * Elem<T>::VEC;
    return (size_t)2 * kWDT * NC * 128 + (size_t)2 * BKC * (kWDT * sizeof(T) + 16) + (size_t)3 * 10 * kWDT * 4;
}

// ============================================================ small kernels
// W[o][c][k] -> wt[wg][step][cc][oo] for oo in [o0, o0 + ogn), padded with zeros to ogk; steps in the
// order of the data kernel (offset group, tap, chunk of the group)
template <typename T, bool SPLIT>
__global__ void __launch_bounds__(256) pack_weight_bwd_kernel(const T *w, T *wt, TiledShape s, int ogk, int o0,
                                                              int ogn, long total)
{
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC;
    // one 16-byte vector of VEC consecutive output channels (the reduction of the grad-column product) per thread
    for (long v = (long)blockIdx.x * blockDim.x + threadIdx.x; v < total / VEC; v += (long)gridDim.x * blockDim.x) {
        const long i = v * VEC;
        const int oo = (int)(i % ogk);
        long r = i / ogk;
        const int cc = (int)(r % BKC); r /= BKC;
        const int st = (int)(r % (s.K * s.nchunk));
        const int wg = (int)(r / (s.K * s.nchunk));
        const int cpc = s.cpg / BKC;   // same step order as tiled_bwd_data_kernel
        const int k = (st / cpc) % s.K, j = (st / (cpc * s.K)) * cpc + st % cpc;
        alignas(16) T tmp[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++)
            tmp[e] = oo + e < ogn ? w[((long)(wg * s.og + o0 + oo + e) * s.cg + j * BKC + cc) * s.K + k] : (T)0;
        *reinterpret_cast<uint4 *>(wt + i) = operand_vec<T, SPLIT>(tmp);
    }
}

// W[o][c][k] (float) -> wt[wg][step][cc][high halves of 128 nbp output channels | their low halves] in bfloat16, for
// tiled_bwd_col32f_kernel; channels past ogn are zeros; steps in the order of the data kernel.  One thread = 8
// consecutive output channels of one plane.
__global__ void __launch_bounds__(256) pack_weight_bwd_planes_kernel(const float *w, bf16_t *wt, TiledShape s, int nbp,
                                                                     int o0, int ogn, long total)
{
    constexpr int BKC = 32;
    const int pw = 128 * nbp;            // plane width
    for (long v = (long)blockIdx.x * blockDim.x + threadIdx.x; v < total / 8; v += (long)gridDim.x * blockDim.x) {
        const long i = v * 8;
        const int op = (int)(i % (2 * pw)), plane = op / pw, oo = op - plane * pw;
        long r = i / (2 * pw);
        const int cc = (int)(r % BKC); r /= BKC;
        const int st = (int)(r % (s.K * s.nchunk));
        const int wg = (int)(r / (s.K * s.nchunk));
        const int cpc = s.cpg / BKC;
        const int k = (st / cpc) % s.K, j = (st / (cpc * s.K)) * cpc + st % cpc;
        float e[8];
#pragma unroll
        for (int q = 0; q < 8; q++)
            e[q] = oo + q < ogn ? w[((long)(wg * s.og + o0 + oo + q) * s.cg + j * BKC + cc) * s.K + k] : 0.f;
        uint32_t out[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t h = pack_bf16x2(e[2 * q], e[2 * q + 1]);
            out[q] = plane == 0 ? h
                                : pack_bf16x2(bf16_residual(e[2 * q], h << 16), bf16_residual(e[2 * q + 1], h & 0xffff0000u));
        }
        *reinterpret_cast<uint4 *>(wt + i) = make_uint4(out[0], out[1], out[2], out[3]);
    }
}

// The same re-layout through LDS (needs a 16-byte aligned W): a workgroup takes a block of output channels
// as wide as the padding unit of ogk (128 bytes of wt) and kPackCh channels of a chunk, whose weights are
// runs of kPackCh * K consecutive elements in W, and writes 16-byte vectors of consecutive output channels.
constexpr int kPackCh = 8;
template <typename T, bool SPLIT>
__global__ void __launch_bounds__(256) pack_weight_bwd_lds_kernel(const T *w, T *wt, TiledShape s, int ogk, int o0,
                                                                  int ogn)
{
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC, R = 128 / (int)sizeof(T), CB = BKC / kPackCh;
    extern __shared__ __align__(16) unsigned char smem[];
    int b = blockIdx.x;
    const int cb = b % CB; b /= CB;
    const int obk = b % (ogk / R); b /= ogk / R;
    const int j = b % s.nchunk;
    const int wg = b / s.nchunk;
    const int run = kPackCh * s.K;                   // elements of a row
    const int rs = run * (int)sizeof(T) + 4;         // LDS row stride in bytes (an odd number of banks)
    const int vpr = run * (int)sizeof(T) / 16;
    for (int i = threadIdx.x; i < R * vpr; i += 256) {
        const int r = i / vpr, v = i - r * vpr;
        const int oo = obk * R + r;
        uint4 val = make_uint4(0, 0, 0, 0);
        if (oo < ogn)
            val = *reinterpret_cast<const uint4 *>(
                reinterpret_cast<const char *>(w + ((long)(wg * s.og + o0 + oo) * s.cg + j * BKC + cb * kPackCh) * s.K) +
                (size_t)v * 16);
        unsigned *d = reinterpret_cast<unsigned *>(smem + r * rs + v * 16);
        d[0] = val.x; d[1] = val.y; d[2] = val.z; d[3] = val.w;
    }
    __syncthreads();
    const int cpc = s.cpg / BKC;   // same step order as tiled_bwd_data_kernel
    for (int i = threadIdx.x; i < s.K * kPackCh * (R / VEC); i += 256) {
        const int ov = i % (R / VEC), q = i / (R / VEC);
        const int cc = q % kPackCh, k = q / kPackCh;
        alignas(16) T tmp[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) tmp[e] = reinterpret_cast<const T *>(smem + (ov * VEC + e) * rs)[cc * s.K + k];
        const int st = ((j / cpc) * s.K + k) * cpc + j % cpc;
        const long di = (((long)wg * s.K * s.nchunk + st) * BKC + cb * kPackCh + cc) * ogk + obk * R + ov * VEC;
        *reinterpret_cast<uint4 *>(wt + di) = operand_vec<T, SPLIT>(tmp);
    }
}

// fp32 channels-last accumulator [N][vol][C] -> grad_input [N][C][vol] of type T
template <typename T>
__global__ void __launch_bounds__(256) unpack_grad_input_kernel(const float *gxcl, T *gx, int C, int vol)
{
    __shared__ float tile[32][33];
    const int b = blockIdx.z, v0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const float *ib = gxcl + (long)b * C * vol;
    T *ob = gx + (long)b * C * vol;
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        const int v = v0 + ty + i, c = c0 + tx;
        if (c < C && v < vol) tile[ty + i][tx] = ib[(long)v * C + c];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        const int c = c0 + ty + i, v = v0 + tx;
        if (c < C && v < vol) ob[(long)c * vol + v] = f32_to_elem<T>(tile[tx][ty + i]);
    }
}

// The same for bfloat16 with 16-byte accesses on both sides: 64 x 64 element tiles; needs vol and C to be
// multiples of 8 and a 16-byte aligned grad_input.
__global__ void __launch_bounds__(256) unpack_grad_input_bf16_kernel(const float *gxcl, bf16_t *gx, int C, int vol)
{
    constexpr int RS = 66;                             // LDS row stride in elements (33 words)
    __shared__ bf16_t tile[64 * RS];                   // [c][v]
    const int b = blockIdx.z, v0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
    const float *ib = gxcl + (long)b * C * vol;
    bf16_t *ob = gx + (long)b * C * vol;
    for (int i = threadIdx.x; i < 1024; i += 256) {    // 64 positions x 16 vectors of 4 channels
        const int v = v0 + i / 16, c = c0 + (i % 16) * 4;
        if (c < C && v < vol) {
            const float4 q = *reinterpret_cast<const float4 *>(ib + (long)v * C + c);
            bf16_t *t = tile + ((i % 16) * 4) * RS + i / 16;
            t[0] = f32_to_bf16(q.x); t[RS] = f32_to_bf16(q.y); t[2 * RS] = f32_to_bf16(q.z); t[3 * RS] = f32_to_bf16(q.w);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 512; i += 256) {     // 64 channels x 8 vectors of 8 positions
        const int c = c0 + i / 8, v = v0 + (i % 8) * 8;
        if (c < C && v < vol) {
            const unsigned *t = reinterpret_cast<const unsigned *>(tile + (i / 8) * RS + (i % 8) * 8);
            *reinterpret_cast<uint4 *>(ob + (long)c * vol + v) = make_uint4(t[0], t[1], t[2], t[3]);
        }
    }
}

// fp32 accumulator [group][chunk*K + tap][og][BKC] -> grad_weight [Cout][cg][K] of type T
template <typename T>
__global__ void __launch_bounds__(256) cvt_grad_weight_kernel(const float *src, T *dst, TiledShape s, long n)
{
    constexpr int BKC = 8 * Elem<T>::VEC;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int k = (int)(i % s.K);
        const int cl = (int)((i / s.K) % s.cg);
        const int o = (int)(i / ((long)s.K * s.cg));
        const int wg = o / s.og, ol = o - wg * s.og, j = cl / BKC, cc = cl - j * BKC;
        dst[i] = f32_to_elem<T>(src[(((long)wg * s.nchunk * s.K + j * s.K + k) * s.og + ol) * BKC + cc]);
    }
}

// The same through LDS (needs a 16-byte aligned grad_weight): a workgroup takes kCvtRows output channels of one
// channel chunk; per tap their accumulator rows are one contiguous piece, and in grad_weight they are runs
// of BKC * K consecutive elements.
constexpr int kCvtRows = 4;
template <typename T>
__global__ void __launch_bounds__(256) cvt_grad_weight_lds_kernel(const float *src, T *dst, TiledShape s)
{
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC, R = kCvtRows;
    extern __shared__ __align__(16) unsigned char smem[];
    const int nrb = (s.og + R - 1) / R;
    int b = blockIdx.x;
    const int rb = b % nrb; b /= nrb;
    const int j = b % s.nchunk;
    const int wg = b / s.nchunk;
    const int run = BKC * s.K;
    const int rs = run * (int)sizeof(T) + 16;        // LDS row stride in bytes
    const int nr = min(R, s.og - rb * R);
    // accumulator [tap][row][channel] -> LDS [row][channel][tap], converted
    for (int i = threadIdx.x; i < s.K * nr * (BKC / 4); i += 256) {
        const int c4 = i % (BKC / 4), q = i / (BKC / 4);
        const int r = q % nr, k = q / nr;
        const float4 v = *reinterpret_cast<const float4 *>(
            src + (((long)wg * s.nchunk * s.K + j * s.K + k) * s.og + rb * R + r) * BKC + c4 * 4);
        T *d = reinterpret_cast<T *>(smem + r * rs) + (c4 * 4) * s.K + k;
        d[0] = f32_to_elem<T>(v.x); d[s.K] = f32_to_elem<T>(v.y);
        d[2 * s.K] = f32_to_elem<T>(v.z); d[3 * s.K] = f32_to_elem<T>(v.w);
    }
    __syncthreads();
    const int vpr = run * (int)sizeof(T) / 16;
    for (int i = threadIdx.x; i < nr * vpr; i += 256) {
        const int r = i / vpr, v = i - r * vpr;
        *reinterpret_cast<uint4 *>(reinterpret_cast<char *>(dst + ((long)(wg * s.og + rb * R + r) * s.cg + j * BKC) * s.K) +
                                   (size_t)v * 16) = *reinterpret_cast<const uint4 *>(smem + r * rs + v * 16);
    }
}

// grad_out [N][Cout][P] -> MFMA fragments for the grad-weight kernel:
//   goutp[wg][tile of kWMT positions][32-row block][k-group][lane] = 16 bytes =
//   gout[wg*og + block*32 + lane%32][positions tile*kWMT + (2*kgroup + lane/32)*VEC + 0..VEC-1]
// with positions numbered over the whole batch (m = b*P + p); rows past og and positions past N*P are zero.
template <typename T, bool SPLIT>
__global__ void __launch_bounds__(256) pack_gout_kernel(const T *gout, T *goutp, TiledShape s, int ntile, int OBT, long total,
                                                        bool vec)
{
    constexpr int VEC = Elem<T>::VEC, NKGT = kWMT / (2 * VEC);
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int lane = (int)(i & 63);
        long r = i >> 6;
        const int kg = (int)(r % NKGT); r /= NKGT;
        const int ob = (int)(r % OBT); r /= OBT;
        const int tile = (int)(r % ntile);
        const int wg = (int)(r / ntile);
        const int ol = ob * 32 + (lane & 31);
        const long m0 = (long)tile * kWMT + (2 * kg + (lane >> 5)) * VEC;
        alignas(16) T e[VEC];
        if (vec) {
            // P is a multiple of VEC: the VEC positions lie in one sample and are one aligned 16-byte piece of the row
            uint4 v = make_uint4(0, 0, 0, 0);
            if (ol < s.og && m0 < s.M) {
                const int b = (int)(m0 / s.P), p = (int)(m0 - (long)b * s.P);
                v = *reinterpret_cast<const uint4 *>(gout + ((long)b * s.Cout + wg * s.og + ol) * s.P + p);
            }
            reinterpret_cast<uint4 *>(goutp)[i] = operand_vec16<T, SPLIT>(v);
            continue;
        }
#pragma unroll
        for (int q = 0; q < VEC; q++) {
            const long m = m0 + q;
            T v = (T)0;
            if (ol < s.og && m < s.M) {
                const int b = (int)(m / s.P), p = (int)(m - (long)b * s.P);
                v = gout[((long)b * s.Cout + wg * s.og + ol) * s.P + p];
            }
            e[q] = v;
        }
        reinterpret_cast<uint4 *>(goutp)[i] = operand_vec<T, SPLIT>(e);
    }
}

// gb[o] = sum_{b,p} gout[b,o,p]   (dconv3d_gpu.cu:1329): one workgroup of 16 wavefronts per output channel
template <typename T>
__global__ void __launch_bounds__(1024) bias_grad_kernel(const T *gout, T *gb, int N, int Cout, int P)
{
    bias_grad_body<T, 1024>(gout, gb, N, Cout, P, blockIdx.x);
}

// fp32 scratch of the split data kernel -> offset / mask gradient in its storage type
__global__ void __launch_bounds__(256) aux_finish_kernel(const float *src, void *dst, int adt, long n)
{
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        st_aux(dst, i, adt, src[i]);
}

inline unsigned grid1d(long n, int cap = 8192)
{
    long g = (n + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > cap ? cap : g));
}

}  // namespace

// ------------------------------------------------------------------ host
// Output channels of a pass, padded with zero rows of the transposed weights: float to a multiple of 128 bytes of a
// tile row; bfloat16 to 128 channels, the unit of tiled_bwd_col32_kernel, which then serves every bfloat16 width
// (192 -> 192 channels on 8x30x54: backward pass 0.47 -> 0.42 ms against the 128-position kernel on 192 channels;
// 320 -> 320: 0.78 -> 0.67; 64 -> 64 unchanged).
int d2c_bwd_ogk(int og, int dtype) { const int rw = dtype == D2C_BF16 ? 128 : 32; return (og + rw - 1) / rw * rw; }

// Output channels one pass of the data kernel reduces over: 32 k-groups of the
// stationary operand fit the register file (512 bf16 / 256 float channels).
int d2c_bwd_pass_channels(int dtype) { return 32 * (dtype == D2C_BF16 ? 16 : 8); }

bool d2c_tiled_bwd_data_supported(const TiledShape &s, int)
{
    return s.cg % s.cpg == 0;  // an offset group must lie inside one weight group
}

bool d2c_tiled_bwd_weight_supported(const TiledShape &, int)
{
    return true;   // the packed grad_out copy takes care of tiles that straddle samples or end early
}

// One pass reduces over all output channels of a weight group (the list-based grad_input needs that).
bool d2c_tiled_bwd_single_pass(const TiledShape &s, int dtype) { return s.og <= d2c_bwd_pass_channels(dtype); }

// Workgroups per position tile of the data kernel: 1 when the tiles alone fill the chip.
int d2c_bwd_data_split(const TiledShape &s, int dtype)
{
    const int mt = dtype == D2C_BF16 ? 128 : 256;
    const long wgs = (long)((s.M + mt - 1) / mt) * s.groups;
    if (wgs >= 128) return 1;
    const int S = s.nchunk * s.K;
    const long want = (256 + wgs - 1) / wgs;
    return (int)(want < S ? want : S);
}

template <typename T>
int d2c_tiled_bwd_data_launch(const TiledShape &s, const void *gout, const void *xcl, const void *off,
                              const void *mask, const void *w, void *wt, float *gxcl, void *gcolbuf, void *goff,
                              void *gmask, float *auxacc, hipStream_t st, int phase, int g_lo, int g_n,
                              bool weights_packed)
{
    // Weight groups wider than one pass get their grad-column rows from the product-only kernels too: the first pass
    // writes the rows, every later one adds to them.
    // phase: 1 = the weight re-layout (and the clears), 2 = the kernel, 3 = both.  g_n > 0 (grad-column product on
    // tiled_bwd_col32_kernel only, see d2c_bwd_sliceable): the rows of the offset groups [g_lo, g_lo + g_n) only,
    // `gcolbuf` pointing where chunk 0 would start.
    constexpr int BKC = 8 * Elem<T>::VEC;
    const int omax = d2c_bwd_pass_channels(Elem<T>::DT);
    const bool sliced = g_n > 0;
    int nsplit = auxacc ? d2c_bwd_data_split(s, Elem<T>::DT) : 1;
    if (gcolbuf && !gxcl && !goff && !gmask) {
        // Only the grad-column product is wanted: every (tile, step) writes its own part of the result, so the
        // steps can be cut into ranges at no cost but the reload of the stationary operand.  Workgroups are
        // dispatched range-major (blockIdx.z slowest), which keeps those running at one time on the same weight
        // tiles; the cut is the one whose last round of workgroups is fullest.
        const int ncu = d2c_num_cus();
        if (ncu <= 0) return D2C_ERR_LAUNCH;
        // (the 256-position kernel of bfloat16 problems walks half-steps; reloading its stationary operand costs
        // about two of them)
        const int og1 = s.og < omax ? s.og : omax;     // (the first pass; sized for it)
        const bool c32 = bwd_col32_ok(d2c_bwd_ogk(og1, Elem<T>::DT), og1, Elem<T>::DT);
        const bool c32f = bwd_col32f_ok(og1, Elem<T>::DT, s.f32split != 0);
        const int MT = c32 ? kCol32MT : 32 * (8 / (BKC / 32));
        const long items = (long)((s.M + MT - 1) / MT) * s.groups;
        const int S = (sliced ? g_n * (s.cpg / BKC) : s.nchunk) * s.K * (c32 ? 2 : 1), reload = c32 || c32f ? 2 : 1;
        long best = ((items + ncu - 1) / ncu) * (S + reload);
        nsplit = 1;
        for (int k = 2; k <= 16 && k <= S; k++) {
            const long cost = ((items * k + ncu - 1) / ncu) * ((S + k - 1) / k + reload);
            if (cost < best) { best = cost; nsplit = k; }
        }
    }
    const long n_mask = (long)s.N * s.G * s.K * s.P, n_off = n_mask * s.nd;
    float *auxoff = nullptr, *auxmask = nullptr;
    if ((nsplit > 1 || s.og > omax) && (goff || gmask) && auxacc) {
        auxoff = auxacc;
        auxmask = auxacc + n_off;
        if (phase & 1) {
            D2cProfScope prof(D2C_PROF_PACK, st);
            d2c_fill_zero(auxacc, (size_t)(n_off + n_mask) * sizeof(float), st);
        }
    }
    if (gxcl && (phase & 1)) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        d2c_fill_zero(gxcl, (size_t)s.N * s.vol * s.Cin * sizeof(float), st);
    }
    // Weight groups wider than one pass can hold are reduced in several passes; every
    // quantity downstream of the grad-column product is linear in it, so the passes add up.
    for (int o0 = 0; o0 < s.og; o0 += omax) {
        const int ogn = s.og - o0 < omax ? s.og - o0 : omax;
        int ogk = d2c_bwd_ogk(ogn, Elem<T>::DT);
        // (a later pass of the grad-column product on its own: padded to what tiled_bwd_col32_kernel takes, which
        // the buffer of the first pass has room for)
        const bool only_col = gcolbuf && !gxcl && !goff && !gmask;
        if (only_col && o0 > 0 && bwd_col32_ok((ogk + 127) / 128 * 128, ogn, Elem<T>::DT)) ogk = (ogk + 127) / 128 * 128;
        const long total = (long)s.groups * s.K * s.nchunk * BKC * ogk;
        // two-term bfloat16 operands for this pass (float problems): wherever the description asks for them, and for
        // the grad-column product on its own by default (f32split == 2)
        const bool col_only = gcolbuf && !gxcl && !goff && !gmask && bwd_col_lds<T>(ogk, false) <= 160 * 1024;
        const bool split_pass = sizeof(T) == 4 && (s.f32split == 1 || (s.f32split == 2 && col_only));
        // (weights_packed: `wt` already holds them, from an earlier call on the same weights)
        const bool planes = col_only && bwd_col32f_ok(ogn, Elem<T>::DT, split_pass);
        if ((phase & 1) && !weights_packed && planes) {
            if constexpr (sizeof(T) == 4) {
                D2cProfScope prof(D2C_PROF_PACK, st);
                const int nbp = ogn > 128 ? 2 : 1;
                const long tot = (long)s.groups * s.K * s.nchunk * BKC * 2 * 128 * nbp;
                hipLaunchKernelGGL(pack_weight_bwd_planes_kernel, dim3(grid1d(tot / 8)), dim3(256), 0, st, (const float *)w,
                                   (bf16_t *)wt, s, nbp, o0, ogn, tot);
            }
        } else if ((phase & 1) && !weights_packed) {
            D2cProfScope prof(D2C_PROF_PACK, st);
            constexpr int R = 128 / (int)sizeof(T);
            constexpr bool SPT = sizeof(T) == 4;       // (split operands exist for float problems only)
            const bool split = SPT && split_pass;
            auto k_lds = split ? &pack_weight_bwd_lds_kernel<T, SPT> : &pack_weight_bwd_lds_kernel<T, false>;
            auto k_elem = split ? &pack_weight_bwd_kernel<T, SPT> : &pack_weight_bwd_kernel<T, false>;
            const size_t lds = (size_t)R * ((size_t)kPackCh * s.K * sizeof(T) + 4);
            if (lds <= 64 * 1024 && reinterpret_cast<uintptr_t>(w) % 16 == 0)
                hipLaunchKernelGGL(k_lds, dim3((unsigned)(s.groups * s.nchunk * (ogk / R) * (BKC / kPackCh))), dim3(256), lds,
                                   st, (const T *)w, (T *)wt, s, ogk, o0, ogn);
            else
                hipLaunchKernelGGL(k_elem, dim3(grid1d(total)), dim3(256), 0, st, (const T *)w, (T *)wt, s, ogk, o0, ogn,
                                   total);
        }
        if (int rc = d2c_check_launch("pack_weight_bwd_kernel")) return rc;
        if (!(phase & 2)) continue;
        const int cpc2 = 2 * (s.cpg / BKC);
        BwdDataArgs a{s, gout, xcl, off, mask, wt, gxcl, gcolbuf, goff, gmask, ogk, o0, ogn, o0 > 0 ? 1 : 0,
                      auxoff, auxmask, sliced ? g_lo * cpc2 * s.K : 0, sliced ? (g_lo + g_n) * cpc2 * s.K : 0};
        const int nkg = ogk / (2 * Elem<T>::VEC);
        int rc;
        if (col_only && bwd_col32_ok(ogk, ogn, Elem<T>::DT)) {
            rc = launch_bwd_col32(a, nsplit, st);
        } else if (planes) {
            rc = launch_bwd_col32f(a, nsplit, st);
        } else if (sliced) {
            d2c_set_error("grad-column product: slices are made by tiled_bwd_col32_kernel only");
            return D2C_ERR_LAUNCH;
        } else if (col_only) {
            if (nkg <= 4) rc = launch_bwd_col<T, 4>(a, nsplit, st, split_pass);
            else if (nkg <= 8) rc = launch_bwd_col<T, 8>(a, nsplit, st, split_pass);
            else if (nkg <= 16) rc = launch_bwd_col<T, 16>(a, nsplit, st, split_pass);
            else rc = launch_bwd_col<T, 32>(a, nsplit, st, split_pass);
        } else {
            if (nkg <= 4) rc = launch_bwd_data<T, 4>(a, nsplit, st, split_pass);
            else if (nkg <= 8) rc = launch_bwd_data<T, 8>(a, nsplit, st, split_pass);
            else if (nkg <= 16) rc = launch_bwd_data<T, 16>(a, nsplit, st, split_pass);
            else rc = launch_bwd_data<T, 32>(a, nsplit, st, split_pass);
        }
        if (rc) return rc;
    }
    if (auxoff && (phase & 2)) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        if (goff) hipLaunchKernelGGL(aux_finish_kernel, dim3(grid1d(n_off)), dim3(256), 0, st, auxoff, goff, s.adt, n_off);
        if (gmask)
            hipLaunchKernelGGL(aux_finish_kernel, dim3(grid1d(n_mask)), dim3(256), 0, st, auxmask, gmask, s.adt, n_mask);
        if (int rc = d2c_check_launch("aux_finish_kernel")) return rc;
    }
    return D2C_OK;
}

// bytes of grad_out in fragment order (see pack_gout_kernel)
size_t d2c_bwd_goutp_bytes(const TiledShape &s, int dtype)
{
    const int vec = dtype == D2C_BF16 ? 8 : 4;
    const long ntile = (s.M + kWMT - 1) / kWMT, OBT = (s.og + 63) / 64 * 2;
    // (float: 24 bytes per entry where the copy holds three bfloat16 terms, see pack_gout3_kernel)
    return (size_t)s.groups * ntile * OBT * (kWMT / (2 * vec)) * 64 * (dtype == D2C_BF16 ? 16 : 24);
}

// How the position tiles of the grad-weight items are cut into workgroups (see BwdWeightArgs), found by simulating
// the dispatch and remembered per (items, tiles, compute units).
constexpr int kGwPieceCost = 10;     // what a workgroup costs beside its tiles (pipeline fill, adding its block), in tiles
struct GwPieces {
    int nmain, main_len, ntail, tail_len;
};
static GwPieces gw_pieces(long items, int ntile, int ncu, int max_main = 1)
{
    static std::mutex mu;
    static std::map<std::tuple<long, int, int, int>, GwPieces> memo;
    const auto key = std::make_tuple(items, ntile, ncu, max_main);
    {
        std::lock_guard<std::mutex> lock(mu);
        const auto it = memo.find(key);
        if (it != memo.end()) return it->second;
    }
    GwPieces r{1, ntile, 0, 1};
    std::vector<long> cu((size_t)ncu);
    auto makespan = [&](int nm, int ml, int nt, int tl) {
        std::fill(cu.begin(), cu.end(), 0L);
        long end = 0;
        auto run = [&](int len) {
            if (len <= 0) return;
            std::pop_heap(cu.begin(), cu.end(), std::greater<long>());
            cu.back() += len + kGwPieceCost;
            end = std::max(end, cu.back());
            std::push_heap(cu.begin(), cu.end(), std::greater<long>());
        };
        for (long i = 0; i < items; i++)
            for (int q = 0; q < nm; q++) run(std::min(ml, ntile - q * ml));
        for (long i = 0; i < items; i++)
            for (int q = 0; q < nt; q++) run(std::min(tl, ntile - nm * ml - q * tl));
        return end;
    };
    long best = -1;
    auto consider = [&](int nm, int ml, int nt, int tl, long handicap) {
        if (items * (nm + nt) > 16384) return;
        const long c = makespan(nm, ml, nt, tl) + handicap;
        if (best < 0 || c < best) { best = c; r = GwPieces{nm, ml, nt, tl}; }
    };
    // round-robin dealing (as a run of equal pieces, which costs the same)
    for (int k = 1; k <= 32 && k <= ntile; k += (k < 8 ? 1 : 4)) consider(k, (ntile + k - 1) / k, 0, 1, 0);
    // One main workgroup per item that takes most of its tiles, about as many as the whole launch should take, and
    // tail workgroups for the rest.  (Only with a single main piece per item: measured at 216 items x 405 tiles,
    // 8 % ahead of the deal to 7 on paper, 5 % faster; with two main pieces per item, at 108 items x 405 and
    // 108 x 3240 tiles, 9 % and 1 % ahead on paper, 9 % and 25 % slower: the workgroups of an item drift apart and
    // share less in L2.)
    // (tiled_bwd_weight_col_kernel, which gathers nothing, takes up to `max_main` main pieces per item: fewer pieces
    // than the round-robin deal needs for the same balance, and every piece ends in fp32 atomics of its whole block)
    const long ideal = (items * (ntile + kGwPieceCost) + ncu - 1) / ncu;
    for (int nm = 1; nm <= max_main; nm++) {
        if (!((nm + 1) * ideal > ntile && nm * ideal < ntile)) continue;
        for (int ml = (int)(ideal - ideal / 8); ml <= (int)(ideal + ideal / 8) && nm * ml < ntile; ml += 1 + (int)ideal / 64) {
            if ((nm + 1) * ml <= ntile) continue;
            const int rest = ntile - nm * ml;
            for (int f = 1; f <= 4; f++) consider(nm, ml, f, (rest + f - 1) / f, 0);
        }
    }
    std::lock_guard<std::mutex> lock(mu);
    memo[key] = r;
    return r;
}

// grad_weight from the sampled columns (tiled_bwd_weight_col_kernel, tiled_bwd_weight_col3_kernel): problems in three
// dimensions whose weight groups hold whole sets of kColChunks channel chunks.
bool d2c_bwd_weight_from_col(const TiledShape &s, int dtype)
{
    return (dtype == D2C_BF16 || dtype == D2C_F32) && s.nd == 3 && s.nchunk % kColChunks == 0;
}
// float problems over kept columns on three-term bfloat16 operands: weight groups of whole sets of kCol3Chunks chunks
bool d2c_bwd_weight_col3(const TiledShape &s) { return s.nd == 3 && s.nchunk % kCol3Chunks == 0; }
// ... from the columns that the forward call kept (d2c_fwd_writes_columns): the same shapes
bool d2c_bwd_weight_from_kept_col(const TiledShape &s, int dtype) { return d2c_bwd_weight_from_col(s, dtype); }
// bytes of the sampled columns [chunk][tap][whole 64-position tiles][64 bfloat16 / 32 float] of `nchunks` channel
// chunks (0: all)
size_t d2c_bwd_col_bytes(const TiledShape &s, int dtype, int nchunks)
{
    const long ntile = (s.M + kWDT - 1) / kWDT;
    const int bkc = dtype == D2C_BF16 ? 64 : 32;
    return (size_t)(nchunks > 0 ? nchunks : s.Cin / bkc) * s.K * ntile * kWDT * 128;
}

// The backward pass of this shape can run slice by slice over its offset groups (grad-column product, offset / mask
// gradient, grad_input and the grad-weight product of one slice after the other, with buffers for the grad-column
// rows and the sampled columns of ONE slice): bfloat16 problems on tiled_bwd_col32_kernel with one weight group.
bool d2c_bwd_sliceable(const TiledShape &s, int dtype)
{
    return dtype == D2C_BF16 && s.nd == 3 && s.groups == 1 && s.G > 1 && s.og <= d2c_bwd_pass_channels(dtype) &&
           bwd_col32_ok(d2c_bwd_ogk(s.og, dtype), s.og, dtype) && d2c_bwd_weight_from_col(s, dtype);
}

template <typename T>
int d2c_tiled_bwd_weight_launch(const TiledShape &s, const void *gout, const void *xcl, const void *off,
                                const void *mask, void *goutp, float *gwacc, void *gw, const void *col, long col_rows,
                                hipStream_t st, int phase, int jp_lo, int jp_n)
{
    // phase: 1 = the clear of the sums and the fragment-ordered copy of grad_out, 2 = the kernel, 4 = the conversion of
    // the sums; 7 = all.  jp_n > 0 (product over the sampled columns only): the pairs of channel chunks
    // [jp_lo, jp_lo + jp_n) of every weight group, `col` pointing where chunk 0 would start.
    const long nw = (long)s.Cout * s.cg * s.K;
    const int steps = s.nchunk * s.K;
    const int otiles = (s.og + 511) / 512;
    const int ntp = (s.M + kWMT - 1) / kWMT;     // tiles of the packed grad_out copy
    const int ntile = (s.M + kWDT - 1) / kWDT;   // position tiles of the kernel
    const bool from_col = col != nullptr;
    // float problems over kept columns: the product on three-term bfloat16 operands (tiled_bwd_weight_col3_kernel)
    bool col3 = false;
    if constexpr (sizeof(T) == 4) col3 = from_col && d2c_bwd_weight_col3(s);
    const int OBT = (s.og + 63) / 64 * 2;
    const long total = (long)s.groups * ntp * OBT * (kWMT / (2 * Elem<T>::VEC)) * 64;
    if ((phase & 1) && col3) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        d2c_fill_zero(gwacc, (size_t)nw * sizeof(float), st);
        hipLaunchKernelGGL(pack_gout3_kernel, dim3(grid1d(total, 16384)), dim3(256), 0, st, (const float *)gout,
                           (uint4 *)goutp, s, ntp, OBT, total);
        if (int rc = d2c_check_launch("pack_gout3_kernel")) return rc;
    } else if (phase & 1) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        d2c_fill_zero(gwacc, (size_t)nw * sizeof(float), st);
        // (the channels-last input is followed by a 256-byte row of zeros, written by the kernel that packed it:
        // what dead corners read)
        const bool vec = s.P % Elem<T>::VEC == 0 && reinterpret_cast<uintptr_t>(gout) % 16 == 0;
        constexpr bool SPT = sizeof(T) == 4;
        // (the product over kept columns runs on the float instruction whatever the flags say)
        auto k_gout = (SPT && s.f32split == 1 && !from_col) ? &pack_gout_kernel<T, SPT> : &pack_gout_kernel<T, false>;
        hipLaunchKernelGGL(k_gout, dim3(grid1d(total, 16384)), dim3(256), 0, st, (const T *)gout, (T *)goutp, s, ntp, OBT,
                           total, vec);
        if (int rc = d2c_check_launch("pack_gout_kernel")) return rc;
    }
    // One workgroup runs per compute unit at a time (LDS).  The pieces (see BwdWeightArgs) are the ones whose
    // dispatch, simulated in gw_pieces (workgroups start in grid order on the unit that is free first), finishes
    // first.
    const int ncu = d2c_num_cus();
    if (ncu <= 0) return D2C_ERR_LAUNCH;
    if (from_col && !d2c_bwd_weight_from_kept_col(s, (int)Elem<T>::DT)) {
        d2c_set_error("grad_weight: tiled_bwd_weight_col_kernel does not take this shape");
        return D2C_ERR_LAUNCH;
    }
    if (jp_n > 0 && !from_col) {
        d2c_set_error("grad_weight: slices are made by tiled_bwd_weight_col_kernel only");
        return D2C_ERR_LAUNCH;
    }
    if (col3) {
        if (jp_n > 0) {
            d2c_set_error("grad_weight: tiled_bwd_weight_col3_kernel takes no slices");
            return D2C_ERR_LAUNCH;
        }
        if (phase & 2) {
            const int otiles3 = (s.og + kCol3Rows - 1) / kCol3Rows;
            const long items3 = (long)(s.nchunk / kCol3Chunks) * s.K * otiles3 * s.groups;
            const GwPieces pc = gw_pieces(items3, ntile, ncu, 4);
            BwdWeightCol3Args c{s, col, (const uint4 *)goutp, reinterpret_cast<const uint2 *>((const uint4 *)goutp + total),
                                gwacc, col_rows, otiles3, pc.nmain, pc.main_len, pc.ntail, pc.tail_len};
            if (int rc = d2c_allow_lds((const void *)tiled_bwd_weight_col3_kernel, (int)kCol3Lds, "tiled_bwd_weight_col3_kernel"))
                return rc;
            D2cProfScope prof(D2C_PROF_BWD_WEIGHT, st, "tiled_bwd_weight_col3_kernel");
            hipLaunchKernelGGL(tiled_bwd_weight_col3_kernel, dim3((unsigned)(items3 * (pc.nmain + pc.ntail))), dim3(kThreads),
                               kCol3Lds, st, c);
            if (int rc = d2c_check_launch("tiled_bwd_weight_col3_kernel")) return rc;
        }
        phase &= ~2;
    }
    if (jp_n <= 0) { jp_lo = 0; jp_n = s.nchunk / kColChunks; }
    const long items = (long)(from_col ? jp_n * s.K : steps) * otiles * s.groups;
    const GwPieces pc = gw_pieces(items, ntile, ncu, from_col ? 4 : 1);
    const int nmain = pc.nmain, main_len = pc.main_len, ntail = pc.ntail, tail_len = pc.tail_len;
    if (from_col && (phase & 2)) {
        BwdWeightColArgs c{s, col, goutp, gwacc, col_rows, otiles, nmain, main_len, ntail, tail_len, jp_lo, jp_n};
        D2cProfScope prof(D2C_PROF_BWD_WEIGHT, st, "tiled_bwd_weight_col_kernel");
        hipLaunchKernelGGL(tiled_bwd_weight_col_kernel<T>, dim3((unsigned)(items * (nmain + ntail))), dim3(kThreads), 0, st, c);
        if (int rc = d2c_check_launch("tiled_bwd_weight_col_kernel")) return rc;
    }
    BwdWeightDmaArgs a{{s, gout, xcl, off, mask, goutp, gwacc, otiles, nmain, main_len, ntail, tail_len},
                       (unsigned)((size_t)s.N * s.vol * s.Cin * sizeof(T))};
    if (!from_col && (phase & 2)) {
        const dim3 grid((unsigned)(items * (nmain + ntail)));
        bool aux16 = false;
        if constexpr (sizeof(T) == 2) aux16 = s.adt == D2C_BF16;
        D2cProfScope prof(D2C_PROF_BWD_WEIGHT, st, "tiled_bwd_weight_dma_kernel");
        auto go_sp = [&](auto aux_c, auto sized_c, auto nc_c, auto split_c) -> bool {
            constexpr bool A16 = decltype(aux_c)::value, SZ = decltype(sized_c)::value, SP = decltype(split_c)::value;
            constexpr int NC = decltype(nc_c)::value;
            constexpr size_t lds = bwd_weight_dma_lds<T, NC>();
            if (d2c_allow_lds((const void *)tiled_bwd_weight_dma_kernel<T, A16, SZ, NC, SP>, 160 * 1024,
                              "tiled_bwd_weight_dma_kernel") != D2C_OK)
                return false;
            hipLaunchKernelGGL((tiled_bwd_weight_dma_kernel<T, A16, SZ, NC, SP>), grid, dim3(kThreads + 64), lds, st, a);
            return true;
        };
        auto go_nc = [&](auto aux_c, auto sized_c, auto nc_c) -> bool {
            if constexpr (sizeof(T) == 4) {
                if (s.f32split == 1) return go_sp(aux_c, sized_c, nc_c, std::true_type{});
            }
            return go_sp(aux_c, sized_c, nc_c, std::false_type{});
        };
        const bool sized = s.ss.on != 0;
        // offsets fixed along one / two axes: 4 / 2 corner rows per sampling point (offsets-tensor source only)
        const int nfree = (s.nd == 3 && !sized) ? __builtin_popcount(s.axes & 7) : 3;
        auto go = [&](auto aux_c, auto sized_c) -> bool {
            if constexpr (!decltype(sized_c)::value) {
                if (nfree == 2) return go_nc(aux_c, sized_c, std::integral_constant<int, 4>{});
                if (nfree == 1) return go_nc(aux_c, sized_c, std::integral_constant<int, 2>{});
            }
            return go_nc(aux_c, sized_c, std::integral_constant<int, 8>{});
        };
        bool ok;
        if constexpr (sizeof(T) == 2) {
            if (aux16) ok = sized ? go(std::true_type{}, std::true_type{}) : go(std::true_type{}, std::false_type{});
            else ok = sized ? go(std::false_type{}, std::true_type{}) : go(std::false_type{}, std::false_type{});
        } else {
            ok = sized ? go(std::false_type{}, std::true_type{}) : go(std::false_type{}, std::false_type{});
        }
        if (!ok) return D2C_ERR_LAUNCH;   // (d2c_allow_lds has set the error text)
    }
    if (int rc = d2c_check_launch("tiled_bwd_weight_dma_kernel")) return rc;
    if (!(phase & 4)) return D2C_OK;
    D2cProfScope prof(D2C_PROF_PACK, st);
    constexpr int BKC = 8 * Elem<T>::VEC;
    const size_t cvt_lds = (size_t)kCvtRows * ((size_t)BKC * s.K * sizeof(T) + 16);
    if (cvt_lds <= 64 * 1024 && reinterpret_cast<uintptr_t>(gw) % 16 == 0)
        hipLaunchKernelGGL(cvt_grad_weight_lds_kernel<T>,
                           dim3((unsigned)(s.groups * s.nchunk * ((s.og + kCvtRows - 1) / kCvtRows))), dim3(256), cvt_lds,
                           st, gwacc, (T *)gw, s);
    else
        hipLaunchKernelGGL(cvt_grad_weight_kernel<T>, dim3(grid1d(nw)), dim3(256), 0, st, gwacc, (T *)gw, s, nw);
    return d2c_check_launch("cvt_grad_weight_kernel");
}

template <typename T>
int d2c_tiled_unpack_gx(const TiledShape &s, const float *gxcl, void *gx, hipStream_t st)
{
    dim3 grid((s.vol + 31) / 32, (s.Cin + 31) / 32, s.N);
    D2cProfScope prof(D2C_PROF_PACK, st);
    if constexpr (sizeof(T) == 2) {
        if (s.vol % 8 == 0 && s.Cin % 8 == 0 && reinterpret_cast<uintptr_t>(gx) % 16 == 0) {
            hipLaunchKernelGGL(unpack_grad_input_bf16_kernel, dim3((s.vol + 63) / 64, (s.Cin + 63) / 64, s.N), dim3(256), 0,
                               st, gxcl, (bf16_t *)gx, s.Cin, s.vol);
            return d2c_check_launch("unpack_grad_input_bf16_kernel");
        }
    }
    hipLaunchKernelGGL(unpack_grad_input_kernel<T>, grid, dim3(256), 0, st, gxcl, (T *)gx, s.Cin, s.vol);
    return d2c_check_launch("unpack_grad_input_kernel");
}

template <typename T>
int d2c_tiled_bias_grad(const TiledShape &s, const void *gout, void *gb, hipStream_t st)
{
    D2cProfScope prof(D2C_PROF_PACK, st);
    hipLaunchKernelGGL(bias_grad_kernel<T>, dim3(s.Cout), dim3(1024), 0, st, (const T *)gout, (T *)gb, s.N, s.Cout, s.P);
    return d2c_check_launch("bias_grad_kernel");
}

#define INST(T)                                                                                                    \
    template int d2c_tiled_bwd_data_launch<T>(const TiledShape &, const void *, const void *, const void *,        \
                                              const void *, const void *, void *, float *, void *, void *, void *, \
                                              float *, hipStream_t, int, int, int, bool);                                   \
    template int d2c_tiled_bwd_weight_launch<T>(const TiledShape &, const void *, const void *, const void *,      \
                                                const void *, void *, float *, void *, const void *, long, hipStream_t, \
                                                int, int, int);                                                     \
    template int d2c_tiled_unpack_gx<T>(const TiledShape &, const float *, void *, hipStream_t);                   \
    template int d2c_tiled_bias_grad<T>(const TiledShape &, const void *, void *, hipStream_t);
INST(bf16_t)
INST(float)
