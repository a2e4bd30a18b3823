// Forward pass as an implicit GEMM on the matrix cores.
//
//   out[b, o, p] = bias[o] + sum_{c, k} W[o, c, k] * alpha[b,g,k,p] * trilinear(x[b, c], pos(b,g,k,p))
//
// GEMM view: rows = output channels, columns = output positions (N*P of
// them), reduction = (channel chunk, tap).  The sampled operand is produced on
// the fly: for one (chunk, tap) step every thread gathers the 8 corners of its
// position as 16-byte channel vectors from the channels-last copy of the
// input, interpolates in fp32 with the modulation folded into the corner
// weights, and drops the result into an LDS tile in MFMA operand order.  The
// im2col column buffer of the reference (dconv3d_gpu.cu:297) never exists.
//
// One workgroup = 512 threads = MT positions x NT output channels.  Steps are
// software-pipelined over three stages: while the matrix cores work on step s,
// the corner rows of step s+1 and the weight fragments of step s+1 are in
// flight and the offsets of step s+2 are being fetched; nothing waits on
// memory inside a step except at its one barrier.
#include "d2c_mma.hpp"
#include "d2c_tiled.hpp"

namespace {

constexpr int kNV = 8;         // 16-byte vectors per sampled row (one chunk)
constexpr int kRS = kNV * 16 + 16;  // LDS row stride in bytes (padded: conflict-free 16-byte reads)
constexpr int kThreads = 512;
constexpr int kMT = 128;       // positions per workgroup

struct FwdArgs {
    TiledShape s;
    const void *xcl;   // [N][vol][Cin]
    const void *off, *mask;
    const void *wp;    // packed weights, see pack_weight_fwd
    const void *bias;
    void *out;
    // Few tiles (small N*P): the steps are dealt to `nsplit` workgroups per tile, which add their partial
    // sums into a zeroed fp32 array laid out like `out`; a finishing kernel adds the bias and converts.
    float *outacc;
    int nsplit;
    unsigned zrow;     // byte offset (from xcl) of a 128-byte row of zeros: what dead corners read
};

// Tiles that are neighbours in space go to the same XCD (workgroups are dealt
// round-robin over the 8 XCDs), so that its L2 sees a compact part of the input.
D2C_DEV int xcd_swizzle(int bid, int n)
{
    const int x = bid & 7, idx = bid >> 3;
    const int q = n >> 3, r = n & 7;
    return x * q + (x < r ? x : r) + idx;
}

template <typename T, bool AUX16, int MT, int WAVES_O, int WAVES_P>
__global__ void __launch_bounds__(kThreads) tiled_fwd_kernel(FwdArgs a)
{
    constexpr int VEC = Elem<T>::VEC;
    constexpr int BKC = kNV * VEC;
    constexpr int WPOS = MT / WAVES_P;    // positions per MMA wave
    constexpr int PB = WPOS / 32;         // 32-position blocks per MMA wave
    constexpr int OB = 2;                 // 32-channel blocks per MMA wave
    constexpr int NT = 64 * WAVES_O;      // output channels per workgroup
    constexpr int NKG = kNV / 2;          // k-groups per step
    constexpr int ITEMS = MT * kNV / kThreads;   // (position, vector) items per thread
    static_assert(ITEMS >= 1 && ITEMS * kThreads == MT * kNV, "gather items divide evenly");
    static_assert(WAVES_O * WAVES_P <= kThreads / 64 && PB >= 1, "MMA wave layout");

    __shared__ __align__(16) unsigned char s_tile[2][MT * kRS];
    __shared__ float s_w[2][8][MT];
    __shared__ int s_idx[2][MT];
    __shared__ int s_flag[2][MT];

    const TiledShape &s = a.s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tile = xcd_swizzle(blockIdx.x, gridDim.x);
    const int otile = blockIdx.y / a.nsplit, split = blockIdx.y - otile * a.nsplit, wg = blockIdx.z;
    const int m0 = tile * MT;
    const int S = s.nchunk * s.K;                           // steps of the whole reduction
    const int st_lo = (int)((long)S * split / a.nsplit);    // this workgroup's share of them
    const int st_hi = (int)((long)S * (split + 1) / a.nsplit);
    const int dzc = s.H * s.W * s.Cin, dyc = s.W * s.Cin;   // element strides of a step in z / y

    // --- per-position constants of the coordinate threads
    int cb = 0, cp = 0, coz = 0, coy = 0, cox = 0;
    bool cvalid = false;
    if (tid < MT) {
        const int m = m0 + tid;
        cvalid = m < s.M;
        if (cvalid) {
            cb = m / s.P; cp = m - cb * s.P;
            cox = cp % s.Wo; coy = (cp / s.Wo) % s.Ho; coz = cp / (s.Wo * s.Ho);
        }
    }

    // offsets and modulation of step st: fetched early (coords_issue), turned into corner weights
    // (modulation folded in, dead corners zero), base offset and live mask late (coords_finish)
    float craw[4];
    auto coords_issue = [&](int st) {
        if (tid < MT && cvalid) {
            const int j = st / s.K, k = st - j * s.K;
            const int g = (wg * s.cg + j * BKC) / s.cpg;
            if (s.nd == 3) {
                const long ob = (((long)cb * s.G + g) * s.K + k) * 3 * s.P + cp;
                craw[0] = ld_auxT<AUX16>(a.off, ob);
                craw[1] = ld_auxT<AUX16>(a.off, ob + s.P);
                craw[2] = ld_auxT<AUX16>(a.off, ob + 2 * (long)s.P);
            } else {
                craw[0] = 0.f; craw[1] = 0.f;
                craw[2] = ld_auxT<AUX16>(a.off, (((long)cb * s.G + g) * s.K + k) * s.P + cp);
            }
            craw[3] = a.mask ? ld_auxT<AUX16>(a.mask, (((long)cb * s.G + g) * s.K + k) * s.P + cp) : 1.f;
        }
    };
    auto coords_finish = [&](int st, int buf) {
        if (tid < MT) {
            float w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            int idx = 0;
            unsigned live = 0;
            if (cvalid) {
                const int k = st % s.K;
                int bz, by, bx;
                tap_base(s.geo, k, coz, coy, cox, bz, by, bx);
                const Tap3<float> t = make_tap3<float>(bz, by, bx, craw[0], craw[1], craw[2], s.D, s.H, s.W);
                live = t.live;
                idx = (cb * s.vol + (t.z0 * s.H + t.y0) * s.W + t.x0) * s.Cin;   // element offset of corner 000
#pragma unroll
                for (int c = 0; c < 8; c++) w[c] = ((live >> c) & 1u) ? tap3_weight(t, c) * craw[3] : 0.f;
            }
#pragma unroll
            for (int c = 0; c < 8; c++) s_w[buf][c][tid] = w[c];
            s_idx[buf][tid] = idx;
            s_flag[buf][tid] = (int)live;
        }
    };

    // --- gather: item i of this thread = (position, 16-byte channel vector)
    uint4 gv[ITEMS][8];
    auto gather_issue = [&](int st, int buf) {
        const int j = st / s.K;
        const int c0 = wg * s.cg + j * BKC;
        // 32-bit byte offsets from a uniform base: the whole input is below 4 GiB (checked on the host)
        const char *base = reinterpret_cast<const char *>(a.xcl);
#pragma unroll
        for (int i = 0; i < ITEMS; i++) {
            const int item = tid + i * kThreads;
            const int pos = item / kNV, vec = item % kNV;
            const int idx = s_idx[buf][pos] + c0 + vec * VEC;
            const unsigned live = (unsigned)s_flag[buf][pos];
#pragma unroll
            for (int c = 0; c < 8; c++) {
                const unsigned o = (unsigned)(idx + ((c >> 2) & 1) * dzc + ((c >> 1) & 1) * dyc + (c & 1) * s.Cin)
                                   * (unsigned)sizeof(T);
                gv[i][c] = ((live >> c) & 1u) ? *reinterpret_cast<const uint4 *>(base + o) : make_uint4(0, 0, 0, 0);
            }
        }
    };
    auto interp_store = [&](int cbuf, int tbuf) {
#pragma unroll
        for (int i = 0; i < ITEMS; i++) {
            const int item = tid + i * kThreads;
            const int pos = item / kNV, vec = item % kNV;
            VecAcc<T> acc;
            acc.zero();
#pragma unroll
            for (int c = 0; c < 8; c++) acc.fma(s_w[cbuf][c][pos], gv[i][c]);
            *reinterpret_cast<uint4 *>(&s_tile[tbuf][pos * kRS + vec * 16]) = acc.pack();
        }
    };

    // --- MMA role
    const bool mma_wave = wave < WAVES_O * WAVES_P;
    const int wave_o = wave % WAVES_O, wave_p = wave / WAVES_O;
    const int OBT = s.ogp / 32;  // 32-channel blocks per weight group in the packed weights
    f32x16 acc[OB][PB];
#pragma unroll
    for (int ob = 0; ob < OB; ob++)
#pragma unroll
        for (int pb = 0; pb < PB; pb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[ob][pb][r] = 0.f;

    // weight fragments of one whole step live in registers; those of the next step are requested
    // as soon as the matrix cores have taken the current ones
    const uint4 *wp4 = reinterpret_cast<const uint4 *>(a.wp);
    uint4 af[NKG][OB];
    auto wfrag = [&](int st, int kg, int ob) {
        const long wbase = (((long)wg * S + st) * OBT + (otile * (NT / 32) + wave_o * OB)) * NKG * 64 + lane;
        return wp4[wbase + ((long)ob * NKG + kg) * 64];
    };
    auto mma_step = [&](int st, int tbuf) {
        if (!mma_wave) return;
        const unsigned char *tb = &s_tile[tbuf][(wave_p * WPOS + (lane & 31)) * kRS + (lane >> 5) * 16];
#pragma unroll
        for (int kg = 0; kg < NKG; kg++) {
            uint4 bf[PB];
#pragma unroll
            for (int pb = 0; pb < PB; pb++)
                bf[pb] = *reinterpret_cast<const uint4 *>(tb + pb * 32 * kRS + kg * 32);
#pragma unroll
            for (int ob = 0; ob < OB; ob++)
#pragma unroll
                for (int pb = 0; pb < PB; pb++) mma_kgroup<T>(acc[ob][pb], af[kg][ob], bf[pb]);
            if (st + 1 < st_hi) {
#pragma unroll
                for (int ob = 0; ob < OB; ob++) af[kg][ob] = wfrag(st + 1, kg, ob);
            }
        }
    };

    // --- pipeline (buffers alternate with the parity of the step number)
    coords_issue(st_lo);
    if (mma_wave) {
#pragma unroll
        for (int kg = 0; kg < NKG; kg++)
#pragma unroll
            for (int ob = 0; ob < OB; ob++) af[kg][ob] = wfrag(st_lo, kg, ob);
    }
    coords_finish(st_lo, st_lo & 1);
    if (st_lo + 1 < st_hi) coords_issue(st_lo + 1);
    __syncthreads();
    gather_issue(st_lo, st_lo & 1);
    if (st_lo + 1 < st_hi) coords_finish(st_lo + 1, (st_lo + 1) & 1);
    if (st_lo + 2 < st_hi) coords_issue(st_lo + 2);
    interp_store(st_lo & 1, st_lo & 1);
    __syncthreads();
    for (int st = st_lo; st < st_hi; st++) {
        if (st + 1 < st_hi) gather_issue(st + 1, (st + 1) & 1);
        mma_step(st, st & 1);
        if (st + 2 < st_hi) coords_finish(st + 2, st & 1);
        if (st + 3 < st_hi) coords_issue(st + 3);
        if (st + 1 < st_hi) interp_store((st + 1) & 1, (st + 1) & 1);
        __syncthreads();
    }

    // --- epilogue: bias, convert, store (32 consecutive positions per row of a block)
    if (mma_wave) {
        T *out = reinterpret_cast<T *>(a.out);
        const T *bias = reinterpret_cast<const T *>(a.bias);
#pragma unroll
        for (int pb = 0; pb < PB; pb++) {
            const int m = m0 + wave_p * WPOS + pb * 32 + (lane & 31);
            if (m >= s.M) continue;
            const int b = m / s.P, p = m - b * s.P;
#pragma unroll
            for (int ob = 0; ob < OB; ob++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int ol = otile * NT + wave_o * 64 + ob * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (ol < s.og) {
                        const int o = wg * s.og + ol;
                        float v = acc[ob][pb][r];
                        if (a.outacc) {
                            atomicAdd(a.outacc + ((long)b * s.Cout + o) * s.P + p, v);
                        } else {
                            if (bias) v += elem_to_f32<T>(bias[o]);
                            out[((long)b * s.Cout + o) * s.P + p] = f32_to_elem<T>(v);
                        }
                    }
                }
            }
        }
    }
}


// ---------------------------------------------------------------------------
// The same forward pass with the corner rows moved global -> LDS by DMA loads
// (global_load_lds_dwordx4: no staging registers, so the rows of step s+2 are
// in flight while step s runs on the matrix cores and step s+1 is interpolated).
// One workgroup = 512 threads = 64 positions x NT output channels.  One DMA
// instruction of a wavefront fetches the 8 corner rows (8 x 128 bytes) of one
// position: lane = (corner, 16-byte vector); corners that are out of range or
// cut off by the early-out read a row of zeros instead.
constexpr int kDMT = 64;                   // positions per workgroup
constexpr int kRawPos = 8 * kNV * 16;      // raw bytes per position: 8 corners x 128

template <typename T, bool AUX16, int WAVES_O, int WAVES_P>
__global__ void __launch_bounds__(kThreads + 64) tiled_fwd_dma_kernel(FwdArgs a)
{
    constexpr int MT = kDMT;
    constexpr int VEC = Elem<T>::VEC;
    constexpr int BKC = kNV * VEC;
    constexpr int WPOS = MT / WAVES_P;    // positions per MMA wave
    constexpr int PB = WPOS / 32;         // 32-position blocks per MMA wave
    constexpr int OB = 2;                 // 32-channel blocks per MMA wave
    constexpr int NT = 64 * WAVES_O;      // output channels per workgroup
    constexpr int NKG = kNV / 2;          // k-groups per step
    static_assert(MT * kNV == kThreads, "one (position, vector) item per thread");
    static_assert(WAVES_O * WAVES_P <= kThreads / 64 && PB >= 1, "MMA wave layout");

    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char *s_raw = smem;                                   // [2][MT][8 corners][128 B]
    unsigned char *s_tile = s_raw + 2 * MT * kRawPos;              // [2][MT][kRS]
    float *s_w = reinterpret_cast<float *>(s_tile + 2 * MT * kRS); // [3][8][MT]
    int *s_idx = reinterpret_cast<int *>(s_w + 3 * 8 * MT);        // [3][MT]
    int *s_flag = s_idx + 3 * MT;                                  // [3][MT]

    const TiledShape &s = a.s;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tile = xcd_swizzle(blockIdx.x, gridDim.x);
    const int otile = blockIdx.y / a.nsplit, split = blockIdx.y - otile * a.nsplit, wg = blockIdx.z;
    const int m0 = tile * MT;
    const int S = s.nchunk * s.K;
    const int st_lo = (int)((long)S * split / a.nsplit);
    const int st_hi = (int)((long)S * (split + 1) / a.nsplit);
    const int dzc = s.H * s.W * s.Cin, dyc = s.W * s.Cin;

    // --- coordinates: a ninth wavefront (one position per lane) that does nothing else, so that this
    // arithmetic runs beside the work of the other eight instead of in front of their barrier
    const bool cwave = wave == 8;        // coordinates
    const bool worker = wave < 8;
    const int ctid = tid - kThreads;
    int cb = 0, cp = 0, coz = 0, coy = 0, cox = 0;
    bool cvalid = false;
    if (cwave) {
        const int m = m0 + ctid;
        cvalid = m < s.M;
        if (cvalid) {
            cb = m / s.P; cp = m - cb * s.P;
            cox = cp % s.Wo; coy = (cp / s.Wo) % s.Ho; coz = cp / (s.Wo * s.Ho);
        }
    }
    float craw[4];
    auto coords_issue = [&](int st) {
        if (cwave && cvalid) {
            const int j = st / s.K, k = st - j * s.K;
            const int g = (wg * s.cg + j * BKC) / s.cpg;
            const long ab = (((long)cb * s.G + g) * s.K + k) * s.P + cp;
            if (s.nd == 3) {
                const long ob = 3 * ab - 2 * (long)cp;
                craw[0] = ld_auxT<AUX16>(a.off, ob);
                craw[1] = ld_auxT<AUX16>(a.off, ob + s.P);
                craw[2] = ld_auxT<AUX16>(a.off, ob + 2 * (long)s.P);
            } else {
                craw[0] = 0.f; craw[1] = 0.f;
                craw[2] = ld_auxT<AUX16>(a.off, ab);
            }
            craw[3] = a.mask ? ld_auxT<AUX16>(a.mask, ab) : 1.f;
        }
    };
    auto coords_finish = [&](int st, int buf) {
        if (cwave) {
            float w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            int idx = 0;
            unsigned live = 0;
            if (cvalid) {
                const int k = st % s.K;
                int bz, by, bx;
                tap_base(s.geo, k, coz, coy, cox, bz, by, bx);
                const Tap3<float> t = make_tap3<float>(bz, by, bx, craw[0], craw[1], craw[2], s.D, s.H, s.W);
                live = t.live;
                idx = (cb * s.vol + (t.z0 * s.H + t.y0) * s.W + t.x0) * s.Cin;   // element offset of corner 000
#pragma unroll
                for (int c = 0; c < 8; c++) w[c] = ((live >> c) & 1u) ? tap3_weight(t, c) * craw[3] : 0.f;
            }
#pragma unroll
            for (int c = 0; c < 8; c++) s_w[(buf * 8 + c) * MT + ctid] = w[c];
            s_idx[buf * MT + ctid] = idx;
            s_flag[buf * MT + ctid] = (int)live;
        }
    };

    // --- corner rows of step st -> s_raw[rbuf]: worker wavefront w requests positions 8w .. 8w+7, one
    // instruction per position, lane = (corner, 16-byte vector)
    const int dcorner = lane >> 3, dvec = lane & 7;
    const int dcoff = ((dcorner >> 2) & 1) * dzc + ((dcorner >> 1) & 1) * dyc + (dcorner & 1) * s.Cin;
    auto dma_issue = [&](int st, int rbuf, int tbuf) {
        if (!worker) return;
        const int j = st / s.K;
        const int c0 = wg * s.cg + j * BKC;
        const char *base = reinterpret_cast<const char *>(a.xcl);
        // table entries of this wavefront's 8 positions: one LDS read (lane i holds position i), then
        // lane-indexed moves to scalar registers
        const int vidx = s_idx[tbuf * MT + wave * (MT / 8) + (lane & 7)];
        const int vflag = s_flag[tbuf * MT + wave * (MT / 8) + (lane & 7)];
#pragma unroll
        for (int i = 0; i < MT / 8; i++) {
            const int pos = wave * (MT / 8) + i;
            const int idx = __builtin_amdgcn_readlane(vidx, i);
            const unsigned live = (unsigned)__builtin_amdgcn_readlane(vflag, i);
            const unsigned o = ((live >> dcorner) & 1u)
                                   ? (unsigned)(idx + c0 + dcoff + dvec * VEC) * (unsigned)sizeof(T)
                                   : a.zrow + (unsigned)dvec * 16u;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(base + o),
                                             (__attribute__((address_space(3))) void *)(s_raw + (rbuf * MT + pos) * kRawPos),
                                             16, 0, 0);
        }
    };
    // --- interpolation: thread = (position, 16-byte vector)
    const int ipos = tid >> 3, ivec = tid & 7;
    auto interp_store = [&](int rbuf, int tbuf, int dbuf) {
        if (!worker) return;
        const unsigned char *rp = s_raw + (rbuf * MT + ipos) * kRawPos + ivec * 16;
        VecAcc<T> acc;
        acc.zero();
#pragma unroll
        for (int c = 0; c < 8; c++)
            acc.fma(s_w[(tbuf * 8 + c) * MT + ipos], *reinterpret_cast<const uint4 *>(rp + c * (kNV * 16)));
        *reinterpret_cast<uint4 *>(s_tile + (dbuf * MT + ipos) * kRS + ivec * 16) = acc.pack();
    };

    // --- MMA role
    const bool mma_wave = wave < WAVES_O * WAVES_P;
    const int wave_o = wave % WAVES_O, wave_p = wave / WAVES_O;
    const int OBT = s.ogp / 32;
    f32x16 acc[OB][PB];
#pragma unroll
    for (int ob = 0; ob < OB; ob++)
#pragma unroll
        for (int pb = 0; pb < PB; pb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[ob][pb][r] = 0.f;
    const uint4 *wp4 = reinterpret_cast<const uint4 *>(a.wp);
    uint4 af[NKG][OB];
    auto wfrag = [&](int st, int kg, int ob) {
        const long wbase = (((long)wg * S + st) * OBT + (otile * (NT / 32) + wave_o * OB)) * NKG * 64 + lane;
        return wp4[wbase + ((long)ob * NKG + kg) * 64];
    };
    auto mma_step = [&](int st, int dbuf) {
        if (!mma_wave) return;
        const unsigned char *tb = s_tile + (dbuf * MT + wave_p * WPOS + (lane & 31)) * kRS + (lane >> 5) * 16;
#pragma unroll
        for (int kg = 0; kg < NKG; kg++) {
            uint4 bf[PB];
#pragma unroll
            for (int pb = 0; pb < PB; pb++)
                bf[pb] = *reinterpret_cast<const uint4 *>(tb + pb * 32 * kRS + kg * 32);
#pragma unroll
            for (int ob = 0; ob < OB; ob++)
#pragma unroll
                for (int pb = 0; pb < PB; pb++) mma_kgroup<T>(acc[ob][pb], af[kg][ob], bf[pb]);
            if (st + 1 < st_hi) {
#pragma unroll
                for (int ob = 0; ob < OB; ob++) af[kg][ob] = wfrag(st + 1, kg, ob);
            }
        }
    };

    // --- pipeline.  Iteration `it`: rows of step it+2 requested, step it on the matrix cores, step it+1
    // interpolated, coordinates of step it+3 computed.  Corner tables rotate over 3 buffers, raw rows and
    // tiles over 2.  Everything requested in one iteration has that whole iteration to arrive.
    for (int q = 0; q < 3; q++) {
        if (st_lo + q < st_hi) {
            coords_issue(st_lo + q);
            coords_finish(st_lo + q, (st_lo + q) % 3);
        }
    }
    if (mma_wave) {
#pragma unroll
        for (int kg = 0; kg < NKG; kg++)
#pragma unroll
            for (int ob = 0; ob < OB; ob++) af[kg][ob] = wfrag(st_lo, kg, ob);
    }
    __syncthreads();
    dma_issue(st_lo, st_lo & 1, st_lo % 3);
    if (st_lo + 1 < st_hi) dma_issue(st_lo + 1, (st_lo + 1) & 1, (st_lo + 1) % 3);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    interp_store(st_lo & 1, st_lo % 3, st_lo & 1);
    if (st_lo + 3 < st_hi) coords_issue(st_lo + 3);
    // One loop per role (separate register budgets), the same synchronisation point per iteration in each.
    if (worker) {
        for (int it = st_lo; it < st_hi; it++) {
            __builtin_amdgcn_s_waitcnt(0);     // the transfers requested in the last iteration have landed
            __syncthreads();
            mma_step(it, it & 1);
            if (it + 2 < st_hi) dma_issue(it + 2, it & 1, (it + 2) % 3);
            if (it + 1 < st_hi) interp_store((it + 1) & 1, (it + 1) % 3, (it + 1) & 1);
        }
    } else {
        for (int it = st_lo; it < st_hi; it++) {
            __syncthreads();
            if (it + 3 < st_hi) coords_finish(it + 3, it % 3);   // offsets requested one iteration ago
            if (it + 4 < st_hi) coords_issue(it + 4);
        }
    }

    // --- epilogue: bias, convert, store
    if (mma_wave) {
        T *out = reinterpret_cast<T *>(a.out);
        const T *bias = reinterpret_cast<const T *>(a.bias);
#pragma unroll
        for (int pb = 0; pb < PB; pb++) {
            const int m = m0 + wave_p * WPOS + pb * 32 + (lane & 31);
            if (m >= s.M) continue;
            const int b = m / s.P, p = m - b * s.P;
#pragma unroll
            for (int ob = 0; ob < OB; ob++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int ol = otile * NT + wave_o * 64 + ob * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (ol < s.og) {
                        const int o = wg * s.og + ol;
                        float v = acc[ob][pb][r];
                        if (a.outacc) {
                            atomicAdd(a.outacc + ((long)b * s.Cout + o) * s.P + p, v);
                        } else {
                            if (bias) v += elem_to_f32<T>(bias[o]);
                            out[((long)b * s.Cout + o) * s.P + p] = f32_to_elem<T>(v);
                        }
                    }
                }
            }
        }
    }
}

constexpr size_t kFwdDmaLds = (size_t)2 * kDMT * kRawPos + (size_t)2 * kDMT * kRS + (size_t)3 * 10 * kDMT * 4;

template <typename T, bool AUX16, int WO, int WP>
int launch_fwd_dma(const FwdArgs &a, hipStream_t st)
{
    const int ntile = (a.s.M + kDMT - 1) / kDMT;
    const int NT = 64 * WO;
    if (hipFuncSetAttribute((const void *)tiled_fwd_dma_kernel<T, AUX16, WO, WP>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
        return d2c_check_launch("hipFuncSetAttribute(tiled_fwd_dma_kernel)");
    dim3 grid(ntile, a.s.ogp / NT * a.nsplit, a.s.groups);
    D2cProfScope prof(D2C_PROF_FWD, st);
    hipLaunchKernelGGL((tiled_fwd_dma_kernel<T, AUX16, WO, WP>), grid, dim3(kThreads + 64), kFwdDmaLds, st, a);
    return d2c_check_launch("tiled_fwd_dma_kernel");
}

// out = outacc + bias, in the element type of the output
template <typename T>
__global__ void __launch_bounds__(256) fwd_finish_kernel(const float *acc, const T *bias, T *out, int Cout, int P, long n)
{
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        float v = acc[i];
        if (bias) v += elem_to_f32<T>(bias[(i / P) % Cout]);
        out[i] = f32_to_elem<T>(v);
    }
}

template <typename T, bool AUX16, int MT, int WO, int WP>
int launch_fwd(const FwdArgs &a, hipStream_t st)
{
    const int ntile = (a.s.M + MT - 1) / MT;
    const int NT = 64 * WO;
    dim3 grid(ntile, a.s.ogp / NT * a.nsplit, a.s.groups);
    D2cProfScope prof(D2C_PROF_FWD, st);
    hipLaunchKernelGGL((tiled_fwd_kernel<T, AUX16, MT, WO, WP>), grid, dim3(kThreads), 0, st, a);
    return d2c_check_launch("tiled_fwd_kernel");
}

template <typename T, bool AUX16>
int launch_fwd_cfg(const FwdArgs &a, int nt, hipStream_t st)
{
    switch (nt) {
    case 512: return launch_fwd<T, AUX16, kMT, 8, 1>(a, st);
    case 256: return launch_fwd<T, AUX16, kMT, 4, 2>(a, st);
    case 128: return launch_fwd<T, AUX16, kMT, 2, 4>(a, st);
    default: return launch_fwd<T, AUX16, kMT, 1, 4>(a, st);
    }
}

}  // namespace

// Wide weight groups on problems with enough position tiles run the DMA-gather kernel (64-position tiles, all
// 512 output channels per workgroup); everything else the register-gather kernel (128-position tiles).
bool d2c_fwd_use_dma(int og, int M, int groups) { return og > 256 && (long)((M + kDMT - 1) / kDMT) * groups >= 128; }

int d2c_fwd_pos_tile(int og, int M, int groups) { return d2c_fwd_use_dma(og, M, groups) ? kDMT : kMT; }

// Output channels per workgroup: as wide as the weight group needs (the sampled
// tile is then produced once), but narrower when there are too few position
// tiles to occupy the chip.
int d2c_fwd_out_tile(int og, int M, int groups)
{
    if (d2c_fwd_use_dma(og, M, groups)) return 512;
    int nt = og > 256 ? 512 : (og > 128 ? 256 : (og > 64 ? 128 : 64));
    const int ntile = (M + kMT - 1) / kMT;
    while (nt > 64 && ntile * ((og + nt - 1) / nt) < 128) nt >>= 1;
    return nt;
}

// Workgroups per (position tile, output tile): 1 when the tiles alone fill the chip.
int d2c_fwd_split(const TiledShape &s)
{
    const int mt = d2c_fwd_pos_tile(s.og, s.M, s.groups), nt = d2c_fwd_out_tile(s.og, s.M, s.groups);
    const long wgs = (long)((s.M + mt - 1) / mt) * (s.ogp / nt) * s.groups;
    if (wgs >= 128) return 1;
    const int S = s.nchunk * s.K;
    const long want = (256 + wgs - 1) / wgs;
    return (int)(want < S ? want : S);
}

template <typename T>
int d2c_tiled_fwd_launch(const TiledShape &s, const void *xcl, const void *off, const void *mask, const void *wp,
                         const void *bias, void *out, float *outacc, hipStream_t st)
{
    const int nsplit = outacc ? d2c_fwd_split(s) : 1;
    const long n = (long)s.N * s.Cout * s.P;
    // the channels-last input is followed by a row of zeros (see forward_t)
    const unsigned zrow = (unsigned)((size_t)s.N * s.vol * s.Cin * sizeof(T));
    FwdArgs a{s, xcl, off, mask, wp, bias, out, nsplit > 1 ? outacc : nullptr, nsplit, zrow};
    if (nsplit > 1) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        d2c_fill_zero(outacc, (size_t)n * sizeof(float), st);
    }
    const int nt = d2c_fwd_out_tile(s.og, s.M, s.groups);
    const bool dma = d2c_fwd_use_dma(s.og, s.M, s.groups);
    int rc;
    bool aux16 = false;
    if constexpr (sizeof(T) == 2) aux16 = s.adt == D2C_BF16;
    if (dma) {
        if constexpr (sizeof(T) == 2) {
            if (aux16) rc = launch_fwd_dma<T, true, 8, 1>(a, st);
        }
        if (!aux16) rc = launch_fwd_dma<T, false, 8, 1>(a, st);
    } else {
        if constexpr (sizeof(T) == 2) {
            if (aux16) rc = launch_fwd_cfg<T, true>(a, nt, st);
        }
        if (!aux16) rc = launch_fwd_cfg<T, false>(a, nt, st);
    }
    if (rc || nsplit == 1) return rc;
    long g = (n + 255) / 256;
    if (g > 8192) g = 8192;
    D2cProfScope prof(D2C_PROF_PACK, st);
    hipLaunchKernelGGL(fwd_finish_kernel<T>, dim3((unsigned)g), dim3(256), 0, st, outacc, (const T *)bias, (T *)out,
                       s.Cout, s.P, n);
    return d2c_check_launch("fwd_finish_kernel");
}
template int d2c_tiled_fwd_launch<bf16_t>(const TiledShape &, const void *, const void *, const void *, const void *,
                                          const void *, void *, float *, hipStream_t);
template int d2c_tiled_fwd_launch<float>(const TiledShape &, const void *, const void *, const void *, const void *,
                                         const void *, void *, float *, hipStream_t);
