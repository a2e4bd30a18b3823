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
    // Schedule of the DMA-gather kernel, whose workgroups are persistent (one per compute unit).  A work item is
    // one (position tile, output tile, weight group) with all its steps.  Items [0, sk_full) are dealt whole,
    // round-robin.  The remaining items, fewer than one round, have their steps cut into sk_cut equal ranges;
    // the (range, item) pieces are dealt round-robin in range-major order, so that the workgroups running at
    // one time are at about the same steps and share their weight fragments in L2.  The pieces add into
    // `outacc`, here laid out [item - sk_full][output channel of the tile][position of the tile].
    int sk_items, sk_full, sk_ntile, sk_otiles, sk_cut;
    // Statistics for a normalisation behind the convolution (GroupNorm), or NULL: the sum and the sum of squares of
    // the values as stored, per position tile and output channel, fp32 [position tile][2][Cout][2] -- a tile of 64
    // positions lies in one sample or straddles two (slot 0: the sample of its first position, slot 1: the next
    // one); every entry has exactly one writer (no atomics: they would all land on the same few cache lines), and
    // stats_reduce_kernel adds the tiles of a sample up.  Filled by the DMA-gather kernel and its finishing kernel.
    float *stats;
    // The sampled, modulated columns kept for the backward pass (or NULL): what the matrix step multiplies with the
    // weights, [chunk][tap][col_rows][BKC] in the element type, col_rows = position tiles x 64 (zeros past the last
    // position) -- the layout tiled_bwd_weight_col_kernel reads.  Written by the DMA-gather kernel.
    void *col;
    long col_rows;
};

// Tiles that are neighbours in space go to the same XCD (workgroups are dealt
// round-robin over the 8 XCDs), so that its L2 sees a compact part of the input.
D2C_DEV int xcd_swizzle(int bid, int n)
{
    const int x = bid & 7, idx = bid >> 3;
    const int q = n >> 3, r = n & 7;
    return x * q + (x < r ? x : r) + idx;
}

template <typename T, bool AUX16, int MT, int WAVES_O, int WAVES_P, bool SIZED>
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
            tap_offsets_issue<AUX16, SIZED>(s, a.off, cb, g, k, cp, craw);
            craw[3] = a.mask ? ld_auxT<AUX16>(a.mask, mask_index(s, cb, g, k, cp)) : 1.f;
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
                tap_offsets_finish<AUX16, SIZED>(s, k, craw);
                const Tap3<float> t = tiled_tap3(s, bz, by, bx, craw[0], craw[1], craw[2]);
                live = t.live;
                idx = (cb * s.vol + (t.z0 * s.H + t.y0) * s.W + t.x0) * s.Cin;   // element offset of corner 000
                typedef typename std::conditional<AUX16, bf16_t, float>::type AT;
                const float al = (s.mact && a.mask) ? mask_act<AT>(s.mact, craw[3]) : craw[3];
#pragma unroll
                for (int c = 0; c < 8; c++) w[c] = ((live >> c) & 1u) ? tap3_weight(t, c) * al : 0.f;
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
                for (int pb = 0; pb < PB; pb++) mma_kgroup<T, kF32SplitFwd>(acc[ob][pb], af[kg][ob], bf[pb]);
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
    if (mma_wave && a.stats && !a.outacc) {
        // the same stores, and on the way the sum and the sum of squares of the stored values per (sample, output
        // channel), added into the [N][Cout][2] result (zeroed by the launcher): the 32 lanes that hold the positions
        // of a channel add up first when they lie in one sample (they nearly always do), so that one lane adds
        T *out = reinterpret_cast<T *>(a.out);
        const T *bias = reinterpret_cast<const T *>(a.bias);
#pragma unroll
        for (int pb = 0; pb < PB; pb++) {
            const int m = m0 + wave_p * WPOS + pb * 32 + (lane & 31);
            const bool ok = m < s.M;
            const int b = ok ? m / s.P : -1, p = ok ? m - b * s.P : 0;
            const int b0 = __shfl(b, lane & 32, 64);                    // sample of the half's first position
            const unsigned long long odd = __ballot(ok && b != b0);
            const bool uniform = ((odd >> (lane & 32)) & 0xffffffffull) == 0ull;
#pragma unroll
            for (int ob = 0; ob < OB; ob++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int ol = otile * NT + wave_o * 64 + ob * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    const bool live = ok && ol < s.og;                  // (ol is uniform over the half)
                    const int o = wg * s.og + ol;
                    float fv = 0.f;
                    if (live) {
                        float v = acc[ob][pb][r];
                        if (bias) v += elem_to_f32<T>(bias[o]);
                        const T sv = f32_to_elem<T>(d2c_epilogue(v, s.act, s.act_scale));
                        out[((long)b * s.Cout + o) * s.P + p] = sv;
                        fv = elem_to_f32<T>(sv);
                    }
                    if (ol >= s.og) continue;
                    if (uniform) {
                        float q0 = fv, q1 = fv * fv;
#pragma unroll
                        for (int d = 1; d < 32; d <<= 1) { q0 += __shfl_xor(q0, d, 64); q1 += __shfl_xor(q1, d, 64); }
                        if ((lane & 31) == 0 && b0 >= 0) {
                            atomicAdd(a.stats + ((long)b0 * s.Cout + o) * 2, q0);
                            atomicAdd(a.stats + ((long)b0 * s.Cout + o) * 2 + 1, q1);
                        }
                    } else if (live) {
                        atomicAdd(a.stats + ((long)b * s.Cout + o) * 2, fv);
                        atomicAdd(a.stats + ((long)b * s.Cout + o) * 2 + 1, fv * fv);
                    }
                }
            }
        }
    } else if (mma_wave) {
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
                            out[((long)b * s.Cout + o) * s.P + p] = f32_to_elem<T>(d2c_epilogue(v, s.act, s.act_scale));
                        }
                    }
                }
            }
        }
    }
}


// ---------------------------------------------------------------------------
// The same forward pass with the corner rows moved global -> LDS by DMA loads
// (global_load_lds_dwordx4: no staging registers; the rows of step s+2 are
// requested during the matrix-core phase of iteration s, a few requests
// between each pair of MFMAs, and are in flight over the interpolation of
// step s+1 and the barrier).
// One workgroup = 512 + 64 threads = 64 positions x NT output channels.  One DMA
// instruction of a wavefront fetches the 8 corner rows (8 x 128 bytes) of one
// position: lane = (corner, 16-byte vector); corners that are out of range or
// cut off by the early-out read a row of zeros instead.
//
// Workgroups are persistent: each walks a list of segments (a work item and a
// range of its steps, see FwdArgs) as ONE sequence of steps, so that the
// pipeline stays full from one segment into the next; only the matrix-core
// wavefronts notice a segment's end (they store or add their accumulators).
constexpr int kDMT = 64;                   // positions per workgroup

// Workgroup barrier that waits for this wavefront's LDS operations only: its global loads and DMA transfers
// stay in flight across it (a __syncthreads() would wait for them as well).
D2C_DEV void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

constexpr int kMaxSeg = 128;               // segments per workgroup (the launcher sizes the grid for this)

// A position in the step sequence of a workgroup.  The segments are listed in LDS once, at the start; all
// fields are uniform over the workgroup and live in scalar registers.
//
// Step order within a work item: offset group (outer), tap, chunk of that offset group (inner), so that the chunks
// that share the sampling points of a (group, tap) follow each other and the coordinate wavefront computes a table
// once for all of them.  The walker counts chunk, tap and group along (no division per step).
struct SegWalk {
    int seg;                      // index of the current segment
    int item;                     // its work item, -1 past the end of the sequence
    int st, st_hi;                // current step, end of the current segment
    int tile, otile, wg;          // the item's position tile, output tile, weight group
    int j, k, g;                  // the step's chunk within the weight group, tap, offset group
    int jj;                       // chunk within the offset group
    bool fresh;                   // first step of its (group, tap) in this segment: sampling points not seen yet
};
D2C_DEV void seg_load(SegWalk &w, const int4 *s_seg, int nseg, const TiledShape &s)
{
    if (w.seg < nseg) {
        const int4 u = s_seg[2 * w.seg], v = s_seg[2 * w.seg + 1];
        w.item = __builtin_amdgcn_readfirstlane(u.x);
        w.st = __builtin_amdgcn_readfirstlane(u.y);
        w.st_hi = __builtin_amdgcn_readfirstlane(u.z);
        w.tile = __builtin_amdgcn_readfirstlane(v.x);
        w.otile = __builtin_amdgcn_readfirstlane(v.y);
        w.wg = __builtin_amdgcn_readfirstlane(v.z);
        const int t = w.st / s.cpc, gi = t / s.K;
        w.jj = w.st - t * s.cpc;
        w.k = t - gi * s.K;
        w.j = gi * s.cpc + w.jj;
        w.g = (w.wg * s.cg + w.j * s.bkc) / s.cpg;
    } else {
        w.item = -1; w.st = 0; w.st_hi = 0x7fffffff;
        w.j = 0; w.k = 0; w.g = 0; w.jj = 0;
    }
    w.fresh = true;
}
// one step on; true when that entered a new segment
D2C_DEV bool seg_advance(SegWalk &w, const int4 *s_seg, int nseg, const TiledShape &s)
{
    if (++w.st < w.st_hi) {
        if (++w.jj < s.cpc) {
            w.j++; w.fresh = false;
        } else {
            w.jj = 0; w.fresh = true;
            if (++w.k < s.K) w.j -= s.cpc - 1;
            else { w.k = 0; w.j++; w.g++; }
        }
        return false;
    }
    w.seg++;
    seg_load(w, s_seg, nseg, s);
    return true;
}

// (The LDS regions are passed as restrict-qualified pointers: that gives their accesses alias scopes, without
// which the compiler makes every LDS store wait for all DMA transfers in flight, whatever region they fill.)
// NC: corner rows fetched and interpolated per sampling point: 8, or 4 / 2 when offsets along one / two axes are fixed
// (TiledShape::axes; the corners on the far side of a fixed axis have weight zero and no slot at all).
template <typename T, bool AUX16, int WAVES_O, int WAVES_P, bool SIZED, int NC, bool COLS>
D2C_DEV void fwd_dma_body(const FwdArgs &a, unsigned char *__restrict__ s_raw, unsigned char *__restrict__ s_tile,
                          float *__restrict__ s_w, int2 *__restrict__ s_if,
                          int *__restrict__ s_meta, int4 *__restrict__ s_seg)
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
    constexpr int RAWPOS = NC * kNV * 16;   // raw bytes per position
    constexpr int PPI = 8 / NC;             // positions per DMA instruction

    const TiledShape &s = a.s;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int S = s.nchunk * s.K;
    const int OBT = s.ogp / 32;
    const int dzc = s.H * s.W * s.Cin, dyc = s.W * s.Cin;

    // --- the step sequence of this workgroup: its whole items, then its pieces of the last round's items
    const int nwg = (int)gridDim.x;
    const int bid = xcd_swizzle(blockIdx.x, nwg);
    const int ntail = a.sk_items - a.sk_full, npiece = ntail * a.sk_cut;
    const int nwhole_mine = bid < a.sk_full ? (a.sk_full - bid + nwg - 1) / nwg : 0;
    const int npiece_mine = bid < npiece ? (npiece - bid + nwg - 1) / nwg : 0;
    const int nseg = nwhole_mine + npiece_mine;        // <= kMaxSeg
    if (nseg == 0) return;
    if (tid < nseg) {
        int item, lo, hi;
        if (tid < nwhole_mine) {
            item = bid + tid * nwg; lo = 0; hi = S;
        } else {
            const int piece = bid + (tid - nwhole_mine) * nwg, range = piece / ntail;
            item = a.sk_full + (piece - range * ntail);
            lo = (int)((long)S * range / a.sk_cut);
            hi = (int)((long)S * (range + 1) / a.sk_cut);
        }
        s_seg[2 * tid] = make_int4(item, lo, hi, 0);
        s_seg[2 * tid + 1] = make_int4(item % a.sk_ntile, (item / a.sk_ntile) % a.sk_otiles,
                                       item / (a.sk_ntile * a.sk_otiles), 0);
    }
    __syncthreads();
    int total = 0;
    for (int q = 0; q < nseg; q++) total += __builtin_amdgcn_readfirstlane(s_seg[2 * q].z - s_seg[2 * q].y);
    SegWalk w0;
    w0.seg = 0;
    seg_load(w0, s_seg, nseg, s);

    // --- coordinates: a ninth wavefront (one position per lane) that does nothing else, so that this
    // arithmetic runs beside the work of the other eight instead of in front of their barrier
    const bool cwave = wave == 8;        // coordinates
    const bool worker = wave < 8;
    const int ctid = tid - kThreads;
    // The lane's position within a work item.  Offsets are requested (issue) one iteration before they are
    // turned into a table row (finish).
    // (size-map source: the part of the offsets that the taps of a position share, size - 1 per axis, is formed
    // here once per work item; a step then costs three multiplications and no load)
    typedef typename std::conditional<AUX16, bf16_t, float>::type AT;
    const CoordConst cc = coord_const(s);
    const int ncomp = s.nd == 3 ? 3 : 1;                               // offset components per tap
    const long cstride = s.nd == 3 ? (long)s.P * (long)sizeof(AT) : 0;
    const long off_tap = (long)ncomp * s.P * (long)sizeof(AT);         // bytes per (sample, group, tap) of the offsets
    const long mask_tap = (long)s.P * (long)sizeof(AT);                // ... of the mask
    // Lane l of the coordinate wavefront keeps the constants of tap l (taps 64 and up are computed when met):
    // where the tap sits in the kernel, as float, and for the size-map source its kernel-grid coordinates.
    float tap_z = 0.f, tap_y = 0.f, tap_x = 0.f, tap_bz = 0.f, tap_by = 0.f, tap_bx = 0.f;
    auto tap_consts = [&](int k, float &tz, float &ty, float &tx, float &bz, float &by, float &bx) {
        const int kx = k % s.geo.kw, ky = (k / s.geo.kw) % s.geo.kh, kz = k / (s.geo.kw * s.geo.kh);
        tz = (float)(kz * s.geo.dd); ty = (float)(ky * s.geo.dh); tx = (float)(kx * s.geo.dw);
        if constexpr (SIZED) {
            bz = rnd<AT>(s.ss.base[0][kz]); by = rnd<AT>(s.ss.base[1][ky]); bx = rnd<AT>(s.ss.base[2][kx]);
        }
    };
    if (cwave && ctid < s.K) tap_consts(ctid, tap_z, tap_y, tap_x, tap_bz, tap_by, tap_bx);
    struct PosC {
        float fz, fy, fx;          // o * stride - pad per axis, as float
        int vox0;                  // voxel index of the sample's origin
        unsigned aoff, moff;       // byte offsets of (sample - first sample of the tile, position) in offsets / mask
        bool valid;
        float s0, s1, s2;
    };
    const char *off_item = nullptr, *mask_item = nullptr;      // uniform: the tile's first sample
    auto pos_of = [&](const SegWalk &w) {
        PosC c{0.f, 0.f, 0.f, 0, 0u, 0u, false, 0.f, 0.f, 0.f};
        const int m0 = w.item >= 0 ? w.tile * MT : 0;
        const int b_lo = fdiv(m0, s.dP);
        off_item = reinterpret_cast<const char *>(a.off) + (long)b_lo * s.obs * (long)sizeof(AT);
        mask_item = reinterpret_cast<const char *>(a.mask) + (long)b_lo * s.mbs * (long)sizeof(AT);
        const int m = m0 + ctid;
        c.valid = w.item >= 0 && m < s.M;
        if (c.valid) {
            const int b = fdiv(m, s.dP), p = m - b * s.P;
            const int oz = fdiv(p, s.dHW), rem = p - oz * (s.Wo * s.Ho);
            const int oy = fdiv(rem, s.dW), ox = rem - oy * s.Wo;
            c.fz = (float)(oz * s.geo.sd - s.geo.pd);
            c.fy = (float)(oy * s.geo.sh - s.geo.ph);
            c.fx = (float)(ox * s.geo.sw - s.geo.pw);
            c.vox0 = b * s.vol;
            // (a lane without a position keeps offset 0: its loads read the tile's first position)
            c.aoff = (unsigned)(b - b_lo) * ((unsigned)s.obs * (unsigned)sizeof(AT)) + (unsigned)p * (unsigned)sizeof(AT);
            c.moff = (unsigned)(b - b_lo) * ((unsigned)s.mbs * (unsigned)sizeof(AT)) + (unsigned)p * (unsigned)sizeof(AT);
            if (SIZED && cwave) {
                float t[3];
                tap_offsets_issue<AUX16, true>(s, a.off, b, 0, 0, p, t);
                size_minus_one<AUX16>(s, t);
                c.s0 = t[0]; c.s1 = t[1]; c.s2 = t[2];
            }
        }
        return c;
    };
    float craw[4] = {0.f, 0.f, 0.f, 1.f};
    auto coords_issue = [&](const SegWalk &w, const PosC &c) {
        if (cwave && w.fresh) {
            const int gk = w.g * s.K + w.k;
            if constexpr (!SIZED) coord_offsets_issue<AUX16>(off_item + gk * off_tap, cstride, c.aoff, craw);
            if (a.mask) craw[3] = ld_aux_at<AUX16>(mask_item + gk * mask_tap, c.moff);
        }
    };
    auto coords_finish = [&](const SegWalk &w, const PosC &c, int buf) {
        if (cwave && !w.fresh) {
            // same sampling points as the step before (another chunk of the offset group): its table, copied
            const int pbuf = (buf + 2) % 3;
#pragma unroll
            for (int q = 0; q < 8; q++) s_w[(buf * 8 + q) * MT + ctid] = s_w[(pbuf * 8 + q) * MT + ctid];
            s_if[buf * MT + ctid] = s_if[pbuf * MT + ctid];
        } else if (cwave) {
            float tz, ty, tx, bz = 0.f, by = 0.f, bx = 0.f;
            if (w.k < 64) {
                tz = lane_value(tap_z, w.k);
                ty = lane_value(tap_y, w.k);
                tx = lane_value(tap_x, w.k);
                if constexpr (SIZED) {
                    bz = lane_value(tap_bz, w.k);
                    by = lane_value(tap_by, w.k);
                    bx = lane_value(tap_bx, w.k);
                }
            } else {
                tap_consts(w.k, tz, ty, tx, bz, by, bx);
            }
            if constexpr (SIZED) {
                craw[0] = rnd<AT>(bz * c.s0); craw[1] = rnd<AT>(by * c.s1); craw[2] = rnd<AT>(bx * c.s2);
            }
            coord_offsets_select(cc, craw);
            if (s.mact && a.mask) craw[3] = mask_act<AT>(s.mact, craw[3]);
            const CornerRow r = corner_row(cc, (c.fz + tz) + craw[0], (c.fy + ty) + craw[1], (c.fx + tx) + craw[2],
                                           craw[3], c.vox0, c.valid);
#pragma unroll
            for (int q = 0; q < 8; q++) s_w[(buf * 8 + q) * MT + ctid] = r.w[q];
            s_if[buf * MT + ctid] = make_int2(r.idx, (int)r.live);
        }
        // what the workers need to know of the step: its first input channel and where its weight fragments start
        // (they walk no step sequence of their own)
        if (cwave && ctid == 0) {
            s_meta[buf * 4] = w.wg * s.cg + w.j * BKC;
            s_meta[buf * 4 + 1] = (w.wg * S + w.j * s.K + w.k) * OBT + w.otile * (NT / 32);
            // COLS: the row of the column buffer where this step's tile goes (the first output tile writes it)
            if constexpr (COLS)
                s_meta[buf * 4 + 2] = w.otile == 0 ? (int)((((long)(w.wg * s.nchunk + w.j)) * s.K + w.k) * a.col_rows) + w.tile * MT
                                                   : -1;
        }
    };
    // a table that fetches rows of zeros: steps past the end of a sequence shorter than the pipeline
    auto coords_none = [&](int buf) {
        if (cwave) {
#pragma unroll
            for (int q = 0; q < 8; q++) s_w[(buf * 8 + q) * MT + ctid] = 0.f;
            s_if[buf * MT + ctid] = make_int2(0, 0);
            if (ctid == 0) { s_meta[buf * 4] = 0; s_meta[buf * 4 + 1] = 0; s_meta[buf * 4 + 2] = -1; }
        }
    };

    // --- corner rows of a step -> s_raw[rbuf]: worker wavefront w requests positions 8w .. 8w+7, one
    // instruction per position, lane = (corner, 16-byte vector)
    // (with fewer than 8 corners an instruction covers 8 / NC positions: lane = (position, corner slot, vector); slot j
    // is the corner whose bits are those of j spread over the free axes)
    const int dslot = (lane >> 3) % NC, dsub = (lane >> 3) / NC, dvec = lane & 7;
    const int dcorner = NC == 8 ? dslot : corner_of_slot(dslot, s.axes);
    const int dcoff = ((dcorner >> 2) & 1) * dzc + ((dcorner >> 1) & 1) * dyc + (dcorner & 1) * s.Cin;
    // one request: the rows of position(s) wave * 8 + i * PPI (+ dsub); `vidx` / `vflag` hold the table entries of the
    // wavefront's 8 positions (lane i: position i)
    auto dma_request = [&](int i, int vidx, int vflag, int c0, int rbuf) {
        const char *base = reinterpret_cast<const char *>(a.xcl);
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
                               : a.zrow + (unsigned)dvec * 16u;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(base + o),
                                         (__attribute__((address_space(3))) void *)(s_raw + (rbuf * MT + pos0) * RAWPOS),
                                         16, 0, 0);
    };
    // (past the end of the sequence the tables are those of three steps before, or the ones of coords_none: the
    // same number of transfers in every iteration, which lets the compiler count the loads in flight instead of
    // waiting for all)
    auto dma_issue = [&](int rbuf, int tbuf) {
        if (!worker) return;
        const int c0 = __builtin_amdgcn_readfirstlane(s_meta[tbuf * 4]);
        // table entries of this wavefront's 8 positions: one LDS read (lane i holds position i), then
        // lane-indexed moves to scalar registers
        const int2 vif = s_if[tbuf * MT + wave * (MT / 8) + (lane & 7)];
#pragma unroll
        for (int i = 0; i < MT / 8 / PPI; i++) dma_request(i, vif.x, vif.y, c0, rbuf);
    };
    // --- interpolation: thread = (position, 16-byte vector)
    const int ipos = tid >> 3, ivec = tid & 7;
    int wslot[NC];      // row of the weight table that belongs to corner slot c
#pragma unroll
    for (int c = 0; c < NC; c++) wslot[c] = (NC == 8 ? c : corner_of_slot(c, s.axes)) * MT;
    // (the rows are read behind the compiler's back, see lds_row_read: the transfers requested during the matrix
    // step, for the step after the one interpolated here, stay in flight; `between(c)` runs after corner slot c)
    auto interp_rows = [&](int rbuf, int tbuf, auto between) {
        const unsigned rp = lds_address(s_raw + (rbuf * MT + ipos) * RAWPOS + ivec * 16);
        VecAcc<T> va;
        va.zero();
        if constexpr (NC == 2) {
            u32x4_t r0 = lds_row_read<0>(rp), r1 = lds_row_read<kNV * 16>(rp);
            const float w0 = s_w[tbuf * 8 * MT + wslot[0] + ipos], w1 = s_w[tbuf * 8 * MT + wslot[1] + ipos];
            lds_rows_wait(r0, r1);
            va.fma(w0, __builtin_bit_cast(uint4, r0));
            between(0);
            va.fma(w1, __builtin_bit_cast(uint4, r1));
            between(1);
        } else {
#pragma unroll
            for (int h = 0; h < NC / 4; h++) {
                constexpr int R = kNV * 16;
                u32x4_t r0 = h ? lds_row_read<4 * R>(rp) : lds_row_read<0>(rp);
                u32x4_t r1 = h ? lds_row_read<5 * R>(rp) : lds_row_read<R>(rp);
                u32x4_t r2 = h ? lds_row_read<6 * R>(rp) : lds_row_read<2 * R>(rp);
                u32x4_t r3 = h ? lds_row_read<7 * R>(rp) : lds_row_read<3 * R>(rp);
                float w[4];
#pragma unroll
                for (int c = 0; c < 4; c++) w[c] = s_w[tbuf * 8 * MT + wslot[h * 4 + c] + ipos];
                lds_rows_wait(r0, r1, r2, r3);
                va.fma(w[0], __builtin_bit_cast(uint4, r0));
                between(h * 4);
                va.fma(w[1], __builtin_bit_cast(uint4, r1));
                between(h * 4 + 1);
                va.fma(w[2], __builtin_bit_cast(uint4, r2));
                between(h * 4 + 2);
                va.fma(w[3], __builtin_bit_cast(uint4, r3));
                between(h * 4 + 3);
            }
        }
        return va;
    };
    // COLS: the tile of a step also goes to the column buffer, one 16-byte streaming store per thread.  It is kept
    // for one step and issued in the matrix step of the next iteration, behind that step's last row request
    // (col_flush): it then has most of a step to complete before the wait at the top of the iteration comes round
    // again (that wait counts stores as well as loads), and meets the vector-memory path when the row requests are
    // out (N=2, C=512, 8x30x54: kernel +10 % with the store right behind the wait, +6 % in front of the
    // interpolation, +4 % here; as a plain instead of a streaming store +26 %).
    typedef unsigned u32x4_c __attribute__((ext_vector_type(4)));
    u32x4_c col_v = {0u, 0u, 0u, 0u};
    int col_row = -1;                                  // (wavefront-uniform)
    // (float: the interpolated values themselves, not the two-term operand form the matrix step reads)
    auto col_keep = [&](const VecAcc<T> &va, const uint4 &v, int tbuf) {
        if constexpr (COLS) {
            if constexpr (sizeof(T) == 4)
                col_v = u32x4_c{__float_as_uint(va.a[0]), __float_as_uint(va.a[1]), __float_as_uint(va.a[2]),
                                __float_as_uint(va.a[3])};
            else col_v = u32x4_c{v.x, v.y, v.z, v.w};
            col_row = __builtin_amdgcn_readfirstlane(s_meta[tbuf * 4 + 2]);
        }
    };
    auto col_flush = [&]() {
        if constexpr (COLS) {
            // (a thread's 16 bytes of its tile: position tid / 8, vector tid % 8 of a 128-byte row)
            if (col_row >= 0)
                __builtin_nontemporal_store(col_v, reinterpret_cast<u32x4_c *>(reinterpret_cast<char *>(a.col)
                                                       + (long)col_row * (BKC * (long)sizeof(T)) + tid * 16));
        }
    };
    auto interp_store = [&](int rbuf, int tbuf, int dbuf) {
        if (!worker) return;
        VecAcc<T> va = interp_rows(rbuf, tbuf, [](int) {});
        const uint4 v = va.pack();
        *reinterpret_cast<uint4 *>(s_tile + (dbuf * MT + ipos) * kRS + ivec * 16) = v;
        col_keep(va, v, tbuf);
    };

    // --- MMA role
    const bool mma_wave = wave < WAVES_O * WAVES_P;
    const int wave_o = wave % WAVES_O, wave_p = wave / WAVES_O;
    f32x16 acc[OB][PB];
#pragma unroll
    for (int ob = 0; ob < OB; ob++)
#pragma unroll
        for (int pb = 0; pb < PB; pb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[ob][pb][r] = 0.f;
    const uint4 *wp4 = reinterpret_cast<const uint4 *>(a.wp);
    uint4 af[NKG][OB];
    // (wstep: the table's entry for the step; past the end of the sequence a stale one, the fragments are not used)
    auto wfrag = [&](int wstep, int kg, int ob) {
        const long wbase = ((long)wstep + wave_o * OB) * NKG * 64 + lane;
        return wp4[wbase + ((long)ob * NKG + kg) * 64];
    };
    // The vector-memory path of a CU takes one request of a wavefront at a time (1 KiB = 16 clocks) and a wavefront
    // stalls at issue while the path is busy: requests issued back to back serialise with everything else the
    // wavefront does.  So they are spread over the iteration: the DMA requests of step it+2 between the MFMAs of
    // step it (in its first half, so that they have landed when the interpolation starts), the weight-fragment
    // loads of step it+1 between the corners of the interpolation.
    static_assert(WAVES_O * WAVES_P == 8 && NKG * OB == 8, "all workers are matrix wavefronts; a fragment per corner");
    auto mma_dma_step = [&](int dbuf, int rbuf, int tbuf) {
        const unsigned char *tb = s_tile + (dbuf * MT + wave_p * WPOS + (lane & 31)) * kRS + (lane >> 5) * 16;
        const int c0 = __builtin_amdgcn_readfirstlane(s_meta[tbuf * 4]);
        // table entries of this wavefront's 8 positions: one LDS read (lane i holds position i), then
        // lane-indexed moves to scalar registers
        const int2 vif = s_if[tbuf * MT + wave * (MT / 8) + (lane & 7)];
        constexpr int DPK = 4;                                // requests per k-group
#pragma unroll
        for (int kg = 0; kg < NKG; kg++) {
            uint4 bf[PB];
#pragma unroll
            for (int pb = 0; pb < PB; pb++)
                bf[pb] = *reinterpret_cast<const uint4 *>(tb + pb * 32 * kRS + kg * 32);
#pragma unroll
            for (int ob = 0; ob < OB; ob++)
#pragma unroll
                for (int pb = 0; pb < PB; pb++) mma_kgroup<T, kF32SplitFwd>(acc[ob][pb], af[kg][ob], bf[pb]);
#pragma unroll
            for (int q = 0; q < DPK; q++) {
                const int i = kg * DPK + q;
                if (i >= MT / 8 / PPI) break;
                dma_request(i, vif.x, vif.y, c0, rbuf);
            }
            // (the kept columns of this step's tile: behind the last row requests, while matrix instructions remain)
            if (kg == (MT / 8 / PPI + DPK - 1) / DPK) col_flush();
        }
    };
    // interpolation of one step; the weight fragments of that step are fetched on the way
    auto interp_wload_store = [&](int rbuf, int tbuf, int dbuf) {
        const int wstep = __builtin_amdgcn_readfirstlane(s_meta[tbuf * 4 + 1]);
        VecAcc<T> va = interp_rows(rbuf, tbuf, [&](int c) {
#pragma unroll
            for (int f = c * (8 / NC); f < (c + 1) * (8 / NC); f++) af[f / OB][f % OB] = wfrag(wstep, f / OB, f % OB);
        });
        const uint4 v = va.pack();
        *reinterpret_cast<uint4 *>(s_tile + (dbuf * MT + ipos) * kRS + ivec * 16) = v;
        col_keep(va, v, tbuf);
    };
    // end of a segment: whole items get bias, conversion and store; pieces of an item add into its fp32 tile
    auto flush_acc = [&](const SegWalk &w) {
        if (!mma_wave) return;
        // (an opaque copy of the lane number: the address arithmetic below depends on nothing else that changes
        // from step to step, and must not be computed ahead of the step loop and kept in registers)
        int elane = lane;
        asm volatile("" : "+v"(elane));
        const int ot0 = wave_o * 64 + 4 * (elane >> 5);      // first output channel of this lane within the tile
        const int nvalid = s.og - (w.otile * NT + ot0);       // channels from there on that exist
        const int o0 = w.wg * s.og + w.otile * NT + ot0;
        if (w.item >= a.sk_full) {
            float *tp = a.outacc + ((long)(w.item - a.sk_full) * NT + ot0) * MT + wave_p * WPOS + (elane & 31);
#pragma unroll
            for (int pb = 0; pb < PB; pb++)
#pragma unroll
                for (int ob = 0; ob < OB; ob++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int oo = ob * 32 + 8 * (r >> 2) + (r & 3);
                        if (oo < nvalid) atomicAdd(tp + oo * MT + pb * 32, acc[ob][pb][r]);
                        acc[ob][pb][r] = 0.f;
                    }
        } else if (a.stats) {
            // the same stores, and on the way the sum and the sum of squares of the stored values per output channel
            // and sample slot: over the positions a lane holds, then over the 32 lanes of its half
            const T *bias = reinterpret_cast<const T *>(a.bias);
            const int b_lo = (w.tile * MT) / s.P;
            bool okq[PB], hiq[PB];
            T *opq[PB];
#pragma unroll
            for (int pb = 0; pb < PB; pb++) {
                const int m = w.tile * MT + wave_p * WPOS + pb * 32 + (elane & 31);
                okq[pb] = m < s.M;
                const int b = m / s.P;
                hiq[pb] = b != b_lo;
                opq[pb] = reinterpret_cast<T *>(a.out) + ((long)b * s.Cout + o0) * s.P + (m - b * s.P);
            }
            float *sp = a.stats + ((long)w.tile * 2 * s.Cout + o0) * 2;
#pragma unroll
            for (int ob = 0; ob < OB; ob++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int oo = ob * 32 + 8 * (r >> 2) + (r & 3);
                    float q4[4] = {0.f, 0.f, 0.f, 0.f};     // slot 0: sum, sum of squares; slot 1 likewise
#pragma unroll
                    for (int pb = 0; pb < PB; pb++) {
                        if (okq[pb] && oo < nvalid) {
                            float v = acc[ob][pb][r];
                            if (bias) v += elem_to_f32<T>(bias[o0 + oo]);
                            const T sv = f32_to_elem<T>(d2c_epilogue(v, s.act, s.act_scale));
                            opq[pb][(long)oo * s.P] = sv;
                            const float fv = elem_to_f32<T>(sv);
                            q4[0] += hiq[pb] ? 0.f : fv; q4[1] += hiq[pb] ? 0.f : fv * fv;
                            q4[2] += hiq[pb] ? fv : 0.f; q4[3] += hiq[pb] ? fv * fv : 0.f;
                        }
                        acc[ob][pb][r] = 0.f;
                    }
#pragma unroll
                    for (int d = 1; d < 32; d <<= 1)
#pragma unroll
                        for (int i = 0; i < 4; i++) q4[i] += __shfl_xor(q4[i], d, 64);
                    if ((elane & 31) == 0 && oo < nvalid) {
                        if (WAVES_P == 1) {
                            sp[oo * 2] = q4[0]; sp[oo * 2 + 1] = q4[1];
                            sp[(s.Cout + oo) * 2] = q4[2]; sp[(s.Cout + oo) * 2 + 1] = q4[3];
                        } else {
                            // (several wavefronts share a channel's positions: the slots were zeroed)
                            atomicAdd(sp + oo * 2, q4[0]); atomicAdd(sp + oo * 2 + 1, q4[1]);
                            atomicAdd(sp + (s.Cout + oo) * 2, q4[2]); atomicAdd(sp + (s.Cout + oo) * 2 + 1, q4[3]);
                        }
                    }
                }
        } else {
            const T *bias = reinterpret_cast<const T *>(a.bias);
#pragma unroll
            for (int pb = 0; pb < PB; pb++) {
                const int m = w.tile * MT + wave_p * WPOS + pb * 32 + (elane & 31);
                const bool ok = m < s.M;
                const int b = m / s.P, p = m - b * s.P;
                T *op = reinterpret_cast<T *>(a.out) + ((long)b * s.Cout + o0) * s.P + p;
#pragma unroll
                for (int ob = 0; ob < OB; ob++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int oo = ob * 32 + 8 * (r >> 2) + (r & 3);
                        if (ok && oo < nvalid) {
                            float v = acc[ob][pb][r];
                            if (bias) v += elem_to_f32<T>(bias[o0 + oo]);
                            op[(long)oo * s.P] = f32_to_elem<T>(d2c_epilogue(v, s.act, s.act_scale));
                        }
                        acc[ob][pb][r] = 0.f;
                    }
            }
        }
    };

    // --- pipeline.  Iteration `it` of the step sequence: step it on the matrix cores with the rows of step it+2
    // requested on the way, step it+1 interpolated with its weight fragments requested on the way, coordinates
    // of step it+3 computed.  Corner tables rotate over 3 buffers,
    // raw rows and tiles over 2.  A wavefront interpolates the positions whose rows it requested itself, so the
    // rows need no barrier, only that wavefront's own wait.
    SegWalk wc = w0;                  // coordinates: the step whose table is computed next (its offsets are requested
                                      // one iteration before)
    PosC pc = pos_of(wc);
    for (int q = 0; q < 3; q++) {
        if (q < total) {
            coords_issue(wc, pc);
            coords_finish(wc, pc, q);
            if (seg_advance(wc, s_seg, nseg, s)) pc = pos_of(wc);
        } else {
            coords_none(q);
        }
    }
    SegWalk wm = w0;                  // the step on the matrix cores
    __syncthreads();
    if (mma_wave) {
        const int wstep = __builtin_amdgcn_readfirstlane(s_meta[1]);
#pragma unroll
        for (int kg = 0; kg < NKG; kg++)
#pragma unroll
            for (int ob = 0; ob < OB; ob++) af[kg][ob] = wfrag(wstep, kg, ob);
    }
    dma_issue(0, 0);
    dma_issue(1, 1);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    interp_store(0, 0, 0);
    if (3 < total) {
        coords_issue(wc, pc);
    }
    // One loop per role (separate register budgets), the same synchronisation point per iteration in each.
    if (worker) {
        // (one inner loop per segment, so that the code that stores the accumulators stays out of the loop
        // over steps; nothing but the accumulators knows where a segment ends)
        int it = 0;
        while (wm.item >= 0) {
            for (; wm.st < wm.st_hi; wm.st++, it++) {
                lds_barrier();
                // everything this wavefront has in flight is due: the weight fragments of this step (requested
                // during the last interpolation) and the rows of step it+1 (requested during the last matrix step)
                __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0)
                mma_dma_step(it & 1, it & 1, (it + 2) % 3);
                // (past the end of the sequence the interpolation works on stale rows into the tile nobody reads)
                interp_wload_store((it + 1) & 1, (it + 1) % 3, (it + 1) & 1);
            }
            flush_acc(wm);
            wm.seg++;
            seg_load(wm, s_seg, nseg, s);
        }
    } else {
        // (at default priority: with its short instruction sequence, issuing ahead of the two workers of its SIMD
        // costs 3 % on the 512-channel tile and gains nothing on the 256-channel one)
        for (int it = 0; it < total; it++) {
            lds_barrier();
            if (it + 3 < total) {                      // offsets requested one iteration ago
                coords_finish(wc, pc, it % 3);
                if (seg_advance(wc, s_seg, nseg, s)) pc = pos_of(wc);
            }
            if (it + 4 < total) {
                coords_issue(wc, pc);
            }
        }
    }
}

template <typename T, bool AUX16, int WAVES_O, int WAVES_P, bool SIZED, int NC, bool COLS = false>
__global__ void __launch_bounds__(kThreads + 64) tiled_fwd_dma_kernel(FwdArgs a)
{
    constexpr int MT = kDMT;
    // (separate arrays, not slices of one: the compiler then knows which of them a DMA transfer fills, and
    // lets accesses to the others go ahead while transfers are in flight)
    __shared__ __align__(16) unsigned char s_raw[2 * MT * NC * kNV * 16];   // [2][MT][NC corners][128 B]
    __shared__ __align__(16) unsigned char s_tile[2 * MT * kRS];      // [2][MT][kRS]
    __shared__ float s_w[3 * 8 * MT];                                 // [3][8][MT]
    __shared__ int2 s_if[3 * MT];                                     // [3][MT] (offset of corner 000, live corners)
    __shared__ int s_meta[3 * 4];                                     // [3][first channel, weight-fragment row]
    __shared__ int4 s_seg[2 * kMaxSeg];                               // [kMaxSeg][2]
    fwd_dma_body<T, AUX16, WAVES_O, WAVES_P, SIZED, NC, COLS>(a, s_raw, s_tile, s_w, s_if, s_meta, s_seg);
}

// out = fp32 tile + bias for the items whose steps were shared out (see FwdArgs).  One block = 32 output
// channels of one such item.
template <typename T>
__global__ void __launch_bounds__(256) fwd_dma_finish_kernel(FwdArgs a, int NT)
{
    constexpr int MT = kDMT;
    const TiledShape &s = a.s;
    const int item = a.sk_full + blockIdx.x;
    const int tile = item % a.sk_ntile, otile = (item / a.sk_ntile) % a.sk_otiles, wg = item / (a.sk_ntile * a.sk_otiles);
    const float *acc = a.outacc + (long)blockIdx.x * NT * MT;
    const T *bias = reinterpret_cast<const T *>(a.bias);
    T *out = reinterpret_cast<T *>(a.out);
    const int b_lo = (tile * MT) / s.P;
    static_assert(MT == 64, "one wavefront = the positions of one channel");
    for (int e = threadIdx.x; e < 32 * MT; e += 256) {
        const int ot = blockIdx.y * 32 + e / MT, pl = e % MT;
        const int ol = otile * NT + ot, m = tile * MT + pl;
        float fv = 0.f;
        const bool ok = ol < s.og && m < s.M;
        const int o = wg * s.og + ol, b = ok ? m / s.P : b_lo, p = m - b * s.P;
        if (ok) {
            float v = acc[(long)ot * MT + pl];
            if (bias) v += elem_to_f32<T>(bias[o]);
            const T sv = f32_to_elem<T>(d2c_epilogue(v, s.act, s.act_scale));
            out[((long)b * s.Cout + o) * s.P + p] = sv;
            fv = elem_to_f32<T>(sv);
        }
        if (a.stats) {
            // (e / MT is uniform over a wavefront: its 64 lanes are the positions of one channel)
            const bool hi = b != b_lo;
            float q4[4] = {hi ? 0.f : fv, hi ? 0.f : fv * fv, hi ? fv : 0.f, hi ? fv * fv : 0.f};
#pragma unroll
            for (int d = 1; d < 64; d <<= 1)
#pragma unroll
                for (int i = 0; i < 4; i++) q4[i] += __shfl_xor(q4[i], d, 64);
            if (pl == 0 && ol < s.og) {
                float *sp = a.stats + ((long)tile * 2 * s.Cout + o) * 2;
                sp[0] = q4[0]; sp[1] = q4[1];
                sp[s.Cout * 2] = q4[2]; sp[s.Cout * 2 + 1] = q4[3];
            }
        }
    }
}

// chan_stats[n][c] = sums over the position tiles of sample n (see FwdArgs::stats); one thread per (n, c)
__global__ void __launch_bounds__(256) stats_reduce_kernel(const float *part, float *chan_stats, int N, int Cout, int P, int M)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N * Cout) return;
    const int n = i / Cout, c = i - n * Cout;
    const int t_lo = (int)(((long)n * P) / kDMT), t_hi = (int)((min((long)(n + 1) * P, (long)M) - 1) / kDMT);
    float s0 = 0.f, s1 = 0.f;
    for (int t = t_lo; t <= t_hi; t++) {
        const int slot = n - (t * kDMT) / P;           // 0, or 1 for the tile that began in the sample before
        const float *q = part + (((long)t * 2 + slot) * Cout + c) * 2;
        s0 += q[0]; s1 += q[1];
    }
    chan_stats[2 * i] = s0;
    chan_stats[2 * i + 1] = s1;
}

template <typename T, bool AUX16, int WO, int WP>
int launch_fwd_dma(FwdArgs a, float *outacc, hipStream_t st)
{
    const bool sized = a.s.ss.on != 0;
    constexpr int NT = 64 * WO;
    const int ncu = d2c_num_cus();
    if (ncu <= 0) return D2C_ERR_LAUNCH;
    a.sk_ntile = (a.s.M + kDMT - 1) / kDMT;
    a.sk_otiles = a.s.ogp / NT;
    a.sk_items = a.sk_ntile * a.sk_otiles * a.s.groups;
    // The last, partial round: cut its items into the number of step ranges that is estimated to finish first
    // (a piece costs its steps plus about two steps' time for adding its result).
    // A workgroup lists at most kMaxSeg segments: very large problems get more workgroups than compute units
    // (and no cut of their last round, which is a small part of them).
    const int S = a.s.nchunk * a.s.K;
    const int maxwhole = kMaxSeg / 2;
    const int nwg_whole = a.sk_items > (long)ncu * maxwhole ? (a.sk_items + maxwhole - 1) / maxwhole : ncu;
    const int tail = nwg_whole == ncu ? a.sk_items % ncu : 0;
    a.sk_full = a.sk_items;
    a.sk_cut = 1;
    if (tail && outacc) {
        long best = S;
        for (int k = 2; k <= kMaxSeg / 2 && k <= S; k++) {
            const long rounds = ((long)tail * k + ncu - 1) / ncu;
            const long cost = rounds * ((S + k - 1) / k + 2);
            if (cost < best) { best = cost; a.sk_cut = k; }
        }
        if (a.sk_cut > 1 && best * 10 < (long)S * 9) a.sk_full = a.sk_items - tail; else a.sk_cut = 1;
    }
    const int nshare = a.sk_items - a.sk_full;
    a.outacc = nshare ? outacc : nullptr;
    a.nsplit = 1;
    if (nshare) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        d2c_fill_zero(outacc, (size_t)nshare * NT * kDMT * sizeof(float), st);
    }
    {
        const int nwg = nshare ? ncu : (a.sk_items < nwg_whole ? a.sk_items : nwg_whole);
        D2cProfScope prof(D2C_PROF_FWD, st, "tiled_fwd_dma_kernel");
        // offsets fixed along one / two axes (the layers that deform in space or in time only): 4 / 2 corner rows
        const int nfree = a.s.nd == 3 ? __builtin_popcount(a.s.axes & 7) : 3;
        // (the variants that also write the columns: all three offset axes)
        if (a.col && nfree == 3) {
            if (sized) hipLaunchKernelGGL((tiled_fwd_dma_kernel<T, AUX16, WO, WP, true, 8, true>), dim3(nwg), dim3(kThreads + 64), 0, st, a);
            else hipLaunchKernelGGL((tiled_fwd_dma_kernel<T, AUX16, WO, WP, false, 8, true>), dim3(nwg), dim3(kThreads + 64), 0, st, a);
        } else if (sized) hipLaunchKernelGGL((tiled_fwd_dma_kernel<T, AUX16, WO, WP, true, 8>), dim3(nwg), dim3(kThreads + 64), 0, st, a);
        else if (nfree == 2) hipLaunchKernelGGL((tiled_fwd_dma_kernel<T, AUX16, WO, WP, false, 4>), dim3(nwg), dim3(kThreads + 64), 0, st, a);
        else if (nfree == 1) hipLaunchKernelGGL((tiled_fwd_dma_kernel<T, AUX16, WO, WP, false, 2>), dim3(nwg), dim3(kThreads + 64), 0, st, a);
        else hipLaunchKernelGGL((tiled_fwd_dma_kernel<T, AUX16, WO, WP, false, 8>), dim3(nwg), dim3(kThreads + 64), 0, st, a);
        if (int rc = d2c_check_launch("tiled_fwd_dma_kernel")) return rc;
    }
    if (nshare) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        hipLaunchKernelGGL(fwd_dma_finish_kernel<T>, dim3(nshare, NT / 32), dim3(256), 0, st, a, NT);
        return d2c_check_launch("fwd_dma_finish_kernel");
    }
    return 0;
}

// out = epilogue(outacc + bias), in the element type of the output
template <typename T>
__global__ void __launch_bounds__(256) fwd_finish_kernel(const float *acc, const T *bias, T *out, int Cout, int P, long n,
                                                         int act, float act_scale)
{
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        float v = acc[i];
        if (bias) v += elem_to_f32<T>(bias[(i / P) % Cout]);
        out[i] = f32_to_elem<T>(d2c_epilogue(v, act, act_scale));
    }
}

template <typename T, bool AUX16, int MT, int WO, int WP>
int launch_fwd(const FwdArgs &a, hipStream_t st)
{
    const int ntile = (a.s.M + MT - 1) / MT;
    const int NT = 64 * WO;
    dim3 grid(ntile, a.s.ogp / NT * a.nsplit, a.s.groups);
    D2cProfScope prof(D2C_PROF_FWD, st, "tiled_fwd_kernel");
    if (a.s.ss.on) hipLaunchKernelGGL((tiled_fwd_kernel<T, AUX16, MT, WO, WP, true>), grid, dim3(kThreads), 0, st, a);
    else hipLaunchKernelGGL((tiled_fwd_kernel<T, AUX16, MT, WO, WP, false>), grid, dim3(kThreads), 0, st, a);
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

// Which of the two forward kernels a shape runs on: the DMA-gather kernel (64-position tiles, 512 or 256 output channels
// per workgroup, persistent, the steps of its last round of work items shared out) or the register-gather kernel
// (128-position tiles).  Weight groups wider than 128 output channels take the DMA kernel when they fill the chip
// with whole tiles (128 and more) or have at least 1024 steps in all: with few tiles it cuts their steps into as
// many pieces as there are compute units (512 -> 512 channels on 8x15x27, 51 tiles: 0.74 -> 0.22 ms; 1024 -> 1024
// on 4x8x14, 7 tiles of 432 steps: 0.46 -> 0.21 ms), which pays from about a thousand steps on (4 tiles of 48 steps,
// 512 channels on 4 rows of 64 positions: 13 % slower; 2 tiles of 216 steps: 30 % slower).  Narrow weight groups leave
// most of its output tile empty, but it is bound by its sampling, not by its matrix work: with enough tiles to fill
// the chip without cutting their steps it is 1.3 - 2.2 x faster there too (1024 -> 108 channels on 8x30x54: 1.44 ->
// 0.65 ms), and at the 128 tiles of 64 -> 64 channels on 8x32x32 it is 25 % slower.
constexpr int kDmaTilesNarrow = 160, kDmaTilesWide = 128, kDmaStepsWide = 1024, kColsTiles = 48;
static long dma_tiles(const TiledShape &s) { return (long)((s.M + kDMT - 1) / kDMT) * s.groups; }
bool d2c_fwd_use_dma(const TiledShape &s)
{
    const long tiles = dma_tiles(s);
    if (s.og <= 128) return tiles >= kDmaTilesNarrow;
    return tiles >= kDmaTilesWide || tiles * s.nchunk * s.K >= kDmaStepsWide;
}

int d2c_fwd_pos_tile(const TiledShape &s) { return d2c_fwd_use_dma(s) ? kDMT : kMT; }

// Output channels per workgroup: as wide as the weight group needs (the sampled
// tile is then produced once), but narrower when there are too few position
// tiles to occupy the chip.
int d2c_fwd_out_tile(const TiledShape &s)
{
    const int og = s.og;
    if (d2c_fwd_use_dma(s)) return og > 256 ? 512 : 256;
    int nt = og > 256 ? 512 : (og > 128 ? 256 : (og > 64 ? 128 : 64));
    const int ntile = (s.M + kMT - 1) / kMT;
    while (nt > 64 && ntile * ((og + nt - 1) / nt) < 128) nt >>= 1;
    return nt;
}

// Workgroups per (position tile, output tile): 1 when the tiles alone fill the chip.
int d2c_fwd_split(const TiledShape &s)
{
    // the DMA-gather kernel shares out the steps of its last round of work items, whatever their number
    if (d2c_fwd_use_dma(s)) return 2;
    const int mt = d2c_fwd_pos_tile(s), nt = d2c_fwd_out_tile(s);
    const long wgs = (long)((s.M + mt - 1) / mt) * (s.ogp / nt) * s.groups;
    if (wgs >= 128) return 1;
    const int S = s.nchunk * s.K;
    const long want = (256 + wgs - 1) / wgs;
    return (int)(want < S ? want : S);
}

// Whether the forward kernels of this shape add up per-channel statistics themselves (FwdArgs::stats): the
// DMA-gather kernel, on samples of at least one position tile (a tile then meets at most two samples).
int d2c_fwd_split(const TiledShape &s);
// The forward kernel of this shape adds the statistics of its output up while it stores: the DMA-gather kernel
// (per position tile, see FwdArgs::stats) and the register-gather kernel when every workgroup holds whole sums (no
// steps shared out between workgroups).
bool d2c_fwd_fills_stats(const TiledShape &s)
{
    if (d2c_fwd_use_dma(s)) return s.P >= kDMT;
    return d2c_fwd_split(s) == 1;
}
size_t d2c_fwd_stats_ws(const TiledShape &s)
{
    if (!d2c_fwd_use_dma(s)) return 0;     // (the register-gather kernel adds into the result itself)
    return d2c_align_up((size_t)((s.M + kDMT - 1) / kDMT) * 2 * s.Cout * 2 * sizeof(float));
}

// Whether the forward kernel of this shape can write the sampled columns for the backward pass (FwdArgs::col): the
// DMA-gather kernel on problems with offsets along all three axes and at least kColsTiles position tiles (below that
// the backward kernels that read the columns lose to the ones that sample again: 256 -> 256 channels on 4x15x27, 26
// tiles: 0.25 -> 0.30 ms).
bool d2c_fwd_writes_columns(const TiledShape &s, int dtype)
{
    return (dtype == D2C_BF16 || dtype == D2C_F32) && s.nd == 3 && (s.axes & 7) == 7 &&
           d2c_fwd_use_dma(s) && dma_tiles(s) >= kColsTiles;
}
long d2c_columns_rows(const TiledShape &s) { return (long)((s.M + kDMT - 1) / kDMT) * kDMT; }
// `stats` / `stats_part`: the [N][Cout][2] result and the per-tile scratch of d2c_fwd_stats_ws() bytes, or NULL.
// `col`: where the sampled columns go (d2c_fwd_writes_columns), or NULL.
template <typename T>
int d2c_tiled_fwd_launch(const TiledShape &s, const void *xcl, const void *off, const void *mask, const void *wp,
                         const void *bias, void *out, float *outacc, hipStream_t st, float *stats, float *stats_part,
                         void *col)
{
    const bool dma = d2c_fwd_use_dma(s);
    const int nsplit = (outacc && !dma) ? d2c_fwd_split(s) : 1;
    const long n = (long)s.N * s.Cout * s.P;
    // the channels-last input is followed by a row of zeros (see forward_t)
    const unsigned zrow = (unsigned)((size_t)s.N * s.vol * s.Cin * sizeof(T));
    FwdArgs a{s, xcl, off, mask, wp, bias, out, nsplit > 1 ? outacc : nullptr, nsplit, zrow, 0, 0, 0, 0, 1,
              stats ? (dma ? stats_part : (nsplit == 1 ? stats : nullptr)) : nullptr, nullptr, 0};
    if (col && d2c_fwd_writes_columns(s, (int)Elem<T>::DT)) {
        a.col = col;
        a.col_rows = d2c_columns_rows(s);
    }
    if (a.stats && !dma) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        d2c_fill_zero(a.stats, (size_t)s.N * s.Cout * 2 * sizeof(float), st);
    }
    if (a.stats && dma && d2c_fwd_out_tile(s) != 512) {
        // (the 256-channel tile has two wavefronts per channel, which add into their slots)
        D2cProfScope prof(D2C_PROF_PACK, st);
        d2c_fill_zero(a.stats, d2c_fwd_stats_ws(s), st);
    }
    if (nsplit > 1) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        d2c_fill_zero(outacc, (size_t)n * sizeof(float), st);
    }
    const int nt = d2c_fwd_out_tile(s);
    int rc = 0;
    bool aux16 = false;
    if constexpr (sizeof(T) == 2) aux16 = s.adt == D2C_BF16;
    if (dma) {
        if (nt == 512) {
            if constexpr (sizeof(T) == 2) {
                if (aux16) rc = launch_fwd_dma<T, true, 8, 1>(a, outacc, st);
            }
            if (!aux16) rc = launch_fwd_dma<T, false, 8, 1>(a, outacc, st);
        } else {
            if constexpr (sizeof(T) == 2) {
                if (aux16) rc = launch_fwd_dma<T, true, 4, 2>(a, outacc, st);
            }
            if (!aux16) rc = launch_fwd_dma<T, false, 4, 2>(a, outacc, st);
        }
        if (rc || !a.stats) return rc;
        D2cProfScope prof(D2C_PROF_PACK, st);
        hipLaunchKernelGGL(stats_reduce_kernel, dim3((unsigned)((s.N * s.Cout + 255) / 256)), dim3(256), 0, st, a.stats,
                           stats, s.N, s.Cout, s.P, s.M);
        return d2c_check_launch("stats_reduce_kernel");
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
                       s.Cout, s.P, n, s.act, s.act_scale);
    return d2c_check_launch("fwd_finish_kernel");
}
template int d2c_tiled_fwd_launch<bf16_t>(const TiledShape &, const void *, const void *, const void *, const void *,
                                          const void *, void *, float *, hipStream_t, float *, float *, void *);
template int d2c_tiled_fwd_launch<float>(const TiledShape &, const void *, const void *, const void *, const void *,
                                         const void *, void *, float *, hipStream_t, float *, float *, void *);
