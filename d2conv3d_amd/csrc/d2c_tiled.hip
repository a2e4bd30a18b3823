// Tiled kernel families: eligibility, workspace carving, operand packing and
// dispatch.  Forward / backward kernels live in d2c_tiled_fwd.hip and
// d2c_tiled_bwd.hip.
#include "d2c_tiled.hpp"
#include "d2c_mma.hpp"

int d2c_fwd_out_tile(const TiledShape &s);
template <typename T>
int d2c_tiled_fwd_launch(const TiledShape &s, const void *xcl, const void *off, const void *mask, const void *wp,
                         const void *bias, void *out, float *outacc, hipStream_t st, float *stats, float *stats_part,
                         void *col = nullptr);
bool d2c_fwd_writes_columns(const TiledShape &s, int dtype);
long d2c_columns_rows(const TiledShape &s);
bool d2c_fwd_fills_stats(const TiledShape &s);
size_t d2c_fwd_stats_ws(const TiledShape &s);
int d2c_fwd_split(const TiledShape &s);

bool d2c_tiled_bwd_data_supported(const TiledShape &s, int dtype);
bool d2c_tiled_bwd_weight_supported(const TiledShape &s, int dtype);
int d2c_bwd_ogk(int og, int dtype);
int d2c_bwd_pass_channels(int dtype);
bool d2c_tiled_bwd_single_pass(const TiledShape &s, int dtype);
template <typename T>
int d2c_tiled_bwd_data_launch(const TiledShape &s, const void *gout, const void *xcl, const void *off,
                              const void *mask, const void *w, void *wt, float *gxcl, void *gcolbuf, void *goff,
                              void *gmask, float *auxacc, hipStream_t st, int phase = 3, int g_lo = 0, int g_n = 0,
                              bool weights_packed = false);
bool d2c_bwd_sliceable(const TiledShape &s, int dtype);
int d2c_backward_slices();
int d2c_bwd_data_split(const TiledShape &s, int dtype);
template <typename T>
int d2c_gx_owner_launch(const TiledShape &s, const void *gcol, const SampleLists &L, float *gxcl, hipStream_t st,
                        int c_lo = 0, int c_n = 0);
void d2c_lists_ws(const TiledShape &s, int dtype, size_t *counts, size_t *entries, size_t *ovf);
SampleLists d2c_lists_make(const TiledShape &s, int dtype, void *counts, void *entries, void *ovf);
int d2c_lists_clear(const SampleLists &L, hipStream_t st);
bool d2c_lists_supported(const TiledShape &s);
int d2c_lists_build(const TiledShape &s, const void *off, const void *mask, const SampleLists &L, hipStream_t st);
int d2c_lists_fill(const TiledShape &s, const void *off, const void *mask, const SampleLists &L, hipStream_t st);
int d2c_gx_mode();
int d2c_col_weight_mode();
template <typename T>
int d2c_aux_grad_launch(const TiledShape &s, const void *xcl, const void *off, const void *mask, const void *gcol,
                        void *goff, void *gmask, const SampleLists *lists, void *col, bool col_in_place, hipStream_t st,
                        int g_lo = 0, int g_n = 0);
template <typename T>
int d2c_tiled_bwd_weight_launch(const TiledShape &s, const void *gout, const void *xcl, const void *off,
                                const void *mask, void *goutp, float *gwacc, void *gw, const void *col, long col_rows,
                                hipStream_t st, int phase = 7, int jp_lo = 0, int jp_n = 0);
bool d2c_bwd_weight_from_col(const TiledShape &s, int dtype);
bool d2c_bwd_weight_from_kept_col(const TiledShape &s, int dtype);
size_t d2c_bwd_col_bytes(const TiledShape &s, int dtype, int nchunks = 0);
size_t d2c_bwd_goutp_bytes(const TiledShape &s, int dtype);
template <typename T> int d2c_tiled_unpack_gx(const TiledShape &s, const float *gxcl, void *gx, hipStream_t st);
template <typename T> int d2c_tiled_bias_grad(const TiledShape &s, const void *gout, void *gb, hipStream_t st);

bool d2c_depthwise_supported(const TiledShape &s);
template <typename T>
int d2c_depthwise_forward(const TiledShape &s, const void *xcl, const void *off, const void *mask, const void *wt,
                          const void *bias, void *out, hipStream_t st);
template <typename T>
int d2c_dw_gx_owner_launch(const TiledShape &s, const void *goutcl, const void *wt, const SampleLists &L, float *gxcl,
                           hipStream_t st);
template <typename T>
int d2c_depthwise_backward(const TiledShape &s, const void *goutcl, const void *xcl, const void *off, const void *mask,
                           const void *wt, float *gxcl, void *goff, void *gmask, float *auxacc, float *gwacc, void *gw,
                           hipStream_t st);

static bool mfma_channels_ok(const d2c_conv3d_desc &q);

namespace {

inline int vec_of(int dtype) { return dtype == D2C_BF16 ? 8 : 4; }
inline int bkc_of(int dtype) { return 8 * vec_of(dtype); }

// The 1-D operator as a 3-D problem on a 1 x 1 x L volume with a 1 x 1 x k kernel.
d2c_conv3d_desc as_3d(const d2c_conv1d_desc &q)
{
    d2c_conv3d_desc r;
    r.N = q.N; r.Cin = q.Cin; r.Cout = q.Cout; r.D = 1; r.H = 1; r.W = q.L;
    r.kd = 1; r.kh = 1; r.kw = q.k; r.sd = 1; r.sh = 1; r.sw = q.s; r.pd = 0; r.ph = 0; r.pw = q.p;
    r.dd = 1; r.dh = 1; r.dw = q.d; r.groups = q.groups; r.offset_groups = q.offset_groups;
    r.Do = 1; r.Ho = 1; r.Wo = q.Lo; r.dtype = q.dtype; r.aux_dtype = q.aux_dtype;
    r.epilogue = D2C_EPILOGUE_NONE; r.epilogue_scale = 1.f; r.offset_axes = 0; r.backward_flags = 0;
    r.deform_channels = 0; r.mask_activation = D2C_MASK_ACT_NONE;
    return r;
}

TiledShape tiled_shape(const d2c_conv3d_desc &q, int nd = 3, int quirks = 0, const d2c_size_map_desc *sz = nullptr)
{
    TiledShape s;
    s.ss.on = sz ? 1 : 0;
    s.ss.mode = sz ? sz->mode : 0;
    s.ss.act = sz ? sz->activation : 0;
    for (int i = 0; i < D2C_SIZE_MAX_K; i++) {
        s.ss.base[0][i] = sz ? sz->base_z[i] : 0.f;
        s.ss.base[1][i] = sz ? sz->base_y[i] : 0.f;
        s.ss.base[2][i] = sz ? sz->base_x[i] : 0.f;
    }
    s.nd = nd; s.quirks = quirks;
    s.N = q.N; s.Cin = q.Cin; s.Cout = q.Cout; s.D = q.D; s.H = q.H; s.W = q.W;
    s.K = q.kd * q.kh * q.kw; s.G = q.offset_groups; s.groups = q.groups;
    s.Do = q.Do; s.Ho = q.Ho; s.Wo = q.Wo;
    s.cg = q.Cin / q.groups; s.og = q.Cout / q.groups; s.cpg = q.Cin / q.offset_groups;
    s.nchunk = s.cg / bkc_of(q.dtype);
    s.bkc = bkc_of(q.dtype);
    s.cpc = (s.cg < s.cpg ? s.cg : s.cpg) / s.bkc;
    s.adt = q.aux_dtype;
    s.act = q.epilogue; s.act_scale = q.epilogue_scale;
    s.P = q.Do * q.Ho * q.Wo; s.vol = q.D * q.H * q.W; s.M = q.N * s.P;
    s.axes = (nd == 3 && (q.offset_axes & 7)) ? (q.offset_axes & 7) : 7;
    s.keep = 0xffu;
    if (!(s.axes & 1)) s.keep &= 0x0fu;     // z fixed: dz = 0 corners
    if (!(s.axes & 2)) s.keep &= 0x33u;     // y fixed: dy = 0
    if (!(s.axes & 4)) s.keep &= 0x55u;     // x fixed: dx = 0
    s.dP = make_fastdiv(s.P); s.dHW = make_fastdiv(q.Ho * q.Wo); s.dW = make_fastdiv(q.Wo);
    // samples of the offsets (or the size map) and of the mask: tensors of their own, or both inside the layer's
    // deformation tensor of `deform_channels` channels
    s.obs = q.deform_channels > 0 ? (long)q.deform_channels * s.P
                                  : (sz ? (long)mode_channels(sz->mode) * s.P : (long)s.G * s.K * (nd == 3 ? 3 : 1) * s.P);
    s.mbs = q.deform_channels > 0 ? (long)q.deform_channels * s.P : (long)s.G * s.K * s.P;
    s.mact = q.mask_activation;
    // float problems: 1 = every backward matrix kernel on two-term bfloat16 operands (asked for in the description),
    // 2 = the grad-column product alone, like the forward kernels (the default: every tolerance gate stays green)
    s.f32split = q.dtype != D2C_F32 ? 0 : ((q.backward_flags & D2C_BWD_F32_SPLIT) ? 1 : (kF32SplitFwd ? 2 : 0));
    const int nt = d2c_fwd_out_tile(s);
    s.ogp = (s.og + nt - 1) / nt * nt;
    s.geo = make_geom(q);
    return s;
}

// The tiled kernels let dead corners read a 256-byte row of zeros that follows the channels-last input; the first
// workgroup of the pack kernel writes it (the batch size is the grid's z extent; C is a multiple of the channel
// chunk there, so the row is 128-byte aligned).
template <typename T> D2C_DEV void pack_zero_row(T *xcl, int C, int vol, int zero_row)
{
    if (zero_row && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x < 64)
        reinterpret_cast<unsigned *>(xcl + (long)gridDim.z * C * vol)[threadIdx.x] = 0u;
}

// x [C][vol] -> xcl [vol][C] of one batch element: a 32 x 32 element tile through LDS
template <typename T> D2C_DEV void pack_tile32(const T *xb, T *ob, int C, int vol, int v0, int c0)
{
    __shared__ T tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        const int c = c0 + ty + i, v = v0 + tx;
        if (c < C && v < vol) tile[ty + i][tx] = xb[(long)c * vol + v];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        const int v = v0 + ty + i, c = c0 + tx;
        if (c < C && v < vol) ob[(long)v * C + c] = tile[tx][ty + i];
    }
}

// The same for bfloat16 with 16-byte accesses on both sides (2-byte accesses of 32 lanes move 64 bytes per
// request): a 64 x 64 element tile; needs vol and C to be multiples of 8 and 16-byte aligned tensors.
D2C_DEV void pack_tile64_bf16(const bf16_t *xb, bf16_t *ob, int C, int vol, int v0, int c0)
{
    constexpr int RS = 66;                             // LDS row stride in elements (33 words)
    __shared__ bf16_t tile[64 * RS];                   // [v][c]
    for (int i = threadIdx.x; i < 512; i += 256) {     // 64 channels x 8 vectors of 8 positions
        const int c = c0 + i / 8, v = v0 + (i % 8) * 8;
        if (c < C && v < vol) {                        // (vol % 8 == 0: the vector is inside or outside as a whole)
            const uint4 q = *reinterpret_cast<const uint4 *>(xb + (long)c * vol + v);
            const unsigned u[4] = {q.x, q.y, q.z, q.w};
            bf16_t *t = tile + ((i % 8) * 8) * RS + i / 8;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                t[(2 * e) * RS] = (bf16_t)(u[e] & 0xffffu);
                t[(2 * e + 1) * RS] = (bf16_t)(u[e] >> 16);
            }
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 512; i += 256) {     // 64 positions x 8 vectors of 8 channels
        const int v = v0 + i / 8, c = c0 + (i % 8) * 8;
        if (c < C && v < vol) {
            const unsigned *t = reinterpret_cast<const unsigned *>(tile + (i / 8) * RS + (i % 8) * 8);
            *reinterpret_cast<uint4 *>(ob + (long)v * C + c) = make_uint4(t[0], t[1], t[2], t[3]);
        }
    }
}

// x [N][C][vol] -> xcl [N][vol][C]
template <typename T>
__global__ void __launch_bounds__(256) pack_input_kernel(const T *x, T *xcl, int C, int vol, int zero_row)
{
    pack_zero_row(xcl, C, vol, zero_row);
    const long bo = (long)blockIdx.z * C * vol;
    pack_tile32<T>(x + bo, xcl + bo, C, vol, blockIdx.x * 32, blockIdx.y * 32);
}

__global__ void __launch_bounds__(256) pack_input_bf16_kernel(const bf16_t *x, bf16_t *xcl, int C, int vol, int zero_row)
{
    pack_zero_row(xcl, C, vol, zero_row);
    const long bo = (long)blockIdx.z * C * vol;
    pack_tile64_bf16(x + bo, xcl + bo, C, vol, blockIdx.x * 64, blockIdx.y * 64);
}

// Everything a depthwise call needs before its main kernels, as one launch: up to two tensors to channels-last (the
// input, grad_out), the weights W[c][0][k] -> wt[k][c], a range of the workspace cleared, the bias gradient.  A
// workgroup finds its job from its index; jobs a call does not need have no workgroups.
struct DwPrepArgs {
    struct Pack {
        const void *src;
        void *dst;
        int C, vol, wide;     // wide: 64 x 64 bfloat16 tiles (see pack_tile64_bf16)
        int nbx, nby, nblk;   // tiles along vol and C; workgroups of the job (tiles x batch)
    } pack[2];
    const void *w;
    void *wt;
    int wC, wK, nblk_w;
    void *zrow;                // the row of zeros behind the channels-last input (wC elements)
    uint32_t *zero;
    size_t zero_words;
    int nblk_z;
    const void *gout;          // bias gradient: one workgroup per channel
    void *gb;
    int bN, bC, bP, nblk_b;
};
template <typename T> __global__ void __launch_bounds__(256) dw_prepare_kernel(DwPrepArgs a)
{
    int b = blockIdx.x;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const DwPrepArgs::Pack &pk = a.pack[j];
        if (b < pk.nblk) {
            const int bx = b % pk.nbx, by = (b / pk.nbx) % pk.nby;
            const long bo = (long)(b / (pk.nbx * pk.nby)) * pk.C * pk.vol;
            if constexpr (sizeof(T) == 2) {
                if (pk.wide) {
                    pack_tile64_bf16((const bf16_t *)pk.src + bo, (bf16_t *)pk.dst + bo, pk.C, pk.vol, bx * 64, by * 64);
                    return;
                }
            }
            pack_tile32<T>((const T *)pk.src + bo, (T *)pk.dst + bo, pk.C, pk.vol, bx * 32, by * 32);
            return;
        }
        b -= pk.nblk;
    }
    if (b < a.nblk_w) {
        const T *w = (const T *)a.w;
        T *wt = (T *)a.wt;
        const int n = a.wC * a.wK;
        for (int i = b * 256 + threadIdx.x; i < n; i += a.nblk_w * 256) wt[i] = w[(i % a.wC) * a.wK + i / a.wC];
        if (b == 0)
            for (int i = threadIdx.x; i < a.wC; i += 256) ((T *)a.zrow)[i] = (T)0;
        return;
    }
    b -= a.nblk_w;
    if (b < a.nblk_z) {
        for (size_t i = (size_t)b * 256 + threadIdx.x; i < a.zero_words; i += (size_t)a.nblk_z * 256) a.zero[i] = 0u;
        return;
    }
    b -= a.nblk_z;
    if (b < a.nblk_b) bias_grad_body<T, 256>((const T *)a.gout, (T *)a.gb, a.bN, a.bC, a.bP, b);
}

// Forward weight operand in MFMA fragment order:
//   wp[wg][step = chunk*K + k][o-block of 32][k-group][lane] = 16 bytes =
//   W[wg*og + ob*32 + lane%32][chunk*BKC + (2*kg + lane/32)*VEC + 0..VEC-1][k]
// (rows past og are zero), so a wavefront's fragment load is 1 KiB contiguous.
template <typename T>
__global__ void __launch_bounds__(256) pack_weight_fwd_kernel(const T *w, T *wp, TiledShape s, long total)
{
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC;
    const int OBT = s.ogp / 32, S = s.nchunk * s.K;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int lane = (int)(i & 63);
        const int kg = (int)((i >> 6) & 3);
        long r = i >> 8;
        const int obg = (int)(r % OBT); r /= OBT;
        const int st = (int)(r % S);
        const int wg = (int)(r / S);
        const int j = st / s.K, k = st - j * s.K;
        const int ol = obg * 32 + (lane & 31);
        const int ch = j * BKC + (2 * kg + (lane >> 5)) * VEC;
        alignas(16) T tmp[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++)
            tmp[e] = ol < s.og ? w[((long)(wg * s.og + ol) * s.cg + ch + e) * s.K + k] : (T)0;
        *reinterpret_cast<uint4 *>(wp + i * VEC) = operand_vec<T, kF32SplitFwd>(tmp);
    }
}

// The same re-layout through LDS: a workgroup takes kPackRows output channels of one channel chunk, whose
// weights are runs of BKC * K consecutive elements in W, reads them with 16-byte loads and writes whole
// 16-byte fragment vectors (kPackRows consecutive lanes each).  Needs a 16-byte aligned W and rows that fit LDS.
constexpr int kPackRows = 8;
template <typename T>
__global__ void __launch_bounds__(256) pack_weight_fwd_lds_kernel(const T *w, T *wp, TiledShape s)
{
    constexpr int VEC = Elem<T>::VEC, BKC = 8 * VEC, R = kPackRows;
    extern __shared__ __align__(16) unsigned char smem[];
    const int OBT = s.ogp / 32, S = s.nchunk * s.K;
    int b = blockIdx.x;
    const int part = b % (32 / R); b /= 32 / R;
    const int obg = b % OBT; b /= OBT;
    const int j = b % s.nchunk;
    const int wg = b / s.nchunk;
    const int run = BKC * s.K;                       // elements of a row
    const int rs = run * (int)sizeof(T) + 4;         // LDS row stride in bytes (an odd number of banks)
    const int ol0 = obg * 32 + part * R;
    const int vpr = run * (int)sizeof(T) / 16;       // 16-byte vectors of a row
    for (int i = threadIdx.x; i < R * vpr; i += 256) {
        const int r = i / vpr, v = i - r * vpr;
        const int ol = ol0 + r;
        uint4 val = make_uint4(0, 0, 0, 0);
        if (ol < s.og)
            val = *reinterpret_cast<const uint4 *>(
                reinterpret_cast<const char *>(w + ((long)(wg * s.og + ol) * s.cg + j * BKC) * s.K) + (size_t)v * 16);
        unsigned *d = reinterpret_cast<unsigned *>(smem + r * rs + v * 16);
        d[0] = val.x; d[1] = val.y; d[2] = val.z; d[3] = val.w;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < s.K * 8 * R; i += 256) {
        const int r = i % R, q = i / R;
        const int khi = q & 7, k = q >> 3;           // khi = 2 * k-group + lane / 32
        const T *src = reinterpret_cast<const T *>(smem + r * rs) + khi * VEC * s.K + k;
        alignas(16) T tmp[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) tmp[e] = src[e * s.K];
        const int lane = (khi & 1) * 32 + part * R + r;
        const long vi = ((((long)wg * S + j * s.K + k) * OBT + obg) * 4 + (khi >> 1)) * 64 + lane;
        *reinterpret_cast<uint4 *>(wp + vi * VEC) = operand_vec<T, kF32SplitFwd>(tmp);
    }
}

// Size-map source, backward: fp32 sums per axis [N][3][P] -> gradient of the raw size prediction [N][channels][P]
// (the axes a channel feeds add up; times the derivative of the size activation), in the storage type of the map.
template <bool AUX16>
__global__ void __launch_bounds__(256) size_grad_finish_kernel(TiledShape s, const float *acc, const void *raw, void *graw)
{
    const int nc = mode_channels(s.ss.mode);
    const long total = (long)s.N * s.P;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const long n = i / s.P, p = i - n * s.P;
        for (int c = 0; c < nc; c++) {
            float v = 0.f;
#pragma unroll
            for (int ax = 0; ax < 3; ax++)
                if (axis_channel(s.ss.mode, ax) == c) v += acc[(n * 3 + ax) * s.P + p];
            const long ri = n * s.obs + (long)c * s.P + p;
            v *= size_act_grad(s.ss.act, ld_auxT<AUX16>(raw, ri));
            if constexpr (AUX16) reinterpret_cast<bf16_t *>(graw)[ri] = f32_to_bf16(v);
            else reinterpret_cast<float *>(graw)[ri] = v;
        }
    }
}

// Size-map source, backward: raw map -> (size - 1) per axis as float [N][3][P] (0 for an axis the mode does not
// predict), once per call: the kernels of the backward pass form a tap's offsets from it per (tile, tap).
template <bool AUX16>
__global__ void __launch_bounds__(256) size_minus_one_kernel(TiledShape s, const void *raw, float *sm1)
{
    const long total = (long)s.N * s.P;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const long n = i / s.P, p = i - n * s.P;
        float c[3];
#pragma unroll
        for (int ax = 0; ax < 3; ax++) {
            const int ch = axis_channel(s.ss.mode, ax);
            c[ax] = ch < 0 ? 0.f : ld_auxT<AUX16>(raw, n * s.obs + (long)ch * s.P + p);
        }
        size_minus_one<AUX16>(s, c);
#pragma unroll
        for (int ax = 0; ax < 3; ax++) sm1[(n * 3 + ax) * s.P + p] = c[ax];
    }
}

struct FwdWs {
    size_t xcl, wp, outacc, total;
};
// Caller-held prepared region (d2c_conv3d_prepared_bytes): channels-last input + zero row | forward weights in
// fragment order | backward weights transposed per step (single-pass reductions only)
struct PreparedLayout {
    size_t xcl, wp, wt, wt_bytes, total;
};
FwdWs fwd_ws(const d2c_conv3d_desc &q, const TiledShape &s)
{
    const size_t es = d2c_elem_size(q.dtype);
    FwdWs w;
    w.xcl = 0;
    w.wp = d2c_align_up((size_t)s.N * s.vol * s.Cin * es + 256);   // input, then a 256-byte row of zeros
    w.outacc = w.wp + d2c_align_up((size_t)s.groups * s.nchunk * s.K * s.ogp * bkc_of(q.dtype) * es);
    // fp32 partial sums of the output, used only when the forward kernel splits its steps (as whole tiles of
    // 64 positions x padded output channels in the DMA-gather kernel)
    w.total = w.outacc;
    if (d2c_fwd_split(s) > 1)
        w.total += d2c_align_up((size_t)((s.M + 63) / 64 * 64) * s.ogp * s.groups * sizeof(float));
    return w;
}

PreparedLayout prepared_layout(const d2c_conv3d_desc &q, const TiledShape &s)
{
    const size_t es = d2c_elem_size(q.dtype);
    PreparedLayout p;
    p.xcl = 0;
    p.wp = d2c_align_up((size_t)s.N * s.vol * s.Cin * es + 256);
    p.wt = p.wp + d2c_align_up((size_t)s.groups * s.nchunk * s.K * s.ogp * bkc_of(q.dtype) * es);
    const int omax = d2c_bwd_pass_channels(q.dtype);
    p.wt_bytes = s.og <= omax ? d2c_align_up((size_t)s.groups * s.K * s.nchunk * bkc_of(q.dtype) * d2c_bwd_ogk(s.og, q.dtype) * es) : 0;
    p.total = p.wt + p.wt_bytes;
    return p;
}

template <typename T>
int pack_input(const TiledShape &s, const void *x, void *xcl, hipStream_t st, bool zero_row = false)
{
    dim3 grid((s.vol + 31) / 32, (s.Cin + 31) / 32, s.N);
    D2cProfScope prof(D2C_PROF_PACK, st);
    if constexpr (sizeof(T) == 2) {
        if (s.vol % 8 == 0 && s.Cin % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
            reinterpret_cast<uintptr_t>(xcl) % 16 == 0) {
            hipLaunchKernelGGL(pack_input_bf16_kernel, dim3((s.vol + 63) / 64, (s.Cin + 63) / 64, s.N), dim3(256), 0, st,
                               (const bf16_t *)x, (bf16_t *)xcl, s.Cin, s.vol, (int)zero_row);
            return d2c_check_launch("pack_input_bf16_kernel");
        }
    }
    hipLaunchKernelGGL(pack_input_kernel<T>, grid, dim3(256), 0, st, (const T *)x, (T *)xcl, s.Cin, s.vol, (int)zero_row);
    return d2c_check_launch("pack_input_kernel");
}

// The jobs of dw_prepare_kernel for one call (gout == nullptr: no grad_out copy; zero_bytes == 0: nothing to clear;
// gb == nullptr: no bias gradient).
template <typename T>
int dw_prepare(const TiledShape &s, const void *x, void *xcl, const void *gout, void *goutcl, const void *w, void *wt,
               void *zero, size_t zero_bytes, void *gb, hipStream_t st)
{
    DwPrepArgs a{};
    auto job = [&](DwPrepArgs::Pack &pk, const void *src, void *dst, int C, int vol) {
        pk.src = src; pk.dst = dst; pk.C = C; pk.vol = vol;
        pk.wide = sizeof(T) == 2 && vol % 8 == 0 && C % 8 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(dst) % 16 == 0;
        const int tl = pk.wide ? 64 : 32;
        pk.nbx = (vol + tl - 1) / tl; pk.nby = (C + tl - 1) / tl;
        pk.nblk = pk.nbx * pk.nby * s.N;
    };
    job(a.pack[0], x, xcl, s.Cin, s.vol);
    if (gout) job(a.pack[1], gout, goutcl, s.Cout, s.P);
    a.w = w; a.wt = wt; a.wC = s.Cin; a.wK = s.K;
    a.zrow = (T *)xcl + (size_t)s.N * s.vol * s.Cin;
    a.nblk_w = std::min((s.Cin * s.K + 255) / 256, 1024);
    a.zero = (uint32_t *)zero; a.zero_words = zero_bytes / 4;
    a.nblk_z = (int)std::min<size_t>((a.zero_words + 1023) / 1024, 2048);
    a.gout = gout; a.gb = gb; a.bN = s.N; a.bC = s.Cout; a.bP = s.P;
    a.nblk_b = (gb && gout) ? s.Cout : 0;
    const long nblk = (long)a.pack[0].nblk + a.pack[1].nblk + a.nblk_w + a.nblk_z + a.nblk_b;
    D2cProfScope prof(D2C_PROF_PACK, st);
    hipLaunchKernelGGL(dw_prepare_kernel<T>, dim3((unsigned)nblk), dim3(256), 0, st, a);
    return d2c_check_launch("dw_prepare_kernel");
}

bool is_depthwise(const d2c_conv3d_desc &q)
{
    if (q.dtype != D2C_BF16 && q.dtype != D2C_F32) return false;
    return q.groups == q.Cin && q.Cout == q.Cin && q.Cin > 1 && d2c_depthwise_supported(tiled_shape(q));
}

// depthwise workspace: channels-last input + one row of zeros | weights [K][C] | grad_input accumulator | grad_weight accumulator |
// channels-last grad_out | sample lists (bucket counts, buckets of 32-byte entries, overflow array)
struct DwWs {
    size_t xcl, wt, gxcl, gwacc, auxacc, goutcl, counts, entries, ovf, total_fwd, total_bwd;
};
DwWs dw_ws(const d2c_conv3d_desc &q, const TiledShape &s)
{
    const size_t es = d2c_elem_size(q.dtype);
    DwWs w;
    w.xcl = 0;
    w.wt = d2c_align_up(((size_t)s.N * s.vol + 1) * s.Cin * es);   // input, then a row of zeros
    w.total_fwd = w.wt + d2c_align_up((size_t)s.K * s.Cin * es);
    w.gxcl = w.total_fwd;
    w.gwacc = w.gxcl + d2c_align_up((size_t)s.N * s.vol * s.Cin * sizeof(float));
    w.auxacc = w.gwacc + d2c_align_up((size_t)s.K * s.Cin * sizeof(float));
    // (grad_weight sums, offset / mask gradient sums and bucket counts follow each other: one clear)
    size_t c, en, ov;
    d2c_lists_ws(s, D2C_F32, &c, &en, &ov);      // (32-byte entries whatever the element type)
    w.counts = w.auxacc + d2c_align_up((size_t)s.N * s.G * s.K * s.P * 4 * sizeof(float));
    w.goutcl = w.counts + c;
    w.entries = w.goutcl + d2c_align_up((size_t)s.N * s.P * s.Cout * es);
    w.ovf = w.entries + en;
    w.total_bwd = w.ovf + ov;
    return w;
}

template <typename T>
int forward_t(const d2c_conv3d_desc &q, const void *x, const void *off, const void *mask, const void *w,
              const void *bias, void *out, void *ws, hipStream_t st, int nd = 3, const d2c_size_map_desc *sz = nullptr,
              float *stats = nullptr, const D2cPrepared *prep = nullptr, void *columns = nullptr)
{
    const TiledShape s = tiled_shape(q, nd, 0, sz);
    char *base = (char *)ws;
    if (nd == 3 && is_depthwise(q)) {
        const DwWs d = dw_ws(q, s);
        if (int rc = dw_prepare<T>(s, x, base + d.xcl, nullptr, nullptr, w, base + d.wt, nullptr, 0, nullptr, st)) return rc;
        return d2c_depthwise_forward<T>(s, base + d.xcl, off, mask, base + d.wt, bias, out, st);
    }
    const FwdWs l = fwd_ws(q, s);
    // (a caller-held prepared region takes the place of the workspace's channels-last input and packed weights; what it
    // already holds from an earlier call is not made again)
    const PreparedLayout pl = prepared_layout(q, s);
    char *xcl_p = prep ? (char *)prep->base + pl.xcl : base + l.xcl;
    char *wp_p = prep ? (char *)prep->base + pl.wp : base + l.wp;
    if (!(prep && (prep->reuse & D2C_REUSE_INPUT)))
        if (int rc = pack_input<T>(s, x, xcl_p, st, true)) return rc;   // with the row of zeros behind it
    const long total = (long)s.groups * s.nchunk * s.K * (s.ogp / 32) * 4 * 64;
    long g = (total + 255) / 256;
    if (g > 8192) g = 8192;
    if (!(prep && (prep->reuse & D2C_REUSE_FORWARD_WEIGHTS))) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        const size_t lds = (size_t)kPackRows * ((size_t)bkc_of(q.dtype) * s.K * sizeof(T) + 4);
        if (lds <= 64 * 1024 && reinterpret_cast<uintptr_t>(w) % 16 == 0)
            hipLaunchKernelGGL(pack_weight_fwd_lds_kernel<T>,
                               dim3((unsigned)(s.groups * s.nchunk * (s.ogp / 32) * (32 / kPackRows))), dim3(256), lds, st,
                               (const T *)w, (T *)wp_p, s);
        else
            hipLaunchKernelGGL(pack_weight_fwd_kernel<T>, dim3((unsigned)g), dim3(256), 0, st, (const T *)w,
                               (T *)wp_p, s, total);
    }
    if (int rc = d2c_check_launch("pack_weight_fwd_kernel")) return rc;
    // (the per-tile sums of the output statistics go behind everything else in the workspace)
    return d2c_tiled_fwd_launch<T>(s, xcl_p, off, mask, wp_p, bias, out, (float *)(base + l.outacc), st,
                                   stats, stats ? (float *)(base + l.total) : nullptr, columns);
}

// grad_input by sample lists (see d2c_invlist.hip): from whole grad-column rows, i.e. the reduction over all output
// channels of a weight group (in one pass of the product-only kernels, or in several whose rows are added up).
bool use_lists(const d2c_conv3d_desc &q, const TiledShape &s)
{
    return d2c_gx_mode() >= 1 && d2c_lists_supported(s) && d2c_tiled_bwd_data_supported(s, q.dtype) &&
           (s.nd == 3 || d2c_tiled_bwd_single_pass(s, q.dtype));
}

// grad_offset / grad_mask by the kernel of d2c_aux_grad.hip (from the grad-column rows).  (Weight groups wider than
// one pass of the grad-column product get whole rows too: the later passes over their output channels add to the
// rows, see d2c_tiled_bwd_data_launch.
// That needs the product-only kernels, i.e. grad_input from sample lists: where grad_input is scattered with
// atomics by the fused kernel, wide weight groups keep the fused kernel's passes.)
bool use_aux_kernel(const d2c_conv3d_desc &q, const TiledShape &s)
{
    if (!d2c_tiled_bwd_data_supported(s, q.dtype)) return false;
    // (1-D problems with wide weight groups keep the fused kernel: their float32 gradients are held to the literal
    // gate, which the two-term operands of the product-only kernel miss there)
    return d2c_tiled_bwd_single_pass(s, q.dtype) || (s.nd == 3 && d2c_gx_mode() >= 1 && d2c_lists_supported(s));
}

// grad_weight as a matrix product over sampled columns that the offset / mask gradient kernel writes on its way
// (needs that kernel to run: the caller wants grad_offset or grad_mask)
// (0 sample again, 1 columns in a buffer of their own, 2 columns over the grad-column rows: the description's
// backward_flags, or where those say nothing the process-wide test hook)
int gw_mode(const d2c_conv3d_desc &q)
{
    const int f = q.backward_flags & D2C_BWD_GW_MASK;
    return f == D2C_BWD_GW_DEFAULT ? d2c_col_weight_mode() : (f == D2C_BWD_GW_RESAMPLE ? 0 : f);
}
bool use_col_weight(const d2c_conv3d_desc &q, const TiledShape &s)
{
    if (q.dtype != D2C_BF16 && gw_mode(q) != 1) return false;
    return gw_mode(q) && use_aux_kernel(q, s) && d2c_bwd_weight_from_col(s, q.dtype);
}
// ... written over the grad-column rows (mode 2): grad_input is taken from those rows first, from sample lists
// that a pass of their own files
// (bfloat16 only: float problems asked for it sample again, as they always did)
bool col_in_place(const d2c_conv3d_desc &q, const TiledShape &s)
{
    return gw_mode(q) == 2 && q.dtype == D2C_BF16 && use_col_weight(q, s);
}

// The backward pass slice by slice over the offset groups (see d2c_bwd_sliceable): `gs` groups per slice of the
// grad-column rows (0: not sliced), `cgs` groups per block of sampled columns that one launch of the grad-weight
// product takes (a multiple of gs that holds an even number of channel chunks).
struct BwdSlices {
    int gs, cgs;
};
BwdSlices bwd_slices(const d2c_conv3d_desc &q, const TiledShape &s)
{
    BwdSlices r{0, 0};
    // the description's backward_flags, or where those say nothing the process-wide test hook; by default the pass
    // is not sliced (one pass over all groups is the faster one: the grad_input kernel needs the parallelism of all
    // channel chunks at once)
    int n = (q.backward_flags >> 8) & 0xff;
    if (n == 0) n = d2c_backward_slices();
    if (n < 2 || gw_mode(q) == 2 || d2c_gx_mode() < 1 || s.ss.on || !d2c_bwd_sliceable(s, q.dtype) ||
        !d2c_tiled_bwd_data_supported(s, q.dtype) || !d2c_lists_supported(s))
        return r;
    if (n > s.G) n = s.G;
    r.gs = (s.G + n - 1) / n;
    r.cgs = ((r.gs * (s.cpg / 64)) % 2 == 0) ? r.gs : 2 * r.gs;
    return r;
}

struct BwdWs {
    size_t xcl, wt, gxcl, gwacc, goutp, auxacc, gcol, counts, entries, ovf, gsacc, sm1, col, total;
};
// `saved_columns`: the caller brings the sampled columns of the forward call (no column region, no slices)
BwdWs bwd_ws(const d2c_conv3d_desc &q, const TiledShape &s, bool saved_columns = false)
{
    const size_t es = d2c_elem_size(q.dtype);
    BwdWs w;
    w.xcl = 0;
    w.wt = d2c_align_up((size_t)s.N * s.vol * s.Cin * es + 256);   // input, then a 256-byte row of zeros
    const int omax = d2c_bwd_pass_channels(q.dtype);
    const int ogk = d2c_bwd_ogk(s.og < omax ? s.og : omax, q.dtype);
    w.gxcl = w.wt + d2c_align_up((size_t)s.groups * s.K * s.nchunk * bkc_of(q.dtype) * ogk * es);
    w.gwacc = w.gxcl + d2c_align_up((size_t)s.N * s.vol * s.Cin * sizeof(float));
    w.goutp = w.gwacc + d2c_align_up((size_t)s.Cout * s.cg * s.K * sizeof(float));
    w.auxacc = w.goutp + d2c_align_up(d2c_bwd_goutp_bytes(s, q.dtype));
    // fp32 scratch of the offset / mask gradient, used when the data kernel splits its steps or reduces the output
    // channels in several passes (the partial sums then add up in fp32, whatever the storage type of the result)
    w.total = w.auxacc;
    if (d2c_bwd_data_split(s, q.dtype) > 1 || !d2c_tiled_bwd_single_pass(s, q.dtype))
        w.total += d2c_align_up((size_t)s.N * s.G * s.K * s.P * (s.nd + 1) * sizeof(float));
    w.gcol = w.counts = w.entries = w.ovf = 0;
    const BwdSlices sl = saved_columns ? BwdSlices{0, 0} : bwd_slices(q, s);
    if (use_lists(q, s) || use_aux_kernel(q, s)) {
        w.gcol = w.total;
        // (+ 64 rows behind the last one: what the last tile of the grad-weight product reads when the columns took
        // the rows' place)
        const size_t chunks = sl.gs ? (size_t)sl.gs * (s.cpg / bkc_of(q.dtype)) : (size_t)(s.Cin / bkc_of(q.dtype));
        w.total = w.gcol + d2c_align_up((chunks * s.K * s.M + 64) * bkc_of(q.dtype) * es);
    }
    if (use_lists(q, s)) {
        size_t c, en, ov;
        d2c_lists_ws(s, q.dtype, &c, &en, &ov);
        w.counts = w.total;
        w.entries = w.counts + c;
        w.ovf = w.entries + en;
        w.total = w.ovf + ov;
    }
    // size-map source: fp32 sums of the size gradient per axis
    w.gsacc = w.total;
    if (s.ss.on) w.total += d2c_align_up((size_t)s.N * 3 * s.P * sizeof(float));
    w.sm1 = w.total;       // ... and (size - 1) per axis
    if (s.ss.on) w.total += d2c_align_up((size_t)s.N * 3 * s.P * sizeof(float));
    w.col = w.total;       // sampled columns for the grad-weight product
    if (!saved_columns && use_col_weight(q, s) && !col_in_place(q, s))
        w.total += d2c_align_up(d2c_bwd_col_bytes(s, q.dtype, sl.cgs ? sl.cgs * (s.cpg / 64) : 0));
    return w;
}

template <typename T>
int backward_t(const d2c_conv3d_desc &q, const void *gout, const void *x, const void *off, const void *mask,
               const void *w, void *gx, void *goff, void *gmask, void *gw, void *gb, void *ws, hipStream_t st,
               int nd = 3, int quirks = 0, const d2c_size_map_desc *sz = nullptr, const D2cPrepared *prep = nullptr,
               const void *columns = nullptr)
{
    TiledShape s = tiled_shape(q, nd, quirks, sz);
    char *base = (char *)ws;
    if (!mask) gmask = nullptr;
    const void *size_raw = off;   // (size-map source; `off` becomes the per-axis (size - 1) below)
    if (nd == 3 && is_depthwise(q)) {
        const DwWs d = dw_ws(q, s);
        float *gxcl = gx ? (float *)(base + d.gxcl) : nullptr;
        float *gwacc = gw ? (float *)(base + d.gwacc) : nullptr;
        const bool grads = gx || goff || gmask || gw;
        // one launch: input and grad_out channels-last ([N][P][C]), the weights [K][C], the clear of the grad_weight sums,
        // offset / mask gradient sums and bucket counts (which follow each other), the bias gradient
        if (!grads) return gb ? d2c_tiled_bias_grad<T>(s, gout, gb, st) : D2C_OK;
        if (int rc = dw_prepare<T>(s, x, base + d.xcl, gout, base + d.goutcl, w, base + d.wt,
                                   grads ? base + d.gwacc : nullptr, grads ? d.goutcl - d.gwacc : 0, gb, st))
            return rc;
        if (grads) {
            const bool lists = gx && d2c_gx_mode() >= 1 && d2c_lists_supported(s);
            SampleLists L{nullptr, nullptr, nullptr, 0, 0, 0};
            if (lists) {
                L = d2c_lists_make(s, D2C_F32, base + d.counts, base + d.entries, base + d.ovf);
                if (int rc = d2c_lists_fill(s, off, mask, L, st)) return rc;
            }
            if (goff || gmask || gw || !lists)
                if (int rc = d2c_depthwise_backward<T>(s, base + d.goutcl, base + d.xcl, off, mask, base + d.wt,
                                                      lists ? nullptr : gxcl, goff, gmask, (float *)(base + d.auxacc),
                                                      gwacc, gw, st))
                    return rc;
            if (lists)
                if (int rc = d2c_dw_gx_owner_launch<T>(s, base + d.goutcl, base + d.wt, L, gxcl, st)) return rc;
            if (gx)
                if (int rc = d2c_tiled_unpack_gx<T>(s, gxcl, gx, st)) return rc;
        }
        return D2C_OK;
    }
    const BwdWs l = bwd_ws(q, s, columns != nullptr);
    const PreparedLayout pl = prepared_layout(q, s);
    char *xcl_p = prep ? (char *)prep->base + pl.xcl : base + l.xcl;
    // (the transposed weights of the region serve single-pass reductions; wider weight groups re-pack per pass)
    const bool wt_prep = prep && pl.wt_bytes > 0;
    char *wt_p = wt_prep ? (char *)prep->base + pl.wt : base + l.wt;
    const bool wt_packed = wt_prep && (prep->reuse & D2C_REUSE_BACKWARD_WEIGHTS);
    if (!(prep && (prep->reuse & D2C_REUSE_INPUT)))
        if (int rc = pack_input<T>(s, x, xcl_p, st, true)) return rc;   // with the row of zeros behind it
    if (s.ss.on) {
        D2cProfScope prof(D2C_PROF_PACK, st);
        long gr = ((long)s.N * s.P + 255) / 256;
        if (gr > 8192) gr = 8192;
        float *sm1 = (float *)(base + l.sm1);
        if (s.adt == D2C_BF16)
            hipLaunchKernelGGL(size_minus_one_kernel<true>, dim3((unsigned)gr), dim3(256), 0, st, s, size_raw, sm1);
        else
            hipLaunchKernelGGL(size_minus_one_kernel<false>, dim3((unsigned)gr), dim3(256), 0, st, s, size_raw, sm1);
        if (int rc = d2c_check_launch("size_minus_one_kernel")) return rc;
        s.ss.on = 2;
        off = sm1;
    }
    bool gw_from_col = false, gw_in_place = false, gw_done = false;
    // (`columns`: the sampled columns the forward call kept -- the offset / mask gradient kernel then writes none, the
    // grad-weight product takes these, and the settings that save workspace by other means do not apply)
    const BwdSlices sl = columns ? BwdSlices{0, 0} : bwd_slices(q, s);
    if ((gx || goff || gmask) && sl.gs > 0) {
        // Slice by slice over the offset groups: the grad-column rows of a slice are made, read by the offset / mask
        // gradient kernel (which files the slice's samples and writes its sampled columns) and by the grad_input
        // kernel, and the grad-weight product takes the columns of a block of slices, before the next slice
        // overwrites the rows: the buffers hold one slice (one block), and what a kernel reads was written a moment ago.
        constexpr int BKC = 8 * Elem<T>::VEC;
        const size_t es = sizeof(T);
        float *gxcl = gx ? (float *)(base + l.gxcl) : nullptr;
        const bool lists = gx != nullptr, auxk = goff || gmask;
        gw_from_col = gw && auxk && use_col_weight(q, s);
        SampleLists L{nullptr, nullptr, nullptr, 0, 0, 0};
        if (lists) {
            L = d2c_lists_make(s, Elem<T>::DT, base + l.counts, base + l.entries, base + l.ovf);
            if (int rc = auxk ? d2c_lists_clear(L, st) : d2c_lists_build(s, off, mask, L, st)) return rc;
        }
        if (int rc = d2c_tiled_bwd_data_launch<T>(s, gout, xcl_p, off, mask, w, wt_p, nullptr, base + l.gcol,
                                                 nullptr, nullptr, (float *)(base + l.auxacc), st, 1, 0, 0, wt_packed))
            return rc;
        if (gw_from_col)
            if (int rc = d2c_tiled_bwd_weight_launch<T>(s, gout, xcl_p, off, mask, base + l.goutp,
                                                       (float *)(base + l.gwacc), gw, base + l.col, 0, st, 1))
                return rc;
        const int cpc = s.cpg / BKC;
        const long mpad = (long)((s.M + 63) / 64) * 64;
        for (int g0 = 0; g0 < s.G; g0 += sl.gs) {
            const int gn = s.G - g0 < sl.gs ? s.G - g0 : sl.gs;
            const int c_lo = g0 * cpc, blk_lo = g0 / sl.cgs * sl.cgs;
            // (the kernels address chunk c at c * K * rows * BKC elements from the pointer they get: the pointer that
            // puts the slice's first chunk at the start of the buffer)
            char *gcol_v = reinterpret_cast<char *>(reinterpret_cast<uintptr_t>(base + l.gcol)
                                                    - (uintptr_t)((size_t)c_lo * s.K * s.M * BKC * es));
            char *col_v = reinterpret_cast<char *>(reinterpret_cast<uintptr_t>(base + l.col)
                                                   - (uintptr_t)((size_t)blk_lo * cpc * s.K * mpad * BKC * es));
            if (int rc = d2c_tiled_bwd_data_launch<T>(s, gout, xcl_p, off, mask, w, wt_p, nullptr, gcol_v,
                                                     nullptr, nullptr, (float *)(base + l.auxacc), st, 2, g0, gn))
                return rc;
            if (auxk)
                if (int rc = d2c_aux_grad_launch<T>(s, xcl_p, off, mask, gcol_v, goff, gmask, lists ? &L : nullptr,
                                                    gw_from_col ? col_v : nullptr, false, st, g0, gn))
                    return rc;
            if (lists)
                if (int rc = d2c_gx_owner_launch<T>(s, gcol_v, L, gxcl, st, c_lo, gn * cpc)) return rc;
            const int g1 = g0 + gn;
            if (gw_from_col && (g1 == s.G || g1 % sl.cgs == 0))
                if (int rc = d2c_tiled_bwd_weight_launch<T>(s, gout, xcl_p, off, mask, base + l.goutp,
                                                           (float *)(base + l.gwacc), gw, col_v, mpad, st, 2,
                                                           blk_lo * cpc / 2, (g1 - blk_lo) * cpc / 2))
                    return rc;
        }
        if (gx)
            if (int rc = d2c_tiled_unpack_gx<T>(s, gxcl, gx, st)) return rc;
        if (gw_from_col) {
            if (int rc = d2c_tiled_bwd_weight_launch<T>(s, gout, xcl_p, off, mask, base + l.goutp,
                                                       (float *)(base + l.gwacc), gw, base + l.col, 0, st, 4))
                return rc;
            gw_done = true;
        }
    } else if (gx || goff || gmask) {
        if (d2c_tiled_bwd_data_supported(s, q.dtype)) {
            float *gxcl = gx ? (float *)(base + l.gxcl) : nullptr;
            const bool lists = gx && use_lists(q, s);
            const bool auxk = (goff || gmask) && use_aux_kernel(q, s);
            // grad_input from sample lists: filled by the offset / mask gradient kernel on its way when that
            // runs, by a pass of their own otherwise
            // size-map source: `goff` is the gradient of the raw size map; the offset / mask gradient kernel adds
            // into fp32 sums per axis, which a finishing kernel folds into it
            void *goff_k = goff;
            if (s.ss.on && goff) {
                goff_k = base + l.gsacc;
                D2cProfScope prof(D2C_PROF_PACK, st);
                d2c_fill_zero(goff_k, (size_t)s.N * 3 * s.P * sizeof(float), st);
            }
            gw_from_col = gw && (columns ? d2c_bwd_weight_from_kept_col(s, q.dtype) : (auxk && use_col_weight(q, s)));
            // (the sampled columns over the grad-column rows: grad_input has to be done with the rows before the
            // offset / mask gradient kernel runs, so the samples are filed by a pass of their own)
            gw_in_place = gw_from_col && !columns && col_in_place(q, s);
            SampleLists L{nullptr, nullptr, nullptr, 0, 0, 0};
            if (lists) {
                L = d2c_lists_make(s, Elem<T>::DT, base + l.counts, base + l.entries, base + l.ovf);
                if (int rc = (auxk && !gw_in_place) ? d2c_lists_clear(L, st) : d2c_lists_build(s, off, mask, L, st)) return rc;
            }
            if (int rc = d2c_tiled_bwd_data_launch<T>(s, gout, xcl_p, off, mask, w, wt_p,
                                                     lists ? nullptr : gxcl, (lists || auxk) ? base + l.gcol : nullptr,
                                                     auxk ? nullptr : goff, auxk ? nullptr : gmask,
                                                     (float *)(base + l.auxacc), st, 3, 0, 0, wt_packed))
                return rc;
            if (lists && gw_in_place)
                if (int rc = d2c_gx_owner_launch<T>(s, base + l.gcol, L, gxcl, st)) return rc;
            if (gw_in_place) {
                D2cProfScope prof(D2C_PROF_PACK, st);
                d2c_fill_zero(base + l.gcol + (size_t)(s.Cin / bkc_of(q.dtype)) * s.K * s.M * bkc_of(q.dtype) * sizeof(T),
                              (size_t)64 * bkc_of(q.dtype) * sizeof(T), st);
            }
            if (auxk)
                if (int rc = d2c_aux_grad_launch<T>(s, xcl_p, off, mask, base + l.gcol, goff_k, gmask,
                                                    (lists && !gw_in_place) ? &L : nullptr,
                                                    (gw_from_col && !columns) ? (gw_in_place ? base + l.gcol : base + l.col) : nullptr,
                                                    gw_in_place, st))
                    return rc;
            if (s.ss.on && goff) {
                D2cProfScope prof(D2C_PROF_PACK, st);
                long gr = ((long)s.N * s.P + 255) / 256;
                if (gr > 8192) gr = 8192;
                if (s.adt == D2C_BF16)
                    hipLaunchKernelGGL(size_grad_finish_kernel<true>, dim3((unsigned)gr), dim3(256), 0, st, s,
                                       (const float *)goff_k, size_raw, goff);
                else
                    hipLaunchKernelGGL(size_grad_finish_kernel<false>, dim3((unsigned)gr), dim3(256), 0, st, s,
                                       (const float *)goff_k, size_raw, goff);
                if (int rc = d2c_check_launch("size_grad_finish_kernel")) return rc;
            }
            if (lists && !gw_in_place)
                if (int rc = d2c_gx_owner_launch<T>(s, base + l.gcol, L, gxcl, st)) return rc;
            if (gx)
                if (int rc = d2c_tiled_unpack_gx<T>(s, gxcl, gx, st)) return rc;
        } else {
            // shapes the fused kernel does not hold on chip: direct kernels (f32 staging in the same region)
            if (int rc = d2c_generic_conv3d_backward(q, gout, x, off, mask, w, gx, goff, gmask, nullptr, nullptr,
                                                     base + l.gxcl, st))
                return rc;
        }
    }
    if (gw && !gw_done) {
        if (columns && d2c_bwd_weight_from_kept_col(s, q.dtype)) gw_from_col = true;   // (also when nothing else was wanted)
        if (d2c_tiled_bwd_weight_supported(s, q.dtype)) {
            if (int rc = d2c_tiled_bwd_weight_launch<T>(s, gout, xcl_p, off, mask, base + l.goutp,
                                                       (float *)(base + l.gwacc),
                                                       gw, gw_from_col ? (columns ? (char *)columns : (gw_in_place ? base + l.gcol : base + l.col)) : nullptr,
                                                       gw_in_place ? (long)s.M : (long)((s.M + 63) / 64) * 64, st))
                return rc;
        } else {
            if (int rc = d2c_generic_conv3d_backward(q, gout, x, off, mask, w, nullptr, nullptr, nullptr, gw, nullptr,
                                                     nullptr, st))
                return rc;
        }
    }
    if (gb) return d2c_tiled_bias_grad<T>(s, gout, gb, st);
    return D2C_OK;
}

}  // namespace

static bool mfma_channels_ok(const d2c_conv3d_desc &q)
{
    if (q.dtype != D2C_BF16 && q.dtype != D2C_F32) return false;
    // the tiled kernels address the channels-last input with 32-bit byte offsets
    if ((size_t)q.N * q.Cin * q.D * q.H * q.W * d2c_elem_size(q.dtype) + 256 >= (1ull << 32)) return false;
    // ... form voxel indices with 24-bit multiplications (corner_row), and address the offsets of the (at most two)
    // samples a position tile meets with 32-bit byte offsets from the first one
    if ((long)q.D * q.H >= (1 << 23) || q.W >= (1 << 23)) return false;
    if ((size_t)2 * q.offset_groups * q.kd * q.kh * q.kw * 3 * q.Do * q.Ho * q.Wo * 4 >= (1ull << 32)) return false;
    // ... and the grad-column rows of one (chunk, tap), 128 bytes per position, through a buffer descriptor
    if ((size_t)q.N * q.Do * q.Ho * q.Wo * 128 + 256 >= (1ull << 32)) return false;
    const int bkc = bkc_of(q.dtype);
    const int cg = q.Cin / q.groups, cpg = q.Cin / q.offset_groups;
    return cg % bkc == 0 && cpg % bkc == 0;
}

// ---- 1-D operator on the matrix-core kernels -----------------------------
// Served when the channel counts fit the chunking and both backward kernels
// can take the shape; otherwise the direct 1-D kernels run.
bool d2c_tiled1d_supported(const d2c_conv1d_desc &q1)
{
    const d2c_conv3d_desc q = as_3d(q1);
    if (!mfma_channels_ok(q)) return false;
    const TiledShape s = tiled_shape(q, 1, q1.reference_quirks);
    return d2c_tiled_bwd_data_supported(s, q.dtype) && d2c_tiled_bwd_weight_supported(s, q.dtype);
}
size_t d2c_tiled1d_forward_ws(const d2c_conv1d_desc &q1)
{
    const d2c_conv3d_desc q = as_3d(q1);
    return fwd_ws(q, tiled_shape(q, 1, 0)).total;
}
size_t d2c_tiled1d_backward_ws(const d2c_conv1d_desc &q1)
{
    const d2c_conv3d_desc q = as_3d(q1);
    return bwd_ws(q, tiled_shape(q, 1, 0)).total;
}
int d2c_tiled1d_forward(const d2c_conv1d_desc &q1, const void *x, const void *off, const void *mask, const void *w,
                        const void *bias, void *out, void *ws, hipStream_t st)
{
    const d2c_conv3d_desc q = as_3d(q1);
    if (q.dtype == D2C_BF16) return forward_t<bf16_t>(q, x, off, mask, w, bias, out, ws, st, 1);
    return forward_t<float>(q, x, off, mask, w, bias, out, ws, st, 1);
}
int d2c_tiled1d_backward(const d2c_conv1d_desc &q1, const void *gout, const void *x, const void *off,
                         const void *mask, const void *w, void *gx, void *goff, void *gmask, void *gw, void *gb,
                         void *ws, hipStream_t st)
{
    const d2c_conv3d_desc q = as_3d(q1);
    if (q.dtype == D2C_BF16)
        return backward_t<bf16_t>(q, gout, x, off, mask, w, gx, goff, gmask, gw, gb, ws, st, 1, q1.reference_quirks);
    return backward_t<float>(q, gout, x, off, mask, w, gx, goff, gmask, gw, gb, ws, st, 1, q1.reference_quirks);
}

bool d2c_tiled_supported(const d2c_conv3d_desc &q)
{
    if (q.dtype != D2C_BF16 && q.dtype != D2C_F32) return false;
    if (is_depthwise(q)) return true;
    return mfma_channels_ok(q);
}

int d2c_tiled_algo(const d2c_conv3d_desc &q) { return is_depthwise(q) ? D2C_ALGO_DEPTHWISE : D2C_ALGO_MFMA; }

// Offsets and mask read inside the layer's deformation tensor, modulation activation in the sampler
// (d2c_conv3d_desc::deform_channels, mask_activation): matrix-core kernels whose backward pass runs the offset / mask
// gradient kernel.
bool d2c_tiled_packed_supported(const d2c_conv3d_desc &q)
{
    if (is_depthwise(q) || !mfma_channels_ok(q)) return false;
    const size_t P = (size_t)q.Do * q.Ho * q.Wo;
    if (q.deform_channels > 0 && (size_t)2 * q.deform_channels * P * 4 >= (1ull << 32)) return false;
    return use_aux_kernel(q, tiled_shape(q));
}

// Offsets held at zero along some axes (offset_axes) are honoured by the tiled kernels only: every part of the
// backward pass has to stay on them too, or the direct kernels that take over would sample with the unzeroed offsets.
bool d2c_tiled_axes_supported(const d2c_conv3d_desc &q)
{
    if (is_depthwise(q) || !mfma_channels_ok(q)) return false;
    const TiledShape s = tiled_shape(q);
    return d2c_tiled_bwd_data_supported(s, q.dtype) && d2c_tiled_bwd_weight_supported(s, q.dtype);
}

size_t d2c_tiled_forward_ws(const d2c_conv3d_desc &q, bool with_stats)
{
    const TiledShape s = tiled_shape(q);
    if (is_depthwise(q)) return dw_ws(q, s).total_fwd;
    return fwd_ws(q, s).total + (with_stats && d2c_fwd_fills_stats(s) ? d2c_fwd_stats_ws(s) : 0);
}

size_t d2c_tiled_backward_ws(const d2c_conv3d_desc &q, const d2c_size_map_desc *sz, bool saved_columns)
{
    const TiledShape s = tiled_shape(q, 3, 0, sz);
    return is_depthwise(q) ? dw_ws(q, s).total_bwd : bwd_ws(q, s, saved_columns).total;
}

// Bytes of the sampled columns that a forward call can keep for the backward call of the same step:
// [chunk][tap][rows][64 bfloat16 / 32 float], rows = position tiles x 64.  0 where the forward kernel does not write them or
// the backward pass cannot multiply over them.
size_t d2c_tiled_columns_bytes(const d2c_conv3d_desc &q, const d2c_size_map_desc *sz)
{
    if (is_depthwise(q) || !mfma_channels_ok(q)) return 0;
    if (sz && !d2c_tiled_sized_supported(q, true)) return 0;
    const TiledShape s = tiled_shape(q, 3, 0, sz);
    if (!d2c_fwd_writes_columns(s, q.dtype) || !d2c_bwd_weight_from_kept_col(s, q.dtype) || !use_aux_kernel(q, s)) return 0;
    const long rows = d2c_columns_rows(s), chunks = s.Cin / bkc_of(q.dtype);
    if (chunks * s.K * rows >= (1L << 31)) return 0;      // (the kernel counts rows in 32 bits)
    return (size_t)chunks * s.K * rows * bkc_of(q.dtype) * d2c_elem_size(q.dtype);
}

// The matrix-core kernels can form the offsets from a size map themselves; the backward pass then needs the
// offset / mask gradient kernel (one pass over the output channels of a weight group).
bool d2c_tiled_sized_supported(const d2c_conv3d_desc &q, bool backward)
{
    if (q.offset_groups != 1 || is_depthwise(q) || !mfma_channels_ok(q)) return false;
    if (!backward) return true;
    return use_aux_kernel(q, tiled_shape(q));
}

int d2c_tiled_forward(const d2c_conv3d_desc &q, const void *x, const void *off, const void *mask, const void *w,
                      const void *bias, void *out, void *ws, hipStream_t st, const d2c_size_map_desc *sz, float *stats,
                      const D2cPrepared *prep, void *columns)
{
    if (q.dtype == D2C_BF16) return forward_t<bf16_t>(q, x, off, mask, w, bias, out, ws, st, 3, sz, stats, prep, columns);
    return forward_t<float>(q, x, off, mask, w, bias, out, ws, st, 3, sz, stats, prep, columns);
}

// Bytes of the caller-held prepared region of a description (0: the kernel family keeps nothing worth holding)
size_t d2c_tiled_prepared_bytes(const d2c_conv3d_desc &q)
{
    if (is_depthwise(q) || !mfma_channels_ok(q)) return 0;
    return prepared_layout(q, tiled_shape(q)).total;
}

// The forward kernels of this description add up per-channel statistics of the output on their way.
bool d2c_tiled_forward_fills_stats(const d2c_conv3d_desc &q)
{
    return !is_depthwise(q) && mfma_channels_ok(q) && d2c_fwd_fills_stats(tiled_shape(q));
}

int d2c_tiled_backward(const d2c_conv3d_desc &q, const void *gout, const void *x, const void *off,
                       const void *mask, const void *w, void *gx, void *goff, void *gmask, void *gw, void *gb,
                       void *ws, hipStream_t st, const d2c_size_map_desc *sz, const D2cPrepared *prep,
                       const void *columns)
{
    if (q.dtype == D2C_BF16)
        return backward_t<bf16_t>(q, gout, x, off, mask, w, gx, goff, gmask, gw, gb, ws, st, 3, 0, sz, prep, columns);
    return backward_t<float>(q, gout, x, off, mask, w, gx, goff, gmask, gw, gb, ws, st, 3, 0, sz, prep, columns);
}
