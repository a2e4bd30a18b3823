/*
 * d2conv.h -- C ABI of the MI355X (gfx950) D2Conv3D operator library.
 *
 * One entry point per native function that the reference's Python extension
 * binds (ops/dconv-native/csrc/ops/dconv.cpp:6-12):
 *
 *   d2c_conv3d_forward    <- deform_conv3d_forward_cuda   (dconv3d_gpu.h:5-16,  dconv3d_gpu.cu:460-560)
 *   d2c_conv3d_backward   <- deform_conv3d_backward_cuda  (dconv3d_gpu.h:18-30, dconv3d_gpu.cu:1261-1332)
 *   d2c_conv1d_forward    <- deform_conv1d_forward_cuda   (dconv1d_gpu.h:6-18,  dconv1d_gpu.cu:102-204)
 *   d2c_conv1d_backward   <- deform_conv1d_backward_cuda  (dconv1d_gpu.h:20-32, dconv1d_gpu.cu:403-542)
 *   d2c_get/set_max_intermediate_elements
 *                         <- get/set_max_intermediate_elements (dconv3d_gpu.cu:12-14, dconv.cpp:9-11)
 *   d2c_conv3d_check / d2c_conv1d_check
 *                         <- SANITY_CHECK_DCONV_GROUPS and the size checks
 *                            (dconv_gpu_common.h:17-24, dconv3d_gpu.cu:504-512)
 *
 * Conventions
 *   - All pointers are device pointers to contiguous tensors in the reference's
 *     layouts:  x [N,Cin,D,H,W], offset [N,G*3*K,Do,Ho,Wo] with channel order
 *     (g, kd, kh, kw, (dz,dy,dx)), mask [N,G*K,Do,Ho,Wo] (may be NULL),
 *     weight [Cout,Cin/groups,kd,kh,kw], bias [Cout] (may be NULL),
 *     out [N,Cout,Do,Ho,Wo]; 1-D: x [N,Cin,L], offset/mask [N,G*K,Lo].
 *   - `dtype` is the element type of x, weight, bias, out and of their
 *     gradients; `aux_dtype` is the element type of offset, mask and their
 *     gradients (equal to dtype, or D2C_F32 when dtype is D2C_BF16).
 *   - The library allocates nothing.  Scratch memory comes from the caller:
 *     ask d2c_*_workspace_bytes() and pass a device buffer of at least that
 *     size, 256-byte aligned.  Its contents are undefined afterwards.
 *   - Every output is fully overwritten; the caller need not clear it.
 *     In the backward calls a NULL gradient pointer skips that gradient.
 *   - `stream` is a hipStream_t (NULL = the default stream).  Calls only
 *     enqueue work; they do not synchronise.
 *   - Return value 0 = success; otherwise a D2C_ERR_* code, with a text for
 *     the calling thread in d2c_last_error().  Nothing throws across the ABI.
 */
#ifndef D2CONV_H
#define D2CONV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { D2C_F32 = 0, D2C_F64 = 1, D2C_BF16 = 2 };

enum {
    D2C_OK = 0,
    D2C_ERR_SHAPE = 1,      /* a check of the reference failed (message names it) */
    D2C_ERR_DTYPE = 2,
    D2C_ERR_WORKSPACE = 3,  /* workspace NULL, misaligned or too small */
    D2C_ERR_LAUNCH = 4,     /* HIP reported an error at launch */
    D2C_ERR_UNSUPPORTED = 5
};

/* Which kernel family a description is served by (d2c_conv3d_algo). */
enum {
    D2C_ALGO_AUTO = 0,
    D2C_ALGO_GENERIC = 1,   /* direct kernels, any shape, f32/f64/bf16 */
    D2C_ALGO_MFMA = 2,      /* implicit GEMM on matrix cores, f32/bf16 */
    D2C_ALGO_DEPTHWISE = 3  /* groups == Cin == Cout, bandwidth kernels */
};

#define D2C_EPILOGUE_NONE 0
#define D2C_EPILOGUE_RELU 1

/* d2c_conv3d_desc::mask_activation */
#define D2C_MASK_ACT_NONE    0
#define D2C_MASK_ACT_SIGMOID 1
#define D2C_MASK_ACT_RELU    2
#define D2C_MASK_ACT_TANH    3

/* d2c_conv3d_desc::backward_flags: how the matrix-core backward pass trades workspace for time.
 * Both d2c_conv3d_backward_workspace_bytes() and d2c_conv3d_backward() read the field from the description they
 * are given, so the size asked for and the call agree per description.  0 = the defaults. */
#define D2C_BWD_GW_DEFAULT   0   /* grad_weight as a matrix product over sampled columns in a buffer of their own */
#define D2C_BWD_GW_COLUMNS   1   /* the same, said explicitly */
#define D2C_BWD_GW_IN_PLACE  2   /* the columns written over the grad-column rows: no buffer of their own
                                  * (bfloat16; float32 problems then sample again) */
#define D2C_BWD_GW_RESAMPLE  3   /* no columns at all: the grad-weight kernel samples the input again */
#define D2C_BWD_GW_MASK      3
/* bits 8..15: number of slices over the offset groups that the backward pass runs in (0 or 1: one pass over all
 * groups).  Buffers of grad-column rows and sampled columns then hold one slice; several offset groups, one weight
 * group and 128 .. 512 output channels only (other descriptions ignore the bits). */
#define D2C_BWD_SLICES(n)    (((n) & 0xff) << 8)
/* float32 problems on the matrix-core kernels: the forward kernels and the grad-column product of the backward pass
 * (from which grad_input, grad_offset and grad_mask follow) carry every float operand as the sum of two bfloat16
 * values on the bfloat16 matrix instruction (a quarter of the matrix-pipe time of the float instruction; results
 * within about 4e-6 of their sums' scale instead of 1e-7, inside 1e-4 relative / 1e-5 absolute at every size
 * measured).  With this bit ALL backward matrix kernels do so -- also the grad-weight kernel that samples again
 * (D2C_BWD_GW_RESAMPLE, 1-D problems, calls that want neither grad_offset nor grad_mask), whose elements (sums over
 * all positions, tens to hundreds in size) then miss 1e-5 absolute -- and the 1-D and fallback kernels.  The
 * grad-weight product over sampled columns is not touched by it: that one takes every float apart into three
 * bfloat16 terms, which keeps float32's accuracy.  Off by default. */
#define D2C_BWD_F32_SPLIT    0x10000

typedef struct d2c_conv3d_desc {
    int32_t N, Cin, Cout;
    int32_t D, H, W;
    int32_t kd, kh, kw;
    int32_t sd, sh, sw;
    int32_t pd, ph, pw;
    int32_t dd, dh, dw;
    int32_t groups, offset_groups;
    int32_t Do, Ho, Wo;   /* spatial size of offset / mask / out as passed by the caller */
    int32_t dtype, aux_dtype;
    /* What the forward kernels do to a value (bias included) before they store it: nothing, or
     * epilogue_scale * max(value, 0) -- the ReLU / ScaledReLU that follows every deformable convolution of the
     * reference's refinement modules (network/modules/refinement.py:38-43, network/layers.py:409-419), saving the
     * separate pass over the output.  The backward call ignores these fields: it expects the gradient with respect
     * to the value before the activation (grad_out * epilogue_scale where out > 0, else 0). */
    int32_t epilogue;     /* D2C_EPILOGUE_NONE or D2C_EPILOGUE_RELU */
    float epilogue_scale;
    /* Which axes the sampling points are displaced along: bit 0 = z (temporal), bit 1 = y, bit 2 = x; 0 means all
     * three.  For a cleared axis the offsets are taken as zero whatever the tensor holds, and its grad_offset
     * channels come back zero: the Spatial (y, x: 6) and Temporal (z: 1) layers of the reference, which overwrite
     * those channels of a cloned offsets tensor (dconv_native/modules.py:87-120).  With an axis fixed a sampling
     * point sits on a voxel plane of it and the four corners on the far plane have weight zero; the kernels do not
     * fetch them.  Served by the matrix-core kernels only: other descriptions answer D2C_ERR_UNSUPPORTED (zero the
     * channels in a copy of the tensor instead). */
    int32_t offset_axes;
    /* D2C_BWD_GW_* | D2C_BWD_SLICES(n); 0 = defaults.  Forward calls ignore it. */
    int32_t backward_flags;
    /* The deformation branch of the self-deforming layers (network/layers.py:107-132, dconv_native/modules.py:71-84)
     * writes offsets and modulation into ONE tensor [N, deform_channels, Do, Ho, Wo] and the reference splits it and
     * applies the modulation activation before the operator sees either part.  deform_channels > 0 lets the operator
     * read that tensor where it lies: `offset` (or the size map of the d2c_conv3d_sized_* calls) and `mask` then
     * point at their first channels INSIDE it, consecutive samples are deform_channels * Do*Ho*Wo elements apart in
     * both, and grad_offset / grad_mask point likewise into one gradient tensor of that shape (channels of it
     * that belong to neither are not written).  mask_activation != D2C_MASK_ACT_NONE makes the sampler apply that
     * function to every mask value it reads (rounded to aux_dtype, like the tensor the reference's activation
     * writes), and grad_mask comes back with respect to the raw values.  0 / 0: tensors of their own, mask used as it is.
     * Matrix-core kernels only (and, in the backward call, offset groups that lie inside one weight group):
     * other descriptions answer D2C_ERR_UNSUPPORTED. */
    int32_t deform_channels;
    int32_t mask_activation;
} d2c_conv3d_desc;

typedef struct d2c_conv1d_desc {
    int32_t N, Cin, Cout;
    int32_t L, k, s, p, d;
    int32_t groups, offset_groups;
    int32_t Lo;
    int32_t dtype, aux_dtype;
    int32_t reference_quirks; /* !=0: integer-position rule of dconv1d_gpu.cu:332-336 in grad_offset/grad_mask */
} d2c_conv1d_desc;

/* get_output_size, dconv_gpu_common.h:13-15 */
int32_t d2c_output_size(int32_t in, int32_t k, int32_t stride, int32_t pad, int32_t dil);

int d2c_conv3d_check(const d2c_conv3d_desc *desc);
int d2c_conv3d_algo(const d2c_conv3d_desc *desc);
/* 1 when a description with deform_channels > 0 and / or a mask_activation is served (forward and backward; with
 * `size_map` != NULL: through the d2c_conv3d_sized_* calls), else 0: the caller then splits the deformation tensor
 * and applies the activation itself, as the reference does (network/layers.py:107-120). */
struct d2c_size_map_desc;
int d2c_conv3d_packed_supported(const d2c_conv3d_desc *desc, const struct d2c_size_map_desc *size_map);
size_t d2c_conv3d_forward_workspace_bytes(const d2c_conv3d_desc *desc);
size_t d2c_conv3d_backward_workspace_bytes(const d2c_conv3d_desc *desc);

int d2c_conv3d_forward(const d2c_conv3d_desc *desc, const void *x, const void *offset,
                       const void *mask, const void *weight, const void *bias, void *out,
                       void *workspace, size_t workspace_bytes, void *stream);

/*
 * d2c_conv3d_forward without a workspace argument and without any allocation.  It has no counterpart in the
 * reference; it is for callers that cannot allocate device memory around the call: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The scratch memory is an array of
 * D2C_STATIC_WORKSPACE_BYTES inside the library's device image (each GPU the library runs on holds its own
 * copy until the process ends); the call makes no hipMalloc / hipFree and uses no allocating library routine.
 * A description whose d2c_conv3d_forward_workspace_bytes() exceeds that size is refused with
 * D2C_ERR_WORKSPACE.  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU
 * (different streams or threads) race; serialise them.  Otherwise identical to d2c_conv3d_forward
 * (same kernels, same results).  Instrumentation (d2c_profile_enable) must be off: it creates events.
 */
#define D2C_STATIC_WORKSPACE_BYTES (32u << 20)
size_t d2c_static_workspace_bytes(void);
int d2c_conv3d_forward_static(const d2c_conv3d_desc *desc, const void *x, const void *offset,
                              const void *mask, const void *weight, const void *bias, void *out,
                              void *stream);

int d2c_conv3d_backward(const d2c_conv3d_desc *desc, const void *grad_out, const void *x,
                        const void *offset, const void *mask, const void *weight,
                        void *grad_x, void *grad_offset, void *grad_mask, void *grad_weight,
                        void *grad_bias, void *workspace, size_t workspace_bytes, void *stream);

/*
 * The sampled columns of a forward call, kept for the backward call of the same training step (optional).
 * The reference samples the input a second time in its backward pass (ops/dconv-native/csrc/ops/dconv3d_gpu.cu:
 * 1037-1088, the im2col call in front of the grad-weight product) and so does d2c_conv3d_backward.  A caller with
 * memory to spare hands d2c_conv3d_forward_columns a buffer of d2c_conv3d_columns_bytes() bytes (256-byte aligned;
 * taps x the size of the input, in the element type): the forward kernel writes there what it multiplies with the
 * weights anyway, and d2c_conv3d_backward_columns, given that buffer UNCHANGED together with the same tensors, runs
 * its grad-weight product over it instead of sampling again (N=2, C=512, 8x30x54, bfloat16: 2.46 -> 2.39 ms per step
 * for 717 MB held between the two calls, and 0.72 GB less backward workspace; N=2, C=256, 8x30x54, float32: 2.77 ->
 * 2.25 ms for 717 MB).  Results are those of the plain calls up to the order of floating-point sums; float32
 * columns are the interpolated floats themselves and their product keeps float32's accuracy (three bfloat16 terms
 * per float on the bfloat16 matrix instruction, or the float32 instruction), whatever D2C_BWD_F32_SPLIT says.  `size_map` as in d2c_conv3d_forward_stats: NULL, or the description of
 * the size map that `offset` then is.  d2c_conv3d_columns_bytes() is 0 where this is not served (anything but
 * bfloat16 and float32 problems on the matrix-core kernels with at least 48 tiles of 64 output positions (times
 * weight groups), offsets along all three axes and an even number of 64- / 32-channel chunks per weight group); the
 * two calls then
 * fail with D2C_ERR_UNSUPPORTED and the caller uses the plain ones.  The memory-saving bits of
 * d2c_conv3d_desc::backward_flags are ignored by d2c_conv3d_backward_columns.
 */
struct d2c_size_map_desc;
size_t d2c_conv3d_columns_bytes(const d2c_conv3d_desc *desc, const struct d2c_size_map_desc *size_map);
int d2c_conv3d_forward_columns(const d2c_conv3d_desc *desc, const struct d2c_size_map_desc *size_map, const void *x,
                               const void *offset, const void *mask, const void *weight, const void *bias, void *out,
                               void *columns, size_t columns_bytes, void *workspace, size_t workspace_bytes,
                               void *stream);
size_t d2c_conv3d_backward_columns_workspace_bytes(const d2c_conv3d_desc *desc,
                                                   const struct d2c_size_map_desc *size_map);
int d2c_conv3d_backward_columns(const d2c_conv3d_desc *desc, const struct d2c_size_map_desc *size_map,
                                const void *grad_out, const void *x, const void *offset, const void *mask,
                                const void *weight, const void *columns, size_t columns_bytes, void *grad_x,
                                void *grad_offset, void *grad_mask, void *grad_weight, void *grad_bias,
                                void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same two calls with a caller-held "prepared" region (no counterpart in the reference, whose column pipeline
 * re-lays nothing out): the matrix-core kernels work on a channels-last copy of the input and on weights in the
 * order their matrix instructions read them, which every call makes anew in its workspace.  A caller that keeps a
 * region of d2c_conv3d_prepared_bytes() bytes (256-byte aligned) per layer lets the calls make them THERE and
 * tells later calls what it still holds:
 *   D2C_REUSE_INPUT             the region holds the copy of THIS input `x` (made by a call on the same x):
 *                               the backward call of a training step after its forward call;
 *   D2C_REUSE_FORWARD_WEIGHTS   ... the forward operand of THIS weight tensor: forward calls while the weights
 *                               do not change (inference);
 *   D2C_REUSE_BACKWARD_WEIGHTS  ... the backward operand of this weight tensor (made by a backward call).
 * Parts not named are made by the call (and may be named in the next one).  Results are those of the plain calls
 * (the same kernels on the same operands).  d2c_conv3d_prepared_bytes() is 0 for descriptions the other kernel families serve; the calls
 * then ignore `prepared` and `reuse`.  The workspace is needed as before.
 */
#define D2C_REUSE_INPUT            1
#define D2C_REUSE_FORWARD_WEIGHTS  2
#define D2C_REUSE_BACKWARD_WEIGHTS 4
size_t d2c_conv3d_prepared_bytes(const d2c_conv3d_desc *desc);
int d2c_conv3d_forward_prepared(const d2c_conv3d_desc *desc, const void *x, const void *offset, const void *mask,
                                const void *weight, const void *bias, void *out, void *prepared,
                                size_t prepared_bytes, int32_t reuse, void *workspace, size_t workspace_bytes,
                                void *stream);
int d2c_conv3d_backward_prepared(const d2c_conv3d_desc *desc, const void *grad_out, const void *x,
                                 const void *offset, const void *mask, const void *weight, void *grad_x,
                                 void *grad_offset, void *grad_mask, void *grad_weight, void *grad_bias,
                                 void *prepared, size_t prepared_bytes, int32_t reuse, void *workspace,
                                 size_t workspace_bytes, void *stream);

int d2c_conv1d_check(const d2c_conv1d_desc *desc);
int d2c_conv1d_algo(const d2c_conv1d_desc *desc);   /* D2C_ALGO_GENERIC or D2C_ALGO_MFMA */
size_t d2c_conv1d_forward_workspace_bytes(const d2c_conv1d_desc *desc);
size_t d2c_conv1d_backward_workspace_bytes(const d2c_conv1d_desc *desc);

int d2c_conv1d_forward(const d2c_conv1d_desc *desc, const void *x, const void *offset,
                       const void *mask, const void *weight, const void *bias, void *out,
                       void *workspace, size_t workspace_bytes, void *stream);

int d2c_conv1d_backward(const d2c_conv1d_desc *desc, const void *grad_out, const void *x,
                        const void *offset, const void *mask, const void *weight,
                        void *grad_x, void *grad_offset, void *grad_mask, void *grad_weight,
                        void *grad_bias, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Sampling bookkeeping of the forward pass, for index-exactness checks
 * (trilinear_interpolate, dconv3d_gpu.cu:59-86): per (n, g*K+k, p)
 *   base[.][3] = floor(z), floor(y), floor(x) as int32 (positions beyond 4
 *                voxels outside the volume are clamped there first),
 *   flags[.]   = bit c set (c = 4*dz + 2*dy + dx) when corner c is read.
 */
int d2c_conv3d_corner_index(const d2c_conv3d_desc *desc, const void *offset, int32_t *base,
                            uint8_t *flags, void *stream);

/*
 * The sampler alone, for what samples other tensors at the operator's sampling points: the reference's modulation
 * loss reads a ground-truth mask at every deformed tap with torch's grid_sample on a zero-padded copy
 * (loss/region.py:97-125), which is the forward pass's trilinear rule on a one-channel input.
 *   src [N, src_channels, D, H, W] (element type `dtype`), offset as in d2c_conv3d_forward,
 *   out [N, G*K*src_channels, Do, Ho, Wo]: out[n, (g*K + k)*src_channels + c, p] = trilinear(src[n, c], pos(n, g, k, p)),
 * 0 for positions outside (-1, size), corners outside the volume read as 0 (dconv3d_gpu.cu:48-109); no
 * modulation, no weights.  Only N, D, H, W, the kernel / stride / padding / dilation fields, offset_groups, Do, Ho,
 * Wo, dtype and aux_dtype of the description are used (Cin, Cout, groups must still pass d2c_conv3d_check).
 */
int d2c_conv3d_sample(const d2c_conv3d_desc *desc, int32_t src_channels, const void *src, const void *offset,
                      void *out, void *stream);

/*
 * Histogram of an offset field per axis (the debug output that the reference's trainer expects from a hook its
 * repository does not contain, trainer.py:99-101): hist[3][nbins + 2] of uint64 in device memory, overwritten;
 * per axis (z, y, x): [0] values below lo, [1 .. nbins] the nbins equal-width bins of [lo, hi), [nbins + 1] values
 * at or above hi (NaN included).  1 <= nbins <= 1024.
 */
int d2c_conv3d_offset_histogram(const d2c_conv3d_desc *desc, const void *offset, float lo, float hi,
                                int32_t nbins, uint64_t *hist, void *stream);

/* Accepted for interface parity; the library never materialises the column
 * buffer that this limit governs in the reference (dconv3d_gpu.cu:536-553). */
uint64_t d2c_get_max_intermediate_elements(void);
void d2c_set_max_intermediate_elements(uint64_t m);

/* Test hook, not for production callers: force a kernel family (D2C_ALGO_*;
 * D2C_ALGO_AUTO restores the default choice).  A forced family that cannot
 * serve a description makes the call fail with D2C_ERR_UNSUPPORTED.  The
 * setting is one per process (an atomic; every device and thread sees it) and
 * both the *_workspace_bytes queries and the calls read it: changing it from
 * another thread between a query and its call makes that call fail with
 * D2C_ERR_WORKSPACE at worst, never write out of bounds, but the hook is not
 * meant to be flipped while calls are in flight.  The same holds for
 * d2c_set_grad_input_mode() below. */
void d2c_set_algo_override(int algo);

/*
 * Instrumentation (no counterpart in the reference): when enabled, the main
 * kernels are bracketed by HIP events on the stream they are launched on.
 * d2c_profile_read() waits for the recorded events, adds their elapsed times
 * to the totals of kernel `id` (D2C_PROF_*) and returns them; d2c_profile_reset
 * clears the totals.  Enabling it creates events, i.e. it is not for hot loops
 * that must not allocate.
 */
enum {
    D2C_PROF_FWD = 0,         /* forward implicit-GEMM / depthwise kernel */
    D2C_PROF_BWD_DATA = 1,    /* grad-column product (+ grad_offset / grad_mask / scatter when fused) */
    D2C_PROF_BWD_WEIGHT = 2,  /* grad_weight kernel */
    D2C_PROF_PACK = 3,        /* layout changes, clears, conversions, sample lists (sum) */
    D2C_PROF_GX_OWNER = 4,    /* grad_input accumulation from the sample lists */
    D2C_PROF_BWD_AUX = 5,     /* grad_offset / grad_mask from the grad-column rows */
    D2C_PROF_COUNT = 6
};
void d2c_profile_enable(int on);
void d2c_profile_reset(void);
int d2c_profile_read(int id, double *total_ms, int *launches);
/* Name of the kernel last launched under `id` since the last reset ("" if none): the name a profiler trace
 * shows, without template arguments. */
const char *d2c_profile_kernel_name(int id);

/* ---- dynamic-dilation front end -------------------------------------------------------
 * The step in front of the operator in the size-conditioned layers: the predicted size map
 * becomes tap offsets.  Replaces, in one kernel each way, the torch operations of
 * network/layers.py:171-181 (_apply_size_activation), utils/grid.py:83-93 (axes the mode does
 * not predict get size 1) and utils/grid.py:95-98 / dconv_native/grid.py:62-80
 * (offsets_from_size_map):
 *     offsets[n, 3*k + a, p] = base_a[k_a] * (act(size_raw)[n, channel(a), p] - 1),
 *     k = (kz*kh + ky)*kw + kx;  base_a = linspace(-dil_a*(k_a/2), dil_a*(k_a/2), k_a), passed in.
 * size_raw is [N, 3 | 2 | 2 | 1, P] for mode XYZ | XXZ (z, x; y = x) | XY (y, x) | X (y = x),
 * offsets is [N, 3*K, P]; both in `dtype` (float32 or bfloat16).  The backward call turns
 * grad_offsets into grad_size_raw (activation derivative included). */
#define D2C_SIZE_MAX_K 16
enum { D2C_SIZE_XYZ = 0, D2C_SIZE_XXZ = 1, D2C_SIZE_XY = 2, D2C_SIZE_X = 3 };
enum {
    D2C_SIZE_ACT_LINEAR = 0,        /* x */
    D2C_SIZE_ACT_ELU = 1,           /* ELU(x) + 1 */
    D2C_SIZE_ACT_RELU = 2,          /* ReLU(x + 1) */
    D2C_SIZE_ACT_RELU_PLUS_ONE = 3  /* ReLU(x + 1e-3) + 1 */
};
typedef struct d2c_size_map_desc {
    int32_t N, P;             /* samples, positions per sample (Do*Ho*Wo) */
    int32_t kd, kh, kw;
    int32_t mode, activation;
    int32_t dtype;
    float base_z[D2C_SIZE_MAX_K], base_y[D2C_SIZE_MAX_K], base_x[D2C_SIZE_MAX_K];
} d2c_size_map_desc;
int d2c_size_map_offsets_forward(const d2c_size_map_desc *desc, const void *size_raw, void *offsets, void *stream);
int d2c_size_map_offsets_backward(const d2c_size_map_desc *desc, const void *size_raw, const void *grad_offsets,
                                  void *grad_size_raw, void *stream);

/* The deformable convolution fed by the size map itself (no counterpart as ONE call in the reference: it replaces
 * network/layers.py:171-181 + utils/grid.py:72-98 + deform_conv3d_forward/backward_cuda for the size-conditioned
 * layers, network/layers.py:184-313).  `size_raw` [N, 3|2|2|1, Do, Ho, Wo] is the prediction before the size
 * activation, in the element type `aux_dtype` of the mask; the convolution description must have
 * offset_groups == 1 and `sdesc` the same N, kernel extents and P = Do*Ho*Wo.  Where the matrix-core kernels serve
 * the description, the sampler forms base_a[k_a] * (act(size_raw) - 1) where it needs a tap's offsets and no
 * [N, 3K, P] offsets tensor (nor its gradient) exists; other descriptions expand the map inside the workspace
 * and run the ordinary kernels.  Results equal d2c_size_map_offsets_forward followed by d2c_conv3d_forward (bit
 * for bit in the forward pass).  `grad_size_raw` (may be NULL) has the shape of size_raw. */
size_t d2c_conv3d_sized_forward_workspace_bytes(const d2c_conv3d_desc *desc, const d2c_size_map_desc *sdesc);
size_t d2c_conv3d_sized_backward_workspace_bytes(const d2c_conv3d_desc *desc, const d2c_size_map_desc *sdesc);
int d2c_conv3d_sized_forward(const d2c_conv3d_desc *desc, const d2c_size_map_desc *sdesc, const void *x,
                             const void *size_raw, const void *mask, const void *weight, const void *bias, void *out,
                             void *workspace, size_t workspace_bytes, void *stream);
int d2c_conv3d_sized_backward(const d2c_conv3d_desc *desc, const d2c_size_map_desc *sdesc, const void *grad_out,
                              const void *x, const void *size_raw, const void *mask, const void *weight, void *grad_x,
                              void *grad_size_raw, void *grad_mask, void *grad_weight, void *grad_bias,
                              void *workspace, size_t workspace_bytes, void *stream);

/* ---- normalisation behind the convolution ------------------------------------------------------------------
 * Every deformable convolution of the reference's refinement modules is followed by an activation and a
 * GroupNorm (network/modules/refinement.py:38-43: Sequential(ConvType, ActivationType, NormType)).
 * d2c_conv3d_forward_stats is d2c_conv3d_forward (sdesc == NULL, `offset` = the offsets tensor) or
 * d2c_conv3d_sized_forward (sdesc != NULL, `offset` = the raw size map) that also returns
 *     chan_stats[n][c] = (sum_p out[n,c,p], sum_p out[n,c,p]^2)        float32 [N][Cout][2],
 * of the values as stored (bias and epilogue applied, rounded to `dtype`).  The matrix-core kernels for wide
 * weight groups add these sums up where they store the output (per position tile, without atomics; a small kernel
 * adds the tiles of a sample up); other descriptions run d2c_channel_stats behind the convolution.  Workspace:
 * d2c_conv3d_forward_stats_workspace_bytes().
 * d2c_group_norm_forward / _backward are torch.nn.functional.group_norm and its gradients (biased variance,
 * var = sumsq / m - mean^2 in float32) from such statistics: one pass over x each way plus a reduction pass for the
 * backward sums; gamma, beta (may be NULL: 1, 0) and their gradients in `dtype`. */
typedef struct d2c_group_norm_desc {
    int32_t N, C, P;          /* samples, channels, positions per channel */
    int32_t groups;           /* normalisation groups; must divide C */
    int32_t dtype;            /* D2C_F32 or D2C_BF16 */
    float eps;
} d2c_group_norm_desc;
size_t d2c_conv3d_forward_stats_workspace_bytes(const d2c_conv3d_desc *desc, const d2c_size_map_desc *sdesc);
int d2c_conv3d_forward_stats(const d2c_conv3d_desc *desc, const d2c_size_map_desc *sdesc, const void *x,
                             const void *offset, const void *mask, const void *weight, const void *bias, void *out,
                             float *chan_stats, void *workspace, size_t workspace_bytes, void *stream);
int d2c_channel_stats(const d2c_group_norm_desc *desc, const void *x, float *chan_stats, void *stream);
int d2c_group_norm_forward(const d2c_group_norm_desc *desc, const void *x, const float *chan_stats, const void *gamma,
                           const void *beta, void *y, void *stream);
size_t d2c_group_norm_backward_workspace_bytes(const d2c_group_norm_desc *desc);
int d2c_group_norm_backward(const d2c_group_norm_desc *desc, const void *grad_y, const void *x,
                            const float *chan_stats, const void *gamma, void *grad_x, void *grad_gamma,
                            void *grad_beta, void *workspace, size_t workspace_bytes, void *stream);

/* ---- plain depthwise conv3d (no sampling) ------------------------------------------------
 * The operator of the reference's second extension, ops/fast-depthwise-conv3d, which its
 * backbone uses for the channel-separated 3x3x3 convolutions (network/backbone/resnet.py:110):
 *   d2c_dwconv3d_forward   <- conv_depthwise3d_cuda           (csrc/grouped_conv3d.cu:22-92, 385-470)
 *   d2c_dwconv3d_backward  <- conv_depthwise3d_backward_cuda  (csrc/grouped_conv3d.cu:93-276, 510-665)
 *   d2c_dwconv3d_check     <- conv_depthwise_shape_check      (csrc/grouped_conv3d.cu:279-345)
 * x [N,C,D,H,W], weight [Cout,1,kd,kh,kw] with Cout a multiple of C (output channel co reads
 * input channel co / (Cout/C)), bias [Cout] or NULL, out [N,Cout,Do,Ho,Wo]; all in `dtype`
 * (float32, float64 or bfloat16; sums in float32, float64 for float64).  In the backward call
 * a NULL gradient pointer skips that gradient; grad_weight and grad_bias need the workspace. */
typedef struct d2c_dwconv3d_desc {
    int32_t N, C, Cout;
    int32_t D, H, W;
    int32_t kd, kh, kw;
    int32_t sd, sh, sw;
    int32_t pd, ph, pw;
    int32_t dd, dh, dw;
    int32_t Do, Ho, Wo;       /* must equal (in + 2p - (d(k-1)+1))/s + 1 */
    int32_t dtype;
} d2c_dwconv3d_desc;
int d2c_dwconv3d_check(const d2c_dwconv3d_desc *desc);
size_t d2c_dwconv3d_backward_workspace_bytes(const d2c_dwconv3d_desc *desc);
int d2c_dwconv3d_forward(const d2c_dwconv3d_desc *desc, const void *x, const void *weight, const void *bias,
                         void *out, void *stream);
int d2c_dwconv3d_backward(const d2c_dwconv3d_desc *desc, const void *grad_out, const void *x, const void *weight,
                          void *grad_x, void *grad_weight, void *grad_bias, void *workspace,
                          size_t workspace_bytes, void *stream);

/* Test hook for the matrix-core backward pass: 1 (default) builds grad_input from
 * per-voxel sample lists, every element written once; 0 scatters with fp32 atomics
 * like the reference (dconv3d_gpu.cu:637).  A value n >= 2 is mode 1 with lists
 * that hold at most n samples per voxel before the overflow path takes the rest
 * (by default the capacity follows from the shape).  Workspace sizes depend on the mode.
 * One setting per process, for tests only (see d2c_set_algo_override). */
void d2c_set_grad_input_mode(int mode);

/* Test hooks, not for production callers (those set d2c_conv3d_desc::backward_flags, which wins over the hooks
 * wherever it says something): the grad-weight path of the matrix-core backward pass for
 * descriptions whose backward_flags leave it at the default -- 1 (the library's default) lets the offset / mask
 * gradient kernel write the sampled columns, over which grad_weight then runs as a plain matrix product (the
 * reference's formulation, dconv3d_gpu.cu:1037-1088, with the column buffer filled by the kernel that has the
 * corner values in registers anyway); 2 is the same with the columns written over the grad-column rows (no buffer
 * of their own; grad_input is then taken from the rows first, from sample lists that a pass of their own files,
 * which costs part of the gain); 0 makes the grad-weight kernel sample the input again, which is also what happens
 * whenever the caller wants neither grad_offset nor grad_mask.  Workspace sizes depend on the mode.  One setting
 * per process (see d2c_set_algo_override). */
void d2c_set_grad_weight_mode(int mode);

/* ... and the number of slices over the offset groups for descriptions whose backward_flags name none (see
 * D2C_BWD_SLICES): 0 or 1 = one pass over all groups (the library's default), n >= 2 = n slices. */
void d2c_set_backward_slices(int n);

const char *d2c_last_error(void);
/* Version of this interface.  2: d2c_conv3d_desc ends in backward_flags, deform_channels and mask_activation, and the
 * _prepared, _columns, _sized, _stats, sample / histogram entry points exist.  A binding checks it before it fills a
 * description. */
int d2c_version(void);

#ifdef __cplusplus
}
#endif
#endif /* D2CONV_H */
