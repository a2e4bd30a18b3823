// Host interface of the tiled kernel families (matrix-core implicit GEMM and
// the depthwise bandwidth kernels).
#pragma once
#include "d2c_common.hpp"

bool d2c_tiled_supported(const d2c_conv3d_desc &q);
int d2c_tiled_algo(const d2c_conv3d_desc &q);  // D2C_ALGO_MFMA or D2C_ALGO_DEPTHWISE
// whether a description that reads offsets and mask inside one deformation tensor, or applies a modulation
// activation in the sampler, is served (in both directions)
bool d2c_tiled_packed_supported(const d2c_conv3d_desc &q);
// whether a description with some offset axes fixed (offset_axes != 7) stays on the tiled kernels in both directions
bool d2c_tiled_axes_supported(const d2c_conv3d_desc &q);
size_t d2c_tiled_forward_ws(const d2c_conv3d_desc &q, bool with_stats = false);
// `sz` != nullptr: the offsets are formed from a raw size map (`off` is that map [N, channels(mode), P], `goff` the
// gradient with respect to it); only where d2c_tiled_sized_supported() says so.
// `saved_columns`: for a backward call that is handed the sampled columns of its forward call (d2c_tiled_columns_bytes)
size_t d2c_tiled_backward_ws(const d2c_conv3d_desc &q, const d2c_size_map_desc *sz = nullptr, bool saved_columns = false);
size_t d2c_tiled_columns_bytes(const d2c_conv3d_desc &q, const d2c_size_map_desc *sz = nullptr);
bool d2c_tiled_sized_supported(const d2c_conv3d_desc &q, bool backward);
// `stats` != nullptr (only where d2c_tiled_forward_fills_stats() says so): fp32 [N][Cout][2], the sum and the sum of
// squares of the stored output per (sample, channel).
bool d2c_tiled_forward_fills_stats(const d2c_conv3d_desc &q);
// `prep` != nullptr: a caller-held region of d2c_tiled_prepared_bytes() bytes that takes the place of the
// workspace's channels-last input and packed weights; the parts named in `reuse` (D2C_REUSE_*) are taken as they are.
struct D2cPrepared {
    void *base;
    int reuse;
};
size_t d2c_tiled_prepared_bytes(const d2c_conv3d_desc &q);
int d2c_tiled_forward(const d2c_conv3d_desc &q, const void *x, const void *off, const void *mask, const void *w,
                      const void *bias, void *out, void *ws, hipStream_t st, const d2c_size_map_desc *sz = nullptr,
                      float *stats = nullptr, const D2cPrepared *prep = nullptr, void *columns = nullptr);
int d2c_tiled_backward(const d2c_conv3d_desc &q, const void *gout, const void *x, const void *off,
                       const void *mask, const void *w, void *gx, void *goff, void *gmask, void *gw, void *gb,
                       void *ws, hipStream_t st, const d2c_size_map_desc *sz = nullptr, const D2cPrepared *prep = nullptr,
                       const void *columns = nullptr);

// 1-D operator served by the same matrix-core kernels (1 x 1 x L volume).
bool d2c_tiled1d_supported(const d2c_conv1d_desc &q);
size_t d2c_tiled1d_forward_ws(const d2c_conv1d_desc &q);
size_t d2c_tiled1d_backward_ws(const d2c_conv1d_desc &q);
int d2c_tiled1d_forward(const d2c_conv1d_desc &q, const void *x, const void *off, const void *mask, const void *w,
                        const void *bias, void *out, void *ws, hipStream_t st);
int d2c_tiled1d_backward(const d2c_conv1d_desc &q, const void *gout, const void *x, const void *off,
                         const void *mask, const void *w, void *gx, void *goff, void *gmask, void *gw, void *gb,
                         void *ws, hipStream_t st);
