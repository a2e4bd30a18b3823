/*
 * TEST INFRASTRUCTURE ONLY.  CPU oracle for the D2Conv3D operator path: a
 * restatement in plain C of the reference's CUDA pipeline
 * (ops/dconv-native/csrc/ops/dconv3d_gpu.cu, dconv1d_gpu.cu).  It is the
 * checker for tests, the smoke check and the benchmark's CPU-baseline leg and
 * is never linked into, or called from, the shipped library.
 *
 * All tensors are contiguous, in the reference's layouts:
 *   x     [N, Cin, D, H, W]            offset [N, G*3*K, Do, Ho, Wo]
 *   mask  [N, G*K, Do, Ho, Wo] or NULL weight [Cout, Cin/groups, kd, kh, kw]
 *   bias  [Cout] or NULL               out    [N, Cout, Do, Ho, Wo]
 * offset channel order is (g, kd, kh, kw, (dz, dy, dx)).
 */
#ifndef D2C_ORACLE_H
#define D2C_ORACLE_H
#include <stdint.h>

typedef struct {
    int N, Cin, Cout;
    int D, H, W;
    int kd, kh, kw;
    int sd, sh, sw;
    int pd, ph, pw;
    int dd, dh, dw;
    int groups, offset_groups;
    int Do, Ho, Wo;
} oracle_conv3d_desc;

typedef struct {
    int N, Cin, Cout;
    int L, k, s, p, d;
    int groups, offset_groups;
    int Lo;
} oracle_conv1d_desc;

/* dconv_gpu_common.h:13-15 */
int oracle_output_size(int in, int k, int stride, int pad, int dil);

#define ORACLE_DECL(T, S)                                                                      \
    int oracle_conv3d_forward_##S(const T *x, const T *off, const T *mask, const T *w,         \
                                  const T *bias, T *out, const oracle_conv3d_desc *q);         \
    int oracle_conv3d_backward_##S(const T *gout, const T *x, const T *off, const T *mask,     \
                                   const T *w, T *gx, T *goff, T *gmask, T *gw, T *gb,         \
                                   const oracle_conv3d_desc *q);                               \
    int oracle_conv3d_corners_##S(const T *off, const oracle_conv3d_desc *q, int32_t *base,    \
                                  uint8_t *flags);                                             \
    int oracle_conv1d_forward_##S(const T *x, const T *off, const T *mask, const T *w,         \
                                  const T *bias, T *out, const oracle_conv1d_desc *q);         \
    int oracle_conv1d_backward_##S(const T *gout, const T *x, const T *off, const T *mask,     \
                                   const T *w, T *gx, T *goff, T *gmask, T *gw, T *gb,         \
                                   const oracle_conv1d_desc *q, int quirks);
ORACLE_DECL(float, f32)
ORACLE_DECL(double, f64)
#undef ORACLE_DECL

int oracle_num_threads(void);
#endif
