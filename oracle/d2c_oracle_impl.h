/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference operator.
 *
 * This file is included twice by d2c_oracle.c, once with T = float and once
 * with T = double (the two element types the reference dispatches on,
 * ops/dconv-native/csrc/ops/dconv3d_gpu.cu:235).  Nothing in the shipped
 * library links or calls it; only tests, the smoke check and the CPU-baseline
 * leg of the benchmark do.
 *
 * Every function names the reference lines it restates.  The reference
 * pipeline is kept as is: sample into a column buffer, GEMM per weight group,
 * and in the backward pass grad-column GEMM -> offset/mask gradient ->
 * scatter into grad_input -> re-sample -> grad-weight GEMM.
 * The GEMMs stand in for cuBLAS (summation order unspecified there); they
 * accumulate in double so that the oracle is the more accurate side of any
 * tolerance comparison.
 */

#define CAT_(a, b) a##_##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUFFIX)

/* ---- dconv3d_gpu.cu:48-109  trilinear_interpolate --------------------- */
static T FN(trilinear)(const T *in, int depth, int height, int width,
                       T d, T h, T w)
{
    if (d <= -1 || depth <= d || h <= -1 || height <= h || w <= -1 || width <= w)
        return 0;
    int d0 = (int)FLOOR(d), h0 = (int)FLOOR(h), w0 = (int)FLOOR(w);
    int d1 = d0 + 1, h1 = h0 + 1, w1 = w0 + 1;
    T pt[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (d0 >= 0 && h0 >= 0 && w0 >= 0)
        pt[0] = in[(d0 * height + h0) * width + w0];
    if (d0 >= 0 && h0 >= 0 && w1 <= width - 1)
        pt[1] = in[(d0 * height + h0) * width + w1];
    if (d0 >= 0 && h1 <= height - 1 && w0 >= 0)
        pt[2] = in[(d0 * height + h1) * width + w0];
    if (d0 >= 0 && h1 <= height - 1 && w1 <= width - 1)
        pt[3] = in[(d0 * height + h1) * width + w1];
    if (d1 <= depth - 1 && h0 >= 0 && w0 >= 0)
        pt[4] = in[(d1 * height + h0) * width + w0];
    if (d1 <= depth - 1 && h0 >= 0 && w1 <= width - 1)
        pt[5] = in[(d1 * height + h0) * width + w1];
    if (d1 <= depth - 1 && h1 <= height - 1 && w0 >= 0)
        pt[6] = in[(d1 * height + h1) * width + w0];
    if (d1 <= depth - 1 && h1 <= height - 1 && w1 <= width - 1)
        pt[7] = in[(d1 * height + h1) * width + w1];
    T a[8];
    a[0] = (d1 - d) * (h1 - h) * (w1 - w);
    a[1] = (d1 - d) * (h1 - h) * (w - w0);
    a[2] = (d1 - d) * (h - h0) * (w1 - w);
    a[3] = (d1 - d) * (h - h0) * (w - w0);
    a[4] = (d - d0) * (h1 - h) * (w1 - w);
    a[5] = (d - d0) * (h1 - h) * (w - w0);
    a[6] = (d - d0) * (h - h0) * (w1 - w);
    a[7] = (d - d0) * (h - h0) * (w - w0);
    T res = 0;
    for (int i = 0; i < 8; i++)
        res = FMA(pt[i], a[i], res);
    return res;
}

/* sampling position, dconv3d_gpu.cu:187-194: the integer part is formed in
 * int, converted once, and added to the offset with one rounding. */
static inline T FN(pos)(int o, int s, int p, int i, int dil, T off)
{
    return (T)((o * s - p) + i * dil) + off;
}

/* ---- dconv3d_gpu.cu:111-203  deformable_im2col_gpu_kernel -------------- */
static void FN(im2col3d)(const T *x, const T *off, const T *mask,
                         const oracle_conv3d_desc *q, T *col)
{
    const int K = q->kd * q->kh * q->kw;
    const long P = (long)q->Do * q->Ho * q->Wo;
    const int cpg = q->Cin / q->offset_groups;
    const long vol = (long)q->D * q->H * q->W;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < q->N; b++)
        for (int c = 0; c < q->Cin; c++) {
            const int g = c / cpg;
            const T *xin = x + ((long)b * q->Cin + c) * vol;
            const T *op = off + ((long)b * q->offset_groups + g) * 3 * K * P;
            const T *mp = mask ? mask + ((long)b * q->offset_groups + g) * K * P : 0;
            T *cp = col + ((long)b * q->Cin + c) * K * P;
            for (int i = 0; i < q->kd; i++)
                for (int j = 0; j < q->kh; j++)
                    for (int l = 0; l < q->kw; l++) {
                        const int k = (i * q->kh + j) * q->kw + l;
                        for (int oz = 0; oz < q->Do; oz++)
                            for (int oy = 0; oy < q->Ho; oy++)
                                for (int ox = 0; ox < q->Wo; ox++) {
                                    const long p = ((long)oz * q->Ho + oy) * q->Wo + ox;
                                    const T a = mp ? mp[k * P + p] : (T)1;
                                    const T z = FN(pos)(oz, q->sd, q->pd, i, q->dd, op[(3 * k + 0) * P + p]);
                                    const T y = FN(pos)(oy, q->sh, q->ph, j, q->dh, op[(3 * k + 1) * P + p]);
                                    const T xx = FN(pos)(ox, q->sw, q->pw, l, q->dw, op[(3 * k + 2) * P + p]);
                                    cp[k * P + p] = a * FN(trilinear)(xin, q->D, q->H, q->W, z, y, xx);
                                }
                    }
        }
}

/* out[b, o, p] = sum_r W[o, r] * col[b, r, p]   (dconv3d_gpu.cu:319-353,
 * cuBLAS N,N with m=P, n=O_g, k=C_g*K; here with double accumulation). */
static void FN(gemm_w_col)(const T *w, const T *col, T *out, const T *bias,
                           int N, int Cin, int Cout, int groups, int K, long P)
{
    const int cg = Cin / groups, og = Cout / groups;
    const long R = (long)cg * K;
#pragma omp parallel
    {
        double *acc = (double *)malloc(sizeof(double) * (size_t)P);
#pragma omp for collapse(2) schedule(static)
        for (int b = 0; b < N; b++)
            for (int o = 0; o < Cout; o++) {
                const int wg = o / og;
                const T *wr = w + (long)o * R;
                const T *cb = col + ((long)b * Cin + (long)wg * cg) * K * P;
                const double b0 = bias ? (double)bias[o] : 0.0;
                for (long p = 0; p < P; p++) acc[p] = 0.0;
                for (long r = 0; r < R; r++) {
                    const double wv = (double)wr[r];
                    const T *cr = cb + r * P;
                    for (long p = 0; p < P; p++) acc[p] += wv * (double)cr[p];
                }
                T *ob = out + ((long)b * Cout + o) * P;
                /* dconv3d_gpu.cu:555-557: bias is added to the rounded GEMM result */
                for (long p = 0; p < P; p++) ob[p] = bias ? (T)((T)acc[p] + (T)b0) : (T)acc[p];
            }
        free(acc);
    }
}

/* gcol[b, r, p] = sum_o W[o, r] * gout[b, o, p]   (dconv3d_gpu.cu:976-1000) */
static void FN(gemm_wt_gout)(const T *w, const T *gout, T *gcol,
                             int N, int Cin, int Cout, int groups, int K, long P)
{
    const int cg = Cin / groups, og = Cout / groups;
    const long R = (long)cg * K;
#pragma omp parallel
    {
        double *acc = (double *)malloc(sizeof(double) * (size_t)P);
#pragma omp for collapse(2) schedule(static)
        for (int b = 0; b < N; b++)
            for (long rr = 0; rr < (long)Cin * K; rr++) {
                const int c = (int)(rr / K);
                const int wg = c / cg;
                const long r = rr - (long)wg * cg * K; /* row inside the weight group */
                for (long p = 0; p < P; p++) acc[p] = 0.0;
                for (int oo = 0; oo < og; oo++) {
                    const int o = wg * og + oo;
                    const double wv = (double)w[(long)o * R + r];
                    const T *gr = gout + ((long)b * Cout + o) * P;
                    for (long p = 0; p < P; p++) acc[p] += wv * (double)gr[p];
                }
                T *gc = gcol + ((long)b * Cin * K + rr) * P;
                for (long p = 0; p < P; p++) gc[p] = (T)acc[p];
            }
        free(acc);
    }
}

/* gW[o, r] = sum_b sum_p gout[b, o, p] * col[b, r, p]
 * (dconv3d_gpu.cu:1054-1088: per-batch GEMM then sum over the batch). */
static void FN(gemm_gout_colt)(const T *gout, const T *col, T *gw,
                               int N, int Cin, int Cout, int groups, int K, long P)
{
    const int cg = Cin / groups, og = Cout / groups;
    const long R = (long)cg * K;
#pragma omp parallel for collapse(2) schedule(static)
    for (int o = 0; o < Cout; o++)
        for (long r = 0; r < R; r++) {
            const int wg = o / og;
            double acc = 0.0;
            for (int b = 0; b < N; b++) {
                const T *gr = gout + ((long)b * Cout + o) * P;
                const T *cr = col + (((long)b * Cin + (long)wg * cg) * K + r) * P;
                double a = 0.0;
                for (long p = 0; p < P; p++) a += (double)gr[p] * (double)cr[p];
                acc += a;
            }
            gw[(long)o * R + r] = (T)acc;
        }
}

int FN(oracle_conv3d_forward)(const T *x, const T *off, const T *mask, const T *w,
                              const T *bias, T *out, const oracle_conv3d_desc *q)
{
    const int K = q->kd * q->kh * q->kw;
    const long P = (long)q->Do * q->Ho * q->Wo;
    T *col = (T *)malloc(sizeof(T) * (size_t)q->N * q->Cin * K * P);
    if (!col) return 1;
    FN(im2col3d)(x, off, mask, q, col);
    FN(gemm_w_col)(w, col, out, bias, q->N, q->Cin, q->Cout, q->groups, K, P);
    free(col);
    return 0;
}

/* ---- dconv3d_gpu.cu:708-754  get_coordinate_weights -------------------- */
static void FN(coord_weights)(const T *im, int depth, int height, int width,
                              T z, T y, T x, T *out)
{
    int z0 = (int)FLOOR(z), y0 = (int)FLOOR(y), x0 = (int)FLOOR(x);
    int z1 = z0 + 1, y1 = y0 + 1, x1 = x0 + 1;
    int vz0 = 0 <= z0 && z0 < depth, vy0 = 0 <= y0 && y0 < height, vx0 = 0 <= x0 && x0 < width;
    int vz1 = 0 <= z1 && z1 < depth, vy1 = 0 <= y1 && y1 < height, vx1 = 0 <= x1 && x1 < width;
    T C000 = (vz0 && vy0 && vx0) ? im[(z0 * height + y0) * width + x0] : 0;
    T C001 = (vz0 && vy0 && vx1) ? im[(z0 * height + y0) * width + x1] : 0;
    T C010 = (vz0 && vy1 && vx0) ? im[(z0 * height + y1) * width + x0] : 0;
    T C011 = (vz0 && vy1 && vx1) ? im[(z0 * height + y1) * width + x1] : 0;
    T C100 = (vz1 && vy0 && vx0) ? im[(z1 * height + y0) * width + x0] : 0;
    T C101 = (vz1 && vy0 && vx1) ? im[(z1 * height + y0) * width + x1] : 0;
    T C110 = (vz1 && vy1 && vx0) ? im[(z1 * height + y1) * width + x0] : 0;
    T C111 = (vz1 && vy1 && vx1) ? im[(z1 * height + y1) * width + x1] : 0;
    T dz = z - z0, dy = y - y0, dx = x - x0;
    out[0] = ((C100 - C000) * (1 - dx) + (C101 - C001) * dx) * (1 - dy)
           + ((C110 - C010) * (1 - dx) + (C111 - C011) * dx) * dy;
    out[1] = ((C010 - C000) * (1 - dz) + (C110 - C100) * dz) * (1 - dx)
           + ((C011 - C001) * (1 - dz) + (C111 - C101) * dz) * dx;
    out[2] = ((C001 - C000) * (1 - dz) + (C101 - C100) * dz) * (1 - dy)
           + ((C011 - C010) * (1 - dz) + (C111 - C110) * dz) * dy;
}

/* ---- dconv3d_gpu.cu:756-864  deformable_col2im_coord_gpu_kernel -------- */
static void FN(coord_grad3d)(const T *gcol, const T *x, const T *off, const T *mask,
                             const oracle_conv3d_desc *q, T *goff, T *gmask)
{
    const int K = q->kd * q->kh * q->kw;
    const long P = (long)q->Do * q->Ho * q->Wo;
    const int G = q->offset_groups, cpg = q->Cin / G;
    const long vol = (long)q->D * q->H * q->W;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < q->N; b++)
        for (int gk = 0; gk < G * K; gk++) {
            const int g = gk / K, k = gk % K;
            const int l = k % q->kw, j = (k / q->kw) % q->kh, i = k / (q->kw * q->kh);
            for (int oz = 0; oz < q->Do; oz++)
                for (int oy = 0; oy < q->Ho; oy++)
                    for (int ox = 0; ox < q->Wo; ox++) {
                        const long p = ((long)oz * q->Ho + oy) * q->Wo + ox;
                        const long ob = ((long)b * G + g) * 3 * K * P + (long)3 * k * P + p;
                        const long ab = ((long)b * G + g) * K * P + (long)k * P + p;
                        const T a = mask ? mask[ab] : (T)1;
                        const T z = FN(pos)(oz, q->sd, q->pd, i, q->dd, off[ob]);
                        const T y = FN(pos)(oy, q->sh, q->ph, j, q->dh, off[ob + P]);
                        const T xx = FN(pos)(ox, q->sw, q->pw, l, q->dw, off[ob + 2 * P]);
                        T val[3] = {0, 0, 0}, aval = 0;
                        for (int cc = 0; cc < cpg; cc++) {
                            const int c = g * cpg + cc;
                            const T cv = gcol[(((long)b * q->Cin + c) * K + k) * P + p];
                            const T *xin = x + ((long)b * q->Cin + c) * vol;
                            if (mask)
                                aval += cv * FN(trilinear)(xin, q->D, q->H, q->W, z, y, xx);
                            T wt[3];
                            FN(coord_weights)(xin, q->D, q->H, q->W, z, y, xx, wt);
                            val[0] += wt[0] * cv;
                            val[1] += wt[1] * cv;
                            val[2] += wt[2] * cv;
                        }
                        goff[ob] += a * val[0];
                        goff[ob + P] += a * val[1];
                        goff[ob + 2 * P] += a * val[2];
                        if (mask) gmask[ab] += aval;
                    }
        }
}

/* ---- dconv3d_gpu.cu:562-643  deformable_col2im_gpu_kernel --------------
 * The reference scatters with atomicAdd; here each (b, c) plane is owned by
 * one thread and the adds run in (k, p) order. */
static void FN(col2im3d)(const T *gcol, const T *off, const T *mask,
                         const oracle_conv3d_desc *q, T *gx)
{
    const int K = q->kd * q->kh * q->kw;
    const long P = (long)q->Do * q->Ho * q->Wo;
    const int G = q->offset_groups, cpg = q->Cin / G;
    const long vol = (long)q->D * q->H * q->W;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < q->N; b++)
        for (int c = 0; c < q->Cin; c++) {
            const int g = c / cpg;
            T *gp = gx + ((long)b * q->Cin + c) * vol;
            for (int k = 0; k < K; k++) {
                const int l = k % q->kw, j = (k / q->kw) % q->kh, i = k / (q->kw * q->kh);
                for (int oz = 0; oz < q->Do; oz++)
                    for (int oy = 0; oy < q->Ho; oy++)
                        for (int ox = 0; ox < q->Wo; ox++) {
                            const long p = ((long)oz * q->Ho + oy) * q->Wo + ox;
                            const long ob = ((long)b * G + g) * 3 * K * P + (long)3 * k * P + p;
                            const T a = mask ? mask[((long)b * G + g) * K * P + (long)k * P + p] : (T)1;
                            const T z = FN(pos)(oz, q->sd, q->pd, i, q->dd, off[ob]);
                            const T y = FN(pos)(oy, q->sh, q->ph, j, q->dh, off[ob + P]);
                            const T xx = FN(pos)(ox, q->sw, q->pw, l, q->dw, off[ob + 2 * P]);
                            const T base = a * gcol[(((long)b * q->Cin + c) * K + k) * P + p];
                            for (int dz = 0; dz <= 1; dz++)
                                for (int dy = 0; dy <= 1; dy++)
                                    for (int dx = 0; dx <= 1; dx++) {
                                        int zp = (int)FLOOR(z) + dz, yp = (int)FLOOR(y) + dy, xp = (int)FLOOR(xx) + dx;
                                        if (0 <= zp && zp < q->D && 0 <= yp && yp < q->H && 0 <= xp && xp < q->W
                                            && FABS(z - zp) < 1 && FABS(y - yp) < 1 && FABS(xx - xp) < 1) {
                                            T wgt = (1 - FABS(z - zp)) * (1 - FABS(y - yp)) * (1 - FABS(xx - xp));
                                            gp[((long)zp * q->H + yp) * q->W + xp] += wgt * base;
                                        }
                                    }
                        }
            }
        }
}

/* ---- dconv3d_gpu.cu:1261-1332 + :933-1089 ------------------------------
 * gx, goff, gmask, gw are overwritten (the reference allocates them zeroed,
 * :1305-1308); gb = gout.sum(0,2,3,4) (:1329).  gmask/gb may be NULL. */
int FN(oracle_conv3d_backward)(const T *gout, const T *x, const T *off, const T *mask,
                               const T *w, T *gx, T *goff, T *gmask, T *gw, T *gb,
                               const oracle_conv3d_desc *q)
{
    const int K = q->kd * q->kh * q->kw;
    const long P = (long)q->Do * q->Ho * q->Wo;
    const int G = q->offset_groups;
    const long vol = (long)q->D * q->H * q->W;
    T *col = (T *)malloc(sizeof(T) * (size_t)q->N * q->Cin * K * P);
    if (!col) return 1;
    memset(gx, 0, sizeof(T) * (size_t)q->N * q->Cin * vol);
    memset(goff, 0, sizeof(T) * (size_t)q->N * G * 3 * K * P);
    if (mask && gmask) memset(gmask, 0, sizeof(T) * (size_t)q->N * G * K * P);
    FN(gemm_wt_gout)(w, gout, col, q->N, q->Cin, q->Cout, q->groups, K, P);
    FN(coord_grad3d)(col, x, off, mask, q, goff, gmask);
    FN(col2im3d)(col, off, mask, q, gx);
    FN(im2col3d)(x, off, mask, q, col);
    FN(gemm_gout_colt)(gout, col, gw, q->N, q->Cin, q->Cout, q->groups, K, P);
    if (gb)
        for (int o = 0; o < q->Cout; o++) {
            double acc = 0.0;
            for (int b = 0; b < q->N; b++) {
                const T *gr = gout + ((long)b * q->Cout + o) * P;
                for (long p = 0; p < P; p++) acc += (double)gr[p];
            }
            gb[o] = (T)acc;
        }
    free(col);
    return 0;
}

/* Corner bookkeeping of one sampling position, for the bit-exact index test:
 * base[.,0..2] = floor(z), floor(y), floor(x); flags bit c (c = 4*dz+2*dy+dx)
 * is set when corner c is read by the forward pass, i.e. the early-out of
 * dconv3d_gpu.cu:59-61 did not fire and the gate of :71-86 holds. */
int FN(oracle_conv3d_corners)(const T *off, const oracle_conv3d_desc *q,
                              int32_t *base, uint8_t *flags)
{
    const int K = q->kd * q->kh * q->kw;
    const long P = (long)q->Do * q->Ho * q->Wo;
    const int G = q->offset_groups;
    for (int b = 0; b < q->N; b++)
        for (int gk = 0; gk < G * K; gk++) {
            const int k = gk % K;
            const int l = k % q->kw, j = (k / q->kw) % q->kh, i = k / (q->kw * q->kh);
            for (int oz = 0; oz < q->Do; oz++)
                for (int oy = 0; oy < q->Ho; oy++)
                    for (int ox = 0; ox < q->Wo; ox++) {
                        const long p = ((long)oz * q->Ho + oy) * q->Wo + ox;
                        const long ob = ((long)b * G * K + gk) * 3 * P + p;
                        const long idx = ((long)b * G * K + gk) * P + p;
                        const T z = FN(pos)(oz, q->sd, q->pd, i, q->dd, off[ob]);
                        const T y = FN(pos)(oy, q->sh, q->ph, j, q->dh, off[ob + P]);
                        const T xx = FN(pos)(ox, q->sw, q->pw, l, q->dw, off[ob + 2 * P]);
                        uint8_t f = 0;
                        /* floor of a far-out-of-range or non-finite position is clamped so
                         * that the stored int32 is defined; such taps have no live corner. */
                        T zc = z < -4 ? -4 : (z > q->D + 4 ? q->D + 4 : z);
                        T yc = y < -4 ? -4 : (y > q->H + 4 ? q->H + 4 : y);
                        T xc = xx < -4 ? -4 : (xx > q->W + 4 ? q->W + 4 : xx);
                        int d0 = (int)FLOOR(zc), h0 = (int)FLOOR(yc), w0 = (int)FLOOR(xc);
                        if (!(z <= -1 || q->D <= z || y <= -1 || q->H <= y || xx <= -1 || q->W <= xx)) {
                            int d1 = d0 + 1, h1 = h0 + 1, w1 = w0 + 1;
                            if (d0 >= 0 && h0 >= 0 && w0 >= 0) f |= 1;
                            if (d0 >= 0 && h0 >= 0 && w1 <= q->W - 1) f |= 2;
                            if (d0 >= 0 && h1 <= q->H - 1 && w0 >= 0) f |= 4;
                            if (d0 >= 0 && h1 <= q->H - 1 && w1 <= q->W - 1) f |= 8;
                            if (d1 <= q->D - 1 && h0 >= 0 && w0 >= 0) f |= 16;
                            if (d1 <= q->D - 1 && h0 >= 0 && w1 <= q->W - 1) f |= 32;
                            if (d1 <= q->D - 1 && h1 <= q->H - 1 && w0 >= 0) f |= 64;
                            if (d1 <= q->D - 1 && h1 <= q->H - 1 && w1 <= q->W - 1) f |= 128;
                        }
                        base[idx * 3 + 0] = d0;
                        base[idx * 3 + 1] = h0;
                        base[idx * 3 + 2] = w0;
                        flags[idx] = f;
                    }
        }
    return 0;
}

/* ======================= 1-D (dconv1d_gpu.cu) ============================ */

/* dconv1d_gpu.cu:12-15 */
static inline T FN(lerp)(T v0, T v1, T t) { return FMA(t, v1, FMA(-t, v0, v0)); }

/* dconv1d_gpu.cu:17-56 */
static void FN(im2col1d)(const T *x, const T *off, const T *mask,
                         const oracle_conv1d_desc *q, T *col)
{
    const int K = q->k, G = q->offset_groups, cpg = q->Cin / G;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < q->N; b++)
        for (int c = 0; c < q->Cin; c++) {
            const int g = c / cpg;
            const T *xin = x + ((long)b * q->Cin + c) * q->L;
            for (int i = 0; i < K; i++)
                for (int ox = 0; ox < q->Lo; ox++) {
                    const T o = off[((long)b * G * K + g * K + i) * q->Lo + ox];
                    const T a = mask ? mask[((long)b * G * K + g * K + i) * q->Lo + ox] : (T)1;
                    const T xx = (T)(ox * q->s - q->p + i * q->d) + o;
                    const int x0 = (int)FLOOR(xx), x1 = x0 + 1;
                    const T v0 = (x0 >= 0 && x0 < q->L) ? xin[x0] : 0;
                    const T v1 = (x1 >= 0 && x1 < q->L) ? xin[x1] : 0;
                    col[(((long)b * q->Cin + c) * K + i) * q->Lo + ox] = a * FN(lerp)(v0, v1, xx - x0);
                }
        }
}

int FN(oracle_conv1d_forward)(const T *x, const T *off, const T *mask, const T *w,
                              const T *bias, T *out, const oracle_conv1d_desc *q)
{
    T *col = (T *)malloc(sizeof(T) * (size_t)q->N * q->Cin * q->k * q->Lo);
    if (!col) return 1;
    FN(im2col1d)(x, off, mask, q, col);
    /* dconv1d_gpu.cu:167-201 */
    FN(gemm_w_col)(w, col, out, bias, q->N, q->Cin, q->Cout, q->groups, q->k, q->Lo);
    free(col);
    return 0;
}

/* dconv1d_gpu.cu:403-542.  quirks != 0 reproduces the integer-position
 * workaround of :332-336 (x0 is lowered by one when x - x0 < 1e-8 while x1
 * keeps its value). */
int FN(oracle_conv1d_backward)(const T *gout, const T *x, const T *off, const T *mask,
                               const T *w, T *gx, T *goff, T *gmask, T *gw, T *gb,
                               const oracle_conv1d_desc *q, int quirks)
{
    const int K = q->k, G = q->offset_groups, cpg = q->Cin / G;
    T *col = (T *)malloc(sizeof(T) * (size_t)q->N * q->Cin * K * q->Lo);
    if (!col) return 1;
    memset(gx, 0, sizeof(T) * (size_t)q->N * q->Cin * q->L);
    FN(gemm_wt_gout)(w, gout, col, q->N, q->Cin, q->Cout, q->groups, K, q->Lo);
    /* :298-353 offset / mask gradient */
    for (int b = 0; b < q->N; b++)
        for (int g = 0; g < G; g++)
            for (int i = 0; i < K; i++)
                for (int ox = 0; ox < q->Lo; ox++) {
                    const long ai = ((long)b * G * K + g * K + i) * q->Lo + ox;
                    const T o = off[ai];
                    const T a = mask ? mask[ai] : (T)1;
                    const T xx = (T)(ox * q->s - q->p + i * q->d) + o;
                    int x0 = (int)FLOOR(xx);
                    const int x1 = x0 + 1;
                    if (quirks && (double)(xx - x0) < 1e-8) x0 -= 1;
                    T val = 0, aval = 0;
                    for (int c = g * cpg; c < (g + 1) * cpg; c++) {
                        const T *xin = x + ((long)b * q->Cin + c) * q->L;
                        const T v0 = (0 <= x0 && x0 < q->L) ? xin[x0] : 0;
                        const T v1 = (0 <= x1 && x1 < q->L) ? xin[x1] : 0;
                        const T cv = col[(((long)b * q->Cin + c) * K + i) * q->Lo + ox];
                        aval += cv * FN(lerp)(v0, v1, xx - x0);
                        val += (v1 - v0) * cv * a;
                    }
                    goff[ai] = val;
                    if (gmask) gmask[ai] = aval;
                }
    /* :206-251 scatter into grad_input */
    for (int b = 0; b < q->N; b++)
        for (int c = 0; c < q->Cin; c++) {
            const int g = c / cpg;
            T *gp = gx + ((long)b * q->Cin + c) * q->L;
            for (int i = 0; i < K; i++)
                for (int ox = 0; ox < q->Lo; ox++) {
                    const long ai = ((long)b * G * K + g * K + i) * q->Lo + ox;
                    const T a = mask ? mask[ai] : (T)1;
                    const T xx = (T)(ox * q->s - q->p + i * q->d) + off[ai];
                    const T grad = a * col[(((long)b * q->Cin + c) * K + i) * q->Lo + ox];
                    const int x0 = (int)FLOOR(xx), x1 = x0 + 1;
                    if (0 <= x0 && x0 < q->L) gp[x0] += (1 - (xx - x0)) * grad;
                    if (0 <= x1 && x1 < q->L && x1 - xx < 1) gp[x1] += (xx - x0) * grad;
                }
        }
    FN(im2col1d)(x, off, mask, q, col);
    FN(gemm_gout_colt)(gout, col, gw, q->N, q->Cin, q->Cout, q->groups, K, q->Lo);
    if (gb)
        for (int o = 0; o < q->Cout; o++) {
            double acc = 0.0;
            for (int b = 0; b < q->N; b++)
                for (int p = 0; p < q->Lo; p++) acc += (double)gout[((long)b * q->Cout + o) * q->Lo + p];
            gb[o] = (T)acc;
        }
    free(col);
    return 0;
}

#undef FN
#undef CAT
#undef CAT_
