/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's dilated
 * 3x3 / 3x3x3 convolution kernels.  Included twice by msd_oracle.c, once per
 * scalar type (T = float, double; SFX = f32, f64).
 *
 * Conventions shared by all functions in this file:
 *   - a tensor view is a base pointer plus five element strides
 *     {batch, channel, z, y, x}; 2D data is passed with size[0] == 1 and an
 *     arbitrary z stride, and its 3x3 kernel has no z taps (nz == 1);
 *   - size = {D, H, W};
 *   - the weight tensor is contiguous (c_out, c_in, 3, 3) or (c_out, c_in, 3, 3, 3).
 */

#define CAT_(a, b) a##_##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SFX)

/* Element offset of voxel (z, y, x) in a view. */
#define VOFF(s, z, y, x) ((z) * (s)[2] + (y) * (s)[3] + (x) * (s)[4])

/*
 * Forward pass, with or without the ReLU clamp.
 * Follows conv2d_forward.cu:139-173 (ReLU: :171, plain: :69-91) and
 * conv3d_forward.cu:156-195: o starts at bias[c_out]; channels are the outer
 * loop and the taps run row-major inside; the clamp is max(0, o).
 * Each output row is accumulated in a scratch row so that every output sees
 * its additions in exactly that order while the compiler vectorises over x.
 */
void FN(msd_oracle_conv_forward)(int ndim, int relu, int64_t B, int64_t C, int64_t Wd,
                                 const int64_t *size, int dil,
                                 const T *x, const int64_t *xs,
                                 const T *k, const T *bias,
                                 T *y, const int64_t *ys)
{
    const int64_t D = size[0], H = size[1], W = size[2];
    const int nz = (ndim == 3) ? 3 : 1;
    const int K = nz * 9;
    int64_t *rx = (int64_t *)malloc(sizeof(int64_t) * 3 * (size_t)W);
    for (int r = 0; r < 3; r++)
        for (int64_t w = 0; w < W; w++)
            rx[r * W + w] = msd_oracle_reflect((int)(w + (r - 1) * dil), (int)W);

#pragma omp parallel
    {
        T *acc = (T *)malloc(sizeof(T) * (size_t)W);
#pragma omp for collapse(2) schedule(static)
        for (int64_t bz = 0; bz < B * D; bz++) {
            for (int64_t h = 0; h < H; h++) {
                const int64_t b = bz / D, z = bz % D;
                for (int64_t co = 0; co < Wd; co++) {
                    for (int64_t w = 0; w < W; w++) acc[w] = bias[co];
                    for (int64_t ci = 0; ci < C; ci++) {
                        const T *xc = x + b * xs[0] + ci * xs[1];
                        const T *kc = k + (co * C + ci) * K;
                        for (int p = 0; p < nz; p++) {
                            const int64_t zz = (ndim == 3)
                                ? msd_oracle_reflect((int)(z + (p - 1) * dil), (int)D) : 0;
                            for (int q = 0; q < 3; q++) {
                                const int64_t hh = msd_oracle_reflect((int)(h + (q - 1) * dil), (int)H);
                                const T *row = xc + zz * xs[2] + hh * xs[3];
                                for (int r = 0; r < 3; r++) {
                                    const T kv = kc[(p * 3 + q) * 3 + r];
                                    const int64_t *rr = rx + r * W;
                                    const int64_t sx = xs[4];
                                    for (int64_t w = 0; w < W; w++)
                                        acc[w] += row[rr[w] * sx] * kv;
                                }
                            }
                        }
                    }
                    T *yo = y + b * ys[0] + co * ys[1] + z * ys[2] + h * ys[3];
                    if (relu)
                        for (int64_t w = 0; w < W; w++) yo[w * ys[4]] = acc[w] > (T)0 ? acc[w] : (T)0;
                    else
                        for (int64_t w = 0; w < W; w++) yo[w * ys[4]] = acc[w];
                }
            }
        }
        free(acc);
    }
    free(rx);
}

/*
 * Gradient with respect to the input, ACCUMULATED into gx (gx += ...).
 * Follows conv2d_backward_x.cu:149-207 and conv3d_backward_x.cu:167-240:
 * a gather over the three slots p = -1, 0, +1 per axis that reads the output
 * gradient at reflect(h - dil * p) and multiplies it with weight tap prog[p+1],
 * where prog = {0, 1, 2} except prog[2] = 0 when h < dil and prog[0] = 2 when
 * size <= h + dil (the border tap swap).  With relu != 0 a term only counts
 * when 0 < out at the gathered position (:197 / :229).  g starts at zero, runs
 * over c_out (outer) and the slots (row-major inner) and is added to gx once.
 * `out` is ignored when relu == 0.
 */
void FN(msd_oracle_conv_backward_x)(int ndim, int relu, int64_t B, int64_t C, int64_t Wd,
                                    const int64_t *size, int dil,
                                    const T *out, const int64_t *os,
                                    const T *gy, const int64_t *gs,
                                    const T *k,
                                    T *gx, const int64_t *xs)
{
    const int64_t D = size[0], H = size[1], W = size[2];
    const int nz = (ndim == 3) ? 3 : 1;
    const int K = nz * 9;

#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t bz = 0; bz < B * D; bz++) {
        for (int64_t h = 0; h < H; h++) {
            const int64_t b = bz / D, z = bz % D;
            int prog_z[3] = {0, 1, 2}, prog_h[3] = {0, 1, 2};
            if (ndim == 3) {
                if (z < dil) prog_z[2] = 0;
                if (D <= z + dil) prog_z[0] = 2;
            }
            if (h < dil) prog_h[2] = 0;
            if (H <= h + dil) prog_h[0] = 2;
            for (int64_t w = 0; w < W; w++) {
                int prog_w[3] = {0, 1, 2};
                if (w < dil) prog_w[2] = 0;
                if (W <= w + dil) prog_w[0] = 2;
                for (int64_t ci = 0; ci < C; ci++) {
                    T g = (T)0;
                    for (int64_t co = 0; co < Wd; co++) {
                        const T *gyc = gy + b * gs[0] + co * gs[1];
                        const T *oc = relu ? out + b * os[0] + co * os[1] : NULL;
                        const T *kc = k + (co * C + ci) * K;
                        for (int p = 0; p < nz; p++) {
                            const int64_t zp = (ndim == 3)
                                ? msd_oracle_reflect((int)(z - dil * (p - 1)), (int)D) : 0;
                            const int p_ = (ndim == 3) ? prog_z[p] : 0;
                            for (int q = 0; q < 3; q++) {
                                const int64_t hq = msd_oracle_reflect((int)(h - dil * (q - 1)), (int)H);
                                const int q_ = prog_h[q];
                                for (int r = 0; r < 3; r++) {
                                    const int64_t wr = msd_oracle_reflect((int)(w - dil * (r - 1)), (int)W);
                                    const int r_ = prog_w[r];
                                    if (!relu || (T)0 < oc[VOFF(os, zp, hq, wr)])
                                        g += gyc[VOFF(gs, zp, hq, wr)] * kc[(p_ * 3 + q_) * 3 + r_];
                                }
                            }
                        }
                    }
                    gx[b * xs[0] + ci * xs[1] + VOFF(xs, z, h, w)] += g;
                }
            }
        }
    }
}

/*
 * Gradient with respect to the weights, ACCUMULATED into gk (contiguous).
 * Follows conv2d_backward_k.cu:82-111 and conv3d_backward_k.cu:89-121:
 * gk[co,ci,tap] += sum over batch and voxels of
 *     x[reflect(v + dil * tap)] * gy[v] * (0 < out[v] ? 1 : 0).
 * The reference sums with float atomics in no fixed order; here every sum is
 * carried in double and rounded once, which is the value any order
 * approximates.  `out` is ignored when relu == 0.
 */
void FN(msd_oracle_conv_backward_k)(int ndim, int relu, int64_t B, int64_t C, int64_t Wd,
                                    const int64_t *size, int dil,
                                    const T *out, const int64_t *os,
                                    const T *gy, const int64_t *gs,
                                    const T *x, const int64_t *xs,
                                    T *gk)
{
    const int64_t D = size[0], H = size[1], W = size[2];
    const int nz = (ndim == 3) ? 3 : 1;
    const int K = nz * 9;

#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int64_t co = 0; co < Wd; co++) {
        for (int64_t ci = 0; ci < C; ci++) {
            double sum[27];
            for (int t = 0; t < 27; t++) sum[t] = 0.0;
            for (int64_t b = 0; b < B; b++) {
                const T *gyc = gy + b * gs[0] + co * gs[1];
                const T *oc = relu ? out + b * os[0] + co * os[1] : NULL;
                const T *xc = x + b * xs[0] + ci * xs[1];
                for (int64_t z = 0; z < D; z++)
                for (int64_t h = 0; h < H; h++)
                for (int64_t w = 0; w < W; w++) {
                    T m = gyc[VOFF(gs, z, h, w)];
                    if (relu && !((T)0 < oc[VOFF(os, z, h, w)])) m = (T)0;
                    if (m == (T)0) continue;
                    for (int p = 0; p < nz; p++) {
                        const int64_t z_ = (ndim == 3)
                            ? msd_oracle_reflect((int)(z + (p - 1) * dil), (int)D) : 0;
                        for (int q = 0; q < 3; q++) {
                            const int64_t h_ = msd_oracle_reflect((int)(h + (q - 1) * dil), (int)H);
                            for (int r = 0; r < 3; r++) {
                                const int64_t w_ = msd_oracle_reflect((int)(w + (r - 1) * dil), (int)W);
                                sum[(p * 3 + q) * 3 + r] +=
                                    (double)xc[VOFF(xs, z_, h_, w_)] * (double)m;
                            }
                        }
                    }
                }
            }
            T *g = gk + (co * C + ci) * K;
            for (int t = 0; t < K; t++) g[t] += (T)sum[t];
        }
    }
}

/*
 * Gradient with respect to the bias, ACCUMULATED into gb.
 * relu != 0: conv2d_backward_bias.cu:34-48 / conv3d_backward_bias.cu:36-50,
 *            gb[co] += sum of gy where 0 < out.
 * relu == 0: msd_custom_convolutions.cpp:180-211, gb += gy.sum over all but the
 *            channel axis.
 * Summed in double for the same reason as the weight gradient.
 */
void FN(msd_oracle_conv_backward_bias)(int ndim, int relu, int64_t B, int64_t Wd,
                                       const int64_t *size,
                                       const T *out, const int64_t *os,
                                       const T *gy, const int64_t *gs,
                                       T *gb)
{
    const int64_t D = size[0], H = size[1], W = size[2];
    (void)ndim;
    for (int64_t co = 0; co < Wd; co++) {
        double s = 0.0;
        for (int64_t b = 0; b < B; b++)
            for (int64_t z = 0; z < D; z++)
            for (int64_t h = 0; h < H; h++)
            for (int64_t w = 0; w < W; w++) {
                const int64_t go = b * gs[0] + co * gs[1] + VOFF(gs, z, h, w);
                if (!relu || (T)0 < out[b * os[0] + co * os[1] + VOFF(os, z, h, w)])
                    s += (double)gy[go];
            }
        gb[co] += (T)s;
    }
}

#undef VOFF
#undef FN
#undef CAT
#undef CAT_
