/*
 * CPU oracle for the cu32 conv3D hot path of Dragon-Alpha (fp32, NHWC 2-D convolution:
 * forward, backward-data "deltaX", backward-filter "deltaW", the filter re-layout helpers and
 * the split-K partial-buffer summation).
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is the checker the HIP kernels are compared with; it is
 * never linked into, imported by, or called from the shipped library. Only the tests, the
 * smoke check and the benchmark's cpu_baseline leg may use it.
 *
 * Every function restates, in plain C, an algorithm the reference holds as CPU test code or as
 * a trivial index-mapping kernel; the reference location it follows is cited on each function.
 * Paths are relative to the reference checkout:
 *   Tense   = src/zutil_src/z/util/math/vector/Tense.java
 *   Vector  = src/zutil_src/z/util/math/vector/Vector.java
 *   cu32/conv = src/cu32_src/Cuda_conv3D/Cuda_conv3D
 *   cu32/dX   = src/cu32_src/Cuda_dconv3D_deltaX/Cuda_dconv3D_deltaX
 *   cu32/dW   = src/cu32_src/Cuda_dconv3D_deltaW/Cuda_dconv3D_deltaW
 *
 * Layouts (J/math/Cuda_conv3D.java:11): X[N,IH,IW,IC], W[OC,FH,FW,IC], Y[N,OH,OW,OC], all
 * dense row-major fp32. OH = (IH + 2*ph - FH)/sh + 1 (Cuda_conv3D.java:154-155).
 *
 * Pinning status (what independent evidence each function is checked against, in
 * tests/test_oracle.py): the reference ships no golden vectors for this path, so every function
 * is pinned by library routines (torch conv2d / conv2d_input / conv2d_weight in fp64 on the
 * CPU), closed forms (all-ones tap counts, impulse response, 1x1 == matrix product),
 * invariants (adjointness between the three operators, stride-s == subsampled stride-1) and a
 * pure-Python brute force on tiny shapes. No function in this file is "parity unpinned".
 */
#include <stddef.h>
#include <stdint.h>
#include <math.h>
#include <float.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define X_AT(n, ih, iw, ic) X[(((size_t)(n) * IH + (ih)) * IW + (iw)) * IC + (ic)]
#define W_AT(oc, fh, fw, ic) W[(((size_t)(oc) * FH + (fh)) * FW + (fw)) * IC + (ic)]
#define Y_AT(n, oh, ow, oc) Y[(((size_t)(n) * OH + (oh)) * OW + (ow)) * OC + (oc)]

int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void oracle_set_num_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ------------------------------------------------------------------------------------------
 * Forward.
 * ---------------------------------------------------------------------------------------- */

/* Tense.conv3D_naive (Tense.java:143-173): float tensors, DOUBLE accumulator, taps visited in
 * (fh, fw, ic) order, out-of-bounds taps skipped, result rounded to float once. The product is a
 * FLOAT product (Tense.java:168: `v += X[..] * W[..]` with float operands: Java rounds it to float
 * before widening it for the addition). */
void oracle_conv3D_naive(const float *X, int IH, int IW,
                         const float *W, int FH, int FW,
                         float *Y, int OH, int OW,
                         int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++)
        for (int oh = 0; oh < OH; oh++) {
            const int ih_s = oh * sh - ph;
            for (int ow = 0; ow < OW; ow++) {
                const int iw_s = ow * sw - pw;
                for (int oc = 0; oc < OC; oc++) {
                    double v = 0;
                    for (int fh = 0; fh < FH; fh++)
                        for (int fw = 0; fw < FW; fw++) {
                            const int ih = ih_s + fh, iw = iw_s + fw;
                            if (ih < 0 || iw < 0 || ih >= IH || iw >= IW) continue;
                            const float *x = &X_AT(n, ih, iw, 0);
                            const float *w = &W_AT(oc, fh, fw, 0);
                            for (int ic = 0; ic < IC; ic++) v += (double)(float)(x[ic] * w[ic]);
                        }
                    Y_AT(n, oh, ow, oc) = (float)v;
                }
            }
        }
}

/* Tense.conv3D_naive_double (Tense.java:175-205): same loops, the result kept in double.
 * Inputs stay fp32 here (a float*float product is exact in double), so this is the
 * "mathematical" answer the 1e-4 parity bound is measured against. */
void oracle_conv3D_f64(const float *X, int IH, int IW,
                       const float *W, int FH, int FW,
                       double *Y, int OH, int OW,
                       int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++)
        for (int oh = 0; oh < OH; oh++) {
            const int ih_s = oh * sh - ph;
            for (int ow = 0; ow < OW; ow++) {
                const int iw_s = ow * sw - pw;
                for (int oc = 0; oc < OC; oc++) {
                    double v = 0;
                    for (int fh = 0; fh < FH; fh++)
                        for (int fw = 0; fw < FW; fw++) {
                            const int ih = ih_s + fh, iw = iw_s + fw;
                            if (ih < 0 || iw < 0 || ih >= IH || iw >= IW) continue;
                            const float *x = &X_AT(n, ih, iw, 0);
                            const float *w = &W_AT(oc, fh, fw, 0);
                            for (int ic = 0; ic < IC; ic++) v += (double)x[ic] * (double)w[ic];
                        }
                    Y_AT(n, oh, ow, oc) = v;
                }
            }
        }
}

/* CONV_3D_NAIVE (cu32/conv/test.cuh:80-109): the native project's own CPU check; identical loop
 * nest with a FLOAT accumulator. This is the direct-convolution CPU path timed as the
 * benchmark's cpu_baseline. The inner product over ic is written so the compiler may
 * vectorise it (reassociation inside one tap only). */
void oracle_conv3D_f32acc(const float *X, int IH, int IW,
                          const float *W, int FH, int FW,
                          float *Y, int OH, int OW,
                          int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++)
        for (int oh = 0; oh < OH; oh++) {
            const int ih_s = oh * sh - ph;
            for (int ow = 0; ow < OW; ow++) {
                const int iw_s = ow * sw - pw;
                for (int oc = 0; oc < OC; oc++) {
                    float v = 0;
                    for (int fh = 0; fh < FH; fh++)
                        for (int fw = 0; fw < FW; fw++) {
                            const int ih = ih_s + fh, iw = iw_s + fw;
                            if (ih < 0 || iw < 0 || ih >= IH || iw >= IW) continue;
                            const float *x = &X_AT(n, ih, iw, 0);
                            const float *w = &W_AT(oc, fh, fw, 0);
                            float t = 0;
#pragma omp simd reduction(+ : t)
                            for (int ic = 0; ic < IC; ic++) t += x[ic] * w[ic];
                            v += t;
                        }
                    Y_AT(n, oh, ow, oc) = v;
                }
            }
        }
}

/* ------------------------------------------------------------------------------------------
 * Backward-data (deltaX).
 * ---------------------------------------------------------------------------------------- */

#define DY_AT(n, oh, ow, oc) dY[(((size_t)(n) * OH + (oh)) * OW + (ow)) * OC + (oc)]
#define DX_AT(n, ih, iw, ic) dX[(((size_t)(n) * IH + (ih)) * IW + (iw)) * IC + (ic)]

/* Tense.deconv3D_deltaX_img2col (Tense.java:334-376) and its native twin
 * deconv3D_deltaX_img2col (cu32/dX/test.cuh:89-131): for every (ic, n, ih, iw) a FLOAT
 * accumulator runs over k = (oc, fh, fw); deltaY is read on the stride-dilated lattice
 * (oh = ih - oph + fh must be a multiple of sh) and the filter is read rotated by 180 degrees,
 * oph = FH - 1 - ph. */
void oracle_deltaX_img2col(const float *dY, int OH, int OW,
                           const float *W, int FH, int FW,
                           float *dX, int IH, int IW,
                           int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    const int OHp = OH + (OH - 1) * (sh - 1), OWp = OW + (OW - 1) * (sw - 1);
    const int oph = FH - ph - 1, opw = FW - pw - 1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++)
        for (int ih = 0; ih < IH; ih++)
            for (int iw = 0; iw < IW; iw++)
                for (int ic = 0; ic < IC; ic++) {
                    float v = 0;
                    for (int oc = 0; oc < OC; oc++)
                        for (int fh = 0; fh < FH; fh++)
                            for (int fw = 0; fw < FW; fw++) {
                                const int oh = ih - oph + fh, ow = iw - opw + fw;
                                if (oh < 0 || ow < 0 || oh >= OHp || ow >= OWp) continue;
                                if (oh % sh != 0 || ow % sw != 0) continue;
                                v += DY_AT(n, oh / sh, ow / sw, oc) * W_AT(oc, FH - 1 - fh, FW - 1 - fw, ic);
                            }
                    DX_AT(n, ih, iw, ic) = v;
                }
}

/* The same operator with a double accumulator and double result: the mathematical answer used
 * for the parity bound. Written as the adjoint scatter-free gather
 *   deltaX[n,ih,iw,ic] = sum_{oc,fh,fw : (ih+ph-fh) % sh == 0 ...} deltaY[n,(ih+ph-fh)/sh,(iw+pw-fw)/sw,oc] * W[oc,fh,fw,ic]
 * which is the formula of cu32/dX/micro.cuh:207-231 with the rotation unrolled. */
void oracle_deltaX_f64(const float *dY, int OH, int OW,
                       const float *W, int FH, int FW,
                       double *dX, int IH, int IW,
                       int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++)
        for (int ih = 0; ih < IH; ih++)
            for (int iw = 0; iw < IW; iw++)
                for (int ic = 0; ic < IC; ic++) {
                    double v = 0;
                    for (int fh = 0; fh < FH; fh++) {
                        const int th = ih + ph - fh;
                        if (th < 0 || th % sh != 0) continue;
                        const int oh = th / sh;
                        if (oh >= OH) continue;
                        for (int fw = 0; fw < FW; fw++) {
                            const int tw = iw + pw - fw;
                            if (tw < 0 || tw % sw != 0) continue;
                            const int ow = tw / sw;
                            if (ow >= OW) continue;
                            for (int oc = 0; oc < OC; oc++)
                                v += (double)DY_AT(n, oh, ow, oc) * (double)W_AT(oc, fh, fw, ic);
                        }
                    }
                    DX_AT(n, ih, iw, ic) = v;
                }
}

/* ------------------------------------------------------------------------------------------
 * Backward-filter (deltaW).
 * ---------------------------------------------------------------------------------------- */

#define DW_AT(oc, fh, fw, ic) dW[(((size_t)(oc) * FH + (fh)) * FW + (fw)) * IC + (ic)]

/* Tense.deconv3d_deltaW_naive (Tense.java:1277-1320): the reference transposes X to
 * Xe[IC,IH,IW,N], dilates deltaY to deltaYpe[OC,OHp,OWp,N] and calls conv3D_naive (stride 1,
 * pad (ph,pw)) with deltaYpe as the "filter". Unrolled, that is a DOUBLE accumulator per
 * (oc,fh,fw,ic) running over (oh, ow, n) in that order, dilation zeros contributing nothing,
 * positions that fall outside X skipped. */
void oracle_deltaW_naive(const float *X, int IH, int IW,
                         const float *dY, int OH, int OW,
                         float *dW, int FH, int FW,
                         int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int oc = 0; oc < OC; oc++)
        for (int fh = 0; fh < FH; fh++)
            for (int fw = 0; fw < FW; fw++)
                for (int ic = 0; ic < IC; ic++) {
                    double v = 0;
                    for (int oh = 0; oh < OH; oh++) {
                        const int ih = oh * sh - ph + fh;
                        if (ih < 0 || ih >= IH) continue;
                        for (int ow = 0; ow < OW; ow++) {
                            const int iw = ow * sw - pw + fw;
                            if (iw < 0 || iw >= IW) continue;
                            for (int n = 0; n < N; n++)
                                v += (double)(float)(X_AT(n, ih, iw, ic) * DY_AT(n, oh, ow, oc));   /* float product, as conv3D_naive */
                        }
                    }
                    DW_AT(oc, fh, fw, ic) = (float)v;
                }
}

/* Same sum kept in double (parity reference), K visited in the GPU kernels' (n, oh, ow) order
 * (cu32/dW/dconv3d_dW_GemmSK_kernel.cuh:131-262: GK = N*OH*OW ordered n, oh, ow). */
void oracle_deltaW_f64(const float *X, int IH, int IW,
                       const float *dY, int OH, int OW,
                       double *dW, int FH, int FW,
                       int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int oc = 0; oc < OC; oc++)
        for (int fh = 0; fh < FH; fh++)
            for (int fw = 0; fw < FW; fw++)
                for (int ic = 0; ic < IC; ic++) {
                    double v = 0;
                    for (int n = 0; n < N; n++)
                        for (int oh = 0; oh < OH; oh++) {
                            const int ih = oh * sh - ph + fh;
                            if (ih < 0 || ih >= IH) continue;
                            for (int ow = 0; ow < OW; ow++) {
                                const int iw = ow * sw - pw + fw;
                                if (iw < 0 || iw >= IW) continue;
                                v += (double)X_AT(n, ih, iw, ic) * (double)DY_AT(n, oh, ow, oc);
                            }
                        }
                    DW_AT(oc, fh, fw, ic) = v;
                }
}

/* deconv3D_deltaW_img2col2 (cu32/dW/test.cuh:77-120): the native project's CPU check, FLOAT
 * accumulator over k = (n, oh, ow). Used as the cpu_baseline for backward-filter. */
void oracle_deltaW_f32acc(const float *X, int IH, int IW,
                          const float *dY, int OH, int OW,
                          float *dW, int FH, int FW,
                          int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int oc = 0; oc < OC; oc++)
        for (int fh = 0; fh < FH; fh++)
            for (int fw = 0; fw < FW; fw++)
                for (int ic = 0; ic < IC; ic++) {
                    float v = 0;
                    for (int n = 0; n < N; n++)
                        for (int oh = 0; oh < OH; oh++) {
                            const int ih = oh * sh - ph + fh;
                            if (ih < 0 || ih >= IH) continue;
                            for (int ow = 0; ow < OW; ow++) {
                                const int iw = ow * sw - pw + fw;
                                if (iw < 0 || iw >= IW) continue;
                                v += X_AT(n, ih, iw, ic) * DY_AT(n, oh, ow, oc);
                            }
                        }
                    DW_AT(oc, fh, fw, ic) = v;
                }
}

/* One split-K slice of backward-filter, as kernel_GemmSK_8_8 defines it
 * (cu32/dW/dconv3d_dW_GemmSK_kernel.cuh:131-157): GK = N*OH*OW ordered (n, oh, ow);
 * GK_slice = (GK / GZ) >> 3 << 3 (cu32/dW/micro.cuh:343-349); slice z covers
 * k in [z*GK_slice, (z+1)*GK_slice) and the last slice runs to GK. Double accumulate/out so
 * that a partial result can be checked independently of summation order. */
void oracle_deltaW_slice_f64(const float *X, int IH, int IW,
                             const float *dY, int OH, int OW,
                             double *dW, int FH, int FW,
                             int N, int IC, int OC, int sh, int sw, int ph, int pw,
                             int GZ, int z)
{
    const int GK = N * OH * OW;
    const int GK_slice = (GK / GZ) >> 3 << 3;
    const int k0 = GK_slice * z, k1 = (z != GZ - 1) ? k0 + GK_slice : GK;
#pragma omp parallel for collapse(2) schedule(static)
    for (int oc = 0; oc < OC; oc++)
        for (int fh = 0; fh < FH; fh++)
            for (int fw = 0; fw < FW; fw++)
                for (int ic = 0; ic < IC; ic++) {
                    double v = 0;
                    for (int k = k0; k < k1; k++) {
                        const int n = k / (OH * OW), r = k - n * (OH * OW);
                        const int oh = r / OW, ow = r - oh * OW;
                        const int ih = oh * sh - ph + fh, iw = ow * sw - pw + fw;
                        if (ih < 0 || ih >= IH || iw < 0 || iw >= IW) continue;
                        v += (double)X_AT(n, ih, iw, ic) * (double)DY_AT(n, oh, ow, oc);
                    }
                    DW_AT(oc, fh, fw, ic) = v;
                }
}

/* buf_summary_kernel4 (cu32/dW/dconv3d_dW_GemmSK_bufSum.cuh:32-70): deltaW += sum over
 * p = 0..part-1 of deltaW_buf[p], in that fixed order, fp32 Kahan-compensated. The arithmetic
 * is restated operation by operation; "volatile" keeps the C compiler from simplifying the
 * compensation away. Bit-exact target for the GPU entry. */
void oracle_buf_summary(const float *deltaW_buf, float *deltaW, int part, int sizeW)
{
    for (int i = 0; i < sizeW; i++) {
        volatile float dw = deltaW[i];
        volatile float c = 0.0f;
        for (int p = 0; p < part; p++) {
            volatile float b = deltaW_buf[(size_t)p * sizeW + i];
            b = b - c;
            volatile float t = dw + b;
            volatile float d = t - dw;
            c = d - b;
            dw = t;
        }
        deltaW[i] = dw;
    }
}

/* ------------------------------------------------------------------------------------------
 * Filter re-layouts ("remode").
 * ---------------------------------------------------------------------------------------- */

/* kremode_kernel_4 (cu32/conv/conv3D_kernel_remode.cuh:39-72): W[OC,FH,FW,IC] -> CW[FH,FW,IC,OC]. */
void oracle_kernel_remode(const float *W, float *CW, int FH, int FW, int OC, int IC)
{
    for (int oc = 0; oc < OC; oc++)
        for (int fh = 0; fh < FH; fh++)
            for (int fw = 0; fw < FW; fw++)
                for (int ic = 0; ic < IC; ic++)
                    CW[(((size_t)fh * FW + fw) * IC + ic) * OC + oc] = W_AT(oc, fh, fw, ic);
}

/* ks_remode_kernel_4 (cu32/dX/dconv3D_dX_kernelSplit_remode.cuh:33-68), kernel-split layout v1:
 * for each (y,x) in [0,sh)x[0,sw) a block of stride OC*mCFH*mCFW*IC holding
 * CW[y,x][oc][fhr][fwr][ic] = W[oc][y + (CFH_y-1-fhr)*sh][x + (CFW_x-1-fwr)*sw][ic]
 * with the block's own CFH_y = (FH - y + sh - 1)/sh, CFW_x likewise, packed from the block start.
 * Elements of the block beyond OC*CFH_y*CFW_x*IC are left untouched, as in the reference. */
void oracle_ks_remode(const float *W, int FH, int FW, float *CW, int mCFH, int mCFW,
                      int OC, int IC, int sh, int sw)
{
    for (int y = 0; y < sh; y++)
        for (int x = 0; x < sw; x++) {
            float *blk = CW + (size_t)(y * sw + x) * OC * mCFH * mCFW * IC;
            const int CFH = (FH - y + sh - 1) / sh, CFW = (FW - x + sw - 1) / sw;
            for (int oc = 0; oc < OC; oc++)
                for (int fhr = 0; fhr < CFH; fhr++)
                    for (int fwr = 0; fwr < CFW; fwr++)
                        for (int ic = 0; ic < IC; ic++) {
                            const int fh = y + (CFH - 1 - fhr) * sh, fw = x + (CFW - 1 - fwr) * sw;
                            const float w = (fh < FH && fw < FW) ? W_AT(oc, fh, fw, ic) : 0.0f;
                            blk[(((size_t)oc * CFH + fhr) * CFW + fwr) * IC + ic] = w;
                        }
        }
}

/* ks_remodev2_kernel_4 (cu32/dX/dconv3D_dX_kernelSplit_remode_v2.cuh:34-68), layout v2 (the one
 * the Java engine uses, CudaFloat32EngineBase.java:1886,1940,1985):
 * CW[y,x][fhr][fwr][oc][ic], same block stride and same tap mapping as v1. */
void oracle_ks_remodev2(const float *W, int FH, int FW, float *CW, int mCFH, int mCFW,
                        int OC, int IC, int sh, int sw)
{
    for (int y = 0; y < sh; y++)
        for (int x = 0; x < sw; x++) {
            float *blk = CW + (size_t)(y * sw + x) * OC * mCFH * mCFW * IC;
            const int CFH = (FH - y + sh - 1) / sh, CFW = (FW - x + sw - 1) / sw;
            for (int fhr = 0; fhr < CFH; fhr++)
                for (int fwr = 0; fwr < CFW; fwr++)
                    for (int oc = 0; oc < OC; oc++)
                        for (int ic = 0; ic < IC; ic++) {
                            const int fh = y + (CFH - 1 - fhr) * sh, fw = x + (CFW - 1 - fwr) * sw;
                            const float w = (fh < FH && fw < FW) ? W_AT(oc, fh, fw, ic) : 0.0f;
                            blk[(((size_t)fhr * CFW + fwr) * OC + oc) * IC + ic] = w;
                        }
        }
}

/* Backward-data through the kernel-split decomposition, consuming the v2 layout exactly as
 * ks_kernel_8_8R does (cu32/dX/dconv3D_dX_kernelSplit_R_kernel.cuh:76-140): for each (y,x),
 * ph' = ph - y, ihs = the first ih >= 0 with (ih + ph') % sh == 0, and
 *   deltaX[n, ihs + sh*i, iws + sw*j, ic] =
 *     sum_{fhr,fwr,oc} deltaY[n, (ih+ph')/sh - (CFH-1) + fhr, (iw+pw')/sw - (CFW-1) + fwr, oc] * CW[y,x][fhr][fwr][oc][ic].
 * Double accumulate/out. Agreement of this function with oracle_deltaX_f64 is what pins the
 * v2 layout as a correct decomposition. */
void oracle_deltaX_kernelSplit_f64(const float *dY, int OH, int OW,
                                   const float *CW, int FH, int FW,
                                   double *dX, int IH, int IW,
                                   int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    const int mCFH = (FH + sh - 1) / sh, mCFW = (FW + sw - 1) / sw;
    const size_t CWstride = (size_t)mCFH * mCFW * OC * IC;
    for (size_t i = 0; i < (size_t)N * IH * IW * IC; i++) dX[i] = 0.0;
    for (int y = 0; y < sh; y++)
        for (int x = 0; x < sw; x++) {
            const float *blk = CW + (size_t)(y * sw + x) * CWstride;
            const int CFH = (FH - y + sh - 1) / sh, CFW = (FW - x + sw - 1) / sw;
            const int phy = ph - y, pwx = pw - x;
            const int ihs = -phy + (phy > 0 ? ((phy + sh - 1) / sh * sh) : 0);
            const int iws = -pwx + (pwx > 0 ? ((pwx + sw - 1) / sw * sw) : 0);
            if (CFH <= 0 || CFW <= 0) continue; /* sub-lattice keeps its zeros */
#pragma omp parallel for collapse(2) schedule(static)
            for (int n = 0; n < N; n++)
                for (int ih = ihs; ih < IH; ih += sh)
                    for (int iw = iws; iw < IW; iw += sw) {
                        const int ohs = (ih + phy) / sh - (CFH - 1), ows = (iw + pwx) / sw - (CFW - 1);
                        for (int ic = 0; ic < IC; ic++) {
                            double v = 0;
                            for (int fhr = 0; fhr < CFH; fhr++)
                                for (int fwr = 0; fwr < CFW; fwr++) {
                                    const int oh = ohs + fhr, ow = ows + fwr;
                                    if (oh < 0 || ow < 0 || oh >= OH || ow >= OW) continue;
                                    for (int oc = 0; oc < OC; oc++)
                                        v += (double)DY_AT(n, oh, ow, oc) *
                                             (double)blk[(((size_t)fhr * CFW + fwr) * OC + oc) * IC + ic];
                                }
                            DX_AT(n, ih, iw, ic) = v;
                        }
                    }
        }
}

/* ------------------------------------------------------------------------------------------
 * Comparison helpers.
 * ---------------------------------------------------------------------------------------- */

/* Vector.samePercentRelative(float[],float[],int,float) (Vector.java:4109-4126): fraction of
 * elements with A==B, or |A-B+eps| / |A+B+eps| < threshold (eps = Float.MIN_VALUE, the
 * smallest subnormal), or both NaN. The pass criterion of the reference's own tests. */
float oracle_samePercentRelative(const float *A, const float *B, long length, float threshold)
{
    const float eps = 1.401298464324817e-45f; /* Float.MIN_VALUE */
    long sum = 0;
    for (long i = 0; i < length; i++) {
        if (A[i] == B[i]) { sum++; continue; }
        const float div = fabsf((A[i] - B[i] + eps) / (A[i] + B[i] + eps));
        if (div < threshold) { sum++; continue; }
        if (isnan(A[i]) && isnan(B[i])) { sum++; continue; }
    }
    return ((float)sum) / (float)length;
}

/* The parity bound of this build: max over elements of |got - want| / max(|want|, floor_abs/rel)
 * i.e. relative error with an absolute floor (rel 1e-4, abs 1e-5 near zero when called with
 * rel=1e-4, floor_abs=1e-5). Returns the worst ratio err / allowed; <= 1 passes. */
double oracle_max_err_ratio(const float *got, const double *want, long length, double rel, double floor_abs)
{
    double worst = 0;
    for (long i = 0; i < length; i++) {
        const double err = fabs((double)got[i] - want[i]);
        double allowed = rel * fabs(want[i]);
        if (allowed < floor_abs) allowed = floor_abs;
        if (isnan(err)) return INFINITY;
        const double r = err / allowed;
        if (r > worst) worst = r;
    }
    return worst;
}
