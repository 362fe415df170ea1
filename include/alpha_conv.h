/*
 * alpha_conv.h — C ABI of the MI355X (gfx950) replacement for Dragon-Alpha's cu32 conv3D hot path.
 *
 * One entry point per JNI native method of the reference classes
 *   z.dragon.engine.cuda.impl.math.Cuda_conv3D          (10 methods)
 *   z.dragon.engine.cuda.impl.math.Cuda_dconv3D_deltaX  (13 methods)
 *   z.dragon.engine.cuda.impl.math.Cuda_dconv3D_deltaW  ( 6 methods)
 * with the same argument order and meaning as the reference's native implementations
 * (cited per function as <project>/A.cu:<line>, where
 *   conv = src/cu32_src/Cuda_conv3D/Cuda_conv3D,
 *   dX   = src/cu32_src/Cuda_dconv3D_deltaX/Cuda_dconv3D_deltaX,
 *   dW   = src/cu32_src/Cuda_dconv3D_deltaW/Cuda_dconv3D_deltaW).
 * The JNI shim (csrc/jni_shim.cpp) exports the exact Java_z_dragon_..._<method> symbols and
 * forwards to these functions after copying the stream handles out of the jlongArray.
 *
 * Conventions (identical to the reference):
 *   - fp32 everywhere. X[N,IH,IW,IC], W[OC,FH,FW,IC], Y[N,OH,OW,OC], dense row-major (NHWC).
 *   - N, IC and OC are multiples of 4 (the engine pads them); pad channels hold zeros.
 *   - OH = (IH + 2*ph - FH)/sh + 1, OW likewise.
 *   - All pointers are DEVICE pointers, borrowed for the duration of the enqueued work. Nothing
 *     is allocated or freed; scratch (CW, deltaW_buf) is supplied by the caller.
 *   - `streams` is an array of `length` stream handles (hipStream_t cast to int64, exactly what
 *     the Java side holds as jlong). Work is only ENQUEUED; the caller observes completion with
 *     events on those streams. This implementation enqueues everything on streams[0].
 *   - Outputs are overwritten (no alpha/beta, no bias).
 *   - `texture` variants and `useTexture` flags are performance hints in the reference; here they
 *     select nothing (same kernels, same results).
 *
 * Return value: 0 on success, otherwise a hipError_t value (or ALPHA_CONV_EINVAL for arguments
 * the kernels cannot serve). alpha_conv_last_error() returns a thread-local message.
 */
#ifndef ALPHA_CONV_H
#define ALPHA_CONV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ALPHA_CONV_EINVAL 10001

/* ---- library ---------------------------------------------------------------------------- */
const char *alpha_conv_version(void);
const char *alpha_conv_last_error(void);

/* Compute-unit count and peak engine clock (kHz) of the current device. Stands in for the one
 * field of the reference's CudaDevice class this path uses: the multiprocessor count that caps the
 * split-K factor (CudaFloat32EngineBase.java:73). */
int alpha_conv_device_info(int *compute_units, int *clock_khz);

/* Debugging switch: kernel family used inside the entries (tests and comparisons; not part of the drop-in contract):
 * 0 = auto, 1 = implicit GEMM only (LDS-halo kernel where eligible, else the generic one),
 * 2 = Winograd F(2x2,3x3) where eligible, 3 = the generic kernels only,
 * 4 = backward-filter through the tap-per-workgroup kernel wherever it fits, 5 = through the row-streaming kernel
 * wherever it fits (forward and backward-data as 0), 6 = forward from CW through the kernel without LDS wherever it fits.
 * Also read once from the environment variable ALPHA_HIP_CONV_ALGO = auto|igemm|winograd|generic|taps|rows|direct.
 * No counterpart in the reference (its Winograd experiments are compiled out, conv/conv3D.cuh:39-44). */
int alpha_conv_set_fwd_algo(int algo);
int alpha_conv_get_fwd_algo(void);
/* Scratch for the calling thread's next calls (no counterpart in the reference, whose natives get no scratch beyond CW and
 * deltaW_buf): device memory the caller lends until it binds NULL again; kernels enqueued by this thread's calls in
 * between may write it, so it must stay untouched until they have finished (stream order). With at least 1 MiB the
 * forward and stride-1 backward-data entries deal layers of few work items per compute unit out in equal shares (the
 * items left over are cut along the reduction, their pieces added by a short second kernel in a fixed order: results are
 * bit-identical from run to run, and differ from the unbound path's in the last bits of those items only). Per thread:
 * concurrent callers do not see each other's binding. */
int alpha_conv_bind_workspace(float *workspace, long bytes);
/* No counterpart in the reference. Beside a bound workspace: `count` 32-bit words of device memory (128 cover every layer)
 * that are ZERO when bound and that only this library's kernels write until NULL is bound again; every kernel leaves them
 * zero. With them the pieces of the items left over are added by the workgroup that delivers an item's last piece - a
 * ticket per item decides WHO adds, never the order, so the bits are those of the second kernel - and the second launch
 * is saved. Kernels that share the words must not overlap on the device (the rule of the workspace). Per thread. */
int alpha_conv_bind_tickets(unsigned *tickets, int count);
/* Debugging switch of the same kind for 1x1 stride-1 forward / backward-data where the kernel of direct_conv.hip does not
 * take the layer: -1 = chosen by shape, 0 = the filter-resident kernel, 1 = the kernel without LDS wherever it fits.
 * Also read once from the environment variable ALPHA_PW_DIRECT = 0|1. No counterpart in the reference. */
int alpha_conv_set_pointwise_algo(int algo);
/* And for kernel-split backward-data through the kernel without LDS (all phases of one size, deltaY channels a multiple
 * of 32): -1 = by shape, 0 = every wavefront works on items of its own, 1 = the eight wavefronts of a workgroup share
 * every group of items, each taking an eighth of the reduction (what layers with few items per compute unit get by
 * shape). Also read once from the environment variable ALPHA_KS_SHARED = 0|1. No counterpart in the reference. */
int alpha_conv_set_kernel_split_sharing(int sharing);
/* And for backward-filter through the persistent kernel (delta_w_stream.hip), where its workgroups are not one piece of
 * an item each: -1 = by shape, 0 = the line of items in equal shares, 1 = every item in equal pieces and the (piece, item)
 * units dealt out whole, wherever GridZ allows (what large tensors with few items get by shape). The split-K helpers
 * (alpha_dconv3D_deltaW_least_GridZ, the engine's options) follow the switch. Also read once from the environment
 * variable ALPHA_DW_UNITS = 0|1. No counterpart in the reference. */
int alpha_conv_set_deltaW_units(int units);

/* ---- Cuda_conv3D: forward ------------------------------------------------------------------ */

/* conv/A.cu:14   Java: Cuda_conv3D.conv3D */
int alpha_conv3D(const int64_t *streams, int length,
                 const float *X, int IH, int IW,
                 const float *W, int FH, int FW,
                 float *Y, int OH, int OW,
                 int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* conv/A.cu:38   Java: Cuda_conv3D.conv3D_texture */
int alpha_conv3D_texture(const int64_t *streams, int length,
                         const float *X, int IH, int IW,
                         const float *W, int FH, int FW,
                         float *Y, int OH, int OW,
                         int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* conv/A.cu:64   Java: Cuda_conv3D.conv3DV2 */
int alpha_conv3DV2(int useTexture, const int64_t *streams, int length,
                   const float *X, int IH, int IW,
                   const float *W, int FH, int FW,
                   float *Y, int OH, int OW,
                   int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* conv/A.cu:89   Java: Cuda_conv3D.conv3D_np  (ph = pw = 0) */
int alpha_conv3D_np(const int64_t *streams, int length,
                    const float *X, int IH, int IW,
                    const float *W, int FH, int FW,
                    float *Y, int OH, int OW,
                    int N, int IC, int OC, int sh, int sw);

/* conv/A.cu:112  Java: Cuda_conv3D.conv3D_W1  (1x1 filter, stride 1, pad 0) */
int alpha_conv3D_W1(const int64_t *streams, int length,
                    const float *X, int IH, int IW,
                    const float *W, float *Y,
                    int N, int IC, int OC);

/* conv/A.cu:137  Java: Cuda_conv3D.kernel_remode   W[OC,FH,FW,IC] -> CW[FH,FW,IC,OC] */
int alpha_kernel_remode(int64_t stream, const float *W, float *CW, int FH, int FW, int OC, int IC);

/* conv/A.cu:149  Java: Cuda_conv3D.conv3D_GemmR   (CW = remoded filter). W is the filter CW was made from, as the
 * Java engine passes it (the reference hands both to its kernels, conv/A.cu:165-170): layers with 4 stored input
 * channels read its 16-byte taps in place; NULL is accepted and keeps every layer on CW. The same holds for the other
 * entries that take W and CW. */
int alpha_conv3D_GemmR(const int64_t *streams, int length,
                       const float *X, int IH, int IW,
                       const float *W, const float *CW, int FH, int FW,
                       float *Y, int OH, int OW,
                       int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* conv/A.cu:174  Java: Cuda_conv3D.conv3D_GemmR_texture */
int alpha_conv3D_GemmR_texture(const int64_t *streams, int length,
                               const float *X, int IH, int IW,
                               const float *W, const float *CW, int FH, int FW,
                               float *Y, int OH, int OW,
                               int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* conv/A.cu:201  Java: Cuda_conv3D.conv3D_GemmV2R */
int alpha_conv3D_GemmV2R(int useTexture, const int64_t *streams, int length,
                         const float *X, int IH, int IW,
                         const float *W, const float *CW, int FH, int FW,
                         float *Y, int OH, int OW,
                         int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* conv/A.cu:227  Java: Cuda_conv3D.conv3D_GemmR_W1 */
int alpha_conv3D_GemmR_W1(const int64_t *streams, int length,
                          const float *X, int IH, int IW,
                          const float *W, const float *CW, float *Y,
                          int N, int IC, int OC);

/* ---- Cuda_dconv3D_deltaX: backward-data ------------------------------------------------------ */

/* dX/A.cu:14   Java: Cuda_dconv3D_deltaX.dconv3D_deltaX_s1  (stride 1) */
int alpha_dconv3D_deltaX_s1(const int64_t *streams, int length,
                            const float *deltaY, int OH, int OW,
                            const float *W, int FH, int FW,
                            float *deltaX, int IH, int IW,
                            int N, int IC, int OC, int ph, int pw);

/* dX/A.cu:38   Java: dconv3D_deltaX_s1_texture */
int alpha_dconv3D_deltaX_s1_texture(const int64_t *streams, int length,
                                    const float *deltaY, int OH, int OW,
                                    const float *W, int FH, int FW,
                                    float *deltaX, int IH, int IW,
                                    int N, int IC, int OC, int ph, int pw);

/* dX/A.cu:64   Java: dconv3D_deltaX_V2_s1 */
int alpha_dconv3D_deltaX_V2_s1(int useTexture, const int64_t *streams, int length,
                               const float *deltaY, int OH, int OW,
                               const float *W, int FH, int FW,
                               float *deltaX, int IH, int IW,
                               int N, int IC, int OC, int ph, int pw);

/* dX/A.cu:88   Java: dconv3D_deltaX_W1  (1x1, stride 1, pad 0) */
int alpha_dconv3D_deltaX_W1(const int64_t *streams, int length,
                            const float *deltaY, const float *W,
                            float *deltaX, int IH, int IW,
                            int N, int IC, int OC);

/* dX/A.cu:115  Java: ks_remode   W -> CW[sh*sw][OC][CFH][CFW][IC]  (layout v1; CFH = ceil(FH/sh)) */
int alpha_ks_remode(int64_t stream, const float *W, int FH, int FW,
                    float *CW, int CFH, int CFW, int OC, int IC, int sh, int sw);

/* dX/A.cu:128  Java: ks_remodev2 W -> CW[sh*sw][CFH][CFW][OC][IC]  (layout v2, the one consumed below) */
int alpha_ks_remodev2(int64_t stream, const float *W, int FH, int FW,
                      float *CW, int CFH, int CFW, int OC, int IC, int sh, int sw);

/* dX/A.cu:141  Java: dconv3D_deltaX_kernelSplit  (any stride; CW in layout v2) */
int alpha_dconv3D_deltaX_kernelSplit(const int64_t *streams, int length,
                                     const float *deltaY, int OH, int OW,
                                     const float *CW, int FH, int FW,
                                     float *deltaX, int IH, int IW,
                                     int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* dX/A.cu:166  Java: dconv3D_deltaX_ksImsR  (IH % sh == 0, IW % sw == 0) */
int alpha_dconv3D_deltaX_ksImsR(const int64_t *streams, int length,
                                const float *deltaY, int OH, int OW,
                                const float *CW, int FH, int FW,
                                float *deltaX, int IH, int IW,
                                int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* dX/A.cu:191  Java: dconv3D_deltaX_ksImsR_texture */
int alpha_dconv3D_deltaX_ksImsR_texture(const int64_t *streams, int length,
                                        const float *deltaY, int OH, int OW,
                                        const float *CW, int FH, int FW,
                                        float *deltaX, int IH, int IW,
                                        int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* dX/A.cu:218  Java: dconv3D_deltaX_ksIms2R  (sh = sw = 2, IH and IW even) */
int alpha_dconv3D_deltaX_ksIms2R(const int64_t *streams, int length,
                                 const float *deltaY, int OH, int OW,
                                 const float *CW, int FH, int FW,
                                 float *deltaX, int IH, int IW,
                                 int N, int IC, int OC, int ph, int pw);

/* dX/A.cu:243  Java: dconv3D_deltaX_ksIms2R_texture */
int alpha_dconv3D_deltaX_ksIms2R_texture(const int64_t *streams, int length,
                                         const float *deltaY, int OH, int OW,
                                         const float *CW, int FH, int FW,
                                         float *deltaX, int IH, int IW,
                                         int N, int IC, int OC, int ph, int pw);

/* dX/A.cu:270  Java: dconv3D_deltaX_ksV2_Ims2R */
int alpha_dconv3D_deltaX_ksV2_Ims2R(int useTexture, const int64_t *streams, int length,
                                    const float *deltaY, int OH, int OW,
                                    const float *CW, int FH, int FW,
                                    float *deltaX, int IH, int IW,
                                    int N, int IC, int OC, int ph, int pw);

/* dX/A.cu:300  Java: dconv3D_deltaX_crossAdd  (small IC; reads W, not CW).
 * The reference zero-fills deltaX and scatters with atomicAdd (summation order varies from run
 * to run). This implementation gathers instead: same mathematical result, no atomics, no
 * memset, bit-reproducible. */
int alpha_dconv3D_deltaX_crossAdd(const int64_t *streams, int length,
                                  const float *deltaY, int OH, int OW,
                                  const float *W, int FH, int FW,
                                  float *deltaX, int IH, int IW,
                                  int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* ---- Cuda_dconv3D_deltaW: backward-filter ---------------------------------------------------- */

/* dW/A.cu:16   Java: Cuda_dconv3D_deltaW.dconv3D_deltaW  (single pass over GK = N*OH*OW) */
int alpha_dconv3D_deltaW(const int64_t *streams, int length,
                         const float *X, int IH, int IW,
                         const float *deltaY, int OH, int OW,
                         float *deltaW, int FH, int FW,
                         int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* dW/A.cu:39   Java: dconv3D_deltaW_W1  (1x1, stride 1, pad 0) */
int alpha_dconv3D_deltaW_W1(const int64_t *streams, int length,
                            const float *X, int IH, int IW,
                            const float *deltaY, float *deltaW,
                            int N, int IC, int OC);

/* dW/A.cu:66   Java: buf_summary   deltaW += sum_{p<part} deltaW_buf[p], fixed order, fp32 Kahan */
int alpha_buf_summary(int64_t stream, const float *deltaW_buf, float *deltaW, int part, int sizeW);

/* dW/A.cu:79   Java: dconv3D_deltaW_GemmSK.  Split-K: deltaW and the GridZ-1 buffers of deltaW_buf (sizeW floats
 * each) receive partial sums that add up to the result; the caller sums them with alpha_buf_summary(part = GridZ-1).
 * Every element of all of them is written (zeros where a buffer is not needed). No atomics: bit-reproducible.
 * Which pixels a buffer holds: the reference's partition (buffer z the pixels [z*GK_slice, (z+1)*GK_slice), GK_slice =
 * (GK/GridZ) >> 3 << 3, the last slice the remainder) in the kernels behind alpha_conv_set_fwd_algo(4) and for layers
 * the default kernel does not take; the default kernel deals the pixels out evenly over the compute units instead. */
int alpha_dconv3D_deltaW_GemmSK(const int64_t *streams, int length, int GridZ,
                                const float *X, int IH, int IW,
                                const float *deltaY, int OH, int OW,
                                float *deltaW, float *deltaW_buf, int FH, int FW,
                                int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* dW/A.cu:106  Java: dconv3D_deltaW_GemmV2SK  (same contract as GemmSK) */
int alpha_dconv3D_deltaW_GemmV2SK(const int64_t *streams, int length, int GridZ,
                                  const float *X, int IH, int IW,
                                  const float *deltaY, int OH, int OW,
                                  float *deltaW, float *deltaW_buf, int FH, int FW,
                                  int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* dW/A.cu:132  Java: dconv3D_deltaW_GemmSK_W1  (1x1 split-K) */
int alpha_dconv3D_deltaW_GemmSK_W1(const int64_t *streams, int length, int GridZ,
                                   const float *X, int IH, int IW,
                                   const float *deltaY, float *deltaW, float *deltaW_buf,
                                   int N, int IC, int OC);

/* No counterpart in the reference (its split-K factor is the Java engine's choice,
 * CudaFloat32EngineBase.java:1707-1715, sized for devices of at most 128 multiprocessors). The
 * least GridZ' <= GridZ with which alpha_dconv3D_deltaW_GemmSK / _GemmV2SK / _GemmSK_W1 on a device
 * of `units` compute units cut this layer exactly as they do with GridZ - their persistent kernel
 * deals the pixels evenly among the compute units whatever GridZ is, and buffers beyond what it needs
 * are only filled with zeros -, or GridZ itself for layers that kernel does not serve. A caller that
 * passes the result instead of GridZ allocates and sums fewer partial results. Pure host arithmetic:
 * no device is touched. */
int alpha_dconv3D_deltaW_least_GridZ(int units, int GridZ, int OH, int OW, int FH, int FW, int N, int IC, int OC);

/* No counterpart in the reference. For callers that cannot allocate device memory or hand over a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Same computation as alpha_dconv3D_deltaW_GemmSK followed by alpha_buf_summary(deltaW_buf, deltaW,
 * GridZ - 1, OC*FH*FW*IC) on streams[0], bit for bit, but the GridZ - 1 partial results live in a
 * static device array of ALPHA_CONV_STATIC_SCRATCH_BYTES inside the library (one copy per GPU, held
 * until the process ends) and the call neither allocates nor frees anything. deltaW is complete
 * when streams[0] has run the enqueued work. (GridZ - 1) * OC*FH*FW*IC * 4 bytes beyond the array's
 * size is refused with ALPHA_CONV_EINVAL. All calls on one GPU share the array: calls whose work
 * overlaps in time on one GPU race (order them on one stream or with events).
 * alpha_conv_device_info() resolves the array's address for the current device; a caller that
 * captures graphs calls it once per device before capturing. */
#define ALPHA_CONV_STATIC_SCRATCH_BYTES (32u << 20)
int alpha_dconv3D_deltaW_GemmSK_static(const int64_t *streams, int length, int GridZ,
                                       const float *X, int IH, int IW,
                                       const float *deltaY, int OH, int OW,
                                       float *deltaW, int FH, int FW,
                                       int N, int IC, int OC, int sh, int sw, int ph, int pw);

/* ---- this build's additional forward algorithm ------------------------------------------- */

/* Winograd F(2x2,3x3) forward for FH = FW = 3, stride 1. No counterpart among the reference's
 * JNI methods. U is scratch of alpha_winograd_filter_size(IC, OC) floats supplied by the caller
 * (the transformed filter, 16 * IC * OC); alpha_winograd_filter_transform fills it from
 * W[OC,3,3,IC]; alpha_conv3D_winograd then consumes it. U is opaque: its element order depends on IC
 * (the two calls agree on it) and only these two entries may interpret it. */
long alpha_winograd_filter_size(int IC, int OC);
int alpha_winograd_filter_transform(int64_t stream, const float *W, float *U, int IC, int OC);
int alpha_conv3D_winograd(const int64_t *streams, int length,
                          const float *X, int IH, int IW,
                          const float *U,
                          float *Y, int OH, int OW,
                          int N, int IC, int OC, int ph, int pw);

/* The same algorithm for backward-data of a 3x3 stride-1 layer (deltaX = forward convolution of deltaY with the
 * rotated filter, OC channels in, IC out, padding 2 - p). No counterpart in the reference (its backward-data natives,
 * Cuda_dconv3D_deltaX.java:311-478, take W and no scratch); a caller that wants it supplies U
 * (alpha_winograd_filter_size(IC, OC) floats) like CW of the kernel-split entries. ph, pw <= 2. */
int alpha_winograd_filter_transform_deltaX(int64_t stream, const float *W, float *U, int IC, int OC);
int alpha_dconv3D_deltaX_winograd(const int64_t *streams, int length,
                                  const float *deltaY, int OH, int OW,
                                  const float *U,
                                  float *deltaX, int IH, int IW,
                                  int N, int IC, int OC, int ph, int pw);

/* Backward-filter of a 3x3 stride-1 layer by Winograd F(3x3,2x2): arguments and split-K contract of
 * alpha_dconv3D_deltaW_GemmSK (slice z writes deltaW, z = 0, or deltaW_buf[z-1]; alpha_buf_summary finishes), without FH, FW,
 * sh, sw. The slices are ranges of 2x2 output tiles instead of the reference's pixel ranges
 * (cu32/dW/dconv3d_dW_GemmSK_kernel.cuh:131-262), so the partial results differ from the direct entry's while their sum
 * is the same up to rounding. No counterpart in the reference. */
int alpha_dconv3D_deltaW_GemmSK_winograd(const int64_t *streams, int length, int GridZ,
                                         const float *X, int IH, int IW,
                                         const float *deltaY, int OH, int OW,
                                         float *deltaW, float *deltaW_buf,
                                         int N, int IC, int OC, int ph, int pw);

/* ---- forward with the bias added in the kernel's epilogue --------------------------------------
 * The reference has no native for this: its engine method conv3D_biased (CudaFloat32EngineBase.java:1478-1560,
 * EngineBase.java:178-185) runs the conv3D entry and then Cuda_function.linear_dual2D_row(Y, Bias, ...) =
 * Y[., oc] = 1*Y[., oc] + 1*Bias[oc] + 0 as a second pass over Y on its own stream. These entries give the same
 * result (Bias has OC entries, OC the stored, x4-padded channel count) without the second pass; a maintainer binds
 * them as new natives of Cuda_conv3D next to conv3D / conv3D_GemmR and calls them from conv3D_biased. */
int alpha_conv3D_biased(const int64_t *streams, int length,
                        const float *X, int IH, int IW,
                        const float *W, int FH, int FW,
                        const float *Bias,
                        float *Y, int OH, int OW,
                        int N, int IC, int OC, int sh, int sw, int ph, int pw);
int alpha_conv3D_GemmR_biased(const int64_t *streams, int length,
                              const float *X, int IH, int IW,
                              const float *W, const float *CW, int FH, int FW,
                              const float *Bias,
                              float *Y, int OH, int OW,
                              int N, int IC, int OC, int sh, int sw, int ph, int pw);
int alpha_conv3D_winograd_biased(const int64_t *streams, int length,
                                 const float *X, int IH, int IW,
                                 const float *U, const float *Bias,
                                 float *Y, int OH, int OW,
                                 int N, int IC, int OC, int ph, int pw);

/* Backward-filter plus the bias gradient deltaB[oc] = sum over all pixels of deltaY[., oc] (the reference computes it
 * with a separate reduction, eg.field_sum(deltaY, OC), nn/unit/simple/Conv3D.java:160). Same split-K contract as
 * alpha_dconv3D_deltaW_GemmSK: slice z of GK_slice = (GK/GridZ)>>3<<3 pixels writes its partial column sums to deltaB
 * (z = 0) or deltaB_buf[(z-1)*OC ..]; the caller finishes with alpha_buf_summary(stream, deltaB_buf, deltaB, GridZ-1, OC)
 * next to the one for deltaW. deltaB_buf holds (GridZ-1)*OC floats (may be NULL when GridZ = 1). Bit-reproducible. */
int alpha_dconv3D_deltaW_GemmSK_deltaB(const int64_t *streams, int length, int GridZ,
                                       const float *X, int IH, int IW,
                                       const float *deltaY, int OH, int OW,
                                       float *deltaW, float *deltaW_buf,
                                       float *deltaB, float *deltaB_buf,
                                       int FH, int FW, int N, int IC, int OC,
                                       int sh, int sw, int ph, int pw);

/* ---- this build's fused epilogues: batch normalisation and leaky ReLU around the convolution ------------------------
 * The reference runs them as separate passes over the convolution's output: conv3D, then batchNorm2D_row /
 * batchNorm_affined2D_row (Cuda_function.java:3829, 3862; in inference, statistics given), then leakyRelu2D (:1607) -
 * after every convolution of its ResNets (experiments/alpha_code/src/cifar10/resnet18/Net.java:42-58) - and, going back,
 * leakyRelu2D_deltaX_v1 (:1640) before dconv3D_deltaX. Here they ride in the convolution kernels' epilogues where a
 * kernel has the fused form (the LDS-halo kernels, the stem kernel, the generic kernel, the non-persistent Winograd
 * kernel) and are one more pass over the output otherwise (1x1 streaming kernel, persistent Winograd kernel). */
typedef struct alpha_conv_epilogue {
    const float *Bias;     /* NULL or [OC]: added first */
    const float *X_mean;   /* NULL or [OC], with X_var: y = (y - X_mean) * rsqrt(X_var + eps) */
    const float *X_var;
    float eps;
    const float *A;        /* NULL or [OC], with B: y = A * y + B */
    const float *B;
    float k;               /* leaky ReLU: y = y > 0 ? y : k * y; k = 1 leaves y alone */
} alpha_conv_epilogue;

/* Y = leakyRelu(batchNorm(conv3D(X, W) + Bias)), filter read as W[OC,FH,FW,IC] (conv/A.cu:14 + the row functions) */
int alpha_conv3D_fused(const int64_t *streams, int length,
                       const float *X, int IH, int IW,
                       const float *W, int FH, int FW,
                       const alpha_conv_epilogue *epilogue,
                       float *Y, int OH, int OW,
                       int N, int IC, int OC, int sh, int sw, int ph, int pw);
/* the same from the re-laid-out filter CW (conv/A.cu:149) */
int alpha_conv3D_GemmR_fused(const int64_t *streams, int length,
                             const float *X, int IH, int IW,
                             const float *W, const float *CW, int FH, int FW,
                             const alpha_conv_epilogue *epilogue,
                             float *Y, int OH, int OW,
                             int N, int IC, int OC, int sh, int sw, int ph, int pw);
/* the same through Winograd F(2x2,3x3) from the transformed filter U */
int alpha_conv3D_winograd_fused(const int64_t *streams, int length,
                                const float *X, int IH, int IW, const float *U,
                                const alpha_conv_epilogue *epilogue,
                                float *Y, int OH, int OW, int N, int IC, int OC, int ph, int pw);
/* deltaX = dconv3D_deltaX_s1(deltaY, W) * (Xf > 0 ? 1 : k): stride-1 backward-data (dX/A.cu:14) fused with the backward of
 * the leaky ReLU whose output Xf[N,IH,IW,IC] is this layer's input (leakyRelu2D_deltaX_v1 applied to the result). */
int alpha_dconv3D_deltaX_s1_leakyRelu(const int64_t *streams, int length,
                                      const float *deltaY, int OH, int OW,
                                      const float *W, int FH, int FW,
                                      const float *Xf, float k,
                                      float *deltaX, int IH, int IW,
                                      int N, int IC, int OC, int ph, int pw);
/* the same for any stride, from the kernel-split filter layout of alpha_ks_remodev2 (dX/A.cu:141) */
int alpha_dconv3D_deltaX_kernelSplit_leakyRelu(const int64_t *streams, int length,
                                               const float *deltaY, int OH, int OW,
                                               const float *CW, int FH, int FW,
                                               const float *Xf, float k,
                                               float *deltaX, int IH, int IW,
                                               int N, int IC, int OC, int sh, int sw, int ph, int pw);
/* The row functions themselves (one HBM-bound pass; X == Y allowed), argument order of the reference's natives:
 * lengthv = height * mem_stride elements, mem_width data elements per row, the mem_stride - mem_width pad elements are
 * written as zeros. row_lengthv (the length of X_mean / X_var) must equal mem_stride. */
int alpha_leakyRelu2D(int64_t stream, const float *X, float k, float *Y, int lengthv, int mem_width, int mem_stride);
int alpha_leakyRelu2D_deltaX_v1(int64_t stream, float *deltaX, const float *deltaY, const float *Y, float k,
                                int lengthv, int mem_width, int mem_stride);
int alpha_batchNorm2D_row(int64_t stream, const float *X, const float *X_mean, const float *X_var, float eps, int row_lengthv,
                          float *Y, int lengthv, int mem_width, int mem_stride);
int alpha_batchNorm_affined2D_row(int64_t stream, const float *X, const float *X_mean, const float *X_var, float eps,
                                  const float *A, const float *B, int row_lengthv,
                                  float *Y, int lengthv, int mem_width, int mem_stride);

/* ---- backward of batch normalisation around the convolution ---------------------------------------------------------
 * The reference's training step runs these between leakyRelu2D_deltaX and dconv3D_deltaX
 * (CudaFloat32EngineBase.java:4385-4760: batchNorm2D_deltaX_v1 / _v2, batchNorm2D_gradients_v1 / _v2). The tensor is
 * [N = field_length rows, M = row_lengthv columns] (rows = pixels of the batch, columns = channels, M == mem_stride).
 *
 * Field sums (Cuda_reduce.java:697, 746, 939; reduce/A.cu:486 and twins): per column m
 *     deltaB[m] = deltaXp1[m] = sum_n deltaY[n, m]            deltaA[m] = deltaXp2[m] = sum_n deltaY[n, m] * X_norm[n, m]
 * with X_norm = (Y - B) / A (affine_v1), = the second tensor itself (affine_v2), = (X - X_mean) * rsqrt(X_var + eps)
 * (batchNorm_v2). deltaA_buf / deltaB_buf hold field_nextN(N, M) * M floats each (may be NULL when that is 1) and a
 * result may be the head of its own buffer, as the Java engine passes them. Everything is enqueued on stream1 (stream2 is
 * accepted and left idle). Deterministic: fixed summation order, bit-identical from run to run. The reference's natives
 * return the number of rows left after their last stage; here that value goes to *nextN (may be NULL) and the return
 * value is the status, as for every entry of this header. */
int alpha_field_affine_deltaAB_v1(int64_t stream1, int64_t stream2, const float *deltaY, const float *Y, const float *A, const float *B,
                                  int N, int M, float *deltaA_buf, float *deltaA, float *deltaB_buf, float *deltaB,
                                  int mem_width, int mem_stride, int partNum, int *nextN);
int alpha_field_affine_deltaAB_v2(int64_t stream1, int64_t stream2, const float *deltaY, const float *X_norm,
                                  int N, int M, float *deltaA_buf, float *deltaA, float *deltaB_buf, float *deltaB,
                                  int mem_width, int mem_stride, int partNum, int *nextN);
int alpha_field_batchNorm_deltaAB_v2(int64_t stream1, int64_t stream2, const float *deltaY, const float *X, const float *X_mean,
                                     const float *X_var, float eps, int N, int M, float *deltaA_buf, float *deltaA,
                                     float *deltaB_buf, float *deltaB, int mem_width, int mem_stride, int partNum, int *nextN);
/* Row functions (Cuda_function.java:3890, 3923, 3958, 3992; function/extra_batchNorm*_row_deltaX_v*.cuh):
 *     deltaX = scale * (deltaY - (deltaXp1 + deltaXp2 * X_norm) / N),   N = lengthv / row_lengthv,
 * scale = rsqrt(X_var + eps) (times A for the affine forms); v1 takes X_norm from the layer's output Y (Y itself, or
 * (Y - B) / A), v2 from its input X. Pad elements (mem_width <= column < mem_stride) are written as zeros, and so are NaN
 * results of the affine v1 form (A == 0), as in the reference. deltaX may be deltaY. */
int alpha_batchNorm2D_row_deltaX_v1(int64_t stream, const float *deltaY, const float *Y, const float *X_var, float eps,
                                    const float *deltaXp1, const float *deltaXp2, int row_lengthv, float *deltaX,
                                    int lengthv, int mem_width, int mem_stride);
int alpha_batchNorm2D_row_deltaX_v2(int64_t stream, const float *deltaY, const float *X, const float *X_mean, const float *X_var, float eps,
                                    const float *deltaXp1, const float *deltaXp2, int row_lengthv, float *deltaX,
                                    int lengthv, int mem_width, int mem_stride);
int alpha_batchNorm_affined2D_row_deltaX_v1(int64_t stream, const float *deltaY, const float *Y, const float *X_var, float eps,
                                            const float *A, const float *B, const float *deltaXp1, const float *deltaXp2,
                                            int row_lengthv, float *deltaX, int lengthv, int mem_width, int mem_stride);
int alpha_batchNorm_affined2D_row_deltaX_v2(int64_t stream, const float *deltaY, const float *X, const float *X_mean, const float *X_var,
                                            float eps, const float *A, const float *deltaXp1, const float *deltaXp2,
                                            int row_lengthv, float *deltaX, int lengthv, int mem_width, int mem_stride);

#ifdef __cplusplus
}
#endif
#endif /* ALPHA_CONV_H */
