/*
 * alpha_engine.h — host-side counterpart of the reference's Java algorithm selection for the conv3D path
 * (src/alpha_src/z/dragon/engine/cuda/CudaFloat32EngineBase.java:1323-2005), restated in C++ because there is no JVM
 * in the build environment. Two layers:
 *   alpha_plan_*    pure integer functions: which native entry the Java engine would call for a layer, with how many
 *                   stream handles, whether it remodes the filter, the split-K factor GridZ and the scratch size.
 *   alpha_engine_*  an object that owns the scratch buffers (the Java engine takes them from its memory pool and frees
 *                   them when the returned Syncer completes) and calls the natives of alpha_conv.h in the same order
 *                   as the Java code: remode -> conv entry; split-K entry -> buf_summary; ks_remodev2 -> kernel-split.
 * Flags and thresholds are the reference's fluent setters with their defaults.
 */
#ifndef ALPHA_ENGINE_H
#define ALPHA_ENGINE_H

#include <stdint.h>

#include "alpha_conv.h"   /* alpha_conv_epilogue */

#ifdef __cplusplus
extern "C" {
#endif

/* CudaFloat32EngineBase.java:1324-1352 (forward), :1630-1663 (deltaW), :1765-1793 (deltaX) */
typedef struct alpha_engine_config {
    int conv3D_useTexture;        /* true */
    int conv3D_remode;            /* true */
    float conv3D_remode_V2_Q;     /* 1.05 */
    float conv3D_V2_Q;            /* 1.25 */
    int deltaW_SplitKThreshold;   /* 512 */
    int deltaW_SK_MaxPartNum;     /* clip(#compute units, 16, 128)  (:73) */
    float deltaW_SK_V2_Q;         /* 1.15 */
    int deltaX_s1_useTexture;     /* true */
    int deltaX_ks_useTexture;     /* false */
    float deltaX_s1_V2_Q;         /* 1.1 */
    float deltaX_ks_V2_Q;         /* 1.1 */
    int conv3D_winograd;          /* this build only (no reference flag): 1 = 3x3 stride-1 forward through Winograd F(2x2,3x3); default 0 */
    int deltaW_SK_fillUnits;      /* this build only: when > 0, the split-K factor is raised (never lowered) until the launch has two
                                     workgroups (one when output rows are wider than 36 pixels) for each of this many compute units,
                                     slices staying >= 256 pixels; default 0 = the reference's GridZ exactly */
    int cache_filter_transforms;  /* this build only: 1 = keep kernel_remode / ks_remodev2 / Winograd filter transforms between calls,
                                     keyed by the filter's address and geometry; the caller reports weight updates with
                                     alpha_engine_filter_changed(). Default 0: re-transform on every call like the reference
                                     (CudaFloat32EngineBase.java:1373-1380, 1879-1889) */
    int deltaX_winograd;          /* this build only: 1 = backward-data of 3x3 stride-1 layers (padding <= 2, more than 8 input
                                     channels) through Winograd F(2x2,3x3); default 0 */
    int deltaW_winograd;          /* this build only: > 0 = backward-filter of 3x3 stride-1 layers (split-K case) through Winograd
                                     F(3x3,2x2). 1: with the reference's GridZ; > 1: the number of compute units to fill - GridZ becomes
                                     that many workgroups' worth of slices (at least 64 tiles each). Default 0 */
    int deltaW_SK_leastUnits;     /* this build only: > 0 = the number of compute units of the device; the split-K factor is then lowered
                                     to the least value with which the persistent backward-filter kernel cuts the layer the same way -
                                     it deals the pixels evenly among the compute units whatever GridZ is, so a larger GridZ only adds
                                     buffers of zeros for buf_summary to add -, and raised, within the reference's own cap of GK / 256,
                                     where the reference's value has fewer buffers than that kernel's cut needs pieces per item (2 on
                                     4x4 maps at N = 512; first layers - 4 stored input channels -, whose kernel runs GridZ x groups of
                                     16 taps x blocks of 64 output channels workgroups). alpha_engine_config_default: 0 = the reference's GridZ exactly;
                                     alpha_engine_create sets it to the device's compute units */
    int conv_workspace;           /* this build only: 1 = forward and stride-1 backward-data calls lend the library 1 MiB of the engine's
                                     scratch for the duration of the call (alpha_conv_bind_workspace), with which the kernel without
                                     LDS deals a layer of few items per compute unit out in equal shares (7x7x512 and 14x14x256 maps at
                                     N = 64: 6 and 12 items each plus a piece of one, instead of 6 or 7 and 12 or 13), and the engine's
                                     ticket words (alpha_conv_bind_tickets), with which the pieces are added inside that kernel;
                                     2 = the scratch without the ticket words (a second short kernel adds the pieces).
                                     alpha_engine_config_default: 0; alpha_engine_create: 1 */
} alpha_engine_config;

/* Native entry chosen by a plan; names are the Java native method names. */
enum alpha_entry {
    ALPHA_E_conv3D = 1, ALPHA_E_conv3D_texture, ALPHA_E_conv3DV2, ALPHA_E_conv3D_np, ALPHA_E_conv3D_W1,
    ALPHA_E_conv3D_GemmR, ALPHA_E_conv3D_GemmR_texture, ALPHA_E_conv3D_GemmV2R, ALPHA_E_conv3D_GemmR_W1,
    ALPHA_E_dconv3D_deltaX_s1, ALPHA_E_dconv3D_deltaX_s1_texture, ALPHA_E_dconv3D_deltaX_V2_s1, ALPHA_E_dconv3D_deltaX_W1,
    ALPHA_E_dconv3D_deltaX_kernelSplit, ALPHA_E_dconv3D_deltaX_ksImsR, ALPHA_E_dconv3D_deltaX_ksImsR_texture,
    ALPHA_E_dconv3D_deltaX_ksIms2R, ALPHA_E_dconv3D_deltaX_ksIms2R_texture, ALPHA_E_dconv3D_deltaX_ksV2_Ims2R,
    ALPHA_E_dconv3D_deltaX_crossAdd,
    ALPHA_E_dconv3D_deltaW, ALPHA_E_dconv3D_deltaW_W1, ALPHA_E_dconv3D_deltaW_GemmSK, ALPHA_E_dconv3D_deltaW_GemmV2SK,
    ALPHA_E_dconv3D_deltaW_GemmSK_W1,
    ALPHA_E_conv3D_winograd,  /* this build's additional forward algorithm; never chosen unless conv3D_winograd is set */
    ALPHA_E_dconv3D_deltaX_winograd,  /* the same for backward-data; never chosen unless deltaX_winograd is set */
    ALPHA_E_dconv3D_deltaW_GemmSK_winograd   /* Winograd F(3x3,2x2) backward-filter; never chosen unless deltaW_winograd is set */
};

typedef struct alpha_conv_plan {
    int entry;            /* enum alpha_entry */
    int streams;          /* length of the stream array the Java engine would pass */
    int remode;           /* 1 when kernel_remode / ks_remodev2 runs first */
    int V2;               /* the "V2" variant was chosen */
    int useTexture;       /* flag passed to entries that take one */
    int GridZ;            /* split-K factor (deltaW), 1 = single pass */
    long scratch_floats;  /* CW or deltaW_buf size */
    double Q;             /* padding scale-up the decision was based on */
} alpha_conv_plan;

/* Integer helpers of the Java native classes. GN, GM are the implicit-GEMM extents each class uses:
 * forward (OC, N*OH*OW), deltaX (IC, N*IH*IW), deltaW (OC, FH*FW*IC); the V2 variants pass (OC, N) etc. and multiply
 * blockNum by the spatial size themselves. Cuda_conv3D.java:19-126, Cuda_dconv3D_deltaX.java:19-190, Cuda_dconv3D_deltaW.java:19-128. */
int alpha_blockNum(int GN, int GM);
int alpha_streamSize(int GN, int GM, int cap);
double alpha_paddingScaleUp(int IH, int IW, int OH, int OW, int FH, int FW, int sh, int sw);

void alpha_engine_config_default(alpha_engine_config *c, int compute_units);

/* EngineCore.conv3D_param_check (EngineCore.java:630-678, non-strict) minus its sh <= FH rule: NULL when the sizes are
 * consistent, else the reason. The engine calls refuse (ALPHA_CONV_EINVAL) what this refuses. */
const char *alpha_engine_param_check(int OH, int OW, int IH, int IW, int FH, int FW, int N, int IC, int OC,
                                     int sh, int sw, int ph, int pw);

void alpha_plan_conv3D(const alpha_engine_config *c, int IH, int IW, int OH, int OW, int FH, int FW, int N, int IC, int OC,
                       int sh, int sw, int ph, int pw, alpha_conv_plan *out);
void alpha_plan_deltaW(const alpha_engine_config *c, int IH, int IW, int OH, int OW, int FH, int FW, int N, int IC, int OC,
                       int sh, int sw, alpha_conv_plan *out);
void alpha_plan_deltaX(const alpha_engine_config *c, int IH, int IW, int OH, int OW, int FH, int FW, int N, int IC, int OC,
                       int sh, int sw, alpha_conv_plan *out);

/* Engine object. `stream` is the hipStream_t (as int64) every call is enqueued on; it is replicated plan.streams times
 * in the stream array handed to the natives. Argument order of the three operators follows EngineBase.java:171-199
 * (output first). Scratch is recycled in stream order (one stream per engine); alpha_engine_sync() waits for the stream. */
typedef struct alpha_engine alpha_engine;
alpha_engine *alpha_engine_create(int64_t stream);
void alpha_engine_destroy(alpha_engine *e);
alpha_engine_config *alpha_engine_get_config(alpha_engine *e);
const char *alpha_engine_last_error(alpha_engine *e);
int alpha_engine_sync(alpha_engine *e);
/* With cache_filter_transforms: the values at W (NULL = every filter) changed; their cached transforms are dropped. */
void alpha_engine_filter_changed(alpha_engine *e, const float *W);

int alpha_engine_conv3D(alpha_engine *e, float *Y, int OH, int OW, const float *X, int IH, int IW, const float *W, int FH, int FW,
                        int N, int IC, int OC, int sh, int sw, int ph, int pw, alpha_conv_plan *plan_out);
/* EngineBase.conv3D_biased (EngineBase.java:178-185; CudaFloat32EngineBase.java:1478-1560): the plan is conv3D's; the
 * bias is added in the convolution kernel's epilogue instead of by a second pass over Y. lengthv and width are the
 * reference's row-function arguments (N*OH*OW*OC and the logical OC): checked for consistency, otherwise unused. */
int alpha_engine_conv3D_biased(alpha_engine *e, float *Y, int OH, int OW, const float *X, int IH, int IW, const float *W,
                               int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                               const float *Bias, int lengthv, int width, alpha_conv_plan *plan_out);
/* conv3D, batch normalisation with given statistics and leaky ReLU as one operator (this build's addition; the reference
 * composes eg.conv3D, eg.batchNorm and eg.leakyRelu: experiments/alpha_code/src/cifar10/resnet18/Net.java:42-58). The plan
 * is conv3D's; the row functions run in the convolution kernel's epilogue where the kernel has the fused form. */
int alpha_engine_conv3D_fused(alpha_engine *e, float *Y, int OH, int OW, const float *X, int IH, int IW, const float *W,
                              int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                              const alpha_conv_epilogue *epilogue, alpha_conv_plan *plan_out);
int alpha_engine_dconv3D_deltaW(alpha_engine *e, float *deltaW, int FH, int FW, const float *X, int IH, int IW,
                                const float *deltaY, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                                alpha_conv_plan *plan_out);
/* dconv3D_deltaW followed by field_sum(deltaY, OC) (nn/unit/simple/Conv3D.java:150-162) as one operator: deltaB[OC] is
 * produced by the backward-filter kernel from the deltaY it reads anyway. */
int alpha_engine_dconv3D_deltaW_deltaB(alpha_engine *e, float *deltaW, float *deltaB, int FH, int FW, const float *X, int IH, int IW,
                                       const float *deltaY, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                                       alpha_conv_plan *plan_out);
int alpha_engine_dconv3D_deltaX(alpha_engine *e, float *deltaX, int IH, int IW, const float *deltaY, int OH, int OW,
                                const float *W, int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                                alpha_conv_plan *plan_out);

/* dconv3D_deltaX followed by the backward of the leaky ReLU (slope k) whose output Xf[N,IH,IW,IC] is this layer's input
 * (eg.leakyRelu_deltaX on the result), as one operator: the plan is dconv3D_deltaX's; the mask is applied in the kernel's
 * epilogue for the stride-1 entries and by leakyRelu2D_deltaX_v1 in place after the others. */
int alpha_engine_dconv3D_deltaX_leakyRelu(alpha_engine *e, float *deltaX, int IH, int IW, const float *deltaY, int OH, int OW,
                                          const float *W, int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                                          const float *Xf, float k, alpha_conv_plan *plan_out);

/* Backward of the batch normalisation that follows a convolution, as one operator each (field sums, then the row function):
 * EngineBase.batchNorm2D_deltaX_v1 / _v2 without A (CudaFloat32EngineBase.java:4385-4475), with A (:4478-4576), and with
 * deltaA / deltaB as further results batchNorm2D_gradients_v1 / _v2 (:4648-4760). v1 reads the layer's output Y (and B
 * when affine), v2 its input X and X_mean. A == NULL: not affine (B, deltaA, deltaB must be NULL too); deltaA and deltaB
 * go together. field_length rows of row_lengthv == stride elements, lengthv = field_length * row_lengthv. */
int alpha_engine_batchNorm2D_deltaX_v1(alpha_engine *e, float *deltaX, const float *deltaY, const float *Y, const float *X_var, float eps,
                                       const float *A, const float *B, float *deltaA, float *deltaB,
                                       int field_length, int row_lengthv, int lengthv, int width, int stride);
int alpha_engine_batchNorm2D_deltaX_v2(alpha_engine *e, float *deltaX, const float *deltaY, const float *X, const float *X_mean,
                                       const float *X_var, float eps, const float *A, float *deltaA, float *deltaB,
                                       int field_length, int row_lengthv, int lengthv, int width, int stride);

#ifdef __cplusplus
}
#endif
#endif /* ALPHA_ENGINE_H */
