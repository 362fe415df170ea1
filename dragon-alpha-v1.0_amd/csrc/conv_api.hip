// C ABI of the conv3D hot path (declared in include/alpha_conv.h): argument checks and the mapping
// of every reference entry point onto the gfx950 kernels. Everything is enqueued on streams[0];
// nothing is allocated, freed or synchronised here.
#include "../../include/alpha_conv.h"
#include "common.hpp"

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

using namespace alpha;

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_status(hipError_t e, const char *what)
{
    if (e == hipSuccess) return 0;
    return fail((int)e, "%s: %s", what, hipGetErrorString(e));
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline hipStream_t stream0(const int64_t *streams) { return reinterpret_cast<hipStream_t>((intptr_t)streams[0]); }

#define CHECK_STREAMS()                                                                    \
    do {                                                                                   \
        if (streams == nullptr || length < 1) return fail(ALPHA_CONV_EINVAL, "%s: empty stream array", __func__); \
    } while (0)

#define CHECK_PTR(p)                                                                                        \
    do {                                                                                                    \
        if ((p) == nullptr || !aligned16(p)) return fail(ALPHA_CONV_EINVAL, "%s: %s is null or not 16-byte aligned", __func__, #p); \
    } while (0)

int check_dims(const char *fn, int N, int IC, int OC, int IH, int IW, int OH, int OW, int FH, int FW, int sh, int sw, int ph, int pw)
{
    if (N < 1 || IC < 4 || OC < 4 || IH < 1 || IW < 1 || OH < 1 || OW < 1 || FH < 1 || FW < 1 || sh < 1 || sw < 1 || ph < 0 || pw < 0)
        return fail(ALPHA_CONV_EINVAL, "%s: non-positive dimension", fn);
    if ((IC & 3) || (OC & 3)) return fail(ALPHA_CONV_EINVAL, "%s: IC and OC must be multiples of 4 (got %d, %d)", fn, IC, OC);
    if ((long)N * IH * IW * IC >= (1L << 31) || (long)N * OH * OW * OC >= (1L << 31) || (long)OC * FH * FW * IC >= (1L << 31))
        return fail(ALPHA_CONV_EINVAL, "%s: tensor exceeds 2^31 elements", fn);
    // every output pixel's window must lie inside the padded input, as the engine's own check demands
    // (EngineCore.java:653-665); a smaller output than the formula's is legal there and here
    if ((long)(OH - 1) * sh + FH > (long)IH + 2 * ph || (long)(OW - 1) * sw + FW > (long)IW + 2 * pw)
        return fail(ALPHA_CONV_EINVAL, "%s: output %dx%d does not fit input %dx%d with filter %dx%d, stride %d,%d, padding %d,%d",
                    fn, OH, OW, IH, IW, FH, FW, sh, sw, ph, pw);
    return 0;
}

enum FilterLayout { FILTER_W, FILTER_CW };

// Scratch a caller lends to the calls it makes on this thread (alpha_conv_bind_workspace): per thread, so concurrent
// callers never see each other's.
thread_local float *t_workspace = nullptr;
thread_local size_t t_workspace_bytes = 0;
// Ticket words lent with it (alpha_conv_bind_tickets): zero between launches.
thread_local unsigned *t_tickets = nullptr;
thread_local int t_tickets_count = 0;

// Debugging switch (tests and comparisons force the generic kernels with it); not part of the drop-in contract. The only
// mutable process-wide setting of the library: atomic, read once per call, so a call sees one value throughout.
std::atomic<int> g_fwd_algo{-1};   // -1: not yet read from the environment

int fwd_algo()
{
    int v = g_fwd_algo.load(std::memory_order_relaxed);
    if (v < 0) {
        const char *e = getenv("ALPHA_HIP_CONV_ALGO");
        v = 0;
        if (e && !strcmp(e, "igemm")) v = 1;
        else if (e && !strcmp(e, "winograd")) v = 2;
        else if (e && !strcmp(e, "generic")) v = 3;
        else if (e && !strcmp(e, "taps")) v = 4;
        else if (e && !strcmp(e, "rows")) v = 5;
        else if (e && !strcmp(e, "direct")) v = 6;
        int expected = -1;
        if (!g_fwd_algo.compare_exchange_strong(expected, v)) v = expected;   // a setter was quicker
    }
    return v;
}

// Which 1x1 stride-1 kernel: the one without LDS (pointwise_direct.hip) re-reads the filter per group of tiles and per
// block of 64 produced channels, the filter-resident one (pointwise.hip) stages it once per compute unit.
// Measured on 32x56x56 pixels: 256 -> 64 channels 0.036 ms direct against 0.043 ms filter-resident; 64 -> 256 channels
// 0.042 against 0.035 ms, and 256 -> 1024 on 64x14x14 pixels 0.089 against 0.068 ms: the direct kernel wins where one
// block of 64 produced channels covers the output and the reduction is long. A debugging switch forces the choice
// (alpha_conv_set_pointwise_algo, or ALPHA_PW_DIRECT=0/1 in the environment, read once per process): the parity tests
// run both kernels on every shape.
std::atomic<int> g_pw_algo{-2};   // -2: not yet read from the environment, -1: by shape, 0: filter-resident, 1: without LDS

// The same kind of switch for the kernel-split kernel without LDS (direct_conv_phased.hip): whether a workgroup's
// wavefronts share every group of work items (-1: by shape; alpha_conv_set_kernel_split_sharing, or ALPHA_KS_SHARED=0/1
// in the environment, read once per process).
std::atomic<int> g_ks_sharing{-2};

int ks_sharing()
{
    int v = g_ks_sharing.load(std::memory_order_relaxed);
    if (v == -2) {
        const char *e = getenv("ALPHA_KS_SHARED");
        v = e ? (atoi(e) != 0 ? 1 : 0) : -1;
        int expected = -2;
        if (!g_ks_sharing.compare_exchange_strong(expected, v)) v = expected;   // a setter was quicker
    }
    return v;
}

int pointwise_algo()
{
    int v = g_pw_algo.load(std::memory_order_relaxed);
    if (v == -2) {
        const char *e = getenv("ALPHA_PW_DIRECT");
        v = e ? (atoi(e) != 0 ? 1 : 0) : -1;
        int expected = -2;
        if (!g_pw_algo.compare_exchange_strong(expected, v)) v = expected;   // a setter was quicker
    }
    return v;
}

bool pointwise_direct_preferred(int K, int N, long M)
{
    const int forced = pointwise_algo();
    if (forced >= 0) return forced != 0 && (K % 32) == 0;
    // its wavefronts own tiles of 16 pixels: with fewer tiles than SIMDs the kernel of direct_conv.hip, which cuts the
    // reduction among a workgroup's wavefronts, is the faster (832 -> 48 channels on 64x7x7 pixels: 0.007 against 0.019 ms)
    if ((K % 32) != 0 || M < 64L * device_cu_count()) return false;
    // long reductions into one block of 64 produced channels; 48 or fewer go to direct_conv.hip's blocks of 16, 32 or 48
    // (192 -> 16 / 32 / 48 on 64x28x28 pixels: 0.011 / 0.013 / 0.014 against 0.015 ms, 128 -> 32 on 32x56x56: 0.015 against 0.019)
    if (K >= 128) return N > 48 && N <= 64;
    // short reductions into many channels, where the output's stores are the time (backward-data of the same layers:
    // 32 -> 192 / 256 on 64x28x28 0.011 / 0.013 against 0.014 / 0.015 ms, 32 -> 512 on 256x14x14 0.023 against 0.027, 96 -> 192
    // 0.022 against 0.024; with 64 reduced channels the filter-resident kernel keeps the layer: 64 -> 256 0.019 against 0.021)
    return (K == 32 || K == 96) && N >= 128;
}

// Through direct_conv.hip (no LDS): every layer with more than one tap or a stride (every 3x3 layer of the benchmark
// configurations: 3-14 % faster than the LDS-halo kernel; small layers - a few work items per compute unit, which the
// workgroup's wavefronts share - several times: 3x3 256 -> 256 on 8x14x14 pixels 0.021 against 0.068 ms, 5x5 48 -> 128 on
// 64x7x7 0.014 against 0.103 ms, 3x3 64 -> 64 on one 56x56 image 0.007 against 0.019 ms; a strided 1x1 layer 3 % faster than
// through the filter-resident kernel), and 1x1 layers with a long reduction whose work items divide evenly enough among
// the compute units (256 -> 1024 channels on 64x14x14 pixels: 0.053 against 0.060 ms through the filter-resident kernel;
// 256 -> 64 on 32x56x56 pixels: 0.030 against 0.032 ms through pointwise_direct.hip; 64 -> 256 there: 0.036 against
// 0.031 ms through the filter-resident kernel, which keeps that shape).
// Whether a workgroup of direct_conv.hip's kernel has 16 or more items (tile of 16 pixels, block of produced channels) -
// from there on its wavefronts take whole items of their own.
bool direct_conv_whole_items(long M, int CO)
{
    const long cus = device_cu_count();
    return cus > 0 && ((M + 15) / 16 * ((CO + 63) / 64) + cus - 1) / cus >= 16;
}

bool direct_conv_preferred(int FH, int FW, int sh, int sw, long M, int AC, int CO)
{
    if (sh > 1 || sw > 1 || FH * FW > 1) return true;
    const bool ws = t_workspace != nullptr && t_workspace_bytes >= (1u << 20);
    return AC >= 256 && direct_conv_balanced(M, CO, ws);
}

// The rest of a fused epilogue as a pass of its own over a dense [pixels, C] output (kernels that add a bias only).
int epilogue_pass(const char *fn, hipStream_t s, float *Y, const Epilogue &ep, long pixels, int C)
{
    return hip_status(launch_epilogue_rows(s, Y, Y, ep, pixels * C, C, C), fn);
}

// Forward: Y = conv(X, filter). FILTER_W reads W[OC,FH,FW,IC]; FILTER_CW reads CW[FH,FW,IC,OC]. `ep` (when not NULL
// and fused) replaces `bias`: applied inside the kernel where it has the fused form, else by one more pass over Y.
int forward(const char *fn, const int64_t *streams, int length,
            const float *X, int IH, int IW, const float *F, FilterLayout layout, int FH, int FW,
            float *Y, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
            const float *bias = nullptr, const Epilogue *ep = nullptr, const float *W_too = nullptr)
{
    // W_too: the entries that take CW also receive W[OC,FH,FW,IC], the filter CW was made from (the reference's
    // conv3D_GemmR hands both on, conv/A.cu:165-170); the kernel for 4 stored channels reads its 16-byte taps in place
    const float *W_inplace = layout == FILTER_W ? F : (aligned16(W_too) ? W_too : nullptr);
    if (streams == nullptr || length < 1) return fail(ALPHA_CONV_EINVAL, "%s: empty stream array", fn);
    if (!X || !F || !Y || !aligned16(X) || !aligned16(F) || !aligned16(Y) || !aligned16(bias))
        return fail(ALPHA_CONV_EINVAL, "%s: null or misaligned pointer", fn);
    if (int e = check_dims(fn, N, IC, OC, IH, IW, OH, OW, FH, FW, sh, sw, ph, pw)) return e;
    if (ep && !ep->fused) { bias = ep->bias; ep = nullptr; }
    const int algo = fwd_algo();

    if (IC == 4 && W_inplace && (algo == 0 || algo == 6)) {
        // both operands straight from memory
        hipError_t e = launch_stem_direct(stream0(streams), X, W_inplace, Y, N, IH, IW, OH, OW, OC, FH, FW, sh, sw, ph, pw, bias, ep);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (IC == 4 && algo != 3) {
        hipError_t e = launch_stem_conv(stream0(streams), X, F, layout == FILTER_CW, Y, N, IH, IW, IC, OH, OW, OC, FH, FW, sh, sw, ph, pw, bias, ep);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (layout == FILTER_CW && (algo == 6 || (algo == 0 && direct_conv_preferred(FH, FW, sh, sw, (long)N * OH * OW, IC, OC)))) {
        // both operands straight from memory
        hipError_t e = launch_direct_conv(stream0(streams), X, F, Y, N, IH, IW, IC, OH, OW, OC, FH, FW, sh, sw, ph, pw,
                                          0, IC * OC, OC, (long)FH * FW * IC * OC, bias, ep, t_workspace, t_workspace_bytes, t_tickets, t_tickets_count);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (FH == 1 && FW == 1 && ph == 0 && pw == 0 && sh == 1 && sw == 1 && OH == IH && OW == IW && layout == FILTER_CW && algo != 3 &&
        pointwise_direct_preferred(IC, OC, (long)N * OH * OW)) {
        hipError_t e = launch_pointwise_direct(stream0(streams), X, F, Y, (long)N * OH * OW, IC, OC, bias, ep);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (FH == 1 && FW == 1 && ph == 0 && pw == 0 && algo != 3) {
        // W[OC][IC] is [N][K]; CW[IC][OC] is [K][N]; a stride only thins the input pixels that are read
        hipError_t e = launch_pointwise(stream0(streams), X, F, Y, N, IH, IW, OH, OW, sh, sw, IC, OC, layout == FILTER_CW, ep ? nullptr : bias);
        if (e == hipSuccess && ep) return epilogue_pass(fn, stream0(streams), Y, *ep, (long)N * OH * OW, OC);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (algo == 0 && layout == FILTER_CW && FH == 1 && FW == 1 && (IC >= 32 || direct_conv_whole_items((long)N * OH * OW, OC))) {
        // a 1x1 layer that none of the kernels above took (produced channels not a multiple of 64, more than 256 reduced
        // ones ...): the kernel without LDS before the LDS-halo and the generic ones (192 -> 96 channels on 64x28x28 pixels:
        // 0.023 against 0.035 ms; 832 -> 48 on 64x7x7: 0.007 against 0.019 ms; with 16 reduced channels - a single step per
        // item - only where a workgroup has whole items: 16 -> 192 backward-data on 64x28x28 0.015 against 0.020 ms through
        // the generic kernel; where all items are shared by the wavefronts the generic kernel is the faster)
        hipError_t e = launch_direct_conv(stream0(streams), X, F, Y, N, IH, IW, IC, OH, OW, OC, FH, FW, sh, sw, ph, pw,
                                          0, IC * OC, OC, (long)FH * FW * IC * OC, bias, ep, t_workspace, t_workspace_bytes, t_tickets, t_tickets_count);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (algo != 3) {
        // W[OC,FH,FW,IC] as it is: taken by the 3x3 stride-1 kernel (128-bit fragment loads; measured the same speed as
        // from CW), refused by the others, which then leaves the generic kernel
        hipError_t e = layout == FILTER_CW
            ? launch_tap_conv(stream0(streams), X, F, Y, N, IH, IW, IC, OH, OW, OC, FH, FW, ph, pw,
                              0, FW * IC * OC, IC * OC, OC, bias, sh, sw, 1, ep)
            : launch_tap_conv(stream0(streams), X, F, Y, N, IH, IW, IC, OH, OW, OC, FH, FW, ph, pw,
                              0, FW * IC, IC, 1, bias, sh, sw, FH * FW * IC, ep);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }

    GatherConvArgs a{};
    a.A = X; a.B = F; a.O = Y; a.ep = ep ? *ep : bias_epilogue(bias);
    a.CO = OC;
    a.AH = IH; a.AW = IW; a.AC = IC;
    a.sh = sh; a.sw = sw; a.ph = ph; a.pw = pw;
    a.o_off = 0; a.o_sn = OH * OW * OC; a.o_sh = OW * OC; a.o_sw = OC;
    a.b_off = 0;
    if (layout == FILTER_CW) {
        a.b_sth = FW * IC * OC; a.b_stw = IC * OC; a.b_sc = OC; a.b_sn = 1;
    } else {
        a.b_sth = FW * IC; a.b_stw = IC; a.b_sc = 1; a.b_sn = FH * FW * IC;
    }
    return hip_status(launch_gather_conv(stream0(streams), a, FH, FW, OH, OW, N), fn);
}

// Backward-data, stride 1, reading W[OC,FH,FW,IC] in place rotated by 180 degrees:
// deltaX[n,ih,iw,ic] = sum_{t_h,t_w,oc} deltaY[n, ih - (FH-1-ph) + t_h, iw - (FW-1-pw) + t_w, oc] * W[oc, FH-1-t_h, FW-1-t_w, ic]
// `ep` (NULL, or a gate epilogue): deltaX is multiplied by the derivative of the leaky ReLU that produced this layer's input.
int deltaX_s1(const char *fn, const int64_t *streams, int length,
              const float *dY, int OH, int OW, const float *W, int FH, int FW,
              float *dX, int IH, int IW, int N, int IC, int OC, int ph, int pw, const Epilogue *ep = nullptr)
{
    if (streams == nullptr || length < 1) return fail(ALPHA_CONV_EINVAL, "%s: empty stream array", fn);
    if (!dY || !W || !dX || !aligned16(dY) || !aligned16(W) || !aligned16(dX))
        return fail(ALPHA_CONV_EINVAL, "%s: null or misaligned pointer", fn);
    if (int e = check_dims(fn, N, IC, OC, IH, IW, OH, OW, FH, FW, 1, 1, ph, pw)) return e;
    if (FH - 1 - ph < 0 || FW - 1 - pw < 0) return fail(ALPHA_CONV_EINVAL, "%s: padding larger than FH-1", fn);
    const int algo = fwd_algo();

    if (algo == 6 || (algo == 0 && direct_conv_preferred(FH, FW, 1, 1, (long)N * IH * IW, OC, IC))) {
        // both operands straight from memory; W rotated by 180 degrees is read in place (input channel contiguous)
        hipError_t e = launch_direct_conv(stream0(streams), dY, W, dX, N, OH, OW, OC, IH, IW, IC, FH, FW, 1, 1, FH - 1 - ph, FW - 1 - pw,
                                          (FH * FW - 1) * IC, -IC, FH * FW * IC, (long)OC * FH * FW * IC, nullptr, ep,
                                          t_workspace, t_workspace_bytes, t_tickets, t_tickets_count);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (FH == 1 && FW == 1 && ph == 0 && pw == 0 && OH == IH && OW == IW && algo != 3 && pointwise_direct_preferred(OC, IC, (long)N * IH * IW)) {
        // deltaX[m][ic] = sum_oc deltaY[m][oc] * W[oc][ic]: W is [K][N]
        hipError_t e = launch_pointwise_direct(stream0(streams), dY, W, dX, (long)N * IH * IW, OC, IC, nullptr, ep);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (FH == 1 && FW == 1 && ph == 0 && pw == 0 && algo != 3) {
        // deltaX[m][ic] = sum_oc deltaY[m][oc] * W[oc][ic]: W is [K][N]
        hipError_t e = launch_pointwise(stream0(streams), dY, W, dX, N, IH, IW, IH, IW, 1, 1, OC, IC, 1);
        if (e == hipSuccess && ep) return epilogue_pass(fn, stream0(streams), dX, *ep, (long)N * IH * IW, IC);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (algo == 0 && FH == 1 && FW == 1 && (OC >= 32 || direct_conv_whole_items((long)N * IH * IW, IC))) {
        // a 1x1 layer that none of the kernels above took: as in forward()
        hipError_t e = launch_direct_conv(stream0(streams), dY, W, dX, N, OH, OW, OC, IH, IW, IC, FH, FW, 1, 1, FH - 1 - ph, FW - 1 - pw,
                                          (FH * FW - 1) * IC, -IC, FH * FW * IC, (long)OC * FH * FW * IC, nullptr, ep,
                                          t_workspace, t_workspace_bytes, t_tickets, t_tickets_count);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (algo != 3) {
        hipError_t e = launch_tap_conv(stream0(streams), dY, W, dX, N, OH, OW, OC, IH, IW, IC, FH, FW, FH - 1 - ph, FW - 1 - pw,
                                       ((FH - 1) * FW + (FW - 1)) * IC, -FW * IC, -IC, FH * FW * IC, nullptr, 1, 1, 1, ep);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }

    GatherConvArgs a{};
    a.A = dY; a.B = W; a.O = dX; a.ep = ep ? *ep : bias_epilogue(nullptr);
    a.CO = IC;
    a.AH = OH; a.AW = OW; a.AC = OC;
    a.sh = 1; a.sw = 1; a.ph = FH - 1 - ph; a.pw = FW - 1 - pw;
    a.o_off = 0; a.o_sn = IH * IW * IC; a.o_sh = IW * IC; a.o_sw = IC;
    a.b_off = ((FH - 1) * FW + (FW - 1)) * IC;
    a.b_sth = -FW * IC; a.b_stw = -IC; a.b_sc = FH * FW * IC; a.b_sn = 1;
    return hip_status(launch_gather_conv(stream0(streams), a, FH, FW, IH, IW, N), fn);
}

// Backward-data for any stride as sh*sw dense sub-problems ("kernel split"): phase (y, x) owns the
// taps fh = y (mod sh), fw = x (mod sw) and produces the deltaX sub-lattice ih = ihs (mod sh),
// iw = iws (mod sw). from_CW: filter taken from the v2 kernel-split layout; otherwise from W in place.
int deltaX_phases(const char *fn, const int64_t *streams, int length,
                  const float *dY, int OH, int OW, const float *F, bool from_CW, int FH, int FW,
                  float *dX, int IH, int IW, int N, int IC, int OC, int sh, int sw, int ph, int pw, const Epilogue *ep = nullptr)
{
    if (streams == nullptr || length < 1) return fail(ALPHA_CONV_EINVAL, "%s: empty stream array", fn);
    if (!dY || !F || !dX || !aligned16(dY) || !aligned16(F) || !aligned16(dX))
        return fail(ALPHA_CONV_EINVAL, "%s: null or misaligned pointer", fn);
    if (int e = check_dims(fn, N, IC, OC, IH, IW, OH, OW, FH, FW, sh, sw, ph, pw)) return e;

    const int mCFH = (FH + sh - 1) / sh, mCFW = (FW + sw - 1) / sw;
    const int CWstride = mCFH * mCFW * OC * IC;
    hipStream_t s = stream0(streams);
    if (sh * sw > 64) return fail(ALPHA_CONV_EINVAL, "%s: more than 64 phases (sh*sw)", fn);
    if (!from_CW && fwd_algo() != 3) {
        // 4 stored input channels (the gradient of a stem's input): one stride-1 convolution of deltaY into the
        // sh*sw*4 values of each sh x sw block of deltaX
        hipError_t e = launch_delta_x_stem(s, dY, F, dX, N, IH, IW, IC, OH, OW, OC, FH, FW, sh, sw, ph, pw, ep);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (FH == 1 && FW == 1 && ph == 0 && pw == 0 && sh * sw > 1 && IH == sh * OH && IW == sw * OW && !(ep && ep->fused) &&
        (fwd_algo() == 0 || fwd_algo() == 6) && (long)OC * IC < 40L * (OC + sh * sw * IC)) {
        // a 1x1 filter under a larger stride: one matrix product scattered over deltaX, zeros in between. The filter is
        // [OC][IC] in both layouts (W as it is; phase 0 of the kernel-split layout, the only one with a tap). For the layers
        // that memory bounds - fewer than 20 FLOP per byte of deltaY read and deltaX written -: its wavefronts own tiles
        // of pixels with all their channels, which is how the bytes move best and the matrix pipes work worst (14x14x1024
        // <- 7x7x2048 at N = 64: 196 tiles, 0.65 ms); with more channels the phases below take the layer.
        hipError_t e = launch_pointwise_scatter(s, dY, F, dX, N, OH, OW, OC, IC, sh, sw);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    // the phases as dense stride-1 problems
    struct Phase { GatherConvArgs a; int th, tw, OHt, OWt; };
    std::vector<Phase> phases;
    for (int y = 0; y < sh; y++)
        for (int x = 0; x < sw; x++) {
            const int CFH = (FH - y + sh - 1) / sh, CFW = (FW - x + sw - 1) / sw;
            const int phy = ph - y, pwx = pw - x;
            const int ihs = -phy + (phy > 0 ? (phy + sh - 1) / sh * sh : 0);
            const int iws = -pwx + (pwx > 0 ? (pwx + sw - 1) / sw * sw : 0);
            const int OHt = IH > ihs ? (IH - ihs + sh - 1) / sh : 0;
            const int OWt = IW > iws ? (IW - iws + sw - 1) / sw : 0;
            if (OHt == 0 || OWt == 0) continue;

            GatherConvArgs a{};
            a.A = dY; a.B = F; a.O = dX;
            a.ep = ep ? *ep : bias_epilogue(nullptr);
            a.CO = IC;
            a.AH = OH; a.AW = OW; a.AC = OC;
            a.sh = 1; a.sw = 1;
            a.ph = (CFH - 1) - (ihs + phy) / sh;
            a.pw = (CFW - 1) - (iws + pwx) / sw;
            a.o_off = (ihs * IW + iws) * IC; a.o_sn = IH * IW * IC; a.o_sh = sh * IW * IC; a.o_sw = sw * IC;
            if (from_CW) {
                a.b_off = (y * sw + x) * CWstride;
                a.b_sth = CFW * OC * IC; a.b_stw = OC * IC; a.b_sc = IC; a.b_sn = 1;
            } else {
                a.b_off = ((y + (CFH - 1) * sh) * FW + (x + (CFW - 1) * sw)) * IC;
                a.b_sth = -sh * FW * IC; a.b_stw = -sw * IC; a.b_sc = FH * FW * IC; a.b_sn = 1;
            }
            const int th = CFH > 0 && CFW > 0 ? CFH : 0, tw = CFH > 0 && CFW > 0 ? CFW : 0;
            if (th == 0) a.b_off = 0;
            phases.push_back(Phase{a, th, tw, OHt, OWt});
        }
    // Up to four phases of the same size (IH % sh == 0, IW % sw == 0: the reference's Ims case): ONE launch of the kernel
    // without LDS, every wavefront running all phases on its tiles of coarse pixels.
    const int algo = fwd_algo();
    if ((algo == 0 || algo == 6) && sh * sw <= 4 && IH % sh == 0 && IW % sw == 0 && (int)phases.size() == sh * sw) {
        int TH[4], TW[4], pph[4], ppw[4], boff[4], bsth[4], ooff[4];
        bool same = true;
        for (int f = 0; f < sh * sw; f++) {
            const GatherConvArgs &a = phases[f].a;
            TH[f] = phases[f].th; TW[f] = phases[f].tw; pph[f] = a.ph; ppw[f] = a.pw; boff[f] = a.b_off; bsth[f] = a.b_sth; ooff[f] = a.o_off;
            same = same && phases[f].OHt == phases[0].OHt && phases[f].OWt == phases[0].OWt;
        }
        if (same) {
            const GatherConvArgs &a0 = phases[0].a;
            const long b_elems = from_CW ? (long)sh * sw * CWstride : (long)OC * FH * FW * IC;
            hipError_t e = launch_direct_conv_phased(s, dY, F, dX, N, OH, OW, OC, IC, phases[0].OHt, phases[0].OWt, sh * sw, TH, TW, pph, ppw,
                                                     boff, bsth, a0.b_stw, a0.b_sc, b_elems, ooff, a0.o_sn, a0.o_sh, a0.o_sw,
                                                     (long)N * IH * IW * IC, ep, ks_sharing());
            if (e != hipErrorNotSupported) return hip_status(e, fn);
        }
    }
    // Stride 2 x 2 with even sizes (the reference's Ims2 case): the four phases in ONE launch, sharing one LDS halo per
    // unit (the reference runs its phases in one grid too: dconv3D_dX_kernelSplit_Ims2R_kernel.cuh:18, dim3(.., .., 4)).
    // Everything else, and whatever that kernel refuses: one launch of the generic kernel per phase.
    if (algo != 3 && sh == 2 && sw == 2 && (IH & 1) == 0 && (IW & 1) == 0 && phases.size() == 4) {
        int TH[4], TW[4], pph[4], ppw[4], boff[4], bsth[4], ooff[4];
        for (int f = 0; f < 4; f++) {
            const GatherConvArgs &a = phases[f].a;
            TH[f] = phases[f].th; TW[f] = phases[f].tw; pph[f] = a.ph; ppw[f] = a.pw; boff[f] = a.b_off; bsth[f] = a.b_sth; ooff[f] = a.o_off;
        }
        const GatherConvArgs &a0 = phases[0].a;
        hipError_t e = launch_tap_conv_merged(s, dY, F, dX, N, OH, OW, OC, IC, phases[0].OHt, phases[0].OWt, TH, TW, pph, ppw, boff, bsth,
                                              a0.b_stw, a0.b_sc, ooff, a0.o_sn, a0.o_sh, a0.o_sw, ep);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    for (const Phase &f : phases)
        if (int e = hip_status(launch_gather_conv(s, f.a, f.th, f.tw, f.OHt, f.OWt, N), fn)) return e;
    return 0;
}

int deltaW_impl(const char *fn, const int64_t *streams, int length, int GridZ,
           const float *X, int IH, int IW, const float *dY, int OH, int OW,
           float *dW, float *dW_buf, int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
           float *dB = nullptr, float *dB_buf = nullptr)
{
    if (streams == nullptr || length < 1) return fail(ALPHA_CONV_EINVAL, "%s: empty stream array", fn);
    if (!X || !dY || !dW || !aligned16(X) || !aligned16(dY) || !aligned16(dW) || !aligned16(dB) || !aligned16(dB_buf))
        return fail(ALPHA_CONV_EINVAL, "%s: null or misaligned pointer", fn);
    if (GridZ < 1) return fail(ALPHA_CONV_EINVAL, "%s: GridZ must be >= 1", fn);
    if (GridZ > 1 && (!dW_buf || !aligned16(dW_buf))) return fail(ALPHA_CONV_EINVAL, "%s: deltaW_buf is null or misaligned", fn);
    if (dB && GridZ > 1 && !dB_buf) return fail(ALPHA_CONV_EINVAL, "%s: deltaB_buf is null", fn);
    if (int e = check_dims(fn, N, IC, OC, IH, IW, OH, OW, FH, FW, sh, sw, ph, pw)) return e;

    DeltaWArgs a{};
    a.X = X; a.dY = dY; a.dW = dW; a.dW_buf = dW_buf;
    a.IH = IH; a.IW = IW; a.IC = IC; a.OH = OH; a.OW = OW; a.OC = OC; a.FW = FW;
    a.sh = sh; a.sw = sw; a.ph = ph; a.pw = pw;
    a.GM = FH * FW * IC;
    a.GK = N * OH * OW;
    a.GZ = GridZ;
    a.GK_slice = (a.GK / GridZ) >> 3 << 3;
    const int algo = fwd_algo();
    // Which kernel (all but the first two share the slice partition and the outputs):
    //  - 4 stored input channels, GridZ of 2 or more: the kernel of delta_w_stem.hip (its own equal cut of the pixels);
    //  - layers whose channel counts fill 64 x 64 blocks well enough (below), GridZ of 2 or more: the persistent kernel of
    //    delta_w_stream.hip (its own partition of the pixels among deltaW and the buffers; a bias gradient takes a pass of
    //    its own over deltaY then, so layers where another kernel produces it on the way stay with that kernel);
    //  - 1x1 stride 1 with channel counts in multiples of 64: the register kernel of delta_w_pointwise.hip;
    //  - layers whose channel counts fill the 64 x 64 blocks of the tap-per-workgroup kernel to 75 % or more: that kernel
    //    (any filter, stride and padding); the bias gradient, when asked for, then takes a pass of its own over deltaY -
    //    unless the row-streaming kernel, which produces it on the way, would fill the device anyway;
    //  - other stride-1 3x3 / 1x1 layers: the row-streaming kernel; whatever is left: the generic kernel.
    // algo 3 forces the generic kernel, 4 the tap-per-workgroup kernel wherever it fits, 5 the row-streaming kernel
    // wherever it fits (comparisons and tests).
    const bool w1 = FH == 1 && FW == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0;
    const long icb = (IC + 63) / 64, ocb = (OC + 63) / 64;
    const bool blocks_filled = 4L * IC * OC >= 3L * icb * 64 * ocb * 64;
    // what the persistent kernel needs of its blocks (64 x 64 channels, or 16 x 1 to 3 channels per lane on either side
    // where that holds the channels in as many blocks: 96 = 2 x 48, 32 = 1 x 32) to win: 40 % where the row-streaming kernel is the alternative
    // (96 -> 208 channels 3x3: 0.066 against 0.103 ms; 32 -> 32: 0.107 against 0.074), 15 % where the generic kernel is
    // (5x5, 16 -> 48: 0.026 against 0.043 ms; 16 -> 32: 0.078 against 0.047)
    const bool rows_shape = sh == 1 && sw == 1 && ((FH == 3 && FW == 3) || (FH == 1 && FW == 1));
    const bool stream_filled = deltaW_stream_block_fill(IC, OC) >= (rows_shape ? 40 : 15);
    const bool rows_fill = sh == 1 && sw == 1 && ((FH == 3 && FW == 3) || (FH == 1 && FW == 1)) && icb * ((OC + 31) / 32) * GridZ >= 2L * device_cu_count();
    if (algo == 0 && IC == 4 && GridZ >= 2) {
        // 4 stored input channels (a network's first layer): the 16 columns of an MFMA operand are 16 taps
        hipError_t e = launch_deltaW_stem(stream0(streams), X, dY, dW, dW_buf, N, IH, IW, OH, OW, OC, FH, FW, sh, sw, ph, pw, GridZ);
        if (e == hipSuccess && dB) e = launch_col_sum(stream0(streams), dY, dB, dB_buf, OC, a.GK, a.GK_slice, GridZ);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (algo == 0 && stream_filled && !(dB && (rows_fill || w1))) {
        // the same arithmetic with the reduction dealt out evenly (its own partition of the pixels among the buffers)
        hipError_t e = launch_deltaW_stream(stream0(streams), X, dY, dW, dW_buf, N, IH, IW, IC, OH, OW, OC, FH, FW, sh, sw, ph, pw, GridZ);
        if (e == hipSuccess && dB) e = launch_col_sum(stream0(streams), dY, dB, dB_buf, OC, a.GK, a.GK_slice, GridZ);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (algo != 3 && algo != 4 && algo != 5 && w1) {
        hipError_t e = launch_deltaW_pointwise(stream0(streams), X, dY, dW, dW_buf, a.GK, IC, OC, a.GK_slice, GridZ, dB, dB_buf);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (algo == 4 || (algo != 3 && algo != 5 && blocks_filled && !(dB && rows_fill))) {
        hipError_t e = launch_deltaW_taps(stream0(streams), X, dY, dW, dW_buf, N, IH, IW, IC, OH, OW, OC, FH, FW, sh, sw, ph, pw, a.GK_slice, GridZ);
        if (e == hipSuccess && dB) e = launch_col_sum(stream0(streams), dY, dB, dB_buf, OC, a.GK, a.GK_slice, GridZ);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    if (algo != 3) {
        hipError_t e = launch_deltaW_rows(stream0(streams), X, dY, dW, dW_buf, N, IH, IW, IC, OH, OW, OC, FH, FW, sh, sw, ph, pw,
                                          a.GK_slice, GridZ, dB, dB_buf);
        if (e != hipErrorNotSupported) return hip_status(e, fn);
    }
    // the generic kernel has no bias-gradient path: the column sums of deltaY get a pass of their own
    if (dB)
        if (int e = hip_status(launch_col_sum(stream0(streams), dY, dB, dB_buf, OC, a.GK, a.GK_slice, GridZ), fn)) return e;
    return hip_status(launch_deltaW(stream0(streams), a), fn);
}

// ---- split-K partial sums in device memory that belongs to the library ---------------------------------------------
// For callers that cannot allocate (HIP graph capture, serving loops, harnesses that forbid hipMalloc): the partial
// sums of alpha_dconv3D_deltaW_GemmSK_static live in this file-scope array instead of a deltaW_buf from the caller.
// Every device that loads the library holds its own copy until the process ends. In host code the array's name is
// only a handle: its device address is asked for once per device (with that device current) and kept here.
constexpr size_t STATIC_SCRATCH_FLOATS = ALPHA_CONV_STATIC_SCRATCH_BYTES / sizeof(float);
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];

constexpr int MAX_DEVICES = 64;
std::atomic<float *> g_scratch_ptr[MAX_DEVICES];
std::atomic<unsigned> g_scratch_generation{0};   // device_generation() the addresses above were asked in

// Device address of `scratch` on the current device, or nullptr with the error recorded.
float *static_scratch(const char *fn)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { hip_status(e, fn); return nullptr; }
    if (dev < 0 || dev >= MAX_DEVICES) { fail(ALPHA_CONV_EINVAL, "%s: device index %d out of range", fn, dev); return nullptr; }
    const unsigned gen = device_generation().load(std::memory_order_acquire);
    if (g_scratch_generation.load(std::memory_order_acquire) != gen) {   // a device was reset: ask again
        for (auto &q : g_scratch_ptr) q.store(nullptr, std::memory_order_release);
        g_scratch_generation.store(gen, std::memory_order_release);
    }
    float *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {   // a racing first call asks twice and stores the same address
        void *sym = nullptr;
        e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
        if (e != hipSuccess || sym == nullptr) {
            fail(e != hipSuccess ? (int)e : ALPHA_CONV_EINVAL, "%s: hipGetSymbolAddress(scratch): %s", fn, hipGetErrorString(e));
            return nullptr;
        }
        ptr = static_cast<float *>(sym);
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    return ptr;
}

}  // namespace

#pragma GCC visibility push(default)
extern "C" {

const char *alpha_conv_version(void) { return "alpha-conv-hip gfx950 0.1"; }
const char *alpha_conv_last_error(void) { return g_err; }

int alpha_conv_device_info(int *compute_units, int *clock_khz)
{
    int dev = 0, cu = 0, clk = 0;
    if (int e = hip_status(hipGetDevice(&dev), __func__)) return e;
    if (int e = hip_status(hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev), __func__)) return e;
    if (int e = hip_status(hipDeviceGetAttribute(&clk, hipDeviceAttributeClockRate, dev), __func__)) return e;
    if (compute_units) *compute_units = cu;
    if (clock_khz) *clock_khz = clk;
    // the per-device set-up call of the library: also resolves this device's copy of the static scratch array, so that a
    // caller who asks for the device first never triggers that lookup inside a captured region
    if (static_scratch(__func__) == nullptr) return ALPHA_CONV_EINVAL;
    return 0;
}

int alpha_conv_bind_workspace(float *workspace, long bytes)
{
    if (workspace != nullptr && (!aligned16(workspace) || bytes < 0))
        return fail(ALPHA_CONV_EINVAL, "alpha_conv_bind_workspace: misaligned workspace or negative size");
    t_workspace = workspace;
    t_workspace_bytes = workspace ? (size_t)bytes : 0;
    return 0;
}

int alpha_conv_bind_tickets(unsigned *tickets, int count)
{
    if (count < 0 || (tickets != nullptr && (reinterpret_cast<uintptr_t>(tickets) & 3) != 0))
        return fail(ALPHA_CONV_EINVAL, "alpha_conv_bind_tickets: misaligned words or negative count");
    t_tickets = tickets;
    t_tickets_count = tickets ? count : 0;
    return 0;
}
int alpha_conv_get_fwd_algo(void) { return fwd_algo(); }
int alpha_conv_set_pointwise_algo(int algo)
{
    if (algo < -1 || algo > 1) return fail(ALPHA_CONV_EINVAL, "alpha_conv_set_pointwise_algo: algo must be -1, 0 or 1");
    g_pw_algo.store(algo);
    return 0;
}
int alpha_conv_set_kernel_split_sharing(int sharing)
{
    if (sharing < -1 || sharing > 1) return fail(ALPHA_CONV_EINVAL, "alpha_conv_set_kernel_split_sharing: sharing must be -1, 0 or 1");
    g_ks_sharing.store(sharing);
    return 0;
}
int alpha_conv_set_deltaW_units(int units)
{
    if (units < -1 || units > 1) return fail(ALPHA_CONV_EINVAL, "alpha_conv_set_deltaW_units: units must be -1, 0 or 1");
    deltaW_stream_set_units(units);
    return 0;
}
int alpha_conv_set_fwd_algo(int algo)
{
    if (algo < 0 || algo > 6) return fail(ALPHA_CONV_EINVAL, "alpha_conv_set_fwd_algo: algo must be 0..6");
    g_fwd_algo.store(algo);
    return 0;
}

// ---- forward -------------------------------------------------------------------------------
int alpha_conv3D(const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, int FH, int FW,
                 float *Y, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    return forward(__func__, streams, length, X, IH, IW, W, FILTER_W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw);
}
int alpha_conv3D_texture(const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, int FH, int FW,
                         float *Y, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    return forward(__func__, streams, length, X, IH, IW, W, FILTER_W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw);
}
int alpha_conv3DV2(int useTexture, const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, int FH, int FW,
                   float *Y, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    (void)useTexture;
    return forward(__func__, streams, length, X, IH, IW, W, FILTER_W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw);
}
int alpha_conv3D_np(const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, int FH, int FW,
                    float *Y, int OH, int OW, int N, int IC, int OC, int sh, int sw)
{
    return forward(__func__, streams, length, X, IH, IW, W, FILTER_W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, 0, 0);
}
int alpha_conv3D_W1(const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, float *Y,
                    int N, int IC, int OC)
{
    return forward(__func__, streams, length, X, IH, IW, W, FILTER_W, 1, 1, Y, IH, IW, N, IC, OC, 1, 1, 0, 0);
}
int alpha_kernel_remode(int64_t stream, const float *W, float *CW, int FH, int FW, int OC, int IC)
{
    CHECK_PTR(W);
    CHECK_PTR(CW);
    if (FH < 1 || FW < 1 || OC < 4 || IC < 4 || (OC & 3) || (IC & 3))
        return fail(ALPHA_CONV_EINVAL, "%s: bad filter dims", __func__);
    return hip_status(launch_kernel_remode(reinterpret_cast<hipStream_t>((intptr_t)stream), W, CW, FH, FW, OC, IC), __func__);
}
int alpha_conv3D_GemmR(const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, const float *CW,
                       int FH, int FW, float *Y, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    return forward(__func__, streams, length, X, IH, IW, CW, FILTER_CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw, nullptr, nullptr, W);
}
int alpha_conv3D_GemmR_texture(const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, const float *CW,
                               int FH, int FW, float *Y, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    return forward(__func__, streams, length, X, IH, IW, CW, FILTER_CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw, nullptr, nullptr, W);
}
int alpha_conv3D_GemmV2R(int useTexture, const int64_t *streams, int length, const float *X, int IH, int IW, const float *W,
                         const float *CW, int FH, int FW, float *Y, int OH, int OW, int N, int IC, int OC,
                         int sh, int sw, int ph, int pw)
{
    (void)useTexture;
    return forward(__func__, streams, length, X, IH, IW, CW, FILTER_CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw, nullptr, nullptr, W);
}
int alpha_conv3D_GemmR_W1(const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, const float *CW,
                          float *Y, int N, int IC, int OC)
{
    return forward(__func__, streams, length, X, IH, IW, CW, FILTER_CW, 1, 1, Y, IH, IW, N, IC, OC, 1, 1, 0, 0, nullptr, nullptr, W);
}

// ---- backward-data ---------------------------------------------------------------------------
int alpha_dconv3D_deltaX_s1(const int64_t *streams, int length, const float *deltaY, int OH, int OW, const float *W, int FH, int FW,
                            float *deltaX, int IH, int IW, int N, int IC, int OC, int ph, int pw)
{
    return deltaX_s1(__func__, streams, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw);
}
int alpha_dconv3D_deltaX_s1_texture(const int64_t *streams, int length, const float *deltaY, int OH, int OW, const float *W,
                                    int FH, int FW, float *deltaX, int IH, int IW, int N, int IC, int OC, int ph, int pw)
{
    return deltaX_s1(__func__, streams, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw);
}
int alpha_dconv3D_deltaX_V2_s1(int useTexture, const int64_t *streams, int length, const float *deltaY, int OH, int OW,
                               const float *W, int FH, int FW, float *deltaX, int IH, int IW, int N, int IC, int OC, int ph, int pw)
{
    (void)useTexture;
    return deltaX_s1(__func__, streams, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw);
}
int alpha_dconv3D_deltaX_W1(const int64_t *streams, int length, const float *deltaY, const float *W, float *deltaX,
                            int IH, int IW, int N, int IC, int OC)
{
    return deltaX_s1(__func__, streams, length, deltaY, IH, IW, W, 1, 1, deltaX, IH, IW, N, IC, OC, 0, 0);
}
int alpha_ks_remode(int64_t stream, const float *W, int FH, int FW, float *CW, int CFH, int CFW, int OC, int IC, int sh, int sw)
{
    CHECK_PTR(W);
    CHECK_PTR(CW);
    if (FH < 1 || FW < 1 || OC < 4 || IC < 4 || (OC & 3) || (IC & 3) || sh < 1 || sw < 1 || CFH != (FH + sh - 1) / sh || CFW != (FW + sw - 1) / sw)
        return fail(ALPHA_CONV_EINVAL, "%s: bad filter dims", __func__);
    return hip_status(launch_ks_remode(reinterpret_cast<hipStream_t>((intptr_t)stream), 1, W, FH, FW, CW, CFH, CFW, OC, IC, sh, sw), __func__);
}
int alpha_ks_remodev2(int64_t stream, const float *W, int FH, int FW, float *CW, int CFH, int CFW, int OC, int IC, int sh, int sw)
{
    CHECK_PTR(W);
    CHECK_PTR(CW);
    if (FH < 1 || FW < 1 || OC < 4 || IC < 4 || (OC & 3) || (IC & 3) || sh < 1 || sw < 1 || CFH != (FH + sh - 1) / sh || CFW != (FW + sw - 1) / sw)
        return fail(ALPHA_CONV_EINVAL, "%s: bad filter dims", __func__);
    return hip_status(launch_ks_remode(reinterpret_cast<hipStream_t>((intptr_t)stream), 2, W, FH, FW, CW, CFH, CFW, OC, IC, sh, sw), __func__);
}
int alpha_dconv3D_deltaX_kernelSplit(const int64_t *streams, int length, const float *deltaY, int OH, int OW, const float *CW,
                                     int FH, int FW, float *deltaX, int IH, int IW, int N, int IC, int OC,
                                     int sh, int sw, int ph, int pw)
{
    return deltaX_phases(__func__, streams, length, deltaY, OH, OW, CW, true, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw);
}
int alpha_dconv3D_deltaX_ksImsR(const int64_t *streams, int length, const float *deltaY, int OH, int OW, const float *CW,
                                int FH, int FW, float *deltaX, int IH, int IW, int N, int IC, int OC,
                                int sh, int sw, int ph, int pw)
{
    return deltaX_phases(__func__, streams, length, deltaY, OH, OW, CW, true, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw);
}
int alpha_dconv3D_deltaX_ksImsR_texture(const int64_t *streams, int length, const float *deltaY, int OH, int OW, const float *CW,
                                        int FH, int FW, float *deltaX, int IH, int IW, int N, int IC, int OC,
                                        int sh, int sw, int ph, int pw)
{
    return deltaX_phases(__func__, streams, length, deltaY, OH, OW, CW, true, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw);
}
int alpha_dconv3D_deltaX_ksIms2R(const int64_t *streams, int length, const float *deltaY, int OH, int OW, const float *CW,
                                 int FH, int FW, float *deltaX, int IH, int IW, int N, int IC, int OC, int ph, int pw)
{
    return deltaX_phases(__func__, streams, length, deltaY, OH, OW, CW, true, FH, FW, deltaX, IH, IW, N, IC, OC, 2, 2, ph, pw);
}
int alpha_dconv3D_deltaX_ksIms2R_texture(const int64_t *streams, int length, const float *deltaY, int OH, int OW, const float *CW,
                                         int FH, int FW, float *deltaX, int IH, int IW, int N, int IC, int OC, int ph, int pw)
{
    return deltaX_phases(__func__, streams, length, deltaY, OH, OW, CW, true, FH, FW, deltaX, IH, IW, N, IC, OC, 2, 2, ph, pw);
}
int alpha_dconv3D_deltaX_ksV2_Ims2R(int useTexture, const int64_t *streams, int length, const float *deltaY, int OH, int OW,
                                    const float *CW, int FH, int FW, float *deltaX, int IH, int IW, int N, int IC, int OC,
                                    int ph, int pw)
{
    (void)useTexture;
    return deltaX_phases(__func__, streams, length, deltaY, OH, OW, CW, true, FH, FW, deltaX, IH, IW, N, IC, OC, 2, 2, ph, pw);
}
int alpha_dconv3D_deltaX_crossAdd(const int64_t *streams, int length, const float *deltaY, int OH, int OW, const float *W,
                                  int FH, int FW, float *deltaX, int IH, int IW, int N, int IC, int OC,
                                  int sh, int sw, int ph, int pw)
{
    return deltaX_phases(__func__, streams, length, deltaY, OH, OW, W, false, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw);
}

// ---- backward-filter ----------------------------------------------------------------------------
int alpha_dconv3D_deltaW(const int64_t *streams, int length, const float *X, int IH, int IW, const float *deltaY, int OH, int OW,
                         float *deltaW, int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    return deltaW_impl(__func__, streams, length, 1, X, IH, IW, deltaY, OH, OW, deltaW, nullptr, FH, FW, N, IC, OC, sh, sw, ph, pw);
}
int alpha_dconv3D_deltaW_W1(const int64_t *streams, int length, const float *X, int IH, int IW, const float *deltaY,
                            float *deltaW, int N, int IC, int OC)
{
    return deltaW_impl(__func__, streams, length, 1, X, IH, IW, deltaY, IH, IW, deltaW, nullptr, 1, 1, N, IC, OC, 1, 1, 0, 0);
}
int alpha_buf_summary(int64_t stream, const float *deltaW_buf, float *deltaW, int part, int sizeW)
{
    CHECK_PTR(deltaW);
    if (part < 0 || sizeW < 1) return fail(ALPHA_CONV_EINVAL, "%s: bad part/sizeW", __func__);
    if (part == 0) return 0;
    CHECK_PTR(deltaW_buf);
    return hip_status(launch_buf_summary(reinterpret_cast<hipStream_t>((intptr_t)stream), deltaW_buf, deltaW, part, sizeW), __func__);
}
int alpha_dconv3D_deltaW_GemmSK(const int64_t *streams, int length, int GridZ, const float *X, int IH, int IW,
                                const float *deltaY, int OH, int OW, float *deltaW, float *deltaW_buf, int FH, int FW,
                                int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    return deltaW_impl(__func__, streams, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, deltaW_buf, FH, FW, N, IC, OC, sh, sw, ph, pw);
}
int alpha_dconv3D_deltaW_GemmV2SK(const int64_t *streams, int length, int GridZ, const float *X, int IH, int IW,
                                  const float *deltaY, int OH, int OW, float *deltaW, float *deltaW_buf, int FH, int FW,
                                  int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    return deltaW_impl(__func__, streams, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, deltaW_buf, FH, FW, N, IC, OC, sh, sw, ph, pw);
}
int alpha_dconv3D_deltaW_GemmSK_W1(const int64_t *streams, int length, int GridZ, const float *X, int IH, int IW,
                                   const float *deltaY, float *deltaW, float *deltaW_buf, int N, int IC, int OC)
{
    return deltaW_impl(__func__, streams, length, GridZ, X, IH, IW, deltaY, IH, IW, deltaW, deltaW_buf, 1, 1, N, IC, OC, 1, 1, 0, 0);
}

// Split-K backward-filter that allocates nothing and takes no workspace: the GridZ - 1 partial results go to the
// library's static array, and the Kahan sum over them (buf_summary) is enqueued behind the split-K kernel on streams[0],
// so deltaW is complete when the stream reaches the end of this call's work. Same kernels, slices and summation order as
// alpha_dconv3D_deltaW_GemmSK followed by alpha_buf_summary: the results are bit-identical to that pair.
// Every slice's kernel overwrites its whole partial tensor (empty slices write zeros), so nothing of an earlier call
// is read. All calls on one device share the array: two calls whose work overlaps in time on one device race.
int alpha_dconv3D_deltaW_least_GridZ(int units, int GridZ, int OH, int OW, int FH, int FW, int N, int IC, int OC)
{
    return deltaW_stream_least_GridZ(units, N, OH, OW, IC, OC, FH, FW, GridZ);
}

int alpha_dconv3D_deltaW_GemmSK_static(const int64_t *streams, int length, int GridZ, const float *X, int IH, int IW,
                                       const float *deltaY, int OH, int OW, float *deltaW, int FH, int FW,
                                       int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    CHECK_STREAMS();
    if (GridZ < 1) return fail(ALPHA_CONV_EINVAL, "%s: GridZ must be >= 1", __func__);
    if (int e = check_dims(__func__, N, IC, OC, IH, IW, OH, OW, FH, FW, sh, sw, ph, pw)) return e;
    const size_t sizeW = (size_t)OC * FH * FW * IC, need = (size_t)(GridZ - 1) * sizeW;
    if (need > STATIC_SCRATCH_FLOATS)
        return fail(ALPHA_CONV_EINVAL, "%s: (GridZ - 1) * OC*FH*FW*IC = %zu floats of partial sums exceed the static scratch of %zu floats; "
                                       "lower GridZ or use alpha_dconv3D_deltaW_GemmSK with a deltaW_buf", __func__, need, STATIC_SCRATCH_FLOATS);
    float *buf = static_scratch(__func__);
    if (buf == nullptr) return ALPHA_CONV_EINVAL;
    if (int e = deltaW_impl(__func__, streams, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, buf, FH, FW, N, IC, OC, sh, sw, ph, pw))
        return e;
    if (GridZ == 1) return 0;
    return hip_status(launch_buf_summary(stream0(streams), buf, deltaW, GridZ - 1, (int)sizeW), __func__);
}

// ---- Winograd F(2x2,3x3): additional forward algorithm of this build ----------------------------------------
long alpha_winograd_filter_size(int IC, int OC) { return 16L * IC * OC; }
int alpha_winograd_filter_transform(int64_t stream, const float *W, float *U, int IC, int OC)
{
    CHECK_PTR(W);
    CHECK_PTR(U);
    if (IC < 4 || OC < 4 || (IC & 3) || (OC & 3)) return fail(ALPHA_CONV_EINVAL, "%s: IC and OC must be multiples of 4", __func__);
    return hip_status(launch_winograd_filter(reinterpret_cast<hipStream_t>((intptr_t)stream), W, U, IC, OC), __func__);
}
int alpha_conv3D_winograd(const int64_t *streams, int length, const float *X, int IH, int IW, const float *U, float *Y,
                          int OH, int OW, int N, int IC, int OC, int ph, int pw)
{
    CHECK_STREAMS();
    CHECK_PTR(X);
    CHECK_PTR(U);
    CHECK_PTR(Y);
    if (int e = check_dims(__func__, N, IC, OC, IH, IW, OH, OW, 3, 3, 1, 1, ph, pw)) return e;
    hipError_t e = launch_winograd(stream0(streams), X, U, Y, N, IH, IW, IC, OH, OW, OC, ph, pw);
    if (e == hipErrorNotSupported) return fail(ALPHA_CONV_EINVAL, "%s: needs OH = IH + 2*ph - 2, OW = IW + 2*pw - 2", __func__);
    return hip_status(e, __func__);
}

// Backward-data of a 3x3 stride-1 layer is a forward convolution of deltaY (OC channels in, IC out, padding 2 - p, taps
// rotated): the same Winograd kernels compute it from a filter transformed accordingly.
int alpha_winograd_filter_transform_deltaX(int64_t stream, const float *W, float *U, int IC, int OC)
{
    CHECK_PTR(W);
    CHECK_PTR(U);
    if (IC < 4 || OC < 4 || (IC & 3) || (OC & 3)) return fail(ALPHA_CONV_EINVAL, "%s: IC and OC must be multiples of 4", __func__);
    return hip_status(launch_winograd_filter(reinterpret_cast<hipStream_t>((intptr_t)stream), W, U, IC, OC, true), __func__);
}
int alpha_dconv3D_deltaX_winograd(const int64_t *streams, int length, const float *deltaY, int OH, int OW, const float *U,
                                  float *deltaX, int IH, int IW, int N, int IC, int OC, int ph, int pw)
{
    CHECK_STREAMS();
    CHECK_PTR(deltaY);
    CHECK_PTR(U);
    CHECK_PTR(deltaX);
    if (int e = check_dims(__func__, N, IC, OC, IH, IW, OH, OW, 3, 3, 1, 1, ph, pw)) return e;
    if (ph > 2 || pw > 2) return fail(ALPHA_CONV_EINVAL, "%s: padding must be at most 2", __func__);
    hipError_t e = launch_winograd(stream0(streams), deltaY, U, deltaX, N, OH, OW, OC, IH, IW, IC, 2 - ph, 2 - pw);
    if (e == hipErrorNotSupported) return fail(ALPHA_CONV_EINVAL, "%s: needs OH = IH + 2*ph - 2, OW = IW + 2*pw - 2", __func__);
    return hip_status(e, __func__);
}

// Backward-filter of a 3x3 stride-1 layer by Winograd F(3x3,2x2): the split-K contract of dconv3D_deltaW_GemmSK (slice z ->
// deltaW or deltaW_buf[z-1], buf_summary finishes), the slices being ranges of 2x2 output tiles.
int alpha_dconv3D_deltaW_GemmSK_winograd(const int64_t *streams, int length, int GridZ, const float *X, int IH, int IW,
                                         const float *deltaY, int OH, int OW, float *deltaW, float *deltaW_buf,
                                         int N, int IC, int OC, int ph, int pw)
{
    CHECK_STREAMS();
    CHECK_PTR(X);
    CHECK_PTR(deltaY);
    CHECK_PTR(deltaW);
    if (GridZ < 1) return fail(ALPHA_CONV_EINVAL, "%s: GridZ must be >= 1", __func__);
    if (GridZ > 1 && (!deltaW_buf || !aligned16(deltaW_buf))) return fail(ALPHA_CONV_EINVAL, "%s: deltaW_buf is null or misaligned", __func__);
    if (int e = check_dims(__func__, N, IC, OC, IH, IW, OH, OW, 3, 3, 1, 1, ph, pw)) return e;
    hipError_t e = launch_deltaW_winograd(stream0(streams), X, deltaY, deltaW, deltaW_buf, N, IH, IW, IC, OH, OW, OC, ph, pw, GridZ);
    if (e == hipErrorNotSupported) return fail(ALPHA_CONV_EINVAL, "%s: needs a 3x3 stride-1 layer with tensors below 2 GB", __func__);
    return hip_status(e, __func__);
}

// ---- backward-filter with the bias gradient (column sums of deltaY) from the same pass over deltaY -------------------
int alpha_dconv3D_deltaW_GemmSK_deltaB(const int64_t *streams, int length, int GridZ, const float *X, int IH, int IW,
                                       const float *deltaY, int OH, int OW, float *deltaW, float *deltaW_buf,
                                       float *deltaB, float *deltaB_buf, int FH, int FW, int N, int IC, int OC,
                                       int sh, int sw, int ph, int pw)
{
    CHECK_PTR(deltaB);
    return deltaW_impl(__func__, streams, length, GridZ, X, IH, IW, deltaY, OH, OW, deltaW, deltaW_buf, FH, FW, N, IC, OC,
                       sh, sw, ph, pw, deltaB, deltaB_buf);
}

// ---- forward with the bias added in the kernel epilogue -------------------------------------------------------------
int alpha_conv3D_biased(const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, int FH, int FW,
                        const float *Bias, float *Y, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    CHECK_PTR(Bias);
    return forward(__func__, streams, length, X, IH, IW, W, FILTER_W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw, Bias);
}
int alpha_conv3D_GemmR_biased(const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, const float *CW,
                              int FH, int FW, const float *Bias, float *Y, int OH, int OW, int N, int IC, int OC,
                              int sh, int sw, int ph, int pw)
{
    CHECK_PTR(Bias);
    return forward(__func__, streams, length, X, IH, IW, CW, FILTER_CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw, Bias, nullptr, W);
}
int alpha_conv3D_winograd_biased(const int64_t *streams, int length, const float *X, int IH, int IW, const float *U,
                                 const float *Bias, float *Y, int OH, int OW, int N, int IC, int OC, int ph, int pw)
{
    CHECK_STREAMS();
    CHECK_PTR(X);
    CHECK_PTR(U);
    CHECK_PTR(Bias);
    CHECK_PTR(Y);
    if (int e = check_dims(__func__, N, IC, OC, IH, IW, OH, OW, 3, 3, 1, 1, ph, pw)) return e;
    hipError_t e = launch_winograd(stream0(streams), X, U, Y, N, IH, IW, IC, OH, OW, OC, ph, pw, Bias);
    if (e == hipErrorNotSupported) return fail(ALPHA_CONV_EINVAL, "%s: needs OH = IH + 2*ph - 2, OW = IW + 2*pw - 2", __func__);
    return hip_status(e, __func__);
}

// ---- fused epilogues: batch normalisation and leaky ReLU around the convolution ---------------------------------------
namespace {
// The C-ABI epilogue as the kernels' Epilogue; 0 when it is inconsistent.
int make_epilogue(const char *fn, const alpha_conv_epilogue *in, Epilogue *out)
{
    if (in == nullptr) return fail(ALPHA_CONV_EINVAL, "%s: epilogue is null", fn);
    if ((in->X_mean == nullptr) != (in->X_var == nullptr)) return fail(ALPHA_CONV_EINVAL, "%s: X_mean and X_var go together", fn);
    if ((in->A == nullptr) != (in->B == nullptr)) return fail(ALPHA_CONV_EINVAL, "%s: A and B go together", fn);
    if (!aligned16(in->Bias) || !aligned16(in->X_mean) || !aligned16(in->X_var) || !aligned16(in->A) || !aligned16(in->B))
        return fail(ALPHA_CONV_EINVAL, "%s: misaligned epilogue pointer", fn);
    Epilogue e{};
    e.bias = in->Bias; e.mean = in->X_mean; e.var = in->X_var; e.A = in->A; e.B = in->B;
    e.eps = in->eps; e.slope = in->k;
    e.fused = (in->X_mean || in->A || in->k != 1.f) ? 1 : 0;   // a bias alone is every kernel's fast path
    *out = e;
    return 0;
}
int row_function(const char *fn, int64_t stream, const float *X, float *Y, const Epilogue &ep, int lengthv, int mem_width, int mem_stride)
{
    if (!X || !Y || !aligned16(X) || !aligned16(Y)) return fail(ALPHA_CONV_EINVAL, "%s: null or misaligned pointer", fn);
    if (lengthv < 0 || mem_stride < 4 || (mem_stride & 3) || mem_width < 1 || mem_width > mem_stride || lengthv % mem_stride != 0)
        return fail(ALPHA_CONV_EINVAL, "%s: need lengthv = height * mem_stride, mem_stride a multiple of 4, 1 <= mem_width <= mem_stride", fn);
    return hip_status(launch_epilogue_rows(reinterpret_cast<hipStream_t>((intptr_t)stream), X, Y, ep, lengthv, mem_width, mem_stride), fn);
}
}  // namespace

int alpha_conv3D_fused(const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, int FH, int FW,
                       const alpha_conv_epilogue *epilogue, float *Y, int OH, int OW, int N, int IC, int OC,
                       int sh, int sw, int ph, int pw)
{
    Epilogue ep;
    if (int e = make_epilogue(__func__, epilogue, &ep)) return e;
    return forward(__func__, streams, length, X, IH, IW, W, FILTER_W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw, nullptr, &ep);
}
int alpha_conv3D_GemmR_fused(const int64_t *streams, int length, const float *X, int IH, int IW, const float *W, const float *CW,
                             int FH, int FW, const alpha_conv_epilogue *epilogue, float *Y, int OH, int OW, int N, int IC, int OC,
                             int sh, int sw, int ph, int pw)
{
    Epilogue ep;
    if (int e = make_epilogue(__func__, epilogue, &ep)) return e;
    return forward(__func__, streams, length, X, IH, IW, CW, FILTER_CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw, nullptr, &ep, W);
}
int alpha_conv3D_winograd_fused(const int64_t *streams, int length, const float *X, int IH, int IW, const float *U,
                                const alpha_conv_epilogue *epilogue, float *Y, int OH, int OW, int N, int IC, int OC, int ph, int pw)
{
    CHECK_STREAMS();
    CHECK_PTR(X);
    CHECK_PTR(U);
    CHECK_PTR(Y);
    Epilogue ep;
    if (int e = make_epilogue(__func__, epilogue, &ep)) return e;
    if (int e = check_dims(__func__, N, IC, OC, IH, IW, OH, OW, 3, 3, 1, 1, ph, pw)) return e;
    hipError_t e = launch_winograd(stream0(streams), X, U, Y, N, IH, IW, IC, OH, OW, OC, ph, pw, nullptr, &ep);
    if (e == hipErrorNotSupported) return fail(ALPHA_CONV_EINVAL, "%s: needs OH = IH + 2*ph - 2, OW = IW + 2*pw - 2", __func__);
    return hip_status(e, __func__);
}
int alpha_dconv3D_deltaX_s1_leakyRelu(const int64_t *streams, int length, const float *deltaY, int OH, int OW, const float *W,
                                      int FH, int FW, const float *Xf, float k, float *deltaX, int IH, int IW,
                                      int N, int IC, int OC, int ph, int pw)
{
    CHECK_PTR(Xf);
    Epilogue ep{};
    ep.gate = Xf; ep.slope = k; ep.fused = 1;
    return deltaX_s1(__func__, streams, length, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw, &ep);
}
int alpha_dconv3D_deltaX_kernelSplit_leakyRelu(const int64_t *streams, int length, const float *deltaY, int OH, int OW,
                                               const float *CW, int FH, int FW, const float *Xf, float k, float *deltaX,
                                               int IH, int IW, int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    CHECK_PTR(Xf);
    Epilogue ep{};
    ep.gate = Xf; ep.slope = k; ep.fused = 1;
    return deltaX_phases(__func__, streams, length, deltaY, OH, OW, CW, true, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw, &ep);
}
int alpha_leakyRelu2D(int64_t stream, const float *X, float k, float *Y, int lengthv, int mem_width, int mem_stride)
{
    Epilogue ep{};
    ep.slope = k; ep.fused = 1;
    return row_function(__func__, stream, X, Y, ep, lengthv, mem_width, mem_stride);
}
int alpha_leakyRelu2D_deltaX_v1(int64_t stream, float *deltaX, const float *deltaY, const float *Y, float k,
                                int lengthv, int mem_width, int mem_stride)
{
    CHECK_PTR(Y);
    Epilogue ep{};
    ep.gate = Y; ep.slope = k; ep.fused = 1;
    return row_function(__func__, stream, deltaY, deltaX, ep, lengthv, mem_width, mem_stride);
}
int alpha_batchNorm2D_row(int64_t stream, const float *X, const float *X_mean, const float *X_var, float eps, int row_lengthv,
                          float *Y, int lengthv, int mem_width, int mem_stride)
{
    CHECK_PTR(X_mean);
    CHECK_PTR(X_var);
    if (row_lengthv != mem_stride) return fail(ALPHA_CONV_EINVAL, "%s: row_lengthv must equal mem_stride", __func__);
    Epilogue ep{};
    ep.mean = X_mean; ep.var = X_var; ep.eps = eps; ep.slope = 1.f; ep.fused = 1;
    return row_function(__func__, stream, X, Y, ep, lengthv, mem_width, mem_stride);
}
int alpha_batchNorm_affined2D_row(int64_t stream, const float *X, const float *X_mean, const float *X_var, float eps,
                                  const float *A, const float *B, int row_lengthv, float *Y, int lengthv, int mem_width, int mem_stride)
{
    CHECK_PTR(X_mean);
    CHECK_PTR(X_var);
    CHECK_PTR(A);
    CHECK_PTR(B);
    if (row_lengthv != mem_stride) return fail(ALPHA_CONV_EINVAL, "%s: row_lengthv must equal mem_stride", __func__);
    Epilogue ep{};
    ep.mean = X_mean; ep.var = X_var; ep.eps = eps; ep.A = A; ep.B = B; ep.slope = 1.f; ep.fused = 1;
    return row_function(__func__, stream, X, Y, ep, lengthv, mem_width, mem_stride);
}

// ---- backward of batch normalisation: the field sums and the row functions ------------------------------------------
namespace {
int bn_sums(const char *fn, int64_t stream1, int form, const float *deltaY, const float *S, const float *mean, const float *var, float eps,
            const float *A, const float *B, int N, int M, float *deltaA_buf, float *deltaA, float *deltaB_buf, float *deltaB,
            int mem_width, int mem_stride, int partNum, int *nextN)
{
    if (!deltaY || !S || !deltaA || !deltaB || !aligned16(deltaY) || !aligned16(S) || !aligned16(deltaA) || !aligned16(deltaB) ||
        !aligned16(deltaA_buf) || !aligned16(deltaB_buf) || !aligned16(mean) || !aligned16(var) || !aligned16(A) || !aligned16(B))
        return fail(ALPHA_CONV_EINVAL, "%s: null or misaligned pointer", fn);
    if (N < 1 || M < 4 || (M & 3) || mem_stride < 4 || (mem_stride & 3) || mem_width < 1 || mem_width > mem_stride || M % mem_stride != 0)
        return fail(ALPHA_CONV_EINVAL, "%s: need N >= 1, M a multiple of mem_stride, mem_stride a multiple of 4, 1 <= mem_width <= mem_stride", fn);
    if (M != mem_stride) return fail(ALPHA_CONV_EINVAL, "%s: rows of more than one mem_stride are not supported", fn);
    if ((long)N * M >= (1L << 31)) return fail(ALPHA_CONV_EINVAL, "%s: tensor exceeds 2^31 elements", fn);
    if (partNum < 1) partNum = 1;
    int n = bn_field_nextN(N, M);
    if (n > partNum && (!deltaA_buf || !deltaB_buf)) return fail(ALPHA_CONV_EINVAL, "%s: buffers are null", fn);
    if (int e = hip_status(launch_bn_field_sums(reinterpret_cast<hipStream_t>((intptr_t)stream1), form, deltaY, S, mean, var, eps, A, B, N, M,
                                                n > partNum ? deltaA_buf : nullptr, deltaA, n > partNum ? deltaB_buf : nullptr, deltaB, mem_width), fn))
        return e;
    // the value the reference returns: rows left after its last stage (Cuda_reduce field_*_deltaAB: "return nextN")
    while (n > partNum) {
        const int next = bn_field_nextN(n, M);
        if (next >= n) break;
        n = next;
    }
    if (nextN) *nextN = n;
    return 0;
}

int bn_dx(const char *fn, int64_t stream, int form, bool affine, const float *deltaY, const float *S, const float *mean, const float *var,
          float eps, const float *A, const float *B, const float *p1, const float *p2, int row_lengthv, float *deltaX, int lengthv,
          int mem_width, int mem_stride)
{
    if (!deltaY || !S || !var || !p1 || !p2 || !deltaX || !aligned16(deltaY) || !aligned16(S) || !aligned16(var) || !aligned16(p1) ||
        !aligned16(p2) || !aligned16(deltaX) || !aligned16(mean) || !aligned16(A) || !aligned16(B))
        return fail(ALPHA_CONV_EINVAL, "%s: null or misaligned pointer", fn);
    if (lengthv < 0 || mem_stride < 4 || (mem_stride & 3) || mem_width < 1 || mem_width > mem_stride || lengthv % mem_stride != 0)
        return fail(ALPHA_CONV_EINVAL, "%s: need lengthv = height * mem_stride, mem_stride a multiple of 4, 1 <= mem_width <= mem_stride", fn);
    if (row_lengthv != mem_stride) return fail(ALPHA_CONV_EINVAL, "%s: row_lengthv must equal mem_stride", fn);
    return hip_status(launch_bn_delta_x(reinterpret_cast<hipStream_t>((intptr_t)stream), form, affine, deltaY, S, mean, var, eps, A, B, p1, p2,
                                        row_lengthv, deltaX, lengthv, mem_width), fn);
}
}  // namespace

int alpha_field_affine_deltaAB_v1(int64_t stream1, int64_t stream2, const float *deltaY, const float *Y, const float *A, const float *B,
                                  int N, int M, float *deltaA_buf, float *deltaA, float *deltaB_buf, float *deltaB,
                                  int mem_width, int mem_stride, int partNum, int *nextN)
{
    (void)stream2;   // everything is ordered on stream1; the caller records its event on both streams
    CHECK_PTR(A);
    CHECK_PTR(B);
    return bn_sums(__func__, stream1, 1, deltaY, Y, nullptr, nullptr, 0.f, A, B, N, M, deltaA_buf, deltaA, deltaB_buf, deltaB, mem_width, mem_stride, partNum, nextN);
}
int alpha_field_affine_deltaAB_v2(int64_t stream1, int64_t stream2, const float *deltaY, const float *X_norm,
                                  int N, int M, float *deltaA_buf, float *deltaA, float *deltaB_buf, float *deltaB,
                                  int mem_width, int mem_stride, int partNum, int *nextN)
{
    (void)stream2;
    return bn_sums(__func__, stream1, 0, deltaY, X_norm, nullptr, nullptr, 0.f, nullptr, nullptr, N, M, deltaA_buf, deltaA, deltaB_buf, deltaB, mem_width, mem_stride, partNum, nextN);
}
int alpha_field_batchNorm_deltaAB_v2(int64_t stream1, int64_t stream2, const float *deltaY, const float *X, const float *X_mean,
                                     const float *X_var, float eps, int N, int M, float *deltaA_buf, float *deltaA,
                                     float *deltaB_buf, float *deltaB, int mem_width, int mem_stride, int partNum, int *nextN)
{
    (void)stream2;
    CHECK_PTR(X_mean);
    CHECK_PTR(X_var);
    return bn_sums(__func__, stream1, 2, deltaY, X, X_mean, X_var, eps, nullptr, nullptr, N, M, deltaA_buf, deltaA, deltaB_buf, deltaB, mem_width, mem_stride, partNum, nextN);
}
int alpha_batchNorm2D_row_deltaX_v1(int64_t stream, const float *deltaY, const float *Y, const float *X_var, float eps,
                                    const float *deltaXp1, const float *deltaXp2, int row_lengthv, float *deltaX,
                                    int lengthv, int mem_width, int mem_stride)
{
    return bn_dx(__func__, stream, 0, false, deltaY, Y, nullptr, X_var, eps, nullptr, nullptr, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv, mem_width, mem_stride);
}
int alpha_batchNorm2D_row_deltaX_v2(int64_t stream, const float *deltaY, const float *X, const float *X_mean, const float *X_var, float eps,
                                    const float *deltaXp1, const float *deltaXp2, int row_lengthv, float *deltaX,
                                    int lengthv, int mem_width, int mem_stride)
{
    CHECK_PTR(X_mean);
    return bn_dx(__func__, stream, 2, false, deltaY, X, X_mean, X_var, eps, nullptr, nullptr, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv, mem_width, mem_stride);
}
int alpha_batchNorm_affined2D_row_deltaX_v1(int64_t stream, const float *deltaY, const float *Y, const float *X_var, float eps,
                                            const float *A, const float *B, const float *deltaXp1, const float *deltaXp2,
                                            int row_lengthv, float *deltaX, int lengthv, int mem_width, int mem_stride)
{
    CHECK_PTR(A);
    CHECK_PTR(B);
    return bn_dx(__func__, stream, 1, true, deltaY, Y, nullptr, X_var, eps, A, B, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv, mem_width, mem_stride);
}
int alpha_batchNorm_affined2D_row_deltaX_v2(int64_t stream, const float *deltaY, const float *X, const float *X_mean, const float *X_var,
                                            float eps, const float *A, const float *deltaXp1, const float *deltaXp2,
                                            int row_lengthv, float *deltaX, int lengthv, int mem_width, int mem_stride)
{
    CHECK_PTR(X_mean);
    CHECK_PTR(A);
    return bn_dx(__func__, stream, 2, true, deltaY, X, X_mean, X_var, eps, A, nullptr, deltaXp1, deltaXp2, row_lengthv, deltaX, lengthv, mem_width, mem_stride);
}

}  // extern "C"
#pragma GCC visibility pop
