// Launcher of the convolution without LDS (direct_conv_kernel.hpp), its second kernel for the pieces in lent scratch, and
// the estimate of how evenly a layer divides.
#include "direct_conv_kernel.hpp"

namespace alpha {


// The second launch of the form without tickets: one workgroup of 256 threads per item left over.
__global__ __launch_bounds__(256) void direct_conv_fixup_kernel(const DirectConvArgs p)
{
    dc_add_pieces<false>(p, blockIdx.x, threadIdx.x);
}

// Share of the SIMDs' time that is work when `items` equal items are dealt to `cus` workgroups as the kernel does: a
// workgroup with n items spends f(n) whole items per SIMD and a quarter of each item left over (counted 10 % dearer:
// the partial sums' way through LDS, shorter loops). With a workspace (and all items shared) the items that do not
// divide by the workgroups are cut into pieces, so the largest share is base items and one piece.
static double direct_conv_balance(long items, int cus, bool workspace)
{
    const long wgs = items < cus ? items : cus;
    auto cost = [](long n) { const long f = dc_whole_items((int)(n < (1 << 30) ? n : (1 << 30))); return (double)f + 1.1 * 0.25 * (double)(n - 4 * f); };
    const long n_hi = (items + wgs - 1) / wgs, n_lo = items / wgs;
    double worst = cost(n_hi) > cost(n_lo) ? cost(n_hi) : cost(n_lo);
    const long left = items - n_lo * wgs;
    if (workspace && left > 0 && wgs / left >= 2 && n_lo >= 1 && dc_whole_items((int)n_lo + 1) == 0) {
        const long split = wgs / left < 8 ? wgs / left : 8;
        worst = cost(n_lo) + 1.1 * 0.25 / (double)split;
    }
    return (double)items / (4.0 * (double)cus) / worst;
}

// Whether the kernel's work items (16 pixels x 64 produced channels) divide evenly enough among the compute units for it
// to beat the LDS-halo kernels on a stride-1 layer. Measured (forward, 3x3, N = 64, against the kernel with the prefetched
// halo): 56x56x64 (49 items per workgroup) 0.111 against 0.115 ms, 28x28x128 (24 or 25) 0.110 against 0.123 ms, 14x14x256
// (12 or 13: balance 0.91) 0.121 against 0.124 ms, 7x7x512 (6 or 7: 0.80) 0.126 against 0.141 ms.
bool direct_conv_balanced(long M, int CO, bool workspace)
{
    const int cus = device_cu_count();
    if (cus < 1 || M < 1) return false;
    return direct_conv_balance(((M + 15) / 16) * ((CO + 63) / 64), cus, workspace) >= 0.75;
}

// O[N, OHt, OWt, CO] = convolution of A[N, AH, AW, AC] (stride sh x sw, padding ph x pw, TH x TW taps) with the filter B
// whose element (tap = th * TW + tw, c, co) is at b_off + tap * b_tap + c * b_k + co: CW[FH, FW, IC, OC] forward
// (0, IC * OC, OC), W[OC, FH, FW, IC] rotated by 180 degrees for stride-1 backward-data ((FH*FW - 1) * IC, -IC, FH*FW*IC).
// Returns hipErrorNotSupported (nothing launched) when the layer does not fit: AC not a multiple of 16, a filter beyond
// 16 x 16, tensors of 2 GB. (An odd number of steps TH * TW * AC / 16 is taken, without whole items: see the kernel.)
// `ws` (may be NULL), ws_bytes: scratch for the duration of the launch. With it, a layer whose items do not divide by the
// workgroups and are few per workgroup (fewer than 16: all of them shared by the workgroup's wavefronts) is dealt out in
// equal shares of whole items, the items left over are cut along the reduction into one piece per workgroup, and a second
// short launch adds the pieces: 1568 items on 256 workgroups are 6 each + an eighth of one, not 6 or 7.
// `tickets` (may be NULL), n_tickets: 32-bit words that are zero before the launch, one per item left over (fewer than half
// the compute units); with them the workgroup that delivers an item's last piece adds the pieces and there is no second
// launch. The kernel leaves them zero. Launches that share them, like launches that share `ws`, must not overlap.
hipError_t launch_direct_conv(hipStream_t stream, const float *A, const float *B, float *O, int N, int AH, int AW, int AC,
                              int OHt, int OWt, int CO, int TH, int TW, int sh, int sw, int ph, int pw,
                              int b_off, int b_tap, int b_k, long b_elems, const float *bias, const Epilogue *ep,
                              float *ws, size_t ws_bytes, unsigned *tickets, int n_tickets)
{
    if (AC < 16 || (AC & 15) || CO < 4 || (CO & 3) || TH < 1 || TW < 1 || TH > 16 || TW > 16) return hipErrorNotSupported;
    const long M = (long)N * OHt * OWt;
    const long a_bytes = (long)N * AH * AW * AC * 4, b_bytes = b_elems * 4, o_bytes = M * CO * 4;
    if (M < 1 || a_bytes >= (1L << 31) || o_bytes >= (1L << 31) || b_bytes >= (1L << 30)) return hipErrorNotSupported;
    const int cus = device_cu_count();
    if (cus < 1) return hipErrorNotSupported;
    DirectConvArgs a{};
    a.A = A; a.B = B; a.O = O;
    a.M = (int)M; a.AH = AH; a.AW = AW; a.AC = AC; a.CO = CO;
    a.TH = TH; a.TW = TW; a.sh = sh; a.sw = sw; a.ph = ph; a.pw = pw;
    a.b_off = b_off; a.b_tap = b_tap; a.b_k = b_k;
    a.a_bytes = (int)a_bytes; a.b_bytes = (int)b_bytes; a.o_bytes = (int)o_bytes;
    a.tiles = (int)((M + 15) / 16);
    a.nblocks = (CO + 63) / 64;
    if ((long)a.tiles * a.nblocks >= (1L << 30)) return hipErrorNotSupported;
    a.items = a.tiles * a.nblocks;
    a.d_OW = make_fastdiv(OWt);
    a.d_OHW = make_fastdiv(OHt * OWt);
    a.d_TW = make_fastdiv(TW);
    a.ep = ep ? *ep : bias_epilogue(bias);
    const int wgs = cus < a.items ? cus : a.items;   // one workgroup of eight wavefronts per compute unit
    a.wgs = wgs;
    // few items per workgroup and a filter beyond an XCD's 4 MB of L2: every workgroup streams its blocks' filter slices, and
    // an XCD whose workgroups hold all blocks at once fetches them again and again (7x7x512 -> 512 at N = 64, 9.4 MB of
    // filter: 313 MB of L2 fills; 124 MB with an XCD's workgroups on neighbouring shares, at the same speed or 0.5 % better)
    a.xcd_major = (wgs & 7) == 0 && a.nblocks > 1 && a.items / wgs < 16 && b_bytes > (4L << 20) ? 1 : 0;
    a.ws = nullptr;
    a.tickets = nullptr;
    {
        // Produced channels per lane: the least with which as many blocks (of 16 per-lane groups) hold the channels as
        // 64-wide ones would - 96 channels are two blocks of 48 (3 per lane: 12 MFMAs a step and tile instead of 16 on one
        // full and one half-empty block) -, where the channel count is a multiple of it
        const int n = (CO + 16 * a.nblocks - 1) / (16 * a.nblocks);
        const int nj = (n < 4 && CO % n == 0) ? n : 4;
        // an odd number of steps per item: the kernels that add an empty step, where a workgroup has whole items at all
        if (((TH * TW * (AC >> 4)) & 1) && dc_whole_items((a.items + wgs - 1) / wgs) > 0) return launch_direct_conv_odd(stream, a, nj);
        if (nj < 4) return launch_direct_conv_narrow(stream, a, nj);
    }
    a.base = a.items / wgs;
    a.items_left = a.items - a.base * wgs;
    a.split = a.items_left > 0 ? wgs / a.items_left : 0;
    if (a.split > 8) a.split = 8;   // pieces of an eighth of the steps, cut in eight again among the wavefronts, are short enough
    {
        // Worth it where the workgroups that would hold base + 1 items set the time (all items shared: fewer than 16 per
        // workgroup) and what a workgroup saves - an item less the piece it gets, at 128 cycles per step of an item shared
        // by four SIMDs - outweighs the second launch (some 8 k cycles).
        const long KS = (long)TH * TW * (AC >> 4);
        const bool shared_only = a.base >= 1 && dc_whole_items(a.base + 1) == 0;
        if (ws != nullptr && (reinterpret_cast<uintptr_t>(ws) & 15) == 0 && a.items_left > 0 && a.split >= 2 && shared_only &&
            ws_bytes >= (size_t)a.items_left * a.split * 1024 * sizeof(float) && KS * 128 * (a.split - 1) / a.split > 8192 && KS >= 8L * a.split)
            a.ws = ws;
        a.tickets = a.ws != nullptr && tickets != nullptr && n_tickets >= a.items_left ? tickets : nullptr;
    }
    if (a.ws != nullptr) {
        if (a.ep.fused) {
            if (hipError_t e = ensure_dynamic_lds<direct_conv_kernel<true, true>>(DC_LDS_BYTES); e != hipSuccess) return e;
            hipLaunchKernelGGL((direct_conv_kernel<true, true>), dim3(wgs), dim3(512), DC_LDS_BYTES, stream, a);
        } else {
            if (hipError_t e = ensure_dynamic_lds<direct_conv_kernel<false, true>>(DC_LDS_BYTES); e != hipSuccess) return e;
            hipLaunchKernelGGL((direct_conv_kernel<false, true>), dim3(wgs), dim3(512), DC_LDS_BYTES, stream, a);
        }
        if (hipError_t e = hipGetLastError(); e != hipSuccess || a.tickets != nullptr) return e;
        hipLaunchKernelGGL(direct_conv_fixup_kernel, dim3(a.items_left), dim3(256), 0, stream, a);
        return hipGetLastError();
    }
    if (a.ep.fused) {
        if (hipError_t e = ensure_dynamic_lds<direct_conv_kernel<true>>(DC_LDS_BYTES); e != hipSuccess) return e;
        hipLaunchKernelGGL(direct_conv_kernel<true>, dim3(wgs), dim3(512), DC_LDS_BYTES, stream, a);
    } else {
        if (hipError_t e = ensure_dynamic_lds<direct_conv_kernel<false>>(DC_LDS_BYTES); e != hipSuccess) return e;
        hipLaunchKernelGGL(direct_conv_kernel<false>, dim3(wgs), dim3(512), DC_LDS_BYTES, stream, a);
    }
    return hipGetLastError();
}

}  // namespace alpha
