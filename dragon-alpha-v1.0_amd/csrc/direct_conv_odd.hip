// The convolution without LDS (direct_conv_kernel.hpp) for layers with an odd number of steps (filter taps x 16 reduced
// channels) per item: an empty step after every item's, so that the loop over whole items, which multiplies two steps per
// turn, takes them. A translation unit of its own: the other kernels compile to the code they were before these existed.
#include "direct_conv_kernel.hpp"

namespace alpha {

template <bool EPI, int NJ>
static hipError_t dc_launch_odd(hipStream_t stream, const DirectConvArgs &a)
{
    constexpr auto kern = direct_conv_kernel<EPI, false, NJ, true>;
    if (hipError_t e = ensure_dynamic_lds<kern>(DC_LDS_BYTES); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(a.wgs), dim3(512), DC_LDS_BYTES, stream, a);
    return hipGetLastError();
}

hipError_t launch_direct_conv_odd(hipStream_t stream, const DirectConvArgs &a, int nj)
{
    if (a.ws != nullptr || ((a.TH * a.TW * (a.AC >> 4)) & 1) == 0) return hipErrorNotSupported;
    switch (nj * 2 + (a.ep.fused ? 1 : 0)) {
    case 2: return dc_launch_odd<false, 1>(stream, a);
    case 3: return dc_launch_odd<true, 1>(stream, a);
    case 4: return dc_launch_odd<false, 2>(stream, a);
    case 5: return dc_launch_odd<true, 2>(stream, a);
    case 6: return dc_launch_odd<false, 3>(stream, a);
    case 7: return dc_launch_odd<true, 3>(stream, a);
    case 8: return dc_launch_odd<false, 4>(stream, a);
    case 9: return dc_launch_odd<true, 4>(stream, a);
    default: return hipErrorNotSupported;
    }
}

}  // namespace alpha
