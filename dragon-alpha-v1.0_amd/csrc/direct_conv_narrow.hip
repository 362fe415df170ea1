// The convolution without LDS (direct_conv_kernel.hpp) with 1, 2 or 3 produced channels per lane: blocks of 16, 32 or 48
// produced channels (96 channels: two full blocks of 48). A translation unit of its own: the kernels with 4 per lane
// compile to the code they were before these existed.
#include "direct_conv_kernel.hpp"

namespace alpha {

template <bool EPI, int NJ>
static hipError_t dc_launch_narrow(hipStream_t stream, const DirectConvArgs &a)
{
    constexpr auto kern = direct_conv_kernel<EPI, false, NJ>;
    if (hipError_t e = ensure_dynamic_lds<kern>(DC_LDS_BYTES); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(a.wgs), dim3(512), DC_LDS_BYTES, stream, a);
    return hipGetLastError();
}

hipError_t launch_direct_conv_narrow(hipStream_t stream, const DirectConvArgs &a, int nj)
{
    if (a.ws != nullptr) return hipErrorNotSupported;
    switch (nj * 2 + (a.ep.fused ? 1 : 0)) {
    case 2: return dc_launch_narrow<false, 1>(stream, a);
    case 3: return dc_launch_narrow<true, 1>(stream, a);
    case 4: return dc_launch_narrow<false, 2>(stream, a);
    case 5: return dc_launch_narrow<true, 2>(stream, a);
    case 6: return dc_launch_narrow<false, 3>(stream, a);
    case 7: return dc_launch_narrow<true, 3>(stream, a);
    default: return hipErrorNotSupported;
    }
}

}  // namespace alpha
