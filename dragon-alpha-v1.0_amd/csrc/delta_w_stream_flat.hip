// The persistent backward-filter kernel with pixel groups by image (delta_w_stream_kernel.hpp, FLAT), in a translation
// unit of its own.
#include "delta_w_stream_kernel.hpp"

namespace alpha {

hipError_t launch_deltaW_stream_flat(hipStream_t stream, const DwStreamFlatArgs &a, size_t lds)
{
    constexpr auto kern = delta_w_stream_kernel<6, true, DwStreamFlatArgs>;
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(a.wgs), dim3(512), lds, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
