// The persistent backward-filter kernel (delta_w_stream_kernel.hpp) with 1, 2 or 3 output channels per lane: blocks of 16,
// 32 or 48 output channels. A translation unit of its own.
#include "delta_w_stream_kernel.hpp"

namespace alpha {

hipError_t launch_deltaW_stream_narrow_y(hipStream_t stream, const DwStreamArgs &a, size_t lds, int NI)
{
    switch (NI) {
    case 1: return dws_launch<1, 4>(stream, a, lds);
    case 2: return dws_launch<2, 4>(stream, a, lds);
    case 3: return dws_launch<3, 4>(stream, a, lds);
    default: return hipErrorNotSupported;
    }
}

}  // namespace alpha
