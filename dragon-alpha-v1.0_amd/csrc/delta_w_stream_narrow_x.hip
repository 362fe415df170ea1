// The persistent backward-filter kernel (delta_w_stream_kernel.hpp) with 1, 2 or 3 input channels per lane: blocks of 16,
// 32 or 48 input channels (96 input channels: two full blocks of 48). A translation unit of its own.
#include "delta_w_stream_kernel.hpp"

namespace alpha {

hipError_t launch_deltaW_stream_narrow_x(hipStream_t stream, const DwStreamArgs &a, size_t lds, int NJ)
{
    switch (NJ) {
    case 1: return dws_launch<4, 1>(stream, a, lds);
    case 2: return dws_launch<4, 2>(stream, a, lds);
    case 3: return dws_launch<4, 3>(stream, a, lds);
    default: return hipErrorNotSupported;
    }
}

}  // namespace alpha
