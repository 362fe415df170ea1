// The persistent backward-filter kernel (delta_w_stream_kernel.hpp) with 1, 2 or 3 output AND input channels per lane.
// A translation unit of its own.
#include "delta_w_stream_kernel.hpp"

namespace alpha {

hipError_t launch_deltaW_stream_narrow_xy(hipStream_t stream, const DwStreamArgs &a, size_t lds, int NI, int NJ)
{
    switch (NI * 4 + NJ) {
    case 1 * 4 + 1: return dws_launch<1, 1>(stream, a, lds);
    case 1 * 4 + 2: return dws_launch<1, 2>(stream, a, lds);
    case 1 * 4 + 3: return dws_launch<1, 3>(stream, a, lds);
    case 2 * 4 + 1: return dws_launch<2, 1>(stream, a, lds);
    case 2 * 4 + 2: return dws_launch<2, 2>(stream, a, lds);
    case 2 * 4 + 3: return dws_launch<2, 3>(stream, a, lds);
    case 3 * 4 + 1: return dws_launch<3, 1>(stream, a, lds);
    case 3 * 4 + 2: return dws_launch<3, 2>(stream, a, lds);
    case 3 * 4 + 3: return dws_launch<3, 3>(stream, a, lds);
    default: return hipErrorNotSupported;
    }
}

}  // namespace alpha
