// The epilogue of a convolution as a pass of its own over a [height, stride] tensor (HBM-bound, 128-bit accesses): what
// follows a kernel that has no fused form of it, and the library's twins of the row functions the reference applies to
// convolution outputs (leakyRelu2D, leakyRelu2D_deltaX_v1, batchNorm2D_row, batchNorm_affined2D_row:
// Cuda_function.java:1607, 1640, 3829, 3862). A row has `width` data elements and stride - width pad elements
// (stride = width rounded up to 4) which are kept at zero, as the reference's memory layout demands.
#include "common.hpp"

namespace alpha {

__global__ __launch_bounds__(256) void epilogue_rows_kernel(const float *__restrict__ X, float *__restrict__ Y, const Epilogue ep,
                                                            long quads, int width, int stride)
{
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < quads; i += (long)gridDim.x * 256) {
        const float4 v = *reinterpret_cast<const float4 *>(X + 4 * i);
        const int c = (int)((4 * i) % stride);   // stride % 4 == 0: the four elements lie in one row
        float r[4] = {v.x, v.y, v.z, v.w};
        if (ep.gate) {
            const float4 g = *reinterpret_cast<const float4 *>(ep.gate + 4 * i);
            const float gg[4] = {g.x, g.y, g.z, g.w};
#pragma unroll
            for (int j = 0; j < 4; j++) r[j] = c + j < width ? ep_gate(r[j], gg[j], ep.slope) : 0.f;
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float sub = 0.f, mul = 1.f, add = 0.f;
                if (c + j < width) {
                    ep_channel(ep, c + j, sub, mul, add);
                    r[j] = ep_finish(r[j], sub, mul, add, ep.slope);
                } else {
                    r[j] = 0.f;
                }
            }
        }
        *reinterpret_cast<float4 *>(Y + 4 * i) = make_float4(r[0], r[1], r[2], r[3]);
    }
}

// Y = epilogue(X) over lengthv = height * stride elements; X == Y (in place) is allowed.
hipError_t launch_epilogue_rows(hipStream_t s, const float *X, float *Y, const Epilogue &ep, long lengthv, int width, int stride)
{
    if (lengthv <= 0) return hipSuccess;
    if (stride < 4 || (stride & 3) || width < 1 || width > stride || lengthv % stride != 0) return hipErrorInvalidValue;
    const long quads = lengthv / 4;
    long blocks = (quads + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(epilogue_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, s, X, Y, ep, quads, width, stride);
    return hipGetLastError();
}

}  // namespace alpha
