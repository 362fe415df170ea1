// Measurement helper, not part of the product library: a kernel that does nothing but 128-bit LDS reads with a given
// byte stride between the lanes of a wavefront, so that the LDS counters (SQ_LDS_BANK_CONFLICT, SQ_LDS_IDX_ACTIVE) and the
// time per read of a known access pattern can be put beside those of the real kernels. Built as libalpha_probe.so and
// loaded only by bench.py --probe-lds.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float floatx4 __attribute__((ext_vector_type(4)));

// lane L of every wavefront reads 16 bytes at (L * stride_bytes + 16 * (i % 4)) % 64 KB, `iters` times, eight reads in flight
__global__ __launch_bounds__(256) void lds_read128_kernel(float *out, int stride_bytes, int iters)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    for (int i = threadIdx.x; i < 16384; i += 256) lds[i] = (float)(i & 255);
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const unsigned base = ((unsigned)lane * (unsigned)stride_bytes) & 0xFFF0u;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < iters; i++) {
        floatx4 v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const unsigned a = (base + 16u * (unsigned)(k & 3)) & 0xFFF0u;
            asm volatile("ds_read_b128 %0, %1" : "=v"(v[k]) : "v"(a));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int k = 0; k < 8; k++) acc += v[k];
    }
    out[blockIdx.x * 256 + threadIdx.x] = acc[0] + acc[1] + acc[2] + acc[3];
}

// Returns 0 or the HIP error. `out` holds blocks * 256 floats; each of the 4 * blocks wavefronts issues 8 * iters reads.
extern "C" __attribute__((visibility("default"))) int alpha_probe_lds_read128(int64_t stream, float *out, int stride_bytes, int iters, int blocks)
{
    if (!out || stride_bytes < 0 || (stride_bytes & 15) || iters < 1 || blocks < 1) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(lds_read128_kernel, dim3(blocks), dim3(256), 65536, reinterpret_cast<hipStream_t>((intptr_t)stream), out, stride_bytes, iters);
    return (int)hipGetLastError();
}
