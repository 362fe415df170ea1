// Filter re-layouts and the split-K partial-buffer summation. All are pure HBM-bandwidth
// kernels: 128-bit accesses, lanes along the contiguous axis of whichever side can be.
#include "common.hpp"

namespace alpha {

// W[OC][K] -> CW[K][OC] with K = FH*FW*IC: a matrix transpose through a padded 64x64 LDS tile so
// that both the read (along K) and the write (along OC) are coalesced.
__global__ __launch_bounds__(256) void kernel_remode_kernel(const float *__restrict__ W, float *__restrict__ CW,
                                                            int OC, int K)
{
    __shared__ float tile[64][65];
    const int k0 = blockIdx.x * 64, oc0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;  // 16 x 16
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int oc = oc0 + ty + 16 * r, k = k0 + tx * 4;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (oc < OC && k < K) v = *reinterpret_cast<const float4 *>(W + (size_t)oc * K + k);  // K % 4 == 0
        tile[ty + 16 * r][tx * 4 + 0] = v.x;
        tile[ty + 16 * r][tx * 4 + 1] = v.y;
        tile[ty + 16 * r][tx * 4 + 2] = v.z;
        tile[ty + 16 * r][tx * 4 + 3] = v.w;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int k = k0 + ty + 16 * r, oc = oc0 + tx * 4;
        if (k < K && oc < OC) {  // OC % 4 == 0
            float4 v;
            v.x = tile[tx * 4 + 0][ty + 16 * r];
            v.y = tile[tx * 4 + 1][ty + 16 * r];
            v.z = tile[tx * 4 + 2][ty + 16 * r];
            v.w = tile[tx * 4 + 3][ty + 16 * r];
            *reinterpret_cast<float4 *>(CW + (size_t)k * OC + oc) = v;
        }
    }
}

hipError_t launch_kernel_remode(hipStream_t s, const float *W, float *CW, int FH, int FW, int OC, int IC)
{
    const int K = FH * FW * IC;
    if (K <= 0 || OC <= 0) return hipSuccess;
    dim3 grid((K + 63) / 64, (OC + 63) / 64);
    hipLaunchKernelGGL(kernel_remode_kernel, grid, dim3(256), 0, s, W, CW, OC, K);
    return hipGetLastError();
}

// Kernel-split filter layouts for strided backward-data. Phase (y, x) holds the taps
// fh = y + (CFH_y-1-fhr)*sh, fw = x + (CFW_x-1-fwr)*sw packed from the start of its block of
// OC*mCFH*mCFW*IC floats; V2 orders a block [fhr][fwr][oc][ic], V1 orders it [oc][fhr][fwr][ic].
template <bool V2>
__global__ __launch_bounds__(256) void ks_remode_kernel(const float *__restrict__ W, int FH, int FW,
                                                        float *__restrict__ CW, int mCFH, int mCFW,
                                                        int OC, int IC, int sh, int sw)
{
    const int by = blockIdx.y;
    const int y = by / sw, x = by - y * sw;
    const int CFH = (FH - y + sh - 1) / sh, CFW = (FW - x + sw - 1) / sw;
    float *blk = CW + (size_t)by * OC * mCFH * mCFW * IC;
    const int n4 = (OC * CFH * CFW * IC) >> 2;
    const int IC4 = IC >> 2;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += gridDim.x * blockDim.x) {
        int r = i;
        const int ic = (r % IC4) * 4;
        r /= IC4;
        int oc, fhr, fwr;
        if (V2) {
            oc = r % OC; r /= OC;
            fwr = r % CFW; fhr = r / CFW;
        } else {
            fwr = r % CFW; r /= CFW;
            fhr = r % CFH; oc = r / CFH;
        }
        const int fh = y + (CFH - 1 - fhr) * sh, fw = x + (CFW - 1 - fwr) * sw;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (fh < FH && fw < FW) v = *reinterpret_cast<const float4 *>(W + (((size_t)oc * FH + fh) * FW + fw) * IC + ic);
        *reinterpret_cast<float4 *>(blk + (size_t)i * 4) = v;
    }
}

hipError_t launch_ks_remode(hipStream_t s, int version, const float *W, int FH, int FW, float *CW,
                            int mCFH, int mCFW, int OC, int IC, int sh, int sw)
{
    const int n4 = (OC * mCFH * mCFW * IC) >> 2;
    if (n4 <= 0 || sh <= 0 || sw <= 0) return hipSuccess;
    int bx = (n4 + 255) / 256;
    if (bx > 4096) bx = 4096;
    dim3 grid(bx, sh * sw);
    if (version == 2)
        hipLaunchKernelGGL(ks_remode_kernel<true>, grid, dim3(256), 0, s, W, FH, FW, CW, mCFH, mCFW, OC, IC, sh, sw);
    else
        hipLaunchKernelGGL(ks_remode_kernel<false>, grid, dim3(256), 0, s, W, FH, FW, CW, mCFH, mCFW, OC, IC, sh, sw);
    return hipGetLastError();
}

// deltaW += sum_{p < part} deltaW_buf[p], summed in the fixed order p = 0, 1, ... with fp32 Kahan
// compensation (the reference's recurrence, operation for operation). The adds of one element form a serial
// chain, but the loads do not depend on it: one thread owns ONE element (so even a 16 K-element filter gives
// hundreds of wavefronts) and requests U partials at a time, the next U before the current ones run through the chain.
// Every load is unconditional - a batch that reaches past the last partial reads the last one again - and a partial
// that is not there is left out of the chain by a select (adding a zero would still apply the compensation), so no
// partial is ever waited for on its own: with U = 64 the 127 partials of the Java engine's largest split-K factor are in
// flight at once and the kernel waits for memory once.
template <int U>
__global__ __launch_bounds__(256) void buf_summary_kernel(const float *__restrict__ buf, float *__restrict__ dW,
                                                          int part, int sizeW)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= sizeW) return;
    float dw = dW[i], c = 0.f;
    float b[U], nb[U];
    const float *src = buf + i;
    const int last = part - 1;
#pragma unroll
    for (int u = 0; u < U; u++) b[u] = src[(size_t)(u < last ? u : last) * sizeW];
    for (int p = 0; p < part; p += U) {
        const bool more = p + U < part;   // uniform
        if (more) {
#pragma unroll
            for (int u = 0; u < U; u++) nb[u] = src[(size_t)(p + U + u < last ? p + U + u : last) * sizeW];
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const bool live = p + u < part;   // uniform
            const float y = b[u] - c;
            const float s = dw + y;
            const float cn = (s - dw) - y;
            c = live ? cn : c;
            dw = live ? s : dw;
        }
        if (more) {
#pragma unroll
            for (int u = 0; u < U; u++) b[u] = nb[u];
        }
    }
    dW[i] = dw;
}

hipError_t launch_buf_summary(hipStream_t s, const float *buf, float *dW, int part, int sizeW)
{
    if (sizeW <= 0 || part <= 0) return hipSuccess;
    // One element per thread: a filter of 16 K elements is 256 wavefronts. Workgroups of one or two wavefronts spread them
    // over all compute units (each wavefront waits for its own partials; four on one unit share that unit's load path).
    const int block = sizeW >= 256 * 256 ? 256 : sizeW >= 128 * 256 ? 128 : 64;
    const dim3 grid((sizeW + block - 1) / block);
    if (part <= 4) hipLaunchKernelGGL(buf_summary_kernel<4>, grid, dim3(block), 0, s, buf, dW, part, sizeW);
    else if (part <= 32) hipLaunchKernelGGL(buf_summary_kernel<16>, grid, dim3(block), 0, s, buf, dW, part, sizeW);
    else hipLaunchKernelGGL(buf_summary_kernel<64>, grid, dim3(block), 0, s, buf, dW, part, sizeW);
    return hipGetLastError();
}

// Bias gradient without a backward-filter kernel to ride in: dst_z[oc] = sum over the pixels k of K slice z of
// deltaY[k, oc], slice 0 -> dB, slice z -> dB_buf[z-1] (the partition of the split-K entries). One workgroup per
// (64 channels, slice): 16 lanes cover the channels with 128-bit loads, the 16 lane rows take pixels k, k+16, ...; the
// rows are added through LDS in a fixed order, so the result is bit-reproducible.
__global__ __launch_bounds__(256) void col_sum_kernel(const float *__restrict__ dY, float *__restrict__ dB,
                                                      float *__restrict__ dB_buf, int OC, int GK, int GK_slice, int GZ)
{
    __shared__ float4 part[16][17];
    const int z = blockIdx.y, oc = blockIdx.x * 64 + (threadIdx.x & 15) * 4, row = threadIdx.x >> 4;
    const int k_start = GK_slice * z, k_end = (z != GZ - 1) ? k_start + GK_slice : GK;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (oc < OC)   // OC % 4 == 0
        for (int k = k_start + row; k < k_end; k += 16) {
            const float4 v = *reinterpret_cast<const float4 *>(dY + (size_t)k * OC + oc);
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
    part[row][threadIdx.x & 15] = s;
    __syncthreads();
    if (row == 0 && oc < OC) {
        for (int r = 1; r < 16; r++) {
            const float4 v = part[r][threadIdx.x & 15];
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
        float *dst = (z == 0) ? dB : dB_buf + (size_t)(z - 1) * OC;
        *reinterpret_cast<float4 *>(dst + oc) = s;
    }
}

hipError_t launch_col_sum(hipStream_t s, const float *dY, float *dB, float *dB_buf, int OC, int GK, int GK_slice, int GZ)
{
    if (OC <= 0 || GK <= 0) return hipSuccess;
    hipLaunchKernelGGL(col_sum_kernel, dim3((OC + 63) / 64, GZ), dim3(256), 0, s, dY, dB, dB_buf, OC, GK, GK_slice, GZ);
    return hipGetLastError();
}

}  // namespace alpha
