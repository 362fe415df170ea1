// Backward-filter as a split-K implicit GEMM on fp32 MFMA, gfx950.
//
//   deltaW[oc, (fh,fw,ic)] = sum_k deltaY[k, oc] * Xcol[k, (fh,fw,ic)],   k = (n, oh, ow)
//
// Both operands are contiguous along their non-K axis in memory (deltaY along oc, X along ic), so
// both are staged in LDS as [k][m] rows (stride +8 floats) and fed to the MFMA with 32-bit reads,
// lanes running across oc / columns. Each workgroup owns a tile of oc x columns and one K slice
// (blockIdx.z); slices write to deltaW (z = 0) or deltaW_buf[z-1]; nothing is accumulated with
// atomics, so a fixed launch gives bit-identical results on every run.
#include "common.hpp"

namespace alpha {

template <int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(256, 2) void delta_w_kernel(const DeltaWArgs p)
{
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32, BK = 32;
    constexpr int YS = BM + 8, XS = BN + 8;
    constexpr int Y_TILE = BK * YS, X_TILE = BK * XS;
    constexpr int LPR_Y = BM / 4, RPP_Y = 256 / LPR_Y, Y_PASSES = BK / RPP_Y;
    constexpr int LPR_X = BN / 4, RPP_X = 256 / LPR_X, X_PASSES = BK / RPP_X;
    static_assert(WM * WN == 4, "4 wavefronts per workgroup");

    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *Ys = smem;
    float *Xs = smem + 2 * Y_TILE;

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, h = lane >> 5;

    const int c0 = blockIdx.x * BN;   // first column (fh,fw,ic flattened)
    const int oc0 = blockIdx.y * BM;
    const int z = blockIdx.z;

    const int IH = p.IH, IW = p.IW, IC = p.IC, OC = p.OC, GM = p.GM;
    const int OW = p.d_OW.d, OHW = p.d_OHW.d, FW = p.d_FW.d;

    const int k_start = p.GK_slice * z;
    const int k_end = (z != p.GZ - 1) ? k_start + p.GK_slice : p.GK;
    float *dst = (z == 0) ? p.dW : p.dW_buf + (size_t)(z - 1) * OC * GM;

    // this thread's column quad of the X tile: fixed for the whole K loop
    const int xcol = c0 + (t % LPR_X) * 4;
    const bool xcolv = xcol < GM;
    const int xtap = fdiv(xcol, p.d_IC), x_ic = xcol - xtap * IC;
    const int x_fh = fdiv(xtap, p.d_FW), x_fw = xtap - x_fh * FW;
    const int xkrow = t / LPR_X;

    const int ycol = oc0 + (t % LPR_Y) * 4;
    const bool ycolv = ycol < OC;
    const int ykrow = t / LPR_Y;

    // (the vector type, not the float4 struct: copies of the struct keep these arrays in scratch memory)
    floatx4 yreg[Y_PASSES], xreg[X_PASSES];
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};

    auto load_global = [&](int kbase) {
#pragma unroll
        for (int q = 0; q < Y_PASSES; q++) {
            const int k = kbase + ykrow + RPP_Y * q;
            const bool ok = ycolv && k < k_end;
            yreg[q] = ok ? *reinterpret_cast<const floatx4 *>(p.dY + (size_t)k * OC + ycol) : zero4;
        }
#pragma unroll
        for (int q = 0; q < X_PASSES; q++) {
            const int k = kbase + xkrow + RPP_X * q;
            const int n = fdiv(k, p.d_OHW), rem = k - n * OHW;
            const int oh = fdiv(rem, p.d_OW), ow = rem - oh * OW;
            const int ih = oh * p.sh - p.ph + x_fh, iw = ow * p.sw - p.pw + x_fw;
            const bool ok = xcolv && k < k_end && (unsigned)ih < (unsigned)IH && (unsigned)iw < (unsigned)IW;
            const int off = ((n * IH + ih) * IW + iw) * IC + x_ic;
            xreg[q] = ok ? *reinterpret_cast<const floatx4 *>(p.X + off) : zero4;
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int q = 0; q < Y_PASSES; q++)
            *reinterpret_cast<floatx4 *>(Ys + buf * Y_TILE + (ykrow + RPP_Y * q) * YS + (t % LPR_Y) * 4) = yreg[q];
#pragma unroll
        for (int q = 0; q < X_PASSES; q++)
            *reinterpret_cast<floatx4 *>(Xs + buf * X_TILE + (xkrow + RPP_X * q) * XS + (t % LPR_X) * 4) = xreg[q];
    };

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    const int nIter = (k_end - k_start + BK - 1) / BK;
    if (nIter > 0) {
        load_global(k_start);
        store_lds(0);
    }
    __syncthreads();

    for (int it = 0; it < nIter; it++) {
        const int buf = it & 1;
        const bool more = it + 1 < nIter;
        if (more) load_global(k_start + (it + 1) * BK);

        const float *ys = Ys + buf * Y_TILE + (4 * h) * YS + wm * TM * 32 + l32;
        const float *xs = Xs + buf * X_TILE + (4 * h) * XS + wn * TN * 32 + l32;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            float a[TM][4], b[TN][4];
#pragma unroll
            for (int s = 0; s < 4; s++) {
#pragma unroll
                for (int i = 0; i < TM; i++) a[i][s] = ys[(8 * g + s) * YS + i * 32];
#pragma unroll
                for (int j = 0; j < TN; j++) b[j][s] = xs[(8 * g + s) * XS + j * 32];
            }
#pragma unroll
            for (int s = 0; s < 4; s++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][s], b[j][s], acc[i][j], 0, 0, 0);
        }
        if (more) store_lds(buf ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = c0 + (wn * TN + j) * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int oc = oc0 + (wm * TM + i) * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                if (oc < OC && col < GM) dst[(size_t)oc * GM + col] = acc[i][j][r];
            }
        }
}

template <int WM, int WN, int TM, int TN>
static hipError_t launch_dw_cfg(hipStream_t stream, const DeltaWArgs &a)
{
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    constexpr size_t lds = (size_t)2 * 32 * ((BM + 8) + (BN + 8)) * sizeof(float);
    constexpr auto kern = delta_w_kernel<WM, WN, TM, TN>;
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    dim3 grid((a.GM + BN - 1) / BN, (a.OC + BM - 1) / BM, a.GZ);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, a);
    return hipGetLastError();
}

hipError_t launch_deltaW(hipStream_t stream, const DeltaWArgs &a0)
{
    DeltaWArgs a = a0;
    if (a.OC <= 0 || a.GM <= 0 || a.GZ <= 0) return hipSuccess;
    a.d_IC = make_fastdiv(a.IC);
    a.d_FW = make_fastdiv(a.FW);
    a.d_OW = make_fastdiv(a.OW);
    a.d_OHW = make_fastdiv(a.OH * a.OW);
    if (a.OC <= 32 && a.GM <= 32) return launch_dw_cfg<2, 2, 1, 1>(stream, a);  // 64x64 tile, masked
    if (a.OC >= 128 && a.GM >= 128) return launch_dw_cfg<2, 2, 2, 2>(stream, a);
    if (a.GM >= 128) return launch_dw_cfg<2, 2, 1, 2>(stream, a);
    return launch_dw_cfg<2, 2, 1, 1>(stream, a);
}

}  // namespace alpha
