// Generic implicit-GEMM gather convolution on fp32 MFMA (v_mfma_f32_32x32x2_f32), gfx950.
//
// One kernel template serves every "output pixel gathers a window of an NHWC tensor" operator of
// the path: forward (filter in either layout), stride-1 backward-data, the 1x1 cases and each
// phase of kernel-split backward-data. Ragged sizes are handled by masks inside the tile, not by
// extra launches. Specialised fast paths for the 3x3 stride-1 layers live in conv3x3.hip.
//
// Tiling: 256 threads = 4 wavefronts arranged WM x WN; each wavefront owns TM x TN MFMA tiles of
// 32x32, so a workgroup computes BM = WM*TM*32 pixels by BN = WN*TN*32 channels. K advances in
// chunks of 32 through double-buffered LDS tiles (one barrier per chunk); the global loads of
// chunk i+1 are issued before the MFMAs of chunk i.
//
// LDS layouts (floats):
//   A (pixels x k)      : As[row][36]   k contiguous, row stride 36 -> 128-bit reads by 16 lanes hit
//                         64 distinct banks.
//   B, channel-contiguous: Bs[k][BN+8]  read 32 bits at a time, lanes across channels.
//   B, k-contiguous      : Bs[col][36]  same scheme as A.
// K permutation: within an 8-wide k group the lane half h (lane/32) supplies k = 8g + 4h + s at MFMA
// step s, so one 128-bit LDS read feeds four MFMAs. A and B use the same permutation, which leaves
// the sum unchanged.
#include "common.hpp"

namespace alpha {

template <int WM, int WN, int TM, int TN, bool B_NMAJOR>
__global__ __launch_bounds__(256, 2) void gather_conv_kernel(const GatherConvArgs p)
{
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32, BK = 32;
    constexpr int AS = BK + 4;
    constexpr int BSN = BN + 8;
    constexpr int BSK = BK + 4;
    constexpr int A_TILE = BM * AS;
    constexpr int B_TILE = B_NMAJOR ? BK * BSN : BN * BSK;
    constexpr int A_PASSES = BM / 32;
    constexpr int B_PASSES = BN / 32;
    static_assert(WM * WN == 4, "4 wavefronts per workgroup");

    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *As = smem;
    float *Bs = smem + 2 * A_TILE;

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, h = lane >> 5;

    // Consecutive M tiles share input rows; keep them on one XCD (workgroups are dealt to the 8
    // XCDs round-robin) so the halo re-reads hit that XCD's L2.
    const int G = gridDim.x;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int tile_m = xcd * (G >> 3) + min(xcd, G & 7) + idx;
    const int m0 = tile_m * BM;
    const int n0 = blockIdx.y * BN;

    const int AH = p.AH, AW = p.AW, AC = p.AC, K = p.K, CO = p.CO;
    const int OWt = p.d_OWt.d, OHWt = p.d_OHWt.d, TW = p.d_TW.d;

    // ---- per-thread A rows -------------------------------------------------------------------
    int a_ih0[A_PASSES], a_iw0[A_PASSES], a_base[A_PASSES];
#pragma unroll
    for (int q = 0; q < A_PASSES; q++) {
        const int m = m0 + (t >> 3) + 32 * q;
        if (m < p.M) {
            const int n = fdiv(m, p.d_OHWt), rem = m - n * OHWt;
            const int i = fdiv(rem, p.d_OWt), j = rem - i * OWt;
            a_ih0[q] = i * p.sh - p.ph;
            a_iw0[q] = j * p.sw - p.pw;
            a_base[q] = n * p.a_sn;
        } else {
            a_ih0[q] = -(1 << 28);
            a_iw0[q] = 0;
            a_base[q] = 0;
        }
    }
    const int kq = (t & 7) * 4;

    // ---- per-thread B positions ----------------------------------------------------------------
    constexpr int LPR = BN / 4;          // lanes per k-row (channel-contiguous B)
    constexpr int RPP = 256 / LPR;       // k-rows per pass
    const int b_col = B_NMAJOR ? n0 + (t % LPR) * 4 : 0;
    const int b_krow = t / LPR;

    // (the vector type, not the float4 struct: copies of the struct keep these arrays in scratch memory)
    floatx4 areg[A_PASSES], breg[B_PASSES];
    const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};

    auto load_global = [&](int it) {
        const int k = it * BK + kq;
        const bool kv = k < K;
        const int tap = fdiv(k, p.d_AC), c = k - tap * AC;
        const int th = fdiv(tap, p.d_TW), tw = tap - th * TW;
#pragma unroll
        for (int q = 0; q < A_PASSES; q++) {
            const int ih = a_ih0[q] + th, iw = a_iw0[q] + tw;
            const bool ok = kv && (unsigned)ih < (unsigned)AH && (unsigned)iw < (unsigned)AW;
            const int off = a_base[q] + (ih * AW + iw) * AC + c;
            areg[q] = ok ? *reinterpret_cast<const floatx4 *>(p.A + off) : zero4;
        }
        if (B_NMAJOR) {
#pragma unroll
            for (int q = 0; q < B_PASSES; q++) {
                const int kb = it * BK + b_krow + RPP * q;
                const int tapb = fdiv(kb, p.d_AC), cb = kb - tapb * AC;
                const int thb = fdiv(tapb, p.d_TW), twb = tapb - thb * TW;
                const bool ok = kb < K && b_col < CO;
                const int off = p.b_off + thb * p.b_sth + twb * p.b_stw + cb * p.b_sc + b_col;
                breg[q] = ok ? *reinterpret_cast<const floatx4 *>(p.B + off) : zero4;
            }
        } else {
            const int koff = p.b_off + th * p.b_sth + tw * p.b_stw + c;
#pragma unroll
            for (int q = 0; q < B_PASSES; q++) {
                const int col = n0 + (t >> 3) + 32 * q;
                const bool ok = kv && col < CO;
                const int off = koff + col * p.b_sn;
                breg[q] = ok ? *reinterpret_cast<const floatx4 *>(p.B + off) : zero4;
            }
        }
    };

    auto store_lds = [&](int buf) {
        float *as = As + buf * A_TILE;
        float *bs = Bs + buf * B_TILE;
#pragma unroll
        for (int q = 0; q < A_PASSES; q++)
            *reinterpret_cast<floatx4 *>(as + ((t >> 3) + 32 * q) * AS + kq) = areg[q];
        if (B_NMAJOR) {
#pragma unroll
            for (int q = 0; q < B_PASSES; q++)
                *reinterpret_cast<floatx4 *>(bs + (b_krow + RPP * q) * BSN + (t % LPR) * 4) = breg[q];
        } else {
#pragma unroll
            for (int q = 0; q < B_PASSES; q++)
                *reinterpret_cast<floatx4 *>(bs + ((t >> 3) + 32 * q) * BSK + kq) = breg[q];
        }
    };

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    const int nIter = (K + BK - 1) / BK;
    if (nIter > 0) {
        load_global(0);
        store_lds(0);
    }
    __syncthreads();

    for (int it = 0; it < nIter; it++) {
        const int buf = it & 1;
        const bool more = it + 1 < nIter;
        if (more) load_global(it + 1);

        const float *as = As + buf * A_TILE + (wm * TM * 32 + l32) * AS + 4 * h;
        const float *bs = B_NMAJOR ? Bs + buf * B_TILE + (4 * h) * BSN + wn * TN * 32 + l32
                                   : Bs + buf * B_TILE + (wn * TN * 32 + l32) * BSK + 4 * h;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            floatx4 a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) a[i] = *reinterpret_cast<const floatx4 *>(as + i * 32 * AS + 8 * g);
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if (B_NMAJOR) {
#pragma unroll
                    for (int s = 0; s < 4; s++) b[j][s] = bs[(8 * g + s) * BSN + j * 32];
                } else {
                    b[j] = *reinterpret_cast<const floatx4 *>(bs + j * 32 * BSK + 8 * g);
                }
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

    // ---- epilogue: the tile goes through LDS so that every output row leaves as whole 16-byte-per-lane segments
    // (stored straight from the MFMA layout, 4 bytes per lane, the same tile cost 8-10x its size in write traffic) ----
    constexpr int OS = BN + 4;
    float *Os = smem;                                            // [BM][OS]; the loop's last barrier freed the tiles
    int *rowoff = reinterpret_cast<int *>(smem + BM * OS);       // [BM] output offset of each row, -1 beyond M
    for (int r = t; r < BM; r += 256) {
        const int m = m0 + r;
        int off = -1;
        if (m < p.M) {
            const int n = fdiv(m, p.d_OHWt), rem = m - n * OHWt;
            const int i = fdiv(rem, p.d_OWt), j = rem - i * OWt;
            off = p.o_off + n * p.o_sn + i * p.o_sh + j * p.o_sw;
        }
        rowoff[r] = off;
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = (wn * TN + j) * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = (wm * TM + i) * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                Os[row * OS + col] = acc[i][j][r];
            }
        }
    __syncthreads();
    for (int idx = t; idx < BM * (BN / 4); idx += 256) {
        const int row = idx / (BN / 4), c4 = (idx % (BN / 4)) * 4;
        const int ro = rowoff[row];
        if (ro >= 0 && n0 + c4 < CO)   // CO % 4 == 0: the four columns are valid together
            *reinterpret_cast<float4 *>(p.O + ro + n0 + c4) =
                epilogue4(*reinterpret_cast<const float4 *>(Os + row * OS + c4), p.ep, n0 + c4, (size_t)(ro + n0 + c4));
    }
}

template <int WM, int WN, int TM, int TN, bool B_NMAJOR>
static hipError_t launch_cfg(hipStream_t stream, const GatherConvArgs &a)
{
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    constexpr int A_TILE = BM * 36;
    constexpr int B_TILE = B_NMAJOR ? 32 * (BN + 8) : BN * 36;
    constexpr size_t lds_loop = (size_t)(2 * A_TILE + 2 * B_TILE) * sizeof(float);
    constexpr size_t lds_out = (size_t)(BM * (BN + 4) + BM) * sizeof(float);   // output staging + row offsets
    constexpr size_t lds = lds_loop > lds_out ? lds_loop : lds_out;
    constexpr auto kern = gather_conv_kernel<WM, WN, TM, TN, B_NMAJOR>;
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    dim3 grid((a.M + BM - 1) / BM, (a.CO + BN - 1) / BN, 1);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, a);
    return hipGetLastError();
}

hipError_t launch_gather_conv(hipStream_t stream, const GatherConvArgs &a0, int TH, int TW, int OHt, int OWt, int N)
{
    GatherConvArgs a = a0;
    a.M = N * OHt * OWt;
    a.K = TH * TW * a.AC;
    if (a.M <= 0 || a.CO <= 0) return hipSuccess;  // nothing to write
    a.a_sn = a.AH * a.AW * a.AC;
    a.d_AC = make_fastdiv(a.AC);
    a.d_TW = make_fastdiv(TW > 0 ? TW : 1);
    a.d_OWt = make_fastdiv(OWt);
    a.d_OHWt = make_fastdiv(OHt * OWt);
    const bool nmajor = (a.b_sn == 1);
    if (a.CO <= 32) {
        return nmajor ? launch_cfg<4, 1, 1, 1, true>(stream, a) : launch_cfg<4, 1, 1, 1, false>(stream, a);
    } else if (a.CO <= 64 || (a.CO % 128 != 0 && a.CO < 192)) {
        return nmajor ? launch_cfg<2, 2, 2, 1, true>(stream, a) : launch_cfg<2, 2, 2, 1, false>(stream, a);
    }
    return nmajor ? launch_cfg<2, 2, 2, 2, true>(stream, a) : launch_cfg<2, 2, 2, 2, false>(stream, a);
}

}  // namespace alpha
