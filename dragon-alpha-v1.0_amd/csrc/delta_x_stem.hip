// Backward-data for layers with 4 stored input channels and strides of 1 or 2 - the gradient with respect to the input
// of a network stem such as 7x7 stride 2 on RGB - fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950. Filter read as
// W[OC, FH, FW, 4] in place; no scratch.
//
// With 4 produced channels a GEMM tile over (pixel, channel) is almost empty. The sh*sw pixels of deltaX that share
// a "coarse" pixel (u, v) - ih = sh*u + a, iw = sw*v + b - read the same small window of deltaY, each through its own
// subset of the filter taps:
//   deltaX[n, sh*u + a, sw*v + b, ic] = sum over dh, dw, oc of deltaY[n, u + dh, v + dw, oc] * W[oc, fh(a, dh), fw(b, dw), ic]
//   fh(a, dh) = sh*(c_a - dh) + r_a,  c_a = (a + ph) / sh,  r_a = (a + ph) % sh   (a tap outside [0, FH) contributes zero)
// so the layer is ONE stride-1 convolution of deltaY over a DH x DW window (4 x 4 for 7x7 stride 2) into
// sh*sw*4 <= 16 columns = (a, b, ic), written depth-to-space. 16 columns are a full MFMA column block: rows = 16
// coarse pixels of a row, k = output channels.
//
// A workgroup (4 wavefronts) is persistent and walks blocks of RB x 16 coarse pixels. Wavefront w owns output
// channels 16w .. 16w+15 of the reduction for the WHOLE block and keeps its share of the filter in registers for the
// whole kernel (DH*DW float4: lane (l16, q) holds W[16w + 4q + s][tap][column l16], s = 0..3, 64 registers for a 4 x 4
// window) - read once from memory per workgroup, straight from W, so no packed copy of the filter is needed. The deltaY
// halo of a block ((RB+DH-1) x (16+DW-1) pixels x 64 channels) is staged in LDS; a lane's 128-bit read of pixel
// (R, l16 + dw), channels 16w + 4q .. +3, feeds the MFMAs of every block row that sees halo row R (up to DH of them)
// times 4 channel steps: 44 LDS reads per 512 MFMAs. The four wavefronts' partial sums are added through LDS in the
// order 0, 1, 2, 3 (the halo's memory, reused) and leave as 128-bit stores, the sw phases of 16 neighbouring coarse
// pixels forming contiguous runs. The next block's halo is requested into registers before the MFMA loop and written
// to LDS after it; loads and stores are unconditional (buffer descriptors; what must read as zero or must not be
// written gets an offset beyond the descriptor), so the only waits are the ones around the halo hand-over.
#include "common.hpp"

namespace alpha {

typedef float floatx4 __attribute__((ext_vector_type(4)));

struct DxStemArgs {
    const float *dY;   // [N][OH][OW][OC]
    const float *W;    // [OC][FH][FW][4]
    float *dX;         // [N][IH][IW][4]
    int N, OH, OW, OC, FH, FW, IH, IW;
    int sh, sw, lsw, nph;      // strides (1 or 2), log2(sw), sh*sw
    int dmin_h, dmin_w;        // first offset of the window
    int c_h[2], r_h[2], c_w[2], r_w[2];
    int nb_v, nb_uv, blocks;   // blocks per row of blocks, per image, in total
    FastDiv d_nbv, d_nbuv;
    Epilogue ep;
};

constexpr int DXS_RB_MAX = 8;      // coarse rows per block: 8, or 7 or 6 where that deals the blocks out more evenly
constexpr int DXS_PS = 72;         // floats per halo pixel: 64 channels + 8 (conflict-free 128-bit reads at 288 bytes)
constexpr int DXS_RS = 20;         // floats per pixel in the reduction buffer: 16 columns + 4
constexpr unsigned DXS_NEVER = 0x80000000u;   // beyond any descriptor of this kernel (tensors are below 2 GB)

template <int V> struct DxsInt { static constexpr int value = V; };
template <int I, int N, class F>
__device__ __forceinline__ void dxs_static_for(F &&f)
{
    if constexpr (I < N) {
        f(DxsInt<I>{});
        dxs_static_for<I + 1, N>(f);
    }
}

template <int DH, int DW, int RB>
__global__ __launch_bounds__(256, 2) void delta_x_stem_kernel(const DxStemArgs p)
{
    constexpr int HR = RB + DH - 1, HC = 16 + DW - 1, PS = DXS_PS, RS = DXS_RS;
    constexpr int NE = HR * HC * 16;              // float4 elements of a halo
    constexpr int NI = (NE + 255) / 256;          // per thread
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int t = threadIdx.x, lane = t & 63;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l16 = lane & 15, q = lane >> 4;

    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.dY), 0, p.N * p.OH * p.OW * p.OC * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.dX, 0, p.N * p.IH * p.IW * 16, 0x00020000);

    // ---- this wavefront's share of the filter -> registers, once ----------------------------------------------------
    floatx4 Bf[DH][DW];
    {
        const int phase = l16 >> 2, ic = l16 & 3;
        const int a = phase >> p.lsw, b = phase & (p.sw - 1);
        const bool col_ok = phase < p.nph;
        const int ca = a ? p.c_h[1] : p.c_h[0], ra = a ? p.r_h[1] : p.r_h[0];
        const int cb = b ? p.c_w[1] : p.c_w[0], rb = b ? p.r_w[1] : p.r_w[0];
        const int oc = 16 * w + 4 * q;
#pragma unroll
        for (int dh = 0; dh < DH; dh++)
#pragma unroll
            for (int dw = 0; dw < DW; dw++) {
                const int mh = ca - (p.dmin_h + dh), mw = cb - (p.dmin_w + dw);
                const int fh = p.sh * mh + ra, fw = p.sw * mw + rb;
                const bool ok = col_ok && mh >= 0 && mw >= 0 && fh < p.FH && fw < p.FW;
#pragma unroll
                for (int s = 0; s < 4; s++)
                    Bf[dh][dw][s] = (ok && oc + s < p.OC) ? p.W[(((oc + s) * p.FH + fh) * p.FW + fw) * 4 + ic] : 0.f;
            }
    }

    // ---- blocks of this workgroup: workgroups g = x (mod 8) share an XCD and take the contiguous range x of the blocks,
    // so that the halos neighbouring blocks share are served by that XCD's L2 ------------------------------------------
    const int G8 = gridDim.x >> 3;
    const int xcd = blockIdx.x & 7;
    int blk = (int)((long)p.blocks * xcd >> 3) + (blockIdx.x >> 3);
    const int blk_end = (int)((long)p.blocks * (xcd + 1) >> 3);

    floatx4 pf[NI];
    // requests the halo of block `b` (all zeros when b is past the end)
    auto request = [&](int b) {
        const bool live = b < blk_end;
        const int bb = live ? b : 0;
        const int n = fdiv(bb, p.d_nbuv);
        const int rem = bb - n * p.nb_uv;
        const int bu = fdiv(rem, p.d_nbv), bv = rem - bu * p.nb_v;
        const int oh0 = bu * RB + p.dmin_h, ow0 = bv * 16 + p.dmin_w;
        const int base = ((n * p.OH + oh0) * p.OW + ow0) * p.OC;   // may point before the image: only used where valid
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int e = t + 256 * i;
            const int px = e >> 4, c4 = e & 15;
            const int hr = px / HC, hc = px - hr * HC;
            const int oh = oh0 + hr, ow = ow0 + hc;
            const bool ok = live && (NE % 256 == 0 || e < NE) && (unsigned)oh < (unsigned)p.OH && (unsigned)ow < (unsigned)p.OW && 4 * c4 < p.OC;
            const unsigned off = ok ? (unsigned)((base + (hr * p.OW + hc) * p.OC + 4 * c4) * 4) : DXS_NEVER;
            pf[i] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(y_rsrc, off, 0, 0));
        }
    };
    auto deposit = [&]() {
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int e = t + 256 * i;
            if (NE % 256 == 0 || e < NE) *reinterpret_cast<floatx4 *>(smem + (e >> 4) * PS + 4 * (e & 15)) = pf[i];
        }
    };

    request(blk);
    deposit();                 // waits for the loads
    request(blk + G8);
    __syncthreads();

    const float *a_lane = smem + l16 * PS + 16 * w + 4 * q;
    constexpr int NJ = (RB * 16 * 4 + 255) / 256;   // float4 results per thread, at most (4 phases)

    for (; blk < blk_end; blk += G8) {
        floatx4 acc[RB];
#pragma unroll
        for (int i = 0; i < RB; i++) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};

        // ---- halo rows R, window columns dw: one read serves every block row R - dh ------------------------------------
        floatx4 a[2];
        a[0] = *reinterpret_cast<const floatx4 *>(a_lane);
        dxs_static_for<0, HR * DW>([&](auto step) {
            constexpr int idx = decltype(step)::value;
            constexpr int R = idx / DW, dw = idx % DW;
            if constexpr (idx + 1 < HR * DW) {
                constexpr int R1 = (idx + 1) / DW, dw1 = (idx + 1) % DW;
                a[(idx + 1) & 1] = *reinterpret_cast<const floatx4 *>(a_lane + (R1 * HC + dw1) * PS);
            }
#pragma unroll
            for (int s = 0; s < 4; s++)
#pragma unroll
                for (int dh = 0; dh < DH; dh++) {
                    const int tile = R - dh;
                    if (tile >= 0 && tile < RB)
                        acc[tile] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[idx & 1][s], Bf[dh][dw][s], acc[tile], 0, 0, 0);
                }
        });
        __syncthreads();       // everyone has finished reading the halo

        // ---- partial sums of the four wavefronts through LDS (the halo's memory) --------------------------------------
#pragma unroll
        for (int i = 0; i < RB; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) smem[((w * RB + i) * 16 + 4 * q + r) * RS + l16] = acc[i][r];
        __syncthreads();

        const int n = fdiv(blk, p.d_nbuv);
        const int rem = blk - n * p.nb_uv;
        const int bu = fdiv(rem, p.d_nbv), bv = rem - bu * p.nb_v;
        floatx4 out[NJ];
        unsigned out_off[NJ];
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            // consecutive threads: b, then the 16 pixels of the row (a contiguous run of deltaX), then a, then the block row
            const int idx = t + 256 * j;
            const int b = idx & (p.sw - 1);
            const int px = (idx >> p.lsw) & 15;
            const int rest = idx >> (p.lsw + 4);
            const int a_ = rest & (p.sh - 1), tile = rest >> (p.sh - 1);
            const bool in = tile < RB;
            const int tl = in ? tile : 0;
            const float *src = smem + (tl * 16 + px) * RS + 4 * (a_ * p.sw + b);
            floatx4 v = *reinterpret_cast<const floatx4 *>(src);
#pragma unroll
            for (int ww = 1; ww < 4; ww++) v += *reinterpret_cast<const floatx4 *>(src + ww * RB * 16 * RS);
            const int ih = p.sh * (bu * RB + tl) + a_, iw = p.sw * (bv * 16 + px) + b;
            const bool ok = in && ih < p.IH && iw < p.IW;
            const int elem = ((n * p.IH + ih) * p.IW + iw) * 4;
            if (p.ep.fused && ok) {
                const float4 r4 = epilogue4(make_float4(v[0], v[1], v[2], v[3]), p.ep, 0, (size_t)elem);
                v = floatx4{r4.x, r4.y, r4.z, r4.w};
            }
            out[j] = v;
            out_off[j] = ok ? (unsigned)(elem * 4) : DXS_NEVER;
        }
        __syncthreads();       // the sums have been read

        deposit();             // next block's halo (requested before the MFMA loop) -> LDS
#pragma unroll
        for (int j = 0; j < NJ; j++)
            buffer_store_b128_guarded<2>(out[j], x_rsrc, out_off[j], 0);   // non-temporal: streamed out
        request(blk + 2 * G8);
        __syncthreads();
    }
}

template <auto K> struct DxsKernel { static constexpr auto value = K; };

// deltaX[N, IH, IW, 4] from deltaY[N, OH, OW, OC] and W[OC, FH, FW, 4]. Returns hipErrorNotSupported (nothing launched)
// when the layer does not fit: IC != 4, a stride above 2, OC above 64 or not a multiple of 4, a window above 4 x 4.
hipError_t launch_delta_x_stem(hipStream_t stream, const float *dY, const float *W, float *dX, int N, int IH, int IW, int IC,
                               int OH, int OW, int OC, int FH, int FW, int sh, int sw, int ph, int pw, const Epilogue *ep)
{
    if (IC != 4 || sh < 1 || sh > 2 || sw < 1 || sw > 2 || OC < 4 || OC > 64 || (OC & 3)) return hipErrorNotSupported;
    if ((size_t)N * OH * OW * OC * 4 >= (1ull << 31) || (size_t)N * IH * IW * 16 >= (1ull << 31)) return hipErrorNotSupported;
    DxStemArgs a{};
    a.dY = dY; a.W = W; a.dX = dX; a.ep = ep ? *ep : bias_epilogue(nullptr);
    a.N = N; a.OH = OH; a.OW = OW; a.OC = OC; a.FH = FH; a.FW = FW; a.IH = IH; a.IW = IW;
    a.sh = sh; a.sw = sw; a.lsw = sw - 1; a.nph = sh * sw;
    // window of deltaY offsets per axis: phase a reads offsets c_a - m for the taps f = s*m + r_a < F
    auto axis = [](int s, int pad, int F, int *c, int *r, int &dmin, int &dmax) {
        bool any = false;
        for (int x = 0; x < 2; x++) {
            const int xx = x < s ? x : 0;
            c[x] = (xx + pad) / s; r[x] = (xx + pad) % s;
            if (x >= s || F <= r[x]) continue;
            const int M = (F - r[x] + s - 1) / s;
            const int lo = c[x] - M + 1, hi = c[x];
            if (!any || lo < dmin) dmin = lo;
            if (!any || hi > dmax) dmax = hi;
            any = true;
        }
        return any;
    };
    int hmin = 0, hmax = 0, wmin = 0, wmax = 0;
    if (!axis(sh, ph, FH, a.c_h, a.r_h, hmin, hmax) || !axis(sw, pw, FW, a.c_w, a.r_w, wmin, wmax)) return hipErrorNotSupported;
    const int DH = hmax - hmin + 1, DW = wmax - wmin + 1;
    if (DH > 4 || DW > 4) return hipErrorNotSupported;
    a.dmin_h = hmin; a.dmin_w = wmin;
    const int U = (IH + sh - 1) / sh, V = (IW + sw - 1) / sw;
    const int cus = device_cu_count();
    if (cus < 1) return hipErrorNotSupported;
    int grid = 2 * cus;
    grid = (grid + 7) / 8 * 8;               // whole groups of 8: workgroup g runs on XCD g % 8
    a.nb_v = (V + 15) / 16;
    // Rows per block: a workgroup's blocks cost whole rounds, so the block height that wastes the least of the last round
    // wins (a block of RB rows costs about RB + 1: its halo has DH - 1 more rows to stage and its hand-over is fixed).
    // 112 x 112 coarse pixels at N = 64 on 512 workgroups: 6272 blocks of 8 rows are 12.25 rounds (13 x 9 = 117), 7168
    // blocks of 7 rows are 14 (14 x 8 = 112).
    int RB = DXS_RB_MAX;
    long best = -1;
    for (int rb = DXS_RB_MAX; rb >= 6; rb--) {
        const long blocks = (long)N * ((U + rb - 1) / rb) * a.nb_v;
        const long cost = ((blocks + grid - 1) / grid) * (rb + 1);
        if (best < 0 || cost < best) { best = cost; RB = rb; }
    }
    const int nb_u = (U + RB - 1) / RB;
    a.nb_uv = nb_u * a.nb_v;
    if ((long)N * a.nb_uv >= (1l << 30)) return hipErrorNotSupported;
    a.blocks = N * a.nb_uv;
    a.d_nbv = make_fastdiv(a.nb_v);
    a.d_nbuv = make_fastdiv(a.nb_uv);
    const bool small = DH <= 2 && DW <= 2;
    const int HR = RB + (small ? 2 : 4) - 1, HC = 16 + (small ? 2 : 4) - 1;
    size_t lds = (size_t)HR * HC * DXS_PS * sizeof(float);
    const size_t red = (size_t)4 * RB * 16 * DXS_RS * sizeof(float);
    if (lds < red) lds = red;
    auto go = [&](auto kern) -> hipError_t {
        if (hipError_t e = ensure_dynamic_lds<decltype(kern)::value>(lds); e != hipSuccess) return e;
        hipLaunchKernelGGL(decltype(kern)::value, dim3(grid), dim3(256), lds, stream, a);
        return hipGetLastError();
    };
    if (small) {
        if (RB == 8) return go(DxsKernel<delta_x_stem_kernel<2, 2, 8>>{});
        if (RB == 7) return go(DxsKernel<delta_x_stem_kernel<2, 2, 7>>{});
        return go(DxsKernel<delta_x_stem_kernel<2, 2, 6>>{});
    }
    if (RB == 8) return go(DxsKernel<delta_x_stem_kernel<4, 4, 8>>{});
    if (RB == 7) return go(DxsKernel<delta_x_stem_kernel<4, 4, 7>>{});
    return go(DxsKernel<delta_x_stem_kernel<4, 4, 6>>{});
}

}  // namespace alpha
