// Backward-filter for stride-1 layers by streaming output rows, fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950.
//
//   deltaW[oc, fh, fw, ic] = sum over pixels k = (n, oh, ow) of the K slice of  deltaY[k, oc] * X[n, oh-ph+fh, ow-pw+fw, ic]
//
// A workgroup (4 wavefronts) owns one K slice (blockIdx.z, the reference's partition), OCB = 16*OCT output
// channels and 64 input channels, for ALL filter taps. It walks the output rows of its slice; per row it holds in
// LDS the deltaY row (double buffered) and the FH input rows that row touches (a ring of FH+1 row slots, so the
// one new input row of the next output row is fetched while the current row is being multiplied). Both operands
// are read from LDS 32 bits at a time, lanes across channels (the reduction index of this GEMM is the pixel,
// which is the slow axis of both tensors). Wavefront w owns input channels [16w, 16w+16): per 4 pixels it
// reads OCT deltaY fragments and FH*FW shifted X fragments and issues OCT*FH*FW MFMAs, so each X element read
// from memory is used for every tap it participates in and every deltaY element for all FH*FW taps.
// Pixels outside the K slice (a slice may begin or end inside a row) are staged as zeros. No atomics: slice z
// stores to deltaW (z = 0) or deltaW_buf[z-1]; a fixed launch gives bit-identical results.
//
// LDS strides: 32-bit reads of 64 lanes are conflict-free when the four 16-lane groups (consecutive pixels) start
// 16 banks apart: row strides are 16 or 48 floats modulo 64 (X: 80; deltaY: 48 for 32 channels, 80 for 64).
#include "common.hpp"

namespace alpha {

struct DwRowsArgs {
    const float *X;
    const float *dY;
    float *dW;
    float *dW_buf;
    int N, IH, IW, IC, OH, OW, OC;
    int ph, pw;
    int GK, GK_slice, GZ;
    int OWp;   // OW rounded up to a multiple of 4 (pixels beyond OW are staged as zeros)
    int PW;    // OWp + FW - 1 input columns staged per row; staged column cp holds iw = cp - pw
    FastDiv d_OW, d_OH;
};

constexpr int DWR_XS = 80;   // X row slot pixel stride (floats): 64 channels + 16

template <int FH, int FW, int OCT>
__global__ __launch_bounds__(256, 1) void delta_w_rows_kernel(const DwRowsArgs p)
{
    constexpr int OCB = 16 * OCT;
    constexpr int YS = OCB + 16;             // 48 or 80: both 16 or 48 modulo 64
    constexpr int YQ = OCT;                  // float4 per thread per deltaY row   (OWp <= 64, host-checked)
    constexpr int XQ = 4;                    // float4 per thread per X row        (PW*16 <= 1024, host-checked)
    constexpr int SLOTS = FH + 1;

    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *Ybuf = smem;                               // [2][OWp][YS]
    float *Xring = smem + 2 * p.OWp * YS;             // [SLOTS][PW][DWR_XS]
    const int ybuf_floats = p.OWp * YS, slot_floats = p.PW * DWR_XS;

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int ic0 = blockIdx.x * 64, oc0 = blockIdx.y * OCB, z = blockIdx.z;
    const int OW = p.OW, OH = p.OH;

    const int k_start = p.GK_slice * z;
    const int k_end = (z != p.GZ - 1) ? k_start + p.GK_slice : p.GK;
    float *dst = (z == 0) ? p.dW : p.dW_buf + (size_t)(z - 1) * p.OC * (FH * FW) * p.IC;

    floatx4 acc[FH][FW][OCT];
#pragma unroll
    for (int a = 0; a < FH; a++)
#pragma unroll
        for (int b = 0; b < FW; b++)
#pragma unroll
            for (int c = 0; c < OCT; c++) acc[a][b][c] = floatx4{0.f, 0.f, 0.f, 0.f};

    // ---- staging helpers (loads from clamped addresses, zeroing applied when the registers are stored) ----------
    float4 yreg[YQ], xreg[XQ];
    unsigned ymask = 0, xmask = 0;
    const int y_quads = p.OWp * (OCB / 4), x_quads = p.PW * 16;

    auto load_y = [&](int gr) {   // deltaY row gr (global output row n*OH + oh)
        ymask = 0;
#pragma unroll
        for (int u = 0; u < YQ; u++) {
            const int idx = t + 256 * u;
            const int ow = idx / (OCB / 4), cq = (idx % (OCB / 4)) * 4;
            const int k = gr * OW + ow;
            const bool ok = idx < y_quads && ow < OW && k >= k_start && k < k_end && oc0 + cq < p.OC;
            yreg[u] = *reinterpret_cast<const float4 *>(p.dY + (((size_t)k * p.OC + oc0 + cq) & (size_t)(-(long)ok)));
            ymask |= (unsigned)ok << u;
        }
    };
    auto store_y = [&](int buf) {
#pragma unroll
        for (int u = 0; u < YQ; u++) {
            const int idx = t + 256 * u;
            if (idx < y_quads) {
                const int ow = idx / (OCB / 4), cq = (idx % (OCB / 4)) * 4;
                const bool ok = (ymask >> u) & 1u;
                *reinterpret_cast<float4 *>(Ybuf + buf * ybuf_floats + ow * YS + cq) =
                    make_float4(ok ? yreg[u].x : 0.f, ok ? yreg[u].y : 0.f, ok ? yreg[u].z : 0.f, ok ? yreg[u].w : 0.f);
            }
        }
    };
    auto load_x = [&](int n, int ih) {   // input row (n, ih); rows outside the image become zeros
        xmask = 0;
        const bool rowv = (unsigned)ih < (unsigned)p.IH;
#pragma unroll
        for (int u = 0; u < XQ; u++) {
            const int idx = t + 256 * u;
            const int cp = idx >> 4, cq = (idx & 15) * 4;
            const int iw = cp - p.pw;
            const bool ok = rowv && idx < x_quads && (unsigned)iw < (unsigned)p.IW && ic0 + cq < p.IC;
            const int off = (((n * p.IH + ih) * p.IW + iw) * p.IC + ic0 + cq) & -(int)ok;
            xreg[u] = *reinterpret_cast<const float4 *>(p.X + off);
            xmask |= (unsigned)ok << u;
        }
    };
    auto store_x = [&](int slot) {
#pragma unroll
        for (int u = 0; u < XQ; u++) {
            const int idx = t + 256 * u;
            if (idx < x_quads) {
                const bool ok = (xmask >> u) & 1u;
                *reinterpret_cast<float4 *>(Xring + slot * slot_floats + (idx >> 4) * DWR_XS + (idx & 15) * 4) =
                    make_float4(ok ? xreg[u].x : 0.f, ok ? xreg[u].y : 0.f, ok ? xreg[u].z : 0.f, ok ? xreg[u].w : 0.f);
            }
        }
    };
    // all FH input rows of output row (n, oh), fetched synchronously (first row of the slice / of an image)
    auto stage_window = [&](int n, int oh) {
#pragma unroll
        for (int fh = 0; fh < FH; fh++) {
            load_x(n, oh - p.ph + fh);
            store_x((oh + fh) % SLOTS);
        }
    };

    if (k_start < k_end) {
        const int gr_first = fdiv(k_start, p.d_OW), gr_last = fdiv(k_end - 1, p.d_OW);
        int n = fdiv(gr_first, p.d_OH), oh = gr_first - n * OH;
        load_y(gr_first);
        store_y(0);
        stage_window(n, oh);
        __syncthreads();

        const int steps = p.OWp >> 2;
        for (int gr = gr_first, it = 0; gr <= gr_last; gr++, it++) {
            const bool has_next = gr < gr_last;
            int n2 = n, oh2 = oh + 1;
            if (oh2 == OH) { oh2 = 0; n2 = n + 1; }
            const bool same_image = n2 == n;
            if (has_next) {
                load_y(gr + 1);
                if (same_image) load_x(n, oh2 - p.ph + FH - 1);
            }

            // ---- multiply this row: pixels in groups of 4 (lane group q takes pixel 4*k4 + q) ---------------------
            const float *yb = Ybuf + (it & 1) * ybuf_floats + q * YS + l16;
            const float *xb[FH];
#pragma unroll
            for (int fh = 0; fh < FH; fh++) xb[fh] = Xring + ((oh + fh) % SLOTS) * slot_floats + q * DWR_XS + 16 * w + l16;

            float a0[OCT], b0[FH][FW], a1[OCT], b1[FH][FW];
            auto frags = [&](int k4, float (&a)[OCT], float (&b)[FH][FW]) {
#pragma unroll
                for (int c = 0; c < OCT; c++) a[c] = yb[k4 * 4 * YS + 16 * c];
#pragma unroll
                for (int fh = 0; fh < FH; fh++)
#pragma unroll
                    for (int fw = 0; fw < FW; fw++) b[fh][fw] = xb[fh][(k4 * 4 + fw) * DWR_XS];
            };
            auto mfmas = [&](const float (&a)[OCT], const float (&b)[FH][FW]) {
#pragma unroll
                for (int fh = 0; fh < FH; fh++)
#pragma unroll
                    for (int fw = 0; fw < FW; fw++)
#pragma unroll
                        for (int c = 0; c < OCT; c++)
                            acc[fh][fw][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[c], b[fh][fw], acc[fh][fw][c], 0, 0, 0);
            };
            frags(0, a0, b0);
            for (int k4 = 0; k4 < steps; k4 += 2) {
                if (k4 + 1 < steps) frags(k4 + 1, a1, b1);
                mfmas(a0, b0);
                if (k4 + 1 < steps) {
                    if (k4 + 2 < steps) frags(k4 + 2, a0, b0);
                    mfmas(a1, b1);
                }
            }

            if (has_next) {
                store_y((it + 1) & 1);
                if (same_image) store_x((oh2 + FH - 1) % SLOTS);
            }
            __syncthreads();
            if (has_next && !same_image) {   // first row of the next image: its whole window is new
                stage_window(n2, oh2);
                __syncthreads();
            }
            n = n2;
            oh = oh2;
        }
    }

    // ---- store: lane holds input channel ic0 + 16w + l16 and output channels 16c + 4q + r --------------------------
    const int ic = ic0 + 16 * w + l16;
#pragma unroll
    for (int fh = 0; fh < FH; fh++)
#pragma unroll
        for (int fw = 0; fw < FW; fw++)
#pragma unroll
            for (int c = 0; c < OCT; c++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int oc = oc0 + 16 * c + 4 * q + r;
                    if (oc < p.OC && ic < p.IC) dst[(((size_t)oc * FH + fh) * FW + fw) * p.IC + ic] = acc[fh][fw][c][r];
                }
}

template <int FH, int FW, int OCT>
static hipError_t launch_dwr(hipStream_t stream, const DwRowsArgs &a)
{
    constexpr int OCB = 16 * OCT, YS = OCB + 16;
    if (a.OWp > 64 || a.PW * 16 > 1024) return hipErrorNotSupported;
    const size_t lds = ((size_t)2 * a.OWp * YS + (size_t)(FH + 1) * a.PW * DWR_XS) * sizeof(float);
    if (lds > 160 * 1024) return hipErrorNotSupported;
    auto kern = delta_w_rows_kernel<FH, FW, OCT>;
    static size_t configured = 0;
    if (lds > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        configured = lds;
    }
    dim3 grid((a.IC + 63) / 64, (a.OC + OCB - 1) / OCB, a.GZ);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, a);
    return hipGetLastError();
}

// Returns hipErrorNotSupported (nothing launched) when the layer does not fit; the caller then uses the generic kernel.
hipError_t launch_deltaW_rows(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                              int N, int IH, int IW, int IC, int OH, int OW, int OC, int FH, int FW,
                              int sh, int sw, int ph, int pw, int GK_slice, int GZ)
{
    if (sh != 1 || sw != 1) return hipErrorNotSupported;
    if (OH != IH + 2 * ph - FH + 1 || OW != IW + 2 * pw - FW + 1) return hipErrorNotSupported;
    if (IC < 16 || OC < 16) return hipErrorNotSupported;
    DwRowsArgs a{};
    a.X = X; a.dY = dY; a.dW = dW; a.dW_buf = dW_buf;
    a.N = N; a.IH = IH; a.IW = IW; a.IC = IC; a.OH = OH; a.OW = OW; a.OC = OC;
    a.ph = ph; a.pw = pw;
    a.GK = N * OH * OW; a.GK_slice = GK_slice; a.GZ = GZ;
    a.OWp = (OW + 3) & ~3;
    a.PW = a.OWp + FW - 1;
    a.d_OW = make_fastdiv(OW);
    a.d_OH = make_fastdiv(OH);
    if (FH == 3 && FW == 3) return launch_dwr<3, 3, 2>(stream, a);
    if (FH == 1 && FW == 1) return launch_dwr<1, 1, 4>(stream, a);
    return hipErrorNotSupported;
}

}  // namespace alpha
