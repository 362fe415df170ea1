// Backward-filter for 4 stored input channels (the first layer of a network: 3 colour channels stored as 4), any filter
// up to 128 taps, any stride and padding; fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950, operands straight from memory.
//
//   deltaW[oc, fh, fw, c] = sum over pixels k = (n, oh, ow) of deltaY[k, oc] * X[n, oh*sh - ph + fh, ow*sw - pw + fw, c]
//
// With IC = 4 the 64 x 64 (oc, ic) blocks of delta_w_stream.hip are one sixteenth full, and the generic kernel spends its
// time on im2col addresses (7x7 stride 2 on 64x224x224: 0.35 ms, three times the forward kernel). Here the 16 columns of
// an MFMA operand are 16 TAPS: lane (l16, q) loads
//   ya = deltaY[n, oh, 4g + q][oc0 + 4*l16 .. +3]      xa = X[n, oh*sh - ph + fh_t, (4g + q)*sw - pw + fw_t][0 .. 3]
// for tap t = 16 * (tap group) + l16, and MFMA (i, j) multiplies component i of ya (output channels oc0 + 4*l16 + i) with
// component j of xa (channel j of the 16 taps): 16 MFMAs per group of four pixels and tap group give a 64 x (16 taps x 4
// channels) block of deltaW. The reduction index of the MFMA is the pixel, as in delta_w_stream.hip, and so are the ring of
// D groups in registers and the descriptor per output row of deltaY; X is addressed through a descriptor per image with
// an offset per lane (rows above and below the image fall outside it, columns left and right are tested per lane).
//
// Work: (slice z of the pixels) x (set s of tap groups) x (block of 64 output channels), one workgroup each; the slices
// are this kernel's own equal cut of the pixel groups into GridZ parts - the caller only adds deltaW and the buffers up
// (dW/A.cu:66-76) -, slice 0 goes to deltaW, slice z to deltaW_buf[z - 1]. In a workgroup the eight wavefronts are
// (tap groups of the set) x (equal parts of the slice); the parts' accumulators are added through LDS in the order of
// their numbers: no atomics, bit-identical results from run to run.
#include "common.hpp"

namespace alpha {

struct DwStemArgs {
    const float *X;    // [N, IH, IW, 4]
    const float *dY;   // [N, OH, OW, OC]
    float *dW;         // [OC, FH, FW, 4]
    float *dW_buf;     // [GZ - 1][OC, FH, FW, 4]
    int IH, IW, OH, OW, OC, FH, FW;
    int sh, sw, ph, pw;
    int GZ, taps;
    int TGW;           // tap groups per workgroup: 1, 2, 4 or 8
    int S, OCB;        // sets of TGW tap groups, blocks of 64 output channels
    int GPR;           // pixel groups (4 pixels) per output row = ceil(OW / 4)
    int TG;            // pixel groups in all = N * OH * GPR
    FastDiv d_OH, d_GPR, d_FW, d_S, d_OCB;
};

template <int D>
__global__ __launch_bounds__(512, 1) void delta_w_stem_kernel(const DwStemArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float dwm_smem[];   // [8 wavefronts][16 units][64 lanes] float4
    floatx4 *part = reinterpret_cast<floatx4 *>(dwm_smem);
    const int t = threadIdx.x, lane = t & 63;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l16 = lane & 15, q = lane >> 4;
    // blockIdx = (z * S + s) * OCB + ocb
    const int zs = fdiv((int)blockIdx.x, p.d_OCB), ocb = (int)blockIdx.x - zs * p.OCB;
    const int z = fdiv(zs, p.d_S), s = zs - z * p.S;
    const int PP = 8 / p.TGW;                         // parts of the slice per tap group
    const int tg = w & (p.TGW - 1), pp = w / p.TGW;   // this wavefront's tap group within the set, and its part
    const int tap = (s * p.TGW + tg) * 16 + l16;
    const bool tap_ok = tap < p.taps;
    const int fh = fdiv(tap_ok ? tap : 0, p.d_FW), fw = (tap_ok ? tap : 0) - fh * p.FW;

    const int OW = p.OW, OH = p.OH, GPR = p.GPR;
    constexpr unsigned NEVER = 0x80000000u;   // beyond every descriptor
    const int oc_l = 64 * ocb + 4 * l16;
    const unsigned y_lane = oc_l < p.OC ? (unsigned)((q * p.OC + oc_l) * 4) : NEVER;
    const int y_gstride = 16 * p.OC, x_gstride = 4 * p.sw * 16;   // bytes per pixel group
    const size_t y_row_bytes = (size_t)OW * p.OC * 4, x_img_bytes = (size_t)p.IH * p.IW * 16;

    // ---- this wavefront's run of pixel groups: part pp of slice z -------------------------------------------------------
    const int lo = (int)((long)p.TG * z / p.GZ), hi = (int)((long)p.TG * (z + 1) / p.GZ);
    const int g_lo = __builtin_amdgcn_readfirstlane(lo + (int)((long)(hi - lo) * pp / PP));
    const int g_hi = __builtin_amdgcn_readfirstlane(lo + (int)((long)(hi - lo) * (pp + 1) / PP));
    const int total = g_hi - g_lo;

    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    // ---- load cursor: the output row being requested (scalar), its descriptors, the group within it; per lane the column
    //      of X under this lane's tap and pixel, and the byte offset of that element in the image -----------------------
    __amdgpu_buffer_rsrc_t y_rsrc, x_rsrc;
    const int gr0 = fdiv(g_lo, p.d_GPR);   // global output row n * OH + oh
    int cur_g = g_lo - gr0 * GPR, left = total;
    const int n0 = fdiv(gr0, p.d_OH);
    int oh = gr0 - n0 * OH;
    const char *y_row = reinterpret_cast<const char *>(p.dY) + (size_t)gr0 * y_row_bytes;
    const char *x_img = reinterpret_cast<const char *>(p.X) + (size_t)n0 * x_img_bytes;
    int y_goff = 0;
    int iw_l = (4 * cur_g + q) * p.sw - p.pw + fw;
    unsigned x_off = (unsigned)(((oh * p.sh - p.ph + fh) * p.IW + iw_l) * 16);   // "negative" above the image: outside the descriptor
    const int row_back = GPR * 4 * p.sw;                                          // columns a finished row has moved on
    const unsigned x_next_row = (unsigned)((p.sh * p.IW - row_back) * 16), x_next_img = (unsigned)(-(OH * p.sh * p.IW) * 16);
    auto setup_row = [&]() {   // descriptors of row (n, oh) and of image n; `left` <= 0: nothing more to read, empty descriptors
        const bool live = left > 0;
        y_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(y_row), 0, live ? (int)y_row_bytes : 0, 0x00020000);
        x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(x_img), 0, live ? (int)x_img_bytes : 0, 0x00020000);
        y_goff = cur_g * y_gstride;
    };
    floatx4 ya[D], xa[D];
    auto load = [&](int d) {
        const bool col_ok = tap_ok && (unsigned)iw_l < (unsigned)p.IW;
        ya[d] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(y_rsrc, y_lane + (unsigned)y_goff, 0, 0));
        xa[d] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, col_ok ? x_off : NEVER, 0, 0));
        // on to the next group; the next row when this one is done (uniform)
        cur_g++;
        left--;
        y_goff += y_gstride;
        x_off += (unsigned)x_gstride;
        iw_l += 4 * p.sw;
        if (cur_g == GPR) {
            cur_g = 0;
            y_row += y_row_bytes;
            x_off += x_next_row;
            iw_l -= row_back;
            oh++;
            if (oh == OH) {
                oh = 0;
                x_img += x_img_bytes;
                x_off += x_next_img;
            }
            setup_row();
        }
    };
    auto multiply = [&](int d) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ya[d][i], xa[d][j], acc[i][j], 0, 0, 0);
    };
    if (total > 0) {
        setup_row();
#pragma unroll
        for (int d = 0; d < D; d++) load(d);   // groups past the end read through empty descriptors: zeros, never multiplied
        int g = 0;
        for (; g + D <= total; g += D) {
#pragma unroll
            for (int d = 0; d < D; d++) {
                multiply(d);
                load(d);
                __builtin_amdgcn_sched_barrier(0);   // keeps the refill next to its slot
            }
        }
        const int rest = total - g;   // < D groups, already in slots 0 .. rest-1
#pragma unroll
        for (int d = 0; d < D - 1; d++)
            if (d < rest) multiply(d);
    }

    // ---- the parts of a tap group added in the order 0, 1, 2, ...; unit u = 4 i + rr is one 128-bit store per lane:
    // acc[i][j][rr] = deltaW[oc = 64 ocb + 4 (4q + rr) + i][tap][c = j] ----------------------------------------------------
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int rr = 0; rr < 4; rr++)
            part[(w * 16 + 4 * i + rr) * 64 + lane] = floatx4{acc[i][0][rr], acc[i][1][rr], acc[i][2][rr], acc[i][3][rr]};
    __syncthreads();
    const size_t sizeW = (size_t)p.OC * p.taps * 4;
    float *dst = z == 0 ? p.dW : p.dW_buf + (size_t)(z - 1) * sizeW;
    for (int u = pp; u < 16; u += PP) {   // uniform: the PP wavefronts of a tap group take every PP-th unit
        const int i = u >> 2, rr = u & 3;
        floatx4 v = part[(tg * 16 + u) * 64 + lane];   // wavefront x = part * TGW + tap group
        for (int x = 1; x < PP; x++) v += part[((x * p.TGW + tg) * 16 + u) * 64 + lane];
        const int oc = ocb * 64 + 4 * (4 * q + rr) + i;
        if (tap_ok && oc < p.OC)
            *reinterpret_cast<float4 *>(dst + ((size_t)oc * p.taps + tap) * 4) = make_float4(v[0], v[1], v[2], v[3]);
    }
}

// Returns hipErrorNotSupported (nothing launched) when the layer does not fit: more than 128 taps, images of X of 2 GB,
// rows beyond the 32-bit offsets; the caller then uses another kernel.
hipError_t launch_deltaW_stem(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                              int N, int IH, int IW, int OH, int OW, int OC, int FH, int FW, int sh, int sw, int ph, int pw, int GZ)
{
    if ((OC & 3) || OC < 4 || FH < 1 || FW < 1 || FH * FW > 128 || sh < 1 || sw < 1 || GZ < 1 || N < 1) return hipErrorNotSupported;
    if (GZ > 1 && dW_buf == nullptr) return hipErrorNotSupported;
    // every output pixel's window inside the padded input (a smaller output than the formula's is fine)
    if ((long)(OH - 1) * sh + FH > (long)IH + 2 * ph || (long)(OW - 1) * sw + FW > (long)IW + 2 * pw) return hipErrorNotSupported;
    // 32-bit byte offsets: within a row of deltaY, within an image of X (with the window's overhang on every side)
    if ((long)(OW + 4) * OC * 4 >= (1L << 30)) return hipErrorNotSupported;
    if (((long)(IH + (long)OH * sh + FH + ph) * IW + (long)(OW + 4) * sw + FW + pw) * 16 >= (1L << 31)) return hipErrorNotSupported;
    const int cus = device_cu_count();
    if (cus < 1) return hipErrorNotSupported;
    DwStemArgs a{};
    a.X = X; a.dY = dY; a.dW = dW; a.dW_buf = dW_buf;
    a.IH = IH; a.IW = IW; a.OH = OH; a.OW = OW; a.OC = OC; a.FH = FH; a.FW = FW;
    a.sh = sh; a.sw = sw; a.ph = ph; a.pw = pw;
    a.GZ = GZ;
    a.taps = FH * FW;
    a.OCB = (OC + 63) / 64;
    a.GPR = (OW + 3) / 4;
    const long TG = (long)N * OH * a.GPR;
    if (TG >= (1L << 30) || (long)GZ * 8 * a.OCB >= (1L << 30)) return hipErrorNotSupported;
    a.TG = (int)TG;
    // As many tap groups per workgroup (they share the rows of deltaY in L1) as still leave a workgroup per compute unit
    const int tgn = (a.taps + 15) / 16;   // 1 .. 8
    int tgw = 1;
    while (tgw < tgn) tgw *= 2;
    while (tgw > 1 && (long)GZ * ((tgn + tgw - 1) / tgw) * a.OCB < cus) tgw /= 2;
    a.TGW = tgw;
    a.S = (tgn + tgw - 1) / tgw;
    a.d_OH = make_fastdiv(OH);
    a.d_GPR = make_fastdiv(a.GPR);
    a.d_FW = make_fastdiv(FW);
    a.d_S = make_fastdiv(a.S);
    a.d_OCB = make_fastdiv(a.OCB);
    constexpr auto kern = delta_w_stem_kernel<6>;
    const size_t lds = (size_t)8 * 16 * 64 * sizeof(floatx4);
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)(GZ * a.S * a.OCB)), dim3(512), lds, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
