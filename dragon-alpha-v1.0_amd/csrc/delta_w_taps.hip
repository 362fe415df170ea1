// Backward-filter with one filter tap per workgroup, operands straight from memory, fp32 MFMA
// v_mfma_f32_16x16x4_f32, gfx950. Any filter size, stride and padding.
//
//   deltaW[oc, fh, fw, ic] = sum over pixels k = (n, oh, ow) of the K slice of
//                            deltaY[k, oc] * X[n, oh*sh - ph + fh, ow*sw - pw + fw, ic]
//
// Why: the split-K factor GridZ comes from the caller (the Java engine sizes it for at most 128 multiprocessors), so on
// small feature maps a kernel that keeps all taps of a tile in one workgroup launches fewer workgroups than the device
// has compute units (8x8x256->256 at GridZ 3: 192). With the tap in the grid - as the reference does for its small-map
// kernels (dconv3d_dW_GemmV2SK_kernel.cuh:17-24, gridDim.z = GZ*FH*FW) - the same layer gives 432.
//
// A workgroup owns one tap, one 64 x 64 block of (output channel, input channel) and one K slice; its KS wavefronts
// split the slice's output rows (each takes an equal contiguous share of its pixel groups) and their accumulators are added
// through LDS in the order 0, 1, 2, ... - no atomics, a fixed (shape, GridZ) gives bit-identical results.
//
// The reduction index is the pixel, the slow axis of both tensors, and a lane's natural 128-bit load brings 4 CHANNELS
// of one pixel. Rows and columns are therefore interleaved over 16 MFMAs: lane (l16, q) loads
//   ya = deltaY[n, oh, 4g + q][oc0 + 4*l16 .. +3]      xa = X[n, ih, (4g + q)*sw + fw - pw][ic0 + 4*l16 .. +3]
// and MFMA (i, j) multiplies component i of ya with component j of xa: rows = output channels oc0 + 4*l16 + i, columns =
// input channels ic0 + 4*l16 + j, k = the four pixels of group g of the row. Two 256-byte-coalesced loads feed 16 MFMAs;
// nothing is staged in LDS and nothing synchronises inside the loop; a ring of D pixel groups in registers hides the
// latency. The nine workgroups that read the same rows (shifted by their taps) run side by side on one XCD, so the
// re-reads are served by that XCD's L2.
//
// Everything that must read as zero does so through the buffer descriptors, which are rebuilt (scalar instructions) for
// every row: the deltaY descriptor covers exactly the row's pixels that lie inside the K slice and the image row, the X
// descriptor exactly input row ih (no bytes at all when ih is a padding row); a lane's offset that falls outside -
// padding columns on either side, pixels past the end of the row, channels past the last - returns zeros.
#include "common.hpp"

namespace alpha {

struct DwTapsArgs {
    const float *X;
    const float *dY;
    float *dW;
    float *dW_buf;
    int IH, IW, IC, OH, OW, OC, FH, FW;
    int sh, sw, ph, pw;
    int GK, GK_slice, GZ;
    int icb_count, ocb_count, taps;
    int groups;       // sharing groups (slice, input-channel block): their workgroups read the same X rows
    int per_group;    // workgroups of a sharing group = ocb_count * taps
    int xcd_map;      // 1: sharing group g runs on XCD g % 8 (workgroups are dealt round-robin to the 8 XCDs)
    int GPR;          // pixel groups (4 pixels) per output row = ceil(OW / 4)
    FastDiv d_OW, d_OH, d_per_group, d_icb, d_taps, d_FW, d_GPR;
};

template <int V> struct DwtInt { static constexpr int value = V; };

template <int KS, int D>
__global__ __launch_bounds__(64 * KS, 3) void delta_w_taps_kernel(const DwTapsArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float smem[];   // [KS-1][16 accumulators][64 lanes] float4
    const int t = threadIdx.x, lane = t & 63;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l16 = lane & 15, q = lane >> 4;

    // ---- which (slice, input-channel block, output-channel block, tap) ---------------------------------------------
    int grp, r;
    if (p.xcd_map) {
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        const int gl = fdiv(idx, p.d_per_group);
        r = idx - gl * p.per_group;
        grp = gl * 8 + xcd;
    } else {
        grp = fdiv(blockIdx.x, p.d_per_group);
        r = blockIdx.x - grp * p.per_group;
    }
    if (grp >= p.groups) return;
    const int z = fdiv(grp, p.d_icb), icb = grp - z * p.icb_count;
    const int ocb = fdiv(r, p.d_taps), tap = r - ocb * p.taps;
    const int fh = fdiv(tap, p.d_FW), fw = tap - fh * p.FW;

    const int k_start = p.GK_slice * z;
    const int k_end = (z != p.GZ - 1) ? k_start + p.GK_slice : p.GK;
    const int OW = p.OW, OH = p.OH, GPR = p.GPR;
    // Global output rows (n*OH + oh) the slice touches, as pixel groups in row order; the wavefronts take equal
    // contiguous shares of the groups (a share may begin and end inside a row).
    const int gr_first = fdiv(k_start, p.d_OW), gr_last = k_start < k_end ? (int)fdiv(k_end - 1, p.d_OW) : gr_first - 1;
    const int all_groups = (gr_last - gr_first + 1) * GPR;
    const int g_lo = __builtin_amdgcn_readfirstlane((int)((long)all_groups * w / KS));
    const int g_hi = __builtin_amdgcn_readfirstlane((int)((long)all_groups * (w + 1) / KS));
    const int total = g_hi - g_lo;   // pixel groups of this wavefront

    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    constexpr unsigned NEVER = 0x40000000u;   // plus or minus any offset within a row (host-checked < 2^28): out of range
    const int oc_l = 64 * ocb + 4 * l16, ic_l = 64 * icb + 4 * l16;
    const unsigned y_lane = oc_l < p.OC ? (unsigned)((q * p.OC + oc_l) * 4) : NEVER;
    const unsigned x_lane = ic_l < p.IC ? (unsigned)(((q * p.sw + fw - p.pw) * p.IC + ic_l) * 4) : NEVER;   // may be "negative"
    const int y_gstride = 16 * p.OC, x_gstride = 16 * p.sw * p.IC;   // bytes per pixel group

    // ---- load cursor: the row being requested (all scalar), its descriptors, the group within it ----------------------
    // rel = first pixel of the row relative to the slice's first pixel; oh, n = the row's place; the row's deltaY and the
    // image's X as byte addresses. Advancing by one row is additions only.
    __amdgpu_buffer_rsrc_t y_rsrc, x_rsrc;
    const int row0 = fdiv(g_lo, p.d_GPR);
    int cur_g = g_lo - row0 * GPR, left = total;
    int gr = gr_first + row0;
    int n = fdiv(gr, p.d_OH), oh = gr - n * OH;
    int rel = gr * OW - k_start;
    const int k_len = k_end - k_start;
    const size_t y_row_bytes = (size_t)OW * p.OC * 4, x_img_bytes = (size_t)p.IH * p.IW * p.IC * 4;
    const char *y_row = reinterpret_cast<const char *>(p.dY) + (size_t)gr * y_row_bytes;
    const char *x_img = reinterpret_cast<const char *>(p.X) + (size_t)n * x_img_bytes;
    const int x_row_bytes = p.IW * p.IC * 4;
    int y_goff = 0, x_goff = 0;
    auto setup_row = [&]() {   // descriptors of row (n, oh); `left` <= 0: nothing more to read, empty descriptors
        const int c_lo = max(0, -rel), c_hi = min(OW, k_len - rel);
        const bool live = left > 0;
        y_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(y_row) + c_lo * p.OC * 4, 0,
                                                   live && c_hi > c_lo ? (c_hi - c_lo) * p.OC * 4 : 0, 0x00020000);
        y_goff = cur_g * y_gstride - c_lo * p.OC * 4;
        const int ih = oh * p.sh - p.ph + fh;
        const bool inside = live && (unsigned)ih < (unsigned)p.IH;
        x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(x_img) + (inside ? ih : 0) * x_row_bytes, 0,
                                                   inside ? x_row_bytes : 0, 0x00020000);
        x_goff = cur_g * x_gstride;
    };
    floatx4 ya[D], xa[D];
    auto load = [&](int d) {
        ya[d] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(y_rsrc, y_lane + (unsigned)y_goff, 0, 0));
        xa[d] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, x_lane + (unsigned)x_goff, 0, 0));
        // on to the next group; the next row when this one is done (scalar work only: no memory operation in a branch)
        cur_g++;
        left--;
        y_goff += y_gstride;
        x_goff += x_gstride;
        if (cur_g == GPR) {
            cur_g = 0;
            rel += OW;
            y_row += y_row_bytes;
            oh++;
            if (oh == OH) {
                oh = 0;
                x_img += x_img_bytes;
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

    // ---- sum the wavefronts' parts in the order 0, 1, 2, ... and store -----------------------------------------------
    floatx4 *red = reinterpret_cast<floatx4 *>(smem);
    if (KS > 1) {
        if (w > 0) {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) red[((w - 1) * 16 + i * 4 + j) * 64 + lane] = acc[i][j];
        }
        __syncthreads();
    }
    if (w == 0) {
#pragma unroll 1   // one part's 16 registers at a time (unrolled, all parts are loaded before the first addition)
        for (int part = 1; part < KS; part++)
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] += red[((part - 1) * 16 + i * 4 + j) * 64 + lane];
        float *dst = (z == 0) ? p.dW : p.dW_buf + (size_t)(z - 1) * p.OC * p.taps * p.IC;
        // acc[i][j][r] = deltaW[oc = 64 ocb + 4 (4q + r) + i][tap][ic = 64 icb + 4 l16 + j]
        if (ic_l < p.IC) {
#pragma unroll
            for (int rr = 0; rr < 4; rr++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int oc = ocb * 64 + 4 * (4 * q + rr) + i;
                    if (oc < p.OC)
                        *reinterpret_cast<float4 *>(dst + ((size_t)oc * p.taps + tap) * p.IC + ic_l) =
                            make_float4(acc[i][0][rr], acc[i][1][rr], acc[i][2][rr], acc[i][3][rr]);
                }
        }
    }
}

template <int KS, int D>
static hipError_t launch_dwt(hipStream_t stream, const DwTapsArgs &a, int grid)
{
    constexpr auto kern = delta_w_taps_kernel<KS, D>;
    const size_t lds = (size_t)(KS - 1) * 16 * 64 * sizeof(floatx4) + 16;
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * KS), lds, stream, a);
    return hipGetLastError();
}

// Returns hipErrorNotSupported (nothing launched) when the layer does not fit; the caller then uses another kernel.
hipError_t launch_deltaW_taps(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                              int N, int IH, int IW, int IC, int OH, int OW, int OC, int FH, int FW,
                              int sh, int sw, int ph, int pw, int GK_slice, int GZ)
{
    if ((IC & 3) || (OC & 3) || IC < 4 || OC < 4 || FH < 1 || FW < 1 || sh < 1 || sw < 1 || GZ < 1) return hipErrorNotSupported;
    // every output pixel's window inside the padded input (a smaller output than the formula's is fine)
    if ((long)(OH - 1) * sh + FH > (long)IH + 2 * ph || (long)(OW - 1) * sw + FW > (long)IW + 2 * pw) return hipErrorNotSupported;
    // 32-bit byte offsets within a row, well below the "never in range" offset
    if ((long)(OW + 4) * OC * 4 >= (1L << 28) || ((long)(OW + 4) * sw + FW + pw) * IC * 4 >= (1L << 28)) return hipErrorNotSupported;
    const long GK = (long)N * OH * OW;
    if (GK >= (1L << 31) || GK_slice < 0 || (long)(GZ - 1) * GK_slice > GK) return hipErrorNotSupported;
    DwTapsArgs a{};
    a.X = X; a.dY = dY; a.dW = dW; a.dW_buf = dW_buf;
    a.IH = IH; a.IW = IW; a.IC = IC; a.OH = OH; a.OW = OW; a.OC = OC; a.FH = FH; a.FW = FW;
    a.sh = sh; a.sw = sw; a.ph = ph; a.pw = pw;
    a.GK = (int)GK; a.GK_slice = GK_slice; a.GZ = GZ;
    a.icb_count = (IC + 63) / 64;
    a.ocb_count = (OC + 63) / 64;
    a.taps = FH * FW;
    a.groups = GZ * a.icb_count;
    a.per_group = a.ocb_count * a.taps;
    a.xcd_map = (a.groups % 8) == 0;
    a.GPR = (OW + 3) / 4;
    a.d_OW = make_fastdiv(OW);
    a.d_OH = make_fastdiv(OH);
    a.d_per_group = make_fastdiv(a.per_group);
    a.d_icb = make_fastdiv(a.icb_count);
    a.d_taps = make_fastdiv(a.taps);
    a.d_FW = make_fastdiv(FW);
    a.d_GPR = make_fastdiv(a.GPR);
    const long wgs = (long)a.groups * a.per_group;
    if (wgs >= (1L << 30)) return hipErrorNotSupported;
    return launch_dwt<4, 6>(stream, a, (int)wgs);
}

}  // namespace alpha
