// (Arguments and kernel of delta_w_stream.hip and delta_w_stream_flat.hip.)
// Backward-filter with the reduction dealt out evenly: one persistent workgroup per compute unit, operands straight from
// memory, fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950. Any filter size, stride and padding.
//
//   deltaW[oc, fh, fw, ic] = sum over pixels k = (n, oh, ow) of deltaY[k, oc] * X[n, oh*sh - ph + fh, ow*sw - pw + fw, ic]
//
// Why: delta_w_taps.hip launches one workgroup per (filter tap, 64 x 64 block of channels, K slice), and their number
// rarely suits the device: 432 equal workgroups on 256 compute units leave 80 units idle half the time, 1152 are 4.5 per
// unit. What the caller fixes is only that deltaW and the GridZ - 1 buffers of deltaW_buf ADD UP to the result (it sums
// them with buf_summary, dW/A.cu:66-76) - which pixels go into which buffer is the kernel's business. So here an item is
// (tap, 64 x 64 block) with ALL its pixels, as groups of four pixels of an output row; the items one after the other form
// a line, the line is cut into one equal share per workgroup, and the pieces of an item - it meets at most
// workgroups / items + 2 shares - go to deltaW, deltaW_buf[0], deltaW_buf[1], ... in order; (item, buffer) pairs beyond an
// item's pieces are filled with zeros. (Or every item is cut into R equal pieces and the R x items units are dealt out
// whole: see the kernel.) The partition is a function of the shape, GridZ and the device's compute units: no atomics,
// bit-identical results from run to run.
//
// Inside a piece the arithmetic is delta_w_taps.hip's: lane (l16, q) loads
//   ya = deltaY[n, oh, 4g + q][oc0 + 4*l16 .. +3]      xa = X[n, ih, (4g + q)*sw + fw - pw][ic0 + 4*l16 .. +3]
// and MFMA (i, j) multiplies component i of ya with component j of xa; the eight wavefronts take equal contiguous runs of
// the piece's pixel groups (a ring of D groups in registers hides the latency, descriptors per output row return zeros for
// padding) and their accumulators are added through LDS in the order 0, 1, 2, ...
// FLAT: short output rows leave most of a row's last group empty - half of every group on 2x2 maps, three of eight pixels
// on rows of 5. There a group is four consecutive pixels of the IMAGE (row-major), the descriptors cover an image, vertical
// padding falls outside them, and every lane keeps its pixel's column and offset in X (a few vector instructions per
// group) for the horizontal padding. That bookkeeping costs 5-13 % of the kernel's time, so rows that waste less than
// three sixteenths of their groups' pixels (7, 14 pixels: an eighth) keep the groups by row.
#pragma once
#include "common.hpp"

namespace alpha {

struct DwStreamArgs {
    const float *X;
    const float *dY;
    float *dW;
    float *dW_buf;
    int IH, IW, IC, OH, OW, OC, FH, FW;
    int sh, sw, ph, pw;
    int GZ, icb_count, ocb_count, taps, items;
    int GPR;      // pixel groups (4 pixels) per output row = ceil(OW / 4); flat: per image = ceil(OH * OW / 4)
    int TG;       // pixel groups per item = N * OH * GPR; flat: N * GPR
    long L;       // items * TG
    int wgs;
    int R;        // > 0: every item is cut into R equal pieces, whole (piece, item) units per workgroup (see below); 0: the line of items
    FastDiv d_OH, d_FW, d_GPR, d_taps, d_ocb;
};

// The arguments of the kernel with pixel groups by image (FLAT): the same and the divisor by the row length. (A struct of
// its own, and a translation unit of its own for that kernel: the kernel with groups by row then compiles to the code it
// was before the other existed - with the fields in one struct it measured 3.7 % slower on 8x8 maps, 256 -> 256 channels.)
struct DwStreamFlatArgs : DwStreamArgs {
    FastDiv d_OW;
};

// Shares [L*s/G, L*(s+1)/G): the share that holds position P is the largest s with L*s/G <= P.
__host__ __device__ inline int dws_share_of(long P, long L, int G)
{
    return (int)(((P + 1) * G - 1) / L);
}

// A lane's NI (NJ) consecutive channels of deltaY (X) as the low components of a float4: one 128-, 96-, 64- or 32-bit load.
template <int N>
static __device__ __forceinline__ floatx4 dws_load(__amdgpu_buffer_rsrc_t rsrc, unsigned voffset)
{
    if constexpr (N == 4) {
        return __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voffset, 0, 0));
    } else if constexpr (N == 3) {
        // (the builtin's result converted as a whole: indexing it directly compiles to a load of the first word only)
        typedef float floatx3 __attribute__((ext_vector_type(3)));
        const floatx3 v = __builtin_bit_cast(floatx3, __builtin_amdgcn_raw_buffer_load_b96(rsrc, voffset, 0, 0));
        return floatx4{v[0], v[1], v[2], 0.f};
    } else if constexpr (N == 2) {
        typedef float floatx2 __attribute__((ext_vector_type(2)));
        const floatx2 v = __builtin_bit_cast(floatx2, __builtin_amdgcn_raw_buffer_load_b64(rsrc, voffset, 0, 0));
        return floatx4{v[0], v[1], 0.f, 0.f};
    } else {
        return floatx4{__builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, voffset, 0, 0)), 0.f, 0.f, 0.f};
    }
}

// NI, NJ: output (input) channels per lane, 1 to 4: a block of the filter is 16 NI output x 16 NJ input channels, and a
// group of four pixels costs NI x NJ MFMAs. 4 x 4 = the 64 x 64 blocks; 96 input channels are two blocks of 48 with NJ = 3
// (12 MFMAs a group on full blocks instead of 16 on one full and one half-empty block).
template <int D, bool FLAT = false, class Args = DwStreamArgs, int NI = 4, int NJ = 4>
__global__ __launch_bounds__(512, 1) void delta_w_stream_kernel(const Args p)
{
    extern __shared__ __attribute__((aligned(16))) float dws_smem[];   // [8 wavefronts][16 units][64 lanes] float4
    floatx4 *part = reinterpret_cast<floatx4 *>(dws_smem);
    const int t = threadIdx.x, lane = t & 63;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l16 = lane & 15, q = lane >> 4;
    const int G = p.wgs, b = blockIdx.x;
    // consecutive shares run on one XCD (workgroups are dealt round-robin to the 8 XCDs): the taps of a block, which read
    // the same rows, then share an L2
    const int s = (G & 7) == 0 ? (b & 7) * (G >> 3) + (b >> 3) : b;
    // R > 0: every item is cut into R equal pieces and unit u = r * items + i is piece r of item i; the shares are whole units,
    // [U s / G, U (s + 1) / G) of the U = R * items. The items' pieces over the same pixels are neighbours - the same XCD,
    // or two -, start together and are equally long, so the rows one of them fetches are in L2 for the others. (In the
    // line of items, R = 0, the shares of different items over the same pixels drift apart in time: with tensors beyond
    // the caches every item then fetches its rows again - 9 x 51 MB on 56x56x64 at N = 32.)
    long pos, hi;
    if (p.R > 0) {
        const long U = (long)p.R * p.items;
        pos = U * s / G;
        hi = U * (s + 1) / G;
    } else {
        pos = p.L * s / G;
        hi = p.L * (s + 1) / G;
    }
    const int OW = p.OW, OH = p.OH, GPR = p.GPR;
    const size_t sizeW = (size_t)p.OC * p.taps * p.IC;
    constexpr unsigned NEVER = 0x40000000u;   // plus or minus any offset within a row (host-checked < 2^28): out of range
    const int y_gstride = 16 * p.OC, x_gstride = 16 * p.sw * p.IC;   // bytes per pixel group
    const size_t y_row_bytes = (size_t)OW * p.OC * 4, x_img_bytes = (size_t)p.IH * p.IW * p.IC * 4;
    const int x_row_bytes = p.IW * p.IC * 4;

    while (pos < hi) {   // uniform over the workgroup
        int item, ga, gb, ord, npieces;
        if (p.R > 0) {
            ord = (int)pos / p.items;
            item = (int)pos - ord * p.items;
            npieces = p.R;
            ga = (int)((long)p.TG * ord / p.R);
            gb = (int)((long)p.TG * (ord + 1) / p.R);
            pos++;
        } else {
            item = (int)(pos / p.TG);
            const long P0 = (long)item * p.TG;
            ga = (int)(pos - P0);
            gb = (int)((hi < P0 + p.TG ? hi : P0 + p.TG) - P0);
            const int s_first = dws_share_of(P0, p.L, G), s_last = dws_share_of(P0 + p.TG - 1, p.L, G);
            ord = s - s_first;
            npieces = s_last - s_first + 1;
            pos = P0 + gb;
        }

        const int blk = fdiv(item, p.d_taps), tap = item - blk * p.taps;
        const int icb = fdiv(blk, p.d_ocb), ocb = blk - icb * p.ocb_count;
        const int fh = fdiv(tap, p.d_FW), fw = tap - fh * p.FW;
        const int oc_l = 16 * NI * ocb + NI * l16, ic_l = 16 * NJ * icb + NJ * l16;
        const unsigned y_lane = oc_l < p.OC ? (unsigned)((q * p.OC + oc_l) * 4) : NEVER;
        const unsigned x_lane = ic_l < p.IC ? (unsigned)(((q * p.sw + fw - p.pw) * p.IC + ic_l) * 4) : NEVER;   // may be "negative"

        // ---- this wavefront's run of the piece's pixel groups ---------------------------------------------------------------
        const int n_g = gb - ga;
        const int g_lo = __builtin_amdgcn_readfirstlane(ga + (int)((long)n_g * w / 8));
        const int g_hi = __builtin_amdgcn_readfirstlane(ga + (int)((long)n_g * (w + 1) / 8));
        const int total = g_hi - g_lo;

        floatx4 acc[NI][NJ];
#pragma unroll
        for (int i = 0; i < NI; i++)
#pragma unroll
            for (int j = 0; j < NJ; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

        // ---- load cursor: the row being requested (all scalar), its descriptors, the group within it -----------------------
        //      (FLAT: the image being requested, its descriptors, the group within it; per lane the pixel's column and
        //      its byte offset in the image of X)
        __amdgpu_buffer_rsrc_t y_rsrc, x_rsrc;
        const int gr0 = fdiv(g_lo, p.d_GPR);   // global output row n * OH + oh; FLAT: image n
        int cur_g = g_lo - gr0 * GPR, left = total;
        const int n0 = FLAT ? gr0 : fdiv(gr0, p.d_OH);
        int oh = FLAT ? 0 : gr0 - n0 * OH;
        const size_t y_img_bytes = (size_t)OH * y_row_bytes;
        const char *y_row = reinterpret_cast<const char *>(p.dY) + (FLAT ? (size_t)n0 * y_img_bytes : (size_t)gr0 * y_row_bytes);
        const char *x_img = reinterpret_cast<const char *>(p.X) + (size_t)n0 * x_img_bytes;
        int y_goff = 0, x_goff = 0;
        // FLAT, per lane: pixel 4 cur_g + q of the image is (oh_l, ow_l); its tap's element of X is x_off bytes into the image
        // (negative or beyond the image above and below it: outside the descriptor). Four pixels on are `rows4` rows and
        // `cols4` columns, and one row more where the column passes the end of its row.
        int ow_l = 0, ow_first = 0;
        unsigned x_off = 0, x_first = 0;
        int cols4 = 0, x_step = 0, x_wrap = 0;
        if constexpr (FLAT) {
            const int rows4 = fdiv(4, p.d_OW);
            const int x_row4 = p.sh * p.IW * p.IC * 4, x_col4 = p.sw * p.IC * 4;
            cols4 = 4 - rows4 * OW;
            x_step = rows4 * x_row4 + cols4 * x_col4;
            x_wrap = x_row4 - OW * x_col4;
        }
        auto place = [&](int pix, int &ow_out, unsigned &off_out) {   // FLAT: pixel `pix` of an image
            if constexpr (FLAT) {
                const int oh_l = fdiv(pix, p.d_OW);
                ow_out = pix - oh_l * OW;
                off_out = (unsigned)((((oh_l * p.sh + fh - p.ph) * p.IW + ow_out * p.sw + fw - p.pw) * p.IC + ic_l) * 4);
            }
        };
        auto setup_row = [&]() {   // descriptors of row (n, oh); `left` <= 0: nothing more to read, empty descriptors
            const bool live = left > 0;
            if (FLAT) {
                y_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(y_row), 0, live ? (int)y_img_bytes : 0, 0x00020000);
                x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(x_img), 0, live ? (int)x_img_bytes : 0, 0x00020000);
                y_goff = cur_g * y_gstride;
                return;
            }
            y_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(y_row), 0, live ? (int)y_row_bytes : 0, 0x00020000);
            y_goff = cur_g * y_gstride;
            const int ih = oh * p.sh - p.ph + fh;
            const bool inside = live && (unsigned)ih < (unsigned)p.IH;
            x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(x_img) + (inside ? ih : 0) * (long)x_row_bytes, 0,
                                                       inside ? x_row_bytes : 0, 0x00020000);
            x_goff = cur_g * x_gstride;
        };
        floatx4 ya[D], xa[D];
        auto load = [&](int d) {
            if (FLAT) {
                const bool col_ok = ic_l < p.IC && (unsigned)(ow_l * p.sw + fw - p.pw) < (unsigned)p.IW;
                ya[d] = dws_load<NI>(y_rsrc, y_lane + (unsigned)y_goff);
                xa[d] = dws_load<NJ>(x_rsrc, col_ok ? x_off : 0x80000000u);
                cur_g++;
                left--;
                y_goff += y_gstride;
                ow_l += cols4;
                const int wrap = ow_l >= OW ? -1 : 0;   // per lane, without a branch
                ow_l -= OW & wrap;
                x_off += (unsigned)(x_step + (x_wrap & wrap));
                if (cur_g == GPR) {   // the next image (uniform)
                    cur_g = 0;
                    y_row += y_img_bytes;
                    x_img += x_img_bytes;
                    ow_l = ow_first;
                    x_off = x_first;
                    setup_row();
                }
                return;
            }
            ya[d] = dws_load<NI>(y_rsrc, y_lane + (unsigned)y_goff);
            xa[d] = dws_load<NJ>(x_rsrc, x_lane + (unsigned)x_goff);
            // on to the next group; the next row when this one is done (scalar work only: no memory operation in a branch)
            cur_g++;
            left--;
            y_goff += y_gstride;
            x_goff += x_gstride;
            if (cur_g == GPR) {
                cur_g = 0;
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
            for (int i = 0; i < NI; i++)
#pragma unroll
                for (int j = 0; j < NJ; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ya[d][i], xa[d][j], acc[i][j], 0, 0, 0);
        };
        if (total > 0) {
            if (FLAT) {   // where this lane's pixel of an image's first group lies, and its pixel of this run's first group
                place(q, ow_first, x_first);
                place(4 * cur_g + q, ow_l, x_off);
            }
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

        // ---- the eight parts added in the order 0, 1, 2, ...; unit u = 4 i + rr is one 128-bit store per lane:
        // acc[i][j][rr] = deltaW[oc = 16 NI ocb + NI (4q + rr) + i][tap][ic = 16 NJ icb + NJ l16 + j] ---------------------------
        if constexpr (NI == 4 && NJ == 4) {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int rr = 0; rr < 4; rr++)
                    part[(w * 16 + 4 * i + rr) * 64 + lane] = floatx4{acc[i][0][rr], acc[i][1][rr], acc[i][2][rr], acc[i][3][rr]};
            __syncthreads();
            float *dst = ord == 0 ? p.dW : p.dW_buf + (size_t)(ord - 1) * sizeW;
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const int u = w + 8 * k, i = u >> 2, rr = u & 3;
                floatx4 v = part[u * 64 + lane];
#pragma unroll
                for (int x = 1; x < 8; x++) v += part[(x * 16 + u) * 64 + lane];
                const int oc = ocb * 64 + 4 * (4 * q + rr) + i;
                if (ic_l < p.IC && oc < p.OC)
                    *reinterpret_cast<float4 *>(dst + ((size_t)oc * p.taps + tap) * p.IC + ic_l) = make_float4(v[0], v[1], v[2], v[3]);
            }
            // ---- zeros into the buffers none of the item's pieces writes: piece `ord` of `npieces` takes every npieces-th ------
            for (int z = npieces + ord; z < p.GZ; z += npieces) {
                float *zd = p.dW_buf + (size_t)(z - 1) * sizeW;   // z >= npieces >= 1
                for (int e = t; e < 64 * 16; e += 512) {            // 64 output channels x 16 float4 of input channels
                    const int oc = ocb * 64 + (e >> 4), ic = icb * 64 + 4 * (e & 15);
                    if (oc < p.OC && ic < p.IC)
                        *reinterpret_cast<float4 *>(zd + ((size_t)oc * p.taps + tap) * p.IC + ic) = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < NI; i++)
#pragma unroll
                for (int rr = 0; rr < 4; rr++) {
                    floatx4 v = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = 0; j < NJ; j++) v[j] = acc[i][j][rr];
                    part[(w * 16 + 4 * i + rr) * 64 + lane] = v;
                }
            __syncthreads();
            float *dst = ord == 0 ? p.dW : p.dW_buf + (size_t)(ord - 1) * sizeW;
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const int u = w + 8 * k, i = u >> 2, rr = u & 3;
                if (u < 4 * NI) {   // uniform
                    floatx4 v = part[u * 64 + lane];
#pragma unroll
                    for (int x = 1; x < 8; x++) v += part[(x * 16 + u) * 64 + lane];
                    const int oc = ocb * 16 * NI + NI * (4 * q + rr) + i;
                    if (ic_l < p.IC && oc < p.OC) {
                        float *o = dst + ((size_t)oc * p.taps + tap) * p.IC + ic_l;
#pragma unroll
                        for (int j = 0; j < NJ; j++) o[j] = v[j];
                    }
                }
            }
            for (int z = npieces + ord; z < p.GZ; z += npieces) {
                float *zd = p.dW_buf + (size_t)(z - 1) * sizeW;
                for (int e = t; e < 16 * NI * 4 * NJ; e += 512) {   // 16 NI output channels x 4 NJ float4 of input channels
                    const int oc = ocb * 16 * NI + e / (4 * NJ), ic = icb * 16 * NJ + 4 * (e % (4 * NJ));
                    if (oc < p.OC && ic < p.IC)
                        *reinterpret_cast<float4 *>(zd + ((size_t)oc * p.taps + tap) * p.IC + ic) = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
        }
        __syncthreads();   // the next piece writes `part` again
    }
}

// Launch of the kernel with NI x NJ channels per lane (groups by row).
template <int NI, int NJ>
static hipError_t dws_launch(hipStream_t stream, const DwStreamArgs &a, size_t lds)
{
    constexpr auto kern = delta_w_stream_kernel<6, false, DwStreamArgs, NI, NJ>;
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(a.wgs), dim3(512), lds, stream, a);
    return hipGetLastError();
}

// delta_w_stream_narrow_*.hip: the kernels with fewer than 4 x 4 channels per lane, NI (NJ) output (input) channels
hipError_t launch_deltaW_stream_narrow_x(hipStream_t stream, const DwStreamArgs &a, size_t lds, int NJ);            // NI = 4
hipError_t launch_deltaW_stream_narrow_y(hipStream_t stream, const DwStreamArgs &a, size_t lds, int NI);            // NJ = 4
hipError_t launch_deltaW_stream_narrow_xy(hipStream_t stream, const DwStreamArgs &a, size_t lds, int NI, int NJ);   // both below 4

}  // namespace alpha
