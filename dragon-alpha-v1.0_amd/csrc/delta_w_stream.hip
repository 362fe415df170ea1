// Launcher of the persistent backward-filter kernel (delta_w_stream_kernel.hpp) and the split-K factors it needs.
#include "delta_w_stream_kernel.hpp"

namespace alpha {

// the kernel with pixel groups by image: delta_w_stream_flat.hip
hipError_t launch_deltaW_stream_flat(hipStream_t stream, const DwStreamFlatArgs &a, size_t lds);

// The largest number of shares an item meets when the line of `items` items of TG groups is cut into G shares.
static int dws_max_pieces(long items, long TG, int G)
{
    const long L = items * TG;
    int most = 0;
    for (long item = 0; item < items; item++) {
        const long P0 = item * TG, P1 = P0 + TG - 1;
        const int n = (int)(((P1 + 1) * G - 1) / L) - (int)(((P0 + 1) * G - 1) / L) + 1;
        if (n > most) most = n;
    }
    return most;
}

// Pixel groups as four consecutive pixels of an image (row-major) instead of an output row: where a row's groups are
// empty to a quarter or more (rows of 1, 2, 3, 5, 6 or 9 pixels). Images beyond 512 MB do not fit the 32-bit offsets
// within an image.
static bool dws_flat_rows(int OH, int OW, int OC)
{
    const int slots = (OW + 3) / 4 * 4;
    return 4 * (slots - OW) >= slots && (long)OH * OW * OC * 4 < (1L << 29);
}

static int dws_per_lane(int C)
{
    const int blocks = (C + 63) / 64, n = (C + 16 * blocks - 1) / (16 * blocks);
    return (n < 4 && C % n == 0) ? n : 4;
}

// How full the kernel's blocks of the filter are, in per cent: channels / (blocks x 16 x channels per lane), both sides.
int deltaW_stream_block_fill(int IC, int OC)
{
    if (IC < 1 || OC < 1) return 0;
    const long ib = (IC + 63) / 64 * 16L * dws_per_lane(IC), ob = (OC + 63) / 64 * 16L * dws_per_lane(OC);
    return (int)(100L * IC * OC / (ib * ob));
}

// The least split-K factor <= GZ with which launch_deltaW_stream on a device of `units` compute units cuts the layer
// exactly as it does with GZ (the same R pieces per item, or the same line of shares), or GZ itself where the kernel
// does not take the layer or the split-K entries may not choose it (channel counts that fill 64 x 64 blocks to less than
// 40 %). With it the kernel has no buffers to fill with zeros and the caller's buf_summary none to add for nothing.
int deltaW_stream_least_GridZ(int units, int N, int OH, int OW, int IC, int OC, int FH, int FW, int GZ)
{
    if ((IC & 3) || (OC & 3) || IC < 4 || OC < 4 || FH < 1 || FW < 1 || GZ < 2 || units < 1 || N < 1 || OH < 1 || OW < 1) return GZ;
    const long icb = (IC + 63) / 64, ocb = (OC + 63) / 64;
    if (deltaW_stream_block_fill(IC, OC) < 40) return GZ;   // the stricter of the split-K entries' two thresholds (the stride is not known here)
    // (the input's size is not known here: the launcher's other condition for groups by image, an image of X below 512 MB)
    const bool flat = dws_flat_rows(OH, OW, OC);
    const long items = icb * ocb * FH * FW, TG = flat ? (long)N * (((long)OH * OW + 3) / 4) : (long)N * OH * ((OW + 3) / 4);
    if (items >= (1L << 20) || TG >= (1L << 30) || items * TG < 8L * units || items > 4096) return GZ;
    long R = units / items;
    if (R > GZ) R = GZ;
    if (R >= 1 && 20 * R * items >= 19L * units) return R < 2 ? 2 : (int)R;
    const int most = dws_max_pieces(items, TG, units);
    if (most > GZ) return R >= 1 ? (R < 2 ? 2 : (int)R) : GZ;   // R pieces per item on fewer workgroups (see the launcher)
    return most < 2 ? 2 : most;
}

// The split-K factor a host layer that owns GridZ should pass: deltaW_stream_least_GridZ where GZ is enough for the kernel's
// own cut, and where it is not (the reference sizes GridZ for the slices of its kernels: 2 on 4x4 maps at N = 512, where 72
// items on 256 compute units meet up to 5 shares each) the pieces per item that cut wants, up to GZ_cap.
int deltaW_stream_fill_GridZ(int units, int N, int OH, int OW, int IC, int OC, int FH, int FW, int GZ, int GZ_cap)
{
    const int least = deltaW_stream_least_GridZ(units, N, OH, OW, IC, OC, FH, FW, GZ);
    if (least != GZ || GZ < 2 || GZ_cap <= GZ || (IC & 3) || (OC & 3) || IC < 4 || OC < 4 || FH < 1 || FW < 1 || units < 1 || N < 1 || OH < 1 || OW < 1) return least;
    const long icb = (IC + 63) / 64, ocb = (OC + 63) / 64;
    if (deltaW_stream_block_fill(IC, OC) < 40) return least;
    const bool flat = dws_flat_rows(OH, OW, OC);
    const long items = icb * ocb * FH * FW, TG = flat ? (long)N * (((long)OH * OW + 3) / 4) : (long)N * OH * ((OW + 3) / 4);
    if (items >= (1L << 20) || TG >= (1L << 30) || items * TG < 8L * units || items > 4096) return least;
    const long R = units / items;
    const long want = (R >= 1 && 20 * R * items >= 19L * units) ? R : dws_max_pieces(items, TG, units);
    return want > GZ && want <= GZ_cap ? (int)want : least;
}

// Returns hipErrorNotSupported (nothing launched) when the layer does not fit; the caller then uses another kernel.
hipError_t launch_deltaW_stream(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                                int N, int IH, int IW, int IC, int OH, int OW, int OC, int FH, int FW,
                                int sh, int sw, int ph, int pw, int GZ)
{
    if ((IC & 3) || (OC & 3) || IC < 4 || OC < 4 || FH < 1 || FW < 1 || sh < 1 || sw < 1 || GZ < 2) return hipErrorNotSupported;
    // every output pixel's window inside the padded input (a smaller output than the formula's is fine)
    if ((long)(OH - 1) * sh + FH > (long)IH + 2 * ph || (long)(OW - 1) * sw + FW > (long)IW + 2 * pw) return hipErrorNotSupported;
    // 32-bit byte offsets within a row, well below the "never in range" offset
    if ((long)(OW + 4) * OC * 4 >= (1L << 28) || ((long)(OW + 4) * sw + FW + pw) * IC * 4 >= (1L << 28)) return hipErrorNotSupported;
    const long GK = (long)N * OH * OW;
    if (GK >= (1L << 31)) return hipErrorNotSupported;
    const int cus = device_cu_count();
    if (cus < 1) return hipErrorNotSupported;
    DwStreamFlatArgs a{};
    a.X = X; a.dY = dY; a.dW = dW; a.dW_buf = dW_buf;
    a.IH = IH; a.IW = IW; a.IC = IC; a.OH = OH; a.OW = OW; a.OC = OC; a.FH = FH; a.FW = FW;
    a.sh = sh; a.sw = sw; a.ph = ph; a.pw = pw;
    a.GZ = GZ;
    a.icb_count = (IC + 63) / 64;
    a.ocb_count = (OC + 63) / 64;
    // Channels per lane: the least with which the same number of blocks (of 16 per-lane groups) holds the channels - 96
    // channels are two blocks of 48 (3 per lane) instead of one of 64 and one half-empty -, where the channel count is a
    // multiple of it (a lane's group never straddles the end of a pixel's channels). With pixel groups by image: 4.
    int ni = dws_per_lane(OC), nj = dws_per_lane(IC);
    if (dws_flat_rows(OH, OW, OC) && (long)IH * IW * IC * 4 < (1L << 29)) ni = nj = 4;
    a.taps = FH * FW;
    const long items = (long)a.icb_count * a.ocb_count * a.taps;
    const bool flat = dws_flat_rows(OH, OW, OC) && (long)IH * IW * IC * 4 < (1L << 29);
    a.GPR = flat ? (OH * OW + 3) / 4 : (OW + 3) / 4;
    const long TG = flat ? (long)N * a.GPR : (long)N * OH * a.GPR;
    if (items >= (1L << 20) || TG >= (1L << 30)) return hipErrorNotSupported;
    a.items = (int)items;
    a.TG = (int)TG;
    a.L = items * TG;
    a.wgs = cus;   // one workgroup of eight wavefronts per compute unit
    // at least eight pixel groups per workgroup (one per wavefront); smaller layers go to the kernels with one workgroup per slice
    if (a.L < 8L * a.wgs || items > 4096) return hipErrorNotSupported;
    // Every item in R equal pieces where R * items workgroups are (nearly) all of them; else the line of items in equal
    // shares. Either way the pieces of an item go to deltaW and the GridZ - 1 buffers.
    long R = cus / items;
    if (R > GZ) R = GZ;
    if (R >= 1 && 20 * R * items >= 19L * cus) {
        a.R = (int)R;
    } else {
        a.R = 0;
        if (dws_max_pieces(items, TG, a.wgs) > GZ) {
            // fewer items than workgroups and fewer buffers than the shares an item would meet (the Java engine passes
            // GridZ = 2 for 4x4 maps at N = 512): R = GridZ pieces per item on R x items workgroups, the rest idle - still
            // several times faster than the kernels with one workgroup per slice (3x3 96 -> 208 there: 0.463 ms)
            if (R < 1) return hipErrorNotSupported;
            a.R = (int)R;
        }
    }
    a.d_OH = make_fastdiv(OH);
    a.d_OW = make_fastdiv(OW);
    a.d_FW = make_fastdiv(FW);
    a.d_GPR = make_fastdiv(a.GPR);
    a.d_taps = make_fastdiv(a.taps);
    a.d_ocb = make_fastdiv(a.ocb_count);
    const size_t lds = (size_t)8 * 16 * 64 * sizeof(floatx4);
    if (flat) return launch_deltaW_stream_flat(stream, a, lds);
    if (ni < 4 && nj < 4) return launch_deltaW_stream_narrow_xy(stream, a, lds, ni, nj);
    if (nj < 4) return launch_deltaW_stream_narrow_x(stream, a, lds, nj);
    if (ni < 4) return launch_deltaW_stream_narrow_y(stream, a, lds, ni);
    constexpr auto kern = delta_w_stream_kernel<6>;
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(a.wgs), dim3(512), lds, stream, static_cast<const DwStreamArgs &>(a));
    return hipGetLastError();
}

}  // namespace alpha
