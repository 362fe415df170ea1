// Launcher of the persistent backward-filter kernel (delta_w_stream_kernel.hpp) and the split-K factors it needs.
#include "delta_w_stream_kernel.hpp"
#include <atomic>
#include <cstdlib>

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

// Whether layers outside the first rule below are cut into whole units (pieces x items): -1 by shape, 0 never, 1 wherever
// the buffers allow it. A debugging switch (deltaW_stream_set_units, or ALPHA_DW_UNITS=0/1 in the environment, read once
// per process): the parity tests run both cuts on small shapes.
static std::atomic<int> g_dws_units{-2};

static int dws_units_switch()
{
    int v = g_dws_units.load(std::memory_order_relaxed);
    if (v == -2) {
        const char *e = getenv("ALPHA_DW_UNITS");
        v = e ? (atoi(e) != 0 ? 1 : 0) : -1;
        int expected = -2;
        if (!g_dws_units.compare_exchange_strong(expected, v)) v = expected;   // a setter was quicker
    }
    return v;
}

void deltaW_stream_set_units(int units) { g_dws_units.store(units < 0 ? -1 : units != 0); }

// How the kernel cuts a layer of `items` items of TG pixel groups on G workgroups with GZ - 1 buffers:
//   pieces > 0, units: every item in `pieces` equal pieces, the pieces x items units dealt out whole, piece-major;
//   pieces > 0, !units: the line of items in G equal shares, of which an item meets at most `pieces`;
//   pieces == 0: the kernel does not take the layer.
struct DwsCut {
    int pieces;
    bool units;
};

static DwsCut dws_cut(long items, long TG, int G, int GZ, long bytes)
{
    // at least eight pixel groups per workgroup (one per wavefront); smaller layers go to the kernels with one workgroup per slice
    if (items * TG < 8L * G || items > 4096 || GZ < 2) return {0, false};
    // (1) R x items workgroups are (nearly) all of them: one unit each
    long R = G / items;
    if (R > GZ) R = GZ;
    if (R >= 1 && 20 * R * items >= 19L * G) return {(int)R, true};
    const int most = dws_max_pieces(items, TG, G);
    // (2) Tensors well beyond the L2s (56 MB: measured between 50 and 65) whose shares of the line start at 32 or more
    // different places of the pixel range (G / gcd(items, G): 27, 72, 200 items on 256 workgroups; with 144 items pairs
    // of shares run over the same pixels, with 576 eight at a time, and the line stays the faster cut): every workgroup
    // then streams pixels of its own and the L2s serve nobody twice (5x5 96 -> 256 on 64x27x27: 3.8 GB fetched for 65 MB
    // of tensors). Whole units instead, ceil(P items / G) per workgroup: the workgroups of an XCD go through the same
    // piece of the pixels at the same time, each for an item of its own. P minimises the modelled time, a unit's
    // end (partial sums through LDS, stores, the loads of the next from cold) counted as 64 pixel groups.
    const int forced = dws_units_switch();
    long gcd = items;
    for (long b = G; b != 0;) { const long r = gcd % b; gcd = b; b = r; }
    constexpr long UNIT_END = 64;   // pixel groups
    const long line_time = (items * TG + G - 1) / G + 2 * UNIT_END;
    long best_time = 0;
    int best_P = 0;
    for (int P = 1; P <= GZ && 8L * P <= TG; P++) {
        const long t = (P * items + G - 1) / G * ((TG + P - 1) / P + UNIT_END);
        if (best_P == 0 || t < best_time) best_time = t, best_P = P;
    }
    const bool by_shape = bytes > (56L << 20) && gcd * 32 <= G && 100 * best_time <= 108 * line_time;
    if (best_P > 0 && (forced == 1 || (forced < 0 && by_shape))) return {best_P, true};
    // (3) the line of items; with fewer buffers than the shares an item would meet (the Java engine passes GridZ = 2 for
    // 4x4 maps at N = 512, where 72 items on 256 workgroups meet up to 5 shares each) whole units all the same, some
    // workgroups idle - still several times faster than the kernels with one workgroup per slice (3x3 96 -> 208 there: 0.463 ms)
    if (most > GZ) return best_P > 0 ? DwsCut{best_P, true} : DwsCut{0, false};
    return {most, false};
}

// A 1x1 filter at stride 1 without padding reads pixel k of X for pixel k of deltaY: the rows and images are one run of
// pixels, and the kernel takes it as a single row (or a row per image where that is too long for the 32-bit offsets within
// a row) - no pixel group is left partly empty at the end of a 7- or 14-pixel row, and no row ever ends.
static void dws_pointwise_rows(int &N, int &OH, int &OW, int IC, int OC)
{
    const long P = (long)OH * OW, C = IC > OC ? IC : OC;
    if (((long)N * P + 8) * C * 4 < (1L << 28)) { OW = (int)(N * P); OH = 1; N = 1; }
    else if ((P + 8) * C * 4 < (1L << 28)) { OW = (int)P; OH = 1; }
}

// Pixel groups as four consecutive pixels of an image (row-major) instead of an output row: where a row's groups are
// empty to three sixteenths or more (rows of 1, 2, 3, 5, 6, 9 or 13 pixels). Images beyond 512 MB do not fit the 32-bit offsets
// within an image.
static bool dws_flat_rows(int OH, int OW, int OC)
{
    const int slots = (OW + 3) / 4 * 4;
    return 16 * (slots - OW) >= 3 * slots && (long)OH * OW * OC * 4 < (1L << 29);
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

// The cut of a layer as the split-K helpers below know it (no input size, no stride): `bytes` is counted on the output's
// pixels for both tensors, here and in the launcher.
static DwsCut dws_cut_of_layer(int units, int N, int OH, int OW, int IC, int OC, int FH, int FW, int GZ)
{
    if ((IC & 3) || (OC & 3) || IC < 4 || OC < 4 || FH < 1 || FW < 1 || GZ < 2 || units < 1 || N < 1 || OH < 1 || OW < 1) return {0, false};
    // the stricter of the split-K entries' two thresholds (the stride is not known here)
    if (deltaW_stream_block_fill(IC, OC) < 40) return {0, false};
    const long icb = (IC + 63) / 64, ocb = (OC + 63) / 64;
    const long bytes = (long)N * OH * OW * ((long)IC + OC) * 4;
    if (FH == 1 && FW == 1) dws_pointwise_rows(N, OH, OW, IC, OC);   // (taken to be at stride 1 without padding, as nearly all are)
    // (the input's size is not known here: the launcher's other condition for groups by image, an image of X below 512 MB)
    const bool flat = dws_flat_rows(OH, OW, OC);
    const long items = icb * ocb * FH * FW, TG = flat ? (long)N * (((long)OH * OW + 3) / 4) : (long)N * OH * ((OW + 3) / 4);
    if (items >= (1L << 20) || TG >= (1L << 30)) return {0, false};
    return dws_cut(items, TG, units, GZ, bytes);
}

// The least split-K factor <= GZ with which launch_deltaW_stream on a device of `units` compute units cuts the layer
// exactly as it does with GZ (the same pieces per item, or the same line of shares), or GZ itself where the kernel
// does not take the layer or the split-K entries may not choose it (channel counts that fill their blocks to less than
// 40 %). With it the kernel has no buffers to fill with zeros and the caller's buf_summary none to add for nothing.
int deltaW_stream_least_GridZ(int units, int N, int OH, int OW, int IC, int OC, int FH, int FW, int GZ)
{
    const DwsCut c = dws_cut_of_layer(units, N, OH, OW, IC, OC, FH, FW, GZ);
    if (c.pieces == 0) return GZ;
    return c.pieces < 2 ? 2 : c.pieces;
}

// The split-K factor a host layer that owns GridZ should pass: deltaW_stream_least_GridZ where GZ is enough for the cut
// the kernel would make with GZ_cap buffers, and where it is not (the reference sizes GridZ for the slices of its
// kernels: 2 on 4x4 maps at N = 512, where 72 items on 256 compute units meet up to 5 shares each) the factor that cut needs.
int deltaW_stream_fill_GridZ(int units, int N, int OH, int OW, int IC, int OC, int FH, int FW, int GZ, int GZ_cap)
{
    const int least = deltaW_stream_least_GridZ(units, N, OH, OW, IC, OC, FH, FW, GZ);
    if (GZ < 2 || GZ_cap <= GZ) return least;
    const DwsCut c = dws_cut_of_layer(units, N, OH, OW, IC, OC, FH, FW, GZ_cap);
    return c.pieces > GZ ? c.pieces : least;
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
    if (FH == 1 && FW == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0 && OH == IH && OW == IW) {
        dws_pointwise_rows(N, OH, OW, IC, OC);
        IH = OH;
        IW = OW;
    }
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
    // whole units (every item in R equal pieces) or the line of items in equal shares; either way the pieces of an item go
    // to deltaW and the GridZ - 1 buffers
    const DwsCut cut = dws_cut(items, TG, a.wgs, GZ, (long)N * OH * OW * ((long)IC + OC) * 4);
    if (cut.pieces == 0) return hipErrorNotSupported;
    a.R = cut.units ? cut.pieces : 0;
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
