// Forward convolution of layers with 4 stored input channels - network stems such as 7x7 stride 2 on RGB - with both
// operands straight from memory: no LDS, no barrier in the main loop, fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950.
//
//   Y[m, oc] = sum over taps (fh, fw) and channels c < 4 of X[n, oh*sh - ph + fh, ow*sw - pw + fw, c] * W[oc, fh, fw, c]
//
// The reduction index of one MFMA is FOUR TAPS of one channel (stem_conv.hip's scheme): lane (l16, q) loads the float4 -
// all four channels - of the input pixel that tap 4g + q touches for output pixel l16 of a tile, and the float4 of filter
// tap 4g + q for output channel 4*l16 + j, j = 0..3; component s (the channel) of both feeds MFMA (s, j). A step is one
// group g of four taps: one 128-bit load per tile and four for the filter, shared by the T <= 4 tiles a wavefront
// owns, feed 16 T MFMAs (12 T when the fourth stored channel has zero weights everywhere: layers with three logical
// channels). The last tap (7x7 and 3x3 have 4 k + 1 taps) would fill a group on its own, three quarters of it padding:
// in that step the reduction index is the CHANNEL instead - lane (l16, q) loads channel q of the last tap's pixel and of
// the filter's last tap with 32-bit loads -, one MFMA per tile and j instead of three or four.
// A lane's accumulators are 4 consecutive output channels of a pixel: results leave as 128-bit stores.
// The filter is read as W[OC, FH, FW, 4] in place - its 4-channel taps are exactly the 16-byte units the lanes need - and
// stays in L1 / L2 (64 channels of a 7x7 filter: 50 KB).
//
// Where a tile's pixels are is worked out per lane once per group of tiles (window origin, masks of the window rows and
// columns inside the image); a lane's tap offsets and the mask bits its taps need are registers computed once (the
// step loop is unrolled over the tap groups, so they are indexed statically). Per step and tile: and, compare, add,
// select. Loads run one step ahead through a cursor over (group of tiles, tap group); with an odd number of steps per
// group of tiles the two register sets swap roles from one group to the next (template parameter P).
//
// Against stem_conv.hip (window staged in LDS per block of 16 x 16 output pixels, results through an LDS patch): no
// staging phase, no barriers, no output transpose; the window's re-reads go to L1 / L2 instead.
#include "common.hpp"
#include <type_traits>

namespace alpha {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx3 __attribute__((ext_vector_type(3)));

struct StemDirectArgs {
    const float *X;   // [N, IH, IW, 4]
    const float *W;   // [OC, FH, FW, 4]
    float *Y;         // [M, OC] dense
    int M, IH, IW, OC;
    int FH, FW, taps, sh, sw, ph, pw;
    int x_bytes, w_bytes, y_bytes;
    int tiles, nblocks, groups, items, wgs;   // items = nblocks * groups
    int TPR, rows;    // OW % 16 == 0: tiles per output row and output rows N * OH; else TPR = 0
    FastDiv d_TPR;
    FastDiv d_OW, d_OHW, d_FW, d_OH;
    Epilogue ep;
};

template <int V> struct SdInt { static constexpr int value = V; };
constexpr unsigned SD_NEVER = 0x80000000u;   // beyond every descriptor (tensors below 2 GB, host-checked)

// Bits f < F (F <= 15) with 0 <= x0 + f < L: the window positions inside the image along one axis.
__device__ inline unsigned sd_range_mask(int x0, int F, int L)   // works on uniform and on per-lane values
{
    const int lo = max(0, -x0), hi = min(F, L - x0);
    return hi > lo ? ((1u << hi) - 1u) & ~((1u << lo) - 1u) : 0u;
}

// G: tap groups (ceil(taps / 4)). Eight wavefronts per workgroup, two per SIMD; the items (block of 64 output channels,
// tile of 16 pixels) are dealt to the workgroups as contiguous shares equal to within one.
template <int G, bool EPI>
__global__ __launch_bounds__(512, 1) void stem_direct_kernel(const StemDirectArgs p)
{
    __shared__ int any_ch3;
    const int t = threadIdx.x, lane = t & 63;
    const int l16 = lane & 15, q = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int i_lo = (int)((long)p.items * blockIdx.x / p.wgs), i_hi = (int)((long)p.items * (blockIdx.x + 1) / p.wgs);

    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.X), 0, p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.W), 0, p.w_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.Y, 0, p.y_bytes, 0x00020000);

    // ---- does any weight of the fourth stored channel differ from zero? (layers with three logical channels arrive with
    // it zero-filled in X and W: its MFMA step, a quarter of all, is then left out) ---------------------------------------
    if (t == 0) any_ch3 = 0;
    __syncthreads();
    {
        int nz = 0;
        const int n_taps_all = p.OC * p.taps;
        for (int idx = t; idx < n_taps_all; idx += 512) nz |= p.W[(size_t)idx * 4 + 3] != 0.f;
        if (nz) any_ch3 = 1;   // every writer writes the same value
    }
    __syncthreads();
    const bool use_ch3 = any_ch3 != 0;

    // ---- per-lane tap data: byte offset of tap 4g + q from a window's origin, and the window row / column it needs --------
    int toff[G];
    unsigned need[G];
#pragma unroll
    for (int g = 0; g < G; g++) {
        // the last group is the last tap alone (taps = 4 (G - 1) + 1, host-checked): there the reduction index of the MFMA
        // is the CHANNEL, lane (l16, q) loads channel q of that tap's pixel - one MFMA per tile and j, not one per channel
        const int tap = g < G - 1 ? 4 * g + q : 4 * g;
        const int fh = fdiv(tap, p.d_FW), fw = tap - fh * p.FW;
        toff[g] = (fh * p.IW + fw) * 16 + (g < G - 1 ? 0 : 4 * q);
        need[g] = (1u << fh) | (1u << (16 + fw));
    }

    // The tiles of group gidx. Where the rows are whole tiles (OW % 16 == 0) a group is the same 16 columns of four
    // consecutive output rows - their windows overlap most, and whether every tap of every pixel lies inside the image is
    // then the same question for all four: true for most groups, which take the short way in `request` below -; else
    // four consecutive tiles. Tiles past the end get the index p.tiles: no live pixel, nothing stored.
    auto tile_of = [&](const int gidx, const int i) {   // uniform
        if (p.TPR > 0) {
            const int sb = fdiv(gidx, p.d_TPR), tx = gidx - sb * p.TPR, row = 4 * sb + i;
            return row < p.rows ? row * p.TPR + tx : p.tiles;
        }
        const int tl = 4 * gidx + i;
        return tl < p.tiles ? tl : p.tiles;
    };
    // `count` groups of T tiles. T = 4: groups g0 + first, g0 + first + 8, ...; T = 1: the single tiles number first,
    // first + 8, ... of the groups from g0 on (tile k belongs to group g0 + k / 4).
    auto run = [&](auto tc, auto scc, const int nb, const int g0, const int first, const int count) {
        constexpr int T = decltype(tc)::value;
        constexpr int SC = decltype(scc)::value;
        if (count <= 0) return;
        const int n_l = nb * 64 + 4 * l16;
        const bool n_ok = n_l < p.OC;   // OC % 4 == 0: a lane's four channels are valid together
        unsigned b_voff[4];
#pragma unroll
        for (int j = 0; j < 4; j++) b_voff[j] = n_ok ? (unsigned)(((n_l + j) * p.taps + q) * 16) : SD_NEVER;
        const bool last_ok = q < SC;   // the last step's channel q exists (with three channels the fourth is never read)
        const unsigned o_lane = n_ok ? (unsigned)((4 * q * p.OC + n_l) * 4) : SD_NEVER;
        float sub[4], mul[4], add[4];
        floatx4 bias = floatx4{0.f, 0.f, 0.f, 0.f};
        if (EPI) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                sub[j] = 0.f; mul[j] = 1.f; add[j] = 0.f;
                if (n_ok && !p.ep.gate) ep_channel(p.ep, n_l + j, sub[j], mul[j], add[j]);
            }
        } else if (p.ep.bias != nullptr && n_ok) {
            bias = *reinterpret_cast<const floatx4 *>(p.ep.bias + n_l);
        }

        // three channels: 96-bit loads, so that the unused fourth component takes no registers
        using frag = std::conditional_t<SC == 3, floatx3, floatx4>;
        frag a[2][T], b[2][4];
        // ---- load cursor: one step ahead of the multiplications ------------------------------------------------------------
        int c_idx = first, c_groups_left = count;
        bool c_inside = false;   // every tap of every pixel of the cursor's tiles lies inside the image (uniform)
        auto tile_at = [&](const int idx, const int i) { return T == 4 ? tile_of(g0 + idx, i) : tile_of(g0 + (idx >> 2), idx & 3); };
        int org[T];       // byte offset of this lane's pixel's window origin; may lie before the tensor
        unsigned rc[T];   // bit fh: window row fh is inside the image; bit 16 + fw: window column fw is
        const unsigned full = ((1u << p.FH) - 1u) | (((1u << p.FW) - 1u) << 16);
        auto locate = [&]() {
            bool all_full = true;
            if (p.TPR > 0) {
                // rows are whole tiles and a group is the same 16 columns of consecutive output rows: the columns - the only
                // per-lane part - are worked out once per group, the image and the window rows of each tile in scalar
                // arithmetic
                const int gidx = __builtin_amdgcn_readfirstlane(T == 4 ? g0 + c_idx : g0 + (c_idx >> 2));
                const int sb = fdiv(gidx, p.d_TPR), tx = gidx - sb * p.TPR;
                const int iw0 = (tx * 16 + l16) * p.sw - p.pw;
                const unsigned cols_in = sd_range_mask(iw0, p.FW, p.IW) << 16;
                const int col_off = iw0 * 16;
                bool rows_full = true;
#pragma unroll
                for (int i = 0; i < T; i++) {
                    const int row = 4 * sb + (T == 4 ? i : (c_idx & 3));
                    const bool live = row < p.rows;
                    const int n = fdiv(live ? row : 0, p.d_OH), oh = (live ? row : 0) - n * (int)p.d_OH.d;
                    const int ih0 = oh * p.sh - p.ph;
                    const unsigned rows_in = live ? sd_range_mask(ih0, p.FH, p.IH) : 0u;
                    org[i] = __builtin_amdgcn_readfirstlane((n * p.IH + ih0) * p.IW * 16) + col_off;
                    rc[i] = (unsigned)__builtin_amdgcn_readfirstlane((int)rows_in) | cols_in;
                    rows_full = rows_full && rows_in == (full & 0xffffu);
                }
                c_inside = rows_full && __all(cols_in == (full & 0xffff0000u)) != 0;
                return;
            }
#pragma unroll
            for (int i = 0; i < T; i++) {
                const int m = tile_at(c_idx, i) * 16 + l16;
                const bool live = m < p.M;
                const int mm = live ? m : 0;
                const int n = fdiv(mm, p.d_OHW), rem = mm - n * (int)p.d_OHW.d;
                const int oh = fdiv(rem, p.d_OW), ow = rem - oh * (int)p.d_OW.d;
                const int ih0 = oh * p.sh - p.ph, iw0 = ow * p.sw - p.pw;
                org[i] = ((n * p.IH + ih0) * p.IW + iw0) * 16;
                rc[i] = (live ? sd_range_mask(ih0, p.FH, p.IH) : 0u) | (sd_range_mask(iw0, p.FW, p.IW) << 16);
                all_full = all_full && rc[i] == full;
            }
            c_inside = __all(all_full) != 0;
        };
        auto request = [&](int slot, auto gc) {   // the loads of tap group g of the cursor's tiles
            constexpr int g = decltype(gc)::value;
            unsigned voff[T];
            if (c_inside) {   // uniform: one addition per tile (taps past the last, in the last group, stay out of range)
#pragma unroll
                for (int i = 0; i < T; i++)
                    voff[i] = (g == G - 1 && !last_ok) ? SD_NEVER : (unsigned)(org[i] + toff[g]);
            } else {
#pragma unroll
                for (int i = 0; i < T; i++)
                    voff[i] = ((rc[i] & need[g]) == need[g] && (g < G - 1 || last_ok)) ? (unsigned)(org[i] + toff[g]) : SD_NEVER;
            }
            if constexpr (g == G - 1) {   // one channel of the last tap per lane, into component 0
#pragma unroll
                for (int i = 0; i < T; i++) a[slot][i][0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(x_rsrc, voff[i], 0, 0));
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const unsigned bv = last_ok ? b_voff[j] - (unsigned)(12 * q) : SD_NEVER;   // tap 4 (G - 1) of the lane's channel, its component q
                    b[slot][j][0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(w_rsrc, bv, g * 64, 0));
                }
                return;
            }
#pragma unroll
            for (int i = 0; i < T; i++) {
                if constexpr (SC == 3) a[slot][i] = __builtin_bit_cast(floatx3, __builtin_amdgcn_raw_buffer_load_b96(x_rsrc, voff[i], 0, 0));
                else a[slot][i] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, voff[i], 0, 0));
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if constexpr (SC == 3) b[slot][j] = __builtin_bit_cast(floatx3, __builtin_amdgcn_raw_buffer_load_b96(w_rsrc, b_voff[j], g * 64, 0));
                else b[slot][j] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, b_voff[j], g * 64, 0));
            }
        };
        floatx4 acc[T][4];
        auto multiply = [&](int slot, const int channels) {   // channels: SC, or 1 in the last step (component 0 = the lane's channel)
#pragma unroll
            for (int s = 0; s < channels; s++)
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int i = 0; i < T; i++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[slot][i][s], b[slot][j][s], acc[i][j], 0, 0, 0);
        };
        // one group of tiles; P: the register set that holds its first step
        auto group = [&](auto pc, const int idx) {
            constexpr int P = decltype(pc)::value;
#pragma unroll
            for (int i = 0; i < T; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
            auto step = [&](auto kc, auto self) {
                constexpr int k = decltype(kc)::value;
                if constexpr (k < G) {
                    if constexpr (k + 1 < G) {
                        request((P + k + 1) & 1, SdInt<k + 1>{});
                    } else {
                        // the first step of the next group of tiles (past the last group: this group's again, unused)
                        if (c_groups_left > 1) {
                            c_groups_left--;
                            c_idx += 8;
                            locate();
                        }
                        request((P + k + 1) & 1, SdInt<0>{});
                    }
                    multiply((P + k) & 1, k < G - 1 ? SC : 1);
                    __builtin_amdgcn_sched_barrier(0);
                    self(SdInt<k + 1>{}, self);
                }
            };
            step(SdInt<0>{}, step);
            // ---- results: lane holds pixels 16 (tile + i) + 4q + r, output channels 64 nb + 4 l16 + j ------------------------
#pragma unroll
            for (int i = 0; i < T; i++) {
                const int tile = tile_at(idx, i);
                if (tile >= p.tiles) continue;   // uniform
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int o_off = __builtin_amdgcn_readfirstlane((tile * 16 + r) * p.OC * 4);   // rows past M: beyond the descriptor
                    floatx4 v = floatx4{acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]};
                    if (EPI) {
                        if (p.ep.gate) {   // uniform
                            const floatx4 gt = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(
                                __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.ep.gate), 0, p.y_bytes, 0x00020000), o_lane, o_off, 0));
#pragma unroll
                            for (int j = 0; j < 4; j++) v[j] = ep_gate(v[j], gt[j], p.ep.slope);
                        } else {
#pragma unroll
                            for (int j = 0; j < 4; j++) v[j] = ep_finish(v[j], sub[j], mul[j], add[j], p.ep.slope);
                        }
                    } else {
                        v += bias;   // zeros without a bias: the additions gather the lane's four channels into the store's registers anyway
                    }
                    // streamed out (non-temporal): 64 channels per pixel of a stem's large map, 205 MB at 224x224, N = 64, that this
                    // kernel never reads again and that would only displace the input's rows from L2 (0.1232 -> 0.1220 ms)
                    buffer_store_b128_guarded<2>(v, y_rsrc, o_lane, o_off);
                }
            }
        };
        locate();
        request(0, SdInt<0>{});
        for (int g2 = 0; g2 < count; g2++) {
            if ((G & 1) && (g2 & 1)) group(SdInt<1>{}, first + 8 * g2);
            else group(SdInt<0>{}, first + 8 * g2);
        }
    };

    // The workgroup's share as runs of groups of one block of output channels each (item = nb * groups + group). A run's
    // groups are dealt to the eight wavefronts round-robin, so that at any time the workgroup works on neighbouring
    // tiles, whose windows overlap (rows oh and oh + 1 of a 7x7 stride-2 layer share five of seven input rows): the
    // re-reads then hit the L2 of the workgroup's XCD. The groups dealt out whole are a multiple of four, so that every
    // SIMD (wavefronts w and w + 4) gets the same number; the tiles of the up to three groups left go out one by one.
    int i = i_lo;
    while (i < i_hi) {
        const int nb = i / p.groups, g0 = i - nb * p.groups;
        const int cnt = min(i_hi - i, p.groups - g0);
        const int n4 = cnt & ~3;
        const int mine4 = n4 > w ? (n4 - w + 7) >> 3 : 0;
        const int rest = 4 * (cnt - n4), mine1 = rest > w ? (rest - w + 7) >> 3 : 0;
        if (use_ch3) {
            run(SdInt<4>{}, SdInt<4>{}, nb, g0, w, mine4);
            run(SdInt<1>{}, SdInt<4>{}, nb, g0 + n4, w, mine1);
        } else {
            run(SdInt<4>{}, SdInt<3>{}, nb, g0, w, mine4);
            run(SdInt<1>{}, SdInt<3>{}, nb, g0 + n4, w, mine1);
        }
        i += cnt;
    }
}

// Y[N, OH, OW, OC] = convolution of X[N, IH, IW, 4] with W[OC, FH, FW, 4] (stride sh x sw, padding ph x pw). Returns
// hipErrorNotSupported (nothing launched) when the layer does not fit: a filter of other than 49 or 9 taps, tensors of 2 GB.
hipError_t launch_stem_direct(hipStream_t stream, const float *X, const float *W, float *Y, int N, int IH, int IW, int OH, int OW,
                              int OC, int FH, int FW, int sh, int sw, int ph, int pw, const float *bias, const Epilogue *ep)
{
    const int taps = FH * FW, G = (taps + 3) / 4;
    if ((taps != 49 && taps != 9) || FH > 15 || FW > 15 || OC < 4 || (OC & 3)) return hipErrorNotSupported;   // 4 (G - 1) + 1 taps
    const long M = (long)N * OH * OW;
    const long x_bytes = (long)N * IH * IW * 16, w_bytes = (long)OC * taps * 16, y_bytes = M * OC * 4;
    if (M < 1 || x_bytes >= (1L << 31) || y_bytes >= (1L << 31) || w_bytes >= (1L << 30)) return hipErrorNotSupported;
    const int cus = device_cu_count();
    if (cus < 1) return hipErrorNotSupported;
    StemDirectArgs a{};
    a.X = X; a.W = W; a.Y = Y;
    a.M = (int)M; a.IH = IH; a.IW = IW; a.OC = OC;
    a.FH = FH; a.FW = FW; a.taps = taps; a.sh = sh; a.sw = sw; a.ph = ph; a.pw = pw;
    a.x_bytes = (int)x_bytes; a.w_bytes = (int)w_bytes; a.y_bytes = (int)y_bytes;
    a.tiles = (int)((M + 15) / 16);
    a.nblocks = (OC + 63) / 64;
    if ((long)a.tiles * a.nblocks >= (1L << 30)) return hipErrorNotSupported;
    if ((OW & 15) == 0) {   // rows are whole tiles: a group is the same 16 columns of four consecutive output rows
        a.TPR = OW / 16;
        a.rows = N * OH;
        a.groups = ((a.rows + 3) / 4) * a.TPR;
    } else {
        a.TPR = 0;
        a.rows = 0;
        a.groups = (a.tiles + 3) / 4;
    }
    a.d_TPR = make_fastdiv(a.TPR > 0 ? a.TPR : 1);
    a.items = a.groups * a.nblocks;
    a.d_OW = make_fastdiv(OW);
    a.d_OHW = make_fastdiv(OH * OW);
    a.d_FW = make_fastdiv(FW);
    a.d_OH = make_fastdiv(OH);
    a.ep = ep ? *ep : bias_epilogue(bias);
    int wgs = cus;   // one workgroup of eight wavefronts per compute unit
    if (wgs * 2 > a.items) wgs = (a.items + 1) / 2;
    a.wgs = wgs;
    if (G == 13) {
        if (a.ep.fused) hipLaunchKernelGGL((stem_direct_kernel<13, true>), dim3(wgs), dim3(512), 0, stream, a);
        else hipLaunchKernelGGL((stem_direct_kernel<13, false>), dim3(wgs), dim3(512), 0, stream, a);
    } else {
        if (a.ep.fused) hipLaunchKernelGGL((stem_direct_kernel<3, true>), dim3(wgs), dim3(512), 0, stream, a);
        else hipLaunchKernelGGL((stem_direct_kernel<3, false>), dim3(wgs), dim3(512), 0, stream, a);
    }
    return hipGetLastError();
}

}  // namespace alpha
