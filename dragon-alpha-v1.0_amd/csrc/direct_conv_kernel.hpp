// (Arguments and kernel of direct_conv.hip and direct_conv_narrow.hip.)
// Convolution with both operands straight from memory - no LDS, no barrier -, fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950.
// Any filter size, stride and padding; filter with the produced channel contiguous (CW[FH, FW, IC, OC] forward,
// W[OC, FH, FW, IC] rotated by 180 degrees for stride-1 backward-data).
//
//   O[m, co] = sum over taps (th, tw) and channels c of A[n, oh*sh - ph + th, ow*sw - pw + tw, c] * B[(th, tw), c, co]
//
// For whom: strided layers. A stride-2 3x3 layer touches every input pixel 2.25 times, so a halo in LDS buys little
// and costs a lot (four input pixels per output pixel: the LDS-halo kernel's unit of 112 output pixels needs 150 KB,
// one workgroup per compute unit, nothing overlaps its staging). Here an input pixel's re-reads come out of L1 / L2.
//
// The pointwise_direct.hip scheme with a tap loop around it: a wavefront owns T <= 4 tiles of 16 output pixels and one
// block of 64 produced channels; per step (one tap, 16 reduced channels)
//   a_t = A[pixel l16 of tile t at this tap][16c + 4q .. +3]       one 128-bit load per tile
//   b_s = B[tap][16c + 4q + s][n0 + 4*l16 .. +3], s = 0..3           four 128-bit loads, shared by the T tiles
// and MFMA (t, s, j) multiplies component s of a_t with component j of b_s: 16 T MFMAs per T + 4 loads. A lane's
// accumulators are 4 consecutive produced channels of a pixel: results leave as 128-bit stores without a transpose.
// Where a tile's pixels are (they may straddle image rows and images) is worked out per lane once per group of tiles;
// per tap a lane's load offset is that origin plus the tap's (uniform) term, or an offset beyond the buffer descriptor
// where the tap falls into the padding (the load then returns zeros): five vector instructions per tile and tap, none
// per load. Loads run one step ahead of the multiplications through a cursor over (group, tap, channels), so the
// pipeline does not drain between tiles.
//
// Work items are (block of produced channels, tile). A workgroup's share is a contiguous range of them: an even number
// per SIMD is processed whole (a wavefront's part as groups of 4, 3, 2 or 1 tiles with one loop per group size, every
// load and store unconditional, every wait an exact count), and the up to seven items left over are processed by the
// whole workgroup together, the reduction (taps x channels) cut into eight parts, the partial sums added through LDS.
#pragma once
#include "common.hpp"

namespace alpha {

typedef float floatx4 __attribute__((ext_vector_type(4)));

struct DirectConvArgs {
    const float *A;   // [N, AH, AW, AC]
    const float *B;   // element (tap, c, co) at b_off + tap * b_tap + c * b_k + co (floats); b_tap may be negative
    float *O;         // [M, CO] dense
    int M, AH, AW, AC, CO;
    int TH, TW, sh, sw, ph, pw;
    int b_off, b_tap, b_k;
    int a_bytes, b_bytes, o_bytes;
    int tiles, nblocks, items, wgs;
    // Shares equal to the item: with a workspace every workgroup takes `base` items and the items_left = items - wgs * base
    // left over are cut `split` ways along the reduction, one piece each for the first items_left * split workgroups; piece
    // (item e, part z) leaves its partial sums in ws[(e * split + z) * 1024 ..]. Who adds them: with `tickets` (one word per
    // item left over, zero before the launch and after it) the workgroup that delivers an item's last piece; without,
    // direct_conv_fixup_kernel in a second launch. The order of the addition is z = 0, 1, ... either way.
    float *ws;
    unsigned *tickets;
    int base, items_left, split;
    int xcd_major;   // shares dealt XCD by XCD (see the kernel)
    FastDiv d_OW, d_OHW, d_TW;
    Epilogue ep;
};

template <int V> struct DcInt { static constexpr int value = V; };
template <bool V> struct DcBool { static constexpr bool value = V; };
constexpr unsigned DC_NEVER = 0x80000000u;   // beyond every descriptor (tensors below 2 GB, host-checked)

constexpr int DC_AUX_SC1 = 16;   // cache-policy bit of the buffer instructions: coherent at device scope (across the XCDs' L2s)
constexpr int DC_SPLIT_T = 4;   // tiles per group where the workgroup shares the reduction (LDS: 8 x 4 DC_SPLIT_T x 1 KB)
constexpr size_t DC_LDS_BYTES = 8 * 4 * DC_SPLIT_T * 64 * sizeof(floatx4);

// A workgroup has eight wavefronts, two per SIMD (wavefronts w and w + 4 of a workgroup run on SIMD w % 4). What must be
// even is the work per SIMD. A workgroup's n items: f = the largest even number with 4 f <= n go whole to each SIMD, half
// to each of its two wavefronts (both stay busy to the end: a wavefront alone on a SIMD fills the MFMA pipe less well),
// but none where that would be a single item per wavefront (groups of one tile: five loads per 16 MFMAs, where a group of
// four tiles has eight per 64); the items left - fewer than 8, or all n < 16 - are processed by all eight wavefronts together
// in groups of up to four tiles, wavefront w on part 2 (w % 4) + w / 4 of
// eight parts of the reduction steps - a SIMD's two parts together are a quarter of the steps -, and the eight partial
// results are added through LDS in a fixed order. 12544 items on 256 workgroups: 49 = 4 x 12 + 1 per workgroup, 12.25
// per SIMD, where whole items alone would make it 13 on some SIMDs.
// Bits f < F (F <= 16) with 0 <= x0 + f < L: the window positions inside the image along one axis.
__device__ inline unsigned dc_range_mask(int x0, int F, int L)
{
    const int lo = max(0, -x0), hi = min(F, L - x0);
    return hi > lo ? ((1u << hi) - 1u) & ~((1u << lo) - 1u) : 0u;
}

// whole items per SIMD of a workgroup with n items
__host__ __device__ inline int dc_whole_items(int n)
{
    const int f = (n >> 2) & ~1;
    return f < 4 ? 0 : f;
}

// O[item's 16 pixels][its 64 channels] = epilogue(sum over z < split of ws[(e * split + z)][16][64]), the pieces added in
// the order z = 0, 1, ...: 256 threads per item left over, a thread per 128-bit store. COHERENT: the pieces were written
// during this launch, possibly through another XCD's L2 - read them at device scope.
template <bool COHERENT>
__device__ __forceinline__ void dc_add_pieces(const DirectConvArgs &p, const int e, const int t)
{
    const int row = t >> 4, c4 = t & 15;
    const int item = p.wgs * p.base + e;
    const int nb = item / p.tiles, tile = item - nb * p.tiles;
    const __amdgpu_buffer_rsrc_t ws_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.ws, 0, p.items_left * p.split * 4096, 0x00020000);
    const unsigned src = (unsigned)(((e * p.split * 16 + row) * 64 + 4 * c4) * 4);
    // all pieces requested before the first addition (split <= 8; the loads past the last piece repeat it, unused)
    floatx4 piece[8];
#pragma unroll
    for (int z = 0; z < 8; z++)
        piece[z] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(ws_rsrc, src, (z < p.split ? z : p.split - 1) * 4096,
                                                                                      COHERENT ? DC_AUX_SC1 : 0));
    floatx4 v = piece[0];
#pragma unroll
    for (int z = 1; z < 8; z++)
        if (z < p.split) v += piece[z];   // uniform
    const int m = tile * 16 + row, col = nb * 64 + 4 * c4;
    if (m < p.M && col < p.CO) {
        const size_t elem = (size_t)m * p.CO + col;
        const float4 r = epilogue4(make_float4(v[0], v[1], v[2], v[3]), p.ep, col, elem);
        *reinterpret_cast<float4 *>(p.O + elem) = r;
    }
}

// NJ produced channels of a lane as the low components of a float4: one 128-, 96-, 64- or 32-bit load (the builtin's result
// converted as a whole: indexed element by element it compiles to a load of the first word only).
template <int NJ>
static __device__ __forceinline__ floatx4 dc_load(__amdgpu_buffer_rsrc_t rsrc, unsigned voffset, int soffset)
{
    if constexpr (NJ == 4) {
        return __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voffset, soffset, 0));
    } else if constexpr (NJ == 3) {
        typedef float floatx3 __attribute__((ext_vector_type(3)));
        const floatx3 v = __builtin_bit_cast(floatx3, __builtin_amdgcn_raw_buffer_load_b96(rsrc, voffset, soffset, 0));
        return floatx4{v[0], v[1], v[2], 0.f};
    } else if constexpr (NJ == 2) {
        typedef float floatx2 __attribute__((ext_vector_type(2)));
        const floatx2 v = __builtin_bit_cast(floatx2, __builtin_amdgcn_raw_buffer_load_b64(rsrc, voffset, soffset, 0));
        return floatx4{v[0], v[1], 0.f, 0.f};
    } else {
        return floatx4{__builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, voffset, soffset, 0)), 0.f, 0.f, 0.f};
    }
}

// NJ: produced channels per lane, 1 to 4 - a block of produced channels is 16 NJ wide and a step costs 4 NJ MFMAs a tile.
// 4 = the 64-wide blocks; 96 produced channels are two blocks of 48 with NJ = 3 instead of one full and one half-empty
// block of 64. (NJ < 4 without the lent scratch, whose pieces are 64 wide.)
// ODD: for layers with an odd number of steps per item (48 channels under a 3x3 filter: 27; 48 under a 1x1 filter: 3). The
// loop over whole items multiplies two steps per turn; here an item's steps are followed by one empty step - its loads
// of A lie beyond the descriptor and return zeros - so that such layers have whole items too. (Without it all their items
// are shared by the workgroup's eight wavefronts in runs of a single group: 1x1 48 -> 192 on 64x28x28 pixels 0.028 ms
// where 32 -> 192 takes 0.014.) Without the lent scratch.
template <bool EPI, bool WS = false, int NJ = 4, bool ODD = false>
__global__ __launch_bounds__(512, 1) void direct_conv_kernel(const DirectConvArgs p)
{
    static_assert(NJ == 4 || !WS, "pieces in the lent scratch are 64 channels wide");
    static_assert(!ODD || !WS, "the form with an empty step takes no lent scratch");
    extern __shared__ __attribute__((aligned(16))) float dc_smem[];
    floatx4 *part = reinterpret_cast<floatx4 *>(dc_smem);   // [8 wavefronts][4 DC_SPLIT_T units][64 lanes]
    const int t = threadIdx.x, lane = t & 63;
    const int l16 = lane & 15, q = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);
    // Workgroups go round-robin to the eight XCDs, each with its own L2. Where a workgroup holds few items and the filter
    // is larger than an L2 (xcd_major) share sb of the line of items goes to workgroup (sb % (wgs / 8)) * 8 +
    // sb / (wgs / 8): an XCD's workgroups then hold neighbouring shares, one or two blocks' filters per L2 instead of all.
    const int sb = p.xcd_major ? (int)(blockIdx.x & 7) * (p.wgs >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    const int g_lo = WS ? sb * p.base : (int)((long)p.items * sb / p.wgs);
    const int g_hi = WS ? g_lo + p.base : (int)((long)p.items * (sb + 1) / p.wgs);
    // An odd number of steps per item (48 channels under a 3x3 filter: 27): the loop over whole items multiplies two steps
    // per turn, so such a layer has no whole items - all of them are shared, in runs of a single group, whose parts
    // may be odd.
    const int f = (!ODD && (((p.AC >> 4) * p.TH * p.TW) & 1)) ? 0 : dc_whole_items(g_hi - g_lo);
    const int i_lo = g_lo + (w & 3) * f + (w >> 2) * (f >> 1), i_hi = i_lo + (f >> 1);
    const int CH = p.AC >> 4, taps = p.TH * p.TW, KS = taps * CH;   // steps per group
    const int KW = ODD ? KS + 1 : KS;                                // the same with the empty step, for whole items
    const bool pointwise = taps == 1 && p.sh == 1 && p.sw == 1 && p.ph == 0 && p.pw == 0;

    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.A), 0, p.a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.B), 0, p.b_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t o_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.O, 0, p.o_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ws_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.ws, 0, WS ? p.items_left * p.split * 4096 : 0, 0x00020000);

    // `count` groups of T tiles each, from tile0 on, block nb of the produced channels, reduction steps [k_lo, k_lo + k_n)
    // of every group. SPLIT (every wavefront of the workgroup calls it with its own steps; count 1 and k_n >= 0 of either
    // parity, or several groups and k_n even and at least 2): the wavefronts' partial results are added through LDS, and
    // the first loads of the next group are in flight meanwhile. Otherwise k_n is even and at least 2.
    int ep_nb = -1;   // the block of produced channels the epilogue terms below belong to
    float sub[4], mul[4], add[4];
    floatx4 bias = floatx4{0.f, 0.f, 0.f, 0.f};
    // The groups of a run begin `stride` tiles apart (T: one after the other).
    auto run = [&](auto tc, auto sp, const int nb, const int tile0, const int count, const int k_lo, const int k_n, const int stride) {
        constexpr int T = decltype(tc)::value;
        constexpr int MODE = decltype(sp)::value;   // 0: whole items; 1: shared by the workgroup; 2: the same, sums to the workspace; 3: shared by a SIMD's two wavefronts
        constexpr bool SPLIT = MODE != 0;
        if (count <= 0) return;
        const int n_l = nb * 16 * NJ + NJ * l16;
        const unsigned b_lane = n_l < p.CO ? (unsigned)((4 * q * p.b_k + n_l) * 4) : DC_NEVER;
        const unsigned o_lane = n_l < p.CO ? (unsigned)((4 * q * p.CO + n_l) * 4) : DC_NEVER;
        // the epilogue's per-channel terms: once per block of produced channels (they are loaded from memory and the loads
        // are waited for), so that the loop below carries twelve registers, not the epilogue's pointers
        if (nb != ep_nb) {
            ep_nb = nb;
            bias = floatx4{0.f, 0.f, 0.f, 0.f};
            if (EPI) {
#pragma unroll
                for (int j = 0; j < NJ; j++) {
                    sub[j] = 0.f; mul[j] = 1.f; add[j] = 0.f;
                    if (n_l < p.CO && !p.ep.gate) ep_channel(p.ep, n_l + j, sub[j], mul[j], add[j]);
                }
            } else if (p.ep.bias != nullptr && n_l < p.CO) {
                if constexpr (NJ == 4) {
                    bias = *reinterpret_cast<const floatx4 *>(p.ep.bias + n_l);
                } else {
#pragma unroll
                    for (int j = 0; j < NJ; j++) bias[j] = p.ep.bias[n_l + j];
                }
            }
        }
        floatx4 a[2][T], b[2][4];
        // ---- load cursor: one step ahead of the multiplications, through (group, tap, 16 channels) ----------------------
        // (the division runs on the vector unit; without the explicit move to a scalar register the compiler keeps the whole
        // cursor, which restarts from these values at every group, in vector registers)
        const int tap_lo = __builtin_amdgcn_readfirstlane(k_lo / CH), ch_lo = __builtin_amdgcn_readfirstlane(k_lo - tap_lo * CH);
        int c_tile = tile0, c_tap = tap_lo, c_ch = ch_lo, c_left = count * k_n;
        bool c_empty = false;   // ODD, whole items: the step being requested next is an item's empty one
        int org[T];          // byte offset of (this lane's pixel's window origin, channel 4q); may lie before the tensor
        unsigned rc[T];      // bit th: window row th is inside the image; bit 16 + tw: window column tw is
        unsigned voff[T];    // this tap's load offset, or DC_NEVER in the padding
        auto locate = [&]() {
            if (pointwise) {   // uniform: a 1x1 stride-1 layer without padding reads pixel m itself
#pragma unroll
                for (int i = 0; i < T; i++) {
                    const int m = (c_tile + i) * 16 + l16;
                    org[i] = (m * p.AC + 4 * q) * 4;
                    rc[i] = m < p.M ? 0x00010001u : 0u;
                }
                return;
            }
#pragma unroll
            for (int i = 0; i < T; i++) {
                const int m = (c_tile + i) * 16 + l16;
                const bool live = m < p.M;
                const int mm = live ? m : 0;
                const int n = fdiv(mm, p.d_OHW), rem = mm - n * (int)p.d_OHW.d;
                const int oh = fdiv(rem, p.d_OW), ow = rem - oh * (int)p.d_OW.d;
                const int ih0 = oh * p.sh - p.ph, iw0 = ow * p.sw - p.pw;
                org[i] = (((n * p.AH + ih0) * p.AW + iw0) * p.AC + 4 * q) * 4;
                rc[i] = (live ? dc_range_mask(ih0, p.TH, p.AH) : 0u) | (dc_range_mask(iw0, p.TW, p.AW) << 16);
            }
        };
        auto aim = [&]() {   // offsets of tap c_tap
            const int th = fdiv(c_tap, p.d_TW), tw = c_tap - th * p.TW;
            const int term = (th * p.AW + tw) * p.AC * 4;
            const unsigned need = (1u << th) | (1u << (16 + tw));
#pragma unroll
            for (int i = 0; i < T; i++) voff[i] = (rc[i] & need) == need ? (unsigned)(org[i] + term) : DC_NEVER;
        };
        auto request = [&](int slot, const bool wrap = false) {   // wrap (SPLIT): these are the loads of a group's last step
            // past the last step the loads repeat the last step's (unused)
            const int a_off = c_ch * 64;
            const int b_off = __builtin_amdgcn_readfirstlane((p.b_off + c_tap * p.b_tap + c_ch * 16 * p.b_k) * 4);
#pragma unroll
            for (int i = 0; i < T; i++)
                a[slot][i] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, voff[i], a_off, 0));
#pragma unroll
            for (int s = 0; s < 4; s++)
                b[slot][s] = dc_load<NJ>(b_rsrc, b_lane + (unsigned)(s * p.b_k * 4), b_off);
            if (c_left > 1) {   // bookkeeping: scalar, and vector arithmetic without memory operations
                c_left--;
                if (SPLIT && wrap) {   // the next group's steps begin at k_lo again
                    c_tap = tap_lo;
                    c_ch = ch_lo;
                    c_tile += stride;
                    locate();
                    aim();
                } else {
                    c_ch++;
                    if (c_ch == CH) {
                        c_ch = 0;
                        c_tap++;
                        if (ODD && !SPLIT && c_tap == taps && !c_empty) {
                            // the empty step: A out of range for every tile, B once more from the last step's place; the
                            // next turn of the cursor passes the end of the taps again
                            c_empty = true;
                            c_tap = taps - 1;
                            c_ch = CH - 1;
#pragma unroll
                            for (int i = 0; i < T; i++) voff[i] = DC_NEVER;
                        } else {
                            if (!SPLIT && c_tap == taps) {
                                c_empty = false;
                                c_tap = 0;
                                c_tile += stride;
                                locate();
                            }
                            aim();
                        }
                    }
                }
            }
        };
        if (!SPLIT || k_n > 0) {
            locate();
            aim();
            request(0);
        }
        for (int g = 0; g < count; g++) {
            const int tile = tile0 + g * stride;
            floatx4 acc[T][NJ];
#pragma unroll
            for (int i = 0; i < T; i++)
#pragma unroll
                for (int j = 0; j < NJ; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
            auto multiply = [&](int slot) {
#pragma unroll
                for (int s = 0; s < 4; s++)
#pragma unroll
                    for (int j = 0; j < NJ; j++)
#pragma unroll
                        for (int i = 0; i < T; i++)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[slot][i][s], b[slot][s][j], acc[i][j], 0, 0, 0);
            };
            for (int ks = 0; ks + 1 < k_n; ks += 2) {
                request(1, ks + 2 >= k_n);
                multiply(0);
                __builtin_amdgcn_sched_barrier(0);
                request(0);
                multiply(1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (SPLIT && (k_n & 1)) multiply(0);
            // ---- results: lane holds pixels 16(tile + i) + 4q + r, produced channels 64 nb + 4 l16 + j -----------------
            // the NJ produced channels of pixel 4 q + r of tile i, as the low components of a float4
            auto column = [&](const int i, const int r) __attribute__((always_inline)) {
                if constexpr (NJ == 4) {
                    return floatx4{acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]};
                } else {
                    floatx4 v = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = 0; j < NJ; j++) v[j] = acc[i][j][r];
                    return v;
                }
            };
            auto emit = [&](const int i, const int r, floatx4 v) {   // pixel 16 (tile + i) + 4 q + r, channels n_l .. n_l + NJ - 1
                const int o_off = __builtin_amdgcn_readfirstlane(((tile + i) * 16 + r) * p.CO * 4);   // rows past M: beyond the descriptor
                if (EPI) {
                    if (p.ep.gate) {   // uniform
                        const floatx4 gt = dc_load<NJ>(
                            __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.ep.gate), 0, p.o_bytes, 0x00020000), o_lane, o_off);
#pragma unroll
                        for (int j = 0; j < NJ; j++) v[j] = ep_gate(v[j], gt[j], p.ep.slope);
                    } else {
#pragma unroll
                        for (int j = 0; j < NJ; j++) v[j] = ep_finish(v[j], sub[j], mul[j], add[j], p.ep.slope);
                    }
                } else {
                    v += bias;
                }
                // non-temporal: the output is streamed out, nothing of it is read again here, and it does not displace the
                // input's and the filter's lines from L2 (1x1, 256 -> 1024 channels: 0.0523 -> 0.0508 ms; 56x56x64 3x3: 0.1097 -> 0.1087)
                buffer_store_guarded<NJ, 2>(v, o_rsrc, o_lane, o_off);
            };
            if constexpr (!SPLIT) {
#pragma unroll
                for (int i = 0; i < T; i++)
#pragma unroll
                    for (int r = 0; r < 4; r++) emit(i, r, column(i, r));
            } else if constexpr (MODE == 3) {
                // The SIMD's two wavefronts (w and w ^ 4) hold the sums over the first and the second half of the steps:
                // each keeps every other unit u = 4 i + r (w < 4 the even ones), hands the rest to its partner through
                // LDS, adds what it receives and stores its units. One barrier pair per workgroup.
                static_assert(T <= DC_SPLIT_T, "LDS holds 4 DC_SPLIT_T units per wavefront");
                const int keep = w >> 2;
#pragma unroll
                for (int i = 0; i < T; i++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (((4 * i + r) & 1) != keep)   // uniform
                            part[(w * 4 * DC_SPLIT_T + 4 * i + r) * 64 + lane] = column(i, r);
                lds_barrier();
#pragma unroll
                for (int i = 0; i < T; i++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (((4 * i + r) & 1) == keep)   // uniform
                            emit(i, r, column(i, r) + part[((w ^ 4) * 4 * DC_SPLIT_T + 4 * i + r) * 64 + lane]);
                lds_barrier();   // whoever writes `part` next
            } else {
                // unit u = 4 i + r (one 128-bit store per lane); partial results [wavefront][unit][lane]
                static_assert(T <= DC_SPLIT_T, "LDS holds 4 DC_SPLIT_T units per wavefront");
#pragma unroll
                for (int i = 0; i < T; i++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        part[(w * 4 * DC_SPLIT_T + 4 * i + r) * 64 + lane] = column(i, r);
                lds_barrier();   // orders LDS only: the next group's loads and this group's stores stay in flight across it
                for (int u = w; u < 4 * T; u += 8) {   // uniform
                    floatx4 v = part[u * 64 + lane];
#pragma unroll
                    for (int x = 1; x < 8; x++) v += part[(x * 4 * DC_SPLIT_T + u) * 64 + lane];
                    if constexpr (MODE == 2) {
                        // row 4 q + (u & 3) of the piece's 16 x 64 block (T == 1), channels 4 l16 .. + 3; `stride` carries the
                        // piece. Stored through to device scope (sc1): the workgroup that adds the pieces may sit on another XCD
                        const unsigned dst = (unsigned)(((stride * 16 + 4 * q + (u & 3)) * 64 + 4 * l16) * 4);
                        buffer_store_b128_guarded<DC_AUX_SC1>(v, ws_rsrc, dst, 0);
                    } else {
                        emit(u >> 2, u & 3, v);
                    }
                }
                lds_barrier();   // the next group writes `part` again
            }
        }
    };

    // The whole items, f / 2 tiles per wavefront as groups of 4, 3, 2 and 1 tiles (4a + 3b for six tiles or more, 3 + 2 for
    // five). Where the workgroup's 4 f tiles lie in one block of produced channels the groups are dealt to the eight
    // wavefronts round-robin - all wavefronts run groups of the same size at the same time, on neighbouring tiles, so the
    // rows their windows share are fetched into L2 once -; else every wavefront takes its f / 2 tiles as one contiguous run.
    auto groups_of = [&](const int cnt, int &n4, int &n3, int &n2, int &n1) {
        n4 = n3 = n2 = n1 = 0;
        if (cnt >= 6) {
            n3 = (4 - (cnt & 3)) & 3;
            n4 = (cnt - 3 * n3) >> 2;
        } else if (cnt == 5) {
            n3 = 1; n2 = 1;
        } else if (cnt == 4) {
            n4 = 1;
        } else if (cnt == 3) {
            n3 = 1;
        } else if (cnt == 2) {
            n2 = 1;
        } else if (cnt == 1) {
            n1 = 1;
        }
    };
    const int nb_first = g_lo / p.tiles;
    // 8 to 15 items (no whole items: one or two per wavefront would be groups of a single tile): every SIMD takes a group
    // of two or three tiles of its own, the steps halved between its two wavefronts - an eighth of the steps per
    // wavefront, as where all eight share a group, costs each of them the group's pixel arithmetic for an eighth of its
    // MFMAs (14x14x256 at N = 64, 12 items per workgroup: 0.50 vector instructions per MFMA).
    const int pc = (f == 0 && g_hi - g_lo >= 8 && g_hi - g_lo < 20 && g_lo + 4 * ((g_hi - g_lo) >> 2) <= (nb_first + 1) * p.tiles) ? (g_hi - g_lo) >> 2 : 0;
    if (pc > 0) {   // uniform
        const int tile0 = g_lo - nb_first * p.tiles + (w & 3) * pc;
        const int h_lo = (w >> 2) ? KS / 2 : 0, h_n = (w >> 2) ? KS - KS / 2 : KS / 2;
        if (pc == 4) run(DcInt<4>{}, DcInt<3>{}, nb_first, tile0, 1, h_lo, h_n, 4);
        else if (pc == 3) run(DcInt<3>{}, DcInt<3>{}, nb_first, tile0, 1, h_lo, h_n, 3);
        else run(DcInt<2>{}, DcInt<3>{}, nb_first, tile0, 1, h_lo, h_n, 2);
    } else if (f > 0 && g_lo + 4 * f <= (nb_first + 1) * p.tiles) {   // uniform
        const int t0 = g_lo - nb_first * p.tiles;
        int n4, n3, n2, n1;
        groups_of(f >> 1, n4, n3, n2, n1);
        int base = t0;
        run(DcInt<4>{}, DcInt<0>{}, nb_first, base + 4 * w, n4, 0, KW, 32);
        base += 32 * n4;
        run(DcInt<3>{}, DcInt<0>{}, nb_first, base + 3 * w, n3, 0, KW, 24);
        base += 24 * n3;
        run(DcInt<2>{}, DcInt<0>{}, nb_first, base + 2 * w, n2, 0, KW, 16);
        base += 16 * n2;
        run(DcInt<1>{}, DcInt<0>{}, nb_first, base + w, n1, 0, KW, 8);
    } else {
        int i = i_lo;
        while (i < i_hi) {
            const int nb = i / p.tiles, tile0 = i - nb * p.tiles;
            const int cnt = min(i_hi - i, p.tiles - tile0);
            int n4, n3, n2, n1;
            groups_of(cnt, n4, n3, n2, n1);
            run(DcInt<4>{}, DcInt<0>{}, nb, tile0, n4, 0, KW, 4);
            run(DcInt<3>{}, DcInt<0>{}, nb, tile0 + 4 * n4, n3, 0, KW, 3);
            run(DcInt<2>{}, DcInt<0>{}, nb, tile0 + 4 * n4 + 3 * n3, n2, 0, KW, 2);
            run(DcInt<1>{}, DcInt<0>{}, nb, tile0 + 4 * n4 + 3 * n3 + 2 * n2, n1, 0, KW, 1);
            i += cnt;
        }
    }
    // the workgroup's items left over (uniform over the workgroup: every wavefront meets the same barriers)
    const int part_idx = 2 * (w & 3) + (w >> 2);
    const int k_lo = KS * part_idx / 8, k_n = KS * (part_idx + 1) / 8 - k_lo;
    int i = g_lo + 4 * (pc > 0 ? pc : f);
    while (i < g_hi) {
        const int nb = i / p.tiles, tile0 = i - nb * p.tiles;
        // groups of sizes equal to within one tile (13 tiles: 4 + 3 + 3 + 3, not 4 + 4 + 4 + 1: a group of one tile pays the
        // first loads and the two barriers for a quarter of the work, with five loads per 16 MFMAs)
        const int run_len = min(g_hi - i, p.tiles - tile0), ngroups = (run_len + DC_SPLIT_T - 1) / DC_SPLIT_T;
        const int cnt = (run_len + ngroups - 1) / ngroups;
        auto groups = [&](const int T, const int first, const int count) {
            if (T == 4) run(DcInt<4>{}, DcInt<1>{}, nb, first, count, k_lo, k_n, 4);
            else if (T == 3) run(DcInt<3>{}, DcInt<1>{}, nb, first, count, k_lo, k_n, 3);
            else if (T == 2) run(DcInt<2>{}, DcInt<1>{}, nb, first, count, k_lo, k_n, 2);
            else if (T == 1) run(DcInt<1>{}, DcInt<1>{}, nb, first, count, k_lo, k_n, 1);
        };
        if ((KS & 15) == 0) {   // every wavefront's part is an even number of steps: groups of one size are one run
            const int n_big = run_len - ngroups * (cnt - 1);   // groups of cnt tiles, the others have cnt - 1
            groups(cnt, tile0, n_big);
            groups(cnt - 1, tile0 + n_big * cnt, ngroups - n_big);
            i += run_len;
        } else {
            groups(cnt, tile0, 1);
            i += cnt;
        }
    }
    if constexpr (WS) {
        // this workgroup's piece of an item left over after the equal shares: part z of `split` of the reduction, cut in
        // eight again among the wavefronts; the sums of the eight go to the workspace, not to O
        if ((int)blockIdx.x < p.items_left * p.split) {   // uniform
            const int e = (int)blockIdx.x / p.split, z = (int)blockIdx.x - e * p.split;
            const int item = p.wgs * p.base + e;
            const int nb = item / p.tiles, tile0 = item - nb * p.tiles;
            const int parts = 8 * p.split, idx = 8 * z + part_idx;
            const int z_lo = (int)((long)KS * idx / parts), z_n = (int)((long)KS * (idx + 1) / parts) - z_lo;
            run(DcInt<1>{}, DcInt<2>{}, nb, tile0, 1, z_lo, z_n, e * p.split + z);
            if (p.tickets != nullptr) {   // uniform over the launch
                // The piece is in memory at device scope once its stores have been acknowledged; then the ticket: the
                // workgroup that draws the last one of an item adds the pieces, in index order whoever it is. Nobody waits
                // for anybody. The ticket word is left zero for the next launch.
                __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
                __builtin_amdgcn_s_barrier();
                int *last = reinterpret_cast<int *>(dc_smem);   // `part` is free: the group ended with a barrier
                if (t == 0)
                    *last = __hip_atomic_fetch_add(p.tickets + e, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)(p.split - 1);
                lds_barrier();
                if (*last) {   // uniform
                    if (t < 256) dc_add_pieces<true>(p, e, t);
                    if (t == 0) __hip_atomic_store(p.tickets + e, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
    }
}

// direct_conv_narrow.hip: the kernels with fewer than four produced channels per lane (no lent scratch)
hipError_t launch_direct_conv_narrow(hipStream_t stream, const DirectConvArgs &a, int nj);
// direct_conv_odd.hip: the kernels for an odd number of steps per item, nj = 1 to 4 produced channels per lane (no lent scratch)
hipError_t launch_direct_conv_odd(hipStream_t stream, const DirectConvArgs &a, int nj);

}  // namespace alpha
