// Kernel-split backward-data (stride > 1) with both operands straight from memory - the phased form of
// direct_conv.hip -, fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950. No LDS, no barrier.
//
// deltaX of a strided layer is sh*sw dense stride-1 problems ("phases"), one per sub-lattice of deltaX, each with its
// own subset of the filter taps. Phase f:
//   O[o_off[f] + n*o_sn + i*o_sh + j*o_sw + co] = sum over th < TH[f], tw < TW[f], c < AC of
//       A[n, i - ph[f] + th, j - pw[f] + tw, c] * B[b_off[f] + th*b_sth[f] + tw*b_stw + c*b_k + co]
// for the "coarse" pixels (n, i, j), i < OHt, j < OWt - the same set for every phase. A work item is (phase, block of
// 64 produced channels, tile of 16 coarse pixels) and costs its phase's number of taps; a wavefront owns T <= 4 tiles of
// one phase at a time and the scheme is direct_conv.hip's: per step (one tap, 16 reduced channels) one 128-bit load per
// tile and four for the filter feed 16 T MFMAs, loads run one step ahead through a cursor over (group, tap, channels),
// results leave as 128-bit stores. A phase without taps (filter smaller than the stride) writes zeros.
//
// Shares: the items in the order (block, chunk of 32 tiles, phase, tile) form a line of cost - an item's steps (taps x
// chunks of 16 reduced channels) plus 2 for its stores -; the wavefronts' shares are equal stretches of it, cut between items. A share then differs from the
// mean by at most one item - a quarter of the cost of a tile with all its phases - and still consists of runs of tiles
// of one phase, so that a filter fragment serves up to four tiles; the line is dealt out XCD by XCD, so the phases of a
// chunk of tiles, which read the same pixels, share an L2 (phase-major order: deltaY fetched 7 times).
// (Whole tiles with all phases: shares of 3 and 4 on 56x56 -> 28x28, 64 channels - 3136 tiles on 1024 SIMDs; shares cut
// inside tiles with the cut tiles run alone: the filter is then read per tile, 0.6 GB from L2, and nothing is gained.)
// Small maps with many channels (14x14x512 <- 7x7 at N = 64: 784 items of up to 128 steps for 1024 SIMDs) have fewer than
// four of their costliest items per SIMD, and shares cut between items are then far from equal. There the line is dealt
// to the workgroups instead, and a workgroup's eight wavefronts work on every group of its items together: the steps
// (tap, 16 channels) of a group cut into eight parts, the partial sums added through LDS in a fixed order.
#include "common.hpp"

namespace alpha {

typedef float floatx4 __attribute__((ext_vector_type(4)));

struct DirectPhasedArgs {
    const float *A;   // [N, AH, AW, AC]
    const float *B;
    float *O;
    int M, AH, AW, AC, CO;   // M = N * OHt * OWt coarse pixels
    int nph;
    int f_TH[4], f_TW[4], f_ph[4], f_pw[4], f_b_off[4], f_b_sth[4], f_o_off[4];
    int b_stw, b_k;
    int o_sn, o_sh, o_sw;
    int a_bytes, b_bytes, o_bytes;
    int tiles, nblocks, items, waves;
    long total_cost;         // items * sum over the phases of (TH * TW * AC / 16 + DCP_STORE_COST)
    int shared;              // the line of items is dealt to the workgroups, whose wavefronts share every group (few items per SIMD)
    FastDiv d_OW, d_OHW;
    Epilogue ep;
};

template <int V> struct DcpInt { static constexpr int value = V; };
constexpr int DCP_TB = 32;                    // tiles per chunk of the line of items
// An item's cost on the line of items: its steps, plus this for its stores (in steps; 1 to 4 measure the same, 6 and 8
// slower, on 56x56x64 <- 28x28x128 3x3 stride 2 and on 1x1 stride 2 layers of 512 to 2048 channels)
constexpr int DCP_STORE_COST = 2;
constexpr size_t DCP_LDS_BYTES = 8 * 16 * 64 * sizeof(floatx4);   // shared groups: [wavefront][unit = 4 tile + r][lane]
constexpr unsigned DCP_NEVER = 0x80000000u;   // beyond every descriptor (tensors below 2 GB, host-checked)

template <bool EPI, bool SHARED = false>
__global__ __launch_bounds__(512, 1) void direct_conv_phased_kernel(const DirectPhasedArgs p)
{
    const int t = threadIdx.x, lane = t & 63;
    const int l16 = lane & 15, q = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(t >> 6);   // wavefronts w and w + 4 of a workgroup share SIMD w % 4
    const int CH = p.AC >> 4;   // even (host-checked): every phase has an even number of steps

    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.A), 0, p.a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.B), 0, p.b_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t o_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.O, 0, p.o_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t g_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(EPI ? p.ep.gate : p.A), 0, EPI ? p.o_bytes : 0, 0x00020000);

    // phase data by (uniform) index
    auto TH = [&](int f) { return f == 0 ? p.f_TH[0] : f == 1 ? p.f_TH[1] : f == 2 ? p.f_TH[2] : p.f_TH[3]; };
    auto TW = [&](int f) { return f == 0 ? p.f_TW[0] : f == 1 ? p.f_TW[1] : f == 2 ? p.f_TW[2] : p.f_TW[3]; };
    auto PH = [&](int f) { return f == 0 ? p.f_ph[0] : f == 1 ? p.f_ph[1] : f == 2 ? p.f_ph[2] : p.f_ph[3]; };
    auto PW = [&](int f) { return f == 0 ? p.f_pw[0] : f == 1 ? p.f_pw[1] : f == 2 ? p.f_pw[2] : p.f_pw[3]; };
    auto BOFF = [&](int f) { return f == 0 ? p.f_b_off[0] : f == 1 ? p.f_b_off[1] : f == 2 ? p.f_b_off[2] : p.f_b_off[3]; };
    auto BSTH = [&](int f) { return f == 0 ? p.f_b_sth[0] : f == 1 ? p.f_b_sth[1] : f == 2 ? p.f_b_sth[2] : p.f_b_sth[3]; };
    auto OOFF = [&](int f) { return f == 0 ? p.f_o_off[0] : f == 1 ? p.f_o_off[1] : f == 2 ? p.f_o_off[2] : p.f_o_off[3]; };

    // `count` groups of T tiles each, from tile0 on, block nb of the produced channels, phase f. SHARED (called by
    // all eight wavefronts of the workgroup): this wavefront multiplies one of eight parts of the group's steps - an even
    // number of them, possibly none - and the eight partial results are added through LDS.
    extern __shared__ __attribute__((aligned(16))) float dcp_smem[];
    floatx4 *part = reinterpret_cast<floatx4 *>(dcp_smem);
    auto run = [&](auto tc, const int f, const int nb, const int tile0, const int count) {
        constexpr int T = decltype(tc)::value;
        if (count <= 0) return;
        const int fTH = TH(f), fTW = TW(f), fPH = PH(f), fPW = PW(f), fBOFF = BOFF(f), fBSTH = BSTH(f);
        // SHARED: part x of the group's pairs of steps, x = 2 (w % 4) + w / 4 - a SIMD's two wavefronts hold neighbouring parts
        const int pairs = (fTH * fTW * CH) >> 1, x = 2 * (w & 3) + (w >> 2);
        const int k_lo = SHARED ? 2 * (pairs * x >> 3) : 0;
        const int steps = SHARED ? 2 * (pairs * (x + 1) >> 3) - k_lo : 2 * pairs;   // steps of a group that this wavefront multiplies
        const int n_l = nb * 64 + 4 * l16;
        const bool n_ok = n_l < p.CO;
        const unsigned b_lane = n_ok ? (unsigned)((4 * q * p.b_k + n_l) * 4) : DCP_NEVER;
        floatx4 a[2][T], b[2][4];
        // ---- load cursor: one step ahead of the multiplications, through (group, phase, tap, 16 channels) ----------------
        int c_tile = tile0, c_th = 0, c_tw = 0, c_ch = 0, c_left = count * steps;
        int th_lo = 0, tw_lo = 0, ch_lo = 0;   // SHARED: step k_lo = ((th_lo * fTW) + tw_lo) * CH + ch_lo, where the cursor begins every group
        if (SHARED && steps > 0) {
            const int tap_lo = __builtin_amdgcn_readfirstlane(k_lo / CH);
            ch_lo = __builtin_amdgcn_readfirstlane(k_lo - tap_lo * CH);
            th_lo = __builtin_amdgcn_readfirstlane(tap_lo / fTW);
            tw_lo = __builtin_amdgcn_readfirstlane(tap_lo - th_lo * fTW);
            c_th = th_lo; c_tw = tw_lo; c_ch = ch_lo;
        }
        int org[T], pi[T], pj[T];   // lane l16's coarse pixel of tile i: byte offset of A[n, i, j, 4q], and (i, j)
        int obase[T];               // where that pixel's results go in O (elements, phase offset and channel apart); dead pixels: beyond O
        unsigned voff[T];           // this tap's load offset, or DCP_NEVER in the padding
        unsigned opix[T][4];        // byte offset of the lane's result pixels 4q + r in O (phase offset apart), or DCP_NEVER
        auto locate = [&]() {
#pragma unroll
            for (int i = 0; i < T; i++) {
                const int m = (c_tile + i) * 16 + l16;
                const bool live = m < p.M;
                const int mm = live ? m : 0;
                const int n = fdiv(mm, p.d_OHW), rem = mm - n * (int)p.d_OHW.d;
                const int ii = fdiv(rem, p.d_OW), jj = rem - ii * (int)p.d_OW.d;
                org[i] = (((n * p.AH + ii) * p.AW + jj) * p.AC + 4 * q) * 4;
                pi[i] = live ? ii : -0x1000000;   // every window row of a dead pixel is outside
                pj[i] = jj;
                obase[i] = live ? n * p.o_sn + ii * p.o_sh + jj * p.o_sw : 0x20000000;
            }
        };
        auto aim = [&]() {   // offsets of tap (c_th, c_tw)
            const int dy = c_th - fPH, dx = c_tw - fPW;
            const int term = (dy * p.AW + dx) * p.AC * 4;
#pragma unroll
            for (int i = 0; i < T; i++) {
                const bool ok = (unsigned)(pi[i] + dy) < (unsigned)p.AH && (unsigned)(pj[i] + dx) < (unsigned)p.AW;
                voff[i] = ok ? (unsigned)(org[i] + term) : DCP_NEVER;
            }
        };
        // `last` (SHARED): the step loaded is the last of this wavefront's part of the group
        auto request = [&](int slot, const bool last = false) {
            // past the last step the loads repeat the last step's (unused)
            const int a_off = c_ch * 64;
            const int b_off = __builtin_amdgcn_readfirstlane((fBOFF + c_th * fBSTH + c_tw * p.b_stw + c_ch * 16 * p.b_k) * 4);
#pragma unroll
            for (int i = 0; i < T; i++)
                a[slot][i] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, voff[i], a_off, 0));
#pragma unroll
            for (int s = 0; s < 4; s++)
                b[slot][s] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, b_lane + (unsigned)(s * p.b_k * 4), b_off, 0));
            if (c_left > 1) {   // bookkeeping: scalar, and vector arithmetic without memory operations
                c_left--;
                if (SHARED && last) {   // the next group, from this wavefront's first step
                    c_th = th_lo; c_tw = tw_lo; c_ch = ch_lo;
                    c_tile += T;
                    locate();
                    aim();
                } else {
                    c_ch++;
                    if (c_ch == CH) {
                        c_ch = 0;
                        c_tw++;
                        if (c_tw == fTW) {
                            c_tw = 0;
                            c_th++;
                            if (!SHARED && c_th == fTH) {   // the next group
                                c_th = 0;
                                c_tile += T;
                                locate();
                            }
                        }
                        aim();
                    }
                }
            }
        };
        if (steps > 0) {
            locate();
            aim();
            request(0);
        }
        for (int g = 0; g < count; g++) {
            const int tile = tile0 + g * T;
            if (steps == 0) {   // a phase without taps has no cursor: place the group's pixels here (uniform)
                c_tile = tile;
                locate();
            }
            // where this lane's results go: pixels 16(tile + i) + 4q + r, produced channels 64 nb + 4 l16 + j. The cursor
            // worked out every pixel's place in O when it reached this group (lane l16 holds pixel l16's; it moves on to the
            // next group's only after this group's first request): pixel 4q + r's comes from lane 4q + r, one cross-lane
            // read instead of two divisions per pixel.
            unsigned mine[2];   // SHARED: this wavefront finishes the units u = 4 i + r = w and w + 8 of the group
            if constexpr (!SHARED) {
#pragma unroll
                for (int i = 0; i < T; i++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int ob = __builtin_amdgcn_ds_bpermute((4 * q + r) * 4, obase[i]);
                        opix[i][r] = n_ok ? (unsigned)((ob + n_l) * 4) : DCP_NEVER;
                    }
            } else {
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int i = (w >> 2) + 2 * h;   // uniform
                    int from = obase[0];
#pragma unroll
                    for (int y = 1; y < T; y++) from = i == y ? obase[y] : from;
                    const int ob = __builtin_amdgcn_ds_bpermute((4 * q + (w & 3)) * 4, from);
                    mine[h] = n_ok && i < T ? (unsigned)((ob + n_l) * 4) : DCP_NEVER;
                }
            }
            {
                floatx4 acc[T][4];
#pragma unroll
                for (int i = 0; i < T; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
                auto multiply = [&](int slot) {
#pragma unroll
                    for (int s = 0; s < 4; s++)
#pragma unroll
                        for (int j = 0; j < 4; j++)
#pragma unroll
                            for (int i = 0; i < T; i++)
                                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[slot][i][s], b[slot][s][j], acc[i][j], 0, 0, 0);
                };
                for (int ks = 0; ks < steps; ks += 2) {
                    request(1, ks + 2 >= steps);
                    multiply(0);
                    __builtin_amdgcn_sched_barrier(0);
                    request(0);
                    multiply(1);
                    __builtin_amdgcn_sched_barrier(0);
                }
                const int o_off = OOFF(f) * 4;
                auto emit = [&](floatx4 v, const unsigned at) __attribute__((always_inline)) {
                    if (EPI) {   // the derivative of the leaky ReLU whose output is this layer's input
                        const floatx4 gt = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(g_rsrc, at, o_off, 0));
#pragma unroll
                        for (int j = 0; j < 4; j++) v[j] = ep_gate(v[j], gt[j], p.ep.slope);
                    }
                    buffer_store_b128_guarded<2>(v, o_rsrc, at, o_off);   // non-temporal, as in direct_conv.hip
                };
                if constexpr (!SHARED) {
#pragma unroll
                    for (int i = 0; i < T; i++)
#pragma unroll
                        for (int r = 0; r < 4; r++) emit(floatx4{acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]}, opix[i][r]);
                } else if (pairs == 0) {
                    // a phase without taps (uniform): nothing to add, every wavefront writes the zeros of its units (from
                    // registers of their own, not a constant the compiler may keep elsewhere: the guarded store holds its
                    // data registers for two wait states)
#pragma unroll
                    for (int h = 0; h < 2; h++)
                        if (w + 8 * h < 4 * T) emit(acc[0][h], mine[h]);
                } else {
                    // unit u = 4 i + r (one 128-bit store per lane); partial results [wavefront][unit][lane], added in the
                    // order of the wavefronts' numbers; wavefront w finishes the units u = w and w + 8
#pragma unroll
                    for (int i = 0; i < T; i++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            part[(w * 16 + 4 * i + r) * 64 + lane] = floatx4{acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]};
                    lds_barrier();   // orders LDS only: the next group's loads and this group's stores stay in flight across it
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const int u = w + 8 * h;
                        if (u < 4 * T) {   // uniform
                            floatx4 v = part[u * 64 + lane];
#pragma unroll
                            for (int y = 1; y < 8; y++) v += part[(y * 16 + u) * 64 + lane];
                            emit(v, mine[h]);
                        }
                    }
                    lds_barrier();   // the next group writes `part` again
                }
            }
        }
    };

    // ---- this wavefront's share: an equal stretch of the line of items, each as long as its cost (its steps
    //      + 2 for its stores), cut between items. The line runs through (block of produced channels, chunk of DCP_TB
    //      tiles, phase, tile): the phases of a chunk of tiles - which read the same pixels of deltaY - lie next to each
    //      other, and the line is dealt to the wavefronts XCD by XCD (workgroups go round-robin to the 8 XCDs, each with
    //      its own L2), so the second to fourth reader of a pixel finds it in L2 ------------------------------------------
    const int G = gridDim.x;
    // A share belongs to a SIMD (what has to be even is the work per SIMD, whose two wavefronts halve it): the items that
    // begin in it differ from the mean by at most one item per SIMD, not per wavefront.
    const int wg_order = (G & 7) == 0 ? (int)(blockIdx.x & 7) * (G >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    const int order = SHARED ? wg_order : wg_order * 4 + (w & 3), shares = SHARED ? G : p.waves;
    const long s_lo = p.total_cost * order / shares, s_hi = p.total_cost * (order + 1) / shares;
    const long s_mid = s_lo + (s_hi - s_lo) / 2;
    // SHARED: the share is the workgroup's, and its wavefronts go through it together
    const long pos_lo = SHARED || w < 4 ? s_lo : s_mid, pos_hi = SHARED || w >= 4 ? s_hi : s_mid;
    int csum = 0;   // cost of a tile with all its phases
    for (int f = 0; f < p.nph; f++) csum += TH(f) * TW(f) * CH + DCP_STORE_COST;
    const long per_nb = (long)p.tiles * csum;
    long pos = pos_lo;
    while (pos < pos_hi) {
        // the (block, chunk, phase) segment that holds position pos
        const int nb = (int)(pos / per_nb);
        const long r = pos - (long)nb * per_nb;
        const int chunk = (int)(r / ((long)DCP_TB * csum));
        const int tile_c = chunk * DCP_TB, tb = min(DCP_TB, p.tiles - tile_c);
        long seg = (long)nb * per_nb + (long)tile_c * csum;   // where the chunk begins
        int f = 0, cost = TH(0) * TW(0) * CH + DCP_STORE_COST;
        while (f + 1 < p.nph && pos >= seg + (long)tb * cost) {
            seg += (long)tb * cost;
            f++;
            cost = TH(f) * TW(f) * CH + DCP_STORE_COST;
        }
        const long seg_end = seg + (long)tb * cost;
        // items of this segment whose beginning lies in [pos_lo, pos_hi)
        const long lo = pos_lo > seg ? pos_lo - seg : 0, hi = min(pos_hi, seg_end) - seg;
        int it = (int)((lo + cost - 1) / cost);
        const int it_end = (int)((hi + cost - 1) / cost);
        // groups of 4, 3, 2 and 1 tiles - 4a + 3b for six tiles or more, 3 + 2 for five
        const int cnt = it_end - it, tile0 = tile_c + it;
        int n4 = 0, n3 = 0, n2 = 0, n1 = 0;
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
        run(DcpInt<4>{}, f, nb, tile0, n4);
        run(DcpInt<3>{}, f, nb, tile0 + 4 * n4, n3);
        run(DcpInt<2>{}, f, nb, tile0 + 4 * n4 + 3 * n3, n2);
        run(DcpInt<1>{}, f, nb, tile0 + 4 * n4 + 3 * n3 + 2 * n2, n1);
        pos = seg_end;
    }
}

// Up to four phases over the coarse pixels (n, i < OHt, j < OWt); see the formula at the top. TH[f] = 0 marks a phase
// without taps (written as zeros). `ep`: NULL, or a gate epilogue (nothing else is applied to backward-data). Returns
// hipErrorNotSupported (nothing launched) when the layer does not fit: more than four phases, AC not a multiple of 32,
// CO not a multiple of 4, tensors of 2 GB.
hipError_t launch_direct_conv_phased(hipStream_t stream, const float *A, const float *B, float *O, int N, int AH, int AW, int AC, int CO,
                                     int OHt, int OWt, int nph, const int *TH, const int *TW, const int *ph, const int *pw,
                                     const int *b_off, const int *b_sth, int b_stw, int b_k, long b_elems,
                                     const int *o_off, int o_sn, int o_sh, int o_sw, long o_elems, const Epilogue *ep, int sharing)
{
    if (nph < 1 || nph > 4 || AC < 32 || (AC & 31) || CO < 4 || (CO & 3) || OHt < 1 || OWt < 1) return hipErrorNotSupported;
    if (ep && ep->fused && !ep->gate) return hipErrorNotSupported;
    const long M = (long)N * OHt * OWt;
    const long a_bytes = (long)N * AH * AW * AC * 4, b_bytes = b_elems * 4, o_bytes = o_elems * 4;
    if (M < 1 || M >= (1L << 30) || a_bytes >= (1L << 31) || o_bytes >= (1L << 31) || b_bytes >= (1L << 30)) return hipErrorNotSupported;
    const int cus = device_cu_count();
    if (cus < 1) return hipErrorNotSupported;
    DirectPhasedArgs a{};
    a.A = A; a.B = B; a.O = O;
    a.M = (int)M; a.AH = AH; a.AW = AW; a.AC = AC; a.CO = CO;
    a.nph = nph;
    long cost = 0, taps = 0;
    for (int f = 0; f < nph; f++) {
        const bool any = TH[f] > 0 && TW[f] > 0;
        if (TH[f] < 0 || TW[f] < 0 || TH[f] > 64 || TW[f] > 64) return hipErrorNotSupported;
        a.f_TH[f] = any ? TH[f] : 0; a.f_TW[f] = any ? TW[f] : 0;
        a.f_ph[f] = ph[f]; a.f_pw[f] = pw[f];
        a.f_b_off[f] = any ? b_off[f] : 0; a.f_b_sth[f] = any ? b_sth[f] : 0;
        a.f_o_off[f] = o_off[f];
        taps += a.f_TH[f] * a.f_TW[f];
        cost += (long)a.f_TH[f] * a.f_TW[f] * (AC >> 4) + DCP_STORE_COST;
    }
    if (taps == 0) return hipErrorNotSupported;
    a.b_stw = b_stw; a.b_k = b_k;
    a.o_sn = o_sn; a.o_sh = o_sh; a.o_sw = o_sw;
    a.a_bytes = (int)a_bytes; a.b_bytes = (int)b_bytes; a.o_bytes = (int)o_bytes;
    a.tiles = (int)((M + 15) / 16);
    a.nblocks = (CO + 63) / 64;
    if ((long)a.tiles * a.nblocks >= (1L << 30) || (long)a.tiles * taps * (AC >> 4) >= (1L << 30)) return hipErrorNotSupported;
    a.items = a.tiles * a.nblocks;
    a.total_cost = (long)a.items * cost;
    a.d_OW = make_fastdiv(OWt);
    a.d_OHW = make_fastdiv(OHt * OWt);
    a.ep = ep ? *ep : bias_epilogue(nullptr);
    int wgs = cus;   // one workgroup of eight wavefronts per compute unit
    if ((long)wgs * 8 > (long)a.items * nph) wgs = (int)(((long)a.items * nph + 7) / 8);   // an item per phase
    a.waves = wgs * 4;   // the SIMDs the line of items is dealt to
    // Fewer than two and a half of the costliest items per SIMD: shares cut between items would be uneven, the
    // workgroups' wavefronts share every group instead. 3x3 stride 2 backward-data, deltaY -> deltaX, shared against own
    // items: 64x7x7x512 -> 14x14x256 (1.8 per SIMD) 0.0709 against 0.0790 ms, 128x4x4x512 -> 8x8x256 (1.2) 0.0450 against
    // 0.0659, 128x8x8x256 -> 16x16x128 (2.4) 0.0493 against 0.0496, 64x14x14x256 -> 28x28x128 (3.6) 0.0772 against 0.0678.
    long cost_max = 0;
    for (int f = 0; f < nph; f++) cost_max = std::max(cost_max, (long)a.f_TH[f] * a.f_TW[f] * (AC >> 4) + DCP_STORE_COST);
    a.shared = sharing < 0 ? 2 * a.total_cost < 5 * cost_max * a.waves : sharing != 0;
    if (a.shared) {
        if (a.ep.fused) {
            if (hipError_t e = ensure_dynamic_lds<direct_conv_phased_kernel<true, true>>(DCP_LDS_BYTES); e != hipSuccess) return e;
            hipLaunchKernelGGL((direct_conv_phased_kernel<true, true>), dim3(wgs), dim3(512), DCP_LDS_BYTES, stream, a);
        } else {
            if (hipError_t e = ensure_dynamic_lds<direct_conv_phased_kernel<false, true>>(DCP_LDS_BYTES); e != hipSuccess) return e;
            hipLaunchKernelGGL((direct_conv_phased_kernel<false, true>), dim3(wgs), dim3(512), DCP_LDS_BYTES, stream, a);
        }
        return hipGetLastError();
    }
    if (a.ep.fused) hipLaunchKernelGGL(direct_conv_phased_kernel<true>, dim3(wgs), dim3(512), 0, stream, a);
    else hipLaunchKernelGGL(direct_conv_phased_kernel<false>, dim3(wgs), dim3(512), 0, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
