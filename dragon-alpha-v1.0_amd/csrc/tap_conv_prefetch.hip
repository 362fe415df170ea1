// Stride-1 tap convolution whose input halo is prefetched: while the MFMA loop works on one pass (32 input channels of
// one unit of pixels), the halo of the next pass - the next 32 channels of the same unit, or the first 32 of the
// workgroup's next unit - is loaded into a second LDS buffer, a few 16-byte elements per thread and tap. The variant
// that stages a whole 64-channel halo between the MFMA loops (tap_conv.hip) left the matrix cores idle for a sixth of
// the time: the two workgroups of a compute unit fall into step (they end their loops together whatever their sizes
// and start times), so both stage and store at the same time, and so does every compute unit of the device, which
// turns the input traffic into bursts.
//
// Same tiling as tap_conv.hip: a workgroup (4 wavefronts) owns P = 16*TILES consecutive output pixels of the flattened
// (n, oh, ow) index and 64 output channels; wavefront w computes channels [16w, 16w+16) of all TILES tiles. The grid is
// persistent; a workgroup's units are known in advance (round-robin within its XCD's run, then at most one piece of a
// left-over unit), which is what lets it fetch the next unit's rows early.
//
// LDS: two buffers of [lds_rows][PWt][40] floats (32 channels + 8: a pixel stride of 160 bytes = 16*(4k+2) keeps the
// 128-bit reads conflict-free) and one spare 16-byte slot. Synchronisation: one barrier per pass (everyone has
// finished reading the current buffer, everyone's prefetch writes into the other one have landed); the output goes
// from the accumulators straight to memory.
//
// Restrictions (the launcher answers hipErrorNotSupported and the caller uses tap_conv.hip): 3x3 taps, stride 1, AC a
// multiple of 32, padded rows of at most 64 pixels, at most 32 halo rows per unit, both buffers within 80 KB.
#include "common.hpp"

namespace alpha {

struct TapPfArgs {
    const float *A;   // input activations [N, AH, AW, AC]
    const float *B;   // filter; element (th, tw, c, co) at b_off + th*b_sth + tw*b_stw + c*b_sc + co*b_sn
    float *O;         // output [N, OH, OW, CO] dense
    Epilogue ep;         // EPI = false: only ep.bias is applied; EPI = true: the whole epilogue
    int M, CO;        // N*OH*OW pixels, output channels
    int AH, AW, AC;
    int TH, TW, ph, pw;
    int PHt, PWt;     // AH + 2ph, AW + 2pw
    int lds_rows;     // halo rows reserved per buffer
    int buf_floats;   // floats per LDS buffer
    int a_bytes;      // size of A, < 2^31
    int b_off, b_sth, b_stw, b_sc, b_sn;   // either b_sn == 1 (output channel contiguous) or b_sc == 1 (input channel contiguous)
    int full_units, pieces, piece_split, piece_tiles;   // as in tap_conv.hip
    FastDiv d_OW, d_OHW, d_PHt;
};

template <int V> struct PfInt { static constexpr int value = V; };
template <int I, int N, class F>
static __device__ __forceinline__ void pf_static_for(F &&f)
{
    if constexpr (I < N) {
        f(PfInt<I>{});
        pf_static_for<I + 1, N>(f);
    }
}
constexpr int PF_ICC = 32;            // input channels per pass
constexpr int PF_PS = PF_ICC + 8;     // LDS pixel stride (floats)
constexpr unsigned PF_OUT_OF_RANGE = 0x80000000u;   // beyond any descriptor (< 2 GB, host-checked): the load returns zeros

// Halo of the pixels [m0, m_hi): first padded global row (n*PHt + ih + ph) and number of rows.
struct PfHalo {
    int pgr0, rows;
};

static __device__ __forceinline__ PfHalo pf_halo(const TapPfArgs &p, int m0, int m_hi)
{
    const int OHW = p.d_OHW.d;
    const int n_first = fdiv(m0, p.d_OHW);
    const int oh_first = fdiv(m0 - n_first * OHW, p.d_OW);
    const int m_last = m_hi - 1;
    const int n_last = fdiv(m_last, p.d_OHW);
    const int oh_last = fdiv(m_last - n_last * OHW, p.d_OW);
    PfHalo h;
    h.pgr0 = n_first * p.PHt + oh_first;
    h.rows = n_last * p.PHt + oh_last + p.TH - 1 - h.pgr0 + 1;
    return h;
}

// TILES: tiles of a whole unit; CG: column groups of 32 padded pixels per row (1 or 2); EPT: halo elements a thread
// requests per tap; BK: the filter is contiguous along the input channel (W[OC,FH,FW,IC] as it is) instead of along the
// output channel; RP2: rows of at most 16 padded pixels, a halo element is this thread's share of TWO rows (CG = 1).
template <int TILES, int CG, int EPT, bool BK, bool RP2, bool EPI>
__global__ __launch_bounds__(256, 2) void tap_conv_prefetch_kernel(const TapPfArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *Hs = smem;   // through a pointer variable: a vector access to smem[...] itself is given the alignment of a float
    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int oc0 = blockIdx.y * 64;
    const int PHt = p.PHt, PWt = p.PWt, OHW = p.d_OHW.d, OW = p.d_OW.d;
    const int row_floats = PWt * PF_PS;
    const int spare = 2 * p.buf_floats;   // write-only slot behind the buffers
    const int npass = p.AC / PF_ICC;

    // ---- this workgroup's items: whole units first, then its pieces --------------------------------------------
    const int G = gridDim.x;
    const int xcd = blockIdx.x & 7, xi = blockIdx.x >> 3;
    const int wgs = (G >> 3) + (xcd < (G & 7) ? 1 : 0);   // workgroups on this XCD
    const int u_lo = xcd * (p.full_units >> 3) + min(xcd, p.full_units & 7);
    const int u_n = (p.full_units >> 3) + (xcd < (p.full_units & 7) ? 1 : 0);
    const int c_lo = xcd * (p.pieces >> 3) + min(xcd, p.pieces & 7);
    const int c_n = (p.pieces >> 3) + (xcd < (p.pieces & 7) ? 1 : 0);
    const int n_whole = xi < u_n ? (u_n - xi + wgs - 1) / wgs : 0;
    const int n_piece = xi < c_n ? (c_n - xi + wgs - 1) / wgs : 0;
    const int n_items = n_whole + n_piece;
    // item idx -> pixels [m0, m_hi) and the body that handles them (0: TILES tiles, 1: four, 2: two); false for an
    // empty piece (the last unit may be partial) and past the end
    auto item = [&](int idx, int &m0, int &m_hi, int &body) {
        if (idx >= n_items) return false;
        if (idx < n_whole) {
            m0 = (u_lo + xi + idx * wgs) * 16 * TILES;
            m_hi = min(m0 + 16 * TILES, p.M);
            body = 0;
            return true;
        }
        const int piece = c_lo + xi + (idx - n_whole) * wgs;
        const int u = piece / p.piece_split, k = piece - u * p.piece_split;
        const int unit = p.full_units + u;
        m0 = unit * 16 * TILES + k * 16 * p.piece_tiles;
        m_hi = min(min(m0 + 16 * p.piece_tiles, (unit + 1) * 16 * TILES), p.M);
        body = p.piece_tiles > 2 ? 1 : 2;
        return m0 < m_hi;
    };
    auto next_item = [&](int idx, int &m0, int &m_hi, int &body) {   // first non-empty item at or after idx, or n_items
        while (idx < n_items && !item(idx, m0, m_hi, body)) idx++;
        return idx;
    };

    // ---- halo mover ------------------------------------------------------------------------------------------------
    // Thread t moves channels [4*(t&7), +4) of padded column 32*cg + (t>>3) of a row; element e of a pass is (row
    // e / CG, column group e % CG). Rows of at most 16 pixels (RP2): column (t>>3)&15 of row 2e + (t>>7). Columns past
    // the end of the row repeat the last column (the same bytes to the same place), rows past the halo's last row
    // repeat the last row. What depends on the row - where it starts in A, whether it lies inside the image, where it
    // goes in LDS - is the same for every pass of a unit: lane i of a wavefront computes it for row i once per unit
    // (two registers), and a tap fetches the rows it requests with v_readlane into scalar registers. The load takes
    // (descriptor, per-thread offset, scalar offset); padding columns and rows make the per-thread offset out of range
    // and zeros arrive without a select.
    constexpr unsigned NEVER = 0x40000000u;   // RP2 adds a column and a row offset: two of these still do not wrap (A < 1 GB, host-checked)
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.A), 0, p.a_bytes, 0x00020000);
    unsigned voff[CG];
    int loff[CG];
#pragma unroll
    for (int cg = 0; cg < CG; cg++) {
        const int cp = min(RP2 ? (t >> 3) & 15 : 32 * cg + (t >> 3), PWt - 1), iw = cp - p.pw;
        voff[cg] = (unsigned)iw < (unsigned)p.AW ? (unsigned)((iw * p.AC + (t & 7) * 4) * 4) : (RP2 ? NEVER : PF_OUT_OF_RANGE);
        loff[cg] = (cp * PF_PS + (t & 7) * 4) * 4;   // bytes
    }
    const bool second_row = RP2 && t >= 128;
    // per-lane table of a halo's rows: byte offset of the row in A (-1: padding row) and byte offset of the row in a buffer
    struct RowTable {
        int g, l;
    };
    auto row_table = [&](const PfHalo &h, bool on) {
        const int r = min(lane, h.rows - 1);
        const int pgr = h.pgr0 + r;
        const int n = fdiv(pgr, p.d_PHt), ih = pgr - n * PHt - p.ph;
        RowTable tb_;
        tb_.g = ((unsigned)ih < (unsigned)p.AH && on) ? (n * p.AH + ih) * p.AW * p.AC * 4 : -1;
        tb_.l = r * row_floats * 4;
        return tb_;
    };
    // The row(s) being requested: scalar offset in A (channels of the pass included), padding or not, place in LDS.
    struct RowState {
        int soff, rowoff;     // first (or only) row
        unsigned kill;
        int soff2, rowoff2;   // RP2: second row; soff/soff2 are then NEVER for a padding row
    };
    // row index (RP2: rows 2*index, 2*index+1) of the table, channels [ic0, ic0 + 32), for the buffer at byte offset tb
    auto next_row = [&](RowState &row, int index, const RowTable &tab, int ic0, int tb) {
        if (!RP2) {
            const int g = __builtin_amdgcn_readlane(tab.g, index);
            row.soff = g >= 0 ? g + ic0 * 4 : 0;
            row.kill = g >= 0 ? 0u : PF_OUT_OF_RANGE;
            row.rowoff = tb + __builtin_amdgcn_readlane(tab.l, index);
        } else {
            const int g = __builtin_amdgcn_readlane(tab.g, 2 * index), g2 = __builtin_amdgcn_readlane(tab.g, 2 * index + 1);
            row.soff = g >= 0 ? g + ic0 * 4 : (int)NEVER;
            row.soff2 = g2 >= 0 ? g2 + ic0 * 4 : (int)NEVER;
            row.rowoff = tb + __builtin_amdgcn_readlane(tab.l, 2 * index);
            row.rowoff2 = tb + __builtin_amdgcn_readlane(tab.l, 2 * index + 1);
        }
    };
    // request this thread's element of column group cg of that row; dst: its place in LDS (bytes). With nothing to
    // prefetch (the table says padding everywhere) zeros go to the buffer nobody will read.
    auto request = [&](auto cg_c, const RowState &row, float4 &v, int &dst) {
        constexpr int cg = decltype(cg_c)::value;
        if (!RP2) {
            v = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)(voff[cg] | row.kill), row.soff, 0));
            dst = row.rowoff + loff[cg];
        } else {
            const int so = second_row ? row.soff2 : row.soff;
            v = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)(voff[0] + (unsigned)so), 0, 0));
            dst = (second_row ? row.rowoff2 : row.rowoff) + loff[0];
        }
    };

    // ---- filter fragments straight from global memory (see tap_conv.hip) ----------------------------------------
    // lane (l16, q) of wavefront w needs, for channel group g of a tap, B[c = 16g + 4q + s][oc0 + 16w + l16], s = 0..3.
    // Output channel contiguous: eight 32-bit loads at (scalar base of the tap) + (fixed per-lane offset). Input
    // channel contiguous: the four s of a group are neighbours, two 128-bit loads.
    const int b_co = oc0 + 16 * w + l16;
    const bool b_cov = b_co < p.CO;   // columns beyond CO are never stored; clamp their loads to a valid address
    unsigned b_lane[2][4];
#pragma unroll
    for (int g = 0; g < 2; g++)
#pragma unroll
        for (int s = 0; s < 4; s++)
            b_lane[g][s] = BK ? (unsigned)(((b_cov ? b_co : 0) * p.b_sn + 16 * g + 4 * q) * 4)
                              : (unsigned)(((16 * g + 4 * q + s) * p.b_sc + (b_cov ? b_co : 0)) * 4);
    auto load_b = [&](float (&b)[2][4], int icbase, int th, int tw) {
        const int sbase = __builtin_amdgcn_readfirstlane(p.b_off + th * p.b_sth + tw * p.b_stw + icbase * p.b_sc);
        const char *sb = reinterpret_cast<const char *>(p.B + sbase);
#pragma unroll
        for (int g = 0; g < 2; g++) {
            if (BK) {
                asm volatile("" : "+v"(b_lane[g][0]));   // value unchanged; keeps the zero-extension next to the load
                const float4 v = *reinterpret_cast<const float4 *>(sb + b_lane[g][0]);
                b[g][0] = v.x; b[g][1] = v.y; b[g][2] = v.z; b[g][3] = v.w;
            } else {
#pragma unroll
                for (int s = 0; s < 4; s++) {
                    asm volatile("" : "+v"(b_lane[g][s]));
                    b[g][s] = *reinterpret_cast<const float *>(sb + b_lane[g][s]);
                }
            }
        }
    };

    // Everything outside the MFMA loops runs at a raised priority: a wavefront that issues MFMAs back to back keeps the
    // SIMD's vector issue port, and the other workgroup's address arithmetic and stores at the same priority wait for
    // thousands of cycles (unit set-up 15000 cycles instead of 1000, measured).
    __builtin_amdgcn_s_setprio(3);
    const float bias_v = (p.ep.bias != nullptr && b_cov) ? p.ep.bias[b_co] : 0.f;
    // EPI: this lane's channel constants of the fused epilogue (the channel is the same for every unit of the workgroup)
    float e_sub = 0.f, e_mul = 1.f, e_add = 0.f;
    if (EPI && b_cov) ep_channel(p.ep, b_co, e_sub, e_mul, e_add);
    const int o_lane = b_cov ? (4 * q * p.CO + b_co) * 4 : (int)PF_OUT_OF_RANGE;   // output byte offset of this lane within a tile
    int buf = 0;          // buffer that holds the halo of the pass about to run
    float bA[2][4];       // filter fragment of that pass's first tap
    load_b(bA, 0, 0, 0);

    // ---- first item: its first pass is staged with nothing to overlap ------------------------------------------
    int m0 = 0, m_hi = 0, body = 0;
    int idx = next_item(0, m0, m_hi, body);
    if (idx >= n_items) return;
    RowTable tab_cur = row_table(pf_halo(p, m0, m_hi), true);
    {
        const PfHalo h = pf_halo(p, m0, m_hi);
        constexpr int ROWS8 = RP2 ? 16 : 8 / CG;   // rows that eight elements cover
        for (int r0 = 0; r0 < h.rows; r0 += ROWS8) {
            float4 v[8];
            int dst[8];
            pf_static_for<0, 8>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                RowState row;
                next_row(row, min((RP2 ? r0 / 2 : r0) + i / CG, 31), tab_cur, 0, 0);
                request(PfInt<i % CG>{}, row, v[i], dst[i]);
            });
#pragma unroll
            for (int i = 0; i < 8; i++) *reinterpret_cast<float4 *>(reinterpret_cast<char *>(Hs) + dst[i]) = v[i];
        }
        __syncthreads();
    }

    // ---- one unit ------------------------------------------------------------------------------------------------------
    auto run_unit = [&](auto tiles_c, const int m0, const int m_hi, const bool has_next, const RowTable &tab_next) {
        constexpr int T = decltype(tiles_c)::value;
        const PfHalo h = pf_halo(p, m0, m_hi);

        // per-lane LDS byte offset of each tile's pixel at tap (0,0), plus this lane group's channels
        int cur[T];
#pragma unroll
        for (int i = 0; i < T; i++) {
            const int m = min(m0 + 16 * i + l16, m_hi - 1);
            const int n = fdiv(m, p.d_OHW), rem = m - n * OHW;
            const int oh = fdiv(rem, p.d_OW), ow = rem - oh * OW;
            cur[i] = (buf * p.buf_floats + ((n * PHt + oh - h.pgr0) * PWt + ow) * PF_PS + 4 * q) * 4;
        }
        floatx4 acc[T];
#pragma unroll
        for (int i = 0; i < T; i++) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};

        auto read_a = [&](floatx4 (&a)[T], auto tw_c, int ck) {   // tap column tw and chunk ck: a constant offset
            constexpr int tw = decltype(tw_c)::value;
#pragma unroll
            for (int i = 0; i < T; i++)
                a[i] = *reinterpret_cast<const floatx4 *>(reinterpret_cast<const char *>(Hs) + cur[i] + (tw * PF_PS + 16 * ck) * 4);
        };
        auto mfma_chunk = [&](const floatx4 (&a)[T], const float (&b)[4]) {
#pragma unroll
            for (int s = 0; s < 4; s++)
#pragma unroll
                for (int i = 0; i < T; i++)
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i][s], b[s], acc[i], 0, 0, 0);
        };
        auto spread_reads = [&]() {   // LDS reads of the next chunk issue in the shadow of this chunk's first MFMAs
#pragma unroll
            for (int i = 0; i < T; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // 1 MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // 1 LDS read
            }
        };

        floatx4 aP[T], aQ[T];   // A fragments ping-pong: the next chunk is read while the current one is multiplied
        float bB[2][4];
        float4 pv[2][EPT];      // requested halo elements, two taps' worth in flight
        int pd[2][EPT];
#pragma unroll
        for (int i = 0; i < EPT; i++) pv[0][i] = pv[1][i] = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int pass = 0; pass < npass; pass++) {
            const int ic0 = pass * PF_ICC;
            const bool last_pass = pass + 1 == npass;
            // what to prefetch: the next 32 channels of this halo, or the first 32 of the next unit's
            const RowTable &tab = last_pass ? tab_next : tab_cur;
            const int t_ic0 = last_pass ? 0 : ic0 + PF_ICC;
            const int tb = (buf ^ 1) * p.buf_floats * 4;   // bytes
            const int n_ic = last_pass ? 0 : ic0 + PF_ICC;   // filter fragment after this pass's last tap
#pragma unroll
            for (int i = 0; i < EPT; i++) pd[1][i] = spare * 4;   // tap 0 commits "the tap before": nothing
            RowState row;

            __builtin_amdgcn_s_setprio(0);
            read_a(aP, PfInt<0>{}, 0);   // cur[] is at filter row 0 of buffer buf here
            // The nine taps, unrolled: which filter fragment and element registers a tap uses, its offset within the
            // filter row and the halo row it requests are all known at compile time; what is left per tap is one
            // scalar base for the filter fragment, and per filter row one add per tile.
            pf_static_for<0, 9>([&](auto kc) {
                constexpr int K = decltype(kc)::value;
                constexpr int PAR = K & 1, TW_ = K % 3;
                constexpr bool TAIL = K == 8;
                constexpr int NK = TAIL ? 0 : K + 1;   // the tap after this one
                float (&bU)[2][4] = PAR ? bB : bA;
                float (&bL)[2][4] = PAR ? bA : bB;
                __builtin_amdgcn_sched_barrier(0);
                if (!TAIL) {
                    pf_static_for<0, EPT>([&](auto ic) {
                        constexpr int i = decltype(ic)::value, e = K * EPT + i;
                        if (e % CG == 0) next_row(row, e / CG, tab, t_ic0, tb);
                        request(PfInt<e % CG>{}, row, pv[PAR][i], pd[PAR][i]);
                    });
                }
                load_b(bL, TAIL ? n_ic : ic0, NK / 3, NK % 3);
                __builtin_amdgcn_sched_barrier(0);
                read_a(aQ, PfInt<TW_>{}, 1);
                mfma_chunk(aP, bU[0]);
                spread_reads();
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < EPT; i++)   // the elements requested one tap ago
                    *reinterpret_cast<float4 *>(reinterpret_cast<char *>(Hs) + pd[PAR ^ 1][i]) = pv[PAR ^ 1][i];
                if (!TAIL) {
                    if (TW_ == 2) {   // on to the next filter row
#pragma unroll
                        for (int i = 0; i < T; i++) cur[i] += 4 * row_floats;
                    }
                    read_a(aP, PfInt<NK % 3>{}, 0);
                    mfma_chunk(aQ, bU[1]);
                    spread_reads();
                } else {
                    mfma_chunk(aQ, bU[1]);
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            __builtin_amdgcn_s_setprio(3);
#pragma unroll
            for (int g = 0; g < 2; g++)
#pragma unroll
                for (int s = 0; s < 4; s++) bA[g][s] = bB[g][s];
            __syncthreads();   // buffer buf has been read by everyone, the other one is complete
            buf ^= 1;
            {
                const int d = 4 * ((buf ? p.buf_floats : -p.buf_floats) - 2 * row_floats);   // filter row 0 of the other buffer
#pragma unroll
                for (int i = 0; i < T; i++) cur[i] += d;
            }
        }

        // ---- epilogue: accumulators straight to memory ----------------------------------------------------------------
        // Lane (l16, q) holds pixels 16i + 4q + r, channel 16w + l16: one store instruction writes 64 contiguous bytes
        // of four pixel rows; the other three quarters of those rows come from the other wavefronts and meet in L2.
        // (A transpose through LDS gives whole 256-byte rows per instruction but needs two barriers, and its LDS traffic
        // queues behind the reads of the other workgroup's MFMA loop: 12000 cycles per unit, measured.)
        // The descriptor ends at the unit's last pixel, so rows past it are dropped by the range check.
        const __amdgpu_buffer_rsrc_t o_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.O, 0, m_hi * p.CO * 4, 0x00020000);
        if constexpr (!EPI) {
#pragma unroll
            for (int i = 0; i < T; i++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int soff = __builtin_amdgcn_readfirstlane((m0 + 16 * i + r) * p.CO * 4);
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, acc[i][r] + bias_v), o_rsrc, o_lane, soff, 0);
                }
        } else if (p.ep.gate != nullptr) {   // uniform: backward of the leaky ReLU that produced this tensor's twin `gate`
            const __amdgpu_buffer_rsrc_t g_rsrc =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.ep.gate), 0, m_hi * p.CO * 4, 0x00020000);
#pragma unroll
            for (int i = 0; i < T; i++) {
                float g[4];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int soff = __builtin_amdgcn_readfirstlane((m0 + 16 * i + r) * p.CO * 4);
                    g[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(g_rsrc, o_lane, soff, 0));
                }
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int soff = __builtin_amdgcn_readfirstlane((m0 + 16 * i + r) * p.CO * 4);
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, ep_gate(acc[i][r], g[r], p.ep.slope)), o_rsrc, o_lane, soff, 0);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < T; i++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int soff = __builtin_amdgcn_readfirstlane((m0 + 16 * i + r) * p.CO * 4);
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, ep_finish(acc[i][r], e_sub, e_mul, e_add, p.ep.slope)),
                                                          o_rsrc, o_lane, soff, 0);
                }
        }
    };

    while (idx < n_items) {
        int n_m0 = 0, n_hi = 0, n_body = 0;
        const int nidx = next_item(idx + 1, n_m0, n_hi, n_body);
        const bool has_next = nidx < n_items;
        PfHalo nh{0, 1};
        if (has_next) nh = pf_halo(p, n_m0, n_hi);
        const RowTable tab_next = row_table(nh, has_next);
        if (body == 0) run_unit(PfInt<TILES>{}, m0, m_hi, has_next, tab_next);
        else if (body == 1) run_unit(PfInt<4>{}, m0, m_hi, has_next, tab_next);
        else run_unit(PfInt<2>{}, m0, m_hi, has_next, tab_next);
        idx = nidx; m0 = n_m0; m_hi = n_hi; body = n_body;
        tab_cur = tab_next;
    }
}

// Rows of LDS halo the worst unit needs: output rows spanned by P consecutive pixels, TH-1 extra rows, and TH-1 more
// for every image border crossed.
static int tap_pf_lds_rows(int M, int P, int OH, int OW, int TH, int PHt)
{
    const int OHW = OH * OW;
    int worst = 0;
    const int units = (M + P - 1) / P;
    const int scan = units < 4096 ? units : 4096;
    for (int u = 0; u < scan; u++) {
        const long m0 = (long)u * P, m1 = (m0 + P < M ? m0 + P : M) - 1;
        const int n0 = (int)(m0 / OHW), oh0 = (int)(m0 % OHW) / OW;
        const int n1 = (int)(m1 / OHW), oh1 = (int)(m1 % OHW) / OW;
        const int rows = (n1 * PHt + oh1 + TH - 1) - (n0 * PHt + oh0) + 1;
        if (rows > worst) worst = rows;
    }
    if (units > scan) {   // analytic bound for what was not scanned
        const int span = (P + OW - 2) / OW + 1;
        const int cross = (P + OHW - 2) / OHW + 1;
        const int bound = (span - 1) + TH + cross * (PHt - OH > 0 ? PHt - OH : 0);
        if (bound > worst) worst = bound;
    }
    return worst;
}

template <int TILES, int CG, int EPT, bool BK, bool RP2, bool EPI>
static hipError_t launch_pf3(hipStream_t stream, TapPfArgs a, size_t lds, int cus)
{
    constexpr auto kern = tap_conv_prefetch_kernel<TILES, CG, EPT, BK, RP2, EPI>;
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    const int units = (a.M + TILES * 16 - 1) / (TILES * 16), ocb = (a.CO + 63) / 64;
    int G = 2 * cus / ocb;   // two workgroups per compute unit
    if (G < 1) G = 1;
    if (G > units) G = units;
    a.full_units = (units / G) * G;
    a.pieces = 0; a.piece_split = 1; a.piece_tiles = TILES;
    const int left = units - a.full_units;
    if (left > 0) {
        int split = G / left;                  // pieces per left-over unit that still give every workgroup at most one
        if (split > TILES / 2) split = TILES / 2;
        if (split >= 2) {
            a.piece_split = split;
            a.piece_tiles = (TILES + split - 1) / split;   // <= 4 for TILES <= 8
            a.pieces = left * split;
        } else {
            a.full_units = units;              // more than half a round is left: whole units for the first workgroups
        }
    }
    hipLaunchKernelGGL(kern, dim3(G, ocb, 1), dim3(256), lds, stream, a);
    return hipGetLastError();
}

template <int TILES, int CG, int EPT, bool BK, bool RP2>
static hipError_t launch_pf2(hipStream_t stream, const TapPfArgs &a, size_t lds, int cus)
{
    return a.ep.fused ? launch_pf3<TILES, CG, EPT, BK, RP2, true>(stream, a, lds, cus) : launch_pf3<TILES, CG, EPT, BK, RP2, false>(stream, a, lds, cus);
}

template <int TILES, int CG, int EPT, bool RP2 = false>
static hipError_t launch_pf(hipStream_t stream, const TapPfArgs &a, size_t lds, int cus)
{
    return a.b_sn != 1 ? launch_pf2<TILES, CG, EPT, true, RP2>(stream, a, lds, cus) : launch_pf2<TILES, CG, EPT, false, RP2>(stream, a, lds, cus);
}

// Returns hipErrorNotSupported when the shape does not fit this kernel; otherwise launches.
hipError_t launch_tap_conv_prefetch(hipStream_t stream, const float *A, const float *B, float *O,
                                    int N, int AH, int AW, int AC, int OH, int OW, int CO,
                                    int TH, int TW, int ph, int pw,
                                    int b_off, int b_sth, int b_stw, int b_sc, int b_sn, const Epilogue &ep, int cus)
{
    if (b_sn != 1 && (b_sc != 1 || (b_sn | b_sth | b_stw | b_off) % 4 != 0)) return hipErrorNotSupported;   // 128-bit fragment loads
    if (OH != AH + 2 * ph - TH + 1 || OW != AW + 2 * pw - TW + 1) return hipErrorNotSupported;
    if (AC % PF_ICC != 0 || TH != 3 || TW != 3) return hipErrorNotSupported;
    const int PHt = AH + 2 * ph, PWt = AW + 2 * pw;
    if (PWt < 3 || PWt > 64) return hipErrorNotSupported;
    const bool rp2 = PWt <= 16;
    const long M = (long)N * OH * OW;
    if ((long)N * PHt >= (1L << 24) || M >= (1L << 30)) return hipErrorNotSupported;
    const long a_bytes = (long)N * AH * AW * AC * 4;
    if (a_bytes >= (1L << 31) || M * CO * 4 >= (1L << 31)) return hipErrorNotSupported;
    if (PWt <= 16 && a_bytes >= (1L << 30)) return hipErrorNotSupported;

    TapPfArgs a{};
    a.A = A; a.B = B; a.O = O; a.ep = ep;
    a.M = (int)M; a.CO = CO;
    a.AH = AH; a.AW = AW; a.AC = AC;
    a.TH = TH; a.TW = TW; a.ph = ph; a.pw = pw;
    a.PHt = PHt; a.PWt = PWt;
    a.a_bytes = (int)a_bytes;
    a.b_off = b_off; a.b_sth = b_sth; a.b_stw = b_stw; a.b_sc = b_sc; a.b_sn = b_sn;
    a.d_OW = make_fastdiv(OW);
    a.d_OHW = make_fastdiv(OH * OW);
    a.d_PHt = make_fastdiv(PHt);

    // pixels per workgroup: 7 tiles (112) when that divides the row/image structure better, else 8 (128)
    const int OHW = OH * OW;
    int tiles = 8;
    if ((OHW % 112 == 0 || (2 * OW) % 112 == 0 || 112 % OW == 0) && !(OHW % 128 == 0 || 128 % OW == 0)) tiles = 7;
    const int cg = PWt <= 32 ? 1 : 2;
    for (int attempt = 0; attempt < 2; attempt++) {
        const int P = tiles * 16;
        a.lds_rows = tap_pf_lds_rows(a.M, P, OH, OW, TH, PHt);
        const size_t bufsz = (size_t)a.lds_rows * PWt * PF_PS;
        a.buf_floats = (int)bufsz;
        const size_t lds = (2 * bufsz + 4) * sizeof(float);
        const int elems = rp2 ? (a.lds_rows + 1) / 2 : a.lds_rows * cg, ept = (elems + TH * TW - 2) / (TH * TW - 1);
        if (lds <= 80 * 1024 && ept <= 2 && rp2) {
            if (tiles == 7) return ept == 1 ? launch_pf<7, 1, 1, true>(stream, a, lds, cus) : launch_pf<7, 1, 2, true>(stream, a, lds, cus);
            return ept == 1 ? launch_pf<8, 1, 1, true>(stream, a, lds, cus) : launch_pf<8, 1, 2, true>(stream, a, lds, cus);
        }
        if (lds <= 80 * 1024 && ept <= 2) {
            if (tiles == 7) {
                if (cg == 1) return ept == 1 ? launch_pf<7, 1, 1>(stream, a, lds, cus) : launch_pf<7, 1, 2>(stream, a, lds, cus);
                return ept == 1 ? launch_pf<7, 2, 1>(stream, a, lds, cus) : launch_pf<7, 2, 2>(stream, a, lds, cus);
            }
            if (cg == 1) return ept == 1 ? launch_pf<8, 1, 1>(stream, a, lds, cus) : launch_pf<8, 1, 2>(stream, a, lds, cus);
            return ept == 1 ? launch_pf<8, 2, 1>(stream, a, lds, cus) : launch_pf<8, 2, 2>(stream, a, lds, cus);
        }
        tiles = (tiles == 8) ? 7 : 8;
    }
    return hipErrorNotSupported;
}

}  // namespace alpha
