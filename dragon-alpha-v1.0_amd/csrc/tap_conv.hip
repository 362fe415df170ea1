// Stride-1 convolution with the input window staged ONCE in LDS ("tap convolution"), fp32 MFMA
// v_mfma_f32_16x16x4_f32, gfx950. Serves forward 3x3/5x5... stride 1 and stride-1 backward-data.
//
// A workgroup (4 wavefronts) owns P = 16*TILES consecutive output pixels of the flattened
// (n, oh, ow) index and a slice of 64 output channels. For each chunk of 64 input channels it
//   1. copies the zero-padded input rows those pixels touch into LDS once
//      (rows are "padded global rows" n*(AH+2ph) + ih + ph, so a pixel range may cross image borders);
//   2. walks the filter in "half taps" (one tap, 32 input channels). Every lane reads its pixel's 4
//      consecutive channels with one 128-bit LDS read at base(pixel) + tap offset — no address
//      arithmetic or bounds tests in the inner loop. The filter fragment of a half tap (8 floats per
//      lane) comes straight from global memory (it is L2/L1 resident: every workgroup reads the same
//      few hundred KB) and is prefetched one half tap ahead, so the main loop has no barrier at all.
// Each input element is read from memory once per workgroup instead of once per tap.
//
// Wavefront w computes output channels [16w, 16w+16) for all TILES pixel tiles (TILES*4 accumulator
// registers).
//
// LDS layout (floats): halo[row][col][64+8]. Pixel stride 72 floats = 288 bytes: measured on gfx950,
// a 128-bit LDS read is conflict-free when the 32 lanes of each half wavefront touch 32 distinct
// 16-byte slots modulo 512 bytes; with 16 consecutive pixels x 2 channel quads per half wavefront
// that needs a pixel stride of 16*(4k+2) bytes (272 gives a 2-way conflict, 288 none).
// K permutation inside a group of 16 channels: lane group q = lane/16 supplies channel 16g + 4q + s
// at MFMA step s, for both operands.
#include "common.hpp"

namespace alpha {

struct TapConvArgs {
    const float *A;   // input activations [N, AH, AW, AC]
    const float *B;   // filter; element (th, tw, c, co) at b_off + th*b_sth + tw*b_stw + c*b_sc + co
    float *O;         // output [N, OH, OW, CO] dense
    int M, CO;        // N*OH*OW pixels, output channels
    int AH, AW, AC;
    int TH, TW, ph, pw;
    int PHt, PWt;     // AH + 2ph, AW + 2pw
    int sh, sw;       // output pixel (oh, ow) reads the padded input window at (oh*sh, ow*sw)
    int PWp, RP;      // LDS row: sw planes of PWp = ceil(PWt/sw) pixels (padded column cp in plane cp % sw at cp / sw); RP = sw*PWp
    int lds_rows;     // halo rows reserved in LDS
    int b_off, b_sth, b_stw, b_sc;
    Epilogue ep;         // applied as the rows leave for memory
    int full_units;   // units of 16*TILES pixels that are processed whole, dealt round-robin to the persistent workgroups
    int pieces;       // the remaining units cut into piece_split pieces of piece_tiles tiles each, one piece per workgroup
    int piece_split, piece_tiles;
    FastDiv d_OW, d_OHW, d_PHt, d_PWt, d_sw;
    // merged kernel-split backward-data only (tap_conv_merged_kernel): output pixel (n, i, j) of phase f goes to
    // O + f_o_off[f] + n*o_sn + i*o_sh + j*o_sw; tap (th, tw) of phase f reads the halo at (row + th + f_row[f],
    // column + tw + f_col[f]) and the filter at f_b_off[f] + th*f_b_sth[f] + tw*b_stw + c*b_sc + co
    int o_sn, o_sh, o_sw;
    int f_TH[4], f_TW[4], f_row[4], f_col[4], f_b_off[4], f_b_sth[4], f_o_off[4];
};

template <int V> struct TapInt { static constexpr int value = V; };
template <int I, int N, class F>
static __device__ __forceinline__ void pf_phase_loop(F &&f)
{
    if constexpr (I < N) {
        f(TapInt<I>{});
        pf_phase_loop<I + 1, N>(f);
    }
}
constexpr int TC_ICC = 64;            // input channels per halo pass
constexpr int TC_PS = TC_ICC + 8;     // LDS pixel stride (floats)
constexpr int TC_OS = 64 + 4;         // output staging row stride (floats)

// Where a lane reads its filter fragment: element index = half-tap base (uniform) + lane offset. The three functions
// below are the whole address computation of the filter loads, shared by the kernel and by the host-side walk
// alpha_selfcheck_tap_filter_extent, which the CPU tests use to prove that no load leaves the filter.
// RAGGED: the second half tap of the last pass may start at or beyond AC (AC % 64 in [4, 32]); every lane of such a
// half tap is masked, and its base is pulled back to the last channel quad so that the masked lanes' address
// (base + 0) stays inside the filter.
template <bool RAGGED>
__host__ __device__ __forceinline__ int tap_filter_half_tap_base(int b_off, int b_sth, int b_stw, int b_sc, int AC, int icbase, int th, int tw)
{
    const int icb = RAGGED ? (icbase < AC - 4 ? icbase : AC - 4) : icbase;
    return b_off + th * b_sth + tw * b_stw + icb * b_sc;
}
template <bool RAGGED>
__host__ __device__ __forceinline__ unsigned tap_filter_lane_mask(int AC, int icbase, int g, int q)
{
    return RAGGED ? (unsigned)-(int)(icbase + 16 * g + 4 * q < AC) : ~0u;
}
__host__ __device__ __forceinline__ unsigned tap_filter_lane_bytes(int b_sc, int g, int q, int s, int co)
{
    return (unsigned)(((16 * g + 4 * q + s) * b_sc + co) * 4);
}

// Stages the zero-padded input rows pgr0 .. pgr0 + rows - 1 ("padded global rows" n*PHt + ih + ph), channels
// ic0 .. ic0 + 63, into Hs[row][sw planes][PWp][TC_PS]: zero outside the image and beyond AC. A thread keeps its place in
// the row: 16 lanes per pixel (64 channels), padded column 16*cg + t/16 of column group cg. What depends on the column is
// computed once per 64 columns, what depends on the row is uniform (scalar registers); per element the vector unit is
// left with two address operations and the zero-fill selects. (Computing pixel, row and column of every element from a
// flat index cost ~60 vector instructions per element, and those take issue slots from the MFMAs of the workgroup that
// shares the compute unit.) A step stages RS rows of CGS column groups (16 columns each), at most eight loads in flight
// per thread; narrow images take more rows per step, wide ones more column groups (and several trips along the row).
static __device__ __forceinline__ void tap_stage_halo(const TapConvArgs &p, float *Hs, const int ic0, const int pgr0, const int rows, const int t)
{
    const int PHt = p.PHt, PWt = p.PWt, RP = p.RP;
    auto stage = [&](auto cgs_c, auto rs_c) {
        constexpr int CGS = decltype(cgs_c)::value, RS = decltype(rs_c)::value;
        const int cq4 = (t & 15) * 4;
        const bool ch_ok = ic0 + cq4 < p.AC;
        const int row_floats = RP * TC_PS, spare = p.lds_rows * row_floats;
        for (int c0 = 0; c0 < PWt; c0 += 16 * CGS) {
            int goff[CGS], loff[CGS];
            bool cok[CGS];
#pragma unroll
            for (int cg = 0; cg < CGS; cg++) {
                const int cp = c0 + 16 * cg + (t >> 4), iw = cp - p.pw;
                cok[cg] = cp < PWt && (unsigned)iw < (unsigned)p.AW && ch_ok;
                goff[cg] = cok[cg] ? iw * p.AC + ic0 + cq4 : 0;
                const int cq = fdiv(cp, p.d_sw), cr = cp - cq * p.sw;
                // threads past the end of the row write their zeros to a spare slot behind the halo
                loff[cg] = cp < PWt ? (cr * p.PWp + cq) * TC_PS + cq4 : spare;
            }
            for (int r = 0; r < rows; r += RS) {
                float4 v[RS][CGS];
                bool rok[RS];
#pragma unroll
                for (int rr = 0; rr < RS; rr++) {
                    const int pgr = pgr0 + min(r + rr, rows - 1);   // past the last row: the last row again
                    const int n = fdiv(pgr, p.d_PHt), ih = pgr - n * PHt - p.ph;
                    rok[rr] = (unsigned)ih < (unsigned)p.AH;
                    const int rowbase = rok[rr] ? (n * p.AH + ih) * p.AW * p.AC : 0;
                    const int rowmask = rok[rr] ? -1 : 0;
#pragma unroll
                    for (int cg = 0; cg < CGS; cg++)   // outside the image: element 0, zeroed below
                        v[rr][cg] = *reinterpret_cast<const float4 *>(p.A + rowbase + (goff[cg] & rowmask));
                }
#pragma unroll
                for (int rr = 0; rr < RS; rr++) {
                    const int rowoff = min(r + rr, rows - 1) * row_floats;
#pragma unroll
                    for (int cg = 0; cg < CGS; cg++) {
                        const bool ok = rok[rr] && cok[cg];   // per-component selects keep v[] in registers
                        const int dst = loff[cg] == spare ? spare : rowoff + loff[cg];
                        *reinterpret_cast<float4 *>(Hs + dst) = make_float4(ok ? v[rr][cg].x : 0.f, ok ? v[rr][cg].y : 0.f,
                                                                            ok ? v[rr][cg].z : 0.f, ok ? v[rr][cg].w : 0.f);
                    }
                }
            }
        }
    };
    if (PWt <= 16) stage(TapInt<1>{}, TapInt<8>{});
    else if (PWt <= 32) stage(TapInt<2>{}, TapInt<4>{});
    else if (PWt <= 48) stage(TapInt<3>{}, TapInt<2>{});
    else stage(TapInt<4>{}, TapInt<2>{});
}

// RAGGED: AC is not a multiple of 64, so the last pass has channels beyond AC whose filter fragments
// must be zeroed (kept out of the common case: the extra selects would pull the wait for the
// prefetched fragment in front of the MFMAs).
// One unit: output pixels [m0, min(m0 + 16*TILES, m_lim)) x output channels [oc0, oc0 + 64).
template <int TILES, bool RAGGED>
__device__ __forceinline__ void tap_conv_unit(const TapConvArgs &p, float *smem, const int m0, const int m_lim, const int oc0)
{
    constexpr int P = TILES * 16;
    float *Hs = smem;   // [lds_rows][sw planes][PWp][TC_PS] (+ one spare slot); reused as output staging [P][TC_OS]

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int OW = p.d_OW.d, OHW = p.d_OHW.d, PHt = p.PHt, RP = p.RP;

    // first padded global row held in LDS, and how many rows this unit needs (<= p.lds_rows, host-checked)
    const int n_first = fdiv(m0, p.d_OHW);
    const int oh_first = fdiv(m0 - n_first * OHW, p.d_OW);
    const int pgr0 = n_first * PHt + oh_first * p.sh;
    const int m_last = min(m0 + P, m_lim) - 1;
    const int n_last = fdiv(m_last, p.d_OHW);
    const int oh_last = fdiv(m_last - n_last * OHW, p.d_OW);
    const int rows = n_last * PHt + oh_last * p.sh + p.TH - 1 - pgr0 + 1;

    // per-lane LDS offset (floats) of each tile's pixel at tap (0,0), plus this lane group's channel offset
    int abase[TILES];
#pragma unroll
    for (int i = 0; i < TILES; i++) {
        const int m = min(m0 + 16 * i + l16, m_lim - 1);
        const int n = fdiv(m, p.d_OHW), rem = m - n * OHW;
        const int oh = fdiv(rem, p.d_OW), ow = rem - oh * OW;
        abase[i] = ((n * PHt + oh * p.sh - pgr0) * RP + ow) * TC_PS + 4 * q;
    }

    floatx4 acc[TILES];
#pragma unroll
    for (int i = 0; i < TILES; i++) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};

    // ---- filter fragments straight from global memory -------------------------------------------------
    // lane (l16, q) of wavefront w needs, for channel group g of a half tap, B[c = 16g + 4q + s][oc0 + 16w + l16].
    // Address = (uniform base of the half tap, kept in scalar registers) + (per-lane 32-bit byte offset, fixed for the
    // whole kernel): the scalar-base form of the load instruction, no vector arithmetic. The empty asm keeps the
    // zero-extension of the offset next to the load; hoisted out of the tap loop (as it is otherwise) the offsets
    // become 64-bit register pairs and every load is preceded by a 64-bit vector add.
    const int b_co = oc0 + 16 * w + l16;
    const bool b_cov = b_co < p.CO;   // columns beyond CO are never stored; clamp their loads to a valid address
    unsigned b_lane[2][4];
#pragma unroll
    for (int g = 0; g < 2; g++)
#pragma unroll
        for (int s = 0; s < 4; s++) b_lane[g][s] = tap_filter_lane_bytes(p.b_sc, g, q, s, b_cov ? b_co : 0);
    auto load_b = [&](float (&b)[2][4], int icbase, int th, int tw) {
        const int sbase = __builtin_amdgcn_readfirstlane(tap_filter_half_tap_base<RAGGED>(p.b_off, p.b_sth, p.b_stw, p.b_sc, p.AC, icbase, th, tw));
        const char *sb = reinterpret_cast<const char *>(p.B + sbase);
#pragma unroll
        for (int g = 0; g < 2; g++) {
            // RAGGED: channels beyond AC (AC % 4 == 0: four at a time) are fetched from the half tap's first element
            const unsigned ok = tap_filter_lane_mask<RAGGED>(p.AC, icbase, g, q);
#pragma unroll
            for (int s = 0; s < 4; s++) {
                if (!RAGGED) asm volatile("" : "+v"(b_lane[g][s]));   // value unchanged
                b[g][s] = *reinterpret_cast<const float *>(sb + (b_lane[g][s] & ok));
            }
        }
    };
    // channels beyond AC: the halo holds zeros there, but 0 * (whatever the clamped load returned) must
    // not turn into NaN, so the fragment is zeroed when it is used
    auto mask_b = [&](float (&b)[2][4], int icbase) {
        if (!RAGGED) return;
#pragma unroll
        for (int g = 0; g < 2; g++) {
            const bool ok = icbase + 16 * g + 4 * q < p.AC;
#pragma unroll
            for (int s = 0; s < 4; s++) b[g][s] = ok ? b[g][s] : 0.f;
        }
    };

    const int taps = p.TH * p.TW;

    // A fragments of one 16-channel chunk: chunk ck (0..3) of the current tap starts 16*ck floats into the pixel. The
    // per-lane offsets cur[] point at the current tap and are moved by a uniform amount from tap to tap (adding the
    // tap's offset at every read cost one vector add per tile and chunk, and a vector instruction takes five to
    // nine cycles from the MFMAs). A strided layer keeps the columns of a row de-interleaved
    // (plane tw % sw), so that the 16 pixels of a tile are neighbours in LDS whatever the stride and the bank
    // pattern is the stride-1 one.
    int cur[TILES];
    auto tap_offset = [&](int th, int tw) {
        const int twq = fdiv(tw, p.d_sw), twr = tw - twq * p.sw;
        return (th * RP + twr * p.PWp + twq) * TC_PS;
    };
#pragma unroll
    for (int i = 0; i < TILES; i++) cur[i] = abase[i];
    auto read_a = [&](floatx4 (&a)[TILES], int ck) {
#pragma unroll
        for (int i = 0; i < TILES; i++) a[i] = *reinterpret_cast<const floatx4 *>(Hs + cur[i] + 16 * ck);
    };
    auto mfma_chunk = [&](const floatx4 (&a)[TILES], const float (&b)[4]) {
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
            for (int i = 0; i < TILES; i++)
                acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i][s], b[s], acc[i], 0, 0, 0);
    };
    // LDS reads of the next chunk issue in the shadow of this chunk's first MFMAs
    auto spread_reads = [&]() {
#pragma unroll
        for (int i = 0; i < TILES; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // 1 MFMA
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // 1 LDS read
        }
    };

    float bA[2][4], bB[2][4];
    floatx4 aP[TILES], aQ[TILES];   // A fragments ping-pong: the next chunk is read while the current one is multiplied
    load_b(bA, 0, 0, 0);   // first half tap; in flight while the halo is staged
    for (int ic0 = 0; ic0 < p.AC; ic0 += TC_ICC) {
        if (ic0 > 0) __syncthreads();   // everyone finished reading the previous pass's halo
        // Two workgroups share a compute unit so that one stages while the other multiplies. A wavefront that issues
        // MFMAs back to back keeps the SIMD's vector issue port occupied, and the address arithmetic of a staging
        // wavefront of the other workgroup at the same priority hardly ever gets a turn: staging ended exactly
        // when the other workgroup's MFMA loop did. Staging and the epilogue therefore run at a raised priority.
        __builtin_amdgcn_s_setprio(2);
        // ---- stage the halo (at raised priority, see above) ----
        tap_stage_halo(p, Hs, ic0, pgr0, rows, t);
        __syncthreads();

        // ---- main loop: one tap (four 16-channel chunks) per iteration ------------------------------------
        // Filter fragments ping-pong between bA and bB one half tap (two chunks) ahead, A fragments between aP
        // and aQ one chunk ahead. Every prefetch is unconditional (a branch around it would make every wait in the
        // loop assume the shorter queue): after the last tap it fetches the first half tap of the next pass, or
        // harmlessly re-fetches tap (0,0) of this one at the very end. The scheduling barriers pin each prefetch in
        // front of the chunk that hides its latency; left alone the compiler sinks the loads to their first use.
        __builtin_amdgcn_s_setprio(0);
        int th = 0, tw = 0, coff = 0;   // cur[] is at tap (0, 0) here
        read_a(aP, 0);
        for (int tap = 0; tap < taps; tap++) {
            int nth = th, ntw = tw + 1, nic = ic0;
            if (ntw == p.TW) { ntw = 0; nth = th + 1; }
            if (tap + 1 == taps) { nth = 0; ntw = 0; nic = ic0 + TC_ICC < p.AC ? ic0 + TC_ICC : ic0; }
            __builtin_amdgcn_sched_barrier(0);
            load_b(bB, ic0 + 32, th, tw);
            __builtin_amdgcn_sched_barrier(0);
            mask_b(bA, ic0);
            read_a(aQ, 1);
            mfma_chunk(aP, bA[0]);
            spread_reads();
            __builtin_amdgcn_sched_barrier(0);
            read_a(aP, 2);
            mfma_chunk(aQ, bA[1]);
            spread_reads();
            __builtin_amdgcn_sched_barrier(0);
            load_b(bA, nic, nth, ntw);
            __builtin_amdgcn_sched_barrier(0);
            mask_b(bB, ic0 + 32);
            read_a(aQ, 3);
            mfma_chunk(aP, bB[0]);
            spread_reads();
            __builtin_amdgcn_sched_barrier(0);
            {   // on to the next tap (after the last one: back to tap (0, 0))
                const int noff = tap_offset(nth, ntw), d = noff - coff;
                coff = noff;
#pragma unroll
                for (int i = 0; i < TILES; i++) cur[i] += d;
            }
            read_a(aP, 0);   // after the last tap of a pass: re-read once the next halo is staged
            mfma_chunk(aQ, bB[1]);
            spread_reads();
            __builtin_amdgcn_sched_barrier(0);
            th = nth;
            tw = ntw;
        }
    }
    (void)bA;
    (void)aP;
    __builtin_amdgcn_s_setprio(2);

    // ---- epilogue: transpose through LDS so every output pixel row is written as whole 256-byte lines ----
    __syncthreads();   // all wavefronts are done reading the halo
    float *Os = Hs;    // [P][TC_OS]
#pragma unroll
    for (int i = 0; i < TILES; i++)
#pragma unroll
        for (int r = 0; r < 4; r++) Os[(16 * i + 4 * q + r) * TC_OS + 16 * w + l16] = acc[i][r];
    __syncthreads();
    for (int idx = t; idx < P * 16; idx += 256) {
        const int pix = idx >> 4, cq = (idx & 15) * 4;
        const int m = m0 + pix;
        if (m < m_lim && oc0 + cq < p.CO)
            *reinterpret_cast<float4 *>(p.O + (size_t)m * p.CO + oc0 + cq) =
                epilogue4(*reinterpret_cast<const float4 *>(Os + pix * TC_OS + cq), p.ep, oc0 + cq, (size_t)m * p.CO + oc0 + cq);
    }
}

// Kernel-split backward-data for stride 2 x 2 with all four phases in ONE unit. The four output pixels of a 2 x 2 block
// (one per phase) read the same small window of deltaY, each through its own subset of the filter taps, so a unit of
// P "coarse" pixels stages the halo once per 64 channels and runs every tap of every phase on it - as many MFMAs per
// staged byte as a dense convolution with the whole filter, where a phase on its own has a quarter of them (one to four
// taps of a 3x3 filter). Accumulators exist per phase (compile-time index); the sequence of taps runs through the phases,
// filter fragments and input fragments prefetched across phase and pass boundaries exactly as in tap_conv_unit.
// A phase without taps (filter smaller than the stride) keeps its zeros and writes them.
template <int TILES, bool RAGGED>
__device__ __forceinline__ void tap_conv_merged_unit(const TapConvArgs &p, float *smem, const int m0, const int m_lim, const int oc0)
{
    constexpr int P = TILES * 16, NPH = 4;
    float *Hs = smem;

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int OW = p.d_OW.d, OHW = p.d_OHW.d, PHt = p.PHt, RP = p.RP;

    const int n_first = fdiv(m0, p.d_OHW);
    const int oh_first = fdiv(m0 - n_first * OHW, p.d_OW);
    const int pgr0 = n_first * PHt + oh_first;
    const int m_last = min(m0 + P, m_lim) - 1;
    const int n_last = fdiv(m_last, p.d_OHW);
    const int oh_last = fdiv(m_last - n_last * OHW, p.d_OW);
    const int rows = n_last * PHt + oh_last + p.TH - 1 - pgr0 + 1;   // p.TH, p.TW: the window all phases read together

    int abase[TILES];
#pragma unroll
    for (int i = 0; i < TILES; i++) {
        const int m = min(m0 + 16 * i + l16, m_lim - 1);
        const int n = fdiv(m, p.d_OHW), rem = m - n * OHW;
        const int oh = fdiv(rem, p.d_OW), ow = rem - oh * OW;
        abase[i] = ((n * PHt + oh - pgr0) * RP + ow) * TC_PS + 4 * q;
    }

    floatx4 acc[NPH][TILES];
#pragma unroll
    for (int f = 0; f < NPH; f++)
#pragma unroll
        for (int i = 0; i < TILES; i++) acc[f][i] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int b_co = oc0 + 16 * w + l16;
    const bool b_cov = b_co < p.CO;
    unsigned b_lane[2][4];
#pragma unroll
    for (int g = 0; g < 2; g++)
#pragma unroll
        for (int s = 0; s < 4; s++) b_lane[g][s] = tap_filter_lane_bytes(p.b_sc, g, q, s, b_cov ? b_co : 0);
    auto load_b = [&](float (&b)[2][4], int icbase, int f, int th, int tw) {   // f, th, tw uniform
        const int sbase = __builtin_amdgcn_readfirstlane(
            tap_filter_half_tap_base<RAGGED>(p.f_b_off[f], p.f_b_sth[f], p.b_stw, p.b_sc, p.AC, icbase, th, tw));
        const char *sb = reinterpret_cast<const char *>(p.B + sbase);
#pragma unroll
        for (int g = 0; g < 2; g++) {
            const unsigned ok = tap_filter_lane_mask<RAGGED>(p.AC, icbase, g, q);
#pragma unroll
            for (int s = 0; s < 4; s++) {
                if (!RAGGED) asm volatile("" : "+v"(b_lane[g][s]));
                b[g][s] = *reinterpret_cast<const float *>(sb + (b_lane[g][s] & ok));
            }
        }
    };
    auto mask_b = [&](float (&b)[2][4], int icbase) {
        if (!RAGGED) return;
#pragma unroll
        for (int g = 0; g < 2; g++) {
            const bool ok = icbase + 16 * g + 4 * q < p.AC;
#pragma unroll
            for (int s = 0; s < 4; s++) b[g][s] = ok ? b[g][s] : 0.f;
        }
    };
    // the first phase that has taps, from phase f on (NPH when there is none); uniform
    auto next_phase = [&](int f) {
        while (f < NPH && p.f_TH[f] * p.f_TW[f] == 0) f++;
        return f;
    };
    auto tap_offset = [&](int f, int th, int tw) { return ((th + p.f_row[f]) * RP + tw + p.f_col[f]) * TC_PS; };

    int cur[TILES];
    auto read_a = [&](floatx4 (&a)[TILES], int ck) {
#pragma unroll
        for (int i = 0; i < TILES; i++) a[i] = *reinterpret_cast<const floatx4 *>(Hs + cur[i] + 16 * ck);
    };
    auto spread_reads = [&]() {
#pragma unroll
        for (int i = 0; i < TILES; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    };

    const int f0 = next_phase(0);
    if (f0 < NPH) {
        float bA[2][4], bB[2][4];
        floatx4 aP[TILES], aQ[TILES];
        load_b(bA, 0, f0, 0, 0);
        for (int ic0 = 0; ic0 < p.AC; ic0 += TC_ICC) {
            if (ic0 > 0) __syncthreads();
            __builtin_amdgcn_s_setprio(2);
            tap_stage_halo(p, Hs, ic0, pgr0, rows, t);
            __syncthreads();
            __builtin_amdgcn_s_setprio(0);
            int coff = tap_offset(f0, 0, 0);
#pragma unroll
            for (int i = 0; i < TILES; i++) cur[i] = abase[i] + coff;
            read_a(aP, 0);
            pf_phase_loop<0, NPH>([&](auto fc) {
                constexpr int F = decltype(fc)::value;
                auto mfma_chunk = [&](const floatx4 (&a)[TILES], const float (&b)[4]) {
#pragma unroll
                    for (int s = 0; s < 4; s++)
#pragma unroll
                        for (int i = 0; i < TILES; i++)
                            acc[F][i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i][s], b[s], acc[F][i], 0, 0, 0);
                };
                const int TWf = p.f_TW[F], taps = p.f_TH[F] * TWf;
                int th = 0, tw = 0;
                for (int tap = 0; tap < taps; tap++) {
                    // what comes next: the phase's next tap, the first tap of the next phase that has any, or - after
                    // the last phase - the first tap of the next pass (of this pass again at the very end: unused)
                    int nf = F, nth = th, ntw = tw + 1, nic = ic0;
                    if (ntw == TWf) { ntw = 0; nth = th + 1; }
                    if (tap + 1 == taps) {
                        nth = 0; ntw = 0;
                        nf = next_phase(F + 1);
                        if (nf == NPH) { nf = f0; nic = ic0 + TC_ICC < p.AC ? ic0 + TC_ICC : ic0; }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    load_b(bB, ic0 + 32, F, th, tw);
                    __builtin_amdgcn_sched_barrier(0);
                    mask_b(bA, ic0);
                    read_a(aQ, 1);
                    mfma_chunk(aP, bA[0]);
                    spread_reads();
                    __builtin_amdgcn_sched_barrier(0);
                    read_a(aP, 2);
                    mfma_chunk(aQ, bA[1]);
                    spread_reads();
                    __builtin_amdgcn_sched_barrier(0);
                    load_b(bA, nic, nf, nth, ntw);
                    __builtin_amdgcn_sched_barrier(0);
                    mask_b(bB, ic0 + 32);
                    read_a(aQ, 3);
                    mfma_chunk(aP, bB[0]);
                    spread_reads();
                    __builtin_amdgcn_sched_barrier(0);
                    {
                        const int noff = tap_offset(nf, nth, ntw), d = noff - coff;
                        coff = noff;
#pragma unroll
                        for (int i = 0; i < TILES; i++) cur[i] += d;
                    }
                    read_a(aP, 0);   // after the last tap of a pass: re-read once the next halo is staged
                    mfma_chunk(aQ, bB[1]);
                    spread_reads();
                    __builtin_amdgcn_sched_barrier(0);
                    th = nth;
                    tw = ntw;
                }
            });
        }
        (void)bA;
        (void)aP;
    }
    __builtin_amdgcn_s_setprio(2);

    // ---- epilogue: phase by phase through LDS, every pixel's channels leave as whole 256-byte lines ----------------------
    float *Os = Hs;    // [P][TC_OS]
#pragma unroll
    for (int f = 0; f < NPH; f++) {
        __syncthreads();   // the halo (or the previous phase's staging) has been read by everyone
#pragma unroll
        for (int i = 0; i < TILES; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) Os[(16 * i + 4 * q + r) * TC_OS + 16 * w + l16] = acc[f][i][r];
        __syncthreads();
        for (int idx = t; idx < P * 16; idx += 256) {
            const int pix = idx >> 4, cq = (idx & 15) * 4;
            const int m = m0 + pix;
            if (m < m_lim && oc0 + cq < p.CO) {
                const int n = fdiv(m, p.d_OHW), rem = m - n * OHW;
                const int i = fdiv(rem, p.d_OW), j = rem - i * OW;
                const size_t elem = (size_t)(p.f_o_off[f] + n * p.o_sn + i * p.o_sh + j * p.o_sw + oc0 + cq);
                *reinterpret_cast<float4 *>(p.O + elem) = epilogue4(*reinterpret_cast<const float4 *>(Os + pix * TC_OS + cq), p.ep, oc0 + cq, elem);
            }
        }
    }
}

// Persistent grid over 16-pixel tiles: each XCD (workgroups are dealt round-robin to the 8 XCDs) works on a contiguous
// run of tiles, each of its workgroups on a contiguous share of that run, equal to within one tile; a share is processed
// in units of 4, 3 or 2 tiles so that no MFMA is spent on tiles that do not exist (whole units of one size left some
// compute units a quarter more work than others: 3136 tiles on 256 compute units).
template <bool RAGGED>
__global__ __launch_bounds__(256, 2) void tap_conv_merged_kernel(const TapConvArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int oc0 = blockIdx.y * 64;
    const int G = gridDim.x;
    const int X = G < 8 ? G : 8;                           // groups of workgroups: the XCDs (fewer workgroups than XCDs: one each)
    const int xcd = blockIdx.x % X, xi = blockIdx.x / X;
    const int wgs = G / X + (xcd < G % X ? 1 : 0);         // workgroups of this group
    const int T = p.full_units;                            // tiles in all
    const int x_lo = xcd * (T / X) + min(xcd, T % X), x_n = T / X + (xcd < T % X ? 1 : 0);   // this group's run
    const int q = x_n / wgs, r = x_n - q * wgs;
    int tile = x_lo + xi * q + min(xi, r);
    int left = q + (xi < r ? 1 : 0);
    bool first = true;
    while (left > 0) {
        if (!first) __syncthreads();   // the previous unit's output staging has been read
        first = false;
        const int m0 = tile * 16;
        if (left >= 6 || left == 4) {
            tap_conv_merged_unit<4, RAGGED>(p, smem, m0, p.M, oc0);
            tile += 4; left -= 4;
        } else if (left == 5 || left == 3) {
            tap_conv_merged_unit<3, RAGGED>(p, smem, m0, min(p.M, m0 + 48), oc0);
            tile += 3; left -= 3;
        } else {   // 2, or a single tile (a share of one tile: the second tile is computed and not stored)
            tap_conv_merged_unit<2, RAGGED>(p, smem, m0, min(p.M, m0 + 16 * left), oc0);
            tile += 2; left -= 2;
        }
    }
}

// The grid is persistent: as many workgroups as the device holds at once (per block of 64 output channels), each taking
// whole units round-robin. Units that would make a partial last round are cut into pieces of fewer tiles, one piece
// per workgroup, so that every workgroup does the same amount of work (c4b: 896 units on 512 workgroups).
// Consecutive units share halo rows: each XCD (workgroups are dealt round-robin to the 8 XCDs) works on a contiguous
// run of units, so the shared rows are served by that XCD's L2.
template <int TILES, bool RAGGED>
__global__ __launch_bounds__(256, 2) void tap_conv_kernel(const TapConvArgs p)
{
    constexpr int P = TILES * 16;
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int oc0 = blockIdx.y * 64;
    const int G = gridDim.x;
    const int xcd = blockIdx.x & 7, xi = blockIdx.x >> 3;
    const int wgs = (G >> 3) + (xcd < (G & 7) ? 1 : 0);   // workgroups on this XCD
    bool first = true;
    auto whole_units = [&]() {
        const int U = p.full_units;
        const int lo = xcd * (U >> 3) + min(xcd, U & 7), n = (U >> 3) + (xcd < (U & 7) ? 1 : 0);
        for (int i = xi; i < n; i += wgs) {
            if (!first) __syncthreads();   // the previous unit's output staging has been read
            first = false;
            tap_conv_unit<TILES, RAGGED>(p, smem, (lo + i) * P, p.M, oc0);
        }
    };
    auto one_piece = [&]() {
        const int U = p.pieces;
        const int lo = xcd * (U >> 3) + min(xcd, U & 7), n = (U >> 3) + (xcd < (U & 7) ? 1 : 0);
        for (int i = xi; i < n; i += wgs) {
            const int piece = lo + i;
            const int unit = p.full_units + piece / p.piece_split, k = piece - (piece / p.piece_split) * p.piece_split;
            const int m0 = unit * P + k * 16 * p.piece_tiles;
            const int m_lim = min(min(m0 + 16 * p.piece_tiles, (unit + 1) * P), p.M);
            if (m0 >= m_lim) continue;
            if (!first) __syncthreads();
            first = false;
            if (p.piece_tiles > 2) tap_conv_unit<4, RAGGED>(p, smem, m0, m_lim, oc0);
            else tap_conv_unit<2, RAGGED>(p, smem, m0, m_lim, oc0);
        }
    };
    whole_units();
    one_piece();
}

// Rows of LDS halo the worst unit needs: output rows spanned by P consecutive pixels, TH-1 extra rows,
// and TH-1 more for every image border crossed.
static int tap_conv_lds_rows(int M, int P, int OH, int OW, int TH, int sh, int PHt)
{
    const int OHW = OH * OW;
    int worst = 0;
    const int units = (M + P - 1) / P;
    const int scan = units < 4096 ? units : 4096;
    for (int u = 0; u < scan; u++) {
        const long m0 = (long)u * P, m1 = (m0 + P < M ? m0 + P : M) - 1;
        const int n0 = (int)(m0 / OHW), oh0 = (int)(m0 % OHW) / OW;
        const int n1 = (int)(m1 / OHW), oh1 = (int)(m1 % OHW) / OW;
        const int rows = (n1 * PHt + oh1 * sh + TH - 1) - (n0 * PHt + oh0 * sh) + 1;
        if (rows > worst) worst = rows;
    }
    if (units > scan) {   // analytic bound for what was not scanned
        const int span = (P + OW - 2) / OW + 1;
        const int cross = (P + OHW - 2) / OHW + 1;
        const int bound = (span - 1) * sh + TH + cross * (PHt - OH * sh > 0 ? PHt - OH * sh : 0);
        if (bound > worst) worst = bound;
    }
    return worst;
}

template <int TILES, bool RAGGED>
static hipError_t launch_tc(hipStream_t stream, TapConvArgs a, size_t lds, int cus)
{
    constexpr auto kern = tap_conv_kernel<TILES, RAGGED>;
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    const int units = (a.M + TILES * 16 - 1) / (TILES * 16), ocb = (a.CO + 63) / 64;
    const int slots = cus * (2 * lds <= 160 * 1024 ? 2 : 1);   // workgroups the device holds at once
    int G = slots / ocb;
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

hipError_t launch_tap_conv_prefetch(hipStream_t stream, const float *A, const float *B, float *O,
                                    int N, int AH, int AW, int AC, int OH, int OW, int CO,
                                    int TH, int TW, int ph, int pw,
                                    int b_off, int b_sth, int b_stw, int b_sc, int b_sn, const Epilogue &ep, int cus);

// Returns hipErrorNotSupported when the shape does not fit this kernel (caller falls back to the
// generic implicit GEMM); otherwise launches.
hipError_t launch_tap_conv(hipStream_t stream, const float *A, const float *B, float *O,
                           int N, int AH, int AW, int AC, int OH, int OW, int CO,
                           int TH, int TW, int ph, int pw,
                           int b_off, int b_sth, int b_stw, int b_sc, const float *bias, int sh, int sw, int b_sn, const Epilogue *ep)
{
    if (sh < 1 || sw < 1 || sh > 4 || sw > 4) return hipErrorNotSupported;
    if (OH != (AH + 2 * ph - TH) / sh + 1 || OW != (AW + 2 * pw - TW) / sw + 1) return hipErrorNotSupported;
    if (AC < 32 || TH > 7 || TW > 7) return hipErrorNotSupported;
    const long M = (long)N * OH * OW;
    if ((long)N * (AH + 2 * ph) >= (1L << 24)) return hipErrorNotSupported;

    TapConvArgs a{};
    a.A = A; a.B = B; a.O = O; a.ep = ep ? *ep : bias_epilogue(bias);
    a.M = (int)M; a.CO = CO;
    a.AH = AH; a.AW = AW; a.AC = AC;
    a.TH = TH; a.TW = TW; a.ph = ph; a.pw = pw;
    a.PHt = AH + 2 * ph; a.PWt = AW + 2 * pw;
    a.sh = sh; a.sw = sw;
    a.PWp = (a.PWt + sw - 1) / sw; a.RP = sw * a.PWp;
    a.d_sw = make_fastdiv(sw);
    a.b_off = b_off; a.b_sth = b_sth; a.b_stw = b_stw; a.b_sc = b_sc;
    a.d_OW = make_fastdiv(OW);
    a.d_OHW = make_fastdiv(OH * OW);
    a.d_PHt = make_fastdiv(a.PHt);
    a.d_PWt = make_fastdiv(a.PWt);

    const int cus = device_cu_count();
    if (cus < 1) return hipErrorNotSupported;
    if (sh == 1 && sw == 1) {   // the variant that prefetches the halo, where it applies
        const hipError_t e = launch_tap_conv_prefetch(stream, A, B, O, N, AH, AW, AC, OH, OW, CO, TH, TW, ph, pw,
                                                      b_off, b_sth, b_stw, b_sc, b_sn, a.ep, cus);
        if (e != hipErrorNotSupported) return e;
    }
    if (b_sn != 1) return hipErrorNotSupported;   // the kernel below reads the filter along the output channel only
    // pixels per workgroup: 7 tiles (112) when that divides the row/image structure better, else 8 (128)
    const int OHW = OH * OW;
    int tiles = 8;
    if ((OHW % 112 == 0 || (2 * OW) % 112 == 0 || 112 % OW == 0) && !(OHW % 128 == 0 || 128 % OW == 0)) tiles = 7;
    // stride 1: two workgroups per CU; a strided layer touches sh*sw input pixels per output pixel and gets the whole LDS
    const size_t budget = (sh == 1 && sw == 1) ? 80 * 1024 : 160 * 1024;
    for (int attempt = 0; attempt < 2; attempt++) {
        const int P = tiles * 16;
        a.lds_rows = tap_conv_lds_rows(a.M, P, OH, OW, TH, sh, a.PHt);
        size_t halo = (size_t)a.lds_rows * a.RP * TC_PS + 4;   // + one spare 16-byte slot
        const size_t stage = (size_t)P * TC_OS;
        if (halo < stage) halo = stage;
        const size_t lds = halo * sizeof(float);
        if (lds <= budget) {
            const bool ragged = (AC % TC_ICC) != 0;
            if (tiles == 7) return ragged ? launch_tc<7, true>(stream, a, lds, cus) : launch_tc<7, false>(stream, a, lds, cus);
            return ragged ? launch_tc<8, true>(stream, a, lds, cus) : launch_tc<8, false>(stream, a, lds, cus);
        }
        tiles = (tiles == 8) ? 7 : 8;
    }
    return hipErrorNotSupported;
}

// Kernel-split backward-data for stride 2 x 2 with even output sizes: all four phases in one launch, one halo per unit
// (see tap_conv_merged_unit). Phase f is the dense stride-1 problem
//   O[o_off[f] + n*o_sn + i*o_sh + j*o_sw + co] = sum_{th < TH[f], tw < TW[f], c < AC} A[n, i - ph[f] + th, j - pw[f] + tw, c]
//                                                 * B[b_off[f] + th*b_sth[f] + tw*b_stw + c*b_sc + co]
// for i < OHt, j < OWt (the same for every phase); TH[f] = 0 marks a phase without taps, which is written as zeros.
// Returns hipErrorNotSupported (nothing launched) when the layer does not fit.
hipError_t launch_tap_conv_merged(hipStream_t stream, const float *A, const float *B, float *O, int N, int AH, int AW, int AC, int CO,
                                  int OHt, int OWt, const int *TH, const int *TW, const int *ph, const int *pw, const int *b_off,
                                  const int *b_sth, int b_stw, int b_sc, const int *o_off, int o_sn, int o_sh, int o_sw, const Epilogue *ep)
{
    if (AC < 32 || (CO & 3) || OHt < 1 || OWt < 1) return hipErrorNotSupported;
    const int cus = device_cu_count();
    if (cus < 1) return hipErrorNotSupported;
    int PH = 0, PW = 0;
    for (int f = 0; f < 4; f++) {
        if (TH[f] == 0 || TW[f] == 0) continue;
        if (TH[f] < 0 || TW[f] < 0 || ph[f] < 0 || pw[f] < 0) return hipErrorNotSupported;
        if (ph[f] > PH) PH = ph[f];
        if (pw[f] > PW) PW = pw[f];
    }
    TapConvArgs a{};
    int WH = 1, WW = 1;
    for (int f = 0; f < 4; f++) {
        const bool any = TH[f] > 0 && TW[f] > 0;
        a.f_TH[f] = any ? TH[f] : 0; a.f_TW[f] = any ? TW[f] : 0;
        a.f_row[f] = any ? PH - ph[f] : 0; a.f_col[f] = any ? PW - pw[f] : 0;
        a.f_b_off[f] = any ? b_off[f] : 0; a.f_b_sth[f] = any ? b_sth[f] : 0;
        a.f_o_off[f] = o_off[f];
        if (any && a.f_row[f] + TH[f] > WH) WH = a.f_row[f] + TH[f];
        if (any && a.f_col[f] + TW[f] > WW) WW = a.f_col[f] + TW[f];
    }
    if (WH > 7 || WW > 7) return hipErrorNotSupported;
    a.A = A; a.B = B; a.O = O; a.ep = ep ? *ep : bias_epilogue(nullptr);
    a.CO = CO;
    a.AH = AH; a.AW = AW; a.AC = AC;
    a.TH = WH; a.TW = WW; a.ph = PH; a.pw = PW;
    a.PHt = AH + PH > OHt + WH - 1 ? AH + PH : OHt + WH - 1;
    a.PWt = AW + PW > OWt + WW - 1 ? AW + PW : OWt + WW - 1;
    a.sh = 1; a.sw = 1;
    a.PWp = a.PWt; a.RP = a.PWt;
    a.d_sw = make_fastdiv(1);
    a.b_stw = b_stw; a.b_sc = b_sc;
    a.o_sn = o_sn; a.o_sh = o_sh; a.o_sw = o_sw;
    const long M = (long)N * OHt * OWt;
    if (M >= (1L << 30) || (long)N * a.PHt >= (1L << 24)) return hipErrorNotSupported;
    a.M = (int)M;
    a.d_OW = make_fastdiv(OWt);
    a.d_OHW = make_fastdiv(OHt * OWt);
    a.d_PHt = make_fastdiv(a.PHt);
    a.d_PWt = make_fastdiv(a.PWt);
    // LDS rows of the worst unit: up to 64 pixels from any tile boundary on
    constexpr int P = 64;
    {
        const int OHW = OHt * OWt, tiles = (a.M + 15) / 16;
        int worst = 0;
        const int scan = tiles < 65536 ? tiles : 65536;
        for (int u = 0; u < scan; u++) {
            const long m0 = (long)u * 16, m1 = (m0 + P < a.M ? m0 + P : a.M) - 1;
            const int n0 = (int)(m0 / OHW), oh0 = (int)(m0 % OHW) / OWt;
            const int n1 = (int)(m1 / OHW), oh1 = (int)(m1 % OHW) / OWt;
            const int rows = (n1 * a.PHt + oh1 + WH - 1) - (n0 * a.PHt + oh0) + 1;
            if (rows > worst) worst = rows;
        }
        if (tiles > scan) {   // analytic bound for what was not scanned
            const int span = (P + OWt - 2) / OWt + 1, cross = (P + OHW - 2) / OHW + 1;
            const int bound = (span - 1) + WH + cross * (a.PHt - OHt > 0 ? a.PHt - OHt : 0);
            if (bound > worst) worst = bound;
        }
        a.lds_rows = worst;
    }
    size_t halo = (size_t)a.lds_rows * a.RP * TC_PS + 4;
    const size_t stage = (size_t)P * TC_OS;
    if (halo < stage) halo = stage;
    const size_t lds = halo * sizeof(float);
    if (lds > 80 * 1024) return hipErrorNotSupported;
    const int tiles = (a.M + 15) / 16, ocb = (CO + 63) / 64;
    a.full_units = tiles;
    int G = 2 * cus / ocb;
    if (G < 1) G = 1;
    if (G > (tiles + 1) / 2) G = (tiles + 1) / 2;   // at least two tiles per workgroup
    if ((AC % TC_ICC) != 0) {
        if (hipError_t e = ensure_dynamic_lds<tap_conv_merged_kernel<true>>(lds); e != hipSuccess) return e;
        hipLaunchKernelGGL(tap_conv_merged_kernel<true>, dim3(G, ocb, 1), dim3(256), lds, stream, a);
    } else {
        if (hipError_t e = ensure_dynamic_lds<tap_conv_merged_kernel<false>>(lds); e != hipSuccess) return e;
        hipLaunchKernelGGL(tap_conv_merged_kernel<false>, dim3(G, ocb, 1), dim3(256), lds, stream, a);
    }
    return hipGetLastError();
}

}  // namespace alpha

// Host-side walk over every filter address tap_conv_kernel generates for one block of 64 output channels per lane
// (same loop structure as tap_conv_unit: first half tap, then per tap the second half tap and the next tap's first
// one), using the kernel's own address functions. Writes the smallest and largest element index read.
#pragma GCC visibility push(default)
extern "C" int alpha_selfcheck_tap_filter_extent(int AC, int CO, int TH, int TW, int b_off, int b_sth, int b_stw, int b_sc,
                                                 long *lo_out, long *hi_out)
{
    using namespace alpha;
    if (AC < 4 || (AC & 3) || CO < 4 || TH < 1 || TW < 1 || !lo_out || !hi_out) return -1;
    const bool ragged = (AC % TC_ICC) != 0;
    long lo = (1L << 62), hi = -(1L << 62);
    auto visit = [&](int icbase, int th, int tw) {
        const int sbase = ragged ? tap_filter_half_tap_base<true>(b_off, b_sth, b_stw, b_sc, AC, icbase, th, tw)
                                 : tap_filter_half_tap_base<false>(b_off, b_sth, b_stw, b_sc, AC, icbase, th, tw);
        for (int oc0 = 0; oc0 < CO; oc0 += 64)
            for (int w = 0; w < 4; w++)
                for (int lane = 0; lane < 64; lane++) {
                    const int l16 = lane & 15, q = lane >> 4;
                    const int b_co = oc0 + 16 * w + l16;
                    const int co = b_co < CO ? b_co : 0;
                    for (int g = 0; g < 2; g++) {
                        const unsigned ok = ragged ? tap_filter_lane_mask<true>(AC, icbase, g, q) : tap_filter_lane_mask<false>(AC, icbase, g, q);
                        for (int s = 0; s < 4; s++) {
                            const long idx = (long)sbase + (long)((tap_filter_lane_bytes(b_sc, g, q, s, co) & ok) / 4);
                            if (idx < lo) lo = idx;
                            if (idx > hi) hi = idx;
                        }
                    }
                }
    };
    visit(0, 0, 0);
    const int taps = TH * TW;
    for (int ic0 = 0; ic0 < AC; ic0 += TC_ICC) {
        int th = 0, tw = 0;
        for (int tap = 0; tap < taps; tap++) {
            int nth = th, ntw = tw + 1, nic = ic0;
            if (ntw == TW) { ntw = 0; nth = th + 1; }
            if (tap + 1 == taps) { nth = 0; ntw = 0; nic = ic0 + TC_ICC < AC ? ic0 + TC_ICC : ic0; }
            visit(ic0 + 32, th, tw);
            visit(nic, nth, ntw);
            th = nth; tw = ntw;
        }
    }
    *lo_out = lo;
    *hi_out = hi;
    return 0;
}
#pragma GCC visibility pop
