// Backward-filter for stride-1 layers by streaming output rows, fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950.
//
//   deltaW[oc, fh, fw, ic] = sum over pixels k = (n, oh, ow) of the K slice of  deltaY[k, oc] * X[n, oh-ph+fh, ow-pw+fw, ic]
//
// A workgroup (4 wavefronts) owns one K slice (blockIdx.z, the reference's partition), OCB = 16*OCT output
// channels and 64 input channels, for ALL filter taps. It walks the output rows of its slice; per row it holds in
// LDS the deltaY row (double buffered) and the FH input rows that row touches (a ring of FH+1 row slots, so the
// one new input row of the next output row is fetched while the current row is being multiplied). Both operands
// are read from LDS 32 bits at a time, lanes across channels (the reduction index of this GEMM is the pixel,
// which is the slow axis of both tensors). Wavefront w owns input channels [16w, 16w+16): per 4 pixels it
// reads OCT deltaY fragments and FH*FW shifted X fragments and issues OCT*FH*FW MFMAs, so each X element read
// from memory is used for every tap it participates in and every deltaY element for all FH*FW taps.
// Pixels outside the K slice (a slice may begin or end inside a row) are staged as zeros. No atomics: slice z
// stores to deltaW (z = 0) or deltaW_buf[z-1]; a fixed launch gives bit-identical results.
//
// Narrow images: R output rows ("a chunk") are multiplied per step so that a step always has up to 64 pixels of
// work; the ring then holds 2R + FH - 1 input rows and R new ones are fetched per step.
//
// LDS strides: 32-bit reads of 64 lanes are conflict-free when the four 16-lane groups (consecutive pixels) start
// 16 banks apart: pixel strides are 16 or 48 floats modulo 64 (X: 80; deltaY: 48 for 32 channels, 80 for 64); with
// 16 channels the deltaY stride is 32 (two groups share banks: a 2-way conflict on 1 of 10 reads). An unpadded,
// XOR-permuted layout (74 KB instead of 96 KB for 56-pixel rows, so two workgroups per compute unit) was measured
// slower: its per-tap lane offsets cost more address arithmetic and LDS instructions than the co-residency gains.
#include "common.hpp"

namespace alpha {

struct DwRowsArgs {
    const float *X;
    const float *dY;
    float *dW;
    float *dW_buf;
    float *dB;        // NULL, or the bias gradient: slice z writes sum over its pixels of deltaY[., oc] to dB (z = 0)
    float *dB_buf;    // or dB_buf[z-1][OC]
    int N, IH, IW, IC, OH, OW, OC;
    int ph, pw;
    int GK, GK_slice, GZ;
    int OWp;     // OW rounded up to a multiple of 4 (pixels beyond OW are staged as zeros)
    int PW;      // OWp + FW - 1 input columns staged per row; staged column cp holds iw = cp - pw
    int PWA;     // columns allocated per row slot: PW, or PW + 8 zero columns when R = 1 (see the single-row loop)
    int R;       // output rows multiplied per step (a "chunk"); R*OWp <= 64 and R*PW <= 64
    int CPI;     // chunks per image = ceil(OH / R)
    int SLOTS;   // input-row slots in LDS = 2R + FH - 1
    int steps2;  // groups of 4 pixels per chunk, rounded up to an even count (the deltaY pixels added are zeros)
    FastDiv d_OW, d_OH, d_OWp, d_PW, d_R, d_SLOTS;
};

constexpr int DWR_XS = 80;   // X row slot pixel stride (floats): 64 channels + 16

// ONE_ROW: one output row per chunk (p.R == 1), which lets the compiler drop the multi-row loop and its bookkeeping.
template <int FH, int FW, int OCT, bool ONE_ROW>
__global__ __launch_bounds__(256, OCT <= 2 ? 2 : 1) void delta_w_rows_kernel(const DwRowsArgs p)   // <= 256 registers where two workgroups fit a compute unit
{
    constexpr int OCB = 16 * OCT;
    constexpr int YS = OCB + 16;             // deltaY pixel stride (floats): 32, 48 or 80
    constexpr int YQ = OCT;                  // float4 per thread per deltaY chunk (R*OWp <= 64, host-checked)
    constexpr int XQ = 4;                    // float4 per thread per R new X rows  (R*PW <= 64, host-checked)

    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int R = ONE_ROW ? 1 : p.R, OWp = p.OWp, PW = p.PW, SLOTS = p.SLOTS;
    const int ybuf_floats = p.steps2 * 4 * YS, slot_floats = p.PWA * DWR_XS;
    float *Ybuf = smem;                               // [2][R*OWp][YS]
    float *Xring = smem + 2 * ybuf_floats;            // [SLOTS][PW][DWR_XS]

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int ic0 = blockIdx.x * 64, oc0 = blockIdx.y * OCB, z = blockIdx.z;
    const int OW = p.OW, OH = p.OH;

    const int k_start = p.GK_slice * z;
    const int k_end = (z != p.GZ - 1) ? k_start + p.GK_slice : p.GK;
    float *dst = (z == 0) ? p.dW : p.dW_buf + (size_t)(z - 1) * p.OC * (FH * FW) * p.IC;

    constexpr int BG = 64 / OCB;             // lane groups of a wavefront when lanes run over the OCB channels
    const bool do_bias = p.dB != nullptr && blockIdx.x == 0;
    float bsum = 0.f;
    floatx4 acc[FH][FW][OCT];
#pragma unroll
    for (int a = 0; a < FH; a++)
#pragma unroll
        for (int b = 0; b < FW; b++)
#pragma unroll
            for (int c = 0; c < OCT; c++) acc[a][b][c] = floatx4{0.f, 0.f, 0.f, 0.f};

    // ---- staging helpers. Loads go through buffer descriptors, one over this slice's pixels of deltaY and one over
    // the image of X that is being read: an offset outside the descriptor returns zeros, which is exactly what pixels
    // outside the slice, rows above and below the image and (through a per-thread offset that is out of range from the
    // start) padding columns, padding pixels and channels past the end need. A thread stages the same places of every
    // chunk: its byte offset within the chunk and its LDS place are computed once, per chunk a load costs one add.
    // (Vector instructions issued while staging take issue slots from the MFMAs - a wave has its SIMD to itself here -
    // and compares, selects and 64-bit address arithmetic per element were a tenth of the kernel's time.)
    // Threads beyond the last element repeat the last element (same bytes to the same place). ---------------------
    constexpr int NEVER = 0x40000000;   // plus any offset within a slice or an image (host-checked < 2^29): still out of range
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(p.dY) + (size_t)k_start * p.OC, 0, k_start < k_end ? (k_end - k_start) * p.OC * 4 : 0, 0x00020000);
    const int x_image_bytes = p.IH * p.IW * p.IC * 4;
    float4 yreg[YQ], xreg[XQ];
    const int y_quads = p.steps2 * 4 * (OCB / 4);   // includes the zero pixels that pad the chunk to an even step count
    int y_voff[YQ], y_rr[YQ], y_lds[YQ];
#pragma unroll
    for (int u = 0; u < YQ; u++) {
        const int idx = min(t + 256 * u, y_quads - 1);
        const int px = idx / (OCB / 4), cq = (idx % (OCB / 4)) * 4;
        const int rr = fdiv(px, p.d_OWp), ow = px - rr * OWp;
        const bool ok = rr < R && ow < OW && oc0 + cq < p.OC;
        y_rr[u] = rr;
        y_voff[u] = ok ? ((rr * OW + ow) * p.OC + oc0 + cq) * 4 : NEVER;
        y_lds[u] = px * YS + cq;
    }
    const int x_quads = R * PW * 16;
    int x_voff[XQ], x_rr[XQ], x_lds[XQ];
#pragma unroll
    for (int u = 0; u < XQ; u++) {
        const int idx = min(t + 256 * u, x_quads - 1);
        const int px = idx >> 4, cq = (idx & 15) * 4;
        const int rr = fdiv(px, p.d_PW), cp = px - rr * PW;
        const int iw = cp - p.pw;
        const bool ok = (unsigned)iw < (unsigned)p.IW && ic0 + cq < p.IC;
        x_rr[u] = rr;
        x_voff[u] = ok ? ((rr * p.IW + iw) * p.IC + ic0 + cq) * 4 : NEVER;
        x_lds[u] = cp * DWR_XS + cq;
    }

    // deltaY rows oh0 .. oh0+R-1 of image n; chunk pixel (rr, ow) lives at LDS pixel index rr*OWp + ow
    auto load_y = [&](int n, int oh0) {
        const int rel = __builtin_amdgcn_readfirstlane((((n * OH + oh0) * OW) - k_start) * p.OC * 4);   // may be negative
#pragma unroll
        for (int u = 0; u < YQ; u++) {
            int off = y_voff[u] + rel;
            if (!ONE_ROW) off = y_rr[u] < OH - oh0 ? off : NEVER;   // the image's last chunk may have fewer rows
            yreg[u] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(y_rsrc, off, 0, 0));
        }
    };
    auto store_y = [&](int buf) {
#pragma unroll
        for (int u = 0; u < YQ; u++) *reinterpret_cast<float4 *>(Ybuf + buf * ybuf_floats + y_lds[u]) = yreg[u];
    };
    // R padded input rows rp0 .. rp0+R-1 of image n (padded row rp holds ih = rp - ph; rows outside the image are out
    // of the descriptor's range: zeros); padded row rp lives in slot rp % SLOTS
    auto load_x = [&](int n, int rp0) {
        const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float *>(p.X) + (size_t)n * p.IH * p.IW * p.IC, 0, x_image_bytes, 0x00020000);
        const int rel = __builtin_amdgcn_readfirstlane((rp0 - p.ph) * p.IW * p.IC * 4);   // may be negative
#pragma unroll
        for (int u = 0; u < XQ; u++)
            xreg[u] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, x_voff[u] + rel, 0, 0));
    };
    auto store_x = [&](int rp0, int nrows) {   // nrows < R: only the first nrows of the R rows are kept
        const int s0 = rp0 - fdiv(rp0, p.d_SLOTS) * SLOTS;          // uniform
        if (ONE_ROW) {
            float *slot = Xring + s0 * slot_floats;
#pragma unroll
            for (int u = 0; u < XQ; u++) *reinterpret_cast<float4 *>(slot + x_lds[u]) = xreg[u];
        } else {
#pragma unroll
            for (int u = 0; u < XQ; u++) {
                if (x_rr[u] < nrows) {
                    int slot = s0 + x_rr[u];                             // x_rr < R <= SLOTS
                    slot -= slot >= SLOTS ? SLOTS : 0;
                    *reinterpret_cast<float4 *>(Xring + slot * slot_floats + x_lds[u]) = xreg[u];
                }
            }
        }
    };
    // the whole window of chunk (n, oh0): padded rows oh0 .. oh0+R+FH-2 in up to FH pieces of R rows, all fetched
    // before the first is stored so that their latencies overlap
    auto stage_window = [&](int n, int oh0) {
        float4 wreg[FH][XQ];
#pragma unroll
        for (int pc = 0; pc < FH; pc++) {
            load_x(n, oh0 + pc * R);
#pragma unroll
            for (int u = 0; u < XQ; u++) wreg[pc][u] = xreg[u];
        }
#pragma unroll
        for (int pc = 0; pc < FH; pc++) {
            const int nrows = min(R, R + FH - 1 - pc * R);     // <= 0: nothing left for this piece
#pragma unroll
            for (int u = 0; u < XQ; u++) xreg[u] = wreg[pc][u];
            if (nrows > 0) store_x(oh0 + pc * R, nrows);
        }
    };

    if (k_start < k_end) {
        const int gr_first = fdiv(k_start, p.d_OW), gr_last = fdiv(k_end - 1, p.d_OW);
        int n = fdiv(gr_first, p.d_OH);
        int ci = fdiv(gr_first - n * OH, p.d_R);                      // chunk within the image
        const int n_last = fdiv(gr_last, p.d_OH);
        const int ci_last = fdiv(gr_last - n_last * OH, p.d_R);
        load_y(n, ci * R);
        store_y(0);
        stage_window(n, ci * R);
        // columns PW .. PWA-1 of every slot stay zero for the whole kernel (nothing is staged there)
        for (int idx = t; idx < SLOTS * (p.PWA - PW) * (DWR_XS / 4); idx += 256) {
            const int per_slot = (p.PWA - PW) * (DWR_XS / 4);
            const int slot = idx / per_slot, rest = idx - slot * per_slot;
            *reinterpret_cast<float4 *>(Xring + slot * slot_floats + PW * DWR_XS + rest * 4) = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        __syncthreads();

        const int steps2 = p.steps2;
        for (int it = 0;; it++) {
            const int oh0 = ci * R;
            const bool has_next = n < n_last || ci < ci_last;
            int n2 = n, ci2 = ci + 1;
            if (ci2 == p.CPI) { ci2 = 0; n2 = n + 1; }
            const bool same_image = n2 == n;
            if (has_next) {
                load_y(n2, ci2 * R);
                if (same_image) load_x(n, oh0 + R + FH - 1);   // the R new padded rows of the next chunk
            }

            // ---- bias gradient: column sums of the staged deltaY chunk (its masked pixels are zeros). Wavefront w adds
            // pixels [16w, 16w+16) in a fixed order; only the workgroups of the first input-channel block do it. --------
            if (do_bias) {
                const float *yc = Ybuf + (it & 1) * ybuf_floats + (lane & (OCB - 1));
#pragma unroll
                for (int j = 0; j < 16 / BG; j++) {
                    const int px = 16 * w + BG * j + (lane / OCB);
                    if (px < p.steps2 * 4) bsum += yc[px * YS];
                }
            }

            // ---- multiply this chunk: pixels in groups of 4 (lane group q takes pixel 4*k4 + q of the chunk) --------
            const float *yb = Ybuf + (it & 1) * ybuf_floats + q * YS + l16;
            const float *xb = Xring + q * DWR_XS + 16 * w + l16;
            const int s0 = oh0 - fdiv(oh0, p.d_SLOTS) * SLOTS;           // ring slot of the chunk's first padded row

            // Read position of the next step, kept in scalar registers: deltaY advances 4 pixels per step; the input
            // position advances 4 columns and, at the end of an output row, one ring slot. Steps that pad the chunk
            // to an even count (their deltaY pixels are zeros) and the read-ahead past the last step stay on the
            // last real input position, so that nothing uninitialised is ever multiplied.
            int yo = 0, col = 0, px = 0, xo[FH], nslot = s0 + FH;
            nslot -= nslot >= SLOTS ? SLOTS : 0;
#pragma unroll
            for (int fh = 0; fh < FH; fh++) {
                int slot = s0 + fh;
                slot -= slot >= SLOTS ? SLOTS : 0;
                xo[fh] = slot * slot_floats;
            }
            const int px_last = R * OWp - 4;

            float a0[OCT], b0[FH][FW], a1[OCT], b1[FH][FW];
            auto frags = [&](float (&a)[OCT], float (&b)[FH][FW]) {
#pragma unroll
                for (int c = 0; c < OCT; c++) a[c] = yb[yo + 16 * c];
#pragma unroll
                for (int fh = 0; fh < FH; fh++) {
                    const float *xr = xb + xo[fh] + col * DWR_XS;
#pragma unroll
                    for (int fw = 0; fw < FW; fw++) b[fh][fw] = xr[fw * DWR_XS];
                }
                yo += 4 * YS;
                const bool move = px < px_last;
                const bool wrap = move && col + 4 == OWp;
                px += 4;
                col = wrap ? 0 : (move ? col + 4 : col);
#pragma unroll
                for (int fh = 0; fh + 1 < FH; fh++) xo[fh] = wrap ? xo[fh + 1] : xo[fh];
                xo[FH - 1] = wrap ? nslot * slot_floats : xo[FH - 1];
                const int ns = nslot + 1 == SLOTS ? 0 : nslot + 1;
                nslot = wrap ? ns : nslot;
            };
            auto mfmas = [&](const float (&a)[OCT], const float (&b)[FH][FW]) {
#pragma unroll
                for (int fh = 0; fh < FH; fh++)
#pragma unroll
                    for (int fw = 0; fw < FW; fw++)
#pragma unroll
                        for (int c = 0; c < OCT; c++)
                            acc[fh][fw][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[c], b[fh][fw], acc[fh][fw][c], 0, 0, 0);
            };
            // One step = FH*FW*OCT MFMAs on the fragments read during the previous step, with the reads and address
            // arithmetic of the next step spread between them (a wave has the SIMD to itself, so whatever is not
            // issued in the shadow of an MFMA is lost time). Reads are unconditional: a branch around them would turn
            // the wait before the MFMAs into a wait for everything.
            auto interleave = [&]() {
#pragma unroll
                for (int g = 0; g < FH + 1; g++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);   // 2 MFMA
                    __builtin_amdgcn_sched_group_barrier(0x006, 4, 0);   // up to 4 VALU / SALU
                    __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);   // up to 3 LDS reads
                }
            };
            // Half-way through the chunk the next chunk's rows (requested above, arrived by now) go to their LDS places:
            // the other deltaY buffer and the ring slots the current chunk does not read. Done after the loop instead,
            // these stores, their barrier and the refill of the read pipeline cost 2500 cycles per chunk with no MFMA
            // in flight (a chunk of 56 pixels multiplies for 11400).
            const int mid = (steps2 / 2) & ~1;
            auto store_next = [&]() {
                if (has_next) {
                    store_y((it + 1) & 1);
                    if (same_image) store_x(oh0 + R + FH - 1, R);
                }
            };
            if constexpr (ONE_ROW) {
                // One output row per chunk: the read positions only ever advance by 4 pixels, so they live in
                // per-lane pointers bumped by a constant (scalar bookkeeping is not free either: every scalar
                // instruction of the wave delays its next MFMA by two to three cycles, and the general path below
                // spends ~23 of them per step). The step that pads the chunk to an even count and the read-ahead
                // past the last step run into the 8 zero columns behind the row.
                const float *yp = yb;
                const float *xp[FH];
#pragma unroll
                for (int fh = 0; fh < FH; fh++) xp[fh] = xb + xo[fh];
                auto frags1 = [&](float (&a)[OCT], float (&b)[FH][FW]) {
#pragma unroll
                    for (int c = 0; c < OCT; c++) a[c] = yp[16 * c];
#pragma unroll
                    for (int fh = 0; fh < FH; fh++) {
#pragma unroll
                        for (int fw = 0; fw < FW; fw++) b[fh][fw] = xp[fh][fw * DWR_XS];
                        xp[fh] += 4 * DWR_XS;
                    }
                    yp += 4 * YS;
                };
                frags1(a0, b0);
                for (int k4 = 0; k4 < mid; k4 += 2) {
                    __builtin_amdgcn_sched_barrier(0);
                    frags1(a1, b1);
                    mfmas(a0, b0);
                    interleave();
                    __builtin_amdgcn_sched_barrier(0);
                    frags1(a0, b0);
                    mfmas(a1, b1);
                    interleave();
                }
                store_next();
                for (int k4 = mid; k4 < steps2; k4 += 2) {
                    __builtin_amdgcn_sched_barrier(0);
                    frags1(a1, b1);
                    mfmas(a0, b0);
                    interleave();
                    __builtin_amdgcn_sched_barrier(0);
                    frags1(a0, b0);
                    mfmas(a1, b1);
                    interleave();
                }
            } else {
                frags(a0, b0);
                for (int k4 = 0; k4 < mid; k4 += 2) {
                    __builtin_amdgcn_sched_barrier(0);
                    frags(a1, b1);
                    mfmas(a0, b0);
                    interleave();
                    __builtin_amdgcn_sched_barrier(0);
                    frags(a0, b0);
                    mfmas(a1, b1);
                    interleave();
                }
                store_next();
                for (int k4 = mid; k4 < steps2; k4 += 2) {
                    __builtin_amdgcn_sched_barrier(0);
                    frags(a1, b1);
                    mfmas(a0, b0);
                    interleave();
                    __builtin_amdgcn_sched_barrier(0);
                    frags(a0, b0);
                    mfmas(a1, b1);
                    interleave();
                }
            }

            if (!has_next) break;
            __syncthreads();
            if (!same_image) {   // first chunk of the next image: its whole window is new
                stage_window(n2, 0);
                __syncthreads();
            }
            n = n2;
            ci = ci2;
        }
    }

    if (do_bias) {
        // lanes of a wavefront that share a channel (wavefront shuffles), then the four wavefronts through LDS in order
        if (BG >= 2) bsum += __shfl_xor(bsum, 32);
        if (BG >= 4) bsum += __shfl_xor(bsum, 16);
        __syncthreads();   // the staging buffers are free
        if (lane < OCB) smem[w * OCB + lane] = bsum;
        __syncthreads();
        if (t < OCB && oc0 + t < p.OC) {
            float *bdst = (z == 0) ? p.dB : p.dB_buf + (size_t)(z - 1) * p.OC;
            bdst[oc0 + t] = ((smem[t] + smem[OCB + t]) + smem[2 * OCB + t]) + smem[3 * OCB + t];
        }
    }

    // ---- store: lane holds input channel ic0 + 16w + l16 and output channels 16c + 4q + r --------------------------
    const int ic = ic0 + 16 * w + l16;
#pragma unroll
    for (int fh = 0; fh < FH; fh++)
#pragma unroll
        for (int fw = 0; fw < FW; fw++)
#pragma unroll
            for (int c = 0; c < OCT; c++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int oc = oc0 + 16 * c + 4 * q + r;
                    if (oc < p.OC && ic < p.IC) dst[(((size_t)oc * FH + fh) * FW + fw) * p.IC + ic] = acc[fh][fw][c][r];
                }
}

template <int FH, int FW, int OCT, bool ONE_ROW>
static hipError_t launch_dwr_rows(hipStream_t stream, const DwRowsArgs &a, size_t lds)
{
    constexpr auto kern = delta_w_rows_kernel<FH, FW, OCT, ONE_ROW>;
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    constexpr int OCB = 16 * OCT;
    dim3 grid((a.IC + 63) / 64, (a.OC + OCB - 1) / OCB, a.GZ);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, a);
    return hipGetLastError();
}

template <int FH, int FW, int OCT>
static hipError_t launch_dwr(hipStream_t stream, DwRowsArgs a)
{
    constexpr int OCB = 16 * OCT, YS = OCB + 16;
    // rows per step: as many as keep the chunk within 64 pixels and the R new input rows within 64 staged columns
    int limit = 64 / a.PW;
    if (limit > 64 / a.OWp) limit = 64 / a.OWp;
    if (limit < 1) return hipErrorNotSupported;
    if (limit > a.OH) limit = a.OH;
    const int nchunks = (a.OH + limit - 1) / limit;
    a.R = (a.OH + nchunks - 1) / nchunks;
    a.CPI = (a.OH + a.R - 1) / a.R;
    a.SLOTS = 2 * a.R + FH - 1;
    a.PWA = a.R == 1 ? a.PW + 8 : a.PW;
    a.steps2 = ((a.R * a.OWp) / 4 + 1) & ~1;
    a.d_R = make_fastdiv(a.R);
    a.d_SLOTS = make_fastdiv(a.SLOTS);
    a.d_OWp = make_fastdiv(a.OWp);
    a.d_PW = make_fastdiv(a.PW);
    {   // the staging loads address a slice of deltaY and an image of X with 32-bit offsets that must stay below 2^29
        const long last = (long)a.GK - (long)a.GK_slice * (a.GZ - 1);
        const long slice = last > a.GK_slice ? last : a.GK_slice;
        if ((slice + (long)a.R * a.OW) * a.OC * 4 >= (1L << 29)) return hipErrorNotSupported;
        if ((long)(a.IH + a.R + FH) * a.IW * a.IC * 4 >= (1L << 29)) return hipErrorNotSupported;
    }
    const size_t lds = ((size_t)2 * a.steps2 * 4 * YS + (size_t)a.SLOTS * a.PWA * DWR_XS) * sizeof(float);
    if (lds > 160 * 1024) return hipErrorNotSupported;
    return a.R == 1 ? launch_dwr_rows<FH, FW, OCT, true>(stream, a, lds) : launch_dwr_rows<FH, FW, OCT, false>(stream, a, lds);
}

// Returns hipErrorNotSupported (nothing launched) when the layer does not fit; the caller then uses the generic kernel.
hipError_t launch_deltaW_rows(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                              int N, int IH, int IW, int IC, int OH, int OW, int OC, int FH, int FW,
                              int sh, int sw, int ph, int pw, int GK_slice, int GZ, float *dB, float *dB_buf)
{
    if (sh != 1 || sw != 1) return hipErrorNotSupported;
    if (OH != IH + 2 * ph - FH + 1 || OW != IW + 2 * pw - FW + 1) return hipErrorNotSupported;
    if (IC < 16 || OC < 16) return hipErrorNotSupported;
    DwRowsArgs a{};
    a.X = X; a.dY = dY; a.dW = dW; a.dW_buf = dW_buf; a.dB = dB; a.dB_buf = dB_buf;
    a.N = N; a.IH = IH; a.IW = IW; a.IC = IC; a.OH = OH; a.OW = OW; a.OC = OC;
    a.ph = ph; a.pw = pw;
    a.GK = N * OH * OW; a.GK_slice = GK_slice; a.GZ = GZ;
    a.OWp = (OW + 3) & ~3;
    a.PW = a.OWp + FW - 1;
    a.d_OW = make_fastdiv(OW);
    a.d_OH = make_fastdiv(OH);
    if (FH == 3 && FW == 3) {
        // 32 output channels per workgroup unless that leaves most of the 256 CUs without a workgroup
        const long wgs = (long)((IC + 63) / 64) * ((OC + 31) / 32) * GZ;
        return wgs >= 200 ? launch_dwr<3, 3, 2>(stream, a) : launch_dwr<3, 3, 1>(stream, a);
    }
    if (FH == 1 && FW == 1) return launch_dwr<1, 1, 4>(stream, a);
    return hipErrorNotSupported;
}

}  // namespace alpha
