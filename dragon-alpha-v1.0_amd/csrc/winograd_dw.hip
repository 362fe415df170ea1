// Backward-filter of 3x3 stride-1 layers by Winograd F(3x3, 2x2), fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950.
//
//   deltaW[oc, fh, fw, ic] = sum over 2x2 tiles t of the output image of
//       sum_{a,b<2} deltaY[t; a, b, oc] * X[t; a + fh, b + fw, ic]              (X[t]: the 4x4 input patch under tile t)
//     = A^T [ sum_t (G y_t G^T)[oc] .* (B^T x_t B)[ic] ] A
//   with G = [[1,0],[.5,.5],[.5,-.5],[0,1]],  B^T = [[1,0,-1,0],[0,1,1,0],[0,-1,1,0],[0,-1,0,1]],
//        A^T = [[1,1,1,0],[0,1,-1,0],[0,1,1,1]]:
// 16 multiplies per tile and channel pair where the direct sum has 36. The sum over tiles is the reduction index of 16
// GEMMs (one per transform position xi), M[xi][oc][ic] += Yh[xi][t][oc] * Xh[xi][t][ic]; the output transform is applied
// once, at the end, to the accumulators. The reference has no such algorithm (its backward-filter natives are
// cu32/dW/dconv3d_dW.cuh); this is an additional path of this build with the split-K contract of the GemmSK entries:
// slice z of the tiles writes its partial result to deltaW (z = 0) or deltaW_buf[z-1], no atomics, and a fixed launch
// gives bit-identical results. (The partition is over tiles, not over the reference's pixel ranges: the partial results
// differ from the direct kernels', their sum does not, up to rounding.)
//
// A workgroup owns one slice, 64 output channels and 32 input channels, and has six wavefronts. Four multiply: wavefront w
// accumulates output channels [16w, 16w+16) x 32 input channels x 16 xi = 128 registers. Tiles advance in chunks of 8.
// Two wavefronts stage the patches: a thread loads the 4x4 patch of one (tile, pair of input channels) two chunks before
// it is transformed and writes Xh[tile][32][16 xi] into the LDS buffer that is multiplied in the chunk after; one barrier
// per chunk joins the two kinds (wavefronts of one kind doing both jobs needed scheduling directives, spilled, or moved
// the accumulators through AGPRs). deltaY does not pass through LDS: a multiplying wavefront is the only user of its 16
// output channels, so its lanes load their own 2x2 tiles and transform them in registers into MFMA operands.
// In LDS the 16 xi of a (tile, channel) are contiguous, so a lane's patch operand for four xi is one 128-bit read (an
// operand per xi as a 32-bit read - three LDS instructions per two MFMAs - cost 30 cycles per pair of MFMAs). A (tile,
// channel) takes 80 bytes, its four 16-byte groups of xi stored permuted (group g at position g ^ (channel / 16 % 4)): the
// 16 lanes of a read (16 consecutive channels) and the 16 lanes of a staging write (channels 2 apart) then both touch 16
// different 16-byte bank groups.
#include "common.hpp"
#include <type_traits>

namespace alpha {

struct WinoDwArgs {
    const float *X;      // [N, IH, IW, IC]
    const float *dY;     // [N, OH, OW, OC]
    float *dW;           // [OC, 3, 3, IC]
    float *dW_buf;       // [GZ-1][OC, 3, 3, IC]
    int IH, IW, IC, OH, OW, OC, ph, pw;
    int TC, TR, TRC;     // tile columns, tile rows, tiles per image
    int ntiles, S, GZ;   // N*TRC; tiles per slice (a multiple of 8); slices
    int x_bytes, y_bytes;   // X at most 1 GB, deltaY below 2 GB
    // a thread's tile moves on by 8 per chunk: (ty, tx) += (adv_ty, adv_tx), then at most one wrap of tx and one of ty;
    // its patch origin in X and its tile origin in deltaY (element offsets) move by dx0 / dy0 plus wx1 / wy1 when tx
    // wraps and wx2 / wy2 when ty wraps (into the next image)
    int adv_ty, adv_tx, dx0, dy0, wx1, wy1, wx2, wy2;
    FastDiv d_TC, d_TRC;
};

constexpr int WD_TK = 8;                        // tiles per chunk
constexpr int WD_CS = 20;                       // floats per (tile, channel): 16 xi + 4 (see the layout note above)
constexpr int WD_XBUF = WD_TK * 32 * WD_CS;     // Xh[tile][32 input channels][16 xi + 4]: one LDS buffer
constexpr int WD_BUF = WD_XBUF;
constexpr unsigned WD_OOR = 0x80000000u;        // beyond both descriptors: the load returns 0
constexpr unsigned WD_OOR_COL = 0x40000000u;    // added to a valid offset of X (at most 1 GB) or to WD_OOR: beyond too

__global__ __launch_bounds__(384) void winograd_dw_kernel(const WinoDwArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float wd_smem[];   // Xh[2][WD_BUF]
    float *smem = wd_smem;

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int ic0 = blockIdx.x * 32, oc0 = blockIdx.y * 64, z = blockIdx.z;
    const int tile_begin = z * p.S;
    const int tile_end = min(p.ntiles, tile_begin + p.S);
    const int nchunks = tile_end > tile_begin ? (tile_end - tile_begin + WD_TK - 1) / WD_TK : 0;

    floatx4 acc[16][2];
#pragma unroll
    for (int x = 0; x < 16; x++) {
        acc[x][0] = floatx4{0.f, 0.f, 0.f, 0.f};
        acc[x][1] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // Tile positions are kept per thread from chunk to chunk and moved on by additions only (no division, no multiplication:
    // recomputing a chunk's offsets from tile indices cost more issue slots than the chunk's MFMAs).
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.X), 0, p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.dY), 0, p.y_bytes, 0x00020000);
    const int row_elems = p.IW * p.IC;
    struct TileCur {
        int tile, ty, tx, x00, y00;   // x00 / y00: element offsets of X[n, 2ty-ph, 2tx-pw, channel] (may be negative) / deltaY[n, 2ty, 2tx, channel]
    };
    auto cur_init = [&](TileCur &c, int tile, int x_channel, int y_channel) {
        c.tile = tile;
        const int n = fdiv(tile, p.d_TRC), rem = tile - n * p.TRC;
        c.ty = fdiv(rem, p.d_TC);
        c.tx = rem - c.ty * p.TC;
        c.x00 = (n * p.IH + 2 * c.ty - p.ph) * row_elems + (2 * c.tx - p.pw) * p.IC + x_channel;
        c.y00 = ((n * p.OH + 2 * c.ty) * p.OW + 2 * c.tx) * p.OC + y_channel;
    };
    auto cur_advance = [&](TileCur &c) {   // 8 tiles on
        c.tile += WD_TK;
        c.tx += p.adv_tx;
        c.ty += p.adv_ty;
        c.x00 += p.dx0;
        c.y00 += p.dy0;
        const bool w1 = c.tx >= p.TC;
        c.tx -= w1 ? p.TC : 0;
        c.ty += w1 ? 1 : 0;
        c.x00 += w1 ? p.wx1 : 0;
        c.y00 += w1 ? p.wy1 : 0;
        const bool w2 = c.ty >= p.TR;
        c.ty -= w2 ? p.TR : 0;
        c.x00 += w2 ? p.wx2 : 0;
        c.y00 += w2 ? p.wy2 : 0;
    };
    typedef std::integral_constant<int, 0> Set0;
    typedef std::integral_constant<int, 1> Set1;

    // ---- wavefronts 4 and 5 stage the patches: a thread takes (tile, pair of input channels) - 16 64-bit loads two chunks
    //      ahead, B^T x B, eight 128-bit LDS writes into the buffer that is multiplied in the next chunk. Offsets outside the
    //      tensor (padding, tiles past the slice, channels past the end) are beyond the descriptor and read as zeros. -------
    if (t >= 256) {
        if (nchunks == 0) return;
        __builtin_amdgcn_s_setprio(3);   // few instructions, and the multiplying wavefronts wait for them at the barrier
        const int item = t - 256, st = item >> 4, x_ch = 2 * (item & 15);
        const bool xc_ok = ic0 + x_ch < p.IC;          // IC % 4 == 0: a pair is valid as a whole
        const int swz_wx = (x_ch >> 4) & 3;            // (channel / 16) % 4 of the channels this thread writes
        TileCur cur;
        cur_init(cur, tile_begin + st, ic0 + x_ch, 0);
        float2 xr[2][4][4];   // raw patches: set s holds a chunk of parity s, requested two chunks before it is transformed
        auto request = [&](auto set_c) {   // the 16 loads of the chunk the tile cursor stands on
            constexpr int SET = decltype(set_c)::value;
            const bool ok = cur.tile < tile_end && xc_ok;
            const int ih0 = 2 * cur.ty - p.ph, iw0 = 2 * cur.tx - p.pw;
            unsigned rowterm[4], colterm[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const unsigned rv = (unsigned)cur.x00 * 4u + (unsigned)(i * row_elems) * 4u, cv = (unsigned)(i * p.IC) * 4u;
                rowterm[i] = (ok && (unsigned)(ih0 + i) < (unsigned)p.IH) ? rv : WD_OOR;
                colterm[i] = ((unsigned)(iw0 + i) < (unsigned)p.IW) ? cv : WD_OOR_COL;
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    xr[SET][i][j] = __builtin_bit_cast(float2, __builtin_amdgcn_raw_buffer_load_b64(x_rsrc, rowterm[i] + colterm[j], 0, 0));
        };
        // Xh = B^T x B per channel; the 4 xi of a row are one 128-bit element of the (tile, channel)
        auto transform = [&](auto set_c, int buf, bool store) {
            constexpr int SET = decltype(set_c)::value;
            float *Xh = smem + buf * WD_BUF + (st * 32 + x_ch) * WD_CS;
#pragma unroll
            for (int k = 0; k < 2; k++) {
                float r[4][4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float x0 = k ? xr[SET][0][j].y : xr[SET][0][j].x, x1 = k ? xr[SET][1][j].y : xr[SET][1][j].x;
                    const float x2 = k ? xr[SET][2][j].y : xr[SET][2][j].x, x3 = k ? xr[SET][3][j].y : xr[SET][3][j].x;
                    r[0][j] = x0 - x2;
                    r[1][j] = x1 + x2;
                    r[2][j] = x2 - x1;
                    r[3][j] = x3 - x1;
                }
                if (store) {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        *reinterpret_cast<floatx4 *>(Xh + k * WD_CS + ((i ^ swz_wx) << 2)) =
                            floatx4{r[i][0] - r[i][2], r[i][1] + r[i][2], r[i][2] - r[i][1], r[i][3] - r[i][1]};
                }
            }
        };
        request(Set0{});
        transform(Set0{}, 0, true);   // chunk 0, waited for
        cur_advance(cur);
        request(Set1{});              // chunk 1
        cur_advance(cur);
        request(Set0{});              // chunk 2
        __syncthreads();
        // chunk c: chunk c+1 (requested two chunks ago) is transformed into the other buffer, chunk c+3 requested into the
        // set it leaves. Two chunks per round so that the sets are fixed registers; the loads of the second half are issued
        // even when that chunk does not exist (only its LDS writes and its barrier are skipped).
        for (int c = 0; c < nchunks; c += 2) {
            transform(Set1{}, 1, true);
            cur_advance(cur);
            request(Set1{});
            __syncthreads();
            const bool more = c + 1 < nchunks;
            transform(Set0{}, 0, more);
            cur_advance(cur);
            request(Set0{});
            if (more) __syncthreads();
        }
        return;
    }

    // ---- wavefronts 0-3 multiply. deltaY does not go through LDS: wavefront w is the only one that needs output channels
    //      [16w, 16w+16), so lane (l16, q) loads the 2x2 tiles of channel 16w + l16 for its two tiles of a chunk (q and
    //      4 + q) itself, two chunks ahead, and transforms them in registers into the 32 MFMA operands of the chunk. The
    //      patches come from LDS. ------------------------------------------------------------------------------------------
    if (nchunks > 0) {
        const int y_ch = oc0 + 16 * w + l16;
        const bool yc_ok = y_ch < p.OC;
        const int y_px = p.OC, y_row = p.OW * p.OC;
        TileCur ca, cb;
        cur_init(ca, tile_begin + q, 0, y_ch);
        cur_init(cb, tile_begin + 4 + q, 0, y_ch);
        float yraw[2][2][4];   // [set][kk][pixel]
        auto request_one = [&](const TileCur &c, float (&y)[4]) {
            const bool ok = c.tile < tile_end && yc_ok;
            const bool right = 2 * c.tx + 1 < p.OW, below = 2 * c.ty + 1 < p.OH;
            const unsigned o = (unsigned)c.y00 * 4u;
            const unsigned o00 = ok ? o : WD_OOR, o01 = (ok && right) ? o + (unsigned)y_px * 4u : WD_OOR;
            const unsigned o10 = (ok && below) ? o + (unsigned)y_row * 4u : WD_OOR;
            const unsigned o11 = (ok && right && below) ? o + (unsigned)(y_row + y_px) * 4u : WD_OOR;
            y[0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(y_rsrc, o00, 0, 0));
            y[1] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(y_rsrc, o01, 0, 0));
            y[2] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(y_rsrc, o10, 0, 0));
            y[3] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(y_rsrc, o11, 0, 0));
        };
        auto request = [&](auto set_c) {
            constexpr int SET = decltype(set_c)::value;
            request_one(ca, yraw[SET][0]);
            request_one(cb, yraw[SET][1]);
        };
        // Yh' = G' y G'^T with G' = [[1,0],[1,1],[1,-1],[0,1]] = G without its factors 1/2, which are applied to the
        // accumulators once, at the end
        float ya[2][16];
        auto transform = [&](auto set_c) {
            constexpr int SET = decltype(set_c)::value;
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                const float y00v = yraw[SET][kk][0], y01v = yraw[SET][kk][1], y10v = yraw[SET][kk][2], y11v = yraw[SET][kk][3];
                float g[4][2];
                g[0][0] = y00v; g[0][1] = y01v;
                g[1][0] = y00v + y10v; g[1][1] = y01v + y11v;
                g[2][0] = y00v - y10v; g[2][1] = y01v - y11v;
                g[3][0] = y10v; g[3][1] = y11v;
#pragma unroll
                for (int a = 0; a < 4; a++) {
                    ya[kk][4 * a + 0] = g[a][0];
                    ya[kk][4 * a + 1] = g[a][0] + g[a][1];
                    ya[kk][4 * a + 2] = g[a][0] - g[a][1];
                    ya[kk][4 * a + 3] = g[a][1];
                }
            }
        };
        int rdx0[4], rdx1[4];   // float offsets of this lane's patch operands for xi group gx (tile q; channels l16, 16 + l16)
#pragma unroll
        for (int gx = 0; gx < 4; gx++) {
            rdx0[gx] = (q * 32 + l16) * WD_CS + (gx << 2);
            rdx1[gx] = (q * 32 + 16 + l16) * WD_CS + ((gx ^ 1) << 2);
        }
        // One chunk = 8 groups of 8 MFMAs: (4 tiles kk, 4 xi) x (two blocks of input channels); two 128-bit LDS reads per
        // group, one group ahead. The two MFMAs into one accumulator (kk = 0, 1) are 4 groups apart.
        auto multiply = [&](int buf) {
            const float *B = smem + buf * WD_BUF;
            auto frag = [&](int g, floatx4 &fb0, floatx4 &fb1) {
                const int kk = g >> 2, gx = g & 3;
                fb0 = *reinterpret_cast<const floatx4 *>(B + rdx0[gx] + kk * 4 * 32 * WD_CS);
                fb1 = *reinterpret_cast<const floatx4 *>(B + rdx1[gx] + kk * 4 * 32 * WD_CS);
            };
            floatx4 b0[2], b1[2];
            frag(0, b0[0], b1[0]);
#pragma unroll
            for (int g = 0; g < 8; g++) {
                if (g + 1 < 8) frag(g + 1, b0[(g + 1) & 1], b1[(g + 1) & 1]);
#pragma unroll
                for (int x = 0; x < 4; x++) {
                    const int xi = 4 * (g & 3) + x;
                    const float a = ya[g >> 2][xi];
                    acc[xi][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b0[g & 1][x], acc[xi][0], 0, 0, 0);
                    acc[xi][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b1[g & 1][x], acc[xi][1], 0, 0, 0);
                }
            }
        };
        request(Set0{});       // chunk 0
        cur_advance(ca);
        cur_advance(cb);
        request(Set1{});       // chunk 1
        __syncthreads();
        for (int c = 0; c < nchunks; c += 2) {
            transform(Set0{});
            cur_advance(ca);
            cur_advance(cb);
            request(Set0{});   // chunk c + 2
            multiply(0);
            __syncthreads();
            const bool more = c + 1 < nchunks;
            transform(Set1{});
            cur_advance(ca);
            cur_advance(cb);
            request(Set1{});   // chunk c + 3
            if (more) {
                multiply(1);
                __syncthreads();
            }
        }
    }

    // ---- deltaW block = A^T M A per lane, which holds all 16 xi of output channels 16w + 4q + r, input channels
    //      16j + l16; M[a][b] takes the factors of G left out above (1/2 for a in {1,2}, 1/2 for b in {1,2}); 16 lanes
    //      store 64 consecutive bytes ---------------------------------------------------------------------------------------
    float *dst = (z == 0) ? p.dW : p.dW_buf + (size_t)(z - 1) * p.OC * 9 * p.IC;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int ic = ic0 + 16 * j + l16;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int oc = oc0 + 16 * w + 4 * q + r;
            float s[3][4];
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const float cb = (b == 1 || b == 2) ? 0.5f : 1.f;
                const float m0 = acc[b][j][r] * cb, m1 = acc[4 + b][j][r] * (0.5f * cb), m2 = acc[8 + b][j][r] * (0.5f * cb),
                            m3 = acc[12 + b][j][r] * cb;
                s[0][b] = m0 + m1 + m2;
                s[1][b] = m1 - m2;
                s[2][b] = m1 + m2 + m3;
            }
            if (oc < p.OC && ic < p.IC) {
                float *o = dst + (size_t)oc * 9 * p.IC + ic;
#pragma unroll
                for (int k = 0; k < 3; k++) {
                    o[(3 * k + 0) * p.IC] = s[k][0] + s[k][1] + s[k][2];
                    o[(3 * k + 1) * p.IC] = s[k][1] - s[k][2];
                    o[(3 * k + 2) * p.IC] = s[k][1] + s[k][2] + s[k][3];
                }
            }
        }
    }
}

// Same contract as launch_deltaW_rows for 3x3 stride-1 layers (slice z -> deltaW or deltaW_buf[z-1]); returns
// hipErrorNotSupported (nothing launched) when the layer does not fit.
hipError_t launch_deltaW_winograd(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                                  int N, int IH, int IW, int IC, int OH, int OW, int OC, int ph, int pw, int GZ)
{
    if (OH != IH + 2 * ph - 2 || OW != IW + 2 * pw - 2) return hipErrorNotSupported;
    if (IC < 4 || OC < 4 || (OC & 3) || N < 1 || OH < 1 || OW < 1 || GZ < 1) return hipErrorNotSupported;
    if (!winograd_deltaW_fits(N, IH, IW, IC, OH, OW, OC)) return hipErrorNotSupported;
    const long x_bytes = (long)N * IH * IW * IC * 4, y_bytes = (long)N * OH * OW * OC * 4;
    // the patch offsets are sums of a row term and a column term that mark "outside" by 2 GB and 1 GB: X must end below 1 GB
    if (x_bytes + 8L * IC > (1L << 30) || y_bytes >= (1L << 31)) return hipErrorNotSupported;
    WinoDwArgs a{};
    a.X = X; a.dY = dY; a.dW = dW; a.dW_buf = dW_buf;
    a.IH = IH; a.IW = IW; a.IC = IC; a.OH = OH; a.OW = OW; a.OC = OC; a.ph = ph; a.pw = pw;
    a.TC = (OW + 1) / 2;
    a.TR = (OH + 1) / 2;
    a.TRC = a.TR * a.TC;
    const long nt = (long)N * a.TRC;
    if (nt >= (1L << 30)) return hipErrorNotSupported;
    a.ntiles = (int)nt;
    a.GZ = GZ;
    {   // 8 tiles on: whole images, whole tile rows, tile columns; then at most one wrap of the column and one of the row
        const int adv_n = WD_TK / a.TRC, rest = WD_TK % a.TRC;
        a.adv_ty = rest / a.TC;
        a.adv_tx = rest % a.TC;
        const long imgX = (long)IH * IW * IC, imgY = (long)OH * OW * OC;
        const long rowX = 2L * IW * IC, rowY = 2L * OW * OC, colX = 2L * IC, colY = 2L * OC;
        a.dx0 = (int)(adv_n * imgX + a.adv_ty * rowX + a.adv_tx * colX);
        a.dy0 = (int)(adv_n * imgY + a.adv_ty * rowY + a.adv_tx * colY);
        a.wx1 = (int)(rowX - a.TC * colX);
        a.wy1 = (int)(rowY - a.TC * colY);
        a.wx2 = (int)(imgX - a.TR * rowX);
        a.wy2 = (int)(imgY - a.TR * rowY);
    }
    a.S = (int)(((nt + GZ - 1) / GZ + WD_TK - 1) / WD_TK * WD_TK);
    a.x_bytes = (int)x_bytes; a.y_bytes = (int)y_bytes;
    a.d_TC = make_fastdiv(a.TC);
    a.d_TRC = make_fastdiv(a.TRC);
    constexpr auto kern = winograd_dw_kernel;
    const size_t lds = (size_t)2 * WD_BUF * sizeof(float);
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((IC + 31) / 32, (OC + 63) / 64, GZ), dim3(384), lds, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
