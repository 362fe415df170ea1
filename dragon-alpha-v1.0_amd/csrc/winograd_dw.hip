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
// A workgroup owns one slice, 64 output channels and 32 input channels. Four of its eight wavefronts multiply: wavefront w
// accumulates output channels [16w, 16w+16) x 32 input channels x 16 xi = 128 registers. The other four stage: tiles
// advance in chunks of 8; a staging thread loads the 4x4 patch of one (tile, input channel) and the 2x2 tile of one (tile,
// pair of output channels) a chunk before they are transformed, and writes Xh[tile][32][16 xi], Yh[tile][64][16 xi] into
// the LDS buffer that is multiplied in the chunk after. In LDS the 16 xi of a (tile, channel) are contiguous, so a lane's
// operand for four xi is one 128-bit read (an operand per xi as a 32-bit read - three LDS instructions per two MFMAs -
// cost 30 cycles per pair of MFMAs); the four 16-byte groups of a (tile, channel) are stored permuted (group g at position
// g ^ (channel / 4 % 4)), which spreads the 16 lanes of a read over all banks.
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
constexpr int WD_XBUF = WD_TK * 32 * 16;        // Xh[tile][32 input channels][16 xi]
constexpr int WD_YBUF = WD_TK * 64 * 16;        // Yh[tile][64 output channels][16 xi]
constexpr int WD_BUF = WD_XBUF + WD_YBUF;
constexpr unsigned WD_OOR = 0x80000000u;        // beyond both descriptors: the load returns 0
constexpr unsigned WD_OOR_COL = 0x40000000u;    // added to a valid offset of X (at most 1 GB) or to WD_OOR: beyond too

__global__ __launch_bounds__(512) void winograd_dw_kernel(const WinoDwArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float wd_smem[];   // [2][WD_BUF]
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

    // ---- staging: thread -> tile st of the chunk; input channel ic0 + sc for the patch, output channels oc0 + 2 sc,
    //      oc0 + 2 sc + 1 for the deltaY tile. Offsets outside the tensors (padding, rows / columns past an odd output
    //      size, tiles past the slice, channels past the end) are beyond the descriptors and read as zeros. The thread's
    //      tile position is kept from chunk to chunk and moved on by additions only (no division, no multiplication:
    //      recomputing 20 offsets per chunk from the tile index cost more issue slots than the chunk's 64 MFMAs). --------
    const int pt = t & 255, st = pt >> 5, sc = pt & 31;   // staging wavefronts (t >= 256) only
    const bool xc_ok = ic0 + sc < p.IC, yc_ok = oc0 + 2 * sc < p.OC;   // OC % 4 == 0: a pair is valid as a whole
    const int swz_w = (sc >> 2) & 3, swz_wy = (sc >> 1) & 3;            // (channel / 4) % 4 of the channel(s) this thread writes
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.X), 0, p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.dY), 0, p.y_bytes, 0x00020000);
    const int row_elems = p.IW * p.IC;
    int tile_cur = tile_begin + st, ty, tx, x00, y00;   // x00: element offset of X[n, 2ty-ph, 2tx-pw, ic0+sc] (may be negative)
    {
        const int n = fdiv(tile_cur, p.d_TRC), rem = tile_cur - n * p.TRC;
        ty = fdiv(rem, p.d_TC);
        tx = rem - ty * p.TC;
        x00 = (n * p.IH + 2 * ty - p.ph) * row_elems + (2 * tx - p.pw) * p.IC + ic0 + sc;
        y00 = ((n * p.OH + 2 * ty) * p.OW + 2 * tx) * p.OC + oc0 + 2 * sc;
    }
    auto advance_tile = [&]() {
        tile_cur += WD_TK;
        tx += p.adv_tx;
        ty += p.adv_ty;
        x00 += p.dx0;
        y00 += p.dy0;
        const bool w1 = tx >= p.TC;
        tx -= w1 ? p.TC : 0;
        ty += w1 ? 1 : 0;
        x00 += w1 ? p.wx1 : 0;
        y00 += w1 ? p.wy1 : 0;
        const bool w2 = ty >= p.TR;
        ty -= w2 ? p.TR : 0;
        x00 += w2 ? p.wx2 : 0;
        y00 += w2 ? p.wy2 : 0;
    };
    unsigned xo[4][4], yo[2][2], rowterm[4], colterm[4];
    auto x_terms = [&]() {
        const bool ok = tile_cur < tile_end && xc_ok;
        const int ih0 = 2 * ty - p.ph, iw0 = 2 * tx - p.pw;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const unsigned rv = (unsigned)x00 * 4u + (unsigned)(i * row_elems) * 4u, cv = (unsigned)(i * p.IC) * 4u;   // i-th terms are uniform
            rowterm[i] = (ok && (unsigned)(ih0 + i) < (unsigned)p.IH) ? rv : WD_OOR;
            colterm[i] = ((unsigned)(iw0 + i) < (unsigned)p.IW) ? cv : WD_OOR_COL;
        }
    };
    auto x_offsets = [&](int i) {
#pragma unroll
        for (int j = 0; j < 4; j++) xo[i][j] = rowterm[i] + colterm[j];
    };
    const int y_px = p.OC, y_row = p.OW * p.OC;
    auto y_offsets = [&]() {   // everything computed, then selected: no divergent branches among the MFMAs
        const bool ok = tile_cur < tile_end && yc_ok;
        const bool right = 2 * tx + 1 < p.OW, below = 2 * ty + 1 < p.OH;
        const unsigned o = (unsigned)y00 * 4u;
        yo[0][0] = ok ? o : WD_OOR;
        yo[0][1] = (ok && right) ? o + (unsigned)y_px * 4u : WD_OOR;
        yo[1][0] = (ok && below) ? o + (unsigned)y_row * 4u : WD_OOR;
        yo[1][1] = (ok && right && below) ? o + (unsigned)(y_row + y_px) * 4u : WD_OOR;
    };
    float xr[2][4][4];     // raw patches: set s holds a chunk of parity s, requested two chunks before it is transformed
    float2 yr[2][2][2];    // raw deltaY tiles
    auto load_one = [&](auto set_c, int e) {   // e < 16: patch element e; 16..19: deltaY element e - 16
        constexpr int SET = decltype(set_c)::value;
        if (e < 16) xr[SET][e >> 2][e & 3] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(x_rsrc, xo[e >> 2][e & 3], 0, 0));
        else yr[SET][(e - 16) >> 1][(e - 16) & 1] = __builtin_bit_cast(float2, __builtin_amdgcn_raw_buffer_load_b64(y_rsrc, yo[(e - 16) >> 1][(e - 16) & 1], 0, 0));
    };
    // Xh = B^T x B; Yh' = G' y G'^T with G' = [[1,0],[1,1],[1,-1],[0,1]] = G without its factors 1/2, which are applied to
    // the accumulators once, at the end
    float xrow[4][4];
    float2 yg[4][2];
    auto x_rows = [&](auto set_c) {
        constexpr int SET = decltype(set_c)::value;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            xrow[0][j] = xr[SET][0][j] - xr[SET][2][j];
            xrow[1][j] = xr[SET][1][j] + xr[SET][2][j];
            xrow[2][j] = xr[SET][2][j] - xr[SET][1][j];
            xrow[3][j] = xr[SET][3][j] - xr[SET][1][j];
        }
    };
    auto x_store = [&](float *Xh, int i) {   // xi = 4i .. 4i+3: group i of this (tile, channel)
        const floatx4 v = floatx4{xrow[i][0] - xrow[i][2], xrow[i][1] + xrow[i][2], xrow[i][2] - xrow[i][1], xrow[i][3] - xrow[i][1]};
        *reinterpret_cast<floatx4 *>(Xh + ((i ^ swz_w) << 2)) = v;
    };
    auto add2 = [](float2 a, float2 c) { return make_float2(a.x + c.x, a.y + c.y); };
    auto sub2 = [](float2 a, float2 c) { return make_float2(a.x - c.x, a.y - c.y); };
    auto y_rows = [&](auto set_c) {
        constexpr int SET = decltype(set_c)::value;
#pragma unroll
        for (int b = 0; b < 2; b++) {
            yg[0][b] = yr[SET][0][b];
            yg[1][b] = add2(yr[SET][0][b], yr[SET][1][b]);
            yg[2][b] = sub2(yr[SET][0][b], yr[SET][1][b]);
            yg[3][b] = yr[SET][1][b];
        }
    };
    auto y_store = [&](float *Yh, int a) {   // xi = 4a .. 4a+3 of the thread's two channels
        const float2 v1 = add2(yg[a][0], yg[a][1]), v2 = sub2(yg[a][0], yg[a][1]);
        *reinterpret_cast<floatx4 *>(Yh + ((a ^ swz_wy) << 2)) = floatx4{yg[a][0].x, v1.x, v2.x, yg[a][1].x};
        *reinterpret_cast<floatx4 *>(Yh + 16 + ((a ^ swz_wy) << 2)) = floatx4{yg[a][0].y, v1.y, v2.y, yg[a][1].y};
    };
    const int xh_write = (st * 32 + sc) * 16, yh_write = WD_XBUF + (st * 64 + 2 * sc) * 16;

    // Wavefronts 0-3 multiply, wavefronts 4-7 stage: each SIMD holds one of either kind, so the staging instructions
    // (loads, transforms, LDS writes: about 150 per chunk) fill the issue slots between the other wavefront's MFMAs without
    // any of them sharing registers with the 128 accumulators. One barrier per chunk joins them: while chunk c is
    // multiplied out of LDS buffer c & 1, chunk c+1 (requested from memory a chunk earlier) is transformed and written to
    // the other buffer and chunk c+2 is requested.
    typedef std::integral_constant<int, 0> Set0;
    typedef std::integral_constant<int, 1> Set1;
    if (t >= 256) {
        if (nchunks > 0) {
            auto request = [&](auto set_c) {   // the 20 loads of the chunk the tile cursor stands on
                x_terms();
#pragma unroll
                for (int i = 0; i < 4; i++) x_offsets(i);
                y_offsets();
#pragma unroll
                for (int e = 0; e < 20; e++) load_one(set_c, e);   // past the slice: out of range, zeros
            };
            auto transform = [&](auto set_c, int buf, bool store) {
                x_rows(set_c);
                y_rows(set_c);
                if (store) {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        x_store(smem + buf * WD_BUF + xh_write, i);
                        y_store(smem + buf * WD_BUF + yh_write, i);
                    }
                }
            };
            request(Set0{});
            transform(Set0{}, 0, true);   // chunk 0, waited for
            advance_tile();
            request(Set1{});              // chunk 1
            advance_tile();
            request(Set0{});              // chunk 2
            __syncthreads();
            // chunk c: chunk c+1 (requested two chunks ago) is transformed into the other buffer, chunk c+3 requested into
            // the set it leaves. Two chunks per round so that the sets are fixed registers; the loads of the second half
            // are issued even when that chunk does not exist (only its LDS writes and its barrier are skipped).
            for (int c = 0; c < nchunks; c += 2) {
                transform(Set1{}, 1, true);
                advance_tile();
                request(Set1{});
                __syncthreads();
                const bool more = c + 1 < nchunks;
                transform(Set0{}, 0, more);
                advance_tile();
                request(Set0{});
                if (more) __syncthreads();
            }
        }
        return;
    }

    if (nchunks > 0) {
        // One chunk = 8 groups of 8 MFMAs: (4 tiles kk, 4 xi) x (two blocks of input channels); three 128-bit LDS reads per
        // group, one group ahead. The two MFMAs into one accumulator (kk = 0, 1) are 4 groups apart.
        const int swz_r = (l16 >> 2) & 3;
        int rdx[4], rdy[4];   // float offsets of this lane's operands for xi group gx (tile q, channel l16 / 16w + l16)
#pragma unroll
        for (int gx = 0; gx < 4; gx++) {
            rdx[gx] = (q * 32 + l16) * 16 + ((gx ^ swz_r) << 2);
            rdy[gx] = WD_XBUF + (q * 64 + 16 * w + l16) * 16 + ((gx ^ swz_r) << 2);
        }
        __syncthreads();
        for (int c = 0; c < nchunks; c++) {
            const float *B = smem + (c & 1) * WD_BUF;
            auto frag = [&](int g, floatx4 &fa, floatx4 &fb0, floatx4 &fb1) {
                const int kk = g >> 2, gx = g & 3;
                fa = *reinterpret_cast<const floatx4 *>(B + rdy[gx] + kk * 4 * 64 * 16);
                fb0 = *reinterpret_cast<const floatx4 *>(B + rdx[gx] + kk * 4 * 32 * 16);
                fb1 = *reinterpret_cast<const floatx4 *>(B + rdx[gx] + kk * 4 * 32 * 16 + 16 * 16);
            };
            floatx4 a[2], b0[2], b1[2];
            frag(0, a[0], b0[0], b1[0]);
#pragma unroll
            for (int g = 0; g < 8; g++) {
                if (g + 1 < 8) frag(g + 1, a[(g + 1) & 1], b0[(g + 1) & 1], b1[(g + 1) & 1]);
#pragma unroll
                for (int x = 0; x < 4; x++) {
                    const int xi = 4 * (g & 3) + x;
                    acc[xi][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g & 1][x], b0[g & 1][x], acc[xi][0], 0, 0, 0);
                    acc[xi][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g & 1][x], b1[g & 1][x], acc[xi][1], 0, 0, 0);
                }
            }
            __syncthreads();
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
    hipLaunchKernelGGL(kern, dim3((IC + 31) / 32, (OC + 63) / 64, GZ), dim3(512), lds, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
