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
// A workgroup owns one slice, 64 output channels and 32 input channels, and has eight wavefronts, two per SIMD: one that
// multiplies and one that stages. Multiplying wavefront w accumulates output channels [16w, 16w+16) x 32 input channels x
// 16 xi = 128 registers; tiles advance in chunks of 8. A staging thread loads the 4x4 patch of one (tile, input channel)
// two chunks before it is transformed and writes Xh[tile][channel][16 xi] into the LDS buffer that is multiplied in the
// chunk after; one barrier per chunk joins the two kinds (wavefronts of one kind doing both jobs needed scheduling
// directives, spilled, or moved the accumulators through AGPRs). deltaY does not pass through LDS: a multiplying wavefront
// is the only user of its 16 output channels, so its lanes load their own 2x2 tiles and transform them in registers into
// MFMA operands.
// What a chunk costs beyond its 64 MFMAs per SIMD is the number of vector instructions the SIMD issues beside them (each
// takes 5-9 cycles out of the MFMA stream, whichever wavefront issues it). The transforms need 56 per SIMD and chunk;
// where tiles are and which of their pixels exist must not add to that. One wavefront therefore computes, once per 64
// tiles, a table in LDS with each tile's load offsets - four row terms and four column terms of its patch, the four
// pixels of its deltaY tile, "outside" encoded as an offset beyond the descriptor - and every other thread gets the
// offsets of its tile with two or three 128-bit LDS reads and adds its channel (tile cursors kept per thread and advanced by
// additions cost 24-67 vector instructions per wavefront and chunk; the staging work on two of the four SIMDs made
// those two 3.7 k cycles per chunk against 2.05 k of MFMAs). Measured and not kept: a staging thread per (tile, four
// channels) with 128-bit loads, one wavefront per chunk, each chunk spread over four chunk periods so that every SIMD
// has a quarter of one chunk's staging per period (fewer instructions in total, but 10 % slower: a request then has one
// period to arrive instead of two).
// In LDS the 16 xi of a (tile, channel) are contiguous, so a lane's patch operand for four xi is one 128-bit read (an
// operand per xi as a 32-bit read - three LDS instructions per two MFMAs - cost 30 cycles per pair of MFMAs). A (tile,
// channel) takes 80 bytes and a tile 32 x 80 + 256: the 32 lanes of a staging write (32 channels of a tile) and the 32
// lanes of a half wavefront's read (16 channels of two tiles) then touch 32 different 16-byte bank groups.
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
    int x_bytes, y_bytes;   // X below 1 GB (512 MB when IC % 32 != 0), deltaY below 2 GB (1 GB when OC % 64 != 0)
    FastDiv d_TC, d_TRC;
};

constexpr int WD_TK = 8;                        // tiles per chunk
constexpr int WD_CS = 20;                       // floats per (tile, channel): 16 xi + 4
constexpr int WD_TS = 32 * WD_CS + 64;          // floats per tile: 176 16-byte groups = 16 (mod 32), see the layout note above
constexpr int WD_BUF = WD_TK * WD_TS;           // Xh[tile][32 input channels][16 xi + 4]: one LDS buffer
constexpr int WD_TG = 64;                       // tiles per group of the offset table (8 chunks)
constexpr unsigned WD_OOR = 0x80000000u;        // row term / deltaY pixel outside: beyond both descriptors, the load returns 0
constexpr unsigned WD_OOR_COL = 0x40000000u;    // column term outside (X ends below 1 GB)
constexpr unsigned WD_OOR_XCH = 0x20000000u;    // input channel past the end (X ends below 512 MB when IC % 32 != 0)
constexpr unsigned WD_OOR_YCH = 0x40000000u;    // output channel past the end (deltaY ends below 1 GB when OC % 64 != 0)
// no sum of these with valid terms wraps around 2^32: 0x80000000 + 0x40000000 + 0x20000000 + (valid terms < 0x20000000)

__global__ __launch_bounds__(512) void winograd_dw_kernel(const WinoDwArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float wd_smem[];   // Xh[2][WD_BUF], XT[2][64][8], YT[2][64][4]
    float *smem = wd_smem;
    unsigned *XT = reinterpret_cast<unsigned *>(wd_smem + 2 * WD_BUF);
    unsigned *YT = XT + 2 * WD_TG * 8;

    const int t = threadIdx.x;
    const int lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
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

    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.X), 0, p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.dY), 0, p.y_bytes, 0x00020000);
    typedef std::integral_constant<int, 0> Set0;
    typedef std::integral_constant<int, 1> Set1;
    typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

    // Offsets of the 64 tiles of group g of the slice (lane = tile), into table slot g & 1. Patch of tile (n, ty, tx): rows
    // 2ty - ph + i, columns 2tx - pw + j; a load's byte offset is row term i + column term j + 4 * channel.
    auto table = [&](int g) {
        const int tile = tile_begin + g * WD_TG + lane;
        const bool ok = tile < tile_end;
        const int tl = ok ? tile : tile_begin;
        const int n = fdiv(tl, p.d_TRC), rem = tl - n * p.TRC;
        const int ty = fdiv(rem, p.d_TC), tx = rem - ty * p.TC;
        const int ih0 = 2 * ty - p.ph, iw0 = 2 * tx - p.pw;
        const int row_elems = p.IW * p.IC;
        const unsigned x00 = (unsigned)(((n * p.IH + ih0) * p.IW + iw0) * p.IC) * 4u;   // may stand before the tensor
        uintx4 rt, ct, yo;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            rt[i] = (ok && (unsigned)(ih0 + i) < (unsigned)p.IH) ? x00 + (unsigned)(i * row_elems) * 4u : WD_OOR;
            ct[i] = ((unsigned)(iw0 + i) < (unsigned)p.IW) ? (unsigned)(i * p.IC) * 4u : WD_OOR_COL;
        }
        const unsigned y00 = (unsigned)(((n * p.OH + 2 * ty) * p.OW + 2 * tx) * p.OC) * 4u;
        const bool right = 2 * tx + 1 < p.OW, below = 2 * ty + 1 < p.OH;
        yo[0] = ok ? y00 : WD_OOR;
        yo[1] = (ok && right) ? y00 + (unsigned)p.OC * 4u : WD_OOR;
        yo[2] = (ok && below) ? y00 + (unsigned)(p.OW * p.OC) * 4u : WD_OOR;
        yo[3] = (ok && right && below) ? y00 + (unsigned)((p.OW + 1) * p.OC) * 4u : WD_OOR;
        const int e = (g & 1) * WD_TG + lane;
        *reinterpret_cast<uintx4 *>(XT + e * 8) = rt;
        *reinterpret_cast<uintx4 *>(XT + e * 8 + 4) = ct;
        *reinterpret_cast<uintx4 *>(YT + e * 4) = yo;
    };
    if (t >= 256) {
        if (nchunks == 0) return;   // an empty slice: the multiplying wavefronts write its zeros
        // ---- wavefronts 4-7 stage the patches: a thread takes (tile, input channel) - 16 loads two chunks ahead, B^T x B,
        //      four 128-bit LDS writes into the buffer that is multiplied in the next chunk --------------------------------
        if (w == 4) table(0);
        __syncthreads();
        const int item = t - 256, st = item >> 5, x_ch = item & 31;
        const unsigned ch4 = ic0 + x_ch < p.IC ? (unsigned)(ic0 + x_ch) * 4u : WD_OOR_XCH;
        float xr[2][4][4];   // raw patches: set s holds a chunk of parity s, requested two chunks before it is transformed
        auto request = [&](auto set_c, int chunk) {
            constexpr int SET = decltype(set_c)::value;
            const int tt = chunk * WD_TK + st;
            const unsigned *e = XT + (((tt >> 6) & 1) * WD_TG + (tt & 63)) * 8;
            const uintx4 rt = *reinterpret_cast<const uintx4 *>(e);
            uintx4 ct = *reinterpret_cast<const uintx4 *>(e + 4);
            ct += ch4;
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    xr[SET][i][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(x_rsrc, rt[i] + ct[j], 0, 0));
        };
        // Xh = B^T x B; the 4 xi of a row are one 128-bit element of the (tile, channel)
        auto transform = [&](auto set_c, int buf, bool store) {
            constexpr int SET = decltype(set_c)::value;
            float *Xh = smem + buf * WD_BUF + st * WD_TS + x_ch * WD_CS;
            float r[4][4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float x0 = xr[SET][0][j], x1 = xr[SET][1][j], x2 = xr[SET][2][j], x3 = xr[SET][3][j];
                r[0][j] = x0 - x2;
                r[1][j] = x1 + x2;
                r[2][j] = x2 - x1;
                r[3][j] = x3 - x1;
            }
            if (store) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    *reinterpret_cast<floatx4 *>(Xh + (i << 2)) =
                        floatx4{r[i][0] - r[i][2], r[i][1] + r[i][2], r[i][2] - r[i][1], r[i][3] - r[i][1]};
            }
        };
        request(Set0{}, 0);
        transform(Set0{}, 0, true);   // chunk 0, waited for
        request(Set1{}, 1);
        request(Set0{}, 2);
        __syncthreads();
        // chunk c: chunk c+1 (requested two chunks ago) is transformed into the other buffer, chunk c+3 requested into the
        // set it leaves. Two chunks per round so that the sets are fixed registers; the loads of the second half are issued
        // even when that chunk does not exist (only its LDS writes and its barrier are skipped). Every eighth chunk the
        // first staging wavefront writes the table of the next 64 tiles.
        for (int c = 0; c < nchunks; c += 2) {
            if ((c & 7) == 0 && w == 4) table((c >> 3) + 1);
            transform(Set1{}, 1, true);
            request(Set1{}, c + 3);
            __syncthreads();
            const bool more = c + 1 < nchunks;
            transform(Set0{}, 0, more);
            request(Set0{}, c + 4);
            if (more) __syncthreads();
        }
        return;
    } else if (nchunks > 0) {
        // ---- wavefronts 0-3 multiply. Wavefront w is the only one that needs output channels [16w, 16w+16), so lane
        //      (l16, q) loads the 2x2 tiles of channel 16w + l16 for its two tiles of a chunk (q and 4 + q) itself, two
        //      chunks ahead, and transforms them in registers into the 32 MFMA operands of the chunk. The patches come
        //      from LDS. -------------------------------------------------------------------------------------------------
        __syncthreads();
        const int y_ch = oc0 + 16 * w + l16;
        const unsigned ych4 = y_ch < p.OC ? (unsigned)y_ch * 4u : WD_OOR_YCH;
        float yraw[2][2][4];   // [set][kk][pixel]
        auto request = [&](auto set_c, int chunk) {
            constexpr int SET = decltype(set_c)::value;
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                const int tt = chunk * WD_TK + 4 * kk + q;
                uintx4 o = *reinterpret_cast<const uintx4 *>(YT + (((tt >> 6) & 1) * WD_TG + (tt & 63)) * 4);
                o += ych4;
#pragma unroll
                for (int k = 0; k < 4; k++)
                    yraw[SET][kk][k] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(y_rsrc, o[k], 0, 0));
            }
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
        // this lane's patch operands: tile q (and 4 + q), channels l16 and 16 + l16, xi group gx
        const float *rd = smem + q * WD_TS + l16 * WD_CS;
        // One chunk = 8 groups of 8 MFMAs: (4 tiles kk, 4 xi) x (two blocks of input channels); two 128-bit LDS reads per
        // group, one group ahead. The two MFMAs into one accumulator (kk = 0, 1) are 4 groups apart.
        auto multiply = [&](int buf) {
            const float *B = rd + buf * WD_BUF;
            auto frag = [&](int g, floatx4 &fb0, floatx4 &fb1) {
                const int kk = g >> 2, gx = g & 3;
                fb0 = *reinterpret_cast<const floatx4 *>(B + kk * 4 * WD_TS + (gx << 2));
                fb1 = *reinterpret_cast<const floatx4 *>(B + kk * 4 * WD_TS + 16 * WD_CS + (gx << 2));
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
        request(Set0{}, 0);
        request(Set1{}, 1);
        __syncthreads();
        for (int c = 0; c < nchunks; c += 2) {
            transform(Set0{});
            request(Set0{}, c + 2);
            multiply(0);
            __syncthreads();
            const bool more = c + 1 < nchunks;
            transform(Set1{});
            request(Set1{}, c + 3);
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
    // the load offsets are sums of terms that mark "outside" by 2 GB (row, deltaY pixel), 1 GB (column, output channel) and
    // 512 MB (input channel): the tensors must end below the smallest mark that can meet a valid offset
    if (x_bytes + 16L * IC > ((IC & 31) ? (1L << 29) : (1L << 30))) return hipErrorNotSupported;
    if (y_bytes >= ((OC & 63) ? (1L << 30) : (1L << 31))) return hipErrorNotSupported;
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
    a.S = (int)(((nt + GZ - 1) / GZ + WD_TK - 1) / WD_TK * WD_TK);
    a.x_bytes = (int)x_bytes; a.y_bytes = (int)y_bytes;
    a.d_TC = make_fastdiv(a.TC);
    a.d_TRC = make_fastdiv(a.TRC);
    constexpr auto kern = winograd_dw_kernel;
    const size_t lds = (size_t)2 * WD_BUF * sizeof(float) + (size_t)2 * WD_TG * (8 + 4) * sizeof(unsigned);
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((IC + 31) / 32, (OC + 63) / 64, GZ), dim3(512), lds, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
