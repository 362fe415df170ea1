// Winograd F(2x2, 3x3) forward convolution, fully fused (input transform -> 16 MFMA GEMMs -> output
// transform in one kernel), fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950. For FH = FW = 3, stride 1.
//
//   Y_tile = A^T [ sum_ic (G g G^T) .* (B^T d B) ] A      with 2x2 output tiles from 4x4 input patches.
//
// The reference ships no Winograd (its experiments are compiled out); this is an additional algorithm of this
// build behind the same forward entries, checked against the same CPU direct convolution.
//
// A workgroup (4 wavefronts) owns 32 consecutive tiles of the flattened (n, tile row, tile column) index
// (= 128 output pixels) and 64 output channels; wavefront w owns output channels [16w, 16w+16) for all 16
// transform positions xi, i.e. 16 x 2 accumulator tiles. Because a lane then holds all 16 xi values of
// its (tile, channel) pairs, the output transform is pure per-lane register arithmetic.
// Input channels advance in chunks of 16: every thread loads the 4x4 patch of one (tile, channel pair) of the
// next chunk from global memory before the MFMAs of the current chunk, transforms it afterwards and writes
// V[xi][tile][16 channels] into the other LDS buffer. A fragment = one conflict-free 128-bit LDS read (a 16-lane
// group reads 16 tiles x 64 contiguous bytes); the transformed-filter fragment U[xi][ic][oc] comes straight from
// L2 four xi ahead.
#include "common.hpp"

namespace alpha {

struct WinoArgs {
    const float *X;   // [N, IH, IW, IC]
    const float *U;   // [16][IC][OC] transformed filter
    float *Y;         // [N, OH, OW, OC]
    Epilogue ep;         // applied as the rows leave for memory
    int N, IH, IW, IC, OH, OW, OC;
    int ph, pw;
    int TR, TC;       // tile rows / columns per image: ceil(OH/2), ceil(OW/2)
    int ntiles;       // N*TR*TC
    int x_bytes;      // size of X in bytes (< 2 GB)
    FastDiv d_TC, d_TRC;
};

constexpr int WG_TILES = 32;
constexpr int WG_VBUF = 16 * WG_TILES * 16;   // floats per V buffer: [xi][tile][16 channels]

// U[xi = 4a + b](ic, oc) = (G g G^T)[a][b],  G = [[1,0,0],[.5,.5,.5],[.5,-.5,.5],[0,0,1]],  g = W[oc][.][.][ic].
// Two layouts, chosen by IC alone so that the transform and the kernel that reads it agree: U[xi][ic][oc] for the kernel
// below, and for IC % 16 == 0 (winograd_stream.hip) U[xi][ic / 4][oc][ic % 4], where the four input channels of an
// MFMA operand are one 128-bit element.
// With `backward` the transform is that of the filter of backward-data seen as a forward convolution of deltaY: reduced
// channels = the layer's OC, produced channels = the layer's IC, taps rotated by 180 degrees,
// g'[i][j](reduced oc, produced ic) = W[oc][2-i][2-j][ic]. IC and OC below are then the reduced and the produced count
// (the layer's OC and IC), LD the layer's IC (the stride of W's taps).
__global__ __launch_bounds__(256) void winograd_filter_kernel(const float *__restrict__ W, float *__restrict__ U, int IC, int OC, int grouped,
                                                              int backward)
{
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= IC * OC) return;
    int ic, oc, pos, xi_stride = IC * OC, step;   // element (xi, ic, oc) at U[xi * xi_stride + pos]
    if (grouped) {   // threads over (ic / 4, oc, ic % 4), ic % 4 fastest: consecutive threads write consecutive elements
        const int g = idx / (4 * OC), r = idx - g * 4 * OC;
        oc = r >> 2;
        ic = 4 * g + (r & 3);
        pos = idx;
    } else {         // threads over (ic, oc), oc fastest
        ic = idx / OC;
        oc = idx - ic * OC;
        pos = idx;
    }
    step = xi_stride;
    float g[3][3];
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < 3; j++)
            g[i][j] = backward ? W[((size_t)(ic * 3 + (2 - i)) * 3 + (2 - j)) * OC + oc] : W[((size_t)(oc * 3 + i) * 3 + j) * IC + ic];
    float t[4][3];
#pragma unroll
    for (int j = 0; j < 3; j++) {
        t[0][j] = g[0][j];
        t[1][j] = 0.5f * (g[0][j] + g[1][j] + g[2][j]);
        t[2][j] = 0.5f * (g[0][j] - g[1][j] + g[2][j]);
        t[3][j] = g[2][j];
    }
#pragma unroll
    for (int a = 0; a < 4; a++) {
        const float u0 = t[a][0], u1 = 0.5f * (t[a][0] + t[a][1] + t[a][2]), u2 = 0.5f * (t[a][0] - t[a][1] + t[a][2]), u3 = t[a][2];
        U[(size_t)(4 * a + 0) * step + pos] = u0;
        U[(size_t)(4 * a + 1) * step + pos] = u1;
        U[(size_t)(4 * a + 2) * step + pos] = u2;
        U[(size_t)(4 * a + 3) * step + pos] = u3;
    }
}

__global__ __launch_bounds__(256, 2) void winograd_f2x2_kernel(const WinoArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float smem[];   // V[2][WG_VBUF]; reused as output staging [128 px][68]

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int tile0 = blockIdx.x * WG_TILES;
    const int oc0 = blockIdx.y * 64;
    const int TC = p.TC, TRC = p.d_TRC.d;

    floatx4 acc[16][2];
#pragma unroll
    for (int x = 0; x < 16; x++) {
        acc[x][0] = floatx4{0.f, 0.f, 0.f, 0.f};
        acc[x][1] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // ---- input transform: thread t -> (tile t/8, channel pair t%8 of the 16-channel chunk); 16 float2 loads ----------
    const int xt = t >> 3, xq = (t & 7) * 2;
    int x_base = 0, x_ih0 = -(1 << 28), x_iw0 = 0;
    {
        const int tile = tile0 + xt;
        if (tile < p.ntiles) {
            const int n = fdiv(tile, p.d_TRC), rem = tile - n * TRC;
            const int ty = fdiv(rem, p.d_TC), tx = rem - ty * TC;
            x_base = n * p.IH * p.IW * p.IC;
            x_ih0 = 2 * ty - p.ph;
            x_iw0 = 2 * tx - p.pw;
        }
    }
    // Loads go through buffer descriptors: address = descriptor base + uniform offset (scalar register: the chunk's
    // first channel) + per-lane 32-bit offset (fixed for the whole kernel), and an offset beyond the descriptor's size
    // returns 0. A thread loads the same 16 pixels of its tile for every channel chunk, so the per-lane offsets are
    // computed once, pixels outside the image get an offset that is out of range (their zeros come from the range
    // check), and a load costs no vector arithmetic. (Computing a 64-bit address per load took ~5 vector instructions
    // for each of the 80 loads of a chunk - more issue slots than the chunk's 128 MFMAs.)
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.X), 0, p.x_bytes, 0x00020000);
    constexpr unsigned OUT_OF_RANGE = 0x80000000u;   // descriptors are below 2 GB (host-checked)
    float2 d[4][4];
    unsigned p_off[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int ih = x_ih0 + i, iw = x_iw0 + j;
            const bool ok = (unsigned)ih < (unsigned)p.IH && (unsigned)iw < (unsigned)p.IW;
            p_off[i][j] = ok ? (unsigned)(x_base + (ih * p.IW + iw) * p.IC + xq) * 4u : OUT_OF_RANGE;
        }
    auto load_patch = [&](int icc) {   // icc: first channel of the 16-channel chunk
        // IC % 4 == 0: a channel pair is valid as a whole; only the last chunk of a ragged IC has invalid pairs
        const bool cv = icc + xq < p.IC;
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const unsigned off = (icc + 16 <= p.IC || cv) ? p_off[i][j] : OUT_OF_RANGE;
                d[i][j] = __builtin_bit_cast(float2, __builtin_amdgcn_raw_buffer_load_b64(x_rsrc, off, icc * 4, 0));
            }
    };
    auto transform_store = [&](int buf) {   // V = B^T d B, B^T = [[1,0,-1,0],[0,1,1,0],[0,-1,1,0],[0,1,0,-1]]
        float *V = smem + buf * WG_VBUF + xt * 16 + xq;
        auto sub = [](float2 a, float2 b) { return make_float2(a.x - b.x, a.y - b.y); };
        auto add = [](float2 a, float2 b) { return make_float2(a.x + b.x, a.y + b.y); };
        float2 r[4][4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            r[0][j] = sub(d[0][j], d[2][j]);
            r[1][j] = add(d[1][j], d[2][j]);
            r[2][j] = sub(d[2][j], d[1][j]);
            r[3][j] = sub(d[1][j], d[3][j]);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float2 v0 = sub(r[i][0], r[i][2]), v1 = add(r[i][1], r[i][2]), v2 = sub(r[i][2], r[i][1]), v3 = sub(r[i][1], r[i][3]);
            *reinterpret_cast<float2 *>(V + (4 * i + 0) * WG_TILES * 16) = v0;
            *reinterpret_cast<float2 *>(V + (4 * i + 1) * WG_TILES * 16) = v1;
            *reinterpret_cast<float2 *>(V + (4 * i + 2) * WG_TILES * 16) = v2;
            *reinterpret_cast<float2 *>(V + (4 * i + 3) * WG_TILES * 16) = v3;
        }
    };

    // ---- transformed-filter fragments from L2: lane (l16, q) needs U[xi][icc + 4q + s][oc0 + 16w + l16] ------------
    const int b_co = oc0 + 16 * w + l16;
    const int b_col = b_co < p.OC ? b_co : 0;   // columns beyond OC are never stored
    const int xi_stride = p.IC * p.OC;
    const __amdgpu_buffer_rsrc_t u_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.U), 0, 16 * xi_stride * 4, 0x00020000);
    unsigned u_lane[4];   // byte offset of this lane's elements inside a (frequency, 16-channel chunk) block of U
#pragma unroll
    for (int s = 0; s < 4; s++) u_lane[s] = (unsigned)((4 * q + s) * p.OC + b_col) * 4u;
    auto load_b = [&](float (&b)[4], int xi, int icc) {
        // channels beyond IC (last chunk of a ragged IC) read the next frequency's block or, at the very end, get the
        // range check's zero; the fragment is zeroed where it is used
        const int block = (xi * xi_stride + icc * p.OC) * 4;   // uniform
#pragma unroll
        for (int s = 0; s < 4; s++) b[s] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(u_rsrc, u_lane[s], block, 0));
    };

    const int nchunks = (p.IC + 15) >> 4;
    load_patch(0);
    transform_store(0);
    float bring[4][4];
#pragma unroll
    for (int x = 0; x < 4; x++) load_b(bring[x], x, 0);
    __syncthreads();

    for (int c = 0; c < nchunks; c++) {
        const int buf = c & 1;
        const bool more = c + 1 < nchunks;
        if (more) load_patch((c + 1) * 16);
        __builtin_amdgcn_sched_barrier(0);

        const float *V = smem + buf * WG_VBUF + l16 * 16 + 4 * q;
#pragma unroll
        for (int xi = 0; xi < 16; xi++) {
            const floatx4 a0 = *reinterpret_cast<const floatx4 *>(V + xi * WG_TILES * 16);
            const floatx4 a1 = *reinterpret_cast<const floatx4 *>(V + xi * WG_TILES * 16 + 16 * 16);
            float b[4];
#pragma unroll
            for (int s = 0; s < 4; s++) b[s] = bring[xi & 3][s];
            // refill this ring slot with the fragment needed four positions later (possibly in the next chunk)
            {
                const int nx = xi + 4;
                const int nxi = nx & 15, nicc = (nx < 16 ? c : c + 1) * 16;
                load_b(bring[xi & 3], nxi, nicc < p.IC ? nicc : 0);
            }
            if (c * 16 + 4 * q >= p.IC) {
#pragma unroll
                for (int s = 0; s < 4; s++) b[s] = 0.f;   // ragged last chunk: channels beyond IC
            }
#pragma unroll
            for (int s = 0; s < 4; s++) {
                acc[xi][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[s], b[s], acc[xi][0], 0, 0, 0);
                acc[xi][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[s], b[s], acc[xi][1], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (more) transform_store(buf ^ 1);
        __syncthreads();
    }

    // ---- output transform in registers: Y = A^T M A, A^T = [[1,1,1,0],[0,1,-1,-1]]; then LDS-staged store ---------
    float *Os = smem;   // [128 pixels: tile*4 + 2*dy + dx][68]
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float m[4][4];
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int b = 0; b < 4; b++) m[a][b] = acc[4 * a + b][mt][r];
            float s0[4], s1[4];
#pragma unroll
            for (int b = 0; b < 4; b++) {
                s0[b] = m[0][b] + m[1][b] + m[2][b];
                s1[b] = m[1][b] - m[2][b] - m[3][b];
            }
            const int tl = 16 * mt + 4 * q + r;   // tile within the workgroup
            float *o = Os + (tl * 4) * 68 + 16 * w + l16;
            o[0 * 68] = s0[0] + s0[1] + s0[2];
            o[1 * 68] = s0[1] - s0[2] - s0[3];
            o[2 * 68] = s1[0] + s1[1] + s1[2];
            o[3 * 68] = s1[1] - s1[2] - s1[3];
        }
    __syncthreads();
    for (int idx = t; idx < WG_TILES * 4 * 16; idx += 256) {
        const int px = idx >> 4, cq = (idx & 15) * 4;
        const int tl = px >> 2, dy = (px >> 1) & 1, dx = px & 1;
        const int tile = tile0 + tl;
        if (tile < p.ntiles && oc0 + cq < p.OC) {
            const int n = fdiv(tile, p.d_TRC), rem = tile - n * TRC;
            const int ty = fdiv(rem, p.d_TC), tx = rem - ty * TC;
            const int oh = 2 * ty + dy, ow = 2 * tx + dx;
            if (oh < p.OH && ow < p.OW) {
                const size_t elem = (((size_t)n * p.OH + oh) * p.OW + ow) * p.OC + oc0 + cq;
                *reinterpret_cast<float4 *>(p.Y + elem) = epilogue4(*reinterpret_cast<const float4 *>(Os + px * 68 + cq), p.ep, oc0 + cq, elem);
            }
        }
    }
}

hipError_t launch_winograd_filter(hipStream_t s, const float *W, float *U, int IC, int OC, bool backward)
{
    if (IC <= 0 || OC <= 0) return hipSuccess;
    const int red = backward ? OC : IC, prod = backward ? IC : OC;   // reduced and produced channels of the convolution that reads U
    hipLaunchKernelGGL(winograd_filter_kernel, dim3((IC * OC + 255) / 256), dim3(256), 0, s, W, U, red, prod,
                       winograd_grouped_filter(red) ? 1 : 0, backward ? 1 : 0);
    return hipGetLastError();
}

hipError_t launch_winograd(hipStream_t stream, const float *X, const float *U, float *Y,
                           int N, int IH, int IW, int IC, int OH, int OW, int OC, int ph, int pw, const float *bias, const Epilogue *ep)
{
    if (OH != IH + 2 * ph - 2 || OW != IW + 2 * pw - 2) return hipErrorNotSupported;
    if (!winograd_forward_fits(N, IH, IW, IC, OH, OW, OC)) return hipErrorNotSupported;
    if (winograd_grouped_filter(IC)) {   // the persistent variant and its filter layout; no other kernel reads that layout
        if (ep == nullptr || !ep->fused) return launch_winograd_stream(stream, X, U, Y, N, IH, IW, IC, OH, OW, OC, ph, pw, ep ? ep->bias : bias);
        // that kernel adds a bias only: the rest of the epilogue is one more pass over Y
        if (hipError_t e = launch_winograd_stream(stream, X, U, Y, N, IH, IW, IC, OH, OW, OC, ph, pw, nullptr); e != hipSuccess) return e;
        return launch_epilogue_rows(stream, Y, Y, *ep, (long)N * OH * OW * OC, OC, OC);
    }
    WinoArgs a{};
    a.X = X; a.U = U; a.Y = Y; a.ep = ep ? *ep : bias_epilogue(bias);
    a.N = N; a.IH = IH; a.IW = IW; a.IC = IC; a.OH = OH; a.OW = OW; a.OC = OC;
    a.ph = ph; a.pw = pw;
    a.TR = (OH + 1) / 2; a.TC = (OW + 1) / 2;
    const long nt = (long)N * a.TR * a.TC;
    if (nt >= (1L << 30) || 16L * IC * OC * 4 >= (1L << 31) || (long)N * IH * IW * IC * 4 >= (1L << 31)) return hipErrorNotSupported;   // buffer descriptors below 2 GB
    a.x_bytes = (int)((long)N * IH * IW * IC * 4);
    a.ntiles = (int)nt;
    a.d_TC = make_fastdiv(a.TC);
    a.d_TRC = make_fastdiv(a.TR * a.TC);
    size_t lds = (size_t)2 * WG_VBUF * sizeof(float);
    const size_t stage = (size_t)WG_TILES * 4 * 68 * sizeof(float);
    if (lds < stage) lds = stage;
    if (hipError_t e = ensure_dynamic_lds<winograd_f2x2_kernel>(lds); e != hipSuccess) return e;
    dim3 grid((a.ntiles + WG_TILES - 1) / WG_TILES, (OC + 63) / 64);
    hipLaunchKernelGGL(winograd_f2x2_kernel, grid, dim3(256), lds, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
