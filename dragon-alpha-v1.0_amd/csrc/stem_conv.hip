// Forward convolution of layers with at most 4 (stored) input channels - network stems such as 7x7 stride 2 on RGB -
// fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950.
//
// With IC = 4 an implicit GEMM over k = (fh, fw, ic) spends its time on address generation: every 16-byte load is a
// different filter tap. Here the reduction index of one MFMA is FOUR TAPS of one channel instead: lane (l16, q) reads
// the float4 (all 4 channels) of the input pixel that tap 4g + q touches for output pixel l16, and the float4 of
// filter tap 4g + q for output channel l16; component s of both feeds MFMA step s. One 128-bit LDS read per operand
// and tile therefore feeds 4 MFMAs covering 4 taps x 4 channels, with no im2col arithmetic at all (a lane's tap
// offsets are 13 registers computed once). Taps are padded to a multiple of 4 with zero weights (7x7: 49 -> 52).
//
// A workgroup (4 wavefronts) is persistent: it stages its 64 output channels of the filter in LDS once and then walks
// 16 x 16 blocks of output pixels; per block it stages the input window ((16-1)*sh + FH rows) once. Wavefront w owns
// output rows 4w .. 4w+3 of the block (4 tiles of 16 pixels) for all 64 channels. Results leave through a
// wavefront-private LDS patch as whole 256-byte pixel rows.
//
// LDS banks: the A reads of a half wavefront are pixels l16*sw + q (+ const), q in {0,1}: distinct 16-byte slots for
// sw = 2, the same address (broadcast) where they coincide for sw = 1. The filter is stored [tap][oc][4] with the oc
// index XORed by 16 for odd taps, which puts the two taps of a half wavefront into different halves of the banks.
#include "common.hpp"

namespace alpha {

typedef float floatx4 __attribute__((ext_vector_type(4)));

struct StemArgs {
    const float *X;   // [N][IH][IW][4]
    const float *F;   // f_cw ? CW[FH][FW][4][OC] : W[OC][FH][FW][4]
    float *Y;         // [N][OH][OW][OC]
    int N, IH, IW, OH, OW, OC;
    int FW, sh, sw, ph, pw;
    int f_cw;
    Epilogue ep;         // applied as the rows leave for memory
    int taps, groups;   // FH*FW and ceil(taps / 4)
    int IHB, IWB;       // input window of a block: 15*sh + FH rows, 15*sw + FW columns
    int blocks;         // N * bh_count * bw_count
    FastDiv d_bw, d_bhw, d_FW, d_IWB;
};

constexpr int ST_OS = 64 + 4;       // output staging row stride (floats)
constexpr int ST_MAXG = 13;         // tap groups supported (52 taps)
template <int V> struct StemChannels { static constexpr int value = V; };

__global__ __launch_bounds__(256, 2) void stem_conv_kernel(const StemArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *Ws = smem;                                  // [groups*4][64][4], oc index swizzled
    float *Xs = smem + p.groups * 4 * 64 * 4;          // [IHB][IWB][4]; reused as output staging [4][16][ST_OS]
    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int oc0 = blockIdx.y * 64;
    const int IWB = p.IWB, taps = p.taps;

    // ---- filter -> LDS, once. Layers with 3 logical channels arrive with the fourth stored channel zero-filled in X
    // and in the filter: when every weight of channel 3 in this workgroup's 64 output channels is zero, the MFMA step
    // of that channel (a quarter of all steps) is left out ------------------------------------------------------------
    int ch3 = 0;
    for (int idx = t; idx < p.groups * 4 * 64; idx += 256) {
        const int slot = idx >> 6, ocl = idx & 63, oc = oc0 + ocl;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (slot < taps && oc < p.OC) {
            if (!p.f_cw) {
                v = *reinterpret_cast<const float4 *>(p.F + ((size_t)oc * taps + slot) * 4);
            } else {
                const float *f = p.F + (size_t)slot * 4 * p.OC + oc;
                v = make_float4(f[0], f[p.OC], f[2 * p.OC], f[3 * p.OC]);
            }
        }
        ch3 |= v.w != 0.f;
        *reinterpret_cast<float4 *>(Ws + ((slot << 6) + (ocl ^ ((slot & 1) << 4))) * 4) = v;
    }
    const bool use_ch3 = __syncthreads_or(ch3) != 0;

    // ---- per-lane offsets (floats) ---------------------------------------------------------------------------------
    int toff[ST_MAXG];   // input offset of tap 4g + q relative to the output pixel's window origin
#pragma unroll
    for (int g = 0; g < ST_MAXG; g++) {
        const int tap = 4 * g + q;
        const int fh = fdiv(tap, p.d_FW), fw = tap - fh * p.FW;
        toff[g] = tap < taps ? (fh * IWB + fw) * 4 : 0;   // padding taps have zero weights: any valid address will do
    }
    int xbase[4], wl[4];
#pragma unroll
    for (int i = 0; i < 4; i++) xbase[i] = ((4 * w + i) * p.sh * IWB + l16 * p.sw) * 4;
#pragma unroll
    for (int j = 0; j < 4; j++) wl[j] = ((q << 6) + ((16 * j + l16) ^ ((q & 1) << 4))) * 4;
    float *Os = Xs + w * (16 * ST_OS);

    const int window_quads = p.IHB * IWB;
    // A thread stages the same window positions for every block: row, column and relative offset are computed once
    // (the first eight of them; a window of more than 2048 pixels takes the general path below).
    int st_r[8], st_c[8], st_off[8];
#pragma unroll
    for (int u = 0; u < 8; u++) {
        const int idx = min(t + 256 * u, window_quads - 1);
        st_r[u] = fdiv(idx, p.d_IWB);
        st_c[u] = idx - st_r[u] * IWB;
        st_off[u] = (st_r[u] * p.IW + st_c[u]) * 4;
    }
    // columns of the output block this lane stores: pixel 4*pp + q, channels oc0 + 4*l16 .. +3
    int out_off[4];
#pragma unroll
    for (int pp = 0; pp < 4; pp++) out_off[pp] = (4 * pp + q) * p.OC + oc0 + 4 * l16;
    const bool oc_ok = oc0 + 4 * l16 < p.OC;   // OC % 4 == 0: four channels valid together
    for (int blk = blockIdx.x; blk < p.blocks; blk += gridDim.x) {
        const int n = fdiv(blk, p.d_bhw), rem = blk - n * p.d_bhw.d;
        const int bh = fdiv(rem, p.d_bw), bw = rem - bh * p.d_bw.d;
        const int oh0 = bh * 16, ow0 = bw * 16;
        const int ih0 = oh0 * p.sh - p.ph, iw0 = ow0 * p.sw - p.pw;

        __syncthreads();   // filter staged (first block) / previous block's output patches drained
        // ---- input window -> LDS: 8 loads in flight per thread, zeros outside the image ------------------------------
        {
            float4 v[8];
            unsigned okmask = 0;
            const int blockbase = ((n * p.IH + ih0) * p.IW + iw0) * 4;   // uniform; may lie before the image
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const bool ok = t + 256 * u < window_quads && (unsigned)(ih0 + st_r[u]) < (unsigned)p.IH &&
                                (unsigned)(iw0 + st_c[u]) < (unsigned)p.IW;
                v[u] = *reinterpret_cast<const float4 *>(p.X + (ok ? blockbase + st_off[u] : 0));
                okmask |= (unsigned)ok << u;
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int idx = t + 256 * u;
                const bool ok = (okmask >> u) & 1u;
                if (idx < window_quads)
                    *reinterpret_cast<float4 *>(Xs + idx * 4) =
                        make_float4(ok ? v[u].x : 0.f, ok ? v[u].y : 0.f, ok ? v[u].z : 0.f, ok ? v[u].w : 0.f);
            }
        }
        for (int base = 256 * 8; base < window_quads; base += 256 * 8) {   // windows of more than 2048 pixels
            float4 v[8];
            unsigned okmask = 0;
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int idx = base + t + 256 * u;
                const int r = fdiv(idx, p.d_IWB), c = idx - r * IWB;
                const int ih = ih0 + r, iw = iw0 + c;
                const bool ok = idx < window_quads && (unsigned)ih < (unsigned)p.IH && (unsigned)iw < (unsigned)p.IW;
                const int off = (((n * p.IH + ih) * p.IW + iw) * 4) & -(int)ok;
                v[u] = *reinterpret_cast<const float4 *>(p.X + off);
                okmask |= (unsigned)ok << u;
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int idx = base + t + 256 * u;
                const bool ok = (okmask >> u) & 1u;
                if (idx < window_quads)
                    *reinterpret_cast<float4 *>(Xs + idx * 4) =
                        make_float4(ok ? v[u].x : 0.f, ok ? v[u].y : 0.f, ok ? v[u].z : 0.f, ok ? v[u].w : 0.f);
            }
        }
        __syncthreads();

        floatx4 acc[4][4];
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
        auto multiply = [&](auto sc) {
            constexpr int SC = decltype(sc)::value;   // channels multiplied: 4, or 3 when channel 3 has zero weights
#pragma unroll
            for (int g = 0; g < ST_MAXG; g++) {
                if (g < p.groups) {   // uniform
                    floatx4 a[4], b[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) a[i] = *reinterpret_cast<const floatx4 *>(Xs + xbase[i] + toff[g]);
#pragma unroll
                    for (int j = 0; j < 4; j++) b[j] = *reinterpret_cast<const floatx4 *>(Ws + wl[j] + g * (4 * 64 * 4));
#pragma unroll
                    for (int s = 0; s < SC; s++)
#pragma unroll
                        for (int i = 0; i < 4; i++)
#pragma unroll
                            for (int j = 0; j < 4; j++)
                                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i][s], b[j][s], acc[i][j], 0, 0, 0);
                }
            }
        };
        if (use_ch3) multiply(StemChannels<4>{});
        else multiply(StemChannels<3>{});
        __syncthreads();   // every wavefront is done with the window: its space becomes the output patches

        // ---- lane holds Y[oh0 + 4w + i][ow0 + 4q + r][oc0 + 16j + l16] ---------------------------------------------------
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int oh = oh0 + 4 * w + i;
            float *yrow = p.Y + ((size_t)(n * p.OH + oh) * p.OW + ow0) * p.OC;   // uniform
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) Os[(4 * q + r) * ST_OS + 16 * j + l16] = acc[i][j][r];
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int pp = 0; pp < 4; pp++) {
                const int col = 4 * pp + q, ow = ow0 + col;
                const float4 v = *reinterpret_cast<const float4 *>(Os + col * ST_OS + 4 * l16);
                if (oh < p.OH && ow < p.OW && oc_ok)
                    *reinterpret_cast<float4 *>(yrow + out_off[pp]) =
                        epilogue4(v, p.ep, oc0 + 4 * l16, (size_t)(yrow - p.Y) + out_off[pp]);
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

// Returns hipErrorNotSupported (nothing launched) unless IC (stored) is 4 and the filter has at most 52 taps.
hipError_t launch_stem_conv(hipStream_t stream, const float *X, const float *F, int f_cw, float *Y,
                            int N, int IH, int IW, int IC, int OH, int OW, int OC, int FH, int FW, int sh, int sw, int ph, int pw,
                            const float *bias, const Epilogue *ep)
{
    if (IC != 4 || FH * FW > 4 * ST_MAXG || OC < 4 || (OC & 3)) return hipErrorNotSupported;
    if ((size_t)N * IH * IW * 4 >= (1ull << 31) || (size_t)N * OH * OW * OC >= (1ull << 31)) return hipErrorNotSupported;
    StemArgs a{};
    a.X = X; a.F = F; a.Y = Y; a.f_cw = f_cw; a.ep = ep ? *ep : bias_epilogue(bias);
    a.N = N; a.IH = IH; a.IW = IW; a.OH = OH; a.OW = OW; a.OC = OC;
    a.FW = FW; a.sh = sh; a.sw = sw; a.ph = ph; a.pw = pw;
    a.taps = FH * FW;
    a.groups = (a.taps + 3) / 4;
    a.IHB = 15 * sh + FH;
    a.IWB = 15 * sw + FW;
    const int bh = (OH + 15) / 16, bw = (OW + 15) / 16;
    a.blocks = N * bh * bw;
    a.d_bw = make_fastdiv(bw);
    a.d_bhw = make_fastdiv(bh * bw);
    a.d_FW = make_fastdiv(FW);
    a.d_IWB = make_fastdiv(a.IWB);
    const size_t window = (size_t)a.IHB * a.IWB * 4, patches = 4 * 16 * ST_OS;
    const size_t lds = ((size_t)a.groups * 4 * 64 * 4 + (window > patches ? window : patches)) * sizeof(float);
    if (lds + 256 > 80 * 1024) return hipErrorNotSupported;   // two workgroups per compute unit (256 bytes: the block-wide OR)
    static int cu_count[64] = {0};   // per device; a racing first call writes the same value
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return hipErrorNotSupported;
    if (cu_count[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) return hipErrorNotSupported;
        cu_count[dev] = n;
    }
    if (hipError_t e = ensure_dynamic_lds<stem_conv_kernel>(lds); e != hipSuccess) return e;
    const int ocb = (OC + 63) / 64;
    int gx = 2 * cu_count[dev] / ocb;
    if (gx < 1) gx = 1;
    if (gx > a.blocks) gx = a.blocks;
    hipLaunchKernelGGL(stem_conv_kernel, dim3(gx, ocb), dim3(256), lds, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
