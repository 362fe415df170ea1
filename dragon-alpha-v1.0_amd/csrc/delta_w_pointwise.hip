// Backward-filter of 1x1 stride-1 layers without LDS staging, fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950.
//
//   deltaW[oc, ic] = sum over pixels k of the K slice of  deltaY[k, oc] * X[k, ic]
//
// The reduction index is the pixel, the slow axis of both tensors, so a lane's natural 128-bit load brings 4
// CHANNELS of one pixel - not what one MFMA operand register holds (one row/column, 4 consecutive k). It becomes the
// right thing when the rows and columns are interleaved over several MFMAs: lane (l16, q) loads
//   ya = deltaY[pixel 4g + q][oc0 + 4*l16 .. +3]      xa = X[pixel 4g + q][ic0 + 4*l16 .. +3]
// and MFMA (i, j) multiplies component i of ya with component j of xa: its 16 rows are the output channels
// oc0 + 4*l16 + i, its 16 columns the input channels ic0 + 4*l16 + j, its 4 k's the four pixels of group g. Sixteen
// MFMAs per pair of loads cover a 64 x 64 block of deltaW; both loads are fully coalesced 256-byte rows, nothing is
// staged or synchronised, and a ring of D pixel groups in registers hides the memory latency.
//
// A workgroup has 8 wavefronts: TPW blocks of 64 x 64 outputs times 8/TPW parts of the slice's pixels; the parts are
// summed through LDS in a fixed order, so a fixed (shape, GridZ) gives bit-identical results. Slice z of the
// reference's partition stores to deltaW (z = 0) or deltaW_buf[z-1].
#include "common.hpp"

namespace alpha {

typedef float floatx4 __attribute__((ext_vector_type(4)));

struct DwPointwiseArgs {
    const float *X;
    const float *dY;
    float *dW;
    float *dW_buf;
    float *dB;       // NULL, or the bias gradient (column sums of deltaY): slice z writes to dB (z = 0)
    float *dB_buf;   // or dB_buf[z-1][OC]
    int IC, OC;
    int GK, GK_slice, GZ;
    int tiles, icb_count;   // 64 x 64 output blocks: tiles = (OC/64) * (IC/64), block index = ocb * icb_count + icb
    int TPW;                // blocks per workgroup (1, 2, 4 or 8); 8 / TPW wavefronts share a block
};

template <int V> struct DwpFlag { static constexpr int value = V; };
constexpr int DWP_D = 8;    // pixel groups in flight per wavefront

__global__ __launch_bounds__(512, 1) void delta_w_pointwise_kernel(const DwPointwiseArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float smem[];   // [KSPLIT-1][TPW][16 accumulators][64 lanes] float4
    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int TPW = p.TPW, KSPLIT = 8 / TPW;
    const int tw = w % TPW, kpart = w / TPW;
    // The workgroups of a slice read the same pixels (deltaY or X, whichever their blocks share). Workgroups are dealt
    // round-robin to the 8 XCDs, each with its own L2: when the slices divide among the XCDs, slice z runs on XCD z % 8,
    // its workgroups next to each other in time, and the second reader of a row finds it in that L2.
    int bx = blockIdx.x, z = blockIdx.y;
    if ((p.GZ & 7) == 0) {
        const int lin = blockIdx.x + gridDim.x * blockIdx.y, xcd = lin & 7, idx = lin >> 3;
        bx = idx % (int)gridDim.x;
        z = xcd + 8 * (idx / (int)gridDim.x);
    }
    const int tile = bx * TPW + tw;
    const bool live = tile < p.tiles;
    const int ocb = live ? tile / p.icb_count : 0, icb = live ? tile - ocb * p.icb_count : 0;

    const int k_start = p.GK_slice * z;
    const int k_end = (z != p.GZ - 1) ? k_start + p.GK_slice : p.GK;
    // pixel groups (4 pixels) of this wavefront's part; GK and GK_slice are multiples of 4
    const int groups = (k_end - k_start) >> 2;
    // (uniform over the wavefront; said so explicitly, because the pixel-group offset of a load must be a scalar)
    const int g0 = __builtin_amdgcn_readfirstlane((k_start >> 2) + (int)((long)groups * kpart / KSPLIT));
    const int g1 = __builtin_amdgcn_readfirstlane(live ? (k_start >> 2) + (int)((long)groups * (kpart + 1) / KSPLIT) : g0);

    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    // Loads through buffer descriptors: descriptor base + uniform offset of the pixel group (scalar register) + fixed
    // per-lane offset, no vector arithmetic per load (a 64-bit address per load cost 6 vector instructions per 16 MFMAs).
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.dY), 0, p.GK * p.OC * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.X), 0, p.GK * p.IC * 4, 0x00020000);
    const unsigned y_lane = (unsigned)(q * p.OC + ocb * 64 + 4 * l16) * 4u;
    const unsigned x_lane = (unsigned)(q * p.IC + icb * 64 + 4 * l16) * 4u;
    floatx4 ya[DWP_D], xa[DWP_D];
    const bool do_bias = p.dB != nullptr && live && icb == 0;   // one wavefront set per block row of deltaW
    floatx4 bsum = floatx4{0.f, 0.f, 0.f, 0.f};
    auto load = [&](int d, int g) {   // g is clamped by the caller to a group of this part
        ya[d] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(y_rsrc, y_lane, g * 16 * p.OC, 0));
        xa[d] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, x_lane, g * 16 * p.IC, 0));
    };
    // The ring loop is free of branches on purpose: the loads of a slot are waited for by count (14 younger loads may
    // stay in flight), and the count is only known when every load and every use is executed unconditionally. With a
    // branch around the MFMAs of a slot each round of the ring began with a wait for all 16 loads.
    // The ring exists twice, with and without the column sums of deltaY for the bias gradient (4 vector instructions
    // per 16 MFMAs that a call without deltaB, and every workgroup but those of the first input-channel block, skip).
    auto ring = [&](auto with_bias) {
        constexpr bool WB = decltype(with_bias)::value != 0;
        auto multiply = [&](int d) {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ya[d][i], xa[d][j], acc[i][j], 0, 0, 0);
            if (WB) bsum += ya[d];
        };
#pragma unroll
        for (int d = 0; d < DWP_D; d++) load(d, min(g0 + d, g1 - 1));
        int g = g0;
        for (; g + DWP_D <= g1; g += DWP_D) {
#pragma unroll
            for (int d = 0; d < DWP_D; d++) {
                multiply(d);
                load(d, min(g + d + DWP_D, g1 - 1));   // past the end: the last group again, unused
                __builtin_amdgcn_sched_barrier(0);      // keeps the refill next to its slot (the scheduler batches them)
            }
        }
        const int rest = g1 - g;   // < DWP_D groups, already in slots 0 .. rest-1
#pragma unroll
        for (int d = 0; d < DWP_D - 1; d++)
            if (d < rest) multiply(d);
    };
    if (g0 < g1) {
        if (__builtin_amdgcn_readfirstlane((int)do_bias)) ring(DwpFlag<1>{});
        else ring(DwpFlag<0>{});
    }

    // ---- bias gradient: lanes q = 0..3 hold different pixels of the same 4 channels (wavefront shuffles), the parts
    // follow through LDS below ---------------------------------------------------------------------------------------
    if (do_bias) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            bsum[i] += __shfl_xor(bsum[i], 16);
            bsum[i] += __shfl_xor(bsum[i], 32);
        }
    }
    floatx4 *bred = reinterpret_cast<floatx4 *>(smem) + (size_t)(KSPLIT - 1) * TPW * 16 * 64;   // [KSPLIT-1][TPW][16 lanes]
    if (do_bias && kpart > 0 && q == 0) bred[((kpart - 1) * TPW + tw) * 16 + l16] = bsum;

    // ---- sum the parts in the order 0, 1, 2, ... and store ------------------------------------------------------
    floatx4 *red = reinterpret_cast<floatx4 *>(smem);
    if (kpart > 0) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) red[(((kpart - 1) * TPW + tw) * 16 + i * 4 + j) * 64 + lane] = acc[i][j];
    }
    __syncthreads();
    if (kpart == 0 && live) {
        for (int part = 1; part < KSPLIT; part++)
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const floatx4 v = red[(((part - 1) * TPW + tw) * 16 + i * 4 + j) * 64 + lane];
                    acc[i][j] += v;
                }
        if (do_bias && q == 0) {
            for (int part = 1; part < KSPLIT; part++) bsum += bred[((part - 1) * TPW + tw) * 16 + l16];
            float *bdst = (z == 0) ? p.dB : p.dB_buf + (size_t)(z - 1) * p.OC;
            *reinterpret_cast<float4 *>(bdst + ocb * 64 + 4 * l16) = make_float4(bsum[0], bsum[1], bsum[2], bsum[3]);
        }
        float *dst = (z == 0) ? p.dW : p.dW_buf + (size_t)(z - 1) * p.OC * p.IC;
        // acc[i][j][r] = deltaW[oc = 64 ocb + 4 (4q + r) + i][ic = 64 icb + 4 l16 + j]
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int oc = ocb * 64 + 4 * (4 * q + r) + i;
                *reinterpret_cast<float4 *>(dst + (size_t)oc * p.IC + icb * 64 + 4 * l16) =
                    make_float4(acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]);
            }
    }
}

// Returns hipErrorNotSupported (nothing launched) unless IC and OC are multiples of 64; the caller then uses another
// kernel.
hipError_t launch_deltaW_pointwise(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                                   int GK, int IC, int OC, int GK_slice, int GZ, float *dB, float *dB_buf)
{
    if ((IC & 63) || (OC & 63) || IC < 64 || OC < 64 || (GK & 3) || (GK_slice & 3) || GK < 4) return hipErrorNotSupported;
    if ((size_t)GK * (size_t)(IC > OC ? IC : OC) * 4 >= (1ull << 31)) return hipErrorNotSupported;   // buffer descriptors below 2 GB
    static int cu_count[64] = {0};   // per device; a racing first call writes the same value
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return hipErrorNotSupported;
    if (cu_count[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) return hipErrorNotSupported;
        cu_count[dev] = n;
    }
    DwPointwiseArgs a{};
    a.X = X; a.dY = dY; a.dW = dW; a.dW_buf = dW_buf; a.dB = dB; a.dB_buf = dB_buf;
    a.IC = IC; a.OC = OC; a.GK = GK; a.GK_slice = GK_slice; a.GZ = GZ;
    a.icb_count = IC / 64;
    a.tiles = (OC / 64) * a.icb_count;
    // as many blocks per workgroup as still leave a workgroup for every compute unit
    a.TPW = 1;
    for (int tpw = 8; tpw > 1; tpw >>= 1)
        if (tpw <= a.tiles && (long)((a.tiles + tpw - 1) / tpw) * GZ >= cu_count[dev]) { a.TPW = tpw; break; }
    const size_t lds = (size_t)(8 / a.TPW - 1) * a.TPW * (16 * 64 + 16) * sizeof(floatx4) + 16;   // accumulators + bias sums of the parts
    if (hipError_t e = ensure_dynamic_lds<delta_w_pointwise_kernel>(lds); e != hipSuccess) return e;
    dim3 grid((a.tiles + a.TPW - 1) / a.TPW, GZ);
    hipLaunchKernelGGL(delta_w_pointwise_kernel, grid, dim3(512), lds, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
