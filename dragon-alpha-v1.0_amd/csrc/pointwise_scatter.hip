// Backward-data of a 1x1 convolution whose stride exceeds the filter (sh, sw >= 1, sh * sw > 1, no padding, IH = sh * OH,
// IW = sw * OW), both operands straight from memory, fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950. No LDS, no barrier.
//
//   deltaX[n, sh*i, sw*j, ic] = sum_oc deltaY[n, i, j, oc] * W[oc, ic]        every other pixel of deltaX = 0
//
// Kernel split sees this layer as sh * sw phases of which one has the only tap and the others write zeros; run that way
// the zero phases cost work items, address arithmetic and a share of the line of items each. Here the layer is what it
// is: ONE matrix product over the pixels of deltaY whose rows are scattered - pixel (i, j) owns the sh x sw block of
// deltaX at (sh*i, sw*j), gets the product into the block's first pixel and zeros into the rest -, HBM-bound (two thirds
// of its bytes are stores). The product is pointwise_direct.hip's: a wavefront owns T <= 4 tiles of 16 pixels, per step of
// 16 reduced channels one 128-bit load per tile and four for the filter feed 16 T MFMAs, loads one step ahead through a
// cursor; a lane's accumulators are 4 consecutive channels of a pixel and leave as 128-bit stores, the zeros beside them
// (16 lanes = 256 contiguous bytes of a pixel; a block's first row is 2 x 256 contiguous bytes for sw = 2).
// Measured on 64 x 56 x 56 x 64 <- 28 x 28 x 128, stride 2: 0.0161 ms against 0.0165 ms through the phases - the zero phases
// were not the cost; 51 MB of stores at the 4.1-4.8 TB/s the device writes and a launch's 3-4 us are (stores with the
// non-temporal cache policy measured the same).
#include "common.hpp"

namespace alpha {

struct PwScatterArgs {
    const float *A;   // deltaY [M][K]
    const float *B;   // W [K][N]
    float *O;         // deltaX [Nimg, IH, IW, N]
    int M, K, N;      // M = Nimg * OH * OW; K % 32 == 0, N % 4 == 0
    int OW, IW, sh, sw;
    int tiles, nblocks, waves;
    int o_bytes;
    FastDiv d_OW, d_OHW;
    int OHW, IHW;     // OH * OW, IH * IW
};

template <int V> struct PwsInt { static constexpr int value = V; };

// S2: the stride is 2 x 2 (the block's four stores unrolled; any other stride loops over the block)
template <bool S2>
__global__ __launch_bounds__(256, 4) void pointwise_scatter_kernel(const PwScatterArgs p)
{
    const int t = threadIdx.x, lane = t & 63;
    const int l16 = lane & 15, q = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (t >> 6));
    const int t_lo = (int)((long)p.tiles * wave / p.waves), t_hi = (int)((long)p.tiles * (wave + 1) / p.waves);
    const int K = p.K, N = p.N, KS = K >> 4;

    constexpr unsigned NEVER = 0x80000000u;   // beyond every descriptor (tensors below 2 GB, host-checked)
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.A), 0, p.M * K * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.B), 0, K * N * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t o_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.O, 0, p.o_bytes, 0x00020000);
    const unsigned a_lane = (unsigned)((l16 * K + 4 * q) * 4);   // rows past M: beyond the descriptor, zeros

    auto run = [&](auto tc, int tile0, int count) {
        constexpr int T = decltype(tc)::value;
        if (count <= 0) return;
        floatx4 a[2][T], b[2][4];
        int c_tile = tile0, c_nb = 0, c_ks = 0, c_left = count * p.nblocks * KS;
        auto request = [&](int slot) {
            const int a_off = __builtin_amdgcn_readfirstlane((c_tile * 16 * K + c_ks * 16) * 4);
            const int n_l = c_nb * 64 + 4 * l16;
            const unsigned b_lane = n_l < N ? (unsigned)((4 * q * N + n_l) * 4) : NEVER;
            const int b_off = __builtin_amdgcn_readfirstlane(c_ks * 16 * N * 4);
#pragma unroll
            for (int i = 0; i < T; i++)
                a[slot][i] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_lane + (unsigned)(i * 16 * K * 4), a_off, 0));
#pragma unroll
            for (int s = 0; s < 4; s++)
                b[slot][s] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, b_lane + (unsigned)(s * N * 4), b_off, 0));
            if (c_left > 1) {   // scalar bookkeeping only
                c_left--;
                c_ks++;
                if (c_ks == KS) {
                    c_ks = 0;
                    c_nb++;
                    if (c_nb == p.nblocks) {
                        c_nb = 0;
                        c_tile += T;
                    }
                }
            }
        };
        request(0);
        for (int g = 0; g < count; g++) {
            const int tile = tile0 + g * T;
            // where this lane's pixels 16 (tile + i) + 4 q + r land in deltaX: byte offset of the block's first pixel, channel 0
            unsigned pix[T][4];
#pragma unroll
            for (int i = 0; i < T; i++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int m = (tile + i) * 16 + 4 * q + r;
                    const bool live = m < p.M;
                    const int mm = live ? m : 0;
                    const int n = fdiv(mm, p.d_OHW), rem = mm - n * p.OHW;
                    const int oi = fdiv(rem, p.d_OW), oj = rem - oi * p.OW;
                    pix[i][r] = live ? (unsigned)(((n * p.IHW + oi * p.sh * p.IW + oj * p.sw) * N) * 4) : NEVER;
                }
            for (int nb = 0; nb < p.nblocks; nb++) {
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
                for (int ks = 0; ks < KS; ks += 2) {   // KS is even (K % 32 == 0, host-checked)
                    request(1);
                    multiply(0);
                    __builtin_amdgcn_sched_barrier(0);
                    request(0);
                    multiply(1);
                    __builtin_amdgcn_sched_barrier(0);
                }
                // ---- results and the zeros of their blocks: channels 64 nb + 4 l16 .. + 3 --------------------------------
                const int n_l = nb * 64 + 4 * l16;
                const bool n_ok = n_l < N;
                const floatx4 zero = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < T; i++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const unsigned base = n_ok && pix[i][r] != NEVER ? pix[i][r] + (unsigned)(n_l * 4) : NEVER;
                        const floatx4 v = floatx4{acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]};
                        if constexpr (S2) {
                            const int row = __builtin_amdgcn_readfirstlane(p.IW * N * 4);
                            buffer_store_b128_guarded(v, o_rsrc, base, 0);
                            buffer_store_b128_guarded(zero, o_rsrc, base, N * 4);
                            buffer_store_b128_guarded(zero, o_rsrc, base, row);
                            buffer_store_b128_guarded(zero, o_rsrc, base, row + N * 4);
                        } else {
                            for (int y = 0; y < p.sh; y++)        // uniform
                                for (int x = 0; x < p.sw; x++) {
                                    const int o_off = __builtin_amdgcn_readfirstlane((y * p.IW + x) * N * 4);
                                    buffer_store_b128_guarded((y | x) == 0 ? v : zero, o_rsrc, base, o_off);
                                }
                        }
                    }
            }
        }
    };

    // the share as groups of two tiles and one of one: many wavefronts with few registers each (four workgroups per compute
    // unit) suit a kernel that waits for memory, not for the matrix pipes
    const int cnt = t_hi - t_lo;
    run(PwsInt<2>{}, t_lo, cnt >> 1);
    run(PwsInt<1>{}, t_lo + (cnt & ~1), cnt & 1);
}

// deltaX[Nimg, sh*OH, sw*OW, N] from deltaY[Nimg, OH, OW, K] and W[K][N] (1x1 filter, no padding): the product into every
// block's first pixel, zeros elsewhere. Returns hipErrorNotSupported (nothing launched) when the layer does not fit: K not
// a multiple of 32, a stride of 1 x 1, more than 16 pixels per block, tensors of 2 GB.
hipError_t launch_pointwise_scatter(hipStream_t stream, const float *dY, const float *W, float *dX, int Nimg, int OH, int OW,
                                    int K, int N, int sh, int sw)
{
    if (K < 32 || (K & 31) || N < 4 || (N & 3) || sh < 1 || sw < 1 || sh * sw < 2 || sh * sw > 16) return hipErrorNotSupported;
    const long M = (long)Nimg * OH * OW;
    const long o_bytes = M * sh * sw * N * 4;
    if (M < 1 || M * K * 4 >= (1L << 31) || o_bytes >= (1L << 31) || (long)K * N * 4 >= (1L << 30)) return hipErrorNotSupported;
    const int cus = device_cu_count();
    if (cus < 1) return hipErrorNotSupported;
    PwScatterArgs a{};
    a.A = dY; a.B = W; a.O = dX;
    a.M = (int)M; a.K = K; a.N = N;
    a.OW = OW; a.IW = sw * OW; a.sh = sh; a.sw = sw;
    a.OHW = OH * OW; a.IHW = sh * OH * sw * OW;
    a.o_bytes = (int)o_bytes;
    a.tiles = (int)((M + 15) / 16);
    a.nblocks = (N + 63) / 64;
    a.d_OW = make_fastdiv(OW);
    a.d_OHW = make_fastdiv(OH * OW);
    // four workgroups of four wavefronts per compute unit; fewer when there are fewer tiles than wavefronts
    long wgs = 4L * cus;
    if (wgs * 4 > a.tiles) wgs = (a.tiles + 3) / 4;
    a.waves = (int)(wgs * 4);
    if (sh == 2 && sw == 2) hipLaunchKernelGGL(pointwise_scatter_kernel<true>, dim3((unsigned)wgs), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(pointwise_scatter_kernel<false>, dim3((unsigned)wgs), dim3(256), 0, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
