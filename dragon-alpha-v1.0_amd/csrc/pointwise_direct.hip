// 1x1 stride-1 convolution (forward from CW, backward-data from W) with BOTH operands straight from memory, fp32 MFMA
// v_mfma_f32_16x16x4_f32, gfx950. No LDS, no barrier.
//
//   O[m, n] = sum_k A[m, k] * B[k, n]        m = pixel, k = reduced channels, n = produced channels; B is [K][N]
//
// The filter-resident kernel of pointwise.hip pays for its residency at the start of every launch: 2048 wavefronts
// wait for 64 KB of filter per compute unit and a first tile each before the first MFMA (a sixth of the kernel on the
// 56x56 bottleneck layers), and its results cross LDS on their way out. Here a wavefront owns T tiles of 16 pixels and
// one block of 64 produced channels and multiplies in steps of 16 reduced channels:
//   a_t  = A[16t + l16][k0 + 4q .. +3]                (lane (l16, q); one 128-bit load per tile)
//   b_s  = B[k0 + 4q + s][n0 + 4*l16 .. +3], s = 0..3  (four 128-bit loads, shared by the T tiles)
// MFMA (t, s, j) multiplies component s of a_t with component j of b_s: rows = the 16 pixels of tile t, k = the four
// reduced channels k0 + 4q + s (q = 0..3), columns = the produced channels n0 + 4*l16 + j. The 16 T MFMAs of a step use
// T + 4 loads, and the accumulators of a lane hold 4 consecutive produced channels of a pixel: the results leave as
// 128-bit stores, 256 contiguous bytes per pixel from 16 lanes, without a transpose. The filter (64 KB at most) is
// read from L2 again by every wavefront, once per T tiles.
//
// Work is dealt out in tiles: wavefront i of the grid (two per SIMD) owns the tiles [tiles*i/W, tiles*(i+1)/W), as
// groups of 4, 3, 2 or 1 tiles with one loop per group size (a single path per loop: loads and stores are
// unconditional, so every wait is an exact count), all produced-channel blocks of a group before the next group (the
// A tiles are then re-read from L1/L2).
#include "common.hpp"

namespace alpha {

struct PwDirectArgs {
    const float *A;
    const float *B;
    float *O;
    int M, K, N;      // K % 16 == 0, N % 4 == 0
    int tiles;        // ceil(M / 16)
    int nblocks;      // ceil(N / 64)
    int waves;        // wavefronts of the grid
    Epilogue ep;
};

template <int V> struct PwdInt { static constexpr int value = V; };

// Loads run one step (16 reduced channels, 64 MFMAs per group of four tiles) ahead of the multiplications; two steps
// ahead measured the same.
template <bool EPI>
__global__ __launch_bounds__(256, 2) void pointwise_direct_kernel(const PwDirectArgs p)
{
    const int t = threadIdx.x, lane = t & 63;
    const int l16 = lane & 15, q = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (t >> 6));
    const int t_lo = (int)((long)p.tiles * wave / p.waves), t_hi = (int)((long)p.tiles * (wave + 1) / p.waves);
    const int K = p.K, N = p.N, KS = K >> 4;

    constexpr unsigned NEVER = 0x40000000u;
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.A), 0, p.M * K * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.B), 0, K * N * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t o_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.O, 0, p.M * N * 4, 0x00020000);
    const unsigned a_lane = (unsigned)((l16 * K + 4 * q) * 4);   // rows past M: beyond the descriptor, zeros

    // One loop per group size T: groups [first, first + count) of T tiles each.
    auto run = [&](auto tc, int tile0, int count) {
        constexpr int T = decltype(tc)::value;
        if (count <= 0) return;
        floatx4 a[2][T], b[2][4];
        // Load cursor: one step ahead of the multiplications, through (group, block of produced channels, step).
        int c_tile = tile0, c_nb = 0, c_ks = 0, c_left = count * p.nblocks * KS;
        auto request = [&](int slot) {
            // past the last step the descriptors' ranges are not left: the loads repeat the last step's (unused)
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
                // ---- results: lane holds pixels 16(tile + i) + 4q + r, produced channels 64 nb + 4 l16 + j -------------
                const int n_l = nb * 64 + 4 * l16;
                const unsigned o_lane = n_l < N ? (unsigned)((4 * q * N + n_l) * 4) : NEVER;
                float sub[4], mul[4], add[4];
                floatx4 bias = floatx4{0.f, 0.f, 0.f, 0.f};
                if (EPI) {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        sub[j] = 0.f; mul[j] = 1.f; add[j] = 0.f;
                        if (n_l < N && !p.ep.gate) ep_channel(p.ep, n_l + j, sub[j], mul[j], add[j]);
                    }
                } else if (p.ep.bias != nullptr && n_l < N) {
                    bias = *reinterpret_cast<const floatx4 *>(p.ep.bias + n_l);
                }
#pragma unroll
                for (int i = 0; i < T; i++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int o_off = __builtin_amdgcn_readfirstlane(((tile + i) * 16 + r) * N * 4);
                        floatx4 v = floatx4{acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]};
                        if (EPI) {
                            if (p.ep.gate) {   // uniform
                                const floatx4 gt = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(
                                    __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.ep.gate), 0, p.M * N * 4, 0x00020000), o_lane, o_off, 0));
#pragma unroll
                                for (int j = 0; j < 4; j++) v[j] = ep_gate(v[j], gt[j], p.ep.slope);
                            } else {
#pragma unroll
                                for (int j = 0; j < 4; j++) v[j] = ep_finish(v[j], sub[j], mul[j], add[j], p.ep.slope);
                            }
                        } else {
                            v += bias;
                        }
                        buffer_store_b128_guarded(v, o_rsrc, o_lane, o_off);
                    }
            }
        }
    };

    // the share as groups of 4, 3, 2 and 1 tiles: 4a + 3b for six tiles or more, 3 + 2 for five
    const int cnt = t_hi - t_lo;
    int n4 = 0, n3 = 0, n2 = 0, n1 = 0;
    if (cnt >= 6) {
        n3 = (4 - (cnt & 3)) & 3;   // cnt - 3*n3 is a multiple of 4 (n3 <= 3, and cnt >= 9 whenever n3 == 3: 6 -> n3 = 2, 7 -> 1)
        n4 = (cnt - 3 * n3) >> 2;
    } else if (cnt == 5) {
        n3 = 1; n2 = 1;
    } else if (cnt == 4) {
        n4 = 1;
    } else if (cnt == 3) {
        n3 = 1;
    } else if (cnt == 2) {
        n2 = 1;
    } else if (cnt == 1) {
        n1 = 1;
    }
    run(PwdInt<4>{}, t_lo, n4);
    run(PwdInt<3>{}, t_lo + 4 * n4, n3);
    run(PwdInt<2>{}, t_lo + 4 * n4 + 3 * n3, n2);
    run(PwdInt<1>{}, t_lo + 4 * n4 + 3 * n3 + 2 * n2, n1);
}

// Returns hipErrorNotSupported (nothing launched) when the layer does not fit; the caller then uses another kernel.
hipError_t launch_pointwise_direct(hipStream_t stream, const float *A, const float *B, float *O, long M, int K, int N,
                                   const float *bias, const Epilogue *ep)
{
    if (M < 1 || K < 32 || (K & 31) || N < 4 || (N & 3)) return hipErrorNotSupported;
    if (M * K * 4 >= (1L << 31) || M * N * 4 >= (1L << 31) || (long)K * N * 4 >= (1L << 30)) return hipErrorNotSupported;
    const int cus = device_cu_count();
    if (cus < 1) return hipErrorNotSupported;
    PwDirectArgs a{};
    a.A = A; a.B = B; a.O = O;
    a.M = (int)M; a.K = K; a.N = N;
    a.tiles = (int)((M + 15) / 16);
    a.nblocks = (N + 63) / 64;
    a.ep = ep ? *ep : bias_epilogue(bias);
    int wgs = 2 * cus;                             // two wavefronts per SIMD
    if (wgs * 4 > a.tiles) wgs = (a.tiles + 3) / 4;   // at least one tile per wavefront
    a.waves = wgs * 4;
    if (a.ep.fused) hipLaunchKernelGGL(pointwise_direct_kernel<true>, dim3(wgs), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(pointwise_direct_kernel<false>, dim3(wgs), dim3(256), 0, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
