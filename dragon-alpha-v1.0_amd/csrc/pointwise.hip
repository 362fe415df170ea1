// 1x1 stride-1 convolution (forward and backward-data) as a streaming GEMM, fp32 MFMA v_mfma_f32_16x16x4_f32, gfx950.
//
//   O[m, n] = sum_k A[m, k] * B(k, n)        m = pixel (N*H*W of them), k = reduced channels, n = produced channels
//
// These layers sit at or below the ridge of the roofline (c5a/c5c: 26 FLOP/byte), so the design goal is one pass
// over A and O at full memory rate, not MFMA occupancy:
//   * the whole filter (K x N <= ~120 KB with padding) is copied into LDS once per workgroup, laid out [n][K+8] so
//     that a lane's 4 consecutive k of one n are one 128-bit read and the 32 lanes of a half wavefront hit 32
//     different 16-byte slots (row stride = 8 floats modulo 16);
//   * one workgroup of 8 wavefronts per compute unit, persistent, owning a contiguous range of 16-pixel tiles that
//     its wavefronts draw from a counter in LDS;
//   * A goes from global memory straight into the MFMA operand layout: lane (l16, q) loads float4
//     A[16t + l16][64kb + 16c + 4q ..] (K permutation: lane group q supplies channel 16c + 4q + s at step s, as the
//     filter read does), one whole tile ahead of the tile being multiplied. No LDS, no barrier for A;
//   * each 16 x 64 block of results is transposed through a wavefront-private LDS patch so that every pixel's 256
//     bytes leave as whole lines.
#include "common.hpp"

namespace alpha {

typedef float floatx4 __attribute__((ext_vector_type(4)));

struct PointwiseArgs {
    const float *A;   // [rows][K]; output pixel m = (n, oh, ow) reads row (n*AH + oh*sh)*AW + ow*sw
    const float *B;   // b_kmajor ? [K][ldn] : [ldn][K]
    float *O;         // [M][ldn]
    int M, K, ldn;    // ldn = all produced channels; a workgroup produces the 16*NT of them starting at 16*NT*blockIdx.y
    int b_kmajor;
    int tiles;        // ceil(M / 16)
    int strided;      // 0: row = m
    int a_bytes;      // size of A in bytes (< 2 GB)
    const float *bias;   // NULL or [ldn]
    int AH, AW, sh, sw;
    FastDiv d_OW, d_OHW;
};

constexpr int PW_OS = 64 + 4;   // staging row stride (floats)
template <int V> struct IntC { static constexpr int value = V; };

template <int NT, int KB>   // N = 16*NT produced channels, K = 64*KB reduced channels
__global__ __launch_bounds__(512, 1) void pointwise_kernel(const PointwiseArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float smem[];
    constexpr int K = 64 * KB, N = 16 * NT, KS = K + 8;
    float *Bs = smem;                                 // [N][KS]
    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    float *Os = smem + N * KS + w * (16 * PW_OS);     // [16][PW_OS], private to the wavefront

    // ---- tiles: the workgroup owns the contiguous range [t_begin, t_end); its wavefronts take the first eight
    // statically and then draw from a counter in LDS, so they finish within one tile of each other whatever the
    // range length (a static split of 24.5 tiles over 8 wavefronts would leave a quarter of the machine idle).
    // The tiles beyond the last multiple of eight are split further, into (tile, group of 64 produced channels) units
    // or, with a single group, (tile, 16 channels) units, dealt to the wavefronts in order (wavefronts w and w + 4
    // share a SIMD): a 25th tile costs every SIMD a quarter of a tile instead of costing one SIMD a whole one.
    const int G = gridDim.x;
    const int t_begin = (int)((long)p.tiles * blockIdx.x / G), t_end = (int)((long)p.tiles * (blockIdx.x + 1) / G);
    constexpr int NG = NT / 4;
    constexpr int UPT = NG > 1 ? NG : 4;              // units per tile
    const int t_main = t_begin + ((t_end - t_begin) & ~7);
    const int units = (t_end - t_main) * UPT;
    const int unit_tile = t_main + w / UPT;           // tile of this wavefront's first unit, if it has one (w < units)
    int *queue = reinterpret_cast<int *>(smem + N * KS + 8 * 16 * PW_OS);
    if (t == 0) *queue = t_begin + 8;

    const int n_off = blockIdx.y * N, ldn = p.ldn;
    // A and O are addressed through buffer descriptors: descriptor base + uniform offset of the tile (scalar register)
    // + a per-lane offset that is fixed for the whole kernel, no vector arithmetic per load or store. Rows past M are
    // beyond the descriptors: their loads return zeros and their stores are dropped, so nothing in the tile loop is
    // conditional and every wait can be counted exactly (a wait placed after a store whose execution is uncertain would
    // have to wait for every store to be acknowledged). A strided layer (input rows thinned) computes its lane offsets
    // per tile.
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.A), 0, p.a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t o_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.O, 0, p.M * ldn * 4, 0x00020000);
    const unsigned a_lane = (unsigned)(l16 * K + 4 * q) * 4u;
    const unsigned o_lane = (unsigned)(q * ldn + n_off + 4 * l16) * 4u;
    auto load_a = [&](floatx4 (&a)[KB][4], int tile_) {
        const int tile = __builtin_amdgcn_readfirstlane(tile_);   // uniform, said so: the tile offset must be a scalar
        unsigned voff = a_lane;
        int soff = tile * 16 * K * 4;
        if (p.strided) {
            const int m = min(tile * 16 + l16, p.M - 1);
            const int n = fdiv(m, p.d_OHW), rem = m - n * p.d_OHW.d;
            const int oh = fdiv(rem, p.d_OW), ow = rem - oh * p.d_OW.d;
            voff = (unsigned)(((n * p.AH + oh * p.sh) * p.AW + ow * p.sw) * K + 4 * q) * 4u;
            soff = 0;
        }
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int c = 0; c < 4; c++)
                a[kb][c] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, voff + (64 * kb + 16 * c) * 4, soff, 0));
    };
    floatx4 aP[KB][4], aQ[KB][4];
    int tile = __builtin_amdgcn_readfirstlane(t_begin + w);

    // ---- filter -> LDS, once, eight 128-bit loads in flight per thread. The first tile's A fragments are requested
    // right after the filter loads: behind them (loads return in order, and the A fragments of all workgroups together
    // are a third of a 256-channel input, far more memory time than the filter, which comes from L2), but before the
    // filter is written to LDS. What this costs (time stamps, K = 256, N = 64): the 64 KB of filter are 512 cache lines
    // per compute unit, the eight wavefronts get their loads issued one after the other over 6 k cycles, the last
    // lines arrive after 12 k, and the first tile starts 14 k cycles into a kernel of 72 k. ------------------------
    constexpr int QUADS = N * K / 4;
    const int first_tile = tile < t_main ? tile : w < units ? unit_tile : t_end - 1;
    if (!p.b_kmajor) {
        // [N][K]: a row of the filter is a row of Bs
        for (int base = 0; base < QUADS; base += 512 * 8) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int idx = min(base + t + 512 * u, QUADS - 1);
                const int n = idx / (K / 4), k4 = (idx % (K / 4)) * 4;
                v[u] = *reinterpret_cast<const float4 *>(p.B + (size_t)(n_off + n) * K + k4);
            }
            if (base + 512 * 8 >= QUADS) load_a(aP, first_tile);
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int idx = base + t + 512 * u;
                if (idx < QUADS) {
                    const int n = idx / (K / 4), k4 = (idx % (K / 4)) * 4;
                    *reinterpret_cast<float4 *>(Bs + n * KS + k4) = v[u];
                }
            }
        }
    } else {
        // [K][ldn]: transposed on the way. A thread takes a cell of 4 k x 4 n: four 128-bit loads (rows k..k+3), a 4x4
        // transpose in registers, four 128-bit LDS stores (rows n..n+3 of Bs). The 64 lanes of a wavefront form a tile
        // of 8 cells along k x 8 along n: a load touches 8 rows x 128 contiguous bytes, and the 32 lanes of a half
        // wavefront store to 32 different 16-byte slots (a row of Bs is 8 floats modulo 16 longer than a power of two).
        // (One lane per k with scalar transposing stores touched 64 cache lines per load and staged in 12-17 k cycles.)
        constexpr int CELLS = 64 * NT * KB, TKT = 2 * KB, ITER = (CELLS + 511) / 512;
        float4 v[ITER][4];
        int k0[ITER], n0[ITER];
#pragma unroll
        for (int it = 0; it < ITER; it++) {
            const int tile8 = min(w + 8 * it, CELLS / 64 - 1);
            k0[it] = 4 * (8 * (tile8 % TKT) + (lane & 7));
            n0[it] = 4 * (8 * (tile8 / TKT) + (lane >> 3));
#pragma unroll
            for (int r = 0; r < 4; r++)
                v[it][r] = *reinterpret_cast<const float4 *>(p.B + (size_t)(k0[it] + r) * ldn + n_off + n0[it]);
        }
        load_a(aP, first_tile);
#pragma unroll
        for (int it = 0; it < ITER; it++) {
            if (w + 8 * it < CELLS / 64) {
                float *dst = Bs + n0[it] * KS + k0[it];
                *reinterpret_cast<float4 *>(dst) = make_float4(v[it][0].x, v[it][1].x, v[it][2].x, v[it][3].x);
                *reinterpret_cast<float4 *>(dst + KS) = make_float4(v[it][0].y, v[it][1].y, v[it][2].y, v[it][3].y);
                *reinterpret_cast<float4 *>(dst + 2 * KS) = make_float4(v[it][0].z, v[it][1].z, v[it][2].z, v[it][3].z);
                *reinterpret_cast<float4 *>(dst + 3 * KS) = make_float4(v[it][0].w, v[it][1].w, v[it][2].w, v[it][3].w);
            }
        }
    }
    __syncthreads();

    const float *bl = Bs + l16 * KS + 4 * q;
    // bias of the columns this lane stores (zeros without one: the add is unconditional, the loop branch-free)
    floatx4 bias4[NT / 4];
#pragma unroll
    for (int jg = 0; jg < NT / 4; jg++)
        bias4[jg] = p.bias ? *reinterpret_cast<const floatx4 *>(p.bias + n_off + 64 * jg + 4 * l16) : floatx4{0.f, 0.f, 0.f, 0.f};
    // the bias and the first tile's fragments are waited for here, so that no load is outstanding when the loop is
    // entered (a load pending at the loop head would make every iteration start with a wait for the previous
    // iteration's stores)
#pragma unroll
    for (int jg = 0; jg < NT / 4; jg++) asm volatile("" : "+v"(bias4[jg]));
#pragma unroll
    for (int kb = 0; kb < KB; kb++)
#pragma unroll
        for (int c = 0; c < 4; c++) asm volatile("" : "+v"(aP[kb][c]));
    // One tile = NG groups of 64 produced channels; a group = GS steps of one filter fragment (128-bit LDS read, two
    // steps ahead of its use) and four MFMAs. The results of a group leave while the next group is multiplied: its
    // patch writes, patch reads and global stores sit in steps 1, 3 and 5 of the following group, so the first
    // lines of a tile are on their way to memory after a quarter of its MFMAs (the 256-channel layers are bound by
    // the rate at which the output can be written, and nothing is written while a workgroup only multiplies).
    constexpr int GS = KB * 16;
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
    // groups g0 .. g0 + NGX - 1 of one tile from the fragments a
    auto process = [&](auto ngx, int tile, int g0, const floatx4 (&a)[KB][4]) {
        constexpr int NGX = decltype(ngx)::value, STEPS = NGX * GS;
        const float *blg = bl + g0 * 64 * KS;
        auto read_b = [&](int i) {
            const int g = i / GS, r = i % GS;
            return *reinterpret_cast<const floatx4 *>(blg + (4 * g + (r & 3)) * 16 * KS + (r >> 2) * 16);
        };
        const int o_tile = __builtin_amdgcn_readfirstlane((tile * 16 * ldn + 64 * g0) * 4);   // uniform
        floatx4 bsel[NGX];
        if constexpr (NGX == NG) {
#pragma unroll
            for (int g = 0; g < NG; g++) bsel[g] = bias4[g];
        } else {
            // one group of a tile (the units behind the last multiple of eight tiles): its bias comes from memory (picked
            // out of bias4[] by g0 the compiler indexes the array, which puts it into scratch)
            bsel[0] = p.bias ? *reinterpret_cast<const floatx4 *>(p.bias + n_off + 64 * g0 + 4 * l16) : zero;
        }

        floatx4 acc[NGX][4], v[4], b[3];
        auto patch_write = [&](const floatx4 (&c)[4]) {
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
#pragma unroll
                for (int r = 0; r < 4; r++) Os[(4 * q + r) * PW_OS + 16 * jj + l16] = c[jj][r];
            __builtin_amdgcn_wave_barrier();   // LDS operations of one wavefront execute in order
        };
        auto patch_read = [&]() {
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = *reinterpret_cast<const floatx4 *>(Os + (4 * i + q) * PW_OS + 4 * l16);
            __builtin_amdgcn_wave_barrier();
        };
        auto store = [&](int g) {
#pragma unroll
            for (int i = 0; i < 4; i++)   // non-temporal stores: the output only streams out (56x56, 64 -> 256 channels: 0.0307 -> 0.0292 ms)
                buffer_store_b128_guarded<2>(v[i] + bsel[g], o_rsrc, o_lane, o_tile + (4 * i * ldn + 64 * g) * 4);
        };
        b[0] = read_b(0);
        b[1] = read_b(1);
#pragma unroll
        for (int i = 0; i < STEPS; i++) {
            const int g = i / GS, r = i % GS, jj = r & 3, kc = r >> 2;
            if (i + 2 < STEPS) b[(i + 2) % 3] = read_b(i + 2);
#pragma unroll
            for (int s = 0; s < 4; s++)
                acc[g][jj] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[kc >> 2][kc & 3][s], b[i % 3][s],
                                                                  kc == 0 && s == 0 ? zero : acc[g][jj], 0, 0, 0);
            if (g > 0 && r == 1) patch_write(acc[g - 1]);
            if (g > 0 && r == 3) patch_read();
            if (g > 0 && r == 5) store(g - 1);
            __builtin_amdgcn_sched_barrier(0);   // nothing moves between steps
        }
        patch_write(acc[NGX - 1]);
        patch_read();
        store(NGX - 1);
    };

    while (tile < t_main) {
        // draw the next tile and start its fragments on their way while this tile is multiplied (past the end:
        // the tile of this wavefront's first unit, or this tile again, unused)
        int ntile = 0;
        if (lane == 0) ntile = atomicAdd(queue, 1);
        ntile = __builtin_amdgcn_readfirstlane(ntile);
        load_a(aQ, ntile < t_main ? ntile : w < units ? unit_tile : tile);
        process(IntC<NG>{}, tile, 0, aP);
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int c = 0; c < 4; c++) aP[kb][c] = aQ[kb][c];
        tile = ntile;
    }
    if constexpr (NG > 1) {
        for (int u = w; u < units; u += 8) {
            if (u != w) load_a(aP, t_main + u / NG);   // only the first unit's fragments were requested ahead
            process(IntC<1>{}, t_main + u / NG, u % NG, aP);
        }
    } else {
        // 16 produced channels of one tile: one accumulator tile, stored straight from the MFMA layout (lane (l16, q)
        // holds pixels 4q + r of channel l16: 64 contiguous bytes of four pixel rows per store)
        for (int u = w; u < units; u += 8) {
            const int utile = t_main + u / 4, jj = u % 4;
            if (u != w) load_a(aP, utile);
            const float *blj = bl + jj * 16 * KS;
            const float bias_l = p.bias ? p.bias[n_off + 16 * jj + l16] : 0.f;
            floatx4 acc = zero, b[3];
            b[0] = *reinterpret_cast<const floatx4 *>(blj);
            b[1] = *reinterpret_cast<const floatx4 *>(blj + 16);
#pragma unroll
            for (int kc = 0; kc < KB * 4; kc++) {
                if (kc + 2 < KB * 4) b[(kc + 2) % 3] = *reinterpret_cast<const floatx4 *>(blj + (kc + 2) * 16);
#pragma unroll
                for (int s = 0; s < 4; s++)
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(aP[kc >> 2][kc & 3][s], b[kc % 3][s], acc, 0, 0, 0);
            }
            const int o_unit = __builtin_amdgcn_readfirstlane((utile * 16 * ldn + 16 * jj) * 4);
            const unsigned o_lane_q = (unsigned)(4 * q * ldn + n_off + l16) * 4u;
#pragma unroll
            for (int r = 0; r < 4; r++)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, acc[r] + bias_l), o_rsrc, o_lane_q, o_unit + r * ldn * 4, 0);
        }
    }
}

template <int NT, int KB>
static hipError_t launch_pw(hipStream_t stream, const PointwiseArgs &a, int cus)
{
    constexpr size_t lds = ((size_t)16 * NT * (64 * KB + 8) + 8 * 16 * PW_OS + 4) * sizeof(float);
    static_assert(lds <= 160 * 1024, "filter + staging must fit in LDS");
    constexpr auto kern = pointwise_kernel<NT, KB>;
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    const int nblocks = a.ldn / (16 * NT);
    int grid = cus / nblocks;                            // one workgroup per compute unit, shared among the N blocks
    if (grid < 1) grid = 1;
    if (grid * 8 > a.tiles) grid = (a.tiles + 7) / 8;   // at least 8 tiles per workgroup when there are few
    hipLaunchKernelGGL(kern, dim3(grid, nblocks), dim3(512), lds, stream, a);
    return hipGetLastError();
}

// O[m][n] = sum_k A[row(m)][k] * B(k, n) for m < M = Nimg*OH*OW, n < N. The produced channels are split into blocks
// of 256, 128 or 64 (the largest that divides N and whose filter block fits in LDS beside the staging patches); with
// more than one block A is read once per block (from L2 for the sizes this serves). Returns hipErrorNotSupported
// (nothing launched) unless K is 64, 128, 192 or 256 and N a multiple of 64; the caller then uses another kernel.
hipError_t launch_pointwise(hipStream_t stream, const float *A, const float *B, float *O, int Nimg, int AH, int AW,
                            int OH, int OW, int sh, int sw, int K, int N, int b_kmajor, const float *bias)
{
    const long Ml = (long)Nimg * OH * OW;
    if (Ml < 1 || (K & 63) || K < 64 || K > 256 || (N & 63) || N < 64) return hipErrorNotSupported;
    if ((size_t)Nimg * AH * AW * K * 4 >= (1ull << 31) || (size_t)Ml * N * 4 >= (1ull << 31)) return hipErrorNotSupported;   // buffer descriptors below 2 GB
    static int cu_count[64] = {0};   // per device; a racing first call writes the same value
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return hipErrorNotSupported;
    if (cu_count[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) return hipErrorNotSupported;
        cu_count[dev] = n;
    }
    const int cus = cu_count[dev];
    PointwiseArgs a{};
    a.A = A; a.B = B; a.O = O;
    a.M = (int)Ml; a.K = K; a.ldn = N; a.b_kmajor = b_kmajor; a.bias = bias;
    a.tiles = (a.M + 15) / 16;
    a.strided = !(sh == 1 && sw == 1 && OH == AH && OW == AW);
    a.AH = AH; a.AW = AW; a.sh = sh; a.sw = sw;
    a.a_bytes = (int)((size_t)Nimg * AH * AW * K * 4);
    a.d_OW = make_fastdiv(OW);
    a.d_OHW = make_fastdiv(OH * OW);
    const int KB = K / 64;
    if (KB == 1) {
        if (N % 256 == 0) return launch_pw<16, 1>(stream, a, cus);
        if (N % 128 == 0) return launch_pw<8, 1>(stream, a, cus);
        return launch_pw<4, 1>(stream, a, cus);
    }
    if (KB == 2) {
        if (N % 128 == 0) return launch_pw<8, 2>(stream, a, cus);
        return launch_pw<4, 2>(stream, a, cus);
    }
    if (KB == 3) return launch_pw<4, 3>(stream, a, cus);
    return launch_pw<4, 4>(stream, a, cus);
}

}  // namespace alpha
