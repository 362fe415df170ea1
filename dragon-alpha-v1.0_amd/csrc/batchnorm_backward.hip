// Backward of batch normalisation over a [N rows, M = row_lengthv] tensor (rows = pixels of the batch, columns = channels;
// a row has `width` data elements and M - width pad elements kept at zero), HBM-bound, 128-bit accesses, gfx950.
// The training step of the reference's conv -> batch-norm -> leaky-ReLU blocks runs these between leakyRelu2D_deltaX and
// dconv3D_deltaX:
//   field sums   deltaB[m] = deltaXp1[m] = sum_n deltaY[n, m]
//                deltaA[m] = deltaXp2[m] = sum_n deltaY[n, m] * X_norm[n, m]
//       (Cuda_reduce.field_affine_deltaAB_v1 / _v2, field_batchNorm_deltaAB_v2: Cuda_reduce.java:697, 746, 939)
//   row function deltaX[n, m] = scale[m] * (deltaY[n, m] - (deltaXp1[m] + deltaXp2[m] * X_norm[n, m]) / N)
//       (Cuda_function.batchNorm2D_row_deltaX_v1 / _v2, batchNorm_affined2D_row_deltaX_v1 / _v2: Cuda_function.java:3890,
//        3923, 3958, 3992), scale = rsqrt(X_var + eps), times A for the affine forms
// where X_norm is, by form:  Y (v1: the layer kept its output),  (Y - B) / A (v1 affine),  (X - X_mean) * rsqrt(X_var + eps)
// (v2: the layer kept its input).
//
// The field sums run in two launches, both deterministic: workgroups of 16 x 16 threads sum a chunk of rows for 64
// columns (each thread its rows in order, the 16 partial sums added through LDS in the order 0..15) into parts[chunk][M],
// then the chunks are added by a second, small kernel (64 lanes per column, fixed order). The caller's buffers (deltaA_buf, deltaB_buf: nextN x M floats each, nextN as
// the reference's field_nextN) hold the chunk sums; a result may alias the head of its buffer, as the Java engine passes
// them (CudaFloat32EngineBase.java:4396-4409).
#include "common.hpp"

namespace alpha {

enum BnForm { BN_NORM_GIVEN = 0, BN_FROM_Y_AFFINE = 1, BN_FROM_X = 2 };

struct BnArgs {
    const float *dY;
    const float *S;        // Y (forms 0, 1) or X (form 2)
    const float *mean, *var, *A, *B;
    float eps;
    int N, M, width;
};

template <int FORM>
__device__ __forceinline__ void bn_column_terms(const BnArgs &p, int c, float4 &sub, float4 &mul)
{
    // X_norm = (S - sub) * mul
    sub = make_float4(0.f, 0.f, 0.f, 0.f);
    mul = make_float4(1.f, 1.f, 1.f, 1.f);
    if (FORM == BN_FROM_Y_AFFINE) {
        const float4 a = *reinterpret_cast<const float4 *>(p.A + c);
        sub = *reinterpret_cast<const float4 *>(p.B + c);
        mul = make_float4(1.f / a.x, 1.f / a.y, 1.f / a.z, 1.f / a.w);
    } else if (FORM == BN_FROM_X) {
        const float4 v = *reinterpret_cast<const float4 *>(p.var + c);
        sub = *reinterpret_cast<const float4 *>(p.mean + c);
        mul = make_float4(rsqrtf(v.x + p.eps), rsqrtf(v.y + p.eps), rsqrtf(v.z + p.eps), rsqrtf(v.w + p.eps));
    }
}

// partsA / partsB [chunks][M]: the sums over rows [chunk * rows_per_chunk, ...) of deltaY * X_norm and of deltaY.
template <int FORM>
__global__ __launch_bounds__(256) void bn_field_sums_kernel(const BnArgs p, float *__restrict__ partsA, float *__restrict__ partsB,
                                                            int rows_per_chunk)
{
    __shared__ float4 redA[16][17], redB[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int c = (blockIdx.x * 16 + tx) * 4;
    const int chunk = blockIdx.y;
    const long r0 = (long)chunk * rows_per_chunk;
    const long r1 = r0 + rows_per_chunk < p.N ? r0 + rows_per_chunk : p.N;
    float4 sa = make_float4(0.f, 0.f, 0.f, 0.f), sb = sa;
    if (c < p.M) {
        float4 sub, mul;
        bn_column_terms<FORM>(p, c, sub, mul);
        for (long r = r0 + ty; r < r1; r += 16) {
            const float4 dy = *reinterpret_cast<const float4 *>(p.dY + r * p.M + c);
            const float4 s = *reinterpret_cast<const float4 *>(p.S + r * p.M + c);
            sa.x += dy.x * ((s.x - sub.x) * mul.x); sa.y += dy.y * ((s.y - sub.y) * mul.y);
            sa.z += dy.z * ((s.z - sub.z) * mul.z); sa.w += dy.w * ((s.w - sub.w) * mul.w);
            sb.x += dy.x; sb.y += dy.y; sb.z += dy.z; sb.w += dy.w;
        }
    }
    redA[ty][tx] = sa;
    redB[ty][tx] = sb;
    __syncthreads();
    if (ty < 2 && c < p.M) {   // ty 0 adds the sixteen partial sums of A in order, ty 1 those of B
        float4(*red)[17] = ty == 0 ? redA : redB;
        float4 v = red[0][tx];
        for (int k = 1; k < 16; k++) { v.x += red[k][tx].x; v.y += red[k][tx].y; v.z += red[k][tx].z; v.w += red[k][tx].w; }
        const float e[4] = {v.x, v.y, v.z, v.w};
        float o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = c + j < p.width ? e[j] : 0.f;   // pad columns stay zero
        float *dst = (ty == 0 ? partsA : partsB) + (size_t)chunk * p.M + c;
        *reinterpret_cast<float4 *>(dst) = make_float4(o[0], o[1], o[2], o[3]);
    }
}

// out[m] = sum over chunks of parts[chunk][m]: 64 lanes per column take chunks k, k + 64, ... in order (their loads are all
// in flight at once), then the 64 sums are added in the order 0..63. `out` may alias parts[0]: a workgroup reads all of
// its columns' parts before it writes, and no other workgroup touches them.
__global__ __launch_bounds__(1024) void bn_sum_parts_kernel(const float *partsA, const float *partsB, float *outA, float *outB, int chunks, int M)
{
    __shared__ float4 red[64][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int c = (blockIdx.x * 16 + tx) * 4;
    const float *parts = blockIdx.y == 0 ? partsA : partsB;
    float *out = blockIdx.y == 0 ? outA : outB;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (c < M)
        for (int k = ty; k < chunks; k += 64) {
            const float4 v = *reinterpret_cast<const float4 *>(parts + (size_t)k * M + c);
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
    red[ty][tx] = s;
    __syncthreads();
    if (ty == 0 && c < M) {
        float4 v = red[0][tx];
        for (int k = 1; k < 64; k++) { v.x += red[k][tx].x; v.y += red[k][tx].y; v.z += red[k][tx].z; v.w += red[k][tx].w; }
        *reinterpret_cast<float4 *>(out + c) = v;
    }
}

// deltaX = scale * (deltaY - rN * (p1 + p2 * X_norm)), pad columns and (affine form from Y: A == 0) NaN results zero.
template <int FORM, bool AFFINE>
__global__ __launch_bounds__(256) void bn_delta_x_kernel(const BnArgs p, const float *__restrict__ p1, const float *__restrict__ p2,
                                                         float *__restrict__ dX, long quads, float rN)
{
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < quads; i += (long)gridDim.x * 256) {
        const int c = (int)((4 * i) % p.M);
        const float4 dy4 = *reinterpret_cast<const float4 *>(p.dY + 4 * i);
        const float4 s4 = *reinterpret_cast<const float4 *>(p.S + 4 * i);
        const float4 v4 = *reinterpret_cast<const float4 *>(p.var + c);
        const float4 q1 = *reinterpret_cast<const float4 *>(p1 + c);
        const float4 q2 = *reinterpret_cast<const float4 *>(p2 + c);
        float4 sub, mul;
        bn_column_terms<FORM>(p, c, sub, mul);
        float4 a4 = make_float4(1.f, 1.f, 1.f, 1.f);
        if (AFFINE) a4 = *reinterpret_cast<const float4 *>(p.A + c);
        const float dy[4] = {dy4.x, dy4.y, dy4.z, dy4.w}, s[4] = {s4.x, s4.y, s4.z, s4.w}, var[4] = {v4.x, v4.y, v4.z, v4.w};
        const float d1[4] = {q1.x, q1.y, q1.z, q1.w}, d2[4] = {q2.x, q2.y, q2.z, q2.w};
        const float sb[4] = {sub.x, sub.y, sub.z, sub.w}, ml[4] = {mul.x, mul.y, mul.z, mul.w}, a[4] = {a4.x, a4.y, a4.z, a4.w};
        float r[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float rstd = rsqrtf(var[j] + p.eps);
            const float xn = FORM == BN_FROM_Y_AFFINE ? (s[j] - sb[j]) / a[j] : (s[j] - sb[j]) * ml[j];
            const float scale = AFFINE ? a[j] * rstd : rstd;
            float v = scale * (dy[j] - rN * (d1[j] + d2[j] * xn));
            if (c + j >= p.width || v != v) v = 0.f;
            r[j] = v;
        }
        // streamed out (non-temporal store: 0.0328 -> 0.0321 ms on 200704 x 64; non-temporal loads of the two inputs cost 6 %)
        __builtin_nontemporal_store(floatx4{r[0], r[1], r[2], r[3]}, reinterpret_cast<floatx4 *>(dX + 4 * i));
    }
}

// The reference's Cuda_reduce.field_nextN (Cuda_reduce.java:35-45): rows left after one stage of its field reductions;
// the caller's buffers hold field_nextN(N, M) x M floats.
int bn_field_nextN(int N, int M)
{
    if (M > 15) {
        if (N > 63) return N >> 6;
        if (N > 15) return 1;
    }
    if (M > 7) {
        if (N > 127) return N >> 7;
        if (N > 31) return 1;
    }
    return (N + 63) >> 6;
}

// form: 0 = X_norm given in S (field_affine_deltaAB_v2), 1 = X_norm = (S - B) / A (field_affine_deltaAB_v1),
// 2 = X_norm = (S - mean) * rsqrt(var + eps) (field_batchNorm_deltaAB_v2). Buffers may be NULL when field_nextN(N, M) is 1.
hipError_t launch_bn_field_sums(hipStream_t s, int form, const float *dY, const float *S, const float *mean, const float *var, float eps,
                                const float *A, const float *B, int N, int M, float *bufA, float *outA, float *bufB, float *outB, int width)
{
    if (N < 1 || M < 4 || (M & 3) || width < 1 || width > M) return hipErrorInvalidValue;
    BnArgs p{dY, S, mean, var, A, B, eps, N, M, width};
    const int col_tiles = (M / 4 + 15) / 16;
    const int capacity = bn_field_nextN(N, M);   // chunks the buffers can hold
    int chunks = 1;
    if (capacity > 1 && bufA && bufB) {
        // two workgroups per compute unit, whatever the channel count: more chunks only lengthen the second kernel's sums
        // (200704 x 64: operator 0.0623 ms with 2048 chunks, 0.0572 with 1024, 0.0544 with 512, 0.0556 with 256)
        const int cus = device_cu_count();
        chunks = (2 * (cus > 0 ? cus : 256) + col_tiles - 1) / col_tiles;
        if (chunks > capacity) chunks = capacity;
        if (chunks > (N + 15) / 16) chunks = (N + 15) / 16;     // sixteen rows per chunk at least
    }
    const int rows_per_chunk = (N + chunks - 1) / chunks;
    chunks = (N + rows_per_chunk - 1) / rows_per_chunk;
    float *pa = chunks > 1 ? bufA : outA, *pb = chunks > 1 ? bufB : outB;
    const dim3 grid(col_tiles, chunks);
    if (form == BN_NORM_GIVEN) hipLaunchKernelGGL(bn_field_sums_kernel<BN_NORM_GIVEN>, grid, dim3(256), 0, s, p, pa, pb, rows_per_chunk);
    else if (form == BN_FROM_Y_AFFINE) hipLaunchKernelGGL(bn_field_sums_kernel<BN_FROM_Y_AFFINE>, grid, dim3(256), 0, s, p, pa, pb, rows_per_chunk);
    else hipLaunchKernelGGL(bn_field_sums_kernel<BN_FROM_X>, grid, dim3(256), 0, s, p, pa, pb, rows_per_chunk);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    if (chunks > 1) {
        hipLaunchKernelGGL(bn_sum_parts_kernel, dim3(col_tiles, 2), dim3(1024), 0, s, bufA, bufB, outA, outB, chunks, M);
        return hipGetLastError();
    }
    return hipSuccess;
}

hipError_t launch_bn_delta_x(hipStream_t s, int form, bool affine, const float *dY, const float *S, const float *mean, const float *var,
                             float eps, const float *A, const float *B, const float *p1, const float *p2, int row_lengthv, float *dX,
                             long lengthv, int width)
{
    const int M = row_lengthv;
    if (lengthv <= 0) return hipSuccess;
    if (M < 4 || (M & 3) || width < 1 || width > M || lengthv % M != 0) return hipErrorInvalidValue;
    BnArgs p{dY, S, mean, var, A, B, eps, (int)(lengthv / M), M, width};
    const float rN = (1.0f * row_lengthv) / (float)lengthv;   // as the reference computes 1 / N
    const long quads = lengthv / 4;
    long blocks = (quads + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    const dim3 grid((unsigned)blocks);
    if (form == BN_NORM_GIVEN) hipLaunchKernelGGL((bn_delta_x_kernel<BN_NORM_GIVEN, false>), grid, dim3(256), 0, s, p, p1, p2, dX, quads, rN);
    else if (form == BN_FROM_Y_AFFINE) hipLaunchKernelGGL((bn_delta_x_kernel<BN_FROM_Y_AFFINE, true>), grid, dim3(256), 0, s, p, p1, p2, dX, quads, rN);
    else if (affine) hipLaunchKernelGGL((bn_delta_x_kernel<BN_FROM_X, true>), grid, dim3(256), 0, s, p, p1, p2, dX, quads, rN);
    else hipLaunchKernelGGL((bn_delta_x_kernel<BN_FROM_X, false>), grid, dim3(256), 0, s, p, p1, p2, dX, quads, rN);
    return hipGetLastError();
}

}  // namespace alpha
