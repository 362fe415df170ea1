// Shared declarations of the gfx950 conv kernels: launch-argument structs, exact integer
// division by launch-time constants, and the host-side launcher prototypes called by the C ABI.
#pragma once
#include "winograd_limits.hpp"
#include <hip/hip_runtime.h>
#include <atomic>
#include <stdint.h>

namespace alpha {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Unsigned division by a run-time constant d >= 1 for dividends n < 2^31:
// q = (mulhi(n, mul) + n) >> shift, exact for every such n (round-up method with a 33-bit
// multiplier whose top bit is the "+ n").
struct FastDiv {
    uint32_t mul, shift, d;
};

inline FastDiv make_fastdiv(uint32_t d)
{
    FastDiv f;
    f.d = d;
    uint32_t s = 0;
    while ((1ull << s) < d) s++;
    f.shift = s;
    f.mul = (uint32_t)(((1ull << 32) * ((1ull << s) - d)) / d + 1);
    return f;
}

__device__ __forceinline__ uint32_t fdiv(uint32_t n, const FastDiv &f)
{
    return (__umulhi(n, f.mul) + n) >> f.shift;
}

// 128-bit buffer store whose data registers may be reused at once. Measured on gfx950: a `buffer_store_dwordx4 ... offen`
// with its soffset in a scalar register, followed within two instructions by a vector instruction that writes one of its
// data registers, now and then stores the NEW value in lanes 12-15 of each group of 16 (one element in a thousand on a
// 51 MB output, different ones from run to run). The compiler guards this hazard with wait states only for stores
// WITHOUT a scalar soffset; here the two wait states follow the store explicitly, tied to the data registers so that no
// write to them can be scheduled in between.
// AUX: the instruction's cache-policy bits (16 = sc1: written through to device scope; 2 = nt: non-temporal, streamed).
template <int AUX = 0>
static __device__ __forceinline__ void buffer_store_b128_guarded(floatx4 v, __amdgpu_buffer_rsrc_t rsrc, unsigned voffset, int soffset)
{
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned, v), rsrc, voffset, soffset, AUX);
    asm volatile("s_nop 1" : "+v"(v));
}

// The same for the N low components of `v` (N = 1 to 4): a 32-, 64-, 96- or 128-bit store, with the wait states of the
// 128-bit one (the hazard was measured on the 128-bit store; the narrower ones with a scalar soffset are guarded alike).
template <int N, int AUX = 0>
static __device__ __forceinline__ void buffer_store_guarded(floatx4 v, __amdgpu_buffer_rsrc_t rsrc, unsigned voffset, int soffset)
{
    if constexpr (N == 4) {
        buffer_store_b128_guarded<AUX>(v, rsrc, voffset, soffset);
    } else if constexpr (N == 3) {
        typedef float floatx3 __attribute__((ext_vector_type(3)));
        typedef unsigned uintx3 __attribute__((ext_vector_type(3)));
        floatx3 d = floatx3{v[0], v[1], v[2]};
        __builtin_amdgcn_raw_buffer_store_b96(__builtin_bit_cast(uintx3, d), rsrc, voffset, soffset, AUX);
        asm volatile("s_nop 1" : "+v"(d));
    } else if constexpr (N == 2) {
        typedef float floatx2 __attribute__((ext_vector_type(2)));
        typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
        floatx2 d = floatx2{v[0], v[1]};
        __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(uintx2, d), rsrc, voffset, soffset, AUX);
        asm volatile("s_nop 1" : "+v"(d));
    } else {
        float d = v[0];
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, d), rsrc, voffset, soffset, AUX);
        asm volatile("s_nop 1" : "+v"(d));
    }
}

// Workgroup barrier that orders LDS accesses only: __syncthreads() also waits for every global load and store of the
// wavefront (its fences cover all address spaces), which stalls a kernel that keeps loads for later in flight.
static __device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Bumped by alpha_rt_resetDevice: a device reset drops function attributes and symbol addresses, so whatever this
// library remembers per device is only valid for the generation it was recorded in.
inline std::atomic<unsigned> &device_generation()
{
    static std::atomic<unsigned> gen{0};
    return gen;
}

// The dynamic LDS limit is a property of (kernel, device): raise it the first time a device needs more than it has.
// One instantiation, and so one table, per kernel. Each device's entry is one atomic word holding the generation it was
// recorded in together with the bytes configured, so an entry recorded before a device reset never matches afterwards,
// whichever thread looks first. A racing first call sets the same attribute twice.
template <auto KERNEL>
inline hipError_t ensure_dynamic_lds(size_t bytes)
{
    static std::atomic<uint64_t> configured[64];   // (generation << 32) | bytes; zero-initialised
    const uint64_t gen = device_generation().load(std::memory_order_acquire);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64 || bytes >= (1ull << 32)) return hipErrorInvalidDevice;
    const uint64_t have = configured[dev].load(std::memory_order_acquire);
    if ((have >> 32) != gen || bytes > (have & 0xffffffffull)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(KERNEL), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) return e;
        configured[dev].store((gen << 32) | (uint64_t)bytes, std::memory_order_release);
    }
    return hipSuccess;
}

// Compute units of the current device (0 if it cannot be read); cached per device, a racing first call writes the same value.
inline int device_cu_count()
{
    static int cu_count[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cu_count[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) return 0;
        cu_count[dev] = n;
    }
    return cu_count[dev];
}

// What happens to a result on its way to memory. Forward:
//     y = leakyRelu( A[c] * ((acc + bias[c] - mean[c]) * rsqrt(var[c] + eps)) + B[c], slope )
// i.e. the bias row-add, batch normalisation with given statistics (with or without its affine part) and the leaky
// ReLU that the reference runs as separate passes over Y (linear_dual2D_row, batchNorm2D_row / batchNorm_affined2D_row,
// leakyRelu2D: Cuda_function.java:1607, 3829, 3862). Every pointer may be NULL (that step is left out; mean and var
// go together, A and B go together); slope = 1 leaves the sign alone. Backward (gate != NULL): the result is
// multiplied by (gate[same element] > 0 ? 1 : slope), the backward of the leaky ReLU whose OUTPUT is `gate`
// (leakyRelu2D_deltaX_v1, Cuda_function.java:1640); nothing else is applied then.
struct Epilogue {
    const float *bias, *mean, *var, *A, *B;
    const float *gate;   // a tensor of the output's shape and layout
    float eps, slope;
    int fused;           // 0: only `bias` is applied (the fast path every kernel has); 1: all of the above
};

inline Epilogue bias_epilogue(const float *bias)
{
    Epilogue e{};
    e.bias = bias;
    e.slope = 1.f;
    return e;
}

// One launch of the generic implicit-GEMM "gather convolution":
//   O[o_off + n*o_sn + i*o_sh + j*o_sw + co] =
//       sum_{th<TH, tw<TW, c<AC}  A[n, i*sh - ph + th, j*sw - pw + tw, c] * B[b_off + th*b_sth + tw*b_stw + c*b_sc + co*b_sn]
// for n < N, i < OHt, j < OWt, co < CO, taps outside [0,AH)x[0,AW) contributing zero.
// GEMM view: M = N*OHt*OWt rows (pixels), CO columns, K = TH*TW*AC ordered (th, tw, c).
// Forward, stride-1 backward-data, 1x1 and each phase of kernel-split backward-data are all
// instances (see conv_api.hip). Exactly one of b_sc, b_sn is 1 (which operand axis is contiguous).
struct GatherConvArgs {
    const float *A;
    const float *B;
    float *O;
    int M, K, CO;
    int AH, AW, AC;
    int sh, sw, ph, pw;
    int a_sn;                       // AH*AW*AC
    int o_off, o_sn, o_sh, o_sw;    // output strides, elements
    int b_off, b_sth, b_stw, b_sc, b_sn;
    Epilogue ep;                    // bias / normalisation / activation applied as the rows leave for memory
    FastDiv d_AC, d_TW, d_OWt, d_OHWt;
};

hipError_t launch_gather_conv(hipStream_t stream, const GatherConvArgs &a, int TH, int TW, int OHt, int OWt, int N);

static __device__ __forceinline__ float4 add_bias4(float4 v, const float *bias, int col)
{
    if (bias) {   // uniform: one bias per output channel, added as the row leaves for memory
        const float4 b = *reinterpret_cast<const float4 *>(bias + col);
        v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
    }
    return v;
}

// per-channel constants of the forward form: y = (acc - sub) * mul + add
static __device__ __forceinline__ void ep_channel(const Epilogue &ep, int c, float &sub, float &mul, float &add)
{
    sub = ep.bias ? -ep.bias[c] : 0.f;
    mul = 1.f;
    add = 0.f;
    if (ep.mean) {
        sub += ep.mean[c];
        mul = rsqrtf(ep.var[c] + ep.eps);
    }
    if (ep.A) {
        mul *= ep.A[c];
        add = ep.B[c];
    }
}
static __device__ __forceinline__ float ep_finish(float acc, float sub, float mul, float add, float slope)
{
    const float y = (acc - sub) * mul + add;
    return y > 0.f ? y : y * slope;
}
static __device__ __forceinline__ float ep_gate(float acc, float g, float slope) { return g > 0.f ? acc : acc * slope; }

// Four consecutive channels col .. col+3 of one output pixel; `elem` = offset of that float4 in the output tensor (where
// the gate is read).
static __device__ __forceinline__ float4 epilogue4(float4 v, const Epilogue &ep, int col, size_t elem)
{
    if (!ep.fused) return add_bias4(v, ep.bias, col);
    if (ep.gate) {
        const float4 g = *reinterpret_cast<const float4 *>(ep.gate + elem);
        return make_float4(ep_gate(v.x, g.x, ep.slope), ep_gate(v.y, g.y, ep.slope), ep_gate(v.z, g.z, ep.slope), ep_gate(v.w, g.w, ep.slope));
    }
    float r[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float sub, mul, add;
        ep_channel(ep, col + j, sub, mul, add);
        r[j] = ep_finish(r[j], sub, mul, add, ep.slope);
    }
    return make_float4(r[0], r[1], r[2], r[3]);
}

// Every forward launcher takes `bias` (NULL = none): bias[co] is added to each output row in the kernel's epilogue.
// Launchers that also take `ep` apply the whole Epilogue when ep != NULL (bias is then ignored); the others are followed
// by launch_epilogue_rows, one more pass over the output.
hipError_t launch_epilogue_rows(hipStream_t s, const float *X, float *Y, const Epilogue &ep, long lengthv, int width, int stride);

// Convolution with the input window staged in LDS (tap_conv.hip, tap_conv_prefetch.hip). Filter element (th, tw, c, co)
// at b_off + th*b_sth + tw*b_stw + c*b_sc + co*b_sn; b_sn = 1 (contiguous along the output channel) fits every shape
// these kernels take, b_sn != 1 with b_sc = 1 (contiguous along the input channel) the 3x3 stride-1 ones.
// Returns hipErrorNotSupported (nothing launched) when the shape does not fit.
hipError_t launch_tap_conv(hipStream_t stream, const float *A, const float *B, float *O,
                           int N, int AH, int AW, int AC, int OH, int OW, int CO,
                           int TH, int TW, int ph, int pw,
                           int b_off, int b_sth, int b_stw, int b_sc, const float *bias = nullptr, int sh = 1, int sw = 1,
                           int b_sn = 1, const Epilogue *ep = nullptr);

// Kernel-split backward-data for stride 2 x 2, all four phases in one launch of the LDS-halo kernel (tap_conv.hip).
hipError_t launch_tap_conv_merged(hipStream_t stream, const float *A, const float *B, float *O, int N, int AH, int AW, int AC, int CO,
                                  int OHt, int OWt, const int *TH, const int *TW, const int *ph, const int *pw, const int *b_off,
                                  const int *b_sth, int b_stw, int b_sc, const int *o_off, int o_sn, int o_sh, int o_sw,
                                  const Epilogue *ep = nullptr);

// 1x1 stride-1 convolution as a streaming GEMM with the filter resident in LDS (pointwise.hip):
// O[(n,oh,ow)][co] = sum_k A[n, oh*sh, ow*sw, k] * B(k, co), B given as [K][N] (b_kmajor) or [N][K]. Returns
// hipErrorNotSupported (nothing launched) when the shape does not fit.
hipError_t launch_pointwise(hipStream_t stream, const float *A, const float *B, float *O, int Nimg, int AH, int AW,
                            int OH, int OW, int sh, int sw, int K, int N, int b_kmajor, const float *bias = nullptr);

// The same GEMM with both operands straight from memory and no LDS (pointwise_direct.hip): O[m][n] = sum_k A[m][k] * B[k][n]
// for dense rows (stride 1) and B given as [K][N]; K a multiple of 32. Applies the whole epilogue `ep` when given (else
// `bias`). Returns hipErrorNotSupported (nothing launched) when the layer does not fit.
hipError_t launch_pointwise_direct(hipStream_t stream, const float *A, const float *B, float *O, long M, int K, int N,
                                   const float *bias = nullptr, const Epilogue *ep = nullptr);
// Convolution with both operands straight from memory (any filter, stride, padding): direct_conv.hip. Filter element
// (tap = th*TW + tw, c, co) at b_off + tap*b_tap + c*b_k + co, `b_elems` floats in all. hipErrorNotSupported (nothing
// launched) when the layer does not fit. direct_conv_balanced: whether its work divides evenly enough among the
// wavefronts to beat the LDS-halo kernels on a stride-1 layer.
hipError_t launch_direct_conv(hipStream_t stream, const float *A, const float *B, float *O, int N, int AH, int AW, int AC,
                              int OHt, int OWt, int CO, int TH, int TW, int sh, int sw, int ph, int pw,
                              int b_off, int b_tap, int b_k, long b_elems, const float *bias, const Epilogue *ep,
                              float *ws = nullptr, size_t ws_bytes = 0, unsigned *tickets = nullptr, int n_tickets = 0);
bool direct_conv_balanced(long M, int CO, bool workspace = false);
// Backward-data of a 1x1 layer whose stride exceeds the filter (no padding, IH = sh*OH, IW = sw*OW): the product into every
// sh x sw block's first pixel, zeros elsewhere (pointwise_scatter.hip). W is [K = OC][N = IC]. hipErrorNotSupported: nothing launched.
hipError_t launch_pointwise_scatter(hipStream_t stream, const float *dY, const float *W, float *dX, int Nimg, int OH, int OW,
                                    int K, int N, int sh, int sw);
// Kernel-split backward-data, up to four phases over the same coarse pixels in one launch, both operands straight from
// memory: direct_conv_phased.hip. Phase f: O[o_off[f] + n*o_sn + i*o_sh + j*o_sw + co] = sum A[n, i - ph[f] + th,
// j - pw[f] + tw, c] * B[b_off[f] + th*b_sth[f] + tw*b_stw + c*b_k + co]. hipErrorNotSupported: nothing launched.
// `sharing`: -1 = by shape, 0 = every wavefront its own items, 1 = a workgroup's wavefronts share every group of items.
hipError_t launch_direct_conv_phased(hipStream_t stream, const float *A, const float *B, float *O, int N, int AH, int AW, int AC, int CO,
                                     int OHt, int OWt, int nph, const int *TH, const int *TW, const int *ph, const int *pw,
                                     const int *b_off, const int *b_sth, int b_stw, int b_k, long b_elems,
                                     const int *o_off, int o_sn, int o_sh, int o_sw, long o_elems, const Epilogue *ep, int sharing = -1);
// Backward-data for 4 stored input channels and strides of 1 or 2 (network stems), filter W[OC,FH,FW,4] in place:
// delta_x_stem.hip. hipErrorNotSupported (nothing launched) when the layer does not fit.
hipError_t launch_delta_x_stem(hipStream_t stream, const float *dY, const float *W, float *dX, int N, int IH, int IW, int IC,
                               int OH, int OW, int OC, int FH, int FW, int sh, int sw, int ph, int pw, const Epilogue *ep);

// Backward-filter implicit GEMM with split-K over k = (n, oh, ow):
//   dst_z[oc, fh, fw, ic] = sum_{k in slice z} deltaY[k, oc] * X[n, oh*sh - ph + fh, ow*sw - pw + fw, ic]
// slice z = [z*GK_slice, (z+1)*GK_slice), the last one running to GK; dst_0 = deltaW,
// dst_z = deltaW_buf + (z-1)*sizeW.
struct DeltaWArgs {
    const float *X;
    const float *dY;
    float *dW;
    float *dW_buf;
    int IH, IW, IC, OH, OW, OC, FW;
    int sh, sw, ph, pw;
    int GM;        // FH*FW*IC   (columns)
    int GK, GK_slice, GZ;
    FastDiv d_IC, d_FW, d_OW, d_OHW;
};

hipError_t launch_deltaW(hipStream_t stream, const DeltaWArgs &a);

// Row-streaming backward-filter for stride-1 3x3 and 1x1 layers (delta_w_rows.hip); same split-K contract as
// launch_deltaW. Returns hipErrorNotSupported (nothing launched) when the layer does not fit.
hipError_t launch_deltaW_rows(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                              int N, int IH, int IW, int IC, int OH, int OW, int OC, int FH, int FW,
                              int sh, int sw, int ph, int pw, int GK_slice, int GZ, float *dB = nullptr, float *dB_buf = nullptr);

// Backward-filter with the reduction dealt out evenly to one persistent workgroup per compute unit (delta_w_stream.hip):
// deltaW and the GZ - 1 buffers add up to the result, but which pixels go into which buffer is the kernel's choice (an
// item's pieces in order; buffers beyond them are zero-filled). Returns hipErrorNotSupported (nothing launched) when GZ
// is 1 or too small for the pieces of an item.
hipError_t launch_deltaW_stream(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                                int N, int IH, int IW, int IC, int OH, int OW, int OC, int FH, int FW,
                                int sh, int sw, int ph, int pw, int GZ);
int deltaW_stream_least_GridZ(int units, int N, int OH, int OW, int IC, int OC, int FH, int FW, int GZ);
int deltaW_stream_block_fill(int IC, int OC);
void deltaW_stream_set_units(int units);   // -1 by shape, 0 never, 1 wherever the buffers allow: whole units instead of the line of items
int deltaW_stream_fill_GridZ(int units, int N, int OH, int OW, int IC, int OC, int FH, int FW, int GZ, int GZ_cap);

// Backward-filter with the filter tap in the grid and both operands straight from memory (delta_w_taps.hip): any filter,
// stride and padding; same slice partition and outputs. Returns hipErrorNotSupported (nothing launched) when it does not fit.
hipError_t launch_deltaW_taps(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                              int N, int IH, int IW, int IC, int OH, int OW, int OC, int FH, int FW,
                              int sh, int sw, int ph, int pw, int GK_slice, int GZ);

// Winograd F(2x2,3x3) forward (winograd.hip): U = transformed filter [16][IC][OC].
// Forward convolution for IC (stored) = 4 with the filter resident in LDS (stem_conv.hip); F is W[OC,FH,FW,4] or, with
// f_cw, CW[FH,FW,4,OC]. Returns hipErrorNotSupported (nothing launched) when the layer does not fit.
hipError_t launch_stem_conv(hipStream_t stream, const float *X, const float *F, int f_cw, float *Y,
                            int N, int IH, int IW, int IC, int OH, int OW, int OC, int FH, int FW, int sh, int sw, int ph, int pw,
                            const float *bias = nullptr, const Epilogue *ep = nullptr);

// The same layers with both operands straight from memory (stem_direct.hip): W[OC,FH,FW,4] in place. Returns
// hipErrorNotSupported (nothing launched) for filters other than 3x3 and 7x7.
hipError_t launch_stem_direct(hipStream_t stream, const float *X, const float *W, float *Y, int N, int IH, int IW, int OH, int OW,
                              int OC, int FH, int FW, int sh, int sw, int ph, int pw, const float *bias, const Epilogue *ep);

// Backward-filter of 1x1 stride-1 layers from registers (delta_w_pointwise.hip); same slice partition and outputs.
// Returns hipErrorNotSupported (nothing launched) unless IC and OC are multiples of 64.
hipError_t launch_deltaW_pointwise(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                                   int GK, int IC, int OC, int GK_slice, int GZ, float *dB = nullptr, float *dB_buf = nullptr);

// winograd_grouped_filter(IC) and the size limits of the Winograd kernels: winograd_limits.hpp
// backward: the filter of backward-data as a forward convolution of deltaY (OC reduced, IC produced, taps rotated);
// launch_winograd(deltaY, U, deltaX, N, OH, OW, OC, IH, IW, IC, 2 - ph, 2 - pw) then computes deltaX.
hipError_t launch_winograd_filter(hipStream_t s, const float *W, float *U, int IC, int OC, bool backward = false);
hipError_t launch_winograd(hipStream_t stream, const float *X, const float *U, float *Y,
                           int N, int IH, int IW, int IC, int OH, int OW, int OC, int ph, int pw, const float *bias = nullptr,
                           const Epilogue *ep = nullptr);
// The same as one MFMA stream per persistent workgroup (winograd_stream.hip), for IC % 16 == 0; returns
// hipErrorNotSupported (nothing launched) otherwise.
hipError_t launch_winograd_stream(hipStream_t stream, const float *X, const float *U, float *Y,
                                  int N, int IH, int IW, int IC, int OH, int OW, int OC, int ph, int pw, const float *bias = nullptr);

// Backward-filter of 3x3 stride-1 layers by Winograd F(3x3,2x2) (winograd_dw.hip); slice z (a range of 2x2 output tiles)
// -> deltaW or deltaW_buf[z-1]. Returns hipErrorNotSupported (nothing launched) when the layer does not fit.
hipError_t launch_deltaW_winograd(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                                  int N, int IH, int IW, int IC, int OH, int OW, int OC, int ph, int pw, int GZ);

// Re-layout / reduction helpers.
hipError_t launch_kernel_remode(hipStream_t s, const float *W, float *CW, int FH, int FW, int OC, int IC);
hipError_t launch_ks_remode(hipStream_t s, int version, const float *W, int FH, int FW, float *CW,
                            int mCFH, int mCFW, int OC, int IC, int sh, int sw);
hipError_t launch_buf_summary(hipStream_t s, const float *buf, float *dW, int part, int sizeW);
// Column sums of deltaY[GK][OC] per K slice (bias gradient), same slice partition and destinations as backward-filter.
// Backward-filter for 4 stored input channels (delta_w_stem.hip): its own equal cut of the pixels into GridZ slices,
// slice 0 to deltaW, slice z to deltaW_buf[z - 1]. hipErrorNotSupported: nothing launched.
hipError_t launch_deltaW_stem(hipStream_t stream, const float *X, const float *dY, float *dW, float *dW_buf,
                              int N, int IH, int IW, int OH, int OW, int OC, int FH, int FW, int sh, int sw, int ph, int pw, int GZ);
hipError_t launch_col_sum(hipStream_t s, const float *dY, float *dB, float *dB_buf, int OC, int GK, int GK_slice, int GZ);

// Backward of batch normalisation (batchnorm_backward.hip). form: 0 = X_norm given in S, 1 = X_norm = (S - B) / A,
// 2 = X_norm = (S - mean) * rsqrt(var + eps). Field sums: deltaA = sum_n deltaY * X_norm, deltaB = sum_n deltaY per column.
int bn_field_nextN(int N, int M);
hipError_t launch_bn_field_sums(hipStream_t s, int form, const float *dY, const float *S, const float *mean, const float *var, float eps,
                                const float *A, const float *B, int N, int M, float *bufA, float *outA, float *bufB, float *outB, int width);
hipError_t launch_bn_delta_x(hipStream_t s, int form, bool affine, const float *dY, const float *S, const float *mean, const float *var,
                             float eps, const float *A, const float *B, const float *p1, const float *p2, int row_lengthv, float *dX,
                             long lengthv, int width);

}  // namespace alpha
