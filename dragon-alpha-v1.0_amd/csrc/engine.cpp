// Host-side counterpart of the reference's CudaFloat32EngineBase convolution section
// (src/alpha_src/z/dragon/engine/cuda/CudaFloat32EngineBase.java:1323-2005): which native entry is
// called for a layer, with how many stream handles, which split-K factor and which scratch buffers.
// The reference does this in Java above the JNI boundary; there is no JVM here, so the same integer
// decisions are restated in C++ and exported through the C ABI (alpha_plan_* are pure functions,
// alpha_engine_* additionally own the scratch memory the Java engine would take from its pool and
// then call the natives exactly as the Java code does).
#include "../../include/alpha_conv.h"
#include "../../include/alpha_engine.h"
#include "winograd_limits.hpp"

namespace alpha {
// delta_w_stream.hip (host code): the least split-K factor with which the persistent backward-filter kernel cuts a layer as it does with GZ
int deltaW_stream_least_GridZ(int units, int N, int OH, int OW, int IC, int OC, int FH, int FW, int GZ);
int deltaW_stream_fill_GridZ(int units, int N, int OH, int OW, int IC, int OC, int FH, int FW, int GZ, int GZ_cap);
}

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <map>
#include <tuple>
#include <mutex>
#include <vector>

namespace {

// Tiles of the reference's power-of-two strip decomposition of one GEMM extent: whole 128-wide
// tiles, then one strip for every set bit 64, 32, 16, 8 and one for a remainder of 4..7
// (Cuda_conv3D.java:19-41 and its twins in the deltaX / deltaW classes).
int strips_tiles(int g) { return (g >> 7) + __builtin_popcount(g & 0x7C); }

// Kernel launches (= streams wanted) along one extent: 1 for a power of two, else one per strip
// (Cuda_conv3D.java:70-97).
int strips_streams(int g)
{
    if ((g & (g - 1)) == 0) return 1;
    return (g > 127 ? 1 : 0) + __builtin_popcount(g & 0x7C);
}

int stream_count(int gn, int gm, int cap) { return std::min(strips_streams(gn) * strips_streams(gm), cap); }

}  // namespace

extern "C" {
#pragma GCC visibility push(default)

int alpha_blockNum(int GN, int GM) { return strips_tiles(GN) * strips_tiles(GM); }
int alpha_streamSize(int GN, int GM, int cap) { return stream_count(GN, GM, cap); }

double alpha_paddingScaleUp(int IH, int IW, int OH, int OW, int FH, int FW, int sh, int sw)
{
    // Cuda_conv3D.java:129-135
    return 1.0 * (((OH - 1) * sh + FH) * ((OW - 1) * sw + FW)) / (IH * IW);
}

void alpha_engine_config_default(alpha_engine_config *c, int compute_units)
{
    // CudaFloat32EngineBase.java:1324-1352, 1630-1663, 1765-1793 and :73 (MaxPartNum = clip(#SM, 16, 128))
    c->conv3D_useTexture = 1;
    c->conv3D_remode = 1;
    c->conv3D_remode_V2_Q = 1.05f;
    c->conv3D_V2_Q = 1.25f;
    c->deltaW_SplitKThreshold = 512;
    c->deltaW_SK_MaxPartNum = std::max(16, std::min(128, compute_units));
    c->deltaW_SK_V2_Q = 1.15f;
    c->deltaX_s1_useTexture = 1;
    c->deltaX_ks_useTexture = 0;
    c->deltaX_s1_V2_Q = 1.1f;
    c->deltaX_ks_V2_Q = 1.1f;
    c->conv3D_winograd = 0;
    c->deltaX_winograd = 0;
    c->deltaW_winograd = 0;
    c->deltaW_SK_fillUnits = 0;
    c->deltaW_SK_leastUnits = 0;
    c->conv_workspace = 0;
    c->cache_filter_transforms = 0;
}

// ---- forward: CudaFloat32EngineBase.conv3D (:1355-1474) ----------------------------------------------
void alpha_plan_conv3D(const alpha_engine_config *c, int IH, int IW, int OH, int OW, int FH, int FW, int N, int IC, int OC,
                       int sh, int sw, int ph, int pw, alpha_conv_plan *out)
{
    memset(out, 0, sizeof(*out));
    const double Q = alpha_paddingScaleUp(IH, IW, OH, OW, FH, FW, sh, sw);
    out->Q = Q;
    // a layer beyond the Winograd kernels' 32-bit offsets stays on the entries below
    // (and so does one whose output is smaller than the formula's, which the engine's check allows and the kernels do not take)
    if (c->conv3D_winograd && FH == 3 && FW == 3 && sh == 1 && sw == 1 && OH == IH + 2 * ph - 2 && OW == IW + 2 * pw - 2 &&
        alpha::winograd_forward_fits(N, IH, IW, IC, OH, OW, OC)) {
        out->entry = ALPHA_E_conv3D_winograd;
        out->remode = 1;   // the filter transform takes the place of kernel_remode
        out->streams = 1;
        out->scratch_floats = 16L * IC * OC;
        return;
    }
    if (c->conv3D_remode && OC > 31 && N * OH * OW > 31) {
        const bool V2 = N > 63 && OC > 63 && Q > c->conv3D_remode_V2_Q;
        out->remode = 1;
        out->V2 = V2;
        out->streams = V2 ? stream_count(OC, N, 10) : stream_count(OC, N * OH * OW, 10);
        out->useTexture = c->conv3D_useTexture;
        // The W1 natives carry no stride or padding (1x1, stride 1, pad 0). The Java engine can send every 1x1 layer
        // there because its argument check refuses sh > FH (EngineCore.java:650-651); this host layer also serves
        // strided 1x1 layers, through the general entries.
        const bool w1 = FH == 1 && FW == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0;
        if (w1) out->entry = ALPHA_E_conv3D_GemmR_W1;
        else if (V2) out->entry = ALPHA_E_conv3D_GemmV2R;
        else if (c->conv3D_useTexture) out->entry = ALPHA_E_conv3D_GemmR_texture;
        else out->entry = ALPHA_E_conv3D_GemmR;
        out->scratch_floats = (long)FH * FW * IC * OC;
    } else {
        const bool V2 = N > 127 && OC > 127 && Q >= c->conv3D_V2_Q;
        out->V2 = V2;
        out->streams = V2 ? stream_count(OC, N, 10) : stream_count(OC, N * OH * OW, 10);
        out->useTexture = c->conv3D_useTexture && OC > 15;
        if (FH == 1 && FW == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0) out->entry = ALPHA_E_conv3D_W1;
        else if (ph == 0 && pw == 0) out->entry = ALPHA_E_conv3D_np;
        else if (V2) out->entry = ALPHA_E_conv3DV2;
        else if (out->useTexture) out->entry = ALPHA_E_conv3D_texture;
        else out->entry = ALPHA_E_conv3D;
    }
}

// ---- backward-filter: CudaFloat32EngineBase.dconv3D_deltaW (:1666-1762) ------------------------------------
void alpha_plan_deltaW(const alpha_engine_config *c, int IH, int IW, int OH, int OW, int FH, int FW, int N, int IC, int OC,
                       int sh, int sw, alpha_conv_plan *out)
{
    memset(out, 0, sizeof(*out));
    const int GK = N * OH * OW;
    const double Q = alpha_paddingScaleUp(IH, IW, OH, OW, FH, FW, sh, sw);
    out->Q = Q;
    if (GK < c->deltaW_SplitKThreshold) {
        out->streams = stream_count(OC, FH * FW * IC, 12);
        out->GridZ = 1;
        out->entry = (FH == 1 && FW == 1 && sh == 1 && sw == 1) ? ALPHA_E_dconv3D_deltaW_W1 : ALPHA_E_dconv3D_deltaW;
        return;
    }
    const bool V2 = OC > 63 && IC > 63 && Q >= c->deltaW_SK_V2_Q;
    out->V2 = V2;
    out->streams = V2 ? stream_count(OC, IC, 12) : stream_count(OC, FH * FW * IC, 12);
    // tile counts of forward, backward-data and backward-filter (Cuda_conv3D.blockNum[V2] and twins)
    const int b1 = V2 ? strips_tiles(OC) * strips_tiles(N) * OH * OW : strips_tiles(OC) * strips_tiles(N * OH * OW);
    const int b2 = V2 ? strips_tiles(IC) * strips_tiles(N) * IH * IW : strips_tiles(IC) * strips_tiles(N * IH * IW);
    const int b3 = V2 ? strips_tiles(OC) * strips_tiles(IC) * FH * FW : strips_tiles(OC) * strips_tiles(FH * FW * IC);
    int GridZ = (b1 + b2) / (b3 << 1);
    if (GridZ < 2) GridZ = 2;
    if (GridZ > c->deltaW_SK_MaxPartNum) GridZ = c->deltaW_SK_MaxPartNum;
    const int GridZ2 = GK >> 8;
    if (GridZ > GridZ2) GridZ = GridZ2;
    if (c->deltaW_SK_fillUnits > 0) {
        // The reference sizes GridZ for GPUs of at most 128 SMs; on a wider device a layer with few filter tiles leaves
        // compute units idle. One workgroup of the backward-filter kernels covers 64 input channels x 32 output
        // channels (64 for 1x1 filters) of one K slice.
        const int ocb = (FH == 1 && FW == 1) ? 64 : 32;
        const int tiles = ((IC + 63) / 64) * ((OC + ocb - 1) / ocb);
        // rows of up to 36 pixels leave LDS for two co-resident workgroups per compute unit; wider rows for one
        const int per_unit = (OW <= 36) ? 2 : 1;
        int want = (per_unit * c->deltaW_SK_fillUnits + tiles - 1) / tiles;
        if (want > GridZ2) want = GridZ2;
        if (want > GridZ) GridZ = want;
    }
    const bool winograd = c->deltaW_winograd && FH == 3 && FW == 3 && sh == 1 && sw == 1 &&
                          alpha::winograd_deltaW_fits(N, IH, IW, IC, OH, OW, OC);
    if (winograd && c->deltaW_winograd > 1) {
        // One workgroup of the Winograd kernel covers 32 input x 64 output channels of one slice of tiles and has a
        // compute unit to itself: values above 1 are the number of compute units to fill (slices of at least 64 tiles).
        const int tiles = ((IC + 31) / 32) * ((OC + 63) / 64);
        int want = (c->deltaW_winograd + tiles - 1) / tiles;
        const int most = N * ((OH + 1) / 2) * ((OW + 1) / 2) / 64;
        if (want > most) want = most;
        if (want < 1) want = 1;
        GridZ = want;
    }
    if (c->deltaW_SK_leastUnits > 0 && !winograd)
        GridZ = alpha::deltaW_stream_fill_GridZ(c->deltaW_SK_leastUnits, N, OH, OW, IC, OC, FH, FW, GridZ, GridZ2);
    if (c->deltaW_SK_leastUnits > 0 && IC == 4 && FH * FW <= 128) {
        // 4 stored input channels: the kernel of delta_w_stem.hip runs GridZ x (groups of 16 taps) x (blocks of 64 output
        // channels) workgroups at most; a 3x3 first layer at the reference's 128 fills half of 256 compute units
        const int per_slice = ((FH * FW + 15) / 16) * ((OC + 63) / 64);
        int want = c->deltaW_SK_leastUnits / per_slice;   // rounded down: one workgroup more than compute units is a second round
        if (want > GridZ2) want = GridZ2;
        if (want > GridZ) GridZ = want;
    }
    out->GridZ = GridZ;
    out->scratch_floats = (long)OC * FH * FW * IC * (GridZ - 1);
    if (winograd) {
        out->entry = ALPHA_E_dconv3D_deltaW_GemmSK_winograd;
        out->streams = 1;
        return;
    }
    if (FH == 1 && FW == 1 && sh == 1 && sw == 1) out->entry = ALPHA_E_dconv3D_deltaW_GemmSK_W1;   // W1 natives: stride 1 only
    else if (V2) out->entry = ALPHA_E_dconv3D_deltaW_GemmV2SK;
    else out->entry = ALPHA_E_dconv3D_deltaW_GemmSK;
}

// ---- backward-data: CudaFloat32EngineBase.dconv3D_deltaX (:1796-2005) ---------------------------------------
void alpha_plan_deltaX(const alpha_engine_config *c, int IH, int IW, int OH, int OW, int FH, int FW, int N, int IC, int OC,
                       int sh, int sw, alpha_conv_plan *out)
{
    memset(out, 0, sizeof(*out));
    if (IC <= 8 || (IC <= 16 && sh * sw >= 4)) {
        out->entry = ALPHA_E_dconv3D_deltaX_crossAdd;
        out->streams = stream_count(OC, N * OH * OW, 7);
        return;
    }
    if (FH == 1 && FW == 1 && sh == 1 && sw == 1) {   // the W1 native ignores stride; strided 1x1 goes to kernel split
        out->entry = ALPHA_E_dconv3D_deltaX_W1;
        out->streams = stream_count(IC, N * IH * IW, 10);
        return;
    }
    if (c->deltaX_winograd && sh == 1 && sw == 1 && FH == 3 && FW == 3 && OH - IH + 2 <= 4 && OW - IW + 2 <= 4 &&   // padding <= 2
        alpha::winograd_forward_fits(N, OH, OW, OC, IH, IW, IC)) {
        out->entry = ALPHA_E_dconv3D_deltaX_winograd;
        out->streams = 1;
        out->scratch_floats = 16L * IC * OC;
        return;
    }
    if (sh == 1 && sw == 1) {
        // Cuda_dconv3D_deltaX.s1_paddingScaleUp
        const double Q = 1.0 * ((IH - 1 + FH) * (IW - 1 + FW)) / (OH * OW);
        const bool V2 = N > 63 && IC > 63 && Q > c->deltaX_s1_V2_Q;
        out->Q = Q;
        out->V2 = V2;
        out->streams = V2 ? stream_count(IC, N, 10) : stream_count(IC, N * IH * IW, 10);
        out->useTexture = c->deltaX_s1_useTexture && IC > 15;
        out->entry = V2 ? ALPHA_E_dconv3D_deltaX_V2_s1 : (out->useTexture ? ALPHA_E_dconv3D_deltaX_s1_texture : ALPHA_E_dconv3D_deltaX_s1);
        return;
    }
    const int CFH = (FH + sh - 1) / sh, CFW = (FW + sw - 1) / sw;
    out->remode = 1;
    out->scratch_floats = (long)OC * CFH * CFW * IC * sh * sw;
    out->useTexture = c->deltaX_ks_useTexture && IC > 15;
    const int ks_streams = stream_count(IC, N * ((IH + sh - 1) / sh) * ((IW + sw - 1) / sw), 10);
    if (sh == 2 && sw == 2 && (IH & 1) == 0 && (IW & 1) == 0) {
        // Cuda_dconv3D_deltaX.Ims2_paddingScaleUp
        const int OH0 = (IH >> 1) + ((FH + 1) >> 1) - 1, OW0 = (IW >> 1) + ((FW + 1) >> 1) - 1;
        const int OH1 = (IH >> 1) + (FH >> 1) - 1, OW1 = (IW >> 1) + (FW >> 1) - 1;
        const double Q = 0.25 * ((OH0 + OH1) * (OW0 + OW1)) / (OH * OW);
        const bool V2 = N > 63 && IC > 63 && Q > c->deltaX_ks_V2_Q;
        out->Q = Q;
        out->V2 = V2;
        out->streams = V2 ? stream_count(IC, N, 10) : ks_streams;
        out->entry = V2 ? ALPHA_E_dconv3D_deltaX_ksV2_Ims2R
                        : (out->useTexture ? ALPHA_E_dconv3D_deltaX_ksIms2R_texture : ALPHA_E_dconv3D_deltaX_ksIms2R);
        return;
    }
    out->streams = ks_streams;
    if (IH % sh == 0 && IW % sw == 0)
        out->entry = out->useTexture ? ALPHA_E_dconv3D_deltaX_ksImsR_texture : ALPHA_E_dconv3D_deltaX_ksImsR;
    else
        out->entry = ALPHA_E_dconv3D_deltaX_kernelSplit;
}

// ---- engine object: owns scratch and calls the natives the way the Java engine does --------------------------------
struct alpha_engine {
    alpha_engine_config cfg;
    int64_t stream;
    std::mutex mu;
    // Scratch pool, by size in bytes. Every operator is enqueued on the one stream of this engine, so a block used by
    // one operator can be handed to the next as soon as the first has been enqueued: stream order keeps their kernels
    // apart (the Java engine, which spreads work over several streams, waits for the operator's Syncer instead).
    std::multimap<size_t, void *> free_blocks;
    std::vector<std::pair<size_t, void *>> in_flight;     // blocks of the operator being enqueued
    // Transformed filters kept between calls (cfg.cache_filter_transforms): key -> (bytes, block)
    struct FilterKey {
        const void *W;
        int kind, FH, FW, IC, OC, sh, sw;   // kind 0: CW of kernel_remode, 1: Winograd U, 2: kernel-split CW (ks_remodev2), 3: Winograd U of backward-data
        bool operator<(const FilterKey &o) const
        {
            return std::tie(W, kind, FH, FW, IC, OC, sh, sw) < std::tie(o.W, o.kind, o.FH, o.FW, o.IC, o.OC, o.sh, o.sw);
        }
    };
    std::map<FilterKey, std::pair<size_t, void *>> filter_cache;
    // Ticket words lent to the library beside the workspace (alpha_conv_bind_tickets): zeroed once here, left zero by
    // every kernel; all of this engine's kernels run on its one stream, so no two of them use the words at a time.
    unsigned *tickets = nullptr;
    static constexpr int n_tickets = 128;
    char err[256];
};

static void release_blocks(alpha_engine *e)
{
    std::lock_guard<std::mutex> g(e->mu);
    for (auto &b : e->in_flight) e->free_blocks.emplace(b.first, b.second);
    e->in_flight.clear();
}

struct BlockScope {   // returns the operator's scratch to the pool when the operator has been enqueued
    alpha_engine *e;
    ~BlockScope() { release_blocks(e); }
};

static void *take_block(alpha_engine *e, size_t bytes);

// Lends the library scratch for the calls the operator makes on this thread (alpha_conv_bind_workspace): taken from the
// engine's pool like every other block of the operator, so it is recycled in stream order after the operator's kernels.
struct WorkspaceScope {
    bool bound = false;
    explicit WorkspaceScope(alpha_engine *e)
    {
        if (!e->cfg.conv_workspace) return;
        constexpr size_t bytes = 1u << 20;
        if (void *p = take_block(e, bytes)) bound = alpha_conv_bind_workspace(static_cast<float *>(p), (long)bytes) == 0;
        if (bound && e->tickets && e->cfg.conv_workspace == 1) alpha_conv_bind_tickets(e->tickets, alpha_engine::n_tickets);
    }
    ~WorkspaceScope()
    {
        if (bound) {
            alpha_conv_bind_tickets(nullptr, 0);
            alpha_conv_bind_workspace(nullptr, 0);
        }
    }
};

static void *take_block(alpha_engine *e, size_t bytes)
{
    std::lock_guard<std::mutex> g(e->mu);
    auto it = e->free_blocks.lower_bound(bytes);
    void *p = nullptr;
    size_t sz = bytes;
    if (it != e->free_blocks.end() && it->first <= bytes * 2 + 4096) {
        p = it->second;
        sz = it->first;
        e->free_blocks.erase(it);
    } else if (hipMalloc(&p, bytes) != hipSuccess) {
        return nullptr;
    }
    e->in_flight.emplace_back(sz, p);
    return p;
}

// Scratch for a transformed filter. Without the cache it is an ordinary pool block and *fresh is always set (the caller
// runs the transform); with it, the block of an earlier call with the same filter address and geometry is returned with
// *fresh = false, and a new block stays out of the pool until alpha_engine_filter_changed() names its filter.
static float *filter_block(alpha_engine *e, int kind, const float *W, int FH, int FW, int IC, int OC, int sh, int sw,
                           size_t bytes, bool *fresh)
{
    *fresh = true;
    if (!e->cfg.cache_filter_transforms) return static_cast<float *>(take_block(e, bytes));
    const alpha_engine::FilterKey key{W, kind, FH, FW, IC, OC, sh, sw};
    {
        std::lock_guard<std::mutex> g(e->mu);
        auto it = e->filter_cache.find(key);
        if (it != e->filter_cache.end()) {
            *fresh = false;
            return static_cast<float *>(it->second.second);
        }
    }
    void *p = take_block(e, bytes);
    if (!p) return nullptr;
    std::lock_guard<std::mutex> g(e->mu);
    size_t sz = bytes;
    for (auto it = e->in_flight.begin(); it != e->in_flight.end(); ++it)
        if (it->second == p) {   // keep it: it is no longer the operator's to give back
            sz = it->first;
            e->in_flight.erase(it);
            break;
        }
    e->filter_cache[key] = std::make_pair(sz, p);
    return static_cast<float *>(p);
}

// A transform into a freshly cached block failed: the block must not be handed out as a finished transform.
static void forget_filter_block(alpha_engine *e, const float *block)
{
    std::lock_guard<std::mutex> g(e->mu);
    for (auto it = e->filter_cache.begin(); it != e->filter_cache.end(); ++it)
        if (it->second.second == block) {
            e->free_blocks.emplace(it->second.first, it->second.second);
            e->filter_cache.erase(it);
            return;
        }
}

void alpha_engine_filter_changed(alpha_engine *e, const float *W)
{
    std::lock_guard<std::mutex> g(e->mu);
    for (auto it = e->filter_cache.begin(); it != e->filter_cache.end();) {
        if (W == nullptr || it->first.W == W) {
            // kernels already enqueued may still read the block; whoever takes it from the pool next writes to it on
            // the same stream, after them
            e->free_blocks.emplace(it->second.first, it->second.second);
            it = e->filter_cache.erase(it);
        } else {
            ++it;
        }
    }
}

alpha_engine *alpha_engine_create(int64_t stream)
{
    alpha_engine *e = new alpha_engine();
    int cu = 0, clk = 0;
    if (alpha_conv_device_info(&cu, &clk) != 0) cu = 0;
    alpha_engine_config_default(&e->cfg, cu);
    // The one setting in which an engine object departs from the Java engine's defaults: the split-K factor is lowered to
    // what the persistent backward-filter kernel needs on this device (the same cut of the layer, no buffers of zeros for
    // buf_summary to add). Set it to 0 for the Java engine's GridZ exactly.
    e->cfg.deltaW_SK_leastUnits = cu;
    e->cfg.conv_workspace = 1;   // and forward / backward-data calls may use a piece of the engine's scratch (see the header)
    e->stream = stream;
    e->err[0] = 0;
    void *words = nullptr;
    if (cu > 0 && hipMalloc(&words, alpha_engine::n_tickets * sizeof(unsigned)) == hipSuccess) {
        if (hipMemset(words, 0, alpha_engine::n_tickets * sizeof(unsigned)) == hipSuccess) e->tickets = static_cast<unsigned *>(words);
        else (void)hipFree(words);
    }
    return e;
}

alpha_engine_config *alpha_engine_get_config(alpha_engine *e) { return &e->cfg; }
const char *alpha_engine_last_error(alpha_engine *e) { return e->err; }

int alpha_engine_sync(alpha_engine *e)
{
    hipError_t rc = hipStreamSynchronize(reinterpret_cast<hipStream_t>((intptr_t)e->stream));
    release_blocks(e);
    return (int)rc;
}

void alpha_engine_destroy(alpha_engine *e)
{
    if (!e) return;
    alpha_engine_sync(e);
    for (auto &b : e->free_blocks) (void)hipFree(b.second);
    for (auto &b : e->filter_cache) (void)hipFree(b.second.second);
    if (e->tickets) (void)hipFree(e->tickets);
    delete e;
}

// EngineCore.conv3D_param_check (EngineCore.java:630-678), non-strict form, minus the sh <= FH rule (see alpha_plan_conv3D).
// Refusing inconsistent shapes here matters: the natives trust their arguments and would write out of bounds.
static const char *param_check(int OH, int OW, int IH, int IW, int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    if (OH <= 0 || OW <= 0) return "output size <= 0";
    if (N <= 0 || IC <= 0 || OC <= 0) return "N, IC or OC <= 0";
    if (sh <= 0 || sw <= 0) return "stride <= 0";
    if (ph < 0 || pw < 0) return "padding < 0";
    if (FH <= ph || FW <= pw) return "filter size <= padding";
    if (FH > IH + (ph << 1) || FW > IW + (pw << 1)) return "filter larger than padded input";
    if (IH - FH + (ph << 1) < (OH - 1) * sh) return "(IH - FH + 2*ph) < (OH - 1)*sh";
    if (IW - FW + (pw << 1) < (OW - 1) * sw) return "(IW - FW + 2*pw) < (OW - 1)*sw";
    if ((IC & 3) || (OC & 3)) return "IC and OC must be padded to multiples of 4";
    return nullptr;
}

const char *alpha_engine_param_check(int OH, int OW, int IH, int IW, int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw)
{
    return param_check(OH, OW, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw);
}

static int fail(alpha_engine *e, int rc, const char *what)
{
    snprintf(e->err, sizeof(e->err), "%s: %s", what, rc == -1 ? "scratch allocation failed" : alpha_conv_last_error());
    return rc;
}

int alpha_engine_conv3D(alpha_engine *e, float *Y, int OH, int OW, const float *X, int IH, int IW, const float *W, int FH, int FW,
                        int N, int IC, int OC, int sh, int sw, int ph, int pw, alpha_conv_plan *plan_out)
{
    if (const char *why = param_check(OH, OW, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw)) {
        snprintf(e->err, sizeof(e->err), "%s: illegal size: %s", "alpha_engine_conv3D", why);
        return ALPHA_CONV_EINVAL;
    }
    BlockScope scope{e};
    WorkspaceScope workspace(e);
    alpha_conv_plan p;
    alpha_plan_conv3D(&e->cfg, IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, ph, pw, &p);
    if (plan_out) *plan_out = p;
    int64_t streams[16];
    for (int i = 0; i < p.streams; i++) streams[i] = e->stream;
    int rc = 0;
    if (p.entry == ALPHA_E_conv3D_winograd) {
        bool fresh;
        float *U = filter_block(e, 1, W, 3, 3, IC, OC, 1, 1, (size_t)p.scratch_floats * sizeof(float), &fresh);
        if (!U) return fail(e, -1, "conv3D");
        if (fresh && (rc = alpha_winograd_filter_transform(streams[0], W, U, IC, OC))) { forget_filter_block(e, U); return fail(e, rc, "winograd_filter_transform"); }
        rc = alpha_conv3D_winograd(streams, p.streams, X, IH, IW, U, Y, OH, OW, N, IC, OC, ph, pw);
    } else if (p.remode) {
        bool fresh;
        float *CW = filter_block(e, 0, W, FH, FW, IC, OC, 1, 1, (size_t)p.scratch_floats * sizeof(float), &fresh);
        if (!CW) return fail(e, -1, "conv3D");
        if (fresh && (rc = alpha_kernel_remode(streams[0], W, CW, FH, FW, OC, IC))) { forget_filter_block(e, CW); return fail(e, rc, "kernel_remode"); }
        switch (p.entry) {
        case ALPHA_E_conv3D_GemmR_W1: rc = alpha_conv3D_GemmR_W1(streams, p.streams, X, IH, IW, W, CW, Y, N, IC, OC); break;
        case ALPHA_E_conv3D_GemmV2R:
            rc = alpha_conv3D_GemmV2R(p.useTexture, streams, p.streams, X, IH, IW, W, CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw);
            break;
        case ALPHA_E_conv3D_GemmR_texture:
            rc = alpha_conv3D_GemmR_texture(streams, p.streams, X, IH, IW, W, CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw);
            break;
        default: rc = alpha_conv3D_GemmR(streams, p.streams, X, IH, IW, W, CW, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw); break;
        }
    } else {
        switch (p.entry) {
        case ALPHA_E_conv3D_W1: rc = alpha_conv3D_W1(streams, p.streams, X, IH, IW, W, Y, N, IC, OC); break;
        case ALPHA_E_conv3D_np: rc = alpha_conv3D_np(streams, p.streams, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw); break;
        case ALPHA_E_conv3DV2:
            rc = alpha_conv3DV2(p.useTexture, streams, p.streams, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw);
            break;
        case ALPHA_E_conv3D_texture:
            rc = alpha_conv3D_texture(streams, p.streams, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw);
            break;
        default: rc = alpha_conv3D(streams, p.streams, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw, ph, pw); break;
        }
    }
    return rc ? fail(e, rc, "conv3D") : 0;
}

// CudaFloat32EngineBase.conv3D_biased (:1478-1560): same selection as conv3D; there the bias is a second pass
// (linear_dual2D_row on Y after an event), here it rides in the conv kernel's epilogue, so every remode entry collapses
// onto the GemmR form and every other entry onto the plain form.
static int conv3D_with_epilogue(alpha_engine *e, const char *what, float *Y, int OH, int OW, const float *X, int IH, int IW,
                                const float *W, int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                                const alpha_conv_epilogue *ep, alpha_conv_plan *plan_out)
{
    BlockScope scope{e};
    WorkspaceScope workspace(e);
    alpha_conv_plan p;
    alpha_plan_conv3D(&e->cfg, IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, ph, pw, &p);
    if (plan_out) *plan_out = p;
    int64_t streams[16];
    for (int i = 0; i < p.streams; i++) streams[i] = e->stream;
    int rc = 0;
    if (p.entry == ALPHA_E_conv3D_winograd) {
        bool fresh;
        float *U = filter_block(e, 1, W, 3, 3, IC, OC, 1, 1, (size_t)p.scratch_floats * sizeof(float), &fresh);
        if (!U) return fail(e, -1, what);
        if (fresh && (rc = alpha_winograd_filter_transform(streams[0], W, U, IC, OC))) { forget_filter_block(e, U); return fail(e, rc, "winograd_filter_transform"); }
        rc = alpha_conv3D_winograd_fused(streams, p.streams, X, IH, IW, U, ep, Y, OH, OW, N, IC, OC, ph, pw);
    } else if (p.remode) {
        bool fresh;
        float *CW = filter_block(e, 0, W, FH, FW, IC, OC, 1, 1, (size_t)p.scratch_floats * sizeof(float), &fresh);
        if (!CW) return fail(e, -1, what);
        if (fresh && (rc = alpha_kernel_remode(streams[0], W, CW, FH, FW, OC, IC))) { forget_filter_block(e, CW); return fail(e, rc, "kernel_remode"); }
        rc = alpha_conv3D_GemmR_fused(streams, p.streams, X, IH, IW, W, CW, FH, FW, ep, Y, OH, OW, N, IC, OC, sh, sw, ph, pw);
    } else {
        rc = alpha_conv3D_fused(streams, p.streams, X, IH, IW, W, FH, FW, ep, Y, OH, OW, N, IC, OC, sh, sw, ph, pw);
    }
    return rc ? fail(e, rc, what) : 0;
}

int alpha_engine_conv3D_biased(alpha_engine *e, float *Y, int OH, int OW, const float *X, int IH, int IW, const float *W,
                               int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                               const float *Bias, int lengthv, int width, alpha_conv_plan *plan_out)
{
    if (const char *why = param_check(OH, OW, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw)) {
        snprintf(e->err, sizeof(e->err), "%s: illegal size: %s", "alpha_engine_conv3D_biased", why);
        return ALPHA_CONV_EINVAL;
    }
    // EngineCore.func_param_check_row(lengthv, OC_4x, OC, OC_4x): the rows of Y are the OC channels of one pixel
    if (Bias == nullptr || (long)lengthv != (long)N * OH * OW * OC || width < 1 || width > OC) {
        snprintf(e->err, sizeof(e->err), "alpha_engine_conv3D_biased: Bias is null, or lengthv != N*OH*OW*OC, or width not in [1, OC]");
        return ALPHA_CONV_EINVAL;
    }
    alpha_conv_epilogue ep{};
    ep.Bias = Bias;
    ep.k = 1.f;
    return conv3D_with_epilogue(e, "conv3D_biased", Y, OH, OW, X, IH, IW, W, FH, FW, N, IC, OC, sh, sw, ph, pw, &ep, plan_out);
}

// conv3D followed by batch normalisation with given statistics and leaky ReLU (the inference form of the reference's
// conv -> bn -> leakyRelu blocks, experiments/alpha_code/src/cifar10/resnet18/Net.java:42-58), as one operator: same plan
// as conv3D, the row functions in the convolution kernel's epilogue.
int alpha_engine_conv3D_fused(alpha_engine *e, float *Y, int OH, int OW, const float *X, int IH, int IW, const float *W,
                              int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                              const alpha_conv_epilogue *epilogue, alpha_conv_plan *plan_out)
{
    if (const char *why = param_check(OH, OW, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw)) {
        snprintf(e->err, sizeof(e->err), "%s: illegal size: %s", "alpha_engine_conv3D_fused", why);
        return ALPHA_CONV_EINVAL;
    }
    if (epilogue == nullptr) {
        snprintf(e->err, sizeof(e->err), "alpha_engine_conv3D_fused: epilogue is null");
        return ALPHA_CONV_EINVAL;
    }
    return conv3D_with_epilogue(e, "conv3D_fused", Y, OH, OW, X, IH, IW, W, FH, FW, N, IC, OC, sh, sw, ph, pw, epilogue, plan_out);
}

int alpha_engine_dconv3D_deltaW(alpha_engine *e, float *deltaW, int FH, int FW, const float *X, int IH, int IW,
                                const float *deltaY, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                                alpha_conv_plan *plan_out)
{
    if (const char *why = param_check(OH, OW, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw)) {
        snprintf(e->err, sizeof(e->err), "%s: illegal size: %s", "alpha_engine_dconv3D_deltaW", why);
        return ALPHA_CONV_EINVAL;
    }
    BlockScope scope{e};
    alpha_conv_plan p;
    alpha_plan_deltaW(&e->cfg, IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, &p);
    if (p.entry == ALPHA_E_dconv3D_deltaW_GemmSK_winograd && (OH != IH + 2 * ph - 2 || OW != IW + 2 * pw - 2)) {
        // an output smaller than the formula's is legal for the engine but not for the Winograd kernel: the default plan
        alpha_engine_config plain = e->cfg;
        plain.deltaW_winograd = 0;
        alpha_plan_deltaW(&plain, IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, &p);
    }
    if (plan_out) *plan_out = p;
    int64_t streams[16];
    for (int i = 0; i < p.streams; i++) streams[i] = e->stream;
    int rc = 0;
    if (p.GridZ == 1 && p.entry == ALPHA_E_dconv3D_deltaW_GemmSK_winograd) {
        rc = alpha_dconv3D_deltaW_GemmSK_winograd(streams, p.streams, 1, X, IH, IW, deltaY, OH, OW, deltaW, nullptr, N, IC, OC, ph, pw);
        return rc ? fail(e, rc, "dconv3D_deltaW") : 0;
    }
    if (p.GridZ == 1) {
        rc = p.entry == ALPHA_E_dconv3D_deltaW_W1
                 ? alpha_dconv3D_deltaW_W1(streams, p.streams, X, IH, IW, deltaY, deltaW, N, IC, OC)
                 : alpha_dconv3D_deltaW(streams, p.streams, X, IH, IW, deltaY, OH, OW, deltaW, FH, FW, N, IC, OC, sh, sw, ph, pw);
        return rc ? fail(e, rc, "dconv3D_deltaW") : 0;
    }
    float *buf = static_cast<float *>(take_block(e, (size_t)p.scratch_floats * sizeof(float)));
    if (!buf) return fail(e, -1, "dconv3D_deltaW");
    switch (p.entry) {
    case ALPHA_E_dconv3D_deltaW_GemmSK_winograd:
        rc = alpha_dconv3D_deltaW_GemmSK_winograd(streams, p.streams, p.GridZ, X, IH, IW, deltaY, OH, OW, deltaW, buf, N, IC, OC, ph, pw);
        break;
    case ALPHA_E_dconv3D_deltaW_GemmSK_W1:
        rc = alpha_dconv3D_deltaW_GemmSK_W1(streams, p.streams, p.GridZ, X, IH, IW, deltaY, deltaW, buf, N, IC, OC);
        break;
    case ALPHA_E_dconv3D_deltaW_GemmV2SK:
        rc = alpha_dconv3D_deltaW_GemmV2SK(streams, p.streams, p.GridZ, X, IH, IW, deltaY, OH, OW, deltaW, buf, FH, FW, N, IC, OC,
                                           sh, sw, ph, pw);
        break;
    default:
        rc = alpha_dconv3D_deltaW_GemmSK(streams, p.streams, p.GridZ, X, IH, IW, deltaY, OH, OW, deltaW, buf, FH, FW, N, IC, OC,
                                         sh, sw, ph, pw);
        break;
    }
    if (rc) return fail(e, rc, "dconv3D_deltaW");
    rc = alpha_buf_summary(streams[0], buf, deltaW, p.GridZ - 1, OC * FH * FW * IC);
    return rc ? fail(e, rc, "buf_summary") : 0;
}

// Backward-filter and bias gradient in one operator: nn/unit/simple/Conv3D.java:150-162 calls eg.dconv3D_deltaW and then
// eg.field_sum(deltaY, OC); here the column sums ride in the backward-filter kernel (one pass over deltaY) and both
// results are finished by the same Kahan buf_summary.
int alpha_engine_dconv3D_deltaW_deltaB(alpha_engine *e, float *deltaW, float *deltaB, int FH, int FW, const float *X, int IH, int IW,
                                       const float *deltaY, int OH, int OW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                                       alpha_conv_plan *plan_out)
{
    if (const char *why = param_check(OH, OW, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw)) {
        snprintf(e->err, sizeof(e->err), "%s: illegal size: %s", "alpha_engine_dconv3D_deltaW_deltaB", why);
        return ALPHA_CONV_EINVAL;
    }
    BlockScope scope{e};
    alpha_conv_plan p;
    // deltaW_SK_leastUnits lowers GridZ to what the persistent backward-filter kernel needs; with a bias gradient the
    // library may serve the layer through a kernel that produces the column sums on the way and keeps the slice
    // partition (1x1 layers, layers whose slices fill the device), which the lowered GridZ would leave under-filled:
    // this operator always plans with the Java engine's GridZ.
    alpha_engine_config cfg = e->cfg;
    cfg.deltaW_SK_leastUnits = 0;
    alpha_plan_deltaW(&cfg, IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, &p);
    if (p.entry == ALPHA_E_dconv3D_deltaW_GemmSK_winograd && (OH != IH + 2 * ph - 2 || OW != IW + 2 * pw - 2)) {
        // an output smaller than the formula's is legal for the engine but not for the Winograd kernel: the default plan
        cfg.deltaW_winograd = 0;
        alpha_plan_deltaW(&cfg, IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, &p);
    }
    if (plan_out) *plan_out = p;
    int64_t streams[16];
    for (int i = 0; i < p.streams; i++) streams[i] = e->stream;
    const size_t sizeW = (size_t)OC * FH * FW * IC;
    float *buf = nullptr, *bbuf = nullptr;
    if (p.GridZ > 1) {
        buf = static_cast<float *>(take_block(e, (sizeW + OC) * (p.GridZ - 1) * sizeof(float)));
        if (!buf) return fail(e, -1, "dconv3D_deltaW_deltaB");
        bbuf = buf + sizeW * (p.GridZ - 1);
    }
    int rc = alpha_dconv3D_deltaW_GemmSK_deltaB(streams, p.streams, p.GridZ, X, IH, IW, deltaY, OH, OW, deltaW, buf, deltaB, bbuf,
                                                FH, FW, N, IC, OC, sh, sw, ph, pw);
    if (rc) return fail(e, rc, "dconv3D_deltaW_deltaB");
    if (p.GridZ > 1) {
        if ((rc = alpha_buf_summary(streams[0], buf, deltaW, p.GridZ - 1, (int)sizeW))) return fail(e, rc, "buf_summary");
        if ((rc = alpha_buf_summary(streams[0], bbuf, deltaB, p.GridZ - 1, OC))) return fail(e, rc, "buf_summary");
    }
    return 0;
}

// Backward of batch normalisation: CudaFloat32EngineBase.batchNorm2D_deltaX_v1 / _v2 (:4385-4475, affine :4478-4576) and
// batchNorm2D_gradients_v1 / _v2 (:4648-4760). Stage 1: the field sums deltaXp1 = sum deltaY, deltaXp2 = sum deltaY * X_norm
// (into deltaB / deltaA when the caller wants them - the gradients forms -, else into scratch); stage 2: the row function.
// The Java engine runs stage 1 on two streams and joins them with an event; here one stream orders everything.
static int bn_backward(alpha_engine *e, const char *what, bool from_x, float *deltaX, const float *deltaY, const float *S,
                       const float *X_mean, const float *X_var, float eps, const float *A, const float *B, float *deltaA, float *deltaB,
                       int field_length, int row_lengthv, int lengthv, int width, int stride)
{
    if (field_length < 1 || row_lengthv < 4 || (long)field_length * row_lengthv != lengthv) {
        snprintf(e->err, sizeof(e->err), "%s: need lengthv = field_length * row_lengthv", what);
        return ALPHA_CONV_EINVAL;
    }
    BlockScope scope{e};
    const int M = row_lengthv;
    // buffers as the Java engine sizes them: nextN x M floats each (Cuda_reduce.field_nextN), with the sums at their heads
    // when the caller does not ask for them
    int nextN = (M > 15 && field_length > 63) ? field_length >> 6 : (M > 15 && field_length > 15) ? 1
              : (M > 7 && field_length > 127) ? field_length >> 7 : (M > 7 && field_length > 31) ? 1 : (field_length + 63) >> 6;
    if (nextN < 1) nextN = 1;
    float *buf = static_cast<float *>(take_block(e, (size_t)2 * nextN * M * sizeof(float)));
    if (!buf) return fail(e, -1, what);
    float *bufB = buf, *bufA = buf + (size_t)nextN * M;
    float *p1 = deltaB ? deltaB : bufB, *p2 = deltaA ? deltaA : bufA;
    int rc;
    if (from_x) rc = alpha_field_batchNorm_deltaAB_v2(e->stream, e->stream, deltaY, S, X_mean, X_var, eps, field_length, M, bufA, p2, bufB, p1, width, stride, 1, nullptr);
    else if (A) rc = alpha_field_affine_deltaAB_v1(e->stream, e->stream, deltaY, S, A, B, field_length, M, bufA, p2, bufB, p1, width, stride, 1, nullptr);
    else rc = alpha_field_affine_deltaAB_v2(e->stream, e->stream, deltaY, S, field_length, M, bufA, p2, bufB, p1, width, stride, 1, nullptr);
    if (rc) return fail(e, rc, what);
    if (from_x) {
        rc = A ? alpha_batchNorm_affined2D_row_deltaX_v2(e->stream, deltaY, S, X_mean, X_var, eps, A, p1, p2, M, deltaX, lengthv, width, stride)
               : alpha_batchNorm2D_row_deltaX_v2(e->stream, deltaY, S, X_mean, X_var, eps, p1, p2, M, deltaX, lengthv, width, stride);
    } else {
        rc = A ? alpha_batchNorm_affined2D_row_deltaX_v1(e->stream, deltaY, S, X_var, eps, A, B, p1, p2, M, deltaX, lengthv, width, stride)
               : alpha_batchNorm2D_row_deltaX_v1(e->stream, deltaY, S, X_var, eps, p1, p2, M, deltaX, lengthv, width, stride);
    }
    return rc ? fail(e, rc, what) : 0;
}

int alpha_engine_batchNorm2D_deltaX_v1(alpha_engine *e, float *deltaX, const float *deltaY, const float *Y, const float *X_var, float eps,
                                       const float *A, const float *B, float *deltaA, float *deltaB,
                                       int field_length, int row_lengthv, int lengthv, int width, int stride)
{
    if ((A == nullptr) != (B == nullptr) || (!A && (deltaA || deltaB)) || (deltaA == nullptr) != (deltaB == nullptr)) {
        snprintf(e->err, sizeof(e->err), "alpha_engine_batchNorm2D_deltaX_v1: A and B go together, deltaA and deltaB go together and need A");
        return ALPHA_CONV_EINVAL;
    }
    return bn_backward(e, "batchNorm2D_deltaX_v1", false, deltaX, deltaY, Y, nullptr, X_var, eps, A, B, deltaA, deltaB,
                       field_length, row_lengthv, lengthv, width, stride);
}

int alpha_engine_batchNorm2D_deltaX_v2(alpha_engine *e, float *deltaX, const float *deltaY, const float *X, const float *X_mean,
                                       const float *X_var, float eps, const float *A, float *deltaA, float *deltaB,
                                       int field_length, int row_lengthv, int lengthv, int width, int stride)
{
    if ((!A && (deltaA || deltaB)) || (deltaA == nullptr) != (deltaB == nullptr)) {
        snprintf(e->err, sizeof(e->err), "alpha_engine_batchNorm2D_deltaX_v2: deltaA and deltaB go together and need A");
        return ALPHA_CONV_EINVAL;
    }
    return bn_backward(e, "batchNorm2D_deltaX_v2", true, deltaX, deltaY, X, X_mean, X_var, eps, A, nullptr, deltaA, deltaB,
                       field_length, row_lengthv, lengthv, width, stride);
}

// Xf != NULL: deltaX is multiplied by the derivative of the leaky ReLU (slope k) whose output Xf is this layer's input - in
// the kernel's epilogue for the stride-1 entries, by leakyRelu2D_deltaX_v1 in place after the others.
static int deltaX_impl(alpha_engine *e, const char *what, float *deltaX, int IH, int IW, const float *deltaY, int OH, int OW,
                       const float *W, int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                       const float *Xf, float k, alpha_conv_plan *plan_out)
{
    if (const char *why = param_check(OH, OW, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw)) {
        snprintf(e->err, sizeof(e->err), "%s: illegal size: %s", what, why);
        return ALPHA_CONV_EINVAL;
    }
    BlockScope scope{e};
    WorkspaceScope workspace(e);
    alpha_conv_plan p;
    alpha_plan_deltaX(&e->cfg, IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, &p);
    if (p.entry == ALPHA_E_dconv3D_deltaX_winograd && (OH != IH + 2 * ph - 2 || OW != IW + 2 * pw - 2)) {
        // an output smaller than the formula's is legal for the engine but not for the Winograd kernels: the default plan
        alpha_engine_config plain = e->cfg;
        plain.deltaX_winograd = 0;
        alpha_plan_deltaX(&plain, IH, IW, OH, OW, FH, FW, N, IC, OC, sh, sw, &p);
    }
    if (plan_out) *plan_out = p;
    int64_t streams[16];
    for (int i = 0; i < p.streams; i++) streams[i] = e->stream;
    int rc = 0;
    bool gated = Xf == nullptr;   // nothing to apply, or applied by the kernel
    if (Xf != nullptr && (p.entry == ALPHA_E_dconv3D_deltaX_W1 || p.entry == ALPHA_E_dconv3D_deltaX_V2_s1 ||
                          p.entry == ALPHA_E_dconv3D_deltaX_s1_texture || p.entry == ALPHA_E_dconv3D_deltaX_s1)) {
        const bool w1 = p.entry == ALPHA_E_dconv3D_deltaX_W1;
        rc = alpha_dconv3D_deltaX_s1_leakyRelu(streams, p.streams, deltaY, w1 ? IH : OH, w1 ? IW : OW, W, FH, FW, Xf, k, deltaX, IH, IW,
                                               N, IC, OC, w1 ? 0 : ph, w1 ? 0 : pw);
        return rc ? fail(e, rc, what) : 0;
    }
    switch (p.entry) {
    case ALPHA_E_dconv3D_deltaX_crossAdd:
        rc = alpha_dconv3D_deltaX_crossAdd(streams, p.streams, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw);
        break;
    case ALPHA_E_dconv3D_deltaX_winograd: {
        bool fresh;
        float *U = filter_block(e, 3, W, 3, 3, IC, OC, 1, 1, (size_t)p.scratch_floats * sizeof(float), &fresh);
        if (!U) return fail(e, -1, what);
        if (fresh && (rc = alpha_winograd_filter_transform_deltaX(streams[0], W, U, IC, OC))) { forget_filter_block(e, U); return fail(e, rc, "winograd_filter_transform_deltaX"); }
        rc = alpha_dconv3D_deltaX_winograd(streams, p.streams, deltaY, OH, OW, U, deltaX, IH, IW, N, IC, OC, ph, pw);
        break;
    }
    case ALPHA_E_dconv3D_deltaX_W1:
        rc = alpha_dconv3D_deltaX_W1(streams, p.streams, deltaY, W, deltaX, IH, IW, N, IC, OC);
        break;
    case ALPHA_E_dconv3D_deltaX_V2_s1:
        rc = alpha_dconv3D_deltaX_V2_s1(p.useTexture, streams, p.streams, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw);
        break;
    case ALPHA_E_dconv3D_deltaX_s1_texture:
        rc = alpha_dconv3D_deltaX_s1_texture(streams, p.streams, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw);
        break;
    case ALPHA_E_dconv3D_deltaX_s1:
        rc = alpha_dconv3D_deltaX_s1(streams, p.streams, deltaY, OH, OW, W, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw);
        break;
    default: {
        const int CFH = (FH + sh - 1) / sh, CFW = (FW + sw - 1) / sw;
        bool fresh;
        float *CW = filter_block(e, 2, W, FH, FW, IC, OC, sh, sw, (size_t)p.scratch_floats * sizeof(float), &fresh);
        if (!CW) return fail(e, -1, what);
        if (fresh && (rc = alpha_ks_remodev2(streams[0], W, FH, FW, CW, CFH, CFW, OC, IC, sh, sw))) { forget_filter_block(e, CW); return fail(e, rc, "ks_remodev2"); }
        if (Xf != nullptr) {   // every kernel-split entry runs the same kernels: the mask rides in their epilogue
            rc = alpha_dconv3D_deltaX_kernelSplit_leakyRelu(streams, p.streams, deltaY, OH, OW, CW, FH, FW, Xf, k, deltaX, IH, IW, N, IC, OC,
                                                            sh, sw, ph, pw);
            gated = true;
            break;
        }
        switch (p.entry) {
        case ALPHA_E_dconv3D_deltaX_ksV2_Ims2R:
            rc = alpha_dconv3D_deltaX_ksV2_Ims2R(p.useTexture, streams, p.streams, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw);
            break;
        case ALPHA_E_dconv3D_deltaX_ksIms2R_texture:
            rc = alpha_dconv3D_deltaX_ksIms2R_texture(streams, p.streams, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw);
            break;
        case ALPHA_E_dconv3D_deltaX_ksIms2R:
            rc = alpha_dconv3D_deltaX_ksIms2R(streams, p.streams, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, ph, pw);
            break;
        case ALPHA_E_dconv3D_deltaX_ksImsR_texture:
            rc = alpha_dconv3D_deltaX_ksImsR_texture(streams, p.streams, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw);
            break;
        case ALPHA_E_dconv3D_deltaX_ksImsR:
            rc = alpha_dconv3D_deltaX_ksImsR(streams, p.streams, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw);
            break;
        default:
            rc = alpha_dconv3D_deltaX_kernelSplit(streams, p.streams, deltaY, OH, OW, CW, FH, FW, deltaX, IH, IW, N, IC, OC, sh, sw, ph, pw);
            break;
        }
    }
    }
    if (rc == 0 && !gated)
        rc = alpha_leakyRelu2D_deltaX_v1(streams[0], deltaX, deltaX, Xf, k, N * IH * IW * IC, IC, IC);
    return rc ? fail(e, rc, what) : 0;
}

int alpha_engine_dconv3D_deltaX(alpha_engine *e, float *deltaX, int IH, int IW, const float *deltaY, int OH, int OW,
                                const float *W, int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                                alpha_conv_plan *plan_out)
{
    return deltaX_impl(e, "alpha_engine_dconv3D_deltaX", deltaX, IH, IW, deltaY, OH, OW, W, FH, FW, N, IC, OC, sh, sw, ph, pw, nullptr, 1.f,
                       plan_out);
}

int alpha_engine_dconv3D_deltaX_leakyRelu(alpha_engine *e, float *deltaX, int IH, int IW, const float *deltaY, int OH, int OW,
                                          const float *W, int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                                          const float *Xf, float k, alpha_conv_plan *plan_out)
{
    if (Xf == nullptr) {
        snprintf(e->err, sizeof(e->err), "alpha_engine_dconv3D_deltaX_leakyRelu: Xf is null");
        return ALPHA_CONV_EINVAL;
    }
    return deltaX_impl(e, "alpha_engine_dconv3D_deltaX_leakyRelu", deltaX, IH, IW, deltaY, OH, OW, W, FH, FW, N, IC, OC, sh, sw, ph, pw, Xf, k,
                       plan_out);

}

#pragma GCC visibility pop
}  // extern "C"
