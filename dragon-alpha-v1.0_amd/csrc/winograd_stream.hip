// Winograd F(2x2, 3x3) forward convolution as one uninterrupted MFMA stream per workgroup, gfx950, for input channel
// counts that are multiples of 16. Same arithmetic as winograd.hip (input transform -> 16 MFMA GEMMs, one per transform
// position xi -> output transform, v_mfma_f32_16x16x4_f32, the transformed filter U[16][IC/4][OC][4] fetched from L2 through
// a register ring); what differs is what happens between two output blocks.
//
// An item is 32 consecutive tiles of the flattened (n, tile row, tile column) index (2x2 output pixels each) times 64
// output channels; a step is one 16-channel chunk of one item. The grid is persistent (two workgroups of 4 wavefronts
// per compute unit) and a workgroup walks a contiguous range of items as one sequence of steps. Three cursors run along
// that sequence, none of them stops at an item boundary:
//   * the MFMAs of step k (wavefront w: output channels [16w, 16w+16) x 32 tiles x 16 xi = 128 accumulator registers),
//   * the filter ring, four xi ahead of the MFMAs,
//   * the input patches: the 4x4 patch of (tile, channel pair) for step k+2 is requested from memory during step k,
//     transformed (B^T d B, per thread) and written as V[xi][tile][16 channels] into the other LDS buffer during step
//     k+1, in the shadow of that step's MFMAs, and multiplied in step k+2.
// So the only thing outside the MFMA stream is an item's output transform (A^T m A per lane, which holds all 16 xi of
// its (tile, channel) pairs) and its stores, which leave the registers directly: 16 lanes write 64 consecutive bytes.
// Items that do not divide evenly among the workgroups are cut into halves of 16 tiles (the second MFMA row block is
// left out) as far as the workgroups reach, so the longest workgroup is half an item above most of the others.
#include "common.hpp"
#include <type_traits>

namespace alpha {

struct WinoStreamArgs {
    const float *X;      // [N, IH, IW, IC]
    const float *U;      // [16][IC/4][OC][4]
    float *Y;            // [N, OH, OW, OC]
    const float *bias;   // NULL or [OC]
    int IH, IW, IC, OH, OW, OC, ph, pw;
    int TC, TRC;         // tile columns per image row, tiles per image
    int ntiles, groups;  // N*TRC; groups of 32 tiles; item id = (block of 64 output channels) * groups + group
    int x_bytes, u_bytes, y_bytes;   // X and U below 2 GB, Y at most 1 GB
    int whole;           // items every workgroup takes: workgroup b owns [b*whole, (b+1)*whole)
    int extra;           // workgroups below this take item gridDim.x*whole + b as well
    int halves;          // the next so many workgroups, b' = b - extra, take half (b' & 1) of item gridDim.x*whole + extra + b'/2
    FastDiv d_TC, d_TRC, d_groups;
};

constexpr int WS_TILES = 32;
constexpr int WS_VBUF = 16 * WS_TILES * 16;   // floats per V buffer: [xi][tile][16 channels]
constexpr unsigned WS_OOR = 0x80000000u;      // beyond every descriptor: loads return 0, stores are dropped

__global__ __launch_bounds__(256, 2) void winograd_stream_kernel(const WinoStreamArgs p)
{
    extern __shared__ __attribute__((aligned(16))) float ws_smem[];   // V[2][WS_VBUF], otab[2][32][4]
    float *smem = ws_smem;

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int xt = t >> 3, xq = (t & 7) * 2;   // input transform: thread -> (tile xt, channel pair xq of the chunk)
    const int b = blockIdx.x, G = gridDim.x;
    const bool has_half = b >= p.extra && b < p.extra + p.halves;
    const int nitems = p.whole + (b < p.extra ? 1 : 0) + (has_half ? 1 : 0);
    const int nchunks = p.IC >> 4;
    const unsigned xi_stride4 = (unsigned)p.IC * p.OC * 4;   // bytes between two transform positions of U
    const unsigned chunk_stride4 = 16u * p.OC * 4;           // bytes between two 16-channel chunks of U

    struct Item {
        int tile_first, tile_end, oc0, half;
    };
    auto item_of = [&](int k) {   // uniform
        Item it;
        int id, hoff = 0;
        it.half = 0;
        if (k < p.whole) id = b * p.whole + k;
        else if (b < p.extra) id = G * p.whole + b;
        else {
            const int hb = b - p.extra;
            id = G * p.whole + p.extra + (hb >> 1);
            it.half = 1;
            hoff = (hb & 1) * 16;
        }
        const int ocb = fdiv(id, p.d_groups), g = id - ocb * p.groups;
        it.oc0 = ocb * 64;
        it.tile_first = g * WS_TILES + hoff;
        const int end = it.tile_first + (it.half ? 16 : WS_TILES);
        it.tile_end = end < p.ntiles ? end : p.ntiles;
        return it;
    };

    floatx4 acc[16][2];   // every item's first step starts them from zero

    // ---- input patches: descriptor base + uniform channel offset + per-lane pixel offset (fixed for an item) ----------
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.X), 0, p.x_bytes, 0x00020000);
    float2 d[4][4];
    unsigned p_off[4][4];
    auto patch_offsets = [&](const Item &it) {
        // computed for every lane, selected at the end: no divergent branches in the MFMA stream
        const int tile = it.tile_first + xt;
        const bool tile_ok = tile < it.tile_end;
        const int n = fdiv(tile, p.d_TRC), rem = tile - n * p.TRC;
        const int ty = fdiv(rem, p.d_TC), tx = rem - ty * p.TC;
        const int ih0 = 2 * ty - p.ph, iw0 = 2 * tx - p.pw;
        const int x_base = n * p.IH * p.IW * p.IC + xq;
        int rowpart[4], colpart[4];
        bool row_ok[4], col_ok[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            row_ok[i] = tile_ok && (unsigned)(ih0 + i) < (unsigned)p.IH;
            rowpart[i] = x_base + (ih0 + i) * p.IW * p.IC;
            col_ok[i] = (unsigned)(iw0 + i) < (unsigned)p.IW;
            colpart[i] = (iw0 + i) * p.IC;
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                p_off[i][j] = (row_ok[i] && col_ok[j]) ? (unsigned)(rowpart[i] + colpart[j]) * 4u : WS_OOR;
    };
    auto load_patch_element = [&](int e, int icc) {   // e = 4i + j
        d[e >> 2][e & 3] = __builtin_bit_cast(float2, __builtin_amdgcn_raw_buffer_load_b64(x_rsrc, p_off[e >> 2][e & 3], icc * 4, 0));
    };
    auto load_patch = [&](int icc) {
#pragma unroll
        for (int e = 0; e < 16; e++) load_patch_element(e, icc);
    };
    // V = B^T d B, B^T = [[1,0,-1,0],[0,1,1,0],[0,-1,1,0],[0,1,0,-1]]
    auto sub = [](float2 a, float2 c) { return make_float2(a.x - c.x, a.y - c.y); };
    auto add = [](float2 a, float2 c) { return make_float2(a.x + c.x, a.y + c.y); };
    float2 r[4][4];   // B^T d, alive between the two halves of the transform
    auto transform_columns = [&]() {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            r[0][j] = sub(d[0][j], d[2][j]);
            r[1][j] = add(d[1][j], d[2][j]);
            r[2][j] = sub(d[2][j], d[1][j]);
            r[3][j] = sub(d[1][j], d[3][j]);
        }
    };
    auto transform_half_row_store = [&](float *Vw, int i, int h) {   // V positions 4i + 2h, 4i + 2h + 1
        const float2 va = h == 0 ? sub(r[i][0], r[i][2]) : sub(r[i][2], r[i][1]);
        const float2 vb = h == 0 ? add(r[i][1], r[i][2]) : sub(r[i][1], r[i][3]);
        *reinterpret_cast<float2 *>(Vw + (4 * i + 2 * h + 0) * WS_TILES * 16) = va;
        *reinterpret_cast<float2 *>(Vw + (4 * i + 2 * h + 1) * WS_TILES * 16) = vb;
    };

    // ---- transformed filter U[16][IC/4][OC][4]: lane (l16, q) needs channels chunk*16 + 4q .. + 3 of column
    //      oc0 + 16w + l16, one 128-bit element (a ring refill is one load instead of four); columns beyond OC read
    //      something finite or the range check's zero and are never stored --------------------------------------------
    const __amdgpu_buffer_rsrc_t u_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.U), 0, p.u_bytes, 0x00020000);
    const unsigned u_lane = (unsigned)(q * p.OC + 16 * w + l16) * 16u;   // group q of the chunk's four groups of 4 channels
    floatx4 bring[4];
    auto load_b = [&](floatx4 &bb, unsigned block) {   // block: uniform byte offset of (xi, chunk, oc0)
        bb = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(u_rsrc, u_lane, block, 0));
    };

    // ---- output: lane (l16, q) holds tiles 16mt + 4q + r (r = accumulator component) of channel oc0 + 16w + l16 ---------
    // The byte offsets of a tile's four pixels (channel 0; beyond the descriptor where the tile or the pixel does not
    // exist) are computed once per item by 32 threads, in the shadow of the item's first step, and kept in LDS:
    // otab[item parity][tile][4]. The output transform then costs one LDS read and four additions per tile for addresses.
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.Y, 0, p.y_bytes, 0x00020000);
    unsigned *otab = reinterpret_cast<unsigned *>(smem + 2 * WS_VBUF);
    auto write_offset_table = [&](const Item &it, int parity) {
        const int tile = it.tile_first + (t & 31);
        const bool ok = tile < it.tile_end;
        const int n = fdiv(tile, p.d_TRC), rem = tile - n * p.TRC;
        const int ty = fdiv(rem, p.d_TC), tx = rem - ty * p.TC;
        const int oh = 2 * ty, ow = 2 * tx;
        const unsigned row4 = (unsigned)p.OW * p.OC * 4u, px4 = (unsigned)p.OC * 4u;
        const unsigned o = (unsigned)(((n * p.OH + oh) * p.OW + ow) * p.OC) * 4u;
        const bool right = ok && ow + 1 < p.OW, below = ok && oh + 1 < p.OH;
        uint4 e;
        e.x = ok ? o : WS_OOR;
        e.y = right ? o + px4 : WS_OOR;
        e.z = below ? o + row4 : WS_OOR;
        e.w = (right && below) ? o + row4 + px4 : WS_OOR;
        if (t < 32) *reinterpret_cast<uint4 *>(otab + parity * 128 + t * 4) = e;
    };
    float bias_v = 0.f;     // of the current item's channel
    unsigned col4 = 0;      // its byte offset; 1 GB (beyond the descriptor, also when added to WS_OOR) for channels >= OC
    auto item_column = [&](const Item &it) {
        const int col = it.oc0 + 16 * w + l16;
        const bool col_ok = col < p.OC;
        col4 = col_ok ? (unsigned)col * 4u : 0x40000000u;
        bias_v = 0.f;
        if (p.bias) bias_v = p.bias[col_ok ? col : 0];
    };
    auto store_item = [&](auto half_c, int parity) {
        constexpr bool HALF = decltype(half_c)::value;
#pragma unroll
        for (int mt = 0; mt < 2; mt++) {
            if (mt == 1 && HALF) break;
#pragma unroll
            for (int rr = 0; rr < 4; rr++) {
                const uint4 o = *reinterpret_cast<const uint4 *>(otab + parity * 128 + (16 * mt + 4 * q + rr) * 4);
                // Y = A^T m A, A^T = [[1,1,1,0],[0,1,-1,-1]], m[a][c] = acc[4a + c]
                float s0[4], s1[4];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const float m0 = acc[c][mt][rr], m1 = acc[4 + c][mt][rr], m2 = acc[8 + c][mt][rr], m3 = acc[12 + c][mt][rr];
                    s0[c] = m0 + m1 + m2;
                    s1[c] = m1 - m2 - m3;
                }
                const float y00 = s0[0] + s0[1] + s0[2] + bias_v, y01 = s0[1] - s0[2] - s0[3] + bias_v;
                const float y10 = s1[0] + s1[1] + s1[2] + bias_v, y11 = s1[1] - s1[2] - s1[3] + bias_v;
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, y00), y_rsrc, o.x + col4, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, y01), y_rsrc, o.y + col4, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, y10), y_rsrc, o.z + col4, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, y11), y_rsrc, o.w + col4, 0, 0);
            }
        }
    };

    // ---- start: V of step 0, the patch of step 1 on its way, the ring filled ------------------------------------------
    Item cur = item_of(0);
    int pk = 0, pc = 0;   // patch cursor: item and chunk of the patch in d
    auto advance_patch_cursor = [&]() {   // one step on; a new item brings new pixel offsets
        pc++;
        if (pc == nchunks) {
            pc = 0;
            pk++;
            if (pk < nitems) patch_offsets(item_of(pk));   // beyond the last step: patches nobody multiplies, valid addresses
        }
    };
    patch_offsets(cur);
    load_patch(0);
    transform_columns();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        transform_half_row_store(smem + xt * 16 + xq, i, 0);
        transform_half_row_store(smem + xt * 16 + xq, i, 1);
    }
    advance_patch_cursor();
    load_patch(pc * 16);
    {
        const unsigned u0 = (unsigned)cur.oc0 * 16u;
#pragma unroll
        for (int x = 0; x < 4; x++) load_b(bring[x], u0 + x * xi_stride4);
    }
    __syncthreads();

    // ---- one step: 16 xi x (2 LDS fragments, 4 filter elements, 8 MFMAs); in their shadow the next step's V ----------
    // Every xi is a scheduling region of its own (nothing crosses its borders), in program order: the LDS fragments of
    // the next xi, the ring refill, 8 MFMAs, and a slice of the preparation of the steps to come. Left to itself the
    // scheduler dissolves the ring (loads issued right before their use) and moves the patch loads to the end of the
    // step and their transform to the start of the next one, with nothing in between to cover the latency. The slices
    // are thin because the four wavefronts of a compute unit run in step and share its memory pipelines: 16 patch loads
    // or 8 LDS writes per wavefront at one place keep them all waiting (measured: 930 and 570 cycles of a 6300-cycle
    // step); two loads and one write per xi pass unnoticed.
    //   xi 0      columns of B^T d B for the next step's patch (it arrived during the last step)
    //   xi 1-8    half a row of the transform each: 2 of the 16 V positions written to the other LDS buffer
    //   xi 2      the patch cursor moves on to the step after the next
    //   xi 3-10   two of its 16 loads each, into the registers the finished rows have left
    //   xi 12     first step of an item only: the item's output offsets into LDS
    auto chunk = [&](auto half_c, auto first_c, int buf, unsigned ucur, unsigned unext, int k) {
        constexpr bool HALF = decltype(half_c)::value;
        constexpr bool FIRST = decltype(first_c)::value;   // first step of an item: the accumulators start from zero
        const float *V = smem + buf * WS_VBUF + l16 * 16 + 4 * q;
        float *Vw = smem + (buf ^ 1) * WS_VBUF + xt * 16 + xq;
        floatx4 a0 = *reinterpret_cast<const floatx4 *>(V);
        floatx4 a1 = a0;
        if (!HALF) a1 = *reinterpret_cast<const floatx4 *>(V + 16 * 16);
        const floatx4 zero = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int xi = 0; xi < 16; xi++) {
            __builtin_amdgcn_sched_barrier(0);
            floatx4 a0n = a0, a1n = a1;
            if (xi < 15) {
                a0n = *reinterpret_cast<const floatx4 *>(V + (xi + 1) * WS_TILES * 16);
                if (!HALF) a1n = *reinterpret_cast<const floatx4 *>(V + (xi + 1) * WS_TILES * 16 + 16 * 16);
            }
            const floatx4 bb = bring[xi & 3];
            {   // refill this ring slot with the fragment needed four positions later (possibly in the next step)
                const int nx = xi + 4;
                load_b(bring[xi & 3], nx < 16 ? ucur + nx * xi_stride4 : unext + (nx - 16) * xi_stride4);
            }
#pragma unroll
            for (int s = 0; s < 4; s++) {
                acc[xi][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[s], bb[s], (FIRST && s == 0) ? zero : acc[xi][0], 0, 0, 0);
                if (!HALF) acc[xi][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[s], bb[s], (FIRST && s == 0) ? zero : acc[xi][1], 0, 0, 0);
            }
            if (xi == 0) transform_columns();
            if (xi >= 1 && xi <= 8) transform_half_row_store(Vw, (xi - 1) >> 1, (xi - 1) & 1);
            if (xi == 2) advance_patch_cursor();
            if (xi >= 3 && xi <= 10) {
                load_patch_element(2 * (xi - 3), pc * 16);
                load_patch_element(2 * (xi - 3) + 1, pc * 16);
            }
            if (FIRST && xi == 12) write_offset_table(cur, k & 1);
            // order inside the region: each MFMA is followed by at most one memory instruction of each kind and a few
            // vector ALU instructions, so that no run of them is longer than the MFMA in front of it
#pragma unroll
            for (int m = 0; m < 8; m++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // 1 MFMA
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // 1 load from memory
                __builtin_amdgcn_sched_group_barrier(0x080, 1, 0);   // 1 LDS instruction
                __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);   // vector ALU
            }
            a0 = a0n;
            a1 = a1n;
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // whole items first, then the half item if this workgroup has one: two copies of the steps, one after the other
    int buf = 0;
    auto run_item = [&](auto half_c, int k) {
        const bool has_next = k + 1 < nitems;
        Item nxt = cur;
        if (has_next) nxt = item_of(k + 1);
        item_column(cur);
        const unsigned u_item = (unsigned)cur.oc0 * 16u;
        const unsigned u_after = has_next ? (unsigned)nxt.oc0 * 16u : 0u;   // where the ring goes on after this item
        chunk(half_c, std::true_type{}, buf, u_item, nchunks > 1 ? u_item + chunk_stride4 : u_after, k);
        __syncthreads();
        buf ^= 1;
        for (int c = 1; c < nchunks; c++) {
            const unsigned ucur = u_item + c * chunk_stride4;
            chunk(half_c, std::false_type{}, buf, ucur, c + 1 < nchunks ? ucur + chunk_stride4 : u_after, k);
            __syncthreads();
            buf ^= 1;
        }
        store_item(half_c, k & 1);
        cur = nxt;
    };
    const int nfull = has_half ? nitems - 1 : nitems;
    for (int k = 0; k < nfull; k++) run_item(std::false_type{}, k);
    if (nfull < nitems) run_item(std::true_type{}, nfull);
}

hipError_t launch_winograd_stream(hipStream_t stream, const float *X, const float *U, float *Y,
                                  int N, int IH, int IW, int IC, int OH, int OW, int OC, int ph, int pw, const float *bias)
{
    if (OH != IH + 2 * ph - 2 || OW != IW + 2 * pw - 2) return hipErrorNotSupported;
    if (IC < 16 || IC % 16 != 0 || OC < 1 || N < 1 || OH < 1 || OW < 1) return hipErrorNotSupported;
    if (!winograd_forward_fits(N, IH, IW, IC, OH, OW, OC)) return hipErrorNotSupported;
    const long x_bytes = (long)N * IH * IW * IC * 4, y_bytes = (long)N * OH * OW * OC * 4, u_bytes = 16L * IC * OC * 4;
    if (x_bytes >= (1L << 31) || y_bytes > (1L << 30) || u_bytes >= (1L << 31)) return hipErrorNotSupported;
    const int cus = device_cu_count();
    if (cus < 1) return hipErrorNotSupported;

    WinoStreamArgs a{};
    a.X = X; a.U = U; a.Y = Y; a.bias = bias;
    a.IH = IH; a.IW = IW; a.IC = IC; a.OH = OH; a.OW = OW; a.OC = OC; a.ph = ph; a.pw = pw;
    a.TC = (OW + 1) / 2;
    a.TRC = ((OH + 1) / 2) * a.TC;
    const long nt = (long)N * a.TRC;
    if (nt >= (1L << 30)) return hipErrorNotSupported;
    a.ntiles = (int)nt;
    a.groups = (a.ntiles + WS_TILES - 1) / WS_TILES;
    a.x_bytes = (int)x_bytes; a.y_bytes = (int)y_bytes; a.u_bytes = (int)u_bytes;
    a.d_TC = make_fastdiv(a.TC);
    a.d_TRC = make_fastdiv(a.TRC);
    a.d_groups = make_fastdiv(a.groups);
    const long items = (long)a.groups * ((OC + 63) / 64);
    if (items >= (1L << 30)) return hipErrorNotSupported;
    // The items beyond a whole number per workgroup go out as halves as far as the workgroups reach - a workgroup takes one
    // more item or one half -: `left` items on `grid` workgroups are 2 left - grid whole ones and 2 (grid - left) halves when
    // left > grid / 2, else 2 left halves (28x28x128 at N = 64, 784 items on 512 workgroups: 32 + 480 instead of 272 whole
    // ones, 0.068 -> 0.062 ms). Fewer items than workgroups: one each - as halves on twice the workgroups every half streams
    // the item's filter again, and the layers with few items are the ones with large filters (7x7x512 at N = 64, 256 items:
    // 0.069 ms whole, 0.078 ms in halves).
    const int slots = 2 * cus;
    const int grid = items < slots ? (int)items : slots;
    a.whole = (int)(items / grid);
    const int left = (int)(items - (long)a.whole * grid);   // < grid
    if (2 * left <= grid) {
        a.halves = 2 * left;
    } else {
        a.extra = 2 * left - grid;
        a.halves = 2 * (grid - left);
    }

    constexpr auto kern = winograd_stream_kernel;
    const size_t lds = (size_t)2 * WS_VBUF * sizeof(float) + 2 * WS_TILES * 4 * sizeof(unsigned);   // V[2], otab[2]
    if (hipError_t e = ensure_dynamic_lds<kern>(lds); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, stream, a);
    return hipGetLastError();
}

}  // namespace alpha
