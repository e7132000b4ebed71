// 3x3 / stride 1 / pad 1 convolution on NHWC fp32 tensors by the Winograd minimal-filtering
// algorithm F(2x2, 3x3) (Lavin & Gray, "Fast Algorithms for Convolutional Neural Networks",
// 2015), for the convolution layers of the VGG16 stages (vgg16/gpus=4_straight/stage0.py:12-14).
// The third-party library behind the reference's torch.nn.Conv2d picks the same family of
// algorithms for fp32 3x3 filters.
//
//   Y = A^T [ (G g G^T) .* (B^T d B) ] A        per 2x2 output tile and (in, out) channel pair,
//
// which turns the convolution into 16 independent GEMMs (one per position of the 4x4 transformed
// tile) of shape [tiles x C] * [C x K]: 16 multiplies per 4 outputs instead of 36, i.e. 2.25x
// fewer MFMA operations than the direct kernel.  All arithmetic is fp32; the transforms only add,
// subtract and halve, and the result differs from a direct fp32 convolution by about one more
// rounding error (measured 2e-6 against 1e-6 on unit-scale data).
//
// One persistent kernel does everything between the NHWC input and the NHWC output:
//   * a block (512 threads, one per CU) owns work items of 16 x 16 output pixels (64 tiles) x 64
//     output channels and walks the input channels in chunks of 8;
//   * the 18 x 18 x 8-channel input halo tile of a chunk is fetched once (32-byte pixel segments) and
//     parked in LDS; the input transform B^T d B is computed from there by all threads and written
//     back to LDS in the order in which the MFMA A-fragments are read (one contiguous 1 KB per wave
//     and fragment: no bank conflicts on either side);
//   * the transformed filter U = G g G^T is prepared once per call by a small kernel, in the exact
//     order in which a wave needs it, so every B-fragment is one coalesced 1 KB global load into
//     registers (reloaded right after its last use) and never touches LDS;
//   * a wave keeps 8 of the 16 GEMM accumulators of its 32 tiles x 32 channels (128 registers per
//     lane): two waves per SIMD, so that one wave's loads, transforms and LDS traffic run while the
//     other's MFMAs execute -- a single wave issues in order and cannot overlap them itself.  The two
//     waves that share a (tiles, channels) block each apply the output transform A^T M A to their
//     rows of M (it is linear) and the partial results are added in the LDS staging tile; bias, ReLU
//     and the optional output mask follow as the tile is stored as whole NHWC pixel rows.
#include <type_traits>

#include "pd_internal.h"

namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int WG_THREADS = 512;
constexpr int WG_PIX = 16;                       // a block covers WG_PIX x WG_PIX output pixels
constexpr int WG_TILES = 64;                     // = 8 x 8 tiles of 2 x 2 pixels
constexpr int WG_BN = 64;                        // output channels per block
constexpr int WG_CC = 8;                         // input channels per reduction chunk
constexpr int WG_G = 16;                         // positions of the transformed 4 x 4 tile
constexpr int WG_GW = 8;                         // ... of which a wave accumulates 8
constexpr int WG_FRAG = 256;                     // floats in one wave-wide fragment (64 lanes x 4)
constexpr int WG_V_STAGE = WG_G * 2 * WG_FRAG;   // floats of transformed input per chunk: [g][wm][lane][4]
constexpr int WG_OP = WG_BN + 4;                 // pitch of the output staging tile
constexpr int WG_XCD = 8;
constexpr int WG_HALO = WG_PIX + 2;              // input halo tile: 18 rows x (16 + 2 per segment) pixels
// The halo tile in LDS: four planes (channel half, column parity) of 18 rows x 12 16-byte units; the
// unit of (half, row, col) is ((half * 2 + (col & 1)) * 18 + row) * 12 + (col >> 1).  The eight tiles
// of a tile row then read eight consecutive units and the next tile row lands 8 units further
// (mod 16): a wave's 128-bit reads of one patch position are free of bank conflicts.
// Each plane ends with two units of zeros (what a stacked batch's tiles read for the patch row that lies in the
// neighbouring image).
//
// Segments.  A work item's 16 x 16 pixels need not be one square of the image: with SEG = 2 (4) they are two (four)
// pieces of 16 rows x 8 (4) columns, consecutive in a row-major numbering of all such pieces of the stacked batch.
// An image width of 56 (28) pixels is then covered exactly by 7 pieces per 16 rows instead of 4 (2) squares of
// which the last is half (a quarter) empty.  Every piece has its own halo, so the halo tile is 18 rows x
// (16 + 2 SEG) columns, the pieces' halos side by side; a tile of piece s finds its patch s units further right.
constexpr int WG_RAW_PITCH = 12;
constexpr int WG_PLANE = WG_HALO * WG_RAW_PITCH + 2;           // 16-byte units of one plane
constexpr int WG_RAW_STAGE = 4 * WG_PLANE * 4;                 // floats
// LDS map (floats): two stages of transformed input, two stages of raw halo tile, output staging tile
constexpr int WG_RAW_OFF = 2 * WG_V_STAGE;
constexpr int WG_OUT_OFF = WG_RAW_OFF + 2 * WG_RAW_STAGE;
constexpr int WG_LDS_FLOATS = WG_OUT_OFF + 256 * WG_OP;
static_assert(WG_LDS_FLOATS * 4 <= 160 * 1024, "LDS budget of one CU");

struct WinoArgs {
    const float* x;         // [N,H,W,C]
    const float* u;         // transformed filter, see winograd_filter_kernel
    const float* bias;      // [K] or null
    const float* mask;      // [N,H,W,C] or null: x is taken as 0 where mask <= 0
    const float* out_mask;  // [N,H,W,K] or null: y is written as 0 where out_mask <= 0
    float* y;               // [N,H,W,K]
    float* pool_y;          // pooling variant: [N,H/2,W/2,K], written instead of y
    uint8_t* pool_idx;      // pooling variant: [N,H/2,W/2,K] window position (bits 0-1) and sign (bit 2)
    const uint8_t* unpool_idx;   // unpooling variant: [N,H,W,K] index bytes of the 2x2 pooling that produced this
                                 // convolution's input (the convolution is an input gradient)
    float* unpool_y;        // unpooling variant: [N,2H,2W,K], the gradient in front of that pooling
    int N, H, W, C, K;
    int img_h;              // stacked variant: rows of one image (N is then 1 and H the rows of the whole batch)
    int relu;
    int tiles_x, tiles_y, k_blocks, n_chunks;
    int segs_per_row, n_segs;     // segmented variant: pieces per 16 rows of the stacked batch, pieces in all
    int n_items, items_per_xcd;   // work items (pixel tile x channel block) in all / per die
};

// U = G g G^T for every (out channel k, in channel c), G = [[1,0,0],[.5,.5,.5],[.5,-.5,.5],[0,0,1]].
// Output order: [k / 64][c / 8][g][(k % 64) / 32][(c % 8) / 4][k % 32][c % 4] -- for a block's 64
// channels and one chunk, position g, the two 1 KB halves are exactly what the lanes of the waves
// with wn = 0 / 1 load (lane = 32 * ((c % 8) / 4) + k % 32 holds four consecutive c).  Rows
// k >= K of the last block of 64 are zero.  With rot180 the filter is taken as
// f[k][r][s][c] = w[c][2-r][2-s][k] (w is then [C][3][3][K]): the input-gradient filter.
//
// One thread transforms the filters of one out channel and four consecutive in channels, so a wave is
// one of those 1 KB halves and each of its 16 stores is one contiguous kilobyte.  The four waves of a
// block take four neighbouring chunks where C allows, so that the block reads whole 128-byte lines of w.
// vec: w is 16-byte aligned (128-bit loads along c).
__device__ __forceinline__ float4 wf_half_sum(float4 a, float4 b, float4 c) {
    return make_float4(0.5f * (a.x + b.x + c.x), 0.5f * (a.y + b.y + c.y), 0.5f * (a.z + b.z + c.z),
                       0.5f * (a.w + b.w + c.w));
}
__device__ __forceinline__ float4 wf_half_alt(float4 a, float4 b, float4 c) {
    return make_float4(0.5f * (a.x - b.x + c.x), 0.5f * (a.y - b.y + c.y), 0.5f * (a.z - b.z + c.z),
                       0.5f * (a.w - b.w + c.w));
}

__global__ __launch_bounds__(256) void winograd_filter_kernel(const float* __restrict__ w, float* __restrict__ u,
                                                              int K, int C, int k_pad, int rot180, int vec) {
    const int n_chunks = C / WG_CC;
    const long unit = (long)blockIdx.x * 4 + threadIdx.x / 64;   // (block of 64 k, chunk, half of the block)
    if (unit >= (long)(k_pad / 32) * n_chunks) return;
    int half, chunk;
    if (n_chunks % 4 == 0) {
        chunk = (int)(unit % 4) + 4 * (int)((unit / 8) % (n_chunks / 4));
        half = (int)((unit / 4) % 2);
    } else {
        half = (int)(unit % 2);
        chunk = (int)((unit / 2) % n_chunks);
    }
    const int kb = (int)(unit / (2 * n_chunks));
    const int lane = threadIdx.x % 64;
    const int k = kb * WG_BN + half * 32 + lane % 32;
    const int c0 = chunk * WG_CC + (lane / 32) * 4;
    float4 g[3][3];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int s = 0; s < 3; ++s) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (k < K) {
                if (rot180) {
                    const float* src = w + ((size_t)c0 * 9 + (2 - r) * 3 + (2 - s)) * K + k;
                    v = make_float4(src[0], src[(size_t)9 * K], src[(size_t)18 * K], src[(size_t)27 * K]);
                } else {
                    const float* src = w + ((size_t)k * 9 + r * 3 + s) * C + c0;
                    if (vec) v = *reinterpret_cast<const float4*>(src);
                    else v = make_float4(src[0], src[1], src[2], src[3]);
                }
            }
            g[r][s] = v;
        }
    float4 t[4][3];
#pragma unroll
    for (int s = 0; s < 3; ++s) {
        t[0][s] = g[0][s];
        t[1][s] = wf_half_sum(g[0][s], g[1][s], g[2][s]);
        t[2][s] = wf_half_alt(g[0][s], g[1][s], g[2][s]);
        t[3][s] = g[2][s];
    }
    float* dst = u + ((size_t)(kb * n_chunks + chunk) * WG_G) * (2 * WG_FRAG) + half * WG_FRAG + lane * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float4 o[4] = {t[i][0], wf_half_sum(t[i][0], t[i][1], t[i][2]),
                             wf_half_alt(t[i][0], t[i][1], t[i][2]), t[i][2]};
#pragma unroll
        for (int m = 0; m < 4; ++m)
            *reinterpret_cast<float4*>(dst + (size_t)(i * 4 + m) * (2 * WG_FRAG)) = o[m];
    }
}

// Decoded work item: one 16 x 16 pixel tile of one image x one block of 64 output channels.
struct WinoItem { int n, y0, x0, kb; };

__device__ __forceinline__ WinoItem wino_decode(const WinoArgs& a, int item) {
    WinoItem w;
    w.kb = item % a.k_blocks;
    const int tile = item / a.k_blocks;
    const int per_img = a.tiles_x * a.tiles_y;
    w.n = tile / per_img;
    const int rem = tile - w.n * per_img;
    const int ty = rem / a.tiles_x;
    w.y0 = ty * WG_PIX;
    w.x0 = (rem - ty * a.tiles_x) * WG_PIX;
    return w;
}

// Piece s of a work item: first output row and column, and whether it exists (the last item may have fewer).
// SEG = 1: the item's square.
struct SegPos { int y0, x0; bool ok; };
template <int SEG>
__device__ __forceinline__ SegPos seg_pos(const WinoArgs& a, int item, int s) {
    SegPos p;
    if (SEG == 1) {
        const WinoItem w = wino_decode(a, item);
        p.y0 = w.y0; p.x0 = w.x0; p.ok = true;
    } else {
        const int sg = (item / a.k_blocks) * SEG + s;
        const int rb = sg / a.segs_per_row;
        p.y0 = rb * WG_PIX;
        p.x0 = (sg - rb * a.segs_per_row) * (WG_PIX / SEG);
        p.ok = sg < a.n_segs;
    }
    return p;
}

// Persistent kernel: gridDim.x (a multiple of 8, at most one block per CU) blocks share the work items.
// Block b lives on die b % 8 and takes the items  (b % 8) * items_per_xcd + b / 8 + i * gridDim.x / 8,
// i = 0, 1, ...: at any time the blocks of one die work on neighbouring items (the channel blocks of one
// pixel tile, then the next tile), which share input and filter lines in that die's L2.
//
// The reduction chunks of all of a block's items form one sequence of steps that runs through a
// three-stage pipeline without draining between items:
//   stage 1 (steps q+3, q+2): the halo tile travels global -> registers (a whole step in flight) -> LDS;
//             the mask, if any, and the zero padding are applied on the way,
//   stage 2 (step q+1): every thread reads 2 x 4 pixels of its tile's patch from that LDS tile, forms one
//             row of B^T d, applies . B and writes the 4 transformed vectors where the MFMA fragments are
//             read from,
//   stage 3 (step q): 32 MFMAs per wave, with each filter fragment reloaded (for step q+1) after its
//             last use.
// One barrier per step.  After the last chunk of an item: output transform, cross-wave sum in LDS, bias,
// ReLU, output mask and 128-bit NHWC stores.
//
// STACKED: the batch is taken as one image of N * img_h rows (NHWC images follow each other in memory
// row after row), so that work items straddle images instead of padding every image to a multiple of
// 16 rows.  img_h is even, hence no 2 x 2 tile straddles two images; a tile in the first (last) tile row
// of an image must see zeros in the first (last) row of its 4 x 4 patch, where the stacked layout holds
// the neighbouring image's row.  Only the threads that form row 0 (d0 - d2) resp. row 3 (d1 - d3) of
// B^T d read those rows: for such a tile their row pointer goes to a patch of zeros in LDS (the two units
// behind a plane's rows, which no piece is ever written to) -- set once per work item, nothing per step.
//
// UNPOOL: the launch computes the input gradient of a convolution whose input came out of a 2 x 2 max
// pooling with index bytes (the pooling epilogue above, or the pooling kernel).  The epilogue then also
// applies that pooling's backward: every value goes to its window's recorded position in the
// full-resolution gradient if the recorded maximum was positive (the ReLU in front of the pooling), the
// window's other three positions get zeros, and y itself is stored with the same mask -- what the
// pooling backward kernel would compute from y, without the kernel and without its re-read of y.
template <bool MASK, bool POOL, bool STACKED, bool UNPOOL = false, int SEG = 1>
__global__ __launch_bounds__(WG_THREADS, 1) void winograd_fwd_kernel(const WinoArgs a) {
    static_assert(SEG == 1 || (STACKED && !MASK), "segments go with the stacked batch");
    constexpr int SEGW = WG_PIX / SEG;           // columns of a piece
    constexpr int HALO_W = WG_PIX + 2 * SEG;     // columns of the halo tile
    constexpr int PIECES = WG_HALO * HALO_W * 2; // 16-byte pieces (pixel, 4-channel half) of one chunk of it
    static_assert(PIECES <= 2 * WG_THREADS && HALO_W <= 2 * WG_RAW_PITCH, "halo tile");
    __shared__ __attribute__((aligned(16))) float lds[WG_LDS_FLOATS];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gx8 = gridDim.x / WG_XCD;
    const int xcd = blockIdx.x % WG_XCD, slot = blockIdx.x / WG_XCD;
    const int item0 = xcd * a.items_per_xcd + slot;
    int lim = a.n_items - xcd * a.items_per_xcd;
    lim = lim < a.items_per_xcd ? lim : a.items_per_xcd;            // items of this die
    const int n_my = slot < lim ? (lim - slot + gx8 - 1) / gx8 : 0;
    if (n_my == 0) return;                                           // whole block, before any barrier

    // ---- stage 1 role: pieces p = tid and tid + 512 of the halo tile; piece = (halo pixel, channel half)
    int hy[2], hx[2], hseg[2], raw_dst[2];       // (hx: column inside the piece's own halo; hseg: the piece)
    uint32_t pcg[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int p = tid + WG_THREADS * j, pix = p >> 1, half = p & 1;
        hy[j] = pix / HALO_W;
        const int col = pix - hy[j] * HALO_W;
        hseg[j] = SEG == 1 ? 0 : col / (SEGW + 2);
        hx[j] = col - hseg[j] * (SEGW + 2);
        pcg[j] = half * 16;
        raw_dst[j] = ((half * 2 + (col & 1)) * WG_PLANE + hy[j] * WG_RAW_PITCH + (col >> 1)) * 4;
    }
    const bool second_piece = tid + WG_THREADS < PIECES;
    const float* ximg = a.x;
    const float* mimg = MASK ? a.mask : a.x;
    const uint32_t img_bytes = (uint32_t)a.H * a.W * a.C * 4;
    uint32_t loff[2];
    // byte offsets of the thread's pieces for the i-th item of this block; padding (and everything
    // past the last item) gets an offset beyond the buffer's size, for which a buffer load returns 0
    auto set_load_item = [&](int i) {
        if (i < n_my) {
            if (SEG == 1) {
                const size_t img = (size_t)wino_decode(a, item0 + i * gx8).n * a.H * a.W * a.C;
                ximg = a.x + img;
                if (MASK) mimg = a.mask + img;
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const SegPos sp = seg_pos<SEG>(a, item0 + i * gx8, hseg[j]);
                const int gy = sp.y0 - 1 + hy[j], gx = sp.x0 - 1 + hx[j];
                loff[j] = (sp.ok && gy >= 0 && gy < a.H && gx >= 0 && gx < a.W && (j == 0 || second_piece))
                              ? (uint32_t)((gy * a.W + gx) * a.C) * 4 + pcg[j] : 0x80000000u;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 2; ++j) loff[j] = 0x80000000u;
        }
    };
    float4_t rawr[2], rawm[MASK ? 2 : 1];
    auto load_raw = [&](int chunk) {
        const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void*)ximg, 0, img_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t mr = __builtin_amdgcn_make_buffer_rsrc((void*)mimg, 0, img_bytes, 0x00020000);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            rawr[j] = __builtin_bit_cast(float4_t,
                                         __builtin_amdgcn_raw_buffer_load_b128(xr, loff[j], chunk * (WG_CC * 4), 0));
            if (MASK)
                rawm[MASK ? j : 0] = __builtin_bit_cast(
                    float4_t, __builtin_amdgcn_raw_buffer_load_b128(mr, loff[j], chunk * (WG_CC * 4), 0));
        }
    };
    auto store_raw_at = [&](float* dst, int j) {
        float4_t v = rawr[j];
        if (MASK) {
#pragma unroll
            for (int c = 0; c < 4; ++c) v[c] = rawm[MASK ? j : 0][c] > 0.f ? v[c] : 0.f;
        }
        if (j == 0 || second_piece) *(float4_t*)dst = v;
    };
    auto store_raw = [&](int stage, int j) {
        store_raw_at(lds + WG_RAW_OFF + stage * WG_RAW_STAGE + raw_dst[j], j);
    };

    // ---- stage 2 role: tile tt, channel half cg and row ti of B^T d, which is  Ra + sgn * Rb  of two
    //      of the tile's four input rows: d0-d2, d1+d2, d2-d1, d1-d3 ------------------------------------
    const int ti = wave & 3;
    const int twm = wave >> 2;                 // which half of the tiles (= wm of the consuming waves)
    const int cg = lane >> 5;
    const int tt = twm * 32 + (lane & 31);
    const int row_a = ti == 0 ? 0 : ti == 2 ? 2 : 1;
    const int row_b = ti == 2 ? 1 : ti == 3 ? 3 : 2;
    const float sgn = ti == 1 ? 1.f : -1.f;
    const int tseg = SEG == 1 ? 0 : (tt & 7) / (8 / SEG);     // the piece the thread's tile belongs to
    const int unit0 = cg * 2 * WG_PLANE + 2 * (tt >> 3) * WG_RAW_PITCH + (tt & 7) + tseg;
    const int src_a = (unit0 + row_a * WG_RAW_PITCH) * 4, src_b = (unit0 + row_b * WG_RAW_PITCH) * 4;
    // row offsets of the thread's tile in the i-th item of this block: src_a / src_b, or the zeros
    auto patch_rows = [&](int i, int& oa, int& ob) {
        oa = src_a;
        ob = src_b;
        if (STACKED && i < n_my) {
            const int r0 = seg_pos<SEG>(a, item0 + i * gx8, tseg).y0 + 2 * (tt >> 3);   // the tile's first output row
            const int zeros = (cg * 2 * WG_PLANE + WG_HALO * WG_RAW_PITCH) * 4;
            if (ti == 0 && r0 % a.img_h == 0) oa = zeros;
            if (ti == 3 && (r0 + 2) % a.img_h == 0) ob = zeros;
        }
    };
    float4_t t[4];
    float4_t dc[2][2];                         // column s of the patch waits in dc[s & 1] until its section
    auto read_col_at = [&](const float* ra, const float* rb, int s) {   // the same through per-lane pointers
        const int o = ((s & 1) * WG_PLANE + (s >> 1)) * 4;
        dc[s & 1][0] = *(const float4_t*)(ra + o);
        dc[s & 1][1] = *(const float4_t*)(rb + o);
    };
    auto transform_col = [&](int s) { t[s] = dc[s & 1][0] + sgn * dc[s & 1][1]; };
    float4_t vout;
    auto transform_out = [&](int m) {
        if (m == 0) vout = t[0] - t[2];
        else if (m == 1) vout = t[1] + t[2];
        else if (m == 2) vout = t[2] - t[1];
        else vout = t[1] - t[3];
    };
    auto store_out = [&](float* vst, int m) {
        *(float4_t*)(vst + (ti * 4 + m) * (2 * WG_FRAG) + twm * WG_FRAG + lane * 4) = vout;
    };
    auto store_out_at = [&](float* pv, int m) { *(float4_t*)(pv + m * (2 * WG_FRAG)) = vout; };

    // ---- stage 3 role: wave (gh, wm, wn) owns GEMMs gh*8..+7 of tiles wm*32..+31 x channels wn*32..+31
    const int gh = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1;
    const __amdgpu_buffer_rsrc_t ur = __builtin_amdgcn_make_buffer_rsrc(
        (void*)a.u, 0, (uint32_t)a.k_blocks * a.n_chunks * WG_G * (2 * WG_FRAG) * 4, 0x00020000);
    const uint32_t u_lane = (uint32_t)((gh * WG_GW * 2 + wn) * WG_FRAG + lane * 4) * 4;
    auto load_u = [&](int ustep, int gl) {   // ustep = kb * n_chunks + chunk
        return __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                                ur, u_lane, (ustep * WG_G + gl) * (2 * WG_FRAG * 4), 0));
    };
    const int a_lane = (gh * WG_GW * 2 + wm) * WG_FRAG + lane * 4;

    float16_t acc[WG_GW];
    float4_t uf[WG_GW];
    auto zero_acc = [&]() {
#pragma unroll
        for (int g = 0; g < WG_GW; ++g)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[g][e] = 0.f;
    };

    // cursors: (index in this block's item list, chunk) of the step each stage works on next
    int l_i = 0, l_cc = 0;                     // stage 1 (raw loads)
    int u_i = 0, u_cc = 0, u_kb;               // filter fragments
    auto advance_l = [&]() {
        if (++l_cc == a.n_chunks) { l_cc = 0; set_load_item(++l_i); }
    };
    auto advance_u = [&]() {                   // stays on the last step once the sequence ends
        if (u_cc + 1 < a.n_chunks) ++u_cc;
        else if (u_i + 1 < n_my) { u_cc = 0; u_kb = wino_decode(a, item0 + (++u_i) * gx8).kb; }
    };

    // ---- prologue: steps 0 and 1 into LDS, step 2 into registers, step 0 transformed
    set_load_item(0);
    u_kb = wino_decode(a, item0).kb;
    load_raw(l_cc);
    advance_l();
#pragma unroll
    for (int g = 0; g < WG_GW; ++g) uf[g] = load_u(u_kb * a.n_chunks + u_cc, g);
    advance_u();
    store_raw(0, 0);
    store_raw(0, 1);
    load_raw(l_cc);
    advance_l();
    store_raw(1, 0);
    store_raw(1, 1);
    load_raw(l_cc);
    advance_l();
    if (STACKED && tid < 64) {                 // the zeros: the two units behind the rows of the 4 planes, both stages
        const int stage = tid >> 5, plane = (tid >> 3) & 3, e = tid & 7;
        lds[WG_RAW_OFF + stage * WG_RAW_STAGE + (plane * WG_PLANE + WG_HALO * WG_RAW_PITCH) * 4 + e] = 0.f;
    }
    // patch rows of the step that stage 2 reads next: item p_i of this block, chunk p_cc
    int p_i = 0, p_cc = 0;
    const float* pra;
    const float* prb;
    auto set_patch_rows = [&](int stage) {
        int oa, ob;
        patch_rows(p_i, oa, ob);
        pra = lds + WG_RAW_OFF + stage * WG_RAW_STAGE + oa;
        prb = lds + WG_RAW_OFF + stage * WG_RAW_STAGE + ob;
    };
    auto advance_p = [&](int stage) {          // (pra, prb have just moved to that stage)
        if (++p_cc == a.n_chunks) {
            p_cc = 0;
            ++p_i;
            set_patch_rows(stage);
        }
    };
    set_patch_rows(0);
    __syncthreads();
#pragma unroll
    for (int s = 0; s < 4; ++s) { read_col_at(pra, prb, s); transform_col(s); }
#pragma unroll
    for (int m = 0; m < 4; ++m) { transform_out(m); store_out(lds, m); }
    __syncthreads();
    float4_t af[2][2];                         // A fragments of GEMM pair p wait in af[p & 1] for one section
    af[0][0] = *(const float4_t*)(lds + a_lane);
    af[0][1] = *(const float4_t*)(lds + a_lane + (2 * WG_FRAG));
    pra += WG_RAW_STAGE;                       // step 1 sits in the second stage
    prb += WG_RAW_STAGE;
    if (STACKED) advance_p(1);
    read_col_at(pra, prb, 0);

    // Per step: four sections of 8 MFMAs (GEMM pair gp) each, every MFMA followed by a small piece of
    // the other stages' work; the scheduler may not move anything across the sub-step boundaries.  LDS
    // reads are issued at least one section before their use.  The step's barrier sits in the last
    // section, which then requests the first fragments and patch column of the next step while its own
    // MFMAs (operands already in registers) run.  The reduction index of MFMA j pairs channel j (lanes
    // 0-31) with channel 4+j (lanes 32-63).
    // The LDS stages alternate with the parity of the step.  Every per-lane address that depends on it is a
    // pointer carried through the loop and moved to the other stage once per step, after its last use in the
    // step (one vector addition each, instead of rebuilding index * 4 + stage offset for every use).
    int q = 0;                                 // step of stage 3
    int dv = WG_V_STAGE, dr = WG_RAW_STAGE;    // signed distances to the other stage, flipped every step
    const float* pa = lds + a_lane;                                            // A fragments: stage q & 1
    float* pv = lds + WG_V_STAGE + ti * 4 * (2 * WG_FRAG) + twm * WG_FRAG + lane * 4;   // stage 2 output: (q+1) & 1
    // (pra, prb, the patch rows, point into stage (q+1) & 1)
    float* pw0 = lds + WG_RAW_OFF + raw_dst[0];                                // stage 1 output: q & 1
    float* pw1 = lds + WG_RAW_OFF + raw_dst[1];
    for (int m_i = 0; m_i < n_my; ++m_i) {
    zero_acc();
    for (int m_cc = 0; m_cc < a.n_chunks; ++m_cc, ++q) {
        const int ustep = u_kb * a.n_chunks + u_cc;
#pragma unroll
        for (int gp = 0; gp < WG_GW / 2; ++gp) {
            const int g0 = 2 * gp, g1 = 2 * gp + 1, cur = gp & 1;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int j = k >> 1;
                if ((k & 1) == 0)
                    acc[g0] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][0][j], uf[g0][j], acc[g0], 0, 0, 0);
                else
                    acc[g1] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][1][j], uf[g1][j], acc[g1], 0, 0, 0);
                if (k == 0) {
                    if (gp < 3) {              // A fragments of the next section
                        af[cur ^ 1][0] = *(const float4_t*)(pa + (g0 + 2) * (2 * WG_FRAG));
                        af[cur ^ 1][1] = *(const float4_t*)(pa + (g1 + 2) * (2 * WG_FRAG));
                    } else {
                        store_out_at(pv, 3);
                        __syncthreads();       // stage 2 of step q+1 and stage 1 of step q+2 are in LDS
                        af[0][0] = *(const float4_t*)(pa);         // (pa, pra, prb moved on in section 2)
                        af[0][1] = *(const float4_t*)(pa + (2 * WG_FRAG));
                        read_col_at(pra, prb, 0);
                    }
                }
                // stage 2 of step q+1: columns 0..3 of the patch, then the four output vectors
                if (gp == 0 && k == 1) read_col_at(pra, prb, 1);
                if (gp == 0 && k == 3) transform_col(0);
                if (gp == 0 && k == 4) read_col_at(pra, prb, 2);
                if (gp == 0 && k == 6) transform_col(1);
                if (gp == 1 && k == 1) read_col_at(pra, prb, 3);
                if (gp == 1 && k == 3) transform_col(2);
                if (gp == 1 && k == 6) transform_col(3);
                if (gp == 2 && (k == 1 || k == 3 || k == 5)) transform_out(k >> 1);
                if (gp == 2 && (k == 2 || k == 4 || k == 6)) store_out_at(pv, (k >> 1) - 1);
                if (gp == 2 && k == 7) transform_out(3);
                // stage 1: the registers hold step q+2 (requested a step ago); then request step q+3
                if (gp == 1 && k == 2) store_raw_at(pw0, 0);
                if (gp == 1 && k == 4) store_raw_at(pw1, 1);
                if (gp == 1 && k == 5) load_raw(l_cc);
                // the pointers move to the other stage after their last use of the step
                if (gp == 1 && k == 7) {
                    pra -= dr;
                    prb -= dr;
                    if (STACKED) advance_p(dr > 0 ? 0 : 1);
                }
                if (gp == 2 && k == 2) pw0 += dr;
                if (gp == 2 && k == 4) pw1 += dr;
                if (gp == 2 && k == 6) pa += dv;
                if (gp == 3 && k == 1) pv -= dv;
                if (k == 7) {                  // the filter fragments of this pair, for step q+1
                    uf[g0] = load_u(ustep, g0);
                    uf[g1] = load_u(ustep, g1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        advance_l();
        advance_u();
        dv = -dv;
        dr = -dr;
    }
        {
            // ---- epilogue of item m_i.  Each wave applies A^T . A to its two rows of M (lane-local);
            //      the waves with gh = 0 write their part to the staging tile, then the others add theirs.
            const WinoItem w = wino_decode(a, item0 + m_i * gx8);
            const int k0 = w.kb * WG_BN;
            float* stg = lds + WG_OUT_OFF;
            const size_t oimg = SEG == 1 ? (size_t)w.n * a.H * a.W * a.K : 0;
            const int kl = wn * 32 + (lane & 31);
            // accumulator element e of this lane is tile wm*32 + 8*(e/4) + 4*(lane>>5) + e%4, channel kl;
            // its 2 x 2 output pixels sit at a per-lane base plus an offset that depends on (e, i) only
            float* stg_lane = stg + ((8 * wm) * WG_PIX + 8 * (lane >> 5)) * WG_OP + kl;
            auto stg_index = [&](int e, int i) {
                return ((2 * (e / 4) + (i >> 1)) * WG_PIX + 2 * (e % 4) + (i & 1)) * WG_OP;
            };
            auto out_rows = [&](auto first_row, auto upper_rows, bool add) {
                constexpr int E0 = decltype(first_row)::value;
                constexpr bool UPPER = decltype(upper_rows)::value;    // this wave holds rows 2, 3 of M (gh = 1)
#pragma unroll
                for (int e = E0; e < E0 + 8; ++e) {
                    // the accumulators stay in the accumulation registers until the row that needs them
                    // (read through an explicit instruction: the register allocator would otherwise
                    // move all of them to ordinary registers at once)
                    float mv[WG_GW];
#pragma unroll
                    for (int g = 0; g < WG_GW; ++g)
                        asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(mv[g]) : "a"(acc[g][e]));
                    float s0[4], s1[4];
#pragma unroll
                    for (int m = 0; m < 4; ++m) {
                        // rows (M0, M1) of M for gh = 0, rows (M2, M3) for gh = 1:
                        // A^T = [1 1 1 0; 0 1 -1 -1] applied to the rows this wave holds
                        s0[m] = UPPER ? mv[m] : mv[m] + mv[4 + m];
                        s1[m] = UPPER ? -mv[m] - mv[4 + m] : mv[4 + m];
                    }
                    const float part[4] = {s0[0] + s0[1] + s0[2], s0[1] - s0[2] - s0[3], s1[0] + s1[1] + s1[2],
                                           s1[1] - s1[2] - s1[3]};
                    // (each staging element belongs to one lane of one wave per phase: plain read-add-write)
                    if (add) {
                        float prev[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) prev[i] = stg_lane[stg_index(e, i)];
#pragma unroll
                        for (int i = 0; i < 4; ++i) stg_lane[stg_index(e, i)] = prev[i] + part[i];
                    } else {                   // (not 0 + part: that addition would be kept, for the sign of zero)
#pragma unroll
                        for (int i = 0; i < 4; ++i) stg_lane[stg_index(e, i)] = part[i];
                    }
                    // four rows at a time may overlap (their chains of additions and LDS round trips are
                    // independent); more would need more registers than a wave has left here
                    if ((e & 3) == 3) __builtin_amdgcn_sched_barrier(0);
                }
            };
            // Output mask (the ReLU backward of the layer that produced this convolution's input): the thread
            // that stores pixel rows prow + 2 it of column pcol, channels k4..k4+3 fetches their mask values
            // while its wave has nothing else to do -- the waves with gh = 1 during the first phase, the others
            // during the second -- eight loads in flight, and keeps one bit per element ("mask > 0").  Inside
            // the store loop each load would be a full round trip to memory.
            constexpr int NV = 256 * (WG_BN / 4) / WG_THREADS;
            const int k4 = (tid & 15) * 4, pcol = (tid >> 4) & 15, prow = tid >> 8;
            const uint32_t out_bytes = (uint32_t)a.H * a.W * a.K * 4;
            // the thread's pixel column pcol lies in piece pcol / SEGW: rows sy0 + ..., column sx0 + pcol
            const SegPos sp = seg_pos<SEG>(a, item0 + m_i * gx8, SEG == 1 ? 0 : pcol / SEGW);
            const int sy0 = sp.y0, sx0 = sp.x0 - (SEG == 1 ? 0 : (pcol / SEGW) * SEGW);
            const bool col_ok = sp.ok && sx0 + pcol < a.W && k0 + k4 < a.K;
            const uint32_t obase = (uint32_t)(((sy0 + prow) * a.W + sx0 + pcol) * a.K + k0 + k4) * 4;
            const int row_stride = 2 * a.W * a.K * 4;
            uint32_t mbits = 0;
            auto fetch_mask = [&]() {
                const __amdgpu_buffer_rsrc_t omr =
                    __builtin_amdgcn_make_buffer_rsrc((void*)(a.out_mask + oimg), 0, out_bytes, 0x00020000);
                float4_t mk[NV];
#pragma unroll
                for (int it = 0; it < NV; ++it) {
                    const uint32_t voff = (col_ok && sy0 + prow + 2 * it < a.H) ? obase : 0x80000000u;
                    mk[it] = __builtin_bit_cast(
                        float4_t, __builtin_amdgcn_raw_buffer_load_b128(omr, voff, it * row_stride, 2));
                }
#pragma unroll
                for (int it = 0; it < NV; ++it)
#pragma unroll
                    for (int c = 0; c < 4; ++c) mbits |= (mk[it][c] > 0.f ? 1u : 0u) << (it * 4 + c);
            };
            // unpooling variant: the index bytes of the thread's eight stores (four channels each), requested
            // where the mask would be
            uint32_t iw[UNPOOL ? NV : 1];
            auto fetch_idx = [&]() {
                const __amdgpu_buffer_rsrc_t ir = __builtin_amdgcn_make_buffer_rsrc(
                    (void*)(a.unpool_idx + oimg), 0, out_bytes / 4, 0x00020000);
#pragma unroll
                for (int it = 0; it < NV; ++it) {
                    const uint32_t voff = (col_ok && sy0 + prow + 2 * it < a.H) ? obase / 4 : 0x80000000u;
                    iw[UNPOOL ? it : 0] = __builtin_amdgcn_raw_buffer_load_b32(ir, voff, it * (row_stride / 4), 2);
                }
            };
            if (UNPOOL && gh == 1) fetch_idx();
            if (!POOL && !UNPOOL && a.out_mask && gh == 1) fetch_mask();
            // bias of the thread's four channels for the store phase (k4 is the same there and in the pooling
            // variant): requested at the start of the second summation phase, which hides the round trip;
            // channels past K (and a null bias, as a buffer of size 0) read 0
            float4_t b4;
            auto load_bias = [&]() {
                const __amdgpu_buffer_rsrc_t br = __builtin_amdgcn_make_buffer_rsrc(
                    (void*)a.bias, 0, a.bias ? (uint32_t)a.K * 4 : 0u, 0x00020000);
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    b4[c] = __builtin_bit_cast(
                        float, __builtin_amdgcn_raw_buffer_load_b32(br, (uint32_t)(k0 + k4 + c) * 4, 0, 0));
            };
            using std::integral_constant;
            if (gh == 0) out_rows(integral_constant<int, 0>{}, integral_constant<bool, false>{}, false);
            else out_rows(integral_constant<int, 8>{}, integral_constant<bool, true>{}, false);
            __syncthreads();
            load_bias();
            if (gh == 0) {
                if (UNPOOL) fetch_idx();
                if (!POOL && !UNPOOL && a.out_mask) fetch_mask();
                out_rows(integral_constant<int, 8>{}, integral_constant<bool, false>{}, true);
            } else {
                out_rows(integral_constant<int, 0>{}, integral_constant<bool, true>{}, true);
            }
            __syncthreads();
            if constexpr (POOL) {
                // 2x2 max pooling of the tile (bias and ReLU first), written with one index byte per element
                // instead of the full-resolution output: bits 0-1 = position of the first maximum in the
                // window (row-major), bit 2 = "maximum > 0".  Thread -> channels k4..k4+3, pooled column
                // (tid >> 4) & 7, pooled rows (tid >> 7) + 4 it; tiles start at even pixels, so no window
                // straddles two tiles.
                const int Hp = a.H >> 1, Wp = a.W >> 1;
                const int pc = (tid >> 4) & 7, pr0 = tid >> 7;
                const size_t pimg = SEG == 1 ? (size_t)w.n * Hp * Wp * a.K : 0;
                const uint32_t pool_elems = (uint32_t)Hp * Wp * a.K;
                const __amdgpu_buffer_rsrc_t pyr =
                    __builtin_amdgcn_make_buffer_rsrc((void*)(a.pool_y + pimg), 0, pool_elems * 4, 0x00020000);
                const __amdgpu_buffer_rsrc_t pir =
                    __builtin_amdgcn_make_buffer_rsrc((void*)(a.pool_idx + pimg), 0, pool_elems, 0x00020000);
                // (pooled column pc lies in piece pc / (SEGW / 2))
                const SegPos pp = seg_pos<SEG>(a, item0 + m_i * gx8, SEG == 1 ? 0 : pc / (SEGW / 2));
                const int py0 = pp.y0 >> 1, px0 = (pp.x0 >> 1) - (SEG == 1 ? 0 : (pc / (SEGW / 2)) * (SEGW / 2));
                const bool col_ok = pp.ok && px0 + pc < Wp && k0 + k4 < a.K;
                // (once per ReLU setting: no test of a run-time flag per element, and selects instead of
                // branches for the running maximum)
                auto pool_rows = [&](auto with_relu) {
                constexpr bool RELU = decltype(with_relu)::value;
#pragma unroll
                for (int it = 0; it < 2; ++it) {
                    const int pr = pr0 + 4 * it;
                    const bool ok = col_ok && py0 + pr < Hp;
                    const uint32_t eoff = (uint32_t)(((py0 + pr) * Wp + px0 + pc) * a.K + k0 + k4);
                    const float* src = stg + ((2 * pr) * WG_PIX + 2 * pc) * WG_OP + k4;
                    float4_t v[4];
                    v[0] = *(const float4_t*)(src) + b4;
                    v[1] = *(const float4_t*)(src + WG_OP) + b4;
                    v[2] = *(const float4_t*)(src + WG_PIX * WG_OP) + b4;
                    v[3] = *(const float4_t*)(src + (WG_PIX + 1) * WG_OP) + b4;
                    float4_t best;
                    uint32_t packed = 0;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        float q[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) q[j] = (RELU && !(v[j][c] > 0.f)) ? 0.f : v[j][c];   // as the plain epilogue
                        float b = q[0];
                        uint32_t arg = 0;
#pragma unroll
                        for (int j = 1; j < 4; ++j) {
                            const bool take = q[j] > b || q[j] != q[j];
                            b = take ? q[j] : b;
                            arg = take ? (uint32_t)j : arg;
                        }
                        best[c] = b;
                        packed |= (arg | (b > 0.f ? 4u : 0u)) << (8 * c);
                    }
                    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, best), pyr,
                                                           ok ? eoff * 4 : 0x80000000u, 0, 0);
                    __builtin_amdgcn_raw_buffer_store_b32(packed, pir, ok ? eoff : 0x80000000u, 0, 0);
                }
                };
                if (a.relu) pool_rows(integral_constant<bool, true>{});
                else pool_rows(integral_constant<bool, false>{});
            } else {
                // bias, ReLU, output mask (bits fetched above) and the NHWC stores.  Thread -> pixel column
                // (tid >> 4) & 15, channels k4..k4+3, pixel rows (tid >> 8) + 2 it: one base offset, a scalar
                // stride per row pair.  Pixels outside the image get an offset beyond the buffer's size: such a
                // store is dropped.
                // The loop exists once per (ReLU, mask) combination: with the two tests inside it every
                // iteration would wait for its own LDS read.
                const __amdgpu_buffer_rsrc_t yr =
                    __builtin_amdgcn_make_buffer_rsrc((void*)(a.y + oimg), 0, out_bytes, 0x00020000);
                const float* src = stg + (prow * WG_PIX + pcol) * WG_OP + k4;
                auto store_rows = [&](auto with_relu, auto with_mask) {
                    constexpr bool RELU = decltype(with_relu)::value, MASKED = decltype(with_mask)::value;
    #pragma unroll
                    for (int it = 0; it < NV; ++it) {
                        // The row offset is added to the vector offset, not passed as the scalar one: after a
                        // 128-bit buffer store with a register as scalar offset the compiler schedules vector
                        // writes to the store's data registers with no wait state, and on this part the first
                        // dword of the stored rows then came out overwritten (lanes 12-15 of every 16).  With an
                        // immediate scalar offset it inserts the wait state itself.
                        const uint32_t voff = ((col_ok && sy0 + prow + 2 * it < a.H) ? obase : 0x80000000u) +
                                              (uint32_t)(it * row_stride);
                        float4_t v = *(const float4_t*)(src + it * 2 * WG_PIX * WG_OP) + b4;
                        if (RELU) {
    #pragma unroll
                            for (int c = 0; c < 4; ++c) v[c] = v[c] > 0.f ? v[c] : 0.f;
                        }
                        if (MASKED) {
    #pragma unroll
                            for (int c = 0; c < 4; ++c) v[c] = (mbits >> (it * 4 + c)) & 1u ? v[c] : 0.f;
                        }
                        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), yr, voff, 0, 2);
                    }
                };
                using yes = integral_constant<bool, true>;
                using no = integral_constant<bool, false>;
                if constexpr (UNPOOL) {
                    // y with the mask of bit 2, and the four positions of every window of the gradient in front
                    // of the pooling: (2 row + i, 2 column + j) gets the value where the byte says 4 | 2 i + j
                    const __amdgpu_buffer_rsrc_t fr = __builtin_amdgcn_make_buffer_rsrc(
                        (void*)(a.unpool_y + 4 * oimg), 0, out_bytes * 4, 0x00020000);
                    const uint32_t fbase = (uint32_t)((2 * (sy0 + prow) * 2 * a.W + 2 * (sx0 + pcol)) * a.K + k0 + k4) * 4;
                    const uint32_t frow = (uint32_t)(2 * a.W * a.K) * 4;        // one full-resolution row
                    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    #pragma unroll
                    for (int it = 0; it < NV; ++it) {
                        const bool ok = col_ok && sy0 + prow + 2 * it < a.H;
                        const uint32_t voff = (ok ? obase : 0x80000000u) + (uint32_t)(it * row_stride);
                        const uint32_t foff = (ok ? fbase : 0x80000000u) + (uint32_t)it * (4 * frow);
                        const float4_t v = *(const float4_t*)(src + it * 2 * WG_PIX * WG_OP) + b4;
                        uint32_t code[4];
    #pragma unroll
                        for (int c = 0; c < 4; ++c) code[c] = (iw[UNPOOL ? it : 0] >> (8 * c)) & 7u;
                        float4_t kept;
    #pragma unroll
                        for (int c = 0; c < 4; ++c) kept[c] = (code[c] & 4u) ? v[c] : 0.f;
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, kept), yr, voff, 0, 2);
    #pragma unroll
                        for (int pos = 0; pos < 4; ++pos) {
                            float4_t o;
    #pragma unroll
                            for (int c = 0; c < 4; ++c) o[c] = code[c] == (4u | pos) ? v[c] : 0.f;
                            __builtin_amdgcn_raw_buffer_store_b128(
                                __builtin_bit_cast(u32x4, o), fr,
                                foff + (uint32_t)(pos >> 1) * frow + (uint32_t)((pos & 1) * a.K * 4), 0, 2);
                        }
                    }
                } else if (a.relu) {
                    if (a.out_mask) store_rows(yes{}, yes{});
                    else store_rows(yes{}, no{});
                } else {
                    if (a.out_mask) store_rows(no{}, yes{});
                    else store_rows(no{}, no{});
                }
            }
        }
        // the next epilogue's staging writes come after at least one more barrier (n_chunks >= 1)
    }
}

bool wino_shape_ok(int C, int K) { return C % WG_CC == 0 && K % 4 == 0; }

}  // namespace

extern "C" int pd_conv3x3_winograd_supported(int C, int K) { return (C > 0 && K > 0 && wino_shape_ok(C, K)) ? 1 : 0; }

extern "C" int pd_conv3x3_winograd_filter_bytes(int C, int K, uint64_t* bytes) {
    PD_REQUIRE(bytes != nullptr, PD_EINVAL, "pd_conv3x3_winograd_filter_bytes: NULL pointer");
    PD_REQUIRE(C > 0 && K > 0 && wino_shape_ok(C, K), PD_ESHAPE,
               "pd_conv3x3_winograd_filter_bytes: needs C %% 8 == 0 and K %% 4 == 0 (C=%d K=%d)", C, K);
    const uint64_t k_pad = (uint64_t)((K + WG_BN - 1) / WG_BN) * WG_BN;
    *bytes = (uint64_t)WG_G * k_pad * (uint64_t)C * sizeof(float);
    return PD_OK;
}

extern "C" int pd_conv3x3_winograd_filter_f32(const float* w, float* u, int C, int K, int rot180, void* stream) {
    PD_REQUIRE(w && u && w != u, PD_EINVAL, "pd_conv3x3_winograd_filter_f32: NULL or aliased pointer");
    PD_REQUIRE(C > 0 && K > 0 && wino_shape_ok(C, K), PD_ESHAPE,
               "pd_conv3x3_winograd_filter_f32: needs C %% 8 == 0 and K %% 4 == 0 (C=%d K=%d)", C, K);
    PD_REQUIRE(pd_aligned(u, 16), PD_EINVAL, "pd_conv3x3_winograd_filter_f32: u must be 16-byte aligned");
    const int k_pad = (K + WG_BN - 1) / WG_BN * WG_BN;
    const long units = (long)(k_pad / 32) * (C / WG_CC);   // one wave each
    winograd_filter_kernel<<<(unsigned)((units + 3) / 4), 256, 0, (hipStream_t)stream>>>(
        w, u, K, C, k_pad, rot180, pd_aligned(w, 16) ? 1 : 0);
    PD_CHECK_LAUNCH("pd_conv3x3_winograd_filter_f32");
    return PD_OK;
}

namespace {

int g_pieces_mode = 0;   // pd_conv3x3_winograd_set_pieces: 0 = by item count, 1 = wherever the shape allows, -1 = never

int wino_fwd_launch(const char* who, const float* x, const float* u, const float* bias, const float* in_mask,
                    const float* out_mask, float* y, float* pool_y, uint8_t* pool_idx, int N, int H, int W, int C,
                    int K, int relu, void* stream, const uint8_t* unpool_idx = nullptr, float* unpool_y = nullptr) {
    PD_REQUIRE(N > 0 && H > 0 && W > 0 && C > 0 && K > 0, PD_ESHAPE, "%s: dimensions must be positive", who);
    PD_REQUIRE(wino_shape_ok(C, K), PD_ESHAPE, "%s: needs C %% 8 == 0 and K %% 4 == 0 (C=%d K=%d)", who, C, K);
    PD_REQUIRE((long)H * W * (C > K ? C : K) < (1L << 29), PD_ESHAPE, "%s: image too large", who);
    PD_REQUIRE((long)C * WG_G * WG_BN * 4 < (1L << 31), PD_ESHAPE, "%s: too many input channels", who);
    PD_REQUIRE(x && u, PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE(pd_aligned(x, 16) && pd_aligned(u, 16) && pd_aligned(y, 16) && pd_aligned(in_mask, 16) &&
                   pd_aligned(out_mask, 16), PD_EINVAL, "%s: tensors must be 16-byte aligned", who);
    WinoArgs a;
    a.x = x; a.u = u; a.bias = bias; a.mask = in_mask; a.out_mask = out_mask; a.y = y;
    a.pool_y = pool_y; a.pool_idx = pool_idx;
    a.unpool_idx = unpool_idx; a.unpool_y = unpool_y;
    a.N = N; a.H = H; a.W = W; a.C = C; a.K = K;
    a.img_h = 0;
    // images whose height is even but no multiple of the 16-row tile are stacked into one tall image
    // (see the kernel): N * ceil(H / 16) tile rows become ceil(N * H / 16)
    // (not with an input mask: that variant has no registers to spare for it)
    // (with the unpooling epilogue the full-resolution gradient, four times y, must fit a buffer descriptor too)
    const bool stacked = !in_mask && N > 1 && H % 2 == 0 && H % WG_PIX != 0 &&
                         (long)N * H * W * (C > K ? C : K) < (1L << 29) && (!unpool_y || (long)N * H * W * K < (1L << 27));
    if (stacked) { a.img_h = H; a.H = N * H; a.N = 1; }
    a.relu = relu != 0;
    a.tiles_x = (W + WG_PIX - 1) / WG_PIX;
    a.tiles_y = (a.H + WG_PIX - 1) / WG_PIX;
    a.k_blocks = (K + WG_BN - 1) / WG_BN;
    a.n_chunks = C / WG_CC;
    // one persistent block per CU (the kernel needs a CU's whole register file), in multiples of 8
    int dev = 0, cus = 0;
    PD_HIP(hipGetDevice(&dev));
    PD_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const long cu_blocks = (long)(cus / WG_XCD) * WG_XCD > 0 ? (long)(cus / WG_XCD) * WG_XCD : WG_XCD;
    // A stacked batch whose width is a multiple of 8 (4) but not of 16 pixels can use work items of two (four)
    // pieces: no padding columns, 7/8 of the items at widths 56 and 28.  What counts is the number of items the
    // busiest block gets (the blocks of a die share its items evenly): pieces are used when that number falls
    // (64 images of 56 x 56 with 256 output channels: 13 instead of 14 items per block), not when both divide
    // into the same number of rounds (28 x 28 with 512 channels: 7 and 6.1 -> 7; the squares then win by their
    // smaller halo).
    const long square_items = (long)a.N * a.tiles_x * a.tiles_y * a.k_blocks;
    int seg = !stacked || W % WG_PIX == 0 ? 1 : W % 8 == 0 ? 2 : W % 4 == 0 ? 4 : 1;
    a.segs_per_row = W / (WG_PIX / seg);
    a.n_segs = a.segs_per_row * a.tiles_y;
    const long piece_items = (long)((a.n_segs + seg - 1) / seg) * a.k_blocks;
    auto busiest = [&](long n) {
        const long per_xcd = (n + WG_XCD - 1) / WG_XCD, per_die_blocks = cu_blocks / WG_XCD;
        return (per_xcd + per_die_blocks - 1) / per_die_blocks;
    };
    if (seg > 1 && (g_pieces_mode < 0 || (g_pieces_mode == 0 && busiest(piece_items) >= busiest(square_items)))) seg = 1;
    const long items = seg == 1 ? square_items : piece_items;
    PD_REQUIRE(items <= 0x7ffffff0L, PD_ESHAPE, "%s: too many tiles", who);
    a.n_items = (int)items;
    a.items_per_xcd = (int)((items + WG_XCD - 1) / WG_XCD);
    long blocks = cu_blocks;
    if (blocks > (long)a.items_per_xcd * WG_XCD) blocks = (long)a.items_per_xcd * WG_XCD;
    dim3 grid((unsigned)blocks);
    hipStream_t s = (hipStream_t)stream;
    if (seg == 2) {
        if (unpool_y) winograd_fwd_kernel<false, false, true, true, 2><<<grid, WG_THREADS, 0, s>>>(a);
        else if (a.pool_y) winograd_fwd_kernel<false, true, true, false, 2><<<grid, WG_THREADS, 0, s>>>(a);
        else winograd_fwd_kernel<false, false, true, false, 2><<<grid, WG_THREADS, 0, s>>>(a);
    } else if (seg == 4) {
        if (unpool_y) winograd_fwd_kernel<false, false, true, true, 4><<<grid, WG_THREADS, 0, s>>>(a);
        else if (a.pool_y) winograd_fwd_kernel<false, true, true, false, 4><<<grid, WG_THREADS, 0, s>>>(a);
        else winograd_fwd_kernel<false, false, true, false, 4><<<grid, WG_THREADS, 0, s>>>(a);
    } else if (unpool_y) {
        if (stacked) winograd_fwd_kernel<false, false, true, true><<<grid, WG_THREADS, 0, s>>>(a);
        else winograd_fwd_kernel<false, false, false, true><<<grid, WG_THREADS, 0, s>>>(a);
    } else if (stacked) {
        if (a.pool_y) winograd_fwd_kernel<false, true, true><<<grid, WG_THREADS, 0, s>>>(a);
        else winograd_fwd_kernel<false, false, true><<<grid, WG_THREADS, 0, s>>>(a);
    } else {
        if (a.pool_y) winograd_fwd_kernel<false, true, false><<<grid, WG_THREADS, 0, s>>>(a);
        else if (in_mask) winograd_fwd_kernel<true, false, false><<<grid, WG_THREADS, 0, s>>>(a);
        else winograd_fwd_kernel<false, false, false><<<grid, WG_THREADS, 0, s>>>(a);
    }
    PD_CHECK_LAUNCH(who);
    return PD_OK;
}

}  // namespace

extern "C" int pd_conv3x3_winograd_set_pieces(int mode) {
    PD_REQUIRE(mode >= -1 && mode <= 1, PD_EINVAL, "pd_conv3x3_winograd_set_pieces: mode is -1, 0 or 1");
    g_pieces_mode = mode;
    return PD_OK;
}

extern "C" int pd_conv3x3_winograd_fwd_nhwc_f32(const float* x, const float* u, const float* bias,
                                                const float* in_mask, const float* out_mask, float* y, int N, int H,
                                                int W, int C, int K, int relu, void* stream) {
    const char* who = "pd_conv3x3_winograd_fwd_nhwc_f32";
    PD_REQUIRE(y, PD_EINVAL, "%s: NULL pointer", who);
    return wino_fwd_launch(who, x, u, bias, in_mask, out_mask, y, nullptr, nullptr, N, H, W, C, K, relu, stream);
}

extern "C" int pd_conv3x3_winograd_fwd_unpool_nhwc_f32(const float* x, const float* u, const uint8_t* idx, float* y,
                                                       float* y_full, int N, int H, int W, int C, int K,
                                                       void* stream) {
    const char* who = "pd_conv3x3_winograd_fwd_unpool_nhwc_f32";
    PD_REQUIRE(y && y_full && idx, PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE(pd_aligned(y_full, 16) && pd_aligned(idx, 4), PD_EINVAL,
               "%s: the full-resolution output must be 16-byte aligned, the index bytes 4-byte aligned", who);
    PD_REQUIRE(H > 0 && W > 0 && K > 0 && (long)H * W * K < (1L << 27), PD_ESHAPE,
               "%s: image too large for the full-resolution output", who);
    return wino_fwd_launch(who, x, u, nullptr, nullptr, nullptr, y, nullptr, nullptr, N, H, W, C, K, 0, stream, idx,
                           y_full);
}

extern "C" int pd_conv3x3_winograd_fwd_pool_nhwc_f32(const float* x, const float* u, const float* bias,
                                                     float* y_pool, uint8_t* idx, int N, int H, int W, int C, int K,
                                                     int relu, void* stream) {
    const char* who = "pd_conv3x3_winograd_fwd_pool_nhwc_f32";
    PD_REQUIRE(H >= 2 && W >= 2, PD_ESHAPE, "%s: the image must hold at least one 2x2 window", who);
    PD_REQUIRE(y_pool && idx, PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE(pd_aligned(y_pool, 16) && pd_aligned(idx, 4), PD_EINVAL,
               "%s: the pooled output must be 16-byte aligned, the index bytes 4-byte aligned", who);
    return wino_fwd_launch(who, x, u, bias, nullptr, nullptr, nullptr, y_pool, idx, N, H, W, C, K, relu, stream);
}

// =====================================================================================================
// Weight gradient in the Winograd domain.
//
//   dU[g][k][c] = sum over tiles of  dM[g][tile][k] * V[g][tile][c],   dM = A dY A^T,  V = B^T d B,
//   dw[k][.][.][c] = G^T dU[.][k][c] G
//
// (the derivative of Y = A^T [U .* V] A with U = G g G^T): 16 GEMMs [K x tiles] * [tiles x C] whose
// reduction runs over all 2 x 2 output tiles of the batch, again 16 multiplies where the direct
// algorithm needs 36.  A persistent 512-thread block owns one (64 out-channel, 64 in-channel) block pair
// and a contiguous range of strips (1 x 8 tiles = 2 x 16 output pixels), keeps all 16 x 64 x 64 sums in
// its accumulators (8 GEMMs x 32 x 32 per wave) and writes them once at the end; two small kernels add
// the blocks' partial sums in fixed order and apply G^T . G (deterministic, no atomics).
//
// Per strip (= one pipeline step, 32 MFMAs per wave):
//   * x: the 4 x 18 pixel x 64 channel patch goes global -> registers (a step in flight) -> LDS; every
//     thread then forms one row of B^T d for one (tile, 4 channels), applies . B and writes V[g][tile][c]
//     (the two 32-channel halves of odd tiles are swapped, so the B-fragment reads below, which take an
//     even tile in lanes 0-31 and an odd one in lanes 32-63, hit different banks);
//   * dY never touches LDS: the MFMA A operand of lane (k, h) is dM[g][tile 2j+h][k], so each lane loads
//     the 4 x 4 dY values of its own k for its four tiles (128-byte runs across a half wave), a step
//     ahead, and forms the dM values it needs with a few additions right before the MFMAs.  The signs of
//     A's last row/column are left out here and applied in the final transform.
//   * dbias[k] is the sum of dM[1][1] (= the sum of a tile's four dY values) over all tiles.
// =====================================================================================================
namespace {

constexpr int WW_THREADS = 512;
constexpr int WW_TILES = 8;                          // tiles per strip
constexpr int WW_PATCH_W = 2 * WW_TILES + 2;         // input columns of a strip's patch
constexpr int WW_ROW_PIECES = 320;                   // 16-byte pieces per patch row, padded from 18*16 to 5 waves
constexpr int WW_V_STAGE = WG_G * WW_TILES * 64;     // floats: [g][tile][c]
constexpr int WW_RAW_STAGE = 4 * WW_PATCH_W * 64;    // floats: [row][pixel][c]
constexpr int WW_RAW_OFF = 2 * WW_V_STAGE;
constexpr int WW_ZERO_OFF = WW_RAW_OFF + 2 * WW_RAW_STAGE;   // upright strips: one patch row (4 pixels) of zeros
constexpr int WW_LDS_FLOATS = WW_ZERO_OFF + 4 * 64;
constexpr int WW_VROWS = 2 * WW_TILES;               // output rows of an upright strip
constexpr int WW_BLOCKS = 256;                       // persistent blocks: 8 dies x 32
constexpr int WW_PART_FLOATS = WG_G * 64 * 64;       // one block's partial dU
constexpr int WW_PART_STRIDE = WW_PART_FLOATS;       // floats between two blocks' partials

struct WinoWgradArgs {
    const float* x;      // [N,H,W,C]
    const float* dy;     // [N,H,W,K]
    float* part;         // [pair][rank][16][64][64]
    float* part_db;      // [pair][rank][2][64]
    int N, H, W, C, K;
    int sx, sy;          // strips per row pair, row pairs per image (upright strips: strips side by side, unused)
    int n_strips, strips_per_rank;
    int rows_all;        // upright strips: N * H, the rows of the batch taken as one tall image
    int c_blocks, n_pairs, ranks;
};

struct StripPos { int n, y0, x0, row; };      // row = n * H + y0, the strip's first output row counted over all images
// (upright strips: row = first output row in the stacked batch, y0 = row % H, n unused)

// Strips are numbered down the image first (row pair fastest), then across, then over images: a block's
// consecutive strips share two of their four input rows, which the second one finds in cache.
__device__ __forceinline__ StripPos strip_decode(const WinoWgradArgs& a, int s) {
    StripPos p;
    const int per_img = a.sx * a.sy;
    p.n = s / per_img;
    const int rem = s - p.n * per_img;
    const int tx = rem / a.sy;
    p.x0 = tx * (2 * WW_TILES);
    p.y0 = 2 * (rem - tx * a.sy);
    p.row = p.n * a.H + p.y0;
    return p;
}
// Upright strips (8 tiles on top of each other: 16 output rows x 2 columns of the batch taken as one image of
// N * H rows) are numbered across the image first: neighbours share two of their four patch columns.
__device__ __forceinline__ StripPos vstrip_decode(const WinoWgradArgs& a, int s) {
    StripPos p;
    const int sr = s / a.sx;
    p.n = 0;
    p.x0 = 2 * (s - sr * a.sx);
    p.row = WW_VROWS * sr;
    p.y0 = p.row % a.H;
    return p;
}
// (y0 is kept only for the cursor that needs it; H >= 14, so two subtractions at most)
template <bool WITH_Y0 = false>
__device__ __forceinline__ void vstrip_next(const WinoWgradArgs& a, StripPos& p) {
    p.x0 += 2;
    if (p.x0 >= a.W) {
        p.x0 = 0;
        p.row += WW_VROWS;
        if (WITH_Y0) {
            p.y0 += WW_VROWS;
            if (p.y0 >= a.H) p.y0 -= a.H;
            if (p.y0 >= a.H) p.y0 -= a.H;
        }
    }
}

__device__ __forceinline__ void strip_next(const WinoWgradArgs& a, StripPos& p) {
    p.y0 += 2;
    p.row += 2;
    if (p.y0 >= a.H) {
        p.row -= p.y0;
        p.y0 = 0;
        p.x0 += 2 * WW_TILES;
        if (p.x0 >= a.W) { p.x0 = 0; ++p.n; p.row += a.H; }
    }
}

// VERT: upright strips.  A strip of 2 x 16 pixels pads image widths of 56, 28 and 14 pixels to 64, 32 and 16; eight
// tiles on top of each other fit every even width, and with the batch taken as one image of N * H rows (H even, so
// no tile straddles two images) only the batch's last strip row can be partly empty.  The patch is then 18 rows x 4
// pixels (as many pixels as 4 x 18).  A tile in the first (last) tile row of an image must see zeros in the first
// (last) row of its 4 x 4 window, where the stacked layout holds the neighbouring image's row: only the threads
// that form row 0 (d0 - d2) resp. row 3 (d1 - d3) of B^T d read those rows, and for such a tile they read a row of
// zeros in LDS instead.  Needs H >= 14 (one conditional subtraction finds a tile's row inside its image).
template <bool VERT>
__global__ __launch_bounds__(WW_THREADS, 1) void winograd_wgrad_kernel(const WinoWgradArgs a) {
    __shared__ __attribute__((aligned(16))) float lds[WW_LDS_FLOATS];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // block -> (pair, rank): the 32 blocks of a die cover all pairs of a contiguous strip range, so the
    // pairs that read the same x and dY strips run side by side on one L2
    int pair, rank;
    if (a.n_pairs <= 32) {
        const int xcd = blockIdx.x % WG_XCD, slot = blockIdx.x / WG_XCD;
        pair = slot % a.n_pairs;
        rank = xcd * (32 / a.n_pairs) + slot / a.n_pairs;
    } else {                                   // more pairs than a die has blocks: plain round robin
        pair = blockIdx.x % a.n_pairs;
        rank = blockIdx.x / a.n_pairs;
    }
    const int kb = pair / a.c_blocks, cb = pair % a.c_blocks;
    const int s_begin = rank * a.strips_per_rank;
    int s_end = s_begin + a.strips_per_rank;
    s_end = s_end < a.n_strips ? s_end : a.n_strips;
    const int n_my = s_end > s_begin ? s_end - s_begin : 0;

    // ---- stage 1 role: pieces p = tid + 512 j of the patch: row p / 320 (uniform in a wave), pixel
    //      (p % 320) / 16 (pixels 18, 19 are padding of the piece grid), channels 4 (p % 16) .. +3.
    //      A patch row is read through its own buffer descriptor over that image row (this block's 64
    //      channels onwards): the pixel offset (x0 - 1 + pixel) * C is negative left of the image, which
    //      as an unsigned offset lies beyond the descriptor's size like the columns right of the image,
    //      so both read 0; rows outside the image get an empty descriptor.
    uint32_t xoff[3];
    int raw_dst[3], prow[3];
    bool live[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int p = tid + WW_THREADS * j;
        if (VERT) {      // a wave = one patch row: 4 pixels x 16 channel groups, one contiguous kilobyte
            prow[j] = wave + 8 * j;
            const int ppx = lane >> 4, pcg = lane & 15;
            live[j] = prow[j] < WW_VROWS + 2;
            xoff[j] = live[j] ? (uint32_t)(((ppx - 1) * a.C + pcg * 4) * 4) : 0x80000000u;
            raw_dst[j] = ((live[j] ? prow[j] : 0) * 4 + ppx) * 64 + pcg * 4;
            continue;
        }
        prow[j] = __builtin_amdgcn_readfirstlane(p / WW_ROW_PIECES);
        const int rem = p % WW_ROW_PIECES, ppx = rem >> 4, pcg = rem & 15;
        live[j] = ppx < WW_PATCH_W && p < 4 * WW_ROW_PIECES;
        xoff[j] = live[j] ? (uint32_t)(((ppx - 1) * a.C + pcg * 4) * 4) : 0x80000000u;
        raw_dst[j] = ((prow[j] & 3) * WW_PATCH_W + (live[j] ? ppx : 0)) * 64 + pcg * 4;
    }
    float4_t rawr[3];
    // row descriptors, kept cheap in scalar instructions: per patch row a loop-invariant 64-bit base (row -1 +
    // prow of image 0) to which the strip's running row index times the row pitch is added; a row outside
    // the image (one unsigned comparison) or of a strip past the end gets size 0, and then its base is unused
    const uint32_t row_pitch_x = (uint32_t)(a.W * a.C) * 4;
    const uint32_t row_bytes_x = (uint32_t)(a.W * a.C - cb * 64) * 4;
    const char* xrow0[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) xrow0[j] = (const char*)(a.x + cb * 64) + (int64_t)(prow[j] - 1) * row_pitch_x;
    const bool third_row_live = VERT ? wave < 2 : wave < 4;   // the third round of pieces: the patch's last row(s) only
    auto load_raw = [&](const StripPos& p, bool valid) {
        const uint32_t strip_off = (uint32_t)(p.x0 * a.C) * 4;
        const uint32_t live_bytes = valid ? row_bytes_x : 0u;
        const uint64_t strip_row = (uint64_t)(uint32_t)p.row * row_pitch_x;
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            // (upright strips: p.row counts rows of the whole batch, and a row of the neighbouring image is data)
            const uint32_t gy = (uint32_t)((VERT ? p.row : p.y0) - 1 + prow[j]);
            const uint32_t row_bytes = (j < 2 || third_row_live) ? live_bytes : 0u;
            const uint32_t bytes = gy < (uint32_t)(VERT ? a.rows_all : a.H) ? row_bytes : 0u;
            const __amdgpu_buffer_rsrc_t r =
                __builtin_amdgcn_make_buffer_rsrc((void*)(xrow0[j] + strip_row), 0, bytes, 0x00020000);
            rawr[j] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(r, xoff[j] + strip_off, 0, 0));
        }
    };
    auto store_raw = [&](int stage, int j) {
        if (live[j]) *(float4_t*)(lds + WW_RAW_OFF + stage * WW_RAW_STAGE + raw_dst[j]) = rawr[j];
    };

    // ---- stage 2 role: tile tt (of the strip's 8), channels 4 cg .. +3, row ti of B^T d = Ra + sgn * Rb
    const int ti = wave & 3;
    const int tt = (wave >> 2) * 4 + (lane >> 4), cg = lane & 15;
    const int row_a = ti == 0 ? 0 : ti == 2 ? 2 : 1;
    const int row_b = ti == 2 ? 1 : ti == 3 ? 3 : 2;
    const float sgn = ti == 1 ? 1.f : -1.f;
    const int src_a = VERT ? ((2 * tt + row_a) * 4) * 64 + cg * 4 : (row_a * WW_PATCH_W + 2 * tt) * 64 + cg * 4;
    const int src_b = VERT ? ((2 * tt + row_b) * 4) * 64 + cg * 4 : (row_b * WW_PATCH_W + 2 * tt) * 64 + cg * 4;
    // upright strips: where this thread reads rows Ra / Rb of the strip being transformed -- src_a / src_b, or the
    // row of zeros when the tile's window row lies in the neighbouring image (ti = 0: row 0, ti = 3: row 3)
    // (offsets from the start of LDS, raw stage included)
    int sa = 0, sb = 0;
    auto set_window_rows = [&](const StripPos& p, int stage) {
        if (!VERT) return;
        const int base = WW_RAW_OFF + stage * WW_RAW_STAGE;
        sa = base + src_a;
        sb = base + src_b;
        if (ti == 0 || ti == 3) {
            int t = p.y0 + 2 * tt;              // the tile's first output row inside its image (y0 < H, 2 tt <= 14 <= H)
            t = t >= a.H ? t - a.H : t;
            if (ti == 0 && t == 0) sa = WW_ZERO_OFF + cg * 4;
            if (ti == 3 && t + 2 == a.H) sb = WW_ZERO_OFF + cg * 4;
        }
    };
    const int v_dst = (ti * 4 * WW_TILES + tt) * 64 + ((cg * 4) ^ (32 * (tt & 1)));
    float4_t t[4], dc[2], vout;
    auto read_col = [&](const float* rs, int s) {
        if (VERT) {
            dc[0] = *(const float4_t*)(lds + sa + s * 64);
            dc[1] = *(const float4_t*)(lds + sb + s * 64);
        } else {
            dc[0] = *(const float4_t*)(rs + src_a + s * 64);
            dc[1] = *(const float4_t*)(rs + src_b + s * 64);
        }
    };
    auto transform_col = [&](int s) { t[s] = dc[0] + sgn * dc[1]; };
    auto transform_out = [&](int m) {
        if (m == 0) vout = t[0] - t[2];
        else if (m == 1) vout = t[1] + t[2];
        else if (m == 2) vout = t[2] - t[1];
        else vout = t[1] - t[3];
    };
    auto store_out = [&](float* vst, int m) { *(float4_t*)(vst + v_dst + m * (WW_TILES * 64)) = vout; };

    // ---- stage 3 role: wave (gh, wm, wn): GEMMs gh*8..+7, out channels wm*32..+31, in channels wn*32..+31;
    //      lane (h, cl): row/column cl, tiles 2j + h of the strip
    const int gh = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1;
    const int h = lane >> 5, cl = lane & 31;
    const int b_src = (gh * 8 * WW_TILES + h) * 64 + ((wn ^ h) * 32 + cl);
    // dY: value (row a, column b, tile 2j+h) of out channel k sits at (a*W + 4j + 2h + b) * K + k from the
    // strip's first pixel; a row is read through a descriptor that ends with the image row
    uint32_t dyoff[4][2];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int b = 0; b < 2; ++b)
            dyoff[j][b] = VERT ? (uint32_t)(((4 * j + 2 * h) * a.W + b) * a.K + kb * 64 + wm * 32 + cl) * 4
                               : (uint32_t)((4 * j + 2 * h + b) * a.K + kb * 64 + wm * 32 + cl) * 4;
    float dyr[2][2][4];                        // [row a][column b][j]
    const uint32_t row_pitch_dy = (uint32_t)(a.W * a.K) * 4;
    auto load_dy = [&](const StripPos& p, bool valid) {
        // upright strips: tile 2j + h lies 2 (2j + h) rows further down (in dyoff); one descriptor per row parity,
        // from the strip's first pixel of that row to the end of the strip's last row inside the batch
        int vrows = a.rows_all - p.row;
        vrows = vrows < WW_VROWS ? vrows : WW_VROWS;
        const uint32_t live_bytes = !valid ? 0u : VERT ? (uint32_t)((vrows * a.W - p.x0) * a.K) * 4
                                                       : (uint32_t)((a.W - p.x0) * a.K) * 4;
        const char* row0 = (const char*)a.dy + (uint64_t)(uint32_t)(p.row * a.W + p.x0) * (uint32_t)(a.K * 4);
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            // the strip's first row always lies in the image, its second may not (odd H)
            // (readfirstlane: the compiler forms the saturating difference in a vector register, and a descriptor
            // built from one is taken as different per lane -- a loop around every load)
            const uint32_t bytes = VERT ? (r == 0 ? live_bytes : (uint32_t)__builtin_amdgcn_readfirstlane((int)(
                                               live_bytes > row_pitch_dy ? live_bytes - row_pitch_dy : 0u)))
                                        : (r == 0 || p.y0 + 1 < a.H) ? live_bytes : 0u;
            const __amdgpu_buffer_rsrc_t rs =
                __builtin_amdgcn_make_buffer_rsrc((void*)(row0 + (r ? row_pitch_dy : 0u)), 0, bytes, 0x00020000);
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    dyr[r][b][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, dyoff[j][b], 0, 0));
        }
    };
    float rr[2][2][4];                         // rows 2gh, 2gh+1 of A dY (signs of row 3 left out): [ii][b][j]
    const float rr_c0 = gh ? -1.f : 0.f, rr_c1 = gh ? 0.f : 1.f;

    float16_t acc[WG_GW];
#pragma unroll
    for (int g = 0; g < WG_GW; ++g)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[g][e] = 0.f;
    float db_acc = 0.f;

    if (n_my > 0) {
        // cursors of the stages: strip of the next raw-x request (3 ahead of the multiply), of the next
        // dY request (1 ahead)
        StripPos lp = VERT ? vstrip_decode(a, s_begin) : strip_decode(a, s_begin), dp = lp;
        StripPos tp = lp;                      // upright strips: the strip whose patch stage 2 reads next
        int l_left = n_my, d_left = n_my;      // strips not yet requested
        auto next_l = [&]() { --l_left; if (VERT) vstrip_next(a, lp); else strip_next(a, lp); };
        auto next_d = [&]() { --d_left; if (VERT) vstrip_next(a, dp); else strip_next(a, dp); };
        if (VERT && tid < 4 * 64) lds[WW_ZERO_OFF + tid] = 0.f;

        // ---- prologue: strips 0 and 1 into LDS, strip 2 into registers, strip 0 transformed, dY of strip 0
        load_raw(lp, l_left > 0); next_l();
        load_dy(dp, d_left > 0); next_d();
#pragma unroll
        for (int j = 0; j < 3; ++j) store_raw(0, j);
        load_raw(lp, l_left > 0); next_l();
#pragma unroll
        for (int j = 0; j < 3; ++j) store_raw(1, j);
        load_raw(lp, l_left > 0); next_l();
        __syncthreads();
        set_window_rows(tp, 0);
#pragma unroll
        for (int s = 0; s < 4; ++s) { read_col(lds + WW_RAW_OFF, s); transform_col(s); }
#pragma unroll
        for (int m = 0; m < 4; ++m) { transform_out(m); store_out(lds, m); }
        if (VERT) { vstrip_next<true>(a, tp); set_window_rows(tp, 1); }      // strip 1 sits in the second raw stage
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        float bf[2][2][4];                     // B fragments of GEMM pair p wait in bf[p & 1]: [g of the pair][j]
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
            for (int j = 0; j < 4; ++j) bf[0][g][j] = lds[b_src + (g * WW_TILES + 2 * j) * 64];
        read_col(lds + WW_RAW_OFF + WW_RAW_STAGE, 0);

        for (int q = 0; q < n_my; ++q) {
            const float* vs = lds + (q & 1) * WW_V_STAGE + b_src;
            const float* vs_next = lds + ((q + 1) & 1) * WW_V_STAGE + b_src;
            float* vn = lds + ((q + 1) & 1) * WW_V_STAGE;
            const float* rs = lds + WW_RAW_OFF + ((q + 1) & 1) * WW_RAW_STAGE;
            const float* rs_next = lds + WW_RAW_OFF + (q & 1) * WW_RAW_STAGE;
            // rows of A dY for this wave's GEMMs, from the dY values requested a step ago
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    // rows (0, 0+1) for the first GEMM half, (0-1, 1) for the second: one fma each with the
                    // wave's constants instead of computing both forms and selecting
                    rr[0][b][j] = __builtin_fmaf(rr_c0, dyr[1][b][j], dyr[0][b][j]);
                    rr[1][b][j] = __builtin_fmaf(rr_c1, dyr[0][b][j], dyr[1][b][j]);
                }
            // all sixteen are formed here, before the next strip's dY is requested: the requests then land in the
            // registers the old values leave (left to itself the compiler forms the second row's values where
            // they are used, keeps the old dY alive until then and copies the new one over it at the loop's end,
            // sixteen moves per step)
#pragma unroll
            for (int ii = 0; ii < 2; ++ii)
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(rr[ii][b][j]) : : "memory");
            // (the old dY values count as used once more after that: a value that dies in the multiply-add gets the
            // result written over it, and the result, which lives on, would again keep the request's register busy)
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int j = 0; j < 4; ++j) asm volatile("" : : "v"(dyr[r][b][j]));
            load_dy(dp, d_left > 0);           // strip q+1
            next_d();
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int gp = 0; gp < WG_GW / 2; ++gp) {
                const int g0 = 2 * gp, g1 = 2 * gp + 1, cur = gp & 1, ii = gp >> 1;
                // A operands of the pair: columns (0, 1) or (2, 3) of  rr . A^T  (sign of column 3 left out)
                float a0[4], a1[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    a0[j] = (gp & 1) ? rr[ii][0][j] - rr[ii][1][j] : rr[ii][0][j];
                    a1[j] = (gp & 1) ? rr[ii][1][j] : rr[ii][0][j] + rr[ii][1][j];
                }
                // the waves that write the bias gradient at the end: their a1 is now the sum of dY over a
                // tile's four pixels
                if (gp == 2 && gh == 0 && wn == 0) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) db_acc += a1[j];
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int j = k >> 1;
                    if ((k & 1) == 0)
                        acc[g0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[j], bf[cur][0][j], acc[g0], 0, 0, 0);
                    else
                        acc[g1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[j], bf[cur][1][j], acc[g1], 0, 0, 0);
                    if (k == 0) {
                        if (gp < 3) {          // B fragments of the next section
#pragma unroll
                            for (int g = 0; g < 2; ++g)
#pragma unroll
                                for (int jj = 0; jj < 4; ++jj)
                                    bf[cur ^ 1][g][jj] = vs[((g0 + 2 + g) * WW_TILES + 2 * jj) * 64];
                        } else {
                            store_out(vn, 3);
                            __syncthreads();   // stage 2 of strip q+1 and stage 1 of strip q+2 are in LDS
#pragma unroll
                            for (int g = 0; g < 2; ++g)
#pragma unroll
                                for (int jj = 0; jj < 4; ++jj)
                                    bf[0][g][jj] = vs_next[(g * WW_TILES + 2 * jj) * 64];
                            read_col(rs_next, 0);
                        }
                    }
                    // stage 2 of strip q+1
                    if (gp == 0 && k == 2) transform_col(0);
                    if (gp == 0 && k == 3) read_col(rs, 1);
                    if (gp == 0 && k == 5) transform_col(1);
                    if (gp == 0 && k == 6) read_col(rs, 2);
                    if (gp == 1 && k == 1) transform_col(2);
                    if (gp == 1 && k == 2) read_col(rs, 3);
                    // (strip q+1's last patch read; the next one, in the last section, is strip q+2's first)
                    if (VERT && gp == 1 && k == 3) { vstrip_next<true>(a, tp); set_window_rows(tp, q & 1); }
                    if (gp == 1 && k == 4) transform_col(3);
                    if (gp == 2 && (k == 1 || k == 3 || k == 5)) transform_out(k >> 1);
                    if (gp == 2 && (k == 2 || k == 4 || k == 6)) store_out(vn, (k >> 1) - 1);
                    if (gp == 2 && k == 7) transform_out(3);
                    // stage 1: the registers hold strip q+2 (requested a step ago); then request strip q+3
                    if (gp == 1 && k >= 5) store_raw(q & 1, k - 5);
                    if (gp == 2 && k == 0) { load_raw(lp, l_left > 0); next_l(); }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    }

    // ---- the block's sums: partial dU in [g][k][c] order, partial dbias per (tile half, k)
    // element e = (g * 64 + k) * 64 + c of a pair's dU lies at [e / 256][rank][e % 256]: the ranks' values of
    // one kilobyte of elements are adjacent, so the kernel that sums over the ranks reads contiguous memory
    float* part = a.part + (size_t)pair * a.ranks * WW_PART_STRIDE + (size_t)rank * 256;
    const size_t chunk_pitch = (size_t)a.ranks * 256;
#pragma unroll
    for (int g = 0; g < WG_GW; ++g)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            float v;
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(acc[g][e]));
            const int k = wm * 32 + 8 * (e / 4) + 4 * h + (e % 4);
            const int el = ((gh * WG_GW + g) * 64 + k) * 64 + wn * 32 + cl;
            part[(size_t)(el >> 8) * chunk_pitch + (el & 255)] = v;
        }
    if (gh == 0 && wn == 0) a.part_db[((size_t)(pair * a.ranks + rank) * 2 + h) * 64 + wm * 32 + cl] = db_acc;
}

constexpr int WW_SUM_GROUPS = 4;   // rank groups summed by different blocks (more loads in flight)

// Sums of the ranks' partial dU (and partial dbias) of every pair: blockIdx.y picks a quarter of the
// ranks, a thread owns four consecutive elements and keeps eight 16-byte loads in flight.  The order of
// all additions is fixed.  du4 / db4: [group][pair][...].
__global__ __launch_bounds__(256) void winograd_wgrad_sum_kernel(const float* __restrict__ part,
                                                                 const float* __restrict__ part_db,
                                                                 float* __restrict__ du4, float* __restrict__ db4,
                                                                 int n_pairs, int ranks) {
    const int per_pair = WW_PART_FLOATS / 4;
    const int grp = blockIdx.y, r0 = grp * ranks / WW_SUM_GROUPS, r1 = (grp + 1) * ranks / WW_SUM_GROUPS;
    const long id = (long)blockIdx.x * 256 + threadIdx.x;
    if (id < (long)n_pairs * per_pair) {
        const int pair = (int)(id / per_pair), i = (int)(id % per_pair);
        // (layout [element / 256][rank][element % 256], see the kernel that writes it)
        const float* src = part + (size_t)pair * ranks * WW_PART_STRIDE + (size_t)(i >> 6) * ranks * 256 + (i & 63) * 4;
        float4_t acc[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc[u] = float4_t{0.f, 0.f, 0.f, 0.f};
        for (int r = r0; r < r1; r += 8) {
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (r + u < r1) acc[u] += *(const float4_t*)(src + (size_t)(r + u) * 256);
        }
        ((float4_t*)du4)[(size_t)grp * n_pairs * per_pair + id] =
            ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
    }
    if (id < (long)n_pairs * 64) {
        const int pair = (int)(id / 64), k = (int)(id % 64);
        float sb[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) sb[u] = 0.f;
        for (int r = 2 * r0; r < 2 * r1; r += 16) {
#pragma unroll
            for (int u = 0; u < 16; ++u)
                if (r + u < 2 * r1) sb[u] += part_db[((size_t)pair * ranks * 2 + r + u) * 64 + k];
        }
#pragma unroll
        for (int w = 8; w >= 1; w >>= 1)
#pragma unroll
            for (int u = 0; u < w; ++u) sb[u] += sb[u + w];
        db4[(size_t)grp * n_pairs * 64 + id] = sb[0];
    }
}

// dw[k][r][s][c] = (G^T dU[.][k][c] G)[r][s] with the signs of A's last row / column restored, and dbias.
__global__ __launch_bounds__(256) void winograd_wgrad_final_kernel(const float* __restrict__ du4,
                                                                   const float* __restrict__ db4,
                                                                   float* __restrict__ dw, float* __restrict__ db,
                                                                   int K, int C, int c_blocks, int n_pairs) {
    const long id = (long)blockIdx.x * 256 + threadIdx.x;
    if (id >= (long)K * C) return;
    const int c = (int)(id % C), k = (int)(id / C);
    const int pair = (k / 64) * c_blocks + c / 64;
    const float* src = du4 + (size_t)pair * WW_PART_FLOATS + (k % 64) * 64 + (c % 64);
    const size_t gstride = (size_t)n_pairs * WW_PART_FLOATS;
    float u[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            const float* e = src + (i * 4 + m) * 64 * 64;
            const float v = (e[0] + e[gstride]) + (e[2 * gstride] + e[3 * gstride]);
            u[i][m] = ((i == 3) != (m == 3)) ? -v : v;
        }
    float t[4][3];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        t[i][0] = u[i][0] + 0.5f * (u[i][1] + u[i][2]);
        t[i][1] = 0.5f * (u[i][1] - u[i][2]);
        t[i][2] = u[i][3] + 0.5f * (u[i][1] + u[i][2]);
    }
    float* out = dw + (size_t)k * 9 * C + c;
#pragma unroll
    for (int s = 0; s < 3; ++s) {
        out[(0 * 3 + s) * C] = t[0][s] + 0.5f * (t[1][s] + t[2][s]);
        out[(1 * 3 + s) * C] = 0.5f * (t[1][s] - t[2][s]);
        out[(2 * 3 + s) * C] = t[3][s] + 0.5f * (t[1][s] + t[2][s]);
    }
    if (db && c == 0) {
        const float* e = db4 + (size_t)((k / 64) * c_blocks) * 64 + (k % 64);
        const size_t bs = (size_t)n_pairs * 64;
        db[k] = (e[0] + e[bs]) + (e[2 * bs] + e[3 * bs]);
    }
}

bool wino_wgrad_shape_ok(int C, int K) {
    if (C % 64 != 0 || K % 64 != 0) return false;
    const int pairs = (C / 64) * (K / 64);
    return pairs <= WW_BLOCKS && (pairs & (pairs - 1)) == 0;
}

}  // namespace

static int g_wgrad_strips = 0;
extern "C" int pd_conv3x3_winograd_set_wgrad_strips(int mode) {
    PD_REQUIRE(mode >= 0 && mode <= 2, PD_EINVAL, "pd_conv3x3_winograd_set_wgrad_strips: mode is 0, 1 or 2");
    g_wgrad_strips = mode;
    return PD_OK;
}

extern "C" int pd_conv3x3_winograd_wgrad_supported(int C, int K) {
    return (C > 0 && K > 0 && wino_wgrad_shape_ok(C, K)) ? 1 : 0;
}

extern "C" int pd_conv3x3_winograd_wgrad_workspace_bytes(int C, int K, uint64_t* bytes) {
    PD_REQUIRE(bytes != nullptr, PD_EINVAL, "pd_conv3x3_winograd_wgrad_workspace_bytes: NULL pointer");
    PD_REQUIRE(C > 0 && K > 0 && wino_wgrad_shape_ok(C, K), PD_ESHAPE,
               "pd_conv3x3_winograd_wgrad_workspace_bytes: needs C and K multiples of 64 with C*K/4096 a power "
               "of two <= 256 (C=%d K=%d)", C, K);
    const uint64_t pairs = (uint64_t)(C / 64) * (K / 64);
    // per block: partial dU and 2 x 64 partial dbias; per pair and rank group: summed dU and dbias
    *bytes = ((uint64_t)WW_BLOCKS * (WW_PART_STRIDE + 128) + WW_SUM_GROUPS * pairs * (WW_PART_FLOATS + 64)) * sizeof(float);
    return PD_OK;
}

extern "C" int pd_conv3x3_winograd_wgrad_nhwc_f32(const float* x, const float* dy, float* dw, float* dbias,
                                                  void* workspace, uint64_t workspace_bytes, int N, int H, int W,
                                                  int C, int K, void* stream) {
    const char* who = "pd_conv3x3_winograd_wgrad_nhwc_f32";
    PD_REQUIRE(N > 0 && H > 0 && W > 0 && C > 0 && K > 0, PD_ESHAPE, "%s: dimensions must be positive", who);
    PD_REQUIRE(wino_wgrad_shape_ok(C, K), PD_ESHAPE, "%s: unsupported channel counts C=%d K=%d", who, C, K);
    PD_REQUIRE((long)W * (C > K ? C : K) < (1L << 28), PD_ESHAPE, "%s: image row too large", who);
    // the kernel counts pixels over all images in 32 bits, a few strips past the last one included
    PD_REQUIRE(((long)N * H + 2L * H + 8) * W < (1L << 31), PD_ESHAPE, "%s: too many pixels", who);
    PD_REQUIRE(x && dy && dw && workspace, PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE(pd_aligned(x, 16) && pd_aligned(dy, 16) && pd_aligned(workspace, 16), PD_EINVAL,
               "%s: tensors must be 16-byte aligned", who);
    uint64_t need = 0;
    pd_conv3x3_winograd_wgrad_workspace_bytes(C, K, &need);
    PD_REQUIRE(workspace_bytes >= need, PD_EINVAL, "%s: workspace too small (%llu < %llu bytes)", who,
               (unsigned long long)workspace_bytes, (unsigned long long)need);
    WinoWgradArgs a;
    a.x = x; a.dy = dy;
    a.N = N; a.H = H; a.W = W; a.C = C; a.K = K;
    // upright strips where strips of 2 x 16 pixels would pad the width (g_wgrad_strips: 0 = that rule, 1 = never,
    // 2 = wherever the upright kernel applies)
    // (an upright strip's dY is addressed with 32-bit byte offsets over its 16 rows)
    const bool upright_ok = H % 2 == 0 && W % 2 == 0 && H >= 14 && (long)WW_VROWS * W * K * 4 < (1L << 31);
    const bool upright = upright_ok && (g_wgrad_strips == 2 || (g_wgrad_strips == 0 && W % (2 * WW_TILES) != 0));
    a.rows_all = N * H;
    a.sx = upright ? W / 2 : (W + 2 * WW_TILES - 1) / (2 * WW_TILES);
    a.sy = (H + 1) / 2;
    const long strips = upright ? (long)((a.rows_all + WW_VROWS - 1) / WW_VROWS) * a.sx : (long)N * a.sx * a.sy;
    PD_REQUIRE(strips <= 0x7ffffff0L, PD_ESHAPE, "%s: too many strips", who);
    a.n_strips = (int)strips;
    a.c_blocks = C / 64;
    a.n_pairs = a.c_blocks * (K / 64);
    a.ranks = WW_BLOCKS / a.n_pairs;
    a.strips_per_rank = (int)((strips + a.ranks - 1) / a.ranks);
    float* ws = (float*)workspace;
    a.part = ws;
    a.part_db = ws + (size_t)WW_BLOCKS * WW_PART_STRIDE;
    float* du = a.part_db + (size_t)WW_BLOCKS * 128;
    float* dbsum = du + (size_t)WW_SUM_GROUPS * a.n_pairs * WW_PART_FLOATS;
    hipStream_t s = (hipStream_t)stream;
    if (upright) winograd_wgrad_kernel<true><<<WW_BLOCKS, WW_THREADS, 0, s>>>(a);
    else winograd_wgrad_kernel<false><<<WW_BLOCKS, WW_THREADS, 0, s>>>(a);
    PD_CHECK_LAUNCH(who);
    const long sum_threads = (long)a.n_pairs * (WW_PART_FLOATS / 4);
    winograd_wgrad_sum_kernel<<<dim3((unsigned)((sum_threads + 255) / 256), WW_SUM_GROUPS), 256, 0, s>>>(
        a.part, a.part_db, du, dbsum, a.n_pairs, a.ranks);
    PD_CHECK_LAUNCH(who);
    winograd_wgrad_final_kernel<<<(unsigned)(((long)K * C + 255) / 256), 256, 0, s>>>(du, dbsum, dw, dbias, K, C,
                                                                                     a.c_blocks, a.n_pairs);
    PD_CHECK_LAUNCH(who);
    return PD_OK;
}
