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
constexpr int WG_HALO = WG_PIX + 2;              // input halo tile: 18 x 18 pixels
constexpr int WG_PIECES = WG_HALO * WG_HALO * 2; // 16-byte pieces (pixel, 4-channel half) of one chunk of it
// The halo tile in LDS: four planes (channel half, column parity) of 18 rows x 12 16-byte units; the
// unit of (half, row, col) is ((half * 2 + (col & 1)) * 18 + row) * 12 + (col >> 1).  The eight tiles
// of a tile row then read eight consecutive units and the next tile row lands 8 units further
// (mod 16): a wave's 128-bit reads of one patch position are free of bank conflicts.
constexpr int WG_RAW_PITCH = 12;
constexpr int WG_RAW_STAGE = 4 * WG_HALO * WG_RAW_PITCH * 4;   // floats
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
    int N, H, W, C, K;
    int relu;
    int tiles_x, tiles_y, k_blocks, n_chunks;
    int n_items, items_per_xcd;   // work items (pixel tile x channel block) in all / per die
};

// U = G g G^T for every (out channel k, in channel c), G = [[1,0,0],[.5,.5,.5],[.5,-.5,.5],[0,0,1]].
// Output order: [k / 64][c / 8][g][(k % 64) / 32][(c % 8) / 4][k % 32][c % 4] -- for a block's 64
// channels and one chunk, position g, the two 1 KB halves are exactly what the lanes of the waves
// with wn = 0 / 1 load (lane = 32 * ((c % 8) / 4) + k % 32 holds four consecutive c).  Rows
// k >= K of the last block of 64 are zero.  With rot180 the filter is taken as
// f[k][r][s][c] = w[c][2-r][2-s][k] (w is then [C][3][3][K]): the input-gradient filter.
__global__ __launch_bounds__(256) void winograd_filter_kernel(const float* __restrict__ w, float* __restrict__ u,
                                                              int K, int C, int k_pad, int rot180) {
    const long id = (long)blockIdx.x * 256 + threadIdx.x;
    if (id >= (long)k_pad * C) return;
    int k, c;
    if (rot180) { k = (int)(id % k_pad); c = (int)(id / k_pad); }
    else { c = (int)(id % C); k = (int)(id / C); }
    float g[3][3];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int s = 0; s < 3; ++s) {
            float v = 0.f;
            if (k < K) v = rot180 ? w[((size_t)c * 9 + (2 - r) * 3 + (2 - s)) * K + k]
                                  : w[((size_t)k * 9 + r * 3 + s) * C + c];
            g[r][s] = v;
        }
    float t[4][3];
#pragma unroll
    for (int s = 0; s < 3; ++s) {
        t[0][s] = g[0][s];
        t[1][s] = 0.5f * (g[0][s] + g[1][s] + g[2][s]);
        t[2][s] = 0.5f * (g[0][s] - g[1][s] + g[2][s]);
        t[3][s] = g[2][s];
    }
    const int n_chunks = C / WG_CC;
    const size_t base = ((size_t)((k / WG_BN) * n_chunks + c / WG_CC) * WG_G) * (2 * WG_FRAG) +
                        ((k % WG_BN) / 32) * WG_FRAG + ((c % WG_CC) / 4) * 128 + (k % 32) * 4 + (c % 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float o[4] = {t[i][0], 0.5f * (t[i][0] + t[i][1] + t[i][2]), 0.5f * (t[i][0] - t[i][1] + t[i][2]),
                            t[i][2]};
#pragma unroll
        for (int m = 0; m < 4; ++m) u[base + (size_t)(i * 4 + m) * (2 * WG_FRAG)] = o[m];
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
template <bool MASK>
__global__ __launch_bounds__(WG_THREADS, 1) void winograd_fwd_kernel(const WinoArgs a) {
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
    int hy[2], hx[2], raw_dst[2];
    uint32_t pcg[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int p = tid + WG_THREADS * j, pix = p >> 1, half = p & 1;
        hy[j] = pix / WG_HALO;
        hx[j] = pix - hy[j] * WG_HALO;
        pcg[j] = half * 16;
        raw_dst[j] = (((half * 2 + (hx[j] & 1)) * WG_HALO + hy[j]) * WG_RAW_PITCH + (hx[j] >> 1)) * 4;
    }
    const bool second_piece = tid + WG_THREADS < WG_PIECES;
    const float* ximg = a.x;
    const float* mimg = MASK ? a.mask : a.x;
    const uint32_t img_bytes = (uint32_t)a.H * a.W * a.C * 4;
    uint32_t loff[2];
    // byte offsets of the thread's pieces for the i-th item of this block; padding (and everything
    // past the last item) gets an offset beyond the buffer's size, for which a buffer load returns 0
    auto set_load_item = [&](int i) {
        if (i < n_my) {
            const WinoItem w = wino_decode(a, item0 + i * gx8);
            const size_t img = (size_t)w.n * a.H * a.W * a.C;
            ximg = a.x + img;
            if (MASK) mimg = a.mask + img;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int gy = w.y0 - 1 + hy[j], gx = w.x0 - 1 + hx[j];
                loff[j] = (gy >= 0 && gy < a.H && gx >= 0 && gx < a.W && (j == 0 || second_piece))
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
    auto store_raw = [&](int stage, int j) {
        float4_t v = rawr[j];
        if (MASK) {
#pragma unroll
            for (int c = 0; c < 4; ++c) v[c] = rawm[MASK ? j : 0][c] > 0.f ? v[c] : 0.f;
        }
        if (j == 0 || second_piece) *(float4_t*)(lds + WG_RAW_OFF + stage * WG_RAW_STAGE + raw_dst[j]) = v;
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
    const int unit0 = (cg * 2 * WG_HALO + 2 * (tt >> 3)) * WG_RAW_PITCH + (tt & 7);
    const int src_a = (unit0 + row_a * WG_RAW_PITCH) * 4, src_b = (unit0 + row_b * WG_RAW_PITCH) * 4;
    float4_t t[4];
    float4_t dc[2][2];                         // column s of the patch waits in dc[s & 1] until its section
    auto read_col = [&](const float* rs, int s) {
        const int o = (((s & 1) * WG_HALO) * WG_RAW_PITCH + (s >> 1)) * 4;
        dc[s & 1][0] = *(const float4_t*)(rs + src_a + o);
        dc[s & 1][1] = *(const float4_t*)(rs + src_b + o);
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
    __syncthreads();
#pragma unroll
    for (int s = 0; s < 4; ++s) { read_col(lds + WG_RAW_OFF, s); transform_col(s); }
#pragma unroll
    for (int m = 0; m < 4; ++m) { transform_out(m); store_out(lds, m); }
    __syncthreads();
    float4_t af[2][2];                         // A fragments of GEMM pair p wait in af[p & 1] for one section
    af[0][0] = *(const float4_t*)(lds + a_lane);
    af[0][1] = *(const float4_t*)(lds + a_lane + (2 * WG_FRAG));
    read_col(lds + WG_RAW_OFF + WG_RAW_STAGE, 0);

    // Per step: four sections of 8 MFMAs (GEMM pair gp) each, every MFMA followed by a small piece of
    // the other stages' work; the scheduler may not move anything across the sub-step boundaries.  LDS
    // reads are issued at least one section before their use.  The step's barrier sits in the last
    // section, which then requests the first fragments and patch column of the next step while its own
    // MFMAs (operands already in registers) run.  The reduction index of MFMA j pairs channel j (lanes
    // 0-31) with channel 4+j (lanes 32-63).
    int q = 0;                                 // step of stage 3
    for (int m_i = 0; m_i < n_my; ++m_i) {
    zero_acc();
    for (int m_cc = 0; m_cc < a.n_chunks; ++m_cc, ++q) {
        const float* vs = lds + (q & 1) * WG_V_STAGE + a_lane;
        const float* vs_next = lds + ((q + 1) & 1) * WG_V_STAGE + a_lane;
        float* vn = lds + ((q + 1) & 1) * WG_V_STAGE;
        const float* rs = lds + WG_RAW_OFF + ((q + 1) & 1) * WG_RAW_STAGE;   // step q+1, transformed now
        const float* rs_next = lds + WG_RAW_OFF + (q & 1) * WG_RAW_STAGE;    // step q+2, stored in section 1
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
                        af[cur ^ 1][0] = *(const float4_t*)(vs + (g0 + 2) * (2 * WG_FRAG));
                        af[cur ^ 1][1] = *(const float4_t*)(vs + (g1 + 2) * (2 * WG_FRAG));
                    } else {
                        store_out(vn, 3);
                        __syncthreads();       // stage 2 of step q+1 and stage 1 of step q+2 are in LDS
                        af[0][0] = *(const float4_t*)(vs_next);
                        af[0][1] = *(const float4_t*)(vs_next + (2 * WG_FRAG));
                        read_col(rs_next, 0);
                    }
                }
                // stage 2 of step q+1: columns 0..3 of the patch, then the four output vectors
                if (gp == 0 && k == 1) read_col(rs, 1);
                if (gp == 0 && k == 3) transform_col(0);
                if (gp == 0 && k == 4) read_col(rs, 2);
                if (gp == 0 && k == 6) transform_col(1);
                if (gp == 1 && k == 1) read_col(rs, 3);
                if (gp == 1 && k == 3) transform_col(2);
                if (gp == 1 && k == 6) transform_col(3);
                if (gp == 2 && (k == 1 || k == 3 || k == 5)) transform_out(k >> 1);
                if (gp == 2 && (k == 2 || k == 4 || k == 6)) store_out(vn, (k >> 1) - 1);
                if (gp == 2 && k == 7) transform_out(3);
                // stage 1: the registers hold step q+2 (requested a step ago); then request step q+3
                if (gp == 1 && k == 2) store_raw(q & 1, 0);
                if (gp == 1 && k == 4) store_raw(q & 1, 1);
                if (gp == 1 && k == 5) load_raw(l_cc);
                if (k == 7) {                  // the filter fragments of this pair, for step q+1
                    uf[g0] = load_u(ustep, g0);
                    uf[g1] = load_u(ustep, g1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        advance_l();
        advance_u();
    }
        {
            // ---- epilogue of item m_i.  Each wave applies A^T . A to its two rows of M (lane-local);
            //      the waves with gh = 0 write their part to the staging tile, then the others add theirs.
            const WinoItem w = wino_decode(a, item0 + m_i * gx8);
            const int k0 = w.kb * WG_BN;
            float* stg = lds + WG_OUT_OFF;
            const size_t oimg = (size_t)w.n * a.H * a.W * a.K;
            const int kl = wn * 32 + (lane & 31);
            // accumulator element e of this lane is tile wm*32 + 8*(e/4) + 4*(lane>>5) + e%4, channel kl;
            // its 2 x 2 output pixels sit at a per-lane base plus an offset that depends on (e, i) only
            float* stg_lane = stg + ((8 * wm) * WG_PIX + 8 * (lane >> 5)) * WG_OP + kl;
            auto stg_index = [&](int e, int i) {
                return ((2 * (e / 4) + (i >> 1)) * WG_PIX + 2 * (e % 4) + (i & 1)) * WG_OP;
            };
            auto out_rows = [&](bool add) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
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
                        s0[m] = add ? mv[m] : mv[m] + mv[4 + m];
                        s1[m] = add ? -mv[m] - mv[4 + m] : mv[4 + m];
                    }
                    const float part[4] = {s0[0] + s0[1] + s0[2], s0[1] - s0[2] - s0[3], s1[0] + s1[1] + s1[2],
                                           s1[1] - s1[2] - s1[3]};
                    // (each staging element belongs to one lane of one wave per phase: plain read-add-write)
                    float prev[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) prev[i] = add ? stg_lane[stg_index(e, i)] : 0.f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) stg_lane[stg_index(e, i)] = prev[i] + part[i];
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            if (gh == 0) out_rows(false);
            __syncthreads();
            if (gh == 1) out_rows(true);
            __syncthreads();
            // bias, ReLU, output mask and the NHWC stores.  Thread -> pixel column (tid >> 4) & 15, channels
            // k4..k4+3, pixel rows (tid >> 8) + 2 it: one base offset, a scalar stride per row pair.  Pixels
            // outside the image get an offset beyond the buffer's size: such a store is dropped.
            constexpr int NV = 256 * (WG_BN / 4) / WG_THREADS;
            const int k4 = (tid & 15) * 4, pcol = (tid >> 4) & 15, prow = tid >> 8;
            float4_t b4 = {0.f, 0.f, 0.f, 0.f};
            if (a.bias) {
#pragma unroll
                for (int c = 0; c < 4; ++c) b4[c] = k0 + k4 + c < a.K ? a.bias[k0 + k4 + c] : 0.f;
            }
            const uint32_t out_bytes = (uint32_t)a.H * a.W * a.K * 4;
            const __amdgpu_buffer_rsrc_t yr =
                __builtin_amdgcn_make_buffer_rsrc((void*)(a.y + oimg), 0, out_bytes, 0x00020000);
            const __amdgpu_buffer_rsrc_t omr = __builtin_amdgcn_make_buffer_rsrc(
                (void*)((a.out_mask ? a.out_mask : a.y) + oimg), 0, out_bytes, 0x00020000);
            const bool col_ok = w.x0 + pcol < a.W && k0 + k4 < a.K;
            const uint32_t obase = (uint32_t)(((w.y0 + prow) * a.W + w.x0 + pcol) * a.K + k0 + k4) * 4;
            const int row_stride = 2 * a.W * a.K * 4;
            const float* src = stg + (prow * WG_PIX + pcol) * WG_OP + k4;
#pragma unroll
            for (int it = 0; it < NV; ++it) {
                const uint32_t voff = (col_ok && w.y0 + prow + 2 * it < a.H) ? obase : 0x80000000u;
                float4_t v = *(const float4_t*)(src + it * 2 * WG_PIX * WG_OP) + b4;
                if (a.relu) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) v[c] = v[c] > 0.f ? v[c] : 0.f;
                }
                if (a.out_mask) {
                    const float4_t mk = __builtin_bit_cast(
                        float4_t, __builtin_amdgcn_raw_buffer_load_b128(omr, voff, it * row_stride, 2));
#pragma unroll
                    for (int c = 0; c < 4; ++c) v[c] = mk[c] > 0.f ? v[c] : 0.f;
                }
                typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), yr, voff, it * row_stride, 2);
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
    const int k_pad = (K + WG_BN - 1) / WG_BN * WG_BN;
    const long total = (long)k_pad * C;
    winograd_filter_kernel<<<(unsigned)((total + 255) / 256), 256, 0, (hipStream_t)stream>>>(w, u, K, C, k_pad, rot180);
    PD_CHECK_LAUNCH("pd_conv3x3_winograd_filter_f32");
    return PD_OK;
}

extern "C" int pd_conv3x3_winograd_fwd_nhwc_f32(const float* x, const float* u, const float* bias,
                                                const float* in_mask, const float* out_mask, float* y, int N, int H,
                                                int W, int C, int K, int relu, void* stream) {
    const char* who = "pd_conv3x3_winograd_fwd_nhwc_f32";
    PD_REQUIRE(N > 0 && H > 0 && W > 0 && C > 0 && K > 0, PD_ESHAPE, "%s: dimensions must be positive", who);
    PD_REQUIRE(wino_shape_ok(C, K), PD_ESHAPE, "%s: needs C %% 8 == 0 and K %% 4 == 0 (C=%d K=%d)", who, C, K);
    PD_REQUIRE((long)H * W * (C > K ? C : K) < (1L << 29), PD_ESHAPE, "%s: image too large", who);
    PD_REQUIRE((long)C * WG_G * WG_BN * 4 < (1L << 31), PD_ESHAPE, "%s: too many input channels", who);
    PD_REQUIRE(x && u && y, PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE(pd_aligned(x, 16) && pd_aligned(u, 16) && pd_aligned(y, 16) && pd_aligned(in_mask, 16) &&
                   pd_aligned(out_mask, 16), PD_EINVAL, "%s: tensors must be 16-byte aligned", who);
    WinoArgs a;
    a.x = x; a.u = u; a.bias = bias; a.mask = in_mask; a.out_mask = out_mask; a.y = y;
    a.N = N; a.H = H; a.W = W; a.C = C; a.K = K;
    a.relu = relu != 0;
    a.tiles_x = (W + WG_PIX - 1) / WG_PIX;
    a.tiles_y = (H + WG_PIX - 1) / WG_PIX;
    a.k_blocks = (K + WG_BN - 1) / WG_BN;
    a.n_chunks = C / WG_CC;
    const long items = (long)N * a.tiles_x * a.tiles_y * a.k_blocks;
    PD_REQUIRE(items <= 0x7ffffff0L, PD_ESHAPE, "%s: too many tiles", who);
    a.n_items = (int)items;
    a.items_per_xcd = (int)((items + WG_XCD - 1) / WG_XCD);
    // one persistent block per CU (the kernel needs a CU's whole register file), in multiples of 8
    int dev = 0, cus = 0;
    PD_HIP(hipGetDevice(&dev));
    PD_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    long blocks = (long)(cus / WG_XCD) * WG_XCD;
    if (blocks < WG_XCD) blocks = WG_XCD;
    if (blocks > (long)a.items_per_xcd * WG_XCD) blocks = (long)a.items_per_xcd * WG_XCD;
    dim3 grid((unsigned)blocks);
    hipStream_t s = (hipStream_t)stream;
    if (in_mask) winograd_fwd_kernel<true><<<grid, WG_THREADS, 0, s>>>(a);
    else winograd_fwd_kernel<false><<<grid, WG_THREADS, 0, s>>>(a);
    PD_CHECK_LAUNCH(who);
    return PD_OK;
}
