// 3x3 / stride 1 / pad 1 convolution, fp32, on the gfx950 matrix cores
// (v_mfma_f32_32x32x2_f32): forward (+bias, +ReLU), input gradient, weight and bias
// gradient.  Activations are NHWC, filters KRSC (out-ch, kh, kw, in-ch).
//
// These are the kernels behind the torch.nn.Conv2d(k=3, s=1, p=1) layers of the
// reference's VGG16 stages (runtime/image_classification/models/vgg16/
// gpus=4_straight/stage0.py:12-14 ... stage3.py:12-17), which there run in cuDNN:
// forward in StageRuntime._run_forward (runtime/runtime.py:529-530), the two gradients
// inside torch.autograd.backward (runtime/runtime.py:606-608).
//
// Bound: MFMA fp32 (157.3 TFLOP/s).  Work per call: 2*9*C*K*N*H*W flop.
//
// Forward / input gradient (implicit GEMM, rows = pixels, cols = out channels,
// reduction = 9 taps x C):
//   a 256-thread block owns a TH x TW pixel tile (256 pixels) x 64 out channels; each
//   of its 4 waves owns 64 pixels x 64 channels = 2x2 MFMA tiles.  The reduction runs
//   in chunks of CC input channels: the (TH+2)x(TW+2) input halo tile and the
//   9 x 64 x CC filter slice are staged in LDS once per chunk and all nine taps read
//   the SAME halo tile at shifted addresses (no im2col copy).  Both LDS arrays are
//   channel-contiguous with a row pitch of CC+4 floats, so an operand fragment for
//   four consecutive MFMAs is one conflict-free 128-bit LDS read.
//   The input gradient is the same kernel run on dY with the filter rotated by 180
//   degrees and its channel roles swapped (pd_conv3x3_filter_rot180).
// Weight gradient (rows = out channels, cols = in channels, reduction = pixels):
//   a block owns 64 out x 64 in channels x 9 taps, each wave one 32x32 (k,c) block for
//   all 9 taps (9 MFMA tiles = 144 accumulator registers).  Blocks stride over pixel
//   tiles, stage dY and the X halo tile in LDS, and write per-block partial sums that a
//   second kernel reduces in a fixed order (deterministic, no atomics).  The bias
//   gradient falls out of the same dY tile.
#include <mutex>

#include "pd_internal.h"

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

namespace {

constexpr int CONV_THREADS = 256;
constexpr int BN = 64;  // out channels per block (forward / dgrad)

struct ConvArgs {
    const float* x;     // [N,H,W,C]
    const float* w;     // [K,3,3,C]
    const float* bias;  // [K] or null
    const float* mask;  // [N,H,W,C] or null: x is taken as 0 where mask <= 0 (fused ReLU backward)
    float* y;           // [N,H,W,K]
    const float* out_mask;  // [N,H,W,K] or null: y is written as 0 where out_mask <= 0 (the ReLU
                            // backward of the layer that produced this convolution's input)
    int N, H, W, C, K;
    int relu;
    int tiles_x, tiles_y;
    int n_tiles, k_blocks, tiles_per_xcd;
    int c_vec;          // C % 4 == 0 and x/w 16-byte aligned: 128-bit global loads
    int y_vec;          // K % 4 == 0 and y 16-byte aligned: 128-bit stores through the LDS transpose
};

constexpr int N_XCD = 8;  // MI355X: 8 accelerator dies, each with its own L2; workgroups are
                          // handed to them round-robin by linear workgroup id

// Global -> register staging of one reduction chunk (input halo tile + filter slice).
// All loads of a chunk are issued back to back (fixed trip counts, no divergent
// branches: out-of-range elements read a safe address and are zeroed by a select), so
// a thread has ~15 128-bit loads in flight instead of one.
template <int TH, int TW, int CC, bool MASK, bool VEC>
struct FwdStage {
    static constexpr int HW_ = TW + 2;
    static constexpr int HALO = (TH + 2) * (TW + 2);
    static constexpr int CP = CC + 4;
    static constexpr int Q = CC / 4;
    static constexpr int IN_ITERS = (HALO * Q + CONV_THREADS - 1) / CONV_THREADS;
    static constexpr int W_ITERS = (9 * BN * Q + CONV_THREADS - 1) / CONV_THREADS;

    // Raw loaded values.  Nothing here is *used* before store(): zero-filling of out-of-range
    // elements and the ReLU mask are applied when the registers are written to LDS, so the
    // loads stay in flight across the whole multiply phase that sits between load() and
    // store() (a use right after the load would force a wait for all of them).
    float4_t rin[IN_ITERS];
    float4_t rm[MASK ? IN_ITERS : 1];
    float4_t rw[W_ITERS];
    uint32_t ok_in, ok_w;   // bit it: element it is inside the tensor

    __device__ __forceinline__ void load(const ConvArgs& a, const float* __restrict__ xn,
                                         const float* __restrict__ mn, int y0, int x0, int k0, int c0, int tid) {
        ok_in = 0;
        ok_w = 0;
#pragma unroll
        for (int it = 0; it < IN_ITERS; ++it) {
            const int id = tid + it * CONV_THREADS;
            const int p = id / Q, q4 = (id % Q) * 4;
            const int gy = y0 + p / HW_ - 1, gx = x0 + p % HW_ - 1;
            const int c = c0 + q4;
            const bool ok = id < HALO * Q && gy >= 0 && gy < a.H && gx >= 0 && gx < a.W && c < a.C;
            ok_in |= (uint32_t)ok << it;
            const size_t off = ok ? ((size_t)gy * a.W + gx) * a.C + c : 0;
            if (VEC) {
                rin[it] = *(const float4_t*)(xn + off);
                if (MASK) rm[it] = *(const float4_t*)(mn + off);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const bool okj = ok && c + j < a.C;
                    rin[it][j] = okj ? xn[off + j] : 0.f;
                    if (MASK) rm[it][j] = okj ? mn[off + j] : 0.f;
                }
            }
        }
#pragma unroll
        for (int it = 0; it < W_ITERS; ++it) {
            const int id = tid + it * CONV_THREADS;
            const int row = id / Q, q4 = (id % Q) * 4;
            const int tap = row / BN, k = k0 + row % BN;
            const int c = c0 + q4;
            const bool ok = id < 9 * BN * Q && k < a.K && c < a.C;
            ok_w |= (uint32_t)ok << it;
            const size_t off = ok ? ((size_t)k * 9 + tap) * a.C + c : 0;
            if (VEC) {
                rw[it] = *(const float4_t*)(a.w + off);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) rw[it][j] = (ok && c + j < a.C) ? a.w[off + j] : 0.f;
            }
        }
    }

    __device__ __forceinline__ void store(float* in_tile, float* w_tile, int tid) const {
        const float4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int it = 0; it < IN_ITERS; ++it) {
            const int id = tid + it * CONV_THREADS;
            float4_t v = rin[it];
            if (MASK) {
                // gradient of a fused ReLU: dY counts only where the forward output was positive
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = rm[it][j] > 0.f ? v[j] : 0.f;
            }
            v = ((ok_in >> it) & 1u) ? v : zero;
            if (id < HALO * Q) *(float4_t*)(in_tile + (id / Q) * CP + (id % Q) * 4) = v;
        }
#pragma unroll
        for (int it = 0; it < W_ITERS; ++it) {
            const int id = tid + it * CONV_THREADS;
            const float4_t v = ((ok_w >> it) & 1u) ? rw[it] : zero;
            if (id < 9 * BN * Q) *(float4_t*)(w_tile + (id / Q) * CP + (id % Q) * 4) = v;
        }
    }
};

template <int TH, int TW, int CC, bool MASK, bool VEC>
__global__ __launch_bounds__(CONV_THREADS, 2) void conv3x3_fwd_kernel(const ConvArgs a) {
    static_assert(TH * TW == 256, "a block owns 256 pixels");
    static_assert(TW == 8 || TW == 16 || TW == 32, "an MFMA row tile is 32/TW rows of TW pixels");
    using Stage = FwdStage<TH, TW, CC, MASK, VEC>;
    constexpr int HW_ = Stage::HW_;
    constexpr int HALO = Stage::HALO;
    constexpr int CP = Stage::CP;
    constexpr int STEPS = 9 * (CC / 8);   // (tap, k-group) pairs per chunk
    constexpr int OP = BN + 4;            // pitch of the output staging tile
    constexpr int LDS_FLOATS = (HALO * CP + 9 * BN * CP) > 256 * OP ? (HALO * CP + 9 * BN * CP) : 256 * OP;
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
    float* const in_tile = lds;
    float* const w_tile = lds + HALO * CP;

    const int tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int idx = lane % 32, h = lane / 32;

    // XCD-aware tile order: workgroup id -> (die, sequence on that die).  Each die walks a
    // contiguous range of pixel tiles, and the out-channel blocks of one tile follow each
    // other on the same die, so halo rows/columns and re-read input tiles hit that die's L2.
    // (One block per tile, not persistent blocks: blocks that start staggered find their
    // neighbours' halo lines already in L2, blocks running in lockstep miss together --
    // measured 1.06x vs 1.46x of the algorithmic HBM bytes.)
    const int xcd = blockIdx.x % N_XCD, seq = blockIdx.x / N_XCD;
    int b = xcd * a.tiles_per_xcd + seq / a.k_blocks;
    if (b >= a.n_tiles) return;
    const int k0 = (seq % a.k_blocks) * BN;
    const int tx = b % a.tiles_x;
    b /= a.tiles_x;
    const int ty = b % a.tiles_y;
    const int n = b / a.tiles_y;
    const int y0 = ty * TH, x0 = tx * TW;

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // LDS offsets of this lane's two pixel rows (tap 0,0) and two filter rows.
    int a_off[2], b_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int q = (wave * 2 + i) * 32 + idx;
        a_off[i] = ((q / TW) * HW_ + (q % TW)) * CP + 4 * h;
        b_off[i] = (i * 32 + idx) * CP + 4 * h;
    }

    const float* xn = a.x + (size_t)n * a.H * a.W * a.C;
    const float* mn = MASK ? a.mask + (size_t)n * a.H * a.W * a.C : nullptr;

    // Software pipeline over the reduction chunks: the global loads of chunk i+1 are in
    // flight while chunk i is multiplied out of LDS.
    Stage st;
    st.load(a, xn, mn, y0, x0, k0, 0, tid);
    for (int c0 = 0; c0 < a.C; c0 += CC) {
        __syncthreads();  // everyone is done reading the previous chunk
        st.store(in_tile, w_tile, tid);
        __syncthreads();
        if (c0 + CC < a.C) st.load(a, xn, mn, y0, x0, k0, c0 + CC, tid);
        // ---- STEPS x (4 LDS reads + 16 MFMAs) ----------------------------------------------
#pragma unroll
        for (int step = 0; step < STEPS; ++step) {
            const int tap = step / (CC / 8), g = step % (CC / 8);
            const int shift = ((tap / 3) * HW_ + (tap % 3)) * CP;
            float4_t fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) fa[i] = *(const float4_t*)(in_tile + a_off[i] + shift + 8 * g);
#pragma unroll
            for (int j = 0; j < 2; ++j) fb[j] = *(const float4_t*)(w_tile + tap * BN * CP + b_off[j] + 8 * g);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
            // Instruction order for the scheduler: the four fragment reads of the NEXT step are spread
            // over the first twelve MFMAs of this one (3 MFMAs, 1 LDS read, ...), so their latency is
            // covered by this wave's own MFMAs instead of stalling it at the top of every step.
            if (step == 0) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                __builtin_amdgcn_sched_group_barrier(0x008, 3, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        }
    }

    // ---- epilogue: bias + ReLU, then the 256 x 64 result tile is transposed through LDS
    //      (reusing the operand tiles) so that every lane writes 16 contiguous bytes and a wave
    //      covers whole 256-byte pixel rows of the NHWC output -------------------------------
    float* yn = a.y + (size_t)n * a.H * a.W * a.K;
    if (a.y_vec) {
        // the output mask (if any) is fetched before the transpose, so its latency is covered by
        // the LDS traffic and the barriers below
        constexpr int NV = 256 * (BN / 4) / CONV_THREADS;
        float4_t mk[NV];
        if (a.out_mask) {
            const float* mn = a.out_mask + (size_t)n * a.H * a.W * a.K;
#pragma unroll
            for (int it = 0; it < NV; ++it) {
                const int id = tid + it * CONV_THREADS;
                const int q = id / (BN / 4), k4 = (id % (BN / 4)) * 4;
                const int gy = y0 + q / TW, gx = x0 + q % TW;
                if (gy < a.H && gx < a.W && k0 + k4 < a.K)
                    mk[it] = __builtin_nontemporal_load((const float4_t*)(mn + ((size_t)gy * a.W + gx) * a.K + k0 + k4));
            }
        }
        __syncthreads();  // all waves are done reading the operand tiles
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int k = k0 + j * 32 + idx;
            const float bv = (a.bias && k < a.K) ? a.bias[k] : 0.f;
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int q = (wave * 2 + i) * 32 + 8 * (e / 4) + 4 * h + (e % 4);
                    float v = acc[i][j][e] + bv;
                    if (a.relu) v = v > 0.f ? v : 0.f;
                    lds[q * OP + j * 32 + idx] = v;
                }
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < NV; ++it) {
            const int id = tid + it * CONV_THREADS;
            const int q = id / (BN / 4), k4 = (id % (BN / 4)) * 4;
            const int gy = y0 + q / TW, gx = x0 + q % TW;
            if (gy < a.H && gx < a.W && k0 + k4 < a.K) {
                float4_t v = *(const float4_t*)(lds + q * OP + k4);
                if (a.out_mask) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) v[c] = mk[it][c] > 0.f ? v[c] : 0.f;
                }
                __builtin_nontemporal_store(v, (float4_t*)(yn + ((size_t)gy * a.W + gx) * a.K + k0 + k4));
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int k = k0 + j * 32 + idx;
            if (k >= a.K) continue;
            const float bv = a.bias ? a.bias[k] : 0.f;
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int q = (wave * 2 + i) * 32 + 8 * (e / 4) + 4 * h + (e % 4);
                    const int gy = y0 + q / TW, gx = x0 + q % TW;
                    if (gy < a.H && gx < a.W) {
                        const size_t o = ((size_t)gy * a.W + gx) * a.K + k;
                        float v = acc[i][j][e] + bv;
                        if (a.relu) v = v > 0.f ? v : 0.f;
                        if (a.out_mask && !(a.out_mask[(size_t)n * a.H * a.W * a.K + o] > 0.f)) v = 0.f;
                        yn[o] = v;
                    }
                }
        }
    }
}

// Epilogue of the few-channel forward kernels: the 2 x 2 accumulator tiles of a wave (32 pixels x 32
// channels each) to y.  Accumulator element e of tile i is pixel q = (wave*2 + i)*32 + 8*(e/4) + 4h + e%4 of
// the block's TH x TW pixels (h = lane / 32), row q / TW, column q % TW (the column part 4h + e%4 < 8 never
// carries into the row), channel j*32 + lane % 32.  The upper half of the j = 0 register is exchanged with
// the lower half of the j = 1 register (one v_permlane32_swap), after which a register holds all 64
// channels of one pixel: every store instruction writes one 256-byte run, and the pixel (h = 0 or 1) is the
// same for the whole wave, so its row and column go into a scalar offset -- or, when the channel count is
// a compile-time constant (KT != 0), the column into the instruction's offset field.  Channels outside
// the tensor get an offset beyond the buffer, which drops the store; pixels outside the image are skipped
// (wave-uniform); FULL = the tile lies inside the image, no per-pixel test.
template <int TW, int KT, bool FULL>
__device__ __forceinline__ void smallc_store_tile(const float16_t (&acc)[2][2], const __amdgpu_buffer_rsrc_t yr,
                                                  float bias_lane, int y0, int x0, int k0, int H, int W,
                                                  int K_rt, bool relu, int wave, int lane) {
    static_assert(TW == 8 || TW == 16 || TW == 32, "tile widths the pixel mapping assumes");
    const int K = KT ? KT : K_rt;
    const int rows_left = H - y0 - wave * (64 / TW);                   // wave-uniform
    const int cols_left = W - x0;
    const int k = k0 + lane;                                           // after the exchange: 64 channels a pixel
    const uint32_t lane_off = k < K ? (uint32_t)((y0 * W + x0) * K + k) * 4 : 0x80000000u;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            // (copies first: a bit cast applied to a vector element expression reads the vector's first element)
            const float lo = acc[i][0][e], hi = acc[i][1][e];
            const auto sw = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, lo),
                                                             __builtin_bit_cast(uint32_t, hi), false, false);
            const int qq = i * 32 + 8 * (e / 4) + (e % 4);
            const int r_rel = qq / TW;                               // compile-time
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {                         // the pixels of the two lane halves
                const int c_rel = qq % TW + 4 * hh;                  // compile-time
                if (!FULL && !(r_rel < rows_left && c_rel < cols_left)) continue;
                const uint32_t bits = sw[hh];                        // (a copy first, as above)
                float v = __builtin_bit_cast(float, bits) + bias_lane;
                if (relu) v = v > 0.f ? v : 0.f;
                if (KT) {
                    const int soff = (wave * (64 / TW) + r_rel) * W * (KT * 4);
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), yr,
                                                          lane_off + c_rel * (KT * 4), soff, 0);
                } else {
                    const int soff = ((wave * (64 / TW) + r_rel) * W + c_rel) * (K * 4);
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), yr, lane_off, soff, 0);
                }
            }
        }
}

// Forward for very few input channels (9*C <= 32: the first VGG layer, C = 3).  The whole
// reduction (9 taps x C) fits one 32-wide k range, so instead of padding C to 8 per tap the
// (tap, channel) pairs are packed densely: 16 MFMA k-steps per tile instead of 36.  The A
// operand is gathered straight from the halo tile with per-lane offsets.  The kernel writes 64 output
// values per input value, and its 64 MFMAs per wave are few: everything else a wave executes (index
// arithmetic, bounds checks, address formation) has to stay well below them, hence C as a template
// parameter (CT = 0: any C, divisions at run time), halo rows loaded as contiguous runs, and stores
// whose row and column offsets are scalar.
template <int TH, int TW, int CT>
__global__ __launch_bounds__(CONV_THREADS, 2) void conv3x3_fwd_smallc_kernel(const ConvArgs a) {
    static_assert(TH * TW == 256, "a block owns 256 pixels");
    static_assert(TW == 8 || TW == 16 || TW == 32, "tile widths the pixel mapping of the epilogue assumes");
    constexpr int HW_ = TW + 2;
    constexpr int HALO = (TH + 2) * (TW + 2);
    constexpr int WP = 36;   // filter row pitch (32 k + 4)
    __shared__ float in_tile[HALO * 4 + 4];
    __shared__ __attribute__((aligned(16))) float w_tile[BN * WP];

    const int tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int idx = lane % 32, h = lane / 32;
    const int C = CT ? CT : a.C, NC = 9 * C;

    const int xcd = blockIdx.x % N_XCD, seq = blockIdx.x / N_XCD;
    int b = xcd * a.tiles_per_xcd + seq / a.k_blocks;
    if (b >= a.n_tiles) return;
    const int k0 = (seq % a.k_blocks) * BN;
    const int tx = b % a.tiles_x;
    b /= a.tiles_x;
    const int ty = b % a.tiles_y;
    const int n = b / a.tiles_y;
    const int y0 = ty * TH, x0 = tx * TW;

    // Stage the halo tile ([pixel][4], zero padded) and the filter ([k][9C -> 32]); all global loads are
    // issued before the first LDS store, so a block waits for memory once.  A halo row is one contiguous
    // run of (TW + 2) * C floats and the filter block one run of 64 * 9C floats: buffer loads with
    // out-of-range offsets supply the zero padding.
    constexpr int ROW_MAX = HW_ * (CT ? CT : 3);              // floats per halo row (9C <= 32: C <= 3)
    constexpr int IN_ITERS = ((TH + 2) * ROW_MAX + CONV_THREADS - 1) / CONV_THREADS;
    constexpr int W_ITERS = (BN * 9 * (CT ? CT : 3) + CONV_THREADS - 1) / CONV_THREADS;
    const int row_len = HW_ * C;
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.x + (size_t)n * a.H * a.W * C), 0, (uint32_t)a.H * a.W * C * 4, 0x00020000);
    const int kn = a.K - k0 < BN ? a.K - k0 : BN;             // filters of this block
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.w + (size_t)k0 * NC), 0, (uint32_t)kn * NC * 4, 0x00020000);
    float rin[IN_ITERS], rw[W_ITERS];
#pragma unroll
    for (int it = 0; it < IN_ITERS; ++it) {
        const int id = tid + it * CONV_THREADS;
        const int r = id / row_len, col = id - r * row_len;  // halo row, float within the row
        const int gy = y0 + r - 1, gxc = (x0 - 1) * C + col;  // image row, float within the image row
        const bool ok = r < TH + 2 && gy >= 0 && gy < a.H && gxc >= 0 && gxc < a.W * C;
        rin[it] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                xr, ok ? (uint32_t)(gy * a.W * C + gxc) * 4 : 0x80000000u, 0, 0));
    }
#pragma unroll
    for (int it = 0; it < W_ITERS; ++it)
        rw[it] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                               wr, (uint32_t)(tid + it * CONV_THREADS) * 4, 0, 0));
    // the pad lanes of the two tiles (channel 3 of every pixel, reduction indices 9C..31) are zeroed first
    for (int id = tid; id < HALO + 1; id += CONV_THREADS) in_tile[id * 4 + 3] = 0.f;
    if (C < 3)
        for (int id = tid; id < HALO; id += CONV_THREADS) in_tile[id * 4 + 2] = 0.f;
    if (C < 2)
        for (int id = tid; id < HALO; id += CONV_THREADS) in_tile[id * 4 + 1] = 0.f;
    if (tid < 3) in_tile[HALO * 4 + tid] = 0.f;
    for (int id = tid; id < BN * (32 - NC); id += CONV_THREADS) {
        const int k = id / (32 - NC);
        w_tile[k * WP + NC + (id - k * (32 - NC))] = 0.f;
    }
#pragma unroll
    for (int it = 0; it < IN_ITERS; ++it) {
        const int id = tid + it * CONV_THREADS;
        const int r = id / row_len, col = id - r * row_len;
        const int px = col / C, cc = col - px * C;
        if (r < TH + 2) in_tile[(r * HW_ + px) * 4 + cc] = rin[it];
    }
#pragma unroll
    for (int it = 0; it < W_ITERS; ++it) {
        const int id = tid + it * CONV_THREADS;
        const int k = id / NC;
        if (k < BN) w_tile[k * WP + (id - k * NC)] = rw[it];
    }
    // per-lane gather offsets for the reduction indices kk = 8g + 4h + s (two candidates per (g, s), known
    // at compile time when C is)
    int goff[4][4];
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            auto off_of = [&](int kk) {
                const int tap = kk / C, c = kk % C;
                return kk < NC ? ((tap / 3) * HW_ + (tap % 3)) * 4 + c : -1;
            };
            goff[g][s] = h ? off_of(8 * g + 4 + s) : off_of(8 * g + s);
        }
    __syncthreads();

    float16_t acc[2][2];
    int pbase[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int q = (wave * 2 + i) * 32 + idx;
        pbase[i] = ((q / TW) * HW_ + (q % TW)) * 4;
    }
    const float16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        float4_t fb[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[j] = *(const float4_t*)(w_tile + (j * 32 + idx) * WP + 8 * g + 4 * h);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            float fa[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) fa[i] = in_tile[goff[g][s] >= 0 ? pbase[i] + goff[g][s] : HALO * 4];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j][s],
                                                                     (g == 0 && s == 0) ? zero16 : acc[i][j], 0, 0, 0);
        }
    }

    const uint32_t img_bytes = (uint32_t)a.H * a.W * a.K * 4;
    const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.y + (size_t)n * a.H * a.W * a.K), 0, img_bytes, 0x00020000);
    const float bv = (a.bias && k0 + lane < a.K) ? a.bias[k0 + lane] : 0.f;
    if (y0 + TH <= a.H && x0 + TW <= a.W)           // block-uniform
        smallc_store_tile<TW, 0, true>(acc, yr, bv, y0, x0, k0, a.H, a.W, a.K, a.relu, wave, lane);
    else
        smallc_store_tile<TW, 0, false>(acc, yr, bv, y0, x0, k0, a.H, a.W, a.K, a.relu, wave, lane);
}

// The same kernel for a layer with a single block of output channels (K <= 64), as a persistent loop: a
// block keeps the filter in LDS, walks over pixel tiles of its die's range and requests tile t+1's halo
// rows before it multiplies and stores tile t, so that neither the load latency nor the draining of the
// stores sits between two tiles' MFMAs (the loads are older than the stores, so waiting for them leaves
// the stores in flight).  One barrier per tile: the halo tile is double-buffered.
template <int TH, int TW, int CT>
__global__ __launch_bounds__(CONV_THREADS, 4) void conv3x3_fwd_smallc_persist_kernel(const ConvArgs a) {
    constexpr int KT = BN;          // exactly one full block of output channels: column offsets of the
                                    // stores become instruction immediates
    static_assert(TH * TW == 256, "a block owns 256 pixels");
    static_assert(TW == 8 || TW == 16 || TW == 32, "tile widths the pixel mapping of the epilogue assumes");
    constexpr int HW_ = TW + 2;
    constexpr int HALO = (TH + 2) * (TW + 2);
    constexpr int WP = 36;
    constexpr int IN_STAGE = HALO * 4 + 4;
    __shared__ float in_tile[2 * IN_STAGE];
    __shared__ __attribute__((aligned(16))) float w_tile[BN * WP];

    const int tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int idx = lane % 32, h = lane / 32;
    const int C = CT ? CT : a.C, NC = 9 * C;

    // tiles xcd * tiles_per_xcd + slot + i * slots of die xcd = blockIdx.x % 8
    const int xcd = blockIdx.x % N_XCD, slot = blockIdx.x / N_XCD, slots = gridDim.x / N_XCD;
    int t_lim = a.n_tiles - xcd * a.tiles_per_xcd;
    t_lim = t_lim < a.tiles_per_xcd ? t_lim : a.tiles_per_xcd;
    if (slot >= t_lim) return;                                   // whole block, before any barrier
    const int tile0 = xcd * a.tiles_per_xcd + slot;
    const int n_my = (t_lim - slot + slots - 1) / slots;

    constexpr int ROW_MAX = HW_ * (CT ? CT : 3);
    constexpr int IN_ITERS = ((TH + 2) * ROW_MAX + CONV_THREADS - 1) / CONV_THREADS;
    constexpr int W_ITERS = (BN * 9 * (CT ? CT : 3) + CONV_THREADS - 1) / CONV_THREADS;
    const int row_len = HW_ * C;
    // loader roles, fixed for the whole kernel: halo row r, float col of that row
    int in_row[IN_ITERS], in_col[IN_ITERS], in_lds[IN_ITERS];
#pragma unroll
    for (int it = 0; it < IN_ITERS; ++it) {
        const int id = tid + it * CONV_THREADS;
        const int r = id / row_len, col = id - r * row_len;
        const int px = col / C, cc = col - px * C;
        in_row[it] = r < TH + 2 ? r : (1 << 30);
        in_col[it] = col;
        in_lds[it] = r < TH + 2 ? (r * HW_ + px) * 4 + cc : -1;
    }
    const uint32_t x_img_bytes = (uint32_t)a.H * a.W * C * 4;
    float rin[IN_ITERS];
    struct Pos { int n, y0, x0; };
    auto decode = [&](int tile) {
        Pos p;
        int b = tile;
        const int tx = b % a.tiles_x;
        b /= a.tiles_x;
        p.y0 = (b % a.tiles_y) * TH;
        p.n = b / a.tiles_y;
        p.x0 = tx * TW;
        return p;
    };
    auto load_halo = [&](int tile) {
        const Pos p = decode(tile);
        const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(a.x + (size_t)p.n * a.H * a.W * C), 0, x_img_bytes, 0x00020000);
        const int xc0 = (p.x0 - 1) * C;
#pragma unroll
        for (int it = 0; it < IN_ITERS; ++it) {
            const int gy = p.y0 - 1 + in_row[it], gxc = xc0 + in_col[it];
            const bool ok = gy >= 0 && gy < a.H && gxc >= 0 && gxc < a.W * C;
            rin[it] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                    xr, ok ? (uint32_t)(gy * a.W * C + gxc) * 4 : 0x80000000u, 0, 0));
        }
    };
    auto store_halo = [&](int stage) {
#pragma unroll
        for (int it = 0; it < IN_ITERS; ++it)
            if (in_lds[it] >= 0) in_tile[stage * IN_STAGE + in_lds[it]] = rin[it];
    };

    load_halo(tile0);
    {
        // the filter block ([k][9C -> 32], zero padded), once
        const __amdgpu_buffer_rsrc_t wr =
            __builtin_amdgcn_make_buffer_rsrc((void*)a.w, 0, (uint32_t)KT * NC * 4, 0x00020000);
        float rw[W_ITERS];
#pragma unroll
        for (int it = 0; it < W_ITERS; ++it)
            rw[it] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                   wr, (uint32_t)(tid + it * CONV_THREADS) * 4, 0, 0));
        for (int id = tid; id < BN * (32 - NC); id += CONV_THREADS) {
            const int k = id / (32 - NC);
            w_tile[k * WP + NC + (id - k * (32 - NC))] = 0.f;
        }
#pragma unroll
        for (int it = 0; it < W_ITERS; ++it) {
            const int id = tid + it * CONV_THREADS;
            const int k = id / NC;
            if (k < BN) w_tile[k * WP + (id - k * NC)] = rw[it];
        }
    }
    // pad lanes of both halo stages (channels C..3 of every pixel, and the all-zero pixel behind the tile)
    for (int id = tid; id < 2 * IN_STAGE; id += CONV_THREADS) {
        const int o = id % IN_STAGE;
        if (o >= HALO * 4 || (o & 3) >= C) in_tile[id] = 0.f;
    }
    store_halo(0);

    int goff[4][4];
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            auto off_of = [&](int kk) {
                const int tap = kk / C, c = kk % C;
                return kk < NC ? ((tap / 3) * HW_ + (tap % 3)) * 4 + c : HALO * 4 - 0;
            };
            goff[g][s] = h ? off_of(8 * g + 4 + s) : off_of(8 * g + s);
        }
    // per-lane LDS offsets of the two pixels this lane feeds; unused reduction indices read the zero
    // pixel (its offset is absolute: the pixel base must not be added, hence the flag)
    int pbase[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int q = (wave * 2 + i) * 32 + idx;
        pbase[i] = ((q / TW) * HW_ + (q % TW)) * 4;
    }
    const float bv = a.bias ? a.bias[lane] : 0.f;
    const uint32_t y_img_bytes = (uint32_t)a.H * a.W * KT * 4;
    const float16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    __syncthreads();

    for (int ti = 0; ti < n_my; ++ti) {
        const int tile = tile0 + ti * slots;
        const float* cur = in_tile + (ti & 1) * IN_STAGE;
        if (ti + 1 < n_my) load_halo(tile + slots);
        float16_t acc[2][2];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float4_t fb[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) fb[j] = *(const float4_t*)(w_tile + (j * 32 + idx) * WP + 8 * g + 4 * h);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const bool used = goff[g][s] < HALO * 4;
                float fa[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) fa[i] = cur[used ? pbase[i] + goff[g][s] : HALO * 4];
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            fa[i], fb[j][s], (g == 0 && s == 0) ? zero16 : acc[i][j], 0, 0, 0);
            }
        }
        // The next tile's halo goes to LDS before this tile's stores are issued: the memory counter retires
        // in order, so waiting for those loads behind 64 fresh stores would wait for the stores to drain.
        if (ti + 1 < n_my) store_halo((ti + 1) & 1);
        const Pos p = decode(tile);
        const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(a.y + (size_t)p.n * a.H * a.W * KT), 0, y_img_bytes, 0x00020000);
        if (p.y0 + TH <= a.H && p.x0 + TW <= a.W)
            smallc_store_tile<TW, KT, true>(acc, yr, bv, p.y0, p.x0, 0, a.H, a.W, KT, a.relu, wave, lane);
        else
            smallc_store_tile<TW, KT, false>(acc, yr, bv, p.y0, p.x0, 0, a.H, a.W, KT, a.relu, wave, lane);
        __syncthreads();
    }
}

// w[K][3][3][C]  ->  out[C][3][3][K] with out[c][r][s][k] = w[k][2-r][2-s][c].
__global__ __launch_bounds__(256) void filter_rot180_kernel(const float* __restrict__ w, float* __restrict__ out,
                                                            int K, int C) {
    const int total = K * 9 * C;
    const int id = blockIdx.x * 256 + threadIdx.x;
    if (id >= total) return;
    const int k = id % K;
    const int tap = (id / K) % 9;
    const int c = id / (9 * K);
    out[id] = w[((size_t)k * 9 + (8 - tap)) * C + c];
}

// ------------------------------------------------------------------------------------------
// Weight gradient
// ------------------------------------------------------------------------------------------
struct WgradArgs {
    const float* x;    // [N,H,W,C]
    const float* dy;   // [N,H,W,K]
    const float* mask; // [N,H,W,K] or null: dy is taken as 0 where mask <= 0 (fused ReLU backward)
    float* part_w;     // [gridDim.x][K][9][C]   per-block partial sums
    float* part_b;     // [gridDim.x][K]         (null: no bias gradient)
    int N, H, W, C, K;
    int tiles_x, tiles_y, n_tiles;
    int c_vec, k_vec;
};

template <int TH, int TW>
__global__ __launch_bounds__(CONV_THREADS, 2) void conv3x3_wgrad_kernel(const WgradArgs a) {
    constexpr int PIX = TH * TW;
    constexpr int HW_ = TW + 2;
    constexpr int HALO = (TH + 2) * (TW + 2);
    constexpr int CS = 64;  // channels per LDS row (both tiles)
    __shared__ __attribute__((aligned(16))) float dy_tile[PIX * CS];
    __shared__ __attribute__((aligned(16))) float x_tile[HALO * CS];

    const int tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int idx = lane % 32, h = lane / 32;
    const int kt = wave / 2, ct = wave % 2;
    const int k0 = blockIdx.y * 64, c0 = blockIdx.z * 64;
    // this wave's 32 in-channels hold nothing when C is small: skip its MFMAs
    const bool wave_active = (c0 + ct * 32) < a.C && (k0 + kt * 32) < a.K;

    float16_t acc[9];
#pragma unroll
    for (int t = 0; t < 9; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;
    float bsum = 0.f;

    for (int tile = blockIdx.x; tile < a.n_tiles; tile += gridDim.x) {
        int b = tile;
        const int tx = b % a.tiles_x;
        b /= a.tiles_x;
        const int ty = b % a.tiles_y;
        const int n = b / a.tiles_y;
        const int y0 = ty * TH, x0 = tx * TW;
        const float* xn = a.x + (size_t)n * a.H * a.W * a.C;
        const float* dyn = a.dy + (size_t)n * a.H * a.W * a.K;

        // The tile's global loads are issued in two batches (dY + first part of X, then the
        // rest of X): fixed trip counts and selects instead of branches, so a thread has
        // 8-12 128-bit loads in flight at a time without outgrowing the register file
        // next to the 144 accumulators.
        constexpr int DY_ITERS = (PIX * (CS / 4) + CONV_THREADS - 1) / CONV_THREADS;
        constexpr int X_ITERS = (HALO * (CS / 4) + CONV_THREADS - 1) / CONV_THREADS;
        constexpr int X_SPLIT = X_ITERS / 3;
        const float4_t zero = {0.f, 0.f, 0.f, 0.f};
        auto load_x = [&](int it) -> float4_t {
            const int id = tid + it * CONV_THREADS;
            const int p = id / (CS / 4), q4 = (id % (CS / 4)) * 4;
            const int gy = y0 + p / HW_ - 1, gx = x0 + p % HW_ - 1;
            const int c = c0 + q4;
            const bool ok = id < HALO * (CS / 4) && gy >= 0 && gy < a.H && gx >= 0 && gx < a.W && c < a.C;
            const float* src = ok ? xn + ((size_t)gy * a.W + gx) * a.C + c : xn;
            float4_t v;
            if (a.c_vec) {
                v = *(const float4_t*)src;
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = (ok && c + j < a.C) ? src[j] : 0.f;
            }
            return ok ? v : zero;
        };
        auto store_x = [&](int it, float4_t v) {
            const int id = tid + it * CONV_THREADS;
            if (id < HALO * (CS / 4)) *(float4_t*)(x_tile + (id / (CS / 4)) * CS + (id % (CS / 4)) * 4) = v;
        };
        {
            float4_t rdy[DY_ITERS], rx[X_SPLIT];
#pragma unroll
            for (int it = 0; it < DY_ITERS; ++it) {
                const int id = tid + it * CONV_THREADS;
                const int p = id / (CS / 4), q4 = (id % (CS / 4)) * 4;
                const int gy = y0 + p / TW, gx = x0 + p % TW;
                const int k = k0 + q4;
                const bool ok = id < PIX * (CS / 4) && gy < a.H && gx < a.W && k < a.K;
                const size_t off = ok ? ((size_t)gy * a.W + gx) * a.K + k : 0;
                const float* src = dyn + off;
                float4_t v;
                if (a.k_vec) {
                    v = *(const float4_t*)src;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = (ok && k + j < a.K) ? src[j] : 0.f;
                }
                if (a.mask) {
                    const float* msrc = a.mask + (size_t)n * a.H * a.W * a.K + off;
                    float4_t m;
                    if (a.k_vec) {
                        m = *(const float4_t*)msrc;
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j) m[j] = (ok && k + j < a.K) ? msrc[j] : 0.f;
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = m[j] > 0.f ? v[j] : 0.f;
                }
                rdy[it] = ok ? v : zero;
            }
#pragma unroll
            for (int it = 0; it < X_SPLIT; ++it) rx[it] = load_x(it);
            __syncthreads();  // everyone is done reading the previous tile
#pragma unroll
            for (int it = 0; it < DY_ITERS; ++it) {
                const int id = tid + it * CONV_THREADS;
                if (id < PIX * (CS / 4))
                    *(float4_t*)(dy_tile + (id / (CS / 4)) * CS + (id % (CS / 4)) * 4) = rdy[it];
            }
#pragma unroll
            for (int it = 0; it < X_SPLIT; ++it) store_x(it, rx[it]);
        }
        {
            float4_t rx[X_ITERS - X_SPLIT];
#pragma unroll
            for (int it = X_SPLIT; it < X_ITERS; ++it) rx[it - X_SPLIT] = load_x(it);
#pragma unroll
            for (int it = X_SPLIT; it < X_ITERS; ++it) store_x(it, rx[it - X_SPLIT]);
        }
        __syncthreads();
        if (wave_active) {
            // reduction over the tile's pixels, two per MFMA: lane-half h takes pixel 2*pp + h
#pragma unroll 2
            for (int pp = 0; pp < PIX / 2; ++pp) {
                const int p = 2 * pp + h;
                const float av = dy_tile[p * CS + kt * 32 + idx];
                bsum += av;
                const int xb = ((p / TW) * HW_ + (p % TW)) * CS + ct * 32 + idx;
#pragma unroll
                for (int t = 0; t < 9; ++t) {
                    const float bv = x_tile[xb + ((t / 3) * HW_ + (t % 3)) * CS];
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[t], 0, 0, 0);
                }
            }
        }
    }

    // partial dW[k][tap][c]: accumulator element e of lane (idx,h) is row k = 8*(e/4)+4h+e%4, col c = idx
    float* pw = a.part_w + (size_t)blockIdx.x * a.K * 9 * a.C;
    const int c = c0 + ct * 32 + idx;
    if (wave_active && c < a.C) {
#pragma unroll
        for (int t = 0; t < 9; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int k = k0 + kt * 32 + 8 * (e / 4) + 4 * h + (e % 4);
                if (k < a.K) pw[((size_t)k * 9 + t) * a.C + c] = acc[t][e];
            }
    }
    if (a.part_b && blockIdx.z == 0 && ct == 0) {
        // the two lane halves summed alternate pixels of the same out channel
        const float other = __shfl_xor(bsum, 32, 64);
        const int k = k0 + kt * 32 + idx;
        if (h == 0 && k < a.K) a.part_b[(size_t)blockIdx.x * a.K + k] = bsum + other;
    }
}

// Weight gradient, pipelined variant (C and K multiples of 4, 16-byte aligned tensors): one block
// of 8 waves per CU.  A tile's global loads (dY, the ReLU mask, the X halo: 14 128-bit loads per
// thread) stay in registers while the previous tile is multiplied, and both LDS tiles are
// double-buffered: the registers are written to the other buffer in the middle of the multiply
// phase, leaving one barrier per tile and no phase in which the matrix pipe waits for memory.
// The zero fill and the mask are applied when the registers go to LDS.  Waves 0-3 reduce the
// first half of a tile's pixels, waves 4-7 the second half (two waves per SIMD: a single wave
// cannot issue MFMAs back to back at the full rate), each into its own partial sum.
constexpr int WGP_THREADS = 512;

template <int TH, int TW, bool MASKED>
struct WgradStage {
    static constexpr int PIX = TH * TW, HW_ = TW + 2, HALO = (TH + 2) * (TW + 2), CS = 64;
    static constexpr int DY_ITERS = (PIX * (CS / 4) + WGP_THREADS - 1) / WGP_THREADS;
    static constexpr int X_ITERS = (HALO * (CS / 4) + WGP_THREADS - 1) / WGP_THREADS;
    float4_t rdy[DY_ITERS], rm[MASKED ? DY_ITERS : 1], rx[X_ITERS];
    uint32_t ok_dy, ok_x;

    __device__ __forceinline__ void load(const WgradArgs& a, int tile, int k0, int c0, int tid) {
        int b = tile;
        const int tx = b % a.tiles_x;
        b /= a.tiles_x;
        const int ty = b % a.tiles_y;
        const int n = b / a.tiles_y;
        const int y0 = ty * TH, x0 = tx * TW;
        const float* xn = a.x + (size_t)n * a.H * a.W * a.C;
        const float* dyn = a.dy + (size_t)n * a.H * a.W * a.K;
        const float* mn = MASKED ? a.mask + (size_t)n * a.H * a.W * a.K : dyn;
        ok_dy = ok_x = 0;
#pragma unroll
        for (int it = 0; it < DY_ITERS; ++it) {
            const int id = tid + it * WGP_THREADS;
            const int p = id / (CS / 4), q4 = (id % (CS / 4)) * 4;
            const int gy = y0 + p / TW, gx = x0 + p % TW;
            const int k = k0 + q4;
            const bool ok = id < PIX * (CS / 4) && gy < a.H && gx < a.W && k < a.K;
            const size_t off = ok ? ((size_t)gy * a.W + gx) * a.K + k : 0;
            rdy[it] = *(const float4_t*)(dyn + off);
            if (MASKED) rm[it] = *(const float4_t*)(mn + off);
            ok_dy |= (ok ? 1u : 0u) << it;
        }
#pragma unroll
        for (int it = 0; it < X_ITERS; ++it) {
            const int id = tid + it * WGP_THREADS;
            const int p = id / (CS / 4), q4 = (id % (CS / 4)) * 4;
            const int gy = y0 + p / HW_ - 1, gx = x0 + p % HW_ - 1;
            const int c = c0 + q4;
            const bool ok = id < HALO * (CS / 4) && gy >= 0 && gy < a.H && gx >= 0 && gx < a.W && c < a.C;
            const size_t off = ok ? ((size_t)gy * a.W + gx) * a.C + c : 0;     // a select, not a branch
            rx[it] = *(const float4_t*)(xn + off);
            ok_x |= (ok ? 1u : 0u) << it;
        }
    }

    __device__ __forceinline__ void store(float* dy_tile, float* x_tile, int tid) const {
        const float4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int it = 0; it < DY_ITERS; ++it) {
            const int id = tid + it * WGP_THREADS;
            float4_t v = rdy[it];
            if (MASKED)
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = rm[it][j] > 0.f ? v[j] : 0.f;
            if (id < PIX * (CS / 4))
                *(float4_t*)(dy_tile + (id / (CS / 4)) * CS + (id % (CS / 4)) * 4) = ((ok_dy >> it) & 1u) ? v : zero;
        }
#pragma unroll
        for (int it = 0; it < X_ITERS; ++it) {
            const int id = tid + it * WGP_THREADS;
            if (id < HALO * (CS / 4))
                *(float4_t*)(x_tile + (id / (CS / 4)) * CS + (id % (CS / 4)) * 4) = ((ok_x >> it) & 1u) ? rx[it] : zero;
        }
    }
};

template <int TH, int TW, bool MASKED>
__global__ __launch_bounds__(WGP_THREADS, 1) void conv3x3_wgrad_pipe_kernel(const WgradArgs a) {
    using Stage = WgradStage<TH, TW, MASKED>;
    constexpr int PIX = Stage::PIX, HW_ = Stage::HW_, HALO = Stage::HALO, CS = Stage::CS;
    constexpr int BUF = PIX * CS + HALO * CS;       // floats per buffer: dY tile, then X halo tile
    __shared__ __attribute__((aligned(16))) float lds[2 * BUF];

    const int tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int idx = lane % 32, h = lane / 32;
    const int half = wave / 4;                     // which half of the tile's pixel pairs
    const int kt = (wave % 4) / 2, ct = wave % 2;
    const int k0 = blockIdx.y * 64, c0 = blockIdx.z * 64;
    const bool wave_active = (c0 + ct * 32) < a.C && (k0 + kt * 32) < a.K;

    float16_t acc[9];
#pragma unroll
    for (int t = 0; t < 9; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;
    float bsum = 0.f;

    // reduction over pixel pairs [pp0, pp1) of the tile in `buf`: lane-half h takes pixel 2*pp + h
    auto multiply = [&](const float* buf, int pp0, int pp1) {
        const float* dy_tile = buf + kt * 32 + idx;
        const float* x_tile = buf + PIX * CS + ct * 32 + idx;
#pragma unroll 2
        for (int pp = pp0; pp < pp1; ++pp) {
            const int p = 2 * pp + h;
            const float av = dy_tile[p * CS];
            bsum += av;
            const int xb = ((p / TW) * HW_ + (p % TW)) * CS;
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                const float bv = x_tile[xb + ((t / 3) * HW_ + (t % 3)) * CS];
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[t], 0, 0, 0);
            }
        }
    };

    Stage st;
    int tile = blockIdx.x;
    int cur = 0;
    if (tile < a.n_tiles) {
        st.load(a, tile, k0, c0, tid);
        st.store(lds, lds + PIX * CS, tid);
    }
    __syncthreads();
    for (; tile < a.n_tiles; tile += gridDim.x) {
        const int next = tile + gridDim.x;
        const float* buf = lds + cur * BUF;
        float* other = lds + (cur ^ 1) * BUF;
        if (next < a.n_tiles) st.load(a, next, k0, c0, tid);
        const int pp0 = half * (PIX / 4);
        if (wave_active) multiply(buf, pp0, pp0 + PIX / 8);
        if (next < a.n_tiles) st.store(other, other + PIX * CS, tid);
        if (wave_active) multiply(buf, pp0 + PIX / 8, pp0 + PIX / 4);
        __syncthreads();    // `buf` may be overwritten, `other` is complete
        cur ^= 1;
    }

    float* pw = a.part_w + (size_t)(blockIdx.x * 2 + half) * a.K * 9 * a.C;
    const int c = c0 + ct * 32 + idx;
    if (wave_active && c < a.C) {
#pragma unroll
        for (int t = 0; t < 9; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int k = k0 + kt * 32 + 8 * (e / 4) + 4 * h + (e % 4);
                if (k < a.K) pw[((size_t)k * 9 + t) * a.C + c] = acc[t][e];
            }
    }
    if (a.part_b && blockIdx.z == 0 && ct == 0) {
        const float other = __shfl_xor(bsum, 32, 64);
        const int k = k0 + kt * 32 + idx;
        if (h == 0 && k < a.K) a.part_b[(size_t)(blockIdx.x * 2 + half) * a.K + k] = bsum + other;
    }
}

// Weight gradient for very few input channels (9*C <= 32, i.e. the first VGG layer with
// C = 3): all 9*C (tap, channel) pairs fit the 32 columns of ONE MFMA tile, so a pixel pair
// costs 2 MFMAs (two 32-row out-channel tiles) instead of 18.  The kernel is then bound by
// reading dY.  Each of the 4 waves reduces a quarter of the tile's pixels and writes its own
// partial sums ([gridDim.x * 4] partials).
template <int TH, int TW>
__global__ __launch_bounds__(CONV_THREADS, 2) void conv3x3_wgrad_smallc_kernel(const WgradArgs a) {
    constexpr int PIX = TH * TW;
    constexpr int HW_ = TW + 2;
    constexpr int HALO = (TH + 2) * (TW + 2);
    constexpr int CS = 64;
    __shared__ __attribute__((aligned(16))) float dy_tile[PIX * CS];
    __shared__ float x_tile[HALO * 4 + 4];   // [halo pixel][4], last slot stays 0 for unused columns

    const int tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int idx = lane % 32, h = lane / 32;
    const int k0 = blockIdx.y * 64;
    const int C = a.C, NC = 9 * a.C;
    // column idx of the MFMA tile = (tap, c); columns >= 9*C read the zero slot
    const int tap = idx / C, c = idx % C;
    const int col_off = idx < NC ? ((tap / 3) * HW_ + (tap % 3)) * 4 + c : -1;

    float16_t acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;
    float bsum[2] = {0.f, 0.f};
    if (tid == 0) x_tile[HALO * 4] = 0.f;

    constexpr int DY_ITERS = PIX * (CS / 4) / CONV_THREADS;
    constexpr int X_ITERS = (HALO * 4 + CONV_THREADS - 1) / CONV_THREADS;
    float4_t rdy[DY_ITERS];
    float rx[X_ITERS];
    uint32_t dy_ok = 0, x_ok = 0;              // which of them lie inside the image
    // global -> registers for one pixel tile; the loads of tile i+1 are issued before the multiply
    // loop of tile i and stay in flight over it (out-of-range elements read a safe address and are
    // zeroed when the registers are written to LDS: a select here would wait for the loads)
    auto load_tile = [&](int tile) {
        dy_ok = x_ok = 0;
        int b = tile;
        const int tx = b % a.tiles_x;
        b /= a.tiles_x;
        const int ty = b % a.tiles_y;
        const int n = b / a.tiles_y;
        const int y0 = ty * TH, x0 = tx * TW;
        const float* xn = a.x + (size_t)n * a.H * a.W * C;
        const float* dyn = a.dy + (size_t)n * a.H * a.W * a.K;
        const float* mn = a.mask ? a.mask + (size_t)n * a.H * a.W * a.K : nullptr;
#pragma unroll
        for (int it = 0; it < DY_ITERS; ++it) {
            const int id = tid + it * CONV_THREADS;
            const int p = id / (CS / 4), q4 = (id % (CS / 4)) * 4;
            const int gy = y0 + p / TW, gx = x0 + p % TW;
            const int k = k0 + q4;
            const bool ok = gy < a.H && gx < a.W && k < a.K;
            const size_t off = ok ? ((size_t)gy * a.W + gx) * a.K + k : 0;
            float4_t v;
            if (a.k_vec) {
                v = *(const float4_t*)(dyn + off);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = (ok && k + j < a.K) ? dyn[off + j] : 0.f;
            }
            if (mn) {
                float4_t m;
                if (a.k_vec) {
                    m = *(const float4_t*)(mn + off);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) m[j] = (ok && k + j < a.K) ? mn[off + j] : 0.f;
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = m[j] > 0.f ? v[j] : 0.f;
            }
            rdy[it] = v;
            dy_ok |= (uint32_t)ok << it;
        }
#pragma unroll
        for (int it = 0; it < X_ITERS; ++it) {
            const int id = tid + it * CONV_THREADS;
            const int p = id / 4, cc = id % 4;
            const int gy = y0 + p / HW_ - 1, gx = x0 + p % HW_ - 1;
            const bool ok = id < HALO * 4 && cc < C && gy >= 0 && gy < a.H && gx >= 0 && gx < a.W;
            rx[it] = xn[ok ? ((size_t)gy * a.W + gx) * C + cc : 0];
            x_ok |= (uint32_t)ok << it;
        }
    };
    if ((int)blockIdx.x < a.n_tiles) load_tile(blockIdx.x);

    for (int tile = blockIdx.x; tile < a.n_tiles; tile += gridDim.x) {
        __syncthreads();  // previous tile fully consumed
#pragma unroll
        for (int it = 0; it < DY_ITERS; ++it) {
            const int id = tid + it * CONV_THREADS;
            const float4_t zero = {0.f, 0.f, 0.f, 0.f};
            *(float4_t*)(dy_tile + (id / (CS / 4)) * CS + (id % (CS / 4)) * 4) = (dy_ok >> it) & 1 ? rdy[it] : zero;
        }
#pragma unroll
        for (int it = 0; it < X_ITERS; ++it) {
            const int id = tid + it * CONV_THREADS;
            if (id < HALO * 4) x_tile[id] = (x_ok >> it) & 1 ? rx[it] : 0.f;
        }
        __syncthreads();
        if (tile + (int)gridDim.x < a.n_tiles) load_tile(tile + gridDim.x);
        // this wave's quarter of the pixels, two per MFMA
#pragma unroll 4
        for (int pp = 0; pp < PIX / 8; ++pp) {
            const int p = wave * (PIX / 4) + 2 * pp + h;
            const float a0 = dy_tile[p * CS + idx];
            const float a1 = dy_tile[p * CS + 32 + idx];
            bsum[0] += a0;
            bsum[1] += a1;
            const float bv = x_tile[col_off >= 0 ? ((p / TW) * HW_ + (p % TW)) * 4 + col_off : HALO * 4];
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, bv, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, bv, acc[1], 0, 0, 0);
        }
    }

    // the four waves' sums (each covered a quarter of every tile's pixels) are added in wave order
    // through the now idle dy tile, so the block writes one partial instead of four
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) dy_tile[(wave * 32 + t * 16 + e) * 64 + lane] = acc[t][e];
    float* bsum_tile = dy_tile + 4 * 32 * 64;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const float tot = bsum[t] + __shfl_xor(bsum[t], 32, 64);
        if (h == 0) bsum_tile[wave * 64 + t * 32 + idx] = tot;
    }
    __syncthreads();
    float* pw = a.part_w + (size_t)blockIdx.x * a.K * NC;
#pragma unroll
    for (int it = 0; it < 32 * 64 / CONV_THREADS; ++it) {
        const int id = tid + it * CONV_THREADS;          // (t, e, lane) of an accumulator element
        const int te = id / 64, ln = id % 64;
        const float v = (dy_tile[te * 64 + ln] + dy_tile[(32 + te) * 64 + ln]) +
                        (dy_tile[(64 + te) * 64 + ln] + dy_tile[(96 + te) * 64 + ln]);
        const int t = te / 16, e = te % 16, col = ln % 32;
        const int k = k0 + t * 32 + 8 * (e / 4) + 4 * (ln / 32) + (e % 4);
        if (col < NC && k < a.K) pw[(size_t)k * NC + col] = v;
    }
    if (a.part_b && tid < 64 && k0 + tid < a.K)
        a.part_b[(size_t)blockIdx.x * a.K + k0 + tid] =
            (bsum_tile[tid] + bsum_tile[64 + tid]) + (bsum_tile[128 + tid] + bsum_tile[192 + tid]);
}

// The same few-channel weight gradient with the per-MFMA overhead removed (dY rows of whole float4, no
// ReLU mask, an image addressable with 32-bit byte offsets): the multiply loop is fully unrolled and every
// LDS address in it is a per-lane base plus a compile-time offset (lanes of unused columns point at a
// region of zeros, the lanes of column 9C at a region of ones, so that column accumulates the bias
// gradient); tiles are fetched with buffer loads whose out-of-range offsets supply the zero padding, with
// per-lane offsets computed once and the tile's position as a scalar offset.
template <int TH, int TW>
__global__ __launch_bounds__(CONV_THREADS, 2) void conv3x3_wgrad_smallc_fast_kernel(const WgradArgs a) {
    constexpr int PIX = TH * TW;
    constexpr int HW_ = TW + 2;
    constexpr int HALO = (TH + 2) * (TW + 2);
    constexpr int CS = 64;
    constexpr int WROWS = PIX / 4 / TW;                          // pixel rows per wave
    static_assert(PIX % (4 * TW) == 0 && TW % 2 == 0, "a wave owns whole pixel rows, pixels in pairs");
    constexpr int ZR = ((WROWS - 1) * HW_ + TW) * 4 + 4;        // floats a compile-time offset can reach
    __shared__ __attribute__((aligned(16))) float dy_tile[PIX * CS];
    __shared__ float x_tile[HALO * 4 + 2 * ZR];                 // [halo pixel][4], zeros, ones

    const int tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int idx = lane % 32, h = lane / 32;
    const int k0 = blockIdx.y * 64;
    const int C = a.C, NC = 9 * a.C;
    const int tap = idx / C, c = idx % C;
    const int xbase = idx < NC ? (wave * WROWS * HW_ + h) * 4 + ((tap / 3) * HW_ + (tap % 3)) * 4 + c
                               : (idx == NC ? HALO * 4 + ZR : HALO * 4);
    const int dybase = (wave * (PIX / 4) + h) * CS + idx;
    for (int i = tid; i < ZR; i += CONV_THREADS) {
        x_tile[HALO * 4 + i] = 0.f;
        x_tile[HALO * 4 + ZR + i] = 1.f;
    }

    float16_t acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;

    // loader roles, fixed for the whole kernel
    constexpr int DY_ITERS = PIX * (CS / 4) / CONV_THREADS;
    constexpr int X_ITERS = ((TH + 2) * HW_ * 3 + CONV_THREADS - 1) / CONV_THREADS;     // C <= 3
    const int row_len = HW_ * C;
    int dy_row[DY_ITERS], dy_col[DY_ITERS];
    uint32_t dy_lane[DY_ITERS];              // byte offset inside the tile's part of the image
#pragma unroll
    for (int it = 0; it < DY_ITERS; ++it) {
        const int id = tid + it * CONV_THREADS;
        const int p = id / (CS / 4), q4 = (id % (CS / 4)) * 4;
        dy_row[it] = k0 + q4 < a.K ? p / TW : (1 << 30);        // channels beyond K: never inside
        dy_col[it] = p % TW;
        dy_lane[it] = (uint32_t)(((p / TW) * a.W + p % TW) * a.K + q4) * 4;
    }
    int x_row[X_ITERS], x_col[X_ITERS], x_lds[X_ITERS], x_lane[X_ITERS];
#pragma unroll
    for (int it = 0; it < X_ITERS; ++it) {
        const int id = tid + it * CONV_THREADS;
        const int r = id / row_len, col = id - r * row_len;
        x_row[it] = r < TH + 2 ? r : (1 << 30);
        x_col[it] = col;
        x_lds[it] = r < TH + 2 ? (r * HW_ + col / C) * 4 + col % C : -1;
        x_lane[it] = (r * a.W * C + col) * 4;
    }
    const uint32_t dy_img_bytes = (uint32_t)a.H * a.W * a.K * 4, x_img_bytes = (uint32_t)a.H * a.W * C * 4;

    float4_t rdy[DY_ITERS];
    float rx[X_ITERS];
    auto load_tile = [&](int tile) {
        int b = tile;
        const int tx = b % a.tiles_x;
        b /= a.tiles_x;
        const int ty = b % a.tiles_y;
        const int n = b / a.tiles_y;
        const int y0 = ty * TH, x0 = tx * TW;
        const __amdgpu_buffer_rsrc_t dr = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(a.dy + (size_t)n * a.H * a.W * a.K), 0, dy_img_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(a.x + (size_t)n * a.H * a.W * C), 0, x_img_bytes, 0x00020000);
        const int rows_left = a.H - y0, cols_left = a.W - x0;
        const int dy_soff = ((y0 * a.W + x0) * a.K + k0) * 4;
#pragma unroll
        for (int it = 0; it < DY_ITERS; ++it) {
            const bool ok = dy_row[it] < rows_left && dy_col[it] < cols_left;
            rdy[it] = __builtin_bit_cast(
                float4_t, __builtin_amdgcn_raw_buffer_load_b128(dr, ok ? dy_lane[it] : 0x80000000u, dy_soff, 0));
        }
        // halo rows start one pixel up and left of the tile: the tile's offset may be negative, so it
        // goes into the per-lane offset
        const int x_toff = ((y0 - 1) * a.W + (x0 - 1)) * C * 4;
        const int xc0 = (x0 - 1) * C;
#pragma unroll
        for (int it = 0; it < X_ITERS; ++it) {
            const int gy = y0 - 1 + x_row[it], gxc = xc0 + x_col[it];
            const bool ok = gy >= 0 && gy < a.H && gxc >= 0 && gxc < a.W * C;
            rx[it] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                   xr, ok ? (uint32_t)(x_lane[it] + x_toff) : 0x80000000u, 0, 0));
        }
    };
    if ((int)blockIdx.x < a.n_tiles) load_tile(blockIdx.x);

    for (int tile = blockIdx.x; tile < a.n_tiles; tile += gridDim.x) {
        __syncthreads();  // previous tile fully consumed
#pragma unroll
        for (int it = 0; it < DY_ITERS; ++it) *(float4_t*)(dy_tile + (tid + it * CONV_THREADS) * 4) = rdy[it];
#pragma unroll
        for (int it = 0; it < X_ITERS; ++it)
            if (x_lds[it] >= 0) x_tile[x_lds[it]] = rx[it];
        __syncthreads();
        if (tile + (int)gridDim.x < a.n_tiles) load_tile(tile + gridDim.x);
        // this wave's quarter of the pixels, two per MFMA (pixel 2pp + h of the wave's rows)
#pragma unroll
        for (int pp = 0; pp < PIX / 8; ++pp) {
            const float a0 = dy_tile[dybase + 2 * pp * CS];
            const float a1 = dy_tile[dybase + 2 * pp * CS + 32];
            const float bv = x_tile[xbase + (((2 * pp) / TW) * HW_ + (2 * pp) % TW) * 4];
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, bv, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, bv, acc[1], 0, 0, 0);
        }
    }

    // the four waves' sums (each covered a quarter of every tile's pixels) are added in wave order
    // through the now idle dy tile, so the block writes one partial; column 9C is the bias gradient
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) dy_tile[(wave * 32 + t * 16 + e) * 64 + lane] = acc[t][e];
    __syncthreads();
    float* pw = a.part_w + (size_t)blockIdx.x * a.K * NC;
#pragma unroll
    for (int it = 0; it < 32 * 64 / CONV_THREADS; ++it) {
        const int id = tid + it * CONV_THREADS;          // (t, e, lane) of an accumulator element
        const int te = id / 64, ln = id % 64;
        const float v = (dy_tile[te * 64 + ln] + dy_tile[(32 + te) * 64 + ln]) +
                        (dy_tile[(64 + te) * 64 + ln] + dy_tile[(96 + te) * 64 + ln]);
        const int t = te / 16, e = te % 16, col = ln % 32;
        const int k = k0 + t * 32 + 8 * (e / 4) + 4 * (ln / 32) + (e % 4);
        if (col < NC && k < a.K) pw[(size_t)k * NC + col] = v;
        if (col == NC && k < a.K && a.part_b) a.part_b[(size_t)blockIdx.x * a.K + k] = v;
    }
}

// out[i] = sum_b part[b][i] in a fixed order (deterministic).  A block owns 64 outputs;
// its 4 waves each sum a quarter of the partials, then combine through LDS.
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float* __restrict__ part, float* __restrict__ out,
                                                              int n_part, int n) {
    __shared__ float red[4][64];
    const int lane = threadIdx.x % 64, w = threadIdx.x / 64;
    const int i = blockIdx.x * 64 + lane;
    // eight independent sums per lane: eight loads in flight instead of a chain of round trips (the order
    // of the additions is fixed, so the result is reproducible)
    float t[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (i < n) {
        int b = w;
        for (; b + 28 < n_part; b += 32)
#pragma unroll
            for (int u = 0; u < 8; ++u) t[u] += part[(size_t)(b + 4 * u) * n + i];
        for (; b < n_part; b += 4) t[0] += part[(size_t)b * n + i];
    }
    red[w][lane] = ((t[0] + t[1]) + (t[2] + t[3])) + ((t[4] + t[5]) + (t[6] + t[7]));
    __syncthreads();
    if (w == 0 && i < n) out[i] = (red[0][lane] + red[1][lane]) + (red[2][lane] + red[3][lane]);
}

struct TileShape {
    int th, tw;
};

// Pick the pixel tile that wastes the fewest MFMA rows on this image size.
TileShape pick_tile(int H, int W) {
    const TileShape cand[3] = {{16, 16}, {8, 32}, {32, 8}};
    TileShape best = cand[0];
    double best_eff = -1.0;
    for (const TileShape& t : cand) {
        const double th = (double)((H + t.th - 1) / t.th) * t.th;
        const double tw = (double)((W + t.tw - 1) / t.tw) * t.tw;
        const double eff = ((double)H * W) / (th * tw);
        if (eff > best_eff + 1e-9) {
            best_eff = eff;
            best = t;
        }
    }
    return best;
}

constexpr int WGRAD_TH = 8, WGRAD_TW = 16;
constexpr int WGRAD_MAX_BLOCKS = 512;

// Number of pixel-range blocks (= partial sums to reduce): with the (K/64) x (C/64) channel blocks
// about WGRAD_MAX_BLOCKS workgroups in total, i.e. two rounds of one block per CU.
int wgrad_blocks(int N, int H, int W, int C, int K) {
    const long tiles = (long)N * ((H + WGRAD_TH - 1) / WGRAD_TH) * ((W + WGRAD_TW - 1) / WGRAD_TW);
    const long pairs = 9 * C <= 32 ? (K + 63) / 64 : (long)((K + 63) / 64) * ((C + 63) / 64);
    long nb = WGRAD_MAX_BLOCKS / pairs;
    if (nb < 1) nb = 1;
    return (int)(tiles < nb ? tiles : nb);
}

int check_dims(const char* who, int N, int H, int W, int C, int K) {
    PD_REQUIRE(N > 0 && H > 0 && W > 0 && C > 0 && K > 0, PD_ESHAPE, "%s: dimensions must be positive", who);
    PD_REQUIRE((long)N * H * W * (C > K ? C : K) < (1L << 40), PD_ESHAPE, "%s: tensor too large", who);
    return PD_OK;
}

}  // namespace

static int conv3x3_fwd_launch(const float* x, const float* w, const float* bias, const float* mask,
                              const float* out_mask, float* y, int N, int H, int W, int C, int K, int relu,
                              void* stream) {
    int rc = check_dims("pd_conv3x3_fwd_nhwc_f32", N, H, W, C, K);
    if (rc != PD_OK) return rc;
    PD_REQUIRE(x && w && y, PD_EINVAL, "pd_conv3x3_fwd_nhwc_f32: NULL pointer");
    ConvArgs a;
    a.x = x; a.w = w; a.bias = bias; a.mask = mask; a.y = y; a.out_mask = out_mask;
    a.N = N; a.H = H; a.W = W; a.C = C; a.K = K;
    a.relu = relu != 0;
    a.c_vec = (C % 4 == 0) && pd_aligned(x, 16) && pd_aligned(w, 16) && (!mask || pd_aligned(mask, 16));
    a.y_vec = (K % 4 == 0) && pd_aligned(y, 16) && (!out_mask || pd_aligned(out_mask, 16));
    const TileShape t = pick_tile(H, W);
    a.tiles_x = (W + t.tw - 1) / t.tw;
    a.tiles_y = (H + t.th - 1) / t.th;
    const long ntiles = (long)N * a.tiles_x * a.tiles_y;
    a.k_blocks = (K + BN - 1) / BN;
    a.tiles_per_xcd = (int)((ntiles + N_XCD - 1) / N_XCD);
    const long nblk = (long)N_XCD * a.tiles_per_xcd * a.k_blocks;
    PD_REQUIRE(nblk <= 0x7fffffffL, PD_ESHAPE, "pd_conv3x3_fwd_nhwc_f32: too many tiles");
    a.n_tiles = (int)ntiles;
    dim3 grid((unsigned)nblk);                       // one block per (pixel tile, out-channel block)
    hipStream_t s = (hipStream_t)stream;
    const bool small_c = C <= 8;
    // the few-channel kernel addresses one image with 32-bit byte offsets
    // persistent variant: four blocks per CU, in multiples of the number of dies
    int dev = 0, cus = 0;
    PD_HIP(hipGetDevice(&dev));
    PD_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    long pblocks = 4L * (cus / N_XCD) * N_XCD;
    if (pblocks < N_XCD) pblocks = N_XCD;
    if (pblocks > (long)a.tiles_per_xcd * N_XCD) pblocks = (long)a.tiles_per_xcd * N_XCD;
    const dim3 pgrid((unsigned)pblocks);
    const bool dense_taps = 9 * C <= 32 && !mask && !out_mask && (long)H * W * (K > C ? K : C) * 4 < (1L << 31);
#define PD_LAUNCH_FWD(TH_, TW_)                                                                        \
    do {                                                                                               \
        if (dense_taps && K == BN && C == 3)                                                            \
            conv3x3_fwd_smallc_persist_kernel<TH_, TW_, 3><<<pgrid, CONV_THREADS, 0, s>>>(a);          \
        else if (dense_taps && C == 3) conv3x3_fwd_smallc_kernel<TH_, TW_, 3><<<grid, CONV_THREADS, 0, s>>>(a);  \
        else if (dense_taps) conv3x3_fwd_smallc_kernel<TH_, TW_, 0><<<grid, CONV_THREADS, 0, s>>>(a);       \
        else if (!a.c_vec && mask) conv3x3_fwd_kernel<TH_, TW_, 8, true, false><<<grid, CONV_THREADS, 0, s>>>(a); \
        else if (!a.c_vec) conv3x3_fwd_kernel<TH_, TW_, 8, false, false><<<grid, CONV_THREADS, 0, s>>>(a);  \
        else if (small_c && mask) conv3x3_fwd_kernel<TH_, TW_, 8, true, true><<<grid, CONV_THREADS, 0, s>>>(a); \
        else if (small_c) conv3x3_fwd_kernel<TH_, TW_, 8, false, true><<<grid, CONV_THREADS, 0, s>>>(a); \
        else if (mask) conv3x3_fwd_kernel<TH_, TW_, 16, true, true><<<grid, CONV_THREADS, 0, s>>>(a);  \
        else conv3x3_fwd_kernel<TH_, TW_, 16, false, true><<<grid, CONV_THREADS, 0, s>>>(a);           \
    } while (0)
    if (t.tw == 16) PD_LAUNCH_FWD(16, 16);
    else if (t.tw == 32) PD_LAUNCH_FWD(8, 32);
    else PD_LAUNCH_FWD(32, 8);
#undef PD_LAUNCH_FWD
    PD_CHECK_LAUNCH("pd_conv3x3_fwd_nhwc_f32");
    return PD_OK;
}

extern "C" int pd_conv3x3_fwd_nhwc_f32(const float* x, const float* w, const float* bias, float* y, int N, int H,
                                       int W, int C, int K, int relu, void* stream) {
    return conv3x3_fwd_launch(x, w, bias, nullptr, nullptr, y, N, H, W, C, K, relu, stream);
}

extern "C" int pd_conv3x3_dgrad_nhwc_f32(const float* dy, const float* w_rot, const float* relu_out,
                                         const float* x_rectified, float* dx, int N, int H, int W, int K, int C,
                                         void* stream) {
    // the forward kernel with the roles of the channel counts swapped: input = dy (K channels),
    // filter = rot180(w) [C][3][3][K], output = dx (C channels)
    return conv3x3_fwd_launch(dy, w_rot, nullptr, relu_out, x_rectified, dx, N, H, W, K, C, 0, stream);
}

extern "C" int pd_conv3x3_filter_rot180_f32(const float* w, float* out, int K, int C, void* stream) {
    PD_REQUIRE(K > 0 && C > 0, PD_ESHAPE, "pd_conv3x3_filter_rot180_f32: dimensions must be positive");
    PD_REQUIRE(w && out && w != out, PD_EINVAL, "pd_conv3x3_filter_rot180_f32: NULL or aliased pointer");
    const int total = K * 9 * C;
    filter_rot180_kernel<<<dim3((total + 255) / 256), dim3(256), 0, (hipStream_t)stream>>>(w, out, K, C);
    PD_CHECK_LAUNCH("pd_conv3x3_filter_rot180_f32");
    return PD_OK;
}

extern "C" int pd_conv3x3_wgrad_workspace_bytes(int N, int H, int W, int C, int K, uint64_t* bytes) {
    int rc = check_dims("pd_conv3x3_wgrad_workspace_bytes", N, H, W, C, K);
    if (rc != PD_OK) return rc;
    PD_REQUIRE(bytes != nullptr, PD_EINVAL, "pd_conv3x3_wgrad_workspace_bytes: NULL pointer");
    // partial sums per pixel-range block: 1 in the few-channel kernel, 2 in the pipelined one
    const uint64_t nb = (uint64_t)wgrad_blocks(N, H, W, C, K) * (9 * C <= 32 ? 1 : 2);
    *bytes = nb * ((uint64_t)K * 9 * C + (uint64_t)K) * sizeof(float);
    return PD_OK;
}

// The launches behind both weight-gradient entry points; ``workspace`` holds at least
// pd_conv3x3_wgrad_workspace_bytes() bytes, every one of which the first launch writes before the
// reduction reads it (nothing has to be cleared).
static int wgrad_launch(const float* x, const float* dy, const float* relu_out, float* dw, float* dbias,
                        void* workspace, int N, int H, int W, int C, int K, void* stream) {
    WgradArgs a;
    a.x = x; a.dy = dy; a.mask = relu_out;
    a.N = N; a.H = H; a.W = W; a.C = C; a.K = K;
    a.tiles_x = (W + WGRAD_TW - 1) / WGRAD_TW;
    a.tiles_y = (H + WGRAD_TH - 1) / WGRAD_TH;
    a.n_tiles = N * a.tiles_x * a.tiles_y;
    const bool small_c = 9 * C <= 32;
    const int nblk = wgrad_blocks(N, H, W, C, K);
    const bool vec = (C % 4 == 0) && pd_aligned(x, 16) && (K % 4 == 0) && pd_aligned(dy, 16) && (!relu_out || pd_aligned(relu_out, 16));
    const int nb = nblk * (small_c ? 1 : (vec ? 2 : 1));     // number of partial sums
    a.part_w = (float*)workspace;
    a.part_b = dbias ? a.part_w + (size_t)nb * K * 9 * C : nullptr;
    a.c_vec = (C % 4 == 0) && pd_aligned(x, 16);
    a.k_vec = (K % 4 == 0) && pd_aligned(dy, 16) && (!relu_out || pd_aligned(relu_out, 16));
    hipStream_t s = (hipStream_t)stream;
    if (small_c) {
        dim3 grid(nblk, (K + 63) / 64);
        // the lean kernel: whole float4 of dY, no ReLU mask, 32-bit byte offsets inside one image
        if (a.k_vec && !relu_out && (long)H * W * (K > C ? K : C) * 4 < (1L << 31))
            conv3x3_wgrad_smallc_fast_kernel<WGRAD_TH, WGRAD_TW><<<grid, CONV_THREADS, 0, s>>>(a);
        else
            conv3x3_wgrad_smallc_kernel<WGRAD_TH, WGRAD_TW><<<grid, CONV_THREADS, 0, s>>>(a);
    } else {
        dim3 grid(nblk, (K + 63) / 64, (C + 63) / 64);
        if (a.c_vec && a.k_vec && relu_out) conv3x3_wgrad_pipe_kernel<WGRAD_TH, WGRAD_TW, true><<<grid, WGP_THREADS, 0, s>>>(a);
        else if (a.c_vec && a.k_vec) conv3x3_wgrad_pipe_kernel<WGRAD_TH, WGRAD_TW, false><<<grid, WGP_THREADS, 0, s>>>(a);
        else conv3x3_wgrad_kernel<WGRAD_TH, WGRAD_TW><<<grid, CONV_THREADS, 0, s>>>(a);
    }
    PD_CHECK_LAUNCH("pd_conv3x3_wgrad_nhwc_f32");
    const int nw = K * 9 * C;
    reduce_partials_kernel<<<dim3((nw + 63) / 64), dim3(256), 0, s>>>(a.part_w, dw, nb, nw);
    PD_CHECK_LAUNCH("pd_conv3x3_wgrad_nhwc_f32(reduce)");
    if (dbias) {
        reduce_partials_kernel<<<dim3((K + 63) / 64), dim3(256), 0, s>>>(a.part_b, dbias, nb, K);
        PD_CHECK_LAUNCH("pd_conv3x3_wgrad_nhwc_f32(reduce bias)");
    }
    return PD_OK;
}

extern "C" int pd_conv3x3_wgrad_nhwc_f32(const float* x, const float* dy, const float* relu_out, float* dw,
                                         float* dbias, void* workspace, uint64_t workspace_bytes, int N, int H, int W,
                                         int C, int K, void* stream) {
    int rc = check_dims("pd_conv3x3_wgrad_nhwc_f32", N, H, W, C, K);
    if (rc != PD_OK) return rc;
    PD_REQUIRE(x && dy && dw && workspace, PD_EINVAL, "pd_conv3x3_wgrad_nhwc_f32: NULL pointer");
    uint64_t need = 0;
    pd_conv3x3_wgrad_workspace_bytes(N, H, W, C, K, &need);
    PD_REQUIRE(workspace_bytes >= need, PD_EINVAL, "pd_conv3x3_wgrad_nhwc_f32: workspace too small (%llu < %llu)",
               (unsigned long long)workspace_bytes, (unsigned long long)need);
    PD_REQUIRE(pd_aligned(workspace, 16), PD_EINVAL, "pd_conv3x3_wgrad_nhwc_f32: workspace must be 16-byte aligned");
    return wgrad_launch(x, dy, relu_out, dw, dbias, workspace, N, H, W, C, K, stream);
}

// ---- the same weight gradient for callers that cannot allocate ----------------------------------------
// The partial sums go to a fixed array in device memory instead of a caller's workspace.  Each GPU the
// library runs on holds its own copy of the array, at its own address, until the process ends.  In host
// code the array's name is only a handle for hipGetSymbolAddress; the address it returns for the current
// device is what kernels and copies get.
constexpr uint64_t WGRAD_SCRATCH_BYTES = PD_CONV3X3_WGRAD_NOALLOC_MAX_WORKSPACE;
static __device__ __align__(256) unsigned char scratch[WGRAD_SCRATCH_BYTES];

constexpr int WGRAD_SCRATCH_MAX_DEVICES = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[WGRAD_SCRATCH_MAX_DEVICES];   // per device, filled on the first call there

static int scratch_of_current_device(const char* who, void** out) {
    int dev = -1;
    PD_HIP(hipGetDevice(&dev));
    PD_REQUIRE(dev >= 0 && dev < WGRAD_SCRATCH_MAX_DEVICES, PD_EINVAL, "%s: device ordinal %d not supported", who, dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        PD_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        PD_REQUIRE(p != nullptr && pd_aligned(p, 256), PD_EINVAL, "%s: no device address for the scratch array", who);
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return PD_OK;
}

extern "C" int pd_conv3x3_wgrad_noalloc_nhwc_f32(const float* x, const float* dy, const float* relu_out, float* dw,
                                                 float* dbias, int N, int H, int W, int C, int K, void* stream) {
    const char* who = "pd_conv3x3_wgrad_noalloc_nhwc_f32";
    int rc = check_dims(who, N, H, W, C, K);
    if (rc != PD_OK) return rc;
    PD_REQUIRE(x && dy && dw, PD_EINVAL, "%s: NULL pointer", who);
    uint64_t need = 0;
    pd_conv3x3_wgrad_workspace_bytes(N, H, W, C, K, &need);
    PD_REQUIRE(need <= WGRAD_SCRATCH_BYTES, PD_ESHAPE,
               "%s: this shape needs %llu bytes of partial sums, the built-in scratch array holds %llu; use "
               "pd_conv3x3_wgrad_nhwc_f32 with a workspace", who, (unsigned long long)need,
               (unsigned long long)WGRAD_SCRATCH_BYTES);
    void* ws = nullptr;
    rc = scratch_of_current_device(who, &ws);
    if (rc != PD_OK) return rc;
    return wgrad_launch(x, dy, relu_out, dw, dbias, ws, N, H, W, C, K, stream);
}
