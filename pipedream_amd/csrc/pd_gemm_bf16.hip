// bf16 GEMM with fp32 accumulation on the gfx950 matrix cores
// (v_mfma_f32_32x32x16_bf16), strided-batched, for the transformer stage: the
// projections (QKV, attention output, FFN), the attention products Q K^T and P V, and
// all their gradients.
//
// The reference has no such stage on this branch (PipeDream-2BW lives elsewhere,
// README.md:7-8); the kernel plays the role cuBLAS plays for torch.nn.Linear in the
// reference's stages (runtime/runtime.py:529-530, :606-608).
//
// Bound: MFMA bf16 (2.5 PFLOP/s dense).  2*M*N*K flop per batch entry.
//
// C[M,N] = op(A)[M,K] op(B)[K,N]; op(A) is stored [M][lda] (trans_a = 0, k-contiguous) or
// [K][lda] (trans_a = 1); op(B) is stored [K][ldb] (trans_b = 0) or [N][ldb]
// (trans_b = 1, k-contiguous).
//
// A block of WM x WN waves owns a BM x BN tile; K runs in chunks of 64 through a
// double-buffered LDS tile.  LDS bandwidth, not the matrix cores, limits small tiles: a
// wave with a (32*TM) x (32*TN) tile reads (TM+TN) KB of fragments per TM*TN MFMAs, so the
// large configuration gives every wave 128 x 64 and a block 256 x 256.
//   * k-contiguous operand: LDS rows [row][64 k] with a pitch of 72 bf16; one
//     conflict-free 128-bit read is one MFMA operand (8 k-values per lane).
//   * row-contiguous operand (k is the slow index in memory): the tile is copied as it
//     lies, [k][rows], with a pitch of rows+32, and the fragments are fetched with the
//     transposing LDS read of gfx950 (ds_read_b64_tr_b16): inside each group of 16 lanes,
//     input lane i supplies 4 consecutive elements and output lane j receives element
//     (j % 4) of input lanes j/4, j/4+4, j/4+8, j/4+12.  With input lane i addressing
//     [k0 + i/4][r0 + 4*(i%4)], output lane j holds row r0+j at k0..k0+3: two such reads are
//     the eight k-values of one MFMA operand, and no transposition pass is needed.
// Workgroups are numbered so that the 32 that run together on one accelerator die
// (workgroup id mod 8) cover a compact 8 x 4 patch of tiles and share operand panels in
// that die's L2.
// Epilogue: (+ bias[N] fp32) (+ residual[M][N] bf16) -> bf16, or fp32 with optional
// accumulation into C (weight gradients summed over micro-batches).
#include <type_traits>

#include "pd_internal.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int BK = 64;            // k per chunk
constexpr int KC_PITCH = BK + 8;  // LDS row pitch of a k-contiguous tile, in bf16 (144 bytes)
constexpr int N_XCD = 8;
constexpr int GROUP_M = 8;        // tile rows per ordering group

struct GemmBf16Args {
    const uint16_t* A;
    const uint16_t* B;
    void* C;
    const float* bias;          // [N] or null
    const uint16_t* residual;   // [M][ldr] bf16 or null (bf16 output only)
    int M, N, K;
    int lda, ldb, ldc, ldr;
    int batch_inner;            // batch = outer * batch_inner + inner
    long long sa_o, sa_i, sb_o, sb_i, sc_o, sc_i;   // batch strides in elements
    float alpha;
    float beta;                 // fp32 output: C = alpha*acc + beta*C
    int out_f32;
    int tiles_m, tiles_n, total_tiles, tiles_per_xcd;
    int vec_store;              // C (and residual, aux) can be written with 16-byte vectors
    // GELU in the epilogue (bf16 output): act 1 = forward, also stores aux_out = gelu(C) (C as rounded to
    // bf16, which is what the backward reads); act 2 = backward, C = value * gelu'(aux_in)
    int act;
    uint16_t* aux_out;          // [M][ld_aux]
    const uint16_t* aux_in;     // [M][ld_aux]
    int ld_aux;
};

// erf by Abramowitz & Stegun 7.1.26 (absolute error below 1.5e-7, far inside a bf16 result's rounding): a
// few multiply-adds, one reciprocal and one exponential, instead of the library erff, whose register demand
// inside the 256 x 256 kernels' epilogue (all 256 registers hold accumulators there) spilled a kilobyte per lane.
__device__ __forceinline__ float erf_as(float x) {
    const float ax = fabsf(x);
    const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * ax);
    const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
    const float r = 1.0f - poly * __expf(-ax * ax);
    return x < 0.f ? -r : r;
}
__device__ __forceinline__ float gelu_f(float x) { return 0.5f * x * (1.0f + erf_as(x * 0.70710678118654752f)); }
__device__ __forceinline__ float gelu_grad_f(float x) {
    const float cdf = 0.5f * (1.0f + erf_as(x * 0.70710678118654752f));
    const float pdf = 0.39894228040143268f * __expf(-0.5f * x * x);
    return cdf + x * pdf;
}

__device__ __forceinline__ uint16_t f2bf(float f) { return pd_f2bf(f); }
__device__ __forceinline__ float bf2f(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// Epilogue of one wave: its (32*TM) x (32*TN) accumulator tile -> C.
// An MFMA accumulator holds one column and 16 scattered rows per lane, so storing it
// directly gives 2-byte (bf16) stores in 64-byte runs.  Instead each 32-row block is
// written to a wave-private LDS region as fp32 [32][32*TN] (pitch +8 floats: the two
// half-waves, which hold rows r and r+4, then hit different banks) and read back row-wise,
// so a lane converts and stores 8 consecutive bf16 (16 bytes; or 4 fp32) and a wave writes
// whole 128-byte lines.  bias is added before staging; the residual is added (in fp32, one
// rounding) and beta*C accumulated on the vectorised side.  `vec` = N, ldc, ldr and the
// batch offsets are multiples of 8 and C / residual are 16-byte aligned; otherwise the
// element-wise path is used.
// One staged 32-row block of a wave's tile -> C, for a block that lies inside the matrix: all LDS reads first,
// then the operand loads, then the arithmetic and the 16-byte stores.  F32: fp32 output (BETA: accumulated into
// C); RES: bf16 residual added; ACT: 1 = also store gelu(C) to aux_out, 2 = multiply by gelu'(aux_in).
template <int TN, bool F32, bool BETA, bool RES, int ACT>
__device__ __forceinline__ void store_rows_full(const GemmBf16Args& a, const float* stage, int row0, int col0,
                                                long long c_off, int lane) {
    constexpr int COLS = 32 * TN, P = COLS + 8;
    if constexpr (F32) {
        constexpr int LPR = COLS / 4, ITER = 32 * LPR / 64;
        const int c4 = (lane % LPR) * 4, r_in = lane / LPR;
        float4_t v[ITER], old[ITER];
#pragma unroll
        for (int it = 0; it < ITER; ++it) v[it] = *(const float4_t*)(stage + (it * (64 / LPR) + r_in) * P + c4);
        float* const base = (float*)a.C + c_off + (long long)(row0 + r_in) * a.ldc + col0 + c4;
        if (BETA) {
#pragma unroll
            for (int it = 0; it < ITER; ++it) old[it] = *(const float4_t*)(base + (long long)it * (64 / LPR) * a.ldc);
        }
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            if (BETA) v[it] += a.beta * old[it];
            *(float4_t*)(base + (long long)it * (64 / LPR) * a.ldc) = v[it];
        }
    } else {
        constexpr int LPR = COLS / 8, ITER = 32 * LPR / 64;
        const int c8 = (lane % LPR) * 8, r_in = lane / LPR;
        float4_t v0[ITER], v1[ITER];
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            const float* src = stage + (it * (64 / LPR) + r_in) * P + c8;
            v0[it] = *(const float4_t*)src;
            v1[it] = *(const float4_t*)(src + 4);
        }
        u16x8 extra[(RES || ACT == 2) ? ITER : 1];
        if (RES) {
            const uint16_t* rb = a.residual + c_off + (long long)(row0 + r_in) * a.ldr + col0 + c8;
#pragma unroll
            for (int it = 0; it < ITER; ++it) extra[it] = *(const u16x8*)(rb + (long long)it * (64 / LPR) * a.ldr);
        }
        if (ACT == 2) {
            const uint16_t* xb = a.aux_in + (long long)(row0 + r_in) * a.ld_aux + col0 + c8;
#pragma unroll
            for (int it = 0; it < ITER; ++it) extra[it] = *(const u16x8*)(xb + (long long)it * (64 / LPR) * a.ld_aux);
        }
        uint16_t* const cb = (uint16_t*)a.C + c_off + (long long)(row0 + r_in) * a.ldc + col0 + c8;
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            float v[8] = {v0[it][0], v0[it][1], v0[it][2], v0[it][3], v1[it][0], v1[it][1], v1[it][2], v1[it][3]};
            if (RES) {
#pragma unroll
                for (int q = 0; q < 8; ++q) v[q] += bf2f(extra[it][q]);
            }
            if (ACT == 2) {
#pragma unroll
                for (int q = 0; q < 8; ++q) v[q] *= gelu_grad_f(bf2f(extra[it][q]));
            }
            u16x8 o;
#pragma unroll
            for (int q = 0; q < 8; ++q) o[q] = f2bf(v[q]);
            *(u16x8*)(cb + (long long)it * (64 / LPR) * a.ldc) = o;
            if (ACT == 1) {
                u16x8 gg;
#pragma unroll
                for (int q = 0; q < 8; ++q) gg[q] = f2bf(gelu_f(bf2f(o[q])));
                *(u16x8*)(a.aux_out + (long long)(row0 + r_in + it * (64 / LPR)) * a.ld_aux + col0 + c8) = gg;
            }
        }
    }
}

// A wave's whole tile, inside the matrix, in one output form: stage each 32-row block, then store it.
template <int TM, int TN, bool F32, bool BETA, bool RES, int ACT>
__device__ __forceinline__ void store_tile_full(const GemmBf16Args& a, float16_t (&acc)[TM][TN], const float (&bv)[TN],
                                                int m0w, int n0w, long long c_off, float* stage, int lane) {
    constexpr int P = 32 * TN + 8;
    const int idx = lane % 32, h = lane / 32;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                stage[(8 * (e / 4) + 4 * h + (e % 4)) * P + j * 32 + idx] = a.alpha * acc[i][j][e] + bv[j];
        store_rows_full<TN, F32, BETA, RES, ACT>(a, stage, m0w + i * 32, n0w, c_off, lane);
    }
}

template <int TM, int TN>
__device__ __forceinline__ void store_tile(const GemmBf16Args& a, float16_t (&acc)[TM][TN], int m0w, int n0w,
                                           long long c_off, float* stage, int lane) {
    constexpr int COLS = 32 * TN, P = COLS + 8;
    const int idx = lane % 32, h = lane / 32;
    if (!a.vec_store) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int col = n0w + j * 32 + idx;
                if (col >= a.N) continue;
                const float bv = a.bias ? a.bias[col] : 0.f;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int row = m0w + i * 32 + 8 * (e / 4) + 4 * h + (e % 4);
                    if (row >= a.M) continue;
                    float v = a.alpha * acc[i][j][e] + bv;
                    const long long off = c_off + (long long)row * a.ldc + col;
                    if (a.out_f32) {
                        float* p = (float*)a.C + off;
                        if (a.beta != 0.f) v += a.beta * *p;
                        *p = v;
                    } else {
                        if (a.residual) v += bf2f(a.residual[c_off + (long long)row * a.ldr + col]);
                        if (a.act == 2) v *= gelu_grad_f(bf2f(a.aux_in[(long long)row * a.ld_aux + col]));
                        const uint16_t o = f2bf(v);
                        ((uint16_t*)a.C)[off] = o;
                        if (a.act == 1) a.aux_out[(long long)row * a.ld_aux + col] = f2bf(gelu_f(bf2f(o)));
                    }
                }
            }
        return;
    }
    float bv[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int col = n0w + j * 32 + idx;
        bv[j] = (a.bias && col < a.N) ? a.bias[col] : 0.f;
    }
    // The wave's tile lies inside the matrix (every transformer product): one loop per output form, without a
    // test inside, so that the LDS reads, the operand loads and the stores of a 32-row block are issued in
    // batches.  (With the form and the bounds tested per 16-byte vector every read waited for its own round
    // trip: 47 000 cycles for a 128 x 128 wave tile, more than the 256 x 256 kernel's whole k loop at K = 1024.)
    if (m0w + 32 * TM <= a.M && n0w + 32 * TN <= a.N) {
        if (a.out_f32) {
            if (a.beta != 0.f) store_tile_full<TM, TN, true, true, false, 0>(a, acc, bv, m0w, n0w, c_off, stage, lane);
            else store_tile_full<TM, TN, true, false, false, 0>(a, acc, bv, m0w, n0w, c_off, stage, lane);
        } else if (a.act == 1) store_tile_full<TM, TN, false, false, false, 1>(a, acc, bv, m0w, n0w, c_off, stage, lane);
        else if (a.act == 2) store_tile_full<TM, TN, false, false, false, 2>(a, acc, bv, m0w, n0w, c_off, stage, lane);
        else if (a.residual) store_tile_full<TM, TN, false, false, true, 0>(a, acc, bv, m0w, n0w, c_off, stage, lane);
        else store_tile_full<TM, TN, false, false, false, 0>(a, acc, bv, m0w, n0w, c_off, stage, lane);
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                stage[(8 * (e / 4) + 4 * h + (e % 4)) * P + j * 32 + idx] = a.alpha * acc[i][j][e] + bv[j];
        // same wave wrote and reads: LDS operations of one wave complete in order
        if (a.out_f32) {
            constexpr int LPR = COLS / 4;          // lanes per row
            const int c4 = (lane % LPR) * 4, r_in = lane / LPR;
#pragma unroll
            for (int it = 0; it < 32 * LPR / 64; ++it) {
                const int r = it * (64 / LPR) + r_in;
                const int row = m0w + i * 32 + r, col = n0w + c4;
                float4_t v = *(const float4_t*)(stage + r * P + c4);
                if (row < a.M && col < a.N) {
                    float4_t* p = (float4_t*)((float*)a.C + c_off + (long long)row * a.ldc + col);
                    if (a.beta != 0.f) v += a.beta * *p;
                    *p = v;
                }
            }
        } else {
            constexpr int LPR = COLS / 8;
            const int c8 = (lane % LPR) * 8, r_in = lane / LPR;
#pragma unroll
            for (int it = 0; it < 32 * LPR / 64; ++it) {
                const int r = it * (64 / LPR) + r_in;
                const int row = m0w + i * 32 + r, col = n0w + c8;
                const float4_t v0 = *(const float4_t*)(stage + r * P + c8);
                const float4_t v1 = *(const float4_t*)(stage + r * P + c8 + 4);
                if (row < a.M && col < a.N) {
                    float v[8] = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
                    if (a.residual) {
                        const u16x8 rr = *(const u16x8*)(a.residual + c_off + (long long)row * a.ldr + col);
#pragma unroll
                        for (int q = 0; q < 8; ++q) v[q] += bf2f(rr[q]);
                    }
                    if (a.act == 2) {
                        const u16x8 xx = *(const u16x8*)(a.aux_in + (long long)row * a.ld_aux + col);
#pragma unroll
                        for (int q = 0; q < 8; ++q) v[q] *= gelu_grad_f(bf2f(xx[q]));
                    }
                    u16x8 o;
#pragma unroll
                    for (int q = 0; q < 8; ++q) o[q] = f2bf(v[q]);
                    *(u16x8*)((uint16_t*)a.C + c_off + (long long)row * a.ldc + col) = o;
                    if (a.act == 1) {
                        u16x8 gg;
#pragma unroll
                        for (int q = 0; q < 8; ++q) gg[q] = f2bf(gelu_f(bf2f(o[q])));
                        *(u16x8*)(a.aux_out + (long long)row * a.ld_aux + col) = gg;
                    }
                }
            }
        }
    }
}

// One operand tile of ROWS rows x 64 k, staged global -> registers -> LDS by NT threads.
// KC: memory is [row][k]; LDS keeps that order.  !KC: memory is [k][row]; LDS keeps that too.
template <int ROWS, bool KC, int NT>
struct TileH {
    static constexpr int PITCH = KC ? KC_PITCH : ROWS + 32;
    static constexpr int SIZE = KC ? ROWS * KC_PITCH : BK * (ROWS + 32);
    static constexpr int VECS = ROWS * BK / 8;            // 16-byte vectors per chunk
    static constexpr int PER_THREAD = VECS / NT;
    static_assert(VECS % NT == 0, "tile must divide evenly over the block");

    u16x8 r[PER_THREAD];
    uint32_t ok;     // bit t: vector t lies inside the matrix (others are stored as zeros)

    __device__ __forceinline__ void load(const uint16_t* __restrict__ g, int ld, int row0, int k0, int rows,
                                         int k_extent, int tid) {
        ok = 0;
#pragma unroll
        for (int t = 0; t < PER_THREAD; ++t) {
            const int id = tid + t * NT;
            size_t off;
            bool in;
            if (KC) {
                const int row = row0 + id / (BK / 8), k = k0 + (id % (BK / 8)) * 8;
                in = row < rows && k < k_extent;
                off = (size_t)row * ld + k;
            } else {
                const int k = k0 + id / (ROWS / 8), row = row0 + (id % (ROWS / 8)) * 8;
                in = row < rows && k < k_extent;
                off = (size_t)k * ld + row;
            }
            r[t] = *(const u16x8*)(g + (in ? off : 0));
            ok |= (in ? 1u : 0u) << t;
        }
    }

    __device__ __forceinline__ void store(uint16_t* lds, int tid) const {
        const u16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < PER_THREAD; ++t) {
            const int id = tid + t * NT;
            int pos;
            if (KC) pos = (id / (BK / 8)) * KC_PITCH + (id % (BK / 8)) * 8;
            else pos = (id / (ROWS / 8)) * PITCH + (id % (ROWS / 8)) * 8;
            *(u16x8*)(lds + pos) = ((ok >> t) & 1u) ? r[t] : zero;
        }
    }

    // MFMA operand for rows row0..row0+31 (lane%32) and k = 16*s + 8*(lane/32) .. +7.
    __device__ __forceinline__ static bf16x8 fragment(const uint16_t* lds, int row0, int s, int lane) {
        if (KC) {
            return *(const bf16x8*)(lds + (row0 + lane % 32) * KC_PITCH + 16 * s + 8 * (lane / 32));
        } else {
            typedef __attribute__((address_space(3))) short4_t* lds_ptr;
            const int g = lane / 16, i = lane % 16;
            const uint16_t* p = lds + (16 * s + 8 * (g / 2) + i / 4) * PITCH + row0 + 16 * (g % 2) + 4 * (i % 4);
            const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p);
            const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * PITCH));
            short8_t v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            return __builtin_bit_cast(bf16x8, v);
        }
    }
};

template <int BM, int BN, int WM, int WN, bool A_KC, bool B_KC>
__global__ __launch_bounds__(64 * WM * WN) void pd_gemm_bf16_kernel(const GemmBf16Args a) {
    constexpr int NT = 64 * WM * WN;
    constexpr int TM = BM / (32 * WM), TN = BN / (32 * WN);
    using TA = TileH<BM, A_KC, NT>;
    using TB = TileH<BN, B_KC, NT>;
    constexpr int STAGING = (WM * WN) * 32 * (32 * TN + 8) * 2;       // epilogue staging, in bf16 units
    constexpr int LDS_ELEMS = 2 * (TA::SIZE + TB::SIZE) > STAGING ? 2 * (TA::SIZE + TB::SIZE) : STAGING;
    __shared__ __attribute__((aligned(16))) uint16_t lds[LDS_ELEMS];
    constexpr int BUF = TA::SIZE + TB::SIZE;      // one buffer = A tile followed by B tile

    const int tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int wm = wave / WN, wn = wave % WN;

    // workgroup -> (batch entry, tile): consecutive workgroups go to different dies, so the
    // die index is taken out first and each die walks its own contiguous range of tiles
    const int lin = (blockIdx.x % N_XCD) * a.tiles_per_xcd + blockIdx.x / N_XCD;
    if (lin >= a.total_tiles) return;
    const int per_batch = a.tiles_m * a.tiles_n;
    const int batch = lin / per_batch, t = lin % per_batch;
    const int group = t / (GROUP_M * a.tiles_n), first_m = group * GROUP_M;
    const int gsz = min(a.tiles_m - first_m, GROUP_M);
    const int in_group = t % (GROUP_M * a.tiles_n);
    const int m0 = (first_m + in_group % gsz) * BM, n0 = (in_group / gsz) * BN;

    const int bo = batch / a.batch_inner, bi = batch % a.batch_inner;
    const uint16_t* A = a.A + bo * a.sa_o + bi * a.sa_i;
    const uint16_t* B = a.B + bo * a.sb_o + bi * a.sb_i;
    const long long c_off = bo * a.sc_o + bi * a.sc_i;

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    TA ta;
    TB tb;
    const int nk = (a.K + BK - 1) / BK;
    ta.load(A, a.lda, m0, 0, a.M, a.K, tid);
    tb.load(B, a.ldb, n0, 0, a.N, a.K, tid);
    ta.store(lds, tid);
    tb.store(lds + TA::SIZE, tid);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) {
            ta.load(A, a.lda, m0, (kt + 1) * BK, a.M, a.K, tid);
            tb.load(B, a.ldb, n0, (kt + 1) * BK, a.N, a.K, tid);
        }
#pragma unroll
        for (int s = 0; s < BK / 16; ++s) {
            bf16x8 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[i] = TA::fragment(lds + cur * BUF, (wm * TM + i) * 32, s, lane);
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[j] = TB::fragment(lds + cur * BUF + TA::SIZE, (wn * TN + j) * 32, s, lane);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) {
            ta.store(lds + (cur ^ 1) * BUF, tid);
            tb.store(lds + (cur ^ 1) * BUF + TA::SIZE, tid);
        }
        __syncthreads();
    }

    // all waves are past the last barrier of the loop: the operand tiles are dead
    store_tile<TM, TN>(a, acc, m0 + wm * TM * 32, n0 + wn * TN * 32, c_off, (float*)lds + wave * (32 * (32 * TN + 8)), lane);
}

// ---------------------------------------------------------------------------------------
// Large-tile kernel: global -> LDS without passing through registers.
//
// With one 256 x 256 tile per CU, a chunk's loads must be issued several chunks ahead to
// cover memory latency, and there are no registers to hold that much data in flight.
// gfx950's 128-bit direct-to-LDS load (global_load_lds_dwordx4) writes lane l's 16 bytes
// to <LDS base> + 16*l, so a wave moves 1 KB per instruction and NS-1 chunks of 32 k are
// kept in flight in an NS-stage LDS ring.  Because the LDS placement is fixed, bank
// conflicts are avoided by permuting what each lane *fetches*:
//   * k-contiguous operand: stage rows are [row][32 k] = 64 bytes; the 16-byte slot q of row
//     r holds k-group q ^ ((r >> 2) & 3), which makes the 128-bit fragment reads of 16
//     consecutive rows hit 16 different bank groups;
//   * row-contiguous operand: stage rows are [k][rows]; the 64-byte granule index is XORed
//     with k % 4, so the four k-rows touched by one group of a transposing read differ.
// The fragment reads are issued through inline assembly: the compiler cannot tell which
// ring stage a direct-to-LDS load writes and would otherwise wait for *all* outstanding
// loads before every LDS read; here the wait is an explicit vmcnt that leaves the younger
// chunks in flight.  Requires K % 32 == 0 (no zero fill on this path); rows beyond M or N
// are fetched from a clamped (valid) row and never stored.
typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef __attribute__((address_space(1))) const void* global_void_ptr;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int DK = 32;   // k per ring stage
constexpr int NS = 4;    // ring stages

// One operand's part of the ring (4 waves): where each lane fetches from and where the
// fragments are read.
template <int ROWS, bool KC>
struct DmaTile {
    static constexpr int BYTES = ROWS * DK * 2;     // one stage
    static constexpr int PER_WAVE = ROWS / 64;      // 1 KB transfers per wave and chunk
    static_assert(ROWS % 64 == 0 && NS * BYTES + 16 * ROWS * 2 + 4 * ROWS * 2 <= 65536 + BYTES,
                  "stage offsets must fit the 16-bit LDS instruction offset");

    uint32_t off[PER_WAVE];   // byte offset of this lane's 16 bytes from the tile origin, chunk 0

    __device__ __forceinline__ void init(int ld, int row0, int rows, int wave, int lane) {
#pragma unroll
        for (int t = 0; t < PER_WAVE; ++t) {
            const int n = wave + 4 * t;
            if (KC) {
                const int row = n * 16 + lane / 4;
                const int kq = (lane % 4) ^ ((row >> 2) & 3);
                off[t] = (uint32_t)(min(row, rows - 1 - row0) * ld + kq * 8) * 2u;
            } else {
                const int e = n * 512 + lane * 8;
                const int k = e / ROWS, c = (e % ROWS) / 8;
                int col = ((((c / 4) ^ (k % 4)) * 4) + c % 4) * 8;
                if (row0 + col >= rows) col = 0;
                off[t] = (uint32_t)(k * ld + col) * 2u;
            }
        }
    }
    // tile origin and per-chunk advance, in bytes (both wave-uniform)
    __device__ __forceinline__ static const char* origin(const uint16_t* g, int ld, int row0) {
        return (const char*)(KC ? g + (size_t)row0 * ld : g + row0);
    }
    __device__ __forceinline__ static size_t chunk_bytes(int ld) { return KC ? (size_t)DK * 2 : (size_t)DK * ld * 2; }

    // Byte offset (inside a stage) of this lane's fragment address for 32-row block `blk`, k-step S.
    __device__ __forceinline__ static uint32_t frag_offset(int blk, int lane, int S) {
        if (KC) {
            const int r = lane % 32;
            return (uint32_t)((blk * 32 + r) * 64 + ((((2 * S + lane / 32)) ^ ((r >> 2) & 3)) * 16));
        } else {
            const int g = lane / 16, i = lane % 16;
            const int k = 8 * (g / 2) + i / 4;       // k-step and second half go into the instruction offset
            const int gran = blk ^ (k % 4);
            return (uint32_t)((k * ROWS + gran * 32 + 16 * (g % 2) + 4 * (i % 4)) * 2);
        }
    }
};

// One MFMA operand (8 bf16 per lane).  A k-contiguous operand is one 128-bit read; a
// row-contiguous operand is two transposing 64-bit reads (k..k+3 and k+4..k+7).  The ring
// stage (and for the transposing reads the k-step) is an instruction offset.
template <bool KC>
struct Frag;
template <>
struct Frag<true> {
    u32x4 v;
    static constexpr int UNITS = 1;
    template <int ROWS, int S, int U, int STG>
    __device__ __forceinline__ void read(uint32_t addr) {
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(STG * ROWS * DK * 2) : "memory");
    }
    __device__ __forceinline__ void tie() { asm volatile("" : "+v"(v)); }
    __device__ __forceinline__ bf16x8 get() const { return __builtin_bit_cast(bf16x8, v); }
};
template <>
struct Frag<false> {
    u32x2 lo, hi;
    static constexpr int UNITS = 2;
    template <int ROWS, int S, int U, int STG>
    __device__ __forceinline__ void read(uint32_t addr) {
        if (U == 0)
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
                         : "=v"(lo) : "v"(addr), "n"(STG * ROWS * DK * 2 + S * 16 * ROWS * 2) : "memory");
        else
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
                         : "=v"(hi) : "v"(addr), "n"(STG * ROWS * DK * 2 + S * 16 * ROWS * 2 + 4 * ROWS * 2) : "memory");
    }
    __device__ __forceinline__ void tie() { asm volatile("" : "+v"(lo), "+v"(hi)); }
    __device__ __forceinline__ bf16x8 get() const {
        const u32x4 v = {lo[0], lo[1], hi[0], hi[1]};
        return __builtin_bit_cast(bf16x8, v);
    }
};

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    // vmcnt is split over bits [3:0] and [15:14]; expcnt and lgkmcnt left unconstrained
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// 4 waves (2 x 2), one per SIMD; each owns (BM/2) x (BN/2).  With a single wave per SIMD
// nothing else hides a gap in its instruction stream, so the order is fixed by hand: every
// MFMA is followed by at most one LDS read or direct-to-LDS load (a scheduling barrier
// after each slot keeps the compiler from regrouping them), and the matrix pipe stays
// busy while the wave issues the memory instructions of the next k-step.  Addresses cost
// no vector instructions in the loop: LDS reads use a per-lane base plus an instruction
// offset for the ring stage (the chunk loop is unrolled NS times), the direct-to-LDS loads a
// scalar base pointer plus a per-lane 32-bit offset that never changes.
//
// Per chunk kt (two k-steps of 16), living in ring stage kt % NS:
//   step 0: MFMAs on the step-0 fragments; reads the step-1 fragments of stage kt
//   wait until chunk kt+1 has landed (vmcnt leaves the NS-2 younger chunks in flight), barrier:
//     every wave now holds all of chunk kt in registers, so stage kt is free
//   step 1: MFMAs on the step-1 fragments; reads the step-0 fragments of stage kt+1 and
//     issues the loads of chunk kt+NS into stage kt
template <int BM, int BN, bool A_KC, bool B_KC>
struct DmaGemm {
    static constexpr int TM = BM / 64, TN = BN / 64, NM = TM * TN;
    using TA = DmaTile<BM, A_KC>;
    using TB = DmaTile<BN, B_KC>;
    using FA = Frag<A_KC>;
    using FB = Frag<B_KC>;
    static constexpr int RING_B = NS * TA::BYTES;                  // B stages follow the A stages
    static constexpr int RING = NS * (TA::BYTES + TB::BYTES);
    static constexpr int IPT = TA::PER_WAVE + TB::PER_WAVE;        // loads per lane and chunk
    static constexpr int NR = TM * FA::UNITS + TN * FB::UNITS;     // LDS reads per k-step
    static constexpr int READ_SLOTS = NM >= 8 ? (NM * 3) / 4 : NM;  // reads go to the early slots
    static_assert((NS - 1) * IPT < 64, "ring depth");

    struct Frags {
        FA a[TM];
        FB b[TN];
        __device__ __forceinline__ void tie() {
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i].tie();
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j].tie();
        }
    };
    struct Ctx {
        TA ta;
        TB tb;
        const char* a_org;      // tile origins (uniform)
        const char* b_org;
        size_t a_step, b_step;  // bytes per chunk
        char* ring;
        int wave;               // uniform
        uint32_t fa_addr[TM][2], fb_addr[TN][2];   // LDS byte address of fragment (i, k-step s), stage 0
    };

    // LDS read number r of k-step S, ring stage STG, into `f` (A fragments first, then B)
    template <int S, int STG>
    __device__ __forceinline__ static void read_unit(Frags& f, int r, const Ctx& c) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            if (r == i * FA::UNITS) f.a[i].template read<BM, S, 0, STG>(c.fa_addr[i][S]);
            if (FA::UNITS == 2 && r == i * FA::UNITS + 1) f.a[i].template read<BM, S, 1, STG>(c.fa_addr[i][S]);
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            if (r == TM * FA::UNITS + j * FB::UNITS) f.b[j].template read<BN, S, 0, STG>(c.fb_addr[j][S]);
            if (FB::UNITS == 2 && r == TM * FA::UNITS + j * FB::UNITS + 1) f.b[j].template read<BN, S, 1, STG>(c.fb_addr[j][S]);
        }
    }

    // direct-to-LDS load number d of chunk `chunk` into ring stage STG
    template <int STG>
    __device__ __forceinline__ static void dma_unit(const Ctx& c, int d, int chunk) {
#pragma unroll
        for (int t = 0; t < TA::PER_WAVE; ++t)
            if (d == t)
                __builtin_amdgcn_global_load_lds((global_void_ptr)(c.a_org + chunk * c.a_step + c.ta.off[t]),
                                                 (lds_void_ptr)(c.ring + STG * TA::BYTES + (c.wave + 4 * t) * 1024), 16, 0, 0);
#pragma unroll
        for (int t = 0; t < TB::PER_WAVE; ++t)
            if (d == TA::PER_WAVE + t)
                __builtin_amdgcn_global_load_lds((global_void_ptr)(c.b_org + chunk * c.b_step + c.tb.off[t]),
                                                 (lds_void_ptr)(c.ring + RING_B + STG * TB::BYTES + (c.wave + 4 * t) * 1024), 16, 0, 0);
    }

    // One k-step: MFMAs on `cur`; if READ, the NR reads of k-step RS of stage RSTG go into `nxt`;
    // if DMA, chunk `chunk` is loaded into stage DSTG.  Ends with all reads complete.
    template <bool READ, int RS, int RSTG, bool DMA, int DSTG>
    __device__ __forceinline__ static void step(float16_t (&acc)[TM][TN], Frags& cur, Frags& nxt, const Ctx& c, int chunk) {
        cur.tie();
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            if (READ) {
#pragma unroll
                for (int r = 0; r < NR; ++r)
                    if (r * READ_SLOTS / NR == m) read_unit<RS, RSTG>(nxt, r, c);
            }
            if (DMA) {
#pragma unroll
                for (int d = 0; d < IPT; ++d)
                    if (d * NM / IPT == m) dma_unit<DSTG>(c, d, chunk);
            }
            const int i = m / TN, j = m % TN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cur.a[i].get(), cur.b[j].get(), acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (READ) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }

    // chunk kt0 + U (ring stage U) of the unrolled loop
    template <int U>
    __device__ __forceinline__ static void chunk(float16_t (&acc)[TM][TN], Frags& f0, Frags& f1, const Ctx& c, int kt0, int nk) {
        step<true, 1, U, false, 0>(acc, f0, f1, c, 0);
        wait_vmcnt<(NS - 2) * IPT>();      // chunk kt+1 has landed
        __builtin_amdgcn_s_barrier();
        // loads past the end re-fetch the last chunk into a stage nobody reads again: the number of
        // loads in flight stays the same in every iteration (one code path, constant vmcnt)
        step<true, 0, (U + 1) % NS, true, U>(acc, f1, f0, c, min(kt0 + U + NS, nk - 1));
    }
};

template <int BM, int BN, bool A_KC, bool B_KC>
__global__ __launch_bounds__(256, (BM * BN <= 128 * 128 ? 2 : 1)) void pd_gemm_bf16_dma_kernel(const GemmBf16Args a) {
    using G = DmaGemm<BM, BN, A_KC, B_KC>;
    using TA = typename G::TA;
    using TB = typename G::TB;
    constexpr int TM = G::TM, TN = G::TN, IPT = G::IPT;
    __shared__ __attribute__((aligned(1024))) char ring[G::RING];

    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int wm = wave / 2, wn = wave % 2;

    const int lin = (blockIdx.x % N_XCD) * a.tiles_per_xcd + blockIdx.x / N_XCD;
    if (lin >= a.total_tiles) return;
    const int per_batch = a.tiles_m * a.tiles_n;
    const int batch = lin / per_batch, t = lin % per_batch;
    const int group = t / (GROUP_M * a.tiles_n), first_m = group * GROUP_M;
    const int gsz = min(a.tiles_m - first_m, GROUP_M);
    const int in_group = t % (GROUP_M * a.tiles_n);
    const int m0 = (first_m + in_group % gsz) * BM, n0 = (in_group / gsz) * BN;

    const int bo = batch / a.batch_inner, bi = batch % a.batch_inner;
    const uint16_t* A = a.A + bo * a.sa_o + bi * a.sa_i;
    const uint16_t* B = a.B + bo * a.sb_o + bi * a.sb_i;
    const long long c_off = bo * a.sc_o + bi * a.sc_i;

    typename G::Ctx c;
    c.ta.init(a.lda, m0, a.M, wave, lane);
    c.tb.init(a.ldb, n0, a.N, wave, lane);
    c.a_org = TA::origin(A, a.lda, m0);
    c.b_org = TB::origin(B, a.ldb, n0);
    c.a_step = TA::chunk_bytes(a.lda);
    c.b_step = TB::chunk_bytes(a.ldb);
    c.ring = ring;
    c.wave = wave;
    const int nk = a.K / DK;       // a multiple of NS
    // fill the ring: chunks 0 .. NS-1 into stages 0 .. NS-1
#pragma unroll
    for (int d = 0; d < IPT; ++d) G::template dma_unit<0>(c, d, 0);
#pragma unroll
    for (int d = 0; d < IPT; ++d) G::template dma_unit<1>(c, d, 1);
#pragma unroll
    for (int d = 0; d < IPT; ++d) G::template dma_unit<2>(c, d, 2);
#pragma unroll
    for (int d = 0; d < IPT; ++d) G::template dma_unit<3>(c, d, 3);
    static_assert(NS == 4, "the ring fill and the unrolled loop below are written for 4 stages");
    // The first chunks are on their way: everything the loads do not need is set up behind them (fragment
    // addresses, cleared accumulators), inside the round trip to memory instead of in front of it.
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t ring_base = (uint32_t)(size_t)(lds_void_ptr)ring;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
        for (int i = 0; i < TM; ++i) c.fa_addr[i][s] = ring_base + TA::frag_offset(wm * TM + i, lane, A_KC ? s : 0);
#pragma unroll
        for (int j = 0; j < TN; ++j) c.fb_addr[j][s] = ring_base + G::RING_B + TB::frag_offset(wn * TN + j, lane, B_KC ? s : 0);
    }

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    wait_vmcnt<(NS - 1) * IPT>();      // chunk 0 has landed
    __builtin_amdgcn_s_barrier();

    typename G::Frags f0, f1;
#pragma unroll
    for (int r = 0; r < G::NR; ++r) G::template read_unit<0, 0>(f0, r, c);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

    for (int kt0 = 0; kt0 < nk; kt0 += NS) {
        G::template chunk<0>(acc, f0, f1, c, kt0, nk);
        G::template chunk<1>(acc, f0, f1, c, kt0, nk);
        G::template chunk<2>(acc, f0, f1, c, kt0, nk);
        G::template chunk<3>(acc, f0, f1, c, kt0, nk);
    }
    wait_vmcnt<0>();                // the trailing loads must not outlive the block's LDS allocation
    __builtin_amdgcn_s_barrier();   // every wave has taken its last fragments: the ring becomes staging space
    static_assert(4 * 32 * (32 * TN + 8) * 4 <= G::RING, "staging fits the ring");
    store_tile<TM, TN>(a, acc, m0 + wm * TM * 32, n0 + wn * TN * 32, c_off, (float*)ring + wave * (32 * (32 * TN + 8)), lane);
}

template <int BM, int BN>
int launch_gemm_bf16_dma(int ta, int tb, GemmBf16Args g, int batch, hipStream_t s) {
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    g.total_tiles = g.tiles_m * g.tiles_n * batch;
    g.tiles_per_xcd = (g.total_tiles + N_XCD - 1) / N_XCD;
    const dim3 grid(g.tiles_per_xcd * N_XCD);
    if (!ta && tb) pd_gemm_bf16_dma_kernel<BM, BN, true, true><<<grid, 256, 0, s>>>(g);
    else if (!ta && !tb) pd_gemm_bf16_dma_kernel<BM, BN, true, false><<<grid, 256, 0, s>>>(g);
    else if (ta && !tb) pd_gemm_bf16_dma_kernel<BM, BN, false, false><<<grid, 256, 0, s>>>(g);
    else pd_gemm_bf16_dma_kernel<BM, BN, false, true><<<grid, 256, 0, s>>>(g);
    PD_CHECK_LAUNCH("pd_gemm_bf16");
    return PD_OK;
}

template <int BM, int BN, int WM, int WN>
int launch_gemm_bf16(int ta, int tb, GemmBf16Args g, int batch, hipStream_t s) {
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    g.total_tiles = g.tiles_m * g.tiles_n * batch;
    g.tiles_per_xcd = (g.total_tiles + N_XCD - 1) / N_XCD;
    const dim3 grid(g.tiles_per_xcd * N_XCD);
    constexpr int NT = 64 * WM * WN;
    if (!ta && tb) pd_gemm_bf16_kernel<BM, BN, WM, WN, true, true><<<grid, NT, 0, s>>>(g);
    else if (!ta && !tb) pd_gemm_bf16_kernel<BM, BN, WM, WN, true, false><<<grid, NT, 0, s>>>(g);
    else if (ta && !tb) pd_gemm_bf16_kernel<BM, BN, WM, WN, false, false><<<grid, NT, 0, s>>>(g);
    else pd_gemm_bf16_kernel<BM, BN, WM, WN, false, true><<<grid, NT, 0, s>>>(g);
    PD_CHECK_LAUNCH("pd_gemm_bf16");
    return PD_OK;
}

}  // namespace

// tile choice forced by pd_gemm_bf16_set_tile (0 = the built-in choice)
static int g_force_bm = 0, g_force_bn = 0;

static int gemm_bf16_run(int trans_a, int trans_b, int M, int N, int K, const uint16_t* A, int lda,
                         const uint16_t* B, int ldb, void* C, int ldc, int out_f32, float alpha, float beta,
                         const float* bias, const uint16_t* residual, int ldr, int batch_outer, int batch_inner,
                         const int64_t* strides, void* stream, int act, uint16_t* aux_out, const uint16_t* aux_in,
                         int ld_aux) {
    PD_REQUIRE(M >= 0 && N >= 0 && K >= 0 && batch_outer >= 1 && batch_inner >= 1, PD_ESHAPE,
               "pd_gemm_bf16: bad dimensions");
    if (M == 0 || N == 0) return PD_OK;
    PD_REQUIRE(A && B && C, PD_EINVAL, "pd_gemm_bf16: NULL operand");
    PD_REQUIRE((long)batch_outer * batch_inner <= 65535, PD_ESHAPE, "pd_gemm_bf16: too many batch entries");
    PD_REQUIRE(batch_outer * batch_inner == 1 || strides, PD_EINVAL, "pd_gemm_bf16: batched call without strides");
    // 128-bit loads: leading dimensions, the vectorised extents and all batch offsets in units of 8 elements
    PD_REQUIRE(lda % 8 == 0 && ldb % 8 == 0 && pd_aligned(A, 16) && pd_aligned(B, 16), PD_ESHAPE,
               "pd_gemm_bf16: A/B must be 16-byte aligned with leading dimensions that are multiples of 8");
    PD_REQUIRE((trans_a ? M : K) % 8 == 0 && (trans_b ? K : N) % 8 == 0, PD_ESHAPE,
               "pd_gemm_bf16: the contiguous extent of each operand must be a multiple of 8");
    PD_REQUIRE(lda >= (trans_a ? M : K) && ldb >= (trans_b ? K : N) && ldc >= N, PD_ESHAPE,
               "pd_gemm_bf16: leading dimension smaller than the row length");
    PD_REQUIRE(!residual || (!out_f32 && ldr >= N), PD_EINVAL, "pd_gemm_bf16: residual needs bf16 output and ldr >= N");
    PD_REQUIRE(out_f32 || beta == 0.f, PD_EINVAL, "pd_gemm_bf16: beta needs fp32 output");
    GemmBf16Args g;
    g.A = A; g.B = B; g.C = C; g.bias = bias; g.residual = residual;
    g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.ldr = ldr;
    g.batch_inner = batch_inner;
    g.sa_o = g.sa_i = g.sb_o = g.sb_i = g.sc_o = g.sc_i = 0;
    if (strides) {
        g.sa_o = strides[0]; g.sa_i = strides[1]; g.sb_o = strides[2];
        g.sb_i = strides[3]; g.sc_o = strides[4]; g.sc_i = strides[5];
        PD_REQUIRE(g.sa_o % 8 == 0 && g.sa_i % 8 == 0 && g.sb_o % 8 == 0 && g.sb_i % 8 == 0, PD_ESHAPE,
                   "pd_gemm_bf16: A/B batch strides must be multiples of 8 elements");
    }
    g.alpha = alpha;
    g.beta = beta;
    g.out_f32 = out_f32 != 0;
    g.act = act; g.aux_out = aux_out; g.aux_in = aux_in; g.ld_aux = ld_aux;
    g.vec_store = N % 8 == 0 && ldc % 8 == 0 && pd_aligned(C, 16) && g.sc_o % 8 == 0 && g.sc_i % 8 == 0 &&
                  (!residual || (ldr % 8 == 0 && pd_aligned(residual, 16))) &&
                  (!act || (ld_aux % 8 == 0 && pd_aligned(act == 1 ? (const void*)aux_out : (const void*)aux_in, 16)));
    const int batch = batch_outer * batch_inner;
    hipStream_t s = (hipStream_t)stream;
    PD_REQUIRE((long long)((M + 63) / 64) * ((N + 63) / 64) * batch < (1ll << 28), PD_ESHAPE, "pd_gemm_bf16: too many tiles");
    const long tiles256 = (long)((M + 255) / 256) * ((N + 255) / 256) * batch;
    const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128) * batch;
    // direct-to-LDS kernel: whole ring rounds of k, and per-lane byte offsets that fit 32 bits
    const bool dma_ok = K % (DK * NS) == 0 && (long long)256 * (lda > ldb ? lda : ldb) * 2 < (1ll << 31);
    const bool wide = M >= 256 && N >= 256;       // a 256 x 256 tile is mostly inside the matrix
    if (g_force_bm && dma_ok) {
        if (g_force_bm == 256 && g_force_bn == 256) return launch_gemm_bf16_dma<256, 256>(trans_a, trans_b, g, batch, s);
        if (g_force_bm == 128 && g_force_bn == 128) return launch_gemm_bf16_dma<128, 128>(trans_a, trans_b, g, batch, s);
    }
    // 256 x 256 tiles (one block per CU, half the LDS reads per MFMA) from 192 tiles on, i.e. three quarters of
    // the CUs busy: 4096 x 4096 x 1024 takes 41 us against 49 with 128 x 128 tiles, 4096 x 3072 x 1024 (192
    // tiles) 34 against 39; products with fewer large tiles (4096 x 1024: 64) run two 128 x 128 blocks per CU.
    if (dma_ok && wide && tiles256 >= 192) return launch_gemm_bf16_dma<256, 256>(trans_a, trans_b, g, batch, s);
    if (dma_ok && M >= 128 && N >= 128) return launch_gemm_bf16_dma<128, 128>(trans_a, trans_b, g, batch, s);
    if (wide && tiles256 >= 192) return launch_gemm_bf16<256, 256, 2, 4>(trans_a, trans_b, g, batch, s);
    // narrow outputs (attention: N = head dimension): tall tiles, all waves stacked along M
    if (N <= 64 && M >= 256) return launch_gemm_bf16<256, 64, 4, 1>(trans_a, trans_b, g, batch, s);
    if (M >= 128 && N >= 128 && tiles128 >= 128) return launch_gemm_bf16<128, 128, 2, 2>(trans_a, trans_b, g, batch, s);
    return launch_gemm_bf16<64, 64, 2, 2>(trans_a, trans_b, g, batch, s);
}

extern "C" int pd_gemm_bf16_set_tile(int bm, int bn) {
    const bool known = (bm == 0 && bn == 0) || (bm == 128 && bn == 128) || (bm == 256 && bn == 256);
    PD_REQUIRE(known, PD_EINVAL, "pd_gemm_bf16_set_tile: tiles are 128 x 128 or 256 x 256 (0, 0 = built-in choice)");
    g_force_bm = bm;
    g_force_bn = bn;
    return PD_OK;
}

extern "C" int pd_gemm_bf16(int trans_a, int trans_b, int M, int N, int K, const uint16_t* A, int lda,
                            const uint16_t* B, int ldb, void* C, int ldc, int out_f32, float alpha, float beta,
                            const float* bias, const uint16_t* residual, int ldr, int batch_outer, int batch_inner,
                            const int64_t* strides /* sa_o, sa_i, sb_o, sb_i, sc_o, sc_i or NULL */, void* stream) {
    return gemm_bf16_run(trans_a, trans_b, M, N, K, A, lda, B, ldb, C, ldc, out_f32, alpha, beta, bias, residual, ldr,
                         batch_outer, batch_inner, strides, stream, 0, nullptr, nullptr, 0);
}

extern "C" int pd_gemm_bf16_gelu(int backward, int trans_a, int trans_b, int M, int N, int K, const uint16_t* A,
                                 int lda, const uint16_t* B, int ldb, uint16_t* C, int ldc, const float* bias,
                                 uint16_t* aux, int ld_aux, void* stream) {
    PD_REQUIRE(aux && ld_aux >= N, PD_EINVAL, "pd_gemm_bf16_gelu: aux must be an [M][ld_aux] matrix with ld_aux >= N");
    PD_REQUIRE(!backward || !bias, PD_EINVAL, "pd_gemm_bf16_gelu: the backward form takes no bias");
    return gemm_bf16_run(trans_a, trans_b, M, N, K, A, lda, B, ldb, C, ldc, 0, 1.0f, 0.0f, bias, nullptr, 0, 1, 1,
                         nullptr, stream, backward ? 2 : 1, backward ? nullptr : aux, backward ? aux : nullptr, ld_aux);
}

// ---------------------------------------------------------------------------------------
// fp32 products on the bf16 matrix pipes.  An fp32 value is the exact sum of three bf16 values
// (x1 = bf16(x), x2 = bf16(x - x1), x3 = bf16(x - x1 - x2): 3 x 8 significant bits), and a bf16 x bf16 product is
// exact in fp32, so  a . b = a1 b1 + (a1 b2 + a2 b1) + (a2 b2 + a1 b3 + a3 b1) + terms below 2^-24 a b  needs six bf16
// MFMAs where the fp32 MFMA needs one at a sixteenth of the rate -- and, unlike the fp32 MFMA, they run beside
// vector instructions.  The six products are one bf16 GEMM over a reduction six times as long: this kernel writes
// an operand's six slots -- A side: terms 1 3 2 2 1 1, B side: 3 1 1 2 2 1, small products first -- next to each
// other along the reduction index (side by side in a row, or stacked as six row blocks for an operand whose rows
// are the reduction index).
namespace {

__device__ __forceinline__ uint32_t split_rne(float f) {           // bf16 bits of f, round to nearest even
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x0040u;
    const uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    // a finite value that would round to infinity keeps its leading bits instead (the remainder carries the rest)
    return ((r & 0x7f80u) == 0x7f80u && (u & 0x7f800000u) != 0x7f800000u) ? (u >> 16) : r;
}

typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void split3_bf16_kernel(const float* __restrict__ x, long long rows, int cols,
                                                          long long ld, uint16_t* __restrict__ out, int b_side,
                                                          int stacked) {
    const int c4 = cols / 4;
    const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
    if (id >= rows * c4) return;
    const long long r = id / c4;
    const int c = (int)(id % c4) * 4;
    const float4_t v = *(const float4_t*)(x + r * ld + c);
    u16x4 t[3];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float rem = v[k];
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const uint32_t h = split_rne(rem);
            t[i][k] = (uint16_t)h;
            const float hf = __uint_as_float(h << 16);
            // (an infinity or a NaN is carried by the first term alone)
            rem = (h & 0x7f80u) == 0x7f80u ? 0.f : rem - hf;
        }
    }
    const int a_terms[6] = {0, 2, 1, 1, 0, 0}, b_terms[6] = {2, 0, 0, 1, 1, 0};
#pragma unroll
    for (int s = 0; s < 6; ++s) {
        const u16x4 val = t[b_side ? b_terms[s] : a_terms[s]];
        uint16_t* dst = stacked ? out + ((long long)s * rows + r) * cols + c : out + r * (6ll * cols) + (long long)s * cols + c;
        *(u16x4*)dst = val;
    }
}

}  // namespace

extern "C" int pd_split3_bf16_f32(const float* x, int64_t rows, int64_t cols, int64_t ld, uint16_t* out, int b_side,
                                  int stacked, void* stream) {
    PD_REQUIRE(rows >= 0 && cols >= 0 && cols % 4 == 0 && ld >= cols && ld % 4 == 0 && cols < (1ll << 30), PD_ESHAPE,
               "pd_split3_bf16_f32: cols and ld must be multiples of 4, ld >= cols");
    if (rows == 0 || cols == 0) return PD_OK;
    PD_REQUIRE(x && out && pd_aligned(x, 16) && pd_aligned(out, 8), PD_EINVAL,
               "pd_split3_bf16_f32: NULL or unaligned pointer");
    const long long threads = rows * (cols / 4);
    PD_REQUIRE((threads + 255) / 256 <= 0x7fffffffll, PD_ESHAPE, "pd_split3_bf16_f32: too large");
    split3_bf16_kernel<<<dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(
        x, rows, (int)cols, ld, out, b_side != 0, stacked != 0);
    PD_CHECK_LAUNCH("pd_split3_bf16_f32");
    return PD_OK;
}
