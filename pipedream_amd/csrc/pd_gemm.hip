// fp32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32), used by the
// Linear / LSTM / projection layers of a stage: forward  Y = X W^T + b,
// input gradient dX = dY W, weight gradient dW = dY^T X.
//
// Replaces the cuBLAS calls torch.nn.Linear / torch.nn.LSTM make inside the
// reference's stage modules (e.g. runtime/image_classification/models/vgg16/
// gpus=4_straight/stage3.py:19-25) and their autograd backward
// (runtime/runtime.py:529-530 forward, :606-608 backward).
//
// Bound: MFMA fp32 (157.3 TFLOP/s).  2*M*N*K flop per call.
//
// Tiling: a 256-thread block (4 waves, 2x2) owns a BM x BN tile of C; each wave
// owns (BM/2) x (BN/2) = TM x TN MFMA tiles of 32x32.  K is consumed in chunks of
// 16 staged through LDS in the operand's own memory order (no transposition on
// the way in): a k-contiguous operand is read back with one 128-bit LDS load
// per four MFMAs, a row-contiguous one with 32-bit loads.  The k index is
// permuted identically for A and B (lane-half h takes k = 8g + 4h + s at MFMA
// step s), which a sum over k does not care about.
#include "pd_internal.h"

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

namespace {

constexpr int BK = 16;
constexpr int GEMM_THREADS = 256;

struct GemmArgs {
    const float* A;
    const float* B;
    float* C;
    const float* bias;  // [N] or null
    int M, N, K;
    int lda, ldb, ldc;
    float beta;         // C = acc + beta*C_old (0 -> overwrite, C_old not read)
    int relu;
    int a_vec, b_vec;   // 128-bit global loads allowed for A / B
    int k_per_split;    // blockIdx.z owns k in [z*k_per_split, (z+1)*k_per_split) and writes C + z*c_split
    long long c_split;  // elements between the partial results of consecutive splits
    uint32_t a_bytes, b_bytes;  // extents of A and B for the fast path's buffer descriptors (0 = fast path off)
};

// Operand tile in LDS.  KC (k-contiguous): [ROWS][BK+4]; otherwise [BK][ROWS+4].
template <int ROWS, bool KC>
struct Tile {
    static constexpr int STRIDE = KC ? (BK + 4) : (ROWS + 4);
    static constexpr int SIZE = KC ? ROWS * STRIDE : BK * STRIDE;

    // Global -> registers.  `rows` is the extent of the row index (M or N), `k_extent` = K.
    // Each thread moves ROWS*BK/4/256 float4s.
    static constexpr int VEC_PER_THREAD = ROWS * BK / 4 / GEMM_THREADS;

    __device__ static void load(float4_t (&r)[VEC_PER_THREAD], const float* __restrict__ g, int ld, int row0, int k0,
                                int rows, int k_extent, bool vec, int tid) {
#pragma unroll
        for (int v = 0; v < VEC_PER_THREAD; ++v) {
            int id = tid + v * GEMM_THREADS;
            int row, k;
            if (KC) {
                row = id / (BK / 4);
                k = (id % (BK / 4)) * 4;
            } else {
                k = id / (ROWS / 4);
                row = (id % (ROWS / 4)) * 4;
            }
            int gr = row0 + row, gk = k0 + k;
            float4_t x = {0.f, 0.f, 0.f, 0.f};
            if (KC) {
                if (gr < rows) {
                    const float* p = g + (size_t)gr * ld + gk;
                    if (vec && gk + 3 < k_extent) {
                        x = *(const float4_t*)p;
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (gk + j < k_extent) x[j] = p[j];
                    }
                }
            } else {
                if (gk < k_extent) {
                    const float* p = g + (size_t)gk * ld + gr;
                    if (vec && gr + 3 < rows) {
                        x = *(const float4_t*)p;
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (gr + j < rows) x[j] = p[j];
                    }
                }
            }
            r[v] = x;
        }
    }

    // Fast path for full tiles of 16-byte-aligned operands: per-thread byte offsets of the chunk at k = 0
    // (computed once), the chunk's k offset goes into the scalar offset of a buffer load, so the inner
    // loop spends no vector instructions on addresses or bounds.
    __device__ static void offsets(uint32_t (&off)[VEC_PER_THREAD], int ld, int row0, int tid) {
#pragma unroll
        for (int v = 0; v < VEC_PER_THREAD; ++v) {
            const int id = tid + v * GEMM_THREADS;
            if (KC) off[v] = (uint32_t)((row0 + id / (BK / 4)) * ld + (id % (BK / 4)) * 4) * 4;
            else off[v] = (uint32_t)((id / (ROWS / 4)) * ld + row0 + (id % (ROWS / 4)) * 4) * 4;
        }
    }
    __device__ static void load_fast(float4_t (&r)[VEC_PER_THREAD], __amdgpu_buffer_rsrc_t rs,
                                     const uint32_t (&off)[VEC_PER_THREAD], int ld, int k) {
        const int soff = (KC ? k : k * ld) * 4;
#pragma unroll
        for (int v = 0; v < VEC_PER_THREAD; ++v)
            r[v] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(rs, off[v], soff, 0));
    }

    __device__ static void store(float* lds, const float4_t (&r)[VEC_PER_THREAD], int tid) {
#pragma unroll
        for (int v = 0; v < VEC_PER_THREAD; ++v) {
            int id = tid + v * GEMM_THREADS;
            int row, k;
            if (KC) {
                row = id / (BK / 4);
                k = (id % (BK / 4)) * 4;
                *(float4_t*)(lds + row * STRIDE + k) = r[v];
            } else {
                k = id / (ROWS / 4);
                row = (id % (ROWS / 4)) * 4;
                *(float4_t*)(lds + k * STRIDE + row) = r[v];
            }
        }
    }

    // Fragment for MFMA steps s=0..3 of k-group g: lane (idx = lane%32, h = lane/32)
    // supplies element [row0+idx][8g + 4h + s].
    __device__ static float4_t frag(const float* lds, int row, int g, int h) {
        if (KC) {
            return *(const float4_t*)(lds + row * STRIDE + 8 * g + 4 * h);
        } else {
            float4_t f;
#pragma unroll
            for (int s = 0; s < 4; ++s) f[s] = lds[(8 * g + 4 * h + s) * STRIDE + row];
            return f;
        }
    }
};

template <int BM, int BN, bool A_KC, bool B_KC, bool FULL>
__global__ __launch_bounds__(GEMM_THREADS) void pd_gemm_f32_kernel(const GemmArgs a) {
    constexpr int TM = BM / 64, TN = BN / 64;  // MFMA tiles per wave in m / n
    using TA = Tile<BM, A_KC>;
    using TB = Tile<BN, B_KC>;
    __shared__ __attribute__((aligned(16))) float lds_a[2][TA::SIZE];
    __shared__ __attribute__((aligned(16))) float lds_b[2][TB::SIZE];

    const int tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int wm = wave / 2, wn = wave % 2;
    const int idx = lane % 32, h = lane / 32;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    float4_t ra[TA::VEC_PER_THREAD], rb[TB::VEC_PER_THREAD];
    const int k_begin = blockIdx.z * a.k_per_split;
    const int k_end = min(a.K, k_begin + a.k_per_split);
    const int nk = (k_end - k_begin + BK - 1) / BK;
    float* const C = a.C + blockIdx.z * a.c_split;
    uint32_t oa[TA::VEC_PER_THREAD], ob[TB::VEC_PER_THREAD];
    const __amdgpu_buffer_rsrc_t rsa = __builtin_amdgcn_make_buffer_rsrc((void*)a.A, 0, a.a_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsb = __builtin_amdgcn_make_buffer_rsrc((void*)a.B, 0, a.b_bytes, 0x00020000);
    if (FULL) {
        TA::offsets(oa, a.lda, m0, tid);
        TB::offsets(ob, a.ldb, n0, tid);
        TA::load_fast(ra, rsa, oa, a.lda, k_begin);
        TB::load_fast(rb, rsb, ob, a.ldb, k_begin);
    } else {
        TA::load(ra, a.A, a.lda, m0, k_begin, a.M, k_end, a.a_vec, tid);
        TB::load(rb, a.B, a.ldb, n0, k_begin, a.N, k_end, a.b_vec, tid);
    }
    TA::store(lds_a[0], ra, tid);
    TB::store(lds_b[0], rb, tid);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) {  // prefetch the next chunk into registers while this one is multiplied
            if (FULL) {
                TA::load_fast(ra, rsa, oa, a.lda, k_begin + (kt + 1) * BK);
                TB::load_fast(rb, rsb, ob, a.ldb, k_begin + (kt + 1) * BK);
            } else {
                TA::load(ra, a.A, a.lda, m0, k_begin + (kt + 1) * BK, a.M, k_end, a.a_vec, tid);
                TB::load(rb, a.B, a.ldb, n0, k_begin + (kt + 1) * BK, a.N, k_end, a.b_vec, tid);
            }
        }
#pragma unroll
        for (int g = 0; g < BK / 8; ++g) {
            float4_t fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[i] = TA::frag(lds_a[cur], wm * (BM / 2) + i * 32 + idx, g, h);
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[j] = TB::frag(lds_b[cur], wn * (BN / 2) + j * 32 + idx, g, h);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) {
            TA::store(lds_a[cur ^ 1], ra, tid);
            TB::store(lds_b[cur ^ 1], rb, tid);
        }
        __syncthreads();
    }

    // Epilogue.  Accumulator element e of lane (idx, h): row = 8*(e/4) + 4*h + e%4, col = idx.
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = n0 + wn * (BN / 2) + j * 32 + idx;
            if (!FULL && col >= a.N) continue;
            const float bv = a.bias ? a.bias[col] : 0.f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = m0 + wm * (BM / 2) + i * 32 + 8 * (e / 4) + 4 * h + (e % 4);
                if (!FULL && row >= a.M) continue;
                float* p = C + (size_t)row * a.ldc + col;
                float v = acc[i][j][e] + bv;
                if (a.beta != 0.f) v += a.beta * *p;
                if (a.relu) v = v > 0.f ? v : 0.f;
                *p = v;
            }
        }
}

template <int BM, int BN>
int launch_gemm(int trans_a, int trans_b, const GemmArgs& g, hipStream_t s, int splits = 1) {
    dim3 grid((g.N + BN - 1) / BN, (g.M + BM - 1) / BM, splits);
    // A is k-contiguous when it is NOT transposed; B (stored [K][N]) is k-contiguous when it IS.
    // Full tiles of aligned operands whose extents fit a 32-bit byte offset take the fast loader.
    const int k_span = splits > 1 ? g.k_per_split : g.K;
    const bool full = g.M % BM == 0 && g.N % BN == 0 && k_span % BK == 0 && g.K % BK == 0 && g.a_vec && g.b_vec &&
                      g.a_bytes != 0 && g.b_bytes != 0;
#define PD_GEMM_LAUNCH(AKC, BKC)                                                                 \
    do {                                                                                          \
        if (full) pd_gemm_f32_kernel<BM, BN, AKC, BKC, true><<<grid, GEMM_THREADS, 0, s>>>(g);    \
        else pd_gemm_f32_kernel<BM, BN, AKC, BKC, false><<<grid, GEMM_THREADS, 0, s>>>(g);        \
    } while (0)
    if (!trans_a && trans_b) PD_GEMM_LAUNCH(true, true);
    else if (!trans_a && !trans_b) PD_GEMM_LAUNCH(true, false);
    else if (trans_a && !trans_b) PD_GEMM_LAUNCH(false, false);
    else PD_GEMM_LAUNCH(false, true);
#undef PD_GEMM_LAUNCH
    PD_CHECK_LAUNCH("pd_gemm_f32");
    return PD_OK;
}

// ---------------------------------------------------------------------------------------
// Skinny split-k kernel: M <= 128 (the LSTM recurrent products with M = batch, the
// classifier layers with M = 64), A k-contiguous.  A block owns up to 64 rows (blockIdx.y) x
// 128 columns of one k range and is bound by fetching its operands, so they are streamed with
// 128-bit direct-to-LDS loads (lane l's 16 bytes land at <base> + 16*l) through a ring of 8
// or 4 stages of 16 k, all but one or two in flight, and multiplied as they arrive.
// Because the LDS placement of such a load is fixed, the lanes fetch a permutation that
// makes the fragment reads conflict-free: the 16-byte slot q of row r of a k-contiguous
// stage holds k-group q ^ ((r >> 2) & 3); a row-contiguous stage ([k][128 columns]) has its
// two 256-byte halves swapped for k % 8 >= 4.
// The fragment reads are inline assembly: the compiler cannot tell which ring stage a
// direct-to-LDS load writes and would wait for all loads in flight before any LDS read;
// here the wait is an explicit vmcnt that leaves the younger stages in flight.  Stage
// numbers past the end of the k range re-fetch the last stage (and are not multiplied), so
// the number of loads in flight is the same in every iteration.
typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef __attribute__((address_space(1))) const void* global_void_ptr;

constexpr int SK_COLS = 128;             // tile columns
// (ring stages of BK = 16, SK_STAGES below: 8 or 4)

// Rows per block: WM = 1: 64, waves 1 x 4, 64 x 32 each (the one launched).  WM = 2: 128, waves 2 x 2, 64 x 64 each.
template <int WM, bool B_KC, int SK_STAGES>
struct Skinny {
    static constexpr int BM = 64 * WM;
    static constexpr int WN = 4 / WM;
    static constexpr int TN = SK_COLS / (32 * WN);
    static constexpr int A_STAGE = BM * BK * 4, B_STAGE = SK_COLS * BK * 4;
    static constexpr int B_BASE = SK_STAGES * A_STAGE;
    static constexpr int LDS_BYTES = SK_STAGES * (A_STAGE + B_STAGE);
    static constexpr int A_PER_WAVE = BM / 16 / 4, B_PER_WAVE = SK_COLS / 16 / 4;
    static constexpr int IPT = A_PER_WAVE + B_PER_WAVE;      // loads per lane and stage
    static constexpr int IN_FLIGHT = SK_STAGES - 2;           // younger stages outstanding at the wait

    size_t src_a[A_PER_WAVE], src_b[B_PER_WAVE];
    uint32_t fa_addr[2][2], fb_addr[TN][2];       // [fragment][k-group g] LDS byte addresses, stage 0

    __device__ __forceinline__ void init(const GemmArgs& a, int m0, int n0, int wave, int lane, uint32_t lds_base) {
        const int wm = wave / WN, wn = wave % WN;
        const int idx = lane % 32, h = lane / 32;
#pragma unroll
        for (int t = 0; t < A_PER_WAVE; ++t) {
            const int row = (wave + 4 * t) * 16 + lane / 4;
            const int kq = (lane % 4) ^ ((row >> 2) & 3);
            src_a[t] = (size_t)min(m0 + row, a.M - 1) * a.lda + kq * 4;
        }
#pragma unroll
        for (int t = 0; t < B_PER_WAVE; ++t) {
            const int n = wave + 4 * t;
            if (B_KC) {
                const int row = n * 16 + lane / 4;
                const int kq = (lane % 4) ^ ((row >> 2) & 3);
                src_b[t] = (size_t)min(n0 + row, a.N - 1) * a.ldb + kq * 4;
            } else {
                const int k = 2 * n + lane / 32;
                int col = ((lane % 32) ^ (((k >> 2) & 1) << 4)) * 4;
                if (n0 + col >= a.N) col = 0;
                src_b[t] = (size_t)k * a.ldb + n0 + col;
            }
        }
#pragma unroll
        for (int g = 0; g < 2; ++g) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int r = (wm * 2 + i) * 32 + idx;
                fa_addr[i][g] = lds_base + r * 64 + (((2 * g + h) ^ ((r >> 2) & 3)) * 16);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int r = (wn * TN + j) * 32 + idx;
                if (B_KC) fb_addr[j][g] = lds_base + B_BASE + r * 64 + (((2 * g + h) ^ ((r >> 2) & 3)) * 16);
                else fb_addr[j][g] = lds_base + B_BASE + ((8 * g + 4 * h) * SK_COLS + (r ^ (h << 6))) * 4;
            }
        }
    }

    template <int ST>
    __device__ __forceinline__ void issue(const GemmArgs& a, char* lds, int k, int wave) const {
#pragma unroll
        for (int t = 0; t < A_PER_WAVE; ++t)
            __builtin_amdgcn_global_load_lds((global_void_ptr)(a.A + src_a[t] + k),
                                             (lds_void_ptr)(lds + ST * A_STAGE + (wave + 4 * t) * 1024), 16, 0, 0);
#pragma unroll
        for (int t = 0; t < B_PER_WAVE; ++t)
            __builtin_amdgcn_global_load_lds((global_void_ptr)(a.B + src_b[t] + (B_KC ? (size_t)k : (size_t)k * a.ldb)),
                                             (lds_void_ptr)(lds + B_BASE + ST * B_STAGE + (wave + 4 * t) * 1024), 16, 0, 0);
    }

    // fragments of ring stage ST: fa[i][g], fb[j][g] (4 consecutive k-steps each)
    template <int ST>
    __device__ __forceinline__ void read(float4_t (&fa)[2][2], float4_t (&fb)[TN][2]) const {
#pragma unroll
        for (int g = 0; g < 2; ++g) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fa[i][g]) : "v"(fa_addr[i][g]), "n"(ST * A_STAGE) : "memory");
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if (B_KC) {
                    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fb[j][g]) : "v"(fb_addr[j][g]), "n"(ST * B_STAGE) : "memory");
                } else {
                    float q0, q1, q2, q3;
                    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(q0) : "v"(fb_addr[j][g]), "n"(ST * B_STAGE) : "memory");
                    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(q1) : "v"(fb_addr[j][g]), "n"(ST * B_STAGE + SK_COLS * 4) : "memory");
                    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(q2) : "v"(fb_addr[j][g]), "n"(ST * B_STAGE + 2 * SK_COLS * 4) : "memory");
                    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(q3) : "v"(fb_addr[j][g]), "n"(ST * B_STAGE + 3 * SK_COLS * 4) : "memory");
                    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(q0), "+v"(q1), "+v"(q2), "+v"(q3));
                    fb[j][g] = float4_t{q0, q1, q2, q3};
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int g = 0; g < 2; ++g) {
#pragma unroll
            for (int i = 0; i < 2; ++i) asm volatile("" : "+v"(fa[i][g]));
#pragma unroll
            for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(fb[j][g]));
        }
    }
};

template <int N>
__device__ __forceinline__ void sk_wait_vmcnt() {
    // vmcnt is split over bits [3:0] and [15:14]; expcnt and lgkmcnt left unconstrained
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

template <int WM, bool B_KC, int SK_STAGES>
__global__ __launch_bounds__(GEMM_THREADS) void pd_gemm_skinny_kernel(const GemmArgs a) {
    using S = Skinny<WM, B_KC, SK_STAGES>;
    constexpr int TN = S::TN;
    __shared__ __attribute__((aligned(1024))) char lds[S::LDS_BYTES];
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int wm = wave / S::WN, wn = wave % S::WN;
    const int idx = lane % 32, h = lane / 32;
    const int m0 = blockIdx.y * S::BM, n0 = blockIdx.x * SK_COLS;
    const int k_begin = blockIdx.z * a.k_per_split;
    const int k_end = min(a.K, k_begin + a.k_per_split);
    const int total = k_end > k_begin ? (k_end - k_begin) / BK : 0;      // stages to multiply
    float* const C = a.C + blockIdx.z * a.c_split;

    float16_t acc[2][TN];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    if (total > 0) {
        S sk;
        sk.init(a, m0, n0, wave, lane, (uint32_t)(size_t)(lds_void_ptr)lds);
        // k of stage number i, clamped to the last stage of the range
#define SK_K(i) (k_begin + min((i), total - 1) * BK)
#define SK_FILL(ST) if constexpr (ST < SK_STAGES - 1) sk.template issue<ST>(a, lds, SK_K(ST), wave);
        SK_FILL(0) SK_FILL(1) SK_FILL(2) SK_FILL(3) SK_FILL(4) SK_FILL(5) SK_FILL(6)
#undef SK_FILL
        static_assert(SK_STAGES == 8 || SK_STAGES == 4, "the ring fill and the unrolled loop are written for 4 or 8 stages");
        // Stage i (ring slot ST): wait until it has landed everywhere; every wave is then also past
        // its reads of stage i-1, so that slot is refilled with stage i + SK_STAGES - 1; then read and multiply.
#define SK_STAGE(ST)                                                                                      \
        if constexpr (ST < SK_STAGES) {                                                                       \
            const int i = i0 + ST;                                                                            \
            sk_wait_vmcnt<S::IN_FLIGHT * S::IPT>();                                                          \
            __builtin_amdgcn_s_barrier();                                                                     \
            sk.template issue<(ST + SK_STAGES - 1) % SK_STAGES>(a, lds, SK_K(i + SK_STAGES - 1), wave);      \
            if (i < total) {                                                                                  \
                float4_t fa[2][2], fb[TN][2];                                                                 \
                sk.template read<ST % SK_STAGES>(fa, fb);                                                     \
                _Pragma("unroll") for (int g = 0; g < 2; ++g)                                                 \
                _Pragma("unroll") for (int q = 0; q < 4; ++q)                                                 \
                _Pragma("unroll") for (int ii = 0; ii < 2; ++ii)                                              \
                _Pragma("unroll") for (int jj = 0; jj < TN; ++jj)                                             \
                    acc[ii][jj] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[ii][g][q], fb[jj][g][q], acc[ii][jj], 0, 0, 0); \
            }                                                                                                 \
        }
        for (int i0 = 0; i0 < total; i0 += SK_STAGES) {
            SK_STAGE(0) SK_STAGE(1) SK_STAGE(2) SK_STAGE(3) SK_STAGE(4) SK_STAGE(5) SK_STAGE(6) SK_STAGE(7)
        }
#undef SK_STAGE
#undef SK_K
        sk_wait_vmcnt<0>();     // the trailing re-fetches must not outlive the block's LDS allocation
    }

    if (m0 + S::BM <= a.M && n0 + SK_COLS <= a.N) {
        // the whole tile lies inside the matrix (the LSTM products): 64 stores per lane without a test each
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                float* const base = C + (size_t)(m0 + (wm * 2 + i) * 32 + 4 * h) * a.ldc + n0 + (wn * TN + j) * 32 + idx;
#pragma unroll
                for (int e = 0; e < 16; ++e) base[(size_t)(8 * (e / 4) + (e % 4)) * a.ldc] = acc[i][j][e];
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = n0 + (wn * TN + j) * 32 + idx;
            if (col >= a.N) continue;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = m0 + (wm * 2 + i) * 32 + 8 * (e / 4) + 4 * h + (e % 4);
                if (row < a.M) C[(size_t)row * a.ldc + col] = acc[i][j][e];
            }
        }
}

// out = (sum over splits of partials) (+ bias) (+ beta*out) (relu): 4 elements per thread
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partials, int splits, int M, int N,
                                                           const float* __restrict__ bias, int relu, float beta,
                                                           float* __restrict__ C, int ldc) {
    const int n4 = N / 4;
    const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
    if (id >= (long long)M * n4) return;
    const int row = (int)(id / n4), col = (int)(id % n4) * 4;
    const size_t per = (size_t)M * N;
    // eight partials in flight at a time (one at a time the loop is a chain of round trips to memory),
    // added in a fixed order
    const float* src = partials + (size_t)row * N + col;
    float4_t v = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < splits; s0 += 8) {
        float4_t p[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const bool live = s0 + u < splits;
            p[u] = *(const float4_t*)(src + (size_t)(live ? s0 + u : s0) * per);
            if (!live) p[u] = float4_t{0.f, 0.f, 0.f, 0.f};
        }
        v += ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
    }
    if (bias) v += *(const float4_t*)(bias + col);
    float* p = C + (size_t)row * ldc + col;
    if (beta != 0.f) v += beta * *(const float4_t*)p;
    if (relu)
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = v[j] > 0.f ? v[j] : 0.f;
    *(float4_t*)p = v;
}

}  // namespace

// Byte extent of an operand with `rows` rows of leading dimension `ld`, or 0 if it does not fit the 32-bit
// offsets of the fast loader.
static uint32_t operand_bytes(long rows, long ld) {
    const long b = rows * ld * 4;
    return b < (1L << 31) ? (uint32_t)b : 0u;
}

extern "C" int pd_gemm_f32(int trans_a, int trans_b, int M, int N, int K, const float* A, int lda, const float* B,
                           int ldb, float beta, float* C, int ldc, const float* bias, int relu, void* stream) {
    PD_REQUIRE(M >= 0 && N >= 0 && K >= 0, PD_ESHAPE, "pd_gemm_f32: negative dimension");
    if (M == 0 || N == 0) return PD_OK;
    PD_REQUIRE(A && B && C, PD_EINVAL, "pd_gemm_f32: NULL operand");
    PD_REQUIRE(lda >= (trans_a ? M : K) && ldb >= (trans_b ? K : N) && ldc >= N, PD_ESHAPE,
               "pd_gemm_f32: leading dimension smaller than the row length");
    GemmArgs g;
    g.A = A; g.B = B; g.C = C; g.bias = bias;
    g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc;
    g.beta = beta;
    g.relu = relu != 0;
    g.a_vec = pd_aligned(A, 16) && lda % 4 == 0;
    g.b_vec = pd_aligned(B, 16) && ldb % 4 == 0;
    g.k_per_split = K;
    g.c_split = 0;
    g.a_bytes = operand_bytes(trans_a ? K : M, lda);
    g.b_bytes = operand_bytes(trans_b ? N : K, ldb);
    hipStream_t s = (hipStream_t)stream;
    // Small problems use 64x64 tiles so that more of the 256 CUs get a block.
    long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    if (tiles128 >= 256) return launch_gemm<128, 128>(trans_a, trans_b, g, s);
    return launch_gemm<64, 64>(trans_a, trans_b, g, s);
}

extern "C" int pd_gemm_splitk_f32(int trans_a, int trans_b, int M, int N, int K, const float* A, int lda,
                                  const float* B, int ldb, float* partials, int splits, void* stream) {
    PD_REQUIRE(M > 0 && N > 0 && K > 0 && splits >= 1 && splits <= 1024, PD_ESHAPE, "pd_gemm_splitk_f32: bad dimensions");
    PD_REQUIRE(A && B && partials, PD_EINVAL, "pd_gemm_splitk_f32: NULL operand");
    PD_REQUIRE(lda >= (trans_a ? M : K) && ldb >= (trans_b ? K : N), PD_ESHAPE,
               "pd_gemm_splitk_f32: leading dimension smaller than the row length");
    GemmArgs g;
    g.A = A; g.B = B; g.C = partials; g.bias = nullptr;
    g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = N;
    g.beta = 0.f;
    g.relu = 0;
    g.a_vec = pd_aligned(A, 16) && lda % 4 == 0;
    g.b_vec = pd_aligned(B, 16) && ldb % 4 == 0;
    // every split gets a whole number of 16-wide k chunks; trailing splits may be empty and then write zeros
    g.k_per_split = (((K + splits - 1) / splits) + BK - 1) / BK * BK;
    g.c_split = (long long)M * N;
    g.a_bytes = operand_bytes(trans_a ? K : M, lda);
    g.b_bytes = operand_bytes(trans_b ? N : K, ldb);
    hipStream_t s = (hipStream_t)stream;
    if (!trans_a && M <= 128 && N % 4 == 0 && g.a_vec && g.b_vec && g.k_per_split % BK == 0 && K % BK == 0 &&
        (size_t)128 * (lda > ldb ? lda : ldb) * 4 < (1ull << 31)) {
        const dim3 grid((N + SK_COLS - 1) / SK_COLS, 1, splits);
        // up to 64 rows: one block row, 8 ring stages (96 KB; these products stream large weight matrices from HBM
        // once).  65 to 128 rows (the LSTM recurrences): two block rows of 64 and 4 stages (48 KB).  For the same
        // number of blocks that halves the k split, and with it the partial results written here and read back by
        // the consumer (16 -> 8 MB per LSTM time step); three such blocks fit a CU, of one launch or of the
        // recurrences of two minibatches running on different streams.
        if (M <= 64) {
            if (trans_b) pd_gemm_skinny_kernel<1, true, 8><<<grid, GEMM_THREADS, 0, s>>>(g);
            else pd_gemm_skinny_kernel<1, false, 8><<<grid, GEMM_THREADS, 0, s>>>(g);
        } else {
            const dim3 grid2((N + SK_COLS - 1) / SK_COLS, 2, splits);
            if (trans_b) pd_gemm_skinny_kernel<1, true, 4><<<grid2, GEMM_THREADS, 0, s>>>(g);
            else pd_gemm_skinny_kernel<1, false, 4><<<grid2, GEMM_THREADS, 0, s>>>(g);
        }
        PD_CHECK_LAUNCH("pd_gemm_splitk_f32");
        return PD_OK;
    }
    if (M > 64 && N >= 128) return launch_gemm<128, 128>(trans_a, trans_b, g, s, splits);
    return launch_gemm<64, 64>(trans_a, trans_b, g, s, splits);
}

extern "C" int pd_splitk_reduce_f32(const float* partials, int splits, int M, int N, const float* bias, int relu,
                                    float beta, float* C, int ldc, void* stream) {
    PD_REQUIRE(M > 0 && N > 0 && N % 4 == 0 && splits >= 1 && ldc >= N && ldc % 4 == 0, PD_ESHAPE,
               "pd_splitk_reduce_f32: need N and ldc multiples of 4");
    PD_REQUIRE(partials && C && pd_aligned(partials, 16) && pd_aligned(C, 16) && (!bias || pd_aligned(bias, 16)), PD_EINVAL,
               "pd_splitk_reduce_f32: NULL or unaligned pointer");
    const long long total = (long long)M * (N / 4);
    splitk_reduce_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(
        partials, splits, M, N, bias, relu != 0, beta, C, ldc);
    PD_CHECK_LAUNCH("pd_splitk_reduce_f32");
    return PD_OK;
}
