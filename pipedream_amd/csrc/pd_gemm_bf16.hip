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
// (trans_b = 1, k-contiguous).  A 256-thread block owns a BM x BN tile, each of its 4 waves
// (BM/2) x (BN/2); K runs in chunks of 32 through LDS, where both operands are kept
// k-contiguous with a pitch of 40 bf16 so that one conflict-free 128-bit LDS read feeds
// one MFMA (8 k-values per lane).  An operand that is not k-contiguous in memory is
// transposed on the way into LDS: a thread loads the same 8 columns of two adjacent
// k-rows and writes eight packed (k, k+1) pairs.
// Epilogue: (+ bias[N] fp32) (+ residual[M][N] bf16) -> bf16, or fp32 with optional
// accumulation into C (weight gradients summed over micro-batches).
#include "pd_internal.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

namespace {

constexpr int BKH = 32;           // k per chunk
constexpr int PITCH = BKH + 8;    // LDS row pitch in bf16 elements (80 bytes)
constexpr int GB_THREADS = 256;

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
};

__device__ __forceinline__ uint16_t f2bf(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float bf2f(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// One operand tile of ROWS rows x 32 k, k-contiguous in LDS.
template <int ROWS, bool KC>
struct TileH {
    static constexpr int SIZE = ROWS * PITCH;
    // KC: ROWS*4 16-byte vectors, one row-quarter each.  !KC: 16 k-pairs x ROWS/8 column groups.
    static constexpr int TASKS = KC ? ROWS * 4 : 16 * (ROWS / 8);
    static constexpr int PER_THREAD = (TASKS + GB_THREADS - 1) / GB_THREADS;

    u16x8 r0[PER_THREAD], r1[PER_THREAD];

    __device__ __forceinline__ void load(const uint16_t* __restrict__ g, int ld, int row0, int k0, int rows,
                                         int k_extent, int tid) {
        const u16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < PER_THREAD; ++t) {
            const int id = tid + t * GB_THREADS;
            if (KC) {
                const int row = id / 4, kq = (id % 4) * 8;
                const bool ok = id < TASKS && row0 + row < rows && k0 + kq < k_extent;
                const uint16_t* src = ok ? g + (size_t)(row0 + row) * ld + k0 + kq : g;
                u16x8 v = *(const u16x8*)src;
                r0[t] = ok ? v : zero;
            } else {
                const int kp = id / (ROWS / 8), cg = (id % (ROWS / 8)) * 8;
                const int k = k0 + 2 * kp;
                const bool okc = id < TASKS && row0 + cg < rows;
                const bool ok0 = okc && k < k_extent, ok1 = okc && k + 1 < k_extent;
                const uint16_t* s0 = ok0 ? g + (size_t)k * ld + row0 + cg : g;
                const uint16_t* s1 = ok1 ? g + (size_t)(k + 1) * ld + row0 + cg : g;
                u16x8 v0 = *(const u16x8*)s0;
                u16x8 v1 = *(const u16x8*)s1;
                r0[t] = ok0 ? v0 : zero;
                r1[t] = ok1 ? v1 : zero;
            }
        }
    }

    __device__ __forceinline__ void store(uint16_t* lds, int tid) const {
#pragma unroll
        for (int t = 0; t < PER_THREAD; ++t) {
            const int id = tid + t * GB_THREADS;
            if (id >= TASKS) continue;
            if (KC) {
                const int row = id / 4, kq = (id % 4) * 8;
                *(u16x8*)(lds + row * PITCH + kq) = r0[t];
            } else {
                const int kp = id / (ROWS / 8), cg = (id % (ROWS / 8)) * 8;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t pair = (uint32_t)r0[t][j] | ((uint32_t)r1[t][j] << 16);
                    *(uint32_t*)(lds + (cg + j) * PITCH + 2 * kp) = pair;
                }
            }
        }
    }
};

template <int BM, int BN, bool A_KC, bool B_KC>
__global__ __launch_bounds__(GB_THREADS) void pd_gemm_bf16_kernel(const GemmBf16Args a) {
    constexpr int TM = BM / 64, TN = BN / 64;
    using TA = TileH<BM, A_KC>;
    using TB = TileH<BN, B_KC>;
    __shared__ __attribute__((aligned(16))) uint16_t lds_a[2][TA::SIZE];
    __shared__ __attribute__((aligned(16))) uint16_t lds_b[2][TB::SIZE];

    const int tid = threadIdx.x;
    const int wave = tid / 64, lane = tid % 64;
    const int wm = wave / 2, wn = wave % 2;
    const int idx = lane % 32, h = lane / 32;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int bo = blockIdx.z / a.batch_inner, bi = blockIdx.z % a.batch_inner;
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
    const int nk = (a.K + BKH - 1) / BKH;
    ta.load(A, a.lda, m0, 0, a.M, a.K, tid);
    tb.load(B, a.ldb, n0, 0, a.N, a.K, tid);
    ta.store(lds_a[0], tid);
    tb.store(lds_b[0], tid);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) {
            ta.load(A, a.lda, m0, (kt + 1) * BKH, a.M, a.K, tid);
            tb.load(B, a.ldb, n0, (kt + 1) * BKH, a.N, a.K, tid);
        }
#pragma unroll
        for (int s = 0; s < BKH / 16; ++s) {
            bf16x8 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                fa[i] = *(const bf16x8*)(lds_a[cur] + (wm * (BM / 2) + i * 32 + idx) * PITCH + 16 * s + 8 * h);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                fb[j] = *(const bf16x8*)(lds_b[cur] + (wn * (BN / 2) + j * 32 + idx) * PITCH + 16 * s + 8 * h);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) {
            ta.store(lds_a[cur ^ 1], tid);
            tb.store(lds_b[cur ^ 1], tid);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = n0 + wn * (BN / 2) + j * 32 + idx;
            if (col >= a.N) continue;
            const float bv = a.bias ? a.bias[col] : 0.f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = m0 + wm * (BM / 2) + i * 32 + 8 * (e / 4) + 4 * h + (e % 4);
                if (row >= a.M) continue;
                float v = a.alpha * acc[i][j][e] + bv;
                const long long off = c_off + (long long)row * a.ldc + col;
                if (a.out_f32) {
                    float* p = (float*)a.C + off;
                    if (a.beta != 0.f) v += a.beta * *p;
                    *p = v;
                } else {
                    if (a.residual) v += bf2f(a.residual[c_off + (long long)row * a.ldr + col]);
                    ((uint16_t*)a.C)[off] = f2bf(v);
                }
            }
        }
}

template <int BM, int BN>
int launch_gemm_bf16(int ta, int tb, const GemmBf16Args& g, int batch, hipStream_t s) {
    dim3 grid((g.N + BN - 1) / BN, (g.M + BM - 1) / BM, batch);
    if (!ta && tb) pd_gemm_bf16_kernel<BM, BN, true, true><<<grid, GB_THREADS, 0, s>>>(g);
    else if (!ta && !tb) pd_gemm_bf16_kernel<BM, BN, true, false><<<grid, GB_THREADS, 0, s>>>(g);
    else if (ta && !tb) pd_gemm_bf16_kernel<BM, BN, false, false><<<grid, GB_THREADS, 0, s>>>(g);
    else pd_gemm_bf16_kernel<BM, BN, false, true><<<grid, GB_THREADS, 0, s>>>(g);
    PD_CHECK_LAUNCH("pd_gemm_bf16");
    return PD_OK;
}

}  // namespace

extern "C" int pd_gemm_bf16(int trans_a, int trans_b, int M, int N, int K, const uint16_t* A, int lda,
                            const uint16_t* B, int ldb, void* C, int ldc, int out_f32, float alpha, float beta,
                            const float* bias, const uint16_t* residual, int ldr, int batch_outer, int batch_inner,
                            const int64_t* strides /* sa_o, sa_i, sb_o, sb_i, sc_o, sc_i or NULL */, void* stream) {
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
    const int batch = batch_outer * batch_inner;
    hipStream_t s = (hipStream_t)stream;
    const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128) * batch;
    if (N >= 128 && M >= 128 && tiles128 >= 256) return launch_gemm_bf16<128, 128>(trans_a, trans_b, g, batch, s);
    return launch_gemm_bf16<64, 64>(trans_a, trans_b, g, batch, s);
}
