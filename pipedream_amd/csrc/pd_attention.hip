// Fused attention for the bf16 transformer stage: P = softmax(Q K^T / sqrt(d)), ctx = P V, and its
// backward pass, without ever writing the [batch, heads, seq, seq] score / probability tensors:
// the forward keeps one number per query (log2 of the softmax denominator, shifted), the backward
// recomputes P from it.  Three kernels: forward, backward query side (dQ), backward key side
// (dK, dV).
//
// The reference's checked-out branch has no transformer stage (PipeDream-2BW lives on another
// branch, README.md:7-8); the kernels do for such a stage's attention what cuBLAS + ATen do for the
// torch.nn layers of the reference's stages (runtime/runtime.py:529-530 forward, :606-608 backward).
//
// Bound: MFMA bf16 / vector ALU (seq * seq exponentials per head); algorithmic HBM traffic = qkv
// (and ctx, dctx in the backward) read once per kernel, ctx / dqkv written once.
//
// One block = one (batch, head) pair x 128 queries (or keys), 8 waves of 16.  The other side's two
// [seq][64] matrices are staged in LDS once per block with a row pitch of 72 bf16, which serves both
// the 128-bit fragment reads (8 consecutive k per lane) and the transposing reads.  Everything is
// computed in the orientation in which no accumulator ever has to change layout; shown for the
// forward (v_mfma_f32_16x16x32_bf16: lane l holds A row / B column l % 16, k-slots 8 (l / 16) + 0..7,
// and accumulator column l % 16, rows 4 (l / 16) + 0..3):
//   S^T = K Q^T   A = K rows from LDS (k = head dimension), B = this wave's Q rows straight from
//                 global memory; the accumulator of key tile t holds, in lane l, query l % 16 and
//                 keys 16 t + 4 (l / 16) + e, e = 0..3
//   softmax       over the keys of a query = over a lane's registers and the lanes l ^ 16, l ^ 32,
//                 l ^ 48: two shuffles per reduction
//   O^T = V^T P^T the B operand (8 keys per lane) is exactly the packed accumulators of key tiles 2u
//                 and 2u+1, so P goes from the softmax into the second product without touching
//                 LDS; a sum over keys does not care in which order the MFMA visits them, and the A
//                 operand (V^T) is fetched with the transposing LDS read ds_read_b64_tr_b16 at the
//                 matching keys.
// The backward kernels use the same two moves: "first product lands in the layout of the second
// product's B operand" and "transposed A operand through ds_read_b64_tr_b16".
#include "pd_internal.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int AT_D = 64;               // head dimension
constexpr int AT_THREADS = 512;        // 8 waves x 16 queries (keys)
constexpr int AT_QB = 128;             // queries (keys) per block
constexpr int AT_P = AT_D + 8;         // LDS row pitch (bf16)
constexpr float AT_LOG2E = 1.44269504088896340736f;

__device__ __forceinline__ uint16_t at_f2bf(float f) { return pd_f2bf(f); }
__device__ __forceinline__ float at_bf2f(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// rows [0, S) x 64 columns of a [.][ld] bf16 matrix -> LDS with pitch AT_P
template <int S>
__device__ __forceinline__ void at_stage(uint16_t* lds, const uint16_t* __restrict__ g, int ld, int tid) {
    constexpr int ITERS = S * (AT_D / 8) / AT_THREADS;
    static_assert(S * (AT_D / 8) % AT_THREADS == 0, "rows divide over the block");
    u16x8 r[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {         // all loads in flight before the first LDS store
        const int id = tid + it * AT_THREADS;
        r[it] = *(const u16x8*)(g + (size_t)(id / (AT_D / 8)) * ld + (id % (AT_D / 8)) * 8);
    }
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int id = tid + it * AT_THREADS;
        *(u16x8*)(lds + (id / (AT_D / 8)) * AT_P + (id % (AT_D / 8)) * 8) = r[it];
    }
}

// MFMA operand with 8 consecutive head-dimension values: row `row` of an LDS matrix, k-step s
__device__ __forceinline__ bf16x8 at_frag(const uint16_t* lds, int row, int s, int g) {
    return __builtin_bit_cast(bf16x8, *(const u16x8*)(lds + row * AT_P + 32 * s + 8 * g));
}

// Transposed MFMA A operand for the product over rows (keys or queries) 32u .. 32u+31 of an LDS matrix
// [row][64]: lane (li, g) receives column 16 dt + li at rows 32u + 4g + (0..3) (slots 0-3) and the
// same + 16 (slots 4-7), matching two packed 16-row accumulator tiles.  Inside a 16-lane group, input
// lane i addresses [row0 + i/4][col0 + 4 (i % 4)] and output lane j receives column col0 + j at rows
// row0 .. row0 + 3.
__device__ __forceinline__ bf16x8 at_frag_t(const uint16_t* lds, int u, int dt, int li, int g) {
    typedef __attribute__((address_space(3))) short4_t* lds_ptr;
    const uint16_t* p = lds + (32 * u + 4 * g + li / 4) * AT_P + 16 * dt + 4 * (li % 4);
    const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p);
    const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 16 * AT_P));
    const short8_t v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(bf16x8, v);
}

__device__ __forceinline__ void at_store4(uint16_t* p, const float4_t& v) {
    *(u16x4*)p = u16x4{at_f2bf(v[0]), at_f2bf(v[1]), at_f2bf(v[2]), at_f2bf(v[3])};
}

// ---- forward ---------------------------------------------------------------------------------------
// lse2[bh][q] = m * c + log2(sum_k 2^((s_k - m) c)), c = log2(e) / sqrt(d): P[q][k] = 2^(s_k c - lse2[q]).
template <int S, bool WRITE_P>
__global__ __launch_bounds__(AT_THREADS) void attention_fwd_kernel(const uint16_t* __restrict__ qkv,
                                                                  uint16_t* __restrict__ ctx,
                                                                  uint16_t* __restrict__ probs,
                                                                  float* __restrict__ lse2, int heads, float c) {
    constexpr int NT = S / 16;          // key tiles of 16
    __shared__ __attribute__((aligned(16))) uint16_t k_lds[S * AT_P];
    __shared__ __attribute__((aligned(16))) uint16_t v_lds[S * AT_P];

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int li = lane % 16, g = lane / 16;
    const int bh = blockIdx.y, b = bh / heads, h = bh % heads;
    const int H = heads * AT_D, ld = 3 * H;
    const uint16_t* base = qkv + (size_t)b * S * ld + h * AT_D;     // Q of this head; K at +H, V at +2H
    at_stage<S>(k_lds, base + H, ld, tid);
    at_stage<S>(v_lds, base + 2 * H, ld, tid);

    const int q = blockIdx.x * AT_QB + wave * 16 + li;              // this lane's query (always < S)
    bf16x8 qf[2];
#pragma unroll
    for (int s = 0; s < 2; ++s)
        qf[s] = __builtin_bit_cast(bf16x8, *(const u16x8*)(base + (size_t)q * ld + 32 * s + 8 * g));
    __syncthreads();

    float4_t sc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 2; ++s)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(at_frag(k_lds, 16 * t + li, s, g), qf[s], acc, 0, 0, 0);
        sc[t] = acc;
    }

    float m = -INFINITY;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) m = fmaxf(m, sc[t][e]);
    m = fmaxf(m, __shfl_xor(m, 16, 64));
    m = fmaxf(m, __shfl_xor(m, 32, 64));
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            sc[t][e] = __builtin_amdgcn_exp2f((sc[t][e] - m) * c);      // hardware exp2
            sum += sc[t][e];
        }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    const float inv = 1.0f / sum;
    if (lse2 && g == 0) lse2[(size_t)bh * S + q] = m * c + __builtin_amdgcn_logf(sum);   // v_log_f32 is log2

    uint16_t* prow = WRITE_P ? probs + ((size_t)bh * S + q) * S + 4 * g : nullptr;
    float4_t oacc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) oacc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < NT / 2; ++u) {
        u16x8 p;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            p[e] = at_f2bf(sc[2 * u][e] * inv);
            p[4 + e] = at_f2bf(sc[2 * u + 1][e] * inv);
        }
        if (WRITE_P) {
            *(u16x4*)(prow + 32 * u) = u16x4{p[0], p[1], p[2], p[3]};
            *(u16x4*)(prow + 32 * u + 16) = u16x4{p[4], p[5], p[6], p[7]};
        }
        const bf16x8 pf = __builtin_bit_cast(bf16x8, p);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
            oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(at_frag_t(v_lds, u, dt, li, g), pf, oacc[dt], 0, 0, 0);
    }

    uint16_t* crow = ctx + ((size_t)b * S + q) * H + h * AT_D + 4 * g;      // ctx[b*S + q][h*64 + 16 dt + 4 g + e]
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) at_store4(crow + 16 * dt, oacc[dt]);
}

// ---- backward, query side -----------------------------------------------------------------------------
// Per query block: P^T = 2^(K Q^T c - lse2), dP^T = V dO^T, dS^T = P^T o (dP^T - delta) / sqrt(d) with
// delta_q = sum_d dO[q][d] O[q][d] (= sum_k dP[q][k] P[q][k]), dQ^T = K^T dS^T.  The key tiles are
// processed two at a time, so nothing of size seq lives in registers.  delta is also written out
// for the key-side kernel.
template <int S>
__global__ __launch_bounds__(AT_THREADS) void attention_bwd_q_kernel(const uint16_t* __restrict__ qkv,
                                                                    const uint16_t* __restrict__ ctx,
                                                                    const uint16_t* __restrict__ dctx,
                                                                    const float* __restrict__ lse2,
                                                                    float* __restrict__ delta_out,
                                                                    uint16_t* __restrict__ dqkv, int heads, float c,
                                                                    float scale) {
    constexpr int NT = S / 16;
    __shared__ __attribute__((aligned(16))) uint16_t k_lds[S * AT_P];
    __shared__ __attribute__((aligned(16))) uint16_t v_lds[S * AT_P];

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int li = lane % 16, g = lane / 16;
    const int bh = blockIdx.y, b = bh / heads, h = bh % heads;
    const int H = heads * AT_D, ld = 3 * H;
    const uint16_t* base = qkv + (size_t)b * S * ld + h * AT_D;
    at_stage<S>(k_lds, base + H, ld, tid);
    at_stage<S>(v_lds, base + 2 * H, ld, tid);

    const int q = blockIdx.x * AT_QB + wave * 16 + li;
    const size_t orow = ((size_t)b * S + q) * H + h * AT_D;
    bf16x8 qf[2], dof[2];
    float delta = 0.f;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        qf[s] = __builtin_bit_cast(bf16x8, *(const u16x8*)(base + (size_t)q * ld + 32 * s + 8 * g));
        const u16x8 d8 = *(const u16x8*)(dctx + orow + 32 * s + 8 * g);
        const u16x8 o8 = *(const u16x8*)(ctx + orow + 32 * s + 8 * g);
        dof[s] = __builtin_bit_cast(bf16x8, d8);
#pragma unroll
        for (int j = 0; j < 8; ++j) delta += at_bf2f(d8[j]) * at_bf2f(o8[j]);
    }
    delta += __shfl_xor(delta, 16, 64);
    delta += __shfl_xor(delta, 32, 64);
    const float l2 = lse2[(size_t)bh * S + q];
    if (g == 0) delta_out[(size_t)bh * S + q] = delta;
    __syncthreads();

    float4_t qacc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) qacc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
    for (int u = 0; u < NT / 2; ++u) {
        u16x8 dsp;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int t = 2 * u + half;
            float4_t sa = {0.f, 0.f, 0.f, 0.f}, da = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(at_frag(k_lds, 16 * t + li, s, g), qf[s], sa, 0, 0, 0);
                da = __builtin_amdgcn_mfma_f32_16x16x32_bf16(at_frag(v_lds, 16 * t + li, s, g), dof[s], da, 0, 0, 0);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // P is rounded to bf16 as the forward pass did before using it
                const float p = at_bf2f(at_f2bf(__builtin_amdgcn_exp2f(sa[e] * c - l2)));
                dsp[4 * half + e] = at_f2bf(scale * p * (da[e] - delta));
            }
        }
        const bf16x8 dsf = __builtin_bit_cast(bf16x8, dsp);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
            qacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(at_frag_t(k_lds, u, dt, li, g), dsf, qacc[dt], 0, 0, 0);
    }

    uint16_t* qrow = dqkv + ((size_t)b * S + q) * ld + h * AT_D + 4 * g;     // the Q third of dqkv
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) at_store4(qrow + 16 * dt, qacc[dt]);
}

// ---- backward, key side --------------------------------------------------------------------------------
// Per key block, looping over all queries: S = Q K^T and dP = dO V^T now have the queries on the MFMA
// rows (A operands = Q and dO rows from LDS, B = this wave's K and V rows from global memory), so lane
// l holds key l % 16 and queries 16 t + 4 (l / 16) + e: P and dS land packed as B operands of the sums
// over queries dV^T = dO^T P and dK^T = Q^T dS, whose A operands are transposing reads of dO and Q.
template <int S>
__global__ __launch_bounds__(AT_THREADS) void attention_bwd_kv_kernel(const uint16_t* __restrict__ qkv,
                                                                     const uint16_t* __restrict__ dctx,
                                                                     const float* __restrict__ lse2,
                                                                     const float* __restrict__ delta,
                                                                     uint16_t* __restrict__ dqkv, int heads, float c,
                                                                     float scale) {
    constexpr int NT = S / 16;
    __shared__ __attribute__((aligned(16))) uint16_t q_lds[S * AT_P];
    __shared__ __attribute__((aligned(16))) uint16_t do_lds[S * AT_P];

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int li = lane % 16, g = lane / 16;
    const int bh = blockIdx.y, b = bh / heads, h = bh % heads;
    const int H = heads * AT_D, ld = 3 * H;
    const uint16_t* base = qkv + (size_t)b * S * ld + h * AT_D;
    at_stage<S>(q_lds, base, ld, tid);
    at_stage<S>(do_lds, dctx + (size_t)b * S * H + h * AT_D, H, tid);

    const int key = blockIdx.x * AT_QB + wave * 16 + li;
    bf16x8 kf[2], vf[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        kf[s] = __builtin_bit_cast(bf16x8, *(const u16x8*)(base + (size_t)key * ld + H + 32 * s + 8 * g));
        vf[s] = __builtin_bit_cast(bf16x8, *(const u16x8*)(base + (size_t)key * ld + 2 * H + 32 * s + 8 * g));
    }
    const float* l2p = lse2 + (size_t)bh * S + 4 * g;
    const float* dlp = delta + (size_t)bh * S + 4 * g;
    __syncthreads();

    float4_t kacc[4], vacc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) kacc[dt] = vacc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
    for (int u = 0; u < NT / 2; ++u) {
        u16x8 pp, dsp;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int t = 2 * u + half;
            float4_t sa = {0.f, 0.f, 0.f, 0.f}, da = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(at_frag(q_lds, 16 * t + li, s, g), kf[s], sa, 0, 0, 0);
                da = __builtin_amdgcn_mfma_f32_16x16x32_bf16(at_frag(do_lds, 16 * t + li, s, g), vf[s], da, 0, 0, 0);
            }
            const float4_t l2 = *(const float4_t*)(l2p + 16 * t);       // queries 16 t + 4 g + (0..3)
            const float4_t dl = *(const float4_t*)(dlp + 16 * t);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint16_t pb = at_f2bf(__builtin_amdgcn_exp2f(sa[e] * c - l2[e]));
                pp[4 * half + e] = pb;
                dsp[4 * half + e] = at_f2bf(scale * at_bf2f(pb) * (da[e] - dl[e]));
            }
        }
        const bf16x8 pf = __builtin_bit_cast(bf16x8, pp), dsf = __builtin_bit_cast(bf16x8, dsp);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
            vacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(at_frag_t(do_lds, u, dt, li, g), pf, vacc[dt], 0, 0, 0);
            kacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(at_frag_t(q_lds, u, dt, li, g), dsf, kacc[dt], 0, 0, 0);
        }
    }

    uint16_t* krow = dqkv + ((size_t)b * S + key) * ld + H + h * AT_D + 4 * g;    // the K third; V third at +H
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
        at_store4(krow + 16 * dt, kacc[dt]);
        at_store4(krow + H + 16 * dt, vacc[dt]);
    }
}

int at_check(const char* who, int batch, int seq, int heads, int head_dim) {
    PD_REQUIRE(batch > 0 && heads > 0, PD_ESHAPE, "%s: batch and heads must be positive", who);
    PD_REQUIRE(head_dim == AT_D && (seq == 512 || seq == 256 || seq == 128), PD_ESHAPE,
               "%s: needs head_dim 64 and seq 128, 256 or 512 (got %d, %d)", who, head_dim, seq);
    PD_REQUIRE((long long)batch * heads <= 65535, PD_ESHAPE, "%s: too many (batch, head) pairs", who);
    return PD_OK;
}

}  // namespace

extern "C" int pd_attention_fwd_supported(int seq, int head_dim) {
    return head_dim == AT_D && (seq == 512 || seq == 256 || seq == 128);
}

extern "C" int pd_attention_fwd_bf16(const uint16_t* qkv, uint16_t* ctx, uint16_t* probs, float* lse2, int batch,
                                     int seq, int heads, int head_dim, void* stream) {
    int rc = at_check("pd_attention_fwd_bf16", batch, seq, heads, head_dim);
    if (rc != PD_OK) return rc;
    PD_REQUIRE(qkv && ctx, PD_EINVAL, "pd_attention_fwd_bf16: NULL pointer");
    PD_REQUIRE(pd_aligned(qkv, 16) && pd_aligned(ctx, 8) && (!probs || pd_aligned(probs, 8)), PD_EINVAL,
               "pd_attention_fwd_bf16: qkv must be 16-byte, ctx and probs 8-byte aligned");
    const float c = AT_LOG2E / sqrtf((float)head_dim);
    const dim3 grid(seq / AT_QB, batch * heads);
    hipStream_t s = (hipStream_t)stream;
#define PD_AT_FWD(S_)                                                                                        \
    do {                                                                                                     \
        if (probs) attention_fwd_kernel<S_, true><<<grid, AT_THREADS, 0, s>>>(qkv, ctx, probs, lse2, heads, c); \
        else attention_fwd_kernel<S_, false><<<grid, AT_THREADS, 0, s>>>(qkv, ctx, probs, lse2, heads, c);      \
    } while (0)
    if (seq == 512) PD_AT_FWD(512);
    else if (seq == 256) PD_AT_FWD(256);
    else PD_AT_FWD(128);
#undef PD_AT_FWD
    PD_CHECK_LAUNCH("pd_attention_fwd_bf16");
    return PD_OK;
}

extern "C" int pd_attention_bwd_bf16(const uint16_t* qkv, const uint16_t* ctx, const uint16_t* dctx, const float* lse2,
                                     float* delta, uint16_t* dqkv, int batch, int seq, int heads, int head_dim,
                                     void* stream) {
    int rc = at_check("pd_attention_bwd_bf16", batch, seq, heads, head_dim);
    if (rc != PD_OK) return rc;
    PD_REQUIRE(qkv && ctx && dctx && lse2 && delta && dqkv, PD_EINVAL, "pd_attention_bwd_bf16: NULL pointer");
    PD_REQUIRE(pd_aligned(qkv, 16) && pd_aligned(ctx, 16) && pd_aligned(dctx, 16) && pd_aligned(lse2, 16) &&
                   pd_aligned(delta, 16) && pd_aligned(dqkv, 8),
               PD_EINVAL, "pd_attention_bwd_bf16: qkv, ctx, dctx, lse2, delta must be 16-byte, dqkv 8-byte aligned");
    const float scale = 1.0f / sqrtf((float)head_dim), c = AT_LOG2E * scale;
    const dim3 grid(seq / AT_QB, batch * heads);
    hipStream_t s = (hipStream_t)stream;
#define PD_AT_BWD(S_)                                                                                                  \
    do {                                                                                                               \
        attention_bwd_q_kernel<S_><<<grid, AT_THREADS, 0, s>>>(qkv, ctx, dctx, lse2, delta, dqkv, heads, c, scale);     \
        PD_CHECK_LAUNCH("pd_attention_bwd_bf16(dQ)");                                                                  \
        attention_bwd_kv_kernel<S_><<<grid, AT_THREADS, 0, s>>>(qkv, dctx, lse2, delta, dqkv, heads, c, scale);         \
    } while (0)
    if (seq == 512) PD_AT_BWD(512);
    else if (seq == 256) PD_AT_BWD(256);
    else PD_AT_BWD(128);
#undef PD_AT_BWD
    PD_CHECK_LAUNCH("pd_attention_bwd_bf16(dK, dV)");
    return PD_OK;
}
