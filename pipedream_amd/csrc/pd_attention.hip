// Fused attention forward for the bf16 transformer stage: P = softmax(scale * Q K^T), ctx = P V,
// one kernel instead of a batched GEMM, a softmax pass and a second batched GEMM over the
// [batch, heads, seq, seq] score tensor.  P is still written (bf16) because the backward pass
// reads it; the scores themselves never leave registers.
//
// The reference's checked-out branch has no transformer stage (PipeDream-2BW lives on another
// branch, README.md:7-8); the kernel does for such a stage's attention what cuBLAS + ATen do
// for the torch.nn layers of the reference's stages (runtime/runtime.py:529-530).
//
// Bound: MFMA bf16 / vector ALU (seq * seq exponentials per head); algorithmic HBM traffic =
// qkv read once, P and ctx written once.
//
// One block = one (batch, head) pair x 128 queries, 8 waves of 16 queries.  K and V of the
// head ([seq][64]) are staged in LDS once per block.  Everything is computed transposed so
// that no accumulator ever has to change layout:
//   S^T = K Q^T   v_mfma_f32_16x16x32_bf16, A = K rows from LDS (k = head dimension), B = this
//                 wave's Q rows straight from global memory; the accumulator of key tile t holds,
//                 in lane l, query l % 16 and keys 16 t + 4 (l / 16) + e, e = 0..3
//   softmax       over the keys of a query = over a lane's registers and the 4 lanes l, l^16,
//                 l^32, l^48: two shuffles per reduction
//   O^T = V^T P^T the B operand (8 keys per lane) is exactly the packed accumulators of key tiles
//                 2u and 2u+1, so P goes from the softmax into the second product without
//                 touching LDS; the sum over keys does not care in which order the MFMA visits
//                 them, and the A operand (V^T) is fetched with the transposing LDS read
//                 ds_read_b64_tr_b16 at the matching keys.
#include "pd_internal.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int AT_D = 64;               // head dimension
constexpr int AT_THREADS = 512;        // 8 waves x 16 queries
constexpr int AT_QB = 128;             // queries per block
constexpr int AT_KP = AT_D + 8;        // K row pitch in LDS (bf16): conflict-free 128-bit fragment reads
constexpr int AT_VP = AT_D + 16;       // V row pitch in LDS (bf16): spreads the 4 key rows of a transposing read

__device__ __forceinline__ uint16_t at_f2bf(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <int S>
__global__ __launch_bounds__(AT_THREADS) void attention_fwd_kernel(const uint16_t* __restrict__ qkv,
                                                                  uint16_t* __restrict__ ctx,
                                                                  uint16_t* __restrict__ probs, int heads,
                                                                  float scale_log2e) {
    constexpr int NT = S / 16;          // key tiles of 16
    __shared__ __attribute__((aligned(16))) uint16_t k_lds[S * AT_KP];
    __shared__ __attribute__((aligned(16))) uint16_t v_lds[S * AT_VP];

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int li = lane % 16, g = lane / 16;
    const int bh = blockIdx.y, b = bh / heads, h = bh % heads;
    const int H = heads * AT_D, ld = 3 * H;
    const uint16_t* base = qkv + (size_t)b * S * ld + h * AT_D;     // Q of this head; K at +H, V at +2H

    // ---- K and V of the head -> LDS (8 bf16 per thread and load) -----------------------------
    for (int id = tid; id < S * (AT_D / 8); id += AT_THREADS) {
        const int row = id / (AT_D / 8), c8 = (id % (AT_D / 8)) * 8;
        const u16x8 kv = *(const u16x8*)(base + (size_t)row * ld + H + c8);
        const u16x8 vv = *(const u16x8*)(base + (size_t)row * ld + 2 * H + c8);
        *(u16x8*)(k_lds + row * AT_KP + c8) = kv;
        *(u16x8*)(v_lds + row * AT_VP + c8) = vv;
    }

    // ---- this wave's 16 queries: B operand of S^T = K Q^T, two k-steps of 32 --------------------
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
        for (int s = 0; s < 2; ++s) {
            const bf16x8 kf = __builtin_bit_cast(bf16x8, *(const u16x8*)(k_lds + (16 * t + li) * AT_KP + 32 * s + 8 * g));
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[s], acc, 0, 0, 0);
        }
        sc[t] = acc;
    }

    // ---- softmax over the keys of each query --------------------------------------------------
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
            // e^(scale (s - m)) = 2^(scale log2(e) (s - m)) on the hardware exp2
            sc[t][e] = __builtin_amdgcn_exp2f((sc[t][e] - m) * scale_log2e);
            sum += sc[t][e];
        }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    const float inv = 1.0f / sum;

    // ---- P -> bf16: stored for the backward pass, and packed as the B operand of O^T = V^T P^T ----
    uint16_t* prow = probs + ((size_t)bh * S + q) * S + 4 * g;
    float4_t oacc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) oacc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    typedef __attribute__((address_space(3))) short4_t* lds_ptr;
#pragma unroll
    for (int u = 0; u < NT / 2; ++u) {
        u16x8 p;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            p[e] = at_f2bf(sc[2 * u][e] * inv);
            p[4 + e] = at_f2bf(sc[2 * u + 1][e] * inv);
        }
        *(u16x4*)(prow + 32 * u) = u16x4{p[0], p[1], p[2], p[3]};
        *(u16x4*)(prow + 32 * u + 16) = u16x4{p[4], p[5], p[6], p[7]};
        const bf16x8 pf = __builtin_bit_cast(bf16x8, p);
        // V^T fragments at the same keys: slots 0-3 = keys 32u + 4g + (0..3), slots 4-7 = the same + 16.
        // Transposing read: input lane i of a 16-lane group addresses [key0 + i/4][dim0 + 4 (i % 4)],
        // output lane j then holds dimension dim0 + j at keys key0 .. key0 + 3.
        const uint16_t* vb = v_lds + (32 * u + 4 * g + li / 4) * AT_VP + 4 * (li % 4);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
            const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(vb + 16 * dt));
            const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(vb + 16 * AT_VP + 16 * dt));
            const short8_t v8 = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, v8), pf, oacc[dt], 0, 0, 0);
        }
    }

    // ---- ctx[b*S + q][h*64 + 16 dt + 4 g + e] ---------------------------------------------------
    uint16_t* crow = ctx + ((size_t)b * S + q) * H + h * AT_D + 4 * g;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
        *(u16x4*)(crow + 16 * dt) =
            u16x4{at_f2bf(oacc[dt][0]), at_f2bf(oacc[dt][1]), at_f2bf(oacc[dt][2]), at_f2bf(oacc[dt][3])};
}

// Backward, query side: dP = dO V^T, dS = scale * P o (dP - delta) with delta_q = sum_d dO[q][d] O[q][d]
// (= sum_k dP[q][k] P[q][k]), dQ = dS K.  Same block shape and the same transposed formulation as
// the forward kernel with the roles V -> A operand of the first product, K -> transposed operand of
// the second: dP^T = V dO^T lands in the layout of the stored P, and the packed dS^T accumulators are
// the B operand of dQ^T = K^T dS^T.  dS (bf16, scale folded in) is written out for the two products
// that reduce over queries (dK = dS^T Q, dV = P^T dO), which stay strided-batched GEMMs.
template <int S>
__global__ __launch_bounds__(AT_THREADS) void attention_bwd_kernel(const uint16_t* __restrict__ qkv,
                                                                  const uint16_t* __restrict__ probs,
                                                                  const uint16_t* __restrict__ ctx,
                                                                  const uint16_t* __restrict__ dctx,
                                                                  uint16_t* __restrict__ ds_out,
                                                                  uint16_t* __restrict__ dqkv, int heads, float scale) {
    constexpr int NT = S / 16;
    __shared__ __attribute__((aligned(16))) uint16_t v_lds[S * AT_KP];     // fragment reads along d
    __shared__ __attribute__((aligned(16))) uint16_t k_lds[S * AT_VP];     // transposing reads

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int li = lane % 16, g = lane / 16;
    const int bh = blockIdx.y, b = bh / heads, h = bh % heads;
    const int H = heads * AT_D, ld = 3 * H;
    const uint16_t* base = qkv + (size_t)b * S * ld + h * AT_D;

    for (int id = tid; id < S * (AT_D / 8); id += AT_THREADS) {
        const int row = id / (AT_D / 8), c8 = (id % (AT_D / 8)) * 8;
        const u16x8 kv = *(const u16x8*)(base + (size_t)row * ld + H + c8);
        const u16x8 vv = *(const u16x8*)(base + (size_t)row * ld + 2 * H + c8);
        *(u16x8*)(k_lds + row * AT_VP + c8) = kv;
        *(u16x8*)(v_lds + row * AT_KP + c8) = vv;
    }

    const int q = blockIdx.x * AT_QB + wave * 16 + li;
    const size_t orow = ((size_t)b * S + q) * H + h * AT_D;
    bf16x8 dof[2];
    float delta = 0.f;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        const u16x8 d8 = *(const u16x8*)(dctx + orow + 32 * s + 8 * g);
        const u16x8 o8 = *(const u16x8*)(ctx + orow + 32 * s + 8 * g);
        dof[s] = __builtin_bit_cast(bf16x8, d8);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            delta += __uint_as_float((uint32_t)d8[j] << 16) * __uint_as_float((uint32_t)o8[j] << 16);
    }
    delta += __shfl_xor(delta, 16, 64);
    delta += __shfl_xor(delta, 32, 64);
    __syncthreads();

    const uint16_t* prow = probs + ((size_t)bh * S + q) * S + 4 * g;
    uint16_t* dsrow = ds_out + ((size_t)bh * S + q) * S + 4 * g;
    float4_t qacc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) qacc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    typedef __attribute__((address_space(3))) short4_t* lds_ptr;
#pragma unroll 2
    for (int u = 0; u < NT / 2; ++u) {
        u16x8 dsp;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int t = 2 * u + half;
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const bf16x8 vf = __builtin_bit_cast(bf16x8, *(const u16x8*)(v_lds + (16 * t + li) * AT_KP + 32 * s + 8 * g));
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, dof[s], acc, 0, 0, 0);
            }
            const u16x4 p4 = *(const u16x4*)(prow + 16 * t);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                dsp[4 * half + e] = at_f2bf(scale * __uint_as_float((uint32_t)p4[e] << 16) * (acc[e] - delta));
        }
        *(u16x4*)(dsrow + 32 * u) = u16x4{dsp[0], dsp[1], dsp[2], dsp[3]};
        *(u16x4*)(dsrow + 32 * u + 16) = u16x4{dsp[4], dsp[5], dsp[6], dsp[7]};
        const bf16x8 dsf = __builtin_bit_cast(bf16x8, dsp);
        const uint16_t* kb = k_lds + (32 * u + 4 * g + li / 4) * AT_VP + 4 * (li % 4);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
            const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(kb + 16 * dt));
            const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(kb + 16 * AT_VP + 16 * dt));
            const short8_t k8 = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            qacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, k8), dsf, qacc[dt], 0, 0, 0);
        }
    }

    uint16_t* qrow = dqkv + ((size_t)b * S + q) * ld + h * AT_D + 4 * g;     // the Q third of dqkv
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
        *(u16x4*)(qrow + 16 * dt) =
            u16x4{at_f2bf(qacc[dt][0]), at_f2bf(qacc[dt][1]), at_f2bf(qacc[dt][2]), at_f2bf(qacc[dt][3])};
}

}  // namespace

extern "C" int pd_attention_fwd_supported(int seq, int head_dim) {
    return head_dim == AT_D && (seq == 512 || seq == 256 || seq == 128);
}

extern "C" int pd_attention_fwd_bf16(const uint16_t* qkv, uint16_t* ctx, uint16_t* probs, int batch, int seq,
                                     int heads, int head_dim, void* stream) {
    PD_REQUIRE(batch > 0 && heads > 0, PD_ESHAPE, "pd_attention_fwd_bf16: batch and heads must be positive");
    PD_REQUIRE(pd_attention_fwd_supported(seq, head_dim), PD_ESHAPE,
               "pd_attention_fwd_bf16: needs head_dim 64 and seq 128, 256 or 512 (got %d, %d)", head_dim, seq);
    PD_REQUIRE(qkv && ctx && probs, PD_EINVAL, "pd_attention_fwd_bf16: NULL pointer");
    PD_REQUIRE(pd_aligned(qkv, 16) && pd_aligned(ctx, 8) && pd_aligned(probs, 8), PD_EINVAL,
               "pd_attention_fwd_bf16: qkv must be 16-byte, ctx and probs 8-byte aligned");
    PD_REQUIRE((long long)batch * heads <= 65535, PD_ESHAPE, "pd_attention_fwd_bf16: too many (batch, head) pairs");
    const float scale_log2e = 1.44269504088896340736f / sqrtf((float)head_dim);
    const dim3 grid(seq / AT_QB, batch * heads);
    hipStream_t s = (hipStream_t)stream;
    if (seq == 512) attention_fwd_kernel<512><<<grid, AT_THREADS, 0, s>>>(qkv, ctx, probs, heads, scale_log2e);
    else if (seq == 256) attention_fwd_kernel<256><<<grid, AT_THREADS, 0, s>>>(qkv, ctx, probs, heads, scale_log2e);
    else attention_fwd_kernel<128><<<grid, AT_THREADS, 0, s>>>(qkv, ctx, probs, heads, scale_log2e);
    PD_CHECK_LAUNCH("pd_attention_fwd_bf16");
    return PD_OK;
}

extern "C" int pd_attention_bwd_bf16(const uint16_t* qkv, const uint16_t* probs, const uint16_t* ctx,
                                     const uint16_t* dctx, uint16_t* ds, uint16_t* dqkv, int batch, int seq, int heads,
                                     int head_dim, void* stream) {
    PD_REQUIRE(batch > 0 && heads > 0, PD_ESHAPE, "pd_attention_bwd_bf16: batch and heads must be positive");
    PD_REQUIRE(pd_attention_fwd_supported(seq, head_dim), PD_ESHAPE,
               "pd_attention_bwd_bf16: needs head_dim 64 and seq 128, 256 or 512 (got %d, %d)", head_dim, seq);
    PD_REQUIRE(qkv && probs && ctx && dctx && ds && dqkv, PD_EINVAL, "pd_attention_bwd_bf16: NULL pointer");
    PD_REQUIRE(pd_aligned(qkv, 16) && pd_aligned(ctx, 16) && pd_aligned(dctx, 16) && pd_aligned(probs, 8) &&
                   pd_aligned(ds, 8) && pd_aligned(dqkv, 8),
               PD_EINVAL, "pd_attention_bwd_bf16: qkv, ctx, dctx must be 16-byte, probs, ds, dqkv 8-byte aligned");
    PD_REQUIRE((long long)batch * heads <= 65535, PD_ESHAPE, "pd_attention_bwd_bf16: too many (batch, head) pairs");
    const float scale = 1.0f / sqrtf((float)head_dim);
    const dim3 grid(seq / AT_QB, batch * heads);
    hipStream_t s = (hipStream_t)stream;
    if (seq == 512) attention_bwd_kernel<512><<<grid, AT_THREADS, 0, s>>>(qkv, probs, ctx, dctx, ds, dqkv, heads, scale);
    else if (seq == 256) attention_bwd_kernel<256><<<grid, AT_THREADS, 0, s>>>(qkv, probs, ctx, dctx, ds, dqkv, heads, scale);
    else attention_bwd_kernel<128><<<grid, AT_THREADS, 0, s>>>(qkv, probs, ctx, dctx, ds, dqkv, heads, scale);
    PD_CHECK_LAUNCH("pd_attention_bwd_bf16");
    return PD_OK;
}
