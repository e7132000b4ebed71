// Sequence-to-sequence pieces of the translation stages: the label-smoothing criterion and the
// variable-length sequence helpers of the bidirectional encoder layer.
//
// They stand in for
//   * LabelSmoothing.forward (runtime/translation/seq2seq/train/smoothing.py:23-34) and the backward pass
//     autograd derives from it: fp32 log-softmax over the vocabulary, NLL + smoothing term, padding rows
//     dropped, sum divided by the batch size;
//   * revert_varlen_tensor (runtime/translation/seq2seq/csrc/pack_utils_kernel.cu:7-62): every sequence of
//     a [T, B, F] tensor reversed in time over its own length, zeros behind it;
//   * set_mask_cpp (runtime/translation/seq2seq/csrc/pack_utils.cpp:13-31) and the multiplication by that
//     mask in EmuBidirLSTM.emu_bidir_lstm (runtime/translation/seq2seq/models/encoder.py:51-55).
//
// All of it is HBM-bound.  Algorithmic traffic: the criterion's forward reads every logit once (the row
// stays in registers between the max, the sums and the loss), its backward reads every logit once and
// writes every gradient once; the sequence helpers read and write every element once.  The reference
// builds a table of T*B source offsets on the host and uploads it for every call; here the kernels take
// the B lengths (device memory) and derive the source row themselves.
#include "pd_internal.h"

#include <math.h>

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int SQ_THREADS = 256;
constexpr int SQ_WAVES = SQ_THREADS / 64;

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
// e^(x - m) for x <= m (or a little above): the hardware's 2^x on (x - m) * log2(e).  The difference is
// taken first, so the argument's rounding error is relative to the difference, not to the logits: the
// result is within about 1e-7 * (1 + |x - m|) of exact, relative.
__device__ __forceinline__ float exp_diff(float x, float m) {
    return __builtin_amdgcn_exp2f((x - m) * 1.44269504088896340736f);
}

// Block-wide reductions over the four waves; every thread gets the result.  `red` is reused: the trailing
// barrier lets the next reduction overwrite it.
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    if (threadIdx.x % 64 == 0) red[threadIdx.x / 64] = v;
    __syncthreads();
    v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    return v;
}
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    if (threadIdx.x % 64 == 0) red[threadIdx.x / 64] = v;
    __syncthreads();
    v = (red[0] + red[1]) + (red[2] + red[3]);
    __syncthreads();
    return v;
}

// row_loss = confidence * (lse - x[target]) + smoothing * (lse - mean(x)); 0 for padding rows.
__device__ __forceinline__ void smoothing_row_result(float m, float s, float sx, const float* x, int64_t t, int V,
                                                     float confidence, float smoothing, float* row_loss,
                                                     float* lse) {
    const float l = m + logf(s);
    *lse = l;
    // a target outside [0, V) that is not the padding index poisons the loss instead of reading out of bounds
    const float xt = (t >= 0 && t < V) ? x[t] : NAN;
    *row_loss = confidence * (l - xt) + smoothing * (l - sx / (float)V);
}

// One block per row, one pass over the row (4 | V, rows 16-byte aligned): every thread keeps a running
// maximum and a sum of exponentials relative to it ("online" softmax) over groups of 8 float4 that are
// loaded together; the sum is rescaled once per group when the maximum grows.  Few registers, so many
// rows are in flight per CU.  A padding row costs no traffic.
constexpr int LS_GROUP = 8;

__global__ __launch_bounds__(SQ_THREADS) void label_smoothing_fwd_kernel(
    const float* __restrict__ logits, const int64_t* __restrict__ target, float* __restrict__ row_loss,
    float* __restrict__ lse, int V, int64_t ld, int64_t padding_idx, float confidence, float smoothing) {
    __shared__ float red[SQ_WAVES];
    const int r = blockIdx.x;
    const int64_t t = target[r];
    if (t == padding_idx) {                      // uniform over the block
        if (threadIdx.x == 0) { row_loss[r] = 0.f; lse[r] = 0.f; }
        return;
    }
    const float* x = logits + (int64_t)r * ld;
    float m = -INFINITY, s = 0.f, sx = 0.f;
    for (int c0 = threadIdx.x * 4; c0 < V; c0 += LS_GROUP * SQ_THREADS * 4) {
        float4_t v[LS_GROUP];
#pragma unroll
        for (int i = 0; i < LS_GROUP; ++i) {
            const int c = c0 + i * SQ_THREADS * 4;
            if (c < V) v[i] = *(const float4_t*)(x + c);
        }
        float gm = m;
#pragma unroll
        for (int i = 0; i < LS_GROUP; ++i)
            if (c0 + i * SQ_THREADS * 4 < V)
                gm = fmaxf(gm, fmaxf(fmaxf(v[i][0], v[i][1]), fmaxf(v[i][2], v[i][3])));
        if (gm != m) s *= exp_diff(m, gm);       // (m = -inf before the first finite element: s = 0 * 0)
        m = gm;
        const float mm = m == -INFINITY ? 0.f : m;   // a group of -inf logits adds e^(-inf) = 0, not NaN
#pragma unroll
        for (int i = 0; i < LS_GROUP; ++i)
            if (c0 + i * SQ_THREADS * 4 < V) {
                s += (exp_diff(v[i][0], mm) + exp_diff(v[i][1], mm)) + (exp_diff(v[i][2], mm) + exp_diff(v[i][3], mm));
                sx += (v[i][0] + v[i][1]) + (v[i][2] + v[i][3]);
            }
    }
    // a thread that saw no element (V < 1024) holds m = -inf, s = 0
    const float bm = block_max(m, red);
    s = block_sum(m == -INFINITY ? 0.f : s * exp_diff(m, bm), red);
    sx = block_sum(sx, red);
    if (threadIdx.x == 0) smoothing_row_result(bm, s, sx, x, t, V, confidence, smoothing, row_loss + r, lse + r);
}

// Any V and alignment: three strided passes over the row (the second and third are served by the caches
// for rows of ordinary length).
__global__ __launch_bounds__(SQ_THREADS) void label_smoothing_fwd_generic_kernel(
    const float* __restrict__ logits, const int64_t* __restrict__ target, float* __restrict__ row_loss,
    float* __restrict__ lse, int V, int64_t ld, int64_t padding_idx, float confidence, float smoothing) {
    __shared__ float red[SQ_WAVES];
    const int r = blockIdx.x;
    const int64_t t = target[r];
    if (t == padding_idx) {
        if (threadIdx.x == 0) { row_loss[r] = 0.f; lse[r] = 0.f; }
        return;
    }
    const float* x = logits + (int64_t)r * ld;
    float m = -INFINITY;
    for (int c = threadIdx.x; c < V; c += SQ_THREADS) m = fmaxf(m, x[c]);
    m = block_max(m, red);
    float s = 0.f, sx = 0.f;
    for (int c = threadIdx.x; c < V; c += SQ_THREADS) {
        s += exp_diff(x[c], m);
        sx += x[c];
    }
    s = block_sum(s, red);
    sx = block_sum(sx, red);
    if (threadIdx.x == 0) smoothing_row_result(m, s, sx, x, t, V, confidence, smoothing, row_loss + r, lse + r);
}

// loss = sum(row_loss) / divisor, added in a fixed order (one block).
__global__ __launch_bounds__(SQ_THREADS) void label_smoothing_sum_kernel(const float* __restrict__ row_loss,
                                                                         float* __restrict__ loss, int R,
                                                                         float divisor) {
    __shared__ float red[SQ_WAVES];
    float t[4] = {0.f, 0.f, 0.f, 0.f};
    int r = threadIdx.x;
    for (; r + 3 * SQ_THREADS < R; r += 4 * SQ_THREADS)
#pragma unroll
        for (int u = 0; u < 4; ++u) t[u] += row_loss[r + u * SQ_THREADS];
    for (; r < R; r += SQ_THREADS) t[0] += row_loss[r];
    const float s = block_sum((t[0] + t[1]) + (t[2] + t[3]), red);
    if (threadIdx.x == 0) loss[0] = s / divisor;
}

// dlogits[r][c] = (softmax(x_r)[c] - confidence * [c == target_r] - smoothing / V) * grad_loss / divisor,
// 0 for padding rows.  grid = (ceil(V / 4 / 256), R); VEC: 4 | V and 16-byte aligned rows on both sides.
template <bool VEC>
__global__ __launch_bounds__(SQ_THREADS) void label_smoothing_bwd_kernel(
    const float* __restrict__ logits, const int64_t* __restrict__ target, const float* __restrict__ lse,
    const float* __restrict__ grad_loss, float* __restrict__ dlogits, int V, int64_t ld, int64_t ldd,
    int64_t padding_idx, float confidence, float smoothing, float divisor) {
    const int r = blockIdx.y;
    const int c = (blockIdx.x * SQ_THREADS + threadIdx.x) * 4;
    if (c >= V) return;
    const int64_t t = target[r];
    const float* x = logits + (int64_t)r * ld;
    float* d = dlogits + (int64_t)r * ldd;
    const bool pad = t == padding_idx;
    const float scale = grad_loss[0] / divisor;
    const float l = lse[r];
    const float uniform = smoothing / (float)V;
    if (VEC) {
        float4_t o = {0.f, 0.f, 0.f, 0.f};
        if (!pad) {
            const float4_t v = *(const float4_t*)(x + c);
#pragma unroll
            for (int k = 0; k < 4; ++k)
                o[k] = (exp_diff(v[k], l) - (c + k == t ? confidence : 0.f) - uniform) * scale;
        }
        *(float4_t*)(d + c) = o;
    } else {
        for (int k = c; k < V && k < c + 4; ++k)
            d[k] = pad ? 0.f : (exp_diff(x[k], l) - (k == t ? confidence : 0.f) - uniform) * scale;
    }
}

// out[t][b][:] = t < len[b] ? in[src(t, b)][b][:] : 0 with src = len[b] - 1 - t (REVERSE) or t.
// Rows are row_units units of type VT long and in_pitch / out_pitch units apart (a row may be one half of
// a wider row: the two directions of a bidirectional layer side by side);
// grid = (ceil(row_units / 256), B, T).  in == out is allowed only without REVERSE.  A length above T is the caller's mistake; positions whose source row would lie
// behind the tensor read as 0.
template <typename VT, bool REVERSE>
__global__ __launch_bounds__(SQ_THREADS) void varlen_kernel(const VT* __restrict__ in, VT* __restrict__ out,
                                                            const int64_t* __restrict__ lengths, int B,
                                                            int T, int64_t row_units, int64_t in_pitch,
                                                            int64_t out_pitch) {
    const int64_t u = (int64_t)blockIdx.x * SQ_THREADS + threadIdx.x;
    if (u >= row_units) return;
    const int b = blockIdx.y, t = blockIdx.z;
    const int64_t len = lengths[b];
    VT v = {};
    if (t < len) {
        const int64_t src = REVERSE ? len - 1 - t : t;
        if (src < T) v = in[(src * B + b) * in_pitch + u];
    }
    out[((int64_t)t * B + b) * out_pitch + u] = v;
}

template <bool REVERSE>
int varlen_launch(const char* who, const void* in, void* out, const int64_t* lengths, int64_t T, int64_t B,
                  int64_t row_bytes, int64_t in_pitch, int64_t out_pitch, hipStream_t s) {
    PD_REQUIRE(T >= 0 && B >= 0 && row_bytes >= 0, PD_ESHAPE, "%s: negative dimension", who);
    PD_REQUIRE(in_pitch >= row_bytes && out_pitch >= row_bytes, PD_ESHAPE, "%s: row pitch below the row length",
               who);
    if (T == 0 || B == 0 || row_bytes == 0) return PD_OK;
    PD_REQUIRE(in && out && lengths, PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE(REVERSE ? in != out : true, PD_EINVAL, "%s: cannot reverse in place", who);
    PD_REQUIRE(B <= 65535 && T <= 65535, PD_ESHAPE, "%s: T and B must be <= 65535 (T=%ld B=%ld)", who, (long)T,
               (long)B);
    auto fits = [&](int64_t a) {
        return row_bytes % a == 0 && in_pitch % a == 0 && out_pitch % a == 0 && pd_aligned(in, (size_t)a) &&
               pd_aligned(out, (size_t)a);
    };
    PD_REQUIRE(fits(2), PD_EINVAL, "%s: rows and pitches must be whole numbers of 2-byte elements", who);
    const int unit = fits(16) ? 16 : fits(4) ? 4 : 2;
    const int64_t units = row_bytes / unit, ip = in_pitch / unit, op = out_pitch / unit;
    PD_REQUIRE((units + SQ_THREADS - 1) / SQ_THREADS <= 0x7fffffffL, PD_ESHAPE, "%s: rows too long", who);
    const dim3 grid((unsigned)((units + SQ_THREADS - 1) / SQ_THREADS), (unsigned)B, (unsigned)T);
    if (unit == 16)
        varlen_kernel<uint4_t, REVERSE><<<grid, SQ_THREADS, 0, s>>>((const uint4_t*)in, (uint4_t*)out, lengths,
                                                                  (int)B, (int)T, units, ip, op);
    else if (unit == 4)
        varlen_kernel<uint32_t, REVERSE><<<grid, SQ_THREADS, 0, s>>>((const uint32_t*)in, (uint32_t*)out, lengths,
                                                                   (int)B, (int)T, units, ip, op);
    else
        varlen_kernel<uint16_t, REVERSE><<<grid, SQ_THREADS, 0, s>>>((const uint16_t*)in, (uint16_t*)out, lengths,
                                                                   (int)B, (int)T, units, ip, op);
    PD_CHECK_LAUNCH(who);
    return PD_OK;
}

}  // namespace

extern "C" int pd_label_smoothing_fwd_f32(const float* logits, const int64_t* target, float* loss, float* row_loss,
                                          float* lse, int R, int V, int64_t ld, int64_t padding_idx,
                                          float smoothing, float divisor, void* stream) {
    const char* who = "pd_label_smoothing_fwd_f32";
    PD_REQUIRE(R > 0 && V > 0, PD_ESHAPE, "%s: empty row or class dimension", who);
    PD_REQUIRE(logits && target && loss && row_loss && lse, PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE(ld >= V, PD_ESHAPE, "%s: ld < V", who);
    PD_REQUIRE(divisor > 0.f, PD_EINVAL, "%s: divisor must be positive", who);
    hipStream_t s = (hipStream_t)stream;
    const float confidence = 1.f - smoothing;
    const bool vec = V % 4 == 0 && ld % 4 == 0 && pd_aligned(logits, 16);
    if (vec)
        label_smoothing_fwd_kernel<<<dim3(R), SQ_THREADS, 0, s>>>(logits, target, row_loss, lse, V, ld, padding_idx,
                                                               confidence, smoothing);
    else
        label_smoothing_fwd_generic_kernel<<<dim3(R), SQ_THREADS, 0, s>>>(logits, target, row_loss, lse, V, ld,
                                                                          padding_idx, confidence, smoothing);
    PD_CHECK_LAUNCH(who);
    label_smoothing_sum_kernel<<<dim3(1), SQ_THREADS, 0, s>>>(row_loss, loss, R, divisor);
    PD_CHECK_LAUNCH("pd_label_smoothing_fwd_f32(sum)");
    return PD_OK;
}

extern "C" int pd_label_smoothing_bwd_f32(const float* logits, const int64_t* target, const float* lse,
                                          const float* grad_loss, float* dlogits, int R, int V, int64_t ld,
                                          int64_t ldd, int64_t padding_idx, float smoothing, float divisor,
                                          void* stream) {
    const char* who = "pd_label_smoothing_bwd_f32";
    PD_REQUIRE(R > 0 && V > 0, PD_ESHAPE, "%s: empty row or class dimension", who);
    PD_REQUIRE(R <= 65535 * 32768L, PD_ESHAPE, "%s: too many rows", who);
    PD_REQUIRE(logits && target && lse && grad_loss && dlogits, PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE(ld >= V && ldd >= V, PD_ESHAPE, "%s: leading dimension < V", who);
    PD_REQUIRE(divisor > 0.f, PD_EINVAL, "%s: divisor must be positive", who);
    const float confidence = 1.f - smoothing;
    const bool vec = V % 4 == 0 && ld % 4 == 0 && ldd % 4 == 0 && pd_aligned(logits, 16) && pd_aligned(dlogits, 16);
    const unsigned bx = (unsigned)(((V + 3) / 4 + SQ_THREADS - 1) / SQ_THREADS);
    hipStream_t s = (hipStream_t)stream;
    // grid.y is limited to 65535 rows per launch
    for (int r0 = 0; r0 < R; r0 += 65535) {
        const int rows = R - r0 < 65535 ? R - r0 : 65535;
        const dim3 grid(bx, (unsigned)rows);
        if (vec)
            label_smoothing_bwd_kernel<true><<<grid, SQ_THREADS, 0, s>>>(
                logits + (int64_t)r0 * ld, target + r0, lse + r0, grad_loss, dlogits + (int64_t)r0 * ldd, V, ld, ldd,
                padding_idx, confidence, smoothing, divisor);
        else
            label_smoothing_bwd_kernel<false><<<grid, SQ_THREADS, 0, s>>>(
                logits + (int64_t)r0 * ld, target + r0, lse + r0, grad_loss, dlogits + (int64_t)r0 * ldd, V, ld, ldd,
                padding_idx, confidence, smoothing, divisor);
        PD_CHECK_LAUNCH(who);
    }
    return PD_OK;
}

extern "C" int pd_revert_varlen(const void* in, void* out, const int64_t* lengths, int64_t T, int64_t B,
                                int64_t row_bytes, int64_t in_pitch, int64_t out_pitch, void* stream) {
    return varlen_launch<true>("pd_revert_varlen", in, out, lengths, T, B, row_bytes, in_pitch, out_pitch,
                               (hipStream_t)stream);
}

extern "C" int pd_length_mask_apply(const void* in, void* out, const int64_t* lengths, int64_t T, int64_t B,
                                    int64_t row_bytes, int64_t in_pitch, int64_t out_pitch, void* stream) {
    return varlen_launch<false>("pd_length_mask_apply", in, out, lengths, T, B, row_bytes, in_pitch, out_pitch,
                                (hipStream_t)stream);
}

// Host code, like the function it stands in for: lengths and mask are host memory.
extern "C" int pd_set_mask_u8(const int64_t* lengths, int64_t B, int64_t T, uint8_t* mask) {
    PD_REQUIRE(B >= 0 && T >= 0, PD_ESHAPE, "pd_set_mask_u8: negative dimension");
    if (B == 0 || T == 0) return PD_OK;
    PD_REQUIRE(lengths && mask, PD_EINVAL, "pd_set_mask_u8: NULL pointer");
    for (int64_t t = 0; t < T; ++t)
        for (int64_t b = 0; b < B; ++b) mask[t * B + b] = lengths[b] > t ? 1 : 0;
    return PD_OK;
}
