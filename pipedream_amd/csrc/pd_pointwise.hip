// HBM-bound epilogue kernels of a stage: ReLU, 2x2 max-pooling (NHWC) and the
// softmax cross-entropy criterion, forward and backward.
//
// They stand in for the torch.nn.ReLU / MaxPool2d modules of the reference's
// generated stages (runtime/image_classification/models/vgg16/gpus=4_straight/
// stage0.py:13, stage1.py:10-11) and for the nn.CrossEntropyLoss criterion the
// caller appends as the last module
// (runtime/image_classification/main_with_runtime.py:126; runtime/runtime.py:523-526).
//
// Algorithmic traffic: every activation byte is read once and written once.
#include "pd_internal.h"

typedef float float4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int PW_THREADS = 256;

// ---- ReLU -----------------------------------------------------------------------
__global__ __launch_bounds__(PW_THREADS) void relu_fwd_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                              uint64_t n, bool vec) {
    uint64_t i = ((uint64_t)blockIdx.x * PW_THREADS + threadIdx.x) * 4;
    if (i >= n) return;
    if (vec && i + 3 < n) {
        float4_t v = *(const float4_t*)(x + i);
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = v[k] > 0.f ? v[k] : 0.f;
        *(float4_t*)(y + i) = v;
    } else {
        for (uint64_t k = i; k < n && k < i + 4; ++k) y[k] = x[k] > 0.f ? x[k] : 0.f;
    }
}

// dx = dy where the forward OUTPUT is positive (same mask as "input > 0").
__global__ __launch_bounds__(PW_THREADS) void relu_bwd_kernel(const float* __restrict__ dy, const float* __restrict__ y,
                                                              float* __restrict__ dx, uint64_t n, bool vec) {
    uint64_t i = ((uint64_t)blockIdx.x * PW_THREADS + threadIdx.x) * 4;
    if (i >= n) return;
    if (vec && i + 3 < n) {
        float4_t g = *(const float4_t*)(dy + i);
        float4_t o = *(const float4_t*)(y + i);
#pragma unroll
        for (int k = 0; k < 4; ++k) g[k] = o[k] > 0.f ? g[k] : 0.f;
        *(float4_t*)(dx + i) = g;
    } else {
        for (uint64_t k = i; k < n && k < i + 4; ++k) dx[k] = y[k] > 0.f ? dy[k] : 0.f;
    }
}

// ---- dropout: y = x * mask * scale (mask is 0/1 bytes) --------------------------------
__global__ __launch_bounds__(PW_THREADS) void mask_scale_kernel(const float* __restrict__ x,
                                                                const uint8_t* __restrict__ mask,
                                                                float* __restrict__ y, uint64_t n, float scale) {
    uint64_t i = (uint64_t)blockIdx.x * PW_THREADS + threadIdx.x;
    if (i < n) y[i] = mask[i] ? x[i] * scale : 0.f;
}

// ---- 2x2 / stride-2 max pooling, NHWC ---------------------------------------------
// One thread handles 4 consecutive channels of one output pixel.  Ties go to the first
// maximum in window scan order (dy=0,dx=0 -> 0,1 -> 1,0 -> 1,1) and NaNs win, which is
// the rule of torch's max_pool2d.
__device__ __forceinline__ bool pool_better(float v, float best) { return v > best || v != v; }

__global__ __launch_bounds__(PW_THREADS) void maxpool2_fwd_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                                  int N, int H, int W, int C, int relu) {
    const int Ho = H / 2, Wo = W / 2, C4 = C / 4;
    uint64_t id = (uint64_t)blockIdx.x * PW_THREADS + threadIdx.x;
    uint64_t total = (uint64_t)N * Ho * Wo * C4;
    if (id >= total) return;
    int c4 = id % C4;
    uint64_t p = id / C4;
    int ox = p % Wo;
    p /= Wo;
    int oy = p % Ho;
    int n = p / Ho;
    const float* base = x + (((uint64_t)n * H + 2 * oy) * W + 2 * ox) * C + c4 * 4;
    float4_t best = *(const float4_t*)base;
    float4_t v1 = *(const float4_t*)(base + C);
    float4_t v2 = *(const float4_t*)(base + (uint64_t)W * C);
    float4_t v3 = *(const float4_t*)(base + (uint64_t)W * C + C);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        if (pool_better(v1[k], best[k])) best[k] = v1[k];
        if (pool_better(v2[k], best[k])) best[k] = v2[k];
        if (pool_better(v3[k], best[k])) best[k] = v3[k];
        // ReLU commutes with max: relu(max(window)) == max(relu(window))
        if (relu && best[k] < 0.f) best[k] = 0.f;
    }
    *(float4_t*)(y + (((uint64_t)n * Ho + oy) * Wo + ox) * C + c4 * 4) = best;
}

// dx has the input's shape; every input element belongs to exactly one window (rows/cols
// beyond 2*floor(H/2) belong to none and get 0), so dx is written, not accumulated.
// If relu_mask is set the pooled input was a ReLU output and dx is additionally zeroed
// where x <= 0 (the ReLU backward fused in).
__global__ __launch_bounds__(PW_THREADS) void maxpool2_bwd_kernel(const float* __restrict__ x,
                                                                  const float* __restrict__ dy, float* __restrict__ dx,
                                                                  int N, int H, int W, int C, int relu_mask) {
    const int Ho = H / 2, Wo = W / 2, C4 = C / 4;
    const int Hc = (H + 1) / 2, Wc = (W + 1) / 2;  // windows incl. the ragged edge
    uint64_t id = (uint64_t)blockIdx.x * PW_THREADS + threadIdx.x;
    uint64_t total = (uint64_t)N * Hc * Wc * C4;
    if (id >= total) return;
    int c4 = id % C4;
    uint64_t p = id / C4;
    int ox = p % Wc;
    p /= Wc;
    int oy = p % Hc;
    int n = p / Hc;
    const bool inside = oy < Ho && ox < Wo;
    const uint64_t off = (((uint64_t)n * H + 2 * oy) * W + 2 * ox) * C + c4 * 4;
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    const bool has_x1 = 2 * ox + 1 < W, has_y1 = 2 * oy + 1 < H;
    if (!inside) {
        *(float4_t*)(dx + off) = zero;
        if (has_x1) *(float4_t*)(dx + off + C) = zero;
        if (has_y1) *(float4_t*)(dx + off + (uint64_t)W * C) = zero;
        if (has_x1 && has_y1) *(float4_t*)(dx + off + (uint64_t)W * C + C) = zero;
        return;
    }
    float4_t v[4];
    v[0] = *(const float4_t*)(x + off);
    v[1] = *(const float4_t*)(x + off + C);
    v[2] = *(const float4_t*)(x + off + (uint64_t)W * C);
    v[3] = *(const float4_t*)(x + off + (uint64_t)W * C + C);
    float4_t g = *(const float4_t*)(dy + (((uint64_t)n * Ho + oy) * Wo + ox) * C + c4 * 4);
    float4_t o[4] = {zero, zero, zero, zero};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        int arg = 0;
        float best = v[0][k];
#pragma unroll
        for (int j = 1; j < 4; ++j)
            if (pool_better(v[j][k], best)) {
                best = v[j][k];
                arg = j;
            }
        float gk = g[k];
        if (relu_mask && !(best > 0.f)) gk = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j][k] = (j == arg) ? gk : 0.f;
    }
    *(float4_t*)(dx + off) = o[0];
    *(float4_t*)(dx + off + C) = o[1];
    *(float4_t*)(dx + off + (uint64_t)W * C) = o[2];
    *(float4_t*)(dx + off + (uint64_t)W * C + C) = o[3];
}

// ---- the same pooling with an index tensor ---------------------------------------------
// The forward also writes one byte per output element: bits 0-1 = position of the maximum in the window
// (scan order as above), bit 2 = "the maximum is positive".  The backward then needs the pooled gradient
// and that byte instead of the whole input: 4 + 1 bytes read per output element instead of 4 + 16.
__device__ __forceinline__ uint32_t pool_pick(float v0, float v1, float v2, float v3, float* best_out) {
    float best = v0;
    uint32_t arg = 0;
    if (pool_better(v1, best)) { best = v1; arg = 1; }
    if (pool_better(v2, best)) { best = v2; arg = 2; }
    if (pool_better(v3, best)) { best = v3; arg = 3; }
    *best_out = best;
    return arg | (best > 0.f ? 4u : 0u);
}

__global__ __launch_bounds__(PW_THREADS) void maxpool2_fwd_idx_kernel(const float* __restrict__ x,
                                                                      float* __restrict__ y,
                                                                      uint32_t* __restrict__ idx, int N, int H, int W,
                                                                      int C, int relu) {
    const int Ho = H / 2, Wo = W / 2, C4 = C / 4;
    uint64_t id = (uint64_t)blockIdx.x * PW_THREADS + threadIdx.x;
    uint64_t total = (uint64_t)N * Ho * Wo * C4;
    if (id >= total) return;
    int c4 = id % C4;
    uint64_t p = id / C4;
    int ox = p % Wo;
    p /= Wo;
    int oy = p % Ho;
    int n = p / Ho;
    const float* base = x + (((uint64_t)n * H + 2 * oy) * W + 2 * ox) * C + c4 * 4;
    const float4_t v0 = *(const float4_t*)base;
    const float4_t v1 = *(const float4_t*)(base + C);
    const float4_t v2 = *(const float4_t*)(base + (uint64_t)W * C);
    const float4_t v3 = *(const float4_t*)(base + (uint64_t)W * C + C);
    float4_t best;
    uint32_t packed = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float b;
        packed |= pool_pick(v0[k], v1[k], v2[k], v3[k], &b) << (8 * k);
        if (relu && b < 0.f) b = 0.f;
        best[k] = b;
    }
    const uint64_t o = (((uint64_t)n * Ho + oy) * Wo + ox) * C + c4 * 4;
    *(float4_t*)(y + o) = best;
    idx[o / 4] = packed;
}

// dx [N,H,W,C] from dy [N,H/2,W/2,C] and the index bytes: the window position named by the byte gets the
// gradient (0 if relu_mask is set and the maximum was not positive), the other three and the ragged edge 0.
__global__ __launch_bounds__(PW_THREADS) void maxpool2_bwd_idx_kernel(const float* __restrict__ dy,
                                                                      const uint32_t* __restrict__ idx,
                                                                      float* __restrict__ dx, int N, int H, int W, int C,
                                                                      int relu_mask) {
    const int Ho = H / 2, Wo = W / 2, C4 = C / 4;
    const int Hc = (H + 1) / 2, Wc = (W + 1) / 2;  // windows incl. the ragged edge
    uint64_t id = (uint64_t)blockIdx.x * PW_THREADS + threadIdx.x;
    uint64_t total = (uint64_t)N * Hc * Wc * C4;
    if (id >= total) return;
    int c4 = id % C4;
    uint64_t p = id / C4;
    int ox = p % Wc;
    p /= Wc;
    int oy = p % Hc;
    int n = p / Hc;
    const bool inside = oy < Ho && ox < Wo;
    const uint64_t off = (((uint64_t)n * H + 2 * oy) * W + 2 * ox) * C + c4 * 4;
    const bool has_x1 = 2 * ox + 1 < W, has_y1 = 2 * oy + 1 < H;
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    float4_t o[4] = {zero, zero, zero, zero};
    if (inside) {
        const uint64_t po = (((uint64_t)n * Ho + oy) * Wo + ox) * C + c4 * 4;
        const float4_t g = *(const float4_t*)(dy + po);
        const uint32_t packed = idx[po / 4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t b = (packed >> (8 * k)) & 0xffu;
            const float gk = (relu_mask && !(b & 4u)) ? 0.f : g[k];
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j][k] = (j == (int)(b & 3u)) ? gk : 0.f;
        }
    }
    *(float4_t*)(dx + off) = o[0];
    if (has_x1) *(float4_t*)(dx + off + C) = o[1];
    if (has_y1) *(float4_t*)(dx + off + (uint64_t)W * C) = o[2];
    if (has_x1 && has_y1) *(float4_t*)(dx + off + (uint64_t)W * C + C) = o[3];
}

// ---- softmax cross-entropy ------------------------------------------------------------
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

// One block per row: row max and log-sum-exp via wave shuffles + an LDS exchange between
// the 4 waves.  row_loss[b] = lse - x[target] (0 for ignored rows, NaN for a target outside [0, C)),
// lse[b] kept for backward.
__global__ __launch_bounds__(PW_THREADS) void xent_fwd_kernel(const float* __restrict__ logits,
                                                              const int64_t* __restrict__ target,
                                                              float* __restrict__ row_loss, float* __restrict__ lse,
                                                              int C, int ld, int64_t ignore_index) {
    __shared__ float red[4];
    const int b = blockIdx.x;
    const float* x = logits + (uint64_t)b * ld;
    const int w = threadIdx.x / 64, lane = threadIdx.x % 64;
    float m = -INFINITY;
    for (int c = threadIdx.x; c < C; c += PW_THREADS) m = fmaxf(m, x[c]);
    m = wave_max(m);
    if (lane == 0) red[w] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float s = 0.f;
    for (int c = threadIdx.x; c < C; c += PW_THREADS) s += expf(x[c] - m);
    s = wave_sum(s);
    if (lane == 0) red[w] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float tot = (red[0] + red[1]) + (red[2] + red[3]);
        float l = m + logf(tot);
        lse[b] = l;
        int64_t t = target[b];
        // a label outside [0, C) that is not the ignore index poisons the loss instead of reading out of bounds
        row_loss[b] = (t == ignore_index) ? 0.f : ((t >= 0 && t < C) ? l - x[t] : NAN);
    }
}

// loss = sum(row_loss) / count(target != ignore_index); also stores the count.
__global__ __launch_bounds__(PW_THREADS) void xent_mean_kernel(const float* __restrict__ row_loss,
                                                               const int64_t* __restrict__ target,
                                                               float* __restrict__ loss, float* __restrict__ count_out,
                                                               int B, int64_t ignore_index) {
    __shared__ float red[2][4];
    float s = 0.f, n = 0.f;
    for (int b = threadIdx.x; b < B; b += PW_THREADS) {
        s += row_loss[b];
        n += (target[b] != ignore_index) ? 1.f : 0.f;
    }
    s = wave_sum(s);
    n = wave_sum(n);
    const int w = threadIdx.x / 64;
    if (threadIdx.x % 64 == 0) {
        red[0][w] = s;
        red[1][w] = n;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float ts = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
        float tn = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
        loss[0] = ts / tn;
        count_out[0] = tn;
    }
}

// dlogits[b][c] = (softmax - onehot) * grad_loss / count      (0 for ignored rows)
__global__ __launch_bounds__(PW_THREADS) void xent_bwd_kernel(const float* __restrict__ logits,
                                                              const int64_t* __restrict__ target,
                                                              const float* __restrict__ lse,
                                                              const float* __restrict__ grad_loss,
                                                              const float* __restrict__ count, float* __restrict__ dx,
                                                              int C, int ld, int ldd, int64_t ignore_index) {
    const int b = blockIdx.x;
    const float* x = logits + (uint64_t)b * ld;
    float* d = dx + (uint64_t)b * ldd;
    const int64_t t = target[b];
    const float scale = grad_loss[0] / count[0];
    const float l = lse[b];
    for (int c = threadIdx.x; c < C; c += PW_THREADS) {
        float v = 0.f;
        if (t != ignore_index) v = (expf(x[c] - l) - (c == t ? 1.f : 0.f)) * scale;
        d[c] = v;
    }
}

// Column sums of a row-major [M][N] matrix, split over gridDim.y row ranges:
// out[split][col].  (bias gradients: Linear db = sum_b dY, conv db = sum_{n,h,w} dY.)
__global__ __launch_bounds__(PW_THREADS) void colsum_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                            uint64_t M, int N, uint64_t ld, float beta) {
    __shared__ float part[4][64];
    const int col = blockIdx.x * 64 + threadIdx.x % 64;
    const int w = threadIdx.x / 64;
    const uint64_t rows_per = (M + gridDim.y - 1) / gridDim.y;
    const uint64_t r0 = blockIdx.y * rows_per;
    const uint64_t r1 = (r0 + rows_per < M) ? r0 + rows_per : M;
    float s = 0.f;
    if (col < N) {
        // 8 independent loads in flight per lane (a chain of dependent adds would be latency-bound);
        // the order of the additions is fixed, so the result is reproducible
        float t[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        uint64_t r = r0 + w;
        for (; r + 28 < r1; r += 32)
#pragma unroll
            for (int u = 0; u < 8; ++u) t[u] += x[(r + 4 * u) * ld + col];
        for (; r < r1; r += 4) t[0] += x[r * ld + col];
        s = ((t[0] + t[1]) + (t[2] + t[3])) + ((t[4] + t[5]) + (t[6] + t[7]));
    }
    part[w][threadIdx.x % 64] = s;
    __syncthreads();
    if (w == 0 && col < N) {
        float t = (part[0][threadIdx.x] + part[1][threadIdx.x]) + (part[2][threadIdx.x] + part[3][threadIdx.x]);
        float* o = out + (uint64_t)blockIdx.y * N + col;
        *o = beta != 0.f ? t + beta * *o : t;
    }
}

int blocks_for(uint64_t work_items, unsigned* out) {
    uint64_t b = (work_items + PW_THREADS - 1) / PW_THREADS;
    if (b > 0x7fffffffull) return -1;
    *out = (unsigned)b;
    return 0;
}

}  // namespace

extern "C" int pd_relu_fwd_f32(const float* x, float* y, uint64_t n, void* stream) {
    if (n == 0) return PD_OK;
    PD_REQUIRE(x && y, PD_EINVAL, "pd_relu_fwd_f32: NULL pointer");
    unsigned blocks;
    PD_REQUIRE(blocks_for((n + 3) / 4, &blocks) == 0, PD_ESHAPE, "pd_relu_fwd_f32: too large");
    bool vec = pd_aligned(x, 16) && pd_aligned(y, 16);
    relu_fwd_kernel<<<dim3(blocks), dim3(PW_THREADS), 0, (hipStream_t)stream>>>(x, y, n, vec);
    PD_CHECK_LAUNCH("pd_relu_fwd_f32");
    return PD_OK;
}

extern "C" int pd_relu_bwd_f32(const float* dy, const float* y, float* dx, uint64_t n, void* stream) {
    if (n == 0) return PD_OK;
    PD_REQUIRE(dy && y && dx, PD_EINVAL, "pd_relu_bwd_f32: NULL pointer");
    unsigned blocks;
    PD_REQUIRE(blocks_for((n + 3) / 4, &blocks) == 0, PD_ESHAPE, "pd_relu_bwd_f32: too large");
    bool vec = pd_aligned(dy, 16) && pd_aligned(y, 16) && pd_aligned(dx, 16);
    relu_bwd_kernel<<<dim3(blocks), dim3(PW_THREADS), 0, (hipStream_t)stream>>>(dy, y, dx, n, vec);
    PD_CHECK_LAUNCH("pd_relu_bwd_f32");
    return PD_OK;
}

extern "C" int pd_mask_scale_f32(const float* x, const uint8_t* mask, float* y, uint64_t n, float scale, void* stream) {
    if (n == 0) return PD_OK;
    PD_REQUIRE(x && mask && y, PD_EINVAL, "pd_mask_scale_f32: NULL pointer");
    unsigned blocks;
    PD_REQUIRE(blocks_for(n, &blocks) == 0, PD_ESHAPE, "pd_mask_scale_f32: too large");
    mask_scale_kernel<<<dim3(blocks), dim3(PW_THREADS), 0, (hipStream_t)stream>>>(x, mask, y, n, scale);
    PD_CHECK_LAUNCH("pd_mask_scale_f32");
    return PD_OK;
}

extern "C" int pd_maxpool2x2_fwd_nhwc_f32(const float* x, float* y, int N, int H, int W, int C, int relu,
                                          void* stream) {
    PD_REQUIRE(N >= 0 && H >= 0 && W >= 0 && C >= 0, PD_ESHAPE, "pd_maxpool2x2_fwd: negative dimension");
    PD_REQUIRE(C % 4 == 0, PD_ESHAPE, "pd_maxpool2x2_fwd: channels must be a multiple of 4 (got %d)", C);
    uint64_t total = (uint64_t)N * (H / 2) * (W / 2) * (C / 4);
    if (total == 0) return PD_OK;
    PD_REQUIRE(x && y, PD_EINVAL, "pd_maxpool2x2_fwd: NULL pointer");
    PD_REQUIRE(pd_aligned(x, 16) && pd_aligned(y, 16), PD_EINVAL, "pd_maxpool2x2_fwd: pointers must be 16-byte aligned");
    unsigned blocks;
    PD_REQUIRE(blocks_for(total, &blocks) == 0, PD_ESHAPE, "pd_maxpool2x2_fwd: too large");
    maxpool2_fwd_kernel<<<dim3(blocks), dim3(PW_THREADS), 0, (hipStream_t)stream>>>(x, y, N, H, W, C, relu);
    PD_CHECK_LAUNCH("pd_maxpool2x2_fwd");
    return PD_OK;
}

extern "C" int pd_maxpool2x2_bwd_nhwc_f32(const float* x, const float* dy, float* dx, int N, int H, int W, int C,
                                          int relu_mask, void* stream) {
    PD_REQUIRE(N >= 0 && H >= 0 && W >= 0 && C >= 0, PD_ESHAPE, "pd_maxpool2x2_bwd: negative dimension");
    PD_REQUIRE(C % 4 == 0, PD_ESHAPE, "pd_maxpool2x2_bwd: channels must be a multiple of 4 (got %d)", C);
    uint64_t total = (uint64_t)N * ((H + 1) / 2) * ((W + 1) / 2) * (C / 4);
    if (total == 0) return PD_OK;
    PD_REQUIRE(x && dy && dx, PD_EINVAL, "pd_maxpool2x2_bwd: NULL pointer");
    PD_REQUIRE(pd_aligned(x, 16) && pd_aligned(dy, 16) && pd_aligned(dx, 16), PD_EINVAL,
               "pd_maxpool2x2_bwd: pointers must be 16-byte aligned");
    unsigned blocks;
    PD_REQUIRE(blocks_for(total, &blocks) == 0, PD_ESHAPE, "pd_maxpool2x2_bwd: too large");
    maxpool2_bwd_kernel<<<dim3(blocks), dim3(PW_THREADS), 0, (hipStream_t)stream>>>(x, dy, dx, N, H, W, C, relu_mask);
    PD_CHECK_LAUNCH("pd_maxpool2x2_bwd");
    return PD_OK;
}

extern "C" int pd_maxpool2x2_fwd_idx_nhwc_f32(const float* x, float* y, uint8_t* idx, int N, int H, int W, int C,
                                              int relu, void* stream) {
    const char* who = "pd_maxpool2x2_fwd_idx";
    PD_REQUIRE(N >= 0 && H >= 0 && W >= 0 && C >= 0, PD_ESHAPE, "%s: negative dimension", who);
    PD_REQUIRE(C % 4 == 0, PD_ESHAPE, "%s: channels must be a multiple of 4 (got %d)", who, C);
    uint64_t total = (uint64_t)N * (H / 2) * (W / 2) * (C / 4);
    if (total == 0) return PD_OK;
    PD_REQUIRE(x && y && idx, PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE(pd_aligned(x, 16) && pd_aligned(y, 16) && pd_aligned(idx, 4), PD_EINVAL,
               "%s: tensors must be 16-byte aligned (index bytes: 4)", who);
    unsigned blocks;
    PD_REQUIRE(blocks_for(total, &blocks) == 0, PD_ESHAPE, "%s: too large", who);
    maxpool2_fwd_idx_kernel<<<dim3(blocks), dim3(PW_THREADS), 0, (hipStream_t)stream>>>(x, y, (uint32_t*)idx, N, H, W,
                                                                                    C, relu);
    PD_CHECK_LAUNCH(who);
    return PD_OK;
}

extern "C" int pd_maxpool2x2_bwd_idx_nhwc_f32(const float* dy, const uint8_t* idx, float* dx, int N, int H, int W,
                                              int C, int relu_mask, void* stream) {
    const char* who = "pd_maxpool2x2_bwd_idx";
    PD_REQUIRE(N >= 0 && H >= 0 && W >= 0 && C >= 0, PD_ESHAPE, "%s: negative dimension", who);
    PD_REQUIRE(C % 4 == 0, PD_ESHAPE, "%s: channels must be a multiple of 4 (got %d)", who, C);
    uint64_t total = (uint64_t)N * ((H + 1) / 2) * ((W + 1) / 2) * (C / 4);
    if (total == 0) return PD_OK;
    PD_REQUIRE(dx, PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE((dy && idx) || (uint64_t)(H / 2) * (W / 2) == 0, PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE(pd_aligned(dy, 16) && pd_aligned(dx, 16) && pd_aligned(idx, 4), PD_EINVAL,
               "%s: tensors must be 16-byte aligned (index bytes: 4)", who);
    unsigned blocks;
    PD_REQUIRE(blocks_for(total, &blocks) == 0, PD_ESHAPE, "%s: too large", who);
    maxpool2_bwd_idx_kernel<<<dim3(blocks), dim3(PW_THREADS), 0, (hipStream_t)stream>>>(dy, (const uint32_t*)idx, dx, N,
                                                                                    H, W, C, relu_mask);
    PD_CHECK_LAUNCH(who);
    return PD_OK;
}

extern "C" int pd_xent_fwd_f32(const float* logits, const int64_t* target, float* loss, float* row_loss, float* lse,
                               float* count, int B, int C, int ld, int64_t ignore_index, void* stream) {
    PD_REQUIRE(B > 0 && C > 0, PD_ESHAPE, "pd_xent_fwd_f32: empty batch or class dimension");
    PD_REQUIRE(logits && target && loss && row_loss && lse && count, PD_EINVAL, "pd_xent_fwd_f32: NULL pointer");
    PD_REQUIRE(ld >= C, PD_ESHAPE, "pd_xent_fwd_f32: ld < C");
    hipStream_t s = (hipStream_t)stream;
    xent_fwd_kernel<<<dim3(B), dim3(PW_THREADS), 0, s>>>(logits, target, row_loss, lse, C, ld, ignore_index);
    PD_CHECK_LAUNCH("pd_xent_fwd_f32");
    xent_mean_kernel<<<dim3(1), dim3(PW_THREADS), 0, s>>>(row_loss, target, loss, count, B, ignore_index);
    PD_CHECK_LAUNCH("pd_xent_fwd_f32(mean)");
    return PD_OK;
}

extern "C" int pd_xent_bwd_f32(const float* logits, const int64_t* target, const float* lse, const float* grad_loss,
                               const float* count, float* dlogits, int B, int C, int ld, int ldd,
                               int64_t ignore_index, void* stream) {
    PD_REQUIRE(B > 0 && C > 0, PD_ESHAPE, "pd_xent_bwd_f32: empty batch or class dimension");
    PD_REQUIRE(logits && target && lse && grad_loss && count && dlogits, PD_EINVAL, "pd_xent_bwd_f32: NULL pointer");
    PD_REQUIRE(ld >= C && ldd >= C, PD_ESHAPE, "pd_xent_bwd_f32: leading dimension < C");
    xent_bwd_kernel<<<dim3(B), dim3(PW_THREADS), 0, (hipStream_t)stream>>>(logits, target, lse, grad_loss, count,
                                                                         dlogits, C, ld, ldd, ignore_index);
    PD_CHECK_LAUNCH("pd_xent_bwd_f32");
    return PD_OK;
}

extern "C" int pd_colsum_f32(const float* x, float* out, uint64_t M, int N, uint64_t ld, int splits, float beta,
                             void* stream) {
    PD_REQUIRE(N >= 0 && splits >= 1 && splits <= 65535, PD_ESHAPE, "pd_colsum_f32: bad N or splits");
    if (N == 0) return PD_OK;
    PD_REQUIRE(x && out, PD_EINVAL, "pd_colsum_f32: NULL operand");
    PD_REQUIRE(ld >= (uint64_t)N, PD_ESHAPE, "pd_colsum_f32: ld < N");
    colsum_kernel<<<dim3((N + 63) / 64, splits), dim3(PW_THREADS), 0, (hipStream_t)stream>>>(x, out, M, N, ld, beta);
    PD_CHECK_LAUNCH("pd_colsum_f32");
    return PD_OK;
}
