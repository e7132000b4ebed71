// HBM-bound kernels of the bf16 transformer stage: LayerNorm, softmax, GELU (forward and
// backward), bf16 <-> fp32 casts, bf16 add and column sums.  bf16 in memory, fp32
// arithmetic; row reductions are wavefront reductions (one 64-lane wave per row, rows
// staged in registers), cross-wave sums go through LDS.
//
// No counterpart on the reference's checked-out branch (PipeDream-2BW is on another
// branch, README.md:7-8); they play the role of torch.nn.LayerNorm / softmax / GELU.
//
// Algorithmic traffic: each activation element is read once and written once per kernel
// (2 B each); LayerNorm backward reads x and dy and writes dx (6 B/element).
#include "pd_internal.h"

typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int TR_THREADS = 256;
constexpr int MAX_VEC = 4;   // rows up to 64 lanes * 8 elements * MAX_VEC = 2048 elements

__device__ __forceinline__ float bf2f(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
__device__ __forceinline__ uint16_t f2bf(float f) { return pd_f2bf(f); }
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// A row of `n` bf16 values held by one wave: vector v of lane l covers elements
// [(v*64 + l)*8, +8).
struct RowRegs {
    float x[MAX_VEC][8];
    int nvec;

    __device__ __forceinline__ void load(const uint16_t* __restrict__ row, int n, int lane) {
        nvec = (n + 511) / 512;
#pragma unroll
        for (int v = 0; v < MAX_VEC; ++v) {
            const int e = (v * 64 + lane) * 8;
            if (v < nvec && e < n) {
                const u16x8 r = *(const u16x8*)(row + e);
#pragma unroll
                for (int k = 0; k < 8; ++k) x[v][k] = bf2f(r[k]);
            } else {
#pragma unroll
                for (int k = 0; k < 8; ++k) x[v][k] = 0.f;
            }
        }
    }
};

__device__ __forceinline__ void store_row(uint16_t* __restrict__ row, int n, int lane, int v, const float (&y)[8]) {
    const int e = (v * 64 + lane) * 8;
    if (e < n) {
        u16x8 r;
#pragma unroll
        for (int k = 0; k < 8; ++k) r[k] = f2bf(y[k]);
        *(u16x8*)(row + e) = r;
    }
}

// ---- LayerNorm ------------------------------------------------------------------------
__global__ __launch_bounds__(TR_THREADS) void layernorm_fwd_kernel(const uint16_t* __restrict__ x,
                                                                   const float* __restrict__ gamma,
                                                                   const float* __restrict__ beta,
                                                                   uint16_t* __restrict__ y, float* __restrict__ mean,
                                                                   float* __restrict__ rstd, int M, int H, float eps) {
    const int lane = threadIdx.x % 64;
    const int row = blockIdx.x * 4 + threadIdx.x / 64;
    if (row >= M) return;
    RowRegs r;
    r.load(x + (size_t)row * H, H, lane);
    float s = 0.f;
#pragma unroll
    for (int v = 0; v < MAX_VEC; ++v)
#pragma unroll
        for (int k = 0; k < 8; ++k) s += r.x[v][k];
    const float mu = wave_sum(s) / (float)H;
    float q = 0.f;
#pragma unroll
    for (int v = 0; v < MAX_VEC; ++v)
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int e = (v * 64 + lane) * 8 + k;
            const float d = e < H ? r.x[v][k] - mu : 0.f;
            q += d * d;
        }
    const float rs = rsqrtf(wave_sum(q) / (float)H + eps);
    if (lane == 0) {
        mean[row] = mu;
        rstd[row] = rs;
    }
#pragma unroll
    for (int v = 0; v < MAX_VEC; ++v) {
        const int e = (v * 64 + lane) * 8;
        if (v < r.nvec && e < H) {
            float o[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) o[k] = (r.x[v][k] - mu) * rs * gamma[e + k] + beta[e + k];
            store_row(y + (size_t)row * H, H, lane, v, o);
        }
    }
}

// dx for each row; per-block partial sums of dgamma / dbeta over the block's rows.
// A block handles ROWS_PER_BLOCK rows, each wave every 4th of them.
constexpr int LN_ROWS_PER_BLOCK = 8;

__global__ __launch_bounds__(TR_THREADS) void layernorm_bwd_kernel(const uint16_t* __restrict__ dy,
                                                                   const uint16_t* __restrict__ x,
                                                                   const float* __restrict__ gamma,
                                                                   const float* __restrict__ mean,
                                                                   const float* __restrict__ rstd,
                                                                   uint16_t* __restrict__ dx,
                                                                   const uint16_t* __restrict__ residual,
                                                                   float* __restrict__ part_dgamma,
                                                                   float* __restrict__ part_dbeta, int M, int H) {
    extern __shared__ float red[];   // [2][4][H]
    const int lane = threadIdx.x % 64, w = threadIdx.x / 64;
    float dg[MAX_VEC][8], db[MAX_VEC][8];
#pragma unroll
    for (int v = 0; v < MAX_VEC; ++v)
#pragma unroll
        for (int k = 0; k < 8; ++k) dg[v][k] = db[v][k] = 0.f;
    const int nvec = (H + 511) / 512;
    for (int rr = w; rr < LN_ROWS_PER_BLOCK; rr += 4) {
        const int row = blockIdx.x * LN_ROWS_PER_BLOCK + rr;
        if (row >= M) break;
        RowRegs rx, rd;
        rx.load(x + (size_t)row * H, H, lane);
        rd.load(dy + (size_t)row * H, H, lane);
        const float mu = mean[row], rs = rstd[row];
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int v = 0; v < MAX_VEC; ++v) {
            const int e = (v * 64 + lane) * 8;
            if (v < nvec && e < H) {
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const float xh = (rx.x[v][k] - mu) * rs;
                    const float gdy = gamma[e + k] * rd.x[v][k];
                    s1 += gdy;
                    s2 += gdy * xh;
                    dg[v][k] += rd.x[v][k] * xh;
                    db[v][k] += rd.x[v][k];
                }
            }
        }
        s1 = wave_sum(s1) / (float)H;
        s2 = wave_sum(s2) / (float)H;
#pragma unroll
        for (int v = 0; v < MAX_VEC; ++v) {
            const int e = (v * 64 + lane) * 8;
            if (v < nvec && e < H) {
                float o[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const float xh = (rx.x[v][k] - mu) * rs;
                    o[k] = rs * (gamma[e + k] * rd.x[v][k] - s1 - xh * s2);
                }
                if (residual) {       // the gradient that reaches the layer's input past the normalisation
                    const u16x8 r = *(const u16x8*)(residual + (size_t)row * H + e);
#pragma unroll
                    for (int k = 0; k < 8; ++k) o[k] += bf2f(r[k]);
                }
                store_row(dx + (size_t)row * H, H, lane, v, o);
            }
        }
    }
    float* rg = red + (size_t)w * H;
    float* rb = red + (size_t)(4 + w) * H;
#pragma unroll
    for (int v = 0; v < MAX_VEC; ++v) {
        const int e = (v * 64 + lane) * 8;
        if (v < nvec && e < H) {
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                rg[e + k] = dg[v][k];
                rb[e + k] = db[v][k];
            }
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < H; e += TR_THREADS) {
        part_dgamma[(size_t)blockIdx.x * H + e] = (red[e] + red[H + e]) + (red[2 * H + e] + red[3 * H + e]);
        part_dbeta[(size_t)blockIdx.x * H + e] =
            (red[4 * H + e] + red[5 * H + e]) + (red[6 * H + e] + red[7 * H + e]);
    }
}

// ---- softmax over the last dimension ---------------------------------------------------------
__global__ __launch_bounds__(TR_THREADS) void softmax_fwd_kernel(const uint16_t* __restrict__ x,
                                                                 uint16_t* __restrict__ y, long long rows, int n) {
    const int lane = threadIdx.x % 64;
    const long long row = (long long)blockIdx.x * 4 + threadIdx.x / 64;
    if (row >= rows) return;
    RowRegs r;
    r.load(x + row * n, n, lane);
    float m = -INFINITY;
#pragma unroll
    for (int v = 0; v < MAX_VEC; ++v)
        if (v < r.nvec) {            // wave-uniform: rows shorter than 2048 skip the unused vectors
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if ((v * 64 + lane) * 8 + k < n) m = fmaxf(m, r.x[v][k]);
        }
    m = wave_max(m);
    float s = 0.f;
#pragma unroll
    for (int v = 0; v < MAX_VEC; ++v)
        if (v < r.nvec) {
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const bool in = (v * 64 + lane) * 8 + k < n;
                // e^(x-m) = 2^((x-m) log2 e) on the hardware exp2 (about 1 ulp; the result is rounded to bf16)
                r.x[v][k] = in ? __builtin_amdgcn_exp2f((r.x[v][k] - m) * 1.44269504088896340736f) : 0.f;
                s += r.x[v][k];
            }
        }
    const float inv = 1.0f / wave_sum(s);
#pragma unroll
    for (int v = 0; v < MAX_VEC; ++v) {
        if (v < r.nvec) {
            float o[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) o[k] = r.x[v][k] * inv;
            store_row(y + row * n, n, lane, v, o);
        }
    }
}

// dx = y * (dy - sum(dy * y))
__global__ __launch_bounds__(TR_THREADS) void softmax_bwd_kernel(const uint16_t* __restrict__ y,
                                                                 const uint16_t* __restrict__ dy,
                                                                 uint16_t* __restrict__ dx, long long rows, int n) {
    const int lane = threadIdx.x % 64;
    const long long row = (long long)blockIdx.x * 4 + threadIdx.x / 64;
    if (row >= rows) return;
    RowRegs ry, rd;
    ry.load(y + row * n, n, lane);
    rd.load(dy + row * n, n, lane);
    float s = 0.f;
#pragma unroll
    for (int v = 0; v < MAX_VEC; ++v)
        if (v < ry.nvec) {
#pragma unroll
            for (int k = 0; k < 8; ++k) s += ry.x[v][k] * rd.x[v][k];
        }
    s = wave_sum(s);
#pragma unroll
    for (int v = 0; v < MAX_VEC; ++v) {
        if (v < ry.nvec) {
            float o[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) o[k] = ry.x[v][k] * (rd.x[v][k] - s);
            store_row(dx + row * n, n, lane, v, o);
        }
    }
}

// ---- element-wise (8 bf16 per thread) ------------------------------------------------------
enum { EW_GELU_FWD, EW_GELU_BWD, EW_ADD };

template <int OP>
__global__ __launch_bounds__(TR_THREADS) void ew_bf16_kernel(const uint16_t* __restrict__ a,
                                                             const uint16_t* __restrict__ b,
                                                             uint16_t* __restrict__ y, uint64_t n) {
    const uint64_t i = ((uint64_t)blockIdx.x * TR_THREADS + threadIdx.x) * 8;
    if (i >= n) return;
    const u16x8 va = *(const u16x8*)(a + i);
    u16x8 vb = {0, 0, 0, 0, 0, 0, 0, 0};
    if (OP != EW_GELU_FWD) vb = *(const u16x8*)(b + i);
    u16x8 out;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float x = bf2f(va[k]);
        float r;
        if (OP == EW_GELU_FWD) {
            r = 0.5f * x * (1.0f + erff(x * 0.70710678118654752f));
        } else if (OP == EW_GELU_BWD) {   // a = pre-activation x, b = dy
            const float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752f));
            const float pdf = 0.39894228040143268f * expf(-0.5f * x * x);
            r = bf2f(vb[k]) * (cdf + x * pdf);
        } else {
            r = x + bf2f(vb[k]);
        }
        out[k] = f2bf(r);
    }
    *(u16x8*)(y + i) = out;
}

__global__ __launch_bounds__(TR_THREADS) void cast_f32_bf16_kernel(const float* __restrict__ x,
                                                                   uint16_t* __restrict__ y, uint64_t n) {
    const uint64_t i = ((uint64_t)blockIdx.x * TR_THREADS + threadIdx.x) * 4;
    if (i >= n) return;
    if (i + 3 < n) {
        const float4_t v = *(const float4_t*)(x + i);
        typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
        u16x4 o = {f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
        *(u16x4*)(y + i) = o;
    } else {
        for (uint64_t k = i; k < n; ++k) y[k] = f2bf(x[k]);
    }
}

__global__ __launch_bounds__(TR_THREADS) void cast_bf16_f32_kernel(const uint16_t* __restrict__ x,
                                                                   float* __restrict__ y, uint64_t n) {
    const uint64_t i = ((uint64_t)blockIdx.x * TR_THREADS + threadIdx.x) * 4;
    if (i >= n) return;
    for (uint64_t k = i; k < n && k < i + 4; ++k) y[k] = bf2f(x[k]);
}

// Column sums of a bf16 [M][N] matrix into fp32 partials out[split][N].  A lane owns 8
// adjacent columns (one 16-byte load per row), a block 512 columns; its 4 waves take every
// 4th row of the split and are combined through LDS in a fixed order.
__global__ __launch_bounds__(TR_THREADS) void colsum_bf16_kernel(const uint16_t* __restrict__ x,
                                                                 float* __restrict__ out, uint64_t M, int N,
                                                                 uint64_t ld, int vec) {
    __shared__ float part[4][512];
    const int lane = threadIdx.x % 64, w = threadIdx.x / 64;
    const int col = blockIdx.x * 512 + lane * 8;
    const uint64_t rows_per = (M + gridDim.y - 1) / gridDim.y;
    const uint64_t r0 = blockIdx.y * rows_per;
    const uint64_t r1 = (r0 + rows_per < M) ? r0 + rows_per : M;
    float s[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) s[k] = 0.f;
    if (vec && col + 8 <= N) {
        for (uint64_t r = r0 + w; r < r1; r += 4) {
            const u16x8 v = *(const u16x8*)(x + r * ld + col);
#pragma unroll
            for (int k = 0; k < 8; ++k) s[k] += bf2f(v[k]);
        }
    } else {
        for (uint64_t r = r0 + w; r < r1; r += 4)
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (col + k < N) s[k] += bf2f(x[r * ld + col + k]);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) part[w][lane * 8 + k] = s[k];
    __syncthreads();
    for (int c = threadIdx.x; c < 512; c += TR_THREADS) {
        const int gc = blockIdx.x * 512 + c;
        if (gc < N) out[(uint64_t)blockIdx.y * N + gc] = (part[0][c] + part[1][c]) + (part[2][c] + part[3][c]);
    }
}

int row_args_ok(const char* who, long long rows, int n) {
    PD_REQUIRE(rows > 0 && n > 0, PD_ESHAPE, "%s: empty input", who);
    PD_REQUIRE(n % 8 == 0 && n <= 64 * 8 * MAX_VEC, PD_ESHAPE, "%s: row length must be a multiple of 8 and <= %d", who,
               64 * 8 * MAX_VEC);
    PD_REQUIRE((rows + 3) / 4 <= 0x7fffffffLL, PD_ESHAPE, "%s: too many rows", who);
    return PD_OK;
}

}  // namespace

extern "C" int pd_layernorm_fwd_bf16(const uint16_t* x, const float* gamma, const float* beta, uint16_t* y, float* mean,
                                     float* rstd, int M, int H, float eps, void* stream) {
    int rc = row_args_ok("pd_layernorm_fwd_bf16", M, H);
    if (rc != PD_OK) return rc;
    PD_REQUIRE(x && gamma && beta && y && mean && rstd, PD_EINVAL, "pd_layernorm_fwd_bf16: NULL pointer");
    PD_REQUIRE(pd_aligned(x, 16) && pd_aligned(y, 16), PD_EINVAL, "pd_layernorm_fwd_bf16: 16-byte alignment");
    layernorm_fwd_kernel<<<dim3((M + 3) / 4), dim3(TR_THREADS), 0, (hipStream_t)stream>>>(x, gamma, beta, y, mean, rstd,
                                                                                         M, H, eps);
    PD_CHECK_LAUNCH("pd_layernorm_fwd_bf16");
    return PD_OK;
}

extern "C" int pd_layernorm_bwd_partials(int M) { return (M + LN_ROWS_PER_BLOCK - 1) / LN_ROWS_PER_BLOCK; }

extern "C" int pd_layernorm_bwd_bf16(const uint16_t* dy, const uint16_t* x, const float* gamma, const float* mean,
                                     const float* rstd, uint16_t* dx, const uint16_t* residual, float* part_dgamma,
                                     float* part_dbeta, int M, int H, void* stream) {
    int rc = row_args_ok("pd_layernorm_bwd_bf16", M, H);
    if (rc != PD_OK) return rc;
    PD_REQUIRE(dy && x && gamma && mean && rstd && dx && part_dgamma && part_dbeta, PD_EINVAL,
               "pd_layernorm_bwd_bf16: NULL pointer");
    PD_REQUIRE(pd_aligned(x, 16) && pd_aligned(dy, 16) && pd_aligned(dx, 16) && pd_aligned(residual, 16), PD_EINVAL,
               "pd_layernorm_bwd_bf16: 16-byte alignment");
    const size_t lds = (size_t)8 * H * sizeof(float);
    PD_REQUIRE(lds <= 160 * 1024, PD_ESHAPE, "pd_layernorm_bwd_bf16: H too large for the LDS reduction");
    if (lds > 64 * 1024)
        PD_HIP(hipFuncSetAttribute((const void*)layernorm_bwd_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)lds));
    layernorm_bwd_kernel<<<dim3(pd_layernorm_bwd_partials(M)), dim3(TR_THREADS), lds, (hipStream_t)stream>>>(
        dy, x, gamma, mean, rstd, dx, residual, part_dgamma, part_dbeta, M, H);
    PD_CHECK_LAUNCH("pd_layernorm_bwd_bf16");
    return PD_OK;
}

extern "C" int pd_softmax_fwd_bf16(const uint16_t* x, uint16_t* y, int64_t rows, int n, void* stream) {
    int rc = row_args_ok("pd_softmax_fwd_bf16", rows, n);
    if (rc != PD_OK) return rc;
    PD_REQUIRE(x && y, PD_EINVAL, "pd_softmax_fwd_bf16: NULL pointer");
    PD_REQUIRE(pd_aligned(x, 16) && pd_aligned(y, 16), PD_EINVAL, "pd_softmax_fwd_bf16: 16-byte alignment");
    softmax_fwd_kernel<<<dim3((unsigned)((rows + 3) / 4)), dim3(TR_THREADS), 0, (hipStream_t)stream>>>(x, y, rows, n);
    PD_CHECK_LAUNCH("pd_softmax_fwd_bf16");
    return PD_OK;
}

extern "C" int pd_softmax_bwd_bf16(const uint16_t* y, const uint16_t* dy, uint16_t* dx, int64_t rows, int n,
                                   void* stream) {
    int rc = row_args_ok("pd_softmax_bwd_bf16", rows, n);
    if (rc != PD_OK) return rc;
    PD_REQUIRE(y && dy && dx, PD_EINVAL, "pd_softmax_bwd_bf16: NULL pointer");
    PD_REQUIRE(pd_aligned(y, 16) && pd_aligned(dy, 16) && pd_aligned(dx, 16), PD_EINVAL,
               "pd_softmax_bwd_bf16: 16-byte alignment");
    softmax_bwd_kernel<<<dim3((unsigned)((rows + 3) / 4)), dim3(TR_THREADS), 0, (hipStream_t)stream>>>(y, dy, dx, rows, n);
    PD_CHECK_LAUNCH("pd_softmax_bwd_bf16");
    return PD_OK;
}

static int ew_launch(int op, const uint16_t* a, const uint16_t* b, uint16_t* y, uint64_t n, void* stream,
                     const char* who) {
    if (n == 0) return PD_OK;
    PD_REQUIRE(a && y && (op == EW_GELU_FWD || b), PD_EINVAL, "%s: NULL pointer", who);
    PD_REQUIRE(n % 8 == 0, PD_ESHAPE, "%s: element count must be a multiple of 8", who);
    PD_REQUIRE(pd_aligned(a, 16) && pd_aligned(y, 16) && (!b || pd_aligned(b, 16)), PD_EINVAL, "%s: 16-byte alignment",
               who);
    const uint64_t blocks = (n / 8 + TR_THREADS - 1) / TR_THREADS;
    PD_REQUIRE(blocks <= 0x7fffffffull, PD_ESHAPE, "%s: too large", who);
    hipStream_t s = (hipStream_t)stream;
    if (op == EW_GELU_FWD) ew_bf16_kernel<EW_GELU_FWD><<<dim3((unsigned)blocks), dim3(TR_THREADS), 0, s>>>(a, b, y, n);
    else if (op == EW_GELU_BWD) ew_bf16_kernel<EW_GELU_BWD><<<dim3((unsigned)blocks), dim3(TR_THREADS), 0, s>>>(a, b, y, n);
    else ew_bf16_kernel<EW_ADD><<<dim3((unsigned)blocks), dim3(TR_THREADS), 0, s>>>(a, b, y, n);
    PD_CHECK_LAUNCH(who);
    return PD_OK;
}

extern "C" int pd_gelu_fwd_bf16(const uint16_t* x, uint16_t* y, uint64_t n, void* stream) {
    return ew_launch(EW_GELU_FWD, x, nullptr, y, n, stream, "pd_gelu_fwd_bf16");
}
extern "C" int pd_gelu_bwd_bf16(const uint16_t* x, const uint16_t* dy, uint16_t* dx, uint64_t n, void* stream) {
    return ew_launch(EW_GELU_BWD, x, dy, dx, n, stream, "pd_gelu_bwd_bf16");
}
extern "C" int pd_add_bf16(const uint16_t* a, const uint16_t* b, uint16_t* y, uint64_t n, void* stream) {
    return ew_launch(EW_ADD, a, b, y, n, stream, "pd_add_bf16");
}

extern "C" int pd_cast_f32_to_bf16(const float* x, uint16_t* y, uint64_t n, void* stream) {
    if (n == 0) return PD_OK;
    PD_REQUIRE(x && y, PD_EINVAL, "pd_cast_f32_to_bf16: NULL pointer");
    PD_REQUIRE(pd_aligned(x, 16) && pd_aligned(y, 8), PD_EINVAL, "pd_cast_f32_to_bf16: alignment");
    const uint64_t blocks = ((n + 3) / 4 + TR_THREADS - 1) / TR_THREADS;
    PD_REQUIRE(blocks <= 0x7fffffffull, PD_ESHAPE, "pd_cast_f32_to_bf16: too large");
    cast_f32_bf16_kernel<<<dim3((unsigned)blocks), dim3(TR_THREADS), 0, (hipStream_t)stream>>>(x, y, n);
    PD_CHECK_LAUNCH("pd_cast_f32_to_bf16");
    return PD_OK;
}

extern "C" int pd_cast_bf16_to_f32(const uint16_t* x, float* y, uint64_t n, void* stream) {
    if (n == 0) return PD_OK;
    PD_REQUIRE(x && y, PD_EINVAL, "pd_cast_bf16_to_f32: NULL pointer");
    const uint64_t blocks = ((n + 3) / 4 + TR_THREADS - 1) / TR_THREADS;
    PD_REQUIRE(blocks <= 0x7fffffffull, PD_ESHAPE, "pd_cast_bf16_to_f32: too large");
    cast_bf16_f32_kernel<<<dim3((unsigned)blocks), dim3(TR_THREADS), 0, (hipStream_t)stream>>>(x, y, n);
    PD_CHECK_LAUNCH("pd_cast_bf16_to_f32");
    return PD_OK;
}

namespace {

// Several column sums in two launches (the bias and LayerNorm parameter gradients of one transformer
// layer's backward: twelve launches of a few microseconds each otherwise).  A job is a bf16 matrix [M][N]
// (first launch: fp32 partials of `splits` row ranges, as colsum_bf16_kernel; second launch: their sum)
// or an fp32 matrix of partials that only needs the second launch.  out = sum (+ beta * out).
constexpr int CB_MAX_JOBS = 8;
struct ColsumJob {
    const void* x;       // bf16 [M][ld] or fp32 [M][ld]
    float* part;         // bf16 jobs: [splits][N]
    float* out;          // [N]
    uint64_t M, ld;
    int N;
    int is_bf16;
    float beta;
    int tile1, tile2;    // first block of the job in the first (512 columns a block) / second (64) launch
};
struct ColsumBatch {
    ColsumJob job[CB_MAX_JOBS];
    int n;
};

__global__ __launch_bounds__(TR_THREADS) void colsum_batch_partial_kernel(const ColsumBatch b) {
    __shared__ float part[4][512];
    int j = 0;
#pragma unroll
    for (int q = 1; q < CB_MAX_JOBS; ++q) j += (q < b.n && (int)blockIdx.x >= b.job[q].tile1) ? 1 : 0;
    const ColsumJob& job = b.job[j];          // (jobs without a first launch have an empty tile range)
    const uint16_t* x = (const uint16_t*)job.x;
    const int N = job.N;
    const uint64_t M = job.M, ld = job.ld;
    const int lane = threadIdx.x % 64, w = threadIdx.x / 64;
    const int col0 = ((int)blockIdx.x - job.tile1) * 512;
    const int col = col0 + lane * 8;
    const uint64_t rows_per = (M + gridDim.y - 1) / gridDim.y;
    const uint64_t r0 = blockIdx.y * rows_per;
    const uint64_t r1 = (r0 + rows_per < M) ? r0 + rows_per : M;
    const bool vec = ((uintptr_t)x & 15) == 0 && ld % 8 == 0;
    float s[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) s[k] = 0.f;
    if (vec && col + 8 <= N) {
        for (uint64_t r = r0 + w; r < r1; r += 4) {
            const u16x8 v = *(const u16x8*)(x + r * ld + col);
#pragma unroll
            for (int k = 0; k < 8; ++k) s[k] += bf2f(v[k]);
        }
    } else {
        for (uint64_t r = r0 + w; r < r1; r += 4)
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (col + k < N) s[k] += bf2f(x[r * ld + col + k]);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) part[w][lane * 8 + k] = s[k];
    __syncthreads();
    for (int c = threadIdx.x; c < 512; c += TR_THREADS) {
        const int gc = col0 + c;
        if (gc < N) job.part[(uint64_t)blockIdx.y * N + gc] = (part[0][c] + part[1][c]) + (part[2][c] + part[3][c]);
    }
}

__global__ __launch_bounds__(TR_THREADS) void colsum_batch_final_kernel(const ColsumBatch b, int splits) {
    __shared__ float part[4][64];
    int j = 0;
#pragma unroll
    for (int q = 1; q < CB_MAX_JOBS; ++q) j += (q < b.n && (int)blockIdx.x >= b.job[q].tile2) ? 1 : 0;
    const ColsumJob& job = b.job[j];
    const float* x = job.is_bf16 ? job.part : (const float*)job.x;
    const uint64_t M = job.is_bf16 ? (uint64_t)splits : job.M, ld = job.is_bf16 ? (uint64_t)job.N : job.ld;
    const int N = job.N;
    const int col = ((int)blockIdx.x - job.tile2) * 64 + threadIdx.x % 64;
    const int w = threadIdx.x / 64;
    float s = 0.f;
    if (col < N) {
        float t[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        uint64_t r = w;
        for (; r + 28 < M; r += 32)
#pragma unroll
            for (int u = 0; u < 8; ++u) t[u] += x[(r + 4 * u) * ld + col];
        for (; r < M; r += 4) t[0] += x[r * ld + col];
        s = ((t[0] + t[1]) + (t[2] + t[3])) + ((t[4] + t[5]) + (t[6] + t[7]));
    }
    part[w][threadIdx.x % 64] = s;
    __syncthreads();
    if (w == 0 && col < N) {
        const float t = (part[0][threadIdx.x] + part[1][threadIdx.x]) + (part[2][threadIdx.x] + part[3][threadIdx.x]);
        float* o = job.out + col;
        *o = job.beta != 0.f ? t + job.beta * *o : t;
    }
}

}  // namespace

extern "C" int pd_colsum_batch_workspace_floats(int n_jobs, const int* is_bf16, const int* N, int splits,
                                                uint64_t* floats) {
    PD_REQUIRE(floats && (n_jobs == 0 || (is_bf16 && N)), PD_EINVAL, "pd_colsum_batch_workspace_floats: NULL pointer");
    PD_REQUIRE(n_jobs >= 0 && n_jobs <= CB_MAX_JOBS && splits >= 1 && splits <= 65535, PD_ESHAPE,
               "pd_colsum_batch_workspace_floats: at most %d jobs, 1..65535 splits", CB_MAX_JOBS);
    uint64_t total = 0;
    for (int j = 0; j < n_jobs; ++j)
        if (is_bf16[j]) total += (uint64_t)splits * (uint64_t)(N[j] > 0 ? N[j] : 0);
    *floats = total;
    return PD_OK;
}

extern "C" int pd_colsum_batch(int n_jobs, const void* const* x, const int* is_bf16, float* const* out,
                               const uint64_t* M, const int* N, const uint64_t* ld, const float* beta,
                               float* workspace, uint64_t workspace_floats, int splits, void* stream) {
    const char* who = "pd_colsum_batch";
    if (n_jobs == 0) return PD_OK;
    PD_REQUIRE(n_jobs > 0 && n_jobs <= CB_MAX_JOBS && splits >= 1 && splits <= 65535, PD_ESHAPE,
               "%s: at most %d jobs, 1..65535 splits", who, CB_MAX_JOBS);
    PD_REQUIRE(x && is_bf16 && out && M && N && ld && beta, PD_EINVAL, "%s: NULL argument array", who);
    ColsumBatch b;
    b.n = n_jobs;
    uint64_t used = 0;
    int tiles1 = 0, tiles2 = 0;
    for (int j = 0; j < n_jobs; ++j) {
        PD_REQUIRE(x[j] && out[j], PD_EINVAL, "%s: NULL operand in job %d", who, j);
        PD_REQUIRE(N[j] > 0 && M[j] > 0 && ld[j] >= (uint64_t)N[j], PD_ESHAPE, "%s: bad shape in job %d", who, j);
        ColsumJob& job = b.job[j];
        job.x = x[j]; job.out = out[j]; job.M = M[j]; job.ld = ld[j]; job.N = N[j];
        job.is_bf16 = is_bf16[j] != 0; job.beta = beta[j];
        job.part = nullptr;
        job.tile1 = tiles1; job.tile2 = tiles2;
        if (job.is_bf16) {
            job.part = workspace + used;
            used += (uint64_t)splits * N[j];
            tiles1 += (N[j] + 511) / 512;
        }
        tiles2 += (N[j] + 63) / 64;
    }
    PD_REQUIRE(used == 0 || (workspace && workspace_floats >= used), PD_EINVAL,
               "%s: workspace too small (%llu < %llu floats)", who, (unsigned long long)workspace_floats,
               (unsigned long long)used);
    if (tiles1 > 0) {
        colsum_batch_partial_kernel<<<dim3(tiles1, splits), dim3(TR_THREADS), 0, (hipStream_t)stream>>>(b);
        PD_CHECK_LAUNCH(who);
    }
    colsum_batch_final_kernel<<<dim3(tiles2), dim3(TR_THREADS), 0, (hipStream_t)stream>>>(b, splits);
    PD_CHECK_LAUNCH(who);
    return PD_OK;
}

extern "C" int pd_colsum_bf16(const uint16_t* x, float* out, uint64_t M, int N, uint64_t ld, int splits, void* stream) {
    PD_REQUIRE(N >= 0 && splits >= 1 && splits <= 65535, PD_ESHAPE, "pd_colsum_bf16: bad N or splits");
    if (N == 0) return PD_OK;
    PD_REQUIRE(x && out, PD_EINVAL, "pd_colsum_bf16: NULL operand");
    PD_REQUIRE(ld >= (uint64_t)N, PD_ESHAPE, "pd_colsum_bf16: ld < N");
    const int vec = pd_aligned(x, 16) && ld % 8 == 0;
    colsum_bf16_kernel<<<dim3((N + 511) / 512, splits), dim3(TR_THREADS), 0, (hipStream_t)stream>>>(x, out, M, N, ld, vec);
    PD_CHECK_LAUNCH("pd_colsum_bf16");
    return PD_OK;
}
