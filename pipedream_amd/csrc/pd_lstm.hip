// LSTM cell (gate non-linearities + state update) and embedding lookup, forward and
// backward: the HBM-bound parts of the GNMT-style stage.  The matrix products around
// them (input projection for all time steps, the per-step recurrent product, the weight
// gradients) run on the fp32 MFMA GEMM.
//
// They stand in for torch.nn.LSTM / torch.nn.Embedding of the reference's translation
// stages (runtime/translation/models/gnmt_large/gpus=4/stage0.py:10-19; gate order and
// parameter layout are torch's: rows [i | f | g | o] of weight_ih / weight_hh / bias).
//
// Algorithmic traffic per (batch row, hidden unit) and time step:
//   forward : read 4 gate pre-activations + c_prev, write 4 activated gates + c + h = 44 B
//   backward: read 4 gates + c_prev + c + dh (+dy) + dc, write 4 dgates + dc        = 60-64 B
#include "pd_internal.h"

typedef float float4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int LSTM_THREADS = 256;
constexpr long LSTM_SCALAR_UNITS = 1L << 19;   // up to here (batch x hidden units) the cell kernels take one unit per thread

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

// gates: [B][4H] pre-activations (x W_ih^T + h W_hh^T), overwritten with the ACTIVATED
// gates i,f,g,o which the backward pass needs.  One thread = V consecutive hidden units: 4 (128-bit
// accesses) for large batches; 1 at the recurrence's own size (batch 128 x 1024 units), where four units
// per thread leave two waves per CU, each with some twenty transcendental evaluations in a row -- the
// kernel is then bound by one wave's instruction latency, not by memory.  Every unit sees the same
// operations in the same order either way.
template <int V>
__global__ __launch_bounds__(LSTM_THREADS) void lstm_cell_fwd_kernel(float* __restrict__ gates,
                                                                     const float* __restrict__ rec, int n_rec,
                                                                     const float* __restrict__ b_ih,
                                                                     const float* __restrict__ b_hh,
                                                                     const float* __restrict__ c_prev,
                                                                     float* __restrict__ c_out,
                                                                     float* __restrict__ h_out, int B, int H) {
    typedef float vec_t __attribute__((ext_vector_type(V)));
    const int HV = H / V;
    const int id = blockIdx.x * LSTM_THREADS + threadIdx.x;
    if (id >= B * HV) return;
    const int b = id / HV, j = (id % HV) * V;
    float* g = gates + (size_t)b * 4 * H;
    vec_t gi = *(const vec_t*)(g + j);
    vec_t gf = *(const vec_t*)(g + H + j);
    vec_t gg = *(const vec_t*)(g + 2 * H + j);
    vec_t go = *(const vec_t*)(g + 3 * H + j);
    // split-k partial sums of h_{t-1} W_hh^T, added in a fixed order, four partials (16 loads) in flight at
    // a time: one at a time the loop is a chain of round trips to memory
    for (int s0 = 0; s0 < n_rec; s0 += 4) {
        vec_t p[4][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const bool live = s0 + u < n_rec;
            const float* r = rec + ((size_t)(live ? s0 + u : s0) * B + b) * 4 * H;
#pragma unroll
            for (int q = 0; q < 4; ++q) p[u][q] = *(const vec_t*)(r + q * H + j);
            if (!live) {
#pragma unroll
                for (int q = 0; q < 4; ++q) p[u][q] = vec_t(0.f);
            }
        }
        gi += (p[0][0] + p[1][0]) + (p[2][0] + p[3][0]);
        gf += (p[0][1] + p[1][1]) + (p[2][1] + p[3][1]);
        gg += (p[0][2] + p[1][2]) + (p[2][2] + p[3][2]);
        go += (p[0][3] + p[1][3]) + (p[2][3] + p[3][3]);
    }
    if (b_ih) {
        gi += *(const vec_t*)(b_ih + j) + *(const vec_t*)(b_hh + j);
        gf += *(const vec_t*)(b_ih + H + j) + *(const vec_t*)(b_hh + H + j);
        gg += *(const vec_t*)(b_ih + 2 * H + j) + *(const vec_t*)(b_hh + 2 * H + j);
        go += *(const vec_t*)(b_ih + 3 * H + j) + *(const vec_t*)(b_hh + 3 * H + j);
    }
    vec_t cp = vec_t(0.f);
    if (c_prev) cp = *(const vec_t*)(c_prev + (size_t)b * H + j);
    vec_t c, h;
#pragma unroll
    for (int k = 0; k < V; ++k) {
        gi[k] = sigmoidf_(gi[k]);
        gf[k] = sigmoidf_(gf[k]);
        gg[k] = tanhf(gg[k]);
        go[k] = sigmoidf_(go[k]);
        c[k] = gf[k] * cp[k] + gi[k] * gg[k];
        h[k] = go[k] * tanhf(c[k]);
    }
    *(vec_t*)(g + j) = gi;
    *(vec_t*)(g + H + j) = gf;
    *(vec_t*)(g + 2 * H + j) = gg;
    *(vec_t*)(g + 3 * H + j) = go;
    *(vec_t*)(c_out + (size_t)b * H + j) = c;
    *(vec_t*)(h_out + (size_t)b * H + j) = h;
}

// dh = dy (+ dh_rec); dc = dc_next + dh*o*(1-tanh(c)^2); dgates are gradients with respect
// to the pre-activations; dc_next is overwritten with the gradient for c_prev.
template <int V>
__global__ __launch_bounds__(LSTM_THREADS) void lstm_cell_bwd_kernel(const float* __restrict__ gates,
                                                                     const float* __restrict__ c_prev,
                                                                     const float* __restrict__ c,
                                                                     const float* __restrict__ dy,
                                                                     const float* __restrict__ dh_rec, int n_rec,
                                                                     float* __restrict__ dc_io,
                                                                     float* __restrict__ dgates, int B, int H,
                                                                     int first_step) {
    typedef float vec_t __attribute__((ext_vector_type(V)));
    const int HV = H / V;
    const int id = blockIdx.x * LSTM_THREADS + threadIdx.x;
    if (id >= B * HV) return;
    const int b = id / HV, j = (id % HV) * V;
    const float* g = gates + (size_t)b * 4 * H;
    const vec_t gi = *(const vec_t*)(g + j);
    const vec_t gf = *(const vec_t*)(g + H + j);
    const vec_t gg = *(const vec_t*)(g + 2 * H + j);
    const vec_t go = *(const vec_t*)(g + 3 * H + j);
    const size_t o = (size_t)b * H + j;
    vec_t cp = vec_t(0.f);
    if (c_prev) cp = *(const vec_t*)(c_prev + o);
    const vec_t ct = *(const vec_t*)(c + o);
    vec_t dh = *(const vec_t*)(dy + o);
    if (dh_rec) {
        // the split-k partial sums of dgates W_hh, eight loads in flight at a time, added in a fixed order
        for (int s0 = 0; s0 < n_rec; s0 += 8) {
            vec_t p[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const bool live = s0 + u < n_rec;
                p[u] = *(const vec_t*)(dh_rec + (size_t)(live ? s0 + u : s0) * B * H + o);
                if (!live) p[u] = vec_t(0.f);
            }
            dh += ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
        }
    }
    vec_t dc = vec_t(0.f);
    if (!first_step) dc = *(const vec_t*)(dc_io + o);
    vec_t di, df, dg, dO, dcp;
#pragma unroll
    for (int k = 0; k < V; ++k) {
        const float tc = tanhf(ct[k]);
        const float dck = dc[k] + dh[k] * go[k] * (1.0f - tc * tc);
        dO[k] = dh[k] * tc * go[k] * (1.0f - go[k]);
        di[k] = dck * gg[k] * gi[k] * (1.0f - gi[k]);
        df[k] = dck * cp[k] * gf[k] * (1.0f - gf[k]);
        dg[k] = dck * gi[k] * (1.0f - gg[k] * gg[k]);
        dcp[k] = dck * gf[k];
    }
    float* d = dgates + (size_t)b * 4 * H;
    *(vec_t*)(d + j) = di;
    *(vec_t*)(d + H + j) = df;
    *(vec_t*)(d + 2 * H + j) = dg;
    *(vec_t*)(d + 3 * H + j) = dO;
    *(vec_t*)(dc_io + o) = dcp;
}

// y = a + b  (the residual connections between LSTM layers)
__global__ __launch_bounds__(LSTM_THREADS) void add_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                           float* __restrict__ y, uint64_t n, bool vec) {
    uint64_t i = ((uint64_t)blockIdx.x * LSTM_THREADS + threadIdx.x) * 4;
    if (i >= n) return;
    if (vec && i + 3 < n) {
        *(float4_t*)(y + i) = *(const float4_t*)(a + i) + *(const float4_t*)(b + i);
    } else {
        for (uint64_t k = i; k < n && k < i + 4; ++k) y[k] = a[k] + b[k];
    }
}

// out[p][:] = weight[ids[p]][:]; one block per token, 4 floats per thread per pass.
__global__ __launch_bounds__(LSTM_THREADS) void embedding_fwd_kernel(const int64_t* __restrict__ ids,
                                                                     const float* __restrict__ weight,
                                                                     float* __restrict__ out, int D, int64_t V) {
    const int64_t v = ids[blockIdx.x];
    const float* src = weight + (size_t)(v < 0 || v >= V ? 0 : v) * D;
    float* dst = out + (size_t)blockIdx.x * D;
    for (int j = threadIdx.x * 4; j < D; j += LSTM_THREADS * 4) *(float4_t*)(dst + j) = *(const float4_t*)(src + j);
}

// dweight[v][:] = sum over positions p with ids[p] == v of dout[p][:], positions in
// increasing order (deterministic, no atomics); rows without a hit and the padding row
// are zeros.  Two launches: a fill with zeros, then one block per token position: the block
// of the first position that holds a row's id sums all of that row's positions, every other
// block leaves as soon as it meets an earlier position with its id (one scan of the ids per
// position, 64 at a time with a ballot, instead of one per vocabulary row).
__global__ __launch_bounds__(LSTM_THREADS) void zero_fill_kernel(float4_t* __restrict__ dst, size_t n4) {
    const size_t i = (size_t)blockIdx.x * LSTM_THREADS + threadIdx.x;
    if (i < n4) dst[i] = float4_t{0.f, 0.f, 0.f, 0.f};
}

__global__ __launch_bounds__(LSTM_THREADS) void embedding_bwd_kernel(const int64_t* __restrict__ ids,
                                                                     const float* __restrict__ dout,
                                                                     float* __restrict__ dweight, int n_tokens, int D,
                                                                     int64_t V, int64_t padding_idx) {
    const int me = blockIdx.x;
    const int64_t v = ids[me];
    if (v < 0 || v >= V || v == padding_idx) return;
    const int lane = threadIdx.x % 64;
    // every thread owns D/(4*256) float4 columns; D <= 4096 supported by the accumulators below
    float4_t acc[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[r] = (float4_t){0.f, 0.f, 0.f, 0.f};
    bool owner = false;                        // the same in every thread of the block
    for (int p0 = 0; p0 < n_tokens; p0 += 64) {
        const int p = p0 + lane;
        const bool hit = p < n_tokens && ids[p] == v;
        unsigned long long m = __ballot(hit);
        if (!owner && m) {
            if (p0 + __ffsll((long long)m) - 1 != me) return;   // an earlier position owns this row
            owner = true;
        }
        while (m) {
            const int bit = __ffsll((long long)m) - 1;
            m &= m - 1;
            const float* src = dout + (size_t)(p0 + bit) * D;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int j = (r * LSTM_THREADS + threadIdx.x) * 4;
                if (j < D) acc[r] += *(const float4_t*)(src + j);
            }
        }
    }
    float* dst = dweight + (size_t)v * D;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int j = (r * LSTM_THREADS + threadIdx.x) * 4;
        if (j < D) *(float4_t*)(dst + j) = acc[r];
    }
}

}  // namespace

extern "C" int pd_lstm_cell_fwd_f32(float* gates, const float* rec, int n_rec, const float* b_ih, const float* b_hh,
                                    const float* c_prev, float* c_out, float* h_out, int B, int H, void* stream) {
    PD_REQUIRE(n_rec >= 0 && (n_rec == 0 || (rec && pd_aligned(rec, 16))), PD_EINVAL,
               "pd_lstm_cell_fwd_f32: rec must be a 16-byte aligned pointer when n_rec > 0");
    PD_REQUIRE(B > 0 && H > 0 && H % 4 == 0, PD_ESHAPE, "pd_lstm_cell_fwd_f32: need B > 0 and H a positive multiple of 4");
    PD_REQUIRE(gates && c_out && h_out, PD_EINVAL, "pd_lstm_cell_fwd_f32: NULL pointer");
    PD_REQUIRE((b_ih == nullptr) == (b_hh == nullptr), PD_EINVAL, "pd_lstm_cell_fwd_f32: pass both biases or neither");
    PD_REQUIRE(pd_aligned(gates, 16) && pd_aligned(c_out, 16) && pd_aligned(h_out, 16) &&
                   (!c_prev || pd_aligned(c_prev, 16)) && (!b_ih || (pd_aligned(b_ih, 16) && pd_aligned(b_hh, 16))),
               PD_EINVAL, "pd_lstm_cell_fwd_f32: pointers must be 16-byte aligned");
    if ((long)B * H <= LSTM_SCALAR_UNITS) {
        const int total = B * H;
        lstm_cell_fwd_kernel<1><<<dim3((total + LSTM_THREADS - 1) / LSTM_THREADS), dim3(LSTM_THREADS), 0,
                                  (hipStream_t)stream>>>(gates, rec, n_rec, b_ih, b_hh, c_prev, c_out, h_out, B, H);
    } else {
        const int total = B * (H / 4);
        lstm_cell_fwd_kernel<4><<<dim3((total + LSTM_THREADS - 1) / LSTM_THREADS), dim3(LSTM_THREADS), 0,
                                  (hipStream_t)stream>>>(gates, rec, n_rec, b_ih, b_hh, c_prev, c_out, h_out, B, H);
    }
    PD_CHECK_LAUNCH("pd_lstm_cell_fwd_f32");
    return PD_OK;
}

extern "C" int pd_lstm_cell_bwd_f32(const float* gates, const float* c_prev, const float* c, const float* dy,
                                    const float* dh_rec, int n_rec, float* dc_io, float* dgates, int B, int H,
                                    int first_step, void* stream) {
    PD_REQUIRE(!dh_rec || n_rec >= 1, PD_EINVAL, "pd_lstm_cell_bwd_f32: dh_rec needs n_rec >= 1");
    PD_REQUIRE(B > 0 && H > 0 && H % 4 == 0, PD_ESHAPE, "pd_lstm_cell_bwd_f32: need B > 0 and H a positive multiple of 4");
    PD_REQUIRE(gates && c && dy && dc_io && dgates, PD_EINVAL, "pd_lstm_cell_bwd_f32: NULL pointer");
    PD_REQUIRE(pd_aligned(gates, 16) && pd_aligned(c, 16) && pd_aligned(dy, 16) && pd_aligned(dc_io, 16) &&
                   pd_aligned(dgates, 16) && (!c_prev || pd_aligned(c_prev, 16)) && (!dh_rec || pd_aligned(dh_rec, 16)),
               PD_EINVAL, "pd_lstm_cell_bwd_f32: pointers must be 16-byte aligned");
    if ((long)B * H <= LSTM_SCALAR_UNITS) {
        const int total = B * H;
        lstm_cell_bwd_kernel<1><<<dim3((total + LSTM_THREADS - 1) / LSTM_THREADS), dim3(LSTM_THREADS), 0,
                                  (hipStream_t)stream>>>(gates, c_prev, c, dy, dh_rec, n_rec, dc_io, dgates, B, H,
                                                         first_step);
    } else {
        const int total = B * (H / 4);
        lstm_cell_bwd_kernel<4><<<dim3((total + LSTM_THREADS - 1) / LSTM_THREADS), dim3(LSTM_THREADS), 0,
                                  (hipStream_t)stream>>>(gates, c_prev, c, dy, dh_rec, n_rec, dc_io, dgates, B, H,
                                                         first_step);
    }
    PD_CHECK_LAUNCH("pd_lstm_cell_bwd_f32");
    return PD_OK;
}

// The time loop of one layer, issued from native code: per step one k-split product (none at the first step)
// and one cell launch, all on `stream`.  Shapes and pointers are checked once, by the first step's calls.
extern "C" int pd_lstm_recurrence_fwd_f32(float* gates, const float* w_hh, const float* b_ih, const float* b_hh,
                                          float* rec, int splits, float* c, float* y, int T, int B, int H,
                                          void* stream) {
    PD_REQUIRE(T > 0 && B > 0 && H > 0 && H % 4 == 0 && splits >= 1, PD_ESHAPE,
               "pd_lstm_recurrence_fwd_f32: need T, B > 0, H a positive multiple of 4 and splits >= 1");
    PD_REQUIRE(gates && w_hh && c && y && (T == 1 || rec), PD_EINVAL, "pd_lstm_recurrence_fwd_f32: NULL pointer");
    const size_t bh = (size_t)B * H;
    for (int t = 0; t < T; ++t) {
        if (t > 0) {
            const int rc = pd_gemm_splitk_f32(0, 1, B, 4 * H, H, y + (t - 1) * bh, H, w_hh, H, rec, splits, stream);
            if (rc != PD_OK) return rc;
        }
        const int rc = pd_lstm_cell_fwd_f32(gates + t * 4 * bh, rec, t > 0 ? splits : 0, b_ih, b_hh,
                                            t > 0 ? c + (t - 1) * bh : nullptr, c + t * bh, y + t * bh, B, H, stream);
        if (rc != PD_OK) return rc;
    }
    return PD_OK;
}

extern "C" int pd_lstm_recurrence_bwd_f32(const float* gates, const float* c, const float* dy, const float* w_hh,
                                          float* dh_rec, int splits, float* dc, float* dgates, int T, int B, int H,
                                          void* stream) {
    PD_REQUIRE(T > 0 && B > 0 && H > 0 && H % 4 == 0 && splits >= 1, PD_ESHAPE,
               "pd_lstm_recurrence_bwd_f32: need T, B > 0, H a positive multiple of 4 and splits >= 1");
    PD_REQUIRE(gates && c && dy && w_hh && dc && dgates && (T == 1 || dh_rec), PD_EINVAL,
               "pd_lstm_recurrence_bwd_f32: NULL pointer");
    const size_t bh = (size_t)B * H;
    for (int t = T - 1; t >= 0; --t) {
        int rc = pd_lstm_cell_bwd_f32(gates + t * 4 * bh, t > 0 ? c + (t - 1) * bh : nullptr, c + t * bh, dy + t * bh,
                                      t < T - 1 ? dh_rec : nullptr, splits, dc, dgates + t * 4 * bh, B, H,
                                      t == T - 1, stream);
        if (rc != PD_OK) return rc;
        if (t > 0) {      // dh_{t-1} += dgates_t W_hh: [B][4H] x [4H][H], split over 4H
            rc = pd_gemm_splitk_f32(0, 0, B, H, 4 * H, dgates + t * 4 * bh, 4 * H, w_hh, H, dh_rec, splits, stream);
            if (rc != PD_OK) return rc;
        }
    }
    return PD_OK;
}

extern "C" int pd_add_f32(const float* a, const float* b, float* y, uint64_t n, void* stream) {
    if (n == 0) return PD_OK;
    PD_REQUIRE(a && b && y, PD_EINVAL, "pd_add_f32: NULL pointer");
    const uint64_t blocks = ((n + 3) / 4 + LSTM_THREADS - 1) / LSTM_THREADS;
    PD_REQUIRE(blocks <= 0x7fffffffull, PD_ESHAPE, "pd_add_f32: too large");
    const bool vec = pd_aligned(a, 16) && pd_aligned(b, 16) && pd_aligned(y, 16);
    add_kernel<<<dim3((unsigned)blocks), dim3(LSTM_THREADS), 0, (hipStream_t)stream>>>(a, b, y, n, vec);
    PD_CHECK_LAUNCH("pd_add_f32");
    return PD_OK;
}

extern "C" int pd_embedding_fwd_f32(const int64_t* ids, const float* weight, float* out, int n_tokens, int D,
                                    int64_t V, void* stream) {
    PD_REQUIRE(n_tokens >= 0 && D > 0 && D % 4 == 0 && V > 0, PD_ESHAPE,
               "pd_embedding_fwd_f32: need D a positive multiple of 4 and V > 0");
    if (n_tokens == 0) return PD_OK;
    PD_REQUIRE(ids && weight && out, PD_EINVAL, "pd_embedding_fwd_f32: NULL pointer");
    PD_REQUIRE(pd_aligned(weight, 16) && pd_aligned(out, 16), PD_EINVAL, "pd_embedding_fwd_f32: 16-byte alignment");
    embedding_fwd_kernel<<<dim3(n_tokens), dim3(LSTM_THREADS), 0, (hipStream_t)stream>>>(ids, weight, out, D, V);
    PD_CHECK_LAUNCH("pd_embedding_fwd_f32");
    return PD_OK;
}

extern "C" int pd_embedding_bwd_f32(const int64_t* ids, const float* dout, float* dweight, int n_tokens, int D,
                                    int64_t V, int64_t padding_idx, void* stream) {
    PD_REQUIRE(n_tokens >= 0 && D > 0 && D % 4 == 0 && D <= 4096 && V > 0 && V <= 0x7fffffff, PD_ESHAPE,
               "pd_embedding_bwd_f32: need D a multiple of 4 in (0, 4096] and 0 < V < 2^31");
    PD_REQUIRE(dweight && (n_tokens == 0 || (ids && dout)), PD_EINVAL, "pd_embedding_bwd_f32: NULL pointer");
    PD_REQUIRE(pd_aligned(dweight, 16) && pd_aligned(dout, 16), PD_EINVAL, "pd_embedding_bwd_f32: 16-byte alignment");
    const size_t n4 = (size_t)V * D / 4;
    PD_REQUIRE(n4 / LSTM_THREADS < 0x7fffffffull, PD_ESHAPE, "pd_embedding_bwd_f32: table too large");
    zero_fill_kernel<<<dim3((unsigned)((n4 + LSTM_THREADS - 1) / LSTM_THREADS)), dim3(LSTM_THREADS), 0,
                       (hipStream_t)stream>>>((float4_t*)dweight, n4);
    PD_CHECK_LAUNCH("pd_embedding_bwd_f32");
    if (n_tokens > 0)
        embedding_bwd_kernel<<<dim3((unsigned)n_tokens), dim3(LSTM_THREADS), 0, (hipStream_t)stream>>>(
            ids, dout, dweight, n_tokens, D, V, padding_idx);
    PD_CHECK_LAUNCH("pd_embedding_bwd_f32");
    return PD_OK;
}
