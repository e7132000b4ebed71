// Fused multi-tensor SGD-momentum / Adam step that also performs the weight
// stash: parameters are read from the loaded ring slot and written to the
// ring's write slot, so no separate get_params copy is needed.
//
// HBM-bound.  Algorithmic traffic per parameter:
//   SGD-momentum: read grad, p, buf; write p', buf'            = 20 B
//   Adam        : read grad, p, m, v; write p', m', v'         = 28 B (+2 B bf16 copy)
//
// Reference behaviour restated: runtime/optimizer.py:137-159 (grad scaling,
// base_optimizer.step(), copy into the oldest slot); arithmetic of
// torch.optim.SGD / torch.optim.Adam (_single_tensor_sgd / _single_tensor_adam),
// with the same operation order as their CPU kernels (fused multiply-add where
// `add(alpha=)` / `lerp` use one, separate roundings elsewhere).
#include "pd_internal.h"

typedef float float4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int OPT_THREADS = 64;                                // one wave per block
constexpr int OPT_UNROLL = 1;                                  // float4 vectors per thread: a block streams 1 KiB
                                                               // of every operand (measured: 4 KiB per block costs
                                                               // 2-3 % of the bandwidth, 16 KiB 8 %)
constexpr int OPT_CHUNK = OPT_THREADS * OPT_UNROLL * 4;        // elements per block
constexpr int OPT_MAX_TENSORS = 32;                            // descriptors per launch

struct OptArgs {
    pd_tensor_desc t[OPT_MAX_TENSORS];
    uint32_t block_start[OPT_MAX_TENSORS + 1];  // prefix sum of per-tensor block counts
    uint32_t vec_ok;                            // bit i: all pointers of tensor i are 16-B aligned
    int n_tensors;
    int grad_fmt;                               // PD_F32 / PD_BF16 / PD_F16: what desc.grad points at
    int out_fmt;                                // PD_BF16 / PD_F16: format of the 16-bit copy (desc.bf16_out)
};

struct SgdHyper {
    float lr, momentum, one_minus_damp, wd;
    float loss_scale, update_interval;
    int nesterov, first_step, has_momentum;
};

struct AdamHyper {
    float w1;             // 1 - beta1
    float beta2, one_minus_beta2;
    float eps, wd;
    float step_size;      // lr / bc1                (mode 0) | lr*sqrt(bc2)/bc1 (mode 1)
    float bc2_sqrt;       // sqrt(1 - beta2^t)       (mode 0) | unused            (mode 1)
    float loss_scale, update_interval;
    int eps_mode;
};

__device__ __forceinline__ float scale_grad(float g, float loss_scale, float update_interval) {
    if (loss_scale != 1.0f) g = __fdiv_rn(g, loss_scale);
    if (update_interval != 1.0f) g = __fdiv_rn(g, update_interval);
    return g;
}

__device__ __forceinline__ void sgd_elem(float g, float p, float& buf, float& p_new, const SgdHyper& h) {
    g = scale_grad(g, h.loss_scale, h.update_interval);
    if (h.wd != 0.0f) g = __fmaf_rn(h.wd, p, g);
    if (h.has_momentum) {
        if (h.first_step) {
            buf = g;
        } else {
            buf = __fmaf_rn(h.one_minus_damp, g, __fmul_rn(buf, h.momentum));
        }
        g = h.nesterov ? __fmaf_rn(h.momentum, buf, g) : buf;
    }
    p_new = __fmaf_rn(-h.lr, g, p);
}

__device__ __forceinline__ void adam_elem(float g, float p, float& m, float& v, float& p_new, const AdamHyper& h) {
    g = scale_grad(g, h.loss_scale, h.update_interval);
    if (h.wd != 0.0f) g = __fmaf_rn(h.wd, p, g);
    // exp_avg.lerp_(grad, 1 - beta1)
    float diff = __fsub_rn(g, m);
    m = (fabsf(h.w1) < 0.5f) ? __fmaf_rn(h.w1, diff, m) : __fmaf_rn(__fsub_rn(h.w1, 1.0f), diff, g);
    // exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
    v = __fadd_rn(__fmul_rn(v, h.beta2), __fmul_rn(__fmul_rn(h.one_minus_beta2, g), g));
    float denom;
    if (h.eps_mode == 0) {
        denom = __fadd_rn(__fdiv_rn(__fsqrt_rn(v), h.bc2_sqrt), h.eps);
    } else {
        denom = __fadd_rn(__fsqrt_rn(v), h.eps);
    }
    // param.addcdiv_(exp_avg, denom, value=-step_size)
    p_new = __fadd_rn(p, __fdiv_rn(__fmul_rn(-h.step_size, m), denom));
}

// 16-bit formats of the mixed-precision step: gradients arrive in the model's format and are widened, the
// new parameters are also written in it (both conversions round to nearest even)
__device__ __forceinline__ float half_to_f32(uint16_t h, int fmt) {
    return fmt == PD_F16 ? (float)__builtin_bit_cast(_Float16, h) : __uint_as_float((uint32_t)h << 16);
}

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f);

__device__ __forceinline__ uint16_t f32_to_half(float f, int fmt) {
    return fmt == PD_F16 ? __builtin_bit_cast(uint16_t, (_Float16)f) : f32_to_bf16_rne(f);
}

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Uniform (per block) lookup of the tensor that owns this block: the number of tensors that start at or
// before it.  All prefix sums are fetched at once and compared without a branch -- a binary search is a
// chain of five dependent scalar loads in front of a wave's first memory request, which cost 3-5 % of the
// kernel's bandwidth.  Entries past n_tensors hold the total block count, which no block index reaches.
__device__ __forceinline__ int find_tensor(const OptArgs& a, uint32_t b) {
    int ti = 0;
#pragma unroll
    for (int k = 1; k < OPT_MAX_TENSORS; ++k) ti += (b >= a.block_start[k]) ? 1 : 0;
    return ti;
}

// GRAD16: gradients arrive in the 16-bit format a.grad_fmt (else fp32).  OUT_RT: the 16-bit copy of the new
// parameters is written in the format a.out_fmt (else bf16).  The plain fp32 step is its own instantiation and
// carries none of that.
template <bool ADAM, bool GRAD16, bool OUT_RT>
__global__ __launch_bounds__(OPT_THREADS) void pd_optim_kernel(const OptArgs a, const SgdHyper sh, const AdamHyper ah) {
    const int ti = find_tensor(a, blockIdx.x);
    const pd_tensor_desc& t = a.t[ti];
    const uint64_t n = t.n;
    const uint64_t chunk0 = (uint64_t)(blockIdx.x - a.block_start[ti]) * OPT_CHUNK;
    const bool vec_ok = (a.vec_ok >> ti) & 1u;
    const bool has_s0 = ADAM || sh.has_momentum;

    if (vec_ok && chunk0 + OPT_CHUNK <= n) {
        // Full, aligned chunk: every access is a 128-bit vector; all loads are
        // issued before the first use so each wave keeps 3-4 KiB in flight.
        float4_t g[OPT_UNROLL], p[OPT_UNROLL], s0[OPT_UNROLL], s1[OPT_UNROLL];
        const uint64_t v0 = chunk0 / 4 + threadIdx.x;
#pragma unroll
        for (int u = 0; u < OPT_UNROLL; ++u) {
            const uint64_t i = v0 + (uint64_t)u * OPT_THREADS;
            if (GRAD16) {
                typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
                const u16x4 h = __builtin_nontemporal_load((const u16x4*)t.grad + i);
#pragma unroll
                for (int k = 0; k < 4; ++k) g[u][k] = half_to_f32(h[k], a.grad_fmt);
            } else {
                g[u] = __builtin_nontemporal_load((const float4_t*)t.grad + i);
            }
            p[u] = __builtin_nontemporal_load((const float4_t*)t.p_in + i);
            if (has_s0) s0[u] = __builtin_nontemporal_load((const float4_t*)t.state0 + i);
            if (ADAM) s1[u] = __builtin_nontemporal_load((const float4_t*)t.state1 + i);
        }
#pragma unroll
        for (int u = 0; u < OPT_UNROLL; ++u) {
            const uint64_t i = v0 + (uint64_t)u * OPT_THREADS;
            float4_t pn;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                float pk;
                if (ADAM) {
                    float m = s0[u][k], v = s1[u][k];
                    adam_elem(g[u][k], p[u][k], m, v, pk, ah);
                    s0[u][k] = m;
                    s1[u][k] = v;
                } else {
                    float b = has_s0 ? s0[u][k] : 0.0f;
                    sgd_elem(g[u][k], p[u][k], b, pk, sh);
                    s0[u][k] = b;
                }
                pn[k] = pk;
            }
            __builtin_nontemporal_store(pn, (float4_t*)t.p_out + i);
            if (has_s0) __builtin_nontemporal_store(s0[u], (float4_t*)t.state0 + i);
            if (ADAM) __builtin_nontemporal_store(s1[u], (float4_t*)t.state1 + i);
            if (t.bf16_out) {
                typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
                u16x4 h;
                if (OUT_RT) h = u16x4{f32_to_half(pn[0], a.out_fmt), f32_to_half(pn[1], a.out_fmt),
                                     f32_to_half(pn[2], a.out_fmt), f32_to_half(pn[3], a.out_fmt)};
                else h = u16x4{f32_to_bf16_rne(pn[0]), f32_to_bf16_rne(pn[1]), f32_to_bf16_rne(pn[2]), f32_to_bf16_rne(pn[3])};
                *((u16x4*)t.bf16_out + i) = h;
            }
        }
    } else {
        // Ragged tail or unaligned tensor: scalar accesses, still coalesced.
        for (int u = 0; u < OPT_UNROLL * 4; ++u) {
            const uint64_t i = chunk0 + (uint64_t)u * OPT_THREADS + threadIdx.x;
            if (i >= n) break;
            float g = GRAD16 ? half_to_f32(((const uint16_t*)t.grad)[i], a.grad_fmt) : t.grad[i], p = t.p_in[i], pn;
            if (ADAM) {
                float m = t.state0[i], v = t.state1[i];
                adam_elem(g, p, m, v, pn, ah);
                t.state0[i] = m;
                t.state1[i] = v;
            } else {
                float b = has_s0 ? t.state0[i] : 0.0f;
                sgd_elem(g, p, b, pn, sh);
                if (has_s0) t.state0[i] = b;
            }
            t.p_out[i] = pn;
            if (t.bf16_out) t.bf16_out[i] = OUT_RT ? f32_to_half(pn, a.out_fmt) : f32_to_bf16_rne(pn);
        }
    }
}

template <bool ADAM>
int launch_optim(const pd_tensor_desc* descs, int n_tensors, const SgdHyper& sh, const AdamHyper& ah,
                 bool need_s0, void* stream, const char* who, int grad_fmt = PD_F32, int out_fmt = PD_BF16) {
    PD_REQUIRE(n_tensors >= 0, PD_EINVAL, "%s: n_tensors < 0", who);
    PD_REQUIRE(grad_fmt == PD_F32 || grad_fmt == PD_BF16 || grad_fmt == PD_F16, PD_EINVAL, "%s: unknown gradient format %d",
               who, grad_fmt);
    PD_REQUIRE(out_fmt == PD_BF16 || out_fmt == PD_F16, PD_EINVAL, "%s: unknown 16-bit output format %d", who, out_fmt);
    const bool grad16 = grad_fmt != PD_F32, out_rt = out_fmt != PD_BF16;
    if (n_tensors == 0) return PD_OK;
    PD_REQUIRE(descs != nullptr, PD_EINVAL, "%s: descs is NULL", who);
    int i = 0;
    while (i < n_tensors) {
        OptArgs a;
        a.n_tensors = 0;
        a.vec_ok = 0;
        a.block_start[0] = 0;
        uint64_t blocks = 0;
        while (i < n_tensors && a.n_tensors < OPT_MAX_TENSORS) {
            const pd_tensor_desc& d = descs[i];
            if (d.n == 0) { ++i; continue; }
            PD_REQUIRE(d.grad && d.p_in && d.p_out, PD_EINVAL, "%s: tensor %d has a NULL grad/param pointer", who, i);
            PD_REQUIRE(!need_s0 || d.state0, PD_EINVAL, "%s: tensor %d has no state0 buffer", who, i);
            PD_REQUIRE(!ADAM || d.state1, PD_EINVAL, "%s: tensor %d has no state1 buffer", who, i);
            PD_REQUIRE(pd_aligned(d.grad, grad_fmt == PD_F32 ? 4 : 2) && pd_aligned(d.p_in, 4) && pd_aligned(d.p_out, 4),
                       PD_EINVAL, "%s: tensor %d is not aligned to its element size", who, i);
            uint64_t nb = (d.n + OPT_CHUNK - 1) / OPT_CHUNK;
            if (blocks + nb > 0x7fffffffull) {
                PD_REQUIRE(a.n_tensors > 0, PD_ESHAPE, "%s: tensor %d too large for one launch", who, i);
                break;  // flush what we have, continue with this tensor in the next launch
            }
            bool ok = pd_aligned(d.grad, grad_fmt == PD_F32 ? 16 : 8) && pd_aligned(d.p_in, 16) && pd_aligned(d.p_out, 16) &&
                      (!d.state0 || pd_aligned(d.state0, 16)) && (!d.state1 || pd_aligned(d.state1, 16)) &&
                      (!d.bf16_out || pd_aligned(d.bf16_out, 8));
            int k = a.n_tensors++;
            a.t[k] = d;
            if (ok) a.vec_ok |= (1u << k);
            blocks += nb;
            a.block_start[k + 1] = (uint32_t)blocks;
            ++i;
        }
        if (a.n_tensors == 0) break;
        for (int k = a.n_tensors + 1; k <= OPT_MAX_TENSORS; ++k) a.block_start[k] = (uint32_t)blocks;
        a.grad_fmt = grad_fmt;
        a.out_fmt = out_fmt;
        const dim3 grid((unsigned)blocks), block(OPT_THREADS);
        if (grad16) pd_optim_kernel<ADAM, true, true><<<grid, block, 0, (hipStream_t)stream>>>(a, sh, ah);
        else if (out_rt) pd_optim_kernel<ADAM, false, true><<<grid, block, 0, (hipStream_t)stream>>>(a, sh, ah);
        else pd_optim_kernel<ADAM, false, false><<<grid, block, 0, (hipStream_t)stream>>>(a, sh, ah);
        PD_CHECK_LAUNCH(who);
    }
    return PD_OK;
}

}  // namespace

static int sgd_step(const pd_tensor_desc* descs, int n_tensors, double lr, double momentum, double dampening,
                    double weight_decay, int nesterov, int first_step, double loss_scale, double update_interval,
                    int grad_fmt, int out_fmt, void* stream) {
    PD_REQUIRE(loss_scale != 0.0 && update_interval != 0.0, PD_EINVAL, "pd_sgd_step: zero loss_scale/update_interval");
    SgdHyper sh;
    sh.lr = (float)lr;
    sh.momentum = (float)momentum;
    sh.one_minus_damp = (float)(1.0 - dampening);
    sh.wd = (float)weight_decay;
    sh.loss_scale = (float)loss_scale;
    sh.update_interval = (float)update_interval;
    sh.nesterov = nesterov != 0;
    sh.first_step = first_step != 0;
    sh.has_momentum = momentum != 0.0;
    AdamHyper ah = {};
    return launch_optim<false>(descs, n_tensors, sh, ah, sh.has_momentum, stream, "pd_sgd_step", grad_fmt, out_fmt);
}

extern "C" int pd_sgd_step(const pd_tensor_desc* descs, int n_tensors, double lr, double momentum, double dampening,
                           double weight_decay, int nesterov, int first_step, double loss_scale,
                           double update_interval, void* stream) {
    return sgd_step(descs, n_tensors, lr, momentum, dampening, weight_decay, nesterov, first_step, loss_scale,
                    update_interval, PD_F32, PD_BF16, stream);
}

extern "C" int pd_sgd_step_mixed(const pd_tensor_desc* descs, int n_tensors, double lr, double momentum,
                                 double dampening, double weight_decay, int nesterov, int first_step,
                                 double loss_scale, double update_interval, int grad_format, int out_format,
                                 void* stream) {
    return sgd_step(descs, n_tensors, lr, momentum, dampening, weight_decay, nesterov, first_step, loss_scale,
                    update_interval, grad_format, out_format, stream);
}

static int adam_step(const pd_tensor_desc* descs, int n_tensors, double lr, double beta1, double beta2, double eps,
                     double weight_decay, int64_t step, int eps_mode, double loss_scale, double update_interval,
                     int grad_fmt, int out_fmt, void* stream) {
    PD_REQUIRE(step >= 1, PD_EINVAL, "pd_adam_step: step must be >= 1");
    PD_REQUIRE(eps_mode == 0 || eps_mode == 1, PD_EINVAL, "pd_adam_step: eps_mode must be 0 or 1");
    PD_REQUIRE(loss_scale != 0.0 && update_interval != 0.0, PD_EINVAL, "pd_adam_step: zero loss_scale/update_interval");
    // Bias corrections in double on the host, as torch does with Python floats.
    double bc1 = 1.0 - __builtin_pow(beta1, (double)step);
    double bc2 = 1.0 - __builtin_pow(beta2, (double)step);
    AdamHyper ah;
    ah.w1 = (float)(1.0 - beta1);
    ah.beta2 = (float)beta2;
    ah.one_minus_beta2 = (float)(1.0 - beta2);
    ah.eps = (float)eps;
    ah.wd = (float)weight_decay;
    if (eps_mode == 0) {
        ah.step_size = (float)(lr / bc1);
        ah.bc2_sqrt = (float)__builtin_sqrt(bc2);
    } else {
        ah.step_size = (float)(lr * __builtin_sqrt(bc2) / bc1);
        ah.bc2_sqrt = 1.0f;
    }
    ah.loss_scale = (float)loss_scale;
    ah.update_interval = (float)update_interval;
    ah.eps_mode = eps_mode;
    SgdHyper sh = {};
    return launch_optim<true>(descs, n_tensors, sh, ah, true, stream, "pd_adam_step", grad_fmt, out_fmt);
}

extern "C" int pd_adam_step(const pd_tensor_desc* descs, int n_tensors, double lr, double beta1, double beta2,
                            double eps, double weight_decay, int64_t step, int eps_mode, double loss_scale,
                            double update_interval, void* stream) {
    return adam_step(descs, n_tensors, lr, beta1, beta2, eps, weight_decay, step, eps_mode, loss_scale, update_interval,
                     PD_F32, PD_BF16, stream);
}

extern "C" int pd_adam_step_mixed(const pd_tensor_desc* descs, int n_tensors, double lr, double beta1, double beta2,
                                  double eps, double weight_decay, int64_t step, int eps_mode, double loss_scale,
                                  double update_interval, int grad_format, int out_format, void* stream) {
    return adam_step(descs, n_tensors, lr, beta1, beta2, eps, weight_decay, step, eps_mode, loss_scale, update_interval,
                     grad_format, out_format, stream);
}
