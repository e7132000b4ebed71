/*
 * pipedream_amd.h -- C ABI of libpipedream_amd.so (gfx950 / MI355X).
 *
 * The reference (msr-fiddle/pipedream) has no FFI on its per-stage training
 * step: the path is Python over torch.  Each entry point below therefore cites
 * the reference Python routine whose device work it replaces (paths relative
 * to the reference checkout).  The Python classes in pipedream_amd/ keep the
 * reference's class API and call these functions through ctypes.
 *
 * Conventions
 *   - every function returns 0 on success, a negative PD_E* code for an
 *     argument/shape error detected on the host, or a positive hipError_t;
 *     pd_last_error() returns a thread-local message for the last failure;
 *   - all tensor pointers are DEVICE pointers owned by the caller and must stay
 *     valid until `stream` has executed the launch; nothing here allocates
 *     device memory unless the comment says so;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *     launches are asynchronous;
 *   - fp32 unless a name says otherwise; activations of the conv kernels are
 *     NHWC ("channels last"), filters are KRSC (out-ch, kh, kw, in-ch).
 */
#ifndef PIPEDREAM_AMD_H
#define PIPEDREAM_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PD_OK 0
#define PD_EINVAL (-1)   /* bad argument / null pointer / misaligned pointer   */
#define PD_ESHAPE (-2)   /* shape not supported by the kernel                  */
#define PD_ERANGE (-3)   /* index out of range (ring slot, queue index, ...)   */
#define PD_ENOMEM (-4)   /* host allocation failed                             */

#define PD_ABI_VERSION 1

int pd_abi_version(void);
const char* pd_last_error(void);

/* ------------------------------------------------------------------------- *
 * Weight-version ring.
 * Replaces the deque of cloned state_dicts of OptimizerWithWeightStashing
 * (runtime/optimizer.py:58-62 initialize_queue, :64-85 get_params, :87-116
 * set_params/load_old_params/load_new_params, :156-159 rotation in step).
 *
 * The ring is host-side bookkeeping over ONE caller-allocated flat device
 * buffer of n_versions slots, each slot_stride_bytes long (a multiple of 256).
 * queue index 0 is the oldest entry, n_versions-1 the newest, exactly like the
 * reference's deque(maxlen=num_versions).  All selection logic is integer-only
 * and runs on the host, so which version a backward pass sees is bit-exact.
 * ------------------------------------------------------------------------- */
typedef struct pd_ring pd_ring;

/* All n_versions entries start at version 0 (optimizer.py:58-62). */
int pd_ring_create(void* base, uint64_t slot_stride_bytes, int n_versions, pd_ring** out);
int pd_ring_destroy(pd_ring* ring);
int pd_ring_num_versions(const pd_ring* ring);
/* queue[queue_index] -> physical slot and the version it holds. */
int pd_ring_entry(const pd_ring* ring, int queue_index, int* slot, int64_t* version);
/* device address of a physical slot */
int pd_ring_slot_ptr(const pd_ring* ring, int slot, void** dev_ptr);
/* The physical slot the next push will overwrite (= queue[0]'s storage,
 * optimizer.py:157 `buffered_state_dicts = self.queue[0][0]`). */
int pd_ring_write_slot(const pd_ring* ring, int* slot);
/* deque.append((oldest storage, version)): queue[0]'s slot becomes the newest
 * entry holding `version` (optimizer.py:158).  Returns that slot. */
int pd_ring_push(pd_ring* ring, int64_t version, int* slot);
/* Copy slot `src` into every other slot: the nv clones of initialize_queue
 * (optimizer.py:60-61).  128-bit coalesced copies. n_bytes <= slot stride. */
int pd_ring_broadcast(const pd_ring* ring, int src_slot, uint64_t n_bytes, void* stream);

/* Plain 128-bit coalesced device copy / fill (get_params' per-tensor copy_,
 * optimizer.py:83; zero_grad, optimizer.py:118-120).  n_bytes multiple of 4. */
int pd_copy(void* dst, const void* src, uint64_t n_bytes, void* stream);
int pd_fill_zero(void* dst, uint64_t n_bytes, void* stream);

/* ------------------------------------------------------------------------- *
 * Fused optimizer step + stash.
 * Replaces `p.grad.div_(update_interval)`, the loss-scale division,
 * base_optimizer.step() and the get_params(clone=False) copy into the oldest
 * ring slot (runtime/optimizer.py:137-159) with one pass that reads grad,
 * param and state once and writes the new param into p_out (the ring's write
 * slot; p_out may equal p_in) and the state in place.
 *
 * A launch covers a list of tensors; the flat-buffer case is one tensor.
 * ------------------------------------------------------------------------- */
typedef struct pd_tensor_desc {
    const float* grad;    /* [n] gradient                                        */
    const float* p_in;    /* [n] parameters to update (the loaded version)       */
    float*       p_out;   /* [n] where the updated parameters go                 */
    float*       state0;  /* [n] SGD momentum buffer / Adam exp_avg (may be NULL
                             for SGD with momentum == 0)                         */
    float*       state1;  /* [n] Adam exp_avg_sq (NULL for SGD)                  */
    uint16_t*    bf16_out;/* [n] optional bf16 copy of p_out (NULL = none)       */
    uint64_t     n;       /* elements                                            */
} pd_tensor_desc;

/* torch.optim.SGD maths (selected at runtime/sgd.py:17, run at optimizer.py:151):
 *   g = grad / loss_scale / update_interval          (each only when != 1)
 *   g += weight_decay * p                            (when weight_decay != 0)
 *   buf = first_step ? g : momentum*buf + (1-dampening)*g   (when momentum != 0)
 *   g = nesterov ? g + momentum*buf : buf
 *   p_out = p_in - lr*g
 * `descs` is a HOST array; it is copied into kernel arguments. */
int pd_sgd_step(const pd_tensor_desc* descs, int n_tensors,
                double lr, double momentum, double dampening, double weight_decay,
                int nesterov, int first_step,
                double loss_scale, double update_interval, void* stream);

/* The same two steps for 16-bit model parameters with fp32 masters -- the branch of
 * OptimizerWithWeightStashing.step that runtime/optimizer.py:137-155 takes when model_parameters is given
 * (apex.fp16_utils.model_grads_to_master_grads, the division by loss_scale, the base optimizer on the
 * masters, master_params_to_model_params) as one launch: desc.grad points at the MODEL's gradient in
 * grad_format (PD_F32, PD_BF16 or PD_F16; widened exactly), p_in / p_out / state are the fp32 masters
 * and state, and desc.bf16_out receives the new parameters rounded to out_format (PD_BF16 or PD_F16):
 * the 16-bit model copy, written straight into the version ring's slot. */
#define PD_F32 0
#define PD_BF16 1
#define PD_F16 2
int pd_sgd_step_mixed(const pd_tensor_desc* descs, int n_tensors,
                      double lr, double momentum, double dampening, double weight_decay,
                      int nesterov, int first_step, double loss_scale, double update_interval,
                      int grad_format, int out_format, void* stream);
int pd_adam_step_mixed(const pd_tensor_desc* descs, int n_tensors,
                       double lr, double beta1, double beta2, double eps, double weight_decay,
                       int64_t step, int eps_mode, double loss_scale, double update_interval,
                       int grad_format, int out_format, void* stream);

/* torch.optim.Adam maths (selected at runtime/adam.py:16):
 * eps_mode 0 = installed-torch form  p -= (lr/bc1) * m / (sqrt(v)/sqrt(bc2) + eps)
 * eps_mode 1 = PyTorch-1.1 form      p -= (lr*sqrt(bc2)/bc1) * m / (sqrt(v) + eps)
 * `step` is the 1-based step count AFTER the increment. */
int pd_adam_step(const pd_tensor_desc* descs, int n_tensors,
                 double lr, double beta1, double beta2, double eps, double weight_decay,
                 int64_t step, int eps_mode,
                 double loss_scale, double update_interval, void* stream);

/* ------------------------------------------------------------------------- *
 * Stage compute.  These replace the library kernels (cuBLAS / cuDNN / ATen)
 * that the torch.nn modules of a reference stage call in
 * StageRuntime._run_forward (runtime/runtime.py:505-546) and that
 * torch.autograd.backward replays in run_backward (runtime/runtime.py:606-608).
 * ------------------------------------------------------------------------- */

/* Row-major fp32 GEMM on MFMA:  C[M,N] = op(A) op(B) (+ bias[N]) (+ beta*C) (ReLU)
 * op(A) is [M,K]: A is stored [M][lda] (trans_a=0) or [K][lda] (trans_a=1);
 * op(B) is [K,N]: B is stored [K][ldb] (trans_b=0) or [N][ldb] (trans_b=1).
 * torch.nn.Linear forward  = (0,1): Y = X W^T + b   (stage3.py:19 Linear layers)
 * its input gradient       = (0,0): dX = dY W
 * its weight gradient      = (1,0): dW = dY^T X */
int pd_gemm_f32(int trans_a, int trans_b, int M, int N, int K,
                const float* A, int lda, const float* B, int ldb,
                float beta, float* C, int ldc, const float* bias, int relu, void* stream);
/* The same product split over k for problems with too few output tiles to fill the GPU (the
 * recurrent LSTM products with M = batch, the VGG classifier layers with M = 64):
 * partials[s][M][N] (dense) = op(A)[:, k in split s] op(B)[k in split s, :].  The caller sums the
 * partials in index order (deterministic): pd_splitk_reduce_f32, or the LSTM cell kernels. */
int pd_gemm_splitk_f32(int trans_a, int trans_b, int M, int N, int K,
                       const float* A, int lda, const float* B, int ldb,
                       float* partials, int splits, void* stream);
/* C[M][ldc] = sum_s partials[s] (+ bias[N]) (+ beta*C) (ReLU); N and ldc multiples of 4. */
int pd_splitk_reduce_f32(const float* partials, int splits, int M, int N, const float* bias, int relu,
                         float beta, float* C, int ldc, void* stream);

/* out[s][n] = sum over the s-th of `splits` row ranges of x[m][n]  (bias gradients).
 * With splits == 1 and beta != 0 the sum is added to beta*out. */
int pd_colsum_f32(const float* x, float* out, uint64_t M, int N, uint64_t ld, int splits, float beta, void* stream);

/* torch.nn.ReLU forward / backward (stage0.py:13). dx = dy where y > 0. */
int pd_relu_fwd_f32(const float* x, float* y, uint64_t n, void* stream);
int pd_relu_bwd_f32(const float* dy, const float* y, float* dx, uint64_t n, void* stream);

/* torch.nn.Dropout (stage3.py:20,23) given its keep-mask (one byte per element, 0/1):
 * y = mask ? x*scale : 0, scale = 1/(1-p); the same call applied to dy is the backward. */
int pd_mask_scale_f32(const float* x, const uint8_t* mask, float* y, uint64_t n, float scale, void* stream);

/* torch.nn.MaxPool2d(kernel_size=2, stride=2) on NHWC tensors (stage1.py:11).
 * y is [N, H/2, W/2, C].  relu != 0 applies a ReLU to the pooled value, which equals
 * pooling a ReLU'd input (the ReLU + MaxPool2d pair at the head of stage1.py:10-11).
 * Backward writes all of dx; first maximum wins ties.
 * relu_mask != 0 additionally zeroes dx where the window maximum is <= 0. */
int pd_maxpool2x2_fwd_nhwc_f32(const float* x, float* y, int N, int H, int W, int C, int relu, void* stream);
int pd_maxpool2x2_bwd_nhwc_f32(const float* x, const float* dy, float* dx, int N, int H, int W, int C,
                               int relu_mask, void* stream);
/* The same pooling with an index tensor: the forward also writes one byte per output element (bits 0-1:
 * position of the first maximum in the window, row-major; bit 2: the maximum is positive); the backward
 * reads the pooled gradient and that byte instead of the whole input (5 instead of 20 bytes read per
 * output element) and writes dx [N,H,W,C]. */
int pd_maxpool2x2_fwd_idx_nhwc_f32(const float* x, float* y, uint8_t* idx, int N, int H, int W, int C, int relu,
                                   void* stream);
int pd_maxpool2x2_bwd_idx_nhwc_f32(const float* dy, const uint8_t* idx, float* dx, int N, int H, int W, int C,
                                   int relu_mask, void* stream);

/* torch.nn.CrossEntropyLoss(reduction='mean') -- the criterion the caller appends to
 * the module list (main_with_runtime.py:126, applied at runtime/runtime.py:523-526).
 * loss[0] = mean over non-ignored rows of (logsumexp(x_b) - x_b[target_b]);
 * row_loss[B], lse[B], count[1] are outputs kept for the backward pass.
 * Backward: dlogits = (softmax(x) - onehot(target)) * grad_loss[0] / count[0]. */
int pd_xent_fwd_f32(const float* logits, const int64_t* target, float* loss, float* row_loss, float* lse,
                    float* count, int B, int C, int ld, int64_t ignore_index, void* stream);
int pd_xent_bwd_f32(const float* logits, const int64_t* target, const float* lse, const float* grad_loss,
                    const float* count, float* dlogits, int B, int C, int ld, int ldd,
                    int64_t ignore_index, void* stream);

/* torch.nn.Conv2d(C, K, kernel_size=3, stride=1, padding=1) on NHWC activations with a
 * KRSC filter (the memory order of a channels_last [K,C,3,3] weight); the conv layers of
 * the VGG16 stages (vgg16/gpus=4_straight/stage0.py:12-14).  Optional bias and fused
 * ReLU (stage0.py:13).  y is [N,H,W,K]. */
int pd_conv3x3_fwd_nhwc_f32(const float* x, const float* w, const float* bias, float* y,
                            int N, int H, int W, int C, int K, int relu, void* stream);
/* out[c][r][s][k] = w[k][2-r][2-s][c]: with this filter the forward kernel computes the
 * input gradient. */
int pd_conv3x3_filter_rot180_f32(const float* w, float* out, int K, int C, void* stream);
/* Input gradient dx[N,H,W,C] = conv3x3(dy[N,H,W,K], w_rot[C][3][3][K]).  If relu_out is not
 * NULL it is the forward output of the fused conv+ReLU layer and dy is taken as 0 where
 * relu_out <= 0 (the ReLU backward applied while the tile is loaded).  If x_rectified is not
 * NULL it is this layer's own input [N,H,W,C], itself the output of a ReLU, and dx is written
 * as 0 where x_rectified <= 0: the ReLU backward of the PRODUCING layer applied in this
 * kernel's epilogue, so that layer's gradient kernels need no mask (torch.nn.ReLU(inplace=True)
 * between two convolutions, vgg16/gpus=4_straight/stage0.py:13-15). */
int pd_conv3x3_dgrad_nhwc_f32(const float* dy, const float* w_rot, const float* relu_out,
                              const float* x_rectified, float* dx,
                              int N, int H, int W, int K, int C, void* stream);
/* Tuning and test hook for the three pd_conv3x3_winograd_fwd* entry points.  A batch of images whose height is
 * even but no multiple of 16 is processed as one tall image; if its width is a multiple of 8 (4) but not of 16
 * pixels, a work item can then be two (four) pieces of 16 x 8 (16 x 4) pixels instead of one 16 x 16 square, which
 * leaves no padding columns.  mode 0 (default): pieces when they lower the number of work items of the busiest
 * compute unit; 1: pieces wherever the shape allows; -1: never.  Results are bit-identical either way.
 * Process-wide, not thread-safe against concurrent convolution calls.  No counterpart in the reference. */
int pd_conv3x3_winograd_set_pieces(int mode);
/* Tuning and test hook for pd_conv3x3_winograd_wgrad_nhwc_f32.  Its blocks sum over strips of eight 2 x 2 tiles:
 * 2 x 16 pixels of one image, or, upright, 16 rows x 2 columns of the batch taken as one image of N * H rows
 * (H, W even, H >= 14), which leaves no padding columns at widths that are no multiple of 16.  mode 0 (default):
 * upright strips exactly where the width is no multiple of 16; 1: never; 2: wherever the shape allows.  Results
 * differ by the summation order only.  Process-wide.  No counterpart in the reference. */
int pd_conv3x3_winograd_set_wgrad_strips(int mode);

/* The same convolution (and, with rot180, its input gradient) by the Winograd algorithm
 * F(2x2, 3x3) in fp32: 2.25x fewer multiplications; results agree with the direct kernels to
 * fp32 rounding (about 2e-6 relative).  Needs C % 8 == 0 and K % 4 == 0
 * (pd_conv3x3_winograd_supported() returns 1).  pd_conv3x3_winograd_filter_f32() writes the
 * transformed filter (pd_conv3x3_winograd_filter_bytes() bytes) for a convolution with C input
 * and K output channels: from w[K][3][3][C], or with rot180 != 0 from the forward filter
 * w[C][3][3][K] of the layer whose input gradient is wanted (then "C" is that layer's output and
 * "K" its input channel count).  pd_conv3x3_winograd_fwd_nhwc_f32() then computes
 * y[N,H,W,K] from x[N,H,W,C]; in_mask / out_mask (may be NULL) have the meaning of relu_out /
 * x_rectified in pd_conv3x3_dgrad_nhwc_f32.  (torch.nn.Conv2d, vgg16/gpus=4_straight/stage0.py:12-14.) */
int pd_conv3x3_winograd_supported(int C, int K);
int pd_conv3x3_winograd_filter_bytes(int C, int K, uint64_t* bytes);
int pd_conv3x3_winograd_filter_f32(const float* w, float* u, int C, int K, int rot180, void* stream);
int pd_conv3x3_winograd_fwd_nhwc_f32(const float* x, const float* u, const float* bias,
                                     const float* in_mask, const float* out_mask, float* y,
                                     int N, int H, int W, int C, int K, int relu, void* stream);
/* The same forward followed by 2x2 / stride-2 max pooling in the kernel's epilogue (a convolution and the
 * ReLU + MaxPool2d behind it: vgg16/gpus=4_straight/stage0.py:14 + stage1.py:10-11 when they share a
 * stage, vgg16/gpus=2/stage0.py:16-17 + stage1.py:10-11).  Writes y_pool [N,H/2,W/2,K] and one index
 * byte per pooled element (bits 0-1: position of the first maximum in the window, row-major; bit 2: the
 * maximum is positive) instead of the full-resolution output; pd_maxpool2x2_bwd_idx_nhwc_f32 turns the
 * pooled gradient back into the convolution's output gradient. */
int pd_conv3x3_winograd_fwd_pool_nhwc_f32(const float* x, const float* u, const float* bias, float* y_pool,
                                          uint8_t* idx, int N, int H, int W, int C, int K, int relu,
                                          void* stream);
/* The same kernel as the input gradient of a convolution whose input came out of such a pooling (this
 * epilogue's, or pd_maxpool2x2_fwd_idx_nhwc_f32's) behind a ReLU: x is the convolution's output gradient,
 * u its filter transformed with rot180, idx [N,H,W,K] the pooling's index bytes.  Besides y [N,H,W,K],
 * the gradient with respect to the pooled tensor masked where the recorded maximum was not positive, it
 * writes y_full [N,2H,2W,K] = pd_maxpool2x2_bwd_idx_nhwc_f32(y, idx, relu_mask = 1): the backward of the
 * MaxPool2d + ReLU pair (stage1.py:10-11) leaves the convolution kernel's epilogue instead of a kernel of
 * its own that re-reads y.  Needs the full-resolution size to be exactly 2H x 2W. */
int pd_conv3x3_winograd_fwd_unpool_nhwc_f32(const float* x, const float* u, const uint8_t* idx, float* y,
                                            float* y_full, int N, int H, int W, int C, int K, void* stream);
/* Weight (and optional bias) gradient of the same convolution in the Winograd domain: sums
 * dU = sum over 2x2 output tiles of (A dY A^T) (B^T d B) in persistent blocks, adds the blocks' partial
 * sums in fixed order and applies G^T . G.  Deterministic; agrees with pd_conv3x3_wgrad_nhwc_f32 to
 * fp32 rounding.  Needs C and K multiples of 64 with (C/64)*(K/64) a power of two <= 256
 * (pd_conv3x3_winograd_wgrad_supported() returns 1) and a workspace of
 * pd_conv3x3_winograd_wgrad_workspace_bytes() bytes.  dw is [K][3][3][C]; dbias may be NULL.
 * (Backward of torch.nn.Conv2d, vgg16/gpus=4_straight/stage0.py:12-14.) */
int pd_conv3x3_winograd_wgrad_supported(int C, int K);
int pd_conv3x3_winograd_wgrad_workspace_bytes(int C, int K, uint64_t* bytes);
int pd_conv3x3_winograd_wgrad_nhwc_f32(const float* x, const float* dy, float* dw, float* dbias,
                                       void* workspace, uint64_t workspace_bytes,
                                       int N, int H, int W, int C, int K, void* stream);
/* Weight and (optional, dbias may be NULL) bias gradient of the same convolution:
 * dw[k][r][s][c] = sum_{n,y,x} dy[n,y,x,k] * x[n,y+r-1,x+s-1,c].  Deterministic two-pass
 * reduction through a caller-provided workspace of pd_conv3x3_wgrad_workspace_bytes().
 * relu_out (may be NULL) masks dy as in pd_conv3x3_dgrad_nhwc_f32. */
int pd_conv3x3_wgrad_workspace_bytes(int N, int H, int W, int C, int K, uint64_t* bytes);
int pd_conv3x3_wgrad_nhwc_f32(const float* x, const float* dy, const float* relu_out, float* dw, float* dbias,
                              void* workspace, uint64_t workspace_bytes,
                              int N, int H, int W, int C, int K, void* stream);
/* pd_conv3x3_wgrad_nhwc_f32 for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc); it has no counterpart in the reference.
 * Same arguments without the workspace, same results bit for bit: the partial sums go to a fixed array
 * of PD_CONV3X3_WGRAD_NOALLOC_MAX_WORKSPACE bytes in device memory that every GPU the library runs on
 * holds until the process ends.  The call allocates and frees nothing.  A shape whose
 * pd_conv3x3_wgrad_workspace_bytes() exceeds that size is refused with PD_ESHAPE (the few-channel first
 * layer fits at any batch size; 64-channel layers up to about 100k pixels per call).  All calls on one
 * GPU share the array: calls that overlap on one GPU (different streams or threads) race.
 * The first call on a device looks up the array's device address (hipGetSymbolAddress, under a mutex)
 * and keeps it; make that first call outside graph capture.  The address is that of the device current
 * at the call (hipGetDevice), so `stream` must belong to the current device. */
#define PD_CONV3X3_WGRAD_NOALLOC_MAX_WORKSPACE (16u << 20)
int pd_conv3x3_wgrad_noalloc_nhwc_f32(const float* x, const float* dy, const float* relu_out, float* dw,
                                      float* dbias, int N, int H, int W, int C, int K, void* stream);

/* torch.nn.LSTM cell (gnmt_large/gpus=4/stage0.py:14-19), gate order i,f,g,o.
 * Forward, one time step: gates[B][4H] holds x W_ih^T on entry, to which the n_rec split-k
 * partial products rec[n_rec][B][4H] of h_prev W_hh^T (pd_gemm_splitk_f32; n_rec may be 0)
 * and the biases are added; on exit it holds the activated gates.  Biases and c_prev may be
 * NULL (= 0).  c = f*c_prev + i*g, h = o*tanh(c). */
int pd_lstm_cell_fwd_f32(float* gates, const float* rec, int n_rec, const float* b_ih, const float* b_hh,
                         const float* c_prev, float* c_out, float* h_out, int B, int H, void* stream);
/* Backward of that step: dh = dy + sum of the n_rec partials dh_rec[n_rec][B][H] (dh_rec may be
 * NULL); dc_io holds dL/dc_t from the next step on entry (ignored when first_step != 0, i.e.
 * for the last time step) and dL/dc_prev on exit; dgates[B][4H] = gradients of the gate
 * pre-activations. */
int pd_lstm_cell_bwd_f32(const float* gates, const float* c_prev, const float* c, const float* dy,
                         const float* dh_rec, int n_rec, float* dc_io, float* dgates, int B, int H,
                         int first_step, void* stream);
/* The time loop of one torch.nn.LSTM layer (stage0.py:14-19; batch_first=False, zero initial state) over the
 * two calls above, issued from native code: a layer of T = 50 steps is 99 launches and one call.
 * Forward: gates[T][B][4H] holds x_t W_ih^T on entry and the activated gates on exit; c[T][B][H] and
 * y[T][B][H] (= h_t) are written; rec[splits][B][4H] is scratch for the k-split products h_{t-1} W_hh^T
 * (w_hh[4H][H]; may be NULL when T == 1).  Backward: dy[T][B][H] is dL/dy; dgates[T][B][4H] is written;
 * dh_rec[splits][B][H] and dc[B][H] are scratch.  The weight and input gradients are plain products of dgates
 * (pd_gemm_f32).  All pointers 16-byte aligned. */
int pd_lstm_recurrence_fwd_f32(float* gates, const float* w_hh, const float* b_ih, const float* b_hh, float* rec,
                               int splits, float* c, float* y, int T, int B, int H, void* stream);
int pd_lstm_recurrence_bwd_f32(const float* gates, const float* c, const float* dy, const float* w_hh,
                               float* dh_rec, int splits, float* dc, float* dgates, int T, int B, int H,
                               void* stream);
/* y = a + b: the residual connections `out13 = out13 + out10` (stage0.py:32, 36). */
int pd_add_f32(const float* a, const float* b, float* y, uint64_t n, void* stream);
/* torch.nn.Embedding (stage0.py:10): out[p][:] = weight[ids[p]][:].  Backward writes the
 * whole dense dweight[V][D] (zeros for unused rows and for padding_idx; pass -1 for none),
 * summing duplicates in position order. */
int pd_embedding_fwd_f32(const int64_t* ids, const float* weight, float* out, int n_tokens, int D, int64_t V,
                         void* stream);
int pd_embedding_bwd_f32(const int64_t* ids, const float* dout, float* dweight, int n_tokens, int D, int64_t V,
                         int64_t padding_idx, void* stream);

/* ------------------------------------------------------------------------- *
 * bf16 transformer stage (6 pre-LN layers, bf16 compute, fp32 master weights).
 * The reference's checked-out branch has no such stage (PipeDream-2BW is on another
 * branch, README.md:7-8); these entry points do for it what cuBLAS / ATen do for the
 * torch.nn layers of the reference's stages (runtime/runtime.py:529-530, :606-608).
 * bf16 tensors are passed as uint16_t*.
 * ------------------------------------------------------------------------- */

/* Strided-batched bf16 GEMM, fp32 accumulation on MFMA:
 *   C = alpha * op(A) op(B) (+ bias[N]) (+ residual) (+ beta*C, fp32 output only)
 * Layout flags as pd_gemm_f32.  C is bf16 (out_f32 = 0) or fp32.  Batch entry
 * (o, i), o < batch_outer, i < batch_inner, offsets the operands by
 * strides = {sa_o, sa_i, sb_o, sb_i, sc_o, sc_i} elements (NULL when unbatched); the
 * residual shares C's offsets.  Leading dimensions, contiguous extents and A/B batch
 * strides must be multiples of 8 elements. */
int pd_gemm_bf16(int trans_a, int trans_b, int M, int N, int K,
                 const uint16_t* A, int lda, const uint16_t* B, int ldb,
                 void* C, int ldc, int out_f32, float alpha, float beta,
                 const float* bias, const uint16_t* residual, int ldr,
                 int batch_outer, int batch_inner, const int64_t* strides, void* stream);
/* Tuning and test hook: force the tile of the direct-to-LDS kernel behind pd_gemm_bf16 / pd_gemm_bf16_gelu
 * for products it can take (K a multiple of 128): (128, 128) or (256, 256); (0, 0) restores the built-in
 * choice (256 x 256 when there are at least 192 such tiles, else 128 x 128).  Process-wide,
 * not thread-safe against concurrent GEMM calls.  No counterpart in the reference (its GEMMs are library calls). */
int pd_gemm_bf16_set_tile(int bm, int bn);

/* Operand preparation for an fp32 product computed on the bf16 matrix pipes (no counterpart in the reference,
 * whose fp32 products are library calls).  x[rows][ld] (cols used) is written as six bf16 slots of three terms
 * x1 = bf16(x), x2 = bf16(x - x1), x3 = bf16(x - x1 - x2) (x = x1 + x2 + x3 exactly): slots 1 3 2 2 1 1 for the
 * A operand (b_side = 0), 3 1 1 2 2 1 for the B operand (b_side = 1).  stacked = 0: out[rows][6 cols], the slots
 * side by side (an operand whose columns are the reduction index); stacked = 1: out[6 rows][cols], six row blocks
 * (rows are the reduction index).  pd_gemm_bf16 over the six-fold reduction with fp32 output then adds
 * a3 b1 + a1 b3 + a2 b1 + a2 b2 + a1 b2 + a1 b1: the fp32 product up to 2^-24 relative per term, with fp32
 * accumulation.  cols and ld multiples of 4; x 16-byte, out 8-byte aligned. */
int pd_split3_bf16_f32(const float* x, int64_t rows, int64_t cols, int64_t ld, uint16_t* out, int b_side,
                       int stacked, void* stream);

/* The same GEMM (unbatched, bf16 output) with the exact GELU of a feed-forward block in its epilogue.
 * backward = 0:  C = op(A) op(B) + bias  (the pre-activation, kept for the backward) and aux = gelu(C),
 *                with C taken as rounded to bf16, both written by the kernel;
 * backward = 1:  C = (op(A) op(B)) * gelu'(aux), aux = the stored pre-activation: the gradient with respect
 *                to it, straight from the GEMM that produces the gradient of the activation.
 * aux is [M][ld_aux] bf16.  erf is evaluated by Abramowitz & Stegun 7.1.26 (absolute error < 1.5e-7). */
int pd_gemm_bf16_gelu(int backward, int trans_a, int trans_b, int M, int N, int K, const uint16_t* A, int lda,
                      const uint16_t* B, int ldb, uint16_t* C, int ldc, const float* bias, uint16_t* aux,
                      int ld_aux, void* stream);

/* LayerNorm over the last dimension H (multiple of 8, <= 2048): bf16 in/out, fp32 affine
 * parameters and statistics.  Backward writes dx (+ residual, bf16 [M][H] or NULL: the gradient that
 * bypasses the normalisation in a pre-LN layer, dx = LN'(dy) + residual) and per-block partial sums of
 * dgamma / dbeta, [pd_layernorm_bwd_partials(M)][H] each, to be summed with pd_colsum_f32 or pd_colsum_batch. */
int pd_layernorm_fwd_bf16(const uint16_t* x, const float* gamma, const float* beta, uint16_t* y,
                          float* mean, float* rstd, int M, int H, float eps, void* stream);
int pd_layernorm_bwd_partials(int M);
int pd_layernorm_bwd_bf16(const uint16_t* dy, const uint16_t* x, const float* gamma, const float* mean,
                          const float* rstd, uint16_t* dx, const uint16_t* residual, float* part_dgamma,
                          float* part_dbeta, int M, int H, void* stream);

/* Fused attention of one transformer layer.  qkv is [batch*seq][3H] (Q | K | V, the heads contiguous
 * inside each, H = heads*head_dim).  Forward: ctx [batch*seq][H] = softmax(Q K^T / sqrt(head_dim)) V; the
 * scores stay in registers (fp32).  Optional outputs (NULL to skip): probs [batch][heads][seq][seq], the
 * bf16 probabilities, and lse2 [batch][heads][seq] (fp32), log2 of the softmax denominator in the scaled
 * base-2 domain, from which the backward pass recomputes the probabilities:
 * P[q][k] = 2^(s_qk log2(e) / sqrt(head_dim) - lse2[q]).
 * Supported shapes: pd_attention_fwd_supported() != 0 (head_dim 64, seq 128 / 256 / 512); other shapes
 * use pd_gemm_bf16 + pd_softmax_fwd_bf16 / pd_softmax_bwd_bf16. */
int pd_attention_fwd_supported(int seq, int head_dim);
int pd_attention_fwd_bf16(const uint16_t* qkv, uint16_t* ctx, uint16_t* probs, float* lse2, int batch, int seq,
                          int heads, int head_dim, void* stream);
/* Backward: dqkv [batch*seq][3H] from dctx = dL/dctx, the forward's ctx and lse2.  Two kernels: the
 * query side (dQ; also writes delta [batch][heads][seq] = sum_d dctx*ctx, workspace owned by the
 * caller) and the key side (dK, dV).  Neither reads or writes a [seq][seq] tensor. */
int pd_attention_bwd_bf16(const uint16_t* qkv, const uint16_t* ctx, const uint16_t* dctx, const float* lse2,
                          float* delta, uint16_t* dqkv, int batch, int seq, int heads, int head_dim, void* stream);
/* Row softmax (row length multiple of 8, <= 2048) and its backward dx = y*(dy - sum(dy*y)). */
int pd_softmax_fwd_bf16(const uint16_t* x, uint16_t* y, int64_t rows, int n, void* stream);
int pd_softmax_bwd_bf16(const uint16_t* y, const uint16_t* dy, uint16_t* dx, int64_t rows, int n, void* stream);

/* Exact (erf) GELU and its backward dx = dy * gelu'(x); element-wise add; casts; column sums
 * of a bf16 matrix into fp32 partials out[splits][N]. */
int pd_gelu_fwd_bf16(const uint16_t* x, uint16_t* y, uint64_t n, void* stream);
int pd_gelu_bwd_bf16(const uint16_t* x, const uint16_t* dy, uint16_t* dx, uint64_t n, void* stream);
int pd_add_bf16(const uint16_t* a, const uint16_t* b, uint16_t* y, uint64_t n, void* stream);
int pd_cast_f32_to_bf16(const float* x, uint16_t* y, uint64_t n, void* stream);
int pd_cast_bf16_to_f32(const uint16_t* x, float* y, uint64_t n, void* stream);
int pd_colsum_bf16(const uint16_t* x, float* out, uint64_t M, int N, uint64_t ld, int splits, void* stream);
/* Up to 8 column sums in two launches (all bias and LayerNorm parameter gradients of one layer's backward
 * instead of a dozen launches of a few microseconds): job j sums the rows of x[j], a bf16 matrix
 * (is_bf16[j] != 0: `splits` row ranges first, into the workspace, then their sum) or an fp32 matrix (e.g.
 * the partials pd_layernorm_bwd_bf16 leaves), [M[j]][N[j]] with leading dimension ld[j], into out[j][N[j]]
 * (+ beta[j] * out[j]).  The argument arrays are host arrays; workspace: device memory of
 * pd_colsum_batch_workspace_floats() floats.  (torch.nn.Linear / LayerNorm backward, as pd_colsum_bf16.) */
int pd_colsum_batch_workspace_floats(int n_jobs, const int* is_bf16, const int* N, int splits, uint64_t* floats);
int pd_colsum_batch(int n_jobs, const void* const* x, const int* is_bf16, float* const* out, const uint64_t* M,
                    const int* N, const uint64_t* ld, const float* beta, float* workspace,
                    uint64_t workspace_floats, int splits, void* stream);

/* The label-smoothing criterion of the translation stages, LabelSmoothing.forward
 * (runtime/translation/seq2seq/train/smoothing.py:23-34): logits [R][V] (R = seq*batch rows of leading
 * dimension ld), fp32 log-softmax per row,
 *   row_loss = (1 - smoothing) * (lse - x[target]) + smoothing * (lse - mean(x)),  0 where target ==
 *   padding_idx,   loss[0] = sum(row_loss) / divisor   (divisor = the batch size, smoothing.py:33).
 * row_loss[R] and lse[R] are outputs; the backward pass reads lse:
 *   dlogits = (softmax(x) - (1 - smoothing) * onehot(target) - smoothing / V) * grad_loss[0] / divisor,
 * 0 in padding rows.  A target outside [0, V) other than padding_idx makes the loss NaN. */
int pd_label_smoothing_fwd_f32(const float* logits, const int64_t* target, float* loss, float* row_loss,
                               float* lse, int R, int V, int64_t ld, int64_t padding_idx, float smoothing,
                               float divisor, void* stream);
int pd_label_smoothing_bwd_f32(const float* logits, const int64_t* target, const float* lse,
                               const float* grad_loss, float* dlogits, int R, int V, int64_t ld, int64_t ldd,
                               int64_t padding_idx, float smoothing, float divisor, void* stream);

/* revert_varlen_tensor (runtime/translation/seq2seq/csrc/pack_utils_kernel.cu:25-62, bound to Python at
 * pack_utils.cpp:37): in/out are [T][B] rows of row_bytes bytes (any element type of 2 or 4 bytes),
 * consecutive rows in_pitch / out_pitch bytes apart (= row_bytes for a dense tensor; larger when the rows
 * are one half of a wider tensor, e.g. one direction of a bidirectional layer's [T][B][2H] output),
 *   out[t][b] = t < lengths[b] ? in[lengths[b] - 1 - t][b] : 0.
 * lengths is B int64 values in DEVICE memory (the reference takes a host tensor, builds T*B offsets on the
 * host and uploads them on every call); 0 < lengths[b] <= T is the caller's duty.  in != out.
 * pd_length_mask_apply: out[t][b] = t < lengths[b] ? in[t][b] : 0 -- the product with the mask of
 * set_mask_cpp in EmuBidirLSTM.emu_bidir_lstm (seq2seq/models/encoder.py:51,55); in == out is allowed. */
int pd_revert_varlen(const void* in, void* out, const int64_t* lengths, int64_t T, int64_t B, int64_t row_bytes,
                     int64_t in_pitch, int64_t out_pitch, void* stream);
int pd_length_mask_apply(const void* in, void* out, const int64_t* lengths, int64_t T, int64_t B,
                         int64_t row_bytes, int64_t in_pitch, int64_t out_pitch, void* stream);
/* set_mask_cpp (runtime/translation/seq2seq/csrc/pack_utils.cpp:13-31): host code on host memory, as in
 * the reference: mask[t][b] = lengths[b] > t for t < T (the reference takes T = lengths[0]). */
int pd_set_mask_u8(const int64_t* lengths, int64_t B, int64_t T, uint8_t* mask);

#ifdef __cplusplus
}
#endif
#endif /* PIPEDREAM_AMD_H */
