"""Stage building blocks: ``torch.nn.Module``s whose forward and backward run on the
hand-written HIP kernels of ``libpipedream_amd.so``.

They carry the parameter names, shapes and initialisation of the ``torch.nn`` layers
used by the reference's generated stage modules (``weight`` / ``bias``; e.g.
runtime/image_classification/models/vgg16/gpus=4_straight/stage0.py:10-33), so their
``state_dict()`` is interchangeable with the reference's.  Every backward reads the
parameter tensors as they are *at backward time*, i.e. the weight version that
``load_old_params`` made current -- the semantics of the reference's in-place
``load_state_dict`` (runtime/optimizer.py:87-112).
"""
import math

import torch

from . import ops


# --------------------------------------------------------------------------------------
# Linear
# --------------------------------------------------------------------------------------
class _LinearFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, relu):
        x2 = x.reshape(-1, x.shape[-1])
        if x2.stride(-1) != 1 or (x2.size(0) > 1 and x2.stride(0) < x2.size(1)):
            x2 = x2.contiguous()
        y = ops.gemm(x2, weight, trans_b=True, bias=bias, relu=relu)
        ctx.relu = relu
        ctx.has_bias = bias is not None
        ctx.x_shape = x.shape
        ctx.save_for_backward(x2, weight, y if relu else None)
        return y.view(*x.shape[:-1], weight.shape[0])

    @staticmethod
    def backward(ctx, dy):
        x2, weight, y = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.shape[-1])
        if ctx.relu:
            dy2 = ops.relu_backward(dy2, y)
        elif dy2.stride(-1) != 1 or (dy2.size(0) > 1 and dy2.stride(0) < dy2.size(1)):
            dy2 = dy2.contiguous()
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = ops.gemm(dy2, weight).view(ctx.x_shape)
        if ctx.needs_input_grad[1]:
            dw = ops.gemm(dy2, x2, trans_a=True)
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = ops.colsum(dy2)
        return dx, dw, db, None


class _Linear16Fn(torch.autograd.Function):
    """The same layer with 16-bit (bfloat16) parameters and activations, as the modules of a stage built with
    ``StageRuntime(fp16=True)`` hold them (runtime/runtime.py:227-229): products on the bf16 MFMA GEMM with
    fp32 accumulation, gradients returned in the parameters' format (what the mixed-precision optimizer step
    reads, runtime/optimizer.py:137-145)."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        x2 = ops.cast_bf16(x.reshape(-1, x.shape[-1])) if x.dtype == torch.float32 else x.reshape(-1, x.shape[-1])
        x2 = x2.contiguous()
        y = ops.gemm_bf16(x2, weight, trans_b=True, bias=ops.cast_f32(bias) if bias is not None else None)
        ctx.has_bias = bias is not None
        ctx.x_shape, ctx.x_dtype = x.shape, x.dtype
        ctx.save_for_backward(x2, weight)
        return y.view(*x.shape[:-1], weight.shape[0])

    @staticmethod
    def backward(ctx, dy):
        x2, weight = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.shape[-1]).contiguous()
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = ops.gemm_bf16(dy2, weight).view(ctx.x_shape)
            if ctx.x_dtype == torch.float32:
                dx = ops.cast_f32(dx)
        if ctx.needs_input_grad[1]:
            dw = ops.gemm_bf16(dy2, x2, trans_a=True)
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = ops.cast_bf16(ops.colsum_bf16(dy2))
        return dx, dw, db


class Linear(torch.nn.Module):
    """``torch.nn.Linear`` (optionally with the following ReLU fused into the GEMM epilogue).  Converted to
    bfloat16 (``module.bfloat16()``, or ``StageRuntime(fp16=True, half_dtype=torch.bfloat16)``) the layer runs on
    the bf16 GEMM; float16 parameters have no kernel here and raise."""

    def __init__(self, in_features, out_features, bias=True, relu=False):
        super(Linear, self).__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.relu = relu
        self.weight = torch.nn.Parameter(torch.empty(out_features, in_features))
        self.bias = torch.nn.Parameter(torch.empty(out_features)) if bias else None
        self.reset_parameters()

    def reset_parameters(self):
        torch.nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            bound = 1 / math.sqrt(self.in_features) if self.in_features > 0 else 0
            torch.nn.init.uniform_(self.bias, -bound, bound)

    def forward(self, x):
        if self.weight.dtype != torch.float32:
            if self.weight.dtype != torch.bfloat16:
                raise NotImplementedError("Linear with %s parameters: the 16-bit GEMM of this build is bfloat16 "
                                          "(StageRuntime(fp16=True, half_dtype=torch.bfloat16))" % self.weight.dtype)
            if self.relu:
                raise NotImplementedError("Linear(relu=True) has no 16-bit kernel; follow the layer with GELU or "
                                          "keep the stage in fp32")
            return _Linear16Fn.apply(x, self.weight, self.bias)
        return _LinearFn.apply(x, self.weight, self.bias, self.relu)

    def extra_repr(self):
        return "in_features={}, out_features={}, bias={}, relu={}".format(
            self.in_features, self.out_features, self.bias is not None, self.relu)


# --------------------------------------------------------------------------------------
# Conv2d 3x3
# --------------------------------------------------------------------------------------
class PoolGradLink(object):
    """Couples a ReLU + 2x2 max pooling (``MaxPool2d(relu=True)``, or ``Conv2d(relu=True, pool=True)``) with
    the convolution that takes its output, so that the pooling's backward can leave that convolution's
    input-gradient kernel: give the same link to both layers.

    Forward: the pooling layer leaves its index bytes with the link (``offer``); the convolution, called
    next with that very tensor, takes them (``take``) and keeps them for its backward.  Backward: the
    convolution computes its input gradient and, in the same kernel, the gradient in front of the pooling,
    returns the former to autograd as usual and leaves the latter with the link (``deposit``); the pooling
    layer's backward asks for it (``claim``) with the gradient autograd hands it, and gets it only if that
    gradient is the tensor the convolution returned -- otherwise (another consumer added its gradient, the
    shapes have no fused kernel, ...) it runs its own backward kernel on what it received.  Results are the
    same either way; nothing depends on the link being honoured."""

    def __init__(self):
        self._offer = None      # (pooled output, index bytes) of the forward in progress
        self._deposit = None    # (pooled gradient, full-resolution gradient) of the backward in progress

    def offer(self, pooled, idx):
        self._offer = (pooled, idx)

    def take(self, x):
        offer, self._offer = self._offer, None
        if offer is not None and offer[0].data_ptr() == x.data_ptr() and offer[0].shape == x.shape:
            return offer[1]
        return None

    def deposit(self, pooled_grad, full_grad):
        self._deposit = (pooled_grad, full_grad)

    def claim(self, dy, h, w):
        deposit, self._deposit = self._deposit, None
        if (deposit is not None and deposit[0].data_ptr() == dy.data_ptr() and deposit[0].shape == dy.shape
                and tuple(deposit[1].shape[2:]) == (h, w)):
            return deposit[1]
        return None


class _Conv3x3Fn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, relu, grad_premasked=False, input_rectified=False, pool=False,
                input_link=None, output_link=None):
        x = ops.to_nhwc(x)
        ctx.input_rectified = input_rectified
        ctx.relu = relu
        ctx.has_bias = bias is not None
        ctx.pool = pool
        # the index bytes of the pooling that produced x, if that layer shares a link with this one
        ctx.input_link = input_link
        ctx.unpool_idx = input_link.take(x) if input_link is not None else None
        ctx.output_link = output_link if (pool and relu) else None
        if pool:
            # convolution (+ReLU) and the 2x2 pooling behind it in one kernel: the backward rebuilds the
            # convolution's output gradient from the pooled gradient and the index bytes, already masked
            # by the ReLU, so the full-resolution output is neither written nor kept
            y, idx = ops.conv3x3_forward_pool(x, weight, bias, relu)
            ctx.save_for_backward(x, weight, idx)
            if ctx.output_link is not None:
                ctx.output_link.offer(y, idx)
            return y
        y = ops.conv3x3_forward(x, weight, bias, relu)
        # with grad_premasked the consumer's backward (a pooling layer with relu=True) has already
        # zeroed dy wherever y == 0, so the gradient kernels need not read y at all
        ctx.save_for_backward(x, weight, y if (relu and not grad_premasked) else None)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, y = ctx.saved_tensors
        dy = ops.to_nhwc(dy)
        if ctx.pool:
            full = ctx.output_link.claim(dy, x.shape[2], x.shape[3]) if ctx.output_link is not None else None
            dy = full if full is not None else ops.maxpool2x2_idx_backward(dy, y, x.shape[2], x.shape[3],
                                                                           relu_mask=ctx.relu)
            y = None
        # the ReLU backward (dy where y > 0) is applied by the gradient kernels while they
        # load dy, so no masked copy of dy is ever written
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            idx = ctx.unpool_idx
            if idx is not None and y is None and ops.conv3x3_input_grad_unpool_supported(dy, weight):
                # x is the output of a ReLU + pooling: the mask of its index bytes is the mask of
                # input_rectified, and the pooling's backward comes out of the same kernel
                dx, full = ops.conv3x3_input_grad_unpool(dy, weight, idx)
                ctx.input_link.deposit(dx, full)
            else:
                dx = ops.conv3x3_input_grad(dy, weight, relu_out=y, x_rectified=x if ctx.input_rectified else None)
        if ctx.needs_input_grad[1] or (ctx.has_bias and ctx.needs_input_grad[2]):
            dw, db = ops.conv3x3_weight_grad(x, dy, with_bias=ctx.has_bias, relu_out=y)
        return dx, dw, db, None, None, None, None, None, None


class Conv2d(torch.nn.Module):
    """``torch.nn.Conv2d(in, out, kernel_size=3, stride=1, padding=1)`` (the only
    convolution shape in the reference's VGG16 stages), optionally with the following
    ReLU fused into the epilogue.  The weight has torch's logical shape [out, in, 3, 3]
    and channels_last memory order; activations are kept in NHWC order.

    ``grad_premasked=True`` (only with ``relu=True``) declares that the layer's output goes only to a
    layer whose backward already drops the gradient where this output is zero -- ``MaxPool2d(relu=True)``,
    which is the identity on an already rectified input in the forward pass -- so the ReLU backward need
    not be applied (and the output not be read) again here.  ``input_rectified=True`` makes this layer
    such a consumer: it declares that the layer's input is the output of a ReLU (a preceding
    ``Conv2d(relu=True, grad_premasked=True)``) and zeroes the input gradient where the input is zero
    as it is stored.  Results are identical either way.

    ``pool=True`` appends ``MaxPool2d(2, 2)`` to the layer (after the ReLU, if any): the layer returns the
    pooled tensor, computed in the convolution kernel's epilogue where that kernel supports it, and the
    pooling module that follows in the reference's layer list is declared with
    ``MaxPool2d(..., applied_by_producer=True)``.

    ``input_link`` / ``output_link``: a ``PoolGradLink`` shared with the pooling layer that produces this
    layer's input, resp. (with ``relu=True, pool=True``) with the convolution that takes this layer's pooled
    output; the pooling's backward then comes out of the consuming convolution's input-gradient kernel."""

    def __init__(self, in_channels, out_channels, kernel_size=3, stride=1, padding=1, bias=True, relu=False,
                 grad_premasked=False, input_rectified=False, pool=False, input_link=None, output_link=None):
        super(Conv2d, self).__init__()
        norm = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
        if norm(kernel_size) != (3, 3) or norm(stride) != (1, 1) or norm(padding) != (1, 1):
            raise NotImplementedError("only Conv2d(kernel_size=3, stride=1, padding=1) has a HIP kernel")
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.relu = relu
        if grad_premasked and not relu:
            raise ValueError("grad_premasked only makes sense with relu=True")
        self.grad_premasked = grad_premasked
        self.input_rectified = input_rectified
        self.pool = pool
        self.input_link = input_link
        self.output_link = output_link
        w = torch.empty(out_channels, in_channels, 3, 3)
        torch.nn.init.kaiming_uniform_(w, a=math.sqrt(5))
        self.weight = torch.nn.Parameter(w.contiguous(memory_format=torch.channels_last))
        if bias:
            bound = 1 / math.sqrt(in_channels * 9)
            self.bias = torch.nn.Parameter(torch.empty(out_channels).uniform_(-bound, bound))
        else:
            self.bias = None

    def forward(self, x):
        return _Conv3x3Fn.apply(x, self.weight, self.bias, self.relu, self.grad_premasked, self.input_rectified,
                                self.pool, self.input_link, self.output_link)

    def extra_repr(self):
        return "{}, {}, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1), relu={}".format(
            self.in_channels, self.out_channels, self.relu)


# --------------------------------------------------------------------------------------
# ReLU / MaxPool
# --------------------------------------------------------------------------------------
class _ReLUFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        y = ops.relu(x)
        ctx.save_for_backward(y)
        return y

    @staticmethod
    def backward(ctx, dy):
        (y,) = ctx.saved_tensors
        return ops.relu_backward(dy, y)


class ReLU(torch.nn.Module):
    """``torch.nn.ReLU``.  ``inplace`` is accepted for signature compatibility; the result
    is always a new tensor (the stash keeps every in-flight activation anyway)."""

    def __init__(self, inplace=False):
        super(ReLU, self).__init__()
        self.inplace = inplace

    def forward(self, x):
        return _ReLUFn.apply(x)


class _MaxPool2x2Fn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, relu, link=None):
        x = ops.to_nhwc(x)
        y, idx = ops.maxpool2x2_idx(x, relu=relu)
        ctx.relu = relu
        ctx.hw = (x.shape[2], x.shape[3])
        ctx.link = link if relu else None
        ctx.save_for_backward(idx)      # one byte per output element; the input is not needed again
        if ctx.link is not None:
            ctx.link.offer(y, idx)
        return y

    @staticmethod
    def backward(ctx, dy):
        (idx,) = ctx.saved_tensors
        dy = ops.to_nhwc(dy)
        full = ctx.link.claim(dy, ctx.hw[0], ctx.hw[1]) if ctx.link is not None else None
        if full is None:
            full = ops.maxpool2x2_idx_backward(dy, idx, ctx.hw[0], ctx.hw[1], relu_mask=ctx.relu)
        return full, None, None


class MaxPool2d(torch.nn.Module):
    """``torch.nn.MaxPool2d(kernel_size=2, stride=2)`` on NHWC activations.  ``relu=True``: a ReLU in front
    of the pooling (stage1.py:10-11), fused.  ``applied_by_producer=True``: the convolution in front of
    this module was built with ``pool=True`` and has already pooled (and rectified) its output; the module
    keeps its place in the layer list and passes the tensor through.  ``link`` (with ``relu=True``): a
    ``PoolGradLink`` shared with the convolution that takes this layer's output."""

    def __init__(self, kernel_size=2, stride=2, padding=0, dilation=1, ceil_mode=False, relu=False,
                 applied_by_producer=False, link=None):
        super(MaxPool2d, self).__init__()
        self.relu = relu
        self.applied_by_producer = applied_by_producer
        self.link = link
        ks = kernel_size if isinstance(kernel_size, int) else kernel_size[0]
        st = ks if stride is None else (stride if isinstance(stride, int) else stride[0])
        if ks != 2 or st != 2 or padding not in (0, (0, 0)) or dilation not in (1, (1, 1)) or ceil_mode:
            raise NotImplementedError("only MaxPool2d(kernel_size=2, stride=2) has a HIP kernel")

    def forward(self, x):
        if self.applied_by_producer:
            return x
        return _MaxPool2x2Fn.apply(x, self.relu, self.link)


class _DropoutFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, mask, scale):
        ctx.scale = scale
        ctx.save_for_backward(mask)
        return ops.mask_scale(x, mask, scale)

    @staticmethod
    def backward(ctx, dy):
        (mask,) = ctx.saved_tensors
        if dy.stride() != mask.stride():
            dy = dy.contiguous()
        return ops.mask_scale(dy, mask, ctx.scale), None, None


class Dropout(torch.nn.Module):
    """``torch.nn.Dropout(p)``.  The keep-mask comes from ``mask_fn(x) -> uint8 tensor`` when
    one is set (parity runs inject host-generated masks so that both sides drop the same
    elements), otherwise from torch's device generator; applying it is a HIP kernel."""

    def __init__(self, p=0.5, inplace=False):
        super(Dropout, self).__init__()
        if p < 0 or p >= 1:
            raise ValueError("dropout probability has to be in [0, 1), got {}".format(p))
        self.p = p
        self.mask_fn = None

    def forward(self, x):
        if not self.training or self.p == 0:
            return x
        if self.mask_fn is not None:
            mask = self.mask_fn(x)
        else:
            mask = (torch.rand_like(x) >= self.p).to(torch.uint8)
        return _DropoutFn.apply(x, mask, 1.0 / (1.0 - self.p))


class Flatten(torch.nn.Module):
    """``out.view(out.size(0), -1)`` of the reference's stages (stage3.py:35-36): features
    in C,H,W order whatever the memory order of the incoming activation."""

    def forward(self, x):
        return x.contiguous().view(x.size(0), -1)


# --------------------------------------------------------------------------------------
# Embedding / LSTM / residual add
# --------------------------------------------------------------------------------------
class _EmbeddingFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ids, weight, padding_idx):
        ctx.padding_idx = padding_idx
        ctx.num_embeddings = weight.shape[0]
        ctx.save_for_backward(ids)
        return ops.embedding_forward(ids, weight)

    @staticmethod
    def backward(ctx, dout):
        (ids,) = ctx.saved_tensors
        return None, ops.embedding_backward(ids, dout, ctx.num_embeddings, ctx.padding_idx), None


class Embedding(torch.nn.Module):
    """``torch.nn.Embedding(num_embeddings, embedding_dim, padding_idx)`` with a dense
    weight gradient (torch's default)."""

    def __init__(self, num_embeddings, embedding_dim, padding_idx=None):
        super(Embedding, self).__init__()
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.padding_idx = padding_idx
        self.weight = torch.nn.Parameter(torch.empty(num_embeddings, embedding_dim))
        torch.nn.init.normal_(self.weight)
        if padding_idx is not None:
            with torch.no_grad():
                self.weight[padding_idx].fill_(0)

    def forward(self, ids):
        return _EmbeddingFn.apply(ids, self.weight, self.padding_idx)


class _LSTMFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w_ih, w_hh, b_ih, b_hh):
        y, (gates, c) = ops.lstm_forward(x, w_ih, w_hh, b_ih, b_hh)
        ctx.save_for_backward(x, y, gates, c, w_ih, w_hh)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, y, gates, c, w_ih, w_hh = ctx.saved_tensors
        dx, dw_ih, dw_hh, db = ops.lstm_backward(dy, x, y, gates, c, w_ih, w_hh, need_dx=ctx.needs_input_grad[0])
        return dx, dw_ih, dw_hh, db, db.clone()


class LSTM(torch.nn.Module):
    """Single-layer uni-directional ``torch.nn.LSTM(input_size, hidden_size)`` on
    sequence-first input ``[T, B, I]`` from zero initial state; returns ``(output, None)``
    so that ``lstm(x)[0]`` reads like the reference's stages (stage0.py:28-29).  Parameter
    names and layout are torch's (``weight_ih_l0`` ... ``bias_hh_l0``, gates i,f,g,o)."""

    def __init__(self, input_size, hidden_size, num_layers=1, bias=True, batch_first=False, dropout=0,
                 bidirectional=False):
        super(LSTM, self).__init__()
        if num_layers != 1 or not bias or batch_first or dropout or bidirectional:
            raise NotImplementedError("only LSTM(input_size, hidden_size) with torch's other defaults is built")
        self.input_size = input_size
        self.hidden_size = hidden_size
        k = 1.0 / math.sqrt(hidden_size)
        self.weight_ih_l0 = torch.nn.Parameter(torch.empty(4 * hidden_size, input_size).uniform_(-k, k))
        self.weight_hh_l0 = torch.nn.Parameter(torch.empty(4 * hidden_size, hidden_size).uniform_(-k, k))
        self.bias_ih_l0 = torch.nn.Parameter(torch.empty(4 * hidden_size).uniform_(-k, k))
        self.bias_hh_l0 = torch.nn.Parameter(torch.empty(4 * hidden_size).uniform_(-k, k))

    def forward(self, x):
        return _LSTMFn.apply(x, self.weight_ih_l0, self.weight_hh_l0, self.bias_ih_l0, self.bias_hh_l0), None


class _RevertVarlenFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, lengths):
        ctx.save_for_backward(lengths)
        return ops.revert_varlen(x.contiguous(), lengths)

    @staticmethod
    def backward(ctx, dy):
        (lengths,) = ctx.saved_tensors
        return ops.revert_varlen(dy.contiguous(), lengths), None


def _device_lengths(lengths, like, seq_len):
    """``lengths`` as B int64 values on ``like``'s device.  A host tensor is checked the way
    revert_varlen_tensor checks it (seq2seq/csrc/pack_utils_kernel.cu:17-36) -- all of it rather than the
    last entry only, and against the sequence length, beyond which the reference reads out of bounds --
    a device tensor is taken as it is (checking it would stall the stream)."""
    if lengths.dim() != 1:
        raise ValueError("'lengths' argument should be a 1D int64 tensor")
    if lengths.numel() != like.shape[1]:
        raise ValueError("Expected `len(lengths)` to be equal to batch_size, but got %d (batch_size=%d)"
                         % (lengths.numel(), like.shape[1]))
    if lengths.device.type == "cpu":
        if lengths.numel() and (int(lengths.min()) <= 0 or int(lengths.max()) > seq_len):
            raise ValueError("Length of all samples has to be greater than 0 and at most the sequence length, "
                             "but found an element in 'lengths' outside (0, %d]" % seq_len)
        lengths = lengths.to(torch.int64).to(like.device, non_blocking=True)
    return lengths.to(torch.int64).contiguous()


def revert_varlen(x, lengths):
    """``Revert_varlen.apply`` of seq2seq/models/encoder.py:13-23: reverses every sequence of ``x`` [T, B, ...]
    over its own length; its backward is the same operation on the gradient."""
    return _RevertVarlenFn.apply(x, _device_lengths(lengths, x, x.shape[0]))


class _BidirMergeFn(torch.autograd.Function):
    """[forward-direction output masked by length | backward-direction output reverted] side by side:
    ``torch.cat([out0 * mask, revert_varlen(out1, lengths)], dim=2)`` of encoder.py:51-57 without the
    intermediate tensors (both kernels write their half of the result in place)."""

    @staticmethod
    def forward(ctx, out0, out1, lengths):
        T, B, H = out0.shape
        y = torch.empty((T, B, 2 * H), dtype=out0.dtype, device=out0.device)
        ops.length_mask_apply(out0.contiguous(), lengths, out=y[:, :, :H])
        ops.revert_varlen(out1.contiguous(), lengths, out=y[:, :, H:])
        ctx.save_for_backward(lengths)
        ctx.hidden = H
        return y

    @staticmethod
    def backward(ctx, dy):
        (lengths,) = ctx.saved_tensors
        H = ctx.hidden
        dy = dy.contiguous()
        return (ops.length_mask_apply(dy[:, :, :H], lengths), ops.revert_varlen(dy[:, :, H:], lengths), None)


class _BidirParameters(torch.nn.Module):
    """The eight parameters of ``torch.nn.LSTM(input_size, hidden_size, bidirectional=True)`` under torch's
    names and initialisation (uniform(-1/sqrt(H), 1/sqrt(H)))."""

    def __init__(self, input_size, hidden_size):
        super(_BidirParameters, self).__init__()
        k = 1.0 / math.sqrt(hidden_size)
        for suffix in ("", "_reverse"):
            for name, shape in (("weight_ih_l0", (4 * hidden_size, input_size)),
                                ("weight_hh_l0", (4 * hidden_size, hidden_size)),
                                ("bias_ih_l0", (4 * hidden_size,)), ("bias_hh_l0", (4 * hidden_size,))):
                setattr(self, name + suffix, torch.nn.Parameter(torch.empty(*shape).uniform_(-k, k)))


class EmuBidirLSTM(torch.nn.Module):
    """``EmuBidirLSTM`` of seq2seq/models/encoder.py:25-64: a bidirectional LSTM layer on padded
    sequence-first input ``[T, B, I]`` with per-sample ``lengths``, built from two uni-directional layers;
    the backward direction runs on the time-reversed sequences and its output is reversed back.  Output
    ``[T, B, 2H]``, zeros behind every sequence's end.

    Parameters live in ``bidir`` under ``torch.nn.LSTM(bidirectional=True)``'s names and are shared with
    ``layer1`` (forward direction) and ``layer2`` (``*_reverse``), as in encoder.py:32-41, so the
    ``state_dict()`` keys are the reference's.  The reference switches to cuDNN's packed-sequence
    bidirectional LSTM for batches above 128 (encoder.py:60-64); this layer computes the same values with
    the two-layer form at every batch size."""

    def __init__(self, input_size, hidden_size, num_layers=1, bias=True, batch_first=False, bidirectional=True):
        super(EmuBidirLSTM, self).__init__()
        assert num_layers == 1, "emulation bidirectional lstm works for a single layer only"
        assert batch_first is False, "emulation bidirectional lstm works for batch_first = False only"
        assert bidirectional is True, "use for bidirectional lstm only"
        assert bias is True, "only the layer with bias is built"
        self.bidir = _BidirParameters(input_size, hidden_size)
        self.layer1 = LSTM(input_size, hidden_size)
        self.layer2 = LSTM(input_size, hidden_size)
        for name in ("weight_ih_l0", "weight_hh_l0", "bias_ih_l0", "bias_hh_l0"):
            setattr(self.layer1, name, getattr(self.bidir, name))
            setattr(self.layer2, name, getattr(self.bidir, name + "_reverse"))

    def forward(self, input, lengths):
        lengths = _device_lengths(lengths, input, input.shape[0])
        out1 = self.layer2(_RevertVarlenFn.apply(input, lengths))[0]
        out0 = self.layer1(input)[0]
        return _BidirMergeFn.apply(out0, out1, lengths)


class _AddFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b):
        return ops.add(a, b)

    @staticmethod
    def backward(ctx, dy):
        return dy, dy


def add(a, b):
    """Residual connection ``a + b`` on the HIP add kernel."""
    return _AddFn.apply(a, b)


# --------------------------------------------------------------------------------------
# bf16 pre-LN transformer layer (fp32 master parameters, bf16 compute)
# --------------------------------------------------------------------------------------
def _accumulate(p, fresh_fn, acc_fn):
    """Weight-gradient accumulation fused into the producing kernel: the first micro-batch
    of an update interval creates ``p.grad`` (fp32), later ones add into it in the GEMM /
    column-sum epilogue, so no separate accumulate pass runs."""
    if p.grad is None:
        p.grad = fresh_fn()
    else:
        acc_fn(p.grad)


class _TransformerLayerFn(torch.autograd.Function):
    """x -> x + Attn(LN1(x)) -> . + FFN(LN2(.)), hand-written backward; every matrix product is
    the bf16 MFMA GEMM, every reduction / pointwise op one of the bf16 HIP kernels."""

    @staticmethod
    def forward(ctx, x, heads, eps, ln1_w, ln1_b, qkv_w, qkv_b, o_w, o_b, ln2_w, ln2_b, fc1_w, fc1_b, fc2_w, fc2_b):
        B, S, H = x.shape
        x2d = x.contiguous().view(B * S, H)
        bw = ops.bf16_weight
        h1, mean1, rstd1 = ops.layernorm_forward(x2d, ln1_w, ln1_b, eps)
        qkv = ops.gemm_bf16(h1, bw(qkv_w), trans_b=True, bias=qkv_b)
        att, att_aux = ops.attention_forward(qkv, B, S, heads)
        x2 = ops.gemm_bf16(att, bw(o_w), trans_b=True, bias=o_b, residual=x2d)
        h2, mean2, rstd2 = ops.layernorm_forward(x2, ln2_w, ln2_b, eps)
        f, g = ops.gemm_bf16_gelu(h2, bw(fc1_w), trans_b=True, bias=fc1_b)      # g = gelu(f) in the epilogue
        y = ops.gemm_bf16(g, bw(fc2_w), trans_b=True, bias=fc2_b, residual=x2)
        ctx.dims = (B, S, H, heads)
        ctx.params = (ln1_w, ln1_b, qkv_w, qkv_b, o_w, o_b, ln2_w, ln2_b, fc1_w, fc1_b, fc2_w, fc2_b)
        ctx.save_for_backward(x2d, h1, mean1, rstd1, qkv, att_aux, att, x2, h2, mean2, rstd2, f, g)
        return y.view(B, S, H)

    @staticmethod
    def backward(ctx, dy):
        B, S, H, heads = ctx.dims
        x2d, h1, mean1, rstd1, qkv, att_aux, att, x2, h2, mean2, rstd2, f, g = ctx.saved_tensors
        ln1_w, ln1_b, qkv_w, qkv_b, o_w, o_b, ln2_w, ln2_b, fc1_w, fc1_b, fc2_w, fc2_b = ctx.params
        bw = ops.bf16_weight
        dy2 = dy.contiguous().view(B * S, H)
        sums = ops.ColsumBatch()

        def linear_backward(d_out, inp, w, b, through_gelu_of=None):
            # parameters are read (and their bf16 image taken) at backward time: the version
            # load_old_params made current
            _accumulate(w, lambda: ops.gemm_bf16_wgrad(d_out, inp), lambda acc: ops.gemm_bf16_wgrad(d_out, inp, acc))
            # (the bias gradient, a column sum of d_out, waits for the end of the layer: all column sums of
            # the layer's backward then take two launches)
            if b.grad is None:
                b.grad = torch.empty(b.shape, dtype=torch.float32, device=d_out.device)
                sums.add(d_out, b.grad, 0.0)
            else:
                sums.add(d_out, b.grad, 1.0)
            if through_gelu_of is not None:       # the input is gelu(f): return the gradient with respect to f
                return ops.gemm_bf16_gelu_backward(d_out, bw(w), through_gelu_of)
            return ops.gemm_bf16(d_out, bw(w))

        def layernorm_backward(d_out, inp, w, b, mean, rstd, residual):
            # (+ residual: the branch of the gradient that bypasses the normalisation, added as dx is stored)
            if w.grad is None:
                dx, dg, db = ops.layernorm_backward(d_out, inp, w, mean, rstd, batch=sums, residual=residual)
                w.grad, b.grad = dg, db
            else:
                dx, _, _ = ops.layernorm_backward(d_out, inp, w, mean, rstd, w.grad, b.grad, batch=sums,
                                                  residual=residual)
            return dx

        # y = fc2(gelu(fc1(LN2(x2)))) + x2
        df = linear_backward(dy2, g, fc2_w, fc2_b, through_gelu_of=f)
        dh2 = linear_backward(df, h2, fc1_w, fc1_b)
        dx2 = layernorm_backward(dh2, x2, ln2_w, ln2_b, mean2, rstd2, dy2)
        # x2 = o(attn(qkv(LN1(x)))) + x
        datt = linear_backward(dx2, att, o_w, o_b)
        dqkv = ops.attention_backward(datt, qkv, att_aux, B, S, heads, ctx=att)
        dh1 = linear_backward(dqkv, h1, qkv_w, qkv_b)
        dx = layernorm_backward(dh1, x2d, ln1_w, ln1_b, mean1, rstd1, dx2)
        sums.run()
        return (dx.view(B, S, H), None, None) + (None,) * 12


class TransformerLayer(torch.nn.Module):
    """Pre-LayerNorm transformer layer: multi-head self-attention (no mask) and a GELU
    feed-forward block, each with a residual connection.  Parameters are fp32 masters
    (``ln1``, ``qkv``, ``proj``, ``ln2``, ``fc1``, ``fc2`` with torch's ``weight``/``bias``
    names); activations are bf16 ``[batch, seq, hidden]``.  Weight gradients are produced in
    fp32 and accumulated across micro-batches inside the producing kernels, so autograd
    sees only the activation path."""

    def __init__(self, hidden, heads, ffn, eps=1e-5):
        super(TransformerLayer, self).__init__()
        self.hidden, self.heads, self.ffn, self.eps = hidden, heads, ffn, eps
        self.ln1 = torch.nn.LayerNorm(hidden, eps=eps)
        self.qkv = torch.nn.Linear(hidden, 3 * hidden)
        self.proj = torch.nn.Linear(hidden, hidden)
        self.ln2 = torch.nn.LayerNorm(hidden, eps=eps)
        self.fc1 = torch.nn.Linear(hidden, ffn)
        self.fc2 = torch.nn.Linear(ffn, hidden)

    def forward(self, x):
        # the torch.nn members are parameter containers only; their forward is never called
        return _TransformerLayerFn.apply(
            x, self.heads, self.eps, self.ln1.weight, self.ln1.bias, self.qkv.weight, self.qkv.bias,
            self.proj.weight, self.proj.bias, self.ln2.weight, self.ln2.bias, self.fc1.weight, self.fc1.bias,
            self.fc2.weight, self.fc2.bias)


class _CastFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, to_bf16):
        ctx.to_bf16 = to_bf16
        return ops.cast_bf16(x) if to_bf16 else ops.cast_f32(x)

    @staticmethod
    def backward(ctx, dy):
        return (ops.cast_f32(dy) if ctx.to_bf16 else ops.cast_bf16(dy)), None


class _GeluFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        ctx.save_for_backward(x)
        return ops.gelu(x)

    @staticmethod
    def backward(ctx, dy):
        (x,) = ctx.saved_tensors
        return ops.gelu_backward(x, dy.contiguous())


class GELU(torch.nn.Module):
    """``torch.nn.GELU()`` (erf form) on bfloat16 activations."""

    def forward(self, x):
        if x.dtype != torch.bfloat16:
            raise NotImplementedError("GELU: only bfloat16 activations have a kernel")
        return _GeluFn.apply(x.contiguous())


def to_bf16(x):
    return x if x.dtype == torch.bfloat16 else _CastFn.apply(x, True)


def to_f32(x):
    return x if x.dtype == torch.float32 else _CastFn.apply(x, False)


# --------------------------------------------------------------------------------------
# Criterion
# --------------------------------------------------------------------------------------
class _CrossEntropyFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, target, ignore_index):
        x2 = logits.reshape(-1, logits.shape[-1])
        if x2.stride(-1) != 1:
            x2 = x2.contiguous()
        t = target.reshape(-1).contiguous()
        loss, (lse, count) = ops.cross_entropy_forward(x2, t, ignore_index)
        ctx.ignore_index = ignore_index
        ctx.shape = logits.shape
        ctx.save_for_backward(x2, t, lse, count)
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        x2, t, lse, count = ctx.saved_tensors
        d = ops.cross_entropy_backward(x2, t, lse, count, grad_loss.contiguous(), ctx.ignore_index)
        return d.view(ctx.shape), None, None


class _LabelSmoothingFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, target, padding_idx, smoothing, divisor):
        x2 = logits.reshape(-1, logits.shape[-1])
        if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) < x2.shape[1]):
            x2 = x2.contiguous()
        t = target.reshape(-1).contiguous()
        loss, lse = ops.label_smoothing_forward(x2, t, padding_idx, smoothing, divisor)
        ctx.args = (padding_idx, smoothing, divisor)
        ctx.shape = logits.shape
        ctx.save_for_backward(x2, t, lse)
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        x2, t, lse = ctx.saved_tensors
        d = ops.label_smoothing_backward(x2, t, lse, grad_loss.contiguous(), *ctx.args)
        return d.view(ctx.shape), None, None, None, None


class LabelSmoothing(torch.nn.Module):
    """NLL loss with label smoothing, the criterion of the translation stages
    (seq2seq/train/smoothing.py:7-34, created at seq2seq/utils.py:31): ``output`` is [T, B, V] logits,
    ``target`` the T*B token ids; rows whose target is ``padding_idx`` are dropped, the sum over the other
    rows of ``(1-smoothing) * nll + smoothing * mean(-log_softmax)`` is divided by the batch size B."""

    def __init__(self, padding_idx, smoothing=0.0):
        super(LabelSmoothing, self).__init__()
        self.padding_idx = padding_idx
        self.confidence = 1.0 - smoothing
        self.smoothing = smoothing

    def forward(self, output, target):
        if output.dim() < 2:
            raise ValueError("LabelSmoothing: output must be [T, B, V], got %s" % (tuple(output.shape),))
        return _LabelSmoothingFn.apply(output, target, self.padding_idx, self.smoothing, float(output.size(1)))


class CrossEntropyLoss(torch.nn.Module):
    """``torch.nn.CrossEntropyLoss()`` with mean reduction -- the criterion
    runtime/image_classification/main_with_runtime.py:126 creates."""

    def __init__(self, ignore_index=-100):
        super(CrossEntropyLoss, self).__init__()
        self.ignore_index = ignore_index

    def forward(self, logits, target):
        # (bfloat16 logits of a 16-bit stage are widened first: the loss is evaluated in fp32)
        return _CrossEntropyFn.apply(to_f32(logits), target, self.ignore_index)
