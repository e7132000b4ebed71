"""Tensor-level wrappers of the compute entry points of the C ABI.

Each function checks shapes, dtypes, devices and memory order on the host (a kernel is
never launched on operands it was not written for), allocates the output with torch
(device memory and streams are the only things torch provides here) and launches on
torch's current stream.
"""
import ctypes

import torch

from . import _cabi

_vp = ctypes.c_void_p


def _ptr(t):
    return _vp(t.data_ptr()) if t is not None else None


def _check(t, name, dtype=torch.float32):
    _cabi.require_device(t, name)
    if t.dtype != dtype:
        raise TypeError("%s must be %s, got %s" % (name, dtype, t.dtype))
    return t


def _rowmajor2d(t, name):
    _check(t, name)
    if t.dim() != 2 or t.stride(1) != 1 or (t.size(0) > 1 and t.stride(0) < t.size(1)):
        raise ValueError("%s must be a row-major 2-D matrix, got shape %s stride %s"
                         % (name, tuple(t.shape), t.stride()))
    return t


def gemm(a, b, trans_a=False, trans_b=False, bias=None, relu=False, out=None, beta=0.0):
    """out[M,N] = op(a) @ op(b) (+ bias) (+ beta*out) (ReLU); fp32 MFMA kernel."""
    _rowmajor2d(a, "a")
    _rowmajor2d(b, "b")
    M, K = (a.size(1), a.size(0)) if trans_a else (a.size(0), a.size(1))
    Kb, N = (b.size(1), b.size(0)) if trans_b else (b.size(0), b.size(1))
    if K != Kb:
        raise ValueError("gemm: inner dimensions differ (%d vs %d)" % (K, Kb))
    if out is None:
        if beta != 0.0:
            raise ValueError("gemm: beta needs an existing out")
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    else:
        _rowmajor2d(out, "out")
        if tuple(out.shape) != (M, N):
            raise ValueError("gemm: out has shape %s, expected %s" % (tuple(out.shape), (M, N)))
    if bias is not None:
        _check(bias, "bias")
        if bias.numel() != N or not bias.is_contiguous():
            raise ValueError("gemm: bias must be a contiguous vector of N=%d" % N)
    lda = a.stride(0) if a.size(0) > 1 else a.size(1)
    ldb = b.stride(0) if b.size(0) > 1 else b.size(1)
    ldc = out.stride(0) if out.size(0) > 1 else out.size(1)
    _cabi.lib().pd_gemm_f32(int(trans_a), int(trans_b), M, N, K, _ptr(a), lda, _ptr(b), ldb, float(beta),
                            _ptr(out), ldc, _ptr(bias), int(relu), _cabi.stream_ptr())
    return out


def colsum(x, out=None, beta=0.0):
    """Column sums of a row-major matrix (two deterministic passes for tall inputs)."""
    _rowmajor2d(x, "x")
    M, N = x.shape
    ld = x.stride(0) if M > 1 else N
    lib = _cabi.lib()
    if out is None:
        out = torch.empty(N, dtype=torch.float32, device=x.device)
    else:
        _check(out, "out")
        if out.numel() != N or not out.is_contiguous():
            raise ValueError("colsum: out must be a contiguous vector of N=%d" % N)
    splits = min(512, max(1, M // 1024))
    if splits == 1:
        lib.pd_colsum_f32(_ptr(x), _ptr(out), M, N, ld, 1, float(beta), _cabi.stream_ptr())
    else:
        part = torch.empty((splits, N), dtype=torch.float32, device=x.device)
        lib.pd_colsum_f32(_ptr(x), _ptr(part), M, N, ld, splits, 0.0, _cabi.stream_ptr())
        lib.pd_colsum_f32(_ptr(part), _ptr(out), splits, N, N, 1, float(beta), _cabi.stream_ptr())
    return out


def _dense_same_order(a, b):
    return a.shape == b.shape and a.stride() == b.stride()


def _is_dense(t):
    return t.is_contiguous() or (t.dim() == 4 and t.is_contiguous(memory_format=torch.channels_last))


def relu(x):
    _check(x, "x")
    if not _is_dense(x):
        x = x.contiguous()
    y = torch.empty_like(x)
    _cabi.lib().pd_relu_fwd_f32(_ptr(x), _ptr(y), x.numel(), _cabi.stream_ptr())
    return y


def relu_backward(dy, y):
    """dx = dy * (y > 0); dy is brought into y's memory order if needed."""
    _check(dy, "dy")
    _check(y, "y")
    if not _dense_same_order(dy, y):
        d2 = torch.empty_like(y)
        d2.copy_(dy)
        dy = d2
    dx = torch.empty_like(y)
    _cabi.lib().pd_relu_bwd_f32(_ptr(dy), _ptr(y), _ptr(dx), y.numel(), _cabi.stream_ptr())
    return dx


def to_nhwc(x):
    """A logically-NCHW 4-D tensor whose memory order is N,H,W,C."""
    if x.dim() != 4:
        raise ValueError("expected a 4-D NCHW tensor, got %d-D" % x.dim())
    return x.contiguous(memory_format=torch.channels_last)


def _nhwc_dims(x):
    n, c, h, w = x.shape
    if not x.is_contiguous(memory_format=torch.channels_last):
        raise ValueError("tensor is not in NHWC memory order")
    return n, h, w, c


def maxpool2x2(x):
    _check(x, "x")
    x = to_nhwc(x)
    n, h, w, c = _nhwc_dims(x)
    y = torch.empty((n, c, h // 2, w // 2), dtype=torch.float32, device=x.device,
                    memory_format=torch.channels_last)
    _cabi.lib().pd_maxpool2x2_fwd_nhwc_f32(_ptr(x), _ptr(y), n, h, w, c, _cabi.stream_ptr())
    return y


def maxpool2x2_backward(x, dy, relu_mask=False):
    _check(x, "x")
    _check(dy, "dy")
    n, h, w, c = _nhwc_dims(x)
    dy = to_nhwc(dy)
    if tuple(dy.shape) != (n, c, h // 2, w // 2):
        raise ValueError("maxpool2x2_backward: dy has shape %s" % (tuple(dy.shape),))
    dx = torch.empty_like(x)
    _cabi.lib().pd_maxpool2x2_bwd_nhwc_f32(_ptr(x), _ptr(dy), _ptr(dx), n, h, w, c, int(relu_mask),
                                           _cabi.stream_ptr())
    return dx


def cross_entropy_forward(logits, target, ignore_index=-100):
    """Mean softmax cross-entropy.  Returns (loss[()], (lse, count)) for the backward."""
    _rowmajor2d(logits, "logits")
    _check(target, "target", torch.int64)
    B, C = logits.shape
    if target.numel() != B or not target.is_contiguous():
        raise ValueError("cross_entropy: target must be a contiguous vector of B=%d" % B)
    dev = logits.device
    loss = torch.empty((), dtype=torch.float32, device=dev)
    row_loss = torch.empty(B, dtype=torch.float32, device=dev)
    lse = torch.empty(B, dtype=torch.float32, device=dev)
    count = torch.empty(1, dtype=torch.float32, device=dev)
    ld = logits.stride(0) if B > 1 else C
    _cabi.lib().pd_xent_fwd_f32(_ptr(logits), _ptr(target), _ptr(loss), _ptr(row_loss), _ptr(lse), _ptr(count),
                                B, C, ld, int(ignore_index), _cabi.stream_ptr())
    return loss, (lse, count)


def cross_entropy_backward(logits, target, lse, count, grad_loss, ignore_index=-100):
    B, C = logits.shape
    _check(grad_loss, "grad_loss")
    grad_loss = grad_loss.reshape(1).contiguous()
    d = torch.empty((B, C), dtype=torch.float32, device=logits.device)
    ld = logits.stride(0) if B > 1 else C
    _cabi.lib().pd_xent_bwd_f32(_ptr(logits), _ptr(target), _ptr(lse), _ptr(grad_loss), _ptr(count), _ptr(d),
                                B, C, ld, C, int(ignore_index), _cabi.stream_ptr())
    return d
