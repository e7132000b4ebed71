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

# Optional per-launch timing: when `kernel_timer` is a dict, every timed launch appends a
# (start, end, work) triple of HIP events recorded on the launch stream under the kernel's
# name; `work` is the algorithmic flop (or byte) count of that launch.
kernel_timer = None


class _timed(object):
    __slots__ = ("name", "work", "start")

    def __init__(self, name, work):
        self.name = name
        self.work = work

    def __enter__(self):
        if kernel_timer is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record()

    def __exit__(self, *exc):
        if kernel_timer is not None:
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            kernel_timer.setdefault(self.name, []).append((self.start, end, self.work))
        return False


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
    if _use_split_bf16(M, N, K, trans_a, trans_b, relu, a, b, out):
        return _gemm_split_bf16(a, b, trans_a, trans_b, M, N, K, bias, out, beta)
    splits = splitk_factor(M, N, K, trans_a)
    plan = _row_plan(M, N, K) if splits == 1 and _ROW_PLAN else None
    if plan is not None and N % 4 == 0 and ldc % 4 == 0 and out.data_ptr() % 16 == 0:
        # whole rounds of 768 blocks on the upper rows, then the few tile rows left over as a k-split of their own
        rows, top_splits, tail_splits = plan
        lib = _cabi.lib()
        with _timed("gemm_f32", 2.0 * M * N * K):
            for r0, r1, sp in ((0, rows, top_splits), (rows, M, tail_splits)):
                a_part = a[:, r0:r1] if trans_a else a[r0:r1]
                if sp == 1:
                    lib.pd_gemm_f32(int(trans_a), int(trans_b), r1 - r0, N, K, _ptr(a_part), lda, _ptr(b), ldb,
                                    float(beta), _ptr(out[r0:]), ldc, _ptr(bias), int(relu), _cabi.stream_ptr())
                    continue
                part = torch.empty((sp, r1 - r0, N), dtype=torch.float32, device=a.device)
                lib.pd_gemm_splitk_f32(int(trans_a), int(trans_b), r1 - r0, N, K, _ptr(a_part), lda, _ptr(b), ldb,
                                       _ptr(part), sp, _cabi.stream_ptr())
                lib.pd_splitk_reduce_f32(_ptr(part), sp, r1 - r0, N, _ptr(bias), int(relu), float(beta),
                                         _ptr(out[r0:]), ldc, _cabi.stream_ptr())
        return out
    # M <= 128: the streaming kernel behind pd_gemm_splitk_f32 also wins without a split (one partial)
    skinny = not trans_a and M <= 128 and K % 16 == 0 and K >= 256 and N >= 128
    if (splits > 1 or skinny) and N % 4 == 0 and ldc % 4 == 0 and out.data_ptr() % 16 == 0:
        # too few output tiles for 256 CUs: split k over more blocks, then one fused reduce + epilogue
        part = torch.empty((splits, M, N), dtype=torch.float32, device=a.device)
        with _timed("gemm_f32_splitk", 2.0 * M * N * K):
            _cabi.lib().pd_gemm_splitk_f32(int(trans_a), int(trans_b), M, N, K, _ptr(a), lda, _ptr(b), ldb, _ptr(part),
                                           splits, _cabi.stream_ptr())
        _cabi.lib().pd_splitk_reduce_f32(_ptr(part), splits, M, N, _ptr(bias), int(relu), float(beta), _ptr(out), ldc,
                                         _cabi.stream_ptr())
        return out
    with _timed("gemm_f32", 2.0 * M * N * K):
        _cabi.lib().pd_gemm_f32(int(trans_a), int(trans_b), M, N, K, _ptr(a), lda, _ptr(b), ldb, float(beta),
                                _ptr(out), ldc, _ptr(bias), int(relu), _cabi.stream_ptr())
    return out


# Large fp32 products on the bf16 matrix pipes: "auto" (products of at least SPLIT_BF16_MIN_WORK multiply-adds
# whose shape the bf16 kernel takes), "never" (always the fp32 MFMA kernels), "always" (whenever the shape allows).
_GEMM_F32_ALGO = "auto"
SPLIT_BF16_MIN_WORK = 1 << 32


def set_gemm_f32_algorithm(mode):
    """How ``gemm`` computes large fp32 products.  "mfma_f32": the fp32 MFMA kernels.  "split_bf16": each operand
    as the exact sum of three bf16 terms, six bf16 MFMA products per term pair, fp32 accumulation
    (pd_split3_bf16_f32 + pd_gemm_bf16 over a six-fold reduction) -- 1.5 to 1.7 times as fast on the LSTM
    projections and the classifier, and closer to the fp64 product than the fp32 MFMA kernel (fewer roundings of the
    running sum).  "auto" (default): split_bf16 for products of at least 2^32 multiply-adds, else mfma_f32."""
    global _GEMM_F32_ALGO
    _GEMM_F32_ALGO = {"auto": "auto", "mfma_f32": "never", "split_bf16": "always"}[mode]


def _split_bf16_parts(M, N, K):
    """Number of ranges the six-fold reduction is cut into (partial products, one batch entry each, added by
    pd_splitk_reduce_f32) so that the bf16 kernel's 256 x 256 tiles fill the chip: 1 for at least 192 tiles, else
    256 // tiles if the ranges stay multiples of 128; 0 if the product should not take this path at all."""
    tiles = -(-M // 256) * -(-N // 256)
    if tiles >= 192:
        return 1
    parts = min(256 // tiles, 6)
    while parts > 1 and (6 * K) % (parts * 128) != 0:
        parts -= 1
    return parts if parts > 1 else 0


def _use_split_bf16(M, N, K, trans_a, trans_b, relu, a, b, out):
    if _GEMM_F32_ALGO == "never" or relu or (trans_a and trans_b):
        return False
    parts = _split_bf16_parts(M, N, K)
    # (auto: wide outputs from 2^32 multiply-adds on.  Narrow ones, whose reduction has to be cut into partial
    # products, gain 15-25 % alone -- 6400 x 1024 x 4096: 437 against 506 us -- and next to nothing inside the LSTM
    # stage, where the operand split's 0.4 GB of traffic per product competes with the other stream: left to
    # "split_bf16")
    if _GEMM_F32_ALGO == "auto" and (parts != 1 or M * N * K < SPLIT_BF16_MIN_WORK):
        return False
    # the bf16 kernel's direct-to-LDS path: reduction (6 K) a multiple of 128, rows of 8 elements, 16-byte alignment
    ok = parts > 0 and K % 64 == 0 and M % 8 == 0 and N % 8 == 0 and M >= 256 and N >= 256
    ok = ok and all(t.stride(0) % 4 == 0 and t.data_ptr() % 16 == 0 for t in (a, b, out)) and out.stride(0) % 8 == 0
    return ok and 6 * K * max(M, N) < (1 << 31)


def _gemm_split_bf16(a, b, trans_a, trans_b, M, N, K, bias, out, beta):
    """out = op(a) op(b) (+ bias) (+ beta out) through six bf16 products (see set_gemm_f32_algorithm)."""
    lib, dev = _cabi.lib(), a.device
    parts = _split_bf16_parts(M, N, K)
    # an operand whose rows are the reduction index (a transposed A, a plain B) gets its six slots stacked
    a6 = torch.empty((6 * K, M) if trans_a else (M, 6 * K), dtype=BF16, device=dev)
    b6 = torch.empty((N, 6 * K) if trans_b else (6 * K, N), dtype=BF16, device=dev)
    with _timed("gemm_f32_as_bf16x6", 2.0 * M * N * K):
        lib.pd_split3_bf16_f32(_ptr(a), a.size(0), a.size(1), a.stride(0), _ptr(a6), 0, int(trans_a), _cabi.stream_ptr())
        lib.pd_split3_bf16_f32(_ptr(b), b.size(0), b.size(1), b.stride(0), _ptr(b6), 1, int(not trans_b),
                               _cabi.stream_ptr())
        if parts == 1:
            lib.pd_gemm_bf16(int(trans_a), int(trans_b), M, N, 6 * K, _ptr(a6), a6.stride(0), _ptr(b6), b6.stride(0),
                             _ptr(out), out.stride(0), 1, 1.0, float(beta), _ptr(bias), None, 0, 1, 1, None,
                             _cabi.stream_ptr())
            return out
        # few output tiles: ranges of the six-fold reduction as batch entries, partial products added in index order
        kk = 6 * K // parts
        part = torch.empty((parts, M, N), dtype=torch.float32, device=dev)
        strides = (ctypes.c_int64 * 6)(kk * a6.stride(0) if trans_a else kk, 0, kk if trans_b else kk * b6.stride(0), 0,
                                       M * N, 0)
        lib.pd_gemm_bf16(int(trans_a), int(trans_b), M, N, kk, _ptr(a6), a6.stride(0), _ptr(b6), b6.stride(0),
                         _ptr(part), N, 1, 1.0, 0.0, None, None, 0, parts, 1, strides, _cabi.stream_ptr())
        lib.pd_splitk_reduce_f32(_ptr(part), parts, M, N, _ptr(bias), 0, float(beta), _ptr(out), out.stride(0),
                                 _cabi.stream_ptr())
    return out


SPLITK_TARGET_BLOCKS = 256     # one block per CU
SPLITK_MIN_K = 128             # k per split is never smaller than this
SPLITK_FULL_HOUSE = 768        # blocks of the 128 x 128 kernel the GPU holds at once (three per CU)
SPLITK_DEEP_K = 1024           # ... worth filling by a split only if every part still reduces over this much


def splitk_factor(M, N, K, trans_a=False):
    """Number of k ranges a product is split into so that about one block per CU runs (1 = no split).
    Mirrors the tile choice of pd_gemm_splitk_f32: its streaming kernel for M <= 128 (A not transposed,
    K a multiple of 16) owns up to 64 rows x 128 columns per block; otherwise tiles are 128 x 128 when M > 64
    and N >= 128, else 64 x 64."""
    t_general = 0
    if not trans_a and M <= 128 and K % 16 == 0:
        tiles = -(-N // 128) * -(-M // 64)
    else:
        t = t_general = 128 if (M > 64 and N >= 128) else 64
        tiles = -(-M // t) * -(-N // t)
    if tiles * 2 > SPLITK_TARGET_BLOCKS or K < 2 * SPLITK_MIN_K:
        # between one block per CU and a full house (the 128 x 128 kernel runs three blocks per CU): a deep
        # reduction is split two or three ways so that every CU holds three blocks instead of one or two
        # (4096 x 1024 x 6400, the LSTM weight gradients: 256 tiles -> 768 blocks)
        if t_general == 128 and tiles <= SPLITK_FULL_HOUSE // 2:
            splits = SPLITK_FULL_HOUSE // tiles
            if K // splits >= SPLITK_DEEP_K:
                return splits
        return 1
    return max(1, min(SPLITK_TARGET_BLOCKS // tiles, K // SPLITK_MIN_K, 64))


_ROW_PLAN = True


def _house_time(blocks, k):
    """Time, in steps of k of a full round, that ``blocks`` blocks of the 128 x 128 kernel take to reduce over ``k``
    each: whole rounds of SPLITK_FULL_HOUSE blocks, plus a last round that costs 0.45 + 0.55 x its fill (blocks
    with fewer neighbours on their CU run faster, but not in proportion: measured 0.75 for 400 of 768)."""
    whole, rem = divmod(blocks, SPLITK_FULL_HOUSE)
    return k * (whole + (0.45 + 0.55 * rem / SPLITK_FULL_HOUSE if rem else 0.0))


def _reduce_time(rows, n, splits):
    """pd_splitk_reduce_f32 in the same unit (one step of k of a full round is about 0.18 us): a launch and
    (splits + 1) x rows x n x 4 bytes at about 4 TB/s."""
    return 30 + rows * n * 4 * (splits + 1) / 4e6 / 0.18


def _row_plan(M, N, K):
    """(rows, top_splits, tail_splits) or None.  A product of more than half a full house of 128 x 128 tiles can
    leave a last round nearly empty (64 of 1600 tiles for 6400 x 4096, 400 tiles on 768 places for 6400 x 1024):
    that round lasts almost as long as a full one.  The plan gives the first ``rows`` rows whole rounds -- as they
    are, or split two or three ways over a reduction that is deep enough -- and runs the tile rows left over as a
    k-split of their own that fills one more round.  Chosen by the cost model above; None where the plain launch
    is within 7 % of the best plan."""
    tm, tn = -(-M // 128), -(-N // 128)
    tiles = tm * tn
    if tiles <= SPLITK_FULL_HOUSE // 2:
        return None
    best, best_cost = None, 0.93 * _house_time(tiles, K)
    for top_splits in (1, 2, 3):
        if top_splits > 1 and K // top_splits < SPLITK_DEEP_K:
            break
        per_row = tn * top_splits
        rounds = (tm * per_row) // SPLITK_FULL_HOUSE
        top = min(tm - 1, (rounds * SPLITK_FULL_HOUSE) // per_row)
        if rounds < 1 or top < 1:
            continue
        tail_tiles = (tm - top) * tn
        tail_splits = max(1, min(SPLITK_FULL_HOUSE // tail_tiles, K // SPLITK_MIN_K))
        k_top = -(-K // top_splits)
        cost = _house_time(top * per_row, k_top) + _house_time(tail_tiles * tail_splits, -(-K // tail_splits)) + 30
        if top_splits > 1:
            cost += _reduce_time(top * 128, N, top_splits)
        if tail_splits > 1:
            cost += _reduce_time(M - top * 128, N, tail_splits)
        if cost < best_cost:
            best, best_cost = (top * 128, top_splits, tail_splits), cost
    return best


def gemm_splitk(a, b, trans_a, trans_b, partials):
    """partials[s] = op(a)[:, k range s] @ op(b)[k range s, :] for s < partials.size(0); the consumer sums them."""
    _rowmajor2d(a, "a")
    _rowmajor2d(b, "b")
    M, K = (a.size(1), a.size(0)) if trans_a else (a.size(0), a.size(1))
    Kb, N = (b.size(1), b.size(0)) if trans_b else (b.size(0), b.size(1))
    if K != Kb or partials.dim() != 3 or tuple(partials.shape[1:]) != (M, N) or not partials.is_contiguous():
        raise ValueError("gemm_splitk: shapes %s x %s -> %s do not fit" % (tuple(a.shape), tuple(b.shape),
                                                                            tuple(partials.shape)))
    _check(partials, "partials")
    lda = a.stride(0) if a.size(0) > 1 else a.size(1)
    ldb = b.stride(0) if b.size(0) > 1 else b.size(1)
    with _timed("gemm_f32_splitk", 2.0 * M * N * K):
        _cabi.lib().pd_gemm_splitk_f32(int(trans_a), int(trans_b), M, N, K, _ptr(a), lda, _ptr(b), ldb, _ptr(partials),
                                       partials.size(0), _cabi.stream_ptr())
    return partials


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


def mask_scale(x, mask, scale):
    """y = x * mask * scale with a uint8 0/1 mask of x's shape and memory order."""
    _check(x, "x")
    _check(mask, "mask", torch.uint8)
    if not _is_dense(x):
        x = x.contiguous()
    if not _dense_same_order(mask, x):
        raise ValueError("mask_scale: mask must have the shape and memory order of x")
    y = torch.empty_like(x)
    _cabi.lib().pd_mask_scale_f32(_ptr(x), _ptr(mask), _ptr(y), x.numel(), float(scale), _cabi.stream_ptr())
    return y


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


def maxpool2x2(x, relu=False):
    """2x2/stride-2 max pooling; ``relu=True`` pools a (virtual) ReLU of ``x``."""
    _check(x, "x")
    x = to_nhwc(x)
    n, h, w, c = _nhwc_dims(x)
    y = torch.empty((n, c, h // 2, w // 2), dtype=torch.float32, device=x.device,
                    memory_format=torch.channels_last)
    _cabi.lib().pd_maxpool2x2_fwd_nhwc_f32(_ptr(x), _ptr(y), n, h, w, c, int(relu), _cabi.stream_ptr())
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


def maxpool2x2_idx(x, relu=False):
    """2x2/stride-2 max pooling that also returns one index byte per output element (bits 0-1: position of
    the first maximum in its window, row-major; bit 2: the maximum is positive) -- all the backward needs."""
    _check(x, "x")
    x = to_nhwc(x)
    n, h, w, c = _nhwc_dims(x)
    y = torch.empty((n, c, h // 2, w // 2), dtype=torch.float32, device=x.device,
                    memory_format=torch.channels_last)
    idx = torch.empty((n, c, h // 2, w // 2), dtype=torch.uint8, device=x.device,
                      memory_format=torch.channels_last)
    with _timed("maxpool2x2_fwd_idx", 4.0 * n * c * (h * w + 1.25 * (h // 2) * (w // 2))):
        _cabi.lib().pd_maxpool2x2_fwd_idx_nhwc_f32(_ptr(x), _ptr(y), _ptr(idx), n, h, w, c, int(relu),
                                                   _cabi.stream_ptr())
    return y, idx


def maxpool2x2_idx_backward(dy, idx, h, w, relu_mask=False):
    """dx [N,C,h,w] of a 2x2 pooling from the pooled gradient and the forward's index bytes."""
    _check(dy, "dy")
    _check(idx, "idx", torch.uint8)
    dy = to_nhwc(dy)
    n, ho, wo, c = _nhwc_dims(dy)
    if (ho, wo) != (h // 2, w // 2) or idx.shape != dy.shape or not idx.is_contiguous(memory_format=torch.channels_last):
        raise ValueError("maxpool2x2_idx_backward: dy %s / idx %s do not belong to a %dx%d input"
                         % (tuple(dy.shape), tuple(idx.shape), h, w))
    dx = torch.empty((n, c, h, w), dtype=torch.float32, device=dy.device, memory_format=torch.channels_last)
    with _timed("maxpool2x2_bwd_idx", 4.0 * n * c * (h * w + 1.25 * ho * wo)):
        _cabi.lib().pd_maxpool2x2_bwd_idx_nhwc_f32(_ptr(dy), _ptr(idx), _ptr(dx), n, h, w, c, int(relu_mask),
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


def label_smoothing_forward(logits, target, padding_idx, smoothing, divisor):
    """NLL loss with label smoothing over rows of ``logits`` [R, V] (seq2seq/train/smoothing.py:23-34):
    sum over non-padding rows of (1-smoothing)*nll + smoothing*mean(-logprob), divided by ``divisor``.
    Returns (loss[()], lse[R]); lse feeds the backward."""
    _rowmajor2d(logits, "logits")
    _check(target, "target", torch.int64)
    R, V = logits.shape
    if R == 0 or V == 0:
        raise ValueError("label_smoothing: empty logits %s" % (tuple(logits.shape),))
    if target.numel() != R or not target.is_contiguous():
        raise ValueError("label_smoothing: target must be a contiguous vector of %d rows" % R)
    dev = logits.device
    loss = torch.empty((), dtype=torch.float32, device=dev)
    row_loss = torch.empty(R, dtype=torch.float32, device=dev)
    lse = torch.empty(R, dtype=torch.float32, device=dev)
    ld = logits.stride(0) if R > 1 else V
    with _timed("label_smoothing_fwd", 4.0 * R * V):
        _cabi.lib().pd_label_smoothing_fwd_f32(_ptr(logits), _ptr(target), _ptr(loss), _ptr(row_loss), _ptr(lse),
                                               R, V, ld, int(padding_idx), float(smoothing), float(divisor),
                                               _cabi.stream_ptr())
    return loss, lse


def label_smoothing_backward(logits, target, lse, grad_loss, padding_idx, smoothing, divisor):
    R, V = logits.shape
    _check(grad_loss, "grad_loss")
    grad_loss = grad_loss.reshape(1).contiguous()
    d = torch.empty((R, V), dtype=torch.float32, device=logits.device)
    ld = logits.stride(0) if R > 1 else V
    with _timed("label_smoothing_bwd", 8.0 * R * V):
        _cabi.lib().pd_label_smoothing_bwd_f32(_ptr(logits), _ptr(target), _ptr(lse), _ptr(grad_loss), _ptr(d),
                                               R, V, ld, V, int(padding_idx), float(smoothing), float(divisor),
                                               _cabi.stream_ptr())
    return d


def _varlen_rows(x, name):
    """(T, B, row_bytes, pitch_bytes) of a [T, B, ...] tensor whose (t, b) rows are dense and evenly spaced:
    a contiguous tensor or a slice of the last dimension of one."""
    _cabi.require_device(x, name)
    if x.dim() < 2:
        raise ValueError("%s: input must be [T, B, ...], got shape %s" % (name, tuple(x.shape)))
    if x.element_size() not in (2, 4):
        raise TypeError("%s: element size must be 2 or 4 bytes, got %s" % (name, x.dtype))
    T, B = x.shape[0], x.shape[1]
    row = 1
    for d in reversed(range(2, x.dim())):
        if x.shape[d] != 1 and x.stride(d) != row:
            raise ValueError("%s: trailing dimensions must be dense, got shape %s stride %s"
                             % (name, tuple(x.shape), x.stride()))
        row *= x.shape[d]
    pitch = x.stride(1) if B > 1 else (x.stride(0) // max(B, 1) if T > 1 else row)
    if pitch < row or (T > 1 and x.stride(0) != B * pitch):
        raise ValueError("%s: rows must be evenly spaced, got shape %s stride %s"
                         % (name, tuple(x.shape), x.stride()))
    return T, B, row * x.element_size(), pitch * x.element_size()


def _varlen_call(fn, name, x, lengths, out):
    T, B, row_bytes, in_pitch = _varlen_rows(x, name)
    _check(lengths, "lengths", torch.int64)
    if lengths.dim() != 1 or lengths.numel() != B or not lengths.is_contiguous():
        raise ValueError("Expected `len(lengths)` to be equal to batch_size, but got %d (batch_size=%d)"
                         % (lengths.numel(), B))
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    elif out.shape != x.shape or out.dtype != x.dtype:
        raise ValueError("%s: out must have the input's shape and dtype" % name)
    out_pitch = _varlen_rows(out, name + " (out)")[3]
    with _timed(name, 2.0 * T * B * row_bytes):
        fn(_ptr(x), _ptr(out), _ptr(lengths), T, B, row_bytes, in_pitch, out_pitch, _cabi.stream_ptr())
    return out


def revert_varlen(x, lengths, out=None):
    """Every sequence of ``x`` [T, B, ...] reversed in time over its own length, zeros behind it
    (seq2seq/csrc/pack_utils_kernel.cu:25-62).  ``lengths``: B int64 values on the device, 0 < length <= T.
    ``x`` and ``out`` may be slices of the last dimension of wider tensors; they must not overlap."""
    return _varlen_call(_cabi.lib().pd_revert_varlen, "revert_varlen", x, lengths, out)


def length_mask_apply(x, lengths, out=None):
    """``x * set_mask(lengths).unsqueeze(-1)``: positions t >= lengths[b] of ``x`` [T, B, ...] become 0
    (seq2seq/models/encoder.py:51,55).  ``out`` may be ``x`` itself."""
    return _varlen_call(_cabi.lib().pd_length_mask_apply, "length_mask_apply", x, lengths, out)


def set_mask(lengths):
    """``set_mask_cpp`` (seq2seq/csrc/pack_utils.cpp:13-31): host uint8 mask [lengths[0], B] of a 1-D host
    int64 tensor of lengths."""
    if lengths.dim() != 1 or lengths.device.type != "cpu" or lengths.dtype != torch.int64:
        raise ValueError("'lengths' argument should be a 1D CPU int64 tensor")
    lengths = lengths.contiguous()
    B = lengths.numel()
    T = int(lengths[0]) if B else 0
    mask = torch.empty((T, B), dtype=torch.uint8)
    _cabi.lib().pd_set_mask_u8(_vp(lengths.data_ptr()), B, T, _vp(mask.data_ptr()))
    return mask


# --------------------------------------------------------------------------------------
# 3x3 convolution (stride 1, padding 1), NHWC activations, KRSC filter
# --------------------------------------------------------------------------------------
def _filter_dims(w):
    _check(w, "weight")
    if w.dim() != 4 or w.shape[2:] != (3, 3):
        raise ValueError("conv3x3: weight must be [K, C, 3, 3], got %s" % (tuple(w.shape),))
    if not w.is_contiguous(memory_format=torch.channels_last):
        raise ValueError("conv3x3: weight must be in channels_last (K,R,S,C) memory order")
    return w.shape[0], w.shape[1]


# Which kernel computes 3x3 convolutions and their input gradients: "auto" takes the Winograd
# F(2x2, 3x3) kernel where it applies and pays (8 | C, C >= 16, K >= 32), "direct" always the
# direct kernel, "winograd" the Winograd kernel wherever it applies.
_CONV_ALGO = "auto"


def set_conv_algorithm(name):
    global _CONV_ALGO
    if name not in ("auto", "direct", "winograd"):
        raise ValueError("conv algorithm must be 'auto', 'direct' or 'winograd'")
    _CONV_ALGO = name


def set_conv_pieces(mode):
    """Work items of the Winograd forward / input-gradient kernel for stacked batches whose width is a multiple of
    8 or 4 but not of 16 pixels: "auto" (pieces of 16 x 8 or 16 x 4 pixels when they lower the busiest compute
    unit's item count), "always", "never".  Same results bit for bit."""
    _cabi.lib().pd_conv3x3_winograd_set_pieces({"auto": 0, "always": 1, "never": -1}[mode])


def set_conv_wgrad_strips(mode):
    """Strips of the Winograd weight-gradient kernel: "auto" (upright strips of 16 rows x 2 columns of the stacked
    batch where the width is no multiple of 16 pixels), "flat" (2 x 16 pixels always), "upright" (wherever the shape
    allows).  The results differ by the summation order only."""
    _cabi.lib().pd_conv3x3_winograd_set_wgrad_strips({"auto": 0, "flat": 1, "upright": 2}[mode])


def _use_winograd(c, k, h, w):
    """Whether a convolution with c input and k output channels on h x w images takes the Winograd kernel:
    channel counts it supports, an image it can address with 32-bit offsets (the limits its entry point
    checks), and, unless forced, enough channels for it to pay."""
    if _CONV_ALGO == "direct" or not _cabi.lib().pd_conv3x3_winograd_supported(c, k):
        return False
    if h * w * max(c, k) >= 1 << 29 or c * 16 * 64 * 4 >= 1 << 31:
        return False
    return _CONV_ALGO == "winograd" or (c >= 16 and k >= 32)


def _winograd_conv(x, w, bias, in_mask, out_mask, n, h, wd, c, k, relu, rot180):
    """The convolution with c input and k output channels through the Winograd kernels; ``w`` is its
    own [k,c,3,3] filter, or with ``rot180`` the [c,k,3,3] filter of the layer whose input gradient
    this is."""
    lib = _cabi.lib()
    nbytes = ctypes.c_uint64()
    lib.pd_conv3x3_winograd_filter_bytes(c, k, ctypes.byref(nbytes))
    u = torch.empty(nbytes.value // 4, dtype=torch.float32, device=x.device)
    lib.pd_conv3x3_winograd_filter_f32(_ptr(w), _ptr(u), c, k, int(rot180), _cabi.stream_ptr())
    y = torch.empty((n, k, h, wd), dtype=torch.float32, device=x.device, memory_format=torch.channels_last)
    with _timed("conv3x3_winograd_kernel", 18.0 * c * k * n * h * wd):
        lib.pd_conv3x3_winograd_fwd_nhwc_f32(_ptr(x), _ptr(u), _ptr(bias), _ptr(in_mask), _ptr(out_mask), _ptr(y),
                                             n, h, wd, c, k, int(relu), _cabi.stream_ptr())
    return y


def conv3x3_forward(x, w, bias=None, relu=False):
    """y = conv2d(x, w, bias, stride 1, padding 1) (+ReLU).  x: NHWC-ordered [N,C,H,W]."""
    _check(x, "x")
    n, h, wd, c = _nhwc_dims(x)
    k, cw = _filter_dims(w)
    if cw != c:
        raise ValueError("conv3x3: input has %d channels, filter expects %d" % (c, cw))
    if bias is not None:
        _check(bias, "bias")
        if bias.numel() != k or not bias.is_contiguous():
            raise ValueError("conv3x3: bias must be a contiguous vector of K=%d" % k)
    if _use_winograd(c, k, h, wd):
        return _winograd_conv(x, w, bias, None, None, n, h, wd, c, k, relu, False)
    y = torch.empty((n, k, h, wd), dtype=torch.float32, device=x.device, memory_format=torch.channels_last)
    with _timed("conv3x3_fwd_kernel" if c > 8 else "conv3x3_fwd_kernel_smallc", 18.0 * c * k * n * h * wd):
        _cabi.lib().pd_conv3x3_fwd_nhwc_f32(_ptr(x), _ptr(w), _ptr(bias), _ptr(y), n, h, wd, c, k, int(relu),
                                            _cabi.stream_ptr())
    return y


def conv3x3_forward_pool(x, w, bias=None, relu=False):
    """``maxpool2x2_idx(conv3x3_forward(x, w, bias, relu))``: returns (pooled output, index bytes).  Where the
    Winograd kernel applies, the pooling happens in its epilogue and the full-resolution output is never
    written."""
    _check(x, "x")
    n, h, wd, c = _nhwc_dims(x)
    k, cw = _filter_dims(w)
    if cw != c:
        raise ValueError("conv3x3: input has %d channels, filter expects %d" % (c, cw))
    if not (_use_winograd(c, k, h, wd) and h >= 2 and wd >= 2):
        return maxpool2x2_idx(conv3x3_forward(x, w, bias, relu))
    if bias is not None:
        _check(bias, "bias")
        if bias.numel() != k or not bias.is_contiguous():
            raise ValueError("conv3x3: bias must be a contiguous vector of K=%d" % k)
    lib = _cabi.lib()
    nbytes = ctypes.c_uint64()
    lib.pd_conv3x3_winograd_filter_bytes(c, k, ctypes.byref(nbytes))
    u = torch.empty(nbytes.value // 4, dtype=torch.float32, device=x.device)
    lib.pd_conv3x3_winograd_filter_f32(_ptr(w), _ptr(u), c, k, 0, _cabi.stream_ptr())
    y = torch.empty((n, k, h // 2, wd // 2), dtype=torch.float32, device=x.device,
                    memory_format=torch.channels_last)
    idx = torch.empty((n, k, h // 2, wd // 2), dtype=torch.uint8, device=x.device,
                      memory_format=torch.channels_last)
    with _timed("conv3x3_winograd_kernel", 18.0 * c * k * n * h * wd):
        lib.pd_conv3x3_winograd_fwd_pool_nhwc_f32(_ptr(x), _ptr(u), _ptr(bias), _ptr(y), _ptr(idx), n, h, wd, c, k,
                                                  int(relu), _cabi.stream_ptr())
    return y, idx


def conv3x3_input_grad(dy, w, relu_out=None, x_rectified=None):
    """dx of conv3x3_forward: the forward kernel on dy with the 180-degree-rotated filter.
    ``relu_out`` (the layer's fused-ReLU output) masks dy while it is loaded.  ``x_rectified``
    (the layer's input, when that input is the output of a ReLU) zeroes dx where the input is
    not positive: the producing layer's ReLU backward, applied as dx is stored."""
    _check(dy, "dy")
    if relu_out is not None and not _dense_same_order(relu_out, dy):
        raise ValueError("conv3x3_input_grad: relu_out must have dy's shape and memory order")
    if x_rectified is not None:
        _check(x_rectified, "x_rectified")
        if (x_rectified.dim() != 4 or x_rectified.shape[0] != dy.shape[0] or x_rectified.shape[2:] != dy.shape[2:]
                or x_rectified.shape[1] != w.shape[1]
                or not x_rectified.is_contiguous(memory_format=torch.channels_last)):
            raise ValueError("conv3x3_input_grad: x_rectified must be the layer's channels_last input")
    n, h, wd, k = _nhwc_dims(dy)
    kw, c = _filter_dims(w)
    if kw != k:
        raise ValueError("conv3x3_input_grad: dy has %d channels, filter has %d outputs" % (k, kw))
    if _use_winograd(k, c, h, wd):
        return _winograd_conv(dy, w, None, relu_out, x_rectified, n, h, wd, k, c, False, True)
    lib = _cabi.lib()
    # rotated filter: logical [C, K, 3, 3] in channels_last order = memory [C][3][3][K]
    wr = torch.empty((c, k, 3, 3), dtype=torch.float32, device=w.device, memory_format=torch.channels_last)
    lib.pd_conv3x3_filter_rot180_f32(_ptr(w), _ptr(wr), k, c, _cabi.stream_ptr())
    dx = torch.empty((n, c, h, wd), dtype=torch.float32, device=dy.device, memory_format=torch.channels_last)
    with _timed("conv3x3_fwd_kernel" if k > 8 else "conv3x3_fwd_kernel_smallc", 18.0 * c * k * n * h * wd):
        lib.pd_conv3x3_dgrad_nhwc_f32(_ptr(dy), _ptr(wr), _ptr(relu_out), _ptr(x_rectified), _ptr(dx), n, h, wd, k, c,
                                      _cabi.stream_ptr())
    return dx


def conv3x3_input_grad_unpool_supported(dy, w):
    """Whether conv3x3_input_grad_unpool has a kernel for this gradient (the Winograd kernel applies and the
    full-resolution gradient fits its addressing)."""
    n, h, wd, k = _nhwc_dims(dy)
    kw, c = _filter_dims(w)
    return kw == k and _use_winograd(k, c, h, wd) and h * wd * c < 1 << 27


def conv3x3_input_grad_unpool(dy, w, idx):
    """``conv3x3_input_grad`` for a layer whose input came out of a ReLU + 2x2 max pooling with index
    bytes ``idx`` (``maxpool2x2_idx`` or ``conv3x3_forward_pool``): returns (dx, dx_full) with dx masked
    where the pooled maximum was not positive and ``dx_full = maxpool2x2_idx_backward(dx, idx,
    relu_mask=True)`` for a pooling input of exactly twice the size, both written by the convolution
    kernel's epilogue."""
    _check(dy, "dy")
    _check(idx, "idx", torch.uint8)
    n, h, wd, k = _nhwc_dims(dy)
    kw, c = _filter_dims(w)
    if kw != k:
        raise ValueError("conv3x3_input_grad_unpool: dy has %d channels, filter has %d outputs" % (k, kw))
    if tuple(idx.shape) != (n, c, h, wd) or not idx.is_contiguous(memory_format=torch.channels_last):
        raise ValueError("conv3x3_input_grad_unpool: idx must be the channels_last index bytes of the layer's input")
    if not conv3x3_input_grad_unpool_supported(dy, w):
        raise ValueError("conv3x3_input_grad_unpool: no kernel for this shape (see conv3x3_input_grad_unpool_supported)")
    lib = _cabi.lib()
    nbytes = ctypes.c_uint64()
    lib.pd_conv3x3_winograd_filter_bytes(k, c, ctypes.byref(nbytes))
    u = torch.empty(nbytes.value // 4, dtype=torch.float32, device=dy.device)
    lib.pd_conv3x3_winograd_filter_f32(_ptr(w), _ptr(u), k, c, 1, _cabi.stream_ptr())
    dx = torch.empty((n, c, h, wd), dtype=torch.float32, device=dy.device, memory_format=torch.channels_last)
    full = torch.empty((n, c, 2 * h, 2 * wd), dtype=torch.float32, device=dy.device,
                       memory_format=torch.channels_last)
    with _timed("conv3x3_winograd_kernel", 18.0 * c * k * n * h * wd):
        lib.pd_conv3x3_winograd_fwd_unpool_nhwc_f32(_ptr(dy), _ptr(u), _ptr(idx), _ptr(dx), _ptr(full), n, h, wd, k, c,
                                                    _cabi.stream_ptr())
    return dx, full


def conv3x3_weight_grad(x, dy, with_bias=True, relu_out=None):
    """(dw [K,C,3,3] channels_last, dbias [K] or None).  ``relu_out`` masks dy as in
    conv3x3_input_grad."""
    if relu_out is not None and not _dense_same_order(relu_out, dy):
        raise ValueError("conv3x3_weight_grad: relu_out must have dy's shape and memory order")
    _check(x, "x")
    _check(dy, "dy")
    n, h, wd, c = _nhwc_dims(x)
    n2, h2, w2, k = _nhwc_dims(dy)
    if (n, h, wd) != (n2, h2, w2):
        raise ValueError("conv3x3_weight_grad: x %s and dy %s disagree" % (tuple(x.shape), tuple(dy.shape)))
    lib = _cabi.lib()
    nbytes = ctypes.c_uint64()
    if (relu_out is None and _CONV_ALGO != "direct" and lib.pd_conv3x3_winograd_wgrad_supported(c, k)
            and wd * max(c, k) < 1 << 28 and (n * h + 2 * h + 8) * wd < 1 << 31):
        lib.pd_conv3x3_winograd_wgrad_workspace_bytes(c, k, ctypes.byref(nbytes))
        ws = torch.empty(nbytes.value, dtype=torch.uint8, device=x.device)
        dw = torch.empty((k, c, 3, 3), dtype=torch.float32, device=x.device, memory_format=torch.channels_last)
        db = torch.empty(k, dtype=torch.float32, device=x.device) if with_bias else None
        with _timed("conv3x3_winograd_wgrad", 18.0 * c * k * n * h * wd):
            lib.pd_conv3x3_winograd_wgrad_nhwc_f32(_ptr(x), _ptr(dy), _ptr(dw), _ptr(db), _ptr(ws), nbytes.value,
                                                   n, h, wd, c, k, _cabi.stream_ptr())
        return dw, db
    lib.pd_conv3x3_wgrad_workspace_bytes(n, h, wd, c, k, ctypes.byref(nbytes))
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=x.device)
    dw = torch.empty((k, c, 3, 3), dtype=torch.float32, device=x.device, memory_format=torch.channels_last)
    db = torch.empty(k, dtype=torch.float32, device=x.device) if with_bias else None
    with _timed("conv3x3_wgrad", 18.0 * c * k * n * h * wd):
        lib.pd_conv3x3_wgrad_nhwc_f32(_ptr(x), _ptr(dy), _ptr(relu_out), _ptr(dw), _ptr(db), _ptr(ws), nbytes.value,
                                      n, h, wd, c, k, _cabi.stream_ptr())
    return dw, db


# --------------------------------------------------------------------------------------
# LSTM / embedding / residual add
# --------------------------------------------------------------------------------------
def add(a, b):
    _check(a, "a")
    _check(b, "b")
    if a.shape != b.shape:
        raise ValueError("add: shapes differ (%s vs %s)" % (tuple(a.shape), tuple(b.shape)))
    if not _is_dense(a):
        a = a.contiguous()
    if b.stride() != a.stride():
        b2 = torch.empty_like(a)
        b2.copy_(b)
        b = b2
    y = torch.empty_like(a)
    _cabi.lib().pd_add_f32(_ptr(a), _ptr(b), _ptr(y), a.numel(), _cabi.stream_ptr())
    return y


def lstm_forward(x, w_ih, w_hh, b_ih, b_hh):
    """Single-layer, uni-directional LSTM over x[T,B,I] from zero state.
    Returns (y[T,B,H], saved) where saved = (gates[T,B,4H] activated, c[T,B,H])."""
    _check(x, "x")
    if x.dim() != 3:
        raise ValueError("lstm: input must be [T, B, I]")
    T, B, I = x.shape
    H = w_hh.shape[1]
    if tuple(w_ih.shape) != (4 * H, I) or tuple(w_hh.shape) != (4 * H, H):
        raise ValueError("lstm: weight shapes %s / %s do not fit input %d, hidden %d"
                         % (tuple(w_ih.shape), tuple(w_hh.shape), I, H))
    x2 = x.contiguous().view(T * B, I)
    lib, s = _cabi.lib(), _cabi.stream_ptr
    # input projection of all time steps at once
    gates = gemm(x2, w_ih, trans_b=True).view(T, B, 4 * H)
    y = torch.empty((T, B, H), dtype=torch.float32, device=x.device)
    c = torch.empty((T, B, H), dtype=torch.float32, device=x.device)
    # the recurrent product h_{t-1} W_hh^T has only B rows: split over k, summed inside the cell kernel
    rec = torch.empty((splitk_factor(B, 4 * H, H), B, 4 * H), dtype=torch.float32, device=x.device)
    if kernel_timer is None and w_hh.is_contiguous():
        # the time loop in native code: one call instead of 2 T - 1
        lib.pd_lstm_recurrence_fwd_f32(_ptr(gates), _ptr(w_hh), _ptr(b_ih), _ptr(b_hh), _ptr(rec), rec.size(0),
                                       _ptr(c), _ptr(y), T, B, H, s())
        return y, (gates, c)
    for t in range(T):      # the same loop with an event pair around every product (per-kernel timing)
        if t > 0:
            gemm_splitk(y[t - 1], w_hh, False, True, rec)
        lib.pd_lstm_cell_fwd_f32(_ptr(gates[t]), _ptr(rec), rec.size(0) if t > 0 else 0, _ptr(b_ih), _ptr(b_hh),
                                 _ptr(c[t - 1]) if t > 0 else None, _ptr(c[t]), _ptr(y[t]), B, H, s())
    return y, (gates, c)


def lstm_backward(dy, x, y, gates, c, w_ih, w_hh, need_dx=True):
    """Gradients of lstm_forward: (dx or None, dw_ih, dw_hh, db) with db = db_ih = db_hh."""
    T, B, I = x.shape
    H = w_hh.shape[1]
    dy = dy.contiguous()
    lib, s = _cabi.lib(), _cabi.stream_ptr
    dgates = torch.empty((T, B, 4 * H), dtype=torch.float32, device=x.device)
    dc = torch.empty((B, H), dtype=torch.float32, device=x.device)
    dh_rec = torch.empty((splitk_factor(B, H, 4 * H), B, H), dtype=torch.float32, device=x.device)
    native = kernel_timer is None and w_hh.is_contiguous() and gates.is_contiguous() and c.is_contiguous()
    if native:
        lib.pd_lstm_recurrence_bwd_f32(_ptr(gates), _ptr(c), _ptr(dy), _ptr(w_hh), _ptr(dh_rec), dh_rec.size(0),
                                       _ptr(dc), _ptr(dgates), T, B, H, s())
    for t in (() if native else range(T - 1, -1, -1)):
        lib.pd_lstm_cell_bwd_f32(_ptr(gates[t]), _ptr(c[t - 1]) if t > 0 else None, _ptr(c[t]), _ptr(dy[t]),
                                 _ptr(dh_rec) if t < T - 1 else None, dh_rec.size(0), _ptr(dc), _ptr(dgates[t]), B, H,
                                 int(t == T - 1), s())
        if t > 0:
            gemm_splitk(dgates[t], w_hh, False, False, dh_rec)      # [B,4H] @ [4H,H], split over 4H
    dg2 = dgates.view(T * B, 4 * H)
    x2 = x.contiguous().view(T * B, I)
    dw_ih = gemm(dg2, x2, trans_a=True)
    # h_{t-1} for t >= 1 is y[t-1]; the t = 0 term has h = 0
    if T > 1:
        dw_hh = gemm(dgates[1:].view((T - 1) * B, 4 * H), y[:-1].view((T - 1) * B, H), trans_a=True)
    else:
        dw_hh = torch.zeros_like(w_hh)
    db = colsum(dg2)
    dx = gemm(dg2, w_ih).view(T, B, I) if need_dx else None
    return dx, dw_ih, dw_hh, db


def embedding_forward(ids, weight):
    _check(ids, "ids", torch.int64)
    _check(weight, "weight")
    if weight.dim() != 2 or not weight.is_contiguous():
        raise ValueError("embedding: weight must be a contiguous [V, D] matrix")
    flat = ids.contiguous().view(-1)
    V, D = weight.shape
    out = torch.empty((flat.numel(), D), dtype=torch.float32, device=weight.device)
    _cabi.lib().pd_embedding_fwd_f32(_ptr(flat), _ptr(weight), _ptr(out), flat.numel(), D, V, _cabi.stream_ptr())
    return out.view(*ids.shape, D)


def embedding_backward(ids, dout, num_embeddings, padding_idx=None):
    _check(ids, "ids", torch.int64)
    _check(dout, "dout")
    flat = ids.contiguous().view(-1)
    D = dout.shape[-1]
    d2 = dout.contiguous().view(-1, D)
    dw = torch.empty((num_embeddings, D), dtype=torch.float32, device=dout.device)
    _cabi.lib().pd_embedding_bwd_f32(_ptr(flat), _ptr(d2), _ptr(dw), flat.numel(), D, num_embeddings,
                                     -1 if padding_idx is None else int(padding_idx), _cabi.stream_ptr())
    return dw


# --------------------------------------------------------------------------------------
# bf16 transformer ops
# --------------------------------------------------------------------------------------
BF16 = torch.bfloat16


def cast_bf16(x):
    _check(x, "x")
    x = x.contiguous()
    y = torch.empty(x.shape, dtype=BF16, device=x.device)
    _cabi.lib().pd_cast_f32_to_bf16(_ptr(x), _ptr(y), x.numel(), _cabi.stream_ptr())
    return y


def cast_f32(x):
    _check(x, "x", BF16)
    x = x.contiguous()
    y = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    _cabi.lib().pd_cast_bf16_to_f32(_ptr(x), _ptr(y), x.numel(), _cabi.stream_ptr())
    return y


def bf16_weight(p):
    """bf16 image of a master parameter: the ring's image of the loaded slot when the
    optimizer keeps one, otherwise a fresh cast."""
    views = getattr(p, "_pd_bf16_views", None)
    if views is not None:
        return views[p._pd_arena.live_slot]
    return cast_bf16(p.detach())


def _mat_bf16(t, name):
    _check(t, name, BF16)
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError("%s must be a row-major 2-D bf16 matrix" % name)
    return t


def gemm_bf16(a, b, trans_a=False, trans_b=False, out=None, out_f32=False, alpha=1.0, beta=0.0, bias=None,
              residual=None):
    """out[M,N] = alpha * op(a) op(b) (+bias) (+residual) (+beta*out for fp32 out)."""
    _mat_bf16(a, "a")
    _mat_bf16(b, "b")
    M, K = (a.size(1), a.size(0)) if trans_a else (a.size(0), a.size(1))
    Kb, N = (b.size(1), b.size(0)) if trans_b else (b.size(0), b.size(1))
    if K != Kb:
        raise ValueError("gemm_bf16: inner dimensions differ (%d vs %d)" % (K, Kb))
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32 if out_f32 else BF16, device=a.device)
    else:
        out_f32 = out.dtype == torch.float32
        if tuple(out.shape) != (M, N) or out.stride(1) != 1 or not out.is_cuda:
            raise ValueError("gemm_bf16: bad out tensor")
    if residual is not None:
        _mat_bf16(residual, "residual")
        if tuple(residual.shape) != (M, N):
            raise ValueError("gemm_bf16: residual shape")
    if bias is not None:
        _check(bias, "bias")
    with _timed("gemm_bf16", 2.0 * M * N * K):
        _cabi.lib().pd_gemm_bf16(int(trans_a), int(trans_b), M, N, K, _ptr(a), a.stride(0), _ptr(b), b.stride(0),
                                 _ptr(out), out.stride(0), int(out_f32), float(alpha), float(beta), _ptr(bias),
                                 _ptr(residual), residual.stride(0) if residual is not None else 0, 1, 1, None,
                                 _cabi.stream_ptr())
    return out


def gemm_bf16_gelu(a, b, trans_b=False, bias=None):
    """(f, g) with f = a op(b) + bias and g = gelu(f) (f as rounded to bf16), both from the GEMM kernel's
    epilogue: the first linear layer of a feed-forward block and its activation."""
    _mat_bf16(a, "a")
    _mat_bf16(b, "b")
    M, K = a.shape
    Kb, N = (b.size(1), b.size(0)) if trans_b else (b.size(0), b.size(1))
    if K != Kb:
        raise ValueError("gemm_bf16_gelu: inner dimensions differ (%d vs %d)" % (K, Kb))
    if bias is not None:
        _check(bias, "bias")
    f = torch.empty((M, N), dtype=BF16, device=a.device)
    g = torch.empty((M, N), dtype=BF16, device=a.device)
    with _timed("gemm_bf16", 2.0 * M * N * K):
        _cabi.lib().pd_gemm_bf16_gelu(0, 0, int(trans_b), M, N, K, _ptr(a), a.stride(0), _ptr(b), b.stride(0), _ptr(f),
                                      N, _ptr(bias), _ptr(g), N, _cabi.stream_ptr())
    return f, g


def gemm_bf16_gelu_backward(dy, w, f):
    """df = (dy w) * gelu'(f): the input gradient of the second linear layer of a feed-forward block taken
    through the activation in the GEMM's epilogue; ``f`` is the stored pre-activation [M, N]."""
    _mat_bf16(dy, "dy")
    _mat_bf16(w, "w")
    _mat_bf16(f, "f")
    M, K = dy.shape
    Kb, N = w.shape
    if K != Kb or tuple(f.shape) != (M, N) or not f.is_contiguous():
        raise ValueError("gemm_bf16_gelu_backward: shapes %s x %s -> %s do not fit"
                         % (tuple(dy.shape), tuple(w.shape), tuple(f.shape)))
    df = torch.empty((M, N), dtype=BF16, device=dy.device)
    with _timed("gemm_bf16", 2.0 * M * N * K):
        _cabi.lib().pd_gemm_bf16_gelu(1, 0, 0, M, N, K, _ptr(dy), dy.stride(0), _ptr(w), w.stride(0), _ptr(df), N, None,
                                      _ptr(f), N, _cabi.stream_ptr())
    return df


def gemm_bf16_wgrad(dy, x, acc=None):
    """Weight gradient of a bf16 Linear layer in fp32: ``dy[T, N]^T x[T, K]``, returned as a new [N, K] tensor or
    added to ``acc``.  A product with few output tiles (the 1024 x 1024 attention projection: 64 tiles of
    128 x 128 for 256 CUs) is split over the tokens into partial products, one batch entry each, which a second
    kernel adds in index order (deterministic)."""
    _mat_bf16(dy, "dy")
    _mat_bf16(x, "x")
    T, N = dy.shape
    K = x.shape[1]
    tiles = -(-N // 128) * -(-K // 128)
    splits = min(256 // tiles, T // 1024, 8) if tiles <= 64 else 1
    if splits < 2 or T % (splits * 128) != 0 or N % 4 != 0 or K % 4 != 0:
        if acc is None:
            return gemm_bf16(dy, x, trans_a=True, out_f32=True)
        return gemm_bf16(dy, x, trans_a=True, out=acc, beta=1.0)
    part = torch.empty((splits, N, K), dtype=torch.float32, device=dy.device)
    rows = T // splits
    strides = (ctypes.c_int64 * 6)(rows * dy.stride(0), 0, rows * x.stride(0), 0, N * K, 0)
    lib = _cabi.lib()
    with _timed("gemm_bf16", 2.0 * N * K * T):
        lib.pd_gemm_bf16(1, 0, N, K, rows, _ptr(dy), dy.stride(0), _ptr(x), x.stride(0), _ptr(part), K, 1, 1.0, 0.0,
                         None, None, 0, splits, 1, strides, _cabi.stream_ptr())
    out = acc if acc is not None else torch.empty((N, K), dtype=torch.float32, device=dy.device)
    lib.pd_splitk_reduce_f32(_ptr(part), splits, N, K, None, 0, 1.0 if acc is not None else 0.0, _ptr(out),
                             out.stride(0), _cabi.stream_ptr())
    return out


def _batched(ta, tb, M, N, K, A, a_off, lda, B, b_off, ldb, C, c_off, ldc, alpha, bo, bi, strides):
    arr = (ctypes.c_int64 * 6)(*strides)
    es = 2
    with _timed("gemm_bf16_batched", 2.0 * M * N * K * bo * bi):
        _cabi.lib().pd_gemm_bf16(int(ta), int(tb), M, N, K, _vp(A.data_ptr() + a_off * es), lda,
                                 _vp(B.data_ptr() + b_off * es), ldb, _vp(C.data_ptr() + c_off * es), ldc, 0,
                                 float(alpha), 0.0, None, None, 0, bo, bi, arr, _cabi.stream_ptr())


def attention_forward(qkv, batch, seq, heads, need_probs=False):
    """qkv: [batch*seq, 3H] bf16 (Q | K | V, heads contiguous inside each).  Returns (ctx [batch*seq, H],
    aux) where aux is what attention_backward needs: on the fused path (head dimension 64, seq 128 / 256 /
    512) the fp32 vector lse2 [batch, heads, seq], otherwise -- or with need_probs -- the bf16
    probabilities [batch, heads, seq, seq]."""
    _mat_bf16(qkv, "qkv")
    H = qkv.size(1) // 3
    d = H // heads
    if qkv.size(0) != batch * seq or H * 3 != qkv.size(1) or d * heads != H or not qkv.is_contiguous():
        raise ValueError("attention: qkv shape %s does not fit batch %d seq %d heads %d"
                         % (tuple(qkv.shape), batch, seq, heads))
    dev = qkv.device
    ctx = torch.empty((batch * seq, H), dtype=BF16, device=dev)
    if _cabi.lib().pd_attention_fwd_supported(seq, d):
        probs = torch.empty((batch, heads, seq, seq), dtype=BF16, device=dev) if need_probs else None
        lse2 = None if need_probs else torch.empty((batch, heads, seq), dtype=torch.float32, device=dev)
        with _timed("attention_fwd", 4.0 * batch * heads * seq * seq * d):
            _cabi.lib().pd_attention_fwd_bf16(_ptr(qkv), _ptr(ctx), _ptr(probs), _ptr(lse2), batch, seq, heads, d,
                                              _cabi.stream_ptr())
        return ctx, (probs if need_probs else lse2)
    probs = torch.empty((batch, heads, seq, seq), dtype=BF16, device=dev)
    scale = 1.0 / (d ** 0.5)
    ld = 3 * H
    # scores = scale * Q K^T
    _batched(0, 1, seq, seq, d, qkv, 0, ld, qkv, H, ld, probs, 0, seq, scale, batch, heads,
             (seq * ld, d, seq * ld, d, heads * seq * seq, seq * seq))
    _cabi.lib().pd_softmax_fwd_bf16(_ptr(probs), _ptr(probs), batch * heads * seq, seq, _cabi.stream_ptr())
    # ctx = P V
    _batched(0, 0, seq, d, seq, probs, 0, seq, qkv, 2 * H, ld, ctx, 0, H, 1.0, batch, heads,
             (heads * seq * seq, seq * seq, seq * ld, d, seq * H, d))
    return ctx, probs


def attention_backward(dctx, qkv, aux, batch, seq, heads, ctx=None):
    """Gradient with respect to qkv; `aux` is the second result of attention_forward (lse2 needs `ctx`,
    the forward output, as well)."""
    _mat_bf16(dctx, "dctx")
    H = qkv.size(1) // 3
    d = H // heads
    dctx = dctx.contiguous()
    dev = qkv.device
    ld = 3 * H
    scale = 1.0 / (d ** 0.5)
    dqkv = torch.empty_like(qkv)
    if aux.dtype == torch.float32:
        if ctx is None:
            raise ValueError("attention_backward: the fused path needs ctx")
        _mat_bf16(ctx, "ctx")
        if tuple(ctx.shape) != (batch * seq, H) or not ctx.is_contiguous() or tuple(aux.shape) != (batch, heads, seq):
            raise ValueError("attention_backward: ctx must be a contiguous [batch*seq, H] matrix, lse2 [batch, heads, seq]")
        delta = torch.empty_like(aux)
        with _timed("attention_bwd", 10.0 * batch * heads * seq * seq * d):
            _cabi.lib().pd_attention_bwd_bf16(_ptr(qkv), _ptr(ctx), _ptr(dctx), _ptr(aux), _ptr(delta), _ptr(dqkv),
                                              batch, seq, heads, d, _cabi.stream_ptr())
        return dqkv
    probs = aux
    dP = torch.empty_like(probs)
    sP = (heads * seq * seq, seq * seq)
    # dP = dctx V^T
    _batched(0, 1, seq, seq, d, dctx, 0, H, qkv, 2 * H, ld, dP, 0, seq, 1.0, batch, heads,
             (seq * H, d, seq * ld, d) + sP)
    # dV = P^T dctx
    _batched(1, 0, seq, d, seq, probs, 0, seq, dctx, 0, H, dqkv, 2 * H, ld, 1.0, batch, heads,
             sP + (seq * H, d, seq * ld, d))
    # dS = P * (dP - sum(dP * P)), in place
    _cabi.lib().pd_softmax_bwd_bf16(_ptr(probs), _ptr(dP), _ptr(dP), batch * heads * seq, seq, _cabi.stream_ptr())
    # dQ = scale * dS K ; dK = scale * dS^T Q
    _batched(0, 0, seq, d, seq, dP, 0, seq, qkv, H, ld, dqkv, 0, ld, scale, batch, heads,
             sP + (seq * ld, d, seq * ld, d))
    _batched(1, 0, seq, d, seq, dP, 0, seq, qkv, 0, ld, dqkv, H, ld, scale, batch, heads,
             sP + (seq * ld, d, seq * ld, d))
    return dqkv


def layernorm_forward(x, gamma, beta, eps=1e-5):
    _mat_bf16(x, "x")
    M, H = x.shape
    y = torch.empty_like(x)
    mean = torch.empty(M, dtype=torch.float32, device=x.device)
    rstd = torch.empty(M, dtype=torch.float32, device=x.device)
    _cabi.lib().pd_layernorm_fwd_bf16(_ptr(x), _ptr(gamma), _ptr(beta), _ptr(y), _ptr(mean), _ptr(rstd), M, H,
                                      float(eps), _cabi.stream_ptr())
    return y, mean, rstd


def layernorm_backward(dy, x, gamma, mean, rstd, dgamma_acc=None, dbeta_acc=None, batch=None, residual=None):
    """Returns dx (+ ``residual``, a bf16 matrix of x's shape); dgamma/dbeta are added to the given fp32
    accumulators or returned fresh.  With a ``ColsumBatch`` the sums over the kernel's partial results are
    left to the batch's ``run``."""
    if residual is not None:
        _mat_bf16(residual, "residual")
        if residual.shape != x.shape or not residual.is_contiguous():
            raise ValueError("layernorm_backward: residual must be a contiguous matrix of x's shape")
    M, H = x.shape
    lib = _cabi.lib()
    nb = lib.pd_layernorm_bwd_partials(M)
    dx = torch.empty_like(x)
    pg = torch.empty((nb, H), dtype=torch.float32, device=x.device)
    pb = torch.empty((nb, H), dtype=torch.float32, device=x.device)
    lib.pd_layernorm_bwd_bf16(_ptr(dy), _ptr(x), _ptr(gamma), _ptr(mean), _ptr(rstd), _ptr(dx), _ptr(residual),
                              _ptr(pg), _ptr(pb), M, H, _cabi.stream_ptr())
    outs = []
    for part, acc in ((pg, dgamma_acc), (pb, dbeta_acc)):
        beta = 0.0 if acc is None else 1.0
        if acc is None:
            acc = torch.empty(H, dtype=torch.float32, device=x.device)
        if batch is not None:
            batch.add(part, acc, beta)
        else:
            lib.pd_colsum_f32(_ptr(part), _ptr(acc), nb, H, H, 1, beta, _cabi.stream_ptr())
        outs.append(acc)
    return dx, outs[0], outs[1]


def gelu(x):
    y = torch.empty_like(x)
    _cabi.lib().pd_gelu_fwd_bf16(_ptr(x), _ptr(y), x.numel(), _cabi.stream_ptr())
    return y


def gelu_backward(x, dy):
    dx = torch.empty_like(x)
    _cabi.lib().pd_gelu_bwd_bf16(_ptr(x), _ptr(dy), _ptr(dx), x.numel(), _cabi.stream_ptr())
    return dx


def add_bf16(a, b):
    y = torch.empty_like(a)
    _cabi.lib().pd_add_bf16(_ptr(a), _ptr(b), _ptr(y), a.numel(), _cabi.stream_ptr())
    return y


class ColsumBatch(object):
    """Column sums collected during a backward pass and computed together in two launches: ``add`` a bf16
    matrix (a Linear layer's output gradient) or an fp32 matrix of partial sums with the fp32 vector that
    receives (``beta=0``) or accumulates (``beta=1``) its column sums, then ``run`` once.  The matrices must
    stay alive until ``run``."""
    MAX_JOBS = 8
    SPLITS = 64

    def __init__(self):
        self.jobs = []

    def add(self, x, out, beta):
        if x.dim() != 2 or x.stride(1) != 1 or x.dtype not in (BF16, torch.float32):
            raise ValueError("ColsumBatch.add: x must be a row-major bf16 or fp32 matrix")
        if out.dtype != torch.float32 or out.numel() != x.shape[1] or not out.is_contiguous():
            raise ValueError("ColsumBatch.add: out must be a contiguous fp32 vector of x's column count")
        _cabi.require_device(x, "x")
        _cabi.require_device(out, "out")
        self.jobs.append((x, out, float(beta)))
        if len(self.jobs) == self.MAX_JOBS:
            self.run()

    def run(self):
        jobs, self.jobs = self.jobs, []
        n = len(jobs)
        if n == 0:
            return
        lib = _cabi.lib()
        xs = (ctypes.c_void_p * n)(*[j[0].data_ptr() for j in jobs])
        outs = (ctypes.c_void_p * n)(*[j[1].data_ptr() for j in jobs])
        kinds = (ctypes.c_int * n)(*[1 if j[0].dtype == BF16 else 0 for j in jobs])
        ms = (ctypes.c_uint64 * n)(*[j[0].shape[0] for j in jobs])
        ns = (ctypes.c_int * n)(*[j[0].shape[1] for j in jobs])
        lds = (ctypes.c_uint64 * n)(*[j[0].stride(0) if j[0].shape[0] > 1 else j[0].shape[1] for j in jobs])
        betas = (ctypes.c_float * n)(*[j[2] for j in jobs])
        need = ctypes.c_uint64()
        lib.pd_colsum_batch_workspace_floats(n, kinds, ns, self.SPLITS, ctypes.byref(need))
        ws = torch.empty(max(need.value, 1), dtype=torch.float32, device=jobs[0][0].device)
        lib.pd_colsum_batch(n, xs, kinds, outs, ms, ns, lds, betas, _ptr(ws), need.value, self.SPLITS,
                            _cabi.stream_ptr())


def colsum_bf16(x, acc=None):
    """fp32 column sums of a bf16 matrix; added to ``acc`` when given."""
    M, N = x.shape
    lib = _cabi.lib()
    # about two blocks per CU (a block covers 512 columns), at least 16 rows per split
    splits = max(1, min(512 // -(-N // 512), M // 16, 1024))
    part = torch.empty((splits, N), dtype=torch.float32, device=x.device)
    lib.pd_colsum_bf16(_ptr(x), _ptr(part), M, N, x.stride(0), splits, _cabi.stream_ptr())
    if acc is None:
        acc = torch.empty(N, dtype=torch.float32, device=x.device)
        lib.pd_colsum_f32(_ptr(part), _ptr(acc), splits, N, N, 1, 0.0, _cabi.stream_ptr())
    else:
        lib.pd_colsum_f32(_ptr(part), _ptr(acc), splits, N, N, 1, 1.0, _cabi.stream_ptr())
    return acc
