"""Stage-compute kernels (through the C ABI) against the fp32/fp64 torch CPU library --
the third-party routines the reference's stage modules call.

Tolerances: GEMM results are compared with an fp64 product; an fp32 dot product of
length K carries a relative rounding error of about sqrt(K)*6e-8 on its magnitude
sum |a||b|, so the bound is atol = 2e-6*sqrt(K)*max|a||b| with rtol 1e-5.  Element-wise
kernels must be bit-exact."""
import math

import pytest
import torch
import torch.nn.functional as F

from pipedream_amd import layers, ops

pytestmark = pytest.mark.gpu


def _gemm_case(M, N, K, ta, tb, bias=False, relu=False, beta=0.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn((K, M) if ta else (M, K), generator=g)
    b = torch.randn((N, K) if tb else (K, N), generator=g)
    bv = torch.randn(N, generator=g) if bias else None
    c0 = torch.randn(M, N, generator=g) if beta else None
    want = (a.double().t() if ta else a.double()) @ (b.double().t() if tb else b.double())
    if bias:
        want = want + bv.double()
    if beta:
        want = want + beta * c0.double()
    if relu:
        want = want.clamp_min(0)
    out = c0.cuda() if beta else None
    got = ops.gemm(a.cuda(), b.cuda(), trans_a=ta, trans_b=tb, bias=bv.cuda() if bias else None, relu=relu,
                   out=out, beta=beta)
    torch.cuda.synchronize()
    atol = 2e-6 * math.sqrt(max(K, 1)) * 9.0
    torch.testing.assert_close(got.cpu().double(), want, rtol=1e-5, atol=atol)


@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K", [(64, 64, 16), (64, 1024, 784), (130, 70, 33), (1, 10, 1024), (257, 129, 100),
                                   (5, 3, 1), (2048, 2304, 64)])
def test_gemm_layouts_and_ragged_shapes(M, N, K, ta, tb):
    _gemm_case(M, N, K, ta, tb)


def test_gemm_epilogues():
    _gemm_case(64, 1024, 784, False, True, bias=True, relu=True)
    _gemm_case(100, 50, 37, False, True, bias=True)
    _gemm_case(100, 50, 37, True, False, beta=1.0)
    _gemm_case(300, 300, 300, False, False, bias=True, relu=True, beta=0.5)


@pytest.mark.parametrize("M,N,K,ta,tb", [
    (128, 4096, 1024, False, True),     # LSTM recurrent forward: direct-to-LDS skinny kernel, k-contiguous B
    (128, 1024, 4096, False, False),    # LSTM recurrent backward: row-contiguous B
    (64, 1000, 4096, False, True),      # classifier: N not a multiple of the 128-column tile
    (5, 260, 2048, False, False),       # few rows, ragged columns
    (100, 132, 1040, False, True),      # K a multiple of 16 but not of 128: a short last round
    (64, 256, 1030, False, True),       # K not a multiple of 16: general split kernel
    (96, 512, 2048, True, False),       # transposed A: general split kernel
])
def test_gemm_split_k_paths(M, N, K, ta, tb):
    """Products with too few output tiles are split over k (ops.splitk_factor > 1); partial
    sums are added in a fixed order, so the result is reproducible bit for bit."""
    assert ops.splitk_factor(M, N, K, ta) > 1
    _gemm_case(M, N, K, ta, tb)
    _gemm_case(M, N, K, ta, tb, bias=True, relu=True, beta=0.5)
    g = torch.Generator().manual_seed(1)
    a = torch.randn((K, M) if ta else (M, K), generator=g).cuda()
    b = torch.randn((N, K) if tb else (K, N), generator=g).cuda()
    assert torch.equal(ops.gemm(a, b, trans_a=ta, trans_b=tb), ops.gemm(a, b, trans_a=ta, trans_b=tb))
    # explicit partials: more splits than k chunks leaves trailing partials at zero
    part = torch.full((70, M, N), float("nan")).cuda()
    ops.gemm_splitk(a, b, ta, tb, part)
    want = (a.double().t() if ta else a.double()) @ (b.double().t() if tb else b.double())
    torch.testing.assert_close(part.double().sum(0), want, rtol=1e-5, atol=2e-6 * math.sqrt(K) * 9.0)


def test_gemm_strided_views_and_identity():
    # leading dimension larger than the row; unaligned base (scalar load path)
    big = torch.randn(70, 90).cuda()
    a = big[:, 1:34]          # 33 cols, ld 90, 4-byte aligned only
    b = torch.randn(20, 33).cuda()
    got = ops.gemm(a, b, trans_b=True)
    torch.testing.assert_close(got.cpu().double(), a.cpu().double() @ b.cpu().double().t(), rtol=1e-5, atol=1e-4)
    # exactness: multiplying by the identity returns the operand bit-for-bit
    x = torch.randn(96, 64).cuda()
    assert torch.equal(ops.gemm(x, torch.eye(64).cuda()), x)
    assert torch.equal(ops.gemm(torch.eye(96).cuda(), x), x)
    assert torch.equal(ops.gemm(x, torch.eye(96).cuda(), trans_a=True), x.t().contiguous())


def test_gemm_rejects_bad_operands():
    a = torch.randn(4, 5).cuda()
    with pytest.raises(ValueError):
        ops.gemm(a, torch.randn(4, 6).cuda())
    with pytest.raises(ValueError):
        ops.gemm(a.t(), torch.randn(4, 6).cuda())     # not row-major
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.gemm(torch.randn(4, 5), torch.randn(5, 6))
    with pytest.raises(TypeError):
        ops.gemm(a.double(), torch.randn(5, 6).cuda().double())


@pytest.mark.parametrize("M,N", [(1, 1), (7, 130), (5000, 64), (200000, 10)])
def test_colsum(M, N):
    x = torch.randn(M, N)
    got = ops.colsum(x.cuda())
    torch.testing.assert_close(got.cpu().double(), x.double().sum(0), rtol=1e-5, atol=2e-6 * math.sqrt(M) * 4)


def test_relu_forward_backward_bit_exact():
    for n in (1, 5, 1024, 100003):
        x = torch.randn(n)
        dy = torch.randn(n)
        y = ops.relu(x.cuda())
        assert torch.equal(y.cpu(), x.clamp_min(0))
        dx = ops.relu_backward(dy.cuda(), y)
        assert torch.equal(dx.cpu(), dy * (x > 0))


@pytest.mark.parametrize("shape", [(2, 8, 6, 6), (3, 4, 7, 9), (1, 64, 224, 224), (2, 12, 2, 5)])
def test_maxpool_forward_backward_bit_exact(shape):
    g = torch.Generator().manual_seed(1)
    # quantised values force ties; torch's rule (first maximum in scan order) must hold
    x = (torch.randn(shape, generator=g) * 2).round() / 2
    x.requires_grad_(True)
    y_ref = F.max_pool2d(x, 2, 2)
    dy = torch.randn(y_ref.shape, generator=g)
    if y_ref.numel():
        y_ref.backward(dy)
    xg = x.detach().cuda().contiguous(memory_format=torch.channels_last)
    y = ops.maxpool2x2(xg)
    assert y.shape == y_ref.shape and torch.equal(y.cpu(), y_ref.detach())
    dx = ops.maxpool2x2_backward(xg, dy.cuda())
    assert torch.equal(dx.cpu(), x.grad if x.grad is not None else torch.zeros(shape))
    # fused ReLU mask: same as masking afterwards
    dxm = ops.maxpool2x2_backward(xg, dy.cuda(), relu_mask=True)
    assert torch.equal(dxm.cpu(), dx.cpu() * (x.detach() > 0))


@pytest.mark.parametrize("shape", [(2, 8, 6, 6), (3, 4, 7, 9), (1, 64, 224, 224), (2, 12, 2, 5), (1, 4, 1, 3)])
@pytest.mark.parametrize("relu", [False, True])
def test_maxpool_with_index_bytes_bit_exact(shape, relu):
    """The pooling the layers use: the forward also writes one byte per output element (window position of
    the first maximum, sign of the maximum), the backward reads only the pooled gradient and that byte.
    Against torch's max_pool2d and its autograd (after a ReLU when relu=True), bit for bit, with ties."""
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(shape, generator=g) * 2).round() / 2
    x.requires_grad_(True)
    if shape[2] >= 2 and shape[3] >= 2:
        y_ref = F.max_pool2d(F.relu(x) if relu else x, 2, 2)
    else:       # no window fits (torch refuses such an input): empty output, zero input gradient
        y_ref = torch.zeros(shape[0], shape[1], shape[2] // 2, shape[3] // 2)
    dy = torch.randn(y_ref.shape, generator=g)
    if y_ref.numel():
        y_ref.backward(dy)
    want_dx = x.grad if x.grad is not None else torch.zeros(shape)
    xg = x.detach().cuda().contiguous(memory_format=torch.channels_last)
    y, idx = ops.maxpool2x2_idx(xg, relu=relu)
    assert y.shape == y_ref.shape and torch.equal(y.cpu(), y_ref.detach())
    assert idx.dtype == torch.uint8 and idx.shape == y.shape
    dx = ops.maxpool2x2_idx_backward(dy.cuda(), idx, shape[2], shape[3], relu_mask=relu)
    assert dx.shape == x.shape
    # (relu=True: torch's ReLU passes no gradient at x <= 0; at a window whose maximum is not positive
    # max_pool2d sends the gradient to its first zero, which the ReLU then drops: zeros either way)
    assert torch.equal(dx.cpu(), want_dx)
    # the byte itself: position bits address the maximum, bit 2 says whether it is positive
    if y.numel():
        n, c, h, w = shape
        win = x.detach()[:, :, :h // 2 * 2, :w // 2 * 2].reshape(n, c, h // 2, 2, w // 2, 2).permute(0, 1, 2, 4, 3, 5)
        win = win.reshape(n, c, h // 2, w // 2, 4)
        b = idx.cpu().long()
        picked = torch.gather(win, 4, (b & 3).unsqueeze(-1)).squeeze(-1)
        assert torch.equal(picked, win.max(dim=4).values)
        assert torch.equal((b & 4) != 0, picked > 0) and int((b >> 3).max()) == 0


def test_maxpool_with_index_bytes_propagates_nan_like_torch():
    """A NaN in a window wins (torch's max_pool2d rule) and receives the window's gradient."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(2, 8, 6, 6, generator=g)
    x[0, 1, 2, 3] = float("nan")
    x[1, 5, 5, 5] = float("nan")
    x[1, 5, 4, 4] = float("nan")          # two NaNs in one window: the first in scan order is picked
    xr = x.clone().requires_grad_(True)
    y_ref = F.max_pool2d(xr, 2, 2)
    dy = torch.randn(y_ref.shape, generator=g)
    y_ref.backward(dy)
    y, idx = ops.maxpool2x2_idx(x.cuda().contiguous(memory_format=torch.channels_last))
    assert torch.equal(torch.isnan(y.cpu()), torch.isnan(y_ref.detach()))
    assert torch.equal(torch.nan_to_num(y.cpu(), nan=7.0), torch.nan_to_num(y_ref.detach(), nan=7.0))
    dx = ops.maxpool2x2_idx_backward(dy.cuda(), idx, 6, 6)
    assert torch.equal(dx.cpu(), xr.grad)


@pytest.mark.parametrize("B,C", [(64, 10), (64, 1000), (7, 32320), (1, 3)])
def test_cross_entropy_vs_torch(B, C):
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(B, C, generator=g) * 3).requires_grad_(True)
    t = torch.randint(0, C, (B,), generator=g)
    if B > 2:
        t[1] = -100
    ref = F.cross_entropy(x, t)
    ref.backward(torch.tensor(0.7))
    loss, (lse, count) = ops.cross_entropy_forward(x.detach().cuda(), t.cuda())
    torch.testing.assert_close(loss.cpu(), ref.detach(), rtol=1e-5, atol=1e-6)
    d = ops.cross_entropy_backward(x.detach().cuda(), t.cuda(), lse, count, torch.tensor(0.7).cuda())
    torch.testing.assert_close(d.cpu(), x.grad, rtol=1e-5, atol=1e-7)
    if B > 2:
        assert not d[1].any()


@pytest.mark.parametrize("bad", [-1, 10, 1 << 40])
def test_cross_entropy_target_out_of_range_gives_nan_loss(bad):
    """A label outside [0, C) that is not the ignore index: the loss is NaN (no read outside the row), the
    other rows' log-sum-exp values and the backward kernel run as usual."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(6, 10, generator=g)
    t = torch.randint(0, 10, (6,), generator=g)
    t[3] = bad
    loss, (lse, count) = ops.cross_entropy_forward(x.cuda(), t.cuda())
    assert torch.isnan(loss).item()
    torch.testing.assert_close(lse.cpu(), torch.logsumexp(x, dim=1), rtol=1e-5, atol=1e-6)
    d = ops.cross_entropy_backward(x.cuda(), t.cuda(), lse, count, torch.tensor(1.0).cuda())
    torch.cuda.synchronize()
    # rows with valid labels get their usual gradient; the bad row gets softmax / count (no one-hot entry)
    keep = [i for i in range(6) if i != 3]
    xr = x[keep].clone().requires_grad_(True)
    (F.cross_entropy(xr, t[keep], reduction="sum") / 6).backward()
    torch.testing.assert_close(d.cpu()[keep], xr.grad, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(d.cpu()[3], torch.softmax(x[3], 0) / 6, rtol=1e-5, atol=1e-7)


def test_linear_layer_matches_torch_nn():
    torch.manual_seed(3)
    ref = torch.nn.Linear(37, 21)
    mine = layers.Linear(37, 21, relu=True)
    mine.load_state_dict(ref.state_dict())
    mine = mine.cuda()
    x = torch.randn(4, 9, 37, requires_grad=True)
    xg = x.detach().cuda().requires_grad_(True)
    y_ref = torch.relu(ref(x))
    y = mine(xg)
    torch.testing.assert_close(y.cpu(), y_ref.detach(), rtol=1e-5, atol=1e-5)
    dy = torch.randn(y_ref.shape)
    y_ref.backward(dy)
    y.backward(dy.cuda())
    torch.testing.assert_close(xg.grad.cpu(), x.grad, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(mine.weight.grad.cpu(), ref.weight.grad, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(mine.bias.grad.cpu(), ref.bias.grad, rtol=1e-5, atol=1e-5)
    assert list(mine.state_dict().keys()) == list(ref.state_dict().keys())


@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False), (True, True)])
def test_gemm_many_tiles_and_deep_split(ta, tb):
    """6400 x 4096 (1600 tiles of 128 x 128) and 2048 x 2048 with a reduction of 4096 (256 tiles: split three ways
    so that three blocks share each CU).  Against torch's product of the same operands in fp64."""
    from pipedream_amd import ops
    g = torch.Generator().manual_seed(7)
    for (M, N, K) in ((6400, 4096, 64), (2048, 2048, 4096)):
        a = torch.randn((K, M) if ta else (M, K), generator=g).cuda()
        b = torch.randn((N, K) if tb else (K, N), generator=g).cuda()
        bias = torch.randn(N, generator=g).cuda()
        got = ops.gemm(a, b, trans_a=ta, trans_b=tb, bias=bias)
        want = (a.double().t() if ta else a.double()) @ (b.double().t() if tb else b.double()) + bias.double()
        err = float((got.double() - want).norm() / want.norm())
        assert err < 1e-6, (M, N, K, err)
        torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5 * (K ** 0.5))
    assert ops.splitk_factor(2048, 2048, 4096) == 3 and ops.splitk_factor(4096, 1024, 6400, True) == 3
    assert ops.splitk_factor(6400, 4096, 1024) == 1 and ops.splitk_factor(6400, 1024, 4096) == 1


@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K,plan", [(6400, 4096, 1024, (6144, 1, 8)), (6400, 1024, 2560, (6144, 2, 20))])
def test_gemm_tile_rows_left_over_after_whole_rounds_are_split_over_k(ta, tb, M, N, K, plan):
    """6400 x 4096: 1600 tiles = two rounds of 768 blocks + 64; the two tile rows left over run as a k-split of their
    own.  6400 x 1024 with a deep reduction: 400 tiles; the first 48 tile rows, split two ways, are one round of
    768 blocks and the two left over a second, small one.  Bias, ReLU and beta reach both parts; the result equals
    the one-launch product up to the summation order, and torch's fp64 product to 1e-6."""
    from pipedream_amd import ops
    assert ops._row_plan(M, N, K) == plan
    assert ops._row_plan(6144, 4096, 1024) is None and ops._row_plan(2048, 2048, 4096) is None
    assert ops._row_plan(8192, 4096, 1024) is None        # 512 tiles left over: most of a round anyway
    assert ops._row_plan(6400, 1024, 1024) is None        # too shallow to split the upper rows
    g = torch.Generator().manual_seed(11)
    a = torch.randn((K, M) if ta else (M, K), generator=g).cuda()
    b = torch.randn((N, K) if tb else (K, N), generator=g).cuda()
    bias = torch.randn(N, generator=g).cuda()
    prior = torch.randn(M, N, generator=g).cuda()
    want = torch.relu((a.double().t() if ta else a.double()) @ (b.double().t() if tb else b.double()) + bias.double()
                      + 0.5 * prior.double())
    outs = []
    for planned in (True, False):
        ops._ROW_PLAN = planned
        try:
            outs.append(ops.gemm(a, b, trans_a=ta, trans_b=tb, bias=bias, relu=True, out=prior.clone(), beta=0.5))
        finally:
            ops._ROW_PLAN = True
    for got in outs:
        assert float((got.double() - want).norm() / want.norm()) < 1e-6
    rows = plan[0]
    if plan[1] == 1:
        assert torch.equal(outs[0][:rows], outs[1][:rows])
    torch.testing.assert_close(outs[0], outs[1], rtol=1e-5, atol=1e-5 * K ** 0.5)    # sums of K terms of size ~1
    assert not torch.equal(outs[0][rows:], outs[1][rows:])    # the tail did take the other path


@pytest.fixture
def _gemm_algorithm_back_to_auto():
    from pipedream_amd import ops
    yield
    ops.set_gemm_f32_algorithm("auto")


@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False)])
def test_gemm_as_six_bf16_products_is_closer_to_fp64_than_the_fp32_kernel(ta, tb, _gemm_algorithm_back_to_auto):
    """Large fp32 products run on the bf16 matrix pipes: each operand as the exact sum of three bf16 terms, six
    products per term pair, fp32 accumulation.  Against torch's fp64 product the result must be at least as close
    as the fp32 MFMA kernel's (it is about three times closer: fewer roundings of the running sum), with bias and
    beta applied; the default takes that path for this shape and not for a narrow or a small one."""
    from pipedream_amd import ops
    M, N, K = 4096, 3072, 1408
    assert ops._use_split_bf16(M, N, K, ta, tb, False, *(torch.empty(8, 8, device="cuda"),) * 3)
    assert ops._split_bf16_parts(6400, 1024, 4096) == 2 and ops._split_bf16_parts(4096, 1024, 6400) == 4
    assert ops._split_bf16_parts(M, N, K) == 1 and ops._split_bf16_parts(512, 512, 4096) == 6
    assert not ops._use_split_bf16(6400, 1024, 4096, ta, tb, False, *(torch.empty(8, 8, device="cuda"),) * 3)
    assert not ops._use_split_bf16(1024, 1024, 1024, ta, tb, False, *(torch.empty(8, 8, device="cuda"),) * 3)
    assert not ops._use_split_bf16(M, N, K, ta, tb, True, *(torch.empty(8, 8, device="cuda"),) * 3)     # ReLU epilogue
    g = torch.Generator().manual_seed(21)
    a = torch.randn((K, M) if ta else (M, K), generator=g).cuda()
    b = (torch.randn((N, K) if tb else (K, N), generator=g) * 0.05).cuda()
    bias = torch.randn(N, generator=g).cuda()
    prior = torch.randn(M, N, generator=g).cuda()
    want = (a.double().t() if ta else a.double()) @ (b.double().t() if tb else b.double()) + bias.double() + 0.5 * prior.double()
    err = {}
    for mode in ("mfma_f32", "split_bf16", "auto"):
        ops.set_gemm_f32_algorithm(mode)
        out = ops.gemm(a, b, trans_a=ta, trans_b=tb, bias=bias, out=prior.clone(), beta=0.5)
        err[mode] = (float((out.double() - want).norm() / want.norm()), float((out.double() - want).abs().max()), out)
    assert err["split_bf16"][0] <= err["mfma_f32"][0] and err["split_bf16"][1] <= 1.5 * err["mfma_f32"][1], err
    assert err["split_bf16"][0] < 4e-7
    assert torch.equal(err["auto"][2], err["split_bf16"][2])


@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False)])
def test_gemm_as_six_bf16_products_with_few_output_tiles(ta, tb, _gemm_algorithm_back_to_auto):
    """A narrow output (1024 columns: 28 tiles of 256 x 256): the six-fold reduction is cut into ranges that run as
    batch entries, and their partial products are added in index order with bias and beta."""
    from pipedream_amd import ops
    M, N, K = 1792, 1024, 1536
    assert ops._split_bf16_parts(M, N, K) == 6
    g = torch.Generator().manual_seed(22)
    a = torch.randn((K, M) if ta else (M, K), generator=g).cuda()
    b = (torch.randn((N, K) if tb else (K, N), generator=g) * 0.05).cuda()
    bias = torch.randn(N, generator=g).cuda()
    prior = torch.randn(M, N, generator=g).cuda()
    want = (a.double().t() if ta else a.double()) @ (b.double().t() if tb else b.double()) + bias.double() + 0.5 * prior.double()
    err = {}
    for mode in ("mfma_f32", "split_bf16"):
        ops.set_gemm_f32_algorithm(mode)
        out = ops.gemm(a, b, trans_a=ta, trans_b=tb, bias=bias, out=prior.clone(), beta=0.5)
        err[mode] = float((out.double() - want).norm() / want.norm())
    assert err["split_bf16"] <= err["mfma_f32"] and err["split_bf16"] < 4e-7, err


def test_three_way_bf16_split_is_exact_and_keeps_special_values():
    """pd_split3_bf16_f32: the three terms add up to the fp32 value exactly (normal numbers), slot order per side,
    both placements; infinities and NaNs stay in the first term, a value that bf16 would round to infinity does not."""
    from pipedream_amd import _cabi, ops
    g = torch.Generator().manual_seed(3)
    x = torch.randn(64, 128, generator=g) * torch.exp2(torch.randint(-60, 60, (64, 128), generator=g).float())
    x[0, :8] = torch.tensor([float("inf"), float("-inf"), float("nan"), 3.4e38, -3.4e38, 0.0, -0.0, 1.0])
    x = x.cuda()
    lib = _cabi.lib()
    for b_side, slots in ((0, (0, 2, 1, 1, 0, 0)), (1, (2, 0, 0, 1, 1, 0))):
        flat = torch.empty(64, 6 * 128, dtype=torch.bfloat16, device="cuda")
        tall = torch.empty(6 * 64, 128, dtype=torch.bfloat16, device="cuda")
        lib.pd_split3_bf16_f32(ops._ptr(x), 64, 128, 128, ops._ptr(flat), b_side, 0, _cabi.stream_ptr())
        lib.pd_split3_bf16_f32(ops._ptr(x), 64, 128, 128, ops._ptr(tall), b_side, 1, _cabi.stream_ptr())
        parts = [flat[:, s * 128:(s + 1) * 128] for s in range(6)]
        bits = lambda t: t.contiguous().view(torch.int16)      # (NaN is not equal to itself)
        for s in range(6):
            assert torch.equal(bits(parts[s]), bits(tall[s * 64:(s + 1) * 64]))
            assert torch.equal(bits(parts[s]), bits(parts[slots.index(slots[s])]))       # equal terms are equal slots
        t = [parts[slots.index(i)].float() for i in range(3)]
        total = (t[0].double() + t[1].double() + t[2].double()).float()
        ok = torch.isfinite(x)
        assert torch.equal(total[ok], x[ok])
        assert torch.isinf(t[0][0, 0]) and torch.isinf(t[0][0, 1]) and torch.isnan(t[0][0, 2])
        assert float(t[1][0, :3].abs().sum()) == 0.0 and float(t[2][0, :3].abs().sum()) == 0.0
        assert torch.isfinite(t[0][0, 3]) and torch.isfinite(t[0][0, 4])
