"""3x3 convolution kernels (forward, input gradient, weight/bias gradient) through the C
ABI against the torch CPU library (the third-party routine the reference's Conv2d layers
call) in fp64, plus a brute-force direct convolution on a tiny case that pins the index
conventions (tap order, padding, which operand is flipped).

Every test runs under both convolution algorithms: "direct" and "winograd" (F(2x2, 3x3), taken
where its shape conditions hold, the direct kernel elsewhere).  The Winograd kernel is pinned by the
same library results at the same tolerance, by the brute-force case below through a filter that is
not symmetric under any flip, and by an impulse response that must reproduce each filter tap.

Tolerance: fp32 accumulation over R terms against an fp64 result: rtol 1e-5 plus
atol = 4e-7 * sqrt(R) * (typical |term| sum scale) as set per test."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from pipedream_amd import layers, ops

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["direct", "winograd"])
def conv_algorithm(request):
    ops.set_conv_algorithm(request.param)
    yield request.param
    ops.set_conv_algorithm("auto")


def _nhwc(t):
    return t.cuda().contiguous(memory_format=torch.channels_last)


@pytest.fixture(autouse=True)
def _pieces_back_to_auto():
    yield
    ops.set_conv_pieces("auto")


def request_pieces(mode):
    """Work items made of pieces (stacked batches of width 8 k or 4 k) are chosen by item count, which tiny test
    shapes never reach: force them, or rule them out (the fixture above restores the built-in choice)."""
    ops.set_conv_pieces(mode)


def _direct_conv(x, w, b):
    """Brute-force NCHW 3x3 / pad 1 convolution in numpy float64."""
    N, C, H, W = x.shape
    K = w.shape[0]
    xp = np.zeros((N, C, H + 2, W + 2))
    xp[:, :, 1:-1, 1:-1] = x
    y = np.zeros((N, K, H, W))
    for n in range(N):
        for k in range(K):
            for yy in range(H):
                for xx in range(W):
                    y[n, k, yy, xx] = (xp[n, :, yy:yy + 3, xx:xx + 3] * w[k]).sum() + b[k]
    return y


def test_forward_against_brute_force():
    rng = np.random.RandomState(0)
    x = rng.randn(2, 3, 5, 7)
    w = rng.randn(4, 3, 3, 3)
    b = rng.randn(4)
    want = _direct_conv(x, w, b)
    got = ops.conv3x3_forward(_nhwc(torch.tensor(x, dtype=torch.float32)),
                              _nhwc(torch.tensor(w, dtype=torch.float32)),
                              torch.tensor(b, dtype=torch.float32).cuda())
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-5)
    # the torch library agrees with the brute force, so it can serve as the oracle below
    lib = F.conv2d(torch.tensor(x), torch.tensor(w), torch.tensor(b), padding=1)
    np.testing.assert_allclose(lib.numpy(), want, rtol=1e-10, atol=1e-10)


SHAPES = [
    # N, C, K, H, W
    (2, 3, 64, 32, 32),      # first VGG layer: 3 input channels
    (2, 64, 64, 32, 48),
    (1, 64, 128, 28, 28),    # ragged tiles
    (2, 128, 128, 14, 14),
    (1, 16, 32, 9, 5),       # fewer channels than a block, odd sizes
    (1, 8, 8, 1, 1),
    (1, 20, 70, 17, 33),     # channel counts that are not multiples of the tile
    (3, 5, 6, 8, 8),         # C not a multiple of 4: scalar load path
    (1, 64, 64, 7, 19),      # odd height and width: half tiles at the image edges (Winograd strips)
    (3, 128, 64, 9, 40),
    (2, 3, 64, 17, 19),      # 3 channels, ragged tiles on both edges
    (1, 3, 40, 9, 70),       # 3 channels, wide-tile shape, fewer filters than a block
    (2, 3, 100, 40, 7),      # 3 channels, tall-tile shape, two filter blocks (the second ragged)
    (1, 2, 8, 5, 40),        # 2 and 1 channels: the dense-tap kernel with run-time channel count
    (2, 1, 16, 33, 9),
]


@pytest.mark.parametrize("N,C,K,H,W", SHAPES)
def test_forward_backward_vs_library(N, C, K, H, W):
    g = torch.Generator().manual_seed(N * 1000 + C)
    x = torch.randn(N, C, H, W, generator=g)
    w = torch.randn(K, C, 3, 3, generator=g) / math.sqrt(9 * C)
    b = torch.randn(K, generator=g)
    dy = torch.randn(N, K, H, W, generator=g)
    xd, wd, bd = x.double().requires_grad_(), w.double().requires_grad_(), b.double().requires_grad_()
    y_ref = F.conv2d(xd, wd, bd, padding=1)
    y_ref.backward(dy.double())

    xg, wg = _nhwc(x), _nhwc(w)
    y = ops.conv3x3_forward(xg, wg, b.cuda())
    assert y.is_contiguous(memory_format=torch.channels_last)
    torch.testing.assert_close(y.cpu().double(), y_ref.detach(), rtol=1e-5, atol=4e-7 * math.sqrt(9 * C) * 4)
    dx = ops.conv3x3_input_grad(_nhwc(dy), wg)
    torch.testing.assert_close(dx.cpu().double(), xd.grad, rtol=1e-5, atol=4e-7 * math.sqrt(9 * K) * 4)
    dw, db = ops.conv3x3_weight_grad(xg, _nhwc(dy))
    R = N * H * W
    torch.testing.assert_close(dw.cpu().double(), wd.grad, rtol=1e-5, atol=4e-7 * math.sqrt(R) * 4)
    torch.testing.assert_close(db.cpu().double(), bd.grad, rtol=1e-5, atol=4e-7 * math.sqrt(R) * 4)


def _random_shapes(count, seed):
    rng = np.random.RandomState(seed)
    shapes = []
    for _ in range(count):
        c = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 24, 40, 64, 72, 128]))
        k = int(rng.choice([1, 4, 6, 8, 20, 32, 36, 64, 100, 128]))
        shapes.append((int(rng.randint(1, 4)), c, k, int(rng.randint(1, 41)), int(rng.randint(1, 41))))
    return shapes


@pytest.mark.parametrize("N,C,K,H,W", _random_shapes(24, seed=20))
def test_layer_on_random_shapes_vs_library(N, C, K, H, W):
    """Seeded sweep over channel counts and image sizes on both sides of every kernel's dispatch conditions
    (few-channel, vector / scalar loads, Winograd and its ragged tiles, partial filter blocks): the layer
    with fused ReLU, and with the pooling in its epilogue where a window fits, against torch in fp64 --
    output, input gradient, weight and bias gradients."""
    g = torch.Generator().manual_seed(N + 10 * C + 1000 * K + H * W)
    x = torch.randn(N, C, H, W, generator=g)
    # (the pooling kernels take channel counts that are multiples of 4)
    for pool in ([False, True] if H >= 2 and W >= 2 and K % 4 == 0 else [False]):
        layer = layers.Conv2d(C, K, relu=True, pool=pool)
        w, b = layer.weight.detach().clone(), layer.bias.detach().clone()
        layer = layer.cuda()
        xd, wd, bd = x.double().requires_grad_(), w.double().requires_grad_(), b.double().requires_grad_()
        y_ref = F.relu(F.conv2d(xd, wd, bd, padding=1))
        if pool:
            y_ref = F.max_pool2d(y_ref, 2, 2)
        dy = torch.randn(y_ref.shape, generator=g)
        # A pre-activation within rounding of 0, or two window elements within rounding of each other, may
        # fall on the other side in fp32 and move a gradient entry to another place: such outputs get no
        # upstream gradient (a handful at most; the values themselves are still compared).
        pre = F.conv2d(xd.detach(), wd.detach(), bd.detach(), padding=1)
        if pool:
            r = F.relu(pre)[:, :, :H // 2 * 2, :W // 2 * 2]
            win = r.reshape(N, K, H // 2, 2, W // 2, 2).permute(0, 1, 2, 4, 3, 5).reshape(N, K, H // 2, W // 2, 4)
            top = win.sort(dim=4, descending=True).values
            pw = pre[:, :, :H // 2 * 2, :W // 2 * 2].reshape(N, K, H // 2, 2, W // 2, 2).permute(0, 1, 2, 4, 3, 5)
            clear = (pw.reshape(N, K, H // 2, W // 2, 4).abs() > 1e-4).all(dim=4)
            safe = clear & ((top[..., 0] == 0) | (top[..., 0] - top[..., 1] > 1e-4))
        else:
            safe = pre.abs() > 1e-4
        dy = dy * safe
        y_ref.backward(dy.double())
        xg = x.cuda().requires_grad_(True)
        y = layer(xg)
        assert y.shape == y_ref.shape
        torch.testing.assert_close(y.detach().cpu().double(), y_ref.detach(), rtol=1e-5,
                                   atol=4e-7 * math.sqrt(9 * C) * 4)
        y.backward(dy.cuda())
        scale = lambda t: float(t.abs().max()) + 1e-30
        torch.testing.assert_close(xg.grad.cpu().double(), xd.grad, rtol=1e-5, atol=2e-5 * scale(xd.grad))
        torch.testing.assert_close(layer.weight.grad.cpu().double(), wd.grad, rtol=1e-5, atol=2e-5 * scale(wd.grad))
        torch.testing.assert_close(layer.bias.grad.cpu().double(), bd.grad, rtol=1e-5, atol=2e-5 * scale(bd.grad))


def test_fused_relu_and_no_bias():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(2, 16, 12, 12, generator=g)
    w = torch.randn(24, 16, 3, 3, generator=g) / 12
    y = ops.conv3x3_forward(_nhwc(x), _nhwc(w), None, relu=True)
    want = F.conv2d(x.double(), w.double(), None, padding=1).clamp_min(0)
    torch.testing.assert_close(y.cpu().double(), want, rtol=1e-5, atol=1e-5)
    dw, db = ops.conv3x3_weight_grad(_nhwc(x), y, with_bias=False)
    assert db is None


def test_fused_relu_mask_in_gradient_kernels():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(2, 24, 20, 28, generator=g)
    w = torch.randn(40, 24, 3, 3, generator=g) / 15
    dy = torch.randn(2, 40, 20, 28, generator=g)
    y = ops.conv3x3_forward(_nhwc(x), _nhwc(w), None, relu=True)
    masked = ops.relu_backward(_nhwc(dy), y)
    dx_ref = ops.conv3x3_input_grad(masked, _nhwc(w))
    dw_ref, db_ref = ops.conv3x3_weight_grad(_nhwc(x), masked)
    dx = ops.conv3x3_input_grad(_nhwc(dy), _nhwc(w), relu_out=y)
    dw, db = ops.conv3x3_weight_grad(_nhwc(x), _nhwc(dy), relu_out=y)
    # same arithmetic on the same masked values: bit-identical
    assert torch.equal(dx, dx_ref) and torch.equal(dw, dw_ref) and torch.equal(db, db_ref)


@pytest.mark.parametrize("C,K,H,W", [(24, 40, 20, 28), (6, 10, 9, 11), (64, 64, 32, 32)])
def test_input_gradient_masked_by_rectified_input(C, K, H, W):
    # x_rectified zeroes dx where the layer's input is zero, as the producing layer's ReLU backward would
    g = torch.Generator().manual_seed(9)
    x = _nhwc(torch.randn(2, C, H, W, generator=g).clamp_min(0))
    w = _nhwc(torch.randn(K, C, 3, 3, generator=g) / 15)
    dy = _nhwc(torch.randn(2, K, H, W, generator=g))
    y = ops.conv3x3_forward(x, w, None, relu=True)
    dx_ref = ops.relu_backward(ops.conv3x3_input_grad(dy, w, relu_out=y), x)
    dx = ops.conv3x3_input_grad(dy, w, relu_out=y, x_rectified=x)
    assert torch.equal(dx, dx_ref)
    assert (dx[x <= 0] == 0).all() and (dx != 0).any()
    with pytest.raises(ValueError):
        ops.conv3x3_input_grad(dy, w, x_rectified=dy if C != K else x[:1])


def test_premasked_layer_chain_matches_unfused_chain():
    # conv+ReLU -> conv+ReLU -> pool, with the ReLU backward moved into the consumers' kernels
    torch.manual_seed(12)
    plain = torch.nn.Sequential(layers.Conv2d(8, 16, relu=True), layers.Conv2d(16, 16, relu=True),
                                layers.MaxPool2d(2, 2)).cuda()
    fused = torch.nn.Sequential(layers.Conv2d(8, 16, relu=True, grad_premasked=True),
                                layers.Conv2d(16, 16, relu=True, grad_premasked=True, input_rectified=True),
                                layers.MaxPool2d(2, 2, relu=True)).cuda()
    fused.load_state_dict(plain.state_dict())
    x = torch.randn(2, 8, 12, 12).cuda()
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ya, yb = plain(xa), fused(xb)
    assert torch.equal(ya, yb)
    dy = torch.randn_like(ya)
    ya.backward(dy)
    yb.backward(dy)
    assert torch.equal(xa.grad, xb.grad)
    for pa, pb in zip(plain.parameters(), fused.parameters()):
        assert torch.equal(pa.grad, pb.grad)


@pytest.mark.parametrize("N,C,K,H,W", [(2, 16, 32, 12, 12),     # one tile per image
                                        (1, 64, 64, 32, 48),     # several tiles, one channel block
                                        (2, 24, 100, 17, 19),    # ragged tiles, odd sizes, K % 64 != 0
                                        (1, 128, 128, 14, 14),   # the last VGG16 block's size
                                        (3, 8, 16, 2, 2),        # a single window
                                        (1, 3, 8, 10, 10)])      # few channels: separate pooling kernel
def test_convolution_with_pooling_in_its_epilogue_equals_the_two_layers(N, C, K, H, W):
    """Conv2d(relu=True, pool=True) against the two layers it replaces, under the same algorithm: the pooled
    output and every gradient bit for bit (the fused epilogue pools the same sums, and both backward passes
    hand the same masked gradient to the same gradient kernels); the module that keeps the pooling's place
    in the layer list passes its input through.  The values themselves are checked against torch in fp64,
    the gradients against the unfused, unflagged layers at the usual tolerance."""
    torch.manual_seed(N + C + K)
    plain = torch.nn.Sequential(layers.Conv2d(C, K, relu=True, grad_premasked=True),
                                layers.MaxPool2d(2, 2, relu=True)).cuda()
    fused = torch.nn.Sequential(layers.Conv2d(C, K, relu=True, pool=True),
                                layers.MaxPool2d(2, 2, relu=True, applied_by_producer=True)).cuda()
    fused.load_state_dict(plain.state_dict())
    x = torch.randn(N, C, H, W).cuda()
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ya, yb = plain(xa), fused(xb)
    assert ya.shape == (N, K, H // 2, W // 2)
    assert torch.equal(ya, yb)
    dy = torch.randn_like(ya)
    ya.backward(dy)
    yb.backward(dy)
    assert torch.equal(xa.grad, xb.grad)
    for pa, pb in zip(plain.parameters(), fused.parameters()):
        assert torch.equal(pa.grad, pb.grad)
    # and against torch (fp64) for the values themselves
    ref = F.max_pool2d(F.relu(F.conv2d(x.cpu().double(), plain[0].weight.detach().cpu().double(),
                                       plain[0].bias.detach().cpu().double(), padding=1)), 2, 2)
    torch.testing.assert_close(yb.detach().cpu().double(), ref, rtol=1e-5, atol=2e-5)
    simple = torch.nn.Sequential(layers.Conv2d(C, K, relu=True), layers.MaxPool2d(2, 2)).cuda()
    simple.load_state_dict(plain.state_dict())
    xc = x.clone().requires_grad_(True)
    simple(xc).backward(dy)
    scale = float(xc.grad.abs().max())
    torch.testing.assert_close(xb.grad, xc.grad, rtol=1e-5, atol=1e-5 * scale)
    for pc, pb in zip(simple.parameters(), fused.parameters()):
        torch.testing.assert_close(pb.grad, pc.grad, rtol=1e-5, atol=1e-5 * float(pc.grad.abs().max()))


def _wgrad_shapes(count, seed):
    rng = np.random.RandomState(seed)
    shapes = [(4, 64, 64, 97, 131),      # several strips per block, images change inside a block's range
              (1, 64, 64, 1, 1), (2, 128, 64, 1, 37), (3, 64, 128, 29, 1), (1, 256, 64, 5, 16)]
    for _ in range(count):
        shapes.append((int(rng.randint(1, 6)), int(rng.choice([64, 128])), int(rng.choice([64, 128, 256])),
                       int(rng.randint(1, 51)), int(rng.randint(1, 51))))
    return shapes


@pytest.mark.parametrize("N,C,K,H,W", _wgrad_shapes(10, seed=7))
def test_winograd_weight_gradient_on_ragged_images(N, C, K, H, W, conv_algorithm):
    """The Winograd weight-gradient kernel alone (channel counts it takes, no ReLU mask) on image sizes that
    leave half strips at the right and bottom edges, single rows and columns, and strip ranges that cross
    from one image into the next: weight and bias gradients against torch in fp64."""
    if conv_algorithm != "winograd":
        pytest.skip("covers the Winograd kernel")
    g = torch.Generator().manual_seed(H * 100 + W)
    x = torch.randn(N, C, H, W, generator=g)
    dy = torch.randn(N, K, H, W, generator=g)
    wd = torch.zeros(K, C, 3, 3, dtype=torch.float64, requires_grad=True)
    bd = torch.zeros(K, dtype=torch.float64, requires_grad=True)
    F.conv2d(x.double(), wd, bd, padding=1).backward(dy.double())
    dw, db = ops.conv3x3_weight_grad(_nhwc(x), _nhwc(dy))
    R = N * H * W
    torch.testing.assert_close(dw.cpu().double(), wd.grad, rtol=1e-5, atol=4e-7 * math.sqrt(R) * 4)
    torch.testing.assert_close(db.cpu().double(), bd.grad, rtol=1e-5, atol=4e-7 * math.sqrt(R) * 4)


@pytest.fixture
def _wgrad_strips_back_to_auto():
    yield
    ops.set_conv_wgrad_strips("auto")


@pytest.mark.parametrize("N,C,K,H,W", [(3, 64, 64, 14, 14), (5, 64, 128, 14, 6), (2, 128, 64, 28, 28), (1, 64, 64, 56, 56),
                                       (3, 64, 64, 18, 22), (2, 64, 64, 16, 32), (7, 64, 64, 14, 2), (1, 64, 256, 30, 46)])
def test_winograd_weight_gradient_upright_strips(N, C, K, H, W, conv_algorithm, _wgrad_strips_back_to_auto):
    """Strips of eight tiles on top of each other over the batch taken as one image of N * H rows: strips that
    straddle two or three images (H = 14: every strip), a last strip row that is partly empty (N * H no multiple of
    16), widths of one to 28 tile columns.  Weight and bias gradients against torch in fp64, and against the
    flat strips of 2 x 16 pixels, from which they differ by the summation order only."""
    if conv_algorithm != "winograd":
        pytest.skip("covers the Winograd kernel")
    g = torch.Generator().manual_seed(H * 100 + W)
    x = torch.randn(N, C, H, W, generator=g)
    dy = torch.randn(N, K, H, W, generator=g)
    wd = torch.zeros(K, C, 3, 3, dtype=torch.float64, requires_grad=True)
    bd = torch.zeros(K, dtype=torch.float64, requires_grad=True)
    F.conv2d(x.double(), wd, bd, padding=1).backward(dy.double())
    R = N * H * W
    got = {}
    for mode in ("upright", "flat"):
        ops.set_conv_wgrad_strips(mode)
        dw, db = ops.conv3x3_weight_grad(_nhwc(x), _nhwc(dy))
        torch.testing.assert_close(dw.cpu().double(), wd.grad, rtol=1e-5, atol=4e-7 * math.sqrt(R) * 4)
        torch.testing.assert_close(db.cpu().double(), bd.grad, rtol=1e-5, atol=4e-7 * math.sqrt(R) * 4)
        got[mode] = dw
    assert not torch.equal(got["upright"], got["flat"])       # the other kernel did run
    # an image whose values are confined to its first and last rows: what a neighbour's rows would add shows up here
    x2 = torch.zeros(N, C, H, W)
    x2[:, :, 0] = torch.randn(N, C, W, generator=g)
    x2[:, :, H - 1] = torch.randn(N, C, W, generator=g)
    wd.grad = None
    bd.grad = None
    F.conv2d(x2.double(), wd, bd, padding=1).backward(dy.double())
    ops.set_conv_wgrad_strips("upright")
    dw, _ = ops.conv3x3_weight_grad(_nhwc(x2), _nhwc(dy))
    torch.testing.assert_close(dw.cpu().double(), wd.grad, rtol=1e-5, atol=4e-7 * math.sqrt(R) * 4)


def test_winograd_impulse_response_and_brute_force():
    # the Winograd path on shapes it accepts: (a) brute-force direct convolution of a small case with
    # random (asymmetric) filters; (b) a unit impulse must return the flipped filter taps around it
    ops.set_conv_algorithm("winograd")
    rng = np.random.RandomState(1)
    x = rng.randn(1, 8, 6, 7)
    w = rng.randn(4, 8, 3, 3)
    b = rng.randn(4)
    got = ops.conv3x3_forward(_nhwc(torch.tensor(x, dtype=torch.float32)), _nhwc(torch.tensor(w, dtype=torch.float32)),
                              torch.tensor(b, dtype=torch.float32).cuda())
    np.testing.assert_allclose(got.cpu().numpy(), _direct_conv(x, w, b), rtol=1e-5, atol=2e-5)
    x = torch.zeros(1, 16, 20, 37)
    x[0, 5, 9, 30] = 1.0
    w = torch.randn(32, 16, 3, 3)
    y = ops.conv3x3_forward(_nhwc(x), _nhwc(w)).cpu()
    for r in range(3):
        for s_ in range(3):
            # y[k, 9 - (r-1), 30 - (s-1)] = w[k, 5, r, s]
            torch.testing.assert_close(y[0, :, 10 - r, 31 - s_], w[:, 5, r, s_], rtol=1e-5, atol=1e-5)
    y[0, :, 8:11, 29:32] = 0
    assert y.abs().max() < 1e-5
    # input gradient = correlation with the unflipped taps
    dy = torch.zeros(1, 32, 20, 37)
    dy[0, 7, 0, 36] = 1.0                        # a corner: padding on two sides
    dx = ops.conv3x3_input_grad(_nhwc(dy), _nhwc(w)).cpu()
    torch.testing.assert_close(dx[0, :, 0, 36], w[7, :, 1, 1], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(dx[0, :, 1, 35], w[7, :, 2, 0], rtol=1e-5, atol=1e-5)


def test_identity_filter_is_exact(conv_algorithm):
    if conv_algorithm != "direct":
        pytest.skip("bit-exact pass-through is a property of the direct kernel only")
    # a centre-tap identity filter must reproduce the input bit for bit
    x = torch.randn(2, 32, 20, 20)
    w = torch.zeros(32, 32, 3, 3)
    for c in range(32):
        w[c, c, 1, 1] = 1.0
    y = ops.conv3x3_forward(_nhwc(x), _nhwc(w))
    assert torch.equal(y.cpu(), x)
    # shifting filter: tap (r=0,s=2) reads x[y-1, x+1]
    w = torch.zeros(32, 32, 3, 3)
    for c in range(32):
        w[c, c, 0, 2] = 1.0
    y = ops.conv3x3_forward(_nhwc(x), _nhwc(w)).cpu()
    want = torch.zeros_like(x)
    want[:, :, 1:, :-1] = x[:, :, :-1, 1:]
    assert torch.equal(y, want)


def test_conv_layer_module_matches_torch_nn():
    torch.manual_seed(11)
    ref = torch.nn.Conv2d(8, 16, 3, padding=1)
    mine = layers.Conv2d(8, 16, relu=True)
    mine.load_state_dict(ref.state_dict())
    assert mine.weight.is_contiguous(memory_format=torch.channels_last)
    mine = mine.cuda()
    x = torch.randn(2, 8, 10, 10, requires_grad=True)
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


def test_conv_rejects_bad_operands():
    x = torch.randn(1, 4, 6, 6).cuda()           # NCHW memory order
    w = _nhwc(torch.randn(8, 4, 3, 3))
    with pytest.raises(ValueError, match="NHWC"):
        ops.conv3x3_forward(x, w)
    with pytest.raises(ValueError, match="channels"):
        ops.conv3x3_forward(_nhwc(torch.randn(1, 5, 6, 6)), w)
    with pytest.raises(NotImplementedError):
        layers.Conv2d(4, 8, kernel_size=5, padding=2)


@pytest.mark.parametrize("C,K", [(8, 4), (24, 36), (32, 64), (64, 100), (128, 128)])
@pytest.mark.parametrize("rot180", [0, 1])
@pytest.mark.parametrize("offset", [0, 1])
def test_transformed_filter_layout_and_values(C, K, rot180, offset, conv_algorithm):
    # U = G g G^T in fp64, placed by the documented order [k/64][c/8][g][(k%64)/32][(c%8)/4][k%32][c%4];
    # rows k >= K of the last block of 64 must be zero.  offset 1: a filter that is only 4-byte aligned.
    if conv_algorithm != "winograd":
        pytest.skip("one algorithm is enough: the transform does not depend on it")
    import ctypes

    from pipedream_amd import _cabi
    lib = _cabi.lib()
    rng = np.random.RandomState(C * 1000 + K * 2 + rot180)
    # memory order of the operand: [K][3][3][C], or with rot180 [C][3][3][K]
    mem = rng.randn(*((C, 3, 3, K) if rot180 else (K, 3, 3, C)))
    flat = torch.zeros(mem.size + 4, dtype=torch.float32).cuda()
    wdev = flat[offset:offset + mem.size]
    wdev.copy_(torch.tensor(mem.reshape(-1), dtype=torch.float32))
    nbytes = ctypes.c_uint64()
    lib.pd_conv3x3_winograd_filter_bytes(C, K, ctypes.byref(nbytes))
    u = torch.full((nbytes.value // 4,), float("nan"), dtype=torch.float32).cuda()
    lib.pd_conv3x3_winograd_filter_f32(wdev.data_ptr(), u.data_ptr(), C, K, rot180, _cabi.stream_ptr())
    torch.cuda.synchronize()
    mem32 = wdev.cpu().numpy().astype(np.float64).reshape(mem.shape)
    # f[k][r][s][c]
    f = mem32[:, ::-1, ::-1, :].transpose(3, 1, 2, 0) if rot180 else mem32
    G = np.array([[1, 0, 0], [.5, .5, .5], [.5, -.5, .5], [0, 0, 1]])
    U = np.einsum("ir,krsc,js->kcij", G, f, G).reshape(K, C, 16)
    k_pad = (K + 63) // 64 * 64
    want = np.zeros((k_pad // 64, C // 8, 16, 2, 2, 32, 4))
    for k in range(K):
        for c in range(C):
            want[k // 64, c // 8, :, (k % 64) // 32, (c % 8) // 4, k % 32, c % 4] = U[k, c]
    assert u.numel() == want.size
    np.testing.assert_allclose(u.cpu().numpy().reshape(want.shape), want, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("N,C,K,H,W", [(4, 8, 64, 6, 10),      # one reduction chunk: a new work item every step
                                        (3, 16, 32, 14, 14),    # the last VGG16 block's images
                                        (5, 24, 40, 22, 18),    # ragged in both directions, K % 64 != 0
                                        (3, 32, 64, 28, 28),
                                        (7, 8, 8, 2, 34),       # images of one tile row
                                        (2, 16, 16, 56, 24),
                                        # widths of 8 k (4 k) pixels: work items of two (four) pieces
                                        (2, 16, 64, 56, 56),
                                        (3, 8, 128, 28, 12),    # two blocks of output channels
                                        (2, 8, 16, 8, 40),      # five pieces per 16 rows: items straddle them
                                        (5, 8, 8, 6, 4),        # one piece per 16 rows
                                        (3, 16, 32, 10, 72)])
@pytest.mark.parametrize("pieces", ["never", "always"])
def test_batch_of_images_whose_height_is_no_multiple_of_the_tile(N, C, K, H, W, pieces, conv_algorithm):
    """Images of even height that is no multiple of 16 rows are processed as one tall image (work items
    straddle images).  Nothing may leak across an image boundary: every image of the batch must come out
    bit for bit as when it is convolved alone (a batch of one never takes that path), in the forward
    pass, the pooled forward pass and the input gradient (plain and with the rectified-input mask).  The
    batch is also checked against torch in fp64."""
    if conv_algorithm != "winograd":
        pytest.skip("a property of the Winograd kernels' work items")
    if pieces == "always" and not (W % 16 != 0 and W % 4 == 0 and H % 16 != 0):
        pytest.skip("this width has no work items made of pieces")
    request_pieces(pieces)
    torch.manual_seed(N * 100 + H)
    x = _nhwc(torch.randn(N, C, H, W))
    w = _nhwc(torch.randn(K, C, 3, 3) / math.sqrt(9 * C))
    b = torch.randn(K).cuda()
    dy = _nhwc(torch.randn(N, K, H, W))

    def one(t, n):
        return t[n:n + 1].contiguous(memory_format=torch.channels_last)

    y = ops.conv3x3_forward(x, w, b, relu=True)
    yp, idx = ops.conv3x3_forward_pool(x, w, b, relu=True)
    dx = ops.conv3x3_input_grad(dy, w)
    dxm = ops.conv3x3_input_grad(dy, w, x_rectified=x)
    for n in range(N):
        assert torch.equal(y[n], ops.conv3x3_forward(one(x, n), w, b, relu=True)[0]), n
        yp1, idx1 = ops.conv3x3_forward_pool(one(x, n), w, b, relu=True)
        assert torch.equal(yp[n], yp1[0]) and torch.equal(idx[n], idx1[0]), n
        assert torch.equal(dx[n], ops.conv3x3_input_grad(one(dy, n), w)[0]), n
        assert torch.equal(dxm[n], ops.conv3x3_input_grad(one(dy, n), w, x_rectified=one(x, n))[0]), n
    xd = x.cpu().double().requires_grad_(True)
    ref = F.conv2d(xd, w.cpu().double(), b.cpu().double(), padding=1)
    torch.testing.assert_close(y.cpu().double(), F.relu(ref).detach(), rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(yp.cpu().double(), F.max_pool2d(F.relu(ref), 2, 2).detach(), rtol=1e-5, atol=2e-5)
    ref.backward(dy.cpu().double())
    torch.testing.assert_close(dx.cpu().double(), xd.grad, rtol=1e-5, atol=2e-5)


@pytest.mark.parametrize("N,C,K,H,W", [(2, 16, 32, 16, 16),     # pooled 8 x 8: one tile
                                        (3, 64, 64, 28, 28),     # pooled 14 x 14: stacked batch
                                        (1, 32, 64, 40, 72),     # several tiles, ragged
                                        (2, 8, 24, 12, 20),
                                        (2, 16, 32, 56, 56),     # pooled 28 x 28: work items of four pieces
                                        (2, 8, 32, 112, 112),    # pooled 56 x 56: work items of two pieces
                                        (3, 8, 8, 12, 48)])
@pytest.mark.parametrize("producer", ["conv_pool", "maxpool"])
@pytest.mark.parametrize("pieces", ["never", "always"])
def test_pooling_backward_in_the_consuming_convolution_kernel(N, C, K, H, W, producer, pieces, conv_algorithm):
    """ReLU + MaxPool2d followed by a convolution, with and without a PoolGradLink between them: the linked pair
    lets the convolution's input-gradient kernel write the gradient in front of the pooling; every output
    and every gradient must equal the unlinked pair's bit for bit (the same values reach the same kernels),
    and the pooling backward kernel must not run in the linked pair."""
    if conv_algorithm != "winograd":
        pytest.skip("the fused epilogue belongs to the Winograd kernel")
    if pieces == "always" and not ((W // 2) % 16 != 0 and (W // 2) % 4 == 0 and N > 1 and (H // 2) % 16 != 0):
        pytest.skip("the pooled width has no work items made of pieces")
    request_pieces(pieces)
    torch.manual_seed(N + C + H)

    def build(linked):
        link = layers.PoolGradLink() if linked else None
        if producer == "conv_pool":
            first = [layers.Conv2d(C, C, relu=True, pool=True, output_link=link),
                     layers.MaxPool2d(2, 2, relu=True, applied_by_producer=True)]
        else:
            first = [layers.Conv2d(C, C, relu=True, grad_premasked=True), layers.MaxPool2d(2, 2, relu=True, link=link)]
        # (the consumer reads no mask of its own: in the stages it is followed by a layer that masks its gradient)
        return torch.nn.Sequential(*first, layers.Conv2d(C, K, input_link=link)).cuda()

    plain, linked = build(False), build(True)
    linked.load_state_dict(plain.state_dict())
    x = torch.randn(N, C, H, W).cuda()
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ya, yb = plain(xa), linked(xb)
    assert torch.equal(ya, yb)
    dy = torch.randn_like(ya)
    ya.backward(dy)
    ops.kernel_timer = {}                      # records the name of every timed launch
    try:
        yb.backward(dy)
        torch.cuda.synchronize()
        ran = set(ops.kernel_timer)
    finally:
        ops.kernel_timer = None
    assert "maxpool2x2_bwd_idx" not in ran and "conv3x3_winograd_kernel" in ran, ran
    assert torch.equal(xa.grad, xb.grad)
    for pa, pb in zip(plain.parameters(), linked.parameters()):
        assert torch.equal(pa.grad, pb.grad)
    # and the values: torch in fp64
    ref = torch.nn.Sequential(torch.nn.Conv2d(C, C, 3, padding=1), torch.nn.ReLU(), torch.nn.MaxPool2d(2, 2),
                              torch.nn.Conv2d(C, K, 3, padding=1)).double()
    ref[0].weight.data.copy_(plain[0].weight.detach().cpu())
    ref[0].bias.data.copy_(plain[0].bias.detach().cpu())
    ref[3].weight.data.copy_(plain[2].weight.detach().cpu())
    ref[3].bias.data.copy_(plain[2].bias.detach().cpu())
    xr = x.cpu().double().requires_grad_(True)
    ref(xr).backward(dy.cpu().double())
    scale = float(xr.grad.abs().max())
    torch.testing.assert_close(xb.grad.cpu().double(), xr.grad, rtol=1e-5, atol=2e-5 * max(scale, 1.0))


def _even_shapes(count, seed):
    rng = np.random.RandomState(seed)
    out = []
    for _ in range(count):
        # (the gradient kernel reduces over K: a multiple of 8; it writes C channels: a multiple of 4)
        out.append((int(rng.randint(1, 6)), int(rng.choice([8, 12, 24, 40, 64])), int(rng.choice([8, 16, 32, 64, 72])),
                    2 * int(rng.randint(1, 24)), 2 * int(rng.randint(1, 24))))
    return out


@pytest.mark.parametrize("N,C,K,H,W", _even_shapes(16, seed=31))
def test_fused_input_gradient_and_unpooling_on_random_shapes(N, C, K, H, W, conv_algorithm):
    """``conv3x3_input_grad_unpool`` (input gradient of a C -> K convolution on H x W images + backward of the
    ReLU / 2x2 pooling that produced its input) against the two kernels it replaces, bit for bit, on random even
    sizes: batches stacked into one tall image or not, ragged tiles, channel counts off the block sizes."""
    if conv_algorithm != "winograd":
        pytest.skip("the fused epilogue belongs to the Winograd kernel")
    torch.manual_seed(N * 1000 + H * 10 + W)
    full = _nhwc(torch.randn(N, C, 2 * H, 2 * W))
    pooled, idx = ops.maxpool2x2_idx(full, relu=True)
    w = _nhwc(torch.randn(K, C, 3, 3) / math.sqrt(9 * C))
    dy = _nhwc(torch.randn(N, K, H, W))
    assert ops.conv3x3_input_grad_unpool_supported(dy, w)
    dx, dfull = ops.conv3x3_input_grad_unpool(dy, w, idx)
    want_dx = ops.conv3x3_input_grad(dy, w, x_rectified=pooled)
    assert torch.equal(dx, want_dx)
    assert torch.equal(dfull, ops.maxpool2x2_idx_backward(want_dx, idx, 2 * H, 2 * W, relu_mask=True))


def test_pieces_equal_squares_at_vgg_size(conv_algorithm):
    """64 images of 56 x 56 pixels, 128 -> 256 channels (conv3_1 of VGG16), and 28 x 28, 256 -> 512 (conv4_1): the
    forward pass, the pooled forward pass and the input gradient (plain, and with the pooling backward in its
    epilogue) with work items of two / four pieces are bit-identical to the 16 x 16 squares, and the built-in
    choice gives those bits too."""
    if conv_algorithm != "winograd":
        pytest.skip("a property of the Winograd kernels' work items")
    for (C, K, HW) in ((128, 256, 56), (256, 512, 28)):
        gen = torch.Generator(device="cuda").manual_seed(HW)
        x = torch.randn(64, C, HW, HW, device="cuda", generator=gen).contiguous(memory_format=torch.channels_last)
        w = (torch.randn(K, C, 3, 3, device="cuda", generator=gen) / math.sqrt(9 * C)).contiguous(
            memory_format=torch.channels_last)
        b = torch.randn(K, device="cuda", generator=gen)
        dy = torch.randn(64, K, HW, HW, device="cuda", generator=gen).contiguous(memory_format=torch.channels_last)
        idx = torch.randint(0, 8, (64, C, HW, HW), device="cuda", generator=gen, dtype=torch.uint8).contiguous(
            memory_format=torch.channels_last)
        out = {}
        for mode in ("never", "always", "auto"):
            ops.set_conv_pieces(mode)
            out[mode] = (ops.conv3x3_forward(x, w, b, relu=True),) + ops.conv3x3_forward_pool(x, w, b, relu=True) + \
                (ops.conv3x3_input_grad(dy, w),) + ops.conv3x3_input_grad_unpool(dy, w, idx)
        for mode in ("always", "auto"):
            assert all(torch.equal(p, q) for p, q in zip(out["never"], out[mode])), (C, K, HW, mode)
