"""bf16 transformer stage (6 pre-LN layers, fp32 master weights, Adam, 2 double-buffered
weight versions, gradient accumulation over 4 micro-batches) on the HIP kernels against the
CPU oracle (oracle/models.py TransformerStage0: torch's bf16 CPU kernels).

The reference has no such stage on its checked-out branch, so the semantics are the
oracle's ("parity unpinned by the reference").  Tolerance: rel 2e-2 (the north-star's bf16
bar), taken in relative L2 norm per tensor; products with fp32 output are held to 1e-5
against an fp32 product of the same bf16-rounded operands."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import models
from oracle import stash_oracle as so

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _rel(a, b):
    a, b = a.detach().float().cpu().double(), b.detach().float().double()
    return float((a - b).norm() / (b.norm() + 1e-300))


@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K", [(64, 64, 32), (128, 256, 64), (200, 72, 40), (512, 1024, 1024), (8, 8, 8)])
def test_gemm_bf16_layouts(M, N, K, ta, tb):
    from pipedream_amd import ops
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn((K, M) if ta else (M, K), generator=g).to(BF)
    b = torch.randn((N, K) if tb else (K, N), generator=g).to(BF)
    want = (a.float().t() if ta else a.float()) @ (b.float().t() if tb else b.float())
    got32 = ops.gemm_bf16(a.cuda(), b.cuda(), trans_a=ta, trans_b=tb, out_f32=True)
    torch.testing.assert_close(got32.cpu(), want, rtol=1e-5, atol=2e-6 * math.sqrt(K) * 9)
    got16 = ops.gemm_bf16(a.cuda(), b.cuda(), trans_a=ta, trans_b=tb)
    assert torch.equal(got16.cpu(), got32.cpu().to(BF))        # bf16 output = RNE of the fp32 result


def test_gemm_bf16_epilogues():
    from pipedream_amd import ops
    g = torch.Generator().manual_seed(0)
    a = torch.randn(96, 64, generator=g).to(BF)
    b = torch.randn(48, 64, generator=g).to(BF)
    bias = torch.randn(48, generator=g)
    res = torch.randn(96, 48, generator=g).to(BF)
    want = 0.5 * (a.float() @ b.float().t()) + bias + res.float()
    got = ops.gemm_bf16(a.cuda(), b.cuda(), trans_b=True, alpha=0.5, bias=bias.cuda(), residual=res.cuda())
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    acc = torch.ones(96, 48).cuda()
    ops.gemm_bf16(a.cuda(), b.cuda(), trans_b=True, out=acc, beta=1.0)
    torch.testing.assert_close(acc.cpu(), a.float() @ b.float().t() + 1, rtol=1e-5, atol=1e-4)
    with pytest.raises(Exception):
        ops.gemm_bf16(a.cuda()[:, :60], b.cuda()[:, :60], trans_b=True)     # K not a multiple of 8


@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K", [(4096, 4096, 128), (4088, 4104, 256), (4096, 3072, 128), (3992, 3600, 256),
                                   (1000, 1016, 384), (4000, 3592, 224), (3584, 3584, 96)])
@pytest.mark.parametrize("tile", [128, 256])
def test_gemm_bf16_large_tiles(M, N, K, ta, tb, tile):
    """K a multiple of 128 runs the direct-to-LDS ring kernel (one to three ring rounds), here with each of
    its two tile sizes forced in turn (the built-in choice takes 256 x 256 tiles from 192 of them on); other K
    the register-staged kernels; M and N that are not tile multiples exercise the clamped loads and the masked
    vector stores.  The fp32 reference product is computed on the device by torch from the same bf16 inputs."""
    from pipedream_amd import _cabi, ops
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn((K, M) if ta else (M, K), generator=g).to(BF).cuda()
    b = torch.randn((N, K) if tb else (K, N), generator=g).to(BF).cuda()
    want = (a.float().t() if ta else a.float()) @ (b.float().t() if tb else b.float())
    _cabi.lib().pd_gemm_bf16_set_tile(tile, tile)
    try:
        got32 = ops.gemm_bf16(a, b, trans_a=ta, trans_b=tb, out_f32=True)
        got16 = ops.gemm_bf16(a, b, trans_a=ta, trans_b=tb)
    finally:
        _cabi.lib().pd_gemm_bf16_set_tile(0, 0)
    assert _rel(got32, want.cpu()) < 1e-5
    torch.testing.assert_close(got32, want, rtol=1e-4, atol=2e-6 * math.sqrt(K) * 9)
    assert torch.equal(got16, got32.to(BF))


def test_gemm_bf16_built_in_tile_choice_and_hook_errors():
    """Whatever tile the built-in choice takes (256 x 256 from 192 such tiles on, else 128 x 128), it agrees with
    both forced runs bit for bit (the tile size does not change the order of a dot product's additions)."""
    from pipedream_amd import _cabi, ops
    lib = _cabi.lib()
    with pytest.raises(_cabi.PipedreamAmdError):
        lib.pd_gemm_bf16_set_tile(64, 64)
    g = torch.Generator().manual_seed(11)
    for N, K in ((4096, 1024), (1024, 2048)):
        a = (torch.randn(4096, K, generator=g) / 8).to(BF).cuda()
        b = (torch.randn(N, K, generator=g) / 8).to(BF).cuda()
        auto = ops.gemm_bf16(a, b, trans_b=True, out_f32=True)
        for tile in (128, 256):
            lib.pd_gemm_bf16_set_tile(tile, tile)
            try:
                forced = ops.gemm_bf16(a, b, trans_b=True, out_f32=True)
            finally:
                lib.pd_gemm_bf16_set_tile(0, 0)
            assert torch.equal(auto, forced)


def test_gemm_bf16_large_tile_epilogues():
    """bias + residual (single rounding), alpha, and fp32 accumulation (beta = 1) through the
    vectorised LDS-transposed epilogue, and the element-wise fallback when C is not 16-byte
    aligned."""
    from pipedream_amd import ops
    g = torch.Generator().manual_seed(1)
    M, N, K = 4096, 4096, 128
    a = torch.randn(M, K, generator=g).to(BF).cuda()
    b = torch.randn(N, K, generator=g).to(BF).cuda()
    bias = torch.randn(N, generator=g).cuda()
    res = torch.randn(M, N, generator=g).to(BF).cuda()
    prod = a.float() @ b.float().t()
    got = ops.gemm_bf16(a, b, trans_b=True, alpha=0.5, bias=bias, residual=res)
    want = (0.5 * prod + bias + res.float()).to(BF)
    # fp32 summation order inside the product differs from torch's, so a value within rounding of a
    # bf16 tie may round the other way: at most one bf16 ulp, and rarely
    diff = (got.float() - want.float()).abs()
    assert float(diff.max()) <= float(want.float().abs().max()) * 2 ** -7
    assert float((diff > 0).float().mean()) < 1e-3
    acc = torch.ones(M, N).cuda()
    ops.gemm_bf16(a, b, trans_b=True, out=acc, beta=1.0)
    assert _rel(acc, (prod + 1).cpu()) < 1e-5
    # C shifted by one element: 16-byte vector stores are impossible, the element-wise path must agree
    buf = torch.zeros(M * N + 8, dtype=BF).cuda()
    shifted = buf[1:1 + M * N].view(M, N)
    ops.gemm_bf16(a, b, trans_b=True, out=shifted)
    assert torch.equal(shifted, ops.gemm_bf16(a, b, trans_b=True))


@pytest.mark.parametrize("batch,seq,heads", [(2, 128, 3), (1, 256, 2), (2, 512, 4)])
def test_fused_attention_forward(batch, seq, heads):
    """The fused kernel (head dimension 64) against attention evaluated in fp64 from the same bf16
    q, k, v; probabilities and context are bf16, so one bf16 ulp (2^-8 relative) per element plus
    the rounding of P inside the second product bounds the difference."""
    from pipedream_amd import ops
    d, H = 64, 64 * heads
    g = torch.Generator().manual_seed(seq + heads)
    qkv = (torch.randn(batch * seq, 3 * H, generator=g) * 1.5).to(BF)
    ctx, probs = ops.attention_forward(qkv.cuda(), batch, seq, heads, need_probs=True)
    ctx2, lse2 = ops.attention_forward(qkv.cuda(), batch, seq, heads)
    assert torch.equal(ctx, ctx2) and lse2.dtype == torch.float32 and tuple(lse2.shape) == (batch, heads, seq)
    q, k, v = [t.reshape(batch, seq, heads, d).transpose(1, 2).double() for t in qkv.split(H, dim=-1)]
    p = torch.softmax(q @ k.transpose(-1, -2) / math.sqrt(d), dim=-1)
    want = (p @ v).transpose(1, 2).reshape(batch * seq, H)
    assert tuple(probs.shape) == (batch, heads, seq, seq)
    torch.testing.assert_close(probs.float().cpu().double(), p, rtol=2 ** -7, atol=1e-6)
    assert float((probs.float().sum(-1) - 1).abs().max()) < 2e-2
    assert _rel(ctx, want.float()) < 4e-3
    torch.testing.assert_close(ctx.float().cpu().double(), want, rtol=2e-2, atol=2e-2)
    # lse2 = log2 sum_k exp(s_k / sqrt(d)): the probabilities are recomputed from it in the backward pass
    want_lse = torch.logsumexp(q @ k.transpose(-1, -2) / math.sqrt(d), dim=-1) / math.log(2.0)
    torch.testing.assert_close(lse2.cpu().double(), want_lse, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("batch,seq,heads", [(2, 128, 3), (1, 512, 2)])
def test_fused_attention_backward(batch, seq, heads):
    """dqkv of the fused path (query-side and key-side kernels, probabilities recomputed) against autograd
    in fp64 through softmax(q k^T / sqrt(d)) v on the same bf16 inputs, and against the unfused
    HIP path (batched products + softmax backward)."""
    from pipedream_amd import ops
    d, H = 64, 64 * heads
    g = torch.Generator().manual_seed(7 * seq + heads)
    qkv = (torch.randn(batch * seq, 3 * H, generator=g)).to(BF)
    dctx = (torch.randn(batch * seq, H, generator=g) * 0.1).to(BF)
    ref = qkv.double().requires_grad_()
    q, k, v = [t.reshape(batch, seq, heads, d).transpose(1, 2) for t in ref.split(H, dim=-1)]
    out = (torch.softmax(q @ k.transpose(-1, -2) / math.sqrt(d), dim=-1) @ v).transpose(1, 2).reshape(batch * seq, H)
    out.backward(dctx.double())
    ctx, lse2 = ops.attention_forward(qkv.cuda(), batch, seq, heads)
    _, probs = ops.attention_forward(qkv.cuda(), batch, seq, heads, need_probs=True)
    fused = ops.attention_backward(dctx.cuda(), qkv.cuda(), lse2, batch, seq, heads, ctx=ctx)
    plain = ops.attention_backward(dctx.cuda(), qkv.cuda(), probs, batch, seq, heads)
    for name, lo in (("dq", 0), ("dk", H), ("dv", 2 * H)):
        want = ref.grad[:, lo:lo + H].float()
        assert _rel(fused[:, lo:lo + H], want) < 2e-2, (name, _rel(fused[:, lo:lo + H], want))
        assert _rel(fused[:, lo:lo + H], plain[:, lo:lo + H].float().cpu()) < 2e-2, name


def test_layernorm_softmax_gelu_vs_torch():
    from pipedream_amd import ops
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(70, 256, generator=g) * 2 + 0.5).to(BF)
    gamma, beta = torch.randn(256, generator=g), torch.randn(256, generator=g)
    dy = torch.randn(70, 256, generator=g).to(BF)
    xf = x.float().requires_grad_()
    gf, bf = gamma.clone().requires_grad_(), beta.clone().requires_grad_()
    ref = F.layer_norm(xf, (256,), gf, bf, 1e-5)
    ref.backward(dy.float())
    y, mean, rstd = ops.layernorm_forward(x.cuda(), gamma.cuda(), beta.cuda(), 1e-5)
    assert _rel(y, ref) < 4e-3
    dx, dg, db = ops.layernorm_backward(dy.cuda(), x.cuda(), gamma.cuda(), mean, rstd)
    assert _rel(dx, xf.grad) < 4e-3 and _rel(dg, gf.grad) < 1e-5 and _rel(db, bf.grad) < 1e-5
    acc_g, acc_b = torch.ones(256).cuda(), torch.ones(256).cuda()
    ops.layernorm_backward(dy.cuda(), x.cuda(), gamma.cuda(), mean, rstd, acc_g, acc_b)
    assert _rel(acc_g, gf.grad + 1) < 1e-5 and _rel(acc_b, bf.grad + 1) < 1e-5
    # with the residual branch of a pre-LN layer added as dx is stored, and the parameter sums left to a batch
    res = torch.randn(70, 256, generator=g).to(BF)
    batch = ops.ColsumBatch()
    dxr, dg2, db2 = ops.layernorm_backward(dy.cuda(), x.cuda(), gamma.cuda(), mean, rstd, batch=batch,
                                           residual=res.cuda())
    batch.run()
    assert _rel(dxr, xf.grad + res.float()) < 4e-3 and _rel(dg2, gf.grad) < 1e-5 and _rel(db2, bf.grad) < 1e-5

    from pipedream_amd import _cabi
    import ctypes
    s = (torch.randn(33, 512, generator=g) * 3).to(BF)
    sf = s.float().requires_grad_()
    p_ref = torch.softmax(sf, -1)
    dp = torch.randn(33, 512, generator=g).to(BF)
    p_ref.backward(dp.float())
    sg = s.cuda()
    pg = torch.empty_like(sg)
    _cabi.lib().pd_softmax_fwd_bf16(ctypes.c_void_p(sg.data_ptr()), ctypes.c_void_p(pg.data_ptr()), 33, 512,
                                    _cabi.stream_ptr())
    assert _rel(pg, p_ref) < 4e-3
    dsg = torch.empty_like(sg)
    _cabi.lib().pd_softmax_bwd_bf16(ctypes.c_void_p(pg.data_ptr()), ctypes.c_void_p(dp.cuda().data_ptr()),
                                    ctypes.c_void_p(dsg.data_ptr()), 33, 512, _cabi.stream_ptr())
    assert _rel(dsg, sf.grad) < 1e-2

    z = torch.randn(64, 128, generator=g).to(BF)
    zf = z.float().requires_grad_()
    gz = F.gelu(zf)
    gz.backward(dy[:64, :128].float())
    assert _rel(ops.gelu(z.cuda()), gz) < 4e-3
    assert _rel(ops.gelu_backward(z.cuda(), dy[:64, :128].contiguous().cuda()), zf.grad) < 4e-3
    # casts are exact round-to-nearest-even / exact widening
    w = torch.randn(1000, generator=g)
    assert torch.equal(ops.cast_bf16(w.cuda()).cpu(), w.to(BF))
    assert torch.equal(ops.cast_f32(w.to(BF).cuda()).cpu(), w.to(BF).float())


def _pair(n_layers, hidden, heads, ffn, seed=0):
    from pipedream_amd.stages import transformer
    torch.manual_seed(seed)
    ref = models.TransformerStage0(n_layers, hidden, heads, ffn)
    mine = transformer.Stage0(n_layers, hidden, heads, ffn)
    mine.load_state_dict(ref.state_dict())
    assert list(mine.state_dict().keys()) == list(ref.state_dict().keys())
    return ref, mine.cuda()


def test_layer_forward_backward_vs_oracle():
    ref, mine = _pair(2, 128, 4, 256)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 64, 128, generator=g)
    dy = (torch.randn(2, 64, 128, generator=g) * 0.1).to(BF)
    xr = x.clone().requires_grad_()
    yr = ref(xr)
    yr.backward(dy)
    xg = x.cuda().requires_grad_()
    y = mine(xg)
    y.backward(dy.cuda())
    assert y.dtype == BF and _rel(y, yr) < 2e-2
    assert _rel(xg.grad, xr.grad) < 2e-2
    grads = dict((k, p.grad) for k, p in mine.named_parameters())
    for k, p in ref.named_parameters():
        assert grads[k].dtype == torch.float32
        assert _rel(grads[k], p.grad) < 2e-2, (k, _rel(grads[k], p.grad))


def test_2bw_adam_accumulation_matches_oracle():
    """2 weight versions, Adam on fp32 masters every 4 micro-batches with averaged gradients,
    one micro-batch in flight; bf16 weight images kept per version by the optimizer kernel."""
    from pipedream_amd import adam
    ref, mine = _pair(2, 128, 4, 256, seed=3)
    kw = dict(lr=1e-3, betas=(0.9, 0.999))
    opt = adam.AdamWithWeightStashing([mine], list(mine.parameters()), None, 1.0, 2, update_interval=4,
                                      bf16_image=True, **kw)
    ora = so.StashingOptimizerOracle("Adam", [ref], ref.parameters(), 2, update_interval=4, **kw)
    assert opt.update_interval == 4 and opt.num_versions == 2
    g = torch.Generator().manual_seed(4)
    n, W = 12, 1
    xs = [torch.randn(2, 32, 128, generator=g) for _ in range(n)]
    gs = [(torch.randn(2, 32, 128, generator=g) * 0.1).to(BF) for _ in range(n)]
    pend_ref, pend = [], []
    for kind, k in so.one_f_one_b(n, W):
        if kind == "F":
            yr, y = ref(xs[k]), mine(xs[k].cuda())
            assert _rel(y, yr) < 2e-2
            pend_ref.append(yr)
            pend.append(y)
        else:
            for o in (ora, opt):
                o.zero_grad()
                o.load_old_params()
            assert opt.current_version.version == ora.current_version
            pend_ref.pop(0).backward(gs[k])
            pend.pop(0).backward(gs[k].cuda())
            for o in (ora, opt):
                o.load_new_params()
                o.step()
            assert opt.queue.versions() == ora.versions()
            assert opt.latest_version.version == ora.latest_version == (k + 1) // 4
    # bf16 image of the live slot is the rounding of the fp32 masters
    from pipedream_amd import ops
    for p in mine.parameters():
        assert torch.equal(ops.bf16_weight(p), p.detach().to(BF))
    got = mine.state_dict()
    n_updates, lr = 3, kw["lr"]
    for key, v in ref.state_dict().items():
        err = _rel(got[key], v)
        if v.dim() == 2 or key.endswith(".weight"):
            assert err < 2e-2, (key, err)
        else:
            # Bias vectors.  Adam's early steps move an element by ~lr whatever the size of its
            # gradient, so where the gradient is pure rounding noise the step direction is
            # arbitrary in both implementations: the key bias of attention has an exactly
            # zero gradient (softmax ignores a per-query constant), and zero-initialised
            # LayerNorm biases consist of nothing but these steps.  Such elements can differ
            # by at most 2*lr per update; everything else must stay close in norm.
            assert float((got[key].cpu() - v).abs().max()) <= 2.02 * lr * n_updates, key
            assert err < 0.1, (key, err)


def test_full_size_layer_properties():
    """hidden 1024, 16 heads, FFN 4096, micro-batch 8 x 512 tokens: one layer forward and
    backward at the benchmark shape against the oracle."""
    ref, mine = _pair(1, 1024, 16, 4096, seed=5)
    assert sum(p.numel() for p in mine.parameters()) * 6 == 75577344
    g = torch.Generator().manual_seed(6)
    x = torch.randn(8, 512, 1024, generator=g)
    dy = (torch.randn(8, 512, 1024, generator=g) * 0.05).to(BF)
    xg = x.cuda().requires_grad_()
    y = mine(xg)
    y.backward(dy.cuda())
    assert torch.isfinite(y.float()).all() and torch.isfinite(xg.grad).all()
    xr = x.clone().requires_grad_()
    yr = ref(xr)
    yr.backward(dy)
    assert _rel(y, yr) < 2e-2 and _rel(xg.grad, xr.grad) < 2e-2
    grads = dict((k, p.grad) for k, p in mine.named_parameters())
    for k, p in ref.named_parameters():
        assert _rel(grads[k], p.grad) < 2e-2, (k, _rel(grads[k], p.grad))


def test_full_size_stage_six_layers_vs_oracle():
    """The whole stage at its benchmark size -- 6 layers, hidden 1024, 16 heads, FFN 4096, micro-batch
    8 x 512 tokens -- forward and backward against the oracle: output, input gradient and every one of the
    72 parameter gradients within rel-L2 2e-2, i.e. the bf16 error grown over six layers stays inside the bar.
    The worst figures are printed."""
    ref, mine = _pair(6, 1024, 16, 4096, seed=7)
    assert sum(p.numel() for p in mine.parameters()) == 75577344
    g = torch.Generator().manual_seed(8)
    x = torch.randn(8, 512, 1024, generator=g)
    dy = (torch.randn(8, 512, 1024, generator=g) * 0.05).to(BF)
    xg = x.cuda().requires_grad_()
    y = mine(xg)
    y.backward(dy.cuda())
    xr = x.clone().requires_grad_()
    yr = ref(xr)
    yr.backward(dy)
    errs = {"output": _rel(y, yr), "input gradient": _rel(xg.grad, xr.grad)}
    grads = dict((k, p.grad) for k, p in mine.named_parameters())
    for k, p in ref.named_parameters():
        assert grads[k].dtype == torch.float32 and grads[k].shape == p.grad.shape
        errs[k] = _rel(grads[k], p.grad)
    worst = sorted(errs.items(), key=lambda kv: -kv[1])[:5]
    print("six-layer stage at full size, worst rel-L2 errors:", [(k, "%.2e" % v) for k, v in worst])
    print("output %.2e, input gradient %.2e" % (errs["output"], errs["input gradient"]))
    bad = {k: v for k, v in errs.items() if not v < 2e-2}
    assert not bad, bad


def test_weight_gradient_split_over_tokens():
    """``ops.gemm_bf16_wgrad``: the 1024 x 1024 product (64 tiles) is split over the 4096 tokens into four partial
    products added in index order; a wider one is not.  Fresh and accumulated, against fp64."""
    from pipedream_amd import ops
    g = torch.Generator().manual_seed(9)
    for (T, N, K) in ((4096, 1024, 1024), (4096, 1024, 512), (2048, 1024, 4096), (1000, 256, 128)):
        dy = (torch.randn(T, N, generator=g) / 8).to(BF).cuda()
        x = torch.randn(T, K, generator=g).to(BF).cuda()
        want = dy.double().t() @ x.double()
        got = ops.gemm_bf16_wgrad(dy, x)
        assert got.dtype == torch.float32 and _rel(got, want.cpu()) < 1e-5
        acc = torch.randn(N, K, generator=g).cuda()
        want2 = acc.double() + want
        ops.gemm_bf16_wgrad(dy, x, acc)
        assert _rel(acc, want2.cpu()) < 1e-5


def test_batched_column_sums_match_the_single_ones():
    """``ops.ColsumBatch``: bf16 matrices (odd and unaligned shapes among them) and fp32 partial-sum matrices in
    one batch, fresh outputs and accumulation, against fp64 sums; nine jobs, so the batch runs twice."""
    from pipedream_amd import ops
    torch.manual_seed(3)
    shapes = [(4096, 1024, True), (4096, 3072, True), (37, 1000, True), (513, 72, True), (16, 1024, False),
              (40, 1024, False), (4096, 4096, True), (5, 3, True), (7, 130, False)]
    batch = ops.ColsumBatch()
    checks = []
    for i, (M, N, is_bf16) in enumerate(shapes):
        x = torch.randn(M, N, device="cuda")
        x = x.to(torch.bfloat16) if is_bf16 else x
        if i % 2:
            out = torch.randn(N, device="cuda")
            want = out.double().cpu() + x.double().sum(0).cpu()
            batch.add(x, out, 1.0)
        else:
            out = torch.full((N,), float("nan"), device="cuda")
            want = x.double().sum(0).cpu()
            batch.add(x, out, 0.0)
        checks.append((out, want, M))
    batch.run()
    for out, want, M in checks:
        torch.testing.assert_close(out.double().cpu(), want, rtol=1e-5, atol=2e-6 * M)
    with pytest.raises(ValueError):
        batch.add(torch.zeros(4, 4, device="cuda"), torch.zeros(3, device="cuda"), 0.0)


@pytest.fixture(params=[0, 256], ids=["built_in_tile", "tile_256"])
def gemm_tile(request):
    from pipedream_amd import _cabi
    _cabi.lib().pd_gemm_bf16_set_tile(request.param, request.param)
    yield request.param
    _cabi.lib().pd_gemm_bf16_set_tile(0, 0)


@pytest.mark.parametrize("M,N,K", [(4096, 4096, 1024), (512, 1024, 256), (200, 72, 64), (64, 8, 8)])
def test_gemm_with_gelu_in_its_epilogue(M, N, K, gemm_tile):
    """``gemm_bf16_gelu`` / ``gemm_bf16_gelu_backward`` against the GEMM followed by the element-wise kernels
    (the same operations; only the erf approximation and one bf16 rounding differ) and against torch in fp32."""
    from pipedream_amd import ops
    torch.manual_seed(M + N)
    a = (torch.randn(M, K) / math.sqrt(K)).to(BF).cuda()
    w = torch.randn(N, K).to(BF).cuda()
    bias = torch.randn(N).cuda()
    f, g = ops.gemm_bf16_gelu(a, w, trans_b=True, bias=bias)
    f0 = ops.gemm_bf16(a, w, trans_b=True, bias=bias)
    assert torch.equal(f, f0)                                     # the pre-activation is the plain GEMM's
    assert _rel(g, ops.gelu(f0).cpu()) < 2e-3                     # bf16 steps apart at most
    assert _rel(g, F.gelu(f0.float().cpu())) < 4e-3
    dy = (torch.randn(M, 256) / 16).to(BF).cuda()
    w2 = torch.randn(256, N).to(BF).cuda()
    df = ops.gemm_bf16_gelu_backward(dy, w2, f)
    two_step = ops.gelu_backward(f, ops.gemm_bf16(dy, w2))
    assert _rel(df, two_step.cpu()) < 4e-3
    ff = f.float().cpu().requires_grad_()
    F.gelu(ff).backward(dy.float().cpu() @ w2.float().cpu())
    assert _rel(df, ff.grad) < 6e-3
