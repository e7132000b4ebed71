"""Translation-stage pieces on the HIP kernels against the CPU oracle (oracle/seq2seq_oracle.py): the
label-smoothing criterion, revert_varlen / the length mask, the bidirectional encoder layer and the
reference's GNMT stage 0 as generated.

Tolerances: the byte-moving kernels (revert_varlen, length mask) are bit-exact.  The criterion computes
in fp32: loss rel 1e-5; its gradient rel 1e-5 of the gradient's scale (entries are softmax values times
grad/B).  LSTM-based layers as in test_gpu_gnmt.py: rel 1e-5 with an absolute term of a few ulp."""
import pytest
import torch

from oracle import models
from oracle import seq2seq_oracle as sq

pytestmark = pytest.mark.gpu


def _criterion_case(T, B, V, pad_frac, seed, scale=3.0):
    g = torch.Generator().manual_seed(seed)
    out = torch.randn(T, B, V, generator=g) * scale
    tgt = torch.randint(1, V, (T * B,), generator=g)
    tgt[torch.rand(T * B, generator=g) < pad_frac] = 0
    return out, tgt


@pytest.mark.parametrize("T,B,V", [(3, 4, 33),       # scalar kernel (V not a multiple of 4)
                                    (5, 3, 32), (2, 3, 2048),    # fewer elements than one group of loads
                                    (2, 5, 5000), (3, 2, 8192),  # one group, ragged / full
                                    (2, 3, 32320),               # four groups (the GNMT vocabulary)
                                    (1, 2, 40000)])
@pytest.mark.parametrize("smoothing", [0.0, 0.1])
def test_label_smoothing_matches_oracle(T, B, V, smoothing):
    from pipedream_amd import layers
    out, tgt = _criterion_case(T, B, V, 0.25, seed=V + T)
    xr = out.clone().requires_grad_(True)
    want = sq.label_smoothing(xr, tgt, 0, smoothing)
    (want * 1.7).backward()
    x = out.cuda().requires_grad_(True)
    got = layers.LabelSmoothing(0, smoothing)(x, tgt.cuda())
    (got * 1.7).backward()
    torch.testing.assert_close(got.cpu(), want.detach(), rtol=1e-5, atol=1e-6)
    scale = float(xr.grad.abs().max())
    torch.testing.assert_close(x.grad.cpu(), xr.grad, rtol=1e-5, atol=1e-5 * scale)
    pad_rows = (tgt == 0).view(T, B)
    assert not x.grad[pad_rows.cuda()].any()


def test_label_smoothing_on_strided_logits_and_all_padding():
    from pipedream_amd import ops
    out, tgt = _criterion_case(4, 3, 64, 0.3, seed=9)
    wide = torch.zeros(12, 96)
    wide[:, :64] = out.view(12, 64)
    xs = wide.cuda()[:, :64]                      # row pitch 96
    loss, lse = ops.label_smoothing_forward(xs, tgt.cuda(), 0, 0.1, 3.0)
    torch.testing.assert_close(loss.cpu(), sq.label_smoothing(out, tgt, 0, 0.1), rtol=1e-5, atol=1e-6)
    d = ops.label_smoothing_backward(xs, tgt.cuda(), lse, torch.ones((), device="cuda"), 0, 0.1, 3.0)
    xr = out.clone().requires_grad_(True)
    sq.label_smoothing(xr, tgt, 0, 0.1).backward()
    torch.testing.assert_close(d.cpu().view(4, 3, 64), xr.grad, rtol=1e-5, atol=1e-7)
    zero, _ = ops.label_smoothing_forward(xs, torch.zeros_like(tgt).cuda(), 0, 0.1, 3.0)
    assert float(zero) == 0.0


def test_label_smoothing_with_infinite_logits_behaves_like_the_reference():
    """Logits of -inf (a masked part of the vocabulary): the reference's smoothing term is the mean of all
    log-probabilities, -inf, times the smoothing factor -- NaN even for smoothing 0 (0 * inf).  Same here;
    the log-sum-exp itself stays finite (a whole group of -inf logits in one thread adds 0, not NaN)."""
    from pipedream_amd import ops
    out, tgt = _criterion_case(2, 3, 16384, 0.0, seed=4)
    out[:, :, 4000:13000] = float("-inf")
    tgt[(tgt >= 4000) & (tgt < 13000)] = 1
    assert torch.isnan(sq.label_smoothing(out, tgt, 0, 0.0))
    loss, lse = ops.label_smoothing_forward(out.view(6, -1).cuda(), tgt.cuda(), 0, 0.0, 3.0)
    assert torch.isnan(loss)
    torch.testing.assert_close(lse.cpu(), torch.logsumexp(out.view(6, -1), dim=-1), rtol=1e-6, atol=1e-6)


def test_label_smoothing_target_out_of_range_poisons_the_loss():
    from pipedream_amd import ops
    x = torch.randn(4, 16).cuda()
    t = torch.tensor([1, 2, 16, 3]).cuda()
    loss, _ = ops.label_smoothing_forward(x, t, 0, 0.1, 1.0)
    assert torch.isnan(loss)


def test_label_smoothing_full_size_properties():
    """GNMT size: 50 x 128 rows over a vocabulary of 32320 (827 MB of logits).  Checked through properties
    that hold at any size: shifting a row's logits by a constant changes neither the loss nor the gradient;
    a non-padding row of the gradient sums to 0 and, after undoing the target and smoothing terms, is a
    probability distribution; padding rows are exactly 0; the loss equals the sum over row blocks computed
    separately (and those blocks are checked against the oracle on a sample)."""
    from pipedream_amd import ops
    T, B, V, s = 50, 128, 32320, 0.1
    g = torch.Generator(device="cuda").manual_seed(11)
    x = torch.randn(T * B, V, device="cuda", generator=g) * 2
    tgt = torch.randint(1, V, (T * B,), device="cuda", generator=g)
    tgt[torch.rand(T * B, device="cuda", generator=g) < 0.2] = 0
    one = torch.ones((), device="cuda")
    loss, lse = ops.label_smoothing_forward(x, tgt, 0, s, float(B))
    d = ops.label_smoothing_backward(x, tgt, lse, one, 0, s, float(B))
    pad = tgt == 0
    assert not d[pad].any()
    rows = d[~pad].double()
    assert float(rows.sum(dim=1).abs().max()) < 1e-6 / B * 10
    p = rows * B + s / V
    p[torch.arange(p.shape[0], device="cuda"), tgt[~pad]] += 1.0 - s
    assert float(p.min()) > -1e-7 and float((p.sum(dim=1) - 1).abs().max()) < 1e-5
    # shift invariance
    shift = torch.randn(T * B, 1, device="cuda", generator=g) * 5
    loss2, lse2 = ops.label_smoothing_forward(x + shift, tgt, 0, s, float(B))
    torch.testing.assert_close(loss2, loss, rtol=1e-5, atol=0)
    # additivity over row blocks, and a sample of blocks against the oracle
    parts = []
    for r0 in range(0, T * B, 1280):
        part, _ = ops.label_smoothing_forward(x[r0:r0 + 1280], tgt[r0:r0 + 1280], 0, s, float(B))
        parts.append(float(part))
    assert sum(parts) == pytest.approx(float(loss), rel=1e-5)
    for blk in (0, 3):
        r0 = blk * 1280
        want = sq.label_smoothing(x[r0:r0 + 1280].cpu().view(10, 128, V), tgt[r0:r0 + 1280].cpu(), 0, s)
        assert parts[blk] == pytest.approx(float(want), rel=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.int32])
@pytest.mark.parametrize("shape,lengths", [((6, 4, 8), [6, 4, 4, 1]),      # 16-byte units (fp32)
                                            ((5, 3, 3), [5, 2, 1]),         # 4- or 2-byte units
                                            ((7, 2, 2, 5), [7, 7]),         # trailing dims fold into the row
                                            ((1, 1, 1), [1]),
                                            ((9, 130, 20), None)])          # batch above 128
def test_revert_varlen_and_mask_are_bit_exact(dtype, shape, lengths):
    from pipedream_amd import ops, pack_utils
    g = torch.Generator().manual_seed(sum(shape))
    T, B = shape[0], shape[1]
    if lengths is None:
        lengths = torch.randint(1, T + 1, (B,), generator=g).sort(descending=True).values.tolist()
        lengths[0] = T
    x = (torch.randn(shape, generator=g) * 100).to(dtype)
    lt = torch.tensor(lengths)
    want = sq.revert_varlen(x.view(torch.int16) if dtype == torch.bfloat16 else x, lt)
    got = pack_utils.revert_varlen_tensor(x.cuda(), lt).cpu()
    assert torch.equal(got.view(torch.int16) if dtype == torch.bfloat16 else got, want)
    mask = sq.set_mask(lt).bool()
    masked = ops.length_mask_apply(x.cuda(), lt.cuda()).cpu()
    keep = mask.view(T, B, *([1] * (len(shape) - 2))).expand(shape)
    assert torch.equal(masked[keep], x[keep]) and not masked[~keep].any()
    # in place
    xc = x.cuda()
    assert ops.length_mask_apply(xc, lt.cuda(), out=xc) is xc
    assert torch.equal(xc.cpu()[keep], x[keep]) and not xc.cpu()[~keep].any()


def test_revert_varlen_into_and_out_of_half_rows():
    from pipedream_amd import ops
    g = torch.Generator().manual_seed(5)
    T, B, H = 6, 3, 12
    lt = torch.tensor([6, 3, 2])
    wide_in = torch.randn(T, B, 2 * H, generator=g)
    wide_out = torch.full((T, B, 2 * H), 7.0).cuda()
    ops.revert_varlen(wide_in.cuda()[:, :, H:], lt.cuda(), out=wide_out[:, :, :H])
    assert torch.equal(wide_out[:, :, :H].cpu(), sq.revert_varlen(wide_in[:, :, H:], lt))
    assert bool((wide_out[:, :, H:] == 7.0).all())          # the other half is untouched


def test_revert_varlen_gradient_is_revert_varlen():
    from pipedream_amd import layers
    lt = torch.tensor([5, 4, 2])
    x = torch.randn(5, 3, 6).cuda().requires_grad_(True)
    dy = torch.randn(5, 3, 6)
    layers.revert_varlen(x, lt).backward(dy.cuda())
    assert torch.equal(x.grad.cpu(), sq.revert_varlen(dy, lt))


def test_varlen_argument_errors():
    from pipedream_amd import ops, pack_utils
    x = torch.zeros(4, 3, 8).cuda()
    with pytest.raises(ValueError, match="batch_size"):
        ops.revert_varlen(x, torch.tensor([4, 2]).cuda())
    with pytest.raises(ValueError, match="1D CPU int64"):
        pack_utils.revert_varlen_tensor(x, torch.tensor([4, 2, 1]).cuda())
    with pytest.raises(ValueError, match="greater than 0"):
        pack_utils.revert_varlen_tensor(x, torch.tensor([4, 2, 0]))
    with pytest.raises(TypeError):
        ops.revert_varlen(x.double(), torch.tensor([4, 2, 1]).cuda())
    with pytest.raises(ValueError, match="dense"):
        ops.revert_varlen(x[:, :, ::2], torch.tensor([4, 2, 1]).cuda())


def _copy_params(mine, ref):
    mine.load_state_dict(ref.state_dict())
    return mine.cuda()


def test_emu_bidir_lstm_matches_oracle():
    from pipedream_amd import layers
    torch.manual_seed(6)
    T, B, I, H = 7, 5, 24, 32
    ref = sq.EmuBidirLSTM(I, H)
    mine = _copy_params(layers.EmuBidirLSTM(I, H), ref)
    assert mine.layer1.weight_ih_l0 is mine.bidir.weight_ih_l0          # still shared after the move
    lt = torch.tensor([7, 6, 6, 3, 1])
    x = torch.randn(T, B, I, requires_grad=True)
    xg = x.detach().cuda().requires_grad_(True)
    y_ref = ref(x, lt)
    y = mine(xg, lt.cuda())
    torch.testing.assert_close(y.cpu(), y_ref.detach(), rtol=1e-5, atol=1e-6)
    dy = torch.randn(T, B, 2 * H)
    y_ref.backward(dy)
    y.backward(dy.cuda())
    torch.testing.assert_close(xg.grad.cpu(), x.grad, rtol=1e-5, atol=1e-6)
    for (k, p), (_, q) in zip(mine.bidir.named_parameters(), ref.bidir.named_parameters()):
        torch.testing.assert_close(p.grad.cpu(), q.grad, rtol=1e-5, atol=2e-6, msg=k)


def test_reference_gnmt_stage0_with_criterion_and_stashed_adam_matches_oracle():
    """The reference's stage 0 as generated (two inputs, two outputs) followed by a linear classifier and
    the label-smoothing criterion, trained for a few 1F1B steps with stashed Adam on both sides."""
    from oracle import stash_oracle as so
    from pipedream_amd import adam, layers
    from pipedream_amd.stages import gnmt
    torch.manual_seed(7)
    V, H, T, B = 61, 32, 6, 4
    ref = models.GnmtBidirStage0(V, H, dropout=0.0)
    ref_cls = torch.nn.Linear(H, V)
    mine = _copy_params(gnmt.BidirStage0(V, H, dropout=0.0), ref)
    mine_cls = _copy_params(layers.Linear(H, V), ref_cls)
    assert list(mine.state_dict().keys()) == list(ref.state_dict().keys())
    W, nv, n = 1, 2, 5
    kw = dict(lr=2e-3, betas=(0.9, 0.999))
    opt = adam.AdamWithWeightStashing([mine, mine_cls], list(mine.parameters()) + list(mine_cls.parameters()),
                                      None, 1.0, nv, **kw)
    ora = so.StashingOptimizerOracle("Adam", [ref, ref_cls],
                                     list(ref.parameters()) + list(ref_cls.parameters()), nv, **kw)
    crit = layers.LabelSmoothing(0, 0.1)
    g = torch.Generator().manual_seed(8)
    lt = torch.tensor([6, 5, 3, 2])
    batches = []
    for _ in range(n):
        ids = torch.randint(1, V, (T, B), generator=g)
        ids = ids * sq.set_mask(lt).long()                       # padding tokens behind every sequence
        batches.append((ids, torch.roll(ids, -1, 0).reshape(-1)))
    pend_ref, pend = [], []
    for kind, k in so.one_f_one_b(n, W):
        ids, tgt = batches[k]
        if kind == "F":
            o17, o21 = ref(ids, lt)
            lr_ = sq.label_smoothing(ref_cls(o17 + o21), tgt, 0, 0.1)
            m17, m21 = mine(ids.cuda(), lt.cuda())
            lm = crit(mine_cls(layers.add(m17, m21)), tgt.cuda())
            torch.testing.assert_close(lm.cpu(), lr_.detach(), rtol=1e-5, atol=1e-6)
            pend_ref.append(lr_)
            pend.append(lm)
        else:
            for o in (ora, opt):
                o.zero_grad()
                o.load_old_params()
            pend_ref.pop(0).backward()
            pend.pop(0).backward()
            grads = dict((key, p.grad) for key, p in mine.named_parameters())
            for key, p in ref.named_parameters():
                scale = float(p.grad.abs().max())
                torch.testing.assert_close(grads[key].cpu(), p.grad, rtol=1e-5, atol=1e-5 * scale,
                                           msg=lambda m, key=key: "grad %s: %s" % (key, m))
            for o in (ora, opt):
                o.load_new_params()
                o.step()
            assert opt.queue.versions() == ora.versions()
    # Adam moves a parameter by lr * m / (sqrt(v) + eps): where a gradient entry happens to lie within
    # ~1e-7 of zero, a rounding difference of 1e-9 in it changes the step by ~1e-2 * lr (a handful of the
    # 60 000 entries per step).  The gradients themselves are compared entry by entry above; the parameters
    # get an absolute term of 5e-2 * lr per entry and 1e-5 on the whole tensor in relative L2 norm.
    got = dict(mine.state_dict())
    for key, v in ref.state_dict().items():
        torch.testing.assert_close(got[key].cpu(), v, rtol=1e-5, atol=5e-2 * kw["lr"],
                                   msg=lambda m, key=key: "%s: %s" % (key, m))
        assert float((got[key].cpu().double() - v.double()).norm() / v.double().norm()) < 1e-5, key


def test_full_size_reference_gnmt_stage0_forward_backward():
    """The reference's stage 0 at its real size (vocabulary 32320, hidden 1024, T = 50, batch 128, sequence
    lengths between 1 and 50, 91 million parameters): one forward/backward against the CPU oracle, compared
    in relative L2 norm."""
    from pipedream_amd.stages import gnmt
    torch.manual_seed(9)
    ref = models.GnmtBidirStage0(dropout=0.0)
    mine = _copy_params(gnmt.BidirStage0(dropout=0.0), ref)
    g = torch.Generator().manual_seed(10)
    T, B = 50, 128
    lt = torch.randint(1, T + 1, (B,), generator=g).sort(descending=True).values
    lt[0] = T
    ids = torch.randint(1, 32320, (T, B), generator=g) * sq.set_mask(lt).long()
    d17 = torch.randn(T, B, 1024, generator=g) * 1e-2
    d21 = torch.randn(T, B, 1024, generator=g) * 1e-2
    r17, r21 = ref(ids, lt)
    torch.autograd.backward([r17, r21], [d17, d21])
    m17, m21 = mine(ids.cuda(), lt.cuda())
    torch.autograd.backward([m17, m21], [d17.cuda(), d21.cuda()])

    def rel(a, b):
        a, b = a.detach().cpu().double(), b.detach().double()
        return float((a - b).norm() / (b.norm() + 1e-300))

    assert rel(m17, r17) < 1e-5 and rel(m21, r21) < 1e-5
    grads = dict((k, p.grad) for k, p in mine.named_parameters())
    for k, p in ref.named_parameters():
        assert rel(grads[k], p.grad) < 2e-5, (k, rel(grads[k], p.grad))
