"""GNMT-style stage (embedding + 4 LSTM layers with residuals, AdamWithWeightStashing,
stash depth 3) on the HIP kernels against the CPU oracle (torch.nn.Embedding / torch.nn.LSTM,
the third-party routines the reference's translation stages call).

Tolerances: fp32; outputs and gradients rel 1e-5 with an absolute term of a few ulp of the
tensor's scale (LSTM states are O(1), sums over T*B terms); parameters after the stashed
Adam steps rtol 1e-5 / atol 1e-6.  Dropout is off (p=0) so both sides are deterministic."""
import pytest
import torch

from oracle import models
from oracle import stash_oracle as so

pytestmark = pytest.mark.gpu


def _rel(a, b):
    a, b = a.detach().cpu().double(), b.detach().double()
    return float((a - b).norm() / (b.norm() + 1e-300))


def test_lstm_layer_matches_torch():
    from pipedream_amd import layers
    torch.manual_seed(0)
    ref = torch.nn.LSTM(24, 32)
    mine = layers.LSTM(24, 32)
    mine.load_state_dict(ref.state_dict())
    assert list(mine.state_dict().keys()) == list(ref.state_dict().keys())
    mine = mine.cuda()
    x = torch.randn(7, 5, 24, requires_grad=True)
    xg = x.detach().cuda().requires_grad_(True)
    y_ref = ref(x)[0]
    y = mine(xg)[0]
    torch.testing.assert_close(y.cpu(), y_ref.detach(), rtol=1e-5, atol=1e-6)
    dy = torch.randn(7, 5, 32)
    y_ref.backward(dy)
    y.backward(dy.cuda())
    torch.testing.assert_close(xg.grad.cpu(), x.grad, rtol=1e-5, atol=1e-6)
    for (k, p), (_, q) in zip(mine.named_parameters(), ref.named_parameters()):
        torch.testing.assert_close(p.grad.cpu(), q.grad, rtol=1e-5, atol=2e-6, msg=k)


@pytest.mark.parametrize("T,B,I,H", [(7, 5, 24, 32), (1, 3, 16, 16), (12, 128, 256, 256), (6, 100, 128, 1024)])
def test_lstm_time_loop_in_native_code_equals_the_step_by_step_calls(T, B, I, H):
    """ops.lstm_forward / lstm_backward issue a layer's time loop through pd_lstm_recurrence_fwd/bwd_f32; with the
    per-launch timer on they call the product and the cell once per step instead.  Same kernels on the same
    operands: every result bit for bit.  (100 and 128 rows: the recurrence product's two block rows of 64.)"""
    from pipedream_amd import ops
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, B, I, generator=g).cuda()
    w_ih = (torch.randn(4 * H, I, generator=g) * 0.1).cuda()
    w_hh = (torch.randn(4 * H, H, generator=g) * 0.1).cuda()
    b_ih, b_hh = torch.randn(4 * H, generator=g).cuda(), torch.randn(4 * H, generator=g).cuda()
    dy = torch.randn(T, B, H, generator=g).cuda()

    def run():
        y, (gates, c) = ops.lstm_forward(x, w_ih, w_hh, b_ih, b_hh)
        return (y, gates, c) + tuple(ops.lstm_backward(dy, x, y, gates, c, w_ih, w_hh))
    native = run()
    ops.kernel_timer = {}
    try:
        stepwise = run()
        assert (T == 1) == ("gemm_f32_splitk" not in ops.kernel_timer)     # the other path did run
    finally:
        ops.kernel_timer = None
    for a, b in zip(native, stepwise):
        assert torch.equal(a, b)
    ref = torch.nn.LSTM(I, H).cuda()
    with torch.no_grad():
        for p, v in zip(ref.parameters(), (w_ih, w_hh, b_ih, b_hh)):
            p.copy_(v)
    xr = x.clone().requires_grad_(True)
    yr = ref(xr)[0]
    yr.backward(dy)
    torch.testing.assert_close(native[0], yr.detach(), rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(native[3], xr.grad, rtol=1e-4, atol=1e-4)


def test_embedding_matches_torch_including_duplicates_and_padding():
    from pipedream_amd import layers
    torch.manual_seed(1)
    ref = torch.nn.Embedding(50, 16, padding_idx=0)
    mine = layers.Embedding(50, 16, padding_idx=0)
    mine.load_state_dict(ref.state_dict())
    mine = mine.cuda()
    ids = torch.randint(0, 50, (9, 13))
    ids[0, :4] = 0          # padding tokens
    ids[1, :] = 7           # many duplicates
    out_ref = ref(ids)
    out = mine(ids.cuda())
    assert torch.equal(out.cpu(), out_ref.detach())
    d = torch.randn(9, 13, 16)
    out_ref.backward(d)
    out.backward(d.cuda())
    torch.testing.assert_close(mine.weight.grad.cpu(), ref.weight.grad, rtol=1e-6, atol=1e-6)
    assert not mine.weight.grad[0].any()


def test_gnmt_stage_with_stashed_adam_matches_oracle():
    from pipedream_amd import adam
    from pipedream_amd.stages import gnmt
    torch.manual_seed(2)
    V, H, T, B = 97, 32, 6, 5
    ref = models.GnmtStage0(V, H, dropout=0.0)
    mine = gnmt.Stage0(V, H, dropout=0.0)
    mine.load_state_dict(ref.state_dict())
    mine = mine.cuda()
    W, nv, n = 2, 3, 7
    kw = dict(lr=1e-3, betas=(0.9, 0.999))
    opt = adam.AdamWithWeightStashing([mine], list(mine.parameters()), None, 1.0, nv, **kw)
    ora = so.StashingOptimizerOracle("Adam", [ref], ref.parameters(), nv, **kw)
    g = torch.Generator().manual_seed(3)
    ids = [torch.randint(0, V, (T, B), generator=g) for _ in range(n)]
    gs = [torch.randn(T, B, H, generator=g) * 1e-2 for _ in range(n)]
    pend_ref, pend = [], []
    for kind, k in so.one_f_one_b(n, W):
        if kind == "F":
            yr, y = ref(ids[k]), mine(ids[k].cuda())
            torch.testing.assert_close(y.cpu(), yr.detach(), rtol=1e-5, atol=1e-6)
            pend_ref.append(yr)
            pend.append(y)
        else:
            for o in (ora, opt):
                o.zero_grad()
                o.load_old_params()
            assert opt.current_version.version == ora.current_version == so.backward_version(k, W)
            pend_ref.pop(0).backward(gs[k])
            pend.pop(0).backward(gs[k].cuda())
            for o in (ora, opt):
                o.load_new_params()
                o.step()
            assert opt.queue.versions() == ora.versions()
    got = mine.state_dict()
    for key, v in ref.state_dict().items():
        torch.testing.assert_close(got[key].cpu(), v, rtol=1e-5, atol=1e-6, msg=key)


def test_full_size_gnmt_stage_forward_backward():
    """vocab 32320, hidden 1024, T=50, B=128 (66 682 880 parameters): one forward/backward
    against the CPU library, compared in relative L2 norm."""
    from pipedream_amd.stages import gnmt
    torch.manual_seed(4)
    ref = models.GnmtStage0(dropout=0.0)
    mine = gnmt.Stage0(dropout=0.0)
    mine.load_state_dict(ref.state_dict())
    assert sum(p.numel() for p in mine.parameters()) == 66682880
    mine = mine.cuda()
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, 32320, (50, 128), generator=g)
    dy = torch.randn(50, 128, 1024, generator=g) * 1e-2
    yr = ref(ids)
    yr.backward(dy)
    y = mine(ids.cuda())
    y.backward(dy.cuda())
    assert _rel(y, yr) < 1e-5
    grads = dict((k, p.grad) for k, p in mine.named_parameters())
    for k, p in ref.named_parameters():
        assert _rel(grads[k], p.grad) < 2e-5, (k, _rel(grads[k], p.grad))


def test_embedding_gradient_sums_duplicates_in_position_order():
    # 1500 positions over 40 rows of 1280 columns (more than one pass of the block over the columns), ids that
    # are out of range or the padding row contribute nothing, every other row is the fp32 sum of its positions
    # taken in increasing order: bit for bit, and rows without a position are zero
    from pipedream_amd import ops
    torch.manual_seed(5)
    V, D, n = 40, 1280, 1500
    ids = torch.randint(0, 30, (n,))
    ids[::97] = 3                      # padding row
    ids[5] = -1
    ids[6] = V + 2
    dout = torch.randn(n, D)
    got = ops.embedding_backward(ids.cuda(), dout.cuda(), V, padding_idx=3).cpu()
    want = torch.zeros(V, D)
    for p in range(n):
        v = int(ids[p])
        if 0 <= v < V and v != 3:
            want[v] += dout[p]
    assert torch.equal(got, want)
    assert not got[30:].any() and not got[3].any()


def test_forward_beside_backward_on_a_stream_ring_gives_the_same_bits():
    """``schedule.MinibatchStreams``: minibatch j runs forward, backward and update on stream j mod (W + 1), so
    the forward recurrence of a new minibatch runs beside the backward recurrence of the oldest one.  At the
    stage's real width (hidden 1024, batch 128; a short sequence), with no host synchronisation inside the run:
    outputs, parameters and Adam state equal the single-stream run bit for bit, versions included."""
    from pipedream_amd import adam, schedule
    from pipedream_amd.stages import gnmt
    V, H, T, B, W, n = 1000, 1024, 6, 128, 2, 8
    g = torch.Generator().manual_seed(5)
    ids = [torch.randint(0, V, (T, B), generator=g).cuda() for _ in range(n)]
    gs = [(torch.randn(T, B, H, generator=g) * 1e-2).cuda() for _ in range(n)]

    def run(ring):
        torch.manual_seed(4)
        m = gnmt.Stage0(V, H, dropout=0.0).cuda()
        opt = adam.AdamWithWeightStashing([m], list(m.parameters()), None, 1.0, W + 1, lr=1e-3, betas=(0.9, 0.999))
        outs, pend = [], []
        if ring is not None:
            ring.join()
        for kind, k in so.one_f_one_b(n, W):
            if kind == "F":
                with (ring.forward(k) if ring is not None else torch.cuda.stream(torch.cuda.current_stream())):
                    pend.append(m(ids[k]))
                    outs.append(pend[-1].detach())
            else:
                with (ring.backward(k) if ring is not None else torch.cuda.stream(torch.cuda.current_stream())):
                    opt.zero_grad()
                    opt.load_old_params()
                    pend.pop(0).backward(gs[k])
                    opt.load_new_params()
                    opt.step()
        if ring is not None:
            ring.leave()
        state = [opt.state[p][name] for p in m.parameters() for name in ("exp_avg", "exp_avg_sq")]
        return ([o.cpu() for o in outs], [p.detach().cpu() for p in m.parameters()], [t.cpu() for t in state],
                opt.queue.versions())

    one = run(None)
    many = run(schedule.MinibatchStreams(W))
    assert one[3] == many[3]
    for a, b in zip(one[:3], many[:3]):
        assert len(a) == len(b) and all(torch.equal(x, y) for x, y in zip(a, b))
