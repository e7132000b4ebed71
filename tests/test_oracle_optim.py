"""Pins the optimizer arithmetic and the stashing wrapper of the oracle.

* numpy SGD / Adam against the installed torch.optim library (the third-party code the
  reference calls at runtime/optimizer.py:40-41, :151) and against hand-computed values;
* the truth table of the reference's own known-answer test
  (runtime/tests/backprop/sgd_with_stashing.py:59-70) on the CPU restatement of
  OptimizerWithWeightStashing;
* the negative control of runtime/tests/backprop/sgd_vanilla.py (on torch >= 1.5 autograd
  refuses the stale weights outright instead of silently using them).
"""
import numpy as np
import pytest
import torch

from oracle import stash_oracle as so


def _rand(n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n, generator=g)


@pytest.mark.parametrize("momentum,dampening,wd,nesterov", [
    (0.0, 0.0, 0.0, False), (0.9, 0.0, 0.0, False), (0.9, 0.0, 5e-4, False),
    (0.9, 0.1, 1e-4, False), (0.9, 0.0, 1e-4, True)])
def test_sgd_numpy_vs_torch(momentum, dampening, wd, nesterov):
    p0 = _rand(1000, 1)
    p = torch.nn.Parameter(p0.clone())
    opt = torch.optim.SGD([p], lr=0.05, momentum=momentum, dampening=dampening, weight_decay=wd,
                          nesterov=nesterov, foreach=False)
    pn, buf = p0.numpy().copy(), None
    for step in range(5):
        g = _rand(1000, 10 + step)
        p.grad = g.clone()
        opt.step()
        pn, buf = so.sgd_step_numpy(pn, g.numpy(), buf, 0.05, momentum, dampening, wd, nesterov)
        np.testing.assert_allclose(pn, p.detach().numpy(), rtol=1e-5, atol=1e-6)
        if momentum:
            np.testing.assert_allclose(buf, opt.state[p]["momentum_buffer"].numpy(), rtol=1e-5, atol=1e-6)


def test_sgd_hand_values():
    # p=1, g=0.5, wd=0.1 -> g'=0.6; first step buf=0.6; p=1-0.1*0.6=0.94
    p, buf = so.sgd_step_numpy(np.array([1.0], np.float32), np.array([0.5], np.float32), None,
                               lr=0.1, momentum=0.9, dampening=0.5, weight_decay=0.1)
    assert abs(p[0] - 0.94) < 1e-6 and abs(buf[0] - 0.6) < 1e-6
    # second step, g=0.5: g'=0.5+0.094=0.594; buf=0.9*0.6+0.5*0.594=0.837; p=0.94-0.0837
    p, buf = so.sgd_step_numpy(p, np.array([0.5], np.float32), buf, lr=0.1, momentum=0.9, dampening=0.5,
                               weight_decay=0.1)
    assert abs(buf[0] - 0.837) < 1e-6 and abs(p[0] - 0.8563) < 1e-6
    # nesterov: g' + mu*buf
    p, buf = so.sgd_step_numpy(np.array([0.0], np.float32), np.array([1.0], np.float32), None, lr=1.0,
                               momentum=0.5, nesterov=True)
    assert abs(p[0] + 1.5) < 1e-6


@pytest.mark.parametrize("wd", [0.0, 1e-2])
def test_adam_numpy_vs_torch(wd):
    p0 = _rand(1000, 2)
    p = torch.nn.Parameter(p0.clone())
    opt = torch.optim.Adam([p], lr=1e-3, betas=(0.9, 0.999), weight_decay=wd, foreach=False)
    pn = p0.numpy().copy()
    m = np.zeros_like(pn)
    v = np.zeros_like(pn)
    for step in range(1, 8):
        g = _rand(1000, 20 + step)
        p.grad = g.clone()
        opt.step()
        pn, m, v = so.adam_step_numpy(pn, g.numpy(), m, v, step, 1e-3, 0.9, 0.999, 1e-8, wd)
        np.testing.assert_allclose(pn, p.detach().numpy(), rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(m, opt.state[p]["exp_avg"].numpy(), rtol=1e-5, atol=1e-7)
        np.testing.assert_allclose(v, opt.state[p]["exp_avg_sq"].numpy(), rtol=1e-5, atol=1e-9)


def test_adam_hand_values_and_eps_modes():
    # first step from zero state: m=(1-b1)g, v=(1-b2)g^2, m_hat=g, v_hat=g^2 -> p -= lr*g/(|g|+eps')
    g = np.array([0.5, -2.0], np.float32)
    for mode in (0, 1):
        p, m, v = so.adam_step_numpy(np.zeros(2, np.float32), g, np.zeros(2, np.float32),
                                     np.zeros(2, np.float32), 1, lr=0.1, eps=1e-8, eps_mode=mode)
        np.testing.assert_allclose(p, [-0.1, 0.1], rtol=1e-5)
        np.testing.assert_allclose(m, 0.1 * g, rtol=1e-6)
        np.testing.assert_allclose(v, 0.001 * g * g, rtol=1e-5)
    # with a large eps the two placements differ by the factor sqrt(bc2) on eps:
    # mode 0: lr*g/(|g| + eps) ; mode 1: lr*g/(|g| + eps/sqrt(bc2)),  sqrt(bc2)=sqrt(0.001)
    g = np.array([1.0], np.float32)
    z = np.zeros(1, np.float32)
    p0, _, _ = so.adam_step_numpy(z, g, z, z, 1, lr=1.0, eps=1.0, eps_mode=0)
    p1, _, _ = so.adam_step_numpy(z, g, z, z, 1, lr=1.0, eps=1.0, eps_mode=1)
    assert abs(p0[0] + 1.0 / 2.0) < 1e-6
    assert abs(p1[0] + 1.0 / (1.0 + 1.0 / np.sqrt(0.001))) < 1e-5


def _truth_table(num_versions):
    torch.manual_seed(0)
    x = [torch.randn(4, 4).requires_grad_(True)]
    x += [x[0].clone().detach().requires_grad_(True) for _ in range(2)]
    y = torch.randn(4, 4)
    model = torch.nn.Sequential(torch.nn.Linear(4, 4), torch.nn.ReLU(), torch.nn.Linear(4, 4))
    opt = so.StashingOptimizerOracle("SGD", [model], model.parameters(), num_versions, lr=1e-1)
    preds = [model(xi) for xi in x]
    assert torch.equal(preds[0], preds[1]) and torch.equal(preds[0], preds[2])
    loss_fn = torch.nn.MSELoss()
    grads = []
    for pred, xi in zip(preds, x):
        opt.zero_grad()
        opt.load_old_params()
        loss_fn(pred, y).backward()
        grads.append(xi.grad.clone())
        opt.load_new_params()
        opt.step()
    assert not torch.equal(preds[0], model(x[0]))
    return [torch.equal(grads[0], grads[1]), torch.equal(grads[0], grads[2])]


def test_reference_truth_table_on_oracle():
    # sgd_with_stashing.py:68-70
    assert _truth_table(1) == [False, False]
    assert _truth_table(2) == [True, False]
    assert _truth_table(3) == [True, True]


def test_vanilla_sgd_negative_control():
    """sgd_vanilla.py: without stashing the second backward does not see the weights of its
    forward.  PyTorch 1.1 silently produced a different gradient; torch >= 1.5 detects the
    in-place update and raises.  Either way plain SGD is not usable for 1F1B."""
    torch.manual_seed(0)
    x1 = torch.randn(8, 16).requires_grad_(True)
    x2 = x1.clone().detach().requires_grad_(True)
    y = torch.randn(8, 4)
    model = torch.nn.Sequential(torch.nn.ReLU(), torch.nn.Linear(16, 4))
    opt = torch.optim.SGD(model.parameters(), 1e-1)
    l1 = torch.nn.functional.mse_loss(model(x1), y)
    l2 = torch.nn.functional.mse_loss(model(x2), y)
    l1.backward()
    opt.step()
    try:
        l2.backward()
        assert not torch.equal(x1.grad, x2.grad)
    except RuntimeError as e:
        assert "inplace" in str(e) or "in-place" in str(e)


def test_oracle_stash_skips_running_stats():
    """optimizer.py:76-78, :93-94: BatchNorm running statistics are never rolled back."""
    torch.manual_seed(0)
    model = torch.nn.Sequential(torch.nn.Linear(4, 4), torch.nn.BatchNorm1d(4))
    opt = so.StashingOptimizerOracle("SGD", [model], model.parameters(), 2, lr=0.1)
    model(torch.randn(8, 4)).sum().backward()
    rm = model[1].running_mean.clone()
    assert rm.abs().sum() > 0
    opt.load_old_params()
    assert torch.equal(model[1].running_mean, rm)
    opt.load_new_params()
    opt.step()
    opt.load_old_params()
    assert torch.equal(model[1].running_mean, rm)
    assert opt.versions() == [0, 1]


def test_oracle_macrobatch_equals_accumulate_then_step():
    torch.manual_seed(0)
    def make():
        torch.manual_seed(1)
        return torch.nn.Linear(6, 3)
    a, b = make(), make()
    opt = so.StashingOptimizerOracle("SGD", [a], a.parameters(), 4, macrobatch=True, lr=0.1, momentum=0.9)
    assert opt.num_versions == 2 and opt.update_interval == 2
    ref = torch.optim.SGD(b.parameters(), lr=0.1, momentum=0.9)
    xs = [torch.randn(5, 6) for _ in range(6)]
    for i in range(0, 6, 2):
        ref.zero_grad()
        (b(xs[i]).pow(2).mean() / 2 + b(xs[i + 1]).pow(2).mean() / 2).backward()
        ref.step()
    for i in range(6):
        opt.zero_grad()
        opt.load_new_params()   # forward on the newest weights, no pipelining here
        loss = a(xs[i]).pow(2).mean()
        loss.backward()
        opt.step()
    for pa, pb in zip(a.parameters(), b.parameters()):
        torch.testing.assert_close(pa, pb, rtol=1e-5, atol=1e-6)


def test_mixed_precision_branch_of_the_oracle_against_hand_values():
    """The branch of ``step`` taken with model parameters (runtime/optimizer.py:137-155), pinned by what the
    arithmetic fixes: with plain SGD the master after n steps is ``m0 - lr * sum(float(g16)) / loss_scale``
    computed step by step in fp32; the model is the rounded master at every step; a power-of-two loss scale
    applied to the gradients changes nothing; and the masters keep updates too small for the 16-bit model
    (a model updated in its own precision would not move)."""
    import copy
    dtype = torch.bfloat16
    torch.manual_seed(0)
    model = torch.nn.Linear(6, 5, bias=False).to(dtype)
    twin = copy.deepcopy(model)
    masters = [p.detach().clone().float().requires_grad_() for p in model.parameters()]
    masters2 = [p.detach().clone().float().requires_grad_() for p in twin.parameters()]
    lr = 2.0 ** -12
    a = so.StashingOptimizerOracle("SGD", [model], masters, 2, model_parameters=list(model.parameters()),
                                   loss_scale=1.0, lr=lr)
    b = so.StashingOptimizerOracle("SGD", [twin], masters2, 2, model_parameters=list(twin.parameters()),
                                   loss_scale=256.0, lr=lr)
    m0 = masters[0].detach().clone()
    w0 = model.weight.detach().clone()
    g = torch.Generator().manual_seed(1)
    want = m0.clone()
    for step in range(20):
        grad = torch.randn(5, 6, generator=g).to(dtype)
        model.weight.grad = grad.clone()
        twin.weight.grad = (grad.float() * 256.0).to(dtype)          # exact: a power of two
        for o in (a, b):
            o.load_old_params()
            o.load_new_params()
            o.step()
        want = want - lr * grad.float()
        assert torch.equal(masters[0].detach(), want)                 # fp32, step by step
        assert torch.equal(masters2[0].detach(), want)                # the loss scale divides out exactly
        assert torch.equal(model.weight.detach(), want.to(dtype))     # the model is the rounded master
        assert a.versions() == [step, step + 1]
    # the updates (about 2^-12 each) are below half an ulp of most bf16 weights: stepping the model in its
    # own precision leaves those weights where they were, the masters moved
    stalled = w0.clone()
    g = torch.Generator().manual_seed(1)
    for step in range(20):
        stalled = (stalled.float() - lr * torch.randn(5, 6, generator=g).to(dtype).float()).to(dtype)
    big = w0.float().abs() > 0.25
    assert big.any() and torch.equal(stalled[big], w0[big])
    assert not torch.equal(masters[0].detach()[big], m0[big])
